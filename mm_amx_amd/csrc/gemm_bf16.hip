// bf16 x bf16 -> fp32 MFMA tile GEMM instantiations (v_mfma_f32_32x32x16_bf16).
#include "gemm_tile.hpp"

namespace mmx {

int launch_gemm_tiles_bf16(const void* A, int64_t lda, const void* Bp, int M, int K, int N, int n0, int n1,
                           const Epilogue& ep, hipStream_t st) {
    GemmArgs g;
    TileCfg t;
    int mode;
    const int grid = prepare_gemm(g, t, mode, 2, A, lda, Bp, M, K, N, n0, n1, ep);
    if (grid < 0) return grid;
    switch (ep.out_dtype) {
    case MMX_F32: return launch_tiles<__bf16, float>(g, t, mode, grid, st);
    case MMX_BF16: return launch_tiles<__bf16, uint16_t>(g, t, mode, grid, st);
    case MMX_I8: return launch_tiles<__bf16, int8_t>(g, t, mode, grid, st);
    default: return set_error(MMX_E_INVALID, "bf16 GEMM: output dtype %d not supported", ep.out_dtype);
    }
}

}  // namespace mmx
