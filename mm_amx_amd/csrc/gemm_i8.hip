// int8 x int8 -> int32 MFMA tile GEMM instantiations (v_mfma_i32_32x32x32_i8).
#include "gemm_tile.hpp"

namespace mmx {

int launch_gemm_tiles_i8(const void* A, int64_t lda, const void* Bp, int M, int K, int N, int n0, int n1,
                         const Epilogue& ep, hipStream_t st) {
    GemmArgs g;
    TileCfg t;
    int mode;
    const int grid = prepare_gemm(g, t, mode, 1, A, lda, Bp, M, K, N, n0, n1, ep);
    if (grid < 0) return grid;
    switch (ep.out_dtype) {
    case MMX_F32: return launch_tiles<int8_t, float>(g, t, mode, grid, st);
    case MMX_BF16: return launch_tiles<int8_t, uint16_t>(g, t, mode, grid, st);
    case MMX_I8: return launch_tiles<int8_t, int8_t>(g, t, mode, grid, st);
    case MMX_I32: return launch_tiles<int8_t, int32_t>(g, t, mode, grid, st);
    default: return set_error(MMX_E_INVALID, "int8 GEMM: output dtype %d not supported", ep.out_dtype);
    }
}

}  // namespace mmx
