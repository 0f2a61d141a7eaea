// bf16 x int8-weight MFMA tile GEMM (on-the-fly dequantisation, include/kernels_amx.hpp:1447-1497): launch geometry and
// dispatch on the output type.
#include "gemm_tile.hpp"

namespace mmx {

int launch_tiles_w8_out_f32(const GemmArgs& g, TileCfg t, int mode, int grid, hipStream_t st);
int launch_tiles_w8_out_bf16(const GemmArgs& g, TileCfg t, int mode, int grid, hipStream_t st);
int launch_tiles_w8_out_i8(const GemmArgs& g, TileCfg t, int mode, int grid, hipStream_t st);

int launch_gemm_tiles_w8(const void* A, int64_t lda, const void* Bp, int M, int K, int N, int n0, int n1,
                         const Epilogue& ep, const SplitRequest& rq, hipStream_t st) {
    GemmArgs g;
    TileCfg t;
    int mode;
    const int grid = prepare_gemm(g, t, mode, 2, A, lda, Bp, M, K, N, n0, n1, ep, rq, true);
    if (grid < 0) return grid;
    switch (ep.out_dtype) {
    case MMX_F32: return launch_tiles_w8_out_f32(g, t, mode, grid, st);
    case MMX_BF16: return launch_tiles_w8_out_bf16(g, t, mode, grid, st);
    case MMX_I8: return launch_tiles_w8_out_i8(g, t, mode, grid, st);
    default: return set_error(MMX_E_INVALID, "bf16 x int8-weight GEMM: output dtype %d not supported", ep.out_dtype);
    }
}

}  // namespace mmx
