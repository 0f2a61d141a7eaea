// bf16 x bf16 MFMA tile GEMM (v_mfma_f32_32x32x16_bf16): launch geometry and dispatch on the output type.
#include "gemm_tile.hpp"

namespace mmx {

int launch_tiles_bf16_out_f32(const GemmArgs& g, TileCfg t, int mode, int grid, hipStream_t st);
int launch_tiles_bf16_out_bf16(const GemmArgs& g, TileCfg t, int mode, int grid, hipStream_t st);
int launch_tiles_bf16_out_i8(const GemmArgs& g, TileCfg t, int mode, int grid, hipStream_t st);

int launch_gemm_tiles_bf16(const void* A, int64_t lda, const void* Bp, int M, int K, int N, int n0, int n1,
                           const Epilogue& ep, const SplitRequest& rq, hipStream_t st) {
    GemmArgs g;
    TileCfg t;
    int mode;
    const int grid = prepare_gemm(g, t, mode, 2, A, lda, Bp, M, K, N, n0, n1, ep, rq);
    if (grid < 0) return grid;
    switch (ep.out_dtype) {
    case MMX_F32: return launch_tiles_bf16_out_f32(g, t, mode, grid, st);
    case MMX_BF16: return launch_tiles_bf16_out_bf16(g, t, mode, grid, st);
    case MMX_I8: return launch_tiles_bf16_out_i8(g, t, mode, grid, st);
    default: return set_error(MMX_E_INVALID, "bf16 GEMM: output dtype %d not supported", ep.out_dtype);
    }
}

// Bytes of workspace the plan for this shape would use (0: no K split), assuming operands the ring pipeline takes.
size_t plan_workspace_bytes(int elesz, bool w8, int M, int K, int Ncols, uint32_t steps, int k_splits) {
    const int64_t kbytes = (int64_t)K * elesz;
    if (kbytes % 128) return 0;
    const SplitRequest rq = {k_splits, reinterpret_cast<char*>(256), ~(size_t)0};
    if (steps & MMX_PP_SILU_GATE) return 0;
    const Plan p = choose_plan(M, Ncols, (int)(kbytes / 128), false, w8, 2, rq, elesz == 1);
    if (p.S <= 1) return 0;
    const size_t tiles = (size_t)((M + p.t.bm - 1) / p.t.bm) * ((Ncols + p.t.bn - 1) / p.t.bn);
    return WS_COUNTER_BYTES + tiles * p.S * p.t.bm * p.t.bn * 4;
}

}  // namespace mmx
