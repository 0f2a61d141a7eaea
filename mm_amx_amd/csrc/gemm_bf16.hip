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

// 17-32 rows over bf16 weights with a workspace at hand, and at most one 16-column panel per CU: the chunked decode
// kernel then has one workgroup per CU walk the whole of K, and the 64-row tile with a K split is ahead of it where the
// plan has one (weights rotated over 540 MB: 11008 x 4096 at M = 17 / 24 / 32 30.4 / 32.5 / 34.0 -> 25.0 / 25.5 / 26.2 us,
// 4096 x 4096 at M = 24 / 32 14.0 / 14.6 -> 13.6 / 13.8). With more panels than CUs (8192 x 8192, 4096 x 11008) or a short
// K at M < 24 the decode kernel is level or ahead, and it stays.
int decode_resident();
bool few_rows_prefer_tiles_bf16(const void* A, int64_t lda, int M, int K, int Ncols, uint32_t steps, const SplitRequest& rq) {
    if (M < 17 || M > 32 || !rq.ws || rq.k_splits == 1 || (steps & MMX_PP_SILU_GATE) || forced_tile().bm) return false;
    if (decode_resident() == 1) return false;   // a decode form asked for by name
    const int64_t kbytes = (int64_t)K * 2;
    if (kbytes % 128 || (reinterpret_cast<uintptr_t>(A) & 15) || (lda & 15) || load_mode() != 2) return false;
    if (Ncols > 16 * num_cus() || (M < 24 && K < 8192) || K >= (1 << 22) || lda >= (1 << 26)) return false;
    const Plan p = choose_plan(M, Ncols, (int)(kbytes / 128), false, false, 2, rq);
    return p.t.bm == 64 && p.S > 1;
}

// Bytes of workspace the plan for this shape would use (0: no K split), assuming operands the ring pipeline takes.
size_t plan_workspace_bytes(int elesz, bool w8, int M, int K, int Ncols, uint32_t steps, int k_splits) {
    const int64_t kbytes = (int64_t)K * elesz;
    if (kbytes % 128) return 0;
    const SplitRequest rq = {k_splits, reinterpret_cast<char*>(256), ~(size_t)0};
    if (steps & MMX_PP_SILU_GATE) return 0;
    const Plan p = choose_plan(M, Ncols, (int)(kbytes / 128), false, w8, 2, rq);
    if (p.S <= 1) return 0;
    const size_t tiles = (size_t)((M + p.t.bm - 1) / p.t.bm) * ((Ncols + p.t.bn - 1) / p.t.bn);
    return WS_COUNTER_BYTES + tiles * p.S * p.t.bm * p.t.bn * 4;
}

}  // namespace mmx
