/*
 * fc_oracle.h — CPU restatement of the mm_amx fully-connected GEMM path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library links, loads or calls
 * this code; it exists so that the HIP path can be checked against the arithmetic
 * of the reference (usstq/mm_amx) on any x86-64 host, with or without AMX.
 *
 * Every function states the reference file:line whose arithmetic it follows
 * (paths are relative to the reference checkout).
 *
 * Pinning status (how each function is checked before it is trusted):
 *   orc_gemm_bf16          pinned  — against the compiled reference (real AMX tdpbf16ps)
 *                                    bit-for-bit, and against an fp64 GEMM by tolerance
 *   orc_gemm_i8            pinned  — integer arithmetic, against the compiled reference
 *                                    and an int64 brute force
 *   orc_pp_*               pinned  — against the compiled reference BiasGeluStore for
 *                                    per-tensor scales; per-output-channel DEQUANT has no
 *                                    counterpart in the reference: it is pinned by the
 *                                    identity per_oc(all equal s) == per_tensor(s) and by
 *                                    column-by-column equality with per-tensor runs
 *   orc_gelu               pinned  — against the compiled reference bit-for-bit, closed
 *                                    forms of the five zones, |gelu - erf form| <= 3.4e-4
 *   orc_repack_amx         pinned  — against the compiled reference repackB_1x2
 *   orc_repack_mfma        spec    — defines this project's own layout (no reference
 *                                    counterpart); checked to be a bijection + zero pad
 *   orc_quantize_weights   pinned  — against the compiled reference Matmul<bf16,int8>
 *   orc_gemv_w8            pinned  — through orc_gemm_bf16 on exactly converted weights
 *   orc_bf16_scale_trunc_s8, orc_quantize_scale_trunc, orc_repack_1xL_s8
 *                          pinned  — the element expression of repackB_1xL<int8_t, L> (fc16m.cpp:80-81) is compiled
 *                                    from the reference's own bfloat16 class (include/bf16.hpp) in the reference
 *                                    shim and compared on all 65536 bf16 inputs x several scales (values inside
 *                                    int8's range: beyond it the reference's conversion is undefined); the tile
 *                                    order by its index formula on matrices whose entries encode their position.
 *                                    fc16m.cpp itself needs xbyak (through test_bw.hpp) and cannot be compiled here.
 *   orc_gemm_x8, orc_matvec_x8
 *                          pinned  — integer arithmetic: against an int64 product everywhere, and against the
 *                                    compiled reference where the reference has the form at all
 *                                    (Matmul<uint8_t,int8_t> and the three MatmulVector forms; the reference's
 *                                    Matmul with unsigned B does not compile: its repackB_1x2 has no uint8_t form)
 *   orc_quantize_int4,     spec    — PARITY UNPINNED against the reference, which has no int4 algorithm (it
 *   orc_pack_int4                    only times a byte-copying stand-in): these define what the device code
 *                                    must produce; checked by what the mathematics fixes (|w - q deq| <=
 *                                    deq/2, |q| <= 7, the column maximum maps to +-7, zero columns, the
 *                                    layout is a bijection with zero padding) and by answers worked
 *                                    out by hand (ties to even, one packed dword)
 *   orc_matvec_*           pinned  — against the compiled reference MatmulVector/GemAvB
 *                                    for ceil(K/kStep) <= 4 (the reference is wrong beyond)
 *   orc_rcp14              pinned  — against the vrcp14ps instruction itself on all 2^32 inputs
 *                                    (any AVX-512 host) and against committed vectors elsewhere
 *   orc_exp_poly, orc_silu PARITY UNPINNED at the bit level: their source (tests/amx-mlp.cpp)
 *                          needs xbyak and cannot be compiled here, so no run of the reference
 *                          stands behind them.  Both are short straight-line sequences
 *                          restated operation for operation (every instruction they use is
 *                          pinned: fused multiply-add, floor, round-to-nearest convert,
 *                          vrcp14ps); what is checked is the mathematics: |exp_poly - exp| and
 *                          |silu - x/(1+e^-x)| bounds, silu(0) = 0, limits, overflow to inf.
 *   orc_mlp_*              pinned per GEMM stage (same as orc_gemm_bf16); the SiLU stage
 *                          inherits the note above.
 */
#ifndef FC_ORACLE_H
#define FC_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* post-op step bits, same values as amx_kernel::PP::Steps (include/kernels_amx.hpp:540-550) */
enum { ORC_PP_DEQUANT = 1, ORC_PP_BIAS = 2, ORC_PP_GELU = 4, ORC_PP_QUANT = 8 };
/* element types */
enum { ORC_F32 = 0, ORC_BF16 = 1, ORC_I8 = 2, ORC_I32 = 3 };

typedef struct {
    uint32_t steps;           /* ORC_PP_* bits                                         */
    int out_dtype;            /* ORC_F32 / ORC_BF16 / ORC_I8                            */
    const float* bias;        /* [N] when ORC_PP_BIAS                                   */
    float deq_scale;          /* per-tensor dequant scale (reference field deq_scale)  */
    const float* deq_per_oc;  /* [N] per-output-channel dequant (extension); wins if set */
    float q_scale;            /* per-tensor quant scale (reference q_scale_common)      */
    const float* q_per_oc;    /* [N] per-output-channel quant (reference q_scale_per_oc) */
} orc_pp;

/* ---- scalar conversions -------------------------------------------------------- */
uint16_t orc_f32_to_bf16(float x);        /* RNE, vcvtneps2bf16 semantics               */
float orc_bf16_to_f32(uint16_t b);
void orc_f32_to_bf16_n(const float* src, uint16_t* dst, size_t n);
void orc_bf16_to_f32_n(const uint16_t* src, float* dst, size_t n);

/* ---- GEMM cores ------------------------------------------------------------------ */
/* C[M,N] (fp32) = A[M,K] (bf16) x B (bf16).  B is [K,N] (transB=0) or [N,K] (transB=1).
 * lda/ldb/ldc are in ELEMENTS.  Accumulation order is that of AMX tdpbf16ps as driven
 * by the reference's kernels.  nthreads<=0: all cores. */
void orc_gemm_bf16(const uint16_t* A, int64_t lda, const uint16_t* B, int64_t ldb, int transB,
                   float* C, int64_t ldc, int M, int K, int N, int nthreads);
/* same product accumulated in double and rounded once to fp32 (independent check) */
void orc_gemm_bf16_f64(const uint16_t* A, int64_t lda, const uint16_t* B, int64_t ldb, int transB,
                       float* C, int64_t ldc, int M, int K, int N, int nthreads);
/* C[M,N] (int32) = A[M,K] (s8) x B (s8), exact */
void orc_gemm_i8(const int8_t* A, int64_t lda, const int8_t* B, int64_t ldb, int transB,
                 int32_t* C, int64_t ldc, int M, int K, int N, int nthreads);

/* C[M,N] (int32, modulo 2^32) = A x B with the bytes of A and/or B read as unsigned (tdpbusd / tdpbsud / tdpbuud,
 * include/kernels_amx.hpp:1057-1101); lda/ldb/ldc in elements */
void orc_gemm_x8(int a_unsigned, int b_unsigned, const void* A, int64_t lda, const void* B, int64_t ldb, int transB,
                 int32_t* C, int64_t ldc, int M, int K, int N);
void orc_matvec_x8(int a_unsigned, int b_unsigned, const void* A, int64_t lda, const void* b, int32_t* c, int M, int K);
/* the same without the AVX-512BW path (scalar-order check of the fast one) */
void orc_gemm_i8_generic(const int8_t* A, int64_t lda, const int8_t* B, int64_t ldb, int transB,
                         int32_t* C, int64_t ldc, int M, int K, int N);

/* ---- epilogue -------------------------------------------------------------------- */
float orc_gelu(float x);
void orc_gelu_n(const float* src, float* dst, size_t n);
/* apply the post-op chain to accumulators acc[M,N] (ld in elements) and store to C
 * (row stride ldc_bytes).  Column n of acc is output channel n (bias[n], scale[n]). */
void orc_pp_f32(const float* acc, int64_t ldacc, int M, int N, const orc_pp* pp, void* C, int64_t ldc_bytes);
void orc_pp_i32(const int32_t* acc, int64_t ldacc, int M, int N, const orc_pp* pp, void* C, int64_t ldc_bytes);

/* ---- weight repack ---------------------------------------------------------------- */
/* element size 2 (bf16) or 1 (int8).  B is [K,N] (transpose=0) or [N,K] (transpose=1),
 * row stride ldb_bytes. */
size_t orc_repack_amx_bytes(int elesz, int K, int N);
/* AMX 1x2 tile order of repackB_1x2; columns >= N of the last panel are written as zero
 * (the reference leaves unspecified bytes there). */
void orc_repack_amx(int elesz, const void* B, int64_t ldb_bytes, int K, int N, int transpose, void* out);
size_t orc_repack_mfma_bytes(int elesz, int K, int N);
/* gfx950 MFMA-fragment order used by the HIP kernels:
 *   out[panel = n/32][kstep = k/KS][lane][16 bytes], KS = 16/elesz * 2 (bf16: 16, int8: 32),
 *   lane = (n%32) + 32*((k%KS)/(KS/2)), byte = (k % (KS/2)) * elesz;
 *   K padded with zeros to a multiple of 128 bytes per column, N to a multiple of 32. */
void orc_repack_mfma(int elesz, const void* B, int64_t ldb_bytes, int K, int N, int transpose, void* out);

/* ---- weight compression ------------------------------------------------------------ */
/* per-tensor symmetric quantisation of a bf16 weight matrix [rows, cols] to int8;
 * returns the dequant scale (max/127) and writes the quant scale (127/max). */
float orc_quantize_weights(const uint16_t* W, int64_t ldw, int rows, int cols,
                           int8_t* Wq, int64_t ldq, float* quant_scale);

/* y[M,N] (bf16) = bf16( (x[M,K] bf16 · float(Wq[K,N] int8)) * scale[n] ), fp32 AMX-order
 * accumulation.  Wq is [K,N] (transW=0) or [N,K] (transW=1).  If acc_out != NULL the raw
 * fp32 accumulators are also returned. */
/* repackB_1xL<int8_t, L> (weight_compression/fc16m.cpp:61-99): q = trunc(bf16_rne(float(w) * scale)) */
int8_t orc_bf16_scale_trunc_s8(uint16_t w, float scale);
void orc_quantize_scale_trunc(const uint16_t* W, int64_t ldw, int rows, int cols, float scale, int8_t* Wq, int64_t ldq);
void orc_repack_1xL_s8(const uint16_t* B, int64_t ldb, int K, int N, int L, float scale, int8_t* out);

/* int4 weight compression (definition of this project; the reference only times a stand-in,
 * weight_compression/wcompress.hpp:90-134) and its packed layout */
void orc_quantize_int4(const uint16_t* W, int64_t ldw, int K, int N, int transpose, int8_t* q, float* deq);
size_t orc_pack_int4_bytes(int K, int N);
void orc_pack_int4(const int8_t* q, int K, int N, uint8_t* out);

void orc_gemv_w8(const uint16_t* x, int64_t ldx, const int8_t* Wq, int64_t ldw, int transW,
                 const float* scale, uint16_t* y, int64_t ldy, float* acc_out, int M, int K, int N,
                 int nthreads);

/* The same result (bit for bit) computed as the reference computes it: weights packed once in the order of
 * repackB_1xL<int8_t,2> (orc_pack_1x2_s8: K*N bytes), then streamed and converted in registers, N split over threads
 * in 32-column groups (weight_compression/fc16m.cpp:61-99, 451-502, 620-663).  K % 32 == 0, N % 32 == 0, M <= 16;
 * returns -1 for shapes it does not take.  This is the form whose time means something. */
void orc_pack_1x2_s8(const int8_t* W, int64_t ldw, int K, int N, int8_t* out);
int orc_gemv_w8_stream(const uint16_t* x, int64_t ldx, const int8_t* Wpacked, const float* scale, uint16_t* y,
                       int64_t ldy, int M, int K, int N, int nthreads);

/* ---- matrix x vector ------------------------------------------------------------- */
/* c[M] = A[M,K]·b[K]; bf16 in AMX order (MatmulVector), fp32 out */
void orc_matvec_bf16(const uint16_t* A, int64_t lda, const uint16_t* b, float* c, int M, int K);
/* GemAvB order (vdpbf16ps, two interleaved accumulators) */
void orc_gemavb_bf16(const uint16_t* A, int64_t lda, const uint16_t* b, float* c, int M, int K);
void orc_matvec_i8(const int8_t* A, int64_t lda, const int8_t* b, int32_t* c, int M, int K);

/* ---- fused MLP --------------------------------------------------------------------- */
float orc_exp_poly(float x);  /* exp_ps_avx512 */
float orc_rcp14(float x);     /* vrcp14ps, bit for bit */
void orc_rcp14_n(const float* src, float* dst, size_t n);
void orc_silu_n(const float* src, float* dst, size_t n);
void orc_exp_poly_n(const float* src, float* dst, size_t n);
float orc_silu(float x);      /* silu_ps_avx512 */
/* h[M,N] bf16 = bf16( silu(gate) * up ) from fp32 accumulators */
void orc_silu_mul_bf16(const float* gate, const float* up, uint16_t* h, size_t n);
/* x[M,K] bf16; w_gate,w_up [N,K] bf16; w_down [K,N] bf16 (torch nn.Linear.weight layouts).
 * h_out [M,N] bf16 (may be NULL), y [M,K] bf16.  split_k: 1 = the reference's 2-way
 * split-K of down_proj in units of 256-element K blocks. */
void orc_mlp(const uint16_t* x, const uint16_t* w_gate, const uint16_t* w_up, const uint16_t* w_down,
             uint16_t* h_out, uint16_t* y, int M, int K, int N, int split_k, int nthreads);
/* down stage only: y[M,Kout] = bf16(h[M,N] · w_down[Kout,N]^T) */
void orc_mlp_down(const uint16_t* h, const uint16_t* w_down, uint16_t* y, int M, int Kout, int N,
                  int split_k, int nthreads);

/* ---- misc -------------------------------------------------------------------------- */
/* work partition used by the reference's N-split (include/misc.hpp:521-535) */
void orc_splitter(int n, int team, int tid, int* n_start, int* n_end);
const char* orc_isa(void); /* which clone of the hot loop runs on this host */

#ifdef __cplusplus
}
#endif
#endif
