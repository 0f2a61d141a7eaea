/*
 * mm_amx_amd.h — C ABI of the MI355X (gfx950) fully-connected GEMM path.
 *
 * Plain C, device pointers and sizes only; every call is asynchronous on the HIP stream
 * passed in (NULL = the default stream) and returns 0 on success or a negative MMX_E_* code,
 * with a per-thread message available from mmx_last_error().  Nothing is thrown across this
 * boundary.  No entry point allocates or frees device memory.
 *
 * The reference (usstq/mm_amx) has no FFI boundary of its own: its interface is a set of
 * C++ templates in include/kernels_amx.hpp.  Each entry point below names the reference
 * interface it stands in for; the C++ classes with the reference's names are layered on
 * top of this ABI in include/mm_amx_amd/kernels_gfx950.hpp.
 */
#ifndef MM_AMX_AMD_H
#define MM_AMX_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element types */
enum { MMX_F32 = 0, MMX_BF16 = 1, MMX_I8 = 2, MMX_I32 = 3, MMX_I4 = 4 /* packed weights only */,
       MMX_U8 = 5 /* unsigned bytes: mmx_repack_b, mmx_gemm_u8, mmx_matvec_u8 only */ };

/* error codes */
enum {
    MMX_OK = 0,
    MMX_E_INVALID = -1,     /* bad argument (shape, alignment, null pointer, unknown dtype) */
    MMX_E_UNSUPPORTED = -2, /* valid request this build has no kernel for */
    MMX_E_HIP = -3,         /* a HIP runtime call failed */
    MMX_E_DEVICE = -4       /* no gfx950 device */
};

/* Post-op steps: the values of amx_kernel::PP::Steps (include/kernels_amx.hpp:540-550),
 * plus MMX_PP_SILU_GATE for the fused gate/up epilogue of tests/amx-mlp.cpp:707-737. */
enum {
    MMX_PP_NONE = 0,
    MMX_PP_DEQUANT = 1,
    MMX_PP_BIAS = 2,
    MMX_PP_GELU = 4,
    MMX_PP_QUANT = 8,
    MMX_PP_SILU_GATE = 16
};

/*
 * Epilogue descriptor — the data members of amx_kernel::PP::BiasGeluStore<D, steps>
 * (include/kernels_amx.hpp:552-583) as plain data, because a host functor cannot be called
 * per 32x32 block from a GPU kernel.  Applied per element, in this order, each step one
 * correctly rounded fp32 operation (no fused multiply-add across steps):
 *     r = float(acc)                          (int32 accumulators only, round-to-nearest-even)
 *     r = r * deq                             MMX_PP_DEQUANT   deq = deq_scale_per_oc[n] if set, else deq_scale
 *     r = r + bias[n]                         MMX_PP_BIAS
 *     r = gelu_erf_minimax(r)                 MMX_PP_GELU      (include/kernels_amx.hpp:242-289)
 *     r = r * q                               MMX_PP_QUANT     q = q_scale_per_oc[n] if set, else q_scale
 *     store: MMX_F32 as is; MMX_BF16 round-to-nearest-even; MMX_I8 round-to-nearest-even then
 *            saturate to [-128,127]; MMX_I32 (only with steps == 0 on int8 inputs) raw accumulator.
 * With MMX_PP_SILU_GATE the packed weights hold gate and up projections in alternating
 * 32-column panels (see mmx_repack_gate_up) and the output has half as many columns:
 *     C[m, c] = bf16( silu(acc_gate[m, c]) * acc_up[m, c] )   (BIAS/GELU/QUANT must be off)
 * over compressed weights (int8, int4) MMX_PP_DEQUANT may be set with it (an extension, the reference's MLP is
 * bf16 only): each sum is first multiplied by the dequant scale of its own packed column,
 *     C[m, c] = bf16( silu(acc_gate * deq[gate column]) * (acc_up * deq[up column]) )
 * deq_scale_per_oc is an extension: the reference has a per-tensor dequant scale only.
 */
typedef struct mmx_epilogue {
    uint32_t steps;
    int32_t out_dtype;
    void* C;            /* device, [M, n1-n0 columns starting at column n0 of the full C row] */
    int64_t ldc_bytes;  /* row stride of C in bytes; C points at row 0, column 0 of the FULL matrix */
    const float* bias;  /* device [N] */
    float deq_scale;
    const float* deq_scale_per_oc; /* device [N] or NULL */
    float q_scale;
    const float* q_scale_per_oc;   /* device [N] or NULL */
} mmx_epilogue;

/* message for the last failing call made by this thread ("" if none) */
const char* mmx_last_error(void);

/* Selects `device` and checks that it is a gfx950.  Idempotent, callable from any thread.  (Kernels that need
 * more than 64 KiB of LDS have their limit raised at their first launch on a device, under a lock.)
 * Stands in for initXTILE() (include/misc.hpp:376-396), the reference's one-time set-up. */
int mmx_init(int device);

/* ---- weight repack: amx_kernel::repackB_1x2 (include/kernels_amx.hpp:761-816) --------------
 * B is [K, N] (transpose = 0) or [N, K] (transpose = 1, the torch nn.Linear.weight layout),
 * row stride ldb_bytes, dtype MMX_BF16 or MMX_I8.  The result is in MFMA-fragment order:
 *     packed[panel = n/32][kstep = k/KS][lane 0..63][16 bytes],  KS = 16 (bf16) / 32 (int8),
 *     lane = n%32 + 32*((k%KS)/(KS/2)),  byte offset in the lane = (k%(KS/2))*sizeof(T),
 * zero padded in K up to a multiple of 128 bytes per column and in N up to a multiple of 32.
 * dtype MMX_U8 (unsigned weights, for mmx_gemm_u8): the int8 layout holding u - 128, i.e. every byte with its sign
 * bit inverted (the padding stays zero). */
size_t mmx_packed_b_bytes(int dtype, int K, int N);
int mmx_repack_b(int dtype, const void* B, int64_t ldb_bytes, int K, int N, int transpose, void* packed,
                 void* stream);

/* MLP::setup (tests/amx-mlp.cpp:752-766): interleaves W_gate and W_up (both [N, K] bf16,
 * torch layout) into one packed matrix of 2N columns, alternating 32-column panels
 * (gate panel p, up panel p), for use with MMX_PP_SILU_GATE.  N % 32 == 0. */
int mmx_repack_gate_up(const void* w_gate, const void* w_up, int64_t ldw_bytes, int K, int N, void* packed,
                       void* stream);

/* Weight compression of amx_kernel::Matmul<bf16,int8,float> (include/kernels_amx.hpp:1363-1377,
 * 465-523): per-tensor symmetric quantisation of a bf16 matrix [rows, cols] to int8, scale
 * 127/max|w|.  scales_out (device, 2 floats) receives {quant_scale, dequant_scale};
 * absmax_scratch is a device uint32 the call uses as scratch. */
int mmx_quantize_weights(const void* W, int64_t ldw_bytes, int rows, int cols, void* Wq, int64_t ldq_bytes,
                         float* scales_out, uint32_t* absmax_scratch, void* stream);

/* The quantising half of repackB_1xL<int8_t, L> (weight_compression/fc16m.cpp:61-99), the way fc16m makes its int8
 * weights (:123, :630-649 with quantize_i8_scale, :51): q = trunc(bf16_rne(float(w) * scale)) per element - the
 * product is rounded to bf16 first (ov::bfloat16::operator*, include/bf16.hpp:181-183), then converted toward zero
 * (:80-81).  Where the reference's conversion is undefined the result is defined here: values beyond int8's range
 * saturate, NaN gives 0.  W is [rows, cols] bf16, Wq [rows, cols] int8; the tile order of that function is
 * replaced by mmx_repack_b on Wq, and the kernels' per-tensor dequant scale is 1 / scale (:280). */
int mmx_quantize_weights_scaled(const void* W, int64_t ldw_bytes, int rows, int cols, float scale, void* Wq,
                                int64_t ldq_bytes, void* stream);

/* int4 weight compression.  The reference only times a stand-in that copies bytes
 * (weight_compression/wcompress.hpp:90-134, README.md:216-244: "we haven't found efficient instructions to
 * implement a fully-functional dequant() for INT4"); this is the real thing for the decode path.  Per output
 * channel n, symmetric: a = max_k |w[k][n]|, q[k][n] = clamp(rint(w[k][n] * (7 / a)), -7, 7) in fp32 (q = 0 for
 * a = 0), deq_scales_out[n] = a / 7.  Non-finite weights: NaNs do not take part in the maximum; a NaN weight, and
 * every infinite weight (its column has a = inf, so 7 / a = 0 and the product is NaN), quantises to 0, and such a
 * column's deq scale is inf.  W is [K, N] bf16 (transpose = 0) or [N, K] (transpose = 1, torch layout),
 * row stride ldw_bytes.  packed receives mmx_packed_b_bytes(MMX_I4, K, N) bytes: 32-column panels of 1 KiB
 * fragments, a fragment = 32 columns x 64 of k; the lane g * 32 + c (c = column in the panel, g = 0, 1) owns
 * bytes [16 (g*32+c), +16): dword i holds k = 64 f + 32 g + 8 i + e in bits [4e, 4e+4), two's complement;
 * K is padded with zeros to a multiple of 256.  Use: mmx_gemm(MMX_BF16, MMX_I4, ...) with M <= 32 and
 * MMX_PP_DEQUANT with deq_scale_per_oc = deq_scales_out; the accumulators equal those of the bf16 GEMM on the
 * (exactly representable) integers q. */
int mmx_quantize_pack_int4(const void* W, int64_t ldw_bytes, int K, int N, int transpose, void* packed,
                           float* deq_scales_out, void* stream);

/* int8 packed weights -> bf16 packed weights (exact): the conversion of include/kernels_amx.hpp:490-506 as a
 * one-off, for callers that want a bf16 copy of compressed weights (mmx_gemm itself converts on the fly). */
int mmx_dequant_packed(const void* packed_i8, int K, int N, void* packed_bf16, void* stream);

/* ---- C[:, n0:n1] = PP( A · B[:, n0:n1] ): amx_kernel::Matmul<TA,TB,TC>::operator()
 * (include/kernels_amx.hpp:1169-1314; int8-weight specialisation :1319-1516) -----------------
 * a_dtype/b_dtype: (BF16,BF16), (I8,I8), (BF16,I8) = bf16 activations on int8-compressed weights, converted to
 * bf16 in registers on their way to the MFMA (exact; any M: :1381-1441 for small M, :1447-1497 for large M;
 * tiles of 128 or 256 columns), or (BF16,I4) = int4-compressed weights (M <= 32 only).
 * A is [M, K] row-major with row stride lda_bytes; Bpacked comes from mmx_repack_b for the
 * FULL [K, N]; n0 % 32 == 0, 0 <= n0 < n1 <= N.  M <= 32 takes the bandwidth-bound decode
 * kernel (the M<=16 paths of the reference and weight_compression/fc16m.cpp:451-502), larger
 * M the MFMA tile kernel. */
int mmx_gemm(int a_dtype, int b_dtype, const void* A, int64_t lda_bytes, const void* Bpacked, int M, int K,
             int N, int n0, int n1, const mmx_epilogue* ep, void* stream);

/* ---- the same product with K split over several workgroups per output tile ---------------------------------
 * AMX_MLP::Linear (tests/amx-mlp.cpp:560-593) gives each half of the K blocks of `down` to its own core and lets
 * the one that finishes last add the two fp32 partial results and round to bf16 (:648-682).  Here a tile's K range
 * is cut into k_splits slices of whole 512-byte blocks of K per row (256 bf16, the reference's K block; slice s
 * takes blocks [s*q, (s+1)*q), q = ceil(blocks / k_splits), so k_splits = 2 is the reference's partition), one
 * workgroup each; each parks its fp32 / int32 partial tile in `workspace`, and the workgroup that arrives last
 * adds them in slice order (so the result does not depend on the arrival order) and applies the post-op.  It
 * pays where a shape has fewer tiles than the GPU has CUs, or tiles bound by the bytes a CU can pull in.
 *   k_splits  0 = the library chooses (possibly no split), 1 = none, 2..4 = exactly that many slices
 *             (MMX_E_INVALID if K is too short or the workspace too small, MMX_E_UNSUPPORTED for M <= 32,
 *             SILU_GATE, unaligned A or K * sizeof(T) not a multiple of 128).  The decode kernels (M <= 32)
 *             take 0 or 1 only: with 0 and a workspace, launches over bf16, int8 or int4 weights whose x does
 *             not fit in LDS and whose column range has 32-column panels for at most two thirds of the CUs walk K in
 *             2-4 slices of their own choosing, combined the same way (same layout of the workspace).
 *   workspace device memory, 256-byte aligned, mmx_gemm_workspace_bytes() or more (64 MiB + 16 KiB always
 *             suffices for k_splits = 0; with less, the choice is restricted to what fits).  Its first 16 KiB are
 *             arrival counters: zero them once after allocation; every call leaves them zero.  Calls that share
 *             a workspace must not overlap in time (different streams need different workspaces).
 * With workspace = NULL this is mmx_gemm. */
int mmx_gemm_splitk(int a_dtype, int b_dtype, const void* A, int64_t lda_bytes, const void* Bpacked, int M, int K,
                    int N, int n0, int n1, const mmx_epilogue* ep, int k_splits, void* workspace,
                    size_t workspace_bytes, void* stream);
/* Workspace the call above would use for this shape (0 if it would not split).  steps = the post-op steps.  For decode
 * shapes (M <= 32) the figure is an upper bound: it looks at the number of panels and the length of K only, and a launch
 * whose x fits in LDS, or whose K or alignment takes another kernel, does not split after all.  The answer depends on the
 * device's CU count: call mmx_init first. */
size_t mmx_gemm_workspace_bytes(int a_dtype, int b_dtype, int M, int K, int N, int n0, int n1, uint32_t steps,
                                int k_splits);

/* mmx_gemm_splitk for callers that cannot allocate device memory (code under HIP graph capture, serving loops,
 * harnesses that forbid hipMalloc).  No counterpart in the reference.  The workspace is a 64 MiB + 16 KiB array
 * built into the library, one copy per GPU, held until the process ends; the call allocates and frees nothing.
 * Same arguments, results and errors as mmx_gemm_splitk with a workspace of that size (so k_splits = 0 always
 * fits; an explicit k_splits whose partial tiles need more returns MMX_E_INVALID and says how much).  mmx_init()
 * must have been called for the current device.  The array is shared by every call on that GPU and keeps the last
 * call's partial sums; its arrival counters are zero when the library is loaded and every completed call leaves
 * them zero.  Calls that overlap in time on one GPU (two streams, two threads) race on it: use mmx_gemm_splitk
 * with a workspace per stream there. */
int mmx_gemm_splitk_static(int a_dtype, int b_dtype, const void* A, int64_t lda_bytes, const void* Bpacked, int M,
                           int K, int N, int n0, int n1, const mmx_epilogue* ep, int k_splits, void* stream);

/* ---- c[M] = A[M, K] · b[K]: amx_kernel::MatmulVector::operator() (include/kernels_amx.hpp:959)
 * and amx_kernel::GemAvB::operator() (:1534).  dtype MMX_BF16 (c fp32) or MMX_I8 (c int32). */
int mmx_matvec(int dtype, const void* A, int64_t lda_bytes, const void* b, void* c, int M, int K, void* stream);

/* ---- the unsigned 8-bit forms: amx_kernel::Matmul<uint8_t|int8_t, uint8_t|int8_t> (tdpbusd / tdpbsud / tdpbuud,
 * include/kernels_amx.hpp:1057-1101, accumulator int32 :825) and amx_kernel::MatmulVector in the same forms
 * (:839-850).  a_dtype / b_dtype are MMX_I8 or MMX_U8, at least one of them MMX_U8.  (In the reference only
 * Matmul<uint8_t, int8_t> can be instantiated - its repackB_1x2 has no uint8_t form, :293, :393, :810 - and all three
 * MatmulVector forms; here all combinations exist.)  The matrix cores multiply signed bytes, so an unsigned operand
 * u is computed as (u - 128) + 128: Bpacked comes from mmx_repack_b with the dtype of B (MMX_U8 stores u - 128), A is
 * shifted per call, the signed product runs through the int8 kernels of mmx_gemm into int32 scratch, and a last pass
 * adds 128 x the column sums of the weights / row sums of the activations (+ 16384 K when both are unsigned), in
 * int32 arithmetic modulo 2^32 like the AMX accumulators, and applies the post-op `ep` (as for mmx_gemm on int8
 * inputs; MMX_I32 output = the raw sums).  Exact; three launches more than mmx_gemm.
 * scratch: device memory, 256-byte aligned, mmx_gemm_u8_scratch_bytes() bytes, free to reuse once the call's work on
 * `stream` has finished (0 from the query = arguments it does not take). */
size_t mmx_gemm_u8_scratch_bytes(int a_dtype, int b_dtype, int M, int K, int N, int n0, int n1);
int mmx_gemm_u8(int a_dtype, int b_dtype, const void* A, int64_t lda_bytes, const void* Bpacked, int M, int K, int N,
                int n0, int n1, const mmx_epilogue* ep, void* scratch, size_t scratch_bytes, void* stream);
/* c[M] (int32) = A[M, K] . b[K] with A and b each signed or unsigned bytes (at least one MMX_U8). */
int mmx_matvec_u8(int a_dtype, int b_dtype, const void* A, int64_t lda_bytes, const void* b, void* c, int M, int K,
                  void* stream);

/* ---- fused Llama MLP: AMX_MLP::MLP::run (tests/amx-mlp.cpp:778-783) ---------------------------
 * x [M, K] bf16; w_gate_up from mmx_repack_gate_up (K x 2N); w_down from mmx_repack_b of the
 * [K, N] torch down_proj weight with transpose = 1 (so it is an N x K "B"); h is caller
 * scratch [M, N] bf16; y [M, K] bf16.  Two launches on `stream`: gate/up GEMM with the SiLU*up
 * epilogue, then down GEMM. */
int mmx_mlp(const void* x, int64_t ldx_bytes, const void* w_gate_up, const void* w_down, void* h, int64_t ldh_bytes,
            void* y, int64_t ldy_bytes, int M, int K, int N, void* stream);

/* The same with the down projection's K split over `down_k_splits` slices (0 = the library chooses, 2 = the
 * reference's do_splitK, tests/amx-mlp.cpp:768 and :560-593); workspace as for mmx_gemm_splitk.  workspace = NULL
 * runs without slices; at M <= 32 (decode kernels) the library chooses unless down_k_splits = 1. */
int mmx_mlp_splitk(const void* x, int64_t ldx_bytes, const void* w_gate_up, const void* w_down, void* h,
                   int64_t ldh_bytes, void* y, int64_t ldy_bytes, int M, int K, int N, int down_k_splits,
                   void* workspace, size_t workspace_bytes, void* stream);

/* ---- introspection / tuning (no reference counterpart) --------------------------------------- */
/* Force the MFMA tile shape ("256x256", "256x192", "128x256", "128x192", "128x128", "128x64", "64x128" (aligned
 * operands and no SILU_GATE only; otherwise 128x128 is used), "" = automatic)
 * for the calling thread's later calls. */
int mmx_set_tile(const char* shape);
/* Name of the kernel variant the last mmx_gemm call of this thread launched. */
const char* mmx_last_kernel(void);
/* Sets a kernel option.  "load_mode": how the MFMA tile kernel brings A and B tiles into LDS —
 * 2 (default) direct HBM->LDS loads in a hand-scheduled ring pipeline, 0 through registers (the
 * fallback for operands beyond 32-bit offsets).  Shapes whose K tail or alignment need masked
 * loads use a masked kernel whatever this is set to.  "decode_halves": whether the streaming decode
 * kernel for M <= 4 splits every 32-column panel over two workgroups — -1 (default) where that fills the
 * CUs better, 0 never, 1 always while x takes at most 46 KiB of LDS (the two forms add the partial sums in
 * different orders).  "waves": 8 (default) lets the 256x192 tile kernel run as eight wavefronts per
 * workgroup, 4 keeps the four-wavefront form (same results).  "decode_valu": whether the
 * streaming decode kernel at M = 1 over int8-compressed weights uses v_dot2_f32_bf16 and a cross-lane add
 * instead of the matrix cores — -1 (default) where at most one workgroup per CU is launched (it is the faster form
 * there), 0 never, 1 always; the two forms agree to fp32 summation order.  "decode_resident": whether a decode
 * launch (M <= 32; K = 4096, 5120, 8192 or 11008 over int8-compressed weights, 2048 or 4096 over bf16 weights; at
 * most two 32-column panels per CU; x within a CU's LDS) runs as one workgroup per CU that keeps x in LDS and walks
 * its one or two panels — -1 (default) where x is too large for the streaming kernel's two workgroups per CU and,
 * over int8 weights, wherever no workgroup gets a second panel (and only while decode_halves and decode_valu are
 * left at -1); 0 never; 1 wherever the shape allows (same bits as the streaming kernel).  "decode_pair": how that
 * kernel walks a workgroup's second panel over int8-compressed weights — 1 (default) a second group of eight waves walks
 * it at the same time as the first panel, against the same copy of x; 0 the same eight waves walk it after the first
 * (same bits either way). */
int mmx_set_option(const char* name, int value);  /* like mmx_set_tile: affects the calling thread's later calls only */
#ifdef __cplusplus
}
#endif
#endif
