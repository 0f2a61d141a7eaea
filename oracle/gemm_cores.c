/*
 * gemm_cores.c — accumulation cores of the CPU oracle (TEST INFRASTRUCTURE ONLY).
 *
 * Built with floating-point contraction allowed: every product formed here is a product of
 * two bf16 values (8-bit significands), which is exact in fp32, so a fused multiply-add and
 * a multiply followed by an add round identically.  Nothing else in this file multiplies.
 */
#include "fc_oracle.h"

#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define CLONES __attribute__((target_clones("avx512f", "avx2", "default")))

typedef float v16f __attribute__((vector_size(64)));
typedef double v8d __attribute__((vector_size(64)));
typedef int32_t v16i __attribute__((vector_size(64)));

static inline __attribute__((always_inline)) v16f ld16f(const float* p) { v16f v; memcpy(&v, p, sizeof v); return v; }
static inline __attribute__((always_inline)) void st16f(float* p, v16f v) { memcpy(p, &v, sizeof v); }
static inline __attribute__((always_inline)) v16i ld16i(const int32_t* p) { v16i v; memcpy(&v, p, sizeof v); return v; }

static inline float bf16_as_f32(uint16_t b) {
    uint32_t u = (uint32_t)b << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

static int pick_threads(int nthreads) {
#ifdef _OPENMP
    return nthreads > 0 ? nthreads : omp_get_max_threads();
#else
    (void)nthreads;
    return 1;
#endif
}

/* B (bf16, [K,N] or [N,K]) -> fp32 [K][Np], Np = N rounded up to 16, zero padded. */
static float* widen_b(const uint16_t* B, int64_t ldb, int transB, int K, int N, int Np, int nt) {
    float* Bf = (float*)aligned_alloc(64, (size_t)K * Np * sizeof(float));
    if (!Bf) return NULL;
#pragma omp parallel for num_threads(nt) schedule(static)
    for (int k = 0; k < K; k++) {
        float* row = Bf + (size_t)k * Np;
        if (!transB) {
            const uint16_t* src = B + (size_t)k * ldb;
            for (int n = 0; n < N; n++) row[n] = bf16_as_f32(src[n]);
        } else {
            for (int n = 0; n < N; n++) row[n] = bf16_as_f32(B[(size_t)n * ldb + k]);
        }
        for (int n = N; n < Np; n++) row[n] = 0.0f;
    }
    return Bf;
}

#define MR 4

/*
 * One 16-column strip of C for rows [m0, m0+mr).
 *
 * Accumulation order = what AMX tdpbf16ps does when driven by the reference's kernels
 * (include/kernels_amx.hpp:1262-1275 large M, :1229-1237 M<=16; tests/amx-mlp.cpp:273-317):
 * K is walked in blocks of 32; inside a block the even-k products are summed in k order
 * into one fp32 partial, the odd-k products into another, and (even + odd) is then added
 * to the running accumulator.  This is the ordering of the reference's own scalar check,
 * include/tensor2D.hpp:345-357.
 *
 * K tail (include/kernels_amx.hpp:1276-1289 with the repack at :326-338 / :415-425): the
 * last A tile is loaded backed off to start at K-32 and the B tile holds the tail rows
 * bottom-aligned under zero rows, so the products that matter sit at slot (k - (K-32)) of
 * the tile; the slot's parity, not k's, decides which partial they join.
 */
CLONES static void strip_amx_order(const float* Af, int64_t lda, const float* Bf, int Np, int K,
                                   int mr, float* out /* [mr][16] */) {
    const int Kbody = K - (K % 32);
    v16f acc[MR];
    for (int r = 0; r < MR; r++) acc[r] = (v16f){0};
    for (int kb = 0; kb < Kbody; kb += 32) {
        v16f p0[MR], p1[MR];
        for (int r = 0; r < MR; r++) { p0[r] = (v16f){0}; p1[r] = (v16f){0}; }
        for (int p = 0; p < 32; p += 2) {
            const v16f b0 = ld16f(Bf + (size_t)(kb + p) * Np);
            const v16f b1 = ld16f(Bf + (size_t)(kb + p + 1) * Np);
            for (int r = 0; r < mr; r++) {
                const float a0 = Af[r * lda + kb + p];
                const float a1 = Af[r * lda + kb + p + 1];
                p0[r] += a0 * b0;
                p1[r] += a1 * b1;
            }
        }
        for (int r = 0; r < mr; r++) acc[r] += (p0[r] + p1[r]);
    }
    if (K != Kbody) {
        const int kt0 = K - 32; /* first k of the backed-off tile */
        v16f p0[MR], p1[MR];
        for (int r = 0; r < MR; r++) { p0[r] = (v16f){0}; p1[r] = (v16f){0}; }
        for (int k = Kbody; k < K; k++) {
            const int slot = k - kt0;
            const v16f b = ld16f(Bf + (size_t)k * Np);
            for (int r = 0; r < mr; r++) {
                const float a = Af[r * lda + k];
                if (slot & 1) p1[r] += a * b; else p0[r] += a * b;
            }
        }
        for (int r = 0; r < mr; r++) acc[r] += (p0[r] + p1[r]);
    }
    for (int r = 0; r < mr; r++) st16f(out + r * 16, acc[r]);
}

static float* widen_a(const uint16_t* A, int64_t lda, int M, int K, int nt) {
    float* Af = (float*)aligned_alloc(64, (((size_t)M * K * sizeof(float)) + 63) / 64 * 64);
    if (!Af) return NULL;
#pragma omp parallel for num_threads(nt) schedule(static)
    for (int m = 0; m < M; m++)
        for (int k = 0; k < K; k++) Af[(size_t)m * K + k] = bf16_as_f32(A[(size_t)m * lda + k]);
    return Af;
}

void orc_gemm_bf16(const uint16_t* A, int64_t lda, const uint16_t* B, int64_t ldb, int transB,
                   float* C, int64_t ldc, int M, int K, int N, int nthreads) {
    const int nt = pick_threads(nthreads);
    const int Np = (N + 15) / 16 * 16;
    float* Bf = widen_b(B, ldb, transB, K, N, Np, nt);
    float* Af = widen_a(A, lda, M, K, nt);
    if (!Bf || !Af) abort();
    const int nblk = Np / 16;
#pragma omp parallel for num_threads(nt) schedule(dynamic, 1)
    for (int nb = 0; nb < nblk; nb++) {
        float tmp[MR * 16];
        const int ncols = (N - nb * 16) < 16 ? (N - nb * 16) : 16;
        for (int m0 = 0; m0 < M; m0 += MR) {
            const int mr = (M - m0) < MR ? (M - m0) : MR;
            strip_amx_order(Af + (size_t)m0 * K, K, Bf + nb * 16, Np, K, mr, tmp);
            for (int r = 0; r < mr; r++)
                memcpy(C + (size_t)(m0 + r) * ldc + nb * 16, tmp + r * 16, ncols * sizeof(float));
        }
    }
    free(Bf);
    free(Af);
}

/* Independent check: the same product accumulated in double, rounded once. */
CLONES static void strip_f64(const float* Af, int64_t lda, const float* Bf, int Np, int K, int mr,
                             float* out) {
    for (int r = 0; r < mr; r++) {
        v8d lo = (v8d){0}, hi = (v8d){0};
        for (int k = 0; k < K; k++) {
            const double a = Af[r * lda + k];
            const float* b = Bf + (size_t)k * Np;
            for (int j = 0; j < 8; j++) { lo[j] += a * (double)b[j]; hi[j] += a * (double)b[8 + j]; }
        }
        for (int j = 0; j < 8; j++) { out[r * 16 + j] = (float)lo[j]; out[r * 16 + 8 + j] = (float)hi[j]; }
    }
}

void orc_gemm_bf16_f64(const uint16_t* A, int64_t lda, const uint16_t* B, int64_t ldb, int transB,
                       float* C, int64_t ldc, int M, int K, int N, int nthreads) {
    const int nt = pick_threads(nthreads);
    const int Np = (N + 15) / 16 * 16;
    float* Bf = widen_b(B, ldb, transB, K, N, Np, nt);
    float* Af = widen_a(A, lda, M, K, nt);
    if (!Bf || !Af) abort();
    const int nblk = Np / 16;
#pragma omp parallel for num_threads(nt) schedule(dynamic, 1)
    for (int nb = 0; nb < nblk; nb++) {
        float tmp[MR * 16];
        const int ncols = (N - nb * 16) < 16 ? (N - nb * 16) : 16;
        for (int m0 = 0; m0 < M; m0 += MR) {
            const int mr = (M - m0) < MR ? (M - m0) : MR;
            strip_f64(Af + (size_t)m0 * K, K, Bf + nb * 16, Np, K, mr, tmp);
            for (int r = 0; r < mr; r++)
                memcpy(C + (size_t)(m0 + r) * ldc + nb * 16, tmp + r * 16, ncols * sizeof(float));
        }
    }
    free(Bf);
    free(Af);
}

/* ------------------------------------------------------------------------------------------------------------
 * matmul16m_Wint8B as a weight stream (weight_compression/fc16m.cpp:451-502, N split over threads as
 * MultiThreaded<int8_t>, :620-663).  The weights are packed once, ahead of time, in the order of repackB_1xL<int8_t,2>
 * (:61-99: 32-column groups in computation order, K in blocks of 32, two tiles per block, a tile = 16 pairs of k x
 * 16 columns x (k, k + 1)), so a thread reads one contiguous stream; at call time every int8 weight is read once,
 * converted in registers (deq_Kx32, :309-333: exact, |w| <= 128 has eight significant bits) and multiplied into the
 * running sums.  Same accumulation order as the AMX chain above (blocks of 32 k, even and odd k summed apart, then
 * added to the accumulator): the result is bit for bit that of orc_gemv_w8, which the tests pin.
 * K % 32 == 0, N % 32 == 0, M <= 16. */
void orc_pack_1x2_s8(const int8_t* W, int64_t ldw, int K, int N, int8_t* out) {
    int8_t* dst = out;
    for (int n0 = 0; n0 < N; n0 += 32)
        for (int k0 = 0; k0 < K; k0 += 32)
            for (int l = 0; l < 2; l++)
                for (int k = 0; k < 32; k += 2)
                    for (int n = 0; n < 16; n++) {
                        *dst++ = W[(size_t)(k0 + k) * ldw + n0 + l * 16 + n];
                        *dst++ = W[(size_t)(k0 + k + 1) * ldw + n0 + l * 16 + n];
                    }
}

typedef int16_t v16h __attribute__((vector_size(32)));
/* 16 columns x (k, k + 1) interleaved -> the 16 weights of k and the 16 of k + 1, as fp32 */
static inline __attribute__((always_inline)) void ld_pair(const int8_t* p, v16f* even, v16f* odd) {
    v16h v;
    memcpy(&v, p, sizeof v);
    const v16h lo = (v16h)((v16h)(v << 8) >> 8), hi = v >> 8;  /* sign-extended low / high bytes (little endian) */
    *even = __builtin_convertvector(lo, v16f);
    *odd = __builtin_convertvector(hi, v16f);
}

#define GMR 4
CLONES static void gemv_group32(const float* xf, int64_t ldx, const int8_t* Wp /* this group's stream */, int K, int mr,
                                float* out /* [mr][32] */) {
    v16f acc[GMR][2];
    for (int r = 0; r < GMR; r++) acc[r][0] = acc[r][1] = (v16f){0};
    for (int kb = 0; kb < K; kb += 32, Wp += 1024) {
        v16f p0[GMR][2], p1[GMR][2];
        for (int r = 0; r < GMR; r++) p0[r][0] = p0[r][1] = p1[r][0] = p1[r][1] = (v16f){0};
        for (int p = 0; p < 16; p++) {
            v16f b0a, b1a, b0b, b1b;
            ld_pair(Wp + p * 32, &b0a, &b1a);        /* tile 0: columns 0..15 */
            ld_pair(Wp + 512 + p * 32, &b0b, &b1b);  /* tile 1: columns 16..31 */
            for (int r = 0; r < mr; r++) {
                const float a0 = xf[r * ldx + kb + 2 * p], a1 = xf[r * ldx + kb + 2 * p + 1];
                p0[r][0] += a0 * b0a;
                p0[r][1] += a0 * b0b;
                p1[r][0] += a1 * b1a;
                p1[r][1] += a1 * b1b;
            }
        }
        for (int r = 0; r < mr; r++) {
            acc[r][0] += (p0[r][0] + p1[r][0]);
            acc[r][1] += (p0[r][1] + p1[r][1]);
        }
    }
    for (int r = 0; r < mr; r++) {
        st16f(out + r * 32, acc[r][0]);
        st16f(out + r * 32 + 16, acc[r][1]);
    }
}

int orc_gemv_w8_stream(const uint16_t* x, int64_t ldx, const int8_t* Wpacked, const float* scale, uint16_t* y,
                       int64_t ldy, int M, int K, int N, int nthreads) {
    if (K % 32 || N % 32 || M < 1 || M > 16) return -1;
    const int nt = pick_threads(nthreads);
    float* xf = widen_a(x, ldx, M, K, 1);
    if (!xf) abort();
    const int groups = N / 32;
#pragma omp parallel num_threads(nt)
    {
#ifdef _OPENMP
        const int t = omp_get_thread_num(), team = omp_get_num_threads();
#else
        const int t = 0, team = 1;
#endif
        int g0, g1;
        orc_splitter(groups, team, t, &g0, &g1);
        float tmp[GMR * 32];
        for (int g = g0; g < g1; g++) {
            const int n0 = g * 32;
            for (int m0 = 0; m0 < M; m0 += GMR) {
                const int mr = M - m0 < GMR ? M - m0 : GMR;
                gemv_group32(xf + (size_t)m0 * K, K, Wpacked + (size_t)g * K * 32, K, mr, tmp);
                for (int r = 0; r < mr; r++)
                    for (int c = 0; c < 32; c++)  /* scale_Kx16 (fc16m.cpp:349-359): one rounded multiply, then bf16 */
                        y[(size_t)(m0 + r) * ldy + n0 + c] = orc_f32_to_bf16(tmp[r * 32 + c] * scale[n0 + c]);
            }
        }
    }
    free(xf);
    return 0;
}

/* int8 x int8 -> int32: tdpbssd (include/kernels_amx.hpp:1096-1101) is exact integer
 * arithmetic, so any order gives the reference's accumulators. */
CLONES static void strip_i8(const int8_t* A, int64_t lda, const int32_t* Bi, int Np, int K, int mr,
                            int32_t* out) {
    v16i acc[MR];
    for (int r = 0; r < MR; r++) acc[r] = (v16i){0};
    for (int k = 0; k < K; k++) {
        const v16i b = ld16i(Bi + (size_t)k * Np);
        for (int r = 0; r < mr; r++) acc[r] += (int32_t)A[r * lda + k] * b;
    }
    for (int r = 0; r < mr; r++) memcpy(out + r * 16, &acc[r], 64);
}

/* The same sums with AVX-512BW: B widened once to int16 pairs [K/2][Np][(k, k + 1)], a row's pair (a[k], a[k + 1])
 * broadcast, vpmaddwd forms a[k] b[k] + a[k + 1] b[k + 1] exactly in int32 (|products| <= 2^14).  Integer sums are
 * the same in any order, so this is the function above, faster. */
#include <immintrin.h>
__attribute__((target("avx512f,avx512bw"))) static void strip_i8_madd(const int8_t* A, int64_t lda, const int16_t* Bp, int Np, int K2,
                                                                       int mr, int32_t* out) {
    __m512i acc[MR];
    for (int r = 0; r < MR; r++) acc[r] = _mm512_setzero_si512();
    for (int k2 = 0; k2 < K2; k2++) {
        const __m512i b = _mm512_loadu_si512((const void*)(Bp + ((size_t)k2 * Np) * 2));
        for (int r = 0; r < mr; r++) {
            const int a0 = A[r * lda + 2 * k2], a1 = A[r * lda + 2 * k2 + 1];
            const __m512i ap = _mm512_set1_epi32((int)(((uint32_t)(uint16_t)(int16_t)a1 << 16) | (uint16_t)(int16_t)a0));
            acc[r] = _mm512_add_epi32(acc[r], _mm512_madd_epi16(ap, b));
        }
    }
    for (int r = 0; r < mr; r++) _mm512_storeu_si512((void*)(out + r * 16), acc[r]);
}

void orc_gemm_i8(const int8_t* A, int64_t lda, const int8_t* B, int64_t ldb, int transB, int32_t* C,
                 int64_t ldc, int M, int K, int N, int nthreads) {
    const int nt = pick_threads(nthreads);
    const int Np = (N + 15) / 16 * 16;
    __builtin_cpu_init();
    const int fast = __builtin_cpu_supports("avx512bw") && K % 2 == 0;
    int32_t* Bi = NULL;
    int16_t* Bp = NULL;
    if (fast) {
        Bp = (int16_t*)aligned_alloc(64, (size_t)K * Np * sizeof(int16_t));
        if (!Bp) abort();
#pragma omp parallel for num_threads(nt) schedule(static)
        for (int k2 = 0; k2 < K / 2; k2++) {
            int16_t* row = Bp + (size_t)k2 * Np * 2;
            for (int n = 0; n < Np; n++)
                for (int e = 0; e < 2; e++) {
                    const int k = 2 * k2 + e;
                    row[2 * n + e] = n < N ? (transB ? B[(size_t)n * ldb + k] : B[(size_t)k * ldb + n]) : 0;
                }
        }
    } else {
        Bi = (int32_t*)aligned_alloc(64, (size_t)K * Np * sizeof(int32_t));
        if (!Bi) abort();
#pragma omp parallel for num_threads(nt) schedule(static)
        for (int k = 0; k < K; k++) {
            int32_t* row = Bi + (size_t)k * Np;
            for (int n = 0; n < N; n++) row[n] = transB ? B[(size_t)n * ldb + k] : B[(size_t)k * ldb + n];
            for (int n = N; n < Np; n++) row[n] = 0;
        }
    }
    const int nblk = Np / 16;
#pragma omp parallel for num_threads(nt) schedule(dynamic, 1)
    for (int nb = 0; nb < nblk; nb++) {
        int32_t tmp[MR * 16];
        const int ncols = (N - nb * 16) < 16 ? (N - nb * 16) : 16;
        for (int m0 = 0; m0 < M; m0 += MR) {
            const int mr = (M - m0) < MR ? (M - m0) : MR;
            if (fast) strip_i8_madd(A + (size_t)m0 * lda, lda, Bp + (size_t)nb * 32, Np, K / 2, mr, tmp);
            else strip_i8(A + (size_t)m0 * lda, lda, Bi + nb * 16, Np, K, mr, tmp);
            for (int r = 0; r < mr; r++)
                memcpy(C + (size_t)(m0 + r) * ldc + nb * 16, tmp + r * 16, ncols * sizeof(int32_t));
        }
    }
    free(Bi);
    free(Bp);
}

/* the generic form on its own, for the test that holds the fast one to it */
void orc_gemm_i8_generic(const int8_t* A, int64_t lda, const int8_t* B, int64_t ldb, int transB, int32_t* C,
                         int64_t ldc, int M, int K, int N) {
    const int Np = (N + 15) / 16 * 16;
    int32_t* Bi = (int32_t*)aligned_alloc(64, (size_t)K * Np * sizeof(int32_t));
    if (!Bi) abort();
    for (int k = 0; k < K; k++) {
        int32_t* row = Bi + (size_t)k * Np;
        for (int n = 0; n < N; n++) row[n] = transB ? B[(size_t)n * ldb + k] : B[(size_t)k * ldb + n];
        for (int n = N; n < Np; n++) row[n] = 0;
    }
    for (int nb = 0; nb < Np / 16; nb++) {
        int32_t tmp[MR * 16];
        const int ncols = (N - nb * 16) < 16 ? (N - nb * 16) : 16;
        for (int m0 = 0; m0 < M; m0 += MR) {
            const int mr = (M - m0) < MR ? (M - m0) : MR;
            strip_i8(A + (size_t)m0 * lda, lda, Bi + nb * 16, Np, K, mr, tmp);
            for (int r = 0; r < mr; r++)
                memcpy(C + (size_t)(m0 + r) * ldc + nb * 16, tmp + r * 16, ncols * sizeof(int32_t));
        }
    }
    free(Bi);
}

const char* orc_isa(void) {
    __builtin_cpu_init();
    if (__builtin_cpu_supports("avx512f")) return "avx512f";
    if (__builtin_cpu_supports("avx2")) return "avx2";
    return "generic";
}
