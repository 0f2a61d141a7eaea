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

void orc_gemm_i8(const int8_t* A, int64_t lda, const int8_t* B, int64_t ldb, int transB, int32_t* C,
                 int64_t ldc, int M, int K, int N, int nthreads) {
    const int nt = pick_threads(nthreads);
    const int Np = (N + 15) / 16 * 16;
    int32_t* Bi = (int32_t*)aligned_alloc(64, (size_t)K * Np * sizeof(int32_t));
    if (!Bi) abort();
#pragma omp parallel for num_threads(nt) schedule(static)
    for (int k = 0; k < K; k++) {
        int32_t* row = Bi + (size_t)k * Np;
        for (int n = 0; n < N; n++) row[n] = transB ? B[(size_t)n * ldb + k] : B[(size_t)k * ldb + n];
        for (int n = N; n < Np; n++) row[n] = 0;
    }
    const int nblk = Np / 16;
#pragma omp parallel for num_threads(nt) schedule(dynamic, 1)
    for (int nb = 0; nb < nblk; nb++) {
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
