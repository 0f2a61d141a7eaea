/*
 * ref_shim.cpp — C entry points around the REAL reference kernels (TEST INFRASTRUCTURE ONLY).
 *
 * This file contains no kernel arithmetic of its own: it #includes the reference's
 * header-only library where it lies (-I/root/reference/include, never copied) and forwards
 * plain pointers to amx_kernel::Matmul / MatmulVector / GemAvB / repackB_1x2 /
 * PP::BiasGeluStore.  It is built only where the reference checkout and an AMX-capable
 * host exist, into oracle/_ref/libmmamx_ref.so, and is used by the CPU-side tests to pin the
 * portable restatement in fc_oracle.c bit-for-bit against the real thing.
 *
 * Driver logic restated here (not kernel code): the N-split over threads of
 * main.cpp:442-479 (MatmulMTOMP) — one Matmul object per thread, column ranges from
 * splitter() in units of 32.
 */
#include <cstdint>
#include <cstring>
#include <thread>
#include <vector>

#include "kernels_amx.hpp"

using ov::bfloat16;
namespace PP = amx_kernel::PP;

namespace {

template <typename T>
tensor2D<T> view(const void* p, int d0, int d1, int64_t stride_bytes) {
    return tensor2D<T>(d0, d1, reinterpret_cast<T*>(const_cast<void*>(p)), (int)stride_bytes);
}

/* a post-op that hands back the raw accumulator tile (fp32 or int32) */
template <typename TC>
struct RawStore {
    TC* C;
    int64_t ldc; /* elements */
    void operator()(tensor2D<TC>& buffC, int m, int n, int valid_m, int valid_n) {
        for (int i = 0; i < valid_m; i++)
            for (int j = 0; j < valid_n; j++) C[(int64_t)(m + i) * ldc + n + j] = buffC(i, j);
    }
};

template <typename MM, typename TA, typename TB, typename P>
void run_nsplit(int nthreads, bool transB, tensor2D<TA>& A, tensor2D<TB>& B, int N, P pp) {
    if (nthreads <= 1) {
        MM mm(true, transB);
        mm(A, B, 0, N, pp);
        return;
    }
    int work = rndup(N, 32) / 32;
    std::vector<std::thread> th;
    for (int t = 0; t < nthreads; t++) {
        th.emplace_back([&, t]() {
            int s, e;
            splitter(work, nthreads, t, s, e);
            int n0 = s * 32, n1 = e * 32;
            if (n1 > N) n1 = N;
            if (n1 <= n0) return;
            MM mm(true, transB);
            mm(A, B, n0, n1, pp);
        });
    }
    for (auto& t : th) t.join();
}

template <typename D, PP::Steps steps>
PP::BiasGeluStore<D, steps> make_pp(tensor2D<D>& C, float* bias, float deq, float q, float* q_per_oc) {
    PP::BiasGeluStore<D, steps> pp(C, bias);
    if (steps & PP::DEQUANT) pp.set_deq_scale(deq);
    if (steps & PP::QUANT) {
        if (q_per_oc) pp.set_q_scale(q_per_oc);
        else pp.set_q_scale(q);
    }
    return pp;
}

} // namespace

extern "C" {

int ref_init() { return initXTILE() ? 1 : 0; }

/* raw accumulators -------------------------------------------------------------------- */
void ref_gemm_bf16_acc(const void* A, int64_t lda_bytes, const void* B, int64_t ldb_bytes, int transB, float* C,
                       int64_t ldc, int M, int K, int N, int nthreads) {
    auto tA = view<bfloat16>(A, M, K, lda_bytes);
    auto tB = transB ? view<bfloat16>(B, N, K, ldb_bytes) : view<bfloat16>(B, K, N, ldb_bytes);
    RawStore<float> pp{C, ldc};
    run_nsplit<amx_kernel::Matmul<bfloat16, bfloat16>>(nthreads, transB, tA, tB, N, pp);
}

void ref_gemm_i8_acc(const void* A, int64_t lda_bytes, const void* B, int64_t ldb_bytes, int transB, int32_t* C,
                     int64_t ldc, int M, int K, int N, int nthreads) {
    auto tA = view<int8_t>(A, M, K, lda_bytes);
    auto tB = transB ? view<int8_t>(B, N, K, ldb_bytes) : view<int8_t>(B, K, N, ldb_bytes);
    RawStore<int32_t> pp{C, ldc};
    run_nsplit<amx_kernel::Matmul<int8_t, int8_t>>(nthreads, transB, tA, tB, N, pp);
}

/* full FC with the reference's own post-op.  mode selects (TA, D, steps):
 *   0 bf16 -> f32  NONE            1 bf16 -> bf16 NONE          2 bf16 -> bf16 BIAS_GELU
 *   3 bf16 -> f32  BIAS_GELU       4 bf16 -> bf16 BIAS
 *   10 s8 -> f32  NONE             11 s8 -> s8 DEQUANT|BIAS|QUANT
 *   12 s8 -> s8 DEQUANT_BIAS_GELU_QUANT   13 s8 -> bf16 DEQUANT   14 s8 -> f32 DEQUANT|BIAS
 * returns 0 on success, -1 for an unknown mode. */
int ref_fc(int mode, const void* A, int64_t lda_bytes, const void* B, int64_t ldb_bytes, int transB, void* C,
           int64_t ldc_bytes, int M, int K, int N, float* bias, float deq, float q, float* q_per_oc,
           int nthreads) {
#define BF16_CASE(id, D, S)                                                                              \
    case id: {                                                                                           \
        auto tA = view<bfloat16>(A, M, K, lda_bytes);                                                    \
        auto tB = transB ? view<bfloat16>(B, N, K, ldb_bytes) : view<bfloat16>(B, K, N, ldb_bytes);      \
        auto tC = view<D>(C, M, N, ldc_bytes);                                                           \
        auto pp = make_pp<D, (PP::Steps)(S)>(tC, bias, deq, q, q_per_oc);                                \
        run_nsplit<amx_kernel::Matmul<bfloat16, bfloat16>>(nthreads, transB, tA, tB, N, pp);             \
        return 0;                                                                                        \
    }
#define S8_CASE(id, D, S)                                                                                \
    case id: {                                                                                           \
        auto tA = view<int8_t>(A, M, K, lda_bytes);                                                      \
        auto tB = transB ? view<int8_t>(B, N, K, ldb_bytes) : view<int8_t>(B, K, N, ldb_bytes);          \
        auto tC = view<D>(C, M, N, ldc_bytes);                                                           \
        auto pp = make_pp<D, (PP::Steps)(S)>(tC, bias, deq, q, q_per_oc);                                \
        run_nsplit<amx_kernel::Matmul<int8_t, int8_t>>(nthreads, transB, tA, tB, N, pp);                 \
        return 0;                                                                                        \
    }
    switch (mode) {
        BF16_CASE(0, float, PP::NONE)
        BF16_CASE(1, bfloat16, PP::NONE)
        BF16_CASE(2, bfloat16, PP::BIAS_GELU)
        BF16_CASE(3, float, PP::BIAS_GELU)
        BF16_CASE(4, bfloat16, PP::BIAS)
        S8_CASE(10, float, PP::NONE)
        S8_CASE(11, int8_t, PP::DEQUANT | PP::BIAS | PP::QUANT)
        S8_CASE(12, int8_t, PP::DEQUANT_BIAS_GELU_QUANT)
        S8_CASE(13, bfloat16, PP::DEQUANT)
        S8_CASE(14, float, PP::DEQUANT | PP::BIAS)
    default: return -1;
    }
#undef BF16_CASE
#undef S8_CASE
}

/* Matmul<bf16,int8,float>: bf16 weights quantised per tensor inside the op, single thread
 * (the reference's software pipeline reads 1 KiB past the packed weights, so it is not
 * driven from several threads here).  Returns the dequant scale the op chose. */
float ref_fc_w8(const void* A, int64_t lda_bytes, const void* B, int64_t ldb_bytes, int transB, float* C,
                int64_t ldc_bytes, int M, int K, int N) {
    auto tA = view<bfloat16>(A, M, K, lda_bytes);
    auto tB = transB ? view<bfloat16>(B, N, K, ldb_bytes) : view<bfloat16>(B, K, N, ldb_bytes);
    auto tC = view<float>(C, M, N, ldc_bytes);
    PP::BiasGeluStore<float, PP::DEQUANT> pp(tC);
    amx_kernel::Matmul<bfloat16, int8_t, float> mm(true, transB);
    mm(tA, tB, 0, N, pp);
    return mm.dequant_scale_B;
}

/* repackB_1x2; out must hold ceil(N/32) * roundup(K,kStep)*32 elements */
void ref_repack(int elesz, const void* B, int64_t ldb_bytes, int K, int N, int transpose, void* out) {
    if (elesz == 2) {
        auto tB = transpose ? view<bfloat16>(B, N, K, ldb_bytes) : view<bfloat16>(B, K, N, ldb_bytes);
        auto Bo = amx_kernel::repackB_1x2(tB, transpose);
        for (int r = 0; r < Bo.dims[0]; r++)
            memcpy((char*)out + (size_t)r * Bo.dims[1] * 2, &Bo(r, 0), (size_t)Bo.dims[1] * 2);
    } else {
        auto tB = transpose ? view<int8_t>(B, N, K, ldb_bytes) : view<int8_t>(B, K, N, ldb_bytes);
        auto Bo = amx_kernel::repackB_1x2(tB, transpose);
        for (int r = 0; r < Bo.dims[0]; r++)
            memcpy((char*)out + (size_t)r * Bo.dims[1], &Bo(r, 0), (size_t)Bo.dims[1]);
    }
}

void ref_matvec_bf16(const void* A, int64_t lda_bytes, const void* b, float* c, int M, int K) {
    auto tA = view<bfloat16>(A, M, K, lda_bytes);
    amx_kernel::MatmulVector<bfloat16, bfloat16> mv;
    mv(tA, reinterpret_cast<const bfloat16*>(b), c);
}

void ref_matvec_i8(const void* A, int64_t lda_bytes, const void* b, int32_t* c, int M, int K) {
    auto tA = view<int8_t>(A, M, K, lda_bytes);
    amx_kernel::MatmulVector<int8_t, int8_t> mv;
    mv(tA, reinterpret_cast<const int8_t*>(b), c);
}

void ref_gemavb(const void* A, int64_t lda_bytes, void* b, float* c, int M, int K) {
    auto tA = view<bfloat16>(A, M, K, lda_bytes);
    amx_kernel::GemAvB g;
    g(tA, reinterpret_cast<bfloat16*>(b), c);
}

void ref_gelu(const float* x, float* y, int n) {
    for (int i = 0; i < n; i += 16) {
        float in[16] = {0}, out[16];
        int cnt = (n - i) < 16 ? (n - i) : 16;
        memcpy(in, x + i, cnt * sizeof(float));
        __m512 v = _mm512_loadu_ps(in);
        __m512 r = amx_kernel::functional::gelu_erf_minmax_approx(v);
        _mm512_storeu_ps(out, r);
        memcpy(y + i, out, cnt * sizeof(float));
    }
}

/* the hardware's own reciprocal approximation, used only to measure how far the oracle's
 * correctly rounded SiLU reciprocal is from what the reference's host would produce */
void ref_rcp14(const float* x, float* y, int n) {
    for (int i = 0; i < n; i += 16) {
        float in[16] = {1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1}, out[16];
        int cnt = (n - i) < 16 ? (n - i) : 16;
        memcpy(in, x + i, cnt * sizeof(float));
        _mm512_storeu_ps(out, _mm512_rcp14_ps(_mm512_loadu_ps(in)));
        memcpy(y + i, out, cnt * sizeof(float));
    }
}

/* compares fn with the vrcp14ps instruction on every one of the 2^32 bit patterns (NaN results compare
 * as NaN); returns the number of mismatches and the first mismatching input */
long long ref_rcp14_check_all(float (*fn)(float), unsigned* first_bad) {
    long long bad = 0;
    unsigned first = 0;
    int have_first = 0;
#pragma omp parallel for schedule(static) reduction(+ : bad)
    for (long long base = 0; base < (1ll << 32); base += 16) {
        unsigned in[16], out[16];
        for (int i = 0; i < 16; i++) in[i] = (unsigned)(base + i);
        _mm512_storeu_si512((void*)out, _mm512_castps_si512(_mm512_rcp14_ps(_mm512_castsi512_ps(_mm512_loadu_si512((const void*)in)))));
        for (int i = 0; i < 16; i++) {
            float xf;
            memcpy(&xf, &in[i], 4);
            const float g = fn(xf);
            unsigned gb;
            memcpy(&gb, &g, 4);
            const bool hw_nan = (out[i] & 0x7fffffffu) > 0x7f800000u, g_nan = (gb & 0x7fffffffu) > 0x7f800000u;
            if (hw_nan ? !g_nan : gb != out[i]) {
                bad++;
#pragma omp critical
                if (!have_first || in[i] < first) { first = in[i]; have_first = 1; }
            }
        }
    }
    if (first_bad) *first_bad = first;
    return bad;
}

/* The unsigned operand combinations of the int8 GEMM and mat-vec (tdpbusd / tdpbsud / tdpbuud,
 * include/kernels_amx.hpp:1057-1101 and :839-850).  Of the GEMM only <uint8_t, int8_t> can be instantiated: with
 * TB = uint8_t the reference's own repackB_1x2<uint8_t> does not compile (kpack_tile_B0B1 has no uint8_t overload,
 * :293, :393, :810), so the s8 x u8 and u8 x u8 GEMMs exist as branches of TILE_DP only.  The mat-vec takes its
 * vector as a plain pointer and instantiates in all three forms. */
void ref_gemm_u8s8_acc(const void* A, int64_t lda_bytes, const void* B, int64_t ldb_bytes, int transB, int32_t* C,
                       int64_t ldc, int M, int K, int N, int nthreads) {
    RawStore<int32_t> pp{C, ldc};
    auto tA = view<uint8_t>(A, M, K, lda_bytes);
    auto tB = transB ? view<int8_t>(B, N, K, ldb_bytes) : view<int8_t>(B, K, N, ldb_bytes);
    run_nsplit<amx_kernel::Matmul<uint8_t, int8_t>>(nthreads, transB, tA, tB, N, pp);
}

void ref_matvec_x8(int a_unsigned, int b_unsigned, const void* A, int64_t lda_bytes, const void* b, int32_t* c, int M, int K) {
    if (a_unsigned && b_unsigned) {
        auto tA = view<uint8_t>(A, M, K, lda_bytes);
        amx_kernel::MatmulVector<uint8_t, uint8_t> mv;
        mv(tA, reinterpret_cast<const uint8_t*>(b), c);
    } else if (a_unsigned) {
        auto tA = view<uint8_t>(A, M, K, lda_bytes);
        amx_kernel::MatmulVector<uint8_t, int8_t> mv;
        mv(tA, reinterpret_cast<const int8_t*>(b), c);
    } else {
        auto tA = view<int8_t>(A, M, K, lda_bytes);
        amx_kernel::MatmulVector<int8_t, uint8_t> mv;
        mv(tA, reinterpret_cast<const uint8_t*>(b), c);
    }
}

/* The element expression of repackB_1xL<int8_t, L> (weight_compression/fc16m.cpp:80-81: "*dst++ = src0[n] * scale"
 * with src0 an ov::bfloat16* and dst an int8_t*), evaluated by the reference's own bfloat16 class.  The function
 * around it cannot be compiled here (its file needs xbyak); this is the part of it that has arithmetic. */
void ref_bf16_scale_to_s8(const uint16_t* src, float scale, int8_t* dst, size_t n) {
    const bfloat16* s = reinterpret_cast<const bfloat16*>(src);
    for (size_t i = 0; i < n; i++) dst[i] = s[i] * scale;
}

} // extern "C"
