/*
 * fc_oracle.c — epilogues, repack, weight compression, mat-vec and MLP of the CPU oracle.
 * TEST INFRASTRUCTURE ONLY (see fc_oracle.h).
 *
 * Built with -ffp-contract=off: every multiply and add below rounds separately, exactly as
 * the reference's separate AVX-512 mul/add instructions do; fused operations are written
 * out as fmaf() where the reference uses an fmadd instruction.
 */
#include "fc_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* ------------------------------------------------------------------------------------ */
/* bf16: include/bf16.hpp:91-102 (round_to_nearest_even) for normal numbers, which is also
 * what vcvtne2ps2bf16 (include/kernels_amx.hpp:654) produces; the instruction additionally
 * treats fp32 denormals as zero and quiets NaNs, which the bit formula alone would not. */
uint16_t orc_f32_to_bf16(float x) {
    uint32_t u = f2u(x);
    if ((u & 0x7f800000u) == 0x7f800000u && (u & 0x007fffffu)) return (uint16_t)((u >> 16) | 0x0040u);
    if ((u & 0x7f800000u) == 0) return (uint16_t)((u >> 16) & 0x8000u);
    uint32_t bias = 0x00007fffu + ((u >> 16) & 1u);
    return (uint16_t)((u + bias) >> 16);
}
/* include/bf16.hpp:70-76 */
float orc_bf16_to_f32(uint16_t b) { return u2f((uint32_t)b << 16); }
void orc_f32_to_bf16_n(const float* s, uint16_t* d, size_t n) { for (size_t i = 0; i < n; i++) d[i] = orc_f32_to_bf16(s[i]); }
void orc_bf16_to_f32_n(const uint16_t* s, float* d, size_t n) { for (size_t i = 0; i < n; i++) d[i] = orc_bf16_to_f32(s[i]); }

/* ------------------------------------------------------------------------------------ */
/* include/kernels_amx.hpp:242-289 — oneDNN's gelu_erf minimax polynomial.
 * x*0.5*(1 + x*P(x^2)), Horner with fused multiply-adds, then three selects. */
float orc_gelu(float x) {
    static const uint32_t coef[15] = {
        0x1f1c83fdu, 0xa3198977u, 0x268a7927u, 0xa998c963u, 0x2c67ddb2u, 0xaf013b2cu, 0x315d4a4fu, 0xb3969b11u,
        0x35a776e9u, 0xb79b0914u, 0x3970b255u, 0xbb1b7399u, 0x3ca3621fu, 0xbe082bc7u, 0x3f4c4228u};
    const float x2 = x * x;
    const float x_pos = u2f(f2u(x) & 0x7fffffffu);
    const float x_half = x * 0.5f;
    float poly = u2f(coef[0]);
    for (int i = 1; i < 15; i++) poly = fmaf(poly, x2, u2f(coef[i]));
    poly = fmaf(poly, x, 1.0f);
    poly = poly * x_half;
    /* cmpnlt: "not (x < -5)" is true for NaN, so NaN stays NaN */
    if (x < u2f(0xc0a00000u)) x = 0.0f;
    /* cmpnle: "not (|x| <= 5)" */
    if (!(x_pos <= u2f(0x40a00000u))) poly = x;
    if (x_pos <= u2f(0x33800000u)) poly = x_half;
    return poly;
}
void orc_gelu_n(const float* s, float* d, size_t n) { for (size_t i = 0; i < n; i++) d[i] = orc_gelu(s[i]); }

/* vcvtps2dq under the default MXCSR (round to nearest even; out of range or NaN gives the
 * "integer indefinite" 0x80000000), then vpmovsdb signed saturation
 * (include/kernels_amx.hpp:658-661). */
static inline int8_t cvt_f32_to_s8_sat(float r) {
    int32_t d;
    if (!(r >= -2147483648.0f && r < 2147483648.0f)) d = INT32_MIN;
    else d = (int32_t)nearbyintf(r);
    if (d > 127) d = 127;
    if (d < -128) d = -128;
    return (int8_t)d;
}

/* include/kernels_amx.hpp:586-672 — BiasGeluStore::operator(): per element
 *   [cvt i32->f32] [x deq] [+ bias[n]] [gelu] [x q[n]]  then store as bf16 / int8 / fp32.
 * Extension (not in the reference): deq_per_oc[n] replaces the per-tensor deq_scale, same
 * position in the chain, still one rounded multiply. */
static inline void pp_store(float r, int n, const orc_pp* pp, void* crow) {
    if (pp->steps & ORC_PP_DEQUANT) r = r * (pp->deq_per_oc ? pp->deq_per_oc[n] : pp->deq_scale);
    if (pp->steps & ORC_PP_BIAS) r = r + pp->bias[n];
    if (pp->steps & ORC_PP_GELU) r = orc_gelu(r);
    if (pp->steps & ORC_PP_QUANT) r = r * (pp->q_per_oc ? pp->q_per_oc[n] : pp->q_scale);
    switch (pp->out_dtype) {
    case ORC_BF16: ((uint16_t*)crow)[n] = orc_f32_to_bf16(r); break;
    case ORC_I8: ((int8_t*)crow)[n] = cvt_f32_to_s8_sat(r); break;
    default: ((float*)crow)[n] = r; break;
    }
}

void orc_pp_f32(const float* acc, int64_t ldacc, int M, int N, const orc_pp* pp, void* C, int64_t ldc_bytes) {
#pragma omp parallel for schedule(static)
    for (int m = 0; m < M; m++) {
        void* crow = (char*)C + (size_t)m * ldc_bytes;
        for (int n = 0; n < N; n++) pp_store(acc[(size_t)m * ldacc + n], n, pp, crow);
    }
}

void orc_pp_i32(const int32_t* acc, int64_t ldacc, int M, int N, const orc_pp* pp, void* C, int64_t ldc_bytes) {
#pragma omp parallel for schedule(static)
    for (int m = 0; m < M; m++) {
        void* crow = (char*)C + (size_t)m * ldc_bytes;
        /* vcvtdq2ps: int32 -> fp32, round to nearest even (include/kernels_amx.hpp:631-634) */
        for (int n = 0; n < N; n++) pp_store((float)acc[(size_t)m * ldacc + n], n, pp, crow);
    }
}

/* ------------------------------------------------------------------------------------ */
/* include/kernels_amx.hpp:761-816 (repackB_1x2) with kpack_tile_B0B1 (:293-454) and the
 * 16x16 dword transposes (:114-238).  Closed form of where element (k, n) lands:
 *   g = 4/elesz (elements per 32-bit group), kStep = 64/elesz,
 *   panel row n/32, each panel K_pad*32 elements;
 *   offset = kb*(kStep*32) + ((n%32)/16)*(kStep*16) + (krel/g)*(16*g) + (n%16)*g + krel%g,
 *   with kb = k/kStep, krel = k%kStep for full blocks; in the K-tail block the rows are
 *   bottom-aligned (krel = k - (K - kStep)) under zero rows (:326-338, :415-425, :793-800). */
size_t orc_repack_amx_bytes(int elesz, int K, int N) {
    const int kStep = 64 / elesz;
    const size_t Kp = (size_t)(K + kStep - 1) / kStep * kStep;
    const size_t Npan = (size_t)(N + 31) / 32;
    return Npan * Kp * 32 * elesz;
}

void orc_repack_amx(int elesz, const void* B, int64_t ldb_bytes, int K, int N, int transpose, void* out) {
    const int g = 4 / elesz, kStep = 64 / elesz;
    const int Kp = (K + kStep - 1) / kStep * kStep;
    const int Kbody = K - (K % kStep);
    memset(out, 0, orc_repack_amx_bytes(elesz, K, N));
    for (int n = 0; n < N; n++) {
        for (int k = 0; k < K; k++) {
            int kb, krel;
            if (k < Kbody) { kb = k / kStep; krel = k % kStep; }
            else { kb = Kbody / kStep; krel = k - (K - kStep); }
            size_t off = (size_t)(n / 32) * ((size_t)Kp * 32) + (size_t)kb * (kStep * 32) +
                         (size_t)((n % 32) / 16) * (kStep * 16) + (size_t)(krel / g) * (16 * g) +
                         (size_t)(n % 16) * g + (krel % g);
            const char* src = transpose ? (const char*)B + (size_t)n * ldb_bytes + (size_t)k * elesz
                                        : (const char*)B + (size_t)k * ldb_bytes + (size_t)n * elesz;
            memcpy((char*)out + off * elesz, src, elesz);
        }
    }
}

/* This project's device layout (no counterpart in the reference): the unit an MFMA consumes
 * as its B operand — 64 lanes x 16 bytes — is contiguous, units are ordered panel-major
 * then K, exactly the idea of include/kernels_amx.hpp:456-463 applied to gfx950. */
size_t orc_repack_mfma_bytes(int elesz, int K, int N) {
    const int kalign = 128 / elesz;
    const size_t Kp = (size_t)(K + kalign - 1) / kalign * kalign;
    const size_t Npan = (size_t)(N + 31) / 32;
    return Npan * Kp * 32 * elesz;
}

void orc_repack_mfma(int elesz, const void* B, int64_t ldb_bytes, int K, int N, int transpose, void* out) {
    const int KS = 32 / elesz;   /* k per 1 KiB fragment: bf16 16, int8 32 */
    const int half = KS / 2;     /* k per lane */
    const int kalign = 128 / elesz;
    const int Kp = (K + kalign - 1) / kalign * kalign;
    memset(out, 0, orc_repack_mfma_bytes(elesz, K, N));
    for (int n = 0; n < N; n++) {
        for (int k = 0; k < K; k++) {
            const int lane = (n % 32) + 32 * ((k % KS) / half);
            size_t off_bytes = ((size_t)(n / 32) * (Kp / KS) + (size_t)(k / KS)) * 1024 + (size_t)lane * 16 +
                               (size_t)(k % half) * elesz;
            const char* src = transpose ? (const char*)B + (size_t)n * ldb_bytes + (size_t)k * elesz
                                        : (const char*)B + (size_t)k * ldb_bytes + (size_t)n * elesz;
            memcpy((char*)out + off_bytes, src, elesz);
        }
    }
}

/* ------------------------------------------------------------------------------------ */
/* include/kernels_amx.hpp:1363-1377 with get_min_max (:465-488) and bf16_to_i8_tensor
 * (:508-523): scale = 127/max|w| over the whole matrix, q = sat8(rne(w*scale)). */
float orc_quantize_weights(const uint16_t* W, int64_t ldw, int rows, int cols, int8_t* Wq, int64_t ldq,
                           float* quant_scale) {
    float mx = -__FLT_MAX__, mn = __FLT_MAX__;
    for (int r = 0; r < rows; r++)
        for (int c = 0; c < cols; c++) {
            float v = orc_bf16_to_f32(W[(size_t)r * ldw + c]);
            if (v > mx) mx = v;
            if (v < mn) mn = v;
        }
    float amax = fabsf(mx) > fabsf(mn) ? fabsf(mx) : fabsf(mn);
    const float q = 127 / amax;
    const float dq = amax / 127;
    for (int r = 0; r < rows; r++)
        for (int c = 0; c < cols; c++)
            Wq[(size_t)r * ldq + c] = cvt_f32_to_s8_sat(orc_bf16_to_f32(W[(size_t)r * ldw + c]) * q);
    if (quant_scale) *quant_scale = q;
    return dq;
}

/* ------------------------------------------------------------------------------------ */
/* The quantising half of repackB_1xL<int8_t, L> (weight_compression/fc16m.cpp:61-99): every element goes through
 *     *dst++ = src0[n] * scale;                                  (:80-81)
 * with src0 an ov::bfloat16* and dst an int8_t*.  ov::bfloat16::operator*(float) (include/bf16.hpp:181-183) returns
 * a bfloat16 built from the fp32 product, i.e. rounded to nearest even (include/bf16.hpp:14, :95-107), and the
 * assignment to int8_t converts that bfloat16 through operator float() (:70-76) with the language's float -> integer
 * conversion: truncation toward zero.  So q = trunc(bf16_rne(float(w) * scale)).  The language leaves a value
 * outside [-128, 127] (and NaN) undefined; here it saturates (NaN -> 0), and fc16m's own use (fill_rnd weights
 * times quantize_i8_scale = 2, :51, :123) never gets there. */
int8_t orc_bf16_scale_trunc_s8(uint16_t w, float scale) {
    const float prod = orc_bf16_to_f32(w) * scale;
    const float r = orc_bf16_to_f32(orc_f32_to_bf16(prod));
    if (r != r) return 0;
    if (r >= 127.0f) return 127;
    if (r <= -128.0f) return -128;
    return (int8_t)(int)r;  /* C conversion: toward zero */
}

void orc_quantize_scale_trunc(const uint16_t* W, int64_t ldw, int rows, int cols, float scale, int8_t* Wq, int64_t ldq) {
    for (int r = 0; r < rows; r++)
        for (int c = 0; c < cols; c++) Wq[(size_t)r * ldq + c] = orc_bf16_scale_trunc_s8(W[(size_t)r * ldw + c], scale);
}

/* repackB_1xL<int8_t, L> whole (weight_compression/fc16m.cpp:61-99): B [K, N] bf16 (K % 32 == 0, N % (16 L) == 0)
 * -> K*N int8 in the function's own order: column groups of 16 L in computation order, K in blocks of 32, L tiles
 * per block; a tile is 16 pairs of k, each pair 16 columns x (k, k + 1) interleaved (:76-86). */
void orc_repack_1xL_s8(const uint16_t* B, int64_t ldb, int K, int N, int L, float scale, int8_t* out) {
    int8_t* dst = out;
    for (int n0 = 0; n0 < N; n0 += L * 16)
        for (int k0 = 0; k0 < K; k0 += 32)
            for (int l = 0; l < L; l++)
                for (int k = 0; k < 32; k += 2)
                    for (int n = 0; n < 16; n++) {
                        *dst++ = orc_bf16_scale_trunc_s8(B[(size_t)(k0 + k) * ldb + n0 + l * 16 + n], scale);
                        *dst++ = orc_bf16_scale_trunc_s8(B[(size_t)(k0 + k + 1) * ldb + n0 + l * 16 + n], scale);
                    }
}

/* ------------------------------------------------------------------------------------ */
/* The unsigned operand forms of the int8 GEMM and mat-vec (tdpbusd / tdpbsud / tdpbuud,
 * include/kernels_amx.hpp:1057-1101, :839-850): exact integer products summed in int32 modulo 2^32 (the AMX
 * accumulators wrap).  a_unsigned / b_unsigned say how the bytes of A / B are read. */
void orc_gemm_x8(int a_unsigned, int b_unsigned, const void* A, int64_t lda, const void* B, int64_t ldb, int transB,
                 int32_t* C, int64_t ldc, int M, int K, int N) {
    const uint8_t* a8 = (const uint8_t*)A;
    const uint8_t* b8 = (const uint8_t*)B;
#pragma omp parallel for schedule(static)
    for (int m = 0; m < M; m++)
        for (int n = 0; n < N; n++) {
            uint32_t acc = 0;
            for (int k = 0; k < K; k++) {
                const uint8_t ab = a8[(size_t)m * lda + k];
                const uint8_t bb = transB ? b8[(size_t)n * ldb + k] : b8[(size_t)k * ldb + n];
                const int av = a_unsigned ? (int)ab : (int)(int8_t)ab;
                const int bv = b_unsigned ? (int)bb : (int)(int8_t)bb;
                acc += (uint32_t)(av * bv);
            }
            C[(size_t)m * ldc + n] = (int32_t)acc;
        }
}

void orc_matvec_x8(int a_unsigned, int b_unsigned, const void* A, int64_t lda, const void* b, int32_t* c, int M, int K) {
    const uint8_t* a8 = (const uint8_t*)A;
    const uint8_t* b8 = (const uint8_t*)b;
    for (int m = 0; m < M; m++) {
        uint32_t acc = 0;
        for (int k = 0; k < K; k++) {
            const int av = a_unsigned ? (int)a8[(size_t)m * lda + k] : (int)(int8_t)a8[(size_t)m * lda + k];
            const int bv = b_unsigned ? (int)b8[k] : (int)(int8_t)b8[k];
            acc += (uint32_t)(av * bv);
        }
        c[m] = (int32_t)acc;
    }
}

/* int4 weight compression.  The reference has no algorithm to restate here: weight_compression/wcompress.hpp:90-134
 * and README.md:216-244 only time a stand-in that copies bytes ("we haven't found efficient instructions to
 * implement a fully-functional dequant() for INT4").  This is the definition the device code is held to:
 * per output channel n, a = max_k |w[k][n]|, q = clamp(rne(w * (7 / a)), -7, 7) in fp32 (0 for a = 0),
 * deq[n] = a / 7.  W is [K][N] (transpose = 0) or [N][K] (transpose = 1), ldw in elements; q is [K][N]. */
void orc_quantize_int4(const uint16_t* W, int64_t ldw, int K, int N, int transpose, int8_t* q, float* deq) {
    for (int n = 0; n < N; n++) {
        float a = 0.0f;
        for (int k = 0; k < K; k++) {
            const float v = fabsf(orc_bf16_to_f32(transpose ? W[(size_t)n * ldw + k] : W[(size_t)k * ldw + n]));
            if (v > a) a = v;
        }
        const float qs = a > 0.0f ? 7.0f / a : 0.0f;
        deq[n] = a / 7.0f;
        for (int k = 0; k < K; k++) {
            float r = rintf(orc_bf16_to_f32(transpose ? W[(size_t)n * ldw + k] : W[(size_t)k * ldw + n]) * qs);
            if (r != r) r = 0.0f; /* NaN weight, or an infinite one in a column whose maximum (NaN aside) is infinite: 0 */
            r = r < -7.0f ? -7.0f : (r > 7.0f ? 7.0f : r);
            q[(size_t)k * N + n] = (int8_t)r;
        }
    }
}

/* This project's packed int4 layout (no reference counterpart): 32-column panels of 1 KiB fragments, a fragment
 * = 32 columns x 64 of k; lane g*32 + c owns 16 bytes, its dword i holds k = 64 f + 32 g + 8 i + e in bits
 * [4e, 4e+4) as two's complement; K is padded with zeros to a multiple of 256. */
size_t orc_pack_int4_bytes(int K, int N) { return (size_t)((N + 31) / 32) * ((size_t)(K + 255) / 256 * 4) * 1024; }

void orc_pack_int4(const int8_t* q, int K, int N, uint8_t* out) {
    const size_t nfrag = (size_t)(K + 255) / 256 * 4;
    memset(out, 0, orc_pack_int4_bytes(K, N));
    for (int n = 0; n < N; n++)
        for (int k = 0; k < K; k++) {
            const int f = k / 64, g = (k % 64) / 32, i = (k % 32) / 8, e = k % 8;
            const size_t byte = ((size_t)(n / 32) * nfrag + f) * 1024 + (size_t)(g * 32 + n % 32) * 16 + i * 4 + e / 2;
            const uint8_t nib = (uint8_t)q[(size_t)k * N + n] & 0xf;
            out[byte] |= (e & 1) ? (uint8_t)(nib << 4) : nib;
        }
}

/* weight_compression/fc16m.cpp:451-502 (matmul16m_Wint8B) and include/kernels_amx.hpp:1381-1441:
 * int8 weights are converted to bf16 exactly (|w| <= 128 needs 8 significant bits;
 * include/kernels_amx.hpp:490-506, fc16m.cpp:309-333) and fed to the same tdpbf16ps chain, the
 * scale is applied to the fp32 result afterwards (fc16m.cpp:496-500 per tensor; here per
 * output channel, one rounded multiply), then rounded to bf16. */
void orc_gemv_w8(const uint16_t* x, int64_t ldx, const int8_t* Wq, int64_t ldw, int transW, const float* scale,
                 uint16_t* y, int64_t ldy, float* acc_out, int M, int K, int N, int nthreads) {
    const int rows = transW ? N : K, cols = transW ? K : N;
    uint16_t* Wb = (uint16_t*)malloc((size_t)rows * cols * sizeof(uint16_t));
    float* acc = (float*)malloc((size_t)M * N * sizeof(float));
    if (!Wb || !acc) abort();
#pragma omp parallel for schedule(static)
    for (int r = 0; r < rows; r++)
        for (int c = 0; c < cols; c++) Wb[(size_t)r * cols + c] = orc_f32_to_bf16((float)Wq[(size_t)r * ldw + c]);
    orc_gemm_bf16(x, ldx, Wb, cols, transW, acc, N, M, K, N, nthreads);
    for (int m = 0; m < M; m++)
        for (int n = 0; n < N; n++) y[(size_t)m * ldy + n] = orc_f32_to_bf16(acc[(size_t)m * N + n] * scale[n]);
    if (acc_out) memcpy(acc_out, acc, (size_t)M * N * sizeof(float));
    free(Wb);
    free(acc);
}

/* ------------------------------------------------------------------------------------ */
/* include/kernels_amx.hpp:854-1042 — MatmulVector: the same tdpbf16ps chain with a
 * one-column B.  Full 16-row groups read the K tail left-aligned at Kbody (B zero padded
 * below, :874-880); the last group of rows reads it right-aligned at K-32 (B zero padded
 * above, :866-872) — the tail products then sit at different slots of the tile, which
 * changes which of the two partial sums they join when K is odd.  The reference's dispatch
 * is wrong for more than four K tiles (:939-953); this follows the intended product. */
void orc_matvec_bf16(const uint16_t* A, int64_t lda, const uint16_t* b, float* c, int M, int K) {
    const int Ktail = K & 31, Kbody = K - Ktail;
    int Mtail = M & 15, Mbody = M - Mtail;
    if (Ktail && Mtail == 0) { Mtail = 16; Mbody -= 16; }
    for (int m = 0; m < M; m++) {
        const uint16_t* a = A + (size_t)m * lda;
        float acc = 0.0f;
        for (int kb = 0; kb < Kbody; kb += 32) {
            float p0 = 0.0f, p1 = 0.0f;
            for (int p = 0; p < 32; p += 2) {
                p0 += orc_bf16_to_f32(a[kb + p]) * orc_bf16_to_f32(b[kb + p]);
                p1 += orc_bf16_to_f32(a[kb + p + 1]) * orc_bf16_to_f32(b[kb + p + 1]);
            }
            acc += (p0 + p1);
        }
        if (Ktail) {
            const int t0 = (m < Mbody) ? Kbody : K - 32;
            float p0 = 0.0f, p1 = 0.0f;
            for (int k = Kbody; k < K; k++) {
                float pr = orc_bf16_to_f32(a[k]) * orc_bf16_to_f32(b[k]);
                if ((k - t0) & 1) p1 += pr; else p0 += pr;
            }
            acc += (p0 + p1);
        }
        c[m] = acc;
    }
}

/* include/kernels_amx.hpp:1529-1618 — GemAvB: vdpbf16ps on k pairs, pair i of each 32-block
 * goes to accumulator i&1 (:1595-1610), the two are added at the end (:1612).  vdpbf16ps
 * adds the odd element's product first, then the even one, each with one rounding. */
void orc_gemavb_bf16(const uint16_t* A, int64_t lda, const uint16_t* b, float* c, int M, int K) {
    for (int m = 0; m < M; m++) {
        const uint16_t* a = A + (size_t)m * lda;
        float acc[2] = {0.0f, 0.0f};
        for (int k = 0; k < K; k += 2) {
            const int which = (k >> 1) & 1;
            float odd = (k + 1 < K) ? orc_bf16_to_f32(a[k + 1]) * orc_bf16_to_f32(b[k + 1]) : 0.0f;
            float even = orc_bf16_to_f32(a[k]) * orc_bf16_to_f32(b[k]);
            float t = acc[which] + odd;
            acc[which] = t + even;
        }
        c[m] = acc[0] + acc[1];
    }
}

void orc_matvec_i8(const int8_t* A, int64_t lda, const int8_t* b, int32_t* c, int M, int K) {
    for (int m = 0; m < M; m++) {
        int32_t acc = 0;
        for (int k = 0; k < K; k++) acc += (int32_t)A[(size_t)m * lda + k] * (int32_t)b[k];
        c[m] = acc;
    }
}

/* ------------------------------------------------------------------------------------ */
/* tests/amx-mlp.cpp:383-448 — exp_ps_avx512: clamp, n = floor(x*log2e + 0.5),
 * r = x - n*ln2 (fused), degree-5 polynomial (fused), times 2^(n-1), times 2. */
float orc_exp_poly(float x) {
    const float ln_flt_min = u2f(0xc2aeac50u), ln_flt_max = u2f(0x42b17218u);
    const float log2ef = u2f(0x3fb8aa3bu), ln2f = u2f(0x3f317218u);
    const float p1 = u2f(0x3f7ffffbu), p2 = u2f(0x3efffee3u), p3 = u2f(0x3e2aad40u), p4 = u2f(0x3d2b9d0du),
                p5 = u2f(0x3c07cfceu);
    const int zero = x < ln_flt_min;
    float s = x;
    s = (s < ln_flt_max) ? s : ln_flt_max; /* vminps(src, max): returns max unless src < max */
    s = (s > ln_flt_min) ? s : ln_flt_min;
    float aux1 = s;
    s = s * log2ef;
    s = s + 0.5f;
    s = floorf(s);
    aux1 = fmaf(-s, ln2f, aux1);
    s = s - 1.0f;
    int32_t e = (int32_t)nearbyintf(s);
    e = (int32_t)((uint32_t)(e + 127) << 23);
    float aux2 = zero ? 0.0f : u2f((uint32_t)e);
    s = p5;
    s = fmaf(s, aux1, p4);
    s = fmaf(s, aux1, p3);
    s = fmaf(s, aux1, p2);
    s = fmaf(s, aux1, p1);
    s = fmaf(s, aux1, 1.0f);
    s = s * aux2;
    s = s * 2.0f;
    return s;
}

/* vrcp14ps (used by tests/amx-mlp.cpp:453), bit for bit.  The instruction is deterministic and the same
 * on every AVX-512 CPU, but its table is not published; the model below was derived from the
 * instruction's output on all 2^23 mantissas (oracle/derive_rcp14.py) and is checked against the
 * instruction on all 2^32 inputs (tests/test_oracle_ref.py) wherever AVX-512 is present:
 *   - a power of two gives the exact reciprocal;
 *   - otherwise the result depends on the top 16 mantissa bits only: the top 6 select a segment
 *     (a 18-bit intercept a and a 10-bit slope b), the next 10 are the offset d within it, and
 *     the 17-bit significand is (a*256 - b*d) >> 9, the 7 low mantissa bits are zero;
 *   - denormal inputs are normalised first (not flushed); a result beyond the largest float is inf;
 *     results below the normal range are the significand shifted right (nothing is lost: at most
 *     two bits, seven are zero); zero -> inf, inf -> 0, NaN -> quiet NaN; the sign passes through.
 * Each table word is a << 10 | b. */
static const uint32_t rcp14_seg[64] = {
    0x0fffe7f1u, 0x0fc0dbd1u, 0x0f83cbb5u, 0x0f488399u, 0x0f0eef7du, 0x0ed71f65u, 0x0ea0cf4bu, 0x0e6c1b35u,
    0x0e38cb1du, 0x0e06f309u, 0x0dd662f3u, 0x0da72adfu, 0x0d7932cdu, 0x0d4c6ebbu, 0x0d20c6a9u, 0x0cf63297u,
    0x0cccbe87u, 0x0ca44677u, 0x0c7cda69u, 0x0c564e59u, 0x0c30b64bu, 0x0c0bfe3du, 0x0be82a31u, 0x0bc51623u,
    0x0ba2da17u, 0x0b81620bu, 0x0b60b601u, 0x0b40a9f5u, 0x0b215debu, 0x0b02b5dfu, 0x0ae4b9d5u, 0x0ac75dcbu,
    0x0aaaa9c3u, 0x0a8e7db9u, 0x0a72f1b1u, 0x0a57e1a7u, 0x0a3d699fu, 0x0a237597u, 0x0a0a018fu, 0x09f10d87u,
    0x09d8a181u, 0x09c09579u, 0x09a90571u, 0x0991ed6bu, 0x097b4565u, 0x0964f55du, 0x094f1957u, 0x0939a151u,
    0x09248d4bu, 0x090fd545u, 0x08fb793fu, 0x08e7893bu, 0x08d3d935u, 0x08c0852fu, 0x08ad912bu, 0x089add25u,
    0x08888921u, 0x08767d1du, 0x0864b517u, 0x08534d13u, 0x0842250fu, 0x08313d0bu, 0x08209507u, 0x08102d03u};

float orc_rcp14(float x) {
    const uint32_t u = f2u(x);
    const uint32_t sign = u & 0x80000000u;
    int32_t ex = (int32_t)((u >> 23) & 0xffu);
    uint32_t m = u & 0x7fffffu;
    if (ex == 0xff) return m ? u2f(u | 0x00400000u) : u2f(sign);        /* NaN (quieted), inf -> 0 */
    if (ex == 0) {
        if (m == 0) return u2f(sign | 0x7f800000u);                     /* zero -> inf */
        const int k = 31 - __builtin_clz(m);                            /* denormal: normalise, exponent field k - 22 */
        m = (m << (23 - k)) & 0x7fffffu;
        ex = k - 22;
    }
    uint32_t sig;                                                       /* result = sig * 2^(rex - 127 - 16) */
    int32_t rex;
    if (m == 0) {
        sig = 0x10000u;
        rex = 254 - ex;
    } else {
        const uint32_t w = rcp14_seg[m >> 17], d = (m >> 7) & 1023u;
        sig = (((w >> 10) << 8) - (w & 1023u) * d) >> 9;               /* 17 bits, leading one */
        rex = 253 - ex;
    }
    if (rex >= 255) return u2f(sign | 0x7f800000u);                     /* overflow -> inf */
    uint32_t mant24 = sig << 7;                                         /* 24-bit significand */
    if (rex <= 0) {                                                     /* denormal result */
        mant24 >>= (1 - rex);
        return u2f(sign | mant24);
    }
    return u2f(sign | ((uint32_t)rex << 23) | (mant24 & 0x7fffffu));
}

void orc_rcp14_n(const float* src, float* dst, size_t n) {
    for (size_t i = 0; i < n; i++) dst[i] = orc_rcp14(src[i]);
}

/* tests/amx-mlp.cpp:450-456 — silu(x) = x * rcp14(1 + exp(-x)): negate (a subtraction from zero),
 * the exp polynomial, one addition, vrcp14ps, one multiplication. */
float orc_silu(float x) {
    float e = orc_exp_poly(0.0f - x);
    float sig = orc_rcp14(1.0f + e);
    return x * sig;
}

void orc_silu_n(const float* src, float* dst, size_t n) {
    for (size_t i = 0; i < n; i++) dst[i] = orc_silu(src[i]);
}
void orc_exp_poly_n(const float* src, float* dst, size_t n) {
    for (size_t i = 0; i < n; i++) dst[i] = orc_exp_poly(src[i]);
}

/* tests/amx-mlp.cpp:720-734 — runGateUp epilogue: bf16( silu(gate) * up ) */
void orc_silu_mul_bf16(const float* gate, const float* up, uint16_t* h, size_t n) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; i++) h[i] = orc_f32_to_bf16(orc_silu(gate[i]) * up[i]);
}

/* tests/amx-mlp.cpp:648-704 with the partition at :546-593 — down_proj.  With split-K the K
 * blocks of 256 are cut into a first half of ceil(nblk/2) blocks and the rest; each half is
 * accumulated on its own (first block starts from zero, later blocks accumulate into the
 * fp32 C, :199-334), the halves are added (:676-677) and rounded to bf16 (:678). */
void orc_mlp_down(const uint16_t* h, const uint16_t* w_down, uint16_t* y, int M, int Kout, int N, int split_k,
                  int nthreads) {
    float* p0 = (float*)malloc((size_t)M * Kout * sizeof(float));
    float* p1 = NULL;
    if (!p0) abort();
    int n_first = N;
    if (split_k && (N % 256) == 0 && N >= 512) {
        const int nblk = N / 256;
        n_first = ((nblk + 1) / 2) * 256;
    }
    orc_gemm_bf16(h, N, w_down, N, 1, p0, Kout, M, n_first, Kout, nthreads);
    if (n_first < N) {
        p1 = (float*)malloc((size_t)M * Kout * sizeof(float));
        if (!p1) abort();
        orc_gemm_bf16(h + n_first, N, w_down + n_first, N, 1, p1, Kout, M, N - n_first, Kout, nthreads);
    }
    for (size_t i = 0; i < (size_t)M * Kout; i++) y[i] = orc_f32_to_bf16(p1 ? (p0[i] + p1[i]) : p0[i]);
    free(p0);
    free(p1);
}

/* tests/amx-mlp.cpp:740-784 (MLP::setup / run) and :788-841 (mlp_ref):
 *   h = bf16(silu(x·Wg^T) * (x·Wu^T)),  y = bf16(h·Wd^T) */
void orc_mlp(const uint16_t* x, const uint16_t* w_gate, const uint16_t* w_up, const uint16_t* w_down,
             uint16_t* h_out, uint16_t* y, int M, int K, int N, int split_k, int nthreads) {
    float* g = (float*)malloc((size_t)M * N * sizeof(float));
    float* u = (float*)malloc((size_t)M * N * sizeof(float));
    uint16_t* h = h_out ? h_out : (uint16_t*)malloc((size_t)M * N * sizeof(uint16_t));
    if (!g || !u || !h) abort();
    orc_gemm_bf16(x, K, w_gate, K, 1, g, N, M, K, N, nthreads);
    orc_gemm_bf16(x, K, w_up, K, 1, u, N, M, K, N, nthreads);
    orc_silu_mul_bf16(g, u, h, (size_t)M * N);
    orc_mlp_down(h, w_down, y, M, K, N, split_k, nthreads);
    free(g);
    free(u);
    if (!h_out) free(h);
}

/* include/misc.hpp:521-535 */
void orc_splitter(int n, int team, int tid, int* n_start, int* n_end) {
    if (team <= 1 || n == 0) { *n_start = 0; *n_end = n; return; }
    int n1 = (n + team - 1) / team;
    int n2 = n1 - 1;
    int T1 = n - n2 * team;
    int len = tid < T1 ? n1 : n2;
    *n_start = tid <= T1 ? tid * n1 : T1 * n1 + (tid - T1) * n2;
    *n_end = *n_start + len;
}
