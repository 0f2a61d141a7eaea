// Shared device/host helpers of the gfx950 FC-GEMM kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "../../include/mm_amx_amd.h"

namespace mmx {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;
typedef __attribute__((__vector_size__(4 * sizeof(int)))) int i32x4;
typedef __attribute__((__vector_size__(16 * sizeof(int)))) int i32x16;
// 16 raw bytes as a first-class vector value (unlike HIP's uint4 struct it stays in registers when
// held in small arrays)
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// error plumbing (host)
int set_error(int code, const char* fmt, ...);
int check_hip(hipError_t e, const char* what);
void note_kernel(const char* name);
int num_cus();
// Raises a kernel's dynamic LDS limit to `bytes` on the current device, once per device; `done_on_device`
// (one per kernel, a bit per device) records where that has happened.  Safe to call from any thread.
int ensure_dynamic_lds(const void* kernel, int bytes, std::atomic<uint64_t>& done_on_device);

struct Epilogue {
    uint32_t steps;
    int out_dtype;
    char* C;
    int64_t ldc;  // bytes
    const float* bias;
    float deq;
    const float* deq_oc;
    float q;
    const float* q_oc;
    int c_vec_ok;  // C and ldc are 16-byte aligned
};

// A caller's request for a split of K over several workgroups per tile, and the memory for its partial sums.
struct SplitRequest {
    int k_splits;     // 0: choose; 1: none; 2 and up: exactly this many slices
    char* ws;         // workspace (NULL: no split possible)
    size_t ws_bytes;
};

// ---- element-wise epilogue arithmetic -----------------------------------------------------
// All device code is compiled with -ffp-contract=off: a*b+c below never fuses unless written
// as fmaf(), which keeps the rounding sequence of the reference's AVX-512 post-op
// (include/kernels_amx.hpp:628-664).

__device__ __forceinline__ float u2f(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t f2u(float f) { return __builtin_bit_cast(uint32_t, f); }

// include/kernels_amx.hpp:242-289 — the gelu_erf minimax polynomial, same coefficient bits,
// same Horner chain of fused multiply-adds, same three selects.
__device__ __forceinline__ float gelu_erf_minimax(float x) {
    const float x2 = x * x;
    const float x_pos = u2f(f2u(x) & 0x7fffffffu);
    const float x_half = x * 0.5f;
    float p = u2f(0x1f1c83fdu);
    p = __builtin_fmaf(p, x2, u2f(0xa3198977u));
    p = __builtin_fmaf(p, x2, u2f(0x268a7927u));
    p = __builtin_fmaf(p, x2, u2f(0xa998c963u));
    p = __builtin_fmaf(p, x2, u2f(0x2c67ddb2u));
    p = __builtin_fmaf(p, x2, u2f(0xaf013b2cu));
    p = __builtin_fmaf(p, x2, u2f(0x315d4a4fu));
    p = __builtin_fmaf(p, x2, u2f(0xb3969b11u));
    p = __builtin_fmaf(p, x2, u2f(0x35a776e9u));
    p = __builtin_fmaf(p, x2, u2f(0xb79b0914u));
    p = __builtin_fmaf(p, x2, u2f(0x3970b255u));
    p = __builtin_fmaf(p, x2, u2f(0xbb1b7399u));
    p = __builtin_fmaf(p, x2, u2f(0x3ca3621fu));
    p = __builtin_fmaf(p, x2, u2f(0xbe082bc7u));
    p = __builtin_fmaf(p, x2, u2f(0x3f4c4228u));
    p = __builtin_fmaf(p, x, 1.0f);
    p = p * x_half;
    if (x < -5.0f) x = 0.0f;             // zone 1 (NaN keeps x)
    if (!(x_pos <= 5.0f)) p = x;         // zones 1 and 5 (and NaN)
    if (x_pos <= u2f(0x33800000u)) p = x_half;  // zone 3
    return p;
}

// The coefficients once more, for the 16-wide form below: read through a pointer they are fetched by scalar loads
// and live in scalar registers, which makes each Horner step a plain v_fma_f32; written as literals they become
// 64-bit v_fmaak_f32 instructions, which a lone wavefront issues 17 % slower (measured: 1495 against 1261 cycles
// per 16 values).  (The caller passes each word through an empty asm statement, or the compiler folds the known
// values back into literals.)
__constant__ static const uint32_t kGeluCoef[15] = {0x1f1c83fdu, 0xa3198977u, 0x268a7927u, 0xa998c963u, 0x2c67ddb2u,
                                                    0xaf013b2cu, 0x315d4a4fu, 0xb3969b11u, 0x35a776e9u, 0xb79b0914u,
                                                    0x3970b255u, 0xbb1b7399u, 0x3ca3621fu, 0xbe082bc7u, 0x3f4c4228u};

// The same function on the 16 accumulators a lane holds of one 32x32 block.  A wavefront that is alone on its SIMD
// issues one vector instruction every 4 to 5 cycles whatever their dependences, so the 16 Horner chains simply
// advance in lockstep, one coefficient at a time (cf: the 15 coefficients, in scalar registers).  The three
// selects only matter outside 2^-24 < |x| <= 5; they are skipped when no element of any lane of the wavefront is
// out there (v_max/v_min drop a NaN operand: a NaN then comes out of the polynomial as NaN, as it would out of
// the select).  Same result bit for bit.  (Inside the GEMM's epilogue the test and branch cost less than applying
// the selects to every element: 26.9k against 28.7k cycles per 256x192 tile.)
__device__ __forceinline__ void gelu_erf_minimax_x16(float (&r)[16], const float (&cf)[15]) {
    float x2[16], p[16];
#pragma unroll
    for (int v = 0; v < 16; v++) x2[v] = r[v] * r[v];
#pragma unroll
    for (int v = 0; v < 16; v++) p[v] = __builtin_fmaf(cf[0], x2[v], cf[1]);
#pragma unroll
    for (int c = 2; c < 15; c++) {
#pragma unroll
        for (int v = 0; v < 16; v++) p[v] = __builtin_fmaf(p[v], x2[v], cf[c]);
    }
#pragma unroll
    for (int v = 0; v < 16; v++) p[v] = __builtin_fmaf(p[v], r[v], 1.0f);
#pragma unroll
    for (int v = 0; v < 16; v++) p[v] = p[v] * (r[v] * 0.5f);
    float amax = __builtin_fabsf(r[0]), amin = amax;
#pragma unroll
    for (int v = 1; v < 16; v++) {
        amax = __builtin_fmaxf(amax, __builtin_fabsf(r[v]));
        amin = __builtin_fminf(amin, __builtin_fabsf(r[v]));
    }
    const bool needs_select = !(amax <= 5.0f) || !(amin > u2f(0x33800000u));
    // (unlikely: the selects are laid out away from the straight path, which then has no taken branch - the epilogue's
    // code runs once per tile, out of a cold instruction cache, and every taken branch restarts the fetch)
    if (__builtin_expect(__builtin_amdgcn_ballot_w64(needs_select) != 0, 0)) {
#pragma unroll
        for (int v = 0; v < 16; v++) {
            float x = r[v];
            // opaque to the optimiser, so that the selects stay inside this rarely taken branch: as
            // straight-line code they would cost every block 9 more instructions per element
            asm volatile("" : "+v"(x));
            const float x_pos = __builtin_fabsf(x);
            if (x < -5.0f) x = 0.0f;
            if (!(x_pos <= 5.0f)) p[v] = x;
            if (x_pos <= u2f(0x33800000u)) p[v] = r[v] * 0.5f;
        }
    }
#pragma unroll
    for (int v = 0; v < 16; v++) r[v] = p[v];
}

// tests/amx-mlp.cpp:383-448 — exp_ps_avx512, operation for operation.
__device__ __forceinline__ float exp_poly(float x) {
    const float ln_flt_min = u2f(0xc2aeac50u), ln_flt_max = u2f(0x42b17218u);
    const bool zero = x < ln_flt_min;
    float s = (x < ln_flt_max) ? x : ln_flt_max;
    s = (s > ln_flt_min) ? s : ln_flt_min;
    float r = s;
    s = s * u2f(0x3fb8aa3bu);
    s = s + 0.5f;
    s = __builtin_floorf(s);
    r = __builtin_fmaf(-s, u2f(0x3f317218u), r);
    s = s - 1.0f;
    int e = (int)__builtin_rintf(s);
    e = (int)((uint32_t)(e + 127) << 23);
    const float two_n = zero ? 0.0f : u2f((uint32_t)e);
    s = u2f(0x3c07cfceu);
    s = __builtin_fmaf(s, r, u2f(0x3d2b9d0du));
    s = __builtin_fmaf(s, r, u2f(0x3e2aad40u));
    s = __builtin_fmaf(s, r, u2f(0x3efffee3u));
    s = __builtin_fmaf(s, r, u2f(0x3f7ffffbu));
    s = __builtin_fmaf(s, r, 1.0f);
    s = s * two_n;
    s = s * 2.0f;
    return s;
}

// vrcp14ps, bit for bit (the reference's sigmoid uses it, tests/amx-mlp.cpp:453).  A power of two gives
// the exact reciprocal; otherwise the top 6 mantissa bits select a segment (table word = 18-bit
// intercept a << 10 | 10-bit slope b), the next 10 bits are the offset d, the 17-bit significand is
// (a*256 - b*d) >> 9 and the 7 low mantissa bits of the result are zero.  The table was derived from the
// instruction and the model agrees with it on all 2^32 inputs.
__constant__ static const uint32_t kRcp14Seg[64] = {
    0x0fffe7f1u, 0x0fc0dbd1u, 0x0f83cbb5u, 0x0f488399u, 0x0f0eef7du, 0x0ed71f65u, 0x0ea0cf4bu, 0x0e6c1b35u,
    0x0e38cb1du, 0x0e06f309u, 0x0dd662f3u, 0x0da72adfu, 0x0d7932cdu, 0x0d4c6ebbu, 0x0d20c6a9u, 0x0cf63297u,
    0x0cccbe87u, 0x0ca44677u, 0x0c7cda69u, 0x0c564e59u, 0x0c30b64bu, 0x0c0bfe3du, 0x0be82a31u, 0x0bc51623u,
    0x0ba2da17u, 0x0b81620bu, 0x0b60b601u, 0x0b40a9f5u, 0x0b215debu, 0x0b02b5dfu, 0x0ae4b9d5u, 0x0ac75dcbu,
    0x0aaaa9c3u, 0x0a8e7db9u, 0x0a72f1b1u, 0x0a57e1a7u, 0x0a3d699fu, 0x0a237597u, 0x0a0a018fu, 0x09f10d87u,
    0x09d8a181u, 0x09c09579u, 0x09a90571u, 0x0991ed6bu, 0x097b4565u, 0x0964f55du, 0x094f1957u, 0x0939a151u,
    0x09248d4bu, 0x090fd545u, 0x08fb793fu, 0x08e7893bu, 0x08d3d935u, 0x08c0852fu, 0x08ad912bu, 0x089add25u,
    0x08888921u, 0x08767d1du, 0x0864b517u, 0x08534d13u, 0x0842250fu, 0x08313d0bu, 0x08209507u, 0x08102d03u};

// inputs and results outside the normal range: denormal inputs are normalised (not flushed), a result
// beyond the largest float is inf, one below the normal range is the significand shifted right,
// zero -> inf, inf -> 0, NaN -> quiet NaN
static __device__ __attribute__((noinline)) float rcp14_special(float x) {
    const uint32_t u = f2u(x);
    const uint32_t sign = u & 0x80000000u;
    int ex = (int)((u >> 23) & 0xffu);
    uint32_t m = u & 0x7fffffu;
    if (ex == 0xff) return m ? u2f(u | 0x00400000u) : u2f(sign);
    if (ex == 0) {
        if (m == 0) return u2f(sign | 0x7f800000u);
        const int k = 31 - __builtin_clz(m);
        m = (m << (23 - k)) & 0x7fffffu;
        ex = k - 22;
    }
    uint32_t sig;
    int rex;
    if (m == 0) {
        sig = 0x10000u;
        rex = 254 - ex;
    } else {
        const uint32_t w = kRcp14Seg[m >> 17], d = (m >> 7) & 1023u;
        sig = (((w >> 10) << 8) - (w & 1023u) * d) >> 9;
        rex = 253 - ex;
    }
    if (rex >= 255) return u2f(sign | 0x7f800000u);
    uint32_t mant24 = sig << 7;
    if (rex <= 0) return u2f(sign | (mant24 >> (1 - rex)));
    return u2f(sign | ((uint32_t)rex << 23) | (mant24 & 0x7fffffu));
}

__device__ __forceinline__ float rcp14(float x) {
    const uint32_t u = f2u(x);
    const uint32_t ex = (u >> 23) & 0xffu, m = u & 0x7fffffu;
    if (!(ex - 1u < 252u)) return rcp14_special(x);  // exponent field 0, 253, 254, 255: rare
    const uint32_t w = kRcp14Seg[m >> 17], d = (m >> 7) & 1023u;
    const uint32_t sig = (((w >> 10) << 8) - (w & 1023u) * d) >> 9;
    const uint32_t body = m ? (((253u - ex) << 23) | ((sig << 7) & 0x7fffffu)) : ((254u - ex) << 23);
    return u2f((u & 0x80000000u) | body);
}

// tests/amx-mlp.cpp:450-456 — x * vrcp14ps(1 + exp(-x)), operation for operation
__device__ __forceinline__ float silu(float x) {
    const float e = exp_poly(0.0f - x);
    const float sig = rcp14(1.0f + e);
    return x * sig;
}

// silu(gate) * up on the 16 accumulator pairs a lane holds of one 32x32 block: the 16 chains advance in
// lockstep (a lone wavefront cannot issue dependent instructions back to back), the table look-ups of
// the reciprocal are issued together, and the rare operands outside the reciprocal's plain range are
// patched afterwards behind a wave-uniform branch.  Same operations per element as silu() above.
// `seg_of_lane` is kRcp14Seg[lane]: the 64-entry table lives in one register across the wavefront and is
// indexed with ds_bpermute (no memory access, no latency of a load to wait for per block).
__device__ __forceinline__ void silu_mul_x16(const float (&g)[16], const float (&up)[16], float (&r)[16], uint32_t seg_of_lane) {
    float one_plus[16];
#pragma unroll
    for (int v = 0; v < 16; v++) one_plus[v] = 1.0f + exp_poly(0.0f - g[v]);
    uint32_t w[16];
    bool special = false;
#pragma unroll
    for (int v = 0; v < 16; v++) {
        const uint32_t u = f2u(one_plus[v]);
        w[v] = (uint32_t)__builtin_amdgcn_ds_bpermute((int)(((u & 0x7fffffu) >> 17) << 2), (int)seg_of_lane);
        special |= !(((u >> 23) & 0xffu) - 1u < 252u);
    }
#pragma unroll
    for (int v = 0; v < 16; v++) {
        const uint32_t u = f2u(one_plus[v]);
        const uint32_t ex = (u >> 23) & 0xffu, m = u & 0x7fffffu, d = (m >> 7) & 1023u;
        const uint32_t sig = (((w[v] >> 10) << 8) - (w[v] & 1023u) * d) >> 9;
        const uint32_t body = m ? (((253u - ex) << 23) | ((sig << 7) & 0x7fffffu)) : ((254u - ex) << 23);
        r[v] = (g[v] * u2f((u & 0x80000000u) | body)) * up[v];
    }
    if (__builtin_amdgcn_ballot_w64(special) != 0) {
#pragma unroll
        for (int v = 0; v < 16; v++) {
            float x = one_plus[v];
            asm volatile("" : "+v"(x));  // keeps the patch inside this rarely taken branch
            const uint32_t ex = (f2u(x) >> 23) & 0xffu;
            if (!(ex - 1u < 252u)) r[v] = (g[v] * rcp14_special(x)) * up[v];
        }
    }
}

// 8 int8 (two dwords) -> 8 bf16, exact.  The SDWA form of v_cvt_f32_i32 picks and sign-extends the byte itself:
// 12 instructions with the packing against 20 for bit-field extract + int-to-float.
__device__ __forceinline__ bf16x8 s8x8_to_bf16(uint32_t lo, uint32_t hi) {
    float f[8];
#define MMX_CVT8(DST, SRC, BYTE) \
    asm("v_cvt_f32_i32_sdwa %0, sext(%1) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:" BYTE : "=v"(DST) : "v"(SRC))
    MMX_CVT8(f[0], lo, "BYTE_0");
    MMX_CVT8(f[1], lo, "BYTE_1");
    MMX_CVT8(f[2], lo, "BYTE_2");
    MMX_CVT8(f[3], lo, "BYTE_3");
    MMX_CVT8(f[4], hi, "BYTE_0");
    MMX_CVT8(f[5], hi, "BYTE_1");
    MMX_CVT8(f[6], hi, "BYTE_2");
    MMX_CVT8(f[7], hi, "BYTE_3");
#undef MMX_CVT8
    bf16x8 r;
#pragma unroll
    for (int e = 0; e < 8; e++) r[e] = (__bf16)f[e];
    return r;
}

// One dword of the above: the bf16 pair of bytes 2 PAIR and 2 PAIR + 1 of src (three instructions), for callers that
// spread a fragment's conversion over several issue slots.
template <int PAIR>
__device__ __forceinline__ uint32_t s8x2_to_bf16(uint32_t src) {
    float a, b;
    if constexpr (PAIR == 0) {
        asm("v_cvt_f32_i32_sdwa %0, sext(%1) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_0" : "=v"(a) : "v"(src));
        asm("v_cvt_f32_i32_sdwa %0, sext(%1) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_1" : "=v"(b) : "v"(src));
    } else {
        asm("v_cvt_f32_i32_sdwa %0, sext(%1) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_2" : "=v"(a) : "v"(src));
        asm("v_cvt_f32_i32_sdwa %0, sext(%1) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_3" : "=v"(b) : "v"(src));
    }
    bf16x2 r;
    r[0] = (__bf16)a;
    r[1] = (__bf16)b;
    return __builtin_bit_cast(uint32_t, r);
}

// fp32 -> bf16, round to nearest even (vcvtne2ps2bf16, include/kernels_amx.hpp:654)
__device__ __forceinline__ uint16_t to_bf16(float x) {
    __bf16 b = (__bf16)x;
    return __builtin_bit_cast(uint16_t, b);
}
__device__ __forceinline__ float from_bf16(uint16_t b) { return u2f((uint32_t)b << 16); }

// vcvtps2dq (round to nearest even; NaN / out of int32 range -> 0x80000000) followed by
// vpmovsdb signed saturation (include/kernels_amx.hpp:658-661)
__device__ __forceinline__ int8_t to_s8_sat(float r) {
    float t = __builtin_rintf(r);
    if (!(r >= -2147483648.0f && r < 2147483648.0f)) t = -128.0f;
    t = __builtin_fminf(__builtin_fmaxf(t, -128.0f), 127.0f);
    return (int8_t)(int)t;
}

// Four values through to_s8_sat packed into one dword (byte e = element e): round to nearest even, the
// x86 "indefinite" cases (NaN, |r| >= 2^31; -2^31 itself saturates to the same -128) forced to -128,
// then +128 and v_cvt_pk_u8_f32, whose saturation to [0, 255] is the clamp to [-128, 127], and one XOR
// turns the biased bytes back into two's complement.
__device__ __forceinline__ uint32_t to_s8_sat_x4(float r0, float r1, float r2, float r3) {
    const float r[4] = {r0, r1, r2, r3};
    uint32_t packed = 0;
#pragma unroll
    for (int e = 0; e < 4; e++) {
        float t = __builtin_rintf(r[e]);
        if (!(__builtin_fabsf(r[e]) < 2147483648.0f)) t = -128.0f;
        packed = __builtin_amdgcn_cvt_pk_u8_f32(t + 128.0f, (uint32_t)e, packed);
    }
    return packed ^ 0x80808080u;
}

}  // namespace mmx
