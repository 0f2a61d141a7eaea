// Decode-regime FC (M <= 32): y = PP(x · W[:, n0:n1]) over bf16, int8-compressed or int4-compressed weights.
//
// Stands in for the M<=16 / M<=32 branches of amx_kernel::Matmul (include/kernels_amx.hpp:1216-1253,
// 1297-1302), for Matmul<bf16,int8,float> at small M (:1381-1441) and for matmul16m_Wint8B
// (weight_compression/fc16m.cpp:451-502).  The kernel is a weight stream: every byte of W is read
// exactly once, in 1 KiB lane-contiguous fragments of the same packed layout the tile GEMM uses.
// The few activations ride in the other MFMA operand (32 columns, only M of them live), so the
// matrix core does the multiply-accumulate while the vector ALU only converts int8 -> bf16
// (exact: |w| <= 128 has at most 8 significant bits, as in include/kernels_amx.hpp:490-506) or int4 -> bf16
// (the reference has no int4 dequant, only a byte-copying stand-in: weight_compression/wcompress.hpp:90-134).
// K is split across the wavefronts of a workgroup; partial 32x32 blocks are summed through LDS.
#include "common.hpp"

namespace mmx {

// Packed weights are read exactly once per launch: nontemporal loads keep them from displacing x, the
// per-column operands and each other in the caches (int8 GEMV 4096x11008: 11.2 -> 10.5 us; MLP gate/up at
// M=1: 36.3 -> 33.4 us).
// compile-time loop: f(integral_constant<int, B>) ... f(integral_constant<int, E-1>)
template <int B, int E, typename F>
__device__ __forceinline__ void skinny_static_for(F&& f) {
    if constexpr (B < E) {
        f(std::integral_constant<int, B>{});
        skinny_static_for<B + 1, E>(f);
    }
}

#define MMX_WLOAD(ptr) __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(ptr))

struct SkinnyArgs {
    const char* x;
    int64_t ldx;  // bytes
    const char* Wp;
    int64_t panel_stride;  // bytes
    int M, K;
    int nfrag;    // 1 KiB fragments per panel
    int npanels;  // panels in Wp
    int n0, n1;
    int x_vec_ok;
    Epilogue ep;
    // K split of the chunked kernel (kslices > 1): slice blockIdx.y walks its share of the chunks, parks its sums in
    // ws_part and counts itself in at ws_cnt[blockIdx.x]; the slice that arrives last adds them up and stores
    char* ws_part;
    uint32_t* ws_cnt;
    int kslices;
    uint64_t* stamps;  // instrumented build only (-DMMX_STAMPS): 64 bytes per workgroup for its phase stamps, or null
};

// Development aid, compiled in with -DMMX_STAMPS only: thread 0 of workgroup blockIdx.x records the wall clock (100 MHz,
// slots 0 and 7) or the shader clock (the others) at a few points of the workgroup's life.
#ifdef MMX_STAMPS
#define SKINNY_STAMP(i)                                                                                                 \
    do {                                                                                                                \
        if (threadIdx.x == 0 && s.stamps)                                                                               \
            s.stamps[8 * (size_t)blockIdx.x + (i)] = (i) == 0 || (i) == 7 ? __builtin_amdgcn_s_memrealtime() : __builtin_readcyclecounter(); \
    } while (0)
#else
#define SKINNY_STAMP(i) do {} while (0)
#endif

__device__ __forceinline__ bf16x8 load_x8(const char* xrow, int k0, int K, bool live, bool vec_ok) {
    bf16x8 v;
#pragma unroll
    for (int e = 0; e < 8; e++) v[e] = (__bf16)0.0f;
    if (!live || k0 >= K) return v;
    if (vec_ok && k0 + 8 <= K) return *reinterpret_cast<const bf16x8*>(xrow + (int64_t)k0 * 2);
    const __bf16* p = reinterpret_cast<const __bf16*>(xrow);
#pragma unroll
    for (int e = 0; e < 8; e++)
        if (k0 + e < K) v[e] = p[k0 + e];
    return v;
}

// 8 int4 (one dword, element e in bits 4e .. 4e+3, two's complement) -> 8 bf16 holding q / 16, exact.
// v_cvt_off_f32_i4 maps the low nibble of its source to (signed nibble) / 16; its SDWA form picks the byte,
// so the even nibbles come straight from the dword and the odd ones from the dword shifted by four:
// 13 instructions per dword with the packing, against 20 for bit-field extract + int-to-float.  The
// callers multiply the finished sums by 16 (exact).
__device__ __forceinline__ bf16x8 s4x8_to_bf16_div16(uint32_t d) {
    const uint32_t dh = d >> 4;
    float f[8];
#define MMX_CVT4(DST, SRC, BYTE) \
    asm("v_cvt_off_f32_i4_sdwa %0, %1 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:" BYTE : "=v"(DST) : "v"(SRC))
    MMX_CVT4(f[0], d, "BYTE_0");
    MMX_CVT4(f[1], dh, "BYTE_0");
    MMX_CVT4(f[2], d, "BYTE_1");
    MMX_CVT4(f[3], dh, "BYTE_1");
    MMX_CVT4(f[4], d, "BYTE_2");
    MMX_CVT4(f[5], dh, "BYTE_2");
    MMX_CVT4(f[6], d, "BYTE_3");
    MMX_CVT4(f[7], dh, "BYTE_3");
#undef MMX_CVT4
    bf16x8 r;
#pragma unroll
    for (int e = 0; e < 8; e++) r[e] = (__bf16)f[e];
    return r;
}

__device__ __forceinline__ void store_out(const Epilogue& ep, int m, int n, float r) {
    char* row = ep.C + (int64_t)m * ep.ldc;
    switch (ep.out_dtype) {
    case MMX_BF16: reinterpret_cast<uint16_t*>(row)[n] = to_bf16(r); break;
    case MMX_I8: reinterpret_cast<int8_t*>(row)[n] = to_s8_sat(r); break;
    default: reinterpret_cast<float*>(row)[n] = r; break;
    }
}

// Per-column post-op operands of the (at most two) outputs per panel a thread finishes, requested
// before the weight stream starts so that their latency is not paid after it.
template <int NP>
struct FinishOperands {
    float deq[2][NP], bias[2][NP], q[2][NP];
};
template <int NP>
__device__ __forceinline__ void skinny_prefetch(const SkinnyArgs& s, int panel_first, int tid, FinishOperands<NP>& o) {
    const Epilogue& ep = s.ep;
#pragma unroll
    for (int t = 0; t < 2; t++) {
        const int idx = tid + 512 * t;
        const int v = idx >> 6, ln = idx & 63;
        const int nloc = 8 * (v >> 2) + 4 * (ln >> 5) + (v & 3);
        const bool row_live = (ln & 31) < s.M;
#pragma unroll
        for (int p = 0; p < NP; p++) {
            const int n = ((panel_first + p) << 5) + nloc;
            const bool ok = row_live && n < s.n1;  // (with SILU_GATE the only other step is DEQUANT, of gate and up each)
            o.deq[t][p] = ep.deq;
            o.bias[t][p] = 0.0f;
            o.q[t][p] = ep.q;
            if (ok && (ep.steps & MMX_PP_DEQUANT) && ep.deq_oc) o.deq[t][p] = ep.deq_oc[n];
            if (ok && (ep.steps & MMX_PP_BIAS)) o.bias[t][p] = ep.bias[n];
            if (ok && (ep.steps & MMX_PP_QUANT) && ep.q_oc) o.q[t][p] = ep.q_oc[n];
        }
    }
}

// cross-wave reduction of the partial 32x32 blocks + post-op + store (shared by the 8-wave decode kernels)
// ISUM: the partial sums are int32 (int8 activations), stored as bits.
// SPLIT: the workgroup holds one of s.kslices slices of K.  It writes its sums to the workspace at device scope (sc1:
// through to the level all XCDs share), waits until the stores have been acknowledged and counts itself in with a
// device-scope atomicInc that wraps to zero on the last arrival (ready for the next launch).  The last to arrive adds
// the slices' sums in slice order 0, 1, 2, ... - so the result does not depend on who came last - and goes on to the
// post-op; the others are done.  Nobody waits for anybody.
template <int NP, bool ISUM = false, bool SPLIT = false>
__device__ __forceinline__ void skinny_finish(const SkinnyArgs& s, const float (&red)[8][NP][16][64], int panel_first, int tid,
                                              const FinishOperands<NP>& o, int slice = 0) {
    const Epilogue& ep = s.ep;
    float fsum[2][NP];
    int isum2[2][NP];
#pragma unroll
    for (int t = 0; t < 2; t++) {
        const int idx = tid + 512 * t;
        const int v = idx >> 6, ln = idx & 63;
#pragma unroll
        for (int p = 0; p < NP; p++) {
            if constexpr (ISUM) {
                int acc = 0;
#pragma unroll
                for (int w8 = 0; w8 < 8; w8++) acc += reinterpret_cast<const int*>(&red[w8][p][v][ln])[0];
                isum2[t][p] = acc;
            } else {
                float acc = 0.0f;
#pragma unroll
                for (int w8 = 0; w8 < 8; w8++) acc += red[w8][p][v][ln];
                fsum[t][p] = acc;
            }
        }
    }
    if constexpr (SPLIT) {
        const int S = s.kslices;
        if (S > 1) {
            constexpr int AUX_SC1 = 16;             // cache policy operand of the buffer instructions: device scope
            constexpr int UNIT = 2 * NP * 512 * 4;  // bytes of one workgroup's sums
            __amdgpu_buffer_rsrc_t parts =
                __builtin_amdgcn_make_buffer_rsrc(s.ws_part + (int64_t)blockIdx.x * S * UNIT, 0, S * UNIT, 0x00020000);
#pragma unroll
            for (int t = 0; t < 2; t++)
#pragma unroll
                for (int p = 0; p < NP; p++) {
                    uint32_t bits;
                    if constexpr (ISUM) bits = (uint32_t)isum2[t][p];
                    else bits = __builtin_bit_cast(uint32_t, fsum[t][p]);
                    __builtin_amdgcn_raw_buffer_store_b32(bits, parts, slice * UNIT + ((t * NP + p) * 512 + tid) * 4, 0, AUX_SC1);
                }
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // every store of this wave has been acknowledged
            __syncthreads();                                  // ... and every read of the reduction scratch is done
            volatile uint32_t* flag = reinterpret_cast<volatile uint32_t*>(const_cast<float*>(&red[0][0][0][0]));
            if (tid == 0) *flag = atomicInc(s.ws_cnt + blockIdx.x, (uint32_t)S - 1u);
            __syncthreads();
            if (*flag != (uint32_t)S - 1u) return;
            asm volatile("" ::: "memory");
#pragma unroll
            for (int t = 0; t < 2; t++)
#pragma unroll
                for (int p = 0; p < NP; p++) {
                    float fa = 0.0f;
                    int ia = 0;
#pragma unroll
                    for (int sl = 0; sl < 4; sl++) {
                        if (sl < S) {
                            uint32_t bits;
                            if (sl == slice) {
                                if constexpr (ISUM) bits = (uint32_t)isum2[t][p];
                                else bits = __builtin_bit_cast(uint32_t, fsum[t][p]);
                            } else {
                                bits = __builtin_amdgcn_raw_buffer_load_b32(parts, sl * UNIT + ((t * NP + p) * 512 + tid) * 4, 0, AUX_SC1);
                            }
                            if constexpr (ISUM) ia = sl == 0 ? (int)bits : ia + (int)bits;
                            else fa = sl == 0 ? __builtin_bit_cast(float, bits) : fa + __builtin_bit_cast(float, bits);
                        }
                    }
                    if constexpr (ISUM) isum2[t][p] = ia;
                    else fsum[t][p] = fa;
                }
        }
    }
#pragma unroll
    for (int t = 0; t < 2; t++) {
        const int idx = tid + 512 * t;
        const int v = idx >> 6, ln = idx & 63;
        const int m = ln & 31;
        if (m >= s.M) continue;
        const int nloc = 8 * (v >> 2) + 4 * (ln >> 5) + (v & 3);
        float sum[NP];
        int isum[NP];
#pragma unroll
        for (int p = 0; p < NP; p++) {
            if constexpr (ISUM) {
                isum[p] = isum2[t][p];
                sum[p] = (float)isum2[t][p];  // vcvtdq2ps, round to nearest even (include/kernels_amx.hpp:631-634)
            } else {
                sum[p] = fsum[t][p];
            }
        }
        if (ISUM && ep.out_dtype == MMX_I32) {  // raw accumulators (steps == 0)
#pragma unroll
            for (int p = 0; p < NP; p++) {
                const int n = ((panel_first + p) << 5) + nloc;
                if (n < s.n1) reinterpret_cast<int*>(ep.C + (int64_t)m * ep.ldc)[n] = isum[p];
            }
        } else if (ep.steps & MMX_PP_SILU_GATE) {
            if constexpr (NP == 2) {
                const int n = ((panel_first >> 1) << 5) + nloc;  // output column (half width)
                float gate = sum[0], up = sum[1];
                if (ep.steps & MMX_PP_DEQUANT) {  // compressed weights: each of the two sums by the scale of its own column
                    gate = gate * o.deq[t][0];
                    up = up * o.deq[t][1];
                }
                if (n < (s.n1 >> 1)) store_out(ep, m, n, silu(gate) * up);
            }
        } else {
#pragma unroll
            for (int p = 0; p < NP; p++) {
                const int n = ((panel_first + p) << 5) + nloc;
                if (n >= s.n1) continue;
                float r = sum[p];
                if (ep.steps & MMX_PP_DEQUANT) r = r * o.deq[t][p];
                if (ep.steps & MMX_PP_BIAS) r = r + o.bias[t][p];
                if (ep.steps & MMX_PP_GELU) r = gelu_erf_minimax(r);
                if (ep.steps & MMX_PP_QUANT) r = r * o.q[t][p];
                store_out(ep, m, n, r);
            }
        }
    }
}

// WK: weights are bf16 (0), int8 (1) or int4 (2); a 1 KiB fragment is 32 columns x 16, 32 or 64 of k
template <int WK, int NP>
__global__ __launch_bounds__(512) void skinny_kernel(const SkinnyArgs s) {
    constexpr bool W8 = WK == 1, W4 = WK == 2;
    constexpr int U = 4;  // fragments in flight per wave
    __shared__ float red[8][NP][16][64];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, g32 = lane >> 5;
    const int panel_first = (s.n0 >> 5) + blockIdx.x * NP;
    const int panel_end = (s.n1 + 31) >> 5;

    f32x16 acc[NP];
#pragma unroll
    for (int p = 0; p < NP; p++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[p][v] = 0.0f;

    FinishOperands<NP> fin;
    skinny_prefetch<NP>(s, panel_first, tid, fin);

    const int per_wave = (s.nfrag + 7) / 8;
    const int f_begin = wave * per_wave;
    const int f_end = (f_begin + per_wave) < s.nfrag ? (f_begin + per_wave) : s.nfrag;
    const bool live = l32 < s.M;
    const char* xrow = s.x + (int64_t)(live ? l32 : 0) * s.ldx;

    for (int f0 = f_begin; f0 < f_end; f0 += U) {
        u32x4 w[NP][U];
        bf16x8 xa[U], xb[U], xc[U], xd[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int f = f0 + u;
#pragma unroll
            for (int p = 0; p < NP; p++) {
                const int panel = panel_first + p;
                w[p][u] = u32x4{0u, 0u, 0u, 0u};
                if (f < f_end && panel < panel_end && panel < s.npanels)
                    w[p][u] = MMX_WLOAD(s.Wp + (int64_t)panel * s.panel_stride + (int64_t)f * 1024 + lane * 16);
            }
            if constexpr (W4) {
                const int k0 = 64 * f + 32 * g32;
                xa[u] = load_x8(xrow, k0, s.K, live && f < f_end, s.x_vec_ok);
                xb[u] = load_x8(xrow, k0 + 8, s.K, live && f < f_end, s.x_vec_ok);
                xc[u] = load_x8(xrow, k0 + 16, s.K, live && f < f_end, s.x_vec_ok);
                xd[u] = load_x8(xrow, k0 + 24, s.K, live && f < f_end, s.x_vec_ok);
            } else if constexpr (W8) {
                const int k0 = 32 * f + 16 * g32;
                xa[u] = load_x8(xrow, k0, s.K, live && f < f_end, s.x_vec_ok);
                xb[u] = load_x8(xrow, k0 + 8, s.K, live && f < f_end, s.x_vec_ok);
            } else {
                xa[u] = load_x8(xrow, 16 * f + 8 * g32, s.K, live && f < f_end, s.x_vec_ok);
            }
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
#pragma unroll
            for (int p = 0; p < NP; p++) {
                if constexpr (W4) {
                    acc[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(s4x8_to_bf16_div16(w[p][u].x), xa[u], acc[p], 0, 0, 0);
                    acc[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(s4x8_to_bf16_div16(w[p][u].y), xb[u], acc[p], 0, 0, 0);
                    acc[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(s4x8_to_bf16_div16(w[p][u].z), xc[u], acc[p], 0, 0, 0);
                    acc[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(s4x8_to_bf16_div16(w[p][u].w), xd[u], acc[p], 0, 0, 0);
                } else if constexpr (W8) {
                    acc[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(s8x8_to_bf16(w[p][u].x, w[p][u].y), xa[u], acc[p], 0, 0, 0);
                    acc[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(s8x8_to_bf16(w[p][u].z, w[p][u].w), xb[u], acc[p], 0, 0, 0);
                } else {
                    acc[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, w[p][u]), xa[u], acc[p], 0, 0, 0);
                }
            }
        }
    }

#pragma unroll
    for (int p = 0; p < NP; p++)
#pragma unroll
        for (int v = 0; v < 16; v++) red[wave][p][v][lane] = W4 ? acc[p][v] * 16.0f : acc[p][v];  // int4 operands were q / 16
    __syncthreads();

    skinny_finish<NP>(s, red, panel_first, tid, fin);
}

// ---- direct variant for aligned operands whose x does not fit in LDS, few rows (4 < M <= 8); launched for
// plain bf16 weights only (for int8 weights and gate/up pairs the chunked variant below measured faster) ----
// Every lane reads its own 16 (bf16 weights) or 32 (int8 weights) bytes of x per fragment straight from
// global memory (served by L2: all workgroups read the same x) together with the fragment, U of
// them in flight per wave as a rolling window.  Lanes of rows >= M read row 0: in the MFMA an output
// column depends on its own activation row only, and the columns of those lanes are never stored.
// Requires 16-byte aligned x rows and a K that fills whole 128-byte groups of the packed weights.
template <bool W8, int NP>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(4, 4))) void skinny_direct_kernel(const SkinnyArgs s) {
    constexpr int U = (W8 ? 6 : 8) / NP;
    constexpr int XB = W8 ? 64 : 32;  // bytes of a row of x one fragment covers
    __shared__ float red[8][NP][16][64];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, g32 = lane >> 5;
    const int panel_first = (s.n0 >> 5) + blockIdx.x * NP;
    const int panel_end = (s.n1 + 31) >> 5;

    FinishOperands<NP> fin;
    skinny_prefetch<NP>(s, panel_first, tid, fin);
    __builtin_amdgcn_sched_barrier(0);

    f32x16 acc[NP];
#pragma unroll
    for (int p = 0; p < NP; p++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[p][v] = 0.0f;

    const int per_wave = (s.nfrag + 7) / 8;
    const int f_begin = wave * per_wave;
    const int f_last = s.nfrag - 1;
    const char* wbase[NP];
#pragma unroll
    for (int p = 0; p < NP; p++) {
        int panel = panel_first + p;
        panel = (panel < panel_end && panel < s.npanels) ? panel : s.npanels - 1;
        wbase[p] = s.Wp + (int64_t)panel * s.panel_stride + lane * 16;
    }
    const char* xlane = s.x + (int64_t)(l32 < s.M ? l32 : 0) * s.ldx + g32 * (XB / 2);
    const int nbatch = (per_wave + U - 1) / U;

    u32x4 w[NP][U];
    bf16x8 xa[U], xb[W8 ? U : 1];
#define MMX_REQUEST(BT, UU)                                                                 \
    do {                                                                                    \
        int f_ = f_begin + (BT) * U + (UU);                                                 \
        f_ = f_ < f_last ? f_ : f_last;                                                     \
        _Pragma("unroll") for (int p = 0; p < NP; p++)                                      \
            w[p][UU] = MMX_WLOAD(wbase[p] + (int64_t)f_ * 1024);                         \
        xa[UU] = *reinterpret_cast<const bf16x8*>(xlane + (int64_t)f_ * XB);                \
        if constexpr (W8) xb[UU] = *reinterpret_cast<const bf16x8*>(xlane + (int64_t)f_ * XB + 16); \
    } while (0)
    // a fragment index past this wave's share (or past the end of K) contributes nothing: its weights are zeroed
#define MMX_MULTIPLY(BT, UU)                                                                \
    do {                                                                                    \
        const int f_ = f_begin + (BT) * U + (UU);                                           \
        const bool valid_ = (f_ - f_begin) < per_wave && f_ <= f_last; /* scalar */         \
        _Pragma("unroll") for (int p = 0; p < NP; p++) {                                    \
            const u32x4 wv_ = valid_ ? w[p][UU] : u32x4{0u, 0u, 0u, 0u};                    \
            if constexpr (W8) {                                                             \
                acc[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(s8x8_to_bf16(wv_.x, wv_.y), xa[UU], acc[p], 0, 0, 0); \
                acc[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(s8x8_to_bf16(wv_.z, wv_.w), xb[UU], acc[p], 0, 0, 0); \
            } else {                                                                        \
                acc[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, wv_), xa[UU], acc[p], 0, 0, 0); \
            }                                                                               \
        }                                                                                   \
    } while (0)
#pragma unroll
    for (int u = 0; u < U; u++) MMX_REQUEST(0, u);
    for (int bt = 0; bt + 1 < nbatch; bt++) {
#pragma unroll
        for (int u = 0; u < U; u++) {
            MMX_MULTIPLY(bt, u);
            MMX_REQUEST(bt + 1, u);
        }
    }
#pragma unroll
    for (int u = 0; u < U; u++) MMX_MULTIPLY(nbatch - 1, u);
#undef MMX_REQUEST
#undef MMX_MULTIPLY

#pragma unroll
    for (int p = 0; p < NP; p++)
#pragma unroll
        for (int v = 0; v < 16; v++) red[wave][p][v][lane] = acc[p][v];
    __syncthreads();
    skinny_finish<NP>(s, red, panel_first, tid, fin);
}

// ---- chunked variant for aligned operands whose x does not fit in LDS, many rows (8 < M <= 32) ------
// K is walked in chunks of 8*FPW fragments; in a chunk every wave multiplies FPW fragments of each
// panel.  The x a chunk needs ([M][RB bytes], RB = 8*FPW fragments' worth of a row) is fetched by the
// whole workgroup with fully coalesced 16-byte loads (a lane per 16 bytes, rows back to back), written
// to LDS and read from there as MFMA operands: fetched per lane straight from global memory, the 32
// rows of an operand make every load touch 32 cache lines, and the CU's vector cache becomes the
// bottleneck (19 us instead of 12 for the 4096 x 11008 int8 GEMV at M = 16).
// Weights and x of chunk c+W are requested while chunk c is multiplied (W = 3 chunks in flight, more
// measured no faster; all
// loads are ordinary loads, so the compiler's own counting of outstanding loads places the waits).
// Two LDS buffers: chunk c+1 is written while slower waves still read chunk c; the barrier of chunk
// c+1 is what allows chunk c+2 to overwrite chunk c.  16-byte pieces of a row are XOR-swizzled with
// the row so that the 32 rows an operand reads spread over the banks.
// Lanes of rows >= M read row 0 (their output columns are never stored); fragments past the end of K
// get zero weights and a clamped (finite) x.
// WK: weights are bf16 (0), int8 (1) or int4 (2), 3: int8 weights and int8 activations (int32 sums);
// XD: 16-byte x loads per thread per chunk (8 KiB of x each)
template <int WK, int NP, int FPW, int XD, int WIN = 0>  // WIN: chunks in flight (0: what the case's registers hold)
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(4, 4))) void skinny_chunk_kernel(const SkinnyArgs s) {
    constexpr bool W8 = WK == 1, W4 = WK == 2, I8A = WK == 3;
    using accv = std::conditional_t<I8A, i32x16, f32x16>;
    // chunks in flight (what 128 registers hold)
    constexpr int W = WIN ? WIN : (W4 ? (XD >= 4 ? 2 : 3) : ((FPW == 2 && (W8 || NP == 2)) ? 2 : 3));
    constexpr int XB = W4 ? 128 : (W8 ? 64 : 32);  // bytes of a row of x one fragment covers (int8 x int8: 32)
    constexpr int FC = 8 * FPW;          // fragments per chunk
    constexpr int RB = FC * XB;          // bytes of a row of x per chunk
    constexpr int BUF = 8 * XD * 1024;   // one LDS buffer: BUF / RB rows of x (the launcher checks M against it)
    static_assert(RB >= 256 && BUF / RB >= 16, "chunk geometry");
    extern __shared__ __attribute__((aligned(1024))) char smem[];  // 2 x BUF, later the cross-wave reduction
    typedef float Red[8][NP][16][64];
    Red& red = *reinterpret_cast<Red*>(smem);

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, g32 = lane >> 5;
    const int panel_first = (s.n0 >> 5) + blockIdx.x * NP;
    const int panel_end = (s.n1 + 31) >> 5;

    FinishOperands<NP> fin;
    skinny_prefetch<NP>(s, panel_first, tid, fin);

    accv acc[NP];
#pragma unroll
    for (int p = 0; p < NP; p++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[p][v] = 0;

    const int f_last = s.nfrag - 1;
    // chunks [chunk0, nchunk) are this workgroup's: all of them, or slice blockIdx.y of kslices equal shares
    const int nchunk_all = (s.nfrag + FC - 1) / FC;
    const int slice = s.kslices > 1 ? (int)blockIdx.y : 0;
    const int per_slice = (nchunk_all + s.kslices - 1) / s.kslices;
    const int chunk0 = slice * per_slice;
    const int nchunk = chunk0 + per_slice < nchunk_all ? chunk0 + per_slice : nchunk_all;
    const int row_bytes = s.K * (I8A ? 1 : 2);
    const char* wbase[NP];
#pragma unroll
    for (int p = 0; p < NP; p++) {
        int panel = panel_first + p;
        panel = (panel < panel_end && panel < s.npanels) ? panel : s.npanels - 1;
        wbase[p] = s.Wp + (int64_t)panel * s.panel_stride + lane * 16;
    }
    // this thread's share of a chunk of x: XD pieces of 16 bytes; piece t sits at (row xrow[t], 16-byte
    // column xcol[t]) of the chunk and goes to LDS offset xdst[t]
    const char* xsrc[XD];
    int xcol[XD], xdst[XD];
#pragma unroll
    for (int t = 0; t < XD; t++) {
        const int pos = (wave + 8 * t) * 1024 + lane * 16;
        const int r = pos / RB, cl = (pos % RB) / 16;
        xsrc[t] = s.x + (int64_t)(r < s.M ? r : s.M - 1) * s.ldx;
        xcol[t] = cl * 16;
        xdst[t] = r * RB + ((cl ^ (r & 15)) * 16);
    }
    const int mrow = l32 < s.M ? l32 : 0;
    const char* xread = smem + mrow * RB;
    const int xswz = mrow & 15;

    u32x4 w[W][FPW][NP];
    bf16x8 xr[W][XD];
#define MMX_LOAD(C, J)                                                                                         \
    do {                                                                                                       \
        _Pragma("unroll") for (int t = 0; t < XD; t++) {                                                       \
            int kb_ = (C) * RB + xcol[t];                                                                      \
            kb_ = kb_ < row_bytes - 16 ? kb_ : row_bytes - 16;                                                 \
            xr[J][t] = *reinterpret_cast<const bf16x8*>(xsrc[t] + kb_);                                        \
        }                                                                                                      \
        _Pragma("unroll") for (int u = 0; u < FPW; u++) {                                                      \
            int f_ = (C) * FC + wave * FPW + u;                                                                \
            f_ = f_ < f_last ? f_ : f_last;                                                                    \
            _Pragma("unroll") for (int p = 0; p < NP; p++)                                                     \
                w[J][u][p] = MMX_WLOAD(wbase[p] + (int64_t)f_ * 1024);                                      \
        }                                                                                                      \
    } while (0)
#define MMX_CHUNK(C, J)                                                                                        \
    do {                                                                                                       \
        char* buf_ = smem + ((C) & 1) * BUF;                                                                   \
        _Pragma("unroll") for (int t = 0; t < XD; t++) *reinterpret_cast<bf16x8*>(buf_ + xdst[t]) = xr[J][t];  \
        __syncthreads();                                                                                       \
        _Pragma("unroll") for (int u = 0; u < FPW; u++) {                                                      \
            const int fl_ = wave * FPW + u;                                                                    \
            const bool valid_ = (C) * FC + fl_ <= f_last; /* scalar */                                         \
            const char* xb_ = xread + ((C) & 1) * BUF;                                                         \
            if constexpr (I8A) {                                                                               \
                const int c0_ = fl_ * 2 + g32;                                                                 \
                const i32x4 xq_ = *reinterpret_cast<const i32x4*>(xb_ + ((c0_ ^ xswz) * 16));                  \
                _Pragma("unroll") for (int p = 0; p < NP; p++) {                                               \
                    const u32x4 wv_ = valid_ ? w[J][u][p] : u32x4{0u, 0u, 0u, 0u};                             \
                    acc[p] = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, wv_), xq_, acc[p], 0, 0, 0); \
                }                                                                                              \
            } else if constexpr (W4) {                                                                         \
                const int c0_ = fl_ * 8 + g32 * 4;                                                             \
                _Pragma("unroll") for (int i_ = 0; i_ < 4; i_++) {                                             \
                    const bf16x8 xq_ = *reinterpret_cast<const bf16x8*>(xb_ + (((c0_ + i_) ^ xswz) * 16));     \
                    _Pragma("unroll") for (int p = 0; p < NP; p++) {                                           \
                        const u32x4 wv_ = valid_ ? w[J][u][p] : u32x4{0u, 0u, 0u, 0u};                         \
                        acc[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(s4x8_to_bf16_div16(wv_[i_]), xq_, acc[p], 0, 0, 0); \
                    }                                                                                          \
                }                                                                                              \
            } else if constexpr (W8) {                                                                         \
                const int c0_ = fl_ * 4 + g32 * 2;                                                             \
                const bf16x8 xa_ = *reinterpret_cast<const bf16x8*>(xb_ + ((c0_ ^ xswz) * 16));                \
                const bf16x8 xc_ = *reinterpret_cast<const bf16x8*>(xb_ + (((c0_ + 1) ^ xswz) * 16));          \
                _Pragma("unroll") for (int p = 0; p < NP; p++) {                                               \
                    const u32x4 wv_ = valid_ ? w[J][u][p] : u32x4{0u, 0u, 0u, 0u};                             \
                    acc[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(s8x8_to_bf16(wv_.x, wv_.y), xa_, acc[p], 0, 0, 0); \
                    acc[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(s8x8_to_bf16(wv_.z, wv_.w), xc_, acc[p], 0, 0, 0); \
                }                                                                                              \
            } else {                                                                                           \
                const int c0_ = fl_ * 2 + g32;                                                                 \
                const bf16x8 xa_ = *reinterpret_cast<const bf16x8*>(xb_ + ((c0_ ^ xswz) * 16));                \
                _Pragma("unroll") for (int p = 0; p < NP; p++) {                                               \
                    const u32x4 wv_ = valid_ ? w[J][u][p] : u32x4{0u, 0u, 0u, 0u};                             \
                    acc[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, wv_), xa_, acc[p], 0, 0, 0); \
                }                                                                                              \
            }                                                                                                  \
        }                                                                                                      \
    } while (0)

    skinny_static_for<0, W>([&](auto j_c) {
        constexpr int J = decltype(j_c)::value;
        if (chunk0 + J < nchunk) MMX_LOAD(chunk0 + J, J);
    });
    for (int c0 = chunk0; c0 < nchunk; c0 += W) {
        skinny_static_for<0, W>([&](auto j_c) {
            constexpr int J = decltype(j_c)::value;
            if (c0 + J < nchunk) {
                MMX_CHUNK(c0 + J, J);
                if (c0 + J + W < nchunk) MMX_LOAD(c0 + J + W, J);
            }
        });
    }
#undef MMX_LOAD
#undef MMX_CHUNK

    __syncthreads();  // all reads of x are done: the buffers become the reduction scratch
#pragma unroll
    for (int p = 0; p < NP; p++)
#pragma unroll
        for (int v = 0; v < 16; v++) {
            if constexpr (I8A) reinterpret_cast<int*>(&red[wave][p][v][lane])[0] = acc[p][v];  // the sums travel as bits
            else red[wave][p][v][lane] = W4 ? acc[p][v] * 16.0f : acc[p][v];  // int4 operands were q / 16
        }
    __syncthreads();
    if constexpr (WIN != 0 && NP == 1) skinny_finish<NP, I8A, true>(s, red, panel_first, tid, fin, slice);  // (the forms launched with a K split)
    else skinny_finish<NP, I8A>(s, red, panel_first, tid, fin);
}

// ---- streaming variant for the smallest M -----------------------------------------------------------
// When the activations fit in LDS the kernel is organised around one goal: have every byte of the
// weights requested from HBM as early as possible.  x goes from global memory straight into LDS
// (global_load_lds, no registers), the few per-column post-op operands are requested, then each wave
// issues 16 KiB of weight loads.  Loads return in order, so "at most the weight loads outstanding"
// means x has landed: one barrier, and the weights are consumed in arrival order.  x fragments are
// read from LDS (their own counter: they never queue behind the weight stream).  Lanes of rows >= M
// and fragments past the end of K read a row of zeros instead, so the loop has no branches.
// Requires K to fill whole 128-byte groups of the packed weights (no zero padding of x needed).
// 128 VGPRs at most: two workgroups per CU, so that every panel of an 11008-column matrix is resident at once.
// ONE: every wave's share of K is a single batch (the common decode shapes); a variant of its own so that
// each kernel holds one code path and stays within its registers.
// UW: batch of the rolling window if not the full register set (the last batch of a wave's share of K is filled up with
// repeats of the last load, which cost what they are a share of the loads: the launcher picks the batch with the fewest)
template <int WK, int NP, bool ONE, int UW = 0>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(4, 4))) void skinny_stream_kernel(const SkinnyArgs s, int zero_off) {
    constexpr bool W8 = WK == 1, W4 = WK == 2, I8A = WK == 3;  // 3: int8 weights AND int8 activations, int32 sums
    // 4: int8 weights and ONE row of x without the matrix cores: every lane owns one column and half of a fragment's
    // k, v_dot2_f32_bf16 on the converted pairs, and one cross-lane add at the end.  Kept as the measured
    // counterpart of WK = 1 (option "decode_valu"); the post-op is the same code.
    constexpr bool W8V = WK == 4, VALU = W8V;
    static_assert(!VALU || NP == 1, "the VALU form is a single-panel kernel");
    using accv = std::conditional_t<I8A, i32x16, f32x16>;
    // fragments per panel per wave in flight at once (16 KiB of weights; int4: 8 KiB, a fragment holds 64 of k
    // and unpacking it costs more than streaming it)
    constexpr int U = UW ? UW : (W4 ? 8 : 16) / NP;
    // [M][K] bf16, then at zero_off a row of zeros; once x has been used up, the cross-wave reduction scratch
    // (the launcher allocates the larger of the two: stream_lds_bytes)
    extern __shared__ __attribute__((aligned(1024))) char xs[];
    typedef float Red[8][NP][16][64];
    Red& red = *reinterpret_cast<Red*>(xs);

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // scalar: keeps the control flow below uniform
    const int l32 = lane & 31, g32 = lane >> 5;
    const int panel_first = (s.n0 >> 5) + blockIdx.x * NP;
    const int panel_end = (s.n1 + 31) >> 5;
    const int row_bytes = s.K * (I8A ? 1 : 2);
    const int real_bytes = s.M * row_bytes;
    SKINNY_STAMP(0);
    SKINNY_STAMP(1);

    // x -> LDS, 1 KiB per wave per instruction; the lanes past the end of x re-read its last 16 bytes
    // into the gap in front of the zero row (zero_off is the next multiple of 1 KiB)
    {
        const uint32_t lds_base = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)xs);
        for (int off = wave * 1024; off < real_bytes; off += 8 * 1024) {
            int bo = off + lane * 16;
            bo = bo < real_bytes ? bo : real_bytes - 16;
            const int m = bo / row_bytes;
            const char* src = s.x + (int64_t)m * s.ldx + (bo - m * row_bytes);
            const uint32_t m0v = lds_base + off;
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(m0v), "v"(src) : "memory");
        }
        for (int c = tid * 16; c < row_bytes; c += 512 * 16) *reinterpret_cast<u32x4*>(xs + zero_off + c) = u32x4{0u, 0u, 0u, 0u};
    }
    // the few per-column operands of the post-op travel ahead of the weights as well
    FinishOperands<NP> fin;
    skinny_prefetch<NP>(s, panel_first, tid, fin);
    __builtin_amdgcn_sched_barrier(0);

    accv acc[NP];
    float vacc[4] = {0.0f, 0.0f, 0.0f, 0.0f};  // VALU form: four independent chains per lane
#pragma unroll
    for (int p = 0; p < NP; p++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[p][v] = 0;

    // wave w multiplies fragments [w*per_wave, (w+1)*per_wave); indices past the end are clamped for the
    // load and paired with the zero row of x
    const int per_wave = (s.nfrag + 7) / 8;
    const int f_begin = wave * per_wave;
    const int f_last = s.nfrag - 1;
    const char* wbase[NP];
#pragma unroll
    for (int p = 0; p < NP; p++) {
        int panel = panel_first + p;
        panel = (panel < panel_end && panel < s.npanels) ? panel : s.npanels - 1;  // columns past n1 are never stored
        wbase[p] = s.Wp + (int64_t)panel * s.panel_stride + lane * 16;
    }
    const char* zrow = xs + zero_off;
    const char* xrow = (VALU || l32 < s.M) ? xs + (VALU ? 0 : l32) * row_bytes : zrow;
    const int nbatch = (per_wave + U - 1) / U;  // same for every wave
    // U fragments per panel are in flight per wave at all times: register set u holds fragment u of a
    // batch and is re-requested for the next batch as soon as it has been multiplied
    u32x4 w[NP][U];
#define MMX_REQUEST(BT, UU)                                                                                     \
    do {                                                                                                        \
        int f_ = f_begin + (BT) * U + (UU);                                                                     \
        f_ = f_ < f_last ? f_ : f_last;                                                                         \
        _Pragma("unroll") for (int p = 0; p < NP; p++)                                                          \
            w[p][UU] = MMX_WLOAD(wbase[p] + (int64_t)f_ * 1024);                                             \
    } while (0)
#define MMX_MULTIPLY(BT, UU)                                                                                    \
    do {                                                                                                        \
        const int f_ = f_begin + (BT) * U + (UU);                                                               \
        const bool valid_ = (f_ - f_begin) < per_wave && f_ <= f_last; /* scalar */                             \
        const int fc_ = f_ < f_last ? f_ : f_last;                                                              \
        const char* xr_ = valid_ ? xrow : zrow;                                                                 \
        if constexpr (I8A) {                                                                                    \
            const i32x4 xq_ = *reinterpret_cast<const i32x4*>(xr_ + 32 * fc_ + 16 * g32);                       \
            _Pragma("unroll") for (int p = 0; p < NP; p++)                                                      \
                acc[p] = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, w[p][UU]), xq_, acc[p], 0, 0, 0); \
        } else if constexpr (W4) {                                                                              \
            _Pragma("unroll") for (int i_ = 0; i_ < 4; i_++) {                                                  \
                const bf16x8 xq_ = *reinterpret_cast<const bf16x8*>(xr_ + (64 * fc_ + 32 * g32 + 8 * i_) * 2);  \
                _Pragma("unroll") for (int p = 0; p < NP; p++)                                                  \
                    acc[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(s4x8_to_bf16_div16(w[p][UU][i_]), xq_, acc[p], 0, 0, 0); \
            }                                                                                                   \
        } else if constexpr (W8V) {                                                                             \
            const u32x4 xa_ = *reinterpret_cast<const u32x4*>(xr_ + (32 * fc_ + 16 * g32) * 2);                 \
            const u32x4 xb_ = *reinterpret_cast<const u32x4*>(xr_ + (32 * fc_ + 16 * g32 + 8) * 2);             \
            const u32x4 wa_ = __builtin_bit_cast(u32x4, s8x8_to_bf16(w[0][UU].x, w[0][UU].y));                  \
            const u32x4 wb_ = __builtin_bit_cast(u32x4, s8x8_to_bf16(w[0][UU].z, w[0][UU].w));                  \
            _Pragma("unroll") for (int i_ = 0; i_ < 4; i_++) {                                                  \
                const uint32_t wa1_ = wa_[i_], xa1_ = xa_[i_], wb1_ = wb_[i_], xb1_ = xb_[i_];                  \
                vacc[i_] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, wa1_), __builtin_bit_cast(bf16x2, xa1_), vacc[i_], false); \
                vacc[i_] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, wb1_), __builtin_bit_cast(bf16x2, xb1_), vacc[i_], false); \
            }                                                                                                   \
        } else if constexpr (W8) {                                                                              \
            const bf16x8 xa_ = *reinterpret_cast<const bf16x8*>(xr_ + (32 * fc_ + 16 * g32) * 2);               \
            const bf16x8 xb_ = *reinterpret_cast<const bf16x8*>(xr_ + (32 * fc_ + 16 * g32 + 8) * 2);           \
            _Pragma("unroll") for (int p = 0; p < NP; p++) {                                                    \
                acc[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(s8x8_to_bf16(w[p][UU].x, w[p][UU].y), xa_, acc[p], 0, 0, 0); \
                acc[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(s8x8_to_bf16(w[p][UU].z, w[p][UU].w), xb_, acc[p], 0, 0, 0); \
            }                                                                                                   \
        } else {                                                                                                \
            const bf16x8 xa_ = *reinterpret_cast<const bf16x8*>(xr_ + (16 * fc_ + 8 * g32) * 2);                \
            _Pragma("unroll") for (int p = 0; p < NP; p++)                                                      \
                acc[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, w[p][UU]), xa_, acc[p], 0, 0, 0); \
        }                                                                                                       \
    } while (0)
    {
        // A CU accepts only so many outstanding requests: a wave that had to get all of its weight
        // requests accepted before it may look at x would sit there for most of the transfer.  So:
        // a quarter of the first batch (enough, over all waves, to keep HBM busy), then wait for x (loads
        // return in order: "at most these outstanding" means x has landed), publish it, then the rest.
        constexpr int U0 = U / 4;
#pragma unroll
        for (int u = 0; u < U0; u++) MMX_REQUEST(0, u);
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("s_waitcnt vmcnt(%0)\n\ts_waitcnt lgkmcnt(0)\n\ts_barrier" : : "n"(U0 * NP) : "memory");
        __builtin_amdgcn_sched_barrier(0);
        SKINNY_STAMP(2);
#pragma unroll
        for (int u = U0; u < U; u++) MMX_REQUEST(0, u);
    }
    if constexpr (ONE) {  // every offset of this path is a compile-time constant
#pragma unroll
        for (int u = 0; u < U; u++) MMX_MULTIPLY(0, u);
    } else {
        for (int bt = 0; bt + 1 < nbatch; bt++) {
#pragma unroll
            for (int u = 0; u < U; u++) {
                MMX_MULTIPLY(bt, u);
                MMX_REQUEST(bt + 1, u);
            }
        }
#pragma unroll
        for (int u = 0; u < U; u++) MMX_MULTIPLY(nbatch - 1, u);
    }
#undef MMX_REQUEST
#undef MMX_MULTIPLY

    SKINNY_STAMP(3);
    __syncthreads();  // every wave has read its last x: the buffer becomes the reduction scratch
    SKINNY_STAMP(4);
    if constexpr (VALU) {
        // lane (column l32, k half g32): add the other half's sum, then put the column's value where the
        // matrix-core form would hold it (output row 0 of a 32x32 block), so that the post-op below is shared
        float sum = (vacc[0] + vacc[1]) + (vacc[2] + vacc[3]);
        sum += __shfl_xor(sum, 32);
        if (g32 == 0) red[wave][0][4 * (l32 >> 3) + (l32 & 3)][32 * ((l32 >> 2) & 1)] = sum;
    } else {
#pragma unroll
        for (int p = 0; p < NP; p++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                if constexpr (I8A) reinterpret_cast<int*>(&red[wave][p][v][lane])[0] = acc[p][v];  // the sums travel as bits
                else red[wave][p][v][lane] = W4 ? acc[p][v] * 16.0f : acc[p][v];  // int4 operands were q / 16
            }
    }
    __syncthreads();
    skinny_finish<NP, I8A>(s, red, panel_first, tid, fin);
    SKINNY_STAMP(5);
    SKINNY_STAMP(7);
}

// ---- resident-x variant: more rows than two workgroups per CU can hold a copy of ----------------------
// For 10-16 rows of a 4096-wide x the activations are 80-128 KiB: one copy fits in a CU's LDS, two do not.  So there
// is one workgroup per CU, x goes to LDS once, and the workgroup walks its one or two panels (blockIdx.x and
// blockIdx.x + gridDim.x) with the weight stream running across the panel boundary: right after a fragment has been
// multiplied the one D places further on is requested, of this panel or the next, so D KiB per wave are in flight
// until the last panel ends.  (The chunked kernel re-stages x per workgroup, 44 MB for 344 panels, behind a barrier
// per chunk with 24 KiB of weights in flight per workgroup.)
// A wave multiplies the same share of K in every panel, so it needs only that share of every row of x: each wave
// fetches its own slice (global_load_lds, no registers) into its own LDS region and waits for nothing but its own
// loads -- no barrier before the first multiply.  A region holds [M rows][SB + 16 bytes], SB = the slice of a row;
// the 16 bytes of padding make the row pitch an odd number of 16-byte pieces, so the 16 rows x 16 bytes that one LDS
// cycle serves for an MFMA operand fall into different banks.  Lanes of rows >= M read row 0 (their outputs are
// never stored).  K is exactly 8 waves x U fragments (the launcher checks).
// Straight-line code for one or two panels: in a loop whose iterations hand loads on to the next one, the compiler's
// count of outstanding loads falls back to "wait for all of them" (a loop over panels took 14.7 us at M = 1 against
// 10.8 for the streaming kernel).  The requests are separated by scheduler barriers, which keeps them in the order
// written: left alone, the compiler reorders independent loads and then waits for the youngest.  (Loads issued and
// waited for by hand, asm loads and a vmcnt wait that hands the registers on, are not an option: the compiler copies or
// spills the destination registers between the load and the wait, before the data has arrived.)
// Per-column post-op operands go to LDS the same way (wave 0, global_load_lds_dword) at the start of a panel.
// Cross-wave reduction per panel through red[8 waves][16][2][MR] (MR = 16 or 32 rows), behind the regions.
template <bool W8, int U>  // U: fragments per panel and wave (K = 8 waves x U fragments)
__global__ __launch_bounds__(512) void skinny_resident_kernel(const SkinnyArgs s, int region, int red_off, int mr_log2) {
    // Fragments (KiB) a wave keeps in flight.  More is worse at K = 4096: a wave is held at a request until the CU accepts it
    // (4096 x 11008 int8 at M = 16: 13.0 us with 4, 13.1 with 8, 14.1 with 16; 3: 13.3, 2: 14.3; a deeper window for the
    // workgroups with two panels only: 6: 13.0, 8: 13.1, 12: 13.6).
    constexpr int D = U >= 32 ? 8 : 4;  // (a long K with one workgroup per CU: 8192 x 8192 at M = 1 15.1 -> 14.1 us with 8)
    constexpr int XB = W8 ? 64 : 32;    // bytes of a row of x that one fragment covers
    extern __shared__ __attribute__((aligned(1024))) char xs[];
    float* const red = reinterpret_cast<float*>(xs + red_off);
    const float* const oc = reinterpret_cast<const float*>(xs + red_off + (1024 << mr_log2));  // [3][64]

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, g32 = lane >> 5;
    const int row_bytes = s.K * 2;
    const int G = gridDim.x;
    const int panel0 = (s.n0 >> 5) + (int)blockIdx.x;
    const int panels = ((s.n1 + 31) >> 5) - (s.n0 >> 5);
    const int npan = (panels - (int)blockIdx.x + G - 1) / G;  // >= 1: the launcher keeps gridDim.x <= panels
    const Epilogue& ep = s.ep;
    const bool deq_oc = (ep.steps & MMX_PP_DEQUANT) && ep.deq_oc, bias_oc = (ep.steps & MMX_PP_BIAS) != 0,
               q_oc = (ep.steps & MMX_PP_QUANT) && ep.q_oc;

    constexpr int per_wave = U;  // the launcher checks: nfrag = 8 * U
    const int f_begin = wave * per_wave;
    const int SB = per_wave * XB;
    const int rowp = SB + 16;
    const uint32_t lds_base = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)xs);
    {   // this wave's slice of x -> its LDS region, 64 pieces of 16 bytes per instruction (piece = row-major index over
        // [M][SB / 16 + 1]; the padding piece and the pieces past the end re-read a neighbour)
        const uint32_t lds_w = lds_base + (uint32_t)(wave * region);
        const int cpr1 = SB / 16 + 1;
        const int npieces = s.M * cpr1;
        const int slice0 = f_begin * XB;
        int r = lane / cpr1, c = lane - r * cpr1;
        for (int i0 = 0; i0 < npieces; i0 += 64) {
            const int rr = r < s.M ? r : s.M - 1;
            int cb = slice0 + (c < cpr1 - 1 ? c : cpr1 - 2) * 16;
            cb = cb < row_bytes - 16 ? cb : row_bytes - 16;
            const char* src = s.x + (int64_t)rr * s.ldx + cb;
            const uint32_t m0v = lds_w + (uint32_t)(i0 * 16);
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(m0v), "v"(src) : "memory");
            c += 64;
            while (c >= cpr1) {
                c -= cpr1;
                r++;
            }
        }
    }
    // per-column post-op operands of a panel -> oc (wave 0; lanes 32-63 repeat the 32 columns)
    auto stage_operands = [&](int panel) __attribute__((always_inline)) {
        if (wave != 0) return;
        int n = (panel << 5) + l32;
        n = n < s.n1 ? n : s.n1 - 1;
        const uint32_t dst = lds_base + (uint32_t)(red_off + (1024 << mr_log2));
        if (deq_oc) {
            const float* src = ep.deq_oc + n;
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off" : : "s"(dst), "v"(src) : "memory");
        }
        if (bias_oc) {
            const float* src = ep.bias + n;
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off" : : "s"(dst + 256), "v"(src) : "memory");
        }
        if (q_oc) {
            const float* src = ep.q_oc + n;
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off" : : "s"(dst + 512), "v"(src) : "memory");
        }
    };

    const int mrow = l32 < s.M ? l32 : 0;
    const char* const xrow = xs + wave * region + mrow * rowp + g32 * (XB / 2);
    const int64_t wstep = (int64_t)G * s.panel_stride;
    const char* wcur = s.Wp + (int64_t)panel0 * s.panel_stride + (int64_t)f_begin * 1024 + lane * 16;  // this wave's first fragment

    u32x4 w[D];
    f32x16 acc;
#pragma unroll
    for (int v = 0; v < 16; v++) acc[v] = 0.0f;

    // Fragment g of this wave's stream (g / U = panel of the workgroup, g % U = fragment of the wave's share) lives in
    // register set g % D.  (Nontemporal: the weights are read once.  The scheduler barrier keeps the requests in the
    // order written, which the compiler's waits then follow: left alone it reorders them and waits for the youngest.)
#define MMX_REQUEST(GG)                                                                     \
    do {                                                                                    \
        w[(GG) % D] = MMX_WLOAD(((GG) / U ? wcur + wstep : wcur) + ((GG) % U) * 1024);      \
        __builtin_amdgcn_sched_barrier(0);                                                  \
    } while (0)

    const int MR = 1 << mr_log2;
    // cross-wave sum of the panel's partial blocks, post-op, store.  (Barriers by hand: __syncthreads() would also
    // wait for the weight loads of the next panel.)
    auto finish = [&](int panel) __attribute__((always_inline)) {
        if (l32 < MR) {
#pragma unroll
            for (int v = 0; v < 16; v++) red[((((wave * 16 + v) * 2) + g32) << mr_log2) + l32] = acc[v];
        }
#pragma unroll
        for (int v = 0; v < 16; v++) acc[v] = 0.0f;
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" : : : "memory");
#pragma unroll
        for (int t = 0; t < 2; t++) {
            const int idx = tid + 512 * t;
            const int v = idx >> (mr_log2 + 1), g = (idx >> mr_log2) & 1, m = idx & (MR - 1);
            const int nloc = 8 * (v >> 2) + 4 * g + (v & 3);
            const int n = (panel << 5) + nloc;
            if (v >= 16 || m >= s.M || n >= s.n1) continue;
            float r = 0.0f;
#pragma unroll
            for (int w8 = 0; w8 < 8; w8++) r += red[((((w8 * 16 + v) * 2) + g) << mr_log2) + m];
            if (ep.steps & MMX_PP_DEQUANT) r = r * (deq_oc ? oc[nloc] : ep.deq);
            if (ep.steps & MMX_PP_BIAS) r = r + oc[64 + nloc];
            if (ep.steps & MMX_PP_GELU) r = gelu_erf_minimax(r);
            if (ep.steps & MMX_PP_QUANT) r = r * (q_oc ? oc[128 + nloc] : ep.q);
            store_out(ep, m, n, r);
        }
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" : : : "memory");  // the next panel overwrites scratch and operands
    };
    // One batch of U fragments per panel and at most two panels per workgroup (the launcher checks): straight-line
    // code, so the compiler counts the outstanding loads exactly.  Each multiply is followed by the request for the
    // fragment D places further on, of this panel or the next.
    auto run = [&](auto npan_c) __attribute__((always_inline)) {
        constexpr int TOTAL = decltype(npan_c)::value * U;
        // The first fragments behind x.  A wave is held at a request until the CU accepts it, so only U0 go out before
        // the wait for x ("at most these outstanding": this wave's slice of x has landed).
        constexpr int U0 = D < 4 ? D : 4;
        skinny_static_for<0, U0>([&](auto g_c) __attribute__((always_inline)) { MMX_REQUEST(decltype(g_c)::value); });
        asm volatile("s_waitcnt vmcnt(%0)" : : "n"(U0) : "memory");
        __builtin_amdgcn_sched_barrier(0);
        skinny_static_for<U0, D>([&](auto g_c) __attribute__((always_inline)) { MMX_REQUEST(decltype(g_c)::value); });
        skinny_static_for<0, TOTAL>([&](auto g_c) __attribute__((always_inline)) {
            constexpr int g = decltype(g_c)::value, u = g % U;
            if constexpr (u == 0) stage_operands(panel0 + (g / U) * G);
            const bf16x8 xa = *reinterpret_cast<const bf16x8*>(xrow + u * XB);
            if constexpr (W8) {
                const bf16x8 xc = *reinterpret_cast<const bf16x8*>(xrow + u * XB + 16);
                acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(s8x8_to_bf16(w[g % D].x, w[g % D].y), xa, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(s8x8_to_bf16(w[g % D].z, w[g % D].w), xc, acc, 0, 0, 0);
            } else {
                acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, w[g % D]), xa, acc, 0, 0, 0);
            }
            if constexpr (g + D < TOTAL) MMX_REQUEST(g + D);
            if constexpr (u == U - 1) finish(panel0 + (g / U) * G);
        });
    };
    if (npan > 1) run(std::integral_constant<int, 2>{});
    else run(std::integral_constant<int, 1>{});
#undef MMX_REQUEST
}

// ---- resident-x variant, two panels side by side -----------------------------------------------------------
// With more panels than CUs (344 on 256) the kernel above gives some workgroups a second panel to walk after the
// first, alone on the machine and at the rate one small window allows.  Here a workgroup has SIXTEEN waves: waves 0-7
// multiply panel blockIdx.x, waves 8-15 panel blockIdx.x + gridDim.x at the same time (where there is none they only
// keep the barriers company), wave w and wave w + 8 the same share of K against the same slice of x, which wave w fetched: one copy
// of x per CU, two weight streams, as two workgroups per CU would have if x fitted twice.  Same split of K over the
// waves and same order of the sums as the kernels above: the same bits.  One barrier publishes x (a wave of the
// second group reads what a wave of the first fetched), one ends the multiplies, after which the LDS of x becomes
// the reduction scratch of both groups.
template <bool W8, int U>  // U: fragments per panel and wave (K = 8 waves x U fragments)
__global__ __launch_bounds__(1024) void skinny_resident_pair_kernel(const SkinnyArgs s, int region, int oc_off, int mr_log2) {
    constexpr int D = U >= 32 ? 8 : 4;  // fragments (KiB) a wave keeps in flight, as above
    constexpr int XB = W8 ? 64 : 32;    // bytes of a row of x that one fragment covers
    extern __shared__ __attribute__((aligned(1024))) char xs[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int kw = wave & 7, grp = wave >> 3;  // share of K, panel of the pair
    const int l32 = lane & 31, g32 = lane >> 5;
    const int row_bytes = s.K * 2;
    const int G = gridDim.x;
    const int panels = ((s.n1 + 31) >> 5) - (s.n0 >> 5);
    // (a group without a panel only takes part in the barriers: every wave of the workgroup reaches each of them)
    const bool active = !(grp == 1 && (int)blockIdx.x + G >= panels);
    const int panel = (s.n0 >> 5) + (int)blockIdx.x + (active ? grp * G : 0);
    const Epilogue& ep = s.ep;
    const bool deq_oc = (ep.steps & MMX_PP_DEQUANT) && ep.deq_oc, bias_oc = (ep.steps & MMX_PP_BIAS) != 0,
               q_oc = (ep.steps & MMX_PP_QUANT) && ep.q_oc;
    const int MR = 1 << mr_log2;
    float* const red = reinterpret_cast<float*>(xs) + grp * (256 << mr_log2);           // [8 waves][16][2][MR], over x once it is spent
    const float* const oc = reinterpret_cast<const float*>(xs + oc_off) + grp * 192;     // [3][64] per group

    constexpr int per_wave = U;  // the launcher checks: nfrag = 8 * U
    const int f_begin = kw * per_wave;
    const int SB = per_wave * XB;
    const int rowp = SB + 16;
    const uint32_t lds_base = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)xs);
    if (grp == 0) {  // slice kw of x -> region kw (pieces of 16 bytes, row-major over [M][SB / 16 + 1]; see the kernel above)
        const uint32_t lds_w = lds_base + (uint32_t)(kw * region);
        const int cpr1 = SB / 16 + 1;
        const int npieces = s.M * cpr1;
        const int slice0 = f_begin * XB;
        int r = lane / cpr1, c = lane - r * cpr1;
        for (int i0 = 0; i0 < npieces; i0 += 64) {
            const int rr = r < s.M ? r : s.M - 1;
            int cb = slice0 + (c < cpr1 - 1 ? c : cpr1 - 2) * 16;
            cb = cb < row_bytes - 16 ? cb : row_bytes - 16;
            const char* src = s.x + (int64_t)rr * s.ldx + cb;
            const uint32_t m0v = lds_w + (uint32_t)(i0 * 16);
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(m0v), "v"(src) : "memory");
            c += 64;
            while (c >= cpr1) {
                c -= cpr1;
                r++;
            }
        }
    }
    if (kw == 0 && active) {  // the group's per-column post-op operands -> oc (lanes 32-63 repeat the 32 columns)
        int n = (panel << 5) + l32;
        n = n < s.n1 ? n : s.n1 - 1;
        const uint32_t dst = lds_base + (uint32_t)(oc_off + grp * 768);
        if (deq_oc) {
            const float* src = ep.deq_oc + n;
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off" : : "s"(dst), "v"(src) : "memory");
        }
        if (bias_oc) {
            const float* src = ep.bias + n;
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off" : : "s"(dst + 256), "v"(src) : "memory");
        }
        if (q_oc) {
            const float* src = ep.q_oc + n;
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off" : : "s"(dst + 512), "v"(src) : "memory");
        }
    }

    const int mrow = l32 < s.M ? l32 : 0;
    const char* const xrow = xs + kw * region + mrow * rowp + g32 * (XB / 2);
    const char* const wcur = s.Wp + (int64_t)panel * s.panel_stride + (int64_t)f_begin * 1024 + lane * 16;

    u32x4 w[D];
    f32x16 acc;
#pragma unroll
    for (int v = 0; v < 16; v++) acc[v] = 0.0f;

    // the first fragments behind x; "at most these outstanding" = this wave's loads of x and operands have landed;
    // the barrier then publishes every slice to both groups
    constexpr int U0 = D < 4 ? D : 4;
    if (active) {
#pragma unroll
        for (int g = 0; g < U0; g++) {
            w[g % D] = MMX_WLOAD(wcur + g * 1024);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" : : "n"(U0) : "memory");
    __builtin_amdgcn_sched_barrier(0);
    if (active) {
#pragma unroll
        for (int g = U0; g < D; g++) {
            w[g % D] = MMX_WLOAD(wcur + g * 1024);
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int g = 0; g < U; g++) {
            const bf16x8 xa = *reinterpret_cast<const bf16x8*>(xrow + g * XB);
            if constexpr (W8) {
                const bf16x8 xc = *reinterpret_cast<const bf16x8*>(xrow + g * XB + 16);
                acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(s8x8_to_bf16(w[g % D].x, w[g % D].y), xa, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(s8x8_to_bf16(w[g % D].z, w[g % D].w), xc, acc, 0, 0, 0);
            } else {
                acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, w[g % D]), xa, acc, 0, 0, 0);
            }
            if (g + D < U) {
                w[g % D] = MMX_WLOAD(wcur + (g + D < U ? g + D : 0) * 1024);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }
    // every wave has read its last x: the regions become the reduction scratch
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" : : : "memory");
    if (l32 < MR && active) {
#pragma unroll
        for (int v = 0; v < 16; v++) red[((((kw * 16 + v) * 2) + g32) << mr_log2) + l32] = acc[v];
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" : : : "memory");
    if (!active) return;
    const int gtid = tid & 511;  // thread of the group
#pragma unroll
    for (int t = 0; t < 2; t++) {
        const int idx = gtid + 512 * t;
        const int v = idx >> (mr_log2 + 1), g = (idx >> mr_log2) & 1, m = idx & (MR - 1);
        const int nloc = 8 * (v >> 2) + 4 * g + (v & 3);
        const int n = (panel << 5) + nloc;
        if (v >= 16 || m >= s.M || n >= s.n1) continue;
        float r = 0.0f;
#pragma unroll
        for (int w8 = 0; w8 < 8; w8++) r += red[((((w8 * 16 + v) * 2) + g) << mr_log2) + m];
        if (ep.steps & MMX_PP_DEQUANT) r = r * (deq_oc ? oc[nloc] : ep.deq);
        if (ep.steps & MMX_PP_BIAS) r = r + oc[64 + nloc];
        if (ep.steps & MMX_PP_GELU) r = gelu_erf_minimax(r);
        if (ep.steps & MMX_PP_QUANT) r = r * (q_oc ? oc[128 + nloc] : ep.q);
        store_out(ep, m, n, r);
    }
}

// Half-panel variant of the streaming kernel for 1-4 rows of x.  A list of 32-column panels that is only 1-2
// per CU long leaves some CUs with twice the work of others (or idle), and how fast one CU can pull
// weights in is what bounds this kernel.  Here a workgroup (four waves) multiplies HALF a panel
// (16 columns, blockIdx.x = 2 * panel group + half): twice as many, half as large units, all resident at once.
// A load covers the half-panel's part of TWO consecutive fragments (lanes 0-15/32-47: fragment 2u, lanes
// 16-31/48-63: fragment 2u+1), so every lane still fetches its own 16 bytes.  As an MFMA operand that is 16
// columns x two different k-ranges, so each load is multiplied twice, once with the x of either fragment,
// into two accumulators: rows 0-15 of the first and rows 16-31 of the second are the two partial sums of
// the 16 columns (the other rows are never looked at).  K * sizeof(T) is a multiple of 128 on this path,
// so a panel has an even number of fragments.
template <bool W8, int NP, bool ONE, int U>  // U: loads per panel per wave in flight at once (1 KiB each)
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4, 4))) void skinny_half_kernel(const SkinnyArgs s, int zero_off) {
    constexpr int NW = 4;
    __shared__ float red[NW][NP][16][64];
    extern __shared__ __attribute__((aligned(1024))) char xs[];  // [M][K] bf16, then at zero_off a row of zeros

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, g32 = lane >> 5;
    const int half = blockIdx.x & 1;
    const int panel_first = (s.n0 >> 5) + (int)(blockIdx.x >> 1) * NP;
    const int panel_end = (s.n1 + 31) >> 5;
    const int row_bytes = s.K * 2;
    const int real_bytes = s.M * row_bytes;
    const Epilogue& ep = s.ep;

    {   // x -> LDS as in skinny_stream_kernel
        const uint32_t lds_base = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)xs);
        for (int off = wave * 1024; off < real_bytes; off += NW * 1024) {
            int bo = off + lane * 16;
            bo = bo < real_bytes ? bo : real_bytes - 16;
            const int m = bo / row_bytes;
            const char* src = s.x + (int64_t)m * s.ldx + (bo - m * row_bytes);
            const uint32_t m0v = lds_base + off;
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(m0v), "v"(src) : "memory");
        }
        for (int c = tid * 16; c < row_bytes; c += NW * 64 * 16) *reinterpret_cast<u32x4*>(xs + zero_off + c) = u32x4{0u, 0u, 0u, 0u};
    }
    // per-column operands of the post-op: thread -> (accumulator register v < 8, lane) -> column of the half-panel
    float o_deq[2][NP], o_bias[2][NP], o_q[2][NP];
#pragma unroll
    for (int t = 0; t < 2; t++) {
        const int v = (tid + 256 * t) >> 6;
        const int nloc = 16 * half + 8 * (v >> 2) + 4 * g32 + (v & 3);
#pragma unroll
        for (int p = 0; p < NP; p++) {
            const int n = ((panel_first + p) << 5) + nloc;
            const bool ok = l32 < s.M && n < s.n1;
            o_deq[t][p] = ep.deq;
            o_bias[t][p] = 0.0f;
            o_q[t][p] = ep.q;
            if (ok && (ep.steps & MMX_PP_DEQUANT) && ep.deq_oc) o_deq[t][p] = ep.deq_oc[n];
            if (ok && (ep.steps & MMX_PP_BIAS)) o_bias[t][p] = ep.bias[n];
            if (ok && (ep.steps & MMX_PP_QUANT) && ep.q_oc) o_q[t][p] = ep.q_oc[n];
        }
    }
    __builtin_amdgcn_sched_barrier(0);

    f32x16 acc[NP][2];
#pragma unroll
    for (int p = 0; p < NP; p++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[p][0][v] = acc[p][1][v] = 0.0f;

    // wave w multiplies the fragment pairs [w*per_wave, (w+1)*per_wave); indices past the end are clamped
    // for the load and paired with the zero row of x
    const int npairs = s.nfrag >> 1;
    const int per_wave = (npairs + NW - 1) / NW;
    const int u_begin = wave * per_wave;
    const int u_last = npairs - 1;
    const char* wbase[NP];
#pragma unroll
    for (int p = 0; p < NP; p++) {
        int panel = panel_first + p;
        panel = (panel < panel_end && panel < s.npanels) ? panel : s.npanels - 1;  // columns past n1 are never stored
        wbase[p] = s.Wp + (int64_t)panel * s.panel_stride + (l32 >> 4) * 1024 + (g32 * 32 + 16 * half + (l32 & 15)) * 16;
    }
    const char* zrow = xs + zero_off;
    const char* xrow = l32 < s.M ? xs + l32 * row_bytes : zrow;
    const int nbatch = (per_wave + U - 1) / U;  // same for every wave
    u32x4 w[NP][U];
#define MMX_REQUEST(BT, UU)                                                                                     \
    do {                                                                                                        \
        int u_ = u_begin + (BT) * U + (UU);                                                                     \
        u_ = u_ < u_last ? u_ : u_last;                                                                         \
        _Pragma("unroll") for (int p = 0; p < NP; p++)                                                          \
            w[p][UU] = MMX_WLOAD(wbase[p] + (int64_t)u_ * 2048);                                             \
    } while (0)
#define MMX_MULTIPLY(BT, UU)                                                                                    \
    do {                                                                                                        \
        const int u_ = u_begin + (BT) * U + (UU);                                                               \
        const bool valid_ = (u_ - u_begin) < per_wave && u_ <= u_last; /* scalar */                             \
        const int uc_ = u_ < u_last ? u_ : u_last;                                                              \
        const char* xr_ = valid_ ? xrow : zrow;                                                                 \
        if constexpr (W8) {                                                                                     \
            const bf16x8 xa0_ = *reinterpret_cast<const bf16x8*>(xr_ + (64 * uc_ + 16 * g32) * 2);              \
            const bf16x8 xa1_ = *reinterpret_cast<const bf16x8*>(xr_ + (64 * uc_ + 16 * g32 + 8) * 2);          \
            const bf16x8 xb0_ = *reinterpret_cast<const bf16x8*>(xr_ + (64 * uc_ + 32 + 16 * g32) * 2);         \
            const bf16x8 xb1_ = *reinterpret_cast<const bf16x8*>(xr_ + (64 * uc_ + 32 + 16 * g32 + 8) * 2);     \
            _Pragma("unroll") for (int p = 0; p < NP; p++) {                                                    \
                const bf16x8 lo_ = s8x8_to_bf16(w[p][UU].x, w[p][UU].y), hi_ = s8x8_to_bf16(w[p][UU].z, w[p][UU].w); \
                acc[p][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(lo_, xa0_, acc[p][0], 0, 0, 0);             \
                acc[p][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(hi_, xa1_, acc[p][0], 0, 0, 0);             \
                acc[p][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(lo_, xb0_, acc[p][1], 0, 0, 0);             \
                acc[p][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(hi_, xb1_, acc[p][1], 0, 0, 0);             \
            }                                                                                                   \
        } else {                                                                                                \
            const bf16x8 xa_ = *reinterpret_cast<const bf16x8*>(xr_ + (32 * uc_ + 8 * g32) * 2);                \
            const bf16x8 xb_ = *reinterpret_cast<const bf16x8*>(xr_ + (32 * uc_ + 16 + 8 * g32) * 2);           \
            _Pragma("unroll") for (int p = 0; p < NP; p++) {                                                    \
                acc[p][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, w[p][UU]), xa_, acc[p][0], 0, 0, 0); \
                acc[p][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, w[p][UU]), xb_, acc[p][1], 0, 0, 0); \
            }                                                                                                   \
        }                                                                                                       \
    } while (0)
    {
        // as in skinny_stream_kernel: a quarter of the first batch, then wait for x and publish it, then the rest
        constexpr int U0 = U / 4;
#pragma unroll
        for (int u = 0; u < U0; u++) MMX_REQUEST(0, u);
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("s_waitcnt vmcnt(%0)\n\ts_waitcnt lgkmcnt(0)\n\ts_barrier" : : "n"(U0 * NP) : "memory");
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = U0; u < U; u++) MMX_REQUEST(0, u);
    }
    if constexpr (ONE) {
#pragma unroll
        for (int u = 0; u < U; u++) MMX_MULTIPLY(0, u);
    } else {
        for (int bt = 0; bt + 1 < nbatch; bt++) {
#pragma unroll
            for (int u = 0; u < U; u++) {
                MMX_MULTIPLY(bt, u);
                MMX_REQUEST(bt + 1, u);
            }
        }
#pragma unroll
        for (int u = 0; u < U; u++) MMX_MULTIPLY(nbatch - 1, u);
    }
#undef MMX_REQUEST
#undef MMX_MULTIPLY

    // accumulator register v of a lane is row 8 (v / 4) + 4 g32 + v % 4: rows 0-15 are v < 8
#pragma unroll
    for (int p = 0; p < NP; p++)
#pragma unroll
        for (int v = 0; v < 16; v++) red[wave][p][v][lane] = v < 8 ? acc[p][0][v] : acc[p][1][v];
    __syncthreads();

#pragma unroll
    for (int t = 0; t < 2; t++) {
        const int v = (tid + 256 * t) >> 6;
        const int m = l32;
        if (m >= s.M) continue;
        const int nloc = 16 * half + 8 * (v >> 2) + 4 * g32 + (v & 3);
        float sum[NP];
#pragma unroll
        for (int p = 0; p < NP; p++) {
            float a = 0.0f;
#pragma unroll
            for (int wv = 0; wv < NW; wv++) a += red[wv][p][v][lane] + red[wv][p][v + 8][lane];
            sum[p] = a;
        }
        if (ep.steps & MMX_PP_SILU_GATE) {
            if constexpr (NP == 2) {
                const int n = ((panel_first >> 1) << 5) + nloc;  // output column (half width)
                float gate = sum[0], up = sum[1];
                if (ep.steps & MMX_PP_DEQUANT) {
                    gate = gate * o_deq[t][0];
                    up = up * o_deq[t][1];
                }
                if (n < (s.n1 >> 1)) store_out(ep, m, n, silu(gate) * up);
            }
        } else {
#pragma unroll
            for (int p = 0; p < NP; p++) {
                const int n = ((panel_first + p) << 5) + nloc;
                if (n >= s.n1) continue;
                float r = sum[p];
                if (ep.steps & MMX_PP_DEQUANT) r = r * o_deq[t][p];
                if (ep.steps & MMX_PP_BIAS) r = r + o_bias[t][p];
                if (ep.steps & MMX_PP_GELU) r = gelu_erf_minimax(r);
                if (ep.steps & MMX_PP_QUANT) r = r * o_q[t][p];
                store_out(ep, m, n, r);
            }
        }
    }
}

int decode_halves();
int decode_valu();
int decode_resident();
int decode_pair();

// int8 x int8 at M <= 32 can use the decode kernels if x is 16-byte aligned and K fills whole 128-byte groups of
// the packed weights: the streaming form if x fits in LDS, else the chunked one, which walks K in chunks of 256
// dynamic LDS of skinny_stream_kernel: x + the zero row, reused afterwards as the reduction scratch (32 KiB per panel)
// Workspace of a K split: arrival counters first (one per workgroup column, zero between launches), the slices' sums after
// them - the layout the tile kernels use, so one workspace serves both.
constexpr int SPLIT_MAX_PANELS = 4096;
constexpr size_t SPLIT_COUNTER_BYTES = (size_t)SPLIT_MAX_PANELS * 4;

// Slices of K for the chunked kernel: with a panel for at most every second CU the workgroups of a panel walk K in 2-4
// slices (as many as give every CU one workgroup; more - 6, 8 - measured slower), none empty and each at least four
// chunks long, and the last to arrive adds them up (int8 weights, weights rotated over 540 MB: 11008 x 4096 at
// M = 16 / 32 20.4 / 25.1 -> 14.5 / 17.3 us, 8192 x 1024 15.5 / 19.0 -> 9.1 / 10.5; bf16 weights: 11008 x 4096 at
// M = 16 / 32 26.7 / 34.7 -> 19.4 / 22.4, 8192 x 1024 19.7 / 25.4 -> 10.3 / 11.5).  With a panel for up to two thirds of the
// CUs, three slices of at least ten chunks fill the two workgroups a CU holds (11008 x 5120, int8 M = 16 / 32 20.9 / 25.8
// -> 17.1 / 21.7, bf16 27.6 / 35.7 -> 24.2 / 26.7); shorter slices and more panels measured level or behind.
static int chunk_slices(bool w8, int M, int nfrag, int panels, size_t ws_bytes) {
    if (panels <= 0 || panels * 3 > 2 * num_cus() || panels > SPLIT_MAX_PANELS) return 1;
    const int fc = (!w8 && M <= 16) ? 16 : 8;  // fragments per chunk of the kernels launched for these shapes
    const int nchunk = (nfrag + fc - 1) / fc;
    const bool wide = panels * 2 > num_cus();
    int S = wide ? 3 : (num_cus() / panels < 4 ? num_cus() / panels : 4);
    const int shortest = wide ? 10 : 4;
    while (S > 1 && ((nchunk + S - 1) / S < shortest || (S - 1) * ((nchunk + S - 1) / S) >= nchunk ||
                     SPLIT_COUNTER_BYTES + (size_t)panels * S * 4096 > ws_bytes))
        S = wide ? 1 : S - 1;
    return S;
}

// Bytes of workspace a decode launch of this shape can use (0: it takes no K split)
size_t skinny_workspace_bytes(int wk, int M, int K, int n0, int n1) {
    const int nfrag = wk == 2 ? (K + 255) / 256 * 4 : (K * ((wk == 1 || wk == 3) ? 1 : 2) + 127) / 128 * 128 / 32;
    const int panels = ((n1 + 31) >> 5) - (n0 >> 5);
    const int S = chunk_slices(wk != 0, M, nfrag, panels, ~(size_t)0);
    return S > 1 ? SPLIT_COUNTER_BYTES + (size_t)panels * S * 4096 : 0;
}

static inline int stream_lds_bytes(int xbytes, int np) { return xbytes > 32768 * np ? xbytes : 32768 * np; }

bool skinny_i8_eligible(const void* x, int64_t ldx, int M, int K) {
    if (M > 32 || K > (1 << 24)) return false;
    const int zoff = (M * K + 1023) & ~1023;
    return K % 128 == 0 && (zoff + K <= 46 * 1024 || K % 256 == 0) && ((reinterpret_cast<uintptr_t>(x) & 15) == 0) &&
           ((ldx & 15) == 0);
}

// The rolling-window form of the half-panel kernel re-requests its loads in batches of U; the last batch is filled up
// with repeats of the last load.  The repeats cost as much as they are a share of the loads (bf16 2560 x 10240 at
// M = 1, 20 loads per wave: 14.7 us with batches of 16, 10.8 with 10; 11008 x 4096, 86 loads: 18.3 with 16, 16.8 with 8,
// 17.4 with 10), so the batch with the fewest repeats is used; at equal repeats the larger one (4096 x 11008, 32 loads:
// 16.8 / 17.7 us at M = 1 / 4 with 16, 16.7 / 18.3 with 8), over int8 weights the smaller (11008 x 4096: 11.2 with 8, 11.8
// with 12).  Gate/up pairs: batches of 4 per panel (3: +3 %, 2: +5 %, 6: +38 %).
typedef void (*HalfKernel)(const SkinnyArgs, int);
template <bool W8, int NP>
static HalfKernel half_window_kernel(int nfrag) {
    if constexpr (NP == 2) {
        return skinny_half_kernel<W8, 2, false, 4>;
    } else {
        const int n = ((nfrag >> 1) + 3) / 4;  // loads per wave
        auto repeats = [n](int u) { return (n + u - 1) / u * u - n; };
        if constexpr (W8) {
            return repeats(12) < repeats(8) ? skinny_half_kernel<true, 1, false, 12> : skinny_half_kernel<true, 1, false, 8>;
        } else {
            int best = 16;
            for (int u : {10, 8, 6})
                if (repeats(u) < repeats(best)) best = u;
            return best == 16 ? skinny_half_kernel<false, 1, false, 16>
                              : (best == 10 ? skinny_half_kernel<false, 1, false, 10>
                                            : (best == 8 ? skinny_half_kernel<false, 1, false, 8> : skinny_half_kernel<false, 1, false, 6>));
        }
    }
}

// The streaming kernel for single panels and a wave's share of per_wave fragments.  Up to 16: one batch, of the smallest
// register set that holds the share (a share of 10 in a set of 16 is 6 repeated loads and 6 multiplies by zero in 16: int8
// 2560 x 10240 at M = 1 10.0 us against 7.6 for its bytes).  Beyond: the rolling window in batches of 16, 10 or 8,
// whichever repeats the fewest loads, the larger at equal repeats (a share of 20 fragments in batches of 16 is 12 repeats
// in 32 loads: int8 5120 x 13824 at M = 1 20.0 us, 14.3 in batches of 10; bf16 2560 x 10752 16.2 -> 12.0).
// *index: the kernel's place in a list of STREAM_KERNELS per weight type (for per-kernel set-up).
typedef void (*StreamKernel)(const SkinnyArgs, int);
constexpr int STREAM_KERNELS = 9;
template <int WK>
static StreamKernel stream_kernel_for(int per_wave, int* index) {
    static const StreamKernel list[STREAM_KERNELS] = {
        skinny_stream_kernel<WK, 1, true, 4>,  skinny_stream_kernel<WK, 1, true, 6>,  skinny_stream_kernel<WK, 1, true, 8>,
        skinny_stream_kernel<WK, 1, true, 10>, skinny_stream_kernel<WK, 1, true, 12>, skinny_stream_kernel<WK, 1, true>,
        skinny_stream_kernel<WK, 1, false>,    skinny_stream_kernel<WK, 1, false, 10>, skinny_stream_kernel<WK, 1, false, 8>};
    int i;
    if (per_wave <= 16) {
        i = per_wave <= 4 ? 0 : (per_wave <= 6 ? 1 : (per_wave <= 8 ? 2 : (per_wave <= 10 ? 3 : (per_wave <= 12 ? 4 : 5))));
    } else {
        auto repeats = [per_wave](int u) { return (per_wave + u - 1) / u * u - per_wave; };
        i = 6;
        if (repeats(10) < repeats(16)) i = 7;
        if (repeats(8) < repeats(i == 7 ? 10 : 16)) i = 8;
    }
    *index = i;
    return list[i];
}

// wk: weights are bf16 (0), int8 (1) or int4 (2); 3: int8 weights and int8 activations
int launch_skinny(int wk, const void* x, int64_t ldx, const void* Wp, int M, int K, int N, int n0, int n1,
                  const Epilogue& ep, hipStream_t st, const SplitRequest* rq) {
    const bool w8 = wk == 1;
    // the byte counts below are 32-bit: M <= 32 rows of at most 2^24 elements
    if (M > 32 || K > (1 << 24)) return set_error(MMX_E_UNSUPPORTED, "decode kernels take M <= 32 and K <= 2^24 (got M = %d, K = %d)", M, K);
    SkinnyArgs s;
    s.x = static_cast<const char*>(x);
    s.ldx = ldx;
    s.Wp = static_cast<const char*>(Wp);
    s.M = M;
    s.K = K;
    const int kbytes_pad = ((K * ((wk == 1 || wk == 3) ? 1 : 2)) + 127) / 128 * 128;
    s.nfrag = wk == 2 ? (K + 255) / 256 * 4 : kbytes_pad / 32;  // 32 bytes of K per column per fragment
    s.panel_stride = (int64_t)s.nfrag * 1024;
    s.npanels = (N + 31) / 32;
    s.n0 = n0;
    s.n1 = n1;
    s.x_vec_ok = ((reinterpret_cast<uintptr_t>(x) & 15) == 0) && ((ldx & 15) == 0);
    s.ep = ep;
    s.ws_part = nullptr;
    s.ws_cnt = nullptr;
    s.kslices = 1;
    s.stamps = nullptr;
    const int panels = ((n1 + 31) >> 5) - (n0 >> 5);
#ifdef MMX_STAMPS
    if (rq && rq->ws && rq->ws_bytes >= SPLIT_COUNTER_BYTES + ((size_t)96 << 20) + (size_t)64 * 2 * panels)
        s.stamps = reinterpret_cast<uint64_t*>(rq->ws + SPLIT_COUNTER_BYTES + ((size_t)96 << 20));
#endif
    const bool pairs = (ep.steps & MMX_PP_SILU_GATE) != 0;
    if (wk == 3) {
        // int8 activations x int8 weights (int32 sums): the caller has checked skinny_i8_eligible and uses the tile
        // kernel otherwise
        const int zoff = (M * K + 1023) & ~1023;
        if (zoff + K > 46 * 1024) {  // x does not fit in LDS: through LDS chunk by chunk (32 rows x 256 bytes per buffer)
            // (few panels, a workspace at hand: K in slices as for bf16 activations; int32 sums, the same bits in any order)
            const int ksl3 = (rq && rq->ws && rq->k_splits == 0) ? chunk_slices(true, M, s.nfrag, panels, rq->ws_bytes) : 1;
            if (ksl3 > 1) {
                s.ws_cnt = reinterpret_cast<uint32_t*>(rq->ws);
                s.ws_part = rq->ws + SPLIT_COUNTER_BYTES;
                s.kslices = ksl3;
                char name_[40];
                snprintf(name_, sizeof name_, "skinny_chunk_i8_ksplit%d", ksl3);
                note_kernel(name_);
                hipLaunchKernelGGL((skinny_chunk_kernel<3, 1, 1, 1, 6>), dim3(panels, ksl3), dim3(512), 8 * 1 * 16 * 64 * 4, st, s);
                return check_hip(hipGetLastError(), "skinny_chunk_kernel launch");
            }
            note_kernel("skinny_chunk_i8");
            hipLaunchKernelGGL((skinny_chunk_kernel<3, 1, 1, 1>), dim3(panels), dim3(512), 8 * 1 * 16 * 64 * 4, st, s);
            return check_hip(hipGetLastError(), "skinny_chunk_kernel launch");
        }
        note_kernel("skinny_stream_i8");
        int unused;
        hipLaunchKernelGGL(stream_kernel_for<3>((s.nfrag + 7) / 8, &unused), dim3(panels), dim3(512), stream_lds_bytes(zoff + K, 1), st, s, zoff);
        return check_hip(hipGetLastError(), "skinny_stream_kernel launch");
    }
    if (wk == 2) {
        // int4 weights: the streaming kernel if x fits in LDS and K fills whole fragments, else the general one
        if (pairs && (panels & 1)) return set_error(MMX_E_INVALID, "SILU_GATE needs an even number of 32-column panels");
        const int zoff = (M * K * 2 + 1023) & ~1023;
        const int xb = zoff + K * 2;
        if (s.nfrag * 64 == K && xb <= 46 * 1024 && s.x_vec_ok) {
            note_kernel(pairs ? "skinny_stream_w4_gateup" : "skinny_stream_w4");
            if (pairs) {  // gate and up panels side by side: four fragments of each in flight per wave
                if ((s.nfrag + 7) / 8 <= 4)
                    hipLaunchKernelGGL((skinny_stream_kernel<2, 2, true>), dim3(panels / 2), dim3(512), stream_lds_bytes(xb, 2), st, s, zoff);
                else
                    hipLaunchKernelGGL((skinny_stream_kernel<2, 2, false>), dim3(panels / 2), dim3(512), stream_lds_bytes(xb, 2), st, s, zoff);
            } else if ((s.nfrag + 7) / 8 <= 4)  // (register sets sized to the share of K, as for the other weight types)
                hipLaunchKernelGGL((skinny_stream_kernel<2, 1, true, 4>), dim3(panels), dim3(512), stream_lds_bytes(xb, 1), st, s, zoff);
            else if ((s.nfrag + 7) / 8 <= 6)
                hipLaunchKernelGGL((skinny_stream_kernel<2, 1, true, 6>), dim3(panels), dim3(512), stream_lds_bytes(xb, 1), st, s, zoff);
            else if ((s.nfrag + 7) / 8 <= 8)
                hipLaunchKernelGGL((skinny_stream_kernel<2, 1, true>), dim3(panels), dim3(512), stream_lds_bytes(xb, 1), st, s, zoff);
            else
                hipLaunchKernelGGL((skinny_stream_kernel<2, 1, false>), dim3(panels), dim3(512), stream_lds_bytes(xb, 1), st, s, zoff);
            return check_hip(hipGetLastError(), "skinny_stream_kernel launch");
        }
        if (pairs) {  // x too large for LDS or a ragged K: the general kernel
            note_kernel("skinny_w4_gateup");
            hipLaunchKernelGGL((skinny_kernel<2, 2>), dim3(panels / 2), dim3(512), 0, st, s);
            return check_hip(hipGetLastError(), "skinny_kernel launch");
        }
        if (s.nfrag * 64 == K && s.x_vec_ok) {
            // x too large for LDS: through LDS chunk by chunk (two buffers of 16 or 32 rows x 1 KiB)
            const int ksl4 = (rq && rq->ws && rq->k_splits == 0) ? chunk_slices(true, M, s.nfrag, panels, rq->ws_bytes) : 1;
            if (ksl4 > 1) {  // few panels, a workspace at hand: K in slices as for the other weight types
                s.ws_cnt = reinterpret_cast<uint32_t*>(rq->ws);
                s.ws_part = rq->ws + SPLIT_COUNTER_BYTES;
                s.kslices = ksl4;
                char name_[40];
                snprintf(name_, sizeof name_, "skinny_chunk_w4_ksplit%d", ksl4);
                note_kernel(name_);
                if (M <= 16) hipLaunchKernelGGL((skinny_chunk_kernel<2, 1, 1, 2, 3>), dim3(panels, ksl4), dim3(512), 2 * 8 * 2 * 1024, st, s);
                else hipLaunchKernelGGL((skinny_chunk_kernel<2, 1, 1, 4, 2>), dim3(panels, ksl4), dim3(512), 2 * 8 * 4 * 1024, st, s);
                return check_hip(hipGetLastError(), "skinny_chunk_kernel launch");
            }
            note_kernel("skinny_chunk_w4");
            if (M <= 16) hipLaunchKernelGGL((skinny_chunk_kernel<2, 1, 1, 2>), dim3(panels), dim3(512), 2 * 8 * 2 * 1024, st, s);
            else hipLaunchKernelGGL((skinny_chunk_kernel<2, 1, 1, 4>), dim3(panels), dim3(512), 2 * 8 * 4 * 1024, st, s);
            return check_hip(hipGetLastError(), "skinny_chunk_kernel launch");
        }
        note_kernel("skinny_w4");
        hipLaunchKernelGGL((skinny_kernel<2, 1>), dim3(panels), dim3(512), 0, st, s);
        return check_hip(hipGetLastError(), "skinny_kernel launch");
    }
    const int kpad = kbytes_pad / (w8 ? 1 : 2);  // elements of K the packed weights cover
    const int zero_off = (M * K * 2 + 1023) & ~1023;
    const int xbytes = zero_off + K * 2;  // x, a gap up to the next KiB, one row of zeros
    if (kpad == K && s.x_vec_ok && !w8 && !pairs && M >= 2 && M <= 4 && xbytes > 46 * 1024 && xbytes <= 128 * 1024 &&
        decode_halves() != 0 && panels <= num_cus() && (int64_t)s.nfrag * 512 >= 128 * 1024) {
        // A few rows of a long x (the MLP's down projection at M = 2-4: 66-110 KiB with the zero row) and at
        // most one half-panel per CU: the half-panel form with one workgroup per CU still has all of x in LDS.
        static std::atomic<uint64_t> attr_done[5];
        const HalfKernel kernels[5] = {skinny_half_kernel<false, 1, true, 16>, skinny_half_kernel<false, 1, false, 16>,
                                       skinny_half_kernel<false, 1, false, 10>, skinny_half_kernel<false, 1, false, 8>,
                                       skinny_half_kernel<false, 1, false, 6>};
        for (int i = 0; i < 5; i++) {
            const int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(kernels[i]), 128 * 1024, attr_done[i]);
            if (rc) return rc;
        }
        note_kernel("skinny_half_bf16");
        if (((s.nfrag >> 1) + 3) / 4 <= 16)
            hipLaunchKernelGGL((skinny_half_kernel<false, 1, true, 16>), dim3(2 * panels), dim3(256), xbytes, st, s, zero_off);
        else
            hipLaunchKernelGGL((half_window_kernel<false, 1>(s.nfrag)), dim3(2 * panels), dim3(256), xbytes, st, s, zero_off);
        return check_hip(hipGetLastError(), "skinny_half_kernel launch");
    }
    {
        // x fits in one CU's LDS once: one workgroup per CU keeps it there and walks its one or two panels.  Taken where the
        // streaming form cannot hold x twice per CU (4096 x 11008 int8 at M = 10 / 16: 12.3 / 13.1 us against 13.5 / 14.6 for
        // the chunked form; 8192 x 4096 at M = 6: 10.4 against 17.1; over bf16 weights only while no workgroup has a second
        // panel: 4096 x 4096 at M = 12 9.9 against 12.0, but 4096 x 11008 at M = 16 21.2 against 20.9), and over int8
        // weights wherever no workgroup has a second panel (4096 x 4096: M = 1 6.1 against 6.7 us, M = 4 6.4 against 8.0;
        // 8192 x 4096: M = 1 9.5 against 10.9); with two panels on some CUs and few rows the streaming form's two
        // workgroups per CU are ahead (11008 columns, M = 1: 10.8 against 11.4 us; so they are against this kernel with one
        // panel per workgroup and two workgroups per CU: 11.2 with 4 KiB per wave in flight, 10.8 with 2, and ahead only
        // when every CU holds two, 16384 columns: 13.3 against 13.9 us; not kept).
        // decode_resident(): -1 by that rule (and only while decode_valu and decode_halves are left alone), 0 never,
        // 1 wherever the shape allows.
        const int rforce = decode_resident();
        const int mr_log2 = M <= 16 ? 4 : 5;
        const int slice = (s.nfrag >> 3) * (w8 ? 64 : 32);                 // bytes of a row of x per wave
        const int region = (M * (slice + 16) + 1023) & ~1023;              // LDS per wave
        const int red_off = 8 * region;
        const int lds = red_off + (1024 << mr_log2) + 2048;   // regions, reduction scratch, post-op operands
        // K = 8 waves x U fragments for the U that exist: 16, 32 (K = 2048, 4096 of bf16 weights; 4096, 8192 of int8 weights) and,
        // for int8 weights, 20 and 43 (K = 5120, 11008)
        const bool k_ok = s.nfrag == 128 || s.nfrag == 256 || (w8 && (s.nfrag == 160 || s.nfrag == 344));
        const bool shape_ok = kpad == K && s.x_vec_ok && !pairs && k_ok && panels > 0 &&
                              panels <= 2 * num_cus() && lds <= 160 * 1024;
        const bool one_each = panels <= num_cus();
        // (two panels on some CUs: ahead of the chunked form while a good part of the CUs has one, 344 or 432 panels on 256
        // CUs; with two on every CU, 8192 x 16384 at M = 8, the chunked form's two workgroups per CU win, 24.5 against 26.0 us)
        const bool some_two = !one_each && panels * 4 <= 7 * num_cus();
        // Second panels over int8 weights are walked side by side by a second group of eight waves
        // (skinny_resident_pair_kernel: one copy of x, two weight streams; 4096 x 11008 at M = 12 / 16 12.5 / 13.0 -> 12.1 /
        // 12.5 us, 4096 x 13824 at M = 1 / 8 / 16 12.0 / 12.8 / 14.0 -> 11.8 / 12.3 / 13.2, 4096 x 16384 13.8 / 14.4 / 15.5 ->
        // 13.4 / 14.1 / 15.0).  Over bf16 weights the pair is behind the one-after-the-other form (4096 x 11008 at M = 1
        // 18.9 against 18.5 us, 4096 x 16384 27.1 against 23.8) and is not used.  With few rows and fewer than 1.5 panels
        // per CU the streaming form stays ahead (11008 columns, M = 1 / 4: 10.7 / 11.0 against 11.0 / 11.4).
        const int pair_red = 2 * (1024 << mr_log2);
        const int pair_oc_off = 8 * region > pair_red ? 8 * region : pair_red;
        const int pair_lds = pair_oc_off + 2 * 768;
        const bool pair_ok = w8 && !one_each && (s.nfrag == 128 || s.nfrag == 256) && decode_pair() != 0 && pair_lds <= 160 * 1024;
        const bool pair_rule = pair_ok && s.nfrag == 128 && decode_valu() == -1 && decode_halves() == -1 &&
                               (xbytes > 80 * 1024 || panels * 2 >= 3 * num_cus());
        const bool by_rule = (xbytes > 80 * 1024 && (one_each || (w8 && some_two))) ||
                             (w8 && one_each && decode_valu() == -1 && decode_halves() == -1) || pair_rule;
        if (shape_ok && rforce != 0 && (rforce == 1 || by_rule)) {
            typedef void (*ResidentKernel)(const SkinnyArgs, int, int, int);
            static std::atomic<uint64_t> attr_done[6];
            const ResidentKernel kerns[6] = {skinny_resident_kernel<false, 16>, skinny_resident_kernel<false, 32>,
                                             skinny_resident_kernel<true, 16>, skinny_resident_kernel<true, 32>,
                                             skinny_resident_kernel<true, 20>, skinny_resident_kernel<true, 43>};
            const int ki = !w8 ? (s.nfrag == 256 ? 1 : 0) : (s.nfrag == 128 ? 2 : (s.nfrag == 256 ? 3 : (s.nfrag == 160 ? 4 : 5)));
            const ResidentKernel kern = kerns[ki];
            const int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(kern), 160 * 1024, attr_done[ki]);
            if (rc) return rc;
            const int grid = panels < num_cus() ? panels : num_cus();
            if (pair_ok) {
                // second panels: sixteen waves walk both panels of a workgroup at the same time over one copy of x
                typedef void (*PairKernel)(const SkinnyArgs, int, int, int);
                static std::atomic<uint64_t> pair_done[2];
                const PairKernel pkerns[2] = {skinny_resident_pair_kernel<true, 16>, skinny_resident_pair_kernel<true, 32>};
                const int pi = s.nfrag == 256 ? 1 : 0;
                const int rc2 = ensure_dynamic_lds(reinterpret_cast<const void*>(pkerns[pi]), 160 * 1024, pair_done[pi]);
                if (rc2) return rc2;
                note_kernel("skinny_resident_w8_pair");
                hipLaunchKernelGGL(pkerns[pi], dim3(grid), dim3(1024), pair_lds, st, s, region, pair_oc_off, mr_log2);
                return check_hip(hipGetLastError(), "skinny_resident_pair_kernel launch");
            }
            note_kernel(w8 ? "skinny_resident_w8" : "skinny_resident_bf16");
            hipLaunchKernelGGL(kern, dim3(grid), dim3(512), lds, st, s, region, red_off, mr_log2);
            return check_hip(hipGetLastError(), "skinny_resident_kernel launch");
        }
    }
    // The streaming form needs all of x in LDS and at least two workgroups per CU (344 panels of N = 11008 must all
    // be resident): 80 KiB of x each (4096 x 11008 int8 GEMV at M = 5-8: 13.0-13.4 -> 11.5-12.0 us against the chunked
    // form; with one workgroup per CU, M = 12-16, it loses: 16.6-17.7 against 13.7-14.5 us).
    const bool bigx = !pairs && xbytes > 46 * 1024 && xbytes <= 80 * 1024;
    const int per_wave = (s.nfrag + 7) / 8;
    int stream_index = 0;
    const StreamKernel stream_kernel = w8 ? stream_kernel_for<1>(per_wave, &stream_index) : stream_kernel_for<0>(per_wave, &stream_index);
    if (bigx) {
        static std::atomic<uint64_t> attr_done[2][STREAM_KERNELS];
        const int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(stream_kernel), 80 * 1024, attr_done[w8 ? 1 : 0][stream_index]);
        if (rc) return rc;
    }
    if (kpad == K && (xbytes <= 46 * 1024 || bigx) && s.x_vec_ok) {
        // the activations fit in LDS: streaming variant
        if (pairs && (panels & 1)) return set_error(MMX_E_INVALID, "SILU_GATE needs an even number of 32-column panels");
        note_kernel(pairs ? (w8 ? "skinny_stream_w8_gateup" : "skinny_stream_bf16_gateup") : (w8 ? "skinny_stream_w8" : "skinny_stream_bf16"));
        // Half-panel workgroups pay off for up to 4 rows of x (cheap enough to stage per workgroup) if each still has enough
        // weights to stream (measured at M = 1: bf16 units of 80 KiB gain 8 %, of 64 KiB lose to the fixed cost of a
        // workgroup; int8 units of 172 KiB gain 16 %, of 128 KiB lose 1 %, of 64 KiB 20 %) and the list is short enough for balance to matter: at most two rounds of resident
        // workgroups (four waves each; LDS allows min(4, 160 KiB / (reduction scratch + x)) per CU)
        const int units = pairs ? panels / 2 : panels;
        const int lds_wg = 16 * 1024 * (pairs ? 2 : 1) + xbytes;
        const int wg_per_cu = (160 * 1024 / lds_wg) < 4 ? (160 * 1024 / lds_wg) : 4;
        const int64_t unit_bytes = (int64_t)s.nfrag * 512 * (pairs ? 2 : 1);
        const int force = decode_halves();  // -1: by the rule above, 0: never, 1: for every M <= 4 (tests pin the path with it)
        const bool halves = M <= 4 && !bigx && !(pairs && w8) && force != 0 &&
                            (force == 1 || (2 * units <= 2 * num_cus() * wg_per_cu && unit_bytes >= (pairs ? 128 : (w8 ? 160 : 80)) * 1024));
        const int per_wave_h = ((s.nfrag >> 1) + 3) / 4;
#define MMX_STREAM(W8, NP, GRID)                                                                                     \
    do {                                                                                                             \
        if (halves && per_wave_h <= 16 / NP)                                                                         \
            hipLaunchKernelGGL((skinny_half_kernel<W8, NP, true, 16 / NP>), dim3(2 * (GRID)), dim3(256), xbytes, st, s, zero_off); \
        else if (halves) /* the rolling window holds fewer registers where two accumulator pairs need them */      \
            hipLaunchKernelGGL((half_window_kernel<W8, NP>(s.nfrag)), dim3(2 * (GRID)), dim3(256), xbytes, st, s, zero_off); \
        else if (NP == 1)                                                                                            \
            hipLaunchKernelGGL(stream_kernel, dim3(GRID), dim3(512), stream_lds_bytes(xbytes, 1), st, s, zero_off);       \
        else if (per_wave <= 16 / NP)                                                                                \
            hipLaunchKernelGGL((skinny_stream_kernel<W8, NP, true>), dim3(GRID), dim3(512), stream_lds_bytes(xbytes, NP), st, s, zero_off); \
        else                                                                                                         \
            hipLaunchKernelGGL((skinny_stream_kernel<W8, NP, false>), dim3(GRID), dim3(512), stream_lds_bytes(xbytes, NP), st, s, zero_off); \
    } while (0)
        if (halves) note_kernel(pairs ? "skinny_half_bf16_gateup" : (w8 ? "skinny_half_w8" : "skinny_half_bf16"));
        // One row of x over int8 weights: a lane can own a column and half of a fragment's k (v_dot2_f32_bf16, one
        // cross-lane add), which costs half the issue cycles of a 32x32 MFMA that fills 31 unused rows.  It wins while a
        // CU holds a single workgroup (no second one to hide the int8 conversion behind: 4096 x 4096 6.6 against 7.6 us,
        // 4096 x 8192 8.4 against 8.8) and loses once two share a CU (4096 x 11008: 11.3 against 10.6 us).  With bf16
        // weights there is no conversion and the two forms take the same time, so only this one exists.
        // decode_valu(): -1 by that rule, 0 never, 1 always.
        const int vforce = decode_valu();
        const bool valu = w8 && M == 1 && !pairs && !halves && !bigx && vforce != 0 && (vforce == 1 || panels <= num_cus());
        if (valu) {
            note_kernel("skinny_stream_w8_valu");
            int unused;
            hipLaunchKernelGGL(stream_kernel_for<4>(per_wave, &unused), dim3(panels), dim3(512), stream_lds_bytes(xbytes, 1), st, s, zero_off);
        } else if (pairs && w8) {
            if (per_wave <= 8) hipLaunchKernelGGL((skinny_stream_kernel<1, 2, true>), dim3(panels / 2), dim3(512), stream_lds_bytes(xbytes, 2), st, s, zero_off);
            else hipLaunchKernelGGL((skinny_stream_kernel<1, 2, false>), dim3(panels / 2), dim3(512), stream_lds_bytes(xbytes, 2), st, s, zero_off);
        } else if (pairs) MMX_STREAM(false, 2, panels / 2);
        else if (w8) MMX_STREAM(true, 1, panels);
        else MMX_STREAM(false, 1, panels);
#undef MMX_STREAM
        return check_hip(hipGetLastError(), "skinny_stream_kernel launch");
    }
    // K split of the chunked kernel (a workspace at hand, the library left to choose)
    const int ksl = (kpad == K && s.x_vec_ok && !pairs && wk <= 1 && rq && rq->ws && rq->k_splits == 0)
                        ? chunk_slices(w8, M, s.nfrag, panels, rq->ws_bytes) : 1;
    if (kpad == K && s.x_vec_ok && !w8 && !pairs && M <= 8 && ksl == 1) {
        // aligned, x too large for LDS, few rows, plain bf16 weights: every lane reads its own part of x
        // (measured: for int8 weights and for gate/up pairs the chunked kernel below is faster at these M too)
        note_kernel("skinny_direct_bf16");
        hipLaunchKernelGGL((skinny_direct_kernel<false, 1>), dim3(panels), dim3(512), 0, st, s);
        return check_hip(hipGetLastError(), "skinny_direct_kernel launch");
    }
    if (kpad == K && s.x_vec_ok && !(pairs && w8)) {
        // aligned, x too large for LDS, many rows: x goes through LDS chunk by chunk
        if (pairs && (panels & 1)) return set_error(MMX_E_INVALID, "SILU_GATE needs an even number of 32-column panels");
        note_kernel(pairs ? "skinny_chunk_bf16_gateup" : (w8 ? "skinny_chunk_w8" : "skinny_chunk_bf16"));
        // LDS: two x buffers of 8 or 16 KiB, later the reduction scratch (32 KiB per panel)
#define MMX_CHUNKED(W8, NP, FPW, XD, GRID)                                                                          \
    do {                                                                                                            \
        constexpr int lds_ = (2 * 8 * XD * 1024) > (8 * NP * 16 * 64 * 4) ? (2 * 8 * XD * 1024) : (8 * NP * 16 * 64 * 4); \
        hipLaunchKernelGGL((skinny_chunk_kernel<W8, NP, FPW, XD>), dim3(GRID), dim3(512), lds_, st, s);            \
    } while (0)
        dim3 grid(panels);
        if (ksl > 1) {
            s.ws_cnt = reinterpret_cast<uint32_t*>(rq->ws);
            s.ws_part = rq->ws + SPLIT_COUNTER_BYTES;
            s.kslices = ksl;
            grid = dim3(panels, ksl);
            char name_[40];
            snprintf(name_, sizeof name_, "skinny_chunk_%s_ksplit%d", w8 ? "w8" : "bf16", ksl);
            note_kernel(name_);
        }
        // More than one panel per CU but fewer than two, 17-32 rows: a workgroup takes two neighbouring panels and stages x
        // once for both (at these M a chunk of x is 1-2 times the bytes of a panel's chunk of weights, and with one panel per
        // workgroup every workgroup pulls all of x through its CU).  4096 x 11008: int8 weights M = 24 / 32 18.2 / 19.3 ->
        // 16.7 / 17.4 us, bf16 22.6 / 24.6 -> 22.1 / 22.9; 4096 x 13824: 19.5 -> 18.2 and 25.4 -> 24.3 at M = 32.  With exactly
        // one panel per CU or fewer it leaves CUs idle (4096 x 8192: 12.8 -> 16.7), with two or more per CU and at M <= 16
        // it measured level or behind; so did a K split on top of it.
        if (!pairs && wk <= 1 && M > 16 && panels > num_cus() && panels < 2 * num_cus()) {
            note_kernel(w8 ? "skinny_chunk_w8_2p" : "skinny_chunk_bf16_2p");
            const dim3 g2((panels + 1) / 2);  // (an odd last panel: the second one of the last workgroup stores nothing)
            // (bf16 weights: four chunks in flight, 2-4 % ahead of three - 4096 x 11008 at M = 32 23.0 -> 22.4 us; six spill.
            // int8 weights: three, four already spill - 17.6 -> 23.1)
            if (w8) hipLaunchKernelGGL((skinny_chunk_kernel<true, 2, 1, 2>), g2, dim3(512), 65536, st, s);
            else hipLaunchKernelGGL((skinny_chunk_kernel<false, 2, 1, 1, 4>), g2, dim3(512), 65536, st, s);
            return check_hip(hipGetLastError(), "skinny_chunk_kernel launch");
        }
        // rows of x per buffer = 8 KiB * XD / (8 * FPW fragments * 64 or 32 bytes)
        if (pairs) {
            if (M <= 16) MMX_CHUNKED(false, 2, 2, 1, panels / 2);
            else MMX_CHUNKED(false, 2, 1, 1, panels / 2);
        } else if (w8) {
            // With at most one workgroup per CU, six chunks in flight instead of three (11008 x 4096 at M = 8 / 32: 22.0 / 27.4
            // -> 19.1 / 24.7 us; 4096 x 4096 at M = 16: 10.4 -> 9.5); with two per CU three are better (4096 x 11008 at
            // M = 16: 14.6 against 15.0), and nine no longer fit the registers.
            if (panels <= num_cus() && M <= 16) hipLaunchKernelGGL((skinny_chunk_kernel<true, 1, 1, 1, 6>), grid, dim3(512), 32768, st, s);
            else if (panels <= num_cus()) hipLaunchKernelGGL((skinny_chunk_kernel<true, 1, 1, 2, 6>), grid, dim3(512), 32768, st, s);
            else if (M <= 16) MMX_CHUNKED(true, 1, 1, 1, panels);
            else MMX_CHUNKED(true, 1, 1, 2, panels);
        } else {
            // (six chunks in flight with at most one workgroup per CU, as above: 11008 x 4096 at M = 16 / 32 28.9 / 39.3 ->
            // 26.2 / 34.1 us, 4096 x 4096 at M = 32 16.4 -> 14.6)
            if (panels <= num_cus() && M <= 16) hipLaunchKernelGGL((skinny_chunk_kernel<false, 1, 2, 1, 6>), grid, dim3(512), 32768, st, s);
            else if (panels <= num_cus()) hipLaunchKernelGGL((skinny_chunk_kernel<false, 1, 1, 1, 6>), grid, dim3(512), 32768, st, s);
            else if (M <= 16) MMX_CHUNKED(false, 1, 2, 1, panels);
            else MMX_CHUNKED(false, 1, 1, 1, panels);
        }
#undef MMX_CHUNKED
        return check_hip(hipGetLastError(), "skinny_chunk_kernel launch");
    }
    if (pairs) {
        if (panels & 1) return set_error(MMX_E_INVALID, "SILU_GATE needs an even number of 32-column panels");
        note_kernel(w8 ? "skinny_w8_gateup" : "skinny_bf16_gateup");
        if (w8) hipLaunchKernelGGL((skinny_kernel<true, 2>), dim3(panels / 2), dim3(512), 0, st, s);
        else hipLaunchKernelGGL((skinny_kernel<false, 2>), dim3(panels / 2), dim3(512), 0, st, s);
    } else {
        note_kernel(w8 ? "skinny_w8" : "skinny_bf16");
        if (w8) hipLaunchKernelGGL((skinny_kernel<true, 1>), dim3(panels), dim3(512), 0, st, s);
        else hipLaunchKernelGGL((skinny_kernel<false, 1>), dim3(panels), dim3(512), 0, st, s);
    }
    return check_hip(hipGetLastError(), "skinny_kernel launch");
}

}  // namespace mmx
