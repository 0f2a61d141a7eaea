// MFMA tile GEMM for gfx950: C[:, n0:n1] = PP(A · Bpacked[:, n0:n1]).
//
// Stands in for the large-M paths of amx_kernel::Matmul::operator()
// (include/kernels_amx.hpp:1255-1313): the AMX 2x2 register blocking of 16x16 tiles becomes a
// grid of four wavefronts (2x2, or 4x1 for the 64-column tile), each owning a block of 32x32 MFMA
// accumulators; the per-32x32-block post-op through an L1 scratch tile (:1290-1294) becomes an
// epilogue applied to the accumulators in registers: the weights are the first MFMA operand, so a
// lane holds runs of four consecutive columns of one output row, and a swap between the wave's
// halves turns them into 16 consecutive columns stored with 16-byte stores.
//
// Data movement per k-iteration (128 bytes of K per row: 64 bf16 or 128 int8):
//   A  [BM rows x 128 B]  row-major in HBM -> LDS rows of 128 B, 16-byte chunks XOR-swizzled by a
//      function of the row so that the rows an MFMA operand needs spread over the LDS banks;
//   B  [BN/32 panels x 4 fragments x 1 KiB] already in MFMA operand order in HBM -> copied
//      verbatim, every ds_read_b128 of a fragment is lane-contiguous.
// Three ways of bringing the tiles into LDS (template parameter MODE):
//   MODE 2  the product path: global_load_lds_dwordx4 (HBM -> LDS without passing through VGPRs)
//           issued from inline asm into rings of LDS slots (A in whole 128-byte lines per row, B in
//           half-stages of two fragments per panel), hand-scheduled against the MFMAs (see the
//           comment at the pipeline);
//   MODE 0  global -> VGPR -> LDS with 16-byte loads, two LDS stages, rows past M clamped to the
//           last row: the fallback when A or the packed weights are too large for the 32-bit
//           offsets MODE 2 addresses with, and a tested alternative;
//   MODE 3  MODE 0 with per-element masking: the general path for K tails (K*sizeof(T) not a
//           multiple of 128) and for A rows that are not 16-byte aligned.  Rows past M and
//           elements past K are read as zero, never touched in memory.
#pragma once
#include <type_traits>

#include "common.hpp"

namespace mmx {

// compile-time loop: f(integral_constant<int, B>) ... f(integral_constant<int, E-1>); unlike
// "#pragma unroll" it cannot be refused by the unroller's size limit (the accumulator array must
// only ever be indexed by constants, or it would be placed in scratch memory)
template <int B, int E, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (B < E) {
        f(std::integral_constant<int, B>{});
        static_for<B + 1, E>(f);
    }
}

// Reads one accumulator register at the point of use.  Left to the compiler, the AGPR -> VGPR copies
// of all accumulators are placed right behind the main loop, which overflows the vector registers
// and makes the epilogue shuffle values in and out of AGPRs.
template <typename T>
__device__ __forceinline__ T acc_read(T a) {
    T r;
    asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(r) : "a"(a));
    return r;
}

template <typename TIn>
struct Mfma;
template <>
struct Mfma<__bf16> {
    using frag = bf16x8;
    using accv = f32x16;
    static __device__ __forceinline__ accv run(frag a, frag b, accv c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ float to_f32(float v) { return v; }
};
template <>
struct Mfma<int8_t> {
    using frag = i32x4;
    using accv = i32x16;
    static __device__ __forceinline__ accv run(frag a, frag b, accv c) {
        return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0);
    }
    // vcvtdq2ps, round to nearest even (include/kernels_amx.hpp:631-634)
    static __device__ __forceinline__ float to_f32(int v) { return (float)v; }
};

struct GemmArgs {
    const char* A;
    int64_t lda;           // bytes
    const char* Bp;        // packed weights
    int64_t panel_stride;  // bytes per 32-column panel = nk * 4096
    int M;
    int kbytes;   // valid bytes per row of A
    int nk;       // k-iterations of 128 bytes
    int npanels;  // 32-column panels in Bp
    int n0, n1;
    int tiles_m, total_tiles, tiles_per_xcd;
    int a_vec_ok;  // A and lda 16-byte aligned
    Epilogue ep;
};

template <typename TOut>
__device__ __forceinline__ TOut cvt_out(float r);
template <>
__device__ __forceinline__ float cvt_out<float>(float r) { return r; }
template <>
__device__ __forceinline__ uint16_t cvt_out<uint16_t>(float r) { return to_bf16(r); }
template <>
__device__ __forceinline__ int8_t cvt_out<int8_t>(float r) { return to_s8_sat(r); }
template <>
__device__ __forceinline__ int32_t cvt_out<int32_t>(float r) { return (int32_t)r; }

__device__ __forceinline__ u32x4 load_a_chunk_masked(const char* rowptr, int kbyte, int kbytes, bool vec_ok) {
    u32x4 v = u32x4{0u, 0u, 0u, 0u};
    if (kbyte >= kbytes) return v;
    if (vec_ok && kbyte + 16 <= kbytes) return *reinterpret_cast<const u32x4*>(rowptr + kbyte);
    uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
    for (int b = 0; b < 16; b++) {
        if (kbyte + b < kbytes) w[b >> 2] |= (uint32_t)(uint8_t)rowptr[kbyte + b] << (8 * (b & 3));
    }
    return u32x4{w[0], w[1], w[2], w[3]};
}

// LDS ring of the hand-scheduled pipeline: R half-stages of (BM + BN) rows x 64 bytes.
template <int BM, int BN>
struct Ring {
    static constexpr int A_ST = BM * 128;  // A: one stage = 128 bytes of K per row (whole cache lines)
    static constexpr int BH = BN * 64;     // B: one half-stage = 64 bytes of K per column (two fragments per panel)
    static constexpr int RA = 3;           // A stages in LDS
    static constexpr int R = (RA * A_ST + 4 * BH <= 156 * 1024) ? 4 : 3;  // B half-stages in LDS (R <= 2 RA - 2)
    static constexpr int B0 = RA * A_ST;   // the B ring follows the A ring
    static constexpr int BYTES = B0 + R * BH;
};

template <typename TIn, int BM, int BN, int MODE, typename TOut>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void gemm_kernel(const GemmArgs g) {
    using MF = Mfma<TIn>;
    using frag = typename MF::frag;
    using accv = typename MF::accv;
    // the four waves form a 2x2 grid over the tile, or 4x1 when the tile is only 64 columns wide
    constexpr int WGN = BN >= 128 ? 2 : 1, WGM = 4 / WGN;
    constexpr int WM = BM / WGM, WN = BN / WGN;
    constexpr int MI = WM / 32, NJ = WN / 32;
    constexpr int A_BYTES = BM * 128, B_BYTES = BN * 128, STAGE = A_BYTES + B_BYTES;
    constexpr int A_IT = BM / 32, B_IT = BN / 32;  // 16-byte chunks per thread per stage

    extern __shared__ __attribute__((aligned(16))) char smem[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave / WGN, wn = wave % WGN;
    const int l32 = lane & 31, g32 = lane >> 5;

    // XCD-aware tile order: workgroup ids go round-robin over the 8 XCDs, so give each XCD a
    // contiguous run of tiles (m fastest): tiles that share a B panel run on one L2.
    const int L = (blockIdx.x & 7) * g.tiles_per_xcd + (blockIdx.x >> 3);
    if (L >= g.total_tiles) return;
    const int tn = L / g.tiles_m, tm = L % g.tiles_m;
    const int m0 = tm * BM;
    const int ntile0 = g.n0 + tn * BN;
    const int panel0 = ntile0 >> 5;

    accv acc[MI][NJ];
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < NJ; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0;

    u32x4 ra[MODE == 2 ? 1 : A_IT], rb[MODE == 2 ? 1 : B_IT];  // staging registers of modes 0 and 3

    auto fetch = [&](int kt) {
#pragma unroll
        for (int it = 0; it < A_IT; it++) {
            const int c = it * 256 + tid;
            const int row = c >> 3, slot = c & 7;
            const int chunk = slot ^ (row & 7);
            int grow = m0 + row;
            if constexpr (MODE != 3) {
                grow = grow < g.M ? grow : g.M - 1;
                const char* src = g.A + (int64_t)grow * g.lda + kt * 128 + chunk * 16;
                ra[it] = *reinterpret_cast<const u32x4*>(src);
            } else {
                ra[it] = u32x4{0u, 0u, 0u, 0u};
                if (grow < g.M)
                    ra[it] = load_a_chunk_masked(g.A + (int64_t)grow * g.lda, kt * 128 + chunk * 16, g.kbytes,
                                                 g.a_vec_ok);
            }
        }
#pragma unroll
        for (int it = 0; it < B_IT; it++) {
            // 256 chunks = one panel's 4 KiB of this k-iteration.  A tile may reach past the last
            // panel of the packed weights: re-read the last panel instead (those columns are never
            // stored), which keeps the loop free of branches.
            int panel = panel0 + it;
            panel = panel < g.npanels ? panel : g.npanels - 1;
            const char* src = g.Bp + (int64_t)panel * g.panel_stride + (int64_t)kt * 4096 + tid * 16;
            rb[it] = *reinterpret_cast<const u32x4*>(src);
        }
    };
    auto commit = [&](int stage) {
        char* sA = smem + stage * STAGE;
        char* sB = sA + A_BYTES;
#pragma unroll
        for (int it = 0; it < A_IT; it++) *reinterpret_cast<u32x4*>(sA + (it * 256 + tid) * 16) = ra[it];
#pragma unroll
        for (int it = 0; it < B_IT; it++) *reinterpret_cast<u32x4*>(sB + (it * 256 + tid) * 16) = rb[it];
    };

    // Fragment registers are double buffered: the ds_reads of k-step s+1 are issued before the
    // MFMAs of k-step s, so LDS latency is covered by matrix work even with one wave per SIMD.
    frag fa[2][MI], fb[2][NJ];
    auto read_frags = [&](int stage, int s, frag (&a)[MI], frag (&b)[NJ]) {
        const char* sA = smem + stage * STAGE + (wm * WM + l32) * 128;
        const char* sB = smem + stage * STAGE + A_BYTES + (wn * NJ * 4) * 1024 + lane * 16;
        const int slot = (2 * s + g32) ^ (l32 & 7);
#pragma unroll
        for (int i = 0; i < MI; i++) a[i] = *reinterpret_cast<const frag*>(sA + i * 32 * 128 + slot * 16);
#pragma unroll
        for (int j = 0; j < NJ; j++) b[j] = *reinterpret_cast<const frag*>(sB + (j * 4 + s) * 1024);
    };
    auto mma = [&](const frag (&a)[MI], const frag (&b)[NJ]) {
#pragma unroll
        for (int i = 0; i < MI; i++)
#pragma unroll
            for (int j = 0; j < NJ; j++) acc[i][j] = MF::run(b[j], a[i], acc[i][j]);
    };

    if constexpr (MODE == 2) {
        // ---- hand-scheduled ring pipeline -------------------------------------------------------------
        // One wave per SIMD means nothing hides a stall, and a wave issues in order: a burst of LDS
        // reads or of global loads in front of the MFMAs leaves the matrix pipe idle while the burst
        // drains into the LDS / address FIFOs.  So every MFMA is followed by at most one LDS read (for
        // the next k-step) and one HBM->LDS load, and the order is pinned.
        //
        // A half-stage is 64 bytes of K per row = two k-steps.  B lives in a ring of R half-stage slots
        // (two 1 KiB fragments per panel).  A lives in a ring of RA stage slots of 128 bytes per row: an
        // A row is fetched in whole 128-byte cache lines, because the L1 cannot keep half a line until
        // the next half-stage wants it: with 64-byte pieces every A line crosses the L2 -> L1 path twice.
        // (Latency is not what limits the loop - ring depths 3 to 5 take the same cycles - and the
        // kernel's clock is set by power: a third fewer L1 -> L2 requests showed up as a 4 % higher clock.)
        // The loads belonging to half-stage w
        // ("window" w) are the B chunks of half-stage w and, of A, the rows-half (w+1)&1 of stage
        // (w+1)>>1 - so both halves of a stage are complete when its first half-stage starts.
        // While half-stage h is multiplied the windows h+1 .. h+R-1 are in flight.  One workgroup
        // barrier per half-stage; it waits only for window h+1 (s_waitcnt vmcnt(N), the younger loads
        // stay outstanding; loads return in order).
        using RG = Ring<BM, BN>;
        constexpr int R = RG::R, RA = RG::RA, BH = RG::BH, A_ST = RG::A_ST, B0 = RG::B0;
        constexpr int A_IT2 = BM / 64, B_IT2 = BN / 64;   // 16-byte chunks per thread per window
        constexpr int MN = MI * NJ;                       // MFMAs per k-step
        constexpr int NL = A_IT2 + B_IT2;                 // HBM->LDS loads per thread per window
        constexpr int H = (NL + 1) / 2;                   // issued in two groups, one load per MFMA slot
        constexpr int RPS = (MI + NJ + MN - 1) / MN;      // LDS reads per MFMA slot (1 unless the wave tile is tiny)
        static_assert(H <= MN, "not enough MFMA slots to spread the loads over");
        static_assert((R - 2) * NL + H <= 63, "vmcnt is a 6-bit counter");
        static_assert(R >= 3 && R <= 2 * RA - 2, "an A stage slot must be free again when its next user is loaded");

        // A in LDS: rows of 128 bytes; the 16-byte chunk c of row r sits at position c ^ ((r >> 1) & 7), so
        // the 16 rows x 16 bytes that one LDS cycle serves for an MFMA operand fall into 16 different
        // bank groups.  A load instruction covers 8 rows x 128 bytes: lane -> (row, position).
        uint32_t aoff[2][A_IT2], boff[B_IT2];
#pragma unroll
        for (int half = 0; half < 2; half++)
#pragma unroll
            for (int it = 0; it < A_IT2; it++) {
                const int row = half * (BM / 2) + it * 32 + (tid >> 3);
                int grow = m0 + row;
                grow = grow < g.M ? grow : g.M - 1;
                aoff[half][it] = (uint32_t)grow * (uint32_t)g.lda + (uint32_t)(((tid & 7) ^ ((tid >> 4) & 7)) * 16);
            }
#pragma unroll
        for (int it = 0; it < B_IT2; it++) {
            const int c = it * 256 + tid;
            int panel = panel0 + (c >> 7);  // 128 chunks = one panel's two fragments of this half-stage
            panel = panel < g.npanels ? panel : g.npanels - 1;
            boff[it] = (uint32_t)(panel - panel0) * (uint32_t)g.panel_stride + (uint32_t)((c & 127) * 16);
        }
        const char* const b_base = g.Bp + (int64_t)panel0 * g.panel_stride;
        const uint32_t lds_wave = __builtin_amdgcn_readfirstlane(
            (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)(smem + wave * 1024));
        const int last_hs = 2 * g.nk - 1, last_st = g.nk - 1;

        using std::integral_constant;
        typedef integral_constant<int, 0> c0;
        typedef integral_constant<int, 1> c1;
        typedef integral_constant<int, H> cH;
        typedef integral_constant<int, NL> cNL;

        const int a_x0 = (wm * WM + l32) * 128 + ((g32 ^ ((l32 >> 1) & 7)) * 16);
        const int b_frag_off = B0 + wn * NJ * 2 * 1024 + lane * 16;

        // Everything a k-step needs besides its operands: where its LDS reads come from and where its
        // loads go.  A wave issues in order and an MFMA slot is 32 cycles = about six instructions, so
        // these values are computed, a few per slot, in the idle slots of the PREVIOUS k-step (and pinned
        // there: left to the compiler the whole address arithmetic lands in front of the first load of the
        // k-step, which holds up the MFMAs behind it by several slots).
        struct KParams {
            uint32_t m0B, m0A;   // LDS destinations of this wave's B chunk 0 / A round 0
            const char* srcB;    // global sources (the lane offsets are boff / aoff)
            const char* srcA;
            uint32_t rdA, rdB;   // LDS byte offsets of this lane's first A / B fragment
        };
        // k-step KS (0/1) of half-stage h = 2 st + PAR; as/nas = A slot of this / the next stage, bs = B slot.
        // k-step 0 issues the second group of window h+R-1, k-step 1 the first group of window h+R (its B
        // chunks go into the slot this half-stage has just vacated).  Of A, window w carries the rows-half
        // (w+1)&1 of stage (w+1)>>1.  Past the end the last data are fetched again, into slots that are free.
        auto prepare = [&](auto part_c, KParams& n, auto par_c, auto ks_c, int h, int as, int nas, int bs) {
            constexpr int PART = decltype(part_c)::value, PAR = decltype(par_c)::value, KS = decltype(ks_c)::value;
            constexpr int HALF = (PAR + R + KS) & 1;
            const int w = h + R - 1 + KS;
            if constexpr (PART == 0) {
                const int bslot = KS == 0 ? (bs == 0 ? R - 1 : bs - 1) : bs;
                int aslot = as + ((PAR + R + KS) >> 1);
                aslot = aslot >= RA ? aslot - RA : aslot;
                n.m0B = lds_wave + B0 + bslot * BH;
                n.m0A = lds_wave + aslot * A_ST + HALF * (BM / 2) * 128;
                asm volatile("" : "+s"(n.m0B), "+s"(n.m0A));
            } else if constexpr (PART == 1) {
                const int hs = w < last_hs ? w : last_hs;
                n.srcB = b_base + (int64_t)hs * 2048;
                asm volatile("" : "+s"(n.srcB));
            } else if constexpr (PART == 2) {
                int st = (w + 1) >> 1;
                st = st < last_st ? st : last_st;
                n.srcA = g.A + (int64_t)st * 128;
                asm volatile("" : "+s"(n.srcA));
            } else {
                // A operand of k-step s (0..3 within the stage): position (2 s + g32) ^ ((row >> 1) & 7) of the row
                if constexpr (KS == 0) {  // reads k-step 1 of this half-stage
                    n.rdA = as * A_ST + (a_x0 ^ ((4 * PAR + 2) * 16));
                    n.rdB = bs * BH + b_frag_off + 1024;
                } else {                  // reads k-step 0 of the next half-stage
                    const int nbs = bs + 1 < R ? bs + 1 : 0;
                    n.rdA = PAR == 0 ? as * A_ST + (a_x0 ^ (4 * 16)) : nas * A_ST + a_x0;
                    n.rdB = nbs * BH + b_frag_off;
                }
                asm volatile("" : "+v"(n.rdA), "+v"(n.rdB));
            }
        };
        // load number Q of a window: B chunks first, then A rounds of 32 rows
        auto dma = [&](auto q_c, auto half_c, const KParams& kp) {
            constexpr int Q = decltype(q_c)::value, HALF = decltype(half_c)::value;
            if constexpr (Q < B_IT2) {
                const uint32_t off = boff[Q];
                asm volatile("s_add_u32 m0, %0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                             :
                             : "s"(kp.m0B), "v"(off), "s"(kp.srcB), "n"(Q * 4096)
                             : "memory", "scc");
            } else {
                const uint32_t off = aoff[HALF][Q - B_IT2];
                asm volatile("s_add_u32 m0, %0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                             :
                             : "s"(kp.m0A), "v"(off), "s"(kp.srcA), "n"((Q - B_IT2) * 4096)
                             : "memory", "scc");
            }
        };

        // one k-step: MFMAs on (ca, cb); meanwhile fill (na, nb) for the next k-step, issue loads [Q0, Q1)
        // and let `prep(part)` work out the parameters of the next k-step in the last slots
        auto kstep = [&](const frag (&ca)[MI], const frag (&cb)[NJ], frag (&na)[MI], frag (&nb)[NJ], const KParams& kp,
                         auto q0_c, auto q1_c, auto half_c, auto&& prep) {
            constexpr int Q0 = decltype(q0_c)::value, Q1 = decltype(q1_c)::value;
            const char* sA = smem + kp.rdA;
            const char* sB = smem + kp.rdB;
            static_for<0, MN>([&](auto t_c) {
                constexpr int t = decltype(t_c)::value;
                acc[t / NJ][t % NJ] = MF::run(cb[t % NJ], ca[t / NJ], acc[t / NJ][t % NJ]);
                static_for<t * RPS, (t + 1) * RPS>([&](auto rd_c) {
                    constexpr int rd = decltype(rd_c)::value;
                    if constexpr (rd < NJ) nb[rd] = *reinterpret_cast<const frag*>(sB + rd * 2 * 1024);
                    else if constexpr (rd < NJ + MI) na[rd - NJ] = *reinterpret_cast<const frag*>(sA + (rd - NJ) * 32 * 128);
                });
                if constexpr (Q0 + t < Q1) dma(integral_constant<int, Q0 + t>{}, half_c, kp);
                // four parts of the next k-step's parameters in the last four slots (all in the last one
                // where a k-step has fewer)
                static_for<0, 4>([&](auto part_c) {
                    constexpr int part = decltype(part_c)::value;
                    constexpr int slot = MN >= 4 ? MN - 4 + part : MN - 1;
                    if constexpr (slot == t) prep(part_c);
                });
                __builtin_amdgcn_sched_barrier(0);
            });
        };
        // prologue: the first rows-half of stage 0 (it belongs to no window), windows 0 .. R-2 completely,
        // and the first group of window R-1
        {
            KParams kp;
            kp.m0A = lds_wave;
            kp.srcA = g.A;
            static_for<0, A_IT2>([&](auto it_c) { dma(integral_constant<int, B_IT2 + decltype(it_c)::value>{}, c0{}, kp); });
            static_for<0, R>([&](auto w_c) {
                constexpr int W = decltype(w_c)::value;
                constexpr int HALF = (W + 1) & 1;
                const int hs = W < last_hs ? W : last_hs;
                int st = (W + 1) >> 1;
                st = st < last_st ? st : last_st;
                kp.m0B = lds_wave + B0 + W * BH;
                kp.m0A = lds_wave + (((W + 1) >> 1) % RA) * A_ST + HALF * (BM / 2) * 128;
                kp.srcB = b_base + (int64_t)hs * 2048;
                kp.srcA = g.A + (int64_t)st * 128;
                static_for<0, (W < R - 1 ? NL : H)>([&](auto q_c) { dma(q_c, integral_constant<int, HALF>{}, kp); });
            });
        }
        KParams kpa, kpb;  // parameters of the k-step being executed / of the one after it
        static_for<0, 4>([&](auto part_c) { prepare(part_c, kpa, c0{}, c0{}, 0, 0, RA > 1 ? 1 : 0, 0); });
        asm volatile("s_waitcnt vmcnt(%0)" : : "n"((R - 2) * NL + H) : "memory");  // window 0 and all before it have landed
        __syncthreads();
        {
            const char* sA = smem + a_x0;
            const char* sB = smem + b_frag_off;
#pragma unroll
            for (int i = 0; i < MI; i++) fa[0][i] = *reinterpret_cast<const frag*>(sA + i * 32 * 128);
#pragma unroll
            for (int j = 0; j < NJ; j++) fb[0][j] = *reinterpret_cast<const frag*>(sB + j * 2 * 1024);
        }
        __builtin_amdgcn_sched_barrier(0);

        // half-stage h = 2 st + PAR: A stage slot as (the next stage's slot is nas), B slot bs; on entry kpa
        // describes its k-step 0, on exit k-step 0 of half-stage h+1
        auto half_stage = [&](auto par_c, int h, int as, int nas, int bs) {
            constexpr int PAR = decltype(par_c)::value;
            // k-step 0: read k-step 1 of this half-stage; second group of the loads of window h+R-1
            kstep(fa[0], fb[0], fa[1], fb[1], kpa, cH{}, cNL{}, integral_constant<int, (PAR + R) & 1>{},
                  [&](auto part_c) { prepare(part_c, kpb, par_c, c1{}, h, as, nas, bs); });
            // every wave now holds all of half-stage h in registers; window h+1 must have landed, the
            // (R-2) younger ones may still be in flight
            asm volatile("s_waitcnt vmcnt(%0)" : : "n"((R - 2) * NL) : "memory");
            __syncthreads();
            __builtin_amdgcn_sched_barrier(0);
            // k-step 1: read k-step 0 of the next half-stage; first group of the loads of window h+R
            const int nbs = bs + 1 < R ? bs + 1 : 0;
            int as_n = as, nas_n = nas;  // slots as half-stage h+1 sees them
            if constexpr (PAR == 1) {
                as_n = nas;
                nas_n = nas + 1 < RA ? nas + 1 : 0;
            }
            kstep(fa[1], fb[1], fa[0], fb[0], kpb, c0{}, cH{}, integral_constant<int, (PAR + R + 1) & 1>{},
                  [&](auto part_c) { prepare(part_c, kpa, integral_constant<int, 1 - PAR>{}, c0{}, h + 1, as_n, nas_n, nbs); });
        };
        int as = 0, bs = 0;
        for (int st = 0; st <= last_st; st++) {
            const int nas = as + 1 < RA ? as + 1 : 0;
            half_stage(c0{}, 2 * st, as, nas, bs);
            bs = bs + 1 < R ? bs + 1 : 0;
            half_stage(c1{}, 2 * st + 1, as, nas, bs);
            bs = bs + 1 < R ? bs + 1 : 0;
            as = nas;
        }
        asm volatile("s_waitcnt vmcnt(0)" : : : "memory");  // the re-fetched slots past the end must land before the wave ends
    } else {
    fetch(0);
    commit(0);
    __syncthreads();
    read_frags(0, 0, fa[0], fb[0]);

    // Scheduling groups: alternate one MFMA of the current k-step with one LDS read of the next
    // (mask 0x008 = MFMA, 0x100 = DS read), then the remaining MFMAs.
#define MMX_INTERLEAVE()                                                   \
    for (int r_ = 0; r_ < MI + NJ; r_++) {                                 \
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                 \
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);                 \
    }                                                                      \
    __builtin_amdgcn_sched_group_barrier(0x008, MI * NJ - (MI + NJ), 0);   \
    __builtin_amdgcn_sched_barrier(0)

    for (int kt = 0; kt < g.nk; kt++) {
        const int stage = kt & 1;
        // the last iteration re-fetches its own stage into the idle buffer: harmless, and it keeps
        // the loop body free of branches so that the schedule below is one straight block
        const int kt_next = (kt + 1 < g.nk) ? kt + 1 : kt;
        fetch(kt_next);
        __builtin_amdgcn_sched_barrier(0);
        read_frags(stage, 1, fa[1], fb[1]);
        mma(fa[0], fb[0]);
        MMX_INTERLEAVE();
        read_frags(stage, 2, fa[0], fb[0]);
        mma(fa[1], fb[1]);
        MMX_INTERLEAVE();
        read_frags(stage, 3, fa[1], fb[1]);
        mma(fa[0], fb[0]);
        MMX_INTERLEAVE();
        // Everything this wave reads from the current stage is now in registers, and the next
        // stage has had three k-steps to land: synchronise here, then start reading the next
        // stage while the last k-step of this one is multiplied.
        commit(stage ^ 1);
            __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
        read_frags(stage ^ 1, 0, fa[0], fb[0]);
        mma(fa[1], fb[1]);
        MMX_INTERLEAVE();
    }
#undef MMX_INTERLEAVE
    }

    // the explicit accumulator reads below are invisible to the compiler's hazard checks: let the last
    // MFMAs retire (a 32x32 MFMA needs up to 18 wait states before its result may be read)
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");

    // ---- epilogue: accumulators -> post-op -> global memory, block by block ---------------------------
    // The weights are the first MFMA operand, so a lane holds ONE output row of a 32x32 block
    // (m = lane % 32) and four runs of four consecutive columns (n = 8q + 4(lane / 32) + 0..3, q = 0..3).
    // The two half-waves swap two of their runs (v_permlane32_swap), after which each lane owns 16
    // consecutive columns of its row and writes them with 16-byte stores: no LDS, no barrier.
    const Epilogue& ep = g.ep;
    const bool silu_gate = (ep.steps & MMX_PP_SILU_GATE) != 0;
    const int out_n1 = silu_gate ? (g.n1 >> 1) : g.n1;
    const int wave_col0 = ntile0 + wn * WN;  // first column of this wave, in accumulator columns

    // 16 per-column values of block column bcol for this lane: index v <-> column bcol + 8(v/4) + 4 g32 + v%4
    auto load_per_oc = [&](const float* p, int bcol, float (&dst)[16]) {
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const int n = bcol + 8 * q + 4 * g32;
            if (n + 4 <= g.n1 && (reinterpret_cast<uintptr_t>(p) & 15) == 0) {
                const f32x4 t = *reinterpret_cast<const f32x4*>(p + n);
#pragma unroll
                for (int e = 0; e < 4; e++) dst[4 * q + e] = t[e];
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++) dst[4 * q + e] = (n + e < g.n1) ? p[n + e] : 0.0f;
            }
        }
    };
    // stores the 16 values r[] (or raw int32 accumulators) of one block: row grow, output columns
    // ocol + 8(v/4) + 4 g32 + v%4
    auto store_block = [&](const float (&r)[16], const accv& raw, int grow, int ocol) {
        constexpr int SZ = sizeof(TOut);
        constexpr int DW = SZ;  // dwords per run of four elements
        uint32_t w[4][DW];
#pragma unroll
        for (int q = 0; q < 4; q++) {
            if constexpr (std::is_same<TOut, float>::value) {
#pragma unroll
                for (int e = 0; e < 4; e++) w[q][e] = f2u(r[4 * q + e]);
            } else if constexpr (std::is_same<TOut, int32_t>::value) {
#pragma unroll
                for (int e = 0; e < 4; e++) w[q][e] = (uint32_t)raw[4 * q + e];
            } else if constexpr (std::is_same<TOut, uint16_t>::value) {
                w[q][0] = (uint32_t)to_bf16(r[4 * q]) | ((uint32_t)to_bf16(r[4 * q + 1]) << 16);
                w[q][1] = (uint32_t)to_bf16(r[4 * q + 2]) | ((uint32_t)to_bf16(r[4 * q + 3]) << 16);
            } else {
                w[q][0] = to_s8_sat_x4(r[4 * q], r[4 * q + 1], r[4 * q + 2], r[4 * q + 3]);
            }
        }
        // lower half-wave: runs 0,1 of both halves = columns 0..15; upper half-wave: runs 2,3 = 16..31
        uint32_t o[4 * DW];
#pragma unroll
        for (int d = 0; d < DW; d++) {
            const auto s02 = __builtin_amdgcn_permlane32_swap(w[0][d], w[2][d], false, false);
            const auto s13 = __builtin_amdgcn_permlane32_swap(w[1][d], w[3][d], false, false);
            o[d] = s02[0];
            o[DW + d] = s02[1];
            o[2 * DW + d] = s13[0];
            o[3 * DW + d] = s13[1];
        }
        const int c0 = ocol + 16 * g32;
        if (grow >= g.M || c0 >= out_n1) return;
        char* dst = ep.C + (int64_t)grow * ep.ldc + (int64_t)c0 * SZ;
        if (ep.c_vec_ok && c0 + 16 <= out_n1) {
#pragma unroll
            for (int t = 0; t < DW; t++)
                *reinterpret_cast<u32x4*>(dst + 16 * t) = u32x4{o[4 * t], o[4 * t + 1], o[4 * t + 2], o[4 * t + 3]};
        } else {
#pragma unroll
            for (int e = 0; e < 16; e++) {
                if (c0 + e < out_n1) {
                    const uint32_t word = o[e * SZ / 4];
                    if constexpr (SZ == 4) reinterpret_cast<uint32_t*>(dst)[e] = word;
                    else if constexpr (SZ == 2) reinterpret_cast<uint16_t*>(dst)[e] = (uint16_t)(word >> (16 * (e & 1)));
                    else reinterpret_cast<uint8_t*>(dst)[e] = (uint8_t)(word >> (8 * (e & 3)));
                }
            }
        }
    };

    if (silu_gate) {
        if constexpr (NJ % 2 == 0) {
            const uint32_t seg_of_lane = kRcp14Seg[lane];
            static_for<0, NJ / 2>([&](auto jc) __attribute__((always_inline)) {
                constexpr int j = 2 * decltype(jc)::value;
                static_for<0, MI>([&](auto ic) __attribute__((always_inline)) {
                    constexpr int i = decltype(ic)::value;
                    float gt[16], up[16], r[16];
#pragma unroll
                    for (int v = 0; v < 16; v++) {
                        gt[v] = MF::to_f32(acc_read(acc[i][j][v]));
                        up[v] = MF::to_f32(acc_read(acc[i][j + 1][v]));
                    }
                    silu_mul_x16(gt, up, r, seg_of_lane);
                    store_block(r, acc[i][j], m0 + wm * WM + 32 * i + l32, ((wave_col0 + 32 * j) >> 1));
                    __builtin_amdgcn_sched_barrier(0);
                });
            });
        }
    } else {
        static_for<0, NJ>([&](auto jc) __attribute__((always_inline)) {
            constexpr int j = decltype(jc)::value;
            const int bcol = wave_col0 + 32 * j;
            float deq_v[16], bias_v[16], q_v[16];
            if ((ep.steps & MMX_PP_DEQUANT) && ep.deq_oc) load_per_oc(ep.deq_oc, bcol, deq_v);
            if (ep.steps & MMX_PP_BIAS) load_per_oc(ep.bias, bcol, bias_v);
            if ((ep.steps & MMX_PP_QUANT) && ep.q_oc) load_per_oc(ep.q_oc, bcol, q_v);
            static_for<0, MI>([&](auto ic) __attribute__((always_inline)) {
                constexpr int i = decltype(ic)::value;
                float r[16];
#pragma unroll
                for (int v = 0; v < 16; v++) r[v] = MF::to_f32(acc_read(acc[i][j][v]));
                if (ep.steps & MMX_PP_DEQUANT) {
                    if (ep.deq_oc) {
#pragma unroll
                        for (int v = 0; v < 16; v++) r[v] = r[v] * deq_v[v];
                    } else {
#pragma unroll
                        for (int v = 0; v < 16; v++) r[v] = r[v] * ep.deq;
                    }
                }
                if (ep.steps & MMX_PP_BIAS) {
#pragma unroll
                    for (int v = 0; v < 16; v++) r[v] = r[v] + bias_v[v];
                }
                if (ep.steps & MMX_PP_GELU) gelu_erf_minimax_x16(r);
                if (ep.steps & MMX_PP_QUANT) {
                    if (ep.q_oc) {
#pragma unroll
                        for (int v = 0; v < 16; v++) r[v] = r[v] * q_v[v];
                    } else {
#pragma unroll
                        for (int v = 0; v < 16; v++) r[v] = r[v] * ep.q;
                    }
                }
                store_block(r, acc[i][j], m0 + wm * WM + 32 * i + l32, bcol);
                __builtin_amdgcn_sched_barrier(0);
            });
        });
    }
}

// ---- host side ---------------------------------------------------------------------------------

struct TileCfg {
    int bm, bn;
};
TileCfg forced_tile();
int load_mode();

// Pick the tile that minimises (tiles per CU, rounded up) x (work per tile) / (per-tile efficiency).
// Workgroups that share a CU share its matrix pipe, so what counts is how many tiles the busiest CU
// has to finish.  The efficiency factors are measured on the 1024 x 4096 x 11008 FC: larger tiles
// re-use each LDS fragment for more MFMAs and load fewer bytes per flop.
static inline TileCfg choose_tile(int M, int Ncols, bool need_pairs) {
    const TileCfg f = forced_tile();
    if (f.bm) return f;
    static const struct { int bm, bn; float eff; } cand[] = {
        {256, 256, 1.00f}, {256, 192, 0.97f}, {128, 256, 0.90f}, {128, 192, 0.86f}, {128, 128, 0.80f}, {128, 64, 0.48f}};
    const int cus = num_cus();
    float best = 1e30f;
    TileCfg pick = {128, 128};
    for (const auto& c : cand) {
        if (need_pairs && (c.bn % 128) != 0) continue;
        const int tiles = ((M + c.bm - 1) / c.bm) * ((Ncols + c.bn - 1) / c.bn);
        const int per_cu = (tiles + cus - 1) / cus;
        const float t = (float)per_cu * (float)(c.bm * c.bn) / c.eff;
        if (t < best) { best = t; pick = {c.bm, c.bn}; }
    }
    return pick;
}

template <typename T> constexpr const char* type_tag();
template <> constexpr const char* type_tag<__bf16>() { return "bf16"; }
template <> constexpr const char* type_tag<uint16_t>() { return "bf16"; }
template <> constexpr const char* type_tag<int8_t>() { return "i8"; }
template <> constexpr const char* type_tag<int32_t>() { return "i32"; }
template <> constexpr const char* type_tag<float>() { return "f32"; }

template <typename TIn, int BM, int BN, int MODE, typename TOut>
static int launch_cfg(const GemmArgs& g, int grid, hipStream_t st) {
    constexpr int lds = MODE == 2 ? Ring<BM, BN>::BYTES : 2 * (BM + BN) * 128;
    auto kern = gemm_kernel<TIn, BM, BN, MODE, TOut>;
    static bool attr_done = false;  // one flag and one name per instantiation
    static char name[64];
    if (!name[0]) {
        static const char* const loads[] = {"regs", "", "ring", "masked"};
        snprintf(name, sizeof name, "gemm_%s_%dx%d_%s_out_%s", type_tag<TIn>(), BM, BN, loads[MODE], type_tag<TOut>());
    }
    if (!attr_done) {
        int rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, lds),
                           "hipFuncSetAttribute(MaxDynamicSharedMemorySize)");
        if (rc) return rc;
        attr_done = true;
    }
    note_kernel(name);
    hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds, st, g);
    return check_hip(hipGetLastError(), name);
}

#define MMX_LAUNCH(TIn, BM, BN, MODE, TOut) \
    launch_cfg<TIn, BM, BN, MODE, TOut>(g, grid, st)
#define MMX_LAUNCH_MODES(TIn, BM, BN, TOut) \
    (mode == 2 ? MMX_LAUNCH(TIn, BM, BN, 2, TOut) : MMX_LAUNCH(TIn, BM, BN, 0, TOut))

template <typename TIn, typename TOut>
static int launch_tiles(const GemmArgs& g, TileCfg t, int mode, int grid, hipStream_t st) {
    if (mode == 3) return MMX_LAUNCH(TIn, 128, 128, 3, TOut);  // the masked path exists for one tile shape
    if (t.bm == 256 && t.bn == 256) return MMX_LAUNCH_MODES(TIn, 256, 256, TOut);
    if (t.bm == 256 && t.bn == 192) return MMX_LAUNCH_MODES(TIn, 256, 192, TOut);
    if (t.bm == 128 && t.bn == 256) return MMX_LAUNCH_MODES(TIn, 128, 256, TOut);
    if (t.bm == 128 && t.bn == 192) return MMX_LAUNCH_MODES(TIn, 128, 192, TOut);
    if (t.bm == 128 && t.bn == 128) return MMX_LAUNCH_MODES(TIn, 128, 128, TOut);
    if (t.bm == 128 && t.bn == 64 && mode == 2) return MMX_LAUNCH(TIn, 128, 64, 2, TOut);  // ring pipeline only
    return set_error(MMX_E_UNSUPPORTED, "no MFMA tile kernel for %dx%d", t.bm, t.bn);
}

// Fills the launch geometry; returns the grid size (or a negative error code).
static inline int prepare_gemm(GemmArgs& g, TileCfg& t, int& mode, int elesz, const void* A, int64_t lda, const void* Bp,
                               int M, int K, int N, int n0, int n1, const Epilogue& ep) {
    g.A = static_cast<const char*>(A);
    g.lda = lda;
    g.Bp = static_cast<const char*>(Bp);
    g.M = M;
    g.kbytes = K * elesz;
    g.nk = (g.kbytes + 127) / 128;
    g.panel_stride = (int64_t)g.nk * 4096;
    g.npanels = (N + 31) / 32;
    g.n0 = n0;
    g.n1 = n1;
    g.a_vec_ok = ((reinterpret_cast<uintptr_t>(A) & 15) == 0) && ((lda & 15) == 0);
    g.ep = ep;
    const bool pairs = (ep.steps & MMX_PP_SILU_GATE) != 0;
    // the unmasked loads need aligned rows and a K that fills whole k-iterations
    const bool fast_ok = g.a_vec_ok && (g.kbytes % 128 == 0);
    mode = fast_ok ? load_mode() : 3;
    // mode 2 addresses A through 32-bit per-thread offsets
    if (mode == 2 && ((int64_t)M * lda >= ((int64_t)1 << 32) - 4096 || g.panel_stride >= ((int64_t)1 << 28))) mode = 0;
    t = choose_tile(M, n1 - n0, pairs);
    if (mode == 3) t = {128, 128};
    if (mode != 2 && t.bn == 64) t = {128, 128};  // the 64-wide tile exists for the ring pipeline only
    if (pairs && (t.bn % 128) != 0)
        return set_error(MMX_E_INVALID, "SILU_GATE needs a tile width that is a multiple of 128");
    g.tiles_m = (M + t.bm - 1) / t.bm;
    const int tiles_n = (n1 - n0 + t.bn - 1) / t.bn;
    g.total_tiles = g.tiles_m * tiles_n;
    g.tiles_per_xcd = (g.total_tiles + 7) / 8;
    return g.tiles_per_xcd * 8;
}

}  // namespace mmx
