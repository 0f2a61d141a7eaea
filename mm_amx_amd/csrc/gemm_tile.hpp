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
#include <atomic>
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
    static constexpr bool W8 = false;
    static __device__ __forceinline__ accv run(frag a, frag b, accv c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ float to_f32(float v) { return v; }
};
// bf16 activations on int8-compressed weights, converted (exactly) on their way from LDS to the MFMA operand:
// the on-the-fly dequantisation of amx_kernel::Matmul<bf16,int8,float> (include/kernels_amx.hpp:1447-1497).
// A packed int8 fragment holds 32 of k per column, 16 consecutive k per lane: it feeds two bf16 MFMAs (the
// lane's first and second eight k), and the A operand is read from the matching places of its row.
struct w8_t {};
template <>
struct Mfma<w8_t> {
    using frag = bf16x8;
    using accv = f32x16;
    static constexpr bool W8 = true;
    static __device__ __forceinline__ accv run(frag a, frag b, accv c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ float to_f32(float v) { return v; }
};
template <>
struct Mfma<int8_t> {
    using frag = i32x4;
    using accv = i32x16;
    static constexpr bool W8 = false;
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
    int tiles_m, total_tiles, tiles_per_xcd;  // total_tiles and tiles_per_xcd count (tile, K slice) units
    int a_vec_ok;  // A and lda 16-byte aligned
    int ksplit;    // K slices per tile (1: every workgroup walks the whole of K)
    int kq;        // k-iterations per slice
    char* ws_part;     // partial accumulators of the K slices: [tile][slice][BM*BN] 4-byte words
    uint32_t* ws_cnt;  // one arrival counter per tile, zero between launches
    uint64_t* stamps;  // instrumented build only: 64 bytes per workgroup for its phase stamps, or null
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

// LDS ring of the hand-scheduled pipeline: RA stages of A (BM rows x 128 bytes) and R half-stages of B (BN columns
// x 64 bytes).  The ring is as deep as 156 KiB of LDS allow (R <= 2 RA - 2, see the pipeline): the loads of R - 1
// half-stages are in flight while one is multiplied, and a small tile multiplies a half-stage in far less time
// than a load takes (128x64: 128 cycles of MFMA issue against 1000+ cycles of L2 latency - with three half-stages
// in flight that tile was bound by latency, 350 cycles per half-stage).  The large tiles get 3 or 4 as before:
// their half-stages are long enough.
template <int BM, int BN, bool W8 = false>
struct Ring {
    static constexpr int A_ST = BM * 128;  // A: one stage = 128 bytes of K per row (whole cache lines)
    static constexpr int BH = BN * (W8 ? 32 : 64);  // B: one half-stage = 64 bytes of K per column (two fragments per panel;
                                                    // one fragment of 32 bytes per column for int8 weights under bf16 A)
    static constexpr int NL = BM / 64 + BH / 4096;  // HBM->LDS loads per thread per half-stage
    static constexpr int stages_for(int r) { return (r + 3) / 2; }
    static constexpr bool fits(int r) {
        return stages_for(r) * A_ST + r * BH <= 156 * 1024 && (r - 2) * NL + (NL + 1) / 2 <= 63;  // LDS; vmcnt is a 6-bit counter
    }
    static constexpr int depth() {
        int r = 3;
        for (int c = 4; c <= 12; c++)
            if (fits(c)) r = c;
        return r;
    }
    static constexpr int R = depth();          // B half-stages in LDS
    static constexpr int RA = stages_for(R);   // A stages in LDS
    static constexpr int B0 = RA * A_ST;       // the B ring follows the A ring
    static constexpr int BYTES = B0 + R * BH;
};

// SMAX: the largest number of K slices per tile this instantiation can combine (1: no K split; the
// code of the split is then absent and the kernel is the plain one).
// Development aid, compiled in with -DMMX_STAMPS only: workgroup L records the shader clock at a few points of
// its life in the 64 bytes at ws_part + 96 MiB + 64 L; the host passes that address (GemmArgs::stamps) only when the
// caller's workspace reaches that far, so an ordinary workspace is never written outside.
#ifdef MMX_STAMPS
#define MMX_STAMP(i)                                                                                                   \
    do {                                                                                                               \
        if (threadIdx.x == 0 && g.stamps) {                                                                            \
            uint64_t* st_ = g.stamps + 8 * (size_t)L;                                                                  \
            st_[i] = (i) == 0 || (i) == 7 ? __builtin_amdgcn_s_memrealtime() : __builtin_readcyclecounter();          \
        }                                                                                                              \
    } while (0)
#else
#define MMX_STAMP(i) do {} while (0)
#endif

// NW: wavefronts per workgroup.  4 = one per SIMD, each with up to 512 registers (the large accumulator blocks need
// them); 8 = two per SIMD with 256 registers each, half as large a block per wave: the second wave of a SIMD
// fills the issue slots the first leaves empty, above all in the epilogue, whose vector instructions a lone
// wave issues at under half the rate the SIMD executes them (ring pipeline only).
template <typename TIn, int BM, int BN, int MODE, typename TOut, int SMAX, int NW = 4>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(NW / 4, NW / 4))) void gemm_kernel(const GemmArgs g) {
    static_assert(NW == 4 || (NW == 8 && MODE == 2), "eight wavefronts exist for the ring pipeline only");
    constexpr int NT = NW * 64;  // threads
    using MF = Mfma<TIn>;
    using frag = typename MF::frag;
    using accv = typename MF::accv;
    using acc_t = typename std::conditional<std::is_same<TIn, int8_t>::value, int, float>::type;
    constexpr bool W8 = MF::W8;
    // per panel and k-iteration the packed weights hold 4 KiB (four fragments; two of 32 k each for int8 under bf16 A)
    constexpr int BP_IT = W8 ? 2048 : 4096;
    // the waves form a (NW/2) x 2 grid over the tile, or NW x 1 when the tile is only 64 columns wide
    // int8 weights under bf16 A: every wave converts the fragments it multiplies, so the waves sit side by side
    // (four columns of waves in the 256-column tiles; a wave keeps two panels, which the gate/up store needs):
    // a fragment is then converted by NW/4 waves instead of NW/2
    constexpr int WGN = (W8 && (BN == 256 || BM == 64)) ? 4 : (BN >= 128 ? 2 : 1), WGM = NW / WGN;
    constexpr int WM = BM / WGM, WN = BN / WGN;
    constexpr int MI = WM / 32, NJ = WN / 32;
    constexpr int A_BYTES = BM * 128, B_BYTES = BN / 32 * BP_IT, STAGE = A_BYTES + B_BYTES;
    constexpr int A_IT = BM / 32, B_IT = BN * (BP_IT / 32) / 4096;  // 16-byte chunks per thread per stage

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
    // K split: the slices of a tile are neighbours in L, so they run on one XCD and meet in its L2
    int tile = L, slice = 0, kt0 = 0, nk = g.nk;
    if constexpr (SMAX > 1) {
        tile = L / g.ksplit;
        slice = L - tile * g.ksplit;
        kt0 = slice * g.kq;
        nk = g.nk - kt0 < g.kq ? g.nk - kt0 : g.kq;
    }
    const char* const a_base = g.A + (int64_t)kt0 * 128;
    const int tn = tile / g.tiles_m, tm = tile % g.tiles_m;
    MMX_STAMP(0);
    MMX_STAMP(1);
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

    // The per-column operands of the post-op (bias, per-channel dequant and quant scales) of this tile's BN columns
    // go into LDS behind the operand buffers, straight from memory (global_load_lds_dword: 64 columns per
    // instruction, no registers) and ahead of every operand load, so they have long landed when the epilogue
    // reads them: fetched at the point of use, each column block paid a trip to memory with the matrix pipe idle.
    constexpr int OC_OFF = MODE == 2 ? Ring<BM, BN, W8>::BYTES : 2 * STAGE;
    {
        const Epilogue& e0 = g.ep;
        const float* const src_of[3] = {(e0.steps & MMX_PP_BIAS) ? e0.bias : nullptr,
                                        (e0.steps & MMX_PP_DEQUANT) ? e0.deq_oc : nullptr,
                                        (e0.steps & MMX_PP_QUANT) ? e0.q_oc : nullptr};
        const uint32_t oc_lds = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)(smem + OC_OFF));
        const int wave_s = __builtin_amdgcn_readfirstlane(wave);  // (uniform: the LDS address goes through M0)
        if (wave_s * 64 < BN) {
            int n = ntile0 + wave_s * 64 + lane;
            n = n < g.n1 ? n : g.n1 - 1;  // columns past the range are never stored: any valid address will do
#pragma unroll
            for (int a = 0; a < 3; a++) {
                if (src_of[a]) {
                    const float* src = src_of[a] + n;
                    const uint32_t m0v = oc_lds + a * BN * 4 + wave_s * 256;
                    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off" : : "s"(m0v), "v"(src) : "memory");
                }
            }
        }
    }

    float gelu_c[15];  // the GELU polynomial's coefficients, fetched into scalar registers ahead of the main loop
#pragma unroll
    for (int c = 0; c < 15; c++) {
        uint32_t bits = kGeluCoef[c];
        asm volatile("" : "+s"(bits));  // opaque: keeps the coefficient in a scalar register (see gelu_erf_minimax_x16)
        gelu_c[c] = u2f(bits);
    }

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
            const int c = it * 256 + tid;
            int panel = panel0 + c / (BP_IT / 16);
            panel = panel < g.npanels ? panel : g.npanels - 1;
            const char* src = g.Bp + (int64_t)panel * g.panel_stride + (int64_t)kt * BP_IT + (c % (BP_IT / 16)) * 16;
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
        const char* sB = smem + stage * STAGE + A_BYTES + (wn * NJ) * BP_IT + lane * 16;
        // k-step s of the stage: the lane's eight k are 16 s + 8 g32 + 0..7, or, under an int8 fragment f = s / 2
        // (whose lane holds 16 consecutive k), 32 f + 16 g32 + 8 (s % 2) + 0..7
        const int chunk = W8 ? 4 * (s >> 1) + 2 * g32 + (s & 1) : 2 * s + g32;
        const int slot = chunk ^ (l32 & 7);
#pragma unroll
        for (int i = 0; i < MI; i++) a[i] = *reinterpret_cast<const frag*>(sA + i * 32 * 128 + slot * 16);
#pragma unroll
        for (int j = 0; j < NJ; j++) {
            if constexpr (W8) {
                const u32x4 raw = *reinterpret_cast<const u32x4*>(sB + (j * 2 + (s >> 1)) * 1024);
                b[j] = (s & 1) ? s8x8_to_bf16(raw[2], raw[3]) : s8x8_to_bf16(raw[0], raw[1]);
            } else {
                b[j] = *reinterpret_cast<const frag*>(sB + (j * 4 + s) * 1024);
            }
        }
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
        using RG = Ring<BM, BN, W8>;
        constexpr int R = RG::R, RA = RG::RA, BH = RG::BH, A_ST = RG::A_ST, B0 = RG::B0;
        constexpr int BP_HS = BP_IT / 2;                  // bytes per panel and half-stage
        // A window's B chunks are NBI wave-wide loads of 1 KiB, dealt to the waves in turn: wave w issues loads
        // w, w + NW, ...  Where NBI is not a multiple of NW the first NBI % NW waves issue one more than the
        // others ("class 0" / "class 1"): the pipeline below exists once per class, because the number of a
        // wave's loads in flight is part of its wait counts.
        constexpr int NBI = BH / 1024;
        constexpr int NCLS0 = NBI % NW == 0 ? NW : NBI % NW;   // waves of class 0
        const int wave_u = __builtin_amdgcn_readfirstlane(wave);
        auto ring = [&](auto cls_c) __attribute__((always_inline)) {
        constexpr int CLS = decltype(cls_c)::value;
        constexpr int A_IT2 = BM * 4 / NT, B_IT2 = CLS == 0 ? (NBI + NW - 1) / NW : NBI / NW; // 16-byte chunks per thread per window
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
        uint32_t aoff[2][A_IT2], boff[B_IT2 > 0 ? B_IT2 : 1];  // (a wave class without B loads: NBI < NW)
#pragma unroll
        for (int half = 0; half < 2; half++)
#pragma unroll
            for (int it = 0; it < A_IT2; it++) {
                const int row = half * (BM / 2) + it * (NT / 8) + (tid >> 3);
                int grow = m0 + row;
                grow = grow < g.M ? grow : g.M - 1;
                aoff[half][it] = (uint32_t)grow * (uint32_t)g.lda + (uint32_t)(((tid & 7) ^ ((tid >> 4) & 7)) * 16);
            }
#pragma unroll
        for (int it = 0; it < B_IT2; it++) {
            const int c = it * NT + tid;
            int panel = panel0 + c / (BP_HS / 16);  // 128 chunks = one panel's two fragments of this half-stage (64 = one int8 fragment)
            panel = panel < g.npanels ? panel : g.npanels - 1;
            boff[it] = (uint32_t)(panel - panel0) * (uint32_t)g.panel_stride + (uint32_t)((c % (BP_HS / 16)) * 16);
        }
        const char* const b_base = g.Bp + (int64_t)panel0 * g.panel_stride + (int64_t)kt0 * BP_IT;
        const uint32_t lds_wave = __builtin_amdgcn_readfirstlane(
            (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)(smem + wave * 1024));
        const int last_hs = 2 * nk - 1, last_st = nk - 1;

        using std::integral_constant;
        typedef integral_constant<int, 0> c0;
        typedef integral_constant<int, 1> c1;
        typedef integral_constant<int, H> cH;
        typedef integral_constant<int, NL> cNL;

        // A operand of k-step s = 2 PAR + KS of a stage: chunk 2 s + g32 of the row; under int8 fragments (16
        // consecutive k per lane) chunk 4 PAR + 2 g32 + KS.  Chunks sit at position chunk ^ ((row >> 1) & 7).
        constexpr int KS1 = W8 ? 1 : 2;  // chunk distance from k-step 0 to k-step 1 of a half-stage
        const int a_x0 = (wm * WM + l32) * 128 + (((W8 ? 2 * g32 : g32) ^ ((l32 >> 1) & 7)) * 16);
        const int b_frag_off = B0 + wn * NJ * BP_HS + lane * 16;
        u32x4 braw[W8 ? NJ : 1];  // int8 fragments as read from LDS: each feeds both k-steps of its half-stage

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
                n.srcB = b_base + (int64_t)hs * BP_HS;
                asm volatile("" : "+s"(n.srcB));
            } else if constexpr (PART == 2) {
                int st = (w + 1) >> 1;
                st = st < last_st ? st : last_st;
                n.srcA = a_base + (int64_t)st * 128;
                asm volatile("" : "+s"(n.srcA));
            } else {
                // A operand of k-step s (0..3 within the stage): position (2 s + g32) ^ ((row >> 1) & 7) of the row
                if constexpr (KS == 0) {  // reads k-step 1 of this half-stage
                    n.rdA = as * A_ST + (a_x0 ^ ((4 * PAR + KS1) * 16));
                    n.rdB = bs * BH + b_frag_off + 1024;  // (unused with int8 fragments: the second half is in registers)
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
                             : "s"(kp.m0B), "v"(off), "s"(kp.srcB), "n"(Q * NT * 16)
                             : "memory", "scc");
            } else {
                const uint32_t off = aoff[HALF][Q - B_IT2];
                asm volatile("s_add_u32 m0, %0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                             :
                             : "s"(kp.m0A), "v"(off), "s"(kp.srcA), "n"((Q - B_IT2) * NT * 16)
                             : "memory", "scc");
            }
        };

        // one k-step: MFMAs on (ca, cb); meanwhile fill (na, nb) for the next k-step, issue loads [Q0, Q1)
        // and let `prep(part)` work out the parameters of the next k-step in the last slots
        // ks_c: which k-step of its half-stage this is (the fragments it fetches are those of the other one)
        auto kstep = [&](const frag (&ca)[MI], const frag (&cb)[NJ], frag (&na)[MI], frag (&nb)[NJ], const KParams& kp,
                         auto q0_c, auto q1_c, auto half_c, auto ks_c, auto&& prep) {
            constexpr int Q0 = decltype(q0_c)::value, Q1 = decltype(q1_c)::value, KS = decltype(ks_c)::value;
            const char* sA = smem + kp.rdA;
            const char* sB = smem + kp.rdB;
            static_for<0, MN>([&](auto t_c) {
                constexpr int t = decltype(t_c)::value;
                acc[t / NJ][t % NJ] = MF::run(cb[t % NJ], ca[t / NJ], acc[t / NJ][t % NJ]);
                static_for<t * RPS, (t + 1) * RPS>([&](auto rd_c) {
                    constexpr int rd = decltype(rd_c)::value;
                    if constexpr (rd < NJ) {
                        if constexpr (!W8) {
                            nb[rd] = *reinterpret_cast<const frag*>(sB + rd * BP_HS);
                        } else if constexpr (KS == 1) {  // next: k-step 0 of the next half-stage - fetch its int8 fragment
                            braw[rd] = *reinterpret_cast<const u32x4*>(sB + rd * BP_HS);
                        }
                    } else if constexpr (rd < NJ + MI) na[rd - NJ] = *reinterpret_cast<const frag*>(sA + (rd - NJ) * 32 * 128);
                });
                // int8 fragments -> the next k-step's bf16 operands, one dword (two weights, three instructions) at a time
                // and spread over the k-step's MFMA slots: a wave issues in order, and a whole fragment's conversion in
                // one slot (12 instructions) takes twice as long as the MFMA it should hide behind.  k-step 1 converts
                // the first halves of the fragments it has just fetched, so it starts a few slots behind their reads.
                if constexpr (W8) {
                    constexpr int D = 4 * NJ;                                       // dwords to produce
                    constexpr int S0 = KS == 1 ? (NJ + 1 < MN / 2 ? NJ + 1 : MN / 2) : 0;  // first slot that converts
                    static_for<0, D>([&](auto d_c) {
                        constexpr int d = decltype(d_c)::value;
                        if constexpr (S0 + d * (MN - S0) / D == t) {
                            constexpr int j = d / 4, e = d % 4;
                            const uint32_t src = braw[j][(KS == 1 ? 0 : 2) + e / 2];
                            u32x4 w = __builtin_bit_cast(u32x4, nb[j]);
                            w[e] = s8x2_to_bf16<e % 2>(src);
                            nb[j] = __builtin_bit_cast(frag, w);
                        }
                    });
                }
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
            kp.srcA = a_base;
            static_for<0, A_IT2>([&](auto it_c) { dma(integral_constant<int, B_IT2 + decltype(it_c)::value>{}, c0{}, kp); });
            static_for<0, R>([&](auto w_c) {
                constexpr int W = decltype(w_c)::value;
                constexpr int HALF = (W + 1) & 1;
                const int hs = W < last_hs ? W : last_hs;
                int st = (W + 1) >> 1;
                st = st < last_st ? st : last_st;
                kp.m0B = lds_wave + B0 + W * BH;
                kp.m0A = lds_wave + (((W + 1) >> 1) % RA) * A_ST + HALF * (BM / 2) * 128;
                kp.srcB = b_base + (int64_t)hs * BP_HS;
                kp.srcA = a_base + (int64_t)st * 128;
                static_for<0, (W < R - 1 ? NL : H)>([&](auto q_c) { dma(q_c, integral_constant<int, HALF>{}, kp); });
            });
        }
        KParams kpa, kpb;  // parameters of the k-step being executed / of the one after it
        static_for<0, 4>([&](auto part_c) { prepare(part_c, kpa, c0{}, c0{}, 0, 0, RA > 1 ? 1 : 0, 0); });
        asm volatile("s_waitcnt vmcnt(%0)" : : "n"((R - 2) * NL + H) : "memory");  // window 0 and all before it have landed
        __syncthreads();
        MMX_STAMP(2);
        {
            const char* sA = smem + a_x0;
            const char* sB = smem + b_frag_off;
#pragma unroll
            for (int i = 0; i < MI; i++) fa[0][i] = *reinterpret_cast<const frag*>(sA + i * 32 * 128);
#pragma unroll
            for (int j = 0; j < NJ; j++) {
                if constexpr (W8) {
                    braw[j] = *reinterpret_cast<const u32x4*>(sB + j * BP_HS);
                    fb[0][j] = s8x8_to_bf16(braw[j][0], braw[j][1]);
                } else {
                    fb[0][j] = *reinterpret_cast<const frag*>(sB + j * BP_HS);
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);

        // half-stage h = 2 st + PAR: A stage slot as (the next stage's slot is nas), B slot bs; on entry kpa
        // describes its k-step 0, on exit k-step 0 of half-stage h+1
        auto half_stage = [&](auto par_c, int h, int as, int nas, int bs) {
            constexpr int PAR = decltype(par_c)::value;
            // k-step 0: read k-step 1 of this half-stage; second group of the loads of window h+R-1
            kstep(fa[0], fb[0], fa[1], fb[1], kpa, cH{}, cNL{}, integral_constant<int, (PAR + R) & 1>{}, c0{},
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
            kstep(fa[1], fb[1], fa[0], fb[0], kpb, c0{}, cH{}, integral_constant<int, (PAR + R + 1) & 1>{}, c1{},
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
        };  // ring
        if constexpr (NCLS0 == NW) {
            ring(std::integral_constant<int, 0>{});
        } else {
            if (wave_u < NCLS0) ring(std::integral_constant<int, 0>{});
            else ring(std::integral_constant<int, 1>{});
        }
    } else {
    fetch(kt0);
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

    for (int kt = 0; kt < nk; kt++) {
        const int stage = kt & 1;
        // the last iteration re-fetches its own stage into the idle buffer: harmless, and it keeps
        // the loop body free of branches so that the schedule below is one straight block
        const int kt_next = (kt + 1 < nk) ? kt + 1 : kt;
        fetch(kt0 + kt_next);
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
    MMX_STAMP(3);

    // ---- K split: park the partial sums, the last slice to arrive combines them ---------------------------
    // Every slice writes its accumulators to its own part of the workspace (each lane 16 bytes per store,
    // in the order it holds them, so the reader's lanes find their own elements again) and counts itself
    // in.  The slice that finds all others counted adds the partial sums in slice order 0, 1, 2, ... - its
    // own from registers - so the result does not depend on which slice came last, and goes on to the
    // post-op.  The counter wraps to zero with the last arrival (atomicInc), ready for the next launch.
    // Nobody waits for anybody.
    // The partial sums cross from one workgroup to another, possibly on another XCD with its own L2:
    // they are written and read at device scope (sc1: written through to, and read from, the level all
    // XCDs share), the writer waits until its stores have been acknowledged before it counts itself in,
    // and the counter is a device-scope atomic.  A device-scope fence would do the same for ordinary
    // stores, but it writes back and invalidates the whole L2 - 25 us on a kernel of 15.
    bool combine = false;
    constexpr int AUX_SC1 = 16;  // cache policy operand of the buffer instructions: device scope
    constexpr int TILE_BYTES = BM * BN * 4;
    __amdgpu_buffer_rsrc_t parts;                                             // this tile's partial sums, all slices
    const int part_lane = wave * (MI * NJ * 4096) + lane * 16;                // this lane's place in a slice's tile
    if constexpr (SMAX > 1) {
        if (g.ksplit > 1) {
            parts = __builtin_amdgcn_make_buffer_rsrc(g.ws_part + (int64_t)tile * g.ksplit * TILE_BYTES, 0, g.ksplit * TILE_BYTES, 0x00020000);
            const int mine = slice * TILE_BYTES + part_lane;
            static_for<0, MI * NJ>([&](auto bc) __attribute__((always_inline)) {
                constexpr int b = decltype(bc)::value;
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    u32x4 w;
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const acc_t a = acc_read(acc[b / NJ][b % NJ][4 * q + e]);
                        w[e] = __builtin_bit_cast(uint32_t, a);
                    }
                    __builtin_amdgcn_raw_buffer_store_b128(w, parts, mine + (b * 4 + q) * 1024, 0, AUX_SC1);
                }
            });
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // every store of this wave has been acknowledged
            __syncthreads();
            if (tid == 0) *reinterpret_cast<volatile uint32_t*>(smem) = atomicInc(g.ws_cnt + tile, (uint32_t)g.ksplit - 1u);
            __syncthreads();
            if (*reinterpret_cast<volatile uint32_t*>(smem) != (uint32_t)g.ksplit - 1u) {
                MMX_STAMP(6);
                return;
            }
            asm volatile("" ::: "memory");
            MMX_STAMP(4);
            combine = true;
        }
    }
    // the other slices' sums of block b (held by this lane), requested one block ahead of their use
    acc_t pf[2][SMAX][16];
    auto part_load = [&](auto bc, acc_t (&dst)[SMAX][16]) __attribute__((always_inline)) {
        constexpr int b = decltype(bc)::value;
        static_for<0, SMAX>([&](auto sc) __attribute__((always_inline)) {
            constexpr int sl = decltype(sc)::value;
            if (sl < g.ksplit && sl != slice) {
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const u32x4 w = __builtin_amdgcn_raw_buffer_load_b128(parts, sl * TILE_BYTES + part_lane + (b * 4 + q) * 1024, 0, AUX_SC1);
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const uint32_t bits = w[e];  // (a bit_cast straight from the vector element reads element 0 with this compiler)
                        dst[sl][4 * q + e] = __builtin_bit_cast(acc_t, bits);
                    }
                }
            }
        });
    };
    // block (i, j) of the finished sum: the accumulators, or slice 0 + slice 1 + ... in that order
    auto block_values = [&](auto ic, auto jc, auto step_c, acc_t (&vals)[16]) __attribute__((always_inline)) {
        constexpr int i = decltype(ic)::value, j = decltype(jc)::value, step = decltype(step_c)::value;
        if constexpr (SMAX > 1) {
            if (combine) {
                static_for<0, SMAX>([&](auto sc) __attribute__((always_inline)) {
                    constexpr int sl = decltype(sc)::value;
                    if (sl < g.ksplit) {
                        acc_t x[16];
                        if (sl == slice) {
#pragma unroll
                            for (int v = 0; v < 16; v++) x[v] = acc_read(acc[i][j][v]);
                        } else {
#pragma unroll
                            for (int v = 0; v < 16; v++) x[v] = pf[step & 1][sl][v];
                        }
#pragma unroll
                        for (int v = 0; v < 16; v++) vals[v] = sl == 0 ? x[v] : vals[v] + x[v];
                    }
                });
                return;
            }
        }
#pragma unroll
        for (int v = 0; v < 16; v++) vals[v] = acc_read(acc[i][j][v]);
    };

    // ---- epilogue: accumulators -> post-op -> global memory, block by block ---------------------------
    // The weights are the first MFMA operand, so a lane holds ONE output row of a 32x32 block
    // (m = lane % 32) and four runs of four consecutive columns (n = 8q + 4(lane / 32) + 0..3, q = 0..3).
    // The two half-waves swap two of their runs (v_permlane32_swap), after which each lane owns 16
    // consecutive columns of its row and writes them with 16-byte stores: no LDS, no barrier.
    const Epilogue& ep = g.ep;
    const bool silu_gate = (ep.steps & MMX_PP_SILU_GATE) != 0;
    const int out_n1 = silu_gate ? (g.n1 >> 1) : g.n1;
    const int wave_col0 = ntile0 + wn * WN;  // first column of this wave, in accumulator columns

    // 16 per-column values (array a of the LDS copy: 0 bias, 1 dequant scale, 2 quant scale) of the block column that
    // starts at column lcol of the tile, for this lane: index v <-> column lcol + 8(v/4) + 4 g32 + v%4
    auto load_per_oc = [&](int a, int lcol, float (&dst)[16]) {
        const char* base = smem + OC_OFF + a * BN * 4 + (lcol + 4 * g32) * 4;
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const f32x4 t = *reinterpret_cast<const f32x4*>(base + q * 32);
#pragma unroll
            for (int e = 0; e < 4; e++) dst[4 * q + e] = t[e];
        }
    };
    // stores the 16 values r[] (or the raw int32 sums) of one block: row grow, output columns
    // ocol + 8(v/4) + 4 g32 + v%4
    auto store_block = [&](const float (&r)[16], const acc_t (&raw)[16], int grow, int ocol) {
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
        if constexpr (SZ == 4) {
            // 4-byte outputs: a lane's 16 columns are four 16-byte pieces, and a store instruction that takes piece t of
            // every lane touches 32 rows with 32 bytes each.  The four lanes of a quad (rows 4i .. 4i+3 of the same 16
            // columns) transpose their pieces first (two butterfly steps over DPP: lane q ends up with piece q of each
            // of the four rows), so that instruction t writes 64 contiguous bytes of row 4i + t per quad and, with the
            // other half-wave, whole 128-byte lines of 8 rows: a quarter of the memory requests (256x192 tile, fp32 out:
            // 25.4k -> 14.3k cycles).  The same for 2-byte outputs (two pieces per lane) was measured and lost: behind
            // a GELU the store is not what the epilogue waits for, and the exchange adds instructions (12.4k -> 13.9k).
            // (Every lane takes part, also those whose own row or columns are not stored.)
            uint32_t tr[16];
#pragma unroll
            for (int e = 0; e < 16; e++) tr[e] = o[e];
            const bool b0 = (lane & 1) != 0, b1 = (lane & 2) != 0;
#pragma unroll
            for (int pr = 0; pr < 2; pr++)  // pieces (0,1) and (2,3) between lanes q and q ^ 1
#pragma unroll
                for (int d = 0; d < 4; d++) {
                    uint32_t& lo = tr[(2 * pr) * 4 + d];
                    uint32_t& hi = tr[(2 * pr + 1) * 4 + d];
                    const uint32_t send = b0 ? lo : hi;
                    const uint32_t recv = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)send, 0xB1, 0xF, 0xF, true);  // quad_perm [1,0,3,2]
                    lo = b0 ? recv : lo;
                    hi = b0 ? hi : recv;
                }
#pragma unroll
            for (int pr = 0; pr < 2; pr++)  // pieces (0,2) and (1,3) between lanes q and q ^ 2
#pragma unroll
                for (int d = 0; d < 4; d++) {
                    uint32_t& lo = tr[pr * 4 + d];
                    uint32_t& hi = tr[(pr + 2) * 4 + d];
                    const uint32_t send = b1 ? lo : hi;
                    const uint32_t recv = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)send, 0x4E, 0xF, 0xF, true);  // quad_perm [2,3,0,1]
                    lo = b1 ? recv : lo;
                    hi = b1 ? hi : recv;
                }
            if (ep.c_vec_ok && c0 + 16 <= out_n1) {
                const int row0 = grow - (l32 & 3);  // first row of the quad
                char* qdst = ep.C + (int64_t)row0 * ep.ldc + (int64_t)(c0 + 4 * (l32 & 3)) * SZ;
#pragma unroll
                for (int t = 0; t < 4; t++)
                    if (row0 + t < g.M)
                        *reinterpret_cast<u32x4*>(qdst + (int64_t)t * ep.ldc) = u32x4{tr[4 * t], tr[4 * t + 1], tr[4 * t + 2], tr[4 * t + 3]};
                return;
            }
        }
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

    if (silu_gate) {  // (never combined with a K split: the host refuses it)
        if constexpr (NJ % 2 == 0) {
            const uint32_t seg_of_lane = kRcp14Seg[lane];
            static_for<0, NJ / 2>([&](auto jc) __attribute__((always_inline)) {
                constexpr int j = 2 * decltype(jc)::value;
                static_for<0, MI>([&](auto ic) __attribute__((always_inline)) {
                    constexpr int i = decltype(ic)::value;
                    float gt[16], up[16], r[16];
                    acc_t raw[16];
#pragma unroll
                    for (int v = 0; v < 16; v++) {
                        raw[v] = acc_read(acc[i][j][v]);
                        gt[v] = MF::to_f32(raw[v]);
                        up[v] = MF::to_f32(acc_read(acc[i][j + 1][v]));
                    }
                    if (ep.steps & MMX_PP_DEQUANT) {  // compressed weights: gate and up each by the scale of its own column
                        if (ep.deq_oc) {
                            float dg[16], du[16];
                            load_per_oc(1, wn * WN + 32 * j, dg);
                            load_per_oc(1, wn * WN + 32 * j + 32, du);
#pragma unroll
                            for (int v = 0; v < 16; v++) gt[v] = gt[v] * dg[v], up[v] = up[v] * du[v];
                        } else {
#pragma unroll
                            for (int v = 0; v < 16; v++) gt[v] = gt[v] * ep.deq, up[v] = up[v] * ep.deq;
                        }
                    }
                    silu_mul_x16(gt, up, r, seg_of_lane);
                    store_block(r, raw, m0 + wm * WM + 32 * i + l32, ((wave_col0 + 32 * j) >> 1));
                    __builtin_amdgcn_sched_barrier(0);
                });
            });
        }
    } else {
        // blocks are finished in the order step = j * MI + i; block b = i * NJ + j of the workspace
        if constexpr (SMAX > 1) {
            if (combine) part_load(std::integral_constant<int, 0>{}, pf[0]);
        }
        static_for<0, NJ>([&](auto jc) __attribute__((always_inline)) {
            constexpr int j = decltype(jc)::value;
            const int bcol = wave_col0 + 32 * j;
            float deq_v[16], bias_v[16], q_v[16];
            if ((ep.steps & MMX_PP_DEQUANT) && ep.deq_oc) load_per_oc(1, wn * WN + 32 * j, deq_v);
            if (ep.steps & MMX_PP_BIAS) load_per_oc(0, wn * WN + 32 * j, bias_v);
            if ((ep.steps & MMX_PP_QUANT) && ep.q_oc) load_per_oc(2, wn * WN + 32 * j, q_v);
            static_for<0, MI>([&](auto ic) __attribute__((always_inline)) {
                constexpr int i = decltype(ic)::value;
                constexpr int step = j * MI + i;
                if constexpr (SMAX > 1 && step + 1 < MI * NJ) {
                    constexpr int ni = (step + 1) % MI, nj = (step + 1) / MI;
                    if (combine) part_load(std::integral_constant<int, ni * NJ + nj>{}, pf[(step + 1) & 1]);
                }
                acc_t raw[16];
                block_values(ic, jc, std::integral_constant<int, step>{}, raw);
                float r[16];
#pragma unroll
                for (int v = 0; v < 16; v++) r[v] = MF::to_f32(raw[v]);
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
                if (ep.steps & MMX_PP_GELU) gelu_erf_minimax_x16(r, gelu_c);
                if (ep.steps & MMX_PP_QUANT) {
                    if (ep.q_oc) {
#pragma unroll
                        for (int v = 0; v < 16; v++) r[v] = r[v] * q_v[v];
                    } else {
#pragma unroll
                        for (int v = 0; v < 16; v++) r[v] = r[v] * ep.q;
                    }
                }
                store_block(r, raw, m0 + wm * WM + 32 * i + l32, bcol);
                __builtin_amdgcn_sched_barrier(0);
            });
        });
    }
    MMX_STAMP(5);
    MMX_STAMP(7);
}

// ---- host side ---------------------------------------------------------------------------------

struct TileCfg {
    int bm, bn;
};
TileCfg forced_tile();
int load_mode();
int wave_count();
int ensure_dynamic_lds(const void* kernel, int bytes, std::atomic<uint64_t>& done_on_device);

// Where the partial sums of a K split live: the first WS_COUNTER_BYTES hold one arrival counter per tile
// (zero between launches), the partial tiles follow.
constexpr int WS_MAX_TILES = 4096;
constexpr size_t WS_COUNTER_BYTES = (size_t)WS_MAX_TILES * 4;
constexpr int KSPLIT_MAX = 4;  // slices a kernel instantiation can combine (its SMAX)

// K slices are whole blocks of 512 bytes of K per row (256 bf16: the K block of AMX_MLP::Linear,
// tests/amx-mlp.cpp:548-566, whose two-way split S = 2 reproduces): slice s covers k-iterations
// [s * kq, min((s + 1) * kq, nk)).
static inline int slice_kiters(int nk, int S) { return 4 * (((nk + 3) / 4 + S - 1) / S); }

struct Plan {
    TileCfg t;
    int S;
};

// Pick the tile shape and the number of K slices that minimise a model of the launch's duration, in
// shader cycles of the busiest CU: rounds of resident workgroups x (prologue + main loop + epilogue
// [+ parking and combining partial sums]).  The main loop takes the longer of MFMA issue (BM*BN/32 cycles
// per k-iteration of 128 bytes, at the measured issue efficiency of the shape) and of pulling its
// (BM + BN) * 128 bytes per k-iteration through the CU's L2 -> L1 path (about 48 bytes per cycle).
// A K split is considered where the slices of all tiles are resident at once.
static inline Plan choose_plan(int M, int Ncols, int nk, bool need_pairs, bool wide_only, int mode, const SplitRequest& rq, bool int8_a = false) {
    static const struct { int bm, bn; float eff; } cand[] = {
        {256, 256, 0.92f}, {256, 192, 0.90f}, {128, 256, 0.86f}, {128, 192, 0.84f}, {128, 128, 0.80f}, {128, 64, 0.70f},
        {64, 128, 0.27f}};  // (64 rows: two MFMAs per k-step and wave leave the loads nothing to hide behind: 940 cycles per k-iteration)
    const TileCfg f = forced_tile();
    const int cus = num_cus();
    // measured: a CU takes 36.6 bytes per clock from L2 with all CUs pulling; parking a 64 KiB partial tile and counting
    // takes 5.5k cycles, adding one in 2.9k
    const float l1_bytes_per_clk = 36.6f, ws_bytes_per_clk = 22.5f;
    float best = 1e30f;
    Plan pick = {{128, 128}, 1};
    for (const auto& c : cand) {
        if (f.bm && (f.bm != c.bm || f.bn != c.bn)) continue;
        if (need_pairs && (c.bn % 128) != 0) continue;
        if (wide_only && c.bn == 64) continue;                      // (no 64-column tile for int8 weights under bf16 A)
        if (need_pairs && c.bm == 64) continue;                     // (the 64-row tile stores no gate/up pairs)
        if (mode == 3 && !(c.bm == 128 && c.bn == 128)) continue;   // the masked path exists for one tile shape
        if (mode != 2 && (c.bn == 64 || c.bm == 64)) continue;      // the 64-wide and 64-row tiles exist for the ring pipeline only
        const int tiles = ((M + c.bm - 1) / c.bm) * ((Ncols + c.bn - 1) / c.bn);
        for (int S = 1; S <= KSPLIT_MAX; S++) {
            if (rq.k_splits > 0 && S != rq.k_splits) continue;
            if (S > 1) {
                if (need_pairs || c.bn == 64 || !rq.ws || tiles > WS_MAX_TILES) break;
                const int kq = slice_kiters(nk, S);
                if ((S - 1) * kq >= nk) continue;  // an empty last slice
                if (WS_COUNTER_BYTES + (size_t)tiles * S * c.bm * c.bn * 4 > rq.ws_bytes) continue;
                if (rq.k_splits == 0 && (tiles * S > cus || kq < 8)) continue;
            }
            const int kit = S > 1 ? slice_kiters(nk, S) : nk;
            // int8 weights under bf16 A: every wave converts its own fragments, 12 vector instructions per MFMA operand,
            // which a block of only two row-blocks per wave cannot hide behind its MFMAs (measured issue efficiencies)
            // (64 rows: one row-block pair per converted fragment; measured 980 cycles per k-iteration)
            // (128 rows, re-fitted on a sweep of forced tiles over 4096 x 11008, 4096 x 4096 and 11008 x 4096 at M = 64-1024:
            // with 0.62 / 0.60 / 0.50 the plan missed the 128x256 tile with a K split by 13-22 % at 11008 x 4096, M = 384-1024;
            // with 0.70 / 0.50 / 0.43 its choice is within 2 % of the best forced tile on all 21 shapes)
            const float eff = !wide_only ? c.eff : (c.bm == 256 ? 0.85f : (c.bm == 64 ? 0.26f : (c.bn == 256 ? 0.70f : (c.bn == 192 ? 0.50f : 0.43f))));
            const float mfma = (float)(c.bm * c.bn / 32) / eff, bytes = (float)((c.bm + c.bn) * 128) / l1_bytes_per_clk;
            const float loop = (float)kit * (mfma > bytes ? mfma : bytes);
            const float epi = (float)(c.bm * c.bn / 256) * 100.0f;  // between a plain store (45) and a GELU (170): the plan must
                                                                   // not depend on the post-op, or a GEMM and its fused form would sum differently
            const float split = S > 1 ? 2500.0f + (float)(c.bm * c.bn * 4) * (float)S / ws_bytes_per_clk : 0.0f;
            const int per_cu = (tiles * S + cus - 1) / cus;
            // a K split has to win by a margin: its extra traffic costs clock as well as cycles (the part runs these kernels
            // at its power limit; 128x128 in two slices against 128x64: 2 % fewer cycles, 8 % lower clock)
            // (not for int8 x int8: on a sweep of forced tiles the plan without the margin is within 4 % of the best tile on
            // all 24 shapes, with it 9-16 % behind on 4096 x 4096 at M = 192-256 and 11008 x 4096 at M = 384-512)
            const float t = (float)per_cu * (3700.0f + loop + epi + split) * (S > 1 && !int8_a ? 1.15f : 1.0f);
            if (t < best) { best = t; pick = {{c.bm, c.bn}, S}; }
        }
    }
    return pick;
}

template <typename T> constexpr const char* type_tag();
template <> constexpr const char* type_tag<__bf16>() { return "bf16"; }
template <> constexpr const char* type_tag<w8_t>() { return "w8"; }
template <> constexpr const char* type_tag<uint16_t>() { return "bf16"; }
template <> constexpr const char* type_tag<int8_t>() { return "i8"; }
template <> constexpr const char* type_tag<int32_t>() { return "i32"; }
template <> constexpr const char* type_tag<float>() { return "f32"; }

template <typename TIn, int BM, int BN, int MODE, typename TOut, int SMAX, int NW = 4>
static int launch_cfg(const GemmArgs& g, int grid, hipStream_t st) {
    constexpr bool W8 = Mfma<TIn>::W8;
    // operand buffers, then three arrays of BN per-column post-op operands
    constexpr int lds = (MODE == 2 ? Ring<BM, BN, W8>::BYTES : 2 * (BM * 128 + BN * (W8 ? 64 : 128))) + 3 * BN * 4;
    static_assert(lds <= 160 * 1024, "LDS of a CU");
    auto kern = gemm_kernel<TIn, BM, BN, MODE, TOut, SMAX, NW>;
    static std::atomic<uint64_t> attr_done{0};  // one per instantiation: the devices whose LDS limit has been raised
    int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(kern), lds, attr_done);
    if (rc) return rc;
    static const char* const loads[] = {"regs", "", "ring", "masked"};
    char name[96];
    snprintf(name, sizeof name, "gemm_%s_%dx%d_%s%s_out_%s%s", type_tag<TIn>(), BM, BN, loads[MODE], NW == 8 ? "8w" : "", type_tag<TOut>(),
             g.ksplit == 2 ? "_ksplit2" : g.ksplit == 3 ? "_ksplit3" : g.ksplit == 4 ? "_ksplit4" : "");
    note_kernel(name);
    hipLaunchKernelGGL(kern, dim3(grid), dim3(NW * 64), lds, st, g);
    return check_hip(hipGetLastError(), name);
}

// The K split exists for the ring pipeline (MODE 2) and tiles at least 128 columns wide.
#define MMX_LAUNCH(TIn, BM, BN, MODE, TOut, SMAX) \
    launch_cfg<TIn, BM, BN, MODE, TOut, SMAX>(g, grid, st)
#define MMX_LAUNCH_MODES(TIn, BM, BN, TOut)                                                  \
    (g.ksplit > 1 ? MMX_LAUNCH(TIn, BM, BN, 2, TOut, KSPLIT_MAX)                              \
                  : (mode == 2 ? MMX_LAUNCH(TIn, BM, BN, 2, TOut, 1) : MMX_LAUNCH(TIn, BM, BN, 0, TOut, 1)))

template <typename TIn, typename TOut>
static int launch_tiles(const GemmArgs& g, TileCfg t, int mode, int grid, hipStream_t st) {
    if (g.ksplit > 1 && mode != 2) return set_error(MMX_E_UNSUPPORTED, "the K split needs the ring pipeline (aligned A, K a multiple of 128 bytes)");
    if (mode == 3) return MMX_LAUNCH(TIn, 128, 128, 3, TOut, 1);  // the masked path exists for one tile shape
    if (t.bm == 256 && t.bn == 256) {
        // two waves per SIMD (a 64x128 block each): MLP gate/up at M = 2048 325 -> 312 us, same bits
        // (not over int8 weights: there the four-wavefront forms are as fast or faster, 91.5 against 98.2 us for 256x192)
        if constexpr (!Mfma<TIn>::W8)
            if (wave_count() == 8 && mode == 2 && g.ksplit == 1) return launch_cfg<TIn, 256, 256, 2, TOut, 1, 8>(g, grid, st);
        return MMX_LAUNCH_MODES(TIn, 256, 256, TOut);
    }
    // (eight wavefronts were measured on the 128-row tiles as well: within +-3 % of four, not instantiated)
    if (t.bm == 128 && t.bn == 256) return MMX_LAUNCH_MODES(TIn, 128, 256, TOut);
    if (t.bm == 128 && t.bn == 128) return MMX_LAUNCH_MODES(TIn, 128, 128, TOut);
    if (t.bm == 256 && t.bn == 192) {
        // two waves per SIMD, half the accumulator block each (ring pipeline, no K split)
        if constexpr (!Mfma<TIn>::W8)
            if (wave_count() == 8 && mode == 2 && g.ksplit == 1) return launch_cfg<TIn, 256, 192, 2, TOut, 1, 8>(g, grid, st);
        return MMX_LAUNCH_MODES(TIn, 256, 192, TOut);
    }
    if (t.bm == 128 && t.bn == 192) return MMX_LAUNCH_MODES(TIn, 128, 192, TOut);
    if constexpr (!Mfma<TIn>::W8) {
        if (t.bm == 128 && t.bn == 64 && mode == 2 && g.ksplit == 1) return MMX_LAUNCH(TIn, 128, 64, 2, TOut, 1);  // ring pipeline only
    }
    {
        if (t.bm == 64 && t.bn == 128 && mode == 2)  // ring pipeline only
            return g.ksplit > 1 ? MMX_LAUNCH(TIn, 64, 128, 2, TOut, KSPLIT_MAX) : MMX_LAUNCH(TIn, 64, 128, 2, TOut, 1);
    }
    return set_error(MMX_E_UNSUPPORTED, "no MFMA tile kernel for %dx%d", t.bm, t.bn);
}

// Fills the launch geometry; returns the grid size (or a negative error code).
// w8: bf16 A on int8-compressed packed weights (elesz = 2, the size of an element of A).
static inline int prepare_gemm(GemmArgs& g, TileCfg& t, int& mode, int elesz, const void* A, int64_t lda, const void* Bp,
                               int M, int K, int N, int n0, int n1, const Epilogue& ep, const SplitRequest& rq, bool w8 = false) {
    g.A = static_cast<const char*>(A);
    g.lda = lda;
    g.Bp = static_cast<const char*>(Bp);
    g.M = M;
    g.kbytes = K * elesz;
    g.nk = (g.kbytes + 127) / 128;
    g.panel_stride = w8 ? (int64_t)((K + 127) / 128) * 4096 : (int64_t)g.nk * 4096;  // int8 panels: K padded to 128
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
    SplitRequest use = rq;
    if (mode != 2 || pairs) {
        if (rq.k_splits > 1)
            return set_error(MMX_E_UNSUPPORTED, "a K split needs 16-byte aligned rows of A, K a multiple of 128 bytes and no SILU_GATE");
        use.k_splits = 1;
    }
    if (use.k_splits > KSPLIT_MAX) return set_error(MMX_E_INVALID, "at most %d K slices", KSPLIT_MAX);
    if (use.k_splits > 1 && !use.ws) return set_error(MMX_E_INVALID, "a K split needs a workspace");
    const Plan plan = choose_plan(M, n1 - n0, g.nk, pairs, w8, mode, use, elesz == 1);
    if (use.k_splits > 1 && plan.S != use.k_splits)
        return set_error(MMX_E_INVALID, "%d K slices do not fit: K too short, the workspace too small, or more than %d tiles",
                         use.k_splits, WS_MAX_TILES);
    t = plan.t;
    if (pairs && (t.bn % 128) != 0)
        return set_error(MMX_E_INVALID, "SILU_GATE needs a tile width that is a multiple of 128");
    g.ksplit = plan.S;
    g.kq = plan.S > 1 ? slice_kiters(g.nk, plan.S) : g.nk;
    g.ws_cnt = reinterpret_cast<uint32_t*>(use.ws);
    g.ws_part = use.ws ? use.ws + WS_COUNTER_BYTES : nullptr;
    g.stamps = nullptr;
    g.tiles_m = (M + t.bm - 1) / t.bm;
    const int tiles_n = (n1 - n0 + t.bn - 1) / t.bn;
    g.total_tiles = g.tiles_m * tiles_n * g.ksplit;
    g.tiles_per_xcd = (g.total_tiles + 7) / 8;
#ifdef MMX_STAMPS
    if (use.ws && use.ws_bytes >= WS_COUNTER_BYTES + ((size_t)96 << 20) + (size_t)64 * g.tiles_per_xcd * 8)
        g.stamps = reinterpret_cast<uint64_t*>(g.ws_part + ((size_t)96 << 20));
#endif
    return g.tiles_per_xcd * 8;
}

}  // namespace mmx
