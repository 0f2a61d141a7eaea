// One-off weight preparation kernels: repack to MFMA-fragment order, gate/up interleave,
// per-tensor int8 weight compression, packed int8 -> packed bf16.
//
// Stands in for amx_kernel::repackB_1x2 (include/kernels_amx.hpp:761-816), MLP::setup's gate/up
// interleave (tests/amx-mlp.cpp:758-765) and the weight compression inside
// amx_kernel::Matmul<bf16,int8,float> (include/kernels_amx.hpp:1363-1377, 465-523).
// These move bytes once per weight matrix; they are written for clarity, each thread producing one
// 16-byte lane slot of the packed result.
#include "common.hpp"

namespace mmx {

// Packed layout: [panel = n/32][f = k/KS][lane][16 B], KS = 32/ES elements, lane = n%32 + 32*((k%KS)/(KS/2)).
// flip: the sign bit of every byte is inverted on the way (unsigned 8-bit weights u -> u - 128 as a signed byte; the
// zero padding is left at zero)
template <int ES>
__global__ void repack_kernel(const char* __restrict__ B, int64_t ldb, int K, int N, int transpose,
                              char* __restrict__ out, int nfrag, int64_t total_slots, int flip) {
    constexpr int HALF = 16 / ES;  // elements per lane slot
    const int64_t slot = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (slot >= total_slots) return;
    const int lane = (int)(slot & 63);
    const int64_t pf = slot >> 6;
    const int f = (int)(pf % nfrag);
    const int panel = (int)(pf / nfrag);
    const int n = panel * 32 + (lane & 31);
    const int k0 = f * (2 * HALF) + (lane >> 5) * HALF;
    alignas(16) char buf[16];
#pragma unroll
    for (int e = 0; e < HALF; e++) {
        const int k = k0 + e;
        const bool ok = (n < N) && (k < K);
        const char* src = transpose ? B + (int64_t)n * ldb + (int64_t)k * ES : B + (int64_t)k * ldb + (int64_t)n * ES;
        if (ES == 2) {
            reinterpret_cast<uint16_t*>(buf)[e] = ok ? *reinterpret_cast<const uint16_t*>(src) : (uint16_t)0;
        } else {
            buf[e] = ok ? (char)(*src ^ (flip ? 0x80 : 0)) : (char)0;
        }
    }
    *reinterpret_cast<uint4*>(out + slot * 16) = *reinterpret_cast<const uint4*>(buf);
}

int launch_repack(int elesz, const void* B, int64_t ldb, int K, int N, int transpose, void* out, hipStream_t st, int flip) {
    const int kpad_bytes = (K * elesz + 127) / 128 * 128;
    const int nfrag = kpad_bytes / 32;
    const int64_t npanels = (N + 31) / 32;
    const int64_t slots = npanels * nfrag * 64;
    const int threads = 256;
    const int64_t blocks = (slots + threads - 1) / threads;
    if (blocks > 0x7fffffff) return set_error(MMX_E_INVALID, "weight matrix too large to repack in one launch");
    if (elesz == 2)
        hipLaunchKernelGGL((repack_kernel<2>), dim3((unsigned)blocks), dim3(threads), 0, st,
                           static_cast<const char*>(B), ldb, K, N, transpose, static_cast<char*>(out), nfrag, slots, 0);
    else
        hipLaunchKernelGGL((repack_kernel<1>), dim3((unsigned)blocks), dim3(threads), 0, st,
                           static_cast<const char*>(B), ldb, K, N, transpose, static_cast<char*>(out), nfrag, slots, flip);
    return check_hip(hipGetLastError(), "repack_kernel launch");
}

// gate and up ([N, K] bf16 each) -> one packed matrix of 2N columns: panel 2p = gate columns
// [32p, 32p+32), panel 2p+1 = up columns [32p, 32p+32).
__global__ void repack_gate_up_kernel(const char* __restrict__ Wg, const char* __restrict__ Wu, int64_t ldw, int K,
                                      int N, char* __restrict__ out, int nfrag, int64_t total_slots) {
    const int64_t slot = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (slot >= total_slots) return;
    const int lane = (int)(slot & 63);
    const int64_t pf = slot >> 6;
    const int f = (int)(pf % nfrag);
    const int panel = (int)(pf / nfrag);
    const char* W = (panel & 1) ? Wu : Wg;
    const int n = (panel >> 1) * 32 + (lane & 31);
    const int k0 = f * 16 + (lane >> 5) * 8;
    alignas(16) uint16_t buf[8];
#pragma unroll
    for (int e = 0; e < 8; e++) {
        const int k = k0 + e;
        buf[e] = (n < N && k < K) ? *reinterpret_cast<const uint16_t*>(W + (int64_t)n * ldw + (int64_t)k * 2) : (uint16_t)0;
    }
    *reinterpret_cast<uint4*>(out + slot * 16) = *reinterpret_cast<const uint4*>(buf);
}

int launch_repack_gate_up(const void* wg, const void* wu, int64_t ldw, int K, int N, void* out, hipStream_t st) {
    const int nfrag = ((K * 2 + 127) / 128 * 128) / 32;
    const int64_t slots = (int64_t)(2 * N / 32) * nfrag * 64;
    const int threads = 256;
    const int64_t blocks = (slots + threads - 1) / threads;
    if (blocks > 0x7fffffff) return set_error(MMX_E_INVALID, "weight matrix too large to repack in one launch");
    hipLaunchKernelGGL(repack_gate_up_kernel, dim3((unsigned)blocks), dim3(threads), 0, st, static_cast<const char*>(wg),
                       static_cast<const char*>(wu), ldw, K, N, static_cast<char*>(out), nfrag, slots);
    return check_hip(hipGetLastError(), "repack_gate_up_kernel launch");
}

// ---- per-tensor weight compression ---------------------------------------------------------------
__global__ void zero_u32_kernel(uint32_t* p) { *p = 0u; }

// max |w| over the matrix: the bit pattern of a non-negative float orders like an unsigned integer
__global__ void absmax_kernel(const char* __restrict__ W, int64_t ldw, int rows, int cols, uint32_t* out) {
    uint32_t m = 0;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < (int64_t)rows * cols;
         i += (int64_t)gridDim.x * blockDim.x) {
        const int r = (int)(i / cols), c = (int)(i % cols);
        const uint32_t bits = (uint32_t)(*reinterpret_cast<const uint16_t*>(W + (int64_t)r * ldw + (int64_t)c * 2)) << 16;
        const uint32_t a = bits & 0x7fffffffu;
        if (a <= 0x7f800000u && a > m) m = a;  // NaNs do not take part, as with vmaxps/vminps accumulators
    }
    for (int off = 32; off > 0; off >>= 1) {
        const uint32_t o = __shfl_xor(m, off);
        m = o > m ? o : m;
    }
    if ((threadIdx.x & 63) == 0) atomicMax(out, m);
}

// q = sat8(rne(w * (127/max))) (include/kernels_amx.hpp:508-523); scales_out = {127/max, max/127}
__global__ void quantize_kernel(const char* __restrict__ W, int64_t ldw, int rows, int cols, char* __restrict__ Wq,
                                int64_t ldq, const uint32_t* absmax_bits, float* scales_out) {
    const float amax = u2f(*absmax_bits);
    const float q = 127 / amax;
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        scales_out[0] = q;
        scales_out[1] = amax / 127;
    }
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < (int64_t)rows * cols;
         i += (int64_t)gridDim.x * blockDim.x) {
        const int r = (int)(i / cols), c = (int)(i % cols);
        const float w = from_bf16(*reinterpret_cast<const uint16_t*>(W + (int64_t)r * ldw + (int64_t)c * 2));
        Wq[(int64_t)r * ldq + c] = (char)to_s8_sat(w * q);
    }
}

int launch_quantize(const void* W, int64_t ldw, int rows, int cols, void* Wq, int64_t ldq, float* scales_out,
                    uint32_t* scratch, hipStream_t st) {
    const int64_t n = (int64_t)rows * cols;
    int blocks = (int)((n + 255) / 256 < 4096 ? (n + 255) / 256 : 4096);
    if (blocks < 1) blocks = 1;
    hipLaunchKernelGGL(zero_u32_kernel, dim3(1), dim3(1), 0, st, scratch);
    hipLaunchKernelGGL(absmax_kernel, dim3(blocks), dim3(256), 0, st, static_cast<const char*>(W), ldw, rows, cols, scratch);
    hipLaunchKernelGGL(quantize_kernel, dim3(blocks), dim3(256), 0, st, static_cast<const char*>(W), ldw, rows, cols,
                       static_cast<char*>(Wq), ldq, scratch, scales_out);
    return check_hip(hipGetLastError(), "quantize kernels launch");
}

// q = trunc(bf16_rne(float(w) * scale)): the element conversion of repackB_1xL<int8_t, L>
// (weight_compression/fc16m.cpp:80-81, "*dst++ = src0[n] * scale" with src0 an ov::bfloat16* and dst an int8_t*: the
// product is a bfloat16 again, include/bf16.hpp:181-183, and its conversion to int8_t goes through float and
// truncates toward zero).  Values the language leaves undefined are defined here: beyond int8's range saturates,
// NaN gives 0.
__global__ void quantize_scale_trunc_kernel(const char* __restrict__ W, int64_t ldw, int rows, int cols, float scale,
                                            char* __restrict__ Wq, int64_t ldq) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < (int64_t)rows * cols;
         i += (int64_t)gridDim.x * blockDim.x) {
        const int r = (int)(i / cols), c = (int)(i % cols);
        const float w = from_bf16(*reinterpret_cast<const uint16_t*>(W + (int64_t)r * ldw + (int64_t)c * 2));
        const float t = from_bf16(to_bf16(w * scale));
        int q = 0;
        if (t == t) q = t >= 127.0f ? 127 : (t <= -128.0f ? -128 : (int)t);  // float -> int: toward zero
        Wq[(int64_t)r * ldq + c] = (char)q;
    }
}

int launch_quantize_scale_trunc(const void* W, int64_t ldw, int rows, int cols, float scale, void* Wq, int64_t ldq, hipStream_t st) {
    const int64_t n = (int64_t)rows * cols;
    int blocks = (int)((n + 255) / 256 < 4096 ? (n + 255) / 256 : 4096);
    if (blocks < 1) blocks = 1;
    hipLaunchKernelGGL(quantize_scale_trunc_kernel, dim3(blocks), dim3(256), 0, st, static_cast<const char*>(W), ldw, rows, cols,
                       scale, static_cast<char*>(Wq), ldq);
    return check_hip(hipGetLastError(), "quantize_scale_trunc_kernel launch");
}

// ---- packed int8 -> packed bf16 (exact) -------------------------------------------------------------
// int8 slot (panel, f, lane): 16 consecutive k of column n -> bf16 fragments 2f and 2f+1 ... the
// 16 k's starting at 32f + 16g split into two runs of 8: run h goes to bf16 fragment 2f+g,
// lane (n%32) + 32*h.
__global__ void dequant_packed_kernel(const char* __restrict__ in, char* __restrict__ out, int nfrag8, int nfrag16,
                                      int64_t total_slots) {
    const int64_t slot = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (slot >= total_slots) return;
    const int lane = (int)(slot & 63);
    const int64_t pf = slot >> 6;
    const int f = (int)(pf % nfrag8);
    const int64_t panel = pf / nfrag8;
    const uint4 v = *reinterpret_cast<const uint4*>(in + slot * 16);
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    const int g = lane >> 5, l32 = lane & 31;
#pragma unroll
    for (int h = 0; h < 2; h++) {
        alignas(16) uint16_t o[8];
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const int b = h * 8 + e;
            o[e] = to_bf16((float)(int8_t)((w[b >> 2] >> (8 * (b & 3))) & 0xff));
        }
        // the bf16 layout pads K to 64, the int8 one to 128: fragments past the bf16 padding hold only zeros
        if (2 * f + g < nfrag16) {
            const int64_t of = (panel * nfrag16 + 2 * f + g) * 64 + l32 + 32 * h;
            *reinterpret_cast<uint4*>(out + of * 16) = *reinterpret_cast<const uint4*>(o);
        }
    }
}

int launch_dequant_packed(const void* in, int K, int N, void* out, hipStream_t st) {
    const int nfrag8 = ((K + 127) / 128 * 128) / 32;
    const int nfrag16 = ((K + 63) / 64 * 64) / 16;
    const int64_t slots = (int64_t)((N + 31) / 32) * nfrag8 * 64;
    const int64_t blocks = (slots + 255) / 256;
    if (blocks > 0x7fffffff) return set_error(MMX_E_INVALID, "weight matrix too large");
    hipLaunchKernelGGL(dequant_packed_kernel, dim3((unsigned)blocks), dim3(256), 0, st, static_cast<const char*>(in),
                       static_cast<char*>(out), nfrag8, nfrag16, slots);
    return check_hip(hipGetLastError(), "dequant_packed_kernel launch");
}

// ---- c[M] = A[M,K] · b[K] ---------------------------------------------------------------------------
// amx_kernel::MatmulVector (include/kernels_amx.hpp:833-1043) and GemAvB (:1529-1618): one
// wavefront per row of A, lanes stride over K, wave reduction.
template <bool I8>
__global__ void matvec_kernel(const char* __restrict__ A, int64_t lda, const char* __restrict__ b, void* c, int M, int K) {
    const int row = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (row >= M) return;
    const char* a = A + (int64_t)row * lda;
    if (I8) {
        int acc = 0;
        for (int k = lane; k < K; k += 64) acc += (int)(int8_t)a[k] * (int)(int8_t)b[k];
        for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off);
        if (lane == 0) static_cast<int*>(c)[row] = acc;
    } else {
        float acc = 0.0f;
        for (int k = lane; k < K; k += 64)
            acc = __builtin_fmaf(from_bf16(reinterpret_cast<const uint16_t*>(a)[k]),
                                 from_bf16(reinterpret_cast<const uint16_t*>(b)[k]), acc);
        for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off);
        if (lane == 0) static_cast<float*>(c)[row] = acc;
    }
}

// The form for rows that are 16-byte aligned (the attention use: q against a cache of keys, one row per
// token, K = head size): LPR lanes share a row and fetch 16 bytes each, a wavefront covers 64/LPR rows at
// a time and UNR such groups per trip, so that every lane has UNR independent loads in flight.  Elements
// after the last whole 16 bytes of a row are added one by one.
template <bool I8, int LPR, int UNR>
__global__ void __launch_bounds__(256) matvec_rows_kernel(const char* __restrict__ A, int64_t lda, const char* __restrict__ b,
                                                          void* c, int M, int K) {
    constexpr int RPW = 64 / LPR, EPC = I8 ? 16 : 8;
    const int lane = threadIdx.x & 63, sub = lane % LPR, rsel = lane / LPR;
    const int64_t wave = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const int64_t nwaves = (int64_t)gridDim.x * (blockDim.x >> 6);
    const int nchunks = K / EPC;
    const uint4* bq = reinterpret_cast<const uint4*>(b);
    for (int64_t row0 = wave * (RPW * UNR); row0 < M; row0 += nwaves * (RPW * UNR)) {
        const char* a[UNR];
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
            const int64_t r = row0 + u * RPW + rsel;
            a[u] = A + (r < M ? r : (int64_t)M - 1) * lda;
        }
        float facc[UNR];
        int iacc[UNR];
#pragma unroll
        for (int u = 0; u < UNR; ++u) facc[u] = 0.0f, iacc[u] = 0;
        for (int ch = sub; ch < nchunks; ch += LPR) {
            const uint4 bv = bq[ch];
            uint4 av[UNR];
#pragma unroll
            for (int u = 0; u < UNR; ++u) {  // read once: keep the rows out of the way of what the caches hold
                typedef unsigned v4u __attribute__((ext_vector_type(4)));
                const v4u t = __builtin_nontemporal_load(reinterpret_cast<const v4u*>(a[u]) + ch);
                av[u] = make_uint4(t.x, t.y, t.z, t.w);
            }
#pragma unroll
            for (int u = 0; u < UNR; ++u) {
                const uint32_t aw[4] = {av[u].x, av[u].y, av[u].z, av[u].w}, bw[4] = {bv.x, bv.y, bv.z, bv.w};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    if (I8) {
                        iacc[u] = __builtin_amdgcn_sdot4((int)aw[i], (int)bw[i], iacc[u], false);
                    } else {
                        facc[u] = __builtin_fmaf(__uint_as_float(aw[i] << 16), __uint_as_float(bw[i] << 16), facc[u]);
                        facc[u] = __builtin_fmaf(__uint_as_float(aw[i] & 0xffff0000u), __uint_as_float(bw[i] & 0xffff0000u), facc[u]);
                    }
                }
            }
        }
        for (int k = nchunks * EPC + sub; k < K; k += LPR) {
#pragma unroll
            for (int u = 0; u < UNR; ++u) {
                if (I8)
                    iacc[u] += (int)(int8_t)a[u][k] * (int)(int8_t)b[k];
                else
                    facc[u] = __builtin_fmaf(from_bf16(reinterpret_cast<const uint16_t*>(a[u])[k]),
                                             from_bf16(reinterpret_cast<const uint16_t*>(b)[k]), facc[u]);
            }
        }
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
#pragma unroll
            for (int off = LPR / 2; off > 0; off >>= 1) {
                if (I8)
                    iacc[u] += __shfl_xor(iacc[u], off);
                else
                    facc[u] += __shfl_xor(facc[u], off);
            }
            const int64_t r = row0 + u * RPW + rsel;
            if (sub == 0 && r < M) {
                if (I8)
                    static_cast<int*>(c)[r] = iacc[u];
                else
                    static_cast<float*>(c)[r] = facc[u];
            }
        }
    }
}

template <bool I8, int LPR>
static void launch_matvec_rows(const void* A, int64_t lda, const void* b, void* c, int M, int K, hipStream_t st) {
    constexpr int UNR = 4, rows_per_block = 4 * (64 / LPR) * UNR;
    // one trip per wavefront: many short workgroups keep more requests in flight than a grid-stride loop does
    // (2^21 rows of 256 B: 6.9 TB/s against 6.4 with 4096 workgroups)
    const int64_t blocks = ((int64_t)M + rows_per_block - 1) / rows_per_block;
    hipLaunchKernelGGL((matvec_rows_kernel<I8, LPR, UNR>), dim3((unsigned)blocks), dim3(256), 0, st, static_cast<const char*>(A),
                       lda, static_cast<const char*>(b), c, M, K);
}

int launch_matvec(bool i8, const void* A, int64_t lda, const void* b, void* c, int M, int K, hipStream_t st) {
    if (M <= 0) return MMX_OK;
    const bool aligned = ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(b) | (uintptr_t)lda) & 15) == 0;
    const int nchunks = K / (i8 ? 16 : 8);
    if (aligned && nchunks > 0) {
        if (i8) {
            if (nchunks <= 4) launch_matvec_rows<true, 4>(A, lda, b, c, M, K, st);
            else if (nchunks <= 16) launch_matvec_rows<true, 16>(A, lda, b, c, M, K, st);
            else launch_matvec_rows<true, 64>(A, lda, b, c, M, K, st);
        } else {
            if (nchunks <= 4) launch_matvec_rows<false, 4>(A, lda, b, c, M, K, st);
            else if (nchunks <= 16) launch_matvec_rows<false, 16>(A, lda, b, c, M, K, st);
            else launch_matvec_rows<false, 64>(A, lda, b, c, M, K, st);
        }
        return check_hip(hipGetLastError(), "matvec_rows_kernel launch");
    }
    const int rows_per_block = 4;
    const int blocks = (M + rows_per_block - 1) / rows_per_block;
    if (i8)
        hipLaunchKernelGGL((matvec_kernel<true>), dim3(blocks), dim3(256), 0, st, static_cast<const char*>(A), lda,
                           static_cast<const char*>(b), c, M, K);
    else
        hipLaunchKernelGGL((matvec_kernel<false>), dim3(blocks), dim3(256), 0, st, static_cast<const char*>(A), lda,
                           static_cast<const char*>(b), c, M, K);
    return check_hip(hipGetLastError(), "matvec_kernel launch");
}

// ---- int4: per-column symmetric quantisation + packing in one pass per panel ---------------------------
// One workgroup per 32-column panel.  Phase 1: column maxima of |w|; phase 2: every thread builds one dword
// (8 values of one column) per fragment.  Not a hot path (done once per weight matrix).
template <bool TRANSPOSED>
__global__ __launch_bounds__(256) void quant4_pack_kernel(const char* W, int64_t ldw, int K, int N, char* out, int nfrag,
                                                          float* deq_out) {
    __shared__ float smax[8][32];
    __shared__ float sscale[32];
    const int t = threadIdx.x;
    const int n0 = blockIdx.x * 32;
    auto wval = [&](int k, int n) -> float {
        if (k >= K || n >= N) return 0.0f;
        const char* p = TRANSPOSED ? W + (int64_t)n * ldw + (int64_t)k * 2 : W + (int64_t)k * ldw + (int64_t)n * 2;
        return from_bf16(*reinterpret_cast<const uint16_t*>(p));
    };
    {
        const int c = t & 31, kr = t >> 5;
        float m = 0.0f;
        for (int k = kr; k < K; k += 8) m = fmaxf(m, fabsf(wval(k, n0 + c)));
        smax[kr][c] = m;
    }
    __syncthreads();
    if (t < 32) {
        float a = 0.0f;
#pragma unroll
        for (int r = 0; r < 8; r++) a = fmaxf(a, smax[r][t]);
        sscale[t] = a > 0.0f ? 7.0f / a : 0.0f;
        if (n0 + t < N) deq_out[n0 + t] = a / 7.0f;
    }
    __syncthreads();
    const int i = t & 3, c = (t >> 2) & 31, g = t >> 7;
    const float qs = sscale[c];
    for (int f = 0; f < nfrag; f++) {
        const int k0 = 64 * f + 32 * g + 8 * i;
        uint32_t d = 0;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            float q = rintf(wval(k0 + e, n0 + c) * qs);
            q = (q != q) ? 0.0f : q;  // a NaN weight, or an infinite one (its column's scale is then 0): quantised to 0
            q = fminf(fmaxf(q, -7.0f), 7.0f);
            d |= ((uint32_t)(int)q & 0xfu) << (4 * e);
        }
        *reinterpret_cast<uint32_t*>(out + ((int64_t)blockIdx.x * nfrag + f) * 1024 + t * 4) = d;
    }
}

int launch_quantize_pack_int4(const void* W, int64_t ldw, int K, int N, int transpose, void* packed, float* deq_out,
                              hipStream_t st) {
    const int nfrag = (K + 255) / 256 * 4;
    const int npanels = (N + 31) / 32;
    if (transpose)
        hipLaunchKernelGGL(quant4_pack_kernel<true>, dim3(npanels), dim3(256), 0, st, static_cast<const char*>(W), ldw, K, N,
                           static_cast<char*>(packed), nfrag, deq_out);
    else
        hipLaunchKernelGGL(quant4_pack_kernel<false>, dim3(npanels), dim3(256), 0, st, static_cast<const char*>(W), ldw, K, N,
                           static_cast<char*>(packed), nfrag, deq_out);
    return check_hip(hipGetLastError(), "quant4_pack_kernel launch");
}

}  // namespace mmx
