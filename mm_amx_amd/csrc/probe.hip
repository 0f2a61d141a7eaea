// Measurement aid: what an issue-bound loop of independent 32x32 MFMAs reaches on this device right now.
// On this part the shader clock under matrix load is set by power, and the power by the operand data: the
// same loop runs near 2.4 GHz on all-zero operands and near 1.8 GHz on random ones.  bench.py reports the
// figure next to the GEMM's rate, so that "fraction of the datasheet peak" can be read against what the
// matrix pipes deliver on comparable data with nothing else going on.
#include "common.hpp"

namespace mmx {

int check_hip(hipError_t e, const char* what);
int set_error(int code, const char* fmt, ...);

namespace {

__device__ __forceinline__ float lcg_normal(uint32_t& s) {  // roughly N(0,1): a scaled sum of four uniforms
    float t = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        s = s * 1664525u + 1013904223u;
        t += (float)(s >> 8) * (1.0f / 16777216.0f) - 0.5f;
    }
    return t * 1.732f;
}

// one wave per SIMD, twelve accumulators (the wave tile of the 256x192 GEMM kernel), operands fixed per lane;
// stamps[wave] = {shader cycles, 100 MHz wall ticks} of the loop
template <bool I8>
__global__ __launch_bounds__(256) void mfma_loop_kernel(uint64_t* stamps, int random_operands, int iters) {
    using accv = std::conditional_t<I8, i32x16, f32x16>;
    accv acc[12];
#pragma unroll
    for (int i = 0; i < 12; i++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[i][v] = 0;
    uint32_t s = (blockIdx.x * 256 + threadIdx.x) * 2654435761u + 12345u;
    u32x4 a[4], b[3];  // raw operand bits: 8 bf16 or 16 int8 per lane
#pragma unroll
    for (int i = 0; i < 7; i++) {
        u32x4 r = {0u, 0u, 0u, 0u};
        if (random_operands) {
#pragma unroll
            for (int d = 0; d < 4; d++) {
                if constexpr (I8) {  // uniform in [-127, 127]
                    uint32_t w = 0;
                    for (int e = 0; e < 4; e++) {
                        s = s * 1664525u + 1013904223u;
                        const int q = (int)((s >> 8) % 255u) - 127;
                        w |= (uint32_t)(q & 0xff) << (8 * e);
                    }
                    r[d] = w;
                } else {             // activations ~N(0,1), weights ~N(0,0.02)
                    const float sc = i < 4 ? 1.0f : 0.02f;
                    const uint32_t lo = __builtin_bit_cast(uint32_t, lcg_normal(s) * sc) >> 16;
                    const uint32_t hi = __builtin_bit_cast(uint32_t, lcg_normal(s) * sc) >> 16;
                    r[d] = lo | (hi << 16);
                }
            }
        }
        if (i < 4) a[i] = r;
        else b[i - 4] = r;
    }
    const uint64_t t0 = __builtin_readcyclecounter();
    const uint64_t w0 = wall_clock64();
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int t = 0; t < 12; t++) {
            if constexpr (I8)
                acc[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, b[t % 3]), __builtin_bit_cast(i32x4, a[t / 3]), acc[t], 0, 0, 0);
            else
                acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, b[t % 3]), __builtin_bit_cast(bf16x8, a[t / 3]), acc[t], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    const uint64_t t1 = __builtin_readcyclecounter();
    const uint64_t w1 = wall_clock64();
    float keep = 0.0f;  // the accumulators must stay live
#pragma unroll
    for (int i = 0; i < 12; i++)
#pragma unroll
        for (int v = 0; v < 16; v++) keep += (float)acc[i][v];
    const int wave = (blockIdx.x * 256 + threadIdx.x) >> 6;
    if ((threadIdx.x & 63) == 0) {
        stamps[wave * 2] = t1 - t0;
        stamps[wave * 2 + 1] = (w1 - w0) + (keep == 12345.678f ? 1 : 0);
    }
}


// A grid of resident workgroups that only reads: workgroup g walks the g-th of gridDim.x equal shares of the buffer with
// NW waves, each wave with U pieces of 1 KiB in flight as a rolling window: piece i + U is requested as soon as piece i
// has been consumed (one XOR per dword).  BLOCKED: wave w takes a contiguous run of the share (as the decode kernels'
// waves take runs of a panel's fragments); otherwise the waves go side by side (wave w: pieces w, w + NW, ...).
template <int U, int NW, bool BLOCKED>
__global__ __launch_bounds__(NW * 64) void read_stream_kernel(const char* buf, int pieces_per_wave, uint32_t* sink, uint32_t unlikely) {
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
    constexpr size_t STEP = BLOCKED ? 1024 : (size_t)NW * 1024;
    const char* p = buf + ((size_t)blockIdx.x * pieces_per_wave * NW + (BLOCKED ? (size_t)wave * pieces_per_wave : wave)) * 1024 + lane * 16;
    u32x4 w[U];
    uint32_t x = 0;
    const int last = pieces_per_wave - 1;
#pragma unroll
    for (int u = 0; u < U; u++) w[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p + (size_t)(u < last ? u : last) * STEP));
    for (int i0 = 0; i0 < pieces_per_wave; i0 += U) {
#pragma unroll
        for (int u = 0; u < U; u++) {
            x ^= w[u][0] ^ w[u][1] ^ w[u][2] ^ w[u][3];
            int nx = i0 + U + u;  // past the end: the last piece once more (it stays in the window, unused)
            nx = nx < last ? nx : last;
            w[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p + (size_t)nx * STEP));
        }
    }
#pragma unroll
    for (int u = 0; u < U; u++) x ^= w[u][0] & 1u;  // (the trailing requests must be waited for before the wave ends)
    if (x == unlikely) *sink = x;  // keeps the loads alive; one lane in 2^32 writes 4 harmless bytes
}

}  // namespace

// scratch: 1024 waves x 16 bytes on the device.  Synchronises the stream (it reads the stamps back).
int probe_mfma(bool i8, int random_operands, int iters, void* scratch, hipStream_t st, float* rate_out, float* mhz_out) {
    constexpr int grid = 256;  // one workgroup per CU
    uint64_t* d = static_cast<uint64_t*>(scratch);
    for (int rep = 0; rep < 2; rep++) {  // the first pass lets the clock settle on this data
        if (i8) hipLaunchKernelGGL(mfma_loop_kernel<true>, dim3(grid), dim3(256), 0, st, d, random_operands, iters);
        else hipLaunchKernelGGL(mfma_loop_kernel<false>, dim3(grid), dim3(256), 0, st, d, random_operands, iters);
    }
    int rc = check_hip(hipGetLastError(), "mfma_loop_kernel launch");
    if (rc) return rc;
    static uint64_t host[grid * 4 * 2];
    rc = check_hip(hipMemcpyAsync(host, d, sizeof host, hipMemcpyDeviceToHost, st), "hipMemcpyAsync");
    if (rc) return rc;
    rc = check_hip(hipStreamSynchronize(st), "hipStreamSynchronize");
    if (rc) return rc;
    double cyc = 0, wall = 0;
    for (int i = 0; i < grid * 4; i++) {
        cyc += (double)host[2 * i];
        wall += (double)host[2 * i + 1];
    }
    cyc /= grid * 4;
    wall /= grid * 4;
    if (wall <= 0) return set_error(MMX_E_HIP, "mmx_probe_mfma: the wall clock did not advance");
    const double us = wall / 100.0;  // wall_clock64 ticks at 100 MHz
    const double ops = 2.0 * 32 * 32 * (i8 ? 32 : 16) * 12.0 * iters * 4 * grid;
    *rate_out = (float)(ops / us / 1e6);  // Tflop/s or Top/s
    *mhz_out = (float)(cyc / us);
    return MMX_OK;
}

template <int NW, bool BLOCKED>
static int probe_read_launch(const char* b, int ppw, int workgroups, int kib, uint32_t* s, hipStream_t st) {
    switch (kib) {
    case 2: hipLaunchKernelGGL((read_stream_kernel<2, NW, BLOCKED>), dim3(workgroups), dim3(NW * 64), 0, st, b, ppw, s, 0x9e3779b9u); break;
    case 4: hipLaunchKernelGGL((read_stream_kernel<4, NW, BLOCKED>), dim3(workgroups), dim3(NW * 64), 0, st, b, ppw, s, 0x9e3779b9u); break;
    case 8: hipLaunchKernelGGL((read_stream_kernel<8, NW, BLOCKED>), dim3(workgroups), dim3(NW * 64), 0, st, b, ppw, s, 0x9e3779b9u); break;
    case 16: hipLaunchKernelGGL((read_stream_kernel<16, NW, BLOCKED>), dim3(workgroups), dim3(NW * 64), 0, st, b, ppw, s, 0x9e3779b9u); break;
    case 32: hipLaunchKernelGGL((read_stream_kernel<32, NW, BLOCKED>), dim3(workgroups), dim3(NW * 64), 0, st, b, ppw, s, 0x9e3779b9u); break;
    default: return set_error(MMX_E_INVALID, "mmx_probe_read: kib_in_flight is 2, 4, 8, 16 or 32");
    }
    return check_hip(hipGetLastError(), "read_stream_kernel launch");
}

int probe_read(const void* buf, size_t bytes, int workgroups, int waves, int blocked, int kib_in_flight, void* sink, hipStream_t st) {
    if (waves != 4 && waves != 8) return set_error(MMX_E_INVALID, "mmx_probe_read: waves_per_workgroup is 4 or 8");
    const size_t unit = (size_t)waves * 1024;
    const size_t per_wg = bytes / (size_t)workgroups;
    if (per_wg * workgroups != bytes || per_wg % unit || per_wg == 0 || per_wg / unit > (size_t)1 << 20)
        return set_error(MMX_E_INVALID, "mmx_probe_read: %zu bytes do not divide into %d shares of whole %zu KiB", bytes, workgroups, unit / 1024);
    const int ppw = (int)(per_wg / unit);
    const char* b = static_cast<const char*>(buf);
    uint32_t* s = static_cast<uint32_t*>(sink);
    if (waves == 8) return blocked ? probe_read_launch<8, true>(b, ppw, workgroups, kib_in_flight, s, st) : probe_read_launch<8, false>(b, ppw, workgroups, kib_in_flight, s, st);
    return blocked ? probe_read_launch<4, true>(b, ppw, workgroups, kib_in_flight, s, st) : probe_read_launch<4, false>(b, ppw, workgroups, kib_in_flight, s, st);
}

}  // namespace mmx
