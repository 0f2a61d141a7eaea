// Unsigned 8-bit operands of the int8 GEMM and mat-vec.
//
// Stands in for the uint8_t forms of amx_kernel::Matmul and amx_kernel::MatmulVector (tdpbusd / tdpbsud / tdpbuud,
// include/kernels_amx.hpp:1057-1101 and :839-850; accumulator type int32, :825).  The matrix cores of gfx950 multiply
// signed bytes only, so an unsigned operand is shifted: u = s + 128 with s = u ^ 0x80 read as a signed byte, and
//     (A' + 128 a) (B' + 128 b) = A' B' + 128 a colsum(B') + 128 b rowsum(A') + 16384 a b K       (a, b = 1 if unsigned)
// in int32 arithmetic modulo 2^32, which is what the AMX instructions accumulate in.  The shifted weights are made
// once by the repack (mmx_repack_b with MMX_U8 flips the sign bit of every byte on the way), the shifted activations
// per call into caller scratch; the signed GEMM then runs through the ordinary int8 kernels into an int32 scratch and
// a last pass adds the correction terms and applies the post-op.  None of the reference's drivers uses these forms
// (main.cpp:32-80), no benchmark configuration does, and they take two extra passes over C: written for exactness,
// not for speed.
#include "common.hpp"

namespace mmx {

// A (unsigned) -> A ^ 0x80 into `out` (row stride ldo; nothing is written when out is null) and the row sums of the
// signed values that the GEMM will see: one wave per row
__global__ __launch_bounds__(256) void u8_rows_kernel(const uint8_t* __restrict__ A, int64_t lda, int M, int K, int flip, int8_t* out,
                                                      int64_t ldo, int32_t* rowsum) {
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (row >= M) return;
    int sum = 0;
    for (int k = lane; k < K; k += 64) {
        const uint8_t v = (uint8_t)(A[(int64_t)row * lda + k] ^ (flip ? 0x80 : 0));
        if (out) out[(int64_t)row * ldo + k] = (int8_t)v;
        sum += (int)(int8_t)v;
    }
    for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
    if (lane == 0 && rowsum) rowsum[row] = sum;
}

// column sums of packed int8 weights over K, for columns [n0, n1): one thread per column, walking the column's
// 16-byte lane slots (packed[panel][f][lane][16 B], lane = n % 32 + 32 * half)
__global__ __launch_bounds__(256) void u8_colsum_kernel(const char* __restrict__ Wp, int64_t panel_stride, int nfrag, int n0, int n1,
                                                        int32_t* colsum) {
    const int n = n0 + blockIdx.x * 256 + threadIdx.x;
    if (n >= n1) return;
    const char* base = Wp + (int64_t)(n >> 5) * panel_stride + (n & 31) * 16;
    int sum = 0;
    for (int f = 0; f < nfrag; f++)
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const uint4 v = *reinterpret_cast<const uint4*>(base + (int64_t)f * 1024 + h * 512);
            const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int i = 0; i < 4; i++) sum = __builtin_amdgcn_sdot4((int)w[i], 0x01010101, sum, false);
        }
    colsum[n - n0] = sum;
}

// one element of the result: int32 sum + correction terms -> post-op -> C
__device__ __forceinline__ void u8_finish_one(const int32_t* __restrict__ acc, int64_t ldacc, const int32_t* rowsum, const int32_t* colsum,
                                              int32_t both_term, int m, int n, int n0, const Epilogue& ep) {
    uint32_t v = (uint32_t)acc[(int64_t)m * ldacc + n];
    if (colsum) v += 128u * (uint32_t)colsum[n - n0];
    if (rowsum) v += 128u * (uint32_t)rowsum[m];
    v += (uint32_t)both_term;
    const int32_t sum = (int32_t)v;
    char* row = ep.C + (int64_t)m * ep.ldc;
    if (ep.out_dtype == MMX_I32) {
        reinterpret_cast<int32_t*>(row)[n] = sum;
        return;
    }
    float r = (float)sum;  // vcvtdq2ps, round to nearest even (include/kernels_amx.hpp:631-634)
    if (ep.steps & MMX_PP_DEQUANT) r = r * (ep.deq_oc ? ep.deq_oc[n] : ep.deq);
    if (ep.steps & MMX_PP_BIAS) r = r + ep.bias[n];
    if (ep.steps & MMX_PP_GELU) r = gelu_erf_minimax(r);
    if (ep.steps & MMX_PP_QUANT) r = r * (ep.q_oc ? ep.q_oc[n] : ep.q);
    switch (ep.out_dtype) {
    case MMX_BF16: reinterpret_cast<uint16_t*>(row)[n] = to_bf16(r); break;
    case MMX_I8: reinterpret_cast<int8_t*>(row)[n] = to_s8_sat(r); break;
    default: reinterpret_cast<float*>(row)[n] = r; break;
    }
}

// acc (int32 [M, ld]) + correction terms -> post-op -> C: the steps and order of the tile kernels' store; a thread per
// column, rows blockIdx.y, blockIdx.y + gridDim.y, ... (the grid's second dimension holds 65535 at most)
__global__ __launch_bounds__(256) void u8_finish_kernel(const int32_t* __restrict__ acc, int64_t ldacc, const int32_t* rowsum,
                                                        const int32_t* colsum, int32_t both_term, int M, int n0, int n1,
                                                        const Epilogue ep) {
    const int n = n0 + blockIdx.x * 256 + threadIdx.x;
    if (n >= n1) return;
    for (int m = blockIdx.y; m < M; m += gridDim.y) u8_finish_one(acc, ldacc, rowsum, colsum, both_term, m, n, n0, ep);
}

// c[m] = sum_k A[m, k] b[k] with either operand signed or unsigned: one wave per row
template <bool AU, bool BU>
__global__ __launch_bounds__(256) void matvec_x8_kernel(const uint8_t* __restrict__ A, int64_t lda, const uint8_t* __restrict__ b,
                                                        int32_t* c, int M, int K) {
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (row >= M) return;
    uint32_t sum = 0;  // modulo 2^32, as the int32 accumulators of the AMX tiles
    for (int k = lane; k < K; k += 64) {
        const int a = AU ? (int)A[(int64_t)row * lda + k] : (int)(int8_t)A[(int64_t)row * lda + k];
        const int w = BU ? (int)b[k] : (int)(int8_t)b[k];
        sum += (uint32_t)(a * w);
    }
    for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
    if (lane == 0) c[row] = (int32_t)sum;
}

size_t u8_scratch_bytes(bool a_unsigned, int M, int K, int n1) {
    auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
    size_t total = up((size_t)M * n1 * 4) + up((size_t)M * 4) + up((size_t)n1 * 4);
    if (a_unsigned) total += up((size_t)M * (((size_t)K + 15) & ~(size_t)15));
    return total;
}

int launch_gemm_x8(bool a_unsigned, bool b_unsigned, const void* A, int64_t lda, const void* Bp, int M, int K, int N, int n0, int n1,
                   const Epilogue& ep, char* scratch, hipStream_t st,
                   int (*signed_gemm)(const void* A, int64_t lda, const void* Bp, int M, int K, int N, int n0, int n1, int32_t* acc,
                                      int64_t ldacc_bytes, hipStream_t st)) {
    auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
    int32_t* acc = reinterpret_cast<int32_t*>(scratch);
    int32_t* rowsum = reinterpret_cast<int32_t*>(scratch + up((size_t)M * n1 * 4));
    int32_t* colsum = reinterpret_cast<int32_t*>(reinterpret_cast<char*>(rowsum) + up((size_t)M * 4));
    int8_t* As = reinterpret_cast<int8_t*>(reinterpret_cast<char*>(colsum) + up((size_t)n1 * 4));
    const int64_t lds_ = ((int64_t)K + 15) & ~(int64_t)15;
    // the signed activations the GEMM will see, and their row sums (needed when the weights are unsigned)
    if (a_unsigned || b_unsigned)
        hipLaunchKernelGGL(u8_rows_kernel, dim3((M + 3) / 4), dim3(256), 0, st, static_cast<const uint8_t*>(A), lda, M, K, a_unsigned ? 1 : 0,
                           a_unsigned ? As : nullptr, lds_, b_unsigned ? rowsum : nullptr);
    const int kpad = (K + 127) / 128 * 128;
    if (a_unsigned)
        hipLaunchKernelGGL(u8_colsum_kernel, dim3((n1 - n0 + 255) / 256), dim3(256), 0, st, static_cast<const char*>(Bp), (int64_t)kpad * 32,
                           kpad / 32, n0, n1, colsum);
    int rc = check_hip(hipGetLastError(), "u8 preparation kernels launch");
    if (rc) return rc;
    rc = signed_gemm(a_unsigned ? static_cast<const void*>(As) : A, a_unsigned ? lds_ : lda, Bp, M, K, N, n0, n1, acc, (int64_t)n1 * 4, st);
    if (rc) return rc;
    const int32_t both = (a_unsigned && b_unsigned) ? (int32_t)(16384u * (uint32_t)K) : 0;
    hipLaunchKernelGGL(u8_finish_kernel, dim3((n1 - n0 + 255) / 256, M < 65535 ? M : 65535), dim3(256), 0, st, acc, (int64_t)n1, b_unsigned ? rowsum : nullptr,
                       a_unsigned ? colsum : nullptr, both, M, n0, n1, ep);
    return check_hip(hipGetLastError(), "u8_finish_kernel launch");
}

int launch_matvec_x8(bool a_unsigned, bool b_unsigned, const void* A, int64_t lda, const void* b, void* c, int M, int K, hipStream_t st) {
    const uint8_t* Ap = static_cast<const uint8_t*>(A);
    const uint8_t* bp = static_cast<const uint8_t*>(b);
    int32_t* cp = static_cast<int32_t*>(c);
    const dim3 grid((M + 3) / 4), block(256);
    if (a_unsigned && b_unsigned) hipLaunchKernelGGL((matvec_x8_kernel<true, true>), grid, block, 0, st, Ap, lda, bp, cp, M, K);
    else if (a_unsigned) hipLaunchKernelGGL((matvec_x8_kernel<true, false>), grid, block, 0, st, Ap, lda, bp, cp, M, K);
    else hipLaunchKernelGGL((matvec_x8_kernel<false, true>), grid, block, 0, st, Ap, lda, bp, cp, M, K);
    return check_hip(hipGetLastError(), "matvec_x8_kernel launch");
}

}  // namespace mmx
