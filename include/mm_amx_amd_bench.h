/*
 * mm_amx_amd_bench.h — measurement aids of the gfx950 FC-GEMM path (same library, not part of the operator ABI).
 *
 * These entry points exist for benchmarks: they time launches with HIP events or run probe kernels, and two of
 * them block until the device has finished.  Nothing in the operator surface (mm_amx_amd.h) depends on them and
 * none of them has a counterpart in the reference, whose drivers time on the host (include/timeit.hpp).
 */
#ifndef MM_AMX_AMD_BENCH_H
#define MM_AMX_AMD_BENCH_H

#include "mm_amx_amd.h"

#ifdef __cplusplus
extern "C" {
#endif

/* HIP-event timing of `iters` back-to-back launches of the given gemm on `stream`, launch i
 * using the packed weights Bpacked_rot[i % n_rot] (rotate over several copies so that a
 * bandwidth-bound shape is not served from cache); returns the average milliseconds per launch
 * in *ms_out.  Other arguments as for mmx_gemm_splitk.  Blocks until the last launch has finished. */
int mmx_time_gemm(int a_dtype, int b_dtype, const void* A, int64_t lda_bytes, const void* const* Bpacked_rot, int n_rot,
                  int M, int K, int N, int n0, int n1, const mmx_epilogue* ep, int k_splits, void* workspace,
                  size_t workspace_bytes, void* stream, int iters, float* ms_out);

/* What an issue-bound loop of independent 32x32 MFMAs (dtype MMX_BF16 or MMX_I8) reaches on this device
 * right now, with all-zero operands (random_operands = 0) or with random ones (bf16: N(0,1) x N(0,0.02);
 * int8: uniform): *rate_out in Tflop/s or Top/s, *mhz_out the shader clock during the loop.  The clock of
 * this part under matrix load depends on the operand data; benchmarks report this next to a GEMM's rate.
 * scratch: 16 KiB of device memory.  Blocks until the loop has finished; not thread-safe. */
int mmx_probe_mfma(int dtype, int random_operands, int iters, void* scratch, void* stream, float* rate_out, float* mhz_out);

/* A kernel that does nothing but read: `workgroups` resident workgroups of waves_per_workgroup (4 or 8) wavefronts walk
 * `bytes` bytes at `buf` in equal contiguous shares (bytes must divide into shares of whole waves_per_workgroup KiB),
 * every wavefront keeping kib_in_flight (2, 4, 8, 16 or 32) KiB of nontemporal 16-byte loads outstanding as a rolling
 * window; blocked = 1 gives each wavefront a contiguous run of its workgroup's share (the pattern of the decode
 * kernels), 0 lets the wavefronts of a workgroup go side by side through it.  What the best of these takes is what a
 * decode kernel streaming the same number of weight bytes cannot beat.  sink: 4 bytes of device memory (never written
 * in practice; it keeps the loads alive).  Asynchronous on `stream`, allocates nothing, may be captured into a graph. */
int mmx_probe_read(const void* buf, size_t bytes, int workgroups, int waves_per_workgroup, int blocked, int kib_in_flight,
                   void* sink, void* stream);

#ifdef __cplusplus
}
#endif
#endif
