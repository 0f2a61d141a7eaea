// C ABI of the gfx950 FC-GEMM path: argument validation, dispatch, error reporting.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <mutex>

#include "common.hpp"
#include "../../include/mm_amx_amd_bench.h"

namespace mmx {

static thread_local char g_err[512] = "";
static thread_local char g_kernel[128] = "";
static std::atomic<int> g_cus{0};
static std::mutex g_attr_mutex;

// The K-split workspace of callers that cannot allocate (mmx_gemm_splitk_static): arrival counters and partial
// tiles as in a caller's workspace, held by every GPU the library runs on until the process ends.  All zero when
// the code object is loaded; every completed call leaves the counters zero.  `static_ws` is the host-side stand-in
// of the array: its device address is taken once per device in mmx_init and only that address is ever used.
constexpr size_t STATIC_WS_BYTES = ((size_t)64 << 20) + ((size_t)16 << 10);
static __device__ __align__(256) unsigned char static_ws[STATIC_WS_BYTES];
constexpr int MAX_DEVICES = 64;
static std::atomic<char*> g_static_ws[MAX_DEVICES];

int set_error(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
    return code;
}

int check_hip(hipError_t e, const char* what) {
    if (e == hipSuccess) return MMX_OK;
    return set_error(MMX_E_HIP, "%s: %s", what, hipGetErrorString(e));
}

void note_kernel(const char* name) {
    strncpy(g_kernel, name, sizeof g_kernel - 1);
    g_kernel[sizeof g_kernel - 1] = 0;
}

int num_cus() {
    const int c = g_cus.load(std::memory_order_relaxed);
    return c > 0 ? c : 256;
}

int ensure_dynamic_lds(const void* kernel, int bytes, std::atomic<uint64_t>& done_on_device) {
    int dev = 0;
    int rc = check_hip(hipGetDevice(&dev), "hipGetDevice");
    if (rc) return rc;
    const uint64_t bit = 1ull << (dev & 63);
    if (done_on_device.load(std::memory_order_acquire) & bit) return MMX_OK;
    std::lock_guard<std::mutex> lock(g_attr_mutex);
    if (done_on_device.load(std::memory_order_relaxed) & bit) return MMX_OK;
    rc = check_hip(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes),
                   "hipFuncSetAttribute(MaxDynamicSharedMemorySize)");
    if (!rc) done_on_device.fetch_or(bit, std::memory_order_release);
    return rc;
}


size_t skinny_workspace_bytes(int wk, int M, int K, int n0, int n1);
int launch_gemm_tiles_bf16(const void* A, int64_t lda, const void* Bp, int M, int K, int N, int n0, int n1,
                           const Epilogue& ep, const SplitRequest& rq, hipStream_t st);
int launch_gemm_tiles_i8(const void* A, int64_t lda, const void* Bp, int M, int K, int N, int n0, int n1,
                         const Epilogue& ep, const SplitRequest& rq, hipStream_t st);
int launch_gemm_tiles_w8(const void* A, int64_t lda, const void* Bp, int M, int K, int N, int n0, int n1,
                         const Epilogue& ep, const SplitRequest& rq, hipStream_t st);
size_t plan_workspace_bytes(int elesz, bool w8, int M, int K, int Ncols, uint32_t steps, int k_splits);
bool skinny_i8_eligible(const void* x, int64_t ldx, int M, int K);
int launch_skinny(int wk, const void* x, int64_t ldx, const void* Wp, int M, int K, int N, int n0, int n1,
                  const Epilogue& ep, hipStream_t st, const SplitRequest* rq);
int launch_repack(int elesz, const void* B, int64_t ldb, int K, int N, int transpose, void* out, hipStream_t st, int flip);
size_t u8_scratch_bytes(bool a_unsigned, int M, int K, int n1);
int launch_gemm_x8(bool a_unsigned, bool b_unsigned, const void* A, int64_t lda, const void* Bp, int M, int K, int N, int n0, int n1,
                   const Epilogue& ep, char* scratch, hipStream_t st,
                   int (*signed_gemm)(const void* A, int64_t lda, const void* Bp, int M, int K, int N, int n0, int n1, int32_t* acc,
                                      int64_t ldacc_bytes, hipStream_t st));
int launch_matvec_x8(bool a_unsigned, bool b_unsigned, const void* A, int64_t lda, const void* b, void* c, int M, int K, hipStream_t st);
int launch_repack_gate_up(const void* wg, const void* wu, int64_t ldw, int K, int N, void* out, hipStream_t st);
int launch_quantize(const void* W, int64_t ldw, int rows, int cols, void* Wq, int64_t ldq, float* scales_out,
                    uint32_t* scratch, hipStream_t st);
int launch_quantize_scale_trunc(const void* W, int64_t ldw, int rows, int cols, float scale, void* Wq, int64_t ldq, hipStream_t st);
int launch_dequant_packed(const void* in, int K, int N, void* out, hipStream_t st);
int probe_mfma(bool i8, int random_operands, int iters, void* scratch, hipStream_t st, float* rate_out, float* mhz_out);
int launch_quantize_pack_int4(const void* W, int64_t ldw, int K, int N, int transpose, void* packed, float* deq_out,
                              hipStream_t st);
int probe_read(const void* buf, size_t bytes, int workgroups, int waves, int blocked, int kib_in_flight, void* sink, hipStream_t st);
int launch_matvec(bool i8, const void* A, int64_t lda, const void* b, void* c, int M, int K, hipStream_t st);

struct TileCfg {
    int bm, bn;
};
// tuning knobs: per thread, like the error string, so that one thread's choice never changes another's dispatch
static thread_local TileCfg g_forced = {0, 0};
static thread_local int g_load_mode = 2;
static thread_local int g_decode_halves = -1;
static thread_local int g_decode_valu = -1;
static thread_local int g_decode_resident = -1;
static thread_local int g_waves = 8;
static thread_local int g_decode_pair = 1;
TileCfg forced_tile() { return g_forced; }
int load_mode() { return g_load_mode; }
int decode_halves() { return g_decode_halves; }
int decode_valu() { return g_decode_valu; }
int decode_resident() { return g_decode_resident; }
int wave_count() { return g_waves; }
int decode_pair() { return g_decode_pair; }

static int elesz_of(int dtype) { return dtype == MMX_BF16 ? 2 : (dtype == MMX_I8 || dtype == MMX_U8) ? 1 : 0; }

static int out_size(int dtype) {
    switch (dtype) {
    case MMX_F32: case MMX_I32: return 4;
    case MMX_BF16: return 2;
    case MMX_I8: return 1;
    default: return 0;
    }
}

static int make_epilogue(const mmx_epilogue* in, int a_dtype, int b_dtype, int M, int n0, int n1, Epilogue* out) {
    if (!in) return set_error(MMX_E_INVALID, "epilogue descriptor is NULL");
    if (!in->C) return set_error(MMX_E_INVALID, "epilogue: output pointer C is NULL");
    const int sz = out_size(in->out_dtype);
    if (!sz) return set_error(MMX_E_INVALID, "epilogue: unknown output dtype %d", in->out_dtype);
    const uint32_t known = MMX_PP_DEQUANT | MMX_PP_BIAS | MMX_PP_GELU | MMX_PP_QUANT | MMX_PP_SILU_GATE;
    if (in->steps & ~known) return set_error(MMX_E_INVALID, "epilogue: unknown step bits 0x%x", in->steps);
    // the setters of BiasGeluStore assert that their step is enabled (include/kernels_amx.hpp:561-583);
    // here the converse is enforced: an enabled step must have its operand
    if ((in->steps & MMX_PP_BIAS) && !in->bias) return set_error(MMX_E_INVALID, "epilogue: BIAS step without a bias pointer");
    if (in->steps & MMX_PP_SILU_GATE) {
        // compressed weights need their scales before the non-linearity: DEQUANT (alone) may come with it
        if (in->steps & ~(uint32_t)(MMX_PP_SILU_GATE | MMX_PP_DEQUANT))
            return set_error(MMX_E_INVALID, "epilogue: SILU_GATE excludes every other step but DEQUANT");
        if (in->out_dtype != MMX_BF16 && in->out_dtype != MMX_F32)
            return set_error(MMX_E_INVALID, "epilogue: SILU_GATE stores bf16 or fp32");
        if (a_dtype != MMX_BF16) return set_error(MMX_E_INVALID, "epilogue: SILU_GATE needs bf16 activations");
        if (n0 % 64) return set_error(MMX_E_INVALID, "epilogue: SILU_GATE needs n0 %% 64 == 0");
    }
    if (in->out_dtype == MMX_I32 && !(a_dtype == MMX_I8 && b_dtype == MMX_I8 && in->steps == 0))
        return set_error(MMX_E_INVALID, "epilogue: int32 output is the raw accumulator of an int8 GEMM (steps must be 0)");
    if (in->ldc_bytes % sz) return set_error(MMX_E_INVALID, "epilogue: ldc_bytes %lld is not a multiple of the element size", (long long)in->ldc_bytes);
    if (reinterpret_cast<uintptr_t>(in->C) % sz) return set_error(MMX_E_INVALID, "epilogue: C is not aligned to its element size");
    // C points at column 0 of the full row: a row must hold the columns up to n1 (half of them with SILU_GATE),
    // or rows would overlap (a single row has no stride to speak of)
    const int64_t row_bytes = (int64_t)((in->steps & MMX_PP_SILU_GATE) ? n1 / 2 : n1) * sz;
    if (M > 1 && in->ldc_bytes < row_bytes)
        return set_error(MMX_E_INVALID, "epilogue: ldc_bytes %lld smaller than the %lld bytes of a row of C", (long long)in->ldc_bytes, (long long)row_bytes);
    out->steps = in->steps;
    out->out_dtype = in->out_dtype;
    out->C = static_cast<char*>(in->C);
    out->ldc = in->ldc_bytes;
    out->bias = in->bias;
    out->deq = in->deq_scale;
    out->deq_oc = in->deq_scale_per_oc;
    out->q = in->q_scale;
    out->q_oc = in->q_scale_per_oc;
    out->c_vec_ok = ((reinterpret_cast<uintptr_t>(in->C) & 15) == 0) && ((in->ldc_bytes & 15) == 0);
    return MMX_OK;
}

static int gemm_dispatch(int a_dtype, int b_dtype, const void* A, int64_t lda_bytes, const void* Bpacked, int M, int K,
                         int N, int n0, int n1, const mmx_epilogue* ep_in, const SplitRequest& rq, hipStream_t st) {
    if (!A || !Bpacked) return set_error(MMX_E_INVALID, "mmx_gemm: NULL operand");
    if (M <= 0 || K <= 0 || N <= 0) return set_error(MMX_E_INVALID, "mmx_gemm: M, K, N must be positive (got %d, %d, %d)", M, K, N);
    const bool bf = a_dtype == MMX_BF16 && b_dtype == MMX_BF16;
    const bool i8 = a_dtype == MMX_I8 && b_dtype == MMX_I8;
    const bool w8 = a_dtype == MMX_BF16 && b_dtype == MMX_I8;
    const bool w4 = a_dtype == MMX_BF16 && b_dtype == MMX_I4;
    if (!bf && !i8 && !w8 && !w4) return set_error(MMX_E_INVALID, "mmx_gemm: dtype pair (%d, %d) not supported", a_dtype, b_dtype);
    if (n0 < 0 || n1 > N || n0 >= n1) return set_error(MMX_E_INVALID, "mmx_gemm: column range [%d, %d) outside [0, %d)", n0, n1, N);
    // the reference splits N in units of 32 (main.cpp:461-471)
    if (n0 % 32) return set_error(MMX_E_INVALID, "mmx_gemm: n0 = %d must be a multiple of 32", n0);
    const int esa = elesz_of(a_dtype);
    if (lda_bytes < (int64_t)K * esa) return set_error(MMX_E_INVALID, "mmx_gemm: lda_bytes %lld smaller than a row of A", (long long)lda_bytes);
    if (lda_bytes % esa || reinterpret_cast<uintptr_t>(A) % esa) return set_error(MMX_E_INVALID, "mmx_gemm: A is not aligned to its element size");
    if (reinterpret_cast<uintptr_t>(Bpacked) & 15) return set_error(MMX_E_INVALID, "mmx_gemm: packed weights must be 16-byte aligned");
    Epilogue ep;
    int rc = make_epilogue(ep_in, a_dtype, b_dtype, M, n0, n1, &ep);
    if (rc) return rc;
    if (rq.k_splits < 0) return set_error(MMX_E_INVALID, "mmx_gemm: k_splits = %d", rq.k_splits);
    if (rq.ws && (reinterpret_cast<uintptr_t>(rq.ws) & 255)) return set_error(MMX_E_INVALID, "mmx_gemm: the workspace must be 256-byte aligned");
    // the decode kernels choose their own K split (the chunked form, given a workspace); they take no count of slices
    const bool decode = (M <= 32 && !i8) || (i8 && skinny_i8_eligible(A, lda_bytes, M, K) && forced_tile().bm == 0);
    if (decode && rq.k_splits > 1) return set_error(MMX_E_UNSUPPORTED, "mmx_gemm: the decode kernels (M <= 32) take k_splits = 0 or 1, not a count of slices");
    if ((ep.steps & MMX_PP_SILU_GATE) && ((n1 - n0) % 64)) return set_error(MMX_E_INVALID, "mmx_gemm: SILU_GATE needs (n1 - n0) %% 64 == 0");
    if (M <= 32 && !i8) return launch_skinny(w4 ? 2 : (w8 ? 1 : 0), A, lda_bytes, Bpacked, M, K, N, n0, n1, ep, st, &rq);
    if (i8 && skinny_i8_eligible(A, lda_bytes, M, K) && forced_tile().bm == 0)
        return launch_skinny(3, A, lda_bytes, Bpacked, M, K, N, n0, n1, ep, st, &rq);
    if (w4) return set_error(MMX_E_UNSUPPORTED, "mmx_gemm: bf16 x int4-weight is a decode path (M <= 32)");
    if (w8) return launch_gemm_tiles_w8(A, lda_bytes, Bpacked, M, K, N, n0, n1, ep, rq, st);
    return i8 ? launch_gemm_tiles_i8(A, lda_bytes, Bpacked, M, K, N, n0, n1, ep, rq, st)
              : launch_gemm_tiles_bf16(A, lda_bytes, Bpacked, M, K, N, n0, n1, ep, rq, st);
}

// the signed int8 GEMM into raw int32 accumulators (the middle pass of mmx_gemm_u8)
static int signed_gemm_i32(const void* A, int64_t lda, const void* Bp, int M, int K, int N, int n0, int n1, int32_t* acc,
                           int64_t ldacc_bytes, hipStream_t st) {
    mmx_epilogue e;
    memset(&e, 0, sizeof e);
    e.steps = MMX_PP_NONE;
    e.out_dtype = MMX_I32;
    e.C = acc;
    e.ldc_bytes = ldacc_bytes;
    const SplitRequest none = {1, nullptr, 0};
    return gemm_dispatch(MMX_I8, MMX_I8, A, lda, Bp, M, K, N, n0, n1, &e, none, st);
}

}  // namespace mmx

using namespace mmx;

extern "C" {

const char* mmx_last_error(void) { return g_err; }
const char* mmx_last_kernel(void) { return g_kernel; }

int mmx_init(int device) {
    int count = 0;
    int rc = check_hip(hipGetDeviceCount(&count), "hipGetDeviceCount");
    if (rc) return rc;
    if (device < 0 || device >= count) return set_error(MMX_E_DEVICE, "mmx_init: device %d of %d", device, count);
    rc = check_hip(hipSetDevice(device), "hipSetDevice");
    if (rc) return rc;
    hipDeviceProp_t prop;
    rc = check_hip(hipGetDeviceProperties(&prop, device), "hipGetDeviceProperties");
    if (rc) return rc;
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return set_error(MMX_E_DEVICE, "mmx_init: device %d is %s, this library holds gfx950 code only", device, prop.gcnArchName);
    g_cus = prop.multiProcessorCount;
    if (device < MAX_DEVICES && !g_static_ws[device].load(std::memory_order_acquire)) {
        void* p = nullptr;  // this device's copy of the array (each GPU has its own, at its own address)
        rc = check_hip(hipGetSymbolAddress(&p, HIP_SYMBOL(static_ws)), "hipGetSymbolAddress(static workspace)");
        if (rc) return rc;
        g_static_ws[device].store(static_cast<char*>(p), std::memory_order_release);
    }
    return MMX_OK;
}

size_t mmx_packed_b_bytes(int dtype, int K, int N) {
    if (dtype == MMX_I4) {  // 1 KiB fragments of 32 columns x 64 of k, four fragments at a time
        if (K <= 0 || N <= 0) return 0;
        return (size_t)((N + 31) / 32) * ((size_t)(K + 255) / 256 * 4) * 1024;
    }
    const int es = elesz_of(dtype);
    if (!es || K <= 0 || N <= 0) return 0;
    const size_t kpad_bytes = ((size_t)K * es + 127) / 128 * 128;
    return (size_t)((N + 31) / 32) * 32 * kpad_bytes;
}

int mmx_repack_b(int dtype, const void* B, int64_t ldb_bytes, int K, int N, int transpose, void* packed, void* stream) {
    const int es = elesz_of(dtype);
    if (!es) return set_error(MMX_E_INVALID, "mmx_repack_b: dtype %d is neither bf16 nor (u)int8", dtype);
    if (!B || !packed) return set_error(MMX_E_INVALID, "mmx_repack_b: NULL pointer");
    if (K <= 0 || N <= 0) return set_error(MMX_E_INVALID, "mmx_repack_b: K and N must be positive");
    const int64_t min_ld = (int64_t)(transpose ? K : N) * es;
    if (ldb_bytes < min_ld || ldb_bytes % es) return set_error(MMX_E_INVALID, "mmx_repack_b: ldb_bytes %lld too small or misaligned", (long long)ldb_bytes);
    if (reinterpret_cast<uintptr_t>(packed) & 15) return set_error(MMX_E_INVALID, "mmx_repack_b: packed buffer must be 16-byte aligned");
    return launch_repack(es, B, ldb_bytes, K, N, transpose, packed, static_cast<hipStream_t>(stream), dtype == MMX_U8 ? 1 : 0);
}

int mmx_repack_gate_up(const void* w_gate, const void* w_up, int64_t ldw_bytes, int K, int N, void* packed, void* stream) {
    if (!w_gate || !w_up || !packed) return set_error(MMX_E_INVALID, "mmx_repack_gate_up: NULL pointer");
    // AMX_MLP::Linear::setup asserts N % 32 == 0 (tests/amx-mlp.cpp:552)
    if (K <= 0 || N <= 0 || N % 32) return set_error(MMX_E_INVALID, "mmx_repack_gate_up: N = %d must be a positive multiple of 32", N);
    if (ldw_bytes < (int64_t)K * 2 || ldw_bytes % 2) return set_error(MMX_E_INVALID, "mmx_repack_gate_up: ldw_bytes too small or odd");
    if (reinterpret_cast<uintptr_t>(packed) & 15) return set_error(MMX_E_INVALID, "mmx_repack_gate_up: packed buffer must be 16-byte aligned");
    return launch_repack_gate_up(w_gate, w_up, ldw_bytes, K, N, packed, static_cast<hipStream_t>(stream));
}

int mmx_quantize_weights(const void* W, int64_t ldw_bytes, int rows, int cols, void* Wq, int64_t ldq_bytes, float* scales_out,
                         uint32_t* absmax_scratch, void* stream) {
    if (!W || !Wq || !scales_out || !absmax_scratch) return set_error(MMX_E_INVALID, "mmx_quantize_weights: NULL pointer");
    if (rows <= 0 || cols <= 0 || ldw_bytes < (int64_t)cols * 2 || ldq_bytes < cols)
        return set_error(MMX_E_INVALID, "mmx_quantize_weights: bad shape or stride");
    if ((ldw_bytes & 1) || (reinterpret_cast<uintptr_t>(W) & 1) || (reinterpret_cast<uintptr_t>(scales_out) & 3) ||
        (reinterpret_cast<uintptr_t>(absmax_scratch) & 3))
        return set_error(MMX_E_INVALID, "mmx_quantize_weights: W, scales_out or absmax_scratch is not aligned to its element size");
    return launch_quantize(W, ldw_bytes, rows, cols, Wq, ldq_bytes, scales_out, absmax_scratch, static_cast<hipStream_t>(stream));
}

int mmx_quantize_weights_scaled(const void* W, int64_t ldw_bytes, int rows, int cols, float scale, void* Wq, int64_t ldq_bytes,
                                void* stream) {
    if (!W || !Wq) return set_error(MMX_E_INVALID, "mmx_quantize_weights_scaled: NULL pointer");
    if (rows <= 0 || cols <= 0 || ldw_bytes < (int64_t)cols * 2 || ldq_bytes < cols)
        return set_error(MMX_E_INVALID, "mmx_quantize_weights_scaled: bad shape or stride");
    if ((ldw_bytes & 1) || (reinterpret_cast<uintptr_t>(W) & 1))
        return set_error(MMX_E_INVALID, "mmx_quantize_weights_scaled: W is not aligned to its element size");
    return launch_quantize_scale_trunc(W, ldw_bytes, rows, cols, scale, Wq, ldq_bytes, static_cast<hipStream_t>(stream));
}

int mmx_quantize_pack_int4(const void* W, int64_t ldw_bytes, int K, int N, int transpose, void* packed, float* deq_scales_out,
                           void* stream) {
    if (!W || !packed || !deq_scales_out) return set_error(MMX_E_INVALID, "mmx_quantize_pack_int4: NULL pointer");
    if (K <= 0 || N <= 0) return set_error(MMX_E_INVALID, "mmx_quantize_pack_int4: K and N must be positive");
    const int64_t min_ld = (int64_t)(transpose ? K : N) * 2;
    if (ldw_bytes < min_ld || ldw_bytes % 2) return set_error(MMX_E_INVALID, "mmx_quantize_pack_int4: ldw_bytes %lld too small or odd", (long long)ldw_bytes);
    if (reinterpret_cast<uintptr_t>(W) & 1) return set_error(MMX_E_INVALID, "mmx_quantize_pack_int4: W is not aligned to its element size");
    if (reinterpret_cast<uintptr_t>(packed) & 15) return set_error(MMX_E_INVALID, "mmx_quantize_pack_int4: packed buffer must be 16-byte aligned");
    return launch_quantize_pack_int4(W, ldw_bytes, K, N, transpose, packed, deq_scales_out, static_cast<hipStream_t>(stream));
}

int mmx_dequant_packed(const void* packed_i8, int K, int N, void* packed_bf16, void* stream) {
    if (!packed_i8 || !packed_bf16 || K <= 0 || N <= 0) return set_error(MMX_E_INVALID, "mmx_dequant_packed: bad argument");
    if ((reinterpret_cast<uintptr_t>(packed_i8) | reinterpret_cast<uintptr_t>(packed_bf16)) & 15)
        return set_error(MMX_E_INVALID, "mmx_dequant_packed: buffers must be 16-byte aligned");
    return launch_dequant_packed(packed_i8, K, N, packed_bf16, static_cast<hipStream_t>(stream));
}

int mmx_gemm(int a_dtype, int b_dtype, const void* A, int64_t lda_bytes, const void* Bpacked, int M, int K, int N, int n0,
             int n1, const mmx_epilogue* ep, void* stream) {
    const SplitRequest none = {1, nullptr, 0};
    return gemm_dispatch(a_dtype, b_dtype, A, lda_bytes, Bpacked, M, K, N, n0, n1, ep, none, static_cast<hipStream_t>(stream));
}

int mmx_gemm_splitk(int a_dtype, int b_dtype, const void* A, int64_t lda_bytes, const void* Bpacked, int M, int K, int N, int n0,
                    int n1, const mmx_epilogue* ep, int k_splits, void* workspace, size_t workspace_bytes, void* stream) {
    if (!workspace && k_splits > 1) return set_error(MMX_E_INVALID, "mmx_gemm_splitk: %d K slices need a workspace", k_splits);
    const SplitRequest rq = {workspace ? k_splits : 1, static_cast<char*>(workspace), workspace_bytes};
    return gemm_dispatch(a_dtype, b_dtype, A, lda_bytes, Bpacked, M, K, N, n0, n1, ep, rq, static_cast<hipStream_t>(stream));
}

int mmx_gemm_splitk_static(int a_dtype, int b_dtype, const void* A, int64_t lda_bytes, const void* Bpacked, int M, int K, int N,
                           int n0, int n1, const mmx_epilogue* ep, int k_splits, void* stream) {
    int dev = 0;
    int rc = check_hip(hipGetDevice(&dev), "hipGetDevice");
    if (rc) return rc;
    char* ws = dev < MAX_DEVICES ? g_static_ws[dev].load(std::memory_order_acquire) : nullptr;
    if (!ws) return set_error(MMX_E_INVALID, "mmx_gemm_splitk_static: call mmx_init(%d) first (it takes the address of this device's workspace)", dev);
    if (k_splits > 1 && M > 32) {
        const size_t need = mmx_gemm_workspace_bytes(a_dtype, b_dtype, M, K, N, n0, n1, ep ? ep->steps : 0, k_splits);
        if (need > STATIC_WS_BYTES)
            return set_error(MMX_E_INVALID, "mmx_gemm_splitk_static: %d K slices of this shape need %zu bytes of workspace, the built-in one holds %zu",
                             k_splits, need, STATIC_WS_BYTES);
    }
    const SplitRequest rq = {k_splits, ws, STATIC_WS_BYTES};
    return gemm_dispatch(a_dtype, b_dtype, A, lda_bytes, Bpacked, M, K, N, n0, n1, ep, rq, static_cast<hipStream_t>(stream));
}

size_t mmx_gemm_workspace_bytes(int a_dtype, int b_dtype, int M, int K, int N, int n0, int n1, uint32_t steps, int k_splits) {
    const bool bf = a_dtype == MMX_BF16 && b_dtype == MMX_BF16, i8 = a_dtype == MMX_I8 && b_dtype == MMX_I8;
    const bool w8 = a_dtype == MMX_BF16 && b_dtype == MMX_I8;
    const bool w4 = a_dtype == MMX_BF16 && b_dtype == MMX_I4;
    if (M > 0 && M <= 32 && (bf || w8 || i8 || w4) && K > 0 && N > 0 && n0 >= 0 && n1 <= N && n0 < n1)
        return k_splits == 0 && !(steps & MMX_PP_SILU_GATE) ? skinny_workspace_bytes(i8 ? 3 : (w4 ? 2 : (w8 ? 1 : 0)), M, K, n0, n1) : 0;
    if ((!bf && !i8 && !w8) || M <= 32 || K <= 0 || N <= 0 || n0 < 0 || n1 > N || n0 >= n1 || k_splits < 0) return 0;
    return plan_workspace_bytes(i8 ? 1 : 2, w8, M, K, n1 - n0, steps, k_splits);
}

int mmx_matvec(int dtype, const void* A, int64_t lda_bytes, const void* b, void* c, int M, int K, void* stream) {
    const int es = elesz_of(dtype);
    if (dtype == MMX_U8) return set_error(MMX_E_INVALID, "mmx_matvec: unsigned operands go through mmx_matvec_u8");
    if (!es) return set_error(MMX_E_INVALID, "mmx_matvec: dtype %d is neither bf16 nor int8", dtype);
    if (!A || !b || !c || M <= 0 || K <= 0) return set_error(MMX_E_INVALID, "mmx_matvec: bad argument");
    if (lda_bytes < (int64_t)K * es) return set_error(MMX_E_INVALID, "mmx_matvec: lda_bytes smaller than a row of A");
    if (lda_bytes % es || (reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(b)) % es || reinterpret_cast<uintptr_t>(c) % 4)
        return set_error(MMX_E_INVALID, "mmx_matvec: A, b or c is not aligned to its element size");
    return launch_matvec(dtype == MMX_I8, A, lda_bytes, b, c, M, K, static_cast<hipStream_t>(stream));
}

size_t mmx_gemm_u8_scratch_bytes(int a_dtype, int b_dtype, int M, int K, int N, int n0, int n1) {
    const bool au = a_dtype == MMX_U8, bu = b_dtype == MMX_U8;
    if ((!au && a_dtype != MMX_I8) || (!bu && b_dtype != MMX_I8) || (!au && !bu)) return 0;
    if (M <= 0 || K <= 0 || N <= 0 || n0 < 0 || n1 > N || n0 >= n1) return 0;
    return u8_scratch_bytes(au, M, K, n1);
}

int mmx_gemm_u8(int a_dtype, int b_dtype, const void* A, int64_t lda_bytes, const void* Bpacked, int M, int K, int N, int n0, int n1,
                const mmx_epilogue* ep_in, void* scratch, size_t scratch_bytes, void* stream) {
    const bool au = a_dtype == MMX_U8, bu = b_dtype == MMX_U8;
    if ((!au && a_dtype != MMX_I8) || (!bu && b_dtype != MMX_I8) || (!au && !bu))
        return set_error(MMX_E_INVALID, "mmx_gemm_u8: dtypes (%d, %d): each MMX_I8 or MMX_U8, at least one unsigned", a_dtype, b_dtype);
    if (!A || !Bpacked || !scratch) return set_error(MMX_E_INVALID, "mmx_gemm_u8: NULL operand or scratch");
    if (M <= 0 || K <= 0 || N <= 0) return set_error(MMX_E_INVALID, "mmx_gemm_u8: M, K, N must be positive");
    if (n0 < 0 || n1 > N || n0 >= n1 || n0 % 32) return set_error(MMX_E_INVALID, "mmx_gemm_u8: column range [%d, %d) (n0 a multiple of 32) outside [0, %d)", n0, n1, N);
    if (lda_bytes < K) return set_error(MMX_E_INVALID, "mmx_gemm_u8: lda_bytes smaller than a row of A");
    if (reinterpret_cast<uintptr_t>(scratch) & 255) return set_error(MMX_E_INVALID, "mmx_gemm_u8: the scratch must be 256-byte aligned");
    const size_t need = u8_scratch_bytes(au, M, K, n1);
    if (scratch_bytes < need) return set_error(MMX_E_INVALID, "mmx_gemm_u8: %zu bytes of scratch, %zu needed", scratch_bytes, need);
    Epilogue ep;
    // the post-op is checked as for a signed int8 GEMM (raw int32 output only with steps == 0)
    int rc = make_epilogue(ep_in, MMX_I8, MMX_I8, M, n0, n1, &ep);
    if (rc) return rc;
    if (ep.steps & MMX_PP_SILU_GATE) return set_error(MMX_E_INVALID, "mmx_gemm_u8: SILU_GATE needs bf16 activations");
    return launch_gemm_x8(au, bu, A, lda_bytes, Bpacked, M, K, N, n0, n1, ep, static_cast<char*>(scratch), static_cast<hipStream_t>(stream),
                          signed_gemm_i32);
}

int mmx_matvec_u8(int a_dtype, int b_dtype, const void* A, int64_t lda_bytes, const void* b, void* c, int M, int K, void* stream) {
    const bool au = a_dtype == MMX_U8, bu = b_dtype == MMX_U8;
    if ((!au && a_dtype != MMX_I8) || (!bu && b_dtype != MMX_I8) || (!au && !bu))
        return set_error(MMX_E_INVALID, "mmx_matvec_u8: dtypes (%d, %d): each MMX_I8 or MMX_U8, at least one unsigned", a_dtype, b_dtype);
    if (!A || !b || !c || M <= 0 || K <= 0) return set_error(MMX_E_INVALID, "mmx_matvec_u8: bad argument");
    if (lda_bytes < K) return set_error(MMX_E_INVALID, "mmx_matvec_u8: lda_bytes smaller than a row of A");
    if (reinterpret_cast<uintptr_t>(c) % 4) return set_error(MMX_E_INVALID, "mmx_matvec_u8: c is not aligned to its element size");
    return launch_matvec_x8(au, bu, A, lda_bytes, b, c, M, K, static_cast<hipStream_t>(stream));
}

int mmx_mlp(const void* x, int64_t ldx_bytes, const void* w_gate_up, const void* w_down, void* h, int64_t ldh_bytes, void* y,
            int64_t ldy_bytes, int M, int K, int N, void* stream) {
    return mmx_mlp_splitk(x, ldx_bytes, w_gate_up, w_down, h, ldh_bytes, y, ldy_bytes, M, K, N, 1, nullptr, 0, stream);
}

int mmx_mlp_splitk(const void* x, int64_t ldx_bytes, const void* w_gate_up, const void* w_down, void* h, int64_t ldh_bytes, void* y,
                   int64_t ldy_bytes, int M, int K, int N, int down_k_splits, void* workspace, size_t workspace_bytes, void* stream) {
    if (!x || !w_gate_up || !w_down || !h || !y) return set_error(MMX_E_INVALID, "mmx_mlp: NULL pointer");
    if (N % 32) return set_error(MMX_E_INVALID, "mmx_mlp: N = %d must be a multiple of 32", N);
    mmx_epilogue e1;
    memset(&e1, 0, sizeof e1);
    e1.steps = MMX_PP_SILU_GATE;
    e1.out_dtype = MMX_BF16;
    e1.C = h;
    e1.ldc_bytes = ldh_bytes;
    int rc = mmx_gemm(MMX_BF16, MMX_BF16, x, ldx_bytes, w_gate_up, M, K, 2 * N, 0, 2 * N, &e1, stream);
    if (rc) return rc;
    mmx_epilogue e2;
    memset(&e2, 0, sizeof e2);
    e2.steps = MMX_PP_NONE;
    e2.out_dtype = MMX_BF16;
    e2.C = y;
    e2.ldc_bytes = ldy_bytes;
    // AMX_MLP::MLP::setup builds `down` with do_splitK (tests/amx-mlp.cpp:768): two halves of its K blocks, summed
    // and rounded to bf16 by the half that finishes last (:648-682).  The decode kernels (M <= 32) sum K inside one
    // workgroup per panel or in slices of their own choosing (never a given count).
    if (!workspace || (M <= 32 && down_k_splits == 1))
        return mmx_gemm(MMX_BF16, MMX_BF16, h, ldh_bytes, w_down, M, N, K, 0, K, &e2, stream);
    if (M <= 32) down_k_splits = 0;
    return mmx_gemm_splitk(MMX_BF16, MMX_BF16, h, ldh_bytes, w_down, M, N, K, 0, K, &e2, down_k_splits, workspace, workspace_bytes, stream);
}

int mmx_set_tile(const char* shape) {
    if (!shape || !*shape) { g_forced = {0, 0}; return MMX_OK; }
    int bm = 0, bn = 0;
    if (sscanf(shape, "%dx%d", &bm, &bn) != 2) return set_error(MMX_E_INVALID, "mmx_set_tile: cannot parse '%s'", shape);
    if (!((bm == 256 && (bn == 256 || bn == 192)) || (bm == 128 && (bn == 256 || bn == 192 || bn == 128 || bn == 64)) || (bm == 64 && bn == 128)))
        return set_error(MMX_E_INVALID, "mmx_set_tile: no kernel for %dx%d", bm, bn);
    g_forced = {bm, bn};
    return MMX_OK;
}

int mmx_set_option(const char* name, int value) {
    if (name && !strcmp(name, "load_mode")) {
        if (value != 0 && value != 2) return set_error(MMX_E_INVALID, "mmx_set_option: load_mode is 0 or 2");
        g_load_mode = value;
        return MMX_OK;
    }
    if (name && !strcmp(name, "decode_halves")) {
        if (value < -1 || value > 1) return set_error(MMX_E_INVALID, "mmx_set_option: decode_halves is -1, 0 or 1");
        g_decode_halves = value;
        return MMX_OK;
    }
    if (name && !strcmp(name, "decode_valu")) {
        if (value < -1 || value > 1) return set_error(MMX_E_INVALID, "mmx_set_option: decode_valu is -1, 0 or 1");
        g_decode_valu = value;
        return MMX_OK;
    }
    if (name && !strcmp(name, "decode_resident")) {
        if (value < -1 || value > 1) return set_error(MMX_E_INVALID, "mmx_set_option: decode_resident is -1, 0 or 1");
        g_decode_resident = value;
        return MMX_OK;
    }
    if (name && !strcmp(name, "decode_pair")) {
        if (value != 0 && value != 1) return set_error(MMX_E_INVALID, "mmx_set_option: decode_pair is 0 or 1");
        g_decode_pair = value;
        return MMX_OK;
    }
    if (name && !strcmp(name, "waves")) {
        if (value != 4 && value != 8) return set_error(MMX_E_INVALID, "mmx_set_option: waves is 4 or 8");
        g_waves = value;
        return MMX_OK;
    }
    return set_error(MMX_E_INVALID, "mmx_set_option: unknown option");
}

int mmx_probe_mfma(int dtype, int random_operands, int iters, void* scratch, void* stream, float* rate_out, float* mhz_out) {
    if ((dtype != MMX_BF16 && dtype != MMX_I8) || iters <= 0 || !scratch || !rate_out || !mhz_out)
        return set_error(MMX_E_INVALID, "mmx_probe_mfma: bad argument");
    return probe_mfma(dtype == MMX_I8, random_operands, iters, scratch, static_cast<hipStream_t>(stream), rate_out, mhz_out);
}

int mmx_probe_read(const void* buf, size_t bytes, int workgroups, int waves_per_workgroup, int blocked, int kib_in_flight, void* sink,
                   void* stream) {
    if (!buf || !sink || workgroups <= 0 || workgroups > 65536 || (reinterpret_cast<uintptr_t>(buf) & 15))
        return set_error(MMX_E_INVALID, "mmx_probe_read: bad argument");
    return probe_read(buf, bytes, workgroups, waves_per_workgroup, blocked, kib_in_flight, sink, static_cast<hipStream_t>(stream));
}

int mmx_time_gemm(int a_dtype, int b_dtype, const void* A, int64_t lda_bytes, const void* const* Bpacked_rot, int n_rot, int M,
                  int K, int N, int n0, int n1, const mmx_epilogue* ep, int k_splits, void* workspace, size_t workspace_bytes,
                  void* stream, int iters, float* ms_out) {
    if (!Bpacked_rot || n_rot <= 0 || iters <= 0 || !ms_out) return set_error(MMX_E_INVALID, "mmx_time_gemm: bad argument");
    const SplitRequest rq = {workspace ? k_splits : 1, static_cast<char*>(workspace), workspace_bytes};
    hipStream_t st = static_cast<hipStream_t>(stream);
    hipEvent_t e0, e1;
    int rc = check_hip(hipEventCreate(&e0), "hipEventCreate");
    if (rc) return rc;
    rc = check_hip(hipEventCreate(&e1), "hipEventCreate");
    if (rc) { (void)hipEventDestroy(e0); return rc; }
    rc = check_hip(hipEventRecord(e0, st), "hipEventRecord");
    for (int i = 0; i < iters && !rc; i++)
        rc = gemm_dispatch(a_dtype, b_dtype, A, lda_bytes, Bpacked_rot[i % n_rot], M, K, N, n0, n1, ep, rq, st);
    if (!rc) rc = check_hip(hipEventRecord(e1, st), "hipEventRecord");
    if (!rc) rc = check_hip(hipEventSynchronize(e1), "hipEventSynchronize");
    float ms = 0.0f;
    if (!rc) rc = check_hip(hipEventElapsedTime(&ms, e0, e1), "hipEventElapsedTime");
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (!rc) *ms_out = ms / iters;
    return rc;
}

}  // extern "C"
