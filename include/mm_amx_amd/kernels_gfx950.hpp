// kernels_gfx950.hpp — the operator classes of usstq/mm_amx's include/kernels_amx.hpp, for MI355X.
//
// Host-only C++14, header-only.  Same class names, template parameters, argument order and
// preconditions as the reference, so that a caller of amx_kernel::Matmul / MatmulVector / GemAvB /
// PP::BiasGeluStore / repackB_1x2 re-targets by switching the namespace.  Differences that the
// change of machine forces:
//   * tensor2D<T> memory lives on the GPU (hipMalloc); upload()/download() move host data.
//   * bias and per-channel scale pointers handed to PP::BiasGeluStore are device pointers.
//   * the post-op is a descriptor the kernels are specialised on, not a functor called per block.
//   * every call is asynchronous on a HIP stream (last argument, default stream if omitted).
//   * a failed precondition throws std::runtime_error where the reference asserts.
// Every operation ends in the C ABI of mm_amx_amd.h (libmm_amx_amd.so); nothing is computed here.
#pragma once

#include <hip/hip_runtime_api.h>

#include <cstdint>
#include <cstring>
#include <map>
#include <memory>
#include <mutex>
#include <stdexcept>
#include <string>
#include <type_traits>
#include <vector>

#include "../mm_amx_amd.h"

namespace gfx950_kernel {

// ---- errors -------------------------------------------------------------------------------------
inline void check(int rc, const char* what) {
    if (rc != MMX_OK) throw std::runtime_error(std::string(what) + ": " + mmx_last_error());
}
inline void check_hip(hipError_t e, const char* what) {
    if (e != hipSuccess) throw std::runtime_error(std::string(what) + ": " + hipGetErrorString(e));
}
inline void require(bool ok, const char* msg) {
    if (!ok) throw std::runtime_error(msg);
}

// ---- ov::bfloat16 (include/bf16.hpp:19-122): 16-bit storage, round-to-nearest-even from fp32 ----
struct bfloat16 {
    uint16_t bits;
    bfloat16() : bits(0) {}
    bfloat16(float f) {
        uint32_t u;
        std::memcpy(&u, &f, 4);
        bits = static_cast<uint16_t>((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
    }
    operator float() const {
        const uint32_t u = static_cast<uint32_t>(bits) << 16;
        float f;
        std::memcpy(&f, &u, 4);
        return f;
    }
};
static_assert(sizeof(bfloat16) == 2, "bfloat16 is two bytes");

template <typename T> struct dtype_of;
template <> struct dtype_of<float> { static constexpr int value = MMX_F32; };
template <> struct dtype_of<bfloat16> { static constexpr int value = MMX_BF16; };
template <> struct dtype_of<int8_t> { static constexpr int value = MMX_I8; };
template <> struct dtype_of<int32_t> { static constexpr int value = MMX_I32; };
template <> struct dtype_of<uint8_t> { static constexpr int value = MMX_U8; };

// accumulator type of an input type (include/kernels_amx.hpp:818-828)
template <typename T> struct acc_type { typedef float type; };
template <> struct acc_type<int8_t> { typedef int32_t type; };
template <> struct acc_type<uint8_t> { typedef int32_t type; };  // (:825)

// ---- tensor2D<T> (include/tensor2D.hpp:30-329), resident in HBM -----------------------------------
// dims = {rows, cols}; stride is in BYTES; rows are padded to 64 bytes unless force_compact;
// a view over external device memory does not own it (include/tensor2D.hpp:50-57).
template <typename T>
struct tensor2D {
    int dims[2] = {0, 0};
    int stride = 0;  // bytes
    T* data = nullptr;
    std::shared_ptr<void> owner;

    tensor2D() = default;
    tensor2D(int rows, int cols, bool force_compact = false) { resize(rows, cols, force_compact); }
    tensor2D(int rows, int cols, T* device_ptr, int stride_bytes) : stride(stride_bytes), data(device_ptr) {
        dims[0] = rows;
        dims[1] = cols;
    }

    void resize(int rows, int cols, bool force_compact = false) {
        dims[0] = rows;
        dims[1] = cols;
        stride = cols * static_cast<int>(sizeof(T));
        if (!force_compact && (stride % 64)) stride += 64 - stride % 64;
        // Rows that lie a multiple of 2 KiB apart meet in the same L2 channel; a tile kernel that pulls 8 rows per load
        // instruction then waits for that channel (int8 FC 512 x 4096 x 4096: 16.7 us against 14.2 us with rows
        // 128 bytes further apart).  The reference pads rows to 64 bytes; here a row that would end on such a
        // boundary gets 128 bytes more.
        if (!force_compact && rows > 1 && stride >= 2048 && stride % 2048 == 0) stride += 128;
        void* p = nullptr;
        const size_t bytes = static_cast<size_t>(rows > 0 ? rows : 1) * stride;
        check_hip(hipMalloc(&p, bytes), "tensor2D: hipMalloc");
        owner = std::shared_ptr<void>(p, [](void* q) { (void)hipFree(q); });
        data = static_cast<T*>(p);
    }
    size_t bytes() const { return static_cast<size_t>(dims[0]) * stride; }

    // host [rows, cols] with row stride host_stride_bytes (0 = compact) -> device; blocks until done
    void upload(const T* host, size_t host_stride_bytes = 0) {
        if (!host_stride_bytes) host_stride_bytes = static_cast<size_t>(dims[1]) * sizeof(T);
        check_hip(hipMemcpy2D(data, stride, host, host_stride_bytes, static_cast<size_t>(dims[1]) * sizeof(T), dims[0],
                              hipMemcpyHostToDevice),
                  "tensor2D::upload");
    }
    void download(T* host, size_t host_stride_bytes = 0) const {
        if (!host_stride_bytes) host_stride_bytes = static_cast<size_t>(dims[1]) * sizeof(T);
        check_hip(hipMemcpy2D(host, host_stride_bytes, data, stride, static_cast<size_t>(dims[1]) * sizeof(T), dims[0],
                              hipMemcpyDeviceToHost),
                  "tensor2D::download");
    }
    void zero() { check_hip(hipMemset(data, 0, bytes()), "tensor2D::zero"); }
    tensor2D<T> clone() const {
        tensor2D<T> t;
        t.dims[0] = dims[0], t.dims[1] = dims[1], t.stride = stride;
        void* p = nullptr;
        check_hip(hipMalloc(&p, bytes() ? bytes() : 1), "tensor2D::clone");
        t.owner = std::shared_ptr<void>(p, [](void* q) { (void)hipFree(q); });
        t.data = static_cast<T*>(p);
        check_hip(hipMemcpy(p, data, bytes(), hipMemcpyDeviceToDevice), "tensor2D::clone");
        return t;
    }
};

// device array of n elements (bias, scales), filled from the host
template <typename T>
struct device_vector {
    T* data = nullptr;
    size_t n = 0;
    std::shared_ptr<void> owner;
    device_vector() = default;
    explicit device_vector(size_t count) : n(count) {
        void* p = nullptr;
        check_hip(hipMalloc(&p, (count ? count : 1) * sizeof(T)), "device_vector: hipMalloc");
        owner = std::shared_ptr<void>(p, [](void* q) { (void)hipFree(q); });
        data = static_cast<T*>(p);
    }
    explicit device_vector(const std::vector<T>& host) : device_vector(host.size()) {
        check_hip(hipMemcpy(data, host.data(), n * sizeof(T), hipMemcpyHostToDevice), "device_vector: upload");
    }
    std::vector<T> to_host() const {
        std::vector<T> h(n);
        check_hip(hipMemcpy(h.data(), data, n * sizeof(T), hipMemcpyDeviceToHost), "device_vector: download");
        return h;
    }
};

// ---- post-ops (include/kernels_amx.hpp:538-673) ----------------------------------------------------
namespace PP {

enum Steps {
    NONE = 0,
    DEQUANT = 1 << 0,
    BIAS = 1 << 1,
    GELU = 1 << 2,
    QUANT = 1 << 3,
    BIAS_GELU = BIAS | GELU,
    DEQUANT_BIAS_GELU = DEQUANT | BIAS_GELU,
    DEQUANT_BIAS_GELU_QUANT = DEQUANT_BIAS_GELU | QUANT
};

// PP::BiasGeluStore<D, steps> (include/kernels_amx.hpp:552-583): same public fields and setters.
// set_deq_scale(float*) is an extension (per-output-channel dequant; the reference has one float).
template <typename D, Steps steps>
struct BiasGeluStore {
    static_assert(std::is_same<D, bfloat16>::value || std::is_same<D, int8_t>::value || std::is_same<D, float>::value,
                  "BiasGeluStore only supports output data types bfloat16/int8_t/float");

    BiasGeluStore(tensor2D<D>& C, float* bias = nullptr) : C(C), bias(bias) {}

    tensor2D<D>& C;
    float* bias;  // device [N]
    void set_bias(float* _bias) {
        require((steps & BIAS) != 0, "set_bias: BIAS step not enabled");
        bias = _bias;
    }

    float deq_scale = 1.0f;
    float* deq_scale_per_oc = nullptr;  // device [N]
    void set_deq_scale(float scale = 1.0f) {
        require((steps & DEQUANT) != 0, "set_deq_scale: DEQUANT step not enabled");
        deq_scale = scale;
        deq_scale_per_oc = nullptr;
    }
    void set_deq_scale(float* scale_per_oc) {
        require((steps & DEQUANT) != 0, "set_deq_scale: DEQUANT step not enabled");
        deq_scale = 1.0f;
        deq_scale_per_oc = scale_per_oc;
    }

    float q_scale_common = 0.0f;
    float* q_scale_per_oc = nullptr;  // device [N]
    void set_q_scale(float scale) {
        require((steps & QUANT) != 0, "set_q_scale: QUANT step not enabled");
        q_scale_common = scale;
        q_scale_per_oc = nullptr;
    }
    void set_q_scale(float* scale_per_oc) {
        require((steps & QUANT) != 0, "set_q_scale: QUANT step not enabled");
        q_scale_common = 0;
        q_scale_per_oc = scale_per_oc;
    }

    mmx_epilogue descriptor() const {
        require(!(steps & BIAS) || bias, "BiasGeluStore: BIAS step enabled but no bias set");
        mmx_epilogue e;
        e.steps = static_cast<uint32_t>(steps);
        e.out_dtype = dtype_of<D>::value;
        e.C = C.data;
        e.ldc_bytes = C.stride;
        e.bias = bias;
        e.deq_scale = deq_scale;
        e.deq_scale_per_oc = deq_scale_per_oc;
        e.q_scale = q_scale_common;
        e.q_scale_per_oc = q_scale_per_oc;
        return e;
    }
    int out_rows() const { return C.dims[0]; }
    int out_cols() const { return C.dims[1]; }
};

// Raw accumulator store for int8 x int8 (int32 out): the reference's tests read buffC directly.
struct StoreI32 {
    explicit StoreI32(tensor2D<int32_t>& C) : C(C) {}
    tensor2D<int32_t>& C;
    mmx_epilogue descriptor() const {
        mmx_epilogue e;
        std::memset(&e, 0, sizeof e);
        e.out_dtype = MMX_I32;
        e.C = C.data;
        e.ldc_bytes = C.stride;
        e.deq_scale = 1.0f;
        return e;
    }
    int out_rows() const { return C.dims[0]; }
    int out_cols() const { return C.dims[1]; }
};

}  // namespace PP

// ---- packed weights --------------------------------------------------------------------------------
// What repackB_1x2 returns: the whole [K, N] matrix in MFMA-fragment order (see mm_amx_amd.h).
template <typename T>
struct PackedB {
    int K = 0, N = 0;
    size_t bytes = 0;
    void* data = nullptr;
    std::shared_ptr<void> owner;
    explicit operator bool() const { return data != nullptr; }
    PackedB clone() const {
        PackedB o = *this;
        void* p = nullptr;
        check_hip(hipMalloc(&p, bytes ? bytes : 1), "PackedB::clone");
        o.owner = std::shared_ptr<void>(p, [](void* q) { (void)hipFree(q); });
        o.data = p;
        check_hip(hipMemcpy(p, data, bytes, hipMemcpyDeviceToDevice), "PackedB::clone");
        return o;
    }
};

template <typename T>
inline PackedB<T> alloc_packed(int K, int N) {
    PackedB<T> p;
    p.K = K;
    p.N = N;
    p.bytes = mmx_packed_b_bytes(dtype_of<T>::value, K, N);
    void* d = nullptr;
    check_hip(hipMalloc(&d, p.bytes ? p.bytes : 1), "PackedB: hipMalloc");
    p.owner = std::shared_ptr<void>(d, [](void* q) { (void)hipFree(q); });
    p.data = d;
    return p;
}

// amx_kernel::repackB_1x2<T>(Bi, transpose) (include/kernels_amx.hpp:761-816).  Bi is [K, N], or
// [N, K] when transpose.
template <typename T>
inline PackedB<T> repackB_1x2(const tensor2D<T>& Bi, bool transpose = false, hipStream_t stream = nullptr) {
    const int K = Bi.dims[transpose ? 1 : 0], N = Bi.dims[transpose ? 0 : 1];
    PackedB<T> p = alloc_packed<T>(K, N);
    check(mmx_repack_b(dtype_of<T>::value, Bi.data, Bi.stride, K, N, transpose ? 1 : 0, p.data, stream), "repackB_1x2");
    return p;
}

// repackB_1xL<T, L>(Bi, scale) (weight_compression/fc16m.cpp:61-99): the packed weights of the M <= 16 kernels from a
// bf16 [K, N] matrix, as bf16 (scale 1, as everywhere in the reference) or compressed to int8 on the way: every weight
// becomes int8_t(w * scale), the bf16 product rounded to nearest even and then truncated toward zero (:80-81; saturated
// here where the reference's conversion is undefined).  L = 1..4 tiles of 16 columns side by side only orders the
// reference's cache layout: its preconditions are kept (K a multiple of 32, N of 16 L), the result is this library's
// fragment order.
template <typename T, int L>
inline PackedB<T> repackB_1xL(const tensor2D<bfloat16>& Bi, float scale = 1.0f, hipStream_t stream = nullptr) {
    static_assert(L >= 1 && L <= 4, "L = 1 ... 4");
    static_assert(std::is_same<T, bfloat16>::value || std::is_same<T, int8_t>::value, "T is bfloat16 or int8_t");
    const int K = Bi.dims[0], N = Bi.dims[1];
    require(K % 32 == 0, "repackB_1xL: K must be a multiple of 32");
    require(N % (L * 16) == 0, "repackB_1xL: N must be a multiple of 16 L");
    PackedB<T> p = alloc_packed<T>(K, N);
    if (std::is_same<T, bfloat16>::value) {
        require(scale == 1.0f, "repackB_1xL: a scale is for the int8 form only");
        check(mmx_repack_b(MMX_BF16, Bi.data, Bi.stride, K, N, 0, p.data, stream), "repackB_1xL");
        return p;
    }
    void* q = nullptr;  // the quantised matrix in source order, between the two kernels only
    const size_t qbytes = static_cast<size_t>(K) * static_cast<size_t>(N);
    check_hip(hipMalloc(&q, qbytes > 0 ? qbytes : 1), "repackB_1xL: hipMalloc");
    std::shared_ptr<void> hold(q, [](void* x) { (void)hipFree(x); });
    check(mmx_quantize_weights_scaled(Bi.data, Bi.stride, K, N, scale, q, N, stream), "repackB_1xL: quantise");
    check(mmx_repack_b(MMX_I8, q, N, K, N, 0, p.data, stream), "repackB_1xL: pack");
    check_hip(hipStreamSynchronize(stream), "repackB_1xL");  // (the temporary is freed on return)
    return p;
}

// ---- workspace of the K split -------------------------------------------------------------------------
// AMX_MLP::Linear keeps the partial results of its two K halves in per-thread buffers (work.C,
// tests/amx-mlp.cpp:648-682); here the partial tiles of mmx_gemm_splitk live in one zero-initialised device
// buffer per (device, stream): calls on one stream are ordered, so they can share it, calls on different
// streams must not.  64 MiB + 16 KiB serves every shape when the library chooses the number of slices.
struct Workspace {
    void* data = nullptr;
    size_t bytes = 0;
};
// `need`: what mmx_gemm_workspace_bytes says the call can use; 0 = the call would not split, nothing is allocated.
// A stream that is being captured into a graph gets no NEW buffer (an allocation and a memset there would be captured
// or would invalidate the capture): the call then runs without a K split, whose sums may differ in their last bits
// from the split form an eager call of the same shape takes.  Buffers live until release_workspaces() or the end of
// the process (they are deliberately not freed from a static destructor, which may run after the HIP runtime's own).
inline std::map<std::pair<int, hipStream_t>, Workspace>& workspace_slots() {
    static auto* all = new std::map<std::pair<int, hipStream_t>, Workspace>();
    return *all;
}
inline std::mutex& workspace_mutex() {
    static auto* mu = new std::mutex();
    return *mu;
}
// `forced`: the caller named a count of slices: the library then gets a workspace in any case and reports what does not fit.
inline Workspace workspace_for(hipStream_t stream, size_t need, bool forced = false) {
    if (need == 0 && !forced) return Workspace();
    if (need == 0) need = 1;
    int dev = 0;
    check_hip(hipGetDevice(&dev), "workspace_for: hipGetDevice");
    std::lock_guard<std::mutex> lock(workspace_mutex());
    Workspace& slot = workspace_slots()[std::make_pair(dev, stream)];
    if (slot.bytes < need) {
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(stream, &cap) != hipSuccess) {
            (void)hipGetLastError();  // (the legacy default stream cannot be queried while another stream captures)
            cap = hipStreamCaptureStatusActive;
        }
        if (cap != hipStreamCaptureStatusNone) return slot.bytes ? slot : Workspace();
        constexpr size_t kAlways = (size_t(64) << 20) + (size_t(16) << 10);  // serves every shape with k_splits = 0
        const size_t bytes = need > kAlways ? need : kAlways;
        void* p = nullptr;
        check_hip(hipMalloc(&p, bytes), "workspace_for: hipMalloc");
        check_hip(hipMemset(p, 0, bytes), "workspace_for: hipMemset");  // the arrival counters start at zero
        if (slot.data) {
            check_hip(hipStreamSynchronize(stream), "workspace_for: hipStreamSynchronize");  // launches may still use the old one
            (void)hipFree(slot.data);
        }
        slot = Workspace{p, bytes};
    }
    return slot;
}
// Frees every workspace (call with no launch in flight, e.g. after hipDeviceSynchronize).
inline void release_workspaces() {
    std::lock_guard<std::mutex> lock(workspace_mutex());
    for (auto& kv : workspace_slots())
        if (kv.second.data) (void)hipFree(kv.second.data);
    workspace_slots().clear();
}

// ---- Matmul<TA,TB,TC> (include/kernels_amx.hpp:1045-1315) ---------------------------------------
// C = PP(A · B[:, n0:n1]).  With constB the packed weights are made at the first call and kept
// (1188-1192); otherwise B is repacked on every call.  One object is used by one thread at a time,
// as in the reference; calls are ordered on the stream.
template <typename TA, typename TB, typename TC = typename acc_type<TA>::type>
struct Matmul {
    PackedB<TB> internalB;
    bool constB;
    bool transposeB;
    // K slices per output tile, the split-K of AMX_MLP::Linear (tests/amx-mlp.cpp:560-593, 648-682):
    // 0 = the library chooses, 1 = never, 2 = the reference's two halves, up to 4
    int k_splits = 0;

    // is_s8u8 / is_u8s8 / is_u8u8 (include/kernels_amx.hpp:1057-1061): at least one operand of unsigned bytes
    constexpr static bool is_u8_mode = (std::is_same<TA, uint8_t>::value || std::is_same<TB, uint8_t>::value) &&
                                       (std::is_same<TA, uint8_t>::value || std::is_same<TA, int8_t>::value) &&
                                       (std::is_same<TB, uint8_t>::value || std::is_same<TB, int8_t>::value);
    static_assert(std::is_same<TA, TB>::value || is_u8_mode,
                  "Matmul<TA,TB>: TA == TB except for the <bfloat16,int8_t,float> form and the unsigned byte forms");
    constexpr static bool is_i8_mode = std::is_same<TA, int8_t>::value || is_u8_mode;
    constexpr static int kStep = is_i8_mode ? 64 : 32;
    std::shared_ptr<void> u8_scratch;  // unsigned forms: the shifted activations, correction terms and int32 sums of a call
    size_t u8_scratch_bytes = 0;

    Matmul(bool constB = false, bool transposeB = false) : constB(constB), transposeB(transposeB) {}

    template <typename P>
    void operator()(tensor2D<TA>& matA, tensor2D<TB>& matB, P ppkernel, hipStream_t stream = nullptr) {
        (*this)(matA, matB, 0, matB.dims[transposeB ? 0 : 1], ppkernel, stream);
    }

    template <typename P>
    void operator()(tensor2D<TA>& matA, tensor2D<TB>& matB, int n0, int n1, P ppkernel, hipStream_t stream = nullptr) {
        const int M = matA.dims[0], K = matA.dims[1];
        const int N = matB.dims[transposeB ? 0 : 1];
        require(K == matB.dims[transposeB ? 1 : 0], "Matmul: K of A and B differ");
        require(K >= kStep, "Matmul: K must be at least kStep");  // include/kernels_amx.hpp:1183
        require(ppkernel.out_rows() >= M && ppkernel.out_cols() >= n1, "Matmul: C is smaller than M x n1");
        if (!constB || !internalB) internalB = repackB_1x2(matB, transposeB, stream);
        const mmx_epilogue e = ppkernel.descriptor();
        if (is_u8_mode) {  // tdpbusd / tdpbsud / tdpbuud: mmx_gemm_u8 (three passes, exact)
            const size_t need = mmx_gemm_u8_scratch_bytes(dtype_of<TA>::value, dtype_of<TB>::value, M, K, N, n0, n1);
            if (need > u8_scratch_bytes) {
                void* p = nullptr;
                check_hip(hipStreamSynchronize(stream), "Matmul: hipStreamSynchronize");  // an earlier call may still use the old one
                check_hip(hipMalloc(&p, need), "Matmul: hipMalloc(u8 scratch)");
                u8_scratch = std::shared_ptr<void>(p, [](void* q) { (void)hipFree(q); });
                u8_scratch_bytes = need;
            }
            check(mmx_gemm_u8(dtype_of<TA>::value, dtype_of<TB>::value, matA.data, matA.stride, internalB.data, M, K, N, n0, n1, &e,
                              u8_scratch.get(), u8_scratch_bytes, stream),
                  "Matmul (unsigned bytes)");
            return;
        }
        // (decode launches, M <= 32, choose their own slices: they take the workspace with k_splits = 0 only)
        const Workspace ws = (k_splits == 1 || (M <= 32 && k_splits != 0))
                                 ? Workspace()
                                 : workspace_for(stream, mmx_gemm_workspace_bytes(dtype_of<TA>::value, dtype_of<TB>::value, M, K, N, n0, n1,
                                                                                  e.steps, k_splits),
                                                 k_splits > 1);
        check(mmx_gemm_splitk(dtype_of<TA>::value, dtype_of<TB>::value, matA.data, matA.stride, internalB.data, M, K, N, n0, n1,
                              &e, ws.data ? k_splits : 1, ws.data, ws.bytes, stream),
              "Matmul");
    }
};

// Matmul<bfloat16, int8_t, float> (include/kernels_amx.hpp:1319-1516): takes the bf16 weights,
// compresses them to int8 per tensor at the first call (1363-1377) and sets the post-op's dequant
// scale (1379).  The packed int8 weights are the only copy: M <= 32 streams them through the decode kernels,
// larger M converts the int8 fragments to bf16 between LDS and the MFMA operand (the reference's on-the-fly
// dequantisation, 1447-1497).
template <>
struct Matmul<bfloat16, int8_t, float> {
    PackedB<int8_t> internalBI8;
    bool constB;
    bool transposeB;
    constexpr static int kStep = 32;
    float quant_scale_B = 0.0f;
    float dequant_scale_B = 0.0f;
    int k_splits = 0;  // as in the primary template

    Matmul(bool constB = false, bool transposeB = false) : constB(constB), transposeB(transposeB) {}

    template <typename P>
    void operator()(tensor2D<bfloat16>& matA, tensor2D<bfloat16>& matB, P ppkernel, hipStream_t stream = nullptr) {
        (*this)(matA, matB, 0, matB.dims[transposeB ? 0 : 1], ppkernel, stream);
    }

    template <typename P>
    void operator()(tensor2D<bfloat16>& matA, tensor2D<bfloat16>& matB, int n0, int n1, P ppkernel,
                    hipStream_t stream = nullptr) {
        const int M = matA.dims[0], K = matA.dims[1];
        const int N = matB.dims[transposeB ? 0 : 1];
        require(K == matB.dims[transposeB ? 1 : 0], "Matmul: K of A and B differ");
        require(K >= kStep, "Matmul: K must be at least kStep");
        require(ppkernel.out_rows() >= M && ppkernel.out_cols() >= n1, "Matmul: C is smaller than M x n1");
        if (!constB || !internalBI8) {
            tensor2D<int8_t> Wq(matB.dims[0], matB.dims[1]);
            device_vector<float> scales(2);
            device_vector<uint32_t> scratch(1);
            check(mmx_quantize_weights(matB.data, matB.stride, matB.dims[0], matB.dims[1], Wq.data, Wq.stride, scales.data,
                                       scratch.data, stream),
                  "Matmul<bf16,int8>: quantize");
            internalBI8 = repackB_1x2(Wq, transposeB, stream);
            check_hip(hipStreamSynchronize(stream), "Matmul<bf16,int8>: sync");  // Wq and scales are read back / freed
            const std::vector<float> s = scales.to_host();
            quant_scale_B = s[0];
            dequant_scale_B = s[1];
        }
        ppkernel.set_deq_scale(dequant_scale_B);
        const mmx_epilogue e = ppkernel.descriptor();
        const Workspace ws = (k_splits == 1 || (M <= 32 && k_splits != 0))
                                 ? Workspace()
                                 : workspace_for(stream, mmx_gemm_workspace_bytes(MMX_BF16, MMX_I8, M, K, N, n0, n1, e.steps, k_splits), k_splits > 1);
        check(mmx_gemm_splitk(MMX_BF16, MMX_I8, matA.data, matA.stride, internalBI8.data, M, K, N, n0, n1, &e,
                              ws.data ? k_splits : 1, ws.data, ws.bytes, stream),
              "Matmul<bf16,int8>");
    }
};

// Decode-path Matmul over int4-compressed weights.  The reference has no such class: it only times a stand-in
// that copies bytes in place of an int4 dequant (weight_compression/wcompress.hpp:90-134).  Same call shape as
// Matmul<bfloat16, int8_t, float>: takes the bf16 weights, compresses them per output channel to [-7, 7] at the
// first call and points the post-op's dequant step at the per-channel scales.  M <= 32 only.
struct MatmulW4 {
    device_vector<uint8_t> internalB4;      // packed nibbles
    device_vector<float> dequant_scales_B;  // [N]
    bool constB;
    bool transposeB;

    MatmulW4(bool constB = false, bool transposeB = false) : constB(constB), transposeB(transposeB) {}

    template <typename P>
    void operator()(tensor2D<bfloat16>& matA, tensor2D<bfloat16>& matB, P ppkernel, hipStream_t stream = nullptr) {
        (*this)(matA, matB, 0, matB.dims[transposeB ? 0 : 1], ppkernel, stream);
    }

    template <typename P>
    void operator()(tensor2D<bfloat16>& matA, tensor2D<bfloat16>& matB, int n0, int n1, P ppkernel,
                    hipStream_t stream = nullptr) {
        const int M = matA.dims[0], K = matA.dims[1];
        const int N = matB.dims[transposeB ? 0 : 1];
        require(K == matB.dims[transposeB ? 1 : 0], "MatmulW4: K of A and B differ");
        require(M <= 32, "MatmulW4: int4 weights are a decode path (M <= 32)");
        require(ppkernel.out_rows() >= M && ppkernel.out_cols() >= n1, "MatmulW4: C is smaller than M x n1");
        if (!constB || !internalB4.data) {
            // (freeing the previous buffers waits for the launches that still read them)
            internalB4 = device_vector<uint8_t>(mmx_packed_b_bytes(MMX_I4, K, N));
            dequant_scales_B = device_vector<float>(N);
            check(mmx_quantize_pack_int4(matB.data, matB.stride, K, N, transposeB ? 1 : 0, internalB4.data,
                                         dequant_scales_B.data, stream),
                  "MatmulW4: quantize");
        }
        ppkernel.set_deq_scale(dequant_scales_B.data);
        const mmx_epilogue e = ppkernel.descriptor();
        check(mmx_gemm(MMX_BF16, MMX_I4, matA.data, matA.stride, internalB4.data, M, K, N, n0, n1, &e, stream), "MatmulW4");
    }
};

// ---- MatmulVector (include/kernels_amx.hpp:833-1043): c[M] = A[M, K] · b[K] ------------------------
// vB and vC are device pointers.  The reference admits kStep <= K <= 6 kStep (966); this kernel
// takes any K >= 1, the same bounds are not enforced.
template <typename TA, typename TB, typename TC = typename acc_type<TA>::type>
struct MatmulVector {
    // is_s8u8 / is_u8s8 / is_u8u8 (include/kernels_amx.hpp:839-850)
    constexpr static bool is_u8_mode = (std::is_same<TA, uint8_t>::value || std::is_same<TB, uint8_t>::value) &&
                                       (std::is_same<TA, uint8_t>::value || std::is_same<TA, int8_t>::value) &&
                                       (std::is_same<TB, uint8_t>::value || std::is_same<TB, int8_t>::value);
    static_assert(std::is_same<TA, TB>::value || is_u8_mode, "MatmulVector: TA == TB, or bytes of either sign");
    constexpr static int kStep = (std::is_same<TA, int8_t>::value || is_u8_mode) ? 64 : 32;
    MatmulVector() {}
    void operator()(tensor2D<TA>& matA, const TB* vB, TC* vC, hipStream_t stream = nullptr) {
        if (is_u8_mode)
            check(mmx_matvec_u8(dtype_of<TA>::value, dtype_of<TB>::value, matA.data, matA.stride, vB, vC, matA.dims[0], matA.dims[1], stream),
                  "MatmulVector (unsigned bytes)");
        else
            check(mmx_matvec(dtype_of<TA>::value, matA.data, matA.stride, vB, vC, matA.dims[0], matA.dims[1], stream),
                  "MatmulVector");
    }
};

// ---- GemAvB (include/kernels_amx.hpp:1529-1618): the same product, bf16 only ------------------------
struct GemAvB {
    GemAvB() {}
    void operator()(tensor2D<bfloat16>& matA, bfloat16* vecB, float* vecC, hipStream_t stream = nullptr) {
        require(matA.dims[1] >= 32, "GemAvB: K must be at least 32");  // include/kernels_amx.hpp:1542
        check(mmx_matvec(MMX_BF16, matA.data, matA.stride, vecB, vecC, matA.dims[0], matA.dims[1], stream), "GemAvB");
    }
};

// ---- LinearNxN (torch-ext/amx_mlp.cpp:452-485): y[M, N] fp32 = x[M, K] bf16 · w[N, K]^T ------------
struct LinearNxN {
    std::string name;
    int m_N = 0, m_K = 0;
    PackedB<bfloat16> packed;

    void set_weight(const tensor2D<bfloat16>& weight, hipStream_t stream = nullptr) {
        require(weight.dims[0] % 32 == 0 && weight.dims[1] % 32 == 0,
                "set_weight: N and K must be multiples of 32");  // torch-ext/amx_mlp.cpp:474-475
        m_N = weight.dims[0];
        m_K = weight.dims[1];
        packed = repackB_1x2(weight, true, stream);
    }
    void forward(tensor2D<bfloat16>& x, tensor2D<float>& y, hipStream_t stream = nullptr) {
        require(static_cast<bool>(packed), "forward: set_weight has not been called");
        require(x.dims[1] == m_K, "forward: x must be [M, K]");
        require(y.dims[0] == x.dims[0] && y.dims[1] == m_N, "forward: y must be [M, N]");
        PP::BiasGeluStore<float, PP::NONE> pp(y);
        const mmx_epilogue e = pp.descriptor();
        check(mmx_gemm(MMX_BF16, MMX_BF16, x.data, x.stride, packed.data, x.dims[0], m_K, m_N, 0, m_N, &e, stream),
              "LinearNxN::forward");
    }
    LinearNxN deepcopy() const {  // __deepcopy__ (torch-ext/amx_mlp.cpp:499-510)
        LinearNxN o;
        o.name = name, o.m_N = m_N, o.m_K = m_K;
        if (packed) o.packed = packed.clone();
        return o;
    }
};

// ---- MLP (tests/amx-mlp.cpp:740-784) ------------------------------------------------------------------
// setup(w_gate[N,K], w_up[N,K], w_down[K,N]) with torch nn.Linear.weight layouts;
// run(x[M,K], y[M,K]): y = bf16( bf16(silu(x·Wg^T) * (x·Wu^T)) · Wd^T ).
struct MLP {
    int m_N = 0, m_K = 0, m_M = 0;
    PackedB<bfloat16> gate_up, down;
    tensor2D<bfloat16> actUp;
    // K slices of the down projection: the reference builds `down` with do_splitK = true (two halves,
    // tests/amx-mlp.cpp:768); 0 = the library chooses, 1 = never, 2 = the reference's partition
    int down_k_splits = 0;

    void setup(const tensor2D<bfloat16>& w_gate, const tensor2D<bfloat16>& w_up, const tensor2D<bfloat16>& w_down,
               hipStream_t stream = nullptr) {
        m_N = w_gate.dims[0];
        m_K = w_gate.dims[1];
        require(w_up.dims[0] == m_N && w_up.dims[1] == m_K && w_up.stride == w_gate.stride,
                "setup: w_up must match w_gate");
        require(w_down.dims[0] == m_K && w_down.dims[1] == m_N, "setup: w_down must be [K, N]");
        require(m_N % 32 == 0, "setup: N must be a multiple of 32");
        gate_up = alloc_packed<bfloat16>(m_K, 2 * m_N);
        check(mmx_repack_gate_up(w_gate.data, w_up.data, w_gate.stride, m_K, m_N, gate_up.data, stream), "MLP::setup");
        down = repackB_1x2(w_down, true, stream);
    }
    void setM(int M) {  // tests/amx-mlp.cpp:771-776
        if (m_M < M) {
            actUp.resize(M, m_N);
            m_M = M;
        }
    }
    void run(tensor2D<bfloat16>& x, tensor2D<bfloat16>& y, hipStream_t stream = nullptr) {
        require(static_cast<bool>(gate_up), "run: setup has not been called");
        const int M = x.dims[0];
        require(x.dims[1] == m_K && y.dims[0] == M && y.dims[1] == m_K, "run: x and y must be [M, K]");
        setM(M);
        // the down projection is the GEMM [M, N] x [N, K] (M <= 32: the library chooses its own slices)
        const Workspace ws = down_k_splits == 1 ? Workspace()
                                                : workspace_for(stream, mmx_gemm_workspace_bytes(MMX_BF16, MMX_BF16, M, m_N, m_K, 0, m_K, MMX_PP_NONE,
                                                                                                 M <= 32 ? 0 : down_k_splits),
                                                                M > 32 && down_k_splits > 1);
        check(mmx_mlp_splitk(x.data, x.stride, gate_up.data, down.data, actUp.data, actUp.stride, y.data, y.stride, M, m_K, m_N,
                             ws.data ? down_k_splits : 1, ws.data, ws.bytes, stream),
              "MLP::run");
    }
};

// One-time set-up, where the reference calls initXTILE() (include/misc.hpp:376-396).
inline void init(int device = 0) { check(mmx_init(device), "mmx_init"); }

}  // namespace gfx950_kernel
