"""ctypes binding of the C ABI declared in include/mm_amx_amd.h.

Arguments are torch tensors resident on the GPU; only their ``data_ptr()``, strides and the
current torch HIP stream cross the boundary.
"""
import ctypes as C
import os

import torch

F32, BF16, I8, I32, I4 = 0, 1, 2, 3, 4
PP_NONE, PP_DEQUANT, PP_BIAS, PP_GELU, PP_QUANT, PP_SILU_GATE = 0, 1, 2, 4, 8, 16

_HERE = os.path.dirname(os.path.abspath(__file__))
# MMX_LIB_PATH lets a developer point at an alternative build of the same ABI
_LIB_PATH = os.environ.get("MMX_LIB_PATH") or os.path.join(_HERE, "libmm_amx_amd.so")

EXPORTS = ["mmx_last_error", "mmx_init", "mmx_packed_b_bytes", "mmx_repack_b", "mmx_repack_gate_up",
           "mmx_quantize_weights", "mmx_quantize_pack_int4", "mmx_dequant_packed", "mmx_gemm", "mmx_matvec", "mmx_mlp", "mmx_set_tile",
           "mmx_set_option", "mmx_last_kernel", "mmx_time_gemm", "mmx_probe_mfma"]


class MmxError(RuntimeError):
    pass


class _Epilogue(C.Structure):
    _fields_ = [("steps", C.c_uint32), ("out_dtype", C.c_int32), ("C", C.c_void_p), ("ldc_bytes", C.c_int64),
                ("bias", C.c_void_p), ("deq_scale", C.c_float), ("deq_scale_per_oc", C.c_void_p),
                ("q_scale", C.c_float), ("q_scale_per_oc", C.c_void_p)]


_lib = None
_initialised = set()


def lib_path():
    return _LIB_PATH


def lib():
    """The loaded C-ABI library.  Raises if it has not been built: there is no fallback."""
    global _lib
    if _lib is None:
        if not os.path.isfile(_LIB_PATH):
            raise MmxError(f"{_LIB_PATH} is missing: build it with `python -m mm_amx_amd.build` "
                           "(this package has no CPU or PyTorch fallback)")
        l = C.CDLL(_LIB_PATH)
        l.mmx_last_error.restype = C.c_char_p
        l.mmx_last_kernel.restype = C.c_char_p
        l.mmx_packed_b_bytes.restype = C.c_size_t
        l.mmx_packed_b_bytes.argtypes = [C.c_int, C.c_int, C.c_int]
        l.mmx_init.argtypes = [C.c_int]
        l.mmx_repack_b.argtypes = [C.c_int, C.c_void_p, C.c_int64, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
        l.mmx_repack_gate_up.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
        l.mmx_quantize_weights.argtypes = [C.c_void_p, C.c_int64, C.c_int, C.c_int, C.c_void_p, C.c_int64, C.c_void_p,
                                           C.c_void_p, C.c_void_p]
        l.mmx_quantize_pack_int4.argtypes = [C.c_void_p, C.c_int64, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p,
                                             C.c_void_p]
        l.mmx_dequant_packed.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
        l.mmx_gemm.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_int64, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int,
                               C.c_int, C.POINTER(_Epilogue), C.c_void_p]
        l.mmx_matvec.argtypes = [C.c_int, C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p]
        l.mmx_mlp.argtypes = [C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p,
                              C.c_int64, C.c_int, C.c_int, C.c_int, C.c_void_p]
        l.mmx_set_tile.argtypes = [C.c_char_p]
        l.mmx_set_option.argtypes = [C.c_char_p, C.c_int]
        l.mmx_time_gemm.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_int64, C.POINTER(C.c_void_p), C.c_int, C.c_int,
                                    C.c_int, C.c_int, C.c_int, C.c_int, C.POINTER(_Epilogue), C.c_void_p, C.c_int,
                                    C.POINTER(C.c_float)]
        l.mmx_probe_mfma.argtypes = [C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.POINTER(C.c_float),
                                     C.POINTER(C.c_float)]
        _lib = l
    return _lib


def _check(rc):
    if rc != 0:
        raise MmxError(f"mm_amx_amd error {rc}: {lib().mmx_last_error().decode()}")


def init(device=0):
    if device not in _initialised:
        _check(lib().mmx_init(device))
        _initialised.add(device)


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _dev(t, what):
    if not (isinstance(t, torch.Tensor) and t.is_cuda):
        raise MmxError(f"{what} must be a tensor on the GPU")
    init(t.device.index or 0)
    return t


_DT = {torch.float32: F32, torch.bfloat16: BF16, torch.int8: I8, torch.int32: I32}


def dtype_code(t):
    try:
        return _DT[t.dtype]
    except KeyError:
        raise MmxError(f"dtype {t.dtype} is not part of this path") from None


def _row_stride_bytes(t):
    # torch leaves the stride of a dimension of size 1 arbitrary: a single column is contiguous whatever
    # stride(1) says, and a single row has no row stride to speak of
    if t.dim() != 2 or (t.stride(1) != 1 and t.shape[1] != 1):
        raise MmxError("expected a 2-D tensor with unit stride in its last dimension")
    if t.shape[0] == 1:
        return t.shape[1] * t.element_size()
    return t.stride(0) * t.element_size()


class Epilogue:
    """Plain-data form of amx_kernel::PP::BiasGeluStore (include/kernels_amx.hpp:552-583)."""

    def __init__(self, C_out, steps=PP_NONE, bias=None, deq_scale=1.0, deq_scale_per_oc=None, q_scale=0.0,
                 q_scale_per_oc=None):
        self.C = _dev(C_out, "C")
        self.steps = int(steps)
        self.bias, self.deq_oc, self.q_oc = bias, deq_scale_per_oc, q_scale_per_oc
        self.deq, self.q = float(deq_scale), float(q_scale)
        for v, name in ((bias, "bias"), (deq_scale_per_oc, "deq_scale_per_oc"), (q_scale_per_oc, "q_scale_per_oc")):
            if v is not None and not (v.is_cuda and v.dtype == torch.float32 and v.is_contiguous()):
                raise MmxError(f"{name} must be a contiguous fp32 tensor on the GPU")

    def struct(self):
        p = lambda t: None if t is None else t.data_ptr()
        return _Epilogue(self.steps, dtype_code(self.C), self.C.data_ptr(), _row_stride_bytes(self.C), p(self.bias),
                         self.deq, p(self.deq_oc), self.q, p(self.q_oc))


def packed_b_bytes(dtype, K, N):
    return lib().mmx_packed_b_bytes(dtype, K, N)


def repack_b(B, transpose=False):
    """B [K,N] (or [N,K] with transpose) bf16/int8 on the GPU -> packed weights (uint8 tensor)."""
    _dev(B, "B")
    dt = dtype_code(B)
    K, N = (B.shape[1], B.shape[0]) if transpose else B.shape
    out = torch.empty(packed_b_bytes(dt, K, N), dtype=torch.uint8, device=B.device)
    _check(lib().mmx_repack_b(dt, B.data_ptr(), _row_stride_bytes(B), K, N, int(transpose), out.data_ptr(), _stream()))
    return out


def repack_gate_up(w_gate, w_up):
    """w_gate, w_up [N,K] bf16 -> packed [K, 2N] with gate/up alternating in 32-column panels."""
    _dev(w_gate, "w_gate"), _dev(w_up, "w_up")
    if w_gate.shape != w_up.shape or w_gate.dtype != torch.bfloat16 or w_up.dtype != torch.bfloat16:
        raise MmxError("w_gate and w_up must be bf16 tensors of the same shape")
    if _row_stride_bytes(w_gate) != _row_stride_bytes(w_up):
        raise MmxError("w_gate and w_up must share a row stride")
    N, K = w_gate.shape
    out = torch.empty(packed_b_bytes(BF16, K, 2 * N), dtype=torch.uint8, device=w_gate.device)
    _check(lib().mmx_repack_gate_up(w_gate.data_ptr(), w_up.data_ptr(), _row_stride_bytes(w_gate), K, N,
                                    out.data_ptr(), _stream()))
    return out


def quantize_weights(W):
    """Per-tensor symmetric int8 compression of a bf16 matrix; returns (Wq, scales[2] = {q, dq})."""
    _dev(W, "W")
    if W.dtype != torch.bfloat16:
        raise MmxError("W must be bf16")
    Wq = torch.empty(W.shape, dtype=torch.int8, device=W.device)
    scales = torch.empty(2, dtype=torch.float32, device=W.device)
    scratch = torch.empty(1, dtype=torch.int32, device=W.device)
    _check(lib().mmx_quantize_weights(W.data_ptr(), _row_stride_bytes(W), W.shape[0], W.shape[1], Wq.data_ptr(),
                                      _row_stride_bytes(Wq), scales.data_ptr(), scratch.data_ptr(), _stream()))
    return Wq, scales


def quantize_pack_int4(W, transpose=False):
    """Per-output-channel symmetric int4 compression of a bf16 matrix W [K,N] (or [N,K] with transpose), packed for
    gemm(..., b_dtype=I4) with M <= 32; returns (packed uint8, deq_scales fp32 [N])."""
    _dev(W, "W")
    if W.dtype != torch.bfloat16 or W.dim() != 2:
        raise MmxError("W must be a 2-D bf16 tensor with unit column stride")
    K, N = (W.shape[1], W.shape[0]) if transpose else W.shape
    packed = torch.empty(packed_b_bytes(I4, K, N), dtype=torch.uint8, device=W.device)
    deq = torch.empty(N, dtype=torch.float32, device=W.device)
    _check(lib().mmx_quantize_pack_int4(W.data_ptr(), _row_stride_bytes(W), K, N, int(transpose), packed.data_ptr(),
                                        deq.data_ptr(), _stream()))
    return packed, deq


def dequant_packed(packed_i8, K, N):
    out = torch.empty(packed_b_bytes(BF16, K, N), dtype=torch.uint8, device=packed_i8.device)
    _check(lib().mmx_dequant_packed(packed_i8.data_ptr(), K, N, out.data_ptr(), _stream()))
    return out


def gemm(A, Bpacked, N, ep, b_dtype=None, n0=0, n1=None):
    """C[:, n0:n1] = PP(A · B[:, n0:n1]); A [M,K] bf16/int8, Bpacked from repack_b of the full [K,N]."""
    _dev(A, "A"), _dev(Bpacked, "Bpacked")
    M, K = A.shape
    a_dt = dtype_code(A)
    b_dt = a_dt if b_dtype is None else b_dtype
    n1 = N if n1 is None else n1
    s = ep.struct()
    _check(lib().mmx_gemm(a_dt, b_dt, A.data_ptr(), _row_stride_bytes(A), Bpacked.data_ptr(), M, K, N, n0, n1,
                          C.byref(s), _stream()))


def time_gemm(A, Bpacked_list, N, ep, iters, b_dtype=None, n0=0, n1=None):
    """Average ms per launch over `iters` back-to-back launches, rotating over the weight copies."""
    _dev(A, "A")
    M, K = A.shape
    a_dt = dtype_code(A)
    b_dt = a_dt if b_dtype is None else b_dtype
    n1 = N if n1 is None else n1
    s = ep.struct()
    arr = (C.c_void_p * len(Bpacked_list))(*[b.data_ptr() for b in Bpacked_list])
    ms = C.c_float(0)
    _check(lib().mmx_time_gemm(a_dt, b_dt, A.data_ptr(), _row_stride_bytes(A), arr, len(Bpacked_list), M, K, N, n0,
                               n1, C.byref(s), _stream(), iters, C.byref(ms)))
    return ms.value


def probe_mfma(dtype, random_operands, iters=20000):
    """(Tflop/s or Top/s, shader MHz) of an issue-bound loop of independent MFMAs with zero or random operands."""
    scratch = torch.zeros(16 * 1024, dtype=torch.uint8, device="cuda")
    rate, mhz = C.c_float(0), C.c_float(0)
    _check(lib().mmx_probe_mfma(dtype, int(bool(random_operands)), iters, scratch.data_ptr(), _stream(), C.byref(rate),
                                C.byref(mhz)))
    return rate.value, mhz.value


def matvec(A, b, out=None):
    _dev(A, "A"), _dev(b, "b")
    M, K = A.shape
    dt = dtype_code(A)
    if out is None:
        out = torch.empty(M, dtype=torch.float32 if dt == BF16 else torch.int32, device=A.device)
    _check(lib().mmx_matvec(dt, A.data_ptr(), _row_stride_bytes(A), b.data_ptr(), out.data_ptr(), M, K, _stream()))
    return out


def mlp(x, w_gate_up, w_down, N, h=None, y=None):
    _dev(x, "x")
    M, K = x.shape
    if h is None:
        h = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    if y is None:
        y = torch.empty((M, K), dtype=torch.bfloat16, device=x.device)
    _check(lib().mmx_mlp(x.data_ptr(), _row_stride_bytes(x), w_gate_up.data_ptr(), w_down.data_ptr(), h.data_ptr(),
                         _row_stride_bytes(h), y.data_ptr(), _row_stride_bytes(y), M, K, N, _stream()))
    return h, y


def set_tile(shape=""):
    _check(lib().mmx_set_tile(shape.encode()))


def set_option(name, value):
    _check(lib().mmx_set_option(name.encode(), int(value)))


def last_kernel():
    return lib().mmx_last_kernel().decode()
