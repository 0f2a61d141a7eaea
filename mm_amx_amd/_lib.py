"""ctypes binding of the C ABI declared in include/mm_amx_amd.h.

Arguments are torch tensors resident on the GPU; only their ``data_ptr()``, strides and the
current torch HIP stream cross the boundary.
"""
import ctypes as C
import os

import torch

F32, BF16, I8, I32, I4, U8 = 0, 1, 2, 3, 4, 5
PP_NONE, PP_DEQUANT, PP_BIAS, PP_GELU, PP_QUANT, PP_SILU_GATE = 0, 1, 2, 4, 8, 16

_HERE = os.path.dirname(os.path.abspath(__file__))
# MMX_LIB_PATH lets a developer point at an alternative build of the same ABI
_LIB_PATH = os.environ.get("MMX_LIB_PATH") or os.path.join(_HERE, "libmm_amx_amd.so")

EXPORTS = ["mmx_last_error", "mmx_init", "mmx_packed_b_bytes", "mmx_repack_b", "mmx_repack_gate_up",
           "mmx_quantize_weights", "mmx_quantize_weights_scaled", "mmx_quantize_pack_int4", "mmx_dequant_packed", "mmx_gemm", "mmx_gemm_splitk",
           "mmx_gemm_splitk_static", "mmx_gemm_workspace_bytes", "mmx_gemm_u8_scratch_bytes", "mmx_gemm_u8", "mmx_matvec_u8", "mmx_matvec", "mmx_mlp", "mmx_mlp_splitk", "mmx_set_tile",
           "mmx_set_option", "mmx_last_kernel"]
# measurement aids (include/mm_amx_amd_bench.h)
BENCH_EXPORTS = ["mmx_time_gemm", "mmx_probe_mfma", "mmx_probe_read"]

# a workspace of this size serves every shape when the library chooses the K split itself (include/mm_amx_amd.h)
WORKSPACE_BYTES = (64 << 20) + (16 << 10)


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
        l.mmx_quantize_weights_scaled.argtypes = [C.c_void_p, C.c_int64, C.c_int, C.c_int, C.c_float, C.c_void_p, C.c_int64,
                                                  C.c_void_p]
        l.mmx_quantize_pack_int4.argtypes = [C.c_void_p, C.c_int64, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p,
                                             C.c_void_p]
        l.mmx_dequant_packed.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
        l.mmx_gemm.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_int64, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int,
                               C.c_int, C.POINTER(_Epilogue), C.c_void_p]
        l.mmx_gemm_splitk.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_int64, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int,
                                      C.c_int, C.POINTER(_Epilogue), C.c_int, C.c_void_p, C.c_size_t, C.c_void_p]
        l.mmx_gemm_splitk_static.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_int64, C.c_void_p, C.c_int, C.c_int, C.c_int,
                                             C.c_int, C.c_int, C.POINTER(_Epilogue), C.c_int, C.c_void_p]
        l.mmx_gemm_workspace_bytes.restype = C.c_size_t
        l.mmx_gemm_workspace_bytes.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_uint32, C.c_int]
        l.mmx_gemm_u8_scratch_bytes.restype = C.c_size_t
        l.mmx_gemm_u8_scratch_bytes.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int]
        l.mmx_gemm_u8.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_int64, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int,
                                  C.POINTER(_Epilogue), C.c_void_p, C.c_size_t, C.c_void_p]
        l.mmx_matvec_u8.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p]
        l.mmx_mlp_splitk.argtypes = [C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p,
                                     C.c_int64, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_size_t, C.c_void_p]
        l.mmx_matvec.argtypes = [C.c_int, C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p]
        l.mmx_mlp.argtypes = [C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p,
                              C.c_int64, C.c_int, C.c_int, C.c_int, C.c_void_p]
        l.mmx_set_tile.argtypes = [C.c_char_p]
        l.mmx_set_option.argtypes = [C.c_char_p, C.c_int]
        l.mmx_time_gemm.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_int64, C.POINTER(C.c_void_p), C.c_int, C.c_int,
                                    C.c_int, C.c_int, C.c_int, C.c_int, C.POINTER(_Epilogue), C.c_int, C.c_void_p, C.c_size_t,
                                    C.c_void_p, C.c_int, C.POINTER(C.c_float)]
        l.mmx_probe_mfma.argtypes = [C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.POINTER(C.c_float),
                                     C.POINTER(C.c_float)]
        l.mmx_probe_read.argtypes = [C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
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


_DT = {torch.float32: F32, torch.bfloat16: BF16, torch.int8: I8, torch.int32: I32, torch.uint8: U8}


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
    """B [K,N] (or [N,K] with transpose) bf16/int8/uint8 on the GPU -> packed weights (uint8 tensor).  uint8 weights
    (for gemm_u8) are stored as u - 128 in the int8 layout."""
    _dev(B, "B")
    dt = dtype_code(B)
    if dt not in (BF16, I8, U8):
        raise MmxError("B must be bf16, int8 or uint8")
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


def quantize_weights_scaled(W, scale):
    """q = trunc(bf16_rne(w * scale)) per element, int8: how repackB_1xL<int8_t> (weight_compression/fc16m.cpp:80-81)
    makes fc16m's int8 weights; the matching per-tensor dequant scale is 1 / scale."""
    _dev(W, "W")
    if W.dtype != torch.bfloat16 or W.dim() != 2:
        raise MmxError("W must be a 2-D bf16 tensor")
    Wq = torch.empty(W.shape, dtype=torch.int8, device=W.device)
    _check(lib().mmx_quantize_weights_scaled(W.data_ptr(), _row_stride_bytes(W), W.shape[0], W.shape[1], float(scale),
                                             Wq.data_ptr(), _row_stride_bytes(Wq), _stream()))
    return Wq


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


_workspaces = {}          # (device, raw stream handle) -> uint8 tensor; insertion order = age
_MAX_WORKSPACES = 8       # stream handles are reused after a stream is destroyed: the cache is bounded


def workspace(device=None, nbytes=WORKSPACE_BYTES):
    """The K-split workspace of the current stream on `device` (zeroed once, when it is created).  Calls
    on one stream are ordered, so one workspace per stream is enough; returns None while the stream is
    being captured into a graph and has no workspace of that size yet (an allocation there would be captured
    too).  At most _MAX_WORKSPACES are kept (the oldest is dropped); release_workspaces() drops them all."""
    dev_index = torch.cuda.current_device() if device is None else (device.index or 0)
    key = (dev_index, torch.cuda.current_stream(dev_index).cuda_stream)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        if torch.cuda.is_current_stream_capturing():
            return None
        ws = torch.zeros(max(nbytes, WORKSPACE_BYTES), dtype=torch.uint8, device=f"cuda:{dev_index}")
        torch.cuda.current_stream(dev_index).synchronize()
        _workspaces.pop(key, None)
        _workspaces[key] = ws
        while len(_workspaces) > _MAX_WORKSPACES:
            _workspaces.pop(next(iter(_workspaces)))
    return ws


def release_workspaces():
    """Drops every cached K-split workspace (the memory returns to torch's allocator once no launch uses it)."""
    _workspaces.clear()


def _is_2d(t, what):
    if not isinstance(t, torch.Tensor) or t.dim() != 2:
        raise MmxError(f"{what} must be a 2-D tensor")


def _check_gemm_args(A, Bpacked, N, ep, b_dt, n0, n1):
    """Host-side checks of everything the kernels take on trust: a wrong size here would be an out-of-bounds
    access on the GPU."""
    _is_2d(A, "A")
    M, K = A.shape
    a_dt = dtype_code(A)
    if a_dt not in (BF16, I8):
        raise MmxError("A must be bf16 or int8")
    if not isinstance(N, int) or N <= 0 or not (0 <= n0 < n1 <= N):
        raise MmxError(f"column range [{n0}, {n1}) outside [0, {N})")
    if not isinstance(Bpacked, torch.Tensor) or Bpacked.dtype != torch.uint8 or not Bpacked.is_contiguous():
        raise MmxError("Bpacked must be a contiguous uint8 tensor (from repack_b)")
    need = _packed_bytes_host(b_dt, K, N)
    if Bpacked.numel() < need:
        raise MmxError(f"Bpacked holds {Bpacked.numel()} bytes, a packed [{K}, {N}] matrix takes {need}")
    Cout = ep.C
    _is_2d(Cout, "C")
    ncols = n1 // 2 if ep.steps & PP_SILU_GATE else n1
    if Cout.shape[0] < M or Cout.shape[1] < ncols:
        raise MmxError(f"C is {tuple(Cout.shape)}, the result needs at least [{M}, {ncols}]")
    for v, name in ((ep.bias, "bias"), (ep.deq_oc, "deq_scale_per_oc"), (ep.q_oc, "q_scale_per_oc")):
        if v is not None and v.numel() < n1:
            raise MmxError(f"{name} holds {v.numel()} values, columns up to {n1} are computed")
    return M, K, a_dt


def _packed_bytes_host(dtype, K, N):
    """mmx_packed_b_bytes restated on the host (so that arguments can be checked before the library is loaded)."""
    if K <= 0 or N <= 0:
        return 0
    if dtype == I4:
        return ((N + 31) // 32) * ((K + 255) // 256 * 4) * 1024
    es = {BF16: 2, I8: 1, U8: 1}.get(dtype, 0)
    return ((N + 31) // 32) * 32 * ((K * es + 127) // 128 * 128)


def _split_args(A, k_splits, ws, need):
    """(k_splits, workspace pointer, bytes).  Without an explicit workspace the stream's own one is used, and it is
    only created when the library says the call can use one (`need` = mmx_gemm_workspace_bytes of the call, a
    callable): a shape that never splits allocates nothing."""
    if k_splits == 1 and ws is None:
        return 1, None, 0
    if ws is None:
        nbytes = need()
        if nbytes == 0 and k_splits == 0:
            return 1, None, 0
        ws = workspace(A.device, max(nbytes, 1))  # (an explicit count that does not fit: the library says why)
    if ws is None:
        if k_splits > 1:
            raise MmxError("a K split needs a workspace, and none can be allocated while the stream is being captured")
        return 1, None, 0
    if ws.dtype != torch.uint8 or not ws.is_cuda or not ws.is_contiguous():
        raise MmxError("the workspace must be a contiguous uint8 tensor on the GPU")
    return k_splits, ws.data_ptr(), ws.numel()


def gemm(A, Bpacked, N, ep, b_dtype=None, n0=0, n1=None, k_splits=0, ws=None):
    """C[:, n0:n1] = PP(A · B[:, n0:n1]); A [M,K] bf16/int8, Bpacked from repack_b of the full [K,N].
    k_splits: 0 = the library decides whether to split K over several workgroups per tile, 1 = never,
    2..4 = exactly that many slices; ws = the workspace for the partial sums (default: the stream's own, created at
    the first call that can use one).  A first call of a shape made while the stream is being captured into a graph
    finds no workspace and runs unsplit: its sums can differ in the last bits from an eager call of the same shape,
    which splits.  Call the shape once eagerly before capturing (or pass ws) to have both take the same form."""
    n1 = N if n1 is None else n1
    b_dt = (dtype_code(A) if isinstance(A, torch.Tensor) else None) if b_dtype is None else b_dtype
    M, K, a_dt = _check_gemm_args(A, Bpacked, N, ep, b_dt, n0, n1)
    _dev(A, "A"), _dev(Bpacked, "Bpacked")
    s = ep.struct()
    ks, wsp, wsb = _split_args(A, k_splits, ws, lambda: gemm_workspace_bytes(a_dt, b_dt, M, K, N, ep.steps, k_splits, n0, n1))
    _check(lib().mmx_gemm_splitk(a_dt, b_dt, A.data_ptr(), _row_stride_bytes(A), Bpacked.data_ptr(), M, K, N, n0, n1,
                                 C.byref(s), ks, wsp, wsb, _stream()))


def gemm_static(A, Bpacked, N, ep, b_dtype=None, n0=0, n1=None, k_splits=0):
    """gemm() on the workspace built into the library (mmx_gemm_splitk_static): allocates nothing."""
    n1 = N if n1 is None else n1
    b_dt = (dtype_code(A) if isinstance(A, torch.Tensor) else None) if b_dtype is None else b_dtype
    M, K, a_dt = _check_gemm_args(A, Bpacked, N, ep, b_dt, n0, n1)
    _dev(A, "A"), _dev(Bpacked, "Bpacked")
    s = ep.struct()
    _check(lib().mmx_gemm_splitk_static(a_dt, b_dt, A.data_ptr(), _row_stride_bytes(A), Bpacked.data_ptr(), M, K, N, n0, n1,
                                        C.byref(s), k_splits, _stream()))


def gemm_u8(A, Bpacked, N, ep, b_unsigned, n0=0, n1=None, scratch=None):
    """The int8 GEMM with unsigned bytes in A (a uint8 tensor) and/or in the weights (b_unsigned: Bpacked comes from
    repack_b of a uint8 matrix): mmx_gemm_u8.  scratch: a uint8 tensor of gemm_u8_scratch_bytes() bytes (made here if
    not given)."""
    n1 = N if n1 is None else n1
    _is_2d(A, "A")
    if A.dtype not in (torch.int8, torch.uint8):
        raise MmxError("A must be int8 or uint8")
    a_dt, b_dt = dtype_code(A), (U8 if b_unsigned else I8)
    if a_dt != U8 and b_dt != U8:
        raise MmxError("gemm_u8 is for unsigned operands: use gemm for int8 x int8")
    M, K = A.shape
    view = A.view(torch.int8) if A.dtype == torch.uint8 else A
    _check_gemm_args(view, Bpacked, N, ep, I8, n0, n1)
    _dev(A, "A"), _dev(Bpacked, "Bpacked")
    need = lib().mmx_gemm_u8_scratch_bytes(a_dt, b_dt, M, K, N, n0, n1)
    if scratch is None:
        scratch = torch.empty(need, dtype=torch.uint8, device=A.device)
    if scratch.dtype != torch.uint8 or not scratch.is_cuda or not scratch.is_contiguous() or scratch.numel() < need:
        raise MmxError(f"scratch must be a contiguous uint8 tensor of at least {need} bytes on the GPU")
    s = ep.struct()
    _check(lib().mmx_gemm_u8(a_dt, b_dt, A.data_ptr(), _row_stride_bytes(A), Bpacked.data_ptr(), M, K, N, n0, n1, C.byref(s),
                             scratch.data_ptr(), scratch.numel(), _stream()))


def matvec_u8(A, b, out=None):
    """c[M] (int32) = A[M,K] . b[K], A and b each int8 or uint8, at least one uint8 (mmx_matvec_u8)."""
    _is_2d(A, "A")
    M, K = A.shape
    if A.dtype not in (torch.int8, torch.uint8) or not isinstance(b, torch.Tensor) or b.dtype not in (torch.int8, torch.uint8):
        raise MmxError("A and b must be int8 or uint8")
    if A.dtype != torch.uint8 and b.dtype != torch.uint8:
        raise MmxError("matvec_u8 is for unsigned operands: use matvec for int8 x int8")
    if b.numel() != K or not b.is_contiguous():
        raise MmxError(f"b must be a contiguous vector of K = {K} elements")
    if out is not None and (out.dtype != torch.int32 or out.numel() < M or not out.is_contiguous()):
        raise MmxError(f"out must be a contiguous int32 vector of at least M = {M} elements")
    _dev(A, "A"), _dev(b, "b")
    if out is None:
        out = torch.empty(M, dtype=torch.int32, device=A.device)
    _check(lib().mmx_matvec_u8(dtype_code(A), dtype_code(b), A.data_ptr(), _row_stride_bytes(A), b.data_ptr(), out.data_ptr(), M, K,
                               _stream()))
    return out


def gemm_workspace_bytes(a_dtype, b_dtype, M, K, N, steps=PP_NONE, k_splits=0, n0=0, n1=None):
    return lib().mmx_gemm_workspace_bytes(a_dtype, b_dtype, M, K, N, n0, N if n1 is None else n1, int(steps), k_splits)


def time_gemm(A, Bpacked_list, N, ep, iters, b_dtype=None, n0=0, n1=None, k_splits=0, ws=None):
    """Average ms per launch over `iters` back-to-back launches, rotating over the weight copies."""
    n1 = N if n1 is None else n1
    b_dt = (dtype_code(A) if isinstance(A, torch.Tensor) else None) if b_dtype is None else b_dtype
    for Bp in Bpacked_list:
        M, K, a_dt = _check_gemm_args(A, Bp, N, ep, b_dt, n0, n1)
        _dev(Bp, "Bpacked")
    _dev(A, "A")
    s = ep.struct()
    arr = (C.c_void_p * len(Bpacked_list))(*[b.data_ptr() for b in Bpacked_list])
    ms = C.c_float(0)
    ks, wsp, wsb = _split_args(A, k_splits, ws, lambda: gemm_workspace_bytes(a_dt, b_dt, M, K, N, ep.steps, k_splits, n0, n1))
    _check(lib().mmx_time_gemm(a_dt, b_dt, A.data_ptr(), _row_stride_bytes(A), arr, len(Bpacked_list), M, K, N, n0,
                               n1, C.byref(s), ks, wsp, wsb, _stream(), iters, C.byref(ms)))
    return ms.value


def probe_mfma(dtype, random_operands, iters=20000):
    """(Tflop/s or Top/s, shader MHz) of an issue-bound loop of independent MFMAs with zero or random operands."""
    scratch = torch.zeros(16 * 1024, dtype=torch.uint8, device="cuda")
    rate, mhz = C.c_float(0), C.c_float(0)
    _check(lib().mmx_probe_mfma(dtype, int(bool(random_operands)), iters, scratch.data_ptr(), _stream(), C.byref(rate),
                                C.byref(mhz)))
    return rate.value, mhz.value


def probe_read(buf, workgroups, kib_in_flight, sink, waves=8, blocked=False):
    """One launch of the read-only kernel over the uint8 tensor `buf` (asynchronous; see mm_amx_amd_bench.h)."""
    _check(lib().mmx_probe_read(buf.data_ptr(), buf.numel(), int(workgroups), int(waves), int(bool(blocked)), int(kib_in_flight),
                                sink.data_ptr(), _stream()))


def matvec(A, b, out=None):
    """c[M] = A[M,K] · b[K]; bf16 (c fp32) or int8 (c int32)."""
    _is_2d(A, "A")
    M, K = A.shape
    dt = dtype_code(A)
    if dt not in (BF16, I8):
        raise MmxError("A must be bf16 or int8")
    if not isinstance(b, torch.Tensor) or b.dtype != A.dtype or b.numel() != K or not b.is_contiguous():
        raise MmxError(f"b must be a contiguous {A.dtype} vector of K = {K} elements")
    want = torch.float32 if dt == BF16 else torch.int32
    if out is not None and (out.dtype != want or out.numel() < M or not out.is_contiguous()):
        raise MmxError(f"out must be a contiguous {want} vector of at least M = {M} elements")
    _dev(A, "A"), _dev(b, "b")
    if out is None:
        out = torch.empty(M, dtype=want, device=A.device)
    _dev(out, "out")
    _check(lib().mmx_matvec(dt, A.data_ptr(), _row_stride_bytes(A), b.data_ptr(), out.data_ptr(), M, K, _stream()))
    return out


def mlp(x, w_gate_up, w_down, N, h=None, y=None, down_k_splits=0, ws=None):
    """h = bf16(silu(x·Wg) * (x·Wu)), y = bf16(h·Wd): x [M,K] bf16, w_gate_up from repack_gate_up, w_down from
    repack_b(transpose=True) of the [K,N] down_proj weight.  down_k_splits: K slices of the down projection
    (0 = the library chooses, 1 = none, 2 = the reference's two-way split)."""
    _is_2d(x, "x")
    M, K = x.shape
    if x.dtype != torch.bfloat16:
        raise MmxError("x must be bf16")
    if not isinstance(N, int) or N <= 0 or N % 32:
        raise MmxError("N must be a positive multiple of 32")
    for t, name, need in ((w_gate_up, "w_gate_up", _packed_bytes_host(BF16, K, 2 * N)), (w_down, "w_down", _packed_bytes_host(BF16, N, K))):
        if not isinstance(t, torch.Tensor) or t.dtype != torch.uint8 or not t.is_contiguous() or t.numel() < need:
            raise MmxError(f"{name} must be a contiguous uint8 tensor of at least {need} bytes (packed weights)")
    for t, name, cols in ((h, "h", N), (y, "y", K)):
        if t is not None:
            _is_2d(t, name)
            if t.dtype != torch.bfloat16 or t.shape[0] < M or t.shape[1] < cols:
                raise MmxError(f"{name} must be bf16 of at least [{M}, {cols}]")
    _dev(x, "x"), _dev(w_gate_up, "w_gate_up"), _dev(w_down, "w_down")
    if h is None:
        h = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    if y is None:
        y = torch.empty((M, K), dtype=torch.bfloat16, device=x.device)
    _dev(h, "h"), _dev(y, "y")
    # the down projection is the GEMM [M, N] x [N, K]; decode shapes (M <= 32) choose their own slices
    ks, wsp, wsb = _split_args(x, down_k_splits, ws,
                               lambda: gemm_workspace_bytes(BF16, BF16, M, N, K, PP_NONE, 0 if M <= 32 else down_k_splits))
    _check(lib().mmx_mlp_splitk(x.data_ptr(), _row_stride_bytes(x), w_gate_up.data_ptr(), w_down.data_ptr(), h.data_ptr(),
                                _row_stride_bytes(h), y.data_ptr(), _row_stride_bytes(y), M, K, N, ks, wsp, wsb, _stream()))
    return h, y


def set_tile(shape=""):
    _check(lib().mmx_set_tile(shape.encode()))


def set_option(name, value):
    _check(lib().mmx_set_option(name.encode(), int(value)))


def last_kernel():
    return lib().mmx_last_kernel().decode()
