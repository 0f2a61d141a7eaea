"""ctypes front end of the CPU oracle (TEST INFRASTRUCTURE ONLY).

Only tests, the smoke check and the benchmark's cpu_baseline leg may import this module; the
product package never does.  bf16 data travels as ``numpy.uint16`` bit patterns.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libfc_oracle.so")
_REF_PATH = os.path.join(_HERE, "_ref", "libmmamx_ref.so")

PP_DEQUANT, PP_BIAS, PP_GELU, PP_QUANT = 1, 2, 4, 8
F32, BF16, I8, I32 = 0, 1, 2, 3
_NP_OF = {F32: np.float32, BF16: np.uint16, I8: np.int8, I32: np.int32}


def build(ref=True):
    """Compile the oracle (and, where the reference checkout exists, the reference shim)."""
    subprocess.check_call(["make", "-C", _HERE, "-s", "all"])
    if ref and os.path.isfile("/root/reference/include/kernels_amx.hpp"):
        subprocess.check_call(["make", "-C", _HERE, "-s", "ref"])


class _PP(C.Structure):
    _fields_ = [("steps", C.c_uint32), ("out_dtype", C.c_int), ("bias", C.c_void_p), ("deq_scale", C.c_float),
                ("deq_per_oc", C.c_void_p), ("q_scale", C.c_float), ("q_per_oc", C.c_void_p)]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.isfile(_LIB_PATH):
            build(ref=False)
        _lib = C.CDLL(_LIB_PATH)
        _lib.orc_f32_to_bf16.restype = C.c_uint16
        _lib.orc_f32_to_bf16.argtypes = [C.c_float]
        _lib.orc_gelu.restype = C.c_float
        _lib.orc_gelu.argtypes = [C.c_float]
        _lib.orc_silu.restype = C.c_float
        _lib.orc_silu.argtypes = [C.c_float]
        _lib.orc_exp_poly.restype = C.c_float
        _lib.orc_exp_poly.argtypes = [C.c_float]
        _lib.orc_quantize_weights.restype = C.c_float
        _lib.orc_isa.restype = C.c_char_p
        for name in ("orc_repack_amx_bytes", "orc_repack_mfma_bytes"):
            getattr(_lib, name).restype = C.c_size_t
    return _lib


def _p(a):
    return None if a is None else C.c_void_p(a.ctypes.data)


def _c(a, dt):
    a = np.ascontiguousarray(a, dtype=dt)
    return a


def f32_to_bf16(x):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    lib().orc_f32_to_bf16_n(_p(x), _p(out), C.c_size_t(x.size))
    return out


def bf16_to_f32(b):
    b = _c(b, np.uint16)
    return (b.astype(np.uint32) << 16).view(np.float32)


def _ld(a):
    assert a.strides[1] == a.itemsize
    return a.strides[0] // a.itemsize


def gemm_bf16(A, B, transB=False, nthreads=0, f64=False):
    """A [M,K] uint16, B [K,N] (or [N,K] if transB) uint16 -> fp32 [M,N] (AMX order)."""
    M, K = A.shape
    N = B.shape[0] if transB else B.shape[1]
    assert (B.shape[1] if transB else B.shape[0]) == K
    Cm = np.empty((M, N), np.float32)
    fn = lib().orc_gemm_bf16_f64 if f64 else lib().orc_gemm_bf16
    fn(_p(A), C.c_int64(_ld(A)), _p(B), C.c_int64(_ld(B)), int(transB), _p(Cm), C.c_int64(N), M, K, N, nthreads)
    return Cm


def gemm_i8(A, B, transB=False, nthreads=0):
    M, K = A.shape
    N = B.shape[0] if transB else B.shape[1]
    Cm = np.empty((M, N), np.int32)
    lib().orc_gemm_i8(_p(A), C.c_int64(_ld(A)), _p(B), C.c_int64(_ld(B)), int(transB), _p(Cm), C.c_int64(N), M, K,
                      N, nthreads)
    return Cm


def gemm_x8(A, B, transB=False):
    """int32 product of int8 / uint8 matrices (the dtype of each array says how its bytes are read)."""
    M, K = A.shape
    N = B.shape[0] if transB else B.shape[1]
    Cm = np.empty((M, N), np.int32)
    lib().orc_gemm_x8(int(A.dtype == np.uint8), int(B.dtype == np.uint8), _p(A), C.c_int64(_ld(A)), _p(B), C.c_int64(_ld(B)),
                      int(transB), _p(Cm), C.c_int64(N), M, K, N)
    return Cm


def matvec_x8(A, b):
    M, K = A.shape
    c = np.empty(M, np.int32)
    lib().orc_matvec_x8(int(A.dtype == np.uint8), int(b.dtype == np.uint8), _p(A), C.c_int64(_ld(A)), _p(b), _p(c), M, K)
    return c


def gemm_i8_generic(A, B, transB=False):
    M, K = A.shape
    N = B.shape[0] if transB else B.shape[1]
    Cm = np.empty((M, N), np.int32)
    lib().orc_gemm_i8_generic(_p(A), C.c_int64(_ld(A)), _p(B), C.c_int64(_ld(B)), int(transB), _p(Cm), C.c_int64(N), M, K, N)
    return Cm


def gelu(x):
    x = _c(x, np.float32)
    out = np.empty_like(x)
    lib().orc_gelu_n(_p(x), _p(out), C.c_size_t(x.size))
    return out


def _map(name, x):
    x = _c(x, np.float32)
    out = np.empty_like(x)
    getattr(lib(), name)(_p(x), _p(out), C.c_size_t(x.size))
    return out


def silu(x):
    return _map("orc_silu_n", x)


def exp_poly(x):
    return _map("orc_exp_poly_n", x)


def rcp14(x):
    """vrcp14ps on every element (software model, see oracle/fc_oracle.c)."""
    return _map("orc_rcp14_n", x)


def pp(acc, steps, out_dtype, bias=None, deq=1.0, deq_per_oc=None, q=0.0, q_per_oc=None):
    """Apply the BiasGeluStore chain to fp32 or int32 accumulators [M,N]."""
    M, N = acc.shape
    keep = [_c(a, np.float32) if a is not None else None for a in (bias, deq_per_oc, q_per_oc)]
    s = _PP(steps, out_dtype, _p(keep[0]), deq, _p(keep[1]), q, _p(keep[2]))
    out = np.empty((M, N), _NP_OF[out_dtype])
    fn = lib().orc_pp_i32 if acc.dtype == np.int32 else lib().orc_pp_f32
    acc = np.ascontiguousarray(acc)
    fn(_p(acc), C.c_int64(N), M, N, C.byref(s), _p(out), C.c_int64(out.strides[0]))
    return out


def repack(B, transpose=False, layout="mfma"):
    """B uint16/int8 [K,N] (or [N,K]) -> flat packed bytes (uint8)."""
    es = B.itemsize
    K, N = (B.shape[1], B.shape[0]) if transpose else B.shape
    nbytes = getattr(lib(), f"orc_repack_{layout}_bytes")(es, K, N)
    out = np.empty(nbytes, np.uint8)
    getattr(lib(), f"orc_repack_{layout}")(es, _p(B), C.c_int64(B.strides[0]), K, N, int(transpose), _p(out))
    return out


def quantize_weights(W):
    W = _c(W, np.uint16)
    Wq = np.empty(W.shape, np.int8)
    qs = C.c_float(0)
    dq = lib().orc_quantize_weights(_p(W), C.c_int64(W.shape[1]), W.shape[0], W.shape[1], _p(Wq),
                                    C.c_int64(W.shape[1]), C.byref(qs))
    return Wq, float(dq), float(qs.value)


def quantize_scale_trunc(W, scale):
    """W bf16 bits [rows, cols] -> int8, q = trunc(bf16_rne(w * scale)): repackB_1xL<int8_t> (fc16m.cpp:80-81)."""
    W = _c(W, np.uint16)
    Wq = np.empty(W.shape, np.int8)
    lib().orc_quantize_scale_trunc(_p(W), C.c_int64(W.shape[1]), W.shape[0], W.shape[1], C.c_float(scale), _p(Wq),
                                   C.c_int64(W.shape[1]))
    return Wq


def repack_1xL_s8(B, L, scale):
    """B bf16 bits [K, N] -> K*N int8 in the order of repackB_1xL<int8_t, L> (fc16m.cpp:61-99)."""
    B = _c(B, np.uint16)
    K, N = B.shape
    assert K % 32 == 0 and N % (16 * L) == 0
    out = np.empty(K * N, np.int8)
    lib().orc_repack_1xL_s8(_p(B), C.c_int64(N), K, N, L, C.c_float(scale), _p(out))
    return out


def quantize_int4(W, transpose=False):
    """W bf16 bits [K,N] (or [N,K] with transpose) -> (q int8 [K,N] in [-7,7], deq fp32 [N])"""
    W = _c(W, np.uint16)
    K, N = (W.shape[1], W.shape[0]) if transpose else W.shape
    q = np.empty((K, N), np.int8)
    deq = np.empty(N, np.float32)
    lib().orc_quantize_int4(_p(W), C.c_int64(W.shape[1]), K, N, int(transpose), _p(q), _p(deq))
    return q, deq


def pack_int4(q):
    q = _c(q, np.int8)
    K, N = q.shape
    lib().orc_pack_int4_bytes.restype = C.c_size_t
    out = np.empty(lib().orc_pack_int4_bytes(K, N), np.uint8)
    lib().orc_pack_int4(_p(q), K, N, _p(out))
    return out


def gemv_w8(x, Wq, scale, transW=False, nthreads=0, want_acc=False):
    M, K = x.shape
    N = Wq.shape[0] if transW else Wq.shape[1]
    y = np.empty((M, N), np.uint16)
    acc = np.empty((M, N), np.float32) if want_acc else None
    scale = _c(scale, np.float32)
    lib().orc_gemv_w8(_p(x), C.c_int64(_ld(x)), _p(Wq), C.c_int64(_ld(Wq)), int(transW), _p(scale), _p(y),
                      C.c_int64(N), _p(acc), M, K, N, nthreads)
    return (y, acc) if want_acc else y


def pack_1x2_s8(Wq):
    """int8 [K, N] -> the stream order of repackB_1xL<int8_t,2> (weight_compression/fc16m.cpp:61-99), K*N bytes."""
    Wq = _c(Wq, np.int8)
    K, N = Wq.shape
    assert K % 32 == 0 and N % 32 == 0
    out = np.empty(K * N, np.int8)
    lib().orc_pack_1x2_s8(_p(Wq), C.c_int64(N), K, N, _p(out))
    return out


def gemv_w8_stream(x, Wpacked, scale, N, nthreads=0):
    """gemv_w8 computed as the reference computes it: packed int8 weights (pack_1x2_s8) read once and converted in
    registers.  Same bits as gemv_w8; this is the form whose time means something."""
    M, K = x.shape
    y = np.empty((M, N), np.uint16)
    scale = _c(scale, np.float32)
    rc = lib().orc_gemv_w8_stream(_p(x), C.c_int64(_ld(x)), _p(Wpacked), _p(scale), _p(y), C.c_int64(N), M, K, N, nthreads)
    if rc != 0:
        raise ValueError("gemv_w8_stream takes K % 32 == 0, N % 32 == 0 and M <= 16")
    return y


def matvec_bf16(A, b, order="amx"):
    M, K = A.shape
    c = np.empty(M, np.float32)
    fn = lib().orc_matvec_bf16 if order == "amx" else lib().orc_gemavb_bf16
    fn(_p(A), C.c_int64(_ld(A)), _p(b), _p(c), M, K)
    return c


def matvec_i8(A, b):
    M, K = A.shape
    c = np.empty(M, np.int32)
    lib().orc_matvec_i8(_p(A), C.c_int64(_ld(A)), _p(b), _p(c), M, K)
    return c


def silu_mul_bf16(gate, up):
    gate, up = _c(gate, np.float32), _c(up, np.float32)
    h = np.empty(gate.shape, np.uint16)
    lib().orc_silu_mul_bf16(_p(gate), _p(up), _p(h), C.c_size_t(gate.size))
    return h


def mlp(x, w_gate, w_up, w_down, split_k=True, nthreads=0):
    """x [M,K]; w_gate,w_up [N,K]; w_down [K,N] (all uint16 bf16 bits) -> (h [M,N], y [M,K])."""
    M, K = x.shape
    N = w_gate.shape[0]
    x, w_gate, w_up, w_down = (_c(a, np.uint16) for a in (x, w_gate, w_up, w_down))
    h = np.empty((M, N), np.uint16)
    y = np.empty((M, K), np.uint16)
    lib().orc_mlp(_p(x), _p(w_gate), _p(w_up), _p(w_down), _p(h), _p(y), M, K, N, int(split_k), nthreads)
    return h, y


def mlp_down(h, w_down, split_k=True, nthreads=0):
    M, N = h.shape
    Kout = w_down.shape[0]
    h, w_down = _c(h, np.uint16), _c(w_down, np.uint16)
    y = np.empty((M, Kout), np.uint16)
    lib().orc_mlp_down(_p(h), _p(w_down), _p(y), M, Kout, N, int(split_k), nthreads)
    return y


def splitter(n, team, tid):
    a, b = C.c_int(0), C.c_int(0)
    lib().orc_splitter(n, team, tid, C.byref(a), C.byref(b))
    return a.value, b.value


def isa():
    return lib().orc_isa().decode()


# ---- the compiled reference (present only where it could be built and AMX exists) ----------
_ref = None


def host_has_amx():
    try:
        with open("/proc/cpuinfo") as f:
            flags = f.read()
        return all(t in flags for t in ("amx_tile", "amx_bf16", "amx_int8", "avx512_bf16"))
    except OSError:
        return False


def ref():
    """The real reference behind C entry points, or None if unavailable on this host."""
    global _ref
    if _ref is None:
        if not (os.path.isfile(_REF_PATH) and host_has_amx()):
            _ref = False
        else:
            r = C.CDLL(_REF_PATH)
            r.ref_fc_w8.restype = C.c_float
            _ref = r if r.ref_init() == 1 else False
    return _ref or None
