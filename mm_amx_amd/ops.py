"""The reference's operator surface on torch device tensors.

Same names, argument meaning and error behaviour as the reference's C++ classes
(include/kernels_amx.hpp) and its torch extension (torch-ext/amx_mlp.cpp), so that a test
written against the reference reads the same here.  Every call ends in the C ABI; nothing is
computed in Python or by PyTorch.
"""
import copy
import enum

import torch

from . import _lib as L


class Steps(enum.IntFlag):
    """amx_kernel::PP::Steps (include/kernels_amx.hpp:540-550)."""
    NONE = 0
    DEQUANT = 1
    BIAS = 2
    GELU = 4
    QUANT = 8
    BIAS_GELU = BIAS | GELU
    DEQUANT_BIAS_GELU = DEQUANT | BIAS_GELU
    DEQUANT_BIAS_GELU_QUANT = DEQUANT_BIAS_GELU | QUANT


class BiasGeluStore:
    """amx_kernel::PP::BiasGeluStore<D, steps> (include/kernels_amx.hpp:552-583).

    D is the dtype of the output tensor C (bf16 / int8 / fp32).  The setters raise if their step is
    not enabled, where the reference asserts.  ``set_deq_scale`` also accepts a per-output-channel
    tensor (an extension; the reference has a per-tensor dequant scale only)."""

    def __init__(self, C, steps=Steps.NONE, bias=None):
        if C.dtype not in (torch.bfloat16, torch.int8, torch.float32):
            raise L.MmxError("BiasGeluStore only supports output dtypes bf16 / int8 / float")
        self.C, self.steps, self.bias = C, Steps(steps), bias
        self.deq_scale, self.deq_scale_per_oc = 1.0, None
        self.q_scale_common, self.q_scale_per_oc = 0.0, None

    def set_bias(self, bias):
        if not self.steps & Steps.BIAS:
            raise L.MmxError("set_bias: BIAS step not enabled")
        self.bias = bias

    def set_deq_scale(self, scale=1.0):
        if not self.steps & Steps.DEQUANT:
            raise L.MmxError("set_deq_scale: DEQUANT step not enabled")
        if isinstance(scale, torch.Tensor):
            self.deq_scale, self.deq_scale_per_oc = 1.0, scale
        else:
            self.deq_scale, self.deq_scale_per_oc = float(scale), None

    def set_q_scale(self, scale):
        if not self.steps & Steps.QUANT:
            raise L.MmxError("set_q_scale: QUANT step not enabled")
        if isinstance(scale, torch.Tensor):
            self.q_scale_common, self.q_scale_per_oc = 0.0, scale
        else:
            self.q_scale_common, self.q_scale_per_oc = float(scale), None

    def descriptor(self):
        return L.Epilogue(self.C, int(self.steps), self.bias, self.deq_scale, self.deq_scale_per_oc,
                          self.q_scale_common, self.q_scale_per_oc)


def repackB_1x2(Bi, transpose=False):
    """amx_kernel::repackB_1x2 (include/kernels_amx.hpp:761-816): the packed form of B, here in
    gfx950 MFMA-fragment order rather than AMX tile order."""
    return L.repack_b(Bi, transpose)


def repackB_1xL(Bi, dtype=torch.bfloat16, L_=2, scale=1.0):
    """repackB_1xL<T, L>(Bi, scale) of weight_compression/fc16m.cpp:61-99: the packed form of the bf16 matrix Bi [K, N]
    for the M <= 16 kernels, as bf16 (T = bfloat16, the scale must be 1 as everywhere in the reference) or compressed to
    int8 on the way (T = int8_t: every weight becomes int8_t(w * scale), i.e. the bf16 product rounded to nearest even,
    then truncated toward zero, :80-81; saturated here where the reference's conversion is undefined).  L (1..4 tiles of
    16 columns side by side) only orders the reference's cache layout; the preconditions are kept (K a multiple of 32,
    N of 16 L) and the result is this library's fragment order, which mmx_gemm takes as b_dtype bf16 or int8."""
    if Bi.dtype != torch.bfloat16 or Bi.dim() != 2:
        raise L.MmxError("repackB_1xL: Bi must be a bf16 [K, N] matrix")
    if L_ not in (1, 2, 3, 4):
        raise L.MmxError("repackB_1xL: L must be 1..4")
    K, N = Bi.shape
    if K % 32 or N % (L_ * 16):
        raise L.MmxError(f"repackB_1xL: K = {K} must be a multiple of 32 and N = {N} of {L_ * 16} (fc16m.cpp:66-67)")
    if dtype == torch.bfloat16:
        if scale != 1.0:
            raise L.MmxError("repackB_1xL: a scale is for the int8 form only")
        return L.repack_b(Bi)
    if dtype == torch.int8:
        return L.repack_b(L.quantize_weights_scaled(Bi, float(scale)))
    raise L.MmxError("repackB_1xL: T is bfloat16 or int8")


class Matmul:
    """amx_kernel::Matmul<TA,TB,TC> (include/kernels_amx.hpp:1045-1315) and its dispatcher in
    main.cpp:32-80.  ``weight_int8=True`` gives Matmul<bf16,int8,float> (:1319-1516): the bf16 B is
    compressed to int8 per tensor on first use and the op sets the post-op's dequant scale.

    The packed weights are cached when ``constB`` (as :1188-1192); otherwise B is repacked on
    every call.  Not thread-safe, like the reference; calls are ordered on the current stream."""

    def __init__(self, constB=False, transposeB=False, weight_int8=False):
        self.constB, self.transposeB, self.weight_int8 = constB, transposeB, weight_int8
        self.internalB = None
        self.quant_scale_B = self.dequant_scale_B = None

    def __call__(self, matA, matB, n0=None, n1=None, ppkernel=None):
        if ppkernel is None:
            raise L.MmxError("Matmul needs a post-op (BiasGeluStore)")
        M, K = matA.shape
        Kb, N = (matB.shape[1], matB.shape[0]) if self.transposeB else matB.shape
        if K != Kb:
            raise L.MmxError(f"Matmul: K of A ({K}) and B ({Kb}) differ")
        kstep = 64 if matA.dtype in (torch.int8, torch.uint8) else 32
        if K < kstep:  # include/kernels_amx.hpp:1183
            raise L.MmxError(f"Matmul: K = {K} must be at least {kstep}")
        n0 = 0 if n0 is None else n0
        n1 = N if n1 is None else n1
        if not self.constB or self.internalB is None:
            if self.weight_int8:
                if matB.dtype != torch.bfloat16:
                    raise L.MmxError("weight-compressed Matmul takes a bf16 B")
                Wq, scales = L.quantize_weights(matB)
                q, dq = scales.tolist()
                self.quant_scale_B, self.dequant_scale_B = q, dq
                self.internalB = L.repack_b(Wq, self.transposeB)
            else:
                self.internalB = L.repack_b(matB, self.transposeB)
        if matA.dtype == torch.uint8 or matB.dtype == torch.uint8:
            # the uint8_t forms of Matmul (tdpbusd / tdpbsud / tdpbuud, include/kernels_amx.hpp:1057-1101)
            L.gemm_u8(matA, self.internalB, N, ppkernel.descriptor(), b_unsigned=matB.dtype == torch.uint8, n0=n0, n1=n1)
        elif self.weight_int8:
            ppkernel.set_deq_scale(self.dequant_scale_B)  # include/kernels_amx.hpp:1379
            # the int8 fragments are converted between LDS and the MFMA operand at every M (:1447-1497); no bf16 copy
            L.gemm(matA, self.internalB, N, ppkernel.descriptor(), b_dtype=L.I8, n0=n0, n1=n1)
        else:
            L.gemm(matA, self.internalB, N, ppkernel.descriptor(), n0=n0, n1=n1)


class MatmulVector:
    """amx_kernel::MatmulVector (include/kernels_amx.hpp:833-1043): c[M] = A[M,K] · b[K]."""

    def __call__(self, matA, vB, vC=None):
        if matA.dtype == torch.uint8 or vB.dtype == torch.uint8:  # is_s8u8 / is_u8s8 / is_u8u8 (:839-850)
            return L.matvec_u8(matA, vB, vC)
        return L.matvec(matA, vB, vC)


class GemAvB(MatmulVector):
    """amx_kernel::GemAvB (include/kernels_amx.hpp:1529-1618); same product, bf16 only."""

    def __call__(self, matA, vecB, vecC=None):
        if matA.dtype != torch.bfloat16:
            raise L.MmxError("GemAvB is bf16 only")
        if matA.shape[1] < 32:  # include/kernels_amx.hpp:1542
            raise L.MmxError("GemAvB: K must be at least 32")
        return L.matvec(matA, vecB, vecC)


class LinearNxN:
    """The torch-ext call shape (torch-ext/amx_mlp.cpp:452-485, bound at :795-804):
    ``set_weight(w[N,K] bf16)`` then ``forward(x[M,K] bf16, y[M,N] fp32)`` writing into the
    caller's y and honouring the row strides of x and y."""

    def __init__(self):
        self.name = ""
        self.m_N = self.m_K = 0
        self._packed = None

    def set_weight(self, weight):
        if weight.dtype != torch.bfloat16:
            raise L.MmxError("set_weight: weight must be bf16")
        if weight.dim() != 2:
            raise L.MmxError("set_weight: weight must be 2-D")
        N, K = weight.shape
        if N % 32 or K % 32:  # torch-ext/amx_mlp.cpp:474-475
            raise L.MmxError("set_weight: N and K must be multiples of 32")
        self.m_N, self.m_K = N, K
        self._packed = L.repack_b(weight, transpose=True)

    def forward(self, x, y):
        if self._packed is None:
            raise L.MmxError("forward: set_weight has not been called")
        if x.dim() != 2 or x.shape[1] != self.m_K:
            raise L.MmxError("forward: x must be [M, K]")
        if y.dtype != torch.float32 or tuple(y.shape) != (x.shape[0], self.m_N):
            raise L.MmxError("forward: y must be fp32 [M, N]")
        L.gemm(x, self._packed, self.m_N, L.Epilogue(y, L.PP_NONE))

    def __deepcopy__(self, memo):
        other = LinearNxN()
        other.name, other.m_N, other.m_K = self.name, self.m_N, self.m_K
        other._packed = None if self._packed is None else self._packed.clone()
        return other


class MLP:
    """AMX_MLP::MLP (tests/amx-mlp.cpp:740-784): ``setup(w_gate[N,K], w_up[N,K], w_down[K,N])``
    (torch nn.Linear.weight layouts), then ``run(x[M,K]) -> y[M,K]`` computing
    bf16(silu(x·Wg^T) * (x·Wu^T)) fused in the gate/up epilogue, then the down projection."""

    def __init__(self):
        self.m_N = self.m_K = 0
        self.gate_up = self.down = None
        self.actUp = None

    def setup(self, w_gate, w_up, w_down):
        N, K = w_gate.shape
        if tuple(w_down.shape) != (K, N):
            raise L.MmxError("setup: w_down must be [K, N]")
        self.m_N, self.m_K = N, K
        self.gate_up = L.repack_gate_up(w_gate, w_up)
        self.down = L.repack_b(w_down, transpose=True)

    def run(self, x, y=None):
        if self.gate_up is None:
            raise L.MmxError("run: setup has not been called")
        if x.dim() != 2 or x.shape[1] != self.m_K:
            raise L.MmxError(f"run: x must be [M, {self.m_K}]")
        M = x.shape[0]
        if self.actUp is None or self.actUp.shape[0] < M:  # setM (tests/amx-mlp.cpp:771-776)
            self.actUp = torch.empty((M, self.m_N), dtype=torch.bfloat16, device=x.device)
        h, y = L.mlp(x, self.gate_up, self.down, self.m_N, h=self.actUp[:M], y=y)
        return y

    def __deepcopy__(self, memo):
        other = MLP()
        other.m_N, other.m_K = self.m_N, self.m_K
        other.gate_up, other.down = copy.deepcopy(self.gate_up), copy.deepcopy(self.down)
        return other
