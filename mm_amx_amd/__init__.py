"""mm_amx_amd — MI355X (gfx950) fully-connected GEMM path with the mm_amx operator surface.

The compute lives in ``libmm_amx_amd.so`` (hand-written HIP kernels behind a C ABI, see
``include/mm_amx_amd.h``).  This package is the thin Python host layer used by the tests, the
benchmark and the torch-ext-shaped front end: it binds the ABI with ctypes and passes torch
device pointers and the current torch stream through.  There is no CPU or PyTorch fallback:
if the library is missing or a call fails, an exception is raised.
"""
from ._lib import (BF16, F32, I4, I8, I32, U8, gemm_u8, matvec_u8, PP_BIAS, PP_DEQUANT, PP_GELU, PP_NONE, PP_QUANT, PP_SILU_GATE, MmxError,
                   Epilogue, dequant_packed, gemm, gemm_static, gemm_workspace_bytes, init, last_kernel, lib, lib_path, matvec, mlp, packed_b_bytes,
                   quantize_pack_int4, quantize_weights, quantize_weights_scaled, probe_mfma, probe_read, repack_b, repack_gate_up, set_option, set_tile, time_gemm, workspace, release_workspaces)
from .ops import MLP, BiasGeluStore, GemAvB, LinearNxN, Matmul, MatmulVector, Steps, repackB_1x2, repackB_1xL

__all__ = [
    "BF16", "F32", "I8", "I32", "I4", "U8", "gemm_u8", "matvec_u8", "PP_NONE", "PP_DEQUANT", "PP_BIAS", "PP_GELU", "PP_QUANT", "PP_SILU_GATE", "MmxError",
    "Epilogue", "init", "lib", "lib_path", "packed_b_bytes", "repack_b", "repack_gate_up", "quantize_weights",
    "dequant_packed", "gemm", "gemm_static", "gemm_workspace_bytes", "workspace", "release_workspaces", "matvec", "mlp", "set_tile", "set_option", "last_kernel", "time_gemm", "probe_mfma", "probe_read", "quantize_pack_int4", "quantize_weights_scaled", "Steps",
    "BiasGeluStore", "Matmul", "MatmulVector", "GemAvB", "repackB_1x2", "repackB_1xL", "LinearNxN", "MLP",
]
