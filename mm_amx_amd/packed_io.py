"""Packed weights as a file: the natural offline step either side of the path.

The reference repacks (and, for Matmul<bf16,int8,float>, quantises) at the first call of every
process (include/kernels_amx.hpp:1188-1192, 1363-1377).  The packed form of this library is
position independent (MFMA-fragment order, see include/mm_amx_amd.h), so it can be produced once and
loaded straight into HBM: ``save_packed`` writes the packed bytes, the optional per-channel scales and the
geometry into one safetensors file (plain data, nothing executable), ``load_packed`` brings them back
onto a device and checks the geometry against the byte count the library expects.
"""
import json

import torch
from safetensors import safe_open
from safetensors.torch import save_file

from . import _lib as L

FORMAT = "mm_amx_amd.packed_b/1"
_DT = {"bf16": L.BF16, "int8": L.I8, "int4": L.I4}


def save_packed(path, packed, dtype, K, N, scales=None, layout="b", extra=None):
    """packed: uint8 tensor from repack_b / repack_gate_up / quantize_pack_int4; dtype 'bf16', 'int8' or 'int4'; K, N: the logical [K, N]
    of the packed matrix (for a gate/up pair N is 2 x the projection width, layout='gate_up');
    scales: optional fp32 [N] per-output-channel dequantisation scales."""
    if dtype not in _DT:
        raise L.MmxError("dtype must be 'bf16', 'int8' or 'int4'")
    if packed.dtype != torch.uint8 or packed.numel() != L.packed_b_bytes(_DT[dtype], K, N):
        raise L.MmxError("packed does not have the size of a packed [K, N] matrix of this dtype")
    tensors = {"packed": packed.detach().cpu().contiguous()}
    if scales is not None:
        if scales.numel() != N:
            raise L.MmxError("scales must have one entry per output channel")
        tensors["scales"] = scales.detach().to(torch.float32).cpu().contiguous()
    meta = {"format": FORMAT, "dtype": dtype, "K": str(K), "N": str(N), "layout": layout,
            "extra": json.dumps(extra or {})}
    save_file(tensors, path, metadata=meta)


def load_packed(path, device="cuda"):
    """-> dict(packed, scales or None, dtype, K, N, layout, extra) with the tensors on `device`."""
    with safe_open(path, framework="pt", device="cpu") as f:
        meta = f.metadata() or {}
        if meta.get("format") != FORMAT:
            raise L.MmxError(f"{path}: not a packed-weight file of this library")
        dtype, K, N = meta["dtype"], int(meta["K"]), int(meta["N"])
        packed = f.get_tensor("packed")
        scales = f.get_tensor("scales") if "scales" in f.keys() else None
    if dtype not in _DT or packed.dtype != torch.uint8 or packed.numel() != L.packed_b_bytes(_DT[dtype], K, N):
        raise L.MmxError(f"{path}: geometry and byte count disagree")
    return {"packed": packed.to(device), "scales": None if scales is None else scales.to(device), "dtype": dtype, "K": K,
            "N": N, "layout": meta.get("layout", "b"), "extra": json.loads(meta.get("extra", "{}"))}
