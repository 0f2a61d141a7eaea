"""Synthetic inputs of the benchmark configurations (seeded; no dataset, no checkpoint).

Arrays are numpy; bf16 tensors are uint16 bit patterns.  The same bytes are handed to the GPU
path and to whatever checks it.
"""
import numpy as np


def f32_to_bf16_bits(x):
    """fp32 -> bf16 bits, round to nearest even (normal numbers; the generators below produce no others)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    bias = np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))
    return ((u + bias) >> np.uint32(16)).astype(np.uint16)


def bf16_bits_to_f32(b):
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


def to_device(a, device="cuda"):
    """numpy array -> torch tensor on the GPU, same bytes."""
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


def to_device_bf16(bits, device="cuda"):
    """uint16 bf16 bit patterns (numpy) -> torch.bfloat16 on the GPU, same bytes."""
    import torch
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).to(device).view(torch.bfloat16)


def _normal_bf16(rng, shape, std):
    return f32_to_bf16_bits((rng.standard_normal(shape, dtype=np.float32) * np.float32(std)))


def gemm_bf16_256(seed=1):
    """bf16 256^3, U[-1,1] inputs, fp32 output, no post-op (shape of tests/amx-l2.cpp)."""
    rng = np.random.default_rng(seed)
    A = f32_to_bf16_bits(rng.uniform(-1, 1, (256, 256)).astype(np.float32))
    B = f32_to_bf16_bits(rng.uniform(-1, 1, (256, 256)).astype(np.float32))
    return dict(A=A, B=B, M=256, K=256, N=256)


def ffn_up_bias_gelu(M=1024, K=4096, N=11008, seed=2):
    """Llama-7B FFN up-projection: A ~N(0,1) bf16 [M,K], B ~N(0,0.02) bf16 [K,N], bias ~N(0,0.1) fp32."""
    rng = np.random.default_rng(seed)
    return dict(A=_normal_bf16(rng, (M, K), 1.0), B=_normal_bf16(rng, (K, N), 0.02),
                bias=(rng.standard_normal(N, dtype=np.float32) * np.float32(0.1)), M=M, K=K, N=N)


def int8_fc(M=512, K=4096, N=4096, seed=3):
    """int8 FC with dequant/bias/requant: per-channel w_scale U[1e-3,1e-2], a_scale 0.02, out scale 0.05."""
    rng = np.random.default_rng(seed)
    A = rng.integers(-127, 128, (M, K), dtype=np.int8)
    B = rng.integers(-127, 128, (K, N), dtype=np.int8)
    w_scale = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
    a_scale = np.float32(0.02)
    deq = (a_scale * w_scale).astype(np.float32)  # one fp32 product per channel, computed once
    bias = (rng.standard_normal(N, dtype=np.float32) * np.float32(0.1))
    return dict(A=A, B=B, deq=deq, bias=bias, q=np.float32(1.0) / np.float32(0.05), M=M, K=K, N=N)


def decode_gemv_w8(M=1, K=4096, N=11008, seed=4):
    """Decode GEMV over int8-compressed weights: x ~N(0,1) bf16, W = clip(round(N(0,40))) int8, scale U[1e-3,5e-3]."""
    rng = np.random.default_rng(seed)
    x = _normal_bf16(rng, (M, K), 1.0)
    W = np.clip(np.rint(rng.standard_normal((K, N), dtype=np.float32) * np.float32(40.0)), -127, 127).astype(np.int8)
    scale = rng.uniform(1e-3, 5e-3, N).astype(np.float32)
    return dict(x=x, W=W, scale=scale, M=M, K=K, N=N)


def llama_mlp(M=2048, K=4096, N=11008, seed=5):
    """Llama-7B MLP: x ~N(0,1); W_gate, W_up [N,K] and W_down [K,N] ~N(0,0.02), torch nn.Linear.weight layouts."""
    rng = np.random.default_rng(seed)
    return dict(x=_normal_bf16(rng, (M, K), 1.0), w_gate=_normal_bf16(rng, (N, K), 0.02),
                w_up=_normal_bf16(rng, (N, K), 0.02), w_down=_normal_bf16(rng, (K, N), 0.02), M=M, K=K, N=N)
