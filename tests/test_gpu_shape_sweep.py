"""Seeded sweep over shapes for every input type, with the library choosing tile, wave count and K split itself
(a workspace is passed, so every branch of the plan can be taken): accumulators against the CPU oracle, the fused
store against the oracle's post-op on the GPU's own accumulators, and a column range against the whole-N launch.
Integer results bit-exact; floating point within the bar of tests/gpu_util.check_float_parity."""
import numpy as np
import pytest
import torch

from gpu_util import check_float_parity, dev, dev_bf16, host_bits

pytestmark = pytest.mark.gpu

import mm_amx_amd as mx  # noqa: E402
from mm_amx_amd import workloads as wl  # noqa: E402


@pytest.fixture(scope="module")
def ws():
    mx.init(0)
    w = torch.zeros((64 << 20) + (16 << 10), dtype=torch.uint8, device="cuda")
    yield w
    torch.cuda.synchronize()
    assert not w[:16 << 10].any().item(), "the arrival counters must be left at zero"


def _shapes(seed, count):
    """M from decode sizes to several row tiles, K with and without whole 128-byte groups, ragged N."""
    rng = np.random.default_rng(seed)
    out = []
    for i in range(count):
        M = int(rng.choice([1, 2, 7, 16, 32, 33, 48, 100, 128, 129, 200, 256, 300, 384, 520, 640]))
        K = int(rng.choice([64, 128, 200, 256, 320, 512, 1000, 1024, 1536, 2048, 2560, 3072, 4096]))
        N = int(rng.choice([32, 64, 96, 100, 160, 192, 256, 271, 384, 512, 640, 704, 1024]))
        out.append((M, K, N))
    return out


def _bf16(rng, shape, std):
    return wl.f32_to_bf16_bits((rng.standard_normal(shape) * std).astype(np.float32))


@pytest.mark.parametrize("shape", _shapes(1, 28))
def test_sweep_bf16(po, ws, shape):
    M, K, N = shape
    if K < 32:
        pytest.skip("K >= kStep")
    rng = np.random.default_rng(M * 1000003 + K * 1009 + N)
    A, B = _bf16(rng, (M, K), 1.0), _bf16(rng, (K, N), 0.05)
    bias = (rng.standard_normal(N) * 0.1).astype(np.float32)
    Ad, packed = dev_bf16(A), mx.repack_b(dev_bf16(B))
    acc = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    mx.gemm(Ad, packed, N, mx.Epilogue(acc, mx.PP_NONE), ws=ws)
    kernel = mx.last_kernel()
    check_float_parity(host_bits(acc), po.gemm_bf16(A, B), f"bf16 {shape} {kernel}")
    # the fused store = the oracle's post-op on these accumulators (the plan does not depend on the post-op)
    y = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")
    mx.gemm(Ad, packed, N, mx.Epilogue(y, mx.PP_BIAS | mx.PP_GELU, bias=dev(bias)), ws=ws)
    assert mx.last_kernel() == kernel.replace("out_f32", "out_bf16"), (kernel, mx.last_kernel())
    assert np.array_equal(host_bits(y), po.pp(host_bits(acc), po.PP_BIAS | po.PP_GELU, po.BF16, bias=bias)), kernel
    if N >= 96:  # a column range: same bits as the whole launch where it writes, nothing elsewhere
        n0, n1 = 32, N - 7
        part = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
        mx.gemm(Ad, packed, N, mx.Epilogue(part, mx.PP_NONE), n0=n0, n1=n1, ws=ws)
        p = host_bits(part)
        if mx.last_kernel() == kernel:  # (a narrower range may get another tile or split, i.e. another summation order)
            assert np.array_equal(p[:, n0:n1], host_bits(acc)[:, n0:n1]), kernel
        else:
            check_float_parity(p[:, n0:n1], host_bits(acc)[:, n0:n1], f"bf16 range {shape}")
        assert np.isnan(p[:, :n0]).all() and np.isnan(p[:, n1:]).all()


@pytest.mark.parametrize("shape", _shapes(2, 28))
def test_sweep_int8(po, ws, shape):
    M, K, N = shape
    if K < 64:
        pytest.skip("K >= kStep")
    rng = np.random.default_rng(M * 1000003 + K * 1009 + N)
    A = rng.integers(-127, 128, (M, K), dtype=np.int8)
    B = rng.integers(-127, 128, (K, N), dtype=np.int8)
    deq = rng.uniform(1e-5, 1e-4, N).astype(np.float32)
    bias = (rng.standard_normal(N) * 0.1).astype(np.float32)
    Ad, packed = dev(A), mx.repack_b(dev(B))
    acc = torch.full((M, N), -5, dtype=torch.int32, device="cuda")
    mx.gemm(Ad, packed, N, mx.Epilogue(acc, mx.PP_NONE), ws=ws)
    kernel = mx.last_kernel()
    acc_ref = po.gemm_i8(A, B)
    assert np.array_equal(host_bits(acc), acc_ref), kernel
    steps = po.PP_DEQUANT | po.PP_BIAS | po.PP_QUANT
    out = torch.zeros((M, N), dtype=torch.int8, device="cuda")
    mx.gemm(Ad, packed, N, mx.Epilogue(out, mx.PP_DEQUANT | mx.PP_BIAS | mx.PP_QUANT, bias=dev(bias), deq_scale_per_oc=dev(deq), q_scale=20.0),
            ws=ws)
    assert np.array_equal(host_bits(out), po.pp(acc_ref, steps, po.I8, bias=bias, deq_per_oc=deq, q=20.0)), mx.last_kernel()


@pytest.mark.parametrize("shape", _shapes(3, 28))
def test_sweep_int8_weights(po, ws, shape):
    M, K, N = shape
    if K < 32:
        pytest.skip("K >= kStep")
    rng = np.random.default_rng(M * 1000003 + K * 1009 + N)
    A = _bf16(rng, (M, K), 1.0)
    Wq = np.clip(np.rint(rng.standard_normal((K, N)) * 40.0), -127, 127).astype(np.int8)
    scale = rng.uniform(1e-3, 5e-3, N).astype(np.float32)
    _, acc_ref = po.gemv_w8(A, Wq, np.ones(N, np.float32), want_acc=True)
    Ad, packed = dev_bf16(A), mx.repack_b(dev(Wq))
    acc = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    mx.gemm(Ad, packed, N, mx.Epilogue(acc, mx.PP_NONE), b_dtype=mx.I8, ws=ws)
    kernel = mx.last_kernel()
    check_float_parity(host_bits(acc), acc_ref, f"int8 weights {shape} {kernel}")
    y = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")
    mx.gemm(Ad, packed, N, mx.Epilogue(y, mx.PP_DEQUANT, deq_scale_per_oc=dev(scale)), b_dtype=mx.I8, ws=ws)
    assert np.array_equal(host_bits(y), po.pp(host_bits(acc), po.PP_DEQUANT, po.BF16, deq_per_oc=scale)), (kernel, mx.last_kernel())
