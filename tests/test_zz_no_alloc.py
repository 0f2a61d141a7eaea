"""The entry point that allocates nothing (mmx_gemm_splitk_static): same results as mmx_gemm_splitk with a caller's
workspace of the same size, on two calls in a row, the second with a smaller input."""
import contextlib

import numpy as np
import pytest
import torch

from gpu_util import dev, dev_bf16, host_bits

pytestmark = pytest.mark.gpu

import mm_amx_amd as mx  # noqa: E402
from mm_amx_amd import _lib as L  # noqa: E402
from mm_amx_amd import workloads as wl  # noqa: E402


@contextlib.contextmanager
def _no_device_allocation():
    """The free device memory as the driver reports it (hipMemGetInfo: it sees every hipMalloc and hipFree of the process,
    also those that do not go through torch's caching allocator) and torch's own counter must both be unchanged by the
    calls inside; the queue is drained on either side so that nothing in flight holds memory."""
    torch.cuda.synchronize()
    free0, torch0 = torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated()
    yield
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == torch0
    assert torch.cuda.mem_get_info()[0] >= free0, (free0, torch.cuda.mem_get_info()[0])   # (an allocation would lower it)


def _int8_case(po, M, K, N, seed, k_splits, ws):
    rng = np.random.default_rng(seed)
    A = rng.integers(-127, 128, (M, K), dtype=np.int8)
    B = rng.integers(-127, 128, (K, N), dtype=np.int8)
    deq = (np.float32(0.02) * rng.uniform(1e-3, 1e-2, N).astype(np.float32)).astype(np.float32)
    bias = (rng.standard_normal(N) * 0.1).astype(np.float32)
    steps = po.PP_DEQUANT | po.PP_BIAS | po.PP_QUANT
    Ad, packed = dev(A), mx.repack_b(dev(B))
    kw = dict(bias=dev(bias), deq_scale_per_oc=dev(deq), q_scale=20.0)
    want = torch.zeros((M, N), dtype=torch.int8, device="cuda")
    mx.gemm(Ad, packed, N, mx.Epilogue(want, steps, **kw), k_splits=k_splits, ws=ws)
    k_want = mx.last_kernel()
    got = torch.full((M, N), 77, dtype=torch.int8, device="cuda")
    ep_got = mx.Epilogue(got, steps, **kw)
    with _no_device_allocation():
        mx.gemm_static(Ad, packed, N, ep_got, k_splits=k_splits)
    assert mx.last_kernel() == k_want
    assert np.array_equal(host_bits(got), host_bits(want)), (M, K, N, k_want)
    assert np.array_equal(host_bits(got), po.pp(po.gemm_i8(A, B), steps, po.I8, bias=bias, deq_per_oc=deq, q=20.0))
    return k_want


def _bf16_case(po, M, K, N, seed, k_splits, ws):
    rng = np.random.default_rng(seed)
    A = wl.f32_to_bf16_bits(rng.standard_normal((M, K)).astype(np.float32))
    B = wl.f32_to_bf16_bits((rng.standard_normal((K, N)) * 0.05).astype(np.float32))
    bias = (rng.standard_normal(N) * 0.1).astype(np.float32)
    Ad, packed, bd = dev_bf16(A), mx.repack_b(dev_bf16(B)), dev(bias)
    want = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")
    mx.gemm(Ad, packed, N, mx.Epilogue(want, mx.PP_BIAS | mx.PP_GELU, bias=bd), k_splits=k_splits, ws=ws)
    k_want = mx.last_kernel()
    got = torch.full((M, N), 3.0, dtype=torch.bfloat16, device="cuda")
    ep_got = mx.Epilogue(got, mx.PP_BIAS | mx.PP_GELU, bias=bd)
    with _no_device_allocation():
        mx.gemm_static(Ad, packed, N, ep_got, k_splits=k_splits)
    assert mx.last_kernel() == k_want
    # the same plan adds the same partial sums in the same order: the bits agree, not just the values
    assert np.array_equal(host_bits(got), host_bits(want)), (M, K, N, k_want)
    return k_want


def test_static_workspace_entry_point_matches_the_workspace_one(po):
    mx.init(0)
    ws = torch.zeros(L.WORKSPACE_BYTES, dtype=torch.uint8, device="cuda")
    # two calls in a row, the second smaller: it finds the partial sums of the first still in the array
    k1 = _int8_case(po, 520, 4096, 704, 1, 4, ws)
    k2 = _int8_case(po, 130, 1024, 200, 2, 2, ws)
    assert "ksplit4" in k1 and "ksplit2" in k2
    k3 = _bf16_case(po, 600, 2048, 832, 3, 3, ws)
    k4 = _bf16_case(po, 100, 1024, 96, 4, 2, ws)
    assert "ksplit3" in k3 and "ksplit2" in k4
    # the library's own choice (k_splits = 0): a shape with few tiles is split, a decode shape is not
    k5 = _bf16_case(po, 64, 4096, 512, 5, 0, ws)
    k6 = _bf16_case(po, 8, 1024, 256, 6, 0, ws)
    assert "ksplit" in k5 and "skinny" in k6, (k5, k6)
    # decode shapes with few panels of a long K: the chunked kernel's own K split parks its sums in the same array
    k7 = _bf16_case(po, 24, 8192, 512, 7, 0, ws)
    k8 = _int8_case(po, 24, 8192, 512, 8, 0, ws)
    k9 = _bf16_case(po, 12, 4096, 96, 9, 0, ws)       # ... and a smaller one after them
    assert k7.startswith("skinny_chunk_bf16_ksplit") and k8.startswith("skinny_chunk_i8_ksplit") and "skinny" in k9, (k7, k8, k9)
    torch.cuda.synchronize()
    assert not ws[:16 << 10].any().item()


def test_static_workspace_entry_point_replays_from_a_hip_graph(po):
    """One call of the entry point captured into a HIP graph after a warm-up call (capture forbids allocation, so a
    capture that succeeds is itself the check) and replayed with new inputs: every replay gives the bits of an eager
    call with a caller's workspace."""
    mx.init(0)
    M, K, N, S = 200, 4096, 640, 2
    rng = np.random.default_rng(77)
    B = wl.f32_to_bf16_bits((rng.standard_normal((K, N)) * 0.05).astype(np.float32))
    bias = (rng.standard_normal(N) * 0.1).astype(np.float32)
    packed, bd = mx.repack_b(dev_bf16(B)), dev(bias)
    x = dev_bf16(wl.f32_to_bf16_bits(rng.standard_normal((M, K)).astype(np.float32))).clone()
    y = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")
    ep = mx.Epilogue(y, mx.PP_BIAS | mx.PP_GELU, bias=bd)
    ws = torch.zeros(L.WORKSPACE_BYTES, dtype=torch.uint8, device="cuda")
    g = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        mx.gemm_static(x, packed, N, ep, k_splits=S)   # warm-up on the capture stream
        side.synchronize()
        with torch.cuda.graph(g, stream=side):
            mx.gemm_static(x, packed, N, ep, k_splits=S)
    assert f"ksplit{S}" in mx.last_kernel()
    torch.cuda.synchronize()
    for rep in range(3):
        x.copy_(dev_bf16(wl.f32_to_bf16_bits(rng.standard_normal((M, K)).astype(np.float32))))
        y.zero_()
        if rep == 0:
            g.replay()              # (the runtime may set a graph up on its first launch)
            torch.cuda.synchronize()
        else:
            with _no_device_allocation():
                g.replay()
        got = host_bits(y).copy()
        y2 = torch.zeros_like(y)
        mx.gemm(x, packed, N, mx.Epilogue(y2, mx.PP_BIAS | mx.PP_GELU, bias=bd), k_splits=S, ws=ws)
        torch.cuda.synchronize()
        assert np.array_equal(got, host_bits(y2)), rep


def test_static_workspace_rejects_what_does_not_fit():
    mx.init(0)
    M, K, N = 4096, 4096, 8192   # four int32 partial copies of a 4096 x 8192 result: 512 MiB, whatever the tile
    A = torch.zeros((M, K), dtype=torch.int8, device="cuda")
    packed = mx.repack_b(torch.zeros((K, N), dtype=torch.int8, device="cuda"))
    out = torch.zeros((M, N), dtype=torch.int8, device="cuda")
    with pytest.raises(mx.MmxError, match="built-in one holds"):
        mx.gemm_static(A, packed, N, mx.Epilogue(out, mx.PP_NONE | mx.PP_QUANT, q_scale=1.0), k_splits=4)
    mx.gemm_static(A, packed, N, mx.Epilogue(out, mx.PP_QUANT, q_scale=1.0))   # the library's own choice always fits
    torch.cuda.synchronize()
