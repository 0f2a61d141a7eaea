"""Over-read and over-write detection, after the reference's own device: it writes a NaN/Inf sentinel behind the
last element of every tensor2D (include/tensor2D.hpp:116-125) and keeps its K-tail logic from ever loading it
(include/kernels_amx.hpp:1179-1186).  Here every operand lives inside a larger buffer whose surroundings - the padding
of every row, a row in front and a row behind - hold NaN (bf16) or random bytes (int8), and the output inside a buffer
of canaries: the result must be bit-identical to the one from clean, compact operands, and no canary may change."""
import numpy as np
import pytest
import torch

from gpu_util import dev, dev_bf16, host_bits

pytestmark = pytest.mark.gpu

import mm_amx_amd as mx  # noqa: E402
from mm_amx_amd import workloads as wl  # noqa: E402

NAN_BF16 = 0x7FC0


def _embed(rng, inner, pad_cols, fill):
    """inner [R, C] inside a [R + 2, C + pad_cols] buffer of `fill` (a value, or "random" for int8): returns the big host
    array and the slice that holds inner."""
    R, C = inner.shape
    if isinstance(fill, str):
        big = rng.integers(-128, 128, (R + 2, C + pad_cols)).astype(inner.dtype)
    else:
        big = np.full((R + 2, C + pad_cols), fill, dtype=inner.dtype)
    big[1:R + 1, :C] = inner
    return big, (slice(1, R + 1), slice(0, C))


def _canary_out(M, N, pad_cols, dtype, canary):
    big = torch.full((M + 2, N + pad_cols), canary, dtype=dtype, device="cuda")
    return big, big[1:M + 1, :N]


def _canaries_intact(big, M, N, canary):
    b = big.clone()
    b[1:M + 1, :N] = canary
    return bool((b == canary).all().item())


BF16_SHAPES = [(16, 65, 32), (16, 69, 32), (2, 128, 5), (33, 1024, 17), (128, 96, 16), (200, 512, 320), (256, 1024, 384), (735, 337, 271),
               (1, 4096, 352), (4, 2560, 192), (16, 4096, 704), (24, 8192, 512), (12, 11008, 256)]


@pytest.mark.parametrize("shape", BF16_SHAPES)
@pytest.mark.parametrize("pad", [8, 3])   # 8 elements keep the rows 16-byte aligned (fast kernels), 3 do not (masked / general ones)
def test_bf16_operands_among_nans(shape, pad):
    M, K, N = shape
    rng = np.random.default_rng(M * 7 + K * 3 + N + pad)
    A = wl.f32_to_bf16_bits(rng.standard_normal((M, K)).astype(np.float32))
    B = wl.f32_to_bf16_bits((rng.standard_normal((K, N)) * 0.05).astype(np.float32))
    bias = rng.standard_normal(N).astype(np.float32)
    bigA, sa = _embed(rng, A, pad, NAN_BF16)
    bigB, sb = _embed(rng, B, pad, NAN_BF16)
    Ad, Bd = dev_bf16(bigA)[sa], dev_bf16(bigB)[sb]
    bd = dev(bias)
    # clean run: compact operands, compact output
    want = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")
    mx.gemm(dev_bf16(A), mx.repack_b(dev_bf16(B)), N, mx.Epilogue(want, mx.PP_BIAS | mx.PP_GELU, bias=bd))
    k_clean = mx.last_kernel()
    # the same product from operands surrounded by NaN, into an output surrounded by canaries
    packed = mx.repack_b(Bd)
    assert np.array_equal(host_bits(packed), host_bits(mx.repack_b(dev_bf16(B)))), "the repack read a sentinel"
    bigC, C = _canary_out(M, N, pad, torch.bfloat16, 77.0)
    mx.gemm(Ad, packed, N, mx.Epilogue(C, mx.PP_BIAS | mx.PP_GELU, bias=bd))
    got = host_bits(C)
    f = (got.astype(np.uint32) << 16).view(np.float32)
    assert np.isfinite(f).all(), f"a sentinel entered the result ({mx.last_kernel()})"
    if mx.last_kernel() == k_clean:
        assert np.array_equal(got, host_bits(want)), mx.last_kernel()
    else:   # (unaligned rows take another kernel, whose sums may differ in the last bits)
        w = (host_bits(want).astype(np.uint32) << 16).view(np.float32)
        assert (np.abs(f - w) <= np.maximum(np.abs(w), 1.0) * 2.0 ** -6).all(), (k_clean, mx.last_kernel())
    assert _canaries_intact(bigC, M, N, 77.0), f"{mx.last_kernel()} wrote outside its output"


INT8_SHAPES = [(16, 65, 32), (77, 200, 95), (256, 512, 320), (512, 1024, 256), (1, 4096, 352), (16, 4096, 704), (24, 8192, 512)]


@pytest.mark.parametrize("shape", INT8_SHAPES)
@pytest.mark.parametrize("pad", [16, 5])
def test_int8_operands_among_random_bytes(shape, pad):
    M, K, N = shape
    rng = np.random.default_rng(M * 5 + K + N * 3 + pad)
    A = rng.integers(-127, 128, (M, K), dtype=np.int8)
    B = rng.integers(-127, 128, (K, N), dtype=np.int8)
    bigA, sa = _embed(rng, A, pad, "random")
    bigB, sb = _embed(rng, B, pad, "random")
    want = torch.zeros((M, N), dtype=torch.int32, device="cuda")
    mx.gemm(dev(A), mx.repack_b(dev(B)), N, mx.Epilogue(want, mx.PP_NONE))
    packed = mx.repack_b(dev(bigB)[sb])
    assert np.array_equal(host_bits(packed), host_bits(mx.repack_b(dev(B)))), "the repack read a byte outside B"
    bigC, C = _canary_out(M, N, 3, torch.int32, -123456789)
    mx.gemm(dev(bigA)[sa], packed, N, mx.Epilogue(C, mx.PP_NONE))
    assert np.array_equal(host_bits(C), host_bits(want)), mx.last_kernel()   # int32 sums: exact whatever the kernel
    assert _canaries_intact(bigC, M, N, -123456789), f"{mx.last_kernel()} wrote outside its output"


@pytest.mark.parametrize("shape", [(1, 4096, 352), (4, 2560, 192), (16, 4096, 704), (10, 4096, 8192), (24, 8192, 512), (3, 300, 77)])
def test_decode_over_int8_weights_with_x_among_nans(shape):
    """The decode kernels stage x through LDS in whole pieces and clamp at the end of K: x sits among NaN, the
    per-channel scales inside a buffer of NaN as well."""
    M, K, N = shape
    rng = np.random.default_rng(M + K + N)
    x = wl.f32_to_bf16_bits(rng.standard_normal((M, K)).astype(np.float32))
    W = rng.integers(-127, 128, (K, N), dtype=np.int8)
    scale = rng.uniform(1e-3, 5e-3, N).astype(np.float32)
    packed = mx.repack_b(dev(W))
    want = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")
    mx.gemm(dev_bf16(x), packed, N, mx.Epilogue(want, mx.PP_DEQUANT, deq_scale_per_oc=dev(scale)), b_dtype=mx.I8)
    k_clean = mx.last_kernel()
    bigx, sx = _embed(rng, x, 8, NAN_BF16)
    bigs = np.full(N + 64, np.nan, dtype=np.float32)
    bigs[32:32 + N] = scale
    bigC, C = _canary_out(M, N, 8, torch.bfloat16, 77.0)
    mx.gemm(dev_bf16(bigx)[sx], packed, N, mx.Epilogue(C, mx.PP_DEQUANT, deq_scale_per_oc=dev(bigs)[32:32 + N]), b_dtype=mx.I8)
    assert mx.last_kernel() == k_clean
    assert np.array_equal(host_bits(C), host_bits(want)), k_clean
    assert _canaries_intact(bigC, M, N, 77.0), f"{k_clean} wrote outside its output"


@pytest.mark.parametrize("M", [1, 4, 24, 96, 300])
def test_mlp_among_nans(M):
    """The fused MLP (gate/up with the SiLU-gate store, then down): x, both weight sources and both outputs sit among
    sentinels; h and y equal the clean run's bits."""
    K, N = 512, 1024
    rng = np.random.default_rng(M)
    x = wl.f32_to_bf16_bits(rng.standard_normal((M, K)).astype(np.float32))
    wg, wu = (wl.f32_to_bf16_bits((rng.standard_normal((N, K)) * 0.05).astype(np.float32)) for _ in range(2))
    wd = wl.f32_to_bf16_bits((rng.standard_normal((K, N)) * 0.05).astype(np.float32))
    gu = mx.repack_gate_up(dev_bf16(wg), dev_bf16(wu))
    dn = mx.repack_b(dev_bf16(wd), True)
    h0, y0 = mx.mlp(dev_bf16(x), gu, dn, N, down_k_splits=1)
    bg, sg = _embed(rng, wg, 8, NAN_BF16)
    bu, su = _embed(rng, wu, 8, NAN_BF16)
    bdn, sd = _embed(rng, wd, 8, NAN_BF16)
    assert np.array_equal(host_bits(mx.repack_gate_up(dev_bf16(bg)[sg], dev_bf16(bu)[su])), host_bits(gu))
    assert np.array_equal(host_bits(mx.repack_b(dev_bf16(bdn)[sd], True)), host_bits(dn))
    bx, sx = _embed(rng, x, 8, NAN_BF16)
    bigH, H = _canary_out(M, N, 8, torch.bfloat16, 77.0)
    bigY, Y = _canary_out(M, K, 8, torch.bfloat16, 77.0)
    mx.mlp(dev_bf16(bx)[sx], gu, dn, N, h=H, y=Y, down_k_splits=1)
    assert np.array_equal(host_bits(H), host_bits(h0)) and np.array_equal(host_bits(Y), host_bits(y0))
    assert _canaries_intact(bigH, M, N, 77.0) and _canaries_intact(bigY, M, K, 77.0)


@pytest.mark.parametrize("shape", [(901, 80), (901, 96), (4096, 128), (33, 1000)])
def test_matvec_rows_among_nans(shape):
    """c[M] = A[M, K] . b[K] (MatmulVector / GemAvB, sizes of main.cpp:884-885): the rows of A taken out of a wider
    buffer of NaN, b and c inside longer ones."""
    M, K = shape
    rng = np.random.default_rng(M + K)
    A = wl.f32_to_bf16_bits(rng.standard_normal((M, K)).astype(np.float32))
    b = wl.f32_to_bf16_bits(rng.standard_normal(K).astype(np.float32))
    want = mx.matvec(dev_bf16(A), dev_bf16(b))
    for pad in (8, 3):
        bigA, sa = _embed(rng, A, pad, NAN_BF16)
        bigb = np.full(K + 16, NAN_BF16, dtype=np.uint16)
        bigb[8:8 + K] = b
        bigc = torch.full((M + 16,), 77.0, dtype=torch.float32, device="cuda")
        mx.matvec(dev_bf16(bigA)[sa], dev_bf16(bigb)[8:8 + K], out=bigc[8:8 + M])
        got = bigc[8:8 + M]
        assert torch.isfinite(got).all().item()
        assert torch.allclose(got, want, rtol=1e-5, atol=1e-5), pad    # (unaligned rows take the element-wise kernel: another order of sums)
        assert (bigc[:8] == 77.0).all().item() and (bigc[8 + M:] == 77.0).all().item()
