"""The CPU oracle against vectors produced by the real reference kernels (tests/golden/).

These run on any x86-64 host: they need neither the reference checkout nor AMX.
"""
import math
import os

import numpy as np
import pytest

G = np.load(os.path.join(os.path.dirname(__file__), "golden", "fc_golden.npz"))


def bits(a):
    return np.ascontiguousarray(a).view(np.uint8)


@pytest.mark.parametrize("i", range(5))
def test_bf16_fc_accumulators_and_bias_gelu(po, i):
    A, B, bias = G[f"bf16_{i}_A"], G[f"bf16_{i}_B"], G[f"bf16_{i}_bias"]
    acc = po.gemm_bf16(A, B)
    assert np.array_equal(bits(acc), bits(G[f"bf16_{i}_acc"]))
    accT = po.gemm_bf16(A, np.ascontiguousarray(B.T), transB=True)
    assert np.array_equal(bits(accT), bits(G[f"bf16_{i}_acc"]))
    out = po.pp(acc, po.PP_BIAS | po.PP_GELU, po.BF16, bias=bias)
    assert np.array_equal(out, G[f"bf16_{i}_gelu_bf16"])


@pytest.mark.parametrize("i", range(3))
def test_int8_fc_accumulators_and_requant(po, i):
    A, B, bias, qoc = G[f"i8_{i}_A"], G[f"i8_{i}_B"], G[f"i8_{i}_bias"], G[f"i8_{i}_qoc"]
    deq = float(G[f"i8_{i}_deq"])
    acc = po.gemm_i8(A, B)
    assert np.array_equal(acc, G[f"i8_{i}_acc"])
    assert np.array_equal(acc, (A.astype(np.int64) @ B.astype(np.int64)).astype(np.int32))
    dbq = po.PP_DEQUANT | po.PP_BIAS | po.PP_QUANT
    assert np.array_equal(po.pp(acc, dbq, po.I8, bias=bias, deq=deq, q=20.0), G[f"i8_{i}_dbq"])
    assert np.array_equal(po.pp(acc, dbq, po.I8, bias=bias, deq=deq, q_per_oc=qoc), G[f"i8_{i}_dbq_oc"])
    assert np.array_equal(po.pp(acc, dbq | po.PP_GELU, po.I8, bias=bias, deq=deq, q=20.0), G[f"i8_{i}_dbgq"])


def test_per_channel_dequant_reduces_to_per_tensor(po):
    """The per-output-channel dequant has no reference counterpart; it must equal the pinned
    per-tensor path column by column."""
    A, B, bias = G["i8_1_A"], G["i8_1_B"], G["i8_1_bias"]
    acc = po.gemm_i8(A, B)
    N = acc.shape[1]
    steps = po.PP_DEQUANT | po.PP_BIAS | po.PP_QUANT
    deq = float(G["i8_1_deq"])
    same = po.pp(acc, steps, po.I8, bias=bias, deq_per_oc=np.full(N, deq, np.float32), q=20.0)
    assert np.array_equal(same, G["i8_1_dbq"])
    scales = np.random.default_rng(3).uniform(1e-5, 2e-4, N).astype(np.float32)
    per_oc = po.pp(acc, steps, po.I8, bias=bias, deq_per_oc=scales, q=20.0)
    for n in range(0, N, 7):
        col = po.pp(acc, steps, po.I8, bias=bias, deq=float(scales[n]), q=20.0)
        assert np.array_equal(per_oc[:, n], col[:, n])


def test_gelu_polynomial(po):
    x, y = G["gelu_x"], G["gelu_y"]
    got = po.gelu(x)
    assert np.array_equal(bits(got), bits(y))
    # closed forms of the zones (include/kernels_amx.hpp:269-287)
    assert po.gelu(np.float32([-5.5, -100.0])).tolist() == [0.0, 0.0]
    assert po.gelu(np.float32([5.5, 100.0])).tolist() == [5.5, 100.0]
    tiny = np.float32([2.0 ** -24, -(2.0 ** -25), 1e-30])
    assert np.array_equal(po.gelu(tiny), tiny * np.float32(0.5))
    assert math.isnan(float(po.gelu(np.float32([np.nan]))[0]))
    # it is the erf GELU to 3.4e-4, and NOT the tanh approximation
    xs = np.linspace(-6, 6, 3073).astype(np.float32)
    erf_form = np.array([v * 0.5 * (1 + math.erf(v / math.sqrt(2))) for v in xs.astype(np.float64)])
    assert np.abs(po.gelu(xs) - erf_form).max() < 3.5e-4


@pytest.mark.parametrize("es", [2, 1])
@pytest.mark.parametrize("tr", [0, 1])
def test_repack_amx_tile_order(po, es, tr):
    B, want = G[f"repack_{es}_{tr}_B"], G[f"repack_{es}_{tr}_out"]
    got = po.repack(B, transpose=bool(tr), layout="amx")
    valid = po.repack(np.full_like(B, 0x0101 if es == 2 else 1), transpose=bool(tr), layout="amx") != 0
    assert valid.sum() == B.size * es
    assert np.array_equal(got[valid], want[valid])
    assert not got[~valid].any()


def test_weight_compressed_fc(po):
    A, W = G["w8_A"], G["w8_W"]
    Wq, dq, q = po.quantize_weights(W)
    assert np.float32(dq) == G["w8_dq"]
    y, acc = po.gemv_w8(A, Wq, np.ones(W.shape[1], np.float32), want_acc=True)
    out = po.pp(acc, po.PP_DEQUANT, po.F32, deq=dq)
    assert np.array_equal(bits(out), bits(G["w8_C"]))


@pytest.mark.parametrize("i", range(3))
def test_matvec(po, i):
    A, b = G[f"mv_{i}_A"], G[f"mv_{i}_b"]
    assert np.array_equal(bits(po.matvec_bf16(A, b)), bits(G[f"mv_{i}_amx"]))
    assert np.array_equal(bits(po.matvec_bf16(A, b, order="avb")), bits(G[f"mv_{i}_avb"]))


def test_bf16_rounding(po):
    f = np.float32([1.0, 1.00390625, 1.005859375, 1.01171875, -3.14159, 65504.0, 1e-40, 0.0])
    got = po.f32_to_bf16(f)
    # ties go to even: 1.00390625 = 0x3F808000 -> 0x3F80; 1.01171875 = 0x3F818000 -> 0x3F82
    assert got[0] == 0x3F80 and got[1] == 0x3F80 and got[3] == 0x3F82
    assert got[2] == 0x3F81
    assert got[6] == 0 and got[7] == 0
    back = po.bf16_to_f32(got)
    ok = f != np.float32(1e-40)
    assert np.all(np.abs(back[ok] - f[ok]) <= np.abs(f[ok]) * 2.0 ** -8)


def test_rcp14_model(po):
    """vrcp14ps: the software model against recorded outputs of the instruction (random bit patterns,
    [1, 2), the 1 + e^t values SiLU feeds it, denormals, specials).  NaN results compare as NaN."""
    x, want = G["rcp14_x"], G["rcp14_y"]
    got = po.rcp14(x.view(np.float32)).view(np.uint32)
    nan = (want & 0x7FFFFFFF) > 0x7F800000
    assert ((got & 0x7FFFFFFF) > 0x7F800000)[nan].all()
    assert np.array_equal(got[~nan], want[~nan])
