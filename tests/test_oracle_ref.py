"""The CPU oracle bit-for-bit against the compiled reference (oracle/_ref), on fresh random
inputs at the shapes the reference's own drivers use.  Skipped where the reference cannot
run (no checkout at build time, or no AMX on this host)."""
import ctypes as C

import numpy as np
import pytest

# main.cpp:715-735 (K tails 65..69, N=5, M=2, M/N tails), with the two large-N shapes cut down
FC_SHAPES = [(16, 65, 32), (16, 66, 32), (16, 67, 32), (16, 68, 32), (16, 69, 32), (32, 64, 5), (128, 96, 16),
             (2, 2560, 192), (2, 337, 271), (22, 2560, 96), (704, 320, 256), (705, 320, 257), (720, 320, 273),
             (735, 320, 271), (735, 321, 271), (735, 337, 271), (2, 320, 256)]


def p(a):
    return None if a is None else C.c_void_p(a.ctypes.data)


def bits(a):
    return np.ascontiguousarray(a).view(np.uint8)


@pytest.mark.parametrize("shape", FC_SHAPES)
def test_bf16_accumulators(po, ref, shape):
    M, K, N = shape
    rng = np.random.default_rng(hash(shape) % 2 ** 31)
    A = po.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    B = po.f32_to_bf16((rng.standard_normal((K, N)) * 0.02).astype(np.float32))
    want = np.empty((M, N), np.float32)
    ref.ref_gemm_bf16_acc(p(A), C.c_int64(A.strides[0]), p(B), C.c_int64(B.strides[0]), 0, p(want), C.c_int64(N),
                          M, K, N, 1)
    got = po.gemm_bf16(A, B)
    assert np.array_equal(bits(got), bits(want))
    # N-split over threads (main.cpp:442-479) must not change a single bit
    if N >= 64:
        want2 = np.empty((M, N), np.float32)
        ref.ref_gemm_bf16_acc(p(A), C.c_int64(A.strides[0]), p(B), C.c_int64(B.strides[0]), 0, p(want2),
                              C.c_int64(N), M, K, N, 2)
        assert np.array_equal(bits(want2), bits(want))
    # fp64 accumulation of the same product agrees to fp32 rounding noise
    f64 = po.gemm_bf16(A, B, f64=True)
    assert np.linalg.norm(got - f64) <= 1e-6 * np.linalg.norm(f64)


@pytest.mark.parametrize("shape", FC_SHAPES)
def test_int8_accumulators(po, ref, shape):
    M, K, N = shape
    if K < 64:
        pytest.skip("int8 tiles need K >= 64")
    rng = np.random.default_rng(hash(shape) % 2 ** 31 + 1)
    A = rng.integers(-127, 128, (M, K), dtype=np.int8)
    BT = rng.integers(-127, 128, (N, K), dtype=np.int8)
    want = np.empty((M, N), np.int32)
    ref.ref_gemm_i8_acc(p(A), C.c_int64(A.strides[0]), p(BT), C.c_int64(BT.strides[0]), 1, p(want), C.c_int64(N), M,
                        K, N, 1)
    assert np.array_equal(po.gemm_i8(A, BT, transB=True), want)


def test_headline_shape_slab(po, ref):
    """A slab of the headline FC (K=4096, Gaussian activations, N(0,0.02) weights, BIAS_GELU -> bf16)."""
    M, K, N = 64, 4096, 128
    rng = np.random.default_rng(7)
    A = po.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    B = po.f32_to_bf16((rng.standard_normal((K, N)) * 0.02).astype(np.float32))
    bias = (rng.standard_normal(N) * 0.1).astype(np.float32)
    want = np.zeros((M, N), np.uint16)
    rc = ref.ref_fc(2, p(A), C.c_int64(A.strides[0]), p(B), C.c_int64(B.strides[0]), 0, p(want),
                    C.c_int64(want.strides[0]), M, K, N, p(bias), C.c_float(1.0), C.c_float(1.0), None, 4)
    assert rc == 0
    got = po.pp(po.gemm_bf16(A, B), po.PP_BIAS | po.PP_GELU, po.BF16, bias=bias)
    assert np.array_equal(got, want)


def test_int8_requant_headline_scales(po, ref):
    """DEQUANT|BIAS|QUANT -> int8 at the scales of the int8 FC workload (a_scale*w_scale, q=20)."""
    M, K, N = 96, 4096, 64
    rng = np.random.default_rng(8)
    A = rng.integers(-127, 128, (M, K), dtype=np.int8)
    B = rng.integers(-127, 128, (K, N), dtype=np.int8)
    bias = (rng.standard_normal(N) * 0.1).astype(np.float32)
    acc = po.gemm_i8(A, B)
    steps = po.PP_DEQUANT | po.PP_BIAS | po.PP_QUANT
    for w_scale in (1e-3, 5e-3, 1e-2):
        deq = float(np.float32(0.02) * np.float32(w_scale))
        want = np.zeros((M, N), np.int8)
        rc = ref.ref_fc(11, p(A), C.c_int64(A.strides[0]), p(B), C.c_int64(B.strides[0]), 0, p(want),
                        C.c_int64(want.strides[0]), M, K, N, p(bias), C.c_float(deq), C.c_float(20.0), None, 1)
        assert rc == 0
        got = po.pp(acc, steps, po.I8, bias=bias, deq=deq, q=20.0)
        assert np.array_equal(got, want)
        assert 0.0 < np.mean(np.abs(got.astype(np.int32)) >= 127) < 1.0 or w_scale == 1e-3


@pytest.mark.parametrize("shape", [(1, 256, 64), (4, 4096, 96), (16, 337, 96), (40, 256, 64)])
def test_weight_compressed_path(po, ref, shape):
    M, K, N = shape
    rng = np.random.default_rng(9)
    A = po.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    W = po.f32_to_bf16((rng.standard_normal((K, N)) * 0.02).astype(np.float32))
    want = np.zeros((M, N), np.float32)
    dq = ref.ref_fc_w8(p(A), C.c_int64(A.strides[0]), p(W), C.c_int64(W.strides[0]), 0, p(want),
                       C.c_int64(want.strides[0]), M, K, N)
    Wq, dqo, _ = po.quantize_weights(W)
    assert np.float32(dq) == np.float32(dqo)
    _, acc = po.gemv_w8(A, Wq, np.ones(N, np.float32), want_acc=True)
    assert np.array_equal(bits(po.pp(acc, po.PP_DEQUANT, po.F32, deq=dqo)), bits(want))


@pytest.mark.parametrize("shape", [(901, 80), (901, 96), (64, 128), (37, 32), (33, 127)])
def test_matvec_orders(po, ref, shape):
    M, K = shape
    rng = np.random.default_rng(10)
    Ap = np.zeros((M + 1, K + 64), np.uint16)
    Ap[:M, :K] = po.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    A = Ap[:M, :K]
    b = np.zeros(K + 64, np.uint16)
    b[:K] = po.f32_to_bf16(rng.standard_normal(K).astype(np.float32))
    c = np.zeros(M + 16, np.float32)
    ref.ref_matvec_bf16(p(A), C.c_int64(A.strides[0]), p(b), p(c), M, K)
    assert np.array_equal(bits(po.matvec_bf16(A, b[:K].copy())), bits(c[:M]))
    c2 = np.zeros(M + 16, np.float32)
    ref.ref_gemavb(p(A), C.c_int64(A.strides[0]), p(b), p(c2), M, K)
    assert np.array_equal(bits(po.matvec_bf16(A, b[:K].copy(), order="avb")), bits(c2[:M]))


def test_rcp14_model_on_every_input(po, ref):
    """The software model of vrcp14ps equals the instruction on all 2^32 bit patterns."""
    ref.ref_rcp14_check_all.restype = C.c_longlong
    first = C.c_uint(0)
    bad = ref.ref_rcp14_check_all(C.cast(po.lib().orc_rcp14, C.c_void_p), C.byref(first))
    assert bad == 0, f"{bad} mismatches, first at input bits {first.value:#010x}"


def test_silu_is_the_stated_composition(po, ref):
    """silu(x) = x * vrcp14ps(1 + exp_poly(0 - x)) with the INSTRUCTION in the middle: the oracle's silu
    must give the same bits (tests/amx-mlp.cpp:450-456 is these four operations)."""
    rng = np.random.default_rng(11)
    g = np.concatenate([(rng.standard_normal(200000) * 1.28).astype(np.float32),
                        np.linspace(-100, 100, 20001).astype(np.float32), np.array([0.0, -0.0], np.float32)])
    one_plus = (np.float32(1.0) + po.exp_poly((np.float32(0.0) - g).astype(np.float32))).astype(np.float32)
    r14 = np.empty_like(one_plus)
    ref.ref_rcp14(p(one_plus), p(r14), one_plus.size)
    want = (g * r14).astype(np.float32)
    assert np.array_equal(bits(po.silu(g)), bits(want))


def test_scaled_truncating_quantiser_is_the_reference_expression(po, ref):
    """repackB_1xL<int8_t, L> (weight_compression/fc16m.cpp:80-81): "*dst++ = src0[n] * scale" evaluated by the
    reference's own bfloat16 class (compiled in the shim) on every bf16 input and a set of scales, against the
    oracle's trunc(bf16_rne(w * scale)).  Compared where the conversion to int8 is defined (|value| < 127.5)."""
    allb = np.arange(65536, dtype=np.uint16)
    for scale in (1.0, 2.0, 0.5, 3.0, 127.0 / 3.3, 0.37, -2.0, 1e-3, 1.0 / 3.0):
        want = np.empty(65536, np.int8)
        ref.ref_bf16_scale_to_s8(p(allb), C.c_float(scale), p(want), C.c_size_t(65536))
        got = po.quantize_scale_trunc(allb.reshape(256, 256), scale).reshape(-1)
        with np.errstate(invalid="ignore", over="ignore"):
            v = po.bf16_to_f32(allb).astype(np.float64) * np.float64(np.float32(scale))
        defined = np.isfinite(v) & (np.abs(v) < 127.5)
        assert defined.sum() > 30000
        assert np.array_equal(got[defined], want[defined]), scale


def test_unsigned_byte_forms_against_the_reference(po, ref):
    """Matmul<uint8_t,int8_t> (the one unsigned GEMM the reference can instantiate) and the three unsigned forms of
    MatmulVector (include/kernels_amx.hpp:839-850, 1057-1101) against the oracle's integer products."""
    rng = np.random.default_rng(6)
    for (M, K, N) in ((16, 64, 32), (37, 128, 75), (64, 256, 96), (5, 70, 40), (2, 2560, 64)):
        A = rng.integers(0, 256, (M, K)).astype(np.uint8)
        B = rng.integers(-128, 128, (K, N)).astype(np.int8)
        want = np.empty((M, N), np.int32)
        ref.ref_gemm_u8s8_acc(p(A), C.c_int64(A.strides[0]), p(B), C.c_int64(B.strides[0]), 0, p(want), C.c_int64(N), M, K, N, 1)
        assert np.array_equal(po.gemm_x8(A, B), want)
    for au, bu in ((1, 0), (0, 1), (1, 1)):
        for (M, K) in ((16, 64), (33, 128), (40, 256), (7, 100)):
            A = rng.integers(0, 256, (M, K)).astype(np.uint8) if au else rng.integers(-128, 128, (M, K)).astype(np.int8)
            b = rng.integers(0, 256, K).astype(np.uint8) if bu else rng.integers(-128, 128, K).astype(np.int8)
            want = np.empty(M, np.int32)
            ref.ref_matvec_x8(au, bu, p(A), C.c_int64(A.strides[0]), p(b), p(want), M, K)
            assert np.array_equal(po.matvec_x8(A, b), want), (au, bu, M, K)
