"""Checks of the oracle that rest on mathematics rather than on the reference: closed forms,
invariants and brute force on small inputs (for the parts no reference vector pins)."""
import math

import numpy as np


def test_exp_polynomial_and_silu(po):
    xs = np.linspace(-20, 20, 4001).astype(np.float32)
    e = np.array([po.lib().orc_exp_poly(float(v)) for v in xs], np.float64)
    assert np.max(np.abs(e / np.exp(xs.astype(np.float64)) - 1)) < 3e-7 * 4
    assert po.lib().orc_exp_poly(-200.0) == 0.0
    assert po.lib().orc_exp_poly(200.0) > 1e38
    s = po.silu(xs).astype(np.float64)
    exact = xs.astype(np.float64) / (1 + np.exp(-xs.astype(np.float64)))
    # the sigmoid comes from a 14-bit reciprocal: relative error below 2^-14 (plus the polynomial's)
    assert np.all(np.abs(s - exact) <= np.abs(exact) * (2.0 ** -14 + 2e-6) + 1e-30)
    assert po.lib().orc_silu(0.0) == 0.0
    assert abs(po.lib().orc_silu(30.0) - 30.0) < 30 * 2.0 ** -14
    assert abs(po.lib().orc_silu(-30.0)) < 1e-10


def test_rcp14_properties(po):
    """What the definition of vrcp14ps fixes without the instruction at hand: relative error below 2^-14,
    powers of two exact, monotone, sign symmetric, specials."""
    rng = np.random.default_rng(5)
    x = np.concatenate([np.exp(rng.uniform(-80, 80, 200000)), np.linspace(1, 2, 100001)]).astype(np.float32)
    r = po.rcp14(x).astype(np.float64)
    assert np.max(np.abs(r * x.astype(np.float64) - 1)) < 2.0 ** -14
    p2 = (2.0 ** np.arange(-126, 127)).astype(np.float32)
    assert np.array_equal(po.rcp14(p2), (1.0 / p2.astype(np.float64)).astype(np.float32))
    xs = np.sort(x)
    assert np.all(np.diff(po.rcp14(xs)) <= 0)
    assert np.array_equal(po.rcp14(-x).view(np.uint32), po.rcp14(x).view(np.uint32) | 0x80000000)
    sp = np.array([0.0, -0.0, np.inf, -np.inf], np.float32)
    assert np.array_equal(po.rcp14(sp).view(np.uint32), np.array([0x7F800000, 0xFF800000, 0, 0x80000000], np.uint32))
    assert np.isnan(po.rcp14(np.array([np.nan], np.float32))[0])


def test_mlp_against_fp64(po):
    rng = np.random.default_rng(0)
    M, K, N = 8, 256, 512
    x = po.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    wg = po.f32_to_bf16((rng.standard_normal((N, K)) * 0.05).astype(np.float32))
    wu = po.f32_to_bf16((rng.standard_normal((N, K)) * 0.05).astype(np.float32))
    wd = po.f32_to_bf16((rng.standard_normal((K, N)) * 0.05).astype(np.float32))
    h, y = po.mlp(x, wg, wu, wd, split_k=True)
    xf, g, u, d = (po.bf16_to_f32(a).astype(np.float64) for a in (x, wg, wu, wd))
    gate, up = xf @ g.T, xf @ u.T
    h64 = gate / (1 + np.exp(-gate)) * up
    hf = po.bf16_to_f32(h).astype(np.float64)
    assert np.linalg.norm(hf - h64) / np.linalg.norm(h64) < 3e-3
    y64 = hf @ d.T  # from the oracle's own h: isolates the down stage
    yf = po.bf16_to_f32(y).astype(np.float64)
    assert np.linalg.norm(yf - y64) / np.linalg.norm(y64) < 3e-3
    # the stage-wise entry point gives the same bits as the chained one
    assert np.array_equal(po.mlp_down(h, wd, split_k=True), y)
    # split-K sums two fp32 partials before rounding: differs from unsplit by rounding noise only
    y_ns = po.bf16_to_f32(po.mlp_down(h, wd, split_k=False)).astype(np.float64)
    assert np.linalg.norm(y_ns - yf) / np.linalg.norm(yf) < 3e-3


def test_gemm_linearity_and_transposes(po):
    """Exact-arithmetic inputs (+-0.5 like the reference's fill_rnd, include/tensor2D.hpp:145-172):
    every order of summation gives the same bits, so the product must equal an integer GEMM."""
    rng = np.random.default_rng(1)
    M, K, N = 33, 101, 47
    A = rng.integers(0, 2, (M, K)).astype(np.float32) - 0.5
    B = rng.integers(0, 2, (K, N)).astype(np.float32) - 0.5
    got = po.gemm_bf16(po.f32_to_bf16(A), po.f32_to_bf16(B))
    assert np.array_equal(got, (A.astype(np.float64) @ B.astype(np.float64)).astype(np.float32))
    gotT = po.gemm_bf16(po.f32_to_bf16(A), po.f32_to_bf16(np.ascontiguousarray(B.T)), transB=True)
    assert np.array_equal(got, gotT)


def test_mfma_layout_is_a_zero_padded_bijection(po):
    for es, dt in ((2, np.uint16), (1, np.int8)):
        for K, N in ((64, 32), (70, 45), (256, 96), (129, 33)):
            B = (np.arange(K * N, dtype=np.int64).reshape(K, N) % 119 + 1).astype(dt)
            packed = po.repack(B, layout="mfma")
            kalign = 128 // es
            Kp, Np = -(-K // kalign) * kalign, -(-N // 32) * 32
            assert packed.size == Kp * Np * es
            assert np.count_nonzero(packed.view(dt)) == K * N
            packedT = po.repack(np.ascontiguousarray(B.T), transpose=True, layout="mfma")
            assert np.array_equal(packed, packedT)
            # element (k, n) sits where the documented index says
            KS, half = 32 // es, 16 // es
            v = packed.view(dt)
            for k, n in ((0, 0), (K - 1, N - 1), (K // 2, N // 3), (half, 1), (KS, 31 % N)):
                lane = (n % 32) + 32 * ((k % KS) // half)
                off = ((n // 32) * (Kp // KS) + k // KS) * (1024 // es) + lane * (16 // es) + k % half
                assert v[off] == B[k, n]


def test_quantize_weights_properties(po):
    rng = np.random.default_rng(2)
    W = po.f32_to_bf16((rng.standard_normal((64, 48)) * 0.02).astype(np.float32))
    Wq, dq, q = po.quantize_weights(W)
    Wf = po.bf16_to_f32(W)
    amax = np.abs(Wf).max()
    assert np.float32(q) == np.float32(127) / np.float32(amax)
    assert np.float32(dq) == np.float32(amax) / np.float32(127)
    assert np.abs(Wq.astype(np.int32)).max() == 127
    assert np.max(np.abs(Wq * np.float32(dq) - Wf)) <= 0.5 * dq * 1.001


def test_int4_quantiser_and_layout_properties(po):
    # the int4 compression has no counterpart in the reference (it only times a byte-copying stand-in), so its
    # definition is checked by what the mathematics fixes
    rng = np.random.default_rng(12)
    for K, N in ((64, 32), (300, 45), (256, 96), (70, 33)):
        Wf = (rng.standard_normal((K, N)) * 0.03).astype(np.float32)
        Wf[:, 1] = 0.0                      # a column of zeros
        Wf[3, 2] = -1.0                     # a dominant negative maximum
        W = po.f32_to_bf16(Wf)
        Wf = po.bf16_to_f32(W)
        q, deq = po.quantize_int4(W)
        amax = np.abs(Wf).max(axis=0)
        assert np.array_equal(deq, (amax / np.float32(7)).astype(np.float32))
        assert q.min() >= -7 and q.max() <= 7
        assert np.all(q[:, 1] == 0) and deq[1] == 0
        assert q[3, 2] == -7
        # the maximum of every non-zero column maps to +-7, and every value is within half a step
        nz = amax > 0
        assert np.all(np.abs(q).max(axis=0)[nz] == 7)
        assert np.all(np.abs(q * deq[None, :] - Wf) <= 0.5 * deq[None, :] * 1.001 + 1e-12)
        # brute force of the rounding rule in fp32
        qs = np.where(nz, np.float32(7) / np.where(nz, amax, 1).astype(np.float32), np.float32(0)).astype(np.float32)
        want = np.clip(np.rint((Wf * qs[None, :]).astype(np.float32)), -7, 7).astype(np.int8)
        assert np.array_equal(q, want)
        # the transposed source gives the same result
        qT, deqT = po.quantize_int4(np.ascontiguousarray(W.T), transpose=True)
        assert np.array_equal(qT, q) and np.array_equal(deqT, deq)
        # layout: zero-padded bijection, nibble (k, n) where the documented index says
        packed = po.pack_int4(q)
        nfrag = -(-K // 256) * 4
        assert packed.size == -(-N // 32) * nfrag * 1024
        lo, hi = packed & 0xF, packed >> 4
        nib = np.stack([lo, hi], axis=1).reshape(-1)          # nibble e of a byte stream: byte e//2, low first
        assert np.count_nonzero(nib) == np.count_nonzero(q)
        for k, n in ((0, 0), (K - 1, N - 1), (K // 2, N // 3), (37 % K, 5), (63, 31 % N)):
            f, g, i, e = k // 64, (k % 64) // 32, (k % 32) // 8, k % 8
            idx = (((n // 32) * nfrag + f) * 1024 + (g * 32 + n % 32) * 16 + i * 4) * 2 + e
            assert nib[idx] == (int(q[k, n]) & 0xF)


def test_int4_known_answers(po):
    # by hand: a column whose largest magnitude is 7 has quantisation scale 1, so q = rne(w) with ties to even,
    # and deq = 1; the first dword of the packed column spells the nibbles out
    col = np.array([7.0, -3.5, 2.5, 0.5, -0.5, 6.5, -7.0, 1.0] + [0.0] * 56, np.float32)
    W = np.zeros((64, 32), np.float32)
    W[:, 0] = col
    W[:, 5] = col * 0.25          # the same column at another scale: same q, deq = 1/4
    q, deq = po.quantize_int4(po.f32_to_bf16(W))
    assert q[:8, 0].tolist() == [7, -4, 2, 0, 0, 6, -7, 1] and deq[0] == 1.0
    assert q[:8, 5].tolist() == [7, -4, 2, 0, 0, 6, -7, 1] and deq[5] == 0.25
    packed = po.pack_int4(q).view(np.uint32)
    assert packed.size == 4 * 256                       # 4 fragments (K padded to 256) of 256 dwords
    assert packed[0] == 0x196002C7                      # lane 0 (column 0, k 0..7)
    assert packed[5 * 4] == 0x196002C7                  # lane 5 (column 5)
    assert np.count_nonzero(packed) == 2


def test_gemv_w8_is_exact_conversion_then_gemm(po):
    rng = np.random.default_rng(3)
    M, K, N = 3, 128, 40
    x = po.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    Wq = np.clip(np.rint(rng.standard_normal((K, N)) * 40), -127, 127).astype(np.int8)
    scale = rng.uniform(1e-3, 5e-3, N).astype(np.float32)
    y, acc = po.gemv_w8(x, Wq, scale, want_acc=True)
    yT = po.gemv_w8(x, np.ascontiguousarray(Wq.T), scale, transW=True)
    assert np.array_equal(y, yT)
    ref64 = po.bf16_to_f32(x).astype(np.float64) @ Wq.astype(np.float64)
    assert np.linalg.norm(acc - ref64) / np.linalg.norm(ref64) < 1e-6
    assert np.array_equal(y, po.f32_to_bf16(acc * scale[None, :]))


def test_splitter_partitions(po):
    for n, team in ((344, 8), (5, 8), (128, 3), (1, 1), (0, 4)):
        parts = [po.splitter(n, team, t) for t in range(team)]
        assert parts[0][0] == 0 and parts[-1][1] == n
        for a, b in zip(parts, parts[1:]):
            assert a[1] == b[0]
        sizes = [b - a for a, b in parts]
        assert max(sizes) - min(sizes) <= 1


def test_gelu_deep_negative_tail_is_ill_conditioned(po):
    """Why two implementations of the FC + GELU cannot agree to one bf16 ulp everywhere unless their
    fp32 accumulators are bit-identical: below about -3.5 the reference polynomial's result moves by
    more than one bf16 ulp when its input moves by ONE fp32 ulp."""
    def frac_beyond_one_bf16_ulp(lo, hi):
        x = np.linspace(lo, hi, 200001).astype(np.float32)
        x1 = np.nextafter(x, np.float32(0))
        y, y1 = po.gelu(x).astype(np.float64), po.gelu(x1).astype(np.float64)
        ulp = np.exp2(np.floor(np.log2(np.maximum(np.abs(y), 2.0 ** -126))) - 7)
        return np.mean(np.abs(y - y1) > ulp)
    assert frac_beyond_one_bf16_ulp(-4.9, -4.3) > 0.25
    assert frac_beyond_one_bf16_ulp(-3.0, 5.0) == 0.0


def test_int4_non_finite_weights_are_defined(po):
    """NaNs do not take part in a column's maximum; a NaN weight and every infinite weight quantise to 0; a column
    holding an infinity has an infinite dequant scale (so its finite weights quantise to 0 as well)."""
    W = np.full((8, 4), 0.5, np.float32)
    W[:, 0] = [1.0, -2.0, np.nan, 0.5, 0.25, -1.0, 2.0, 0.0]         # a NaN among finite weights: max 2
    W[:, 1] = [1.0, np.inf, -3.0, 0.5, 0.25, -1.0, 2.0, 0.0]          # an infinity
    W[:, 2] = [np.nan] * 8                                            # nothing but NaNs: max 0
    q, deq = po.quantize_int4(po.f32_to_bf16(W))
    assert list(q[:, 0]) == [4, -7, 0, 2, 1, -4, 7, 0] and deq[0] == np.float32(2.0) / np.float32(7.0)
    assert not q[:, 1].any() and np.isinf(deq[1])
    assert not q[:, 2].any() and deq[2] == 0.0
    assert list(q[:, 3]) == [7] * 8


def test_ffn_up_gelu_against_a_better_rounded_sum_shows_the_same_shortfall(po):
    """The 1-bf16-ulp bar on the FC + BIAS + GELU configuration (K = 4096, A ~ N(0,1), B ~ N(0,0.02), bias ~ N(0,0.1)),
    measured between the reference's own arithmetic (AMX summation order, fp32) and the same product accumulated
    in fp64 and rounded once: over ALL elements even this pair stays below 99.9 %, above a pre-activation of -3.5
    it is met with room to spare.  So 99.9 % over all elements is not reachable by any implementation whose fp32
    accumulators are not bit-identical to AMX's; the GPU tests therefore apply the bar where GELU is well
    conditioned and check the fused epilogue bit for bit on the GPU's own accumulators."""
    from mm_amx_amd import workloads as wl
    w = wl.ffn_up_bias_gelu(M=192)  # 192 x 11008 = 2.1 M elements of the benchmark's own distribution
    acc = po.gemm_bf16(w["A"], w["B"])
    acc64 = po.gemm_bf16(w["A"], w["B"], f64=True)
    steps = po.PP_BIAS | po.PP_GELU
    a = po.bf16_to_f32(po.pp(acc, steps, po.BF16, bias=w["bias"])).astype(np.float64)
    b = po.bf16_to_f32(po.pp(acc64, steps, po.BF16, bias=w["bias"])).astype(np.float64)
    ulp = np.exp2(np.floor(np.log2(np.maximum(np.abs(a), 2.0 ** -126))) - 7)
    within = np.abs(a - b) <= ulp
    pre = acc + w["bias"][None, :]
    good = pre > -3.5
    assert a.size >= 2_000_000
    assert within.mean() < 0.999, within.mean()            # measured 0.99886
    assert within.mean() > 0.998
    assert within[good].mean() >= 0.9999, within[good].mean()  # measured 0.999994
    # the accumulators themselves agree far better than the bar asks: the shortfall is GELU's conditioning, not the sums
    ulp_acc = np.exp2(np.floor(np.log2(np.maximum(np.abs(acc.astype(np.float64)), 2.0 ** -126))) - 7)
    assert (np.abs(acc.astype(np.float64) - acc64) <= ulp_acc).mean() > 0.9999


def test_scaled_truncating_quantiser_by_hand_and_by_brute_force(po):
    """q = trunc(bf16_rne(w * scale)) (repackB_1xL<int8_t>, weight_compression/fc16m.cpp:80-81): answers worked out by
    hand (the bf16 rounding of the product comes BEFORE the truncation and can carry a value across an integer),
    an independent numpy restatement on random inputs, and the function's tile order by its index formula."""
    def q1(x, scale):
        return int(po.quantize_scale_trunc(po.f32_to_bf16(np.array([[x]], np.float32)), scale)[0, 0])
    assert q1(1.296875, 2.0) == 2 and q1(-1.296875, 2.0) == -2          # 2.59375 -> toward zero
    assert q1(0.99609375, 1.0) == 0 and q1(-0.99609375, 1.0) == 0       # just below one
    assert q1(1.0, 1.0) == 1 and q1(63.5, 2.0) == 127 and q1(-64.0, 2.0) == -128
    # 0.33203125 * 3 = 0.99609375 exactly (a bf16): 0; 1.9921875 * (1/3 in fp32) = 0.66406256 -> bf16 0.6640625 -> 0
    assert q1(0.33203125, 3.0) == 0
    # the product 85 * 1.0117188 = 85.996098 rounds to bf16 86.0 BEFORE the truncation: 86, where trunc(product) is 85
    assert q1(85.0, 1.01171875) == 86
    assert q1(100.0, 2.0) == 127 and q1(-100.0, 2.0) == -128 and q1(float("nan"), 2.0) == 0  # defined here: saturate, NaN -> 0
    rng = np.random.default_rng(3)
    W = po.f32_to_bf16(rng.uniform(-60, 60, (64, 48)).astype(np.float32))
    for scale in (2.0, 0.7, 1.9):
        prod = po.bf16_to_f32(W) * np.float32(scale)                     # fp32 product, correctly rounded
        rb = po.bf16_to_f32(po.f32_to_bf16(prod))                        # ... to bf16, nearest even
        want = np.clip(np.trunc(rb), -128, 127).astype(np.int8)
        assert np.array_equal(po.quantize_scale_trunc(W, scale), want)
    # tile order (fc16m.cpp:61-99): with scale 1 and small integer entries the bytes are the entries themselves
    K, N, L = 64, 64, 2
    k_idx, n_idx = np.meshgrid(np.arange(K), np.arange(N), indexing="ij")
    for plane, vals in (("k", k_idx), ("n", n_idx)):
        out = po.repack_1xL_s8(po.f32_to_bf16(vals.astype(np.float32)), L, 1.0)
        i = 0
        for n0 in range(0, N, 16 * L):
            for k0 in range(0, K, 32):
                for l in range(L):
                    tile = out[i:i + 512].reshape(16, 16, 2)             # [k pair][column][k parity]
                    i += 512
                    kk = k0 + 2 * np.arange(16)[:, None, None] + np.arange(2)[None, None, :]
                    nn = n0 + 16 * l + np.arange(16)[None, :, None]
                    want = np.broadcast_to(kk if plane == "k" else nn, (16, 16, 2))
                    assert np.array_equal(tile, want.astype(np.int8))


def test_streamed_gemv_is_the_converted_gemv_bit_for_bit(po):
    """orc_gemv_w8_stream (packed int8 weights read once, converted in registers: the form of matmul16m_Wint8B,
    weight_compression/fc16m.cpp:451-502) against orc_gemv_w8 (weights converted to bf16 up front, then the pinned AMX-order
    GEMM): same bits for every M it takes, any thread count; and its packing is the order of repackB_1xL<int8_t,2>."""
    from mm_amx_amd import workloads as wl
    for M, K, N in ((1, 256, 96), (4, 512, 64), (7, 96, 160), (16, 1024, 32)):
        w = wl.decode_gemv_w8(M=M, K=K, N=N, seed=M)
        want = po.gemv_w8(w["x"], w["W"], w["scale"])
        packed = po.pack_1x2_s8(w["W"])
        for nt in (1, 3):
            assert np.array_equal(po.gemv_w8_stream(w["x"], packed, w["scale"], N, nthreads=nt), want), (M, K, N, nt)
    rng = np.random.default_rng(0)
    Wi = rng.integers(-100, 100, (64, 96)).astype(np.int8)
    assert np.array_equal(po.pack_1x2_s8(Wi), po.repack_1xL_s8(po.f32_to_bf16(Wi.astype(np.float32)), 2, 1.0))


def test_int8_gemm_fast_path_equals_the_generic_one_and_int64(po):
    """orc_gemm_i8 takes a vpmaddwd path where the host has AVX-512BW (even K): the same int32 sums as the generic
    loop and as an int64 product, including the extremes -128 x -128."""
    rng = np.random.default_rng(1)
    for M, K, N, t in ((37, 130, 75, False), (5, 64, 33, True), (64, 256, 48, False), (3, 65, 20, False)):
        A = rng.integers(-128, 128, (M, K)).astype(np.int8)
        B = rng.integers(-128, 128, ((N, K) if t else (K, N))).astype(np.int8)
        A[0, :] = -128
        if t:
            B[0, :] = -128
        else:
            B[:, 0] = -128
        want = A.astype(np.int64) @ (B.T if t else B).astype(np.int64)
        assert np.array_equal(po.gemm_i8(A, B, transB=t), want)
        assert np.array_equal(po.gemm_i8_generic(A, B, transB=t), want)


def test_unsigned_byte_products_against_int64(po):
    """orc_gemm_x8 / orc_matvec_x8 in all four signedness combinations against an int64 product, extremes included,
    and the identity the GPU path rests on: u = (u ^ 0x80 as a signed byte) + 128."""
    rng = np.random.default_rng(8)
    def draw(unsigned, shape):
        a = rng.integers(0, 256, shape).astype(np.uint8) if unsigned else rng.integers(-128, 128, shape).astype(np.int8)
        a.flat[0] = 255 if unsigned else -128
        return a
    for au in (False, True):
        for bu in (False, True):
            for (M, K, N, t) in ((9, 130, 21, False), (3, 64, 40, True)):
                A, B = draw(au, (M, K)), draw(bu, (N, K) if t else (K, N))
                want = (A.astype(np.int64) @ (B.T if t else B).astype(np.int64)).astype(np.int32)
                assert np.array_equal(po.gemm_x8(A, B, transB=t), want)
                b = np.ascontiguousarray((B[0] if t else B[:, 0]))
                assert np.array_equal(po.matvec_x8(A, b), (A.astype(np.int64) @ b.astype(np.int64)).astype(np.int32))
    u = np.arange(256, dtype=np.uint8)
    assert np.array_equal((u ^ 0x80).view(np.int8).astype(np.int32) + 128, u.astype(np.int32))
