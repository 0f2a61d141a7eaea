"""Writes tests/golden/fc_golden.npz: inputs and the outputs of the REAL reference kernels.

Run in a container that has the reference checkout and an AMX-capable CPU:
    make -C oracle ref && python tests/golden/make_golden.py
The fixture holds data only (inputs, expected outputs); the tests that read it need neither
the reference nor AMX.
"""
import ctypes as C
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import pyoracle as po  # noqa: E402


def p(a):
    return None if a is None else C.c_void_p(a.ctypes.data)


def main():
    r = po.ref()
    assert r is not None, "compiled reference unavailable"
    rng = np.random.default_rng(20240607)
    out = {}

    def bf16(shape, std):
        return po.f32_to_bf16((rng.standard_normal(shape) * std).astype(np.float32))

    def ref_fc(mode, A, B, outdt, bias=None, deq=1.0, q=1.0, qoc=None, transB=False):
        M, K = A.shape
        N = B.shape[0] if transB else B.shape[1]
        Cm = np.zeros((M, N), outdt)
        rc = r.ref_fc(mode, p(A), C.c_int64(A.strides[0]), p(B), C.c_int64(B.strides[0]), int(transB), p(Cm),
                      C.c_int64(Cm.strides[0]), M, K, N, p(bias), C.c_float(deq), C.c_float(q), p(qoc), 1)
        assert rc == 0
        return Cm

    # bf16 FC: raw fp32 accumulators and BIAS_GELU -> bf16
    for i, (M, K, N) in enumerate([(16, 65, 32), (32, 64, 5), (2, 337, 271), (88, 77, 66), (8, 4096, 32)]):
        A, B = bf16((M, K), 1.0), bf16((K, N), 0.05)
        bias = (rng.standard_normal(N) * 0.1).astype(np.float32)
        out[f"bf16_{i}_A"], out[f"bf16_{i}_B"], out[f"bf16_{i}_bias"] = A, B, bias
        out[f"bf16_{i}_acc"] = ref_fc(0, A, B, np.float32)
        out[f"bf16_{i}_gelu_bf16"] = ref_fc(2, A, B, np.uint16, bias=bias)
        BT = np.ascontiguousarray(B.T)
        assert np.array_equal(ref_fc(0, A, BT, np.float32, transB=True).view(np.uint32),
                              out[f"bf16_{i}_acc"].view(np.uint32))

    # int8 FC: raw int32 accumulators, DEQUANT|BIAS|QUANT and DEQUANT|BIAS|GELU|QUANT -> int8
    for i, (M, K, N) in enumerate([(16, 69, 32), (88, 77, 66), (4, 1024, 40)]):
        A = rng.integers(-127, 128, (M, K), dtype=np.int8)
        B = rng.integers(-127, 128, (K, N), dtype=np.int8)
        bias = (rng.standard_normal(N) * 0.1).astype(np.float32)
        qoc = rng.uniform(5, 40, N).astype(np.float32)
        acc = np.empty((M, N), np.int32)
        r.ref_gemm_i8_acc(p(A), C.c_int64(A.strides[0]), p(B), C.c_int64(B.strides[0]), 0, p(acc), C.c_int64(N), M,
                          K, N, 1)
        deq = float(np.float32(0.02) * np.float32(0.005))
        out[f"i8_{i}_A"], out[f"i8_{i}_B"], out[f"i8_{i}_bias"], out[f"i8_{i}_qoc"] = A, B, bias, qoc
        out[f"i8_{i}_deq"] = np.float32(deq)
        out[f"i8_{i}_acc"] = acc
        out[f"i8_{i}_dbq"] = ref_fc(11, A, B, np.int8, bias=bias, deq=deq, q=20.0)
        out[f"i8_{i}_dbq_oc"] = ref_fc(11, A, B, np.int8, bias=bias, deq=deq, qoc=qoc)
        out[f"i8_{i}_dbgq"] = ref_fc(12, A, B, np.int8, bias=bias, deq=deq, q=20.0)

    # GELU polynomial
    x = np.concatenate([np.linspace(-6.5, 6.5, 3073, dtype=np.float32),
                        (rng.standard_normal(1000) * 2).astype(np.float32),
                        np.array([0.0, -0.0, 5.0, -5.0, 2.0 ** -24, -(2.0 ** -24), 5.0000005, -5.0000005, 1e-30],
                                 np.float32)])
    y = np.empty_like(x)
    r.ref_gelu(p(x), p(y), x.size)
    out["gelu_x"], out["gelu_y"] = x, y

    # vrcp14ps: the instruction itself on sampled and special inputs (bit patterns in, bit patterns out)
    xb = np.concatenate([
        rng.integers(0, 1 << 32, 20000, dtype=np.uint64).astype(np.uint32),                 # anything
        (np.uint32(0x3F800000) | rng.integers(0, 1 << 23, 10000).astype(np.uint32)),         # [1, 2)
        (np.float32(1.0) + np.exp(rng.standard_normal(10000) * 3).astype(np.float32)).view(np.uint32),  # 1 + e^t
        np.arange(0, 1 << 23, 16411, dtype=np.uint32),                                        # denormals
        np.array([0x00000000, 0x80000000, 0x00000001, 0x001FFFFF, 0x00200000, 0x00200001, 0x00400000, 0x007FFFFF,
                  0x00800000, 0x3F800000, 0x3F800001, 0x3FFFFFFF, 0x40000000, 0x7E800000, 0x7E800001, 0x7F000000,
                  0x7F000001, 0x7F7FFFFF, 0x7F800000, 0xFF800000, 0x7FC00000, 0x7F800001, 0xFFFFFFFF, 0xBFC00000],
                 np.uint32)])
    yb = np.empty_like(xb)
    r.ref_rcp14(p(xb), p(yb), xb.size)
    out["rcp14_x"], out["rcp14_y"] = xb, yb

    # repackB_1x2 (AMX tile order), K and N tails, both element sizes and both transposes
    for es, dt in ((2, np.uint16), (1, np.int8)):
        K, N = 69, 40
        B = rng.integers(1, 120, (K, N)).astype(dt)
        for tr in (0, 1):
            Bin = np.ascontiguousarray(B.T) if tr else B
            nbytes = po.lib().orc_repack_amx_bytes(es, K, N)
            buf = np.zeros(nbytes + 4096, np.uint8)
            r.ref_repack(es, p(Bin), C.c_int64(Bin.strides[0]), K, N, tr, p(buf))
            out[f"repack_{es}_{tr}_B"], out[f"repack_{es}_{tr}_out"] = Bin, buf[:nbytes].copy()

    # weight-compressed FC (Matmul<bf16,int8,float>), per-tensor scale chosen by the op
    A, W = bf16((4, 512), 1.0), bf16((512, 64), 0.02)
    Cm = np.zeros((4, 64), np.float32)
    dq = r.ref_fc_w8(p(A), C.c_int64(A.strides[0]), p(W), C.c_int64(W.strides[0]), 0, p(Cm),
                     C.c_int64(Cm.strides[0]), 4, 512, 64)
    out["w8_A"], out["w8_W"], out["w8_C"], out["w8_dq"] = A, W, Cm, np.float32(dq)

    # mat-vec
    for i, (M, K) in enumerate([(37, 80), (33, 127), (64, 96)]):
        Ap = np.zeros((M + 1, K + 64), np.uint16)
        Ap[:M, :K] = bf16((M, K), 1.0)
        A = Ap[:M, :K]
        b = np.zeros(K + 64, np.uint16)
        b[:K] = bf16((K,), 1.0)
        c = np.zeros(M + 16, np.float32)
        r.ref_matvec_bf16(p(A), C.c_int64(A.strides[0]), p(b), p(c), M, K)
        c2 = np.zeros(M + 16, np.float32)
        r.ref_gemavb(p(A), C.c_int64(A.strides[0]), p(b), p(c2), M, K)
        out[f"mv_{i}_A"], out[f"mv_{i}_b"] = np.ascontiguousarray(A), b[:K].copy()
        out[f"mv_{i}_amx"], out[f"mv_{i}_avb"] = c[:M].copy(), c2[:M].copy()

    path = os.path.join(HERE, "fc_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes,", len(out), "arrays")


if __name__ == "__main__":
    main()
