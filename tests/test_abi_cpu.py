"""CPU-side checks of the C-ABI library: it loads, exports every symbol the header declares, and
rejects bad arguments before touching a device.  No compute call is made here."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "mm_amx_amd", "libmm_amx_amd.so")
HEADER = os.path.join(ROOT, "include", "mm_amx_amd.h")
BENCH_HEADER = os.path.join(ROOT, "include", "mm_amx_amd_bench.h")


@pytest.fixture(scope="module")
def lib():
    if not os.path.isfile(LIB):
        pytest.fail(f"{LIB} has not been built (python -m mm_amx_amd.build)")
    return C.CDLL(LIB)


def declared_functions(header=HEADER):
    text = open(header).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mmx_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_path():
    names = declared_functions()
    for must in ("mmx_repack_b", "mmx_gemm", "mmx_matvec", "mmx_mlp", "mmx_last_error", "mmx_init"):
        assert must in names


def test_every_declared_symbol_is_exported(lib):
    for header in (HEADER, BENCH_HEADER):
        for name in declared_functions(header):
            assert hasattr(lib, name), f"{name} declared in {os.path.basename(header)} but not exported"


def test_python_binding_lists_the_same_exports():
    import mm_amx_amd._lib as L
    assert sorted(L.EXPORTS) == declared_functions()
    assert sorted(L.BENCH_EXPORTS) == declared_functions(BENCH_HEADER)


def test_measurement_aids_are_not_part_of_the_operator_header():
    """Timing and probe entry points live in mm_amx_amd_bench.h; the operator ABI declares none of them."""
    ops = declared_functions()
    assert not [n for n in ops if "probe" in n or "time" in n]


def test_sizes_and_argument_validation(lib):
    lib.mmx_packed_b_bytes.restype = C.c_size_t
    lib.mmx_last_error.restype = C.c_char_p
    # bf16: K padded to 64, N to 32; int8: K padded to 128
    assert lib.mmx_packed_b_bytes(1, 4096, 11008) == 4096 * 11008 * 2
    assert lib.mmx_packed_b_bytes(1, 65, 33) == 128 * 64 * 2
    assert lib.mmx_packed_b_bytes(2, 65, 33) == 128 * 64
    assert lib.mmx_packed_b_bytes(0, 64, 64) == 0
    assert lib.mmx_set_tile(b"17x3") != 0 and b"17x3" in lib.mmx_last_error()
    assert lib.mmx_set_tile(b"256x192") == 0 and lib.mmx_set_tile(b"") == 0
    assert lib.mmx_set_option(b"load_mode", 7) != 0
    assert lib.mmx_set_option(b"nonsense", 1) != 0
    # every documented option takes its documented values and nothing else
    for name, good, bad in ((b"load_mode", (0, 2), (1, 3)), (b"waves", (4, 8), (2, 16)), (b"decode_halves", (-1, 0, 1), (-2, 2)),
                            (b"decode_valu", (-1, 0, 1), (-2, 2)), (b"decode_resident", (-1, 0, 1), (-2, 2)),
                            (b"decode_pair", (0, 1), (-1, 2))):
        for v in bad:
            assert lib.mmx_set_option(name, v) != 0, (name, v)
        for v in good:
            assert lib.mmx_set_option(name, v) == 0, (name, v)
    assert lib.mmx_set_option(b"load_mode", 2) == 0 and lib.mmx_set_option(b"waves", 8) == 0
    assert lib.mmx_set_option(b"decode_halves", -1) == 0 and lib.mmx_set_option(b"decode_valu", -1) == 0
    assert lib.mmx_set_option(b"decode_resident", -1) == 0
    # NULL operands are rejected by validation, before any HIP call
    assert lib.mmx_gemm(1, 1, None, C.c_int64(0), None, 1, 64, 64, 0, 64, None, None) == -1
    assert b"NULL" in lib.mmx_last_error()
    assert lib.mmx_repack_b(7, None, C.c_int64(0), 1, 1, 0, None, None) == -1   # no such dtype
    assert lib.mmx_repack_b(5, None, C.c_int64(0), 1, 1, 0, None, None) == -1   # unsigned bytes, NULL pointers
    assert lib.mmx_gemm_u8(2, 2, None, C.c_int64(0), None, 1, 64, 64, 0, 64, None, None, C.c_size_t(0), None) == -1  # nothing unsigned
    lib.mmx_gemm_u8_scratch_bytes.restype = C.c_size_t
    assert lib.mmx_gemm_u8_scratch_bytes(2, 2, 4, 64, 64, 0, 64) == 0 and lib.mmx_gemm_u8_scratch_bytes(5, 2, 4, 64, 64, 0, 64) > 0


def test_package_fails_loudly_without_the_library(monkeypatch):
    import mm_amx_amd._lib as L
    monkeypatch.setattr(L, "_lib", None)
    monkeypatch.setattr(L, "_LIB_PATH", "/nonexistent/libmm_amx_amd.so")
    with pytest.raises(L.MmxError, match="no CPU or PyTorch fallback"):
        L.lib()


# ---- the Python binding checks shapes and dtypes on the host, before any pointer crosses the boundary ----------
def _cpu_case():
    import torch
    import mm_amx_amd._lib as L
    A = torch.zeros((64, 128), dtype=torch.bfloat16)
    packed = torch.zeros(L._packed_bytes_host(L.BF16, 128, 96), dtype=torch.uint8)
    C_out = torch.zeros((64, 96), dtype=torch.float32)
    return torch, L, A, packed, C_out


def test_host_restatement_of_the_packed_size(lib):
    import mm_amx_amd._lib as L
    lib.mmx_packed_b_bytes.restype = C.c_size_t
    for dt in (L.BF16, L.I8, L.I4):
        for K, N in ((64, 32), (65, 33), (4096, 11008), (300, 45), (1, 1)):
            assert L._packed_bytes_host(dt, K, N) == lib.mmx_packed_b_bytes(dt, K, N)


def test_gemm_rejects_wrong_sizes_before_any_launch():
    torch, L, A, packed, C_out = _cpu_case()

    class Ep:  # the fields gemm() reads, without the GPU-residency check of L.Epilogue
        def __init__(self, Cx, steps=0, bias=None, deq=None, q=None):
            self.C, self.steps, self.bias, self.deq_oc, self.q_oc = Cx, steps, bias, deq, q

    with pytest.raises(L.MmxError, match="C is"):
        L.gemm(A, packed, 96, Ep(C_out[:32]))            # too few rows
    with pytest.raises(L.MmxError, match="C is"):
        L.gemm(A, packed, 96, Ep(C_out[:, :64]))         # too few columns
    with pytest.raises(L.MmxError, match="Bpacked holds"):
        L.gemm(A, packed[:-1], 96, Ep(C_out))
    with pytest.raises(L.MmxError, match="uint8"):
        L.gemm(A, packed.view(torch.int8), 96, Ep(C_out))
    with pytest.raises(L.MmxError, match="bias holds"):
        L.gemm(A, packed, 96, Ep(C_out, L.PP_BIAS, bias=torch.zeros(95)))
    with pytest.raises(L.MmxError, match="deq_scale_per_oc holds"):
        L.gemm(A, packed, 96, Ep(C_out, L.PP_DEQUANT, deq=torch.zeros(10)))
    with pytest.raises(L.MmxError, match="column range"):
        L.gemm(A, packed, 96, Ep(C_out), n0=0, n1=128)
    with pytest.raises(L.MmxError, match="2-D"):
        L.gemm(A[0], packed, 96, Ep(C_out))
    with pytest.raises(L.MmxError, match="not part of this path"):
        L.gemm(A.to(torch.float16), packed, 96, Ep(C_out))
    # SILU_GATE halves the columns of C
    with pytest.raises(L.MmxError, match="C is"):
        L.gemm(A, torch.zeros(L._packed_bytes_host(L.BF16, 128, 128), dtype=torch.uint8), 128, Ep(C_out[:, :63], L.PP_SILU_GATE))
    # everything in order: the call gets as far as asking for GPU tensors, and no further
    with pytest.raises(L.MmxError, match="on the GPU"):
        L.gemm(A, packed, 96, Ep(C_out))


def test_matvec_and_mlp_reject_wrong_sizes_before_any_launch():
    torch, L, A, packed, C_out = _cpu_case()
    with pytest.raises(L.MmxError, match="b must be"):
        L.matvec(A, torch.zeros(127, dtype=torch.bfloat16))
    with pytest.raises(L.MmxError, match="b must be"):
        L.matvec(A, torch.zeros(128, dtype=torch.float32))
    with pytest.raises(L.MmxError, match="b must be"):
        L.matvec(A, torch.zeros(256, dtype=torch.bfloat16)[::2])
    with pytest.raises(L.MmxError, match="out must be"):
        L.matvec(A, torch.zeros(128, dtype=torch.bfloat16), torch.zeros(63, dtype=torch.float32))
    with pytest.raises(L.MmxError, match="out must be"):
        L.matvec(A, torch.zeros(128, dtype=torch.bfloat16), torch.zeros(64, dtype=torch.int32))
    with pytest.raises(L.MmxError, match="on the GPU"):
        L.matvec(A, torch.zeros(128, dtype=torch.bfloat16))
    K, N = 128, 96
    gu = torch.zeros(L._packed_bytes_host(L.BF16, K, 2 * N), dtype=torch.uint8)
    dn = torch.zeros(L._packed_bytes_host(L.BF16, N, K), dtype=torch.uint8)
    with pytest.raises(L.MmxError, match="x must be bf16"):
        L.mlp(A.float(), gu, dn, N)
    with pytest.raises(L.MmxError, match="w_gate_up"):
        L.mlp(A, gu[:-1], dn, N)
    with pytest.raises(L.MmxError, match="w_down"):
        L.mlp(A, gu, dn[:100], N)
    with pytest.raises(L.MmxError, match="h must be"):
        L.mlp(A, gu, dn, N, h=torch.zeros((64, N - 1), dtype=torch.bfloat16))
    with pytest.raises(L.MmxError, match="y must be"):
        L.mlp(A, gu, dn, N, y=torch.zeros((64, K), dtype=torch.float32))
    with pytest.raises(L.MmxError, match="multiple of 32"):
        L.mlp(A, gu, dn, 90)
    with pytest.raises(L.MmxError, match="on the GPU"):
        L.mlp(A, gu, dn, N)
    from mm_amx_amd import ops
    m = ops.MLP()
    with pytest.raises(L.MmxError, match="setup has not"):
        m.run(A)
    m.m_K, m.m_N, m.gate_up, m.down = K, N, gu, dn
    with pytest.raises(L.MmxError, match=r"x must be \[M, 128\]"):
        m.run(torch.zeros((4, 64), dtype=torch.bfloat16))


def test_abi_rejects_overlapping_rows_of_c_and_misaligned_operands(lib):
    lib.mmx_last_error.restype = C.c_char_p

    class Ep(C.Structure):
        _fields_ = [("steps", C.c_uint32), ("out_dtype", C.c_int32), ("C", C.c_void_p), ("ldc_bytes", C.c_int64),
                    ("bias", C.c_void_p), ("deq_scale", C.c_float), ("deq_scale_per_oc", C.c_void_p),
                    ("q_scale", C.c_float), ("q_scale_per_oc", C.c_void_p)]
    gemm = lib.mmx_gemm
    gemm.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_int64, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int,
                     C.POINTER(Ep), C.c_void_p]
    fake = 0x10000  # never dereferenced: validation fails first
    ep = Ep(0, 0, fake, 4 * 63, None, 1.0, None, 0.0, None)   # fp32 rows of 63 < 64 columns
    assert gemm(1, 1, fake, 256, fake, 64, 128, 64, 0, 64, C.byref(ep), None) == -1
    assert b"ldc_bytes" in lib.mmx_last_error()
    ep = Ep(0, 0, fake, -256, None, 1.0, None, 0.0, None)
    assert gemm(1, 1, fake, 256, fake, 64, 128, 64, 0, 64, C.byref(ep), None) == -1
    mv = lib.mmx_matvec
    mv.argtypes = [C.c_int, C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p]
    assert mv(1, fake + 1, 256, fake, fake, 4, 128, None) == -1 and b"aligned" in lib.mmx_last_error()
    assert mv(1, fake, 255, fake, fake, 4, 100, None) == -1
    qw = lib.mmx_quantize_weights
    qw.argtypes = [C.c_void_p, C.c_int64, C.c_int, C.c_int, C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p]
    assert qw(fake + 1, 256, 4, 128, fake, 128, fake, fake, None) == -1 and b"aligned" in lib.mmx_last_error()
    # K split requests that can be refused without a device
    sk = lib.mmx_gemm_splitk
    sk.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_int64, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int,
                   C.POINTER(Ep), C.c_int, C.c_void_p, C.c_size_t, C.c_void_p]
    ep = Ep(0, 0, fake, 4 * 64, None, 1.0, None, 0.0, None)
    assert sk(1, 1, fake, 256, fake, 64, 128, 64, 0, 64, C.byref(ep), 2, None, 0, None) == -1 and b"workspace" in lib.mmx_last_error()
    assert sk(1, 1, fake, 256, fake, 64, 128, 64, 0, 64, C.byref(ep), -1, fake, 1 << 20, None) == -1
    assert sk(1, 1, fake, 256, fake, 64, 128, 64, 0, 64, C.byref(ep), 2, fake + 16, 1 << 20, None) == -1 and b"256-byte" in lib.mmx_last_error()
    assert sk(1, 1, fake, 256, fake, 8, 128, 64, 0, 64, C.byref(ep), 2, fake, 1 << 20, None) == -2 and b"decode" in lib.mmx_last_error()


def test_tuning_knobs_are_per_thread(lib):
    """mmx_set_tile / mmx_set_option change the calling thread's dispatch only; a first call from two threads at once
    must not race on anything."""
    import threading
    lib.mmx_last_error.restype = C.c_char_p
    seen = {}

    def worker(name, shape, ok):
        rc = lib.mmx_set_tile(shape)
        err = lib.mmx_last_error()
        seen[name] = (rc, err)

    t1 = threading.Thread(target=worker, args=("good", b"256x192", True))
    t2 = threading.Thread(target=worker, args=("bad", b"17x3", False))
    t1.start(), t2.start(), t1.join(), t2.join()
    assert seen["good"][0] == 0 and seen["bad"][0] == -1 and b"17x3" in seen["bad"][1]
    assert b"17x3" not in lib.mmx_last_error()  # this thread's error string is its own


def test_workspace_query_covers_the_decode_kernels_k_split():
    """mmx_gemm_workspace_bytes (a host-side computation; 256 CUs assumed before mmx_init has seen a device): decode shapes
    with panels for at most two thirds of the CUs report the counters plus one 4 KiB block of sums per panel and slice,
    every operand type; more panels, k_splits = 1 and SILU_GATE report none."""
    import mm_amx_amd as mx
    counters = 16 << 10
    assert mx.gemm_workspace_bytes(mx.BF16, mx.I8, 32, 8192, 1024) == counters + 32 * 4 * 4096          # 32 panels, 4 slices
    assert mx.gemm_workspace_bytes(mx.BF16, mx.BF16, 16, 11008, 4096) == counters + 128 * 2 * 4096      # 128 panels, 2 slices
    assert mx.gemm_workspace_bytes(mx.BF16, mx.I4, 16, 8192, 1024) == counters + 32 * 4 * 4096
    assert mx.gemm_workspace_bytes(mx.I8, mx.I8, 32, 8192, 1024) == counters + 32 * 4 * 4096
    assert mx.gemm_workspace_bytes(mx.BF16, mx.I8, 32, 8192, 4160) == counters + 130 * 3 * 4096         # 130 panels, 3 slices
    assert mx.gemm_workspace_bytes(mx.BF16, mx.I8, 32, 4096, 4160) == 0                                 # ... too short for three
    assert mx.gemm_workspace_bytes(mx.BF16, mx.I8, 32, 8192, 8192) == 0
    assert mx.gemm_workspace_bytes(mx.BF16, mx.I8, 32, 8192, 1024, k_splits=1) == 0
    assert mx.gemm_workspace_bytes(mx.BF16, mx.BF16, 32, 8192, 1024, steps=mx.PP_SILU_GATE) == 0
    assert mx.gemm_workspace_bytes(mx.BF16, mx.BF16, 64, 4096, 512) > counters                          # the tile kernels' plan


def test_bench_traffic_figures_belong_to_the_current_kernel_sources():
    """bench.py reports a measured HBM traffic only for the kernel source it was measured on (keyed by a hash of the
    file): after a change of such a file the figure has to be measured again, or the bench reports null."""
    import importlib.util
    spec = importlib.util.spec_from_file_location("bench_for_test", os.path.join(ROOT, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    for kernel in bench.MEASURED_TRAFFIC:
        assert bench.measured_traffic(kernel) is not None, f"{kernel}: its source changed after the traffic was measured"


def test_repackB_1xL_checks_the_reference_preconditions():
    """repackB_1xL asserts K % 32 == 0 and N % (16 L) == 0 (weight_compression/fc16m.cpp:66-67); here they raise, as do
    a source that is not bf16, an L outside 1..4 and a scale on the bf16 form - all before anything reaches the library."""
    import torch

    import mm_amx_amd as mx
    good = torch.zeros((64, 64), dtype=torch.bfloat16)
    for bad_call in (lambda: mx.repackB_1xL(torch.zeros((48, 64), dtype=torch.bfloat16), torch.int8, 2, 2.0),
                     lambda: mx.repackB_1xL(torch.zeros((64, 48), dtype=torch.bfloat16), torch.int8, 2, 2.0),
                     lambda: mx.repackB_1xL(torch.zeros((64, 64), dtype=torch.float32), torch.int8, 2, 2.0),
                     lambda: mx.repackB_1xL(good, torch.int8, 5, 2.0),
                     lambda: mx.repackB_1xL(good, torch.bfloat16, 2, 2.0),
                     lambda: mx.repackB_1xL(good, torch.float32, 2, 1.0)):
        with pytest.raises(mx.MmxError):
            bad_call()


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU: --gpus above 1 exits with a message that says so, before anything touches a device."""
    import subprocess
    import sys
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "ONE GPU" in r.stderr and "--gpus must be 1" in r.stderr
    assert not r.stdout.strip()
