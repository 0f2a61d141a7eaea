"""CPU-side checks of the C-ABI library: it loads, exports every symbol the header declares, and
rejects bad arguments before touching a device.  No compute call is made here."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "mm_amx_amd", "libmm_amx_amd.so")
HEADER = os.path.join(ROOT, "include", "mm_amx_amd.h")


@pytest.fixture(scope="module")
def lib():
    if not os.path.isfile(LIB):
        pytest.fail(f"{LIB} has not been built (python -m mm_amx_amd.build)")
    return C.CDLL(LIB)


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mmx_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_path():
    names = declared_functions()
    for must in ("mmx_repack_b", "mmx_gemm", "mmx_matvec", "mmx_mlp", "mmx_last_error", "mmx_init"):
        assert must in names


def test_every_declared_symbol_is_exported(lib):
    for name in declared_functions():
        assert hasattr(lib, name), f"{name} declared in mm_amx_amd.h but not exported"


def test_python_binding_lists_the_same_exports():
    import mm_amx_amd._lib as L
    assert sorted(L.EXPORTS) == declared_functions()


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
    # NULL operands are rejected by validation, before any HIP call
    assert lib.mmx_gemm(1, 1, None, C.c_int64(0), None, 1, 64, 64, 0, 64, None, None) == -1
    assert b"NULL" in lib.mmx_last_error()
    assert lib.mmx_repack_b(5, None, C.c_int64(0), 1, 1, 0, None, None) == -1


def test_package_fails_loudly_without_the_library(monkeypatch):
    import mm_amx_amd._lib as L
    monkeypatch.setattr(L, "_lib", None)
    monkeypatch.setattr(L, "_LIB_PATH", "/nonexistent/libmm_amx_amd.so")
    with pytest.raises(L.MmxError, match="no CPU or PyTorch fallback"):
        L.lib()
