"""The C++ operator classes (include/mm_amx_amd/kernels_gfx950.hpp): they compile with a plain host
compiler, and the parity driver built from tests/cpp passes on the GPU."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DRIVER = os.path.join(ROOT, "tests", "cpp", "test_host_api")


def test_header_compiles_with_host_compiler(tmp_path):
    src = tmp_path / "use.cpp"
    src.write_text('#include "mm_amx_amd/kernels_gfx950.hpp"\n'
                   "using namespace gfx950_kernel;\n"
                   "void f(tensor2D<bfloat16>& A, tensor2D<bfloat16>& B, tensor2D<bfloat16>& C, float* bias) {\n"
                   "    Matmul<bfloat16, bfloat16> mm(true, false);\n"
                   "    mm(A, B, PP::BiasGeluStore<bfloat16, PP::BIAS_GELU>(C, bias));\n"
                   "    Matmul<bfloat16, int8_t> mw(true, false);\n"
                   "    tensor2D<float> Cf(4, 4);\n"
                   "    mw(A, B, 0, 32, PP::BiasGeluStore<float, PP::DEQUANT>(Cf));\n"
                   "}\n")
    subprocess.check_call(["g++", "-std=c++14", "-fsyntax-only", "-Wall", "-Werror", "-D__HIP_PLATFORM_AMD__",
                           "-I/opt/rocm/include", "-I" + os.path.join(ROOT, "include"), str(src)])


@pytest.mark.gpu
def test_cpp_driver_passes_on_gpu():
    if not os.path.isfile(DRIVER):
        pytest.fail(f"{DRIVER} is not built: run `make -C tests/cpp` (or __graft_entry__.build())")
    r = subprocess.run([DRIVER], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
    print(r.stdout)
    assert r.returncode == 0, r.stdout[-4000:]
