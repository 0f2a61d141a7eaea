"""Builds libmm_amx_amd.so (HIP kernels + C ABI) in-tree for gfx950 with hipcc.

    python -m mm_amx_amd.build [--incremental] [--stamps]

By default every source is compiled again; --incremental keeps the object files of earlier runs and
recompiles only what is older than its source or than a header.  --stamps builds a second library,
libmm_amx_amd_stamps.so, whose tile kernels record the shader clock at the phase boundaries of every
workgroup (-DMMX_STAMPS; read by mm_amx_amd.phase_stamps); the shipped library holds no such code.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libmm_amx_amd.so")
# the MFMA tile GEMM is instantiated per (input type, output type) pair in a file of its own, so that the
# pairs compile side by side
SOURCES = ["abi.hip", "gemm_bf16.hip", "gemm_i8.hip", "gemm_w8.hip",
           "gemm_w8_out_bf16.hip", "gemm_w8_out_f32.hip", "gemm_w8_out_i8.hip",
           "gemm_bf16_out_bf16.hip", "gemm_bf16_out_f32.hip", "gemm_bf16_out_i8.hip",
           "gemm_i8_out_i8.hip", "gemm_i8_out_i32.hip", "gemm_i8_out_f32.hip", "gemm_i8_out_bf16.hip",
           "skinny.hip", "repack.hip", "probe.hip", "u8.hip"]
HEADERS = ["common.hpp", "gemm_tile.hpp", os.path.join("..", "..", "include", "mm_amx_amd.h"),
           os.path.join("..", "..", "include", "mm_amx_amd_bench.h")]
# -ffp-contract=off: the epilogues reproduce the reference's separately rounded mul/add sequence;
# fused operations are spelled fmaf().  Packed fp32 VALU instructions stay disabled.
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-Wall", "-Wno-unused-function",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
JOBS = 8


def _stale(obj, src):
    if not os.path.isfile(obj):
        return True
    t = os.path.getmtime(obj)
    deps = [src] + [os.path.join(CSRC, h) for h in HEADERS] + [os.path.abspath(__file__)]
    return any(os.path.getmtime(d) > t for d in deps)


def build(verbose=False, incremental=False, stamps=False):
    lib = LIB.replace(".so", "_stamps.so") if stamps else LIB
    flags = FLAGS + (["-DMMX_STAMPS"] if stamps else [])
    objs = [os.path.join(CSRC, src.replace(".hip", ".stamps.o" if stamps else ".o")) for src in SOURCES]
    todo = [(src, obj) for src, obj in zip(SOURCES, objs)
            if not incremental or _stale(obj, os.path.join(CSRC, src))]
    failed = False
    running = []

    def reap(p_src, p):
        nonlocal failed
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if p.returncode != 0:
            failed = True
            print(f"[build] {p_src} FAILED\n{out}", file=sys.stderr)
        elif out.strip() and verbose:
            print(out)

    for src, obj in todo:
        while len(running) >= JOBS:
            reap(*running.pop(0))
        cmd = ["hipcc"] + flags + ["-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        running.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    for item in running:
        reap(*item)
    if failed:
        raise RuntimeError("hipcc failed")
    subprocess.check_call(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib] + objs)
    if not incremental:
        for obj in objs:
            os.remove(obj)
    return lib


if __name__ == "__main__":
    print(build(verbose=True, incremental="--incremental" in sys.argv[1:], stamps="--stamps" in sys.argv[1:]))
