"""Builds libmm_amx_amd.so (HIP kernels + C ABI) in-tree for gfx950 with hipcc."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libmm_amx_amd.so")
SOURCES = ["abi.hip", "gemm_bf16.hip", "gemm_i8.hip", "skinny.hip", "repack.hip", "probe.hip"]
# -ffp-contract=off: the epilogues reproduce the reference's separately rounded mul/add sequence;
# fused operations are spelled fmaf().  Packed fp32 VALU instructions stay disabled.
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-Wall", "-Wno-unused-function",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def build(verbose=False):
    objs = []
    procs = []
    for src in SOURCES:
        obj = os.path.join(CSRC, src.replace(".hip", ".o"))
        cmd = ["hipcc"] + FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    failed = False
    for src, p in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if p.returncode != 0:
            failed = True
            print(f"[build] {src} FAILED\n{out}", file=sys.stderr)
        elif out.strip() and verbose:
            print(out)
    if failed:
        raise RuntimeError("hipcc failed")
    subprocess.check_call(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs)
    for obj in objs:
        os.remove(obj)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
