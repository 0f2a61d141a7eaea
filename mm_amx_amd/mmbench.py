"""Matmul latency comparison in the shape of the reference's benchmark/mmbench.

``benchmark(transB, constb, M, N, K, duration, cacheMB, check)`` has the arguments and the result
keys (``latency_ms``, ``times``, ``duration``, ``correct``) of the reference's per-backend
``benchmark`` functions (benchmark/mmbench/utils.hpp:42-165, mmamx.cpp:108-131); the backends are
this library (``mmamx``: bf16 A and B, fp32 C, amx_kernel::Matmul semantics incl. constB) and
torch.matmul on the same device tensors (hipBLASLt; the column the reference fills with oneDNN / MKL /
CPU torch, benchmark/mmbench/__main__.py:16-48).  The protocol is the reference's: two warm-up runs,
one run to estimate the latency, then ``duration / estimate`` timed runs, each preceded by a copy of
``cacheMB`` megabytes that evicts the operands from the caches; every run is timed on its own
(HIP events on the launch stream where the reference reads the TSC).

    python -m mm_amx_amd.mmbench --mnk 32 10240 10240 --constb -d 2 -c 512 --check
"""
import argparse
import time

import torch

from . import ops

_CHUNK = 256  # runs timed per synchronisation


class _Task:
    """MatmulTask (benchmark/mmbench/utils.hpp:42-99): operands, optional cache-clearing buffers, reference result."""

    def __init__(self, transb, constb, M, N, K, cacheMB, check):
        g = torch.Generator(device="cuda").manual_seed(M * 131 + N * 17 + K)
        self.transb, self.constb = transb, constb
        self.A = (torch.rand((M, K), device="cuda", generator=g) - 0.5).bfloat16()
        self.B = (torch.rand((N, K) if transb else (K, N), device="cuda", generator=g) - 0.5).bfloat16()
        self.C = torch.zeros((M, N), dtype=torch.float32, device="cuda")
        self.clr = None
        if cacheMB > 0:
            self.clr = (torch.ones(cacheMB << 20, dtype=torch.uint8, device="cuda"),
                        torch.empty(cacheMB << 20, dtype=torch.uint8, device="cuda"))
        self.C0 = None
        if check:
            Bm = self.B.t() if transb else self.B
            self.C0 = (self.A.double() @ Bm.double()).float()

    def clear_cache(self):
        if self.clr is not None:
            self.clr[1].copy_(self.clr[0])


class _Mmamx(_Task):
    def init(self):
        self.op = ops.Matmul(self.constb, self.transb)
        self.pp = ops.BiasGeluStore(self.C)

    def run(self):
        self.op(self.A, self.B, ppkernel=self.pp)


class _Torch(_Task):
    def init(self):
        self.Bm = self.B.t() if self.transb else self.B
        self.out = torch.empty((self.A.shape[0], self.Bm.shape[1]), dtype=torch.bfloat16, device="cuda")

    def run(self):
        torch.matmul(self.A, self.Bm, out=self.out)
        self.C = self.out


_BACKENDS = {"mmamx": _Mmamx, "torch": _Torch}


def _timed_runs(task, times):
    total_ms, done = 0.0, 0
    while done < times:
        n = min(_CHUNK, times - done)
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]
        for a, b in ev:
            task.clear_cache()
            a.record()
            task.run()
            b.record()
        torch.cuda.synchronize()
        total_ms += sum(a.elapsed_time(b) for a, b in ev)
        done += n
    return total_ms


def benchmark(transB, constb, M, N, K, duration, cacheMB, check, backend="mmamx"):
    """One backend on one shape; returns {latency_ms, times, duration[, correct]}."""
    task = _BACKENDS[backend](transB, constb, M, N, K, cacheMB, check)
    task.init()
    for _ in range(2):
        task.clear_cache()
        task.run()
    est_ms = max(_timed_runs(task, 1), 1e-3)
    times = max(1, int(duration * 1e3 / est_ms))
    t0 = time.time()
    total_ms = _timed_runs(task, times)
    ret = {"latency_ms": total_ms / times, "times": times, "duration": time.time() - t0}
    if check:
        got = task.C.float()
        err = (torch.linalg.norm(got.double() - task.C0.double()) / torch.linalg.norm(task.C0.double())).item()
        # fp32 output of this library: 1e-5; the bf16 output of torch.matmul carries its own rounding (2^-9)
        ret["correct"] = bool(err <= (1e-5 if got.dtype == task.C.dtype and backend == "mmamx" else 4e-3))
        ret["rel_err"] = err
    return ret


def main(argv=None):
    ap = argparse.ArgumentParser(prog="python -m mm_amx_amd.mmbench", description=__doc__.split("\n")[0])
    ap.add_argument("-c", "--cacheMB", type=int, default=0)
    ap.add_argument("-d", "--duration", type=float, default=10)
    ap.add_argument("--constb", action="store_true")
    ap.add_argument("--transb", action="store_true")
    ap.add_argument("--check", action="store_true")
    ap.add_argument("--mnk", nargs=3, type=int, default=[32, 10240, 10240])  # benchmark/mmbench/__main__.py:54
    args = ap.parse_args(argv)
    M, N, K = args.mnk
    print(f"benchmark on M,N,K=[{M},{N},{K}] constb={args.constb} transb={args.transb} duration={args.duration} "
          f"cacheMB={args.cacheMB}")
    ops.L.init(0)
    for _ in range(2):
        for name in ("mmamx", "torch"):
            r = benchmark(args.transb, args.constb, M, N, K, args.duration, args.cacheMB, args.check, backend=name)
            tf = 2.0 * M * N * K / (r["latency_ms"] * 1e-3) / 1e12
            print(f"{name:>6}: {r}  ({tf:.1f} TFLOP/s)")


if __name__ == "__main__":
    main()
