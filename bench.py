#!/usr/bin/env python3
"""Benchmark of the FC-GEMM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-extra]

One "step" is one pass of the hot path over one batch of synthetic input: the Llama-7B FFN
up-projection FC, bf16, M=1024, K=4096, N=11008, fused BIAS+GELU epilogue, bf16 output, with the
activations, the packed weights and the bias already resident in HBM when the timed region starts.
Prints ONE JSON line.  `value` is TFLOP/s of that FC (flops = 2*M*N*K, the reference's convention,
main.cpp:279); `roofline` holds the same kernel against the MI355X dense bf16 MFMA peak, timed with
HIP events on the launch stream; `cpu_baseline` is the CPU restatement of the reference path
(oracle/) timed on this machine's host cores on the same workload; `extra` reports the other
configurations of the path (int8 FC, decode GEMV over int8 weights, fused MLP).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_INT8_TOPS = 5000.0     # MI355X dense int8 MFMA
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E

# HBM-side bytes per launch, from two counter runs of this script under `rocprofv3 --pmc FETCH_SIZE` and
# `--pmc WRITE_SIZE` (KiB per dispatch), each scaled by what the same counter reads for the 256 MiB device copy of
# --calibrate-copy (factors 2.000 and 1.000); the summaries are profiles/*_hbm_traffic.txt and
# profiles/skinny_stream_w8_*.txt.  Counters cannot be read from inside the process, so a figure is only reported
# when the kernel that ran is the one profiled AND its source is the one that was profiled (first 16 hex digits of
# the SHA-256 of the kernel's source file): after a change of the kernel the figure reads null until it is re-measured.
MEASURED_TRAFFIC = {
    "gemm_bf16_256x192_ring8w_out_bf16": {"bytes": (81718.2 * 2.000 + 27580.4 * 1.000) * 1024, "source": "mm_amx_amd/csrc/gemm_tile.hpp",
                                          "sha": "497af55a19cd666b"},
    "skinny_stream_w8": {"bytes": (22154.3 * 2.000 + 21.5 * 1.000) * 1024, "source": "mm_amx_amd/csrc/skinny.hip", "sha": "b5f086f849d23a5a"},
    "skinny_resident_w8_pair": {"bytes": (22617.9 * 2.000 + 344.0 * 1.000) * 1024, "source": "mm_amx_amd/csrc/skinny.hip", "sha": "b5f086f849d23a5a"},
}


def measured_traffic(kernel_name):
    import hashlib
    m = MEASURED_TRAFFIC.get(kernel_name)
    if not m:
        return None
    with open(os.path.join(ROOT, m["source"]), "rb") as f:
        sha = hashlib.sha256(f.read()).hexdigest()[:16]
    return m["bytes"] if sha == m["sha"] else None


def host_cores():
    cores = os.cpu_count() or 1
    try:
        cores = len(os.sched_getaffinity(0))
    except AttributeError:
        pass
    return min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))


def time_cpu(fn, budget_s):
    """(repetitions, seconds): fn() repeated until budget_s has passed (after one untimed call)."""
    fn()
    reps, t0 = 0, time.perf_counter()
    while True:
        fn()
        reps += 1
        el = time.perf_counter() - t0
        if el > budget_s:
            return reps, el


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--cpu-seconds", type=float, default=10.0, help="CPU time budget of the headline baseline (the others get a third each)")
    ap.add_argument("--no-extra", action="store_true", help="skip the secondary configurations")
    ap.add_argument("--progress", action="store_true", help="name each section on stderr before it starts")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a 256 MiB device-to-device copy: a kernel of known traffic to scale profiler byte counters by")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (the path would shard over N by column panels, nothing here does); "
                 "--gpus must be 1")

    import numpy as np
    import torch

    import mm_amx_amd as mx
    from mm_amx_amd import workloads as wl
    dev, dev_bf16 = wl.to_device, wl.to_device_bf16

    torch.cuda.set_device(0)
    mx.init(0)

    def progress(name):
        if args.progress:
            print(f"bench.py: {name}", file=sys.stderr, flush=True)

    progress("headline")
    # ---- headline: bf16 FC + BIAS_GELU, M=1024 ------------------------------------------------------
    w = wl.ffn_up_bias_gelu(M=1024)
    M, K, N = w["M"], w["K"], w["N"]
    A = dev_bf16(w["A"])
    Bp = mx.repack_b(dev_bf16(w["B"]))   # one-off, untimed (the reference caches it under constB)
    bias = dev(w["bias"])
    C = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")
    ep = mx.Epilogue(C, mx.PP_BIAS | mx.PP_GELU, bias=bias)
    flops = 2.0 * M * N * K

    def step():
        mx.gemm(A, Bp, N, ep)

    # Spin-up, not part of the W warm-up steps: the first ~100 launches after start-up run at lower
    # clocks (about 115 us instead of 97 us per launch was measured), so bring the device to its
    # steady state before anything is counted.
    for _ in range(300):
        step()
    torch.cuda.synchronize()
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()                       # same stream the kernels are launched on (torch's current stream)
    for _ in range(args.steps):
        step()
    e1.record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    kernel_ms = e0.elapsed_time(e1) / args.steps
    kernel_name = mx.last_kernel()
    value = flops / (ms_per_step * 1e-3) / 1e12
    achieved = flops / (kernel_ms * 1e-3) / 1e12
    # the same launches once more in chunks of ten with an event between the chunks: the median chunk mean (not part
    # of `value`; an event between every two launches would add its own gap to each of them)
    nchunk = max(1, args.steps // 10)
    evs = [torch.cuda.Event(enable_timing=True) for _ in range(nchunk + 1)]
    evs[0].record()
    for i in range(nchunk):
        for _ in range(10):
            step()
        evs[i + 1].record()
    torch.cuda.synchronize()
    per_chunk = sorted(evs[i].elapsed_time(evs[i + 1]) / 10 for i in range(nchunk))
    kernel_median_ms = per_chunk[len(per_chunk) // 2]

    out = {
        "metric": "bf16 FC GEMM TFLOP/s (M=1024, K=4096, N=11008, fused BIAS+GELU, bf16 out)",
        "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "llama7b_ffn_up_bf16_bias_gelu", "M": M, "K": K, "N": N, "kernel": kernel_name,
                   "inputs": "A~N(0,1) bf16, B~N(0,0.02) bf16 repacked once, bias~N(0,0.1) fp32, all resident in HBM",
                   "parity": "not checked in this run (--no-cpu); tests/test_gpu_parity.py::test_ffn_up_bias_gelu_full_size checks this shape"},
        "roofline": {"bound": "mfma", "achieved": round(achieved, 2), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(achieved / PEAK_BF16_TFLOPS, 4),
                     "traffic": measured_traffic(kernel_name),
                     "algorithmic_flop_per_launch": flops,
                     "algorithmic_bytes_per_launch": 2 * M * K + 2 * K * N + 4 * N + 2 * M * N,
                     "kernel_avg_us": round(kernel_ms * 1e3, 2), "kernel_median_us": round(kernel_median_ms * 1e3, 2)},
    }

    if args.calibrate_copy:
        progress("calibrate_copy")
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        out["calibration_copy_bytes"] = {"read": 256 << 20, "written": 256 << 20}
        del src, dst

    # ---- CPU baselines: the oracle (a port of the reference path) and torch-CPU (oneDNN) on this host's cores ----
    # The reference itself cannot travel to this machine; what is timed is the CPU restatement of its arithmetic
    # (oracle/, kind "port") and, as the "oneDNN path" of the reference's own comparisons (benchmark/mmbench/dnnl.cpp),
    # torch's CPU matmul.  Every figure is over a bounded sample of the same workload; protocol as the reference's
    # timeit (warm-up, then repeat for the budget, mean).
    cpu_other = {}
    if not args.no_cpu:
        from oracle import pyoracle as po
        cores = host_cores()
        torch.set_num_threads(cores)
        isa = po.isa()
        amx = "has" if po.host_has_amx() else "has no"

        def onednn_bf16(Abits, Bbits, budget):
            At = torch.from_numpy(Abits.view(np.int16).copy()).view(torch.bfloat16)
            Bt = torch.from_numpy(Bbits.view(np.int16).copy()).view(torch.bfloat16)
            reps, el = time_cpu(lambda: torch.matmul(At, Bt), budget)
            return reps, el

        def gpu_note(fn):
            try:
                return fn()
            except Exception as e:  # a CPU op torch does not have on this host: say so, do not invent a number
                return {"value": None, "note": f"{type(e).__name__}: {e}"[:160]}

        def run_ref():
            acc = po.gemm_bf16(w["A"], w["B"], nthreads=cores)
            po.pp(acc, po.PP_BIAS | po.PP_GELU, po.BF16, bias=w["bias"])
        # parity of what the timed launches wrote, against the oracle on the first rows of the same inputs (untimed;
        # the oracle is the checker here, nothing of it is measured): relative Frobenius error and the share of elements
        # within one bf16 ulp, over all elements and where GELU is well conditioned (pre-activation above -3.5)
        rows = 64
        acc_ref = po.gemm_bf16(np.ascontiguousarray(w["A"][:rows]), w["B"], nthreads=cores)
        want = po.bf16_to_f32(po.pp(acc_ref, po.PP_BIAS | po.PP_GELU, po.BF16, bias=w["bias"])).astype(np.float64)
        got = C[:rows].float().cpu().numpy().astype(np.float64)
        ulp = np.exp2(np.floor(np.log2(np.maximum(np.abs(want), 2.0 ** -126))) - 7)
        within = np.abs(got - want) <= ulp
        well = (acc_ref + w["bias"][None, :]) > -3.5
        out["config"]["parity"] = {
            "against": f"CPU oracle, rows 0..{rows - 1} of the timed output ({rows * N} elements)",
            "rel_frobenius": float(f"{np.linalg.norm(got - want) / np.linalg.norm(want):.3e}"),
            "within_1_bf16_ulp_all": round(float(within.mean()), 6),
            "within_1_bf16_ulp_preact_above_-3.5": round(float(within[well].mean()), 6),
            "bar": "rel_frobenius <= 1e-3 and 99.9 % within 1 bf16 ulp where GELU is well conditioned; below -3.5 one fp32 ulp of "
                   "summation order moves the reference polynomial by more than a bf16 ulp (tests/test_oracle_math.py shows the "
                   "reference's arithmetic against an fp64 sum short of 99.9 % over all elements as well)"}
        reps, el = time_cpu(run_ref, args.cpu_seconds)
        out["cpu_baseline"] = {
            "value": round(flops * reps / el / 1e12, 4), "unit": "TFLOP/s", "cores": cores, "kind": "port",
            "sample": f"{reps} x the full workload (M=1024,K=4096,N=11008 + BIAS_GELU) in {el:.1f} s; portable "
                      f"{isa} restatement of the AMX summation order (the host {amx} AMX; the AMX intrinsics path is not used)",
        }
        r2, e2 = onednn_bf16(w["A"], w["B"], args.cpu_seconds / 3)
        out["cpu_baseline"]["onednn"] = {"value": round(flops * r2 / e2 / 1e12, 4), "unit": "TFLOP/s", "cores": cores,
                                         "sample": f"{r2} x torch.matmul (bf16, CPU, no post-op) of the same shape in {e2:.1f} s"}
        b3 = args.cpu_seconds / 3

        # config 1: bf16 256^3
        w1c = wl.gemm_bf16_256()
        reps, el = time_cpu(lambda: po.gemm_bf16(w1c["A"], w1c["B"], nthreads=cores), min(b3, 1.0))
        r2, e2 = onednn_bf16(w1c["A"], w1c["B"], min(b3, 1.0))
        cpu_other["bf16_gemm_256x256x256"] = {
            "port": {"value": round(2.0 * 256 ** 3 * reps / el / 1e12, 4), "unit": "TFLOP/s", "cores": cores, "sample": f"{reps} x in {el:.2f} s"},
            "onednn": {"value": round(2.0 * 256 ** 3 * r2 / e2 / 1e12, 4), "unit": "TFLOP/s", "cores": cores, "sample": f"{r2} x torch.matmul in {e2:.2f} s"}}

        # config 3: int8 FC with requant
        wic = wl.int8_fc()
        opsi = 2.0 * wic["M"] * wic["K"] * wic["N"]

        def run_i8():
            acc = po.gemm_i8(wic["A"], wic["B"])
            po.pp(acc, po.PP_DEQUANT | po.PP_BIAS | po.PP_QUANT, po.I8, bias=wic["bias"], deq_per_oc=wic["deq"], q=float(wic["q"]))
        reps, el = time_cpu(run_i8, b3)

        def onednn_i8():
            Ai, Bi = torch.from_numpy(wic["A"]), torch.from_numpy(wic["B"])
            r, e = time_cpu(lambda: torch._int_mm(Ai, Bi), b3)
            return {"value": round(opsi * r / e / 1e12, 4), "unit": "TOP/s", "cores": cores, "sample": f"{r} x torch._int_mm (CPU, no post-op) in {e:.1f} s"}
        cpu_other["int8_fc_requant_M512_K4096_N4096"] = {
            "port": {"value": round(opsi * reps / el / 1e12, 4), "unit": "TOP/s", "cores": cores, "sample": f"{reps} x the full workload in {el:.1f} s"},
            "onednn": gpu_note(onednn_i8)}

        # config 4: decode GEMV over int8 weights, M=1, rotating over 8 weight copies (360 MB: nothing stays in a cache).
        # The port is the reference's own form (weight_compression/fc16m.cpp:451-502, 620-663): weights packed once in
        # repackB_1xL order, then every call streams the int8 bytes and converts them in registers, N split over the threads
        wgc = wl.decode_gemv_w8(M=1)
        packed0 = po.pack_1x2_s8(wgc["W"])
        Wcopies = [packed0.copy() for _ in range(8)]
        turn = [0]

        def run_gemv():
            po.gemv_w8_stream(wgc["x"], Wcopies[turn[0] % 8], wgc["scale"], wgc["N"], nthreads=cores)
            turn[0] += 1
        reps, el = time_cpu(run_gemv, b3)
        wbytes = float(wgc["K"]) * wgc["N"]
        Wcopies = [wgc["W"].copy() for _ in range(8)]

        def onednn_gemv():
            xt = torch.from_numpy(wgc["x"].view(np.int16).copy()).view(torch.bfloat16)
            Wt = [torch.from_numpy(Wc).to(torch.bfloat16) for Wc in Wcopies]   # oneDNN has no mixed bf16 x int8 matmul: bf16 weights
            t2 = [0]

            def f():
                torch.matmul(xt, Wt[t2[0] % 8])
                t2[0] += 1
            r, e = time_cpu(f, b3)
            return {"value": round(2 * wbytes * r / e / 1e9, 2), "unit": "GB/s", "cores": cores,
                    "sample": f"{r} x torch.matmul(x bf16 [1,4096], W bf16 [4096,11008]) over 8 rotated copies in {e:.1f} s (bf16 weights: 2 bytes each)"}
        cpu_other["decode_gemv_int8w_K4096_N11008_M1"] = {
            "port": {"value": round(wbytes * reps / el / 1e9, 2), "unit": "GB/s", "cores": cores,
                     "sample": f"{reps} x the full GEMV over 8 rotated copies of the packed int8 weights in {el:.1f} s (weights streamed once "
                               "and converted in registers, as matmul16m_Wint8B does)"},
            "onednn": gpu_note(onednn_gemv)}
        del Wcopies

        # config 5: fused MLP at M=1 and M=2048
        wmc = wl.llama_mlp(M=2048)
        for Mm in (1, 2048):
            xs = np.ascontiguousarray(wmc["x"][:Mm])
            reps, el = time_cpu(lambda: po.mlp(xs, wmc["w_gate"], wmc["w_up"], wmc["w_down"], split_k=True), b3)
            fl = 6.0 * Mm * wmc["K"] * wmc["N"]
            ent = {"port": {"value": round(fl * reps / el / 1e12, 4), "unit": "TFLOP/s", "cores": cores, "sample": f"{reps} x the full MLP in {el:.1f} s",
                            "weight_GBps": round(6.0 * wmc["K"] * wmc["N"] * reps / el / 1e9, 1)}}

            def onednn_mlp():
                xt = torch.from_numpy(xs.view(np.int16).copy()).view(torch.bfloat16)
                g, u, d = (torch.from_numpy(wmc[k].view(np.int16).copy()).view(torch.bfloat16) for k in ("w_gate", "w_up", "w_down"))
                F = torch.nn.functional

                def f():
                    F.linear(F.silu(F.linear(xt, g)) * F.linear(xt, u), d)
                r, e = time_cpu(f, b3)
                return {"value": round(fl * r / e / 1e12, 4), "unit": "TFLOP/s", "cores": cores, "sample": f"{r} x torch (three F.linear + silu, bf16, CPU) in {e:.1f} s"}
            ent["onednn"] = gpu_note(onednn_mlp)
            cpu_other[f"llama7b_mlp_fused_M{Mm}"] = ent
        del wmc

    # ---- the other configurations of the path --------------------------------------------------------
    if not args.no_extra:
        extra = {}

        def avg_ms(Ain, packs, Nn, epi, iters, **kw):
            # a new shape needs about a hundred launches before its time settles (fresh buffers, clocks)
            mx.time_gemm(Ain, packs, Nn, epi, max(100, iters // 2), **kw)
            return mx.time_gemm(Ain, packs, Nn, epi, iters, **kw)

        def med_us(Ain, packs, Nn, epi, **kw):
            # median of eleven means over as many launches as there are weight copies (at least ten)
            n = max(10, len(packs))
            return round(sorted(mx.time_gemm(Ain, packs, Nn, epi, n, **kw) for _ in range(11))[5] * 1e3, 2)

        progress("bf16_gemm_256x256x256")
        # bf16 256^3, fp32 out, no post-op (launch-latency bound; reported, not a roofline case)
        w1 = wl.gemm_bf16_256()
        A1, B1 = dev_bf16(w1["A"]), mx.repack_b(dev_bf16(w1["B"]))
        C1 = torch.zeros((256, 256), dtype=torch.float32, device="cuda")
        ms = avg_ms(A1, [B1], 256, mx.Epilogue(C1, mx.PP_NONE), 200)
        extra["bf16_gemm_256x256x256"] = {"us": round(ms * 1e3, 2), "tflops": round(2.0 * 256 ** 3 / ms / 1e9, 2),
                                          "kernel": mx.last_kernel()}

        progress("bf16_fc_bias_gelu_sweep_M")
        # bf16 FC sweep over M
        sweep = {}
        for Ms in (128, 512, 2048):
            ws = wl.ffn_up_bias_gelu(M=Ms)
            As = dev_bf16(ws["A"])
            Cs = torch.zeros((Ms, N), dtype=torch.bfloat16, device="cuda")
            ms = avg_ms(As, [Bp], N, mx.Epilogue(Cs, mx.PP_BIAS | mx.PP_GELU, bias=bias), 100)
            sweep[str(Ms)] = {"us": round(ms * 1e3, 1), "median_us": med_us(As, [Bp], N, mx.Epilogue(Cs, mx.PP_BIAS | mx.PP_GELU, bias=bias)),
                              "tflops": round(2.0 * Ms * N * K / ms / 1e9, 1),
                              "frac_of_bf16_peak": round(2.0 * Ms * N * K / ms / 1e9 / PEAK_BF16_TFLOPS, 4), "kernel": mx.last_kernel()}
            del As, Cs
        extra["bf16_fc_bias_gelu_sweep_M"] = sweep

        progress("bf16_fc_bias_gelu_M1024_two_streams")
        # The headline FC launched alternately on two streams (independent requests, separate outputs): a launch of
        # 232 workgroups leaves 24 CUs idle and successive launches on one stream are ~5 us apart; two streams let the
        # next launch start on the idle CUs.  Throughput only - a launch on its own is not faster this way.
        s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
        C2 = torch.zeros_like(C)
        ep_2 = mx.Epilogue(C2, mx.PP_BIAS | mx.PP_GELU, bias=bias)

        def pair():
            with torch.cuda.stream(s1):
                mx.gemm(A, Bp, N, ep)
            with torch.cuda.stream(s2):
                mx.gemm(A, Bp, N, ep_2)
        torch.cuda.synchronize()
        for _ in range(50):
            pair()
        torch.cuda.synchronize()
        tp0 = time.perf_counter()
        for _ in range(100):
            pair()
        torch.cuda.synchronize()
        us2 = (time.perf_counter() - tp0) * 1e6 / 200
        extra["bf16_fc_bias_gelu_M1024_two_streams"] = {"us_per_launch": round(us2, 2), "tflops": round(flops / us2 / 1e6, 1),
                                                        "frac_of_bf16_peak": round(flops / us2 / 1e6 / PEAK_BF16_TFLOPS, 4)}
        del C2

        progress("int8_fc_requant_M512_K4096_N4096")
        # int8 FC with dequant/bias/requant
        wi = wl.int8_fc()
        Ai, Bi = dev(wi["A"]), mx.repack_b(dev(wi["B"]))
        Ci = torch.zeros((wi["M"], wi["N"]), dtype=torch.int8, device="cuda")
        epi = mx.Epilogue(Ci, mx.PP_DEQUANT | mx.PP_BIAS | mx.PP_QUANT, bias=dev(wi["bias"]),
                          deq_scale_per_oc=dev(wi["deq"]), q_scale=float(wi["q"]))
        ms = avg_ms(Ai, [Bi], wi["N"], epi, 100)
        ops = 2.0 * wi["M"] * wi["K"] * wi["N"]
        extra["int8_fc_requant_M512_K4096_N4096"] = {
            "us": round(ms * 1e3, 2), "median_us": med_us(Ai, [Bi], wi["N"], epi), "tops": round(ops / ms / 1e9, 1),
            "frac_of_int8_peak": round(ops / ms / 1e9 / PEAK_INT8_TOPS, 4), "kernel": mx.last_kernel()}
        # the same launch with the rows of A 128 bytes further apart (a row stride that is a multiple of 4 KiB puts the 8 rows
        # of a load instruction into one L2 channel; the C++ tensor2D pads such rows, this configuration's layout is compact)
        Apad = torch.zeros((wi["M"], wi["K"] + 128), dtype=torch.int8, device="cuda")
        Apad[:, :wi["K"]] = Ai
        msp = avg_ms(Apad[:, :wi["K"]], [Bi], wi["N"], epi, 100)
        extra["int8_fc_requant_M512_K4096_N4096"]["a_rows_padded_by_128B"] = {"us": round(msp * 1e3, 2), "tops": round(ops / msp / 1e9, 1)}
        del Ai, Bi, Ci, Apad
        # the same int8 kernel on a shape large enough to fill the machine (the Llama-7B FFN shape at M=2048)
        rng = np.random.default_rng(11)
        Mi, Ki, Ni = 2048, 4096, 11008
        Ai = torch.from_numpy(rng.integers(-127, 128, (Mi, Ki), dtype=np.int8)).cuda()
        Bi = mx.repack_b(torch.from_numpy(rng.integers(-127, 128, (Ki, Ni), dtype=np.int8)).cuda())
        Ci = torch.zeros((Mi, Ni), dtype=torch.int8, device="cuda")
        epi = mx.Epilogue(Ci, mx.PP_DEQUANT | mx.PP_BIAS | mx.PP_QUANT, bias=torch.zeros(Ni, dtype=torch.float32, device="cuda"),
                          deq_scale_per_oc=torch.full((Ni,), 1e-4, dtype=torch.float32, device="cuda"), q_scale=20.0)
        ms = avg_ms(Ai, [Bi], Ni, epi, 100)
        ops = 2.0 * Mi * Ki * Ni
        extra["int8_fc_requant_M2048_K4096_N11008"] = {
            "us": round(ms * 1e3, 2), "tops": round(ops / ms / 1e9, 1), "frac_of_int8_peak": round(ops / ms / 1e9 / PEAK_INT8_TOPS, 4),
            "kernel": mx.last_kernel()}
        del Ai, Bi, Ci

        progress("decode_gemv_int8w_K4096_N11008")
        # decode GEMV over int8 weights, rotating over 12 weight copies (540 MB > 256 MB of cache)
        gemv = {}
        for Mg in (1, 4, 16):
            wg = wl.decode_gemv_w8(M=Mg)
            xg, Wg, sg = dev_bf16(wg["x"]), mx.repack_b(dev(wg["W"])), dev(wg["scale"])
            packs = [Wg] + [Wg.clone() for _ in range(11)]
            yg = torch.zeros((Mg, wg["N"]), dtype=torch.bfloat16, device="cuda")
            epg = mx.Epilogue(yg, mx.PP_DEQUANT, deq_scale_per_oc=sg)
            ms = avg_ms(xg, packs, wg["N"], epg, 240, b_dtype=mx.I8)
            wbytes = float(wg["K"]) * wg["N"]
            gemv[str(Mg)] = {"us": round(ms * 1e3, 2), "median_us": med_us(xg, packs, wg["N"], epg, b_dtype=mx.I8),
                             "weight_GBps": round(wbytes / ms / 1e6, 0),
                             "frac_of_hbm_peak": round(wbytes / ms / 1e6 / PEAK_HBM_GBS, 4), "kernel": mx.last_kernel(),
                             "traffic": measured_traffic(mx.last_kernel()) if Mg in (1, 16) else None, "algorithmic_bytes": wbytes}
            if Mg == 1:
                # the same launch in its other form (matrix cores <-> v_dot2_f32_bf16 per lane), for the record
                auto_valu = "valu" in mx.last_kernel()
                mx.set_option("decode_valu", 0 if auto_valu else 1)
                try:
                    ms2 = avg_ms(xg, packs, wg["N"], epg, 240, b_dtype=mx.I8)
                    gemv["1"]["other_form"] = {"us": round(ms2 * 1e3, 2), "kernel": mx.last_kernel()}
                finally:
                    mx.set_option("decode_valu", -1)
            del packs, Wg
        extra["decode_gemv_int8w_K4096_N11008"] = gemv

        progress("decode_gemv_int8w_K4096_M1_sweep_N")
        # The same GEMV (M=1) over the number of output columns, in each of its forms: per-launch cost and rate, and
        # what the balance of 32-column panels over 256 CUs is worth (N = 8192 and 16384 are exactly 1 and 2 panels per CU)
        sweepn = {}
        xg1 = torch.randn((1, 4096), dtype=torch.float32, device="cuda").to(torch.bfloat16)
        for Nn in (4096, 8192, 11008, 16384, 32768):
            ncopy = max(2, int(540e6 // (4096 * Nn)))
            Wn = mx.repack_b(torch.randint(-127, 128, (4096, Nn), dtype=torch.int8, device="cuda"))
            packs = [Wn] + [Wn.clone() for _ in range(ncopy - 1)]
            yn = torch.zeros((1, Nn), dtype=torch.bfloat16, device="cuda")
            epn = mx.Epilogue(yn, mx.PP_DEQUANT, deq_scale=1e-3)
            ent = {}
            for form, (valu, halves, resident) in (("mfma", (0, 0, 0)), ("valu", (1, 0, 0)), ("half_panels", (0, 1, 0)),
                                                   ("resident_x", (-1, -1, 1)), ("auto", (-1, -1, -1))):
                mx.set_option("decode_valu", valu)
                mx.set_option("decode_halves", halves)
                mx.set_option("decode_resident", resident)
                try:
                    msn = avg_ms(xg1, packs, Nn, epn, 200, b_dtype=mx.I8)
                    ent[form] = {"us": round(msn * 1e3, 2), "kernel": mx.last_kernel()}
                finally:
                    mx.set_option("decode_valu", -1)
                    mx.set_option("decode_halves", -1)
                    mx.set_option("decode_resident", -1)
            ent["panels_per_cu"] = round(Nn / 32 / 256, 2)
            ent["auto_weight_GBps"] = round(4096.0 * Nn / ent["auto"]["us"] / 1e3, 0)
            sweepn[str(Nn)] = ent
            del packs, Wn
        extra["decode_gemv_int8w_K4096_M1_sweep_N"] = sweepn

        progress("decode_k_split")
        # Decode shapes with a panel for at most every second CU: the chunked kernel whole (k_splits = 1) and with K cut
        # into slices over several workgroups (k_splits = 0 with a workspace), weights rotated over 540 MB
        ksp = {}
        for w8k, Mk, Kk, Nk in ((True, 16, 11008, 4096), (True, 32, 11008, 4096), (True, 32, 8192, 1024),
                                (False, 16, 11008, 4096), (False, 32, 11008, 4096), (False, 32, 8192, 1024)):
            nbk = Kk * Nk * (1 if w8k else 2)
            if w8k:
                Wk = mx.repack_b(torch.randint(-127, 128, (Kk, Nk), dtype=torch.int8, device="cuda"))
            else:
                Wk = mx.repack_b((torch.randn((Kk, Nk), dtype=torch.float32, device="cuda") * 0.02).to(torch.bfloat16))
            packs = [Wk] + [Wk.clone() for _ in range(max(2, int(540e6 // nbk)) - 1)]
            xk = torch.randn((Mk, Kk), dtype=torch.float32, device="cuda").to(torch.bfloat16)
            epk = mx.Epilogue(torch.zeros((Mk, Nk), dtype=torch.bfloat16, device="cuda"), mx.PP_NONE)
            kwk = {"b_dtype": mx.I8} if w8k else {}
            entk = {}
            for label, ks in (("whole", 1), ("split", 0)):
                msk = avg_ms(xk, packs, Nk, epk, 200, k_splits=ks, **kwk)
                entk[label] = {"us": round(msk * 1e3, 2), "kernel": mx.last_kernel(), "weight_GBps": round(nbk / msk / 1e6, 0)}
            ksp[f"{'int8w' if w8k else 'bf16'}_M{Mk}_K{Kk}_N{Nk}"] = entk
            del packs, Wk
        extra["decode_k_split"] = ksp

        progress("decode_chain_int8w_24_layers_K4096_N11008")
        # Steady state of a chain of decode layers (the topology of main.cpp:660-711: A1 x B1 -> A2, A2 x B2 -> A1, ...,
        # one set of weights per layer): 12 pairs of [1,4096] x [4096,11008] and [1,11008] x [11008,4096] over int8
        # weights (1.08 GB, nothing repeats within the cache), every layer reading the previous layer's output,
        # replayed from a HIP graph so that no host time is in the figure
        Kc, Nc, pairs = 4096, 11008, 12
        rngc = torch.Generator(device="cuda").manual_seed(5)
        W1 = [mx.repack_b(torch.randint(-127, 128, (Kc, Nc), dtype=torch.int8, device="cuda", generator=rngc)) for _ in range(pairs)]
        W2 = [mx.repack_b(torch.randint(-127, 128, (Nc, Kc), dtype=torch.int8, device="cuda", generator=rngc)) for _ in range(pairs)]
        xa = torch.randn((1, Kc), dtype=torch.float32, device="cuda").to(torch.bfloat16)
        hb = torch.zeros((1, Nc), dtype=torch.bfloat16, device="cuda")
        ep1, ep2 = mx.Epilogue(hb, mx.PP_DEQUANT, deq_scale=2e-4), mx.Epilogue(xa, mx.PP_DEQUANT, deq_scale=2e-4)

        def chain():
            for i in range(pairs):
                mx.gemm(xa, W1[i], Nc, ep1, b_dtype=mx.I8)
                mx.gemm(hb, W2[i], Kc, ep2, b_dtype=mx.I8)
        cstream = torch.cuda.Stream()
        with torch.cuda.stream(cstream):
            chain()
            torch.cuda.synchronize()
            gr = torch.cuda.CUDAGraph()
            with torch.cuda.graph(gr, stream=cstream):
                chain()
        torch.cuda.synchronize()
        reps = []
        for _ in range(12):
            a0, a1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a0.record()
            gr.replay()
            a1.record()
            torch.cuda.synchronize()
            reps.append(a0.elapsed_time(a1) * 1e3 / (2 * pairs))
        reps = sorted(reps[2:])
        us = reps[len(reps) // 2]
        extra["decode_chain_int8w_24_layers_K4096_N11008"] = {
            "us_per_layer": round(us, 2), "weight_GBps": round(float(Kc) * Nc / us / 1e3, 0),
            "frac_of_hbm_peak": round(float(Kc) * Nc / us / 1e3 / PEAK_HBM_GBS, 4), "layers": 2 * pairs,
            "note": "graph replay, M=1, each layer reads the previous layer's output; median of 10 replays"}
        del gr, W1, W2

        progress("decode_gemv_int8x_int8w_K4096_N11008")
        # int8 activations x int8 weights at M=1 (int32 sums), same weights and rotation
        w8b = wl.decode_gemv_w8(M=1)
        Wi = mx.repack_b(dev(w8b["W"]))
        packs = [Wi] + [Wi.clone() for _ in range(11)]
        xi = torch.randint(-127, 128, (1, w8b["K"]), dtype=torch.int8, device="cuda")
        yi = torch.zeros((1, w8b["N"]), dtype=torch.bfloat16, device="cuda")
        ms = avg_ms(xi, packs, w8b["N"], mx.Epilogue(yi, mx.PP_DEQUANT, deq_scale_per_oc=dev(w8b["scale"])), 240)
        extra["decode_gemv_int8x_int8w_K4096_N11008"] = {"1": {
            "us": round(ms * 1e3, 2), "weight_GBps": round(float(w8b["K"]) * w8b["N"] / ms / 1e6, 0),
            "frac_of_hbm_peak": round(float(w8b["K"]) * w8b["N"] / ms / 1e6 / PEAK_HBM_GBS, 4), "kernel": mx.last_kernel()}}
        del packs, Wi

        progress("decode_gemv_int4w_K4096_N11008")
        # the same GEMV over int4-compressed weights (22.5 MB), rotating over 24 copies (541 MB)
        gemv4 = {}
        wg = wl.decode_gemv_w8(M=4)
        W4 = torch.randn((wg["K"], wg["N"]), dtype=torch.float32, device="cuda").mul_(0.02).to(torch.bfloat16)
        P4, s4 = mx.quantize_pack_int4(W4)
        packs = [P4] + [P4.clone() for _ in range(23)]
        for Mg in (1, 4):
            xg = dev_bf16(wg["x"][:Mg])
            yg = torch.zeros((Mg, wg["N"]), dtype=torch.bfloat16, device="cuda")
            epg = mx.Epilogue(yg, mx.PP_DEQUANT, deq_scale_per_oc=s4)
            ms = avg_ms(xg, packs, wg["N"], epg, 240, b_dtype=mx.I4)
            wbytes = float(wg["K"]) * wg["N"] / 2
            gemv4[str(Mg)] = {"us": round(ms * 1e3, 2), "weight_GBps": round(wbytes / ms / 1e6, 0),
                              "frac_of_hbm_peak": round(wbytes / ms / 1e6 / PEAK_HBM_GBS, 4), "kernel": mx.last_kernel()}
        del packs, P4, W4
        extra["decode_gemv_int4w_K4096_N11008"] = gemv4

        progress("bf16_x_int8w_gemm_M896_K2560_N10240")
        # bf16 activations on int8-compressed weights at large M: the shape the reference publishes its
        # weight-compressed figure on (perf.log:36: M=896, K=2560, N=10240); the int8 fragments are converted on the fly
        Mw, Kw, Nw = 896, 2560, 10240
        Aw = torch.randn((Mw, Kw), dtype=torch.float32, device="cuda").to(torch.bfloat16)
        Ww = mx.repack_b(torch.randint(-127, 128, (Kw, Nw), dtype=torch.int8, device="cuda"))
        Cw = torch.zeros((Mw, Nw), dtype=torch.float32, device="cuda")
        epw = mx.Epilogue(Cw, mx.PP_DEQUANT, deq_scale=0.01)
        ms = avg_ms(Aw, [Ww], Nw, epw, 100, b_dtype=mx.I8)
        extra["bf16_x_int8w_gemm_M896_K2560_N10240"] = {
            "us": round(ms * 1e3, 2), "tflops": round(2.0 * Mw * Kw * Nw / ms / 1e9, 1),
            "frac_of_bf16_peak": round(2.0 * Mw * Kw * Nw / ms / 1e9 / PEAK_BF16_TFLOPS, 4), "kernel": mx.last_kernel(),
            "weight_bytes_resident": int(Ww.numel())}
        del Aw, Ww, Cw

        progress("bf16_down_proj_K11008_N4096_ksplit")
        # shapes with few output tiles, where K is split over several workgroups per tile (the MLP's down
        # projection at prefill sizes below a full machine): with and without the split
        ksp = {}
        Wdn = mx.repack_b((torch.randn((11008, 4096), dtype=torch.float32, device="cuda") * 0.02).to(torch.bfloat16))
        for Ms in (64, 256):
            hs = torch.randn((Ms, 11008), dtype=torch.float32, device="cuda").to(torch.bfloat16)
            ys = torch.zeros((Ms, 4096), dtype=torch.bfloat16, device="cuda")
            eps = mx.Epilogue(ys, mx.PP_NONE)
            t_split = avg_ms(hs, [Wdn], 4096, eps, 100)
            k_split = mx.last_kernel()
            t_plain = avg_ms(hs, [Wdn], 4096, eps, 100, k_splits=1)
            ksp[str(Ms)] = {"us": round(t_split * 1e3, 2), "kernel": k_split, "us_without_split": round(t_plain * 1e3, 2),
                            "kernel_without_split": mx.last_kernel(), "tflops": round(2.0 * Ms * 11008 * 4096 / t_split / 1e9, 1)}
        extra["bf16_down_proj_K11008_N4096_ksplit"] = ksp
        del Wdn

        progress("llama7b_mlp_fused")
        # fused Llama-7B MLP
        mlp = {}
        wm = wl.llama_mlp(M=2048)
        op = mx.MLP()
        op.setup(dev_bf16(wm["w_gate"]), dev_bf16(wm["w_up"]), dev_bf16(wm["w_down"]))
        for Mm in (1, 2048):
            xm = dev_bf16(wm["x"][:Mm])
            ym = torch.zeros((Mm, wm["K"]), dtype=torch.bfloat16, device="cuda")
            for _ in range(60):
                op.run(xm, ym)
            torch.cuda.synchronize()
            a0, a1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a0.record()
            for _ in range(60):
                op.run(xm, ym)
            a1.record()
            torch.cuda.synchronize()
            ms = a0.elapsed_time(a1) / 60
            fl = 6.0 * Mm * wm["K"] * wm["N"]
            mlp[str(Mm)] = {"us": round(ms * 1e3, 1), "tflops": round(fl / ms / 1e9, 1),
                            "weight_GBps": round(3.0 * wm["K"] * wm["N"] * 2 / ms / 1e6, 0)}
        extra["llama7b_mlp_fused"] = mlp

        progress("llama7b_mlp_stages")
        # the MLP's two GEMMs on their own, with their roofline fractions; at M=1 the weights are rotated
        # (3 copies of gate/up = 541 MB, 6 of down) so that nothing is served from the 256 MB cache
        from mm_amx_amd import _lib as L
        stages = {}
        Km, Nm = wm["K"], wm["N"]
        gu = [L.repack_gate_up(dev_bf16(wm["w_gate"]), dev_bf16(wm["w_up"])) for _ in range(3)]
        dn = [L.repack_b(dev_bf16(wm["w_down"]), transpose=True) for _ in range(6)]
        for Mm in (1, 2048):
            xm = dev_bf16(wm["x"][:Mm])
            hm = torch.zeros((Mm, Nm), dtype=torch.bfloat16, device="cuda")
            ym = torch.zeros((Mm, Km), dtype=torch.bfloat16, device="cuda")
            t1 = avg_ms(xm, gu, 2 * Nm, mx.Epilogue(hm, mx.PP_SILU_GATE), 120)
            k1 = mx.last_kernel()
            t2 = avg_ms(hm, dn, Km, mx.Epilogue(ym, mx.PP_NONE), 120)
            k2 = mx.last_kernel()
            if Mm == 1:
                stages[str(Mm)] = {
                    "gate_up": {"us": round(t1 * 1e3, 1), "frac_of_hbm_peak": round(4.0 * Km * Nm / t1 / 1e6 / PEAK_HBM_GBS, 4), "kernel": k1},
                    "down": {"us": round(t2 * 1e3, 1), "frac_of_hbm_peak": round(2.0 * Km * Nm / t2 / 1e6 / PEAK_HBM_GBS, 4), "kernel": k2}}
            else:
                stages[str(Mm)] = {
                    "gate_up": {"us": round(t1 * 1e3, 1), "frac_of_bf16_peak": round(4.0 * Mm * Km * Nm / t1 / 1e9 / PEAK_BF16_TFLOPS, 4), "kernel": k1},
                    "down": {"us": round(t2 * 1e3, 1), "frac_of_bf16_peak": round(2.0 * Mm * Km * Nm / t2 / 1e9 / PEAK_BF16_TFLOPS, 4), "kernel": k2}}
        del gu, dn
        extra["llama7b_mlp_stages"] = stages

        progress("llama7b_mlp_stack_32_layers")
        # The reference's end-to-end demo at its size (torch-ext/test.py:176-218): a stack of 32 Llama-7B MLPs (RMSNorm +
        # fused MLP, every layer its own 270 MB of weights: 8.7 GB packed + the same again for torch's layers), per-layer
        # time through torch's bf16 linear layers and through this library; at M=1 also replayed from a HIP graph,
        # which shows what the Python/ctypes host layer costs per layer
        del op
        from mm_amx_amd import mlp_llama
        demo = {}
        for Md, rounds in ((256, 10), (1, 20)):
            r = mlp_llama.perf_llama7b_MLP(M=Md, num_layers=32, rounds=rounds, verbose=False, graph=True)
            demo[str(Md)] = {k: ({kk: (round(vv, 1) if isinstance(vv, float) else vv) for kk, vv in v.items()} if isinstance(v, dict)
                                 else float(f"{v:.3e}")) for k, v in r.items()}
            host = r["mm_amx_amd"]["per_layer_us"] - r["mm_amx_amd_graph"]["per_layer_us"]
            demo[str(Md)]["host_side_us_per_layer"] = round(host, 1)
            demo[str(Md)]["host_side_share"] = round(host / r["mm_amx_amd"]["per_layer_us"], 3)
            torch.cuda.empty_cache()
        extra["llama7b_mlp_stack_32_layers"] = demo

        progress("qk_matvec_bf16_T2097152_D128")
        # q against a cache of keys (the mat-vec of test_qk.cpp): 2^21 tokens x head size 128, bf16, 537 MB
        # (more than the 256 MB last-level cache holds)
        T, D = 1 << 21, 128
        keys = torch.randn((T, D), dtype=torch.float32, device="cuda").to(torch.bfloat16)
        q = torch.randn((D,), dtype=torch.float32, device="cuda").to(torch.bfloat16)
        sc = torch.empty(T, dtype=torch.float32, device="cuda")
        mv = mx.MatmulVector()
        for _ in range(20):
            mv(keys, q, sc)
        torch.cuda.synchronize()
        a0, a1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a0.record()
        for _ in range(20):
            mv(keys, q, sc)
        a1.record()
        torch.cuda.synchronize()
        ms = a0.elapsed_time(a1) / 20
        extra["qk_matvec_bf16_T2097152_D128"] = {"us": round(ms * 1e3, 1), "GBps": round(T * D * 2 / ms / 1e6, 0),
                                                 "frac_of_hbm_peak": round(T * D * 2 / ms / 1e6 / PEAK_HBM_GBS, 4)}
        del keys, sc

        progress("streaming_read_floor")
        # What a kernel that only streams the same number of bytes takes, launch after launch, replayed from a HIP graph
        # so that no host time is in the figure, buffers rotated over 541 MB+ (more than the last-level cache holds).
        # The decode kernels are judged against the best of these:
        #   matvec:      the mat-vec kernel over key caches of the size of the decode weights (many short workgroups)
        #   persistent:  a resident grid of 256 / 512 workgroups, each wave a rolling window of 8 / 16 / 32 KiB of loads, and
        #                the two best grids of a wider sweep (688 x 4 waves and 344 x 8 waves, 2 KiB per wave)
        #   device_copy: the runtime's own device-to-device copy of as many bytes (reads AND writes them)
        def graph_us(launch, nl):
            for i in range(nl):
                launch(i)
            torch.cuda.synchronize()
            gr, side = torch.cuda.CUDAGraph(), torch.cuda.Stream()
            with torch.cuda.stream(side):
                with torch.cuda.graph(gr, stream=side):
                    for i in range(nl):
                        launch(i)
            torch.cuda.synchronize()
            gr.replay()
            torch.cuda.synchronize()
            ts = []
            for _ in range(5):
                a0, a1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a0.record()
                gr.replay()
                a1.record()
                torch.cuda.synchronize()
                ts.append(a0.elapsed_time(a1) / nl * 1e3)
            del gr
            return sorted(ts)[2]

        floor = {}
        sink = torch.zeros(1, dtype=torch.int32, device="cuda")
        for label, mult in (("45MB", 1), ("90MB", 2), ("180MB", 4)):
            Tf = 176128 * mult
            nbytes = Tf * D * 2                      # 45 088 768 bytes = 4096 x 11008 = 5504 x 8 KiB
            ncopy = 12 // mult
            ks = [torch.randn((Tf, D), dtype=torch.float32, device="cuda").to(torch.bfloat16) for _ in range(ncopy)]
            flat = [k.view(torch.uint8).view(-1) for k in ks]
            scf = torch.empty(Tf, dtype=torch.float32, device="cuda")
            ent = {}
            us = graph_us(lambda i: mv(ks[i % ncopy], q, scf), ncopy * 10)
            ent["matvec"] = {"us": round(us, 2), "GBps": round(nbytes / us / 1e3)}
            for grid in (256, 512):
                # equal shares of whole 8 KiB per workgroup: the figure is over the bytes actually read
                share = nbytes // grid // 8192 * 8192
                for kib in (8, 16, 32):
                    us = graph_us(lambda i: mx.probe_read(flat[i % ncopy][:share * grid], grid, kib, sink), ncopy * 10)
                    ent[f"persistent_{grid}wg_{kib}KiB"] = {"us": round(us, 2), "bytes": share * grid, "GBps": round(share * grid / us / 1e3),
                                                            "us_scaled_to_all_bytes": round(us * nbytes / (share * grid), 2)}
            # the best grids of a sweep over workgroups x waves x bytes in flight: many small workgroups, little in flight each
            for grid, waves, kib in ((688, 4, 2), (344, 8, 2)):
                unit = waves * kib * 1024
                share = nbytes // grid // unit * unit
                us = graph_us(lambda i: mx.probe_read(flat[i % ncopy][:share * grid], grid, kib, sink, waves=waves), ncopy * 10)
                ent[f"persistent_{grid}wg_{waves}waves_{kib}KiB"] = {"us": round(us, 2), "bytes": share * grid, "GBps": round(share * grid / us / 1e3),
                                                                    "us_scaled_to_all_bytes": round(us * nbytes / (share * grid), 2)}
            dst = torch.empty_like(flat[0])
            us = graph_us(lambda i: dst.copy_(flat[i % ncopy]), ncopy * 10)
            ent["device_copy"] = {"us": round(us, 2), "GBps_read_plus_written": round(2 * nbytes / us / 1e3)}
            best = min(v.get("us_scaled_to_all_bytes", v["us"]) for k, v in ent.items() if k != "device_copy")
            ent["best_read_only_us"] = best
            floor[label] = ent
            del ks, flat, scf, dst
        extra["streaming_read_floor"] = floor

        progress("torch_hipblaslt_same_shapes")
        # The vendor library on the same shapes, same box (torch.matmul / torch._int_mm -> hipBLASLt; the bare product,
        # no bias, no GELU, no requantisation), for context only
        vend = {}

        def t_us(fn, iters=100):
            for _ in range(30):
                fn()
            torch.cuda.synchronize()
            a0, a1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a0.record()
            for _ in range(iters):
                fn()
            a1.record()
            torch.cuda.synchronize()
            return a0.elapsed_time(a1) * 1e3 / iters
        try:
            At = torch.randn((M, K), dtype=torch.float32, device="cuda").to(torch.bfloat16)
            Bt = (torch.randn((K, N), dtype=torch.float32, device="cuda") * 0.02).to(torch.bfloat16)
            us = t_us(lambda: torch.matmul(At, Bt))
            vend["bf16_matmul_M1024_K4096_N11008"] = {"us": round(us, 2), "tflops": round(flops / us / 1e6, 1)}
            Ai8 = torch.randint(-127, 128, (512, 4096), dtype=torch.int8, device="cuda")
            Bi8 = torch.randint(-127, 128, (4096, 4096), dtype=torch.int8, device="cuda")
            us = t_us(lambda: torch._int_mm(Ai8, Bi8))
            vend["int8_int_mm_M512_K4096_N4096"] = {"us": round(us, 2), "tops": round(2.0 * 512 * 4096 * 4096 / us / 1e6, 1)}
            del At, Bt, Ai8, Bi8
        except Exception as e:  # an op this torch build lacks: say so
            vend["note"] = f"{type(e).__name__}: {e}"[:160]
        extra["torch_hipblaslt_same_shapes"] = vend

        progress("mfma_issue_loop")
        # what the matrix pipes deliver with nothing else going on: an issue-bound loop of independent MFMAs,
        # all-zero operands vs operands like the benchmark's (the clock under matrix load depends on the data)
        ceil = {}
        for key, dt, rnd in (("bf16_zero_operands", mx.BF16, 0), ("bf16_gaussian_operands", mx.BF16, 1),
                             ("int8_zero_operands", mx.I8, 0), ("int8_uniform_operands", mx.I8, 1)):
            mx.probe_mfma(dt, rnd, 20000)
            rate, mhz = mx.probe_mfma(dt, rnd, 20000)
            ceil[key] = {"rate": round(rate, 1), "unit": "TFLOP/s" if dt == mx.BF16 else "TOP/s", "shader_mhz": round(mhz)}
        extra["mfma_issue_loop"] = ceil
        if cpu_other:
            extra["cpu_baselines"] = cpu_other
        out["extra"] = extra
    elif cpu_other:
        out["extra"] = {"cpu_baselines": cpu_other}
    # Which CPU figure stands as the baseline of a configuration: the faster of the two.  The port restates the
    # reference's arithmetic (it is the parity oracle: AMX summation order in fp32 / integer FMAs, no VNNI, no bf16 dot
    # products) and is the reference's own algorithm only for the decode GEMV (packed int8 weights streamed and converted in
    # registers); torch's CPU matmul is the oneDNN path the reference compares itself with (benchmark/mmbench/dnnl.cpp).
    def of_record(ent):
        vals = {k: v.get("value") for k, v in ent.items() if isinstance(v, dict) and v.get("value") is not None}
        return max(vals, key=vals.get) if vals else None
    if "cpu_baseline" in out:
        out["cpu_baseline"]["baseline_of_record"] = "onednn" if out["cpu_baseline"]["onednn"]["value"] > out["cpu_baseline"]["value"] else "port"
    for ent in cpu_other.values():
        ent["baseline_of_record"] = of_record(ent)

    print(json.dumps(out))


if __name__ == "__main__":
    main()
