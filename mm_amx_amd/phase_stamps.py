"""Per-workgroup phase timings of the MFMA tile kernels and of the streaming decode kernel, from the instrumented build.

    python -m mm_amx_amd.phase_stamps bf16,1024,4096,11008,256x192,1,8 i8,512,4096,4096,128x64,1 gemv8,1,4096,11008

Each argument is  dtype,M,K,N,tile,k_splits[,waves]  (dtype bf16: the FC with BIAS+GELU and a bf16 store; i8: the int8 FC
with DEQUANT+BIAS+QUANT and an int8 store; w8: bf16 activations on int8-compressed weights, DEQUANT, fp32 store; tile as for
mmx_set_tile, empty = the library's choice; waves 4 or 8), or  gemv8,M,K,N / gemv4,M,K,N  (decode: bf16 activations on
int8 / int4 weights through the streaming kernel, weights rotated over 540 MB).  The instrumented library is built on first use (several
minutes) and whenever a kernel source is newer than it.
The instrumented library (libmm_amx_amd_stamps.so, -DMMX_STAMPS) makes thread 0 of every workgroup write the shader
clock at its phase boundaries behind the K-split workspace; this module launches the shape, reads the stamps back and
prints medians over the workgroups: cycles from start to the first data in LDS, of the main loop, of parking and
combining K slices, of the epilogue, and the clock (cycles per wall-clock tick).  The shipped library has no stamps;
the instrumented one runs the same code plus eight 8-byte stores per workgroup.
"""
import os
import sys

import numpy as np
import torch

import mm_amx_amd as mx
from mm_amx_amd import _lib

# the library is loaded on first use: point the binding at the instrumented build before that
STAMPS_LIB = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libmm_amx_amd_stamps.so")
if "MMX_LIB_PATH" not in os.environ:
    _lib._LIB_PATH = STAMPS_LIB

STAMP_OFFSET = 96 << 20          # the kernels write at workspace partials + 96 MiB + 64 * unit index
COUNTER_BYTES = 16 << 10
STAMP_BYTES = 1 << 20


def run(ws, dt, M, K, N, tile, S, waves=8, out=sys.stdout):
    mx.set_option("waves", waves)
    kw = {}
    if dt == "i8":
        A = torch.randint(-127, 128, (M, K), dtype=torch.int8, device="cuda")
        Bp = mx.repack_b(torch.randint(-127, 128, (K, N), dtype=torch.int8, device="cuda"))
        C = torch.zeros((M, N), dtype=torch.int8, device="cuda")
        ep = mx.Epilogue(C, mx.PP_DEQUANT | mx.PP_BIAS | mx.PP_QUANT, bias=torch.zeros(N, device="cuda"),
                         deq_scale_per_oc=torch.full((N,), 1e-4, device="cuda"), q_scale=20.0)
    elif dt == "w8":
        A = torch.randn((M, K), device="cuda").to(torch.bfloat16)
        Bp = mx.repack_b(torch.randint(-127, 128, (K, N), dtype=torch.int8, device="cuda"))
        C = torch.zeros((M, N), dtype=torch.float32, device="cuda")
        ep = mx.Epilogue(C, mx.PP_DEQUANT, deq_scale=0.01)
        kw = {"b_dtype": mx.I8}
    else:
        A = torch.randn((M, K), device="cuda").to(torch.bfloat16)
        Bp = mx.repack_b((torch.randn((K, N), device="cuda") * 0.02).to(torch.bfloat16))
        C = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")
        ep = mx.Epilogue(C, mx.PP_BIAS | mx.PP_GELU, bias=torch.zeros(N, device="cuda"))
    stamp_off = COUNTER_BYTES + STAMP_OFFSET
    mx.set_tile(tile)
    try:
        mx.time_gemm(A, [Bp], N, ep, 100, k_splits=S, ws=ws, **kw)
        ms = mx.time_gemm(A, [Bp], N, ep, 100, k_splits=S, ws=ws, **kw)
        torch.cuda.synchronize()
        ws[stamp_off:].zero_()
        mx.gemm(A, Bp, N, ep, k_splits=S, ws=ws, **kw)   # one launch: with a K split, which workgroup of a tile arrives last varies
        torch.cuda.synchronize()
        kern = mx.last_kernel()
        S = int(kern.rsplit("ksplit", 1)[1]) if "ksplit" in kern else 1
    finally:
        mx.set_tile("")
        mx.set_option("waves", 8)
    st = ws[stamp_off:].view(torch.int64).cpu().numpy().reshape(-1, 8)
    st = st[st[:, 0] != 0]
    fin = st[st[:, 7] != 0]               # workgroups that ran an epilogue (with a K split: the last to arrive at their tile)
    rt0 = st[:, 0].min()
    wall_us = (fin[:, 7] - fin[:, 0]) / 100.0   # 100 MHz wall-clock ticks
    ghz = np.median((fin[:, 5] - fin[:, 1]) / wall_us) / 1e3

    def ph(a, b, rows=fin):
        rows = rows[(rows[:, a] != 0) & (rows[:, b] != 0)]   # a workgroup that skipped a phase left its stamp at zero
        if not len(rows):
            return "       -"
        d = rows[:, b] - rows[:, a]
        return f"{np.median(d):8.0f} ({d.min():.0f}..{d.max():.0f})"
    print(f"== {dt} {M}x{K}x{N} {kern}: {ms * 1e3:.2f} us/launch, {len(st)} workgroups, {len(fin)} with an epilogue, "
          f"clock ~{ghz:.2f} GHz", file=out)
    print(f"   workgroup life us: median {np.median(wall_us):.2f} max {wall_us.max():.2f}; last end "
          f"{(fin[:, 7].max() - rt0) / 100.0:.2f} us after the first start", file=out)
    line = f"   cycles, median (min..max): start->first data {ph(1, 2)}   main loop {ph(2, 3)}   "
    if S > 1:
        line += f"park+count {ph(3, 4)}   combine+epilogue {ph(4, 5)}"
        parked = st[(st[:, 6] != 0) & (st[:, 3] != 0)]
        if len(parked):
            d = parked[:, 6] - parked[:, 3]
            line += f"\n   parked slices: {len(parked)}, park+count {np.median(d):.0f} ({d.min():.0f}..{d.max():.0f})"
    else:
        line += f"epilogue {ph(3, 5)}"
    print(line, file=out, flush=True)


def run_decode(ws, M, K, N, out=sys.stdout, int4=False):
    """The streaming decode kernel's stamps: 0/7 wall clock at start/end, 1 start, 2 x in LDS, 3 end of the weight stream,
    4 after the barrier, 5 after the reduction and the store (shader clock)."""
    if int4:
        W, deq = mx.quantize_pack_int4((torch.randn((K, N), device="cuda") * 0.05).to(torch.bfloat16))
        wdt, wbytes = mx.I4, K * N // 2
    else:
        W = mx.repack_b(torch.randint(-127, 128, (K, N), dtype=torch.int8, device="cuda"))
        wdt, wbytes = mx.I8, K * N
    packs = [W] + [W.clone() for _ in range(max(2, int(540e6 // wbytes)) - 1)]
    x = torch.randn((M, K), device="cuda").to(torch.bfloat16)
    y = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")
    ep = mx.Epilogue(y, mx.PP_DEQUANT, deq_scale_per_oc=deq) if int4 else mx.Epilogue(y, mx.PP_DEQUANT, deq_scale=1e-3)
    stamp_off = COUNTER_BYTES + STAMP_OFFSET
    mx.set_option("decode_resident", 0)
    mx.set_option("decode_valu", 0)
    try:
        mx.time_gemm(x, packs, N, ep, 200, b_dtype=wdt, ws=ws)
        ms = mx.time_gemm(x, packs, N, ep, 200, b_dtype=wdt, ws=ws)
        kern = mx.last_kernel()
        torch.cuda.synchronize()
        for rep in range(4):                      # four launches in a row, the last one's stamps are read
            ws[stamp_off:].zero_()
            for i in range(4):
                mx.gemm(x, packs[(rep * 4 + i) % len(packs)], N, ep, b_dtype=wdt, ws=ws)
            torch.cuda.synchronize()
    finally:
        mx.set_option("decode_resident", -1)
        mx.set_option("decode_valu", -1)
    st = ws[stamp_off:].view(torch.int64).cpu().numpy().reshape(-1, 8)
    st = st[st[:, 0] != 0]
    if not len(st):
        print(f"== {'gemv4' if int4 else 'gemv8'} {M}x{K}x{N} {kern}: {ms * 1e3:.2f} us/launch, no stamps (this kernel is not instrumented)", file=out)
        return
    t0 = st[:, 0].min()
    start, end = (st[:, 0] - t0) / 100.0, (st[:, 7] - t0) / 100.0
    ghz = np.median((st[:, 5] - st[:, 1]) / np.maximum(end - start, 1e-3)) / 1e3

    def d(a, b):
        return np.median(st[:, b] - st[:, a])
    print(f"== {'gemv4' if int4 else 'gemv8'} {M}x{K}x{N} {kern}: {ms * 1e3:.2f} us/launch, {len(st)} workgroups, clock ~{ghz:.2f} GHz", file=out)
    print(f"   workgroup start after the first: median {np.median(start):.2f} max {start.max():.2f} us; life median "
          f"{np.median(end - start):.2f} max {(end - start).max():.2f} us; last end {end.max():.2f} us", file=out)
    print(f"   cycles, median: start->x in LDS {d(1, 2):.0f}   weight stream + products {d(2, 3):.0f}   barrier {d(3, 4):.0f}   "
          f"reduction + store {d(4, 5):.0f}", file=out, flush=True)


def ensure_library():
    """Build the instrumented library if it is missing or older than a kernel source (the shipped tree holds none)."""
    if "MMX_LIB_PATH" in os.environ:
        return
    from mm_amx_amd import build as B
    srcs = [os.path.join(B.CSRC, f) for f in list(B.SOURCES) + list(B.HEADERS)]
    if not os.path.exists(STAMPS_LIB) or os.path.getmtime(STAMPS_LIB) < max(os.path.getmtime(f) for f in srcs):
        print("phase_stamps: building the instrumented library (several minutes)", file=sys.stderr, flush=True)
        B.build(incremental=True, stamps=True)


def main(argv):
    ensure_library()
    if "stamps" not in os.path.basename(mx.lib_path()):
        sys.exit("phase_stamps: MMX_LIB_PATH does not name an instrumented library (python -m mm_amx_amd.build --stamps)")
    mx.init(0)
    ws = torch.zeros(COUNTER_BYTES + STAMP_OFFSET + STAMP_BYTES, dtype=torch.uint8, device="cuda")
    for a in argv:
        parts = a.split(",")
        if parts[0] in ("gemv8", "gemv4"):
            run_decode(ws, int(parts[1]), int(parts[2]), int(parts[3]), int4=parts[0] == "gemv4")
            continue
        dt, M, K, N, tile, S = parts[:6]
        run(ws, dt, int(M), int(K), int(N), tile, int(S), waves=int(parts[6]) if len(parts) > 6 else 8)


if __name__ == "__main__":
    main(sys.argv[1:])
