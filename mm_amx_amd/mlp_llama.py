"""The reference's end-to-end demo on the GPU: a stack of Llama-7B MLPs (RMSNorm + gate/up/SiLU/down),
once through torch's own bf16 linear layers and once through this library's fused MLP.

Follows torch-ext/test.py:176-218 (``perf_llama7b_MLP``: 32 layers, per-layer time, GFlops, GB/s,
closeness of the two results) and torch-ext/mlp_llama.py:6-19 (the module).  Every layer has its own
weights (32 x 270 MB stay resident in HBM), as in the reference's deep-copied stack.

    python -m mm_amx_amd.mlp_llama --M 256 --layers 32 --rounds 10
"""
import argparse
import time

import torch

from . import ops


class LlamaRMSNorm(torch.nn.Module):
    """torch-ext/test.py:163-173."""

    def __init__(self, eps=1e-6):
        super().__init__()
        self.variance_epsilon = eps

    def forward(self, hidden_states):
        input_dtype = hidden_states.dtype
        hidden_states = hidden_states.to(torch.float32)
        variance = hidden_states.pow(2).mean(-1, keepdim=True)
        hidden_states = hidden_states * torch.rsqrt(variance + self.variance_epsilon)
        return hidden_states.to(input_dtype)


class LlamaMLP(torch.nn.Module):
    """torch-ext/mlp_llama.py:6-19 with bf16 weights on the GPU; ``opt`` switches between torch's linear layers
    and the fused MLP of this library (as ``config.opt`` does in torch-ext/test.py)."""

    def __init__(self, hidden_size=4096, intermediate_size=11008, seed=0, device="cuda"):
        super().__init__()
        g = torch.Generator(device=device).manual_seed(seed)
        mk = lambda o, i: (torch.randn((o, i), device=device, generator=g) * 0.02).to(torch.bfloat16)
        self.hidden_size, self.intermediate_size = hidden_size, intermediate_size
        self.w_gate, self.w_up, self.w_down = mk(intermediate_size, hidden_size), mk(intermediate_size, hidden_size), mk(
            hidden_size, intermediate_size)
        self.fused = ops.MLP()
        self.fused.setup(self.w_gate, self.w_up, self.w_down)
        self.opt = False

    def flops(self, M):  # torch-ext/test.py: 2 flops per weight element and row
        return 2.0 * M * 3 * self.hidden_size * self.intermediate_size

    def numel(self, M):
        return 3 * self.hidden_size * self.intermediate_size

    def forward(self, x):
        if self.opt:
            return self.fused.run(x)
        F = torch.nn.functional
        return F.linear(F.silu(F.linear(x, self.w_gate)) * F.linear(x, self.w_up), self.w_down)


def perf_llama7b_MLP(M=256, num_layers=32, rounds=10, hidden_size=4096, intermediate_size=11008, verbose=True, graph=False):
    layers = []
    for i in range(num_layers):
        layers += [LlamaRMSNorm(), LlamaMLP(hidden_size, intermediate_size, seed=i)]
    net = torch.nn.Sequential(*layers)
    mlps = [m for m in layers if isinstance(m, LlamaMLP)]
    x = torch.randint(-1, 2, (M, hidden_size), dtype=torch.float32, device="cuda").to(torch.bfloat16)
    out = {}
    with torch.no_grad():
        for opt in (False, True):
            for m in mlps:
                m.opt = opt
            y = net(x)  # warm-up
            torch.cuda.synchronize()
            t0 = time.time()
            for _ in range(rounds):
                y = net(x)
            torch.cuda.synchronize()
            dt = (time.time() - t0) / rounds / num_layers
            name = "mm_amx_amd" if opt else "torch"
            out[name] = {"per_layer_us": dt * 1e6, "GFlops": mlps[0].flops(M) * 1e-9 / dt,
                         "GBps": mlps[0].numel(M) * 2 * 1e-9 / dt}
            out["y_" + name] = y.float()
            if verbose:
                print(f"{name:>11}: per-layer dt {dt * 1e6:9.1f} us   GFlops {out[name]['GFlops']:10.0f}   "
                      f"GB/s {out[name]['GBps']:8.0f}")
        if graph:
            # the same stack through this library replayed from a HIP graph: what is left when the host side of every
            # call (Python, ctypes marshalling, launch) is taken out of the per-layer figure
            side = torch.cuda.Stream()
            with torch.cuda.stream(side):
                net(x)  # (an eager pass on this stream first: the K-split workspace of a stream is made outside a capture)
                torch.cuda.synchronize()
                gr = torch.cuda.CUDAGraph()
                with torch.cuda.graph(gr, stream=side):
                    yg = net(x)
            torch.cuda.synchronize()
            gr.replay()
            torch.cuda.synchronize()
            t0 = time.time()
            for _ in range(rounds):
                gr.replay()
            torch.cuda.synchronize()
            dt = (time.time() - t0) / rounds / num_layers
            out["mm_amx_amd_graph"] = {"per_layer_us": dt * 1e6, "GFlops": mlps[0].flops(M) * 1e-9 / dt,
                                       "GBps": mlps[0].numel(M) * 2 * 1e-9 / dt,
                                       "same_bits_as_eager": bool(torch.equal(yg.float(), out["y_mm_amx_amd"]))}
            if verbose:
                print(f"{'graph':>11}: per-layer dt {dt * 1e6:9.1f} us   GFlops {out['mm_amx_amd_graph']['GFlops']:10.0f}   "
                      f"GB/s {out['mm_amx_amd_graph']['GBps']:8.0f}")
            del gr
    y0, y1 = out.pop("y_torch"), out.pop("y_mm_amx_amd")
    out["rel_err"] = (torch.linalg.norm(y1 - y0) / torch.linalg.norm(y0)).item()
    # one layer on the same input: the stack has no residual connections, so rounding differences of
    # the bf16 intermediates are amplified from layer to layer and the end-to-end figure says little
    with torch.no_grad():
        xin = layers[0](x)
        mlps[0].opt = False
        a = mlps[0](xin).float()
        mlps[0].opt = True
        b = mlps[0](xin).float()
    out["rel_err_one_layer"] = (torch.linalg.norm(b - a) / torch.linalg.norm(a)).item()
    if verbose:
        print(f"relative difference of the two paths: one layer {out['rel_err_one_layer']:.2e}, "
              f"after {num_layers} layers {out['rel_err']:.2e}")
    return out


if __name__ == "__main__":
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--M", type=int, default=256)
    ap.add_argument("--layers", type=int, default=32)
    ap.add_argument("--rounds", type=int, default=10)
    ap.add_argument("--graph", action="store_true", help="also replay the stack from a HIP graph")
    a = ap.parse_args()
    ops.L.init(0)
    perf_llama7b_MLP(a.M, a.layers, a.rounds, graph=a.graph)
