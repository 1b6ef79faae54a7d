"""Timing sweep of the `experts` op over the shapes drbh/yamoe plots (perf_plot.py:29-39: six layer shapes x seven
batch sizes, fp16, routing from random logits), one JSON line per point instead of a figure.

    python -m yamoe_amd.sweep [--configs 0,1,..] [--batches 1,2,4,..] [--iters 20] [--capacity seq|tokens] [--torch]

`--capacity seq` passes `seq_len` as `expert_capacity` like the reference script does (perf_plot.py:118: assignments
beyond that rank inside an expert are dropped); `tokens` (default) keeps every assignment.  TFLOP/s counts
6 * hidden^2 flop per kept assignment.  `--torch` also times the plain-torch experts module on the same GPU and inputs
(perf_plot.py:104-146 times `reference.GptOssExperts` in inference mode next to the kernel and plots the ratio): here
`yamoe_amd.reference.GptOssExperts`, in its per-expert form (`train()`: the experts that were picked, each on its own
tokens) and, where its E-fold work and memory fit, in its dense form (`eval()`: every expert on every token).
"""
import argparse
import json
import sys

import torch

CONFIGS = [
    {"seq_len": 512, "hidden_dim": 2880, "num_experts": 32, "top_k": 4},
    {"seq_len": 1024, "hidden_dim": 2880, "num_experts": 32, "top_k": 4},
    {"seq_len": 512, "hidden_dim": 1024, "num_experts": 32, "top_k": 4},
    {"seq_len": 512, "hidden_dim": 2880, "num_experts": 16, "top_k": 2},
    {"seq_len": 2048, "hidden_dim": 1024, "num_experts": 16, "top_k": 2},
    {"seq_len": 768, "hidden_dim": 2048, "num_experts": 64, "top_k": 8},
]
BATCH_SIZES = [1, 2, 4, 8, 16, 32, 64]


def make_point(batch_size, seq_len, hidden_dim, num_experts, top_k, dtype=torch.float16, device="cuda", seed=0):
    """Inputs of one sweep point, drawn on the device (same distributions as perf_plot.py:66-101)."""
    g = torch.Generator(device=device).manual_seed(seed)
    tokens = batch_size * seq_len
    logits = torch.randn(tokens, num_experts, generator=g, device=device)
    weights, indices = torch.topk(logits, top_k, dim=-1)
    weights = torch.softmax(weights, dim=-1)
    routing = torch.zeros(tokens, num_experts, device=device).scatter_(1, indices, weights).to(dtype)

    def draw(*shape):
        out = torch.empty(shape, dtype=dtype, device=device)
        for e in range(shape[0]):   # expert by expert: no fp32 copy of the whole tensor
            out[e] = torch.randn(shape[1:], generator=g, device=device).to(dtype)
        return out
    return dict(hidden=torch.randn(tokens, hidden_dim, generator=g, device=device).to(dtype), router_indices=indices,
                routing_weights=routing, gate_up_proj=draw(num_experts, hidden_dim, 2 * hidden_dim),
                gate_up_proj_bias=torch.ones(num_experts, 2 * hidden_dim, dtype=dtype, device=device),
                down_proj=draw(num_experts, hidden_dim, hidden_dim),
                down_proj_bias=torch.ones(num_experts, hidden_dim, dtype=dtype, device=device))


def time_torch_modules(p, tokens, hidden_dim, num_experts, iters, kernel_out):
    """The torch experts module on the inputs of one point: milliseconds per call of its two forms and the distance of
    its result from the kernel's."""
    import types

    from .reference import GptOssExperts
    cfg = types.SimpleNamespace(hidden_size=hidden_dim, intermediate_size=hidden_dim, num_local_experts=num_experts)
    with torch.device("meta"):
        mod = GptOssExperts(cfg)
    for name in ("gate_up_proj", "gate_up_proj_bias", "down_proj", "down_proj_bias"):
        setattr(mod, name, torch.nn.Parameter(p[name], requires_grad=False))

    def timed(fn):
        fn()
        torch.cuda.synchronize()
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(iters):
            out = fn()
        end.record()
        torch.cuda.synchronize()
        return start.elapsed_time(end) / iters, out

    res = {}
    with torch.no_grad():
        mod.train()
        ms, out = timed(lambda: mod(p["hidden"], p["router_indices"], p["routing_weights"]))
        res["torch_per_expert_ms"] = round(ms, 4)
        diff = (out.float() - kernel_out.float()).norm() / kernel_out.float().norm().clamp_min(1e-30)
        res["rel_l2_vs_torch"] = float("%.3e" % float(diff))
        del out
        if num_experts * tokens * hidden_dim * 3 * 2 <= 24 << 30:   # the dense form holds [E, T, 3 * hidden] values
            mod.eval()
            res["torch_dense_ms"] = round(timed(lambda: mod(p["hidden"], p["router_indices"], p["routing_weights"]))[0], 4)
    return res


def run_point(batch_size, seq_len, hidden_dim, num_experts, top_k, iters=20, warmup=5, capacity="tokens", dtype=torch.float16,
              torch_too=False):
    from . import experts
    p = make_point(batch_size, seq_len, hidden_dim, num_experts, top_k, dtype)
    tokens = batch_size * seq_len
    cap = seq_len if capacity == "seq" else tokens
    args = (p["hidden"], p["router_indices"], p["routing_weights"], p["gate_up_proj"], p["gate_up_proj_bias"],
            p["down_proj"], p["down_proj_bias"], cap, num_experts, top_k)
    counts = torch.bincount(p["router_indices"].reshape(-1), minlength=num_experts)
    kept = int(torch.clamp(counts, max=cap).sum())
    for _ in range(warmup):
        experts(*args)
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    before = torch.cuda.memory_allocated()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(iters):
        out = experts(*args)
    end.record()
    torch.cuda.synchronize()
    ms = start.elapsed_time(end) / iters
    extra = {}
    if torch_too:
        extra = time_torch_modules(p, tokens, hidden_dim, num_experts, max(3, iters // 4), out)
        extra["speedup_vs_torch_per_expert"] = round(extra["torch_per_expert_ms"] / ms, 2)
    return dict(**extra, batch_size=batch_size, seq_len=seq_len, hidden_dim=hidden_dim, num_experts=num_experts, top_k=top_k,
                dtype=str(dtype).replace("torch.", ""), capacity=cap, kept_assignments=kept, ms=round(ms, 4),
                tflops=round(kept * 6 * hidden_dim * hidden_dim / (ms * 1e-3) / 1e12, 2),
                peak_extra_mib=round((torch.cuda.max_memory_allocated() - before) / 2 ** 20, 1),
                finite=bool(torch.isfinite(out.float()).all()))


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--configs", default=",".join(str(i) for i in range(len(CONFIGS))))
    ap.add_argument("--batches", default=",".join(str(b) for b in BATCH_SIZES))
    ap.add_argument("--iters", type=int, default=20)
    ap.add_argument("--capacity", choices=("seq", "tokens"), default="tokens")
    ap.add_argument("--torch", action="store_true", help="also time the plain-torch experts module on the same inputs")
    a = ap.parse_args(argv)
    for ci in (int(c) for c in a.configs.split(",")):
        for b in (int(x) for x in a.batches.split(",")):
            r = run_point(b, iters=a.iters, capacity=a.capacity, torch_too=a.torch, **CONFIGS[ci])
            r["config"] = ci
            print(json.dumps(r), flush=True)
            torch.cuda.empty_cache()


if __name__ == "__main__":
    sys.exit(main())
