"""Comparison leg of the timing sweep: what drbh/yamoe's compare_example.py:195-251 (pairwise MSE / MAE / cosine /
relative L2 / max-abs between the kernel, the GptOssExperts reference and the binned restatement) and
perf_plot.py:204-229 (speed-up and memory ratio against the reference) print, as JSON lines.

    python -m tests.compare_sweep [--configs 0,1,..] [--batches 1,2,..] [--iters 10] [--max-gflop 400]

It lives under tests/ because it runs the CPU oracle, which the product package may not import.  The three
implementations compared per sweep point (yamoe_amd.sweep.make_point: fp16, unit-variance weights, biases of one):
  kernel      yamoe_amd.experts on the GPU
  reference   oracle.experts_loop, fp32 on the CPU: the role of yamoe.reference.GptOssExperts (no capacity)
  binned      oracle.experts_capacity, fp32 on the CPU: the role of vendored/yamoe_ref.binned_experts_ref
The reference scripts time their baseline on the same GPU; here the baseline is the CPU oracle, so `speedup` is
CPU-oracle time over kernel time, and `memory_ratio` is the size of the reference op's padded temporaries
([E,C,H] + [E,C,2H] + [E,C,H], csrc/moe.cpp:138-187) over the peak extra memory the kernel's call allocated.
Points above --max-gflop of oracle work are timed but not compared."""
import argparse
import json
import sys
import time

import torch

from oracle import yamoe_oracle as O
from yamoe_amd import sweep

KEYS = ("hidden", "router_indices", "routing_weights", "gate_up_proj", "gate_up_proj_bias", "down_proj", "down_proj_bias")


def metrics(a, b):
    """compare_example.py:198-214 for one pair (b is the reference side)."""
    a, b = a.double().reshape(-1), b.double().reshape(-1)
    nb = float(torch.norm(b))
    return dict(mse=float(torch.mean((a - b) ** 2)), mae=float(torch.mean((a - b).abs())),
                cosine=float(torch.nn.functional.cosine_similarity(a[None], b[None])),
                rel_l2=float(torch.norm(a - b)) / nb if nb > 0 else float("inf"), max_abs=float((a - b).abs().max()))


def compare_point(batch_size, seq_len, hidden_dim, num_experts, top_k, iters=10, warmup=3, capacity="tokens", max_gflop=400.0):
    import yamoe_amd
    r = sweep.run_point(batch_size, seq_len, hidden_dim, num_experts, top_k, iters=iters, warmup=warmup, capacity=capacity)
    gflop = r["kept_assignments"] * 6 * hidden_dim * hidden_dim / 1e9
    r["compared"] = gflop <= max_gflop
    if not r["compared"]:
        return r
    p = sweep.make_point(batch_size, seq_len, hidden_dim, num_experts, top_k)   # same seed: the tensors run_point timed
    cap = r["capacity"]
    kernel = yamoe_amd.experts(*[p[k] for k in KEYS], cap, num_experts, top_k).float().cpu()
    host = [p[k].cpu() for k in KEYS]
    t0 = time.perf_counter()
    reference = O.experts_loop(*host, compute_dtype=torch.float32)
    cpu_ms = (time.perf_counter() - t0) * 1e3
    binned = O.experts_capacity(*host, cap, compute_dtype=torch.float32)
    r["kernel_vs_reference"] = metrics(kernel, reference)
    r["kernel_vs_binned"] = metrics(kernel, binned)
    r["reference_vs_binned"] = metrics(reference, binned)
    r["oracle_cpu_ms"] = round(cpu_ms, 2)
    r["speedup_vs_cpu_oracle"] = round(cpu_ms / r["ms"], 1)
    padded_mib = num_experts * cap * 4 * hidden_dim * 2 / 2 ** 20        # x [E,C,H] + gate_up [E,C,2H] + out [E,C,H], fp16
    r["reference_padded_mib"] = round(padded_mib, 1)
    r["memory_ratio"] = round(padded_mib / max(r["peak_extra_mib"], 1e-3), 2)
    return r


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--configs", default=",".join(str(i) for i in range(len(sweep.CONFIGS))))
    ap.add_argument("--batches", default="1,2,4")
    ap.add_argument("--iters", type=int, default=10)
    ap.add_argument("--capacity", choices=("seq", "tokens"), default="tokens")
    ap.add_argument("--max-gflop", type=float, default=400.0)
    a = ap.parse_args(argv)
    for ci in (int(c) for c in a.configs.split(",")):
        for b in (int(x) for x in a.batches.split(",")):
            r = compare_point(b, iters=a.iters, capacity=a.capacity, max_gflop=a.max_gflop, **sweep.CONFIGS[ci])
            r["config"] = ci
            print(json.dumps(r), flush=True)
            torch.cuda.empty_cache()


if __name__ == "__main__":
    sys.exit(main())
