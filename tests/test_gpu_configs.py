"""The five measured workloads at their stated sizes against the oracle (forward; the backward workload at full size
is test_gpu_backward.py::test_backward_gptoss20b_full and the GPT-OSS-20B forward is
test_gpu_forward.py::test_forward_gptoss20b_full)."""
import numpy as np
import pytest
import torch

from oracle import yamoe_oracle as O
from tests.util import KEYS, args, oracle_forward, report
from yamoe_amd.workloads import CONFIGS, device_weights, make_config

pytestmark = pytest.mark.gpu


def run_dev(g, capacity):
    import yamoe_amd
    E, K = g["gate_up_proj"].shape[0], g["router_indices"].shape[1]
    out = yamoe_amd.experts(*[g[k] for k in KEYS], capacity, E, K)
    torch.cuda.synchronize()
    return out.cpu()


def test_readme_shape_all_eight_experts_fp32(gpu):
    """README.md:67-112: 16 x 256 tokens, hidden 2880, 8 experts, top-2, fp32, randn weights, zero biases, softmax
    over all experts then top-2 (not renormalised), seed 42.  Capacity = tokens keeps every assignment (fp64 oracle,
    rel-L2 <= 1e-5); the README's literal eighth argument, 256, is the capacity and drops about three quarters of
    them: checked against the capacity rule of the oracle."""
    d, c = make_config("readme", seed=42)
    assert d["gate_up_proj"].shape == (8, 2880, 5760) and d["hidden"].dtype == torch.float32
    g = {k: v.to(gpu) for k, v in d.items()}
    got = run_dev(g, c["T"])
    want = oracle_forward(d, c["T"], compute_dtype=torch.float64)
    assert report("readme fp32 E=8", got, want, 1e-5) < 1e-5
    got = run_dev(g, 256)
    want = oracle_forward(d, 256, compute_dtype=torch.float64)
    counts = np.bincount(d["router_indices"].numpy().ravel(), minlength=8)
    kept = int(np.minimum(counts, 256).sum())
    print("capacity 256 keeps %d of %d assignments" % (kept, counts.sum()), flush=True)
    assert kept < counts.sum() // 2
    assert report("readme fp32 E=8 capacity 256", got, want, 1e-5) < 1e-5


def test_decode_shape_128_experts(gpu):
    """64 tokens, 128 experts of the GPT-OSS-120B shape, top-4, bf16: weights drawn on the device (6.4 GB) and copied
    back for the oracle."""
    c = CONFIGS["decode"]
    host, _ = make_config("decode", seed=0, weights=False)
    g = {k: v.to(gpu) for k, v in host.items()}
    g.update(device_weights(c["E"], c["H"], c["I"], c["dtype"], c["w_std"], 2, gpu))
    counts = np.bincount(host["router_indices"].numpy().ravel(), minlength=c["E"])
    print("decode: %d active experts, at most %d rows" % ((counts > 0).sum(), counts.max()), flush=True)
    got = run_dev(g, c["T"])
    d = {k: v.cpu() for k, v in g.items()}
    want = oracle_forward(d, c["T"])
    assert report("decode E=128", got, want, 1e-2) < 1e-2


def test_zipf_shape_forward(gpu):
    """16 384 tokens, 128 experts, top-4, bf16, Zipf(1.2) expert popularity: the hottest expert holds thousands of
    rows, some experts none."""
    c = CONFIGS["zipf"]
    host, _ = make_config("zipf", seed=0, weights=False)
    g = {k: v.to(gpu) for k, v in host.items()}
    g.update(device_weights(c["E"], c["H"], c["I"], c["dtype"], c["w_std"], 4, gpu))
    counts = np.bincount(host["router_indices"].numpy().ravel(), minlength=c["E"])
    print("zipf: max rows %d, empty experts %d" % (counts.max(), (counts == 0).sum()), flush=True)
    assert counts.max() > 10 * counts.mean() and (counts == 0).sum() > 0
    got = run_dev(g, c["T"])
    d = {k: v.cpu() for k, v in g.items()}
    del g
    torch.cuda.empty_cache()
    want = oracle_forward(d, c["T"])
    assert report("zipf 16384 tokens", got, want, 1e-2) < 1e-2


@pytest.mark.parametrize("tokens,experts", [(65536, 32), (16384, 128)])
def test_token_order_does_not_change_a_row_at_scale(gpu, tokens, experts):
    """Beyond the sizes the oracle is run at: 65 536 tokens on 32 experts (8192 rows per expert, every expert walked in
    bands of row tiles) and 16 384 tokens with Zipf routing on 128 experts, H = I = 2880, top-4, bf16.  A token's output
    depends on its own row only, and the kernels add a row's products in an order that does not depend on where the row
    sits in a tile: the same tokens in another order must give the same bits, row for row.  Spot rows are checked
    against the oracle."""
    import yamoe_amd
    from yamoe_amd.workloads import make_routing
    H = I = 2880
    K = 4
    gen = torch.Generator().manual_seed(tokens)
    idx, dense = make_routing(tokens, experts, K, gen, zipf=1.2 if experts == 128 else 0.0)
    x = (torch.randn(tokens, H, generator=gen)).to(torch.bfloat16)
    w = device_weights(experts, H, I, torch.bfloat16, 0.02, 9, gpu)
    dense = dense.to(torch.bfloat16)
    perm = torch.randperm(tokens, generator=gen)
    a = (w["gate_up_proj"], w["gate_up_proj_bias"], w["down_proj"], w["down_proj_bias"], tokens, experts, K)
    out = yamoe_amd.experts(x.to(gpu), idx.to(gpu), dense.to(gpu), *a)
    out_p = yamoe_amd.experts(x[perm].to(gpu), idx[perm].to(gpu), dense[perm].to(gpu), *a)
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all()
    assert torch.equal(out[perm.to(gpu)], out_p)
    # 64 spot tokens against the oracle (their rows of the batch alone: a token's output needs no other token)
    spot = torch.randperm(tokens, generator=gen)[:64]
    d = dict(hidden=x[spot], router_indices=idx[spot], routing_weights=dense[spot],
             **{k: v.cpu() for k, v in w.items()})
    want = oracle_forward(d, 64)
    assert report("spot rows of %d tokens" % tokens, out[spot.to(gpu)].cpu(), want, 1e-2) < 1e-2
