"""The whole op in double precision (the reference dispatches over double too: csrc/gather.cu:89, csrc/scatter.cu:128,
csrc/experts_backward.cu:236).  Forward and all six gradients through the torch op against the fp64 oracle, relative L2
<= 1e-12: accumulation order is the only difference."""
import pytest
import torch

from oracle import yamoe_oracle as O
from tests.util import args, to_dev
from yamoe_amd.workloads import make_inputs

pytestmark = pytest.mark.gpu

NAMES = ("d_hidden", "d_routing", "d_gate_up_proj", "d_gate_up_proj_bias", "d_down_proj", "d_down_proj_bias")
TOL = 1e-12

SHAPES = [
    # T, H, I, E, K, capacity (0: tokens), zipf, slot weights
    (40, 64, 64, 4, 2, 0, 0.0, False),
    (700, 64, 96, 3, 2, 0, 0.0, False),       # more than 256 rows per expert: several row tiles
    (513, 67, 35, 5, 3, 0, 0.0, True),         # odd sizes: no alignment is asked of double data
    (300, 130, 62, 16, 2, 0, 1.5, False),      # empty experts
    (600, 128, 64, 4, 2, 37, 0.5, True),       # capacity drops assignments
    (1, 8, 6, 2, 1, 0, 0.0, False),
]


@pytest.mark.parametrize("T,H,I,E,K,capacity,zipf,slot_weights", SHAPES)
def test_forward_and_backward_fp64(gpu, T, H, I, E, K, capacity, zipf, slot_weights):
    import yamoe_amd
    print("fp64", T, H, I, E, K, capacity, zipf, slot_weights, flush=True)
    d = make_inputs(T, H, I, E, K, torch.float64, seed=T + H, w_std=0.3, bias_std=0.2, zipf=zipf)
    if slot_weights:
        d["routing_weights"] = torch.gather(d["routing_weights"], 1, d["router_indices"])
    cap = capacity or T
    g = to_dev(d, gpu)
    out = yamoe_amd.experts(*args(g), cap, E, K)
    torch.cuda.synchronize()
    assert out.dtype == torch.float64
    want = O.experts_capacity(*args(d), cap, compute_dtype=torch.float64)
    r = O.rel_l2(out.cpu(), want)
    print("  forward rel_l2 %.2e" % r, flush=True)
    assert r < TOL
    gy = torch.randn(T, H, generator=torch.Generator().manual_seed(7), dtype=torch.float64)
    grads = yamoe_amd.experts_backward(gy.to(gpu), *args(g), cap, E, K)
    torch.cuda.synchronize()
    want_g = O.experts_backward(gy, *args(d), cap, compute_dtype=torch.float64)
    for n, a, b in zip(NAMES, grads, want_g):
        assert a.dtype == torch.float64 and a.shape == b.shape, n
        rr = O.rel_l2(a.cpu(), b)
        print("  %s rel_l2 %.2e" % (n, rr), flush=True)
        assert rr < TOL, (n, rr)


def test_fp64_repeated_expert_and_determinism(gpu):
    """A token that names one expert twice gets the sum of its slots' routing gradients; two runs give the same bits."""
    import yamoe_amd
    T, H, I, E, K = 33, 40, 24, 4, 3
    d = make_inputs(T, H, I, E, K, torch.float64, seed=41, w_std=0.3, bias_std=0.2)
    d["router_indices"][::2, 2] = d["router_indices"][::2, 0]
    gy = torch.randn(T, H, generator=torch.Generator().manual_seed(42), dtype=torch.float64)
    g = to_dev(d, gpu)
    runs = [[t.cpu() for t in yamoe_amd.experts_backward(gy.to(gpu), *args(g), T, E, K)] for _ in range(2)]
    for a, b in zip(*runs):
        assert torch.equal(a, b)
    want = O.experts_backward(gy, *args(d), T, compute_dtype=torch.float64)
    for n, a, b in zip(NAMES, runs[0], want):
        assert O.rel_l2(a, b) < TOL, n
