"""Hidden and intermediate sizes that are not whole 16-byte chunks (the reference asks no alignment of them:
csrc/moe.cpp:138-220 takes any H and I).  Such shapes run on the plain-FMA kernels; forward and all six gradients through
the torch op against the fp64 oracle at the tolerance of the dtype, and the static-workspace forward gives the same bits
as the forward."""
import pytest
import torch

from oracle import yamoe_oracle as O
from tests.util import args, to_dev
from yamoe_amd.workloads import make_inputs

pytestmark = pytest.mark.gpu

NAMES = ("d_hidden", "d_routing", "d_gate_up_proj", "d_gate_up_proj_bias", "d_down_proj", "d_down_proj_bias")
TOL = {torch.float32: 1e-5, torch.bfloat16: 1e-2, torch.float16: 2e-3}

SHAPES = [
    # T, H, I, E, K, capacity (0: tokens), zipf, slot weights
    (300, 67, 35, 5, 3, 0, 0.0, True),         # both sizes odd
    (513, 130, 64, 4, 2, 0, 0.0, False),       # fp32: H not a multiple of 4; 16-bit: of 8
    (700, 64, 99, 3, 2, 0, 0.0, False),        # only I is odd; more than 256 rows per expert
    (400, 257, 36, 16, 2, 0, 1.5, False),      # empty experts
    (600, 66, 34, 4, 2, 37, 0.5, True),        # capacity drops assignments
    (1, 3, 5, 2, 1, 0, 0.0, False),
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,H,I,E,K,capacity,zipf,slot_weights", SHAPES)
def test_sizes_that_are_not_whole_chunks(gpu, dtype, T, H, I, E, K, capacity, zipf, slot_weights):
    import yamoe_amd
    print("plain", dtype, T, H, I, E, K, capacity, zipf, slot_weights, flush=True)
    vec = 16 // torch.empty((), dtype=dtype).element_size()
    assert H % vec or I % vec, "this shape would run on the MFMA kernels"
    d = make_inputs(T, H, I, E, K, dtype, seed=T + H, w_std=0.3, bias_std=0.2, zipf=zipf)
    if slot_weights:
        d["routing_weights"] = torch.gather(d["routing_weights"], 1, d["router_indices"])
    cap = capacity or T
    g = to_dev(d, gpu)
    out = yamoe_amd.experts(*args(g), cap, E, K)
    torch.cuda.synchronize()
    assert out.dtype == dtype
    want = O.experts_capacity(*args(d), cap, compute_dtype=torch.float64)
    r = O.rel_l2(out.cpu(), want)
    print("  forward rel_l2 %.2e" % r, flush=True)
    assert r < TOL[dtype]
    gy = torch.randn(T, H, generator=torch.Generator().manual_seed(7)).to(dtype)
    grads = yamoe_amd.experts_backward(gy.to(gpu), *args(g), cap, E, K)
    torch.cuda.synchronize()
    want_g = O.experts_backward(gy, *args(d), cap, compute_dtype=torch.float64)
    for n, a, b in zip(NAMES, grads, want_g):
        assert a.dtype == dtype and a.shape == b.shape, n
        rr = O.rel_l2(a.cpu(), b)
        print("  %s rel_l2 %.2e" % (n, rr), flush=True)
        assert rr < TOL[dtype], (n, rr)


def test_static_workspace_forward_takes_them_too(gpu):
    from yamoe_amd import _cabi
    T, H, I, E, K = 200, 70, 37, 4, 2
    d = to_dev(make_inputs(T, H, I, E, K, torch.bfloat16, seed=3, w_std=0.3, bias_std=0.2), gpu)
    a = _cabi.experts_forward(*args(d), T)
    b = _cabi.experts_forward_static(*args(d), T, torch.full_like(a, float("nan")))
    torch.cuda.synchronize()
    assert torch.equal(a, b)
