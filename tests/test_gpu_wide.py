"""hidden_states / grad_out of 4 GiB or more.  The GEMM kernels gather token rows with 32-bit byte offsets from the start
of the tensor; beyond that the op permutes the tensor into expert order first and reads it in order (the reference has
no such limit: csrc/gather.cu:6-66 indexes with 64-bit offsets).  The path is forced at small sizes through
YAMOE_GATHER_SPAN_BYTES and must give the bits of the gathering path; one case runs it at its real size and is checked
against the same tokens computed in two halves that stay below the limit."""
import os

import pytest
import torch

from oracle import yamoe_oracle as O
from tests.util import REL_L2_TOL, args, oracle_forward, to_dev
from yamoe_amd.workloads import make_inputs

pytestmark = pytest.mark.gpu


@pytest.fixture
def permute_always():
    os.environ["YAMOE_GATHER_SPAN_BYTES"] = "1"
    yield
    del os.environ["YAMOE_GATHER_SPAN_BYTES"]


SHAPES = [
    # T, H, I, E, K, capacity (0: tokens), zipf
    (700, 128, 64, 3, 2, 0, 0.0),       # several row tiles per expert
    (513, 320, 136, 5, 3, 0, 0.0),      # contraction not a multiple of 64: the register-staged kernels
    (2000, 64, 64, 64, 2, 0, 0.8),      # streamed experts next to tiled ones
    (600, 128, 64, 4, 2, 37, 0.5),      # capacity drops assignments
    (40, 64, 64, 16, 1, 0, 0.0),        # every expert streams
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("T,H,I,E,K,capacity,zipf", SHAPES)
def test_permuted_path_gives_the_bits_of_the_gathering_path(gpu, dtype, T, H, I, E, K, capacity, zipf):
    import yamoe_amd
    print("wide (forced)", dtype, T, H, I, E, K, capacity, zipf, flush=True)
    d = make_inputs(T, H, I, E, K, dtype, seed=T + H, w_std=0.2, bias_std=0.1, zipf=zipf)
    cap = capacity or T
    g = to_dev(d, gpu)
    gy = torch.randn(T, H, generator=torch.Generator().manual_seed(3)).to(dtype).to(gpu)
    want = yamoe_amd.experts(*args(g), cap, E, K)
    want_g = yamoe_amd.experts_backward(gy, *args(g), cap, E, K)
    torch.cuda.synchronize()
    os.environ["YAMOE_GATHER_SPAN_BYTES"] = "1"
    try:
        got = yamoe_amd.experts(*args(g), cap, E, K)
        got_g = yamoe_amd.experts_backward(gy, *args(g), cap, E, K)
        torch.cuda.synchronize()
    finally:
        del os.environ["YAMOE_GATHER_SPAN_BYTES"]
    assert torch.equal(got, want)
    for a, b in zip(got_g, want_g):
        assert torch.equal(a, b)
    assert O.rel_l2(got.cpu(), oracle_forward(d, cap)) < REL_L2_TOL[dtype]


def test_static_workspace_forward_on_the_permuted_path(gpu, permute_always):
    from yamoe_amd import _cabi
    T, H, I, E, K = 500, 128, 64, 4, 2
    d = to_dev(make_inputs(T, H, I, E, K, torch.bfloat16, seed=3, w_std=0.2, bias_std=0.1), gpu)
    a = _cabi.experts_forward(*args(d), T)
    b = _cabi.experts_forward_static(*args(d), T, torch.full_like(a, float("nan")))
    torch.cuda.synchronize()
    assert torch.equal(a, b)


def test_hidden_states_of_more_than_4_gib(gpu):
    """160 000 tokens of 14 336 bf16 values are 4.59 GB.  A token's output and input gradient depend on its own row
    only, so the two halves of the batch (2.3 GB each, on the gathering path) must give the same bits; the weight and
    bias gradients of the halves add up to those of the whole (each half rounds to bf16 once: compared at 1e-2)."""
    import yamoe_amd
    T, H, I, E, K = 160_000, 14_336, 64, 4, 1
    assert T * H * 2 >= 1 << 32 and (T // 2) * H * 2 < 1 << 32
    gen = torch.Generator(device=gpu).manual_seed(11)
    x = torch.randn(T, H, generator=gen, device=gpu, dtype=torch.bfloat16)
    gy = torch.randn(T, H, generator=gen, device=gpu, dtype=torch.bfloat16)
    idx = torch.randint(0, E, (T, K), generator=gen, device=gpu)
    rw = torch.rand(T, E, generator=gen, device=gpu).to(torch.bfloat16)
    w = [(torch.randn(s, generator=gen, device=gpu) * 0.02).to(torch.bfloat16)
         for s in ((E, H, 2 * I), (E, 2 * I), (E, I, H), (E, H))]
    out = yamoe_amd.experts(x, idx, rw, *w, T, E, K)
    grads = yamoe_amd.experts_backward(gy, x, idx, rw, *w, T, E, K)
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all()
    acc = [torch.zeros_like(t, dtype=torch.float32) for t in w]
    h = T // 2
    for lo in (0, h):
        s = slice(lo, lo + h)
        assert torch.equal(out[s], yamoe_amd.experts(x[s], idx[s], rw[s], *w, h, E, K))
        part = yamoe_amd.experts_backward(gy[s], x[s], idx[s], rw[s], *w, h, E, K)
        assert torch.equal(grads[0][s], part[0]) and torch.equal(grads[1][s], part[1])
        for a, p in zip(acc, part[2:]):
            a += p.float()
        del part
    for name, a, b in zip(("d_gate_up_proj", "d_gate_up_proj_bias", "d_down_proj", "d_down_proj_bias"), grads[2:], acc):
        r = O.rel_l2(a.float().cpu(), b.cpu())
        print("  %s against the sum of the halves: rel_l2 %.2e" % (name, r), flush=True)
        assert r < 1e-2, name
    # spot rows against the oracle
    spot = torch.randint(0, T, (32,), generator=gen, device=gpu)
    d = dict(hidden=x[spot].cpu(), router_indices=idx[spot].cpu(), routing_weights=rw[spot].cpu(),
             gate_up_proj=w[0].cpu(), gate_up_proj_bias=w[1].cpu(), down_proj=w[2].cpu(), down_proj_bias=w[3].cpu())
    assert O.rel_l2(out[spot].cpu(), oracle_forward(d, 32)) < 1e-2
