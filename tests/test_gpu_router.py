"""The fused router step (linear -> top-k -> softmax -> dense scores) against the oracle, and the Yamoe layer
built on it (torch-ext/yamoe/layers.py:106-218)."""
import numpy as np
import pytest
import torch

from oracle import yamoe_oracle as O
from tests.util import REL_L2_TOL, report

pytestmark = pytest.mark.gpu


def draw(T, H, E, dtype, seed, bias=True):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, H, generator=g).to(dtype)
    w = (torch.randn(E, H, generator=g) / H ** 0.5 * 2).to(dtype)
    b = torch.randn(E, generator=g).to(dtype) if bias else None
    return x, w, b


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("T,H,E,K", [(4096, 2880, 32, 4), (64, 2880, 128, 4), (1, 64, 8, 2), (77, 128, 5, 5), (300, 256, 200, 16),
                                     (33, 48, 33, 1)])
def test_router_topk(gpu, dtype, T, H, E, K):
    from yamoe_amd import _cabi
    print("router", dtype, T, H, E, K, flush=True)
    x, w, b = draw(T, H, E, dtype, T + E, bias=(E != 5))
    idx, scores, topw, logits = _cabi.router_topk(x.to(gpu), w.to(gpu), None if b is None else b.to(gpu), K)
    torch.cuda.synchronize()
    idx, scores, topw, logits = idx.cpu(), scores.cpu(), topw.cpu(), logits.cpu()
    # the linear: fp32 accumulation in another order than the oracle's, so a logit may land one rounding step away
    _, _, want_logits = O.router(x, w, b, K)
    ulp = {torch.bfloat16: 2.0 ** -7, torch.float16: 2.0 ** -10, torch.float32: 2.0 ** -18}[dtype]
    if dtype == torch.float32:
        # nothing is rounded but the fp32 accumulation itself: against the fp64 product, within 2^-20 of the sum of the
        # terms' magnitudes
        want64 = x.double() @ w.double().t() + (b.double() if b is not None else 0.0)
        scale = x.double().abs() @ w.double().abs().t() + (b.double().abs() if b is not None else 0.0)
        assert torch.all((logits.double() - want64).abs() <= 2.0 ** -20 * scale + 1e-30)
    else:
        diff = (logits.float() - want_logits.float()).abs()
        assert torch.all(diff <= ulp * torch.maximum(want_logits.float().abs(), torch.full_like(diff, 2.0 ** -6)) + 1e-6)
        assert (diff > 0).float().mean() < 0.05
    # top-k, softmax and scatter on the kernel's own logits: picks bit-exact (ties included), weights within one rounding step
    want_idx, want_scores = O.router_from_logits(logits, K)
    assert torch.equal(idx, want_idx)
    assert torch.all((scores.float() - want_scores.float()).abs() <= ulp * want_scores.float())
    assert dtype == torch.float32 or (scores != want_scores).float().mean() < 0.01   # (fp32: the last bit of expf)
    assert torch.equal(torch.gather(scores, 1, idx), topw)
    assert torch.equal(scores != 0, torch.zeros_like(scores, dtype=torch.bool).scatter_(1, idx, topw != 0))


def test_router_ties_pick_lower_expert(gpu):
    from yamoe_amd import _cabi
    # identical weight rows give identical logits: the pick order must be by expert id
    T, H, E, K = 40, 64, 16, 4
    g = torch.Generator().manual_seed(1)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    w = torch.randn(1, H, generator=g).to(torch.bfloat16).repeat(E, 1)
    idx, scores, topw, logits = _cabi.router_topk(x.to(gpu), w.to(gpu), None, K)
    torch.cuda.synchronize()
    assert torch.equal(idx.cpu(), torch.arange(K).repeat(T, 1))
    assert torch.all(topw.cpu().float() == 0.25)


def test_router_rejects(gpu):
    import yamoe_amd
    x, w, b = draw(8, 64, 4, torch.bfloat16, 0)
    with pytest.raises(RuntimeError):
        yamoe_amd.router_topk(x.double().to(gpu), w.double().to(gpu), b.double().to(gpu), 2)   # fp64: not taken
    with pytest.raises(RuntimeError):
        yamoe_amd.router_topk(x.to(gpu), w.to(gpu), b.to(gpu), 5)                               # top_k > E
    with pytest.raises(RuntimeError):
        yamoe_amd.router_topk(x[:, :40].contiguous().to(gpu), w[:, :40].contiguous().to(gpu), b.to(gpu), 2)  # H % 16


class Block(torch.nn.Module):
    """The attributes Yamoe.forward expects from its host module."""

    def __init__(self, H, I, E, K, dtype, seed):
        super().__init__()
        g = torch.Generator().manual_seed(seed)

        def p(*shape, std=0.05):
            return torch.nn.Parameter((torch.randn(*shape, generator=g) * std).to(dtype))
        self.router = torch.nn.Module()
        self.router.weight, self.router.bias = p(E, H, std=0.2), p(E, std=0.5)
        self.experts = torch.nn.Module()
        self.experts.gate_up_proj, self.experts.gate_up_proj_bias = p(E, H, 2 * I), p(E, 2 * I, std=0.1)
        self.experts.down_proj, self.experts.down_proj_bias = p(E, I, H), p(E, H, std=0.1)
        self.num_experts, self.top_k = E, K


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_yamoe_layer_forward(gpu, dtype):
    import yamoe_amd
    B, S, H, I, E, K = 2, 96, 128, 64, 8, 2
    blk = Block(H, I, E, K, dtype, 4)
    x = torch.randn(B, S, H, generator=torch.Generator().manual_seed(5)).to(dtype)
    dev = Block(H, I, E, K, dtype, 4).to(gpu)
    with torch.no_grad():
        out, scores = yamoe_amd.Yamoe.forward(dev, x.to(gpu))
    torch.cuda.synchronize()
    out, scores = out.cpu(), scores.cpu()
    assert out.shape == (B, S, H) and scores.shape == (B * S, E)
    # router: a logit one rounding step away may swap two near-equal experts, so compare what survives that: the
    # scores as a whole, then the expert layer on the layer's own routing
    _, want_scores, _ = O.router(x.reshape(-1, H), blk.router.weight.data, blk.router.bias.data, K)
    assert report("router scores", scores.double(), want_scores.double(), 3e-2) < 3e-2
    idx = torch.topk(scores.float(), K, dim=-1).indices
    want = O.experts_capacity(x.reshape(-1, H), idx, scores, blk.experts.gate_up_proj.data, blk.experts.gate_up_proj_bias.data,
                              blk.experts.down_proj.data, blk.experts.down_proj_bias.data, B * S, compute_dtype=torch.float64)
    tol = REL_L2_TOL[dtype]
    assert report("layer", out.reshape(-1, H).double(), want, tol) < tol
    assert (scores != 0).sum(-1).max() <= K


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_yamoe_layer_reference_capacity_and_timing(gpu, dtype):
    """expert_capacity = "reference" is the rule of torch-ext/yamoe/layers.py:161, ceil(tokens * top_k / experts): with
    a skewed router every expert loaded above the mean loses its overflow, as the capacity oracle says; and the stage
    timing of layers.py:118-122, 200-216 fills the same four keys."""
    import yamoe_amd
    B, S, H, I, E, K = 2, 160, 128, 64, 8, 2
    blk = Block(H, I, E, K, dtype, 14)
    with torch.no_grad():
        blk.router.bias.copy_(torch.linspace(2.0, -2.0, E).to(dtype))    # the first experts are picked far more often
    x = torch.randn(B, S, H, generator=torch.Generator().manual_seed(15)).to(dtype)
    dev = Block(H, I, E, K, dtype, 14).to(gpu)
    with torch.no_grad():
        dev.router.bias.copy_(blk.router.bias)
    dev.expert_capacity = "reference"
    dev._timing_enabled = True
    with torch.no_grad():
        out, scores = yamoe_amd.Yamoe.forward(dev, x.to(gpu))
    torch.cuda.synchronize()
    out, scores = out.cpu(), scores.cpu()
    assert set(dev._timing_stats) == {"router", "topk_softmax", "experts_kernel", "total"}
    assert dev._timing_stats["total"] >= dev._timing_stats["experts_kernel"] > 0
    cap = (B * S * K + E - 1) // E
    idx = torch.topk(scores.float(), K, dim=-1).indices
    counts = np.bincount(idx.numpy().ravel(), minlength=E)
    assert counts.max() > cap, "the routing must overflow an expert for this test to mean anything"
    args = (x.reshape(-1, H), idx, scores, blk.experts.gate_up_proj.data, blk.experts.gate_up_proj_bias.data,
            blk.experts.down_proj.data, blk.experts.down_proj_bias.data)
    want = O.experts_capacity(*args, cap, compute_dtype=torch.float64)
    tol = REL_L2_TOL[dtype]
    assert report("layer, reference capacity", out.reshape(-1, H).double(), want, tol) < tol
    full = O.experts_capacity(*args, B * S, compute_dtype=torch.float64)
    assert O.rel_l2(want, full) > 0.05        # and dropping changes the answer
    dev.expert_capacity = None
    dev._timing_enabled = False
    with torch.no_grad():
        out2, _ = yamoe_amd.Yamoe.forward(dev, x.to(gpu))
    assert report("layer, no drop", out2.cpu().reshape(-1, H).double(), full, tol) < tol


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_yamoe_layer_trains_the_router(gpu, dtype):
    """enable_router_grads = True survives the call (the reference resets it, torch-ext/yamoe/layers.py:110, so its
    router never trains) and loss.backward() through the layer reaches the router's weight and bias, the hidden
    states and the expert parameters with the gradients autograd gives through the oracle's router step and expert
    layer on the layer's own picks."""
    import yamoe_amd
    B, S, H, I, E, K = 2, 96, 128, 64, 8, 2
    blk = Block(H, I, E, K, dtype, 24)
    x = torch.randn(B, S, H, generator=torch.Generator().manual_seed(25)).to(dtype)
    gy = torch.randn(B, S, H, generator=torch.Generator().manual_seed(26)).to(dtype)
    dev = Block(H, I, E, K, dtype, 24).to(gpu)
    dev.enable_router_grads = True
    xd = x.to(gpu).requires_grad_(True)
    out, scores = yamoe_amd.Yamoe.forward(dev, xd)
    assert dev.enable_router_grads is True
    assert out.requires_grad and scores.requires_grad
    (out * gy.to(gpu)).sum().backward()
    torch.cuda.synchronize()
    picks = torch.topk(scores.detach().float().cpu(), K, dim=-1).indices
    cd = torch.float64 if dtype == torch.float32 else torch.float32
    params = [blk.router.weight, blk.router.bias, blk.experts.gate_up_proj, blk.experts.gate_up_proj_bias,
              blk.experts.down_proj, blk.experts.down_proj_bias]
    leaves = [t.detach().to(cd).requires_grad_(True) for t in [x.reshape(-1, H)] + [p.data for p in params]]
    _, want_scores, _ = O.router(leaves[0], leaves[1], leaves[2], K, compute_dtype=cd, picks=picks)
    want_out = O.experts_capacity(leaves[0], picks, want_scores, *leaves[3:], B * S, compute_dtype=cd)
    want = torch.autograd.grad(want_out, leaves, gy.reshape(-1, H).to(cd))
    tol = REL_L2_TOL[dtype] if dtype == torch.float32 else 2e-2   # bf16: scores and logits are rounded along the chain
    assert report("layer out", out.detach().cpu().reshape(-1, H).double(), want_out.detach(), tol) < tol
    got = [xd.grad.reshape(-1, H), dev.router.weight.grad, dev.router.bias.grad, dev.experts.gate_up_proj.grad,
           dev.experts.gate_up_proj_bias.grad, dev.experts.down_proj.grad, dev.experts.down_proj_bias.grad]
    names = ("d_hidden", "d_router_weight", "d_router_bias", "d_gate_up_proj", "d_gate_up_proj_bias", "d_down_proj",
             "d_down_proj_bias")
    for n, a, b in zip(names, got, want):
        assert a is not None, n
        assert report("router training " + n, a.cpu().double(), b.double(), tol) < tol, n


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,H,E,K", [(4096, 2880, 32, 4), (300, 256, 128, 4), (5, 64, 8, 2), (1000, 320, 40, 3), (20, 64, 16, 16)])
def test_router_backward(gpu, dtype, T, H, E, K):
    """yamoe_router_backward against autograd through the oracle's router step on the kernel's own picks: gradients of
    hidden states, router weight and router bias from a random gradient of the dense scores (torch-ext/yamoe/layers.py:
    128-149 differentiated)."""
    from yamoe_amd import _cabi
    print("router backward", dtype, T, H, E, K, flush=True)
    x, w, b = draw(T, H, E, dtype, 3 * T + E)
    idx, scores, _, _ = _cabi.router_topk(x.to(gpu), w.to(gpu), b.to(gpu), K)
    g = torch.randn(T, E, generator=torch.Generator().manual_seed(T)).to(dtype)
    d_x, d_w, d_b = _cabi.router_backward(g.to(gpu), idx, scores, x.to(gpu), w.to(gpu), K)
    torch.cuda.synchronize()
    cd = torch.float64 if dtype == torch.float32 else torch.float32
    leaves = [t.to(cd).requires_grad_(True) for t in (x, w, b)]
    _, want_scores, _ = O.router(*leaves, K, compute_dtype=cd, picks=idx.cpu())
    want = torch.autograd.grad(want_scores, leaves, g.to(cd))
    tol = 1e-5 if dtype == torch.float32 else 2e-2   # 16-bit: d_logits and the stored scores are rounded on the way
    for name, got, ref in zip(("d_hidden", "d_weight", "d_bias"), (d_x, d_w, d_b), want):
        assert report("router backward " + name, got.cpu().double(), ref.double(), tol) < tol, name
    # only the picked experts carry a gradient: with d_scores zero at the picks everything vanishes
    g0 = g.clone().scatter_(1, idx.cpu(), 0.0)
    z_x, z_w, z_b = _cabi.router_backward(g0.to(gpu), idx, scores, x.to(gpu), w.to(gpu), K)
    torch.cuda.synchronize()
    assert float(z_x.abs().max()) == 0 and float(z_w.abs().max()) == 0 and float(z_b.abs().max()) == 0
