"""experts_backward through the torch op against autograd through the CPU oracle."""
import pytest
import torch

from oracle import yamoe_oracle as O
from tests.util import args, to_dev
from yamoe_amd.workloads import make_config, make_inputs

pytestmark = pytest.mark.gpu

NAMES = ("d_hidden", "d_routing", "d_gate_up_proj", "d_gate_up_proj_bias", "d_down_proj", "d_down_proj_bias")
TOL = {torch.float32: 1e-5, torch.bfloat16: 1e-2, torch.float16: 1e-2}


def run_bwd(d, gy, capacity, gpu):
    import yamoe_amd
    g = to_dev(d, gpu)
    E, K = d["gate_up_proj"].shape[0], d["router_indices"].shape[1]
    grads = yamoe_amd.experts_backward(gy.to(gpu), *args(g), capacity, E, K)
    torch.cuda.synchronize()
    return [t.cpu() for t in grads]


def check(grads, want, dtype, label):
    for n, a, b in zip(NAMES, grads, want):
        assert a.shape == b.shape, (n, a.shape, b.shape)
        r, m = O.rel_l2(a, b), O.max_abs(a, b)
        print("%s %s: rel_l2=%.3e max_abs=%.3e" % (label, n, r, m), flush=True)
        assert r < TOL[dtype], (n, r)


SMALL = [
    (40, 64, 64, 4, 2),       # few rows per expert
    (700, 64, 96, 3, 2),      # > 256 rows per expert, I != H
    (513, 264, 136, 5, 3),    # ragged everything
    (300, 520, 64, 16, 2),    # some empty experts (zipf)
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,H,I,E,K", SMALL)
def test_backward_small(gpu, dtype, T, H, I, E, K):
    print("backward_small", dtype, T, H, I, E, K, flush=True)
    d = make_inputs(T, H, I, E, K, dtype, seed=T, w_std=0.05, bias_std=0.1, zipf=1.5 if E >= 16 else 0.0)
    gy = torch.randn(T, H, generator=torch.Generator().manual_seed(2)).to(dtype)
    grads = run_bwd(d, gy, T, gpu)
    want = O.experts_backward(gy, *args(d), T, compute_dtype=torch.float64 if dtype == torch.float32 else torch.float32)
    check(grads, want, dtype, "small")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("capacity", [200, 37, 600])
def test_backward_capacity_16bit(gpu, dtype, capacity):
    """Dropped assignments on the 16-bit kernels: the weight-gradient contraction stops at the capacity (200 rows: a
    partial last slab on the pipelined path; 37: the short path), the input-gradient GEMM gathers grad_out by token
    only for kept rows, dropped slots get a zero routing gradient."""
    T, H, I, E, K = 600, 128, 64, 4, 2
    d = make_inputs(T, H, I, E, K, dtype, seed=9, w_std=0.05, bias_std=0.1, zipf=0.5)
    gy = torch.randn(T, H, generator=torch.Generator().manual_seed(3)).to(dtype)
    grads = run_bwd(d, gy, capacity, gpu)
    want = O.experts_backward(gy, *args(d), capacity, compute_dtype=torch.float32)
    check(grads, want, dtype, "capacity %d" % capacity)
    r = O.route(d["router_indices"], E, capacity)
    dropped = torch.from_numpy(r["inv_pos"].reshape(T, K) < 0)
    d_routing = grads[1].cpu()
    assert torch.all(torch.gather(d_routing, 1, d["router_indices"])[dropped] == 0)


@pytest.mark.parametrize("H,I", [(512, 256), (640, 320), (768, 384), (896, 192), (384, 448), (128, 128)])
def test_backward_contraction_lengths_16bit(gpu, H, I):
    """The input-gradient GEMMs contract over H (down) and 2I (gate_up): 2 to 14 slab pairs of 64, which covers the
    shortest contraction the pipelined loop takes (4 pairs), odd and even pair counts (the three pair buffers of the
    [n][k] weights rotate) and the short path below 4 pairs.  Rows per expert above 256, so that full tiles run."""
    dtype = torch.bfloat16
    T, E, K = 640, 2, 1
    d = make_inputs(T, H, I, E, K, dtype, seed=H + I, w_std=0.05, bias_std=0.1)
    gy = torch.randn(T, H, generator=torch.Generator().manual_seed(7)).to(dtype)
    grads = run_bwd(d, gy, T, gpu)
    want = O.experts_backward(gy, *args(d), T, compute_dtype=torch.float32)
    check(grads, want, dtype, "contraction H=%d I=%d" % (H, I))


@pytest.mark.parametrize("rows", [180, 250])
def test_backward_partial_column_tiles_16bit(gpu, rows):
    """As the forward test of the same name: output widths of 576 (64 columns in the last tile) for both input
    gradients, 640 for the recomputed gate_up, on tiles of six and eight row blocks."""
    dtype = torch.bfloat16
    T, H, I, E, K = 2 * rows, 576, 576, 2, 1
    d = make_inputs(T, H, I, E, K, dtype, seed=rows, w_std=0.05, bias_std=0.1)
    d["router_indices"] = (torch.arange(T) % E).reshape(T, 1)
    gy = torch.randn(T, H, generator=torch.Generator().manual_seed(8)).to(dtype)
    grads = run_bwd(d, gy, T, gpu)
    want = O.experts_backward(gy, *args(d), T, compute_dtype=torch.float32)
    check(grads, want, dtype, "partial column tiles rows=%d" % rows)


@pytest.mark.parametrize("slot_weights", [False, True])
def test_backward_capacity_and_layouts(gpu, slot_weights):
    dtype = torch.float32
    T, H, I, E, K = 200, 64, 64, 4, 2
    d = make_inputs(T, H, I, E, K, dtype, seed=5, w_std=0.05, bias_std=0.1, zipf=1.0)
    if slot_weights:
        d["routing_weights"] = torch.gather(d["routing_weights"], 1, d["router_indices"])
    gy = torch.randn(T, H, generator=torch.Generator().manual_seed(3))
    for C in (30, 0):
        grads = run_bwd(d, gy, C, gpu)
        want = O.experts_backward(gy, *args(d), C, compute_dtype=torch.float64)
        if C == 0:
            assert all(torch.all(g == 0) for g in grads)
        else:
            check(grads, want, dtype, "cap%d" % C)
    # the routing gradient is zero outside the selected experts
    if not slot_weights:
        d_rw = run_bwd(d, gy, T, gpu)[1]
        sel = torch.zeros_like(d_rw, dtype=torch.bool).scatter_(1, d["router_indices"], True)
        assert torch.all(d_rw[~sel] == 0)


def test_autograd_function_matches_op(gpu):
    """_ExpertsFn wires the six gradients to the right inputs (torch-ext/yamoe/layers.py:50-100)."""
    import yamoe_amd
    T, H, I, E, K = 64, 64, 64, 4, 2
    d = to_dev(make_inputs(T, H, I, E, K, torch.float32, seed=9, w_std=0.05, bias_std=0.1), gpu)
    leaves = {k: d[k].clone().requires_grad_(True) for k in
              ("hidden", "routing_weights", "gate_up_proj", "gate_up_proj_bias", "down_proj", "down_proj_bias")}
    out = yamoe_amd.experts_autograd(leaves["hidden"], d["router_indices"], leaves["routing_weights"],
                                     leaves["gate_up_proj"], leaves["gate_up_proj_bias"], leaves["down_proj"],
                                     leaves["down_proj_bias"], T, E, K, True)
    gy = torch.randn_like(out)
    out.backward(gy)
    direct = yamoe_amd.experts_backward(gy, *args(d), T, E, K)
    for (k, leaf), g in zip(leaves.items(), direct):
        assert torch.equal(leaf.grad, g), k


def test_backward_gptoss20b_full(gpu):
    """Backward at the GPT-OSS-20B shape, bf16, against fp32 autograd through the oracle."""
    d, c = make_config("gptoss20b", seed=0)
    gy = torch.randn(c["T"], c["H"], generator=torch.Generator().manual_seed(4)).to(torch.bfloat16)
    grads = run_bwd(d, gy, c["T"], gpu)
    want = O.experts_backward(gy, *args(d), c["T"], compute_dtype=torch.float32)
    check(grads, want, torch.bfloat16, "gptoss20b")


CLAMPED = [
    # dtype, T, H, I, E, K, weight std: pre-activations of std 3 to 8, a good part of them beyond the clamp at 7
    (torch.bfloat16, 700, 256, 128, 4, 2, 0.5),    # asynchronous-copy kernels
    (torch.float16, 700, 256, 128, 4, 2, 0.5),
    (torch.bfloat16, 64, 200, 72, 4, 2, 0.4),      # register-staged kernels (contraction not a multiple of 64)
    (torch.bfloat16, 600, 2880, 512, 2, 1, 0.05),  # the GPT-OSS width, where sqrt(2880) * 0.05 does the same
]


@pytest.mark.parametrize("dtype,T,H,I,E,K,w_std", CLAMPED)
def test_backward_pre_activations_near_the_clamp(gpu, dtype, T, H, I, E, K, w_std):
    """The backward reads the pre-activations back in the activation dtype and tests them against the clamp limit
    (csrc/experts_backward.cu:285-299).  A value just beyond the limit that rounds onto it (bf16: anything in
    (7, 7.016]) must still count as clamped, as it does in the forward and in the oracle's fp32: with plain rounding
    d_hidden and the gate_up gradients of these cases are off by 1.2e-2 to 5e-2, a few elements each wrong by its
    whole size."""
    print("backward_clamp", dtype, T, H, I, E, K, w_std, flush=True)
    d = make_inputs(T, H, I, E, K, dtype, seed=T + H, w_std=w_std, bias_std=0.1)
    gy = torch.randn(T, H, generator=torch.Generator().manual_seed(4)).to(dtype)
    grads = run_bwd(d, gy, T, gpu)
    want = O.experts_backward(gy, *args(d), T, compute_dtype=torch.float32)
    check(grads, want, dtype, "clamp")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T", [300, 5])
def test_stored_pre_activations_keep_the_clamp_decision(gpu, dtype, T):
    """yamoe_gate_up's optional pre-activation output: |value| > 7 in fp32 is never stored as exactly 7 (tile kernels
    for T = 300, streaming kernel for T = 5), values within the limit are the plain rounding."""
    from yamoe_amd import _cabi
    H, I, E, K = 128, 64, 4, 2
    d = make_inputs(T, H, I, E, K, dtype, seed=31, w_std=0.6, bias_std=0.1)
    g = to_dev(d, gpu)
    se, si, counts, offsets, inv = _cabi.route(g["router_indices"], E, T)
    sched = _cabi.build_schedule(counts, offsets, T * K, T, 16)
    act, pre = _cabi.gate_up(g["hidden"], si, g["gate_up_proj"], g["gate_up_proj_bias"], sched, K, want_pre=True)
    torch.cuda.synchronize()
    tok = si.cpu().long() // K
    e = d["router_indices"].reshape(-1)[si.cpu().long()]
    x = d["hidden"].double()[tok]
    want = torch.stack([x[p] @ d["gate_up_proj"][int(e[p])].double() + d["gate_up_proj_bias"][int(e[p])].double()
                        for p in range(T * K)])
    got = pre.cpu().double()
    gate_w, up_w, gate_g, up_g = want[:, 0::2], want[:, 1::2], got[:, 0::2], got[:, 1::2]
    margin = 0.02  # (fp32 accumulation against fp64: leave the values this close to the limit out)
    assert int((gate_w > 7 + margin).sum()) > 50 and int((up_w.abs() > 7 + margin).sum()) > 50
    assert torch.all(gate_g[gate_w > 7 + margin] > 7)
    assert torch.all(up_g[up_w.abs() > 7 + margin].abs() > 7)
    assert torch.all(gate_g[gate_w < 7 - margin] <= 7) and torch.all(up_g[up_w.abs() < 7 - margin].abs() <= 7)
    inside = want.abs() < 6.9
    assert float((got[inside] - want[inside]).abs().max()) < 0.04  # (within a rounding step of the fp64 value)


def test_backward_fp32_pre_activation_on_the_clamp_boundary(gpu):
    """The gradient of the clamp jumps at +-7 (csrc/experts_backward.cu:285-299), so a pre-activation within fp32
    accumulation error of the limit may fall on one side on the GPU and on the other in the oracle's fp64.  This seeded
    case has exactly one such value among its 1.2 million (an up value of -6.9999988 in fp64).  What the contract allows
    there: the forward still agrees to 1e-5; gradients that do not pass through the clamp agree to 1e-5; the others
    agree to 1e-5 everywhere except in the entries that one pre-activation feeds (its token's row of d_hidden, its
    column of the expert's d_gate_up_proj and d_gate_up_proj_bias), and to 5e-3 with those entries counted."""
    import numpy as np
    import yamoe_amd
    T, H, I, E, K, cap = 1025, 280, 240, 7, 5, 366
    d = make_inputs(T, H, I, E, K, torch.float32, seed=1005, w_std=1.0, bias_std=0.1, zipf=1.2)
    d["routing_weights"] = torch.gather(d["routing_weights"], 1, d["router_indices"])
    gy = torch.randn(T, H, generator=torch.Generator().manual_seed(6))
    g = to_dev(d, gpu)
    out = yamoe_amd.experts(*args(g), cap, E, K)
    grads = run_bwd(d, gy, cap, gpu)
    want_out = O.experts_capacity(*args(d), cap, compute_dtype=torch.float64)
    want = O.experts_backward(gy, *args(d), cap, compute_dtype=torch.float64)
    assert O.rel_l2(out.cpu(), want_out) < 1e-5
    # the pre-activations of the kept rows in fp64 that lie within 2e-5 of a clamp limit
    r = O.route(d["router_indices"].numpy(), E, cap)
    x, W, Bs = d["hidden"].double(), d["gate_up_proj"].double(), d["gate_up_proj_bias"].double()
    near = []
    for e in range(E):
        kept, first = min(int(r["counts"][e]), cap), int(r["offsets"][e])
        toks = torch.from_numpy(r["sorted_idx"][first:first + kept].astype(np.int64)) // K
        pre = x[toks] @ W[e] + Bs[e]
        close = (pre.abs() - 7).abs() < 2e-5
        close[:, 0::2] &= pre[:, 0::2] > 0            # the gate half is clamped from above only
        near += [(e, int(toks[i]), int(c)) for i, c in close.nonzero().tolist()]
    print("pre-activations on the boundary:", near, flush=True)
    assert len(near) == 1
    e, tok, col = near[0]
    rel = {n: O.rel_l2(a, b) for n, a, b in zip(NAMES, grads, want)}
    print({n: "%.2e" % v for n, v in rel.items()}, flush=True)
    for n in ("d_routing", "d_down_proj", "d_down_proj_bias"):
        assert rel[n] < 1e-5, (n, rel[n])
    fed = {"d_hidden": (tok, slice(None)), "d_gate_up_proj": (e, slice(None), col), "d_gate_up_proj_bias": (e, col)}
    for n, where in fed.items():
        a, b = grads[NAMES.index(n)].clone().double(), want[NAMES.index(n)].double()
        assert rel[n] < 5e-3, (n, rel[n])
        a[where] = b[where]
        assert O.rel_l2(a, b) < 1e-5, (n, "outside the entries fed by the boundary value", O.rel_l2(a, b))
