"""The whole-op entry points of the C ABI driven the way another host would drive them: through ctypes only, with
caller-owned outputs and one caller-owned workspace that is reused from call to call (the sequence a host follows
that replaces torch-ext/torch_binding.cpp:58-83: workspace query, forward, backward).  Results against the oracle."""
import ctypes

import pytest
import torch

from oracle import yamoe_oracle as O
from tests.test_gpu_routing_grad import UNIT, oracle_act, slot_terms
from tests.util import KEYS
from yamoe_amd.workloads import make_inputs

pytestmark = pytest.mark.gpu

NAMES = ("d_hidden", "d_routing", "d_gate_up_proj", "d_gate_up_proj_bias", "d_down_proj", "d_down_proj_bias")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_forward_and_backward_through_ctypes_with_reused_workspace(gpu, dtype):
    from yamoe_amd import _cabi
    lib = _cabi.lib()
    tol = 1e-2 if dtype == torch.bfloat16 else 1e-5
    cd = torch.float32 if dtype == torch.bfloat16 else torch.float64
    big = make_inputs(700, 192, 128, 8, 2, dtype, seed=61, w_std=0.05, bias_std=0.1, zipf=0.8)
    small = make_inputs(90, 192, 128, 8, 2, dtype, seed=62, w_std=0.05, bias_std=0.1)
    # three assignments: the weight-gradient kernel's look-ups of a partial slab run past the end of the row list
    # into whatever the workspace holds
    tiny = make_inputs(3, 192, 128, 8, 1, dtype, seed=64, w_std=0.05, bias_std=0.1)
    # one workspace, sized for the largest call (the backward of the larger problem), poisoned before the first use
    g_big = [big[k].to(gpu) for k in KEYS]
    p = _cabi.problem(g_big[0], g_big[1], g_big[2], g_big[3], 700)
    need_f = lib.yamoe_experts_workspace_bytes(ctypes.byref(p))
    need_b = lib.yamoe_experts_backward_workspace_bytes(ctypes.byref(p))
    assert 0 < need_f < need_b
    ws = torch.full((need_b,), 0xA5, dtype=torch.uint8, device=gpu)
    for label, d, cap in (("big", big, 700), ("small", small, 90), ("big, capacity 50", big, 50), ("tiny", tiny, 3)):
        print("ctypes whole op:", dtype, label, flush=True)
        g = [d[k].to(gpu) for k in KEYS]
        out = torch.full_like(g[0], float("nan"))
        _cabi.experts_forward(*g, cap, workspace=ws, out=out)
        torch.cuda.synchronize()
        want = O.experts_capacity(*[d[k] for k in KEYS], cap, compute_dtype=cd)
        assert O.rel_l2(out.cpu(), want) < tol, label
        gy = torch.randn(d["hidden"].shape, generator=torch.Generator().manual_seed(5)).to(dtype)
        outs = tuple(torch.full_like(t, float("nan")) for t in (g[0], g[2], g[3], g[4], g[5], g[6]))
        _cabi.experts_backward(gy.to(gpu), *g, cap, workspace=ws, outs=outs)
        torch.cuda.synchronize()
        want_g = O.experts_backward(gy, *[d[k] for k in KEYS], cap, compute_dtype=cd)
        for n, a, b in zip(NAMES, outs, want_g):
            if label == "tiny" and n == "d_routing":
                # three entries, each a dot whose terms may cancel: a relative L2 over them means little, so each is
                # held to the forward error bound of its own dot product (the bound of test_gpu_routing_grad.py)
                r = O.route(d["router_indices"].numpy(), d["gate_up_proj"].shape[0], cap)
                want_e, scale, _ = slot_terms(d, gy, oracle_act(d, r["sorted_idx"], 1), r["sorted_idx"], r["inv_pos"])
                got_e = torch.gather(a.cpu().double(), 1, d["router_indices"])
                b64 = O.experts_backward(gy, *[d[k] for k in KEYS], cap, compute_dtype=torch.float64)[1]
                assert torch.allclose(want_e, torch.gather(b64, 1, d["router_indices"]), rtol=1e-9, atol=1e-12)
                u = UNIT[dtype]
                assert torch.all((got_e - want_e).abs() <= 2 * u * scale + 2 * u * want_e.abs() + 1e-30), (label, n)
                continue
            assert O.rel_l2(a.cpu(), b) < tol, (label, n)
    # a workspace one byte short is refused, nothing is launched
    out = torch.zeros_like(g_big[0])
    with pytest.raises(RuntimeError, match="workspace too small"):
        _cabi.experts_forward(*g_big, 700, workspace=ws[:need_f - 1], out=out)
    assert torch.all(out == 0)


def test_stages_through_ctypes_compose_to_the_forward(gpu):
    """yamoe_route -> yamoe_build_schedule -> yamoe_gate_up -> yamoe_down -> yamoe_combine, each through ctypes, give
    the bits of yamoe_experts_forward; the activations and expert rows in between are checked against the oracle."""
    from yamoe_amd import _cabi
    dtype = torch.bfloat16
    T, H, I, E, K = 900, 256, 192, 6, 2
    d = make_inputs(T, H, I, E, K, dtype, seed=63, w_std=0.05, bias_std=0.1, zipf=1.0)
    g = {k: d[k].to(gpu) for k in KEYS}
    se, si, counts, offsets, inv = _cabi.route(g["router_indices"], E, T)
    sched = _cabi.build_schedule(counts, offsets, T * K, T, 16)
    act, pre = _cabi.gate_up(g["hidden"], si, g["gate_up_proj"], g["gate_up_proj_bias"], sched, K, want_pre=True)
    y = _cabi.down(act, g["down_proj"], g["down_proj_bias"], sched)
    out = _cabi.combine(y, inv, g["router_indices"], g["routing_weights"], T, K, E)
    whole = _cabi.experts_forward(*[g[k] for k in KEYS], T)
    torch.cuda.synchronize()
    assert torch.equal(out, whole)
    # the stages against the oracle, row by row in sorted order
    r = O.route(d["router_indices"].numpy(), E, T)
    assert (si.cpu().numpy() == r["sorted_idx"]).all()
    tok = torch.from_numpy(r["sorted_idx"].astype("int64")) // K
    ex = torch.from_numpy(r["sorted_expert"].astype("int64"))
    x = d["hidden"].float()[tok]
    want_pre = torch.stack([x[p] @ d["gate_up_proj"][ex[p]].float() + d["gate_up_proj_bias"][ex[p]].float()
                            for p in range(T * K)])
    assert O.rel_l2(pre.cpu().float(), want_pre) < 1e-2
    want_act = O.glu(want_pre)
    assert O.rel_l2(act.cpu().float(), want_act) < 1e-2
    want_y = torch.stack([want_act[p] @ d["down_proj"][ex[p]].float() + d["down_proj_bias"][ex[p]].float()
                          for p in range(T * K)])
    assert O.rel_l2(y.cpu().float(), want_y) < 1e-2
