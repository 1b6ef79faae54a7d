"""Pins the CPU oracle (oracle/yamoe_oracle.py) against things that do not share its code:
brute force, library routines, closed-form special cases, finite differences and a hand-made
known-answer fixture.  The reference ships no fixtures for this path, so these are the anchors."""
import json
import math
import os

import numpy as np
import pytest
import torch

from oracle import yamoe_oracle as O
from yamoe_amd.workloads import make_inputs

HERE = os.path.dirname(os.path.abspath(__file__))


# ---- routing ---------------------------------------------------------------------------------------
def brute_route(ids, E, C):
    """O(N^2) definition: position = #(smaller keys) + #(equal keys at lower index)."""
    N = len(ids)
    key = [E if (v < 0 or v >= E) else v for v in ids]
    pos = [sum(1 for j in range(N) if key[j] < key[i] or (key[j] == key[i] and j < i)) for i in range(N)]
    sorted_idx = [0] * N
    for i, p in enumerate(pos):
        sorted_idx[p] = i
    counts = [sum(1 for k in key if k == e) for e in range(E)]
    inv = []
    for i in range(N):
        rank = sum(1 for j in range(i) if key[j] == key[i])
        inv.append(pos[i] if key[i] < E and rank < C else -1)
    return sorted_idx, counts, inv


@pytest.mark.parametrize("N,E,C,seed", [(1, 1, 1, 0), (17, 3, 100, 1), (64, 8, 5, 2), (200, 130, 2, 3), (97, 5, 0, 4)])
def test_route_matches_brute_force(N, E, C, seed):
    rng = np.random.default_rng(seed)
    ids = rng.integers(0, E, size=N)
    if N > 10:
        ids[3] = -1  # invalid ids sort last and are dropped
        ids[7] = E + 2
    r = O.route(ids, E, C)
    sidx, counts, inv = brute_route(ids.tolist(), E, C)
    assert r["sorted_idx"].tolist() == sidx
    assert r["counts"].tolist() == counts
    assert r["inv_pos"].tolist() == inv
    assert r["offsets"].tolist() == [0] + np.cumsum(counts).tolist()
    assert r["bins"].tolist() == np.cumsum(counts).tolist()
    assert r["sorted_expert"].tolist() == ids[np.array(sidx, dtype=np.int64)].tolist() if N else True


def test_route_invariants_large():
    rng = np.random.default_rng(5)
    ids = rng.integers(0, 128, size=65536)
    r = O.route(ids, 128, 700)
    assert sorted(r["sorted_idx"].tolist()) == list(range(65536))
    se = r["sorted_expert"]
    assert np.all(se[1:] >= se[:-1])
    same = se[1:] == se[:-1]
    assert np.all(r["sorted_idx"][1:][same] > r["sorted_idx"][:-1][same])  # stability
    kept = r["inv_pos"] >= 0
    assert kept.sum() == np.minimum(r["counts"], 700).sum()
    assert np.all(r["sorted_idx"][r["inv_pos"][kept]] == np.nonzero(kept)[0])


def test_route_empty():
    r = O.route(np.zeros(0, dtype=np.int64), 4, 3)
    assert r["counts"].tolist() == [0, 0, 0, 0] and r["offsets"].tolist() == [0] * 5


# ---- GLU ---------------------------------------------------------------------------------------------
def test_glu_known_answers():
    with open(os.path.join(HERE, "golden", "glu_kat.json")) as f:
        kat = json.load(f)
    gu = torch.tensor([[c["G"], c["U"]] for c in kat], dtype=torch.float64)
    got = O.glu(gu)[:, 0]
    want = torch.tensor([c["h"] for c in kat], dtype=torch.float64)
    assert torch.allclose(got, want, rtol=1e-12, atol=1e-15)


def test_glu_uses_even_gate_odd_up():
    gu = torch.tensor([[2.0, -1.0, 0.0, 5.0]], dtype=torch.float64)  # pairs (G=2,U=-1), (G=0,U=5)
    assert O.glu(gu).tolist() == [[0.0, 0.0]]  # U=-1 kills the first, G=0 the second
    gu = torch.tensor([[-1.0, 2.0]], dtype=torch.float64)  # swapped roles would give 0
    assert O.glu(gu)[0, 0].item() != 0.0


# ---- forward -------------------------------------------------------------------------------------------
def tiny(seed=0, T=24, H=16, I=12, E=4, K=2, dtype=torch.float64, **kw):
    d = make_inputs(T, H, I, E, K, torch.float32, seed=seed, w_std=0.3, bias_std=0.2, **kw)
    return {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in d.items()}


def args(d):
    return (d["hidden"], d["router_indices"], d["routing_weights"], d["gate_up_proj"], d["gate_up_proj_bias"],
            d["down_proj"], d["down_proj_bias"])


@pytest.mark.parametrize("seed", [0, 1])
def test_loop_equals_dense_formulation(seed):
    d = tiny(seed)
    a = O.experts_loop(*args(d))
    b = O.experts_dense(d["hidden"], d["routing_weights"], d["gate_up_proj"], d["gate_up_proj_bias"],
                        d["down_proj"], d["down_proj_bias"])
    assert O.rel_l2(a, b) < 1e-13


def test_single_expert_is_one_mlp():
    d = tiny(2, E=1, K=1)
    x = d["hidden"]
    gu = x @ d["gate_up_proj"][0] + d["gate_up_proj_bias"][0]
    G, U = gu[:, 0::2], gu[:, 1::2]
    h = (U.clamp(-7, 7) + 1) * torch.minimum(G, torch.tensor(7.0, dtype=G.dtype)) * \
        torch.sigmoid(1.702 * torch.minimum(G, torch.tensor(7.0, dtype=G.dtype)))
    want = (h @ d["down_proj"][0] + d["down_proj_bias"][0]) * d["routing_weights"][:, :1]
    assert O.rel_l2(O.experts_loop(*args(d)), want) < 1e-13


def test_zero_weights_reduce_to_bias_closed_form():
    d = tiny(3)
    d["gate_up_proj"].zero_()
    out = O.experts_loop(*args(d))
    # every token of expert e gets the same vector f(bgu[e]) @ Wd[e] + bd[e]
    E = d["gate_up_proj"].shape[0]
    per_e = torch.stack([O.glu(d["gate_up_proj_bias"][e][None])[0] @ d["down_proj"][e] + d["down_proj_bias"][e]
                         for e in range(E)])
    want = d["routing_weights"] @ per_e
    assert O.rel_l2(out, want) < 1e-13


def test_interleaved_identity_weights_copy_rows():
    # Wgu[e][:, 2j] = Wgu[e][:, 2j+1] = unit vector j  =>  G = U = x, so act = glu applied to (x, x)
    d = tiny(4, H=8, I=8)
    E, H, _ = d["gate_up_proj"].shape
    w = torch.zeros_like(d["gate_up_proj"])
    for j in range(H):
        w[:, j, 2 * j] = 1
        w[:, j, 2 * j + 1] = 1
    d["gate_up_proj"], d["gate_up_proj_bias"] = w, torch.zeros_like(d["gate_up_proj_bias"])
    d["down_proj"] = torch.eye(H, dtype=w.dtype).repeat(E, 1, 1)
    d["down_proj_bias"].zero_()
    x = d["hidden"]
    g = x.clamp(max=7)
    act = (x.clamp(-7, 7) + 1) * g * torch.sigmoid(1.702 * g)
    want = act * d["routing_weights"].sum(1, keepdim=True)
    assert O.rel_l2(O.experts_loop(*args(d)), want) < 1e-13


def test_linear_in_routing_weights():
    d = tiny(5)
    a = O.experts_loop(*args(d))
    d2 = dict(d)
    d2["routing_weights"] = d["routing_weights"] * 3.0
    assert O.rel_l2(O.experts_loop(*args(d2)), 3.0 * a) < 1e-13


def brute_capacity(d, C):
    """Per-slot loops following binned_gather / binned_scatter (yamoe_ref.py:4-35)."""
    x, idx, rw = d["hidden"], d["router_indices"], d["routing_weights"]
    T, K = idx.shape
    E = rw.shape[1]
    out = torch.zeros_like(x)
    seen = [0] * E
    order = sorted(range(T * K), key=lambda f: (int(idx.view(-1)[f]), f))
    for f in order:
        e = int(idx.view(-1)[f])
        if seen[e] >= C:
            continue
        seen[e] += 1
        t = f // K
        gu = x[t] @ d["gate_up_proj"][e] + d["gate_up_proj_bias"][e]
        y = O.glu(gu[None])[0] @ d["down_proj"][e] + d["down_proj_bias"][e]
        out[t] += y * rw[t, e]
    return out


@pytest.mark.parametrize("C", [0, 1, 5, 1000])
def test_capacity_matches_brute_force(C):
    d = tiny(6)
    got = O.experts_capacity(*args(d), C)
    want = brute_capacity(d, C)
    assert O.max_abs(got, want) < 1e-12


def test_capacity_large_equals_loop_and_slot_weights():
    d = tiny(7)
    a = O.experts_capacity(*args(d), 10 ** 6)
    assert O.rel_l2(a, O.experts_loop(*args(d))) < 1e-13
    sel = torch.gather(d["routing_weights"], 1, d["router_indices"])  # [T,K] layout gives the same result
    b = O.experts_capacity(d["hidden"], d["router_indices"], sel, d["gate_up_proj"], d["gate_up_proj_bias"],
                           d["down_proj"], d["down_proj_bias"], 10 ** 6)
    assert O.rel_l2(b, a) < 1e-13


# ---- backward ------------------------------------------------------------------------------------------
def test_backward_gradcheck_fp64():
    d = tiny(8, T=6, H=8, I=4, E=3, K=2)
    idx = d["router_indices"]
    leaves = [d[k].clone().requires_grad_(True) for k in
              ("hidden", "routing_weights", "gate_up_proj", "gate_up_proj_bias", "down_proj", "down_proj_bias")]

    def f(h, rw, wgu, bgu, wd, bd):
        return O.experts_capacity(h, idx, rw, wgu, bgu, wd, bd, 3)

    assert torch.autograd.gradcheck(f, leaves, eps=1e-6, atol=1e-6, rtol=1e-4)


@pytest.mark.parametrize("C,slot_weights", [(1000, False), (4, False), (1000, True)])
def test_backward_closed_form_equals_autograd(C, slot_weights):
    d = tiny(9)
    if slot_weights:
        d["routing_weights"] = torch.gather(d["routing_weights"], 1, d["router_indices"])
    gy = torch.randn(d["hidden"].shape, dtype=torch.float64, generator=torch.Generator().manual_seed(1))
    a = O.experts_backward(gy, *args(d), C, compute_dtype=torch.float64)
    b = O.experts_backward_closed(gy, *args(d), C)
    for ga, gb in zip(a, b):
        assert ga.shape == gb.shape
        assert O.max_abs(ga, gb) < 1e-10


def test_backward_routing_grad_is_zero_outside_selection():
    d = tiny(10)
    gy = torch.ones_like(d["hidden"])
    d_rw = O.experts_backward(gy, *args(d), 1000, compute_dtype=torch.float64)[1]
    sel = torch.zeros_like(d_rw, dtype=torch.bool).scatter_(1, d["router_indices"], True)
    assert torch.all(d_rw[~sel] == 0)
    assert torch.any(d_rw[sel] != 0)


# ---- helper ops on the padded layout ---------------------------------------------------------------------
def test_sort_pairs_two_complement_cases_by_hand():
    x = np.array([3, -1, 0, -128, 3, 127], dtype=np.int16)
    k, p = O.sort_pairs(x, 16)                  # full width: signed order, ties in input order
    assert k.tolist() == [-128, -1, 0, 3, 3, 127] and p.tolist() == [3, 1, 2, 0, 4, 5]
    # low 3 bits only: 3->3, -1->7, 0->0, -128->0, 3->3, 127->7
    k, p = O.sort_pairs(x, 3)
    assert p.tolist() == [2, 3, 0, 4, 1, 5] and k.tolist() == [0, -128, 3, 3, -1, 127]
    k, p = O.sort_pairs(x, 0)                   # no bits: nothing moves
    assert p.tolist() == [0, 1, 2, 3, 4, 5]


@pytest.mark.parametrize("dt", [np.int16, np.int32, np.int64])
def test_sort_pairs_invariants(dt):
    rng = np.random.default_rng(5)
    info = np.iinfo(dt)
    x = rng.integers(info.min, info.max, size=3000, dtype=dt, endpoint=True)
    x[:50] = x[50:100]                           # ties
    k, p = O.sort_pairs(x, info.bits)
    assert np.all(np.diff(k.astype(object)) >= 0)
    assert np.array_equal(x[p.astype(np.int64)], k) and np.array_equal(k, np.sort(x))
    same = k[1:] == k[:-1]
    assert np.all(p[1:][same] > p[:-1][same])    # stable


def test_bincount_cumsum_by_hand():
    out = O.bincount_cumsum([2, 0, 2, 5, -1, 2, 9], out_len=8, minlength=6)
    assert out.tolist() == [1, 1, 4, 4, 4, 5, 0, 0]


@pytest.mark.parametrize("C", [3, 64])
def test_padded_helpers_compose_to_the_expert_op(C):
    """sort -> bincount_cumsum -> gather -> batch_mm -> glu -> batch_mm -> scatter is the reference's
    own composition (torch-ext/yamoe/vendored/yamoe_ref.py:31-70) and must give the op's result."""
    d = tiny(seed=4, T=40, E=5, K=3)
    T, K = d["router_indices"].shape
    E, H = 5, d["hidden"].shape[1]
    flat = d["router_indices"].reshape(-1).numpy().astype(np.int32)
    keys, pos = O.sort_pairs(flat, 32)
    bins = O.bincount_cumsum(keys, E, E)
    x = O.padded_gather(d["hidden"], pos, bins, E, C, K)
    # padding rows are zero
    for e in range(E):
        n = bins[e] - (bins[e - 1] if e else 0)
        assert torch.all(x[e, min(n, C):] == 0)
    gu = O.batch_mm(x, d["gate_up_proj"]) + d["gate_up_proj_bias"][:, None, :]
    y = O.batch_mm(O.glu(gu), d["down_proj"]) + d["down_proj_bias"][:, None, :]
    w_sorted = O.index_select(d["routing_weights"].gather(1, d["router_indices"]).reshape(-1), torch.from_numpy(pos))
    out = O.padded_scatter(y, pos, bins, w_sorted, torch.zeros(T, H, dtype=torch.float64), T, E, C, K)
    want = O.experts_capacity(*args(d), C, compute_dtype=torch.float64)
    assert O.rel_l2(out, want) < 1e-12


def test_gather_then_plain_scatter_counts_kept_slots():
    d = tiny(seed=6, T=30, E=4, K=2)
    T, K, E, C = 30, 2, 4, 9
    flat = d["router_indices"].reshape(-1).numpy().astype(np.int32)
    keys, pos = O.sort_pairs(flat, 32)
    bins = O.bincount_cumsum(keys, E, E)
    x = O.padded_gather(d["hidden"], pos, bins, E, C, K)
    y0 = torch.ones(T, d["hidden"].shape[1], dtype=torch.float64)
    out = O.padded_scatter(x, pos, bins, None, y0, T, E, C, K)
    r = O.route(d["router_indices"], E, C)
    kept = np.zeros(T)
    for p_sorted, f in enumerate(r["sorted_idx"]):
        e = r["sorted_expert"][p_sorted]
        if 0 <= e < E and p_sorted - r["offsets"][e] < C:
            kept[f // K] += 1
    want = y0 + d["hidden"] * torch.from_numpy(kept)[:, None]
    assert O.rel_l2(out, want) < 1e-14


# ---- router step -----------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_router_from_logits_brute_force(dtype):
    g = torch.Generator().manual_seed(9)
    T, E, K = 50, 12, 4
    logits = (torch.randn(T, E, generator=g) * 2).to(dtype)
    logits[:, 3] = logits[:, 7]                       # ties in every row
    logits[5] = 0.25                                  # a row of all-equal logits: picks 0, 1, 2, 3
    idx, scores = O.router_from_logits(logits, K)
    for t in range(T):
        row = [float(v) for v in logits[t]]
        picked = []
        for _ in range(K):
            best = None
            for e in range(E):
                if e not in picked and (best is None or row[e] > row[best]):
                    best = e
            picked.append(best)
        assert idx[t].tolist() == picked
        ex = [math.exp(row[e] - row[picked[0]]) for e in picked]
        for k, e in enumerate(picked):
            want = torch.tensor(ex[k] / sum(ex), dtype=torch.float64).to(dtype)
            assert abs(float(scores[t, e]) - float(want)) <= (2 ** -8 if dtype == torch.bfloat16 else 1e-6) * float(want)
        off = [e for e in range(E) if e not in picked]
        assert all(float(scores[t, e]) == 0.0 for e in off)
    vals = torch.topk(logits.float(), K, dim=-1).values
    assert torch.equal(torch.gather(logits.float(), 1, idx), vals)
    assert torch.allclose(scores.float().sum(-1), torch.ones(T), atol=2e-2 if dtype == torch.bfloat16 else 1e-6)


def test_router_linear_rounds_once():
    g = torch.Generator().manual_seed(10)
    x = torch.randn(7, 32, generator=g).to(torch.bfloat16)
    w = torch.randn(5, 32, generator=g).to(torch.bfloat16)
    b = torch.randn(5, generator=g).to(torch.bfloat16)
    idx, scores, logits = O.router(x, w, b, 2)
    want = (x.double() @ w.double().t() + b.double()).to(torch.bfloat16)
    assert logits.dtype == torch.bfloat16 and (logits.float() - want.float()).abs().max() <= 2 ** -7 * want.float().abs().max()
    assert idx.shape == (7, 2) and scores.shape == (7, 5)


def test_router_is_differentiable_and_picks_override():
    """The router step in fp64 passes a finite-difference gradient check with respect to hidden states, weight and
    bias (the top-k choice is held fixed by the perturbation size), and `picks` reproduces the scores of the
    step's own choice."""
    g = torch.Generator().manual_seed(12)
    x = torch.randn(6, 10, generator=g, dtype=torch.float64, requires_grad=True)
    w = torch.randn(5, 10, generator=g, dtype=torch.float64, requires_grad=True)
    b = torch.randn(5, generator=g, dtype=torch.float64, requires_grad=True)
    idx, scores, _ = O.router(x, w, b, 3, compute_dtype=torch.float64)
    idx2, scores2, _ = O.router(x, w, b, 3, compute_dtype=torch.float64, picks=idx)
    assert torch.equal(idx, idx2) and torch.equal(scores, scores2)
    assert torch.autograd.gradcheck(lambda a, c, d: O.router(a, c, d, 3, compute_dtype=torch.float64, picks=idx)[1], (x, w, b))


def test_torch_baselines_of_the_package_agree_with_the_oracle():
    """yamoe_amd.reference / yamoe_amd.vendored (plain torch, for users to compare the operators against) give what the
    oracle gives: the GPT-OSS modules in training and in inference form, the router, and the capacity-binned formulation
    with and without drops and with dense and per-slot weights."""
    import types

    import yamoe_amd
    from yamoe_amd.workloads import make_inputs
    T, H, I, E, K = 90, 32, 24, 6, 2
    d = make_inputs(T, H, I, E, K, torch.float64, seed=3, w_std=0.3, bias_std=0.2, zipf=0.7)
    a = [d[k] for k in ("hidden", "router_indices", "routing_weights", "gate_up_proj", "gate_up_proj_bias", "down_proj",
                        "down_proj_bias")]
    for cap in (T, 11):
        want = O.experts_capacity(*a, cap)
        got = yamoe_amd.yamoe_ref.binned_experts_ref(*a, cap)
        assert O.rel_l2(got, want) < 1e-13
        per_slot = torch.gather(d["routing_weights"], 1, d["router_indices"])
        got = yamoe_amd.vendored.yamoe_ref.binned_experts_ref(a[0].reshape(3, 30, H), a[1], per_slot, *a[3:], cap)
        assert got.shape == (3, 30, H) and O.rel_l2(got.reshape(T, H), want) < 1e-13
    cfg = types.SimpleNamespace(hidden_size=H, intermediate_size=I, num_local_experts=E, num_experts_per_tok=K)
    mlp = yamoe_amd.gpt_oss_mlp.GptOssMLP(cfg).double()
    assert yamoe_amd.reference.GptOssExperts is yamoe_amd.vendored.gpt_oss_mlp.GptOssExperts
    with torch.no_grad():
        for p, v in zip(mlp.experts.parameters(), a[3:]):
            p.copy_(v)
        mlp.router.weight.copy_(torch.randn(E, H, dtype=torch.float64, generator=torch.Generator().manual_seed(1)))
        mlp.router.bias.copy_(torch.randn(E, dtype=torch.float64, generator=torch.Generator().manual_seed(2)))
    out, scores = mlp(d["hidden"])
    idx, want_scores, _ = O.router(d["hidden"], mlp.router.weight.detach(), mlp.router.bias.detach(), K,
                                   compute_dtype=torch.float64)
    assert O.rel_l2(scores.detach(), want_scores) < 1e-13
    want = O.experts_loop(d["hidden"], idx, want_scores, *a[3:])
    assert O.rel_l2(out.detach(), want) < 1e-13
    # the dense form (what the module does in inference mode off the CPU), called directly
    ex = mlp.experts
    every = d["hidden"].unsqueeze(0).expand(E, -1, -1)
    from yamoe_amd.torch_baseline import clamped_swiglu
    rows = torch.bmm(clamped_swiglu(torch.bmm(every, ex.gate_up_proj) + ex.gate_up_proj_bias.unsqueeze(1)), ex.down_proj)
    rows = rows + ex.down_proj_bias.unsqueeze(1)
    dense = (rows * want_scores.t().unsqueeze(-1)).sum(0)
    assert O.rel_l2(dense.detach(), want) < 1e-13
