"""The routing gradient entry by entry (csrc/experts_backward.cu:83-88, placed once at [token, expert]).

d_routing[t, e] = <grad_out[t], y[p]> with y[p] = act[p] . W_down[e] + b_down[e], the expert's output row before
weighting.  A whole-tensor relative L2 hides a bad entry next to large ones, and with one token there is nothing to
hide behind, so every entry is checked on its own, twice:

  against the oracle   in fp64 from the dtype-rounded inputs.  The kernels keep `act` in the activation dtype, so the
                       best possible result still carries one rounding (relative u) of every act[p, i]: the bound is
                       the forward error bound of that dot product, 2u * (sum_i |d_act_i * act_i| + |<grad_out, b_down>|)
                       with d_act = grad_out[t] . W_down[e]^T, plus one rounding of the stored value.
  against the forward  the same dot taken in fp64 from the activations the gate_up kernel itself produced (through the
                       C ABI).  Nothing is rounded between those and the result except the fp32 accumulation and the
                       final store, so the error allowed is 2^-11 of sqrt(sum_i (d_act_i * act_i)^2) + |<grad_out, b_down>|
                       plus one rounding of the stored value.  A routing gradient formed from an input gradient that
                       was first rounded to the activation dtype has a typical error of 0.6 u of that root sum
                       (u = 2^-9 for bf16): more than twice the bound on a typical entry, and every entry is checked.
"""
import pytest
import torch

from oracle import yamoe_oracle as O
from tests.util import args, to_dev
from yamoe_amd.workloads import make_inputs

pytestmark = pytest.mark.gpu

UNIT = {torch.bfloat16: 2.0 ** -9, torch.float16: 2.0 ** -12, torch.float32: 2.0 ** -21}


def slot_terms(d, gy, act_sorted, sorted_idx, inv_pos):
    """Per flat slot (t, k): value = <gy[t], act[p] . Wd[e] + bd[e]>, abs_scale = sum_i |d_act_i act_i| + |<gy[t], bd[e]>|
    and rms_scale = sqrt(sum_i (d_act_i act_i)^2) + |<gy[t], bd[e]>|, in fp64 from the given activations (rows in
    sorted order); NaN value for dropped slots."""
    T, K = d["router_indices"].shape
    wd, bd = d["down_proj"].double(), d["down_proj_bias"].double()
    g = gy.double()
    value = torch.full((T, K), float("nan"), dtype=torch.float64)
    scale = torch.zeros(T, K, dtype=torch.float64)
    rms = torch.zeros(T, K, dtype=torch.float64)
    for t in range(T):
        for k in range(K):
            p = int(inv_pos[t * K + k])
            if p < 0:
                continue
            e = int(d["router_indices"][t, k])
            a = act_sorted[p].double()
            d_act = wd[e] @ g[t]
            bias = float(g[t] @ bd[e])
            value[t, k] = float(d_act @ a) + bias
            scale[t, k] = float((d_act * a).abs().sum()) + abs(bias)
            rms[t, k] = float((d_act * a).square().sum().sqrt()) + abs(bias)
    return value, scale, rms


def oracle_act(d, sorted_idx, K):
    """Activations in sorted order from the oracle's GLU, fp64."""
    x = d["hidden"].double()
    tok = torch.from_numpy(sorted_idx.astype("int64")) // K
    e = d["router_indices"].reshape(-1)[torch.from_numpy(sorted_idx.astype("int64"))]
    rows = []
    for p in range(len(sorted_idx)):
        ee = int(e[p])
        rows.append(O.glu(x[tok[p]] @ d["gate_up_proj"][ee].double() + d["gate_up_proj_bias"][ee].double()))
    return torch.stack(rows) if rows else torch.zeros(0, d["down_proj"].shape[1], dtype=torch.float64)


def entries(d_routing, d, dense):
    """[T, K] view of the routing gradient at the selected experts."""
    return torch.gather(d_routing, 1, d["router_indices"]) if dense else d_routing


CASES = [
    # dtype, T, H, I, E, K, seed, zipf, slot_weights
    (torch.bfloat16, 1, 64, 96, 8, 1, 32, 1.5, False),   # one token, one slot: the two terms nearly cancel
    (torch.bfloat16, 1, 64, 96, 8, 1, 7, 0.0, True),
    (torch.bfloat16, 1, 128, 64, 4, 4, 3, 0.0, False),    # one token on every expert
    (torch.float16, 1, 64, 64, 2, 1, 5, 0.0, False),
    (torch.bfloat16, 2, 320, 576, 3, 2, 11, 0.0, False),  # I = 576: three column tiles, the last of 64 columns
    (torch.bfloat16, 7, 72, 40, 5, 2, 13, 0.0, False),    # H = 72: the register-staged kernel (contraction not a multiple of 64)
    (torch.float16, 300, 128, 96, 8, 2, 29, 1.5, True),
    (torch.bfloat16, 700, 192, 320, 3, 2, 17, 0.0, False),  # more than 256 rows per expert: several row tiles
    (torch.float32, 5, 64, 96, 8, 2, 19, 0.0, False),
]


@pytest.mark.parametrize("dtype,T,H,I,E,K,seed,zipf,slot_weights", CASES)
def test_routing_grad_every_entry(gpu, dtype, T, H, I, E, K, seed, zipf, slot_weights):
    import yamoe_amd
    from yamoe_amd import _cabi
    print("routing_grad", dtype, T, H, I, E, K, seed, zipf, slot_weights, flush=True)
    d = make_inputs(T, H, I, E, K, dtype, seed=seed, w_std=0.05, bias_std=0.1, zipf=zipf)
    if slot_weights:
        d["routing_weights"] = torch.gather(d["routing_weights"], 1, d["router_indices"])
    dense = not slot_weights
    gy = torch.randn(T, H, generator=torch.Generator().manual_seed(seed + 1)).to(dtype)
    g = to_dev(d, gpu)
    grads = yamoe_amd.experts_backward(gy.to(gpu), *args(g), T, E, K)
    torch.cuda.synchronize()
    got = entries(grads[1].cpu().double(), d, dense)

    r = O.route(d["router_indices"].numpy(), E, T)
    u = UNIT[dtype]
    # 1. against the fp64 oracle
    want, scale, _ = slot_terms(d, gy, oracle_act(d, r["sorted_idx"], K), r["sorted_idx"], r["inv_pos"])
    full = entries(O.experts_backward(gy, *args(d), T, compute_dtype=torch.float64)[1], d, dense)
    assert torch.allclose(want, full, rtol=1e-9, atol=1e-12), "the test's own per-slot dot disagrees with autograd"
    err = (got - want).abs()
    bound = 2 * u * scale + 2 * u * want.abs() + 1e-30
    print("  vs oracle: worst err / bound = %.3f" % float((err / bound).max()), flush=True)
    assert torch.all(err <= bound), (err / bound).max()
    # 2. against the activations the forward kernel produced
    if dtype != torch.float32:
        se, si, counts, offsets, inv = _cabi.route(g["router_indices"], E, T)
        sched = _cabi.build_schedule(counts, offsets, T * K, T, 0)
        act = _cabi.gate_up(g["hidden"], si, g["gate_up_proj"], g["gate_up_proj_bias"], sched, K)
        torch.cuda.synchronize()
        want2, _, rms2 = slot_terms(d, gy, act.cpu(), r["sorted_idx"], r["inv_pos"])
        err2 = (got - want2).abs()
        bound2 = 2.0 ** -11 * rms2 + 2 * u * want2.abs() + 1e-30
        print("  vs forward activations: worst err / bound = %.3f" % float((err2 / bound2).max()), flush=True)
        assert torch.all(err2 <= bound2), (err2 / bound2).max()


def test_routing_grad_repeated_expert(gpu):
    """A token that names one expert in two slots reads one dense weight twice; its gradient is the sum of the two
    slots' dots (autograd through the oracle), written once, the same on every run."""
    import yamoe_amd
    dtype = torch.bfloat16
    T, H, I, E, K = 33, 64, 64, 4, 3
    d = make_inputs(T, H, I, E, K, dtype, seed=41, w_std=0.05, bias_std=0.1)
    d["router_indices"][::2, 2] = d["router_indices"][::2, 0]  # every second token repeats its first expert
    gy = torch.randn(T, H, generator=torch.Generator().manual_seed(42)).to(dtype)
    g = to_dev(d, gpu)
    runs = [yamoe_amd.experts_backward(gy.to(gpu), *args(g), T, E, K)[1].cpu() for _ in range(3)]
    assert torch.equal(runs[0], runs[1]) and torch.equal(runs[0], runs[2])
    want = O.experts_backward(gy, *args(d), T, compute_dtype=torch.float64)[1]
    r = O.rel_l2(runs[0].double(), want)
    print("repeated expert: rel_l2 = %.3e" % r, flush=True)
    assert r < 1e-2
    sel = torch.zeros_like(want, dtype=torch.bool).scatter_(1, d["router_indices"], True)
    assert torch.all(runs[0][~sel] == 0)
