"""Seeded random shapes, dtypes, capacities and routing skews: forward and all six gradients against the oracle.
Shapes straddle the limits between the kernels (16 rows per expert for the streaming path, contraction lengths that
are or are not multiples of 64 for the asynchronous-copy path, partial row and column tiles)."""
import random

import pytest
import torch

from oracle import yamoe_oracle as O
from tests.util import KEYS, REL_L2_TOL

pytestmark = pytest.mark.gpu


def draw_case(rnd):
    dtype = rnd.choice([torch.bfloat16, torch.float16, torch.float32])
    mult = 8 if dtype != torch.float32 else 4
    H = rnd.choice([64, 128, 192, 256, 320, 8 * rnd.randint(3, 50), mult * rnd.randint(4, 60)])
    I = rnd.choice([64, 128, 96, 8 * rnd.randint(3, 40), mult * rnd.randint(4, 50)])
    E = rnd.choice([1, 2, 3, 4, 8, 16, 33, 64])
    K = rnd.randint(1, min(E, 4))
    T = rnd.choice([64, 300, 777, 1500, 2600])
    zipf = rnd.choice([0.0, 0.8, 1.5])
    cap = rnd.choice([T, T, max(1, T * K // (2 * E)), 17, 300])
    return dtype, T, H, I, E, K, cap, zipf, rnd.random() < 0.3


@pytest.mark.parametrize("seed", range(6))
def test_random_cases(gpu, seed):
    import yamoe_amd
    from yamoe_amd.workloads import make_inputs
    rnd = random.Random(1000 + seed)
    for case in range(8):
        dtype, T, H, I, E, K, cap, zipf, slot = draw_case(rnd)
        print("seed %d case %d: %s T=%d H=%d I=%d E=%d K=%d cap=%d zipf=%.1f slot_weights=%s" %
              (seed, case, dtype, T, H, I, E, K, cap, zipf, slot), flush=True)
        d = make_inputs(T, H, I, E, K, dtype, seed=seed * 100 + case, w_std=0.05, bias_std=0.1, zipf=zipf)
        if slot and K != E:
            d["routing_weights"] = torch.gather(d["routing_weights"], 1, d["router_indices"])
        g = [d[k].to(gpu) for k in KEYS]
        tol = REL_L2_TOL[dtype]
        cd = torch.float64 if dtype == torch.float32 else torch.float32
        out = yamoe_amd.experts(*g, cap, E, K)
        gy = torch.randn(T, H, generator=torch.Generator().manual_seed(case + 1)).to(dtype)
        grads = yamoe_amd.experts_backward(gy.to(gpu), *g, cap, E, K)
        torch.cuda.synchronize()
        want = O.experts_capacity(*[d[k] for k in KEYS], cap, compute_dtype=cd)
        want_g = O.experts_backward(gy, *[d[k] for k in KEYS], cap, compute_dtype=cd)
        names = ("out", "d_hidden", "d_routing", "d_gate_up_proj", "d_gate_up_proj_bias", "d_down_proj", "d_down_proj_bias")
        for name, a, b in zip(names, (out,) + tuple(grads), (want,) + tuple(want_g)):
            if float(b.abs().max()) == 0.0:
                assert float(a.abs().max()) == 0.0, name
            else:
                r = O.rel_l2(a.cpu(), b)
                assert r < tol, (name, r)
