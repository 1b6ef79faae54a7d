"""experts_backward through the torch op against autograd through the CPU oracle."""
import pytest
import torch

from oracle import yamoe_oracle as O
from tests.util import args, to_dev
from yamoe_amd.workloads import make_config, make_inputs

pytestmark = pytest.mark.gpu

NAMES = ("d_hidden", "d_routing", "d_gate_up_proj", "d_gate_up_proj_bias", "d_down_proj", "d_down_proj_bias")
TOL = {torch.float32: 2e-5, torch.bfloat16: 1e-2, torch.float16: 1e-2}


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
