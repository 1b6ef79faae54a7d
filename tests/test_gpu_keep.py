"""The training pair: `experts_keep` leaves the activations and pre-activations of the forward for `experts_backward_kept`,
which then skips the recomputation of the gate_up product that the reference's backward (and `experts_backward`) runs
(csrc/experts_backward.cu:164-230).  The forward's result is that of `experts`, bit for bit; the gradients are those of
`experts_backward`, bit for bit where the forward ran every expert on the tile kernels (the recomputation does), and to
the tolerance of the dtype against the oracle everywhere."""
import ctypes

import pytest
import torch

from oracle import yamoe_oracle as O
from tests.util import KEYS, REL_L2_TOL, args, to_dev
from yamoe_amd.workloads import make_inputs

pytestmark = pytest.mark.gpu

NAMES = ("d_hidden", "d_routing", "d_gate_up_proj", "d_gate_up_proj_bias", "d_down_proj", "d_down_proj_bias")

SHAPES = [
    # T, H, I, E, K, capacity (0: tokens), zipf, every expert on the tile kernels in the forward
    (700, 128, 64, 3, 2, 0, 0.0, True),
    (1024, 256, 192, 4, 2, 0, 0.0, True),
    (513, 320, 136, 5, 3, 0, 0.0, True),       # register-staged kernels
    (2000, 64, 64, 64, 2, 0, 0.8, False),      # streamed experts next to tiled ones
    (600, 128, 64, 4, 2, 37, 0.5, True),       # capacity drops assignments
    (40, 64, 64, 16, 1, 0, 0.0, False),        # every expert streams
    (300, 67, 35, 5, 3, 0, 0.0, True),         # odd sizes: the plain-FMA kernels
    (3, 64, 320, 2, 1, 0, 0.0, False),         # a handful of rows: the weight-gradient kernel's last slab runs past them
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32, torch.float64])
@pytest.mark.parametrize("T,H,I,E,K,capacity,zipf,tiled", SHAPES)
def test_keep_and_kept(gpu, dtype, T, H, I, E, K, capacity, zipf, tiled):
    import yamoe_amd
    print("keep", dtype, T, H, I, E, K, capacity, zipf, flush=True)
    d = make_inputs(T, H, I, E, K, dtype, seed=T + H, w_std=0.2, bias_std=0.1, zipf=zipf)
    cap = capacity or T
    g = to_dev(d, gpu)
    gy = torch.randn(T, H, generator=torch.Generator().manual_seed(3)).to(dtype)
    out, kept = yamoe_amd.experts_keep(*args(g), cap, E, K)
    assert torch.equal(out, yamoe_amd.experts(*args(g), cap, E, K))
    grads = yamoe_amd.experts_backward_kept(gy.to(gpu), *args(g), kept, cap, E, K)
    plain = yamoe_amd.experts_backward(gy.to(gpu), *args(g), cap, E, K)
    torch.cuda.synchronize()
    tol = {**REL_L2_TOL, torch.float64: 1e-12}[dtype]
    cd = torch.float64 if dtype in (torch.float32, torch.float64) else torch.float32
    want = O.experts_backward(gy, *args(d), cap, compute_dtype=cd)
    for n, a, b, w in zip(NAMES, grads, plain, want):
        if tiled or dtype in (torch.float32, torch.float64):
            assert torch.equal(a, b), n
        r = O.rel_l2(a.cpu(), w)
        assert r < tol, (n, r)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_autograd_with_saved_activations(gpu, dtype):
    """experts_autograd(save_activations=True) and the Yamoe layer with `save_activations` set: the same gradients as
    without, from a backward that does not run the gate_up product."""
    import types

    import yamoe_amd
    T, H, I, E, K = 600, 128, 64, 4, 2
    d = to_dev(make_inputs(T, H, I, E, K, dtype, seed=9, w_std=0.2, bias_std=0.1), gpu)
    leaves = lambda: [d[k].clone().requires_grad_(True) for k in ("hidden", "routing_weights", "gate_up_proj",
                                                                   "gate_up_proj_bias", "down_proj", "down_proj_bias")]
    runs = []
    for save in (False, True):
        x, rw, wgu, bgu, wd, bd = lv = leaves()
        out = yamoe_amd.experts_autograd(x, d["router_indices"], rw, wgu, bgu, wd, bd, T, E, K, True, save)
        runs.append((out, torch.autograd.grad(out.float().square().sum(), lv)))
    assert torch.equal(runs[0][0], runs[1][0])
    for a, b in zip(runs[0][1], runs[1][1]):
        assert torch.equal(a, b)
    # the layer
    gen = torch.Generator().manual_seed(4)
    router = types.SimpleNamespace(weight=torch.nn.Parameter((torch.randn(E, H, generator=gen) * 0.3).to(dtype).to(gpu)),
                                   bias=torch.nn.Parameter((torch.randn(E, generator=gen) * 0.1).to(dtype).to(gpu)))
    experts = types.SimpleNamespace(**{k: torch.nn.Parameter(d[k].clone()) for k in ("gate_up_proj", "gate_up_proj_bias",
                                                                                      "down_proj", "down_proj_bias")})
    got = []
    for save in (False, True):
        layer = types.SimpleNamespace(router=router, experts=experts, num_experts=E, top_k=K, enable_router_grads=True,
                                      save_activations=save)
        x = d["hidden"].clone().reshape(2, T // 2, H).requires_grad_(True)
        out, _ = yamoe_amd.Yamoe.forward(layer, x)
        ps = [x, router.weight, router.bias, experts.gate_up_proj, experts.down_proj]
        got.append((out, torch.autograd.grad(out.float().square().sum(), ps)))
    assert torch.equal(got[0][0], got[1][0])
    for a, b in zip(got[0][1], got[1][1]):
        assert torch.equal(a, b)


def test_kept_buffer_size_is_checked(gpu):
    from yamoe_amd import _cabi
    T, H, I, E, K = 64, 64, 64, 4, 2
    d = to_dev(make_inputs(T, H, I, E, K, torch.bfloat16, seed=1), gpu)
    p = _cabi.problem(d["hidden"], d["router_indices"], d["routing_weights"], d["gate_up_proj"], T)
    lib = _cabi.lib()
    need = lib.yamoe_experts_kept_bytes(ctypes.byref(p))
    assert need >= T * K * 3 * I * 2
    ws = torch.empty(lib.yamoe_experts_workspace_bytes(ctypes.byref(p)), dtype=torch.uint8, device=gpu)
    out = torch.empty_like(d["hidden"])
    small = torch.empty(need - 256, dtype=torch.uint8, device=gpu)
    ptr = lambda t: ctypes.c_void_p(t.data_ptr())
    rc = lib.yamoe_experts_forward_keep(ctypes.byref(p), *[ptr(d[k]) for k in KEYS], ptr(out), ptr(small), small.numel(),
                                        ptr(ws), ws.numel(), None)
    assert rc != 0 and b"kept" in lib.yamoe_last_error()
