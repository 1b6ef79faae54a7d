"""yamoe_experts_forward_static: the forward on the workspace that is built into the library, through the C ABI.

It runs the kernels of yamoe_experts_forward on a different workspace address, so its output must equal that entry
point's bit for bit; checked on two calls in a row, the second on a smaller problem (the array then still holds the
first call's lists and rows), and once more after the first problem again.  Problems beyond the array are refused.

"Allocates nothing" is checked at two levels: torch's caching allocator sees no request, and the driver's count of
free device memory (hipMemGetInfo, which a hipMalloc or hipFree inside the library would move, whoever made it) is
the same before and after every call but the first on the device (that one may load the code object that holds the
array).  A hipMalloc inside the call would also make the stream capture of the last test fail."""
import ctypes

import pytest
import torch

from tests.util import KEYS
from yamoe_amd.workloads import make_inputs

pytestmark = pytest.mark.gpu


def both(d, capacity, gpu):
    from yamoe_amd import _cabi
    g = [d[k].to(gpu) for k in KEYS]
    want = _cabi.experts_forward(*g, capacity)
    got = torch.full_like(want, float("nan"))
    _cabi.experts_forward_static(*g, capacity, got)     # (the first call on the device looks the array's address up)
    torch.cuda.synchronize()
    before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
    got.fill_(float("nan"))
    _cabi.experts_forward_static(*g, capacity, got)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.cuda.mem_get_info()[0] == free_before, "device memory was allocated or freed during the call"
    return got.cpu(), want.cpu()


def test_static_workspace_forward_matches(gpu):
    from oracle import yamoe_oracle as O
    big = make_inputs(700, 256, 192, 8, 2, torch.bfloat16, seed=51, w_std=0.05, bias_std=0.1, zipf=0.8)   # tiles and streamed experts
    small = make_inputs(40, 128, 64, 4, 2, torch.bfloat16, seed=52, w_std=0.05, bias_std=0.1)
    for label, d, cap in (("first", big, 700), ("second, smaller", small, 40), ("first again, capacity 100", big, 100)):
        print("static workspace:", label, flush=True)
        got, want = both(d, cap, gpu)
        assert torch.equal(got, want), label
        ref = O.experts_capacity(*[d[k] for k in KEYS], cap, compute_dtype=torch.float32)
        assert O.rel_l2(got, ref) < 1e-2


def test_static_workspace_forward_fp32_and_decode_shape(gpu):
    d = make_inputs(300, 64, 96, 4, 2, torch.float32, seed=53, w_std=0.05, bias_std=0.1)
    got, want = both(d, 300, gpu)
    assert torch.equal(got, want)
    d = make_inputs(64, 2880, 2880, 8, 4, torch.bfloat16, seed=54)    # the decode expert shape, 256 assignments
    got, want = both(d, 64, gpu)
    assert torch.equal(got, want)


def test_static_workspace_forward_refuses_large_problems(gpu):
    from yamoe_amd import _cabi
    T, H, I, E, K = 4096, 2880, 2880, 2, 4
    p = _cabi.Problem(T=T, K=K, E=E, H=H, I=I, capacity=T, dtype=_cabi.BF16, idx_i64=1, rw_cols=E)
    assert _cabi.lib().yamoe_experts_workspace_bytes(ctypes.byref(p)) > _cabi.STATIC_SCRATCH_BYTES
    one = torch.zeros(1, device=gpu)
    ptr = ctypes.c_void_p(one.data_ptr())   # never touched: the size check comes first
    rc = _cabi.lib().yamoe_experts_forward_static(ctypes.byref(p), *([ptr] * 8), ptr, None)
    assert rc == -2, rc   # YAMOE_E_WORKSPACE
    assert b"built-in" in _cabi.lib().yamoe_last_error()


def test_static_workspace_forward_in_a_hip_graph(gpu):
    """The callers it is for: captured once (after a first eager call, which looks the array's address up), replayed
    with other work in between, every replay equal to the eager result."""
    from yamoe_amd import _cabi
    d = make_inputs(500, 256, 128, 8, 2, torch.bfloat16, seed=55, w_std=0.05, bias_std=0.1, zipf=0.6)
    g = [d[k].to(gpu) for k in KEYS]
    want = _cabi.experts_forward(*g, 500)
    out = torch.zeros_like(want)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        _cabi.experts_forward_static(*g, 500, out)            # first call on this device happens outside the capture
    torch.cuda.synchronize()
    assert torch.equal(out, want)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        _cabi.experts_forward_static(*g, 500, out)
    small = make_inputs(30, 256, 128, 8, 2, torch.bfloat16, seed=56, w_std=0.05, bias_std=0.1)
    gs = [small[k].to(gpu) for k in KEYS]
    for rep in range(3):
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), rep
        scratch_user = torch.empty(30, 256, dtype=torch.bfloat16, device=gpu)
        _cabi.experts_forward_static(*gs, 30, scratch_user)   # another problem on the same array between replays
        torch.cuda.synchronize()
