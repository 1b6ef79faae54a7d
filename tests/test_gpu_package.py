"""The hub layout on the GPU: `python -m yamoe_amd.package` writes build/<variant>/yamoe/ (the reference's layout,
build.toml:1-36, loaded there by compare_example.py:27-31 through sys.path or kernels.get_local_kernel); a child process
that has only that directory on its path imports `yamoe`, runs the forward and the backward through it and hands the
results back for a check against the oracle.  (The hub's own loader package is not in this image.)"""
import os
import subprocess
import sys

import pytest
import torch

from oracle import yamoe_oracle as O
from tests.util import KEYS

pytestmark = pytest.mark.gpu

CHILD = r"""
import sys
sys.path.insert(0, sys.argv[1])
import torch
import yamoe
assert 'yamoe_amd' not in sys.modules
from yamoe.workloads import make_inputs
T, H, I, E, K = 300, 128, 64, 8, 2
d = make_inputs(T, H, I, E, K, torch.bfloat16, seed=71, w_std=0.05, bias_std=0.1, zipf=0.7)
keys = %r
g = [d[k].cuda() for k in keys]
out = yamoe.experts(*g, T, E, K)
gy = torch.randn(T, H, generator=torch.Generator().manual_seed(72)).to(torch.bfloat16)
grads = yamoe.experts_backward(gy.cuda(), *g, T, E, K)
layer_out = yamoe.experts_autograd(*g, T, E, K, False) if hasattr(yamoe, 'experts_autograd') else out
torch.cuda.synchronize()
assert torch.equal(layer_out, out)
# the torch baselines under the reference's names (torch-ext/yamoe/__init__.py:3-4, 29-31)
ref = yamoe.vendored.yamoe_ref.binned_experts_ref(*[t.float() if t.is_floating_point() else t for t in g], T)
assert (ref - out.float()).norm() / ref.norm() < 1e-2
assert yamoe.reference.GptOssExperts is yamoe.gpt_oss_mlp.GptOssExperts
torch.save(dict(inputs=d, gy=gy, out=out.cpu(), grads=[t.cpu() for t in grads], file=yamoe.__file__), sys.argv[2])
print('child ok')
""" % (KEYS,)


def test_packaged_tree_runs_the_op(gpu, tmp_path):
    from yamoe_amd import package
    dst = package.package(str(tmp_path))
    result = os.path.join(str(tmp_path), "result.pt")
    r = subprocess.run([sys.executable, "-c", CHILD, os.path.dirname(dst), result], capture_output=True, text=True,
                       cwd=str(tmp_path), timeout=240)
    assert r.returncode == 0 and "child ok" in r.stdout, r.stderr[-3000:]
    got = torch.load(result, weights_only=True)
    assert got["file"].startswith(str(tmp_path))     # the packaged copy ran, not the source tree
    d, T = got["inputs"], got["inputs"]["hidden"].shape[0]
    want = O.experts_capacity(*[d[k] for k in KEYS], T, compute_dtype=torch.float32)
    assert O.rel_l2(got["out"], want) < 1e-2
    want_g = O.experts_backward(got["gy"], *[d[k] for k in KEYS], T, compute_dtype=torch.float32)
    for a, b in zip(got["grads"], want_g):
        assert O.rel_l2(a, b) < 1e-2


def test_operators_trace_under_torch_compile(gpu):
    """The operators carry shape functions, so a graph capture (torch.compile with the ahead-of-time eager backend: no
    code generation, just the traced graph run operator by operator) goes through `experts_autograd` forward and
    backward in one graph and gives the bits of the eager call."""
    import yamoe_amd
    from tests.util import args, to_dev
    from yamoe_amd.workloads import make_inputs
    T, H, I, E, K = 300, 128, 64, 4, 2
    d = to_dev(make_inputs(T, H, I, E, K, torch.bfloat16, seed=5, w_std=0.2, bias_std=0.1), gpu)
    leaves = [d[k].clone().requires_grad_(True) for k in ("hidden", "routing_weights", "gate_up_proj", "gate_up_proj_bias",
                                                          "down_proj", "down_proj_bias")]

    def forward(x, rw, wgu, bgu, wd, bd):
        return yamoe_amd.experts_autograd(x, d["router_indices"], rw, wgu, bgu, wd, bd, T, E, K)

    def step(fn):
        out = fn(*leaves)
        return out, torch.autograd.grad(out.float().square().sum(), leaves)

    want_out, want_grads = step(forward)
    got_out, got_grads = step(torch.compile(forward, backend="aot_eager", fullgraph=True))
    torch.cuda.synchronize()
    assert torch.equal(got_out, want_out)
    for a, b in zip(got_grads, want_grads):
        assert torch.equal(a, b)
