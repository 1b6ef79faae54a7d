"""CPU-side checks of the boundary: the C-ABI library loads and exports every symbol the header
declares, argument validation rejects bad shapes before anything touches a GPU, and the torch op is
registered with the reference's schemas."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_symbols():
    text = open(os.path.join(ROOT, "include", "yamoe_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(yamoe_[a-z_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from yamoe_amd import _cabi
    lib = _cabi.lib()
    names = header_symbols()
    assert len(names) >= 14
    for n in names:
        assert hasattr(lib, n), n
    assert sorted(_cabi.SYMBOLS) == names
    assert lib.yamoe_abi_version() == _cabi.ABI_VERSION == 2


def test_size_queries_and_validation_need_no_gpu():
    from yamoe_amd import _cabi
    lib = _cabi.lib()
    p = _cabi.Problem(T=4096, K=4, E=32, H=2880, I=2880, capacity=4096, dtype=_cabi.BF16, idx_i64=1, rw_cols=32)
    fwd = lib.yamoe_experts_workspace_bytes(ctypes.byref(p))
    bwd = lib.yamoe_experts_backward_workspace_bytes(ctypes.byref(p))
    n = 4096 * 4
    assert fwd >= n * 2880 * 2 * 2 and bwd > fwd            # act + y_perm at least
    assert fwd < 2 * n * 2880 * 2 * 2                       # and nothing padded to [E, C, *]
    assert lib.yamoe_schedule_bytes(n, 32) % 256 == 0
    # a hidden size that is not a whole 16-byte chunk is accepted (it runs on the plain-FMA kernels)
    q = _cabi.Problem(**{**{f: getattr(p, f) for f, _ in p._fields_}, **dict(H=2881)})
    assert lib.yamoe_experts_workspace_bytes(ctypes.byref(q)) > 0
    # rejected shapes: routing weights with a wrong width, bad dtype, no slots
    for bad in (dict(rw_cols=7), dict(dtype=9), dict(K=0)):
        q = _cabi.Problem(**{**{f: getattr(p, f) for f, _ in p._fields_}, **bad})
        assert lib.yamoe_experts_workspace_bytes(ctypes.byref(q)) == 0
        assert len(lib.yamoe_last_error()) > 0
    # hidden_states of 4 GiB or more: accepted; the workspace then holds the rows in expert order as well (the kernels
    # gather token rows with 32-bit byte offsets from the tensor's start, so such a tensor is permuted first)
    for T_big, dt, wide in ((745000, _cabi.BF16, False), (746000, _cabi.BF16, True), (372000, _cabi.F32, False),
                            (373000, _cabi.F32, True)):
        q = _cabi.Problem(**{**{f: getattr(p, f) for f, _ in p._fields_}, **dict(T=T_big, capacity=T_big, dtype=dt)})
        es = 2 if dt == _cabi.BF16 else 4
        n = T_big * 4
        base = n * 2880 * es * 2                                   # act + y_perm
        need = lib.yamoe_experts_workspace_bytes(ctypes.byref(q))
        assert base < need < base + n * 2880 * es * (1 if wide else 0) + n * 64, (T_big, dt, need)
        if wide:
            assert need > base + n * 2880 * es
        assert lib.yamoe_experts_backward_workspace_bytes(ctypes.byref(q)) > need
    rc = lib.yamoe_gate_up(None, None, None, None, None, None, None, 746000 * 4, 4, 32, 2880, 2880, _cabi.BF16, None)
    assert rc == -1
    # yamoe_route rejects too many experts before any launch
    rc = lib.yamoe_route(None, 1, 0, 100000, 1, None, None, None, None, None, None, 0, None)
    assert rc == -1 and b"yamoe_route" in lib.yamoe_last_error()
    # entry points refuse null pointers instead of launching
    rc = lib.yamoe_experts_forward(ctypes.byref(p), *([None] * 9), 0, None)
    assert rc == -1


def test_torch_op_schemas_match_reference():
    """The registered schemas are the reference's (torch-ext/torch_binding.cpp:9-56), namespace aside."""
    import yamoe_amd
    ops = yamoe_amd.ops

    def schema(name):
        s = str(getattr(ops, name).default._schema).replace("_yamoe_amd_ops::", "")
        return re.sub(r"\(\$\d+! -> \)", "!", s)       # printed alias sets back to the "Tensor!" they were declared as

    assert schema("experts") == (
        "experts(Tensor hidden_states, Tensor router_indices, Tensor routing_weights, "
        "Tensor gate_up_proj, Tensor gate_up_proj_bias, Tensor down_proj, Tensor down_proj_bias, "
        "int expert_capacity, int num_experts, int top_k) -> Tensor")
    s = schema("experts_backward")
    assert s.startswith("experts_backward(Tensor grad_out, Tensor hidden_states, Tensor router_indices, ")
    assert s.endswith("int expert_capacity, int num_experts, int top_k) -> Tensor[]")
    assert schema("gather") == ("gather(Tensor x, Tensor indices, Tensor bins, Tensor! output, int E, int C, "
                                "int top_k) -> ()")
    assert schema("scatter") == ("scatter(Tensor src, Tensor indices, Tensor bins, Tensor weights, Tensor! y, "
                                 "int T, int E, int C, int top_k) -> ()")
    assert schema("sort") == "sort(Tensor x, int end_bit, Tensor! x_out, Tensor! iota_out) -> ()"
    assert schema("bincount_cumsum") == "bincount_cumsum(Tensor input, Tensor! output, int minlength) -> ()"
    assert schema("index_select_out") == "index_select_out(Tensor! out, Tensor input, Tensor idx_int32) -> Tensor"
    assert schema("batch_mm") == ("batch_mm(Tensor x, Tensor weights, Tensor batch_sizes, Tensor! output, "
                                  "bool trans_b=False) -> Tensor")
    assert schema("router_topk") == "router_topk(Tensor hidden, Tensor weight, Tensor? bias, int top_k) -> (Tensor, Tensor)"
    for name in ("gather", "scatter", "sort", "bincount_cumsum", "batch_mm", "experts", "experts_backward", "Yamoe"):
        assert getattr(yamoe_amd, name) is not None       # the reference package's exports (torch-ext/yamoe/__init__.py)


def test_no_cpu_fallback():
    """CPU tensors are refused: there is no eager or oracle path behind the op."""
    import yamoe_amd
    from yamoe_amd import _cabi
    from yamoe_amd.workloads import make_inputs
    d = make_inputs(8, 64, 64, 4, 2, torch.float32)
    a = [d[k] for k in ("hidden", "router_indices", "routing_weights", "gate_up_proj", "gate_up_proj_bias",
                        "down_proj", "down_proj_bias")]
    with pytest.raises((NotImplementedError, RuntimeError)):
        yamoe_amd.experts(*a, 8, 4, 2)
    with pytest.raises(RuntimeError):
        _cabi.experts_forward(*a, 8)


def test_product_does_not_import_the_oracle():
    for dirpath, _, files in os.walk(os.path.join(ROOT, "yamoe_amd")):
        for f in files:
            if f.endswith((".py", ".hip", ".cpp", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.replace("no oracle", ""), os.path.join(dirpath, f)


def test_workloads_are_seeded_and_shaped():
    from yamoe_amd.workloads import CONFIGS, make_config
    a, c = make_config("decode", seed=3, weights=False)
    b, _ = make_config("decode", seed=3, weights=False)
    assert torch.equal(a["router_indices"], b["router_indices"]) and torch.equal(a["hidden"], b["hidden"])
    assert a["router_indices"].shape == (64, 4) and a["routing_weights"].shape == (64, 128)
    rw = a["routing_weights"].float()
    assert torch.allclose(rw.sum(1), torch.ones(64), atol=2e-2)  # renormalised top-4 (bf16 rounding)
    assert (rw > 0).sum(1).eq(4).all()
    z, _ = make_config("zipf", seed=0, weights=False)
    counts = torch.bincount(z["router_indices"].flatten(), minlength=128)
    assert counts.max() > 10 * counts.float().mean() and (counts == 0).any()
    assert set(CONFIGS) == {"readme", "gptoss20b", "decode", "zipf", "mid512", "mid1024", "mid2048", "mid4096"}


def test_hub_layout_imports_as_yamoe(tmp_path):
    """`python -m yamoe_amd.package` lays out build/<variant>/yamoe/ (the reference's hub layout, build.toml:1-36);
    that directory imports as `yamoe` with the reference's names.  Run in a child process: the operator library
    registers its ops once per process."""
    import subprocess
    import sys
    from yamoe_amd import package
    dst = package.package(str(tmp_path))
    assert os.path.basename(dst) == "yamoe" and re.match(r"torch\d+-cxx11-rocm\d+-x86_64-linux$", os.path.basename(os.path.dirname(dst)))
    assert 'backend = "rocm"' in open(os.path.join(str(tmp_path), "build.toml")).read()
    code = ("import sys; sys.path.insert(0, %r); import yamoe; "
            "names = ['experts', 'experts_backward', 'gather', 'scatter', 'sort', 'bincount_cumsum', 'batch_mm', 'ops', 'Yamoe']; "
            "assert all(getattr(yamoe, n) is not None for n in names); "
            "assert 'yamoe_amd' not in sys.modules; print('ok')" % os.path.dirname(dst))
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, cwd=str(tmp_path))
    assert r.returncode == 0 and r.stdout.strip().endswith("ok"), r.stderr[-2000:]


def test_operators_answer_shape_queries_without_a_gpu():
    """torch.compile and FakeTensorMode ask an operator what it returns without running it: meta tensors through the
    functional operators give the shapes and dtypes the kernels would."""
    import yamoe_amd
    T, H, I, E, K = 12, 64, 48, 4, 2
    m = lambda *shape, dtype=torch.bfloat16: torch.empty(*shape, dtype=dtype, device="meta")
    x, idx, rw = m(T, H), m(T, K, dtype=torch.int64), m(T, E)
    w = (m(E, H, 2 * I), m(E, 2 * I), m(E, I, H), m(E, H))
    out = yamoe_amd.experts(x, idx, rw, *w, T, E, K)
    assert out.shape == (T, H) and out.dtype == torch.bfloat16 and out.device.type == "meta"
    grads = yamoe_amd.experts_backward(m(T, H), x, idx, rw, *w, T, E, K)
    assert [tuple(g.shape) for g in grads] == [(T, H), (T, E), (E, H, 2 * I), (E, 2 * I), (E, I, H), (E, H)]
    indices, scores = yamoe_amd.router_topk(x, m(E, H), m(E), K)
    assert indices.shape == (T, K) and indices.dtype == torch.int64 and scores.shape == (T, E)
    d_hidden, d_weight, d_bias = yamoe_amd.router_topk_backward(scores, indices, scores, x, m(E, H))
    assert d_hidden.shape == (T, H) and d_weight.shape == (E, H) and d_bias.shape == (E,)


def test_kept_bytes_matches_the_shape_function():
    """yamoe_experts_kept_bytes (the buffer `experts_keep` returns) against the size the operator's shape function
    reports to a graph capture."""
    import yamoe_amd
    from yamoe_amd import _cabi
    lib = _cabi.lib()
    for T, K, E, H, I, dt, code in ((12, 2, 4, 64, 48, torch.bfloat16, _cabi.BF16), (4096, 4, 32, 2880, 2880, torch.bfloat16, _cabi.BF16),
                                    (7, 3, 5, 40, 33, torch.float32, _cabi.F32), (9, 1, 2, 8, 5, torch.float64, _cabi.F64)):
        p = _cabi.Problem(T=T, K=K, E=E, H=H, I=I, capacity=T, dtype=code, idx_i64=1, rw_cols=E)
        m = lambda *shape, dtype=dt: torch.empty(*shape, dtype=dtype, device="meta")
        out, kept = yamoe_amd.experts_keep(m(T, H), m(T, K, dtype=torch.int64), m(T, E), m(E, H, 2 * I), m(E, 2 * I),
                                           m(E, I, H), m(E, H), T, E, K)
        assert out.shape == (T, H) and kept.dtype == torch.uint8
        assert kept.numel() == lib.yamoe_experts_kept_bytes(ctypes.byref(p)), (T, K, I)
