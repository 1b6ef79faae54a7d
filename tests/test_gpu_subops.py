"""The reference's public helper ops (torch-ext/torch_binding.cpp:9-56) against the oracle: integer
results bit-exact, floating-point results within the dtype's relative-L2 tolerance."""
import numpy as np
import pytest
import torch

from oracle import yamoe_oracle as O
from tests.util import REL_L2_TOL, report
from yamoe_amd.workloads import make_inputs

pytestmark = pytest.mark.gpu

NP = {torch.int16: np.int16, torch.int32: np.int32, torch.int64: np.int64}


@pytest.mark.parametrize("dt", [torch.int16, torch.int32, torch.int64])
@pytest.mark.parametrize("n,end_bit,span", [
    (1, None, None), (63, None, None), (5000, None, None), (70001, None, None),     # full width, signed keys
    (16384, 5, 32), (16384, 7, 128), (30000, 10, 700), (4097, 1, None), (100, 0, None),
])
def test_sort_bit_exact(gpu, dt, n, end_bit, span):
    import yamoe_amd
    info = np.iinfo(NP[dt])
    bits = info.bits if end_bit is None else end_bit
    print("sort %s n=%d end_bit=%d" % (dt, n, bits), flush=True)
    rng = np.random.default_rng(n + bits)
    if span is None:
        x = rng.integers(info.min, info.max, size=n, dtype=NP[dt], endpoint=True)
        if n > 10:
            x[: n // 4] = x[n // 4: 2 * (n // 4)]           # ties, so that stability shows
    else:
        x = rng.integers(0, span, size=n).astype(NP[dt])     # expert ids, some above 2^end_bit
    want_k, want_p = O.sort_pairs(x, bits)
    xt = torch.from_numpy(x).to(gpu)
    k, p = torch.empty_like(xt), torch.empty_like(xt)
    yamoe_amd.sort(xt, bits, k, p)
    torch.cuda.synchronize()
    assert np.array_equal(k.cpu().numpy(), want_k)
    assert np.array_equal(p.cpu().numpy(), want_p)
    assert np.array_equal(xt.cpu().numpy(), x)               # input untouched


def test_sort_empty_and_errors(gpu):
    import yamoe_amd
    e = torch.empty(0, dtype=torch.int32, device=gpu)
    yamoe_amd.sort(e, 32, torch.empty_like(e), torch.empty_like(e))
    x = torch.zeros(4, dtype=torch.int32, device=gpu)
    with pytest.raises(RuntimeError):
        yamoe_amd.sort(x.float(), 32, x.clone(), x.clone())
    with pytest.raises(RuntimeError):
        yamoe_amd.sort(x, 32, x.to(torch.int64), x.clone())
    with pytest.raises(RuntimeError):
        yamoe_amd.sort(x.reshape(2, 2), 32, x.clone(), x.clone())


@pytest.mark.parametrize("n,bins,out_len", [(0, 4, 4), (1, 1, 1), (16384, 32, 32), (256, 128, 128), (100000, 768, 800),
                                            (50000, 8192, 8192), (3000, 5, 9)])
def test_bincount_cumsum_bit_exact(gpu, n, bins, out_len):
    import yamoe_amd
    print("bincount_cumsum n=%d bins=%d" % (n, bins), flush=True)
    rng = np.random.default_rng(n + bins)
    v = rng.integers(-2, bins + 2, size=n).astype(np.int32)   # a few out of range on both sides
    out = torch.full((out_len,), 77, dtype=torch.int32, device=gpu)
    yamoe_amd.bincount_cumsum(torch.from_numpy(v).to(gpu), out, bins)
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(), O.bincount_cumsum(v, out_len, bins))
    with pytest.raises(RuntimeError):
        yamoe_amd.bincount_cumsum(torch.from_numpy(v).to(gpu), out, out_len + 1)
    with pytest.raises(RuntimeError):
        yamoe_amd.bincount_cumsum(torch.from_numpy(v).to(gpu).to(torch.int64), out, bins)


def routed(T, E, K, seed, skew=True):
    rng = np.random.default_rng(seed)
    p = rng.random(E) ** (3 if skew else 0)
    ids = np.stack([rng.choice(E, size=K, replace=False, p=p / p.sum()) for _ in range(T)]).astype(np.int32)
    keys, pos = O.sort_pairs(ids.reshape(-1), 32)
    bins = O.bincount_cumsum(keys, E, E)
    return ids, pos, bins


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16, torch.float64])
@pytest.mark.parametrize("T,H,E,C,K", [(64, 128, 8, 4, 2), (300, 2880, 32, 50, 4), (17, 36, 3, 40, 1), (128, 130, 4, 0, 2)])
def test_padded_gather_bit_exact(gpu, dtype, T, H, E, C, K):
    import yamoe_amd
    print("gather %s T=%d H=%d E=%d C=%d K=%d" % (dtype, T, H, E, C, K), flush=True)
    ids, pos, bins = routed(T, E, K, T + C)
    x = torch.randn(T, H, generator=torch.Generator().manual_seed(T)).to(dtype)
    out = torch.full((E, C, H), 5.0, dtype=dtype, device=gpu)
    yamoe_amd.gather(x.to(gpu), torch.from_numpy(pos).to(gpu), torch.from_numpy(bins).to(gpu), out, E, C, K)
    torch.cuda.synchronize()
    want = O.padded_gather(x, pos, bins, E, C, K)
    assert torch.equal(out.cpu(), want)                       # copies and zeros only: exact in every dtype
    with pytest.raises(RuntimeError):
        yamoe_amd.gather(x.to(gpu), torch.from_numpy(pos).to(gpu), torch.from_numpy(bins).to(gpu), out, E, C + 1, K)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16, torch.float64])
@pytest.mark.parametrize("T,H,E,C,K,weighted", [(64, 128, 8, 4, 2, True), (300, 2880, 32, 50, 4, True),
                                                (17, 36, 3, 40, 1, False), (90, 130, 4, 1000, 3, True),
                                                (5, 128, 32, 0, 2, True)])   # capacity 0: an empty src, y untouched
def test_padded_scatter(gpu, dtype, T, H, E, C, K, weighted):
    import yamoe_amd
    print("scatter %s T=%d H=%d E=%d C=%d K=%d" % (dtype, T, H, E, C, K), flush=True)
    ids, pos, bins = routed(T, E, K, T + C + 1)
    g = torch.Generator().manual_seed(T + 1)
    src = torch.randn(E, C, H, generator=g).to(dtype)
    w = torch.rand(T * K, generator=g).to(dtype) if weighted else None
    y0 = torch.randn(T, H, generator=g).to(dtype)             # the op accumulates onto what y holds
    y = y0.clone().to(gpu)
    yamoe_amd.scatter(src.to(gpu), torch.from_numpy(pos).to(gpu), torch.from_numpy(bins).to(gpu),
                      w.to(gpu) if weighted else torch.empty(0, dtype=dtype, device=gpu), y, T, E, C, K)
    torch.cuda.synchronize()
    want = O.padded_scatter(src, pos, bins, w, y0, T, E, C, K)
    assert report("scatter", y.cpu().double(), want, REL_L2_TOL[dtype]) < REL_L2_TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16, torch.float64])
def test_index_select_out(gpu, dtype):
    import yamoe_amd
    g = torch.Generator().manual_seed(2)
    v = torch.randn(5000, generator=g).to(dtype)
    idx = torch.randint(0, 5000, (12345,), generator=g, dtype=torch.int32)
    out = torch.empty(12345, dtype=dtype, device=gpu)
    r = yamoe_amd.index_select_out(out, v.to(gpu), idx.to(gpu))
    torch.cuda.synchronize()
    assert r.data_ptr() == out.data_ptr()
    assert torch.equal(out.cpu(), O.index_select(v, idx))
    with pytest.raises(RuntimeError):
        yamoe_amd.index_select_out(out, v.to(gpu), idx.to(gpu).to(torch.int64))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("E,C,K,N", [(4, 8, 64, 128), (32, 100, 2880, 5760), (8, 256, 1024, 1024), (3, 1, 40, 24),
                                     (5, 300, 2880, 2880)])
def test_batch_mm(gpu, dtype, E, C, K, N):
    import yamoe_amd
    print("batch_mm %s E=%d C=%d K=%d N=%d" % (dtype, E, C, K, N), flush=True)
    g = torch.Generator().manual_seed(E + C)
    x = torch.randn(E, C, K, generator=g).to(dtype)
    w = (torch.randn(E, K, N, generator=g) / K ** 0.5).to(dtype)
    out = torch.empty(E, C, N, dtype=dtype, device=gpu)
    r = yamoe_amd.batch_mm(x.to(gpu), w.to(gpu), torch.full((E,), C, dtype=torch.int32, device=gpu), out)
    torch.cuda.synchronize()
    assert r.data_ptr() == out.data_ptr()
    assert report("batch_mm", out.cpu().double(), O.batch_mm(x, w), REL_L2_TOL[dtype]) < REL_L2_TOL[dtype]
    with pytest.raises(RuntimeError):
        yamoe_amd.batch_mm(x.to(gpu), w.to(gpu)[:, :-1], torch.zeros(E, dtype=torch.int32, device=gpu), out)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_helper_pipeline_equals_fused_op(gpu, dtype):
    """The reference's own composition of its helper ops (torch-ext/yamoe/vendored/yamoe_ref.py:31-70)
    run on the HIP helpers must agree with the fused op and with the oracle."""
    import yamoe_amd
    T, H, I, E, K, C = 512, 256, 384, 8, 2, 96
    d = make_inputs(T, H, I, E, K, dtype, seed=11)
    dg = {k: v.to(gpu) for k, v in d.items()}
    flat = dg["router_indices"].reshape(-1).to(torch.int32)
    keys, pos = torch.empty_like(flat), torch.empty_like(flat)
    yamoe_amd.sort(flat, 32, keys, pos)
    bins = torch.empty(E, dtype=torch.int32, device=gpu)
    yamoe_amd.bincount_cumsum(keys, bins, E)
    x = torch.empty(E, C, H, dtype=dtype, device=gpu)
    yamoe_amd.gather(dg["hidden"], pos, bins, x, E, C, K)
    sizes = torch.full((E,), C, dtype=torch.int32, device=gpu)
    gu = yamoe_amd.batch_mm(x, dg["gate_up_proj"], sizes, torch.empty(E, C, 2 * I, dtype=dtype, device=gpu))
    gu = gu + dg["gate_up_proj_bias"][:, None, :]
    act = O.glu(gu.float().cpu()).to(dtype).to(gpu)            # the helpers have no activation op of their own
    y = yamoe_amd.batch_mm(act, dg["down_proj"], sizes, torch.empty(E, C, H, dtype=dtype, device=gpu))
    y = y + dg["down_proj_bias"][:, None, :]
    w_flat = dg["routing_weights"].gather(1, dg["router_indices"]).reshape(-1).contiguous()
    w_sorted = yamoe_amd.index_select_out(torch.empty_like(w_flat), w_flat, pos)
    out = torch.zeros(T, H, dtype=dtype, device=gpu)
    yamoe_amd.scatter(y, pos, bins, w_sorted, out, T, E, C, K)
    fused = yamoe_amd.experts(*[dg[k] for k in ("hidden", "router_indices", "routing_weights", "gate_up_proj",
                                                "gate_up_proj_bias", "down_proj", "down_proj_bias")], C, E, K)
    torch.cuda.synchronize()
    want = O.experts_capacity(*[d[k] for k in ("hidden", "router_indices", "routing_weights", "gate_up_proj",
                                               "gate_up_proj_bias", "down_proj", "down_proj_bias")], C,
                              compute_dtype=torch.float64)
    tol = REL_L2_TOL[dtype] * (3 if dtype != torch.float32 else 1)   # four extra roundings to 16 bits between helpers
    assert report("pipeline vs oracle", out.cpu().double(), want, tol) < tol
    assert report("pipeline vs fused", out.cpu().double(), fused.cpu().double(), tol) < tol
