"""Routing, permute and combine kernels against the oracle: integer results bit-exact."""
import numpy as np
import pytest
import torch

from oracle import yamoe_oracle as O

pytestmark = pytest.mark.gpu

CASES = [
    # N, E, capacity, index dtype, with invalid ids
    (1, 1, 1, torch.int64, False),
    (256, 128, 64, torch.int64, False),      # decode shape
    (16384, 32, 4096, torch.int64, False),   # GPT-OSS-20B shape
    (8192, 8, 256, torch.int32, False),      # README shape with the literal README capacity
    (1000, 7, 100, torch.int32, True),
    (32768, 768, 40, torch.int64, True),     # largest single-block case, most buckets
    (65536, 128, 16384, torch.int64, False),  # multi-block form
    (40001, 5, 9000, torch.int32, True),
    (40000, 700, 100, torch.int64, True),    # multi-block form with a segment table too large for LDS staging
    (0, 4, 3, torch.int64, False),
    # either side of the sizes at which the form changes (one workgroup / two launches / other segment lengths)
    (4096, 16, 300, torch.int64, True),
    (4097, 16, 300, torch.int32, True),
    (32768, 64, 500, torch.int64, False),
    (32769, 64, 500, torch.int32, True),
    (131073, 9, 20000, torch.int64, True),
]


@pytest.mark.parametrize("N,E,C,dt,invalid", CASES)
def test_route_bit_exact(gpu, N, E, C, dt, invalid):
    from yamoe_amd import _cabi
    print("route N=%d E=%d C=%d %s" % (N, E, C, dt), flush=True)
    rng = np.random.default_rng(N + E)
    # skewed popularity so that some experts are empty and some overflow the capacity
    p = rng.random(E) ** 3
    ids = rng.choice(E, size=N, p=p / p.sum()) if N else np.zeros(0, dtype=np.int64)
    if invalid and N:
        ids[rng.integers(0, N, size=N // 50 + 1)] = E + 3
        ids[rng.integers(0, N, size=N // 50 + 1)] = -2
    want = O.route(ids, E, C)
    t = torch.from_numpy(ids.astype(np.int64)).to(dt).to(gpu)
    se, si, counts, offsets, inv = _cabi.route(t, E, C)
    torch.cuda.synchronize()
    assert np.array_equal(counts.cpu().numpy(), want["counts"])
    assert np.array_equal(offsets.cpu().numpy(), want["offsets"])
    assert np.array_equal(si.cpu().numpy(), want["sorted_idx"])
    assert np.array_equal(se.cpu().numpy(), want["sorted_expert"])
    assert np.array_equal(inv.cpu().numpy(), want["inv_pos"])


def test_route_zipf_config(gpu):
    from yamoe_amd import _cabi
    from yamoe_amd.workloads import make_config
    d, c = make_config("zipf", weights=False)
    idx = d["router_indices"]
    want = O.route(idx.numpy(), c["E"], c["T"])
    se, si, counts, offsets, inv = _cabi.route(idx.to(gpu), c["E"], c["T"])
    assert np.array_equal(si.cpu().numpy(), want["sorted_idx"])
    assert np.array_equal(counts.cpu().numpy(), want["counts"])
    assert np.array_equal(inv.cpu().numpy(), want["inv_pos"])
    assert (want["counts"] == 0).sum() > 0 and want["counts"].max() > 10 * want["counts"].mean()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,K,E,H", [(64, 4, 16, 2880), (300, 2, 5, 72), (7, 3, 4, 10)])
def test_permute_and_combine(gpu, dtype, T, K, E, H):
    from yamoe_amd import _cabi
    print("permute/combine", dtype, T, K, E, H, flush=True)
    g = torch.Generator().manual_seed(T + H)
    x = torch.randn(T, H, generator=g).to(dtype)
    idx = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)])
    C = max(1, (T * K) // (2 * E))  # some slots get dropped
    r = O.route(idx.numpy(), E, C)
    se, si, counts, offsets, inv = _cabi.route(idx.to(gpu), E, C)
    xp = _cabi.permute(x.to(gpu), si, K)
    want_xp = x[torch.from_numpy(r["sorted_idx"].astype(np.int64)) // K]
    assert torch.equal(xp.cpu(), want_xp)  # a copy: bit-exact

    # combine: rows of y_perm weighted by dense routing weights, dropped slots skipped
    y = torch.randn(T * K, H, generator=g).to(dtype)
    rw = torch.rand(T, E, generator=g).to(dtype)
    got = _cabi.combine(y.to(gpu), inv, idx.to(gpu), rw.to(gpu), T, K, E).cpu()
    want = torch.zeros(T, H, dtype=torch.float64)
    invp = r["inv_pos"].reshape(T, K)
    for t in range(T):
        for k in range(K):
            if invp[t, k] >= 0:
                want[t] += rw[t, idx[t, k]].double() * y[invp[t, k]].double()
    tol = 1e-6 if dtype == torch.float32 else 1e-2
    assert O.rel_l2(got, want) < tol
    # per-slot [T,K] weights give the same result as the dense layout
    sel = torch.gather(rw, 1, idx)
    got_k = _cabi.combine(y.to(gpu), inv, idx.to(gpu), sel.to(gpu), T, K, E).cpu()
    assert torch.equal(got_k, got)
    # weight 1 (the backward of the permute)
    got1 = _cabi.combine(y.to(gpu), inv, None, None, T, K, E).cpu()
    want1 = torch.zeros(T, H, dtype=torch.float64)
    for t in range(T):
        for k in range(K):
            if invp[t, k] >= 0:
                want1[t] += y[invp[t, k]].double()
    assert O.rel_l2(got1, want1) < tol
    # tokens whose slots were all dropped come out as exact zeros
    all_dropped = (invp < 0).all(axis=1)
    if all_dropped.any():
        assert torch.all(got[torch.from_numpy(all_dropped)] == 0)


@pytest.mark.parametrize("N,E,C,stream_rows", [(256, 128, 64, 16), (16384, 32, 4096, 16), (65536, 128, 300, 16),
                                               (1000, 700, 5, 0), (40, 3, 40, 16),
                                               (300, 40, 30, 32),      # every expert within 32 rows: all of them stream
                                               (300, 40, 300, 32),     # some beyond 32: the limit falls back to 16
                                               (2000, 64, 32, 32),     # capacity 32 keeps everybody within the limit
                                               (256, 128, 256, -1),    # decode: everything streams, in chunks of 32 rows
                                               (160, 40, 160, -1),     # the same with experts of several chunks
                                               (2000, 64, 2000, -1)])  # too many assignments for that: as with 32
def test_schedule_lists(gpu, N, E, C, stream_rows):
    """The device-built work lists: experts with 1..stream_rows kept rows in the streaming list (with -1 and few
    assignments: every expert, in chunks of 32 rows), the
    rest cut into equal row tiles (as few as 256 rows allow, each a multiple of 32 rows but the last), both in
    expert order, none dropped, none duplicated.  A limit above 16 holds only if no expert exceeds it; with such
    experts present the limit is 16."""
    from yamoe_amd import _cabi
    rng = np.random.default_rng(N * 7 + E)
    p = rng.random(E) ** 4
    ids = rng.choice(E, size=N, p=p / p.sum())
    r = O.route(ids, E, C)
    counts = torch.from_numpy(r["counts"]).to(gpu)
    offsets = torch.from_numpy(r["offsets"]).to(gpu)
    sched = _cabi.build_schedule(counts, offsets, N, C, stream_rows).cpu().numpy()
    want_tiles, want_small = [], []
    # -1: every expert streams, in chunks of 32 rows, if there are at most 4 assignments per expert on average
    everything = stream_rows == -1 and N <= 4 * E
    if stream_rows == -1:
        stream_rows = 32
    if not everything and stream_rows > 16 and int(np.minimum(r["counts"], C).max()) > stream_rows:
        stream_rows = 16
    for e in range(E):
        kept = min(int(r["counts"][e]), C)
        if kept == 0:
            continue
        first = int(r["offsets"][e])
        if everything:
            want_small += [(e, first + c, min(32, kept - c)) for c in range(0, kept, 32)]
        elif kept <= stream_rows:
            want_small.append((e, first, kept))
        else:
            g0, n = len(want_tiles), -(-kept // 256)
            per = min(256, (-(-kept // n) + 31) // 32 * 32)
            assert (n - 1) * per < kept <= n * per
            for t in range(n):
                want_tiles.append((e, first + per * t, min(per, kept - per * t), g0, n))
    n_tiles, n_small, n_active, n_kept = sched[:4]
    assert n_tiles == len(want_tiles) and n_small == len(want_small)
    assert n_active == int((np.minimum(r["counts"], C) > 0).sum())
    assert n_kept == int(np.minimum(r["counts"], C).sum())
    max_tiles = N // 256 + min(N, E) + 1
    tiles = sched[48:48 + 8 * n_tiles].reshape(-1, 8)[:, :5]
    assert [tuple(t) for t in tiles.tolist()] == want_tiles
    small = sched[48 + 8 * max_tiles:48 + 8 * max_tiles + 4 * n_small].reshape(-1, 4)[:, :3]
    assert [tuple(t) for t in small.tolist()] == want_small
    # The cut table: 9 cuts that split the tile list into 8 shares of (nearly) equal cost for any number of
    # column tiles; every cut lies on an (expert, column tile) boundary and the cuts are monotone.
    # cost weight of a tile: 3 + 2 per 64 rows; an expert with a single row tile weighs at least 8
    weight = lambda rows: 3 + 2 * ((rows + 63) // 64)
    w_tiles = [max(weight(t[2]), 8) if t[4] == 1 else weight(t[2]) for t in want_tiles]
    assert sched[4] == sum(w_tiles)
    for n_col in (1, 12, 23):
        cuts = []
        for x in range(9):
            first, frac, _, cnt = sched[8 + 4 * x:12 + 4 * x].tolist()
            assert 0 <= frac < 65536
            cuts.append(first * n_col + ((frac * n_col) >> 16) * cnt)
        assert cuts[0] == 0 and cuts[8] == len(want_tiles) * n_col
        assert all(a <= b for a, b in zip(cuts, cuts[1:]))
        # flat list: group-major, then column tile, then the group's row tiles
        flat, bounds = [], {0}
        g = 0
        while g < len(want_tiles):
            cnt = want_tiles[g][4]
            for c in range(n_col):
                flat += w_tiles[g:g + cnt]
                bounds.add(len(flat))
            g += cnt
        assert all(c in bounds for c in cuts)
        if flat:
            shares = [sum(flat[a:b]) for a, b in zip(cuts, cuts[1:])]
            biggest_unit = max(sum(w_tiles[g:g + want_tiles[g][4]]) for g in range(len(want_tiles)))
            assert max(shares) - sum(flat) / 8 <= 2 * biggest_unit + 1e-9
