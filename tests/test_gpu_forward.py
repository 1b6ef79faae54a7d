"""experts() forward through the torch op (-> C ABI -> HIP kernels) against the CPU oracle."""
import numpy as np
import pytest
import torch

from oracle import yamoe_oracle as O
from tests.util import REL_L2_TOL, args, oracle_forward, report, to_dev
from yamoe_amd.workloads import make_config, make_inputs

pytestmark = pytest.mark.gpu


def run_op(d, capacity, gpu):
    import yamoe_amd
    g = to_dev(d, gpu)
    E, K = d["gate_up_proj"].shape[0], d["router_indices"].shape[1]
    out = yamoe_amd.experts(*args(g), capacity, E, K)
    torch.cuda.synchronize()
    return out.cpu()


SMALL = [
    # T, H, I, E, K  -- chosen to hit: streaming path only, MFMA tiles only, both, ragged edges
    (8, 64, 64, 4, 2),        # a few rows per expert: weight-streaming kernel
    (64, 128, 96, 16, 4),     # I != H, streaming
    (700, 64, 64, 2, 1),      # 350 rows per expert: MFMA tiles with a partial second tile
    (1024, 256, 192, 4, 2),   # several column tiles? no: one; K slabs > 1
    (300, 320, 136, 3, 2),    # N and K not multiples of the tile sizes
    (513, 520, 264, 5, 3),    # more than one column tile for gate_up (2I = 528 > 256), K = 520 not /64
    (2000, 64, 64, 64, 2),    # mix: some experts <= 16 rows, some above
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("T,H,I,E,K", SMALL)
def test_forward_small(gpu, dtype, T, H, I, E, K):
    print("forward_small", dtype, T, H, I, E, K, flush=True)
    d = make_inputs(T, H, I, E, K, dtype, seed=T + H, w_std=0.05, bias_std=0.1, zipf=0.8 if E >= 16 else 0.0)
    got = run_op(d, T, gpu)
    want = oracle_forward(d, T)
    r = report("fwd", got, want, REL_L2_TOL[dtype])
    assert r < REL_L2_TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_forward_capacity_drop_and_slot_weights(gpu, dtype):
    T, H, I, E, K = 400, 64, 64, 4, 2
    d = make_inputs(T, H, I, E, K, dtype, seed=11, w_std=0.05, bias_std=0.1, zipf=1.0)
    for C in (0, 7, 60, 150):
        print("capacity", dtype, C, flush=True)
        got = run_op(d, C, gpu)
        want = oracle_forward(d, C)
        if C == 0:
            assert torch.all(got == 0)
        else:
            assert report("cap%d" % C, got, want, REL_L2_TOL[dtype]) < REL_L2_TOL[dtype]
    # [T,K] routing weights and int32 indices are accepted and give the same bits
    base = run_op(d, 60, gpu)
    d2 = dict(d)
    d2["routing_weights"] = torch.gather(d["routing_weights"], 1, d["router_indices"])
    d2["router_indices"] = d["router_indices"].to(torch.int32)
    assert torch.equal(run_op(d2, 60, gpu), base)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows", [180, 250, 100])
def test_forward_partial_column_tiles(gpu, dtype, rows):
    """H = 576 and 2I = 640: the last column tile of the down product has 64 valid columns, that of gate_up 128, on the
    pipelined path (18 and 10 slabs).  180 rows per expert are six 32-row blocks (the tile form that copies six of
    eight row blocks), 250 are eight, 100 take the general form."""
    T, H, I, E, K = 2 * rows, 576, 320, 2, 1
    d = make_inputs(T, H, I, E, K, dtype, seed=rows, w_std=0.05, bias_std=0.1)
    d["router_indices"] = (torch.arange(T) % E).reshape(T, 1)
    got = run_op(d, T, gpu)
    want = oracle_forward(d, T)
    assert report("partial column tiles", got, want, REL_L2_TOL[dtype]) < REL_L2_TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows", [3841, 4096, 4400, 6200, 8192])
def test_forward_experts_with_many_row_tiles(gpu, dtype, rows):
    """An expert with sixteen or more row tiles is walked in bands of eight row tiles (the last band takes the remainder:
    3841 and 4096 rows are bands of 8 + 8 tiles, 4400 of 8 + 10, 6200 of 8 + 8 + 9, 8192 of four 8s), next to one that
    is walked column by column (300 rows); three and two column tiles, the last partial."""
    H, I = 576, 320
    T = rows + 300
    d = make_inputs(T, H, I, 3, 1, dtype, seed=rows, w_std=0.05, bias_std=0.1)
    idx = torch.zeros(T, 1, dtype=torch.int64)
    idx[rows:] = 2                                   # expert 1 stays empty
    idx = idx[torch.randperm(T, generator=torch.Generator().manual_seed(rows))]
    d["router_indices"] = idx
    got = run_op(d, T, gpu)
    want = oracle_forward(d, T)
    assert report("many row tiles", got, want, REL_L2_TOL[dtype]) < REL_L2_TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,E,K,hot", [(100, 32, 1, 70), (64, 128, 4, 0), (128, 40, 1, 100), (33, 9, 1, 33)])
def test_forward_every_expert_streams(gpu, dtype, T, E, K, hot):
    """At most 4 assignments per expert on average: every expert goes through the streaming kernel, an expert with
    more than 32 rows in chunks of 32 (`hot` tokens are sent to expert 3: 70 rows are chunks of 32 + 32 + 6, 100 of
    32 + 32 + 32 + 4, 33 of 32 + 1), and the tile kernels are not launched."""
    H, I = 192, 160
    d = make_inputs(T, H, I, E, K, dtype, seed=T + E, w_std=0.05, bias_std=0.1)
    assert T * K <= 4 * E
    if hot:
        d["router_indices"][:hot, 0] = 3
        d["routing_weights"] = torch.rand(T, E, generator=torch.Generator().manual_seed(1)).to(dtype)
    got = run_op(d, T, gpu)
    want = oracle_forward(d, T)
    assert report("every expert streams", got, want, REL_L2_TOL[dtype]) < REL_L2_TOL[dtype]


def test_forward_uneven_tile_costs(gpu):
    """Eight experts with 2048 rows each and 56 experts with 20 rows each: the shares of the tile list that the
    8 XCDs get are equal in cost, so the shares made of small tiles hold more tiles than the grid has workgroups
    per XCD and the excess goes to workgroups of other XCDs."""
    E, H, I = 64, 128, 128
    ids = np.concatenate([np.repeat(np.arange(8), 2048), np.repeat(np.arange(8, 64), 20)])
    rng = np.random.default_rng(3)
    rng.shuffle(ids)
    T = len(ids)
    d = make_inputs(T, H, I, E, 1, torch.bfloat16, seed=5, w_std=0.05, bias_std=0.1)
    d["router_indices"] = torch.from_numpy(ids.astype(np.int64)).reshape(T, 1)
    d["routing_weights"] = torch.rand(T, E, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16)
    got = run_op(d, T, gpu)
    want = oracle_forward(d, T)
    tol = REL_L2_TOL[torch.bfloat16]
    assert report("uneven tile costs", got.double(), want.double(), tol) < tol


def test_forward_many_assignments(gpu):
    """N = T*K above the single-workgroup routing limit (32 768): three-kernel routing, separate work-list launch,
    skewed expert loads with some experts empty."""
    T, H, I, E, K = 20000, 128, 64, 16, 2
    d = make_inputs(T, H, I, E, K, torch.bfloat16, seed=21, w_std=0.05, bias_std=0.1, zipf=1.2)
    got = run_op(d, T, gpu)
    want = oracle_forward(d, T)
    tol = REL_L2_TOL[torch.bfloat16]
    assert report("many assignments", got.double(), want.double(), tol) < tol


def test_forward_special_cases(gpu):
    """Structure checks that do not depend on the oracle's matmul: one-hot routing returns the
    expert's row, zero weights reduce to the bias closed form, an unused expert changes nothing."""
    dtype = torch.float32
    T, H, I, E, K = 96, 64, 64, 4, 1
    d = make_inputs(T, H, I, E, K, dtype, seed=3, w_std=0.05, bias_std=0.1)
    d["routing_weights"] = torch.zeros(T, E).scatter_(1, d["router_indices"], 1.0)
    d["gate_up_proj"].zero_()
    got = run_op(d, T, gpu)
    per_e = torch.stack([O.glu(d["gate_up_proj_bias"][e][None])[0] @ d["down_proj"][e] + d["down_proj_bias"][e]
                         for e in range(E)])
    want = per_e[d["router_indices"][:, 0]]
    assert O.rel_l2(got, want) < 1e-5
    # determinism: bitwise equal on a second run
    assert torch.equal(run_op(d, T, gpu), got)


def test_forward_gptoss20b_full(gpu):
    """The GPT-OSS-20B shaped layer at full size against the fp32 oracle on the bf16 inputs."""
    d, c = make_config("gptoss20b", seed=0)
    got = run_op(d, c["T"], gpu)
    want = oracle_forward(d, c["T"])
    assert report("gptoss20b", got, want, 1e-2) < 1e-2
    # size-independent properties: linear in the routing weights, and a token routed with all its
    # weight on one expert equals that expert alone
    d2 = dict(d)
    d2["routing_weights"] = (d["routing_weights"].float() * 0.5).to(torch.bfloat16)  # exact scaling in bf16
    half = run_op(d2, c["T"], gpu)
    assert O.rel_l2(half.float() * 2, got.float()) < 1e-2


def test_forward_gptoss20b_full_fp16(gpu):
    """The same layer in fp16 (the dtype of the reference's timing sweep, perf_plot.py:93-101)."""
    d, c = make_config("gptoss20b", seed=3)
    d = {k: (v.to(torch.float16) if v.is_floating_point() else v) for k, v in d.items()}
    got = run_op(d, c["T"], gpu)
    want = oracle_forward(d, c["T"])
    assert report("gptoss20b fp16", got, want, 1e-2) < 1e-2


def test_forward_decode_full_rows(gpu):
    """Decode regime at the real expert shape (fewer experts to keep host generation short)."""
    d = make_inputs(64, 2880, 2880, 32, 4, torch.bfloat16, seed=5)
    counts = np.bincount(d["router_indices"].numpy().ravel(), minlength=32)
    assert counts.max() <= 16  # every expert takes the streaming path
    got = run_op(d, 64, gpu)
    want = oracle_forward(d, 64)
    assert report("decode", got, want, 1e-2) < 1e-2


def test_forward_readme_shape_fp32(gpu):
    """README shape (fp32, randn weights, heavy clamp saturation), two experts' worth of the 8 to
    bound the oracle's time: rel-L2 <= 1e-5."""
    d = make_inputs(4096, 2880, 2880, 2, 2, torch.float32, seed=42, w_std=1.0, bias_std=0.0, renorm=False)
    got = run_op(d, 4096, gpu)
    want = oracle_forward(d, 4096, compute_dtype=torch.float64)
    assert report("readme-fp32", got, want, 1e-5) < 1e-5


def test_op_rejects_bad_arguments(gpu):
    import yamoe_amd
    d = to_dev(make_inputs(8, 64, 64, 4, 2, torch.bfloat16), gpu)
    a = list(args(d))
    with pytest.raises(RuntimeError):
        yamoe_amd.experts(a[0].view(2, 4, 64), *a[1:], 8, 4, 2)  # hidden must be 2D
    with pytest.raises(RuntimeError):
        yamoe_amd.experts(*a, 8, 5, 2)  # num_experts disagrees with the weights
    with pytest.raises(RuntimeError):
        yamoe_amd.experts(a[0], a[1], a[2].float(), *a[3:], 8, 4, 2)  # dtype mismatch
    with pytest.raises(RuntimeError):
        yamoe_amd.experts(a[0], a[1].float(), *a[2:], 8, 4, 2)  # indices must be integers


def test_sweep_point_runs(gpu):
    """One small point of the reference's timing sweep (perf_plot.py:29-39 shapes, scaled down) through the sweep
    driver: fp16, unit-variance weights, both capacity conventions."""
    from yamoe_amd import sweep
    r = sweep.run_point(2, 64, 128, 8, 2, iters=2, warmup=1, capacity="tokens")
    assert r["kept_assignments"] == 2 * 64 * 2 and r["ms"] > 0 and r["finite"]
    r = sweep.run_point(2, 64, 128, 8, 2, iters=2, warmup=1, capacity="seq")
    assert r["kept_assignments"] <= 2 * 64 * 2 and r["capacity"] == 64
    assert len(sweep.CONFIGS) == 6 and sweep.BATCH_SIZES == [1, 2, 4, 8, 16, 32, 64]


def test_forward_and_backward_replay_in_a_hip_graph(gpu):
    """The op makes no host synchronisation and no memset node: captured once into a graph and replayed with
    other work in between, every replay reproduces the eager result bit for bit."""
    import yamoe_amd
    T, H, I, E, K = 700, 128, 128, 8, 2
    d = make_inputs(T, H, I, E, K, torch.bfloat16, seed=31, w_std=0.05, bias_std=0.1, zipf=0.7)
    g = to_dev(d, gpu)
    gy = torch.randn(T, H, generator=torch.Generator().manual_seed(4)).to(torch.bfloat16).to(gpu)
    a = args(g)
    eager_out = yamoe_amd.experts(*a, T, E, K)
    eager_grads = yamoe_amd.experts_backward(gy, *a, T, E, K)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        for _ in range(2):                                    # warm-up on the capture stream
            yamoe_amd.experts(*a, T, E, K)
            yamoe_amd.experts_backward(gy, *a, T, E, K)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        out = yamoe_amd.experts(*a, T, E, K)
        grads = yamoe_amd.experts_backward(gy, *a, T, E, K)
    for rep in range(3):
        out.zero_()
        for t in grads:
            t.fill_(7.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager_out), rep
        for got, want in zip(grads, eager_grads):
            assert torch.equal(got, want), rep
        yamoe_amd.experts(*a, T, E, K)                        # eager work between replays
        torch.cuda.synchronize()


def test_two_streams_at_once(gpu):
    """Calls on different streams share nothing but read-only per-device flags (each call carves its own workspace):
    two problems of different shapes and dtypes, forward and backward, issued alternately on two streams without a
    synchronisation in between, give the results of the same calls made one after the other, bit for bit."""
    import yamoe_amd
    shapes = [(900, 256, 128, 8, 2, torch.bfloat16, 5), (300, 192, 320, 4, 3, torch.float16, 6)]
    work, serial = [], []
    for T, H, I, E, K, dtype, seed in shapes:
        d = make_inputs(T, H, I, E, K, dtype, seed=seed, w_std=0.05, bias_std=0.1, zipf=0.5)
        g = to_dev(d, gpu)
        gy = torch.randn(T, H, generator=torch.Generator().manual_seed(seed)).to(dtype).to(gpu)
        work.append((gy, args(g), T, E, K))
    for gy, a, T, E, K in work:
        serial.append([yamoe_amd.experts(*a, T, E, K)] + list(yamoe_amd.experts_backward(gy, *a, T, E, K)))
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    for rep in range(3):
        got = [[], []]
        for it in range(4):  # alternate, so that launches of the two problems interleave on the device
            for i, (gy, a, T, E, K) in enumerate(work):
                with torch.cuda.stream(streams[i]):
                    r = [yamoe_amd.experts(*a, T, E, K)] + list(yamoe_amd.experts_backward(gy, *a, T, E, K))
                got[i] = r
        torch.cuda.synchronize()
        for i in range(2):
            for x, y in zip(got[i], serial[i]):
                assert torch.equal(x, y), (rep, i)
