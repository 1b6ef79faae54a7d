"""Where a tile of the forward GEMM kernels spends its clocks: a diagnostic build of the library with per-tile clock
stamps (gemm_async.hip compiled with -DYAMOE_TILE_STAMPS) and a run of the GPT-OSS-20B workload's two products on it.

    python -m yamoe_amd.tile_stamps build      compiles yamoe_amd/libyamoe_hip_stamps.so (no GPU needed)
    python -m yamoe_amd.tile_stamps            runs gate_up and down on it and prints the summary (needs the GPU)

Per tile the kernel leaves the shader clock at six points (workgroup entry, work-list look-ups done, first slab landed,
contraction loop done, epilogue values staged, stores issued) plus its shape and the CU it ran on.  The summary gives, per
tile shape, the median clocks of each phase and the loop's clocks per slab of 32 against the MFMA issue time of that
shape, and over the launch the share of the longest CU's span that a CU spends inside tiles.  The stamped build is a separate file; the
product library is not touched.
"""
import ctypes
import os
import sys

from . import build as b

LIB_STAMPS = os.path.join(b.HERE, "libyamoe_hip_stamps.so")


def build_stamped(verbose=True):
    os.makedirs(b.OBJ, exist_ok=True)
    objs = []
    for src in b.HIP_SOURCES:
        obj = os.path.join(b.OBJ, src.replace(".hip", ".o"))
        if src == "gemm_async.hip":
            obj = os.path.join(b.OBJ, "gemm_async_stamps.o")
            b._run([b.HIPCC] + b.HIP_FLAGS + ["-DYAMOE_TILE_STAMPS", "-c", os.path.join(b.CSRC, src), "-o", obj])
        elif not os.path.exists(obj):
            b._run([b.HIPCC] + b.HIP_FLAGS + ["-c", os.path.join(b.CSRC, src), "-o", obj])
        objs.append(obj)
    b._run([b.HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_STAMPS] + objs)
    if verbose:
        print("built", LIB_STAMPS)


def run():
    import numpy as np
    import torch

    from . import _cabi, workloads
    from .workloads import device_weights

    if not os.path.exists(LIB_STAMPS):
        raise SystemExit("%s is missing: run `python -m yamoe_amd.tile_stamps build` first" % LIB_STAMPS)
    dev = torch.device("cuda:0")
    cfg = workloads.CONFIGS["gptoss20b"]
    T, H, I, E, K = cfg["T"], cfg["H"], cfg["I"], cfg["E"], cfg["K"]
    host, _ = workloads.make_config("gptoss20b", seed=0, weights=False)
    d = {k: v.to(dev) for k, v in host.items()}
    d.update(device_weights(E, H, I, torch.bfloat16, cfg["w_std"], 1, dev))
    N = T * K
    se, si, counts, offsets, inv = _cabi.route(d["router_indices"], E, T)
    sched = _cabi.build_schedule(counts, offsets, N, T, 16)
    n_row_tiles = int(sched[0])
    L = ctypes.CDLL(LIB_STAMPS)
    vp, i32 = ctypes.c_void_p, ctypes.c_int32
    L.yamoe_gate_up.argtypes = [vp, vp, vp, vp, vp, vp, vp, i32, i32, i32, i32, i32, i32, vp]
    L.yamoe_down.argtypes = [vp, vp, vp, vp, vp, i32, i32, i32, i32, i32, vp]
    L.yamoe_debug_tile_stamps.argtypes = [vp, i32]
    L.yamoe_debug_tile_stamps.restype = None
    act = torch.empty(N, I, dtype=torch.bfloat16, device=dev)
    y = torch.empty(N, H, dtype=torch.bfloat16, device=dev)
    p, st = _cabi._p, _cabi._stream

    def gate_up():
        rc = L.yamoe_gate_up(p(d["hidden"]), p(si), p(d["gate_up_proj"]), p(d["gate_up_proj_bias"]), p(act), None, p(sched),
                             N, K, E, H, I, _cabi.BF16, st())
        assert rc == 0, rc

    def down():
        rc = L.yamoe_down(p(act), p(d["down_proj"]), p(d["down_proj_bias"]), p(y), p(sched), N, E, H, I, _cabi.BF16, st())
        assert rc == 0, rc

    import time
    for name, fn, n_col, kd in (("gate_up (+ bias + clamped SwiGLU)", gate_up, -(-2 * I // 256), H),
                                ("down (+ bias)", down, -(-H // 256), I)):
        tiles = n_row_tiles * n_col
        buf = torch.zeros(tiles * 8, dtype=torch.int64, device=dev)
        L.yamoe_debug_tile_stamps(None, 0)
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < 1.0:     # the engine clock needs load to leave its idle state
            for _ in range(20):
                fn()
            torch.cuda.synchronize()
        L.yamoe_debug_tile_stamps(p(buf), tiles)
        fn()
        torch.cuda.synchronize()
        L.yamoe_debug_tile_stamps(None, 0)
        s = buf.cpu().numpy().reshape(-1, 8)
        s = s[s[:, 0] > 0]
        rows, cols = s[:, 6] & 0xffff, s[:, 6] >> 16
        n_slabs = kd // 32
        print("== %s: %d tiles, contraction %d (%d slabs of 32)" % (name, len(s), kd, n_slabs))
        print("   phases in shader clocks (median over the tiles of a shape): look-ups = entry to first copy; first slab = "
              "first copy to first MFMA; loop; epilogue = bias / activation / staging in LDS; stores")
        print("   %-22s %6s %8s %10s %8s %9s %7s %8s %12s %10s" % ("rows x columns", "tiles", "look-ups", "first slab", "loop",
                                                                    "epilogue", "stores", "total", "loop / slab", "MFMA issue"))
        shapes = {}
        for r, c in zip(rows.tolist(), cols.tolist()):
            key = ((r + 31) // 32 * 32, c)
            shapes[key] = shapes.get(key, 0) + 1
        for (r32, c), cnt in sorted(shapes.items(), key=lambda kv: -kv[1])[:8]:
            m = (((rows + 31) // 32 * 32) == r32) & (cols == c)
            x = s[m]
            ph = [np.median(x[:, i + 1] - x[:, i]) for i in range(5)]
            total = np.median(x[:, 5] - x[:, 0])
            # MFMA issue clocks per slab: 2 k-steps x (row blocks of the busier wave row) x (column blocks per wave) x 32
            mi = ((r32 // 32) + 1) // 2
            ni = ((c + 31) // 32 + 1) // 2
            issue = 2 * mi * ni * 32
            print("   %-22s %6d %8.0f %10.0f %8.0f %9.0f %7.0f %8.0f %12.0f %10d" % (
                "%d (<= %d) x %d" % (r32, r32, c), cnt, ph[0], ph[1], ph[2], ph[3], ph[4], total, ph[2] / n_slabs, issue))
        # The counters of different CUs are not aligned with each other, so spans are taken CU by CU (first tile's entry
        # to last tile's end); they tick at one rate, and the longest of them is, to a tile start, the launch itself.
        dur = (s[:, 5] - s[:, 0]).astype(np.float64)
        cu = s[:, 7]
        spans, inside, per = [], [], []
        for c in np.unique(cu):
            m = cu == c
            spans.append(float(s[m, 5].max() - s[m, 0].min()))
            inside.append(dur[m].sum())
            per.append(int(m.sum()))
        spans, inside, per = np.array(spans), np.array(inside), np.array(per)
        launch = spans.max()
        print("   launch: %d CUs seen, %.1f tiles each (%d .. %d); the longest CU span (first entry to last end) is %.0f clocks; "
              "a CU is inside tiles %.1f %% of that on average (least busy %.1f %%, busiest %.1f %%) and %.1f %% of its own "
              "span (the rest: between two tiles)" % (len(per), per.mean(), per.min(), per.max(), launch,
                                                       100 * inside.mean() / launch, 100 * inside.min() / launch,
                                                       100 * inside.max() / launch, 100 * (inside / spans).mean()))
        xcc = s[:, 7] >> 8
        per_xcd = np.array([dur[xcc == x].sum() for x in np.unique(xcc)])
        cu_span_xcd = np.array([spans[[int(c) >> 8 == int(x) for c in np.unique(cu)]].max() for x in np.unique(xcc)])
        print("   per XCD: tile clocks %s (mean = 100); longest CU span %s (longest = 100)" % (
            " ".join("%.0f" % v for v in 100 * per_xcd / per_xcd.mean()), " ".join("%.0f" % v for v in 100 * cu_span_xcd / launch)))
        tot = dur.sum()
        parts = [(s[:, i + 1] - s[:, i]).astype(np.float64).sum() / tot for i in range(5)]
        print("   share of all tile clocks: look-ups %.1f %%, first slab %.1f %%, loop %.1f %%, epilogue %.1f %%, stores %.1f %%"
              % tuple(100 * v for v in parts))


if __name__ == "__main__":
    if len(sys.argv) > 1 and sys.argv[1] == "build":
        build_stamped()
    else:
        run()
