#!/usr/bin/env python3
"""Benchmark of the expert-layer forward on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One step = one `experts()` forward (torch op -> C ABI -> HIP kernels) over one synthetic batch of the
GPT-OSS-20B shaped layer: 4096 tokens, hidden = intermediate = 2880, 32 experts, top-4, bf16, inputs
already resident in HBM.  Prints ONE JSON line.  `value` is algorithmic TFLOP/s of the whole op
(6*H*I flop per kept (token, expert) assignment divided by the step time).

Also on the line:
  roofline      the dominant kernel (the gate_up grouped GEMM), timed on its own with HIP events on
                the stream it runs on: algorithmic flop per launch / average launch time vs the
                2.5 PFLOP/s dense bf16 MFMA peak
  decode        the 64-token / 128-expert decode workload: algorithmic HBM bytes per step / step time
                vs the 8 TB/s HBM peak
  cpu_baseline  the CPU oracle (oracle/yamoe_oracle.py, the loop-over-experts path the reference itself
                takes on a CPU) timed on this box's host cores on a slice of the same batch
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# the headline metric this file reports: `value` is its first part (forward TFLOP/s of the 20B shape), the `decode`
# object on the same line carries the second (GB/s and fraction of HBM peak)
METRIC = "experts() fwd TFLOP/s & %MFMA peak (20B shape, 4096 tok); decode GB/s %HBM"
PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0      # MI355X HBM3E

# HBM bytes per launch of the gate_up GEMM on the GPT-OSS-20B workload, from rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE runs of this file (profiles/gemm_async_and_stream_gemm_counters.md): 713 500 KiB fetched x 2.0
# (FETCH_SIZE reads half of a 1 GiB copy's bytes on this device) + 94 046 KiB written x 1.0.
GATE_UP_TRAFFIC_BYTES = 1.627e9


def spin_up(fn, ms):
    """Runs `fn` untimed for at least `ms` of wall time.  The device idles at a low engine clock and takes
    some hundreds of milliseconds of load to reach its sustained clock; a timed region that starts right
    after a handful of warm-up launches measures that ramp, not the kernels."""
    import torch
    if ms <= 0:
        return 0
    n, t0 = 0, time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < ms:
        for _ in range(20):
            fn()
        n += 20
        torch.cuda.synchronize()
    return n


def event_time_ms(fn, iters):
    import torch
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(iters):
        fn()
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / iters


def device_weights(E, H, I, dtype, std, seed, device):
    """Weights drawn on the device (N(0, std)); used where drawing on the host would take minutes."""
    import torch
    g = torch.Generator(device=device).manual_seed(seed)

    def draw(shape):
        t = torch.empty(shape, dtype=dtype, device=device)
        for e in range(shape[0]):
            t[e] = (torch.randn(shape[1:], generator=g, device=device) * std).to(dtype)
        return t
    return dict(gate_up_proj=draw((E, H, 2 * I)), gate_up_proj_bias=draw((E, 2 * I)), down_proj=draw((E, I, H)),
                down_proj_bias=draw((E, H)))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--spinup-ms", type=float, default=1000.0,
                    help="untimed load before each timed region so that the engine clock has left its idle state")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-decode", action="store_true")
    ap.add_argument("--extras", action="store_true",
                    help="also time the backward (GPT-OSS-20B shape), the Zipf-skewed and the README fp32 workloads")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one 1 GiB device-to-device copy kernel (a known FETCH_SIZE / WRITE_SIZE for counter runs)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus %d is not supported (the expert layer here is the "
              "single-GPU share of an expert-parallel layout)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    import yamoe_amd
    from yamoe_amd import _cabi, workloads

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.calibrate_copy:
        src = torch.ones(1 << 28, dtype=torch.float32, device=dev)  # 1 GiB
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # ---------------- GPT-OSS-20B shaped layer ----------------------------------------------------------
    cfg = workloads.CONFIGS["gptoss20b"]
    T, H, I, E, K = cfg["T"], cfg["H"], cfg["I"], cfg["E"], cfg["K"]
    host, _ = workloads.make_config("gptoss20b", seed=0, weights=False)
    d = {k: v.to(dev) for k, v in host.items()}
    d.update(device_weights(E, H, I, torch.bfloat16, cfg["w_std"], 1, dev))
    order = ("hidden", "router_indices", "routing_weights", "gate_up_proj", "gate_up_proj_bias", "down_proj",
             "down_proj_bias")
    a = [d[k] for k in order]
    n_rows = T * K  # capacity = T keeps every assignment
    flop = n_rows * workloads.FWD_FLOP_PER_ROW(H, I)

    def step():
        return yamoe_amd.experts(*a, T, E, K)

    spin_up(step, args.spinup_ms)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ev_ms = event_time_ms(step, args.steps)
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    ms_per_step = max(ev_ms, wall_ms)
    value = flop / (ms_per_step * 1e-3) / 1e12

    # ---------------- dominant kernel on its own: gate_up grouped GEMM -----------------------------------
    se, si, counts, offsets, inv = _cabi.route(d["router_indices"], E, T)
    sched = _cabi.build_schedule(counts, offsets, n_rows, T, 16)
    act = _cabi.gate_up(d["hidden"], si, d["gate_up_proj"], d["gate_up_proj_bias"], sched, K)

    def gu_launch():
        _cabi.lib().yamoe_gate_up(
            _cabi._p(d["hidden"]), _cabi._p(si), _cabi._p(d["gate_up_proj"]), _cabi._p(d["gate_up_proj_bias"]),
            _cabi._p(act), None, _cabi._p(sched), n_rows, K, E, H, I, _cabi.BF16, _cabi._stream())
    spin_up(gu_launch, args.spinup_ms / 2)
    gu_ms = event_time_ms(gu_launch, args.steps)
    y = _cabi.down(act, d["down_proj"], d["down_proj_bias"], sched)

    def dn_launch():
        _cabi.lib().yamoe_down(
            _cabi._p(act), _cabi._p(d["down_proj"]), _cabi._p(d["down_proj_bias"]), _cabi._p(y), _cabi._p(sched),
            n_rows, E, H, I, _cabi.BF16, _cabi._stream())
    spin_up(dn_launch, args.spinup_ms / 2)
    dn_ms = event_time_ms(dn_launch, args.steps)
    gu_flop = n_rows * 4 * H * I
    gu_tflops = gu_flop / (gu_ms * 1e-3) / 1e12
    dn_tflops = n_rows * 2 * H * I / (dn_ms * 1e-3) / 1e12
    roofline = dict(bound="mfma", kernel="gemm_async_kernel<bf16, gate_up + clamped SwiGLU>", achieved=round(gu_tflops, 2),
                    peak=PEAK_BF16_TFLOPS, unit="TFLOP/s", frac=round(gu_tflops / PEAK_BF16_TFLOPS, 4),
                    traffic=GATE_UP_TRAFFIC_BYTES, avg_launch_ms=round(gu_ms, 4),
                    down_gemm=dict(achieved=round(dn_tflops, 2), frac=round(dn_tflops / PEAK_BF16_TFLOPS, 4),
                                   avg_launch_ms=round(dn_ms, 4)))

    # ---------------- CPU baseline on a slice of the same batch ------------------------------------------
    cpu_baseline = None
    parity = None
    if not args.no_cpu_baseline:
        from oracle import yamoe_oracle as O
        sample_tokens = T  # the whole batch; repeated until about 10 s of CPU work have been timed
        torch.set_num_threads(min(os.cpu_count() or 1, 16))
        # inputs are converted to the fp32 compute type once, outside the timed region
        hs = {k: d[k][:sample_tokens].cpu() if k in ("hidden", "router_indices", "routing_weights") else d[k].cpu()
              for k in order}
        hs = {k: (v.float() if v.is_floating_point() else v) for k, v in hs.items()}
        hargs = [hs[k] for k in order]
        O.experts_loop(*[t[:64] if i < 3 else t for i, t in enumerate(hargs)], compute_dtype=torch.float32)  # warm-up
        times = []
        while len(times) < 3 or sum(times) < 10.0:
            t1 = time.perf_counter()
            ref = O.experts_loop(*hargs, compute_dtype=torch.float32)
            times.append(time.perf_counter() - t1)
        cpu_s = sorted(times)[len(times) // 2]
        cpu_flop = sample_tokens * K * workloads.FWD_FLOP_PER_ROW(H, I)
        cpu_baseline = dict(value=round(cpu_flop / cpu_s / 1e12, 4), unit="TFLOP/s", cores=torch.get_num_threads(),
                            kind="port", sample="all %d tokens of the same batch, fp32 compute on the bf16 inputs, "
                            "median of %d runs (%.2f s each, %.1f s in all)" % (sample_tokens, len(times), cpu_s, sum(times)))
        got = step()[:sample_tokens].float().cpu()
        parity = dict(rel_l2=float("%.3e" % O.rel_l2(got, ref)), max_abs=float("%.3e" % O.max_abs(got, ref)),
                      tolerance=1e-2, against="fp32 oracle on all %d tokens" % sample_tokens)
        del hs, hargs

    # ---------------- decode workload: 64 tokens, 128 experts ---------------------------------------------
    decode = None
    if not args.no_decode:
        del d, a, act, y
        torch.cuda.empty_cache()
        dc = workloads.CONFIGS["decode"]
        Td, Ed, Kd = dc["T"], dc["E"], dc["K"]
        hostd, _ = workloads.make_config("decode", seed=0, weights=False)
        dd = {k: v.to(dev) for k, v in hostd.items()}
        dd.update(device_weights(Ed, H, I, torch.bfloat16, dc["w_std"], 2, dev))
        ad = [dd[k] for k in order]
        n_active = int((np.bincount(hostd["router_indices"].numpy().ravel(), minlength=Ed) > 0).sum())
        nbytes = workloads.algorithmic_bytes_decode(n_active, Td, Kd, Ed, H, I)

        def dstep():
            return yamoe_amd.experts(*ad, Td, Ed, Kd)

        spin_up(dstep, args.spinup_ms)
        for _ in range(args.warmup):
            dstep()
        d_ms = event_time_ms(dstep, args.steps)
        gbs = nbytes / (d_ms * 1e-3) / 1e9
        decode = dict(metric="experts_fwd_decode_hbm_gbs", value=round(gbs, 1), unit="GB/s", ms_per_step=round(d_ms, 4),
                      frac_of_hbm_peak=round(gbs / PEAK_HBM_GBS, 4), peak=PEAK_HBM_GBS, active_experts=n_active,
                      algorithmic_bytes=nbytes,
                      config=dict(workload="decode: T=64 H=I=2880 E=128 top-4 bf16", tokens=Td, experts=Ed, top_k=Kd))

    extras = None
    if args.extras:
        extras = {}
        try:
            del dd, ad
        except NameError:
            del d, a, act, y
        torch.cuda.empty_cache()

        def timed(fn, n_flop, label, iters=max(3, args.steps // 4)):
            spin_up(fn, args.spinup_ms)
            ms = event_time_ms(fn, iters)
            extras[label] = dict(ms=round(ms, 4), tflops=round(n_flop / (ms * 1e-3) / 1e12, 2),
                                 frac_of_peak=round(n_flop / (ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, 4))

        # backward at the GPT-OSS-20B shape: 18*H*I flop per assignment (forward recompute + dgrad + wgrad)
        hostb, _ = workloads.make_config("gptoss20b", seed=0, weights=False)
        db = {k: v.to(dev) for k, v in hostb.items()}
        db.update(device_weights(E, H, I, torch.bfloat16, cfg["w_std"], 1, dev))
        ab = [db[k] for k in order]
        gy = torch.randn(T, H, device=dev, generator=torch.Generator(device=dev).manual_seed(3)).to(torch.bfloat16)
        timed(lambda: yamoe_amd.experts_backward(gy, *ab, T, E, K), T * K * 18 * H * I, "backward_gptoss20b_bf16")
        del db, ab, gy
        torch.cuda.empty_cache()
        # Zipf-skewed routing, 16384 tokens, 128 experts
        zc = workloads.CONFIGS["zipf"]
        hostz, _ = workloads.make_config("zipf", seed=0, weights=False)
        dz = {k: v.to(dev) for k, v in hostz.items()}
        dz.update(device_weights(zc["E"], H, I, torch.bfloat16, zc["w_std"], 4, dev))
        az = [dz[k] for k in order]
        timed(lambda: yamoe_amd.experts(*az, zc["T"], zc["E"], zc["K"]), zc["T"] * zc["K"] * 6 * H * I,
              "forward_zipf_bf16")
        cz = np.bincount(hostz["router_indices"].numpy().ravel(), minlength=zc["E"])
        n_z = zc["T"] * zc["K"]
        w_bytes = int((cz > 0).sum()) * 3 * H * I * 2               # weights of the non-empty experts, read once
        roof_ms = max(n_z * 6 * H * I / (PEAK_BF16_TFLOPS * 1e12), w_bytes / (PEAK_HBM_GBS * 1e9)) * 1e3
        extras["forward_zipf_bf16"].update(max_rows=int(cz.max()), empty_experts=int((cz == 0).sum()),
                                           roofline_ms=round(roof_ms, 4))
        # its routing kernels (three launches at this N) and the row permute on their own
        r_ms = event_time_ms(lambda: _cabi.route(dz["router_indices"], zc["E"], zc["T"]), 50)
        se_z, si_z, _, _, _ = _cabi.route(dz["router_indices"], zc["E"], zc["T"])
        p_ms = event_time_ms(lambda: _cabi.permute(dz["hidden"], si_z, zc["K"]), 50)
        extras["routing_zipf"] = dict(assignments=n_z, route_ms=round(r_ms, 4), permute_ms=round(p_ms, 4),
                                      permute_gbs=round((2 * n_z * H * 2 + 4 * n_z) / (p_ms * 1e-3) / 1e9, 1))
        del se_z, si_z
        del dz, az
        torch.cuda.empty_cache()
        # README shape, fp32 (peak 157.3 TFLOP/s fp32 MFMA)
        rc = workloads.CONFIGS["readme"]
        hostr, _ = workloads.make_config("readme", seed=42, weights=False)
        dr = {k: v.to(dev) for k, v in hostr.items()}
        dr.update(device_weights(rc["E"], H, I, torch.float32, 1.0, 5, dev))
        dr["gate_up_proj_bias"].zero_()
        dr["down_proj_bias"].zero_()
        ar = [dr[k] for k in order]
        timed(lambda: yamoe_amd.experts(*ar, rc["T"], rc["E"], rc["K"]), rc["T"] * rc["K"] * 6 * H * I,
              "forward_readme_fp32")
        extras["forward_readme_fp32"]["frac_of_peak"] = round(extras["forward_readme_fp32"]["tflops"] / 157.3, 4)

        del dr, ar
        torch.cuda.empty_cache()
        # For scale: the vendor library's dense GEMM (torch.matmul) on the same flop counts and operand layouts as the
        # two forward GEMMs: [T*K, H] x [H, 2I] and [T*K, I] x [I, H], one matrix instead of 32 experts, no bias, no GLU.
        gl = torch.Generator(device=dev).manual_seed(7)
        xa = torch.randn(T * K, H, device=dev, generator=gl).to(torch.bfloat16)
        for label, n_out in (("library_dense_gemm_gate_up_shape", 2 * I), ("library_dense_gemm_down_shape", H)):
            wb = (torch.randn(H, n_out, device=dev, generator=gl) * 0.02).to(torch.bfloat16)
            timed(lambda: torch.matmul(xa, wb), 2 * T * K * H * n_out, label)
            del wb
        del xa

    line = dict(metric=METRIC, value=round(value, 2), unit="TFLOP/s", n_gpus=1, steps=args.steps,
                warmup=args.warmup, spinup_ms=args.spinup_ms, ms_per_step=round(ms_per_step, 4), higher_is_better=True, scaling="weak",
                vs_baseline=None, dtype="bf16", data="synthetic",
                config=dict(workload="gptoss20b: T=4096 H=I=2880 E=32 top-4 bf16, clamped SwiGLU, capacity=T",
                            tokens=T, hidden=H, intermediate=I, experts=E, top_k=K,
                            algorithmic_flop=flop),
                frac_of_mfma_peak=round(value / PEAK_BF16_TFLOPS, 4), roofline=roofline, cpu_baseline=cpu_baseline,
                parity=parity, decode=decode, extras=extras)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
