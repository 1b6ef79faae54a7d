#!/usr/bin/env python3
"""Benchmark of the expert-layer path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One step = one `experts()` forward (torch op -> C ABI -> HIP kernels) over one synthetic batch of the
GPT-OSS-20B shaped layer: 4096 tokens, hidden = intermediate = 2880, 32 experts, top-4, bf16, inputs
already resident in HBM.  Prints ONE JSON line.  `value` is algorithmic TFLOP/s of the whole op
(6*H*I flop per kept (token, expert) assignment divided by the step time).

Also on the line:
  roofline      the dominant kernel (the gate_up grouped GEMM), timed on its own with HIP events on
                the stream it runs on: algorithmic flop per launch / average launch time vs the
                2.5 PFLOP/s dense bf16 MFMA peak; `traffic` (HBM bytes per launch) is read from the
                counter summary kept under profiles/ and says so
  cpu_baseline  the CPU oracle (oracle/yamoe_oracle.py, the loop-over-experts path the reference itself
                takes on a CPU) timed on this box's host cores on the same batch
  parity        the timed op's output against that oracle run
  configs       all five measured workloads, each with its time, its rate against its own peak (fp32 or bf16
                MFMA, HBM for the decode shape) and its parity against the oracle:
                cfg1 README shape fp32, cfg2 the headline, cfg3 decode, cfg4 Zipf-skewed, cfg5 backward;
                and the 128-expert layer of the decode shape at 512 .. 4096 tokens (between decode and prefill),
                each against max(flop / MFMA peak, weight bytes / HBM peak)
  decode        the cfg3 entry again under the name the metric gives it
"""
import argparse
import ctypes
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
PEAK_FP32_TFLOPS = 157.3   # MI355X fp32 matrix
PEAK_HBM_GBS = 8000.0      # MI355X HBM3E
ORDER = ("hidden", "router_indices", "routing_weights", "gate_up_proj", "gate_up_proj_bias", "down_proj",
         "down_proj_bias")
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "gate_up_traffic.json")


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


def parity_of(got, want, tol, against):
    from oracle import yamoe_oracle as O
    return dict(rel_l2=float("%.3e" % O.rel_l2(got, want)), max_abs=float("%.3e" % O.max_abs(got, want)),
                tolerance=tol, against=against)


def recorded_traffic():
    """HBM bytes per launch of the gate_up GEMM from the committed counter summary (not measured by this run)."""
    try:
        with open(TRAFFIC_FILE) as f:
            t = json.load(f)
        return float(t["bytes_per_launch"]), "profiles/gate_up_traffic.json (%s)" % t.get("from", "counter run")
    except (OSError, KeyError, ValueError):
        return None, None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--spinup-ms", type=float, default=1000.0,
                    help="untimed load before each timed region so that the engine clock has left its idle state")
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the CPU oracle (no cpu_baseline, no parity)")
    ap.add_argument("--no-configs", action="store_true",
                    help="only the headline workload and its dominant kernel (for profiler runs)")
    ap.add_argument("--only", default="", help="with --no-configs: also run this one of decode, mid, zipf, readme, backward")
    ap.add_argument("--extras", action="store_true",
                    help="also time the vendor library's dense GEMM on the two forward GEMM shapes, the routing and "
                         "permute kernels of the Zipf workload on their own, the gate_up launch on zero weights "
                         "(how much of its time is the power limit) and a register-only MFMA loop on random and on "
                         "zero operands (what the matrix pipes sustain with nothing else going on)")
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
    from yamoe_amd.workloads import device_weights

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    torch.set_num_threads(min(os.cpu_count() or 1, 16))
    check = not args.no_cpu_baseline
    if check:
        from oracle import yamoe_oracle as O

    def wanted(name):
        return not args.no_configs or args.only == name

    if args.calibrate_copy:
        src = torch.ones(1 << 28, dtype=torch.float32, device=dev)  # 1 GiB
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    configs = {}

    # ---------------- cfg2: GPT-OSS-20B shaped layer (the headline) --------------------------------------
    cfg = workloads.CONFIGS["gptoss20b"]
    T, H, I, E, K = cfg["T"], cfg["H"], cfg["I"], cfg["E"], cfg["K"]
    host, _ = workloads.make_config("gptoss20b", seed=0, weights=False)
    d = {k: v.to(dev) for k, v in host.items()}
    d.update(device_weights(E, H, I, torch.bfloat16, cfg["w_std"], 1, dev))
    a = [d[k] for k in ORDER]
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
    kernel_iters = max(args.steps, 200)  # the isolated launches are timed over at least 200 of them whatever --steps says
    gu_ms = event_time_ms(gu_launch, kernel_iters)
    y = _cabi.down(act, d["down_proj"], d["down_proj_bias"], sched)

    def dn_launch():
        _cabi.lib().yamoe_down(
            _cabi._p(act), _cabi._p(d["down_proj"]), _cabi._p(d["down_proj_bias"]), _cabi._p(y), _cabi._p(sched),
            n_rows, E, H, I, _cabi.BF16, _cabi._stream())
    spin_up(dn_launch, args.spinup_ms / 2)
    dn_ms = event_time_ms(dn_launch, kernel_iters)
    gu_flop = n_rows * 4 * H * I
    gu_tflops = gu_flop / (gu_ms * 1e-3) / 1e12
    dn_tflops = n_rows * 2 * H * I / (dn_ms * 1e-3) / 1e12
    traffic, traffic_source = recorded_traffic()
    roofline = dict(bound="mfma", kernel="gemm_async_kernel<bf16, gate_up + clamped SwiGLU>", achieved=round(gu_tflops, 2),
                    peak=PEAK_BF16_TFLOPS, unit="TFLOP/s", frac=round(gu_tflops / PEAK_BF16_TFLOPS, 4),
                    traffic=traffic, traffic_source=traffic_source, algorithmic_flop_per_launch=gu_flop,
                    avg_launch_ms=round(gu_ms, 4), launches_timed=kernel_iters,
                    down_gemm=dict(achieved=round(dn_tflops, 2), frac=round(dn_tflops / PEAK_BF16_TFLOPS, 4),
                                   avg_launch_ms=round(dn_ms, 4)))
    data_dependence = None
    if args.extras:
        # the same gate_up launch on operands that do not toggle the datapath: how much of the time is the power limit
        zero_w = torch.zeros_like(d["gate_up_proj"])

        def gu_zero():
            _cabi.lib().yamoe_gate_up(
                _cabi._p(d["hidden"]), _cabi._p(si), _cabi._p(zero_w), _cabi._p(d["gate_up_proj_bias"]),
                _cabi._p(act), None, _cabi._p(sched), n_rows, K, E, H, I, _cabi.BF16, _cabi._stream())
        spin_up(gu_zero, args.spinup_ms)
        z_ms = event_time_ms(gu_zero, args.steps)
        spin_up(gu_launch, args.spinup_ms)
        r_ms = event_time_ms(gu_launch, args.steps)
        data_dependence = dict(gate_up_random_data_ms=round(r_ms, 4), gate_up_zero_weights_ms=round(z_ms, 4),
                               tflops_zero_weights=round(gu_flop / (z_ms * 1e-3) / 1e12, 1))
        del zero_w
    del act, y

    # ---------------- CPU baseline on the same batch, and the parity of the timed op ---------------------
    cpu_baseline = None
    parity = None
    hs = None
    if check:
        # inputs are converted to the fp32 compute type once, outside the timed region
        hs = {k: d[k].cpu() for k in ORDER}
        hs = {k: (v.float() if v.is_floating_point() else v) for k, v in hs.items()}
        hargs = [hs[k] for k in ORDER]
        O.experts_loop(*[t[:64] if i < 3 else t for i, t in enumerate(hargs)], compute_dtype=torch.float32)  # warm-up
        times = []
        while len(times) < 3 or sum(times) < 10.0:
            t1 = time.perf_counter()
            ref = O.experts_loop(*hargs, compute_dtype=torch.float32)
            times.append(time.perf_counter() - t1)
        cpu_s = sorted(times)[len(times) // 2]
        cpu_baseline = dict(value=round(flop / cpu_s / 1e12, 4), unit="TFLOP/s", cores=torch.get_num_threads(),
                            kind="port", sample="all %d tokens of the same batch, fp32 compute on the bf16 inputs, "
                            "median of %d runs (%.2f s each, %.1f s in all)" % (T, len(times), cpu_s, sum(times)))
        parity = parity_of(step().float().cpu(), ref, 1e-2, "fp32 oracle on all %d tokens" % T)
        del ref
    configs["cfg2_gptoss20b_forward_bf16"] = dict(
        ms=round(ms_per_step, 4), tflops=round(value, 2), frac_of_peak=round(value / PEAK_BF16_TFLOPS, 4),
        peak="bf16 MFMA %.0f TFLOP/s" % PEAK_BF16_TFLOPS, parity=parity)

    def timed(fn, iters):
        spin_up(fn, args.spinup_ms)
        return event_time_ms(fn, iters)

    few = max(3, args.steps // 4)

    # ---------------- cfg5: backward at the same shape ------------------------------------------------------
    if wanted("backward"):
        gy = torch.randn(T, H, device=dev, generator=torch.Generator(device=dev).manual_seed(3)).to(torch.bfloat16)
        ms = timed(lambda: yamoe_amd.experts_backward(gy, *a, T, E, K), few)
        b_flop = n_rows * 18 * H * I  # forward recompute 6 + input gradients 6 + weight gradients 6 (per assignment, x H*I)
        tf = b_flop / (ms * 1e-3) / 1e12
        entry = dict(ms=round(ms, 4), tflops=round(tf, 2), frac_of_peak=round(tf / PEAK_BF16_TFLOPS, 4),
                     peak="bf16 MFMA %.0f TFLOP/s" % PEAK_BF16_TFLOPS, algorithmic_flop=b_flop, parity=None)
        if check:
            grads = [g.float().cpu() for g in yamoe_amd.experts_backward(gy, *a, T, E, K)]
            want = O.experts_backward(gy.cpu(), *[hs[k] for k in ORDER], T, compute_dtype=torch.float32)
            names = ("d_hidden", "d_routing", "d_gate_up_proj", "d_gate_up_proj_bias", "d_down_proj", "d_down_proj_bias")
            per = {n: float("%.3e" % O.rel_l2(g, w)) for n, g, w in zip(names, grads, want)}
            entry["parity"] = dict(rel_l2=max(per.values()), per_gradient=per, tolerance=1e-2,
                                   against="fp32 autograd through the oracle, all six gradients (worst shown)")
            del grads, want
        configs["cfg5_gptoss20b_backward_bf16"] = entry

        # a training step of the layer: forward + backward.  With the reference's interface the backward recomputes the
        # first product (experts + experts_backward); the pair experts_keep / experts_backward_kept hands the forward's
        # activations over instead (T*K*3*I values of memory).
        def step_recompute():
            yamoe_amd.experts(*a, T, E, K)
            yamoe_amd.experts_backward(gy, *a, T, E, K)

        def step_kept():
            _, kept = yamoe_amd.experts_keep(*a, T, E, K)
            yamoe_amd.experts_backward_kept(gy, *a, kept, T, E, K)

        ms_re, ms_kept = timed(step_recompute, few), timed(step_kept, few)
        ms_bk = timed(lambda kept=yamoe_amd.experts_keep(*a, T, E, K)[1]: yamoe_amd.experts_backward_kept(gy, *a, kept, T, E, K), few)
        configs["train_step_gptoss20b_bf16"] = dict(
            ms_forward_plus_backward=round(ms_re, 4), ms_with_kept_activations=round(ms_kept, 4),
            ms_backward_kept_alone=round(ms_bk, 4), kept_bytes=int(n_rows * 3 * I * 2),
            note="forward + backward of one layer call; 'kept' = experts_keep + experts_backward_kept (no recomputation of "
                 "the gate_up product in the backward)")
        del gy
    del d, a, hs
    torch.cuda.empty_cache()

    # ---------------- cfg3: decode, 64 tokens, 128 experts ---------------------------------------------------
    decode = None
    if wanted("decode") or wanted("mid"):
        dc = workloads.CONFIGS["decode"]
        Td, Ed, Kd = dc["T"], dc["E"], dc["K"]
        hostd, _ = workloads.make_config("decode", seed=0, weights=False)
        dd = {k: v.to(dev) for k, v in hostd.items()}
        dd.update(device_weights(Ed, H, I, torch.bfloat16, dc["w_std"], 2, dev))
        ad = [dd[k] for k in ORDER]
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
                      algorithmic_bytes=nbytes, parity=None,
                      config=dict(workload="decode: T=64 H=I=2880 E=128 top-4 bf16", tokens=Td, experts=Ed, top_k=Kd))
        if check:
            want = O.experts_capacity(*[dd[k].cpu() for k in ORDER], Td, compute_dtype=torch.float32)
            decode["parity"] = parity_of(dstep().float().cpu(), want, 1e-2, "fp32 oracle, all 64 tokens, device-drawn weights copied back")
        configs["cfg3_decode_bf16"] = dict(ms=round(d_ms, 4), gbs=round(gbs, 1), frac_of_peak=round(gbs / PEAK_HBM_GBS, 4),
                                           peak="HBM %.0f GB/s" % PEAK_HBM_GBS, parity=decode["parity"])
        decode_batches = None
        if args.extras:
            # the same layer with the first 1, 2, 4, ... of the 64 tokens: few experts, little to hide latency behind
            decode_batches = {}
            for tb in (1, 2, 4, 8, 16, 32):
                ab = [dd["hidden"][:tb].contiguous(), dd["router_indices"][:tb].contiguous(),
                      dd["routing_weights"][:tb].contiguous()] + ad[3:]
                act_b = int((np.bincount(hostd["router_indices"][:tb].numpy().ravel(), minlength=Ed) > 0).sum())
                nb = workloads.algorithmic_bytes_decode(act_b, tb, Kd, Ed, H, I)

                def bstep():
                    return yamoe_amd.experts(*ab, tb, Ed, Kd)
                spin_up(bstep, args.spinup_ms / 4)
                b_ms = event_time_ms(bstep, args.steps)
                decode_batches["tokens_%d" % tb] = dict(us=round(b_ms * 1e3, 1), active_experts=act_b,
                                                        gbs=round(nb / (b_ms * 1e-3) / 1e9, 1))
        # ---------------- between decode and prefill: the same 128-expert layer at 512 .. 4096 tokens ----------
        # (16 .. 128 rows per expert: every expert a single row tile; bound by the weight stream like the decode
        # shape, with matrix work that grows with the tokens; reuses the decode workload's weights)
        if wanted("mid"):
            for name in ("mid512", "mid1024", "mid2048", "mid4096"):
                mc = workloads.CONFIGS[name]
                hostm, _ = workloads.make_config(name, seed=0, weights=False)
                am = [hostm[k].to(dev) for k in ORDER[:3]] + ad[3:]
                ms = timed(lambda: yamoe_amd.experts(*am, mc["T"], Ed, Kd), few)
                cm = np.bincount(hostm["router_indices"].numpy().ravel(), minlength=Ed)
                w_bytes = int((cm > 0).sum()) * 3 * H * I * 2
                m_flop = mc["T"] * Kd * 6 * H * I
                roof_ms = max(m_flop / (PEAK_BF16_TFLOPS * 1e12), w_bytes / (PEAK_HBM_GBS * 1e9)) * 1e3
                entry = dict(ms=round(ms, 4), weight_gbs=round(w_bytes / (ms * 1e-3) / 1e9, 1),
                             tflops=round(m_flop / (ms * 1e-3) / 1e12, 1), roofline_ms=round(roof_ms, 4),
                             frac_of_roofline=round(roof_ms / ms, 4), rows_per_expert=[int(cm.min()), int(cm.max())],
                             peak="max(flop / %.0f TFLOP/s, weight bytes / %.0f GB/s)" % (PEAK_BF16_TFLOPS, PEAK_HBM_GBS),
                             parity=None)
                if check and name in ("mid512", "mid4096"):
                    got = yamoe_amd.experts(*am, mc["T"], Ed, Kd).float().cpu()
                    want = O.experts_capacity(*([hostm[k] for k in ORDER[:3]] + [t.cpu() for t in ad[3:]]), mc["T"],
                                              compute_dtype=torch.float32)
                    entry["parity"] = parity_of(got, want, 1e-2, "fp32 oracle, all %d tokens, device-drawn weights copied back" % mc["T"])
                    del got, want
                configs["%s_128experts_forward_bf16" % name] = entry
                del am
        del dd, ad
        torch.cuda.empty_cache()

    # ---------------- cfg4: Zipf-skewed routing, 16384 tokens, 128 experts -----------------------------------
    extras = dict(gate_up_data_dependence=data_dependence) if args.extras else None
    if args.extras and wanted("decode"):
        extras["decode_small_batches"] = decode_batches
    if wanted("zipf"):
        zc = workloads.CONFIGS["zipf"]
        hostz, _ = workloads.make_config("zipf", seed=0, weights=False)
        dz = {k: v.to(dev) for k, v in hostz.items()}
        dz.update(device_weights(zc["E"], H, I, torch.bfloat16, zc["w_std"], 4, dev))
        az = [dz[k] for k in ORDER]
        n_z = zc["T"] * zc["K"]
        ms = timed(lambda: yamoe_amd.experts(*az, zc["T"], zc["E"], zc["K"]), few)
        cz = np.bincount(hostz["router_indices"].numpy().ravel(), minlength=zc["E"])
        w_bytes = int((cz > 0).sum()) * 3 * H * I * 2               # weights of the non-empty experts, read once
        z_flop = n_z * 6 * H * I
        roof_ms = max(z_flop / (PEAK_BF16_TFLOPS * 1e12), w_bytes / (PEAK_HBM_GBS * 1e9)) * 1e3
        tf = z_flop / (ms * 1e-3) / 1e12
        entry = dict(ms=round(ms, 4), tflops=round(tf, 2), frac_of_peak=round(tf / PEAK_BF16_TFLOPS, 4),
                     peak="bf16 MFMA %.0f TFLOP/s" % PEAK_BF16_TFLOPS, max_rows=int(cz.max()),
                     empty_experts=int((cz == 0).sum()), roofline_ms=round(roof_ms, 4), parity=None)
        if check:
            got = yamoe_amd.experts(*az, zc["T"], zc["E"], zc["K"]).float().cpu()
            want = O.experts_capacity(*[dz[k].cpu() for k in ORDER], zc["T"], compute_dtype=torch.float32)
            entry["parity"] = parity_of(got, want, 1e-2, "fp32 oracle, all 16384 tokens, device-drawn weights copied back")
            del got, want
        configs["cfg4_zipf_forward_bf16"] = entry
        if args.extras:
            # its routing kernels (three launches at this N) and the row permute on their own
            r_ms = event_time_ms(lambda: _cabi.route(dz["router_indices"], zc["E"], zc["T"]), 50)
            se_z, si_z, _, _, _ = _cabi.route(dz["router_indices"], zc["E"], zc["T"])
            p_ms = event_time_ms(lambda: _cabi.permute(dz["hidden"], si_z, zc["K"]), 50)
            extras["routing_zipf"] = dict(assignments=n_z, route_ms=round(r_ms, 4), permute_ms=round(p_ms, 4),
                                          permute_gbs=round((2 * n_z * H * 2 + 4 * n_z) / (p_ms * 1e-3) / 1e9, 1))
            del se_z, si_z
        del dz, az
        torch.cuda.empty_cache()

    # ---------------- cfg1: README shape, fp32 -----------------------------------------------------------------
    if wanted("readme"):
        rc = workloads.CONFIGS["readme"]
        hostr, _ = workloads.make_config("readme", seed=42, weights=False)
        dr = {k: v.to(dev) for k, v in hostr.items()}
        dr.update(device_weights(rc["E"], H, I, torch.float32, 1.0, 5, dev, bias_std=0.0))
        ar = [dr[k] for k in ORDER]
        ms = timed(lambda: yamoe_amd.experts(*ar, rc["T"], rc["E"], rc["K"]), few)
        r_flop = rc["T"] * rc["K"] * 6 * H * I
        tf = r_flop / (ms * 1e-3) / 1e12
        entry = dict(ms=round(ms, 4), tflops=round(tf, 2), frac_of_peak=round(tf / PEAK_FP32_TFLOPS, 4),
                     peak="fp32 MFMA %.1f TFLOP/s" % PEAK_FP32_TFLOPS, parity=None)
        if check:
            got = yamoe_amd.experts(*ar, rc["T"], rc["E"], rc["K"]).cpu()
            want = O.experts_capacity(*[dr[k].cpu() for k in ORDER], rc["T"], compute_dtype=torch.float64)
            entry["parity"] = parity_of(got, want, 1e-5, "fp64 oracle, all 4096 tokens, device-drawn weights copied back")
            del got, want
        configs["cfg1_readme_forward_fp32"] = entry
        del dr, ar
        torch.cuda.empty_cache()

    if args.extras:
        # What the matrix pipes themselves sustain: a register-only loop of v_mfma_f32_32x32x16_bf16 (one wave per SIMD
        # on every CU, 4 x 4 accumulator blocks: the forward tile's wave shape, no memory traffic) on pseudo-random and
        # on all-zero operands.  The part runs against its power limit, so the two differ; the random-operand figure,
        # not the 2.5 PFLOP/s peak, is the ceiling of any bf16 GEMM on real data here.
        sink = torch.zeros(4, device=dev)
        flop_out = ctypes.c_double(0.0)
        cus = torch.cuda.get_device_properties(dev).multi_processor_count
        probe = {}
        for label, rnd in (("random_operands", 1), ("zero_operands", 0)):
            def mfma_loop():
                rc = _cabi.lib().yamoe_probe_mfma_rate(cus, 4000, rnd, _cabi._p(sink), ctypes.byref(flop_out), _cabi._stream())
                assert rc == 0
            spin_up(mfma_loop, args.spinup_ms)
            ms = event_time_ms(mfma_loop, 20)
            probe[label] = dict(ms=round(ms, 4), tflops=round(flop_out.value / (ms * 1e-3) / 1e12, 1),
                                frac_of_peak=round(flop_out.value / (ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, 4))
        probe["workgroups"] = cus
        extras["mfma_register_loop"] = probe
        # For scale: the vendor library's dense GEMM (torch.matmul) on the same flop counts and operand layouts as the
        # two forward GEMMs: [T*K, H] x [H, 2I] and [T*K, I] x [I, H], one matrix instead of 32 experts, no bias, no GLU.
        gl = torch.Generator(device=dev).manual_seed(7)
        xa = torch.randn(T * K, H, device=dev, generator=gl).to(torch.bfloat16)
        for label, n_out in (("library_dense_gemm_gate_up_shape", 2 * I), ("library_dense_gemm_down_shape", H)):
            wb = (torch.randn(H, n_out, device=dev, generator=gl) * 0.02).to(torch.bfloat16)
            ms = timed(lambda: torch.matmul(xa, wb), few)
            tf = 2 * T * K * H * n_out / (ms * 1e-3) / 1e12
            extras[label] = dict(ms=round(ms, 4), tflops=round(tf, 2), frac_of_peak=round(tf / PEAK_BF16_TFLOPS, 4))
            del wb
        del xa

    line = dict(metric=METRIC, value=round(value, 2), unit="TFLOP/s", n_gpus=1, steps=args.steps,
                warmup=args.warmup, spinup_ms=args.spinup_ms, ms_per_step=round(ms_per_step, 4), higher_is_better=True, scaling="weak",
                vs_baseline=None, dtype="bf16", data="synthetic",
                config=dict(workload="gptoss20b: T=4096 H=I=2880 E=32 top-4 bf16, clamped SwiGLU, capacity=T",
                            tokens=T, hidden=H, intermediate=I, experts=E, top_k=K,
                            algorithmic_flop=flop),
                frac_of_mfma_peak=round(value / PEAK_BF16_TFLOPS, 4), roofline=roofline, cpu_baseline=cpu_baseline,
                parity=parity, decode=decode, configs=configs, extras=extras)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
