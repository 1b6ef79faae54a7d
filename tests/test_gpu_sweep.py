"""The sweep's comparison leg on one scaled-down point and on the smallest real point of the reference's grid
(perf_plot.py:29-39, config 2 = seq 512, hidden 1024, 32 experts, top-4, batch 1), with the assertions the reference's
scripts leave to the reader (compare_example.py:195-251 prints the table and asserts nothing)."""
import pytest

pytestmark = pytest.mark.gpu


def check(r, dropped):
    assert r["compared"] and r["finite"] and r["ms"] > 0
    for pair in ("kernel_vs_reference", "kernel_vs_binned", "reference_vs_binned"):
        assert set(r[pair]) == {"mse", "mae", "cosine", "rel_l2", "max_abs"}
    kb = r["kernel_vs_binned"]
    assert kb["rel_l2"] < 1e-2 and kb["cosine"] > 0.9999, kb           # the kernel implements the binned semantics
    rb = r["reference_vs_binned"]
    if dropped:   # capacity = seq_len drops assignments: the no-capacity reference must differ, the kernel must not follow it
        assert rb["rel_l2"] > 1e-2 and r["kernel_vs_reference"]["rel_l2"] > 1e-2
    else:
        assert rb["rel_l2"] < 1e-6 and r["kernel_vs_reference"]["rel_l2"] < 1e-2
    assert r["speedup_vs_cpu_oracle"] > 1 and r["memory_ratio"] > 0 and r["reference_padded_mib"] > 0


def test_compare_small_point(gpu):
    from tests import compare_sweep
    r = compare_sweep.compare_point(2, 64, 128, 8, 2, iters=2, warmup=1, capacity="tokens")
    check(r, dropped=False)
    r = compare_sweep.compare_point(4, 32, 128, 4, 2, iters=2, warmup=1, capacity="seq")
    assert r["kept_assignments"] < 4 * 32 * 2
    check(r, dropped=True)


def test_compare_reference_grid_point(gpu):
    from tests import compare_sweep
    from yamoe_amd import sweep
    r = compare_sweep.compare_point(1, iters=3, warmup=1, **sweep.CONFIGS[2])
    print(r, flush=True)
    check(r, dropped=False)
    assert r["memory_ratio"] > 1   # nothing here is padded to [E, C, *]
    r = compare_sweep.compare_point(64, iters=1, warmup=1, max_gflop=1.0, **sweep.CONFIGS[2])
    assert not r["compared"] and "kernel_vs_binned" not in r


def test_sweep_point_against_the_torch_module(gpu):
    """`--torch`: the plain-torch experts module on the same GPU and inputs, both forms timed, results close."""
    from yamoe_amd import sweep
    r = sweep.run_point(2, 64, 128, 8, 2, iters=4, warmup=1, torch_too=True)
    assert r["finite"] and r["torch_per_expert_ms"] > 0 and r["torch_dense_ms"] > 0
    assert r["rel_l2_vs_torch"] < 5e-3 and r["speedup_vs_torch_per_expert"] > 0
