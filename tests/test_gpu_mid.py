"""Between decode and prefill: experts that are a single row tile of the MFMA kernels (more rows than the streaming
limit, at most 256), where the layer is bound by the rate its weights stream in; the same products as
csrc/moe.cpp:161-187 on those experts' rows.  Forward through the torch op against the oracle: row counts on both
sides of the 32-row block and 256-row tile boundaries, and the 128-expert layer at 512 and 4096 tokens at full size."""
import numpy as np
import pytest
import torch

from oracle import yamoe_oracle as O
from tests.util import KEYS, args, oracle_forward, report, to_dev
from yamoe_amd.workloads import CONFIGS, device_weights, make_config, make_inputs

pytestmark = pytest.mark.gpu


def run_op(d, capacity, gpu):
    import yamoe_amd
    g = to_dev(d, gpu)
    E, K = d["gate_up_proj"].shape[0], d["router_indices"].shape[1]
    out = yamoe_amd.experts(*args(g), capacity, E, K)
    torch.cuda.synchronize()
    return out.cpu()


# T, H, I, E, K, capacity (0: tokens), zipf: rows per expert on both sides of the block and tile boundaries
CASES = [
    (300, 128, 128, 8, 2, 0, 0.0),      # ~75 rows per expert: three row blocks; the shortest contraction (4 slabs)
    (130, 192, 320, 4, 1, 0, 0.0),      # ~32 rows: one or two blocks; I = 320: column tiles of 128, 128, 64 (down: 128, 64)
    (1000, 256, 192, 8, 2, 128, 0.0),   # capacity 128: every expert exactly four row blocks
    (1000, 256, 192, 8, 2, 129, 0.0),   # 129: a fifth block with one row
    (1200, 256, 128, 8, 2, 256, 0.0),   # 256 rows: one full row tile
    (1200, 256, 128, 8, 2, 257, 0.0),   # 257: two row tiles
    (2000, 320, 576, 16, 2, 0, 1.2),    # skewed: streamed experts, single row tiles and several row tiles in one call
    (700, 2880, 2880, 8, 2, 0, 0.5),    # the GPT-OSS width (45 + 23 column tiles, the last of 64 columns)
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,H,I,E,K,capacity,zipf", CASES)
def test_forward_mid_regime(gpu, dtype, T, H, I, E, K, capacity, zipf):
    print("mid", dtype, T, H, I, E, K, capacity, zipf, flush=True)
    d = make_inputs(T, H, I, E, K, dtype, seed=T + H + capacity, w_std=0.05, bias_std=0.1, zipf=zipf)
    cap = capacity or T
    kept = np.minimum(np.bincount(d["router_indices"].numpy().ravel(), minlength=E), cap)
    print("  kept rows per expert:", kept.tolist(), flush=True)
    if capacity != 257:
        assert ((kept > 32) & (kept <= 256)).any(), "no expert in the mid range"
    got = run_op(d, cap, gpu)
    want = oracle_forward(d, cap)
    assert report("mid regime", got, want, 1e-2) < 1e-2


@pytest.mark.parametrize("name", ["mid512", "mid4096"])
def test_mid_shapes_128_experts(gpu, name):
    """The 128-expert layer of the GPT-OSS-120B expert shape at 512 and 4096 tokens (16 and 128 rows per expert on
    average), bf16, weights drawn on the device (6.4 GB) and copied back for the oracle."""
    c = CONFIGS[name]
    host, _ = make_config(name, seed=0, weights=False)
    g = {k: v.to(gpu) for k, v in host.items()}
    g.update(device_weights(c["E"], c["H"], c["I"], c["dtype"], c["w_std"], 6, gpu))
    counts = np.bincount(host["router_indices"].numpy().ravel(), minlength=c["E"])
    print("%s: rows per expert %d .. %d" % (name, counts.min(), counts.max()), flush=True)
    import yamoe_amd
    got = yamoe_amd.experts(*[g[k] for k in KEYS], c["T"], c["E"], c["K"])
    torch.cuda.synchronize()
    got = got.cpu()
    d = {k: v.cpu() for k, v in g.items()}
    del g
    torch.cuda.empty_cache()
    want = oracle_forward(d, c["T"])
    assert report(name, got, want, 1e-2) < 1e-2
