"""The oracle against an implementation that is not this repository's: Hugging Face transformers' GptOssExperts
(transformers/models/gpt_oss/modeling_gpt_oss.py), the module the reference's own Python oracle restates
(build/torch28-cxx11-cu129-x86_64-linux/yamoe/reference.py:35-73; its _apply_gate is :49-54).  It has the same weight
layout (gate/up interleaved on the last axis), the same constants (alpha 1.702, limit 7.0) and the same loop over the
experts that were hit; it differs in taking the routing weights per top-k position [T,K] instead of the dense [T,E]
matrix.  CPU only, fp64, tiny shapes; skipped where transformers is not installed."""
import pytest
import torch

from oracle import yamoe_oracle as O
from yamoe_amd.workloads import make_inputs

transformers = pytest.importorskip("transformers")
modeling = pytest.importorskip("transformers.models.gpt_oss.modeling_gpt_oss")


def hf_experts(d, dtype=torch.float64):
    E, H, I2 = d["gate_up_proj"].shape
    cfg = transformers.GptOssConfig(hidden_size=H, intermediate_size=I2 // 2, num_local_experts=E, num_hidden_layers=1,
                                    num_attention_heads=2, num_key_value_heads=1, vocab_size=32)
    m = modeling.GptOssExperts(cfg).to(dtype)
    with torch.no_grad():
        for name in ("gate_up_proj", "gate_up_proj_bias", "down_proj", "down_proj_bias"):
            getattr(m, name).copy_(d[name].to(dtype))
    assert m.alpha == O.GLU_ALPHA and m.limit == O.GLU_LIMIT
    return m


def test_glu_matches_transformers_apply_gate():
    d = make_inputs(4, 8, 8, 2, 1, torch.float64, seed=1)
    m = hf_experts(d)
    g = torch.Generator().manual_seed(7)
    gu = torch.randn(5, 33, 16, generator=g, dtype=torch.float64) * 6.0   # plenty of values beyond the clamps at +-7
    gu[0, 0, :4] = torch.tensor([7.0, -7.0, 7.5, 7.5], dtype=torch.float64)
    assert (gu.abs() > 7).sum() > 100
    assert torch.equal(O.glu(gu), m._apply_gate(gu))
    gu32 = gu.float()
    assert torch.equal(O.glu(gu32), m._apply_gate(gu32))


@pytest.mark.parametrize("T,H,I,E,K,zipf", [(24, 16, 16, 4, 2, 0.0), (40, 24, 8, 8, 3, 1.5), (7, 8, 16, 3, 1, 0.0)])
def test_forward_and_gradients_match_transformers(T, H, I, E, K, zipf):
    d = make_inputs(T, H, I, E, K, torch.float64, seed=T + E, w_std=0.5, bias_std=0.5, zipf=zipf)
    m = hf_experts(d)
    # the module's own forward; with a config-selected implementation the decorator may route elsewhere, so the class's
    # undecorated loop is taken where the decorator keeps it
    forward = getattr(type(m).forward, "__wrapped__", type(m).forward)
    x = d["hidden"].clone().requires_grad_(True)
    w_slots = torch.gather(d["routing_weights"], 1, d["router_indices"]).clone().requires_grad_(True)   # [T,K]
    out_hf = forward(m, x, d["router_indices"], w_slots)
    args = [d[k] for k in ("hidden", "router_indices", "routing_weights", "gate_up_proj", "gate_up_proj_bias", "down_proj",
                           "down_proj_bias")]
    out = O.experts_loop(*args, compute_dtype=torch.float64)
    assert torch.allclose(out, out_hf.detach(), rtol=1e-12, atol=1e-12)
    assert torch.allclose(O.experts_capacity(*args, T, compute_dtype=torch.float64), out_hf.detach(), rtol=1e-12, atol=1e-12)

    gy = torch.randn(T, H, generator=torch.Generator().manual_seed(3), dtype=torch.float64)
    out_hf.backward(gy)
    d_x, d_rw, d_wgu, d_bgu, d_wd, d_bd = O.experts_backward(gy, *args, T, compute_dtype=torch.float64)
    closed = O.experts_backward_closed(gy, *args, T, compute_dtype=torch.float64)
    for got, want, name in ((d_x, x.grad, "hidden"), (d_wgu, m.gate_up_proj.grad, "gate_up_proj"),
                            (d_bgu, m.gate_up_proj_bias.grad, "gate_up_proj_bias"), (d_wd, m.down_proj.grad, "down_proj"),
                            (d_bd, m.down_proj_bias.grad, "down_proj_bias")):
        want = torch.zeros_like(got) if want is None else want
        assert torch.allclose(got, want, rtol=1e-10, atol=1e-12), name
    # routing gradient: dense [T,E] here, per top-k position there; zero off the selection
    assert torch.allclose(torch.gather(d_rw, 1, d["router_indices"]), w_slots.grad, rtol=1e-10, atol=1e-12)
    sel = torch.zeros_like(d_rw, dtype=torch.bool).scatter_(1, d["router_indices"], True)
    assert torch.all(d_rw[~sel] == 0)
    for a, b in zip(closed, (d_x, d_rw, d_wgu, d_bgu, d_wd, d_bd)):
        assert torch.allclose(a, b, rtol=1e-10, atol=1e-12)
