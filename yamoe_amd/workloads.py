"""Seeded synthetic inputs for the expert layer: the five workload shapes this project is measured
on, plus a small free-form builder for tests.  Everything is generated on the CPU generator (so the
same seed gives the same tensors on any machine) in fp32 and then cast.

  readme     README shape of drbh/yamoe (README.md:67-95): T=4096, H=2880, E=8, top-2, fp32, randn
             weights, zero biases, softmax over all experts then top-2 (weights not renormalised)
  gptoss20b  GPT-OSS-20B layer: T=4096, H=I=2880, E=32, top-4, bf16, N(0,0.02) weights and biases,
             softmax -> top-4 -> renormalise
  decode     64 tokens, E=128, top-4, bf16 (GPT-OSS-120B expert shape)
  zipf       16384 tokens, E=128, top-4, bf16, logits = randn + log Zipf(1.2) popularity
  (the backward workload is gptoss20b plus a randn grad_output)
  mid512 .. mid4096  the 128-expert layer (GPT-OSS-120B expert shape) at 512, 1024, 2048 and 4096 tokens, top-4,
             bf16: 16 to 128 rows per expert on average, between the decode and the prefill regime; every expert
             is a single row tile and the layer is bound by the rate at which 6.4 GB of weights stream in
"""
import math

import torch

CONFIGS = {
    "readme": dict(T=4096, H=2880, I=2880, E=8, K=2, dtype=torch.float32, w_std=1.0, bias_std=0.0, renorm=False,
                   zipf=0.0),
    "gptoss20b": dict(T=4096, H=2880, I=2880, E=32, K=4, dtype=torch.bfloat16, w_std=0.02, bias_std=0.02,
                      renorm=True, zipf=0.0),
    "decode": dict(T=64, H=2880, I=2880, E=128, K=4, dtype=torch.bfloat16, w_std=0.02, bias_std=0.02, renorm=True,
                   zipf=0.0),
    "zipf": dict(T=16384, H=2880, I=2880, E=128, K=4, dtype=torch.bfloat16, w_std=0.02, bias_std=0.02, renorm=True,
                 zipf=1.2),
}
for _t in (512, 1024, 2048, 4096):
    CONFIGS["mid%d" % _t] = dict(T=_t, H=2880, I=2880, E=128, K=4, dtype=torch.bfloat16, w_std=0.02, bias_std=0.02,
                                 renorm=True, zipf=0.0)


def make_routing(T, E, K, gen, renorm=True, zipf=0.0):
    """softmax over randn logits (plus log Zipf popularity), top-K, dense [T,E] scatter."""
    logits = torch.randn(T, E, generator=gen)
    if zipf > 0:
        pop = torch.arange(1, E + 1, dtype=torch.float32) ** (-zipf)
        logits = logits + torch.log(pop / pop.sum())
    probs = torch.softmax(logits, dim=-1)
    w, idx = torch.topk(probs, K, dim=-1)
    if renorm:
        w = w / w.sum(dim=-1, keepdim=True)
    dense = torch.zeros(T, E).scatter_(1, idx, w)
    return idx, dense


def make_inputs(T, H, I, E, K, dtype, seed=0, w_std=0.02, bias_std=0.02, renorm=True, zipf=0.0, device="cpu",
                weights=True):
    """Returns a dict: hidden [T,H], router_indices [T,K] int64, routing_weights [T,E] (dense),
    gate_up_proj [E,H,2I], gate_up_proj_bias [E,2I], down_proj [E,I,H], down_proj_bias [E,H]."""
    gen = torch.Generator().manual_seed(seed)
    idx, dense = make_routing(T, E, K, gen, renorm, zipf)
    out = dict(hidden=torch.randn(T, H, generator=gen).to(dtype).to(device), router_indices=idx.to(device),
               routing_weights=dense.to(dtype).to(device))
    if weights:
        # expert by expert: keeps the fp32 staging buffer small for the 128-expert shapes
        def filled(shape, std):
            t = torch.empty(shape, dtype=dtype, device=device)
            for e in range(shape[0]):
                v = torch.randn(shape[1:], generator=gen) * std if std > 0 else torch.zeros(shape[1:])
                t[e] = v.to(dtype).to(device)
            return t
        out["gate_up_proj"] = filled((E, H, 2 * I), w_std)
        out["gate_up_proj_bias"] = filled((E, 2 * I), bias_std)
        out["down_proj"] = filled((E, I, H), w_std)
        out["down_proj_bias"] = filled((E, H), bias_std)
    return out


def device_weights(E, H, I, dtype, std, seed, device, bias_std=None):
    """The four weight tensors drawn on `device` (N(0, std), biases N(0, bias_std), default std), expert by expert.
    For the 128-expert shapes, where drawing 6.4 GB on the host generator takes minutes; the values depend on the
    device's generator, so a CPU check copies them back instead of regenerating them."""
    g = torch.Generator(device=device).manual_seed(seed)
    bias_std = std if bias_std is None else bias_std

    def draw(shape, s):
        t = torch.empty(shape, dtype=dtype, device=device)
        for e in range(shape[0]):
            t[e] = (torch.randn(shape[1:], generator=g, device=device) * s).to(dtype)
        return t
    return dict(gate_up_proj=draw((E, H, 2 * I), std), gate_up_proj_bias=draw((E, 2 * I), bias_std),
                down_proj=draw((E, I, H), std), down_proj_bias=draw((E, H), bias_std))


def make_config(name, seed=0, device="cpu", weights=True):
    c = dict(CONFIGS[name])
    return make_inputs(seed=seed, device=device, weights=weights, **c), c


FWD_FLOP_PER_ROW = lambda H, I: 6 * H * I  # 2*H*2I + 2*I*H per kept (token, expert) assignment


def algorithmic_bytes_decode(n_active, T, K, E, H, I, elem=2):
    """HBM bytes the decode regime must move: the weights and biases of the active experts once,
    hidden states in and out, indices and routing weights."""
    return n_active * (3 * H * I + 2 * I + H) * elem + 2 * T * H * elem + T * K * 8 + T * E * elem
