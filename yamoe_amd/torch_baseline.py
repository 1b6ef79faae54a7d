"""Plain-torch baselines to compare the operators against, on any device torch runs on.

drbh/yamoe ships such baselines next to its kernels and its scripts measure the op against them
(torch-ext/yamoe/__init__.py:3-4, 29-31: `yamoe.vendored.yamoe_ref`, `yamoe.vendored.gpt_oss_mlp`, `yamoe.reference`;
compare_example.py:35-36, perf_plot.py:23).  The same names exist here (`yamoe_amd.reference`,
`yamoe_amd.vendored.yamoe_ref`, `yamoe_amd.vendored.gpt_oss_mlp`) so that those scripts keep working after the import
line is changed.  Nothing in the package calls this module: the operators have no torch path, and this is not one.

Two families, as there:
  * the GPT-OSS modules (router, experts, MLP) with the Hugging Face parameter layout: interleaved gate / up columns,
    clamped SwiGLU, experts applied either token group by token group (training) or densely (inference);
  * the capacity-binned formulation of the op itself: sort assignments by expert, gather up to `expert_capacity` rows per
    expert into a padded [E, C, H] buffer, two batched products, weighted scatter back.
Everything is written with whole-tensor torch calls (no Python loop over tokens), in the dtype of its inputs.
"""
import torch
from torch import nn

GLU_ALPHA = 1.702
GLU_LIMIT = 7.0


def clamped_swiglu(gate_up, alpha=GLU_ALPHA, limit=GLU_LIMIT):
    """[..., 2I] -> [..., I]: even columns gate (clamped from above), odd columns up (clamped on both sides)."""
    gate = gate_up[..., 0::2].clamp(max=limit)
    up = gate_up[..., 1::2].clamp(min=-limit, max=limit)
    return (up + 1) * gate * torch.sigmoid(alpha * gate)


def _expert_ffn(rows, e, gate_up_proj, gate_up_proj_bias, down_proj, down_proj_bias):
    hidden = clamped_swiglu(rows @ gate_up_proj[e] + gate_up_proj_bias[e])
    return hidden @ down_proj[e] + down_proj_bias[e]


# ---- the capacity-binned formulation -----------------------------------------------------------------------------------
def sort_tokens_by_expert(router_indices, num_experts):
    """Flat (token, slot) assignments in expert order.  Returns (positions of the assignments in that order, their
    expert ids, inclusive running count per expert, count per expert).  The sort is stable, so inside an expert the
    assignments keep their token order: that order decides who is dropped when an expert is over capacity."""
    flat = router_indices.reshape(-1)
    experts, order = torch.sort(flat, stable=True)
    per_expert = torch.bincount(experts.clamp(min=0), minlength=num_experts)[:num_experts]
    return order, experts, torch.cumsum(per_expert, dim=0), per_expert


def _slots(indices, bins, expert_capacity):
    """For every sorted position: its expert, its rank inside the expert, and whether the capacity keeps it."""
    n = indices.numel()
    pos = torch.arange(n, device=indices.device)
    expert = torch.bucketize(pos, bins.to(pos.dtype), right=True)
    start = torch.cat([bins.new_zeros(1), bins[:-1]]).to(pos.dtype)
    inside = expert < bins.numel()
    rank = pos - start[expert.clamp(max=bins.numel() - 1)]
    return expert, rank, inside & (rank < expert_capacity)


def binned_gather(x, indices, bins, expert_capacity, top_k):
    """[T, H] -> [E, C, H]: row (e, r) is the token of the r-th assignment of expert e; rows past an expert's count
    (or past the capacity) stay zero."""
    expert, rank, keep = _slots(indices, bins, expert_capacity)
    out = x.new_zeros(bins.numel(), expert_capacity, x.shape[-1])
    out[expert[keep], rank[keep]] = x[indices[keep] // top_k]
    return out


def binned_scatter(x, indices, weights, bins, expert_capacity, top_k):
    """[E, C, H] -> [T, H]: every kept assignment adds its row, times weights[slot] if weights ([T * top_k], in slot
    order) are given, to its token."""
    expert, rank, keep = _slots(indices, bins, expert_capacity)
    rows = x[expert[keep], rank[keep]]
    if weights is not None:
        rows = rows * weights.reshape(-1)[indices[keep]].unsqueeze(-1).to(rows.dtype)
    out = x.new_zeros(indices.numel() // top_k, x.shape[-1])
    return out.index_add_(0, indices[keep] // top_k, rows)


def binned_experts_ref(hidden_states, router_indices, routing_weights, gate_up_proj, gate_up_proj_bias, down_proj,
                       down_proj_bias, expert_capacity):
    """The `experts` operator in torch: [..., H] hidden states, [T, K] expert ids, routing weights dense [T, E] or per
    slot [T, K]; assignments beyond `expert_capacity` inside an expert contribute nothing.  Returns the shape of
    hidden_states."""
    shape = hidden_states.shape
    x = hidden_states.reshape(-1, shape[-1])
    num_experts, top_k = gate_up_proj.shape[0], router_indices.shape[1]
    order, _, bins, _ = sort_tokens_by_expert(router_indices, num_experts)
    binned = binned_gather(x, order, bins, expert_capacity, top_k)
    hidden = clamped_swiglu(torch.bmm(binned, gate_up_proj) + gate_up_proj_bias.unsqueeze(1))
    binned = torch.bmm(hidden, down_proj) + down_proj_bias.unsqueeze(1)
    if routing_weights.shape[1] == num_experts:
        per_slot = torch.gather(routing_weights, 1, router_indices.long().clamp(0, num_experts - 1))
    else:
        per_slot = routing_weights
    return binned_scatter(binned, order, per_slot, bins, expert_capacity, top_k).reshape(shape)


# ---- the GPT-OSS modules ---------------------------------------------------------------------------------------------
class GptOssExperts(nn.Module):
    """The experts of a GPT-OSS MLP block.  `config` needs hidden_size, intermediate_size, num_local_experts."""

    def __init__(self, config):
        super().__init__()
        self.num_experts = config.num_local_experts
        self.hidden_size = config.hidden_size
        self.intermediate_size = self.expert_dim = config.intermediate_size
        e, h, i = self.num_experts, self.hidden_size, self.expert_dim
        self.gate_up_proj = nn.Parameter(torch.empty(e, h, 2 * i))
        self.gate_up_proj_bias = nn.Parameter(torch.empty(e, 2 * i))
        self.down_proj = nn.Parameter(torch.empty(e, i, h))
        self.down_proj_bias = nn.Parameter(torch.empty(e, h))
        self.alpha, self.limit = GLU_ALPHA, GLU_LIMIT

    def _weights(self):
        return self.gate_up_proj, self.gate_up_proj_bias, self.down_proj, self.down_proj_bias

    def forward(self, hidden_states, router_indices=None, routing_weights=None):
        """routing_weights: dense [T, E].  Training (and CPU): only the experts some token selected run, each on its own
        tokens; otherwise every expert runs on every token and the dense weights, zero off the selection, pick."""
        shape = hidden_states.shape
        x = hidden_states.reshape(-1, self.hidden_size)
        if self.training or x.device.type == "cpu":
            out = torch.zeros_like(x)
            chosen = torch.zeros(x.shape[0], self.num_experts, dtype=torch.bool, device=x.device)
            chosen.scatter_(1, router_indices.long().clamp(0, self.num_experts - 1), True)
            for e in chosen.any(dim=0).nonzero().flatten().tolist():
                tokens = chosen[:, e].nonzero().flatten()
                rows = _expert_ffn(x[tokens], e, *self._weights())
                out.index_add_(0, tokens, rows * routing_weights[tokens, e].unsqueeze(-1).to(rows.dtype))
            return out.reshape(shape)
        every = x.unsqueeze(0).expand(self.num_experts, -1, -1)
        hidden = clamped_swiglu(torch.bmm(every, self.gate_up_proj) + self.gate_up_proj_bias.unsqueeze(1))
        rows = torch.bmm(hidden, self.down_proj) + self.down_proj_bias.unsqueeze(1)
        return (rows * routing_weights.t().unsqueeze(-1).to(rows.dtype)).sum(dim=0).reshape(shape)


class GptOssTopKRouter(nn.Module):
    """Linear router, top-k, softmax over the picks.  `config` needs hidden_size, num_local_experts,
    num_experts_per_tok.  Returns (dense scores [T, E], zero off the picks; expert ids [T, K])."""

    def __init__(self, config):
        super().__init__()
        self.top_k = config.num_experts_per_tok
        self.num_experts = config.num_local_experts
        self.hidden_dim = config.hidden_size
        self.weight = nn.Parameter(torch.empty(self.num_experts, self.hidden_dim))
        self.bias = nn.Parameter(torch.empty(self.num_experts))

    def forward(self, hidden_states):
        logits = nn.functional.linear(hidden_states.reshape(-1, self.hidden_dim), self.weight, self.bias)
        top, router_indices = torch.topk(logits, self.top_k, dim=-1)
        scores = torch.zeros_like(logits).scatter_(1, router_indices, torch.softmax(top, dim=-1, dtype=top.dtype))
        return scores, router_indices


class GptOssMLP(nn.Module):
    """Router and experts; returns (output in the shape of the input, dense router scores)."""

    def __init__(self, config):
        super().__init__()
        self.router = GptOssTopKRouter(config)
        self.experts = GptOssExperts(config)

    def forward(self, hidden_states):
        scores, router_indices = self.router(hidden_states)
        return self.experts(hidden_states, router_indices=router_indices, routing_weights=scores), scores
