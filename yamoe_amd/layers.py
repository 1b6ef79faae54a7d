"""Autograd glue for the `experts` op, mirroring `_ExpertsFn` of drbh/yamoe
(torch-ext/yamoe/layers.py:6-100): same saved tensors, same order and arity of returned gradients.
"""
import time

import torch

from ._ops import ops


class _ExpertsFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, hidden_flat, router_indices, routing_weights, gate_up_proj, gate_up_proj_bias, down_proj,
                down_proj_bias, expert_capacity, num_experts, top_k, enable_router_grads, save_activations=False):
        a = (hidden_flat, router_indices, routing_weights, gate_up_proj, gate_up_proj_bias, down_proj, down_proj_bias)
        if save_activations:
            # keep the activations and pre-activations ([T*K, 3I] values) for the backward instead of letting it run
            # the gate_up product again: a fifth of the backward's time for that much memory
            out, kept = ops.experts_keep(*a, expert_capacity, num_experts, top_k)
        else:
            out, kept = ops.experts(*a, expert_capacity, num_experts, top_k), None
        ctx.expert_capacity = expert_capacity
        ctx.num_experts = num_experts
        ctx.top_k = top_k
        ctx.enable_router_grads = bool(enable_router_grads)
        ctx.save_activations = kept is not None
        ctx.save_for_backward(*a, *([kept] if kept is not None else []))
        return out

    @staticmethod
    def backward(ctx, grad_output):
        saved = ctx.saved_tensors
        if ctx.save_activations:
            grads = ops.experts_backward_kept(grad_output.contiguous(), *saved, ctx.expert_capacity, ctx.num_experts,
                                              ctx.top_k)
        else:
            grads = ops.experts_backward(grad_output.contiguous(), *saved, ctx.expert_capacity, ctx.num_experts, ctx.top_k)
        d_hidden, d_routing, d_wgu, d_bgu, d_wd, d_bd = grads
        if not ctx.enable_router_grads:
            d_routing = None
        return d_hidden, None, d_routing, d_wgu, d_bgu, d_wd, d_bd, None, None, None, None, None


def experts_autograd(hidden_flat, router_indices, routing_weights, gate_up_proj, gate_up_proj_bias, down_proj,
                     down_proj_bias, expert_capacity, num_experts, top_k, enable_router_grads=True,
                     save_activations=False):
    """Differentiable `experts`: gradients flow to hidden states, weights, biases and (optionally)
    the routing weights.  `save_activations` keeps the first product's results of the forward for the backward
    (T*K*3*I values of memory) instead of recomputing them there as the reference does
    (csrc/experts_backward.cu:164-230)."""
    return _ExpertsFn.apply(hidden_flat, router_indices, routing_weights, gate_up_proj, gate_up_proj_bias, down_proj,
                            down_proj_bias, expert_capacity, num_experts, top_k, enable_router_grads, save_activations)


class _RouterFn(torch.autograd.Function):
    """The fused router step with its gradient (yamoe_router_topk / yamoe_router_backward): what autograd gives through
    the reference's linear -> topk -> softmax -> scatter_ (torch-ext/yamoe/layers.py:128-149), on the HIP kernels."""

    @staticmethod
    def forward(ctx, x_flat, weight, bias, top_k):
        router_indices, router_scores = ops.router_topk(x_flat, weight, bias, top_k)
        ctx.save_for_backward(x_flat, weight, router_indices, router_scores)
        ctx.has_bias = bias is not None
        ctx.mark_non_differentiable(router_indices)
        return router_indices, router_scores

    @staticmethod
    def backward(ctx, _d_indices, d_scores):
        x_flat, weight, router_indices, router_scores = ctx.saved_tensors
        d_x, d_w, d_b = ops.router_topk_backward(d_scores.contiguous(), router_indices, router_scores, x_flat, weight)
        return d_x, d_w, (d_b if ctx.has_bias else None), None


def router_kernel_takes(x_flat, weight, top_k, with_grad=False):
    """Shapes and dtypes of the fused router kernel (yamoe_router_topk) and, with_grad, of its gradient."""
    step = 8 if x_flat.dtype == torch.float32 else 16
    ok = (x_flat.is_cuda and x_flat.dtype in (torch.bfloat16, torch.float16, torch.float32) and weight.dtype == x_flat.dtype
          and x_flat.shape[1] % step == 0 and weight.shape[0] <= 256 and top_k <= min(16, weight.shape[0]))
    if with_grad:   # the two small products run on the expert GEMM kernels: 16-byte rows on both sides
        ok = ok and weight.shape[0] % (step // 2) == 0
    return ok


class Yamoe(torch.nn.Module):
    """Drop-in `forward` for a GPT-OSS MLP block (router + experts), the role of `Yamoe.forward` in
    drbh/yamoe (torch-ext/yamoe/layers.py:106-218).  The host module provides `self.router`
    (weight [E,H], bias [E]) and `self.experts` (gate_up_proj, gate_up_proj_bias, down_proj,
    down_proj_bias).  Attributes read if present:

      num_experts, top_k     as in the reference (defaults 32 and 4)
      enable_router_grads    kept as the host set it (the reference resets it on every call, layers.py:110)
      expert_capacity        None (default): no assignment is dropped (capacity = tokens);
                             "reference": the reference's rule ceil(tokens * top_k / num_experts) (layers.py:161),
                             which drops the overflow of every expert loaded above the mean; or an int
      _timing_enabled        stage times in ms into self._timing_stats (router, topk_softmax, experts_kernel,
                             total), each closed by a device synchronisation as in layers.py:118-122, 200-216.
                             The fused router kernel does the first two stages in one launch: its time is
                             reported under "router" and "topk_softmax" is 0.
    """

    can_torch_compile: bool = False

    def forward(self, hidden_states):
        batch, seq, hidden = hidden_states.shape
        num_experts = getattr(self, "num_experts", 32)
        top_k = getattr(self, "top_k", 4)
        timing = getattr(self, "_timing_enabled", False)
        stats = {}
        self._timing_stats = stats   # reset on every call, like the reference's (layers.py:119-122)

        def lap(name, since):
            torch.cuda.synchronize()
            now = time.perf_counter()
            stats[name] = (now - since) * 1000
            return now

        if timing:
            torch.cuda.synchronize()
            t0 = time.perf_counter()
        x_flat = hidden_states.reshape(-1, hidden)
        want_router_grads = torch.is_grad_enabled() and getattr(self, "enable_router_grads", False)
        if router_kernel_takes(x_flat, self.router.weight, top_k, with_grad=want_router_grads):
            # linear + top-k + softmax + dense scatter in one kernel (and, for a router that is being trained, the
            # gradient of the four steps on the HIP kernels as well)
            if want_router_grads:
                router_indices, router_scores = _RouterFn.apply(x_flat, self.router.weight, self.router.bias, top_k)
            else:
                router_indices, router_scores = ops.router_topk(x_flat, self.router.weight, self.router.bias, top_k)
            if timing:
                t1 = lap("router", t0)
                stats["topk_softmax"] = 0.0
        else:
            # the same four steps as torch ops on the GPU, for shapes the kernels do not take (more than 256 experts,
            # hidden sizes or, with gradients, expert counts that are not multiples of 16 bytes)
            logits = torch.nn.functional.linear(x_flat, self.router.weight, self.router.bias)
            if timing:
                t1 = lap("router", t0)
            top_vals, router_indices = torch.topk(logits, top_k, dim=-1)
            top_w = torch.nn.functional.softmax(top_vals, dim=-1, dtype=top_vals.dtype)
            router_scores = torch.zeros_like(logits).scatter_(1, router_indices, top_w)
            if timing:
                t1 = lap("topk_softmax", t1)
        I = self.experts.down_proj.shape[1]
        gate_up = self.experts.gate_up_proj[:, :, : 2 * I].contiguous()
        gate_up_bias = self.experts.gate_up_proj_bias[:, : 2 * I].contiguous()
        tokens = x_flat.shape[0]
        capacity = getattr(self, "expert_capacity", None)
        if capacity is None:
            capacity = tokens
        elif capacity == "reference":
            capacity = (tokens * top_k + num_experts - 1) // num_experts
        capacity = int(capacity)
        if timing:
            t1 = lap("setup", t1)    # weight slices and capacity: outside "experts_kernel", as in layers.py:158-165
            del stats["setup"]
        if want_router_grads:
            out = experts_autograd(x_flat, router_indices, router_scores, gate_up, gate_up_bias,
                                   self.experts.down_proj, self.experts.down_proj_bias, capacity, num_experts, top_k,
                                   True, bool(getattr(self, "save_activations", False)))
        else:
            with torch.no_grad():
                out = ops.experts(x_flat, router_indices, router_scores, gate_up, gate_up_bias,
                                  self.experts.down_proj, self.experts.down_proj_bias, capacity, num_experts, top_k)
        if timing:
            lap("experts_kernel", t1)
            lap("total", t0)
        return out.view(batch, seq, hidden), router_scores
