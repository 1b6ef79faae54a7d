"""Loads the in-tree torch operator library and exposes it as `ops`, the counterpart of the
generated `yamoe/_ops.py` of drbh/yamoe (used at torch-ext/yamoe/__init__.py:1, layers.py:3).

There is no fallback: if the native libraries are missing the import fails with the build command.
"""
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_HIP = os.path.join(_HERE, "libyamoe_hip.so")
_LIB_OPS = os.path.join(_HERE, "_yamoe_amd_ops.so")

for _p in (_LIB_HIP, _LIB_OPS):
    if not os.path.exists(_p):
        raise ImportError(
            "%s is missing: build the native libraries with `python -m yamoe_amd.build` "
            "(hipcc --offload-arch=gfx950); there is no CPU or eager fallback" % _p
        )

torch.ops.load_library(_LIB_OPS)
ops = torch.ops._yamoe_amd_ops
for _name in ("experts", "experts_backward", "gather", "scatter", "sort", "bincount_cumsum", "index_select_out", "batch_mm",
              "router_topk", "router_topk_backward", "experts_keep", "experts_backward_kept"):
    if not hasattr(ops, _name):
        raise ImportError("%s is stale (no operator %r): rebuild with `python -m yamoe_amd.build`" % (_LIB_OPS, _name))


def add_op_namespace_prefix(op_name: str) -> str:
    return "_yamoe_amd_ops::" + op_name


# Shapes and dtypes of the outputs for tracing (torch.compile, FakeTensorMode, meta tensors): the kernels themselves run
# on the GPU only, but a graph capture must be able to ask what an operator returns without running it.
def _register_fakes():
    fake = torch.library.register_fake

    @fake("_yamoe_amd_ops::experts")
    def _(hidden_states, router_indices, routing_weights, gate_up_proj, gate_up_proj_bias, down_proj, down_proj_bias,
          expert_capacity, num_experts, top_k):
        return hidden_states.new_empty(hidden_states.shape)

    @fake("_yamoe_amd_ops::experts_backward")
    def _(grad_out, hidden_states, router_indices, routing_weights, gate_up_proj, gate_up_proj_bias, down_proj,
          down_proj_bias, expert_capacity, num_experts, top_k):
        return [t.new_empty(t.shape) for t in (hidden_states, routing_weights, gate_up_proj, gate_up_proj_bias, down_proj,
                                               down_proj_bias)]

    def kept_bytes(hidden_states, router_indices, gate_up_proj):
        # act [N, I] + pre [N, 2I] + 32 rows of I as a pad, each region rounded up to 256 bytes (yamoe_experts_kept_bytes)
        n, i, es = router_indices.shape[0] * router_indices.shape[1], gate_up_proj.shape[2] // 2, hidden_states.element_size()
        up = lambda b: (max(b, 1) + 255) // 256 * 256
        return up(n * i * es) + up(n * 2 * i * es) + up(32 * i * es)

    @fake("_yamoe_amd_ops::experts_keep")
    def _(hidden_states, router_indices, routing_weights, gate_up_proj, gate_up_proj_bias, down_proj, down_proj_bias,
          expert_capacity, num_experts, top_k):
        return (hidden_states.new_empty(hidden_states.shape),
                hidden_states.new_empty((kept_bytes(hidden_states, router_indices, gate_up_proj),), dtype=torch.uint8))

    @fake("_yamoe_amd_ops::experts_backward_kept")
    def _(grad_out, hidden_states, router_indices, routing_weights, gate_up_proj, gate_up_proj_bias, down_proj,
          down_proj_bias, kept, expert_capacity, num_experts, top_k):
        return [t.new_empty(t.shape) for t in (hidden_states, routing_weights, gate_up_proj, gate_up_proj_bias, down_proj,
                                               down_proj_bias)]

    @fake("_yamoe_amd_ops::router_topk")
    def _(hidden, weight, bias, top_k):
        T, E = hidden.shape[0], weight.shape[0]
        return hidden.new_empty((T, top_k), dtype=torch.int64), hidden.new_empty((T, E))

    @fake("_yamoe_amd_ops::router_topk_backward")
    def _(d_scores, indices, scores, hidden, weight):
        return hidden.new_empty(hidden.shape), weight.new_empty(weight.shape), hidden.new_empty((weight.shape[0],))

    for name in ("gather", "scatter", "sort", "bincount_cumsum"):  # these write into their output arguments
        fake("_yamoe_amd_ops::" + name)(lambda *args, **kwargs: None)


_register_fakes()
