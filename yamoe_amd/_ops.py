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
              "router_topk", "router_topk_backward"):
    if not hasattr(ops, _name):
        raise ImportError("%s is stale (no operator %r): rebuild with `python -m yamoe_amd.build`" % (_LIB_OPS, _name))


def add_op_namespace_prefix(op_name: str) -> str:
    return "_yamoe_amd_ops::" + op_name
