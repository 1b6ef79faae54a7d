"""yamoe_amd: the expert-layer path of drbh/yamoe for MI355X (gfx950).

Same surface as the reference package for this path (torch-ext/yamoe/__init__.py:1-12):
`experts`, `experts_backward`, `ops`, `Yamoe`.  Everything runs in hand-written HIP kernels behind
the C ABI of libyamoe_hip.so; importing fails if the native libraries are not built.
"""
from ._ops import ops
from .layers import Yamoe, experts_autograd

experts = ops.experts
experts_backward = ops.experts_backward

__all__ = ["ops", "Yamoe", "experts", "experts_backward", "experts_autograd"]
