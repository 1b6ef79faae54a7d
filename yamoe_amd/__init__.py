"""yamoe_amd: the expert-layer path of drbh/yamoe for MI355X (gfx950).

Same surface as the reference package for this path (torch-ext/yamoe/__init__.py:1-12):
`experts`, `experts_backward`, `gather`, `scatter`, `sort`, `bincount_cumsum`, `batch_mm`, `ops`, `Yamoe`.  Everything runs in hand-written HIP kernels behind
the C ABI of libyamoe_hip.so; the first use of any of them fails if the native libraries are not built.
"""
_OPS = ("gather", "scatter", "sort", "bincount_cumsum", "index_select_out", "batch_mm", "experts", "experts_backward",
        "router_topk", "router_topk_backward")
_LAYERS = ("Yamoe", "experts_autograd")

__all__ = ["ops", *_LAYERS, *_OPS]


def __getattr__(name):
    # Resolved on first use so that `python -m yamoe_amd.build` can run before the libraries exist;
    # any use of the operators without them raises ImportError (there is no other path).
    if name == "ops" or name in _OPS:
        from ._ops import ops

        value = ops if name == "ops" else getattr(ops, name)
    elif name in _LAYERS:
        from . import layers

        value = getattr(layers, name)
    else:
        raise AttributeError("module %r has no attribute %r" % (__name__, name))
    globals()[name] = value
    return value
