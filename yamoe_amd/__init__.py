"""yamoe_amd: the expert-layer path of drbh/yamoe for MI355X (gfx950).

Same surface as the reference package for this path (torch-ext/yamoe/__init__.py:1-12):
`experts`, `experts_backward`, `gather`, `scatter`, `sort`, `bincount_cumsum`, `batch_mm`, `ops`, `Yamoe`.  Everything runs in hand-written HIP kernels behind
the C ABI of libyamoe_hip.so; the first use of any of them fails if the native libraries are not built.
`reference`, `vendored`, `yamoe_ref` and `gpt_oss_mlp` (torch-ext/yamoe/__init__.py:3-4, 29-31) are plain-torch baselines
to compare against (torch_baseline.py); the operators never call them.
"""
_OPS = ("gather", "scatter", "sort", "bincount_cumsum", "index_select_out", "batch_mm", "experts", "experts_backward",
        "router_topk", "router_topk_backward", "experts_keep", "experts_backward_kept")
_LAYERS = ("Yamoe", "experts_autograd")
_TORCH_MODULES = {"reference": ".reference", "vendored": ".vendored", "yamoe_ref": ".vendored.yamoe_ref",
              "gpt_oss_mlp": ".vendored.gpt_oss_mlp"}

__all__ = ["ops", *_LAYERS, *_OPS, *_TORCH_MODULES]


def __getattr__(name):
    # Resolved on first use so that `python -m yamoe_amd.build` can run before the libraries exist;
    # any use of the operators without them raises ImportError (there is no other path).
    if name == "ops" or name in _OPS:
        from ._ops import ops

        value = ops if name == "ops" else getattr(ops, name)
    elif name in _LAYERS:
        from . import layers

        value = getattr(layers, name)
    elif name in _TORCH_MODULES:
        import importlib

        value = importlib.import_module(_TORCH_MODULES[name], __name__)
    else:
        raise AttributeError("module %r has no attribute %r" % (__name__, name))
    globals()[name] = value
    return value
