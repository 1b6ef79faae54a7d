"""ctypes binding of the C ABI in include/yamoe_hip.h (libyamoe_hip.so).

This is the stub a maintainer of another host (or a test) uses to reach the kernels without the
torch operator layer: plain pointers, sizes and a stream handle.  torch is used here only to own
device memory and to name the current stream.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libyamoe_hip.so")

ABI_VERSION = 2   # YAMOE_ABI_VERSION of the header this module mirrors
F32, F16, BF16, F64 = 0, 1, 2, 3
_DTYPE = {torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16, torch.float64: F64}

# every symbol include/yamoe_hip.h declares
SYMBOLS = [
    "yamoe_abi_version", "yamoe_last_error", "yamoe_route_workspace_bytes", "yamoe_route", "yamoe_permute",
    "yamoe_combine", "yamoe_schedule_bytes", "yamoe_build_schedule", "yamoe_gate_up", "yamoe_down",
    "yamoe_experts_workspace_bytes", "yamoe_experts_forward", "yamoe_experts_forward_static",
    "yamoe_experts_backward_workspace_bytes",
    "yamoe_experts_backward", "yamoe_sort_workspace_bytes", "yamoe_sort", "yamoe_bincount_cumsum", "yamoe_padded_gather",
    "yamoe_padded_scatter_workspace_bytes", "yamoe_padded_scatter", "yamoe_index_select", "yamoe_regular_groups",
    "yamoe_batch_mm_workspace_bytes", "yamoe_batch_mm", "yamoe_router_topk", "yamoe_probe_mfma_rate",
    "yamoe_router_backward_workspace_bytes", "yamoe_router_backward",
    "yamoe_experts_kept_bytes", "yamoe_experts_forward_keep", "yamoe_experts_backward_kept",
]


class Problem(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int32) for n in ("T", "K", "E", "H", "I", "capacity", "dtype", "idx_i64", "rw_cols")]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError("%s is missing: run `python -m yamoe_amd.build`" % LIB_PATH)
        L = ctypes.CDLL(LIB_PATH)
        vp, i32, sz = ctypes.c_void_p, ctypes.c_int32, ctypes.c_size_t
        L.yamoe_abi_version.restype = ctypes.c_int
        if L.yamoe_abi_version() != ABI_VERSION:
            raise ImportError("%s has ABI version %d, this binding was written for %d: rebuild with `python -m yamoe_amd.build`"
                              % (LIB_PATH, L.yamoe_abi_version(), ABI_VERSION))
        L.yamoe_last_error.restype = ctypes.c_char_p
        L.yamoe_route_workspace_bytes.restype = sz
        L.yamoe_route_workspace_bytes.argtypes = [i32, i32]
        L.yamoe_route.argtypes = [vp, i32, i32, i32, i32, vp, vp, vp, vp, vp, vp, sz, vp]
        L.yamoe_permute.argtypes = [vp, vp, vp, i32, i32, i32, i32, vp]
        L.yamoe_combine.argtypes = [vp, vp, vp, i32, vp, i32, vp, i32, i32, i32, i32, i32, vp]
        L.yamoe_schedule_bytes.restype = sz
        L.yamoe_schedule_bytes.argtypes = [i32, i32]
        L.yamoe_build_schedule.argtypes = [vp, vp, i32, i32, i32, i32, vp, sz, vp]
        L.yamoe_gate_up.argtypes = [vp, vp, vp, vp, vp, vp, vp, i32, i32, i32, i32, i32, i32, vp]
        L.yamoe_down.argtypes = [vp, vp, vp, vp, vp, i32, i32, i32, i32, i32, vp]
        pp = ctypes.POINTER(Problem)
        L.yamoe_experts_workspace_bytes.restype = sz
        L.yamoe_experts_workspace_bytes.argtypes = [pp]
        L.yamoe_experts_forward.argtypes = [pp] + [vp] * 9 + [sz, vp]
        L.yamoe_experts_forward_static.argtypes = [pp] + [vp] * 8 + [vp]
        L.yamoe_experts_backward_workspace_bytes.restype = sz
        L.yamoe_experts_backward_workspace_bytes.argtypes = [pp]
        L.yamoe_experts_backward.argtypes = [pp] + [vp] * 15 + [sz, vp]
        L.yamoe_experts_kept_bytes.restype = sz
        L.yamoe_experts_kept_bytes.argtypes = [pp]
        L.yamoe_experts_forward_keep.argtypes = [pp] + [vp] * 8 + [vp, sz, vp, sz, vp]
        L.yamoe_experts_backward_kept.argtypes = [pp] + [vp] * 8 + [vp, sz] + [vp] * 6 + [vp, sz, vp]
        L.yamoe_router_topk.argtypes = [vp, vp, vp, i32, i32, i32, i32, i32, vp, vp, vp, vp, vp]
        L.yamoe_router_backward_workspace_bytes.restype = sz
        L.yamoe_router_backward_workspace_bytes.argtypes = [i32, i32, i32]
        L.yamoe_router_backward.argtypes = [vp, vp, vp, vp, vp, i32, i32, i32, i32, i32, vp, vp, vp, vp, sz, vp]
        L.yamoe_probe_mfma_rate.argtypes = [i32, i32, i32, vp, ctypes.POINTER(ctypes.c_double), vp]
        _lib = L
    return _lib


def _check(rc, what):
    if rc != 0:
        raise RuntimeError("%s failed (%d): %s" % (what, rc, lib().yamoe_last_error().decode()))


def _p(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _need_gpu(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("yamoe_amd needs GPU tensors; there is no CPU path")


def dtype_code(t):
    try:
        return _DTYPE[t.dtype]
    except KeyError:
        raise RuntimeError("unsupported dtype %s" % t.dtype)


def route(router_indices, num_experts, capacity):
    """Stable sort by expert: returns sorted_expert, sorted_idx, counts, offsets, inv_pos (int32)."""
    _need_gpu(router_indices)
    idx = router_indices.contiguous().view(-1)
    if idx.dtype not in (torch.int32, torch.int64):
        raise RuntimeError("router_indices must be int32 or int64")
    N, dev = idx.numel(), idx.device
    i32 = dict(dtype=torch.int32, device=dev)
    sorted_expert, sorted_idx, inv_pos = (torch.empty(N, **i32) for _ in range(3))
    counts, offsets = torch.empty(num_experts, **i32), torch.empty(num_experts + 1, **i32)
    wsb = lib().yamoe_route_workspace_bytes(N, num_experts)
    ws = torch.empty(max(wsb, 1), dtype=torch.uint8, device=dev)
    _check(lib().yamoe_route(_p(idx), int(idx.dtype == torch.int64), N, num_experts, capacity, _p(sorted_expert),
                             _p(sorted_idx), _p(counts), _p(offsets), _p(inv_pos), _p(ws), wsb, _stream()),
           "yamoe_route")
    return sorted_expert, sorted_idx, counts, offsets, inv_pos


def build_schedule(counts, offsets, N, capacity, stream_max_rows):
    E = counts.numel()
    nbytes = lib().yamoe_schedule_bytes(N, E)
    sched = torch.empty(nbytes // 4, dtype=torch.int32, device=counts.device)
    _check(lib().yamoe_build_schedule(_p(counts), _p(offsets), N, E, capacity, stream_max_rows, _p(sched), nbytes,
                                      _stream()), "yamoe_build_schedule")
    return sched


def permute(x, sorted_idx, top_k):
    _need_gpu(x, sorted_idx)
    x = x.contiguous()
    N, H = sorted_idx.numel(), x.shape[1]
    out = torch.empty(N, H, dtype=x.dtype, device=x.device)
    _check(lib().yamoe_permute(_p(x), _p(sorted_idx), _p(out), N, top_k, H, dtype_code(x), _stream()), "yamoe_permute")
    return out


def combine(y_perm, inv_pos, router_indices, routing_weights, T, K, E):
    _need_gpu(y_perm, inv_pos)
    H = y_perm.shape[1]
    out = torch.empty(T, H, dtype=y_perm.dtype, device=y_perm.device)
    idx = None if router_indices is None else router_indices.contiguous()
    rw = None if routing_weights is None else routing_weights.contiguous()
    rw_cols = K if rw is None else rw.shape[1]
    i64 = 0 if idx is None else int(idx.dtype == torch.int64)
    _check(lib().yamoe_combine(_p(y_perm), _p(inv_pos), _p(idx), i64, _p(rw), rw_cols, _p(out), T, K, E, H,
                               dtype_code(y_perm), _stream()), "yamoe_combine")
    return out


def gate_up(x, sorted_idx, gate_up_proj, gate_up_proj_bias, sched, top_k, want_pre=False):
    _need_gpu(x, gate_up_proj)
    E, H, I2 = gate_up_proj.shape
    N = sorted_idx.numel()
    act = torch.empty(N, I2 // 2, dtype=x.dtype, device=x.device)
    pre = torch.empty(N, I2, dtype=x.dtype, device=x.device) if want_pre else None
    _check(lib().yamoe_gate_up(_p(x), _p(sorted_idx), _p(gate_up_proj), _p(gate_up_proj_bias), _p(act), _p(pre),
                               _p(sched), N, top_k, E, H, I2 // 2, dtype_code(x), _stream()), "yamoe_gate_up")
    return (act, pre) if want_pre else act


def down(act, down_proj, down_proj_bias, sched):
    _need_gpu(act, down_proj)
    E, I, H = down_proj.shape
    N = act.shape[0]
    y = torch.empty(N, H, dtype=act.dtype, device=act.device)
    _check(lib().yamoe_down(_p(act), _p(down_proj), _p(down_proj_bias), _p(y), _p(sched), N, E, H, I, dtype_code(act),
                            _stream()), "yamoe_down")
    return y


def router_topk(hidden, weight, bias, top_k):
    """yamoe_router_topk with every optional output: (router_indices int64 [T,K], router_scores [T,E],
    topk_weights [T,K], logits [T,E])."""
    _need_gpu(hidden, weight)
    T, H = hidden.shape
    E = weight.shape[0]
    idx = torch.empty(T, top_k, dtype=torch.int64, device=hidden.device)
    scores = torch.empty(T, E, dtype=hidden.dtype, device=hidden.device)
    topw = torch.empty(T, top_k, dtype=hidden.dtype, device=hidden.device)
    logits = torch.empty(T, E, dtype=hidden.dtype, device=hidden.device)
    _check(lib().yamoe_router_topk(_p(hidden), _p(weight), _p(bias), T, H, E, top_k, dtype_code(hidden), _p(idx), _p(scores),
                                   _p(topw), _p(logits), _stream()), "yamoe_router_topk")
    return idx, scores, topw, logits


def router_backward(d_scores, router_indices, router_scores, hidden, weight, top_k, want_bias=True):
    """yamoe_router_backward: (d_hidden [T,H], d_weight [E,H], d_bias [E] or None)."""
    _need_gpu(d_scores, router_indices, router_scores, hidden, weight)
    T, H = hidden.shape
    E = weight.shape[0]
    d_hidden = torch.empty_like(hidden)
    d_weight = torch.empty_like(weight)
    d_bias = torch.empty(E, dtype=hidden.dtype, device=hidden.device) if want_bias else None
    need = lib().yamoe_router_backward_workspace_bytes(T, E, dtype_code(hidden))
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device=hidden.device)
    _check(lib().yamoe_router_backward(_p(d_scores.contiguous()), _p(router_indices.contiguous()), _p(router_scores.contiguous()),
                                       _p(hidden.contiguous()), _p(weight.contiguous()), T, H, E, top_k, dtype_code(hidden),
                                       _p(d_hidden), _p(d_weight), _p(d_bias), _p(ws), need, _stream()),
           "yamoe_router_backward")
    return d_hidden, d_weight, d_bias


def problem(hidden, router_indices, routing_weights, gate_up_proj, capacity):
    T, H = hidden.shape
    E, _, I2 = gate_up_proj.shape
    return Problem(T=T, K=router_indices.shape[1], E=E, H=H, I=I2 // 2, capacity=capacity, dtype=dtype_code(hidden),
                   idx_i64=int(router_indices.dtype == torch.int64), rw_cols=routing_weights.shape[1])


def experts_forward(hidden, router_indices, routing_weights, gate_up_proj, gate_up_proj_bias, down_proj,
                    down_proj_bias, capacity, workspace=None, out=None):
    """yamoe_experts_forward through ctypes; `workspace` (uint8 tensor) and `out` may be preallocated."""
    _need_gpu(hidden, router_indices, routing_weights, gate_up_proj, gate_up_proj_bias, down_proj, down_proj_bias)
    p = problem(hidden, router_indices, routing_weights, gate_up_proj, capacity)
    need = lib().yamoe_experts_workspace_bytes(ctypes.byref(p))
    if need == 0:
        raise RuntimeError(lib().yamoe_last_error().decode())
    if workspace is None:
        workspace = torch.empty(need, dtype=torch.uint8, device=hidden.device)
    if out is None:
        out = torch.empty_like(hidden)
    _check(lib().yamoe_experts_forward(ctypes.byref(p), _p(hidden), _p(router_indices), _p(routing_weights),
                                       _p(gate_up_proj), _p(gate_up_proj_bias), _p(down_proj), _p(down_proj_bias),
                                       _p(out), _p(workspace), workspace.numel(), _stream()), "yamoe_experts_forward")
    return out


def experts_backward(grad_out, hidden, router_indices, routing_weights, gate_up_proj, gate_up_proj_bias, down_proj,
                     down_proj_bias, capacity, workspace=None, outs=None):
    """yamoe_experts_backward through ctypes: returns (d_hidden, d_routing, d_gate_up_proj, d_gate_up_proj_bias,
    d_down_proj, d_down_proj_bias); `workspace` (uint8 tensor) and the six outputs may be preallocated."""
    _need_gpu(grad_out, hidden, router_indices, routing_weights, gate_up_proj, gate_up_proj_bias, down_proj, down_proj_bias)
    p = problem(hidden, router_indices, routing_weights, gate_up_proj, capacity)
    need = lib().yamoe_experts_backward_workspace_bytes(ctypes.byref(p))
    if need == 0:
        raise RuntimeError(lib().yamoe_last_error().decode())
    if workspace is None:
        workspace = torch.empty(need, dtype=torch.uint8, device=hidden.device)
    if outs is None:
        outs = tuple(torch.empty_like(t) for t in (hidden, routing_weights, gate_up_proj, gate_up_proj_bias, down_proj,
                                                   down_proj_bias))
    _check(lib().yamoe_experts_backward(ctypes.byref(p), _p(grad_out), _p(hidden), _p(router_indices), _p(routing_weights),
                                        _p(gate_up_proj), _p(gate_up_proj_bias), _p(down_proj), _p(down_proj_bias),
                                        *[_p(t) for t in outs], _p(workspace), workspace.numel(), _stream()),
           "yamoe_experts_backward")
    return outs


STATIC_SCRATCH_BYTES = 32 << 20  # YAMOE_STATIC_SCRATCH_BYTES of include/yamoe_hip.h


def experts_forward_static(hidden, router_indices, routing_weights, gate_up_proj, gate_up_proj_bias, down_proj,
                           down_proj_bias, capacity, out):
    """yamoe_experts_forward_static: the forward on the library's built-in workspace; allocates nothing (`out` is the
    caller's)."""
    _need_gpu(hidden, router_indices, routing_weights, gate_up_proj, gate_up_proj_bias, down_proj, down_proj_bias, out)
    p = problem(hidden, router_indices, routing_weights, gate_up_proj, capacity)
    _check(lib().yamoe_experts_forward_static(ctypes.byref(p), _p(hidden), _p(router_indices), _p(routing_weights),
                                              _p(gate_up_proj), _p(gate_up_proj_bias), _p(down_proj),
                                              _p(down_proj_bias), _p(out), _stream()), "yamoe_experts_forward_static")
    return out
