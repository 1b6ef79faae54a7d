"""CPU oracle for the yamoe expert-layer path.  TEST INFRASTRUCTURE ONLY.

This module restates, on the CPU, what drbh/yamoe computes on the `experts` / `experts_backward`
path.  It exists to check the HIP kernels; nothing in the product (yamoe_amd/) imports it, and only
tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may call it.

Integer work (routing) is numpy; floating-point work is torch on the CPU (the reference's own
language: its oracles are plain torch).  Each function cites the reference lines it follows
(paths relative to the drbh/yamoe tree).

Pinning (what each function is checked against in tests/test_oracle.py, none of which retypes the
formula under test):
  route                 brute-force O(N^2) rank count on small inputs, numpy stable argsort,
                        permutation / monotonicity / stability invariants
  glu                   hand-computed known answers (tests/golden/glu_kat.json, made with Python's
                        math module in tests/golden/make_glu_kat.py), limits G=0, U=-1, saturation;
                        bit-equal to transformers' GptOssExperts._apply_gate on random data
                        (tests/test_oracle_vs_transformers.py)
  experts_loop          agrees with experts_dense (an independent formulation: all experts on all
                        tokens, dense weights) in fp64; special cases that reduce to one matmul
                        (single expert), to a row copy (interleaved-identity weights), to a
                        bias-only closed form (zero weights), and linearity in routing weights;
                        equal to transformers' GptOssExperts.forward in fp64 (an implementation from outside
                        this repository, per-slot [T,K] routing weights)
  experts_capacity      brute-force per-slot Python loops on tiny inputs; equals experts_loop when
                        capacity >= max load
  experts_backward      torch.autograd.gradcheck of experts_capacity in fp64 (finite differences),
                        agreement between autograd and the closed-form experts_backward_closed, and
                        agreement of both with autograd through transformers' GptOssExperts
  sort_pairs            numpy's stable argsort on the masked key (a library routine), order and
                        stability invariants, two's-complement cases worked by hand
  bincount_cumsum       numpy bincount + cumsum (library), last entry = number of in-range items
  padded_gather / padded_scatter / batch_mm / index_select
                        composed as sort -> bincount_cumsum -> gather -> batch_mm -> glu -> batch_mm
                        -> scatter (the pipeline of torch-ext/yamoe/vendored/yamoe_ref.py:31-70) they
                        must reproduce experts_capacity, which is pinned on its own above; padding
                        rows must be zero; gather followed by unweighted scatter multiplies each
                        token row by its number of kept slots
  router                brute-force Python top-k with the same tie rule on small inputs, torch.topk values
                        (a library routine; values agree whatever its tie order), rows of scores sum to 1 and
                        are zero off the selection
The reference ships no golden vectors or known-answer tests for this path (its tests directory is
git-ignored), so no reference-held fixture exists to check against: every function here is pinned by
independent checks, but agreement with the outputs of the reference's own CUDA op is unpinned.  Where
the reference leaves a choice open this oracle fixes it: equal router logits pick the lower expert id
(torch.topk's order among ties is unspecified), a [T,E] routing tensor with E == K is read as dense, and
the routing gradient is placed once at [token, expert] (the reference's kernel permutes it twice).
"""
import numpy as np
import torch

GLU_LIMIT = 7.0   # csrc/moe.cpp:175; reference.py:16
GLU_ALPHA = 1.702  # csrc/moe.cpp:179; reference.py:15


# ------------------------------------------------------------------------------------------------
# routing
# ------------------------------------------------------------------------------------------------
def route(router_indices, num_experts, capacity):
    """Stable sort of flat (token, slot) assignments by expert id.

    Follows sort_tokens_by_expert (torch-ext/yamoe/vendored/yamoe_ref.py:38-43), the radix sort it
    stands for (csrc/sort.cu:17-59: keys = expert ids, values = iota, stable) and
    bincount + cumsum (csrc/bincount_cumsum.cu:7-56).  Ids outside [0, E) sort last and are dropped.

    Returns dict of int32 arrays: sorted_expert [N], sorted_idx [N], counts [E], offsets [E+1]
    (exclusive; offsets[E] = number of valid ids), bins [E] (inclusive cumsum, the reference's
    `bins`), inv_pos [N] (sorted position of each flat slot, -1 if dropped by the capacity rule:
    rank inside its expert >= capacity, binned_gather yamoe_ref.py:10).
    """
    ids = np.asarray(router_indices).reshape(-1).astype(np.int64)
    N, E = ids.shape[0], int(num_experts)
    key = np.where((ids < 0) | (ids >= E), E, ids)
    order = np.argsort(key, kind="stable").astype(np.int32)
    counts_all = np.bincount(key, minlength=E + 1).astype(np.int64)
    counts = counts_all[:E].astype(np.int32)
    offsets = np.zeros(E + 1, dtype=np.int32)
    offsets[1:] = np.cumsum(counts_all[:E])
    bins = np.cumsum(counts).astype(np.int32)
    sorted_expert = ids[order].astype(np.int32)
    inv_pos = np.full(N, -1, dtype=np.int32)
    pos = np.arange(N, dtype=np.int64)
    skey = key[order]
    valid = skey < E
    rank = pos - offsets[np.minimum(skey, E - 1)]
    kept = valid & (rank < capacity)
    inv_pos[order[kept]] = pos[kept].astype(np.int32)
    return dict(sorted_expert=sorted_expert, sorted_idx=order, counts=counts, offsets=offsets, bins=bins,
                inv_pos=inv_pos)


# ------------------------------------------------------------------------------------------------
# activation
# ------------------------------------------------------------------------------------------------
def glu(gate_up):
    """Clamped SwiGLU on interleaved columns: gate = even, up = odd.
    reference.py:49-54 (build/torch28-cxx11-cu129-x86_64-linux/yamoe/reference.py); csrc/moe.cpp:164-180."""
    gate, up = gate_up[..., ::2], gate_up[..., 1::2]
    gate = gate.clamp(min=None, max=GLU_LIMIT)
    up = up.clamp(min=-GLU_LIMIT, max=GLU_LIMIT)
    return (up + 1) * (gate * torch.sigmoid(gate * GLU_ALPHA))


# ------------------------------------------------------------------------------------------------
# forward
# ------------------------------------------------------------------------------------------------
def experts_loop(hidden, router_indices, routing_weights, gate_up_proj, gate_up_proj_bias, down_proj,
                 down_proj_bias, compute_dtype=None):
    """Loop over the experts that were hit; the path the reference takes in training mode and on the
    CPU (reference.py:38-59; torch-ext/yamoe/vendored/gpt_oss_mlp.py:57-92).  routing_weights is the
    dense [T,E] matrix.  No capacity.  Every op runs in `compute_dtype` (default: the input dtype,
    as the reference does) and the result is accumulated in that dtype with index_add_."""
    dt = compute_dtype or hidden.dtype
    x = hidden.reshape(-1, hidden.shape[-1]).to(dt)
    rw = routing_weights.to(dt)
    wgu, bgu, wd, bd = (t.to(dt) for t in (gate_up_proj, gate_up_proj_bias, down_proj, down_proj_bias))
    E = rw.shape[1]
    out = torch.zeros_like(x)
    mask = torch.nn.functional.one_hot(router_indices.long(), num_classes=E).permute(2, 1, 0)  # [E,K,T]
    hit = torch.greater(mask.sum(dim=(-1, -2)), 0).nonzero()
    for e in hit[:, 0].tolist():
        _, token_idx = torch.where(mask[e])
        cur = x[token_idx]
        gu = cur @ wgu[e] + bgu[e]
        y = glu(gu) @ wd[e] + bd[e]
        out.index_add_(0, token_idx, (y * rw[token_idx, e, None]).to(dt))
    return out


def experts_dense(hidden, routing_weights, gate_up_proj, gate_up_proj_bias, down_proj, down_proj_bias,
                  compute_dtype=None):
    """Every expert on every token, weighted by the dense routing matrix and summed over experts:
    the reference's inference path (reference.py:60-72).  Equal to experts_loop whenever the dense
    weights are zero outside the selected experts."""
    dt = compute_dtype or hidden.dtype
    x = hidden.reshape(-1, hidden.shape[-1]).to(dt)
    rw = routing_weights.to(dt)
    E = rw.shape[1]
    xe = x.repeat(E, 1).view(E, -1, x.shape[-1])
    gu = torch.bmm(xe, gate_up_proj.to(dt)) + gate_up_proj_bias.to(dt)[..., None, :]
    y = torch.bmm(glu(gu), down_proj.to(dt)) + down_proj_bias.to(dt)[..., None, :]
    y = y * rw.transpose(0, 1)[..., None]
    return y.sum(dim=0)


def experts_capacity(hidden, router_indices, routing_weights, gate_up_proj, gate_up_proj_bias, down_proj,
                     down_proj_bias, capacity, compute_dtype=None):
    """The op's own semantics (csrc/moe.cpp:138-220 as restated by binned_experts_ref,
    torch-ext/yamoe/vendored/yamoe_ref.py:46-82): assignments are sorted by expert (stable), the first
    `capacity` of each expert are computed, the rest contribute nothing.  routing_weights may be the
    dense [T,E] matrix or per-slot [T,K].  Differentiable with torch.autograd (the routing is
    integer work done outside the graph).  Accumulation over a token's slots is a plain sum in
    `compute_dtype`."""
    dt = compute_dtype or hidden.dtype
    x = hidden.reshape(-1, hidden.shape[-1]).to(dt)
    T, K = router_indices.shape
    E = gate_up_proj.shape[0]
    r = route(router_indices.detach().cpu().numpy(), E, capacity)
    rw = routing_weights.to(dt)
    if rw.shape[1] == E:
        safe = router_indices.long().clamp(0, E - 1)
        w_sel = torch.gather(rw, 1, safe).reshape(-1)
    else:
        w_sel = rw.reshape(-1)
    wgu, bgu, wd, bd = (t.to(dt) for t in (gate_up_proj, gate_up_proj_bias, down_proj, down_proj_bias))
    out = torch.zeros_like(x)
    for e in range(E):
        n = min(int(r["counts"][e]), int(capacity))
        if n <= 0:
            continue
        first = int(r["offsets"][e])
        flat = torch.from_numpy(r["sorted_idx"][first:first + n].astype(np.int64))
        tok = flat // K
        gu = x[tok] @ wgu[e] + bgu[e]
        y = glu(gu) @ wd[e] + bd[e]
        out = out.index_add(0, tok, y * w_sel[flat, None])
    return out


# ------------------------------------------------------------------------------------------------
# backward
# ------------------------------------------------------------------------------------------------
def experts_backward(grad_out, hidden, router_indices, routing_weights, gate_up_proj, gate_up_proj_bias,
                     down_proj, down_proj_bias, capacity, compute_dtype=torch.float32):
    """Gradients of experts_capacity by torch.autograd: (d_hidden, d_routing, d_gate_up_proj,
    d_gate_up_proj_bias, d_down_proj, d_down_proj_bias), the return order of experts_backward_cuda
    (csrc/experts_backward.cu:340) and of _ExpertsFn.backward (torch-ext/yamoe/layers.py:50-100).
    d_routing has the shape of routing_weights and is zero outside the selected experts, which is
    what autograd through the loop path gives (reference.py:57)."""
    leaves = [t.detach().to(compute_dtype).clone().requires_grad_(True)
              for t in (hidden, routing_weights, gate_up_proj, gate_up_proj_bias, down_proj, down_proj_bias)]
    out = experts_capacity(leaves[0], router_indices, leaves[1], leaves[2], leaves[3], leaves[4], leaves[5],
                           capacity, compute_dtype)
    if not out.requires_grad:  # nothing kept (capacity 0 or no tokens): every gradient is zero
        return tuple(torch.zeros_like(l) for l in leaves)
    grads = torch.autograd.grad(out, leaves, grad_out.reshape(out.shape).to(compute_dtype), allow_unused=True)
    return tuple(torch.zeros_like(l) if g is None else g for g, l in zip(grads, leaves))


def experts_backward_closed(grad_out, hidden, router_indices, routing_weights, gate_up_proj, gate_up_proj_bias,
                            down_proj, down_proj_bias, capacity, compute_dtype=torch.float64):
    """Closed-form backward, one expert at a time, following the formulas of
    csrc/experts_backward.cu:231-311 (with the routing gradient placed at [t, expert] once, not
    permuted twice as :261-264 does)."""
    dt = compute_dtype
    x = hidden.reshape(-1, hidden.shape[-1]).to(dt)
    gy = grad_out.reshape(x.shape).to(dt)
    T, K = router_indices.shape
    E = gate_up_proj.shape[0]
    r = route(router_indices.detach().cpu().numpy(), E, capacity)
    rw = routing_weights.to(dt)
    dense = rw.shape[1] == E
    wgu, bgu, wd, bd = (t.to(dt) for t in (gate_up_proj, gate_up_proj_bias, down_proj, down_proj_bias))
    d_x, d_rw = torch.zeros_like(x), torch.zeros_like(rw)
    d_wgu, d_bgu, d_wd, d_bd = (torch.zeros_like(t) for t in (wgu, bgu, wd, bd))
    for e in range(E):
        n = min(int(r["counts"][e]), int(capacity))
        if n <= 0:
            continue
        first = int(r["offsets"][e])
        flat = torch.from_numpy(r["sorted_idx"][first:first + n].astype(np.int64))
        tok, slot = flat // K, flat % K
        w = rw[tok, e] if dense else rw[tok, slot]
        xe = x[tok]
        pre = xe @ wgu[e] + bgu[e]
        G, U = pre[:, ::2], pre[:, 1::2]
        g = G.clamp(max=GLU_LIMIT)
        u = U.clamp(-GLU_LIMIT, GLU_LIMIT)
        s = torch.sigmoid(GLU_ALPHA * g)
        a = g * s
        h = (u + 1) * a
        ye = h @ wd[e] + bd[e]
        g_ye = gy[tok] * w[:, None]
        dots = (gy[tok] * ye).sum(-1)
        if dense:
            d_rw[tok, e] += dots
        else:
            d_rw[tok, slot] += dots
        d_bd[e] = g_ye.sum(0)
        g_h = g_ye @ wd[e].T
        d_wd[e] = h.T @ g_ye
        d_u = g_h * a * ((U >= -GLU_LIMIT) & (U <= GLU_LIMIT))
        d_g = g_h * (u + 1) * (s + g * s * (1 - s) * GLU_ALPHA) * (G <= GLU_LIMIT)
        d_pre = torch.stack([d_g, d_u], dim=-1).reshape(pre.shape)
        d_bgu[e] = d_pre.sum(0)
        d_wgu[e] = xe.T @ d_pre
        d_x.index_add_(0, tok, d_pre @ wgu[e].T)
    return d_x, d_rw, d_wgu, d_bgu, d_wd, d_bd


# ------------------------------------------------------------------------------------------------
# metrics (definitions of compare_example.py:207-214)
# ------------------------------------------------------------------------------------------------
# ------------------------------------------------------------------------------------------------
# helper ops on the padded [E, C, H] layout
# ------------------------------------------------------------------------------------------------
def sort_pairs(x, end_bit):
    """Stable sort of integer keys on their low `end_bit` bits, carrying positions
    (csrc/sort.cu:17-91: cub::DeviceRadixSort::SortPairs with begin_bit 0, an arange payload of the
    keys' dtype).  With end_bit equal to the key width the order is the signed order (the radix sort
    flips the sign bit of signed keys); with fewer bits the sign bit takes no part and the order is
    that of the unsigned low bits.  Returns (sorted keys, positions cast to the key dtype)."""
    x = np.asarray(x)
    width = x.dtype.itemsize * 8
    assert 0 <= end_bit <= width
    u = x.astype(np.int64).view(np.uint64) & np.uint64((1 << width) - 1 if width < 64 else 0xFFFFFFFFFFFFFFFF)
    if end_bit == width:
        key = u ^ np.uint64(1 << (width - 1))
    else:
        key = u & np.uint64((1 << end_bit) - 1)
    perm = np.argsort(key, kind="stable")
    return x[perm], perm.astype(x.dtype)


def bincount_cumsum(values, out_len, minlength):
    """Inclusive running total of the histogram of `values` over [0, minlength); entries out of
    range are ignored and the rest of the output is zero (csrc/bincount_cumsum.cu:7-97)."""
    v = np.asarray(values).astype(np.int64)
    v = v[(v >= 0) & (v < minlength)]
    out = np.zeros(out_len, dtype=np.int32)
    out[:minlength] = np.cumsum(np.bincount(v, minlength=minlength)[:minlength])
    return out


def padded_gather(x, indices, bins, E, C, top_k):
    """out[e, i] = x[indices[start_e + i] // top_k] for i < bins[e] - start_e, else zero
    (csrc/gather.cu:6-61); start_e = bins[e-1], start_0 = 0."""
    T, H = x.shape
    out = torch.zeros(E, C, H, dtype=x.dtype)
    for e in range(E):
        start = 0 if e == 0 else int(bins[e - 1])
        n = int(bins[e]) - start
        for i in range(min(n, C)):
            tok = int(indices[start + i]) // top_k
            if 0 <= tok < T:
                out[e, i] = x[tok]
    return out


def padded_scatter(src, indices, bins, weights, y, T, E, C, top_k, compute_dtype=torch.float64):
    """y[indices[start_e + i] // top_k] += src[e, i] * weights[start_e + i] over the same rows as
    padded_gather (csrc/scatter.cu:66-105); weights are in sorted order, None means 1.  Accumulated
    in `compute_dtype` on top of y's content and returned in that dtype."""
    acc = y.to(compute_dtype).clone()
    for e in range(E):
        start = 0 if e == 0 else int(bins[e - 1])
        n = int(bins[e]) - start
        for i in range(min(n, C)):
            tok = int(indices[start + i]) // top_k
            if 0 <= tok < T:
                w = 1.0 if weights is None else weights[start + i].to(compute_dtype)
                acc[tok] += src[e, i].to(compute_dtype) * w
    return acc


def index_select(values, idx):
    """out[i] = values[idx[i]] on flat tensors (csrc/index_select.cu:7-16)."""
    return values.reshape(-1)[idx.to(torch.int64)]


def batch_mm(x, weights, compute_dtype=torch.float64):
    """Per-expert product [E, C, K] x [E, K, N]; batch_sizes and trans_b are not used by the
    reference (csrc/batch_mm.cu:7-31 is one bmm)."""
    return torch.bmm(x.to(compute_dtype), weights.to(compute_dtype))


# ------------------------------------------------------------------------------------------------
# router step
# ------------------------------------------------------------------------------------------------
def router_from_logits(logits, top_k, compute_dtype=torch.float32, picks=None):
    """top-k -> softmax over the picked logits -> dense scores (torch-ext/yamoe/layers.py:135-152,
    torch-ext/yamoe/vendored/gpt_oss_mlp.py:134-142).  Picks come in descending order of logit; among equal
    logits the lower expert id first (torch.topk leaves that order open).  The softmax is taken in
    `compute_dtype` and rounded once to the logits' dtype.  `picks` (int64 [T,K]) replaces the top-k when the
    caller already knows which experts were chosen (a gradient check on somebody else's routing); the rest is
    differentiable with respect to the logits.  Returns (router_indices int64 [T,K], router_scores [T,E])."""
    lg = logits.to(compute_dtype)
    order = picks if picks is not None else torch.sort(lg.detach(), dim=-1, descending=True, stable=True).indices[:, :top_k]
    top = torch.gather(lg, 1, order)
    w = torch.softmax(top, dim=-1).to(logits.dtype)
    scores = torch.zeros_like(logits).scatter(1, order, w)
    return order, scores


def router(hidden, weight, bias, top_k, compute_dtype=torch.float32, picks=None):
    """logits = hidden . weight^T + bias in `compute_dtype`, rounded to the activation dtype (the output of the
    reference's F.linear, layers.py:130-132), then router_from_logits.  Returns (indices, scores, logits)."""
    logits = hidden.to(compute_dtype) @ weight.to(compute_dtype).t()
    if bias is not None:
        logits = logits + bias.to(compute_dtype)
    logits = logits.to(hidden.dtype)
    idx, scores = router_from_logits(logits, top_k, compute_dtype, picks)
    return idx, scores, logits


def rel_l2(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return float((a - b).norm() / b.norm().clamp_min(1e-30))


def max_abs(a, b):
    return float((a.double().cpu() - b.double().cpu()).abs().max()) if a.numel() else 0.0
