// Torch operator layer over the C ABI of libyamoe_hip.so.
//
// Registers `experts` and `experts_backward` with the schemas of drbh/yamoe
// (torch-ext/torch_binding.cpp:58-83) for the GPU dispatch key (which torch-ROCm spells CUDA).
// This file is host-only C++: it checks arguments the way experts_cuda does
// (csrc/moe.cpp:58-96), allocates the output and one workspace tensor from torch's caching
// allocator, and hands raw pointers plus the current HIP stream to the library.  No host
// synchronisation, no `.item()`, so the ops can be captured in a HIP graph.
#include <ATen/ATen.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/library.h>

#include <vector>

#include "yamoe_hip.h"

namespace {

int dtype_code(const at::Tensor &t, const char *name) {
  switch (t.scalar_type()) {
    case at::kFloat: return YAMOE_F32;
    case at::kHalf: return YAMOE_F16;
    case at::kBFloat16: return YAMOE_BF16;
    default:
      TORCH_CHECK(false, name, " must be float32, float16 or bfloat16, got ", t.scalar_type());
  }
  return -1;
}

// the whole op and the row movers among the helper ops also take float64, like the reference's
// (AT_DISPATCH_FLOATING_TYPES_AND2: csrc/gather.cu:89, csrc/scatter.cu:128, csrc/experts_backward.cu:236)
int mover_dtype_code(const at::Tensor &t, const char *name) {
  if (t.scalar_type() == at::kDouble) return YAMOE_F64;
  return dtype_code(t, name);
}

void check_rc(int rc, const char *what) {
  TORCH_CHECK(rc == 0, what, " failed (", rc, "): ", yamoe_last_error());
}

struct Checked {
  yamoe_problem p;
  at::Tensor hidden, idx, rw, wgu, bgu, wd, bd;
};

Checked check_inputs(const at::Tensor &hidden_states, const at::Tensor &router_indices,
                     const at::Tensor &routing_weights, const at::Tensor &gate_up_proj,
                     const at::Tensor &gate_up_proj_bias, const at::Tensor &down_proj,
                     const at::Tensor &down_proj_bias, int64_t expert_capacity, int64_t num_experts, int64_t top_k) {
  TORCH_CHECK(hidden_states.is_cuda(), "hidden_states must be on the GPU");
  TORCH_CHECK(router_indices.is_cuda(), "router_indices must be on the GPU");
  TORCH_CHECK(routing_weights.is_cuda(), "routing_weights must be on the GPU");
  TORCH_CHECK(gate_up_proj.is_cuda(), "gate_up_proj must be on the GPU");
  TORCH_CHECK(gate_up_proj_bias.is_cuda(), "gate_up_proj_bias must be on the GPU");
  TORCH_CHECK(down_proj.is_cuda(), "down_proj must be on the GPU");
  TORCH_CHECK(down_proj_bias.is_cuda(), "down_proj_bias must be on the GPU");

  TORCH_CHECK(hidden_states.dim() == 2, "hidden_states must be 2D [T, H]");
  TORCH_CHECK(router_indices.dim() == 2, "router_indices must be 2D [T, K]");
  TORCH_CHECK(routing_weights.dim() == 2, "routing_weights must be 2D [T, E] or [T, K]");
  TORCH_CHECK(gate_up_proj.dim() == 3, "gate_up_proj must be 3D [E, H, 2*I]");
  TORCH_CHECK(gate_up_proj_bias.dim() == 2, "gate_up_proj_bias must be 2D [E, 2*I]");
  TORCH_CHECK(down_proj.dim() == 3, "down_proj must be 3D [E, I, H]");
  TORCH_CHECK(down_proj_bias.dim() == 2, "down_proj_bias must be 2D [E, H]");

  const int64_t T = hidden_states.size(0), H = hidden_states.size(1), E = num_experts, K = top_k;
  TORCH_CHECK(E > 0 && K > 0, "num_experts and top_k must be positive");
  TORCH_CHECK(router_indices.size(0) == T && router_indices.size(1) == K, "router_indices must be [T, K]");
  TORCH_CHECK(routing_weights.size(0) == T && (routing_weights.size(1) == K || routing_weights.size(1) == E),
              "routing_weights must be [T, K] or [T, E]");
  TORCH_CHECK(gate_up_proj.size(0) == E && gate_up_proj.size(1) == H && gate_up_proj.size(2) % 2 == 0,
              "gate_up_proj must be [E, H, 2*I]");
  const int64_t I = gate_up_proj.size(2) / 2;
  TORCH_CHECK(gate_up_proj_bias.size(0) == E && gate_up_proj_bias.size(1) == 2 * I,
              "gate_up_proj_bias must be [E, 2*I]");
  TORCH_CHECK(down_proj.size(0) == E && down_proj.size(1) == I && down_proj.size(2) == H,
              "down_proj must be [E, I, H]");
  TORCH_CHECK(down_proj_bias.size(0) == E && down_proj_bias.size(1) == H, "down_proj_bias must be [E, H]");
  TORCH_CHECK(router_indices.scalar_type() == at::kLong || router_indices.scalar_type() == at::kInt,
              "router_indices must be int64 or int32");
  const auto dt = hidden_states.scalar_type();
  TORCH_CHECK(routing_weights.scalar_type() == dt && gate_up_proj.scalar_type() == dt &&
                  gate_up_proj_bias.scalar_type() == dt && down_proj.scalar_type() == dt &&
                  down_proj_bias.scalar_type() == dt,
              "all floating tensors must share hidden_states' dtype");
  const auto dev = hidden_states.device();
  TORCH_CHECK(router_indices.device() == dev && routing_weights.device() == dev && gate_up_proj.device() == dev &&
                  gate_up_proj_bias.device() == dev && down_proj.device() == dev && down_proj_bias.device() == dev,
              "all tensors must be on the same device");
  TORCH_CHECK(T * K <= (int64_t)1 << 30, "T*K too large");

  Checked c;
  c.hidden = hidden_states.contiguous();
  c.idx = router_indices.contiguous();
  c.rw = routing_weights.contiguous();
  c.wgu = gate_up_proj.contiguous();
  c.bgu = gate_up_proj_bias.contiguous();
  c.wd = down_proj.contiguous();
  c.bd = down_proj_bias.contiguous();
  c.p.T = (int32_t)T;
  c.p.K = (int32_t)K;
  c.p.E = (int32_t)E;
  c.p.H = (int32_t)H;
  c.p.I = (int32_t)I;
  c.p.capacity = (int32_t)std::min<int64_t>(std::max<int64_t>(expert_capacity, 0), INT32_MAX);
  c.p.dtype = mover_dtype_code(hidden_states, "hidden_states");
  c.p.idx_i64 = router_indices.scalar_type() == at::kLong ? 1 : 0;
  c.p.rw_cols = (int32_t)routing_weights.size(1);
  return c;
}

at::Tensor experts(at::Tensor hidden_states, at::Tensor router_indices, at::Tensor routing_weights,
                   at::Tensor gate_up_proj, at::Tensor gate_up_proj_bias, at::Tensor down_proj,
                   at::Tensor down_proj_bias, int64_t expert_capacity, int64_t num_experts, int64_t top_k) {
  Checked c = check_inputs(hidden_states, router_indices, routing_weights, gate_up_proj, gate_up_proj_bias, down_proj,
                           down_proj_bias, expert_capacity, num_experts, top_k);
  const c10::hip::HIPGuardMasqueradingAsCUDA guard(c.hidden.device());
  at::Tensor out = at::empty_like(c.hidden);
  if (c.p.T == 0) return out;
  size_t ws_bytes = yamoe_experts_workspace_bytes(&c.p);
  TORCH_CHECK(ws_bytes > 0, "experts: ", yamoe_last_error());
  at::Tensor ws = at::empty({(int64_t)ws_bytes}, c.hidden.options().dtype(at::kByte));
  void *stream = (void *)c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
  check_rc(yamoe_experts_forward(&c.p, c.hidden.data_ptr(), c.idx.data_ptr(), c.rw.data_ptr(), c.wgu.data_ptr(),
                                 c.bgu.data_ptr(), c.wd.data_ptr(), c.bd.data_ptr(), out.data_ptr(), ws.data_ptr(),
                                 ws_bytes, stream),
           "yamoe_experts_forward");
  return out;
}

std::vector<at::Tensor> experts_backward(const at::Tensor &grad_out, const at::Tensor &hidden_states,
                                         const at::Tensor &router_indices, const at::Tensor &routing_weights,
                                         const at::Tensor &gate_up_proj, const at::Tensor &gate_up_proj_bias,
                                         const at::Tensor &down_proj, const at::Tensor &down_proj_bias,
                                         int64_t expert_capacity, int64_t num_experts, int64_t top_k) {
  TORCH_CHECK(grad_out.is_cuda(), "grad_out must be on the GPU");
  Checked c = check_inputs(hidden_states, router_indices, routing_weights, gate_up_proj, gate_up_proj_bias, down_proj,
                           down_proj_bias, expert_capacity, num_experts, top_k);
  const int64_t T = c.p.T, H = c.p.H, K = c.p.K;
  TORCH_CHECK(grad_out.scalar_type() == c.hidden.scalar_type(), "grad_out must share hidden_states' dtype");
  TORCH_CHECK(grad_out.numel() == T * H || grad_out.numel() == T * K * H, "grad_out numel must be T*H or T*K*H");
  const c10::hip::HIPGuardMasqueradingAsCUDA guard(c.hidden.device());
  // a [T,K,H] gradient is first summed over the slot axis (csrc/experts_backward.cu:224-228)
  at::Tensor gy = grad_out.numel() == T * H ? grad_out.contiguous().view({T, H})
                                            : grad_out.contiguous().view({T, K, H}).sum(1).contiguous();
  at::Tensor d_hidden = at::empty_like(c.hidden);
  at::Tensor d_routing = at::empty_like(c.rw);
  at::Tensor d_wgu = at::empty_like(c.wgu);
  at::Tensor d_bgu = at::empty_like(c.bgu);
  at::Tensor d_wd = at::empty_like(c.wd);
  at::Tensor d_bd = at::empty_like(c.bd);
  size_t ws_bytes = yamoe_experts_backward_workspace_bytes(&c.p);
  TORCH_CHECK(ws_bytes > 0, "experts_backward: ", yamoe_last_error());
  at::Tensor ws = at::empty({(int64_t)ws_bytes}, c.hidden.options().dtype(at::kByte));
  void *stream = (void *)c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
  check_rc(yamoe_experts_backward(&c.p, gy.data_ptr(), c.hidden.data_ptr(), c.idx.data_ptr(), c.rw.data_ptr(),
                                  c.wgu.data_ptr(), c.bgu.data_ptr(), c.wd.data_ptr(), c.bd.data_ptr(),
                                  d_hidden.data_ptr(), d_routing.data_ptr(), d_wgu.data_ptr(), d_bgu.data_ptr(),
                                  d_wd.data_ptr(), d_bd.data_ptr(), ws.data_ptr(), ws_bytes, stream),
           "yamoe_experts_backward");
  return {d_hidden, d_routing, d_wgu, d_bgu, d_wd, d_bd};
}

// The training pair (no counterpart in the reference, which recomputes): `experts_keep` also returns the activations
// and pre-activations as one byte tensor, `experts_backward_kept` takes it back in place of the recomputation.
std::tuple<at::Tensor, at::Tensor> experts_keep(at::Tensor hidden_states, at::Tensor router_indices,
                                                at::Tensor routing_weights, at::Tensor gate_up_proj,
                                                at::Tensor gate_up_proj_bias, at::Tensor down_proj,
                                                at::Tensor down_proj_bias, int64_t expert_capacity, int64_t num_experts,
                                                int64_t top_k) {
  Checked c = check_inputs(hidden_states, router_indices, routing_weights, gate_up_proj, gate_up_proj_bias, down_proj,
                           down_proj_bias, expert_capacity, num_experts, top_k);
  const c10::hip::HIPGuardMasqueradingAsCUDA guard(c.hidden.device());
  at::Tensor out = at::empty_like(c.hidden);
  const size_t kept_bytes = yamoe_experts_kept_bytes(&c.p);
  at::Tensor kept = at::empty({(int64_t)kept_bytes}, c.hidden.options().dtype(at::kByte));
  if (c.p.T == 0) return std::make_tuple(out, kept);
  size_t ws_bytes = yamoe_experts_workspace_bytes(&c.p);
  TORCH_CHECK(ws_bytes > 0, "experts_keep: ", yamoe_last_error());
  at::Tensor ws = at::empty({(int64_t)ws_bytes}, c.hidden.options().dtype(at::kByte));
  void *stream = (void *)c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
  check_rc(yamoe_experts_forward_keep(&c.p, c.hidden.data_ptr(), c.idx.data_ptr(), c.rw.data_ptr(), c.wgu.data_ptr(),
                                      c.bgu.data_ptr(), c.wd.data_ptr(), c.bd.data_ptr(), out.data_ptr(), kept.data_ptr(),
                                      kept_bytes, ws.data_ptr(), ws_bytes, stream),
           "yamoe_experts_forward_keep");
  return std::make_tuple(out, kept);
}

std::vector<at::Tensor> experts_backward_kept(const at::Tensor &grad_out, const at::Tensor &hidden_states,
                                              const at::Tensor &router_indices, const at::Tensor &routing_weights,
                                              const at::Tensor &gate_up_proj, const at::Tensor &gate_up_proj_bias,
                                              const at::Tensor &down_proj, const at::Tensor &down_proj_bias,
                                              const at::Tensor &kept, int64_t expert_capacity, int64_t num_experts,
                                              int64_t top_k) {
  TORCH_CHECK(grad_out.is_cuda(), "grad_out must be on the GPU");
  Checked c = check_inputs(hidden_states, router_indices, routing_weights, gate_up_proj, gate_up_proj_bias, down_proj,
                           down_proj_bias, expert_capacity, num_experts, top_k);
  const int64_t T = c.p.T, H = c.p.H;
  TORCH_CHECK(grad_out.scalar_type() == c.hidden.scalar_type(), "grad_out must share hidden_states' dtype");
  TORCH_CHECK(grad_out.numel() == T * H, "grad_out must be [T, H]");
  TORCH_CHECK(kept.is_cuda() && kept.scalar_type() == at::kByte && kept.is_contiguous() &&
                  (size_t)kept.numel() >= yamoe_experts_kept_bytes(&c.p),
              "kept must be the byte tensor that experts_keep returned for the same problem");
  const c10::hip::HIPGuardMasqueradingAsCUDA guard(c.hidden.device());
  at::Tensor gy = grad_out.contiguous().view({T, H});
  at::Tensor d_hidden = at::empty_like(c.hidden);
  at::Tensor d_routing = at::empty_like(c.rw);
  at::Tensor d_wgu = at::empty_like(c.wgu);
  at::Tensor d_bgu = at::empty_like(c.bgu);
  at::Tensor d_wd = at::empty_like(c.wd);
  at::Tensor d_bd = at::empty_like(c.bd);
  size_t ws_bytes = yamoe_experts_backward_workspace_bytes(&c.p);
  TORCH_CHECK(ws_bytes > 0, "experts_backward_kept: ", yamoe_last_error());
  at::Tensor ws = at::empty({(int64_t)ws_bytes}, c.hidden.options().dtype(at::kByte));
  void *stream = (void *)c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
  check_rc(yamoe_experts_backward_kept(&c.p, gy.data_ptr(), c.hidden.data_ptr(), c.idx.data_ptr(), c.rw.data_ptr(),
                                       c.wgu.data_ptr(), c.bgu.data_ptr(), c.wd.data_ptr(), c.bd.data_ptr(),
                                       kept.data_ptr(), (size_t)kept.numel(), d_hidden.data_ptr(), d_routing.data_ptr(),
                                       d_wgu.data_ptr(), d_bgu.data_ptr(), d_wd.data_ptr(), d_bd.data_ptr(), ws.data_ptr(),
                                       ws_bytes, stream),
           "yamoe_experts_backward_kept");
  return {d_hidden, d_routing, d_wgu, d_bgu, d_wd, d_bd};
}

// ---- helper ops on the reference's layouts (torch-ext/torch_binding.cpp:9-56) -----------------------------
void *current_stream() { return (void *)c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream(); }

void check_i32(const at::Tensor &t, const char *name) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == at::kInt && t.is_contiguous(), name, " must be a contiguous int32 GPU tensor");
}

void gather_op(const at::Tensor &x, const at::Tensor &indices, const at::Tensor &bins, at::Tensor &output, int64_t E,
               int64_t C, int64_t top_k) {
  TORCH_CHECK(x.is_cuda() && x.dim() == 2 && x.is_contiguous(), "x must be a contiguous [T, H] GPU tensor");
  check_i32(indices, "indices");
  check_i32(bins, "bins");
  const int64_t T = x.size(0), H = x.size(1);
  TORCH_CHECK(output.is_cuda() && output.is_contiguous() && output.dim() == 3 && output.size(0) == E &&
                  output.size(1) == C && output.size(2) == H && output.scalar_type() == x.scalar_type(),
              "Output tensor must have shape [E, C, H]");
  TORCH_CHECK(bins.numel() >= E, "bins must have at least E entries");
  const c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
  check_rc(yamoe_padded_gather(x.data_ptr(), indices.data_ptr<int>(), bins.data_ptr<int>(), output.data_ptr(), (int)T,
                               (int)H, (int)E, (int)C, (int)top_k, mover_dtype_code(x, "x"), current_stream()),
           "yamoe_padded_gather");
}

void scatter_op(const at::Tensor &src, const at::Tensor &indices, const at::Tensor &bins, const at::Tensor &weights,
                at::Tensor &y, int64_t T, int64_t E, int64_t C, int64_t top_k) {
  TORCH_CHECK(src.is_cuda() && src.dim() == 3 && src.is_contiguous() && src.size(0) == E && src.size(1) == C,
              "src must be a contiguous [E, C, H] GPU tensor");
  check_i32(indices, "indices");
  check_i32(bins, "bins");
  const int64_t H = src.size(2);
  TORCH_CHECK(y.is_cuda() && y.is_contiguous() && y.dim() == 2 && y.size(0) == T && y.size(1) == H &&
                  y.scalar_type() == src.scalar_type(), "y must be a contiguous [T, H] tensor of src's dtype");
  TORCH_CHECK(indices.numel() == T * top_k, "indices must have T*top_k entries");
  const void *w = nullptr;
  if (weights.defined() && weights.numel() > 0) {
    TORCH_CHECK(weights.is_cuda() && weights.is_contiguous() && weights.scalar_type() == src.scalar_type() &&
                    weights.numel() == T * top_k, "weights must be [T*top_k] of src's dtype");
    w = weights.data_ptr();
  }
  const c10::hip::HIPGuardMasqueradingAsCUDA guard(src.device());
  size_t ws_bytes = yamoe_padded_scatter_workspace_bytes((int)(T * top_k));
  at::Tensor ws = at::empty({(int64_t)ws_bytes}, src.options().dtype(at::kByte));
  check_rc(yamoe_padded_scatter(src.data_ptr(), indices.data_ptr<int>(), bins.data_ptr<int>(), w, y.data_ptr(), (int)T,
                                (int)H, (int)E, (int)C, (int)top_k, mover_dtype_code(src, "src"), ws.data_ptr(), ws_bytes,
                                current_stream()),
           "yamoe_padded_scatter");
}

void sort_op(at::Tensor x, int64_t end_bit, at::Tensor x_out, at::Tensor iota_out) {
  TORCH_CHECK(x.is_cuda() && x.dim() == 1, "x must be a 1-D GPU tensor");
  TORCH_CHECK(x.scalar_type() == at::kShort || x.scalar_type() == at::kInt || x.scalar_type() == at::kLong,
              "x must be int16, int32 or int64");
  TORCH_CHECK(x_out.is_cuda() && x_out.dim() == 1 && x_out.scalar_type() == x.scalar_type() && x_out.numel() == x.numel());
  TORCH_CHECK(iota_out.is_cuda() && iota_out.dim() == 1 && iota_out.scalar_type() == x.scalar_type() &&
              iota_out.numel() == x.numel());
  TORCH_CHECK(x_out.is_contiguous() && iota_out.is_contiguous(), "outputs must be contiguous");
  if (x_out.numel() == 0) return;
  x = x.contiguous();
  const c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
  const int es = (int)x.element_size();
  size_t ws_bytes = yamoe_sort_workspace_bytes((int)x.numel(), es);
  at::Tensor ws = at::empty({(int64_t)ws_bytes}, x.options().dtype(at::kByte));
  check_rc(yamoe_sort(x.data_ptr(), es, (int)x.numel(), (int)end_bit, x_out.data_ptr(), iota_out.data_ptr(), ws.data_ptr(),
                      ws_bytes, current_stream()),
           "yamoe_sort");
}

void bincount_cumsum_op(at::Tensor input, at::Tensor &output, int64_t minlength) {
  TORCH_CHECK(input.is_cuda(), "Input must be a GPU tensor");
  TORCH_CHECK(input.scalar_type() == at::kInt, "Input must be int32");
  TORCH_CHECK(output.is_cuda() && output.scalar_type() == at::kInt && output.is_contiguous(), "Output must be a contiguous int32 GPU tensor");
  TORCH_CHECK(output.numel() >= minlength, "Output tensor must have at least minlength elements");
  input = input.contiguous();
  const c10::hip::HIPGuardMasqueradingAsCUDA guard(input.device());
  check_rc(yamoe_bincount_cumsum(input.data_ptr<int>(), (int)input.numel(), output.data_ptr<int>(), (int)output.numel(),
                                 (int)minlength, current_stream()),
           "yamoe_bincount_cumsum");
}

at::Tensor index_select_out_op(at::Tensor out, at::Tensor in, at::Tensor idx_int32) {
  TORCH_CHECK(in.is_cuda() && idx_int32.is_cuda() && out.is_cuda(), "GPU tensors only");
  TORCH_CHECK(idx_int32.scalar_type() == at::kInt, "idx must be int32");
  TORCH_CHECK(in.is_contiguous() && idx_int32.is_contiguous() && out.is_contiguous(), "contiguous required");
  TORCH_CHECK(out.scalar_type() == in.scalar_type() && out.numel() >= idx_int32.numel(), "out must match input's dtype and idx's length");
  const c10::hip::HIPGuardMasqueradingAsCUDA guard(in.device());
  check_rc(yamoe_index_select(in.data_ptr(), idx_int32.data_ptr<int>(), out.data_ptr(), idx_int32.numel(),
                              mover_dtype_code(in, "input"), current_stream()),
           "yamoe_index_select");
  return out;
}

at::Tensor batch_mm_op(at::Tensor x, at::Tensor weights, at::Tensor batch_sizes, at::Tensor output, bool trans_b) {
  (void)trans_b;  // ignored, as in the reference (csrc/batch_mm.cu:7-31)
  TORCH_CHECK(x.is_cuda(), "x must be on the GPU");
  TORCH_CHECK(weights.is_cuda(), "weights must be on the GPU");
  TORCH_CHECK(batch_sizes.is_cuda(), "batch_sizes must be on the GPU");
  TORCH_CHECK(x.dim() == 3, "x must be 3D tensor");
  TORCH_CHECK(weights.dim() == 3, "weights must be 3D tensor");
  TORCH_CHECK(batch_sizes.dim() == 1, "batch_sizes must be 1D tensor");
  TORCH_CHECK(x.size(0) == weights.size(0) && x.size(0) == batch_sizes.size(0));
  TORCH_CHECK(x.size(2) == weights.size(1));
  const int64_t E = x.size(0), C = x.size(1), Kd = x.size(2), Nd = weights.size(2);
  TORCH_CHECK(weights.scalar_type() == x.scalar_type() && output.scalar_type() == x.scalar_type(), "dtypes must match");
  x = x.contiguous();
  weights = weights.contiguous();
  if (output.numel() != E * C * Nd) output.resize_({E, C, Nd});
  TORCH_CHECK(output.is_contiguous(), "output must be contiguous");
  const c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
  size_t ws_bytes = yamoe_batch_mm_workspace_bytes((int)E, (int)C);
  at::Tensor ws = at::empty({(int64_t)std::max<size_t>(ws_bytes, 1)}, x.options().dtype(at::kByte));
  check_rc(yamoe_batch_mm(x.data_ptr(), weights.data_ptr(), output.data_ptr(), (int)E, (int)C, (int)Kd, (int)Nd,
                          dtype_code(x, "x"), ws.data_ptr(), ws_bytes, current_stream()),
           "yamoe_batch_mm");
  return output;
}

// ---- router step (torch-ext/yamoe/layers.py:128-152): not an op of the reference, which runs it as four torch calls ----
std::tuple<at::Tensor, at::Tensor> router_topk_op(const at::Tensor &hidden, const at::Tensor &weight,
                                                  const c10::optional<at::Tensor> &bias, int64_t top_k) {
  TORCH_CHECK(hidden.is_cuda() && weight.is_cuda(), "router_topk: GPU tensors only");
  TORCH_CHECK(hidden.dim() == 2 && weight.dim() == 2 && hidden.size(1) == weight.size(1),
              "router_topk: hidden [T, H] and weight [E, H] expected");
  TORCH_CHECK(weight.scalar_type() == hidden.scalar_type(), "router_topk: weight dtype must match hidden");
  const int64_t T = hidden.size(0), H = hidden.size(1), E = weight.size(0);
  at::Tensor x = hidden.contiguous(), w = weight.contiguous(), b;
  const void *bp = nullptr;
  if (bias.has_value() && bias->defined()) {
    TORCH_CHECK(bias->is_cuda() && bias->numel() == E && bias->scalar_type() == hidden.scalar_type(),
                "router_topk: bias must be [E] of the activation dtype");
    b = bias->contiguous();
    bp = b.data_ptr();
  }
  const c10::hip::HIPGuardMasqueradingAsCUDA guard(hidden.device());
  at::Tensor indices = at::empty({T, top_k}, hidden.options().dtype(at::kLong));
  at::Tensor scores = at::empty({T, E}, hidden.options());
  check_rc(yamoe_router_topk(x.data_ptr(), w.data_ptr(), bp, (int)T, (int)H, (int)E, (int)top_k, dtype_code(hidden, "hidden"),
                             indices.data_ptr<int64_t>(), scores.data_ptr(), nullptr, nullptr, current_stream()),
           "yamoe_router_topk");
  return std::make_tuple(indices, scores);
}

// gradient of router_topk with respect to hidden, weight and bias, from the gradient of the dense scores
std::tuple<at::Tensor, at::Tensor, at::Tensor> router_topk_backward_op(const at::Tensor &d_scores, const at::Tensor &indices,
                                                                       const at::Tensor &scores, const at::Tensor &hidden,
                                                                       const at::Tensor &weight) {
  TORCH_CHECK(d_scores.is_cuda() && indices.is_cuda() && scores.is_cuda() && hidden.is_cuda() && weight.is_cuda(),
              "router_topk_backward: GPU tensors only");
  TORCH_CHECK(hidden.dim() == 2 && weight.dim() == 2 && hidden.size(1) == weight.size(1),
              "router_topk_backward: hidden [T, H] and weight [E, H] expected");
  const int64_t T = hidden.size(0), H = hidden.size(1), E = weight.size(0);
  TORCH_CHECK(indices.dim() == 2 && indices.size(0) == T && indices.scalar_type() == at::kLong,
              "router_topk_backward: indices must be int64 [T, K]");
  TORCH_CHECK(scores.dim() == 2 && scores.size(0) == T && scores.size(1) == E && d_scores.sizes() == scores.sizes(),
              "router_topk_backward: scores and d_scores must be [T, E]");
  TORCH_CHECK(weight.scalar_type() == hidden.scalar_type() && scores.scalar_type() == hidden.scalar_type() &&
              d_scores.scalar_type() == hidden.scalar_type(), "router_topk_backward: one dtype for all float tensors");
  const int code = dtype_code(hidden, "hidden");
  at::Tensor x = hidden.contiguous(), w = weight.contiguous(), g = d_scores.contiguous(), sc = scores.contiguous(),
             ix = indices.contiguous();
  const c10::hip::HIPGuardMasqueradingAsCUDA guard(hidden.device());
  at::Tensor d_hidden = at::empty_like(x), d_weight = at::empty_like(w), d_bias = at::empty({E}, hidden.options());
  const size_t need = yamoe_router_backward_workspace_bytes((int)T, (int)E, code);
  at::Tensor ws = at::empty({(int64_t)(need > 0 ? need : 1)}, hidden.options().dtype(at::kByte));
  check_rc(yamoe_router_backward(g.data_ptr(), ix.data_ptr<int64_t>(), sc.data_ptr(), x.data_ptr(), w.data_ptr(), (int)T, (int)H,
                                 (int)E, (int)indices.size(1), code, d_hidden.data_ptr(), d_weight.data_ptr(),
                                 d_bias.data_ptr(), ws.data_ptr(), need, current_stream()),
           "yamoe_router_backward");
  return std::make_tuple(d_hidden, d_weight, d_bias);
}

}  // namespace

TORCH_LIBRARY(_yamoe_amd_ops, ops) {
  ops.def("router_topk(Tensor hidden, Tensor weight, Tensor? bias, int top_k) -> (Tensor, Tensor)");
  ops.impl("router_topk", c10::DispatchKey::CUDA, &router_topk_op);
  ops.def("router_topk_backward(Tensor d_scores, Tensor indices, Tensor scores, Tensor hidden, Tensor weight) -> "
          "(Tensor, Tensor, Tensor)");
  ops.impl("router_topk_backward", c10::DispatchKey::CUDA, &router_topk_backward_op);
  ops.def("gather(Tensor x, Tensor indices, Tensor bins, Tensor! output, int E, int C, int top_k) -> ()");
  ops.impl("gather", c10::DispatchKey::CUDA, &gather_op);
  ops.def("scatter(Tensor src, Tensor indices, Tensor bins, Tensor weights, Tensor! y, int T, int E, int C, "
          "int top_k) -> ()");
  ops.impl("scatter", c10::DispatchKey::CUDA, &scatter_op);
  ops.def("sort(Tensor x, int end_bit, Tensor! x_out, Tensor! iota_out) -> ()");
  ops.impl("sort", c10::DispatchKey::CUDA, &sort_op);
  ops.def("bincount_cumsum(Tensor input, Tensor! output, int minlength) -> ()");
  ops.impl("bincount_cumsum", c10::DispatchKey::CUDA, &bincount_cumsum_op);
  ops.def("index_select_out(Tensor! out, Tensor input, Tensor idx_int32) -> Tensor");
  ops.impl("index_select_out", c10::DispatchKey::CUDA, &index_select_out_op);
  ops.def("batch_mm(Tensor x, Tensor weights, Tensor batch_sizes, Tensor! output, bool trans_b=False) -> Tensor");
  ops.impl("batch_mm", c10::DispatchKey::CUDA, &batch_mm_op);

  ops.def("experts("
          "Tensor hidden_states, "
          "Tensor router_indices, "
          "Tensor routing_weights, "
          "Tensor gate_up_proj, "
          "Tensor gate_up_proj_bias, "
          "Tensor down_proj, "
          "Tensor down_proj_bias, "
          "int expert_capacity, "
          "int num_experts, "
          "int top_k) -> Tensor");
  ops.impl("experts", c10::DispatchKey::CUDA, &experts);

  ops.def("experts_backward("
          "Tensor grad_out, "
          "Tensor hidden_states, "
          "Tensor router_indices, "
          "Tensor routing_weights, "
          "Tensor gate_up_proj, "
          "Tensor gate_up_proj_bias, "
          "Tensor down_proj, "
          "Tensor down_proj_bias, "
          "int expert_capacity, "
          "int num_experts, "
          "int top_k) -> Tensor[]");
  ops.impl("experts_backward", c10::DispatchKey::CUDA, &experts_backward);

  ops.def("experts_keep(Tensor hidden_states, Tensor router_indices, Tensor routing_weights, Tensor gate_up_proj, "
          "Tensor gate_up_proj_bias, Tensor down_proj, Tensor down_proj_bias, int expert_capacity, int num_experts, "
          "int top_k) -> (Tensor, Tensor)");
  ops.impl("experts_keep", c10::DispatchKey::CUDA, &experts_keep);
  ops.def("experts_backward_kept(Tensor grad_out, Tensor hidden_states, Tensor router_indices, Tensor routing_weights, "
          "Tensor gate_up_proj, Tensor gate_up_proj_bias, Tensor down_proj, Tensor down_proj_bias, Tensor kept, "
          "int expert_capacity, int num_experts, int top_k) -> Tensor[]");
  ops.impl("experts_backward_kept", c10::DispatchKey::CUDA, &experts_backward_kept);
}
