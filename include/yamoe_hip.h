/*
 * yamoe_hip.h — C ABI of libyamoe_hip.so: the MI355X (gfx950) expert-layer path.
 *
 * Every entry point takes plain device pointers, sizes and a HIP stream handle
 * (passed as void* so that this header needs no HIP include).  Nothing here
 * allocates, frees or synchronises: callers bring the output buffers and one
 * workspace whose size the matching *_workspace_bytes() call returns.  All work
 * is enqueued on `stream` and the call returns at once.
 *
 * Return value: 0 on success, a negative YAMOE_E_* code on a rejected argument,
 * a positive hipError_t if a launch failed.  yamoe_last_error() gives the text
 * of the last failure on the calling thread.
 *
 * Citations name the file:line of drbh/yamoe that each entry point replaces.
 */
#ifndef YAMOE_HIP_H
#define YAMOE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* 2: YAMOE_F64 dtype code; yamoe_experts_forward_static; yamoe_route_workspace_bytes returns the size of a
 *    segments x buckets table above 4096 assignments (it was a constant 256 bytes); stream_max_rows up to 32;
 *    yamoe_probe_mfma_rate; yamoe_router_topk takes fp32; yamoe_router_backward; the whole op takes YAMOE_F64.
 *    Added since, without a change of existing behaviour: yamoe_experts_kept_bytes / _forward_keep / _backward_kept;
 *    stream_max_rows = -1; H and I of any size; hidden_states of 4 GiB or more. */
#define YAMOE_ABI_VERSION 2

/* element type of activations, weights, biases and routing weights.  YAMOE_F64 is taken by the whole forward and
 * backward (yamoe_experts_forward, _forward_static, _backward: plain FMA kernels, a compatibility dtype) and by the
 * row movers among the helper ops (yamoe_padded_gather, yamoe_padded_scatter, yamoe_index_select), which the
 * reference dispatches over double too (csrc/gather.cu:89, csrc/scatter.cu:128, csrc/experts_backward.cu:236);
 * everything else answers YAMOE_E_DTYPE. */
enum { YAMOE_F32 = 0, YAMOE_F16 = 1, YAMOE_BF16 = 2, YAMOE_F64 = 3 };

enum {
  YAMOE_E_ARG = -1,       /* bad size / null pointer / unsupported shape */
  YAMOE_E_WORKSPACE = -2, /* workspace too small */
  YAMOE_E_DTYPE = -3      /* unknown dtype */
};

/* Shape of one experts() call.  Mirrors the integer arguments and tensor sizes
 * of experts_cuda (csrc/moe.cpp:45-96). */
typedef struct yamoe_problem {
  int32_t T;         /* tokens (rows of hidden_states) */
  int32_t K;         /* top_k: experts per token */
  int32_t E;         /* num_experts */
  int32_t H;         /* hidden size */
  int32_t I;         /* intermediate size; gate_up_proj is [E,H,2I], down_proj is [E,I,H] */
  int32_t capacity;  /* expert_capacity: assignments ranked >= capacity inside their expert are dropped */
  int32_t dtype;     /* YAMOE_F32 / YAMOE_F16 / YAMOE_BF16 / YAMOE_F64 */
  int32_t idx_i64;   /* router_indices element type: 1 = int64, 0 = int32 */
  int32_t rw_cols;   /* columns of routing_weights: E (dense [T,E]) or K (per slot [T,K]) */
} yamoe_problem;

int yamoe_abi_version(void);
const char *yamoe_last_error(void);

/* ---- routing: stable sort of (token,slot) assignments by expert -------------
 * Replaces sort_cuda (csrc/sort.cu:61-91) + bincount_cumsum_cuda
 * (csrc/bincount_cumsum.cu:58-97) as called from csrc/moe.cpp:141-144.
 *   router_indices [N]  int32 or int64 expert id per flat slot t*K+k (N = T*K)
 *   sorted_expert  [N]  expert ids in non-decreasing order
 *   sorted_idx     [N]  flat slot of each sorted position; ties keep slot order (stable)
 *   counts         [E]  assignments per expert
 *   offsets        [E+1] exclusive prefix sum of counts; offsets[E] = number of valid ids
 *   inv_pos        [N]  sorted position of each flat slot, or -1 when the slot is
 *                       dropped (rank inside its expert >= capacity, or id outside [0,E))
 * Ids outside [0,E) sort after every valid expert.  Limit: E <= 768 (this bounds every entry point
 * that routes: the whole forward and backward too). */
size_t yamoe_route_workspace_bytes(int32_t N, int32_t E);
int yamoe_route(const void *router_indices, int32_t idx_i64, int32_t N, int32_t E,
                int32_t capacity, int32_t *sorted_expert, int32_t *sorted_idx,
                int32_t *counts, int32_t *offsets, int32_t *inv_pos, void *workspace,
                size_t workspace_bytes, void *stream);

/* ---- token permute: expert-contiguous row gather -----------------------------
 * Replaces gather_cuda (csrc/gather.cu:68-109) without the padded [E,C,H] layout:
 *   x_perm[p,:] = x[sorted_idx[p] / K, :]   for every sorted position p < N. */
int yamoe_permute(const void *x, const int32_t *sorted_idx, void *x_perm, int32_t N,
                  int32_t K, int32_t H, int32_t dtype, void *stream);

/* ---- routing-weighted combine -------------------------------------------------
 * Replaces at::gather_out + index_select_out_cuda + scatter_cuda
 * (csrc/moe.cpp:190-220, csrc/index_select.cu:18-51, csrc/scatter.cu:110-147):
 *   out[t,:] = sum_k w(t,k) * y_perm[inv_pos[t*K+k],:]   (dropped slots skipped)
 * with w(t,k) = routing_weights[t, router_indices[t,k]] when rw_cols == E and
 * routing_weights[t,k] when rw_cols == K.  Sum in fp32 in slot order, one
 * rounding; no atomics, `out` needs no zero fill.  routing_weights == NULL
 * means weight 1 (the backward of the permute, csrc/experts_backward.cu:92-124). */
int yamoe_combine(const void *y_perm, const int32_t *inv_pos, const void *router_indices,
                  int32_t idx_i64, const void *routing_weights, int32_t rw_cols, void *out,
                  int32_t T, int32_t K, int32_t E, int32_t H, int32_t dtype, void *stream);

/* ---- expert GEMMs --------------------------------------------------------------
 * Replace batch_mm (csrc/batch_mm.cu:7-31) plus the ATen bias / clamped-SwiGLU
 * chain (csrc/moe.cpp:161-187) on ragged expert groups (no padding):
 *   gate_up: act[p, j] = (clamp(U,-7,7)+1) * g*sigmoid(1.702 g), g = min(G,7),
 *            G = x_p . Wgu[e][:,2j] + bgu[e][2j],  U = x_p . Wgu[e][:,2j+1] + bgu[e][2j+1]
 *            with x_p = x[sorted_idx[p]/K] gathered on the fly (x is the un-permuted [T,H]).
 *            If pre_act != NULL the biased pre-activations [N,2I] are stored too.
 *   down:    y_perm[p,:] = act[p,:] . Wd[e] + bd[e]
 * Rows p with rank >= capacity inside their expert are not computed.
 * `schedule` is the workspace region filled by yamoe_build_schedule: experts with
 * 1..stream_max_rows kept rows (at most 32; 16-bit dtypes only, pass 0 for fp32) are
 * listed for the weight-streaming kernel, the others are cut into 256-row MFMA tiles.
 * A limit above 16 applies only when no expert has more kept rows than the limit;
 * otherwise experts with up to 16 rows stream and the others are tiled.
 * stream_max_rows = -1 with N <= 4*E (decode: a few rows per expert) lists every expert for the
 * streaming kernel, one with more than 32 rows as several entries of at most 32, and leaves the
 * tile list empty (the whole-op forward then skips the tile kernels' launches); with more
 * assignments than that -1 means 32.
 * yamoe_gate_up / yamoe_down launch both kernels; each walks its own list. */
size_t yamoe_schedule_bytes(int32_t N, int32_t E);
int yamoe_build_schedule(const int32_t *counts, const int32_t *offsets, int32_t N, int32_t E,
                         int32_t capacity, int32_t stream_max_rows, void *schedule,
                         size_t schedule_bytes, void *stream);
int yamoe_gate_up(const void *x, const int32_t *sorted_idx, const void *gate_up_proj,
                  const void *gate_up_proj_bias, void *act, void *pre_act, const void *schedule,
                  int32_t N, int32_t K, int32_t E, int32_t H, int32_t I, int32_t dtype,
                  void *stream);
int yamoe_down(const void *act, const void *down_proj, const void *down_proj_bias, void *y_perm,
               const void *schedule, int32_t N, int32_t E, int32_t H, int32_t I, int32_t dtype,
               void *stream);

/* ---- the whole forward: experts_cuda (csrc/moe.cpp:45-223) -------------------
 * Limits (YAMOE_E_ARG otherwise): E <= 768; T*K < 2^30.
 * hidden_states (and grad_out) of 4 GiB or more are permuted into expert order first (the kernels gather token
 * rows with 32-bit byte offsets from the start of the tensor): the workspace then holds one more [T*K, H] buffer
 * (two for the backward).  yamoe_gate_up, the stage entry point, keeps the 4 GiB limit for its gathered x.
 * H and I may be any size, as in the reference; the MFMA kernels take those that are whole 16-byte chunks (multiples
 * of 8 for the 16-bit dtypes, of 4 for fp32), and every other size, like every fp64 problem, runs on plain FMA tiles
 * (correct to the same tolerances, far slower). */
size_t yamoe_experts_workspace_bytes(const yamoe_problem *p);
int yamoe_experts_forward(const yamoe_problem *p, const void *hidden_states,
                          const void *router_indices, const void *routing_weights,
                          const void *gate_up_proj, const void *gate_up_proj_bias,
                          const void *down_proj, const void *down_proj_bias, void *out,
                          void *workspace, size_t workspace_bytes, void *stream);

/* ---- the whole forward without a workspace argument -------------------------------------------
 * No counterpart in the reference.  For callers that cannot allocate device memory at all, not even
 * a workspace: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
 * Same arguments, kernels and results as yamoe_experts_forward, but the workspace is an array of
 * YAMOE_STATIC_SCRATCH_BYTES that is part of the library's device image (each GPU the library runs
 * on holds its copy until the process ends).  The call allocates and frees nothing; its first call
 * on a device looks the array's address up (one hipGetSymbolAddress, which may load the device
 * image: make that first call before a stream capture begins, not inside it).  Problems whose
 * yamoe_experts_workspace_bytes() exceeds the array are rejected with YAMOE_E_WORKSPACE (at
 * H = I = 2880 in a 16-bit dtype the limit is about 2900 (token, expert) assignments, e.g. 725
 * tokens at top-4).  All calls on one GPU share that GPU's array: two calls whose work overlaps on
 * the same GPU (different streams, or different threads) race; calls on one stream are ordered. */
#define YAMOE_STATIC_SCRATCH_BYTES (32u << 20)
int yamoe_experts_forward_static(const yamoe_problem *p, const void *hidden_states,
                                 const void *router_indices, const void *routing_weights,
                                 const void *gate_up_proj, const void *gate_up_proj_bias,
                                 const void *down_proj, const void *down_proj_bias, void *out,
                                 void *stream);

/* ---- the whole backward: experts_backward_cuda (csrc/experts_backward.cu:126-341)
 * Outputs (all fully written, caller need not zero them):
 *   d_hidden [T,H], d_routing [T,rw_cols] (zero outside the selected experts),
 *   d_gate_up_proj [E,H,2I], d_gate_up_proj_bias [E,2I], d_down_proj [E,I,H],
 *   d_down_proj_bias [E,H].  grad_out is [T,H]. */
size_t yamoe_experts_backward_workspace_bytes(const yamoe_problem *p);
int yamoe_experts_backward(const yamoe_problem *p, const void *grad_out,
                           const void *hidden_states, const void *router_indices,
                           const void *routing_weights, const void *gate_up_proj,
                           const void *gate_up_proj_bias, const void *down_proj,
                           const void *down_proj_bias, void *d_hidden, void *d_routing,
                           void *d_gate_up_proj, void *d_gate_up_proj_bias, void *d_down_proj,
                           void *d_down_proj_bias, void *workspace, size_t workspace_bytes,
                           void *stream);

/* ---- the training pair: a forward that keeps what the backward would recompute ----
 * No counterpart in the reference, whose backward recomputes the first product from hidden_states
 * (csrc/experts_backward.cu:164-230); for callers that run the backward of the same call and can spare
 * the memory (torch autograd with save_activations, a training loop).  yamoe_experts_forward_keep is
 * yamoe_experts_forward that also leaves the activations [T*K, I] and the pre-activations [T*K, 2I] (sorted-row
 * order, activation dtype) in `kept` (yamoe_experts_kept_bytes(p) bytes); yamoe_experts_backward_kept is
 * yamoe_experts_backward on the same problem and inputs that reads them instead of running the gate_up
 * product again (4*H*I of its 16*H*I flop per assignment).  Same workspaces, same outputs; experts that the
 * forward served from its weight-streaming kernel differ from a recomputation in the last bits of their rows. */
size_t yamoe_experts_kept_bytes(const yamoe_problem *p);
int yamoe_experts_forward_keep(const yamoe_problem *p, const void *hidden_states,
                               const void *router_indices, const void *routing_weights,
                               const void *gate_up_proj, const void *gate_up_proj_bias,
                               const void *down_proj, const void *down_proj_bias, void *out,
                               void *kept, size_t kept_bytes, void *workspace, size_t workspace_bytes,
                               void *stream);
int yamoe_experts_backward_kept(const yamoe_problem *p, const void *grad_out, const void *hidden_states,
                                const void *router_indices, const void *routing_weights,
                                const void *gate_up_proj, const void *gate_up_proj_bias,
                                const void *down_proj, const void *down_proj_bias, const void *kept,
                                size_t kept_bytes, void *d_hidden, void *d_routing, void *d_gate_up_proj,
                                void *d_gate_up_proj_bias, void *d_down_proj, void *d_down_proj_bias,
                                void *workspace, size_t workspace_bytes, void *stream);

/* ---- helper ops on the reference's own layouts (torch-ext/torch_binding.cpp:9-56) ---------
 * These serve code written against the reference's public helper ops; the fused forward and
 * backward above do not use them. */

/* sort_cuda (csrc/sort.cu:61-91): stable radix sort of int16/int32/int64 keys on bits
 * [0, end_bit), payload = iota of the key type.  elem_bytes = 2, 4 or 8. */
size_t yamoe_sort_workspace_bytes(int32_t n, int32_t elem_bytes);
int yamoe_sort(const void *x, int32_t elem_bytes, int32_t n, int32_t end_bit, void *x_out,
               void *iota_out, void *workspace, size_t workspace_bytes, void *stream);

/* bincount_cumsum_cuda (csrc/bincount_cumsum.cu:58-97): output[b] = number of inputs <= b for
 * b < minlength (inclusive prefix sum of the bin counts); output[minlength..output_len) = 0.
 * Limit: minlength <= 8192 bins. */
int yamoe_bincount_cumsum(const int32_t *input, int32_t n, int32_t *output, int32_t output_len,
                          int32_t minlength, void *stream);

/* gather_cuda (csrc/gather.cu:68-109): output[e,i,:] = x[indices[start_e+i] / top_k,:] for
 * i < bins[e]-start_e (start_e = bins[e-1], inclusive bins), zero elsewhere; output is [E,C,H]. */
int yamoe_padded_gather(const void *x, const int32_t *indices, const int32_t *bins, void *output,
                        int32_t T, int32_t H, int32_t E, int32_t C, int32_t top_k, int32_t dtype,
                        void *stream);

/* scatter_cuda (csrc/scatter.cu:110-147): y[tok,:] += src[e,i,:] * weights[start_e+i] for the
 * first C rows of every expert; weights == NULL means 1.  No atomics: fp32 sum per output row in
 * slot order on top of the incoming y. */
size_t yamoe_padded_scatter_workspace_bytes(int32_t S);
int yamoe_padded_scatter(const void *src, const int32_t *indices, const int32_t *bins,
                         const void *weights, void *y, int32_t T, int32_t H, int32_t E, int32_t C,
                         int32_t top_k, int32_t dtype, void *workspace, size_t workspace_bytes,
                         void *stream);

/* index_select_out_cuda (csrc/index_select.cu:18-51): out[i] = input[idx[i]]. */
int yamoe_index_select(const void *input, const int32_t *idx, void *out, int64_t n, int32_t dtype,
                       void *stream);

/* counts[e] = rows, offsets[e] = e*rows (offsets has E+1 entries): the regular [E,rows,*] layout
 * described as ragged groups, used by yamoe_batch_mm. */
int yamoe_regular_groups(int32_t *counts, int32_t *offsets, int32_t E, int32_t rows, void *stream);

/* batch_mm (csrc/batch_mm.cu:7-31): output[e] = x[e] . weights[e] for x [E,C,Kd], weights
 * [E,Kd,Nd], output [E,C,Nd], on the grouped MFMA / streaming kernels.  Like the reference,
 * every one of the C rows is computed (batch_sizes is not consulted). */
size_t yamoe_batch_mm_workspace_bytes(int32_t E, int32_t C);
int yamoe_batch_mm(const void *x, const void *weights, void *output, int32_t E, int32_t C,
                   int32_t Kd, int32_t Nd, int32_t dtype, void *workspace, size_t workspace_bytes,
                   void *stream);

/* The router step of Yamoe.forward (torch-ext/yamoe/layers.py:128-152; GptOssTopKRouter.forward,
 * torch-ext/yamoe/vendored/gpt_oss_mlp.py:128-142) in one kernel:
 *   logits = round(hidden . weight^T + bias)            [T,E]  (optional output)
 *   router_indices = top_k experts by logit, descending; equal logits: lower expert id first   [T,K] int64
 *   router_scores  = softmax over the K picked logits (fp32, rounded once), scattered into a
 *                    zero [T,E] row; topk_weights (optional) holds the same K values as [T,K].
 * H must be a multiple of 16 (fp32: of 8), E <= 256, top_k <= min(E, 16).  bias may be NULL.  All three dtypes. */
int yamoe_router_topk(const void *hidden, const void *weight, const void *bias, int32_t T, int32_t H,
                      int32_t E, int32_t top_k, int32_t dtype, int64_t *router_indices,
                      void *router_scores, void *topk_weights, void *logits, void *stream);

/* The gradient of that step (what autograd gives through the reference's four torch calls, layers.py:128-149):
 * from d_scores [T,E], the gradient of the dense router_scores, with p_k = router_scores[t, e_k] and
 * g_k = d_scores[t, e_k] at the token's picks e_k:
 *   d_logits[t, e_k] = p_k (g_k - sum_j p_j g_j), zero at every other expert
 *   d_hidden [T,H] = d_logits . weight     (the router's share of the hidden-state gradient; add the experts' share)
 *   d_weight [E,H] = d_logits^T . hidden,  d_bias [E] = column sums of d_logits  (d_bias may be NULL)
 * All tensors in the activation dtype, fp32 accumulation.  H and E multiples of 8 (fp32: of 4). */
size_t yamoe_router_backward_workspace_bytes(int32_t T, int32_t E, int32_t dtype);
int yamoe_router_backward(const void *d_scores, const int64_t *router_indices, const void *router_scores,
                          const void *hidden, const void *weight, int32_t T, int32_t H, int32_t E,
                          int32_t top_k, int32_t dtype, void *d_hidden, void *d_weight, void *d_bias,
                          void *workspace, size_t workspace_bytes, void *stream);

/* ---- diagnostics ---------------------------------------------------------------------------
 * No counterpart in the reference; not on the path of any op.  A register-only loop of
 * v_mfma_f32_32x32x16_bf16 (one wave per SIMD in each of `workgroups` workgroups of 256 threads,
 * 4 x 4 accumulator blocks, `iters` rounds of 16 MFMAs, no memory traffic in the loop) on
 * pseudo-random (random_operands != 0) or all-zero operands: the rate the matrix pipes of this
 * part sustain, for scale next to the expert GEMMs (the part runs against its power limit, so
 * the rate depends on the operand values).  *flop receives the flop count of the launch. */
int yamoe_probe_mfma_rate(int32_t workgroups, int32_t iters, int32_t random_operands, float *sink,
                          double *flop, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* YAMOE_HIP_H */
