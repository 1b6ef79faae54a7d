// C ABI of libyamoe_hip.so: argument checks, workspace carving and the launch sequences of the
// forward (csrc/moe.cpp:45-223) and backward (csrc/experts_backward.cu:126-341) expert layer.
// No allocation, no host synchronisation, every launch on the caller's stream.
#include <stdarg.h>
#include <stdio.h>

#include <atomic>

#include <cstdlib>
#include "common.h"

namespace yamoe {

static thread_local char g_error[512] = "";

void set_error(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

int check_launch(const char *what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("%s: %s", what, hipGetErrorString(e));
    return (int)e;
  }
  return 0;
}

int ensure_dynamic_lds(const void *kernel, int bytes, DeviceFlags &done, const char *what) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    set_error("%s: hipGetDevice: %s (device %d)", what, hipGetErrorString(e), dev);
    return e != hipSuccess ? (int)e : YAMOE_E_ARG;
  }
  if (done.flag[dev].load(std::memory_order_acquire)) return 0;
  e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e != hipSuccess) {
    set_error("%s: hipFuncSetAttribute(MaxDynamicSharedMemorySize=%d): %s", what, bytes, hipGetErrorString(e));
    return (int)e;
  }
  done.flag[dev].store(true, std::memory_order_release);
  return 0;
}

// kernels defined in the other translation units
template <typename T> int launch_permute(const void *, const int *, void *, int, int, int, hipStream_t);
template <typename T>
int launch_combine(const void *, const int *, const void *, int, const void *, int, void *, int, int, int, int,
                   hipStream_t);
template <typename T>
int launch_combine_backward(const void *, const void *, const int *, const int *, const void *, int, const void *, int,
                            void *, float *, float *, int, int, int, int, hipStream_t);
template <typename T>
int launch_expert_colsum(const void *, const int *, const int *, int, void *, int, int, hipStream_t);
template <typename T>
int gemm_gate_up(const void *, const int *, const void *, const void *, void *, void *, const void *, int, int, int,
                 int, int, hipStream_t);
template <typename T>
int gemm_down(const void *, const void *, const void *, void *, const void *, int, int, int, int, hipStream_t);
template <typename T>
int gemm_dgrad(const void *, const int *, int, const void *, void *, const void *, int, int, int, int, const void *,
               float *, hipStream_t);
template <typename T>
int gemm_wgrad(const void *, const void *, void *, const int *, const int *, int, int, int, int, hipStream_t);
template <typename T>
int glu_backward_rows(const void *, const void *, const float *, const float *, int, const int *, const int *, void *,
                      float *, int, int, hipStream_t);
template <typename T>
int launch_routing_grad(const float *, const int *, const void *, int, int, void *, int, int, int, hipStream_t);
template <typename T>
int stream_gate_up(const void *, const int *, const void *, const void *, void *, void *, const void *, int, int, int,
                   int, int, hipStream_t);
template <typename T>
int stream_down(const void *, const void *, const void *, void *, const void *, int, int, int, int, hipStream_t);

template <typename T>
int gemm_async_gate_up(const void *, const int *, const void *, const void *, void *, void *, const void *, int, int,
                       int, int, int, int, hipStream_t);
template <typename T>
int gemm_async_down(const void *, const void *, const void *, void *, const void *, int, int, int, int, int,
                    hipStream_t);
template <typename T>
int gemm_async_dgrad(const void *, const int *, int, const void *, void *, const void *, int, int, int, int,
                     const void *, float *, hipStream_t);
template <typename T>
int gemm_async_wgrad(const void *, const int *, int, int, const void *, void *, void *, const int *, const int *, int, int,
                     int, int, hipStream_t);
bool wgrad_writes_bias(int Md, int Nd);
bool gemm_async_supported(int Kd, int Nd, int lda, int ldb, long long a_span_bytes);
bool gemm_f32_supported(int Kd, int Nd, int lda, int ldb, long long a_span_bytes);
int gemm_f32_gate_up(const void *, const int *, const void *, const void *, void *, void *, const void *, int, int, int,
                     int, int, hipStream_t);
int gemm_f32_down(const void *, const void *, const void *, void *, const void *, int, int, int, int, hipStream_t);
bool wgrad_async_supported(int Md, int Nd);

template <typename T>
int launch_router_backward_logits(const void *, const long long *, const void *, int, int, int, void *, hipStream_t);

// the plain-FMA path (plain.hip): double precision, and sizes that are not whole 16-byte chunks
template <typename T>
int plain_forward(const void *, const void *, int, const void *, int, const void *, const void *, const void *, const void *,
                  void *, const int *, const int *, const void *, void *, void *, void *, int, int, int, int, int,
                  hipStream_t);
template <typename T>
int plain_backward(const void *, const void *, const void *, int, const void *, int, const void *, const void *, const void *,
                   const void *, void *, void *, void *, void *, void *, void *, const int *, const int *, const int *,
                   const int *, const int *, const void *, void *, void *, void *, void *, void *, void *, void *, void *, int,
                   int, int, int, int, int, int, hipStream_t);
template <typename T> int plain_fill_zero(void *, long long, hipStream_t);

template <typename T> struct HasStreamPath { static constexpr bool value = sizeof(T) == 2; };

// The MFMA tile kernels for the two forward products: the asynchronous-copy pipeline when the dtype
// and shape allow it, the register-staged kernel otherwise.
template <typename T>
// `small_rows`: experts with at most this many kept rows are on the schedule's streaming list, not tiled (0 when
// unknown); it only tightens the grid.
// sorted_idx == nullptr: x holds one row per sorted row, in order (the callers permute a hidden_states tensor of 4 GiB or
// more first: the kernels address gathered rows with 32-bit byte offsets from the start of the tensor).
static int tiles_gate_up(const void *x, const int *sorted_idx, const void *w, const void *bias, void *act, void *pre,
                         const void *sched, int N, int K, int E, int H, int I, int small_rows, hipStream_t stream) {
  const long long span = sorted_idx != nullptr ? (long long)(N / K) * H * (long long)sizeof(T) : 0;
  if constexpr (sizeof(T) == 2) {
    // the gathered source rows span the whole hidden_states tensor: N / K tokens of H elements
    if (gemm_async_supported(H, 2 * I, H, 2 * I, span))
      return gemm_async_gate_up<T>(x, sorted_idx, w, bias, act, pre, sched, N, K, E, H, I, small_rows, stream);
  } else {
    if (gemm_f32_supported(H, 2 * I, H, 2 * I, span))
      return gemm_f32_gate_up(x, sorted_idx, w, bias, act, pre, sched, N, K, E, H, I, stream);
  }
  if (span >= (1ll << 32)) { set_error("tiles_gate_up: gathered rows span 4 GiB or more"); return YAMOE_E_ARG; }
  return gemm_gate_up<T>(x, sorted_idx, w, bias, act, pre, sched, N, K, E, H, I, stream);
}
template <typename T>
static int tiles_down(const void *act, const void *w, const void *bias, void *y, const void *sched, int N, int E,
                      int H, int I, int small_rows, hipStream_t stream) {
  if constexpr (sizeof(T) == 2) {
    if (gemm_async_supported(I, H, I, H, 0))
      return gemm_async_down<T>(act, w, bias, y, sched, N, E, H, I, small_rows, stream);
  } else {
    if (gemm_f32_supported(I, H, I, H, 0)) return gemm_f32_down(act, w, bias, y, sched, N, E, H, I, stream);
  }
  return gemm_down<T>(act, w, bias, y, sched, N, E, H, I, stream);
}

// g_rows == nullptr: g holds one row per sorted row; otherwise row p of the product reads g[g_rows[p] / g_div]
// (g_span_bytes = size of the gathered tensor).  With dot_part the kernels also leave, per row, 2 * ceil(Nd / 256)
// partial sums of <fp32 product row, dot_with row> (dot_with has the output's shape).
template <typename T>
static int tiles_dgrad(const void *g, const int *g_rows, int g_div, long long g_span_bytes, const void *w, void *out,
                       const void *sched, int N, int E, int Kd, int Nd, const void *dot_with, float *dot_part,
                       hipStream_t stream) {
  if constexpr (sizeof(T) == 2) {
    if (gemm_async_supported(Kd, Nd, Kd, Kd, g_rows ? g_span_bytes : 0))
      return gemm_async_dgrad<T>(g, g_rows, g_div, w, out, sched, N, E, Kd, Nd, dot_with, dot_part, stream);
  }
  if (g_rows != nullptr && g_span_bytes >= (1ll << 32)) { set_error("tiles_dgrad: gathered rows span 4 GiB or more"); return YAMOE_E_ARG; }
  return gemm_dgrad<T>(g, g_rows, g_div, w, out, sched, N, E, Kd, Nd, dot_with, dot_part, stream);
}

// True when the weight-gradient kernel for this dtype and shape can gather the rows of its left operand by token
// (the register-staged kernel wants them in expert order).
template <typename T> static bool wgrad_gathers(int Md, int Nd) {
  if constexpr (sizeof(T) == 2) return wgrad_async_supported(Md, Nd);
  return false;
}

// True when the weight-gradient kernel for this dtype and shape also leaves the bias gradient (the per-expert column
// sums of its right operand), so that no launch of expert_colsum_kernel is needed for it.
template <typename T> static bool wgrad_sums_bias(int Md, int Nd) {
  if constexpr (sizeof(T) == 2) return wgrad_writes_bias(Md, Nd);
  return false;
}

// l_rows (with wgrad_gathers only): sorted row p of the left operand is row l_rows[p] / l_div of L; the list holds
// n_rows values below n_rows and is followed by at least 32 readable ints.  d_bias (with wgrad_sums_bias only): [E, Nd].
template <typename T>
static int tiles_wgrad(const void *L, const int *l_rows, int l_div, int n_rows, const void *R, void *dW, void *d_bias,
                       const int *counts, const int *offsets, int capacity, int E, int Md, int Nd, hipStream_t stream) {
  if constexpr (sizeof(T) == 2) {
    if (wgrad_async_supported(Md, Nd))
      return gemm_async_wgrad<T>(L, l_rows, l_div, n_rows, R, dW, d_bias, counts, offsets, capacity, E, Md, Nd, stream);
  }
  if (l_rows != nullptr || d_bias != nullptr) { set_error("tiles_wgrad: this kernel takes its rows in expert order and sums no bias"); return YAMOE_E_ARG; }
  return gemm_wgrad<T>(L, R, dW, counts, offsets, capacity, E, Md, Nd, stream);
}

__global__ void fill_zero_kernel(uint32_t *p, long long n_words) {
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  long long stride = (long long)gridDim.x * blockDim.x;
  for (; i < n_words; i += stride) p[i] = 0u;
}
static int fill_zero(void *p, size_t bytes, hipStream_t stream) {
  long long words = (long long)((bytes + 3) / 4);
  if (words == 0) return 0;
  long long blocks = (words + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, (uint32_t *)p, words);
  return check_launch("fill_zero_kernel");
}

static int check_problem(const yamoe_problem *p, const char *who) {
  if (!p) { set_error("%s: null problem", who); return YAMOE_E_ARG; }
  if (p->T < 0 || p->K <= 0 || p->E <= 0 || p->H <= 0 || p->I <= 0) {
    set_error("%s: need T >= 0 and K, E, H, I > 0 (T=%d K=%d E=%d H=%d I=%d)", who, p->T, p->K, p->E, p->H, p->I);
    return YAMOE_E_ARG;
  }
  if (p->dtype != YAMOE_F32 && p->dtype != YAMOE_F16 && p->dtype != YAMOE_BF16 && p->dtype != YAMOE_F64) {
    set_error("%s: unknown dtype %d", who, p->dtype);
    return YAMOE_E_DTYPE;
  }
  if (p->rw_cols != p->E && p->rw_cols != p->K) {
    set_error("%s: routing_weights must be [T,E] or [T,K] (got %d columns, E=%d K=%d)", who, p->rw_cols, p->E, p->K);
    return YAMOE_E_ARG;
  }
  if ((long long)p->T * p->K > 0x7fffffffLL / 2) {
    set_error("%s: T*K too large", who);
    return YAMOE_E_ARG;
  }
  return 0;
}

// The GEMM kernels address gathered token rows (hidden_states in the gate_up product and its weight gradient, grad_out
// in the input gradient of the down projection) with 32-bit byte offsets from the start of the tensor.  A tensor of
// 4 GiB or more is permuted into expert order first (one more [N, H] buffer each, one more launch that moves
// 2 * N * H elements) and read in order.  YAMOE_GATHER_SPAN_BYTES lowers the limit (the tests use it to run this path
// at small sizes).
static bool gathers_need_permute(const yamoe_problem *p) {
  long long limit = 1ll << 32;
  if (const char *e = getenv("YAMOE_GATHER_SPAN_BYTES")) {
    const long long v = atoll(e);
    if (v > 0 && v < limit) limit = v;
  }
  return (long long)p->T * p->H * (long long)dtype_size(p->dtype) >= limit;
}

// Carves 256-byte aligned regions out of the workspace.
struct Carver {
  char *base;
  size_t used = 0;
  explicit Carver(void *b) : base((char *)b) {}
  void *take(size_t bytes) {
    void *p = base ? base + used : nullptr;
    used += align_up(bytes == 0 ? 1 : bytes, 256);
    return p;
  }
};

struct ForwardBuffers {
  int *sorted_expert, *sorted_idx, *inv_pos, *counts, *offsets;
  void *schedule, *route_ws, *act, *y_perm;
  void *x_perm;  // hidden rows in expert order: only with gathers_need_permute
  size_t schedule_bytes, route_ws_bytes;
};

static size_t carve_forward(const yamoe_problem *p, void *ws, ForwardBuffers *b) {
  const size_t N = (size_t)p->T * p->K, es = dtype_size(p->dtype);
  Carver c(ws);
  b->sorted_expert = (int *)c.take(N * 4);
  b->sorted_idx = (int *)c.take(N * 4);
  b->inv_pos = (int *)c.take(N * 4);
  b->counts = (int *)c.take((size_t)p->E * 4);
  b->offsets = (int *)c.take(((size_t)p->E + 1) * 4);
  b->schedule_bytes = yamoe_schedule_bytes((int)N, p->E);
  b->schedule = c.take(b->schedule_bytes);
  b->route_ws_bytes = yamoe_route_workspace_bytes((int)N, p->E);
  b->route_ws = c.take(b->route_ws_bytes);
  b->act = c.take(N * p->I * es);
  // sized for the larger of H and I: the backward reuses this region for d_act [N, I]
  b->y_perm = c.take(N * (size_t)(p->H > p->I ? p->H : p->I) * es);
  b->x_perm = gathers_need_permute(p) ? c.take(N * p->H * es) : nullptr;
  return c.used;
}

struct BackwardBuffers {
  ForwardBuffers f;
  void *x_perm, *pre, *g_y_perm, *d_act, *d_pre, *d_x_perm;
  void *gy_perm;  // grad_out rows in expert order, un-weighted: only with gathers_need_permute
  float *w_sorted, *row_dot, *dot_part;
  int n_part;
};

static size_t carve_backward(const yamoe_problem *p, void *ws, BackwardBuffers *b) {
  size_t used = carve_forward(p, ws, &b->f);
  const size_t N = (size_t)p->T * p->K, es = dtype_size(p->dtype);
  Carver c(ws ? (char *)ws + used : nullptr);
  // hidden rows in expert order: only where the gate_up weight-gradient kernel cannot gather them itself
  const bool gathers = !gathers_need_permute(p) &&
                       (es == 2 ? wgrad_gathers<bf16_t>(p->H, 2 * p->I) : wgrad_gathers<float>(p->H, 2 * p->I));
  b->x_perm = gathers ? nullptr : b->f.x_perm != nullptr ? b->f.x_perm : c.take(N * p->H * es);
  b->gy_perm = gathers_need_permute(p) ? c.take(N * p->H * es) : nullptr;
  b->pre = c.take(N * 2 * p->I * es);
  b->g_y_perm = c.take(N * p->H * es);
  b->d_pre = c.take(N * 2 * p->I * es);
  // d_act [N, I] reuses the y_perm region (dead after the combine backward)
  b->d_act = b->f.y_perm;
  b->d_x_perm = c.take(N * p->H * es);
  b->w_sorted = (float *)c.take(N * (es == 8 ? sizeof(double) : sizeof(float)));  // (doubles on the double-precision path)
  b->row_dot = (float *)c.take(N * (es == 8 ? sizeof(double) : sizeof(float)));
  // 16-bit data: partial row dots of the down projection's input gradient with the activations, two per 256-column
  // tile of I, written by that GEMM from its fp32 accumulators
  b->n_part = es == 2 ? 2 * ceil_div(p->I, kColTile) : 0;
  b->dot_part = b->n_part ? (float *)c.take(N * (size_t)b->n_part * sizeof(float)) : nullptr;
  // the weight-gradient kernel's copies of an expert's last, partial slab of rows run up to 32 rows past the
  // end of its operand buffers; every operand is followed by another buffer of this workspace, and this pad
  // covers the case where those are smaller than 32 rows of the widest operand
  c.take(32 * (size_t)(p->H > 2 * p->I ? p->H : 2 * p->I) * es);
  return used + c.used;
}

// What a forward can keep for the backward of the same call: the activations [N, I] and the pre-activations [N, 2I]
// in sorted-row order (the backward otherwise recomputes both: the gate_up product once more).
struct Saved {
  void *act, *pre;
};
static size_t carve_saved(const yamoe_problem *p, void *base, Saved *s) {
  const size_t N = (size_t)p->T * p->K, es = dtype_size(p->dtype);
  Carver c(base);
  s->act = c.take(N * p->I * es);
  s->pre = c.take(N * 2 * p->I * es);
  // the weight-gradient kernel's copies of an expert's last, partial slab of rows run up to 32 rows past the end of
  // the activations: into the pre-activations, and for a handful of rows beyond those, into this pad
  c.take(32 * (size_t)p->I * es);
  return c.used;
}

#define YAMOE_TRY(expr)        \
  do {                         \
    int rc_ = (expr);          \
    if (rc_ != 0) return rc_;  \
  } while (0)

template <typename T>
static int forward_impl(const yamoe_problem *p, const void *x, const void *idx, const void *rw, const void *wgu,
                        const void *bgu, const void *wd, const void *bd, void *out, void *ws, const Saved *keep,
                        hipStream_t stream) {
  ForwardBuffers b;
  carve_forward(p, ws, &b);
  void *pre = nullptr;
  if (keep != nullptr) { b.act = keep->act; pre = keep->pre; }  // (the workspace's own act region is then unused)
  const int N = p->T * p->K;
  void *st = (void *)stream;
  if (N == 0 || p->T == 0) return 0;
  const int stream_rows = HasStreamPath<T>::value ? kStreamMaxRows : 0;
  // At most 4 assignments per expert on average (decode): every expert goes to the streaming kernel, in chunks of
  // stream_rows rows where one has more, and the tile kernels, whose lists are then empty, are not launched (two
  // launches of 4.5 us each that found nothing to do at 64 tokens on 128 experts).
  const bool everything = HasStreamPath<T>::value && sched_may_stream_everything(N, p->E);
  YAMOE_TRY(route_and_schedule(idx, p->idx_i64, N, p->E, p->capacity, b.sorted_expert, b.sorted_idx, b.counts, b.offsets,
                               b.inv_pos, b.route_ws, b.route_ws_bytes, everything ? kStreamEverything : stream_rows,
                               b.schedule, b.schedule_bytes, st));
  // with no more assignments than a streamed expert may have rows, every expert is streamed as well
  const bool tiles = !everything && N > stream_rows;
  if (tiles && b.x_perm != nullptr) {  // (a hidden_states tensor too large to gather from: see gathers_need_permute)
    YAMOE_TRY(launch_permute<T>(x, b.sorted_idx, b.x_perm, N, p->K, p->H, stream));
    YAMOE_TRY(tiles_gate_up<T>(b.x_perm, nullptr, wgu, bgu, b.act, pre, b.schedule, N, p->K, p->E, p->H, p->I, stream_rows,
                               stream));
  } else if (tiles) {
    YAMOE_TRY(tiles_gate_up<T>(x, b.sorted_idx, wgu, bgu, b.act, pre, b.schedule, N, p->K, p->E, p->H, p->I, stream_rows,
                               stream));
  }
  if constexpr (HasStreamPath<T>::value)
    YAMOE_TRY(stream_gate_up<T>(x, b.sorted_idx, wgu, bgu, b.act, pre, b.schedule, N, p->K, p->E, p->H, p->I,
                                stream));
  if (tiles) YAMOE_TRY(tiles_down<T>(b.act, wd, bd, b.y_perm, b.schedule, N, p->E, p->H, p->I, stream_rows, stream));
  if constexpr (HasStreamPath<T>::value)
    YAMOE_TRY(stream_down<T>(b.act, wd, bd, b.y_perm, b.schedule, N, p->E, p->H, p->I, stream));
  YAMOE_TRY(launch_combine<T>(b.y_perm, b.inv_pos, idx, p->idx_i64, rw, p->rw_cols, out, p->T, p->K, p->E, p->H,
                              stream));
  return 0;
}

template <typename T>
static int backward_impl(const yamoe_problem *p, const void *gy, const void *x, const void *idx, const void *rw,
                         const void *wgu, const void *bgu, const void *wd, const void *bd, void *d_x, void *d_rw,
                         void *d_wgu, void *d_bgu, void *d_wd, void *d_bd, void *ws, const Saved *kept,
                         hipStream_t stream) {
  BackwardBuffers b;
  carve_backward(p, ws, &b);
  if (kept != nullptr) { b.f.act = kept->act; b.pre = kept->pre; }  // the forward's own: nothing to recompute
  const int N = p->T * p->K, E = p->E, H = p->H, I = p->I, cap = p->capacity < 0 ? 0 : p->capacity;
  const size_t es = sizeof(T);
  void *st = (void *)stream;
  YAMOE_TRY(fill_zero(d_rw, (size_t)p->T * p->rw_cols * es, stream));
  if (N == 0) {
    YAMOE_TRY(fill_zero(d_wgu, (size_t)E * H * 2 * I * es, stream));
    YAMOE_TRY(fill_zero(d_bgu, (size_t)E * 2 * I * es, stream));
    YAMOE_TRY(fill_zero(d_wd, (size_t)E * I * H * es, stream));
    YAMOE_TRY(fill_zero(d_bd, (size_t)E * H * es, stream));
    return 0;
  }
  YAMOE_TRY(route_and_schedule(idx, p->idx_i64, N, E, cap, b.f.sorted_expert, b.f.sorted_idx, b.f.counts, b.f.offsets,
                               b.f.inv_pos, b.f.route_ws, b.f.route_ws_bytes, 0, b.f.schedule, b.f.schedule_bytes, st));
  // forward recompute of the first product only: activations and pre-activations
  const bool permuted = b.gy_perm != nullptr;  // hidden_states and grad_out too large to gather from
  const bool gathers = !permuted && wgrad_gathers<T>(H, 2 * I);
  if (!gathers) YAMOE_TRY(launch_permute<T>(x, b.f.sorted_idx, b.x_perm, N, p->K, H, stream));
  if (kept != nullptr) {
    // activations and pre-activations come from the forward
  } else if (permuted) {
    YAMOE_TRY(tiles_gate_up<T>(b.x_perm, nullptr, wgu, bgu, b.f.act, b.pre, b.f.schedule, N, p->K, E, H, I, 0, stream));
  } else {
    YAMOE_TRY(tiles_gate_up<T>(x, b.f.sorted_idx, wgu, bgu, b.f.act, b.pre, b.f.schedule, N, p->K, E, H, I, 0, stream));
  }
  // combine backward: g_y_perm = grad_out[tok] * w, and the bias part of the routing gradient
  YAMOE_TRY(launch_combine_backward<T>(gy, bd, b.f.sorted_idx, b.f.inv_pos, idx, p->idx_i64, rw, p->rw_cols, b.g_y_perm,
                                       b.w_sorted, b.row_dot, N, p->K, E, H, stream));
  // down projection: bias and weight gradients from the weighted rows; the input gradient from the un-weighted
  // rows of grad_out, gathered by token (its dot with the activations is the rest of the routing gradient)
  // (the bias gradients are the column sums of the weight gradients' right operands: taken by those kernels where
  // they can, by a launch of their own otherwise)
  const bool bd_fused = wgrad_sums_bias<T>(I, H), bgu_fused = wgrad_sums_bias<T>(H, 2 * I);
  if (!bd_fused) YAMOE_TRY(launch_expert_colsum<T>(b.g_y_perm, b.f.counts, b.f.offsets, cap, d_bd, E, H, stream));
  if (permuted) {
    YAMOE_TRY(launch_permute<T>(gy, b.f.sorted_idx, b.gy_perm, N, p->K, H, stream));
    YAMOE_TRY(tiles_dgrad<T>(b.gy_perm, nullptr, 1, 0, wd, b.d_act, b.f.schedule, N, E, /*Kd=*/H, /*Nd=*/I, b.f.act,
                             b.dot_part, stream));
  } else {
    YAMOE_TRY(tiles_dgrad<T>(gy, b.f.sorted_idx, p->K, (long long)p->T * H * (long long)es, wd, b.d_act, b.f.schedule, N, E,
                             /*Kd=*/H, /*Nd=*/I, b.f.act, b.dot_part, stream));
  }
  YAMOE_TRY(tiles_wgrad<T>(b.f.act, nullptr, 1, 0, b.g_y_perm, d_wd, bd_fused ? d_bd : nullptr, b.f.counts, b.f.offsets, cap, E,
                           /*Md=*/I, /*Nd=*/H, stream));
  // GLU backward (scaled by the routing weight) and the routing gradient
  YAMOE_TRY(glu_backward_rows<T>(b.d_act, b.pre, b.w_sorted, b.dot_part, b.n_part, b.f.sorted_idx, b.f.inv_pos, b.d_pre,
                                 b.row_dot, N, I, stream));
  YAMOE_TRY(launch_routing_grad<T>(b.row_dot, b.f.inv_pos, idx, p->idx_i64, p->rw_cols, d_rw, N, p->K, E, stream));
  // gate_up projection
  if (!bgu_fused) YAMOE_TRY(launch_expert_colsum<T>(b.d_pre, b.f.counts, b.f.offsets, cap, d_bgu, E, 2 * I, stream));
  YAMOE_TRY(tiles_dgrad<T>(b.d_pre, nullptr, 1, 0, wgu, b.d_x_perm, b.f.schedule, N, E, /*Kd=*/2 * I, /*Nd=*/H, nullptr,
                           nullptr, stream));
  // (the hidden rows gathered by token where the kernel can do that and hidden_states is below 4 GiB; sorted_idx is
  // followed in the workspace by inv_pos and the rest: readable well past its end)
  if (gathers)
    YAMOE_TRY(tiles_wgrad<T>(x, b.f.sorted_idx, p->K, N, b.d_pre, d_wgu, bgu_fused ? d_bgu : nullptr, b.f.counts, b.f.offsets,
                             cap, E, /*Md=*/H, /*Nd=*/2 * I, stream));
  else
    YAMOE_TRY(tiles_wgrad<T>(b.x_perm, nullptr, 1, 0, b.d_pre, d_wgu, bgu_fused ? d_bgu : nullptr, b.f.counts, b.f.offsets,
                             cap, E, /*Md=*/H, /*Nd=*/2 * I, stream));
  // permute backward: d_hidden[t] = sum_k d_x_perm[inv_pos[t,k]]
  YAMOE_TRY(launch_combine<T>(b.d_x_perm, b.f.inv_pos, idx, p->idx_i64, nullptr, p->K, d_x, p->T, p->K, E, H, stream));
  return 0;
}

// Double precision, and hidden or intermediate sizes that are not whole 16-byte chunks (the unit the MFMA kernels
// copy): the same lists, then the kernels of plain.hip.
static bool takes_plain_path(const yamoe_problem *p) {
  if (p->dtype == YAMOE_F64) return true;
  const int vec = 16 / (int)dtype_size(p->dtype);
  return p->H % vec != 0 || p->I % vec != 0;
}

template <typename T>
static int forward_plain(const yamoe_problem *p, const void *x, const void *idx, const void *rw, const void *wgu,
                       const void *bgu, const void *wd, const void *bd, void *out, void *ws, const Saved *keep,
                       hipStream_t stream) {
  ForwardBuffers b;
  carve_forward(p, ws, &b);
  const int N = p->T * p->K;
  if (N == 0 || p->T == 0) return 0;
  YAMOE_TRY(route_and_schedule(idx, p->idx_i64, N, p->E, p->capacity, b.sorted_expert, b.sorted_idx, b.counts, b.offsets,
                               b.inv_pos, b.route_ws, b.route_ws_bytes, 0, b.schedule, b.schedule_bytes, (void *)stream));
  return plain_forward<T>(x, idx, p->idx_i64, rw, p->rw_cols, wgu, bgu, wd, bd, out, b.sorted_idx, b.inv_pos, b.schedule,
                          keep ? keep->act : b.act, keep ? keep->pre : nullptr, b.y_perm, p->T, p->K, p->E, p->H, p->I, stream);
}

template <typename T>
static int backward_plain(const yamoe_problem *p, const void *gy, const void *x, const void *idx, const void *rw,
                        const void *wgu, const void *bgu, const void *wd, const void *bd, void *d_x, void *d_rw, void *d_wgu,
                        void *d_bgu, void *d_wd, void *d_bd, void *ws, const Saved *kept, hipStream_t stream) {
  BackwardBuffers b;
  carve_backward(p, ws, &b);
  if (kept != nullptr) { b.f.act = kept->act; b.pre = kept->pre; }
  const int N = p->T * p->K, E = p->E, H = p->H, I = p->I, cap = p->capacity < 0 ? 0 : p->capacity;
  if (N == 0) {
    YAMOE_TRY(plain_fill_zero<T>(d_rw, (long long)p->T * p->rw_cols, stream));
    YAMOE_TRY(plain_fill_zero<T>(d_wgu, (long long)E * H * 2 * I, stream));
    YAMOE_TRY(plain_fill_zero<T>(d_bgu, (long long)E * 2 * I, stream));
    YAMOE_TRY(plain_fill_zero<T>(d_wd, (long long)E * I * H, stream));
    YAMOE_TRY(plain_fill_zero<T>(d_bd, (long long)E * H, stream));
    return 0;
  }
  YAMOE_TRY(route_and_schedule(idx, p->idx_i64, N, E, cap, b.f.sorted_expert, b.f.sorted_idx, b.f.counts, b.f.offsets,
                               b.f.inv_pos, b.f.route_ws, b.f.route_ws_bytes, 0, b.f.schedule, b.f.schedule_bytes,
                               (void *)stream));
  return plain_backward<T>(gy, x, idx, p->idx_i64, rw, p->rw_cols, wgu, bgu, wd, bd, d_x, d_rw, d_wgu, d_bgu, d_wd, d_bd,
                      b.f.sorted_expert, b.f.sorted_idx, b.f.inv_pos, b.f.counts, b.f.offsets, b.f.schedule, b.f.act, b.pre,
                      b.g_y_perm, b.d_act, b.d_pre, b.d_x_perm, b.w_sorted, b.row_dot, p->T, p->K, E, H, I, cap,
                      kept == nullptr ? 1 : 0, stream);
}

}  // namespace yamoe

using namespace yamoe;

#define YAMOE_DISPATCH_ALL(dtype, CALL)                                   \
  switch (dtype) {                                                        \
    case YAMOE_F64: { typedef double T; return CALL; }                    \
    case YAMOE_F32: { typedef float T; return CALL; }                     \
    case YAMOE_BF16: { typedef bf16_t T; return CALL; }                   \
    case YAMOE_F16: { typedef f16_t T; return CALL; }                     \
    default: set_error("unknown dtype %d", dtype); return YAMOE_E_DTYPE;  \
  }

#define YAMOE_DISPATCH(dtype, CALL)                                       \
  switch (dtype) {                                                        \
    case YAMOE_F32: { typedef float T; return CALL; }                     \
    case YAMOE_BF16: { typedef bf16_t T; return CALL; }                   \
    case YAMOE_F16: { typedef f16_t T; return CALL; }                     \
    default: set_error("unknown dtype %d", dtype); return YAMOE_E_DTYPE;  \
  }

extern "C" int yamoe_abi_version(void) { return YAMOE_ABI_VERSION; }
extern "C" const char *yamoe_last_error(void) { return g_error; }

static int check_gemm_shape(const char *who, int N, int E, int H, int I, int dtype) {
  if (N < 0 || E <= 0 || H <= 0 || I <= 0) { set_error("%s: bad size", who); return YAMOE_E_ARG; }
  if (dtype != YAMOE_F32 && dtype != YAMOE_F16 && dtype != YAMOE_BF16) {
    set_error("%s: unknown dtype %d", who, dtype);
    return YAMOE_E_DTYPE;
  }
  int vec = 16 / (int)dtype_size(dtype);
  if (H % vec != 0 || I % vec != 0) {
    set_error("%s: H and I must be multiples of %d for this dtype (H=%d I=%d)", who, vec, H, I);
    return YAMOE_E_ARG;
  }
  return 0;
}

template <typename T>
static int gate_up_both(const void *x, const int *sorted_idx, const void *w, const void *bias, void *act, void *pre,
                        const void *sched, int N, int K, int E, int H, int I, hipStream_t stream) {
  YAMOE_TRY(tiles_gate_up<T>(x, sorted_idx, w, bias, act, pre, sched, N, K, E, H, I, 0, stream));
  if constexpr (HasStreamPath<T>::value)
    YAMOE_TRY(stream_gate_up<T>(x, sorted_idx, w, bias, act, pre, sched, N, K, E, H, I, stream));
  return 0;
}
template <typename T>
static int down_both(const void *act, const void *w, const void *bias, void *y, const void *sched, int N, int E, int H,
                     int I, hipStream_t stream) {
  YAMOE_TRY(tiles_down<T>(act, w, bias, y, sched, N, E, H, I, 0, stream));
  if constexpr (HasStreamPath<T>::value) YAMOE_TRY(stream_down<T>(act, w, bias, y, sched, N, E, H, I, stream));
  return 0;
}

extern "C" int yamoe_gate_up(const void *x, const int32_t *sorted_idx, const void *gate_up_proj,
                             const void *gate_up_proj_bias, void *act, void *pre_act, const void *schedule, int32_t N,
                             int32_t K, int32_t E, int32_t H, int32_t I, int32_t dtype, void *stream) {
  YAMOE_TRY(check_gemm_shape("yamoe_gate_up", N, E, H, I, dtype));
  if (N == 0) return 0;
  if (!x || !sorted_idx || !gate_up_proj || !act || !schedule || K <= 0) {
    set_error("yamoe_gate_up: null pointer or K <= 0");
    return YAMOE_E_ARG;
  }
  if ((long long)(N / K) * H * (long long)dtype_size(dtype) >= (1ll << 32)) {
    set_error("yamoe_gate_up: x of 4 GiB or more is not supported (rows gathered with 32-bit byte offsets)");
    return YAMOE_E_ARG;
  }
  YAMOE_DISPATCH(dtype, gate_up_both<T>(x, sorted_idx, gate_up_proj, gate_up_proj_bias, act, pre_act, schedule, N, K,
                                        E, H, I, (hipStream_t)stream));
}

extern "C" int yamoe_down(const void *act, const void *down_proj, const void *down_proj_bias, void *y_perm,
                          const void *schedule, int32_t N, int32_t E, int32_t H, int32_t I, int32_t dtype,
                          void *stream) {
  YAMOE_TRY(check_gemm_shape("yamoe_down", N, E, H, I, dtype));
  if (N == 0) return 0;
  if (!act || !down_proj || !y_perm || !schedule) {
    set_error("yamoe_down: null pointer");
    return YAMOE_E_ARG;
  }
  YAMOE_DISPATCH(dtype, down_both<T>(act, down_proj, down_proj_bias, y_perm, schedule, N, E, H, I,
                                     (hipStream_t)stream));
}

extern "C" size_t yamoe_experts_workspace_bytes(const yamoe_problem *p) {
  if (check_problem(p, "yamoe_experts_workspace_bytes")) return 0;
  ForwardBuffers b;
  return carve_forward(p, nullptr, &b);
}

// checks and dispatch shared by yamoe_experts_forward and yamoe_experts_forward_keep
static int run_forward(const char *who, const yamoe_problem *p, const void *hidden_states, const void *router_indices,
                       const void *routing_weights, const void *gate_up_proj, const void *gate_up_proj_bias,
                       const void *down_proj, const void *down_proj_bias, void *out, void *kept, size_t kept_bytes,
                       bool keeps, void *workspace, size_t workspace_bytes, void *stream) {
  YAMOE_TRY(check_problem(p, who));
  if (p->T == 0) return 0;
  if (!hidden_states || !router_indices || !routing_weights || !gate_up_proj || !gate_up_proj_bias || !down_proj ||
      !down_proj_bias || !out || !workspace || (keeps && !kept)) {
    set_error("%s: null pointer", who);
    return YAMOE_E_ARG;
  }
  size_t need = yamoe_experts_workspace_bytes(p);
  if (workspace_bytes < need) {
    set_error("%s: workspace too small (%zu < %zu)", who, workspace_bytes, need);
    return YAMOE_E_WORKSPACE;
  }
  Saved sv = {};
  if (keeps && kept_bytes < carve_saved(p, kept, &sv)) {
    set_error("%s: the buffer for the kept activations is too small (%zu < %zu)", who, kept_bytes, carve_saved(p, nullptr, &sv));
    return YAMOE_E_WORKSPACE;
  }
  const Saved *keep = keeps ? &sv : nullptr;
  if (takes_plain_path(p)) {
    YAMOE_DISPATCH_ALL(p->dtype, forward_plain<T>(p, hidden_states, router_indices, routing_weights, gate_up_proj,
                                                  gate_up_proj_bias, down_proj, down_proj_bias, out, workspace, keep,
                                                  (hipStream_t)stream));
  }
  YAMOE_DISPATCH(p->dtype, forward_impl<T>(p, hidden_states, router_indices, routing_weights, gate_up_proj,
                                           gate_up_proj_bias, down_proj, down_proj_bias, out, workspace, keep,
                                           (hipStream_t)stream));
}

extern "C" int yamoe_experts_forward(const yamoe_problem *p, const void *hidden_states, const void *router_indices,
                                     const void *routing_weights, const void *gate_up_proj,
                                     const void *gate_up_proj_bias, const void *down_proj, const void *down_proj_bias,
                                     void *out, void *workspace, size_t workspace_bytes, void *stream) {
  return run_forward("yamoe_experts_forward", p, hidden_states, router_indices, routing_weights, gate_up_proj,
                     gate_up_proj_bias, down_proj, down_proj_bias, out, nullptr, 0, false, workspace, workspace_bytes, stream);
}

// ---- the training pair: a forward that keeps what the backward would recompute ----------------------------------
extern "C" size_t yamoe_experts_kept_bytes(const yamoe_problem *p) {
  if (check_problem(p, "yamoe_experts_kept_bytes")) return 0;
  Saved sv;
  return carve_saved(p, nullptr, &sv);
}

extern "C" int yamoe_experts_forward_keep(const yamoe_problem *p, const void *hidden_states, const void *router_indices,
                                          const void *routing_weights, const void *gate_up_proj,
                                          const void *gate_up_proj_bias, const void *down_proj,
                                          const void *down_proj_bias, void *out, void *kept, size_t kept_bytes,
                                          void *workspace, size_t workspace_bytes, void *stream) {
  return run_forward("yamoe_experts_forward_keep", p, hidden_states, router_indices, routing_weights, gate_up_proj,
                     gate_up_proj_bias, down_proj, down_proj_bias, out, kept, kept_bytes, true, workspace, workspace_bytes,
                     stream);
}

// ---- the forward without a workspace argument ----------------------------------------------------------
// The workspace of yamoe_experts_forward_static: one array per GPU, part of the loaded code object, so no call ever
// allocates it.  In host code the array's name is only a handle for hipGetSymbolAddress; the address the kernels get
// is looked up once per device (with that device current) and kept.  Every call on a GPU uses that GPU's array.
static __device__ __align__(256) unsigned char scratch[YAMOE_STATIC_SCRATCH_BYTES];
static std::atomic<void *> g_scratch_ptr[kMaxDevices];

static int static_scratch(void **out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    set_error("yamoe_experts_forward_static: hipGetDevice: %s (device %d)", hipGetErrorString(e), dev);
    return e != hipSuccess ? (int)e : YAMOE_E_ARG;
  }
  void *ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (ptr == nullptr) {
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || ptr == nullptr) {
      set_error("yamoe_experts_forward_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
      return e != hipSuccess ? (int)e : YAMOE_E_ARG;
    }
    g_scratch_ptr[dev].store(ptr, std::memory_order_release);  // two first callers find the same address
  }
  *out = ptr;
  return 0;
}

extern "C" int yamoe_experts_forward_static(const yamoe_problem *p, const void *hidden_states,
                                            const void *router_indices, const void *routing_weights,
                                            const void *gate_up_proj, const void *gate_up_proj_bias,
                                            const void *down_proj, const void *down_proj_bias, void *out,
                                            void *stream) {
  YAMOE_TRY(check_problem(p, "yamoe_experts_forward_static"));
  if (p->T == 0) return 0;
  if (!hidden_states || !router_indices || !routing_weights || !gate_up_proj || !gate_up_proj_bias || !down_proj ||
      !down_proj_bias || !out) {
    set_error("yamoe_experts_forward_static: null pointer");
    return YAMOE_E_ARG;
  }
  const size_t need = yamoe_experts_workspace_bytes(p);
  if (need > (size_t)YAMOE_STATIC_SCRATCH_BYTES) {
    set_error("yamoe_experts_forward_static: this problem needs %zu bytes of workspace, the built-in one holds %zu "
              "(T*K*(I + max(H,I)) elements plus the routing lists); use yamoe_experts_forward with a caller-owned "
              "workspace", need, (size_t)YAMOE_STATIC_SCRATCH_BYTES);
    return YAMOE_E_WORKSPACE;
  }
  void *ws = nullptr;
  YAMOE_TRY(static_scratch(&ws));
  // Nothing in the workspace has to start at zero: every list, counter and row the kernels read is written earlier
  // in the same call, so the contents left by the previous call on this GPU do not matter.
  if (takes_plain_path(p)) {
    YAMOE_DISPATCH_ALL(p->dtype, forward_plain<T>(p, hidden_states, router_indices, routing_weights, gate_up_proj,
                                                  gate_up_proj_bias, down_proj, down_proj_bias, out, ws, nullptr,
                                                  (hipStream_t)stream));
  }
  YAMOE_DISPATCH(p->dtype, forward_impl<T>(p, hidden_states, router_indices, routing_weights, gate_up_proj,
                                           gate_up_proj_bias, down_proj, down_proj_bias, out, ws, nullptr,
                                           (hipStream_t)stream));
}

extern "C" size_t yamoe_experts_backward_workspace_bytes(const yamoe_problem *p) {
  if (check_problem(p, "yamoe_experts_backward_workspace_bytes")) return 0;
  BackwardBuffers b;
  return carve_backward(p, nullptr, &b);
}

static int run_backward(const char *who, const yamoe_problem *p, const void *grad_out, const void *hidden_states,
                        const void *router_indices, const void *routing_weights, const void *gate_up_proj,
                        const void *gate_up_proj_bias, const void *down_proj, const void *down_proj_bias,
                        const void *kept, size_t kept_bytes, bool has_kept, void *d_hidden, void *d_routing,
                        void *d_gate_up_proj, void *d_gate_up_proj_bias, void *d_down_proj, void *d_down_proj_bias,
                        void *workspace, size_t workspace_bytes, void *stream) {
  YAMOE_TRY(check_problem(p, who));
  if (!gate_up_proj || !gate_up_proj_bias || !down_proj || !down_proj_bias || !d_gate_up_proj ||
      !d_gate_up_proj_bias || !d_down_proj || !d_down_proj_bias || !workspace ||
      (p->T > 0 && (!grad_out || !hidden_states || !router_indices || !routing_weights || !d_hidden || !d_routing ||
                    (has_kept && !kept)))) {
    set_error("%s: null pointer", who);
    return YAMOE_E_ARG;
  }
  size_t need = yamoe_experts_backward_workspace_bytes(p);
  if (workspace_bytes < need) {
    set_error("%s: workspace too small (%zu < %zu)", who, workspace_bytes, need);
    return YAMOE_E_WORKSPACE;
  }
  Saved sv = {};
  if (has_kept && kept_bytes < carve_saved(p, (void *)kept, &sv)) {
    set_error("%s: the buffer of kept activations is too small (%zu < %zu)", who, kept_bytes, carve_saved(p, nullptr, &sv));
    return YAMOE_E_WORKSPACE;
  }
  const Saved *k = has_kept && p->T > 0 ? &sv : nullptr;
  if (takes_plain_path(p)) {
    YAMOE_DISPATCH_ALL(p->dtype, backward_plain<T>(p, grad_out, hidden_states, router_indices, routing_weights, gate_up_proj,
                                                   gate_up_proj_bias, down_proj, down_proj_bias, d_hidden, d_routing,
                                                   d_gate_up_proj, d_gate_up_proj_bias, d_down_proj, d_down_proj_bias,
                                                   workspace, k, (hipStream_t)stream));
  }
  YAMOE_DISPATCH(p->dtype, backward_impl<T>(p, grad_out, hidden_states, router_indices, routing_weights, gate_up_proj,
                                            gate_up_proj_bias, down_proj, down_proj_bias, d_hidden, d_routing,
                                            d_gate_up_proj, d_gate_up_proj_bias, d_down_proj, d_down_proj_bias,
                                            workspace, k, (hipStream_t)stream));
}

extern "C" int yamoe_experts_backward(const yamoe_problem *p, const void *grad_out, const void *hidden_states,
                                      const void *router_indices, const void *routing_weights,
                                      const void *gate_up_proj, const void *gate_up_proj_bias, const void *down_proj,
                                      const void *down_proj_bias, void *d_hidden, void *d_routing,
                                      void *d_gate_up_proj, void *d_gate_up_proj_bias, void *d_down_proj,
                                      void *d_down_proj_bias, void *workspace, size_t workspace_bytes, void *stream) {
  return run_backward("yamoe_experts_backward", p, grad_out, hidden_states, router_indices, routing_weights, gate_up_proj,
                      gate_up_proj_bias, down_proj, down_proj_bias, nullptr, 0, false, d_hidden, d_routing, d_gate_up_proj,
                      d_gate_up_proj_bias, d_down_proj, d_down_proj_bias, workspace, workspace_bytes, stream);
}

extern "C" int yamoe_experts_backward_kept(const yamoe_problem *p, const void *grad_out, const void *hidden_states,
                                           const void *router_indices, const void *routing_weights,
                                           const void *gate_up_proj, const void *gate_up_proj_bias,
                                           const void *down_proj, const void *down_proj_bias, const void *kept,
                                           size_t kept_bytes, void *d_hidden, void *d_routing, void *d_gate_up_proj,
                                           void *d_gate_up_proj_bias, void *d_down_proj, void *d_down_proj_bias,
                                           void *workspace, size_t workspace_bytes, void *stream) {
  return run_backward("yamoe_experts_backward_kept", p, grad_out, hidden_states, router_indices, routing_weights,
                      gate_up_proj, gate_up_proj_bias, down_proj, down_proj_bias, kept, kept_bytes, true, d_hidden, d_routing,
                      d_gate_up_proj, d_gate_up_proj_bias, d_down_proj, d_down_proj_bias, workspace, workspace_bytes, stream);
}

// ---- gradient of the router step ------------------------------------------------------------------------
// d_logits from the softmax over the picks (router.hip), then the two products and the column sums on the expert
// layer's own kernels, with the whole batch as the one "expert": d_hidden = d_logits . W (a [T, E] x [E, H] product of
// rows), d_weight = d_logits^T . hidden (a weight-gradient product over the T rows), d_bias = column sums.
struct RouterBackwardBuffers {
  void *d_logits, *schedule;
  int *counts, *offsets;
  size_t schedule_bytes;
};
static size_t carve_router_backward(int T, int E, int dtype, void *ws, RouterBackwardBuffers *b) {
  Carver c(ws);
  b->d_logits = c.take((size_t)T * E * dtype_size(dtype));
  b->counts = (int *)c.take(4);
  b->offsets = (int *)c.take(8);
  b->schedule_bytes = yamoe_schedule_bytes(T, 1);
  b->schedule = c.take(b->schedule_bytes);
  return c.used;
}

extern "C" size_t yamoe_router_backward_workspace_bytes(int32_t T, int32_t E, int32_t dtype) {
  if (T < 0 || E <= 0 || (dtype != YAMOE_F32 && dtype != YAMOE_F16 && dtype != YAMOE_BF16)) return 0;
  RouterBackwardBuffers b;
  return carve_router_backward(T, E, dtype, nullptr, &b);
}

template <typename T>
static int router_backward_impl(const void *d_scores, const long long *indices, const void *scores, const void *hidden,
                                const void *weight, int Tn, int H, int E, int K, void *d_hidden, void *d_weight,
                                void *d_bias, void *ws, hipStream_t stream) {
  RouterBackwardBuffers b;
  carve_router_backward(Tn, E, ElemTraits<T>::kDtype, ws, &b);
  YAMOE_TRY(launch_router_backward_logits<T>(d_scores, indices, scores, Tn, E, K, b.d_logits, stream));
  YAMOE_TRY(yamoe_regular_groups(b.counts, b.offsets, 1, Tn, (void *)stream));
  const int stream_rows = HasStreamPath<T>::value ? kStreamMaxRows : 0;
  YAMOE_TRY(yamoe_build_schedule(b.counts, b.offsets, Tn, 1, Tn, stream_rows, b.schedule, b.schedule_bytes, (void *)stream));
  // d_hidden [T, H] = d_logits [T, E] . weight [E, H]: the down-projection launchers compute rows[., Kd] x w[Kd, Nd]
  YAMOE_TRY(down_both<T>(b.d_logits, weight, nullptr, d_hidden, b.schedule, Tn, 1, /*H=*/H, /*I=*/E, stream));
  // d_weight [E, H] = d_logits^T . hidden, contraction over the T rows (the register-staged kernel: it reads nothing
  // past the end of the caller's tensors)
  YAMOE_TRY(gemm_wgrad<T>(b.d_logits, hidden, d_weight, b.counts, b.offsets, Tn, 1, /*Md=*/E, /*Nd=*/H, stream));
  if (d_bias != nullptr) YAMOE_TRY(launch_expert_colsum<T>(b.d_logits, b.counts, b.offsets, Tn, d_bias, 1, E, stream));
  return 0;
}

extern "C" int yamoe_router_backward(const void *d_scores, const int64_t *router_indices, const void *router_scores,
                                     const void *hidden, const void *weight, int32_t T_, int32_t H, int32_t E,
                                     int32_t top_k, int32_t dtype, void *d_hidden, void *d_weight, void *d_bias,
                                     void *workspace, size_t workspace_bytes, void *stream) {
  YAMOE_TRY(check_gemm_shape("yamoe_router_backward", T_, 1, H, E, dtype));
  if (top_k <= 0 || top_k > E) { set_error("yamoe_router_backward: need 1 <= top_k <= E"); return YAMOE_E_ARG; }
  if (!d_weight) { set_error("yamoe_router_backward: null pointer"); return YAMOE_E_ARG; }
  if (T_ == 0) {
    YAMOE_TRY(fill_zero(d_weight, (size_t)E * H * dtype_size(dtype), (hipStream_t)stream));
    if (d_bias) YAMOE_TRY(fill_zero(d_bias, (size_t)E * dtype_size(dtype), (hipStream_t)stream));
    return 0;
  }
  if (!d_scores || !router_indices || !router_scores || !hidden || !weight || !d_hidden || !workspace) {
    set_error("yamoe_router_backward: null pointer");
    return YAMOE_E_ARG;
  }
  if (workspace_bytes < yamoe_router_backward_workspace_bytes(T_, E, dtype)) {
    set_error("yamoe_router_backward: workspace too small");
    return YAMOE_E_WORKSPACE;
  }
  YAMOE_DISPATCH(dtype, router_backward_impl<T>(d_scores, (const long long *)router_indices, router_scores, hidden, weight,
                                                T_, H, E, top_k, d_hidden, d_weight, d_bias, workspace,
                                                (hipStream_t)stream));
}

// ---- batch_mm on the regular [E, C, *] layout -------------------------------------------------------
extern "C" size_t yamoe_batch_mm_workspace_bytes(int32_t E, int32_t C) {
  if (E <= 0 || C < 0) return 0;
  return align_up((size_t)E * 4, 256) + align_up(((size_t)E + 1) * 4, 256) + yamoe_schedule_bytes(E * C, E);
}

template <typename T>
static int batch_mm_impl(const void *x, const void *w, void *out, int E, int C, int Kd, int Nd, void *ws,
                         hipStream_t stream) {
  Carver c(ws);
  int *counts = (int *)c.take((size_t)E * 4);
  int *offsets = (int *)c.take(((size_t)E + 1) * 4);
  size_t sched_bytes = yamoe_schedule_bytes(E * C, E);
  void *sched = c.take(sched_bytes);
  YAMOE_TRY(yamoe_regular_groups(counts, offsets, E, C, (void *)stream));
  const int stream_rows = HasStreamPath<T>::value ? kStreamMaxRows : 0;
  YAMOE_TRY(yamoe_build_schedule(counts, offsets, E * C, E, C, stream_rows, sched, sched_bytes, (void *)stream));
  // the down-projection launchers compute rows[.,Kd] x w[e][Kd,Nd] with no bias: exactly this product
  return down_both<T>(x, w, nullptr, out, sched, E * C, E, /*H=*/Nd, /*I=*/Kd, stream);
}

extern "C" int yamoe_batch_mm(const void *x, const void *weights, void *output, int32_t E, int32_t C, int32_t Kd,
                              int32_t Nd, int32_t dtype, void *workspace, size_t workspace_bytes, void *stream) {
  YAMOE_TRY(check_gemm_shape("yamoe_batch_mm", E * C, E, Nd, Kd, dtype));
  if (C <= 0) return 0;
  if (!x || !weights || !output || !workspace || workspace_bytes < yamoe_batch_mm_workspace_bytes(E, C)) {
    set_error("yamoe_batch_mm: null pointer or workspace too small");
    return YAMOE_E_ARG;
  }
  YAMOE_DISPATCH(dtype, batch_mm_impl<T>(x, weights, output, E, C, Kd, Nd, workspace, (hipStream_t)stream));
}
