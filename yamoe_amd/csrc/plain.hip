// The expert layer on plain FMA tiles: double precision, and the shapes the MFMA kernels do not take.
//
// The reference dispatches its kernels over double as well (AT_DISPATCH_FLOATING_TYPES_AND2: csrc/gather.cu:89,
// csrc/scatter.cu:128, csrc/experts_backward.cu:236; torch::bmm takes double) and puts no alignment condition on the
// hidden and intermediate sizes, so the op accepts both here too.  The MFMA kernels move 16-byte chunks; a hidden or
// intermediate size that is not a multiple of one chunk, and every double-precision problem, runs on this path
// instead.  It is a compatibility path, not a measured one: the products run on plain FMA tiles (64 x 64 outputs per
// workgroup, 4 x 4 per thread, operands staged in LDS element by element), double accumulates in double and the other
// dtypes in float, and the steps are the ones of csrc/moe.cpp:138-220 and csrc/experts_backward.cu:164-340 on the same
// work lists as the fast path: no padded buffers, no atomics, a fixed summation order.
#include "common.h"

namespace yamoe {
namespace plain {

constexpr int kTile = 64, kStep = 16, kThreads = 256;

template <typename T> struct AccOf { typedef float type; };
template <> struct AccOf<double> { typedef double type; };

// the constants of csrc/moe.cpp:175-179 as doubles (the float 1.702f is 1.70200002...)
constexpr double kLimitD = 7.0, kAlphaD = 1.702;

__device__ inline double glu_fwd(double G, double U) {
  const double g = fmin(G, kLimitD);
  const double u = fmin(fmax(U, -kLimitD), kLimitD);
  const double s = 1.0 / (1.0 + exp(-kAlphaD * g));
  return (u + 1.0) * (g * s);
}
__device__ inline void glu_bwd(double G, double U, double dh, double &dG, double &dU) {
  const double L = kLimitD, A = kAlphaD;
  const double g = fmin(G, L), u = fmin(fmax(U, -L), L);
  const double s = 1.0 / (1.0 + exp(-A * g));
  dU = (U > L || U < -L) ? 0.0 : dh * (g * s);
  dG = (G > L) ? 0.0 : dh * (u + 1.0) * (s + g * s * (1.0 - s) * A);
}
__device__ inline float glu_fwd(float G, float U) { return glu_forward(G, U); }
__device__ inline void glu_bwd(float G, float U, float dh, float &dG, float &dU) { glu_backward(G, U, dh, dG, dU); }

// a pre-activation as the backward reads it back (the 16-bit dtypes keep clamped values off the limit: common.h)
template <typename T> __device__ inline T pre_store(typename AccOf<T>::type v, bool up) {
  if constexpr (sizeof(T) == 2) return pre_activation_store<T>(v, up);
  else return (T)v;
}
template <typename T> __device__ inline typename AccOf<T>::type ld(const T *p, long long i) { return ElemTraits<T>::to_acc(p[i]); }
template <typename T> __device__ inline void st(T *p, long long i, typename AccOf<T>::type v) { p[i] = ElemTraits<T>::from_acc(v); }

enum { EPI_STORE = 0, EPI_GLU = 1 };

template <typename T> struct RowsArgs {
  const T *A;          // [rows, lda]; with a_rows: source row of sorted row p = a_rows[p] / a_div
  const T *B;          // [E][Kd][Nd], or with BNK [E][Nd][Kd]
  const T *bias;       // [E, Nd] or null
  T *C;                // EPI_STORE [rows, Nd]; EPI_GLU act [rows, Nd / 2]
  T *C2;               // EPI_GLU: optional pre-activations [rows, Nd]
  const int *a_rows;
  const int *sched;
  int a_div, Kd, Nd, lda, N, E;
};

// C[p, :] = A[row(p), :] . B[e] (+ bias[e]) for the rows of the schedule's row tiles; a workgroup takes 64 rows of one
// row tile (blockIdx.y = 4 * row tile + quarter) and 64 columns.
template <typename T, int EPI, bool GATHER, bool BNK>
__global__ __launch_bounds__(kThreads) void rows_gemm_kernel(const RowsArgs<T> a) {
  typedef typename AccOf<T>::type A;
  __shared__ A sa[kTile][kStep + 1], sb[kStep][kTile + 1];
  const ScheduleView sv = schedule_view(a.sched, a.N, a.E);
  const int t = blockIdx.y >> 2, quarter = blockIdx.y & 3;
  if (t >= sv.hdr[0]) return;
  const int expert = sv.row_tiles[8 * t], row0 = sv.row_tiles[8 * t + 1] + quarter * kTile;
  const int rows = sv.row_tiles[8 * t + 2] - quarter * kTile;
  if (rows <= 0) return;
  const int n0 = blockIdx.x * kTile;
  const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
  const T *Bp = a.B + (long long)expert * a.Kd * a.Nd;
  A acc[4][4] = {};
  for (int k0 = 0; k0 < a.Kd; k0 += kStep) {
    for (int i = tid; i < kTile * kStep; i += kThreads) {
      const int r = i / kStep, k = i % kStep;
      A v = 0;
      if (r < rows && k0 + k < a.Kd) {
        long long src = row0 + r;
        if (GATHER) src = a.a_rows[row0 + r] / a.a_div;
        v = ld(a.A, src * a.lda + k0 + k);
      }
      sa[r][k] = v;
    }
    for (int i = tid; i < kTile * kStep; i += kThreads) {
      int k, n;
      if (BNK) { n = i / kStep; k = i % kStep; } else { k = i / kTile; n = i % kTile; }
      A v = 0;
      if (k0 + k < a.Kd && n0 + n < a.Nd)
        v = BNK ? ld(Bp, (long long)(n0 + n) * a.Kd + k0 + k) : ld(Bp, (long long)(k0 + k) * a.Nd + n0 + n);
      sb[k][n] = v;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < kStep; ++k) {
      A av[4], bv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) { av[i] = sa[ty * 4 + i][k]; bv[i] = sb[k][tx * 4 + i]; }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] += av[i] * bv[j];
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = ty * 4 + i;
    if (r >= rows) continue;
    const long long p = row0 + r;
    A v[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      v[j] = acc[i][j] + ((a.bias != nullptr && n < a.Nd) ? ld(a.bias, (long long)expert * a.Nd + n) : (A)0);
    }
    if (EPI == EPI_STORE) {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (n0 + tx * 4 + j < a.Nd) st(a.C, p * a.Nd + n0 + tx * 4 + j, v[j]);
    } else {
#pragma unroll
      for (int j = 0; j < 4; j += 2) {  // (Nd is even: a (gate, up) pair is valid or invalid as a whole)
        const int n = n0 + tx * 4 + j;
        if (n < a.Nd) {
          st(a.C, p * (a.Nd / 2) + n / 2, glu_fwd(v[j], v[j + 1]));
          if (a.C2 != nullptr) {
            a.C2[p * a.Nd + n] = pre_store<T>(v[j], false);
            a.C2[p * a.Nd + n + 1] = pre_store<T>(v[j + 1], true);
          }
        }
      }
    }
  }
}

// dW[e] = L_e^T . R_e over the expert's kept rows: L [rows, Md] (with l_rows: gathered), R [rows, Nd]
template <typename T>
__global__ __launch_bounds__(kThreads) void wgrad_kernel(const T *L, const int *l_rows, int l_div, const T *R, T *dW,
                                                         const int *counts, const int *offsets, int capacity, int Md,
                                                         int Nd) {
  typedef typename AccOf<T>::type A;
  __shared__ A sl[kStep][kTile + 1], sr[kStep][kTile + 1];
  const int expert = blockIdx.z, m0 = blockIdx.y * kTile, n0 = blockIdx.x * kTile;
  const int rows = max(min(counts[expert], capacity), 0);
  const long long first = offsets[expert];
  const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
  A acc[4][4] = {};
  for (int k0 = 0; k0 < rows; k0 += kStep) {
    for (int i = tid; i < kStep * kTile; i += kThreads) {
      const int k = i / kTile, c = i % kTile;
      A lv = 0, rv = 0;
      if (k0 + k < rows) {
        long long src = first + k0 + k;
        if (m0 + c < Md) lv = ld(L, (l_rows != nullptr ? (long long)(l_rows[src] / l_div) : src) * Md + m0 + c);
        if (n0 + c < Nd) rv = ld(R, src * Nd + n0 + c);
      }
      sl[k][c] = lv;
      sr[k][c] = rv;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < kStep; ++k) {
      A av[4], bv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) { av[i] = sl[k][ty * 4 + i]; bv[i] = sr[k][tx * 4 + i]; }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] += av[i] * bv[j];
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int m = m0 + ty * 4 + i, n = n0 + tx * 4 + j;
      if (m < Md && n < Nd) st(dW, ((long long)expert * Md + m) * Nd + n, acc[i][j]);
    }
}

__device__ inline long long slot_expert(const void *idx, int i64, long long slot) {
  return i64 ? ((const long long *)idx)[slot] : (long long)((const int *)idx)[slot];
}
// the routing weight of flat slot t*K+k; rw == nullptr means 1
template <typename T>
__device__ inline typename AccOf<T>::type slot_weight(const T *rw, const void *idx, int i64, int t, int k, int K, int E,
                                                      int rw_cols) {
  if (rw == nullptr) return 1;
  if (rw_cols == K && rw_cols != E) return ld(rw, (long long)t * K + k);
  const long long e = slot_expert(idx, i64, (long long)t * K + k);
  if (e < 0 || e >= E) return 0;
  return ld(rw, (long long)t * E + e);
}

// out[t, :] = sum_k w(t, k) * y[inv_pos[t*K+k], :] in slot order (csrc/scatter.cu:66-108 without atomics)
template <typename T>
__global__ void combine_kernel(const T *y, const int *inv_pos, const void *idx, int i64, const T *rw, int rw_cols, T *out,
                               int Tn, int K, int E, int H) {
  typedef typename AccOf<T>::type A;
  const int t = blockIdx.x;
  for (int c = threadIdx.x; c < H; c += blockDim.x) {
    A acc = 0;
    for (int k = 0; k < K; ++k) {
      const int p = inv_pos[(long long)t * K + k];
      if (p >= 0) acc += slot_weight(rw, idx, i64, t, k, K, E, rw_cols) * ld(y, (long long)p * H + c);
    }
    st(out, (long long)t * H + c, acc);
  }
}

// per kept sorted row p (one workgroup): g_y[p, :] = grad_out[tok, :] * w, w_sorted[p] = w
template <typename T>
__global__ void scale_rows_kernel(const T *gy, const int *sorted_idx, const int *inv_pos, const void *idx, int i64,
                                  const T *rw, int rw_cols, T *g_y, typename AccOf<T>::type *w_sorted, int N, int K, int E,
                                  int H) {
  typedef typename AccOf<T>::type A;
  const int p = blockIdx.x;
  const int slot = sorted_idx[p];
  if (slot < 0 || slot >= N || inv_pos[slot] != p) return;  // a dropped slot: nobody reads its row
  const int t = slot / K, k = slot % K;
  const A w = slot_weight(rw, idx, i64, t, k, K, E, rw_cols);
  if (threadIdx.x == 0) w_sorted[p] = w;
  for (int c = threadIdx.x; c < H; c += blockDim.x) st(g_y, (long long)p * H + c, ld(gy, (long long)t * H + c) * w);
}

// out[e, c] = sum over the expert's kept rows of src[p, c], in row order
template <typename T>
__global__ void colsum_kernel(const T *src, const int *counts, const int *offsets, int capacity, T *out, int cols) {
  typedef typename AccOf<T>::type A;
  const int e = blockIdx.y, c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= cols) return;
  const int rows = max(min(counts[e], capacity), 0);
  const long long first = offsets[e];
  A acc = 0;
  for (int r = 0; r < rows; ++r) acc += ld(src, (first + r) * cols + c);
  st(out, (long long)e * cols + c, acc);
}

// per kept sorted row p (one workgroup): row_dot[p] = <d_act[p], act[p]> + <grad_out[tok], b_down[e]> (the routing
// gradient of the slot, csrc/experts_backward.cu:83-88), then d_pre[p] = SwiGLU backward of d_act[p] * w
// (csrc/experts_backward.cu:285-305)
template <typename T>
__global__ __launch_bounds__(kThreads) void glu_backward_kernel(const T *d_act, const T *act, const T *pre, const T *gy,
                                                                const T *b_down, const int *sorted_idx,
                                                                const int *sorted_expert, const int *inv_pos,
                                                                const typename AccOf<T>::type *w_sorted, T *d_pre,
                                                                typename AccOf<T>::type *row_dot, int N, int K, int H,
                                                                int I) {
  typedef typename AccOf<T>::type A;
  __shared__ A part[kThreads];
  const int p = blockIdx.x;
  const int slot = sorted_idx[p];
  if (slot < 0 || slot >= N || inv_pos[slot] != p) return;
  const int t = slot / K, e = sorted_expert[p];
  const A w = w_sorted[p];
  A dot = 0;
  for (int c = threadIdx.x; c < I; c += blockDim.x) {
    const A da = ld(d_act, (long long)p * I + c);
    dot += da * ld(act, (long long)p * I + c);
    A dG, dU;
    glu_bwd(ld(pre, (long long)p * 2 * I + 2 * c), ld(pre, (long long)p * 2 * I + 2 * c + 1), da * w, dG, dU);
    st(d_pre, (long long)p * 2 * I + 2 * c, dG);
    st(d_pre, (long long)p * 2 * I + 2 * c + 1, dU);
  }
  for (int c = threadIdx.x; c < H; c += blockDim.x) dot += ld(gy, (long long)t * H + c) * ld(b_down, (long long)e * H + c);
  part[threadIdx.x] = dot;
  __syncthreads();
  for (int s = kThreads / 2; s > 0; s >>= 1) {  // a fixed tree: the same sum on every run
    if ((int)threadIdx.x < s) part[threadIdx.x] += part[threadIdx.x + s];
    __syncthreads();
  }
  if (threadIdx.x == 0) row_dot[p] = part[0];
}

// d_routing[t, :]: zero, then the dots of the token's kept slots at [t, expert] (dense) or [t, k]; a token that names an
// expert twice gets the sum of both slots (one thread per token: a fixed order)
template <typename T>
__global__ void routing_grad_kernel(const typename AccOf<T>::type *row_dot, const int *inv_pos, const void *idx, int i64,
                                    int rw_cols, T *d_rw, int Tn, int K, int E) {
  typedef typename AccOf<T>::type A;
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= Tn) return;
  for (int c = 0; c < rw_cols; ++c) st(d_rw, (long long)t * rw_cols + c, (A)0);
  const bool per_slot = rw_cols == K && rw_cols != E;
  for (int k = 0; k < K; ++k) {
    const int p = inv_pos[(long long)t * K + k];
    if (p < 0) continue;
    const long long e = slot_expert(idx, i64, (long long)t * K + k);
    if (per_slot) { st(d_rw, (long long)t * K + k, row_dot[p]); continue; }
    if (e < 0 || e >= E) continue;
    A sum = row_dot[p];  // the earlier slots of this token with the same expert, summed before the one rounding
    bool later = false;
    for (int j = 0; j < K; ++j) {
      if (j == k || slot_expert(idx, i64, (long long)t * K + j) != e) continue;
      const int q = inv_pos[(long long)t * K + j];
      if (q < 0) continue;
      if (j < k) sum += row_dot[q]; else later = true;
    }
    if (!later) st(d_rw, (long long)t * E + e, sum);
  }
}

template <typename T> __global__ void fill_kernel(T *p, long long n) {
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (; i < n; i += stride) p[i] = ElemTraits<T>::from_acc(0);
}

template <typename T, int EPI, bool GATHER, bool BNK> static int launch_rows(const RowsArgs<T> &a, hipStream_t stream) {
  const int tiles = sched_max_row_tiles(a.N, a.E);
  hipLaunchKernelGGL((rows_gemm_kernel<T, EPI, GATHER, BNK>), dim3(ceil_div(a.Nd, kTile), 4 * tiles), dim3(kThreads), 0,
                     stream, a);
  return check_launch("plain rows_gemm_kernel");
}

}  // namespace plain

#define PLAIN_TRY(expr)        \
  do {                         \
    int rc_ = (expr);          \
    if (rc_ != 0) return rc_;  \
  } while (0)

// act = glu(x[tok] . Wgu[e] + bgu[e]) (and the pre-activations), y = act . Wd[e] + bd[e], rows in sorted order
template <typename T>
static int plain_gate_up_down(const T *x, const int *sorted_idx, const T *wgu, const T *bgu, const T *wd, const T *bd, T *act,
                              T *pre, T *y, const void *sched, int N, int K, int E, int H, int I, hipStream_t stream) {
  plain::RowsArgs<T> g = {};
  g.A = x; g.B = wgu; g.bias = bgu; g.C = act; g.C2 = pre; g.a_rows = sorted_idx; g.a_div = K; g.sched = (const int *)sched;
  g.Kd = H; g.Nd = 2 * I; g.lda = H; g.N = N; g.E = E;
  PLAIN_TRY((plain::launch_rows<T, plain::EPI_GLU, true, false>(g, stream)));
  if (y != nullptr) {
    plain::RowsArgs<T> d = {};
    d.A = act; d.B = wd; d.bias = bd; d.C = y; d.a_div = 1; d.sched = (const int *)sched;
    d.Kd = I; d.Nd = H; d.lda = I; d.N = N; d.E = E;
    PLAIN_TRY((plain::launch_rows<T, plain::EPI_STORE, false, false>(d, stream)));
  }
  return 0;
}

// The whole forward on the caller's lists (sorted_idx, inv_pos, schedule built with no streaming limit); `pre` (optional)
// receives the pre-activations.
template <typename T>
int plain_forward(const void *x, const void *idx, int idx_i64, const void *rw, int rw_cols, const void *wgu, const void *bgu,
                  const void *wd, const void *bd, void *out, const int *sorted_idx, const int *inv_pos, const void *sched,
                  void *act, void *pre, void *y_perm, int Tn, int K, int E, int H, int I, hipStream_t stream) {
  const int N = Tn * K;
  PLAIN_TRY(plain_gate_up_down<T>((const T *)x, sorted_idx, (const T *)wgu, (const T *)bgu, (const T *)wd, (const T *)bd,
                                  (T *)act, (T *)pre, (T *)y_perm, sched, N, K, E, H, I, stream));
  hipLaunchKernelGGL(plain::combine_kernel<T>, dim3(Tn), dim3(256), 0, stream, (const T *)y_perm, inv_pos, idx, idx_i64,
                     (const T *)rw, rw_cols, (T *)out, Tn, K, E, H);
  return check_launch("plain combine_kernel");
}

// The whole backward.  Buffers: act [N, I], pre [N, 2I], g_y [N, H], d_act [N, I], d_pre [N, 2I], d_x_perm [N, H] in T;
// w_sorted [N], row_dot [N] in the accumulation type (double for double, float otherwise).
template <typename T>
int plain_backward(const void *gy_, const void *x_, const void *idx, int idx_i64, const void *rw_, int rw_cols,
                   const void *wgu_, const void *bgu_, const void *wd_, const void *bd_, void *d_x, void *d_rw, void *d_wgu,
                   void *d_bgu, void *d_wd, void *d_bd, const int *sorted_expert, const int *sorted_idx, const int *inv_pos,
                   const int *counts, const int *offsets, const void *sched, void *act_, void *pre_, void *g_y_,
                   void *d_act_, void *d_pre_, void *d_x_perm_, void *w_sorted_, void *row_dot_, int Tn, int K, int E, int H,
                   int I, int capacity, int recompute, hipStream_t stream) {
  typedef typename plain::AccOf<T>::type A;
  const int N = Tn * K;
  const T *gy = (const T *)gy_, *x = (const T *)x_, *rw = (const T *)rw_;
  const T *wgu = (const T *)wgu_, *bgu = (const T *)bgu_, *wd = (const T *)wd_, *bd = (const T *)bd_;
  T *act = (T *)act_, *pre = (T *)pre_, *g_y = (T *)g_y_, *d_act = (T *)d_act_;
  T *d_pre = (T *)d_pre_, *d_x_perm = (T *)d_x_perm_;
  A *w_sorted = (A *)w_sorted_, *row_dot = (A *)row_dot_;
  // forward recompute of the first product: activations and pre-activations (unless the caller kept the forward's)
  if (recompute) PLAIN_TRY(plain_gate_up_down<T>(x, sorted_idx, wgu, bgu, wd, bd, act, pre, nullptr, sched, N, K, E, H, I, stream));
  // weighted rows of grad_out; bias and weight gradient of the down projection
  hipLaunchKernelGGL(plain::scale_rows_kernel<T>, dim3(N), dim3(256), 0, stream, gy, sorted_idx, inv_pos, idx, idx_i64, rw,
                     rw_cols, g_y, w_sorted, N, K, E, H);
  PLAIN_TRY(check_launch("plain scale_rows_kernel"));
  hipLaunchKernelGGL(plain::colsum_kernel<T>, dim3(ceil_div(H, 256), E), dim3(256), 0, stream, (const T *)g_y, counts, offsets,
                     capacity, (T *)d_bd, H);
  PLAIN_TRY(check_launch("plain colsum_kernel"));
  hipLaunchKernelGGL(plain::wgrad_kernel<T>, dim3(ceil_div(H, plain::kTile), ceil_div(I, plain::kTile), E),
                     dim3(plain::kThreads), 0, stream, (const T *)act, (const int *)nullptr, 1, (const T *)g_y, (T *)d_wd,
                     counts, offsets, capacity, I, H);
  PLAIN_TRY(check_launch("plain wgrad_kernel"));
  // input gradient of the down projection for the un-weighted rows of grad_out, gathered by token
  {
    plain::RowsArgs<T> a = {};
    a.A = gy; a.B = wd; a.C = d_act; a.a_rows = sorted_idx; a.a_div = K; a.sched = (const int *)sched;
    a.Kd = H; a.Nd = I; a.lda = H; a.N = N; a.E = E;   // W_down[e] is [I, H] = [n][k]
    PLAIN_TRY((plain::launch_rows<T, plain::EPI_STORE, true, true>(a, stream)));
  }
  hipLaunchKernelGGL(plain::glu_backward_kernel<T>, dim3(N), dim3(plain::kThreads), 0, stream, (const T *)d_act,
                     (const T *)act, (const T *)pre, gy, bd, sorted_idx, sorted_expert, inv_pos, (const A *)w_sorted, d_pre,
                     row_dot, N, K, H, I);
  PLAIN_TRY(check_launch("plain glu_backward_kernel"));
  hipLaunchKernelGGL(plain::routing_grad_kernel<T>, dim3(ceil_div(Tn, 256)), dim3(256), 0, stream, (const A *)row_dot, inv_pos,
                     idx, idx_i64, rw_cols, (T *)d_rw, Tn, K, E);
  PLAIN_TRY(check_launch("plain routing_grad_kernel"));
  // gate_up projection
  hipLaunchKernelGGL(plain::colsum_kernel<T>, dim3(ceil_div(2 * I, 256), E), dim3(256), 0, stream, (const T *)d_pre, counts,
                     offsets, capacity, (T *)d_bgu, 2 * I);
  PLAIN_TRY(check_launch("plain colsum_kernel"));
  {
    plain::RowsArgs<T> a = {};
    a.A = d_pre; a.B = wgu; a.C = d_x_perm; a.a_div = 1; a.sched = (const int *)sched;
    a.Kd = 2 * I; a.Nd = H; a.lda = 2 * I; a.N = N; a.E = E;   // W_gate_up[e] is [H, 2I] = [n][k]
    PLAIN_TRY((plain::launch_rows<T, plain::EPI_STORE, false, true>(a, stream)));
  }
  hipLaunchKernelGGL(plain::wgrad_kernel<T>, dim3(ceil_div(2 * I, plain::kTile), ceil_div(H, plain::kTile), E),
                     dim3(plain::kThreads), 0, stream, x, sorted_idx, K, (const T *)d_pre, (T *)d_wgu, counts, offsets,
                     capacity, H, 2 * I);
  PLAIN_TRY(check_launch("plain wgrad_kernel"));
  hipLaunchKernelGGL(plain::combine_kernel<T>, dim3(Tn), dim3(256), 0, stream, (const T *)d_x_perm, inv_pos, idx, idx_i64,
                     (const T *)nullptr, K, (T *)d_x, Tn, K, E, H);
  return check_launch("plain combine_kernel");
}

template <typename T> int plain_fill_zero(void *p, long long n, hipStream_t stream) {
  if (n <= 0) return 0;
  long long blocks = (n + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(plain::fill_kernel<T>, dim3((unsigned)blocks), dim3(256), 0, stream, (T *)p, n);
  return check_launch("plain fill_kernel");
}

#define PLAIN_INSTANTIATE(T)                                                                                              \
  template int plain_forward<T>(const void *, const void *, int, const void *, int, const void *, const void *,          \
                                const void *, const void *, void *, const int *, const int *, const void *, void *,      \
                                void *, void *, int, int, int, int, int, hipStream_t);                                    \
  template int plain_backward<T>(const void *, const void *, const void *, int, const void *, int, const void *,         \
                                 const void *, const void *, const void *, void *, void *, void *, void *, void *,       \
                                 void *, const int *, const int *, const int *, const int *, const int *, const void *,  \
                                 void *, void *, void *, void *, void *, void *, void *, void *, int, int, int, int, int, \
                                 int, int, hipStream_t);                                                                  \
  template int plain_fill_zero<T>(void *, long long, hipStream_t);
PLAIN_INSTANTIATE(double)
PLAIN_INSTANTIATE(float)
PLAIN_INSTANTIATE(bf16_t)
PLAIN_INSTANTIATE(f16_t)

}  // namespace yamoe
