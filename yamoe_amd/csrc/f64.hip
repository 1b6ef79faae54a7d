// The expert layer in double precision.
//
// The reference dispatches its kernels over double as well (AT_DISPATCH_FLOATING_TYPES_AND2: csrc/gather.cu:89,
// csrc/scatter.cu:128, csrc/experts_backward.cu:236; torch::bmm takes double), so the op accepts it here too.  It is a
// compatibility dtype, not a measured one: the products run on plain FMA tiles (64 x 64 outputs per workgroup, 4 x 4 per
// thread, operands staged in LDS), everything accumulates in double, and the steps are the ones of
// csrc/moe.cpp:138-220 and csrc/experts_backward.cu:164-340 on the same work lists as the other dtypes: no padded
// buffers, no atomics, a fixed summation order.
#include "common.h"

namespace yamoe {
namespace f64 {

constexpr int kTile = 64, kStep = 16, kThreads = 256;

// the constants of csrc/moe.cpp:175-179 as doubles (the float 1.702f is 1.70200002...)
constexpr double kLimitD = 7.0, kAlphaD = 1.702;

__device__ inline double glu_forward_d(double G, double U) {
  const double g = fmin(G, kLimitD);
  const double u = fmin(fmax(U, -kLimitD), kLimitD);
  const double s = 1.0 / (1.0 + exp(-kAlphaD * g));
  return (u + 1.0) * (g * s);
}
__device__ inline void glu_backward_d(double G, double U, double dh, double &dG, double &dU) {
  const double L = kLimitD, A = kAlphaD;
  const double g = fmin(G, L), u = fmin(fmax(U, -L), L);
  const double s = 1.0 / (1.0 + exp(-A * g));
  dU = (U > L || U < -L) ? 0.0 : dh * (g * s);
  dG = (G > L) ? 0.0 : dh * (u + 1.0) * (s + g * s * (1.0 - s) * A);
}

enum { EPI_STORE = 0, EPI_GLU = 1 };

struct RowsArgs {
  const double *A;     // [rows, lda]; with a_rows: source row of sorted row p = a_rows[p] / a_div
  const double *B;     // [E][Kd][Nd], or with BNK [E][Nd][Kd]
  const double *bias;  // [E, Nd] or null
  double *C;           // EPI_STORE [rows, Nd]; EPI_GLU act [rows, Nd / 2]
  double *C2;          // EPI_GLU: optional pre-activations [rows, Nd]
  const int *a_rows;
  const int *sched;
  int a_div, Kd, Nd, lda, N, E;
};

// C[p, :] = A[row(p), :] . B[e] (+ bias[e]) for the rows of the schedule's row tiles; a workgroup takes 64 rows of one
// row tile (blockIdx.y = 4 * row tile + quarter) and 64 columns.
template <int EPI, bool GATHER, bool BNK>
__global__ __launch_bounds__(kThreads) void rows_gemm_kernel(const RowsArgs a) {
  __shared__ double sa[kTile][kStep + 1], sb[kStep][kTile + 1];
  const ScheduleView sv = schedule_view(a.sched, a.N, a.E);
  const int t = blockIdx.y >> 2, quarter = blockIdx.y & 3;
  if (t >= sv.hdr[0]) return;
  const int expert = sv.row_tiles[8 * t], row0 = sv.row_tiles[8 * t + 1] + quarter * kTile;
  const int rows = sv.row_tiles[8 * t + 2] - quarter * kTile;
  if (rows <= 0) return;
  const int n0 = blockIdx.x * kTile;
  const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
  const double *Bp = a.B + (long long)expert * a.Kd * a.Nd;
  double acc[4][4] = {};
  for (int k0 = 0; k0 < a.Kd; k0 += kStep) {
    for (int i = tid; i < kTile * kStep; i += kThreads) {
      const int r = i / kStep, k = i % kStep;
      double v = 0.0;
      if (r < rows && k0 + k < a.Kd) {
        long long src = row0 + r;
        if (GATHER) src = a.a_rows[row0 + r] / a.a_div;
        v = a.A[src * a.lda + k0 + k];
      }
      sa[r][k] = v;
    }
    for (int i = tid; i < kTile * kStep; i += kThreads) {
      int k, n;
      if (BNK) { n = i / kStep; k = i % kStep; } else { k = i / kTile; n = i % kTile; }
      double v = 0.0;
      if (k0 + k < a.Kd && n0 + n < a.Nd)
        v = BNK ? Bp[(long long)(n0 + n) * a.Kd + k0 + k] : Bp[(long long)(k0 + k) * a.Nd + n0 + n];
      sb[k][n] = v;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < kStep; ++k) {
      double av[4], bv[4];
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
    double v[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      v[j] = acc[i][j] + ((a.bias != nullptr && n < a.Nd) ? a.bias[(long long)expert * a.Nd + n] : 0.0);
    }
    if (EPI == EPI_STORE) {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (n0 + tx * 4 + j < a.Nd) a.C[p * a.Nd + n0 + tx * 4 + j] = v[j];
    } else {
#pragma unroll
      for (int j = 0; j < 4; j += 2) {  // (Nd is even: a (gate, up) pair is valid or invalid as a whole)
        const int n = n0 + tx * 4 + j;
        if (n < a.Nd) {
          a.C[p * (a.Nd / 2) + n / 2] = glu_forward_d(v[j], v[j + 1]);
          if (a.C2 != nullptr) { a.C2[p * a.Nd + n] = v[j]; a.C2[p * a.Nd + n + 1] = v[j + 1]; }
        }
      }
    }
  }
}

// dW[e] = L_e^T . R_e over the expert's kept rows: L [rows, Md] (with l_rows: gathered), R [rows, Nd]
__global__ __launch_bounds__(kThreads) void wgrad_kernel(const double *L, const int *l_rows, int l_div, const double *R,
                                                         double *dW, const int *counts, const int *offsets, int capacity,
                                                         int Md, int Nd) {
  __shared__ double sl[kStep][kTile + 1], sr[kStep][kTile + 1];
  const int expert = blockIdx.z, m0 = blockIdx.y * kTile, n0 = blockIdx.x * kTile;
  const int rows = max(min(counts[expert], capacity), 0);
  const long long first = offsets[expert];
  const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
  double acc[4][4] = {};
  for (int k0 = 0; k0 < rows; k0 += kStep) {
    for (int i = tid; i < kStep * kTile; i += kThreads) {
      const int k = i / kTile, c = i % kTile;
      double lv = 0.0, rv = 0.0;
      if (k0 + k < rows) {
        long long src = first + k0 + k;
        if (m0 + c < Md) lv = L[(l_rows != nullptr ? (long long)(l_rows[src] / l_div) : src) * Md + m0 + c];
        if (n0 + c < Nd) rv = R[src * Nd + n0 + c];
      }
      sl[k][c] = lv;
      sr[k][c] = rv;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < kStep; ++k) {
      double av[4], bv[4];
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
      if (m < Md && n < Nd) dW[((long long)expert * Md + m) * Nd + n] = acc[i][j];
    }
}

__device__ inline long long slot_expert(const void *idx, int i64, long long slot) {
  return i64 ? ((const long long *)idx)[slot] : (long long)((const int *)idx)[slot];
}
// the routing weight of flat slot t*K+k; rw == nullptr means 1
__device__ inline double slot_weight_d(const double *rw, const void *idx, int i64, int t, int k, int K, int E, int rw_cols) {
  if (rw == nullptr) return 1.0;
  if (rw_cols == K && rw_cols != E) return rw[(long long)t * K + k];
  const long long e = slot_expert(idx, i64, (long long)t * K + k);
  if (e < 0 || e >= E) return 0.0;
  return rw[(long long)t * E + e];
}

// out[t, :] = sum_k w(t, k) * y[inv_pos[t*K+k], :] in slot order (csrc/scatter.cu:66-108 without atomics)
__global__ void combine_kernel(const double *y, const int *inv_pos, const void *idx, int i64, const double *rw, int rw_cols,
                               double *out, int T, int K, int E, int H) {
  const int t = blockIdx.x;
  for (int c = threadIdx.x; c < H; c += blockDim.x) {
    double acc = 0.0;
    for (int k = 0; k < K; ++k) {
      const int p = inv_pos[(long long)t * K + k];
      if (p >= 0) acc += slot_weight_d(rw, idx, i64, t, k, K, E, rw_cols) * y[(long long)p * H + c];
    }
    out[(long long)t * H + c] = acc;
  }
}

// per kept sorted row p (one workgroup): g_y[p, :] = grad_out[tok, :] * w, w_sorted[p] = w
__global__ void scale_rows_kernel(const double *gy, const int *sorted_idx, const int *inv_pos, const void *idx, int i64,
                                  const double *rw, int rw_cols, double *g_y, double *w_sorted, int N, int K, int E, int H) {
  const int p = blockIdx.x;
  const int slot = sorted_idx[p];
  if (slot < 0 || slot >= N || inv_pos[slot] != p) return;  // a dropped slot: nobody reads its row
  const int t = slot / K, k = slot % K;
  const double w = slot_weight_d(rw, idx, i64, t, k, K, E, rw_cols);
  if (threadIdx.x == 0) w_sorted[p] = w;
  for (int c = threadIdx.x; c < H; c += blockDim.x) g_y[(long long)p * H + c] = gy[(long long)t * H + c] * w;
}

// out[e, c] = sum over the expert's kept rows of src[p, c], in row order
__global__ void colsum_kernel(const double *src, const int *counts, const int *offsets, int capacity, double *out, int cols) {
  const int e = blockIdx.y, c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= cols) return;
  const int rows = max(min(counts[e], capacity), 0);
  const long long first = offsets[e];
  double acc = 0.0;
  for (int r = 0; r < rows; ++r) acc += src[(first + r) * cols + c];
  out[(long long)e * cols + c] = acc;
}

// per kept sorted row p (one workgroup): row_dot[p] = <d_act[p], act[p]> + <grad_out[tok], b_down[e]> (the routing
// gradient of the slot, csrc/experts_backward.cu:83-88), then d_pre[p] = SwiGLU backward of d_act[p] * w
// (csrc/experts_backward.cu:285-305)
__global__ __launch_bounds__(kThreads) void glu_backward_kernel(const double *d_act, const double *act, const double *pre,
                                                                const double *gy, const double *b_down,
                                                                const int *sorted_idx, const int *sorted_expert,
                                                                const int *inv_pos, const double *w_sorted, double *d_pre,
                                                                double *row_dot, int N, int K, int H, int I) {
  __shared__ double part[kThreads];
  const int p = blockIdx.x;
  const int slot = sorted_idx[p];
  if (slot < 0 || slot >= N || inv_pos[slot] != p) return;
  const int t = slot / K, e = sorted_expert[p];
  const double w = w_sorted[p];
  double dot = 0.0;
  for (int c = threadIdx.x; c < I; c += blockDim.x) {
    const double da = d_act[(long long)p * I + c];
    dot += da * act[(long long)p * I + c];
    double dG, dU;
    glu_backward_d(pre[(long long)p * 2 * I + 2 * c], pre[(long long)p * 2 * I + 2 * c + 1], da * w, dG, dU);
    d_pre[(long long)p * 2 * I + 2 * c] = dG;
    d_pre[(long long)p * 2 * I + 2 * c + 1] = dU;
  }
  for (int c = threadIdx.x; c < H; c += blockDim.x) dot += gy[(long long)t * H + c] * b_down[(long long)e * H + c];
  part[threadIdx.x] = dot;
  __syncthreads();
  for (int s = kThreads / 2; s > 0; s >>= 1) {  // a fixed tree: the same sum on every run
    if ((int)threadIdx.x < s) part[threadIdx.x] += part[threadIdx.x + s];
    __syncthreads();
  }
  if (threadIdx.x == 0) row_dot[p] = part[0];
}

// d_routing[t, :]: zero, then the dots of the token's kept slots at [t, expert] (dense) or [t, k]; a token that names an
// expert twice gets the sum (one thread per token: a fixed order)
__global__ void routing_grad_kernel(const double *row_dot, const int *inv_pos, const void *idx, int i64, int rw_cols,
                                    double *d_rw, int T, int K, int E) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= T) return;
  for (int c = 0; c < rw_cols; ++c) d_rw[(long long)t * rw_cols + c] = 0.0;
  const bool per_slot = rw_cols == K && rw_cols != E;
  for (int k = 0; k < K; ++k) {
    const int p = inv_pos[(long long)t * K + k];
    if (p < 0) continue;
    const long long e = slot_expert(idx, i64, (long long)t * K + k);
    if (per_slot) d_rw[(long long)t * K + k] += row_dot[p];
    else if (e >= 0 && e < E) d_rw[(long long)t * E + e] += row_dot[p];
  }
}

__global__ void fill_kernel(double *p, long long n) {
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (; i < n; i += stride) p[i] = 0.0;
}

template <int EPI, bool GATHER, bool BNK> static int launch_rows(const RowsArgs &a, hipStream_t stream) {
  const int tiles = sched_max_row_tiles(a.N, a.E);
  hipLaunchKernelGGL((rows_gemm_kernel<EPI, GATHER, BNK>), dim3(ceil_div(a.Nd, kTile), 4 * tiles), dim3(kThreads), 0, stream, a);
  return check_launch("f64 rows_gemm_kernel");
}

}  // namespace f64

#define F64_TRY(expr)          \
  do {                         \
    int rc_ = (expr);          \
    if (rc_ != 0) return rc_;  \
  } while (0)

// act = glu(x[tok] . Wgu[e] + bgu[e]) (and the pre-activations), y = act . Wd[e] + bd[e], rows in sorted order
static int f64_gate_up_down(const double *x, const int *sorted_idx, const double *wgu, const double *bgu, const double *wd,
                            const double *bd, double *act, double *pre, double *y, const void *sched, int N, int K, int E,
                            int H, int I, hipStream_t stream) {
  f64::RowsArgs g = {};
  g.A = x; g.B = wgu; g.bias = bgu; g.C = act; g.C2 = pre; g.a_rows = sorted_idx; g.a_div = K; g.sched = (const int *)sched;
  g.Kd = H; g.Nd = 2 * I; g.lda = H; g.N = N; g.E = E;
  F64_TRY((f64::launch_rows<f64::EPI_GLU, true, false>(g, stream)));
  if (y != nullptr) {
    f64::RowsArgs d = {};
    d.A = act; d.B = wd; d.bias = bd; d.C = y; d.a_div = 1; d.sched = (const int *)sched;
    d.Kd = I; d.Nd = H; d.lda = I; d.N = N; d.E = E;
    F64_TRY((f64::launch_rows<f64::EPI_STORE, false, false>(d, stream)));
  }
  return 0;
}

// The whole forward in double on the caller's lists (sorted_idx, inv_pos, schedule built with no streaming limit).
int f64_forward(const void *x, const void *idx, int idx_i64, const void *rw, int rw_cols, const void *wgu, const void *bgu,
                const void *wd, const void *bd, void *out, const int *sorted_idx, const int *inv_pos, const void *sched,
                void *act, void *y_perm, int T, int K, int E, int H, int I, hipStream_t stream) {
  const int N = T * K;
  F64_TRY(f64_gate_up_down((const double *)x, sorted_idx, (const double *)wgu, (const double *)bgu, (const double *)wd,
                           (const double *)bd, (double *)act, nullptr, (double *)y_perm, sched, N, K, E, H, I, stream));
  hipLaunchKernelGGL(f64::combine_kernel, dim3(T), dim3(256), 0, stream, (const double *)y_perm, inv_pos, idx, idx_i64,
                     (const double *)rw, rw_cols, (double *)out, T, K, E, H);
  return check_launch("f64 combine_kernel");
}

// The whole backward in double.  Buffers: act [N, I], pre [N, 2I], g_y [N, H], d_act [N, I], d_pre [N, 2I],
// d_x_perm [N, H], w_sorted [N], row_dot [N].
int f64_backward(const void *gy_, const void *x_, const void *idx, int idx_i64, const void *rw_, int rw_cols,
                 const void *wgu_, const void *bgu_, const void *wd_, const void *bd_, void *d_x, void *d_rw, void *d_wgu,
                 void *d_bgu, void *d_wd, void *d_bd, const int *sorted_expert, const int *sorted_idx, const int *inv_pos,
                 const int *counts, const int *offsets, const void *sched, void *act_, void *pre_, void *g_y_,
                 void *d_act_, void *d_pre_, void *d_x_perm_, void *w_sorted_, void *row_dot_, int T, int K, int E, int H,
                 int I, int capacity, hipStream_t stream) {
  const int N = T * K;
  const double *gy = (const double *)gy_, *x = (const double *)x_, *rw = (const double *)rw_;
  const double *wgu = (const double *)wgu_, *bgu = (const double *)bgu_, *wd = (const double *)wd_, *bd = (const double *)bd_;
  double *act = (double *)act_, *pre = (double *)pre_, *g_y = (double *)g_y_, *d_act = (double *)d_act_;
  double *d_pre = (double *)d_pre_, *d_x_perm = (double *)d_x_perm_, *w_sorted = (double *)w_sorted_, *row_dot = (double *)row_dot_;
  // forward recompute of the first product: activations and pre-activations
  F64_TRY(f64_gate_up_down(x, sorted_idx, wgu, bgu, wd, bd, act, pre, nullptr, sched, N, K, E, H, I, stream));
  // weighted rows of grad_out; bias and weight gradient of the down projection
  hipLaunchKernelGGL(f64::scale_rows_kernel, dim3(N), dim3(256), 0, stream, gy, sorted_idx, inv_pos, idx, idx_i64, rw, rw_cols,
                     g_y, w_sorted, N, K, E, H);
  F64_TRY(check_launch("f64 scale_rows_kernel"));
  hipLaunchKernelGGL(f64::colsum_kernel, dim3(ceil_div(H, 256), E), dim3(256), 0, stream, g_y, counts, offsets, capacity,
                     (double *)d_bd, H);
  F64_TRY(check_launch("f64 colsum_kernel"));
  hipLaunchKernelGGL(f64::wgrad_kernel, dim3(ceil_div(H, f64::kTile), ceil_div(I, f64::kTile), E), dim3(f64::kThreads), 0, stream,
                     act, (const int *)nullptr, 1, g_y, (double *)d_wd, counts, offsets, capacity, I, H);
  F64_TRY(check_launch("f64 wgrad_kernel"));
  // input gradient of the down projection for the un-weighted rows of grad_out, gathered by token
  {
    f64::RowsArgs a = {};
    a.A = gy; a.B = wd; a.C = d_act; a.a_rows = sorted_idx; a.a_div = K; a.sched = (const int *)sched;
    a.Kd = H; a.Nd = I; a.lda = H; a.N = N; a.E = E;   // W_down[e] is [I, H] = [n][k]
    F64_TRY((f64::launch_rows<f64::EPI_STORE, true, true>(a, stream)));
  }
  hipLaunchKernelGGL(f64::glu_backward_kernel, dim3(N), dim3(f64::kThreads), 0, stream, d_act, act, pre, gy, bd, sorted_idx,
                     sorted_expert, inv_pos, w_sorted, d_pre, row_dot, N, K, H, I);
  F64_TRY(check_launch("f64 glu_backward_kernel"));
  hipLaunchKernelGGL(f64::routing_grad_kernel, dim3(ceil_div(T, 256)), dim3(256), 0, stream, row_dot, inv_pos, idx, idx_i64,
                     rw_cols, (double *)d_rw, T, K, E);
  F64_TRY(check_launch("f64 routing_grad_kernel"));
  // gate_up projection
  hipLaunchKernelGGL(f64::colsum_kernel, dim3(ceil_div(2 * I, 256), E), dim3(256), 0, stream, d_pre, counts, offsets, capacity,
                     (double *)d_bgu, 2 * I);
  F64_TRY(check_launch("f64 colsum_kernel"));
  {
    f64::RowsArgs a = {};
    a.A = d_pre; a.B = wgu; a.C = d_x_perm; a.a_div = 1; a.sched = (const int *)sched;
    a.Kd = 2 * I; a.Nd = H; a.lda = 2 * I; a.N = N; a.E = E;   // W_gate_up[e] is [H, 2I] = [n][k]
    F64_TRY((f64::launch_rows<f64::EPI_STORE, false, true>(a, stream)));
  }
  hipLaunchKernelGGL(f64::wgrad_kernel, dim3(ceil_div(2 * I, f64::kTile), ceil_div(H, f64::kTile), E), dim3(f64::kThreads), 0,
                     stream, x, sorted_idx, K, d_pre, (double *)d_wgu, counts, offsets, capacity, H, 2 * I);
  F64_TRY(check_launch("f64 wgrad_kernel"));
  hipLaunchKernelGGL(f64::combine_kernel, dim3(T), dim3(256), 0, stream, d_x_perm, inv_pos, idx, idx_i64, (const double *)nullptr,
                     K, (double *)d_x, T, K, E, H);
  return check_launch("f64 combine_kernel");
}

int f64_fill_zero(void *p, long long n, hipStream_t stream) {
  if (n <= 0) return 0;
  long long blocks = (n + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(f64::fill_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, (double *)p, n);
  return check_launch("f64 fill_kernel");
}

}  // namespace yamoe
