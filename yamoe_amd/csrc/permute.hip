// Row movers of the expert layer: the token permute (expert-contiguous gather of rows) and the
// routing-weighted combine that brings expert outputs back to token order.
//
// Both are pure HBM streaming: one wavefront moves one row in 16-byte chunks per lane, so every
// request is a full coalesced segment.  The combine replaces the reference's atomic scatter-add
// (csrc/scatter.cu:66-108): each output row is owned by one wave, which sums the K expert rows of
// its token through the inverse permutation in fp32 in slot order and rounds once.
#include "common.h"

namespace yamoe {

#ifndef YAMOE_COMBINE_SPLIT_T
#define YAMOE_COMBINE_SPLIT_T 1024
#endif
constexpr int kRowThreads = 256;
constexpr int kRowWaves = kRowThreads / kWave;

// x_perm[p,:] = x[sorted_idx[p] / K,:]   (csrc/gather.cu:6-66 without the padding rows)
template <typename T>
__global__ __launch_bounds__(kRowThreads) void permute_kernel(const T *__restrict__ x,
                                                              const int *__restrict__ sorted_idx,
                                                              T *__restrict__ x_perm, int N, int K,
                                                              int H) {
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = blockIdx.x * kRowWaves + threadIdx.x / kWave;
  const int n_waves = gridDim.x * kRowWaves;
  constexpr int V = ElemTraits<T>::kVec;
  const bool vec_ok = (H % V) == 0;
  for (int p = wave; p < N; p += n_waves) {
    int tok = sorted_idx[p] / K;
    const T *src = x + (size_t)tok * H;
    T *dst = x_perm + (size_t)p * H;
    if (vec_ok) {
      const u32x4 *s4 = (const u32x4 *)src;
      u32x4 *d4 = (u32x4 *)dst;
      for (int c = lane; c < H / V; c += kWave) d4[c] = s4[c];
    } else {
      for (int c = lane; c < H; c += kWave) dst[c] = src[c];
    }
  }
}

template <typename T, bool I64>
__device__ inline float slot_weight(const T *rw, const void *idx, int t, int k, int K, int E,
                                    int rw_cols) {
  if (rw == nullptr) return 1.0f;
  if (rw_cols == K && rw_cols != E) return ElemTraits<T>::to_f32(rw[(size_t)t * K + k]);
  long long e = I64 ? ((const long long *)idx)[(size_t)t * K + k]
                    : (long long)((const int *)idx)[(size_t)t * K + k];
  if (e < 0 || e >= E) return 0.0f;
  return ElemTraits<T>::to_f32(rw[(size_t)t * E + e]);
}

// out[t,:] = sum_k w(t,k) * y_perm[inv_pos[t*K+k],:]
// `split` waves per token (1, or the 4 of a workgroup when there are few tokens: a lone wave goes through a 2880-wide
// row in six dependent rounds of loads).  The K (position, weight) pairs of the token are fetched once (up to
// kMaxSlots of them sit in registers), then every lane streams its 16-byte chunks of the K rows.
constexpr int kMaxSlots = 8;

template <typename T, bool I64>
__global__ __launch_bounds__(kRowThreads) void combine_kernel(
    const T *__restrict__ y_perm, const int *__restrict__ inv_pos, const void *__restrict__ idx,
    const T *__restrict__ rw, int rw_cols, T *__restrict__ out, int Tn, int K, int E, int H, int split) {
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = blockIdx.x * kRowWaves + threadIdx.x / kWave;
  const int n_waves = gridDim.x * kRowWaves;
  constexpr int V = ElemTraits<T>::kVec;
  const bool vec_ok = (H % V) == 0;
  const int part = wave % split, stride = kWave * split;
  for (int t = wave / split; t < Tn; t += n_waves / split) {
    T *dst = out + (size_t)t * H;
    if (vec_ok && K <= kMaxSlots) {
      int pos[kMaxSlots];
      float w[kMaxSlots];
#pragma unroll
      for (int k = 0; k < kMaxSlots; ++k) {
        pos[k] = -1;
        w[k] = 0.0f;
        if (k < K) {
          pos[k] = inv_pos[(size_t)t * K + k];
          if (pos[k] >= 0) w[k] = slot_weight<T, I64>(rw, idx, t, k, K, E, rw_cols);
        }
      }
      for (int c = part * kWave + lane; c < H / V; c += stride) {
        float acc[V];
#pragma unroll
        for (int j = 0; j < V; ++j) acc[j] = 0.0f;
#pragma unroll
        for (int k = 0; k < kMaxSlots; ++k) {
          if (pos[k] < 0) continue;
          u32x4 raw = ((const u32x4 *)(y_perm + (size_t)pos[k] * H))[c];
          const T *v = (const T *)&raw;
#pragma unroll
          for (int j = 0; j < V; ++j) acc[j] += w[k] * ElemTraits<T>::to_f32(v[j]);
        }
        u32x4 o;
        T *ov = (T *)&o;
#pragma unroll
        for (int j = 0; j < V; ++j) ov[j] = ElemTraits<T>::from_f32(acc[j]);
        ((u32x4 *)dst)[c] = o;
      }
    } else {
      for (int c = part * kWave + lane; c < H; c += stride) {
        float acc = 0.0f;
        for (int k = 0; k < K; ++k) {
          int pos = inv_pos[(size_t)t * K + k];
          if (pos < 0) continue;
          float w = slot_weight<T, I64>(rw, idx, t, k, K, E, rw_cols);
          acc += w * ElemTraits<T>::to_f32(y_perm[(size_t)pos * H + c]);
        }
        dst[c] = ElemTraits<T>::from_f32(acc);
      }
    }
  }
}

// Backward of the combine (csrc/experts_backward.cu:37-89) in sorted-row order, for kept rows p = (tok, slot):
//   g_y_perm[p,:] = grad_out[tok,:] * w(tok,slot)
//   w_sorted[p]   = w(tok,slot)
//   dot_bias[p]   = <grad_out[tok,:], down_bias[expert,:]>
// The routing gradient is <grad_out[tok], y[p]> with y[p] = act[p] . W_down + down_bias (the expert's output row
// before weighting).  Instead of recomputing y, the backward uses <grad_out[tok] . W_down^T, act[p]> + dot_bias[p]:
// the first factor is the input gradient of the down projection of the un-weighted row, which the backward needs
// anyway; glu_backward_rows_kernel finishes the sum.  Dropped slots get no row and a zero gradient.
template <typename T, bool I64>
__global__ __launch_bounds__(kRowThreads) void combine_backward_kernel(
    const T *__restrict__ grad_out, const T *__restrict__ down_bias, const int *__restrict__ sorted_idx,
    const int *__restrict__ inv_pos, const void *__restrict__ idx, const T *__restrict__ rw, int rw_cols,
    T *__restrict__ g_y_perm, float *__restrict__ w_sorted, float *__restrict__ dot_bias, int N, int K, int E, int H) {
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = blockIdx.x * kRowWaves + threadIdx.x / kWave;
  const int n_waves = gridDim.x * kRowWaves;
  for (int p = wave; p < N; p += n_waves) {
    int flat = sorted_idx[p];
    if (inv_pos[flat] != p) continue;  // dropped or invalid expert id
    int t = flat / K, k = flat - t * K;
    float w = slot_weight<T, I64>(rw, idx, t, k, K, E, rw_cols);
    long long e = I64 ? ((const long long *)idx)[flat] : (long long)((const int *)idx)[flat];
    const T *g = grad_out + (size_t)t * H;
    const T *bd = down_bias + (size_t)e * H;
    T *o = g_y_perm + (size_t)p * H;
    float dot = 0.0f;
    constexpr int V = ElemTraits<T>::kVec;
    if (H % V == 0) {  // 16 bytes per lane (rows are 16-byte aligned then), four chunks of both rows in flight
      const int n_chunks = H / V;
      for (int c0 = lane; c0 < n_chunks; c0 += 4 * kWave) {
        u32x4 graw[4], braw[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int c = min(c0 + u * kWave, n_chunks - 1);
          graw[u] = ((const u32x4 *)g)[c];
          braw[u] = ((const u32x4 *)bd)[c];
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int c = c0 + u * kWave;
          if (c < n_chunks) {
            const T *gv = (const T *)&graw[u], *bv = (const T *)&braw[u];
            u32x4 oraw;
            T *ov = (T *)&oraw;
#pragma unroll
            for (int j = 0; j < V; ++j) {
              float x = ElemTraits<T>::to_f32(gv[j]);
              dot += x * ElemTraits<T>::to_f32(bv[j]);
              ov[j] = ElemTraits<T>::from_f32(x * w);
            }
            ((u32x4 *)o)[c] = oraw;
          }
        }
      }
    } else {
      for (int c = lane; c < H; c += kWave) {
        float gv = ElemTraits<T>::to_f32(g[c]);
        dot += gv * ElemTraits<T>::to_f32(bd[c]);
        o[c] = ElemTraits<T>::from_f32(gv * w);
      }
    }
    for (int d = kWave / 2; d > 0; d >>= 1) dot += __shfl_xor(dot, d);
    if (lane == 0) {
      w_sorted[p] = w;
      dot_bias[p] = dot;
    }
  }
}

// GLU backward on kept rows (csrc/experts_backward.cu:285-305) plus the row's share of the routing gradient:
//   d_act[p,:] is the input gradient of the down projection for the UN-weighted output gradient of row p,
//   d_pre[p,:] = w_sorted[p] * glu'(pre[p,:]) applied to d_act[p,:]      (interleaved gate/up columns)
//   row_dot[p] = <d_act[p,:], glu(pre[p,:])> + row_dot[p]                (row_dot comes in holding dot_bias[p])
// With dot_part the first term is the sum of the n_part partial sums per row that the input-gradient GEMM took
// from its fp32 accumulators (d_act itself is rounded to the activation dtype); without it (fp32 data) the dot is
// formed here from d_act and the recomputed activations.  One wave per row.
template <typename T>
__global__ __launch_bounds__(kRowThreads) void glu_backward_rows_kernel(
    const T *__restrict__ d_act, const T *__restrict__ pre, const float *__restrict__ w_sorted,
    const float *__restrict__ dot_part, int n_part, const int *__restrict__ sorted_idx,
    const int *__restrict__ inv_pos, T *__restrict__ d_pre, float *__restrict__ row_dot, int N, int I) {
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = blockIdx.x * kRowWaves + threadIdx.x / kWave;
  const int n_waves = gridDim.x * kRowWaves;
  for (int p = wave; p < N; p += n_waves) {
    int flat = sorted_idx[p];
    if (inv_pos[flat] != p) continue;
    const float w = w_sorted[p];
    const T *da = d_act + (size_t)p * I;
    const T *pr = pre + (size_t)p * 2 * I;
    T *dp = d_pre + (size_t)p * 2 * I;
    float dot = 0.0f;
    constexpr int V = ElemTraits<T>::kVec;  // pre-activations per 16 bytes = V / 2 (gate, up) pairs
    if (I % (V / 2) == 0) {
      for (int c = lane; c < I / (V / 2); c += kWave) {
        u32x4 praw = ((const u32x4 *)pr)[c];
        u32x2 draw = ((const u32x2 *)da)[c];
        const T *pv = (const T *)&praw;
        const T *dv = (const T *)&draw;
        u32x4 oraw;
        T *ov = (T *)&oraw;
#pragma unroll
        for (int j = 0; j < V / 2; ++j) {
          float G = ElemTraits<T>::to_f32(pv[2 * j]), U = ElemTraits<T>::to_f32(pv[2 * j + 1]);
          float dh = ElemTraits<T>::to_f32(dv[j]);
          float dG, dU;
          glu_backward(G, U, dh * w, dG, dU);
          if (dot_part == nullptr) dot += dh * glu_forward(G, U);
          ov[2 * j] = ElemTraits<T>::from_f32(dG);
          ov[2 * j + 1] = ElemTraits<T>::from_f32(dU);
        }
        ((u32x4 *)dp)[c] = oraw;
      }
    } else {
      for (int c = lane; c < I; c += kWave) {
        float G = ElemTraits<T>::to_f32(pr[2 * c]), U = ElemTraits<T>::to_f32(pr[2 * c + 1]);
        float dh = ElemTraits<T>::to_f32(da[c]);
        float dG, dU;
        glu_backward(G, U, dh * w, dG, dU);
        if (dot_part == nullptr) dot += dh * glu_forward(G, U);
        dp[2 * c] = ElemTraits<T>::from_f32(dG);
        dp[2 * c + 1] = ElemTraits<T>::from_f32(dU);
      }
    }
    if (dot_part != nullptr)
      for (int c = lane; c < n_part; c += kWave) dot += dot_part[(size_t)p * n_part + c];
    for (int d = kWave / 2; d > 0; d >>= 1) dot += __shfl_xor(dot, d);
    if (lane == 0) row_dot[p] += dot;
  }
}

// d_routing from the per-row values (csrc/experts_backward.cu:83-88, 261-271, placed once): one thread per flat slot
// (token t, slot k).  Per-slot weights [T,K]: d_routing[t,k] = row_dot[row of the slot].  Dense weights [T,E]: the
// first slot of the token that names expert e writes the sum over all of the token's slots that name e (a token
// that lists an expert twice reads one weight twice), in slot order; everything else keeps the zero fill.
template <typename T, bool I64>
__global__ __launch_bounds__(kRowThreads) void routing_grad_kernel(const float *__restrict__ row_dot,
                                                                   const int *__restrict__ inv_pos,
                                                                   const void *__restrict__ idx, int rw_cols,
                                                                   T *__restrict__ d_routing, int N, int K, int E) {
  const int flat = blockIdx.x * kRowThreads + threadIdx.x;
  if (flat >= N) return;
  const int p = inv_pos[flat];
  if (rw_cols == K && rw_cols != E) {
    if (p >= 0) d_routing[flat] = ElemTraits<T>::from_f32(row_dot[p]);
    return;
  }
  auto expert_of = [&](int f) {
    return I64 ? ((const long long *)idx)[f] : (long long)((const int *)idx)[f];
  };
  const int t = flat / K, k = flat - t * K;
  const long long e = expert_of(flat);
  if (e < 0 || e >= E) return;
  float sum = 0.0f;
  bool any = false;
  for (int k2 = 0; k2 < K; ++k2) {
    if (expert_of(t * K + k2) != e) continue;
    if (k2 < k) return;  // an earlier slot of the token owns this entry
    const int p2 = inv_pos[t * K + k2];
    if (p2 >= 0) { sum += row_dot[p2]; any = true; }
  }
  if (any) d_routing[(size_t)t * E + e] = ElemTraits<T>::from_f32(sum);
}

// Column sums over each expert's kept rows: out[e, c] = sum_{rows p of e} src[p, c]
// (d_down_proj_bias and d_gate_up_proj_bias, csrc/experts_backward.cu:277, 308).
// grid (E, ceil(cols / (64 * V))), V = elements per 16 bytes: a workgroup owns one expert and 64 * V columns,
// its waves take every kRowWaves-th row with 16 bytes per lane (eight rows in flight per wave), and the
// per-wave partial sums meet in LDS.  The order of the additions is fixed, so the result is reproducible.
template <typename T>
__global__ __launch_bounds__(kRowThreads) void expert_colsum_kernel(const T *__restrict__ src,
                                                                    const int *__restrict__ counts,
                                                                    const int *__restrict__ offsets,
                                                                    int capacity, T *__restrict__ out,
                                                                    int cols) {
  constexpr int V = ElemTraits<T>::kVec;
  __shared__ float part[kRowWaves][kWave * V];
  const int e = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c0 = (blockIdx.y * kWave + lane) * V;
  const int first = offsets[e], kept = min(counts[e], capacity);
  float acc[V];
#pragma unroll
  for (int v = 0; v < V; ++v) acc[v] = 0.0f;
  if (c0 < cols) {
    const T *p = src + (size_t)first * cols + c0;
    auto add = [&](const u32x4 &raw) {
      const T *h = (const T *)&raw;
#pragma unroll
      for (int v = 0; v < V; ++v) acc[v] += ElemTraits<T>::to_f32(h[v]);
    };
    int r = wave;
    for (; r + 7 * kRowWaves < kept; r += 8 * kRowWaves) {
      u32x4 raw[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) raw[j] = *(const u32x4 *)(p + (size_t)(r + j * kRowWaves) * cols);
#pragma unroll
      for (int j = 0; j < 8; ++j) add(raw[j]);
    }
    for (; r < kept; r += kRowWaves) add(*(const u32x4 *)(p + (size_t)r * cols));
  }
#pragma unroll
  for (int v = 0; v < V; ++v) part[wave][lane * V + v] = acc[v];
  __syncthreads();
  for (int i = threadIdx.x; i < kWave * V; i += kRowThreads) {
    int c = blockIdx.y * kWave * V + i;
    if (c < cols) {
      float sum = 0.0f;
#pragma unroll
      for (int w = 0; w < kRowWaves; ++w) sum += part[w][i];
      out[(size_t)e * cols + c] = ElemTraits<T>::from_f32(sum);
    }
  }
}

// the same for a column count that is not a multiple of the 16-byte vector: a thread per column
template <typename T>
__global__ __launch_bounds__(kRowThreads) void expert_colsum_scalar_kernel(const T *__restrict__ src,
                                                                           const int *__restrict__ counts,
                                                                           const int *__restrict__ offsets,
                                                                           int capacity, T *__restrict__ out,
                                                                           int cols) {
  const int e = blockIdx.x;
  const int c = blockIdx.y * kRowThreads + threadIdx.x;
  if (c >= cols) return;
  int first = offsets[e], kept = min(counts[e], capacity);
  float acc = 0.0f;
  for (int r = 0; r < kept; ++r) acc += ElemTraits<T>::to_f32(src[(size_t)(first + r) * cols + c]);
  out[(size_t)e * cols + c] = ElemTraits<T>::from_f32(acc);
}

template <typename T>
int launch_permute(const void *x, const int *sorted_idx, void *x_perm, int N, int K, int H,
                   hipStream_t stream) {
  if (N == 0) return 0;
  int blocks = min(ceil_div(N, kRowWaves), 256 * 16);
  hipLaunchKernelGGL(permute_kernel<T>, dim3(blocks), dim3(kRowThreads), 0, stream, (const T *)x,
                     sorted_idx, (T *)x_perm, N, K, H);
  return check_launch("permute_kernel");
}

template <typename T>
int launch_combine(const void *y_perm, const int *inv_pos, const void *idx, int idx_i64,
                   const void *rw, int rw_cols, void *out, int Tn, int K, int E, int H,
                   hipStream_t stream) {
  if (Tn == 0) return 0;
  const int split = Tn <= YAMOE_COMBINE_SPLIT_T ? kRowWaves : 1;  // (the grid is a whole number of groups of `split` waves)
  int blocks = min(ceil_div(Tn * split, kRowWaves), 256 * 16);
  if (idx_i64)
    hipLaunchKernelGGL((combine_kernel<T, true>), dim3(blocks), dim3(kRowThreads), 0, stream,
                       (const T *)y_perm, inv_pos, idx, (const T *)rw, rw_cols, (T *)out, Tn, K, E, H, split);
  else
    hipLaunchKernelGGL((combine_kernel<T, false>), dim3(blocks), dim3(kRowThreads), 0, stream,
                       (const T *)y_perm, inv_pos, idx, (const T *)rw, rw_cols, (T *)out, Tn, K, E, H, split);
  return check_launch("combine_kernel");
}

template <typename T>
int launch_combine_backward(const void *grad_out, const void *down_bias, const int *sorted_idx, const int *inv_pos,
                            const void *idx, int idx_i64, const void *rw, int rw_cols, void *g_y_perm, float *w_sorted,
                            float *dot_bias, int N, int K, int E, int H, hipStream_t stream) {
  if (N == 0) return 0;
  int blocks = min(ceil_div(N, kRowWaves), 256 * 16);
  if (idx_i64)
    hipLaunchKernelGGL((combine_backward_kernel<T, true>), dim3(blocks), dim3(kRowThreads), 0, stream,
                       (const T *)grad_out, (const T *)down_bias, sorted_idx, inv_pos, idx, (const T *)rw, rw_cols,
                       (T *)g_y_perm, w_sorted, dot_bias, N, K, E, H);
  else
    hipLaunchKernelGGL((combine_backward_kernel<T, false>), dim3(blocks), dim3(kRowThreads), 0, stream,
                       (const T *)grad_out, (const T *)down_bias, sorted_idx, inv_pos, idx, (const T *)rw, rw_cols,
                       (T *)g_y_perm, w_sorted, dot_bias, N, K, E, H);
  return check_launch("combine_backward_kernel");
}

template <typename T>
int glu_backward_rows(const void *d_act, const void *pre, const float *w_sorted, const float *dot_part, int n_part,
                      const int *sorted_idx, const int *inv_pos, void *d_pre, float *row_dot, int N, int I,
                      hipStream_t stream) {
  if (N == 0) return 0;
  int blocks = min(ceil_div(N, kRowWaves), 256 * 16);
  hipLaunchKernelGGL(glu_backward_rows_kernel<T>, dim3(blocks), dim3(kRowThreads), 0, stream, (const T *)d_act,
                     (const T *)pre, w_sorted, dot_part, n_part, sorted_idx, inv_pos, (T *)d_pre, row_dot, N, I);
  return check_launch("glu_backward_rows_kernel");
}

template <typename T>
int launch_routing_grad(const float *row_dot, const int *inv_pos, const void *idx, int idx_i64, int rw_cols,
                        void *d_routing, int N, int K, int E, hipStream_t stream) {
  if (N == 0) return 0;
  int blocks = ceil_div(N, kRowThreads);
  if (idx_i64)
    hipLaunchKernelGGL((routing_grad_kernel<T, true>), dim3(blocks), dim3(kRowThreads), 0, stream, row_dot, inv_pos, idx,
                       rw_cols, (T *)d_routing, N, K, E);
  else
    hipLaunchKernelGGL((routing_grad_kernel<T, false>), dim3(blocks), dim3(kRowThreads), 0, stream, row_dot, inv_pos, idx,
                       rw_cols, (T *)d_routing, N, K, E);
  return check_launch("routing_grad_kernel");
}

template <typename T>
int launch_expert_colsum(const void *src, const int *counts, const int *offsets, int capacity,
                         void *out, int E, int cols, hipStream_t stream) {
  constexpr int V = ElemTraits<T>::kVec;
  if (cols % V == 0)
    hipLaunchKernelGGL(expert_colsum_kernel<T>, dim3(E, ceil_div(cols, kWave * V)), dim3(kRowThreads), 0, stream,
                       (const T *)src, counts, offsets, capacity, (T *)out, cols);
  else
    hipLaunchKernelGGL(expert_colsum_scalar_kernel<T>, dim3(E, ceil_div(cols, kRowThreads)), dim3(kRowThreads), 0,
                       stream, (const T *)src, counts, offsets, capacity, (T *)out, cols);
  return check_launch("expert_colsum_kernel");
}

#define YAMOE_INSTANTIATE_ROWS(T)                                                                       \
  template int launch_permute<T>(const void *, const int *, void *, int, int, int, hipStream_t);        \
  template int launch_combine<T>(const void *, const int *, const void *, int, const void *, int,       \
                                 void *, int, int, int, int, hipStream_t);                              \
  template int launch_combine_backward<T>(const void *, const void *, const int *, const int *, const void *,   \
                                          int, const void *, int, void *, float *, float *, int, int, int, int,  \
                                          hipStream_t);                                                          \
  template int glu_backward_rows<T>(const void *, const void *, const float *, const float *, int, const int *, \
                                    const int *, void *, float *, int, int, hipStream_t);                        \
  template int launch_routing_grad<T>(const float *, const int *, const void *, int, int, void *, int, int, int, \
                                      hipStream_t);                                                              \
  template int launch_expert_colsum<T>(const void *, const int *, const int *, int, void *, int, int,  \
                                       hipStream_t);
YAMOE_INSTANTIATE_ROWS(float)
YAMOE_INSTANTIATE_ROWS(bf16_t)
YAMOE_INSTANTIATE_ROWS(f16_t)

}  // namespace yamoe

using namespace yamoe;

#define YAMOE_DISPATCH(dtype, CALL)                                \
  switch (dtype) {                                                 \
    case YAMOE_F32: { typedef float T; return CALL; }              \
    case YAMOE_BF16: { typedef bf16_t T; return CALL; }            \
    case YAMOE_F16: { typedef f16_t T; return CALL; }              \
    default: set_error("unknown dtype %d", dtype); return YAMOE_E_DTYPE; \
  }

extern "C" int yamoe_permute(const void *x, const int32_t *sorted_idx, void *x_perm, int32_t N,
                             int32_t K, int32_t H, int32_t dtype, void *stream) {
  if (N < 0 || K <= 0 || H <= 0 || (N > 0 && (!x || !sorted_idx || !x_perm))) {
    set_error("yamoe_permute: bad argument");
    return YAMOE_E_ARG;
  }
  YAMOE_DISPATCH(dtype, launch_permute<T>(x, sorted_idx, x_perm, N, K, H, (hipStream_t)stream));
}

extern "C" int yamoe_combine(const void *y_perm, const int32_t *inv_pos, const void *router_indices,
                             int32_t idx_i64, const void *routing_weights, int32_t rw_cols, void *out,
                             int32_t T_, int32_t K, int32_t E, int32_t H, int32_t dtype, void *stream) {
  if (T_ < 0 || K <= 0 || H <= 0 || E <= 0 || (T_ > 0 && (!y_perm || !inv_pos || !out))) {
    set_error("yamoe_combine: bad argument");
    return YAMOE_E_ARG;
  }
  if (routing_weights && rw_cols != E && rw_cols != K) {
    set_error("yamoe_combine: routing_weights must have E or K columns (got %d)", rw_cols);
    return YAMOE_E_ARG;
  }
  if (routing_weights && rw_cols == E && !router_indices) {
    set_error("yamoe_combine: dense routing_weights need router_indices");
    return YAMOE_E_ARG;
  }
  YAMOE_DISPATCH(dtype, launch_combine<T>(y_perm, inv_pos, router_indices, idx_i64, routing_weights, rw_cols,
                                          out, T_, K, E, H, (hipStream_t)stream));
}
