// The step before the expert layer: router linear -> top-k -> softmax over the selected logits -> dense scores
// (torch-ext/yamoe/layers.py:128-152, torch-ext/yamoe/vendored/gpt_oss_mlp.py:128-142), in one kernel, and the
// gradient of that step.
//
// A workgroup takes 32 tokens.  logits[32, E] = x[32, H] * W[E, H]^T: both operands are k-contiguous in memory,
// which is exactly the register layout of the 32x32x16 MFMA operands (lane l holds 8 consecutive k of row l % 32,
// starting at 8 * (l / 32)), so fragments go from global memory straight into registers, no LDS.  (fp32: a lane's
// 16 bytes are 4 consecutive k starting at 4 * (l / 32), fed to four v_mfma_f32_32x32x2_f32, whose two lane halves are
// the two k of an instruction: any pairing of k values is fine as long as both operands use the same.)  The four waves
// split the contraction, their partial tiles meet in LDS, the bias is added and the logits are rounded to the
// activation dtype as the reference's linear does.  Then one thread per token picks the top-k (ties: lowest expert
// id first) and the softmax of the k picked values is computed in fp32, rounded once, and scattered into the dense
// [T, E] score row (zero elsewhere).
#include "common.h"

namespace yamoe {

constexpr int kRouterTokens = 32;
constexpr int kRouterThreads = 256;
constexpr int kRouterMaxE = 256;
constexpr int kRouterMaxK = 16;

template <typename T> struct RouterMma;
template <> struct RouterMma<bf16_t> {
  __device__ static inline void run(const u32x4 &a, const u32x4 &b, f32x16 &c) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
};
template <> struct RouterMma<f16_t> {
  __device__ static inline void run(const u32x4 &a, const u32x4 &b, f32x16 &c) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
};
template <> struct RouterMma<float> {
  __device__ static inline void run(const u32x4 &a, const u32x4 &b, f32x16 &c) {
    const f32x4 af = __builtin_bit_cast(f32x4, a), bf = __builtin_bit_cast(f32x4, b);
#pragma unroll
    for (int q = 0; q < 4; ++q) c = __builtin_amdgcn_mfma_f32_32x32x2f32(af[q], bf[q], c, 0, 0, 0);
  }
};

// NB = number of 32-expert column blocks (E <= 32 * NB)
template <typename T, int NB>
__global__ __launch_bounds__(kRouterThreads) void router_topk_kernel(const T *__restrict__ x, const T *__restrict__ w,
                                                                     const T *__restrict__ bias, int Tn, int H, int E, int K,
                                                                     long long *__restrict__ indices, T *__restrict__ scores,
                                                                     T *__restrict__ topk_weights, T *__restrict__ logits_out) {
  constexpr int kLd = 32 * NB + 1;  // padded row of the logits tile
  __shared__ float tile[kRouterTokens * kLd];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int rl = lane & 31, g = lane >> 5;
  const int t0 = blockIdx.x * kRouterTokens;

  for (int i = tid; i < kRouterTokens * kLd; i += kRouterThreads) tile[i] = 0.0f;
  __syncthreads();

  f32x16 acc[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[nb][v] = 0.0f;

  // rows past the end re-read the last valid one; their results are never used
  constexpr int V = 16 / (int)sizeof(T);  // elements of a lane's 16 bytes; a step of the contraction is 2 * V of them
  const T *xa = x + (long long)min(t0 + rl, Tn - 1) * H + g * V;
  const T *wb[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) wb[nb] = w + (long long)min(nb * 32 + rl, E - 1) * H + g * V;

  const int n_steps = H / (2 * V);
  for (int s = wave; s < n_steps; s += 4) {
    u32x4 fa = *(const u32x4 *)(xa + s * 2 * V);
    u32x4 fb[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) fb[nb] = *(const u32x4 *)(wb[nb] + s * 2 * V);
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) RouterMma<T>::run(fa, fb[nb], acc[nb]);
  }
  // acc[nb][v]: token 8 * (v / 4) + 4 * g + v % 4, expert nb * 32 + rl; the four waves add up in LDS, one after another
  for (int turn = 0; turn < 4; ++turn) {
    if (wave == turn) {
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int v = 0; v < 16; ++v) tile[(8 * (v >> 2) + 4 * g + (v & 3)) * kLd + nb * 32 + rl] += acc[nb][v];
    }
    __syncthreads();
  }
  // bias, rounding to the activation dtype (the value the reference's top-k sees)
  for (int i = tid; i < kRouterTokens * 32 * NB; i += kRouterThreads) {
    int r = i / (32 * NB), e = i - r * (32 * NB);
    if (e < E) {
      float v = tile[r * kLd + e] + (bias != nullptr ? ElemTraits<T>::to_f32(bias[e]) : 0.0f);
      T q = ElemTraits<T>::from_f32(v);
      tile[r * kLd + e] = ElemTraits<T>::to_f32(q);
      if (logits_out != nullptr && t0 + r < Tn) logits_out[(long long)(t0 + r) * E + e] = q;
    }
  }
  __syncthreads();
  // dense score rows start at zero
  for (int i = tid; i < kRouterTokens * E; i += kRouterThreads) {
    int r = i / E, e = i - r * E;
    if (t0 + r < Tn) scores[(long long)(t0 + r) * E + e] = ElemTraits<T>::from_f32(0.0f);
  }
  __syncthreads();
  if (tid < kRouterTokens && t0 + tid < Tn) {
    float *row = tile + tid * kLd;
    const long long t = t0 + tid;
    int pick[kRouterMaxK];
    float val[kRouterMaxK];
    for (int k = 0; k < K; ++k) {
      int best = -1;
      float bv = 0.0f;
      for (int e = 0; e < E; ++e) {
        float v = row[e];
        bool taken = false;
        for (int j = 0; j < k; ++j) taken |= pick[j] == e;
        if (!taken && (best < 0 || v > bv)) { best = e; bv = v; }
      }
      pick[k] = best;
      val[k] = bv;
    }
    float sum = 0.0f, p[kRouterMaxK];
    for (int k = 0; k < K; ++k) { p[k] = expf(val[k] - val[0]); sum += p[k]; }
    for (int k = 0; k < K; ++k) {
      T q = ElemTraits<T>::from_f32(p[k] / sum);
      indices[t * K + k] = pick[k];
      scores[t * E + pick[k]] = q;
      if (topk_weights != nullptr) topk_weights[t * K + k] = q;
    }
  }
}

template <typename T, int NB>
static int launch_router(const void *x, const void *w, const void *bias, int Tn, int H, int E, int K, long long *indices,
                         void *scores, void *topk_weights, void *logits, hipStream_t stream) {
  hipLaunchKernelGGL((router_topk_kernel<T, NB>), dim3(ceil_div(Tn, kRouterTokens)), dim3(kRouterThreads), 0, stream,
                     (const T *)x, (const T *)w, (const T *)bias, Tn, H, E, K, indices, (T *)scores, (T *)topk_weights,
                     (T *)logits);
  return check_launch("router_topk_kernel");
}

template <typename T>
static int router_dispatch(const void *x, const void *w, const void *bias, int Tn, int H, int E, int K, long long *indices,
                           void *scores, void *topk_weights, void *logits, hipStream_t stream) {
  int nb = ceil_div(E, 32);
  if (nb <= 1) return launch_router<T, 1>(x, w, bias, Tn, H, E, K, indices, scores, topk_weights, logits, stream);
  if (nb <= 2) return launch_router<T, 2>(x, w, bias, Tn, H, E, K, indices, scores, topk_weights, logits, stream);
  if (nb <= 4) return launch_router<T, 4>(x, w, bias, Tn, H, E, K, indices, scores, topk_weights, logits, stream);
  return launch_router<T, 8>(x, w, bias, Tn, H, E, K, indices, scores, topk_weights, logits, stream);
}

// ---- gradient of the step, first part: from the gradient of the dense scores to the gradient of the logits --------
// One thread per token.  With p_k the softmax weights of the token's K picks (the scores the forward stored) and
// g_k = d_scores[t, pick_k]:  d_logits[t, pick_k] = p_k * (g_k - sum_j p_j g_j), zero for every other expert: what
// autograd gives through scatter, softmax over the K picked logits and top-k (torch-ext/yamoe/layers.py:136-149).
template <typename T>
__global__ __launch_bounds__(256) void router_backward_logits_kernel(const T *__restrict__ d_scores,
                                                                     const long long *__restrict__ indices,
                                                                     const T *__restrict__ scores, int Tn, int E, int K,
                                                                     T *__restrict__ d_logits) {
  const long long t = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= Tn) return;
  T *row = d_logits + t * E;
  for (int e = 0; e < E; ++e) row[e] = ElemTraits<T>::from_f32(0.0f);
  float inner = 0.0f;
  for (int k = 0; k < K; ++k) {
    const long long e = indices[t * K + k];
    if (e < 0 || e >= E) continue;
    inner += ElemTraits<T>::to_f32(scores[t * E + e]) * ElemTraits<T>::to_f32(d_scores[t * E + e]);
  }
  for (int k = 0; k < K; ++k) {
    const long long e = indices[t * K + k];
    if (e < 0 || e >= E) continue;
    const float p = ElemTraits<T>::to_f32(scores[t * E + e]), g = ElemTraits<T>::to_f32(d_scores[t * E + e]);
    row[e] = ElemTraits<T>::from_f32(p * (g - inner));
  }
}

template <typename T>
int launch_router_backward_logits(const void *d_scores, const long long *indices, const void *scores, int Tn, int E, int K,
                                  void *d_logits, hipStream_t stream) {
  hipLaunchKernelGGL(router_backward_logits_kernel<T>, dim3(ceil_div(Tn, 256)), dim3(256), 0, stream, (const T *)d_scores,
                     indices, (const T *)scores, Tn, E, K, (T *)d_logits);
  return check_launch("router_backward_logits_kernel");
}
template int launch_router_backward_logits<float>(const void *, const long long *, const void *, int, int, int, void *, hipStream_t);
template int launch_router_backward_logits<bf16_t>(const void *, const long long *, const void *, int, int, int, void *, hipStream_t);
template int launch_router_backward_logits<f16_t>(const void *, const long long *, const void *, int, int, int, void *, hipStream_t);

}  // namespace yamoe

using namespace yamoe;

extern "C" int yamoe_router_topk(const void *hidden, const void *weight, const void *bias, int32_t T_, int32_t H, int32_t E,
                                 int32_t K, int32_t dtype, int64_t *router_indices, void *router_scores, void *topk_weights,
                                 void *logits, void *stream) {
  const int step = dtype == YAMOE_F32 ? 8 : 16;
  if (T_ < 0 || H <= 0 || H % step != 0 || E <= 0 || E > kRouterMaxE || K <= 0 || K > kRouterMaxK || K > E) {
    set_error("yamoe_router_topk: need H %% %d == 0, 1 <= E <= %d, 1 <= top_k <= min(E, %d) (got H=%d E=%d top_k=%d)",
              step, kRouterMaxE, kRouterMaxK, H, E, K);
    return YAMOE_E_ARG;
  }
  if (T_ == 0) return 0;
  if (!hidden || !weight || !router_indices || !router_scores) {
    set_error("yamoe_router_topk: null pointer");
    return YAMOE_E_ARG;
  }
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case YAMOE_BF16:
      return router_dispatch<bf16_t>(hidden, weight, bias, T_, H, E, K, (long long *)router_indices, router_scores,
                                     topk_weights, logits, s);
    case YAMOE_F16:
      return router_dispatch<f16_t>(hidden, weight, bias, T_, H, E, K, (long long *)router_indices, router_scores,
                                    topk_weights, logits, s);
    case YAMOE_F32:
      return router_dispatch<float>(hidden, weight, bias, T_, H, E, K, (long long *)router_indices, router_scores,
                                    topk_weights, logits, s);
    default:
      set_error("yamoe_router_topk: unknown dtype %d", dtype);
      return YAMOE_E_DTYPE;
  }
}
