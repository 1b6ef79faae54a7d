// The public helper ops of drbh/yamoe (torch-ext/torch_binding.cpp:9-56) on the reference's own data
// layouts: `sort`, `bincount_cumsum`, `gather`, `scatter`, `index_select_out`.  (`batch_mm` is served by
// the grouped GEMM kernels, see cabi.hip.)  The fused forward does not use these: it keeps
// expert-contiguous buffers without padding.  They exist so that code written against the reference's
// helper ops keeps working, with the padded [E, C, H] buffers and inclusive `bins` it expects.
#include <type_traits>

#include "common.h"

namespace yamoe {

// ---- sort: stable LSD radix sort of integer keys with an iota payload (csrc/sort.cu:17-91) --------------
// 8-bit digits; one pass = per-wave segment histograms, a scan to per-(digit, segment) cursors, and an
// in-order placement with wavefront-ballot ranking, exactly the scheme of route.hip with 256 buckets.
constexpr int kSortThreads = 1024;
constexpr int kSortWaves = kSortThreads / kWave;
constexpr int kSortSeg = 1024;  // elements per wave segment
constexpr int kRadix = 256;

template <typename K>
__device__ inline unsigned digit_of(K key, int shift, int bits, bool flip_sign) {
  typedef typename std::make_unsigned<K>::type U;
  U u = (U)key;
  if (flip_sign) u ^= (U)((U)1 << (sizeof(K) * 8 - 1));
  return (unsigned)((u >> shift) & (U)((1u << bits) - 1u));
}

template <typename K>
__global__ __launch_bounds__(kSortThreads) void sort_hist_kernel(const K *keys, int n, int shift, int bits,
                                                                 bool flip_sign, int *seg_counts) {
  __shared__ int hist[kSortWaves * kRadix];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int i = tid; i < kSortWaves * kRadix; i += kSortThreads) hist[i] = 0;
  __syncthreads();
  long long seg = (long long)blockIdx.x * kSortWaves + wave;
  long long b = seg * kSortSeg, e = b + kSortSeg;
  if (e > n) e = n;
  for (long long i = b + lane; i < e; i += kWave) atomicAdd(&hist[wave * kRadix + digit_of(keys[i], shift, bits, flip_sign)], 1);
  __syncthreads();
  for (int i = tid; i < kSortWaves * kRadix; i += kSortThreads)
    seg_counts[(size_t)blockIdx.x * kSortWaves * kRadix + i] = hist[i];
}

// one block of 256 threads: thread d owns digit d
__global__ __launch_bounds__(kRadix) void sort_scan_kernel(int *seg_counts, int n_seg) {
  __shared__ int total[kRadix];
  const int d = threadIdx.x;
  int s = 0;
  for (int g = 0; g < n_seg; ++g) s += seg_counts[(size_t)g * kRadix + d];
  total[d] = s;
  __syncthreads();
  int base = 0;
  for (int j = 0; j < d; ++j) base += total[j];
  for (int g = 0; g < n_seg; ++g) {
    int c = seg_counts[(size_t)g * kRadix + d];
    seg_counts[(size_t)g * kRadix + d] = base;
    base += c;
  }
}

template <typename K>
__global__ __launch_bounds__(kSortThreads) void sort_place_kernel(const K *keys, const K *vals, bool iota_vals, int n,
                                                                  int shift, int bits, bool flip_sign,
                                                                  const int *seg_cursors, K *keys_out, K *vals_out) {
  __shared__ int cursor_all[kSortWaves * kRadix];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int i = tid; i < kSortWaves * kRadix; i += kSortThreads)
    cursor_all[i] = seg_cursors[(size_t)blockIdx.x * kSortWaves * kRadix + i];
  __syncthreads();
  int *cursor = cursor_all + wave * kRadix;
  long long seg = (long long)blockIdx.x * kSortWaves + wave;
  long long b = seg * kSortSeg, e = b + kSortSeg;
  if (e > n) e = n;
  const uint64_t lt_mask = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
  for (long long base = b; base < e; base += kWave) {
    long long i = base + lane;
    bool active = i < e;
    K key = active ? keys[i] : (K)0;
    K val = active ? (iota_vals ? (K)i : vals[i]) : (K)0;
    unsigned dg = digit_of(key, shift, bits, flip_sign);
    uint64_t peers = __ballot(active);
    for (int bit = 0; bit < bits; ++bit) {
      bool s = (dg >> bit) & 1;
      uint64_t m = __ballot(active && s);
      peers &= s ? m : ~m;
    }
    int rank = __popcll(peers & lt_mask);
    int start = 0;
    if (active) start = cursor[dg];
    __builtin_amdgcn_wave_barrier();
    if (active) {
      keys_out[start + rank] = key;
      vals_out[start + rank] = val;
      if (rank == 0) cursor[dg] = start + __popcll(peers);
    }
    // the cursor is private to this wave and LDS operations of one wave complete in order: the next step's
    // read sees this step's write without a fence or a volatile access (both would also wait for the global
    // stores above); lanes address the cursor by key, so the compiler cannot carry its values across steps
    __builtin_amdgcn_wave_barrier();
  }
}

template <typename K>
__global__ void sort_copy_iota_kernel(const K *keys, K *keys_out, K *vals_out, int n) {
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) {
    keys_out[i] = keys[i];
    vals_out[i] = (K)i;
  }
}

template <typename K>
static int sort_impl(const void *x, int n, int end_bit, void *x_out, void *iota_out, void *ws, hipStream_t stream) {
  const int width = (int)sizeof(K) * 8;
  if (end_bit > width) end_bit = width;
  if (end_bit <= 0) {
    hipLaunchKernelGGL(sort_copy_iota_kernel<K>, dim3(ceil_div(n, 256)), dim3(256), 0, stream, (const K *)x, (K *)x_out,
                       (K *)iota_out, n);
    return check_launch("sort_copy_iota_kernel");
  }
  const int passes = ceil_div(end_bit, 8);
  const int n_blocks = ceil_div(ceil_div(n, kSortSeg), kSortWaves);
  const int n_seg = n_blocks * kSortWaves;
  K *tmp_k = (K *)ws;
  K *tmp_v = tmp_k + align_up((size_t)n, 64);
  int *seg_counts = (int *)(tmp_v + align_up((size_t)n, 64));
  // ping-pong so that the last pass writes x_out / iota_out
  const K *src_k = (const K *)x;
  const K *src_v = nullptr;
  for (int p = 0; p < passes; ++p) {
    bool to_out = ((passes - 1 - p) % 2) == 0;
    K *dst_k = to_out ? (K *)x_out : tmp_k, *dst_v = to_out ? (K *)iota_out : tmp_v;
    int shift = 8 * p, bits = end_bit - shift < 8 ? end_bit - shift : 8;
    bool flip = (end_bit == width) && (p == passes - 1);
    hipLaunchKernelGGL(sort_hist_kernel<K>, dim3(n_blocks), dim3(kSortThreads), 0, stream, src_k, n, shift, bits, flip,
                       seg_counts);
    hipLaunchKernelGGL(sort_scan_kernel, dim3(1), dim3(kRadix), 0, stream, seg_counts, n_seg);
    hipLaunchKernelGGL(sort_place_kernel<K>, dim3(n_blocks), dim3(kSortThreads), 0, stream, src_k, src_v, p == 0, n, shift,
                       bits, flip, seg_counts, dst_k, dst_v);
    int rc = check_launch("sort pass");
    if (rc) return rc;
    src_k = dst_k;
    src_v = dst_v;
  }
  return 0;
}

// ---- bincount + inclusive cumsum (csrc/bincount_cumsum.cu:7-97) ---------------------------------------
// One workgroup: LDS histogram of the whole input, then a scan.  out[0..minlength) = inclusive prefix
// sums, out[minlength..out_len) = 0 (the reference zeroes the whole buffer first).
constexpr int kBincountMaxBins = 8192;
__global__ __launch_bounds__(1024) void bincount_cumsum_kernel(const int *in, int n, int *out, int out_len, int minlength) {
  __shared__ int hist[kBincountMaxBins];
  __shared__ int carry;
  const int tid = threadIdx.x;
  for (int i = tid; i < minlength; i += blockDim.x) hist[i] = 0;
  if (tid == 0) carry = 0;
  __syncthreads();
  for (int i = tid; i < n; i += blockDim.x) {
    int b = in[i];
    if (b >= 0 && b < minlength) atomicAdd(&hist[b], 1);
  }
  __syncthreads();
  // chunked inclusive scan: each chunk of blockDim.x bins by Hillis-Steele in LDS
  for (int base = 0; base < minlength; base += blockDim.x) {
    int i = base + tid;
    int m = min((int)blockDim.x, minlength - base);
    for (int d = 1; d < m; d <<= 1) {
      int v = 0;
      if (i < minlength && tid >= d) v = hist[i - d];
      __syncthreads();
      if (i < minlength && tid >= d) hist[i] += v;
      __syncthreads();
    }
    if (i < minlength) hist[i] += carry;
    __syncthreads();
    if (tid == 0) carry = hist[base + m - 1];
    __syncthreads();
  }
  for (int i = tid; i < out_len; i += blockDim.x) out[i] = i < minlength ? hist[i] : 0;
}

// ---- padded gather (csrc/gather.cu:6-109): out[e,i,:] = x[idx[start_e+i] / top_k,:] or 0 -----------------
template <typename T>
__global__ __launch_bounds__(256) void padded_gather_kernel(const T *x, const int *idx, const int *bins, T *out, int Tn,
                                                            int H, int E, int C, int top_k) {
  const int lane = threadIdx.x & 63;
  const long long n_rows = (long long)E * C;
  for (long long row = (long long)blockIdx.x * 4 + (threadIdx.x >> 6); row < n_rows; row += (long long)gridDim.x * 4) {
    int e = (int)(row / C), i = (int)(row - (long long)e * C);
    int start = e == 0 ? 0 : bins[e - 1], n = bins[e] - start;
    bool valid = i < n;
    int tok = 0;
    if (valid) {
      tok = idx[start + i] / top_k;
      if (tok < 0 || tok >= Tn) valid = false;
    }
    T *dst = out + row * H;
    const T *src = x + (long long)tok * H;
    constexpr int V = ElemTraits<T>::kVec;
    if (H % V == 0) {
      for (int c = lane; c < H / V; c += 64) {
        u32x4 v = {0, 0, 0, 0};
        if (valid) v = ((const u32x4 *)src)[c];
        ((u32x4 *)dst)[c] = v;
      }
    } else {
      for (int c = lane; c < H; c += 64) dst[c] = valid ? src[c] : ElemTraits<T>::from_f32(0.0f);
    }
  }
}

// ---- padded scatter (csrc/scatter.cu:66-147): y[tok,:] += src[e,i,:] * w[start_e+i] -----------------------
// Done without atomics: pass 1 records, for every flat slot, which padded row (if any) feeds it; pass 2
// owns one output row per wave and adds that token's rows in slot order.
__global__ void scatter_index_kernel(const int *idx, const int *bins, int *slot_row, int S, int E, int C) {
  int p = blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= S) return;
  // expert of sorted position p: first e with bins[e] > p
  int lo = 0, hi = E;
  while (lo < hi) {
    int mid = (lo + hi) >> 1;
    if (bins[mid] > p) hi = mid; else lo = mid + 1;
  }
  if (lo >= E) return;
  int start = lo == 0 ? 0 : bins[lo - 1];
  int i = p - start;
  int flat = idx[p];
  if (i < C && flat >= 0 && flat < S) slot_row[flat] = lo * C + i;
}
template <typename T>
__global__ __launch_bounds__(256) void padded_scatter_kernel(const T *src, const int *slot_row, const int *idx_unused,
                                                             const int *bins, const T *weights, T *y, int Tn, int H, int C,
                                                             int top_k, int E) {
  const int lane = threadIdx.x & 63;
  for (int t = blockIdx.x * 4 + (threadIdx.x >> 6); t < Tn; t += gridDim.x * 4) {
    for (int c = lane; c < H; c += 64) {
      typedef typename ElemTraits<T>::acc_t acc_t;
      acc_t acc = ElemTraits<T>::to_acc(y[(long long)t * H + c]);
      for (int k = 0; k < top_k; ++k) {
        int row = slot_row[t * top_k + k];
        if (row < 0) continue;
        int e = row / C, i = row - e * C;
        int start = e == 0 ? 0 : bins[e - 1];
        acc_t w = weights ? ElemTraits<T>::to_acc(weights[start + i]) : (acc_t)1;
        acc += w * ElemTraits<T>::to_acc(src[(long long)row * H + c]);
      }
      y[(long long)t * H + c] = ElemTraits<T>::from_acc(acc);
    }
  }
}
__global__ void fill_i32_kernel(int *p, int n, int v) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v;
}

// ---- index_select_out (csrc/index_select.cu:7-51): out[i] = in[idx[i]] ------------------------------------
template <typename T>
__global__ void index_select_kernel(const T *in, const int *idx, T *out, long long n) {
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = in[idx[i]];
}

// counts[e] = rows, offsets[e] = e * rows: the regular [E, C, *] layout as a ragged one (for batch_mm)
__global__ void regular_groups_kernel(int *counts, int *offsets, int E, int rows) {
  int e = blockIdx.x * blockDim.x + threadIdx.x;
  if (e < E) counts[e] = rows;
  if (e <= E) offsets[e] = e * rows;
}

}  // namespace yamoe

using namespace yamoe;

extern "C" size_t yamoe_sort_workspace_bytes(int32_t n, int32_t elem_bytes) {
  size_t nn = align_up((size_t)(n > 0 ? n : 1), 64);
  int n_blocks = ceil_div(ceil_div(n > 0 ? n : 1, kSortSeg), kSortWaves);
  return align_up(2 * nn * (size_t)elem_bytes + (size_t)n_blocks * kSortWaves * kRadix * sizeof(int), 256);
}

extern "C" int yamoe_sort(const void *x, int32_t elem_bytes, int32_t n, int32_t end_bit, void *x_out, void *iota_out,
                          void *workspace, size_t workspace_bytes, void *stream) {
  if (n < 0 || (elem_bytes != 2 && elem_bytes != 4 && elem_bytes != 8)) {
    set_error("yamoe_sort: keys must be int16, int32 or int64 and n >= 0");
    return YAMOE_E_ARG;
  }
  if (n == 0) return 0;
  if (!x || !x_out || !iota_out || !workspace) { set_error("yamoe_sort: null pointer"); return YAMOE_E_ARG; }
  if (workspace_bytes < yamoe_sort_workspace_bytes(n, elem_bytes)) {
    set_error("yamoe_sort: workspace too small");
    return YAMOE_E_WORKSPACE;
  }
  hipStream_t st = (hipStream_t)stream;
  if (elem_bytes == 2) return sort_impl<short>(x, n, end_bit, x_out, iota_out, workspace, st);
  if (elem_bytes == 4) return sort_impl<int>(x, n, end_bit, x_out, iota_out, workspace, st);
  return sort_impl<long long>(x, n, end_bit, x_out, iota_out, workspace, st);
}

extern "C" int yamoe_bincount_cumsum(const int32_t *input, int32_t n, int32_t *output, int32_t output_len,
                                     int32_t minlength, void *stream) {
  if (n < 0 || minlength < 0 || output_len < minlength || minlength > kBincountMaxBins || (n > 0 && !input) ||
      (output_len > 0 && !output)) {
    set_error("yamoe_bincount_cumsum: need 0 <= minlength <= min(output_len, %d)", kBincountMaxBins);
    return YAMOE_E_ARG;
  }
  if (output_len == 0) return 0;
  hipLaunchKernelGGL(bincount_cumsum_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, input, n, output, output_len,
                     minlength);
  return check_launch("bincount_cumsum_kernel");
}

#define YAMOE_DISPATCH(dtype, CALL)                                       \
  switch (dtype) {                                                        \
    case YAMOE_F32: { typedef float T; CALL; break; }                     \
    case YAMOE_BF16: { typedef bf16_t T; CALL; break; }                   \
    case YAMOE_F16: { typedef f16_t T; CALL; break; }                     \
    case YAMOE_F64: { typedef double T; CALL; break; }                    \
    default: set_error("unknown dtype %d", dtype); return YAMOE_E_DTYPE;  \
  }

extern "C" int yamoe_padded_gather(const void *x, const int32_t *indices, const int32_t *bins, void *output, int32_t T_,
                                   int32_t H, int32_t E, int32_t C, int32_t top_k, int32_t dtype, void *stream) {
  if (T_ < 0 || H <= 0 || E <= 0 || C < 0 || top_k <= 0) { set_error("yamoe_padded_gather: bad size"); return YAMOE_E_ARG; }
  if ((long long)E * C == 0) return 0;
  if (!x || !indices || !bins || !output) { set_error("yamoe_padded_gather: null pointer"); return YAMOE_E_ARG; }
  long long rows = (long long)E * C;
  int blocks = (int)((rows + 3) / 4 < 65536 ? (rows + 3) / 4 : 65536);
  YAMOE_DISPATCH(dtype, hipLaunchKernelGGL(padded_gather_kernel<T>, dim3(blocks), dim3(256), 0, (hipStream_t)stream,
                                           (const T *)x, indices, bins, (T *)output, T_, H, E, C, top_k));
  return check_launch("padded_gather_kernel");
}

extern "C" size_t yamoe_padded_scatter_workspace_bytes(int32_t S) { return align_up((size_t)(S > 0 ? S : 1) * 4, 256); }

extern "C" int yamoe_padded_scatter(const void *src, const int32_t *indices, const int32_t *bins, const void *weights,
                                    void *y, int32_t T_, int32_t H, int32_t E, int32_t C, int32_t top_k, int32_t dtype,
                                    void *workspace, size_t workspace_bytes, void *stream) {
  if (T_ < 0 || H <= 0 || E <= 0 || C < 0 || top_k <= 0) { set_error("yamoe_padded_scatter: bad size"); return YAMOE_E_ARG; }
  const int S = T_ * top_k;
  if (S == 0 || C == 0) return 0;  // (a capacity of zero keeps no row: y stays as it is, and src may be an empty tensor)
  if (!src || !indices || !bins || !y || !workspace || workspace_bytes < yamoe_padded_scatter_workspace_bytes(S)) {
    set_error("yamoe_padded_scatter: null pointer or workspace too small");
    return YAMOE_E_ARG;
  }
  hipStream_t st = (hipStream_t)stream;
  int *slot_row = (int *)workspace;
  hipLaunchKernelGGL(fill_i32_kernel, dim3(ceil_div(S, 256)), dim3(256), 0, st, slot_row, S, -1);
  hipLaunchKernelGGL(scatter_index_kernel, dim3(ceil_div(S, 256)), dim3(256), 0, st, indices, bins, slot_row, S, E, C);
  int blocks = (T_ + 3) / 4 < 65536 ? (T_ + 3) / 4 : 65536;
  YAMOE_DISPATCH(dtype, hipLaunchKernelGGL(padded_scatter_kernel<T>, dim3(blocks), dim3(256), 0, st, (const T *)src, slot_row,
                                           indices, bins, (const T *)weights, (T *)y, T_, H, C, top_k, E));
  return check_launch("padded_scatter_kernel");
}

extern "C" int yamoe_index_select(const void *input, const int32_t *idx, void *out, int64_t n, int32_t dtype,
                                  void *stream) {
  if (n < 0) { set_error("yamoe_index_select: n < 0"); return YAMOE_E_ARG; }
  if (n == 0) return 0;
  if (!input || !idx || !out) { set_error("yamoe_index_select: null pointer"); return YAMOE_E_ARG; }
  unsigned blocks = (unsigned)((n + 255) / 256);
  YAMOE_DISPATCH(dtype, hipLaunchKernelGGL(index_select_kernel<T>, dim3(blocks), dim3(256), 0, (hipStream_t)stream,
                                           (const T *)input, idx, (T *)out, (long long)n));
  return check_launch("index_select_kernel");
}

extern "C" int yamoe_regular_groups(int32_t *counts, int32_t *offsets, int32_t E, int32_t rows, void *stream) {
  if (E <= 0 || rows < 0 || !counts || !offsets) { set_error("yamoe_regular_groups: bad argument"); return YAMOE_E_ARG; }
  hipLaunchKernelGGL(regular_groups_kernel, dim3(ceil_div(E + 1, 256)), dim3(256), 0, (hipStream_t)stream, counts, offsets,
                     E, rows);
  return check_launch("regular_groups_kernel");
}
