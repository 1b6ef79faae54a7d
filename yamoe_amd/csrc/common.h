// Shared device/host helpers for the gfx950 expert-layer kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "../../include/yamoe_hip.h"

namespace yamoe {

constexpr int kWave = 64;

// Clamped-SwiGLU constants of the GPT-OSS expert MLP (csrc/moe.cpp:175-179).
constexpr float kGluLimit = 7.0f;
constexpr float kGluAlpha = 1.702f;

// Experts with at most this many kept rows take the weight-streaming path: 32 when that covers every expert of the
// call, 16 when some experts need the tile kernels anyway.
constexpr int kStreamMaxRows = 32;
constexpr int kStreamMixedRows = 16;

typedef __bf16 bf16_t;
typedef _Float16 f16_t;

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

template <typename T> struct ElemTraits;
template <> struct ElemTraits<float> {
  static constexpr int kDtype = YAMOE_F32;
  static constexpr int kVec = 4;  // elements per 16-byte chunk
  typedef float acc_t;
  __device__ static inline float to_acc(float v) { return v; }
  __device__ static inline float from_acc(float v) { return v; }
  __device__ static inline float to_f32(float v) { return v; }
  __device__ static inline float from_f32(float v) { return v; }
};
// double appears only in the helper ops that move rows (gather, scatter, index_select), which the reference
// dispatches over double as well (csrc/gather.cu:89, csrc/scatter.cu:128); sums of doubles stay in double
template <> struct ElemTraits<double> {
  static constexpr int kDtype = YAMOE_F64;
  static constexpr int kVec = 2;
  typedef double acc_t;
  __device__ static inline double to_acc(double v) { return v; }
  __device__ static inline double from_acc(double v) { return v; }
  __device__ static inline double from_f32(float v) { return (double)v; }
};
template <> struct ElemTraits<bf16_t> {
  static constexpr int kDtype = YAMOE_BF16;
  static constexpr int kVec = 8;
  typedef float acc_t;
  __device__ static inline float to_acc(bf16_t v) { return (float)v; }
  __device__ static inline bf16_t from_acc(float v) { return (bf16_t)v; }
  __device__ static inline float to_f32(bf16_t v) { return (float)v; }
  __device__ static inline bf16_t from_f32(float v) { return (bf16_t)v; }
};
template <> struct ElemTraits<f16_t> {
  static constexpr int kDtype = YAMOE_F16;
  static constexpr int kVec = 8;
  typedef float acc_t;
  __device__ static inline float to_acc(f16_t v) { return (float)v; }
  __device__ static inline f16_t from_acc(float v) { return (f16_t)v; }
  __device__ static inline float to_f32(f16_t v) { return (float)v; }
  __device__ static inline f16_t from_f32(float v) { return (f16_t)v; }
};

__host__ __device__ inline size_t dtype_size(int dtype) { return dtype == YAMOE_F64 ? 8 : dtype == YAMOE_F32 ? 4 : 2; }

__host__ __device__ inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

// Division of 0 <= n < 2^31 by a divisor fixed per launch, as a multiply-high, an add and a shift (round-up method:
// l = ceil(log2 d), mul = floor(2^32 * (2^l - d) / d) + 1, n / d = (mulhi(n, mul) + n) >> l; the sum stays below 2^32).
struct FastDiv {
  uint32_t mul, shift;
};
__host__ __device__ inline FastDiv make_fast_div(int d) {
  FastDiv f;
  uint32_t l = 0;
  while ((1ull << l) < (unsigned long long)d) ++l;
  f.mul = (uint32_t)(((1ull << 32) * ((1ull << l) - (unsigned long long)d)) / (unsigned long long)d + 1ull);
  f.shift = l;
  return f;
}
__device__ inline int fast_div(int n, FastDiv f) { return (int)((__umulhi((uint32_t)n, f.mul) + (uint32_t)n) >> f.shift); }
__host__ __device__ inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// h = (clamp(U,-L,L) + 1) * g * sigmoid(alpha * g),  g = min(G, L)     (csrc/moe.cpp:164-180)
__device__ inline float glu_forward(float G, float U) {
  float g = fminf(G, kGluLimit);
  float u = fminf(fmaxf(U, -kGluLimit), kGluLimit);
  // sigmoid through the hardware exp2 and reciprocal (each about 1 ulp); exp2(+inf) -> s = 0, the right limit
  float s = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(g * (-kGluAlpha * 1.44269504088896341f)));
  return (u + 1.0f) * (g * s);
}

// Gradients of glu_forward with respect to G and U given dh (csrc/experts_backward.cu:285-299).
__device__ inline void glu_backward(float G, float U, float dh, float &dG, float &dU) {
  float g = fminf(G, kGluLimit);
  float u = fminf(fmaxf(U, -kGluLimit), kGluLimit);
  float s = 1.0f / (1.0f + __expf(-kGluAlpha * g));
  float a = g * s;
  dU = (U > kGluLimit || U < -kGluLimit) ? 0.0f : dh * a;
  float dgl = dh * (u + 1.0f);
  dG = (G > kGluLimit) ? 0.0f : dgl * (s + g * s * (1.0f - s) * kGluAlpha);
}

// A pre-activation as the backward will read it back: rounded to T, except that a value beyond the clamp limit whose
// rounding lands on the limit itself is stored one step further out.  glu_backward tests the stored value against the
// limit; without this, the values in (7, 7.016] of a bf16 run would pass a gradient that the fp32 value, and the
// forward, clamp away (a few elements in ten thousand, but each one wrong by its whole size).  `up`: the up half is
// clamped on both sides, the gate half from above only.
template <typename T> __device__ inline T pre_activation_store(float v, bool up) {
  T r = ElemTraits<T>::from_f32(v);
  if constexpr (sizeof(T) == 2) {
    const uint16_t lim = __builtin_bit_cast(uint16_t, ElemTraits<T>::from_f32(kGluLimit));  // (exactly representable)
    uint16_t bits = __builtin_bit_cast(uint16_t, r);
    if ((bits & 0x7fffu) == lim && (v > kGluLimit || (up && v < -kGluLimit))) r = __builtin_bit_cast(T, (uint16_t)(bits + 1));
  }
  return r;
}

// 16 bytes per lane from global memory straight into LDS at lds_base + lane * 16.
// (lds_base is the same for every lane; saying so keeps it in a scalar register even where the compiler has merged
// its computation with a per-lane address of the same LDS buffer)
__device__ inline void copy16_to_lds(const void *uniform_base, uint32_t lane_byte_off, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1"
               :
               : "v"(lane_byte_off), "s"(uniform_base), "s"(__builtin_amdgcn_readfirstlane(lds_base))
               : "memory", "m0");
}

// ---- schedule: device-built work lists shared by the expert GEMM kernels ---------------------
// Layout of the schedule region (int32 words):
//   [0] n_row_tiles   number of (expert, row-block) entries for the MFMA kernels
//   [1] n_small       number of experts on the weight-streaming path
//   [2] n_active      experts with at least one kept row
//   [3] n_kept        total kept rows
//   [4] weight_total  sum of the experts' cost weights (sched_group_weight)
//   [8 + 4x ...)      x = 0..8: where the tile list is cut so that each of the 8 XCDs gets the same share of
//                     the cost: {first row tile of the expert the cut falls in, f, 0, row tiles of that
//                     expert}, f = the cut's position inside that expert's tiles in 1/65536ths; in a GEMM
//                     with n column tiles the cut is at flat tile index
//                     first * n + ((f * n) >> 16) * row_tiles, i.e. on a column-tile boundary of that expert
//   [48 ...)          row tiles: 8 words each  {expert, first sorted row, valid rows,
//                       index of the expert's first row tile, number of row tiles of the expert, 0,0,0}
//   then              small experts: 4 words each {expert, first sorted row, valid rows, 0}
constexpr int kRowTile = 256;  // rows of one MFMA row tile
constexpr int kColTile = 256;  // columns of one MFMA tile
constexpr int kSchedHeader = 48;
constexpr int kSchedCuts = 8;  // word offset of the XCD cut table
constexpr int kXcds = 8;

// Relative cost of one row tile in the MFMA kernels: a fixed part (prologue, epilogue, copies of the weight
// slabs) plus one part per 64 rows (the MFMA blocks of the slower wave row).
__host__ __device__ inline int sched_tile_weight(int rows) { return 3 + 2 * ((rows + 63) / 64); }
// An expert with a single row tile shares its weight slabs with nobody: every one of its column tiles pulls them from
// HBM at one workgroup's latency-bound rate, which takes about as long as a tile of 150-200 rows however few rows it
// has (measured on the Zipf-skewed workload: 2 % of the step between this floor and none).
constexpr int kLoneTileWeight = 8;
__host__ __device__ inline int sched_group_weight(int tiles, int per_tile, int kept) {
  if (tiles <= 0) return 0;
  int w = (tiles - 1) * sched_tile_weight(per_tile) + sched_tile_weight(kept - (tiles - 1) * per_tile);
  return tiles == 1 && w < kLoneTileWeight ? kLoneTileWeight : w;
}
// flat tile index of cut x of the schedule for a GEMM with n_col_tiles column tiles
__host__ __device__ inline int sched_cut(const int *sched, int x, int n_col_tiles) {
  const int *c = sched + kSchedCuts + 4 * x;
  return c[0] * n_col_tiles + ((c[1] * n_col_tiles) >> 16) * c[3];
}

__host__ __device__ inline int sched_max_row_tiles(int N, int E) {
  // every expert with kept rows adds at most one partly filled tile
  return N / kRowTile + (N < E ? N : E) + 1;
}
// Upper bound of the row-tile count when experts with at most `small_rows` kept rows are not tiled (they are on
// the streaming list): only N / (small_rows + 1) experts can hold more rows than that.  Used for grid sizes only.
__host__ __device__ inline int sched_grid_row_tiles(int N, int E, int small_rows) {
  // (the list may have been built with the lower of the two streaming limits)
  if (small_rows > kStreamMixedRows) small_rows = kStreamMixedRows;
  int tiled = N / (small_rows + 1);
  if (tiled > E) tiled = E;
  return N / kRowTile + tiled + 1;
}
// Every expert may be put on the streaming list in chunks of at most kStreamMaxRows rows (stream_max_rows =
// kStreamEverything) when there are at most 4 assignments per expert on average: the weights of an expert with more
// rows than one chunk are then read once per chunk, which is rare at that load, and the tile kernels are not launched.
constexpr int kStreamEverything = -1;
__host__ __device__ inline bool sched_may_stream_everything(int N, int E) { return N <= 4 * E; }
__host__ __device__ inline int sched_max_small(int N, int E) {
  return (N < E ? N : E) + (sched_may_stream_everything(N, E) ? N / kStreamMaxRows : 0) + 1;
}

struct ScheduleView {
  const int *hdr;
  const int *row_tiles;
  const int *small;
};
__host__ __device__ inline ScheduleView schedule_view(const void *p, int N, int E) {
  const int *w = (const int *)p;
  ScheduleView v;
  v.hdr = w;
  v.row_tiles = w + kSchedHeader;
  v.small = w + kSchedHeader + 8 * sched_max_row_tiles(N, E);
  return v;
}

int route_and_schedule(const void *router_indices, int32_t idx_i64, int32_t N, int32_t E, int32_t capacity,
                       int32_t *sorted_expert, int32_t *sorted_idx, int32_t *counts, int32_t *offsets, int32_t *inv_pos,
                       void *workspace, size_t workspace_bytes, int32_t stream_max_rows, void *schedule,
                       size_t schedule_bytes, void *stream);

// error reporting for the C ABI
void set_error(const char *fmt, ...);
int check_launch(const char *what);

// Kernels that use more than 64 KB of dynamic LDS need hipFuncAttributeMaxDynamicSharedMemorySize raised, once per
// device (every device loads its own copy of the code).  `done` holds one flag per device for one kernel; the
// attribute call is idempotent, so two threads racing through the first call are harmless.
constexpr int kMaxDevices = 64;
struct DeviceFlags {
  std::atomic<bool> flag[kMaxDevices];
};
int ensure_dynamic_lds(const void *kernel, int bytes, DeviceFlags &done, const char *what);

}  // namespace yamoe
