// Weight-streaming path for experts with at most 32 kept rows (the decode regime).
//
// Such an expert does 2*rows flops per weight element, far below the machine balance, so the job
// is to pull each expert's weights through the chip once at HBM rate.  A workgroup owns one
// (expert, 128-column slab) of a [K, N] weight matrix.  Its 4 wavefronts take the 32-row k-steps
// of the slab round-robin; in a step every lane fetches an 8(k) x 8(column) block as eight 16-byte
// loads (a wave reads 32 rows x 256 contiguous bytes), transposes it in registers and feeds it to
// eight v_mfma_f32_16x16x32 instructions whose 16-row A operand is the expert's (zero-padded)
// activations (an expert with 17 to 32 rows has two such operands and runs every column operand through both).  No LDS is touched until the final cross-wave reduction.  Two steps of loads are
// kept in flight per wave, at least 8 waves per CU.
//
// A launch that can hold only a few experts (a handful of tokens: at most kStreamFewBlocks workgroups) has too few
// workgroups to keep HBM busy that way: 4 experts x 23 slabs with two steps of 8 KB in flight per wave are 6 MB on
// the way, where 8 TB/s x 2 us of latency want 16 MB.  Such a launch takes 8 waves per workgroup with three steps in
// flight each instead (a workgroup per CU; 16 waves with two steps each measured 3 % slower), folded into the first
// four before the same finish.
//
// The lane that holds accumulator column c of MFMA j owns output column 8c + j, so the 8
// accumulators of a lane are 8 consecutive output columns: the interleaved (gate, up) pairs of the
// clamped SwiGLU (csrc/moe.cpp:164-180) meet in one lane.
#include "common.h"

namespace yamoe {

constexpr int kStreamWaves = 4;        // waves that finish a slab; a workgroup has 4 or 8
constexpr int kStreamManyWaves = 8;
constexpr int kStreamFewBlocks = 1024;  // launches with fewer (expert, slab) workgroups than this take 8 waves each
constexpr int kSlabCols = 128;

typedef float f32x4v __attribute__((ext_vector_type(4)));

template <typename T> struct Mma16;
template <> struct Mma16<bf16_t> {
  __device__ static inline f32x4v run(const u32x4 &a, const u32x4 &b, f32x4v c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c,
                                                   0, 0, 0);
  }
};
template <> struct Mma16<f16_t> {
  __device__ static inline f32x4v run(const u32x4 &a, const u32x4 &b, f32x4v c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0,
                                                  0, 0);
  }
};

struct StreamArgs {
  const void *A;       // activations [rows, lda], k-contiguous
  const void *B;       // weights [E, Kd, Nd]
  const void *bias;    // [E, Nd] or null
  void *C;             // GLU: act [rows, Nd/2]; else [rows, Nd]
  void *C2;            // GLU: optional pre-activations [rows, Nd]
  const int *a_rows;   // optional gather: source row = a_rows[p] / a_div
  const int *sched;
  int a_div, Kd, Nd, lda, ldc, n_slabs, N, E;
};

// One (expert, slab) of RB blocks of 16 rows (RB = 1: up to 16 rows, RB = 2: 17 to 32): the weights are fetched once
// and every column operand built from them goes through RB MFMAs.
template <typename T, bool GLU, bool GATHER, int WAVES, int DEPTH, int RB>
__device__ inline void stream_slab(const StreamArgs &args, float *red, const int expert, const int first, const int rows,
                                   const int slab) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int c16 = lane & 15, g = lane >> 4;
  const int col0 = slab * kSlabCols + c16 * 8;  // first of this lane's 8 output columns
  const bool col_ok = col0 < args.Nd;
  const T *Bp = (const T *)args.B + (long long)expert * args.Kd * args.Nd + col0;

  // A operand of block b: row 16 b + c16 of the expert (zero beyond `rows`), 8 consecutive k starting at 8 g
  bool a_ok[RB];
  const T *Ap[RB];
#pragma unroll
  for (int b = 0; b < RB; ++b) {
    a_ok[b] = 16 * b + c16 < rows;
    long long a_src = first + (a_ok[b] ? 16 * b + c16 : 0);
    if (GATHER) a_src = args.a_rows[a_src] / args.a_div;
    Ap[b] = (const T *)args.A + a_src * args.lda + g * 8;
  }

  f32x4v acc[RB][8];
#pragma unroll
  for (int b = 0; b < RB; ++b)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[b][j] = (f32x4v){0.f, 0.f, 0.f, 0.f};

  const int n_steps = (args.Kd + 31) / 32;
  u32x4 bw[DEPTH][8], aw[DEPTH][RB];

  auto fetch = [&](int step, u32x4 (&bw)[8], u32x4 (&aw)[RB]) {
    int k0 = step * 32;
    int ka = k0 + g * 8;
#pragma unroll
    for (int b = 0; b < RB; ++b) {
      aw[b] = (u32x4){0, 0, 0, 0};
      if (a_ok[b] && ka < args.Kd) aw[b] = *(const u32x4 *)(Ap[b] + k0);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      int k = ka + i;
      u32x4 v = {0, 0, 0, 0};
      if (col_ok && k < args.Kd) v = __builtin_nontemporal_load((const u32x4 *)(Bp + (long long)k * args.Nd));
      bw[i] = v;
    }
  };
  auto consume = [&](const u32x4 (&bw)[8], const u32x4 (&aw)[RB]) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
      u32x4 col;
#pragma unroll
      for (int d = 0; d < 4; ++d) col[d] = __builtin_amdgcn_perm(bw[2 * d + 1][j >> 1], bw[2 * d][j >> 1], sel);
#pragma unroll
      for (int b = 0; b < RB; ++b) acc[b][j] = Mma16<T>::run(aw[b], col, acc[b][j]);
    }
  };

  // steps wave, wave + WAVES, ... ; DEPTH in flight (the loop is unrolled by DEPTH, so the buffers are fixed registers)
  int step = wave;
#pragma unroll
  for (int d = 0; d < DEPTH - 1; ++d)
    if (step + d * WAVES < n_steps) fetch(step + d * WAVES, bw[d], aw[d]);
  for (bool more = step < n_steps; more;) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      if (more) {
        if (step + (DEPTH - 1) * WAVES < n_steps) fetch(step + (DEPTH - 1) * WAVES, bw[(d + DEPTH - 1) % DEPTH], aw[(d + DEPTH - 1) % DEPTH]);
        consume(bw[d], aw[d]);
        step += WAVES;
        more = step < n_steps;
      }
    }
  }

  // ---- reduce the partial sums and finish, one block of 16 rows after the other -------------------------------
  const int col = col0 + 2 * wave;  // wave w (of the first four) finishes accumulator columns j = 2w, 2w+1: one (gate, up) pair per lane
  float b0 = 0.f, b1 = 0.f;
  if (wave < kStreamWaves && col_ok && args.bias != nullptr) {
    const T *bp = (const T *)args.bias + (long long)expert * args.Nd + col;
    b0 = ElemTraits<T>::to_f32(bp[0]);
    b1 = ElemTraits<T>::to_f32(bp[1]);
  }
#pragma unroll
  for (int b = 0; b < RB; ++b) {
    // more than four waves: waves 4r .. 4r+3 hand their sums to waves 0 .. 3, one group after the other (a fixed order)
    for (int r = 1; r < WAVES / kStreamWaves; ++r) {
      if (wave / kStreamWaves == r) {
#pragma unroll
        for (int j = 0; j < 8; ++j)
#pragma unroll
          for (int v = 0; v < 4; ++v) red[(((wave - kStreamWaves * r) * 8 + j) * 4 + v) * kWave + lane] = acc[b][j][v];
      }
      __syncthreads();
      if (wave < kStreamWaves) {
#pragma unroll
        for (int j = 0; j < 8; ++j)
#pragma unroll
          for (int v = 0; v < 4; ++v) acc[b][j][v] += red[((wave * 8 + j) * 4 + v) * kWave + lane];
      }
      __syncthreads();
    }
    if (wave < kStreamWaves) {
#pragma unroll
      for (int j = 0; j < 8; ++j)
#pragma unroll
        for (int v = 0; v < 4; ++v) red[((wave * 8 + j) * 4 + v) * kWave + lane] = acc[b][j][v];
    }
    __syncthreads();
    if (wave < kStreamWaves && col_ok) {
      float sum[2][4];
#pragma unroll
      for (int jj = 0; jj < 2; ++jj)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          float t = 0.f;
#pragma unroll
          for (int w = 0; w < kStreamWaves; ++w) t += red[((w * 8 + 2 * wave + jj) * 4 + v) * kWave + lane];
          sum[jj][v] = t;
        }
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        int r = 16 * b + g * 4 + v;
        if (r >= rows) continue;
        long long orow = first + r;
        float x0 = sum[0][v] + b0, x1 = sum[1][v] + b1;
        if (GLU) {
          ((T *)args.C)[orow * args.ldc + (col >> 1)] = ElemTraits<T>::from_f32(glu_forward(x0, x1));
          if (args.C2 != nullptr) {
            T *P = (T *)args.C2 + orow * args.Nd + col;
            P[0] = pre_activation_store<T>(x0, false);
            P[1] = pre_activation_store<T>(x1, true);
          }
        } else {
          T *O = (T *)args.C + orow * args.ldc + col;
          O[0] = ElemTraits<T>::from_f32(x0);
          O[1] = ElemTraits<T>::from_f32(x1);
        }
      }
    }
    if (b + 1 < RB) __syncthreads();  // the next block reuses the buffer
  }
}

template <typename T, bool GLU, bool GATHER, int WAVES, int DEPTH>
__global__ __launch_bounds__(64 * WAVES, WAVES == kStreamWaves ? 2 : 1) void stream_gemm_kernel(const StreamArgs args) {
  __shared__ float red[kStreamWaves * 8 * 4 * kWave];  // [wave][j][v][lane]
  const ScheduleView sv = schedule_view(args.sched, args.N, args.E);
  const int n_small = sv.hdr[1];
  const int s = blockIdx.x / args.n_slabs;
  if (s >= n_small) return;
  const int slab = blockIdx.x - s * args.n_slabs;
  const int expert = sv.small[4 * s], first = sv.small[4 * s + 1], rows = sv.small[4 * s + 2];
  if (rows > 16) stream_slab<T, GLU, GATHER, WAVES, DEPTH, 2>(args, red, expert, first, rows, slab);
  else stream_slab<T, GLU, GATHER, WAVES, DEPTH, 1>(args, red, expert, first, rows, slab);
}

template <typename T, bool GLU, bool GATHER>
static int launch_stream(const StreamArgs &a, hipStream_t stream) {
  long long blocks = (long long)sched_max_small(a.N, a.E) * a.n_slabs;
  if (blocks <= 0) return 0;
  if (blocks < kStreamFewBlocks) {
    hipLaunchKernelGGL((stream_gemm_kernel<T, GLU, GATHER, kStreamManyWaves, 3>), dim3((unsigned)blocks),
                       dim3(64 * kStreamManyWaves), 0, stream, a);
  } else {
    hipLaunchKernelGGL((stream_gemm_kernel<T, GLU, GATHER, kStreamWaves, 2>), dim3((unsigned)blocks), dim3(64 * kStreamWaves),
                       0, stream, a);
  }
  return check_launch("stream_gemm_kernel");
}

template <typename T>
int stream_gate_up(const void *x, const int *sorted_idx, const void *w, const void *bias, void *act, void *pre,
                   const void *sched, int N, int K, int E, int H, int I, hipStream_t stream) {
  StreamArgs a = {};
  a.A = x; a.B = w; a.bias = bias; a.C = act; a.C2 = pre; a.a_rows = sorted_idx; a.a_div = K;
  a.sched = (const int *)sched; a.Kd = H; a.Nd = 2 * I; a.lda = H; a.ldc = I;
  a.n_slabs = ceil_div(2 * I, kSlabCols); a.N = N; a.E = E;
  return launch_stream<T, true, true>(a, stream);
}

template <typename T>
int stream_down(const void *act, const void *w, const void *bias, void *y, const void *sched, int N, int E, int H,
                int I, hipStream_t stream) {
  StreamArgs a = {};
  a.A = act; a.B = w; a.bias = bias; a.C = y; a.sched = (const int *)sched;
  a.Kd = I; a.Nd = H; a.lda = I; a.ldc = H;
  a.n_slabs = ceil_div(H, kSlabCols); a.N = N; a.E = E;
  return launch_stream<T, false, false>(a, stream);
}

#define YAMOE_INSTANTIATE_STREAM(T)                                                                                  \
  template int stream_gate_up<T>(const void *, const int *, const void *, const void *, void *, void *, const void *, \
                                 int, int, int, int, int, hipStream_t);                                              \
  template int stream_down<T>(const void *, const void *, const void *, void *, const void *, int, int, int, int,    \
                              hipStream_t);
YAMOE_INSTANTIATE_STREAM(bf16_t)
YAMOE_INSTANTIATE_STREAM(f16_t)

}  // namespace yamoe
