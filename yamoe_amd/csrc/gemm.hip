// Grouped expert GEMMs on gfx950 matrix cores.
//
// One workgroup (4 wavefronts, 2x2) computes a 256x256 output tile with 32x32 MFMA blocks
// (v_mfma_f32_32x32x16_{bf16,f16}, v_mfma_f32_32x32x2_f32), fp32 accumulators, and walks the
// contraction in slabs of 128 bytes per row (64 half-precision or 32 fp32 values).  Both operands
// sit in LDS as [row][k] with k contiguous, so a lane's MFMA operand is one 16-byte ds_read.
//
//  * An operand that is k-contiguous in memory (activations, or weights read "transposed" in the
//    data-gradient products) is copied slab by slab: 8 consecutive lanes fetch the 128 bytes of
//    one row.
//  * An operand that is contiguous along the other axis (the forward weights [K,N], and both
//    operands of the weight-gradient products) is fetched as 16-byte pieces of V consecutive
//    columns for V consecutive k (V = 8 halves or 4 floats), transposed in registers (v_perm_b32
//    for 16-bit data, pure renaming for fp32) and written as V 16-byte k-runs.  8 consecutive lanes
//    hold the 8 k-blocks of one column group, so each LDS write instruction fills whole rows.
//
// The 16-byte chunks of an LDS row are XOR-swizzled with the row number so that the MFMA operand
// reads (32 consecutive rows, same chunk) spread over all banks.
//
// Global loads of slab s+1 are issued before the MFMAs of slab s and written to the other LDS
// buffer afterwards: one barrier per slab.
//
// Tile order: workgroup ids are dealt round-robin over the 8 XCDs by the hardware, so id b is
// remapped to logical tile (b % 8) * per_xcd + b / 8.  Logical tiles run expert-major, then
// column tile, then the expert's row tiles, so the ~32 tiles in flight on one XCD share one
// expert's weight column tiles and activation row tiles through that XCD's L2.
//
// Replaces batch_mm / torch::bmm on padded [E,C,*] buffers (csrc/batch_mm.cu:7-31) and the ATen
// bias + clamped-SwiGLU chain (csrc/moe.cpp:161-187; backward csrc/experts_backward.cu:277-311).
#include <type_traits>

#include "common.h"

namespace yamoe {

constexpr int kBM = 256, kBN = 256;
constexpr int kGemmThreads = 256;
constexpr int kRowBytes = 128;                 // bytes of one LDS tile row (one K slab)
constexpr int kTileBytes = kBM * kRowBytes;    // 32 KB per operand per stage
constexpr int kGemmLds = 4 * kTileBytes;       // A,B x 2 stages = 128 KB

static_assert(kBM == kRowTile && kBN == kColTile, "tiles of the schedule must match the GEMM tile");

enum { OP_KCONTIG = 0, OP_TRANSPOSED = 1 };
enum {
  EPI_STORE = 0,  // C = acc (+ bias)
  EPI_GLU = 1     // act = glu(acc + bias) on interleaved gate/up columns (+ optional pre-activations)
};
enum { PROB_ROWS = 0, PROB_WGRAD = 1 };

struct GemmArgs {
  const void *A;         // PROB_ROWS: [rows, lda] k-contiguous.  PROB_WGRAD: [rows(k), lda] m-contiguous
  const void *B;         // weights of all experts, or [rows(k), ldb] for PROB_WGRAD
  const void *bias;      // [E, Nd] or null
  void *C;               // output
  void *C2;              // EPI_GLU: optional pre-activations [rows, Nd]
  const int *a_rows;     // optional gather of A rows: source row = a_rows[p] / a_div
  const int *sched;      // PROB_ROWS: schedule region
  const int *counts;     // PROB_WGRAD: per-expert counts / offsets
  const int *offsets;
  int a_div;
  int Kd, Nd, Md;        // contraction length, output columns; Md = output rows per expert (PROB_WGRAD)
  int lda, ldb, ldc;     // leading dimensions in elements
  long long b_expert_stride;  // elements between experts in B (PROB_ROWS)
  long long c_expert_stride;  // elements between experts in C (PROB_WGRAD)
  int n_col_tiles, n_row_tiles_wgrad;
  int N, E, capacity;
  // PROB_ROWS + EPI_STORE, optional: dot_part[row][2 * col_tile + wave column] = the fp32 accumulators of the row times
  // dot_with[row][same columns] (a [rows, ldc] tensor), summed over the wave's 128 columns
  const void *dot_with;
  float *dot_part;
};

__device__ inline int lds_swizzle(int row) { return (row ^ (row >> 3)) & 7; }
__device__ inline int lds_chunk_off(int row, int chunk) {
  return row * kRowBytes + ((chunk ^ lds_swizzle(row)) << 4);
}

template <typename T> struct Mma;
template <> struct Mma<bf16_t> {
  __device__ static inline void run(const u32x4 &a, const u32x4 &b, f32x16 &c) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
};
template <> struct Mma<f16_t> {
  __device__ static inline void run(const u32x4 &a, const u32x4 &b, f32x16 &c) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                               __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
};
template <> struct Mma<float> {
  __device__ static inline void run(const u32x4 &a, const u32x4 &b, f32x16 &c) {
    const f32x4 af = __builtin_bit_cast(f32x4, a), bf = __builtin_bit_cast(f32x4, b);
#pragma unroll
    for (int q = 0; q < 4; ++q) c = __builtin_amdgcn_mfma_f32_32x32x2f32(af[q], bf[q], c, 0, 0, 0);
  }
};

// Transpose a VxV block held as V rows of 16 bytes into V columns of 16 bytes.
template <int ESIZE> struct BlockTranspose;
template <> struct BlockTranspose<2> {
  __device__ static inline void run(const u32x4 (&r)[8], u32x4 (&c)[8]) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
#pragma unroll
      for (int d = 0; d < 4; ++d)
        c[j][d] = __builtin_amdgcn_perm(r[2 * d + 1][j >> 1], r[2 * d][j >> 1], sel);
    }
  }
};
template <> struct BlockTranspose<4> {
  // two independent 4x4 blocks: rows 0..3 and rows 4..7
  __device__ static inline void run(const u32x4 (&r)[8], u32x4 (&c)[8]) {
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int d = 0; d < 4; ++d) c[h * 4 + j][d] = r[h * 4 + d][j];
  }
};

// ---- operand loaders -----------------------------------------------------------------------------
// A "tile operand" is 256 rows x one K slab.  fetch() pulls the slab into 8 x 16-byte registers,
// commit() writes them to LDS.  Loads are unconditional at clamped addresses (rows or columns past
// the valid range re-read a valid one; their products are never stored), so the main loop has no
// divergent control flow.  Only the last slab of the contraction can run past k_len; it is fetched
// with TAIL = true, which zero-fills by select.

// k-contiguous rows: thread -> chunk (tid & 7) of rows (tid >> 3) + 32 i.
template <typename T>
struct KContigLoader {
  static constexpr int V = ElemTraits<T>::kVec;
  const char *base;     // wave-uniform
  uint32_t row_off[8];  // byte offset of each of this thread's rows (chunk included) from base
  int chunk, Kd;
  u32x4 regs[8];

  template <bool TAIL>
  __device__ inline void fetch(int k0) {
    const char *slab = base + (long long)k0 * (long long)sizeof(T);
    if (!TAIL) {
#pragma unroll
      for (int i = 0; i < 8; ++i) regs[i] = *(const u32x4 *)(slab + row_off[i]);
    } else {
      const bool ok = k0 + chunk * V < Kd;
      if (!ok) slab = base;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        u32x4 v = *(const u32x4 *)(slab + row_off[i]);
        regs[i] = ok ? v : (u32x4){0, 0, 0, 0};
      }
    }
  }
  __device__ inline void commit(char *lds, int tid) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      int row = (tid >> 3) + 32 * i;
      *(u32x4 *)(lds + lds_chunk_off(row, chunk)) = regs[i];
    }
  }
};

// Operand stored as [k][row] with `row` contiguous: element (k, r) at base + k * ld + r.
// thread -> k-block (lane & 7), row blocks wave*8 + (lane >> 3) (+32 for the second fp32 block).
// The per-lane part of the address is a 32-bit byte offset from a wave-uniform base.
template <typename T, bool GLU_ROWS>
struct TransposedLoader {
  static constexpr int V = ElemTraits<T>::kVec;
  static constexpr int NB = 8 / V;  // row blocks per thread (1 for 16-bit, 2 for fp32)
  const char *base;                 // uniform: (k = 0, row = tile row 0)
  long long ld_bytes;               // uniform
  uint32_t lane_off[NB];            // (kb*V) * ld_bytes + clamped row * sizeof(T)
  int kb, rb, k_valid;
  u32x4 regs[8];

  __device__ inline void setup(const T *b, long long ld, int kb_, int rb_, int k_valid_, int r_valid) {
    base = (const char *)b;
    ld_bytes = ld * (long long)sizeof(T);
    kb = kb_; rb = rb_; k_valid = k_valid_;
#pragma unroll
    for (int h = 0; h < NB; ++h) {
      int r = (rb + 32 * h) * V;
      if (r >= r_valid) r = 0;
      lane_off[h] = (uint32_t)(kb * V) * (uint32_t)ld_bytes + (uint32_t)r * (uint32_t)sizeof(T);
    }
  }
  template <bool TAIL>
  __device__ inline void fetch(int k0) {
    const char *slab = base + (long long)k0 * ld_bytes;
#pragma unroll
    for (int h = 0; h < NB; ++h) {
#pragma unroll
      for (int i = 0; i < V; ++i) {
        if (!TAIL) {
          regs[h * V + i] = *(const u32x4 *)(slab + i * ld_bytes + lane_off[h]);
        } else {
          const bool ok = k0 + kb * V + i < k_valid;
          // a k row past the end re-reads row k0 of the slab (always valid) and is zeroed
          const char *p = ok ? slab + i * ld_bytes + lane_off[h] : slab + (lane_off[h] - (uint32_t)(kb * V) * (uint32_t)ld_bytes);
          u32x4 v = *(const u32x4 *)p;
          regs[h * V + i] = ok ? v : (u32x4){0, 0, 0, 0};
        }
      }
    }
  }
  // LDS row of tile column r: with GLU_ROWS the interleaved (gate, up) columns of each 128-column
  // wave range are split into 64 gate rows followed by 64 up rows.
  __device__ static inline int lds_row(int r) {
    if (!GLU_ROWS) return r;
    int x = r & 127;
    return (r & ~127) | ((x & 1) << 6) | (x >> 1);
  }
  __device__ inline void commit(char *lds) {
    u32x4 cols[8];
    BlockTranspose<sizeof(T)>::run(regs, cols);
#pragma unroll
    for (int h = 0; h < NB; ++h)
#pragma unroll
      for (int j = 0; j < V; ++j) {
        int row = lds_row((rb + 32 * h) * V + j);
        *(u32x4 *)(lds + lds_chunk_off(row, kb)) = cols[h * V + j];
      }
  }
};

// Everything a workgroup knows about its tile.
struct TileInfo {
  int expert, row0, rows_valid, n0, k_len, m0;
  long long a_first;
};

// The contraction loop and the epilogue, specialised on NMI = number of 32-row blocks this wave
// owns (0..4; partial tiles at the end of an expert's rows own fewer).
template <typename T, int A_KIND, int B_KIND, int EPI, int PROB, int NMI, class LA, class LB>
__device__ inline void run_tile(const GemmArgs &args, const TileInfo &ti, LA &la, LB &lb, char *lds) {
  constexpr int BK = kRowBytes / (int)sizeof(T);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  constexpr int NACC = NMI > 0 ? NMI : 1;

  f32x16 acc[NACC][4];
#pragma unroll
  for (int mi = 0; mi < NACC; ++mi)
#pragma unroll
    for (int ni = 0; ni < 4; ++ni)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[mi][ni][v] = 0.0f;

  const int n_slabs = (ti.k_len + BK - 1) / BK;

  auto commit = [&](int buf) {
    char *tA = lds + buf * (2 * kTileBytes), *tB = tA + kTileBytes;
    if constexpr (A_KIND == OP_KCONTIG) la.commit(tA, tid); else la.commit(tA);
    if constexpr (B_KIND == OP_KCONTIG) lb.commit(tB, tid); else lb.commit(tB);
  };
  // MFMA operands of k-step ks+1 are read from LDS while the MFMAs of k-step ks run; the scheduling
  // barriers keep the compiler from sinking the reads next to their first use.
  auto load_frags = [&](const char *tA, const char *tB, int ks, u32x4 (&af)[NACC], u32x4 (&bf)[4]) {
    const int chunk = ks * 2 + (lane >> 5);
#pragma unroll
    for (int ni = 0; ni < 4; ++ni) {
      int row = wn * 128 + ni * 32 + (lane & 31);
      bf[ni] = *(const u32x4 *)(tB + lds_chunk_off(row, chunk));
    }
#pragma unroll
    for (int mi = 0; mi < NMI; ++mi) {
      int row = (mi * 2 + wm) * 32 + (lane & 31);
      af[mi] = *(const u32x4 *)(tA + lds_chunk_off(row, chunk));
    }
  };
  auto mma = [&](const u32x4 (&af)[NACC], const u32x4 (&bf)[4]) {
#pragma unroll
    for (int mi = 0; mi < NMI; ++mi)
#pragma unroll
      for (int ni = 0; ni < 4; ++ni) Mma<T>::run(af[mi], bf[ni], acc[mi][ni]);
  };
  auto compute = [&](int buf) {
    const char *tA = lds + buf * (2 * kTileBytes), *tB = tA + kTileBytes;
    u32x4 af0[NACC], bf0[4], af1[NACC], bf1[4];
    load_frags(tA, tB, 0, af0, bf0);
    __builtin_amdgcn_sched_barrier(0);
    load_frags(tA, tB, 1, af1, bf1);
    mma(af0, bf0);
    __builtin_amdgcn_sched_barrier(0);
    load_frags(tA, tB, 2, af0, bf0);
    mma(af1, bf1);
    __builtin_amdgcn_sched_barrier(0);
    load_frags(tA, tB, 3, af1, bf1);
    mma(af0, bf0);
    __builtin_amdgcn_sched_barrier(0);
    mma(af1, bf1);
    __builtin_amdgcn_sched_barrier(0);
  };

  if (n_slabs > 0) {
    if (n_slabs == 1) { la.template fetch<true>(0); lb.template fetch<true>(0); }
    else { la.template fetch<false>(0); lb.template fetch<false>(0); }
    commit(0);
  }
  __syncthreads();
  int s = 0;
  for (; s + 2 < n_slabs; ++s) {  // slab s+1 is a full one
    la.template fetch<false>((s + 1) * BK);
    lb.template fetch<false>((s + 1) * BK);
    __builtin_amdgcn_sched_barrier(0);  // the loads of the next slab are issued before this slab's MFMAs
    compute(s & 1);
    commit((s & 1) ^ 1);
    __syncthreads();
  }
  if (s + 1 < n_slabs) {  // slab s+1 is the last one and may be partial
    la.template fetch<true>((s + 1) * BK);
    lb.template fetch<true>((s + 1) * BK);
    __builtin_amdgcn_sched_barrier(0);
    compute(s & 1);
    commit((s & 1) ^ 1);
    __syncthreads();
    ++s;
  }
  if (s < n_slabs) compute(s & 1);

  if constexpr (NMI == 0) return;

  // ---- epilogue -------------------------------------------------------------------------------------
  // acc[mi][ni][v]: tile row (mi*2+wm)*32 + 8*(v/4) + 4*(lane/32) + v%4, LDS column row wn*128 + ni*32 + lane%32
  const int lcol = lane & 31;
  const int rsub = (lane >> 5) * 4;
  const int expert = ti.expert, rows_valid = ti.rows_valid, n0 = ti.n0;
  const long long out_row0 = (PROB == PROB_WGRAD) ? ti.m0 : ti.row0;
  const bool full = rows_valid == kBM && n0 + kBN <= args.Nd;
  if constexpr (EPI == EPI_STORE && PROB == PROB_ROWS) {
    // Row dots of the product with a second tensor of the output's shape, from the fp32 accumulators (the routing
    // gradient <grad_out . W_down^T, act>, csrc/experts_backward.cu:83-88): one partial sum per valid row and wave,
    // over the wave's 128 columns of the tile.
    if (args.dot_part != nullptr) {
      const int n_part = 2 * args.n_col_tiles, part_col = 2 * (n0 / kBN) + wn;
#pragma unroll
      for (int mi = 0; mi < NMI; ++mi) {
        float part[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int r = (mi * 2 + wm) * 32 + 8 * (v >> 2) + rsub + (v & 3);
          const T *wp = (const T *)args.dot_with + (out_row0 + min(r, rows_valid - 1)) * args.ldc;
          float sum = 0.0f;
#pragma unroll
          for (int ni = 0; ni < 4; ++ni) {
            const int col = n0 + wn * 128 + ni * 32 + lcol;
            if (col < args.Nd) sum += acc[mi][ni][v] * ElemTraits<T>::to_f32(wp[col]);
          }
          part[v] = sum;
        }
#pragma unroll
        for (int d = 1; d < 32; d <<= 1)
#pragma unroll
          for (int v = 0; v < 16; ++v) part[v] += __shfl_xor(part[v], d);
        if (lcol == 0) {
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const int r = (mi * 2 + wm) * 32 + 8 * (v >> 2) + rsub + (v & 3);
            if (r < rows_valid) args.dot_part[(out_row0 + r) * n_part + part_col] = part[v];
          }
        }
      }
    }
  }
  if constexpr (EPI == EPI_STORE) {
    T *C = (T *)args.C + ((PROB == PROB_WGRAD) ? (long long)expert * args.c_expert_stride : 0);
#pragma unroll
    for (int ni = 0; ni < 4; ++ni) {
      int col = n0 + wn * 128 + ni * 32 + lcol;
      bool col_ok = col < args.Nd;
      float bias = 0.0f;
      if (args.bias != nullptr && col_ok)
        bias = ElemTraits<T>::to_f32(((const T *)args.bias)[(long long)expert * args.Nd + col]);
#pragma unroll
      for (int mi = 0; mi < NMI; ++mi) {
        T *Cp = C + (out_row0 + (mi * 2 + wm) * 32 + rsub) * args.ldc + col;
        if (full) {
#pragma unroll
          for (int v = 0; v < 16; ++v)
            Cp[(long long)(8 * (v >> 2) + (v & 3)) * args.ldc] = ElemTraits<T>::from_f32(acc[mi][ni][v] + bias);
        } else {
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            int r = (mi * 2 + wm) * 32 + 8 * (v >> 2) + rsub + (v & 3);
            if (col_ok && r < rows_valid)
              Cp[(long long)(8 * (v >> 2) + (v & 3)) * args.ldc] = ElemTraits<T>::from_f32(acc[mi][ni][v] + bias);
          }
        }
      }
    }
  } else {
    // gate columns live in ni = 0,1 and the matching up columns in ni = 2,3
    T *C = (T *)args.C;
    T *P = (T *)args.C2;
#pragma unroll
    for (int np = 0; np < 2; ++np) {
      int pair = (n0 + wn * 128) / 2 + np * 32 + lcol;  // index of the (gate, up) pair = act column
      bool col_ok = 2 * pair + 1 < args.Nd;
      float bg = 0.0f, bu = 0.0f;
      if (args.bias != nullptr && col_ok) {
        const T *bp = (const T *)args.bias + (long long)expert * args.Nd + 2 * pair;
        bg = ElemTraits<T>::to_f32(bp[0]);
        bu = ElemTraits<T>::to_f32(bp[1]);
      }
#pragma unroll
      for (int mi = 0; mi < NMI; ++mi) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          int r = (mi * 2 + wm) * 32 + 8 * (v >> 2) + rsub + (v & 3);
          if (full || (col_ok && r < rows_valid)) {
            long long orow = out_row0 + r;
            float G = acc[mi][np][v] + bg, U = acc[mi][np + 2][v] + bu;
            C[orow * args.ldc + pair] = ElemTraits<T>::from_f32(glu_forward(G, U));
            if (P != nullptr) {
              P[orow * args.Nd + 2 * pair] = pre_activation_store<T>(G, false);
              P[orow * args.Nd + 2 * pair + 1] = pre_activation_store<T>(U, true);
            }
          }
        }
      }
    }
  }
}

template <typename T, int A_KIND, int B_KIND, int EPI, int PROB, bool GATHER>
__global__ __launch_bounds__(kGemmThreads) void grouped_gemm_kernel(const GemmArgs args) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  constexpr int V = ElemTraits<T>::kVec;
  constexpr bool GLU_ROWS = EPI == EPI_GLU;
  static_assert(!(EPI == EPI_GLU) || B_KIND == OP_TRANSPOSED, "GLU epilogue expects [K,N] weights");

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1;

  // ---- which tile -------------------------------------------------------------------------------
  TileInfo ti;
  ti.a_first = 0;
  ti.m0 = 0;
  {
    int n_row_tiles = (PROB == PROB_ROWS) ? args.sched[0] : args.E * args.n_row_tiles_wgrad;
    int total = n_row_tiles * args.n_col_tiles;
    int total8 = (total + kXcds - 1) / kXcds * kXcds;
    int b = blockIdx.x;
    if (b >= total8) return;
    int L = (b % kXcds) * (total8 / kXcds) + b / kXcds;
    if (L >= total) return;
    int col_tile;
    if (PROB == PROB_ROWS) {
      const int *tiles = args.sched + kSchedHeader;
      int t0 = L / args.n_col_tiles;
      int gfirst = tiles[8 * t0 + 3], gcount = tiles[8 * t0 + 4];
      int local = L - gfirst * args.n_col_tiles;
      col_tile = local / gcount;
      const int *te = tiles + 8 * (gfirst + local % gcount);
      ti.expert = te[0]; ti.row0 = te[1]; ti.rows_valid = te[2];
      ti.k_len = args.Kd;
    } else {
      int per_expert = args.n_row_tiles_wgrad * args.n_col_tiles;
      ti.expert = L / per_expert;
      int local = L - ti.expert * per_expert;
      col_tile = local / args.n_row_tiles_wgrad;
      ti.m0 = (local % args.n_row_tiles_wgrad) * kBM;
      ti.row0 = 0;
      ti.rows_valid = min(kBM, args.Md - ti.m0);
      ti.k_len = min(args.counts[ti.expert], args.capacity);
      ti.a_first = args.offsets[ti.expert];
    }
    ti.n0 = col_tile * kBN;
  }

  // ---- loaders ------------------------------------------------------------------------------------
  typedef typename std::conditional<A_KIND == OP_KCONTIG, KContigLoader<T>, TransposedLoader<T, false>>::type LA;
  typedef typename std::conditional<B_KIND == OP_KCONTIG, KContigLoader<T>, TransposedLoader<T, GLU_ROWS>>::type LB;
  LA la;
  LB lb;
  if constexpr (A_KIND == OP_KCONTIG) {
    la.chunk = tid & 7;
    la.Kd = ti.k_len;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      int r = min((tid >> 3) + 32 * i, ti.rows_valid - 1);
      // byte offsets fit 32 bits: rows of a tile are near its first row, and gathered sources are
      // checked on the host to span less than 4 GB
      long long src = r;
      if (GATHER && args.a_rows != nullptr) src = args.a_rows[ti.row0 + r] / args.a_div;
      la.row_off[i] = (uint32_t)((src * args.lda + (tid & 7) * V) * (long long)sizeof(T));
    }
    // (a gathering instantiation without a row list reads its rows in order: see gemm_async.hip)
    la.base = (const char *)((const T *)args.A + (GATHER && args.a_rows != nullptr ? 0ll : (long long)ti.row0 * args.lda));
  } else {
    la.setup((const T *)args.A + ti.a_first * args.lda + ti.m0, args.lda, lane & 7, wave * 8 + (lane >> 3), ti.k_len,
             ti.rows_valid);
  }
  if constexpr (B_KIND == OP_KCONTIG) {
    // B element (k, n) at B[expert][n][k]: rows are output columns
    const T *bb = (const T *)args.B + (long long)ti.expert * args.b_expert_stride;
    lb.chunk = tid & 7;
    lb.Kd = ti.k_len;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      int n = min(ti.n0 + (tid >> 3) + 32 * i, args.Nd - 1);
      lb.row_off[i] = (uint32_t)(((long long)n * args.ldb + (tid & 7) * V) * (long long)sizeof(T));
    }
    lb.base = (const char *)bb;
  } else {
    const T *bb = (PROB == PROB_ROWS) ? (const T *)args.B + (long long)ti.expert * args.b_expert_stride + ti.n0
                                      : (const T *)args.B + ti.a_first * args.ldb + ti.n0;
    lb.setup(bb, args.ldb, lane & 7, wave * 8 + (lane >> 3), ti.k_len, args.Nd - ti.n0);
  }

  // 32-row blocks of the tile are dealt alternately to the two wave rows; blocks past the valid
  // rows are skipped.  The branch is uniform per wave, and every wave of the workgroup runs the
  // same number of slabs and barriers whatever its block count.
  const int n_blocks32 = (ti.rows_valid + 31) >> 5;
  const int n_mi = (n_blocks32 - wm + 1) >> 1;
  switch (n_mi) {
    case 4: run_tile<T, A_KIND, B_KIND, EPI, PROB, 4>(args, ti, la, lb, lds); break;
    case 3: run_tile<T, A_KIND, B_KIND, EPI, PROB, 3>(args, ti, la, lb, lds); break;
    case 2: run_tile<T, A_KIND, B_KIND, EPI, PROB, 2>(args, ti, la, lb, lds); break;
    case 1: run_tile<T, A_KIND, B_KIND, EPI, PROB, 1>(args, ti, la, lb, lds); break;
    default: run_tile<T, A_KIND, B_KIND, EPI, PROB, 0>(args, ti, la, lb, lds); break;
  }
}

// Experts that own no kept rows need no special case in the weight-gradient product: k_len = 0
// leaves the accumulators at zero and the epilogue stores them.

template <typename T, int A_KIND, int B_KIND, int EPI, int PROB, bool GATHER>
static int launch_gemm(const GemmArgs &args, int max_row_tiles, hipStream_t stream) {
  auto kernel = grouped_gemm_kernel<T, A_KIND, B_KIND, EPI, PROB, GATHER>;
  static DeviceFlags attr_done;  // one per kernel instantiation
  if (int rc = ensure_dynamic_lds((const void *)kernel, kGemmLds, attr_done, "grouped_gemm_kernel")) return rc;
  long long total = (long long)max_row_tiles * args.n_col_tiles;
  if (total <= 0) return 0;
  total = (total + kXcds - 1) / kXcds * kXcds;
  hipLaunchKernelGGL(kernel, dim3((unsigned)total), dim3(kGemmThreads), kGemmLds, stream, args);
  return check_launch("grouped_gemm_kernel");
}

template <typename T>
int gemm_gate_up(const void *x, const int *sorted_idx, const void *w, const void *bias, void *act, void *pre,
                 const void *sched, int N, int K, int E, int H, int I, hipStream_t stream) {
  GemmArgs a = {};
  a.A = x; a.B = w; a.bias = bias; a.C = act; a.C2 = pre;
  a.a_rows = sorted_idx; a.a_div = K; a.sched = (const int *)sched;
  a.Kd = H; a.Nd = 2 * I; a.lda = H; a.ldb = 2 * I; a.ldc = I;
  a.b_expert_stride = (long long)H * 2 * I;
  a.n_col_tiles = ceil_div(2 * I, kBN);
  a.N = N; a.E = E;
  return launch_gemm<T, OP_KCONTIG, OP_TRANSPOSED, EPI_GLU, PROB_ROWS, true>(a, sched_max_row_tiles(N, E), stream);
}

template <typename T>
int gemm_down(const void *act, const void *w, const void *bias, void *y, const void *sched, int N, int E, int H,
              int I, hipStream_t stream) {
  GemmArgs a = {};
  a.A = act; a.B = w; a.bias = bias; a.C = y; a.sched = (const int *)sched;
  a.Kd = I; a.Nd = H; a.lda = I; a.ldb = H; a.ldc = H;
  a.b_expert_stride = (long long)I * H;
  a.n_col_tiles = ceil_div(H, kBN);
  a.N = N; a.E = E;
  return launch_gemm<T, OP_KCONTIG, OP_TRANSPOSED, EPI_STORE, PROB_ROWS, false>(a, sched_max_row_tiles(N, E), stream);
}

// d_out[p,:] = g[p,:] . W[e]^T with W[e] = [n_out, k] row-major, i.e. k-contiguous "B rows".  With g_rows the
// source row of p is g_rows[p] / g_div (rows of a [T, Kd] tensor gathered by token).
template <typename T>
int gemm_dgrad(const void *g, const int *g_rows, int g_div, const void *w, void *d_out, const void *sched, int N, int E,
               int Kd, int Nd, const void *dot_with, float *dot_part, hipStream_t stream) {
  GemmArgs a = {};
  a.A = g; a.B = w; a.C = d_out; a.sched = (const int *)sched;
  a.dot_with = dot_with; a.dot_part = dot_part;
  a.a_rows = g_rows; a.a_div = g_div;
  a.Kd = Kd; a.Nd = Nd; a.lda = Kd; a.ldb = Kd; a.ldc = Nd;
  a.b_expert_stride = (long long)Nd * Kd;
  a.n_col_tiles = ceil_div(Nd, kBN);
  a.N = N; a.E = E;
  if (g_rows != nullptr)
    return launch_gemm<T, OP_KCONTIG, OP_KCONTIG, EPI_STORE, PROB_ROWS, true>(a, sched_max_row_tiles(N, E), stream);
  return launch_gemm<T, OP_KCONTIG, OP_KCONTIG, EPI_STORE, PROB_ROWS, false>(a, sched_max_row_tiles(N, E), stream);
}

// dW[e] = L_e^T . R_e over the expert's kept rows: L [rows, Md], R [rows, Nd], dW [E, Md, Nd].
template <typename T>
int gemm_wgrad(const void *L, const void *R, void *dW, const int *counts, const int *offsets, int capacity, int E,
               int Md, int Nd, hipStream_t stream) {
  GemmArgs a = {};
  a.A = L; a.B = R; a.C = dW; a.counts = counts; a.offsets = offsets; a.capacity = capacity;
  a.Md = Md; a.Nd = Nd; a.lda = Md; a.ldb = Nd; a.ldc = Nd;
  a.c_expert_stride = (long long)Md * Nd;
  a.n_col_tiles = ceil_div(Nd, kBN);
  a.n_row_tiles_wgrad = ceil_div(Md, kBM);
  a.E = E;
  return launch_gemm<T, OP_TRANSPOSED, OP_TRANSPOSED, EPI_STORE, PROB_WGRAD, false>(a, E * a.n_row_tiles_wgrad, stream);
}

#define YAMOE_INSTANTIATE_GEMM(T)                                                                                   \
  template int gemm_gate_up<T>(const void *, const int *, const void *, const void *, void *, void *, const void *, \
                               int, int, int, int, int, hipStream_t);                                               \
  template int gemm_down<T>(const void *, const void *, const void *, void *, const void *, int, int, int, int,     \
                            hipStream_t);                                                                           \
  template int gemm_dgrad<T>(const void *, const int *, int, const void *, void *, const void *, int, int, int, int, \
                             const void *, float *, hipStream_t);                                                   \
  template int gemm_wgrad<T>(const void *, const void *, void *, const int *, const int *, int, int, int, int,      \
                             hipStream_t);
YAMOE_INSTANTIATE_GEMM(float)
YAMOE_INSTANTIATE_GEMM(bf16_t)
YAMOE_INSTANTIATE_GEMM(f16_t)

}  // namespace yamoe
