// Grouped expert GEMMs for 16-bit data on gfx950, asynchronous-copy pipeline.
//
// Same tiling as gemm.hip (256x256 output tile, 4 wavefronts 2x2, 32x32x16 MFMA, fp32 accumulate)
// but operands never pass through vector registers on their way to LDS:
//
//  * Global -> LDS copies are `global_load_lds_dwordx4`: every lane names its own 16-byte source and
//    the 64 lanes of a wave fill 1 KB of LDS in lane order.  The contraction is cut into slabs of
//    32; the forward's weight slabs rotate through four buffers of 16 KB and are requested three to four
//    slabs (about 3000 MFMA cycles) before they are consumed, which covers HBM latency with one wave
//    per SIMD; the activation rows rotate through two buffers of a slab pair (32 KB) each.
//  * An operand whose rows are k-contiguous in memory ([row][k]) keeps that layout in LDS and is read
//    with one 16-byte ds_read per MFMA operand.  Such operands are copied two slabs at a time (128
//    bytes of a row per copy), so that every request to L2 is a whole cache line: with 64-byte pieces
//    the same kernel makes 1.5 times the L2 requests and runs 10-15 % slower.
//  * [n][k] weights (the input-gradient products) are such an operand too: their B ring is three slab
//    pairs (160 KB of LDS with the A ring), the copies are spread four per wave over every k-step and
//    only every second slab needs a wait and a workgroup barrier.
//  * The forward weights are [k][n] in memory and stay [k][n] in LDS (512 bytes per k row);
//    MFMA operands are read with `ds_read_b64_tr_b16`, the LDS transpose read of gfx950, which
//    hands lane i of a 16-lane group column n0+i for 4 consecutive k.  No register transpose, no
//    LDS store instruction, no staging registers.
//  * LDS swizzles are applied on the global side (a lane picks which 16-byte piece it fetches), as
//    the LDS side of an asynchronous copy is fixed to lane order:
//        [row][k] tiles: piece c (0..7, two slabs) of row r sits at position c ^ ((r >> 1) & 7)
//        [k][n]  tiles: piece c of row k sits at position c ^ ((k & 3) << 2)
//    so that both kinds of MFMA operand reads touch every bank once.
//  * Software pipeline per slab (two k-steps of 16): the operands of the second k-step are read
//    while the MFMAs of the first run; then the wave waits for the next slab's copies, one
//    workgroup barrier, the freed buffer is re-filled with slab s+4, the first operands of slab
//    s+1 are read, and the MFMAs of the second k-step run.  All LDS and HBM latency sits behind
//    MFMAs; only the barrier itself is exposed.
//
// The MFMAs take the weights as their first operand, so that a lane's accumulators are one output row
// and runs of four consecutive columns: the interleaved (gate, up) columns of the clamped SwiGLU
// (csrc/moe.cpp:164-180) meet in one lane, and the staging stores are 4 or 8 bytes wide.
//
// Requirements: contraction length a multiple of 64, leading dimensions multiples of 8 elements.
// Other shapes and fp32 use gemm.hip.
#include <type_traits>

#include "common.h"

namespace yamoe {

namespace async {

constexpr int kBM = 256, kBN = 256, kBK = 32;
constexpr int kThreads = 256;
constexpr int kBandRows = 8;  // row tiles of one band of an expert with many row tiles (see gemm_async_kernel)
constexpr int kAStages = 2, kAStageBytes = 32768;  // A ring: pairs of slabs (256 rows x 128 B)
constexpr int kBStages = 4, kBStageBytes = 16384;  // B ring: single slabs (32 k rows x 512 B)
constexpr int kBRing = kAStages * kAStageBytes;    // byte offset of the B ring
constexpr int kRingBytes = kBRing + kBStages * kBStageBytes;  // 128 KB
constexpr int kStagingBytes = kBM * (kBN * 2 + 16);            // output tile staged for the row-wise store
constexpr int kBiasOff = kStagingBytes > kRingBytes ? kStagingBytes : kRingBytes;  // the tile's 256 bias values
constexpr int kLds = kBiasOff + kBN * 2;
// [n][k] weights (the input-gradient products) keep B in slab pairs as well, three of them: 160 KB with the A ring
constexpr int kBPairStages = 3, kBPairBytes = 32768;
constexpr int kLdsNk = kBRing + kBPairStages * kBPairBytes;

static_assert(kBM == kRowTile && kBN == kColTile, "tiles of the schedule must match the GEMM tile");

enum { EPI_STORE = 0, EPI_GLU = 1 };

struct Args {
  const void *A;        // [rows, lda], k-contiguous
  const void *B;        // [E, Kd, Nd] ([k][n] per expert)
  const void *bias;     // [E, Nd] or null
  void *C;              // EPI_STORE: [rows, ldc]; EPI_GLU: act [rows, Nd/2]
  void *C2;             // EPI_GLU: optional pre-activations [rows, Nd]
  const int *a_rows;    // optional gather of A rows: source row = a_rows[p] / a_div
  const int *sched;
  FastDiv a_div, n_col_div;  // divisions by the gather divisor and by n_col_tiles
  FastDiv band_div;          // division by kBandRows * n_col_tiles
  int Kd, Nd, lda, ldb, ldc, n_col_tiles;
  long long b_expert_stride;
  // EPI_STORE with [n][k] weights, optional: dot_part[row][2 * col_tile + wave column] = the fp32 accumulators of the
  // row times dot_with[row][same columns] (a [rows, ldc] tensor), summed over the wave's 128 columns
  const void *dot_with;
  float *dot_part;
#ifdef YAMOE_TILE_STAMPS
  unsigned long long *stamps;  // [stamps_cap][8]: see yamoe_debug_tile_stamps
  int stamps_cap;
#endif
};

#ifdef YAMOE_TILE_STAMPS
// Diagnostic build (-DYAMOE_TILE_STAMPS, `python -m yamoe_amd.tile_stamps`): thread 0 of every tile of gemm_async_kernel
// leaves eight words at stamps[8 * flat tile index]: the shader clock (s_memtime) at workgroup entry, before the first
// copy, when the first slab has landed, after the contraction loop, before the row-wise stores and at the end, then
// valid rows | valid columns << 16, and where it ran (XCC id << 8 | SE, SH and CU id).
#define YAMOE_STAMP(i) if (tid == 0) stamp_reg[i] = __builtin_amdgcn_s_memtime()
#else
#define YAMOE_STAMP(i)
#endif

template <typename T> struct Mma;
template <> struct Mma<bf16_t> {
  __device__ static inline void run(const u32x4 &a, const u32x4 &b, f32x16 &c) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
};
template <> struct Mma<f16_t> {
  __device__ static inline void run(const u32x4 &a, const u32x4 &b, f32x16 &c) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
};

// two fp32 values rounded to T, packed low / high
template <typename T> __device__ inline uint32_t pack2(float lo, float hi) {
  typedef T T2 __attribute__((ext_vector_type(2)));
  T2 v = {ElemTraits<T>::from_f32(lo), ElemTraits<T>::from_f32(hi)};
  return __builtin_bit_cast(uint32_t, v);
}
// four consecutive elements of T (8-byte aligned) as fp32
template <typename T> __device__ inline void load4_f32(const T *p, float (&out)[4]) {
  typedef T T4 __attribute__((ext_vector_type(4)));
  T4 v = *(const T4 *)p;
#pragma unroll
  for (int i = 0; i < 4; ++i) out[i] = ElemTraits<T>::to_f32(v[i]);
}

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;

// LDS transpose read: lane i of each 16-lane group receives, for j = 0..3, the 16-bit element
// (i % 4) of the 8 bytes addressed by lane 4*j + i/4 of the group.
__device__ inline u32x2 lds_read_tr16(const char *p) {
  s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)p);
  return __builtin_bit_cast(u32x2, v);
}

template <int N> __device__ inline void wait_vmcnt() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }

// what one slab step of the pipeline issues besides its MFMAs
template <bool P1A_, bool P1B_, bool P2A_, bool P2B_, bool NEXT_, int VM_, bool BAR_ = true> struct StepCfg {
  static constexpr bool P1A = P1A_, P1B = P1B_, P2A = P2A_, P2B = P2B_, NEXT = NEXT_, BAR = BAR_;
  static constexpr int VM = VM_;
};

struct TileInfo {
  int expert, row0, rows_valid, n0;
#ifdef YAMOE_TILE_STAMPS
  int slot;
  unsigned long long t_entry, t_lookup;
#endif
};

// NMI / NNI: how many of this wave's four 32-row and four 32-column blocks of the tile hold valid rows / columns.  The
// 32-column blocks alternate between the two wave columns (block cb belongs to wave column cb & 1), so a tile of 64
// or 128 valid columns (the last column tile of a 2880-wide matrix) gives both wave columns a quarter or half of the
// MFMAs instead of all of them to one.
// NAB: how many of the tile's eight 32-row blocks are copied (the others hold no valid row).
template <typename T, int EPI, int NMI, bool BNK, int NNI = 4, int NAB = 8>
__device__ __forceinline__ void run_tile(const Args &args, const TileInfo &ti, const int tid, const char *a_base,
                                const uint32_t (&a_off)[8], const char *b_base, const uint32_t (&b_off)[8],
                                long long b_slab_bytes) {
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform, kept in a scalar register
  const int wm = wave >> 1, wn = wave & 1;
  constexpr int NACC = NMI > 0 ? NMI : 1;
  extern __shared__ __attribute__((aligned(16))) char lds[];
  const uint32_t lds0 = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)lds);  // LDS byte address of the A ring

  f32x16 acc[NACC][4];
#pragma unroll
  for (int mi = 0; mi < NACC; ++mi)
#pragma unroll
    for (int ni = 0; ni < 4; ++ni)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[mi][ni][v] = 0.0f;

  const int n_slabs = args.Kd / kBK;  // even: the contraction length is a multiple of 64
#ifdef YAMOE_TILE_STAMPS
  unsigned long long stamp_reg[6] = {ti.t_entry, ti.t_lookup, 0, 0, 0, 0};
#endif

  // The tile's bias values, one per thread, requested before anything else: they are the oldest entry of the memory
  // queue, so the first wait of the pipeline covers them, and the epilogue finds them in a register instead of
  // paying a memory latency per column block.  ([n][k] weights are the input-gradient products: no bias.)
  const bool has_bias = !BNK && args.bias != nullptr;
  T bias_reg = ElemTraits<T>::from_f32(0.0f);
  if (has_bias) bias_reg = ((const T *)args.bias)[(long long)ti.expert * args.Nd + min(ti.n0 + tid, args.Nd - 1)];

  // ---- copy issue ----------------------------------------------------------------------------------
  // A pair p (slabs 2p, 2p+1): copy i is the 32-row block i of the tile, this wave fills its rows 8*wave + (lane >> 3),
  // 128 bytes each.  Blocks without valid rows (i >= n_ablk) are not copied: nobody reads them, and a tile of 192 rows,
  // the common one, moves an eighth less through the L1 than a full one.  (The count is a template parameter: a
  // run-time test around every copy and a run-time wait count cost more than the copies saved.)
  constexpr int n_ablk = NAB;
  auto issue_a = [&](int pair) {
    const uint32_t stage = lds0 + (uint32_t)(pair & (kAStages - 1)) * kAStageBytes;
    const char *ab = a_base + (long long)pair * (2 * kBK * (int)sizeof(T));
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if (i < n_ablk) copy16_to_lds(ab, a_off[i], stage + (uint32_t)(32 * i + 8 * wave) * 128u);
  };
  // B slab: this wave fills k rows 8*wave + 2*i + (lane >> 5), 512 bytes each.
  auto issue_b = [&](int slab) {
    const uint32_t stage = lds0 + kBRing + (uint32_t)(slab & (kBStages - 1)) * kBStageBytes;
    const char *bb = b_base + (long long)slab * b_slab_bytes;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      copy16_to_lds(bb, b_off[i], stage + (uint32_t)(8 * wave + 2 * i) * 512u);
  };

  // ---- MFMA operand reads ----------------------------------------------------------------------------
  // A operand (block mi, slab parity par, k-step ks): row (mi*2+wm)*32 + lane%32, piece par*4 + ks*2 + lane/32
  // at position piece ^ ((row >> 1) & 7).
  const int rl = lane & 31, g = lane >> 5;
  int a_rd[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) a_rd[ks] = (wm * 32 + rl) * 128 + (((ks * 2 + g) ^ ((rl >> 1) & 7)) << 4);
  // B operand (column block ni, k-step ks, half h): k = ks*16 + g*8 + h*4 + j, 4 columns at
  // (ni*2+wn)*32 + 16*((lane>>4)&1) + 4*q, where j = (lane&15)>>2 and q = lane&3.
  const int j4 = (lane & 15) >> 2, q4 = lane & 3;
  int b_rd[4];
#pragma unroll
  for (int ni = 0; ni < 4; ++ni) {
    int col = (ni * 2 + wn) * 32 + 16 * ((lane >> 4) & 1) + 4 * q4;
    int piece = (col >> 3) ^ (j4 << 2);
    b_rd[ni] = (g * 8 + j4) * 512 + (piece << 4) + (col & 7) * 2;
  }
  // B operand of a [n][k] tile (BNK): stored like A, in slab pairs of 128-byte rows; row (ni*2+wn)*32 + lane%32,
  // one 16-byte read per operand.
  int b_rdk[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) b_rdk[ks] = (wn * 32 + rl) * 128 + (((ks * 2 + g) ^ ((rl >> 1) & 7)) << 4);

  u32x4 fa0[NACC], fa1[NACC], fb0[4], fb1[4];
  // Operand fragments of one k-step in the order the MFMAs want them: B0, A0, B1, B2, B3, A1, A2, A3.
  // Slab s sits in A pair buffer (s>>1)&1 (the odd slab of a pair 64 bytes further, by XOR) and B buffer s&3.
  constexpr int kFrags = NMI > 0 ? NNI + NMI : 0;
  auto read_frag = [&](int s, int ks, int f, u32x4 (&fa)[NACC], u32x4 (&fb)[4]) {
    if (f == 1 || f >= 1 + NNI) {
      const int mi = f == 1 ? 0 : f - NNI;
      const char *sa = lds + ((s >> 1) & (kAStages - 1)) * kAStageBytes;
      fa[mi] = *(const u32x4 *)(sa + (a_rd[ks] ^ ((s & 1) << 6)) + mi * 8192);
    } else {
      const int ni = f == 0 ? 0 : f - 1;
      if constexpr (BNK) {
        const char *sb = lds + kBRing + ((s >> 1) % kBPairStages) * kBPairBytes;
        fb[ni] = *(const u32x4 *)(sb + (b_rdk[ks] ^ ((s & 1) << 6)) + ni * 8192);
      } else {
        const char *sb = lds + kBRing + (s & (kBStages - 1)) * kBStageBytes;
        u32x2 lo = lds_read_tr16(sb + b_rd[ni] + ks * 8192);
        u32x2 hi = lds_read_tr16(sb + b_rd[ni] + ks * 8192 + 2048);
        fb[ni] = (u32x4){lo[0], lo[1], hi[0], hi[1]};
      }
    }
  };
  auto read_frags = [&](int s, int ks, u32x4 (&fa)[NACC], u32x4 (&fb)[4]) {
#pragma unroll
    for (int f = 0; f < kFrags; ++f) read_frag(s, ks, f, fa, fb);
  };
  auto mma = [&](const u32x4 (&fa)[NACC], const u32x4 (&fb)[4]) {
#pragma unroll
    for (int mi = 0; mi < NMI; ++mi)
#pragma unroll
      for (int ni = 0; ni < NNI; ++ni) Mma<T>::run(fb[ni], fa[mi], acc[mi][ni]);
  };
  // One 16-byte-per-lane copy: piece c (0..7) of A pair `pair`, or piece i (0..3) of B slab `slab`.
  auto copy_a = [&](int pair, int c) {
    if (c < n_ablk)
      copy16_to_lds(a_base + (long long)pair * (2 * kBK * (int)sizeof(T)), a_off[c],
                    lds0 + (uint32_t)(pair & (kAStages - 1)) * kAStageBytes + (uint32_t)(32 * c + 8 * wave) * 128u);
  };
  auto copy_b = [&](int slab, int i) {
    copy16_to_lds(b_base + (long long)slab * b_slab_bytes, b_off[i],
                  lds0 + kBRing + (uint32_t)(slab & (kBStages - 1)) * kBStageBytes + (uint32_t)(8 * wave + 2 * i) * 512u);
  };
  // [n][k] weights: piece c (0..7) of B pair `pair`, rows 64*wave + 8*c + (lane >> 3) like A
  auto copy_bp = [&](int pair, int c) {
    copy16_to_lds(b_base + (long long)pair * (2 * b_slab_bytes), b_off[c],
                  lds0 + kBRing + (uint32_t)(pair % kBPairStages) * kBPairBytes + (uint32_t)(64 * wave + 8 * c) * 128u);
  };
  auto issue_bp = [&](int pair) {
#pragma unroll
    for (int c = 0; c < 8; ++c) copy_bp(pair, c);
  };

  // ---- pipeline -----------------------------------------------------------------------------------------
  // A slab is two k-steps with one workgroup barrier between them; after the barrier of slab t nobody reads
  // slab t's buffers any more.  The L1 path moves 64 bytes per clock into LDS and a slab needs 32 KB of
  // copies against 1024 clocks of MFMAs, so the copies are spread as evenly as the buffer lifetimes allow:
  //   second k-step of slab t:  (t odd) first half of A pair (t+1)/2 + 1;  first half of B slab t + 4
  //   first k-step of slab t:   (t even) second half of A pair t/2 + 1;    second half of B slab t + 3
  // which is 6, 2, 2, 6 copies per wave over the four k-steps of a slab pair.  Copies retire in order, so
  // "slab s+1 has landed" is a bound on the number of younger copies in flight at the end of the first
  // k-step of slab s: for even s two B slabs and one A pair (8 + the pair's copies, 16 for a full tile), for odd s 6
  // (2 and 0 for the last two waits).
  if constexpr (BNK) {
    // [n][k] weights, both operands in slab pairs.  After the barrier of an odd slab 2p+1 pair p is dead: A pair p+2
    // goes into its buffer during the next two k-steps and B pair p+3 during the two after those, four copies per wave
    // in every k-step.  Only odd slabs wait (for pair p+1, with the eight copies of B pair p+2 still in flight) and
    // only odd slabs need the workgroup barrier.
    issue_a(0);
    issue_bp(0);
    if (n_slabs > 2) { issue_a(1); issue_bp(1); }
    if (n_slabs >= 8) {
      wait_vmcnt<8 + NAB>();  // pair 0 is there when only A pair 1 (n_ablk copies) and B pair 1 (8) are in flight
    } else {
      if (n_slabs > 4) issue_bp(2);
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
  } else {
    issue_b(0);
    issue_a(0);
    if (n_slabs > 1) issue_b(1);
    if (n_slabs > 2) { issue_b(2); issue_a(1); }
    if (n_slabs > 3) issue_b(3);
    // Only slab 0 (the first 4 + n_ablk copies) has to be there to start; the waits of the slab steps below bound the
    // number of younger copies in flight, and that bound holds for what is left of these 32 as well.
    if (n_slabs >= 8) wait_vmcnt<12 + NAB>();  // B1, B2, B3 (12) and A pair 1 (n_ablk)
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  }
  __syncthreads();
  YAMOE_STAMP(2);
  read_frags(0, 0, fa0, fb0);

  // The instruction order is fixed by hand, because one wave per SIMD has nobody to hide behind: every LDS
  // read and every copy is issued in the shadow of an MFMA (an MFMA occupies the matrix pipe for 8 issue
  // slots), a whole k-step before its result is needed.
  //   first k-step:  MFMAs on set 0 + its copies + the LDS reads of the second k-step into set 1
  //   wait for slab s+1's copies; workgroup barrier
  //   second k-step: MFMAs on set 1 + its copies + the LDS reads of slab s+1's first k-step into set 0
  constexpr int kMma = NNI * NMI;
  constexpr int kSlots = kMma > 2 ? kMma - 2 : 1;  // the last two MFMAs of a k-step carry nothing
  auto slab_step = [&](int s, auto cfg) {
    typedef decltype(cfg) C;
    __builtin_amdgcn_sched_barrier(0);
    {
      constexpr int kA = C::P1A ? 4 : 0, kB = C::P1B ? (BNK ? 4 : 2) : 0, kItems = kA + kB + kFrags;
#pragma unroll
      for (int j = 0; j < (kMma > 0 ? kMma : 1); ++j) {
        if (j < kMma) Mma<T>::run(fb0[j % NNI], fa0[j / NNI], acc[j / NNI][j % NNI]);
        if (j < kSlots) {
#pragma unroll
          for (int i = j * kItems / kSlots; i < (j + 1) * kItems / kSlots; ++i) {
            if (i < kA) copy_a(s / 2 + 1, 4 + i);
            else if (i < kA + kB) { if constexpr (BNK) copy_bp((s + 3) / 2, 4 + i - kA); else copy_b(s + 3, 2 + i - kA); }
            else read_frag(s, 1, i - kA - kB, fa1, fb1);
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    if constexpr (C::VM == 16) wait_vmcnt<8 + NAB>();  // two B slabs (8) and one A pair (n_ablk copies) may be in flight
    else if constexpr (C::VM == 8) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    else if constexpr (C::VM == 6) asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
    else if constexpr (C::VM == 2) asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
    else if constexpr (C::VM == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if constexpr (C::BAR) __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
    {
      constexpr int kA = C::P2A ? 4 : 0, kB = C::P2B ? (BNK ? 4 : 2) : 0, kItems = kA + kB + (C::NEXT ? kFrags : 0);
#pragma unroll
      for (int j = 0; j < (kMma > 0 ? kMma : 1); ++j) {
        if (j < kMma) Mma<T>::run(fb1[j % NNI], fa1[j / NNI], acc[j / NNI][j % NNI]);
        if (j < kSlots) {
#pragma unroll
          for (int i = j * kItems / kSlots; i < (j + 1) * kItems / kSlots; ++i) {
            if (i < kA) copy_a((s + 1) / 2 + 1, i);
            else if (i < kA + kB) { if constexpr (BNK) copy_bp(s / 2 + 2, i - kA); else copy_b(s + 4, i - kA); }
            else read_frag(s + 1, 0, i - kA - kB, fa0, fb0);
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };
  // the same with every decision taken at run time, for contractions shorter than 8 slabs
  auto slab_step_short = [&](int s, bool odd) {
    read_frags(s, 1, fa1, fb1);
    mma(fa0, fb0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (odd && s + 3 < n_slabs) issue_a((s + 1) / 2 + 1);
    if constexpr (!BNK) {
      if (s + kBStages < n_slabs) issue_b(s + kBStages);  // ([n][k]: at most three B pairs, all requested up front)
    }
    if (s + 1 < n_slabs) read_frags(s + 1, 0, fa0, fb0);
    mma(fa1, fb1);
  };
  if (BNK && n_slabs >= 8) {
    slab_step(0, StepCfg<false, false, false, true, true, -1, false>());
    slab_step(1, StepCfg<false, true, true, false, true, 8>());
    int s = 2;
    for (; s + 5 < n_slabs; s += 2) {  // steady state: pair s/2 is consumed, A pair s/2 + 1 and B pair s/2 + 2 arrive
      slab_step(s, StepCfg<true, false, false, true, true, -1, false>());
      slab_step(s + 1, StepCfg<false, true, true, false, true, 8>());
    }
    // the last two pairs (s = n_slabs - 4)
    slab_step(s, StepCfg<true, false, false, false, true, -1, false>());
    slab_step(s + 1, StepCfg<false, false, false, false, true, 0>());
    slab_step(s + 2, StepCfg<false, false, false, false, true, -1, false>());
    slab_step(s + 3, StepCfg<false, false, false, false, false, -1, false>());
  } else if (n_slabs >= 8) {
    // copies of the (first, second) k-step: A half, B half; whether slab s+1 is read; the vmcnt bound (-1: no wait)
    slab_step(0, StepCfg<false, false, false, true, true, 16>());
    slab_step(1, StepCfg<false, true, true, true, true, 6>());
    int s = 2;
    for (; s + 7 < n_slabs; s += 2) {  // steady state
      slab_step(s, StepCfg<true, true, false, true, true, 16>());
      slab_step(s + 1, StepCfg<false, true, true, true, true, 6>());
    }
    // the last six slabs (s = n_slabs - 6): the last copies go out in the first k-step of slab n_slabs - 4
    slab_step(s, StepCfg<true, true, false, true, true, 16>());
    slab_step(s + 1, StepCfg<false, true, true, true, true, 6>());
    slab_step(s + 2, StepCfg<true, true, false, false, true, 16>());
    slab_step(s + 3, StepCfg<false, false, false, false, true, 2>());
    slab_step(s + 4, StepCfg<false, false, false, false, true, 0>());
    slab_step(s + 5, StepCfg<false, false, false, false, false, -1>());
  } else {
    for (int s = 0; s < n_slabs; s += 2) {
      slab_step_short(s, false);
      slab_step_short(s + 1, true);
    }
  }

  YAMOE_STAMP(3);
  // ---- epilogue -------------------------------------------------------------------------------------
  // The output tile is staged in LDS (the slab ring is dead by now) as [row][column] and then written
  // out row by row with 16 bytes per lane, so that a wave stores whole 512-byte (or 256-byte) row
  // segments instead of 2 bytes per lane.
  // The MFMAs run with the operands exchanged (weights as the A operand), so a lane holds one output row and four
  // consecutive columns per register quad:
  // acc[mi][ni][v]: tile row (mi*2+wm)*32 + lane%32, tile column (ni*2+wn)*32 + 8*(v/4) + 4*(lane/32) + v%4
  // which makes the staging stores 8 bytes wide and puts a (gate, up) pair into one lane.
  const int rows_valid = ti.rows_valid, n0 = ti.n0;
  const long long out_row0 = ti.row0;

  // rows of `width` elements, row stride width*2 + 16 bytes
  auto store_rows = [&](T *dst, long long ld, int col0, int width, int col_limit) {
    const int stride = width * 2 + 16;
    const int chunks = width >> 3, rows_per_pass = kThreads / chunks;
    const int c = tid % chunks;
    if (col0 + c * 8 >= col_limit) return;
    T *p = dst + out_row0 * ld + col0 + c * 8;
    for (int r = tid / chunks; r < rows_valid; r += rows_per_pass)
      *(u32x4 *)(p + (long long)r * ld) = *(const u32x4 *)(lds + r * stride + c * 16);
  };
  // the bias of this lane's 16 columns of column block ni, from the copy in LDS
  auto load_bias = [&](int ni, float (&b)[16]) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      float t[4] = {0.0f, 0.0f, 0.0f, 0.0f};
      if (has_bias) load4_f32((const T *)(lds + kBiasOff) + (ni * 2 + wn) * 32 + 8 * q + 4 * g, t);
#pragma unroll
      for (int i = 0; i < 4; ++i) b[4 * q + i] = t[i];
    }
  };
  // natural column order: value = acc + bias[column]   (the plain product, or, with `pre`, the pre-activations as the
  // backward reads them: even columns gate, odd columns up)
  auto stage_biased = [&](auto pre) {
    constexpr int stride = kBN * 2 + 16;
    char *lp = lds + (wm * 32 + rl) * stride + (wn * 32 + 4 * g) * 2;  // one address per lane, the rest are constants
#pragma unroll
    for (int ni = 0; ni < NNI; ++ni) {
      float b[16];
      load_bias(ni, b);
#pragma unroll
      for (int mi = 0; mi < NMI; ++mi)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const f32x16 &a = acc[mi][ni];
          u32x2 v;
          if constexpr (decltype(pre)::value) {
            typedef T T2 __attribute__((ext_vector_type(2)));
            T2 lo = {pre_activation_store<T>(a[4 * q] + b[4 * q], false), pre_activation_store<T>(a[4 * q + 1] + b[4 * q + 1], true)};
            T2 hi = {pre_activation_store<T>(a[4 * q + 2] + b[4 * q + 2], false), pre_activation_store<T>(a[4 * q + 3] + b[4 * q + 3], true)};
            v = (u32x2){__builtin_bit_cast(uint32_t, lo), __builtin_bit_cast(uint32_t, hi)};
          } else {
            v = (u32x2){pack2<T>(a[4 * q] + b[4 * q], a[4 * q + 1] + b[4 * q + 1]),
                        pack2<T>(a[4 * q + 2] + b[4 * q + 2], a[4 * q + 3] + b[4 * q + 3])};
          }
          *(u32x2 *)(lp + mi * 64 * stride + (ni * 64 + 8 * q) * 2) = v;
        }
    }
  };

  if (has_bias) *(T *)(lds + kBiasOff + tid * 2) = bias_reg;  // (outside the ring and the staging area)
  __syncthreads();  // every wave has finished reading the slab ring
  if constexpr (EPI == EPI_STORE && BNK) {
    // Row dots of the product with a second tensor of the output's shape, taken from the fp32 accumulators before they
    // are rounded (the routing gradient <grad_out . W_down^T, act>, csrc/experts_backward.cu:83-88): every wave writes
    // one partial sum per valid row, over its 128 columns of the tile; whoever reads them adds 2 * n_col_tiles values
    // per row in a fixed order.  The tile of the second tensor comes in through LDS by asynchronous copies, all in
    // flight at once (the ring is dead): 512-byte rows, the 16-byte pieces of row r XOR-swizzled with r & 31 on the
    // global side, so that the 32 lanes that read the same columns of 32 consecutive rows touch every bank once.
    if (args.dot_part != nullptr) {
      {
        const uint32_t lds_tile = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)lds);
        const char *src = (const char *)((const T *)args.dot_with + out_row0 * args.ldc + n0);
        const long long ld_bytes = (long long)args.ldc * (long long)sizeof(T);
#pragma unroll 8
        for (int i = 0; i < 32; ++i) {
          const int row = 64 * wave + 2 * i + (lane >> 5);
          int piece = (lane & 31) ^ (row & 31);
          if (n0 + piece * 8 >= args.Nd) piece = 0;  // columns past the end: re-read valid ones, never used
          const uint32_t off = (uint32_t)(min(row, rows_valid - 1) * ld_bytes + piece * 16);
          copy16_to_lds(src, off, lds_tile + (uint32_t)(64 * wave + 2 * i) * 512u);
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      }
      __syncthreads();
      const int n_part = 2 * args.n_col_tiles, part_col = 2 * (n0 / kBN) + wn;
      const char *lp = lds + (wm * 32 + rl) * 512 + g * 8;
#pragma unroll
      for (int mi = 0; mi < NMI; ++mi) {
        const int r = (mi * 2 + wm) * 32 + rl;
        float part = 0.0f;
#pragma unroll
        for (int ni = 0; ni < NNI; ++ni)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            // a run of four columns is valid or invalid as a whole (the column count is a multiple of 8)
            if (n0 + (ni * 2 + wn) * 32 + 8 * q + 4 * g < args.Nd) {
              float w4[4];
              load4_f32((const T *)(lp + mi * 64 * 512 + ((((ni * 2 + wn) * 4 + q) ^ rl) << 4)), w4);
#pragma unroll
              for (int i = 0; i < 4; ++i) part += acc[mi][ni][4 * q + i] * w4[i];
            }
          }
        part += __shfl_xor(part, 32);
        if (g == 0 && r < rows_valid) args.dot_part[(out_row0 + r) * n_part + part_col] = part;
      }
      __syncthreads();  // the staging area is about to be overwritten with the output tile
    }
  }
  if constexpr (EPI == EPI_STORE) {
    stage_biased(std::false_type());
    __syncthreads();
    YAMOE_STAMP(4);
    store_rows((T *)args.C, args.ldc, n0, kBN, args.Nd);
  } else {
    if (args.C2 != nullptr) {  // pre-activations for the backward: the biased product itself
      stage_biased(std::true_type());
      __syncthreads();
      store_rows((T *)args.C2, args.Nd, n0, kBN, args.Nd);
      __syncthreads();
    }
    // A register quad holds (gate, up, gate, up) of two neighbouring activations of one row.
    constexpr int stride = (kBN / 2) * 2 + 16;
    char *lp = lds + (wm * 32 + rl) * stride + (wn * 16 + 2 * g) * 2;
#pragma unroll
    for (int ni = 0; ni < NNI; ++ni) {
      float b[16];
      load_bias(ni, b);
#pragma unroll
      for (int mi = 0; mi < NMI; ++mi)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const f32x16 &a = acc[mi][ni];
          float h0 = glu_forward(a[4 * q] + b[4 * q], a[4 * q + 1] + b[4 * q + 1]);
          float h1 = glu_forward(a[4 * q + 2] + b[4 * q + 2], a[4 * q + 3] + b[4 * q + 3]);
          *(uint32_t *)(lp + mi * 64 * stride + (ni * 32 + 4 * q) * 2) = pack2<T>(h0, h1);
        }
    }
    __syncthreads();
    YAMOE_STAMP(4);
    store_rows((T *)args.C, args.ldc, n0 >> 1, kBN / 2, args.Nd >> 1);
  }
#ifdef YAMOE_TILE_STAMPS
  YAMOE_STAMP(5);
  if (tid == 0 && args.stamps != nullptr && ti.slot < args.stamps_cap) {
    unsigned long long *o = args.stamps + 8ll * ti.slot;
#pragma unroll
    for (int i = 0; i < 6; ++i) o[i] = stamp_reg[i];
    o[6] = (unsigned long long)(uint32_t)ti.rows_valid | ((unsigned long long)(uint32_t)min(kBN, args.Nd - ti.n0) << 16);
    const unsigned hw = __builtin_amdgcn_s_getreg((4 << 0) | (8 << 6) | (7 << 11));    // HW_ID bits 8..15: CU, SH and SE id
    const unsigned xcc = __builtin_amdgcn_s_getreg((20 << 0) | (0 << 6) | (3 << 11));  // XCC_ID
    o[7] = ((unsigned long long)xcc << 8) | hw;
  }
#endif
}

template <typename T, int EPI, bool GATHER, bool BNK>
__global__ __launch_bounds__(kThreads) void gemm_async_kernel(const Args args) {

  // Workgroup b runs on XCD b % 8 and takes tile b / 8 of that XCD's share of the tile list.  The shares have
  // equal cost, not equal length, and are cut on (expert, column tile) boundaries, so the row tiles that read
  // the same weight slabs meet in one L2.  A share longer than gridDim.x / 8 hands its excess to the workgroups
  // of shorter shares (the grid has at least as many workgroups as there are tiles).
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, wm = wave >> 1;
#ifdef YAMOE_TILE_STAMPS
  const unsigned long long t_entry = __builtin_amdgcn_s_memtime();
#endif
  int L;
  {
    const int xcd = blockIdx.x % kXcds, i = blockIdx.x / kXcds, slots = gridDim.x / kXcds;
    const int first = sched_cut(args.sched, xcd, args.n_col_tiles);
    const int count = sched_cut(args.sched, xcd + 1, args.n_col_tiles) - first;
    if (i < count) {
      L = first + i;
    } else {
      int cut[kXcds + 1];
#pragma unroll
      for (int x = 0; x <= kXcds; ++x) cut[x] = sched_cut(args.sched, x, args.n_col_tiles);
      int rank = i - count;  // rank of this workgroup among the idle ones
#pragma unroll
      for (int x = 0; x < kXcds; ++x)
        if (x < xcd) rank += max(slots - (cut[x + 1] - cut[x]), 0);
      L = -1;
#pragma unroll
      for (int x = 0; x < kXcds; ++x) {
        int excess = max(cut[x + 1] - cut[x] - slots, 0);
        if (L < 0) {
          if (rank < excess) L = cut[x] + slots + rank;
          else rank -= excess;
        }
      }
      if (L < 0) return;
    }
  }
  TileInfo ti;
  {
    const int *tiles = args.sched + kSchedHeader;
    int t0 = fast_div(L, args.n_col_div);
    int gfirst = __builtin_amdgcn_readfirstlane(tiles[8 * t0 + 3]), gcount = __builtin_amdgcn_readfirstlane(tiles[8 * t0 + 4]);
    FastDiv by_gcount = {(uint32_t)__builtin_amdgcn_readfirstlane(tiles[8 * t0 + 5]),
                         (uint32_t)__builtin_amdgcn_readfirstlane(tiles[8 * t0 + 6])};
    int local = L - gfirst * args.n_col_tiles;
    int col_tile, row_tile;
    if (gcount < 2 * kBandRows) {
      // the expert's tiles column by column: its few row tiles follow each other and share the column's weight slabs
      col_tile = fast_div(local, by_gcount);
      row_tile = local - col_tile * gcount;
    } else {
      // An expert with many row tiles, in bands of kBandRows row tiles (the last band takes the remainder), each band
      // column by column.  The 32 CUs of an XCD work on 32 consecutive tiles; column by column over the whole expert
      // those are 32 row tiles of one column, which share the weight slabs but fetch 32 different sets of rows, and
      // every row comes through the L2 once per column tile (measured at 8192 rows per expert: 12 times the
      // algorithmic bytes fetched, 4.4 TB/s, and the products 11 % slower than in bands).  In a band they are 4
      // columns of 8 row tiles: 8 sets of rows and 4 sets of slabs for the same 32 tiles.  Bands of 4 to 16 row tiles
      // measure within 1 % of each other; below 16 row tiles the column order is as good or better.
      const int bands = gcount / kBandRows;
      int band = min(fast_div(local, args.band_div), bands - 1);
      const int in_band = local - band * kBandRows * args.n_col_tiles;
      const int band_rows = band == bands - 1 ? gcount - band * kBandRows : kBandRows;
      col_tile = (int)((uint32_t)in_band / (uint32_t)band_rows);
      row_tile = band * kBandRows + in_band - col_tile * band_rows;
    }
    const int *te = tiles + 8 * (gfirst + row_tile);
    // (the same for every lane; said explicitly, so that the operand addresses built from them stay in scalar registers
    // whatever the compiler can prove about the work list's memory)
    ti.expert = __builtin_amdgcn_readfirstlane(te[0]);
    ti.row0 = __builtin_amdgcn_readfirstlane(te[1]);
    ti.rows_valid = __builtin_amdgcn_readfirstlane(te[2]);
    ti.n0 = col_tile * kBN;
#ifdef YAMOE_TILE_STAMPS
    ti.slot = L; ti.t_entry = t_entry;
#endif
  }

  // A copies: copy i fetches rows 32*i + 8*wave + (lane >> 3); LDS position lane & 7 holds piece pos ^ ((row >> 1) & 7)
  // (a gathering instantiation without a row list reads its rows in order, like the others: the form the callers use
  // when the gathered tensor is too large for 32-bit byte offsets from its start and they have permuted it first)
  const bool gathers = GATHER && args.a_rows != nullptr;
  uint32_t a_off[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    int row = 32 * i + 8 * wave + (lane >> 3);
    int piece = (lane & 7) ^ ((row >> 1) & 7);
    int r = min(row, ti.rows_valid - 1);
    long long src = r;
    if (gathers) src = fast_div(args.a_rows[ti.row0 + r], args.a_div);
    a_off[i] = (uint32_t)((src * args.lda + piece * 8) * (long long)sizeof(T));
  }
  const char *a_base = (const char *)((const T *)args.A + (gathers ? 0ll : (long long)ti.row0 * args.lda));

  const long long b_ld_bytes = (long long)args.ldb * (long long)sizeof(T);
  uint32_t b_off[8];
  const char *b_base;
  long long b_slab_bytes;
  if constexpr (BNK) {
    // B is [n][k] (k-contiguous rows, one per output column), copied like A: rows 64*wave + 8*i + (lane >> 3), 128
    // bytes (two slabs) of each per copy, so that every request is a whole cache line; LDS position lane & 7 holds
    // piece pos ^ ((row >> 1) & 7)
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      int row = 64 * wave + 8 * i + (lane >> 3);
      int piece = (lane & 7) ^ ((row >> 1) & 7);
      int r = min(row, args.Nd - 1 - ti.n0);  // columns past the end re-read the last one; never stored
      b_off[i] = (uint32_t)(r * b_ld_bytes + piece * 16);
    }
    b_base = (const char *)((const T *)args.B + (long long)ti.expert * args.b_expert_stride + (long long)ti.n0 * args.ldb);
    b_slab_bytes = kBK * (long long)sizeof(T);
  } else {
    // B is [k][n]: k rows 8*wave + 2*i + (lane >> 5); LDS position lane & 31 holds piece pos ^ ((k & 3) << 2)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      int k = 8 * wave + 2 * i + (lane >> 5);
      int piece = (lane & 31) ^ ((k & 3) << 2);
      int col = ti.n0 + piece * 8;
      if (col >= args.Nd) col = ti.n0;  // columns past the end re-read valid ones; never stored
      b_off[i] = (uint32_t)(k * b_ld_bytes + (long long)(col - ti.n0) * (long long)sizeof(T));
      b_off[4 + i] = 0;
    }
    b_base = (const char *)((const T *)args.B + (long long)ti.expert * args.b_expert_stride + ti.n0);
    b_slab_bytes = kBK * b_ld_bytes;
  }

#ifdef YAMOE_TILE_STAMPS
  // (after the work-list look-ups and the gathered row numbers: a_off depends on both)
  asm volatile("s_waitcnt vmcnt(0)" : : "v"(a_off[0]), "v"(a_off[7]) : "memory");
  ti.t_lookup = __builtin_amdgcn_s_memtime();
#endif
  const int n_blocks32 = (ti.rows_valid + 31) >> 5;
  const int n_mi = (n_blocks32 - wm + 1) >> 1;
  // valid 32-column blocks of this wave column (they alternate between the two); tiles of 64 or 128 valid columns with
  // three or four row blocks per wave have instantiations of their own, everything else computes all four blocks
  const int wn = wave & 1;
  const int n_blocks32_n = (min(kBN, args.Nd - ti.n0) + 31) >> 5;
  const int n_ni = (n_blocks32_n - wn + 1) >> 1;
#define YAMOE_RUN(NMI_, NNI_) run_tile<T, EPI, NMI_, BNK, NNI_>(args, ti, tid, a_base, a_off, b_base, b_off, b_slab_bytes)
#define YAMOE_RUN6(NNI_) run_tile<T, EPI, 3, BNK, NNI_, 6>(args, ti, tid, a_base, a_off, b_base, b_off, b_slab_bytes)
  // six row blocks (161..192 rows, what an expert with a few rows more than two full tiles is cut into): both wave
  // rows have three, and only six of the eight blocks are copied
  const bool six = n_blocks32 == 6;
  if (n_ni <= 2 && n_mi >= 3) {
    if (n_ni <= 1) { if (n_mi == 4) YAMOE_RUN(4, 1); else if (six) YAMOE_RUN6(1); else YAMOE_RUN(3, 1); }
    else { if (n_mi == 4) YAMOE_RUN(4, 2); else if (six) YAMOE_RUN6(2); else YAMOE_RUN(3, 2); }
    return;
  }
  if (six) { YAMOE_RUN6(4); return; }
  switch (n_mi) {
    case 4: YAMOE_RUN(4, 4); break;
    case 3: YAMOE_RUN(3, 4); break;
    case 2: YAMOE_RUN(2, 4); break;
    case 1: YAMOE_RUN(1, 4); break;
    default: YAMOE_RUN(0, 4); break;
  }
#undef YAMOE_RUN
#undef YAMOE_RUN6
}

#ifdef YAMOE_TILE_STAMPS
static unsigned long long *g_tile_stamps = nullptr;
static int g_tile_stamps_cap = 0;
#endif

template <typename T, int EPI, bool GATHER, bool BNK>
static int launch(const Args &args, int max_row_tiles, hipStream_t stream) {
  auto kernel = gemm_async_kernel<T, EPI, GATHER, BNK>;
  constexpr int lds_bytes = BNK ? (kLdsNk > kLds ? kLdsNk : kLds) : kLds;
  static DeviceFlags attr_done;  // one per kernel instantiation
  if (int rc = ensure_dynamic_lds((const void *)kernel, lds_bytes, attr_done, "gemm_async_kernel")) return rc;
  long long total = (long long)max_row_tiles * args.n_col_tiles;
  if (total <= 0) return 0;
  total = (total + kXcds - 1) / kXcds * kXcds;
#ifdef YAMOE_TILE_STAMPS
  Args stamped = args;
  stamped.stamps = g_tile_stamps;
  stamped.stamps_cap = g_tile_stamps_cap;
  hipLaunchKernelGGL(kernel, dim3((unsigned)total), dim3(kThreads), lds_bytes, stream, stamped);
#else
  hipLaunchKernelGGL(kernel, dim3((unsigned)total), dim3(kThreads), lds_bytes, stream, args);
#endif
  return check_launch("gemm_async_kernel");
}


// ---- weight gradients: dW[e] = L[rows of e]^T * R[rows of e] -----------------------------------------------
// (csrc/experts_backward.cu:198, 311).  The contraction runs over the expert's kept rows, so both operands are
// [k][m] / [k][n] in memory: both stay that way in LDS (single-slab buffers of 32 k-rows) and both are read with
// the LDS transpose read.  The last slab of an expert is usually partial: the copies of its missing rows read
// whatever follows in memory (the caller keeps that readable) and the wave that issued them overwrites them with
// zeros in LDS before anybody reads the slab.
struct WgradArgs {
  const void *A;  // [N, Md] rows in expert order; with a_rows: [*, Md], sorted row p is row a_rows[p] / a_div of it
  const void *B;  // [N, Nd]
  void *C;        // [E, Md, Nd]
  const int *counts, *offsets;
  const int *a_rows;
  FastDiv a_div;
  int a_rows_max;  // largest value a_rows may hold
  int capacity, E, Md, Nd, n_m_tiles, n_n_tiles;
  // optional: [E, Nd] column sums of the expert's rows of B (the bias gradient that goes with this weight gradient,
  // csrc/experts_backward.cu:277, 308); needs Md % 128 != 0 (see wgrad_writes_bias)
  void *bias_grad;
};

template <bool P1_, bool P2_, bool NEXT_, bool ZERO_, int VM_> struct WStepCfg {
  static constexpr bool P1 = P1_, P2 = P2_, NEXT = NEXT_, ZERO = ZERO_;
  static constexpr int VM = VM_;
};

// 128 x 256 tiles with a three-slab ring (72 KB of LDS, at most 256 registers per lane), so that two workgroups
// share a CU: an expert's contraction is short (its kept rows), a tile spends a third of its time filling the ring
// and storing its result, and with a second workgroup on the same SIMDs the matrix pipe works through that.
constexpr int kSmallBM = 128, kSmallStages = 3;
constexpr int kSmallAStage = kBK * kSmallBM * 2, kSmallBStage = kBK * kBN * 2;  // 8 KB + 16 KB per slab
constexpr int kSmallBRing = kSmallStages * kSmallAStage;
constexpr int kSmallRing = kSmallStages * (kSmallAStage + kSmallBStage);
constexpr int kSmallStaging = kSmallBM * (kBN * 2 + 16);
constexpr int kSmallLds = kSmallRing > kSmallStaging ? kSmallRing : kSmallStaging;

// bias_tile: this is the last row tile of the gradient and has room below its rows_m valid rows.  Column rows_m of the
// left operand's LDS tile then holds 1 for every valid k (planted after each slab's copies have landed), so that row
// rows_m of the product is 1^T . R, the column sums of the expert's rows of R: the bias gradient, taken by the same
// MFMAs in fp32 instead of by a launch of its own over the same rows (17.5 + 37 us at the GPT-OSS-20B shape).
template <typename T, int NMI, bool GATHER>
__device__ inline void run_wgrad_tile_small(const WgradArgs &args, const int tid, const int expert, const int m0,
                                            const int n0, const int rows_m, const long long first, const int rows,
                                            const bool bias_tile) {
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  constexpr int NACC = NMI > 0 ? NMI : 1;
  extern __shared__ __attribute__((aligned(16))) char lds[];
  const uint32_t lds0 = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)lds);

  f32x16 acc[NACC][4];
#pragma unroll
  for (int mi = 0; mi < NACC; ++mi)
#pragma unroll
    for (int ni = 0; ni < 4; ++ni)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[mi][ni][v] = 0.0f;

  const int n_slabs = (rows + kBK - 1) / kBK;
  const long long lda_bytes = (long long)args.Md * (long long)sizeof(T), ldb_bytes = (long long)args.Nd * (long long)sizeof(T);

  // A copies: piece i (0..1) = k rows 4*(2*wave + i) + (lane >> 4) of the slab, 256 bytes each; LDS position lane & 15
  // holds piece pos ^ ((k & 3) << 2).  B copies as in the large kernel: piece i (0..3) = k rows 8*wave + 2*i + (lane >> 5).
  uint32_t a_off[2], b_off[4];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    int k = 4 * (2 * wave + i) + (lane >> 4);
    int piece = (lane & 15) ^ ((k & 3) << 2);
    int ca = m0 + piece * 8;
    if (ca >= args.Md) ca = m0;
    a_off[i] = (uint32_t)((GATHER ? 0ll : k * lda_bytes) + (long long)(ca - m0) * (long long)sizeof(T));
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    int k = 8 * wave + 2 * i + (lane >> 5);
    int piece = (lane & 31) ^ ((k & 3) << 2);
    int cb = n0 + piece * 8;
    if (cb >= args.Nd) cb = n0;
    b_off[i] = (uint32_t)(k * ldb_bytes + (long long)(cb - n0) * (long long)sizeof(T));
  }
  const char *a_base = (const char *)((const T *)args.A + (GATHER ? 0ll : first * args.Md) + m0);
  const char *b_base = (const char *)((const T *)args.B + first * args.Nd + n0);
  // Gathered A rows: the four k rows of piece i of a slab are rows a_rows[first + 32*slab + 4*(2*wave + i) + 0..3]
  // / a_div of A.  The positions are the same for the whole wave, so the look-ups are scalar loads (rows_of), issued
  // at the start of the half slab whose last slot issues the copy; there the lane picks its row and turns it into a
  // byte offset (row_bytes).  Positions past the expert's rows (up to 31 past the end of the list: the caller keeps
  // that readable) hold somebody else's row or anything at all: the value is clamped to the list's range, and what the
  // copy fetches is zeroed in LDS before use.  The list is read through the constant address space, which makes the loads scalar whatever the
  // compiler can prove about the memory in between (the list was written by an earlier launch).
  typedef const __attribute__((address_space(4))) int *ConstInts;
  ConstInts a_rows = GATHER ? (ConstInts)(uintptr_t)(args.a_rows + first) : (ConstInts)0;
  auto rows_of = [&](int slab, int i, int (&ix)[4]) {
    if constexpr (GATHER) {
      const int k0 = slab * kBK + 4 * (2 * wave + i);
#pragma unroll
      for (int j = 0; j < 4; ++j) ix[j] = a_rows[k0 + j];
    }
  };
  auto row_bytes = [&](int (&ix)[4]) -> uint32_t {
    if constexpr (!GATHER) return 0u;
    // the four values pass through an empty statement: the loads stay where rows_of put them, all four of them, and
    // what follows is three selects rather than loads under branches
    int r0 = ix[0], r1 = ix[1], r2 = ix[2], r3 = ix[3];
    asm volatile("" : "+s"(r0), "+s"(r1), "+s"(r2), "+s"(r3));
    const bool odd = (lane & 16) != 0, high = (lane & 32) != 0;
    const int lo = odd ? r1 : r0, hi = odd ? r3 : r2;
    const uint32_t r = min((uint32_t)(high ? hi : lo), (uint32_t)args.a_rows_max);
    return (uint32_t)fast_div((int)r, args.a_div) * (uint32_t)lda_bytes;
  };
  auto copy_a = [&](int slab, int i, uint32_t row) {
    copy16_to_lds(a_base + (GATHER ? 0ll : (long long)slab * kBK * lda_bytes), a_off[i] + row,
                  lds0 + (uint32_t)(slab % kSmallStages) * kSmallAStage + (uint32_t)(4 * (2 * wave + i)) * 256u);
  };
  auto copy_a_now = [&](int slab, int i) {  // look-up and copy in one go: outside the pipelined loop
    int ix[4] = {0, 0, 0, 0};
    rows_of(slab, i, ix);
    copy_a(slab, i, row_bytes(ix));
  };
  auto copy_b = [&](int slab, int i) {
    copy16_to_lds(b_base + (long long)slab * kBK * ldb_bytes, b_off[i],
                  lds0 + kSmallBRing + (uint32_t)(slab % kSmallStages) * kSmallBStage + (uint32_t)(8 * wave + 2 * i) * 512u);
  };
  auto copy_slab = [&](int slab) {
    copy_a_now(slab, 0); copy_b(slab, 0); copy_b(slab, 1); copy_a_now(slab, 1); copy_b(slab, 2); copy_b(slab, 3);
  };
  auto zero_tail = [&](int slab) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      int k = 4 * (2 * wave + i) + (lane >> 4);
      if (slab * kBK + k >= rows)
        *(u32x4 *)(lds + (slab % kSmallStages) * kSmallAStage + 4 * (2 * wave + i) * 256 + lane * 16) = (u32x4){0, 0, 0, 0};
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      int k = 8 * wave + 2 * i + (lane >> 5);
      if (slab * kBK + k >= rows)
        *(u32x4 *)(lds + kSmallBRing + (slab % kSmallStages) * kSmallBStage + (8 * wave + 2 * i) * 512 + lane * 16) = (u32x4){0, 0, 0, 0};
    }
  };

  // the ones column of slab `slab` (whose copies by this wave have landed): this wave's 8 k rows; lane l and the seven
  // lanes l + 8 j write the same value to the same place (a branch on the lane number here would be the loop's only
  // divergent one)
  const int ones_k = 8 * wave + (lane & 7);
  char *const ones_at = lds + ones_k * 256 + (((rows_m >> 3) ^ ((ones_k & 3) << 2)) << 4) + (rows_m & 7) * 2;
  auto plant_ones = [&](int slab) {
    if (bias_tile)
      *(T *)(ones_at + (slab % kSmallStages) * kSmallAStage) = ElemTraits<T>::from_f32(slab * kBK + ones_k < rows ? 1.0f : 0.0f);
  };

  const int g = lane >> 5, rl = lane & 31, j4 = (lane & 15) >> 2, q4 = lane & 3;
  int a_rd[NACC], b_rd[4];
#pragma unroll
  for (int mi = 0; mi < NACC; ++mi) {
    int col = (mi * 2 + wm) * 32 + 16 * ((lane >> 4) & 1) + 4 * q4;
    a_rd[mi] = (g * 8 + j4) * 256 + ((((col >> 3) ^ (j4 << 2))) << 4) + (col & 7) * 2;
  }
#pragma unroll
  for (int ni = 0; ni < 4; ++ni) {
    int col = wn * 128 + ni * 32 + 16 * ((lane >> 4) & 1) + 4 * q4;
    b_rd[ni] = (g * 8 + j4) * 512 + ((((col >> 3) ^ (j4 << 2))) << 4) + (col & 7) * 2;
  }
  u32x4 fa0[NACC], fa1[NACC], fb0[4], fb1[4];
  constexpr int kFrags = NMI > 0 ? 4 + NMI : 0;
  // fragment order B0, A0, B1, B2, B3, A1
  auto read_frag = [&](int s, int ks, int f, u32x4 (&fa)[NACC], u32x4 (&fb)[4]) {
    const bool is_a = f == 1 || f >= 5;
    const int idx = is_a ? (f == 1 ? 0 : f - 4) : (f == 0 ? 0 : f - 1);
    const char *sp = is_a ? lds + (s % kSmallStages) * kSmallAStage + a_rd[idx] + ks * 4096
                          : lds + kSmallBRing + (s % kSmallStages) * kSmallBStage + b_rd[idx] + ks * 8192;
    u32x2 lo = lds_read_tr16(sp);
    u32x2 hi = lds_read_tr16(sp + (is_a ? 1024 : 2048));
    u32x4 v = (u32x4){lo[0], lo[1], hi[0], hi[1]};
    if (is_a) fa[idx] = v; else fb[idx] = v;
  };
  auto read_frags = [&](int s, int ks, u32x4 (&fa)[NACC], u32x4 (&fb)[4]) {
#pragma unroll
    for (int f = 0; f < kFrags; ++f) read_frag(s, ks, f, fa, fb);
  };

  // pipeline: slab t+3 goes into the buffer slab t leaves at its mid-slab barrier: first half of its copies
  // (A piece 0, B pieces 0-1) in the second k-step of slab t, second half in the first k-step of slab t+1; "slab
  // s+1 has landed" = at most 6 younger copies in flight
  constexpr int kMma = 4 * NMI;
  constexpr int kSlots = kMma > 2 ? kMma - 2 : 1;
  if (n_slabs > 0) {
#pragma unroll
    for (int s = 0; s < kSmallStages; ++s)
      if (s < n_slabs) copy_slab(s);
    if (n_slabs >= 6) asm volatile("s_waitcnt vmcnt(12)" ::: "memory");  // slab 0 is enough to start with
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    plant_ones(0);
#pragma unroll
    for (int s = 0; s < kSmallStages; ++s)
      if (n_slabs < 6 && s < n_slabs && (s + 1) * kBK > rows) zero_tail(s);
    __syncthreads();
    read_frags(0, 0, fa0, fb0);
  }
  // In the pipelined loop the ring stage of every slab is a compile-time constant (the loop is unrolled by the ring
  // depth), so that an operand read is one ds_read with an immediate offset from a per-lane base and a copy's LDS
  // address one scalar add: with the stage computed per slab (a division by 3, then one vector add per read) the
  // loop carried 3.4 vector instructions per MFMA, 30 of them in a block ahead of each slab's first MFMA.
  const char *pa[NACC], *pb[4];
#pragma unroll
  for (int mi = 0; mi < NACC; ++mi) pa[mi] = lds + a_rd[mi];
#pragma unroll
  for (int ni = 0; ni < 4; ++ni) pb[ni] = lds + kSmallBRing + b_rd[ni];
  const uint32_t lds_a_wave = lds0 + (uint32_t)(8 * wave) * 256u, lds_b_wave = lds0 + kSmallBRing + (uint32_t)(8 * wave) * 512u;
  auto read_frag_c = [&](auto stage, int ks, int f, u32x4 (&fa)[NACC], u32x4 (&fb)[4]) {
    constexpr int ST = decltype(stage)::value;
    const bool is_a = f == 1 || f >= 5;
    const int idx = is_a ? (f == 1 ? 0 : f - 4) : (f == 0 ? 0 : f - 1);
    const char *sp = is_a ? pa[idx] + ST * kSmallAStage + ks * 4096 : pb[idx] + ST * kSmallBStage + ks * 8192;
    u32x2 lo = lds_read_tr16(sp);
    u32x2 hi = lds_read_tr16(sp + (is_a ? 1024 : 2048));
    u32x4 v = (u32x4){lo[0], lo[1], hi[0], hi[1]};
    if (is_a) fa[idx] = v; else fb[idx] = v;
  };
  auto copy_a_c = [&](auto stage, int slab, int i, uint32_t row) {
    constexpr int ST = decltype(stage)::value;
    copy16_to_lds(a_base + (GATHER ? 0ll : (long long)slab * kBK * lda_bytes), a_off[i] + row,
                  lds_a_wave + (uint32_t)(ST * kSmallAStage + 4 * i * 256));
  };

  auto copy_b_c = [&](auto stage, int slab, int i) {
    constexpr int ST = decltype(stage)::value;
    copy16_to_lds(b_base + (long long)slab * kBK * ldb_bytes, b_off[i], lds_b_wave + (uint32_t)(ST * kSmallBStage + 2 * i * 512));
  };
  // slab s sits in ring stage ST
  auto slab_step = [&](int s, auto cfg, auto stage) {
    typedef decltype(cfg) C;
    constexpr int ST = decltype(stage)::value;
    typedef std::integral_constant<int, (ST + 1) % kSmallStages> Next;   // slab s + 1
    typedef std::integral_constant<int, (ST + 2) % kSmallStages> Next2;  // slab s + 2; slab s + 3 takes stage ST again
    __builtin_amdgcn_sched_barrier(0);
    {
      constexpr int kC = C::P1 ? 3 : 0, kItems = kC + kFrags;
      int ix[4] = {0, 0, 0, 0};  // gathered rows: the four rows of the A piece copied in this half slab
#pragma unroll
      for (int j = 0; j < (kMma > 0 ? kMma : 1); ++j) {
        if (j < kMma) Mma<T>::run(fb0[j & 3], fa0[j >> 2], acc[j >> 2][j & 3]);
        if (j < kSlots) {
#pragma unroll
          for (int i = j * kItems / kSlots; i < (j + 1) * kItems / kSlots; ++i) {
            if (i < kC) {
              if (i == 0) { if constexpr (GATHER) rows_of(s + 2, 1, ix); else copy_a_c(Next2(), s + 2, 1, 0u); }
              else copy_b_c(Next2(), s + 2, 1 + i);
            }
            else read_frag_c(stage, 1, i - kC, fa1, fb1);
          }
          if (GATHER && kC > 0 && j == kSlots - 1) copy_a_c(Next2(), s + 2, 1, row_bytes(ix));
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    if constexpr (C::VM == 6) asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
    else if constexpr (C::VM == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if constexpr (C::NEXT) plant_ones(s + 1);
    if constexpr (C::ZERO) zero_tail(s + 1);
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
    {
      constexpr int kC = C::P2 ? 3 : 0, kItems = kC + (C::NEXT ? kFrags : 0);
      int ix[4] = {0, 0, 0, 0};  // gathered rows: the four rows of the A piece copied in this half slab
#pragma unroll
      for (int j = 0; j < (kMma > 0 ? kMma : 1); ++j) {
        if (j < kMma) Mma<T>::run(fb1[j & 3], fa1[j >> 2], acc[j >> 2][j & 3]);
        if (j < kSlots) {
#pragma unroll
          for (int i = j * kItems / kSlots; i < (j + 1) * kItems / kSlots; ++i) {
            if (i < kC) {
              if (i == 0) { if constexpr (GATHER) rows_of(s + 3, 0, ix); else copy_a_c(stage, s + 3, 0, 0u); }
              else copy_b_c(stage, s + 3, i - 1);
            }
            else read_frag_c(Next(), 0, i - kC, fa0, fb0);
          }
          if (GATHER && kC > 0 && j == kSlots - 1) copy_a_c(stage, s + 3, 0, row_bytes(ix));
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };
  // the same step with the ring stage taken from the slab number at run time: for the slabs the unrolled loop leaves
  // over and for the last three (the stage they start in depends on the slab count)
  auto slab_step_rt = [&](int s, auto cfg) {
    typedef decltype(cfg) C;
    __builtin_amdgcn_sched_barrier(0);
    {
      constexpr int kC = C::P1 ? 3 : 0, kItems = kC + kFrags;
      int ix[4] = {0, 0, 0, 0};  // gathered rows: the four rows of the A piece copied in this half slab
#pragma unroll
      for (int j = 0; j < (kMma > 0 ? kMma : 1); ++j) {
        if (j < kMma) Mma<T>::run(fb0[j & 3], fa0[j >> 2], acc[j >> 2][j & 3]);
        if (j < kSlots) {
#pragma unroll
          for (int i = j * kItems / kSlots; i < (j + 1) * kItems / kSlots; ++i) {
            if (i < kC) {
              if (i == 0) { if constexpr (GATHER) rows_of(s + 2, 1, ix); else copy_a(s + 2, 1, 0u); }
              else copy_b(s + 2, 1 + i);
            }
            else read_frag(s, 1, i - kC, fa1, fb1);
          }
          if (GATHER && kC > 0 && j == kSlots - 1) copy_a(s + 2, 1, row_bytes(ix));
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    if constexpr (C::VM == 6) asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
    else if constexpr (C::VM == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if constexpr (C::NEXT) plant_ones(s + 1);
    if constexpr (C::ZERO) zero_tail(s + 1);
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
    {
      constexpr int kC = C::P2 ? 3 : 0, kItems = kC + (C::NEXT ? kFrags : 0);
      int ix[4] = {0, 0, 0, 0};  // gathered rows: the four rows of the A piece copied in this half slab
#pragma unroll
      for (int j = 0; j < (kMma > 0 ? kMma : 1); ++j) {
        if (j < kMma) Mma<T>::run(fb1[j & 3], fa1[j >> 2], acc[j >> 2][j & 3]);
        if (j < kSlots) {
#pragma unroll
          for (int i = j * kItems / kSlots; i < (j + 1) * kItems / kSlots; ++i) {
            if (i < kC) {
              if (i == 0) { if constexpr (GATHER) rows_of(s + 3, 0, ix); else copy_a(s + 3, 0, 0u); }
              else copy_b(s + 3, i - 1);
            }
            else read_frag(s + 1, 0, i - kC, fa0, fb0);
          }
          if (GATHER && kC > 0 && j == kSlots - 1) copy_a(s + 3, 0, row_bytes(ix));
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };
  if (n_slabs >= 6) {
    typedef std::integral_constant<int, 0> S0;
    typedef std::integral_constant<int, 1> S1;
    typedef std::integral_constant<int, 2> S2;
    typedef WStepCfg<true, true, true, false, 6> Steady;
    slab_step(0, WStepCfg<false, true, true, false, 6>(), S0());
    int s = 1;
    for (; s + 5 < n_slabs; s += 3) {  // steady state, three slabs per round: stages 1, 2, 0
      slab_step(s, Steady(), S1());
      slab_step(s + 1, Steady(), S2());
      slab_step(s + 2, Steady(), S0());
    }
    for (; s + 3 < n_slabs; ++s) slab_step_rt(s, Steady());  // at most two
    // the last three slabs (s = n_slabs - 3): no new copies; the last slab's missing rows are zeroed
    slab_step_rt(s, WStepCfg<true, false, true, false, 6>());
    slab_step_rt(s + 1, WStepCfg<false, false, true, true, 0>());
    slab_step_rt(s + 2, WStepCfg<false, false, false, false, -1>());
  } else {
    for (int s = 0; s < n_slabs; ++s) {
      if (kFrags > 0) read_frags(s, 1, fa1, fb1);
#pragma unroll
      for (int j = 0; j < kMma; ++j) Mma<T>::run(fb0[j & 3], fa0[j >> 2], acc[j >> 2][j & 3]);
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      if (s + 1 < n_slabs) plant_ones(s + 1);
      if (s + 1 < n_slabs && (s + 2) * kBK > rows) zero_tail(s + 1);
      __syncthreads();
      if (s + kSmallStages < n_slabs) copy_slab(s + kSmallStages);
      if (s + 1 < n_slabs) read_frags(s + 1, 0, fa0, fb0);
#pragma unroll
      for (int j = 0; j < kMma; ++j) Mma<T>::run(fb1[j & 3], fa1[j >> 2], acc[j >> 2][j & 3]);
    }
  }

  // epilogue: stage the tile in LDS, store whole row segments
  constexpr int stride = kBN * 2 + 16;
  // (operands exchanged in the MFMAs, as in the forward kernel) acc[mi][ni][v]: tile row (mi*2+wm)*32 + lane%32,
  // tile column wn*128 + ni*32 + 8*(v/4) + 4*(lane/32) + v%4
  __syncthreads();
  {
    char *lp = lds + (wm * 32 + rl) * stride + (wn * 128 + 4 * g) * 2;
#pragma unroll
    for (int ni = 0; ni < 4; ++ni)
#pragma unroll
      for (int mi = 0; mi < NMI; ++mi)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const f32x16 &a = acc[mi][ni];
          u32x2 v = {pack2<T>(a[4 * q], a[4 * q + 1]), pack2<T>(a[4 * q + 2], a[4 * q + 3])};
          *(u32x2 *)(lp + mi * 64 * stride + (ni * 32 + 8 * q) * 2) = v;
        }
  }
  __syncthreads();
  {
    constexpr int chunks = kBN >> 3, rows_per_pass = kThreads / chunks;
    const int c = tid % chunks;
    if (n0 + c * 8 < args.Nd) {
      T *p = (T *)args.C + ((long long)expert * args.Md + m0) * args.Nd + n0 + c * 8;
      for (int r = tid / chunks; r < rows_m; r += rows_per_pass) {
        // streaming stores: 1.6 GB of gradients per backward pass that nobody reads back soon would otherwise push the
        // operand tiles out of L2
        __builtin_nontemporal_store(*(const u32x4 *)(lds + r * stride + c * 16), (u32x4 *)(p + (long long)r * args.Nd));
      }
      // the row below the valid ones: the column sums
      if (bias_tile && tid < chunks)
        *(u32x4 *)((T *)args.bias_grad + (long long)expert * args.Nd + n0 + c * 8) = *(const u32x4 *)(lds + rows_m * stride + c * 16);
    }
  }
}

template <typename T, bool GATHER>
__global__ __launch_bounds__(kThreads, 2) void wgrad_small_kernel(const WgradArgs args) {
  const int tid = threadIdx.x, wave = tid >> 6, wm = wave >> 1;
  const int per_expert = args.n_m_tiles * args.n_n_tiles;
  const int total = args.E * per_expert;
  const int total8 = (total + kXcds - 1) / kXcds * kXcds;
  const int b = blockIdx.x;
  if (b >= total8) return;
  const int L = (b % kXcds) * (total8 / kXcds) + b / kXcds;
  if (L >= total) return;
  const int expert = L / per_expert, r = L - expert * per_expert;
  const int n0 = (r / args.n_m_tiles) * kBN, m0 = (r % args.n_m_tiles) * kSmallBM;
  const int rows_m = min(kSmallBM, args.Md - m0);
  // (the same for every lane; said explicitly, so that the operand addresses built from them stay in scalar registers)
  int rows = min(__builtin_amdgcn_readfirstlane(args.counts[expert]), args.capacity);
  if (rows < 0) rows = 0;
  const long long first = __builtin_amdgcn_readfirstlane(args.offsets[expert]);
  const bool bias_tile = args.bias_grad != nullptr && rows_m < kSmallBM;  // (the last row tile; see wgrad_writes_bias)
  const int n_blocks32 = (rows_m + (bias_tile ? 1 : 0) + 31) >> 5;
  const int n_mi = (n_blocks32 - wm + 1) >> 1;
  switch (n_mi) {
    case 2: run_wgrad_tile_small<T, 2, GATHER>(args, tid, expert, m0, n0, rows_m, first, rows, bias_tile); break;
    case 1: run_wgrad_tile_small<T, 1, GATHER>(args, tid, expert, m0, n0, rows_m, first, rows, bias_tile); break;
    default: run_wgrad_tile_small<T, 0, GATHER>(args, tid, expert, m0, n0, rows_m, first, rows, bias_tile); break;
  }
}

}  // namespace async

#ifdef YAMOE_TILE_STAMPS
// Where the next launches of gemm_async_kernel leave their per-tile clock stamps (device memory, 8 words per tile, room
// for `tiles` tiles; nullptr switches them off).  Exported by the diagnostic build only.
extern "C" void yamoe_debug_tile_stamps(void *buffer, int32_t tiles) {
  async::g_tile_stamps = (unsigned long long *)buffer;
  async::g_tile_stamps_cap = buffer ? tiles : 0;
}
#endif

// True when the asynchronous-copy kernels can take this product.
bool gemm_async_supported(int Kd, int Nd, int lda, int ldb, long long a_span_bytes) {
  return Kd % (2 * async::kBK) == 0 && Kd >= 2 * async::kBK && Nd % 8 == 0 && lda % 8 == 0 && ldb % 8 == 0 &&
         a_span_bytes < (1ll << 32);
}

template <typename T>
int gemm_async_gate_up(const void *x, const int *sorted_idx, const void *w, const void *bias, void *act, void *pre,
                       const void *sched, int N, int K, int E, int H, int I, int small_rows, hipStream_t stream) {
  async::Args a = {};
  a.A = x; a.B = w; a.bias = bias; a.C = act; a.C2 = pre;
  a.a_rows = sorted_idx; a.a_div = make_fast_div(K); a.sched = (const int *)sched;
  a.Kd = H; a.Nd = 2 * I; a.lda = H; a.ldb = 2 * I; a.ldc = I;
  a.b_expert_stride = (long long)H * 2 * I;
  a.n_col_tiles = ceil_div(2 * I, async::kBN);
  a.n_col_div = make_fast_div(a.n_col_tiles);
  a.band_div = make_fast_div(async::kBandRows * a.n_col_tiles);
  return async::launch<T, async::EPI_GLU, true, false>(a, sched_grid_row_tiles(N, E, small_rows), stream);
}

template <typename T>
int gemm_async_down(const void *act, const void *w, const void *bias, void *y, const void *sched, int N, int E, int H,
                    int I, int small_rows, hipStream_t stream) {
  async::Args a = {};
  a.A = act; a.B = w; a.bias = bias; a.C = y; a.sched = (const int *)sched;
  a.Kd = I; a.Nd = H; a.lda = I; a.ldb = H; a.ldc = H;
  a.b_expert_stride = (long long)I * H;
  a.n_col_tiles = ceil_div(H, async::kBN);
  a.n_col_div = make_fast_div(a.n_col_tiles);
  a.band_div = make_fast_div(async::kBandRows * a.n_col_tiles);
  return async::launch<T, async::EPI_STORE, false, false>(a, sched_grid_row_tiles(N, E, small_rows), stream);
}

// C[rows, Nd] = A[rows, Kd] * W[e]^T with W[e] stored [Nd, Kd]: the input gradients of both projections
// (csrc/experts_backward.cu:279-282, 309-311), without materialising a transposed weight.
// With g_rows the source row of sorted row p is g_rows[p] / g_div (rows of a [T, Kd] tensor gathered by token).
template <typename T>
int gemm_async_dgrad(const void *g, const int *g_rows, int g_div, const void *w, void *out, const void *sched, int N,
                     int E, int Kd, int Nd, const void *dot_with, float *dot_part, hipStream_t stream) {
  async::Args a = {};
  a.A = g; a.B = w; a.bias = nullptr; a.C = out; a.sched = (const int *)sched;
  a.dot_with = dot_with; a.dot_part = dot_part;
  a.a_rows = g_rows; a.a_div = make_fast_div(g_rows != nullptr ? g_div : 1);
  a.Kd = Kd; a.Nd = Nd; a.lda = Kd; a.ldb = Kd; a.ldc = Nd;
  a.b_expert_stride = (long long)Nd * Kd;
  a.n_col_tiles = ceil_div(Nd, async::kBN);
  a.n_col_div = make_fast_div(a.n_col_tiles);
  a.band_div = make_fast_div(async::kBandRows * a.n_col_tiles);
  if (g_rows != nullptr) return async::launch<T, async::EPI_STORE, true, true>(a, sched_max_row_tiles(N, E), stream);
  return async::launch<T, async::EPI_STORE, false, true>(a, sched_max_row_tiles(N, E), stream);
}

// dW[E, Md, Nd] = per expert L^T R over its kept rows.  Both operand buffers must stay readable for 32 rows past
// their last row (the copies of a partial last slab run over; what they fetch is zeroed before use).
bool wgrad_async_supported(int Md, int Nd) { return Md % 8 == 0 && Nd % 8 == 0; }
// True when gemm_async_wgrad can leave the bias gradient (the column sums of the right operand's rows per expert) next
// to the weight gradient: its last 128-row tile of the Md output rows must have a spare row.
bool wgrad_writes_bias(int Md, int Nd) { return wgrad_async_supported(Md, Nd) && Md % async::kSmallBM != 0; }

namespace async {
template <typename T, bool GATHER> static int launch_wgrad(const WgradArgs &a, hipStream_t stream) {
  auto kernel = wgrad_small_kernel<T, GATHER>;
  static DeviceFlags attr_done;  // one per kernel instantiation
  if (int rc = ensure_dynamic_lds((const void *)kernel, kSmallLds, attr_done, "wgrad_small_kernel")) return rc;
  long long total = (long long)a.E * a.n_m_tiles * a.n_n_tiles;
  if (total <= 0) return 0;
  total = (total + kXcds - 1) / kXcds * kXcds;
  hipLaunchKernelGGL(kernel, dim3((unsigned)total), dim3(kThreads), kSmallLds, stream, a);
  return check_launch("wgrad_small_kernel");
}
}  // namespace async

// With l_rows the left operand is not in expert order: sorted row p is row l_rows[p] / l_div of L (rows of a
// [n_rows / l_div, Md] tensor gathered by token, which must span less than 4 GiB); l_rows holds n_rows values below
// n_rows and must stay readable for 32 values more, and L needs no readable rows past its end.
template <typename T>
int gemm_async_wgrad(const void *L, const int *l_rows, int l_div, int n_rows, const void *R, void *dW, void *d_bias,
                     const int *counts, const int *offsets, int capacity, int E, int Md, int Nd, hipStream_t stream) {
  if (d_bias != nullptr && !wgrad_writes_bias(Md, Nd)) {
    set_error("gemm_async_wgrad: no spare row for the bias gradient at Md = %d", Md);
    return YAMOE_E_ARG;
  }
  async::WgradArgs a = {};
  a.A = L; a.B = R; a.C = dW; a.counts = counts; a.offsets = offsets; a.capacity = capacity; a.bias_grad = d_bias;
  a.a_rows = l_rows; a.a_div = make_fast_div(l_rows != nullptr ? l_div : 1); a.a_rows_max = n_rows > 0 ? n_rows - 1 : 0;
  a.E = E; a.Md = Md; a.Nd = Nd;
  a.n_m_tiles = ceil_div(Md, async::kSmallBM);
  a.n_n_tiles = ceil_div(Nd, async::kBN);
  if (l_rows != nullptr) return async::launch_wgrad<T, true>(a, stream);
  return async::launch_wgrad<T, false>(a, stream);
}

#define YAMOE_INSTANTIATE_ASYNC(T)                                                                               \
  template int gemm_async_gate_up<T>(const void *, const int *, const void *, const void *, void *, void *,      \
                                     const void *, int, int, int, int, int, int, hipStream_t);                   \
  template int gemm_async_down<T>(const void *, const void *, const void *, void *, const void *, int, int, int, \
                                  int, int, hipStream_t);                                                             \
  template int gemm_async_dgrad<T>(const void *, const int *, int, const void *, void *, const void *, int, int, int,  \
                                   int, const void *, float *, hipStream_t);                                           \
  template int gemm_async_wgrad<T>(const void *, const int *, int, int, const void *, void *, void *, const int *,     \
                                   const int *, int, int, int, int, hipStream_t);
YAMOE_INSTANTIATE_ASYNC(bf16_t)
YAMOE_INSTANTIATE_ASYNC(f16_t)

}  // namespace yamoe
