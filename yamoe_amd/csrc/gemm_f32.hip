// Grouped expert GEMMs of the forward for fp32 data on gfx950 (the README workload of drbh/yamoe, README.md:67-112;
// replaces batch_mm, csrc/batch_mm.cu:7-31, plus the bias / clamped-SwiGLU chain, csrc/moe.cpp:161-187).
//
// The fp32 matrix instruction (v_mfma_f32_32x32x2_f32, 64 clocks for 4096 flop) is sixteen times slower per
// contraction step than the 16-bit ones, so a tile's operands are cheap next to its arithmetic and the design goes
// the other way from the 16-bit kernels: small tiles, many of them, two workgroups per CU.
//
//  * 128 x 128 output tile, 4 wavefronts 2 x 2, each 64 x 64 (four 32 x 32 accumulator blocks, 64 registers): a
//    256-row tile of the schedule is two of these on top of each other, and a GEMM has four times the tiles of the
//    256 x 256 form, so the last, partly filled round of tiles per CU is a quarter as long (the down projection of
//    the README workload has 1.5 tiles of 256 x 256 per CU: a quarter of the chip idles through its second round).
//  * Operands go global -> LDS with asynchronous 16-byte copies (no staging registers), two stages of 32 KB, one
//    workgroup barrier per slab of 32 (16 000 clocks of matrix work): while a workgroup waits at its barrier or
//    runs its epilogue, the other workgroup on the CU keeps the matrix pipe busy.
//  * Activations [row][k] keep that layout in LDS (128-byte rows, 16-byte pieces XOR-swizzled with the row number
//    on the global side of the copy); a lane's 16-byte read holds four contraction steps.
//  * Weights [k][n] keep that layout too and need no transpose: a lane's operand for one instruction is ONE value,
//    B[k][n of the lane], so an 8-byte read of row k gives a lane columns 2l and 2l+1, i.e. the B operands of the
//    wave's "even" and "odd" accumulator blocks.  The interleaved (gate, up) columns of the clamped SwiGLU
//    therefore meet in one lane, and plain outputs leave as 8-byte stores, 256 contiguous bytes per half wave.
//
// Requirements: contraction length a multiple of 32, leading dimensions multiples of 4 elements; gemm.hip takes
// everything else.
#include "common.h"

namespace yamoe {

namespace f32 {

constexpr int kBM = 128, kBN = 128, kBK = 32;
constexpr int kThreads = 256;
constexpr int kAStage = kBM * kBK * 4;  // 16 KB: 128 rows x 128 bytes
constexpr int kBStage = kBK * kBN * 4;  // 16 KB: 32 k rows x 512 bytes
constexpr int kStage = kAStage + kBStage;
constexpr int kStages = 2;
constexpr int kLds = kStages * kStage;  // 64 KB: two workgroups per CU

static_assert(kRowTile == 2 * kBM, "a row tile of the schedule is two tiles of this kernel");

enum { EPI_STORE = 0, EPI_GLU = 1 };

struct Args {
  const float *A;      // [rows, lda], k-contiguous
  const float *B;      // [E, Kd, Nd]
  const float *bias;   // [E, Nd] or null
  float *C;            // EPI_STORE: [rows, ldc]; EPI_GLU: act [rows, Nd/2]
  float *C2;           // EPI_GLU: optional pre-activations [rows, Nd]
  const int *a_rows;   // optional gather of A rows: source row = a_rows[p] / a_div
  const int *sched;
  int a_div, Kd, Nd, lda, ldb, ldc, n_col_tiles;
  long long b_expert_stride;
};

template <int EPI, bool GATHER>
__global__ __launch_bounds__(kThreads, 2) void gemm_f32_kernel(const Args args) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int rl = lane & 31, g = lane >> 5;

  // ---- which tile: half h of row tile t of the schedule, column tile c.  Tiles run expert-major, then column tile,
  // then the expert's row halves, so the tiles in flight on one XCD share weight columns through its L2; workgroup
  // ids are dealt round-robin over the XCDs, so id b takes logical tile (b % 8) * per_xcd + b / 8.
  int expert, row0, rows_valid, n0;
  {
    const int n_halves = 2 * args.sched[0];
    const int total = n_halves * args.n_col_tiles;
    const int total8 = (total + kXcds - 1) / kXcds * kXcds;
    const int b = blockIdx.x;
    if (b >= total8) return;
    const int L = (b % kXcds) * (total8 / kXcds) + b / kXcds;
    if (L >= total) return;
    const int *tiles = args.sched + kSchedHeader;
    const int t0 = (L / args.n_col_tiles) >> 1;
    const int gfirst = 2 * tiles[8 * t0 + 3], gcount = 2 * tiles[8 * t0 + 4];
    const int local = L - gfirst * args.n_col_tiles;
    const int col_tile = local / gcount;
    const int vt = gfirst + local - col_tile * gcount;
    const int *te = tiles + 8 * (vt >> 1);
    const int h = vt & 1;
    expert = te[0];
    row0 = te[1] + h * kBM;
    rows_valid = min(te[2] - h * kBM, kBM);
    n0 = col_tile * kBN;
    if (rows_valid <= 0) return;  // the lower half of a row tile of at most 128 rows
  }
  const int cols_valid = min(kBN, args.Nd - n0);

  // ---- copies.  A: copy i (0..3) fetches rows 32*i + 8*wave + (lane >> 3), 16 bytes of each; LDS position
  // lane & 7 of the row holds piece pos ^ ((row >> 1) & 7).  B: copy i fetches k rows 8*wave + 2*i + (lane >> 5),
  // piece lane & 31 (no swizzle: a half wave reads 256 contiguous bytes of one k row).
  // (a gathering instantiation without a row list reads its rows in order: see gemm_async.hip)
  const bool gathers = GATHER && args.a_rows != nullptr;
  uint32_t a_off[4], b_off[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = 32 * i + 8 * wave + (lane >> 3);
    const int piece = (lane & 7) ^ ((row >> 1) & 7);
    const int r = min(row, rows_valid - 1);  // rows past the end re-read the last one; never stored
    long long src = r;
    if (gathers) src = args.a_rows[row0 + r] / args.a_div;
    a_off[i] = (uint32_t)((src * args.lda + piece * 4) * 4);
    const int k = 8 * wave + 2 * i + (lane >> 5);
    int col = (lane & 31) * 4;
    if (col >= cols_valid) col = 0;  // columns past the end re-read valid ones; never stored
    b_off[i] = (uint32_t)(((long long)k * args.ldb + col) * 4);
  }
  const char *a_base = (const char *)(args.A + (gathers ? 0ll : (long long)row0 * args.lda));
  const char *b_base = (const char *)(args.B + (long long)expert * args.b_expert_stride + n0);
  const long long b_slab_bytes = (long long)kBK * args.ldb * 4;
  const uint32_t lds0 = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)lds);
  auto issue = [&](int slab) {
    const uint32_t st = lds0 + (uint32_t)(slab & (kStages - 1)) * kStage;
    const char *ab = a_base + (long long)slab * (kBK * 4);
    const char *bb = b_base + (long long)slab * b_slab_bytes;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      copy16_to_lds(ab, a_off[i], st + (uint32_t)(32 * i + 8 * wave) * 128u);
      copy16_to_lds(bb, b_off[i], st + kAStage + (uint32_t)(8 * wave + 2 * i) * 512u);
    }
  };

  // ---- accumulators: acc[mi][par][v] = row wm*64 + mi*32 + 8*(v/4) + 4*g + v%4, column wn*64 + 2*rl + par
  f32x16 acc[2][2];
#pragma unroll
  for (int mi = 0; mi < 2; ++mi)
#pragma unroll
    for (int par = 0; par < 2; ++par)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[mi][par][v] = 0.0f;

  // A operand of block mi in k-step ks (8 contraction steps): row wm*64 + mi*32 + rl, piece 2*ks + g; the four
  // values of the piece feed four instructions, in which the lanes of half g hold k = 8*ks + 4*g + q.
  const int a_row = wm * 64 + rl;
  int a_rd[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) a_rd[ks] = a_row * 128 + (((2 * ks + g) ^ ((a_row >> 1) & 7)) << 4);
  // (rows a_row and a_row + 32 share (row >> 1) & 7, so block mi = 1 is the same offset 4096 bytes further)
  const int b_rd = g * 4 * 512 + (wn * 64 + 2 * rl) * 4;  // k = 4*g (+ 8*ks + q), columns 2*rl and 2*rl + 1 of the wave's 64
  // waves whose 64 columns lie past the end of the matrix, and 32-row blocks past the end of the rows, do no arithmetic
  const bool active_n = wn * 64 < cols_valid;
  const int n_mi = !active_n ? 0 : (rows_valid > wm * 64 + 32 ? 2 : (rows_valid > wm * 64 ? 1 : 0));

  const int n_slabs = args.Kd / kBK;
  issue(0);
  for (int s = 0; s < n_slabs; ++s) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();  // slab s has landed for every wave, and nobody reads the other stage any more
    if (s + 1 < n_slabs) issue(s + 1);
    const char *sa = lds + (s & (kStages - 1)) * kStage;
    const char *sb = sa + kAStage;
    if (n_mi > 0) {
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        f32x4 fa[2];
        fa[0] = *(const f32x4 *)(sa + a_rd[ks]);
        fa[1] = *(const f32x4 *)(sa + a_rd[ks] + 32 * 128);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          typedef float f32x2 __attribute__((ext_vector_type(2)));
          const f32x2 fb = *(const f32x2 *)(sb + b_rd + (8 * ks + q) * 512);
          acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[0][q], fb[0], acc[0][0], 0, 0, 0);
          acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[0][q], fb[1], acc[0][1], 0, 0, 0);
          if (n_mi > 1) {
            acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[1][q], fb[0], acc[1][0], 0, 0, 0);
            acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[1][q], fb[1], acc[1][1], 0, 0, 0);
          }
        }
      }
    }
  }

  // ---- epilogue: straight from the accumulators; a half wave covers 256 (128 for act) contiguous bytes of a row
  if (n_mi == 0) return;
  const int col = n0 + wn * 64 + 2 * rl;  // even: the gate column of pair col / 2
  if (col >= args.Nd) return;
  float b0 = 0.0f, b1 = 0.0f;
  if (args.bias != nullptr) {
    const float *bp = args.bias + (long long)expert * args.Nd + col;
    b0 = bp[0];
    b1 = bp[1];
  }
  typedef float f32x2 __attribute__((ext_vector_type(2)));
#pragma unroll
  for (int mi = 0; mi < 2; ++mi) {
    if (mi < n_mi) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int r = wm * 64 + mi * 32 + 8 * (v >> 2) + 4 * g + (v & 3);
        if (r < rows_valid) {
          const long long orow = row0 + r;
          const float x0 = acc[mi][0][v] + b0, x1 = acc[mi][1][v] + b1;
          if constexpr (EPI == EPI_STORE) {
            *(f32x2 *)(args.C + orow * args.ldc + col) = (f32x2){x0, x1};
          } else {
            args.C[orow * args.ldc + (col >> 1)] = glu_forward(x0, x1);
            if (args.C2 != nullptr) *(f32x2 *)(args.C2 + orow * args.Nd + col) = (f32x2){x0, x1};
          }
        }
      }
    }
  }
}

template <int EPI, bool GATHER>
static int launch(const Args &args, int max_row_tiles, hipStream_t stream) {
  auto kernel = gemm_f32_kernel<EPI, GATHER>;
  static DeviceFlags attr_done;  // one per kernel instantiation
  if (int rc = ensure_dynamic_lds((const void *)kernel, kLds, attr_done, "gemm_f32_kernel")) return rc;
  long long total = 2ll * max_row_tiles * args.n_col_tiles;
  if (total <= 0) return 0;
  total = (total + kXcds - 1) / kXcds * kXcds;
  hipLaunchKernelGGL(kernel, dim3((unsigned)total), dim3(kThreads), kLds, stream, args);
  return check_launch("gemm_f32_kernel");
}

}  // namespace f32

// True when the fp32 asynchronous-copy kernel can take this product (a_span_bytes: size of the tensor that gathered
// rows are addressed in, 0 without a gather).
bool gemm_f32_supported(int Kd, int Nd, int lda, int ldb, long long a_span_bytes) {
  return Kd % f32::kBK == 0 && Kd >= f32::kBK && Nd % 4 == 0 && lda % 4 == 0 && ldb % 4 == 0 && a_span_bytes < (1ll << 32);
}

int gemm_f32_gate_up(const void *x, const int *sorted_idx, const void *w, const void *bias, void *act, void *pre,
                     const void *sched, int N, int K, int E, int H, int I, hipStream_t stream) {
  f32::Args a = {};
  a.A = (const float *)x; a.B = (const float *)w; a.bias = (const float *)bias; a.C = (float *)act; a.C2 = (float *)pre;
  a.a_rows = sorted_idx; a.a_div = K; a.sched = (const int *)sched;
  a.Kd = H; a.Nd = 2 * I; a.lda = H; a.ldb = 2 * I; a.ldc = I;
  a.b_expert_stride = (long long)H * 2 * I;
  a.n_col_tiles = ceil_div(2 * I, f32::kBN);
  return f32::launch<f32::EPI_GLU, true>(a, sched_max_row_tiles(N, E), stream);
}

int gemm_f32_down(const void *act, const void *w, const void *bias, void *y, const void *sched, int N, int E, int H,
                  int I, hipStream_t stream) {
  f32::Args a = {};
  a.A = (const float *)act; a.B = (const float *)w; a.bias = (const float *)bias; a.C = (float *)y;
  a.sched = (const int *)sched; a.a_div = 1;
  a.Kd = I; a.Nd = H; a.lda = I; a.ldb = H; a.ldc = H;
  a.b_expert_stride = (long long)I * H;
  a.n_col_tiles = ceil_div(H, f32::kBN);
  return f32::launch<f32::EPI_STORE, false>(a, sched_max_row_tiles(N, E), stream);
}

}  // namespace yamoe
