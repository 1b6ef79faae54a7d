// Routing for the expert layer: a stable counting sort of the N = T*K (token, slot) assignments by
// expert id, the per-expert counts and exclusive offsets, the inverse permutation, and the work
// lists the expert GEMM kernels walk.
//
// Replaces cub::DeviceRadixSort::SortPairs (csrc/sort.cu:17-91) and bincount_cumsum_kernel
// (csrc/bincount_cumsum.cu:7-56).  The keys have ceil(log2 E) meaningful bits, so one counting pass
// is enough: the input is cut into contiguous segments, one per wavefront; each wave histograms
// its segment, a scan turns (expert-major, segment-minor) counts into write cursors, and each wave
// then walks its segment in order and places every element at cursor[expert] + (number of equal
// keys in lower lanes of the same 64-element step), found with wavefront ballots.  Walking in order
// and ranking by lane keeps equal keys in input order, i.e. the sort is stable.
#include "common.h"

namespace yamoe {

constexpr int kRouteThreads = 1024;
constexpr int kRouteWaves = kRouteThreads / kWave;
constexpr int kRouteMaxBuckets = 769;    // E + 1 must not exceed this (keeps dynamic LDS under 64 KB)
constexpr int kSingleBlockMaxN = 32768;  // the single-workgroup kernel's limit (its keys sit in LDS as 16-bit values)
constexpr int kSingleBlockN = 4096;      // up to this many assignments the single-workgroup kernel is used

template <bool I64>
__device__ inline int load_key(const void *idx, int i, int E) {
  long long v = I64 ? ((const long long *)idx)[i] : (long long)((const int *)idx)[i];
  // ids outside [0,E) go to bucket E, after every valid expert
  return (v < 0 || v >= E) ? E : (int)v;
}
template <bool I64>
__device__ inline int load_raw(const void *idx, int i) {
  return I64 ? (int)((const long long *)idx)[i] : ((const int *)idx)[i];
}

// Lanes of this wave whose key equals mine (only among lanes with `active`).
__device__ inline uint64_t match_key(int key, bool active, int key_bits) {
  uint64_t peers = __ballot(active);
  for (int b = 0; b < key_bits; ++b) {
    bool bit = (key >> b) & 1;
    uint64_t m = __ballot(active && bit);
    peers &= bit ? m : ~m;
  }
  return peers;
}

__device__ inline int bits_for(int buckets) {
  int b = 0;
  while ((1 << b) < buckets) ++b;
  return b;
}

// Histogram of one wave's segment [seg_begin, seg_end) into `hist` (LDS or global, zeroed by caller).
template <bool I64>
__device__ inline void wave_histogram(const void *idx, int seg_begin, int seg_end, int E,
                                      int *hist_lds) {
  const int lane = threadIdx.x & (kWave - 1);
  for (int i = seg_begin + lane; i < seg_end; i += kWave) {
    int key = load_key<I64>(idx, i, E);
    atomicAdd(&hist_lds[key], 1);
  }
}

// Walk one segment in order and place its elements.  `cursor` (LDS, private to this wave) holds
// the next free sorted position per bucket.
template <bool I64>
__device__ inline void wave_place(const void *idx, int seg_begin, int seg_end, int E, int capacity,
                                  int *cursor, const int *offsets_lds,
                                  int *sorted_expert, int *sorted_idx, int *inv_pos) {
  const int lane = threadIdx.x & (kWave - 1);
  const int key_bits = bits_for(E + 1);
  const uint64_t lt_mask = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
  // the raw id of the next step is fetched one step ahead so that its latency hides behind this step
  int raw_next = (seg_begin + lane < seg_end) ? load_raw<I64>(idx, seg_begin + lane) : 0;
  bool bad_next = (seg_begin + lane < seg_end) ? (load_key<I64>(idx, seg_begin + lane, E) == E) : false;
  for (int base = seg_begin; base < seg_end; base += kWave) {
    int i = base + lane;
    bool active = i < seg_end;
    int raw = raw_next;
    int key = bad_next ? E : raw;
    if (!active) key = 0;
    int in = i + kWave;
    if (in < seg_end) {
      raw_next = load_raw<I64>(idx, in);
      bad_next = load_key<I64>(idx, in, E) == E;
    }
    uint64_t peers = match_key(key, active, key_bits);
    int rank = __popcll(peers & lt_mask);
    int start = 0;
    if (active) start = cursor[key];
    __builtin_amdgcn_wave_barrier();
    if (active) {
      int pos = start + rank;
      sorted_expert[pos] = raw;
      sorted_idx[pos] = i;
      bool kept = key < E && (pos - offsets_lds[key]) < capacity;
      inv_pos[i] = kept ? pos : -1;
      if (rank == 0) cursor[key] = start + __popcll(peers);
    }
    // the cursor is private to this wave and LDS operations of one wave complete in order: the next step's
    // read sees this step's write without a fence or a volatile access (both would also wait for the global
    // stores above); lanes address the cursor by key, so the compiler cannot carry its values across steps
    __builtin_amdgcn_wave_barrier();
  }
}

// Exclusive scan over buckets of `total` into `offsets` (both LDS), done by the whole block.
// offsets[b] for b in [0, buckets]; offsets[buckets] = N.
__device__ inline void block_exclusive_scan(const int *total, int *offsets, int buckets,
                                            int *scratch /* kRouteWaves + 1 ints */) {
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  int carry = 0;
  for (int base = 0; base < buckets; base += blockDim.x) {
    int b = base + tid;
    int v = (b < buckets) ? total[b] : 0;
    // inclusive scan inside the wave
    int x = v;
    for (int d = 1; d < kWave; d <<= 1) {
      int y = __shfl_up(x, d);
      if (lane >= d) x += y;
    }
    if (lane == kWave - 1) scratch[wave] = x;
    __syncthreads();
    int wave_off = 0;
    for (int w = 0; w < wave; ++w) wave_off += scratch[w];
    int chunk_total = 0;
    for (int w = 0; w < (int)(blockDim.x / kWave); ++w) chunk_total += scratch[w];
    if (b < buckets) offsets[b] = carry + wave_off + x - v;
    carry += chunk_total;
    __syncthreads();
  }
  if (tid == 0) offsets[buckets] = carry;
  __syncthreads();
}

// ---- work lists ------------------------------------------------------------------------------
// One wave; lane l takes experts l, l+64, ...  Experts with 1..stream_max_rows kept rows go to the
// streaming list, larger ones are cut into row tiles of kRowTile rows.  Both lists stay in expert
// order: positions come from wave prefix sums.
__device__ inline int wave_exclusive_scan(int v, int lane, int &total) {
  int x = v;
  for (int d = 1; d < kWave; d <<= 1) {
    int y = __shfl_up(x, d);
    if (lane >= d) x += y;
  }
  total = __shfl(x, kWave - 1);
  return x - v;
}

__device__ inline void build_schedule_wave(const int *counts, const int *offsets, int N, int E, int capacity,
                                           int stream_max_rows, int *sched, const int lane) {
  int *row_tiles = sched + kSchedHeader;
  int *small = row_tiles + 8 * sched_max_row_tiles(N, E);
  int n_tiles = 0, n_small = 0, n_active = 0, n_kept = 0;
  // Experts of 17 to 32 rows stream only when every expert streams: next to experts that need the tile kernels anyway
  // they are better off as tiles (two half-filled launches one after the other are slower than one: 0.35 against
  // 0.31 ms for 32 experts of about 32 rows, where 0.27 against 0.31 ms is gained when all of them have at most 32).
  const bool everything = stream_max_rows == kStreamEverything;  // (the host checked sched_may_stream_everything)
  if (everything) stream_max_rows = kStreamMaxRows;
  if (!everything && stream_max_rows > kStreamMixedRows) {
    int most = 0;
    for (int base = 0; base < E; base += kWave) {
      int e = base + lane;
      int kept = e < E ? min(counts[e], capacity) : 0;
      most = max(most, kept);
    }
    for (int d = kWave / 2; d > 0; d >>= 1) most = max(most, __shfl_xor(most, d));
    if (most > stream_max_rows) stream_max_rows = kStreamMixedRows;
  }
  for (int base = 0; base < E; base += kWave) {
    int e = base + lane;
    int kept = e < E ? min(counts[e], capacity) : 0;
    if (kept < 0) kept = 0;
    int first = e < E ? offsets[e] : 0;
    // entries on the streaming list: one, or with `everything` one per chunk of kStreamMaxRows rows
    int is_small = everything ? ceil_div(kept, kStreamMaxRows) : (kept > 0 && kept <= stream_max_rows);
    int tiles = (kept > 0 && !is_small) ? ceil_div(kept, kRowTile) : 0;
    int tot_small, tot_tiles, tot_active, tot_kept;
    int pos_small = wave_exclusive_scan(is_small, lane, tot_small);
    int pos_tiles = wave_exclusive_scan(tiles, lane, tot_tiles);
    wave_exclusive_scan(kept > 0 ? 1 : 0, lane, tot_active);
    wave_exclusive_scan(kept, lane, tot_kept);
    for (int c = 0; c < is_small; ++c) {
      int *s = small + 4 * (n_small + pos_small + c);
      s[0] = e; s[1] = first + c * kStreamMaxRows; s[2] = min(kStreamMaxRows, kept - c * kStreamMaxRows); s[3] = 0;
    }
    int gfirst = n_tiles + pos_tiles;
    // An expert's rows are cut into equal tiles (a multiple of 32 rows, the MFMA block), not into full
    // tiles plus a remainder: tiles of one expert then advance through the contraction at the same pace
    // and the weight slabs one of them fetches are still in L2 when the others ask for them.
    int per_tile = tiles > 0 ? min(kRowTile, (ceil_div(kept, tiles) + 31) & ~31) : 0;
    const FastDiv by_tiles = make_fast_div(tiles > 0 ? tiles : 1);  // the GEMM kernels divide by the group size
    for (int t = 0; t < tiles; ++t) {
      int *w = row_tiles + 8 * (gfirst + t);
      w[0] = e; w[1] = first + t * per_tile; w[2] = min(per_tile, kept - t * per_tile); w[3] = gfirst; w[4] = tiles;
      w[5] = (int)by_tiles.mul; w[6] = (int)by_tiles.shift; w[7] = 0;
    }
    n_small += tot_small; n_tiles += tot_tiles; n_active += tot_active; n_kept += tot_kept;
  }
  // Second pass: cut the tile list into 8 shares of equal cost.  Groups (experts with row tiles) are weighed
  // by the sum of their tiles' weights; cut x falls into the group that contains x/8 of the total.
  int w_total = 0;
  for (int pass = 0; pass < 2; ++pass) {
    int w_before = 0, t_before = 0;
    for (int base = 0; base < E; base += kWave) {
      int e = base + lane;
      int kept = e < E ? min(counts[e], capacity) : 0;
      if (kept < 0) kept = 0;
      int is_small = everything || (kept > 0 && kept <= stream_max_rows);
      int tiles = (kept > 0 && !is_small) ? ceil_div(kept, kRowTile) : 0;
      int per_tile = tiles > 0 ? min(kRowTile, (ceil_div(kept, tiles) + 31) & ~31) : 0;
      int w = sched_group_weight(tiles, per_tile, kept);
      int tot_w, tot_t;
      int w_pre = w_before + wave_exclusive_scan(w, lane, tot_w);
      int t_pre = t_before + wave_exclusive_scan(tiles, lane, tot_t);
      if (pass == 1 && tiles > 0) {
        for (int x = 0; x < kXcds; ++x) {
          long long t = (long long)x * w_total;  // compare x * W / 8 with the group's weight interval, times 8
          if (t >= 8ll * w_pre && t < 8ll * (w_pre + w)) {
            int *c = sched + kSchedCuts + 4 * x;
            c[0] = t_pre; c[1] = (int)(((t - 8ll * w_pre) << 16) / (8ll * w)); c[2] = 0; c[3] = tiles;
          }
        }
      }
      w_before += tot_w; t_before += tot_t;
    }
    if (pass == 0) w_total = w_before;
  }
  if (lane == 0) {
    sched[0] = n_tiles; sched[1] = n_small; sched[2] = n_active; sched[3] = n_kept;
    sched[4] = w_total; sched[5] = 0; sched[6] = 0; sched[7] = 0;
    int *c = sched + kSchedCuts + 4 * kXcds;  // the end of the list
    c[0] = n_tiles; c[1] = 0; c[2] = 0; c[3] = 0;
    if (w_total == 0)
      for (int x = 0; x < kXcds; ++x) { int *cx = sched + kSchedCuts + 4 * x; cx[0] = 0; cx[1] = 0; cx[2] = 0; cx[3] = 0; }
    for (int i = kSchedCuts + 4 * (kXcds + 1); i < kSchedHeader; ++i) sched[i] = 0;
  }
}

__global__ __launch_bounds__(kWave) void build_schedule_kernel(const int *counts, const int *offsets, int N, int E,
                                                               int capacity, int stream_max_rows, int *sched) {
  build_schedule_wave(counts, offsets, N, E, capacity, stream_max_rows, sched, threadIdx.x);
}

// ---- single-block form: everything in one launch -------------------------------------------------
// Dynamic LDS: hist[kRouteWaves][buckets] + total[buckets] + offsets[buckets+1] + scratch + the N keys as 16-bit
// values.  The kernel runs once per forward on a cold instruction cache, so its loops stay rolled (straight-line
// code would run at instruction-fetch speed); the keys are read from memory once and kept in LDS for the
// placement pass.
__host__ __device__ inline size_t route_single_lds_bytes(int N, int buckets) {
  size_t ints = (size_t)kRouteWaves * buckets + buckets + buckets + 1 + kRouteWaves + 1;
  return align_up(ints * sizeof(int), 16) + align_up((size_t)(N > 0 ? N : 1) * sizeof(unsigned short), 16);
}

template <bool I64>
__global__ __launch_bounds__(kRouteThreads) void route_single_kernel(
    const void *idx, int N, int E, int capacity, int *sorted_expert, int *sorted_idx, int *counts,
    int *offsets_out, int *inv_pos, int *sched, int stream_max_rows) {
  extern __shared__ int lds[];
  const int buckets = E + 1;
  int *hist = lds;                          // [kRouteWaves][buckets]
  int *total = hist + kRouteWaves * buckets;  // [buckets]
  int *offs = total + buckets;              // [buckets + 1]
  int *scratch = offs + buckets + 1;        // [kRouteWaves + 1]
  unsigned short *keys = (unsigned short *)((char *)lds + align_up(((size_t)kRouteWaves * buckets + 2 * buckets + 1 +
                                                                   kRouteWaves + 1) * sizeof(int), 16));
  const int tid = threadIdx.x, wave = tid / kWave, lane = tid & (kWave - 1);

  for (int i = tid; i < kRouteWaves * buckets; i += blockDim.x) hist[i] = 0;
  __syncthreads();

  int seg = ceil_div(ceil_div(N, kRouteWaves), kWave) * kWave;
  int seg_begin = min(wave * seg, N), seg_end = min(seg_begin + seg, N);
  {
    // four loads in flight per lane; positions past the end are clamped, their keys dropped
    int *h = hist + wave * buckets;
    for (int base = seg_begin; base < seg_end; base += 4 * kWave) {
      int k[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) k[u] = load_key<I64>(idx, min(base + u * kWave + lane, N - 1), E);
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        int i = base + u * kWave + lane;
        if (i < seg_end) {
          keys[i] = (unsigned short)k[u];
          atomicAdd(&h[k[u]], 1);
        }
      }
    }
  }
  __syncthreads();

  for (int b = tid; b < buckets; b += blockDim.x) {
    int s = 0;
    for (int w = 0; w < kRouteWaves; ++w) s += hist[w * buckets + b];
    total[b] = s;
  }
  __syncthreads();
  block_exclusive_scan(total, offs, buckets, scratch);

  // cursors: hist[w][b] <- offs[b] + sum_{w' < w} hist[w'][b]
  for (int b = tid; b < buckets; b += blockDim.x) {
    int run = offs[b];
    for (int w = 0; w < kRouteWaves; ++w) {
      int c = hist[w * buckets + b];
      hist[w * buckets + b] = run;
      run += c;
    }
    if (b < E) {
      counts[b] = total[b];
      offsets_out[b] = offs[b];
    } else {
      offsets_out[E] = offs[E];
    }
  }
  __syncthreads();

  // placement, in input order: position = cursor[key] + number of equal keys in lower lanes of the step
  {
    int *cursor = hist + wave * buckets;
    const int key_bits = bits_for(E + 1);
    const uint64_t lt_mask = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
    for (int base = seg_begin; base < seg_end; base += kWave) {
      const int i = base + lane;
      const bool active = i < seg_end;
      const int k = active ? (int)keys[i] : 0;
      uint64_t peers = match_key(k, active, key_bits);
      int rank = __popcll(peers & lt_mask);
      int start = 0;
      if (active) start = cursor[k];
      __builtin_amdgcn_wave_barrier();
      if (active) {
        int pos = start + rank;
        // a valid id is its own key; the rare invalid one is fetched again for the sorted_expert output
        sorted_expert[pos] = k < E ? k : load_raw<I64>(idx, i);
        sorted_idx[pos] = i;
        bool kept = k < E && (pos - offs[k]) < capacity;
        inv_pos[i] = kept ? pos : -1;
        if (rank == 0) cursor[k] = start + __popcll(peers);
      }
      // the cursor is private to this wave and LDS operations of one wave complete in order: the next step's
      // read sees this step's write without a fence or a volatile access (both would also wait for the global
      // stores above); lanes address the cursor by key, so the compiler cannot carry its values across steps
      __builtin_amdgcn_wave_barrier();
    }
  }
  // the work lists of the GEMM kernels, from the counts and offsets still in LDS (the last wave, after its share
  // of the placement): saves the launch of build_schedule_kernel
  if (sched != nullptr && wave == kRouteWaves - 1) build_schedule_wave(total, offs, N, E, capacity, stream_max_rows, sched, lane);
}

// ---- three-kernel form for large N -----------------------------------------------------------
// seg_counts is [n_seg][buckets] in global memory; one wave per segment of `seg` elements.
template <bool I64>
__global__ __launch_bounds__(kRouteThreads) void route_hist_kernel(const void *idx, int N, int E,
                                                                   int seg, int *seg_counts) {
  extern __shared__ int lds[];
  const int buckets = E + 1;
  const int tid = threadIdx.x, wave = tid / kWave;
  int *hist = lds + wave * buckets;
  for (int i = tid; i < kRouteWaves * buckets; i += blockDim.x) lds[i] = 0;
  __syncthreads();
  int s = blockIdx.x * kRouteWaves + wave;
  int seg_begin = min((long long)s * seg, (long long)N), seg_end = min(seg_begin + seg, N);
  wave_histogram<I64>(idx, seg_begin, seg_end, E, hist);
  __syncthreads();
  for (int i = tid; i < kRouteWaves * buckets; i += blockDim.x)
    seg_counts[(size_t)blockIdx.x * kRouteWaves * buckets + i] = lds[i];
}

// One block: totals, offsets, then per-segment cursors written back over seg_counts.  A wave takes one bucket at a
// time and walks its column of the table 64 segments per step with a wave prefix sum.  Every step is a round trip to
// memory (1.4 us): this is the form for tables too large for LDS (many experts and many assignments at once);
// smaller ones take route_place_scan_kernel.
__global__ __launch_bounds__(kRouteThreads) void route_scan_kernel(int *seg_counts, int n_seg, int E, int *counts,
                                                                   int *offsets_out) {
  extern __shared__ int lds[];
  const int buckets = E + 1;
  int *total = lds;
  int *offs = total + buckets;
  int *scratch = offs + buckets + 1;
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  for (int b = wave; b < buckets; b += kRouteWaves) {
    int s = 0;
    for (int g = lane; g < n_seg; g += kWave) s += seg_counts[(size_t)g * buckets + b];
    for (int d = kWave / 2; d > 0; d >>= 1) s += __shfl_xor(s, d);
    if (lane == 0) total[b] = s;
  }
  __syncthreads();
  block_exclusive_scan(total, offs, buckets, scratch);
  for (int b = wave; b < buckets; b += kRouteWaves) {
    int run = offs[b];
    for (int g0 = 0; g0 < n_seg; g0 += kWave) {
      const int g = g0 + lane;
      const int c = g < n_seg ? seg_counts[(size_t)g * buckets + b] : 0;
      int step_total;
      const int before = wave_exclusive_scan(c, lane, step_total);
      if (g < n_seg) seg_counts[(size_t)g * buckets + b] = run + before;
      run += step_total;
    }
  }
  for (int b = tid; b < buckets; b += blockDim.x) {
    if (b < E) {
      counts[b] = total[b];
      offsets_out[b] = offs[b];
    } else {
      offsets_out[E] = offs[E];
    }
  }
}

// With sched the grid has one workgroup more than there are blocks of segments: its first wave writes the work lists
// of the GEMM kernels from the counts and offsets, next to the placement instead of in a launch of its own.
template <bool I64>
__global__ __launch_bounds__(kRouteThreads) void route_place_kernel(
    const void *idx, int N, int E, int capacity, int seg, const int *seg_cursors,
    const int *offsets_in, int *sorted_expert, int *sorted_idx, int *inv_pos, int n_blocks, const int *counts,
    int stream_max_rows, int *sched) {
  extern __shared__ int lds[];
  const int buckets = E + 1;
  const int tid = threadIdx.x, wave = tid / kWave;
  if ((int)blockIdx.x >= n_blocks) {  // (uniform for the workgroup: nobody of it reaches the barrier below)
    if (sched != nullptr && wave == 0)
      build_schedule_wave(counts, offsets_in, N, E, capacity, stream_max_rows, sched, tid);
    return;
  }
  int *cursor = lds + wave * buckets;
  int *offs = lds + kRouteWaves * buckets;
  for (int i = tid; i < kRouteWaves * buckets; i += blockDim.x)
    lds[i] = seg_cursors[(size_t)blockIdx.x * kRouteWaves * buckets + i];
  for (int b = tid; b <= E; b += blockDim.x) offs[b] = offsets_in[b];
  __syncthreads();
  int s = blockIdx.x * kRouteWaves + wave;
  int seg_begin = min((long long)s * seg, (long long)N), seg_end = min(seg_begin + seg, N);
  wave_place<I64>(idx, seg_begin, seg_end, E, capacity, cursor, offs, sorted_expert, sorted_idx,
                  inv_pos);
}

// ---- two-kernel form: every workgroup of the placement scans the table for itself -----------------------------
// The segments x buckets table of route_hist_kernel is small (65 536 keys in segments of 512 and 128 experts: 66 KB),
// so instead of one workgroup scanning it in a launch of its own, every workgroup of the placement reads all of it
// into LDS and derives what it needs: the bucket totals and offsets, and the cursors of its own 16 segments (a wave
// per bucket column, wave prefix sums over the segments).  Workgroup 0 also writes counts and offsets; with sched
// one workgroup more than there are blocks of segments writes the work lists.
__host__ __device__ inline size_t route_place_scan_lds_ints(int n_seg, int buckets) {
  return (size_t)buckets + (buckets + 1) + (kRouteWaves + 1) + (size_t)kRouteWaves * buckets + (size_t)n_seg * buckets;
}
constexpr size_t kPlaceScanMaxLdsInts = 40000;  // 160 000 bytes

template <bool I64>
__global__ __launch_bounds__(kRouteThreads) void route_place_scan_kernel(
    const void *idx, int N, int E, int capacity, int seg, const int *seg_counts, int n_seg, int *sorted_expert,
    int *sorted_idx, int *inv_pos, int *counts, int *offsets_out, int n_blocks, int stream_max_rows, int *sched) {
  extern __shared__ int lds[];
  const int buckets = E + 1;
  int *total = lds;                              // [buckets]
  int *offs = total + buckets;                   // [buckets + 1]
  int *scratch = offs + buckets + 1;             // [kRouteWaves + 1]
  int *cursors = scratch + kRouteWaves + 1;      // [kRouteWaves][buckets]
  int *table = cursors + kRouteWaves * buckets;  // [n_seg][buckets]
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  const int cells = n_seg * buckets;
  for (int i = tid; i < cells; i += blockDim.x) table[i] = seg_counts[i];
  __syncthreads();
  const int my_first = blockIdx.x * kRouteWaves;  // this workgroup's segments: my_first + 0..15 (none for the extra one)
  for (int b = wave; b < buckets; b += kRouteWaves) {
    int run = 0;
    for (int g0 = 0; g0 < n_seg; g0 += kWave) {
      const int g = g0 + lane;
      const int c = g < n_seg ? table[g * buckets + b] : 0;
      int step_total;
      const int before = wave_exclusive_scan(c, lane, step_total);
      if (g < n_seg && g >= my_first && g < my_first + kRouteWaves) cursors[(g - my_first) * buckets + b] = run + before;
      run += step_total;
    }
    if (lane == 0) total[b] = run;
  }
  __syncthreads();
  block_exclusive_scan(total, offs, buckets, scratch);
  if (blockIdx.x == 0) {
    for (int b = tid; b < buckets; b += blockDim.x) {
      if (b < E) {
        counts[b] = total[b];
        offsets_out[b] = offs[b];
      } else {
        offsets_out[E] = offs[E];
      }
    }
  }
  if ((int)blockIdx.x >= n_blocks) {  // (uniform for the workgroup: nobody of it reaches the barrier below)
    if (sched != nullptr && wave == 0) build_schedule_wave(total, offs, N, E, capacity, stream_max_rows, sched, lane);
    return;
  }
  for (int i = tid; i < kRouteWaves * buckets; i += blockDim.x) cursors[i] += offs[i % buckets];
  __syncthreads();
  const int sgm = my_first + wave;
  const int seg_begin = (int)min((long long)sgm * seg, (long long)N), seg_end = min(seg_begin + seg, N);
  wave_place<I64>(idx, seg_begin, seg_end, E, capacity, cursors + wave * buckets, offs, sorted_expert, sorted_idx, inv_pos);
}

}  // namespace yamoe

using namespace yamoe;

// Keys per wave in the forms with more than one launch: short segments spread the counting and the placement over
// more workgroups, long ones keep the segments x buckets table small.  65 536 keys, 128 experts, three launches:
// 46 / 40 / 48 us with segments of 1024 / 512 / 256 keys (85 us with 2048 and the work lists in a launch of their own),
// two launches with 512: 33 us.  16 384 keys, 32 experts, two launches: 20.5 / 16.3 / 18 us with 512 / 256 / 128 against
// 26 us for the single-workgroup kernel.
static int route_segment(int N) { return N <= 32768 ? 256 : N <= 131072 ? 512 : 2048; }
static_assert(kSingleBlockN <= kSingleBlockMaxN, "the single-workgroup kernel keeps its keys in LDS");

extern "C" size_t yamoe_route_workspace_bytes(int32_t N, int32_t E) {
  if (N <= kSingleBlockN) return 256;
  int seg = route_segment(N);
  int n_seg = ceil_div(ceil_div(N, seg), kRouteWaves) * kRouteWaves;
  return align_up((size_t)n_seg * (E + 1) * sizeof(int), 256);
}

// yamoe_route, optionally with the work lists of yamoe_build_schedule (schedule != nullptr): one launch for N up to
// kSingleBlockN, two above (histograms, then scan + placement), three where the histogram table does not fit LDS;
// with more than one launch the lists come from an extra workgroup of the placement kernel.
int yamoe::route_and_schedule(const void *router_indices, int32_t idx_i64, int32_t N, int32_t E, int32_t capacity,
                              int32_t *sorted_expert, int32_t *sorted_idx, int32_t *counts, int32_t *offsets,
                              int32_t *inv_pos, void *workspace, size_t workspace_bytes, int32_t stream_max_rows,
                              void *schedule, size_t schedule_bytes, void *stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (schedule != nullptr && schedule_bytes < yamoe_schedule_bytes(N, E)) {
    set_error("yamoe_build_schedule: schedule region too small");
    return YAMOE_E_WORKSPACE;
  }
  if (stream_max_rows == kStreamEverything && !sched_may_stream_everything(N, E)) stream_max_rows = kStreamMaxRows;
  if (stream_max_rows < 0 && stream_max_rows != kStreamEverything) stream_max_rows = 0;
  if (stream_max_rows > kStreamMaxRows) stream_max_rows = kStreamMaxRows;
  if (N < 0 || E <= 0 || E + 1 > kRouteMaxBuckets) {
    set_error("yamoe_route: need N >= 0 and 1 <= E < %d (got N=%d E=%d)", kRouteMaxBuckets, N, E);
    return YAMOE_E_ARG;
  }
  if (!counts || !offsets || (N > 0 && (!router_indices || !sorted_expert || !sorted_idx || !inv_pos))) {
    set_error("yamoe_route: null pointer");
    return YAMOE_E_ARG;
  }
  if (capacity < 0) capacity = 0;
  const int buckets = E + 1;
  if (N <= kSingleBlockN) {
    size_t lds = route_single_lds_bytes(N, buckets);
    static DeviceFlags attr_i64, attr_i32;
    const int max_lds = (int)route_single_lds_bytes(kSingleBlockMaxN, kRouteMaxBuckets);
    int rc = idx_i64 ? ensure_dynamic_lds((const void *)route_single_kernel<true>, max_lds, attr_i64, "route_single_kernel")
                     : ensure_dynamic_lds((const void *)route_single_kernel<false>, max_lds, attr_i32, "route_single_kernel");
    if (rc != 0) return rc;
    if (idx_i64)
      hipLaunchKernelGGL(route_single_kernel<true>, dim3(1), dim3(kRouteThreads), lds, stream,
                         router_indices, N, E, capacity, sorted_expert, sorted_idx, counts, offsets, inv_pos, (int *)schedule,
                         stream_max_rows);
    else
      hipLaunchKernelGGL(route_single_kernel<false>, dim3(1), dim3(kRouteThreads), lds, stream,
                         router_indices, N, E, capacity, sorted_expert, sorted_idx, counts, offsets, inv_pos, (int *)schedule,
                         stream_max_rows);
    return check_launch("route_single_kernel");
  }
  if (workspace_bytes < yamoe_route_workspace_bytes(N, E) || !workspace) {
    set_error("yamoe_route: workspace too small (%zu < %zu)", workspace_bytes, yamoe_route_workspace_bytes(N, E));
    return YAMOE_E_WORKSPACE;
  }
  const int seg = route_segment(N);
  const int n_blocks = ceil_div(ceil_div(N, seg), kRouteWaves);
  const int n_seg = n_blocks * kRouteWaves;
  int *seg_counts = (int *)workspace;
  size_t lds_a = (size_t)kRouteWaves * buckets * sizeof(int);
  size_t lds_b = ((size_t)buckets * 2 + 1 + kRouteWaves + 1) * sizeof(int);
  size_t lds_c = ((size_t)kRouteWaves * buckets + buckets) * sizeof(int);
  if (idx_i64)
    hipLaunchKernelGGL(route_hist_kernel<true>, dim3(n_blocks), dim3(kRouteThreads), lds_a, stream,
                       router_indices, N, E, seg, seg_counts);
  else
    hipLaunchKernelGGL(route_hist_kernel<false>, dim3(n_blocks), dim3(kRouteThreads), lds_a, stream,
                       router_indices, N, E, seg, seg_counts);
  int rc = check_launch("route_hist_kernel");
  if (rc) return rc;
  if (route_place_scan_lds_ints(n_seg, buckets) <= kPlaceScanMaxLdsInts) {
    // two launches: the placement's workgroups scan the table themselves
    static DeviceFlags attr_ps64, attr_ps32;
    const int max_lds = (int)(kPlaceScanMaxLdsInts * sizeof(int));
    rc = idx_i64 ? ensure_dynamic_lds((const void *)route_place_scan_kernel<true>, max_lds, attr_ps64, "route_place_scan_kernel")
                 : ensure_dynamic_lds((const void *)route_place_scan_kernel<false>, max_lds, attr_ps32, "route_place_scan_kernel");
    if (rc) return rc;
    const size_t lds_ps = route_place_scan_lds_ints(n_seg, buckets) * sizeof(int);
    const dim3 grid(n_blocks + (schedule != nullptr ? 1 : 0));
    if (idx_i64)
      hipLaunchKernelGGL(route_place_scan_kernel<true>, grid, dim3(kRouteThreads), lds_ps, stream, router_indices, N, E,
                         capacity, seg, seg_counts, n_seg, sorted_expert, sorted_idx, inv_pos, counts, offsets, n_blocks,
                         stream_max_rows, (int *)schedule);
    else
      hipLaunchKernelGGL(route_place_scan_kernel<false>, grid, dim3(kRouteThreads), lds_ps, stream, router_indices, N, E,
                         capacity, seg, seg_counts, n_seg, sorted_expert, sorted_idx, inv_pos, counts, offsets, n_blocks,
                         stream_max_rows, (int *)schedule);
    return check_launch("route_place_scan_kernel");
  }
  hipLaunchKernelGGL(route_scan_kernel, dim3(1), dim3(kRouteThreads), lds_b, stream, seg_counts, n_seg, E, counts, offsets);
  rc = check_launch("route_scan_kernel");
  if (rc) return rc;
  if (idx_i64)
    hipLaunchKernelGGL(route_place_kernel<true>, dim3(n_blocks + (schedule != nullptr ? 1 : 0)), dim3(kRouteThreads), lds_c,
                       stream, router_indices, N, E, capacity, seg, seg_counts, offsets, sorted_expert, sorted_idx, inv_pos,
                       n_blocks, counts, stream_max_rows, (int *)schedule);
  else
    hipLaunchKernelGGL(route_place_kernel<false>, dim3(n_blocks + (schedule != nullptr ? 1 : 0)), dim3(kRouteThreads), lds_c,
                       stream, router_indices, N, E, capacity, seg, seg_counts, offsets, sorted_expert, sorted_idx, inv_pos,
                       n_blocks, counts, stream_max_rows, (int *)schedule);
  return check_launch("route_place_kernel");
}

extern "C" int yamoe_route(const void *router_indices, int32_t idx_i64, int32_t N, int32_t E,
                           int32_t capacity, int32_t *sorted_expert, int32_t *sorted_idx,
                           int32_t *counts, int32_t *offsets, int32_t *inv_pos, void *workspace,
                           size_t workspace_bytes, void *stream_) {
  return route_and_schedule(router_indices, idx_i64, N, E, capacity, sorted_expert, sorted_idx, counts, offsets, inv_pos,
                            workspace, workspace_bytes, 0, nullptr, 0, stream_);
}

extern "C" size_t yamoe_schedule_bytes(int32_t N, int32_t E) {
  size_t words = kSchedHeader + 8 * (size_t)sched_max_row_tiles(N, E) + 4 * (size_t)sched_max_small(N, E);
  return align_up(words * sizeof(int), 256);
}

extern "C" int yamoe_build_schedule(const int32_t *counts, const int32_t *offsets, int32_t N, int32_t E,
                                    int32_t capacity, int32_t stream_max_rows, void *schedule,
                                    size_t schedule_bytes, void *stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (!counts || !offsets || !schedule || N < 0 || E <= 0) {
    set_error("yamoe_build_schedule: bad argument");
    return YAMOE_E_ARG;
  }
  if (schedule_bytes < yamoe_schedule_bytes(N, E)) {
    set_error("yamoe_build_schedule: schedule region too small");
    return YAMOE_E_WORKSPACE;
  }
  if (capacity < 0) capacity = 0;
  if (stream_max_rows == kStreamEverything && !sched_may_stream_everything(N, E)) stream_max_rows = kStreamMaxRows;
  if (stream_max_rows < 0 && stream_max_rows != kStreamEverything) stream_max_rows = 0;
  if (stream_max_rows > kStreamMaxRows) stream_max_rows = kStreamMaxRows;
  hipLaunchKernelGGL(build_schedule_kernel, dim3(1), dim3(kWave), 0, stream, counts, offsets, N, E, capacity,
                     stream_max_rows, (int *)schedule);
  return check_launch("build_schedule_kernel");
}
