// Diagnostic kernels: what the part itself delivers, for scale next to the expert GEMMs.  Not on the path of any op.
#include "common.h"

namespace yamoe {

// A register-only loop of v_mfma_f32_32x32x16_bf16: one wave per SIMD, 4 x 4 accumulator blocks (256 accumulator
// registers, the shape of the forward tile kernel's wave), no memory or LDS traffic inside the loop.  With
// `random_operands` the eight operand fragments hold pseudo-random bf16 values of magnitude up to 1 (every lane its
// own), otherwise zeros: the matrix pipes run against the power limit, so the rate depends on how much the operands
// toggle the datapath.
__global__ __launch_bounds__(256) void mfma_rate_kernel(int iters, int random_operands, float *sink) {
  const uint32_t tid = blockIdx.x * blockDim.x + threadIdx.x;
  u32x4 fa[4], fb[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      uint32_t h = (tid * 8u + i * 4u + j) * 2654435761u;
      h ^= h >> 15; h *= 2246822519u; h ^= h >> 13;
      uint32_t g = h * 3266489917u; g ^= g >> 16;
      // two bf16 values per word: sign and mantissa random, exponent 120..127 (magnitude 2^-7 .. 2)
      const uint32_t a = (h & 0x807f807fu) | ((0x78u + (h >> 8 & 7u)) << 7) | ((0x78u + (h >> 24 & 7u)) << 23);
      const uint32_t b = (g & 0x807f807fu) | ((0x78u + (g >> 8 & 7u)) << 7) | ((0x78u + (g >> 24 & 7u)) << 23);
      fa[i][j] = random_operands ? a : 0u;
      fb[i][j] = random_operands ? b : 0u;
    }
  f32x16 acc[4][4];
#pragma unroll
  for (int mi = 0; mi < 4; ++mi)
#pragma unroll
    for (int ni = 0; ni < 4; ++ni)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[mi][ni][v] = 0.0f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int mi = 0; mi < 4; ++mi)
#pragma unroll
      for (int ni = 0; ni < 4; ++ni)
        acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, fb[ni]),
                                                              __builtin_bit_cast(bf16x8, fa[mi]), acc[mi][ni], 0, 0, 0);
    // keep the operands loop-variant without touching their values' statistics: rotate the fragments
    const u32x4 t = fa[0];
    fa[0] = fa[1]; fa[1] = fa[2]; fa[2] = fa[3]; fa[3] = t;
  }
  float s = 0.0f;
#pragma unroll
  for (int mi = 0; mi < 4; ++mi)
#pragma unroll
    for (int ni = 0; ni < 4; ++ni)
#pragma unroll
      for (int v = 0; v < 16; ++v) s += acc[mi][ni][v];
  if (s == 123.456f) sink[0] = s;  // (never true in practice; keeps the loop alive)
}

}  // namespace yamoe

using namespace yamoe;

extern "C" int yamoe_probe_mfma_rate(int32_t workgroups, int32_t iters, int32_t random_operands, float *sink,
                                     double *flop, void *stream) {
  if (workgroups <= 0 || iters <= 0 || !sink) { set_error("yamoe_probe_mfma_rate: bad argument"); return YAMOE_E_ARG; }
  hipLaunchKernelGGL(mfma_rate_kernel, dim3(workgroups), dim3(256), 0, (hipStream_t)stream, iters, random_operands, sink);
  if (flop) *flop = (double)workgroups * 4.0 * iters * 16.0 * (2.0 * 32 * 32 * 16);
  return check_launch("mfma_rate_kernel");
}
