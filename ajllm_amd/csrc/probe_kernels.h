// Device yardstick: the bf16 MFMA rate this GPU sustains with nothing else going on.
//
// Every wave issues v_mfma_f32_32x32x16_bf16 back to back on four independent accumulators,
// operands in registers, no memory traffic.  With constant operands the matrix pipes run at
// the nominal clock; with random mantissas the multipliers toggle, the chip reaches its power
// limit and the clock drops: that second figure is what a GEMM on real data can approach.
#pragma once
#include "ajq_common.h"

namespace ajq {

constexpr int kProbeThreads = 512;  // two waves per SIMD
constexpr int kProbeChains = 4;

__device__ __forceinline__ uint32_t probe_hash(uint32_t x) {
  x ^= x >> 16;
  x *= 0x7feb352du;
  x ^= x >> 15;
  x *= 0x846ca68bu;
  x ^= x >> 16;
  return x;
}

// sink[blockIdx.x * 512 + threadIdx.x] receives a value that depends on every accumulator;
// clocks[0] = shader cycles, clocks[1] = ticks of the constant 100 MHz counter, both over the
// MFMA loop of workgroup 0, wave 0.
__global__ __launch_bounds__(kProbeThreads) void mfma_rate_kernel(int random_operands, int iters,
                                                                 float* __restrict__ sink,
                                                                 long long* __restrict__ clocks) {
  bf16x8_t a[kProbeChains], b[kProbeChains];
#pragma unroll
  for (int c = 0; c < kProbeChains; ++c)
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      // |value| in [0.5, 2): no overflow however long the loop runs is not needed, the sums may
      // saturate to inf without changing the rate; sign and mantissa bits are random
      const uint32_t h = random_operands ? probe_hash(threadIdx.x * 977u + c * 131u + i * 7u + blockIdx.x * 7919u) : 0u;
      a[c][i] = __builtin_bit_cast(__bf16, (uint16_t)(0x3F00u | (h & 0x80FFu)));
      b[c][i] = __builtin_bit_cast(__bf16, (uint16_t)(0x3F00u | ((h >> 16) & 0x80FFu)));
    }
  f32x16_t acc[kProbeChains];
#pragma unroll
  for (int c = 0; c < kProbeChains; ++c)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[c][r] = 0.f;
  const long long c0 = clock64();
  const long long w0 = wall_clock64();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int c = 0; c < kProbeChains; ++c) acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[c], b[c], acc[c], 0, 0, 0);
  }
  const long long c1 = clock64();
  const long long w1 = wall_clock64();
  float s = 0.f;
#pragma unroll
  for (int c = 0; c < kProbeChains; ++c)
#pragma unroll
    for (int r = 0; r < 16; ++r) s += acc[c][r];
  sink[(size_t)blockIdx.x * kProbeThreads + threadIdx.x] = s;
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    clocks[0] = c1 - c0;
    clocks[1] = w1 - w0;
  }
}

}  // namespace ajq
