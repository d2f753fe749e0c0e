// Decode dequant-GEMV, 1 <= M <= 16:  y[M, N] = x[M, K] @ W_hat[N, K]^T.
//
// HBM-bound and short (a 4096 x 4096 int4 matrix is 8.7 MB, about a microsecond
// of HBM time), so the kernel is built to have every byte in flight as early as
// possible and to do its arithmetic while the bytes arrive:
//  * one workgroup owns one 16-row tile of N and all of K; wave w owns a
//    contiguous run of 128-wide k groups, i.e. a contiguous run of 1 KiB private
//    weight tiles, and loads each with one 128-bit load per lane (a wave-wide
//    load instruction reads one contiguous KiB), non-temporal, issued up front;
//  * weights go global -> registers -> in-register unpack (3 shifts + 4
//    v_and_or_b32 per 8 nibbles) -> MFMA B operand; they never touch LDS;
//  * each wave stages only ITS k-slice of the activations in a wave-private LDS
//    region (rows padded by 16 B: the 16 rows of an A fragment fall in distinct
//    banks) and reads it back as MFMA A fragments, so there is no workgroup
//    barrier before the arithmetic; rows >= M of the A operand repeat row M-1 and
//    their outputs are never stored;
//  * group sums of the activations (needed for the zero-point term) come from a
//    second MFMA against an all-ones B operand, which lands them in exactly the
//    accumulator layout that needs them;
//  * the waves' partial sums meet once, through LDS, in a fixed order: no
//    atomics, results are run-to-run identical.
#pragma once
#include "ajq_common.h"

namespace ajq {

__device__ __forceinline__ uint32_t and_or_b32(uint32_t a, uint32_t mask_sgpr, uint32_t magic_vgpr) {
  uint32_t r;
  // VOP3 on gfx9 takes no literal: the mask rides in an SGPR, the magic in a VGPR
  asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "s"(mask_sgpr), "v"(magic_vgpr));
  return r;
}

// private W4 dword -> 8 bf16 holding 128+q (see w4_to_bf16_biased), 7 VALU ops
__device__ __forceinline__ u32x4_t w4_unpack(uint32_t w, uint32_t mask, uint32_t magic) {
  u32x4_t r;
  r.x = and_or_b32(w, mask, magic);
  r.y = and_or_b32(w >> 4, mask, magic);
  r.z = and_or_b32(w >> 8, mask, magic);
  r.w = and_or_b32(w >> 12, mask, magic);
  return r;
}

// One batch of a wave: TPW consecutive k groups, their weights, meta words and the
// matching slice of the activations, all in registers.
template <int TPW, int kXLoads, int kLoadsPerGroup>
struct GemvBatch {
  u32x4_t x[kXLoads];
  u32x4_t w[TPW][kLoadsPerGroup];
  uint32_t m[TPW];
};

// kWaves waves per workgroup; a wave works through its k groups TPW at a time;
// MROWS >= M is the compile-time row bound that sizes the activation slice.
template <int kWaves, int TPW, int MROWS, bool kW4>
__global__ __launch_bounds__(kWaves * 64) void dequant_gemv_kernel(
    const uint16_t* __restrict__ x, int M, int K, const u32x4_t* __restrict__ wq,
    const uint32_t* __restrict__ meta,     // W4: private meta; W8: unused
    const uint16_t* __restrict__ scales8,  // W8: fp16 [N]; W4: unused
    int N, void* __restrict__ y, int out_f32) {
  constexpr int kSlice = TPW * kGroup;     // k extent of one batch of one wave
  constexpr int kStride = kSlice + 8;      // padded LDS row, bf16 elements
  constexpr int kVecPerRow = kSlice / 8;   // 16-byte vectors per slice row
  constexpr int kVecs = MROWS * kVecPerRow;
  constexpr int kXLoads = (kVecs + 63) / 64;
  constexpr int kLoadsPerGroup = kW4 ? 1 : 2;  // 1 KiB tiles per 128 k
  using Batch = GemvBatch<TPW, kXLoads, kLoadsPerGroup>;

  extern __shared__ u32x4_t smem_raw[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // uniform: scalar branches
  const int nl = lane & 15, kc = lane >> 4;
  const int nt = blockIdx.x;
  const int G = K >> 7;
  uint16_t* xs = reinterpret_cast<uint16_t*>(smem_raw) + wave * (MROWS * kStride);
  float* red = reinterpret_cast<float*>(reinterpret_cast<uint16_t*>(smem_raw) + kWaves * (MROWS * kStride));

  const int per_wave = (G + kWaves - 1) / kWaves;
  const int g_begin = wave * per_wave;
  const int g_end = min(G, g_begin + per_wave);

  const u32x4_t* wtile = wq + (size_t)nt * G * kLoadsPerGroup * 64 + lane;
  const uint32_t* mtile = meta + (size_t)nt * G * 16 + nl;

  // Every load below is unconditional (addresses are clamped into the wave's own
  // range instead), so the number of loads in flight is static and the compiler
  // can wait for exactly the tile it is about to use.
  auto load = [&](Batch& b, int g0) {
#pragma unroll
    for (int i = 0; i < kXLoads; ++i) {
      const int v = min(lane + 64 * i, kVecs - 1);
      const int m = min(v / kVecPerRow, M - 1), c = v % kVecPerRow;
      const int k = min(g0 * kGroup + 8 * c, K - 8);
      b.x[i] = *reinterpret_cast<const u32x4_t*>(x + (size_t)m * K + k);
    }
#pragma unroll
    for (int p = 0; p < TPW; ++p) {
      const int g = min(g0 + p, g_end - 1);
#pragma unroll
      for (int h = 0; h < kLoadsPerGroup; ++h)
        b.w[p][h] = __builtin_nontemporal_load(wtile + ((size_t)g * kLoadsPerGroup + h) * 64);
      if (kW4) b.m[p] = mtile[(size_t)g * 16];
    }
  };

  const uint32_t mask = 0x000F000Fu;
  uint32_t magic = 0x43004300u;
  asm volatile("" : "+v"(magic));  // keep it in a VGPR for v_and_or_b32
  const u32x4_t ones = {0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};
  const int row = min(nl, M - 1);
  const uint16_t* xrow = xs + row * kStride + 8 * kc;
  f32x4_t acc = {0.f, 0.f, 0.f, 0.f};

  auto compute = [&](Batch& b, int g0) {
    // slice of this batch -> wave-private LDS.  LDS operations of one wave execute
    // in order, so the reads of the previous batch are already done.
#pragma unroll
    for (int i = 0; i < kXLoads; ++i) {
      const int v = lane + 64 * i;
      if ((i + 1) * 64 <= kVecs || v < kVecs)
        *reinterpret_cast<u32x4_t*>(xs + (v / kVecPerRow) * kStride + 8 * (v % kVecPerRow)) = b.x[i];
    }
#pragma unroll
    for (int p = 0; p < TPW; ++p) {
      if (g0 + p < g_end) {
        if (kW4) {
          f32x4_t part = {0.f, 0.f, 0.f, 0.f}, asum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const u32x4_t a = *reinterpret_cast<const u32x4_t*>(xrow + p * kGroup + 32 * j);
            const u32x4_t bw = w4_unpack(b.w[p][0][j], mask, magic);
            part = mfma16(a, bw, part);
            asum = mfma16(a, ones, asum);
          }
          const float s = f16_bits_to_f32(b.m[p] & 0xFFFFu);
          const float zc = f16_bits_to_f32(b.m[p] >> 16);
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[i] += s * (part[i] - zc * asum[i]);
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const u32x4_t a = *reinterpret_cast<const u32x4_t*>(xrow + p * kGroup + 32 * j);
            const u32x2_t lo = w8_to_bf16(b.w[p][j >> 1][2 * (j & 1)]);
            const u32x2_t hi = w8_to_bf16(b.w[p][j >> 1][2 * (j & 1) + 1]);
            acc = mfma16(a, u32x4_t{lo.x, lo.y, hi.x, hi.y}, acc);
          }
        }
      }
    }
  };

  // two register sets, ping-pong: the next batch is in flight while one is computed
  if (g_begin < g_end) {
    Batch b0, b1;
    load(b0, g_begin);
    for (int g0 = g_begin; g0 < g_end; g0 += 2 * TPW) {
      const bool has1 = g0 + TPW < g_end;
      if (has1) load(b1, g0 + TPW);
      compute(b0, g0);
      if (g0 + 2 * TPW < g_end) load(b0, g0 + 2 * TPW);
      if (has1) compute(b1, g0 + TPW);
    }
  }

  // ---- the waves' partial sums meet in LDS; wave 0 adds them in wave order
  reinterpret_cast<f32x4_t*>(red)[wave * 64 + lane] = acc;
  __syncthreads();
  if (wave != 0) return;
  f32x4_t sum = reinterpret_cast<f32x4_t*>(red)[lane];
#pragma unroll
  for (int w = 1; w < kWaves; ++w) sum += reinterpret_cast<f32x4_t*>(red)[w * 64 + lane];
  const int n = nt * kTileN + nl;
  float cs = 1.0f;
  if (!kW4) cs = f16_bits_to_f32(scales8[n]);  // per-output-channel scale, once
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = 4 * kc + i;
    if (m < M) {
      const float v = sum[i] * cs;
      if (out_f32)
        reinterpret_cast<float*>(y)[(size_t)m * N + n] = v;
      else
        reinterpret_cast<uint16_t*>(y)[(size_t)m * N + n] = f32_to_bf16_rne(v);
    }
  }
}

// LDS bytes of one workgroup of dequant_gemv_kernel<kWaves, TPW, MROWS, *>
constexpr size_t gemv_lds_bytes(int waves, int tpw, int mrows) {
  return (size_t)waves * mrows * (tpw * kGroup + 8) * 2 + (size_t)waves * 64 * 16;
}

}  // namespace ajq
