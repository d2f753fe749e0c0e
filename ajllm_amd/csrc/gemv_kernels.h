// Decode dequant-GEMV, 1 <= M <= 16:  y[M, N] = x[M, K] @ W_hat[N, K]^T.
//
// HBM-bound.  One workgroup owns one 16-row tile of N and all of K; its waves
// take the 1 KiB weight tiles of that row block round-robin, so a wave's load
// instruction reads one contiguous KiB (64 lanes x 16 B) and the workgroup as a
// whole streams one contiguous region.  Weights go global -> registers ->
// in-register unpack to bf16 -> MFMA B operand; they never touch LDS.  The
// activations are staged once per workgroup in LDS (row-major, rows padded by
// 16 B so the 16 rows of an A fragment fall in distinct banks) and are the
// MFMA A operand with rows >= M zero.  Partial sums of the waves are combined
// through LDS in a fixed order (no atomics: results are run-to-run identical).
#pragma once
#include "ajq_common.h"

namespace ajq {

constexpr int kPrefetch = 4;  // weight tiles a wave keeps in flight per batch

struct GemvSmem {
  // x chunk: M rows x (kchunk + 8) bf16, then the cross-wave reduction area
  __device__ static uint16_t* x(void* base) { return reinterpret_cast<uint16_t*>(base); }
};

template <int kWaves>
__device__ __forceinline__ void stage_x_chunk(const uint16_t* __restrict__ x, int M, int K, int c0,
                                              int clen, uint16_t* xs, int stride) {
  const int vec_per_row = clen >> 3;
  const int total = M * vec_per_row;
  for (int v = threadIdx.x; v < total; v += kWaves * 64) {
    const int m = v / vec_per_row;
    const int c = v - m * vec_per_row;
    const u32x4_t val = *reinterpret_cast<const u32x4_t*>(x + (size_t)m * K + c0 + 8 * c);
    *reinterpret_cast<u32x4_t*>(xs + m * stride + 8 * c) = val;
  }
}

template <int kWaves>
__device__ __forceinline__ void reduce_and_store(f32x4_t acc, float* red, int M, int N, int nt, void* y,
                                                 int out_f32, const float* chan_scale) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  reinterpret_cast<f32x4_t*>(red)[wave * 64 + lane] = acc;
  __syncthreads();
  if (wave != 0) return;
  f32x4_t sum = reinterpret_cast<f32x4_t*>(red)[lane];
#pragma unroll
  for (int w = 1; w < kWaves; ++w) sum += reinterpret_cast<f32x4_t*>(red)[w * 64 + lane];
  const int nl = lane & 15, kc = lane >> 4;
  const int n = nt * kTileN + nl;
  const float cs = chan_scale ? chan_scale[0] : 1.0f;
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

// ------------------------------------------------------------------ W4 ----
template <int kWaves>
__global__ __launch_bounds__(kWaves * 64) void w4a16_gemv_kernel(
    const uint16_t* __restrict__ x, int M, int K, const u32x4_t* __restrict__ wq,
    const uint32_t* __restrict__ meta, int N, void* __restrict__ y, int out_f32, int kchunk) {
  extern __shared__ u32x4_t smem_raw[];
  uint16_t* xs = reinterpret_cast<uint16_t*>(smem_raw);
  const int stride = kchunk + 8;
  float* red = reinterpret_cast<float*>(xs + (size_t)M * stride);

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int nl = lane & 15, kc = lane >> 4;
  const int nt = blockIdx.x;
  const int G = K >> 7;
  const u32x4_t* wtile = wq + (size_t)nt * G * 64 + lane;
  const uint32_t* mtile = meta + (size_t)nt * G * 16 + nl;
  const u32x4_t ones = {0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};
  const u32x4_t zero4 = {0u, 0u, 0u, 0u};
  const bool row_live = nl < M;

  f32x4_t acc = {0.f, 0.f, 0.f, 0.f};

  for (int c0 = 0; c0 < K; c0 += kchunk) {
    const int clen = min(kchunk, K - c0);
    const int g_lo = c0 >> 7, g_hi = (c0 + clen) >> 7;
    // first group of this wave inside the chunk
    int g = g_lo + ((wave - g_lo) % kWaves + kWaves) % kWaves;

    u32x4_t wcur[kPrefetch];
    uint32_t mcur[kPrefetch];
#pragma unroll
    for (int p = 0; p < kPrefetch; ++p) {
      const int gp = g + p * kWaves;
      if (gp < g_hi) {
        wcur[p] = wtile[(size_t)gp * 64];
        mcur[p] = mtile[(size_t)gp * 16];
      }
    }
    __syncthreads();  // everyone is done reading the previous chunk
    stage_x_chunk<kWaves>(x, M, K, c0, clen, xs, stride);
    __syncthreads();

    while (g < g_hi) {
      u32x4_t wnxt[kPrefetch];
      uint32_t mnxt[kPrefetch];
      const int gn = g + kPrefetch * kWaves;
#pragma unroll
      for (int p = 0; p < kPrefetch; ++p) {
        const int gp = gn + p * kWaves;
        if (gp < g_hi) {
          wnxt[p] = wtile[(size_t)gp * 64];
          mnxt[p] = mtile[(size_t)gp * 16];
        }
      }
#pragma unroll
      for (int p = 0; p < kPrefetch; ++p) {
        const int gp = g + p * kWaves;
        if (gp < g_hi) {
          const uint16_t* xrow = xs + nl * stride + (gp * kGroup - c0) + 8 * kc;
          f32x4_t tmp = {0.f, 0.f, 0.f, 0.f}, asum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            u32x4_t a = zero4;
            if (row_live) a = *reinterpret_cast<const u32x4_t*>(xrow + 32 * j);
            const u32x4_t b = w4_to_bf16_biased(wcur[p][j]);
            tmp = mfma16(a, b, tmp);
            asum = mfma16(a, ones, asum);
          }
          const float s = f16_bits_to_f32(mcur[p] & 0xFFFFu);
          const float zc = f16_bits_to_f32(mcur[p] >> 16);
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[i] += s * (tmp[i] - zc * asum[i]);
        }
      }
#pragma unroll
      for (int p = 0; p < kPrefetch; ++p) {
        wcur[p] = wnxt[p];
        mcur[p] = mnxt[p];
      }
      g = gn;
    }
  }
  reduce_and_store<kWaves>(acc, red, M, N, nt, y, out_f32, nullptr);
}

// ------------------------------------------------------------------ W8 ----
template <int kWaves>
__global__ __launch_bounds__(kWaves * 64) void w8a16_gemv_kernel(
    const uint16_t* __restrict__ x, int M, int K, const u32x4_t* __restrict__ wq,
    const uint16_t* __restrict__ scales, int N, void* __restrict__ y, int out_f32, int kchunk) {
  extern __shared__ u32x4_t smem_raw[];
  uint16_t* xs = reinterpret_cast<uint16_t*>(smem_raw);
  const int stride = kchunk + 8;
  float* red = reinterpret_cast<float*>(xs + (size_t)M * stride);

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int nl = lane & 15, kc = lane >> 4;
  const int nt = blockIdx.x;
  const int T = K >> 6;  // 64-wide tiles along K
  const u32x4_t* wtile = wq + (size_t)nt * T * 64 + lane;
  const u32x4_t zero4 = {0u, 0u, 0u, 0u};
  const bool row_live = nl < M;

  f32x4_t acc = {0.f, 0.f, 0.f, 0.f};

  for (int c0 = 0; c0 < K; c0 += kchunk) {
    const int clen = min(kchunk, K - c0);
    const int t_lo = c0 >> 6, t_hi = (c0 + clen) >> 6;
    int t = t_lo + ((wave - t_lo) % kWaves + kWaves) % kWaves;

    u32x4_t wcur[kPrefetch];
#pragma unroll
    for (int p = 0; p < kPrefetch; ++p) {
      const int tp = t + p * kWaves;
      if (tp < t_hi) wcur[p] = wtile[(size_t)tp * 64];
    }
    __syncthreads();
    stage_x_chunk<kWaves>(x, M, K, c0, clen, xs, stride);
    __syncthreads();

    while (t < t_hi) {
      u32x4_t wnxt[kPrefetch];
      const int tn = t + kPrefetch * kWaves;
#pragma unroll
      for (int p = 0; p < kPrefetch; ++p) {
        const int tp = tn + p * kWaves;
        if (tp < t_hi) wnxt[p] = wtile[(size_t)tp * 64];
      }
#pragma unroll
      for (int p = 0; p < kPrefetch; ++p) {
        const int tp = t + p * kWaves;
        if (tp < t_hi) {
          const uint16_t* xrow = xs + nl * stride + (tp * kW8TileK - c0) + 8 * kc;
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            u32x4_t a = zero4;
            if (row_live) a = *reinterpret_cast<const u32x4_t*>(xrow + 32 * j);
            const u32x2_t lo = w8_to_bf16(wcur[p][2 * j]);
            const u32x2_t hi = w8_to_bf16(wcur[p][2 * j + 1]);
            const u32x4_t b = {lo.x, lo.y, hi.x, hi.y};
            acc = mfma16(a, b, acc);
          }
        }
      }
#pragma unroll
      for (int p = 0; p < kPrefetch; ++p) wcur[p] = wnxt[p];
      t = tn;
    }
  }
  // per-output-channel scale, applied once after the cross-wave sum
  __shared__ float chan_scale_s[16];
  if (threadIdx.x < 16) chan_scale_s[threadIdx.x] = f16_bits_to_f32(scales[nt * kTileN + threadIdx.x]);
  // reduce_and_store's barrier orders the write above before its reads
  reduce_and_store<kWaves>(acc, red, M, N, nt, y, out_f32, &chan_scale_s[nl]);
}


}  // namespace ajq
