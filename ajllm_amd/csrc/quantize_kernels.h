// Weight quantize/pack kernels: fp32 [N, K] -> canonical W8 / W4-g128 tensors.
// Every operation that decides an integer is IEEE binary32, round-to-nearest-even,
// so the outputs are bit-identical to the CPU statement of the scheme.
#pragma once
#include "ajq_common.h"

namespace ajq {

// ---------------------------------------------------------------- W8 ------
// One workgroup per output row: absmax over the row, fp16 scale, then
// q = clamp(rint(w / float(scale)), -127, 127).  The row is read twice; the
// second read hits cache (a row is at most a few tens of KiB).
__global__ __launch_bounds__(256) void quantize_w8_kernel(const float* __restrict__ W, int K,
                                                          int8_t* __restrict__ q,
                                                          uint16_t* __restrict__ scales) {
  const int n = blockIdx.x;
  const float4* row = reinterpret_cast<const float4*>(W + (size_t)n * K);
  const int k4 = K >> 2;
  float amax = 0.0f;
  for (int i = threadIdx.x; i < k4; i += 256) {
    float4 v = row[i];
    amax = fmaxf(amax, fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
  }
  for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off));
  __shared__ float wave_max[4];
  if ((threadIdx.x & 63) == 0) wave_max[threadIdx.x >> 6] = amax;
  __syncthreads();
  amax = fmaxf(fmaxf(wave_max[0], wave_max[1]), fmaxf(wave_max[2], wave_max[3]));

  const __half hs = __float2half_rn(amax / 127.0f);
  if (threadIdx.x == 0) scales[n] = __half_as_ushort(hs);
  float d = __half2float(hs);
  if (d == 0.0f) d = 1.0f;

  uint32_t* qrow = reinterpret_cast<uint32_t*>(q + (size_t)n * K);
  for (int i = threadIdx.x; i < k4; i += 256) {
    float4 v = row[i];
    int a = (int)fminf(fmaxf(rintf(v.x / d), -127.0f), 127.0f);
    int b = (int)fminf(fmaxf(rintf(v.y / d), -127.0f), 127.0f);
    int c = (int)fminf(fmaxf(rintf(v.z / d), -127.0f), 127.0f);
    int e = (int)fminf(fmaxf(rintf(v.w / d), -127.0f), 127.0f);
    qrow[i] = (uint32_t)(a & 0xFF) | ((uint32_t)(b & 0xFF) << 8) | ((uint32_t)(c & 0xFF) << 16) |
              ((uint32_t)(e & 0xFF) << 24);
  }
}

// ---------------------------------------------------------------- W4 ------
// 16 lanes own one 128-wide group (8 consecutive weights per lane, one packed
// word out); a 256-thread workgroup covers 16 consecutive groups of the
// flattened [N*K/128] group list.
__global__ __launch_bounds__(256) void quantize_w4_kernel(const float* __restrict__ W,
                                                          long long n_groups,
                                                          int32_t* __restrict__ qweight,
                                                          uint16_t* __restrict__ scales,
                                                          uint8_t* __restrict__ zeros) {
  const long long g = (long long)blockIdx.x * 16 + (threadIdx.x >> 4);
  if (g >= n_groups) return;  // whole 16-lane team leaves together
  const int sub = threadIdx.x & 15;
  const float4* src = reinterpret_cast<const float4*>(W + g * kGroup + sub * 8);
  const float4 v0 = src[0], v1 = src[1];
  float w[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
  float mn = w[0], mx = w[0];
#pragma unroll
  for (int i = 1; i < 8; ++i) {
    mn = fminf(mn, w[i]);
    mx = fmaxf(mx, w[i]);
  }
#pragma unroll
  for (int off = 8; off > 0; off >>= 1) {
    mn = fminf(mn, __shfl_xor(mn, off));
    mx = fmaxf(mx, __shfl_xor(mx, off));
  }
  const __half hs = __float2half_rn((mx - mn) / 15.0f);
  float d = __half2float(hs);
  if (d == 0.0f) d = 1.0f;
  const float zf = fminf(fmaxf(rintf(-mn / d), 0.0f), 15.0f);
  uint32_t word = 0;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    float qf = fminf(fmaxf(rintf(w[i] / d) + zf, 0.0f), 15.0f);
    word |= (uint32_t)(int)qf << (4 * i);
  }
  qweight[g * 16 + sub] = (int32_t)word;
  if (sub == 0) {
    scales[g] = __half_as_ushort(hs);
    zeros[g] = (uint8_t)(int)zf;
  }
}

// ------------------------------------------------------------ repack ------
// canonical W4 -> private tiles.  One thread per private dword.
__global__ __launch_bounds__(256) void repack_w4_kernel(const uint32_t* __restrict__ qweight, int N,
                                                        int K, uint32_t* __restrict__ wq) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  const long long total = (long long)N * (K / 8);
  if (idx >= total) return;
  const int G = K / kGroup;
  const int j = idx & 3;
  const int lane = (idx >> 2) & 63;
  const long long tile = idx >> 8;
  const int g = (int)(tile % G);
  const int nt = (int)(tile / G);
  const int nl = lane & 15, kc = lane >> 4;
  const int n = nt * kTileN + nl;
  const int k = g * kGroup + 32 * j + 8 * kc;
  const uint32_t w = qweight[(size_t)n * (K / 8) + (k >> 3)];
  uint32_t out = 0;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const uint32_t v = (w >> (4 * e)) & 0xFu;
    out |= v << (4 * ((e >> 1) + 4 * (e & 1)));
  }
  wq[idx] = out;
}

__global__ __launch_bounds__(256) void repack_w4_meta_kernel(const uint16_t* __restrict__ scales,
                                                             const uint8_t* __restrict__ zeros, int N,
                                                             int G, uint32_t* __restrict__ meta) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (long long)N * G) return;
  const int nl = idx & 15;
  const long long tile = idx >> 4;
  const int g = (int)(tile % G);
  const int nt = (int)(tile / G);
  const size_t src = (size_t)(nt * kTileN + nl) * G + g;
  const __half zc = __float2half_rn(128.0f + (float)zeros[src]);  // <= 143: exact
  meta[idx] = (uint32_t)scales[src] | ((uint32_t)__half_as_ushort(zc) << 16);
}

__global__ __launch_bounds__(256) void unrepack_w4_kernel(const uint32_t* __restrict__ wq, int N, int K,
                                                          uint32_t* __restrict__ qweight) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  const long long total = (long long)N * (K / 8);
  if (idx >= total) return;
  const int G = K / kGroup;
  const int j = idx & 3;
  const int lane = (idx >> 2) & 63;
  const long long tile = idx >> 8;
  const int g = (int)(tile % G);
  const int nt = (int)(tile / G);
  const int nl = lane & 15, kc = lane >> 4;
  const int n = nt * kTileN + nl;
  const int k = g * kGroup + 32 * j + 8 * kc;
  const uint32_t w = wq[idx];
  uint32_t out = 0;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const uint32_t v = (w >> (4 * ((e >> 1) + 4 * (e & 1)))) & 0xFu;
    out |= v << (4 * e);
  }
  qweight[(size_t)n * (K / 8) + (k >> 3)] = out;
}

__global__ __launch_bounds__(256) void unrepack_w4_meta_kernel(const uint32_t* __restrict__ meta, int N,
                                                               int G, uint16_t* __restrict__ scales,
                                                               uint8_t* __restrict__ zeros) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (long long)N * G) return;
  const int nl = idx & 15;
  const long long tile = idx >> 4;
  const int g = (int)(tile % G);
  const int nt = (int)(tile / G);
  const size_t dst = (size_t)(nt * kTileN + nl) * G + g;
  const uint32_t m = meta[idx];
  scales[dst] = (uint16_t)(m & 0xFFFFu);
  zeros[dst] = (uint8_t)(int)(f16_bits_to_f32(m >> 16) - 128.0f);
}

// canonical W8 [N, K] int8 -> private tiles.  One thread per private dword.
// dword (tile (nt, t), lane (kc, nl), d) holds k = 64t + 32*(d>>1) + 8kc + 4*(d&1) .. +4
template <bool kInverse>
__global__ __launch_bounds__(256) void repack_w8_kernel(const uint32_t* __restrict__ src, int N, int K,
                                                        uint32_t* __restrict__ dst) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  const long long total = (long long)N * (K / 4);
  if (idx >= total) return;
  const int T = K / kW8TileK;
  const int d = idx & 3;
  const int lane = (idx >> 2) & 63;
  const long long tile = idx >> 8;
  const int t = (int)(tile % T);
  const int nt = (int)(tile / T);
  const int nl = lane & 15, kc = lane >> 4;
  const int n = nt * kTileN + nl;
  const int k = t * kW8TileK + 32 * (d >> 1) + 8 * kc + 4 * (d & 1);
  const size_t canon = (size_t)n * (K / 4) + (k >> 2);
  if (kInverse)
    dst[canon] = src[idx];
  else
    dst[idx] = src[canon];
}

}  // namespace ajq
