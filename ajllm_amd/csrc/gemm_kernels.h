// Prefill dequant-GEMM:  y[M, N] = x[M, K] @ W_hat[N, K]^T on bf16 MFMA.
//
// A workgroup owns a BM x BN output tile and walks K in blocks of 128 (one
// int4 quantization group).  Activations: global -> registers -> LDS (row-major,
// rows padded by 16 B), read back as MFMA A fragments.  Weights: each wave loads
// the 1 KiB private tiles of its own columns straight into registers (one
// 128-bit load per lane and tile), unpacks them in registers to bf16 values that
// are EXACT small integers (128+q for int4, q for int8) and feeds them as the
// MFMA B operand; scales stay in fp32 and are applied to fp32 partial sums
// (per group for W4, once per channel for W8), so no weight is ever rounded.
//   W4:  y[m,n] = sum_g s[n,g] * ( sum_{k in g} a[m,k]*(128+q[n,k]) - (128+z[n,g]) * A[m,g] )
// with A[m,g] = sum_{k in g} a[m,k] precomputed by group_sum_kernel.
#pragma once
#include "ajq_common.h"

namespace ajq {

// A[g][m] = sum over the 128 activations of group g in row m (fp32).
// One 16-lane team per (m, g); layout [G][Mpad] so 4 consecutive rows are one float4.
__global__ __launch_bounds__(256) void group_sum_kernel(const uint16_t* __restrict__ x, int M, int K,
                                                        int Mpad, float* __restrict__ gsum) {
  const int G = K >> 7;
  const long long team = (long long)blockIdx.x * 16 + (threadIdx.x >> 4);
  if (team >= (long long)M * G) return;
  const int sub = threadIdx.x & 15;
  const int m = (int)(team / G), g = (int)(team % G);
  const u32x4_t v = *reinterpret_cast<const u32x4_t*>(x + (size_t)m * K + g * kGroup + sub * 8);
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    s += __uint_as_float(v[i] << 16);
    s += __uint_as_float(v[i] & 0xFFFF0000u);
  }
#pragma unroll
  for (int off = 8; off > 0; off >>= 1) s += __shfl_xor(s, off);
  if (sub == 0) gsum[(size_t)g * Mpad + m] = s;
}

constexpr int kBK = 128;
constexpr int kLdsRow = kBK + 8;  // bf16 elements per LDS row (16 B pad)

template <int BM, int BN, int WM, int WN, bool kW4>
__global__ __launch_bounds__((BM / WM) * (BN / WN) * 64) void dequant_gemm_kernel(
    const uint16_t* __restrict__ x, int M, int K, const u32x4_t* __restrict__ wq,
    const uint32_t* __restrict__ meta,     // W4: private meta; W8: unused
    const uint16_t* __restrict__ scales8,  // W8: fp16 [N]; W4: unused
    const float* __restrict__ gsum, int Mpad, int N, void* __restrict__ y, int out_f32) {
  constexpr int kWavesM = BM / WM, kWavesN = BN / WN;
  constexpr int kThreads = kWavesM * kWavesN * 64;
  constexpr int MT = WM / 16, NT = WN / 16;
  constexpr int kChunks = BM * (kBK / 8);            // 16-byte pieces of one A tile
  constexpr int kLoads = kChunks / kThreads;         // per thread
  static_assert(kChunks % kThreads == 0, "A tile must split evenly over the threads");
  constexpr int kBPerTile = kW4 ? 1 : 2;             // 128-bit weight loads per n-tile and k-block

  extern __shared__ u32x4_t smem_raw[];
  uint16_t* lds = reinterpret_cast<uint16_t*>(smem_raw);  // 2 buffers of BM x kLdsRow

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int nl = lane & 15, kc = lane >> 4;
  const int wm = wave / kWavesN, wn = wave % kWavesN;

  // column-major walk over output tiles: consecutive workgroups share a column
  // block of W (and so its private tiles) and differ in the rows of x.
  const int tiles_m = (M + BM - 1) / BM;
  const int tile_m = blockIdx.x % tiles_m, tile_n = blockIdx.x / tiles_m;
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int KB = K / kBK;
  const int ntiles_total = N / kTileN;

  // ---- weight addressing: n16-tile index of each of this wave's column tiles
  const int nt0 = (n0 + wn * WN) / kTileN;
  const size_t tiles_per_row = kW4 ? (size_t)KB : (size_t)KB * 2;

  u32x4_t a_stage[kLoads];
  auto load_a = [&](int kb) {
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
      const int c = threadIdx.x + i * kThreads;
      const int row = c >> 4, col = c & 15;
      const int m = min(m0 + row, M - 1);  // rows past M repeat the last row; never stored
      a_stage[i] = *reinterpret_cast<const u32x4_t*>(x + (size_t)m * K + kb * kBK + col * 8);
    }
  };
  auto store_a = [&](int buf) {
    uint16_t* dst = lds + (size_t)buf * BM * kLdsRow;
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
      const int c = threadIdx.x + i * kThreads;
      const int row = c >> 4, col = c & 15;
      *reinterpret_cast<u32x4_t*>(dst + row * kLdsRow + col * 8) = a_stage[i];
    }
  };

  u32x4_t b_cur[NT][kBPerTile], b_nxt[NT][kBPerTile];
  uint32_t m_cur[NT], m_nxt[NT];
  f32x4_t gs_cur[MT], gs_nxt[MT];
  auto load_b = [&](int kb, u32x4_t (&b)[NT][kBPerTile], uint32_t (&mm)[NT], f32x4_t (&gs)[MT]) {
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const int nt = min(nt0 + t, ntiles_total - 1);
#pragma unroll
      for (int h = 0; h < kBPerTile; ++h)
        b[t][h] = wq[((size_t)nt * tiles_per_row + (size_t)kb * kBPerTile + h) * 64 + lane];
      if (kW4) mm[t] = meta[((size_t)nt * KB + kb) * 16 + nl];
    }
    if (kW4) {
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const int m = m0 + wm * WM + t * 16 + 4 * kc;  // < Mpad by construction
        gs[t] = *reinterpret_cast<const f32x4_t*>(gsum + (size_t)kb * Mpad + m);
      }
    }
  };

  f32x4_t acc[MT][NT];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < NT; ++j) acc[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  load_a(0);
  load_b(0, b_cur, m_cur, gs_cur);
  store_a(0);
  __syncthreads();

  for (int kb = 0; kb < KB; ++kb) {
    const int buf = kb & 1;
    const bool has_next = kb + 1 < KB;
    if (has_next) {
      load_a(kb + 1);
      load_b(kb + 1, b_nxt, m_nxt, gs_nxt);
    }
    const uint16_t* a_lds = lds + (size_t)buf * BM * kLdsRow + (wm * WM + nl) * kLdsRow + 8 * kc;

    f32x4_t part[MT][NT];
    if (kW4) {
#pragma unroll
      for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j) part[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {  // four k32 steps
      u32x4_t bf[NT];
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        if (kW4) {
          bf[t] = w4_to_bf16_biased(b_cur[t][0][j]);
        } else {
          const u32x2_t lo = w8_to_bf16(b_cur[t][j >> 1][2 * (j & 1)]);
          const u32x2_t hi = w8_to_bf16(b_cur[t][j >> 1][2 * (j & 1) + 1]);
          bf[t] = u32x4_t{lo.x, lo.y, hi.x, hi.y};
        }
      }
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        const u32x4_t af = *reinterpret_cast<const u32x4_t*>(a_lds + i * 16 * kLdsRow + 32 * j);
#pragma unroll
        for (int t = 0; t < NT; ++t) {
          if (kW4)
            part[i][t] = mfma16(af, bf[t], part[i][t]);
          else
            acc[i][t] = mfma16(af, bf[t], acc[i][t]);
        }
      }
    }
    if (kW4) {
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        const float s = f16_bits_to_f32(m_cur[t] & 0xFFFFu);
        const float zc = f16_bits_to_f32(m_cur[t] >> 16);
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
          for (int r = 0; r < 4; ++r) acc[i][t][r] += s * (part[i][t][r] - zc * gs_cur[i][r]);
      }
    }
    if (has_next) {
      store_a(buf ^ 1);  // the other buffer was last read before the previous barrier
#pragma unroll
      for (int t = 0; t < NT; ++t) {
#pragma unroll
        for (int h = 0; h < kBPerTile; ++h) b_cur[t][h] = b_nxt[t][h];
        m_cur[t] = m_nxt[t];
      }
#pragma unroll
      for (int t = 0; t < MT; ++t) gs_cur[t] = gs_nxt[t];
    }
    __syncthreads();
  }

  // ---- epilogue
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int n = n0 + wn * WN + t * 16 + nl;
    if (n >= N) continue;
    float cs = 1.0f;
    if (!kW4) cs = f16_bits_to_f32(scales8[n]);
#pragma unroll
    for (int i = 0; i < MT; ++i) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int m = m0 + wm * WM + i * 16 + 4 * kc + r;
        if (m < M) {
          const float v = acc[i][t][r] * cs;
          if (out_f32)
            reinterpret_cast<float*>(y)[(size_t)m * N + n] = v;
          else
            reinterpret_cast<uint16_t*>(y)[(size_t)m * N + n] = f32_to_bf16_rne(v);
        }
      }
    }
  }
}


}  // namespace ajq
