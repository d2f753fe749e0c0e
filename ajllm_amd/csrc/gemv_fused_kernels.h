// Decode GEMV whose activations are produced on the way in (1 <= M <= 16,
// K == kWaves * TPW * 128):
//   kPro == kProNorm:  x = bf16( RMSNorm(h + delta) * gain ),  h + delta also written out
//                      (the residual update and the norm in front of q|k|v and w1|w3);
//   kPro == kProGate:  x = bf16( silu(a) * u ) for ab = (a | u)  (the SwiGLU gate in front of w2);
//   kPro == kProMerge: x = the single-query attention output, merged from the partial results
//                      of its S row chunks (what attn_merge_kernel computes, in front of the
//                      output projection: K = heads * 128, one k group per head).
// The matmul is dequant_gemv_kernel's straight-line variant: one workgroup per 16-row tile of
// N, wave w owns k groups [w * TPW, (w + 1) * TPW), weight loads first.  What changes is where
// a wave's k-slice of the activations comes from: it loads the fp32 sources of its slice (every
// workgroup repeats that work; the sources are a few KB and sit in L2), forms the bf16 values
// in registers and stages them in its private LDS rows as before.  The source loads are issued
// in front of the weight loads: vector loads return in issue order, the sources come from L2 and
// the weights from HBM, so this way the prologue arithmetic runs while the weights travel
// (issued behind them, the sources could not be touched before the last weight tile arrived).  The norm needs the whole
// row's sum of squares: every wave reduces its slice per row, the eight partial sums meet in
// LDS behind one barrier (the weight loads are in flight meanwhile).  Workgroup 0 writes the
// updated residual stream, to a buffer other than the one being read.
#pragma once
#include "gemv_kernels.h"
#include "decode_kernels.h"

namespace ajq {

constexpr int kProNorm = 1, kProGate = 2, kProMerge = 3, kProNormSums = 4;
// kProNormSums: x = bf16( (h / rms) * gain ) as kProNorm forms it, with rms taken from sums of squares that the
// PRODUCER of h left behind (src1 = ssq[rows][parts], per row the sums over 16-column tiles; S = parts): nothing
// is added to h, no workgroup barrier sits in front of the matmul (a wave adds the parts of its rows itself), and the
// activations are rounded exactly where the separate norm kernel rounds them.
// kOut: 0 plain output; kOutResid the residual epilogue (see dequant_gemv_epi_kernel); kOutGate the SwiGLU gate on
// rows interleaved in blocks of 8, y = bf16 [M, N / 2].
constexpr int kOutResid = 1, kOutGate = 2;

// chunks of one (row, head) a lane of the merge prologue takes (the 4 lane quarters take every 4th chunk)
constexpr int merge_chunks_per_lane(int mrows, int tpw) {
  return 8 / (mrows * tpw) > 4 ? 4 : (8 / (mrows * tpw) < 1 ? 1 : 8 / (mrows * tpw));
}

// kOutResid (with the merge prologue): h_out = res_h_in + (x W^T), res_xt = bf16(h_out * gain) for the norm that
// follows (skipped if null), res_ssq[m][tile] the sum of squares of h_out over this workgroup's 16 columns; y is
// not written.
template <int kWaves, int TPW, int MROWS, bool kW4, int kPro, int kOut = 0>
__global__ __launch_bounds__(kWaves * 64) void dequant_gemv_pro_kernel(
    const u32x4_t* __restrict__ wq,
    const uint32_t* __restrict__ meta,     // W4: private meta; W8: unused
    int K,
    int m_flags,  // M | out_f32 << 8
    int N, void* __restrict__ y,
    const uint16_t* __restrict__ scales8,  // W8: fp16 [N]; W4: unused
    const float* __restrict__ src0,        // norm: h_in [M, K];  gate: ab [M, 2K];  merge: partial [M * K / 128][S][132]
    const float* __restrict__ src1,        // norm: delta [M, K] or nullptr
    const float* __restrict__ gain,        // norm: [K]
    float eps,                             // norm
    float* __restrict__ h_out,             // norm: h_in + delta [M, K]; must not alias h_in.  kResid: [M, N]
    int S,                                 // merge: row chunks per (row, head), 1 <= S <= 4 * merge_chunks_per_lane
    const float* __restrict__ res_h_in,    // kResid: [M, N]
    uint16_t* __restrict__ res_xt,         // kResid: bf16 [M, N]
    float* __restrict__ res_ssq) {         // kResid: [16][N / 16]
  const int M = m_flags & 0xFF;
  const bool out_f32 = (m_flags >> 8) != 0;
  constexpr int kSlice = TPW * kGroup;
  constexpr int kStride = kSlice + 8;
  constexpr int kVecPerRow = kSlice / 8;  // 16 (TPW 1), 32 or 64 lanes hold one row's slice
  constexpr int kVecs = MROWS * kVecPerRow;
  constexpr int kXLoads = (kVecs + 63) / 64;
  constexpr int kLoadsPerGroup = kW4 ? 1 : 2;
  constexpr int kRowQuads = (MROWS + 3) / 4;
  static_assert(kVecPerRow <= 64, "a row's slice must fit one wave-wide load");

  extern __shared__ u32x4_t smem_raw[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int nl = lane & 15, kc = lane >> 4;
  const int nt = blockIdx.x;
  const int G = K >> 7;
  uint16_t* xs = reinterpret_cast<uint16_t*>(smem_raw) + wave * (MROWS * kStride);
  float* red = reinterpret_cast<float*>(reinterpret_cast<uint16_t*>(smem_raw) + kWaves * (MROWS * kStride));
  float* ssq = red + kWaves * 64 * 4;  // [MROWS][kWaves] partial sums of squares
  const int g0 = wave * TPW;

  // ---- loads: the fp32 sources of this wave's activation slice, then weights and meta
  u32x4_t w[TPW][kLoadsPerGroup];
  uint32_t mw[TPW];
  float4 a0[kXLoads][2], a1[kXLoads][2], a2[kXLoads][2];
  constexpr int kCpl = merge_chunks_per_lane(MROWS, TPW);
  constexpr int kPairs = kPro == kProMerge ? MROWS * TPW : 1;  // (row, head) pairs of this wave
  float4 pm[kPairs][kCpl], pa[kPairs][kCpl][2];                // merge: (max, denominator, -, -) and 8 sums per chunk
  __builtin_amdgcn_sched_barrier(0);
  if (kPro == kProMerge) {
    const int sgrp = lane >> 4, c = lane & 15;
#pragma unroll
    for (int q = 0; q < kPairs; ++q) {
      const int m = min(q / TPW, M - 1), head = g0 + q % TPW;
      const float* base = src0 + (size_t)(m * G + head) * S * kAttnPartialStride;
#pragma unroll
      for (int j = 0; j < kCpl; ++j) {
        const float* rec = base + (size_t)min(sgrp + 4 * j, S - 1) * kAttnPartialStride;
        pm[q][j] = *reinterpret_cast<const float4*>(rec);
        pa[q][j][0] = *reinterpret_cast<const float4*>(rec + 4 + 8 * c);
        pa[q][j][1] = *reinterpret_cast<const float4*>(rec + 8 + 8 * c);
      }
    }
  }
#pragma unroll
  for (int i = 0; i < kXLoads; ++i) {
    const int v = min(lane + 64 * i, kVecs - 1);
    const int m = min(v / kVecPerRow, M - 1), c = v % kVecPerRow;
    const int k = g0 * kGroup + 8 * c;
    if (kPro == kProNorm || kPro == kProNormSums) {
      const float4* ph = reinterpret_cast<const float4*>(src0 + (size_t)m * K + k);
      a0[i][0] = ph[0];
      a0[i][1] = ph[1];
      if (kPro == kProNorm && src1) {
        const float4* pd = reinterpret_cast<const float4*>(src1 + (size_t)m * K + k);
        a1[i][0] = pd[0];
        a1[i][1] = pd[1];
      } else {
        a1[i][0] = a1[i][1] = float4{0.f, 0.f, 0.f, 0.f};
      }
      const float4* pg = reinterpret_cast<const float4*>(gain + k);
      a2[i][0] = pg[0];
      a2[i][1] = pg[1];
    } else if (kPro == kProGate) {
      const float4* pa_ = reinterpret_cast<const float4*>(src0 + (size_t)m * 2 * K + k);
      const float4* pu = reinterpret_cast<const float4*>(src0 + (size_t)m * 2 * K + K + k);
      a0[i][0] = pa_[0];
      a0[i][1] = pa_[1];
      a1[i][0] = pu[0];
      a1[i][1] = pu[1];
    }
  }
  // kProNormSums: the 64 / MROWS lanes of a row share the parts of its sum of squares
  constexpr int kLanesPerRow = 64 / MROWS;
  constexpr int kPartLoads = kPro == kProNormSums ? (64 + kLanesPerRow - 1) / kLanesPerRow : 1;  // up to 256 parts
  float4 sums[kPartLoads];
  if (kPro == kProNormSums) {
    const int row = lane / kLanesPerRow, piece = lane % kLanesPerRow;
#pragma unroll
    for (int u = 0; u < kPartLoads; ++u) {
      const int j = piece + u * kLanesPerRow;
      const bool live = 4 * j < S && row < M;  // (idle lanes re-read the first 16 bytes)
      const float4 t = *reinterpret_cast<const float4*>(src1 + (live ? (size_t)row * S + 4 * j : 0));
      sums[u] = live ? t : float4{0.f, 0.f, 0.f, 0.f};
    }
  }
  if (kW4) {  // before the weights: scales and zero-points are there when the first tile lands
    const uint32_t* mtile = meta + ((size_t)nt * G + g0) * 16 + nl;
#pragma unroll
    for (int p = 0; p < TPW; ++p) mw[p] = mtile[p * 16];
  }
  {
    const u32x4_t* wtile = wq + ((size_t)nt * G + g0) * kLoadsPerGroup * 64 + lane;
#pragma unroll
    for (int p = 0; p < TPW; ++p)
#pragma unroll
      for (int h = 0; h < kLoadsPerGroup; ++h)
        w[p][h] = __builtin_nontemporal_load(wtile + (p * kLoadsPerGroup + h) * 64);
  }
  constexpr bool kResid = kOut == kOutResid;
  constexpr int kLiveRows = MROWS < 4 ? MROWS : 4;
  float h_old[kLiveRows], gain_n = 0.f;
  if (kResid) {  // behind the weights in issue order, used at the very end
    gain_n = gain[nt * kTileN + nl];
#pragma unroll
    for (int i = 0; i < kLiveRows; ++i) h_old[i] = res_h_in[(size_t)min(4 * kc + i, M - 1) * N + nt * kTileN + nl];
  }
  __builtin_amdgcn_sched_barrier(0);

  // ---- the activations of this slice, 8 per lane and load
  float xv[kXLoads][8];
  if (kPro == kProNorm) {
#pragma unroll
    for (int i = 0; i < kXLoads; ++i) {
      const float4 h0 = a0[i][0], h1 = a0[i][1], d0 = a1[i][0], d1 = a1[i][1];
      xv[i][0] = h0.x + d0.x; xv[i][1] = h0.y + d0.y; xv[i][2] = h0.z + d0.z; xv[i][3] = h0.w + d0.w;
      xv[i][4] = h1.x + d1.x; xv[i][5] = h1.y + d1.y; xv[i][6] = h1.z + d1.z; xv[i][7] = h1.w + d1.w;
      float ss = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += xv[i][e] * xv[i][e];
      // the kVecPerRow consecutive lanes of a row
#pragma unroll
      for (int off = kVecPerRow / 2; off > 0; off >>= 1) ss += __shfl_xor(ss, off);
      const int v = lane + 64 * i;
      if (v < kVecs && (v % kVecPerRow) == 0) ssq[(v / kVecPerRow) * kWaves + wave] = ss;
      if (nt == 0 && v < kVecs && v / kVecPerRow < M) {  // the updated residual stream, once
        float4* po = reinterpret_cast<float4*>(h_out + (size_t)(v / kVecPerRow) * K + g0 * kGroup + 8 * (v % kVecPerRow));
        po[0] = float4{xv[i][0], xv[i][1], xv[i][2], xv[i][3]};
        po[1] = float4{xv[i][4], xv[i][5], xv[i][6], xv[i][7]};
      }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < kXLoads; ++i) {
      const int v = min(lane + 64 * i, kVecs - 1);
      const float* part = ssq + (v / kVecPerRow) * kWaves;
      float total = 0.f;
#pragma unroll
      for (int u = 0; u < kWaves; ++u) total += part[u];
      const Divisor by_rms(sqrtf(total / (float)K + eps));
      const float4 g0v = a2[i][0], g1v = a2[i][1];
      xv[i][0] = by_rms.divide(xv[i][0]) * g0v.x; xv[i][1] = by_rms.divide(xv[i][1]) * g0v.y;
      xv[i][2] = by_rms.divide(xv[i][2]) * g0v.z; xv[i][3] = by_rms.divide(xv[i][3]) * g0v.w;
      xv[i][4] = by_rms.divide(xv[i][4]) * g1v.x; xv[i][5] = by_rms.divide(xv[i][5]) * g1v.y;
      xv[i][6] = by_rms.divide(xv[i][6]) * g1v.z; xv[i][7] = by_rms.divide(xv[i][7]) * g1v.w;
    }
  } else if (kPro == kProNormSums) {
    // a row's total in its first lane, then through the wave's own LDS words to whoever holds a piece of the row
    float total = 0.f;
#pragma unroll
    for (int u = 0; u < kPartLoads; ++u) total += (sums[u].x + sums[u].y) + (sums[u].z + sums[u].w);
    if (kLanesPerRow >= 16) {
      total = team_sum16(total);  // DPP row rotates inside each 16 lanes, then the crossbar for whole rows of 16
#pragma unroll
      for (int off = 16; off < kLanesPerRow; off <<= 1) total += __shfl_xor(total, off);
    } else {
#pragma unroll
      for (int off = kLanesPerRow / 2; off > 0; off >>= 1) total += __shfl_xor(total, off);
    }
    if (MROWS > 1 && lane % kLanesPerRow == 0) ssq[(lane / kLanesPerRow) * kWaves + wave] = total;
#pragma unroll
    for (int i = 0; i < kXLoads; ++i) {
      const int v = min(lane + 64 * i, kVecs - 1);
      // one row: every lane already holds its total
      const Divisor by_rms(sqrtf((MROWS > 1 ? ssq[(v / kVecPerRow) * kWaves + wave] : total) / (float)K + eps));
      const float4 h0 = a0[i][0], h1 = a0[i][1], g0v = a2[i][0], g1v = a2[i][1];
      xv[i][0] = by_rms.divide(h0.x) * g0v.x; xv[i][1] = by_rms.divide(h0.y) * g0v.y;
      xv[i][2] = by_rms.divide(h0.z) * g0v.z; xv[i][3] = by_rms.divide(h0.w) * g0v.w;
      xv[i][4] = by_rms.divide(h1.x) * g1v.x; xv[i][5] = by_rms.divide(h1.y) * g1v.y;
      xv[i][6] = by_rms.divide(h1.z) * g1v.z; xv[i][7] = by_rms.divide(h1.w) * g1v.w;
    }
  } else if (kPro == kProGate) {
#pragma unroll
    for (int i = 0; i < kXLoads; ++i) {
      const float av[8] = {a0[i][0].x, a0[i][0].y, a0[i][0].z, a0[i][0].w, a0[i][1].x, a0[i][1].y, a0[i][1].z, a0[i][1].w};
      const float uv[8] = {a1[i][0].x, a1[i][0].y, a1[i][0].z, a1[i][0].w, a1[i][1].x, a1[i][1].y, a1[i][1].z, a1[i][1].w};
#pragma unroll
      for (int e = 0; e < 8; ++e) xv[i][e] = av[e] * (1.0f / (1.0f + expf(-av[e]))) * uv[e];
    }
  }
  if (kPro == kProMerge) {
    // every (row, head) pair of the wave: lane quarter `sgrp` holds chunks sgrp, sgrp + 4, ... of the
    // 8 dimensions 8c .. 8c + 7; maxima, denominators and sums meet across the quarters, quarter 0
    // normalises and stages the 8 activations
    const int sgrp = lane >> 4, c = lane & 15;
#pragma unroll
    for (int q = 0; q < kPairs; ++q) {
      float mloc = -INFINITY;
#pragma unroll
      for (int j = 0; j < kCpl; ++j)
        if (sgrp + 4 * j < S) mloc = fmaxf(mloc, pm[q][j].x);
      float mall = fmaxf(mloc, __shfl_xor(mloc, 16));
      mall = fmaxf(mall, __shfl_xor(mall, 32));
      float L = 0.f, A[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j < kCpl; ++j) {
        if (sgrp + 4 * j < S) {
          const float cw = pm[q][j].x == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(pm[q][j].x - mall);
          L += pm[q][j].y * cw;
          A[0] += pa[q][j][0].x * cw; A[1] += pa[q][j][0].y * cw; A[2] += pa[q][j][0].z * cw; A[3] += pa[q][j][0].w * cw;
          A[4] += pa[q][j][1].x * cw; A[5] += pa[q][j][1].y * cw; A[6] += pa[q][j][1].z * cw; A[7] += pa[q][j][1].w * cw;
        }
      }
      L += __shfl_xor(L, 16);
      L += __shfl_xor(L, 32);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        A[e] += __shfl_xor(A[e], 16);
        A[e] += __shfl_xor(A[e], 32);
      }
      if (sgrp == 0) {
        u32x4_t pk;
        pk.x = pack2_bf16(A[0] / L, A[1] / L);
        pk.y = pack2_bf16(A[2] / L, A[3] / L);
        pk.z = pack2_bf16(A[4] / L, A[5] / L);
        pk.w = pack2_bf16(A[6] / L, A[7] / L);
        *reinterpret_cast<u32x4_t*>(xs + (q / TPW) * kStride + (q % TPW) * kGroup + 8 * c) = pk;
      }
    }
  }
  // bf16, into the wave's own LDS rows
#pragma unroll
  for (int i = 0; i < (kPro == kProMerge ? 0 : kXLoads); ++i) {
    const int v = lane + 64 * i;
    u32x4_t pk;
    pk.x = pack2_bf16(xv[i][0], xv[i][1]);
    pk.y = pack2_bf16(xv[i][2], xv[i][3]);
    pk.z = pack2_bf16(xv[i][4], xv[i][5]);
    pk.w = pack2_bf16(xv[i][6], xv[i][7]);
    if ((i + 1) * 64 <= kVecs || v < kVecs)
      *reinterpret_cast<u32x4_t*>(xs + (v / kVecPerRow) * kStride + 8 * (v % kVecPerRow)) = pk;
  }

  // ---- the matmul, as in dequant_gemv_kernel.  What depends on the activations alone comes first, while the
  // weights travel: the W4 group sums.  (Holding the A fragments in registers as well, as the plain GEMV does on
  // small launches, bought under 1 % of a decode step here and is not built.)
  constexpr bool kValuSums = gemv_valu_group_sums(kW4, MROWS);
  const uint16_t* xrow = xs + min(nl, M - 1) * kStride + 8 * kc;
  float gs[kValuSums ? MROWS : 1][TPW];
  if constexpr (kValuSums) gemv_group_sums<TPW, MROWS>(xs, kStride, gs);
  __builtin_amdgcn_sched_barrier(0);
  auto fragment = [&](int p, int j) { return *reinterpret_cast<const u32x4_t*>(xrow + p * kGroup + 32 * j); };
  float sc[TPW], zc[TPW];
  if (kW4) {
#pragma unroll
    for (int p = 0; p < TPW; ++p) {
      sc[p] = f16_bits_to_f32(mw[p] & 0xFFFFu);
      zc[p] = f16_bits_to_f32(mw[p] >> 16);
    }
  }
  const W4Consts w4c = w4_consts();
  const u32x4_t ones = {0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};
  f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
  if constexpr (kValuSums) {  // the same arithmetic as dequant_gemv_body, bit for bit
#pragma unroll
    for (int p = 0; p < TPW; ++p) {
      f32x4_t part = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j < 4; ++j) part = mfma16(fragment(p, j), w4_unpack(w[p][0][j], w4c), part);
#pragma unroll
      for (int i = 0; i < MROWS; ++i) acc[i] += sc[p] * (part[i] - zc[p] * gs[i][p]);
    }
  } else if (kW4) {
#pragma unroll
    for (int p = 0; p < TPW; ++p) {
      f32x4_t part = {0.f, 0.f, 0.f, 0.f}, asum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const u32x4_t a = fragment(p, j);
        part = mfma16(a, w4_unpack(w[p][0][j], w4c), part);
        asum = mfma16(a, ones, asum);
      }
#pragma unroll
      for (int i = 0; i < (MROWS < 4 ? MROWS : 4); ++i) acc[i] += sc[p] * (part[i] - zc[p] * asum[i]);
    }
  } else {
#pragma unroll
    for (int p = 0; p < TPW; ++p)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const u32x4_t a = fragment(p, j);
        const u32x2_t lo = w8_to_bf16(w[p][j >> 1][2 * (j & 1)]);
        const u32x2_t hi = w8_to_bf16(w[p][j >> 1][2 * (j & 1) + 1]);
        acc = mfma16(a, u32x4_t{lo.x, lo.y, hi.x, hi.y}, acc);
      }
  }

  // ---- the waves' partial sums meet in LDS; wave 0 adds them in wave order
  asm volatile("" : "+v"(acc));
  constexpr int kLive = MROWS < 4 ? MROWS : 4;
  typedef float live_t __attribute__((ext_vector_type(kLive == 3 ? 4 : kLive)));
  live_t* redv = reinterpret_cast<live_t*>(red);
  live_t mine;
#pragma unroll
  for (int i = 0; i < kLive; ++i) mine[i] = acc[i];
  if (kc < kRowQuads) redv[wave * (16 * kRowQuads) + lane] = mine;
  __syncthreads();
  if (wave != 0 || kc >= kRowQuads) return;
  live_t part[kWaves];
#pragma unroll
  for (int u = 0; u < kWaves; ++u) part[u] = redv[u * (16 * kRowQuads) + lane];
  live_t sum = part[0];
#pragma unroll
  for (int u = 1; u < kWaves; ++u) sum += part[u];
  const int n = nt * kTileN + nl;
  float cs = 1.0f;
  if (!kW4) cs = f16_bits_to_f32(scales8[n]);
  if (kResid) {
    const int ntiles = N / kTileN;
#pragma unroll
    for (int i = 0; i < kLive; ++i) {
      const int m = 4 * kc + i;
      float v = sum[i] * cs;
      asm volatile("" : "+v"(v));  // no fused multiply-add: bit for bit the plain output, then the add
      const float h = h_old[i] + v;
      if (m < M) {
        h_out[(size_t)m * N + n] = h;
        if (res_xt) res_xt[(size_t)m * N + n] = f32_to_bf16_rne(h * gain_n);
      }
      const float sq = team_sum16(m < M ? h * h : 0.f);
      if (nl == 0 && m < M) res_ssq[(size_t)m * ntiles + nt] = sq;
    }
    return;
  }
  if (kOut == kOutGate) {
    // columns 0..7 of the tile are gate projections, 8..15 the matching up projections
#pragma unroll
    for (int i = 0; i < kLive; ++i) {
      const int m = 4 * kc + i;
      const float v = sum[i] * cs;
      const float other = row_ror<8>(v);  // the lane 8 columns away
      if (nl < 8 && m < M)
        reinterpret_cast<uint16_t*>(y)[(size_t)m * (N >> 1) + nt * 8 + nl] =
            f32_to_bf16_rne(v * (1.0f / (1.0f + expf(-v))) * other);
    }
    return;
  }
#pragma unroll
  for (int i = 0; i < kLive; ++i) {
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

// LDS bytes of one workgroup: activation slices, reduction slots, partial sums of squares
constexpr size_t gemv_pro_lds_bytes(int waves, int tpw, int mrows) {
  return gemv_lds_bytes(waves, tpw, mrows) + (size_t)mrows * waves * 4;
}

}  // namespace ajq
