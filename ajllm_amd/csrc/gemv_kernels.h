// Decode dequant-GEMV, 1 <= M <= 16:  y[M, N] = x[M, K] @ W_hat[N, K]^T.
//
// HBM-bound and short: a 4096 x 4096 int4 matrix is 8.7 MB, which the memory
// system delivers in well under two microseconds, and a wave's tiles (contiguous
// KiB) land together in one burst.  What the kernel can influence is how soon
// its loads are in flight and how little work is left once the weights are
// there, so it is laid out around that:
//  * one workgroup owns one 16-row tile of N and all of K; wave w owns a
//    contiguous run of 128-wide k groups, i.e. a contiguous run of 1 KiB private
//    weight tiles, and loads each with one 128-bit load per lane (a wave-wide
//    load instruction reads one contiguous KiB), non-temporal;
//  * a wave issues its weight loads before anything else (vector loads complete
//    in issue order, and every load instruction of the eight waves shares the
//    CU's one address path, so whatever is issued first delays the HBM requests);
//    then ITS k-slice of the activations, which it stages in a wave-private LDS
//    region (rows padded by 16 B; no workgroup barrier) and reads back as MFMA A
//    fragments, and the meta words;
//  * the per-group activation sums the zero-point term needs come from a second
//    MFMA against an all-ones B operand, which lands them in exactly the
//    accumulator layout that uses them;
//  * weights go global -> registers -> in-register unpack (3 shifts + 4
//    v_and_or_b32 per 8 nibbles) -> MFMA B operand; they never touch LDS.  Rows
//    >= M of the A operand repeat row M-1 and their outputs are never stored;
//  * the waves' partial sums meet once, through LDS, in a fixed order: no
//    atomics, results are run-to-run identical.
#pragma once
#include "ajq_common.h"

namespace ajq {

// One batch of a wave: TPW consecutive k groups, their weights, meta words and the
// matching slice of the activations, all in registers.
template <int TPW, int kXLoads, int kLoadsPerGroup>
struct GemvBatch {
  u32x4_t w[TPW][kLoadsPerGroup];
  u32x4_t x[kXLoads];
  uint32_t m[TPW];
};

// kWaves waves per workgroup; a wave works through its k groups TPW at a time;
// MROWS >= M is the compile-time row bound that sizes the activation slice.
// kSingle: K == kWaves * TPW * 128, every wave has exactly one full batch (no
// loop, no clamped addresses, no tail tests).
//
// kEpi adds work around the matmul for batched decode steps, where a launch of its own for the
// residual add, the RMSNorm or the SwiGLU gate costs more than the operation (bits may be combined):
//  * kEpiRowScale: the activations are x~ = bf16((h) * gain), NOT yet normalised, and every output row is
//    multiplied by rstd[m] = rsqrt(sum_k h[m][k]^2 / K + eps): the row scale of an RMSNorm commutes with
//    the matmul.  The sum of squares arrives as `parts` partial sums per row (ssq_in[16][parts], written
//    by the producing kernel's workgroups); every wave adds a fixed share of them while its weights
//    travel and wave 0 adds the waves' shares in wave order: no atomics, run-to-run identical.
//  * kEpiResidual: h_out = h_in + (x W^T) instead of y, together with x~ = bf16(h_out * gain) for the
//    norm that follows and the workgroup's partial sum of squares of its 16 columns, ssq_out[m][tile].
//  * kEpiGate: the 16 rows of a weight tile are 8 rows of the gate projection followed by the 8
//    matching rows of the up projection; y[m][8 tile + j] = bf16(silu(a_j) * u_j), [M, N / 2].
constexpr int kEpiRowScale = 1, kEpiResidual = 2, kEpiGate = 4;
struct GemvEpilogue {
  const float* ssq_in;  // row scale: [16][parts]
  int parts;            //   partial sums per row, a multiple of 4, at most kWaves * 32
  float inv_k, eps;     //   1 / K of the norm, its epsilon
  const float* h_in;    // residual: [M, N]
  const float* gain;    // residual: [N], gain of the norm that follows
  float* h_out;         // residual: [M, N], must not alias h_in
  uint16_t* xt;         // residual: bf16 [M, N]
  float* ssq_out;       // residual: [16][N / 16]
};

// W4 with at most four rows: the zero-point term's group sums, sum_k x over each 128-k group of the wave's
// LDS slice, by the VALU instead of a second MFMA per k-step against an all-ones operand.  With one live row
// an MFMA does sixteen rows' work for one, and the matrix pipe's time per tile (8 MFMAs of 32 cycles) is of
// the order of the tile's share of the memory stream; this halves it.  Team t of the wave (16 lanes) sums
// group t, t + 4, ...: one 16-byte LDS read per lane, seven adds, four row rotates; the result is wave-uniform.
// Rows >= M hold copies of row M - 1 (the staging clamps), so every row is read as it is.
template <int TPW, int MROWS>
__device__ __forceinline__ void gemv_group_sums(const uint16_t* xs, int stride, float (&gs)[MROWS][TPW]) {
  const int lane = threadIdx.x & 63, t = lane >> 4, c = lane & 15;
#pragma unroll
  for (int m = 0; m < MROWS; ++m) {
#pragma unroll
    for (int p0 = 0; p0 < TPW; p0 += 4) {
      const int p = min(p0 + t, TPW - 1);  // teams past the last group repeat it; their sums are not read
      const u32x4_t v = *reinterpret_cast<const u32x4_t*>(xs + m * stride + p * kGroup + 8 * c);
      auto lo = [](uint32_t w) { return __uint_as_float(w << 16); };
      auto hi = [](uint32_t w) { return __uint_as_float(w & 0xFFFF0000u); };
      float sum = ((lo(v.x) + hi(v.x)) + (lo(v.y) + hi(v.y))) + ((lo(v.z) + hi(v.z)) + (lo(v.w) + hi(v.w)));
      sum = team_sum16(sum);
#pragma unroll
      for (int q = 0; q < 4; ++q)
        if (p0 + q < TPW) gs[m][p0 + q] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(sum), 16 * q));
    }
  }
}
// whether a GEMV configuration takes its W4 group sums from gemv_group_sums
constexpr bool gemv_valu_group_sums(bool w4, int mrows) { return w4 && mrows <= 4; }

template <int kWaves, int TPW, int MROWS, bool kW4, bool kSingle, int kEpi, bool kFrags = false>
__device__ __forceinline__ void dequant_gemv_body(
    const u32x4_t* __restrict__ wq,
    const uint32_t* __restrict__ meta,     // W4: private meta; W8: unused
    const uint16_t* __restrict__ x, int K,
    int m_flags,  // M | out_f32 << 8 (one word: the leading arguments arrive preloaded in SGPRs)
    int N, void* __restrict__ y,
    const uint16_t* __restrict__ scales8,  // W8: fp16 [N]; W4: unused
    const GemvEpilogue& ep) {
  const int M = m_flags & 0xFF;
  const bool out_f32 = (m_flags >> 8) != 0;
  constexpr int kSlice = TPW * kGroup;     // k extent of one batch of one wave
  constexpr int kStride = kSlice + 8;      // padded LDS row, bf16 elements
  constexpr int kVecPerRow = kSlice / 8;   // 16-byte vectors per slice row
  constexpr int kVecs = MROWS * kVecPerRow;
  constexpr int kXLoads = (kVecs + 63) / 64;
  constexpr int kLoadsPerGroup = kW4 ? 1 : 2;  // 1 KiB tiles per 128 k
  constexpr int kRowQuads = (MROWS + 3) / 4;   // lane quarters (kc) that hold live output rows
  using Batch = GemvBatch<TPW, kXLoads, kLoadsPerGroup>;

  extern __shared__ u32x4_t smem_raw[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // uniform: scalar branches
  const int nl = lane & 15, kc = lane >> 4;
  const int nt = blockIdx.x;
  const int G = K >> 7;
  uint16_t* xs = reinterpret_cast<uint16_t*>(smem_raw) + wave * (MROWS * kStride);
  float* red = reinterpret_cast<float*>(reinterpret_cast<uint16_t*>(smem_raw) + kWaves * (MROWS * kStride));

  const int per_wave = kSingle ? TPW : (G + kWaves - 1) / kWaves;
  const int g_begin = wave * per_wave;
  const int g_end = kSingle ? g_begin + TPW : min(G, g_begin + per_wave);

  const u32x4_t* wtile = wq + (size_t)nt * G * kLoadsPerGroup * 64 + lane;
  const uint32_t* mtile = meta + (size_t)nt * G * 16 + nl;

  // Every load below is unconditional (addresses are clamped into the wave's own
  // range instead), so the number of loads in flight is static and the compiler
  // can wait for exactly the operand it is about to use.
  // Issue order: the activation slice (an L2 hit: one or two instructions, back long before the first weight
  // tile, so the wave stages it and forms what depends on it alone while the weights travel; vector loads
  // return in issue order), the meta words, the weights.
  auto load = [&](Batch& b, int g0) {
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < kXLoads; ++i) {
      const int v = min(lane + 64 * i, kVecs - 1);
      const int m = min(v / kVecPerRow, M - 1), c = v % kVecPerRow;
      const int k = kSingle ? g0 * kGroup + 8 * c : min(g0 * kGroup + 8 * c, K - 8);
      b.x[i] = *reinterpret_cast<const u32x4_t*>(x + (size_t)m * K + k);
    }
    if (kW4) {
#pragma unroll
      for (int p = 0; p < TPW; ++p)
        b.m[p] = mtile[(size_t)(kSingle ? g0 + p : min(g0 + p, g_end - 1)) * 16];
    }
#pragma unroll
    for (int p = 0; p < TPW; ++p) {
      const int g = kSingle ? g0 + p : min(g0 + p, g_end - 1);
#pragma unroll
      for (int h = 0; h < kLoadsPerGroup; ++h)
        b.w[p][h] = __builtin_nontemporal_load(wtile + ((size_t)g * kLoadsPerGroup + h) * 64);
    }
    // the whole batch is in flight before anything else happens: left alone, the
    // instruction scheduler sinks loads towards their first use and turns one
    // memory round trip into several
    __builtin_amdgcn_sched_barrier(0);
  };

  const W4Consts w4c = w4_consts();
  const u32x4_t ones = {0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};
  const int row = min(nl, M - 1);
  const uint16_t* xrow = xs + row * kStride + 8 * kc;
  f32x4_t acc = {0.f, 0.f, 0.f, 0.f};

  // slice of a batch -> wave-private LDS.  LDS operations of one wave execute in order, so the reads of the
  // previous batch are already done.
  auto stage = [&](const Batch& b) {
#pragma unroll
    for (int i = 0; i < kXLoads; ++i) {
      const int v = lane + 64 * i;
      if ((i + 1) * 64 <= kVecs || v < kVecs)
        *reinterpret_cast<u32x4_t*>(xs + (v / kVecPerRow) * kStride + 8 * (v % kVecPerRow)) = b.x[i];
    }
  };
  // kSingle: formed from the activations alone, before the weights have landed (see the kSingle branch below)
  static_assert(!kFrags || (kSingle && TPW <= 4), "A fragments are held in registers for single-batch waves of up to four tiles");
  constexpr bool kValuSums = gemv_valu_group_sums(kW4, MROWS);
  u32x4_t afr[kFrags ? TPW : 1][4];
  float gs[kValuSums ? MROWS : 1][TPW];
  auto fragment = [&](int p, int j) {
    if constexpr (kFrags) return afr[p][j];
    else return *reinterpret_cast<const u32x4_t*>(xrow + p * kGroup + 32 * j);
  };
  auto compute = [&](Batch& b, int g0) {
    // the meta words arrive before the weights (issued before them): scales and zero-points are ready when the
    // first tile lands
    float sc[TPW], zc[TPW];
    if (kW4) {
#pragma unroll
      for (int p = 0; p < TPW; ++p) {
        sc[p] = f16_bits_to_f32(b.m[p] & 0xFFFFu);
        zc[p] = f16_bits_to_f32(b.m[p] >> 16);
      }
    }
    if (!kSingle) {
      stage(b);
      if constexpr (kValuSums) gemv_group_sums<TPW, MROWS>(xs, kStride, gs);
    }
    if constexpr (kValuSums) {
#pragma unroll
      for (int p = 0; p < TPW; ++p) {
        if (kSingle || g0 + p < g_end) {
          f32x4_t part = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int j = 0; j < 4; ++j) part = mfma16(fragment(p, j), w4_unpack(b.w[p][0][j], w4c), part);
          // (128+q) and (128+z) cancel in fp32 before the scale is applied; only the lane quarter kc = 0
          // holds live rows (row i in component i)
#pragma unroll
          for (int i = 0; i < MROWS; ++i) acc[i] += sc[p] * (part[i] - zc[p] * gs[i][p]);
        }
      }
    } else if (kW4) {
#pragma unroll
      for (int p = 0; p < TPW; ++p) {
        if (kSingle || g0 + p < g_end) {
          // the group's activation sums (for the zero-point term) come from a second
          // MFMA against an all-ones B operand: same layout as the accumulator
          f32x4_t part = {0.f, 0.f, 0.f, 0.f}, asum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const u32x4_t a = fragment(p, j);
            part = mfma16(a, w4_unpack(b.w[p][0][j], w4c), part);
            asum = mfma16(a, ones, asum);
          }
          // (128+q) and (128+z) cancel in fp32 before the scale is applied
#pragma unroll
          for (int i = 0; i < (MROWS < 4 ? MROWS : 4); ++i) acc[i] += sc[p] * (part[i] - zc[p] * asum[i]);
        }
      }
    } else {
#pragma unroll
      for (int p = 0; p < TPW; ++p) {
        if (kSingle || g0 + p < g_end) {
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const u32x4_t a = fragment(p, j);
            const u32x2_t lo = w8_to_bf16(b.w[p][j >> 1][2 * (j & 1)]);
            const u32x2_t hi = w8_to_bf16(b.w[p][j >> 1][2 * (j & 1) + 1]);
            acc = mfma16(a, u32x4_t{lo.x, lo.y, hi.x, hi.y}, acc);
          }
        }
      }
    }
  };

  // two register sets, ping-pong: the next batch is in flight while one is computed
  // ---- what the epilogue variants need from memory is requested behind the first batch of weights
  // (vector loads return in issue order: in front of them it would delay the HBM requests) and used at
  // the end
  constexpr int kLiveRows = MROWS < 4 ? MROWS : 4;
  float* red2 = red + kWaves * 64 * 4;  // [16][kWaves] shares of the rows' sums of squares
  float4 ssq_share[2];
  float h_old[kLiveRows], gain_n = 0.f;
  auto epilogue_loads = [&]() {
    if (kEpi & kEpiRowScale) {
      const int m = lane & 15, c = lane >> 4;
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int j = wave * 4 + c + u * kWaves * 4;  // float4 index inside the row
        const bool live = 4 * j < ep.parts && m < M;  // (idle lanes re-read the first 16 bytes)
        const float4 t = *reinterpret_cast<const float4*>(ep.ssq_in + (live ? (size_t)m * ep.parts + 4 * j : 0));
        ssq_share[u] = live ? t : float4{0.f, 0.f, 0.f, 0.f};
      }
    }
    if (kEpi & kEpiResidual) {
      const int n = nt * kTileN + nl;
      gain_n = ep.gain[n];
#pragma unroll
      for (int i = 0; i < kLiveRows; ++i) h_old[i] = ep.h_in[(size_t)min(4 * kc + i, M - 1) * N + n];
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  if (kSingle) {
    Batch b0;
    load(b0, g_begin);
    epilogue_loads();
    // what needs the activations only, while the weights are on their way: the LDS image, the W4 group sums,
    // and (kFrags: launches of at most one workgroup per CU, where the registers cost no occupancy that
    // matters) the A fragments of every k-step
    stage(b0);
    if constexpr (kFrags) {
#pragma unroll
      for (int p = 0; p < TPW; ++p)
#pragma unroll
        for (int j = 0; j < 4; ++j) afr[p][j] = *reinterpret_cast<const u32x4_t*>(xrow + p * kGroup + 32 * j);
    }
    if constexpr (kValuSums) gemv_group_sums<TPW, MROWS>(xs, kStride, gs);
    __builtin_amdgcn_sched_barrier(0);
    compute(b0, g_begin);
  } else if (g_begin < g_end) {
    Batch b0, b1;
    load(b0, g_begin);
    epilogue_loads();
    for (int g0 = g_begin; g0 < g_end; g0 += 2 * TPW) {
      const bool has1 = g0 + TPW < g_end;
      if (has1) load(b1, g0 + TPW);
      compute(b0, g0);
      if (g0 + 2 * TPW < g_end) load(b0, g0 + 2 * TPW);
      if (has1) compute(b1, g0 + TPW);
    }
  }

  // ---- the waves' partial sums meet in LDS; wave 0 adds them in wave order.
  // Only the lane quarters that hold rows < MROWS take part.
  // (the empty asm pins the accumulator here: otherwise the compiler sinks the
  // epilogue arithmetic, and the loads that feed it, into the conditional store)
  asm volatile("" : "+v"(acc));
  constexpr int kLive = MROWS < 4 ? MROWS : 4;  // accumulator components that hold rows < MROWS
  typedef float live_t __attribute__((ext_vector_type(kLive == 3 ? 4 : kLive)));
  live_t* redv = reinterpret_cast<live_t*>(red);
  live_t mine;
#pragma unroll
  for (int i = 0; i < kLive; ++i) mine[i] = acc[i];
  if (kc < kRowQuads) redv[wave * (16 * kRowQuads) + lane] = mine;
  if (kEpi & kEpiRowScale) {
    // this wave's share of the rows' sums of squares: lane (row m = lane & 15, quarter c) holds 8 parts
    float sh = ((ssq_share[0].x + ssq_share[0].y) + (ssq_share[0].z + ssq_share[0].w)) +
               ((ssq_share[1].x + ssq_share[1].y) + (ssq_share[1].z + ssq_share[1].w));
    sh += __shfl_xor(sh, 16);
    sh += __shfl_xor(sh, 32);
    if (kc == 0) red2[nl * kWaves + wave] = sh;
  }
  __syncthreads();
  if (wave != 0 || kc >= kRowQuads) return;
  live_t part[kWaves];
#pragma unroll
  for (int w = 0; w < kWaves; ++w) part[w] = redv[w * (16 * kRowQuads) + lane];
  live_t sum = part[0];
#pragma unroll
  for (int w = 1; w < kWaves; ++w) sum += part[w];
  const int n = nt * kTileN + nl;
  float cs = 1.0f;
  if (!kW4) cs = f16_bits_to_f32(scales8[n]);  // per-output-channel scale, once
  float rstd[kLive];
#pragma unroll
  for (int i = 0; i < kLive; ++i) {
    rstd[i] = 1.0f;
    if (kEpi & kEpiRowScale) {
      float total = 0.f;
#pragma unroll
      for (int w = 0; w < kWaves; ++w) total += red2[min(4 * kc + i, 15) * kWaves + w];
      rstd[i] = rsqrtf(total * ep.inv_k + ep.eps);
    }
  }
  if (kEpi & kEpiResidual) {
    // the updated residual stream, its bf16 image for the next matmul, and this tile's sums of squares
    const int ntiles = N / kTileN;
#pragma unroll
    for (int i = 0; i < kLive; ++i) {
      const int m = 4 * kc + i;
      float v = sum[i] * cs * rstd[i];
      asm volatile("" : "+v"(v));  // no fused multiply-add: bit for bit the plain output, then the add
      const float h = h_old[i] + v;
      if (m < M) {
        ep.h_out[(size_t)m * N + n] = h;
        if (ep.xt) ep.xt[(size_t)m * N + n] = f32_to_bf16_rne(h * gain_n);
      }
      const float sq = team_sum16(m < M ? h * h : 0.f);  // over the tile's 16 columns (one DPP row)
      if (nl == 0 && m < M) ep.ssq_out[(size_t)m * ntiles + nt] = sq;
    }
    return;
  }
  if (kEpi & kEpiGate) {
    // columns 0..7 of the tile are gate projections, 8..15 the matching up projections
#pragma unroll
    for (int i = 0; i < kLive; ++i) {
      const int m = 4 * kc + i;
      const float v = sum[i] * cs * rstd[i];
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
      const float v = sum[i] * cs * rstd[i];
      if (out_f32)
        reinterpret_cast<float*>(y)[(size_t)m * N + n] = v;
      else
        reinterpret_cast<uint16_t*>(y)[(size_t)m * N + n] = f32_to_bf16_rne(v);
    }
  }
}

template <int kWaves, int TPW, int MROWS, bool kW4, bool kSingle, bool kFrags = false>
__global__ __launch_bounds__(kWaves * 64) void dequant_gemv_kernel(
    const u32x4_t* __restrict__ wq, const uint32_t* __restrict__ meta, const uint16_t* __restrict__ x, int K,
    int m_flags, int N, void* __restrict__ y, const uint16_t* __restrict__ scales8) {
  dequant_gemv_body<kWaves, TPW, MROWS, kW4, kSingle, 0, kFrags>(wq, meta, x, K, m_flags, N, y, scales8, GemvEpilogue{});
}

// the same kernel with work around the matmul (see kEpi above)
template <int kWaves, int TPW, int MROWS, bool kW4, bool kSingle, int kEpi, bool kFrags = false>
__global__ __launch_bounds__(kWaves * 64) void dequant_gemv_epi_kernel(
    const u32x4_t* __restrict__ wq, const uint32_t* __restrict__ meta, const uint16_t* __restrict__ x, int K,
    int m_flags, int N, void* __restrict__ y, const uint16_t* __restrict__ scales8, GemvEpilogue ep) {
  dequant_gemv_body<kWaves, TPW, MROWS, kW4, kSingle, kEpi, kFrags>(wq, meta, x, K, m_flags, N, y, scales8, ep);
}

// LDS bytes of one workgroup of dequant_gemv_kernel<kWaves, TPW, MROWS, *>
constexpr size_t gemv_lds_bytes(int waves, int tpw, int mrows) {
  return (size_t)waves * mrows * (tpw * kGroup + 8) * 2 + (size_t)waves * 64 * 16;
}
// ... of dequant_gemv_epi_kernel: the rows' sums of squares, one share per wave, behind the rest
constexpr size_t gemv_epi_lds_bytes(int waves, int tpw, int mrows) {
  return gemv_lds_bytes(waves, tpw, mrows) + (size_t)16 * waves * 4;
}

}  // namespace ajq
