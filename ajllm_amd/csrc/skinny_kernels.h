// Batched-decode dequant matmul, 17 <= M < 256:  y[M, N] = x[M, K] @ W_hat[N, K]^T.
// The form for any K (K = 2048 and 4096 run skinny_resident_kernels.h, which keeps the activations in registers), the
// 32-row split-K form, and the epilogue both forms share (skinny_finish_unit).
//
// Still bound by the weight stream (a 4096 x 4096 int8 matrix is 16 MB, 32 rows of
// activations are 256 KB), so this is the decode GEMV's layout with more rows:
//  * one workgroup owns NT consecutive 16-row tiles of N, one block of MROWS rows of
//    M and all of K; wave w owns a contiguous run of 128-wide k groups (a contiguous
//    run of the private 1 KiB weight tiles of each row tile) and works through it
//    TPW groups at a time, the next batch in flight while one is computed;
//  * a wave stages ITS k-slice of the activation block in a wave-private LDS region
//    (rows padded by 16 B, no workgroup barrier) and reads it back as MFMA A
//    fragments, one per 16 rows; a weight fragment is unpacked once and meets
//    MROWS / 16 of them, an activation fragment is read once and meets NT weight
//    fragments (NT > 1 is for shapes with more row tiles than the chip has CUs);
//  * W4 zero points: the group sums of the activations come from MFMAs against an
//    all-ones operand, in the accumulator's layout, as in the GEMV;
//  * the waves' partial sums meet once in LDS (each wave's own region, which it no
//    longer needs) and are added in wave order: no atomics, run-to-run identical.
// Every workgroup reads its whole activation block from L2 (MROWS * K * 2 bytes
// against 16 * K * NT weight bytes or half that).  With one row tile per workgroup that
// is four times the int8 weight stream, and the L2s' delivery to the CUs (about 14 TB/s
// over the chip, measured) bounds the kernel instead of HBM: 82 MB for a 16.8 MB matrix
// at K = N = 4096, 293 MB for 58.7 MB at K = 14336.
//
// kSplitK: S workgroups share NT row tiles and take 1 / S of K each, so a row-tile group
// still has S * 8 waves' worth of loads in flight but the activation block is read once
// per group instead of once per tile (4 tiles x 4 splits: 33.6 MB and 117 MB for the two
// shapes above).  A workgroup leaves its partial sums in a caller-lent buffer, draws a
// ticket, and the one that draws the last ticket of its group adds the S partial results
// in split order (whatever order they arrived in: run-to-run identical) and runs the
// epilogue.  Nobody waits for anybody, so the kernel cannot hang on scheduling order.
#pragma once
#include "gemv_kernels.h"

namespace ajq {

template <int NT, int TPW, int kXLoads, int kLoadsPerGroup>
struct SkinnyBatch {
  u32x4_t w[NT][TPW][kLoadsPerGroup];
  u32x4_t x[kXLoads];
  uint32_t m[NT][TPW];
};

// kEpi: the epilogue forms of dequant_gemv_epi_kernel (row scale of an RMSNorm applied to the outputs,
// residual add with the next norm's preparation, SwiGLU gate on interleaved rows) for more rows than a GEMV
// takes; ssq_in is [M][parts], ssq_out [M][N / 16].
// Cross-workgroup part of the split-K form: S splits; `partial` holds S x NT x MROWS / 16 KiB per (row-tile group,
// row block), `tickets` one zeroed word each, which the kernel leaves zeroed.
struct SkinnySplit {
  float* partial;
  unsigned* tickets;
  int S;
};

// What becomes of one finished unit of a 32-row block that starts at row m0: row tile `tile` of N, 16-row block r;
// lane (nl, kc) holds rows 4 kc + i of the block in component i, column nl of the tile.  Channel scale (int8),
// the rows' norm factors, then the plain store, the residual form or the SwiGLU gate on interleaved rows.
template <bool kW4, int kEpi>
__device__ __forceinline__ void skinny_finish_unit(const f32x4_t& sum, int tile, int r, const float (&rstd)[4], int m0, int M,
                                                   int N, int lane, void* __restrict__ y, int out_f32,
                                                   const uint16_t* __restrict__ scales8, const GemvEpilogue& ep) {
  const int nl = lane & 15, kc = lane >> 4;
  const int ntiles = N / kTileN;
  const int n = tile * kTileN + nl;
  float cs = 1.0f;
  if (!kW4) cs = f16_bits_to_f32(scales8[n]);  // per-output-channel scale, once
  if (kEpi & kEpiResidual) {
    const float gain_n = ep.gain[n];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = m0 + 16 * r + 4 * kc + i;
      float v = sum[i] * cs * rstd[i];
      asm volatile("" : "+v"(v));  // no fused multiply-add: bit for bit the plain output, then the add
      const float h = (m < M ? ep.h_in[(size_t)m * N + n] : 0.f) + v;
      if (m < M) {
        ep.h_out[(size_t)m * N + n] = h;
        if (ep.xt) ep.xt[(size_t)m * N + n] = f32_to_bf16_rne(h * gain_n);
      }
      const float sq = team_sum16(m < M ? h * h : 0.f);
      if (nl == 0 && m < M) ep.ssq_out[(size_t)m * ntiles + tile] = sq;
    }
  } else if (kEpi & kEpiGate) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = m0 + 16 * r + 4 * kc + i;
      const float v = sum[i] * cs * rstd[i];
      const float other = row_ror<8>(v);  // the lane 8 columns away
      if (nl < 8 && m < M)
        reinterpret_cast<uint16_t*>(y)[(size_t)m * (N >> 1) + tile * 8 + nl] =
            f32_to_bf16_rne(v * (1.0f / (1.0f + expf(-v))) * other);
    }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = m0 + 16 * r + 4 * kc + i;
      if (m < M) {
        const float v = sum[i] * cs * rstd[i];
        if (out_f32)
          reinterpret_cast<float*>(y)[(size_t)m * N + n] = v;
        else
          reinterpret_cast<uint16_t*>(y)[(size_t)m * N + n] = f32_to_bf16_rne(v);
      }
    }
  }
}

template <int kWaves, int TPW, int MROWS, int NT, bool kW4, int kEpi, int kBatches = 0, bool kSplitK = false>
__device__ __forceinline__ void dequant_skinny_body(
    const u32x4_t* __restrict__ wq,
    const uint32_t* __restrict__ meta,     // W4: private meta; W8: unused
    const uint16_t* __restrict__ x, int K, int M, int N, void* __restrict__ y, int out_f32,
    const uint16_t* __restrict__ scales8,  // W8: fp16 [N]; W4: unused
    const GemvEpilogue& ep, const SkinnySplit& sp = SkinnySplit{}) {
  static_assert(MROWS % 16 == 0, "row block is a whole number of MFMA tiles");
  static_assert(kEpi == 0 || MROWS == 32, "the epilogue forms lay their row sums out for 32-row blocks");
  constexpr int MB = MROWS / 16;
  constexpr int kSlice = TPW * kGroup;     // k extent of one batch of one wave
  constexpr int kStride = kSlice + 8;      // padded LDS row, bf16 elements
  constexpr int kVecPerRow = kSlice / 8;   // 16-byte vectors per slice row
  constexpr int kXLoads = MROWS * kVecPerRow / 64;
  constexpr int kLoadsPerGroup = kW4 ? 1 : 2;
  using Batch = SkinnyBatch<NT, TPW, kXLoads, kLoadsPerGroup>;
  static_assert(NT * MB * 1024 <= MROWS * (kSlice + 8) * 2, "a wave's partial sums must fit its own LDS region");

  extern __shared__ u32x4_t smem_raw[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int nl = lane & 15, kc = lane >> 4;
  // Workgroup -> (row-tile group, row block).  Workgroups are dealt to the 8 XCDs round-robin
  // by index, and each XCD has its own L2: the row blocks of one row-tile group, which read
  // the same weights, are given consecutive slots of ONE XCD, so the weights come out of HBM
  // once and the other row blocks find them in that L2.
  const int ntiles = N / kTileN;
  const int ngroups = (ntiles + NT - 1) / NT;
  const int mblocks = (M + MROWS - 1) / MROWS;
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int S = kSplitK ? sp.S : 1;  // the splits of one (row-tile group, row block) sit in consecutive slots too
  const int ng = xcd + 8 * (slot / (mblocks * S));
  if (ng >= ngroups) return;  // padding of the last round (whole workgroup: no barrier is left waiting)
  const int nt0 = ng * NT;
  const int mblock = (slot / S) % mblocks, split = slot % S;
  const int m0 = mblock * MROWS;
  const int G = K >> 7;
  constexpr int kRegion = MROWS * kStride;  // bf16 elements of one wave's region
  uint16_t* xs = reinterpret_cast<uint16_t*>(smem_raw) + wave * kRegion;

  // this workgroup's groups (all of K, or split `split` of S equal parts), a contiguous run per wave
  const int g_count = G / S, g_first = split * g_count;
  const int per_wave = kBatches > 0 ? TPW * kBatches : (g_count + kWaves - 1) / kWaves;
  const int g_begin = g_first + wave * per_wave;
  const int g_end = min(g_first + g_count, g_begin + per_wave);

  // row tiles past the matrix repeat the last one (their results are not stored)
  const u32x4_t* wtile[NT];
  const uint32_t* mtile[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int nt = min(nt0 + t, ntiles - 1);
    wtile[t] = wq + (size_t)nt * G * kLoadsPerGroup * 64 + lane;
    mtile[t] = meta + (size_t)nt * G * 16 + nl;
  }

  // unconditional loads with clamped addresses: the number in flight is static
  // Issue order: the activations (from L2: back first, vector loads return in issue order), the meta words,
  // the weights.
  auto load = [&](Batch& b, int g0) {
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < kXLoads; ++i) {
      const int v = lane + 64 * i;
      const int m = min(m0 + v / kVecPerRow, M - 1), c = v % kVecPerRow;
      const int k = min(g0 * kGroup + 8 * c, K - 8);
      b.x[i] = *reinterpret_cast<const u32x4_t*>(x + (size_t)m * K + k);
    }
    if (kW4) {
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int p = 0; p < TPW; ++p) b.m[t][p] = mtile[t][(size_t)min(g0 + p, g_end - 1) * 16];
    }
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int p = 0; p < TPW; ++p) {
        const int g = min(g0 + p, g_end - 1);
#pragma unroll
        for (int h = 0; h < kLoadsPerGroup; ++h)
          b.w[t][p][h] = __builtin_nontemporal_load(wtile[t] + ((size_t)g * kLoadsPerGroup + h) * 64);
      }
    __builtin_amdgcn_sched_barrier(0);
  };

  const W4Consts w4c = w4_consts();
  const u32x4_t ones = {0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};
  const uint16_t* xrow = xs + nl * kStride + 8 * kc;  // A fragment of row block 0; block b is 16 rows further
  f32x4_t acc[NT][MB];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int b = 0; b < MB; ++b) acc[t][b] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  auto compute = [&](Batch& b, int g0) {
    float sc[NT][TPW], zc[NT][TPW];
    if (kW4) {
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int p = 0; p < TPW; ++p) {
          sc[t][p] = f16_bits_to_f32(b.m[t][p] & 0xFFFFu);
          zc[t][p] = f16_bits_to_f32(b.m[t][p] >> 16);
        }
    }
    // LDS operations of one wave execute in order: the previous batch's reads are done
#pragma unroll
    for (int i = 0; i < kXLoads; ++i) {
      const int v = lane + 64 * i;
      *reinterpret_cast<u32x4_t*>(xs + (v / kVecPerRow) * kStride + 8 * (v % kVecPerRow)) = b.x[i];
    }
#pragma unroll
    for (int p = 0; p < TPW; ++p) {
      if (g0 + p < g_end) {
        if (kW4) {
          f32x4_t part[NT][MB], asum[MB];
#pragma unroll
          for (int r = 0; r < MB; ++r) {
            asum[r] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int t = 0; t < NT; ++t) part[t][r] = f32x4_t{0.f, 0.f, 0.f, 0.f};
          }
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            u32x4_t w[NT];
#pragma unroll
            for (int t = 0; t < NT; ++t) w[t] = w4_unpack(b.w[t][p][0][j], w4c);
#pragma unroll
            for (int r = 0; r < MB; ++r) {
              const u32x4_t a = *reinterpret_cast<const u32x4_t*>(xrow + r * 16 * kStride + p * kGroup + 32 * j);
              asum[r] = mfma16(a, ones, asum[r]);
#pragma unroll
              for (int t = 0; t < NT; ++t) part[t][r] = mfma16(a, w[t], part[t][r]);
            }
          }
          // (128+q) and (128+z) cancel in fp32 before the scale is applied
#pragma unroll
          for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int r = 0; r < MB; ++r)
#pragma unroll
              for (int i = 0; i < 4; ++i) acc[t][r][i] += sc[t][p] * (part[t][r][i] - zc[t][p] * asum[r][i]);
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            u32x4_t w[NT];
#pragma unroll
            for (int t = 0; t < NT; ++t) {
              const u32x2_t lo = w8_to_bf16(b.w[t][p][j >> 1][2 * (j & 1)]);
              const u32x2_t hi = w8_to_bf16(b.w[t][p][j >> 1][2 * (j & 1) + 1]);
              w[t] = u32x4_t{lo.x, lo.y, hi.x, hi.y};
            }
#pragma unroll
            for (int r = 0; r < MB; ++r) {
              const u32x4_t a = *reinterpret_cast<const u32x4_t*>(xrow + r * 16 * kStride + p * kGroup + 32 * j);
#pragma unroll
              for (int t = 0; t < NT; ++t) acc[t][r] = mfma16(a, w[t], acc[t][r]);
            }
          }
        }
      }
    }
  };

  // row scale: this wave's share of the sums of squares of the block's 32 rows (lane -> row lane & 31, the two
  // half-waves take alternate 16-byte pieces), requested behind the first batch of weights, used at the end
  constexpr int kShareLoads = 32 / kWaves;  // 2 * kWaves * kShareLoads pieces of four: up to 256 parts
  float4 ssq_share[kShareLoads];
  float* red2 = reinterpret_cast<float*>(reinterpret_cast<uint16_t*>(smem_raw) + kWaves * kRegion);  // [32][kWaves]
  auto epilogue_loads = [&]() {
    if (kEpi & kEpiRowScale) {
      const int m = m0 + (lane & 31), half = lane >> 5;
#pragma unroll
      for (int u = 0; u < kShareLoads; ++u) {
        const int j = wave * 2 + half + u * kWaves * 2;
        const bool live = 4 * j < ep.parts && m < M;  // (idle lanes re-read the first 16 bytes)
        const float4 t = *reinterpret_cast<const float4*>(ep.ssq_in + (live ? (size_t)m * ep.parts + 4 * j : 0));
        ssq_share[u] = live ? t : float4{0.f, 0.f, 0.f, 0.f};
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  if (kBatches > 0 && g_begin >= g_end) {
    epilogue_loads();  // (more waves than runs of TPW * kBatches groups: the last waves have none)
  } else if constexpr (kBatches > 0) {
    // the workgroup's groups are a whole number of runs of TPW * kBatches: every wave that has any runs exactly
    // kBatches full batches, the loop is straight-line code and the number of loads in flight is known at every
    // wait (a batch is computed while the next travels)
    Batch b[2];
    load(b[0], g_begin);
    epilogue_loads();
#pragma unroll
    for (int i = 0; i < kBatches; ++i) {
      if (i + 1 < kBatches) load(b[(i + 1) & 1], g_begin + (i + 1) * TPW);
      compute(b[i & 1], g_begin + i * TPW);
    }
  } else if (g_begin >= g_end) {
    epilogue_loads();
  } else {
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

  // ---- partial sums: every wave parks its NT * MB accumulators at the start of its own region
  // (its LDS reads are done: same wave, in order); the (row tile, row block) units are dealt
  // round-robin to the waves, which add them in wave order
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int r = 0; r < MB; ++r) asm volatile("" : "+v"(acc[t][r]));
  f32x4_t* mine = reinterpret_cast<f32x4_t*>(xs);
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int r = 0; r < MB; ++r) mine[(t * MB + r) * 64 + lane] = acc[t][r];
  if (kEpi & kEpiRowScale) {
    float sh = 0.f;
#pragma unroll
    for (int u = 0; u < kShareLoads; ++u) sh += (ssq_share[u].x + ssq_share[u].y) + (ssq_share[u].z + ssq_share[u].w);
    sh += __shfl_xor(sh, 32);
    if (lane < 32) red2[lane * kWaves + wave] = sh;
  }
  __syncthreads();
  // the workgroup's sum of unit u: the waves' partial sums in wave order
  auto unit_sum = [&](int u) -> f32x4_t {
    f32x4_t part[kWaves];
#pragma unroll
    for (int w = 0; w < kWaves; ++w)
      part[w] = reinterpret_cast<const f32x4_t*>(reinterpret_cast<uint16_t*>(smem_raw) + w * kRegion)[u * 64 + lane];
    f32x4_t sum = part[0];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) sum += part[w];
    return sum;
  };
  f32x4_t* shared_partial = nullptr;  // split-K: [S][NT * MB][64] of this (row-tile group, row block)
  if constexpr (kSplitK) {
    __shared__ unsigned drawn;
    const int cell = ng * mblocks + mblock;
    shared_partial = reinterpret_cast<f32x4_t*>(sp.partial) + (size_t)cell * S * (NT * MB * 64);
    // The partial sums travel as device-scope atomic stores and loads (written through and read past the L2 of
    // the XCD, which is not coherent with the other seven): a device-scope release / acquire fence around plain
    // accesses writes back and invalidates the whole L2 each time, measured at 55 us for 256 workgroups.  A wave's
    // stores have completed when it arrives at the barrier (workgroup-scope release), the ticket is drawn after it.
    unsigned long long* cell_partial = reinterpret_cast<unsigned long long*>(shared_partial);
    for (int u = wave; u < NT * MB; u += kWaves) {
      const f32x4_t v = unit_sum(u);
      unsigned long long* dst = cell_partial + (((size_t)split * NT * MB + u) * 64 + lane) * 2;
      __hip_atomic_store(dst, (unsigned long long)__float_as_uint(v[0]) | ((unsigned long long)__float_as_uint(v[1]) << 32),
                         __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(dst + 1, (unsigned long long)__float_as_uint(v[2]) | ((unsigned long long)__float_as_uint(v[3]) << 32),
                         __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __syncthreads();
    if (threadIdx.x == 0) drawn = __hip_atomic_fetch_add(sp.tickets + cell, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (drawn != (unsigned)(S - 1)) return;
    if (threadIdx.x == 0) __hip_atomic_store(sp.tickets + cell, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  for (int u = wave; u < NT * MB; u += kWaves) {
    const int t = u / MB, r = u % MB;
    if (nt0 + t >= ntiles) break;
    f32x4_t sum;
    if constexpr (kSplitK) {
      const unsigned long long* src = reinterpret_cast<const unsigned long long*>(shared_partial) + ((size_t)u * 64 + lane) * 2;
      auto fetch = [&](int q) -> f32x4_t {
        const unsigned long long* at = src + (size_t)q * NT * MB * 128;
        const unsigned long long lo = __hip_atomic_load(at, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const unsigned long long hi = __hip_atomic_load(at + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return f32x4_t{__uint_as_float((uint32_t)lo), __uint_as_float((uint32_t)(lo >> 32)), __uint_as_float((uint32_t)hi),
                       __uint_as_float((uint32_t)(hi >> 32))};
      };
      sum = fetch(0);
      for (int q = 1; q < S; ++q) sum += fetch(q);
    } else {
      sum = unit_sum(u);
    }
    float rstd[4] = {1.0f, 1.0f, 1.0f, 1.0f};
    if (kEpi & kEpiRowScale) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float total = 0.f;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) total += red2[(16 * r + 4 * kc + i) * kWaves + w];
        rstd[i] = rsqrtf(total * ep.inv_k + ep.eps);
      }
    }
    skinny_finish_unit<kW4, kEpi>(sum, nt0 + t, r, rstd, m0, M, N, lane, y, out_f32, scales8, ep);
  }
}

template <int kWaves, int TPW, int MROWS, int NT, bool kW4, int kBatches = 0>
__global__ __launch_bounds__(kWaves * 64, kWaves <= 4 ? 2 : 1) void dequant_skinny_kernel(
    const u32x4_t* __restrict__ wq, const uint32_t* __restrict__ meta, const uint16_t* __restrict__ x, int K, int M, int N,
    void* __restrict__ y, int out_f32, const uint16_t* __restrict__ scales8) {
  dequant_skinny_body<kWaves, TPW, MROWS, NT, kW4, 0, kBatches>(wq, meta, x, K, M, N, y, out_f32, scales8, GemvEpilogue{});
}

template <int kWaves, int TPW, int MROWS, int NT, bool kW4, int kEpi, int kBatches = 0>
__global__ __launch_bounds__(kWaves * 64, kWaves <= 4 ? 2 : 1) void dequant_skinny_epi_kernel(
    const u32x4_t* __restrict__ wq, const uint32_t* __restrict__ meta, const uint16_t* __restrict__ x, int K, int M, int N,
    void* __restrict__ y, int out_f32, const uint16_t* __restrict__ scales8, GemvEpilogue ep) {
  dequant_skinny_body<kWaves, TPW, MROWS, NT, kW4, kEpi, kBatches>(wq, meta, x, K, M, N, y, out_f32, scales8, ep);
}

// the split-K forms (see kSplitK above)
template <int kWaves, int TPW, int MROWS, int NT, bool kW4, int kBatches = 0>
__global__ __launch_bounds__(kWaves * 64, kWaves <= 4 ? 2 : 1) void dequant_skinny_split_kernel(
    const u32x4_t* __restrict__ wq, const uint32_t* __restrict__ meta, const uint16_t* __restrict__ x, int K, int M, int N,
    void* __restrict__ y, int out_f32, const uint16_t* __restrict__ scales8, SkinnySplit sp) {
  dequant_skinny_body<kWaves, TPW, MROWS, NT, kW4, 0, kBatches, true>(wq, meta, x, K, M, N, y, out_f32, scales8,
                                                                       GemvEpilogue{}, sp);
}

template <int kWaves, int TPW, int MROWS, int NT, bool kW4, int kEpi, int kBatches = 0>
__global__ __launch_bounds__(kWaves * 64, kWaves <= 4 ? 2 : 1) void dequant_skinny_split_epi_kernel(
    const u32x4_t* __restrict__ wq, const uint32_t* __restrict__ meta, const uint16_t* __restrict__ x, int K, int M, int N,
    void* __restrict__ y, int out_f32, const uint16_t* __restrict__ scales8, GemvEpilogue ep, SkinnySplit sp) {
  dequant_skinny_body<kWaves, TPW, MROWS, NT, kW4, kEpi, kBatches, true>(wq, meta, x, K, M, N, y, out_f32, scales8, ep, sp);
}

// LDS bytes of one workgroup of dequant_skinny_kernel<kWaves, TPW, MROWS, *>
constexpr size_t skinny_lds_bytes(int waves, int tpw, int mrows) {
  return (size_t)waves * mrows * (tpw * kGroup + 8) * 2;
}
// ... of dequant_skinny_epi_kernel: the 32 rows' sums of squares, one share per wave, behind the waves' regions
constexpr size_t skinny_epi_lds_bytes(int waves, int tpw, int mrows) {
  return skinny_lds_bytes(waves, tpw, mrows) + (size_t)32 * waves * 4;
}

}  // namespace ajq
