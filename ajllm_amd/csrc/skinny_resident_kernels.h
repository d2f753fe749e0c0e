// Weight-streaming dequant matmul for shapes with several 16-row tiles of N per CU and K <= 4096 (17 <= M < 256,
// N / 16 well above the CU count: the concatenated w1 | w3 of a feed-forward block, a vocabulary head).
//
// dequant_skinny_kernel gives every workgroup its own copy of the 32 x K activation block out of L2, and with
// four row tiles per workgroup that copy is as many bytes as the int8 weights it meets (twice the int4 ones); the
// L2s' delivery to the CUs bounds it, not HBM.  Here a workgroup keeps the activation block RESIDENT and walks a run
// of consecutive row tiles past it:
//  * eight waves split K: wave w owns the k-slice [w K / 8, (w + 1) K / 8) (TPW = K / 1024 groups of 128) of every
//    row tile of the workgroup.  It loads its slice of the 32 activation rows once (row-major, through a
//    wave-private LDS region, no barrier), and keeps it as MFMA A fragments in registers: 32 TPW registers;
//  * W4: the slice's group sums (for the zero-point term) are formed once, not once per row tile;
//  * then the row tiles one after the other: the wave's 2 or 1 KiB x TPW of tiles t + 1 and (once tile t is done)
//    t + 2 travel while tile t is computed (two register sets, asm loads with exact waits); the eight waves together read a tile's 16 K bytes
//    as one contiguous run and the workgroup its T tiles as one contiguous sweep, which HBM serves much better than
//    one 64 KiB stream per wave (measured: 4.8 against 6 TB/s and more);
//  * a wave parks each finished tile's partial sums in its LDS region; at the end the (row tile, 16-row block)
//    units are dealt round-robin to the waves, added in wave order (no atomics: run-to-run identical) and finished
//    by the epilogue forms of the weight-streaming kernel (skinny_finish_unit).
// Bytes into a CU per 16 output columns: K (64 / T + 16 b), b = bytes per weight, against K (64 / 4 + 16 b).
#pragma once
#include "gemm_split_kernels.h"
#include "skinny_kernels.h"

namespace ajq {

constexpr int kResWaves = 8;
constexpr int kResMaxUnits = 16;                              // (row tile, 16-row block) units per workgroup, at most
constexpr int kResStride = kGroup + 8;                        // staging: one group of a row, padded, bf16 elements
// a wave's LDS region: the staging of one group of its 16 MB rows, later 1 KiB of partial sums per unit
constexpr int res_region_bytes(int tiles, int mb) {
  return 16 * mb * kResStride * 2 > tiles * mb * 1024 ? 16 * mb * kResStride * 2 : tiles * mb * 1024;
}
// LDS bytes of one workgroup; the epilogue forms add the rows' sums of squares, one share per wave
constexpr size_t res_lds_bytes(int tiles, int mb, bool epi) {
  return (size_t)kResWaves * res_region_bytes(tiles, mb) + (epi ? (size_t)32 * kResWaves * 4 : 0);
}

__device__ __forceinline__ void load16_async_nt(u32x4_t& dst, const void* base, uint32_t voff) {
  asm volatile("global_load_dwordx4 %0, %1, %2 nt" : "=&v"(dst) : "v"(voff), "s"(base) : "memory");
}

template <int TPW, bool kW4>
struct ResidentTile {
  u32x4_t w[TPW][kW4 ? 1 : 2];
  uint32_t m[TPW];
};
// waits until at most kLeft of the wave's loads are in flight; names the set's registers so that no use moves
// above the wait
template <int kLeft, int TPW, bool kW4>
__device__ __forceinline__ void wait_tile(ResidentTile<TPW, kW4>& s) {
#pragma unroll
  for (int p = 0; p < TPW; ++p) {
    if constexpr (kW4)
      asm volatile("s_waitcnt vmcnt(%2)" : "+v"(s.w[p][0]), "+v"(s.m[p]) : "n"(kLeft) : "memory");
    else
      asm volatile("s_waitcnt vmcnt(%2)" : "+v"(s.w[p][0]), "+v"(s.w[p][1]) : "n"(kLeft) : "memory");
  }
}

template <int kLeft>
__device__ __forceinline__ void wait_rows(u32x4_t (&r)[8]) {
  asm volatile("s_waitcnt vmcnt(%8)"
               : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]), "+v"(r[4]), "+v"(r[5]), "+v"(r[6]), "+v"(r[7])
               : "n"(kLeft)
               : "memory");
}
template <int kLeft>
__device__ __forceinline__ void wait_rows(u32x4_t (&r)[4]) {
  asm volatile("s_waitcnt vmcnt(%4)" : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]) : "n"(kLeft) : "memory");
}

template <int TPW, int T, bool kW4, int kEpi, int MB = 2, int kWaves = kResWaves, bool kSplitK = false>
__device__ __forceinline__ void dequant_skinny_resident_body(
    const u32x4_t* __restrict__ wq,
    const uint32_t* __restrict__ meta,     // W4: private meta; W8: unused
    const uint16_t* __restrict__ x, int K, int M, int N, void* __restrict__ y, int out_f32,
    const uint16_t* __restrict__ scales8,  // W8: fp16 [N]; W4: unused
    const GemvEpilogue& ep, const SkinnySplit& sp = SkinnySplit{}) {
  static_assert(kWaves <= kResWaves, "the LDS regions are laid out for at most eight waves");
  static_assert(T >= 1 && T * MB <= kResMaxUnits, "a wave's region holds the partial sums of T row tiles");
  constexpr int kLPG = kW4 ? 1 : 2;              // 1 KiB weight tiles per group
  constexpr int kWL = TPW * (kLPG + (kW4 ? 1 : 0));  // loads per wave and row tile
  using Tile = ResidentTile<TPW, kW4>;

  extern __shared__ u32x4_t smem_raw[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int nl = lane & 15, kc = lane >> 4;
  // workgroup -> (run of T row tiles, row block): the row blocks of one run share an XCD (see dequant_skinny_kernel)
  const int ntiles = N / kTileN;
  const int nruns = (ntiles + T - 1) / T;
  constexpr int kRows = 16 * MB;  // rows of a row block
  const int mblocks = (M + kRows - 1) / kRows;
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  // split-K: S workgroups share a run and take 1 / S of K each (consecutive slots of the run's XCD)
  const int S = kSplitK ? sp.S : 1;
  const int run = xcd + 8 * (slot / (mblocks * S));
  if (run >= nruns) return;  // padding of the last round (whole workgroup: no barrier is left waiting)
  const int mblock = (slot / S) % mblocks, split = slot % S;
  const int m0 = mblock * kRows;
  const int nt0 = run * T;
  const int tiles = min(T, ntiles - nt0);  // >= 1; past the matrix the last row tile is computed again, not stored
  const int G = K >> 7;                    // = S * kWaves * TPW (checked by the host)
  const int g0 = (split * kWaves + wave) * TPW;
  constexpr int kRegionBytes = res_region_bytes(T, MB);
  char* region = reinterpret_cast<char*>(smem_raw) + wave * kRegionBytes;
  uint16_t* xs = reinterpret_cast<uint16_t*>(region);

  // ---- this wave's slice of the weights of row tile nt0 + t: TPW * kLPG KiB, contiguous
  const uint32_t lane16 = (uint32_t)lane * 16u, nl4 = (uint32_t)nl * 4u;
  auto request = [&](Tile& set, int t) __attribute__((always_inline)) {
    const size_t first = (size_t)min(nt0 + t, ntiles - 1) * G + g0;
    const char* wsrc = reinterpret_cast<const char*>(wq) + first * (kLPG * 1024);
    const char* msrc = reinterpret_cast<const char*>(meta) + first * 64;
#pragma unroll
    for (int p = 0; p < TPW; ++p) {
      if (kW4) load4_async(set.m[p], msrc + p * 64, nl4);
#pragma unroll
      for (int h = 0; h < kLPG; ++h) load16_async_nt(set.w[p][h], wsrc + (p * kLPG + h) * 1024, lane16);
    }
  };

  // ---- the activation slice: one group at a time, row-major into the wave's region (rows padded by 16 B so the
  // 16 rows of an A fragment fall in distinct banks), back as A fragments; LDS operations of one wave execute in
  // order, so no barrier is needed
  u32x4_t frag[TPW][4][MB];
  f32x4_t asum[TPW][MB];
  const u32x4_t ones = {0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};
  // row tiles in flight: two register sets (four were measured: 3 % faster at K = 2048, 2-4 % slower at K = 4096,
  // and with 32 rows they do not fit the register file)
  constexpr int kSets = T < 2 ? T : 2;
  static_assert(kSets >= 1 && kSets <= 4, "the waits below count up to three tiles behind the current one");
  Tile set[kSets];
  {
    // all requests of the prologue are asm, so that every wait is exact: the activations (L2 hits) come back while
    // the first row tile's weights are still on their way from memory
    constexpr int kXL = 4 * MB;  // 16-byte vectors per lane and group
    u32x4_t raw[TPW][kXL];
    uint32_t xoff[kXL];
#pragma unroll
    for (int i = 0; i < kXL; ++i) {
      const int v = lane + 64 * i;  // 16-byte vector v of a 32 x 128 block: row v / 16, vector v % 16
      xoff[i] = (uint32_t)((min(m0 + (v >> 4), M - 1) * K + 8 * (v & 15)) * 2);
    }
#pragma unroll
    for (int p = 0; p < TPW; ++p)
#pragma unroll
      for (int i = 0; i < kXL; ++i) load16_async(raw[p][i], reinterpret_cast<const char*>(x) + (g0 + p) * (kGroup * 2), xoff[i]);
#pragma unroll
    for (int t = 0; t < kSets; ++t) request(set[t], t);  // the first row tiles' weights travel while the activations are staged
    constexpr int kAhead = kSets * kWL;
#pragma unroll
    for (int p = 0; p < TPW; ++p) {
      if (p == 0) wait_rows<kAhead + kXL * (TPW - 1)>(raw[0]);
      if (p == 1) wait_rows<kAhead + kXL * (TPW > 1 ? TPW - 2 : 0)>(raw[TPW > 1 ? 1 : 0]);
      if (p == 2) wait_rows<kAhead + kXL * (TPW > 2 ? TPW - 3 : 0)>(raw[TPW > 2 ? 2 : 0]);
      if (p == 3) wait_rows<kAhead>(raw[TPW > 3 ? 3 : 0]);
#pragma unroll
      for (int i = 0; i < kXL; ++i) {
        const int v = lane + 64 * i;
        *reinterpret_cast<u32x4_t*>(xs + (v >> 4) * kResStride + 8 * (v & 15)) = raw[p][i];
      }
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int r = 0; r < MB; ++r)
          frag[p][j][r] = *reinterpret_cast<const u32x4_t*>(xs + (16 * r + nl) * kResStride + 32 * j + 8 * kc);
      if (kW4) {
#pragma unroll
        for (int r = 0; r < MB; ++r) {
          asum[p][r] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int j = 0; j < 4; ++j) asum[p][r] = mfma16(frag[p][j][r], ones, asum[p][r]);
        }
      }
    }
  }

  // ---- row scale: this wave's share of the sums of squares of the block's 32 rows (lane -> row lane & 31, the two
  // half-waves take alternate 16-byte pieces), used at the end
  constexpr int kShareLoads = (32 + kWaves - 1) / kWaves;
  float4 ssq_share[kShareLoads];
  float* red2 = reinterpret_cast<float*>(reinterpret_cast<char*>(smem_raw) + kWaves * kRegionBytes);  // [32][kWaves]
  if (kEpi & kEpiRowScale) {
    const int m = m0 + (lane & 31), half = lane >> 5;
#pragma unroll
    for (int u = 0; u < kShareLoads; ++u) {
      const int j = wave * 2 + half + u * kWaves * 2;
      const bool live = 4 * j < ep.parts && m < M && (lane & 31) < kRows;  // (idle lanes re-read the first 16 bytes)
      const float4 t = *reinterpret_cast<const float4*>(ep.ssq_in + (live ? (size_t)m * ep.parts + 4 * j : 0));
      ssq_share[u] = live ? t : float4{0.f, 0.f, 0.f, 0.f};
    }
  }

  const W4Consts w4c = w4_consts();
  f32x4_t* mine = reinterpret_cast<f32x4_t*>(region);  // [tile][16-row block][lane]
  auto compute = [&](Tile& set, int t) __attribute__((always_inline)) {
    f32x4_t acc[MB];
#pragma unroll
    for (int r = 0; r < MB; ++r) acc[r] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int p = 0; p < TPW; ++p) {
      if (kW4) {
        const float sc = f16_bits_to_f32(set.m[p] & 0xFFFFu), zc = f16_bits_to_f32(set.m[p] >> 16);
        f32x4_t part[MB];
#pragma unroll
        for (int r = 0; r < MB; ++r) part[r] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const u32x4_t w = w4_unpack(set.w[p][0][j], w4c);
#pragma unroll
          for (int r = 0; r < MB; ++r) part[r] = mfma16(frag[p][j][r], w, part[r]);
        }
        // (128+q) and (128+z) cancel in fp32 before the scale is applied
#pragma unroll
        for (int r = 0; r < MB; ++r)
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[r][i] += sc * (part[r][i] - zc * asum[p][r][i]);
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const u32x2_t lo = w8_to_bf16(set.w[p][j >> 1][2 * (j & 1)]);
          const u32x2_t hi = w8_to_bf16(set.w[p][j >> 1][2 * (j & 1) + 1]);
          const u32x4_t w = u32x4_t{lo.x, lo.y, hi.x, hi.y};
#pragma unroll
          for (int r = 0; r < MB; ++r) acc[r] = mfma16(frag[p][j][r], w, acc[r]);
        }
      }
    }
#pragma unroll
    for (int r = 0; r < MB; ++r) mine[(t * MB + r) * 64 + lane] = acc[r];
  };

  // ---- the row tiles, two register sets in turn (the first two tiles' weights were requested in the prologue;
  // a set is requested again as soon as its tile is computed).
  // Straight-line code on purpose: with the sets carried around a loop the compiler may copy a set's registers
  // between the request and the wait, while the loads are still in flight.
#pragma unroll
  for (int t = 0; t < T; ++t) {
    // in flight behind tile t: the tiles up to t + kSets - 1 that exist
    const int behind = t + kSets - 1 < T ? kSets - 1 : T - 1 - t;  // (a constant once the loop is unrolled)
    if (behind == 0) wait_tile<0>(set[t % kSets]);
    if (behind == 1) wait_tile<kWL>(set[t % kSets]);
    if (behind == 2) wait_tile<2 * kWL>(set[t % kSets]);
    if (behind == 3) wait_tile<3 * kWL>(set[t % kSets]);
    compute(set[t % kSets], t);
    if (t + kSets < T) request(set[t % kSets], t + kSets);
  }

  if (kEpi & kEpiRowScale) {
    float sh = 0.f;
#pragma unroll
    for (int u = 0; u < kShareLoads; ++u) sh += (ssq_share[u].x + ssq_share[u].y) + (ssq_share[u].z + ssq_share[u].w);
    sh += __shfl_xor(sh, 32);
    if (lane < 32) red2[lane * kWaves + wave] = sh;
  }
  __syncthreads();
  // ---- the (row tile, 16-row block) units, dealt round-robin to the waves: the waves' partial sums in wave order
  auto unit_sum = [&](int u) -> f32x4_t {
    f32x4_t part[kWaves];
#pragma unroll
    for (int w = 0; w < kWaves; ++w)
      part[w] = reinterpret_cast<const f32x4_t*>(reinterpret_cast<const char*>(smem_raw) + w * kRegionBytes)[u * 64 + lane];
    f32x4_t sum = part[0];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) sum += part[w];
    return sum;
  };
  const unsigned long long* cell_partial = nullptr;  // split-K: [S][T * MB][64] f32x4 of this (run, row block)
  if constexpr (kSplitK) {
    // the exchange of dequant_skinny_kernel's split-K form: partial sums as device-scope relaxed atomic stores
    // (written through the L2, which is not coherent across XCDs), complete at the workgroup barrier; a ticket;
    // the workgroup that draws the last one adds the S partial results in split order and leaves the ticket zero
    __shared__ unsigned drawn;
    const int cell = run * mblocks + mblock;
    unsigned long long* mine_out = reinterpret_cast<unsigned long long*>(sp.partial) + (size_t)cell * S * (T * MB * 128);
    cell_partial = mine_out;
    for (int u = wave; u < MB * tiles; u += kWaves) {
      const f32x4_t v = unit_sum(u);
      unsigned long long* dst = mine_out + (((size_t)split * T * MB + u) * 64 + lane) * 2;
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
  for (int u = wave; u < MB * tiles; u += kWaves) {
    const int t = u / MB, r = u % MB;
    f32x4_t sum;
    if constexpr (kSplitK) {
      const unsigned long long* src = cell_partial + ((size_t)u * 64 + lane) * 2;
      auto fetch = [&](int q) -> f32x4_t {
        const unsigned long long* at = src + (size_t)q * T * MB * 128;
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

template <int TPW, int T, bool kW4, int MB = 2>
__global__ __launch_bounds__(kResWaves * 64, 2) void dequant_skinny_resident_kernel(
    const u32x4_t* __restrict__ wq, const uint32_t* __restrict__ meta, const uint16_t* __restrict__ x, int K, int M, int N,
    void* __restrict__ y, int out_f32, const uint16_t* __restrict__ scales8) {
  dequant_skinny_resident_body<TPW, T, kW4, 0, MB>(wq, meta, x, K, M, N, y, out_f32, scales8, GemvEpilogue{});
}

template <int TPW, int T, bool kW4, int kEpi, int MB = 2>
__global__ __launch_bounds__(kResWaves * 64, 2) void dequant_skinny_resident_epi_kernel(
    const u32x4_t* __restrict__ wq, const uint32_t* __restrict__ meta, const uint16_t* __restrict__ x, int K, int M, int N,
    void* __restrict__ y, int out_f32, const uint16_t* __restrict__ scales8, GemvEpilogue ep) {
  dequant_skinny_resident_body<TPW, T, kW4, kEpi, MB>(wq, meta, x, K, M, N, y, out_f32, scales8, ep);
}

// the split-K forms: seven waves of TPW groups per workgroup and K-part (K = 14336: four parts of 28 groups)
template <int TPW, int T, bool kW4, int MB, int kWaves>
__global__ __launch_bounds__(kWaves * 64, 2) void dequant_skinny_resident_split_kernel(
    const u32x4_t* __restrict__ wq, const uint32_t* __restrict__ meta, const uint16_t* __restrict__ x, int K, int M, int N,
    void* __restrict__ y, int out_f32, const uint16_t* __restrict__ scales8, SkinnySplit sp) {
  dequant_skinny_resident_body<TPW, T, kW4, 0, MB, kWaves, true>(wq, meta, x, K, M, N, y, out_f32, scales8, GemvEpilogue{}, sp);
}

template <int TPW, int T, bool kW4, int kEpi, int MB, int kWaves>
__global__ __launch_bounds__(kWaves * 64, 2) void dequant_skinny_resident_split_epi_kernel(
    const u32x4_t* __restrict__ wq, const uint32_t* __restrict__ meta, const uint16_t* __restrict__ x, int K, int M, int N,
    void* __restrict__ y, int out_f32, const uint16_t* __restrict__ scales8, GemvEpilogue ep, SkinnySplit sp) {
  dequant_skinny_resident_body<TPW, T, kW4, kEpi, MB, kWaves, true>(wq, meta, x, K, M, N, y, out_f32, scales8, ep, sp);
}

}  // namespace ajq
