// Prefill dequant-GEMM on 256 x 128 tiles with the work of a workgroup SPLIT BY ROLE: four waves
// that only multiply and four that only move and dequantize.
//
//   y[M, N] = x[M, K] @ W_hat[N, K]^T,  M >= 256, K % 128 == 0, W4A16 (groups of 128) or W8A16.
//
// Eight waves, two per SIMD.  Waves 0-3 (one per SIMD, wave tile 128 x 64 on
// v_mfma_f32_32x32x16_bf16) read ready bf16 fragments of BOTH operands from LDS and issue MFMAs:
// no unpack arithmetic, no zero-point step, no global load in their instruction streams.  Waves
// 4-7 (again one per SIMD) are the producers:
//   * activations go global -> LDS by DMA (global_load_lds_dwordx4), eight requests per producer
//     and 64-k stage, rows in the swizzled layout the fragment reads expect;
//   * the packed weights of the workgroup's 128 columns come into REGISTERS (two private 1 KiB
//     tiles per producer), are dequantized ONCE per workgroup to exact bf16 integers (q for int8,
//     q - z for int4: the zero-point is subtracted here, so the GEMM needs no per-row sums of the
//     activations, no extra k-step and no workspace) and are written to LDS in MFMA
//     B-fragment order, so a compute wave's B read is one conflict-free ds_read_b128 per lane.
// Scales are never folded into the bf16 operand: W8 applies the channel scale to the fp32 result,
// W4 keeps every accumulator in units of the current group's scale (acc *= s_old / s_new at a
// group boundary, one multiply per element and group) and multiplies by the last unit at the end.
//
// LDS: a ring of THREE 64-k stages, each 32 KiB of activations + 16 KiB of bf16 weights
// (144 KiB), plus two 512 B tables of group units (W4).  One workgroup barrier per stage:
//   compute waves take barrier j four positions before the end of stage j (all their reads of
//   stage j are issued by then) and prefetch stage j + 1's first fragments behind it;
//   a producer, between barriers j - 1 and j: requests the activations of stage j + 2, waits
//   until those of stage j + 1 and its packed weights of stage j + 2 have arrived, writes the
//   dequantized weights of stage j + 2, then fetches the packed weights of stage j + 3.
//   Stage (j + 2) % 3 held stage j - 1, whose reads were all issued before barrier j - 1.
#pragma once
#include <type_traits>

#include "gemm_kernels.h"

namespace ajq {

constexpr int kGSStageABytes = kG2BM * 64 * 2;              // 32 KiB: 256 rows x 64 k bf16
constexpr int kGSStageBBytes = kG2BN * 64 * 2;              // 16 KiB: 128 columns x 64 k bf16
constexpr int kGSStageBytes = kGSStageABytes + kGSStageBBytes;
constexpr int kGSStages = 3;
constexpr int kGSUnitBase = kGSStages * kGSStageBytes;      // W4: two tables of 128 fp32 group units
constexpr size_t kGSLdsBytes = kGSUnitBase + 2 * 512;
constexpr int kGSThreads = 512;

typedef __attribute__((address_space(3))) u32x4_t lds_u32x4_rw_t;
typedef __attribute__((address_space(3))) float lds_f32_rw_t;
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Wint-to-pointer-cast"
__device__ __forceinline__ void lds_write128(uint32_t address, u32x4_t v) { *(lds_u32x4_rw_t*)address = v; }
__device__ __forceinline__ void lds_write_f32(uint32_t address, float v) { *(lds_f32_rw_t*)address = v; }
__device__ __forceinline__ float lds_read_f32(uint32_t address) { return *(lds_f32_rw_t*)address; }
#pragma clang diagnostic pop

// Loads whose results the compiler must not wait for on its own: it cannot see the DMA requests
// issued between them, so its wait counts would cover those as well.  The caller waits with
// wait_loads<N>(...), which names the destination registers so that no use moves above the wait.
__device__ __forceinline__ void load16_async(u32x4_t& dst, const void* base, uint32_t voff) {
  asm volatile("global_load_dwordx4 %0, %1, %2" : "=&v"(dst) : "v"(voff), "s"(base) : "memory");
}
__device__ __forceinline__ void load4_async(uint32_t& dst, const void* base, uint32_t voff) {
  asm volatile("global_load_dword %0, %1, %2" : "=&v"(dst) : "v"(voff), "s"(base) : "memory");
}
// (one overload per register set: naming a register twice would make the compiler copy it in front of the wait)
template <int kLeft>
__device__ __forceinline__ void wait_loads(u32x4_t (&a)[2]) {
  asm volatile("s_waitcnt vmcnt(%2)" : "+v"(a[0]), "+v"(a[1]) : "n"(kLeft) : "memory");
}
template <int kLeft>
__device__ __forceinline__ void wait_loads(u32x4_t (&a)[2], uint32_t (&m)[2]) {
  asm volatile("s_waitcnt vmcnt(%4)" : "+v"(a[0]), "+v"(a[1]), "+v"(m[0]), "+v"(m[1]) : "n"(kLeft) : "memory");
}

// One private W4 dword (8 nibbles of one column, consecutive k) -> 8 bf16 holding q - z EXACTLY.
// The nibble pairs are first placed in the mantissas of two fp16 values 1024 + q (ulp 1 there), a
// mixed-precision FMA takes each half to fp32 and subtracts 1024 + z in one instruction, and the
// high halves of the fp32 results (integers of at most 5 bits) are the bf16 values.
struct W4ExactConsts {
  uint32_t mask, bias;
  float one;
};
__device__ __forceinline__ W4ExactConsts w4_exact_consts() {
  W4ExactConsts c{0x000F000Fu, 0x64006400u, 1.0f};
  asm volatile("" : "+s"(c.mask));
  asm volatile("" : "+v"(c.bias));
  asm volatile("" : "+v"(c.one));  // keeps x * 1 + c an FMA with an fp16 source (v_fma_mix_f32)
  return c;
}
// half = 0: weights 0..3 of the dword (two bf16 pairs), half = 1: weights 4..7
__device__ __forceinline__ u32x2_t w4_unpack_exact_half(uint32_t w, int half, float minus_zero_point,
                                                        const W4ExactConsts& c) {
  typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
  u32x2_t r;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const f16x2_t h = __builtin_bit_cast(f16x2_t, ((w >> (4 * (2 * half + i))) & c.mask) | c.bias);
    const float lo = __builtin_fmaf((float)h.x, c.one, minus_zero_point);
    const float hi = __builtin_fmaf((float)h.y, c.one, minus_zero_point);
    r[i] = __builtin_amdgcn_perm(__float_as_uint(hi), __float_as_uint(lo), 0x07060302u);
  }
  return r;
}

template <bool kW4, bool kGate>
__global__ __launch_bounds__(kGSThreads) void dequant_gemm256s_kernel(const uint16_t* __restrict__ x, int M, int K,
                                                                      const u32x4_t* __restrict__ wq,
                                                                      const uint32_t* __restrict__ meta,     // W4
                                                                      const uint16_t* __restrict__ scales8,  // W8
                                                                      int N, void* __restrict__ y, int out_f32) {
  constexpr int kNB = 2;       // 32-column blocks per compute wave
  constexpr int MT = 4;        // 32-row blocks per compute wave
  constexpr int kPos = 16;     // positions per stage: 4 row blocks x 4 k-steps, one A fragment and kNB MFMAs each
  constexpr int kAhead = 4;
  constexpr int kBN = 64 * kNB;  // columns of the workgroup's tile
  extern __shared__ u32x4_t smem_raw[];
  char* lds = reinterpret_cast<char*>(smem_raw);

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);

  const int tiles_m = (M + kG2BM - 1) / kG2BM;
  const int tile_m = blockIdx.x % tiles_m, tile_n = blockIdx.x / tiles_m;
  const int m0 = min(tile_m * kG2BM, M - kG2BM);
  const int n0 = tile_n * (kGate ? kBN / 2 : kBN);
  const int NSB = K >> 6;  // even: K % 128 == 0
  const int ntiles16 = N / kTileN;
  const int nt16_0 = n0 / kTileN;
  auto col_tile = [&](int T) -> int {
    if (kGate) return ((T >> 1) & 1) * (ntiles16 >> 1) + nt16_0 + (T >> 2) * 2 + (T & 1);
    return min(nt16_0 + T, ntiles16 - 1);
  };
  auto next_stage = [](uint32_t base) -> uint32_t {
    return base == (uint32_t)((kGSStages - 1) * kGSStageBytes) ? 0u : base + (uint32_t)kGSStageBytes;
  };

  if (wave >= 4) {
    // ================================ producers ================================
    const int pw = wave - 4;
    // activations: request q covers rows 8 q .. 8 q + 7 of the tile (1 KiB); chunk c of row r sits in
    // slot c ^ ((r >> 1) & 7) of its 128-byte row.  Producer pw issues q = 8 pw .. 8 pw + 7.
    const int row_in = lane >> 3, slot = lane & 7;
    uint32_t a_voff[2];
#pragma unroll
    for (int par = 0; par < 2; ++par)
      a_voff[par] = (uint32_t)row_in * (uint32_t)K * 2u + (uint32_t)((slot ^ ((4 * par + (row_in >> 1)) & 7)) * 16);
    const char* a_base = reinterpret_cast<const char*>(x) + ((size_t)m0 + 64 * pw) * K * 2;
    auto request_a = [&](const char* a_sb, uint32_t stage_base, int e) {  // request e (0..7) of this producer
      dma16(a_sb + (size_t)e * 8 * K * 2, a_voff[e & 1], stage_base + (uint32_t)((8 * pw + e) * 1024));
    };
    auto issue_a = [&](int sb, uint32_t stage_base) {
      const char* a_sb = a_base + (size_t)sb * 128;
#pragma unroll
      for (int e = 0; e < 8; ++e) request_a(a_sb, stage_base, e);
    };
    // weights: this producer owns the kNB private tiles T = kNB pw + u (16 columns each).  Tile lane (nl, kc)
    // holds, per dword (W4) or dword pair (W8), 8 consecutive k of column nl starting at 32 j + 8 kc: that is
    // lane 16 (T & 1) + nl + 32 (kc & 1) of the fragment of 32-column block T >> 1 and k-step 2 j + (kc >> 1).
    const int nl = lane & 15, kc = lane >> 4;
    const uint32_t lane16 = (uint32_t)lane * 16u;
    auto b_addr = [&](uint32_t stage_base, int u, int jj) -> uint32_t {  // jj: which k-step pair of the stage
      const int T = kNB * pw + u;
      return stage_base + (uint32_t)(kGSStageABytes + (((T >> 1) * 4 + 2 * jj + (kc >> 1)) * 64 + (T & 1) * 16 + nl + 32 * (kc & 1)) * 16);
    };
    const int tiles_k = kW4 ? (K >> 7) : NSB;  // private tiles of one 16-column strip
    const u32x4_t* b_src[kNB];
#pragma unroll
    for (int u = 0; u < kNB; ++u) b_src[u] = wq + (size_t)col_tile(kNB * pw + u) * tiles_k * 64;
    // A producer's memory instructions hold up the compute wave that shares its SIMD while they wait for the
    // CU's one path to the LDS, and four producers released by the same barrier would all queue there at once.
    // So a producer starts its stage a few cycles after its lower neighbour, and spreads its eight requests and
    // its LDS writes between the pieces of the unpacking arithmetic instead of issuing them in a burst.
    auto stagger = [&]() {
      if (pw >= 1) asm volatile("s_nop 15");
      if (pw >= 2) asm volatile("s_nop 15");
      if (pw >= 3) asm volatile("s_nop 15");
    };
    constexpr int kLoads = kNB;  // 16-byte loads of packed weights per stage (W8) or group (W4) and producer

    if (!kW4) {
      // ---- W8: a tile per stage and 16-column strip
      u32x4_t raw_a[kNB], raw_b[kNB], first[2][kNB];
      issue_a(0, 0u);
      issue_a(min(1, NSB - 1), (uint32_t)kGSStageBytes);
#pragma unroll
      for (int sb = 0; sb < 2; ++sb)
#pragma unroll
        for (int u = 0; u < kNB; ++u) load16_async(first[sb][u], b_src[u] + (size_t)min(sb, NSB - 1) * 64, lane16);
#pragma unroll
      for (int u = 0; u < kNB; ++u) load16_async(raw_a[u], b_src[u] + (size_t)min(2, NSB - 1) * 64, lane16);
      wait_loads<0>(first[0]);  // (all of them: the first stage's wait below counts requests that are not in flight yet)
      wait_loads<0>(first[1]);
      wait_loads<0>(raw_a);
#pragma unroll
      for (int sb = 0; sb < 2; ++sb)
#pragma unroll
        for (int u = 0; u < kNB; ++u)
#pragma unroll
          for (int jj = 0; jj < 2; ++jj) {
            const u32x2_t lo = w8_to_bf16(first[sb][u][2 * jj]), hi = w8_to_bf16(first[sb][u][2 * jj + 1]);
            lds_write128(b_addr((uint32_t)(sb * kGSStageBytes), u, jj), u32x4_t{lo.x, lo.y, hi.x, hi.y});
          }
      __syncthreads();
      uint32_t wr_base = (uint32_t)(2 * kGSStageBytes);  // stage of sub-block j + 2
      // one stage: `cur` holds the packed weights of sub-block j + 2, `nxt` receives those of j + 3.  In flight at its
      // start, oldest first: cur (kLoads loads), the activations of j + 1 (8 requests).
      auto stage = [&](int j, u32x4_t (&cur)[kNB], u32x4_t (&nxt)[kNB]) {
#pragma unroll
        for (int u = 0; u < kNB; ++u) load16_async(nxt[u], b_src[u] + (size_t)min(j + 3, NSB - 1) * 64, lane16);
        wait_loads<8 + kLoads>(cur);
        stagger();
        const char* a_sb = a_base + (size_t)min(j + 2, NSB - 1) * 128;
#pragma unroll
        for (int e = 0; e < 4; ++e) {  // piece e: k-step pair e & 1 of tile e >> 1
          const int u = e >> 1, jj = e & 1;
          request_a(a_sb, wr_base, 2 * e);
          const u32x2_t lo = w8_to_bf16(cur[u][2 * jj]);
          __builtin_amdgcn_sched_barrier(0);
          request_a(a_sb, wr_base, 2 * e + 1);
          const u32x2_t hi = w8_to_bf16(cur[u][2 * jj + 1]);
          __builtin_amdgcn_sched_barrier(0);
          lds_write128(b_addr(wr_base, u, jj), u32x4_t{lo.x, lo.y, hi.x, hi.y});
          __builtin_amdgcn_sched_barrier(0);
        }
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(8 + kLoads) : "memory");  // the activations of j + 1 have landed
        wr_base = next_stage(wr_base);
        __syncthreads();  // barrier j
      };
      for (int j = 0; j < NSB; j += 2) {
        stage(j, raw_a, raw_b);
        stage(j + 1, raw_b, raw_a);
      }
      wait_loads<0>(raw_a);  // (names the registers of the last, redundant loads: they stay reserved until these land)
      wait_loads<0>(raw_b);
    } else {
      // ---- W4: a tile per GROUP (two stages) and strip; dwords 0, 1 feed the even stage, 2, 3 the odd one
      const int G = K >> 7;
      const W4ExactConsts wc = w4_exact_consts();
      uint32_t meta_voff[kNB];
#pragma unroll
      for (int u = 0; u < kNB; ++u) meta_voff[u] = (uint32_t)((col_tile(kNB * pw + u) * G * 16 + nl) * 4);
      const uint32_t unit_wr = (uint32_t)(kGSUnitBase + (kNB * pw * 16 + nl) * 4);
      auto minus_zero = [&](uint32_t m) -> float {  // -(1024 + z): the meta word holds fp16(128 + z)
        return -f16_bits_to_f32(m >> 16) - 896.0f;
      };
      auto write_units = [&](uint32_t m, int u, int parity) {
        const float s = f16_bits_to_f32(m & 0xFFFFu);
        if (kc == 0) lds_write_f32(unit_wr + (uint32_t)(u * 64 + parity * 512), s != 0.f ? s : 0x1p-60f);
      };
      u32x4_t raw_a[kNB], raw_b[kNB];
      uint32_t mw_a[kNB], mw_b[kNB];
      issue_a(0, 0u);
      issue_a(1, (uint32_t)kGSStageBytes);
#pragma unroll
      for (int u = 0; u < kNB; ++u) {
        load16_async(raw_b[u], b_src[u], lane16);
        load4_async(mw_b[u], meta, meta_voff[u]);
      }
#pragma unroll
      for (int u = 0; u < kNB; ++u) {
        load16_async(raw_a[u], b_src[u] + (size_t)min(1, G - 1) * 64, lane16);
        load4_async(mw_a[u], meta + (size_t)min(1, G - 1) * 16, meta_voff[u]);
      }
      wait_loads<0>(raw_b, mw_b);  // (all of them: the first group's wait below counts requests not in flight yet)
      wait_loads<0>(raw_a, mw_a);
#pragma unroll
      for (int u = 0; u < kNB; ++u) {
        const float mz = minus_zero(mw_b[u]);
#pragma unroll
        for (int half = 0; half < 2; ++half)
#pragma unroll
          for (int jj = 0; jj < 2; ++jj) {
            const u32x2_t lo = w4_unpack_exact_half(raw_b[u][2 * half + jj], 0, mz, wc);
            const u32x2_t hi = w4_unpack_exact_half(raw_b[u][2 * half + jj], 1, mz, wc);
            lds_write128(b_addr((uint32_t)(half * kGSStageBytes), u, jj), u32x4_t{lo.x, lo.y, hi.x, hi.y});
          }
        write_units(mw_b[u], u, 0);
      }
      __syncthreads();
      uint32_t wr_base = (uint32_t)(2 * kGSStageBytes);
      // one group = stages j (even) and j + 1 (odd) of the compute waves; written here: the two stages of group g1
      // from `cur`; `nxt` receives group g1 + 1 during the odd stage.  In flight at the even stage's start, oldest
      // first: cur (2 kLoads loads), the activations of j + 1 (8 requests).
      auto group = [&](int j, u32x4_t (&cur)[kNB], uint32_t (&mcur)[kNB], u32x4_t (&nxt)[kNB], uint32_t (&mnxt)[kNB]) {
        const int g1 = (j >> 1) + 1;
        wait_loads<8>(cur, mcur);
        float mz[kNB];
#pragma unroll
        for (int u = 0; u < kNB; ++u) mz[u] = minus_zero(mcur[u]);
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          if (half == 1) {
            const int g2 = min(g1 + 1, G - 1);
#pragma unroll
            for (int u = 0; u < kNB; ++u) {
              load16_async(nxt[u], b_src[u] + (size_t)g2 * 64, lane16);
              load4_async(mnxt[u], meta + (size_t)g2 * 16, meta_voff[u]);
            }
          }
          stagger();
          const char* a_sb = a_base + (size_t)min(j + 2 + half, NSB - 1) * 128;
#pragma unroll
          for (int e = 0; e < 4; ++e) {  // piece e: dword 2 half + (e & 1) of tile e >> 1
            const int u = e >> 1, jj = e & 1;
            request_a(a_sb, wr_base, 2 * e);
            const u32x2_t lo = w4_unpack_exact_half(cur[u][2 * half + jj], 0, mz[u], wc);
            __builtin_amdgcn_sched_barrier(0);
            request_a(a_sb, wr_base, 2 * e + 1);
            const u32x2_t hi = w4_unpack_exact_half(cur[u][2 * half + jj], 1, mz[u], wc);
            __builtin_amdgcn_sched_barrier(0);
            lds_write128(b_addr(wr_base, u, jj), u32x4_t{lo.x, lo.y, hi.x, hi.y});
            __builtin_amdgcn_sched_barrier(0);
          }
          if (half == 0) {
#pragma unroll
            for (int u = 0; u < kNB; ++u) write_units(mcur[u], u, g1 & 1);
            asm volatile("s_waitcnt vmcnt(8)" ::: "memory");  // the activations of j + 1 have landed
          } else {
            // those of j + 2; the next group's loads and the requests of stage j + 3 may stay in flight
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(8 + 2 * kLoads) : "memory");
          }
          wr_base = next_stage(wr_base);
          __syncthreads();  // barrier j + half
        }
      };
      for (int j = 0; j < NSB; j += 4) {
        group(j, raw_a, mw_a, raw_b, mw_b);
        if (j + 2 < NSB) group(j + 2, raw_b, mw_b, raw_a, mw_a);
      }
      wait_loads<0>(raw_a, mw_a);  // (names the registers of the last, redundant loads)
      wait_loads<0>(raw_b, mw_b);
    }
    // the last, redundant requests and loads are drained before the output tile is staged over the stages
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (kGate || !out_f32) __syncthreads();  // the barrier inside the bf16 epilogues
    return;
  }

  // ================================ compute waves ================================
  const int wm = wave >> 1, wn = wave & 1;
  const int col = lane & 31, kh = lane >> 5;
  f32x16_t acc[MT][kNB];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int t = 0; t < kNB; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][t][r] = 0.f;

  // stage-relative read addresses.  A fragment of k-step s, row 128 wm + 32 i + col: chunk 2 s + kh in
  // slot (2 s + kh) ^ ((col >> 1) & 7), row block i 4 KiB further.  B fragment of 32-column block
  // kNB wn + t and k-step s: 1 KiB, lane-contiguous.
  uint32_t a_rel[4], b_rel[kNB];
#pragma unroll
  for (int s = 0; s < 4; ++s) a_rel[s] = (uint32_t)((wm * 128 + col) * 128 + (((2 * s + kh) ^ ((col >> 1) & 7)) << 4));
#pragma unroll
  for (int t = 0; t < kNB; ++t) b_rel[t] = (uint32_t)(kGSStageABytes + ((kNB * wn + t) * 4 * 64 + lane) * 16);
  const uint32_t unit_rd = (uint32_t)(kGSUnitBase + (wn * 32 * kNB + col) * 4);

  __syncthreads();  // stages 0 and 1 are in LDS
  __builtin_amdgcn_s_setprio(2);  // the MFMA stream goes first where it competes with the producer of its SIMD

  u32x4_t afr[8];  // ring of A fragments, slot = position % 8
  u32x4_t bf[kNB][4];
#pragma unroll
  for (int p = 0; p < kAhead; ++p) afr[p] = lds_read128(a_rel[p]);
#pragma unroll
  for (int t = 0; t < kNB; ++t)
#pragma unroll
    for (int s = 0; s < 4; ++s) bf[t][s] = lds_read128(b_rel[t] + (uint32_t)(s * 1024));
  float cs[kNB], ratio[kNB];
#pragma unroll
  for (int t = 0; t < kNB; ++t) {
    ratio[t] = 1.0f;
    cs[t] = kW4 ? lds_read_f32(unit_rd + (uint32_t)(t * 128)) : 1.0f;
  }

  uint32_t cur_base = 0u;
  const int G = K >> 7;
  int g = 0;
  // one stage; its parity inside the group arrives as a type so every trip count below is a constant
  auto run_stage = [&](auto parity_tag) {
    constexpr bool odd = decltype(parity_tag)::value != 0;
    const uint32_t nxt_base = next_stage(cur_base);
    uint32_t a_cur[4], a_nxt[4], b_nxt[kNB];
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      a_cur[s] = a_rel[s] + cur_base;
      a_nxt[s] = a_rel[s] + nxt_base;
    }
#pragma unroll
    for (int t = 0; t < kNB; ++t) b_nxt[t] = b_rel[t] + nxt_base;
#pragma unroll
    for (int p = 0; p < kPos; ++p) {
      const int i = p >> 2, s = p & 3;
      if (p == kPos - kAhead) __syncthreads();  // the next stage is complete; every wave is done with the one before this
      const int pa = p + kAhead;
      afr[pa & 7] = pa < kPos ? lds_read128(a_cur[pa & 3] + (uint32_t)((pa >> 2) * 4096)) : lds_read128(a_nxt[pa & 3]);
      if (kW4) {
        if (odd && p == 0) {
          // the next group's unit (past the last group nothing changes)
          const bool more = g + 1 < G;
#pragma unroll
          for (int t = 0; t < kNB; ++t) {
            const float un = more ? lds_read_f32(unit_rd + (uint32_t)(t * 128 + ((g + 1) & 1) * 512)) : cs[t];
            ratio[t] = cs[t] / un;
            cs[t] = un;
          }
        }
        if (odd && (p == 5 || p == 9 || p == 13)) {  // row blocks 0..2 move to the next group's unit
          const int ib = (p - 5) >> 2;
#pragma unroll
          for (int t = 0; t < kNB; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[ib][t][r] *= ratio[t];
        }
        if (!odd && p == 1) {  // row block 3 follows (its last MFMA of the old group was two positions ago)
#pragma unroll
          for (int t = 0; t < kNB; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[3][t][r] *= ratio[t];
        }
      }
#pragma unroll
      for (int t = 0; t < kNB; ++t) acc[i][t] = mfma32(afr[p & 7], bf[t][s], acc[i][t]);
      if (p >= kPos - kAhead) {
        // row block 3 was the last user of this stage's k-step s: its registers take the next stage's
#pragma unroll
        for (int t = 0; t < kNB; ++t) bf[t][s] = lds_read128(b_nxt[t] + (uint32_t)(s * 1024));
      }
      __builtin_amdgcn_sched_barrier(0x2 | 0x4);  // VALU and SALU may cross
    }
    cur_base = nxt_base;
  };
  for (int sb = 0; sb < NSB; sb += 2) {
    run_stage(std::integral_constant<int, 0>{});
    run_stage(std::integral_constant<int, 1>{});
    ++g;
  }
  __builtin_amdgcn_s_setprio(0);
  __syncthreads();  // (the producers have drained their last requests)
  gemm256_store<MT, kW4, kGate>(acc, lds, y, out_f32, N, m0, n0, scales8, lane, wave, wm, wn, col, kh, cs[0], cs[1]);
}

}  // namespace ajq
