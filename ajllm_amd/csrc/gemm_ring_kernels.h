// Prefill dequant-GEMM on 256 x 128 tiles with the tiles in a RING of four 64-k stages and a
// wave of its own for the tile loads (W8A16).
//
// Four compute waves (wave tile 128 x 64 on v_mfma_f32_32x32x16_bf16) unpack the int8 weights of their own
// columns to exact bf16 integers just in time; the per-channel scale is applied once in the epilogue.
//
// Why a loader wave.  A global -> LDS request (global_load_lds_dwordx4, 1 KiB) occupies the CU's
// vector memory path for about 13 cycles, and the wave that issues it cannot issue anything else
// until the path has taken it: a lone wave issues one every 17.5 cycles, four waves issuing
// together see 52 cycles each.  A 64-k sub-block needs 40 of them per workgroup.  Issued by the
// compute waves (one per position, between their MFMAs) they cost 28 % of the kernel: the same
// loop without them runs 1224 instead of 882 TFLOP/s at M = 2048, N = K = 4096.  A fifth wave
// that does nothing else takes the requests off the MFMA waves' instruction streams; it shares a
// SIMD with one compute wave, whose MFMAs issue while the loader waits for the memory path.
// (Five waves need every wave within 256 registers, accumulators included.)
//
//  * A stage holds 64 k of the workgroup's tile: 256 rows x 128 B of activations (32 KiB) and
//    the 8 private weight tiles of its 128 columns (8 KiB).  Four stages, 160 KiB.
//  * ONE barrier per sub-block.  The compute waves take it four positions before the sub-block's
//    end (a position = one A fragment and two MFMAs): by then a wave has issued every LDS read
//    of the sub-block (fragments are requested four positions ahead), and behind the barrier it
//    fetches the next sub-block's first fragments and packed weights while its last MFMAs of
//    this one run, so the MFMA stream does not stop at a block boundary.  The loader takes the
//    same barrier after it has issued the requests for sub-block j + 2 and waited for its
//    requests of sub-block j + 1 (vmcnt(40): the 40 just issued may stay in flight).
//    - Read after write: sub-block j + 1 has landed before any wave passes the barrier of j.
//    - Write after read: stage (j + 2) % 4 held sub-block j - 2; every compute wave has consumed
//      its reads of j - 2 before it arrives at the barrier of j - 1, which the loader passes
//      before it issues anything for j + 2.
//  * The four sub-blocks of a round are unrolled in the compute waves, so every LDS address is a
//    per-lane register plus an immediate (K must be a multiple of 256).
#pragma once
#include <type_traits>

#include "gemm_kernels.h"

namespace ajq {

constexpr int kGRSub = 64;                              // k per stage
constexpr int kGRABytes = kG2BM * kGRSub * 2;           // 32 KiB of activations per stage
constexpr int kGRBBytes = (kG2BN / kTileN) * 1024;      // 8 KiB: 8 private W8 tiles (16 columns x 64 k)
constexpr int kGRBBase = 4 * kGRABytes;                 // the weight ring sits behind the activation ring
constexpr size_t kGRLdsBytes = 4 * (kGRABytes + kGRBBytes);  // 160 KiB
constexpr int kGRThreads = 320;                         // four compute waves and the loader

template <bool kGate>
__global__ __launch_bounds__(kGRThreads) void dequant_gemm256r_w8_kernel(const uint16_t* __restrict__ x, int M, int K,
                                                                        const u32x4_t* __restrict__ wq,
                                                                        const uint16_t* __restrict__ scales8, int N,
                                                                        void* __restrict__ y, int out_f32) {
  constexpr int MT = 4;       // 32-row blocks per compute wave
  constexpr int kPos = 16;    // positions per sub-block: 4 row blocks x 4 k-steps
  constexpr int kAhead = 4;   // A fragments are requested this many positions ahead
  extern __shared__ u32x4_t smem_raw[];
  char* lds = reinterpret_cast<char*>(smem_raw);

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);

  const int tiles_m = (M + kG2BM - 1) / kG2BM;
  const int tile_m = blockIdx.x % tiles_m, tile_n = blockIdx.x / tiles_m;
  const int m0 = min(tile_m * kG2BM, M - kG2BM);
  const int n0 = tile_n * (kGate ? kG2BN / 2 : kG2BN);
  const int NSB = K >> 6;
  const int ntiles16 = N / kTileN;
  const int nt16_0 = n0 / kTileN;
  auto col_tile = [&](int T) -> int {
    if (kGate) return ((T >> 1) & 1) * (ntiles16 >> 1) + nt16_0 + (T >> 2) * 2 + (T & 1);
    return min(nt16_0 + T, ntiles16 - 1);
  };

  if (wave == 4) {
    // ---- the loader.  Activations: a wave-wide request fills 1 KiB = 8 rows of 128 B.  Chunk c of
    // row r sits in slot c ^ ((r >> 1) & 7): rows are 128 B, so even and odd rows fall in different
    // bank halves and the 8 rows of either parity among 16 consecutive ones must take 8 different
    // slots.  For request q (rows 8 q ..), ((r >> 1) & 7) = (4 q + (lane / 8 >> 1)) & 7: two
    // patterns, by the parity of q.  Weights: a private tile is 1 KiB contiguous.
    const int row_in = lane >> 3, slot = lane & 7;
    uint32_t a_voff[2];
#pragma unroll
    for (int par = 0; par < 2; ++par)
      a_voff[par] = (uint32_t)row_in * (uint32_t)K * 2u + (uint32_t)((slot ^ ((4 * par + (row_in >> 1)) & 7)) * 16);
    const char* a_base = reinterpret_cast<const char*>(x) + (size_t)m0 * K * 2;
    const uint32_t lane16 = (uint32_t)lane * 16u;
    const u32x4_t* b_src[8];
#pragma unroll
    for (int T = 0; T < 8; ++T) b_src[T] = wq + (size_t)col_tile(T) * NSB * 64;
    auto issue_all = [&](int sb, int stage) {  // the 40 requests of sub-block sb into `stage`
      const char* a_sb = a_base + (size_t)sb * 128;
      const uint32_t a_to = (uint32_t)(stage * kGRABytes), b_to = (uint32_t)(kGRBBase + stage * kGRBBytes);
#pragma unroll
      for (int q = 0; q < 32; ++q) dma16(a_sb + (size_t)q * 8 * K * 2, a_voff[q & 1], a_to + (uint32_t)(q * 1024));
#pragma unroll
      for (int T = 0; T < 8; ++T) dma16(b_src[T] + (size_t)sb * 64, lane16, b_to + (uint32_t)(T * 1024));
    };
    issue_all(0, 0);
    issue_all(min(1, NSB - 1), 1);
    asm volatile("s_waitcnt vmcnt(40)" ::: "memory");  // sub-block 0 has landed
    __syncthreads();
    for (int sb = 0; sb < NSB; ++sb) {
      issue_all(min(sb + 2, NSB - 1), (sb + 2) & 3);     // past the end: the last one again (fetched, not used)
      asm volatile("s_waitcnt vmcnt(40)" ::: "memory");  // sub-block sb + 1 has landed
      __syncthreads();                                   // the compute waves' barrier of sub-block sb
    }
    // the last, redundant requests are drained before the output tile is staged over the stages
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (kGate || !out_f32) __syncthreads();  // the barrier inside the bf16 epilogues
    return;
  }

  // ---- compute waves
  const int wm = wave >> 1, wn = wave & 1;
  const int col = lane & 31, kh = lane >> 5;
  f32x16_t acc[MT][2];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][t][r] = 0.f;

  // LDS read addresses.  A fragment of k-step s, row r = 128 wm + 32 i + col: chunk 2 s + kh in
  // slot (2 s + kh) ^ ((col >> 1) & 7); stages 0, 1 are reached from a_lo, stages 2, 3 from a_hi
  // (an LDS instruction's immediate offset is 16 bits).
  uint32_t a_lo[4], a_hi[4];
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    a_lo[s] = (uint32_t)((wm * 128 + col) * 128 + (((2 * s + kh) ^ ((col >> 1) & 7)) << 4));
    a_hi[s] = a_lo[s] + 2u * kGRABytes;
  }
  auto a_frag = [&](int stage, int p) -> u32x4_t {  // position p = 4 s + i of the sub-block in `stage`
    const int i = p & 3, s = p >> 2;
    return lds_read128((stage < 2 ? a_lo[s] : a_hi[s]) + (uint32_t)((stage & 1) * kGRABytes + i * 32 * 128));
  };
  // weights: lane (col, kh) of 32-column block t reads, from the private tile that holds its column,
  // the 16 bytes of tile lanes (kc = kh) and (kc = kh + 2): dword pair j of piece h is k-step 2 j + h
  const int nl = col & 15;
  uint32_t b_addr[2];
#pragma unroll
  for (int t = 0; t < 2; ++t)
    b_addr[t] = (uint32_t)(kGRBBase + (wn * 4 + 2 * t + (col >> 4)) * 1024 + (kh * 16 + nl) * 16);
  struct Raw {
    u32x4_t v[2][2];
  };
  auto read_raw = [&](int stage) -> Raw {
    Raw r;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int h = 0; h < 2; ++h) r.v[t][h] = lds_read128(b_addr[t] + (uint32_t)(stage * kGRBBytes + h * 512));
    return r;
  };
  auto unpack = [&](const Raw& r, int t, int s) -> u32x4_t {
    const int j = s >> 1, h = s & 1;
    const u32x2_t lo = w8_to_bf16(r.v[t][h][2 * j]);
    const u32x2_t hi = w8_to_bf16(r.v[t][h][2 * j + 1]);
    return u32x4_t{lo.x, lo.y, hi.x, hi.y};
  };

  __syncthreads();  // sub-block 0 has landed

  u32x4_t afr[8];  // ring of fragments, slot = position % 8
#pragma unroll
  for (int p = 0; p < kAhead; ++p) afr[p] = a_frag(0, p);
  Raw raw = read_raw(0);
  u32x4_t bf[2][4];
#pragma unroll
  for (int t = 0; t < 2; ++t) bf[t][0] = unpack(raw, t, 0);

  for (int sb0 = 0; sb0 < NSB; sb0 += 4) {
#pragma unroll
    for (int st = 0; st < 4; ++st) {  // the sub-block in stage st
      Raw raw_next;
      u32x4_t bf_next[2];
#pragma unroll
      for (int p = 0; p < kPos; ++p) {
        // k-step-major order (position p = 4 s + i): the B fragments of k-step s + 1 are first used four positions
        // on, so their unpacking spreads over two positions, one column block each, and the order the instructions of
        // a position issue in is pinned (an MFMA, a fragment read, up to six converts, an MFMA, up to six converts).
        // A compute wave has its SIMD to itself: converts bunched between two MFMAs (the row-block-major order unpacked
        // both column blocks of a k-step in one position) stall the matrix pipe for their whole issue time.
        // Same results bit for bit; +2-3.5 % over the row-block-major order in a same-process comparison (M = 2048,
        // N = K = 4096: 1067 -> 1102 TFLOP/s); three, nine or twelve converts per group measure no better than none.
        const int i = p & 3, s = p >> 2;
        if (p == kPos - kAhead) {
          // the next sub-block has landed (the loader waited for it), and every wave is done with
          // the sub-block before this one
          __builtin_amdgcn_sched_barrier(0);
          __syncthreads();
          raw_next = read_raw((st + 1) & 3);
        }
        afr[(p + kAhead) & 7] = p + kAhead < kPos ? a_frag(st, p + kAhead) : a_frag((st + 1) & 3, p + kAhead - kPos);
        if (i < 2 && s + 1 < 4) bf[i][s + 1] = unpack(raw, i, s + 1);
        if (p >= kPos - 2) bf_next[p - (kPos - 2)] = unpack(raw_next, p - (kPos - 2), 0);  // the next sub-block's first ones
#pragma unroll
        for (int t = 0; t < 2; ++t) acc[i][t] = mfma32(afr[p & 7], bf[t][s], acc[i][t]);
#pragma unroll
        for (int g = 0; g < 2; ++g) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          if (g == 0) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x002, 6, 0);
        }
        if (i == 3) __builtin_amdgcn_sched_barrier(0);
      }
      raw = raw_next;
#pragma unroll
      for (int t = 0; t < 2; ++t) bf[t][0] = bf_next[t];
    }
  }
  __syncthreads();  // (the loader has drained its last requests)
  gemm256_store<MT, false, kGate>(acc, lds, y, out_f32, N, m0, n0, scales8, lane, wave, wm, wn, col, kh);
}

}  // namespace ajq
