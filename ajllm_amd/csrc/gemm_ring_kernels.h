// Prefill dequant-GEMM on 256 x 128 tiles with the tiles in a RING of four 64-k stages and a
// wave of its own for the tile loads (W8A16).
//
// Same arithmetic and output as dequant_gemm256_kernel<4, false> (4 compute waves, wave tile
// 128 x 64 on v_mfma_f32_32x32x16_bf16, int8 weights unpacked to exact bf16 integers just in
// time, the per-channel scale applied once in the epilogue); what differs is how the tiles travel.
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
  auto a_frag = [&](int stage, int p) -> u32x4_t {  // position p = 4 i + s of the sub-block in `stage`
    const int i = p >> 2, s = p & 3;
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
        const int i = p >> 2, s = p & 3;
        if (p == kPos - kAhead) {
          // the next sub-block has landed (the loader waited for it), and every wave is done with
          // the sub-block before this one
          __syncthreads();
          raw_next = read_raw((st + 1) & 3);
        }
        afr[(p + kAhead) & 7] = p + kAhead < kPos ? a_frag(st, p + kAhead) : a_frag((st + 1) & 3, p + kAhead - kPos);
        if (i == 0 && s + 1 < 4) {
#pragma unroll
          for (int t = 0; t < 2; ++t) bf[t][s + 1] = unpack(raw, t, s + 1);
        }
        if (p == kPos - 2) {
#pragma unroll
          for (int t = 0; t < 2; ++t) bf_next[t] = unpack(raw_next, t, 0);
        }
#pragma unroll
        for (int t = 0; t < 2; ++t) acc[i][t] = mfma32(afr[p & 7], bf[t][s], acc[i][t]);
        __builtin_amdgcn_sched_barrier(0x2 | 0x4);  // VALU and SALU may cross
      }
      raw = raw_next;
#pragma unroll
      for (int t = 0; t < 2; ++t) bf[t][0] = bf_next[t];
    }
  }
  __syncthreads();  // (the loader has drained its last requests)
  gemm256_store<MT, false, kGate>(acc, lds, y, out_f32, N, m0, n0, scales8, lane, wave, wm, wn, col, kh);
}

// ---- W4A16 on the same ring.
//
// A 128-k GROUP (one scale and zero point per column) spans two 64-k stages, so the double-buffered kernel's
// "sum the group apart, then acc += scale * part" cannot be carried over: the wave walks row block after
// row block inside a stage and would need a partial sum per row block.  Instead every accumulator is
// kept in UNITS OF THE CURRENT GROUP'S SCALE: at a group boundary acc *= s_old / s_new (one multiply per
// element, placed two positions behind the row block's last MFMA of the old group), the MFMAs of the new
// group then add its integer-valued products directly, and the epilogue multiplies by the last unit.  A
// zero scale (a constant-zero group) takes 2^-60 as its unit: its products then weigh 1e-18 of a unit, far
// below one ulp of anything they are added to.
//
// What travels per group (not per stage), each double-buffered by the parity of the group: the 8 private
// weight tiles (1 KiB each: 16 columns x 128 k nibbles), the 512 B of meta words and the 4 KiB of group-sum
// pieces of the 256 rows (the operand of the ninth k-step, which adds -(128 + z) * sum(x)).  The loader
// requests group g + 1 during the odd stage of group g - 1; by then the compute waves hold group g - 1's
// weights in registers and have finished its ninth step, which comes FIRST in a group's even stage (20
// positions: 4 ninth-step + 16; the odd stage has 16), so two buffers suffice.  The meta words of group
// g + 1 are read behind the barrier of group g's even stage, its weights behind that of the odd stage.
// Two groups (72 positions, a multiple of the 8 fragment slots) are unrolled: K % 256 == 0.
constexpr int kGR4BBase = 4 * kGRABytes;               // two 8 KiB weight buffers
constexpr int kGR4SideBase = kGR4BBase + 2 * 8192;     // two 4 KiB group-sum buffers
constexpr int kGR4MetaBase = kGR4SideBase + 2 * 4096;  // two 512 B meta buffers
constexpr size_t kGR4LdsBytes = kGR4MetaBase + 2 * 512;

template <bool kGate>
__global__ __launch_bounds__(kGRThreads) void dequant_gemm256r_w4_kernel(const uint16_t* __restrict__ x, int M, int K,
                                                                        const u32x4_t* __restrict__ wq,
                                                                        const uint32_t* __restrict__ meta,
                                                                        const u32x4_t* __restrict__ gs3, int N,
                                                                        void* __restrict__ y, int out_f32) {
  constexpr int MT = 4;
  constexpr int kAhead = 4;
  constexpr int kRound = 72;  // positions of two groups: 20 + 16 + 20 + 16
  extern __shared__ u32x4_t smem_raw[];
  char* lds = reinterpret_cast<char*>(smem_raw);

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);

  const int tiles_m = (M + kG2BM - 1) / kG2BM;
  const int tile_m = blockIdx.x % tiles_m, tile_n = blockIdx.x / tiles_m;
  const int m0 = min(tile_m * kG2BM, M - kG2BM);
  const int n0 = tile_n * (kGate ? kG2BN / 2 : kG2BN);
  const int NSB = K >> 6, G = K >> 7;
  const int ntiles16 = N / kTileN;
  const int nt16_0 = n0 / kTileN;
  auto col_tile = [&](int T) -> int {
    if (kGate) return ((T >> 1) & 1) * (ntiles16 >> 1) + nt16_0 + (T >> 2) * 2 + (T & 1);
    return min(nt16_0 + T, ntiles16 - 1);
  };

  if (wave == 4) {
    // ---- the loader (activations as in the W8 kernel)
    const int row_in = lane >> 3, slot = lane & 7;
    uint32_t a_voff[2];
#pragma unroll
    for (int par = 0; par < 2; ++par)
      a_voff[par] = (uint32_t)row_in * (uint32_t)K * 2u + (uint32_t)((slot ^ ((4 * par + (row_in >> 1)) & 7)) * 16);
    const char* a_base = reinterpret_cast<const char*>(x) + (size_t)m0 * K * 2;
    const uint32_t lane16 = (uint32_t)lane * 16u;
    const u32x4_t* b_src[8];
#pragma unroll
    for (int T = 0; T < 8; ++T) b_src[T] = wq + (size_t)col_tile(T) * G * 64;
    // meta words: request e covers tiles 4 e .. 4 e + 3, word (lane & 15) of tile 4 e + (lane >> 4)
    uint32_t meta_voff[2];
#pragma unroll
    for (int e = 0; e < 2; ++e) meta_voff[e] = (uint32_t)((col_tile(e * 4 + (lane >> 4)) * G * 16 + (lane & 15)) * 4);
    auto issue_a = [&](int sb, int stage) {  // 32 requests
      const char* a_sb = a_base + (size_t)sb * 128;
      const uint32_t a_to = (uint32_t)(stage * kGRABytes);
#pragma unroll
      for (int q = 0; q < 32; ++q) dma16(a_sb + (size_t)q * 8 * K * 2, a_voff[q & 1], a_to + (uint32_t)(q * 1024));
    };
    auto issue_group = [&](int g, int buf) {  // 14 requests
#pragma unroll
      for (int T = 0; T < 8; ++T) dma16(b_src[T] + (size_t)g * 64, lane16, (uint32_t)(kGR4BBase + buf * 8192 + T * 1024));
#pragma unroll
      for (int e = 0; e < 4; ++e)
        dma16(gs3 + (size_t)g * M + m0 + 64 * e, lane16, (uint32_t)(kGR4SideBase + buf * 4096 + e * 1024));
#pragma unroll
      for (int e = 0; e < 2; ++e) dma4(meta + (size_t)g * 16, meta_voff[e], (uint32_t)(kGR4MetaBase + buf * 512 + e * 256));
    };
    issue_group(0, 0);
    issue_group(1, 1);
    issue_a(0, 0);
    issue_a(1, 1);
    asm volatile("s_waitcnt vmcnt(32)" ::: "memory");  // all but stage 1 has landed
    __syncthreads();
    for (int sb = 0; sb < NSB; sb += 2) {
      // even stage: the activations of stage sb + 2
      issue_a(min(sb + 2, NSB - 1), (sb + 2) & 3);
      asm volatile("s_waitcnt vmcnt(32)" ::: "memory");  // stage sb + 1 and the next group have landed
      __syncthreads();
      // odd stage: the activations of stage sb + 3 and group sb / 2 + 2 (past the end: the last ones again)
      issue_a(min(sb + 3, NSB - 1), (sb + 3) & 3);
      issue_group(min((sb >> 1) + 2, G - 1), (sb >> 1) & 1);
      asm volatile("s_waitcnt vmcnt(46)" ::: "memory");  // stage sb + 2 has landed
      __syncthreads();
    }
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

  uint32_t a_lo[4], a_hi[4];
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    a_lo[s] = (uint32_t)((wm * 128 + col) * 128 + (((2 * s + kh) ^ ((col >> 1) & 7)) << 4));
    a_hi[s] = a_lo[s] + 2u * kGRABytes;
  }
  auto a_frag = [&](int stage, int p) -> u32x4_t {
    const int i = p >> 2, s = p & 3;
    return lds_read128((stage < 2 ? a_lo[s] : a_hi[s]) + (uint32_t)((stage & 1) * kGRABytes + i * 32 * 128));
  };
  const uint32_t g_addr = (uint32_t)(kGR4SideBase + (wm * 128 + col) * 16);
  // round position q -> stage, position inside the stage
  auto stage_of = [](int q) { return q < 20 ? 0 : q < 36 ? 1 : q < 56 ? 2 : 3; };
  auto local_of = [](int q) { return q < 20 ? q : q < 36 ? q - 20 : q < 56 ? q - 36 : q - 56; };
  auto frag = [&](int q) -> u32x4_t {  // the A-side operand of round position q (wraps into the next round)
    q %= kRound;
    const int st = stage_of(q), local = local_of(q);
    if ((st & 1) == 0) {
      if (local < 4) return lds_read128(g_addr + (uint32_t)((st >> 1) * 4096 + local * 32 * 16));
      return a_frag(st, local - 4);
    }
    return a_frag(st, local);
  };
  // weights: lane (col, kh) of 32-column block t reads the 16 bytes of tile lanes (kc = kh) and (kc = kh + 2) of
  // the private tile that holds its column: dword j of the first is k-step 2 j, of the second k-step 2 j + 1
  const int nl = col & 15;
  uint32_t b_addr[2];
#pragma unroll
  for (int t = 0; t < 2; ++t)
    b_addr[t] = (uint32_t)(kGR4BBase + (wn * 4 + 2 * t + (col >> 4)) * 1024 + (kh * 16 + nl) * 16);
  const uint32_t m_addr = (uint32_t)(kGR4MetaBase + ((wn * 4 + (col >> 4)) * 16 + nl) * 4);
  struct Raw {
    u32x4_t v[2][2];
  };
  auto read_raw = [&](int buf) -> Raw {
    Raw r;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int q = 0; q < 2; ++q) r.v[t][q] = lds_read128(b_addr[t] + (uint32_t)(buf * 8192 + q * 512));
    return r;
  };
  const W4Consts w4c = w4_consts();
  auto unpack = [&](const Raw& r, int t, int s) -> u32x4_t { return w4_unpack(r.v[t][s & 1][s >> 1], w4c); };
  // ninth-step operand: -(128 + z) against the three pieces of the group sum, lanes kh = 0 only
  auto ninth = [&](uint32_t m) -> u32x4_t {
    const uint32_t z = (m >> 19) & 0xFu;  // fp16(128 + z): z sits in mantissa bits 3..6
    const uint32_t nz = kh == 0 ? (0xC300u | z) : 0u;
    return u32x4_t{nz | (nz << 16), nz, 0u, 0u};
  };
  auto unit_of = [&](uint32_t m) -> float {
    const float s = f16_bits_to_f32(m & 0xFFFFu);
    return s != 0.f ? s : 0x1p-60f;
  };

  __syncthreads();  // stage 0 and groups 0, 1 have landed

  u32x4_t afr[8];  // ring of A-side operands, slot = round position % 8
#pragma unroll
  for (int q = 0; q < kAhead; ++q) afr[q] = frag(q);
  Raw raw = read_raw(0);
  float cs[2], ratio[2] = {1.0f, 1.0f};
  u32x4_t bf9[2], bf[2][4], bf_next[2];
  uint32_t mraw_next[2];
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const uint32_t m = lds_read32(m_addr + (uint32_t)(t * 128));
    cs[t] = unit_of(m);
    bf9[t] = ninth(m);
  }

  Raw raw_next;
  int g0 = 0;
  // one stage of a round; the stage number arrives as a type so that every trip count and address below is
  // a constant when the loop is unrolled
  auto run_stage = [&](auto stage_tag) {
    constexpr int st = decltype(stage_tag)::value;
    constexpr bool even = (st & 1) == 0;
    constexpr int npos = even ? 20 : 16, buf = st >> 1;
    constexpr int q0 = st == 0 ? 0 : st == 1 ? 20 : st == 2 ? 36 : 56;
#pragma unroll
    for (int local = 0; local < npos; ++local) {
      const int q = q0 + local;
      if (local == npos - kAhead) {
        // the next stage has landed, and every wave is done with the stage before this one
        __syncthreads();
        if (even) {
#pragma unroll
          for (int t = 0; t < 2; ++t) mraw_next[t] = lds_read32(m_addr + (uint32_t)(t * 128 + (buf ^ 1) * 512));
        } else {
          raw_next = read_raw(buf ^ 1);
        }
      }
      afr[(q + kAhead) & 7] = frag(q + kAhead);
      if (even && local < 4) {
        // ninth step of row block `local`
        if (local == 1) {  // row block 3 moves to this group's unit (its last MFMA was two positions ago)
#pragma unroll
          for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[3][t][r] *= ratio[t];
        }
        if (local == 2) {
#pragma unroll
          for (int t = 0; t < 2; ++t) bf[t][0] = unpack(raw, t, 0);
        }
#pragma unroll
        for (int t = 0; t < 2; ++t) acc[local & 3][t] = mfma32(afr[q & 7], bf9[t], acc[local & 3][t]);
      } else {
        const int p = even ? local - 4 : local;
        const int i = p >> 2, s = p & 3, s0 = even ? 0 : 4;
        if (!even && local == 0) {
          // the next group's unit; past the last group nothing changes
          const bool more = g0 + buf + 1 < G;
#pragma unroll
          for (int t = 0; t < 2; ++t) {
            const float un = more ? unit_of(mraw_next[t]) : cs[t];
            ratio[t] = cs[t] / un;  // exactly 1 past the last group
            cs[t] = un;
            bf9[t] = ninth(mraw_next[t]);
          }
        }
        if (i == 0 && s + 1 < 4) {
#pragma unroll
          for (int t = 0; t < 2; ++t) bf[t][s + 1] = unpack(raw, t, s0 + s + 1);
        }
        if (even && local == npos - 2) {
#pragma unroll
          for (int t = 0; t < 2; ++t) bf_next[t] = unpack(raw, t, 4);
        }
        if (!even && (local == 5 || local == 9 || local == 13)) {  // row blocks 0..2 move to the next unit
          const int ib = (local - 5) >> 2;
#pragma unroll
          for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[ib][t][r] *= ratio[t];
        }
#pragma unroll
        for (int t = 0; t < 2; ++t) acc[i][t] = mfma32(afr[q & 7], bf[t][s], acc[i][t]);
      }
      __builtin_amdgcn_sched_barrier(0x2 | 0x4);  // VALU and SALU may cross
    }
    if (even) {
#pragma unroll
      for (int t = 0; t < 2; ++t) bf[t][0] = bf_next[t];
    } else {
      raw = raw_next;
    }
  };
  for (; g0 < G; g0 += 2) {
    run_stage(std::integral_constant<int, 0>{});
    run_stage(std::integral_constant<int, 1>{});
    run_stage(std::integral_constant<int, 2>{});
    run_stage(std::integral_constant<int, 3>{});
  }
  // row block 3 has not been moved to the last unit: past the last group that ratio is 1
  __syncthreads();  // (the loader has drained its last requests)
  gemm256_store<MT, true, kGate>(acc, lds, y, out_f32, N, m0, n0, nullptr, lane, wave, wm, wn, col, kh, cs[0], cs[1]);
}

}  // namespace ajq
