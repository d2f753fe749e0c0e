// Prefill dequant-GEMM on 256 x 256 tiles, for shapes with at least a few tiles per CU.
//
//   y[M, N] = x[M, K] @ W_hat[N, K]^T,  M >= 256, K % 128 == 0, W4A16 (groups of 128) or W8A16.
//
// What bounds the 256 x 128 kernels is not the matrix pipe but the one path of a CU that carries
// activations into the LDS (a 1 KiB global -> LDS request occupies it for ~17 cycles, a 1 KiB
// ds_write for ~13): a 256 x 128 tile keeps it busy three quarters of the time, and every wave that
// waits for it holds up its SIMD.  A 256 x 256 tile moves the same 32 KiB of activations per 64 k for
// twice the MFMAs.
//
// Eight waves, two per SIMD, all alike: wave (wm, wn) owns the 128 x 64 block at rows 128 wm and
// columns 64 wn (4 x 2 accumulator blocks of v_mfma_f32_32x32x16_bf16, 128 registers) and carries
// an eighth of the producers' work:
//   * two of the sixteen global -> LDS requests of a stage's activations (256 rows x 32 k);
//   * two of the sixteen private weight tiles (16 columns each): packed words come into registers
//     two or more stages ahead, are dequantized ONCE per workgroup to exact bf16 integers (q for
//     int8, q - z for int4) and written to LDS in MFMA B-fragment order.
// Scales as in the split-role 256 x 128 kernel: W8 per channel in the epilogue; W4 keeps the
// accumulators in units of the current group's scale.
//
// LDS: a ring of FOUR 32-k stages of 16 KiB activations + 16 KiB bf16 weights.  During stage j a
// wave writes its share of stage j + 3 (that buffer held stage j - 1, which every wave left behind
// at barrier j - 1) and, before barrier j, waits for its requests of stage j + 1.  Four stages
// (128 k: one int4 group, two private int8 tiles) are unrolled, so every LDS address is a constant.
#pragma once
#include <type_traits>

#include "gemm_split_kernels.h"

namespace ajq {

constexpr int kGWBM = 256, kGWBN = 256;
constexpr int kGWStageA = kGWBM * 32 * 2;                 // 16 KiB
constexpr int kGWStage = kGWStageA + kGWBN * 32 * 2;      // 32 KiB
constexpr int kGWUnitBase = 4 * kGWStage;                 // W4: two tables of 256 fp32 group units
constexpr int kGWOutStride = 528;                         // bf16 output staging: 512-byte rows, 16 bytes apart
constexpr size_t kGWLdsBytes = (size_t)kGWBM * kGWOutStride;  // 132 KiB (>= the ring and the tables)
constexpr int kGWThreads = 512;
static_assert(kGWLdsBytes >= (size_t)kGWUnitBase + 2 * 1024, "the output staging covers ring and tables");

// kGate: the weights are the w1 | w3 rows of a SwiGLU feed-forward (N = 2 F, F % 128 == 0).  A workgroup then takes
// 128 gate-projection columns and the SAME 128 up-projection columns: its 32-column blocks alternate between the two
// halves, so a wave's two accumulator blocks are a matching pair, and it writes bf16( silu(a) * u ), [M, F].
template <bool kW4, bool kGate = false>
__global__ __launch_bounds__(kGWThreads) void dequant_gemm256w_kernel(const uint16_t* __restrict__ x, int M, int K,
                                                                      const u32x4_t* __restrict__ wq,
                                                                      const uint32_t* __restrict__ meta,     // W4
                                                                      const uint16_t* __restrict__ scales8,  // W8
                                                                      int N, void* __restrict__ y, int out_f32) {
  constexpr int MT = 4;  // 32-row blocks per wave
  extern __shared__ u32x4_t smem_raw[];
  char* lds = reinterpret_cast<char*>(smem_raw);

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave >> 2, wn = wave & 3;
  const int col = lane & 31, kh = lane >> 5;

  const int tiles_m = (M + kGWBM - 1) / kGWBM;
  const int tile_m = blockIdx.x % tiles_m, tile_n = blockIdx.x / tiles_m;
  const int m0 = min(tile_m * kGWBM, M - kGWBM);
  const int n0 = tile_n * (kGate ? kGWBN / 2 : kGWBN);  // kGate: first of the workgroup's 128 columns of each half
  const int NR = K >> 7;  // rounds of four stages
  const int ntiles16 = N / kTileN;
  const int nt16_0 = n0 / kTileN;

  // ---- this wave's share of the producers' work
  // activations: request q covers rows 16 q .. 16 q + 15 (64-byte rows); chunk c of row r sits in slot c ^ ((r >> 2) & 3)
  const int row_in = lane >> 2, slot = lane & 3;
  const uint32_t a_voff = (uint32_t)row_in * (uint32_t)K * 2u + (uint32_t)((slot ^ ((row_in >> 2) & 3)) * 16);
  const char* a_base = reinterpret_cast<const char*>(x) + ((size_t)m0 + 32 * wave) * K * 2;
  auto request_a = [&](int stage_k, int buffer, int h) {  // h = 0, 1: the wave's two requests; stage_k: stage index along K
    dma16(a_base + (size_t)h * 16 * K * 2 + (size_t)stage_k * 64, a_voff, (uint32_t)(buffer * kGWStage + (2 * wave + h) * 1024));
  };
  // weights: tiles T = 2 wave + u; tile lane (nl, kc) holds 8 consecutive k of column nl starting at 8 kc of a
  // 32-k stage: lane 16 u + nl + 32 (kc & 1) of the fragment of 32-column block `wave` and k-step kc >> 1
  const int nl = lane & 15, kc = lane >> 4;
  const uint32_t lane16 = (uint32_t)lane * 16u;
  const uint32_t b_wr = (uint32_t)(kGWStageA + ((wave * 2 + (kc >> 1)) * 64 + nl + 32 * (kc & 1)) * 16);
  auto b_addr = [&](int buffer, int u) -> uint32_t { return (uint32_t)(buffer * kGWStage) + b_wr + (uint32_t)(u * 256); };
  const int tiles_k = kW4 ? NR : 2 * NR;  // private tiles of one 16-column strip
  const u32x4_t* b_src[2];
  uint32_t meta_voff[2];
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    // kGate: wave w's 32-column block is half w & 1 (gate / up), columns 32 (w >> 1) .. of the workgroup's 128
    const int T = kGate ? (wave & 1) * (ntiles16 >> 1) + nt16_0 + (wave >> 1) * 2 + u
                        : min(nt16_0 + 2 * wave + u, ntiles16 - 1);
    b_src[u] = wq + (size_t)T * tiles_k * 64;
    meta_voff[u] = (uint32_t)((T * NR * 16 + nl) * 4);
  }
  const uint32_t unit_wr = (uint32_t)(kGWUnitBase + (wave * 32 + nl) * 4);
  const W4ExactConsts wc = w4_exact_consts();
  auto minus_zero = [&](uint32_t m) -> float { return -f16_bits_to_f32(m >> 16) - 896.0f; };  // -(1024 + z)
  auto write_units = [&](uint32_t m, int u, int parity) {
    const float s = f16_bits_to_f32(m & 0xFFFFu);
    if (kc == 0) lds_write_f32(unit_wr + (uint32_t)(u * 64 + parity * 1024), s != 0.f ? s : 0x1p-60f);
  };
  // one eighth-of-a-tile piece: W8 dword pair jj of a 64-k tile, W4 dword j of a 128-k tile -> 8 bf16 of one stage
  auto piece_w8 = [&](const u32x4_t& r, int jj, int buffer, int u) {
    const u32x2_t lo = w8_to_bf16(r[2 * jj]), hi = w8_to_bf16(r[2 * jj + 1]);
    lds_write128(b_addr(buffer, u), u32x4_t{lo.x, lo.y, hi.x, hi.y});
  };
  auto piece_w4 = [&](const u32x4_t& r, int j, float mz, int buffer, int u) {
    const u32x2_t lo = w4_unpack_exact_half(r[j], 0, mz, wc), hi = w4_unpack_exact_half(r[j], 1, mz, wc);
    lds_write128(b_addr(buffer, u), u32x4_t{lo.x, lo.y, hi.x, hi.y});
  };

  // ---- this wave's share of the arithmetic
  f32x16_t acc[MT][2];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][t][r] = 0.f;
  // A fragment of k-step s, row 128 wm + 32 i + col: chunk 2 s + kh in slot (2 s + kh) ^ ((col >> 2) & 3); row
  // block i 2 KiB further.  B fragment of 32-column block 2 wn + t and k-step s: 1 KiB, lane-contiguous.
  uint32_t a_rel[2], b_rel[2];
#pragma unroll
  for (int s = 0; s < 2; ++s) a_rel[s] = (uint32_t)((wm * 128 + col) * 64 + (((2 * s + kh) ^ ((col >> 2) & 3)) << 4));
#pragma unroll
  for (int t = 0; t < 2; ++t) b_rel[t] = (uint32_t)(kGWStageA + ((2 * wn + t) * 2 * 64 + lane) * 16);
  const uint32_t unit_rd = (uint32_t)(kGWUnitBase + (wn * 64 + col) * 4);

  // ---- prologue: stages 0, 1, 2 and the packed weights the first round unpacks
  u32x4_t raw_p[2], raw_q[2];  // W8: odd / even 64-k tiles; W4: the two groups in flight
  uint32_t mw_p[2], mw_q[2];
  {
#pragma unroll
    for (int st = 0; st < 3; ++st)
#pragma unroll
      for (int h = 0; h < 2; ++h) request_a(st, st, h);
    if (kW4) {
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        load16_async(raw_p[u], b_src[u], lane16);
        load4_async(mw_p[u], meta, meta_voff[u]);
        load16_async(raw_q[u], b_src[u] + (size_t)min(1, NR - 1) * 64, lane16);
        load4_async(mw_q[u], meta + (size_t)min(1, NR - 1) * 16, meta_voff[u]);
      }
      wait_loads<0>(raw_p, mw_p);
      wait_loads<0>(raw_q, mw_q);
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const float mz = minus_zero(mw_p[u]);
#pragma unroll
        for (int j = 0; j < 3; ++j) piece_w4(raw_p[u], j, mz, j, u);
        write_units(mw_p[u], u, 0);
      }
    } else {
      u32x4_t first[2];
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        load16_async(first[u], b_src[u], lane16);
        load16_async(raw_p[u], b_src[u] + (size_t)64, lane16);                              // tile 1 (2 NR >= 2)
        load16_async(raw_q[u], b_src[u] + (size_t)min(2, 2 * NR - 1) * 64, lane16);         // tile 2
      }
      wait_loads<0>(first);
      wait_loads<0>(raw_p);
      wait_loads<0>(raw_q);
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        piece_w8(first[u], 0, 0, u);
        piece_w8(first[u], 1, 1, u);
        piece_w8(raw_p[u], 0, 2, u);
      }
    }
  }
  __syncthreads();

  u32x4_t afr[8];  // ring of A fragments, slot = position % 8 (a stage has 8 positions: 4 row blocks x 2 k-steps)
  u32x4_t bf[2][2];
#pragma unroll
  for (int p = 0; p < 4; ++p) afr[p] = lds_read128(a_rel[p & 1] + (uint32_t)((p >> 1) * 2048));
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int s = 0; s < 2; ++s) bf[t][s] = lds_read128(b_rel[t] + (uint32_t)(s * 1024));
  float cs[2], ratio[2];
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    ratio[t] = 1.0f;
    cs[t] = kW4 ? lds_read_f32(unit_rd + (uint32_t)(t * 128)) : 1.0f;
  }

  // One round = stages 4 q .. 4 q + 3.  Stage r reads buffer r, prefetches from buffer r + 1 and writes the stage
  // three ahead into buffer (r + 3) % 4.  P, Q: W8 the registers of the odd / even 64-k tile in flight, W4 of
  // the group that ends in this round / the next one (they swap from round to round).
  auto round = [&](int q, u32x4_t (&P)[2], uint32_t (&mP)[2], u32x4_t (&Q)[2], uint32_t (&mQ)[2]) {
    float mzq[2] = {0.f, 0.f};
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int cur = r, nxt = (r + 1) & 3, tgt = (r + 3) & 3;
      const int stage_k = min(4 * q + r + 3, 4 * NR - 1);  // past the end: the last stage again (fetched, not used)
#pragma unroll
      for (int p = 0; p < 8; ++p) {
        const int i = p >> 1, s = p & 1;
        // ---- producer duties, spread over the first four positions
        if (p == 0 || p == 2) request_a(stage_k, tgt, p >> 1);
        if (p == 1 || p == 3) {
          const int u = p >> 1;
          if (kW4) {
            // target stage 4 q + r + 3: r = 0 is dword 3 of group q (P); r = 1, 2, 3 are dwords 0, 1, 2 of group q + 1 (Q)
            if (r == 0) {
              piece_w4(P[u], 3, minus_zero(mP[u]), tgt, u);
            } else {
              if (r == 1 && u == 0) {
                wait_loads<13>(Q, mQ);
#pragma unroll
                for (int v = 0; v < 2; ++v) mzq[v] = minus_zero(mQ[v]);
              }
              piece_w4(Q[u], r - 1, mzq[u], tgt, u);
              if (r == 1) write_units(mQ[u], u, (q + 1) & 1);
            }
            if (r == 0 && u == 1) {  // P is free: it takes group q + 2
              const int g2 = min(q + 2, NR - 1);
#pragma unroll
              for (int v = 0; v < 2; ++v) {
                load16_async(P[v], b_src[v] + (size_t)g2 * 64, lane16);
                load4_async(mP[v], meta + (size_t)g2 * 16, meta_voff[v]);
              }
            }
          } else {
            // target stage 4 q + r + 3: r = 0 second half of tile 2 q + 1 (P); r = 1, 2 the halves of tile 2 q + 2 (Q);
            // r = 3 first half of tile 2 q + 3 (P, reloaded during r = 0)
            if (r == 1 && u == 0) wait_loads<7>(Q);
            if (r == 3 && u == 0) wait_loads<7>(P);
            if (r == 0) piece_w8(P[u], 1, tgt, u);
            if (r == 1) piece_w8(Q[u], 0, tgt, u);
            if (r == 2) piece_w8(Q[u], 1, tgt, u);
            if (r == 3) piece_w8(P[u], 0, tgt, u);
            if (r == 0 && u == 1) {
#pragma unroll
              for (int v = 0; v < 2; ++v) load16_async(P[v], b_src[v] + (size_t)min(2 * q + 3, 2 * NR - 1) * 64, lane16);
            }
            if (r == 2 && u == 1) {
#pragma unroll
              for (int v = 0; v < 2; ++v) load16_async(Q[v], b_src[v] + (size_t)min(2 * q + 4, 2 * NR - 1) * 64, lane16);
            }
          }
        }
        if (p == 4) {
          // this wave's requests of stage 4 q + r + 1 have landed; younger and still in flight: two stages of
          // requests and whatever packed words were asked for since
          if (kW4) {
            if (r <= 1) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
            else asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
          } else {
            asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
          }
          __syncthreads();
        }
        // ---- arithmetic
        const int pa = p + 4;
        afr[pa & 7] = pa < 8 ? lds_read128((uint32_t)(cur * kGWStage) + a_rel[pa & 1] + (uint32_t)((pa >> 1) * 2048))
                             : lds_read128((uint32_t)(nxt * kGWStage) + a_rel[pa & 1] + (uint32_t)(((pa - 8) >> 1) * 2048));
        if (kW4) {
          if (r == 3 && p == 0) {  // the next group's unit (past the last group nothing changes)
            const bool more = q + 1 < NR;
#pragma unroll
            for (int t = 0; t < 2; ++t) {
              const float un = more ? lds_read_f32(unit_rd + (uint32_t)(t * 128 + ((q + 1) & 1) * 1024)) : cs[t];
              ratio[t] = cs[t] / un;
              cs[t] = un;
            }
          }
          if (r == 3 && (p == 3 || p == 5 || p == 7)) {  // row blocks 0..2 move to the next group's unit
            const int ib = (p - 3) >> 1;
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
              for (int e = 0; e < 16; ++e) acc[ib][t][e] *= ratio[t];
          }
          if (r == 0 && p == 1) {  // row block 3 follows
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
              for (int e = 0; e < 16; ++e) acc[3][t][e] *= ratio[t];
          }
        }
#pragma unroll
        for (int t = 0; t < 2; ++t) acc[i][t] = mfma32(afr[p & 7], bf[t][s], acc[i][t]);
        if (p >= 6) {
          // row block 3 was the last user of this stage's k-step s: its registers take the next stage's
#pragma unroll
          for (int t = 0; t < 2; ++t) bf[t][s] = lds_read128((uint32_t)(nxt * kGWStage) + b_rel[t] + (uint32_t)(s * 1024));
        }
        if constexpr (!kW4) {
          // int8: the order a position's instructions issue in is pinned (an MFMA, a fragment read, up to six of the
          // converts in flight, the piece's write or a request; twice): left alone the compiler bunches a piece's
          // converts and then issues MFMAs back to back.  +2-5 % in a same-process comparison; the int4 form, whose
          // unpack is three times as long, measures 1-4 % slower with it and keeps the free order.
#pragma unroll
          for (int g = 0; g < 2; ++g) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                        // one MFMA
            if (g == 0 || p >= 6) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // a fragment read
            __builtin_amdgcn_sched_group_barrier(0x002, 6, 0);                        // converts in flight
            if (g == 1 && (p == 1 || p == 3)) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);  // the piece's write
            if (g == 1 && (p == 0 || p == 2)) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);  // a request
          }
          if (p == 3 || p == 7) __builtin_amdgcn_sched_barrier(0);
        } else {
          __builtin_amdgcn_sched_barrier(0x2 | 0x4);  // VALU and SALU may cross
        }
      }
    }
  };
  for (int q = 0; q < NR; q += 2) {
    round(q, raw_p, mw_p, raw_q, mw_q);
    if (q + 1 < NR) {
      if (kW4) round(q + 1, raw_q, mw_q, raw_p, mw_p);
      else round(q + 1, raw_p, mw_p, raw_q, mw_q);
    }
  }
  // The last rounds' redundant loads are still in flight, and past the loop nothing reads their destination
  // registers: unless the wait NAMES them, the compiler hands those registers to the epilogue's first values (the
  // address of the scale loads) in front of the wait, and a late load lands on top of an address.
  if (kW4) {
    wait_loads<0>(raw_p, mw_p);
    wait_loads<0>(raw_q, mw_q);
  } else {
    wait_loads<0>(raw_p);
    wait_loads<0>(raw_q);
  }
  __syncthreads();  // (also: every request into the ring has landed before the output staging overwrites it)

  // ---- epilogue
  float scale[2];
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const int n = kGate ? t * (N >> 1) + n0 + wn * 32 + col : n0 + wn * 64 + t * 32 + col;
    scale[t] = kW4 ? cs[t] : f16_bits_to_f32(scales8[min(n, N - 1)]);
  }
  if (kGate) {
    // block 0 holds the gate projection a, block 1 the up projection u of the same 32 columns: bf16( a sigmoid(a) u ),
    // staged as 256-byte rows 272 bytes apart and stored four rows per wave-wide 128-bit store
    constexpr int kGateStride = 272;
    const int F = N >> 1;
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int row = wm * 128 + i * 32 + (e & 3) + 8 * (e >> 2) + 4 * kh;
        const float a = acc[i][0][e] * scale[0], u = acc[i][1][e] * scale[1];
        *reinterpret_cast<uint16_t*>(lds + row * kGateStride + (wn * 32 + col) * 2) =
            f32_to_bf16_rne(a * (1.0f / (1.0f + expf(-a))) * u);
      }
    __syncthreads();
    const int piece = lane & 15, rsub = lane >> 4;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int row = wave * 32 + j * 4 + rsub;
      const u32x4_t v = *reinterpret_cast<const u32x4_t*>(lds + row * kGateStride + piece * 16);
      *reinterpret_cast<u32x4_t*>(reinterpret_cast<uint16_t*>(y) + (size_t)(m0 + row) * F + n0 + piece * 8) = v;
    }
    return;
  }
  if (!out_f32) {
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int row = wm * 128 + i * 32 + (e & 3) + 8 * (e >> 2) + 4 * kh;
          *reinterpret_cast<uint16_t*>(lds + row * kGWOutStride + (wn * 64 + t * 32 + col) * 2) =
              f32_to_bf16_rne(acc[i][t][e] * scale[t]);
        }
    __syncthreads();
    // a wave stores 32 rows, two 512-byte rows per wave-wide 128-bit store; columns past N are dropped
    const int piece = lane & 31, rsub = lane >> 5;
    const bool live = n0 + piece * 8 < N;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      const int row = wave * 32 + j * 2 + rsub;
      const u32x4_t v = *reinterpret_cast<const u32x4_t*>(lds + row * kGWOutStride + piece * 16);
      if (live) *reinterpret_cast<u32x4_t*>(reinterpret_cast<uint16_t*>(y) + (size_t)(m0 + row) * N + n0 + piece * 8) = v;
    }
    return;
  }
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const int n = n0 + wn * 64 + t * 32 + col;
    if (n >= N) continue;
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int m = m0 + wm * 128 + i * 32 + (e & 3) + 8 * (e >> 2) + 4 * kh;
        reinterpret_cast<float*>(y)[(size_t)m * N + n] = acc[i][t][e] * scale[t];
      }
  }
}

}  // namespace ajq
