// Prefill dequant-GEMM on 128 x 128 output tiles, for shapes that leave the 256 x 128 kernel
// short of workgroups (M between 128 and about 1500 on N = 4096: 32 ... 192 big tiles for 256
// CUs).
//
// Everything enters LDS by DMA (activations, the packed private weight tiles of the workgroup's columns, the W4
// meta words); a wave unpacks the weights of its own columns just in time to exact integers in bf16 (128 + q for
// int4, q for int8) for v_mfma_f32_32x32x16_bf16; scales stay fp32 (per group for W4: acc += s * part, once per
// channel for W8).  The W4 zero-point is a ninth k-step per group: -(128 + z) against the three bf16 pieces of the
// activations' per-row group sums (group_sum3_kernel, a launch of its own in front of this one).  Eight waves as
// 2 x 4 with 64 x 32 wave tiles, K walked in blocks of 128.  What differs: a workgroup has a CU
// to itself, and a k-block is 36 MFMAs per SIMD, about half a microsecond: less than a trip to
// memory.  So the tiles travel in a ring of THREE buffers and
// are requested two k-blocks ahead; at the end of a block a wave waits only for the loads it
// issued one block earlier (s_waitcnt vmcnt(loads per block)).
#pragma once
#include "gemm_kernels.h"

namespace ajq {

constexpr int kG1BM = 128, kG1BN = 128;
constexpr int kG1Ring = 3;
constexpr int kG1TileBytes = kG1BM * 256;  // 32 KiB: one k-block of activations
// LDS map (bytes): three activation tiles, three weight slots (W4 8 KiB, W8 16 KiB), W4 only:
// three 2 KiB group-sum slots and three 512 B meta slots
constexpr int kG1WBase = kG1Ring * kG1TileBytes;
constexpr int kG1W4Slot = 8192, kG1W8Slot = 16384;
constexpr int kG1SideBase = kG1WBase + kG1Ring * kG1W4Slot, kG1SideSlot = 2048;
constexpr int kG1MetaBase = kG1SideBase + kG1Ring * kG1SideSlot, kG1MetaSlot = 512;
constexpr size_t kG1LdsBytesW4 = kG1MetaBase + kG1Ring * kG1MetaSlot;  // 127.5 KiB
constexpr size_t kG1LdsBytesW8 = kG1WBase + kG1Ring * kG1W8Slot;       // 144 KiB

// kWN = waves along N: 2 -> four waves with 64 x 64 wave tiles, 4 -> eight waves with 64 x 32
// wave tiles (two waves per SIMD: each fetches twice the activation fragments per MFMA, but the
// SIMD always has a second instruction stream to issue from).
// kGate (kWN = 4 only): w1 | w3 weights of a SwiGLU feed-forward, output bf16( silu(a) * u ),
// [M, N / 2]; the workgroup's four 32-column blocks alternate between the two halves as in
// the 256 x 128 kernels, here one block per wave, so the pairs meet in an fp32 staging tile.
template <bool kW4, int kWN, bool kGate = false>
__global__ __launch_bounds__(128 * kWN) void dequant_gemm128_kernel(
    const uint16_t* __restrict__ x, int M, int K, const u32x4_t* __restrict__ wq,
    const uint32_t* __restrict__ meta,     // W4: private meta; W8: unused
    const uint16_t* __restrict__ scales8,  // W8: fp16 [N]; W4: unused
    const u32x4_t* __restrict__ gs3,       // W4: [K/128][M] group-sum pieces; W8: unused
    int N, void* __restrict__ y, int out_f32) {
  constexpr int MT = 2;
  constexpr int kSteps = kW4 ? 9 : 8;  // MFMA k-steps per 128-k block
  constexpr int kWaves = 2 * kWN;
  constexpr int TB = 4 / kWN;          // 32-column blocks per wave
  constexpr int kWaveRows = 32 * MT;   // rows of the tile one wave computes
  constexpr int kLoadRows = kG1BM / kWaves;  // rows of the tile one wave loads
  constexpr int kBTiles = kW4 ? 8 : 16;  // 1 KiB private weight tiles per k-block and workgroup
  constexpr int kWSlot = kW4 ? kG1W4Slot : kG1W8Slot;

  extern __shared__ u32x4_t smem_raw[];
  char* lds = reinterpret_cast<char*>(smem_raw);

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave / kWN, wn = wave % kWN;
  const int col = lane & 31, kh = lane >> 5;

  // column-major walk over output tiles: consecutive workgroups share a column block of W
  const int tiles_m = (M + kG1BM - 1) / kG1BM;
  const int tile_m = blockIdx.x % tiles_m, tile_n = blockIdx.x / tiles_m;
  static_assert(!kGate || kWN == 4, "the gate epilogue pairs the blocks of waves 2 j and 2 j + 1");
  const int m0 = min(tile_m * kG1BM, M - kG1BM);  // M >= 128: the last row tile is shifted up
  const int n0 = tile_n * (kGate ? kG1BN / 2 : kG1BN);  // kGate: first of the workgroup's 64 columns of each half
  const int G = K >> 7;
  const int ntiles16 = N / kTileN;

  // ---- global -> LDS.  Activations: wave w fills kLoadRows rows (128 / waves) with wave-wide
  // loads of 4 rows (wave w: rows kLoadRows w ...); chunk c of row r lives in slot c ^ (r & 15) of its row.  Every wave issues
  // the same number of loads per k-block (the count the end-of-block wait relies on): where a
  // piece needs fewer loads than there are waves, two waves fetch the same bytes to the same place.
  const int row_in = lane >> 4, slot16 = lane & 15;
  uint32_t a_voff[4];
#pragma unroll
  for (int v = 0; v < 4; ++v)
    a_voff[v] = (uint32_t)row_in * (uint32_t)K * 2u + (uint32_t)((slot16 ^ (4 * v + row_in)) * 16);
  const char* a_base = reinterpret_cast<const char*>(x) + (size_t)(m0 + kLoadRows * wave) * K * 2;
  const int nt16_0 = n0 / kTileN;
  // the workgroup's T-th private 16-column tile (T = 0 .. 7) in the weight tensor; tiles past the
  // matrix repeat the last one (their columns are never stored)
  auto col_tile = [&](int T) -> int {
    if (kGate) return ((T >> 1) & 1) * (ntiles16 >> 1) + nt16_0 + (T >> 2) * 2 + (T & 1);
    return min(nt16_0 + T, ntiles16 - 1);
  };
  constexpr int kALoads = kLoadRows / 4;
  constexpr int kBLoads = kBTiles / kWaves;
  constexpr int kLoads = kALoads + kBLoads + (kW4 ? 2 : 0);
  const uint32_t lane16 = (uint32_t)lane * 16u;
  const uint32_t meta_voff =
      (uint32_t)((col_tile((wave & 1) * 4 + (lane >> 4)) * G * 16 + (lane & 15)) * 4);
  auto issue_load = [&](int j, int kb, int ring) {
    if (j < kALoads) {
      const char* src = a_base + (size_t)kb * 256 + (size_t)j * 4 * K * 2;
      dma16(src, a_voff[j & 3], (uint32_t)(ring * kG1TileBytes + wave * (kLoadRows * 256) + j * 1024));
    } else if (j < kALoads + kBLoads) {
      const int T = wave * kBLoads + (j - kALoads);
      const u32x4_t* tile;
      if (kW4)
        tile = wq + ((size_t)col_tile(T) * G + kb) * 64;
      else
        tile = wq + ((size_t)col_tile(T >> 1) * (2 * G) + 2 * kb + (T & 1)) * 64;
      dma16(tile, lane16, (uint32_t)(kG1WBase + ring * kWSlot + T * 1024));
    } else if (j == kALoads + kBLoads) {
      const int e = wave & 1;  // group-sum pieces of 64 rows
      dma16(gs3 + (size_t)kb * M + m0 + 64 * e, lane16, (uint32_t)(kG1SideBase + ring * kG1SideSlot + e * 1024));
    } else {
      const int e = wave & 1;  // meta words, 4 tiles per load
      dma4(meta + (size_t)kb * 16, meta_voff, (uint32_t)(kG1MetaBase + ring * kG1MetaSlot + e * 256));
    }
  };

  f32x16_t acc[MT][TB];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int t = 0; t < TB; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][t][r] = 0.f;

  // ---- LDS read offsets of ring slot 0 (advanced by one slot per k-block).  A fragment of
  // k-step s, row r = 64 wm + 32 i + col: chunk 2s + kh sits in slot (2s + kh) ^ (col & 15).
  uint32_t a_off[8];
#pragma unroll
  for (int v = 0; v < 8; ++v)
    a_off[v] = (uint32_t)((wm * kWaveRows + col) * 256 + (((v ^ ((col >> 1) & 7)) << 5) | ((kh ^ (col & 1)) << 4)));
  uint32_t g_off = (uint32_t)(kG1SideBase + (wm * kWaveRows + col) * 16);
  const int c16 = wn * (2 * TB) + (col >> 4), nl = col & 15;
  uint32_t b_off = (uint32_t)(kG1WBase + (kW4 ? c16 : 2 * c16) * 1024 + (kh * 16 + nl) * 16);
  uint32_t m_off = (uint32_t)(kG1MetaBase + (c16 * 16 + nl) * 4);

  // blocks 0 and 1 are requested up front; block 0 has landed when at most one block's loads are out
#pragma unroll
  for (int j = 0; j < kLoads; ++j) issue_load(j, 0, 0);
#pragma unroll
  for (int j = 0; j < kLoads; ++j) issue_load(j, min(1, G - 1), 1);
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kLoads) : "memory");
  __syncthreads();

  const W4Consts w4c = w4_consts();

  int ring = 0;  // slot of the current block
  for (int kb = 0; kb < G; ++kb) {
    // Loads are issued unconditionally (past the end the last block is simply fetched again): a
    // branch between the MFMAs would cut the loop body into separately scheduled pieces.
    const int kb_load = min(kb + 2, G - 1);
    const int ring_load = ring == 0 ? 2 : ring - 1;  // (ring + 2) % 3: the slot read one block ago

    u32x4_t raw[TB][kW4 ? 2 : 4];
    uint32_t mraw[TB];
    auto read_raw = [&](int first, int count) {
#pragma unroll
      for (int t = 0; t < TB; ++t) {
        const int tb = t * (kW4 ? 2048 : 4096);
#pragma unroll
        for (int q = first; q < first + count; ++q)
          raw[t][q] = lds_read128(b_off + tb + q * 512);
      }
    };
    read_raw(0, 2);
    if (kW4) {
#pragma unroll
      for (int t = 0; t < TB; ++t) mraw[t] = lds_read32(m_off + t * 128);
    }

    // ---- B fragments, unpacked one k-step ahead of their first use inside the wave's first
    // 32-row block, so the unpacking (VALU) runs under the MFMAs
    u32x4_t bf[TB][kSteps];
    float sc[TB];
    auto unpack_step = [&](int s) {
#pragma unroll
      for (int t = 0; t < TB; ++t) {
        if (kW4) {
          if (s < 8) {
            bf[t][s] = w4_unpack(raw[t][s & 1][s >> 1], w4c);
          } else {
            // ninth step: -(128 + z) against the three pieces of the group sum (lanes kh = 0 only)
            const uint32_t z = (mraw[t] >> 19) & 0xFu;  // fp16(128 + z): z sits in mantissa bits 3..6
            const uint32_t nz = kh == 0 ? (0xC300u | z) : 0u;
            bf[t][8] = u32x4_t{nz | (nz << 16), nz, 0u, 0u};
            sc[t] = f16_bits_to_f32(mraw[t] & 0xFFFFu);
          }
        } else {
          // W8 tile tau (64 k), piece h (kc = kh + 2h): dwords (2j, 2j+1) are k-step 4 tau + 2j + h
          if (s == 2 && t == 0) read_raw(2, 2);
          const int tau = s >> 2, j = (s >> 1) & 1, h = s & 1;
          const u32x2_t lo = w8_to_bf16(raw[t][2 * tau + h][2 * j]);
          const u32x2_t hi = w8_to_bf16(raw[t][2 * tau + h][2 * j + 1]);
          bf[t][s] = u32x4_t{lo.x, lo.y, hi.x, hi.y};
        }
      }
    };

    // ---- MFMA loop: the A fragment of position p + kAhead is requested before the two MFMAs
    // of position p (position = 32-row block x k-step); the order of LDS reads and MFMAs is
    // pinned, VALU work may move freely.
    constexpr int kPos = MT * kSteps;
    constexpr int kAhead = 4;
    static_assert(kLoads <= kPos, "one load per position");
    auto a_frag = [&](int p) -> u32x4_t {
      const int i = p / kSteps, s = p % kSteps;
      return lds_read128(s < 8 ? a_off[s & 7] + i * 32 * 256 : g_off + i * 32 * 16);
    };
    u32x4_t afr[kAhead + 1];
#pragma unroll
    for (int p = 0; p < kAhead; ++p) afr[p] = a_frag(p);
    unpack_step(0);
    f32x16_t part[TB];
#pragma unroll
    for (int p = 0; p < kPos; ++p) {
      const int i = p / kSteps, s = p % kSteps;
      if (p + kAhead < kPos) afr[(p + kAhead) % (kAhead + 1)] = a_frag(p + kAhead);
      if (i == 0 && s + 1 < kSteps) unpack_step(s + 1);
      if (p < kLoads) issue_load(p, kb_load, ring_load);  // one load per position
      if (kW4) {
        if (s == 0) {
#pragma unroll
          for (int t = 0; t < TB; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) part[t][r] = 0.f;
        }
#pragma unroll
        for (int t = 0; t < TB; ++t) part[t] = mfma32(afr[p % (kAhead + 1)], bf[t][s], part[t]);
        if (s == kSteps - 1) {
#pragma unroll
          for (int t = 0; t < TB; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][t][r] += sc[t] * part[t][r];
        }
      } else {
#pragma unroll
        for (int t = 0; t < TB; ++t) acc[i][t] = mfma32(afr[p % (kAhead + 1)], bf[t][s], acc[i][t]);
      }
      __builtin_amdgcn_sched_barrier(0x2 | 0x4);  // VALU and SALU may cross
    }
    // every read offset moves on one slot of the ring
    const bool wrap = ring == kG1Ring - 1;
    ring = wrap ? 0 : ring + 1;
    const uint32_t da = wrap ? (uint32_t)(-(kG1Ring - 1) * kG1TileBytes) : (uint32_t)kG1TileBytes;
    const uint32_t dw = wrap ? (uint32_t)(-(kG1Ring - 1) * kWSlot) : (uint32_t)kWSlot;
#pragma unroll
    for (int v = 0; v < 8; ++v) a_off[v] += da;
    b_off += dw;
    if (kW4) {
      g_off += wrap ? (uint32_t)(-(kG1Ring - 1) * kG1SideSlot) : (uint32_t)kG1SideSlot;
      m_off += wrap ? (uint32_t)(-(kG1Ring - 1) * kG1MetaSlot) : (uint32_t)kG1MetaSlot;
    }
    // the next block's tiles (requested one block ago) must have landed; this block's requests
    // stay in flight.  Every wave must be done with this block before its slot is refilled.
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kLoads) : "memory");
    __syncthreads();
  }
  // the redundant requests of the last blocks must not land on the output tile staged below
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  // ---- epilogue: accumulator register r of lane (col, kh) is row (r & 3) + 8 * (r >> 2) + 4 * kh.
  // bf16 output is laid out row-major in LDS (the activation slots are free: every wave has
  // passed the barrier above) and leaves in whole 256-byte rows, four rows per wave-wide
  // 128-bit store.  Rows are 272 bytes apart so the two half-waves of a write (rows 4 apart)
  // use different banks.
  constexpr int kOutStride = 272;
  // column of the weight tensor behind the wave's 32-column block t
  auto column = [&](int t) -> int {
    if (kGate) return (wn & 1) * (N >> 1) + n0 + (wn >> 1) * 32 + col;
    return n0 + wn * (32 * TB) + t * 32 + col;
  };
  float cs[TB];
#pragma unroll
  for (int t = 0; t < TB; ++t) cs[t] = kW4 ? 1.0f : f16_bits_to_f32(scales8[min(column(t), N - 1)]);
  if (kGate) {
    // fp32 staging, 128 x 128 (rows 528 bytes apart): wave (wm, wn) writes its block at columns
    // 32 wn; then a lane forms eight outputs of one row from a (block 2 j) and u (block 2 j + 1)
    // and stores 16 bytes: out = bf16( a * sigmoid(a) * u ), [M, N / 2]
    constexpr int kGateStride = 528;
    const int F = N >> 1;
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = wm * kWaveRows + i * 32 + (r & 3) + 8 * (r >> 2) + 4 * kh;
        *reinterpret_cast<float*>(lds + row * kGateStride + (wn * 32 + col) * 4) = acc[i][0][r] * cs[0];
      }
    __syncthreads();
    const int piece = lane & 7, rsub = lane >> 3;  // eight 8-column pieces per row of 64 outputs
    const int block = (piece >> 2) * 64 + (piece & 3) * 8;  // staging column of the piece's first a
#pragma unroll
    for (int j = 0; j < kLoadRows / 8; ++j) {
      const int row = wave * kLoadRows + j * 8 + rsub;
      const float* src = reinterpret_cast<const float*>(lds + row * kGateStride) + block;
      const f32x4_t a0 = *reinterpret_cast<const f32x4_t*>(src), a1 = *reinterpret_cast<const f32x4_t*>(src + 4);
      const f32x4_t u0 = *reinterpret_cast<const f32x4_t*>(src + 32), u1 = *reinterpret_cast<const f32x4_t*>(src + 36);
      float g[8];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        g[e] = a0[e] * (1.0f / (1.0f + expf(-a0[e]))) * u0[e];
        g[4 + e] = a1[e] * (1.0f / (1.0f + expf(-a1[e]))) * u1[e];
      }
      *reinterpret_cast<u32x4_t*>(reinterpret_cast<uint16_t*>(y) + (size_t)(m0 + row) * F + n0 + piece * 8) =
          u32x4_t{pack2_bf16(g[0], g[1]), pack2_bf16(g[2], g[3]), pack2_bf16(g[4], g[5]), pack2_bf16(g[6], g[7])};
    }
    return;
  }
  if (!out_f32) {
#pragma unroll
    for (int t = 0; t < TB; ++t)
#pragma unroll
      for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int row = wm * kWaveRows + i * 32 + (r & 3) + 8 * (r >> 2) + 4 * kh;
          *reinterpret_cast<uint16_t*>(lds + row * kOutStride + (wn * (32 * TB) + t * 32 + col) * 2) =
              f32_to_bf16_rne(acc[i][t][r] * cs[t]);
        }
    __syncthreads();
    // lane -> (row within a group of 4, 16-byte piece of the 256-byte row); columns past N are dropped
    const int piece = lane & 15, rsub = lane >> 4;
    const bool live = n0 + piece * 8 < N;
#pragma unroll
    for (int j = 0; j < kLoadRows / 4; ++j) {
      const int row = wave * kLoadRows + j * 4 + rsub;
      const u32x4_t v = *reinterpret_cast<const u32x4_t*>(lds + row * kOutStride + piece * 16);
      if (live)
        *reinterpret_cast<u32x4_t*>(reinterpret_cast<uint16_t*>(y) + (size_t)(m0 + row) * N + n0 + piece * 8) = v;
    }
    return;
  }
#pragma unroll
  for (int t = 0; t < TB; ++t) {
    const int n = n0 + wn * (32 * TB) + t * 32 + col;
    if (n >= N) continue;
#pragma unroll
    for (int i = 0; i < MT; ++i) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm * kWaveRows + i * 32 + (r & 3) + 8 * (r >> 2) + 4 * kh;
        reinterpret_cast<float*>(y)[(size_t)m * N + n] = acc[i][t][r] * cs[t];
      }
    }
  }
}

}  // namespace ajq
