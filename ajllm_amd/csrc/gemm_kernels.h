// Prefill dequant-GEMM, M >= 256:  y[M, N] = x[M, K] @ W_hat[N, K]^T on bf16 MFMA.
//
// 256 x 128 output tile per workgroup on v_mfma_f32_32x32x16_bf16, K walked in blocks
// of 128 (one int4 quantization group); 8 waves with 64 x 64 wave tiles (W4) or 4 waves
// with 128 x 64 wave tiles and the accumulators in AGPRs (W8).
//
//  * Activations go global -> LDS directly (global_load_lds_dwordx4, no register
//    staging).  One k-block of the tile is 256 rows x 256 B, exactly 64 KiB, rows
//    unpadded; the 16-byte chunk c of row r sits in slot c ^ (r & 15) of its row,
//    so the 32 rows of an A fragment read fall in distinct banks.  A wave-wide
//    load fills 1 KiB of LDS (4 rows) from 4 row segments of 256 B.  Two k-blocks
//    are resident: the next one's loads are issued one at a time between the MFMAs
//    of the current one.
//  * Weights: the packed private tiles (and the W4 meta words) of the workgroup's 128
//    columns also go global -> LDS, once per workgroup; a wave reads the raw words of
//    its own columns and unpacks them just in time, under the MFMAs, into B fragments
//    that hold EXACT small integers (128+q for int4, q for int8).  Scales stay in fp32
//    and are applied to fp32 partial sums (per group for W4, once per channel for W8),
//    so no weight is ever rounded.
//  * W4 zero-point: the per-row group sums of the activations, split into three bf16
//    pieces by group_sum3_kernel, ride in a 4 KiB side buffer; a ninth MFMA k-step per
//    group multiplies them by -(128+z) (exact in bf16), so the fp32 partial sum of
//    a group already is  sum_k a[m,k] * (q[n,k] - z[n,g]),  and what is left for
//    the VALU is one FMA per accumulator element and group (acc += s * part).
//  * A wave walks its 32-row blocks in turn: A fragments are requested from LDS
//    four MFMA pairs ahead and each feeds the two 32-column blocks of the wave.  The
//    loop body is one basic block (no branch between MFMAs).
//  * The last row tile is shifted up to end at row M (M >= 256), so no row is
//    clamped or masked; rows it shares with its neighbour are computed twice
//    with identical results.
//  * bf16 output leaves through LDS in whole 256-byte rows.
#pragma once
#include "ajq_common.h"

namespace ajq {

// gs3[g][m] = 16 bytes: bf16 pieces h, m, l with h + m + l == the sum of the 128
// activations of group g in row m to fp32 precision, then five zeros.
// A 16-lane team sums four consecutive groups of one row (four 128-bit loads in
// flight per lane); K / 128 must be a multiple of 4 or the tail teams clamp.
__global__ __launch_bounds__(256) void group_sum3_kernel(const uint16_t* __restrict__ x, int M, int K,
                                                         u32x4_t* __restrict__ gs3) {
  const int G = K >> 7;
  const int G4 = (G + 3) >> 2;
  const long long team = (long long)blockIdx.x * 16 + (threadIdx.x >> 4);
  if (team >= (long long)M * G4) return;
  const int sub = threadIdx.x & 15;
  const int m = (int)(team / G4), g0 = (int)(team % G4) * 4;
  u32x4_t v[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int g = min(g0 + u, G - 1);
    v[u] = *reinterpret_cast<const u32x4_t*>(x + (size_t)m * K + g * kGroup + sub * 8);
  }
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      s += __uint_as_float(v[u][i] << 16);
      s += __uint_as_float(v[u][i] & 0xFFFF0000u);
    }
#pragma unroll
    for (int off = 8; off > 0; off >>= 1) s += __shfl_xor(s, off);
    if (sub == u && g0 + u < G) {
      // truncation keeps every remainder exactly representable
      const uint32_t hb = __float_as_uint(s) & 0xFFFF0000u;
      const float r1 = s - __uint_as_float(hb);
      const uint32_t mb = __float_as_uint(r1) & 0xFFFF0000u;
      const float r2 = r1 - __uint_as_float(mb);
      const uint32_t lb = (uint32_t)f32_to_bf16_rne(r2);
      gs3[(size_t)(g0 + u) * M + m] = u32x4_t{(hb >> 16) | mb, lb, 0u, 0u};
    }
  }
}

__device__ __forceinline__ f32x16_t mfma32(u32x4_t a, u32x4_t b, f32x16_t c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                 __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}

typedef __attribute__((address_space(3))) void lds_void_t;
// LDS reads by byte address.  The tile kernels declare no static LDS, so their dynamic LDS starts
// at address 0 (the DMA destinations below are absolute addresses too); a read through
// "pointer to the dynamic array + offset" costs a VALU add of that zero per read.
typedef __attribute__((address_space(3))) const u32x4_t lds_u32x4_t;
typedef __attribute__((address_space(3))) const uint32_t lds_u32_t;
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Wint-to-pointer-cast"  // the host pass sees 64-bit pointers
__device__ __forceinline__ u32x4_t lds_read128(uint32_t address) { return *(lds_u32x4_t*)address; }
__device__ __forceinline__ uint32_t lds_read32(uint32_t address) { return *(lds_u32_t*)address; }
#pragma clang diagnostic pop
typedef __attribute__((address_space(1))) const void global_void_t;

// One wave-wide global -> LDS load of 16 bytes per lane: lane l reads base + voff(l) and
// the 1 KiB lands at LDS byte address lds_addr + 16 l.  The address is given as a scalar
// base plus a 32-bit per-lane offset so that no 64-bit vector arithmetic is spent on it
// (the builtin form makes the compiler keep and increment 64-bit VGPR pointers).  The
// loads are not known to the compiler's wait-count bookkeeping: callers wait for them
// with an explicit s_waitcnt vmcnt before a barrier.
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"  // m0 is named as clobbered on purpose
__device__ __forceinline__ void dma16(const void* base, uint32_t voff, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_addr), "v"(voff), "s"(base)
               : "memory", "m0");
}
__device__ __forceinline__ void dma4(const void* base, uint32_t voff, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2"
               :
               : "s"(lds_addr), "v"(voff), "s"(base)
               : "memory", "m0");
}
#pragma clang diagnostic pop

constexpr int kG2BM = 256, kG2BN = 128;
constexpr int kG2TileBytes = kG2BM * 256;  // 64 KiB: one k-block of activations
// LDS map (bytes).  Buffers of a pair differ in one address bit, so one XOR flips a
// read offset from one to the other.
//   [0, 128 Ki)            two activation tiles
//   W4: [128 Ki, 136 Ki)   two 4 KiB side buffers (group-sum pieces)
//       136 Ki, 152 Ki     two 8 KiB weight buffers (8 private tiles each)
//       144 Ki, +512       two 512 B meta buffers
//   W8: 128 Ki, 144 Ki     two 16 KiB weight buffers (16 private tiles each)
constexpr int kG2SideBase = 2 * kG2TileBytes, kG2SideBytes = 4096;
constexpr int kG2W4Base = kG2SideBase + 2 * kG2SideBytes, kG2MetaBase = kG2W4Base + 8192;
constexpr int kG2W8Base = 2 * kG2TileBytes;
constexpr int kG2WStride = 16384, kG2MetaStride = 512;
constexpr size_t kG2LdsBytes = 160 * 1024;

// Epilogue of the 256 x 128 tile kernels.  Accumulator register r of lane (col, kh) is row
// (r & 3) + 8 * (r >> 2) + 4 * kh of its 32 x 32 block.  bf16 output: the tile is laid out row-major
// in LDS (from address 0: the caller guarantees that every wave is done with the tile buffers and that
// no request into them is in flight) and leaves in whole 256-byte rows, four rows per wave-wide
// 128-bit store; 2-byte stores straight from the accumulators took 2-3 times as long.
template <int MT, bool kW4, bool kGate>
__device__ __forceinline__ void gemm256_store(f32x16_t (&acc)[MT][2], char* lds, void* __restrict__ y, int out_f32, int N,
                                              int m0, int n0, const uint16_t* __restrict__ scales8, int lane, int wave,
                                              int wm, int wn, int col, int kh, float unit0 = 1.0f,
                                              float unit1 = 1.0f) {
  constexpr int kWaves = 16 / MT;
  constexpr int kWaveRows = 32 * MT;
  constexpr int kLoadRows = kG2BM / kWaves;
  // Rows are 272 bytes apart so the two half-waves of a write (rows 4 apart) use different banks.
  constexpr int kOutStride = 272;
  // column of the weight tensor behind the wave's 32-column block t
  auto column = [&](int t) -> int {
    if (kGate) return t * (N >> 1) + n0 + wn * 32 + col;
    return n0 + wn * 64 + t * 32 + col;
  };
  float cs[2] = {unit0, unit1};  // W4: what the caller's accumulators are in units of (1 if already scaled)
  if (!kW4) {
#pragma unroll
    for (int t = 0; t < 2; ++t) cs[t] = f16_bits_to_f32(scales8[min(column(t), N - 1)]);
  }
  if (kGate) {
    // block 0 holds the gate projection a, block 1 the up projection u of the same columns:
    // out = bf16( a * sigmoid(a) * u ), [M, N / 2], staged like the plain bf16 tile (64 columns:
    // 128-byte rows 144 bytes apart) and stored eight rows per wave-wide 128-bit store
    constexpr int kGateStride = 144;
    const int F = N >> 1;
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = wm * kWaveRows + i * 32 + (r & 3) + 8 * (r >> 2) + 4 * kh;
        const float a = acc[i][0][r] * cs[0], u = acc[i][1][r] * cs[1];
        *reinterpret_cast<uint16_t*>(lds + row * kGateStride + (wn * 32 + col) * 2) =
            f32_to_bf16_rne(a * (1.0f / (1.0f + expf(-a))) * u);
      }
    __syncthreads();
    const int piece = lane & 7, rsub = lane >> 3;
#pragma unroll
    for (int j = 0; j < kLoadRows / 8; ++j) {
      const int row = wave * kLoadRows + j * 8 + rsub;
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
        for (int r = 0; r < 16; ++r) {
          const int row = wm * kWaveRows + i * 32 + (r & 3) + 8 * (r >> 2) + 4 * kh;
          *reinterpret_cast<uint16_t*>(lds + row * kOutStride + (wn * 64 + t * 32 + col) * 2) =
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
  for (int t = 0; t < 2; ++t) {
    const int n = column(t);
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

// MT = 32-row blocks per wave: 4 -> 4 waves (2 x 2, wave tile 128 x 64), 2 -> 8 waves
// (4 x 2, wave tile 64 x 64, two waves per SIMD).
// kGate: the weights are the w1 | w3 rows of a SwiGLU feed-forward (N = 2 F, F % 64 == 0).  A
// workgroup then takes 64 gate-projection columns and the SAME 64 up-projection columns (its
// eight private tiles come from two places: 32-column blocks alternate between the halves, so a
// wave's two blocks are a matching pair) and writes bf16( silu(a) * u ), [M, F]: the 4-byte
// intermediate [M, 2 F] never exists.
template <int MT, bool kW4, bool kGate = false>
__global__ __launch_bounds__(1024 / MT) void dequant_gemm256_kernel(
    const uint16_t* __restrict__ x, int M, int K, const u32x4_t* __restrict__ wq,
    const uint32_t* __restrict__ meta,     // W4: private meta; W8: unused
    const uint16_t* __restrict__ scales8,  // W8: fp16 [N]; W4: unused
    const u32x4_t* __restrict__ gs3,       // W4: [K/128][M] group-sum pieces; W8: unused
    int N, void* __restrict__ y, int out_f32) {
  constexpr int kSteps = kW4 ? 9 : 8;         // MFMA k-steps per 128-k block
  constexpr int kWaves = 16 / MT;             // 4 or 8
  constexpr int kWaveRows = 32 * MT;          // rows of the tile one wave computes
  constexpr int kLoadRows = kG2BM / kWaves;   // rows of the tile one wave loads
  constexpr int kBTiles = kW4 ? 8 : 16;       // 1 KiB private weight tiles per k-block and workgroup
  constexpr int kWBase = kW4 ? kG2W4Base : kG2W8Base;

  extern __shared__ u32x4_t smem_raw[];
  char* lds = reinterpret_cast<char*>(smem_raw);

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int col = lane & 31, kh = lane >> 5;

  // column-major walk over output tiles: consecutive workgroups share a column block of W
  const int tiles_m = (M + kG2BM - 1) / kG2BM;
  const int tile_m = blockIdx.x % tiles_m, tile_n = blockIdx.x / tiles_m;
  const int m0 = min(tile_m * kG2BM, M - kG2BM);
  const int n0 = tile_n * (kGate ? kG2BN / 2 : kG2BN);  // kGate: first of the workgroup's 64 columns of each half
  const int G = K >> 7;
  const int ntiles16 = N / kTileN;

  // ---- global -> LDS, one k-block ahead, no registers in between.
  // Activations: wave w fills kLoadRows rows with wave-wide loads of 4 rows each.  Chunk c
  // of row r lives in slot c ^ (r & 15) of its row (the LDS serves 16 lanes of a 128-bit
  // read per clock from 64 banks: 16 consecutive rows must fall in 16 different slots);
  // lane (row_in, slot) of load q therefore fetches chunk slot ^ ((4q + row_in) & 15),
  // which depends on q only through q & 3.
  const int row_in = lane >> 4, slot = lane & 15;
  uint32_t a_voff[4];
#pragma unroll
  for (int v = 0; v < 4; ++v)
    a_voff[v] = (uint32_t)row_in * (uint32_t)K * 2u + (uint32_t)((slot ^ (4 * v + row_in)) * 16);
  const char* a_base = reinterpret_cast<const char*>(x) + (size_t)(m0 + kLoadRows * wave) * K * 2;
  const int nt16_0 = n0 / kTileN;
  // the workgroup's T-th private 16-column tile (T = 0 .. 7) in the weight tensor; tiles past the
  // matrix repeat the last one (their columns are never stored)
  auto col_tile = [&](int T) -> int {
    if (kGate) return ((T >> 1) & 1) * (ntiles16 >> 1) + nt16_0 + (T >> 2) * 2 + (T & 1);
    return min(nt16_0 + T, ntiles16 - 1);
  };
  // The loads of one k-block are numbered 0 .. kLoads - 1 so that the main loop can issue
  // them one at a time between its MFMAs.
  constexpr int kALoads = kLoadRows / 4;
  constexpr int kBLoads = kBTiles / kWaves;
  constexpr int kLoads = kALoads + kBLoads + (kW4 ? 2 : 0);
  const uint32_t lane16 = (uint32_t)lane * 16u;
  // meta words of tile (wave & 1) * 4 + (lane >> 4) of the workgroup's eight, word (lane & 15);
  // tiles past the matrix repeat the last one (their columns are never stored)
  const uint32_t meta_voff =
      (uint32_t)((col_tile((wave & 1) * 4 + (lane >> 4)) * G * 16 + (lane & 15)) * 4);
  auto issue_load = [&](int j, int kb, int buf) {
    if (j < kALoads) {
      const char* src = a_base + (size_t)kb * 256 + (size_t)j * 4 * K * 2;
      dma16(src, a_voff[j & 3], (uint32_t)(buf * kG2TileBytes + wave * (kLoadRows * 256) + j * 1024));
    } else if (j < kALoads + kBLoads) {
      // weights: a private tile is 1 KiB contiguous, one wave-wide load each
      const int T = wave * kBLoads + (j - kALoads);
      const u32x4_t* tile;
      if (kW4)
        tile = wq + ((size_t)col_tile(T) * G + kb) * 64;
      else
        tile = wq + ((size_t)col_tile(T >> 1) * (2 * G) + 2 * kb + (T & 1)) * 64;
      dma16(tile, lane16, (uint32_t)(kWBase + buf * kG2WStride + T * 1024));
    } else if (j == kALoads + kBLoads) {
      // group-sum pieces of 64 rows; with eight waves the upper four repeat the lower four
      // (same bytes to the same place) rather than branch
      const int e = wave & 3;
      dma16(gs3 + (size_t)kb * M + m0 + 64 * e, lane16, (uint32_t)(kG2SideBase + buf * kG2SideBytes + e * 1024));
    } else {
      // meta words, 4 tiles per load; odd and even waves take one half each
      const int e = wave & 1;
      dma4(meta + (size_t)kb * 16, meta_voff, (uint32_t)(kG2MetaBase + buf * kG2MetaStride + e * 256));
    }
  };

  f32x16_t acc[MT][2];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][t][r] = 0.f;

  // ---- LDS read offsets.  A fragment of k-step s, row r = kWaveRows wm + 32 i + col: chunk
  // 2s + kh sits in slot (2s + kh) ^ (col & 15) = ((s ^ (col >> 1 & 7)) << 1) | (kh ^ (col & 1)).
  uint32_t a_off[8];
#pragma unroll
  for (int v = 0; v < 8; ++v)
    a_off[v] = (uint32_t)((wm * kWaveRows + col) * 256 + (((v ^ ((col >> 1) & 7)) << 5) | ((kh ^ (col & 1)) << 4)));
  uint32_t g_off = (uint32_t)(kG2SideBase + (wm * kWaveRows + col) * 16);
  // weights: lane (col, kh) of 32-column block t reads, from the 16-row private tile that
  // holds its column, the 16 bytes of tile lanes (kc = kh) and (kc = kh + 2): dword j of the
  // first is k-step 2j, of the second k-step 2j + 1.
  const int c16 = wn * 4 + (col >> 4), nl = col & 15;
  uint32_t b_off = (uint32_t)(kWBase + (kW4 ? c16 : 2 * c16) * 1024 + (kh * 16 + nl) * 16);
  uint32_t m_off = (uint32_t)(kG2MetaBase + (c16 * 16 + nl) * 4);

#pragma unroll
  for (int j = 0; j < kLoads; ++j) issue_load(j, 0, 0);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  const W4Consts w4c = w4_consts();

  for (int kb = 0; kb < G; ++kb) {
    // Loads are issued unconditionally (the last block is simply fetched again): a branch
    // between the MFMAs would cut the loop body into separately scheduled pieces (results are
    // the same either way; the parity tests pass with the branch too).
    const int kb_next = min(kb + 1, G - 1);

    // ---- this block's packed weights, LDS -> registers (W8: the second 64-k tile is
    // fetched a few steps later, shortly before it is unpacked)
    u32x4_t raw[2][kW4 ? 2 : 4];
    uint32_t mraw[2];
    auto read_raw = [&](int first, int count) {
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const int tb = t * (kW4 ? 2048 : 4096);
#pragma unroll
        for (int q = first; q < first + count; ++q)
          raw[t][q] = lds_read128(b_off + tb + q * 512);
      }
    };
    read_raw(0, 2);
    if (kW4) {
#pragma unroll
      for (int t = 0; t < 2; ++t) mraw[t] = lds_read32(m_off + t * 128);
    }

    // ---- B fragments.  They are unpacked one k-step ahead of their first use, inside the
    // wave's first 32-row block, so the unpacking (VALU) runs under the MFMAs.
    u32x4_t bf[2][kSteps];
    float sc[2];
    auto unpack_step = [&](int s) {
#pragma unroll
      for (int t = 0; t < 2; ++t) {
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

    // ---- MFMA loop, software-pipelined by hand: the A fragment of position p + kAhead is
    // requested before the two MFMAs of position p are issued (position = 32-row block x
    // k-step), and the order of LDS reads and MFMAs is pinned; VALU work may move freely.
    constexpr int kPos = MT * kSteps;
#ifndef AJQ_AHEAD
#define AJQ_AHEAD 4
#endif
    constexpr int kAhead = AJQ_AHEAD;
    auto a_frag = [&](int p) -> u32x4_t {
      const int i = p / kSteps, s = p % kSteps;
      return lds_read128(s < 8 ? a_off[s & 7] + i * 32 * 256 : g_off + i * 32 * 16);
    };
    u32x4_t afr[kAhead + 1];
#pragma unroll
    for (int p = 0; p < kAhead; ++p) afr[p] = a_frag(p);
    unpack_step(0);
    f32x16_t part[2];
#pragma unroll
    for (int p = 0; p < kPos; ++p) {
      const int i = p / kSteps, s = p % kSteps;
      if (p + kAhead < kPos) afr[(p + kAhead) % (kAhead + 1)] = a_frag(p + kAhead);
      if (i == 0 && s + 1 < kSteps) unpack_step(s + 1);
      if (p < kLoads) issue_load(p, kb_next, (kb + 1) & 1);  // one load per position
      if (kW4) {
        if (s == 0) {
#pragma unroll
          for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) part[t][r] = 0.f;
        }
#pragma unroll
        for (int t = 0; t < 2; ++t) part[t] = mfma32(afr[p % (kAhead + 1)], bf[t][s], part[t]);
        if (s == kSteps - 1) {
#pragma unroll
          for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][t][r] += sc[t] * part[t][r];
        }
      } else {
#pragma unroll
        for (int t = 0; t < 2; ++t) acc[i][t] = mfma32(afr[p % (kAhead + 1)], bf[t][s], acc[i][t]);
      }
      __builtin_amdgcn_sched_barrier(0x2 | 0x4);  // VALU and SALU may cross
    }
    // flip every read offset to the other buffer
#pragma unroll
    for (int v = 0; v < 8; ++v) a_off[v] ^= (uint32_t)kG2TileBytes;
    g_off ^= (uint32_t)kG2SideBytes;
    b_off ^= (uint32_t)kG2WStride;
    m_off ^= (uint32_t)kG2MetaStride;
    // the next block's tiles must have landed and every wave must be done with this one
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
  }

  gemm256_store<MT, kW4, kGate>(acc, lds, y, out_f32, N, m0, n0, scales8, lane, wave, wm, wn, col, kh);
}

}  // namespace ajq
