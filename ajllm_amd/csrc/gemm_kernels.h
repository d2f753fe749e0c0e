// What the tile GEMM kernels share: the MFMA wrapper, LDS access by byte address, the global -> LDS DMA
// request, the per-row group sums of the 128 x 128 W4 kernel, and the epilogue of the 256 x 128 tiles.
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

}  // namespace ajq
