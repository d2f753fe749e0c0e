// Shared device helpers for the gfx950 quantized-linear kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include "../../include/ajq.h"

namespace ajq {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

constexpr int kGroup = 128;      // int4 quantization group along K
constexpr int kTileN = 16;       // rows of one private-layout tile
constexpr int kW8TileK = 64;     // k extent of one private W8 tile

// D[16x16] += A[16x32] * B[32x16], bf16 in, fp32 accumulate.
// lane l supplies A[row l%16][k 8*(l/16)..+8) and B[k 8*(l/16)..+8)][col l%16];
// it receives D[row 4*(l/16)+i][col l%16] in component i.
__device__ __forceinline__ f32x4_t mfma16(u32x4_t a, u32x4_t b, f32x4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                 __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}

// One private W4 dword (8 nibbles, weight e in nibble (e>>1)+4*(e&1)) -> 8 bf16
// holding 128+q exactly: 0x4300 is bf16(128) and its ulp is 1.
__device__ __forceinline__ u32x4_t w4_to_bf16_biased(uint32_t w) {
  u32x4_t r;
  r.x = (w & 0x000F000Fu) | 0x43004300u;
  r.y = ((w >> 4) & 0x000F000Fu) | 0x43004300u;
  r.z = ((w >> 8) & 0x000F000Fu) | 0x43004300u;
  r.w = ((w >> 12) & 0x000F000Fu) | 0x43004300u;
  return r;
}

// The constants of the W4 unpack as run-time values, the nibble mask in an SGPR and the bf16 bias
// (128.0 twice) in a VGPR: a VOP3 instruction takes no literal on this target, so from
// (w & mask) | bias the compiler forms one v_and_or_b32 only if both already sit in registers
// (with literals it emits an AND and an OR).  The asm statements are empty: they hide the values
// from constant folding and contain no instruction.
struct W4Consts {
  uint32_t mask, bias;
};
__device__ __forceinline__ W4Consts w4_consts() {
  W4Consts c{0x000F000Fu, 0x43004300u};
  asm volatile("" : "+s"(c.mask));
  asm volatile("" : "+v"(c.bias));
  return c;
}

// private W4 dword -> 8 bf16 holding 128+q (see w4_to_bf16_biased): 3 shifts + 4 v_and_or_b32.
// Plain C on purpose: the compiler pads the wait states between an MFMA and a VALU instruction
// that touches its registers only for instructions it can see, not for the text of an asm.
__device__ __forceinline__ u32x4_t w4_unpack(uint32_t w, W4Consts c) {
  u32x4_t r;
  r.x = (w & c.mask) | c.bias;
  r.y = ((w >> 4) & c.mask) | c.bias;
  r.z = ((w >> 8) & c.mask) | c.bias;
  r.w = ((w >> 12) & c.mask) | c.bias;
  return r;
}

// Four int8 (one dword, k order) -> two dwords of bf16 pairs, exact: the compiler turns each
// sign-extending byte extract + convert into one v_cvt_f32_i32 with an SDWA byte select, and one
// v_perm_b32 per pair takes the high halves.  |q| <= 127 has at most 7 significant bits, so the
// high half of the fp32 IS the bf16.
__device__ __forceinline__ u32x2_t w8_to_bf16(uint32_t w) {
  const float f0 = (float)(int)(int8_t)(w);
  const float f1 = (float)(int)(int8_t)(w >> 8);
  const float f2 = (float)(int)(int8_t)(w >> 16);
  const float f3 = (float)((int)w >> 24);
  u32x2_t r;
  r.x = __builtin_amdgcn_perm(__float_as_uint(f1), __float_as_uint(f0), 0x07060302u);
  r.y = __builtin_amdgcn_perm(__float_as_uint(f3), __float_as_uint(f2), 0x07060302u);
  return r;
}

__device__ __forceinline__ float f16_bits_to_f32(uint32_t bits16) {
  return __half2float(__ushort_as_half((unsigned short)bits16));
}

// fp32 -> bf16 bits, round to nearest even (one v_cvt_pk_bf16_f32; NaN stays NaN).
__device__ __forceinline__ uint16_t f32_to_bf16_rne(float f) {
  return __builtin_bit_cast(uint16_t, static_cast<__bf16>(f));
}

// two fp32 -> one dword holding two bf16 (lo in bits 0..15), round to nearest even: a single
// v_cvt_pk_bf16_f32
__device__ __forceinline__ uint32_t pack2_bf16(float lo, float hi) {
  typedef float f32x2_t __attribute__((ext_vector_type(2)));
  typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_t{lo, hi}, bf16x2_t));
}

// Sum over the 16 lanes of a team, result in every lane: four adds whose second operand comes
// through the DPP row rotate (a "row" is 16 lanes), no LDS crossbar round trips.
template <int kRor>
__device__ __forceinline__ float row_ror(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x120 + kRor, 0xF, 0xF, false));
}
// a / b, correctly rounded, for many a over one b: with y the correctly rounded 1 / b (one IEEE division per b),
// q0 = a * y is within an ulp of the quotient, the FMA r = a - q0 * b is exact, and q0 + r * y rounds to the correctly
// rounded a / b (Markstein's theorem).  Three instructions per quotient instead of the ten of the division expansion;
// bit for bit a / b on normal operands (checked on 10^9 random pairs on the GPU; a zero numerator may come out with
// the other sign).
struct Divisor {
  float b, y;
  __device__ __forceinline__ explicit Divisor(float b_) : b(b_), y(1.0f / b_) {}
  __device__ __forceinline__ float divide(float a) const {
    const float q0 = a * y;
    const float r = __builtin_fmaf(-q0, b, a);
    return __builtin_fmaf(r, y, q0);
  }
};
__device__ __forceinline__ float team_sum16(float v) {
  v += row_ror<8>(v);
  v += row_ror<4>(v);
  v += row_ror<2>(v);
  v += row_ror<1>(v);
  return v;
}

}  // namespace ajq
