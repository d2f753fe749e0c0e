// Causal self-attention for a block of T new positions (prefill), head_dim 128, on bf16 MFMA
// with an online softmax: the T x (start + T) score matrix is never materialised.
//
//   out[b, t, h, :] = softmax_j( q[b, h, t, :] . k[b, hk, j, :] / sqrt(128) ) v[b, hk, j, :],
//   j <= start + t,   hk = h / (H / Hkv)
//
// q is fp32 [B, H, T, 128] (already rotated); keys and values are read where the model keeps
// them, in the caches [B, Hkv, max_len, 128] (fp32 or bf16), rows 0 .. start + T - 1; out is
// fp32 [B, T, H * 128], the layout the output projection takes.
//
// A workgroup of 4 waves owns 64 query rows of one (b, h), a wave 16 of them, and walks the
// keys in blocks of 32.  Both products run transposed so that no operand changes layout
// between them:
//   S^T = K Q^T :  A = 16 keys x 32 dims from LDS (rows padded by 16 B), B = the wave's Q
//                  fragments (registers, bf16, pre-scaled by log2(e) / sqrt(128));
//                  lane (g = l / 16, r = l % 16) receives keys 4g..4g+3 of query row r;
//   O^T += V^T P^T: the lane's 8 probabilities of a 32-key block ARE its B fragment
//                  (contraction slot 8g + e <-> key 4g + e, or 16 + 4g + e - 4 for e >= 4), and
//                  the A fragment takes the same keys of V^T, which is how V is laid down in
//                  LDS (transposed on the way in, 2-byte stores).
// Row maxima and sums need only the 4 lanes that share a query row (two shuffles).  The next
// block of keys and values is fetched into registers while the current one is computed.  bf16
// inputs, fp32 scores, probabilities rounded to bf16 for the second product, fp32 output
// accumulators: the usual flash-attention arithmetic, not the eager fp32 one.
#pragma once
#include "ajq_common.h"

namespace ajq {

constexpr int kPfBQ = 64, kPfBK = 32, kPfHD = 128;
constexpr int kPfKStride = kPfHD + 8;   // bf16 elements per K row in LDS
constexpr int kPfVStride = kPfBK + 8;   // bf16 elements per V^T row in LDS (80 B: conflict-free 8-byte reads)

__device__ __forceinline__ u32x4_t pack8_bf16(const float* v) {
  u32x4_t r;
  r.x = f32_to_bf16_rne(v[0]) | ((uint32_t)f32_to_bf16_rne(v[1]) << 16);
  r.y = f32_to_bf16_rne(v[2]) | ((uint32_t)f32_to_bf16_rne(v[3]) << 16);
  r.z = f32_to_bf16_rne(v[4]) | ((uint32_t)f32_to_bf16_rne(v[5]) << 16);
  r.w = f32_to_bf16_rne(v[6]) | ((uint32_t)f32_to_bf16_rne(v[7]) << 16);
  return r;
}
// 8 consecutive cache elements as loaded, and their bf16 form (made when they are needed, so
// that the loads can stay in flight meanwhile)
struct Raw8F32 {
  float4 a, b;
};
__device__ __forceinline__ Raw8F32 load8_raw(const float* p) {
  return Raw8F32{reinterpret_cast<const float4*>(p)[0], reinterpret_cast<const float4*>(p)[1]};
}
__device__ __forceinline__ u32x4_t load8_raw(const uint16_t* p) { return *reinterpret_cast<const u32x4_t*>(p); }
__device__ __forceinline__ u32x4_t to_bf16x8(const Raw8F32& r) {
  const float v[8] = {r.a.x, r.a.y, r.a.z, r.a.w, r.b.x, r.b.y, r.b.z, r.b.w};
  return pack8_bf16(v);
}
__device__ __forceinline__ u32x4_t to_bf16x8(const u32x4_t& r) { return r; }

template <typename CacheT>
__global__ __launch_bounds__(256) void attn_prefill_kernel(const float* __restrict__ q, const CacheT* __restrict__ kcache,
                                                           const CacheT* __restrict__ vcache, int H, int Hkv, int T,
                                                           int start, int max_len, float* __restrict__ out) {
  __shared__ __attribute__((aligned(16))) uint16_t Ks[kPfBK * kPfKStride];
  __shared__ __attribute__((aligned(16))) uint16_t Vt[kPfHD * kPfVStride];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int qblocks = (T + kPfBQ - 1) / kPfBQ;
  const int qb = qblocks - 1 - blockIdx.x;  // the long rows first
  const int bh = blockIdx.y, b = bh / H, h = bh % H, hk = h / (H / Hkv);
  const int q0 = qb * kPfBQ;
  const int qrow = q0 + 16 * wave + r;             // this lane's query row (as B-operand column)
  const int q_pos = start + qrow;                  // its absolute position
  const float qscale = 1.4426950408889634f * 0.08838834764831845f;  // log2(e) / sqrt(128)

  // ---- Q fragments: Q[qrow][32 s + 8 g .. + 8), scaled, bf16
  u32x4_t qf[4];
  {
    const float* qp = q + ((size_t)bh * T + min(qrow, T - 1)) * kPfHD + 8 * g;
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const float4 a = reinterpret_cast<const float4*>(qp + 32 * s)[0], c = reinterpret_cast<const float4*>(qp + 32 * s)[1];
      const float v[8] = {a.x * qscale, a.y * qscale, a.z * qscale, a.w * qscale,
                          c.x * qscale, c.y * qscale, c.z * qscale, c.w * qscale};
      qf[s] = pack8_bf16(v);
    }
  }
  const CacheT* kbase = kcache + ((size_t)b * Hkv + hk) * max_len * kPfHD;
  const CacheT* vbase = vcache + ((size_t)b * Hkv + hk) * max_len * kPfHD;
  const int kv_len = start + T;                               // rows the caches hold for this call
  const int kv_end = min(kv_len, start + q0 + kPfBQ);         // keys any row of this workgroup may see

  float m_run = -INFINITY, l_run = 0.f;
  f32x4_t o[8];
#pragma unroll
  for (int t = 0; t < 8; ++t) o[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  // One block of keys and values in registers, as loaded (8 elements per chunk, two chunks per
  // thread and operand): chunk c of K is (key c / 16, dims 8 (c % 16) ..), of V (key c % 32,
  // dims 8 (c / 32) ..): keys vary fastest across the lanes that store V transposed.
  typedef decltype(load8_raw(kbase)) raw8_t;
  raw8_t kraw[2], vraw[2];
  auto fetch = [&](int kb0) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int c = threadIdx.x + 256 * u;
      kraw[u] = load8_raw(kbase + (size_t)min(kb0 + (c >> 4), kv_len - 1) * kPfHD + 8 * (c & 15));
      vraw[u] = load8_raw(vbase + (size_t)min(kb0 + (c & 31), kv_len - 1) * kPfHD + 8 * (c >> 5));
    }
  };
  fetch(0);
  for (int kb0 = 0; kb0 < kv_end; kb0 += kPfBK) {
    __syncthreads();  // the previous block's fragments have been read
    // ---- K block row-major (16-byte stores), V block transposed (2-byte stores)
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int c = threadIdx.x + 256 * u;
      *reinterpret_cast<u32x4_t*>(Ks + (c >> 4) * kPfKStride + 8 * (c & 15)) = to_bf16x8(kraw[u]);
      const u32x4_t vv8 = to_bf16x8(vraw[u]);
      uint16_t* dst = Vt + (8 * (c >> 5)) * kPfVStride + (c & 31);
      dst[0 * kPfVStride] = (uint16_t)(vv8.x & 0xFFFFu); dst[1 * kPfVStride] = (uint16_t)(vv8.x >> 16);
      dst[2 * kPfVStride] = (uint16_t)(vv8.y & 0xFFFFu); dst[3 * kPfVStride] = (uint16_t)(vv8.y >> 16);
      dst[4 * kPfVStride] = (uint16_t)(vv8.z & 0xFFFFu); dst[5 * kPfVStride] = (uint16_t)(vv8.z >> 16);
      dst[6 * kPfVStride] = (uint16_t)(vv8.w & 0xFFFFu); dst[7 * kPfVStride] = (uint16_t)(vv8.w >> 16);
    }
    __syncthreads();
    // the next block's loads fly while this one is computed
    if (kb0 + kPfBK < kv_end) fetch(kb0 + kPfBK);
    // ---- scores of the two 16-key halves: sc[jb][i] = S[qrow r][key kb0 + 16 jb + 4 g + i] (log2 units)
    f32x4_t sc[2];
#pragma unroll
    for (int jb = 0; jb < 2; ++jb) {
      sc[jb] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        const u32x4_t a = *reinterpret_cast<const u32x4_t*>(Ks + (16 * jb + r) * kPfKStride + 32 * s + 8 * g);
        sc[jb] = mfma16(a, qf[s], sc[jb]);
      }
    }
    float p[8];
    float mx = -INFINITY;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int key_pos = kb0 + 16 * (e >> 2) + 4 * g + (e & 3);
      p[e] = key_pos <= q_pos ? sc[e >> 2][e & 3] : -INFINITY;  // causal mask (also hides rows past kv_len)
      mx = fmaxf(mx, p[e]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16));
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    const float m_new = fmaxf(m_run, mx);
    // a row that has seen no key yet keeps m = -inf: its probabilities and correction are 0 / 1
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float corr = exp2f(m_run - m_use);  // exp2(-inf) = 0 on the first block
    float rowsum = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      p[e] = exp2f(p[e] - m_use);
      rowsum += p[e];
    }
    rowsum += __shfl_xor(rowsum, 16);
    rowsum += __shfl_xor(rowsum, 32);
    l_run = l_run * corr + rowsum;
    m_run = m_new;
    const u32x4_t pf = pack8_bf16(p);
    // ---- O^T[hd 16 t + 4 g + i][qrow r] += sum over the 32 keys
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      const uint16_t* vrow = Vt + (16 * t + r) * kPfVStride + 4 * g;
      const u32x2_t lo = *reinterpret_cast<const u32x2_t*>(vrow);        // keys 4g .. 4g+3
      const u32x2_t hi = *reinterpret_cast<const u32x2_t*>(vrow + 16);   // keys 16+4g .. 16+4g+3
      o[t] *= corr;
      o[t] = mfma16(u32x4_t{lo.x, lo.y, hi.x, hi.y}, pf, o[t]);
    }
  }
  if (qrow >= T) return;
  const float inv = 1.0f / l_run;
  float* dst = out + ((size_t)b * T + qrow) * ((size_t)H * kPfHD) + (size_t)h * kPfHD + 4 * g;
#pragma unroll
  for (int t = 0; t < 8; ++t)
    *reinterpret_cast<float4*>(dst + 16 * t) = float4{o[t][0] * inv, o[t][1] * inv, o[t][2] * inv, o[t][3] * inv};
}

}  // namespace ajq
