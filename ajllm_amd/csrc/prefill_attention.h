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
// A workgroup of 4 waves owns 128 query rows of one (b, h), a wave two groups of 16 of them
// (every key and value fragment read from LDS meets both), and walks the keys in blocks of 32.  Both products run transposed so that no operand changes layout
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

#ifndef AJQ_PF_QG
#define AJQ_PF_QG 2
#endif
constexpr int kPfQG = AJQ_PF_QG;          // groups of 16 query rows per wave
constexpr float kPfSlack = 8.0f;          // log2 of how far a row's scores may exceed its reference point
constexpr int kPfBQ = 64 * kPfQG, kPfBK = 32, kPfHD = 128;
constexpr int kPfKStride = kPfHD + 8;   // bf16 elements per K row in LDS
constexpr int kPfVStride = kPfBK + 8;   // bf16 elements per V^T row in LDS (80 B: conflict-free 8-byte reads)

__device__ __forceinline__ u32x4_t pack8_bf16(const float* v) {
  return u32x4_t{pack2_bf16(v[0], v[1]), pack2_bf16(v[2], v[3]), pack2_bf16(v[4], v[5]), pack2_bf16(v[6], v[7])};
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
__global__ __launch_bounds__(256, 2) void attn_prefill_kernel(const float* __restrict__ q, const CacheT* __restrict__ kcache,
                                                           const CacheT* __restrict__ vcache, int H, int Hkv, int T,
                                                           int start, int max_len, void* __restrict__ out, int out_bf16) {
  // two buffers of each: a block is laid down while the previous one is still being read
  __shared__ __attribute__((aligned(16))) uint16_t Ks2[2][kPfBK * kPfKStride];
  __shared__ __attribute__((aligned(16))) uint16_t Vt2[2][kPfHD * kPfVStride];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int qblocks = (T + kPfBQ - 1) / kPfBQ;
  const int qb = qblocks - 1 - blockIdx.x;  // the long rows first
  const int bh = blockIdx.y, b = bh / H, h = bh % H, hk = h / (H / Hkv);
  const int q0 = qb * kPfBQ;
  const float qscale = 1.4426950408889634f * 0.08838834764831845f;  // log2(e) / sqrt(128)

  // ---- Q fragments of the wave's kPfQG groups of 16 rows: Q[qrow][32 s + 8 g .. + 8), scaled, bf16.
  // Group u of wave w holds rows q0 + 16 (kPfQG w + u) .. + 15; this lane's row of it is qrow[u].
  int qrow[kPfQG], q_pos[kPfQG];
  u32x4_t qf[kPfQG][4];
#pragma unroll
  for (int u = 0; u < kPfQG; ++u) {
    qrow[u] = q0 + 16 * (kPfQG * wave + u) + r;
    q_pos[u] = start + qrow[u];
    const float* qp = q + ((size_t)bh * T + min(qrow[u], T - 1)) * kPfHD + 8 * g;
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const float4 a = reinterpret_cast<const float4*>(qp + 32 * s)[0], c = reinterpret_cast<const float4*>(qp + 32 * s)[1];
      const float v[8] = {a.x * qscale, a.y * qscale, a.z * qscale, a.w * qscale,
                          c.x * qscale, c.y * qscale, c.z * qscale, c.w * qscale};
      qf[u][s] = pack8_bf16(v);
    }
  }
  const CacheT* kbase = kcache + ((size_t)b * Hkv + hk) * max_len * kPfHD;
  const CacheT* vbase = vcache + ((size_t)b * Hkv + hk) * max_len * kPfHD;
  const int kv_len = start + T;                               // rows the caches hold for this call
  const int kv_end = min(kv_len, start + q0 + kPfBQ);         // keys any row of this workgroup may see

  float m_run[kPfQG], l_run[kPfQG];
  f32x4_t o[kPfQG][8];
#pragma unroll
  for (int u = 0; u < kPfQG; ++u) {
    m_run[u] = -INFINITY;
    l_run[u] = 0.f;
#pragma unroll
    for (int t = 0; t < 8; ++t) o[u][t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }

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
  // registers -> LDS: K block row-major (16-byte stores), V block transposed (2-byte stores)
  auto lay_down = [&](int buf) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int c = threadIdx.x + 256 * u;
      *reinterpret_cast<u32x4_t*>(Ks2[buf] + (c >> 4) * kPfKStride + 8 * (c & 15)) = to_bf16x8(kraw[u]);
      const u32x4_t vv8 = to_bf16x8(vraw[u]);
      uint16_t* dst = Vt2[buf] + (8 * (c >> 5)) * kPfVStride + (c & 31);
      dst[0 * kPfVStride] = (uint16_t)(vv8.x & 0xFFFFu); dst[1 * kPfVStride] = (uint16_t)(vv8.x >> 16);
      dst[2 * kPfVStride] = (uint16_t)(vv8.y & 0xFFFFu); dst[3 * kPfVStride] = (uint16_t)(vv8.y >> 16);
      dst[4 * kPfVStride] = (uint16_t)(vv8.z & 0xFFFFu); dst[5 * kPfVStride] = (uint16_t)(vv8.z >> 16);
      dst[6 * kPfVStride] = (uint16_t)(vv8.w & 0xFFFFu); dst[7 * kPfVStride] = (uint16_t)(vv8.w >> 16);
    }
  };
  fetch(0);
  lay_down(0);
  if (kPfBK < kv_end) fetch(kPfBK);
  __syncthreads();
  for (int kb0 = 0; kb0 < kv_end; kb0 += kPfBK) {
    // One barrier per block: block kb0 is complete in buffer `cur` (laid down before the
    // previous barrier); block kb0 + 32 goes from registers into the other buffer, which was
    // last read before that barrier too; block kb0 + 64 starts its flight from memory.
    const int cur = (kb0 / kPfBK) & 1;
    const uint16_t* Ks = Ks2[cur];
    const uint16_t* Vt = Vt2[cur];
    if (kb0 + kPfBK < kv_end) {
      lay_down(cur ^ 1);
      if (kb0 + 2 * kPfBK < kv_end) fetch(kb0 + 2 * kPfBK);
    }
    // ---- scores of the two 16-key halves: sc[u][jb][i] = S[qrow[u]][key kb0 + 16 jb + 4 g + i]
    // (log2 units); a key fragment is read once for all the wave's query groups
    f32x4_t sc[kPfQG][2];
#pragma unroll
    for (int jb = 0; jb < 2; ++jb) {
#pragma unroll
      for (int u = 0; u < kPfQG; ++u) sc[u][jb] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        const u32x4_t a = *reinterpret_cast<const u32x4_t*>(Ks + (16 * jb + r) * kPfKStride + 32 * s + 8 * g);
#pragma unroll
        for (int u = 0; u < kPfQG; ++u) sc[u][jb] = mfma16(a, qf[u][s], sc[u][jb]);
      }
    }
    u32x4_t pf[kPfQG];
    float corr[kPfQG];
    // only blocks that reach past the wave's first query position need the causal mask
    const bool diagonal = kb0 + kPfBK - 1 > start + q0 + 16 * kPfQG * wave;
#pragma unroll
    for (int u = 0; u < kPfQG; ++u) {
      float p[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) p[e] = sc[u][e >> 2][e & 3];
      if (diagonal) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int key_pos = kb0 + 16 * (e >> 2) + 4 * g + (e & 3);
          if (key_pos > q_pos[u]) p[e] = -INFINITY;  // (also hides rows past kv_len)
        }
      }
      float mx = fmaxf(fmaxf(fmaxf(p[0], p[1]), fmaxf(p[2], p[3])), fmaxf(fmaxf(p[4], p[5]), fmaxf(p[6], p[7])));
      mx = fmaxf(mx, __shfl_xor(mx, 16));
      mx = fmaxf(mx, __shfl_xor(mx, 32));
      // The reference point of the row's exponentials moves only when the maximum has grown
      // by more than 2^kPfSlack since it was set: probabilities stay below 2^kPfSlack (fp32
      // sums and bf16 operands take that easily) and the accumulators are rescaled rarely.
      const float m_new = mx > m_run[u] + kPfSlack ? mx : m_run[u];
      corr[u] = __builtin_amdgcn_exp2f(m_run[u] - m_new);  // 1 when unchanged, 0 on the first block
      float rowsum = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        p[e] = __builtin_amdgcn_exp2f(p[e] - m_new);  // v_exp_f32: underflow to 0 is what is wanted
        rowsum += p[e];
      }
      rowsum += __shfl_xor(rowsum, 16);
      rowsum += __shfl_xor(rowsum, 32);
      l_run[u] = l_run[u] * corr[u] + rowsum;
      m_run[u] = m_new;
      pf[u] = pack8_bf16(p);
    }
    bool rescale = false;
#pragma unroll
    for (int u = 0; u < kPfQG; ++u) rescale |= corr[u] != 1.0f;
    if (__builtin_amdgcn_ballot_w64(rescale) != 0) {
#pragma unroll
      for (int u = 0; u < kPfQG; ++u)
#pragma unroll
        for (int t = 0; t < 8; ++t) o[u][t] *= corr[u];
    }
    // ---- O^T[hd 16 t + 4 g + i][qrow] += sum over the 32 keys; a value fragment is read once
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      const uint16_t* vrow = Vt + (16 * t + r) * kPfVStride + 4 * g;
      const u32x2_t lo = *reinterpret_cast<const u32x2_t*>(vrow);        // keys 4g .. 4g+3
      const u32x2_t hi = *reinterpret_cast<const u32x2_t*>(vrow + 16);   // keys 16+4g .. 16+4g+3
      const u32x4_t vf = {lo.x, lo.y, hi.x, hi.y};
#pragma unroll
      for (int u = 0; u < kPfQG; ++u) o[u][t] = mfma16(vf, pf[u], o[u][t]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int u = 0; u < kPfQG; ++u) {
    if (qrow[u] >= T) continue;
    const float inv = 1.0f / l_run[u];
    const size_t at = ((size_t)b * T + qrow[u]) * ((size_t)H * kPfHD) + (size_t)h * kPfHD + 4 * g;
    if (out_bf16) {
      uint16_t* dst = reinterpret_cast<uint16_t*>(out) + at;
#pragma unroll
      for (int t = 0; t < 8; ++t)
        *reinterpret_cast<u32x2_t*>(dst + 16 * t) =
            u32x2_t{pack2_bf16(o[u][t][0] * inv, o[u][t][1] * inv), pack2_bf16(o[u][t][2] * inv, o[u][t][3] * inv)};
    } else {
      float* dst = reinterpret_cast<float*>(out) + at;
#pragma unroll
      for (int t = 0; t < 8; ++t)
        *reinterpret_cast<float4*>(dst + 16 * t) =
            float4{o[u][t][0] * inv, o[u][t][1] * inv, o[u][t][2] * inv, o[u][t][3] * inv};
    }
  }
}

}  // namespace ajq
