// Causal self-attention for a block of T new positions (prefill), head_dim HD = 128, 64 or 32, on bf16 MFMA
// with an online softmax: the T x (start + T) score matrix is never materialised.
//
//   out[b, t, h, :] = softmax_j( q[b, h, t, :] . k[b, hk, j, :] / sqrt(HD) ) v[b, hk, j, :],
//   j <= start + t,   hk = h / (H / Hkv)
//
// q is fp32 [B, H, T, HD] (already rotated); keys and values are read where the model keeps
// them, in the caches [B, Hkv, max_len, HD] (fp32 or bf16), rows 0 .. start + T - 1; out is
// fp32 or bf16 [B, T, H * HD], the layout the output projection takes.  (The layouts below are
// written out for HD = 128; with 64 a row is 128 B = 8 chunks = 4 segments and there are two k-steps, with 32 a row is
// 64 B = 4 chunks = 2 segments and there is one.)
//
// A workgroup of 4 waves owns 128 query rows of one (b, h), a wave two groups of 16 of them
// (every key and value fragment read from LDS meets both), and walks the keys in blocks of 64.
// Both products run transposed so that no operand changes layout between them:
//   S^T = K Q^T :  A = 16 keys x 32 dims from the row-major key tile in LDS, B = the wave's Q
//                  fragments (registers, bf16, pre-scaled by log2(e) / sqrt(HD)); lane
//                  (g = l / 16, r = l % 16) receives keys 4g..4g+3 of query row r.  The
//                  accumulator starts at minus the row's reference point, so the MFMA result is
//                  the exponent itself.
//   O^T += V^T P^T: the lane's 8 probabilities of a 32-key half ARE its B fragment (contraction
//                  slot 8g + e <-> key 4g + e of the first 16-key tile for e < 4, of the second
//                  for e >= 4), and the A fragment takes the same keys of V^T with two
//                  transposing LDS reads (ds_read_b64_tr_b16) from the ROW-MAJOR value tile:
//                  nothing is transposed on the way into LDS.
// Both tiles are unpadded (a row is 256 B); the 16-byte chunks of a row sit in slots permuted by
// the row index so that the fragment reads spread over all banks.
//
// Softmax bookkeeping is kept off the common path.  A row's reference point only moves when an
// exponent would exceed 2^kPfSlack (always on the first block): the test is one compare of the
// lane's sum of new probabilities (a sum of positives bounds each of them; inf passes it too),
// and only then are the maxima taken (across the four lanes of a row with two lane swaps), the
// probabilities recomputed and the accumulators rescaled.  Row sums stay per lane and meet once,
// at the end.  bf16 inputs, fp32 scores, probabilities rounded to bf16 for the second product,
// fp32 accumulators: the usual flash-attention arithmetic, not the eager fp32 one.
#pragma once
#include "ajq_common.h"
#include "gemm_kernels.h"  // dma16: global -> LDS without registers

namespace ajq {

constexpr float kPfSlack = 8.0f;          // log2 of how far a row's exponents may exceed its reference point
constexpr float kPfTrigger = 4096.0f;     // lane sum of 16 probabilities above which the reference point is revisited
constexpr int kPfBQ = 128, kPfBK = 64;

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

// max / sum over the four lanes l, l ^ 16, l ^ 32, l ^ 48 (the lanes that share a query row):
// v_permlane16_swap and v_permlane32_swap hand every lane its partner's value in one VALU
// instruction each, without a trip through the LDS crossbar.
__device__ __forceinline__ float quad_max(float x) {
  typedef uint32_t u32x2v __attribute__((ext_vector_type(2)));
  uint32_t b = __float_as_uint(x);
  u32x2v s = __builtin_amdgcn_permlane16_swap(b, b, false, false);
  x = fmaxf(__uint_as_float(s.x), __uint_as_float(s.y));
  b = __float_as_uint(x);
  s = __builtin_amdgcn_permlane32_swap(b, b, false, false);
  return fmaxf(__uint_as_float(s.x), __uint_as_float(s.y));
}
__device__ __forceinline__ float quad_sum(float x) {
  typedef uint32_t u32x2v __attribute__((ext_vector_type(2)));
  uint32_t b = __float_as_uint(x);
  u32x2v s = __builtin_amdgcn_permlane16_swap(b, b, false, false);
  x = __uint_as_float(s.x) + __uint_as_float(s.y);
  b = __float_as_uint(x);
  s = __builtin_amdgcn_permlane32_swap(b, b, false, false);
  return __uint_as_float(s.x) + __uint_as_float(s.y);
}

typedef short pf_i16x4_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) pf_i16x4_t pf_lds_i16x4_t;
typedef __attribute__((address_space(3))) const u32x4_t pf_lds_u32x4_t;
typedef __attribute__((address_space(3))) unsigned char pf_lds_char_t;
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Wint-to-pointer-cast"  // the host pass sees 64-bit pointers
// Transposing LDS read: within each block of 16 lanes, lane 4 a + j receives element j of the
// 8-byte rows addressed by lanes a, 4 + a, 8 + a and 12 + a of the block.
__device__ __forceinline__ u32x2_t pf_read_tr(uint32_t address) {
  return __builtin_bit_cast(u32x2_t, __builtin_amdgcn_ds_read_tr16_b64_v4i16((pf_lds_i16x4_t*)address));
}
__device__ __forceinline__ u32x4_t pf_read128(uint32_t address) { return *(pf_lds_u32x4_t*)address; }
#pragma clang diagnostic pop

template <typename CacheT, int HD>
__global__ __launch_bounds__(256, 2) void attn_prefill_kernel(const float* __restrict__ q, const CacheT* __restrict__ kcache,
                                                           const CacheT* __restrict__ vcache, int H, int Hkv, int T,
                                                           int start, int max_len, void* __restrict__ out, int out_bf16) {
  static_assert(HD == 128 || HD == 64 || HD == 32, "head_dim 128, 64 or 32");
  constexpr int kPfHD = HD;
  constexpr int RB = 2 * HD;          // bytes of a key (value) row as bf16
  constexpr int C = HD / 8;           // 16-byte chunks per row
  constexpr int KS = HD / 32;         // k-steps of the first product; also the parts a block's DMA is issued in
  constexpr int TT = HD / 16;         // 32-byte segments per row = 16-dim output tiles
  constexpr int kPfTileBytes = kPfBK * RB;  // one block of keys (or values) as bf16: 16 KiB at HD = 128
  // LDS map (byte addresses relative to lds0, the array's LDS address, which is 0 because the kernel
  // declares no other LDS; naming it also keeps the array allocated when nothing else refers to
  // it): two stages of a key tile and a value tile, 16 KiB each.
  //   stage s: keys at s * 32 Ki, values at s * 32 Ki + 16 Ki
  // Key tile: 16-byte chunk c of key row k sits at k * 256 + 16 * (c ^ (k & 15)).
  // Value tile: chunk c of row k sits at k * 256 + 16 * ((((c >> 1) ^ (k & 7)) << 1) | (c & 1))
  // (32-byte segments permuted: a transposing read takes 8 bytes of each of 16 keys).
  __shared__ __attribute__((aligned(1024))) unsigned char lds[4 * kPfTileBytes];
  const uint32_t lds0 = (uint32_t)(uintptr_t)(pf_lds_char_t*)lds;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r = lane & 15, g = lane >> 4;
  // Work order.  The hardware deals workgroups to the 8 XCDs round-robin by linear index and,
  // inside an XCD, hands the next one to whichever CU has room.  A query block's cost grows with
  // its position (causal), so the linear order is: XCD k takes a contiguous eighth of the (b, h)
  // pairs (the heads that share a cache head stay on one XCD and its L2) and walks its query
  // blocks from the longest to the shortest.  (With B * H not a multiple of 8: plain longest first.)
  const int qblocks = (T + kPfBQ - 1) / kPfBQ;
  const int BH = (int)(gridDim.x / (unsigned)qblocks);
  int qb, bh;
  if ((BH & 7) == 0) {
    const int per_xcd = BH >> 3, m = (int)(blockIdx.x >> 3);
    qb = qblocks - 1 - m / per_xcd;
    bh = (int)(blockIdx.x & 7) * per_xcd + m % per_xcd;
  } else {
    qb = qblocks - 1 - (int)blockIdx.x / BH;
    bh = (int)blockIdx.x % BH;
  }
  const int b = bh / H, h = bh % H, hk = h / (H / Hkv);
  const int q0 = qb * kPfBQ;
  const float qscale =  // log2(e) / sqrt(HD)
      1.4426950408889634f * (HD == 128 ? 0.08838834764831845f : HD == 64 ? 0.125f : 0.17677669529663687f);

  const CacheT* kbase = kcache + ((size_t)b * Hkv + hk) * max_len * kPfHD;
  const CacheT* vbase = vcache + ((size_t)b * Hkv + hk) * max_len * kPfHD;
  const int kv_len = start + T;                               // rows the caches hold for this call
  const int kv_end = min(kv_len, start + q0 + kPfBQ);         // keys any row of this workgroup may see
  const int nblk = (kv_end + kPfBK - 1) / kPfBK;
  const int wave_last_pos = start + q0 + 32 * wave + 31;      // last query position of this wave

  float m_run[2], l_run[2];
  f32x4_t negm[2];
  f32x4_t o[2][TT];
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    m_run[u] = 0.f;
    l_run[u] = 0.f;
    negm[u] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int t = 0; t < TT; ++t) o[u][t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }

  // ---- Keys and values on their way into LDS.
  // bf16 caches: global -> LDS directly, one block ahead.  A wave-wide request fills 1 KiB = 4 key
  // rows (8 rows at HD = 64); wave w takes rows 4 w .. 4 w + 3 of every group of 16, so (row & 15) = 4 w + lane / 16 is
  // fixed per lane and the chunk it must fetch for its slot is too.
  // fp32 caches: through registers (converted on the way), one block in registers while the
  // previous one is being read: chunk ci = tid + 256 i (i < 4) is (key ci / 16, dims 8 (ci % 16) ..).
  // Rows past the filled part of the cache repeat its last row (finite values; those keys are masked).
  constexpr bool kDma = sizeof(CacheT) == 2;
  constexpr int kReqRows = 1024 / RB;  // key rows of one wave-wide request: 4 (HD = 128) or 8
  const int krow = kReqRows * wave + lane / C, slot = lane % C;
  const uint32_t k_chunk = (uint32_t)(slot ^ (krow & (C - 1)));
  const uint32_t v_chunk = (uint32_t)((((slot >> 1) ^ (krow & (TT - 1))) << 1) | (slot & 1));
  // part i (0 .. KS - 1) of block jblk: this wave's kReqRows key rows and value rows of the i-th group of 4 * kReqRows
  auto issue_dma = [&](int jblk, int i) {
    const int kb0 = jblk * kPfBK;
    const uint32_t stage = lds0 + (uint32_t)((jblk & 1) * 2 * kPfTileBytes);
    const uint32_t k_to = stage + (uint32_t)((wave + 4 * i) * 1024), v_to = k_to + (uint32_t)kPfTileBytes;
    if (kb0 + kPfBK <= kv_len) {
      const size_t row0 = (size_t)(kb0 + 4 * kReqRows * i) * RB;
      dma16(reinterpret_cast<const char*>(kbase) + row0, (uint32_t)(krow * RB) + k_chunk * 16u, k_to);
      dma16(reinterpret_cast<const char*>(vbase) + row0, (uint32_t)(krow * RB) + v_chunk * 16u, v_to);
    } else {
      const uint32_t row = (uint32_t)min(kb0 + 4 * kReqRows * i + krow, kv_len - 1) * (uint32_t)RB;
      dma16(kbase, row + k_chunk * 16u, k_to);
      dma16(vbase, row + v_chunk * 16u, v_to);
    }
  };
  typedef decltype(load8_raw(kbase)) raw8_t;
  constexpr int kRegParts = kDma ? 0 : kPfBK * C / 256;  // 16-byte chunks of a block per thread: 4 (HD = 128) or 2
  raw8_t kraw[kDma ? 1 : kRegParts], vraw[kDma ? 1 : kRegParts];
  uint32_t k_st[kDma ? 1 : kRegParts], v_st[kDma ? 1 : kRegParts];
  auto fetch = [&](int kb0) {
#pragma unroll
    for (int i = 0; i < kRegParts; ++i) {
      const int ci = threadIdx.x + 256 * i;
      const size_t at = (size_t)min(kb0 + ci / C, kv_len - 1) * kPfHD + 8 * (ci % C);
      kraw[i] = load8_raw(kbase + at);
      vraw[i] = load8_raw(vbase + at);
    }
  };
#pragma unroll
  for (int i = 0; i < kRegParts; ++i) {
    const int ci = threadIdx.x + 256 * i, k = ci / C, c = ci % C;
    k_st[i] = (uint32_t)(k * RB + 16 * (c ^ (k & (C - 1))));
    v_st[i] = (uint32_t)(kPfTileBytes + k * RB + 16 * ((((c >> 1) ^ (k & (TT - 1))) << 1) | (c & 1)));
  }
  auto lay_down = [&](int stage) {
#pragma unroll
    for (int i = 0; i < kRegParts; ++i) {
      *reinterpret_cast<u32x4_t*>(lds + stage * 2 * kPfTileBytes + k_st[i]) = to_bf16x8(kraw[i]);
      *reinterpret_cast<u32x4_t*>(lds + stage * 2 * kPfTileBytes + v_st[i]) = to_bf16x8(vraw[i]);
    }
  };
  // ---- LDS read addresses (of the stage being read; flipped to the other stage after every block).
  // key fragment (tile jb, k-step s): row 16 jb + r, chunk 4 s + g  ->  (16 jb + r) * 256 + 16 * ((4 s + g) ^ r)
  uint32_t k_rd[KS];
#pragma unroll
  for (int s = 0; s < KS; ++s) k_rd[s] = lds0 + (uint32_t)(r * RB + 16 * ((4 * s + g) ^ (r & (C - 1))));
  // value fragment (half hf, slots 4 w2 .. 4 w2 + 3, dims 16 t ..): this lane addresses 8 bytes of key
  // 32 hf + 16 w2 + 4 g + (r >> 2): piece (r & 3) of the 32-byte segment t, which sits in slot t ^ (key & 7)
  const int vkey = 4 * g + (r >> 2);  // (16 w2 and 32 hf do not change key & 7)
  uint32_t v_rd[TT];
#pragma unroll
  for (int t = 0; t < TT; ++t)
    v_rd[t] = lds0 + (uint32_t)(kPfTileBytes + vkey * RB + 32 * (t ^ (vkey & (TT - 1))) + 8 * (r & 3));

  if (kDma) {
#pragma unroll
    for (int i = 0; i < KS; ++i) issue_dma(0, i);
  } else {
    fetch(0);
    lay_down(0);
    if (nblk > 1) fetch(kPfBK);
  }
  // ---- (after the first block's requests, so that both round trips to memory overlap)
  // Q fragments of the wave's two groups of 16 rows: Q[qrow][32 s + 8 g .. + 8), scaled, bf16.
  // Group u of wave w holds rows q0 + 32 w + 16 u .. + 15; this lane's row of it is qrow[u].
  int qrow[2], q_pos[2];
  u32x4_t qf[2][KS];
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    qrow[u] = q0 + 32 * wave + 16 * u + r;
    q_pos[u] = start + qrow[u];
    const float* qp = q + ((size_t)bh * T + min(qrow[u], T - 1)) * kPfHD + 8 * g;
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const float4 a = reinterpret_cast<const float4*>(qp + 32 * s)[0], c = reinterpret_cast<const float4*>(qp + 32 * s)[1];
      const float v[8] = {a.x * qscale, a.y * qscale, a.z * qscale, a.w * qscale,
                          c.x * qscale, c.y * qscale, c.z * qscale, c.w * qscale};
      qf[u][s] = pack8_bf16(v);
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  for (int j = 0; j < nblk; ++j) {
    // One barrier per block: block j is complete in stage j & 1 (it landed before the previous
    // barrier); block j + 1 goes into the other stage, which was last read before that barrier
    // too (fp32 caches: from registers, while block j + 2 starts its flight from memory).
    const int kb0 = j * kPfBK;
    // bf16 caches: the requests for block j + 1 are issued between the products below (one part
    // per k-step), or here by a wave that has no products to form
    const bool more = j + 1 < nblk;
    if (more) {
      if (kDma) {
        if (kb0 > wave_last_pos) {
#pragma unroll
          for (int i = 0; i < KS; ++i) issue_dma(j + 1, i);
        }
      } else {
        lay_down((j + 1) & 1);
        if (j + 2 < nblk) fetch(kb0 + 2 * kPfBK);
      }
    }
    // a wave whose last query lies before the block has nothing to add
    if (kb0 <= wave_last_pos) {
      // ---- exponents of the four 16-key tiles: sc[u][jb][i] = S[qrow[u]][key kb0 + 16 jb + 4 g + i] - m_run[u]
      // (log2 units).  k-step outermost: the eight products of a step are independent, and a key
      // fragment is read once for both query groups.
      f32x4_t sc[2][4];
      u32x4_t ka[4];
#pragma unroll
      for (int jb = 0; jb < 4; ++jb) ka[jb] = pf_read128(k_rd[0] + (uint32_t)(jb * 16 * RB));
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        u32x4_t kn[4];
        if (kDma && s < KS - 1) {  // (the fp32 path has no registers to spare for a second set)
#pragma unroll
          for (int jb = 0; jb < 4; ++jb) kn[jb] = pf_read128(k_rd[s + 1] + (uint32_t)(jb * 16 * RB));
        }
#pragma unroll
        for (int jb = 0; jb < 4; ++jb)
#pragma unroll
          for (int u = 0; u < 2; ++u) sc[u][jb] = mfma16(ka[jb], qf[u][s], s == 0 ? negm[u] : sc[u][jb]);
        if (kDma && more) issue_dma(j + 1, s);
        if (s < KS - 1) {
#pragma unroll
          for (int jb = 0; jb < 4; ++jb) ka[jb] = kDma ? kn[jb] : pf_read128(k_rd[s + 1] + (uint32_t)(jb * 16 * RB));
        }
      }
      // only blocks that reach past the wave's first query position need the causal mask
      if (kb0 + kPfBK - 1 > wave_last_pos - 31) {
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int jb = 0; jb < 4; ++jb)
#pragma unroll
            for (int i = 0; i < 4; ++i)
              if (kb0 + 16 * jb + 4 * g + i > q_pos[u]) sc[u][jb][i] = -INFINITY;  // (also hides rows past kv_len)
      }
      // The reference point of a row moves only when an exponent has outgrown it by more than
      // kPfSlack (and on the first block, where it is still arbitrary).  One query group at a
      // time, so that only one group's exponents and probabilities are live together.
      u32x4_t pf[2][2];
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        float p[16], psum = 0.f;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          p[e] = __builtin_amdgcn_exp2f(sc[u][e >> 2][e & 3]);  // v_exp_f32: underflow to 0 is what is wanted
          psum += p[e];
        }
        const bool revisit = j == 0 || psum > kPfTrigger;
        if (__builtin_amdgcn_ballot_w64(revisit) != 0) {
          float mx = -INFINITY;
#pragma unroll
          for (int e = 0; e < 16; ++e) mx = fmaxf(mx, sc[u][e >> 2][e & 3]);
          mx = quad_max(mx);
          const bool move = j == 0 || mx > kPfSlack;
          const float shift = move ? mx : 0.f;
          const float corr = (move && j != 0) ? __builtin_amdgcn_exp2f(-shift) : 1.0f;
          psum = 0.f;
#pragma unroll
          for (int e = 0; e < 16; ++e) {
            p[e] = __builtin_amdgcn_exp2f(sc[u][e >> 2][e & 3] - shift);
            psum += p[e];
          }
          m_run[u] += shift;
          negm[u] = f32x4_t{-m_run[u], -m_run[u], -m_run[u], -m_run[u]};
          l_run[u] *= corr;
#pragma unroll
          for (int t = 0; t < TT; ++t) o[u][t] *= corr;
        }
        l_run[u] += psum;
        pf[u][0] = pack8_bf16(&p[0]);
        pf[u][1] = pack8_bf16(&p[8]);
      }
      // ---- O^T[hd 16 t + 4 g + i][qrow] += sum over the keys of each 32-key half; a value fragment
      // (two transposing reads: the half's first and second 16-key tile) meets both query groups.
      // The second half's fragments are requested as the first half's are consumed.
      constexpr int kRing = kDma ? (TT < 8 ? TT : 8) : 4;  // fragments in flight (the fp32 path has fewer registers to spare)
      auto v_lo = [&](int i) { return pf_read_tr(v_rd[i % TT] + (uint32_t)((i / TT) * 32 * RB)); };
      auto v_hi = [&](int i) { return pf_read_tr(v_rd[i % TT] + (uint32_t)((i / TT) * 32 * RB + 16 * RB)); };
      u32x2_t vlo[kRing], vhi[kRing];
#pragma unroll
      for (int i = 0; i < kRing; ++i) {
        vlo[i] = v_lo(i);
        vhi[i] = v_hi(i);
      }
#pragma unroll
      for (int i = 0; i < 2 * TT; ++i) {  // i = TT hf + t
        const u32x4_t vf = {vlo[i % kRing].x, vlo[i % kRing].y, vhi[i % kRing].x, vhi[i % kRing].y};
#pragma unroll
        for (int u = 0; u < 2; ++u) o[u][i % TT] = mfma16(vf, pf[u][i / TT], o[u][i % TT]);
        if (i + kRing < 2 * TT) {
          vlo[i % kRing] = v_lo(i + kRing);
          vhi[i % kRing] = v_hi(i + kRing);
        }
      }
    }
    // flip every read address to the other stage
#pragma unroll
    for (int s = 0; s < KS; ++s) k_rd[s] ^= (uint32_t)(2 * kPfTileBytes);
#pragma unroll
    for (int t = 0; t < TT; ++t) v_rd[t] ^= (uint32_t)(2 * kPfTileBytes);
    // the next block must have landed and every wave must be done with this one
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
  }
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const float inv = 1.0f / quad_sum(l_run[u]);
    if (qrow[u] >= T) continue;
    const size_t at = ((size_t)b * T + qrow[u]) * ((size_t)H * kPfHD) + (size_t)h * kPfHD + 4 * g;
    if (out_bf16) {
      uint16_t* dst = reinterpret_cast<uint16_t*>(out) + at;
#pragma unroll
      for (int t = 0; t < TT; ++t)
        *reinterpret_cast<u32x2_t*>(dst + 16 * t) =
            u32x2_t{pack2_bf16(o[u][t][0] * inv, o[u][t][1] * inv), pack2_bf16(o[u][t][2] * inv, o[u][t][3] * inv)};
    } else {
      float* dst = reinterpret_cast<float*>(out) + at;
#pragma unroll
      for (int t = 0; t < TT; ++t)
        *reinterpret_cast<float4*>(dst + 16 * t) =
            float4{o[u][t][0] * inv, o[u][t][1] * inv, o[u][t][2] * inv, o[u][t][3] * inv};
    }
  }
}

}  // namespace ajq
