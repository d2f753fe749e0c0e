// The small operators of one decode step between the quantized linears: residual add +
// RMSNorm, rotary embedding + KV-cache write, single-query attention over the cache, and
// the SwiGLU gate.  All arithmetic is fp32 (the residual stream and the KV cache are fp32);
// outputs that feed a quantized linear are written as bf16, which is what the linear's
// own input cast would produce.  The write position of the step is read from device
// memory, so a recorded HIP graph can be replayed for every token.
#pragma once
#include "ajq_common.h"

namespace ajq {

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off));
  return v;
}

// hidden[b, :] += delta[b, :] (when delta != nullptr; written back), then
// out[b, :] = bf16( (hidden / sqrt(mean(hidden^2) + eps)) * gain ).
// One 256-thread workgroup per row; D % 4 == 0.  The first 4096 elements of a row (four float4 per thread)
// and their gains stay in registers between the two passes: one memory round trip for the usual widths.
__global__ __launch_bounds__(256) void add_rmsnorm_kernel(float* __restrict__ hidden, const float* __restrict__ delta,
                                                          const float* __restrict__ gain, float eps,
                                                          uint16_t* __restrict__ out, int D) {
  constexpr int kKeep = 4;
  const int b = blockIdx.x;
  float4* h4 = reinterpret_cast<float4*>(hidden + (size_t)b * D);
  const float4* d4 = delta ? reinterpret_cast<const float4*>(delta + (size_t)b * D) : nullptr;
  const float4* g4 = reinterpret_cast<const float4*>(gain);
  const int n4 = D >> 2;
  float ss = 0.f;
  auto take = [&](int i) {
    float4 v = h4[i];
    if (d4) {
      const float4 d = d4[i];
      v.x += d.x; v.y += d.y; v.z += d.z; v.w += d.w;
      h4[i] = v;
    }
    ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
    return v;
  };
  float4 keep[kKeep], g[kKeep];
#pragma unroll
  for (int j = 0; j < kKeep; ++j) {
    const int i = threadIdx.x + 256 * j;
    if (i < n4) {
      keep[j] = take(i);
      g[j] = g4[i];
    }
  }
  for (int i = threadIdx.x + 256 * kKeep; i < n4; i += 256) take(i);
  ss = wave_sum(ss);
  __shared__ float part[4];
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = ss;
  __syncthreads();
  ss = (part[0] + part[1]) + (part[2] + part[3]);
  const Divisor by_rms(sqrtf(ss / (float)D + eps));  // (h / rms) * gain, the division as the model code has it
  uint2* o2 = reinterpret_cast<uint2*>(out + (size_t)b * D);
  auto put = [&](int i, const float4& v, const float4& gg) {
    const uint32_t lo = pack2_bf16(by_rms.divide(v.x) * gg.x, by_rms.divide(v.y) * gg.y);
    const uint32_t hi = pack2_bf16(by_rms.divide(v.z) * gg.z, by_rms.divide(v.w) * gg.w);
    o2[i] = uint2{lo, hi};
  };
#pragma unroll
  for (int j = 0; j < kKeep; ++j) {
    const int i = threadIdx.x + 256 * j;
    if (i < n4) put(i, keep[j], g[j]);
  }
  for (int i = threadIdx.x + 256 * kKeep; i < n4; i += 256) put(i, h4[i], g4[i]);  // own writes above: same thread, same addresses
}

// qkv [B, (H + 2 Hkv) * hd] fp32 (q heads, then k heads, then v heads) -> rotated q
// [B, H, hd]; rotated k and plain v are written into the caches [B, Hkv, max_len, hd] at
// row *pos.  Interleaved pairs: (x[2i], x[2i+1]) -> (e c - o s, e s + o c) with the tables'
// row *pos.  One thread per pair.
// The caches hold fp32 or (kBf16) bf16, rounded to nearest even.
__device__ __forceinline__ void store_pair(float* p, float2 v) { *reinterpret_cast<float2*>(p) = v; }
__device__ __forceinline__ void store_pair(uint16_t* p, float2 v) {
  *reinterpret_cast<uint32_t*>(p) = pack2_bf16(v.x, v.y);
}

template <typename CacheT>
__global__ __launch_bounds__(256) void rope_cache_kernel(const float* __restrict__ qkv, const float* __restrict__ cosine,
                                                         const float* __restrict__ sine, const long long* __restrict__ pos,
                                                         float* __restrict__ q_out, CacheT* __restrict__ kcache,
                                                         CacheT* __restrict__ vcache, int B, int H, int Hkv, int hd,
                                                         int max_len) {
  const int half = hd >> 1;
  const int heads = H + 2 * Hkv;
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (long long)B * heads * half) return;
  const int i = (int)(idx % half);
  const int head = (int)((idx / half) % heads);
  const int b = (int)(idx / ((long long)half * heads));
  // the position is device data the host cannot check: held inside the cache so that a stale or
  // unwritten value gives a wrong row, never a wild address
  const long long p = min(max(*pos, 0LL), (long long)max_len - 1);
  const float2 v = *reinterpret_cast<const float2*>(qkv + ((size_t)b * heads + head) * hd + 2 * i);
  if (head >= H + Hkv) {  // value head: stored as it is
    const int hv = head - H - Hkv;
    store_pair(vcache + (((size_t)b * Hkv + hv) * max_len + p) * hd + 2 * i, v);
    return;
  }
  const float c = cosine[p * half + i], s = sine[p * half + i];
  const float2 r = float2{v.x * c - v.y * s, v.x * s + v.y * c};
  if (head < H)
    *reinterpret_cast<float2*>(q_out + ((size_t)b * H + head) * hd + 2 * i) = r;
  else
    store_pair(kcache + (((size_t)b * Hkv + (head - H)) * max_len + p) * hd + 2 * i, r);
}

// Prefill form of the rotation: qkv [B * T, (H + 2 Hkv) * hd] fp32, row b * T + t at absolute
// position start + t.  Rotated queries go to q_out [B, H, T, hd] (the layout the prefill
// attention reads), rotated keys and plain values to rows start + t of the caches
// [B, Hkv, max_len, hd].  One thread per pair.
template <typename CacheT>
__global__ __launch_bounds__(256) void rope_prefill_kernel(const float* __restrict__ qkv, const float* __restrict__ cosine,
                                                           const float* __restrict__ sine, float* __restrict__ q_out,
                                                           CacheT* __restrict__ kcache, CacheT* __restrict__ vcache,
                                                           int B, int T, int H, int Hkv, int hd, int start, int max_len) {
  const int half = hd >> 1;
  const int heads = H + 2 * Hkv;
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (long long)B * T * heads * half) return;
  const int i = (int)(idx % half);
  const int head = (int)((idx / half) % heads);
  const long long row = idx / ((long long)half * heads);  // b * T + t
  const int b = (int)(row / T), t = (int)(row % T);
  const long long p = (long long)start + t;
  const float2 v = *reinterpret_cast<const float2*>(qkv + ((size_t)row * heads + head) * hd + 2 * i);
  if (head >= H + Hkv) {
    store_pair(vcache + (((size_t)b * Hkv + (head - H - Hkv)) * max_len + p) * hd + 2 * i, v);
    return;
  }
  const float c = cosine[p * half + i], s = sine[p * half + i];
  const float2 r = float2{v.x * c - v.y * s, v.x * s + v.y * c};
  if (head < H)
    *reinterpret_cast<float2*>(q_out + (((size_t)b * H + head) * T + t) * hd + 2 * i) = r;
  else
    store_pair(kcache + (((size_t)b * Hkv + (head - H)) * max_len + p) * hd + 2 * i, r);
}

// Single-query attention over cache rows 0 .. *pos for head_dim HD = 128 or 64.  Grid (B * Hkv, S): a
// workgroup of kWaves waves takes chunk s of the rows of one cache head and serves the R = H / Hkv
// query heads that share it, so a cache row is read once whatever R is.  Sixteen lanes share
// one cache row (a lane holds HD / 16 of its dimensions), so a wave works on four rows at a time
// and a workgroup on 4 kWaves, two rounds in flight; every 16-lane team keeps a reference
// exponent, denominator and weighted value sum of its rows per query head.  The teams are
// merged through LDS.  With S == 1 the result is normalised and written as bf16 [B, H * HD];
// otherwise (max, denominator, HD sums) go to `partial` for the merge kernel.  bf16 cache rows are
// widened to fp32 in registers; all arithmetic is fp32 either way.
//
// kStream (caches too large to stay in the last-level cache between steps): rows are fetched with
// non-temporal loads and dealt to the S chunks in blocks of 32 rows, round-robin, so the chunks of
// a cache head sweep one region of memory together instead of S regions far apart.  Without it
// a chunk is a contiguous run of rows and the loads are ordinary ones: a small cache (batch 1)
// stays in the last-level cache from one step to the next.
//
// kWaves = 16 is for launches with enough cache heads to occupy the chip on their own (S = 1): one
// 1024-thread workgroup per cache head writes the finished output, no partial results and no merge launch.

// One partial result of a row chunk: (maximum, denominator, 0, 0, HD weighted value sums); the
// sums start on a 16-byte boundary so that a GEMV prologue can fetch them with 128-bit loads.
constexpr int attn_partial_stride(int hd) { return 4 + hd; }
constexpr int kAttnPartialStride = attn_partial_stride(128);
// Which HD / 16 of a row's dimensions lane c of a team holds (DPL of them: 8, 4 or 2), and how it fetches them.
// 8 per lane, bf16 rows (256 B): 8c .. 8c+7, one 128-bit load.  8 per lane, fp32 rows (512 B): 4c .. 4c+3
// and 64+4c .. 64+4c+3, so each of a team's two 128-bit loads covers 256 contiguous bytes.  4 per lane:
// 4c .. 4c+3, one 128-bit (fp32) or 64-bit (bf16) load.  2 per lane: 2c, 2c+1, one 64-bit or 32-bit load.
template <typename CacheT, int HD> struct LaneDims {
  static_assert(HD == 128 || HD == 64 || HD == 32, "head_dim 128, 64 or 32");
  static constexpr int DPL = HD / 16;
  static constexpr bool split = sizeof(CacheT) == 4 && DPL == 8;
  static constexpr int per_lane = split ? 4 : DPL;   // the lane's first dimension = per_lane * c
  static constexpr int second = split ? 64 : 4;      // DPL == 8: its second four start this many dimensions later
  __device__ static __forceinline__ int dim(int c, int i) { return per_lane * c + (i < 4 ? i : second + i - 4); }
};
template <int DPL> struct KvRow {
  float v[DPL];
};
template <bool kStream, typename T>
__device__ __forceinline__ T load_kv(const T* p) {
  if constexpr (kStream) return __builtin_nontemporal_load(p);
  return *p;
}
__device__ __forceinline__ void widen2(uint32_t w, float& lo, float& hi) {  // two bf16 -> two fp32
  lo = __uint_as_float(w << 16);
  hi = __uint_as_float(w & 0xFFFF0000u);
}
// p: the lane's first dimension of the row
template <bool kStream, int HD>
__device__ __forceinline__ KvRow<HD / 16> load_row(const float* p) {
  using LD = LaneDims<float, HD>;
  KvRow<HD / 16> r;
  if constexpr (LD::DPL == 2) {
    const u32x2_t a = load_kv<kStream>(reinterpret_cast<const u32x2_t*>(p));
    r.v[0] = __uint_as_float(a.x); r.v[1] = __uint_as_float(a.y);
  } else {
    const u32x4_t a = load_kv<kStream>(reinterpret_cast<const u32x4_t*>(p));
    r.v[0] = __uint_as_float(a.x); r.v[1] = __uint_as_float(a.y); r.v[2] = __uint_as_float(a.z); r.v[3] = __uint_as_float(a.w);
    if constexpr (LD::DPL == 8) {
      const u32x4_t b = load_kv<kStream>(reinterpret_cast<const u32x4_t*>(p + LD::second));
      r.v[4] = __uint_as_float(b.x); r.v[5] = __uint_as_float(b.y); r.v[6] = __uint_as_float(b.z); r.v[7] = __uint_as_float(b.w);
    }
  }
  return r;
}
template <bool kStream, int HD>
__device__ __forceinline__ KvRow<HD / 16> load_row(const uint16_t* p) {
  KvRow<HD / 16> r;
  if constexpr (HD / 16 == 8) {
    const u32x4_t v = load_kv<kStream>(reinterpret_cast<const u32x4_t*>(p));
    widen2(v.x, r.v[0], r.v[1]); widen2(v.y, r.v[2], r.v[3]); widen2(v.z, r.v[4], r.v[5]); widen2(v.w, r.v[6], r.v[7]);
  } else if constexpr (HD / 16 == 4) {
    const u32x2_t v = load_kv<kStream>(reinterpret_cast<const u32x2_t*>(p));
    widen2(v.x, r.v[0], r.v[1]); widen2(v.y, r.v[2], r.v[3]);
  } else {
    widen2(load_kv<kStream>(reinterpret_cast<const uint32_t*>(p)), r.v[0], r.v[1]);
  }
  return r;
}
// the step's own key / value row into the cache; a bf16 cache rounds and hands the rounded values back (what a
// later read of the cache would give)
template <int HD>
__device__ __forceinline__ void store_row(float* p, KvRow<HD / 16>& r) {
  using LD = LaneDims<float, HD>;
  if constexpr (LD::DPL == 2) {
    *reinterpret_cast<float2*>(p) = float2{r.v[0], r.v[1]};
  } else {
    *reinterpret_cast<float4*>(p) = float4{r.v[0], r.v[1], r.v[2], r.v[3]};
    if constexpr (LD::DPL == 8) *reinterpret_cast<float4*>(p + LD::second) = float4{r.v[4], r.v[5], r.v[6], r.v[7]};
  }
}
template <int HD>
__device__ __forceinline__ void store_row(uint16_t* p, KvRow<HD / 16>& r) {
  if constexpr (HD / 16 == 8) {
    u32x4_t v;
    v.x = pack2_bf16(r.v[0], r.v[1]); v.y = pack2_bf16(r.v[2], r.v[3]);
    v.z = pack2_bf16(r.v[4], r.v[5]); v.w = pack2_bf16(r.v[6], r.v[7]);
    *reinterpret_cast<u32x4_t*>(p) = v;
    widen2(v.x, r.v[0], r.v[1]); widen2(v.y, r.v[2], r.v[3]); widen2(v.z, r.v[4], r.v[5]); widen2(v.w, r.v[6], r.v[7]);
  } else if constexpr (HD / 16 == 4) {
    u32x2_t v;
    v.x = pack2_bf16(r.v[0], r.v[1]); v.y = pack2_bf16(r.v[2], r.v[3]);
    *reinterpret_cast<u32x2_t*>(p) = v;
    widen2(v.x, r.v[0], r.v[1]); widen2(v.y, r.v[2], r.v[3]);
  } else {
    const uint32_t v = pack2_bf16(r.v[0], r.v[1]);
    *reinterpret_cast<uint32_t*>(p) = v;
    widen2(v, r.v[0], r.v[1]);
  }
}

// kStep: the whole attention part of a decode step in one launch.  `q` is then the fused
// projection output qkv [B, (H + 2 Hkv) * HD] (query heads, key heads, value heads): the
// workgroup rotates its R query heads itself (interleaved pairs, the tables' row *pos); the
// workgroup whose chunk holds row *pos also rotates the new key, writes it and the new value
// into the caches and attends to them from registers.  (Merging the S partial results in the
// workgroup that finishes last was tried and lost: the device-scope fences it needs write back
// and invalidate the XCD's L2, several microseconds per launch; the merge stays a launch.)

// 2^x by the hardware instruction (1 ulp); the softmax below keeps its running maximum and
// scores in the base-2 domain, scores pre-multiplied by log2(e)
__device__ __forceinline__ float exp2_hw(float x) { return __builtin_amdgcn_exp2f(x); }
constexpr float kLog2e = 1.4426950408889634f;

template <int R, typename CacheT, bool kStep, bool kStream, int kWaves, int HD>
__global__ __launch_bounds__(64 * kWaves) void attn_decode_kernel(const float* __restrict__ q, CacheT* __restrict__ kcache,
                                                          CacheT* __restrict__ vcache,
                                                          const long long* __restrict__ pos, int H, int Hkv, int max_len,
                                                          float scale, float* __restrict__ partial, uint16_t* __restrict__ out,
                                                          const float* __restrict__ cosine,
                                                          const float* __restrict__ sine) {
  static_assert(kWaves == 4 || kWaves == 16, "4 waves (row chunks, merged by a second kernel) or 16 (one workgroup per cache head)");
  constexpr int hd = HD;
  constexpr int kTeams = 4 * kWaves;
  using LD = LaneDims<CacheT, HD>;
  constexpr int DPL = LD::DPL;
  using Row = KvRow<DPL>;
  const int bk = blockIdx.x, S = gridDim.y, s = blockIdx.y;
  const int b = bk / Hkv, hk = bk % Hkv;
  const int bh0 = b * H + hk * R;  // first of the R query heads
  const int team = threadIdx.x >> 4, c = threadIdx.x & 15;  // teams of 16 lanes
  const long long p = min(max(*pos, 0LL), (long long)max_len - 1);  // held inside the cache (device data, unchecked by the host)
  const int rows = (int)p + 1;
  const int per = (rows + S - 1) / S;
  const int t_begin = s * per;
  int t_end = min(rows, t_begin + per);
  const int d0 = LD::per_lane * c;      // the lane's first dimension
  // kStep: cosines / sines of the lane's DPL / 2 pairs (interleaved pairs never straddle a lane's four)
  float cs[DPL / 2], sn[DPL / 2];
  const float* qkv_row = q + (size_t)b * (H + 2 * Hkv) * hd + d0;  // kStep only
  if (kStep && DPL == 2) {  // one pair per lane
    cs[0] = cosine[p * (hd / 2) + d0 / 2];
    sn[0] = sine[p * (hd / 2) + d0 / 2];
  } else if (kStep) {
#pragma unroll
    for (int h2 = 0; h2 < DPL / 4; ++h2) {
      const int pair0 = (d0 + h2 * LD::second) / 2;
      const float2 c2 = *reinterpret_cast<const float2*>(cosine + p * (hd / 2) + pair0);
      const float2 s2 = *reinterpret_cast<const float2*>(sine + p * (hd / 2) + pair0);
      cs[2 * h2] = c2.x; cs[2 * h2 + 1] = c2.y;
      sn[2 * h2] = s2.x; sn[2 * h2 + 1] = s2.y;
    }
  }
  auto rotate = [&](Row& r) {
#pragma unroll
    for (int i = 0; i < DPL / 2; ++i) {
      const float e = r.v[2 * i], o = r.v[2 * i + 1];
      r.v[2 * i] = e * cs[i] - o * sn[i];
      r.v[2 * i + 1] = e * sn[i] + o * cs[i];
    }
  };
  // a row of fp32 activations (queries, the step's own key and value) in the lane's dimensions
  auto load_act = [&](const float* src) {
    Row r;
    if constexpr (DPL == 2) {
      const float2 a = *reinterpret_cast<const float2*>(src);
      r.v[0] = a.x; r.v[1] = a.y;
    } else {
      const float4 a = *reinterpret_cast<const float4*>(src);
      r.v[0] = a.x; r.v[1] = a.y; r.v[2] = a.z; r.v[3] = a.w;
      if constexpr (DPL == 8) {
        const float4 b4 = *reinterpret_cast<const float4*>(src + LD::second);
        r.v[4] = b4.x; r.v[5] = b4.y; r.v[6] = b4.z; r.v[7] = b4.w;
      }
    }
    return r;
  };
  Row qr[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    qr[r] = load_act(kStep ? qkv_row + (size_t)(hk * R + r) * hd : q + (size_t)(bh0 + r) * hd + d0);
    if (kStep) rotate(qr[r]);
  }
  const CacheT* kbase = kcache + (size_t)bk * max_len * hd + d0;
  const CacheT* vbase = vcache + (size_t)bk * max_len * hd + d0;
  const float scale2 = scale * kLog2e;  // maxima and the partial results' maxima are base-2 exponents
  float m[R], l[R], acc[R][DPL];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    m[r] = -INFINITY;
    l[r] = 0.f;
#pragma unroll
    for (int i = 0; i < DPL; ++i) acc[r][i] = 0.f;
  }
  auto dot = [&](const Row& a, const Row& k) {
    float d = a.v[0] * k.v[0];
#pragma unroll
    for (int i = 1; i < DPL; ++i) d += a.v[i] * k.v[i];
    return team_sum16(d) * scale2;
  };
  // One cache row against the R queries.  One query head: the textbook running maximum.  Several: the
  // reference exponent m[r] of a team moves only when a new weight would pass 2^12 (always on the team's
  // first row: m = -inf gives +inf); then, for the whole wave, it becomes the running maximum and the sums
  // are rescaled.  Otherwise a row costs its dot product, one exponential and DPL + 1 FMAs per head instead of
  // two exponentials and twice the FMAs (12 % faster at R = 4 on a bf16 cache, 1 % slower at R = 1: the vote).
  auto row = [&](const Row& k, const Row& v) {
    if constexpr (R == 1) {
      const float sc = dot(qr[0], k);
      const float m_new = fmaxf(m[0], sc);
      const float corr = exp2_hw(m[0] - m_new), w = exp2_hw(sc - m_new);
      l[0] = l[0] * corr + w;
#pragma unroll
      for (int i = 0; i < DPL; ++i) acc[0][i] = acc[0][i] * corr + w * v.v[i];
      m[0] = m_new;
      return;
    }
    float sc[R];
    bool far = false;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      sc[r] = dot(qr[r], k);
      far |= !(sc[r] - m[r] <= 12.0f);
    }
    if (__builtin_amdgcn_ballot_w64(far) != 0) {
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const float m_new = fmaxf(m[r], sc[r]);
        const float corr = exp2_hw(m[r] - m_new);
        l[r] *= corr;
#pragma unroll
        for (int i = 0; i < DPL; ++i) acc[r][i] *= corr;
        m[r] = m_new;
      }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const float w = exp2_hw(sc[r] - m[r]);
      l[r] += w;
#pragma unroll
      for (int i = 0; i < DPL; ++i) acc[r][i] += w * v.v[i];
    }
  };
  // the step's own row: the chunk that owns it rotates the key, stores both and attends from registers (team 0)
  const bool own = kStream ? (((int)p / (2 * kTeams)) % S) == s : (t_begin <= (int)p && (int)p < t_end);
  if (kStep && own) {
    t_end = (int)p;
    if (team == 0) {
      Row kn = load_act(qkv_row + (size_t)(H + hk) * hd);
      Row vn = load_act(qkv_row + (size_t)(H + Hkv + hk) * hd);
      rotate(kn);
      store_row<HD>(kcache + ((size_t)bk * max_len + p) * hd + d0, kn);
      store_row<HD>(vcache + ((size_t)bk * max_len + p) * hd + d0, vn);
      row(kn, vn);
    }
  }
  // rows first .. limit-1 in steps of `stride`, two rows per team in flight
  const int first = kStream ? 2 * kTeams * s + team : t_begin + team;
  const int limit = kStream ? ((kStep && own) ? (int)p : rows) : t_end;
  const int stride = kStream ? 2 * kTeams * S : 2 * kTeams;
  for (int t = first; t < limit; t += stride) {
    if (t + kTeams < limit) {
      const Row k0 = load_row<kStream, HD>(kbase + (size_t)t * hd), k1 = load_row<kStream, HD>(kbase + (size_t)(t + kTeams) * hd);
      const Row v0 = load_row<kStream, HD>(vbase + (size_t)t * hd), v1 = load_row<kStream, HD>(vbase + (size_t)(t + kTeams) * hd);
      row(k0, v0);
      row(k1, v1);
    } else {
      const Row k0 = load_row<kStream, HD>(kbase + (size_t)t * hd), v0 = load_row<kStream, HD>(vbase + (size_t)t * hd);
      row(k0, v0);
    }
  }
  // Sixteen partial results meet in LDS: the 16 teams of a 4-wave workgroup, or the 16 waves of the large one,
  // whose four teams are first merged inside the wave (lanes 16 and 32 apart hold the same dimensions).
  if constexpr (kWaves == 16) {
#pragma unroll
    for (int off = 16; off <= 32; off <<= 1) {
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const float mo = __shfl_xor(m[r], off), lo = __shfl_xor(l[r], off);
        const float mn = fmaxf(m[r], mo);
        const float cs_ = m[r] == -INFINITY ? 0.f : exp2_hw(m[r] - mn);   // a team without rows weighs nothing
        const float co = mo == -INFINITY ? 0.f : exp2_hw(mo - mn);
        l[r] = l[r] * cs_ + lo * co;
#pragma unroll
        for (int i = 0; i < DPL; ++i) acc[r][i] = acc[r][i] * cs_ + __shfl_xor(acc[r][i], off) * co;
        m[r] = mn;
      }
    }
  }
  __shared__ float sm[R][16], sl[R][16];
  __shared__ float sacc[R][16][hd];
  const int entry = kWaves == 16 ? (int)(threadIdx.x >> 6) : team;
  if (kWaves == 4 || (threadIdx.x & 48) == 0) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      if (c == 0) { sm[r][entry] = m[r]; sl[r][entry] = l[r]; }
#pragma unroll
      for (int i = 0; i < DPL; ++i) sacc[r][entry][LD::dim(c, i)] = acc[r][i];
    }
  }
  __syncthreads();
  // wave w merges query heads w, w + kWaves, ...; two dimensions per lane from here on (the first HD / 2 lanes)
  const int lane = threadIdx.x & 63;
  const int dl = min(lane, hd / 2 - 1);
  for (int r = threadIdx.x >> 6; r < R; r += kWaves) {
    float M16 = sm[r][0];
#pragma unroll
    for (int w = 1; w < 16; ++w) M16 = fmaxf(M16, sm[r][w]);
    float L = 0.f;
    float2 A = float2{0.f, 0.f};
#pragma unroll
    for (int w = 0; w < 16; ++w) {
      const float cw = sm[r][w] == -INFINITY ? 0.f : exp2_hw(sm[r][w] - M16);
      L += sl[r][w] * cw;
      A.x += sacc[r][w][2 * dl] * cw;
      A.y += sacc[r][w][2 * dl + 1] * cw;
    }
    if (2 * lane >= hd) continue;
    if (S == 1 && out != nullptr) {
      const uint32_t o = pack2_bf16(A.x / L, A.y / L);
      reinterpret_cast<uint32_t*>(out + (size_t)(bh0 + r) * hd)[lane] = o;
    } else {  // several chunks, or a caller that merges them itself (out == nullptr)
      float* dst = partial + ((size_t)(bh0 + r) * S + s) * attn_partial_stride(hd);
      if (lane == 0) *reinterpret_cast<float4*>(dst) = float4{M16, L, 0.f, 0.f};
      *reinterpret_cast<float2*>(dst + 4 + 2 * lane) = A;
    }
  }
}

// merge of the S <= 16 partial results of attn_decode_kernel: one wave per (b, h).  Lane s
// fetches chunk s's maximum and denominator and every lane (the first HD / 2) its two dimensions of all
// chunks at once, so the kernel is one memory round trip, not one per chunk.
template <int HD>
__global__ __launch_bounds__(64) void attn_merge_kernel(const float* __restrict__ partial, int S,
                                                        uint16_t* __restrict__ out) {
  constexpr int hd = HD, stride = attn_partial_stride(HD);
  const int bh = blockIdx.x, lane = threadIdx.x;
  const int dl = min(lane, hd / 2 - 1);
  const float* src = partial + (size_t)bh * S * stride;
  const int sl = min(lane & 15, S - 1);
  const float2 ml = *reinterpret_cast<const float2*>(src + sl * stride);  // (max, denominator) of chunk lane % 16
  float2 a[16];
#pragma unroll
  for (int s = 0; s < 16; ++s)
    a[s] = *reinterpret_cast<const float2*>(src + min(s, S - 1) * stride + 4 + 2 * dl);
  float M = ml.x;
#pragma unroll
  for (int off = 8; off > 0; off >>= 1) M = fmaxf(M, __shfl_xor(M, off));
  const float mine = ml.x == -INFINITY ? 0.f : exp2_hw(ml.x - M);  // weight of chunk lane % 16 (base-2 maxima)
  float L = 0.f;
  float2 A = float2{0.f, 0.f};
#pragma unroll
  for (int s = 0; s < 16; ++s) {
    const float c = __shfl(mine, s), l = __shfl(ml.y, s);
    if (s < S) {
      L += l * c;
      A.x += a[s].x * c;
      A.y += a[s].y * c;
    }
  }
  if (2 * lane >= hd) return;
  const uint32_t o = pack2_bf16(A.x / L, A.y / L);
  reinterpret_cast<uint32_t*>(out + (size_t)bh * hd)[lane] = o;
}

// Greedy choice at the end of a decode step, one workgroup of 1024 threads per sequence:
// token = argmax(logits[b, 0..V)) (the lowest index among equal maxima, as torch.argmax),
// written to token[b] and to out[b, *step]; then hidden[b, :] = embedding[token, :], the next
// step's input.  With `advance` (two int64 counters, `step` may be one of them) the last workgroup
// to finish adds one to both; `ticket` is a zeroed word the kernel leaves zeroed.
__global__ __launch_bounds__(1024) void greedy_pick_kernel(const float* __restrict__ logits, int V, int ld,
                                                           const float* __restrict__ embedding, int D,
                                                           float* __restrict__ hidden, long long* __restrict__ token,
                                                           long long* __restrict__ out, int out_ld,
                                                           const long long* step, long long* advance,
                                                           unsigned* ticket) {
  const int b = blockIdx.x, t = threadIdx.x;
  const float* row = logits + (size_t)b * ld;
  float best = -INFINITY;
  int best_i = 0x7FFFFFFF;
  // four 128-bit loads per thread in flight; a thread meets its elements in ascending index
  // order, so a strict > keeps the first maximum
  const float4* row4 = reinterpret_cast<const float4*>(row);
  const int nvec = V >> 2;
  for (int base = 0; base < nvec; base += 4 * 1024) {
    float4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int idx = base + u * 1024 + t;
      v[u] = idx < nvec ? row4[idx] : float4{-INFINITY, -INFINITY, -INFINITY, -INFINITY};
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int i0 = 4 * (base + u * 1024 + t);
      if (v[u].x > best) { best = v[u].x; best_i = i0; }
      if (v[u].y > best) { best = v[u].y; best_i = i0 + 1; }
      if (v[u].z > best) { best = v[u].z; best_i = i0 + 2; }
      if (v[u].w > best) { best = v[u].w; best_i = i0 + 3; }
    }
  }
  if (4 * nvec + t < V) {  // the last V % 4 columns
    const float v = row[4 * nvec + t];
    if (v > best) { best = v; best_i = 4 * nvec + t; }
  }
  auto better = [](float v, int i, float bv, int bi) { return v > bv || (v == bv && i < bi); };
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float ov = __shfl_xor(best, off);
    const int oi = __shfl_xor(best_i, off);
    if (better(ov, oi, best, best_i)) { best = ov; best_i = oi; }
  }
  __shared__ float sv[16];
  __shared__ int si[16];
  __shared__ int chosen;
  if ((t & 63) == 0) { sv[t >> 6] = best; si[t >> 6] = best_i; }
  __syncthreads();
  if (t == 0) {
    float bv = sv[0];
    int bi = si[0];
    for (int w = 1; w < 16; ++w)
      if (better(sv[w], si[w], bv, bi)) { bv = sv[w]; bi = si[w]; }
    if (bi == 0x7FFFFFFF) bi = 0;  // a row of NaNs: torch picks the NaN; here index 0
    chosen = bi;
    token[b] = bi;
    // `step` may alias advance[0..1] (hence no __restrict__ on either): read it once, through a volatile
    // access so the load stays in front of the fence below
    const long long at = *reinterpret_cast<const volatile long long*>(step);
    out[(size_t)b * out_ld + min(max(at, 0LL), (long long)out_ld - 1)] = bi;  // device data: held inside the row
    if (advance) {
      // the step's two counters (cache row, output column) advance here, once every workgroup has read them:
      // the fence orders this thread's read of *step in front of its ticket, so the workgroup that draws the
      // last ticket writes after every read
      __threadfence();
      if (atomicAdd(ticket, 1u) == gridDim.x - 1) {
        advance[0] += 1;
        advance[1] += 1;
        *ticket = 0u;
      }
    }
  }
  __syncthreads();
  const float4* e4 = reinterpret_cast<const float4*>(embedding + (size_t)chosen * D);
  float4* h4 = reinterpret_cast<float4*>(hidden + (size_t)b * D);
  for (int i = t; i < D / 4; i += 1024) h4[i] = e4[i];
}

// Temperature / nucleus sampling at the end of a decode step (sample_next_token,
// src/ajllm/generation/sampling.py:8-22), one workgroup of 1024 threads per sequence; the tail (token, output column,
// embedding row, the step's counters) is greedy_pick_kernel's.
//   p = softmax(logits / temperature); with top_p < 1 the tokens are kept whose probability mass STRICTLY above them
//   (in descending order) is below top_p -- the reference's `cumulative - sorted_probabilities >= top_p` removed --
//   and the choice is drawn from the kept tokens in proportion to p.
// The draw is the inverse CDF over the kept tokens IN INDEX ORDER at u = uniforms[min(*step, uniform_rows - 1), b]
// (the reference draws with torch.multinomial from the sorted tokens: the same distribution from other random bits).
// Probabilities are compared and added as 40-bit fixed-point integers, so no result depends on the order of a sum:
// the same logits and the same u give the same token on every run.
//   1. row maximum; 2. Z = sum exp((l - max) / T) (a fixed order); weight w = exp(..) * 2^40 / Z as an integer;
//   3. top_p < 1: the float bits of exp(..) order the tokens; four radix passes (8 bits each, 256 bins of summed
//      weight) find the key where the weight above it is below top_p * 2^40 and the weight from it on is not: the
//      last kept token's key (equal keys are kept together);
//   4. the kept weight of every block of 1024 consecutive tokens (a wave per block), a serial walk to the block the
//      draw falls in, then the waves of that block and the lanes of that wave.
// kept (optional, [B]): the number of kept tokens, for tests.  Every walk over bins, blocks and tokens is a workgroup
// prefix sum: no thread loops over LDS words behind a branch.
constexpr int kSampleMaxBlocks = 1024;  // V <= 1024 * 1024
// exp for x <= 0 on the hardware's exp2 (a row is walked up to seven times by ONE workgroup, so the exponential's
// instruction count is the kernel's time: the library routine's thirty-odd instructions made a pass over 32000
// columns 6 us); the same value on every pass, which is all the radix passes need
__device__ __forceinline__ float sample_exp(float x) { return __builtin_amdgcn_exp2f(x * 1.44269504088896341f); }
__device__ __forceinline__ unsigned long long shfl_up_u64(unsigned long long v, int off) {
  const unsigned lo = __shfl_up((unsigned)v, off), hi = __shfl_up((unsigned)(v >> 32), off);
  return ((unsigned long long)hi << 32) | lo;
}
__device__ __forceinline__ unsigned long long wave_sum_u64(unsigned long long v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const unsigned lo = __shfl_xor((unsigned)v, off), hi = __shfl_xor((unsigned)(v >> 32), off);
    v += ((unsigned long long)hi << 32) | lo;
  }
  return v;
}
// inclusive prefix sum of one value per thread over a workgroup of 16 waves, in thread order (two barriers; the
// serial walks this replaces, one thread reading LDS word after word behind a branch, were most of the kernel's time)
__device__ __forceinline__ unsigned long long block_prefix_u64(unsigned long long v, unsigned long long* wave_total,
                                                              int lane, int wave) {
  unsigned long long incl = v;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const unsigned long long up = shfl_up_u64(incl, off);
    if (lane >= off) incl += up;
  }
  if (lane == 63) wave_total[wave] = incl;
  __syncthreads();
  unsigned long long base = 0ull;
#pragma unroll
  for (int w = 0; w < 15; ++w) base += w < wave ? wave_total[w] : 0ull;
  __syncthreads();
  return incl + base;
}
__global__ __launch_bounds__(1024) void sample_pick_kernel(const float* __restrict__ logits, int V, int ld,
                                                           float inv_temperature, float top_p,
                                                           const float* __restrict__ uniforms, int uniform_rows,
                                                           const float* __restrict__ embedding, int D,
                                                           float* __restrict__ hidden, long long* __restrict__ token,
                                                           long long* __restrict__ out, int out_ld, const long long* step,
                                                           long long* advance, unsigned* ticket, int* __restrict__ kept) {
  const int b = blockIdx.x, t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const float* row = logits + (size_t)b * ld;
  // 256 bins in sixteen copies each, one per lane & 15: the keys of a row crowd into a few bins (the exponent byte),
  // and lanes that add to one LDS word queue behind each other
  __shared__ float red[16];
  __shared__ unsigned long long bins[256 * 16];
  __shared__ unsigned long long block_weight[kSampleMaxBlocks];
  __shared__ unsigned long long wave_total[16];
  __shared__ unsigned long long sh_above, sh_rest, sh_total;
  __shared__ unsigned sh_byte;
  __shared__ int sh_block, sh_kept, chosen;
  __shared__ long long sh_at;
  __shared__ float sh_u;

  if (t == 0) {
    // `step` may alias advance[0..1]: read it once, through a volatile access (see greedy_pick_kernel)
    const long long at = *reinterpret_cast<const volatile long long*>(step);
    sh_at = at;
    sh_u = uniforms[(size_t)min(max(at, 0LL), (long long)uniform_rows - 1) * gridDim.x + b];
    sh_kept = 0;
  }

  // every element of the row once, four 128-bit loads per thread in flight (ld % 4 == 0, 16-byte aligned rows)
  const float4* row4 = reinterpret_cast<const float4*>(row);
  const int nvec = V >> 2;
  auto for_each = [&](auto&& fn) {
    for (int base = 0; base < nvec; base += 4 * 1024) {
      float4 v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int idx = base + u * 1024 + t;
        v[u] = idx < nvec ? row4[idx] : float4{-INFINITY, -INFINITY, -INFINITY, -INFINITY};
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        if (base + u * 1024 + t < nvec) {
          fn(v[u].x);
          fn(v[u].y);
          fn(v[u].z);
          fn(v[u].w);
        }
      }
    }
    if (4 * nvec + t < V) fn(row[4 * nvec + t]);  // the last V % 4 columns
  };

  // ---- 1. row maximum
  float m = -INFINITY;
  for_each([&](float l) { m = fmaxf(m, l); });
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off));
  if (lane == 0) red[wave] = m;
  __syncthreads();
  m = red[0];
#pragma unroll
  for (int w = 1; w < 16; ++w) m = fmaxf(m, red[w]);
  __syncthreads();
  // ---- 2. normaliser, summed in a fixed order (a thread's elements in sequence, a fixed tree, waves in order)
  float z = 0.f;
  for_each([&](float l) { z += sample_exp((l - m) * inv_temperature); });
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) z += __shfl_xor(z, off);
  if (lane == 0) red[wave] = z;
  __syncthreads();
  z = red[0];
#pragma unroll
  for (int w = 1; w < 16; ++w) z += red[w];
  const float to_fixed = 0x1p40f / z;
  auto weight_of = [&](float e) -> unsigned long long { return (unsigned long long)(e * to_fixed); };

  // ---- 3. the key of the last kept token
  unsigned threshold = 0u;  // keep keys >= threshold
  if (top_p < 1.0f) {
    const unsigned long long want = (unsigned long long)((double)top_p * 0x1p40);
    unsigned prefix = 0u, prefix_mask = 0u;
    unsigned long long above = 0ull;  // weight of the keys whose leading bytes are above the prefix
    unsigned long long* my_bins = bins + (lane & 15);
    for (int pass = 0; pass < 4; ++pass) {
      const int shift = 24 - 8 * pass;
      for (int i = t; i < 256 * 16; i += 1024) bins[i] = 0ull;
      __syncthreads();
      for_each([&](float l) {
        const float e = sample_exp((l - m) * inv_temperature);
        const unsigned key = __float_as_uint(e);
        if ((key & prefix_mask) == prefix) atomicAdd(&my_bins[((key >> shift) & 255u) << 4], weight_of(e));
      });
      __syncthreads();
      // thread q' < 256 takes byte 255 - q' (descending), so a prefix sum in thread order is the weight from that
      // byte up; the byte where it first reaches the wanted weight is the next digit of the key.  If it never does
      // (rounding at top_p ~ 1), byte 0: everything is kept.
      unsigned long long mine = 0ull;
      if (t < 256) {
#pragma unroll
        for (int w = 0; w < 16; ++w) mine += bins[(255 - t) * 16 + w];
      }
      const unsigned long long from_here = above + block_prefix_u64(mine, wave_total, lane, wave);
      if (t < 256) {
        const unsigned long long over = from_here - mine;  // weight strictly above this byte
        if ((over < want && from_here >= want) || (t == 255 && from_here < want)) {
          sh_byte = (unsigned)(255 - t);
          sh_above = over;
        }
      }
      __syncthreads();
      prefix |= sh_byte << shift;
      prefix_mask |= 255u << shift;
      above = sh_above;
    }
    threshold = prefix;
  }

  // ---- 4. kept weight per block of 1024 consecutive tokens (wave w: blocks w, w + 16, ...)
  const int blocks = (V + 1023) >> 10;
  int kept_here = 0;
  for (int c = wave; c < blocks; c += 16) {
    unsigned long long w_sum = 0ull;
    auto take = [&](int j, float l) {
      if (j < V) {
        const float e = sample_exp((l - m) * inv_temperature);
        if (__float_as_uint(e) >= threshold) {
          w_sum += weight_of(e);
          ++kept_here;
        }
      }
    };
    float4 v[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int j = (c << 10) + (i * 64 + lane) * 4;
      v[i] = j + 3 < 4 * nvec ? row4[j >> 2] : float4{j < V ? row[j] : 0.f, j + 1 < V ? row[j + 1] : 0.f,
                                                        j + 2 < V ? row[j + 2] : 0.f, j + 3 < V ? row[j + 3] : 0.f};
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int j = (c << 10) + (i * 64 + lane) * 4;
      take(j, v[i].x);
      take(j + 1, v[i].y);
      take(j + 2, v[i].z);
      take(j + 3, v[i].w);
    }
    w_sum = wave_sum_u64(w_sum);
    if (lane == 0) block_weight[c] = w_sum;
  }
  if (kept) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) kept_here += __shfl_xor(kept_here, off);
    if (lane == 0) atomicAdd(&sh_kept, kept_here);
  }
  __syncthreads();
  // ---- the block the draw falls in: thread c < blocks holds block c's weight; the draw is an integer in [0, total)
  {
    const unsigned long long mine = t < blocks ? block_weight[t] : 0ull;
    const unsigned long long upto = block_prefix_u64(mine, wave_total, lane, wave);
    if (t == 1023) sh_total = upto;
    if (t == 0) {
      sh_block = blocks - 1;
      sh_rest = 0ull;
      if (kept) kept[b] = sh_kept;
    }
    __syncthreads();
    const unsigned long long total = sh_total;  // >= 1: the maximum's weight alone is 2^40 / Z >= 2^40 / V
    unsigned long long draw = (unsigned long long)((double)fminf(fmaxf(sh_u, 0.f), 1.f) * (double)total);
    if (draw >= total) draw = total - 1;
    if (t < blocks && draw >= upto - mine && draw < upto) {
      sh_block = t;
      sh_rest = draw - (upto - mine);
    }
    __syncthreads();
  }
  // ---- the token inside the block, the same way: thread i holds token 1024 block + i
  {
    const int j = (sh_block << 10) + t;
    unsigned long long mine = 0ull;
    if (j < V) {
      const float e = sample_exp((row[j] - m) * inv_temperature);
      if (__float_as_uint(e) >= threshold) mine = weight_of(e);
    }
    const unsigned long long upto = block_prefix_u64(mine, wave_total, lane, wave);
    const unsigned long long rest = sh_rest;
    if (t == 0) chosen = min(sh_block << 10, V - 1);
    __syncthreads();
    if (rest >= upto - mine && rest < upto) chosen = j;
    __syncthreads();
  }
  if (t == 0) {
    const int bi = min(chosen, V - 1);
    chosen = bi;
    token[b] = bi;
    out[(size_t)b * out_ld + min(max(sh_at, 0LL), (long long)out_ld - 1)] = bi;
    if (advance) {
      __threadfence();
      if (atomicAdd(ticket, 1u) == gridDim.x - 1) {
        advance[0] += 1;
        advance[1] += 1;
        *ticket = 0u;
      }
    }
  }
  __syncthreads();
  if (embedding) {
    const float4* e4 = reinterpret_cast<const float4*>(embedding + (size_t)chosen * D);
    float4* h4 = reinterpret_cast<float4*>(hidden + (size_t)b * D);
    for (int i = t; i < D / 4; i += 1024) h4[i] = e4[i];
  }
}

// ab [B, 2F] fp32 (gate projection, then up projection) -> out[b, f] = bf16( silu(a) * u ),
// silu(a) = a * sigmoid(a).  F % 2 == 0; one thread per pair.
__global__ __launch_bounds__(256) void swiglu_kernel(const float* __restrict__ ab, uint16_t* __restrict__ out, int B,
                                                     int F) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  const int half = F >> 1;
  if (idx >= (long long)B * half) return;
  const int b = (int)(idx / half), i = (int)(idx % half);
  const float2 a = *reinterpret_cast<const float2*>(ab + (size_t)b * 2 * F + 2 * i);
  const float2 u = *reinterpret_cast<const float2*>(ab + (size_t)b * 2 * F + F + 2 * i);
  const float x0 = a.x * (1.0f / (1.0f + expf(-a.x))) * u.x;
  const float x1 = a.y * (1.0f / (1.0f + expf(-a.y))) * u.y;
  reinterpret_cast<uint32_t*>(out + (size_t)b * F)[i] = pack2_bf16(x0, x1);
}

}  // namespace ajq
