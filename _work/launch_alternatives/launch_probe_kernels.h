// Measurement probes around the launch cost of the decode GEMV (bench-only: built into
// libajq_bench.so, never into the operator library).
//
// A 4096 x 4096 int4 matrix is 8.7 MB: at the HBM rate it is read in 1.1 us, while a kernel launch
// in a HIP-graph chain costs more than that before the first byte arrives.  The probes measure the
// alternatives to "one launch per matrix" for a chain of DEPENDENT matrix-vector products (stage
// s + 1 multiplies the output of stage s):
//
//  * chain_kernel: ONE launch for S stages.  256 workgroups (one per CU) of 8 compute waves
//    plus service waves.  The compute waves keep the weights of the next D - 1 stages in flight in
//    registers; the service waves exchange the activations between the workgroups through device
//    memory with agent-scope (L2-bypassing) loads and stores, either behind a flag per producer
//    (kFlags) or as 8-byte records that carry a stamp (kStamped: no separate flag round trip), in
//    one copy or in one copy per XCD.  Every wait is bounded: a spin limit sets an error word and
//    lets the wave go on, so the grid always drains.
//  * pingpong_kernel: one-way latency of such an exchange between two workgroups.
//  * prefetch_kernel / gemv_prefetch_kernel: pulling the next matrix towards the caches while the
//    current GEMV runs, from a second graph branch or from inside the GEMV kernel.
#pragma once
#include "ajq_common.h"

namespace ajq {
namespace probe {

constexpr int K = 4096, N = 4096, G = K / 128, NT = N / 16;
constexpr int kWaves = 8, kTpw = 4;
constexpr size_t kWqStage = (size_t)NT * G * 64;    // u32x4 per matrix
constexpr size_t kMetaStage = (size_t)NT * G * 16;  // u32 per matrix
constexpr double kBytesPerStage = 8732672.0;        // algorithmic bytes of one W4 GEMV, M = 1
constexpr int kNoDependency = 0, kFlags = 1, kStamped = 2;

struct ChainParams {
  const u32x4_t* wq;     // [S][NT][G][64]
  const uint32_t* meta;  // [S][NT][G][16]
  uint32_t* xbuf;        // kFlags: [(S + 1)][R][K / 2] bf16 pairs; kStamped: the same count of 8-byte records
  uint32_t* flags;       // [(S + 1)][R][256]
  uint32_t* err;
  int S, s0, epoch, spin_cap;
};

__device__ __forceinline__ uint32_t ld_u32(const uint32_t* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ unsigned long long ld_u64(const unsigned long long* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_u32(uint32_t* p, uint32_t v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_u64(unsigned long long* p, unsigned long long v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// MODE: kNoDependency / kFlags / kStamped; D: weight batches in flight per compute wave;
// kWeights = false reads matrix 0 every stage (cache hits: the exchange alone is timed);
// NSERV service waves share the exchange; R copies of the exchange buffers (1, or 8 = one per XCD).
template <int MODE, int D, bool kWeights, int NSERV, int R>
__global__ __launch_bounds__(64 * (kWaves + NSERV)) void chain_kernel(ChainParams p) {
  __shared__ u32x4_t xs4[K / 8];  // the stage's activations, bf16
  __shared__ float red[kWaves * 16];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wg = blockIdx.x;
  const int nl = lane & 15, kc = lane >> 4;
  const int copy = R == 1 ? 0 : (wg & (R - 1));
  constexpr int kEntries = K / 2;            // exchange entries per stage (bf16 pairs)
  constexpr int kPart = kEntries / NSERV;    // entries one service wave brings in
  constexpr int kPerLane = kPart / 64;

  if (wave >= kWaves) {
    // ---------------- service waves: they have no weight loads in flight, so their exchange
    // loads return without queueing behind a prefetch (vector loads return in issue order)
    const int j = wave - kWaves;
    for (int s = p.s0; s < p.s0 + p.S; ++s) {
      uint32_t* xs = reinterpret_cast<uint32_t*>(xs4) + j * kPart;
      if (MODE == kStamped) {
        const unsigned long long* src =
            reinterpret_cast<const unsigned long long*>(p.xbuf) + ((size_t)s * R + copy) * kEntries + j * kPart;
        const uint32_t want = (uint32_t)p.epoch * 65536u + (uint32_t)s;
        int spins = 0;
        for (;;) {
          bool ok = true;
          uint32_t v[kPerLane];
#pragma unroll
          for (int i = 0; i < kPerLane; ++i) {
            const unsigned long long e = ld_u64(src + i * 64 + lane);
            v[i] = (uint32_t)e;
            ok = ok && ((uint32_t)(e >> 32) == want);
          }
          if (__all(ok) || s == p.s0) {
#pragma unroll
            for (int i = 0; i < kPerLane; ++i) xs[i * 64 + lane] = v[i];
            break;
          }
          if (++spins > p.spin_cap) {  // bounded wait: flag the error and go on with what is there
            if (lane == 0) atomicOr(p.err, 1u);
            break;
          }
        }
      } else {
        if (MODE == kFlags && s > p.s0) {
          // flags of the producers of this wave's part
          const uint32_t* f = p.flags + ((size_t)s * R + copy) * 256 + j * (256 / NSERV);
          constexpr int kFlagLoads = 4 / NSERV > 0 ? 4 / NSERV : 1;
          int spins = 0;
          for (;;) {
            bool ok = true;
            uint32_t fv[kFlagLoads];
#pragma unroll
            for (int i = 0; i < kFlagLoads; ++i) fv[i] = ld_u32(f + i * 64 + lane);
#pragma unroll
            for (int i = 0; i < kFlagLoads; ++i) ok = ok && fv[i] == (uint32_t)p.epoch;
            if (__all(ok)) break;
            if (++spins > p.spin_cap) {
              if (lane == 0) atomicOr(p.err, 1u);
              break;
            }
          }
        }
        const uint32_t* src = p.xbuf + ((size_t)(MODE == kNoDependency ? p.s0 : s) * R + copy) * kEntries + j * kPart;
        uint32_t v[kPerLane];
#pragma unroll
        for (int i = 0; i < kPerLane; ++i) v[i] = ld_u32(src + i * 64 + lane);
#pragma unroll
        for (int i = 0; i < kPerLane; ++i) xs[i * 64 + lane] = v[i];
      }
      __syncthreads();  // B: activations staged
      __syncthreads();  // A: the compute waves' partial sums are in LDS
      if (j != 0) continue;
      float sum = 0.f;
      if (lane < 16) {
#pragma unroll
        for (int w = 0; w < kWaves; ++w) sum += red[w * 16 + lane];
      }
      const uint32_t b = f32_to_bf16_rne(sum);
      const int i = lane & 7, r = lane >> 3;
      const uint32_t pair = __shfl(b, 2 * i) | (__shfl(b, 2 * i + 1) << 16);
      if (MODE == kStamped) {
        unsigned long long* dst = reinterpret_cast<unsigned long long*>(p.xbuf) + ((size_t)(s + 1) * R + r) * kEntries;
        const uint32_t stamp = (uint32_t)p.epoch * 65536u + (uint32_t)(s + 1);
        if (r < R) st_u64(dst + wg * 8 + i, (unsigned long long)pair | ((unsigned long long)stamp << 32));
      } else {
        uint32_t* dst = p.xbuf + ((size_t)(s + 1) * R + r) * kEntries;
        if (r < R) st_u32(dst + wg * 8 + i, pair);
        if (MODE == kFlags) {
          asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the outputs are acknowledged before the flag leaves
          if (lane < R) st_u32(p.flags + ((size_t)(s + 1) * R + lane) * 256 + wg, (uint32_t)p.epoch);
        }
      }
    }
    return;
  }

  // ---------------- compute waves
  struct Batch {
    u32x4_t w[kTpw];
    uint32_t m[kTpw];
  };
  Batch ring[D];
  const int s_end = p.s0 + p.S;
  auto load = [&](Batch& b, int s) {
    s = min(s, s_end - 1);
    if (!kWeights) s = 0;
    const u32x4_t* wt = p.wq + (size_t)s * kWqStage + ((size_t)wg * G + wave * kTpw) * 64 + lane;
    const uint32_t* mt = p.meta + (size_t)s * kMetaStage + ((size_t)wg * G + wave * kTpw) * 16 + nl;
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int t = 0; t < kTpw; ++t) b.w[t] = __builtin_nontemporal_load(wt + t * 64);
#pragma unroll
    for (int t = 0; t < kTpw; ++t) b.m[t] = mt[t * 16];
    __builtin_amdgcn_sched_barrier(0);
  };
  const u32x4_t ones = {0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};
  auto compute = [&](Batch& b) {
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int t = 0; t < kTpw; ++t) {
      const float sc = f16_bits_to_f32(b.m[t] & 0xFFFFu), zc = f16_bits_to_f32(b.m[t] >> 16);
      f32x4_t part = {0.f, 0.f, 0.f, 0.f}, asum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const u32x4_t a = xs4[(wave * kTpw + t) * 16 + 4 * j + kc];
        part = mfma16(a, w4_to_bf16_biased(b.w[t][j]), part);
        asum = mfma16(a, ones, asum);
      }
      acc += sc * (part - zc * asum);
    }
    if (kc == 0) red[wave * 16 + nl] = acc[0];
  };
#pragma unroll
  for (int d = 0; d < D - 1; ++d) load(ring[d], p.s0 + d);
  for (int s = p.s0; s < s_end; s += D) {
#pragma unroll
    for (int d = 0; d < D; ++d) {
      if (s + d < s_end) {  // uniform
        load(ring[(d + D - 1) % D], s + d + D - 1);
        __syncthreads();  // B
        compute(ring[d]);
        __syncthreads();  // A
      }
    }
  }
}

// One-way latency between two workgroups: block a stores a sequence number, block b answers.
__global__ void pingpong_kernel(uint32_t* fa, uint32_t* fb, int a, int b, int iters, int base, uint32_t* err) {
  if ((int)blockIdx.x != a && (int)blockIdx.x != b) return;
  if (threadIdx.x != 0) return;
  const bool is_a = (int)blockIdx.x == a;
  for (int i = 1; i <= iters; ++i) {
    const uint32_t v = (uint32_t)(base + i);
    int spins = 0;
    if (is_a) {
      st_u32(fa, v);
      while (ld_u32(fb) != v)
        if (++spins > 2000000) { atomicOr(err, 2u); return; }
    } else {
      while (ld_u32(fa) != v)
        if (++spins > 2000000) { atomicOr(err, 2u); return; }
      st_u32(fb, v);
    }
  }
}

// Reads the bytes workgroup blockIdx.x of the GEMV reads (same workgroup -> same XCD), default cache policy.
__global__ __launch_bounds__(512) void prefetch_kernel(const u32x4_t* __restrict__ wq, const uint32_t* __restrict__ meta,
                                                       uint32_t* sink) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const u32x4_t* wt = wq + ((size_t)blockIdx.x * G + wave * kTpw) * 64 + lane;
  u32x4_t v[kTpw];
#pragma unroll
  for (int t = 0; t < kTpw; ++t) v[t] = wt[t * 64];
  const uint32_t m = meta[(size_t)blockIdx.x * G * 16 + threadIdx.x % (G * 16)];
  uint32_t acc = m;
#pragma unroll
  for (int t = 0; t < kTpw; ++t) acc ^= v[t].x ^ v[t].y ^ v[t].z ^ v[t].w;
  if (acc == 0x9E3779B9u && m == 0x12345u) sink[0] = acc;  // never true for the probe's data; keeps the loads
}

// A plain GEMV (M = 1, W4, 8 waves x 4 groups) that can also issue the next matrix's loads
// right behind its own and consume them at its very end.
template <bool kPrefetch>
__global__ __launch_bounds__(512) void gemv_prefetch_kernel(const u32x4_t* __restrict__ wq, const uint32_t* __restrict__ meta,
                                                            const u32x4_t* __restrict__ wq_next, const uint16_t* __restrict__ x,
                                                            uint16_t* __restrict__ y, uint32_t* sink) {
  __shared__ u32x4_t xs4[K / 8];
  __shared__ float red[kWaves * 16];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int nl = lane & 15, kc = lane >> 4;
  const u32x4_t* wt = wq + ((size_t)blockIdx.x * G + wave * kTpw) * 64 + lane;
  const uint32_t* mt = meta + ((size_t)blockIdx.x * G + wave * kTpw) * 16 + nl;
  u32x4_t w[kTpw], nx[kTpw];
  uint32_t m[kTpw];
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int t = 0; t < kTpw; ++t) w[t] = __builtin_nontemporal_load(wt + t * 64);
  const u32x4_t xv = reinterpret_cast<const u32x4_t*>(x)[wave * 64 + lane];
#pragma unroll
  for (int t = 0; t < kTpw; ++t) m[t] = mt[t * 16];
  if (kPrefetch) {
    const u32x4_t* wn = wq_next + ((size_t)blockIdx.x * G + wave * kTpw) * 64 + lane;
#pragma unroll
    for (int t = 0; t < kTpw; ++t) nx[t] = wn[t * 64];
  }
  __builtin_amdgcn_sched_barrier(0);
  xs4[wave * 64 + lane] = xv;  // the wave's own k-slice; LDS operations of one wave execute in order
  const u32x4_t ones = {0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};
  f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int t = 0; t < kTpw; ++t) {
    const float sc = f16_bits_to_f32(m[t] & 0xFFFFu), zc = f16_bits_to_f32(m[t] >> 16);
    f32x4_t part = {0.f, 0.f, 0.f, 0.f}, asum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const u32x4_t a = xs4[(wave * kTpw + t) * 16 + 4 * j + kc];
      part = mfma16(a, w4_to_bf16_biased(w[t][j]), part);
      asum = mfma16(a, ones, asum);
    }
    acc += sc * (part - zc * asum);
  }
  if (kc == 0) red[wave * 16 + nl] = acc[0];
  __syncthreads();
  if (wave == 0 && lane < 16) {
    float sum = 0.f;
#pragma unroll
    for (int v = 0; v < kWaves; ++v) sum += red[v * 16 + lane];
    y[blockIdx.x * 16 + lane] = f32_to_bf16_rne(sum);
  }
  if (kPrefetch) {
    uint32_t a2 = 0;
#pragma unroll
    for (int t = 0; t < kTpw; ++t) a2 ^= nx[t].x ^ nx[t].y ^ nx[t].z ^ nx[t].w;
    if (a2 == 0x9E3779B9u) sink[1] = a2;
  }
}

__global__ void fill_hash_kernel(uint32_t* p, size_t n, uint32_t seed) {
  size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
  for (; i < n; i += (size_t)gridDim.x * blockDim.x) {
    uint32_t h = (uint32_t)i * 2654435761u + seed;
    h ^= h >> 15; h *= 2246822519u; h ^= h >> 13; h *= 3266489917u; h ^= h >> 16;
    p[i] = h;
  }
}
__global__ void fill_const_kernel(uint32_t* p, size_t n, uint32_t v) {
  size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
  for (; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = v;
}

}  // namespace probe
}  // namespace ajq
