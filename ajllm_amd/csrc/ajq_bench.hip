// libajq_bench.so: measurement probes for bench.py.  Nothing here is an operator; the operator
// library (libajq.so) does not contain or need any of it.  Unlike the operators these entry points
// allocate their own device memory and synchronise.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>
#include <math.h>

#include <vector>

#include "../../include/ajq_bench.h"
#include "ajq_common.h"
#include "gemv_kernels.h"
#include "probe_kernels.h"
#include "launch_probe_kernels.h"

using namespace ajq;
using namespace ajq::probe;

namespace {

thread_local char g_error[512] = "";

int fail(int status, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return status;
}

#define HIP_OR_FAIL(call)                                                                              \
  do {                                                                                                 \
    hipError_t e_ = (call);                                                                            \
    if (e_ != hipSuccess) return fail(-5, "%s: %s (%s:%d)", #call, hipGetErrorString(e_), __FILE__, __LINE__); \
  } while (0)

struct Buffers {
  uint32_t *wq = nullptr, *meta = nullptr, *xbuf = nullptr, *flags = nullptr, *err = nullptr, *sink = nullptr;
  uint16_t *x = nullptr, *y = nullptr;
  int S = 0;
  ~Buffers() {
    for (void* ptr : {(void*)wq, (void*)meta, (void*)xbuf, (void*)flags, (void*)err, (void*)sink, (void*)x, (void*)y})
      (void)hipFree(ptr);
  }
};

struct Results {
  ajqb_result* out;
  int cap, n = 0;
  void add(const char* name, double us, int matches, unsigned err, bool moves_a_matrix = true) {
    if (n >= cap) return;
    ajqb_result& r = out[n++];
    snprintf(r.name, sizeof(r.name), "%s", name);
    r.us_per_stage = us;
    r.frac_hbm_peak = (moves_a_matrix && us > 0) ? kBytesPerStage / us * 1e-3 / 8000.0 : 0.0;
    r.matches_reference = matches;
    r.error_word = (int)err;
  }
};

// bf16 pairs of a fixed pattern: the chain's first activations
std::vector<uint32_t> first_activations() {
  std::vector<uint32_t> x0(K / 2);
  auto bf = [](float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
  };
  for (int i = 0; i < K / 2; ++i) x0[i] = bf(sinf(0.37f * (2 * i))) | (bf(sinf(0.37f * (2 * i + 1))) << 16);
  return x0;
}

int init_exchange(Buffers& b, int R, bool stamped) {
  const size_t bytes = (size_t)(b.S + 1) * 8 * (K / 2) * 8;
  HIP_OR_FAIL(hipMemset(b.xbuf, 0, bytes));
  HIP_OR_FAIL(hipMemset(b.flags, 0, (size_t)(b.S + 1) * 8 * 256 * 4));
  HIP_OR_FAIL(hipMemset(b.err, 0, 4));
  const std::vector<uint32_t> x0 = first_activations();
  for (int r = 0; r < R; ++r) {
    if (stamped) {
      std::vector<unsigned long long> x0s(K / 2);
      for (int i = 0; i < K / 2; ++i) x0s[i] = x0[i];
      HIP_OR_FAIL(hipMemcpy(reinterpret_cast<unsigned long long*>(b.xbuf) + (size_t)r * (K / 2), x0s.data(), K * 4,
                            hipMemcpyHostToDevice));
    } else {
      HIP_OR_FAIL(hipMemcpy(b.xbuf + (size_t)r * (K / 2), x0.data(), K * 2, hipMemcpyHostToDevice));
    }
  }
  return 0;
}

int g_epoch = 1;

// Times `reps` passes over the S stages; per_stage_launches runs the same kernel as S launches of
// one stage each (plain stream order supplies the dependency).  `last` receives the last stage's output.
template <int MODE, int D, bool kWeights, int NSERV, int R>
int run_chain(Buffers& b, int reps, bool per_stage_launches, double* us, unsigned* err, std::vector<uint32_t>* last) {
  ChainParams p{};
  p.wq = reinterpret_cast<const u32x4_t*>(b.wq);
  p.meta = b.meta;
  p.xbuf = b.xbuf;
  p.flags = b.flags;
  p.err = b.err;
  p.spin_cap = 200000;
  const int S = b.S;
  auto once = [&]() {
    p.epoch = ++g_epoch;
    if (per_stage_launches) {
      for (int s = 0; s < S; ++s) {
        ChainParams q = p;
        q.S = 1;
        q.s0 = s;
        hipLaunchKernelGGL((chain_kernel<MODE, D, kWeights, NSERV, R>), dim3(256), dim3(64 * (kWaves + NSERV)), 0, 0, q);
      }
    } else {
      p.S = S;
      p.s0 = 0;
      hipLaunchKernelGGL((chain_kernel<MODE, D, kWeights, NSERV, R>), dim3(256), dim3(64 * (kWaves + NSERV)), 0, 0, p);
    }
  };
  hipEvent_t e0, e1;
  HIP_OR_FAIL(hipEventCreate(&e0));
  HIP_OR_FAIL(hipEventCreate(&e1));
  for (int i = 0; i < 3; ++i) once();
  HIP_OR_FAIL(hipDeviceSynchronize());
  HIP_OR_FAIL(hipEventRecord(e0, 0));
  for (int i = 0; i < reps; ++i) once();
  HIP_OR_FAIL(hipEventRecord(e1, 0));
  HIP_OR_FAIL(hipEventSynchronize(e1));
  float ms = 0;
  HIP_OR_FAIL(hipEventElapsedTime(&ms, e0, e1));
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  *us = ms * 1e3 / reps / S;
  HIP_OR_FAIL(hipMemcpy(err, b.err, 4, hipMemcpyDeviceToHost));
  if (last) {
    const bool stamped = MODE == kStamped;
    const int words = stamped ? K : K / 2;
    std::vector<uint32_t> raw(words);
    HIP_OR_FAIL(hipMemcpy(raw.data(), b.xbuf + (size_t)S * R * words, (size_t)words * 4, hipMemcpyDeviceToHost));
    last->resize(K / 2);
    for (int i = 0; i < K / 2; ++i) (*last)[i] = stamped ? raw[2 * i] : raw[i];
  }
  return 0;
}

void launch_gemv(Buffers& b, int i, hipStream_t st) {
  constexpr size_t lds = gemv_lds_bytes(8, 4, 1);
  hipLaunchKernelGGL((dequant_gemv_kernel<8, 4, 1, true, true>), dim3(NT), dim3(512), lds, st,
                     reinterpret_cast<const u32x4_t*>(b.wq) + (size_t)i * kWqStage, b.meta + (size_t)i * kMetaStage,
                     b.x, K, 1, N, (void*)(b.y + (size_t)i * N), (const uint16_t*)nullptr);
}
void launch_prefetch(Buffers& b, int i, hipStream_t st) {
  hipLaunchKernelGGL(prefetch_kernel, dim3(NT), dim3(512), 0, st,
                     reinterpret_cast<const u32x4_t*>(b.wq) + (size_t)i * kWqStage, b.meta + (size_t)i * kMetaStage, b.sink);
}
template <bool kPrefetch>
void launch_simple(Buffers& b, int i, hipStream_t st) {
  hipLaunchKernelGGL((gemv_prefetch_kernel<kPrefetch>), dim3(NT), dim3(512), 0, st,
                     reinterpret_cast<const u32x4_t*>(b.wq) + (size_t)i * kWqStage, b.meta + (size_t)i * kMetaStage,
                     reinterpret_cast<const u32x4_t*>(b.wq) + (size_t)((i + 1) % b.S) * kWqStage, b.x,
                     b.y + (size_t)i * N, b.sink);
}

enum GraphMode { kGemvOnly, kPrefetchOnly, kPacedBranch, kUnpacedBranch, kSimple, kSimplePrefetch };

// One HIP graph over the S matrices, replayed `reps` times.
int run_graph(Buffers& b, GraphMode mode, int reps, double* us) {
  const int S = b.S;
  hipStream_t s1, s2;
  HIP_OR_FAIL(hipStreamCreateWithFlags(&s1, hipStreamNonBlocking));
  HIP_OR_FAIL(hipStreamCreateWithFlags(&s2, hipStreamNonBlocking));
  std::vector<hipEvent_t> ev(S + 2);
  for (auto& e : ev) HIP_OR_FAIL(hipEventCreateWithFlags(&e, hipEventDisableTiming));
  hipGraph_t graph;
  hipGraphExec_t exec;
  HIP_OR_FAIL(hipStreamBeginCapture(s1, hipStreamCaptureModeGlobal));
  bool forked = false;
  for (int i = 0; i < S; ++i) {
    switch (mode) {
      case kGemvOnly: launch_gemv(b, i, s1); break;
      case kPrefetchOnly: launch_prefetch(b, i, s1); break;
      case kSimple: launch_simple<false>(b, i, s1); break;
      case kSimplePrefetch: launch_simple<true>(b, i, s1); break;
      case kPacedBranch:
        if (i + 1 < S) {  // the prefetch of matrix i + 1 may start when GEMV i may start
          HIP_OR_FAIL(hipEventRecord(ev[i], s1));
          HIP_OR_FAIL(hipStreamWaitEvent(s2, ev[i], 0));
          launch_prefetch(b, i + 1, s2);
          forked = true;
        }
        launch_gemv(b, i, s1);
        break;
      case kUnpacedBranch:
        if (i == 0) {  // two chains that meet only at the start and at the end
          HIP_OR_FAIL(hipEventRecord(ev[0], s1));
          HIP_OR_FAIL(hipStreamWaitEvent(s2, ev[0], 0));
          for (int j = 1; j < S; ++j) launch_prefetch(b, j, s2);
          forked = true;
        }
        launch_gemv(b, i, s1);
        break;
    }
  }
  if (forked) {
    HIP_OR_FAIL(hipEventRecord(ev[S], s2));
    HIP_OR_FAIL(hipStreamWaitEvent(s1, ev[S], 0));
  }
  HIP_OR_FAIL(hipStreamEndCapture(s1, &graph));
  HIP_OR_FAIL(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0));
  for (int r = 0; r < 3; ++r) HIP_OR_FAIL(hipGraphLaunch(exec, s1));
  HIP_OR_FAIL(hipStreamSynchronize(s1));
  hipEvent_t e0, e1;
  HIP_OR_FAIL(hipEventCreate(&e0));
  HIP_OR_FAIL(hipEventCreate(&e1));
  HIP_OR_FAIL(hipEventRecord(e0, s1));
  for (int r = 0; r < reps; ++r) HIP_OR_FAIL(hipGraphLaunch(exec, s1));
  HIP_OR_FAIL(hipEventRecord(e1, s1));
  HIP_OR_FAIL(hipEventSynchronize(e1));
  float ms = 0;
  HIP_OR_FAIL(hipEventElapsedTime(&ms, e0, e1));
  *us = ms * 1e3 / reps / S;
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  (void)hipGraphExecDestroy(exec);
  (void)hipGraphDestroy(graph);
  for (auto& e : ev) (void)hipEventDestroy(e);
  (void)hipStreamDestroy(s1);
  (void)hipStreamDestroy(s2);
  return 0;
}

int run_pingpong(Buffers& b, int a, int c, double* us_one_way, unsigned* err) {
  static int base = 0;
  const int iters = 2000;
  hipEvent_t e0, e1;
  HIP_OR_FAIL(hipEventCreate(&e0));
  HIP_OR_FAIL(hipEventCreate(&e1));
  HIP_OR_FAIL(hipMemset(b.flags, 0, 1024));
  base += iters + 8;
  hipLaunchKernelGGL(pingpong_kernel, dim3(16), dim3(64), 0, 0, b.flags, b.flags + 64, a, c, 10, base, b.err);
  base += iters + 8;
  HIP_OR_FAIL(hipDeviceSynchronize());
  HIP_OR_FAIL(hipEventRecord(e0, 0));
  hipLaunchKernelGGL(pingpong_kernel, dim3(16), dim3(64), 0, 0, b.flags, b.flags + 64, a, c, iters, base, b.err);
  HIP_OR_FAIL(hipEventRecord(e1, 0));
  HIP_OR_FAIL(hipEventSynchronize(e1));
  float ms = 0;
  HIP_OR_FAIL(hipEventElapsedTime(&ms, e0, e1));
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  *us_one_way = ms * 1e3 / iters / 2;
  HIP_OR_FAIL(hipMemcpy(err, b.err, 4, hipMemcpyDeviceToHost));
  return 0;
}

}  // namespace

extern "C" {

const char* ajqb_last_error(void) { return g_error; }

int ajqb_mfma_rate(int random_operands, int iters, int workgroups, float* sink, long long* clocks,
                   double* flops_per_launch, void* stream) {
  if (!sink || !clocks) return fail(-1, "ajqb_mfma_rate: sink and clocks must be device buffers");
  if (iters < 1 || workgroups < 1 || workgroups > 65536)
    return fail(-2, "ajqb_mfma_rate: iters=%d, workgroups=%d out of range", iters, workgroups);
  hipLaunchKernelGGL(mfma_rate_kernel, dim3(workgroups), dim3(kProbeThreads), 0, (hipStream_t)stream,
                     random_operands, iters, sink, clocks);
  if (flops_per_launch)
    *flops_per_launch = (double)workgroups * (kProbeThreads / 64) * (double)iters * kProbeChains * 32768.0;
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(-5, "ajqb_mfma_rate: %s", hipGetErrorString(e));
  return 0;
}

int ajqb_launch_alternatives(int stages, int reps, ajqb_result* results, int max_results, int* n_results) {
  if (!results || !n_results || max_results < 1) return fail(-1, "ajqb_launch_alternatives: results buffer missing");
  if (stages < 4 || stages > 128 || reps < 1 || reps > 1000)
    return fail(-2, "ajqb_launch_alternatives: stages=%d (4..128), reps=%d (1..1000) out of range", stages, reps);
  int cus = 0;
  HIP_OR_FAIL(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, 0));
  if (cus < 256)  // the one-launch chain needs its 256 workgroups resident together
    return fail(-4, "ajqb_launch_alternatives: %d compute units, 256 needed for the one-launch chain", cus);
  Buffers b;
  b.S = stages;
  const int S = stages;
  HIP_OR_FAIL(hipMalloc(&b.wq, kWqStage * 16 * S));
  HIP_OR_FAIL(hipMalloc(&b.meta, kMetaStage * 4 * S));
  HIP_OR_FAIL(hipMalloc(&b.xbuf, (size_t)(S + 1) * 8 * (K / 2) * 8));
  HIP_OR_FAIL(hipMalloc(&b.flags, (size_t)(S + 1) * 8 * 256 * 4));
  HIP_OR_FAIL(hipMalloc(&b.err, 4));
  HIP_OR_FAIL(hipMalloc(&b.sink, 64));
  HIP_OR_FAIL(hipMalloc(&b.x, K * 2));
  HIP_OR_FAIL(hipMalloc(&b.y, (size_t)S * N * 2));
  hipLaunchKernelGGL(fill_hash_kernel, dim3(4096), dim3(256), 0, 0, b.wq, kWqStage * 4 * S, 12345u);
  // every group: scale fp16(0.0034), zero-point 7.5 (uniform nibbles are centred: the chain neither grows nor dies)
  hipLaunchKernelGGL(fill_const_kernel, dim3(1024), dim3(256), 0, 0, b.meta, kMetaStage * S, 0x583C1AF7u);
  hipLaunchKernelGGL(fill_const_kernel, dim3(8), dim3(256), 0, 0, reinterpret_cast<uint32_t*>(b.x), (size_t)K / 2, 0x3F803F80u);
  HIP_OR_FAIL(hipDeviceSynchronize());
  Results out{results, max_results};
  double us = 0;
  unsigned err = 0;
  std::vector<uint32_t> ref, got;

  // ---- one launch per matrix (HIP graph), the product path and its yardsticks
  if (int s = run_graph(b, kGemvOnly, reps, &us)) return s;
  out.add("one launch per matrix, library GEMV kernel, graph chain", us, -1, 0);
  if (int s = run_graph(b, kPrefetchOnly, reps, &us)) return s;
  out.add("one launch per matrix, kernel that only reads the bytes, graph chain", us, -1, 0);
  if (int s = run_graph(b, kSimple, reps, &us)) return s;
  out.add("one launch per matrix, plain GEMV kernel, graph chain", us, -1, 0);
  if (int s = run_graph(b, kSimplePrefetch, reps, &us)) return s;
  out.add("same, the next matrix's loads issued inside and consumed at the end", us, -1, 0);
  if (int s = run_graph(b, kPacedBranch, reps, &us)) return s;
  out.add("library GEMV i beside a prefetch kernel of matrix i+1 on a second graph branch", us, -1, 0);
  if (int s = run_graph(b, kUnpacedBranch, reps, &us)) return s;
  out.add("library GEMV chain beside an unpaced prefetch chain (two branches)", us, -1, 0);

  // ---- one launch for all stages, dependent stages
  if (int s = init_exchange(b, 1, false)) return s;
  if (int s = run_chain<kFlags, 1, true, 1, 1>(b, 3, true, &us, &err, &ref)) return s;
  out.add("reference for the results below: the chain kernel, one launch per stage, plain stream", us, -1, err);
  if (int s = run_chain<kNoDependency, 3, true, 1, 1>(b, reps, false, &us, &err, nullptr)) return s;
  out.add("one launch, stages NOT dependent (every stage reads the first activations)", us, -1, err);
  if (int s = run_chain<kFlags, 3, true, 4, 1>(b, reps, false, &us, &err, &got)) return s;
  out.add("one launch, dependent stages, flag per producer, one copy", us, got == ref, err);
  if (int s = init_exchange(b, 8, false)) return s;
  if (int s = run_chain<kFlags, 3, true, 4, 8>(b, reps, false, &us, &err, &got)) return s;
  out.add("one launch, dependent stages, flag per producer, copy per XCD", us, got == ref, err);
  if (int s = run_chain<kFlags, 1, false, 4, 8>(b, reps, false, &us, &err, nullptr)) return s;
  out.add("same without weight traffic (the exchange alone)", us, -1, err, false);
  if (int s = init_exchange(b, 8, true)) return s;
  if (int s = run_chain<kStamped, 3, true, 4, 8>(b, reps, false, &us, &err, &got)) return s;
  out.add("one launch, dependent stages, stamped records, copy per XCD", us, got == ref, err);
  if (int s = run_chain<kStamped, 1, false, 4, 8>(b, reps, false, &us, &err, nullptr)) return s;
  out.add("same without weight traffic (the exchange alone)", us, -1, err, false);
  if (int s = init_exchange(b, 1, false)) return s;
  if (int s = run_chain<kNoDependency, 1, false, 4, 1>(b, reps, false, &us, &err, nullptr)) return s;
  out.add("one launch, no dependency, no weight traffic (stage skeleton alone)", us, -1, err, false);

  // ---- the exchange's one-way latency (workgroups are dealt to the 8 XCDs round robin)
  if (int s = run_pingpong(b, 0, 8, &us, &err)) return s;
  out.add("one-way hop between two workgroups of one XCD, agent-scope store + load", us, -1, err, false);
  if (int s = run_pingpong(b, 0, 1, &us, &err)) return s;
  out.add("one-way hop between workgroups of two XCDs, agent-scope store + load", us, -1, err, false);
  *n_results = out.n;
  return 0;
}

}  // extern "C"
