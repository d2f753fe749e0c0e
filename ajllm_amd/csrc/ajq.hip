// C ABI of libajq.so: argument validation, launch geometry, error reporting.
#include <stdarg.h>
#include <cmath>
#include <algorithm>
#include <atomic>
#include <stdio.h>

#include "ajq_common.h"

#include "quantize_kernels.h"
#include "gemv_kernels.h"
#include "gemv_fused_kernels.h"
#include "gemm_kernels.h"
#include "gemm_ring_kernels.h"
#include "gemm_split_kernels.h"
#include "gemm_wide_kernels.h"
#include "gemm128_kernels.h"
#include "skinny_kernels.h"
#include "skinny_resident_kernels.h"
#include "decode_kernels.h"
#include "prefill_attention.h"

using namespace ajq;

namespace {

thread_local char g_error[512] = "";

int fail(int status, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return status;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(AJQ_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
  return AJQ_OK;
}

constexpr int kMaxGemvM = 16;

// ---- scratch of the entry point that allocates nothing (ajq_w4a16_gemm_noalloc): the per-row,
// per-group activation sums of the W4 tile kernels.  Every GPU the library runs on holds its own
// copy of the array at its own address until the process ends; host code never uses the array's
// name as an address, only the device address that hipGetSymbolAddress returns for the current
// device.
constexpr size_t kScratchBytes = (size_t)16 << 20;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];
constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];

// Device address of `scratch` on the current device, resolved once per device.
int scratch_address(void** out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(AJQ_ERR_HIP, "hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices) return fail(AJQ_ERR_UNSUPPORTED, "device index %d is outside 0..%d", dev, kMaxDevices - 1);
  void* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!ptr) {
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr)
      return fail(AJQ_ERR_HIP, "hipGetSymbolAddress(scratch) on device %d: %s", dev, hipGetErrorString(e));
    g_scratch_ptr[dev].store(ptr, std::memory_order_release);  // every thread resolves the same address
  }
  *out = ptr;
  return AJQ_OK;
}

// Kernels that stage more than 64 KiB in LDS must be opted in once per process
// (and per device); the largest size granted so far is remembered per kernel and device.
template <typename Kernel>
int allow_big_lds(Kernel kernel, size_t bytes) {
  struct Grant {
    const void* kernel;
    size_t bytes[16];
  };
  static thread_local Grant grants[192] = {};
  if (bytes <= 64 * 1024) return AJQ_OK;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16) dev = 0;
  const void* key = reinterpret_cast<const void*>(kernel);
  Grant* g = nullptr;
  for (Grant& e : grants) {
    if (e.kernel == key || e.kernel == nullptr) {
      g = &e;
      break;
    }
  }
  if (g && g->kernel == key && bytes <= g->bytes[dev]) return AJQ_OK;
  hipError_t e = hipFuncSetAttribute(key, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
  if (e != hipSuccess) return fail(AJQ_ERR_HIP, "hipFuncSetAttribute(%zu B LDS): %s", bytes, hipGetErrorString(e));
  if (g) {  // a full table only costs the repeated call
    g->kernel = key;
    g->bytes[dev] = bytes;
  }
  return AJQ_OK;
}

int check_matmul_args(const char* name, const void* x, int M, int K, const void* wq, const void* aux, int N,
                      const void* y, int out_dtype, int k_multiple) {
  if (!x || !wq || !aux || !y) return fail(AJQ_ERR_NULL, "%s: null pointer argument", name);
  if (M < 1 || N < 1 || K < 1) return fail(AJQ_ERR_SHAPE, "%s: M, N, K must be positive (got %d, %d, %d)", name, M, N, K);
  if (K % k_multiple != 0) return fail(AJQ_ERR_SHAPE, "%s: K=%d must be a multiple of %d", name, K, k_multiple);
  if (N % kTileN != 0) return fail(AJQ_ERR_SHAPE, "%s: N=%d must be a multiple of %d", name, N, kTileN);
  if (out_dtype != AJQ_OUT_BF16 && out_dtype != AJQ_OUT_F32)
    return fail(AJQ_ERR_UNSUPPORTED, "%s: out_dtype %d is neither AJQ_OUT_BF16 nor AJQ_OUT_F32", name, out_dtype);
  if (!aligned16(x) || !aligned16(wq) || !aligned16(y))
    return fail(AJQ_ERR_ALIGN, "%s: x, wq and y must be 16-byte aligned", name);
  return AJQ_OK;
}

// 256-row tiles on 32x32x16 MFMA; M >= 256 (the last row tile is shifted, not masked).  Shapes with enough tiles
// take 256 x 256 ones (gemm_wide_kernels.h); otherwise 256 x 128: W8 with K % 256 == 0
// runs the ring kernel (four compute waves that unpack their own weights, a loader wave); W4, and W8 on any other
// K % 128 == 0, the split-role kernel (four compute waves, four producers that dequantize once per workgroup; W4
// needs no group sums there).
#ifndef AJQ_GEMM_WIDE
#define AJQ_GEMM_WIDE 1
#endif
template <bool kW4, bool kGate = false>
int launch_gemm256(const uint16_t* x, int M, int K, const uint32_t* wq, const uint32_t* meta, const uint16_t* scales8,
                   int N, void* y, int out_f32, hipStream_t stream) {
  const int tiles = ((M + kG2BM - 1) / kG2BM) * ((N + kG2BN - 1) / kG2BN);
  if (!kGate || (N / 2) % (kGWBN / 2) == 0) {
    // 256 x 256 tiles move half the activation bytes per MFMA and measure 9-15 % faster per flop, but there are half
    // as many of them: they run when that still fills the CUs' rounds better (a wide tile takes 2 / 1.12 narrow ones)
    const long long wide = (long long)((M + kGWBM - 1) / kGWBM) * ((N + kGWBN - 1) / kGWBN);
    const double cost_wide = (double)((wide + 255) / 256) * (2.0 / 1.12), cost_narrow = (double)((tiles + 255) / 256);
    if (AJQ_GEMM_WIDE && cost_wide < cost_narrow) {
      auto kernel = dequant_gemm256w_kernel<kW4, kGate>;
      if (int s = allow_big_lds(kernel, kGWLdsBytes)) return s;
      hipLaunchKernelGGL(kernel, dim3((unsigned)wide), dim3(kGWThreads), kGWLdsBytes, stream, x, M, K,
                         reinterpret_cast<const u32x4_t*>(wq), meta, scales8, N, y, out_f32);
      return AJQ_OK;
    }
  }
  if (!kW4 && K % 256 == 0) {
    auto ring = dequant_gemm256r_w8_kernel<kGate>;
    if (int s = allow_big_lds(ring, kGRLdsBytes)) return s;
    hipLaunchKernelGGL(ring, dim3(tiles), dim3(kGRThreads), kGRLdsBytes, stream, x, M, K,
                       reinterpret_cast<const u32x4_t*>(wq), scales8, N, y, out_f32);
    return AJQ_OK;
  }
  auto split = dequant_gemm256s_kernel<kW4, kGate>;
  if (int s = allow_big_lds(split, kGSLdsBytes)) return s;
  hipLaunchKernelGGL(split, dim3(tiles), dim3(kGSThreads), kGSLdsBytes, stream, x, M, K,
                     reinterpret_cast<const u32x4_t*>(wq), meta, scales8, N, y, out_f32);
  return AJQ_OK;
}

// 128 x 128 tiles, tiles requested two k-blocks ahead; M >= 128
#ifndef AJQ_G1_WN
#define AJQ_G1_WN 4
#endif
template <bool kW4, bool kGate = false>
int launch_gemm128(const uint16_t* x, int M, int K, const uint32_t* wq, const uint32_t* meta,
                   const uint16_t* scales8, const void* gs3, int N, void* y, int out_f32, hipStream_t stream) {
  auto kernel = dequant_gemm128_kernel<kW4, AJQ_G1_WN, kGate>;
  constexpr size_t lds = kW4 ? kG1LdsBytesW4 : kG1LdsBytesW8;
  if (int s = allow_big_lds(kernel, lds)) return s;
  const int tiles = ((M + kG1BM - 1) / kG1BM) * ((N + kG1BN - 1) / kG1BN);
  hipLaunchKernelGGL(kernel, dim3(tiles), dim3(128 * AJQ_G1_WN), lds, stream, x, M, K,
                     reinterpret_cast<const u32x4_t*>(wq), meta, scales8,
                     reinterpret_cast<const u32x4_t*>(gs3), N, y, out_f32);
  return AJQ_OK;
}

#ifndef AJQ_GEMM256_MIN_M
#define AJQ_GEMM256_MIN_M 256
#endif
constexpr int kGemm256MinM = AJQ_GEMM256_MIN_M;

}  // namespace

extern "C" {

int ajq_version(void) { return 1; }

const char* ajq_last_error(void) { return g_error; }

const char* ajq_status_string(int status) {
  switch (status) {
    case AJQ_OK: return "ok";
    case AJQ_ERR_NULL: return "null pointer";
    case AJQ_ERR_SHAPE: return "unsupported shape";
    case AJQ_ERR_ALIGN: return "misaligned pointer";
    case AJQ_ERR_UNSUPPORTED: return "unsupported option";
    case AJQ_ERR_HIP: return "HIP runtime error";
    case AJQ_ERR_WORKSPACE: return "workspace missing or too small";
    default: return "unknown status";
  }
}

int ajq_quantize_w8(const float* W, int N, int K, int8_t* q, uint16_t* scales, void* stream) {
  if (!W || !q || !scales) return fail(AJQ_ERR_NULL, "ajq_quantize_w8: null pointer argument");
  if (N < 1 || K < 4 || K % 4 != 0)
    return fail(AJQ_ERR_SHAPE, "ajq_quantize_w8: need N >= 1 and K a positive multiple of 4 (got N=%d, K=%d)", N, K);
  if (!aligned16(W) || (reinterpret_cast<uintptr_t>(q) & 3u))
    return fail(AJQ_ERR_ALIGN, "ajq_quantize_w8: W must be 16-byte and q 4-byte aligned");
  hipLaunchKernelGGL(quantize_w8_kernel, dim3(N), dim3(256), 0, (hipStream_t)stream, W, K, q, scales);
  return check_launch("ajq_quantize_w8");
}

int ajq_quantize_w4_g128(const float* W, int N, int K, int32_t* qweight, uint16_t* scales, uint8_t* zeros,
                         void* stream) {
  if (!W || !qweight || !scales || !zeros) return fail(AJQ_ERR_NULL, "ajq_quantize_w4_g128: null pointer argument");
  if (N < 1 || K < kGroup || K % kGroup != 0)
    return fail(AJQ_ERR_SHAPE, "ajq_quantize_w4_g128: need N >= 1 and K a positive multiple of 128 (got N=%d, K=%d)", N, K);
  if (!aligned16(W)) return fail(AJQ_ERR_ALIGN, "ajq_quantize_w4_g128: W must be 16-byte aligned");
  const long long groups = (long long)N * (K / kGroup);
  const long long blocks = (groups + 15) / 16;
  if (blocks > 0x7FFFFFFFLL) return fail(AJQ_ERR_SHAPE, "ajq_quantize_w4_g128: too many groups");
  hipLaunchKernelGGL(quantize_w4_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, W, groups,
                     qweight, scales, zeros);
  return check_launch("ajq_quantize_w4_g128");
}

static int check_repack(const char* name, const void* a, const void* b, int N, int K, int kmul) {
  if (!a || !b) return fail(AJQ_ERR_NULL, "%s: null pointer argument", name);
  if (N < kTileN || N % kTileN != 0 || K < kmul || K % kmul != 0)
    return fail(AJQ_ERR_SHAPE, "%s: need N a multiple of 16 and K a multiple of %d (got N=%d, K=%d)", name, kmul, N, K);
  return AJQ_OK;
}

int ajq_repack_w4(const int32_t* qweight, const uint16_t* scales, const uint8_t* zeros, int N, int K,
                  uint32_t* wq, uint32_t* meta, void* stream) {
  if (int s = check_repack("ajq_repack_w4", qweight, wq, N, K, kGroup)) return s;
  if (!scales || !zeros || !meta) return fail(AJQ_ERR_NULL, "ajq_repack_w4: null pointer argument");
  const long long words = (long long)N * (K / 8);
  hipLaunchKernelGGL(repack_w4_kernel, dim3((unsigned)((words + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                     reinterpret_cast<const uint32_t*>(qweight), N, K, wq);
  const long long metas = (long long)N * (K / kGroup);
  hipLaunchKernelGGL(repack_w4_meta_kernel, dim3((unsigned)((metas + 255) / 256)), dim3(256), 0,
                     (hipStream_t)stream, scales, zeros, N, K / kGroup, meta);
  return check_launch("ajq_repack_w4");
}

int ajq_unrepack_w4(const uint32_t* wq, const uint32_t* meta, int N, int K, int32_t* qweight, uint16_t* scales,
                    uint8_t* zeros, void* stream) {
  if (int s = check_repack("ajq_unrepack_w4", wq, qweight, N, K, kGroup)) return s;
  if (!scales || !zeros || !meta) return fail(AJQ_ERR_NULL, "ajq_unrepack_w4: null pointer argument");
  const long long words = (long long)N * (K / 8);
  hipLaunchKernelGGL(unrepack_w4_kernel, dim3((unsigned)((words + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                     wq, N, K, reinterpret_cast<uint32_t*>(qweight));
  const long long metas = (long long)N * (K / kGroup);
  hipLaunchKernelGGL(unrepack_w4_meta_kernel, dim3((unsigned)((metas + 255) / 256)), dim3(256), 0,
                     (hipStream_t)stream, meta, N, K / kGroup, scales, zeros);
  return check_launch("ajq_unrepack_w4");
}

int ajq_repack_w8(const int8_t* q, int N, int K, uint32_t* wq, void* stream) {
  if (int s = check_repack("ajq_repack_w8", q, wq, N, K, kW8TileK)) return s;
  if (reinterpret_cast<uintptr_t>(q) & 3u) return fail(AJQ_ERR_ALIGN, "ajq_repack_w8: q must be 4-byte aligned");
  const long long words = (long long)N * (K / 4);
  hipLaunchKernelGGL(repack_w8_kernel<false>, dim3((unsigned)((words + 255) / 256)), dim3(256), 0,
                     (hipStream_t)stream, reinterpret_cast<const uint32_t*>(q), N, K, wq);
  return check_launch("ajq_repack_w8");
}

int ajq_unrepack_w8(const uint32_t* wq, int N, int K, int8_t* q, void* stream) {
  if (int s = check_repack("ajq_unrepack_w8", wq, q, N, K, kW8TileK)) return s;
  if (reinterpret_cast<uintptr_t>(q) & 3u) return fail(AJQ_ERR_ALIGN, "ajq_unrepack_w8: q must be 4-byte aligned");
  const long long words = (long long)N * (K / 4);
  hipLaunchKernelGGL(repack_w8_kernel<true>, dim3((unsigned)((words + 255) / 256)), dim3(256), 0,
                     (hipStream_t)stream, wq, N, K, reinterpret_cast<uint32_t*>(q));
  return check_launch("ajq_unrepack_w8");
}

}  // extern "C"

// --------------------------------------------------------------- GEMV -----
namespace {

constexpr int kGemvFragWorkgroups = 256;  // one per CU

template <int kWaves, int TPW, int MROWS, bool kW4, bool kSingle>
int launch_gemv_cfg(const uint16_t* x, int M, int K, const uint32_t* wq, const uint32_t* meta,
                    const uint16_t* scales8, int N, void* y, int out_f32, hipStream_t stream) {
  constexpr size_t lds = gemv_lds_bytes(kWaves, TPW, MROWS);
  static_assert(lds <= 160 * 1024, "GEMV configuration exceeds the 160 KiB LDS of a CU");
  // at most one workgroup per CU: the A fragments of every k-step wait in registers for the weights (measured:
  // 3.87 -> 3.57 us on 4096 x 4096 at one row; on launches of several rounds the registers cost more in
  // occupancy than the early fragments save, 7.16 -> 7.49 us on 14336 x 4096)
  constexpr bool kCanHoldFrags = kSingle && TPW <= 4;
  auto kernel = dequant_gemv_kernel<kWaves, TPW, MROWS, kW4, kSingle, false>;
  if (kCanHoldFrags && N / kTileN <= kGemvFragWorkgroups) kernel = dequant_gemv_kernel<kWaves, TPW, MROWS, kW4, kSingle, kCanHoldFrags>;
  if (int s = allow_big_lds(kernel, lds)) return s;
  hipLaunchKernelGGL(kernel, dim3(N / kTileN), dim3(kWaves * 64), lds, stream,
                     reinterpret_cast<const u32x4_t*>(wq), meta, x, K, M | (out_f32 << 8), N, y, scales8);
  return AJQ_OK;
}

// One wave stages TPW k groups at a time; K == kWaves * TPW * 128 takes the
// straight-line variant of the kernel.
template <int kWaves, int TPW, int MROWS, bool kW4>
int launch_gemv_rows(const uint16_t* x, int M, int K, const uint32_t* wq, const uint32_t* meta,
                     const uint16_t* scales8, int N, void* y, int out_f32, hipStream_t stream) {
  if (K == kWaves * TPW * kGroup)
    return launch_gemv_cfg<kWaves, TPW, MROWS, kW4, true>(x, M, K, wq, meta, scales8, N, y, out_f32, stream);
  return launch_gemv_cfg<kWaves, TPW, MROWS, kW4, false>(x, M, K, wq, meta, scales8, N, y, out_f32, stream);
}

// ---- split-K form of the weight-streaming kernel (see kSplitK in skinny_kernels.h): only with a buffer the caller
// has lent to this host thread's calls (ajq_matmul_workspace_set), which holds the ticket words and the partial sums
constexpr int kSplitTiles = 4, kSplitWays = 4;          // row tiles per workgroup, workgroups per row-tile group
constexpr size_t kSplitTicketBytes = 4096;              // one word per (row-tile group, row block), zeroed
constexpr int kSplitMaxCells = 64;                      // 256 workgroups: one round of the chip
constexpr size_t kSplitCellBytes = (size_t)kSplitWays * kSplitTiles * 2 * 1024;
constexpr size_t kSplitWorkspaceBytes = kSplitTicketBytes + kSplitMaxCells * kSplitCellBytes;
struct SplitWorkspace {
  void* base = nullptr;
  size_t bytes = 0;
};
thread_local SplitWorkspace g_split_ws;

// The split-K resident form for 9 <= M <= 16 at K = 14336 (four workgroups of seven waves share a run of four row
// tiles and take 28 groups of K each; skinny_resident_kernels.h): the GEMV's workgroups each pull their whole
// activation block out of L2, 459 KB at this K for 115 KB of int4 weights.  Measured at M = 16, N = 4096, int8 / int4:
// 17.8 -> 14.7 / 13.4 -> 10.9 us; at M = 8 the int8 GEMV is the faster one, at 32 rows the 32-row split form is level.
bool gemv_split_applies(int M, int N, int K) {
  if (!g_split_ws.base || g_split_ws.bytes < kSplitWorkspaceBytes) return false;
  const int ntiles = N / kTileN;
  return M >= 9 && M <= kMaxGemvM && K == 14336 && ntiles >= kSplitTiles && (ntiles + kSplitTiles - 1) / kSplitTiles <= kSplitMaxCells;
}
template <bool kW4, int kEpi>
int launch_gemv_split(const uint16_t* x, int M, int K, const uint32_t* wq, const uint32_t* meta, const uint16_t* scales8,
                      int N, void* y, int out_f32, const GemvEpilogue& ep, hipStream_t stream) {
  constexpr int T = kSplitTiles, kWaves = 7, TPW = 4;
  const int S = K / kGroup / (kWaves * TPW);
  const int nruns = (N / kTileN + T - 1) / T;
  const dim3 grid(8 * ((nruns + 7) / 8) * S), block(kWaves * 64);
  SkinnySplit sp{reinterpret_cast<float*>(static_cast<char*>(g_split_ws.base) + kSplitTicketBytes),
                 static_cast<unsigned*>(g_split_ws.base), S};
  constexpr size_t lds = res_lds_bytes(T, 1, kEpi != 0);
  if constexpr (kEpi != 0) {
    auto kernel = dequant_skinny_resident_split_epi_kernel<TPW, T, kW4, kEpi, 1, kWaves>;
    if (int s = allow_big_lds(kernel, lds)) return s;
    hipLaunchKernelGGL(kernel, grid, block, lds, stream, reinterpret_cast<const u32x4_t*>(wq), meta, x, K, M, N, y, out_f32,
                       scales8, ep, sp);
  } else {
    auto kernel = dequant_skinny_resident_split_kernel<TPW, T, kW4, 1, kWaves>;
    if (int s = allow_big_lds(kernel, lds)) return s;
    hipLaunchKernelGGL(kernel, grid, block, lds, stream, reinterpret_cast<const u32x4_t*>(wq), meta, x, K, M, N, y, out_f32,
                       scales8, sp);
  }
  return AJQ_OK;
}

// ---- resident-activation form of the weight-streaming kernel (skinny_resident_kernels.h): K = 2048 or 4096, a
// run of T row tiles per workgroup, row blocks of 16 MB rows (MB = 1 for the GEMV's M <= 16, 2 above).  T is the
// shortest run that fits the workgroups into one round of the chip (256: one workgroup per CU); where the longest
// run still leaves more than one round, both forms are priced in bytes a CU pulls over its rounds (rounds x
// workgroups per CU x (32 MB bytes of activations + 16 b T of weights) per unit of K) and the cheaper one runs.
// Measured at 32 rows, K = 4096, int8 / int4, against the other form: N = 4096 (T = 1) 8.3 -> 7.6 / 8.2 -> 6.6 us;
// N = 6144 (T = 2) 10.1 -> 9.4 / 8.7 -> 7.5; N = 28672 (T = 8) 31 -> 24 / 23 -> 19; a 128256-row head (T = 8, four
// rounds) 103 -> 99 / 83 -> 72.
#ifndef AJQ_SKINNY_RESIDENT
#define AJQ_SKINNY_RESIDENT 1
#endif
// from this many workgroups of four row tiles on, the other form runs as four-wave workgroups, two to a CU
#ifndef AJQ_SKINNY_FOUR_WAVE_MIN
#define AJQ_SKINNY_FOUR_WAVE_MIN 512
#endif
template <bool kW4>
long long skinny_cost(int ntiles, int mblocks, int tiles_per_wg, int slots, int mb = 2) {
  const long long wgs = (long long)((ntiles + tiles_per_wg - 1) / tiles_per_wg) * mblocks;
  return ((wgs + slots - 1) / slots) * (slots / 256) * (32 * mb + (kW4 ? 8 : 16) * tiles_per_wg);
}
// row tiles per workgroup of the resident form for (M, N, K), or 0 where the other form is taken (MB = 2 only: with
// a 16-row block the caller has already decided)
template <bool kW4, int MB>
int skinny_resident_tiles(int M, int N, int K) {
  if (!AJQ_SKINNY_RESIDENT || (K != 2048 && K != 4096)) return 0;
  const int ntiles = N / kTileN, mblocks = (M + 16 * MB - 1) / (16 * MB);
  if (MB == 1) {
    for (int t : {2, 3, 4, 6, 8, 16})
      if ((ntiles + t - 1) / t <= 256) return t;
    return 16;
  }
  for (int t : {1, 2, 3, 4, 6, 8})
    if ((long long)((ntiles + t - 1) / t) * mblocks <= 256) return t;
  long long other = skinny_cost<kW4>(ntiles, mblocks, 1, 256);
  other = std::min(other, skinny_cost<kW4>(ntiles, mblocks, 2, 256));
  other = std::min(other, skinny_cost<kW4>(ntiles, mblocks, 4, (ntiles / 4) * mblocks >= AJQ_SKINNY_FOUR_WAVE_MIN ? 512 : 256));
  int best = 0;
  long long cost = other;
  for (int t : {4, 6, 8}) {
    const long long c = skinny_cost<kW4>(ntiles, mblocks, t, 256);
    if (c <= cost) {  // (ties go to the resident form and to the longer run: the better pattern for HBM)
      cost = c;
      best = t;
    }
  }
  return best;
}
// whether a GEMV (M <= 16) runs as the resident form with one 16-row block
bool gemv_takes_resident(int M, int N, int K) {
  return AJQ_SKINNY_RESIDENT && M >= 8 && M <= 16 && (K == 2048 || K == 4096) && N / kTileN > 256;
}

template <int TPW, int T, bool kW4, int kEpi, int MB>
int launch_skinny_resident_cfg(const uint16_t* x, int M, int K, const uint32_t* wq, const uint32_t* meta,
                               const uint16_t* scales8, int N, void* y, int out_f32, const GemvEpilogue& ep,
                               hipStream_t stream) {
  const int ntiles = N / kTileN;
  const int nruns = (ntiles + T - 1) / T, mblocks = (M + 16 * MB - 1) / (16 * MB);
  const dim3 grid(8 * ((nruns + 7) / 8) * mblocks), block(kResWaves * 64);
  if constexpr (kEpi != 0) {
    auto kernel = dequant_skinny_resident_epi_kernel<TPW, T, kW4, kEpi, MB>;
    constexpr size_t lds = res_lds_bytes(T, MB, true);
    if (int s = allow_big_lds(kernel, lds)) return s;
    hipLaunchKernelGGL(kernel, grid, block, lds, stream, reinterpret_cast<const u32x4_t*>(wq), meta, x, K, M, N, y,
                       out_f32, scales8, ep);
  } else {
    auto kernel = dequant_skinny_resident_kernel<TPW, T, kW4, MB>;
    constexpr size_t lds = res_lds_bytes(T, MB, false);
    if (int s = allow_big_lds(kernel, lds)) return s;
    hipLaunchKernelGGL(kernel, grid, block, lds, stream, reinterpret_cast<const u32x4_t*>(wq), meta, x, K, M, N, y,
                       out_f32, scales8);
  }
  return AJQ_OK;
}

template <bool kW4, int kEpi, int MB>
int launch_skinny_resident(int T, const uint16_t* x, int M, int K, const uint32_t* wq, const uint32_t* meta,
                           const uint16_t* scales8, int N, void* y, int out_f32, const GemvEpilogue& ep, hipStream_t stream) {
#define AJQ_RES(P, TT)                \
  if (K == 1024 * P && T == TT)       \
    return launch_skinny_resident_cfg<P, TT, kW4, kEpi, MB>(x, M, K, wq, meta, scales8, N, y, out_f32, ep, stream)
#define AJQ_RES_K(P)                  \
  if constexpr (MB == 2) AJQ_RES(P, 1); \
  AJQ_RES(P, 2);                      \
  AJQ_RES(P, 3);                      \
  AJQ_RES(P, 4);                      \
  AJQ_RES(P, 6);                      \
  AJQ_RES(P, 8);                      \
  if constexpr (MB == 1) AJQ_RES(P, 16)
  AJQ_RES_K(4);
  AJQ_RES_K(2);
#undef AJQ_RES_K
#undef AJQ_RES
  return fail(AJQ_ERR_UNSUPPORTED, "no resident-activation configuration for K = %d, %d row tiles", K, T);
}

// Row bound MROWS is the next power of two >= M; above 4 rows a wave stages two
// k groups at a time instead of four, which keeps the two register sets of the
// ping-pong inside the VGPR budget and the slices inside 80 KiB of LDS.
template <bool kW4>
int launch_gemv(const uint16_t* x, int M, int K, const uint32_t* wq, const uint32_t* meta,
                const uint16_t* scales8, int N, void* y, int out_f32, hipStream_t stream) {
  // 8 <= M, K = 2048 or 4096 and more row tiles than CUs: the resident-activation form of the weight-streaming
  // kernel with a 16-row block (a workgroup keeps its activations in registers and walks a run of row tiles past
  // them; W4, M = 16: 14336 x 4096 10.4 -> 8.5 us, a 32000 x 2048 head 15.4 -> 9.1; below M = 8 and up to 256 row
  // tiles the single-tile kernel is the faster one)
  if (gemv_takes_resident(M, N, K))
    return launch_skinny_resident<kW4, 0, 1>(skinny_resident_tiles<kW4, 1>(M, N, K), x, M, K, wq, meta, scales8, N, y, out_f32,
                                             GemvEpilogue{}, stream);
  if (gemv_split_applies(M, N, K))
    return launch_gemv_split<kW4, 0>(x, M, K, wq, meta, scales8, N, y, out_f32, GemvEpilogue{}, stream);
  if (K == 8 * 2 * kGroup) {  // K = 2048: one batch of two groups per wave, straight-line kernel
    if (M <= 1) return launch_gemv_cfg<8, 2, 1, kW4, true>(x, M, K, wq, meta, scales8, N, y, out_f32, stream);
    if (M <= 2) return launch_gemv_cfg<8, 2, 2, kW4, true>(x, M, K, wq, meta, scales8, N, y, out_f32, stream);
    if (M <= 4) return launch_gemv_cfg<8, 2, 4, kW4, true>(x, M, K, wq, meta, scales8, N, y, out_f32, stream);
    if (M <= 8) return launch_gemv_cfg<8, 2, 8, kW4, true>(x, M, K, wq, meta, scales8, N, y, out_f32, stream);
    return launch_gemv_cfg<8, 2, 16, kW4, true>(x, M, K, wq, meta, scales8, N, y, out_f32, stream);
  }
  if (K == 11 * 4 * kGroup && M <= 8) {  // K = 5632 (44 groups): eleven waves of four groups, straight-line kernel
    if (M <= 1) return launch_gemv_cfg<11, 4, 1, kW4, true>(x, M, K, wq, meta, scales8, N, y, out_f32, stream);
    if (M <= 2) return launch_gemv_cfg<11, 4, 2, kW4, true>(x, M, K, wq, meta, scales8, N, y, out_f32, stream);
    if (M <= 4) return launch_gemv_cfg<11, 4, 4, kW4, true>(x, M, K, wq, meta, scales8, N, y, out_f32, stream);
    return launch_gemv_cfg<11, 4, 8, kW4, true>(x, M, K, wq, meta, scales8, N, y, out_f32, stream);
  }
  if (K == 16 * 7 * kGroup && M <= 4) {  // K = 14336 (112 groups): sixteen waves of seven groups, straight-line kernel
    if (M <= 1) return launch_gemv_cfg<16, 7, 1, kW4, true>(x, M, K, wq, meta, scales8, N, y, out_f32, stream);
    if (M <= 2) return launch_gemv_cfg<16, 7, 2, kW4, true>(x, M, K, wq, meta, scales8, N, y, out_f32, stream);
    return launch_gemv_cfg<16, 7, 4, kW4, true>(x, M, K, wq, meta, scales8, N, y, out_f32, stream);
  }
  if (M <= 1) return launch_gemv_rows<8, 4, 1, kW4>(x, M, K, wq, meta, scales8, N, y, out_f32, stream);
  if (M <= 2) return launch_gemv_rows<8, 4, 2, kW4>(x, M, K, wq, meta, scales8, N, y, out_f32, stream);
  if (M <= 4) return launch_gemv_rows<8, 4, 4, kW4>(x, M, K, wq, meta, scales8, N, y, out_f32, stream);
  if (K == 8 * 4 * kGroup) {  // one batch of four groups per wave covers K: straight-line kernel
    if (M <= 8) return launch_gemv_cfg<8, 4, 8, kW4, true>(x, M, K, wq, meta, scales8, N, y, out_f32, stream);
    return launch_gemv_cfg<8, 4, 16, kW4, true>(x, M, K, wq, meta, scales8, N, y, out_f32, stream);
  }
  if (M <= 8) return launch_gemv_rows<8, 2, 8, kW4>(x, M, K, wq, meta, scales8, N, y, out_f32, stream);
  return launch_gemv_rows<8, 2, 16, kW4>(x, M, K, wq, meta, scales8, N, y, out_f32, stream);
}

// The batch counts built as straight-line code per configuration: those the K of the benchmark models give
// (2048, 4096, 14336: 16, 32 and 112 groups over kWaves * TPW per batch); any other K takes the generic loop.
constexpr bool skinny_static_batches(int waves, int tpw, int batches) {
  const int per_batch = waves * tpw;
  return per_batch * batches == 16 || per_batch * batches == 32 || per_batch * batches == 112;
}

template <int kWaves, int TPW, int MROWS, int NT, bool kW4>
int launch_skinny_cfg(const uint16_t* x, int M, int K, const uint32_t* wq, const uint32_t* meta,
                      const uint16_t* scales8, int N, void* y, int out_f32, hipStream_t stream) {
  constexpr size_t lds = skinny_lds_bytes(kWaves, TPW, MROWS);
  static_assert(lds <= 160 * 1024, "skinny configuration exceeds the 160 KiB LDS of a CU");
  // K of kWaves * TPW * {2, 4, 7, 14} groups (2048, 4096 and 14336 in the configurations used): the batch loop as
  // straight-line code with exact wait counts (a batch is computed while the next travels; the generic loop's
  // conditional loads make the compiler wait for everything in flight): 3-17 % faster at 32 and 64 rows
  auto kernel = dequant_skinny_kernel<kWaves, TPW, MROWS, NT, kW4>;
  const int G = K / kGroup;
  if constexpr (skinny_static_batches(kWaves, TPW, 2))
    if (G == kWaves * TPW * 2) kernel = dequant_skinny_kernel<kWaves, TPW, MROWS, NT, kW4, 2>;
  if constexpr (skinny_static_batches(kWaves, TPW, 4))
    if (G == kWaves * TPW * 4) kernel = dequant_skinny_kernel<kWaves, TPW, MROWS, NT, kW4, 4>;
  if constexpr (skinny_static_batches(kWaves, TPW, 7))
    if (G == kWaves * TPW * 7) kernel = dequant_skinny_kernel<kWaves, TPW, MROWS, NT, kW4, 7>;
  if constexpr (skinny_static_batches(kWaves, TPW, 14))
    if (G == kWaves * TPW * 14) kernel = dequant_skinny_kernel<kWaves, TPW, MROWS, NT, kW4, 14>;
  if (int s = allow_big_lds(kernel, lds)) return s;
  const int ntiles = N / kTileN;
  const int ngroups = (ntiles + NT - 1) / NT, mblocks = (M + MROWS - 1) / MROWS;
  hipLaunchKernelGGL(kernel, dim3(8 * ((ngroups + 7) / 8) * mblocks), dim3(kWaves * 64), lds, stream,
                     reinterpret_cast<const u32x4_t*>(wq), meta, x, K, M, N, y, out_f32, scales8);
  return AJQ_OK;
}

template <int kWaves, int TPW, int MROWS, int NT, bool kW4, int kEpi>
int launch_skinny_epi_cfg(const uint16_t* x, int M, int K, const uint32_t* wq, const uint32_t* meta,
                          const uint16_t* scales8, int N, void* y, int out_f32, const GemvEpilogue& ep, hipStream_t stream) {
  constexpr size_t lds = skinny_epi_lds_bytes(kWaves, TPW, MROWS);
  static_assert(lds <= 160 * 1024, "skinny configuration exceeds the 160 KiB LDS of a CU");
  auto kernel = dequant_skinny_epi_kernel<kWaves, TPW, MROWS, NT, kW4, kEpi>;
  const int G = K / kGroup;  // as in launch_skinny_cfg
  if constexpr (skinny_static_batches(kWaves, TPW, 2))
    if (G == kWaves * TPW * 2) kernel = dequant_skinny_epi_kernel<kWaves, TPW, MROWS, NT, kW4, kEpi, 2>;
  if constexpr (skinny_static_batches(kWaves, TPW, 4))
    if (G == kWaves * TPW * 4) kernel = dequant_skinny_epi_kernel<kWaves, TPW, MROWS, NT, kW4, kEpi, 4>;
  if constexpr (skinny_static_batches(kWaves, TPW, 7))
    if (G == kWaves * TPW * 7) kernel = dequant_skinny_epi_kernel<kWaves, TPW, MROWS, NT, kW4, kEpi, 7>;
  if constexpr (skinny_static_batches(kWaves, TPW, 14))
    if (G == kWaves * TPW * 14) kernel = dequant_skinny_epi_kernel<kWaves, TPW, MROWS, NT, kW4, kEpi, 14>;
  if (int s = allow_big_lds(kernel, lds)) return s;
  const int ntiles = N / kTileN;
  const int ngroups = (ntiles + NT - 1) / NT, mblocks = (M + MROWS - 1) / MROWS;
  hipLaunchKernelGGL(kernel, dim3(8 * ((ngroups + 7) / 8) * mblocks), dim3(kWaves * 64), lds, stream,
                     reinterpret_cast<const u32x4_t*>(wq), meta, x, K, M, N, y, out_f32, scales8, ep);
  return AJQ_OK;
}

// Whether the split-K form takes (M, N, K): a lent buffer, one round of workgroups, a K that four workgroups share
// evenly, and enough of it that the activation traffic saved (each row-tile group of four reads the block once
// instead of four times) outweighs the exchange of partial sums through memory (about 3 us: measured 22.1 -> 17.5 us
// at N = 4096, K = 14336, M = 32 for int8 weights; no gain at K = 4096).
bool skinny_split_applies(int M, int N, int K) {
  if (!g_split_ws.base || g_split_ws.bytes < kSplitWorkspaceBytes) return false;
  const int ntiles = N / kTileN, mblocks = (M + 31) / 32;
  const int cells = ((ntiles + kSplitTiles - 1) / kSplitTiles) * mblocks;
  return K >= 8192 && (K / kGroup) % kSplitWays == 0 && cells <= kSplitMaxCells && ntiles >= kSplitTiles;
}

template <bool kW4, int kEpi, int kBatches>
int launch_skinny_split_kernel(const uint16_t* x, int M, int K, const uint32_t* wq, const uint32_t* meta,
                               const uint16_t* scales8, int N, void* y, int out_f32, const GemvEpilogue& ep,
                               hipStream_t stream) {
  constexpr size_t lds = kEpi ? skinny_epi_lds_bytes(8, 1, 32) : skinny_lds_bytes(8, 1, 32);
  const int ntiles = N / kTileN;
  const int ngroups = (ntiles + kSplitTiles - 1) / kSplitTiles, mblocks = (M + 31) / 32;
  const dim3 grid(8 * ((ngroups + 7) / 8) * mblocks * kSplitWays), block(8 * 64);
  SkinnySplit sp{reinterpret_cast<float*>(static_cast<char*>(g_split_ws.base) + kSplitTicketBytes),
                 static_cast<unsigned*>(g_split_ws.base), kSplitWays};
  if constexpr (kEpi != 0) {
    auto kernel = dequant_skinny_split_epi_kernel<8, 1, 32, kSplitTiles, kW4, kEpi, kBatches>;
    if (int s = allow_big_lds(kernel, lds)) return s;
    hipLaunchKernelGGL(kernel, grid, block, lds, stream, reinterpret_cast<const u32x4_t*>(wq), meta, x, K, M, N, y, out_f32,
                       scales8, ep, sp);
  } else {
    auto kernel = dequant_skinny_split_kernel<8, 1, 32, kSplitTiles, kW4, kBatches>;
    if (int s = allow_big_lds(kernel, lds)) return s;
    hipLaunchKernelGGL(kernel, grid, block, lds, stream, reinterpret_cast<const u32x4_t*>(wq), meta, x, K, M, N, y, out_f32,
                       scales8, sp);
  }
  return AJQ_OK;
}

template <bool kW4, int kEpi>
int launch_skinny_split(const uint16_t* x, int M, int K, const uint32_t* wq, const uint32_t* meta, const uint16_t* scales8,
                        int N, void* y, int out_f32, const GemvEpilogue& ep, hipStream_t stream) {
  // a workgroup's K / 4 as seven or eight waves' runs of four groups (K = 14336: 28 groups): straight-line code
  const int count = K / kGroup / kSplitWays;
  if (count == 28 || count == 32)
    return launch_skinny_split_kernel<kW4, kEpi, 4>(x, M, K, wq, meta, scales8, N, y, out_f32, ep, stream);
  return launch_skinny_split_kernel<kW4, kEpi, 0>(x, M, K, wq, meta, scales8, N, y, out_f32, ep, stream);
}

#ifndef AJQ_SKINNY_FORCE_NT
#define AJQ_SKINNY_FORCE_NT 0
#endif

// M >= 17.  Row blocks of 32 rows of M and 1, 2 or 4 row tiles of N per workgroup.  A workgroup
// moves K * (2 * 32 + bytes per weight * 16 * tiles) bytes (the activations come from L2 once per
// workgroup, so more row tiles mean less traffic per output) and the CUs take the workgroups in
// rounds: the tile count with the smallest rounds x bytes wins (384 row tiles as 192 workgroups of
// two run in one round instead of two: 14.7 -> 11.2 us at M = 32, K = 4096).  Wider row blocks
// lose to more row tiles on the same count.
// row tiles per workgroup of the weight-streaming kernel (see launch_skinny)
template <bool kW4>
int skinny_row_tiles(int M, int N) {
  const int ntiles = N / kTileN;
  const int mblocks = (M + 31) / 32;
  int nt = 1;
  long long best = 0;
  for (int c = 1; c <= 4; c *= 2) {
    const long long wgs = (long long)((ntiles + c - 1) / c) * mblocks;
    const int slots = (c == 4 && (ntiles / 4) * mblocks >= AJQ_SKINNY_FOUR_WAVE_MIN) ? 512 : 256;  // four-wave workgroups share a CU
    const long long cost = ((wgs + slots - 1) / slots) * (64 + (kW4 ? 8 : 16) * c);
    if (c == 1 || cost < best) {
      best = cost;
      nt = c;
    }
  }
  return AJQ_SKINNY_FORCE_NT ? AJQ_SKINNY_FORCE_NT : nt;
}

// the same choice of configuration for the kernel's epilogue forms (row scale / residual / gate)
template <bool kW4, int kEpi>
int launch_skinny_epi(const uint16_t* x, int M, int K, const uint32_t* wq, const uint32_t* meta, const uint16_t* scales8,
                      int N, void* y, int out_f32, const GemvEpilogue& ep, hipStream_t stream) {
  if (skinny_split_applies(M, N, K)) return launch_skinny_split<kW4, kEpi>(x, M, K, wq, meta, scales8, N, y, out_f32, ep, stream);
  if (const int T = skinny_resident_tiles<kW4, 2>(M, N, K))
    return launch_skinny_resident<kW4, kEpi, 2>(T, x, M, K, wq, meta, scales8, N, y, out_f32, ep, stream);
  const int nt = skinny_row_tiles<kW4>(M, N);
  const int ntiles = N / kTileN, mblocks = (M + 31) / 32;
  if (nt == 1) return launch_skinny_epi_cfg<8, 2, 32, 1, kW4, kEpi>(x, M, K, wq, meta, scales8, N, y, out_f32, ep, stream);
  if (nt == 2) return launch_skinny_epi_cfg<8, 1, 32, 2, kW4, kEpi>(x, M, K, wq, meta, scales8, N, y, out_f32, ep, stream);
  if ((ntiles / 4) * mblocks >= AJQ_SKINNY_FOUR_WAVE_MIN)
    return launch_skinny_epi_cfg<4, 1, 32, 4, kW4, kEpi>(x, M, K, wq, meta, scales8, N, y, out_f32, ep, stream);
  return launch_skinny_epi_cfg<8, 1, 32, 4, kW4, kEpi>(x, M, K, wq, meta, scales8, N, y, out_f32, ep, stream);
}

template <bool kW4>
int launch_skinny(const uint16_t* x, int M, int K, const uint32_t* wq, const uint32_t* meta,
                  const uint16_t* scales8, int N, void* y, int out_f32, hipStream_t stream) {
  if (skinny_split_applies(M, N, K))
    return launch_skinny_split<kW4, 0>(x, M, K, wq, meta, scales8, N, y, out_f32, GemvEpilogue{}, stream);
  if (const int T = skinny_resident_tiles<kW4, 2>(M, N, K))
    return launch_skinny_resident<kW4, 0, 2>(T, x, M, K, wq, meta, scales8, N, y, out_f32, GemvEpilogue{}, stream);
  const int ntiles = N / kTileN;
  const int mblocks = (M + 31) / 32;
  int nt = 1;
  long long best = 0;
  for (int c = 1; c <= 4; c *= 2) {
    const long long wgs = (long long)((ntiles + c - 1) / c) * mblocks;
    const int slots = (c == 4 && (ntiles / 4) * mblocks >= AJQ_SKINNY_FOUR_WAVE_MIN) ? 512 : 256;  // four-wave workgroups share a CU
    const long long cost = ((wgs + slots - 1) / slots) * (64 + (kW4 ? 8 : 16) * c);
    if (c == 1 || cost < best) {
      best = cost;
      nt = c;
    }
  }
  if (AJQ_SKINNY_FORCE_NT) nt = AJQ_SKINNY_FORCE_NT;
  if (nt == 1) return launch_skinny_cfg<8, 2, 32, 1, kW4>(x, M, K, wq, meta, scales8, N, y, out_f32, stream);
  if (nt == 2) return launch_skinny_cfg<8, 1, 32, 2, kW4>(x, M, K, wq, meta, scales8, N, y, out_f32, stream);
  // two workgroups of four waves per CU once there are that many: one's start-up and
  // reduction overlap the other's arithmetic (12-15 % faster than one of eight waves)
  if ((ntiles / 4) * mblocks >= AJQ_SKINNY_FOUR_WAVE_MIN)
    return launch_skinny_cfg<4, 1, 32, 4, kW4>(x, M, K, wq, meta, scales8, N, y, out_f32, stream);
  return launch_skinny_cfg<8, 1, 32, 4, kW4>(x, M, K, wq, meta, scales8, N, y, out_f32, stream);
}

// ---- GEMV with work around the matmul for batched decode steps (row scale of a norm on the way out,
// residual add with the next norm's preparation, SwiGLU gate): straight-line configurations only,
// row bound 8 or 16
template <int kWaves, int TPW, int MROWS, bool kW4, int kEpi>
int launch_gemv_epi_cfg(const uint16_t* x, int M, int K, const uint32_t* wq, const uint32_t* meta, const uint16_t* scales8,
                        int N, void* y, int out_f32, const GemvEpilogue& ep, hipStream_t stream) {
  constexpr size_t lds = gemv_epi_lds_bytes(kWaves, TPW, MROWS);
  static_assert(lds <= 160 * 1024, "GEMV configuration exceeds the 160 KiB LDS of a CU");
  auto kernel = dequant_gemv_epi_kernel<kWaves, TPW, MROWS, kW4, true, kEpi, false>;
  if (TPW <= 4 && N / kTileN <= kGemvFragWorkgroups) kernel = dequant_gemv_epi_kernel<kWaves, TPW, MROWS, kW4, true, kEpi, TPW <= 4>;
  if (int s = allow_big_lds(kernel, lds)) return s;
  hipLaunchKernelGGL(kernel, dim3(N / kTileN), dim3(kWaves * 64), lds, stream, reinterpret_cast<const u32x4_t*>(wq),
                     meta, x, K, M | (out_f32 << 8), N, y, scales8, ep);
  return AJQ_OK;
}

constexpr int kMaxEpiM = 255;  // above the GEMV range the weight-streaming kernel carries the same epilogues
// whether the GEMV kernel's straight-line configurations take (M, K); everything else goes to the streaming kernel
bool gemv_epi_straight(int M, int K) {
  return M <= kMaxGemvM && (K == 2048 || K == 4096 || (K == 5632 && M <= 8));
}
bool gemv_epi_supported(int M, int K) { return M >= 1 && M <= kMaxEpiM && K >= kGroup && K % kGroup == 0; }
// the row-scale consumer adds the K / 16 per-tile sums of squares with 32 per wave: eight waves cover 256 of them
// (K <= 4096), the eleven of the straight-line K = 5632 configuration 352
int gemv_rowscale_max_parts(int M, int K) { return (gemv_epi_straight(M, K) && K == 5632) ? 11 * 32 : 8 * 32; }
bool gemv_rowscale_supported(int M, int K) { return gemv_epi_supported(M, K) && K / 16 <= gemv_rowscale_max_parts(M, K); }

template <bool kW4, int kEpi>
int launch_gemv_epi(const uint16_t* x, int M, int K, const uint32_t* wq, const uint32_t* meta, const uint16_t* scales8,
                    int N, void* y, int out_f32, const GemvEpilogue& ep, hipStream_t stream) {
  if (gemv_split_applies(M, N, K)) return launch_gemv_split<kW4, kEpi>(x, M, K, wq, meta, scales8, N, y, out_f32, ep, stream);
  if (!gemv_epi_straight(M, K)) return launch_skinny_epi<kW4, kEpi>(x, M, K, wq, meta, scales8, N, y, out_f32, ep, stream);
  if (gemv_takes_resident(M, N, K))
    return launch_skinny_resident<kW4, kEpi, 1>(skinny_resident_tiles<kW4, 1>(M, N, K), x, M, K, wq, meta, scales8, N, y, out_f32, ep,
                                                stream);
#define AJQ_EPI(W, T, R) return launch_gemv_epi_cfg<W, T, R, kW4, kEpi>(x, M, K, wq, meta, scales8, N, y, out_f32, ep, stream)
  if (K == 2048) {
    if (M <= 1) AJQ_EPI(8, 2, 1);
    if (M <= 4) AJQ_EPI(8, 2, 4);
    if (M <= 8) AJQ_EPI(8, 2, 8);
    AJQ_EPI(8, 2, 16);
  }
  if (K == 4096) {
    if (M <= 1) AJQ_EPI(8, 4, 1);
    if (M <= 4) AJQ_EPI(8, 4, 4);
    if (M <= 8) AJQ_EPI(8, 4, 8);
    AJQ_EPI(8, 4, 16);
  }
  if (M <= 1) AJQ_EPI(11, 4, 1);
  if (M <= 4) AJQ_EPI(11, 4, 4);
  AJQ_EPI(11, 4, 8);
#undef AJQ_EPI
}

int check_epi(const char* name, int M, int K) {
  if (!gemv_epi_supported(M, K))
    return fail(AJQ_ERR_UNSUPPORTED, "%s: M=%d, K=%d is not built (ajq_gemv_epilogue_supported)", name, M, K);
  return AJQ_OK;
}

template <bool kW4>
int gemv_rowscale(const char* name, const uint16_t* xt, const float* ssq, int parts, float eps, int M, int K,
                         const uint32_t* wq, const void* aux, int N, void* y, int out_dtype, int gate, void* stream) {
  if (int s = check_matmul_args(name, xt, M, K, wq, aux, N, y, out_dtype, kGroup)) return s;
  if (int s = check_epi(name, M, K)) return s;
  if (!gemv_rowscale_supported(M, K))
    return fail(AJQ_ERR_UNSUPPORTED, "%s: M=%d, K=%d has more than %d tile sums per row (ajq_gemv_rowscale_supported)", name,
                M, K, gemv_rowscale_max_parts(M, K));
  if (!ssq || !aligned16(ssq)) return fail(ssq ? AJQ_ERR_ALIGN : AJQ_ERR_NULL, "%s: ssq must be non-null and 16-byte aligned", name);
  if (parts != K / 16) return fail(AJQ_ERR_SHAPE, "%s: parts=%d must be K / 16 = %d", name, parts, K / 16);
  if (gate && out_dtype != AJQ_OUT_BF16) return fail(AJQ_ERR_UNSUPPORTED, "%s: the gated output is bf16", name);
  GemvEpilogue ep{};
  ep.ssq_in = ssq;
  ep.parts = parts;
  ep.inv_k = 1.0f / (float)K;
  ep.eps = eps;
  const uint32_t* meta = kW4 ? static_cast<const uint32_t*>(aux) : nullptr;
  const uint16_t* scales = kW4 ? nullptr : static_cast<const uint16_t*>(aux);
  const int s = gate ? launch_gemv_epi<kW4, kEpiRowScale | kEpiGate>(xt, M, K, wq, meta, scales, N, y, 0, ep, (hipStream_t)stream)
                     : launch_gemv_epi<kW4, kEpiRowScale>(xt, M, K, wq, meta, scales, N, y, out_dtype == AJQ_OUT_F32, ep,
                                                          (hipStream_t)stream);
  if (s) return s;
  return check_launch(name);
}

template <bool kW4>
int gemv_gated(const char* name, const uint16_t* x, int M, int K, const uint32_t* wq, const void* aux, int N, void* y,
               void* stream) {
  if (int s = check_matmul_args(name, x, M, K, wq, aux, N, y, AJQ_OUT_BF16, kGroup)) return s;
  if (int s = check_epi(name, M, K)) return s;
  const uint32_t* meta = kW4 ? static_cast<const uint32_t*>(aux) : nullptr;
  const uint16_t* scales = kW4 ? nullptr : static_cast<const uint16_t*>(aux);
  if (int s = launch_gemv_epi<kW4, kEpiGate>(x, M, K, wq, meta, scales, N, y, 0, GemvEpilogue{}, (hipStream_t)stream)) return s;
  return check_launch(name);
}

template <bool kW4>
int gemv_residual(const char* name, const uint16_t* x, int M, int K, const uint32_t* wq, const void* aux, int N,
                         const float* h_in, const float* gain, float* h_out, uint16_t* xt_out, float* ssq_out, void* stream) {
  if (int s = check_matmul_args(name, x, M, K, wq, aux, N, h_out, AJQ_OUT_F32, kGroup)) return s;
  if (int s = check_epi(name, M, K)) return s;
  if (!h_in || !gain || !ssq_out) return fail(AJQ_ERR_NULL, "%s: null pointer argument", name);
  if (h_in == h_out) return fail(AJQ_ERR_NULL, "%s: h_out must be a buffer other than h_in", name);
  GemvEpilogue ep{};
  ep.h_in = h_in;
  ep.gain = gain;
  ep.h_out = h_out;
  ep.xt = xt_out;
  ep.ssq_out = ssq_out;
  const uint32_t* meta = kW4 ? static_cast<const uint32_t*>(aux) : nullptr;
  const uint16_t* scales = kW4 ? nullptr : static_cast<const uint16_t*>(aux);
  if (int s = launch_gemv_epi<kW4, kEpiResidual>(x, M, K, wq, meta, scales, N, nullptr, 1, ep, (hipStream_t)stream)) return s;
  return check_launch(name);
}

// ---- GEMV with the activations produced on the way in (norm / gate prologue)
template <int kWaves, int TPW, int MROWS, bool kW4, int kPro, int kOut = 0>
int launch_gemv_pro_cfg(int M, int K, const uint32_t* wq, const uint32_t* meta, const uint16_t* scales8, int N, void* y,
                        int out_f32, const float* src0, const float* src1, const float* gain, float eps, float* h_out,
                        hipStream_t stream, int S = 0) {
  constexpr size_t lds = gemv_pro_lds_bytes(kWaves, TPW, MROWS);
  static_assert(lds <= 160 * 1024, "GEMV configuration exceeds the 160 KiB LDS of a CU");
  auto kernel = dequant_gemv_pro_kernel<kWaves, TPW, MROWS, kW4, kPro, kOut>;
  if (int s = allow_big_lds(kernel, lds)) return s;
  hipLaunchKernelGGL(kernel, dim3(N / kTileN), dim3(kWaves * 64), lds, stream, reinterpret_cast<const u32x4_t*>(wq),
                     meta, K, M | (out_f32 << 8), N, y, scales8, src0, src1, gain, eps, h_out, S, nullptr, nullptr, nullptr);
  return AJQ_OK;
}

// the merge prologue with the residual epilogue (output projection of a decode step)
template <int TPW, int MROWS, bool kW4>
int launch_gemv_merge_resid_cfg(int M, int K, const uint32_t* wq, const uint32_t* meta, const uint16_t* scales8, int N,
                                const float* partial, int S, const float* h_in, const float* gain, float* h_out,
                                uint16_t* xt, float* ssq, hipStream_t stream) {
  constexpr size_t lds = gemv_pro_lds_bytes(8, TPW, MROWS);
  auto kernel = dequant_gemv_pro_kernel<8, TPW, MROWS, kW4, kProMerge, kOutResid>;
  if (int s = allow_big_lds(kernel, lds)) return s;
  hipLaunchKernelGGL(kernel, dim3(N / kTileN), dim3(8 * 64), lds, stream, reinterpret_cast<const u32x4_t*>(wq), meta, K,
                     M | (1 << 8), N, nullptr, scales8, partial, nullptr, gain, 0.f, h_out, S, h_in, xt, ssq);
  return AJQ_OK;
}

// K = waves * TPW * 128 for (8, 1), (8, 2), (8, 4), (11, 4) waves x groups; the row bound times
// TPW stays <= 32 (eight loads of fp32 sources per lane: more would not fit the registers).
bool gemv_pro_supported(int M, int K) {
  if (M < 1) return false;
  if (K == 1024) return M <= 16;
  if (K == 2048) return M <= 16;
  if (K == 4096 || K == 5632) return M <= 8;
  return false;
}

template <bool kW4, int kPro, int kOut = 0>
int launch_gemv_pro(int M, int K, const uint32_t* wq, const uint32_t* meta, const uint16_t* scales8, int N, void* y,
                    int out_f32, const float* src0, const float* src1, const float* gain, float eps, float* h_out,
                    hipStream_t stream, int S = 0) {
#define AJQ_PRO(W, T, R)                                                                                              \
  return launch_gemv_pro_cfg<W, T, R, kW4, kPro, kOut>(M, K, wq, meta, scales8, N, y, out_f32, src0, src1, gain, eps, \
                                                       h_out, stream, S)
  if (K == 1024) {
    if (M <= 1) AJQ_PRO(8, 1, 1);
    if (M <= 4) AJQ_PRO(8, 1, 4);
    if (M <= 8) AJQ_PRO(8, 1, 8);
    AJQ_PRO(8, 1, 16);
  }
  if (K == 2048) {
    if (M <= 1) AJQ_PRO(8, 2, 1);
    if (M <= 4) AJQ_PRO(8, 2, 4);
    if (M <= 8) AJQ_PRO(8, 2, 8);
    AJQ_PRO(8, 2, 16);
  }
  if (K == 4096) {
    if (M <= 1) AJQ_PRO(8, 4, 1);
    if (M <= 4) AJQ_PRO(8, 4, 4);
    AJQ_PRO(8, 4, 8);
  }
  if (M <= 1) AJQ_PRO(11, 4, 1);
  if (M <= 4) AJQ_PRO(11, 4, 4);
  AJQ_PRO(11, 4, 8);
#undef AJQ_PRO
}

// The output projection with the attention's row chunks merged on its way in: K = heads * 128 with
// K = 2048 (eight waves of two heads) or 4096 (eight waves of four); a lane holds at most
// merge_chunks_per_lane chunks of a (row, head), the four lane quarters every fourth chunk.
int gemv_merge_max_splits(int M, int K) {
  const int tpw = K == 2048 ? 2 : K == 4096 ? 4 : 0;
  if (!tpw || M < 1) return 0;
  const int mrows = M <= 1 ? 1 : M <= 2 ? 2 : M <= 4 ? 4 : 0;
  if (!mrows || mrows * tpw > 8) return 0;
  return 4 * merge_chunks_per_lane(mrows, tpw);
}

template <bool kW4>
int launch_gemv_merge(int M, int K, const uint32_t* wq, const uint32_t* meta, const uint16_t* scales8, int N, void* y,
                      int out_f32, const float* partial, int S, hipStream_t stream) {
#define AJQ_MRG(T, R) \
  return launch_gemv_pro_cfg<8, T, R, kW4, kProMerge>(M, K, wq, meta, scales8, N, y, out_f32, partial, nullptr, nullptr, \
                                                      0.f, nullptr, stream, S)
  if (K == 2048) {
    if (M <= 1) AJQ_MRG(2, 1);
    if (M <= 2) AJQ_MRG(2, 2);
    AJQ_MRG(2, 4);
  }
  if (M <= 1) AJQ_MRG(4, 1);
  AJQ_MRG(4, 2);
#undef AJQ_MRG
}

template <bool kW4>
int launch_gemv_merge_resid(int M, int K, const uint32_t* wq, const uint32_t* meta, const uint16_t* scales8, int N,
                            const float* partial, int S, const float* h_in, const float* gain, float* h_out, uint16_t* xt,
                            float* ssq, hipStream_t stream) {
#define AJQ_MRG(T, R) \
  return launch_gemv_merge_resid_cfg<T, R, kW4>(M, K, wq, meta, scales8, N, partial, S, h_in, gain, h_out, xt, ssq, stream)
  if (K == 2048) {
    if (M <= 1) AJQ_MRG(2, 1);
    if (M <= 2) AJQ_MRG(2, 2);
    AJQ_MRG(2, 4);
  }
  if (M <= 1) AJQ_MRG(4, 1);
  AJQ_MRG(4, 2);
#undef AJQ_MRG
}

template <bool kW4>
int gemv_merge_residual(const char* name, const float* partial, int S, int M, int K, const uint32_t* wq, const void* aux,
                        int N, const float* h_in, const float* gain, float* h_out, uint16_t* xt_out, float* ssq_out,
                        void* stream) {
  if (int s = check_matmul_args(name, partial, M, K, wq, aux, N, h_out, AJQ_OUT_F32, kGroup)) return s;
  const int cap = gemv_merge_max_splits(M, K);
  if (cap == 0 || S < 1 || S > cap)
    return fail(AJQ_ERR_UNSUPPORTED, "%s: M=%d, K=%d, S=%d is not built (ajq_gemv_merge_max_splits gives %d)", name, M, K, S, cap);
  if (!h_in || !gain || !ssq_out) return fail(AJQ_ERR_NULL, "%s: null pointer argument", name);
  if (h_in == h_out) return fail(AJQ_ERR_NULL, "%s: h_out must be a buffer other than h_in", name);
  const uint32_t* meta = kW4 ? static_cast<const uint32_t*>(aux) : nullptr;
  const uint16_t* scales = kW4 ? nullptr : static_cast<const uint16_t*>(aux);
  if (int s = launch_gemv_merge_resid<kW4>(M, K, wq, meta, scales, N, partial, S, h_in, gain, h_out, xt_out, ssq_out,
                                           (hipStream_t)stream))
    return s;
  return check_launch(name);
}

template <bool kW4>
int gemv_norm_sums(const char* name, const float* h, const float* ssq, int parts, const float* gain, float eps, int M, int K,
                   const uint32_t* wq, const void* aux, int N, void* y, int out_dtype, int gate, void* stream) {
  if (int s = check_matmul_args(name, h, M, K, wq, aux, N, y, out_dtype, kGroup)) return s;
  if (!gemv_pro_supported(M, K))
    return fail(AJQ_ERR_UNSUPPORTED, "%s: M=%d, K=%d is not built (ajq_gemv_fused_supported)", name, M, K);
  if (!ssq || !gain || !aligned16(ssq) || !aligned16(gain))
    return fail(ssq && gain ? AJQ_ERR_ALIGN : AJQ_ERR_NULL, "%s: ssq and gain must be non-null and 16-byte aligned", name);
  if (parts != K / 16 || parts > 256)
    return fail(AJQ_ERR_SHAPE, "%s: parts=%d must be K / 16 = %d and at most 256", name, parts, K / 16);
  if (gate && out_dtype != AJQ_OUT_BF16) return fail(AJQ_ERR_UNSUPPORTED, "%s: the gated output is bf16", name);
  const uint32_t* meta = kW4 ? static_cast<const uint32_t*>(aux) : nullptr;
  const uint16_t* scales = kW4 ? nullptr : static_cast<const uint16_t*>(aux);
  const int s = gate ? launch_gemv_pro<kW4, kProNormSums, kOutGate>(M, K, wq, meta, scales, N, y, 0, h, ssq, gain, eps, nullptr,
                                                                    (hipStream_t)stream, parts)
                     : launch_gemv_pro<kW4, kProNormSums>(M, K, wq, meta, scales, N, y, out_dtype == AJQ_OUT_F32, h, ssq, gain,
                                                          eps, nullptr, (hipStream_t)stream, parts);
  if (s) return s;
  return check_launch(name);
}

int check_pro(const char* name, int M, int K, const void* a, const void* b) {
  if (!gemv_pro_supported(M, K))
    return fail(AJQ_ERR_UNSUPPORTED, "%s: M=%d, K=%d is not built (ajq_gemv_fused_supported)", name, M, K);
  if (!a || !aligned16(a) || (b && !aligned16(b)))
    return fail(a ? AJQ_ERR_ALIGN : AJQ_ERR_NULL, "%s: the fp32 sources must be non-null and 16-byte aligned", name);
  return AJQ_OK;
}

// Which kernel runs a matmul of M >= 17 rows.  All three times are modelled from measurements
// at K = 4096 (microseconds per k-block of 128 and round of 256 workgroups, one workgroup per CU).
//  * 256 x 128 tiles: about 1.8 us.
//  * 128 x 128 tiles (M >= 128): about 1.25 us (W4) / 1.15 us (W8): they win where the big tiles
//    leave CUs idle (M = 1024 on N = 4096 is 128 big tiles or 256 small ones).
//  * the weight-streaming kernel sustains about 400 TFLOP/s for M >= 256 and is the only one below
//    M = 128.
#ifndef AJQ_GEMM_TILE
#define AJQ_GEMM_TILE 0  // 0: by the estimate; 128 or 256: that tile kernel for every M it can run
#endif
enum MatmulKernel { kStreaming, kTiles256, kTiles128 };
MatmulKernel pick_matmul_kernel(int M, int N, int K, bool w4) {
  if (AJQ_GEMM_TILE == 128 && M >= kG1BM) return kTiles128;
  if (AJQ_GEMM_TILE == 256 && M >= kG2BM) return kTiles256;
  if (M < kG1BM) return kStreaming;
  const double G = (double)(K / kGroup);
  const double us_stream = 2.0 * M * N * (double)K / 400e6;
  double us_big = 1e30;
  if (M >= kGemm256MinM) {
    const long long tiles = (long long)((M + kG2BM - 1) / kG2BM) * ((N + kG2BN - 1) / kG2BN);
    us_big = (double)((tiles + 255) / 256) * G * 1.8 + 3.0;
  }
  const long long small_ = (long long)((M + kG1BM - 1) / kG1BM) * ((N + kG1BN - 1) / kG1BN);
  const double us_small = (double)((small_ + 255) / 256) * G * (w4 ? 1.25 : 1.15) + 5.0;
  if (us_stream <= us_big && us_stream <= us_small) return kStreaming;
  return us_small < us_big ? kTiles128 : kTiles256;
}

}  // namespace

extern "C" {

int ajq_w4a16_gemv(const uint16_t* x, int M, int K, const uint32_t* wq, const uint32_t* meta, int N, void* y,
                   int out_dtype, void* stream) {
  if (int s = check_matmul_args("ajq_w4a16_gemv", x, M, K, wq, meta, N, y, out_dtype, kGroup)) return s;
  if (M > kMaxGemvM) return fail(AJQ_ERR_SHAPE, "ajq_w4a16_gemv: M=%d exceeds %d; use ajq_w4a16_gemm", M, kMaxGemvM);
  if (int s = launch_gemv<true>(x, M, K, wq, meta, nullptr, N, y, out_dtype == AJQ_OUT_F32, (hipStream_t)stream))
    return s;
  return check_launch("ajq_w4a16_gemv");
}

int ajq_w8a16_gemv(const uint16_t* x, int M, int K, const uint32_t* wq, const uint16_t* scales, int N, void* y,
                   int out_dtype, void* stream) {
  if (int s = check_matmul_args("ajq_w8a16_gemv", x, M, K, wq, scales, N, y, out_dtype, kGroup)) return s;
  if (M > kMaxGemvM) return fail(AJQ_ERR_SHAPE, "ajq_w8a16_gemv: M=%d exceeds %d; use ajq_w8a16_gemm", M, kMaxGemvM);
  if (int s = launch_gemv<false>(x, M, K, wq, nullptr, scales, N, y, out_dtype == AJQ_OUT_F32, (hipStream_t)stream))
    return s;
  return check_launch("ajq_w8a16_gemv");
}

int ajq_gemv_fused_supported(int M, int K) { return gemv_pro_supported(M, K) ? 1 : 0; }

int ajq_gemv_epilogue_supported(int M, int K) { return gemv_epi_supported(M, K) ? 1 : 0; }

int ajq_gemv_rowscale_supported(int M, int K) { return gemv_rowscale_supported(M, K) ? 1 : 0; }

size_t ajq_matmul_workspace_bytes(void) { return kSplitWorkspaceBytes; }

int ajq_matmul_workspace_set(void* workspace, size_t bytes) {
  if (!workspace) {
    g_split_ws = SplitWorkspace{};
    return AJQ_OK;
  }
  if (!aligned16(workspace)) return fail(AJQ_ERR_ALIGN, "ajq_matmul_workspace_set: workspace must be 16-byte aligned");
  if (bytes < kSplitWorkspaceBytes)
    return fail(AJQ_ERR_WORKSPACE, "ajq_matmul_workspace_set: %zu bytes needed, %zu given", kSplitWorkspaceBytes, bytes);
  g_split_ws.base = workspace;
  g_split_ws.bytes = bytes;
  return AJQ_OK;
}

int ajq_w4a16_gemv_gated(const uint16_t* x, int M, int K, const uint32_t* wq, const uint32_t* meta, int N, void* y,
                         void* stream) {
  return gemv_gated<true>("ajq_w4a16_gemv_gated", x, M, K, wq, meta, N, y, stream);
}

int ajq_w8a16_gemv_gated(const uint16_t* x, int M, int K, const uint32_t* wq, const uint16_t* scales, int N, void* y,
                         void* stream) {
  return gemv_gated<false>("ajq_w8a16_gemv_gated", x, M, K, wq, scales, N, y, stream);
}

int ajq_w4a16_gemv_norm_sums(const float* h, const float* ssq, int parts, const float* gain, float eps, int M, int K,
                             const uint32_t* wq, const uint32_t* meta, int N, void* y, int out_dtype, int gate,
                             void* stream) {
  return gemv_norm_sums<true>("ajq_w4a16_gemv_norm_sums", h, ssq, parts, gain, eps, M, K, wq, meta, N, y, out_dtype, gate,
                              stream);
}

int ajq_w8a16_gemv_norm_sums(const float* h, const float* ssq, int parts, const float* gain, float eps, int M, int K,
                             const uint32_t* wq, const uint16_t* scales, int N, void* y, int out_dtype, int gate,
                             void* stream) {
  return gemv_norm_sums<false>("ajq_w8a16_gemv_norm_sums", h, ssq, parts, gain, eps, M, K, wq, scales, N, y, out_dtype, gate,
                               stream);
}

int ajq_w4a16_gemv_rowscale(const uint16_t* xt, const float* ssq, int parts, float eps, int M, int K, const uint32_t* wq,
                            const uint32_t* meta, int N, void* y, int out_dtype, int gate, void* stream) {
  return gemv_rowscale<true>("ajq_w4a16_gemv_rowscale", xt, ssq, parts, eps, M, K, wq, meta, N, y, out_dtype, gate, stream);
}

int ajq_w8a16_gemv_rowscale(const uint16_t* xt, const float* ssq, int parts, float eps, int M, int K, const uint32_t* wq,
                            const uint16_t* scales, int N, void* y, int out_dtype, int gate, void* stream) {
  return gemv_rowscale<false>("ajq_w8a16_gemv_rowscale", xt, ssq, parts, eps, M, K, wq, scales, N, y, out_dtype, gate, stream);
}

int ajq_w4a16_gemv_residual(const uint16_t* x, int M, int K, const uint32_t* wq, const uint32_t* meta, int N,
                            const float* h_in, const float* gain, float* h_out, uint16_t* xt_out, float* ssq_out,
                            void* stream) {
  return gemv_residual<true>("ajq_w4a16_gemv_residual", x, M, K, wq, meta, N, h_in, gain, h_out, xt_out, ssq_out, stream);
}

int ajq_w8a16_gemv_residual(const uint16_t* x, int M, int K, const uint32_t* wq, const uint16_t* scales, int N,
                            const float* h_in, const float* gain, float* h_out, uint16_t* xt_out, float* ssq_out,
                            void* stream) {
  return gemv_residual<false>("ajq_w8a16_gemv_residual", x, M, K, wq, scales, N, h_in, gain, h_out, xt_out, ssq_out, stream);
}

int ajq_w4a16_gemv_norm(const float* h_in, const float* delta, const float* gain, float eps, float* h_out, int M, int K,
                        const uint32_t* wq, const uint32_t* meta, int N, void* y, int out_dtype, void* stream) {
  if (int s = check_matmul_args("ajq_w4a16_gemv_norm", h_in, M, K, wq, meta, N, y, out_dtype, kGroup)) return s;
  if (int s = check_pro("ajq_w4a16_gemv_norm", M, K, gain, delta)) return s;
  if (!h_out || !aligned16(h_out) || h_out == h_in)
    return fail(AJQ_ERR_NULL, "ajq_w4a16_gemv_norm: h_out must be a 16-byte aligned buffer other than h_in");
  if (int s = launch_gemv_pro<true, kProNorm>(M, K, wq, meta, nullptr, N, y, out_dtype == AJQ_OUT_F32, h_in, delta, gain,
                                              eps, h_out, (hipStream_t)stream))
    return s;
  return check_launch("ajq_w4a16_gemv_norm");
}

int ajq_w8a16_gemv_norm(const float* h_in, const float* delta, const float* gain, float eps, float* h_out, int M, int K,
                        const uint32_t* wq, const uint16_t* scales, int N, void* y, int out_dtype, void* stream) {
  if (int s = check_matmul_args("ajq_w8a16_gemv_norm", h_in, M, K, wq, scales, N, y, out_dtype, kGroup)) return s;
  if (int s = check_pro("ajq_w8a16_gemv_norm", M, K, gain, delta)) return s;
  if (!h_out || !aligned16(h_out) || h_out == h_in)
    return fail(AJQ_ERR_NULL, "ajq_w8a16_gemv_norm: h_out must be a 16-byte aligned buffer other than h_in");
  if (int s = launch_gemv_pro<false, kProNorm>(M, K, wq, nullptr, scales, N, y, out_dtype == AJQ_OUT_F32, h_in, delta,
                                               gain, eps, h_out, (hipStream_t)stream))
    return s;
  return check_launch("ajq_w8a16_gemv_norm");
}

int ajq_w4a16_gemv_gate(const float* ab, int M, int K, const uint32_t* wq, const uint32_t* meta, int N, void* y,
                        int out_dtype, void* stream) {
  if (int s = check_matmul_args("ajq_w4a16_gemv_gate", ab, M, K, wq, meta, N, y, out_dtype, kGroup)) return s;
  if (int s = check_pro("ajq_w4a16_gemv_gate", M, K, ab, nullptr)) return s;
  if (int s = launch_gemv_pro<true, kProGate>(M, K, wq, meta, nullptr, N, y, out_dtype == AJQ_OUT_F32, ab, nullptr,
                                              nullptr, 0.f, nullptr, (hipStream_t)stream))
    return s;
  return check_launch("ajq_w4a16_gemv_gate");
}

int ajq_w8a16_gemv_gate(const float* ab, int M, int K, const uint32_t* wq, const uint16_t* scales, int N, void* y,
                        int out_dtype, void* stream) {
  if (int s = check_matmul_args("ajq_w8a16_gemv_gate", ab, M, K, wq, scales, N, y, out_dtype, kGroup)) return s;
  if (int s = check_pro("ajq_w8a16_gemv_gate", M, K, ab, nullptr)) return s;
  if (int s = launch_gemv_pro<false, kProGate>(M, K, wq, nullptr, scales, N, y, out_dtype == AJQ_OUT_F32, ab, nullptr,
                                               nullptr, 0.f, nullptr, (hipStream_t)stream))
    return s;
  return check_launch("ajq_w8a16_gemv_gate");
}

int ajq_gemv_merge_max_splits(int M, int K) { return gemv_merge_max_splits(M, K); }

int ajq_w4a16_gemv_merge(const float* partial, int S, int M, int K, const uint32_t* wq, const uint32_t* meta, int N,
                         void* y, int out_dtype, void* stream) {
  if (int s = check_matmul_args("ajq_w4a16_gemv_merge", partial, M, K, wq, meta, N, y, out_dtype, kGroup)) return s;
  const int cap = gemv_merge_max_splits(M, K);
  if (cap == 0 || S < 1 || S > cap)
    return fail(AJQ_ERR_UNSUPPORTED, "ajq_w4a16_gemv_merge: M=%d, K=%d, S=%d is not built (ajq_gemv_merge_max_splits gives %d)",
                M, K, S, cap);
  if (int s = launch_gemv_merge<true>(M, K, wq, meta, nullptr, N, y, out_dtype == AJQ_OUT_F32, partial, S,
                                      (hipStream_t)stream))
    return s;
  return check_launch("ajq_w4a16_gemv_merge");
}

int ajq_w8a16_gemv_merge(const float* partial, int S, int M, int K, const uint32_t* wq, const uint16_t* scales, int N,
                         void* y, int out_dtype, void* stream) {
  if (int s = check_matmul_args("ajq_w8a16_gemv_merge", partial, M, K, wq, scales, N, y, out_dtype, kGroup)) return s;
  const int cap = gemv_merge_max_splits(M, K);
  if (cap == 0 || S < 1 || S > cap)
    return fail(AJQ_ERR_UNSUPPORTED, "ajq_w8a16_gemv_merge: M=%d, K=%d, S=%d is not built (ajq_gemv_merge_max_splits gives %d)",
                M, K, S, cap);
  if (int s = launch_gemv_merge<false>(M, K, wq, nullptr, scales, N, y, out_dtype == AJQ_OUT_F32, partial, S,
                                       (hipStream_t)stream))
    return s;
  return check_launch("ajq_w8a16_gemv_merge");
}

int ajq_w4a16_gemv_merge_residual(const float* partial, int S, int M, int K, const uint32_t* wq, const uint32_t* meta, int N,
                                  const float* h_in, const float* gain, float* h_out, uint16_t* xt_out, float* ssq_out,
                                  void* stream) {
  return gemv_merge_residual<true>("ajq_w4a16_gemv_merge_residual", partial, S, M, K, wq, meta, N, h_in, gain, h_out, xt_out,
                                   ssq_out, stream);
}

int ajq_w8a16_gemv_merge_residual(const float* partial, int S, int M, int K, const uint32_t* wq, const uint16_t* scales,
                                  int N, const float* h_in, const float* gain, float* h_out, uint16_t* xt_out,
                                  float* ssq_out, void* stream) {
  return gemv_merge_residual<false>("ajq_w8a16_gemv_merge_residual", partial, S, M, K, wq, scales, N, h_in, gain, h_out,
                                    xt_out, ssq_out, stream);
}

// --------------------------------------------------------------- GEMM -----
size_t ajq_w4a16_gemm_workspace_bytes(int M, int K) {
  if (M < kG1BM || K < kGroup) return 0;  // only the 128 x 128 tile kernel needs the group sums
  return (size_t)(K / kGroup) * M * 16;
}

size_t ajq_w4a16_gemm_workspace_bytes_for(int M, int N, int K) {
  if (M <= kMaxGemvM || N < 1 || K < kGroup || pick_matmul_kernel(M, N, K, true) != kTiles128) return 0;
  return ajq_w4a16_gemm_workspace_bytes(M, K);
}

int ajq_w4a16_gemm(const uint16_t* x, int M, int K, const uint32_t* wq, const uint32_t* meta, int N, void* y,
                   int out_dtype, void* workspace, size_t workspace_bytes, void* stream) {
  if (int s = check_matmul_args("ajq_w4a16_gemm", x, M, K, wq, meta, N, y, out_dtype, kGroup)) return s;
  const bool out_f32 = out_dtype == AJQ_OUT_F32;
  const MatmulKernel which = M <= kMaxGemvM ? kStreaming : pick_matmul_kernel(M, N, K, true);
  if (which == kStreaming) {
    const int s = M <= kMaxGemvM ? launch_gemv<true>(x, M, K, wq, meta, nullptr, N, y, out_f32, (hipStream_t)stream)
                                 : launch_skinny<true>(x, M, K, wq, meta, nullptr, N, y, out_f32, (hipStream_t)stream);
    return s ? s : check_launch("ajq_w4a16_gemm");
  }
  if ((long long)M * K * 2 >= (1LL << 32))
    return fail(AJQ_ERR_SHAPE, "ajq_w4a16_gemm: M * K = %lld exceeds the 32-bit activation offsets", (long long)M * K);
  if (which == kTiles256) {  // zero-points are subtracted when the weights are unpacked: no group sums, one launch
    if (int s = launch_gemm256<true>(x, M, K, wq, meta, nullptr, N, y, out_f32, (hipStream_t)stream)) return s;
    return check_launch("ajq_w4a16_gemm");
  }
  const size_t need = ajq_w4a16_gemm_workspace_bytes(M, K);
  if (!workspace || workspace_bytes < need)
    return fail(AJQ_ERR_WORKSPACE, "ajq_w4a16_gemm: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
  if (!aligned16(workspace)) return fail(AJQ_ERR_ALIGN, "ajq_w4a16_gemm: workspace must be 16-byte aligned");
  const long long teams4 = (long long)M * ((K / kGroup + 3) / 4);
  hipLaunchKernelGGL(group_sum3_kernel, dim3((unsigned)((teams4 + 15) / 16)), dim3(256), 0, (hipStream_t)stream, x, M,
                     K, reinterpret_cast<u32x4_t*>(workspace));
  if (int s = launch_gemm128<true>(x, M, K, wq, meta, nullptr, workspace, N, y, out_f32, (hipStream_t)stream)) return s;
  return check_launch("ajq_w4a16_gemm");
}

size_t ajq_noalloc_scratch_bytes(void) { return kScratchBytes; }

int ajq_w4a16_gemm_noalloc(const uint16_t* x, int M, int K, const uint32_t* wq, const uint32_t* meta, int N, void* y,
                           int out_dtype, void* stream) {
  if (M < 1 || K < 1) return fail(AJQ_ERR_SHAPE, "ajq_w4a16_gemm_noalloc: M and K must be positive (got %d, %d)", M, K);
  if (N < 1) return fail(AJQ_ERR_SHAPE, "ajq_w4a16_gemm_noalloc: N must be positive (got %d)", N);
  const size_t need = ajq_w4a16_gemm_workspace_bytes_for(M, N, K);
  if (need > kScratchBytes)
    return fail(AJQ_ERR_WORKSPACE,
                "ajq_w4a16_gemm_noalloc: M=%d, K=%d needs %zu bytes of group sums, the built-in scratch holds %zu "
                "(use ajq_w4a16_gemm with a caller workspace)", M, K, need, kScratchBytes);
  void* ptr = nullptr;
  if (int s = scratch_address(&ptr)) return s;
  return ajq_w4a16_gemm(x, M, K, wq, meta, N, y, out_dtype, ptr, kScratchBytes, stream);
}

int ajq_w8a16_gemm(const uint16_t* x, int M, int K, const uint32_t* wq, const uint16_t* scales, int N, void* y,
                   int out_dtype, void* stream) {
  if (int s = check_matmul_args("ajq_w8a16_gemm", x, M, K, wq, scales, N, y, out_dtype, kGroup)) return s;
  const bool out_f32 = out_dtype == AJQ_OUT_F32;
  const MatmulKernel which = M <= kMaxGemvM ? kStreaming : pick_matmul_kernel(M, N, K, false);
  if (which == kStreaming) {
    const int s = M <= kMaxGemvM ? launch_gemv<false>(x, M, K, wq, nullptr, scales, N, y, out_f32, (hipStream_t)stream)
                                 : launch_skinny<false>(x, M, K, wq, nullptr, scales, N, y, out_f32, (hipStream_t)stream);
    return s ? s : check_launch("ajq_w8a16_gemm");
  }
  if ((long long)M * K * 2 >= (1LL << 32))
    return fail(AJQ_ERR_SHAPE, "ajq_w8a16_gemm: M * K = %lld exceeds the 32-bit activation offsets", (long long)M * K);
  if (int s = which == kTiles128
                  ? launch_gemm128<false>(x, M, K, wq, nullptr, scales, nullptr, N, y, out_f32, (hipStream_t)stream)
                  : launch_gemm256<false>(x, M, K, wq, nullptr, scales, N, y, out_f32, (hipStream_t)stream))
    return s;
  return check_launch("ajq_w8a16_gemm");
}

// ---- w1 | w3 GEMM with the SwiGLU gate formed in the epilogue (tile kernels only)
int ajq_gemm_gate_supported(int M, int N2, int K, int w4) {
  if (M < kG1BM || N2 < 2 * 64 || N2 % 128 != 0 || K < kGroup || K % kGroup != 0) return 0;
  if (AJQ_G1_WN != 4) return 0;
  return pick_matmul_kernel(M, N2, K, w4 != 0) != kStreaming;
}

int ajq_w4a16_gemm_gate(const uint16_t* x, int M, int K, const uint32_t* wq, const uint32_t* meta, int N2, uint16_t* y,
                        void* workspace, size_t workspace_bytes, void* stream) {
  if (int s = check_matmul_args("ajq_w4a16_gemm_gate", x, M, K, wq, meta, N2, y, AJQ_OUT_BF16, kGroup)) return s;
  if (!ajq_gemm_gate_supported(M, N2, K, 1))
    return fail(AJQ_ERR_UNSUPPORTED, "ajq_w4a16_gemm_gate: M=%d, N=%d, K=%d is not a tile-kernel shape with N %% 128 == 0", M,
                N2, K);
  if ((long long)M * K * 2 >= (1LL << 32))
    return fail(AJQ_ERR_SHAPE, "ajq_w4a16_gemm_gate: M * K = %lld exceeds the 32-bit activation offsets", (long long)M * K);
  if (pick_matmul_kernel(M, N2, K, true) == kTiles256) {  // no group sums, no workspace
    if (int s = launch_gemm256<true, true>(x, M, K, wq, meta, nullptr, N2, y, 0, (hipStream_t)stream)) return s;
    return check_launch("ajq_w4a16_gemm_gate");
  }
  const size_t need = ajq_w4a16_gemm_workspace_bytes(M, K);
  if (!workspace || workspace_bytes < need)
    return fail(AJQ_ERR_WORKSPACE, "ajq_w4a16_gemm_gate: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
  if (!aligned16(workspace)) return fail(AJQ_ERR_ALIGN, "ajq_w4a16_gemm_gate: workspace must be 16-byte aligned");
  const long long teams4 = (long long)M * ((K / kGroup + 3) / 4);
  hipLaunchKernelGGL(group_sum3_kernel, dim3((unsigned)((teams4 + 15) / 16)), dim3(256), 0, (hipStream_t)stream, x, M,
                     K, reinterpret_cast<u32x4_t*>(workspace));
  if (int s = launch_gemm128<true, true>(x, M, K, wq, meta, nullptr, workspace, N2, y, 0, (hipStream_t)stream)) return s;
  return check_launch("ajq_w4a16_gemm_gate");
}

int ajq_w8a16_gemm_gate(const uint16_t* x, int M, int K, const uint32_t* wq, const uint16_t* scales, int N2, uint16_t* y,
                        void* stream) {
  if (int s = check_matmul_args("ajq_w8a16_gemm_gate", x, M, K, wq, scales, N2, y, AJQ_OUT_BF16, kGroup)) return s;
  if (!ajq_gemm_gate_supported(M, N2, K, 0))
    return fail(AJQ_ERR_UNSUPPORTED, "ajq_w8a16_gemm_gate: M=%d, N=%d, K=%d is not a tile-kernel shape with N %% 128 == 0", M,
                N2, K);
  if ((long long)M * K * 2 >= (1LL << 32))
    return fail(AJQ_ERR_SHAPE, "ajq_w8a16_gemm_gate: M * K = %lld exceeds the 32-bit activation offsets", (long long)M * K);
  if (int s = pick_matmul_kernel(M, N2, K, false) == kTiles128
                  ? launch_gemm128<false, true>(x, M, K, wq, nullptr, scales, nullptr, N2, y, 0, (hipStream_t)stream)
                  : launch_gemm256<false, true>(x, M, K, wq, nullptr, scales, N2, y, 0, (hipStream_t)stream))
    return s;
  return check_launch("ajq_w8a16_gemm_gate");
}

}  // extern "C"

// --------------------------------------------------- decode-step operators -----
namespace {
constexpr int kAttnMaxSplits = 16;
// Row chunks per cache head.  Measured on (batch x cache heads) = 32 ... 256 at contexts 640 ... 8192: the
// kernel is fastest with 500-800 workgroups in all (two to three per CU; targets of 512 ... 1024 are within
// 5 % of each other); more chunks only add start-up, in-workgroup merges and partial results.  A chunk keeps
// at least 32 rows.
constexpr int kAttnTargetWorkgroups = 768;
// From one (sequence, cache head) pair per CU on, one 1024-thread workgroup per pair reads the whole head:
// the chip is occupied without row chunks, and the merge launch and its partial results go away (256 pairs:
// 5-7 % faster than three chunks and a merge; 128 pairs: 8 % slower than six chunks and a merge).
constexpr int kAttnWholeHeadPairs = 256;
bool attn_whole_heads(int B, int Hkv) { return B * Hkv >= kAttnWholeHeadPairs; }
int attn_splits(int B, int Hkv, int max_len) {
  const int pairs = B * Hkv;
  if (attn_whole_heads(B, Hkv)) return 1;
  int s = (kAttnTargetWorkgroups + pairs / 2) / pairs;
  const int by_rows = max_len / 32;
  if (s > by_rows) s = by_rows;
  return s < 1 ? 1 : (s > kAttnMaxSplits ? kAttnMaxSplits : s);
}

// Caches of a launch above this many bytes (keys + values as allocated) are streamed: non-temporal loads,
// rows dealt to the chunks in blocks.  Below it they are read with ordinary loads, chunk by chunk, and
// stay in the 256 MB last-level cache between steps.  Measured on a 12-layer model's decode step: 12.6 MB
// per layer is 4 % slower streamed, 19 MB 1 % faster, 25 MB 3 % faster, 100 MB 5 % faster (the
// attention launch itself: 15-20 %).
constexpr long long kAttnStreamBytes = 16ll << 20;

template <int R, typename CacheT, bool kStep, int HD>
void launch_attn(const float* q, void* kcache, void* vcache, const long long* pos, int B, int H, int Hkv, int max_len,
                 float scale, int S, float* partial, uint16_t* out, const float* cosine, const float* sine,
                 hipStream_t stream) {
  const long long cache_bytes = 2ll * B * Hkv * max_len * HD * (long long)sizeof(CacheT);
  const bool streamed = cache_bytes > kAttnStreamBytes;
  if (attn_whole_heads(B, Hkv)) {  // S == 1 by attn_splits
    auto kernel = streamed ? attn_decode_kernel<R, CacheT, kStep, true, 16, HD>
                           : attn_decode_kernel<R, CacheT, kStep, false, 16, HD>;
    hipLaunchKernelGGL(kernel, dim3(B * Hkv, 1), dim3(1024), 0, stream, q, reinterpret_cast<CacheT*>(kcache),
                       reinterpret_cast<CacheT*>(vcache), pos, H, Hkv, max_len, scale, partial, out, cosine, sine);
    return;
  }
  auto kernel = streamed ? attn_decode_kernel<R, CacheT, kStep, true, 4, HD> : attn_decode_kernel<R, CacheT, kStep, false, 4, HD>;
  hipLaunchKernelGGL(kernel, dim3(B * Hkv, S), dim3(256), 0, stream, q,
                     reinterpret_cast<CacheT*>(kcache), reinterpret_cast<CacheT*>(vcache), pos, H, Hkv, max_len, scale,
                     partial, out, cosine, sine);
  if (S > 1 && out != nullptr)  // out == nullptr: the caller merges the chunks itself (ajq_w*a16_gemv_merge)
    hipLaunchKernelGGL(attn_merge_kernel<HD>, dim3(B * H), dim3(64), 0, stream, partial, S, out);
}

template <bool kStep, int HD>
auto pick_attn_hd(int R, int cache_dtype) {
  if (cache_dtype == AJQ_KV_F32)
    return R == 1 ? launch_attn<1, float, kStep, HD>
                  : R == 2 ? launch_attn<2, float, kStep, HD> : launch_attn<4, float, kStep, HD>;
  return R == 1 ? launch_attn<1, uint16_t, kStep, HD>
                : R == 2 ? launch_attn<2, uint16_t, kStep, HD> : launch_attn<4, uint16_t, kStep, HD>;
}
template <bool kStep>
auto pick_attn(int R, int cache_dtype, int head_dim) {
  return head_dim == 32 ? pick_attn_hd<kStep, 32>(R, cache_dtype)
                        : head_dim == 64 ? pick_attn_hd<kStep, 64>(R, cache_dtype) : pick_attn_hd<kStep, 128>(R, cache_dtype);
}
}  // namespace

extern "C" {

int ajq_add_rmsnorm(float* hidden, const float* delta, const float* gain, float eps, uint16_t* out, int B, int D,
                    void* stream) {
  if (!hidden || !gain || !out) return fail(AJQ_ERR_NULL, "ajq_add_rmsnorm: null pointer argument");
  if (B < 1 || D < 4 || D % 4 != 0)
    return fail(AJQ_ERR_SHAPE, "ajq_add_rmsnorm: need B >= 1 and D a positive multiple of 4 (got %d, %d)", B, D);
  if (!aligned16(hidden) || !aligned16(gain) || (delta && !aligned16(delta)) || (reinterpret_cast<uintptr_t>(out) & 7u))
    return fail(AJQ_ERR_ALIGN, "ajq_add_rmsnorm: hidden, delta, gain must be 16-byte and out 8-byte aligned");
  hipLaunchKernelGGL(add_rmsnorm_kernel, dim3(B), dim3(256), 0, (hipStream_t)stream, hidden, delta, gain, eps, out, D);
  return check_launch("ajq_add_rmsnorm");
}

int ajq_rope_cache(const float* qkv, const float* cosine, const float* sine, const int64_t* pos, float* q_out,
                   void* kcache, void* vcache, int cache_dtype, int B, int H, int Hkv, int head_dim, int max_len,
                   void* stream) {
  if (!qkv || !cosine || !sine || !pos || !q_out || !kcache || !vcache)
    return fail(AJQ_ERR_NULL, "ajq_rope_cache: null pointer argument");
  if (B < 1 || H < 1 || Hkv < 1 || H % Hkv != 0 || head_dim < 2 || head_dim % 2 != 0 || max_len < 1)
    return fail(AJQ_ERR_SHAPE, "ajq_rope_cache: unsupported shape (B=%d H=%d Hkv=%d head_dim=%d max_len=%d)", B, H, Hkv,
                head_dim, max_len);
  if (cache_dtype != AJQ_KV_F32 && cache_dtype != AJQ_KV_BF16)
    return fail(AJQ_ERR_UNSUPPORTED, "ajq_rope_cache: cache_dtype %d is neither AJQ_KV_F32 nor AJQ_KV_BF16", cache_dtype);
  const long long pairs = (long long)B * (H + 2 * Hkv) * (head_dim / 2);
  const dim3 grid((unsigned)((pairs + 255) / 256));
  const long long* p = reinterpret_cast<const long long*>(pos);
  if (cache_dtype == AJQ_KV_F32)
    hipLaunchKernelGGL(rope_cache_kernel<float>, grid, dim3(256), 0, (hipStream_t)stream, qkv, cosine, sine, p, q_out,
                       reinterpret_cast<float*>(kcache), reinterpret_cast<float*>(vcache), B, H, Hkv, head_dim, max_len);
  else
    hipLaunchKernelGGL(rope_cache_kernel<uint16_t>, grid, dim3(256), 0, (hipStream_t)stream, qkv, cosine, sine, p, q_out,
                       reinterpret_cast<uint16_t*>(kcache), reinterpret_cast<uint16_t*>(vcache), B, H, Hkv, head_dim,
                       max_len);
  return check_launch("ajq_rope_cache");
}

int ajq_rope_prefill(const float* qkv, const float* cosine, const float* sine, float* q_out, void* kcache, void* vcache,
                     int cache_dtype, int B, int T, int H, int Hkv, int head_dim, int start, int max_len, void* stream) {
  if (!qkv || !cosine || !sine || !q_out || !kcache || !vcache)
    return fail(AJQ_ERR_NULL, "ajq_rope_prefill: null pointer argument");
  if (B < 1 || T < 1 || H < 1 || Hkv < 1 || H % Hkv != 0 || head_dim < 2 || head_dim % 2 != 0 || start < 0 ||
      (long long)start + T > max_len)
    return fail(AJQ_ERR_SHAPE, "ajq_rope_prefill: unsupported shape (B=%d T=%d H=%d Hkv=%d head_dim=%d start=%d max_len=%d)",
                B, T, H, Hkv, head_dim, start, max_len);
  if (cache_dtype != AJQ_KV_F32 && cache_dtype != AJQ_KV_BF16)
    return fail(AJQ_ERR_UNSUPPORTED, "ajq_rope_prefill: cache_dtype %d is neither AJQ_KV_F32 nor AJQ_KV_BF16", cache_dtype);
  const long long pairs = (long long)B * T * (H + 2 * Hkv) * (head_dim / 2);
  const long long blocks = (pairs + 255) / 256;
  if (blocks > 0x7FFFFFFFLL) return fail(AJQ_ERR_SHAPE, "ajq_rope_prefill: too many elements");
  const dim3 grid((unsigned)blocks);
  if (cache_dtype == AJQ_KV_F32)
    hipLaunchKernelGGL(rope_prefill_kernel<float>, grid, dim3(256), 0, (hipStream_t)stream, qkv, cosine, sine, q_out,
                       reinterpret_cast<float*>(kcache), reinterpret_cast<float*>(vcache), B, T, H, Hkv, head_dim, start,
                       max_len);
  else
    hipLaunchKernelGGL(rope_prefill_kernel<uint16_t>, grid, dim3(256), 0, (hipStream_t)stream, qkv, cosine, sine, q_out,
                       reinterpret_cast<uint16_t*>(kcache), reinterpret_cast<uint16_t*>(vcache), B, T, H, Hkv, head_dim,
                       start, max_len);
  return check_launch("ajq_rope_prefill");
}

size_t ajq_attn_decode_workspace_bytes(int B, int H) {
  if (B < 1 || H < 1) return 0;
  // sized for the largest split count: the number of cache heads is not known here
  return (size_t)B * H * kAttnMaxSplits * kAttnPartialStride * sizeof(float);
}

int ajq_attn_row_chunks(int B, int Hkv, int max_len) {
  if (B < 1 || Hkv < 1 || max_len < 1) return 0;
  return attn_splits(B, Hkv, max_len);
}

int ajq_attn_decode(const float* q, const void* kcache, const void* vcache, int cache_dtype, const int64_t* pos, int B,
                    int H, int Hkv, int head_dim, int max_len, uint16_t* out, void* workspace, size_t workspace_bytes,
                    void* stream) {
  if (!q || !kcache || !vcache || !pos || !out) return fail(AJQ_ERR_NULL, "ajq_attn_decode: null pointer argument");
  if (head_dim != 128 && head_dim != 64 && head_dim != 32)
    return fail(AJQ_ERR_UNSUPPORTED, "ajq_attn_decode: head_dim %d (128, 64 and 32 are built)", head_dim);
  if (B < 1 || H < 1 || Hkv < 1 || H % Hkv != 0 || max_len < 1)
    return fail(AJQ_ERR_SHAPE, "ajq_attn_decode: unsupported shape (B=%d H=%d Hkv=%d max_len=%d)", B, H, Hkv, max_len);
  const int R = H / Hkv;
  if (R != 1 && R != 2 && R != 4)
    return fail(AJQ_ERR_UNSUPPORTED, "ajq_attn_decode: %d query heads per cache head (1, 2 and 4 are built)", R);
  const int S = attn_splits(B, Hkv, max_len);
  if (S > 1 && (!workspace || workspace_bytes < ajq_attn_decode_workspace_bytes(B, H)))
    return fail(AJQ_ERR_WORKSPACE, "ajq_attn_decode: workspace of %zu bytes needed, %zu given",
                ajq_attn_decode_workspace_bytes(B, H), workspace_bytes);
  const float scale = 1.0f / sqrtf((float)head_dim);
  if (cache_dtype != AJQ_KV_F32 && cache_dtype != AJQ_KV_BF16)
    return fail(AJQ_ERR_UNSUPPORTED, "ajq_attn_decode: cache_dtype %d is neither AJQ_KV_F32 nor AJQ_KV_BF16", cache_dtype);
  if (!aligned16(kcache) || !aligned16(vcache) || !aligned16(q))
    return fail(AJQ_ERR_ALIGN, "ajq_attn_decode: q and the caches must be 16-byte aligned");
  pick_attn<false>(R, cache_dtype, head_dim)(q, const_cast<void*>(kcache), const_cast<void*>(vcache),
                                   reinterpret_cast<const long long*>(pos), B, H, Hkv, max_len, scale, S,
                                   reinterpret_cast<float*>(workspace), out, nullptr, nullptr, (hipStream_t)stream);
  return check_launch("ajq_attn_decode");
}

size_t ajq_attn_step_workspace_bytes(int B, int H) {
  if (B < 1 || H < 1) return 0;
  return ajq_attn_decode_workspace_bytes(B, H);
}

namespace {
// out != nullptr: bf16 attention output (merged by a second launch when there are several row
// chunks); out == nullptr: the chunks' partial results stay in the workspace, at most max_splits of them
int attn_step_impl(const char* name, const float* qkv, const float* cosine, const float* sine, const int64_t* pos,
                   void* kcache, void* vcache, int cache_dtype, int B, int H, int Hkv, int head_dim, int max_len,
                   uint16_t* out, int max_splits, int* splits, void* workspace, size_t workspace_bytes, void* stream) {
  if (!qkv || !cosine || !sine || !pos || !kcache || !vcache) return fail(AJQ_ERR_NULL, "%s: null pointer argument", name);
  if (head_dim != 128 && !((head_dim == 64 || head_dim == 32) && out))
    return fail(AJQ_ERR_UNSUPPORTED, "%s: head_dim %d (128 is built%s)", name, head_dim,
                out ? ", 64 and 32 too" : "; unmerged partial results are read by ajq_w*a16_gemv_merge, which assumes it");
  if (B < 1 || H < 1 || Hkv < 1 || H % Hkv != 0 || max_len < 1)
    return fail(AJQ_ERR_SHAPE, "%s: unsupported shape (B=%d H=%d Hkv=%d max_len=%d)", name, B, H, Hkv, max_len);
  const int R = H / Hkv;
  if (R != 1 && R != 2 && R != 4)
    return fail(AJQ_ERR_UNSUPPORTED, "%s: %d query heads per cache head (1, 2 and 4 are built)", name, R);
  if (cache_dtype != AJQ_KV_F32 && cache_dtype != AJQ_KV_BF16)
    return fail(AJQ_ERR_UNSUPPORTED, "%s: cache_dtype %d is neither AJQ_KV_F32 nor AJQ_KV_BF16", name, cache_dtype);
  if (!aligned16(qkv) || !aligned16(cosine) || !aligned16(sine) || !aligned16(kcache) || !aligned16(vcache))
    return fail(AJQ_ERR_ALIGN, "%s: qkv, the tables and the caches must be 16-byte aligned", name);
  int S = attn_splits(B, Hkv, max_len);
  if (S > max_splits) S = max_splits;
  if ((S > 1 || !out) && (!workspace || workspace_bytes < ajq_attn_step_workspace_bytes(B, H) || !aligned16(workspace)))
    return fail(AJQ_ERR_WORKSPACE, "%s: 16-byte aligned workspace of %zu bytes needed, %zu given", name,
                ajq_attn_step_workspace_bytes(B, H), workspace_bytes);
  if (splits) *splits = S;
  const float scale = 1.0f / sqrtf((float)head_dim);
  pick_attn<true>(R, cache_dtype, head_dim)(qkv, kcache, vcache, reinterpret_cast<const long long*>(pos), B, H, Hkv, max_len,
                                  scale, S, reinterpret_cast<float*>(workspace), out, cosine, sine,
                                  (hipStream_t)stream);
  return check_launch(name);
}
}  // namespace

int ajq_attn_step(const float* qkv, const float* cosine, const float* sine, const int64_t* pos, void* kcache,
                  void* vcache, int cache_dtype, int B, int H, int Hkv, int head_dim, int max_len, uint16_t* out,
                  void* workspace, size_t workspace_bytes, void* stream) {
  if (!out) return fail(AJQ_ERR_NULL, "ajq_attn_step: null pointer argument");
  return attn_step_impl("ajq_attn_step", qkv, cosine, sine, pos, kcache, vcache, cache_dtype, B, H, Hkv, head_dim,
                        max_len, out, kAttnMaxSplits, nullptr, workspace, workspace_bytes, stream);
}

int ajq_attn_step_partial(const float* qkv, const float* cosine, const float* sine, const int64_t* pos, void* kcache,
                          void* vcache, int cache_dtype, int B, int H, int Hkv, int head_dim, int max_len,
                          int max_splits, int* splits, void* workspace, size_t workspace_bytes, void* stream) {
  if (!splits) return fail(AJQ_ERR_NULL, "ajq_attn_step_partial: splits must point to an int");
  if (max_splits < 1) return fail(AJQ_ERR_SHAPE, "ajq_attn_step_partial: max_splits must be at least 1");
  return attn_step_impl("ajq_attn_step_partial", qkv, cosine, sine, pos, kcache, vcache, cache_dtype, B, H, Hkv,
                        head_dim, max_len, nullptr, max_splits, splits, workspace, workspace_bytes, stream);
}

int ajq_greedy_pick(const float* logits, int B, int V, int ld, const float* embedding, int D, float* hidden,
                    int64_t* token, int64_t* out, int out_ld, const int64_t* step, int64_t* advance, uint32_t* ticket,
                    void* stream) {
  if (!logits || !embedding || !hidden || !token || !out || !step)
    return fail(AJQ_ERR_NULL, "ajq_greedy_pick: null pointer argument");
  if ((advance != nullptr) != (ticket != nullptr))
    return fail(AJQ_ERR_NULL, "ajq_greedy_pick: advance and ticket go together (both or neither)");
  if (B < 1 || V < 1 || ld < V || ld % 4 != 0 || D < 4 || D % 4 != 0 || out_ld < 1)
    return fail(AJQ_ERR_SHAPE, "ajq_greedy_pick: unsupported shape (B=%d V=%d ld=%d D=%d out_ld=%d)", B, V, ld, D, out_ld);
  if (!aligned16(logits) || !aligned16(embedding) || !aligned16(hidden))
    return fail(AJQ_ERR_ALIGN, "ajq_greedy_pick: logits, embedding and hidden must be 16-byte aligned");
  hipLaunchKernelGGL(greedy_pick_kernel, dim3(B), dim3(1024), 0, (hipStream_t)stream, logits, V, ld, embedding, D, hidden,
                     reinterpret_cast<long long*>(token), reinterpret_cast<long long*>(out), out_ld,
                     reinterpret_cast<const long long*>(step), reinterpret_cast<long long*>(advance), ticket);
  return check_launch("ajq_greedy_pick");
}

int ajq_sample_pick(const float* logits, int B, int V, int ld, float temperature, float top_p, const float* uniforms,
                    int uniform_rows, const float* embedding, int D, float* hidden, int64_t* token, int64_t* out,
                    int out_ld, const int64_t* step, int64_t* advance, uint32_t* ticket, int32_t* kept, void* stream) {
  if (!logits || !token || !out || !step) return fail(AJQ_ERR_NULL, "ajq_sample_pick: null pointer argument");
  if ((embedding != nullptr) != (hidden != nullptr))
    return fail(AJQ_ERR_NULL, "ajq_sample_pick: embedding and hidden go together (both or neither)");
  if ((advance != nullptr) != (ticket != nullptr))
    return fail(AJQ_ERR_NULL, "ajq_sample_pick: advance and ticket go together (both or neither)");
  if (B < 1 || V < 1 || ld < V || ld % 4 != 0 || out_ld < 1 || (embedding && (D < 4 || D % 4 != 0)))
    return fail(AJQ_ERR_SHAPE, "ajq_sample_pick: unsupported shape (B=%d V=%d ld=%d D=%d out_ld=%d)", B, V, ld, D, out_ld);
  if (!aligned16(logits)) return fail(AJQ_ERR_ALIGN, "ajq_sample_pick: logits must be 16-byte aligned");
  if (V > kSampleMaxBlocks * 1024)
    return fail(AJQ_ERR_UNSUPPORTED, "ajq_sample_pick: V=%d exceeds %d", V, kSampleMaxBlocks * 1024);
  if (!(temperature > 0.f) || !std::isfinite(temperature))
    return fail(AJQ_ERR_SHAPE, "ajq_sample_pick: temperature must be positive and finite (use ajq_greedy_pick for argmax)");
  if (!(top_p > 0.f)) return fail(AJQ_ERR_SHAPE, "ajq_sample_pick: top_p must be in (0, 1] (1: no filter)");
  if (!uniforms || uniform_rows < 1) return fail(AJQ_ERR_NULL, "ajq_sample_pick: uniforms [uniform_rows, B] are needed");
  if (embedding && (!aligned16(embedding) || !aligned16(hidden)))
    return fail(AJQ_ERR_ALIGN, "ajq_sample_pick: embedding and hidden must be 16-byte aligned");
  hipLaunchKernelGGL(sample_pick_kernel, dim3(B), dim3(1024), 0, (hipStream_t)stream, logits, V, ld, 1.0f / temperature,
                     top_p, uniforms, uniform_rows, embedding, D, hidden, reinterpret_cast<long long*>(token),
                     reinterpret_cast<long long*>(out), out_ld, reinterpret_cast<const long long*>(step),
                     reinterpret_cast<long long*>(advance), ticket, kept);
  return check_launch("ajq_sample_pick");
}

int ajq_attn_prefill(const float* q, const void* kcache, const void* vcache, int cache_dtype, int B, int H, int Hkv,
                     int T, int start, int max_len, int head_dim, void* out, int out_dtype, void* stream) {
  if (!q || !kcache || !vcache || !out) return fail(AJQ_ERR_NULL, "ajq_attn_prefill: null pointer argument");
  if (head_dim != 128 && head_dim != 64 && head_dim != 32)
    return fail(AJQ_ERR_UNSUPPORTED, "ajq_attn_prefill: head_dim %d (128, 64 and 32 are built)", head_dim);
  if (B < 1 || H < 1 || Hkv < 1 || H % Hkv != 0 || T < 1 || start < 0 || (long long)start + T > max_len ||
      (long long)B * H > 65535)
    return fail(AJQ_ERR_SHAPE, "ajq_attn_prefill: unsupported shape (B=%d H=%d Hkv=%d T=%d start=%d max_len=%d)", B, H,
                Hkv, T, start, max_len);
  if (cache_dtype != AJQ_KV_F32 && cache_dtype != AJQ_KV_BF16)
    return fail(AJQ_ERR_UNSUPPORTED, "ajq_attn_prefill: cache_dtype %d is neither AJQ_KV_F32 nor AJQ_KV_BF16", cache_dtype);
  if (out_dtype != AJQ_OUT_BF16 && out_dtype != AJQ_OUT_F32)
    return fail(AJQ_ERR_UNSUPPORTED, "ajq_attn_prefill: out_dtype %d is neither AJQ_OUT_BF16 nor AJQ_OUT_F32", out_dtype);
  const int out_bf16 = out_dtype == AJQ_OUT_BF16;
  if (!aligned16(q) || !aligned16(kcache) || !aligned16(vcache) || !aligned16(out))
    return fail(AJQ_ERR_ALIGN, "ajq_attn_prefill: q, the caches and out must be 16-byte aligned");
  const dim3 grid((unsigned)(((T + kPfBQ - 1) / kPfBQ) * B * H));  // (the kernel orders the work by cost)
  const bool f32 = cache_dtype == AJQ_KV_F32;
  auto launch = [&](auto kernel, auto* cache_element) {
    using CacheT = std::remove_pointer_t<decltype(cache_element)>;
    hipLaunchKernelGGL(kernel, grid, dim3(256), 0, (hipStream_t)stream, q, reinterpret_cast<const CacheT*>(kcache),
                       reinterpret_cast<const CacheT*>(vcache), H, Hkv, T, start, max_len, out, out_bf16);
  };
  if (head_dim == 128) {
    if (f32) launch(attn_prefill_kernel<float, 128>, (float*)nullptr);
    else launch(attn_prefill_kernel<uint16_t, 128>, (uint16_t*)nullptr);
  } else if (head_dim == 64) {
    if (f32) launch(attn_prefill_kernel<float, 64>, (float*)nullptr);
    else launch(attn_prefill_kernel<uint16_t, 64>, (uint16_t*)nullptr);
  } else {
    if (f32) launch(attn_prefill_kernel<float, 32>, (float*)nullptr);
    else launch(attn_prefill_kernel<uint16_t, 32>, (uint16_t*)nullptr);
  }
  return check_launch("ajq_attn_prefill");
}

int ajq_swiglu(const float* ab, uint16_t* out, int B, int F, void* stream) {
  if (!ab || !out) return fail(AJQ_ERR_NULL, "ajq_swiglu: null pointer argument");
  if (B < 1 || F < 2 || F % 2 != 0) return fail(AJQ_ERR_SHAPE, "ajq_swiglu: need B >= 1 and even F (got %d, %d)", B, F);
  const long long pairs = (long long)B * (F / 2);
  hipLaunchKernelGGL(swiglu_kernel, dim3((unsigned)((pairs + 255) / 256)), dim3(256), 0, (hipStream_t)stream, ab, out, B,
                     F);
  return check_launch("ajq_swiglu");
}

}  // extern "C"
