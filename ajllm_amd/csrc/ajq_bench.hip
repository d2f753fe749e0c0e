// libajq_bench.so: the device yardstick bench.py quotes beside the tile GEMMs.  Nothing here is an
// operator; the operator library (libajq.so) does not contain or need any of it.
#include <stdarg.h>
#include <stdio.h>

#include "../../include/ajq_bench.h"
#include "ajq_common.h"
#include "probe_kernels.h"

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

}  // extern "C"
