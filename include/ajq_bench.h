/*
 * ajq_bench -- the device yardstick of libajq_bench.so, used by bench.py only.
 *
 * Not an operator and without a counterpart in the reference project; the operator library
 * (libajq.so, include/ajq.h) neither contains nor needs it.  Return value: 0 on success, negative
 * otherwise (ajqb_last_error() gives the thread-local message).
 */
#ifndef AJQ_BENCH_H
#define AJQ_BENCH_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

const char* ajqb_last_error(void);

/* Device yardstick: every wave issues bf16 MFMAs back to back from registers (no memory
 * traffic), so launches timed by the caller give the MFMA rate the GPU sustains -- with constant
 * operands (random_operands = 0: nominal clock) or with random mantissas (1: the power-limited
 * rate real data can approach).  sink: device float[workgroups * 512]; clocks: device int64[2],
 * receives shader cycles and 100 MHz ticks over the loop; *flops_per_launch (host, may be NULL) =
 * flops one launch does.  Asynchronous on `stream`. */
int ajqb_mfma_rate(int random_operands, int iters, int workgroups, float* sink, long long* clocks,
                   double* flops_per_launch, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* AJQ_BENCH_H */
