/*
 * ajq_bench -- measurement probes of libajq_bench.so, used by bench.py only.
 *
 * None of these is an operator and none has a counterpart in the reference project; the operator
 * library (libajq.so, include/ajq.h) neither contains nor needs them.  They allocate their own
 * device memory and synchronise the device.  Return value: 0 on success, negative otherwise
 * (ajqb_last_error() gives the thread-local message).
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

/* One measured way of running a chain of `stages` W4A16 GEMVs (K = N = 4096, M = 1, a distinct
 * matrix per stage): microseconds per stage, the fraction of the 8 TB/s HBM peak that is (0 for rows
 * that move no matrix), whether the last stage's output equals the reference chain's bit for bit
 * (1 / 0; -1 where the row has no output to compare) and the kernels' error word (bit 0: a bounded
 * wait ran into its spin limit). */
typedef struct ajqb_result {
  char name[112];
  double us_per_stage;
  double frac_hbm_peak;
  int matches_reference;
  int error_word;
} ajqb_result;

/* The alternatives to "one launch per matrix" for such a chain, each timed over `reps` passes:
 * launches in a HIP graph (the product path, a read-only kernel, a GEMV that also issues the next
 * matrix's loads, a prefetch kernel on a second graph branch) and ONE launch for all stages with
 * the activations exchanged between workgroups through device memory (flag per producer or stamped
 * records, one copy or one per XCD), plus the one-way latency of that exchange.  Needs a GPU with
 * at least 256 compute units.  results: host array of max_results entries; *n_results = entries written. */
int ajqb_launch_alternatives(int stages, int reps, ajqb_result* results, int max_results, int* n_results);

#ifdef __cplusplus
}
#endif
#endif /* AJQ_BENCH_H */
