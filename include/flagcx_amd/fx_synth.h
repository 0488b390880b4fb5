/*
 * Reproducible synthetic host data for benchmarks and parity runs.  No
 * counterpart in the reference, whose harness fills buffers with closed-form
 * patterns (test/perf/host_api/test_allreduce.cpp:20-32).
 */
#ifndef FLAGCX_AMD_FX_SYNTH_H_
#define FLAGCX_AMD_FX_SYNTH_H_

#include "flagcx_amd/fx_types.h"

#ifdef __cplusplus
extern "C" {
#endif

enum {
  FX_SYNTH_UNIFORM = 0,     /* real uniform in [a, b)        */
  FX_SYNTH_NORMAL = 1,      /* normal, mean a, std-dev b     */
  FX_SYNTH_UNIFORM_INT = 2  /* integer uniform in [a, b]     */
};

/*
 * Fill a HOST buffer of n elements of `dtype` (fp32, fp64, fp16, bf16, int32).
 * Element i depends only on (seed, stream, i): the same call on any machine,
 * with any thread count, yields the same bytes.
 */
int fx_synth_fill(void *dst, size_t n, int dtype, int dist, double a, double b,
                  uint64_t seed, uint64_t stream, int nthreads);

#ifdef __cplusplus
}
#endif
#endif
