/*
 * The reference's host-staged reducing collectives as a timed baseline: what
 * FLAGCX_USE_HOST_COMM=1 does for every rank (hostRunnerAllReduce,
 * hostRunnerReduce, hostRunnerReduceScatter, flagcx/runner/host_runner.cc:236-289,
 * 12-67, 291-346) -- staged host buffers, a synchronous
 * device-to-host copy, the bootstrap ring all-reduce on the host
 * (flagcx/service/bootstrap.cc:787-942: ceil(size/n) chunks, n-1 reduce steps
 * res = local (op) received with the loops of
 * flagcx/service/include/utils.h:697-725, then a ring all-gather; a reduce
 * gathers the chunks on the root instead, :944-996; a reduce-scatter's chunk i is
 * rank i's recvcount elements and stays on rank i, :1039-1066), a
 * host-to-device copy -- with that code's own per-phase timers.  The ranks are
 * simulated ranks of this process, one host thread each; where the reference
 * sends a chunk through a socket, the receiving rank's thread copies it from
 * the sender's buffer (that copy is what the `comm` timer holds here).
 *
 * It exists to be measured beside the device path and to be compared with it:
 * for the types and ops the reference's host loops carry (int8, uint8, int32,
 * uint32, int64, uint64, fp32, fp64; sum, max, min) the result is bit-identical
 * to flagcxAllReduce / flagcxReduce / flagcxReduceScatter with FX_ORDER_HOST.  Other types and ops return
 * flagcxInvalidArgument, as the reference does (utils.h:690-694,
 * bootstrap.cc:872-874).
 */
#ifndef FLAGCX_AMD_FX_HOST_STAGED_H_
#define FLAGCX_AMD_FX_HOST_STAGED_H_

#include "flagcx_amd/fx_types.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Timer slots, in nanoseconds: names and numbers of TIMER_COLL_*
 * (flagcx/service/include/debug.h:87-95).  TOTAL, ALLOC, MEM_D2H, COMM, MEM_H2D,
 * FREE are the host runner's phases (COMM is the whole host collective); CALC
 * and MEM are the ring's own reduce loops and copies into its send buffer,
 * both inside COMM. */
enum {
  FX_TIMER_COLL_TOTAL = 0,
  FX_TIMER_COLL_CALC = 1,
  FX_TIMER_COLL_COMM = 2,
  FX_TIMER_COLL_MEM = 3,
  FX_TIMER_COLL_MEM_D2H = 4,
  FX_TIMER_COLL_MEM_H2D = 5,
  FX_TIMER_COLL_ALLOC = 6,
  FX_TIMER_COLL_FREE = 7,
  FX_TIMERS_COLL_COUNT = 8
};

/* deviceMemcpy of the device-adaptor plugin
 * (flagcx/adaptor/include/flagcx_device_adaptor.h:33-35); NULL = hipMemcpy */
typedef flagcxResult_t (*fxDeviceMemcpyFn)(void *dst, void *src, size_t size,
                                           flagcxMemcpyType_t type,
                                           flagcxStream_t stream, void *args);

typedef struct fxHostStaged *fxHostStaged_t;

/* nranks simulated ranks; the staged buffers are kept between calls and grow
 * on demand, as the reference's are. */
int fxHostStagedCreate(fxHostStaged_t *h, int nranks, fxDeviceMemcpyFn memcpyFn);
/*
 * sendbuffs / recvbuffs: host arrays of nranks DEVICE pointers (recvbuffs[r]
 * may equal sendbuffs[r]).  Blocks until every rank's result is in its
 * recvbuff.  timers: NULL, or nranks * FX_TIMERS_COLL_COUNT slots, rank-major.
 */
int fxHostStagedAllReduce(fxHostStaged_t h, const void *const *sendbuffs,
                          void *const *recvbuffs, size_t count, int dtype,
                          int op, uint64_t *timers);
/* The same for a reduce (recvbuffs[r] is used for r == root only and may be
 * NULL elsewhere) and a reduce-scatter (sendbuffs[r] holds nranks * recvcount
 * elements, recvbuffs[r] receives chunk r). */
int fxHostStagedReduce(fxHostStaged_t h, const void *const *sendbuffs,
                       void *const *recvbuffs, size_t count, int dtype, int op,
                       int root, uint64_t *timers);
int fxHostStagedReduceScatter(fxHostStaged_t h, const void *const *sendbuffs,
                              void *const *recvbuffs, size_t recvcount,
                              int dtype, int op, uint64_t *timers);
int fxHostStagedDestroy(fxHostStaged_t h);

#ifdef __cplusplus
}
#endif
#endif
