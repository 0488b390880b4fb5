/*
 * FlagCX collective entry points over SIMULATED ranks on one GPU.
 *
 * The five collectives keep the exact C signatures of flagcx/include/flagcx.h
 * (flagcxReduce :371-373, flagcxAllReduce :425-428, flagcxReduceScatter
 * :441-444, flagcxAllGather :456-458, flagcxAlltoAllv :480-484) and the
 * custom-op hook flagcxCustomAllReduceImpl that of
 * flagcx/adaptor/kernel/nvidia/custom_allreduce.cu:604-607 (typedef
 * flagcx/core/include/dev_comm_state.h:20-23).  What differs is the
 * communicator: a group of n `flagcxComm_t` living in one process, whose
 * "peer IPC buffers" are ordinary allocations in the same GPU's HBM.  No
 * inter-GPU transport exists here.
 *
 * Calling convention (single-process multi-rank): every rank of the group
 * calls the same collective once; the work is launched when the last rank has
 * posted, on that caller's stream, after waiting for what the other ranks'
 * streams held at that moment; those streams in turn wait for the result.
 * In-place rules are FlagCX's (flagcx.h:369,423,439,454).
 *
 * Two synchronisation modes (FX_SIM_SYNC):
 *   FX_SYNC_GROUP (default)  every call returns at once (flagcx.h:345-346).
 *     Like the calls of one ncclGroupStart/End bracket, a collective is ordered
 *     after work a rank enqueued BEFORE the last rank posted and before work
 *     enqueued AFTER it: a single host thread that loops over the ranks, on one
 *     stream or several, needs nothing else.  flagcxSend / flagcxRecv pairs that
 *     meet inside a flagcxGroupStart / flagcxGroupEnd bracket of that thread,
 *     both halves on one stream, are enqueued together -- one copy launch per
 *     stream -- when the thread's outermost bracket closes, and that
 *     flagcxGroupEnd returns their result.
 *   FX_SYNC_RENDEZVOUS       for one host thread per rank, each on its own
 *     stream, the way separate FlagCX processes behave: a call blocks its host
 *     thread until every rank has posted and the work is enqueued, so whatever
 *     the rank enqueues after the call returns is ordered after the collective.
 *     Handing n threads through the group's lock and ordering n streams
 *     around one launch costs tens of microseconds for eight ranks; the
 *     default mode on one stream needs neither.
 *     A rank that never arrives makes the others return flagcxInternalError
 *     after FX_SIM_RENDEZVOUS_TIMEOUT_MS (environment, default 30000).
 *     flagcxSend / flagcxRecv made between flagcxGroupStart and
 *     flagcxGroupEnd on a host thread do not block: the outermost
 *     flagcxGroupEnd of that thread posts them and waits for their partners,
 *     so every rank's thread can run GroupStart, Send(next), Recv(prev),
 *     GroupEnd; argument errors of such calls are reported at once, everything
 *     else by that flagcxGroupEnd.
 *
 * Scratch (partials of the tree reduce and of the ring reduce-scatter, the
 * host order's floating max / min, staging of in-place all-to-all(v)) is grown
 * by allocating a larger block and keeping the old ones until the group is
 * destroyed: no call waits for the device.  A captured stream cannot
 * allocate: reserve beforehand with fxSimCommConfig(comm, FX_SIM_SCRATCH_BYTES,
 * n) or the environment variable of the same name, else such a call returns
 * flagcxInvalidUsage while the stream is capturing.
 */
#ifndef FLAGCX_AMD_FX_SIM_H_
#define FLAGCX_AMD_FX_SIM_H_

#include "flagcx_amd/fx_types.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Create / destroy a group of nranks communicators on the current device
 * (stand-in for flagcxCommInitRank, flagcx/flagcx.cc:1943-2358, whose
 * bootstrap is multi-process). */
flagcxResult_t fxSimCommInitAll(flagcxComm_t *comms, int nranks);
flagcxResult_t fxSimCommDestroyAll(flagcxComm_t *comms, int nranks);

/* The same group built rank by rank, the way flagcxCommInitRank
 * (flagcx/include/flagcx.h:296-297) is called: every rank passes the same id
 * bytes; the group is complete when nranks ranks have joined.  Each
 * communicator is released with fxSimCommDestroy; the last one frees the group. */
flagcxResult_t fxSimCommInitRank(flagcxComm_t *comm, int nranks, const void *id,
                                 size_t idBytes, int rank);
flagcxResult_t fxSimCommDestroy(flagcxComm_t comm);
flagcxResult_t fxSimCommDevice(const flagcxComm_t comm, int *device);

/*
 * The communicator life cycle under its reference names and signatures
 * (flagcx/include/flagcx.h:282-321,358), so that a harness written against
 * libflagcx -- e.g. the ctypes table of plugin/interservice/flagcx_wrapper.py:
 * 244-330 -- binds to this library unchanged for the calls of this path.
 * flagcxGetUniqueId fills the 256 bytes with a value unique in the process;
 * flagcxCommInitRank joins the in-process group carrying that id (no
 * bootstrap network: all ranks of a group live in one process on one GPU);
 * flagcxCommDestroy releases one rank.  flagcxGetVersion reports
 * FX_SIM_VERSION.  flagcxGetErrorString names the code (the reference returns
 * "Not implemented." for every code, flagcx.cc:1586-1589).  flagcxBarrier makes
 * every rank's stream wait for all the others'.
 */
#define FX_SIM_VERSION 100
flagcxResult_t flagcxGetVersion(int *version);
flagcxResult_t flagcxGetUniqueId(flagcxUniqueId_t uniqueId);
flagcxResult_t flagcxCommInitRank(flagcxComm_t *comm, int nranks,
                                  flagcxUniqueId_t commId, int rank);
flagcxResult_t flagcxCommDestroy(flagcxComm_t comm);
const char *flagcxGetErrorString(flagcxResult_t result);
flagcxResult_t flagcxBarrier(flagcxComm_t comm, flagcxStream_t stream);

/* Configuration keys (defaults come from the same environment variables the
 * reference reads, flagcx/runner/uni_runner_impl.cc:21-26, uni_runner.cc:10-12). */
enum {
  FX_SIM_ALGO = 0,         /* FX_ALGO_*                                   */
  FX_SIM_ORDER = 1,        /* FX_ORDER_*                                  */
  FX_SIM_NSLICES = 2,      /* FLAGCX_UNIRUNNER_NSLICES (default 1)        */
  FX_SIM_NREDSLICES = 3,   /* FLAGCX_UNIRUNNER_NREDSLICES (0 = automatic) */
  FX_SIM_REDSLICESIZE = 4, /* FLAGCX_UNIRUNNER_REDSLICESIZE (65536 elems) */
  FX_SIM_SYNC = 5,         /* FX_SYNC_*; environment FX_SIM_SYNC=group|rendezvous */
  FX_SIM_SCRATCH_BYTES = 6, /* reserve at least this much scratch now           */
  FX_SIM_ARITH = 7         /* FX_ARITH_*; environment FX_SIM_ARITH=element      */
};
/* How fp16 / bf16 sums, maxima and minima are folded by flagcxAllReduce, flagcxReduce, flagcxReduceScatter (direct
 * algorithm, rank order) and flagcxCustomAllReduceImpl. */
enum {
  FX_ARITH_DEFAULT = 0, /* widen to fp32, accumulate, round once; max / min keep
                           the earlier operand on ties and NaN (std::max / min) */
  FX_ARITH_ELEMENT = 1  /* in the element type, as the reference's device kernel
                           does (custom_allreduce.cu:326-361): rounded after every
                           addition, a > b ? a : b (FX_OP_ELEMENT_FOLD of
                           fx_kernels.h)                                        */
};
enum {
  FX_SYNC_GROUP = 0,
  FX_SYNC_RENDEZVOUS = 1
};
enum {
  FX_ALGO_DIRECT = 0, /* one k-way reduce per slice, then all-gather copies */
  FX_ALGO_RING = 1    /* n-1 two-input ring steps, then n-1 copy steps      */
};
enum {
  FX_ORDER_RANK = 0, /* rank 0,1,..,n-1: the custom allreduce's peer loop    */
  FX_ORDER_RING = 1, /* the rotated order a ring yields for each chunk       */
  FX_ORDER_TREE = 2, /* flagcxReduce only: the binomial tree of
                        initUniRunnerStateTreeRed (uni_runner_impl.cc:1266-1557),
                        ceil(log2 n) rounds of two-input reduces               */
  FX_ORDER_HOST = 3  /* what the reference's host path computes
                        (FLAGCX_USE_HOST_COMM=1, flagcx/service/bootstrap.cc:787-942,
                        1039-1066): chunks of ceil(size/n) bytes rounded up to an
                        element, chunk c folded along the ring c+1, c+2, .., c
                        as local (op) received.  AllReduce, Reduce and
                        ReduceScatter; bit-identical to that path for every type
                        it carries, +-0 ties and NaN operands of max / min
                        included (floating max / min run as the ring's n-1
                        two-input steps for that; everything else as one k-way
                        launch per collective)                                 */
};
flagcxResult_t fxSimCommConfig(flagcxComm_t comm, int key, long long value);

/* Where a rank stands (no counterpart in the reference, whose ranks are
 * processes and whose collectives launch in the caller's own call): `joined` =
 * the number of collectives the group had launched when this rank's latest
 * collective call was accepted, `launched` = that number now.  The rank's
 * latest collective has been enqueued, on its stream, once launched > joined;
 * a caller with work to enqueue behind it (copies out of a staging buffer)
 * asks here whether it may. */
flagcxResult_t fxSimCommProgress(flagcxComm_t comm, uint64_t *joined,
                                 uint64_t *launched);

flagcxResult_t flagcxCommCount(const flagcxComm_t comm, int *count);
flagcxResult_t flagcxCommUserRank(const flagcxComm_t comm, int *rank);

flagcxResult_t flagcxReduce(const void *sendbuff, void *recvbuff, size_t count,
                            flagcxDataType_t datatype, flagcxRedOp_t op,
                            int root, flagcxComm_t comm, flagcxStream_t stream);
flagcxResult_t flagcxAllReduce(const void *sendbuff, void *recvbuff,
                               size_t count, flagcxDataType_t datatype,
                               flagcxRedOp_t op, flagcxComm_t comm,
                               flagcxStream_t stream);
flagcxResult_t flagcxReduceScatter(const void *sendbuff, void *recvbuff,
                                   size_t recvcount, flagcxDataType_t datatype,
                                   flagcxRedOp_t op, flagcxComm_t comm,
                                   flagcxStream_t stream);
flagcxResult_t flagcxAllGather(const void *sendbuff, void *recvbuff,
                               size_t sendcount, flagcxDataType_t datatype,
                               flagcxComm_t comm, flagcxStream_t stream);
flagcxResult_t flagcxAlltoAllv(const void *sendbuff, size_t *sendcounts,
                               size_t *sdispls, void *recvbuff,
                               size_t *recvcounts, size_t *rdispls,
                               flagcxDataType_t datatype, flagcxComm_t comm,
                               flagcxStream_t stream);

/* Byte-moving collectives and point-to-point calls, signatures of
 * flagcx.h:385-415,468-470,498-516,653-662.  On one GPU they are batched
 * copies; send/recv pairs are matched as they arrive. */
flagcxResult_t flagcxGather(const void *sendbuff, void *recvbuff, size_t count,
                            flagcxDataType_t datatype, int root,
                            flagcxComm_t comm, flagcxStream_t stream);
flagcxResult_t flagcxScatter(const void *sendbuff, void *recvbuff, size_t count,
                             flagcxDataType_t datatype, int root,
                             flagcxComm_t comm, flagcxStream_t stream);
flagcxResult_t flagcxBroadcast(const void *sendbuff, void *recvbuff,
                               size_t count, flagcxDataType_t datatype,
                               int root, flagcxComm_t comm,
                               flagcxStream_t stream);
flagcxResult_t flagcxAlltoAll(const void *sendbuff, void *recvbuff,
                              size_t count, flagcxDataType_t datatype,
                              flagcxComm_t comm, flagcxStream_t stream);
flagcxResult_t flagcxSend(const void *sendbuff, size_t count,
                          flagcxDataType_t datatype, int peer,
                          flagcxComm_t comm, flagcxStream_t stream);
flagcxResult_t flagcxRecv(void *recvbuff, size_t count,
                          flagcxDataType_t datatype, int peer,
                          flagcxComm_t comm, flagcxStream_t stream);
flagcxResult_t flagcxGroupStart(flagcxComm_t comm);
flagcxResult_t flagcxGroupEnd(flagcxComm_t comm);

/*
 * Custom allreduce hook: this rank's result = k-way reduce over all ranks'
 * registered send windows, in rank order, written to recvbuff.  sendbuff is
 * first staged into this rank's window unless it already is the window.
 * Returns flagcxNotSupported (caller falls through, flagcx.cc:2673-2680) for
 * avg, when no window is registered or when the message exceeds it.  Unlike the reference it accepts
 * every op on every type, odd counts and unaligned recvbuff.
 */
flagcxResult_t flagcxCustomAllReduceImpl(const void *sendbuff, void *recvbuff,
                                         size_t count,
                                         flagcxDataType_t datatype,
                                         flagcxRedOp_t op, flagcxComm_t comm,
                                         flagcxStream_t stream);
/* Register the per-rank staged send windows (the reference's IPC-mapped
 * sendStagedBuff, flagcx.cc:1617-1779; default size 8 MiB, :1606).  `windows`
 * has nranks device pointers of `bytes` each; NULL unregisters. */
flagcxResult_t fxSimRegisterWindows(flagcxComm_t comm, void *const *windows,
                                    size_t bytes);

/* Partition nodes of the reference's DAG builders, for inspection and tests. */
typedef struct fxRedNode {
  int32_t step, rank;
  int32_t in1_buf, in2_buf, out_buf; /* 0 sendbuff, 1 recvbuff, 2 scratch */
  int32_t slice;
  uint64_t in1_off, in2_off, out_off, count; /* elements */
} fxRedNode;
/* initUniRunnerStateSlicedAR (uni_runner_impl.cc:661-1007), reduce nodes only */
size_t fx_part_ring_ar(size_t count, int nranks, int rank, size_t nslices,
                       size_t nred, fxRedNode *nodes);
/* initUniRunnerStateRingRS (uni_runner_impl.cc:1009-1264) */
size_t fx_part_ring_rs(size_t recvcount, int nranks, int rank, size_t nslices,
                       size_t nred, fxRedNode *nodes);
/* initUniRunnerStateLocRed (uni_runner_impl.cc:82-157) */
size_t fx_part_locred(size_t count, int nranks, int rank, size_t nslices,
                      fxRedNode *nodes);

#ifdef __cplusplus
}
#endif
#endif
