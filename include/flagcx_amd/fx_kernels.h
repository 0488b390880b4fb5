/*
 * C ABI of the MI355X (gfx950) reduce / slice / pack kernel layer.
 *
 * Plain pointers and sizes only.  Every function returns a flagcxResult_t
 * value (0 = flagcxSuccess, 1 = device error, 4 = invalid argument,
 * 9 = not supported -- callers fall through on 9 exactly as FlagCX does,
 * flagcx/flagcx.cc:2673-2680).  `stream` is a raw hipStream_t (NULL = the
 * default stream); all launches are enqueue-only.  dtype / op are FlagCX enum
 * values (flagcx/include/flagcx.h:36-66): int8 = 0, uint8 = 1, int32 = 2,
 * uint32 = 3, int64 = 4, uint64 = 5, fp16 = 6, fp32 = 7, fp64 = 8, bf16 = 9;
 * sum = 0, prod = 1, max = 2, min = 3, avg = 4.  All ten types and five ops
 * are carried.  Integer sum / prod wrap modulo 2^width, as the host loops of
 * flagcx/service/include/utils.h:664-725 do.  avg is the sum divided once by
 * the number of inputs (IEEE division before the final rounding; C division of
 * the wrapped sum for integers): FlagCX only forwards avg to vendor libraries
 * (flagcx/adaptor/ccl/rccl_adaptor.cc:124,200), so this definition is this
 * library's own.
 */
#ifndef FLAGCX_AMD_FX_KERNELS_H_
#define FLAGCX_AMD_FX_KERNELS_H_

#include "flagcx_amd/fx_types.h"

#ifdef __cplusplus
extern "C" {
#endif

#define FX_MAX_INPUTS 64      /* k accepted by fx_reduce_copy            */
#define FX_MAX_SLICE_INPUTS 8 /* k accepted by the slice descriptors     */

/*
 * Added to a reduction op (flagcxSum | FX_OP_ELEMENT_FOLD, also flagcxMax,
 * flagcxMin) for flagcxFloat16 / flagcxBfloat16: fold in the element type
 * itself, as the reference's device kernel does (reduceOp on half /
 * nv_bfloat16, flagcx/adaptor/kernel/nvidia/custom_allreduce.cu:326-361).  A
 * sum is then rounded to 16 bits after every addition instead of once at the
 * end, and max / min are a > b ? a : b / a < b ? a : b with a the accumulator:
 * on a tie (+0 and -0) or an unordered pair (NaN) the LATER operand is handed
 * on.  Any other type or op with the flag is flagcxNotSupported, as in that
 * kernel's dispatch (:498-518); for fp32 / fp64 sums the default arithmetic is
 * that kernel's already.  Accepted wherever a dtype / op pair is, except in
 * reduce triggers, whose op field has four bits.
 */
#define FX_OP_ELEMENT_FOLD 0x100

/*
 * k-way element-wise reduce-copy over peer buffers:
 *   out[i] = in[first][i] (op) in[(first+1)%k][i] (op) ... left to right.
 * Replaces lsa_reduce + flagcxLsaAllReduceKernel
 * (flagcx/adaptor/kernel/nvidia/custom_allreduce.cu:337-394) including the
 * tail the reference drops (:383-384) and unaligned buffers it rejects
 * (:633-635).  bf16/fp16 sum/prod accumulate in fp32 and round once.
 * `in` is a host array of k device pointers; out may equal any in[p]
 * (in-place), partial overlap is undefined.  Pointers must be aligned to the
 * element size.  first = 0 is the reference order;
 * another value gives the rotated order a ring produces for that chunk.
 */
int fx_reduce_copy(void *out, const void *const *in, int k, size_t count,
                   int dtype, int op, int first, void *stream);

/*
 * Two-input slice reduce out = in1 (op) in2, for every dtype / op.  Replaces
 * the device function flagcxReduceKernel
 * (flagcx/adaptor/kernel/nvidia/flagcx_reduce_kernel_device.cu:75-86), which
 * is fp32-sum only.  out may alias in1 (ring: output == input1).
 */
int fx_reduce2(void *out, const void *in1, const void *in2, size_t count,
               int dtype, int op, void *stream);

/*
 * The reference's 32-byte slice descriptor, bit for bit
 * (flagcx/include/flagcx_kernel_core.h:146-162,209-230): value[0..2] = in1,
 * in2, out; value[3] = count[31:0] | nthreads[47:32] | datatype[51:48] |
 * redop[55:52] | state[57:56].
 */
typedef struct fxReduceTrigger {
  uint64_t value[4];
} fxReduceTrigger;

enum {
  fxTriggerAvailable = 0,
  fxTriggerEnqueued = 1,
  fxTriggerInprogress = 2,
  fxTriggerComplete = 3
};

/* flagcxReduceTrigger::setValue (flagcx/core/flagcx_reduce_kernel_host.cc:6-26) */
void fx_trigger_set(fxReduceTrigger *t, uint64_t in1, uint64_t in2,
                    uint64_t out, size_t count, size_t nthreads, int dtype,
                    int op, int state);
/* the device-side getters (flagcx_reduce_kernel_device.cu:15-43) */
void fx_trigger_get(const fxReduceTrigger *t, uint64_t *in1, uint64_t *in2,
                    uint64_t *out, uint64_t *count, uint64_t *nthreads,
                    int *dtype, int *op, int *state);

/*
 * Execute n triggers (host array) as batched launches: the stream-ordered
 * replacement of the polling consumer flagcxCollectiveKernel
 * (flagcx_reduce_kernel_device.cu:88-186).  Consecutive triggers with equal
 * dtype/op share a launch; triggers of one launch must not depend on each
 * other.  nthreads and state fields are ignored.
 */
int fx_reduce_triggers(const fxReduceTrigger *triggers, size_t n, void *stream);

/*
 * The reference's reduce FIFO, host side (flagcx/core/flagcx_reduce_kernel_host.cc:46-98):
 * a pinned buffer of uint64 words [capacity, consumed, produced, terminate]
 * followed by `capacity` triggers.  fx_fifo_enqueue returns idx = -1 when the
 * ring is full or the slot has not been collected yet (the caller retries);
 * fx_fifo_poll_state / fx_fifo_set_state are pollState / setState.  One
 * producer thread per ring, as in the reference.
 */
size_t fx_fifo_bytes(size_t capacity);
int fx_fifo_init(uint64_t *fifo, size_t capacity);
int fx_fifo_enqueue(uint64_t *fifo, uint64_t in1, uint64_t in2, uint64_t out,
                    size_t count, size_t nthreads, int dtype, int op, int *idx);
int fx_fifo_poll_state(const uint64_t *fifo, int idx);
int fx_fifo_set_state(uint64_t *fifo, int idx, int state);
int fx_fifo_terminate(uint64_t *fifo);
/*
 * The producer loop of the reference's scheduler for a set of independent
 * triggers (processReadyQueue + processInflightQueue,
 * flagcx/runner/uni_runner_impl.cc:1701-1794): enqueue all n, as slots free up,
 * poll each for Complete and hand its slot back (state Available).  Returns when
 * all n are complete, or flagcxInternalError after spinLimit consecutive polls
 * without progress (no consumer running).  The state field of the triggers
 * passed in is ignored.
 */
int fx_fifo_run_batch(uint64_t *fifo, const fxReduceTrigger *triggers, size_t n,
                      unsigned long long spinLimit);

/*
 * FIFO-compatible consumer: the drop-in for flagcxLaunchCollectiveKernel
 * (flagcx/adaptor/kernel/nvidia/flagcx_reduce_kernel_device.cu:88-192).  A
 * persistent full-width kernel executes every trigger the host enqueues, for
 * every op and type, and marks it Complete; it returns when `terminate`
 * is set and the ring is drained, or after maxIdlePolls consecutive empty
 * polls of the host ring (one to two microseconds each; so it always ends).
 * fifoDevicePointer is hostGetDevicePointer() of the pinned ring, fifoHost
 * the ring itself.  Triggers that sit in the ring at
 * the same time must not depend on each other, unless the consumer was
 * created with FX_FIFO_IN_ORDER=1 in the environment: then one trigger at a
 * time is executed, the next only after the previous one is Complete, as the
 * reference's single-block consumer does, and a trigger may read what an
 * earlier one in the ring wrote.  Capacity <= 1024.  The grid is one
 * workgroup per compute unit (the first talks to the host, the others work) and
 * never more workgroups than the device holds at the same time (a trigger
 * completes when all its workgroups have reported in); FX_FIFO_WGS or
 * FX_FIFO_WGS_PER_CU (environment, read at fx_fifo_consumer_create) ask for
 * another size within that limit.
 * A ring can be served again after its consumer has ended: the new kernel
 * reads `consumed` from the ring when it starts (so it may be enqueued on the
 * same stream while the earlier one is still running); triggers enqueued in
 * between are served first.
 * While the consumer runs, calls that wait for the whole device (hipFree,
 * hipDeviceSynchronize) block until it has ended: set `terminate` first.
 */
typedef struct fxFifoConsumer *fxFifoConsumer_t;
enum { FX_FIFO_RUNNING = 0, FX_FIFO_EXIT_TERMINATE = 1, FX_FIFO_EXIT_IDLE = 2 };
int fx_fifo_consumer_create(fxFifoConsumer_t *consumer, size_t capacity);
int fx_fifo_consumer_launch(fxFifoConsumer_t consumer, void *fifoDevicePointer,
                            const uint64_t *fifoHost,
                            unsigned long long maxIdlePolls, void *stream);
/* after the stream has drained: why the kernel ended, how many triggers it
 * completed, how many it skipped for an unsupported dtype / op */
int fx_fifo_consumer_status(fxFifoConsumer_t consumer, int *exitReason,
                            uint64_t *completed, uint64_t *badTriggers);
int fx_fifo_consumer_destroy(fxFifoConsumer_t consumer);

/* k-way slice descriptor: up to 8 inputs, `count` elements. */
typedef struct fxSliceDesc {
  const void *in[FX_MAX_SLICE_INPUTS];
  void *out;
  uint64_t count;
} fxSliceDesc;

/*
 * Reduce n independent slices (host array), each k-way in input order, with
 * as few launches as possible.  This is what the chunk / slice / red-slice
 * partition of flagcx/runner/uni_runner_impl.cc:661-1007 feeds: one descriptor
 * per reduce node.
 */
int fx_reduce_slices(const fxSliceDesc *slices, size_t n, int k, int dtype,
                     int op, void *stream);

/*
 * Slices whose result goes to several buffers at once: out[0..nout-1] all
 * receive in[0] (op) ... (op) in[k-1].  One pass reads the k inputs once and
 * stores nout times -- what the reference gets from multicast stores
 * (multimem.st in flagcx/adaptor/kernel/nvidia/custom_allreduce.cu, the NVLS
 * variants of the allreduce kernel) and what an all-reduce over n ranks on one
 * GPU needs: (k + nout) * size bytes of traffic instead of the
 * (k + 1 + 2 * (nout - 1)) * size of reduce-then-copy.  op = -1 makes it a
 * broadcast copy (k = 1, count in bytes, dtype ignored).  Every out[j] may
 * alias one in[p] exactly.  Outputs that do not share out[0]'s alignment
 * within 16 bytes are served by a reduce into out[0] plus copies.
 */
typedef struct fxBcastDesc {
  const void *in[FX_MAX_SLICE_INPUTS];
  void *out[FX_MAX_SLICE_INPUTS];
  uint64_t count;
} fxBcastDesc;
int fx_reduce_bcast_slices(const fxBcastDesc *slices, size_t n, int k, int nout,
                           int dtype, int op, void *stream);

/*
 * The same with the k inputs of every slice combined in another association
 * than the input-order fold -- the two the reference's own multi-step paths
 * produce -- in ONE launch, every input read once:
 *   FX_FOLD_CHAIN       in[0] (op) in[1] (op) ... left to right (what
 *                       fx_reduce_bcast_slices does).
 *   FX_FOLD_TREE        the binomial tree of flagcxReduce through the uniRunner
 *                       (flagcx/runner/uni_runner_impl.cc:1314-1326,1372-1477):
 *                       in[a] is tree rank a, i.e. rank (a + root) % n; in round i
 *                       every tree rank a with more than i receive steps computes
 *                       partial(a) = partial(a + 2^i) (op) partial(a), received
 *                       operand first; the result is partial(0).
 *   FX_FOLD_KEEP_LOCAL  the host ring's chain (flagcx/service/bootstrap.cc:853-871
 *                       with std::max / std::min, flagcx/service/include/utils.h:
 *                       707-725): res = in[0]; res = in[j] (op) res for j = 1..k-1,
 *                       the step's local operand first, so that a NaN hides what
 *                       was folded before it exactly as on the ring.
 * Every step of the tree and of the keep-local chain is a complete two-input
 * reduction in the element type (16-bit sums and products are rounded after
 * every step), as when each step is a launch of its own.  flagcxAvg with an
 * order other than FX_FOLD_CHAIN is flagcxNotSupported (a mean is not a tree of
 * two-input means), as are FX_OP_ELEMENT_FOLD and FX_FOLD_KEEP_LOCAL sums or
 * products of three or more fp16 / bf16 inputs (types the host ring does not
 * carry, flagcx/service/include/utils.h:690-694).  With FX_FOLD_TREE or
 * FX_FOLD_KEEP_LOCAL and three or more floating-point inputs, all outputs of a
 * slice must share out[0]'s alignment within 16 bytes (flagcxInvalidArgument
 * otherwise).
 */
enum { FX_FOLD_CHAIN = 0, FX_FOLD_TREE = 1, FX_FOLD_KEEP_LOCAL = 2 };
int fx_reduce_ordered(const fxBcastDesc *slices, size_t n, int k, int nout,
                      int dtype, int op, int order, void *stream);

/*
 * The same for ONE segment with up to FX_MAX_INPUTS inputs and FX_MAX_INPUTS
 * outputs: outs[0..nout) all receive the fold of ins[first], ins[first+1], ...
 * (wrapping), in one launch and with (k + nout) * size bytes of traffic.  This
 * is the all-reduce of more simulated ranks than a descriptor has slots
 * (the reference's LSA kernel reads every peer and stores the result once per
 * rank, custom_allreduce.cu:370-394, for any nRanks).  op = -1 copies ins[0]
 * (k = 1, count in bytes).  Outputs that do not share outs[0]'s alignment
 * within 16 bytes are served by a reduce into outs[0] plus copies.
 */
int fx_reduce_bcast(void *const *outs, int nout, const void *const *ins, int k,
                    size_t count, int dtype, int op, int first, void *stream);

/*
 * Several chunks of one collective over up to FX_MAX_INPUTS ranks in ONE
 * launch -- what a reduce-scatter, an all-gather or a ring-order all-reduce
 * over more ranks than a slice descriptor has slots is made of.  Chunk c takes
 * `count` elements at element offset in_off of the inputs: all k of them, folded
 * in the order first, first + 1, ... (wrapping), or the single input in_sel
 * (in_sel >= 0).  The result goes to element offset out_off of every output
 * (out_sel = -1) or of output out_sel alone.  op = -1 copies (every chunk
 * names its in_sel; offsets and counts in bytes).  Outputs of one chunk that do
 * not share an offset within 16 bytes are refused (flagcxInvalidArgument).
 */
typedef struct fxChunk {
  uint64_t in_off, out_off, count;
  int first, in_sel, out_sel;
} fxChunk;
int fx_reduce_chunks(void *const *outs, int nout, const void *const *ins, int k,
                     const fxChunk *chunks, int nchunks, int dtype, int op,
                     void *stream);

/*
 * All-to-all of equal blocks over n <= FX_MAX_INPUTS ranks in ONE launch:
 * block i of send[r] (block_bytes each) becomes block r of recv[i], for every
 * r and i -- the data movement of flagcxAlltoAll (flagcx/include/flagcx.h:
 * 466-470; the reference builds it from n grouped send / recv pairs per rank,
 * flagcx/adaptor/ccl/rccl_adaptor.cc:222-246).  The kernel works out each
 * block's two addresses from the 2 n base pointers, so nothing grows with
 * n * n but the grid.  No send block may overlap a receive block (in place:
 * stage first); any alignment.
 */
int fx_alltoall(void *const *recv, const void *const *send, int n, size_t block_bytes, void *stream);


/*
 * Copy n independent byte ranges (in[0] -> out, `count` = BYTES): the Cpy node
 * and the all-gather landing copies (uni_runner_impl.cc:322-344,1649-1662;
 * flagcx/core/p2p.cc:257-283) as one launch.
 */
int fx_copy_slices(const fxSliceDesc *slices, size_t n, void *stream);

/*
 * Device-resident descriptor tables for plans that are launched repeatedly.
 * Creation uploads synchronously; launch is enqueue-only.  op = -1 makes a
 * copy plan (count in bytes, dtype ignored, k = 1).
 */
typedef struct fxPlan *fxPlan_t;
int fx_plan_create(fxPlan_t *plan, const fxSliceDesc *slices, size_t n, int k,
                   int dtype, int op);
int fx_plan_launch(fxPlan_t plan, void *stream);
int fx_plan_destroy(fxPlan_t plan);

/*
 * fx_plan_create + fx_plan_launch in one call that allocates nothing.  It has
 * no counterpart in the reference: it is for callers that cannot allocate
 * device memory at the call (code inside a HIP graph capture, tight serving
 * loops, harnesses that forbid it).  The descriptor table and the tile-prefix
 * table, which a plan keeps in memory it allocates, live in a static device
 * array of FX_STATIC_MAX_SLICES descriptors (about 84 KiB per GPU, held until
 * the process ends); the table is filled on `stream` by small kernels whose
 * arguments carry the descriptors, then the same kernel as fx_plan_launch
 * runs.  Same arguments, merging of adjacent slices and results as
 * fx_plan_create (op = -1: copy, count in bytes).  More than
 * FX_STATIC_MAX_SLICES descriptors after merging -> flagcxInvalidArgument (4)
 * and nothing is enqueued.  All calls on one GPU share the one table: a call
 * may be enqueued only when the previous call's kernels on that GPU are
 * ordered before it (same stream, or an event between the streams);
 * overlapping calls race.  The first call on a GPU looks the array's address
 * up once (make it outside a capture).
 */
#define FX_STATIC_MAX_SLICES 1024
int fx_reduce_slices_static(const fxSliceDesc *slices, size_t n, int k,
                            int dtype, int op, void *stream);

/*
 * alltoallv pack: gather npeers segments of sendbuff (element displacements
 * sdispls[i], element counts sendcounts[i]; host arrays) into contiguous
 * slots of `packed`, slot_i = sum_{j<i} sendcounts[j].  unpack is the inverse
 * scatter into recvbuff at rdispls[i].  Segment addressing is that of
 * flagcx/service/bootstrap.cc:1253-1258 and flagcx/runner/uni_runner.cc:197-210;
 * zero counts are skipped (flagcx/adaptor/include/adaptor.h:77).
 */
int fx_pack(void *packed, const void *sendbuff, const size_t *sendcounts,
            const size_t *sdispls, int npeers, int dtype, void *stream);
int fx_unpack(void *recvbuff, const void *packed, const size_t *recvcounts,
              const size_t *rdispls, int npeers, int dtype, void *stream);

/* getFlagcxDataTypeSize (flagcx/flagcx.cc:35-66) for every FlagCX dtype. */
size_t fx_dtype_size(int dtype);

/*
 * Remainder-balanced split used (nested) for rank chunks, slices and
 * red-slices (uni_runner_impl.cc:100-131,433-457,854-866); offsets in elements.
 */
void fx_split(size_t total, size_t parts, size_t idx, size_t *cnt, size_t *off);

/* Automatic red-slice count, single-precision as in uni_runner_impl.cc:694-701. */
size_t fx_nredslices(size_t count, int nranks, size_t nslices,
                     size_t nredslices, size_t redslicesize);

const char *fx_version(void);

#ifdef __cplusplus
}

/*
 * The reference's own launcher of the trigger-ring consumer, under its own
 * name, signature and C++ linkage (declared in
 * flagcx/include/flagcx_kernel_internal.h:56, defined in
 * flagcx/adaptor/kernel/nvidia/flagcx_reduce_kernel_device.cu:188-192, called
 * by runUniRunner, flagcx/runner/uni_runner_impl.cc:1872-1874), so that the
 * reference's scheduler links against libflagcx-kernels-mi355x.so and runs
 * without a source change.  fifoBuffer is hostGetDevicePointer() of the pinned
 * ring; the capacity is read from word 0 of the ring.  nthreads and nblocks
 * are accepted and ignored (this consumer sizes itself to the device, see
 * fx_fifo_consumer_create).  The kernel ends when the ring's terminate word is
 * set and the ring is drained; the bound every wait in it carries is
 * FX_FIFO_MAX_IDLE_POLLS polls of an idle ring (environment; default 2^36).
 * FX_FIFO_IN_ORDER, FX_FIFO_WGS and FX_FIFO_WGS_PER_CU apply as for
 * fx_fifo_consumer_create.  The device memory one launch needs comes from a
 * per-device pool and goes back to it when the kernel has ended.  Failures are
 * reported on stderr (the signature has no result).
 */
void flagcxLaunchCollectiveKernel(void *fifoBuffer, size_t nthreads, size_t nblocks, flagcxStream_t stream);
#endif
#endif /* FLAGCX_AMD_FX_KERNELS_H_ */
