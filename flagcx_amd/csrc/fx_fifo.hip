// Reduce-FIFO compatibility mode: a persistent gfx950 kernel that consumes
// FlagCX's reduce-trigger ring unmodified, plus the host side of that ring.
//
// Ring layout and protocol are the reference's
// (flagcx/include/flagcx_kernel_core.h:44-67,146-162,209-230;
// flagcx/core/flagcx_reduce_kernel_host.cc:6-98; consumer
// flagcx/adaptor/kernel/nvidia/flagcx_reduce_kernel_device.cu:53-186):
//   uint64 words [0] capacity [1] consumed [2] produced [3] terminate, then
//   `capacity` 32-byte triggers; the producer writes a trigger with state
//   Enqueued and bumps `produced`; the consumer executes it and ORs state
//   Complete into value[3]; the producer polls for Complete and resets the slot
//   to Available; `terminate` = 1 ends the consumer once the ring is drained.
//
// What differs from the reference's consumer (one block of 32 threads that
// dequeues with a CAS and runs the reduce itself): here a full-width grid
// shares every trigger -- one workgroup per 16 KiB tile, all of them for a large
// trigger, taking tiles idx, idx + takers, ... -- and the last workgroup to
// finish marks it Complete.  Workgroup 0 does no arithmetic: it alone reads the
// pinned host ring (over PCIe) and mirrors it into device memory, where the
// other workgroups poll it and read up to kBatch upcoming triggers per round
// of reads.  Results are stored through the caches, so reporting in needs no
// cache write-back.  A trigger is Complete once every workgroup that takes part
// of it has reported in, so all workgroups of the grid must be resident at the
// same time: the grid is never larger than what the device holds at once
// (occupancy x compute units, see fx_fifo_consumer_create).  Every polling loop
// is bounded by maxIdlePolls, so even a grid that lost a workgroup ends.
// Triggers that are in the ring at the same time must be independent of each
// other, which is how the reference's scheduler uses it (a node is enqueued
// only after its parents completed, flagcx/runner/uni_runner_impl.cc:1727-1794)
// -- unless the consumer was created in order (FX_FIFO_IN_ORDER=1): then one
// trigger at a time is handed to the workers, the next only after the previous
// one is Complete, which is the reference consumer's own serial behaviour
// (flagcx_reduce_kernel_device.cu:104-185).
#include <sched.h>

#include <cstddef>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <new>
#include <vector>

#include "flagcx_amd/fx_kernels.h"
#include "fx_fifo_share.hpp"
#include "fx_launch.hpp"

using namespace fx;

namespace {

constexpr int kFifoU = 4;
constexpr int kBatch = 64;  // triggers a workgroup inspects per round of mirror reads: one per lane of a wavefront
// Triggers that reach the device several at a time are shared out more thinly:
// an eighth of the workgroups each, eight tiles per workgroup, so that eight
// times as many triggers run side by side and each workgroup's fixed cost per
// trigger is spread over eight tiles (2 MiB triggers with the ring kept full:
// 2.2 us each shared out fully, 1.6 us at a quarter, 1.5 us at an eighth).
// Workgroup 0 decides (it sees how many arrived together) and marks the
// mirrored copy in a bit the ring format leaves unused; the bit never reaches
// the host.
constexpr uint64_t kBulkArrivals = 4;
constexpr uint64_t kBulkBit = 1ull << 63;
constexpr uint32_t kMaxCapacity = 1024;
constexpr uint64_t kMirrorBatch = 64;  // triggers workgroup 0 mirrors per pass

struct FifoMirror {              // device memory, zeroed at creation
  uint64_t produced;             // triggers mirrored so far (written by workgroup 0)
  uint64_t terminate;
  uint64_t completed;            // triggers fully executed
  uint64_t exitReason;           // FX_FIFO_EXIT_*
  uint64_t badTriggers;          // triggers skipped because dtype / op is not carried
  uint64_t startPlus1;           // 1 + the ring's `consumed` when this launch began (0: not read yet)
  uint64_t pad[2];
  uint32_t done[kMaxCapacity];   // per slot: workgroups that finished their share
  uint64_t trig[kMaxCapacity][4];
  // Which trigger number trig[slot] holds (kNoTrigger while it is being
  // rewritten).  A workgroup that is not needed for a trigger does not hold up
  // its completion, so it may still be looking at a slot when the ring has come
  // round and workgroup 0 refills it; the number tells it so.
  uint64_t trigSeq[kMaxCapacity];
};
constexpr uint64_t kNoTrigger = ~0ull;

// The ring, the mirror and the counters are only ever touched with atomics of
// agent or system scope, which go to the coherent level themselves; ordering
// between them comes from waiting for acknowledgements (waitVectorMemory), not
// from cache-wide write-backs or invalidates.  The one cache operation left is
// the invalidate a workgroup does before it loads a trigger's input buffers.
template <class T>
__device__ __forceinline__ T pollSys(const T *p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}
template <class T>
__device__ __forceinline__ T pollDev(const T *p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
template <class T>
__device__ __forceinline__ void storeDev(T *p, T v) {
  __hip_atomic_store(p, v, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
}
template <class T>
__device__ __forceinline__ void storeSys(T *p, T v) {
  __hip_atomic_store(p, v, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}

// Make this wavefront wait until every vector memory operation it has issued is
// complete: loads returned, stores acknowledged at the scope they were issued
// with.  (A workgroup-scope fence alone emits no such wait on this target; the
// fences here only keep the compiler from moving accesses across the wait.)
__device__ __forceinline__ void waitVectorMemory() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0); expcnt and lgkmcnt left alone
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
}

// This workgroup's share of one two-input trigger.
template <int DT, int OP>
__device__ __forceinline__ void runShare(const void *in1, const void *in2, void *out, uint64_t count, Share sh) {
  using R = Red<DT, OP>;
  const void *in[2] = {in1, in2};
  SegWT<2> sg;  // written through: see the count-in below
  sg.keep = 0;  // inputs stream: a trigger's buffers were written by other agents, nothing of them is worth keeping
  const TilePlan tp = makeSeg<R::ES, kFifoU>(static_cast<Seg<2> &>(sg), in, out, count, 2);
  const uint64_t tiles = tp.tiles();
  // (tiles go to whichever workgroups the trigger's share names: no die grouping of columns here)
  for (uint64_t t = sh.idx; t < tiles; t += sh.takers) reduceTile<R, 2, kFifoU>(sg, tp, (uint32_t)t, 0u);
}

template <int DT>
__device__ __forceinline__ bool runShareOp(int op, const void *a, const void *b, void *o, uint64_t n, Share sh) {
  switch (op) {
    case flagcxSum: runShare<DT, flagcxSum>(a, b, o, n, sh); return true;
    case flagcxProd: runShare<DT, flagcxProd>(a, b, o, n, sh); return true;
    case flagcxMax: runShare<DT, flagcxMax>(a, b, o, n, sh); return true;
    case flagcxMin: runShare<DT, flagcxMin>(a, b, o, n, sh); return true;
    case flagcxAvg: runShare<DT, flagcxAvg>(a, b, o, n, sh); return true;
    default: return false;
  }
}

// Who works on trigger number seq: one workgroup per 16 KiB tile (per eight
// tiles for a trigger that arrived in bulk, see kBulkArrivals); the rest is
// shareFor's.
__device__ __forceinline__ Share shareOf(uint32_t rot, const void *in1, const void *in2, void *out, uint64_t count,
                                         int dtype, int op, bool bulk) {
  const int es = (int)dtypeSize(dtype);
  uint64_t tiles = 1;
  if (es != 0 && count != 0 && op >= flagcxSum && op <= flagcxAvg) {
    const bool co = sameLinePhase((uint64_t)(uintptr_t)in1, (uint64_t)(uintptr_t)out) &&
                    sameLinePhase((uint64_t)(uintptr_t)in2, (uint64_t)(uintptr_t)out);
    tiles = planTiles((uint64_t)(uintptr_t)out, count, es, kFifoU, handOutFor(co, 2)).tiles();
  }
  return shareForRot(gridDim.x, blockIdx.x, rot, tiles, bulk);
}

// Value of lane `src` of the wavefront as a wave-uniform 64-bit scalar.
__device__ __forceinline__ uint64_t fromLane(uint64_t v, int src) {
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)v, src);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(v >> 32), src);
  return ((uint64_t)hi << 32) | lo;
}

// Clears the mirror before a consumer launch.  A kernel rather than a memset
// node so that the launch sequence stays safe to record into a HIP graph.
__global__ void __launch_bounds__(kBlock) clearMirror(uint64_t *words, uint32_t n) {
  for (uint32_t i = blockIdx.x * kBlock + threadIdx.x; i < n; i += gridDim.x * kBlock) words[i] = 0;
}

__global__ void __launch_bounds__(kBlock)
fifoConsumer(uint64_t *host, FifoMirror *m, uint32_t cap, uint32_t inOrder, uint64_t maxIdlePolls) {
  __shared__ uint64_t sh[3];                  // [0] state, [1] triggers in this batch, [2] which of them this workgroup works on
  // Where this launch starts: the ring's `consumed` as the previous consumer
  // left it.  Read here, not on the host at enqueue time, because an earlier
  // consumer on the same stream may still be running then.  Workgroup 0 reads it
  // (it is also the one that overwrites it later) and passes it on through the
  // mirror; the others wait for it, bounded like every wait here.
  if (threadIdx.x == 0) {
    uint64_t s1 = 0;
    if (blockIdx.x == 0) {
      s1 = pollSys(host + 1) + 1;
      storeDev(&m->startPlus1, s1);
    } else {
      const uint64_t patience = (maxIdlePolls > (~0ull >> 5)) ? maxIdlePolls : maxIdlePolls * 32;
      for (uint64_t spins = 0; (s1 = pollDev(&m->startPlus1)) == 0 && spins <= patience; spins++)
        __builtin_amdgcn_s_sleep(8);
    }
    sh[0] = s1;
  }
  __syncthreads();
  const uint64_t startPlus1 = sh[0];
  __syncthreads();
  if (startPlus1 == 0) return;                // workgroup 0 never showed up: nothing can be done safely
  const uint64_t startSeq = startPlus1 - 1;
  __shared__ uint64_t shTrig[kBatch][4];     // their words
  __shared__ uint32_t shIdx[kBatch], shTakers[kBatch];   // this workgroup's share of each (see Share)
  enum { kWork = 0, kExitTerminate = FX_FIFO_EXIT_TERMINATE, kExitIdle = FX_FIFO_EXIT_IDLE };
  uint64_t seq = startSeq;
  // the slot of trigger `seq` and its rotation, carried along with seq instead of worked out by division per trigger
  const uint32_t pool = gridDim.x > 1 ? gridDim.x - 1 : 1u, rotBy = rotStep(pool);
  uint32_t slotNow = (uint32_t)(startSeq % cap), rot = rotOf(startSeq, pool);
  uint64_t *hostTrig = host + 4;
  // workgroup 0, wavefront 0 (all of these stay wave-uniform):
  uint64_t mirrored = startSeq;      // triggers copied to the mirror so far
  uint64_t lastSeenCompleted = 0;    // progress of the workers, for the idle count
  bool hostTermSeen = false;
  const uint32_t lane = threadIdx.x;
  const uint64_t idleLimit = (blockIdx.x == 0 || maxIdlePolls > (~0ull >> 5)) ? maxIdlePolls : maxIdlePolls * 32;
  for (;;) {
    if (threadIdx.x < 64) {
      // Wavefront 0 does the polling.  Reads over PCIe cost microseconds each, so
      // they are issued by different lanes of one instruction and the results are
      // broadcast; every branch below depends on broadcast values only.
      uint64_t idle = 0, state, p = 0;  // p: triggers published so far, as last polled
      bool termSeen = false;
      for (;;) {
        uint64_t term, termMirror = 0;
        if (blockIdx.x == 0) {
          if (mirrored <= seq) {  // nothing mirrored is waiting for this workgroup: talk to the host
            // one round of reads: the host's `produced` and `terminate` over PCIe and,
            // alongside them, the workers' progress and the mirror's terminate word
            uint64_t v = 0;
            if (lane < 2) v = pollSys(host + 2 + lane);
            else if (lane == 2) v = pollDev(&m->completed);
            else if (lane == 3) v = pollDev(&m->terminate);
            const uint64_t hp = fromLane(v, 0), ht = fromLane(v, 1);
            const uint64_t c = fromLane(v, 2);
            termMirror = fromLane(v, 3);
            // In order: the next trigger goes out only when everything handed out so far is complete.
            if (mirrored < hp && (!inOrder || c == mirrored - startSeq)) {
              __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "");  // the triggers behind `produced`
              // at most kMirrorBatch triggers per pass (four words per lane); the rest next time round
              const uint64_t arrived = inOrder ? 1 : hp - mirrored;
              const uint64_t upTo = mirrored + (arrived < kMirrorBatch ? arrived : kMirrorBatch);
              const uint64_t words = 4 * (upTo - mirrored);
              const uint32_t mslot = (uint32_t)(mirrored % cap);   // slot of the first trigger of this pass; 32-bit arithmetic from here
              // Refill the slots like a sequence lock: number invalid, words, number
              // valid.  All of these are agent-scope atomic stores (they go to the
              // coherent cache level themselves); between the phases the wavefront
              // waits for one phase's stores to be acknowledged before it issues the
              // next -- no cache write-back each.  The words come over PCIe (over a
              // microsecond); the stores that take the slots out of service -- number
              // invalid, count-in counter back to zero: the previous trigger in a slot
              // is long complete, or the host could not have reused it -- are issued
              // behind those reads and acknowledged while they are in flight.
              uint64_t fetched[4];
#pragma unroll
              for (int r = 0; r < 4; r++) {
                const uint64_t w = lane + 64ull * r;
                fetched[r] = 0;
                if (w < words) fetched[r] = pollSys(hostTrig + 4 * ((mslot + (uint32_t)(w / 4)) % cap) + (w & 3));
              }
              for (uint64_t w = lane; w < words; w += 64)
                if ((w & 3) == 0) {
                  const uint32_t slot = (mslot + (uint32_t)(w / 4)) % cap;
                  __hip_atomic_store(&m->trigSeq[slot], kNoTrigger, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                  __hip_atomic_store(&m->done[slot], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
              waitVectorMemory();
#pragma unroll
              for (int r = 0; r < 4; r++) {
                const uint64_t w = lane + 64ull * r;
                if (w < words) {
                  const uint32_t slot = (mslot + (uint32_t)(w / 4)) % cap;
                  uint64_t word = fetched[r];
                  if ((w & 3) == 3) word = (arrived >= kBulkArrivals) ? (word | kBulkBit) : (word & ~kBulkBit);
                  __hip_atomic_store(&m->trig[slot][w & 3], word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
              }
              waitVectorMemory();
              for (uint64_t w = lane; w < words; w += 64)
                if ((w & 3) == 0)
                  __hip_atomic_store(&m->trigSeq[(mslot + (uint32_t)(w / 4)) % cap], mirrored + w / 4, __ATOMIC_RELAXED,
                                     __HIP_MEMORY_SCOPE_AGENT);
              waitVectorMemory();  // every lane's copies are acknowledged before the new count goes out
              mirrored = upTo;
              if (lane == 0) {
                __hip_atomic_store(&m->produced, upTo, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                // `consumed` counts triggers TAKEN from the ring, as the reference's
                // dequeue does (flagcx_reduce_kernel_device.cu:53-73); the producer only
                // uses it to see whether the ring is full, the slot's state word says
                // when a slot is free again.  Published at once, so that the producer is
                // never held up by this loop's pace.
                __hip_atomic_store(host + 1, upTo, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
              }
              idle = 0;  // the host is alive
            }
            // The host sets terminate after its last enqueue, but two relaxed
            // polls may be served out of order: act on terminate only on the poll
            // AFTER the one that first saw it, when `produced` has been re-read.
            // And only once everything the host has produced is mirrored (a pass
            // takes at most kMirrorBatch triggers).
            if (ht && mirrored >= hp) {
              if (hostTermSeen && lane == 0) storeDev(&m->terminate, ht);
              hostTermSeen = true;
            }
            if (c != lastSeenCompleted) {
              lastSeenCompleted = c;
              idle = 0;  // so are the workers
            }
          }
          if (mirrored > seq) {  // a one-workgroup grid working off its own backlog: no host round this time
            uint64_t t = 0;
            if (lane == 0) t = pollDev(&m->terminate);
            termMirror = fromLane(t, 0);
          }
          term = termMirror;
          // With workers in the grid this workgroup never takes a tile, so it does
          // not look at the triggers it has mirrored at all (three dependent reads
          // each): it goes straight back to the host.
          if (gridDim.x > 1) seq = mirrored;
          p = mirrored;
        } else {
          uint64_t t = 0, q = 0;
          if (lane == 0) {
            t = pollDev(&m->terminate);
            q = pollDev(&m->produced);
          }
          term = fromLane(t, 0);
          p = fromLane(q, 0);
        }
        if (p > seq) { state = kWork; break; }
        if (term) {
          if (termSeen) { state = kExitTerminate; break; }  // same two-step rule as above
          termSeen = true;
          continue;
        }
        // Workgroup 0 decides when the kernel has idled long enough and tells the
        // others through the mirror's terminate word, so that all leave together;
        // their own limit (their polls are several times faster) is only the
        // backstop that makes every loop finite.
        if (++idle > idleLimit) {
          if (blockIdx.x == 0 && lane == 0) storeDev(&m->terminate, (uint64_t)kExitIdle);
          state = kExitIdle;
          break;
        }
        // Workgroup 0 is alone on the PCIe link and each of its rounds already takes
        // over a microsecond; the workers poll device memory, 255 of them.
        if (blockIdx.x == 0) __builtin_amdgcn_s_sleep(4);
        else __builtin_amdgcn_s_sleep(32);
      }
      if (lane == 0) sh[0] = state;
      if (state == kWork) {
        // Reader side of the sequence lock, for up to kBatch triggers at once (lane
        // i looks at trigger seq + i): two dependent rounds of reads serve the whole
        // batch.  The writer takes a slot out of service BEFORE it touches the words
        // and puts the new number in AFTER, so if a slot carries the expected number
        // after its words were read, the words are that trigger's.  If not, the
        // ring has come round: the trigger is complete, which it could not be had
        // this workgroup been one of its workers -- so there is nothing to do.
        // (agent-scope atomic loads read the coherent cache level; each step's
        // loads have returned before the next step's are issued, without
        // invalidating anything in between.)
        const uint64_t ahead = p - seq;
        const uint32_t batch = (uint32_t)(ahead < (uint64_t)kBatch ? ahead : (uint64_t)kBatch);
        const bool mine = lane < batch;
        const uint64_t want = seq + lane;
        const uint32_t slot = (slotNow + lane) % cap;
        uint64_t after = kNoTrigger, w[4] = {0, 0, 0, 0};
        if (mine)
          for (int q = 0; q < 4; q++) w[q] = pollDev(&m->trig[slot][q]);
        waitVectorMemory();
        if (mine) after = pollDev(&m->trigSeq[slot]);
        // Every workgroup has to look at every trigger to learn whether it is one of
        // its workers, so that look must cost next to nothing: lane i decides for
        // trigger seq + i, all lanes at once, and the workgroup then only visits the
        // triggers it takes part in (walking the batch one trigger after the other,
        // 150 instructions each on a single wavefront, was 0.6 us per trigger --
        // the whole per-trigger floor of the pipelined ring).
        bool take = false;
        if (mine) {
          const uint64_t w3 = w[3] & ~kBulkBit;
          const Share share = shareOf((rot + lane * rotBy) % pool, (const void *)(uintptr_t)w[0], (const void *)(uintptr_t)w[1],
                                      (void *)(uintptr_t)w[2], w3 & 0xffffffffull, (int)((w3 >> 48) & 0xf),
                                      (int)((w3 >> 52) & 0xf), (w[3] & kBulkBit) != 0);
          // after != want: overtaken by the ring; idx >= takers: not needed for this trigger
          take = (after == want) && share.idx < share.takers;
          if (take) {
            for (int q = 0; q < 4; q++) shTrig[lane][q] = w[q];
            shIdx[lane] = share.idx;
            shTakers[lane] = share.takers;
          }
        }
        const uint64_t takes = __ballot(take);
        if (lane == 0) {
          sh[1] = batch;
          sh[2] = takes;
        }
      }
    }
    __syncthreads();
    const uint64_t state = sh[0];
    if (state != kWork) {
      if (threadIdx.x == 0 && blockIdx.x == 0) {
        // Workers may still be inside the last triggers.  `consumed` is where the
        // next launch starts, so it must not be published short of them: wait
        // (bounded, like every loop here) until all mirrored triggers are complete.
        const uint64_t owed = mirrored - startSeq;
        const uint64_t patience = (maxIdlePolls > (~0ull >> 5)) ? maxIdlePolls : maxIdlePolls * 32;
        for (uint64_t spins = 0; pollDev(&m->completed) < owed && spins <= patience; spins++)
          __builtin_amdgcn_s_sleep(32);
        storeSys(host + 1, startSeq + pollDev(&m->completed));
        storeDev(&m->exitReason, state);
      }
      break;
    }
    const uint32_t batch = (uint32_t)sh[1];
    for (uint64_t takes = sh[2]; takes != 0; takes &= takes - 1) {
      const uint32_t bi = (uint32_t)__builtin_ctzll(takes);
      const void *in1 = (const void *)(uintptr_t)shTrig[bi][0], *in2 = (const void *)(uintptr_t)shTrig[bi][1];
      void *out = (void *)(uintptr_t)shTrig[bi][2];
      const uint64_t w3 = shTrig[bi][3] & ~kBulkBit;
      const uint64_t count = w3 & 0xffffffffull;
      const int dtype = (int)((w3 >> 48) & 0xf), op = (int)((w3 >> 52) & 0xf);
      Share share;
      share.idx = shIdx[bi];
      share.takers = shTakers[bi];
      // The trigger's buffers may have been written by other agents since this
      // kernel last looked: drop stale cache lines before reading them.  Only a
      // workgroup that takes tiles does so (every workgroup doing it for every batch
      // it inspects costs more than a microsecond per round trip), and one wavefront
      // does it for the workgroup: the caches are the compute unit's and the die's,
      // and the barrier orders the other wavefronts' loads behind it.
      if (threadIdx.x < 64) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "");
      __syncthreads();
      bool ok = true;
      if (count) {
        switch (dtype) {
          case flagcxFloat32: ok = runShareOp<flagcxFloat32>(op, in1, in2, out, count, share); break;
          case flagcxInt32: ok = runShareOp<flagcxInt32>(op, in1, in2, out, count, share); break;
          case flagcxBfloat16: ok = runShareOp<flagcxBfloat16>(op, in1, in2, out, count, share); break;
          case flagcxFloat16: ok = runShareOp<flagcxFloat16>(op, in1, in2, out, count, share); break;
          case flagcxUint32: ok = runShareOp<flagcxUint32>(op, in1, in2, out, count, share); break;
          case flagcxInt8: ok = runShareOp<flagcxInt8>(op, in1, in2, out, count, share); break;
          case flagcxUint8: ok = runShareOp<flagcxUint8>(op, in1, in2, out, count, share); break;
          case flagcxInt64: ok = runShareOp<flagcxInt64>(op, in1, in2, out, count, share); break;
          case flagcxUint64: ok = runShareOp<flagcxUint64>(op, in1, in2, out, count, share); break;
          case flagcxFloat64: ok = runShareOp<flagcxFloat64>(op, in1, in2, out, count, share); break;
          default: ok = false;
        }
      }
      // Every wavefront waits until its own stores are acknowledged (s_waitcnt
      // vmcnt(0); a workgroup barrier alone does not make a wavefront wait for
      // its vector stores), then the barrier collects the four of them.
      waitVectorMemory();
      __syncthreads();
      if (threadIdx.x == 0) {
        const uint32_t slot = (slotNow + bi) % cap;
        // The results were stored through the caches (SegWT) and every wavefront
        // waited for its stores before the barrier above, so they are in memory
        // before this workgroup reports in: no cache write-back here (one per
        // workgroup and trigger cost 7 us on a 16 MiB trigger).
        const uint32_t prev = __hip_atomic_fetch_add(&m->done[slot], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (prev == share.takers - 1) {  // last one out completes the trigger
          // Everybody else has counted in, so everybody's results are in memory; this
          // thread reads none of them, and the counter is put back to zero by workgroup
          // 0 when it next fills the slot: Complete can go out at once.  No cache-wide
          // write-back or invalidate here -- either would stall every workgroup of this
          // die that is busy with another trigger (0.78 against 1.3 us per 256 KiB
          // trigger with the ring kept full).
          if (!ok) __hip_atomic_fetch_add(&m->badTriggers, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          __hip_atomic_store(hostTrig + 4 * slot + 3, w3 | ((uint64_t)fxTriggerComplete << 56), __ATOMIC_RELAXED,
                             __HIP_MEMORY_SCOPE_SYSTEM);
          __hip_atomic_fetch_add(&m->completed, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      }
    }  // the triggers of this batch that this workgroup takes part in
    seq += batch;
    slotNow = (slotNow + batch) % cap;
    rot = (rot + batch * rotBy) % pool;
    __syncthreads();  // the batch arrays are rewritten next
  }
}

}  // namespace

struct fxFifoConsumer {
  FifoMirror *mirror;
  uint32_t capacity;
  uint32_t grid;
  uint32_t inOrder;
};

namespace {

// Grid of the consumer on the current device (see fifoGridFor) and whether the
// environment asks for the in-order mode.
flagcxResult_t consumerShape(uint32_t *grid, uint32_t *inOrder) {
  int dev = 0, cus = 0, resident = 0;  // resident: workgroups of this kernel one compute unit holds at the same time
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
      hipOccupancyMaxActiveBlocksPerMultiprocessor(&resident, fifoConsumer, kBlock, 0) != hipSuccess || resident < 1)
    return flagcxUnhandledDeviceError;
  long wanted = 0;
  if (const char *e = getenv("FX_FIFO_WGS")) wanted = atol(e);
  else if (const char *e = getenv("FX_FIFO_WGS_PER_CU")) wanted = atol(e) * (long)(cus > 0 ? cus : 1);
  *grid = fifoGridFor(cus, resident, wanted);
  const char *io = getenv("FX_FIFO_IN_ORDER");
  *inOrder = (io && atoi(io) != 0) ? 1u : 0u;
  return flagcxSuccess;
}

flagcxResult_t launchConsumer(FifoMirror *mirror, uint32_t grid, uint32_t capacity, uint32_t inOrder, void *fifoDevicePointer,
                              unsigned long long maxIdlePolls, hipStream_t s) {
  static_assert(sizeof(FifoMirror) % sizeof(uint64_t) == 0, "FifoMirror is cleared in 8-byte words");
  const uint32_t words = (uint32_t)(sizeof(FifoMirror) / sizeof(uint64_t));
  flagcxResult_t rc = launchKernel(clearMirror, (words + kBlock - 1) / kBlock, s, (uint64_t *)mirror, words);
  if (rc != flagcxSuccess) return rc;
  // The kernel starts where the last consumer stopped (it reads the ring's
  // `consumed` itself): triggers enqueued before this launch are waiting between
  // `consumed` and `produced` and are served first.
  return launchKernel(fifoConsumer, grid, s, (uint64_t *)fifoDevicePointer, mirror, capacity, inOrder,
                      (uint64_t)maxIdlePolls);
}

// ---- mirrors of flagcxLaunchCollectiveKernel ----
// That entry point has no handle to hang per-ring state on, so the device-side
// mirror a launch needs comes from a per-device pool: taken at launch, handed
// back by a host function enqueued behind the kernel on the same stream (it
// only touches the pool; no device call is made from it).  The pool only grows
// to the number of consumers that ran at the same time, and is kept until the
// process ends.
constexpr int kMaxPoolDevices = 64;
struct MirrorPool {
  std::mutex mu;
  std::vector<FifoMirror *> idle[kMaxPoolDevices];
};
MirrorPool &mirrorPool() {
  static MirrorPool *pool = new MirrorPool();   // never destroyed: a host function may still run at exit
  return *pool;
}
struct MirrorTicket {
  int dev;
  FifoMirror *mirror;
};
void returnMirror(void *arg) {
  MirrorTicket *t = static_cast<MirrorTicket *>(arg);
  {
    MirrorPool &pool = mirrorPool();
    std::lock_guard<std::mutex> lock(pool.mu);
    pool.idle[t->dev].push_back(t->mirror);
  }
  delete t;
}

}  // namespace

extern "C" {
#pragma GCC visibility push(default)

// ---- host side of the ring (flagcx/core/flagcx_reduce_kernel_host.cc) ----

size_t fx_fifo_bytes(size_t capacity) { return (4 + 4 * capacity) * sizeof(uint64_t); }

int fx_fifo_init(uint64_t *fifo, size_t capacity) {
  if (!fifo || capacity == 0 || capacity > kMaxCapacity) return flagcxInvalidArgument;
  fifo[0] = capacity;
  fifo[1] = fifo[2] = fifo[3] = 0;
  memset(fifo + 4, 0, capacity * sizeof(fxReduceTrigger));
  __sync_synchronize();
  return flagcxSuccess;
}

int fx_fifo_enqueue(uint64_t *fifo, uint64_t in1, uint64_t in2, uint64_t out, size_t count, size_t nthreads,
                    int dtype, int op, int *idx) {
  if (!fifo || !idx) return flagcxInvalidArgument;
  *idx = -1;
  const uint64_t cap = fifo[0];
  const uint64_t produced = fifo[2], consumed = __atomic_load_n(&fifo[1], __ATOMIC_ACQUIRE);
  if (produced - consumed >= cap) {  // ring full: the caller retries
    sched_yield();
    return flagcxSuccess;
  }
  const uint64_t slot = produced % cap;
  fxReduceTrigger *t = reinterpret_cast<fxReduceTrigger *>(fifo + 4) + slot;
  const uint64_t state = (__atomic_load_n(&t->value[3], __ATOMIC_ACQUIRE) >> 56) & 0x3;
  if (state != fxTriggerAvailable) {  // slot not collected yet
    sched_yield();
    return flagcxSuccess;
  }
  fxReduceTrigger v;
  fx_trigger_set(&v, in1, in2, out, count, nthreads, dtype, op, fxTriggerEnqueued);
  memcpy(t, &v, sizeof(v));
  __atomic_fetch_add(&fifo[2], 1ull, __ATOMIC_RELEASE);
  *idx = (int)slot;
  return flagcxSuccess;
}

int fx_fifo_poll_state(const uint64_t *fifo, int idx) {
  if (!fifo || idx < 0 || (uint64_t)idx >= fifo[0]) return -1;
  const fxReduceTrigger *t = reinterpret_cast<const fxReduceTrigger *>(fifo + 4) + idx;
  return (int)((__atomic_load_n(&t->value[3], __ATOMIC_ACQUIRE) >> 56) & 0x3);
}

int fx_fifo_set_state(uint64_t *fifo, int idx, int state) {
  if (!fifo || idx < 0 || (uint64_t)idx >= fifo[0]) return flagcxInvalidArgument;
  fxReduceTrigger *t = reinterpret_cast<fxReduceTrigger *>(fifo + 4) + idx;
  uint64_t v = __atomic_load_n(&t->value[3], __ATOMIC_ACQUIRE);
  v = (v & ~(0x3ull << 56)) | (((uint64_t)state & 0x3) << 56);
  __atomic_store_n(&t->value[3], v, __ATOMIC_RELEASE);
  return flagcxSuccess;
}

int fx_fifo_terminate(uint64_t *fifo) {
  if (!fifo) return flagcxInvalidArgument;
  __atomic_store_n(&fifo[3], 1ull, __ATOMIC_RELEASE);
  return flagcxSuccess;
}

int fx_fifo_run_batch(uint64_t *fifo, const fxReduceTrigger *triggers, size_t n, unsigned long long spinLimit) {
  if (!fifo || (n && !triggers) || spinLimit == 0) return flagcxInvalidArgument;
  const uint64_t cap = fifo[0];
  if (cap == 0 || cap > kMaxCapacity) return flagcxInvalidArgument;
  // The ring's own protocol (trigger words, then `produced`; Complete polled per
  // slot; the slot handed back as Available), with the producer's traffic on the
  // shared lines kept to what the protocol needs.  The four header words share
  // one cache line with the consumer's `consumed`, and every access to a line
  // the other side wrote last is a miss, so:
  //  * `consumed` is not read at all: slots are handed out and collected in ring
  //    order here, so at most `cap` are in flight and the slot's own state word
  //    says whether it is free;
  //  * `produced` is bumped once for all the triggers written in one pass, not
  //    once per trigger (the consumer sees it jump; it reads the triggers below it);
  //  * completions are polled at the oldest outstanding slot only.
  // (One trigger per pass with a header read and a bump each cost 0.62 us per
  // trigger against a consumer that does nothing.)
  fxReduceTrigger *slots = reinterpret_cast<fxReduceTrigger *>(fifo + 4);
  const uint64_t first = fifo[2];   // this thread is the ring's only producer
  size_t issued = 0, collected = 0;
  unsigned long long idle = 0;
  while (collected < n) {
    bool progress = false;
    uint64_t wrote = 0;
    while (issued < n && issued - collected < cap) {
      fxReduceTrigger *t = slots + (first + issued) % cap;
      if (((__atomic_load_n(&t->value[3], __ATOMIC_ACQUIRE) >> 56) & 0x3) != fxTriggerAvailable) break;  // an earlier user's slot, not collected yet
      uint64_t in1, in2, out, count, nthreads;
      int dtype, op;
      fx_trigger_get(&triggers[issued], &in1, &in2, &out, &count, &nthreads, &dtype, &op, nullptr);
      fxReduceTrigger v;
      fx_trigger_set(&v, in1, in2, out, count, nthreads, dtype, op, fxTriggerEnqueued);
      memcpy(t, &v, sizeof(v));
      issued++;
      wrote++;
    }
    if (wrote) {
      __atomic_fetch_add(&fifo[2], wrote, __ATOMIC_RELEASE);
      progress = true;
    }
    while (collected < issued) {
      fxReduceTrigger *t = slots + (first + collected) % cap;
      const uint64_t w = __atomic_load_n(&t->value[3], __ATOMIC_ACQUIRE);
      if (((w >> 56) & 0x3) != fxTriggerComplete) break;
      __atomic_store_n(&t->value[3], w & ~(0x3ull << 56), __ATOMIC_RELEASE);   // Available
      collected++;
      progress = true;
    }
    if (progress) idle = 0;
    else if (++idle > spinLimit) return flagcxInternalError;
  }
  return flagcxSuccess;
}

// ---- device side ----

int fx_fifo_consumer_create(fxFifoConsumer_t *consumer, size_t capacity) {
  if (!consumer || capacity == 0 || capacity > kMaxCapacity) return flagcxInvalidArgument;
  *consumer = nullptr;
  fxFifoConsumer *c = new (std::nothrow) fxFifoConsumer();
  if (!c) return flagcxSystemError;
  c->capacity = (uint32_t)capacity;
  if (consumerShape(&c->grid, &c->inOrder) != flagcxSuccess || hipMalloc((void **)&c->mirror, sizeof(FifoMirror)) != hipSuccess) {
    delete c;
    return flagcxUnhandledDeviceError;
  }
  *consumer = c;
  return flagcxSuccess;
}

int fx_fifo_consumer_launch(fxFifoConsumer_t c, void *fifoDevicePointer, const uint64_t *fifoHost,
                            unsigned long long maxIdlePolls, void *stream) {
  if (!c || !fifoDevicePointer || !fifoHost || maxIdlePolls == 0) return flagcxInvalidArgument;
  if (fifoHost[0] != c->capacity) return flagcxInvalidArgument;
  return launchConsumer(c->mirror, c->grid, c->capacity, c->inOrder, fifoDevicePointer, maxIdlePolls, (hipStream_t)stream);
}

int fx_fifo_consumer_status(fxFifoConsumer_t c, int *exitReason, uint64_t *completed, uint64_t *badTriggers) {
  if (!c) return flagcxInvalidArgument;
  uint64_t head[8];  // produced, terminate, completed, exitReason, badTriggers, startPlus1, pad
  static_assert(offsetof(FifoMirror, done) == sizeof(head), "FifoMirror header layout");
  if (hipMemcpy(head, c->mirror, sizeof(head), hipMemcpyDeviceToHost) != hipSuccess) return flagcxUnhandledDeviceError;
  if (completed) *completed = head[2];
  if (exitReason) *exitReason = (int)head[3];
  if (badTriggers) *badTriggers = head[4];
  return flagcxSuccess;
}

int fx_fifo_consumer_destroy(fxFifoConsumer_t c) {
  if (!c) return flagcxSuccess;
  (void)hipFree(c->mirror);
  delete c;
  return flagcxSuccess;
}

#pragma GCC visibility pop
}

// The reference's own entry point, under its own name and C++ linkage
// (flagcx/include/flagcx_kernel_internal.h:56, defined in
// flagcx/adaptor/kernel/nvidia/flagcx_reduce_kernel_device.cu:188-192, called by
// runUniRunner, flagcx/runner/uni_runner_impl.cc:1872-1874), so that the
// scheduler links and runs unmodified: launch the consumer of the ring at
// `fifoBuffer` (the device pointer of the pinned ring) on `stream`.  nthreads
// and nblocks are accepted and ignored -- they size the reference's kernel, one
// block of 32 threads by default; this consumer sizes itself to the device.  The
// capacity is read from word 0 of the ring.  The kernel ends when the ring's
// terminate word is set and the ring is drained, as the reference's does; the
// bound every wait in it carries is FX_FIFO_MAX_IDLE_POLLS polls of an idle ring
// (environment; default 2^36, about a day).  There is no result to return:
// failures are reported on stderr, and a scheduler that then waits for a trigger
// to complete waits forever, as it would after a failed launch of the
// reference's kernel.
struct flagcxStream {   // the device adaptor's stream handle (flagcx/adaptor/include/amd_adaptor.h:13-23)
  hipStream_t base;
};

__attribute__((visibility("default"))) void flagcxLaunchCollectiveKernel(void *fifoBuffer, size_t nthreads, size_t nblocks,
                                                                         flagcxStream_t stream) {
  (void)nthreads;
  (void)nblocks;
  auto fail = [](const char *what) { fprintf(stderr, "flagcxLaunchCollectiveKernel: %s\n", what); };
  if (!fifoBuffer) return fail("no ring");
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxPoolDevices) return fail("no current device");
  // word 0 of the ring: through the host mapping of the pinned buffer when the runtime knows one, else a copy
  uint64_t capacity = 0;
  hipPointerAttribute_t attr;
  memset(&attr, 0, sizeof(attr));
  if (hipPointerGetAttributes(&attr, fifoBuffer) == hipSuccess && attr.hostPointer) {
    capacity = __atomic_load_n(static_cast<const uint64_t *>(attr.hostPointer), __ATOMIC_ACQUIRE);
  } else {
    (void)hipGetLastError();
    if (hipMemcpy(&capacity, fifoBuffer, sizeof(capacity), hipMemcpyDeviceToHost) != hipSuccess) return fail("cannot read the ring's capacity");
  }
  if (capacity == 0 || capacity > kMaxCapacity) return fail("ring capacity out of range (1..1024)");
  uint32_t grid = 0, inOrder = 0;
  if (consumerShape(&grid, &inOrder) != flagcxSuccess) return fail("cannot size the consumer");
  unsigned long long maxIdlePolls = 1ull << 36;
  if (const char *e = getenv("FX_FIFO_MAX_IDLE_POLLS")) {
    const unsigned long long v = strtoull(e, nullptr, 0);
    if (v) maxIdlePolls = v;
  }
  MirrorTicket *ticket = new (std::nothrow) MirrorTicket();
  if (!ticket) return fail("out of memory");
  ticket->dev = dev;
  ticket->mirror = nullptr;
  {
    MirrorPool &pool = mirrorPool();
    std::lock_guard<std::mutex> lock(pool.mu);
    if (!pool.idle[dev].empty()) {
      ticket->mirror = pool.idle[dev].back();
      pool.idle[dev].pop_back();
    }
  }
  if (!ticket->mirror && hipMalloc((void **)&ticket->mirror, sizeof(FifoMirror)) != hipSuccess) {
    delete ticket;
    return fail("cannot allocate the device-side mirror");
  }
  hipStream_t s = stream ? stream->base : nullptr;
  if (launchConsumer(ticket->mirror, grid, (uint32_t)capacity, inOrder, fifoBuffer, maxIdlePolls, s) != flagcxSuccess) {
    returnMirror(ticket);
    return fail("kernel launch failed");
  }
  // behind the kernel on the same stream: the mirror is free again once the consumer has ended
  if (hipLaunchHostFunc(s, returnMirror, ticket) != hipSuccess) {
    (void)hipGetLastError();   // the mirror stays out of the pool (one leaked block); the consumer itself runs
    fail("could not enqueue the mirror's return; it is not reused");
  }
}
