// Shared declarations of the simulated-rank layer: the communicator group, what
// a rank has posted, and the helpers the schedules, the send / recv matcher and
// the entry points all use.  Internal to the library.
#pragma once
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <string>
#include <new>
#include <vector>

#include "flagcx_amd/fx_kernels.h"
#include "flagcx_amd/fx_sim.h"
#include "fx_common.hpp"

struct flagcxStream {
  hipStream_t base;
};

namespace fxsim {


enum Kind {
  kNone = 0, kReduce, kAllReduce, kReduceScatter, kAllGather, kAlltoAllv, kCustomAllReduce,
  kGather, kScatter, kBroadcast, kAlltoAll, kBarrier
};

struct Post {
  bool posted = false;
  const void *send = nullptr;
  void *recv = nullptr;
  hipStream_t stream = nullptr;
  bool marked = false;     // rendezvous mode: the rank's own event already stands on its stream
  bool idle = false;       // rendezvous mode: the rank's stream had nothing left to do when it posted
  std::vector<size_t> sendcounts, sdispls, recvcounts, rdispls;
};

// One half of a point-to-point transfer waiting for its partner.
struct PendingP2p {
  bool isSend;
  int src, dst;            // ranks
  const void *sbuf;
  void *rbuf;
  size_t bytes;
  hipStream_t stream;
  uint64_t id;             // names this half for a sleeping poster (rendezvous mode)
  int owner;               // the rank that posted it
  bool idle, marked;       // rendezvous mode: its stream had nothing left to do / carries a mark of its own
  hipEvent_t mark;         // that mark: an event of this half alone (two halves of one bracket may sit on two streams,
                           // and a collective of the same rank re-records ready[owner]); from and back to Group::markPool
};

// What a sleeping poster finds when its partner has come (rendezvous mode).
struct P2pOutcome {
  flagcxResult_t res;
  hipStream_t where;       // the stream the copy was enqueued on
  hipEvent_t after;        // recorded behind that copy, an event of this copy alone (a rank may enqueue copies for two
                           // partners on two streams); nullptr if nothing was enqueued; back to Group::markPool when used
};

struct Group {
  int n = 0;
  int device = 0;
  std::mutex mu;
  std::string id;          // non-empty when created rank by rank (fxSimCommInitRank)
  int joined = 0, alive = 0;
  std::vector<char> taken;  // ranks that have joined
  std::vector<PendingP2p> p2p;
  hipEvent_t p2pBefore = nullptr, p2pAfter = nullptr;   // made at the first pair whose halves sit on two streams
  uint64_t nextP2pId = 1;
  std::map<uint64_t, P2pOutcome> p2pMatched;      // rendezvous mode: results awaiting their sleeping poster
  std::vector<hipEvent_t> markPool;               // rendezvous mode: events for the marks of pending halves and for the
                                                  // copies made for a sleeping partner, not in use
  // pending collective
  Kind kind = kNone;
  size_t count = 0;
  int dtype = 0, op = 0, root = 0, nposted = 0;
  std::vector<Post> posts;
  std::vector<hipEvent_t> ready;
  hipEvent_t done = nullptr;
  // rendezvous mode: posters sleep here until the collective they joined is launched
  std::condition_variable cv;
  std::atomic<uint64_t> launched{0};   // collectives launched (or abandoned) so far
  hipStream_t launchStream = nullptr;  // rendezvous mode: where the last collective went, for the ranks it woke
  flagcxResult_t lastResult = flagcxSuccess;
  long long timeoutMs = 30000;
  // configuration
  std::atomic<long long> sync{FX_SYNC_GROUP};   // read without the lock by a rank that marks its stream before posting
  long long algo = FX_ALGO_DIRECT, order = FX_ORDER_RANK;
  long long arith = FX_ARITH_DEFAULT;
  long long nslices = 1, nredslices = 0, redslicesize = 65536;
  // scratch: ring reduce-scatter partials / alltoallv staging.  Outgrown
  // blocks stay allocated until the group is destroyed: kernels enqueued earlier
  // may still use them, and freeing would wait for the whole device.
  void *scratch = nullptr;
  size_t scratchBytes = 0;
  std::vector<void *> outgrown;
  std::vector<void *> windows;
  size_t windowBytes = 0;
};

inline long long envParam(const char *name, long long dflt) {
  const char *e = getenv(name);
  if (!e || !*e) return dflt;
  char *end = nullptr;
  long long v = strtoll(e, &end, 0);
  return (end && *end == '\0') ? v : dflt;
}

inline flagcxResult_t R(int rc) { return (flagcxResult_t)rc; }
inline int mod(int a, int n) { return ((a % n) + n) % n; }
inline const char *cadd(const void *p, size_t bytes) { return (const char *)p + bytes; }
inline char *madd(void *p, size_t bytes) { return (char *)p + bytes; }

// Scratch of at least `bytes`.  Growing allocates a new block (at least twice
// the old size, so the blocks kept add up to less than the last one) and
// enqueues nothing that waits for the device.  A stream that is being captured
// cannot allocate: the caller reserves beforehand (FX_SIM_SCRATCH_BYTES) or
// gets flagcxInvalidUsage.
inline flagcxResult_t ensureScratch(Group *g, size_t bytes, hipStream_t s) {
  if (bytes <= g->scratchBytes) return flagcxSuccess;
  hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
  if (s && hipStreamIsCapturing(s, &cap) == hipSuccess && cap != hipStreamCaptureStatusNone) return flagcxInvalidUsage;
  size_t want = g->scratchBytes * 2;
  if (want < bytes) want = bytes;
  void *blk = nullptr;
  if (hipMalloc(&blk, want) != hipSuccess) {
    (void)hipGetLastError();
    if (want == bytes || hipMalloc(&blk, bytes) != hipSuccess) return flagcxUnhandledDeviceError;
    want = bytes;
  }
  if (g->scratch) g->outgrown.push_back(g->scratch);
  g->scratch = blk;
  g->scratchBytes = want;
  return flagcxSuccess;
}

// Rendezvous mode asks a rank's stream whether it is idle and marks it with an
// event that another rank's stream then waits for.  Neither is possible on a
// stream that is being captured (a query is illegal there and invalidates the
// capture; the wait would pull a second stream into it), so a call in that mode
// on such a stream is refused with flagcxInvalidUsage and enqueues nothing.
// Captures are for the single-thread mode, where every rank posts from one thread.
inline bool isCapturing(hipStream_t s) {
  hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
  return s && hipStreamIsCapturing(s, &cap) == hipSuccess && cap != hipStreamCaptureStatusNone;
}

// Descriptor lists of one collective: a handful of entries in the common case
// (one per rank), kept on the stack.
typedef fx::SmallVec<fxSliceDesc, 16> SliceList;
typedef fx::SmallVec<fxBcastDesc, 16> BcastList;
typedef fx::SmallVec<const void *, 16> PtrList;

inline fxSliceDesc copyDesc(const void *src, void *dst, size_t bytes) {
  fxSliceDesc d;
  memset(&d, 0, sizeof(d));
  d.in[0] = src;
  d.out = dst;
  d.count = bytes;
  return d;
}

struct Ctx {
  Group *g;
  hipStream_t s;
  int n;
  size_t ts;
  const void *send(int r) const { return g->posts[r].send; }
  void *recv(int r) const { return g->posts[r].recv; }
};

// The schedules (fx_sim_schedules.cc): what the last rank to post launches.
flagcxResult_t runAllReduce(const Ctx &c);
flagcxResult_t runReduce(const Ctx &c);
flagcxResult_t runReduceScatter(const Ctx &c);
flagcxResult_t runAllGather(const Ctx &c);
flagcxResult_t runAlltoAllv(const Ctx &c);
flagcxResult_t runGather(const Ctx &c);
flagcxResult_t runScatter(const Ctx &c);
flagcxResult_t runBroadcast(const Ctx &c);
flagcxResult_t runAlltoAll(const Ctx &c);
flagcxResult_t runCustomAllReduce(const Ctx &c);

}  // namespace fxsim

struct flagcxComm {
  fxsim::Group *g;
  int rank;
  uint64_t joined = 0;   // how many collectives the group had launched when this rank's last post was accepted
};
