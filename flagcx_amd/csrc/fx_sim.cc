// FlagCX collective entry points over simulated ranks on one GPU.
//
// Reference behaviour followed:
//   chunk/slice/red-slice  flagcx/runner/uni_runner_impl.cc:661-1007 (sliced ring
//                          all-reduce), :1009-1264 (ring reduce-scatter),
//                          :1266-1557 (tree reduce)
//   host-path schedule ... flagcx/service/bootstrap.cc:787-942,1039-1066
//   nranks == 1 .......... copy if out of place, else nothing (:669-691)
//   alltoallv addressing . flagcx/service/bootstrap.cc:1253-1279
//   custom allreduce ..... flagcx/adaptor/kernel/nvidia/custom_allreduce.cu:604-677
// The transport between ranks is elided: a rank reads its peer's buffer where
// the reference would receive a copy of it.
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

namespace {

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

long long envParam(const char *name, long long dflt) {
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
flagcxResult_t ensureScratch(Group *g, size_t bytes, hipStream_t s) {
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

fxSliceDesc copyDesc(const void *src, void *dst, size_t bytes) {
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

// More inputs than a slice descriptor carries: such pieces go through the
// runtime-k kernel, one launch each, so pieces that continue each other in the
// send buffers and in the output are gathered into one run first (the
// red-slice split alone cuts a 64 MiB all-reduce over 16 ranks into 512 pieces
// of 128 KiB).
struct KwayRun {
  size_t sendOff = 0, cnt = 0;
  void *out = nullptr;
  int first = 0;
};

flagcxResult_t launchRun(const Ctx &c, KwayRun &run) {
  if (run.cnt == 0) return flagcxSuccess;
  PtrList in;
  in.resize((size_t)c.n);
  for (int j = 0; j < c.n; j++) in[j] = cadd(c.send(j), run.sendOff * c.ts);
  const flagcxResult_t rc = R(fx_reduce_copy(run.out, in.data(), c.n, run.cnt, c.g->dtype, c.g->op, run.first, c.s));
  run = KwayRun();
  return rc;
}

// k-way reduce of element range [off, off+cnt) of every rank's sendbuff (+sendBase
// elements) into out, in order first, first+1, ...
flagcxResult_t kway(const Ctx &c, SliceList &descs, KwayRun &run, size_t sendOff, size_t cnt, void *out, int first) {
  if (cnt == 0) return flagcxSuccess;
  if (c.n <= FX_MAX_SLICE_INPUTS) {
    fxSliceDesc d;
    memset(&d, 0, sizeof(d));
    for (int j = 0; j < c.n; j++) d.in[j] = cadd(c.send(mod(first + j, c.n)), sendOff * c.ts);
    d.out = out;
    d.count = cnt;
    descs.push_back(d);
    return flagcxSuccess;
  }
  if (run.cnt && first == run.first && sendOff == run.sendOff + run.cnt && out == madd(run.out, run.cnt * c.ts)) {
    run.cnt += cnt;
    return flagcxSuccess;
  }
  const flagcxResult_t rc = launchRun(c, run);
  run.sendOff = sendOff;
  run.cnt = cnt;
  run.out = out;
  run.first = first;
  return rc;
}

flagcxResult_t flushKway(const Ctx &c, SliceList &descs, KwayRun &run) {
  flagcxResult_t rc = launchRun(c, run);
  if (rc != flagcxSuccess || descs.empty()) return rc;
  rc = R(fx_reduce_slices(descs.data(), descs.size(), c.n, c.g->dtype, c.g->op, c.s));
  descs.clear();
  return rc;
}

// The many-rank kernels store one result to several buffers with shared byte
// offsets: the receive buffers must agree in their low four address bits.
inline bool recvsAlignedAlike(const Ctx &c) {
  for (int r = 1; r < c.n; r++)
    if ((((uintptr_t)c.recv(r) ^ (uintptr_t)c.recv(0)) & 15u) != 0) return false;
  return true;
}

// One read, n stores: usable when both the inputs and the outputs of a
// descriptor fit its eight slots.
inline bool canBroadcast(const Ctx &c) { return c.n <= FX_MAX_SLICE_INPUTS; }

// Visit the (slice, red-slice) pieces of a chunk of ccnt elements at element
// offset coff, exactly as the reference nests its three splits.
template <class F>
flagcxResult_t forPieces(const Group *g, size_t ccnt, size_t coff, size_t nred, F f) {
  for (size_t s = 0; s < (size_t)g->nslices; s++) {
    size_t scnt, soff;
    fx_split(ccnt, (size_t)g->nslices, s, &scnt, &soff);
    for (size_t q = 0; q < nred; q++) {
      size_t rcnt, roff;
      fx_split(scnt, nred, q, &rcnt, &roff);
      flagcxResult_t rc = f(coff + soff + roff, soff + roff, rcnt);
      if (rc != flagcxSuccess) return rc;
    }
  }
  return flagcxSuccess;
}

// ---- the host path's schedule (FX_ORDER_HOST) ----
// Element range of chunk i: ceil(size / n) bytes rounded up to whole elements,
// the last non-empty chunk short, later ones empty (bootstrap.cc:900-922).
void hostChunk(size_t count, int n, int i, size_t *cnt, size_t *off) {
  const size_t chunk = (count + (size_t)n - 1) / (size_t)n;  // same as the byte formula divided by the element size
  if (chunk * (size_t)i >= count) {
    *off = count;
    *cnt = 0;
  } else {
    *off = chunk * (size_t)i;
    *cnt = (chunk * (size_t)(i + 1) >= count) ? count - *off : chunk;
  }
}

// Rank order in which a left-to-right fold reproduces the host ring's result for
// chunk c.  The ring computes x_c (op) (x_{c-1} (op) (.. (x_{c+2} (op) x_{c+1}))),
// local operand first (bootstrap.cc:805-871).  For sum / prod / avg the operands
// of one step commute bit for bit, so the fold runs c+1, c+2, .., c.  For max /
// min of integers ((a < b) ? b : a keeps the LOCAL value on a tie) the fold keeps
// its accumulator on a tie instead, so it runs c, c-1, .., c+1: either way the
// last rank of the ring wins ties.  (Floating max / min do not come here: NaN
// makes them order-dependent in a way only the step-by-step chain reproduces.)
void hostOrder(int c, int n, int op, std::vector<int> &order) {
  order.resize(n);
  const bool select = (op == flagcxMax || op == flagcxMin);
  for (int j = 0; j < n; j++) order[j] = select ? mod(c - j, n) : mod(c + 1 + j, n);
}

// Host-order reduce of `nchunks` element ranges (chunk i = [off[i], off[i]+cnt[i]) of
// every send buffer, folded in hostOrder(chunkId[i])) into outs[i][0..nout-1].
struct HostPiece {
  int chunk;
  size_t off, cnt;
  std::vector<void *> outs;
};

// max / min of floating types, exactly as the host ring evaluates them: n-1
// two-input steps res = local (op) received (bootstrap.cc:853-871), the local
// operand first, so that a NaN met on the way decides the result the way it
// does there (std::max / std::min return their FIRST argument whenever the
// comparison is false).  A left-to-right k-way fold cannot express that: once
// rank j's NaN has been kept by rank j, everything folded before it is lost.
// Step j of chunk c: local rank c+1+j, received = the previous partial (rank
// c+1's data in step 1).  Partials travel through scratch; the last step, whose
// local rank is c itself, writes the outputs.  One launch per step for all chunks.
flagcxResult_t chainHostPieces(const Ctx &c, const std::vector<HostPiece> &pieces) {
  Group *g = c.g;
  const int n = c.n;
  // Up to eight ranks: the whole chain of a piece in registers, one launch for
  // all pieces, every input read once (in[0] = rank c+1's data, in[j] = the
  // local operand of step j).  Outputs that do not share their offset within 16
  // bytes fall through to the step-by-step form below.
  if (n <= FX_MAX_SLICE_INPUTS) {
    BcastList bd;
    bool alike = true;
    int nout = 1;
    for (const HostPiece &p : pieces) {
      if (p.cnt == 0) continue;
      nout = (int)p.outs.size();
      if (nout > FX_MAX_SLICE_INPUTS) alike = false;
      fxBcastDesc d;
      memset(&d, 0, sizeof(d));
      for (int j = 0; j < n; j++) d.in[j] = cadd(c.send(mod(p.chunk + 1 + j, n)), p.off * c.ts);
      for (int o = 0; o < nout && o < FX_MAX_SLICE_INPUTS; o++) {
        d.out[o] = p.outs[o];
        alike = alike && ((((uintptr_t)p.outs[o] ^ (uintptr_t)p.outs[0]) & 15u) == 0);
      }
      d.count = p.cnt;
      bd.push_back(d);
    }
    if (bd.empty()) return flagcxSuccess;
    if (alike) return R(fx_reduce_ordered(bd.data(), bd.size(), n, nout, g->dtype, g->op, FX_FOLD_KEEP_LOCAL, c.s));
  }
  std::vector<size_t> soff(pieces.size(), 0);
  size_t total = 0;
  for (size_t i = 0; i < pieces.size(); i++) {
    soff[i] = total;
    total += (pieces[i].cnt * c.ts + 255) & ~(size_t)255;
  }
  if (total == 0) return flagcxSuccess;
  if (n > 2) {
    flagcxResult_t rc = ensureScratch(g, total, c.s);
    if (rc != flagcxSuccess) return rc;
  }
  SliceList plain, copies;
  BcastList bcast;
  int nout = 1;
  for (int j = 1; j < n; j++) {
    plain.clear();
    for (size_t i = 0; i < pieces.size(); i++) {
      const HostPiece &p = pieces[i];
      if (p.cnt == 0) continue;
      const void *local = cadd(c.send(mod(p.chunk + 1 + j, n)), p.off * c.ts);
      const void *received = (j == 1) ? cadd(c.send(mod(p.chunk + 1, n)), p.off * c.ts)
                                      : (const void *)madd(g->scratch, soff[i]);
      nout = (int)p.outs.size();
      if (j == n - 1 && nout > 1 && nout <= FX_MAX_SLICE_INPUTS) {
        fxBcastDesc d;
        memset(&d, 0, sizeof(d));
        d.in[0] = local;
        d.in[1] = received;
        for (int o = 0; o < nout; o++) d.out[o] = p.outs[o];
        d.count = p.cnt;
        bcast.push_back(d);
        continue;
      }
      fxSliceDesc d;
      memset(&d, 0, sizeof(d));
      d.in[0] = local;
      d.in[1] = received;
      d.out = (j == n - 1) ? p.outs[0] : madd(g->scratch, soff[i]);
      d.count = p.cnt;
      plain.push_back(d);
      if (j == n - 1)
        for (int o = 1; o < nout; o++) copies.push_back(copyDesc(p.outs[0], p.outs[o], p.cnt * c.ts));
    }
    flagcxResult_t rc = R(fx_reduce_slices(plain.data(), plain.size(), 2, g->dtype, g->op, c.s));
    if (rc != flagcxSuccess) return rc;
  }
  if (!bcast.empty()) return R(fx_reduce_bcast_slices(bcast.data(), bcast.size(), 2, nout, g->dtype, g->op, c.s));
  return R(fx_copy_slices(copies.data(), copies.size(), c.s));
}

inline bool isFloating(int dtype) {
  return dtype == flagcxFloat16 || dtype == flagcxBfloat16 || dtype == flagcxFloat32 || dtype == flagcxFloat64;
}

flagcxResult_t reduceHostPieces(const Ctx &c, const std::vector<HostPiece> &pieces) {
  if ((c.g->op == flagcxMax || c.g->op == flagcxMin) && isFloating(c.g->dtype)) return chainHostPieces(c, pieces);
  std::vector<int> order;
  BcastList bcast;
  SliceList plain;
  int nout = 0;
  for (const HostPiece &p : pieces) {
    if (p.cnt == 0) continue;
    hostOrder(p.chunk, c.n, c.g->op, order);
    nout = (int)p.outs.size();
    if (c.n <= FX_MAX_SLICE_INPUTS && nout <= FX_MAX_SLICE_INPUTS) {
      if (nout == 1) {
        fxSliceDesc d;
        memset(&d, 0, sizeof(d));
        for (int j = 0; j < c.n; j++) d.in[j] = cadd(c.send(order[j]), p.off * c.ts);
        d.out = p.outs[0];
        d.count = p.cnt;
        plain.push_back(d);
      } else {
        fxBcastDesc d;
        memset(&d, 0, sizeof(d));
        for (int j = 0; j < c.n; j++) d.in[j] = cadd(c.send(order[j]), p.off * c.ts);
        for (int o = 0; o < nout; o++) d.out[o] = p.outs[o];
        d.count = p.cnt;
        bcast.push_back(d);
      }
      continue;
    }
    // more than eight ranks: one runtime-k launch per piece, then copies
    PtrList in;
    in.resize((size_t)c.n);
    for (int j = 0; j < c.n; j++) in[j] = cadd(c.send(order[j]), p.off * c.ts);
    flagcxResult_t rc = R(fx_reduce_copy(p.outs[0], in.data(), c.n, p.cnt, c.g->dtype, c.g->op, 0, c.s));
    if (rc != flagcxSuccess) return rc;
    SliceList copies;
    for (int o = 1; o < nout; o++) copies.push_back(copyDesc(p.outs[0], p.outs[o], p.cnt * c.ts));
    rc = R(fx_copy_slices(copies.data(), copies.size(), c.s));
    if (rc != flagcxSuccess) return rc;
  }
  if (!plain.empty()) {
    flagcxResult_t rc = R(fx_reduce_slices(plain.data(), plain.size(), c.n, c.g->dtype, c.g->op, c.s));
    if (rc != flagcxSuccess) return rc;
  }
  if (!bcast.empty()) return R(fx_reduce_bcast_slices(bcast.data(), bcast.size(), c.n, nout, c.g->dtype, c.g->op, c.s));
  return flagcxSuccess;
}

flagcxResult_t runAllReduce(const Ctx &c) {
  Group *g = c.g;
  const int n = c.n;
  const size_t count = g->count, ts = c.ts;
  if (n == 1) {
    if (count && c.send(0) != c.recv(0)) {
      fxSliceDesc d = copyDesc(c.send(0), c.recv(0), count * ts);
      return R(fx_copy_slices(&d, 1, c.s));
    }
    return flagcxSuccess;
  }
  if (g->order == FX_ORDER_HOST) {  // the host path's chunks and fold order; every rank receives every chunk
    std::vector<HostPiece> pieces(n);
    for (int ch = 0; ch < n; ch++) {
      pieces[ch].chunk = ch;
      hostChunk(count, n, ch, &pieces[ch].cnt, &pieces[ch].off);
      for (int r = 0; r < n; r++) pieces[ch].outs.push_back(madd(c.recv(r), pieces[ch].off * ts));
    }
    return reduceHostPieces(c, pieces);
  }
  const size_t nred = fx_nredslices(count, n, (size_t)g->nslices, (size_t)g->nredslices, (size_t)g->redslicesize);
  SliceList descs;
  if (g->algo == FX_ALGO_RING && g->op != flagcxAvg) {  // a mean is not a chain of two-input means
    // reduce-scatter: step i, rank r reduces chunk (r-i-1)%n: partial from the
    // previous rank (its sendbuff at step 0, its recvbuff afterwards) + own data.
    for (int i = 0; i < n - 1; i++) {
      for (int r = 0; r < n; r++) {
        const int prev = mod(r - 1, n), rx = mod(r - i - 1, n);
        size_t ccnt, coff;
        fx_split(count, n, rx, &ccnt, &coff);
        const void *partial = (i == 0) ? c.send(prev) : (const void *)c.recv(prev);
        flagcxResult_t rc = forPieces(g, ccnt, coff, nred, [&](size_t off, size_t, size_t cnt) {
          if (cnt == 0) return flagcxSuccess;
          fxSliceDesc d;
          memset(&d, 0, sizeof(d));
          d.in[0] = cadd(partial, off * ts);
          d.in[1] = cadd(c.send(r), off * ts);
          d.out = madd(c.recv(r), off * ts);
          d.count = cnt;
          descs.push_back(d);
          return flagcxSuccess;
        });
        if (rc != flagcxSuccess) return rc;
      }
      flagcxResult_t rc = R(fx_reduce_slices(descs.data(), descs.size(), 2, g->dtype, g->op, c.s));
      descs.clear();
      if (rc != flagcxSuccess) return rc;
    }
    // all-gather: step i, rank r receives chunk (r-i)%n from the previous rank.
    for (int i = 0; i < n - 1; i++) {
      for (int r = 0; r < n; r++) {
        const int prev = mod(r - 1, n), rx = mod(r - i, n);
        size_t ccnt, coff;
        fx_split(count, n, rx, &ccnt, &coff);
        if (ccnt) descs.push_back(copyDesc(cadd(c.recv(prev), coff * ts), madd(c.recv(r), coff * ts), ccnt * ts));
      }
      flagcxResult_t rc = R(fx_copy_slices(descs.data(), descs.size(), c.s));
      descs.clear();
      if (rc != flagcxSuccess) return rc;
    }
    return flagcxSuccess;
  }
  // direct, up to eight ranks: every piece is reduced k-way once and stored to
  // all n receive buffers by the same workgroup -- (k + n) * size bytes of
  // traffic instead of the (k + 1 + 2 (n - 1)) * size of reduce-then-copy.
  if (canBroadcast(c)) {
    BcastList bd;
    for (int ch = 0; ch < n; ch++) {
      size_t ccnt, coff;
      fx_split(count, n, ch, &ccnt, &coff);
      const int first = (g->order == FX_ORDER_RING) ? ch : 0;
      flagcxResult_t rc = forPieces(g, ccnt, coff, nred, [&](size_t off, size_t, size_t cnt) {
        if (cnt == 0) return flagcxSuccess;
        fxBcastDesc d;
        memset(&d, 0, sizeof(d));
        for (int j = 0; j < n; j++) d.in[j] = cadd(c.send(mod(first + j, n)), off * ts);
        for (int r = 0; r < n; r++) d.out[r] = madd(c.recv(r), off * ts);
        d.count = cnt;
        bd.push_back(d);
        return flagcxSuccess;
      });
      if (rc != flagcxSuccess) return rc;
    }
    return R(fx_reduce_bcast_slices(bd.data(), bd.size(), n, n, g->dtype, g->op, c.s));
  }
  // more ranks than a descriptor has slots: the runtime-k, runtime-n form of the
  // same one-read-n-stores launch.  Rank order is one launch over the whole
  // buffer; ring order starts chunk ch's fold at rank ch, one launch per chunk.
  PtrList ins;
  fx::SmallVec<void *, 16> outs;
  ins.resize((size_t)n);
  outs.resize((size_t)n);
  auto bcast = [&](size_t off, size_t cnt, int first) {
    for (int j = 0; j < n; j++) ins[j] = cadd(c.send(j), off * ts);
    for (int r = 0; r < n; r++) outs[r] = madd(c.recv(r), off * ts);
    return R(fx_reduce_bcast(outs.data(), n, ins.data(), n, cnt, g->dtype, g->op, first, c.s));
  };
  if (g->order != FX_ORDER_RING) return bcast(0, count, 0);
  if (n <= FX_MAX_INPUTS && recvsAlignedAlike(c)) {   // every chunk in one launch
    fx::SmallVec<fxChunk, 16> chunks;
    for (int ch = 0; ch < n; ch++) {
      size_t ccnt, coff;
      fx_split(count, n, ch, &ccnt, &coff);
      chunks.push_back(fxChunk{coff, coff, ccnt, ch, -1, -1});
    }
    for (int j = 0; j < n; j++) ins[j] = c.send(j);
    for (int r = 0; r < n; r++) outs[r] = c.recv(r);
    return R(fx_reduce_chunks(outs.data(), n, ins.data(), n, chunks.data(), n, g->dtype, g->op, c.s));
  }
  for (int ch = 0; ch < n; ch++) {
    size_t ccnt, coff;
    fx_split(count, n, ch, &ccnt, &coff);
    if (ccnt == 0) continue;
    const flagcxResult_t rc = bcast(coff, ccnt, ch);
    if (rc != flagcxSuccess) return rc;
  }
  return flagcxSuccess;
}

// Receive steps of tree rank a (uni_runner_impl.cc:1314-1326): the root takes
// ceil(log2 n); others ctz(a), clipped so that a + 2^i stays below n.
int treeSteps(int a, int n) {
  int total = 0;
  while ((1 << total) < n) total++;
  if (a == 0) return total;
  int st = __builtin_ctz((unsigned)a);
  if (st && n - a <= (1 << (st - 1))) {
    int rest = n - a - 1;
    for (st = 0; rest; rest >>= 1) st++;
  }
  return st;
}

flagcxResult_t runReduce(const Ctx &c) {
  Group *g = c.g;
  const int n = c.n, root = g->root;
  const size_t count = g->count, ts = c.ts;
  if (count == 0) return flagcxSuccess;
  if (g->order == FX_ORDER_HOST && n > 1) {  // the host path reduce-scatters, then gathers the chunks on the root
    std::vector<HostPiece> pieces(n);
    for (int ch = 0; ch < n; ch++) {
      pieces[ch].chunk = ch;
      hostChunk(count, n, ch, &pieces[ch].cnt, &pieces[ch].off);
      pieces[ch].outs.push_back(madd(c.recv(root), pieces[ch].off * ts));
    }
    return reduceHostPieces(c, pieces);
  }
  if (g->order != FX_ORDER_TREE || n == 1 || g->op == flagcxAvg) {
    PtrList in;
    in.resize((size_t)n);
    for (int j = 0; j < n; j++) in[j] = c.send(j);
    return R(fx_reduce_copy(c.recv(root), in.data(), n, count, g->dtype, g->op, 0, c.s));
  }
  // Tree order: round i, every tree rank a with more than i receive steps
  // computes partial(a) = partial(a + 2^i) (op) partial(a).  Up to eight ranks
  // that is one launch that keeps the partials in registers (in[a] = tree rank
  // a's data); beyond, partials live in a per-rank scratch row, one launch per
  // round, and the root's last round writes recvbuff.
  if (n <= FX_MAX_SLICE_INPUTS) {
    fxBcastDesc d;
    memset(&d, 0, sizeof(d));
    for (int a = 0; a < n; a++) d.in[a] = c.send(mod(a + root, n));
    d.out[0] = c.recv(root);
    d.count = count;
    return R(fx_reduce_ordered(&d, 1, n, 1, g->dtype, g->op, FX_FOLD_TREE, c.s));
  }
  flagcxResult_t rc = ensureScratch(g, (size_t)n * count * ts, c.s);
  if (rc != flagcxSuccess) return rc;
  const int total = treeSteps(0, n);
  auto rankOf = [&](int a) { return mod(a + root, n); };
  auto partial = [&](int a, int round) -> const void * {   // where tree rank a's partial is before `round`
    return (round == 0 || treeSteps(a, n) == 0) ? c.send(rankOf(a)) : madd(g->scratch, (size_t)a * count * ts);
  };
  SliceList descs;
  for (int i = 0; i < total; i++) {
    for (int a = 0; a < n; a++) {
      if (treeSteps(a, n) <= i) continue;
      fxSliceDesc d;
      memset(&d, 0, sizeof(d));
      d.in[0] = partial(a + (1 << i), i);   // received
      d.in[1] = partial(a, i);              // own
      d.out = (a == 0 && i == total - 1) ? c.recv(root) : madd(g->scratch, (size_t)a * count * ts);
      d.count = count;
      descs.push_back(d);
    }
    rc = R(fx_reduce_slices(descs.data(), descs.size(), 2, g->dtype, g->op, c.s));
    descs.clear();
    if (rc != flagcxSuccess) return rc;
  }
  return flagcxSuccess;
}

flagcxResult_t runReduceScatter(const Ctx &c) {
  Group *g = c.g;
  const int n = c.n;
  const size_t rcount = g->count, ts = c.ts;
  if (n == 1) {
    if (rcount && c.send(0) != c.recv(0)) {
      fxSliceDesc d = copyDesc(c.send(0), c.recv(0), rcount * ts);
      return R(fx_copy_slices(&d, 1, c.s));
    }
    return flagcxSuccess;
  }
  if (g->order == FX_ORDER_HOST) {  // chunk r = [r * recvcount, (r+1) * recvcount) ends on rank r
    std::vector<HostPiece> pieces(n);
    for (int r = 0; r < n; r++) {
      pieces[r].chunk = r;
      pieces[r].off = (size_t)r * rcount;
      pieces[r].cnt = rcount;
      pieces[r].outs.push_back(c.recv(r));
    }
    return reduceHostPieces(c, pieces);
  }
  const size_t nred = fx_nredslices(rcount, n, (size_t)g->nslices, (size_t)g->nredslices, (size_t)g->redslicesize);
  SliceList descs;
  KwayRun run;
  if (g->algo == FX_ALGO_RING && g->op != flagcxAvg) {  // a mean is not a chain of two-input means
    // Per-rank scratch of n*recvcount elements holds the travelling partials.
    flagcxResult_t rc = ensureScratch(g, (size_t)n * n * rcount * ts, c.s);
    if (rc != flagcxSuccess) return rc;
    auto scratch = [&](int r) { return madd(g->scratch, (size_t)r * n * rcount * ts); };
    for (int i = 0; i < n - 1; i++) {
      for (int r = 0; r < n; r++) {
        const int prev = mod(r - 1, n), rx = mod(r - i - 2, n);
        const void *partial = (i == 0) ? c.send(prev) : (const void *)scratch(prev);
        rc = forPieces(g, rcount, (size_t)rx * rcount, nred, [&](size_t off, size_t inSlice, size_t cnt) {
          if (cnt == 0) return flagcxSuccess;
          fxSliceDesc d;
          memset(&d, 0, sizeof(d));
          d.in[0] = cadd(partial, off * ts);
          d.in[1] = cadd(c.send(r), off * ts);
          d.out = (i == n - 2) ? madd(c.recv(r), inSlice * ts) : madd(scratch(r), off * ts);
          d.count = cnt;
          descs.push_back(d);
          return flagcxSuccess;
        });
        if (rc != flagcxSuccess) return rc;
      }
      rc = R(fx_reduce_slices(descs.data(), descs.size(), 2, g->dtype, g->op, c.s));
      descs.clear();
      if (rc != flagcxSuccess) return rc;
    }
    return flagcxSuccess;
  }
  if (n > FX_MAX_SLICE_INPUTS && n <= FX_MAX_INPUTS) {   // chunk r of every send buffer onto rank r, all in one launch
    fx::SmallVec<fxChunk, 16> chunks;
    PtrList ins;
    fx::SmallVec<void *, 16> outs;
    for (int r = 0; r < n; r++) {
      chunks.push_back(fxChunk{(size_t)r * rcount, 0, rcount, (g->order == FX_ORDER_RING) ? mod(r + 1, n) : 0, -1, r});
      ins.push_back(c.send(r));
      outs.push_back(c.recv(r));
    }
    return R(fx_reduce_chunks(outs.data(), n, ins.data(), n, chunks.data(), n, g->dtype, g->op, c.s));
  }
  for (int r = 0; r < n; r++) {
    const int first = (g->order == FX_ORDER_RING) ? mod(r + 1, n) : 0;
    flagcxResult_t rc = forPieces(g, rcount, (size_t)r * rcount, nred, [&](size_t off, size_t inSlice, size_t cnt) {
      return kway(c, descs, run, off, cnt, madd(c.recv(r), inSlice * ts), first);
    });
    if (rc != flagcxSuccess) return rc;
  }
  return flushKway(c, descs, run);
}

flagcxResult_t runAllGather(const Ctx &c) {
  const size_t bytes = c.g->count * c.ts;
  if (bytes == 0) return flagcxSuccess;
  if (canBroadcast(c)) {  // each rank's block is read once and stored to every receive buffer
    BcastList bd;
    bd.resize((size_t)c.n);
    for (int r = 0; r < c.n; r++) {
      memset(&bd[r], 0, sizeof(fxBcastDesc));
      bd[r].in[0] = c.send(r);
      for (int j = 0; j < c.n; j++) bd[r].out[j] = madd(c.recv(j), (size_t)r * bytes);
      bd[r].count = bytes;
    }
    return R(fx_reduce_bcast_slices(bd.data(), bd.size(), 1, c.n, 0, -1, c.s));
  }
  if (c.n <= FX_MAX_INPUTS && recvsAlignedAlike(c)) {   // rank q's block into slot q of every rank, all in one launch
    fx::SmallVec<fxChunk, 16> chunks;
    PtrList ins;
    fx::SmallVec<void *, 16> outs;
    for (int q = 0; q < c.n; q++) {
      chunks.push_back(fxChunk{0, (size_t)q * bytes, bytes, 0, q, -1});
      ins.push_back(c.send(q));
      outs.push_back(c.recv(q));
    }
    return R(fx_reduce_chunks(outs.data(), c.n, ins.data(), c.n, chunks.data(), c.n, 0, -1, c.s));
  }
  SliceList descs;
  for (int r = 0; r < c.n; r++)
    for (int j = 0; j < c.n; j++) {
      void *dst = madd(c.recv(j), (size_t)r * bytes);
      if (dst != c.send(r)) descs.push_back(copyDesc(c.send(r), dst, bytes));
    }
  return R(fx_copy_slices(descs.data(), descs.size(), c.s));
}

// When no receive segment overlaps any send segment, every segment goes
// straight from the sender's buffer to the receiver's: one batched launch.
// Otherwise (in-place use) every rank's segments are packed into contiguous
// staging slots and unpacked from the peers' slots: two launches.
flagcxResult_t runAlltoAllv(const Ctx &c) {
  Group *g = c.g;
  const int n = c.n;
  const size_t ts = c.ts;
  std::vector<size_t> base(n + 1, 0);
  struct Range {
    uintptr_t lo, hi;
  };
  std::vector<Range> sendR, recvR;
  for (int r = 0; r < n; r++) {
    size_t tot = 0;
    for (int i = 0; i < n; i++) {
      const size_t cnt = g->posts[r].sendcounts[i];
      if (cnt != g->posts[i].recvcounts[r]) return flagcxInvalidArgument;
      tot += cnt;
      if (cnt && (!c.send(r) || !c.recv(i))) return flagcxInvalidArgument;
      if (cnt) {
        const uintptr_t s = (uintptr_t)c.send(r) + g->posts[r].sdispls[i] * ts;
        const uintptr_t d = (uintptr_t)c.recv(i) + g->posts[i].rdispls[r] * ts;
        sendR.push_back({s, s + cnt * ts});
        recvR.push_back({d, d + cnt * ts});
      }
    }
    base[r + 1] = base[r] + ((tot * ts + 255) & ~(size_t)255);
  }
  if (base[n] == 0) return flagcxSuccess;
  // Does any receive segment overlap any send segment?  First by rank: the span of all a rank sends against the
  // span of all a rank receives (n * n pairs instead of one per pair of segments); only where two spans meet, by
  // segment, in address order.
  bool overlap = false;
  {
    std::vector<Range> sendSpan(n, Range{UINTPTR_MAX, 0}), recvSpan(n, Range{UINTPTR_MAX, 0});
    size_t at = 0;
    for (int r = 0; r < n; r++)
      for (int i = 0; i < n; i++) {
        if (!g->posts[r].sendcounts[i]) continue;
        const Range &sr = sendR[at], &rr = recvR[at];   // pushed pairwise above: rank r's segment for rank i, and where it lands
        at++;
        sendSpan[r].lo = std::min(sendSpan[r].lo, sr.lo);
        sendSpan[r].hi = std::max(sendSpan[r].hi, sr.hi);
        recvSpan[i].lo = std::min(recvSpan[i].lo, rr.lo);
        recvSpan[i].hi = std::max(recvSpan[i].hi, rr.hi);
      }
    bool spansMeet = false;
    for (int r = 0; r < n && !spansMeet; r++)
      for (int i = 0; i < n && !spansMeet; i++)
        spansMeet = recvSpan[i].lo < sendSpan[r].hi && sendSpan[r].lo < recvSpan[i].hi;
    if (spansMeet) {
      struct Tagged {
        uintptr_t lo, hi;
        int recv;
      };
      std::vector<Tagged> all;
      all.reserve(sendR.size() + recvR.size());
      for (const Range &x : sendR) all.push_back(Tagged{x.lo, x.hi, 0});
      for (const Range &x : recvR) all.push_back(Tagged{x.lo, x.hi, 1});
      std::sort(all.begin(), all.end(), [](const Tagged &a, const Tagged &b) { return a.lo < b.lo; });
      uintptr_t reach[2] = {0, 0};   // how far the segments of either kind seen so far extend
      for (const Tagged &x : all) {
        if (reach[1 - x.recv] > x.lo) {
          overlap = true;
          break;
        }
        reach[x.recv] = std::max(reach[x.recv], x.hi);
      }
    }
  }
  if (!overlap) {
    SliceList direct;
    for (size_t a = 0; a < recvR.size(); a++)
      direct.push_back(copyDesc((const void *)sendR[a].lo, (void *)recvR[a].lo, recvR[a].hi - recvR[a].lo));
    return R(fx_copy_slices(direct.data(), direct.size(), c.s));
  }
  flagcxResult_t rc = ensureScratch(g, base[n], c.s);
  if (rc != flagcxSuccess) return rc;
  SliceList pack, unpack;
  for (int r = 0; r < n; r++) {
    size_t slot = 0;
    for (int i = 0; i < n; i++) {
      const size_t cnt = g->posts[r].sendcounts[i];
      if (cnt) {
        void *stage = madd(g->scratch, base[r] + slot * ts);
        pack.push_back(copyDesc(cadd(c.send(r), g->posts[r].sdispls[i] * ts), stage, cnt * ts));
        unpack.push_back(copyDesc(stage, madd(c.recv(i), g->posts[i].rdispls[r] * ts), cnt * ts));
      }
      slot += cnt;
    }
  }
  rc = R(fx_copy_slices(pack.data(), pack.size(), c.s));
  if (rc != flagcxSuccess) return rc;
  return R(fx_copy_slices(unpack.data(), unpack.size(), c.s));
}

// gather / scatter / broadcast / alltoall move bytes only: one batched copy
// launch each (the reference builds them from grouped send/recv pairs,
// flagcx/adaptor/ccl/rccl_adaptor.cc:126-184,222-246).
flagcxResult_t runGather(const Ctx &c) {
  const size_t bytes = c.g->count * c.ts;
  SliceList d;
  for (int r = 0; r < c.n && bytes; r++) {
    void *dst = madd(c.recv(c.g->root), (size_t)r * bytes);
    if (dst != c.send(r)) d.push_back(copyDesc(c.send(r), dst, bytes));
  }
  return R(fx_copy_slices(d.data(), d.size(), c.s));
}

flagcxResult_t runScatter(const Ctx &c) {
  const size_t bytes = c.g->count * c.ts;
  SliceList d;
  for (int r = 0; r < c.n && bytes; r++) {
    const void *src = cadd(c.send(c.g->root), (size_t)r * bytes);
    if (src != c.recv(r)) d.push_back(copyDesc(src, c.recv(r), bytes));
  }
  return R(fx_copy_slices(d.data(), d.size(), c.s));
}

flagcxResult_t runBroadcast(const Ctx &c) {
  const size_t bytes = c.g->count * c.ts;
  if (bytes && canBroadcast(c)) {
    fxBcastDesc b;
    memset(&b, 0, sizeof(b));
    b.in[0] = c.send(c.g->root);
    for (int r = 0; r < c.n; r++) b.out[r] = c.recv(r);
    b.count = bytes;
    return R(fx_reduce_bcast_slices(&b, 1, 1, c.n, 0, -1, c.s));
  }
  if (bytes && c.n <= FX_MAX_INPUTS) {   // more ranks: the run-time form of the same one-read-n-stores copy
    fx::SmallVec<void *, 16> outs;
    for (int r = 0; r < c.n; r++) outs.push_back(c.recv(r));
    const void *src = c.send(c.g->root);
    return R(fx_reduce_bcast(outs.data(), c.n, &src, 1, bytes, 0, -1, 0, c.s));
  }
  SliceList d;
  for (int r = 0; r < c.n && bytes; r++)
    if (c.recv(r) != c.send(c.g->root)) d.push_back(copyDesc(c.send(c.g->root), c.recv(r), bytes));
  return R(fx_copy_slices(d.data(), d.size(), c.s));
}

// Block i of rank r's sendbuff becomes block r of rank i's recvbuff.  The
// one-launch kernel reads and writes concurrently, so if ANY rank's send buffer
// meets ANY rank's receive buffer (a rank in place, rank a receiving into what
// rank b sends, a partial overlap) the blocks go through staging first.
flagcxResult_t runAlltoAll(const Ctx &c) {
  Group *g = c.g;
  const int n = c.n;
  const size_t bytes = g->count * c.ts;
  if (bytes == 0) return flagcxSuccess;
  bool inplace = false;
  const size_t span = (size_t)n * bytes;
  for (int r = 0; r < n && !inplace; r++)
    for (int i = 0; i < n && !inplace; i++) {
      const uintptr_t s = (uintptr_t)c.send(r), d = (uintptr_t)c.recv(i);
      inplace = s < d + span && d < s + span;
    }
  SliceList d;
  if (!inplace) {   // every block straight from its sender to its receiver, one launch
    PtrList sends;
    fx::SmallVec<void *, 16> recvs;
    for (int r = 0; r < n; r++) {
      sends.push_back(c.send(r));
      recvs.push_back(c.recv(r));
    }
    return R(fx_alltoall(recvs.data(), sends.data(), n, bytes, c.s));
  }
  flagcxResult_t rc = ensureScratch(g, (size_t)n * n * bytes, c.s);
  if (rc != flagcxSuccess) return rc;
  for (int r = 0; r < n; r++)
    d.push_back(copyDesc(c.send(r), madd(g->scratch, (size_t)r * n * bytes), (size_t)n * bytes));
  rc = R(fx_copy_slices(d.data(), d.size(), c.s));
  if (rc != flagcxSuccess) return rc;
  PtrList staged;
  fx::SmallVec<void *, 16> recvs;
  for (int r = 0; r < n; r++) {
    staged.push_back(cadd(g->scratch, (size_t)r * n * bytes));
    recvs.push_back(c.recv(r));
  }
  return R(fx_alltoall(recvs.data(), staged.data(), n, bytes, c.s));
}

flagcxResult_t runCustomAllReduce(const Ctx &c) {
  Group *g = c.g;
  if (g->count == 0) return flagcxSuccess;
  {  // stage every rank's sendbuff into its window unless it already is the window
    SliceList stage;
    for (int r = 0; r < c.n; r++)
      if (c.send(r) != g->windows[r]) stage.push_back(copyDesc(c.send(r), g->windows[r], g->count * c.ts));
    if (!stage.empty()) {
      const flagcxResult_t rc = R(fx_copy_slices(stage.data(), stage.size(), c.s));
      if (rc != flagcxSuccess) return rc;
    }
  }
  if (canBroadcast(c)) {  // every rank's result is the same fold of the windows: compute it once
    fxBcastDesc b;
    memset(&b, 0, sizeof(b));
    for (int j = 0; j < c.n; j++) b.in[j] = g->windows[j];
    for (int r = 0; r < c.n; r++) b.out[r] = c.recv(r);
    b.count = g->count;
    return R(fx_reduce_bcast_slices(&b, 1, c.n, c.n, g->dtype, g->op, c.s));
  }
  fx::SmallVec<void *, 16> outs;
  outs.resize((size_t)c.n);
  for (int r = 0; r < c.n; r++) outs[r] = c.recv(r);
  return R(fx_reduce_bcast(outs.data(), c.n, (const void *const *)g->windows.data(), c.n, g->count, g->dtype, g->op, 0,
                           c.s));
}

void resetPending(Group *g) {
  g->kind = kNone;
  g->nposted = 0;
  for (auto &p : g->posts) p = Post();
}

// Drop the pending collective because of a caller error; ranks asleep in a
// rendezvous get the same result.
void abandonPending(Group *g, flagcxResult_t why) {
  resetPending(g);
  g->lastResult = why;
  g->launched++;
  g->cv.notify_all();
}

// Record one rank's call; the last rank to arrive launches the collective.
flagcxResult_t postAndMaybeRun(flagcxComm_t comm, Kind kind, const void *send, void *recv, size_t count, int dtype,
                               int op, int root, flagcxStream_t stream, const size_t *sc = nullptr,
                               const size_t *sd = nullptr, const size_t *rc_ = nullptr, const size_t *rd = nullptr);

}  // namespace

struct flagcxComm {
  Group *g;
  int rank;
  uint64_t joined = 0;   // how many collectives the group had launched when this rank's last post was accepted
};

namespace {

flagcxResult_t postAndMaybeRunImpl(flagcxComm_t comm, Kind kind, const void *send, void *recv, size_t count, int dtype,
                                   int op, int root, flagcxStream_t stream, const size_t *sc, const size_t *sd,
                                   const size_t *rc_, const size_t *rd);

flagcxResult_t postAndMaybeRun(flagcxComm_t comm, Kind kind, const void *send, void *recv, size_t count, int dtype,
                               int op, int root, flagcxStream_t stream, const size_t *sc, const size_t *sd,
                               const size_t *rc_, const size_t *rd) {
  return R(fx::guarded([&]() -> int {
    return postAndMaybeRunImpl(comm, kind, send, recv, count, dtype, op, root, stream, sc, sd, rc_, rd);
  }));
}

flagcxResult_t postAndMaybeRunImpl(flagcxComm_t comm, Kind kind, const void *send, void *recv, size_t count, int dtype,
                                   int op, int root, flagcxStream_t stream, const size_t *sc, const size_t *sd,
                                   const size_t *rc_, const size_t *rd) {
  if (!comm || !comm->g || !stream) return flagcxInvalidArgument;
  Group *g = comm->g;
  const int rank = comm->rank;
  // Rendezvous mode: this rank's thread stays in the call until the launch, so
  // its stream stands where it will stand then.  Every rank marks the spot
  // itself, before queueing for the lock, instead of leaving all the marks to
  // the last rank in.
  // A stream with nothing left to do needs no mark at all: nothing can be added
  // to it while its rank's thread is in here.
  bool marked = false, idle = false;
  if (g->n > 1 && g->sync.load(std::memory_order_relaxed) == FX_SYNC_RENDEZVOUS) {
    if (isCapturing(stream->base)) return flagcxInvalidUsage;   // see isCapturing
    idle = hipStreamQuery(stream->base) == hipSuccess;
    if (!idle) {
      (void)hipGetLastError();   // "not ready" is an answer, not an error to leave behind for the caller's next check
      marked = hipEventRecord(g->ready[rank], stream->base) == hipSuccess;
    }
  }
  std::unique_lock<std::mutex> lock(g->mu);
  if (g->nposted == 0) {
    g->kind = kind;
    g->count = count;
    g->dtype = dtype;
    g->op = op;
    g->root = root;
  } else if (g->kind != kind || g->count != count || g->dtype != dtype || g->op != op || g->root != root) {
    abandonPending(g, flagcxInvalidArgument);  // ranks disagree on the collective
    return flagcxInvalidArgument;
  }
  Post &p = g->posts[rank];
  if (p.posted) {
    abandonPending(g, flagcxInvalidUsage);  // same rank called twice before the others arrived
    return flagcxInvalidUsage;
  }
  p.posted = true;
  p.send = send;
  p.recv = recv;
  p.stream = stream->base;
  p.marked = marked;
  p.idle = idle;
  comm->joined = g->launched;
  if (kind == kAlltoAllv) {
    p.sendcounts.assign(sc, sc + g->n);
    p.sdispls.assign(sd, sd + g->n);
    p.recvcounts.assign(rc_, rc_ + g->n);
    p.rdispls.assign(rd, rd + g->n);
  }
  if (++g->nposted < g->n) {
    if (g->sync != FX_SYNC_RENDEZVOUS) return flagcxSuccess;
    // Wait until the last rank has launched this collective.
    const uint64_t mine = g->launched;
    if (!g->cv.wait_for(lock, std::chrono::milliseconds(g->timeoutMs), [&] { return g->launched != mine; })) {
      resetPending(g);  // a rank never arrived: give up for everybody
      g->lastResult = flagcxInternalError;
      g->launched++;
      g->cv.notify_all();
      return flagcxInternalError;
    }
    // What this rank enqueues next comes after the collective: each woken rank
    // makes its own stream wait (the next collective cannot move the event before
    // this rank has posted again).
    const flagcxResult_t res = g->lastResult;
    const hipStream_t where = g->launchStream, own = stream->base;
    hipEvent_t done = g->done;
    lock.unlock();
    if (res == flagcxSuccess && where != own) {
      if (hipEventQuery(done) == hipSuccess) return res;   // already over: anything enqueued from now on is after it
      (void)hipGetLastError();                             // "not ready" is an answer, not an error
      if (hipStreamWaitEvent(own, done, 0) != hipSuccess) return flagcxUnhandledDeviceError;
    }
    return res;
  }

  // Last rank in: order the launch after everything the other ranks' streams
  // hold right now (their calls are already made, so that covers all they
  // enqueued before calling).  One event per distinct foreign stream.
  Ctx c{g, p.stream, g->n, fx_dtype_size(dtype)};
  flagcxResult_t res = flagcxSuccess;
  for (int r = 0; r < g->n && res == flagcxSuccess; r++) {
    hipStream_t s = g->posts[r].stream;
    if (s == c.s || g->posts[r].idle) continue;
    if (g->posts[r].marked) {   // the rank's thread has recorded its own event
      if (hipStreamWaitEvent(c.s, g->ready[r], 0) != hipSuccess) res = flagcxUnhandledDeviceError;
      continue;
    }
    bool seen = false;
    for (int q = 0; q < r && !seen; q++) seen = (g->posts[q].stream == s);
    if (seen) continue;
    if (hipEventRecord(g->ready[r], s) != hipSuccess || hipStreamWaitEvent(c.s, g->ready[r], 0) != hipSuccess)
      res = flagcxUnhandledDeviceError;
  }
  // The reference device kernel's own arithmetic for the 16-bit types, where asked for and where the schedule is
  // that kernel's (every element folded over the ranks 0, 1, .., n-1 in one pass).
  if (g->arith == FX_ARITH_ELEMENT && (dtype == flagcxFloat16 || dtype == flagcxBfloat16) &&
      (op == flagcxSum || op == flagcxMax || op == flagcxMin) &&
      (kind == kCustomAllReduce ||
       ((kind == kAllReduce || kind == kReduce || kind == kReduceScatter) && g->algo == FX_ALGO_DIRECT &&
        g->order == FX_ORDER_RANK)))
    g->op = op | FX_OP_ELEMENT_FOLD;
  if (res == flagcxSuccess) {
    switch (kind) {
      case kAllReduce: res = runAllReduce(c); break;
      case kReduce: res = runReduce(c); break;
      case kReduceScatter: res = runReduceScatter(c); break;
      case kAllGather: res = runAllGather(c); break;
      case kAlltoAllv: res = runAlltoAllv(c); break;
      case kCustomAllReduce: res = runCustomAllReduce(c); break;
      case kGather: res = runGather(c); break;
      case kScatter: res = runScatter(c); break;
      case kBroadcast: res = runBroadcast(c); break;
      case kAlltoAll: res = runAlltoAll(c); break;
      case kBarrier: break;  // the event waits around this switch are the barrier
      default: res = flagcxInternalError;
    }
  }
  if (res == flagcxSuccess) {
    bool others = false;
    for (int r = 0; r < g->n; r++) others = others || (g->posts[r].stream != c.s);
    if (others) {
      if (hipEventRecord(g->done, c.s) != hipSuccess) res = flagcxUnhandledDeviceError;
      // group mode: the other ranks' calls have returned, so their streams are made to wait here;
      // rendezvous mode: every rank does that for itself when it wakes
      for (int r = 0; r < g->n && res == flagcxSuccess && g->sync != FX_SYNC_RENDEZVOUS; r++) {
        hipStream_t s = g->posts[r].stream;
        bool seen = (s == c.s);
        for (int q = 0; q < r && !seen; q++) seen = (g->posts[q].stream == s);
        if (!seen && hipStreamWaitEvent(s, g->done, 0) != hipSuccess) res = flagcxUnhandledDeviceError;
      }
    }
  }
  g->launchStream = c.s;
  resetPending(g);
  g->lastResult = res;
  g->launched++;
  g->cv.notify_all();
  return res;
}

// Argument screening shared by the reducing collectives: same results as the
// kernel layer (unsupported-but-known -> flagcxNotSupported).
flagcxResult_t screenReduce(int dtype, int op) {
  if (dtype < 0 || dtype >= flagcxNumTypes || op < 0 || op >= flagcxNumRedOps) return flagcxInvalidArgument;
  return flagcxSuccess;
}

std::mutex gRegistryMu;
std::map<std::string, Group *> gRegistry;  // groups still waiting for ranks to join, by id

void freeGroupResources(Group *g) {
  for (auto e : g->ready)
    if (e) (void)hipEventDestroy(e);
  if (g->done) (void)hipEventDestroy(g->done);
  for (auto e : g->markPool) (void)hipEventDestroy(e);
  for (auto &m : g->p2pMatched)
    if (m.second.after) (void)hipEventDestroy(m.second.after);
  for (const PendingP2p &o : g->p2p)
    if (o.mark) (void)hipEventDestroy(o.mark);
  if (g->p2pBefore) (void)hipEventDestroy(g->p2pBefore);
  if (g->p2pAfter) (void)hipEventDestroy(g->p2pAfter);
  if (g->scratch) (void)hipFree(g->scratch);
  for (void *b : g->outgrown) (void)hipFree(b);
  delete g;
}

flagcxResult_t newGroup(int nranks, Group **out) {
  Group *g = new (std::nothrow) Group();
  if (!g) return flagcxSystemError;
  g->n = nranks;
  try {
    g->posts.resize(nranks);
    g->ready.assign(nranks, nullptr);
    g->taken.assign(nranks, 0);
  } catch (...) {
    delete g;
    throw;
  }
  bool ok = hipGetDevice(&g->device) == hipSuccess;
  ok = ok && hipEventCreateWithFlags(&g->done, hipEventDisableTiming) == hipSuccess;
  for (int r = 0; r < nranks && ok; r++)
    ok = hipEventCreateWithFlags(&g->ready[r], hipEventDisableTiming) == hipSuccess;
  if (!ok) {
    for (auto e : g->ready)
      if (e) (void)hipEventDestroy(e);
    if (g->done) (void)hipEventDestroy(g->done);
    delete g;
    return flagcxUnhandledDeviceError;
  }
  // same knobs, same names, same defaults as the reference's uniRunner
  g->nslices = envParam("FLAGCX_UNIRUNNER_NSLICES", 1);
  g->nredslices = envParam("FLAGCX_UNIRUNNER_NREDSLICES", 0);
  g->redslicesize = envParam("FLAGCX_UNIRUNNER_REDSLICESIZE", 65536);
  if (g->nslices < 1) g->nslices = 1;
  if (g->nredslices < 0) g->nredslices = 0;
  if (g->redslicesize < 0) g->redslicesize = 0;
  const char *arith = getenv("FX_SIM_ARITH");
  if (arith && !strcmp(arith, "element")) g->arith = FX_ARITH_ELEMENT;
  const char *sync = getenv("FX_SIM_SYNC");
  if (sync && !strcmp(sync, "rendezvous")) g->sync = FX_SYNC_RENDEZVOUS;
  g->timeoutMs = envParam("FX_SIM_RENDEZVOUS_TIMEOUT_MS", 30000);
  if (g->timeoutMs < 1) g->timeoutMs = 1;
  const long long reserve = envParam("FX_SIM_SCRATCH_BYTES", 0);
  if (reserve > 0 && ensureScratch(g, (size_t)reserve, nullptr) != flagcxSuccess) {
    freeGroupResources(g);
    return flagcxUnhandledDeviceError;
  }
  *out = g;
  return flagcxSuccess;
}

void freeGroup(Group *g) {
  (void)hipDeviceSynchronize();
  freeGroupResources(g);
}

// Group brackets are per host thread (the CCL adaptor's groupStart / groupEnd
// carry no communicator).  In rendezvous mode a send or recv made inside a
// bracket must not sleep until its partner arrives -- every rank's thread would
// sit in its first call and none would reach its second -- so it is written
// down, and the outermost flagcxGroupEnd of the thread posts the bracket's
// halves and then waits for their partners: where the reference issues grouped
// operations too (flagcx/flagcx.cc group semantics; rccl_adaptor.cc:322-332
// forwards the bracket to the vendor library).
struct DeferredP2p {
  Group *g;
  uint64_t id;
  hipStream_t stream;
};
// Rendezvous mode: a send or recv made inside a bracket is only written down;
// the outermost flagcxGroupEnd of the thread posts them all, then waits for the
// partners of those that found none waiting.
struct QueuedP2p {
  flagcxComm_t comm;
  bool isSend;
  const void *sbuf;
  void *rbuf;
  size_t count;
  int dtype, peer;
  flagcxStream_t stream;
};
thread_local int tGroupDepth = 0;
thread_local bool tClosingBracket = false;
thread_local std::vector<DeferredP2p> tDeferred;
thread_local std::vector<QueuedP2p> tQueued;

// Copies of pairs that were matched inside a bracket with both halves on one
// stream (ranks posted one after another by one thread): they leave as one
// launch per stream when the outermost bracket closes, which is where the
// reference issues grouped operations too.  Not in rendezvous mode, where the
// other half's thread is told "done" at the match and may enqueue behind it.
struct BatchedCopies {
  hipStream_t stream;
  std::vector<fxSliceDesc> copies;
};
thread_local std::vector<BatchedCopies> tBatched;

flagcxResult_t flushBatched() {
  std::vector<BatchedCopies> mine;
  mine.swap(tBatched);
  flagcxResult_t first = flagcxSuccess;
  for (BatchedCopies &b : mine) {
    const flagcxResult_t rc = R(fx_copy_slices(b.copies.data(), b.copies.size(), b.stream));
    if (first == flagcxSuccess) first = rc;
  }
  return first;
}

// Wait until the partner of pending half `id` has made its call (it enqueues the
// copy) and hand back its result, with this rank's stream ordered after the
// copy unless that is over already; on time-out the half is withdrawn.  Called
// with g->mu held; returns with it released.
flagcxResult_t awaitPartner(Group *g, std::unique_lock<std::mutex> &lock, uint64_t id, hipStream_t own) {
  const bool matched = g->cv.wait_for(lock, std::chrono::milliseconds(g->timeoutMs),
                                      [&] { return g->p2pMatched.count(id) != 0; });
  if (!matched) {  // the partner never came: withdraw this half
    for (size_t i = 0; i < g->p2p.size(); i++)
      if (g->p2p[i].id == id) {
        if (g->p2p[i].mark) g->markPool.push_back(g->p2p[i].mark);
        g->p2p.erase(g->p2p.begin() + (long)i);
        break;
      }
    lock.unlock();
    return flagcxInternalError;
  }
  const P2pOutcome out = g->p2pMatched[id];
  g->p2pMatched.erase(id);
  lock.unlock();
  flagcxResult_t res = out.res;
  if (out.after) {
    if (res == flagcxSuccess && out.where != own) {
      if (hipEventQuery(out.after) != hipSuccess) {   // not over yet: what this rank enqueues next comes after the copy
        (void)hipGetLastError();                      // "not ready" is an answer, not an error
        if (hipStreamWaitEvent(own, out.after, 0) != hipSuccess) res = flagcxUnhandledDeviceError;
      }
    }
    lock.lock();
    g->markPool.push_back(out.after);   // the wait on it is enqueued (or not needed): the event may be recorded anew
    lock.unlock();
  }
  return res;
}

// send / recv between simulated ranks: the later of the two calls performs the
// copy on its own stream.  If the other side posted on another stream, the copy
// first waits for all that stream holds at that moment (as a collective's
// launch waits for the other ranks' streams: later than the post itself, which
// is safe -- a stream can only be waiting for events recorded before this call)
// and that stream then waits for the copy.
flagcxResult_t postP2pImpl(flagcxComm_t comm, bool isSend, const void *sbuf, void *rbuf, size_t count, int dtype,
                           int peer, flagcxStream_t stream);

flagcxResult_t postP2p(flagcxComm_t comm, bool isSend, const void *sbuf, void *rbuf, size_t count, int dtype, int peer,
                       flagcxStream_t stream) {
  return R(fx::guarded([&]() -> int { return postP2pImpl(comm, isSend, sbuf, rbuf, count, dtype, peer, stream); }));
}

flagcxResult_t postP2pImpl(flagcxComm_t comm, bool isSend, const void *sbuf, void *rbuf, size_t count, int dtype,
                           int peer, flagcxStream_t stream) {
  if (!comm || !comm->g || !stream) return flagcxInvalidArgument;
  Group *g = comm->g;
  const size_t ts = fx_dtype_size(dtype);
  if (ts == 0 || peer < 0 || peer >= g->n) return flagcxInvalidArgument;
  if (count && !(isSend ? sbuf : (const void *)rbuf)) return flagcxInvalidArgument;
  const bool rendezvous = g->sync.load(std::memory_order_relaxed) == FX_SYNC_RENDEZVOUS;
  if (rendezvous && isCapturing(stream->base)) return flagcxInvalidUsage;   // see isCapturing
  if (rendezvous && tGroupDepth > 0 && !tClosingBracket) {
    tQueued.push_back(QueuedP2p{comm, isSend, sbuf, rbuf, count, dtype, peer, stream});
    return flagcxSuccess;
  }
  const int src = isSend ? comm->rank : peer, dst = isSend ? peer : comm->rank;
  const size_t bytes = count * ts;
  hipStream_t s = stream->base;
  std::unique_lock<std::mutex> lock(g->mu);
  for (size_t i = 0; i < g->p2p.size(); i++) {
    PendingP2p &o = g->p2p[i];
    if (o.isSend == isSend || o.src != src || o.dst != dst) continue;
    flagcxResult_t res = flagcxSuccess;
    hipEvent_t behind = nullptr;   // rendezvous mode, two streams: recorded behind the copy for the sleeping partner
    if (o.bytes != bytes) {
      res = flagcxInvalidArgument;  // the two sides disagree on the message size
    } else if (bytes) {
      fxSliceDesc d = copyDesc(isSend ? sbuf : o.sbuf, isSend ? o.rbuf : rbuf, bytes);
      if (o.stream == s && tGroupDepth > 0 && !rendezvous) {
        size_t b = 0;
        while (b < tBatched.size() && tBatched[b].stream != s) b++;
        if (b == tBatched.size()) tBatched.push_back(BatchedCopies{s, {}});
        tBatched[b].copies.push_back(d);
      } else if (o.stream == s) {
        res = R(fx_copy_slices(&d, 1, s));
      } else if (rendezvous) {
        // The other half's thread is inside its call (or its flagcxGroupEnd) until we are done: its stream stands
        // still.  An idle one needs no waiting for, a busy one carries its owner's mark; and the owner makes
        // its own stream wait for the copy when it wakes, through the event recorded behind the copy (`behind`).
        if (o.marked) {
          if (hipStreamWaitEvent(s, o.mark, 0) != hipSuccess) res = flagcxUnhandledDeviceError;
        } else if (!o.idle) {   // posted before the group was switched to this mode: mark its stream from here
          if ((!g->p2pBefore && hipEventCreateWithFlags(&g->p2pBefore, hipEventDisableTiming) != hipSuccess) ||
              hipEventRecord(g->p2pBefore, o.stream) != hipSuccess || hipStreamWaitEvent(s, g->p2pBefore, 0) != hipSuccess)
            res = flagcxUnhandledDeviceError;
        }
        if (res == flagcxSuccess) res = R(fx_copy_slices(&d, 1, s));
        if (res == flagcxSuccess) {
          if (!g->markPool.empty()) {
            behind = g->markPool.back();
            g->markPool.pop_back();
          } else if (hipEventCreateWithFlags(&behind, hipEventDisableTiming) != hipSuccess) {
            behind = nullptr;
            res = flagcxUnhandledDeviceError;
          }
          if (behind && hipEventRecord(behind, s) != hipSuccess) {
            g->markPool.push_back(behind);
            behind = nullptr;
            res = flagcxUnhandledDeviceError;
          }
        }
      } else {
        if ((!g->p2pBefore && hipEventCreateWithFlags(&g->p2pBefore, hipEventDisableTiming) != hipSuccess) ||
            (!g->p2pAfter && hipEventCreateWithFlags(&g->p2pAfter, hipEventDisableTiming) != hipSuccess) ||
            hipEventRecord(g->p2pBefore, o.stream) != hipSuccess || hipStreamWaitEvent(s, g->p2pBefore, 0) != hipSuccess)
          res = flagcxUnhandledDeviceError;
        if (res == flagcxSuccess) res = R(fx_copy_slices(&d, 1, s));
        if (res == flagcxSuccess &&
            (hipEventRecord(g->p2pAfter, s) != hipSuccess || hipStreamWaitEvent(o.stream, g->p2pAfter, 0) != hipSuccess))
          res = flagcxUnhandledDeviceError;
      }
    }
    if (rendezvous) {
      g->p2pMatched[o.id] = P2pOutcome{res, s, behind};
      g->cv.notify_all();
    }
    if (o.mark) g->markPool.push_back(o.mark);   // the wait on it is enqueued: the event may be recorded anew
    g->p2p.erase(g->p2p.begin() + (long)i);
    return res;
  }
  // No partner yet.  In rendezvous mode this thread now stays inside the library until one comes, so the stream's
  // state is final: idle, or marked here for the partner to wait on.
  bool idle = false, marked = false;
  hipEvent_t mark = nullptr;
  if (rendezvous && bytes) {
    idle = hipStreamQuery(s) == hipSuccess;
    if (!idle) {
      (void)hipGetLastError();   // "not ready" is an answer, not an error
      if (!g->markPool.empty()) {
        mark = g->markPool.back();
        g->markPool.pop_back();
      } else if (hipEventCreateWithFlags(&mark, hipEventDisableTiming) != hipSuccess) {
        return flagcxUnhandledDeviceError;
      }
      marked = hipEventRecord(mark, s) == hipSuccess;
      if (!marked) {
        g->markPool.push_back(mark);
        return flagcxUnhandledDeviceError;
      }
    }
  }
  g->p2p.push_back(PendingP2p{isSend, src, dst, sbuf, rbuf, bytes, s, g->nextP2pId++, comm->rank, idle, marked, mark});
  if (!rendezvous) return flagcxSuccess;
  const uint64_t id = g->p2p.back().id;
  if (tClosingBracket) {  // flagcxGroupEnd posts all of the bracket's halves before it waits for any
    tDeferred.push_back(DeferredP2p{g, id, s});
    return flagcxSuccess;
  }
  // Sleep until the partner has made its call and enqueued the copy.
  return awaitPartner(g, lock, id, s);
}

}  // namespace

extern "C" {
#pragma GCC visibility push(default)

flagcxResult_t fxSimCommInitAll(flagcxComm_t *comms, int nranks) {
  if (!comms || nranks < 1 || nranks > FX_MAX_INPUTS) return flagcxInvalidArgument;
  return R(fx::guarded([&]() -> int {
    Group *g = nullptr;
    flagcxResult_t rc = newGroup(nranks, &g);
    if (rc != flagcxSuccess) return rc;
    g->joined = g->alive = nranks;
    int made = 0;
    for (; made < nranks; made++)
      if (!(comms[made] = new (std::nothrow) flagcxComm{g, made})) break;
    if (made < nranks) {
      for (int r = 0; r < made; r++) delete comms[r];
      freeGroup(g);
      return flagcxSystemError;
    }
    return flagcxSuccess;
  }));
}

flagcxResult_t fxSimCommDestroyAll(flagcxComm_t *comms, int nranks) {
  if (!comms || nranks < 1 || !comms[0]) return flagcxInvalidArgument;
  Group *g = comms[0]->g;
  if (g->n != nranks) return flagcxInvalidArgument;
  for (int r = 0; r < nranks; r++) {
    delete comms[r];
    comms[r] = nullptr;
  }
  freeGroup(g);
  return flagcxSuccess;
}

flagcxResult_t fxSimCommInitRank(flagcxComm_t *comm, int nranks, const void *id, size_t idBytes, int rank) {
  if (!comm || !id || idBytes == 0 || nranks < 1 || nranks > FX_MAX_INPUTS || rank < 0 || rank >= nranks)
    return flagcxInvalidArgument;
  return R(fx::guarded([&]() -> int {
    std::lock_guard<std::mutex> lock(gRegistryMu);
    const std::string key((const char *)id, idBytes);
    flagcxComm *c = new flagcxComm{nullptr, rank};
    Group *g;
    auto it = gRegistry.find(key);
    if (it == gRegistry.end()) {
      flagcxResult_t rc = newGroup(nranks, &g);
      if (rc != flagcxSuccess) {
        delete c;
        return rc;
      }
      g->id = key;
      try {
        gRegistry[key] = g;
      } catch (...) {
        delete c;
        freeGroup(g);
        throw;
      }
    } else {
      g = it->second;
      if (g->n != nranks || g->taken[rank]) {  // a different group size, or this rank has joined already
        delete c;
        return flagcxInvalidArgument;
      }
    }
    g->taken[rank] = 1;
    g->joined++;
    g->alive++;
    if (g->joined == nranks) gRegistry.erase(key);  // complete: the id may be reused for a new group
    c->g = g;
    *comm = c;
    return flagcxSuccess;
  }));
}

flagcxResult_t fxSimCommDestroy(flagcxComm_t comm) {
  if (!comm || !comm->g) return flagcxInvalidArgument;
  Group *g = comm->g;
  bool last;
  {
    std::lock_guard<std::mutex> lock(gRegistryMu);
    last = (--g->alive == 0);
    if (last && !g->id.empty()) {
      auto it = gRegistry.find(g->id);
      if (it != gRegistry.end() && it->second == g) gRegistry.erase(it);
    }
  }
  delete comm;
  if (last) freeGroup(g);
  return flagcxSuccess;
}

flagcxResult_t flagcxGetVersion(int *version) {
  if (!version) return flagcxInvalidArgument;
  *version = FX_SIM_VERSION;
  return flagcxSuccess;
}

flagcxResult_t flagcxGetUniqueId(flagcxUniqueId_t uniqueId) {
  if (!uniqueId) return flagcxInvalidArgument;
  static std::atomic<uint64_t> counter{0};
  const uint64_t words[3] = {(uint64_t)std::chrono::steady_clock::now().time_since_epoch().count(), ++counter,
                             (uint64_t)(uintptr_t)&counter};
  memset(uniqueId->internal, 0, sizeof(uniqueId->internal));
  memcpy(uniqueId->internal, words, sizeof(words));
  return flagcxSuccess;
}

flagcxResult_t flagcxCommInitRank(flagcxComm_t *comm, int nranks, flagcxUniqueId_t commId, int rank) {
  if (!commId) return flagcxInvalidArgument;
  return fxSimCommInitRank(comm, nranks, commId->internal, sizeof(commId->internal), rank);
}

flagcxResult_t flagcxCommDestroy(flagcxComm_t comm) { return fxSimCommDestroy(comm); }

const char *flagcxGetErrorString(flagcxResult_t result) {
  switch (result) {
    case flagcxSuccess: return "no error";
    case flagcxUnhandledDeviceError: return "unhandled device error";
    case flagcxSystemError: return "unhandled system error";
    case flagcxInternalError: return "internal error";
    case flagcxInvalidArgument: return "invalid argument";
    case flagcxInvalidUsage: return "invalid usage";
    case flagcxRemoteError: return "remote process exited or there was a network error";
    case flagcxInProgress: return "operation in progress";
    case flagcxUnhandledCCLError: return "unhandled ccl error";
    case flagcxNotSupported: return "not supported";
    default: return "unknown result code";
  }
}

flagcxResult_t flagcxBarrier(flagcxComm_t comm, flagcxStream_t stream) {
  return postAndMaybeRun(comm, kBarrier, nullptr, nullptr, 0, 0, 0, 0, stream);
}

flagcxResult_t fxSimCommProgress(flagcxComm_t comm, uint64_t *joined, uint64_t *launched) {
  if (!comm || !comm->g || !joined || !launched) return flagcxInvalidArgument;
  std::lock_guard<std::mutex> lock(comm->g->mu);
  *joined = comm->joined;
  *launched = comm->g->launched;
  return flagcxSuccess;
}

flagcxResult_t fxSimCommConfig(flagcxComm_t comm, int key, long long value) {
  if (!comm || !comm->g) return flagcxInvalidArgument;
  Group *g = comm->g;
  std::lock_guard<std::mutex> lock(g->mu);
  switch (key) {
    case FX_SIM_ALGO:
      if (value != FX_ALGO_DIRECT && value != FX_ALGO_RING) return flagcxInvalidArgument;
      g->algo = value;
      break;
    case FX_SIM_ORDER:
      if (value < FX_ORDER_RANK || value > FX_ORDER_HOST) return flagcxInvalidArgument;
      g->order = value;
      break;
    case FX_SIM_NSLICES:
      if (value < 1) return flagcxInvalidArgument;
      g->nslices = value;
      break;
    case FX_SIM_NREDSLICES:
      if (value < 0) return flagcxInvalidArgument;
      g->nredslices = value;
      break;
    case FX_SIM_REDSLICESIZE:
      if (value < 0) return flagcxInvalidArgument;
      g->redslicesize = value;
      break;
    case FX_SIM_SYNC:
      if (value != FX_SYNC_GROUP && value != FX_SYNC_RENDEZVOUS) return flagcxInvalidArgument;
      if (g->nposted) return flagcxInvalidUsage;  // not while a collective is half posted
      g->sync = value;
      break;
    case FX_SIM_ARITH:
      if (value != FX_ARITH_DEFAULT && value != FX_ARITH_ELEMENT) return flagcxInvalidArgument;
      g->arith = value;
      break;
    case FX_SIM_SCRATCH_BYTES:  // reserve now what the scratch users would otherwise allocate at their first call
      if (value < 0) return flagcxInvalidArgument;
      return ensureScratch(g, (size_t)value, nullptr);
    default: return flagcxInvalidArgument;
  }
  return flagcxSuccess;
}

flagcxResult_t flagcxCommCount(const flagcxComm_t comm, int *count) {
  if (!comm || !comm->g || !count) return flagcxInvalidArgument;
  *count = comm->g->n;
  return flagcxSuccess;
}

flagcxResult_t flagcxCommUserRank(const flagcxComm_t comm, int *rank) {
  if (!comm || !rank) return flagcxInvalidArgument;
  *rank = comm->rank;
  return flagcxSuccess;
}

flagcxResult_t flagcxAllReduce(const void *sendbuff, void *recvbuff, size_t count, flagcxDataType_t datatype,
                               flagcxRedOp_t op, flagcxComm_t comm, flagcxStream_t stream) {
  flagcxResult_t rc = screenReduce(datatype, op);
  if (rc != flagcxSuccess) return rc;
  if (count && (!sendbuff || !recvbuff)) return flagcxInvalidArgument;
  return postAndMaybeRun(comm, kAllReduce, sendbuff, recvbuff, count, datatype, op, 0, stream);
}

flagcxResult_t flagcxReduce(const void *sendbuff, void *recvbuff, size_t count, flagcxDataType_t datatype,
                            flagcxRedOp_t op, int root, flagcxComm_t comm, flagcxStream_t stream) {
  flagcxResult_t rc = screenReduce(datatype, op);
  if (rc != flagcxSuccess) return rc;
  if (!comm || root < 0 || root >= comm->g->n) return flagcxInvalidArgument;
  // recvbuff may be NULL except on the root (flagcx.h:365-366)
  if (count && (!sendbuff || (comm->rank == root && !recvbuff))) return flagcxInvalidArgument;
  return postAndMaybeRun(comm, kReduce, sendbuff, recvbuff, count, datatype, op, root, stream);
}

flagcxResult_t flagcxReduceScatter(const void *sendbuff, void *recvbuff, size_t recvcount, flagcxDataType_t datatype,
                                   flagcxRedOp_t op, flagcxComm_t comm, flagcxStream_t stream) {
  flagcxResult_t rc = screenReduce(datatype, op);
  if (rc != flagcxSuccess) return rc;
  if (recvcount && (!sendbuff || !recvbuff)) return flagcxInvalidArgument;
  return postAndMaybeRun(comm, kReduceScatter, sendbuff, recvbuff, recvcount, datatype, op, 0, stream);
}

flagcxResult_t flagcxAllGather(const void *sendbuff, void *recvbuff, size_t sendcount, flagcxDataType_t datatype,
                               flagcxComm_t comm, flagcxStream_t stream) {
  if (fx_dtype_size(datatype) == 0) return flagcxInvalidArgument;
  if (sendcount && (!sendbuff || !recvbuff)) return flagcxInvalidArgument;
  return postAndMaybeRun(comm, kAllGather, sendbuff, recvbuff, sendcount, datatype, 0, 0, stream);
}

flagcxResult_t flagcxAlltoAllv(const void *sendbuff, size_t *sendcounts, size_t *sdispls, void *recvbuff,
                               size_t *recvcounts, size_t *rdispls, flagcxDataType_t datatype, flagcxComm_t comm,
                               flagcxStream_t stream) {
  if (fx_dtype_size(datatype) == 0) return flagcxInvalidArgument;
  if (!sendcounts || !sdispls || !recvcounts || !rdispls) return flagcxInvalidArgument;
  return postAndMaybeRun(comm, kAlltoAllv, sendbuff, recvbuff, 0, datatype, 0, 0, stream, sendcounts, sdispls,
                         recvcounts, rdispls);
}

flagcxResult_t flagcxGather(const void *sendbuff, void *recvbuff, size_t count, flagcxDataType_t datatype, int root,
                            flagcxComm_t comm, flagcxStream_t stream) {
  if (fx_dtype_size(datatype) == 0) return flagcxInvalidArgument;
  if (!comm || root < 0 || root >= comm->g->n) return flagcxInvalidArgument;
  if (count && (!sendbuff || (comm->rank == root && !recvbuff))) return flagcxInvalidArgument;
  return postAndMaybeRun(comm, kGather, sendbuff, recvbuff, count, datatype, 0, root, stream);
}

flagcxResult_t flagcxScatter(const void *sendbuff, void *recvbuff, size_t count, flagcxDataType_t datatype, int root,
                             flagcxComm_t comm, flagcxStream_t stream) {
  if (fx_dtype_size(datatype) == 0) return flagcxInvalidArgument;
  if (!comm || root < 0 || root >= comm->g->n) return flagcxInvalidArgument;
  if (count && (!recvbuff || (comm->rank == root && !sendbuff))) return flagcxInvalidArgument;
  return postAndMaybeRun(comm, kScatter, sendbuff, recvbuff, count, datatype, 0, root, stream);
}

flagcxResult_t flagcxBroadcast(const void *sendbuff, void *recvbuff, size_t count, flagcxDataType_t datatype,
                               int root, flagcxComm_t comm, flagcxStream_t stream) {
  if (fx_dtype_size(datatype) == 0) return flagcxInvalidArgument;
  if (!comm || root < 0 || root >= comm->g->n) return flagcxInvalidArgument;
  if (count && (!recvbuff || (comm->rank == root && !sendbuff))) return flagcxInvalidArgument;
  return postAndMaybeRun(comm, kBroadcast, sendbuff, recvbuff, count, datatype, 0, root, stream);
}

flagcxResult_t flagcxAlltoAll(const void *sendbuff, void *recvbuff, size_t count, flagcxDataType_t datatype,
                              flagcxComm_t comm, flagcxStream_t stream) {
  if (fx_dtype_size(datatype) == 0) return flagcxInvalidArgument;
  if (count && (!sendbuff || !recvbuff)) return flagcxInvalidArgument;
  return postAndMaybeRun(comm, kAlltoAll, sendbuff, recvbuff, count, datatype, 0, 0, stream);
}

flagcxResult_t flagcxSend(const void *sendbuff, size_t count, flagcxDataType_t datatype, int peer, flagcxComm_t comm,
                          flagcxStream_t stream) {
  return postP2p(comm, true, sendbuff, nullptr, count, datatype, peer, stream);
}

flagcxResult_t flagcxRecv(void *recvbuff, size_t count, flagcxDataType_t datatype, int peer, flagcxComm_t comm,
                          flagcxStream_t stream) {
  return postP2p(comm, false, nullptr, recvbuff, count, datatype, peer, stream);
}

// Calls are asynchronous and matched across ranks as they arrive, so in group
// mode a bracket has nothing to defer.  In rendezvous mode the sends and recvs
// posted inside the outermost bracket of this thread are waited for here.
flagcxResult_t flagcxGroupStart(flagcxComm_t) {
  tGroupDepth++;
  return flagcxSuccess;
}
flagcxResult_t flagcxGroupEnd(flagcxComm_t) {
  if (tGroupDepth == 0) return flagcxInvalidUsage;  // no bracket open on this thread
  if (--tGroupDepth > 0) return flagcxSuccess;
  return R(fx::guarded([&]() -> int {
    flagcxResult_t first = flushBatched();
    std::vector<QueuedP2p> queued;
    queued.swap(tQueued);
    {
      struct Closing {
        Closing() { tClosingBracket = true; }
        ~Closing() { tClosingBracket = false; }
      } closing;
      for (const QueuedP2p &q : queued) {
        const flagcxResult_t rc = postP2pImpl(q.comm, q.isSend, q.sbuf, q.rbuf, q.count, q.dtype, q.peer, q.stream);
        if (first == flagcxSuccess) first = rc;
      }
    }
    std::vector<DeferredP2p> mine;
    mine.swap(tDeferred);
    for (const DeferredP2p &d : mine) {
      std::unique_lock<std::mutex> lock(d.g->mu);
      const flagcxResult_t rc = awaitPartner(d.g, lock, d.id, d.stream);
      if (first == flagcxSuccess) first = rc;
    }
    return first;
  }));
}

flagcxResult_t fxSimCommDevice(const flagcxComm_t comm, int *device) {
  if (!comm || !comm->g || !device) return flagcxInvalidArgument;
  *device = comm->g->device;
  return flagcxSuccess;
}

flagcxResult_t fxSimRegisterWindows(flagcxComm_t comm, void *const *windows, size_t bytes) {
  if (!comm || !comm->g) return flagcxInvalidArgument;
  Group *g = comm->g;
  return R(fx::guarded([&]() -> int {
    std::lock_guard<std::mutex> lock(g->mu);
    g->windows.clear();
    g->windowBytes = 0;
    if (!windows) return flagcxSuccess;
    for (int r = 0; r < g->n; r++)
      if (!windows[r]) return flagcxInvalidArgument;
    g->windows.assign(windows, windows + g->n);
    g->windowBytes = bytes;
    return flagcxSuccess;
  }));
}

flagcxResult_t flagcxCustomAllReduceImpl(const void *sendbuff, void *recvbuff, size_t count,
                                         flagcxDataType_t datatype, flagcxRedOp_t op, flagcxComm_t comm,
                                         flagcxStream_t stream) {
  if (!comm || !comm->g || !stream) return flagcxInvalidArgument;
  flagcxResult_t rc = screenReduce(datatype, op);
  if (rc != flagcxSuccess) return flagcxNotSupported;  // the hook only ever declines
  Group *g = comm->g;
  const size_t bytes = count * fx_dtype_size(datatype);
  {
    std::lock_guard<std::mutex> lock(g->mu);
    if (g->windows.empty() || bytes > g->windowBytes) return flagcxNotSupported;
  }
  if (count && (!sendbuff || !recvbuff)) return flagcxInvalidArgument;
  // The copy of sendbuff into this rank's window (custom_allreduce.cu:640-642) is made by the
  // rank that launches the collective, for all ranks in one launch: eight separate
  // device-to-device copies cost 18 us, more than the all-reduce itself up to 4 MiB.
  return postAndMaybeRun(comm, kCustomAllReduce, sendbuff, recvbuff, count, datatype, op, 0, stream);
}

#pragma GCC visibility pop
}  // extern "C"
