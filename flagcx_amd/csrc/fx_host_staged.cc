// Host-staged reducing collectives over simulated ranks, with per-phase timers:
// the reference's CPU path end to end -- hostRunnerAllReduce, hostRunnerReduce and
// hostRunnerReduceScatter (flagcx/runner/host_runner.cc:236-289, 12-67, 291-346)
// on top of the bootstrap ring (flagcx/service/bootstrap.cc:787-1066) -- one host
// thread per rank.
#include <hip/hip_runtime.h>

#include <atomic>
#include <chrono>
#include <cstdlib>
#include <cstring>
#include <new>
#include <thread>
#include <vector>

#include "flagcx_amd/fx_host_staged.h"
#include "fx_common.hpp"

namespace {

inline uint64_t nowNs() {
  return (uint64_t)std::chrono::duration_cast<std::chrono::nanoseconds>(
             std::chrono::steady_clock::now().time_since_epoch())
      .count();
}

// All ranks meet here between the steps of the ring (the reference's ranks meet
// in their socket send / recv pairs).
class Meeting {
 public:
  explicit Meeting(int n) : n_(n), waiting_(0), round_(0) {}
  void arrive() {
    const unsigned my = round_.load(std::memory_order_acquire);
    if (waiting_.fetch_add(1, std::memory_order_acq_rel) + 1 == n_) {
      waiting_.store(0, std::memory_order_relaxed);
      round_.store(my + 1, std::memory_order_release);
      return;
    }
    for (unsigned spins = 0; round_.load(std::memory_order_acquire) == my; spins++)
      if (spins > 200) std::this_thread::yield();
  }

 private:
  const int n_;
  std::atomic<int> waiting_;
  std::atomic<unsigned> round_;
};

// res[i] = local[i] (op) received[i]; res may be `received` itself.  The three
// loops of the reference's host path; integer sums are formed on the unsigned
// type so that wrapping is defined (same bits as the int loops there).
template <class T, class U>
void sumLoop(void *res, const void *local, const void *received, size_t n) {
  const T *a = static_cast<const T *>(local), *b = static_cast<const T *>(received);
  T *c = static_cast<T *>(res);
  for (size_t i = 0; i < n; i++) c[i] = (T)((U)a[i] + (U)b[i]);
}
template <class T>
void maxLoop(void *res, const void *local, const void *received, size_t n) {
  const T *a = static_cast<const T *>(local), *b = static_cast<const T *>(received);
  T *c = static_cast<T *>(res);
  for (size_t i = 0; i < n; i++) c[i] = (a[i] < b[i]) ? b[i] : a[i];   // std::max(local, received)
}
template <class T>
void minLoop(void *res, const void *local, const void *received, size_t n) {
  const T *a = static_cast<const T *>(local), *b = static_cast<const T *>(received);
  T *c = static_cast<T *>(res);
  for (size_t i = 0; i < n; i++) c[i] = (b[i] < a[i]) ? b[i] : a[i];   // std::min(local, received)
}

template <class T, class U>
bool applyOp(int op, void *res, const void *local, const void *received, size_t n) {
  switch (op) {
    case flagcxSum: sumLoop<T, U>(res, local, received, n); return true;
    case flagcxMax: maxLoop<T>(res, local, received, n); return true;
    case flagcxMin: minLoop<T>(res, local, received, n); return true;
    default: return false;
  }
}

bool hostReduce(int dtype, int op, void *res, const void *local, const void *received, size_t n) {
  switch (dtype) {
    case flagcxInt8: return applyOp<signed char, unsigned char>(op, res, local, received, n);
    case flagcxUint8: return applyOp<unsigned char, unsigned char>(op, res, local, received, n);
    case flagcxInt32: return applyOp<int32_t, uint32_t>(op, res, local, received, n);
    case flagcxUint32: return applyOp<uint32_t, uint32_t>(op, res, local, received, n);
    case flagcxInt64: return applyOp<int64_t, uint64_t>(op, res, local, received, n);
    case flagcxUint64: return applyOp<uint64_t, uint64_t>(op, res, local, received, n);
    case flagcxFloat32: return applyOp<float, float>(op, res, local, received, n);
    case flagcxFloat64: return applyOp<double, double>(op, res, local, received, n);
    default: return false;
  }
}

bool carried(int dtype, int op) {
  const bool t = dtype == flagcxInt8 || dtype == flagcxUint8 || dtype == flagcxInt32 || dtype == flagcxUint32 ||
                 dtype == flagcxInt64 || dtype == flagcxUint64 || dtype == flagcxFloat32 || dtype == flagcxFloat64;
  return t && (op == flagcxSum || op == flagcxMax || op == flagcxMin);
}

struct RankState {
  char *in = nullptr, *out = nullptr;          // staged host buffers (send side, receive side)
  size_t inBytes = 0, outBytes = 0;
  char *forSend = nullptr, *forRecv = nullptr; // the ring's two chunk buffers
  std::atomic<const char *> sending{nullptr};  // what this rank "sends" in the current step
};

}  // namespace

struct fxHostStaged {
  int n;
  int device;
  fxDeviceMemcpyFn copy;
  std::vector<RankState> ranks;
  fxHostStaged(int nranks) : n(nranks), device(0), copy(nullptr), ranks((size_t)nranks) {}
};

namespace {

bool growTo(char **buf, size_t *have, size_t want) {
  if (*have >= want) return true;
  size_t size = *have ? *have : (size_t)1 << 20;
  while (size < want) size *= 2;
  char *p = static_cast<char *>(malloc(size));
  if (!p) return false;
  free(*buf);
  *buf = p;
  *have = size;
  return true;
}

flagcxResult_t moveBytes(const fxHostStaged *h, void *dst, const void *src, size_t bytes, flagcxMemcpyType_t type) {
  if (bytes == 0) return flagcxSuccess;
  if (h->copy) return h->copy(dst, const_cast<void *>(src), bytes, type, nullptr, nullptr);
  const hipMemcpyKind kind = (type == flagcxMemcpyDeviceToHost) ? hipMemcpyDeviceToHost : hipMemcpyHostToDevice;
  return hipMemcpy(dst, src, bytes, kind) == hipSuccess ? flagcxSuccess : flagcxUnhandledDeviceError;
}

enum Kind { kAllReduce, kReduce, kReduceScatter };

// One rank's whole call.  Every rank runs the same number of meetings whatever
// its chunk lengths are, so nobody is left waiting.  `count` is the element
// count of the call: per rank for all-reduce and reduce, the receive count for
// reduce-scatter (the send side then holds n times as much).
void rankMain(fxHostStaged *h, Meeting *meet, Kind kind, int root, int rank, const void *sendDev, void *recvDev,
              size_t count, int dtype, int op, uint64_t *t, std::atomic<int> *failed) {
  const int n = h->n;
  RankState &me = h->ranks[(size_t)rank];
  const RankState &prev = h->ranks[(size_t)((rank + n - 1) % n)];
  const size_t ts = fx::dtypeSize(dtype);
  const size_t outSize = count * ts;                                         // what this rank receives
  const size_t size = (kind == kReduceScatter) ? outSize * (size_t)n : outSize;   // what it sends
  auto fail = [&](flagcxResult_t rc) { int zero = 0; failed->compare_exchange_strong(zero, (int)rc); };
  (void)hipSetDevice(h->device);
  t[FX_TIMER_COLL_TOTAL] = nowNs();

  // step 1: staged buffers
  uint64_t t0 = nowNs();
  bool ok = growTo(&me.in, &me.inBytes, size) && growTo(&me.out, &me.outBytes, size);   // the ring works in `out`
  t[FX_TIMER_COLL_ALLOC] = nowNs() - t0;
  if (!ok) fail(flagcxSystemError);

  // step 2: device to host
  t0 = nowNs();
  if (ok) {
    const flagcxResult_t rc = moveBytes(h, me.in, sendDev, size, flagcxMemcpyDeviceToHost);
    if (rc != flagcxSuccess) fail(rc);
  }
  t[FX_TIMER_COLL_MEM_D2H] = nowNs() - t0;

  // step 3: the ring collective on the host
  t0 = nowNs();
  // all-reduce, reduce: chunk i is ceil(size / n) bytes rounded up to whole elements, the last non-empty one short,
  // later ones empty (bootstrap.cc:900-922, 951-971); reduce-scatter: chunk i is rank i's recvcount elements (:1058-1061)
  size_t chunkBytes = (size + (size_t)n - 1) / (size_t)n;
  chunkBytes = (chunkBytes + ts - 1) / ts * ts;
  std::vector<size_t> offset((size_t)n, 0), length((size_t)n, 0);
  size_t longest = 0;
  for (size_t i = 0; i < (size_t)n; i++) {
    if (kind == kReduceScatter) {
      offset[i] = i * outSize;
      length[i] = outSize;
    } else if (chunkBytes * i >= size) {
      offset[i] = size;
      length[i] = 0;
    } else {
      offset[i] = chunkBytes * i;
      length[i] = (chunkBytes * (i + 1) >= size) ? size - chunkBytes * i : chunkBytes;
    }
    if (length[i] > longest) longest = length[i];
  }
  uint64_t a0 = nowNs();
  me.forSend = static_cast<char *>(calloc(longest ? longest : 1, 1));
  me.forRecv = static_cast<char *>(calloc(longest ? longest : 1, 1));
  t[FX_TIMER_COLL_ALLOC] += nowNs() - a0;
  if (!me.forSend || !me.forRecv) fail(flagcxSystemError);
  meet->arrive();                               // everybody knows by now whether somebody failed
  const bool run = failed->load() == 0;
  const char *sendbuff = me.in;
  char *recvbuff = me.out;
  if (n == 1) {   // one rank: the collective is a copy (bootstrap.cc:1006-1011, 1027-1032, 1049-1054)
    if (run) memcpy(recvbuff, sendbuff, outSize);
  } else {
    // reduce-scatter: n-1 steps; the partial of chunk c travels c+1 -> c+2 -> .. -> c
    for (int iter = 0; iter < n - 1; iter++) {
      const size_t sendNo = (size_t)((rank + 2 * n - iter - 1) % n), recvNo = (size_t)((rank + 2 * n - iter - 2) % n);
      if (run && length[sendNo]) {
        const uint64_t m0 = nowNs();
        if (iter == 0) memcpy(me.forSend, sendbuff + offset[sendNo], length[sendNo]);
        else std::swap(me.forSend, me.forRecv);
        t[FX_TIMER_COLL_MEM] += nowNs() - m0;
      }
      me.sending.store(me.forSend, std::memory_order_release);
      meet->arrive();                             // the neighbours' send buffers are ready
      if (run && length[recvNo]) {                // "receive": the chunk the previous rank sends is the one we expect
        memcpy(me.forRecv, prev.sending.load(std::memory_order_acquire), length[recvNo]);
      }
      meet->arrive();                             // everybody has taken its chunk: send buffers may be reused
      if (run && length[recvNo]) {
        const uint64_t c0 = nowNs();
        hostReduce(dtype, op, me.forRecv, sendbuff + offset[recvNo], me.forRecv, length[recvNo] / ts);
        t[FX_TIMER_COLL_CALC] += nowNs() - c0;
      }
    }
    if (run) memcpy(recvbuff, me.forRecv, length[(size_t)rank]);   // this rank's reduced chunk, at the front
    if (kind != kReduceScatter) {
      if (run) memmove(recvbuff + offset[(size_t)rank], recvbuff, length[(size_t)rank]);   // to its place
      if (kind == kAllReduce) {
        // all-gather: step i, this rank takes chunk (rank - i - 1) from the previous rank's receive buffer
        for (int i = 0; i < n - 1; i++) {
          meet->arrive();
          const size_t rslice = (size_t)((rank - i - 1 + 2 * n) % n);
          if (run && length[rslice]) memcpy(recvbuff + offset[rslice], prev.out + offset[rslice], length[rslice]);
          meet->arrive();
        }
      } else {
        // gather to the root: every other rank hands over its chunk (bootstrap.cc:980-993)
        meet->arrive();
        if (run && rank == root)
          for (int i = 0; i < n; i++)
            if (i != rank && length[(size_t)i])
              memcpy(recvbuff + offset[(size_t)i], h->ranks[(size_t)i].out + offset[(size_t)i], length[(size_t)i]);
        meet->arrive();
      }
    }
  }
  free(me.forSend);
  free(me.forRecv);
  me.forSend = me.forRecv = nullptr;
  t[FX_TIMER_COLL_COMM] = nowNs() - t0;

  // step 4: host to device
  t0 = nowNs();
  if (run && (kind != kReduce || rank == root)) {   // a reduce lands on the root only (host_runner.cc:46-49)
    const flagcxResult_t rc = moveBytes(h, recvDev, me.out, outSize, flagcxMemcpyHostToDevice);
    if (rc != flagcxSuccess) fail(rc);
  }
  t[FX_TIMER_COLL_MEM_H2D] = nowNs() - t0;

  // step 5: the staged buffers are kept
  t[FX_TIMER_COLL_FREE] = 0;
  t[FX_TIMER_COLL_TOTAL] = nowNs() - t[FX_TIMER_COLL_TOTAL];
}

}  // namespace

extern "C" {
#pragma GCC visibility push(default)

int fxHostStagedCreate(fxHostStaged_t *h, int nranks, fxDeviceMemcpyFn memcpyFn) {
  if (!h || nranks < 1 || nranks > 64) return flagcxInvalidArgument;
  *h = nullptr;
  return fx::guarded([&]() -> int {
    fxHostStaged *p = new fxHostStaged(nranks);
    p->copy = memcpyFn;
    if (hipGetDevice(&p->device) != hipSuccess) {
      delete p;
      return flagcxUnhandledDeviceError;
    }
    *h = p;
    return flagcxSuccess;
  });
}

namespace {
static int runStaged(fxHostStaged_t h, Kind kind, int root, const void *const *sendbuffs, void *const *recvbuffs, size_t count,
              int dtype, int op, uint64_t *timers) {
  if (!h || !sendbuffs || !recvbuffs) return flagcxInvalidArgument;
  if (!carried(dtype, op)) return flagcxInvalidArgument;   // as the reference's host loops
  if (kind == kReduce && (root < 0 || root >= h->n)) return flagcxInvalidArgument;
  for (int r = 0; r < h->n; r++) {
    const bool receives = kind != kReduce || r == root;
    if (count && (!sendbuffs[r] || (receives && !recvbuffs[r]))) return flagcxInvalidArgument;
  }
  return fx::guarded([&]() -> int {
    const int n = h->n;
    std::vector<uint64_t> local((size_t)n * FX_TIMERS_COLL_COUNT, 0);
    uint64_t *t = timers ? timers : local.data();
    if (timers) memset(timers, 0, (size_t)n * FX_TIMERS_COLL_COUNT * sizeof(uint64_t));
    Meeting meet(n);
    std::atomic<int> failed{0};
    std::vector<std::thread> threads;
    threads.reserve((size_t)n);
    for (int r = 0; r < n; r++)
      threads.emplace_back(rankMain, h, &meet, kind, root, r, sendbuffs[r], recvbuffs[r], count, dtype, op,
                           t + (size_t)r * FX_TIMERS_COLL_COUNT, &failed);
    for (auto &th : threads) th.join();
    return failed.load();
  });
}
}  // namespace

int fxHostStagedAllReduce(fxHostStaged_t h, const void *const *sendbuffs, void *const *recvbuffs, size_t count,
                          int dtype, int op, uint64_t *timers) {
  return runStaged(h, kAllReduce, 0, sendbuffs, recvbuffs, count, dtype, op, timers);
}

int fxHostStagedReduce(fxHostStaged_t h, const void *const *sendbuffs, void *const *recvbuffs, size_t count, int dtype,
                       int op, int root, uint64_t *timers) {
  return runStaged(h, kReduce, root, sendbuffs, recvbuffs, count, dtype, op, timers);
}

int fxHostStagedReduceScatter(fxHostStaged_t h, const void *const *sendbuffs, void *const *recvbuffs, size_t recvcount,
                              int dtype, int op, uint64_t *timers) {
  return runStaged(h, kReduceScatter, 0, sendbuffs, recvbuffs, recvcount, dtype, op, timers);
}

int fxHostStagedDestroy(fxHostStaged_t h) {
  if (!h) return flagcxSuccess;
  for (auto &r : h->ranks) {
    free(r.in);
    free(r.out);
  }
  delete h;
  return flagcxSuccess;
}

#pragma GCC visibility pop
}  // extern "C"
