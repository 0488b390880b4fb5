// send / recv between simulated ranks and the group brackets around them.
#include "fx_sim_internal.hpp"

using namespace fxsim;

namespace {

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

#pragma GCC visibility pop
}  // extern "C"
