// FlagCX collective entry points over simulated ranks on one GPU: communicator
// groups, posting (the last rank to arrive launches) and the C entry points.
// The schedules are in fx_sim_schedules.cc, send / recv in fx_sim_p2p.cc.
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
#include "fx_sim_internal.hpp"

using namespace fxsim;

namespace {

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
