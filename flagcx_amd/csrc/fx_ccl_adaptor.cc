// CCL-adaptor plugin for FlagCX over the simulated-rank collectives: exports
// flagcxCCLAdaptorPlugin_v1.  Where FlagCX's RCCL adaptor forwards to a vendor
// library (flagcx/adaptor/ccl/rccl_adaptor.cc:8-345), this one forwards to the
// in-process group of fx_sim.cc, so an unmodified FlagCX runner that drives a
// CCL adaptor (flagcx/runner/homo_runner.cc:8-22) lands in the gfx950 kernels.
// Ranks of one communicator must live in ONE process and share one GPU; the
// unique id is what ties their commInitRank calls together.
#include <hip/hip_runtime.h>

#include <cstdlib>
#include <cstring>
#include <new>

#include "flagcx_amd/fx_ccl_adaptor.h"
#include "flagcx_amd/fx_kernels.h"
#include "flagcx_amd/fx_sim.h"

constexpr int kMaxOutgrown = 128;  // two directions, each at least doubling: never reached in practice
struct flagcxInnerComm {
  flagcxComm_t base;           // simulated-rank communicator
  void *staged[2];             // send / recv staging buffers handed out by getStagedBuffer
  size_t stagedBytes[2];
  void *outgrown[kMaxOutgrown];  // earlier, smaller staging buffers: the caller may still hold them
  int noutgrown;
};

namespace {

flagcxResult_t cclGetVersion(int *version) {
  if (!version) return flagcxInvalidArgument;
  *version = 100;  // 0.1.0 of this adaptor
  return flagcxSuccess;
}

// 4120 bytes of id space; the simulated-rank layer's 256-byte id (unique within
// the process) goes into the front of it.
flagcxResult_t cclGetUniqueId(flagcxInnerUniqueId_t *uniqueId) {
  if (!uniqueId) return flagcxInvalidArgument;
  if (*uniqueId == nullptr) {
    *uniqueId = static_cast<flagcxInnerUniqueId *>(calloc(1, sizeof(flagcxInnerUniqueId)));
    if (*uniqueId == nullptr) return flagcxSystemError;
  }
  flagcxUniqueId id;
  flagcxResult_t rc = flagcxGetUniqueId(&id);
  if (rc != flagcxSuccess) return rc;
  static_assert(sizeof((*uniqueId)->internal) >= sizeof(id.internal), "inner id holds the group id");
  memset((*uniqueId)->internal, 0, sizeof((*uniqueId)->internal));
  memcpy((*uniqueId)->internal, id.internal, sizeof(id.internal));
  return flagcxSuccess;
}

const char *cclGetErrorString(flagcxResult_t r) { return flagcxGetErrorString(r); }

const char *cclGetLastError(flagcxInnerComm_t) { return ""; }

// Device staging buffers cached per communicator and direction; grown on demand
// (at least doubling).  A buffer handed out earlier stays valid until the
// communicator is destroyed: the caller may still hold its address, and freeing
// it would wait for the whole device.
flagcxResult_t cclGetStagedBuffer(const flagcxInnerComm_t comm, void **buff, size_t size, int isRecv) {
  if (!comm || !buff) return flagcxInvalidArgument;
  const int i = isRecv ? 1 : 0;
  if (comm->stagedBytes[i] < size) {
    if (comm->staged[i] && comm->noutgrown == kMaxOutgrown) return flagcxSystemError;
    size_t want = comm->stagedBytes[i] * 2;
    if (want < size) want = size;
    void *blk = nullptr;
    if (hipMalloc(&blk, want) != hipSuccess) return flagcxUnhandledDeviceError;
    if (comm->staged[i]) comm->outgrown[comm->noutgrown++] = comm->staged[i];
    comm->staged[i] = blk;
    comm->stagedBytes[i] = want;
  }
  *buff = comm->staged[i];
  return flagcxSuccess;
}

flagcxResult_t cclCommInitRank(flagcxInnerComm_t *comm, int nranks, flagcxInnerUniqueId *commId, int rank,
                               struct bootstrapState *) {
  if (!comm || !commId) return flagcxInvalidArgument;
  flagcxInnerComm *c = *comm ? *comm : static_cast<flagcxInnerComm *>(calloc(1, sizeof(flagcxInnerComm)));
  if (!c) return flagcxSystemError;
  flagcxResult_t rc = fxSimCommInitRank(&c->base, nranks, commId->internal, FLAGCX_UNIQUE_ID_BYTES, rank);
  if (rc != flagcxSuccess) {
    if (!*comm) free(c);
    return rc;
  }
  *comm = c;
  return flagcxSuccess;
}

flagcxResult_t cclCommFinalize(flagcxInnerComm_t comm) {
  if (!comm) return flagcxInvalidArgument;
  return hipDeviceSynchronize() == hipSuccess ? flagcxSuccess : flagcxUnhandledDeviceError;
}

flagcxResult_t cclCommDestroy(flagcxInnerComm_t comm) {
  if (!comm) return flagcxInvalidArgument;
  for (int i = 0; i < 2; i++)
    if (comm->staged[i]) (void)hipFree(comm->staged[i]);
  for (int i = 0; i < comm->noutgrown; i++) (void)hipFree(comm->outgrown[i]);
  flagcxResult_t rc = comm->base ? fxSimCommDestroy(comm->base) : flagcxSuccess;
  free(comm);
  return rc;
}

flagcxResult_t cclCommAbort(flagcxInnerComm_t comm) { return cclCommDestroy(comm); }
flagcxResult_t cclCommResume(flagcxInnerComm_t) { return flagcxInvalidUsage; }   // as the RCCL adaptor
flagcxResult_t cclCommSuspend(flagcxInnerComm_t) { return flagcxInvalidUsage; }

flagcxResult_t cclCommCount(const flagcxInnerComm_t comm, int *count) {
  return comm ? flagcxCommCount(comm->base, count) : flagcxInvalidArgument;
}
flagcxResult_t cclCommGetDeviceNumber(const flagcxInnerComm_t comm, int *device) {
  return comm ? fxSimCommDevice(comm->base, device) : flagcxInvalidArgument;
}
flagcxResult_t cclCommUserRank(const flagcxInnerComm_t comm, int *rank) {
  return comm ? flagcxCommUserRank(comm->base, rank) : flagcxInvalidArgument;
}
flagcxResult_t cclCommGetAsyncError(flagcxInnerComm_t comm, flagcxResult_t *asyncError) {
  if (!comm || !asyncError) return flagcxInvalidArgument;
  *asyncError = flagcxSuccess;
  return flagcxSuccess;
}

flagcxResult_t cclMemAlloc(void **ptr, size_t size) {
  if (!ptr) return flagcxInvalidArgument;
  return hipMalloc(ptr, size) == hipSuccess ? flagcxSuccess : flagcxUnhandledDeviceError;
}
flagcxResult_t cclMemFree(void *ptr) {
  if (!ptr) return flagcxSuccess;
  return hipFree(ptr) == hipSuccess ? flagcxSuccess : flagcxUnhandledDeviceError;
}

// Every buffer of the one GPU is already reachable by every simulated rank:
// registration has nothing to map.  The handle is the buffer itself.
flagcxResult_t cclCommRegister(const flagcxInnerComm_t comm, void *buff, size_t, void **handle) {
  if (!comm || !buff || !handle) return flagcxInvalidArgument;
  *handle = buff;
  return flagcxSuccess;
}
flagcxResult_t cclCommDeregister(const flagcxInnerComm_t comm, void *) {
  return comm ? flagcxSuccess : flagcxInvalidArgument;
}
flagcxResult_t cclCommWindowRegister(flagcxInnerComm_t, void *, size_t, flagcxInnerWindow_t *, int) {
  return flagcxNotSupported;
}
flagcxResult_t cclCommWindowDeregister(flagcxInnerComm_t, flagcxInnerWindow_t) { return flagcxNotSupported; }

#define FX_BASE(c) ((c) ? (c)->base : nullptr)

flagcxResult_t cclReduce(const void *s, void *r, size_t count, flagcxDataType_t dt, flagcxRedOp_t op, int root,
                         flagcxInnerComm_t comm, flagcxStream_t stream) {
  return flagcxReduce(s, r, count, dt, op, root, FX_BASE(comm), stream);
}
flagcxResult_t cclGather(const void *s, void *r, size_t count, flagcxDataType_t dt, int root, flagcxInnerComm_t comm,
                         flagcxStream_t stream) {
  return flagcxGather(s, r, count, dt, root, FX_BASE(comm), stream);
}
flagcxResult_t cclScatter(const void *s, void *r, size_t count, flagcxDataType_t dt, int root, flagcxInnerComm_t comm,
                          flagcxStream_t stream) {
  return flagcxScatter(s, r, count, dt, root, FX_BASE(comm), stream);
}
flagcxResult_t cclBroadcast(const void *s, void *r, size_t count, flagcxDataType_t dt, int root,
                            flagcxInnerComm_t comm, flagcxStream_t stream) {
  return flagcxBroadcast(s, r, count, dt, root, FX_BASE(comm), stream);
}
flagcxResult_t cclAllReduce(const void *s, void *r, size_t count, flagcxDataType_t dt, flagcxRedOp_t op,
                            flagcxInnerComm_t comm, flagcxStream_t stream) {
  return flagcxAllReduce(s, r, count, dt, op, FX_BASE(comm), stream);
}
flagcxResult_t cclReduceScatter(const void *s, void *r, size_t recvcount, flagcxDataType_t dt, flagcxRedOp_t op,
                                flagcxInnerComm_t comm, flagcxStream_t stream) {
  return flagcxReduceScatter(s, r, recvcount, dt, op, FX_BASE(comm), stream);
}
flagcxResult_t cclAllGather(const void *s, void *r, size_t sendcount, flagcxDataType_t dt, flagcxInnerComm_t comm,
                            flagcxStream_t stream) {
  return flagcxAllGather(s, r, sendcount, dt, FX_BASE(comm), stream);
}
flagcxResult_t cclAlltoAll(const void *s, void *r, size_t count, flagcxDataType_t dt, flagcxInnerComm_t comm,
                           flagcxStream_t stream) {
  return flagcxAlltoAll(s, r, count, dt, FX_BASE(comm), stream);
}
flagcxResult_t cclAlltoAllv(const void *s, size_t *sc, size_t *sd, void *r, size_t *rc, size_t *rd,
                            flagcxDataType_t dt, flagcxInnerComm_t comm, flagcxStream_t stream) {
  return flagcxAlltoAllv(s, sc, sd, r, rc, rd, dt, FX_BASE(comm), stream);
}
flagcxResult_t cclSend(const void *s, size_t count, flagcxDataType_t dt, int peer, flagcxInnerComm_t comm,
                       flagcxStream_t stream) {
  return flagcxSend(s, count, dt, peer, FX_BASE(comm), stream);
}
flagcxResult_t cclRecv(void *r, size_t count, flagcxDataType_t dt, int peer, flagcxInnerComm_t comm,
                       flagcxStream_t stream) {
  return flagcxRecv(r, count, dt, peer, FX_BASE(comm), stream);
}
// The brackets are per host thread in the simulated-rank layer, which is all
// these two can name.
flagcxResult_t cclGroupStart(void) { return flagcxGroupStart(nullptr); }
flagcxResult_t cclGroupEnd(void) { return flagcxGroupEnd(nullptr); }

}  // namespace

extern "C" __attribute__((visibility("default"))) struct flagcxCCLAdaptor_v1 flagcxCCLAdaptorPlugin_v1 = {
    FX_CCL_ADAPTOR_NAME,
    cclGetVersion, cclGetUniqueId, cclGetErrorString, cclGetLastError, cclGetStagedBuffer,
    cclCommInitRank, cclCommFinalize, cclCommDestroy, cclCommAbort, cclCommResume, cclCommSuspend, cclCommCount,
    cclCommGetDeviceNumber, cclCommUserRank, cclCommGetAsyncError, cclMemAlloc, cclMemFree, cclCommRegister,
    cclCommDeregister, cclCommWindowRegister, cclCommWindowDeregister,
    cclReduce, cclGather, cclScatter, cclBroadcast, cclAllReduce, cclReduceScatter, cclAllGather, cclAlltoAll,
    cclAlltoAllv, cclSend, cclRecv,
    cclGroupStart, cclGroupEnd,
};
