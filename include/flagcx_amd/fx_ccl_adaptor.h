/*
 * CCL-adaptor plugin ABI, version 1, as FlagCX's loader expects it
 * (flagcx/adaptor/include/flagcx_ccl_adaptor.h:42-122,229-230; loader
 * flagcx/adaptor/ccl/ccl_plugin_load.cc:22-101).  The plugin library exports
 * ONE data symbol, `flagcxCCLAdaptorPlugin_v1`: a name pointer followed by 34
 * function pointers in this order, all of which the loader requires non-NULL.
 *
 * A unit that includes FlagCX's own flagcx_ccl_adaptor.h must not include this
 * file (same type names); the layouts are identical.
 */
#ifndef FLAGCX_AMD_FX_CCL_ADAPTOR_H_
#define FLAGCX_AMD_FX_CCL_ADAPTOR_H_

#include "flagcx_amd/fx_types.h"

#ifdef __cplusplus
extern "C" {
#endif

#ifndef FLAGCX_CCL_ADAPTOR_H_

struct bootstrapState;
struct flagcxInnerComm;
typedef struct flagcxInnerComm *flagcxInnerComm_t;
struct flagcxInnerWindow;
typedef struct flagcxInnerWindow *flagcxInnerWindow_t;

#define FLAGCX_INNER_UNIQUE_ID_BYTES 4120
typedef union {
  char internal[FLAGCX_INNER_UNIQUE_ID_BYTES];
  uint64_t alignment;
} flagcxInnerUniqueId;
typedef flagcxInnerUniqueId *flagcxInnerUniqueId_t;

struct flagcxCCLAdaptor_v1 {
  const char *name;
  /* basic (5) */
  flagcxResult_t (*getVersion)(int *version);
  flagcxResult_t (*getUniqueId)(flagcxInnerUniqueId_t *uniqueId);
  const char *(*getErrorString)(flagcxResult_t result);
  const char *(*getLastError)(flagcxInnerComm_t comm);
  flagcxResult_t (*getStagedBuffer)(const flagcxInnerComm_t comm, void **buff, size_t size, int isRecv);
  /* communicator (16) */
  flagcxResult_t (*commInitRank)(flagcxInnerComm_t *comm, int nranks, flagcxInnerUniqueId *commId, int rank, struct bootstrapState *bootstrap);
  flagcxResult_t (*commFinalize)(flagcxInnerComm_t comm);
  flagcxResult_t (*commDestroy)(flagcxInnerComm_t comm);
  flagcxResult_t (*commAbort)(flagcxInnerComm_t comm);
  flagcxResult_t (*commResume)(flagcxInnerComm_t comm);
  flagcxResult_t (*commSuspend)(flagcxInnerComm_t comm);
  flagcxResult_t (*commCount)(const flagcxInnerComm_t comm, int *count);
  flagcxResult_t (*commGetDeviceNumber)(const flagcxInnerComm_t comm, int *device);
  flagcxResult_t (*commUserRank)(const flagcxInnerComm_t comm, int *rank);
  flagcxResult_t (*commGetAsyncError)(flagcxInnerComm_t comm, flagcxResult_t *asyncError);
  flagcxResult_t (*memAlloc)(void **ptr, size_t size);
  flagcxResult_t (*memFree)(void *ptr);
  flagcxResult_t (*commRegister)(const flagcxInnerComm_t comm, void *buff, size_t size, void **handle);
  flagcxResult_t (*commDeregister)(const flagcxInnerComm_t comm, void *handle);
  flagcxResult_t (*commWindowRegister)(flagcxInnerComm_t comm, void *buff, size_t size, flagcxInnerWindow_t *win, int winFlags);
  flagcxResult_t (*commWindowDeregister)(flagcxInnerComm_t comm, flagcxInnerWindow_t win);
  /* communication (11) */
  flagcxResult_t (*reduce)(const void *sendbuff, void *recvbuff, size_t count, flagcxDataType_t datatype, flagcxRedOp_t op, int root, flagcxInnerComm_t comm, flagcxStream_t stream);
  flagcxResult_t (*gather)(const void *sendbuff, void *recvbuff, size_t count, flagcxDataType_t datatype, int root, flagcxInnerComm_t comm, flagcxStream_t stream);
  flagcxResult_t (*scatter)(const void *sendbuff, void *recvbuff, size_t count, flagcxDataType_t datatype, int root, flagcxInnerComm_t comm, flagcxStream_t stream);
  flagcxResult_t (*broadcast)(const void *sendbuff, void *recvbuff, size_t count, flagcxDataType_t datatype, int root, flagcxInnerComm_t comm, flagcxStream_t stream);
  flagcxResult_t (*allReduce)(const void *sendbuff, void *recvbuff, size_t count, flagcxDataType_t datatype, flagcxRedOp_t op, flagcxInnerComm_t comm, flagcxStream_t stream);
  flagcxResult_t (*reduceScatter)(const void *sendbuff, void *recvbuff, size_t recvcount, flagcxDataType_t datatype, flagcxRedOp_t op, flagcxInnerComm_t comm, flagcxStream_t stream);
  flagcxResult_t (*allGather)(const void *sendbuff, void *recvbuff, size_t sendcount, flagcxDataType_t datatype, flagcxInnerComm_t comm, flagcxStream_t stream);
  flagcxResult_t (*alltoAll)(const void *sendbuff, void *recvbuff, size_t count, flagcxDataType_t datatype, flagcxInnerComm_t comm, flagcxStream_t stream);
  flagcxResult_t (*alltoAllv)(const void *sendbuff, size_t *sendcounts, size_t *sdispls, void *recvbuff, size_t *recvcounts, size_t *rdispls, flagcxDataType_t datatype, flagcxInnerComm_t comm, flagcxStream_t stream);
  flagcxResult_t (*send)(const void *sendbuff, size_t count, flagcxDataType_t datatype, int peer, flagcxInnerComm_t comm, flagcxStream_t stream);
  flagcxResult_t (*recv)(void *recvbuff, size_t count, flagcxDataType_t datatype, int peer, flagcxInnerComm_t comm, flagcxStream_t stream);
  /* group (2) */
  flagcxResult_t (*groupStart)(void);
  flagcxResult_t (*groupEnd)(void);
};

#endif /* FLAGCX_CCL_ADAPTOR_H_ */

#define FX_CCL_ADAPTOR_NAME "MI355X-SIM"
#define FX_CCL_ADAPTOR_SYMBOL "flagcxCCLAdaptorPlugin_v1"

#ifdef __cplusplus
}
#endif
#endif /* FLAGCX_AMD_FX_CCL_ADAPTOR_H_ */
