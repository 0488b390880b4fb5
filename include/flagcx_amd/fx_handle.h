/*
 * What an application written against FlagCX calls around the collectives:
 * the device handle (a table of device operations, flagcx/include/flagcx.h:
 * 143-195), the deprecated handler group (:199-210), buffer allocation and
 * registration (:223-266) and the communicator's housekeeping (:277, :304-334).
 * Same names, argument meaning and return codes, over the simulated ranks of
 * fx_sim.h and the device-adaptor plugin beside the library.
 *
 * Where the reference forwards a call to its CCL adaptor, the answer here is
 * the one its AMD adaptor gives (flagcx/adaptor/ccl/rccl_adaptor.cc:59-65,
 * 106-117): suspend / resume are flagcxInvalidUsage, window registration is
 * flagcxNotSupported.  Buffers of the one GPU are reachable by every simulated
 * rank, so registration has nothing to map: the handle is the buffer.
 */
#ifndef FLAGCX_AMD_FX_HANDLE_H_
#define FLAGCX_AMD_FX_HANDLE_H_

#include "flagcx_amd/fx_types.h"

#ifdef __cplusplus
extern "C" {
#endif

#ifndef FLAGCX_H_

/* flagcx.h:143-186: the device operations an application may call directly.
 * deviceMemcpy has no trailing `args` here, unlike the adaptor's own entry. */
struct flagcxDeviceHandle {
  flagcxResult_t (*deviceSynchronize)(void);
  flagcxResult_t (*deviceMemcpy)(void *dst, void *src, size_t size, flagcxMemcpyType_t type, flagcxStream_t stream);
  flagcxResult_t (*deviceMemset)(void *ptr, int value, size_t size, flagcxMemType_t type, flagcxStream_t stream);
  flagcxResult_t (*deviceMalloc)(void **ptr, size_t size, flagcxMemType_t type, flagcxStream_t stream);
  flagcxResult_t (*deviceFree)(void *ptr, flagcxMemType_t type, flagcxStream_t stream);
  flagcxResult_t (*setDevice)(int dev);
  flagcxResult_t (*getDevice)(int *dev);
  flagcxResult_t (*getDeviceCount)(int *count);
  flagcxResult_t (*getVendor)(char *vendor);
  flagcxResult_t (*hostGetDevicePointer)(void **pDevice, void *pHost);
  flagcxResult_t (*streamCreate)(flagcxStream_t *stream);
  flagcxResult_t (*streamDestroy)(flagcxStream_t stream);
  flagcxResult_t (*streamCopy)(flagcxStream_t *newStream, void *oldStream);
  flagcxResult_t (*streamFree)(flagcxStream_t stream);
  flagcxResult_t (*streamSynchronize)(flagcxStream_t stream);
  flagcxResult_t (*streamQuery)(flagcxStream_t stream);
  flagcxResult_t (*streamWaitEvent)(flagcxStream_t stream, flagcxEvent_t event);
  flagcxResult_t (*eventCreate)(flagcxEvent_t *event, flagcxEventType_t eventType);
  flagcxResult_t (*eventDestroy)(flagcxEvent_t event);
  flagcxResult_t (*eventRecord)(flagcxEvent_t event, flagcxStream_t stream);
  flagcxResult_t (*eventSynchronize)(flagcxEvent_t event);
  flagcxResult_t (*eventQuery)(flagcxEvent_t event);
  flagcxResult_t (*eventElapsedTime)(float *ms, flagcxEvent_t start, flagcxEvent_t end);
  flagcxResult_t (*ipcMemHandleCreate)(flagcxIpcMemHandle_t *handle, size_t *size);
  flagcxResult_t (*ipcMemHandleGet)(flagcxIpcMemHandle_t handle, void *devPtr);
  flagcxResult_t (*ipcMemHandleOpen)(flagcxIpcMemHandle_t handle, void **devPtr);
  flagcxResult_t (*ipcMemHandleClose)(void *devPtr);
  flagcxResult_t (*ipcMemHandleFree)(flagcxIpcMemHandle_t handle);
};
typedef struct flagcxDeviceHandle *flagcxDeviceHandle_t;

/* flagcx.h:199-204 (deprecated there, still what its older tests use) */
struct flagcxHandlerGroup {
  flagcxUniqueId_t uniqueId;
  flagcxComm_t comm;
  flagcxDeviceHandle_t devHandle;
};
typedef struct flagcxHandlerGroup *flagcxHandlerGroup_t;

/* flagcx.h:216-220 */
typedef enum { flagcxMemCCL = 0, flagcxMemSHMEM = 1 } flagcxMemAllocator_t;

struct flagcxWindow;
typedef struct flagcxWindow *flagcxWindow_t;
#define FLAGCX_WIN_DEFAULT 0x00
#define FLAGCX_WIN_COLL_SYMMETRIC 0x01

#endif /* FLAGCX_H_ */

/* flagcx.h:192,195: loads the device-adaptor plugin that sits beside this
 * library and hands out a table of its operations; Free releases the table. */
flagcxResult_t flagcxDeviceHandleInit(flagcxDeviceHandle_t *devHandle);
flagcxResult_t flagcxDeviceHandleFree(flagcxDeviceHandle_t devHandle);
/* flagcx.h:207,210: a zeroed handler group with its device handle filled in
 * (flagcx.cc:195-218); the caller provides uniqueId and comm. */
flagcxResult_t flagcxHandleInit(flagcxHandlerGroup_t *handler);
flagcxResult_t flagcxHandleFree(flagcxHandlerGroup_t handler);

/* flagcx.h:223-244 (C spelling: the allocator argument is not defaulted).
 * flagcxMemAlloc refuses a NULL ptr or size 0 (flagcx.cc:221-226); flagcxMemFree
 * and flagcxCommDeregister accept NULL (flagcx.cc:248-252, 1397-1398);
 * flagcxMemSHMEM has no provider here: flagcxInternalError, as when the
 * reference's shmem adaptor is not loaded (flagcx.cc:227-231). */
flagcxResult_t flagcxMemAlloc(void **ptr, size_t size, flagcxMemAllocator_t allocator);
flagcxResult_t flagcxMemFree(void *ptr, flagcxMemAllocator_t allocator);
flagcxResult_t flagcxCommRegister(const flagcxComm_t comm, void *buff, size_t size, void **handle,
                                  flagcxMemAllocator_t allocator);
flagcxResult_t flagcxCommDeregister(const flagcxComm_t comm, void *handle, flagcxMemAllocator_t allocator);
/* flagcx.h:253-266: flagcxNotSupported, the AMD adaptor's answer */
flagcxResult_t flagcxCommWindowRegister(flagcxComm_t comm, void *buff, size_t size, flagcxWindow_t *win, int winFlags,
                                        flagcxMemAllocator_t allocator);
flagcxResult_t flagcxCommWindowDeregister(flagcxComm_t comm, flagcxWindow_t win, flagcxMemAllocator_t allocator);

/* flagcx.h:277: always 1 -- the simulated ranks share one GPU */
flagcxResult_t flagcxIsHomoComm(flagcxComm_t comm, int *isHomo);
/* flagcx.h:304: waits for everything enqueued on the communicator's GPU */
flagcxResult_t flagcxCommFinalize(flagcxComm_t comm);
/* flagcx.h:312: releases the rank like flagcxCommDestroy (nothing runs on the
 * device on a communicator's behalf beyond the kernels already enqueued) */
flagcxResult_t flagcxCommAbort(flagcxComm_t comm);
/* flagcx.h:315,318: flagcxInvalidUsage, the AMD adaptor's answer */
flagcxResult_t flagcxCommResume(flagcxComm_t comm);
flagcxResult_t flagcxCommSuspend(flagcxComm_t comm);
/* flagcx.h:324: "" for a communicator, the reference's own text for NULL */
const char *flagcxGetLastError(flagcxComm_t comm);
/* flagcx.h:327: errors are returned by the call that meets them; nothing is
 * left to report asynchronously */
flagcxResult_t flagcxCommGetAsyncError(flagcxComm_t comm, flagcxResult_t *asyncError);
/* flagcx.h:334 */
flagcxResult_t flagcxCommGetDeviceNumber(const flagcxComm_t comm, int *device);

#ifdef __cplusplus
}
#endif
#endif /* FLAGCX_AMD_FX_HANDLE_H_ */
