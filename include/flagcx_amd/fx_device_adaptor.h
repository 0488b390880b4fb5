/*
 * Device-adaptor plugin ABI, version 1, as FlagCX's loader expects it
 * (flagcx/adaptor/include/flagcx_device_adaptor.h:30-116,261-265; loader
 * flagcx/adaptor/device/device_plugin_load.cc:25-103).  The plugin library
 * exports ONE data symbol, `flagcxDeviceAdaptorPlugin_v1`, of this struct
 * type: a 32-byte name followed by 48 function pointers in this exact order.
 * The loader copies sizeof(v1) bytes into its zeroed internal struct, so the
 * post-v1 members are NULL for any plugin.
 *
 * A unit that includes FlagCX's own flagcx_device_adaptor.h must not include
 * this file (same type names); the layouts are identical.
 */
#ifndef FLAGCX_AMD_FX_DEVICE_ADAPTOR_H_
#define FLAGCX_AMD_FX_DEVICE_ADAPTOR_H_

#include <stdbool.h>

#include "flagcx_amd/fx_types.h"

#ifdef __cplusplus
extern "C" {
#endif

#ifndef FLAGCX_DEVICE_ADAPTOR_H_

struct flagcxDevProps {
  char name[256];
  int pciBusId;
  int pciDeviceId;
  int pciDomainId;
};

typedef void (*flagcxLaunchFunc_t)(flagcxStream_t, void *);

#define FX_ADAPTOR_FN(ret, name, args) ret(*name) args

struct flagcxDeviceAdaptor_v1 {
  char name[32];
  /* basic (10) */
  FX_ADAPTOR_FN(flagcxResult_t, deviceSynchronize, (void));
  FX_ADAPTOR_FN(flagcxResult_t, deviceMemcpy, (void *dst, void *src, size_t size, flagcxMemcpyType_t type, flagcxStream_t stream, void *args));
  FX_ADAPTOR_FN(flagcxResult_t, deviceMemset, (void *ptr, int value, size_t size, flagcxMemType_t type, flagcxStream_t stream));
  FX_ADAPTOR_FN(flagcxResult_t, deviceMalloc, (void **ptr, size_t size, flagcxMemType_t type, flagcxStream_t stream));
  FX_ADAPTOR_FN(flagcxResult_t, deviceFree, (void *ptr, flagcxMemType_t type, flagcxStream_t stream));
  FX_ADAPTOR_FN(flagcxResult_t, setDevice, (int dev));
  FX_ADAPTOR_FN(flagcxResult_t, getDevice, (int *dev));
  FX_ADAPTOR_FN(flagcxResult_t, getDeviceCount, (int *count));
  FX_ADAPTOR_FN(flagcxResult_t, getVendor, (char *vendor));
  FX_ADAPTOR_FN(flagcxResult_t, hostGetDevicePointer, (void **pDevice, void *pHost));
  /* GDR (8) */
  FX_ADAPTOR_FN(flagcxResult_t, memHandleInit, (int dev_id, void **memHandle));
  FX_ADAPTOR_FN(flagcxResult_t, memHandleDestroy, (int dev, void *memHandle));
  FX_ADAPTOR_FN(flagcxResult_t, gdrMemAlloc, (void **ptr, size_t size, void *memHandle));
  FX_ADAPTOR_FN(flagcxResult_t, gdrMemFree, (void *ptr, void *memHandle));
  FX_ADAPTOR_FN(flagcxResult_t, hostShareMemAlloc, (void **ptr, size_t size, void *memHandle));
  FX_ADAPTOR_FN(flagcxResult_t, hostShareMemFree, (void *ptr, void *memHandle));
  FX_ADAPTOR_FN(flagcxResult_t, gdrPtrMmap, (void **pcpuptr, void *devptr, size_t sz));
  FX_ADAPTOR_FN(flagcxResult_t, gdrPtrMunmap, (void *cpuptr, size_t sz));
  /* stream (9) */
  FX_ADAPTOR_FN(flagcxResult_t, streamCreate, (flagcxStream_t *stream));
  FX_ADAPTOR_FN(flagcxResult_t, streamDestroy, (flagcxStream_t stream));
  FX_ADAPTOR_FN(flagcxResult_t, streamCopy, (flagcxStream_t *newStream, void *oldStream));
  FX_ADAPTOR_FN(flagcxResult_t, streamFree, (flagcxStream_t stream));
  FX_ADAPTOR_FN(flagcxResult_t, streamSynchronize, (flagcxStream_t stream));
  FX_ADAPTOR_FN(flagcxResult_t, streamQuery, (flagcxStream_t stream));
  FX_ADAPTOR_FN(flagcxResult_t, streamWaitEvent, (flagcxStream_t stream, flagcxEvent_t event));
  FX_ADAPTOR_FN(flagcxResult_t, streamWaitValue64, (flagcxStream_t stream, void *addr, uint64_t value, int flags));
  FX_ADAPTOR_FN(flagcxResult_t, streamWriteValue64, (flagcxStream_t stream, void *addr, uint64_t value, int flags));
  /* event (6) */
  FX_ADAPTOR_FN(flagcxResult_t, eventCreate, (flagcxEvent_t *event, flagcxEventType_t eventType));
  FX_ADAPTOR_FN(flagcxResult_t, eventDestroy, (flagcxEvent_t event));
  FX_ADAPTOR_FN(flagcxResult_t, eventRecord, (flagcxEvent_t event, flagcxStream_t stream));
  FX_ADAPTOR_FN(flagcxResult_t, eventSynchronize, (flagcxEvent_t event));
  FX_ADAPTOR_FN(flagcxResult_t, eventQuery, (flagcxEvent_t event));
  FX_ADAPTOR_FN(flagcxResult_t, eventElapsedTime, (float *ms, flagcxEvent_t start, flagcxEvent_t end));
  /* IPC memory handles (5) */
  FX_ADAPTOR_FN(flagcxResult_t, ipcMemHandleCreate, (flagcxIpcMemHandle_t *handle, size_t *size));
  FX_ADAPTOR_FN(flagcxResult_t, ipcMemHandleGet, (flagcxIpcMemHandle_t handle, void *devPtr));
  FX_ADAPTOR_FN(flagcxResult_t, ipcMemHandleOpen, (flagcxIpcMemHandle_t handle, void **devPtr));
  FX_ADAPTOR_FN(flagcxResult_t, ipcMemHandleClose, (void *devPtr));
  FX_ADAPTOR_FN(flagcxResult_t, ipcMemHandleFree, (flagcxIpcMemHandle_t handle));
  /* kernel launch (4) */
  FX_ADAPTOR_FN(flagcxResult_t, launchKernel, (void *func, unsigned int block_x, unsigned int block_y, unsigned int block_z, unsigned int grid_x, unsigned int grid_y, unsigned int grid_z, void **args, size_t share_mem, void *stream, void *memHandle));
  FX_ADAPTOR_FN(flagcxResult_t, copyArgsInit, (void **args));
  FX_ADAPTOR_FN(flagcxResult_t, copyArgsFree, (void *args));
  FX_ADAPTOR_FN(flagcxResult_t, launchDeviceFunc, (flagcxStream_t stream, flagcxLaunchFunc_t fn, void *args));
  /* others (3) */
  FX_ADAPTOR_FN(flagcxResult_t, getDeviceProperties, (struct flagcxDevProps *props, int dev));
  FX_ADAPTOR_FN(flagcxResult_t, getDevicePciBusId, (char *pciBusId, int len, int dev));
  FX_ADAPTOR_FN(flagcxResult_t, getDeviceByPciBusId, (int *dev, const char *pciBusId));
  /* host function launch (1) */
  FX_ADAPTOR_FN(flagcxResult_t, launchHostFunc, (flagcxStream_t stream, void (*fn)(void *), void *args));
  /* DMA buffer (2) */
  FX_ADAPTOR_FN(flagcxResult_t, dmaSupport, (bool *dmaBufferSupport));
  FX_ADAPTOR_FN(flagcxResult_t, getHandleForAddressRange, (void *handleOut, void *buffer, size_t size, unsigned long long flags));
};

#undef FX_ADAPTOR_FN

#endif /* FLAGCX_DEVICE_ADAPTOR_H_ */

/* Handle layouts owned by this plugin.  The first member is the raw HIP
 * object, as in FlagCX's AMD adaptor header
 * (flagcx/adaptor/include/amd_adaptor.h:13-23), so FlagCX code that reaches
 * into `stream->base` keeps working. */
#define FX_DEVICE_ADAPTOR_NAME "MI355X"
#define FX_DEVICE_ADAPTOR_SYMBOL "flagcxDeviceAdaptorPlugin_v1"
#define FX_VENDOR_STRING "AMD"
#define FX_MAX_VENDOR_LEN 128

#ifdef __cplusplus
}
#endif
#endif /* FLAGCX_AMD_FX_DEVICE_ADAPTOR_H_ */
