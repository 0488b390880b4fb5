// The calls an application written against FlagCX makes around its collectives
// (flagcx/include/flagcx.h:143-334; the reference's own definitions are in
// flagcx/flagcx.cc:163-270,1267-1430,1551-1600,2360-2478), answered for simulated
// ranks on one GPU.  Device operations are the device-adaptor plugin's: the
// handle is a table of forwarders to the plugin that sits beside this library.
#include <dlfcn.h>
#include <hip/hip_runtime.h>

#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>

#include "flagcx_amd/fx_device_adaptor.h"
#include "flagcx_amd/fx_handle.h"
#include "flagcx_amd/fx_sim.h"

namespace {

std::mutex gMu;
const flagcxDeviceAdaptor_v1 *gAdaptor = nullptr;   // loaded once, kept for the life of the process

// The plugin is found next to the library this code is in, not through the
// search path: the pair is built and shipped together.
const flagcxDeviceAdaptor_v1 *adaptor() {
  std::lock_guard<std::mutex> lock(gMu);
  if (gAdaptor) return gAdaptor;
  Dl_info me;
  if (!dladdr((const void *)&flagcxDeviceHandleInit, &me) || !me.dli_fname) return nullptr;
  std::string path(me.dli_fname);
  path.erase(path.find_last_of('/') + 1);
  path += "libflagcx-device-mi355x.so";
  void *h = dlopen(path.c_str(), RTLD_NOW | RTLD_LOCAL);
  if (!h) return nullptr;
  gAdaptor = (const flagcxDeviceAdaptor_v1 *)dlsym(h, FX_DEVICE_ADAPTOR_SYMBOL);
  return gAdaptor;
}

// The one entry whose signature differs between the application's table and the adaptor's.
flagcxResult_t memcpyNoArgs(void *dst, void *src, size_t size, flagcxMemcpyType_t type, flagcxStream_t stream) {
  return gAdaptor->deviceMemcpy(dst, src, size, type, stream, nullptr);
}

}  // namespace

extern "C" {
#pragma GCC visibility push(default)

flagcxResult_t flagcxDeviceHandleInit(flagcxDeviceHandle_t *devHandle) {
  if (!devHandle) return flagcxInvalidArgument;
  *devHandle = nullptr;
  const flagcxDeviceAdaptor_v1 *a = adaptor();
  if (!a) return flagcxInternalError;   // the plugin is missing or does not export its table
  flagcxDeviceHandle *h = (flagcxDeviceHandle *)calloc(1, sizeof(flagcxDeviceHandle));
  if (!h) return flagcxSystemError;
  h->deviceSynchronize = a->deviceSynchronize;
  h->deviceMemcpy = memcpyNoArgs;
  h->deviceMemset = a->deviceMemset;
  h->deviceMalloc = a->deviceMalloc;
  h->deviceFree = a->deviceFree;
  h->setDevice = a->setDevice;
  h->getDevice = a->getDevice;
  h->getDeviceCount = a->getDeviceCount;
  h->getVendor = a->getVendor;
  h->hostGetDevicePointer = a->hostGetDevicePointer;
  h->streamCreate = a->streamCreate;
  h->streamDestroy = a->streamDestroy;
  h->streamCopy = a->streamCopy;
  h->streamFree = a->streamFree;
  h->streamSynchronize = a->streamSynchronize;
  h->streamQuery = a->streamQuery;
  h->streamWaitEvent = a->streamWaitEvent;
  h->eventCreate = a->eventCreate;
  h->eventDestroy = a->eventDestroy;
  h->eventRecord = a->eventRecord;
  h->eventSynchronize = a->eventSynchronize;
  h->eventQuery = a->eventQuery;
  h->eventElapsedTime = a->eventElapsedTime;
  h->ipcMemHandleCreate = a->ipcMemHandleCreate;
  h->ipcMemHandleGet = a->ipcMemHandleGet;
  h->ipcMemHandleOpen = a->ipcMemHandleOpen;
  h->ipcMemHandleClose = a->ipcMemHandleClose;
  h->ipcMemHandleFree = a->ipcMemHandleFree;
  *devHandle = h;
  return flagcxSuccess;
}

flagcxResult_t flagcxDeviceHandleFree(flagcxDeviceHandle_t devHandle) {
  free(devHandle);
  return flagcxSuccess;
}

flagcxResult_t flagcxHandleInit(flagcxHandlerGroup_t *handler) {
  if (!handler) return flagcxInvalidArgument;
  *handler = (flagcxHandlerGroup *)calloc(1, sizeof(flagcxHandlerGroup));
  if (!*handler) return flagcxSystemError;
  const flagcxResult_t rc = flagcxDeviceHandleInit(&(*handler)->devHandle);
  if (rc != flagcxSuccess) {
    free(*handler);
    *handler = nullptr;
  }
  return rc;
}

flagcxResult_t flagcxHandleFree(flagcxHandlerGroup_t handler) {
  if (handler) {
    (void)flagcxDeviceHandleFree(handler->devHandle);
    free(handler);
  }
  return flagcxSuccess;
}

flagcxResult_t flagcxMemAlloc(void **ptr, size_t size, flagcxMemAllocator_t allocator) {
  if (!ptr || size == 0) return flagcxInvalidArgument;
  if (allocator == flagcxMemSHMEM) return flagcxInternalError;
  if (allocator != flagcxMemCCL) return flagcxInvalidArgument;
  return hipMalloc(ptr, size) == hipSuccess ? flagcxSuccess : flagcxUnhandledDeviceError;
}

flagcxResult_t flagcxMemFree(void *ptr, flagcxMemAllocator_t allocator) {
  if (!ptr) return flagcxSuccess;
  if (allocator == flagcxMemSHMEM) return flagcxInternalError;
  if (allocator != flagcxMemCCL) return flagcxInvalidArgument;
  return hipFree(ptr) == hipSuccess ? flagcxSuccess : flagcxUnhandledDeviceError;
}

flagcxResult_t flagcxCommRegister(const flagcxComm_t, void *buff, size_t size, void **handle, flagcxMemAllocator_t) {
  if (!buff || size == 0 || !handle) return flagcxInvalidArgument;
  *handle = buff;
  return flagcxSuccess;
}

flagcxResult_t flagcxCommDeregister(const flagcxComm_t, void *, flagcxMemAllocator_t) { return flagcxSuccess; }

flagcxResult_t flagcxCommWindowRegister(flagcxComm_t, void *, size_t, flagcxWindow_t *win, int, flagcxMemAllocator_t) {
  if (win) *win = nullptr;
  return flagcxNotSupported;
}

flagcxResult_t flagcxCommWindowDeregister(flagcxComm_t, flagcxWindow_t, flagcxMemAllocator_t) {
  return flagcxNotSupported;
}

flagcxResult_t flagcxIsHomoComm(flagcxComm_t comm, int *isHomo) {
  if (!comm || !isHomo) return flagcxInvalidArgument;
  *isHomo = 1;
  return flagcxSuccess;
}

flagcxResult_t flagcxCommFinalize(flagcxComm_t comm) {
  int device = 0;
  const flagcxResult_t rc = fxSimCommDevice(comm, &device);
  if (rc != flagcxSuccess) return rc;
  int current = 0;
  if (hipGetDevice(&current) != hipSuccess) return flagcxUnhandledDeviceError;
  if (current != device && hipSetDevice(device) != hipSuccess) return flagcxUnhandledDeviceError;
  const hipError_t e = hipDeviceSynchronize();
  if (current != device) (void)hipSetDevice(current);
  return e == hipSuccess ? flagcxSuccess : flagcxUnhandledDeviceError;
}

flagcxResult_t flagcxCommAbort(flagcxComm_t comm) { return flagcxCommDestroy(comm); }
flagcxResult_t flagcxCommResume(flagcxComm_t comm) { return comm ? flagcxInvalidUsage : flagcxInvalidArgument; }
flagcxResult_t flagcxCommSuspend(flagcxComm_t comm) { return comm ? flagcxInvalidUsage : flagcxInvalidArgument; }

const char *flagcxGetLastError(flagcxComm_t comm) {
  return comm ? "" : "Undefined: flagcxComm is not fully initialized.";
}

flagcxResult_t flagcxCommGetAsyncError(flagcxComm_t comm, flagcxResult_t *asyncError) {
  if (!comm || !asyncError) return flagcxInvalidArgument;
  *asyncError = flagcxSuccess;
  return flagcxSuccess;
}

flagcxResult_t flagcxCommGetDeviceNumber(const flagcxComm_t comm, int *device) { return fxSimCommDevice(comm, device); }

#pragma GCC visibility pop
}
