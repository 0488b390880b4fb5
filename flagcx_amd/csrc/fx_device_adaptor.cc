// MI355X device-adaptor plugin for FlagCX: exports flagcxDeviceAdaptorPlugin_v1.
//
// Behavioural model: FlagCX's built-in HIP adaptor
// (flagcx/adaptor/device/hip_adaptor.cc), with the holes that keep FlagCX's
// reduce path from running on AMD filled in: hostGetDevicePointer (:375 is
// NULL there; the reduce FIFO needs it, flagcx/runner/uni_runner_impl.cc:1815),
// IPC memory handles (:231-257 return flagcxNotSupported), stream value
// wait/write and event timing (:319-330).  Every entry point is thread-safe
// and keeps no per-thread device state.
#include <hip/hip_runtime.h>

#include <cstdlib>
#include <cstring>
#include <new>

#include "flagcx_amd/fx_device_adaptor.h"

struct flagcxStream {
  hipStream_t base;
};
struct flagcxEvent {
  hipEvent_t base;
};
struct flagcxIpcMemHandle {
  hipIpcMemHandle_t base;
};

namespace {

// The error is handed to the caller as a return code; it is also taken out of
// the runtime's per-thread last-error slot so that it cannot be mistaken for the
// result of a later, unrelated call.
inline flagcxResult_t dev(hipError_t e) {
  if (e == hipSuccess) return flagcxSuccess;
  (void)hipGetLastError();
  return flagcxUnhandledDeviceError;
}

inline flagcxResult_t ready(hipError_t e) {
  if (e == hipSuccess) return flagcxSuccess;
  if (e == hipErrorNotReady) {
    (void)hipGetLastError();  // a pending query is not a sticky error
    return flagcxInProgress;
  }
  return flagcxUnhandledDeviceError;
}

inline hipMemcpyKind kindOf(flagcxMemcpyType_t t) {
  switch (t) {
    case flagcxMemcpyHostToDevice: return hipMemcpyHostToDevice;
    case flagcxMemcpyDeviceToHost: return hipMemcpyDeviceToHost;
    case flagcxMemcpyDeviceToDevice: return hipMemcpyDeviceToDevice;
    default: return hipMemcpyDefault;
  }
}

flagcxResult_t fxDeviceSynchronize(void) { return dev(hipDeviceSynchronize()); }

// stream == NULL is a synchronous copy (hip_adaptor.cc:19-29).
flagcxResult_t fxDeviceMemcpy(void *dst, void *src, size_t size, flagcxMemcpyType_t type, flagcxStream_t stream,
                              void *) {
  if (size == 0) return flagcxSuccess;
  if (!dst || !src) return flagcxInvalidArgument;
  if (!stream) return dev(hipMemcpy(dst, src, size, kindOf(type)));
  return dev(hipMemcpyAsync(dst, src, size, kindOf(type), stream->base));
}

flagcxResult_t fxDeviceMemset(void *ptr, int value, size_t size, flagcxMemType_t type, flagcxStream_t stream) {
  if (size == 0) return flagcxSuccess;
  if (!ptr) return flagcxInvalidArgument;
  if (type == flagcxMemHost) {
    memset(ptr, value, size);
    return flagcxSuccess;
  }
  if (!stream) return dev(hipMemset(ptr, value, size));
  return dev(hipMemsetAsync(ptr, value, size, stream->base));
}

// flagcxMemHost is pinned AND mapped, so hostGetDevicePointer works on it
// (the CUDA adaptor does the same, flagcx/adaptor/device/cuda_adaptor.cc:56-57).
flagcxResult_t fxDeviceMalloc(void **ptr, size_t size, flagcxMemType_t type, flagcxStream_t stream) {
  if (!ptr) return flagcxInvalidArgument;
  switch (type) {
    case flagcxMemHost: return dev(hipHostMalloc(ptr, size, hipHostMallocMapped | hipHostMallocPortable));
    case flagcxMemManaged: return dev(hipMallocManaged(ptr, size, hipMemAttachGlobal));
    case flagcxMemDevice:
      if (stream) return dev(hipMallocAsync(ptr, size, stream->base));
      return dev(hipMalloc(ptr, size));
    default: return flagcxInvalidArgument;
  }
}

flagcxResult_t fxDeviceFree(void *ptr, flagcxMemType_t type, flagcxStream_t stream) {
  if (!ptr) return flagcxSuccess;
  switch (type) {
    case flagcxMemHost: return dev(hipHostFree(ptr));
    case flagcxMemManaged: return dev(hipFree(ptr));
    case flagcxMemDevice:
      if (stream) return dev(hipFreeAsync(ptr, stream->base));
      return dev(hipFree(ptr));
    default: return flagcxInvalidArgument;
  }
}

flagcxResult_t fxSetDevice(int d) { return dev(hipSetDevice(d)); }
flagcxResult_t fxGetDevice(int *d) { return d ? dev(hipGetDevice(d)) : flagcxInvalidArgument; }
flagcxResult_t fxGetDeviceCount(int *c) { return c ? dev(hipGetDeviceCount(c)) : flagcxInvalidArgument; }

flagcxResult_t fxGetVendor(char *vendor) {
  if (!vendor) return flagcxInvalidArgument;
  strncpy(vendor, FX_VENDOR_STRING, FX_MAX_VENDOR_LEN - 1);
  vendor[FX_MAX_VENDOR_LEN - 1] = '\0';
  return flagcxSuccess;
}

flagcxResult_t fxHostGetDevicePointer(void **pDevice, void *pHost) {
  if (!pDevice || !pHost) return flagcxInvalidArgument;
  return dev(hipHostGetDevicePointer(pDevice, pHost, 0));
}

// "GDR" memory: device memory a NIC may register.  Synchronous memory ops are
// requested so a peer never observes a half-finished memcpy.
flagcxResult_t fxGdrMemAlloc(void **ptr, size_t size, void *) {
  if (!ptr) return flagcxInvalidArgument;
  hipError_t e = hipMalloc(ptr, size);
  if (e != hipSuccess) return flagcxUnhandledDeviceError;
  unsigned int on = 1;
  if (hipPointerSetAttribute(&on, HIP_POINTER_ATTRIBUTE_SYNC_MEMOPS, (hipDeviceptr_t)*ptr) != hipSuccess)
    (void)hipGetLastError();  // advisory
  return flagcxSuccess;
}
flagcxResult_t fxGdrMemFree(void *ptr, void *) { return ptr ? dev(hipFree(ptr)) : flagcxSuccess; }

template <class T>
T *newHandle() {
  return static_cast<T *>(calloc(1, sizeof(T)));
}

flagcxResult_t fxStreamCreate(flagcxStream_t *stream) {
  if (!stream) return flagcxInvalidArgument;
  *stream = nullptr;
  flagcxStream *s = newHandle<flagcxStream>();
  if (!s) return flagcxSystemError;
  if (hipStreamCreateWithFlags(&s->base, hipStreamNonBlocking) != hipSuccess) {
    free(s);
    return flagcxUnhandledDeviceError;
  }
  *stream = s;
  return flagcxSuccess;
}

flagcxResult_t fxStreamDestroy(flagcxStream_t stream) {
  if (!stream) return flagcxSuccess;
  hipError_t e = hipStreamDestroy(stream->base);
  free(stream);
  return dev(e);
}

// Wrap a foreign hipStream_t without taking ownership; streamFree releases
// only the wrapper (hip_adaptor.cc:137-150).
flagcxResult_t fxStreamCopy(flagcxStream_t *newStream, void *oldStream) {
  if (!newStream) return flagcxInvalidArgument;
  flagcxStream *s = newHandle<flagcxStream>();
  if (!s) return flagcxSystemError;
  s->base = static_cast<hipStream_t>(oldStream);
  *newStream = s;
  return flagcxSuccess;
}

flagcxResult_t fxStreamFree(flagcxStream_t stream) {
  free(stream);
  return flagcxSuccess;
}

flagcxResult_t fxStreamSynchronize(flagcxStream_t stream) {
  return stream ? dev(hipStreamSynchronize(stream->base)) : flagcxSuccess;
}
flagcxResult_t fxStreamQuery(flagcxStream_t stream) {
  return stream ? ready(hipStreamQuery(stream->base)) : flagcxSuccess;
}
flagcxResult_t fxStreamWaitEvent(flagcxStream_t stream, flagcxEvent_t event) {
  if (!stream || !event) return flagcxSuccess;
  return dev(hipStreamWaitEvent(stream->base, event->base, 0));
}
flagcxResult_t fxStreamWaitValue64(flagcxStream_t stream, void *addr, uint64_t value, int flags) {
  if (!stream || !addr) return flagcxInvalidArgument;
  return dev(hipStreamWaitValue64(stream->base, addr, value, (unsigned int)flags, ~0ull));
}
flagcxResult_t fxStreamWriteValue64(flagcxStream_t stream, void *addr, uint64_t value, int flags) {
  if (!stream || !addr) return flagcxInvalidArgument;
  return dev(hipStreamWriteValue64(stream->base, addr, value, (unsigned int)flags));
}

flagcxResult_t fxEventCreate(flagcxEvent_t *event, flagcxEventType_t type) {
  if (!event) return flagcxInvalidArgument;
  *event = nullptr;
  flagcxEvent *e = newHandle<flagcxEvent>();
  if (!e) return flagcxSystemError;
  unsigned int flags = (type == flagcxEventDefault) ? hipEventDefault : hipEventDisableTiming;
  if (hipEventCreateWithFlags(&e->base, flags) != hipSuccess) {
    free(e);
    return flagcxUnhandledDeviceError;
  }
  *event = e;
  return flagcxSuccess;
}
flagcxResult_t fxEventDestroy(flagcxEvent_t event) {
  if (!event) return flagcxSuccess;
  hipError_t e = hipEventDestroy(event->base);
  free(event);
  return dev(e);
}
flagcxResult_t fxEventRecord(flagcxEvent_t event, flagcxStream_t stream) {
  if (!event || !stream) return flagcxSuccess;
  return dev(hipEventRecord(event->base, stream->base));
}
flagcxResult_t fxEventSynchronize(flagcxEvent_t event) {
  return event ? dev(hipEventSynchronize(event->base)) : flagcxSuccess;
}
flagcxResult_t fxEventQuery(flagcxEvent_t event) { return event ? ready(hipEventQuery(event->base)) : flagcxSuccess; }
flagcxResult_t fxEventElapsedTime(float *ms, flagcxEvent_t start, flagcxEvent_t end) {
  if (!ms || !start || !end) return flagcxInvalidArgument;
  return dev(hipEventElapsedTime(ms, start->base, end->base));
}

flagcxResult_t fxIpcMemHandleCreate(flagcxIpcMemHandle_t *handle, size_t *size) {
  if (!handle) return flagcxInvalidArgument;
  *handle = newHandle<flagcxIpcMemHandle>();
  if (!*handle) return flagcxSystemError;
  if (size) *size = sizeof(hipIpcMemHandle_t);
  return flagcxSuccess;
}
flagcxResult_t fxIpcMemHandleGet(flagcxIpcMemHandle_t handle, void *devPtr) {
  if (!handle || !devPtr) return flagcxInvalidArgument;
  return dev(hipIpcGetMemHandle(&handle->base, devPtr));
}
flagcxResult_t fxIpcMemHandleOpen(flagcxIpcMemHandle_t handle, void **devPtr) {
  if (!handle || !devPtr || *devPtr) return flagcxInvalidArgument;
  return dev(hipIpcOpenMemHandle(devPtr, handle->base, hipIpcMemLazyEnablePeerAccess));
}
flagcxResult_t fxIpcMemHandleClose(void *devPtr) {
  if (!devPtr) return flagcxInvalidArgument;
  return dev(hipIpcCloseMemHandle(devPtr));
}
flagcxResult_t fxIpcMemHandleFree(flagcxIpcMemHandle_t handle) {
  free(handle);
  return flagcxSuccess;
}

// A "device function" is a host function that enqueues work on the stream it
// is given (flagcx/core/group.cc:451-453 launches semaphore kernels this way).
flagcxResult_t fxLaunchDeviceFunc(flagcxStream_t stream, flagcxLaunchFunc_t fn, void *args) {
  if (!fn) return flagcxInvalidArgument;
  if (stream) fn(stream, args);
  return flagcxSuccess;
}

flagcxResult_t fxLaunchHostFunc(flagcxStream_t stream, void (*fn)(void *), void *args) {
  if (!fn) return flagcxInvalidArgument;
  if (!stream) return flagcxSuccess;
  return dev(hipLaunchHostFunc(stream->base, fn, args));
}

flagcxResult_t fxGetDeviceProperties(struct flagcxDevProps *props, int d) {
  if (!props) return flagcxInvalidArgument;
  hipDeviceProp_t p;
  if (hipGetDeviceProperties(&p, d) != hipSuccess) {
    (void)hipGetLastError();
    return flagcxUnhandledDeviceError;
  }
  // Some driver stacks report no marketing name; callers expect a non-empty
  // one, so fall back to the ISA name (e.g. "gfx950:sramecc+:xnack-").
  const char *nm = p.name[0] ? p.name : p.gcnArchName;
  strncpy(props->name, nm[0] ? nm : "AMD GPU", sizeof(props->name) - 1);
  props->name[sizeof(props->name) - 1] = '\0';
  props->pciBusId = p.pciBusID;
  props->pciDeviceId = p.pciDeviceID;
  props->pciDomainId = p.pciDomainID;
  return flagcxSuccess;
}

flagcxResult_t fxGetDevicePciBusId(char *pciBusId, int len, int d) {
  if (!pciBusId || len <= 0) return flagcxInvalidArgument;
  if (hipDeviceGetPCIBusId(pciBusId, len, d) != hipSuccess) {
    (void)hipGetLastError();
    return flagcxUnhandledDeviceError;
  }
  return flagcxSuccess;
}

flagcxResult_t fxGetDeviceByPciBusId(int *d, const char *pciBusId) {
  if (!d || !pciBusId) return flagcxInvalidArgument;
  if (hipDeviceGetByPCIBusId(d, pciBusId) != hipSuccess) {
    (void)hipGetLastError();
    return flagcxUnhandledDeviceError;
  }
  return flagcxSuccess;
}

flagcxResult_t fxDmaSupport(bool *dmaBufferSupport) {
  if (!dmaBufferSupport) return flagcxInvalidArgument;
  *dmaBufferSupport = false;
  return flagcxSuccess;
}

flagcxResult_t fxGetHandleForAddressRange(void *, void *, size_t, unsigned long long) { return flagcxNotSupported; }

}  // namespace

extern "C" __attribute__((visibility("default"))) struct flagcxDeviceAdaptor_v1 flagcxDeviceAdaptorPlugin_v1 = {
    FX_DEVICE_ADAPTOR_NAME,
    // basic
    fxDeviceSynchronize, fxDeviceMemcpy, fxDeviceMemset, fxDeviceMalloc, fxDeviceFree, fxSetDevice, fxGetDevice,
    fxGetDeviceCount, fxGetVendor, fxHostGetDevicePointer,
    // GDR: only alloc/free are meaningful without a NIC
    nullptr, nullptr, fxGdrMemAlloc, fxGdrMemFree, nullptr, nullptr, nullptr, nullptr,
    // stream
    fxStreamCreate, fxStreamDestroy, fxStreamCopy, fxStreamFree, fxStreamSynchronize, fxStreamQuery,
    fxStreamWaitEvent, fxStreamWaitValue64, fxStreamWriteValue64,
    // event
    fxEventCreate, fxEventDestroy, fxEventRecord, fxEventSynchronize, fxEventQuery, fxEventElapsedTime,
    // IPC
    fxIpcMemHandleCreate, fxIpcMemHandleGet, fxIpcMemHandleOpen, fxIpcMemHandleClose, fxIpcMemHandleFree,
    // kernel launch: kernels are launched by the library itself, never through a generic hook
    nullptr, nullptr, nullptr, fxLaunchDeviceFunc,
    // others
    fxGetDeviceProperties, fxGetDevicePciBusId, fxGetDeviceByPciBusId,
    fxLaunchHostFunc,
    fxDmaSupport, fxGetHandleForAddressRange,
};
