// host_device_adaptor.cpp - HIP implementations behind every slot of the
// reference's device-adaptor table (flagcx/adaptor/include/adaptor.h:145-233),
// written against that interface; conventions followed:
//   - any runtime error -> flagcxUnhandledDeviceError (DEVCHECK,
//     flagcx/adaptor/include/amd_adaptor.h:26-31); "not ready" from a query ->
//     flagcxInProgress;
//   - a NULL stream means the blocking form of the call;
//   - streams are created non-blocking; streamCopy wraps a foreign stream without
//     owning it and streamFree releases only the wrapper;
//   - struct flagcxStream / flagcxEvent hold the HIP handle as first member
//     (amd_adaptor.h:14-20).
// Device-to-device copies and device memsets run on this library's kernels.
#include "../../include/flagcx_amd_adaptor.h"

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdlib>
#include <cstring>

struct flagcxStream { hipStream_t base; };
struct flagcxEvent { hipEvent_t base; };
struct flagcxIpcMemHandle { hipIpcMemHandle_t base; };

namespace {

#define DEV(call)                                                              \
  do {                                                                         \
    if ((call) != hipSuccess) return flagcxUnhandledDeviceError;               \
  } while (0)

inline hipStream_t hs(flagcxStream_t s) { return s ? s->base : nullptr; }

// Enum arguments come from C callers and may hold any int: read their bits.
template <typename E>
inline int bitsOf(const E &e) {
  static_assert(sizeof(E) == sizeof(int), "flagcx enums are int sized");
  int v;
  memcpy(&v, &e, sizeof(v));
  return v;
}

flagcxResult_t aDeviceSynchronize(void) { DEV(hipDeviceSynchronize()); return flagcxSuccess; }

flagcxResult_t aDeviceMemcpy(void *dst, void *src, size_t size, flagcxMemcpyType_t type_, flagcxStream_t stream,
                             void *) {
  const int type = bitsOf(type_);
  if (type == flagcxMemcpyDeviceToDevice) return flagcxLocalMemcpy(dst, src, size, stream);
  const hipMemcpyKind kind = type == flagcxMemcpyHostToDevice ? hipMemcpyHostToDevice : hipMemcpyDeviceToHost;
  if (type != flagcxMemcpyHostToDevice && type != flagcxMemcpyDeviceToHost) return flagcxInvalidArgument;
  if (stream) DEV(hipMemcpyAsync(dst, src, size, kind, stream->base));
  else DEV(hipMemcpy(dst, src, size, kind));
  return flagcxSuccess;
}

flagcxResult_t aDeviceMemset(void *ptr, int value, size_t size, flagcxMemType_t type, flagcxStream_t stream) {
  if (bitsOf(type) == flagcxMemHost) {
    if (!ptr && size) return flagcxInvalidArgument;
    memset(ptr, value, size);
    return flagcxSuccess;
  }
  return flagcxLocalMemset(ptr, value, size, stream);
}

flagcxResult_t aDeviceMalloc(void **ptr, size_t size, flagcxMemType_t type, flagcxStream_t stream) {
  if (!ptr) return flagcxInvalidArgument;
  switch (bitsOf(type)) {
    case flagcxMemHost: DEV(hipHostMalloc(ptr, size, hipHostMallocMapped)); break;
    case flagcxMemManaged: DEV(hipMallocManaged(ptr, size, hipMemAttachGlobal)); break;
    case flagcxMemDevice:
      if (stream) DEV(hipMallocAsync(ptr, size, stream->base));
      else DEV(hipMalloc(ptr, size));
      break;
    default: return flagcxInvalidArgument;
  }
  return flagcxSuccess;
}

flagcxResult_t aDeviceFree(void *ptr, flagcxMemType_t type_, flagcxStream_t stream) {
  if (!ptr) return flagcxSuccess;
  const int type = bitsOf(type_);
  if (type == flagcxMemHost) DEV(hipHostFree(ptr));
  else if (type == flagcxMemDevice && stream) DEV(hipFreeAsync(ptr, stream->base));
  else DEV(hipFree(ptr));
  return flagcxSuccess;
}

flagcxResult_t aSetDevice(int dev) { DEV(hipSetDevice(dev)); return flagcxSuccess; }
flagcxResult_t aGetDevice(int *dev) { if (!dev) return flagcxInvalidArgument; DEV(hipGetDevice(dev)); return flagcxSuccess; }
flagcxResult_t aGetDeviceCount(int *n) { if (!n) return flagcxInvalidArgument; DEV(hipGetDeviceCount(n)); return flagcxSuccess; }
flagcxResult_t aGetVendor(char *vendor) { if (!vendor) return flagcxInvalidArgument; strcpy(vendor, "AMD"); return flagcxSuccess; }
flagcxResult_t aHostGetDevicePointer(void **pDevice, void *pHost) {
  if (!pDevice || !pHost) return flagcxInvalidArgument;
  DEV(hipHostGetDevicePointer(pDevice, pHost, 0));
  return flagcxSuccess;
}

flagcxResult_t aGdrMemAlloc(void **ptr, size_t size, void *) {
  if (!ptr) return flagcxInvalidArgument;
  DEV(hipMalloc(ptr, size));
  return flagcxSuccess;
}
flagcxResult_t aGdrMemFree(void *ptr, void *) {
  if (!ptr) return flagcxSuccess;
  DEV(hipFree(ptr));
  return flagcxSuccess;
}

flagcxResult_t aStreamCreate(flagcxStream_t *stream) {
  if (!stream) return flagcxInvalidArgument;
  flagcxStream_t s = static_cast<flagcxStream_t>(calloc(1, sizeof(struct flagcxStream)));
  if (!s) return flagcxSystemError;
  if (hipStreamCreateWithFlags(&s->base, hipStreamNonBlocking) != hipSuccess) { free(s); return flagcxUnhandledDeviceError; }
  *stream = s;
  return flagcxSuccess;
}
flagcxResult_t aStreamDestroy(flagcxStream_t stream) {
  if (!stream) return flagcxSuccess;
  hipError_t e = hipStreamDestroy(stream->base);
  free(stream);
  return e == hipSuccess ? flagcxSuccess : flagcxUnhandledDeviceError;
}
flagcxResult_t aStreamCopy(flagcxStream_t *newStream, void *oldStream) {
  if (!newStream || !oldStream) return flagcxInvalidArgument;
  flagcxStream_t s = static_cast<flagcxStream_t>(calloc(1, sizeof(struct flagcxStream)));
  if (!s) return flagcxSystemError;
  s->base = *static_cast<hipStream_t *>(oldStream); // the caller passes &its_stream
  *newStream = s;
  return flagcxSuccess;
}
flagcxResult_t aStreamFree(flagcxStream_t stream) { free(stream); return flagcxSuccess; }
flagcxResult_t aStreamSynchronize(flagcxStream_t stream) { DEV(hipStreamSynchronize(hs(stream))); return flagcxSuccess; }
flagcxResult_t aStreamQuery(flagcxStream_t stream) {
  hipError_t e = hipStreamQuery(hs(stream));
  if (e == hipSuccess) return flagcxSuccess;
  if (e == hipErrorNotReady) { (void)hipGetLastError(); return flagcxInProgress; }
  return flagcxUnhandledDeviceError;
}
flagcxResult_t aStreamWaitEvent(flagcxStream_t stream, flagcxEvent_t event) {
  if (!event) return flagcxInvalidArgument;
  DEV(hipStreamWaitEvent(hs(stream), event->base, 0));
  return flagcxSuccess;
}

flagcxResult_t aEventCreate(flagcxEvent_t *event, flagcxEventType_t type) {
  if (!event) return flagcxInvalidArgument;
  flagcxEvent_t e = static_cast<flagcxEvent_t>(calloc(1, sizeof(struct flagcxEvent)));
  if (!e) return flagcxSystemError;
  const unsigned flags = bitsOf(type) == flagcxEventDisableTiming ? hipEventDisableTiming : hipEventDefault;
  if (hipEventCreateWithFlags(&e->base, flags) != hipSuccess) { free(e); return flagcxUnhandledDeviceError; }
  *event = e;
  return flagcxSuccess;
}
flagcxResult_t aEventDestroy(flagcxEvent_t event) {
  if (!event) return flagcxSuccess;
  hipError_t e = hipEventDestroy(event->base);
  free(event);
  return e == hipSuccess ? flagcxSuccess : flagcxUnhandledDeviceError;
}
flagcxResult_t aEventRecord(flagcxEvent_t event, flagcxStream_t stream) {
  if (!event) return flagcxInvalidArgument;
  DEV(hipEventRecord(event->base, hs(stream)));
  return flagcxSuccess;
}
flagcxResult_t aEventSynchronize(flagcxEvent_t event) {
  if (!event) return flagcxInvalidArgument;
  DEV(hipEventSynchronize(event->base));
  return flagcxSuccess;
}
flagcxResult_t aEventQuery(flagcxEvent_t event) {
  if (!event) return flagcxInvalidArgument;
  hipError_t e = hipEventQuery(event->base);
  if (e == hipSuccess) return flagcxSuccess;
  if (e == hipErrorNotReady) { (void)hipGetLastError(); return flagcxInProgress; }
  return flagcxUnhandledDeviceError;
}
flagcxResult_t aEventElapsedTime(float *ms, flagcxEvent_t start, flagcxEvent_t end) {
  if (!ms || !start || !end) return flagcxInvalidArgument;
  hipError_t e = hipEventElapsedTime(ms, start->base, end->base);
  if (e == hipSuccess) return flagcxSuccess;
  if (e == hipErrorNotReady) { (void)hipGetLastError(); return flagcxInProgress; }
  return flagcxUnhandledDeviceError;
}

flagcxResult_t aIpcCreate(flagcxIpcMemHandle_t *handle, size_t *size) {
  if (!handle) return flagcxInvalidArgument;
  *handle = static_cast<flagcxIpcMemHandle_t>(calloc(1, sizeof(struct flagcxIpcMemHandle)));
  if (!*handle) return flagcxSystemError;
  if (size) *size = sizeof(hipIpcMemHandle_t);
  return flagcxSuccess;
}
flagcxResult_t aIpcGet(flagcxIpcMemHandle_t handle, void *devPtr) {
  if (!handle || !devPtr) return flagcxInvalidArgument;
  DEV(hipIpcGetMemHandle(&handle->base, devPtr));
  return flagcxSuccess;
}
flagcxResult_t aIpcOpen(flagcxIpcMemHandle_t handle, void **devPtr) {
  if (!handle || !devPtr || *devPtr) return flagcxInvalidArgument;
  DEV(hipIpcOpenMemHandle(devPtr, handle->base, hipIpcMemLazyEnablePeerAccess));
  return flagcxSuccess;
}
flagcxResult_t aIpcClose(void *devPtr) {
  if (!devPtr) return flagcxInvalidArgument;
  DEV(hipIpcCloseMemHandle(devPtr));
  return flagcxSuccess;
}
flagcxResult_t aIpcFree(flagcxIpcMemHandle_t handle) { free(handle); return flagcxSuccess; }

flagcxResult_t aLaunchDeviceFunc(flagcxStream_t stream, flagcxLaunchFunc_t fn, void *args) {
  if (!fn) return flagcxInvalidArgument;
  if (stream) fn(stream, args);
  return flagcxSuccess;
}
flagcxResult_t aLaunchHostFunc(flagcxStream_t stream, void (*fn)(void *), void *args) {
  if (!fn) return flagcxInvalidArgument;
  DEV(hipLaunchHostFunc(hs(stream), fn, args));
  return flagcxSuccess;
}

flagcxResult_t aGetDeviceProperties(struct flagcxDevProps *props, int dev) {
  if (!props) return flagcxInvalidArgument;
  hipDeviceProp_t p;
  DEV(hipGetDeviceProperties(&p, dev));
  strncpy(props->name, p.name, sizeof(props->name) - 1);
  props->name[sizeof(props->name) - 1] = '\0';
  props->pciBusId = p.pciBusID;
  props->pciDeviceId = p.pciDeviceID;
  props->pciDomainId = p.pciDomainID;
  return flagcxSuccess;
}
flagcxResult_t aGetDevicePciBusId(char *pciBusId, int len, int dev) {
  if (!pciBusId || len <= 0) return flagcxInvalidArgument;
  DEV(hipDeviceGetPCIBusId(pciBusId, len, dev));
  return flagcxSuccess;
}
flagcxResult_t aGetDeviceByPciBusId(int *dev, const char *pciBusId) {
  if (!dev || !pciBusId) return flagcxInvalidArgument;
  DEV(hipDeviceGetByPCIBusId(dev, pciBusId));
  return flagcxSuccess;
}
flagcxResult_t aDmaSupport(bool *dmaBufferSupport) {
  if (!dmaBufferSupport) return flagcxInvalidArgument;
  *dmaBufferSupport = false; // no dma-buf export is wired up in this table
  return flagcxSuccess;
}
flagcxResult_t aGetHandleForAddressRange(void *, void *, size_t, unsigned long long) { return flagcxNotSupported; }

} // namespace

#pragma GCC visibility push(default)
extern "C" {

struct flagcxDeviceAdaptor flagcxLocalHipAdaptor = {
    "HIP",
    aDeviceSynchronize, aDeviceMemcpy, aDeviceMemset, aDeviceMalloc, aDeviceFree, aSetDevice, aGetDevice,
    aGetDeviceCount, aGetVendor, aHostGetDevicePointer,
    nullptr, nullptr, aGdrMemAlloc, aGdrMemFree, nullptr, nullptr, nullptr, nullptr,
    aStreamCreate, aStreamDestroy, aStreamCopy, aStreamFree, aStreamSynchronize, aStreamQuery, aStreamWaitEvent,
    aEventCreate, aEventDestroy, aEventRecord, aEventSynchronize, aEventQuery,
    aIpcCreate, aIpcGet, aIpcOpen, aIpcClose, aIpcFree,
    nullptr, nullptr, nullptr, aLaunchDeviceFunc,
    aGetDeviceProperties, aGetDevicePciBusId, aGetDeviceByPciBusId,
    aLaunchHostFunc,
    aDmaSupport, aGetHandleForAddressRange,
    aEventElapsedTime,
};

struct flagcxDeviceAdaptor *flagcxLocalGetDeviceAdaptor(void) { return &flagcxLocalHipAdaptor; }

int flagcxLocalDeviceAdaptorLayout(size_t *out, int cap) {
#define O(m) offsetof(struct flagcxDeviceAdaptor, m),
  const size_t v[] = {sizeof(struct flagcxDeviceAdaptor),
      O(name) O(deviceSynchronize) O(deviceMemcpy) O(deviceMemset) O(deviceMalloc) O(deviceFree) O(setDevice)
      O(getDevice) O(getDeviceCount) O(getVendor) O(hostGetDevicePointer) O(memHandleInit) O(memHandleDestroy)
      O(gdrMemAlloc) O(gdrMemFree) O(hostShareMemAlloc) O(hostShareMemFree) O(gdrPtrMmap) O(gdrPtrMunmap)
      O(streamCreate) O(streamDestroy) O(streamCopy) O(streamFree) O(streamSynchronize) O(streamQuery)
      O(streamWaitEvent) O(eventCreate) O(eventDestroy) O(eventRecord) O(eventSynchronize) O(eventQuery)
      O(ipcMemHandleCreate) O(ipcMemHandleGet) O(ipcMemHandleOpen) O(ipcMemHandleClose) O(ipcMemHandleFree)
      O(launchKernel) O(copyArgsInit) O(copyArgsFree) O(launchDeviceFunc) O(getDeviceProperties)
      O(getDevicePciBusId) O(getDeviceByPciBusId) O(launchHostFunc) O(dmaSupport) O(getHandleForAddressRange)
      O(eventElapsedTime) sizeof(struct flagcxDevProps)};
#undef O
  const int n = (int)(sizeof(v) / sizeof(v[0]));
  for (int i = 0; i < n && i < cap; i++) out[i] = v[i];
  return n;
}

} // extern "C"
#pragma GCC visibility pop
