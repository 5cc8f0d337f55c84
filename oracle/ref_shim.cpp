// ref_shim.cpp - C entry points around the reference's OWN reduce templates.
//
// TEST INFRASTRUCTURE ONLY.  Built only where /root/reference exists, by
// oracle/Makefile, into oracle/_ref/libflagcx_ref.so.  It includes the reference's
// flagcx/service/utils.h from where it lies and instantiates sum<T>, min<T>, max<T>
// (utils.h:681-709) for the eight types GENERATE_ALL_TYPES (utils.h:648-679)
// accepts.  The dtype switch is written out here instead of using that macro
// because its default branch logs through flagcxDebugLog, whose translation unit
// drags in the bootstrap, adaptor and socket code; nothing of the reference is
// stubbed or replaced.  The op switch follows flagcx/service/bootstrap.cc:649-671.
#include "utils.h"

#define DISPATCH(FN)                                                           \
  switch (dtype) {                                                             \
    case flagcxInt8:    FN<char>(res, op1, op2, n); break;                     \
    case flagcxUint8:   FN<unsigned char>(res, op1, op2, n); break;            \
    case flagcxInt32:   FN<int32_t>(res, op1, op2, n); break;                  \
    case flagcxUint32:  FN<uint32_t>(res, op1, op2, n); break;                 \
    case flagcxInt64:   FN<int64_t>(res, op1, op2, n); break;                  \
    case flagcxUint64:  FN<uint64_t>(res, op1, op2, n); break;                 \
    case flagcxFloat:   FN<float>(res, op1, op2, n); break;                    \
    case flagcxFloat64: FN<double>(res, op1, op2, n); break;                   \
    default: return flagcxInvalidArgument;                                     \
  }

extern "C" int ref_binary(int op, int dtype, void *res, const void *op1,
                          const void *op2, size_t n) {
  switch (op) {
    case flagcxSum: DISPATCH(sum) break;
    case flagcxMax: DISPATCH(max) break;
    case flagcxMin: DISPATCH(min) break;
    default: return flagcxInvalidArgument;
  }
  return flagcxSuccess;
}

// Enum values as the reference's headers define them, for the ABI test.
extern "C" int ref_enum(const char *name) {
#define E(x) if (!strcmp(name, #x)) return (int)x;
  E(flagcxSuccess) E(flagcxUnhandledDeviceError) E(flagcxSystemError)
  E(flagcxInternalError) E(flagcxInvalidArgument) E(flagcxInvalidUsage)
  E(flagcxRemoteError) E(flagcxInProgress) E(flagcxUnhandledCCLError)
  E(flagcxNotSupported) E(flagcxInt8) E(flagcxUint8) E(flagcxInt32)
  E(flagcxUint32) E(flagcxInt64) E(flagcxUint64) E(flagcxFloat16) E(flagcxFloat)
  E(flagcxFloat64) E(flagcxBfloat16) E(flagcxSum) E(flagcxProd) E(flagcxMax)
  E(flagcxMin) E(flagcxAvg) E(flagcxCommOpReduce) E(flagcxCommOpAllReduce)
  E(flagcxCommOpReduceScatter) E(flagcxMemcpyDeviceToDevice)
#undef E
  return -1;
}

// Layout of the reference's device-adaptor table as ITS header defines it
// (flagcx/adaptor/include/adaptor.h:145-233): sizeof, every member offset in
// declaration order, sizeof(struct flagcxDevProps).
#include "adaptor.h"
#include <cstddef>
extern "C" int ref_adaptor_layout(size_t *out, int cap) {
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
