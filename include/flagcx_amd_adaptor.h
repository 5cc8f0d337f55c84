/*
 * flagcx_amd_adaptor.h - a complete HIP device-adaptor table for the reference's
 * adaptor layer.
 *
 * struct flagcxDeviceAdaptor below has the member order and types of
 * flagcx/adaptor/include/adaptor.h:145-233 (the table deviceAdaptor points at,
 * flagcx/adaptor/adaptor.cc:109-120); every slot the reference's own table for
 * NVIDIA fills (flagcx/adaptor/device/cuda_adaptor.cc:453-510) is filled here for
 * HIP, including hostGetDevicePointer and eventElapsedTime, which the reference's
 * hip table leaves out.  Device-to-device copies and device memsets go through
 * this library's kernels.  If the reference's adaptor.h was included first its
 * definitions are used.
 */
#ifndef FLAGCX_AMD_ADAPTOR_H_
#define FLAGCX_AMD_ADAPTOR_H_

#include "flagcx_amd.h"
#include <stdbool.h>

#ifdef __cplusplus
extern "C" {
#endif

#ifndef FLAGCX_ADAPTOR_H_

typedef enum { flagcxMemHost = 0, flagcxMemDevice = 1, flagcxMemManaged = 2 } flagcxMemType_t; /* flagcx.h:84-88 */
typedef enum { flagcxEventDefault = 0, flagcxEventDisableTiming = 1 } flagcxEventType_t;      /* flagcx.h:90-93 */
typedef struct flagcxEvent *flagcxEvent_t;
typedef struct flagcxIpcMemHandle *flagcxIpcMemHandle_t;
typedef void (*flagcxLaunchFunc_t)(flagcxStream_t, void *); /* adaptor.h:15 */

struct flagcxDevProps { /* flagcx/core/topo.h:214-221 */
  char name[256];
  int pciBusId;
  int pciDeviceId;
  int pciDomainId;
};

struct flagcxDeviceAdaptor {
  char name[32];
  /* basic */
  flagcxResult_t (*deviceSynchronize)(void);
  flagcxResult_t (*deviceMemcpy)(void *dst, void *src, size_t size, flagcxMemcpyType_t type,
                                 flagcxStream_t stream, void *args);
  flagcxResult_t (*deviceMemset)(void *ptr, int value, size_t size, flagcxMemType_t type, flagcxStream_t stream);
  flagcxResult_t (*deviceMalloc)(void **ptr, size_t size, flagcxMemType_t type, flagcxStream_t stream);
  flagcxResult_t (*deviceFree)(void *ptr, flagcxMemType_t type, flagcxStream_t stream);
  flagcxResult_t (*setDevice)(int dev);
  flagcxResult_t (*getDevice)(int *dev);
  flagcxResult_t (*getDeviceCount)(int *count);
  flagcxResult_t (*getVendor)(char *vendor);
  flagcxResult_t (*hostGetDevicePointer)(void **pDevice, void *pHost);
  /* GDR */
  flagcxResult_t (*memHandleInit)(int dev_id, void **memHandle);
  flagcxResult_t (*memHandleDestroy)(int dev, void *memHandle);
  flagcxResult_t (*gdrMemAlloc)(void **ptr, size_t size, void *memHandle);
  flagcxResult_t (*gdrMemFree)(void *ptr, void *memHandle);
  flagcxResult_t (*hostShareMemAlloc)(void **ptr, size_t size, void *memHandle);
  flagcxResult_t (*hostShareMemFree)(void *ptr, void *memHandle);
  flagcxResult_t (*gdrPtrMmap)(void **pcpuptr, void *devptr, size_t sz);
  flagcxResult_t (*gdrPtrMunmap)(void *cpuptr, size_t sz);
  /* streams */
  flagcxResult_t (*streamCreate)(flagcxStream_t *stream);
  flagcxResult_t (*streamDestroy)(flagcxStream_t stream);
  flagcxResult_t (*streamCopy)(flagcxStream_t *newStream, void *oldStream);
  flagcxResult_t (*streamFree)(flagcxStream_t stream);
  flagcxResult_t (*streamSynchronize)(flagcxStream_t stream);
  flagcxResult_t (*streamQuery)(flagcxStream_t stream);
  flagcxResult_t (*streamWaitEvent)(flagcxStream_t stream, flagcxEvent_t event);
  /* events */
  flagcxResult_t (*eventCreate)(flagcxEvent_t *event, flagcxEventType_t eventType);
  flagcxResult_t (*eventDestroy)(flagcxEvent_t event);
  flagcxResult_t (*eventRecord)(flagcxEvent_t event, flagcxStream_t stream);
  flagcxResult_t (*eventSynchronize)(flagcxEvent_t event);
  flagcxResult_t (*eventQuery)(flagcxEvent_t event);
  /* IPC memory handles */
  flagcxResult_t (*ipcMemHandleCreate)(flagcxIpcMemHandle_t *handle, size_t *size);
  flagcxResult_t (*ipcMemHandleGet)(flagcxIpcMemHandle_t handle, void *devPtr);
  flagcxResult_t (*ipcMemHandleOpen)(flagcxIpcMemHandle_t handle, void **devPtr);
  flagcxResult_t (*ipcMemHandleClose)(void *devPtr);
  flagcxResult_t (*ipcMemHandleFree)(flagcxIpcMemHandle_t handle);
  /* kernel launch */
  flagcxResult_t (*launchKernel)(void *func, unsigned int block_x, unsigned int block_y, unsigned int block_z,
                                 unsigned int grid_x, unsigned int grid_y, unsigned int grid_z, void **args,
                                 size_t share_mem, void *stream, void *memHandle);
  flagcxResult_t (*copyArgsInit)(void **args);
  flagcxResult_t (*copyArgsFree)(void *args);
  flagcxResult_t (*launchDeviceFunc)(flagcxStream_t stream, flagcxLaunchFunc_t fn, void *args);
  /* topology helpers */
  flagcxResult_t (*getDeviceProperties)(struct flagcxDevProps *props, int dev);
  flagcxResult_t (*getDevicePciBusId)(char *pciBusId, int len, int dev);
  flagcxResult_t (*getDeviceByPciBusId)(int *dev, const char *pciBusId);
  /* host function launch */
  flagcxResult_t (*launchHostFunc)(flagcxStream_t stream, void (*fn)(void *), void *args);
  /* DMA buffer */
  flagcxResult_t (*dmaSupport)(bool *dmaBufferSupport);
  flagcxResult_t (*getHandleForAddressRange)(void *handleOut, void *buffer, size_t size, unsigned long long flags);
  /* event timing */
  flagcxResult_t (*eventElapsedTime)(float *ms, flagcxEvent_t start, flagcxEvent_t end);
};

#endif /* FLAGCX_ADAPTOR_H_ */

/* The table.  Slots the reference leaves NULL for every vendor (memHandleInit /
 * Destroy, hostShareMem*, gdrPtrMmap / Munmap, launchKernel, copyArgs*) are NULL
 * here too. */
extern struct flagcxDeviceAdaptor flagcxLocalHipAdaptor;
struct flagcxDeviceAdaptor *flagcxLocalGetDeviceAdaptor(void);

/* sizeof(struct flagcxDeviceAdaptor), the offset of every member in declaration
 * order, then sizeof(struct flagcxDevProps): lets a binder (and this build's
 * tests) check the layout against the reference's header.  Returns the number of
 * values; writes at most cap. */
int flagcxLocalDeviceAdaptorLayout(size_t *out, int cap);

#ifdef __cplusplus
}
#endif
#endif
