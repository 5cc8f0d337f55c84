// fifo_kernels.hip - the reference's device-producer / host-consumer trigger FIFO
// for gfx950.
//
// Layout and protocol are the reference's: a pinned host buffer of 64-bit words
// [capacity, consumed, produced, entries...] with 16-byte entries {fst, snd},
// fst = address, snd = count[0,32) | peerRank[32,52) | datatype[52,56) | prim[56,60)
// (flagcx/include/flagcx_kernel.h:7-49,75-88); the device appends an entry, fences
// to system scope and then bumps `produced`
// (flagcx/kernels/flagcx_kernel_device.cu:53-124); the host copies the entry at
// `consumed` out and bumps `consumed` (flagcx/core/flagcx_kernel_host.cc:52-73).
// Allocation mirrors flagcxFifo::flagcxFifoInit (flagcx_kernel_host.cc:31-45).
// The single-lane demo kernel is the shape of flagcxP2pKernel
// (flagcx/kernels/device_collective_demo.cu:5-34): Send, Recv, Term, Wait.
//
// Difference: every device-side wait (queue full, Wait for the host to drain) is
// bounded by the spin limit that also bounds deviceAsyncLoad, so a host that
// never dequeues cannot wedge the GPU.
#include "../../include/flagcx_amd.h"

#include <hip/hip_runtime.h>

#include <cstring>

namespace flagcx_amd {

long long asyncMaxSpin(); // async_kernels.hip

__device__ __forceinline__ unsigned long long sysLoad(const unsigned long long *p) {
  return __hip_atomic_load(p, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_SYSTEM);
}
__device__ __forceinline__ void sysStore(unsigned long long *p, unsigned long long v) {
  __hip_atomic_store(p, v, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}

// Appends one trigger; returns false if the queue stayed full for maxSpin polls.
__device__ bool fifoEnqueue(unsigned long long *buffer, unsigned long long addr, unsigned long long count,
                            unsigned long long peerRank, unsigned long long datatype, unsigned long long prim,
                            long long maxSpin) {
  const unsigned long long capacity = sysLoad(buffer + 0);
  unsigned long long produced = sysLoad(buffer + 2);
  long long spins = 0;
  while (produced - sysLoad(buffer + 1) >= capacity) {
    if (++spins > maxSpin) return false;
    __builtin_amdgcn_s_sleep(32);
  }
  unsigned long long *entry = buffer + 3 + 2 * (produced % capacity);
  const unsigned long long snd = (count & 0xffffffffull) | ((peerRank & 0xfffffull) << 32) |
                                 ((datatype & 0xfull) << 52) | ((prim & 0xfull) << 56);
  sysStore(entry + 0, addr);
  sysStore(entry + 1, snd);
  __threadfence_system();
  sysStore(buffer + 2, produced + 1);
  return true;
}

// Waits (bounded) until the host has consumed everything produced so far.
__device__ bool fifoDrain(unsigned long long *buffer, long long maxSpin) {
  long long spins = 0;
  while (sysLoad(buffer + 2) != sysLoad(buffer + 1)) {
    if (++spins > maxSpin) return false;
    __builtin_amdgcn_s_sleep(32);
  }
  return true;
}

__global__ void p2pDemoKernel(const void *sendbuff, void *recvbuff, unsigned long long count, int datatype,
                              int sendPeer, int recvPeer, unsigned long long *fifo, long long maxSpin) {
  if (threadIdx.x != 0 || blockIdx.x != 0) return;
  bool ok = fifoEnqueue(fifo, (unsigned long long)(uintptr_t)sendbuff, count, (unsigned)sendPeer,
                        (unsigned)datatype, FLAGCX_LOCAL_PRIM_SEND, maxSpin);
  ok = ok && fifoEnqueue(fifo, (unsigned long long)(uintptr_t)recvbuff, count, (unsigned)recvPeer,
                         (unsigned)datatype, FLAGCX_LOCAL_PRIM_RECV, maxSpin);
  ok = ok && fifoEnqueue(fifo, 0, 0, 0, 0, FLAGCX_LOCAL_PRIM_TERM, maxSpin);
  ok = ok && fifoEnqueue(fifo, 0, 0, 0, 0, FLAGCX_LOCAL_PRIM_WAIT, maxSpin);
  if (ok) fifoDrain(fifo, maxSpin);
}

} // namespace flagcx_amd

using namespace flagcx_amd;

#pragma GCC visibility push(default)
extern "C" {

flagcxResult_t flagcxLocalFifoInit(void **fifoBuffer) {
  if (!fifoBuffer) return flagcxInvalidArgument;
  const size_t bytes = 3 * sizeof(uint64_t) + FLAGCX_LOCAL_FIFO_CAPACITY * sizeof(flagcxLocalDeviceTrigger);
  void *p = nullptr;
  if (hipHostMalloc(&p, bytes, hipHostMallocMapped) != hipSuccess) return flagcxUnhandledDeviceError;
  uint64_t *b = static_cast<uint64_t *>(p);
  memset(p, 0, bytes);
  b[0] = FLAGCX_LOCAL_FIFO_CAPACITY;
  *fifoBuffer = p;
  return flagcxSuccess;
}

flagcxResult_t flagcxLocalFifoDestroy(void *fifoBuffer) {
  if (!fifoBuffer) return flagcxSuccess;
  return hipHostFree(fifoBuffer) == hipSuccess ? flagcxSuccess : flagcxUnhandledDeviceError;
}

flagcxResult_t flagcxLocalFifoDequeue(void *fifoBuffer, flagcxLocalDeviceTrigger *trigger) {
  if (!fifoBuffer || !trigger) return flagcxInvalidArgument;
  volatile uint64_t *buffer = static_cast<volatile uint64_t *>(fifoBuffer);
  const uint64_t capacity = buffer[0];
  const uint64_t cons = buffer[1];
  const uint64_t prod = __atomic_load_n(&buffer[2], __ATOMIC_ACQUIRE);
  if (prod > cons && capacity) {
    const uint64_t idx = cons % capacity;
    trigger->fst = buffer[3 + 2 * idx];
    trigger->snd = buffer[3 + 2 * idx + 1];
    __atomic_store_n(&buffer[1], cons + 1, __ATOMIC_RELEASE);
  } else {
    trigger->fst = 0; // an empty queue yields a zero trigger, as in the reference
    trigger->snd = 0;
  }
  return flagcxSuccess;
}

flagcxResult_t flagcxLocalP2pDemo(const void *sendbuff, void *recvbuff, size_t count,
                                  flagcxDataType_t datatype, int sendPeer, int recvPeer, void *fifoBuffer,
                                  flagcxStream_t stream) {
  if (!fifoBuffer) return flagcxInvalidArgument;
  hipStream_t s = stream ? *reinterpret_cast<hipStream_t *>(stream) : nullptr;
  p2pDemoKernel<<<1, 1, 0, s>>>(sendbuff, recvbuff, (unsigned long long)count, (int)datatype, sendPeer, recvPeer,
                                static_cast<unsigned long long *>(fifoBuffer), asyncMaxSpin());
  return hipGetLastError() == hipSuccess ? flagcxSuccess : flagcxUnhandledDeviceError;
}

} // extern "C"
#pragma GCC visibility pop
