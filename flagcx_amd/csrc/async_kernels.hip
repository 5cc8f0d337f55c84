// async_kernels.hip - the two flag kernels a FLAGCX_DEVICE_FUNC_PATH library must
// export (flagcx/flagcx.cc:552-562 loads "deviceAsyncLoad" and "deviceAsyncStore"
// with dlsym and exits if either is missing).  Their reference versions are
// flagcx/kernels/device_async_kernel.dev:4-23: store sets a device bool, load
// spins until it is set.  Here the wait is bounded: after maxSpin polls the
// kernel gives up and exits, so a flag the host never sets cannot wedge the
// queue.  The bound comes from FLAGCX_FUNC_MAX_SPIN_COUNT, the variable that
// bounds the reference's host-side spin (flagcx/core/launch_kernel.cc:8-9,42-49),
// or from flagcxLocalSetMaxSpinCount; the default is 2^27 polls (minutes).
#include "../../include/flagcx_amd.h"

#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdlib>

namespace flagcx_amd {

__global__ void asyncStoreKernel(unsigned char *value) {
  __hip_atomic_store(value, (unsigned char)1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}

__global__ void asyncLoadKernel(const unsigned char *value, long long maxSpin) {
  for (long long i = 0; i < maxSpin; i++) {
    if (__hip_atomic_load(value, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_SYSTEM)) return;
    __builtin_amdgcn_s_sleep(32);
  }
}

static std::atomic<long long> gMaxSpin{-1};

static long long maxSpin() {
  long long v = gMaxSpin.load(std::memory_order_relaxed);
  if (v >= 0) return v;
  v = 1ll << 27;
  const char *e = getenv("FLAGCX_FUNC_MAX_SPIN_COUNT");
  if (e && *e) {
    char *end = nullptr;
    long long p = strtoll(e, &end, 10);
    if (end != e && p >= 0) v = p;
  }
  gMaxSpin.store(v, std::memory_order_relaxed);
  return v;
}

long long asyncMaxSpin() { return maxSpin(); }

} // namespace flagcx_amd

using namespace flagcx_amd;

#pragma GCC visibility push(default)
extern "C" {

void flagcxLocalSetMaxSpinCount(int64_t polls) {
  gMaxSpin.store(polls < 0 ? -1 : (long long)polls, std::memory_order_relaxed);
}

void deviceAsyncStore(flagcxStream_t stream, void *args) {
  hipStream_t s = stream ? *reinterpret_cast<hipStream_t *>(stream) : nullptr;
  asyncStoreKernel<<<1, 1, 0, s>>>(static_cast<unsigned char *>(args));
}

void deviceAsyncLoad(flagcxStream_t stream, void *args) {
  hipStream_t s = stream ? *reinterpret_cast<hipStream_t *>(stream) : nullptr;
  asyncLoadKernel<<<1, 1, 0, s>>>(static_cast<const unsigned char *>(args), maxSpin());
}

} // extern "C"
#pragma GCC visibility pop
