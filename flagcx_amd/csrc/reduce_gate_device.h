// reduce_gate_device.h - a batch of reductions launched before its inputs have arrived.
//
// The chunks of a pipelined collective are known when the collective starts; only their
// arrival times are not.  The reference's proxy folds a chunk when its receive completes
// (flagcx/core/proxy.cc:1074-1182 is the loop such completions drive).  Here the whole
// batch is ONE ordinary launch, issued up front, whose workgroups hold back until the
// host has said that their descriptor's inputs are complete:
//   - the host keeps a count in pinned memory: descriptors numbered below it may run;
//   - workgroup (0, 0) leads: it polls that count over PCIe and raises a copy in device
//     memory (fetch-max, so that the leaders of two launches that overlap never lower it),
//     and folds its own tile once every descriptor of its launch may run;
//   - every other workgroup reads the device copy once before its loads, and polls it
//     only if its descriptor has not arrived yet.
// Workgroups are dispatched in order, descriptor after descriptor, so those that wait hold
// wavefront slots only behind the ones that can run, and a grid dispatched tile by tile
// keeps the rate of the plain batch launch (a resident grid that draws its tiles by
// ticket stays 5 to 7 % below it).  The read of the device word in front of a wavefront's
// loads is what the gate costs: 5 to 11 % as a vector load (whatever its scope: it queues
// behind the CU's streaming loads), 3 to 4 % as a scalar load, which is how the first look
// is taken when the word could be placed in uncached memory.  An acquire fence behind the
// read would cost tens of microseconds per wavefront (cache-wide maintenance), so coherence
// is per access, as in the reduce queue: data loads carry sc0 sc1 and are issued only after
// the count has been seen.
//
// Every wait is bounded: the leader gives up after maxSpin polls without a change of the
// host's count, marks the gate abandoned (device word ~0, state word in pinned memory) and
// every workgroup of this and later launches on the gate leaves without touching data.
#pragma once

#include "launch.h"
#include "reduce_device.h"
#include "reduce_queue_device.h"

namespace flagcx_amd {

// Returns the count last seen; ~0 when the host has abandoned the gate.  After maxSpin polls
// without a change the leader abandons the gate itself (what it returns then still says
// which descriptors had been opened).
__device__ __forceinline__ uint64_t gateLead(const GateArgs &g) {
  uint64_t last = 0;
  for (int64_t spins = 0;;) {
    uint64_t v = 0;
    if (threadIdx.x == 0) v = systemLoad(g.host);
    v = uniform64(v);
    if (v != last) {
      if (threadIdx.x == 0) __hip_atomic_fetch_max(g.dev, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      last = v;
      spins = 0;
    }
    if (v >= g.all) return v; // includes ~0: the gate is being destroyed
    if (++spins > g.maxSpin) break;
    __builtin_amdgcn_s_sleep(2);
  }
  if (threadIdx.x == 0) {
    systemStore(g.hostState, kGateTimedOut);
    __hip_atomic_fetch_max(g.dev, ~0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  return last;
}

// false: the gate was abandoned.
__device__ __forceinline__ bool gateWait(const GateArgs &g, uint64_t need) {
  for (int64_t spins = 0;;) {
    uint64_t v = 0;
    if (g.scalarRead && spins == 0) {
      // One 8-byte scalar load that bypasses the scalar cache.  The word lives in uncached
      // device memory, so what comes back is what memory holds; the scalar path does not
      // queue behind the CU's streaming vector loads, which is what a vector read of the
      // count costs (3 to 8 % of the launch's rate).  Only the first look takes it.
      asm volatile("s_load_dwordx2 %0, %1, 0x0 glc\n\ts_waitcnt lgkmcnt(0)" : "=s"(v) : "s"(g.dev) : "memory");
    } else {
      if (threadIdx.x == 0) v = agentLoad(g.dev);
      v = uniform64(v);
    }
    if (v == ~0ull) return false;
    if (v > need) return true;
    // the leader's bound comes first; this one only ends a workgroup whose leader is gone
    if (++spins > 8 * g.maxSpin + 1024) break;
    __builtin_amdgcn_s_sleep(8);
  }
  if (threadIdx.x == 0) systemStore(g.hostState, kGateTimedOut);
  return false;
}

template <typename T, int OP, int K, int U>
__global__ void __launch_bounds__(64) reduceGatedBatchKernel(ReduceBatchParams<K> bp, GateArgs g) {
  if (blockIdx.x != 0 || blockIdx.y != 0) {
    // a workgroup beyond its segment's tiles, with no head or tail elements to fold either,
    // has nothing to wait for (segments of one launch may differ in size)
    const ReduceParams<K> &p = bp.seg[blockIdx.y];
    constexpr uint64_t kTileBytes = 64ull * U * 16ull;
    uint64_t tiles = (p.nvec * 16 + p.lead + kTileBytes - 1) / kTileBytes;
    if (p.run > 1) tiles = (tiles + 8ull * p.run - 1) / (8ull * p.run) * (8ull * p.run);
    if (blockIdx.x >= tiles && blockIdx.x != gridDim.x - 1) return;
  }
  bool open;
  if (blockIdx.x == 0 && blockIdx.y == 0) {
    // the leader's own tile is folded last, if its descriptor has been opened at all
    const uint64_t seen = gateLead(g);
    open = seen != ~0ull && seen > g.need[0];
  } else {
    open = gateWait(g, g.need[blockIdx.y]);
  }
  if (!open) return;
  __atomic_signal_fence(__ATOMIC_SEQ_CST); // no load of the data is moved in front of the wait
  reduceWaveBody<T, OP, K, U, true, true>(bp.seg[blockIdx.y]);
}

} // namespace flagcx_amd
