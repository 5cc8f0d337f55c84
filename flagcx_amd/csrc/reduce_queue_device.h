// reduce_queue_device.h - resident consumer of a host-produced queue of reduce
// descriptors: the host-producer / device-consumer half that the reference
// declares next to flagcxReduceTrigger and leaves commented out
// (flagcx/include/flagcx_kernel.h:52-73,96-98).
//
// One launch stays on the GPU and folds every descriptor the host appends, so a
// chunk is reduced when it arrives without a kernel launch per chunk.  The grid
// is 1 leader + W workers, each a single wavefront, all resident at once:
//   leader : polls `produced` in the pinned host header, copies new entries into a
//            device ring, publishes the count the workers poll (device memory, so
//            only one wavefront reads over PCIe), folds the workers' progress
//            words into `consumed` in the host header.
//   worker : draws tickets for units of one or a few KiB tiles in a numbering that
//            runs on across entries (so entries of a few thousand tiles still spread
//            evenly, and whoever is free takes the next unit), and folds each in the
//            same per-tile shape as the launch-per-call kernels.
//
// Coherence is per access, not per cache: a kernel that never ends gets no
// launch-boundary invalidate or write-back, and cache-wide maintenance from
// thousands of wavefronts costs tens of microseconds per entry.  So every data
// load carries sc0 sc1 (re-fetched at system scope: inputs may have been written
// by a copy engine or another stream since this kernel last touched the line),
// every data store carries sc0 sc1 (written through), queue words are scoped
// atomics, and "release" is waiting for the wavefront's own stores (s_waitcnt)
// before the progress word is written.  Only entries whose sources need
// unaligned global loads (no cache-policy bits there) fall back to a system-scope
// acquire fence in front of every unit.
//
// Every wait is bounded by maxSpin polls: a host that stops producing, or a
// worker that never becomes resident, ends in kQueueTimedOut, not in a hang
// (the leader counts polls without new entries or progress and then tells the
// workers to leave; a worker counts polls during which the leader's heartbeat
// word did not move).  A stop entry (k = 0) drains the queue: workers exit when
// they reach it.  A queue with nothing outstanding for `linger` polls parks: the
// kernel ends, so streams that share its hardware queue are held up only while
// there is work, and the producer's next entry launches it again.
#pragma once

#include "launch.h"
#include "reduce_device.h"

namespace flagcx_amd {

__device__ __forceinline__ uint64_t uniform64(uint64_t v) {
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  return ((uint64_t)hi << 32) | lo;
}
__device__ __forceinline__ uint64_t agentLoad(const uint64_t *p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void agentStore(uint64_t *p, uint64_t v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint64_t systemLoad(const uint64_t *p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}
__device__ __forceinline__ void systemStore(uint64_t *p, uint64_t v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// This wavefront's earlier loads have returned and its earlier stores have been
// acknowledged (gfx9 counts both in vmcnt); nothing moves across it at compile time.
__device__ __forceinline__ void waitOwnMemory() {
  __atomic_signal_fence(__ATOMIC_SEQ_CST);
  __builtin_amdgcn_s_waitcnt(0);
  __atomic_signal_fence(__ATOMIC_SEQ_CST);
}

// As above, except that the youngest operation may still be outstanding.
__device__ __forceinline__ void waitAllButYoungest() {
  __atomic_signal_fence(__ATOMIC_SEQ_CST);
  __builtin_amdgcn_s_waitcnt(0x0001); // vmcnt(1), expcnt(0), lgkmcnt(0)
  __atomic_signal_fence(__ATOMIC_SEQ_CST);
}

__device__ __forceinline__ uint32_t waveMin32(uint32_t v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const uint32_t o = __shfl_xor(v, off, 64);
    v = o < v ? o : v;
  }
  return v;
}

__device__ __forceinline__ uint64_t waveSum64(uint64_t v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

// Word `word` of a value every lane holds for the queue word (lane & 15).
__device__ __forceinline__ uint64_t laneWord(uint64_t v, int word) {
  const uint32_t lo = __builtin_amdgcn_readlane((uint32_t)v, word);
  const uint32_t hi = __builtin_amdgcn_readlane((uint32_t)(v >> 32), word);
  return ((uint64_t)hi << 32) | lo;
}

__device__ inline void queueLeader(const QueueKernelArgs &q) {
  const uint32_t nworkers = gridDim.x - 1;
  const uint32_t lane = threadIdx.x;
  // host counts are absolute, the device words (devProduced, progress) relative to q.base
  uint64_t forwarded = q.base, published = q.base, stopAt = ~0ull, beat = 0, produced = q.base;
  uint64_t inWork = 0; // traffic of the entries handed out and not yet finished by every worker
  int64_t spins = 0, idle = 0;
  if (lane == 0) systemStore(q.hostHeader + kQueueState, kQueueRunning);
  for (;;) {
    agentStore(q.devProduced + 1, ++beat); // heartbeat: workers count polls only while this stands still
    if (stopAt == ~0ull) {
      produced = uniform64(systemLoad(q.hostHeader + kQueueProduced)) & ~kQueueParkedBit;
      // four entries per round trip over PCIe: lane = 16 * entry + word
      while (forwarded < produced) {
        const uint64_t i = forwarded + (lane >> 4);
        const uint32_t word = lane & 15;
        const bool valid = i < produced;
        uint64_t w = 1;
        if (valid) {
          const uint64_t slot = i % q.capacity;
          w = systemLoad(reinterpret_cast<const uint64_t *>(q.hostEntries + slot) + word);
          agentStore(reinterpret_cast<uint64_t *>(q.devEntries + slot) + word, w);
        }
        // word 11 = k | flags << 32; k = 0 is the stop entry; flag bit 1: this entry
        // depends on an earlier one and starts only when everything before it is done
        const bool isCtl = valid && word == 11;
        const uint64_t stopMask = __ballot(isCtl && (uint32_t)w == 0);
        const uint64_t waitMask = __ballot(isCtl && ((w >> 32) & kQueueFlagAfterAll) != 0);
        uint64_t upto = forwarded + 4 < produced ? forwarded + 4 : produced;
        // Workers that run far apart lose the DRAM pages and the last-level cache
        // that neighbouring tiles share: hand out entries only while the traffic of
        // the unfinished ones stays inside a window (two entries may always be in work,
        // so that large entries follow one another without a gap).
        // An entry's traffic, (k + 1) * body bytes, is kept in word 12 of its copy in
        // the device ring for the day it retires.
        uint64_t traffic[4];
#pragma unroll
        for (int e = 0; e < 4; e++)
          traffic[e] = laneWord(w, 16 * e + 9) * 16 * ((uint64_t)(uint32_t)laneWord(w, 16 * e + 11) + 1);
        if (valid && word == 12) {
          const uint32_t e = lane >> 4;
          agentStore(reinterpret_cast<uint64_t *>(q.devEntries + i % q.capacity) + 12,
                     e == 0 ? traffic[0] : e == 1 ? traffic[1] : e == 2 ? traffic[2] : traffic[3]);
        }
        uint64_t fits = forwarded, sum = inWork;
#pragma unroll
        for (int e = 0; e < 4; e++)
          if (fits == forwarded + e && fits < upto && (fits - published < 2 || sum + traffic[e] <= q.windowBytes)) {
            sum += traffic[e];
            fits++;
          }
        upto = fits;
        bool blocked = upto <= forwarded;
        if (waitMask) {
          const uint64_t at = forwarded + ((uint64_t)(__ffsll((long long)waitMask) - 1) >> 4);
          if (at > forwarded) {
            if (upto > at) upto = at; // what precedes it goes out now, the entry itself in a later round
          } else if (published < at) {
            blocked = true; // its predecessors are still in flight
          } else {
            upto = at + 1;
          }
        }
        if (blocked) break;
        bool stopping = false;
        if (stopMask) {
          const uint64_t at = forwarded + ((uint64_t)(__ffsll((long long)stopMask) - 1) >> 4);
          if (at < upto) {
            stopAt = at;
            upto = at + 1; // nothing after a stop entry is published
            stopping = true;
          }
        }
        waitOwnMemory(); // the entries are in the device ring before the count says so
        agentStore(q.devProduced, upto - q.base);
#pragma unroll
        for (int e = 0; e < 4; e++)
          if (forwarded + e < upto) inWork += traffic[e];
        forwarded = upto;
        spins = 0;
        if (stopping) break;
      }
    }
    // min over the workers' 32-bit progress words, relative to what is published
    const uint32_t base32 = (uint32_t)(published - q.base);
    uint32_t ahead = ~0u;
    __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void *)q.progress, 0, nworkers * 4u, kRsrcFlags);
    for (uint32_t v0 = 0; v0 < nworkers; v0 += 1024) {
      u32x4 p[4];
#pragma unroll
      for (int u = 0; u < 4; u++)
        p[u] = __builtin_amdgcn_raw_buffer_load_b128(rs, (v0 + u * 256 + lane * 4) * 4u, 0, kAuxSc0 | kAuxSc1);
#pragma unroll
      for (int u = 0; u < 4; u++)
#pragma unroll
        for (int c = 0; c < 4; c++) {
          const uint32_t d = p[u][c] - base32;
          if (v0 + u * 256 + lane * 4 + c < nworkers && d < ahead) ahead = d;
        }
    }
    ahead = __builtin_amdgcn_readfirstlane(waveMin32(ahead));
    if (ahead != 0 && ahead != ~0u) {
      // a worker writes its progress word only after its results were acknowledged
      // by memory, so the count can go to the host as soon as it has been read
      waitOwnMemory();
      systemStore(q.hostHeader + kQueueConsumed, published + ahead);
      // the finished entries leave the traffic window (one lane per entry)
      uint64_t gone = 0;
      for (uint32_t r0 = 0; r0 < ahead; r0 += 64) {
        uint64_t mine = 0;
        if (r0 + lane < ahead)
          mine = agentLoad(reinterpret_cast<const uint64_t *>(q.devEntries + (published + r0 + lane) % q.capacity) + 12);
        gone += waveSum64(mine);
      }
      gone = uniform64(gone);
      inWork = inWork > gone ? inWork - gone : 0;
      published += ahead;
      spins = 0;
    }
    if (stopAt != ~0ull && published > stopAt) {
      waitOwnMemory();
      systemStore(q.hostHeader + kQueueState, kQueueStopped);
      return;
    }
    // Nothing outstanding for q.linger polls: leave the GPU to others.  The park bit
    // goes into the `produced` word itself, only if the count is still the one seen;
    // the producer's next fetch-and-add finds the bit and launches a new consumer.
    if (q.linger > 0 && stopAt == ~0ull && forwarded == produced && published == forwarded) {
      if (++idle > q.linger) {
        uint32_t parked = 0;
        if (lane == 0) {
          uint64_t expected = forwarded;
          parked = __hip_atomic_compare_exchange_strong(q.hostHeader + kQueueProduced, &expected,
                                                        forwarded | kQueueParkedBit, __ATOMIC_ACQ_REL,
                                                        __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM)
                       ? 1u
                       : 0u;
        }
        if (__builtin_amdgcn_readfirstlane(parked)) {
          agentStore(q.devProduced, ~0ull); // workers leave at their next poll
          systemStore(q.hostHeader + kQueueState, kQueueParked);
          return;
        }
        idle = 0; // an entry arrived in between
      }
    } else {
      idle = 0;
    }
    if (++spins > q.maxSpin) {
      agentStore(q.devProduced, ~0ull); // workers leave at their next poll
      systemStore(q.hostHeader + kQueueState, kQueueTimedOut);
      return;
    }
    __builtin_amdgcn_s_sleep(8);
  }
}

// Tiles per unit.  A worker folds one unit at a time: G consecutive KiB tiles of
// every input, all G*K loads issued before the first use.  Few inputs take several
// tiles at a time, so that a wavefront keeps as many bytes in flight as one with
// many inputs does and reads an entry's descriptor once per 8 KiB instead of once
// per KiB (two fp32 inputs, 32 entries of 4 MiB: 4.6 -> 5.9 TB/s).
constexpr int queueUnitTiles(int k) { return k <= 2 ? 8 : k <= 4 ? 4 : 1; }

// Where an entry's body sits inside a 128-byte line of its destination (a multiple of 16).
__device__ __forceinline__ uint32_t queueLead(uint64_t dst, uint64_t headBytes) {
  return (uint32_t)((dst + headBytes) & 127u);
}

// The units first, first + stride, ... of one entry (a ticket is one unit), K inputs known at
// compile time.  ALIGNED:
// every pointer agrees modulo 16 and tiles go through clipped buffer descriptors;
// otherwise the destination's tiling with unaligned 16-byte loads.
template <typename T, int OP, int K, int G, bool ALIGNED>
__device__ __forceinline__ void queueTiles(const uint64_t (&src)[8], uint64_t dst, uint64_t headBytes,
                                           uint64_t bodyBytes, uint32_t lead, uint64_t first, uint64_t stride) {
  constexpr uint32_t kUnitBytes = 1024u * G;
  const uint32_t voff = threadIdx.x * 16u;
  // the first unit is short by `lead` bytes, so that the others start on a 128-byte line
  // of the destination (units that start inside a line share lines with units that other
  // XCDs fold)
  const uint64_t nunits = (bodyBytes + lead + kUnitBytes - 1) / kUnitBytes;
  for (uint64_t u = first; u < nunits; u += stride) {
    const uint64_t boff = u ? u * kUnitBytes - lead : 0;
    const uint64_t off = headBytes + boff;
    const uint64_t left = bodyBytes - boff;
    const uint32_t cap = u ? kUnitBytes : kUnitBytes - lead;
    const uint32_t span = left < cap ? (uint32_t)left : cap;
    u32x4 in[G][K];
    if (ALIGNED) {
#pragma unroll
      for (int j = 0; j < K; j++) {
        __amdgpu_buffer_rsrc_t rs =
            __builtin_amdgcn_make_buffer_rsrc((void *)(uintptr_t)(src[j] + off), 0, span, kRsrcFlags);
#pragma unroll
        for (int g = 0; g < G; g++)
          in[g][j] = __builtin_amdgcn_raw_buffer_load_b128(rs, voff + g * 1024u, 0, kCoherentLoadAux);
      }
    } else {
#pragma unroll
      for (int j = 0; j < K; j++)
#pragma unroll
        for (int g = 0; g < G; g++)
          in[g][j] = voff + g * 1024u < span
                         ? __builtin_nontemporal_load(
                               (const u32x4_unaligned *)(uintptr_t)(src[j] + off + voff + g * 1024u))
                         : u32x4{0, 0, 0, 0};
    }
    __amdgpu_buffer_rsrc_t rd =
        __builtin_amdgcn_make_buffer_rsrc((void *)(uintptr_t)(dst + off), 0, span, kRsrcFlags);
#pragma unroll
    for (int g = 0; g < G; g++)
      if (ALIGNED || voff + g * 1024u < span)
        __builtin_amdgcn_raw_buffer_store_b128(foldVec<T, OP, K>(in[g], K), rd, voff + g * 1024u, 0,
                                               kCoherentStoreAux);
  }
}

template <typename T, int OP, int K>
__device__ __forceinline__ void queueEntry(const uint64_t (&src)[8], uint64_t dst, uint32_t head, uint32_t tail,
                                           uint64_t nvec, bool aligned, uint64_t first, uint64_t stride) {
  constexpr int N = 16 / sizeof(T);
  constexpr int G = queueUnitTiles(K);
  const uint64_t headBytes = (uint64_t)head * sizeof(T);
  const uint32_t lead = queueLead(dst, headBytes);
  if (aligned) {
    queueTiles<T, OP, K, G, true>(src, dst, headBytes, nvec * 16, lead, first, stride);
  } else {
    // plain global loads carry no scope bits: drop whatever this CU and L2 hold
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "");
    queueTiles<T, OP, K, G, false>(src, dst, headBytes, nvec * 16, lead, first, stride);
  }
  // head and tail elements: the worker that owns unit 0, one lane each
  if (first == 0 && threadIdx.x < head + tail) {
    const uint64_t i = threadIdx.x < head ? threadIdx.x : head + nvec * N + (threadIdx.x - head);
    typedef Fold<T, OP> F;
    typename F::acc_t acc = F::init(coherentLoad<T>(src[0], i));
#pragma unroll
    for (int j = 1; j < K; j++) acc = F::step(coherentLoad<T>(src[j], i), acc);
    coherentStore<T>(dst, i, F::fin(acc, K));
  }
}

// Units are numbered through, entry after entry, from the first entry of this launch
// on, and handed out by ticket: counter c of q.counters hands out the units congruent
// to c, in ascending order, to the workers that share it (a worker's counter follows
// from its workgroup number; every counter has workers from all XCDs).  Whoever is
// free takes the next unit, as the hardware dispatcher does for a launched grid, so
// a slow CU or XCD holds nobody else back (units dealt out by congruence to the worker
// number ran 10 % slower: every entry waited for its slowest worker).  The next
// ticket is fetched while the current unit is in flight; tickets drawn beyond the
// published entries are simply held until those entries arrive.  Counters are 1 KiB
// apart, in different memory channels.
// AHEAD: the queue takes entries of more than four inputs (units of one KiB per input)
// and its workers keep the next ticket on its way while they fold a unit; queues of up
// to four inputs (units of 4 or 8 KiB) draw a ticket when they need it and hold no code
// for more inputs.
template <typename T, int OP, bool AHEAD>
__device__ inline void queueWorker(const QueueKernelArgs &q) {
  const uint32_t worker = blockIdx.x - 1;
  const uint32_t nc = q.counters;
  const uint32_t c = (blockIdx.x / 8) % nc;
  uint64_t *const mine = q.tickets + (size_t)c * kQueueTicketStride;
  uint64_t done = 0;     // entries this worker has passed since this launch (entry index = q.base + done)
  uint64_t unitBase = 0; // number of the first unit of entry `done`
  uint64_t produced = 0; // entries known to be in the device ring
  uint64_t reported = 0; // what the progress word says
  uint64_t lastBeat = 0;
  // AHEAD: one ticket in hand and the next on its way; the draw is issued behind a unit's
  // store, so that no load waits for it (memory operations of a wavefront return in the
  // order issued), and is read a whole unit later.  Otherwise a ticket is drawn when the
  // previous unit's store has been issued, and waited for: drawing ahead hides the draw's
  // latency but lets the units in work spread over a window twice as wide, which costs
  // more than the wait when units are 4 or 8 KiB per input (3 inputs 5.95 -> 6.13 TB/s,
  // 4 inputs 6.15 -> 6.4) and less when they are one (8 inputs 6.2 -> 6.0).
  uint64_t ticket = 0, pending = 0;
  if (threadIdx.x == 0) {
    ticket = __hip_atomic_fetch_add(mine, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (AHEAD) pending = __hip_atomic_fetch_add(mine, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  ticket = uniform64(ticket);
  // lane l holds word l & 15 of entry `done` (haveCur) and of entry `done + 1` (haveNext)
  uint64_t cur = 0, next = 0;
  bool haveCur = false, haveNext = false;
  auto report = [&]() {
    // this wavefront's results are acknowledged by memory before the count says so;
    // with AHEAD the one operation that may still be on its way is the youngest, the
    // ticket draw issued behind the last store
    if (AHEAD) waitAllButYoungest();
    else waitOwnMemory();
    if (threadIdx.x == 0)
      __hip_atomic_store(q.progress + worker, (uint32_t)done, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    reported = done;
  };
  for (;;) {
    const uint64_t unit = ticket * nc + c;
    // the entry that holds this unit
    int k;
    uint64_t nunits;
    for (;;) {
      if (done >= produced) {
        if (reported != done) report();
        int64_t spins = 0;
        for (;;) {
          produced = uniform64(agentLoad(q.devProduced));
          if (produced > done) break; // the abort value ~0 ends the wait too
          // an idle queue is the leader's to time out; a worker only gives up by
          // itself when the leader's heartbeat has stopped for maxSpin polls
          const uint64_t beat = uniform64(agentLoad(q.devProduced + 1));
          if (beat != lastBeat) {
            lastBeat = beat;
            spins = 0;
          }
          if (++spins > q.maxSpin) return;
          __builtin_amdgcn_s_sleep(4);
        }
        if (produced == ~0ull) return;
      }
      if (!haveCur) {
        cur = agentLoad(reinterpret_cast<const uint64_t *>(q.devEntries + (q.base + done) % q.capacity) +
                        (threadIdx.x & 15));
        haveCur = true;
      }
      const uint64_t kv = laneWord(cur, 11);
      k = (int)(uint32_t)kv;
      if (k == 0) { // the stop entry: everything before it has been handed out
        done++;
        waitOwnMemory();
        report();
        return;
      }
      const uint64_t unitBytes = 1024ull * (uint32_t)queueUnitTiles(k);
      const uint64_t elemBytes = sizeof(T);
      nunits = (laneWord(cur, 9) * 16 + queueLead(laneWord(cur, 8), (uint32_t)laneWord(cur, 10) * elemBytes) + unitBytes - 1) /
               unitBytes;
      if (nunits == 0) nunits = 1; // head and tail elements only: still somebody's unit
      if (unit < unitBase + nunits) break;
      unitBase += nunits;
      done++;
      cur = next;
      haveCur = haveNext;
      haveNext = false;
    }
    // in flight while this unit is folded: the next entry
    if (!haveNext && done + 1 < produced) {
      next = agentLoad(reinterpret_cast<const uint64_t *>(q.devEntries + (q.base + done + 1) % q.capacity) +
                       (threadIdx.x & 15));
      haveNext = true;
    }
    const uint64_t kv = laneWord(cur, 11);
    const bool vector = ((kv >> 32) & kQueueFlagAligned) != 0;
    uint64_t src[8];
#pragma unroll
    for (int b = 0; b < 8; b++) src[b] = laneWord(cur, b);
    const uint64_t dst = laneWord(cur, 8);
    const uint64_t nvec = laneWord(cur, 9);
    const uint64_t ht = laneWord(cur, 10);
    const uint32_t head = (uint32_t)ht, tail = (uint32_t)(ht >> 32);
    const uint64_t first = unit - unitBase;
    switch (k) {
      case 1: queueEntry<T, OP, 1>(src, dst, head, tail, nvec, vector, first, nunits); break;
      case 2: queueEntry<T, OP, 2>(src, dst, head, tail, nvec, vector, first, nunits); break;
      case 3: queueEntry<T, OP, 3>(src, dst, head, tail, nvec, vector, first, nunits); break;
      case 4: queueEntry<T, OP, 4>(src, dst, head, tail, nvec, vector, first, nunits); break;
      default:
        if constexpr (AHEAD) {
          switch (k) {
            case 5: queueEntry<T, OP, 5>(src, dst, head, tail, nvec, vector, first, nunits); break;
            case 6: queueEntry<T, OP, 6>(src, dst, head, tail, nvec, vector, first, nunits); break;
            case 7: queueEntry<T, OP, 7>(src, dst, head, tail, nvec, vector, first, nunits); break;
            default: queueEntry<T, OP, 8>(src, dst, head, tail, nvec, vector, first, nunits); break;
          }
        }
        break; // the host admits no entry with more inputs than the queue was created for
    }
    if constexpr (AHEAD) {
      ticket = uniform64(pending);
      __atomic_signal_fence(__ATOMIC_SEQ_CST);
      if (threadIdx.x == 0) pending = __hip_atomic_fetch_add(mine, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __atomic_signal_fence(__ATOMIC_SEQ_CST);
    } else {
      // This counter's next unit lies nc further on: if that is beyond the entry, the worker
      // has passed it, and if nothing else is published it says so at once (the progress
      // of a lone small entry does not wait for the ticket draw).
      if (unit + nc >= unitBase + nunits) {
        unitBase += nunits;
        done++;
        cur = next;
        haveCur = haveNext;
        haveNext = false;
        if (done >= produced) report();
      }
      uint64_t drawn = 0;
      if (threadIdx.x == 0) drawn = __hip_atomic_fetch_add(mine, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      ticket = uniform64(drawn);
    }
    // in a long run of entries let the count move every few entries, so that the
    // leader's window and the producer's ring move while the run is still going
    if (done >= reported + 4) report();
  }
}

// At most 128 registers, so that sixteen consumers per CU (the most a queue may ask
// for) are resident whatever the element type and operation.
template <typename T, int OP, bool AHEAD>
__global__ void __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(4))) reduceQueueKernel(QueueKernelArgs q) {
  if (blockIdx.x == 0)
    queueLeader(q);
  else
    queueWorker<T, OP, AHEAD>(q);
}

} // namespace flagcx_amd
