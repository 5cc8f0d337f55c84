// fifo_perf.cpp - C++ timing driver for the host-producer / device-consumer reduce
// queue (flagcxLocalReduceFifo*), beside the launch-per-chunk and batched forms of
// the same work, and the batch launched up front with its descriptors opened one by one:
//
//   fifo_perf [-k nranks] [-t dtype] [-o op] [-c chunkbytes] [-m nchunks] [-w warmup] [-n iters]
//             [-W wavesPerCU] [-L lingerPolls] [-s spinLimit] [-q ringCapacity]
//             [-D windowBytes] [-a separateAllocations] [-g arrivalGapUs] [-x bytesIntoTheBuffers]
//             [-T wavesPerCUOfLaunchedKernels] [-I inputsInFlightOfLaunchedKernels]
//
// A shard of nchunks x chunkbytes per input (default 32 x 4 MiB: the reference's
// staging step, FLAGCX_P2P_CHUNKSIZE, flagcx/core/p2p.h:11-15) is reduced chunk by
// chunk.  Times are host wall clock from the first enqueue (or launch) to the
// moment the last chunk is known to be done; GB/s = (k+1)*bytes/time.
// With -g the chunks are handed over one every arrivalGapUs microseconds of host
// time (chunks that arrive one by one, the case the queue is for) instead of all at
// once; the batch call, which needs every chunk, then starts after the last arrival.
// With -x every buffer starts that many bytes further on (positions inside 128-byte lines).
// Also: latency of ONE small entry, enqueue -> Wait, against launch -> stream sync.
#include "../../include/flagcx_amd.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <thread>
#include <vector>

#define CK(x)                                                                  \
  do {                                                                         \
    hipError_t e_ = (x);                                                       \
    if (e_ != hipSuccess) {                                                    \
      fprintf(stderr, "HIP error %s at %s:%d\n", hipGetErrorString(e_), __FILE__, __LINE__); \
      return 1;                                                                \
    }                                                                          \
  } while (0)
#define FX(x)                                                                  \
  do {                                                                         \
    flagcxResult_t r_ = (x);                                                   \
    if (r_ != flagcxSuccess) {                                                 \
      fprintf(stderr, "flagcx error %d at %s:%d: %s | %s\n", (int)r_, __FILE__, __LINE__, flagcxLocalGetLastError(), \
              fifo ? flagcxLocalReduceFifoGetLastError(fifo) : "");            \
      if (fifo) flagcxLocalReduceFifoDestroy(fifo);                            \
      return 1;                                                                \
    }                                                                          \
  } while (0)

struct flagcxStream {
  hipStream_t base;
};

static double nowUs() {
  return std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now().time_since_epoch()).count();
}

static double median(std::vector<double> v) {
  std::sort(v.begin(), v.end());
  return v[v.size() / 2];
}

int main(int argc, char **argv) {
  int k = 8, dtype = flagcxHalf, op = flagcxAvg, nchunks = 32, warmup = 5, iters = 20;
  size_t chunkBytes = FLAGCX_LOCAL_CHUNKSIZE;
  long long spin = 1ll << 22;
  int tuneWaves = -1;
  long long linger = -1;
  int capacity = 64, separate = 0;
  double gapUs = 0.0;
  size_t shift = 0; // -x: every buffer starts this many bytes further on (positions inside cache lines)
  size_t window = 0;
  int launchWaves = -1, launchLoads = -1; // -T, -I: flagcxLocalTune / flagcxLocalTuneLoads for the launched kernels
  for (int i = 1; i + 1 < argc; i += 2) {
    const char *f = argv[i], *v = argv[i + 1];
    if (!strcmp(f, "-k")) k = atoi(v);
    else if (!strcmp(f, "-t")) dtype = atoi(v);
    else if (!strcmp(f, "-o")) op = atoi(v);
    else if (!strcmp(f, "-c")) chunkBytes = strtoull(v, 0, 0);
    else if (!strcmp(f, "-m")) nchunks = atoi(v);
    else if (!strcmp(f, "-w")) warmup = atoi(v);
    else if (!strcmp(f, "-n")) iters = atoi(v);
    else if (!strcmp(f, "-s")) spin = atoll(v);
    else if (!strcmp(f, "-W")) tuneWaves = atoi(v);
    else if (!strcmp(f, "-L")) linger = atoll(v);
    else if (!strcmp(f, "-q")) capacity = atoi(v);
    else if (!strcmp(f, "-D")) window = strtoull(v, 0, 0);
    else if (!strcmp(f, "-a")) separate = atoi(v);
    else if (!strcmp(f, "-g")) gapUs = atof(v);
    else if (!strcmp(f, "-x")) shift = strtoull(v, 0, 0);
    else if (!strcmp(f, "-T")) launchWaves = atoi(v);
    else if (!strcmp(f, "-I")) launchLoads = atoi(v);
  }
  flagcxLocalReduceFifo_t fifo = nullptr;
  const size_t ts = flagcxLocalGetDataTypeSize((flagcxDataType_t)dtype);
  if (!ts || k < 1 || k > 8 || nchunks < 1 || chunkBytes % ts) return 2;
  FX(flagcxLocalInit());
  flagcxLocalSetMaxSpinCount(spin); // an idle consumer leaves after this many polls
  if (launchWaves >= 0) FX(flagcxLocalTune(k, launchWaves));
  if (launchLoads >= 0) FX(flagcxLocalTuneLoads(k, launchLoads));
  const size_t shardBytes = chunkBytes * (size_t)nchunks;
  const size_t chunkCount = chunkBytes / ts;
  // the k inputs and the output in one allocation, in different HBM channel groups
  // (-a 1: k + 1 separate allocations instead, wherever the allocator puts them)
  std::vector<void *> src(k + 1);
  void *pool = nullptr;
  if (separate) {
    for (int j = 0; j <= k; j++) CK(hipMalloc(&src[j], shardBytes + 4096));
  } else {
    const size_t poolBytes = (size_t)(k + 1) * (shardBytes + 128 * 1024);
    CK(hipMalloc(&pool, poolBytes));
    FX(flagcxLocalPlaceBuffers(pool, poolBytes, shardBytes, k + 1, src.data()));
  }
  for (int j = 0; j <= k; j++) CK(hipMemset(src[j], 0, shardBytes)); // zeros are valid in every type
  if (shift % ts || shift > 4096) return 2;
  for (int j = 0; j <= k; j++) src[j] = (char *)src[j] + shift;
  void *dst = src[k];
  flagcxStream st;
  CK(hipStreamCreateWithFlags(&st.base, hipStreamNonBlocking));
  CK(hipDeviceSynchronize());
  const double algo = (k + 1.0) * (double)shardBytes;
  printf("# k=%d dtype=%d op=%d chunk=%zu B x %d chunks (%.0f MiB per input), warmup=%d iters=%d\n", k, dtype, op,
         chunkBytes, nchunks, shardBytes / 1048576.0, warmup, iters);
  if (gapUs > 0)
    printf("# chunks arrive %.2f us apart: the last one %.1f us after the first, i.e. at most %.1f GB/s\n", gapUs,
           gapUs * (nchunks - 1), algo / (gapUs * (nchunks - 1)) / 1e3);
  // chunk c is available from t0 + c * gapUs on
  auto arrive = [&](double t0, int c) {
    if (gapUs > 0)
      while (nowUs() < t0 + gapUs * c) {
      }
  };

  std::vector<std::vector<const void *>> chunkSrc(nchunks, std::vector<const void *>(k));
  std::vector<flagcxLocalReduceDesc> descs(nchunks);
  for (int c = 0; c < nchunks; c++) {
    for (int j = 0; j < k; j++) chunkSrc[c][j] = (const char *)src[j] + (size_t)c * chunkBytes;
    descs[c].sendbuffs = chunkSrc[c].data();
    descs[c].recvbuff = (char *)dst + (size_t)c * chunkBytes;
    descs[c].count = chunkCount;
  }

  // (1) one launch per chunk
  std::vector<double> t;
  for (int it = 0; it < warmup + iters; it++) {
    const double t0 = nowUs();
    for (int c = 0; c < nchunks; c++) {
      arrive(t0, c);
      FX(flagcxLocalReduce(chunkSrc[c].data(), k, descs[c].recvbuff, chunkCount, (flagcxDataType_t)dtype,
                           (flagcxRedOp_t)op, &st));
    }
    CK(hipStreamSynchronize(st.base));
    if (it >= warmup) t.push_back(nowUs() - t0);
  }
  printf("%-46s %10.1f us  %8.1f GB/s\n", "one launch per chunk, then stream sync", median(t), algo / median(t) / 1e3);

  // (2) all chunks known up front: one batch call
  t.clear();
  for (int it = 0; it < warmup + iters; it++) {
    const double t0 = nowUs();
    arrive(t0, nchunks - 1);
    FX(flagcxLocalReduceBatch(descs.data(), nchunks, k, (flagcxDataType_t)dtype, (flagcxRedOp_t)op, &st));
    CK(hipStreamSynchronize(st.base));
    if (it >= warmup) t.push_back(nowUs() - t0);
  }
  printf("%-46s %10.1f us  %8.1f GB/s\n", "one batch call (all chunks present), sync", median(t), algo / median(t) / 1e3);

  // (2b) the same batch launched up front, its descriptors opened chunk by chunk.  With -g the
  // launch precedes the first arrival (that is what it is for); without, it is inside the time.
  {
    flagcxLocalGate_t gate = nullptr;
    FX(flagcxLocalGateCreate(&gate));
    t.clear();
    for (int it = 0; it < warmup + iters; it++) {
      uint64_t first = 0;
      double t0 = nowUs();
      FX(flagcxLocalReduceBatchGated(gate, descs.data(), nchunks, k, (flagcxDataType_t)dtype, (flagcxRedOp_t)op, &st,
                                     &first));
      if (gapUs > 0) t0 = nowUs();
      for (int c = 0; c < nchunks; c++) {
        arrive(t0, c);
        FX(flagcxLocalGateOpen(gate, first + (uint64_t)c + 1));
      }
      CK(hipStreamSynchronize(st.base));
      if (it >= warmup) t.push_back(nowUs() - t0);
    }
    int gateState = 0;
    FX(flagcxLocalGateQuery(gate, nullptr, nullptr, &gateState));
    printf("%-46s %10.1f us  %8.1f GB/s%s\n", "gated batch launched up front, Open per chunk", median(t),
           algo / median(t) / 1e3, gateState ? "  (GAVE UP WAITING)" : "");
    FX(flagcxLocalGateDestroy(gate));
  }

  // (3) the resident consumer: enqueue chunk by chunk, wait for the last ticket
  FX(flagcxLocalReduceFifoCreate(&fifo, capacity, k, (flagcxDataType_t)dtype, (flagcxRedOp_t)op));
  if (tuneWaves > 0) FX(flagcxLocalReduceFifoSetWaves(fifo, tuneWaves));
  if (linger >= 0) FX(flagcxLocalReduceFifoSetLinger(fifo, linger));
  if (window > 0) FX(flagcxLocalReduceFifoSetWindow(fifo, window));
  FX(flagcxLocalReduceFifoStart(fifo));
  unsigned grid = 0;
  FX(flagcxLocalReduceFifoGetGrid(fifo, &grid));
  t.clear();
  for (int it = 0; it < warmup + iters; it++) {
    const double t0 = nowUs();
    uint64_t ticket = 0;
    for (int c = 0; c < nchunks; c++) {
      arrive(t0, c);
      flagcxResult_t r;
      while ((r = flagcxLocalReduceFifoEnqueueReduce(fifo, chunkSrc[c].data(), k, descs[c].recvbuff, chunkCount,
                                                     &ticket)) == flagcxInProgress) {
      }
      FX(r);
    }
    FX(flagcxLocalReduceFifoWait(fifo, ticket));
    if (it >= warmup) t.push_back(nowUs() - t0);
  }
  printf("%-46s %10.1f us  %8.1f GB/s  (%u resident wavefronts)\n", "resident consumer, enqueue per chunk, Wait",
         median(t), algo / median(t) / 1e3, grid);

  // (4) latency of one small entry (4 KiB per input)
  const size_t smallCount = 4096 / ts;
  t.clear();
  for (int it = 0; it < 200; it++) {
    uint64_t ticket = 0;
    const double t0 = nowUs();
    FX(flagcxLocalReduceFifoEnqueueReduce(fifo, chunkSrc[0].data(), k, dst, smallCount, &ticket));
    FX(flagcxLocalReduceFifoWait(fifo, ticket));
    t.push_back(nowUs() - t0);
  }
  const double fifoLat = median(t);
  // the same entry after the consumer has parked (the enqueue launches it again)
  t.clear();
  for (int it = 0; it < 20; it++) {
    int state = 0;
    for (int spin = 0; spin < 2000 && state != FLAGCX_LOCAL_REDUCE_FIFO_PARKED; spin++) {
      FX(flagcxLocalReduceFifoQuery(fifo, nullptr, nullptr, &state));
      std::this_thread::sleep_for(std::chrono::microseconds(50));
    }
    if (state != FLAGCX_LOCAL_REDUCE_FIFO_PARKED) break; // parking is off (-L 0)
    uint64_t ticket = 0;
    const double t0 = nowUs();
    FX(flagcxLocalReduceFifoEnqueueReduce(fifo, chunkSrc[0].data(), k, dst, smallCount, &ticket));
    FX(flagcxLocalReduceFifoWait(fifo, ticket));
    t.push_back(nowUs() - t0);
  }
  const double parkedLat = t.empty() ? 0.0 : median(t);
  FX(flagcxLocalReduceFifoStop(fifo));
  t.clear();
  for (int it = 0; it < 200; it++) {
    const double t0 = nowUs();
    FX(flagcxLocalReduce(chunkSrc[0].data(), k, dst, smallCount, (flagcxDataType_t)dtype, (flagcxRedOp_t)op, &st));
    CK(hipStreamSynchronize(st.base));
    t.push_back(nowUs() - t0);
  }
  printf("4 KiB entry: enqueue -> Wait %.2f us (consumer on the GPU), %.2f us (parked, launched again); "
         "launch -> stream sync %.2f us\n", fifoLat, parkedLat, median(t));
  FX(flagcxLocalReduceFifoDestroy(fifo));
  fifo = nullptr;
  if (separate)
    for (int j = 0; j <= k; j++) CK(hipFree((char *)src[j] - shift));
  else
    CK(hipFree(pool));
  return 0;
}
