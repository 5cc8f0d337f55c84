// local_perf.cpp - C++ timing driver for the C ABI, in the manner of the
// reference's perf programs (size sweep -b..-e with factor -f, -w warm-up and -n
// timed iterations, defaults 5 and 20 as test/perf/tools.cc:81-86).  It measures
// what a C/C++ caller sees, without any Python in the launch path:
//
//   local_perf [-b minbytes] [-e maxbytes] [-f factor] [-w warmup] [-n iters] [-k nranks] [-t dtype] [-o op]
//
// Per size: back-to-back launches bracketed by two HIP events (per-launch time and
// algorithmic GB/s = (k+1)*bytes/time), and launch -> hipStreamSynchronize wall time.
#include "../../include/flagcx_amd.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#define CK(x)                                                                  \
  do {                                                                         \
    hipError_t e_ = (x);                                                       \
    if (e_ != hipSuccess) {                                                    \
      fprintf(stderr, "HIP error %s at %s:%d\n", hipGetErrorString(e_), __FILE__, __LINE__); \
      return 1;                                                                \
    }                                                                          \
  } while (0)

struct flagcxStream {
  hipStream_t base;
};

int main(int argc, char **argv) {
  size_t minb = 1024, maxb = 1ull << 30;
  int factor = 2, warmup = 5, iters = 20, k = 2, dtype = flagcxFloat, op = flagcxSum;
  for (int i = 1; i + 1 < argc; i += 2) {
    const char *f = argv[i], *v = argv[i + 1];
    if (!strcmp(f, "-b")) minb = strtoull(v, 0, 0);
    else if (!strcmp(f, "-e")) maxb = strtoull(v, 0, 0);
    else if (!strcmp(f, "-f")) factor = atoi(v);
    else if (!strcmp(f, "-w")) warmup = atoi(v);
    else if (!strcmp(f, "-n")) iters = atoi(v);
    else if (!strcmp(f, "-k")) k = atoi(v);
    else if (!strcmp(f, "-t")) dtype = atoi(v);
    else if (!strcmp(f, "-o")) op = atoi(v);
  }
  if (factor < 2 || k < 1 || k > FLAGCX_LOCAL_MAX_RANKS) return 2;
  const size_t ts = flagcxLocalGetDataTypeSize((flagcxDataType_t)dtype);
  if (!ts) return 2;
  if (flagcxLocalInit() != flagcxSuccess) {
    fprintf(stderr, "%s\n", flagcxLocalGetLastError());
    return 1;
  }
  flagcxStream st;
  CK(hipStreamCreateWithFlags(&st.base, hipStreamNonBlocking));
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0));
  CK(hipEventCreate(&e1));
  std::vector<void *> src(k);
  void *dst = nullptr;
  for (int j = 0; j < k; j++) {
    CK(hipMalloc(&src[j], maxb));
    CK(hipMemset(src[j], j + 1, maxb));
  }
  CK(hipMalloc(&dst, maxb));
  printf("# k=%d dtype=%d op=%d warmup=%d iters=%d\n", k, dtype, op, warmup, iters);
  printf("%14s %14s %12s %12s %14s\n", "bytes/buffer", "count", "us/launch", "GB/s", "launch->sync us");
  for (size_t bytes = minb; bytes <= maxb; bytes *= (size_t)factor) {
    const size_t count = bytes / ts;
    auto call = [&]() {
      return flagcxLocalReduce(src.data(), k, dst, count, (flagcxDataType_t)dtype, (flagcxRedOp_t)op, &st);
    };
    for (int i = 0; i < warmup; i++)
      if (call() != flagcxSuccess) { fprintf(stderr, "%s\n", flagcxLocalGetLastError()); return 1; }
    CK(hipStreamSynchronize(st.base));
    const int reps = bytes <= (1u << 20) ? iters * 50 : iters;
    CK(hipEventRecord(e0, st.base));
    for (int i = 0; i < reps; i++) call();
    CK(hipEventRecord(e1, st.base));
    CK(hipEventSynchronize(e1));
    float ms = 0;
    CK(hipEventElapsedTime(&ms, e0, e1));
    const double us = ms * 1e3 / reps;
    std::vector<double> single;
    for (int i = 0; i < iters; i++) {
      auto t0 = std::chrono::steady_clock::now();
      call();
      CK(hipStreamSynchronize(st.base));
      single.push_back(std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count());
    }
    std::sort(single.begin(), single.end());
    printf("%14zu %14zu %12.3f %12.1f %14.2f\n", bytes, count, us, (k + 1.0) * bytes / us / 1e3, single[single.size() / 2]);
    fflush(stdout);
  }
  return 0;
}
