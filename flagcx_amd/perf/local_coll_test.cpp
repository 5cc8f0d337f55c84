// local_coll_test.cpp - C++ caller test in the shape of the reference's unit tests
// (test/unittest/main.cpp:11-398): buffers come from the device-adaptor table
// (deviceMalloc / deviceMemcpy / deviceMemset / streamSynchronize, as the
// reference's devHandle->...), data is the reference's patterns (i % 10 for
// all-reduce, floor(i / recvcount) for reduce-scatter, float(i) for scatter), and
// the collectives run over `nranks` simulated ranks whose buffers all live on this
// GPU.  Unlike the reference's strcmp, results are compared in full.
//
//   local_coll_test [-n nranks (3 or more)] [-c count_per_rank]      exit code 0 = all passed
#include "../../include/flagcx_amd_adaptor.h"

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#define OK(call)                                                               \
  do {                                                                         \
    flagcxResult_t r_ = (call);                                                \
    if (r_ != flagcxSuccess) {                                                 \
      fprintf(stderr, "%s:%d: %s -> %d (%s)\n", __FILE__, __LINE__, #call, (int)r_, flagcxLocalGetLastError()); \
      return 1;                                                                \
    }                                                                          \
  } while (0)

static int failures = 0;
#define EXPECT(cond, what)                                                     \
  do {                                                                         \
    if (!(cond)) { fprintf(stderr, "FAILED %s (%s:%d)\n", what, __FILE__, __LINE__); failures++; } \
    else printf("ok     %s\n", what);                                          \
  } while (0)

int main(int argc, char **argv) {
  int nranks = 8;
  size_t count = 1 << 22; // elements per rank
  for (int i = 1; i + 1 < argc; i += 2) {
    if (!strcmp(argv[i], "-n")) nranks = atoi(argv[i + 1]);
    if (!strcmp(argv[i], "-c")) count = strtoull(argv[i + 1], 0, 0);
  }
  if (nranks < 3 || nranks > FLAGCX_LOCAL_MAX_RANKS || count % (size_t)nranks) return 2; // the checks use ranks 0, 1 and 2
  struct flagcxDeviceAdaptor *dev = flagcxLocalGetDeviceAdaptor();
  const size_t size = count * sizeof(float);
  flagcxStream_t stream;
  OK(dev->streamCreate(&stream));

  std::vector<void *> sendbuff(nranks), recvbuff(nranks);
  void *hostsend = nullptr, *hostrecv = nullptr;
  for (int r = 0; r < nranks; r++) {
    OK(dev->deviceMalloc(&sendbuff[r], size, flagcxMemDevice, stream));
    OK(dev->deviceMalloc(&recvbuff[r], size, flagcxMemDevice, stream));
  }
  OK(dev->deviceMalloc(&hostsend, size, flagcxMemHost, NULL));
  OK(dev->deviceMalloc(&hostrecv, size, flagcxMemHost, NULL));
  float *hs = static_cast<float *>(hostsend), *hr = static_cast<float *>(hostrecv);
  std::vector<const void *> sends(sendbuff.begin(), sendbuff.end());

  // ---- AllReduce: every rank holds i % 10; sum / nranks must give the input back
  for (size_t i = 0; i < count; i++) hs[i] = (float)(i % 10);
  for (int r = 0; r < nranks; r++) OK(dev->deviceMemcpy(sendbuff[r], hostsend, size, flagcxMemcpyHostToDevice, stream, NULL));
  OK(flagcxLocalAllReduce(sends.data(), nranks, recvbuff[0], count, flagcxFloat, flagcxSum, stream));
  OK(dev->deviceMemset(hostrecv, 0, size, flagcxMemHost, stream));
  OK(dev->deviceMemcpy(hostrecv, recvbuff[0], size, flagcxMemcpyDeviceToHost, stream, NULL));
  OK(dev->streamSynchronize(stream));
  for (size_t i = 0; i < count; i++) hr[i] /= (float)nranks;
  EXPECT(memcmp(hostsend, hostrecv, size) == 0, "AllReduce sum of i%10 over all ranks, divided by nranks");

  // ---- Reduce (to one root buffer) with max: identical inputs -> unchanged
  OK(flagcxLocalReduce(sends.data(), nranks, recvbuff[1], count, flagcxFloat, flagcxMax, stream));
  OK(dev->deviceMemcpy(hostrecv, recvbuff[1], size, flagcxMemcpyDeviceToHost, stream, NULL));
  OK(dev->streamSynchronize(stream));
  EXPECT(memcmp(hostsend, hostrecv, size) == 0, "Reduce max of identical buffers");

  // ---- ReduceScatter: value floor(i / recvcount) -> rank r receives nranks * r
  const size_t recvcount = count / (size_t)nranks;
  for (size_t i = 0; i < count; i++) hs[i] = (float)(i / recvcount);
  for (int r = 0; r < nranks; r++) OK(dev->deviceMemcpy(sendbuff[r], hostsend, size, flagcxMemcpyHostToDevice, stream, NULL));
  bool rsok = true;
  for (int r = 0; r < nranks; r++) {
    OK(flagcxLocalReduceScatter(sends.data(), nranks, r, recvbuff[r], recvcount, flagcxFloat, flagcxSum, stream));
    OK(dev->deviceMemcpy(hostrecv, recvbuff[r], recvcount * sizeof(float), flagcxMemcpyDeviceToHost, stream, NULL));
    OK(dev->streamSynchronize(stream));
    for (size_t i = 0; i < recvcount; i++) rsok = rsok && hr[i] == (float)(nranks * r);
  }
  EXPECT(rsok, "ReduceScatter of floor(i/recvcount): shard r == nranks*r");

  // ---- Scatter / Gather / AllGather through the pack / unpack kernels: float(i)
  for (size_t i = 0; i < count; i++) hs[i] = (float)i;
  OK(dev->deviceMemcpy(sendbuff[0], hostsend, size, flagcxMemcpyHostToDevice, stream, NULL));
  std::vector<void *> pieces(nranks);
  for (int r = 0; r < nranks; r++) pieces[r] = recvbuff[r];
  // scatter: root's buffer cut into nranks pieces, piece r to rank r
  OK(flagcxLocalUnpackList(pieces.data(), sendbuff[0], nranks, recvcount * sizeof(float), stream));
  // gather / all-gather: the pieces back into one contiguous buffer (on rank 1)
  std::vector<const void *> cpieces(pieces.begin(), pieces.end());
  OK(flagcxLocalPackList(sendbuff[1], cpieces.data(), nranks, recvcount * sizeof(float), stream));
  OK(dev->deviceMemcpy(hostrecv, sendbuff[1], size, flagcxMemcpyDeviceToHost, stream, NULL));
  OK(dev->streamSynchronize(stream));
  EXPECT(memcmp(hostsend, hostrecv, size) == 0, "Scatter then Gather of float(i) restores the buffer");

  // ---- Broadcast = device-to-device copy from the root through the adaptor table
  for (int r = 1; r < nranks; r++) OK(dev->deviceMemcpy(recvbuff[r], sendbuff[0], size, flagcxMemcpyDeviceToDevice, stream, NULL));
  OK(dev->deviceMemcpy(hostrecv, recvbuff[nranks - 1], size, flagcxMemcpyDeviceToHost, stream, NULL));
  OK(dev->streamSynchronize(stream));
  EXPECT(memcmp(hostsend, hostrecv, size) == 0, "Broadcast of float(i) to the last rank");

  // ---- Broadcast as one call: the root's buffer read once, stored to every other rank
  for (int r = 0; r < nranks; r++) OK(dev->deviceMemset(recvbuff[r], 0, size, flagcxMemDevice, stream));
  {
    std::vector<void *> others;
    for (int r = 1; r < nranks; r++) others.push_back(recvbuff[r]);
    flagcxLocalFanoutDesc f = {sendbuff[0], others.data(), (int)others.size(), size};
    OK(flagcxLocalCopyFanout(&f, 1, stream));
    bool all = true;
    for (int r = 1; r < nranks; r++) {
      OK(dev->deviceMemcpy(hostrecv, recvbuff[r], size, flagcxMemcpyDeviceToHost, stream, NULL));
      OK(dev->streamSynchronize(stream));
      all = all && memcmp(hostsend, hostrecv, size) == 0;
    }
    EXPECT(all, "Broadcast of float(i) to every other rank with one read of the root's buffer");
  }

  // ---- Self send/recv byte pattern (test/perf/test_core_sendrecv.cpp:80-94)
  unsigned char *hb = static_cast<unsigned char *>(hostsend);
  memset(hb, 0xAA, 100);
  memset(hb + 100, 0xBB, 200);
  OK(dev->deviceMemcpy(sendbuff[2], hostsend, 300, flagcxMemcpyHostToDevice, stream, NULL));
  OK(flagcxLocalMemcpy(recvbuff[2], sendbuff[2], 300, stream));
  OK(dev->deviceMemcpy(hostrecv, recvbuff[2], 300, flagcxMemcpyDeviceToHost, stream, NULL));
  OK(dev->streamSynchronize(stream));
  EXPECT(memcmp(hostsend, hostrecv, 300) == 0, "self send/recv of 0xAA x100 + 0xBB x200");

  for (int r = 0; r < nranks; r++) {
    OK(dev->deviceFree(sendbuff[r], flagcxMemDevice, NULL));
    OK(dev->deviceFree(recvbuff[r], flagcxMemDevice, NULL));
  }
  OK(dev->deviceFree(hostsend, flagcxMemHost, NULL));
  OK(dev->deviceFree(hostrecv, flagcxMemHost, NULL));
  OK(dev->streamDestroy(stream));
  printf("%s\n", failures ? "FAILED" : "PASSED");
  return failures ? 1 : 0;
}
