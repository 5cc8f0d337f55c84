// Test double of the device layer, for CPU tests of the plan executor's HOST logic only
// (flagcx_amd/csrc/host_c2c_local.cpp: plan import, step walking, refresh placement, the
// record of cleared ranges, grouping of copies and collectives).  It implements, on host
// memory, the eight C-ABI entry points the executor calls, for int32 and fp32 with sum /
// max / min, and it is strict where the GPU cannot be: every call checks that what the
// executor hands over as "runs concurrently" really is independent, and the harness
// allocates every buffer at its exact size so that AddressSanitizer sees any access past
// the end.  Never linked into the library; nothing outside tests/ uses it.
#include "../../include/flagcx_amd.h"

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

namespace {

[[noreturn]] void die(const char *what) {
  fprintf(stderr, "device_double: %s\n", what);
  abort();
}

bool hit(const void *a, size_t an, const void *b, size_t bn) {
  return (uintptr_t)a < (uintptr_t)b + bn && (uintptr_t)b < (uintptr_t)a + an;
}

size_t sizeOf(flagcxDataType_t dt) {
  static const size_t s[] = {1, 1, 4, 4, 8, 8, 2, 4, 8, 2};
  return (int)dt >= 0 && (int)dt < 10 ? s[(int)dt] : 0;
}

// acc = in_0; acc = OP(in_j, acc): OP(x, acc) with min = (acc < x) ? acc : x, max = (x < acc) ? acc : x
template <typename T>
void fold(const void *const *src, int k, void *dst, size_t n, flagcxRedOp_t op, bool plusZero) {
  std::vector<T> out(n);
  for (size_t i = 0; i < n; i++) {
    T acc = ((const T *)src[0])[i];
    for (int j = 1; j < k; j++) {
      const T x = ((const T *)src[j])[i];
      if (op == flagcxSum) acc = (T)(x + acc);
      else if (op == flagcxMax) acc = (x < acc) ? acc : x;
      else if (op == flagcxMin) acc = (acc < x) ? acc : x;
      else die("unsupported op");
    }
    if (plusZero) acc = (T)(acc + (T)0);
    out[i] = acc;
  }
  memcpy(dst, out.data(), n * sizeof(T)); // all inputs are read before the output is written
}

void foldAny(const void *const *src, int k, void *dst, size_t n, flagcxDataType_t dt, flagcxRedOp_t op, bool plusZero) {
  if (k == 1 && !plusZero) { // the fold of one input is the input, whatever the type (the executor's grouped copies)
    if (dst != src[0]) memmove(dst, src[0], n * sizeOf(dt));
    return;
  }
  if (dt == flagcxInt32) {
    // unsigned arithmetic: sums wrap
    if (op == flagcxSum) fold<uint32_t>(src, k, dst, n, op, false);
    else fold<int32_t>(src, k, dst, n, op, false);
  } else if (dt == flagcxFloat) {
    fold<float>(src, k, dst, n, op, plusZero);
  } else {
    die("the double folds int32 and fp32 only");
  }
}

// descriptors of one call run concurrently on the GPU: nothing one writes may be read or
// written by another (an input that is also the output of the SAME descriptor, element for
// element, is the in-place case and fine)
void checkIndependent(const flagcxLocalReduceDesc *d, int n, int k, size_t ts) {
  for (int a = 0; a < n; a++)
    for (int b = 0; b < n; b++) {
      if (a == b) continue;
      if (hit(d[a].recvbuff, d[a].count * ts, d[b].recvbuff, d[b].count * ts)) die("two descriptors of one batch write the same bytes");
      for (int j = 0; j < k; j++)
        if (hit(d[a].recvbuff, d[a].count * ts, d[b].sendbuffs[j], d[b].count * ts)) die("a descriptor of a batch reads what another writes");
    }
  for (int a = 0; a < n; a++)
    for (int j = 0; j < k; j++)
      if (d[a].sendbuffs[j] != d[a].recvbuff && hit(d[a].recvbuff, d[a].count * ts, d[a].sendbuffs[j], d[a].count * ts))
        die("an input overlaps the output at another offset");
}

} // namespace

extern "C" {

size_t flagcxLocalGetDataTypeSize(flagcxDataType_t dt) { return sizeOf(dt); }

flagcxResult_t flagcxLocalMemcpy(void *dst, const void *src, size_t n, flagcxStream_t) {
  if (n && hit(dst, n, src, n)) die("memcpy: buffers overlap");
  memcpy(dst, src, n);
  return flagcxSuccess;
}

flagcxResult_t flagcxLocalMemset(void *p, int v, size_t n, flagcxStream_t) {
  memset(p, v, n);
  return flagcxSuccess;
}

flagcxResult_t flagcxLocalRefresh(void *buff, size_t start, size_t offset, size_t count, size_t total, flagcxDataType_t dt,
                                  flagcxRedOp_t op, flagcxStream_t) {
  if (op != flagcxSum) return flagcxSuccess; // flagcx/core/c2c_algo.cc:596
  const size_t ts = sizeOf(dt);
  if (offset + count > total) die("refresh: offset + count exceeds totalCount");
  char *b = (char *)buff + start * ts;
  memset(b, 0, offset * ts);
  memset(b + (offset + count) * ts, 0, (total - offset - count) * ts);
  return flagcxSuccess;
}

flagcxResult_t flagcxLocalReduce(const void *const *src, int k, void *dst, size_t n, flagcxDataType_t dt, flagcxRedOp_t op,
                                 flagcxStream_t) {
  flagcxLocalReduceDesc d{src, dst, n};
  checkIndependent(&d, 1, k, sizeOf(dt));
  foldAny(src, k, dst, n, dt, op, false);
  return flagcxSuccess;
}

flagcxResult_t flagcxLocalReduceBatch(const flagcxLocalReduceDesc *d, int n, int k, flagcxDataType_t dt, flagcxRedOp_t op,
                                      flagcxStream_t) {
  checkIndependent(d, n, k, sizeOf(dt));
  for (int i = 0; i < n; i++) foldAny(d[i].sendbuffs, k, d[i].recvbuff, d[i].count, dt, op, false);
  return flagcxSuccess;
}

flagcxResult_t flagcxLocalReduceBatchSparse(const flagcxLocalReduceDesc *d, int n, int nlive, int nzero, flagcxDataType_t dt,
                                            flagcxRedOp_t op, flagcxStream_t) {
  if (nzero > 0 && op != flagcxSum) die("members can be left out of a sum only");
  checkIndependent(d, n, nlive, sizeOf(dt));
  for (int i = 0; i < n; i++) foldAny(d[i].sendbuffs, nlive, d[i].recvbuff, d[i].count, dt, op, nzero > 0);
  return flagcxSuccess;
}

flagcxResult_t flagcxLocalCopyFanout(const flagcxLocalFanoutDesc *d, int n, flagcxStream_t) {
  for (int a = 0; a < n; a++)
    for (int x = 0; x < d[a].ndsts; x++) {
      if (d[a].dsts[x] == d[a].src) continue;
      for (int b = 0; b < n; b++) {
        if (hit(d[a].dsts[x], d[a].bytes, d[b].src, d[b].bytes)) die("fan-out: a destination overlaps a source of the call");
        for (int y = 0; y < d[b].ndsts; y++)
          if ((a != b || x != y) && d[b].dsts[y] != d[b].src && hit(d[a].dsts[x], d[a].bytes, d[b].dsts[y], d[b].bytes))
            die("fan-out: two destinations overlap");
      }
    }
  for (int a = 0; a < n; a++)
    for (int x = 0; x < d[a].ndsts; x++)
      if (d[a].dsts[x] != d[a].src) memcpy(d[a].dsts[x], d[a].src, d[a].bytes);
  return flagcxSuccess;
}

} // extern "C"
