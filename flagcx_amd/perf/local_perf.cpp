// local_perf.cpp - C++ timing driver for the C ABI, in the manner of the
// reference's perf programs (size sweep -b..-e with factor -f, -w warm-up and -n
// timed iterations, defaults 5 and 20 as test/perf/tools.cc:81-86).  It measures
// what a C/C++ caller sees, without any Python in the launch path:
//
//   local_perf [-b minbytes] [-e maxbytes] [-f factor] [-w warmup] [-n iters] [-k nranks] [-t dtype] [-o op]
//   local_perf -L 1 [-n iters]      what a 4 KiB launch costs next to the runtime's own floor
//   local_perf -C 1 [-e bytes]      what this GPU's memory gives to read-only, write-only and mixed streams
//
// Per size: back-to-back launches bracketed by two HIP events (per-launch time and
// algorithmic GB/s = (k+1)*bytes/time), and launch -> hipStreamSynchronize wall time.
//
// -L: the library's 2-input fp32 sum over 4 KiB buffers beside an empty <<<1, 64>>> kernel and a
// 4 KiB hipMemcpyAsync device to device, all three timed the same three ways (back to back
// between two events, one launch between its own event pair, launch -> stream synchronise):
// what is left above the empty launch is the library's own share.
//
// -C: a read-only probe with the streaming shape of the reduce kernels (one-wavefront
// workgroups, one KiB of each of K streams per wavefront through clipped buffer descriptors,
// `nt` loads, optionally paced, resident wavefronts capped through an LDS reservation; lane 0
// stores 16 bytes per tile), swept over wavefronts per CU, inputs in flight and KiB per wavefront,
// best rate reported per K; then the library's fill (write-only), copy (1:1) and
// 8-input bf16 sum (8:1) at the same size.  Rates are bytes moved / time between two events.
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

__global__ void __launch_bounds__(64) emptyKernel() {}

// The least a 2-input sum can do: one 16-byte load per input and lane, one add, one store.
__global__ void __launch_bounds__(64) minimalSumKernel(const float4 *a, const float4 *b, float4 *c) {
  const unsigned i = blockIdx.x * 64u + threadIdx.x;
  const float4 x = a[i], y = b[i];
  c[i] = make_float4(x.x + y.x, x.y + y.y, x.z + y.z, x.w + y.w);
}

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <int K>
struct ProbeArgs {
  const void *src[K];
  void *out;       // 16 bytes per tile
  uint64_t bytes;  // per stream, a multiple of 1 KiB
  int inflight;    // 0: all K loads at once; 1, 2: the next stream is asked for when fewer are outstanding
  uint32_t magic;  // a word that the xor of a lane's loads never equals
};

template <int K, int U>
__global__ void __launch_bounds__(64) readProbeKernel(ProbeArgs<K> p) {
  const uint64_t off = (uint64_t)blockIdx.x * (1024u * U);
  if (off >= p.bytes) return;
  u32x4 in[K][U];
#pragma unroll
  for (int j = 0; j < K; j++) {
    __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void *)((const char *)p.src[j] + off), 0, 1024 * U, 0x00020000);
#pragma unroll
    for (int u = 0; u < U; u++) in[j][u] = __builtin_amdgcn_raw_buffer_load_b128(rs, threadIdx.x * 16u + u * 1024u, 0, 2 /* nt */);
    if (j + 1 < K && p.inflight) {
      if (p.inflight == 2) __builtin_amdgcn_s_waitcnt(0x0F70 | U);
      else __builtin_amdgcn_s_waitcnt(0x0F70 | 0);
    }
  }
  u32x4 acc = in[0][0];
#pragma unroll
  for (int j = 0; j < K; j++)
#pragma unroll
    for (int u = 0; u < U; u++)
      if (j || u) acc ^= in[j][u];
  // Every lane's loads must be needed, or the compiler moves them under the condition of the one
  // store (it did: such a probe "read" 24 TB/s).  So every lane tests what it loaded against a
  // value the data never has, and one lane's vector per tile goes out: 16 bytes written per K KiB read.
  const bool never = (acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == p.magic;
  if (never || threadIdx.x == (blockIdx.x & 63u)) ((u32x4 *)p.out)[blockIdx.x] = acc;
}

// LDS bytes that leave room for at most `waves` one-wavefront workgroups per CU (gfx950 hands
// out 160 KiB per CU in granules of 1280 bytes); 0: no cap.
static int ldsFor(int waves) {
  if (waves <= 0 || waves >= 32) return 0;
  const int each = 128 / (waves + 1) + 1;
  return each * 1280 > 65536 ? 65536 : each * 1280;
}

struct ProbeBest {
  double gbps;
  int waves, inflight, kib;
};

template <int K, int U>
static int readProbeShape(ProbeArgs<K> p, size_t bytes, hipStream_t st, hipEvent_t e0, hipEvent_t e1, ProbeBest *best) {
  const unsigned grid = (unsigned)((bytes + 1024 * U - 1) / (1024 * U));
  for (int inflight : {0, 1, 2}) {
    if (inflight && K == 1) continue;
    for (int waves : {0, 25, 21, 18, 16, 14, 11, 8}) {
      p.inflight = inflight;
      for (int i = 0; i < 2; i++) readProbeKernel<K, U><<<grid, 64, ldsFor(waves), st>>>(p);
      CK(hipEventRecord(e0, st));
      for (int i = 0; i < 5; i++) readProbeKernel<K, U><<<grid, 64, ldsFor(waves), st>>>(p);
      CK(hipEventRecord(e1, st));
      CK(hipEventSynchronize(e1));
      float ms = 0;
      CK(hipEventElapsedTime(&ms, e0, e1));
      const double gbps = (double)K * bytes * 5 / (ms * 1e-3) / 1e9;
      if (gbps > best->gbps) *best = ProbeBest{gbps, waves, inflight, U};
    }
  }
  return 0;
}

// K read streams of `bytes` each; one, two or four KiB of every stream per wavefront.
template <int K>
static int readProbe(const std::vector<void *> &src, void *out, size_t bytes, hipStream_t st, hipEvent_t e0, hipEvent_t e1,
                     ProbeBest *best) {
  ProbeArgs<K> p;
  for (int j = 0; j < K; j++) p.src[j] = src[j];
  p.out = out;
  p.bytes = bytes;
  p.inflight = 0;
  p.magic = 0x9e3779b9u; // the pool holds one repeated byte: the xor of any of its words is 0 or a repeated byte
  *best = ProbeBest{0, 0, 0, 1};
  if (readProbeShape<K, 1>(p, bytes, st, e0, e1, best)) return 1;
  if (readProbeShape<K, 2>(p, bytes, st, e0, e1, best)) return 1;
  if (K <= 4 && readProbeShape<K, (K <= 4 ? 4 : 1)>(p, bytes, st, e0, e1, best)) return 1;
  return 0;
}

// us per call: back to back between two events / one call between its own event pair (median) /
// call -> hipStreamSynchronize (median) / host time of the call itself (64 calls into an idle stream)
template <typename F>
static int threeWays(F call, hipStream_t st, hipEvent_t e0, hipEvent_t e1, int iters, double out[4]) {
  for (int i = 0; i < 200; i++) call();
  CK(hipStreamSynchronize(st));
  const int reps = iters * 50;
  // host time of a call: 64 calls into an idle stream (fewer than its queue holds), several times
  std::vector<double> h;
  for (int r = 0; r < 9; r++) {
    auto h0 = std::chrono::steady_clock::now();
    for (int i = 0; i < 64; i++) call();
    h.push_back(std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - h0).count() / 64);
    CK(hipStreamSynchronize(st));
  }
  std::sort(h.begin(), h.end());
  out[3] = h[h.size() / 2];
  CK(hipEventRecord(e0, st));
  for (int i = 0; i < reps; i++) call();
  CK(hipEventRecord(e1, st));
  CK(hipEventSynchronize(e1));
  float ms = 0;
  CK(hipEventElapsedTime(&ms, e0, e1));
  out[0] = ms * 1e3 / reps;
  std::vector<double> a, b;
  for (int i = 0; i < iters * 5; i++) {
    CK(hipEventRecord(e0, st));
    call();
    CK(hipEventRecord(e1, st));
    CK(hipEventSynchronize(e1));
    CK(hipEventElapsedTime(&ms, e0, e1));
    a.push_back(ms * 1e3);
  }
  for (int i = 0; i < iters * 5; i++) {
    auto t0 = std::chrono::steady_clock::now();
    call();
    CK(hipStreamSynchronize(st));
    b.push_back(std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count());
  }
  std::sort(a.begin(), a.end());
  std::sort(b.begin(), b.end());
  out[1] = a[a.size() / 2];
  out[2] = b[b.size() / 2];
  return 0;
}

int main(int argc, char **argv) {
  size_t minb = 1024, maxb = 1ull << 30;
  int factor = 2, warmup = 5, iters = 20, k = 2, dtype = flagcxFloat, op = flagcxSum, floorMode = 0, ceilingMode = 0;
  bool maxGiven = false;
  for (int i = 1; i + 1 < argc; i += 2) {
    const char *f = argv[i], *v = argv[i + 1];
    if (!strcmp(f, "-b")) minb = strtoull(v, 0, 0);
    else if (!strcmp(f, "-e")) { maxb = strtoull(v, 0, 0); maxGiven = true; }
    else if (!strcmp(f, "-L")) floorMode = atoi(v);
    else if (!strcmp(f, "-C")) ceilingMode = atoi(v);
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
  if (floorMode) {
    void *a = nullptr, *b = nullptr, *c = nullptr;
    CK(hipMalloc(&a, 4096));
    CK(hipMalloc(&b, 4096));
    CK(hipMalloc(&c, 4096));
    CK(hipMemset(a, 1, 4096));
    CK(hipMemset(b, 2, 4096));
    const void *two[2] = {a, b};
    // the four are timed in turn, five rounds, and the median round of each is reported: the host's
    // clock and caches drift over a run, and whoever goes first would carry that
    const char *names[4] = {"library_reduce2_fp32", "empty_kernel_1x64", "minimal_sum_kernel_4x64", "hipMemcpyAsync_d2d"};
    std::vector<double> res[4][4];
    for (int round = 0; round < 5; round++) {
      double t[4];
      if (threeWays([&]() { (void)flagcxLocalReduce(two, 2, c, 1024, flagcxFloat, flagcxSum, &st); }, st.base, e0, e1, iters, t)) return 1;
      for (int i = 0; i < 4; i++) res[0][i].push_back(t[i]);
      if (threeWays([&]() { emptyKernel<<<1, 64, 0, st.base>>>(); }, st.base, e0, e1, iters, t)) return 1;
      for (int i = 0; i < 4; i++) res[1][i].push_back(t[i]);
      if (threeWays([&]() { minimalSumKernel<<<4, 64, 0, st.base>>>((const float4 *)a, (const float4 *)b, (float4 *)c); }, st.base,
                    e0, e1, iters, t))
        return 1;
      for (int i = 0; i < 4; i++) res[2][i].push_back(t[i]);
      if (threeWays([&]() { (void)hipMemcpyAsync(c, a, 4096, hipMemcpyDeviceToDevice, st.base); }, st.base, e0, e1, iters, t)) return 1;
      for (int i = 0; i < 4; i++) res[3][i].push_back(t[i]);
    }
    printf("# 4 KiB: us per call, back to back / one call between events / call -> stream synchronise / host time of the call\n");
    for (int k = 0; k < 4; k++) {
      double m[4];
      for (int i = 0; i < 4; i++) {
        std::sort(res[k][i].begin(), res[k][i].end());
        m[i] = res[k][i][res[k][i].size() / 2];
      }
      printf("floor %s %.3f %.3f %.3f %.3f\n", names[k], m[0], m[1], m[2], m[3]);
    }
    return 0;
  }
  if (ceilingMode) {
    // Every probe walks 16 GiB (or -e bytes), 64 times the 256 MB memory-side cache, which keeps
    // part of what it held whatever the order of accesses (a 2 GiB walk reads 9.4 TB/s, more than
    // the HBM interface moves): K read streams of total / K each, a fill of the whole area, a copy of
    // one half onto the other.  The 8-input sum runs at the headline size, 8 x 256 MiB placed by
    // flagcxLocalPlaceBuffers, over four sets of buffers in turn.
    const size_t total = (maxGiven ? maxb : (16ull << 30)) & ~(size_t)(8 * 1024 - 1);
    char *pool = nullptr;
    void *out = nullptr;
    CK(hipMalloc((void **)&pool, total + total / 8));
    CK(hipMalloc(&out, total / 64 + 4096));
    CK(hipMemset(pool, 0x3c, total + total / 8)); // 0x3c3c: a small normal number in bf16 and fp16
    printf("# %zu bytes walked per probe; GB/s of bytes moved, best of the launch shapes tried\n", total);
    ProbeBest b;
    auto streams = [&](int n) {
      std::vector<void *> v(8, pool);
      for (int j = 0; j < n; j++) v[j] = pool + (total / n) * j;
      return v;
    };
    if (readProbe<1>(streams(1), out, total, st.base, e0, e1, &b)) return 1;
    printf("ceiling read_only_1_stream %.1f waves=%d inflight=%d KiB_per_wave=%d\n", b.gbps, b.waves, b.inflight, b.kib);
    if (readProbe<2>(streams(2), out, total / 2, st.base, e0, e1, &b)) return 1;
    printf("ceiling read_only_2_streams %.1f waves=%d inflight=%d KiB_per_wave=%d\n", b.gbps, b.waves, b.inflight, b.kib);
    if (readProbe<4>(streams(4), out, total / 4, st.base, e0, e1, &b)) return 1;
    printf("ceiling read_only_4_streams %.1f waves=%d inflight=%d KiB_per_wave=%d\n", b.gbps, b.waves, b.inflight, b.kib);
    if (readProbe<8>(streams(8), out, total / 8, st.base, e0, e1, &b)) return 1;
    printf("ceiling read_only_8_streams %.1f waves=%d inflight=%d KiB_per_wave=%d\n", b.gbps, b.waves, b.inflight, b.kib);
    auto rate = [&](auto call, double moved, const char *name) -> int {
      for (int i = 0; i < 3; i++) call();
      CK(hipEventRecord(e0, st.base));
      for (int i = 0; i < 10; i++) call();
      CK(hipEventRecord(e1, st.base));
      CK(hipEventSynchronize(e1));
      float ms = 0;
      CK(hipEventElapsedTime(&ms, e0, e1));
      printf("ceiling %s %.1f\n", name, moved * 10 / (ms * 1e-3) / 1e9);
      return 0;
    };
    if (rate([&]() { (void)flagcxLocalMemset(pool, 0x3c, total, &st); }, (double)total, "write_only_fill")) return 1;
    if (rate([&]() { (void)flagcxLocalMemcpy(pool + total / 2, pool, total / 2, &st); }, (double)total, "copy_1_to_1")) return 1;
    const size_t each = 256ull << 20;
    void *bufs[4][9];
    for (int s = 0; s < 4; s++)
      if (flagcxLocalPlaceBuffers(pool + (size_t)s * 10 * each, 10 * each, each, 9, bufs[s]) != flagcxSuccess) return 1;
    int turn = 0;
    if (rate([&]() { (void)flagcxLocalReduce(bufs[turn & 3], 8, bufs[turn & 3][8], each / 2, flagcxBfloat16, flagcxSum, &st); turn++; },
             9.0 * each, "reduce_8_to_1_bf16_sum"))
      return 1;
    return 0;
  }
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
