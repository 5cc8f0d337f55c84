// copy_kernels.hip - chunk copy, strided pack / unpack, pointer-list flatten /
// unflatten and zero-fill kernels for gfx950.
//
// All movers share one shape: a workgroup is one wavefront; a lane moves one
// 16-byte vector per instruction, so each wavefront-wide access is a coalesced
// 1 KiB request and a tile is U consecutive KiB of one chunk.  blockIdx.y walks
// chunks (or list entries), blockIdx.x walks tiles inside a chunk.  Buffer
// descriptors are clipped to the tile, so ragged chunk ends need no branches.
// A contiguous copy whose two sides differ modulo 16 goes to the one-input reduce
// kernel for misaligned sources (aligned loads, lane shifts); strided forms whose chunk
// sizes or strides are not multiples of 16 split every chunk that way on its own
// (copyWaveRaggedKernel), chunks under 320 bytes go through an element path at the
// widest width every address shares.
// HBM bound: 2 bytes of traffic per payload byte (1 for fills); no LDS, no MFMA.
#include "launch.h"
#include "reduce_device.h"

namespace flagcx_amd {

constexpr int kCopyUnroll = 1;
constexpr uint64_t kMaxGridX = 1u << 24;
constexpr uint64_t kMaxGridY = 65535;
// chunks shorter than this stay on the element path (200 000 misaligned chunks of 200 / 500 / 1000 bytes:
// element path 20 / 26 / 17 % of peak, a workgroup per chunk that splits it 16 / 38 / 55 %)
constexpr uint64_t kRaggedMinBytes = 320;

static unsigned lowBits(uint64_t x) { return (unsigned)(x & 15u); }

struct CopyParams {
  const char *src;
  char *dst;
  uint64_t nchunks, chunkBytes, srcStride, dstStride;
  uint64_t head; // bytes before the 16-byte body (single-chunk case only)
  uint64_t body; // bytes in the body of each chunk
  uint64_t tail; // bytes after the body (single-chunk case only)
  uint32_t flat; // copyWaveRaggedKernel: one workgroup per chunk, blockIdx.x walks the chunks
};

struct ListParams {
  const char *src[FLAGCX_MAX_RANKS];
  char *dst[FLAGCX_MAX_RANKS];
};

// LIST: 0 both sides strided, 1 sources from a pointer list, 2 destinations from one
// TILED: a chunk's first tile is cut short by the destination's position inside its
// 128-byte cache line, so that all later tiles store whole lines (a tile that starts
// inside a line shares its first and last line with tiles that run on other XCDs: two
// partial writes per line, 66-76 % of peak for a 256 MiB copy where whole lines reach
// 83 %).  Chunks whose destinations all start on a line take the kernel without it.
template <int U, int LIST, bool TILED>
__device__ __forceinline__ void copyWaveBody(const CopyParams &p, const ListParams *l) {
  constexpr uint32_t kTileBytes = 64u * U * 16u;
  const uint32_t voff = threadIdx.x * 16u;
  for (uint64_t c = blockIdx.y; c < p.nchunks; c += gridDim.y) {
    const char *s = (LIST == 1 ? l->src[c] : p.src + c * p.srcStride) + p.head;
    char *d = (LIST == 2 ? l->dst[c] : p.dst + c * p.dstStride) + p.head;
    const uint32_t lead = TILED ? (uint32_t)((uintptr_t)d & 127u) : 0;
    const uint64_t ntiles = (p.body + lead + kTileBytes - 1) / kTileBytes;
    for (uint64_t t = blockIdx.x; t < ntiles; t += gridDim.x) {
      const uint64_t off = TILED ? (t ? t * kTileBytes - lead : 0) : t * kTileBytes;
      const uint64_t left = p.body - off;
      const uint32_t cap = TILED ? (t ? kTileBytes : kTileBytes - lead) : kTileBytes;
      const uint32_t span = left < cap ? (uint32_t)left : cap;
      __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void *)(s + off), 0, span, kRsrcFlags);
      __amdgpu_buffer_rsrc_t rd = __builtin_amdgcn_make_buffer_rsrc((void *)(d + off), 0, span, kRsrcFlags);
      u32x4 v[U];
#pragma unroll
      for (int u = 0; u < U; u++) v[u] = __builtin_amdgcn_raw_buffer_load_b128(rs, voff + u * 1024u, 0, kLoadAux);
#pragma unroll
      for (int u = 0; u < U; u++) __builtin_amdgcn_raw_buffer_store_b128(v[u], rd, voff + u * 1024u, 0, kStoreAux);
    }
  }
  // head / tail bytes of an unaligned single chunk: fewer than 32, one lane each
  if (blockIdx.x == gridDim.x - 1 && blockIdx.y == 0) {
    const uint64_t edge = p.head + p.tail;
    if (threadIdx.x < edge) {
      const uint64_t i = threadIdx.x < p.head ? threadIdx.x : p.head + p.body + (threadIdx.x - p.head);
      const char *s = (LIST == 1 ? l->src[0] : p.src);
      char *d = (LIST == 2 ? l->dst[0] : p.dst);
      d[i] = s[i];
    }
  }
}

// The strided form carries 80 bytes of arguments; only the list forms pay for the
// pointer tables.
template <int U, bool TILED>
__global__ void __launch_bounds__(64) copyWaveKernel(CopyParams p) {
  copyWaveBody<U, 0, TILED>(p, nullptr);
}
template <int U, int LIST, bool TILED>
__global__ void __launch_bounds__(64) copyWaveListKernel(CopyParams p, ListParams l) {
  copyWaveBody<U, LIST, TILED>(p, &l);
}

// Several chunks whose sizes, strides or bases are not multiples of 16: every chunk is
// split on its own into the bytes up to the destination's next 16-byte line, a body of
// 16-byte vectors stored aligned (first tile cut short at a cache line, as above), and
// the bytes after it.  A source body at another offset modulo 16 than its destination is
// read with aligned loads, one granule further than the tile, and put in place with lane
// shifts, as reduceWaveShiftKernel does for its sources.
template <int LIST>
__device__ __forceinline__ void copyWaveRaggedBody(const CopyParams &p, const ListParams *l) {
  const uint32_t lane = threadIdx.x;
  // chunks by blockIdx.y and a chunk's tiles by blockIdx.x, or (p.flat, short chunks) chunks by
  // blockIdx.x, which may be longer than the 65535 a grid allows in y, and all tiles of a chunk in turn
  const uint64_t c0 = p.flat ? blockIdx.x : blockIdx.y, cStep = p.flat ? gridDim.x : gridDim.y;
  const uint64_t t0 = p.flat ? 0 : blockIdx.x, tStep = p.flat ? 1 : gridDim.x;
  for (uint64_t c = c0; c < p.nchunks; c += cStep) {
    const char *s = LIST == 1 ? l->src[c] : p.src + c * p.srcStride;
    char *d = LIST == 2 ? l->dst[c] : p.dst + c * p.dstStride;
    uint64_t head = (16u - ((uintptr_t)d & 15u)) & 15u;
    if (head > p.chunkBytes) head = p.chunkBytes;
    const uint64_t body = (p.chunkBytes - head) & ~15ull;
    const uint64_t tail = p.chunkBytes - head - body;
    const char *sb = s + head;
    char *db = d + head;
    const uint32_t lead = (uint32_t)((uintptr_t)db & 127u);
    const uint32_t shift = (uint32_t)((uintptr_t)sb & 15u);
    const char *base = sb - shift;                               // aligned granules that hold the body
    const uint64_t granules = body ? body / 16 + (shift ? 1 : 0) : 0;
    const uint64_t ntiles = (body + lead + 1023) / 1024;
    for (uint64_t t = t0; t < ntiles; t += tStep) {
      const uint64_t off = t ? t * 1024 - lead : 0;
      const uint64_t left = body - off;
      const uint32_t cap = t ? 1024u : 1024u - lead;
      const uint32_t span = left < cap ? (uint32_t)left : cap;
      const uint64_t g0 = off / 16;
      const uint64_t leftG = granules > g0 ? granules - g0 : 0;
      __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
          (void *)(base + g0 * 16), 0, (uint32_t)(leftG < 64 ? leftG : 64) * 16u, kRsrcFlags);
      u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rs, lane * 16u, 0, kLoadAux);
      if (shift) { // the same for every lane of the chunk
        __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(
            (void *)(base + g0 * 16 + 1024), 0, leftG > 64 ? 16u : 0u, kRsrcFlags);
        const u32x4 ahead = __builtin_amdgcn_raw_buffer_load_b128(ra, lane * 16u, 0, kLoadAux);
        u32x4 hi;
#pragma unroll
        for (int w = 0; w < 4; w++) {
          const uint32_t fromNext = __builtin_amdgcn_readfirstlane(ahead[w]); // granule 0 of the next tile
          hi[w] = (uint32_t)__builtin_amdgcn_update_dpp((int)fromNext, (int)v[w], 0x130, 0xf, 0xf, false);
        }
        v = funnel16(v, hi, shift >> 2, shift & 3u);
      }
      __amdgpu_buffer_rsrc_t rd = __builtin_amdgcn_make_buffer_rsrc((void *)(db + off), 0, span, kRsrcFlags);
      __builtin_amdgcn_raw_buffer_store_b128(v, rd, lane * 16u, 0, kStoreAux);
    }
    // the chunk's bytes before and after its body: fewer than 32, one lane each
    if ((p.flat || blockIdx.x == gridDim.x - 1) && lane < head + tail) {
      const uint64_t i = lane < head ? lane : head + body + (lane - head);
      d[i] = s[i];
    }
  }
}
template <int LIST>
__global__ void __launch_bounds__(64) copyWaveRaggedKernel(CopyParams p, ListParams l) {
  copyWaveRaggedBody<LIST>(p, &l);
}

// Element path: W-byte units, chunk by chunk.
template <typename W, int LIST>
__device__ __forceinline__ void copyElemBody(const CopyParams &p, const ListParams *l) {
  const uint64_t n = p.chunkBytes / sizeof(W);
  const uint64_t stride = (uint64_t)gridDim.x * 256;
  for (uint64_t c = blockIdx.y; c < p.nchunks; c += gridDim.y) {
    const W *s = (const W *)(LIST == 1 ? l->src[c] : p.src + c * p.srcStride);
    W *d = (W *)(LIST == 2 ? l->dst[c] : p.dst + c * p.dstStride);
    for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) d[i] = s[i];
  }
}
template <typename W>
__global__ void __launch_bounds__(256) copyElemKernel(CopyParams p) {
  copyElemBody<W, 0>(p, nullptr);
}
template <typename W, int LIST>
__global__ void __launch_bounds__(256) copyElemListKernel(CopyParams p, ListParams l) {
  copyElemBody<W, LIST>(p, &l);
}

template <int LIST>
static int launchCopyT(const CopyParams &p, const ListParams &l, bool vector, unsigned width,
                       hipStream_t stream) {
  const uint64_t gy = p.nchunks < kMaxGridY ? p.nchunks : kMaxGridY;
  if (vector) {
    constexpr uint64_t tileBytes = 64ull * kCopyUnroll * 16ull;
    // does every chunk's destination body start on a 128-byte line?
    bool onLines = true;
    if (LIST == 2) {
      for (uint64_t j = 0; j < p.nchunks; j++) onLines = onLines && (((uintptr_t)l.dst[j] + p.head) & 127u) == 0;
    } else {
      onLines = (((uintptr_t)p.dst + p.head) & 127u) == 0 && (p.nchunks == 1 || (p.dstStride & 127u) == 0);
    }
    uint64_t gx = (p.body + (onLines ? 0 : 127) + tileBytes - 1) / tileBytes;
    if (gx < 1) gx = 1;
    if (gx > kMaxGridX) gx = kMaxGridX;
    const int lds = ldsReservation(launchShapeFor(0, 0).waves);
    const dim3 grid((unsigned)gx, (unsigned)gy);
    if (LIST == 0) {
      if (onLines) copyWaveKernel<kCopyUnroll, false><<<grid, dim3(64), lds, stream>>>(p);
      else copyWaveKernel<kCopyUnroll, true><<<grid, dim3(64), lds, stream>>>(p);
    } else {
      if (onLines) copyWaveListKernel<kCopyUnroll, LIST, false><<<grid, dim3(64), lds, stream>>>(p, l);
      else copyWaveListKernel<kCopyUnroll, LIST, true><<<grid, dim3(64), lds, stream>>>(p, l);
    }
    return (int)hipGetLastError();
  }
  if (p.nchunks > 1 && p.chunkBytes >= kRaggedMinBytes) {
    // Workgroups per chunk.  Every workgroup pays for the split of its chunk, so short chunks
    // (up to 16 tiles) get one workgroup each, and a launch of up to 320 MiB in all gives each
    // workgroup about two tiles; beyond that one tile per workgroup, as the other movers have it.
    // Measured on MI355X, misaligned packs, percent of peak: 200 000 chunks of 1 / 1.5 / 4 / 9 KB
    // 54 / 58 / 40 / 62 with a workgroup per tile, 68 / 72 / 76 / 80 with one per chunk; 64 KiB
    // - 64 MiB chunks, 256 MiB in all: 66-75 with a workgroup per tile, 80-84 with two tiles each;
    // 1 GiB in all: 78-79 against 70-74 (four tiles each).
    const uint64_t perChunk = (p.chunkBytes + 127 + 1023) / 1024 + 1; // tiles of the longest possible body, cut at a line
    uint64_t gx = perChunk;
    CopyParams q = p;
    uint64_t gyr = gy;
    if (perChunk <= 16) {
      q.flat = 1;
      gx = p.nchunks < kMaxGridX ? p.nchunks : kMaxGridX;
      gyr = 1;
    } else {
      const uint64_t all = perChunk * p.nchunks;
      const uint64_t target = all <= 160 * 1024 ? 65536 : all <= 320 * 1024 ? 131072 : 0;
      if (target) {
        const uint64_t most = target / gy ? target / gy : 1;
        if (gx > most) gx = most;
      }
    }
    if (gx > kMaxGridX) gx = kMaxGridX;
    copyWaveRaggedKernel<LIST><<<dim3((unsigned)gx, (unsigned)gyr), dim3(64), ldsReservation(launchShapeFor(0, 0).waves), stream>>>(q, l);
    return (int)hipGetLastError();
  }
  uint64_t gx = (p.chunkBytes / width + 255) / 256;
  const uint64_t cap = (uint64_t)deviceInfo().numCU * 16;
  if (gx > cap) gx = cap;
  if (gx < 1) gx = 1;
  const dim3 grid((unsigned)gx, (unsigned)gy);
#define FLAGCX_ELEM(W)                                                           \
  do {                                                                         \
    if (LIST == 0) copyElemKernel<W><<<grid, dim3(256), 0, stream>>>(p);       \
    else copyElemListKernel<W, LIST><<<grid, dim3(256), 0, stream>>>(p, l);    \
  } while (0)
  switch (width) {
    case 8: FLAGCX_ELEM(uint64_t); break;
    case 4: FLAGCX_ELEM(uint32_t); break;
    case 2: FLAGCX_ELEM(uint16_t); break;
    default: FLAGCX_ELEM(uint8_t); break;
  }
#undef FLAGCX_ELEM
  return (int)hipGetLastError();
}

int launchCopy2D(const Copy2D &c) {
  CopyParams p{};
  ListParams l{};
  p.src = (const char *)c.src;
  p.dst = (char *)c.dst;
  p.nchunks = c.nchunks;
  p.chunkBytes = c.chunkBytes;
  p.srcStride = c.srcStride;
  p.dstStride = c.dstStride;
  const int list = c.srcList ? 1 : (c.dstList ? 2 : 0);

  // Collect every chunk base address modulo 16 on both sides.
  unsigned orBits = 0;       // union of differing low bits -> common alignment
  bool sameMis = true;       // src and dst of each chunk share (addr % 16)
  bool allAligned = true;    // every chunk base is 16-byte aligned
  if (list) {
    for (uint64_t j = 0; j < c.nchunks; j++) {
      const uint64_t s = list == 1 ? (uint64_t)c.srcList[j] : (uint64_t)c.src + j * c.srcStride;
      const uint64_t d = list == 2 ? (uint64_t)c.dstList[j] : (uint64_t)c.dst + j * c.dstStride;
      if (list == 1) l.src[j] = (const char *)c.srcList[j]; else l.dst[j] = (char *)c.dstList[j];
      orBits |= lowBits(s) | lowBits(d);
      if (lowBits(s) != lowBits(d)) sameMis = false;
      if (lowBits(s) || lowBits(d)) allAligned = false;
    }
  } else {
    const uint64_t s = (uint64_t)c.src, d = (uint64_t)c.dst;
    orBits = lowBits(s) | lowBits(d);
    if (c.nchunks > 1) orBits |= lowBits(c.srcStride) | lowBits(c.dstStride);
    sameMis = lowBits(s) == lowBits(d);
    allAligned = (orBits == 0);
  }

  bool vector;
  if (c.nchunks == 1) {
    // one contiguous run: peel bytes up to the destination's next 16-byte line,
    // then vectors; a source at another offset modulo 16 is read unaligned
    const char *src0 = list == 1 ? l.src[0] : p.src;
    char *dst0 = list == 2 ? l.dst[0] : p.dst;
    uint64_t head = (16u - lowBits((uint64_t)dst0)) & 15u;
    if (head > c.chunkBytes) head = c.chunkBytes;
    p.head = head;
    p.body = (c.chunkBytes - head) & ~15ull;
    p.tail = c.chunkBytes - head - p.body;
    vector = sameMis;
    if (!vector) {
      // the two sides sit at different offsets modulo 16: a one-input byte "reduce",
      // which reads the source with aligned loads and puts it in place with lane shifts
      ReduceCall r{};
      r.src[0] = src0;
      r.dst = dst0;
      r.count = c.chunkBytes;
      r.k = 1;
      r.op = 0; // sum of one input: the input
      r.stream = c.stream;
      return reduceLauncherFor(1 /* flagcxUint8 */)(r);
    }
  } else {
    vector = allAligned && (c.chunkBytes & 15u) == 0;
    p.body = c.chunkBytes;
  }
  unsigned width = 1;
  if (!vector) {
    const unsigned bits = orBits | lowBits(c.chunkBytes);
    width = (bits & 1u) ? 1 : (bits & 2u) ? 2 : (bits & 4u) ? 4 : 8;
  }
  switch (list) {
    case 1: return launchCopyT<1>(p, l, vector, width, c.stream);
    case 2: return launchCopyT<2>(p, l, vector, width, c.stream);
    default: return launchCopyT<0>(p, l, vector, width, c.stream);
  }
}

// ------------------------------------------------------------------ fan-out
// One source, several destinations (what a broadcast or an all-gather inside a simulated
// cluster moves): a wavefront loads its KiB once and stores it to every destination, so the
// launch reads each source once instead of once per destination.  blockIdx.y picks the
// copy, blockIdx.x walks its tiles; the first tile is cut short so that the others start
// on a 128-byte line of the first destination.

struct FanSeg {
  const char *src;
  char *dst[kFanMaxDst];
  uint64_t head, body, tail; // bytes up to the 16-byte body, in it, behind it (the same on every side)
  uint32_t ndst, lead;
};
struct FanParams {
  FanSeg seg[kFanMaxSeg];
};

__global__ void __launch_bounds__(64) fanoutWaveKernel(FanParams p) {
  const FanSeg &s = p.seg[blockIdx.y];
  const uint32_t voff = threadIdx.x * 16u;
  const uint64_t ntiles = (s.body + s.lead + 1023) / 1024;
  for (uint64_t t = blockIdx.x; t < ntiles; t += gridDim.x) {
    const uint64_t off = t ? t * 1024 - s.lead : 0;
    const uint64_t left = s.body - off;
    const uint32_t cap = t ? 1024u : 1024u - s.lead;
    const uint32_t span = left < cap ? (uint32_t)left : cap;
    __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void *)(s.src + s.head + off), 0, span, kRsrcFlags);
    const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rs, voff, 0, kLoadAux);
    for (uint32_t d = 0; d < s.ndst; d++) {
      __amdgpu_buffer_rsrc_t rd = __builtin_amdgcn_make_buffer_rsrc((void *)(s.dst[d] + s.head + off), 0, span, kRsrcFlags);
      __builtin_amdgcn_raw_buffer_store_b128(v, rd, voff, 0, kStoreAux);
    }
  }
  // the bytes before and after the body: fewer than 32, one lane each
  if (blockIdx.x == gridDim.x - 1) {
    const uint64_t edge = s.head + s.tail;
    if (threadIdx.x < edge) {
      const uint64_t i = threadIdx.x < s.head ? threadIdx.x : s.head + s.body + (threadIdx.x - s.head);
      const char b = s.src[i];
      for (uint32_t d = 0; d < s.ndst; d++) s.dst[d][i] = b;
    }
  }
}

int launchFanout(const FanoutCall *calls, int n, hipStream_t stream) {
  for (int base = 0; base < n; base += kFanMaxSeg) {
    const int m = n - base < kFanMaxSeg ? n - base : kFanMaxSeg;
    FanParams p{};
    uint64_t maxTiles = 1;
    int maxDst = 0;
    for (int i = 0; i < m; i++) {
      const FanoutCall &c = calls[base + i];
      FanSeg &s = p.seg[i];
      if (c.ndst < 1 || c.ndst > kFanMaxDst) return (int)hipErrorInvalidValue;
      s.src = (const char *)c.src;
      s.ndst = (uint32_t)c.ndst;
      if (c.ndst > maxDst) maxDst = c.ndst;
      for (int d = 0; d < c.ndst; d++) {
        if (lowBits((uint64_t)c.dst[d]) != lowBits((uint64_t)c.src)) return (int)hipErrorInvalidValue;
        s.dst[d] = (char *)c.dst[d];
      }
      uint64_t head = (16u - lowBits((uint64_t)c.src)) & 15u;
      if (head > c.bytes) head = c.bytes;
      s.head = head;
      s.body = (c.bytes - head) & ~15ull;
      s.tail = c.bytes - head - s.body;
      s.lead = s.body ? (uint32_t)(((uintptr_t)c.dst[0] + head) & 127u) : 0;
      const uint64_t tiles = (s.body + s.lead + 1023) / 1024;
      if (tiles > maxTiles) maxTiles = tiles;
    }
    if (maxTiles > kMaxGridX) maxTiles = kMaxGridX;
    // Wavefronts per CU.  Measured on MI355X, one source of 256 MiB to 2 / 3 / 4 / 5 / 6 / 8
    // destinations, TB/s of (1 + n) x 256 MiB: no cap 6.43 / 6.18 / 5.93 / 5.91 / 5.79 / 5.52,
    // 25 per CU 6.43 / 6.19 / 6.17 / 6.09 / 5.97 / 5.58, 21: - / 6.20 / 6.08 / 6.15 / 6.11 / 6.00,
    // 16: 5.88 / 5.95 / 6.03 / 6.05 / 5.99 / 5.99 (workgroups of two wavefronts the same, of
    // four 0.3-0.5 lower; 2 or 4 KiB per wavefront 0.1-0.9 lower under every cap; the same
    // copies one by one: 6.65 of 2 n x 256 MiB, i.e. 1.3-1.55 x the time).
    const int lds = ldsReservation(maxDst >= 3 ? 21 : 0);
    fanoutWaveKernel<<<dim3((unsigned)maxTiles, (unsigned)m), dim3(64), lds, stream>>>(p);
    const int e = (int)hipGetLastError();
    if (e) return e;
  }
  return (int)hipSuccess;
}

// ------------------------------------------------------------------- fills

struct FillParams {
  char *ptr[2];
  uint64_t head[2], body[2], tail[2];
  uint32_t pattern;
};

// Up to two byte ranges in one launch (blockIdx.y picks the range).  Unlike the
// kernels that read, a pure store stream runs best from workgroups of four
// wavefronts, each wavefront storing one consecutive KiB (4 GiB on MI355X:
// 90 % of the HBM peak, against 60 % from one-wavefront workgroups of one KiB and
// 81 % from one-wavefront workgroups of four).
constexpr int kFillWaves = 4;
__global__ void __launch_bounds__(64 * kFillWaves) fillWaveKernel(FillParams p) {
  constexpr uint32_t kTileBytes = 1024u;
  const int r = blockIdx.y;
  char *base = p.ptr[r] + p.head[r];
  const uint64_t body = p.body[r];
  // the first tile is cut short by the range's position inside its 128-byte cache line,
  // so that every later tile stores whole lines: tiles that start inside a line share
  // lines with tiles of other workgroups, and a store stream of partial lines runs at
  // 48 % of peak where whole lines reach 88-90 % (1 GiB, range 16 bytes into a line)
  const uint32_t lead = (uint32_t)((uintptr_t)base & 127u);
  const uint64_t ntiles = (body + lead + kTileBytes - 1) / kTileBytes;
  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
  const uint32_t voff = lane * 16u;
  const u32x4 v = {p.pattern, p.pattern, p.pattern, p.pattern};
  for (uint64_t t = (uint64_t)blockIdx.x * kFillWaves + wave; t < ntiles; t += (uint64_t)gridDim.x * kFillWaves) {
    const uint64_t off = t ? t * kTileBytes - lead : 0;
    const uint64_t left = body - off;
    const uint32_t cap = t ? kTileBytes : kTileBytes - lead;
    const uint32_t span = left < cap ? (uint32_t)left : cap;
    __amdgpu_buffer_rsrc_t rd = __builtin_amdgcn_make_buffer_rsrc((void *)(base + off), 0, span, kRsrcFlags);
    __builtin_amdgcn_raw_buffer_store_b128(v, rd, voff, 0, kStoreAux);
  }
  if (blockIdx.x == gridDim.x - 1 && wave == 0) {
    const uint64_t edge = p.head[r] + p.tail[r];
    if (lane < edge) {
      const uint64_t i = lane < p.head[r] ? lane : p.head[r] + body + (lane - p.head[r]);
      p.ptr[r][i] = (char)(p.pattern & 0xffu);
    }
  }
}

int launchFill(void *p0, uint64_t n0, void *p1, uint64_t n1, int value, hipStream_t stream) {
  FillParams p{};
  void *ptrs[2] = {p0, p1};
  uint64_t lens[2] = {n0, n1};
  int nr = 0;
  uint64_t maxBody = 0;
  for (int r = 0; r < 2; r++) {
    if (lens[r] == 0) continue;
    uint64_t head = (16u - lowBits((uint64_t)ptrs[r])) & 15u;
    if (head > lens[r]) head = lens[r];
    p.ptr[nr] = (char *)ptrs[r];
    p.head[nr] = head;
    p.body[nr] = (lens[r] - head) & ~15ull;
    p.tail[nr] = lens[r] - head - p.body[nr];
    if (p.body[nr] > maxBody) maxBody = p.body[nr];
    nr++;
  }
  if (nr == 0) return (int)hipSuccess;
  const uint32_t b = (uint32_t)(value & 0xff);
  p.pattern = b | (b << 8) | (b << 16) | (b << 24);
  constexpr uint64_t groupBytes = 1024ull * kFillWaves;
  uint64_t gx = (maxBody + 127 + groupBytes - 1) / groupBytes; // a range inside a line has a short first tile
  if (gx < 1) gx = 1;
  if (gx > kMaxGridX) gx = kMaxGridX;
  fillWaveKernel<<<dim3((unsigned)gx, (unsigned)nr), dim3(64 * kFillWaves), 0, stream>>>(p);
  return (int)hipGetLastError();
}

} // namespace flagcx_amd
