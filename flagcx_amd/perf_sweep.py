"""Message-size sweep of the local primitives on one GPU, in the manner of the
reference's perf tests (5 warm-up + 20 timed iterations per size,
test/perf/tools.cc:81-86):

    python -m flagcx_amd.perf_sweep [--min 1024] [--max 1073741824] [--json out.json] [--rotate]

Per size S (bytes per buffer):
  reduce2   2-input fp32 sum of S bytes per buffer          algorithmic bytes 3*S
  pack      8 chunks of S/8 at stride S gathered contiguous  2*S
  unpack    the inverse scatter                              2*S
  memcpy    contiguous device-to-device copy                 2*S
  memset    byte fill (the zero-fill of a refresh)           S
Times are HIP-event medians per launch; GB/s uses the algorithmic bytes.
Small sizes are cache resident; from a few hundred MiB on the data streams from HBM.
With the same buffers launch after launch, part of what one launch wrote (up to 256 MiB)
is still in the memory-side cache for the next.  --rotate uses several sets of buffers
in turn (up to 16, enough for 1.5 GiB per kernel), so that from 8 MiB on no launch
finds its buffers there; the column `sets` says how many.
"""
import argparse
import ctypes as C
import json
import sys

import torch

from flagcx_amd import local as L


def timed(fn, warmup=5, iters=20, sets=1):
    """fn(i) runs the kernel on buffer set i; median and minimum of `iters` single launches."""
    for i in range(max(warmup, sets)):
        fn(i % sets)
    torch.cuda.synchronize()
    ts = []
    for i in range(iters):
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        fn(i % sets)
        e1.record()
        e1.synchronize()
        ts.append(e0.elapsed_time(e1) * 1e3)
    ts.sort()
    return ts[len(ts) // 2], ts[0]


def back_to_back(fn, n, sets=1):
    for i in range(20):
        fn(i % sets)
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    for i in range(n):
        fn(i % sets)
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / n


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--min", type=int, default=1 << 10)
    ap.add_argument("--max", type=int, default=1 << 30)
    ap.add_argument("--json", default=None)
    ap.add_argument("--rotate", action="store_true", help="several sets of buffers in turn")
    args = ap.parse_args()
    torch.cuda.set_device(0)
    lib = L.lib()
    L.check(lib.flagcxLocalInit())
    st = L.current_stream()
    sref = C.byref(st)
    f32, opsum = int(L.DataType.Float32), int(L.RedOp.Sum)
    g = torch.Generator(device="cuda").manual_seed(0)
    rows = []
    size = args.min
    print("%12s %10s | %9s %9s | %9s %9s | %9s %9s | %9s %9s | %9s %9s | %8s" %
          ("bytes", "sets", "reduce2us", "GB/s", "pack us", "GB/s", "unpack us", "GB/s", "memcpy us", "GB/s",
           "memset us", "GB/s", "b2b us"))
    while size <= args.max:
        n = size // 4
        chunk = size // 8
        nsets = 1
        if args.rotate:
            nsets = max(2, min(16, ((3 << 29) + 2 * size - 1) // (2 * size)))
        bufs = []
        for _ in range(nsets):
            a = torch.rand(n, device="cuda", generator=g) * 2 - 1
            b = torch.rand(n, device="cuda", generator=g) * 2 - 1
            c = torch.empty(n, device="cuda")
            # sparse source of 8*size bytes holding 8 chunks of size/8 at stride `size`
            sparse = torch.rand(8 * n, device="cuda", generator=g)
            staged = torch.empty(n, device="cuda")
            bufs.append((a, b, c, sparse, staged, (C.c_void_p * 2)(a.data_ptr(), b.data_ptr())))
        red = lambda i: lib.flagcxLocalReduce(bufs[i][5], 2, bufs[i][2].data_ptr(), n, f32, opsum, sref)
        pk = lambda i: lib.flagcxLocalPack(bufs[i][4].data_ptr(), bufs[i][3].data_ptr(), 8, chunk, size, sref)
        up = lambda i: lib.flagcxLocalUnpack(bufs[i][3].data_ptr(), bufs[i][4].data_ptr(), 8, chunk, size, sref)
        cp = lambda i: lib.flagcxLocalMemcpy(bufs[i][2].data_ptr(), bufs[i][0].data_ptr(), size, sref)
        ms = lambda i: lib.flagcxLocalMemset(bufs[i][2].data_ptr(), 0, size, sref)
        assert red(0) == 0 and pk(0) == 0 and up(0) == 0 and cp(0) == 0 and ms(0) == 0
        r_med, _ = timed(red, sets=nsets)
        p_med, _ = timed(pk, sets=nsets)
        u_med, _ = timed(up, sets=nsets)
        c_med, _ = timed(cp, sets=nsets)
        m_med, _ = timed(ms, sets=nsets)
        b2b = back_to_back(red, 1000 if size <= (1 << 20) else 50, sets=nsets)
        row = {"bytes": size, "sets": nsets, "reduce2_us": r_med, "reduce2_gbps": 3 * size / r_med / 1e3,
               "pack_us": p_med, "pack_gbps": 2 * size / p_med / 1e3,
               "unpack_us": u_med, "unpack_gbps": 2 * size / u_med / 1e3,
               "memcpy_us": c_med, "memcpy_gbps": 2 * size / c_med / 1e3,
               "memset_us": m_med, "memset_gbps": size / m_med / 1e3, "reduce2_b2b_us": b2b}
        rows.append(row)
        print("%12d %10d | %9.2f %9.1f | %9.2f %9.1f | %9.2f %9.1f | %9.2f %9.1f | %9.2f %9.1f | %8.2f" %
              (size, nsets, r_med, row["reduce2_gbps"], p_med, row["pack_gbps"], u_med, row["unpack_gbps"],
               c_med, row["memcpy_gbps"], m_med, row["memset_gbps"], b2b), flush=True)
        del bufs, a, b, c, sparse, staged
        torch.cuda.empty_cache()
        size *= 2
    if args.json:
        with open(args.json, "w") as f:
            json.dump(rows, f)
    return 0


if __name__ == "__main__":
    sys.exit(main())
