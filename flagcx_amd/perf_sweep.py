"""Message-size sweep of the local primitives on one GPU, in the manner of the
reference's perf tests (5 warm-up + 20 timed iterations per size,
test/perf/tools.cc:81-86):

    python -m flagcx_amd.perf_sweep [--min 1024] [--max 1073741824] [--json out.json]

Per size S (bytes per buffer):
  reduce2   2-input fp32 sum of S bytes per buffer          algorithmic bytes 3*S
  pack      8 chunks of S/8 at stride S gathered contiguous  2*S
  unpack    the inverse scatter                              2*S
  memcpy    contiguous device-to-device copy                 2*S
  memset    byte fill (the zero-fill of a refresh)           S
Times are HIP-event medians per launch; GB/s uses the algorithmic bytes.
Small sizes are cache resident; from a few hundred MiB on the data streams from HBM.
"""
import argparse
import ctypes as C
import json
import sys

import torch

from flagcx_amd import local as L


def timed(fn, warmup=5, iters=20):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    ts = []
    for _ in range(iters):
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        fn()
        e1.record()
        e1.synchronize()
        ts.append(e0.elapsed_time(e1) * 1e3)
    ts.sort()
    return ts[len(ts) // 2], ts[0]


def back_to_back(fn, n):
    for _ in range(20):
        fn()
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(n):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / n


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--min", type=int, default=1 << 10)
    ap.add_argument("--max", type=int, default=1 << 30)
    ap.add_argument("--json", default=None)
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
          ("bytes", "", "reduce2us", "GB/s", "pack us", "GB/s", "unpack us", "GB/s", "memcpy us", "GB/s",
           "memset us", "GB/s", "b2b us"))
    while size <= args.max:
        n = size // 4
        a = torch.rand(n, device="cuda", generator=g) * 2 - 1
        b = torch.rand(n, device="cuda", generator=g) * 2 - 1
        c = torch.empty(n, device="cuda")
        ptrs = (C.c_void_p * 2)(a.data_ptr(), b.data_ptr())
        red = lambda: lib.flagcxLocalReduce(ptrs, 2, c.data_ptr(), n, f32, opsum, sref)
        # sparse source of 8*size bytes holding 8 chunks of size/8 at stride `size`
        chunk = size // 8
        sparse = torch.rand(8 * n, device="cuda", generator=g)
        staged = torch.empty(n, device="cuda")
        pk = lambda: lib.flagcxLocalPack(staged.data_ptr(), sparse.data_ptr(), 8, chunk, size, sref)
        up = lambda: lib.flagcxLocalUnpack(sparse.data_ptr(), staged.data_ptr(), 8, chunk, size, sref)
        cp = lambda: lib.flagcxLocalMemcpy(c.data_ptr(), a.data_ptr(), size, sref)
        ms = lambda: lib.flagcxLocalMemset(c.data_ptr(), 0, size, sref)
        assert red() == 0 and pk() == 0 and up() == 0 and cp() == 0 and ms() == 0
        r_med, _ = timed(red)
        p_med, _ = timed(pk)
        u_med, _ = timed(up)
        c_med, _ = timed(cp)
        m_med, _ = timed(ms)
        b2b = back_to_back(red, 1000 if size <= (1 << 20) else 50)
        row = {"bytes": size, "reduce2_us": r_med, "reduce2_gbps": 3 * size / r_med / 1e3,
               "pack_us": p_med, "pack_gbps": 2 * size / p_med / 1e3,
               "unpack_us": u_med, "unpack_gbps": 2 * size / u_med / 1e3,
               "memcpy_us": c_med, "memcpy_gbps": 2 * size / c_med / 1e3,
               "memset_us": m_med, "memset_gbps": size / m_med / 1e3, "reduce2_b2b_us": b2b}
        rows.append(row)
        print("%12d %10s | %9.2f %9.1f | %9.2f %9.1f | %9.2f %9.1f | %9.2f %9.1f | %9.2f %9.1f | %8.2f" %
              (size, "", r_med, row["reduce2_gbps"], p_med, row["pack_gbps"], u_med, row["unpack_gbps"],
               c_med, row["memcpy_gbps"], m_med, row["memset_gbps"], b2b), flush=True)
        del a, b, c, sparse, staged
        size *= 2
    if args.json:
        with open(args.json, "w") as f:
            json.dump(rows, f)
    return 0


if __name__ == "__main__":
    sys.exit(main())
