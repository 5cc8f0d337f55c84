"""Rate of the k-input reduce for every element type and operation on one GPU:

    python -m flagcx_amd.perf_dtypes [--k 8 4 2] [--mib 256] [--sets 2]

Buffers are placed by flagcxLocalPlaceBuffers inside one allocation per set; `--sets`
sets are used in turn, so that no launch finds its buffers in the memory-side cache.
Cells are percent of the 8 TB/s HBM peak, (k+1) * bytes / time from HIP events over
back-to-back launches.  The buffers hold random 16-bit patterns below 16000, which are
finite, normal values in every floating-point type.
"""
import argparse
import ctypes as C
import sys

import torch

from flagcx_amd import local as L

MiB = 1 << 20
NAMES = ["int8", "uint8", "int32", "uint32", "int64", "uint64", "fp16", "fp32", "fp64", "bf16"]
SIZES = [1, 1, 4, 4, 8, 8, 2, 4, 8, 2]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--k", type=int, nargs="+", default=[8, 4, 2])
    ap.add_argument("--mib", type=int, default=256, help="MiB per input")
    ap.add_argument("--sets", type=int, default=2)
    ap.add_argument("--iters", type=int, default=16)
    args = ap.parse_args()
    torch.cuda.set_device(0)
    lib = L.lib()
    L.check(lib.flagcxLocalInit())
    ops = [("sum", L.RedOp.Sum), ("prod", L.RedOp.Prod), ("max", L.RedOp.Max), ("min", L.RedOp.Min), ("avg", L.RedOp.Avg)]
    nbytes = args.mib * MiB
    st = L.current_stream()
    sref = C.byref(st)
    for k in args.k:
        sets = []
        for _ in range(args.sets):
            pool_bytes = (k + 1) * (nbytes + 128 * 1024)
            pool = torch.empty(pool_bytes, dtype=torch.uint8, device="cuda")
            pool.view(torch.int16).random_(0, 16000)
            addrs = L.place_buffers(pool.data_ptr(), pool_bytes, nbytes, k + 1)
            sets.append(((C.c_void_p * k)(*addrs[:k]), addrs[k], pool))
        print("k=%d, %d MiB per input, %d buffer set(s) in turn; percent of 8 TB/s" % (k, args.mib, args.sets), flush=True)
        for dt in range(10):
            count = nbytes // SIZES[dt]
            line = "  %-7s" % NAMES[dt]
            for oname, op in ops:
                def go(i):
                    srcs, dst, _ = sets[i % args.sets]
                    L.check(lib.flagcxLocalReduce(srcs, k, dst, count, dt, int(op), sref))
                for i in range(2 * args.sets):
                    go(i)
                torch.cuda.synchronize()
                e0 = torch.cuda.Event(enable_timing=True)
                e1 = torch.cuda.Event(enable_timing=True)
                e0.record()
                for i in range(args.iters):
                    go(i)
                e1.record()
                torch.cuda.synchronize()
                line += "  %s %5.1f" % (oname, (k + 1) * nbytes / (e0.elapsed_time(e1) / args.iters * 1e-3) / 1e9 / 80.0)
            print(line, flush=True)
        del sets
        torch.cuda.empty_cache()
    return 0


if __name__ == "__main__":
    sys.exit(main())
