"""How the k-input reduce reacts to the relative placement of its inputs, to the cap
on resident wavefronts per CU (flagcxLocalTune) and to the number of inputs a
wavefront keeps in flight (flagcxLocalTuneLoads):

    python -m flagcx_amd.perf_stride [--k 8] [--mib 128] [--dtype bf16] [--loads N] [--sets S]

The inputs are slices of one allocation, `stride` bytes apart (128 MiB .. 1 GiB plus
small offsets), so their addresses alias differently in the HBM channel hash.  For
each stride the table gives percent of the 8 TB/s peak for several caps and for the
library's own per-launch choice ("auto"); the last line gives the worst and best
stride per column.  --loads fixes the inputs in flight per wavefront for the cap
columns (default -1: the library's choice; "auto" is always the library's choice
of both).  --sets S uses S such allocations in turn, so that a launch finds
nothing of its buffers in the memory-side cache (with one set part of the output
of the previous launch is still there and the rates are two to four percent higher).
"""
import argparse
import sys

import torch

from flagcx_amd import local as L

MiB = 1 << 20
STRIDES = [128 * MiB, 128 * MiB + 4096, 128 * MiB + 65536, 129 * MiB + 4096, 256 * MiB, 512 * MiB,
           1024 * MiB, 1024 * MiB + 4096, 1024 * MiB + 65536, 1025 * MiB, 1026 * MiB + 8192, 1057 * MiB + 12288]
CAPS = [8, 10, 12, 14, 16, 18, 21, 25, 0, -1]   # caps that whole LDS granules can express; -1 = the library's choice


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--k", type=int, default=8)
    ap.add_argument("--mib", type=int, default=128, help="MiB per input")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "f32", "i32"])
    ap.add_argument("--loads", type=int, default=-1, help="inputs in flight per wavefront for the cap columns (-1: the library's choice)")
    ap.add_argument("--sets", type=int, default=1, help="buffer sets used in turn")
    args = ap.parse_args()
    k = args.k
    tdt = {"bf16": torch.bfloat16, "f32": torch.float32, "i32": torch.int32}[args.dtype]
    esz = torch.empty(0, dtype=tdt).element_size()
    nbytes = args.mib * MiB
    n = nbytes // esz
    torch.cuda.set_device(0)
    L.check(L.lib().flagcxLocalInit())
    import ctypes as C
    cap0 = C.c_int(0)
    L.check(L.lib().flagcxLocalGetTune(k, C.byref(cap0)))
    default_cap = cap0.value
    bigs, outs = [], []
    for _ in range(args.sets):
        big = torch.empty((max(STRIDES) * (k - 1) + nbytes) // esz + 16, dtype=tdt, device="cuda")
        big.view(torch.int16 if esz == 2 else torch.int32).random_(0, 1000)
        bigs.append(big)
        outs.append(torch.empty(n, dtype=tdt, device="cuda"))
    print("k=%d %s, %d MiB per input, %d buffer set(s), inputs in flight per wavefront in the cap columns: %s; "
          "percent of 8 TB/s, (k+1)*bytes/time" % (k, args.dtype, args.mib, args.sets, "library's choice" if args.loads < 0 else args.loads))
    print("%14s " % "stride" + " ".join("%7s" % ("cap %d" % c if c > 0 else "no cap" if c == 0 else "auto") for c in CAPS))
    worst = {c: 100.0 for c in CAPS}
    best = {c: 0.0 for c in CAPS}
    for st in STRIDES:
        srcs = [[big[j * st // esz: j * st // esz + n] for j in range(k)] for big in bigs]
        row = []
        iters = 20 * args.sets
        for cap in CAPS:
            L.check(L.lib().flagcxLocalTune(k, cap))
            if k >= 2:
                L.check(L.lib().flagcxLocalTuneLoads(k, args.loads if cap >= 0 else -1))
            for i in range(3 * args.sets):
                L.reduce(srcs[i % args.sets], outs[i % args.sets], L.RedOp.Sum)
            torch.cuda.synchronize()
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            e0.record()
            for i in range(iters):
                L.reduce(srcs[i % args.sets], outs[i % args.sets], L.RedOp.Sum)
            e1.record()
            torch.cuda.synchronize()
            pct = (k + 1) * nbytes / (e0.elapsed_time(e1) / iters * 1e-3) / 1e9 / 80.0
            worst[cap] = min(worst[cap], pct)
            best[cap] = max(best[cap], pct)
            row.append("%7.1f" % pct)
        print("%14d " % st + " ".join(row), flush=True)
    L.check(L.lib().flagcxLocalTune(k, default_cap))
    if k >= 2:
        L.check(L.lib().flagcxLocalTuneLoads(k, -1))
    print("setting found for k=%d: %d (-1 = chosen per launch)" % (k, default_cap))
    print("%14s " % "worst..best" + " ".join("%3.0f..%-3.0f" % (worst[c], best[c]) for c in CAPS))
    return 0


if __name__ == "__main__":
    sys.exit(main())
