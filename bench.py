#!/usr/bin/env python3
"""Benchmark of the local N-way reduce on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One "step" is one pass of the hot path over one batch: a single 8-input bf16 sum
(fp32 accumulation) over 256 MiB per input buffer, i.e. one simulated rank's
reducescatter stage of an 8-rank C2C allreduce.  Inputs are resident in HBM before
the timed region.  Prints ONE JSON line on stdout:

  value      algorithmic bytes / wall time of the K timed steps, GB/s
             ((k+1) * n * sizeof(bf16) per step)
  roofline   the same bytes over the kernel's average launch duration measured
             with HIP events on the launch stream, against 8 TB/s of HBM3E
  cpu_baseline  the CPU oracle (a port of the reference's host reduce) timed on
             this machine's cores on a bounded sample of the same workload
  latency_us_4KiB  per-launch time of a 2-input fp32 sum over 4 KiB buffers

Everything on the GPU goes through the C ABI of libflagcx_amd.so; the oracle is
used only for the cpu_baseline leg and a spot check of the result.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
K = 8
N_ELEM = 128 * 1024 * 1024          # 256 MiB of bf16 per input
ALGO_BYTES = (K + 1) * N_ELEM * 2   # k reads + 1 write

# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
# (profiles/reduce8_bf16_sum_256MiB_pmc.txt), scaled by a copy kernel of known size.
MEASURED_TRAFFIC_BYTES = 2415851937


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def cpu_baseline(inputs_bits, sample_elems):
    """Times the oracle on a leading sample of the same inputs (host copies)."""
    from oracle import cpu_oracle as O
    host = [np.ascontiguousarray(t[:sample_elems].cpu().numpy().view(np.uint16)) for t in inputs_bits]
    dst = np.empty(sample_elems, dtype=np.uint16)
    nbytes = (K + 1) * sample_elems * 2
    t1 = O.time_reduce(host, dst, O.BF16, O.SUM, nthreads=1, warmup=1, iters=3)
    ncores = os.cpu_count() or 1
    nth = min(K, ncores)
    tk = O.time_reduce(host, dst, O.BF16, O.SUM, nthreads=nth, warmup=1, iters=3)
    return {
        "value": round(nbytes / t1 / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
        "sample": "first %d of %d elements of the same 8 bf16 inputs (%.0f MiB per input), "
                  "median of 3 passes after 1 warm-up; restatement extension: the reference's "
                  "host path rejects bf16" % (sample_elems, N_ELEM, sample_elems * 2 / 2**20),
        "threads_k": {"value": round(nbytes / tk / 1e9, 3), "threads": nth},
        "host_cores": ncores,
    }, host, dst


def cpu_other_configs():
    """The CPU side of two more benchmark configurations: C1 (2 x fp32 sum, 64 MiB per
    buffer, full size) and C4 (4 x int32 max, a 16 Mi-element sample of 128 Mi)."""
    from oracle import cpu_oracle as O
    rng = np.random.default_rng(0)
    out = []
    n1 = 16 * 1024 * 1024
    fa = rng.uniform(-1, 1, n1).astype(np.float32)
    fb = rng.uniform(-1, 1, n1).astype(np.float32)
    fd = np.empty_like(fa)
    for nth in (1, 2):
        t = O.time_reduce([fa, fb], fd, O.FP32, O.SUM, nthreads=nth, warmup=1, iters=3)
        out.append({"config": "C1 2x fp32 sum, 64 MiB per buffer, full size", "threads": nth,
                    "value": round(3 * fa.nbytes / t / 1e9, 3), "unit": "GB/s"})
    n4 = 16 * 1024 * 1024
    ins = [rng.integers(-2**31, 2**31 - 1, n4, dtype=np.int64).astype(np.int32) for _ in range(4)]
    dst = np.empty(n4, dtype=np.int32)
    for nth in (1, 4):
        t = O.time_reduce(ins, dst, O.INT32, O.MAX, nthreads=nth, warmup=1, iters=3)
        out.append({"config": "C4 4x int32 max, 16 Mi-element sample of 128 Mi", "threads": nth,
                    "value": round(5 * n4 * 4 / t / 1e9, 3), "unit": "GB/s"})
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--cpu-sample", type=int, default=32 * 1024 * 1024,
                    help="elements per input the CPU baseline reduces")
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--cpu-configs", action="store_true",
                    help="cpu_baseline also times the oracle on the C1 and C4 configurations")
    ap.add_argument("--allocator-layout", action="store_true",
                    help="inputs and output as separate torch allocations instead of placed in one")
    ap.add_argument("--rotate-sets", type=int, default=3, metavar="S",
                    help="also time the same launches over S sets of buffers used in turn (0: skip), "
                         "reported as rotating_buffers")
    ap.add_argument("--calibrate-copy", type=int, default=0, metavar="N",
                    help="also run N flagcxLocalMemcpy launches of 256 MiB (a copy of known size "
                         "to scale rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        log("bench.py: this build runs on ONE GPU (the k ranks are k HBM buffers on it); "
            "--gpus %d is not supported" % args.gpus)
        sys.exit(2)

    import torch
    from flagcx_amd import local as L
    if not torch.cuda.is_available():
        log("bench.py: no GPU visible")
        sys.exit(1)
    torch.cuda.set_device(0)
    L.check(L.lib().flagcxLocalInit())

    # The 8 input buffers and the output live in one allocation, at the addresses
    # flagcxLocalPlaceBuffers gives: equal offsets into them fall into different HBM
    # channel groups, which is how a caller that owns the ranks' staging buffers would
    # lay them out.  --allocator-layout takes nine separate torch allocations instead
    # (258 MiB apart on this allocator: all in one channel group).
    nbytes = N_ELEM * 2
    if args.allocator_layout:
        bufs = [torch.empty(N_ELEM, dtype=torch.bfloat16, device="cuda") for _ in range(K + 1)]
        layout = "nine separate torch allocations"
    else:
        pool_bytes = (K + 1) * (nbytes + 128 * 1024)
        pool = torch.empty(pool_bytes, dtype=torch.uint8, device="cuda")
        addrs = L.place_buffers(pool.data_ptr(), pool_bytes, nbytes, K + 1)
        bufs = [pool[a - pool.data_ptr(): a - pool.data_ptr() + nbytes].view(torch.bfloat16) for a in addrs]
        layout = "one allocation, buffers placed by flagcxLocalPlaceBuffers"
    # seeded synthetic inputs: N(0,1) per input from seeds 0..7, rounded to bf16
    inputs = bufs[:K]
    out = bufs[K]
    for seed in range(K):
        g = torch.Generator(device="cuda").manual_seed(seed)
        inputs[seed].copy_(torch.randn(N_ELEM, generator=g, device="cuda", dtype=torch.float32))
    torch.cuda.synchronize()

    def step():
        L.reduce(inputs, out, L.RedOp.Sum)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    ev0 = torch.cuda.Event(enable_timing=True)
    ev1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record()                      # same stream the launches go to
    for _ in range(args.steps):
        step()
    ev1.record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    wall_ms = (t1 - t0) * 1e3 / args.steps
    kern_ms = ev0.elapsed_time(ev1) / args.steps
    value = ALGO_BYTES / (wall_ms * 1e-3) / 1e9
    achieved = ALGO_BYTES / (kern_ms * 1e-3) / 1e9

    # The timed loop above reduces the same nine buffers every step, as the metric is
    # defined; part of the 256 MiB output of one step is then still in the memory-side
    # cache when the next step writes it again.  For comparison: S sets of buffers
    # used in turn, so that no launch finds anything of its own there.
    rotating = None
    if args.rotate_sets >= 2:
        sets, keep = [bufs], []
        for _ in range(args.rotate_sets - 1):
            if args.allocator_layout:
                more = [torch.empty(N_ELEM, dtype=torch.bfloat16, device="cuda") for _ in range(K + 1)]
            else:
                p2 = torch.empty(pool_bytes, dtype=torch.uint8, device="cuda")
                keep.append(p2)
                more = [p2[a - p2.data_ptr(): a - p2.data_ptr() + nbytes].view(torch.bfloat16)
                        for a in L.place_buffers(p2.data_ptr(), pool_bytes, nbytes, K + 1)]
            for j in range(K):
                more[j].copy_(inputs[j])
            sets.append(more)
        nset = len(sets)
        for i in range(2 * nset):
            L.reduce(sets[i % nset][:K], sets[i % nset][K], L.RedOp.Sum)
        torch.cuda.synchronize()
        r0 = torch.cuda.Event(enable_timing=True)
        r1 = torch.cuda.Event(enable_timing=True)
        r0.record()
        for i in range(args.steps):
            L.reduce(sets[i % nset][:K], sets[i % nset][K], L.RedOp.Sum)
        r1.record()
        torch.cuda.synchronize()
        rot_ms = r0.elapsed_time(r1) / args.steps
        same_out = all(torch.equal(sets[i][K].view(torch.int16), out.view(torch.int16)) for i in range(1, nset))
        rotating = {"sets": nset, "value": round(ALGO_BYTES / (rot_ms * 1e-3) / 1e9, 1), "unit": "GB/s",
                    "frac": round(ALGO_BYTES / (rot_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                    "avg_launch_ms": round(rot_ms, 5), "outputs_equal_first_set": bool(same_out)}
        del sets, keep
        torch.cuda.empty_cache()

    for _ in range(args.calibrate_copy):
        L.memcpy(out.data_ptr(), inputs[0].data_ptr(), N_ELEM * 2)
    torch.cuda.synchronize()

    # small-message latency: 2-input fp32 sum over 4 KiB buffers, arguments
    # marshalled once so the loop is one C call per launch
    import ctypes as C
    a = torch.rand(1024, device="cuda")
    b = torch.rand(1024, device="cuda")
    c = torch.empty(1024, device="cuda")
    ptrs = (C.c_void_p * 2)(a.data_ptr(), b.data_ptr())
    st = L.current_stream()
    sref = C.byref(st)
    fn = L.lib().flagcxLocalReduce
    cptr, f32, opsum = c.data_ptr(), int(L.DataType.Float32), int(L.RedOp.Sum)

    def small():
        return fn(ptrs, 2, cptr, 1024, f32, opsum, sref)

    for _ in range(200):
        small()
    torch.cuda.synchronize()
    n_lat = 2000
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(n_lat):
        small()
    e1.record()
    torch.cuda.synchronize()
    lat_stream_us = e0.elapsed_time(e1) * 1e3 / n_lat
    singles = []
    for _ in range(200):
        s0 = time.perf_counter()
        small()
        torch.cuda.synchronize()
        singles.append((time.perf_counter() - s0) * 1e6)
    singles.sort()

    # the same figure as a C caller sees it (no interpreter in the launch path)
    c_lat = None
    perf_bin = os.path.join(ROOT, "flagcx_amd", "lib", "local_perf")
    if os.path.exists(perf_bin):
        import subprocess
        try:
            r = subprocess.run([perf_bin, "-b", "4096", "-e", "4096", "-n", "40"], capture_output=True, text=True,
                               timeout=120)
            row = [l.split() for l in r.stdout.splitlines() if l.strip().startswith("4096")]
            if r.returncode == 0 and row:
                c_lat = {"back_to_back_per_launch": float(row[0][2]), "single_launch_to_sync_median": float(row[0][4])}
        except Exception as e:  # the figure is auxiliary: report why it is missing
            log("bench.py: C latency driver failed: %r" % (e,))

    result = {
        "metric": "hbm_gbps_reduce8_bf16_sum_256MiB", "value": round(value, 1), "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(wall_ms, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "8-input bf16 sum reduce, fp32 accumulation, 256 MiB per input buffer "
                               "(128Mi elements), N(0,1) from seeds 0..7",
                   "nranks": K, "elements": N_ELEM, "bytes_per_step": ALGO_BYTES, "accumulate": "fp32",
                   "buffers": layout},
        "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBPS, 2),
        "rotating_buffers": rotating,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": MEASURED_TRAFFIC_BYTES,
                     "kernel": "reduceWaveKernel<bf16,sum,K=8,U=1>", "avg_launch_ms": round(kern_ms, 5),
                     "algorithmic_bytes_per_launch": ALGO_BYTES},
        "latency_us_4KiB": {"workload": "2-input fp32 sum, 4 KiB per buffer",
                            "c_caller": c_lat,
                            "python_ctypes_caller": {
                                "back_to_back_per_launch": round(lat_stream_us, 3),
                                "single_launch_to_sync_median": round(singles[len(singles) // 2], 3)}},
    }

    if not args.no_cpu:
        bits = [t.view(torch.int16) for t in inputs]
        sample = min(args.cpu_sample, N_ELEM)
        base, host, dst = cpu_baseline(bits, sample)
        result["cpu_baseline"] = base
        if args.cpu_configs:
            base["other_configs"] = cpu_other_configs()
        # spot check of the GPU result against the oracle on the sample
        got = out[:sample].view(torch.int16).cpu().numpy().view(np.uint16)
        result["spot_check_vs_oracle"] = "bit-exact" if got.tobytes() == dst.tobytes() else "MISMATCH"
        if result["spot_check_vs_oracle"] != "bit-exact":
            log("bench.py: GPU result differs from the oracle on the sample")
            print(json.dumps(result))
            sys.exit(1)

    print(json.dumps(result))


if __name__ == "__main__":
    main()
