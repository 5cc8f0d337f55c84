"""Builds flagcx_amd/lib/libflagcx_amd.so for gfx950 with hipcc.

    python -m flagcx_amd.build

The ten element types of the reduce kernels are separate translation units
(reduce_kernels.hip compiled with -DFLAGCX_DT=<enum>) so they build in parallel.
hipcc cross-compiles; no GPU is needed.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIBDIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIBDIR, "libflagcx_amd.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["-O3", "--offload-arch=gfx950", "-std=c++17", "-fPIC", "-ffp-contract=off",
         "-fno-fast-math", "-Wall", "-fvisibility=hidden",
         # keep the compiler from forming packed fp32 VALU ops
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         # and from fusing the last fp32 operation of a fold into the conversion to fp16 (v_fma_mix*):
         # that rounds the exact result once, the fold is defined as fp32 results rounded to fp16
         "-Xclang", "-target-feature", "-Xclang", "-fma-mix-insts"]


def _run(cmd):
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("command failed: %s\n%s\n%s" % (" ".join(cmd), r.stdout, r.stderr))
    return r


def _no_spills(src, defs, remarks):
    """The kernels are sized to run out of registers alone: a kernel that the compiler gave a scratch
    segment (spilled registers, a stack) streams at a fraction of its rate, so the build stops there."""
    name = None
    for line in remarks.splitlines():
        if "remark: Function Name:" in line:
            name = line.split("Function Name:")[1].split("[")[0].strip()
        elif "ScratchSize [bytes/lane]:" in line:
            n = int(line.split("ScratchSize [bytes/lane]:")[1].split("[")[0])
            if n:
                raise RuntimeError("%s %s: kernel %s uses %d bytes of scratch per lane" % (src, " ".join(defs), name, n))


def build(verbose=False, jobs=None):
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(LIBDIR, exist_ok=True)
    units = []
    for dt in range(10):
        units.append((os.path.join(CSRC, "reduce_kernels.hip"), os.path.join(OBJ, "reduce_dt%d.o" % dt),
                      ["-DFLAGCX_DT=%d" % dt]))
    units.append((os.path.join(CSRC, "copy_kernels.hip"), os.path.join(OBJ, "copy_kernels.o"), []))
    units.append((os.path.join(CSRC, "async_kernels.hip"), os.path.join(OBJ, "async_kernels.o"), []))
    units.append((os.path.join(CSRC, "fifo_kernels.hip"), os.path.join(OBJ, "fifo_kernels.o"), []))
    units.append((os.path.join(CSRC, "static_staging.hip"), os.path.join(OBJ, "static_staging.o"), []))
    units.append((os.path.join(CSRC, "c_api.cpp"), os.path.join(OBJ, "c_api.o"), ["-x", "hip"]))
    extra = [os.path.join(CSRC, f) for f in sorted(os.listdir(CSRC)) if f.startswith("host_") and f.endswith(".cpp")]
    for f in extra:
        units.append((f, os.path.join(OBJ, os.path.basename(f)[:-4] + ".o"), ["-x", "hip"]))

    def one(u):
        src, obj, defs = u
        pre, post = [], []
        if "-x" in defs:  # language flag must precede the file
            pre = defs
        else:
            post = defs
        r = _run([HIPCC] + FLAGS + post + ["-Rpass-analysis=kernel-resource-usage", "-c"] + pre + [src, "-o", obj])
        _no_spills(src, post, r.stderr)
        return obj

    jobs = jobs or min(8, os.cpu_count() or 4)
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(one, units))
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs)
    # C++ programs that link the C ABI: timing driver and the collective test
    # (host-only C++; they reach the GPU through the library)
    for prog in ("local_perf", "local_coll_test", "fifo_perf"):
        src = os.path.join(HERE, "perf", prog + ".cpp")
        _run([HIPCC, "-O2", "-std=c++17", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
              "-x", "hip", "--offload-arch=gfx950", src, "-o",
              os.path.join(LIBDIR, prog), "-L" + LIBDIR, "-lflagcx_amd", "-Wl,-rpath,$ORIGIN"])
    if verbose:
        print("built", LIB, os.path.getsize(LIB), "bytes")
    return LIB


if __name__ == "__main__":
    build(verbose=True)
    sys.exit(0)
