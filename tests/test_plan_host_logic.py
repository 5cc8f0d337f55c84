"""The plan executor's host logic on the CPU.  flagcx_amd/csrc/host_c2c_local.cpp is plain C++ over eight
C-ABI entry points; here it is compiled with AddressSanitizer and UBSan against a test double of those
entry points that works on host memory (tests/plan_host_harness/device_double.cpp) and replays
  - the DSL-written fixtures under tests/golden/plans, and
  - the seeded random two-cluster plans of tests/test_plan_random_gpu.py,
fused and literally, against the numpy model of flagcxC2cPlanner::execute.  Every buffer is a heap block of
exactly its size, so an access of the executor past an end aborts the run, and the double aborts when
operations it is told to run concurrently are not independent.  The double is test infrastructure: the
library never links it."""
import os
import random
import shutil
import subprocess

import numpy as np
import pytest

from oracle import c2c_plan_model as M
from tests import test_plan_random_gpu as R
from tests.test_plan_fixtures import CL4, CL8, fixture
from tests.test_plan_fused_gpu import special_values
from oracle import cpu_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HARNESS_DIR = os.path.join(ROOT, "tests", "plan_host_harness")
SOURCES = [os.path.join(HARNESS_DIR, "harness.cpp"), os.path.join(HARNESS_DIR, "device_double.cpp"),
           os.path.join(ROOT, "flagcx_amd", "csrc", "host_c2c_local.cpp")]


@pytest.fixture(scope="module")
def harness(tmp_path_factory):
    gxx = shutil.which("g++")
    if not gxx:
        pytest.skip("no g++")
    exe = str(tmp_path_factory.mktemp("plan_harness") / "harness")
    base = [gxx, "-g", "-std=c++17", "-w"]
    r = subprocess.run(base + ["-O0", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined", "-fno-omit-frame-pointer"] +
                       SOURCES + ["-o", exe], capture_output=True, text=True, timeout=600)
    if r.returncode != 0:     # no sanitizer runtime on this machine: the logic is still compared with the model
        r = subprocess.run(base + ["-O1"] + SOURCES + ["-o", exe], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    return exe


def run_cases(harness, tmp_path, cases):
    """cases: dicts with prefix, clusters, n, chunks, commop, redop, algo, fused, dt, root, scratch, hosts.
    Returns per case (status, message, recv arrays, send arrays)."""
    lines = []
    for i, c in enumerate(cases):
        d = tmp_path / ("case%d" % i)
        d.mkdir()
        for r, h in enumerate(c["hosts"]):
            h.tofile(str(d / ("in_%d.bin" % r)))
        lines.append(" ".join(str(x) for x in [c["prefix"], len(c["clusters"])] + list(c["clusters"]) +
                              [c["n"], c["chunks"], c["commop"], c["redop"], c["algo"], int(c["fused"]), c["dt"], c["root"],
                               int(c["scratch"]), d, d] +
                              (["v"] + [x for mat in c["v_args"] for row in mat for x in row] if c.get("v_args") else [])))
    man = tmp_path / "manifest.txt"
    man.write_text("\n".join(lines) + "\n")
    # leak detection needs ptrace rights that a sandboxed runner may lack; it was run once by hand (no leak)
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:abort_on_error=1", UBSAN_OPTIONS="print_stacktrace=1")
    r = subprocess.run([harness, str(man)], capture_output=True, text=True, timeout=900, env=env)
    assert r.returncode == 0, (r.returncode, r.stdout[-500:], r.stderr[-3000:])
    out = []
    for i, c in enumerate(cases):
        d = tmp_path / ("case%d" % i)
        status, _, msg = (d / "status.txt").read_text().strip().partition(" ")
        npdt = c["hosts"][0].dtype
        out.append((int(status), msg, [np.fromfile(str(d / ("out_%d.bin" % r)), dtype=npdt) for r in range(len(c["clusters"]))],
                    [np.fromfile(str(d / ("send_%d.bin" % r)), dtype=npdt) for r in range(len(c["clusters"]))]))
    return out


def model_recv(c):
    nr, n, npdt = len(c["clusters"]), c["n"], c["hosts"][0].dtype
    m = M.Model(c["prefix"], c["clusters"], n, c["commop"], c["redop"], default_chunks=c["chunks"] or None)
    recv = [np.frombuffer(bytes([0x55]) * (n * npdt.itemsize), dtype=npdt).copy() for _ in range(nr)]
    scr = [np.frombuffer(bytes([0x33]) * (n * npdt.itemsize), dtype=npdt).copy() for _ in range(nr)] if c["scratch"] else None
    with np.errstate(over="ignore"):
        m.execute([h.copy() for h in c["hosts"]], recv, scr, root=c["root"], algorithm=c["algo"], v_args=c.get("v_args"))
    return recv


def same_bits(a, b):
    return a.shape == b.shape and a.tobytes() == b.tobytes()


def test_fixtures_replay_like_the_model_on_the_cpu(harness, tmp_path):
    cases = []
    for name, clusters, commop, chunks, scratch, root in (("allreduce8", CL8, 6, 8, False, -1), ("reducescatter8", CL8, 8, 8, True, -1),
                                                           ("reduce8", CL8, 5, 8, False, 6), ("gather4", CL4, 3, 4, True, 3),
                                                           ("uneven4", CL4, 6, 4, False, -1), ("allgather4", CL4, 7, 4, False, -1)):
        for algo in (0, 1, 2):
            for fused in (True, False):
                n = chunks * 613
                rng = np.random.default_rng(len(cases))
                hosts = [rng.integers(-2**27, 2**27, n, dtype=np.int32) for _ in clusters]
                cases.append(dict(prefix=fixture(name), clusters=clusters, n=n, chunks=chunks, commop=commop, redop=0, algo=algo,
                                  fused=fused, dt=int(O.INT32), root=root, scratch=scratch, hosts=hosts, name=name))
    for c, (status, msg, recv, send) in zip(cases, run_cases(harness, tmp_path, cases)):
        what = (c["name"], c["algo"], c["fused"])
        assert status == 0, (what, msg)
        want = model_recv(c)
        for r in range(len(c["clusters"])):
            assert same_bits(recv[r], want[r]), (what, r)
            assert same_bits(send[r], c["hosts"][r]), (what, r)


# more blocks and other seeds for a longer run: FLAGCX_PLAN_FUZZ_BLOCKS=40 FLAGCX_PLAN_FUZZ_SEED=90000 pytest tests/test_plan_host_logic.py
FUZZ_BLOCKS = int(os.environ.get("FLAGCX_PLAN_FUZZ_BLOCKS", "4"))
FUZZ_SEED = int(os.environ.get("FLAGCX_PLAN_FUZZ_SEED", "31000"))


@pytest.mark.parametrize("block", range(FUZZ_BLOCKS))
def test_random_plans_on_the_cpu_fused_literal_and_model_agree(harness, tmp_path, block):
    """100 seeded random plans per block (other seeds than the GPU test's): int32 fused == literal == model,
    fp32 full of signed zeros, NaNs and infinities fused == literal (NaNs by bits too: the double folds both
    replays with the same host arithmetic)."""
    rnd = random.Random(FUZZ_SEED + block)
    cases = []
    for k in range(100):
        sizes = rnd.choice([(2, 2), (4, 4), (1, 3), (3, 1), (2, 6), (5, 3), (1, 1), (3, 4)])   # clusters of unequal sizes too
        nr = sum(sizes)
        clusters = [0] * sizes[0] + [1] * sizes[1]
        commop = rnd.choice([6, 8])
        redop = rnd.choice([0, 0, 0, 2, 3])
        algo = rnd.choice([0, 1, 2])
        n = R.NCH * nr * rnd.choice([1, 3, 40])
        prefix = str(tmp_path / ("p%d" % k))
        R.make_plan(prefix, rnd, nr, commop, sizes)
        rng = np.random.default_rng(1000 * block + k)
        ints = [rng.integers(-2**20, 2**20, n).astype(np.int32) for _ in range(nr)]
        flts = [special_values(O.FP32, n, 7000 * block + 10 * k + r) for r in range(nr)]
        for hosts, dt in ((ints, int(O.INT32)), (flts, int(O.FP32))):
            for fused in (True, False):
                cases.append(dict(prefix=prefix, clusters=clusters, n=n, chunks=0, commop=commop, redop=redop, algo=algo,
                                  fused=fused, dt=dt, root=-1, scratch=True, hosts=hosts, k=k))
    res = run_cases(harness, tmp_path, cases)
    for i in range(0, len(cases), 4):
        c = cases[i]
        what = (block, c["k"], len(c["clusters"]), c["commop"], c["redop"], c["algo"], c["n"])
        (s0, m0, fi, si), (s1, m1, li, _), (s2, m2, ff, _), (s3, m3, lf, _) = res[i:i + 4]
        assert (s0, s1, s2, s3) == (0, 0, 0, 0), (what, m0, m1, m2, m3)
        want = model_recv(c)
        for r in range(len(c["clusters"])):
            assert same_bits(fi[r], li[r]), ("int32 fused != literal", what, r)
            assert same_bits(li[r], want[r]), ("int32 literal != model", what, r)
            assert same_bits(si[r], c["hosts"][r]), ("send buffer changed", what, r)
            assert same_bits(ff[r], lf[r]), ("fp32 fused != literal", what, r)


def test_hand_written_plans_on_the_cpu(harness, tmp_path):
    """The hand-written plans of the GPU tests through the same harness: the 2 x 2 all-reduces (local fold and
    copy, refresh of scratch, the reference's own operations only), every one-cluster block mover for 1..8 ranks
    and every root, the broadcast from a root in the second cluster, and the Send / Recv homo functions of all
    three types; each fused and literally, against the model."""
    from tests import plan_xml as PX
    from tests.test_plan_fixtures import broadcast_two_clusters, send_recv_plan
    cases = []

    def add(name, prefix, clusters, n, commop, root=-1, scratch=False, algo=2, chunks=0):
        rng = np.random.default_rng(len(cases))
        hosts = [rng.integers(-2**27, 2**27, n, dtype=np.int32) for _ in clusters]
        for fused in (True, False):
            cases.append(dict(prefix=prefix, clusters=clusters, n=n, chunks=chunks, commop=commop, redop=0, algo=algo, fused=fused,
                              dt=int(O.INT32), root=root, scratch=scratch, hosts=hosts, name=name))

    for maker, scratch in ((PX.allreduce_2x2_locred, False), (PX.allreduce_2x2_refresh_scratch, True),
                           (PX.allreduce_2x2_reference_ops_only, False)):
        prefix = str(tmp_path / maker.__name__)
        maker(prefix)
        for algo in (0, 1, 2):
            add(maker.__name__, prefix, CL4, 4 * 501, 8 if scratch else 6, scratch=scratch, algo=algo)
    for commop in (PX.ALLGATHER, PX.GATHER, PX.ALLTOALL, PX.SCATTER, PX.BROADCAST, PX.REDUCE, PX.REDUCESCATTER):
        for nranks in (1, 2, 3, 5, 8):
            for root in {0, nranks - 1, nranks // 2}:
                prefix = str(tmp_path / ("one_%d_%d_%d" % (commop, nranks, root)))
                PX.one_cluster_collective(prefix, commop, nranks, root)
                add("one_cluster_%d" % commop, prefix, [0] * nranks, nranks * 77, commop, root=root)
    for root in (4, 5, 7):
        prefix = str(tmp_path / ("bc%d" % root))
        broadcast_two_clusters(prefix, root)
        add("broadcast_root_%d" % root, prefix, CL8, 4 * 333, 2, root=root)
    prefix = str(tmp_path / "sr")
    send_recv_plan(prefix)
    add("send_recv", prefix, CL4, 6 * 211, 3, root=1, scratch=True)
    # the all-to-all-v fixture: ragged counts and displacements handed over beside the plan
    from tests.test_plan_fixtures import alltoallv_case
    n, v, hosts, want = alltoallv_case(37, np.int32, 9)
    for fused in (True, False):
        cases.append(dict(prefix=fixture("alltoallv4"), clusters=CL4, n=n, chunks=8, commop=10, redop=0, algo=2, fused=fused,
                          dt=int(O.INT32), root=-1, scratch=False, hosts=hosts, name="alltoallv4", v_args=v, closed=want))

    for c, (status, msg, recv, send) in zip(cases, run_cases(harness, tmp_path, cases)):
        what = (c["name"], len(c["clusters"]), c["root"], c["algo"], c["fused"])
        assert status == 0, (what, msg)
        want = model_recv(c)
        for r in range(len(c["clusters"])):
            assert same_bits(recv[r], want[r]), (what, r)
            assert same_bits(send[r], c["hosts"][r]), (what, r)
            if "closed" in c:
                assert same_bits(recv[r], c["closed"][r]), (what, r, "closed form")
