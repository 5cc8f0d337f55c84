"""C2C plan replay: XML import / export round trip (CPU) and execution on the GPU
of hand-authored plans in the reference's plan format.  The reference tree holds no
exported plan file, so these plans are written here (tests/plan_xml.py); expected
results are the closed form of an all-reduce."""
import filecmp
import os

import numpy as np
import pytest

from flagcx_amd import local
from oracle import cpu_oracle as O
from tests import plan_xml as PX
from tests.util import dev_empty, from_dev, same, to_dev

CLUSTERS = [0, 0, 1, 1]


@pytest.mark.parametrize("maker", [PX.allreduce_2x2_locred, PX.allreduce_2x2_refresh_scratch,
                                   PX.allreduce_2x2_reference_ops_only], ids=lambda f: f.__name__)
def test_plan_xml_round_trip(tmp_path, maker):
    a = str(tmp_path / "a")
    b = str(tmp_path / "b")
    maker(a)
    plan = local.Plan(CLUSTERS, 4000, 6, local.RedOp.Sum)
    plan.import_xml(a)
    plan.export_xml(b)
    for r in range(4):
        assert filecmp.cmp("%s_%d.xml" % (a, r), "%s_%d.xml" % (b, r), shallow=False), r
    # a second import of the exported files gives the same export again
    plan2 = local.Plan(CLUSTERS, 4000, 6, local.RedOp.Sum)
    plan2.import_xml(b)
    c = str(tmp_path / "c")
    plan2.export_xml(c)
    for r in range(4):
        assert filecmp.cmp("%s_%d.xml" % (b, r), "%s_%d.xml" % (c, r), shallow=False)


def test_plan_import_errors(tmp_path):
    plan = local.Plan(CLUSTERS, 4000, 6, local.RedOp.Sum)
    with pytest.raises(local.FlagcxError) as e:
        plan.import_xml(str(tmp_path / "missing"))
    assert e.value.code == int(local.Result.InternalError)      # like importXml (c2c_algo.cc:979-980)
    PX.allreduce_2x2_locred(str(tmp_path / "p"))
    bad = local.Plan(CLUSTERS, 4001, 6, local.RedOp.Sum)        # 4 chunks do not divide 4001
    with pytest.raises(local.FlagcxError):
        bad.import_xml(str(tmp_path / "p"))
    with open(str(tmp_path / "q_0.xml"), "w") as f:
        f.write("<NotAPlan></NotAPlan>\n")
    with pytest.raises(local.FlagcxError):
        local.Plan([0], 4, 6, local.RedOp.Sum).import_xml(str(tmp_path / "q"))
    with pytest.raises(local.FlagcxError):                      # execute before import
        local.Plan([0], 4, 6, local.RedOp.Sum).execute([1], [1], None, 7, stream=None)
    prod = local.Plan(CLUSTERS, 4000, 6, local.RedOp.Prod)      # c2c_algo.cc:2047-2053
    prod.import_xml(str(tmp_path / "p"))
    with pytest.raises(local.FlagcxError) as e:
        prod.execute([1] * 4, [1] * 4, None, 7, stream=None)
    assert e.value.code == int(local.Result.NotSupported)


@pytest.mark.gpu
@pytest.mark.parametrize("maker,scratch", [(PX.allreduce_2x2_locred, False),
                                           (PX.allreduce_2x2_refresh_scratch, True),
                                           (PX.allreduce_2x2_reference_ops_only, False)],
                         ids=lambda v: getattr(v, "__name__", str(v)))
@pytest.mark.parametrize("dt", [O.FP32, O.INT32, O.BF16])
def test_plan_execute_allreduce_2x2(tmp_path, maker, scratch, dt):
    import torch
    prefix = str(tmp_path / "plan")
    maker(prefix)
    n = 4 * 25000
    # hetero functions stage in scratch only for the collectives that own one in the reference
    # (c2c_algo.cc:2121-2131): the plan that exchanges its halves in scratch runs as a ReduceScatter
    plan = local.Plan(CLUSTERS, n, 8 if scratch else 6, local.RedOp.Sum)
    plan.import_xml(prefix)
    rng = np.random.default_rng(dt)
    npdt = O.NP_OF[dt]
    if dt == O.FP32:
        hosts = [rng.standard_normal(n).astype(np.float32) for _ in range(4)]
        want = (hosts[0] + hosts[1]) + (hosts[2] + hosts[3])        # cluster sums, then their sum
    elif dt == O.INT32:
        hosts = [rng.integers(-2**28, 2**28, n, dtype=np.int32) for _ in range(4)]
        want = hosts[0] + hosts[1] + hosts[2] + hosts[3]
    else:  # small integers are exact in bf16: the reference's i % 10 pattern, shifted per rank
        vals = [(np.arange(n) % 10 + r).astype(np.float32) for r in range(4)]
        hosts = [(v.view(np.uint32) >> 16).astype(np.uint16) for v in vals]
        want = (sum(vals).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    send = [to_dev(h) for h in hosts]
    keep = [s.clone() for s in send]
    ts = O.type_size(dt)
    recv = [dev_empty(n, ts, fill=0x55) for _ in range(4)]
    scr = [dev_empty(n, ts, fill=0x33) for _ in range(4)] if scratch else None
    plan.execute([s.data_ptr() for s in send], [r.data_ptr() for r in recv],
                 [s.data_ptr() for s in scr] if scr else None, dt)
    torch.cuda.synchronize()
    for r in range(4):
        assert same(from_dev(recv[r], npdt), want), (maker.__name__, r)
        assert torch.equal(send[r], keep[r])                        # user send buffers untouched


@pytest.mark.gpu
@pytest.mark.parametrize("commop", [PX.ALLGATHER, PX.GATHER, PX.ALLTOALL, PX.SCATTER, PX.BROADCAST, PX.REDUCE,
                                    PX.REDUCESCATTER],
                         ids=["allgather", "gather", "alltoall", "scatter", "broadcast", "reduce", "reducescatter"])
def test_plan_execute_one_cluster_block_moves(tmp_path, commop):
    """Out-of-place block movers of one cluster (four ranks): gathers fill every destination
    with one list copy; bytes compared with numpy slicing, the rest of recv untouched."""
    import torch
    nranks, chunk, root = 4, 30001, 2
    prefix = str(tmp_path / "plan")
    PX.one_cluster_collective(prefix, commop, nranks, root)
    n = nranks * chunk
    plan = local.Plan([0] * nranks, n, commop, local.RedOp.Sum)
    plan.import_xml(prefix)
    rng = np.random.default_rng(commop)
    hosts = [rng.integers(-2**28, 2**28, n, dtype=np.int32) for _ in range(nranks)]
    send = [to_dev(h) for h in hosts]
    recv = [dev_empty(n, 4, fill=0x55) for _ in range(nranks)]
    plan.execute([s.data_ptr() for s in send], [r.data_ptr() for r in recv], None, O.INT32, root=root)
    torch.cuda.synchronize()
    untouched = np.full(n, 0x55, dtype=np.int32)
    for r in range(nranks):
        got = from_dev(recv[r], np.int32)
        if commop == PX.ALLGATHER:
            want = np.concatenate([hosts[j][:chunk] for j in range(nranks)])
        elif commop == PX.GATHER:
            want = np.concatenate([hosts[j][:chunk] for j in range(nranks)]) if r == root else untouched
        elif commop == PX.ALLTOALL:
            want = np.concatenate([hosts[j][r * chunk:(r + 1) * chunk] for j in range(nranks)])
        elif commop == PX.SCATTER:
            want = np.concatenate([hosts[root][r * chunk:(r + 1) * chunk], untouched[chunk:]])
        elif commop == PX.BROADCAST:
            want = np.concatenate([hosts[root][:chunk], untouched[chunk:]])
        elif commop == PX.REDUCE:   # int32 sums of values below 2^28 in magnitude: no overflow for four ranks
            want = np.concatenate([sum(h[:chunk] for h in hosts), untouched[chunk:]]) if r == root else untouched
        else:
            want = np.concatenate([sum(h[r * chunk:(r + 1) * chunk] for h in hosts), untouched[chunk:]])
        assert same(got, want), (commop, r)


@pytest.mark.gpu
def test_plan_execute_one_cluster_random_shapes(tmp_path):
    """The same block movers for seeded random rank counts (1..8), roots and chunk sizes."""
    import random
    import torch
    rnd = random.Random(77)
    for case in range(120):
        commop = rnd.choice([PX.ALLGATHER, PX.GATHER, PX.ALLTOALL, PX.SCATTER, PX.BROADCAST, PX.REDUCE, PX.REDUCESCATTER])
        nranks = rnd.randint(1, 8)
        root = rnd.randrange(nranks)
        chunk = rnd.choice([1, 3, 16, 1000, rnd.randint(1, 40_000)])
        prefix = str(tmp_path / ("plan%d" % case))
        PX.one_cluster_collective(prefix, commop, nranks, root)
        n = nranks * chunk
        plan = local.Plan([0] * nranks, n, commop, local.RedOp.Sum)
        plan.import_xml(prefix)
        rng = np.random.default_rng(case)
        hosts = [rng.integers(-2**27, 2**27, n, dtype=np.int32) for _ in range(nranks)]
        send = [to_dev(h) for h in hosts]
        recv = [dev_empty(n, 4, fill=0x55) for _ in range(nranks)]
        plan.execute([s.data_ptr() for s in send], [r.data_ptr() for r in recv], None, O.INT32, root=root)
        torch.cuda.synchronize()
        untouched = np.full(n, 0x55, dtype=np.int32)
        for r in range(nranks):
            got = from_dev(recv[r], np.int32)
            if commop == PX.ALLGATHER:
                want = np.concatenate([hosts[j][:chunk] for j in range(nranks)])
            elif commop == PX.GATHER:
                want = np.concatenate([hosts[j][:chunk] for j in range(nranks)]) if r == root else untouched
            elif commop == PX.ALLTOALL:
                want = np.concatenate([hosts[j][r * chunk:(r + 1) * chunk] for j in range(nranks)])
            elif commop == PX.SCATTER:
                want = np.concatenate([hosts[root][r * chunk:(r + 1) * chunk], untouched[chunk:]])
            elif commop == PX.BROADCAST:
                want = np.concatenate([hosts[root][:chunk], untouched[chunk:]])
            elif commop == PX.REDUCE:
                want = np.concatenate([sum(h[:chunk] for h in hosts), untouched[chunk:]]) if r == root else untouched
            else:
                want = np.concatenate([sum(h[r * chunk:(r + 1) * chunk] for h in hosts), untouched[chunk:]])
            assert same(got, want.astype(np.int32)), (case, commop, nranks, root, chunk, r)
