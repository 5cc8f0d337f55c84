"""Seeded random C2C plans replayed three ways: literally, fused, and by the numpy model of
flagcxC2cPlanner::execute (oracle/c2c_plan_model.py).  The plans mix what the fused replay has
to keep track of: refreshes of either buffer with random windows, hetero copies out of and into
cleared ranges, reduce-type and copy-type homo functions over ranges that are partly cleared, in
place and out of place, every algorithm setting.  int32 inputs: all three must agree bit for bit;
fp32 inputs full of signed zeros, NaNs and infinities: fused == literal bit for bit (NaNs by class)."""
import random

import numpy as np
import pytest

from flagcx_amd import local
from oracle import c2c_plan_model as M
from oracle import cpu_oracle as O
from tests import plan_xml as PX
from tests.test_plan_fused_gpu import special_values
from tests.util import from_dev, same, to_dev

NCH = 16            # chunks per buffer
NOP = 11


def rand_range(rnd, maxlen=NCH):
    n = rnd.randint(1, maxlen)
    o = rnd.randint(0, NCH - n)
    return o, n


def disjoint(a, an, b, bn):
    return a + an <= b or b + bn <= a


def homo_for_cluster(rnd, m, allow_scratch):
    """One homo function per member of a cluster of m ranks (a list of m dicts), or None."""
    op = rnd.choice([PX.ALLREDUCE, PX.ALLREDUCE, PX.REDUCE, PX.REDUCESCATTER, PX.REDUCESCATTER, PX.BROADCAST, PX.ALLGATHER,
                     NOP, PX.LOCRED, PX.LOCCPY, PX.GATHER, PX.SCATTER, PX.ALLTOALL])
    st = rnd.choice([0, 1, 1, 2] if allow_scratch else [0, 1, 1])
    rt = rnd.choice([1, 1, 2] if allow_scratch else [1])
    root = rnd.randrange(m)
    if op == NOP:
        return [PX.homo(NOP, st, rt, 0, 0, NCH, 0) for _ in range(m)]
    if op in (PX.ALLREDUCE, PX.REDUCE, PX.BROADCAST, PX.LOCRED, PX.LOCCPY):
        so, cnt = rand_range(rnd)
        if st == rt and rnd.random() < 0.5 and op not in (PX.LOCCPY,):
            ro = so                                        # in place
        else:
            for _ in range(50):
                ro = rnd.randint(0, NCH - cnt)
                if st != rt or disjoint(so, cnt, ro, cnt):
                    break
            else:
                return None
        return [PX.homo(op, st, rt, so, ro, cnt, 0, rootRank=root if op in (PX.REDUCE, PX.BROADCAST) else -1) for _ in range(m)]
    cnt = rnd.randint(1, NCH // m)
    big = rnd.randint(0, NCH - m * cnt)
    if op == PX.ALLTOALL:                                  # S = m blocks, D = m blocks, never the same range
        for _ in range(50):
            ro = rnd.randint(0, NCH - m * cnt)
            if st != rt or disjoint(big, m * cnt, ro, m * cnt):
                return [PX.homo(op, st, rt, big, ro, cnt, 0) for _ in range(m)]
        return None
    if op == PX.SCATTER:                                   # the root's S = m blocks, D = one block
        for _ in range(50):
            ro = rnd.randint(0, NCH - cnt)
            if st != rt or disjoint(big, m * cnt, ro, cnt):
                return [PX.homo(op, st, rt, big, ro, cnt, 0, rootRank=root) for _ in range(m)]
        return None
    if op == PX.GATHER:                                    # S = one block, the root's D = m blocks
        for _ in range(50):
            so = rnd.randint(0, NCH - cnt)
            if st != rt or disjoint(big, m * cnt, so, cnt):
                return [PX.homo(op, st, rt, so, big, cnt, 0, rootRank=root) for _ in range(m)]
        return None
    if op == PX.REDUCESCATTER:                             # S = m blocks, D = one block
        if st == rt and rnd.random() < 0.5:
            return [PX.homo(op, st, rt, big, big + h * cnt, cnt, 0) for h in range(m)]      # in place: own block
        for _ in range(50):
            ro = rnd.randint(0, NCH - cnt)
            if st != rt or disjoint(big, m * cnt, ro, cnt):
                return [PX.homo(op, st, rt, big, ro, cnt, 0) for _ in range(m)]
        return None
    # all-gather: S = one block, D = m blocks
    if st == rt and rnd.random() < 0.5:
        return [PX.homo(op, st, rt, big + h * cnt, big, cnt, 0) for h in range(m)]          # in place
    for _ in range(50):
        so = rnd.randint(0, NCH - cnt)
        if st != rt or disjoint(big, m * cnt, so, cnt):
            return [PX.homo(op, st, rt, so, big, cnt, 0) for _ in range(m)]
    return None


def hetero_step(rnd, nr, cluster_of):
    """One hetero function per rank: a few transfers between the clusters; on every rank the
    ranges it receives into are disjoint from each other and from the ranges it sends."""
    ops = [[] for _ in range(nr)]
    for _ in range(rnd.randint(0, nr)):
        a = rnd.randrange(nr)
        b = rnd.choice([r for r in range(nr) if cluster_of[r] != cluster_of[a]])
        cnt = rnd.randint(1, 4)
        so, ro = rnd.randint(0, NCH - cnt), rnd.randint(0, NCH - cnt)
        # nothing may be received into a range that the same rank receives into or sends from in this function
        if any(not disjoint(ro, cnt, o, c) for o, c in recv_ranges.get(b, []) + send_ranges.get(b, [])):
            continue
        if any(not disjoint(so, cnt, o, c) for o, c in recv_ranges.get(a, [])):
            continue
        ops[a].append(PX.p2p(a, b, so, cnt, 0))
        ops[b].append(PX.p2p(b, a, ro, cnt, 1))
        recv_ranges.setdefault(b, []).append((ro, cnt))
        send_ranges.setdefault(a, []).append((so, cnt))
    return ops


recv_ranges, send_ranges = {}, {}


def make_plan(prefix, rnd, nr, commop, sizes=None):
    """Writes <prefix>_<rank>.xml for nr ranks in two clusters of sizes[0] and sizes[1] ranks (halves by default)."""
    global recv_ranges, send_ranges
    sizes = sizes or (nr // 2, nr // 2)
    first = (0, sizes[0])
    cluster_of = [0] * sizes[0] + [1] * sizes[1]
    shape = rnd.choice([(1, 0, 1, 0, 1), (1, 0, 1, 1, 1), (0, 1, 1, 0, 1), (1, 0, 2, 0, 1)])
    n_pre, n_het, n_post = shape[0] + shape[1], shape[1] + shape[2] + shape[3], shape[3] + shape[4]
    allow_scratch = True

    def homo_steps(nsteps, maxfuncs):
        per_rank = [[[] for _ in range(nsteps)] for _ in range(nr)]
        for s in range(nsteps):
            for cl in range(2):
                for _ in range(rnd.randint(0, maxfuncs)):
                    fs = homo_for_cluster(rnd, sizes[cl], allow_scratch)
                    if fs is None:
                        continue
                    for h in range(sizes[cl]):
                        per_rank[first[cl] + h][s].append(fs[h])
        return per_rank

    pre, post = homo_steps(n_pre, 2), homo_steps(n_post, 2)
    het = [[None] * n_het for _ in range(nr)]
    inter = [[[] for _ in range(n_het)] for _ in range(nr)]
    for s in range(n_het):
        recv_ranges, send_ranges = {}, {}
        ops = hetero_step(rnd, nr, cluster_of)
        for r in range(nr):
            het[r][s] = [ops[r]]                           # one hetero function per rank and step, maybe without ops
        for cl in range(2):
            if rnd.random() < 0.7:
                fs = homo_for_cluster(rnd, sizes[cl], allow_scratch)
                if fs is not None:
                    for h in range(sizes[cl]):
                        fs[h]["homoType"] = 2
                        inter[first[cl] + h][s].append(fs[h])
    for r in range(nr):
        bufftype = rnd.choice([1, 2, -1])
        # buffType -1 under the pipeline algorithm starts at the cluster's part (c2c_algo.cc:2159-2163),
        # chunk sizes[0] * NCH / nr for the second cluster: the window has to fit behind it
        behind = NCH - (sizes[0] * NCH + nr - 1) // nr
        total = rnd.randint(1, min(NCH // 2, behind) if bufftype == -1 else NCH)
        start = rnd.randint(0, NCH - total)
        off = rnd.randint(0, total)
        cnt = rnd.randint(0, total - off)
        refresh = dict(buffType=bufftype, start=start, offset=off, count=cnt, totalCount=total,
                       redOp=rnd.choice([0, 0, 0, 5]))
        PX.write_rank(prefix, r, NCH, shape, refresh, pre[r], het[r], inter[r], post[r])


def replay(prefix, clusters, n, commop, redop, hosts, dt, algo, fused):
    import torch
    nr = len(clusters)
    npdt = hosts[0].dtype
    ts = npdt.itemsize
    plan = local.Plan(clusters, n, commop, redop)
    plan.import_xml(prefix)
    plan.set_algorithm(algo)
    plan.set_fused(fused)
    send = [to_dev(h) for h in hosts]
    recv = [to_dev(np.frombuffer(bytes([0x55]) * (n * ts), dtype=npdt)) for _ in range(nr)]
    scr = [to_dev(np.frombuffer(bytes([0x33]) * (n * ts), dtype=npdt)) for _ in range(nr)]
    plan.execute([s.data_ptr() for s in send], [r.data_ptr() for r in recv], [s.data_ptr() for s in scr], dt)
    torch.cuda.synchronize()
    return [from_dev(r, npdt) for r in recv], [from_dev(s, npdt) for s in send]


@pytest.mark.gpu
@pytest.mark.parametrize("block", range(6))
def test_random_plans_fused_literal_and_model_agree(tmp_path, block):
    rnd = random.Random(9000 + block)
    for case in range(25):
        sizes = rnd.choice([(2, 2), (4, 4), (2, 2), (4, 4), (1, 3), (2, 6), (5, 3), (3, 4)])   # unequal clusters too
        nr = sum(sizes)
        clusters = [0] * sizes[0] + [1] * sizes[1]
        commop = rnd.choice([6, 8])                        # all-reduce: staging in recv; reduce-scatter: in scratch
        redop = rnd.choice([local.RedOp.Sum, local.RedOp.Sum, local.RedOp.Sum, local.RedOp.Max, local.RedOp.Min])
        algo = rnd.choice([0, 1, 2])
        c = rnd.choice([1, 3, 64, 1000, 4099])
        n = NCH * c
        prefix = str(tmp_path / ("p%d_%d" % (block, case)))
        make_plan(prefix, rnd, nr, commop, sizes)
        tag = (block, case, sizes, commop, int(redop), algo, c)
        # int32: literal == fused == model
        rng = np.random.default_rng(100 * block + case)
        hosts = [rng.integers(-2**20, 2**20, n).astype(np.int32) for _ in range(nr)]
        lit, sent = replay(prefix, clusters, n, commop, redop, hosts, O.INT32, algo, False)
        fus, _ = replay(prefix, clusters, n, commop, redop, hosts, O.INT32, algo, True)
        m = M.Model(prefix, clusters, n, commop, int(redop))
        mrecv = [np.frombuffer(bytes([0x55]) * (n * 4), dtype=np.int32).copy() for _ in range(nr)]
        mscr = [np.frombuffer(bytes([0x33]) * (n * 4), dtype=np.int32).copy() for _ in range(nr)]
        with np.errstate(over="ignore"):
            m.execute([h.copy() for h in hosts], mrecv, mscr, algorithm=algo)
        for r in range(nr):
            assert same(fus[r], lit[r]), ("fused != literal", tag, r)
            assert same(lit[r], mrecv[r]), ("literal != model", tag, r)
            assert same(sent[r], hosts[r]), ("send buffer changed", tag, r)
        # fp32 with special values: fused == literal
        fh = [special_values(O.FP32, n, 1000 * block + 10 * case + r) for r in range(nr)]
        lit, _ = replay(prefix, clusters, n, commop, redop, fh, O.FP32, algo, False)
        fus, _ = replay(prefix, clusters, n, commop, redop, fh, O.FP32, algo, True)
        for r in range(nr):
            assert same(fus[r], lit[r], nan_class=True, dtype=O.FP32), ("fp32 fused != literal", tag, r)


def one_rank_cluster_plan(prefix, refresh, pre=(), het_ops=None):
    """Two ranks, one cluster each: rank 0 carries the function under test, rank 1 its counterpart."""
    for r in range(2):
        het = [[het_ops[r]]] if het_ops else [[[]]]
        PX.write_rank(prefix, r, 4, (1, 0, 1, 0, 1), refresh if r == 0 else PX.NO_REFRESH,
                      [list(pre)] if r == 0 else [[]], het, [[]], [[]])


@pytest.mark.gpu
@pytest.mark.parametrize("fused", [True, False], ids=["fused", "literal"])
@pytest.mark.parametrize("what", ["refresh", "refresh_moved_by_pipeline", "homo_send", "homo_recv", "loccpy_recv",
                                  "hetero_send", "hetero_recv"])
def test_a_function_that_reaches_past_total_count_is_refused(tmp_path, what, fused):
    """No buffer of a collective holds more than totalCount elements (c2c_algo.cc:623,2124): a
    plan whose function reads or writes past that is refused before the function is launched,
    and the receive buffers keep their bytes."""
    import torch
    n = 4 * 1000
    prefix = str(tmp_path / what)
    commop, algo = 6, 2
    ok = dict(buffType=1, start=0, offset=1, count=1, totalCount=4, redOp=0)
    if what == "refresh":
        one_rank_cluster_plan(prefix, dict(ok, start=1))                       # [1, 5) of 4 chunks
    elif what == "refresh_moved_by_pipeline":
        for r in (0, 1):                        # fits at chunk 0, but the second cluster's part starts at chunk 2
            PX.write_rank(prefix, r, 4, (1, 0, 1, 0, 1), dict(ok, buffType=-1) if r == 1 else PX.NO_REFRESH,
                          [[]], [[[]]], [[]], [[]])
        algo = 1
    elif what == "homo_send":
        one_rank_cluster_plan(prefix, PX.NO_REFRESH, [PX.homo(PX.ALLREDUCE, 0, 1, 2, 0, 3, 0)])
    elif what == "homo_recv":
        one_rank_cluster_plan(prefix, PX.NO_REFRESH, [PX.homo(PX.BROADCAST, 0, 1, 0, 3, 2, 0, rootRank=0)])
    elif what == "loccpy_recv":
        one_rank_cluster_plan(prefix, PX.NO_REFRESH, [PX.homo(PX.LOCCPY, 0, 1, 0, 4, 1, 0)])
    elif what == "hetero_send":
        one_rank_cluster_plan(prefix, PX.NO_REFRESH, het_ops=[[PX.p2p(0, 1, 3, 2, 0)], [PX.p2p(1, 0, 0, 2, 1)]])
    else:
        one_rank_cluster_plan(prefix, PX.NO_REFRESH, het_ops=[[PX.p2p(0, 1, 0, 2, 0)], [PX.p2p(1, 0, 3, 2, 1)]])
    plan = local.Plan([0, 1], n, commop, local.RedOp.Sum)
    plan.import_xml(prefix)
    plan.set_algorithm(algo)
    plan.set_fused(fused)
    hosts = [np.arange(n, dtype=np.int32) + r for r in range(2)]
    send = [to_dev(h) for h in hosts]
    fill = np.frombuffer(bytes([0x55]) * (n * 4), dtype=np.int32)
    recv = [to_dev(fill) for _ in range(2)]
    with pytest.raises(local.FlagcxError) as e:
        plan.execute([s.data_ptr() for s in send], [r.data_ptr() for r in recv], None, O.INT32)
    assert "past totalCount" in str(e.value)
    torch.cuda.synchronize()
    for r in range(2):
        assert same(from_dev(recv[r], np.int32), fill)
