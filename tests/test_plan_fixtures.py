"""C2C plan replay against documents written by the reference's own plan DSL
(tests/golden/plans, made by tests/golden/gen_plan_fixtures.py) and against the numpy
restatement of flagcxC2cPlanner::execute (oracle/c2c_plan_model.py); roots in the
second cluster; Send / Recv homo functions of all three homoTypes."""
import importlib.util
import os

import numpy as np
import pytest

from flagcx_amd import local
from oracle import c2c_plan_model as M
from oracle import cpu_oracle as O
from tests import plan_xml as PX
from tests.util import dev_empty, from_dev, same, to_dev

PLANS = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "plans")
CL8 = [0, 0, 0, 0, 1, 1, 1, 1]
# the generator of the fixtures holds the all-to-all-v chunk matrix they were written from
_spec = importlib.util.spec_from_file_location("gen_plan_fixtures", os.path.join(os.path.dirname(PLANS), "gen_plan_fixtures.py"))
GEN = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(GEN)


def fixture(name):
    return os.path.join(PLANS, name)


# ----------------------------------------------------------------- CPU: documents

def test_dsl_documents_need_a_chunk_count():
    plan = local.Plan(CL8, 8 * 64, 6, local.RedOp.Sum)
    with pytest.raises(local.FlagcxError) as e:
        plan.import_xml(fixture("allreduce8"))
    assert e.value.code == int(local.Result.InvalidArgument) and "nChunks" in str(e.value)


def test_reference_example_is_refused_for_its_negative_offsets():
    """flagcx/tools/test.py addresses cluster 1 with `rank - 4` for rank in 0..3: its
    documents for ranks 4..7 hold negative offsets, which the reference's reader would
    turn into huge sizes (strtoull).  They are refused, with the field named."""
    plan = local.Plan(CL8, 8 * 64, 6, local.RedOp.Sum)
    plan.set_chunks(8)
    with pytest.raises(local.FlagcxError) as e:
        plan.import_xml(fixture("test"))
    assert e.value.code == int(local.Result.InvalidArgument)
    assert "negative" in str(e.value) and "test_4.xml" in str(e.value)


@pytest.mark.parametrize("name,clusters,commop,chunks", [("allreduce8", CL8, 6, 8), ("allgather4", [0, 0, 1, 1], 7, 4),
                                                         ("alltoallv4", [0, 0, 1, 1], 10, 8)])
def test_dsl_layout_imports_and_exports_byte_for_byte(tmp_path, name, clusters, commop, chunks):
    """The DSL's pretty-printed layout has the indentation of exportXml
    (flagcx/core/c2c_algo.cc:1050-1087) and no <nChunks> line: exporting what was
    imported gives the fixture back byte for byte once that line is taken out."""
    plan = local.Plan(clusters, chunks * 16, commop, local.RedOp.Sum)
    plan.set_chunks(chunks)
    plan.import_xml(fixture(name))
    out = str(tmp_path / "out")
    plan.export_xml(out)
    for r in range(len(clusters)):
        got = open("%s_%d.xml" % (out, r)).read().splitlines()
        want = open("%s_%d.xml" % (fixture(name), r)).read().splitlines()
        assert got[1] == "  <nChunks>%d</nChunks>" % chunks
        assert got[:1] + got[2:] == want, r


@pytest.mark.parametrize("algo", [M.ALGO_PIPELINE, M.ALGO_INPUT])
def test_model_gives_the_allreduce_closed_form(algo):
    n = 8 * 40
    m = M.Model(fixture("allreduce8"), CL8, n, M.ALLREDUCE, M.SUM, default_chunks=8)
    send = [(np.arange(n) % 10 + r).astype(np.float32) for r in range(8)]      # the reference's i % 10 pattern
    recv = [np.full(n, -7, dtype=np.float32) for _ in range(8)]
    m.execute(send, recv, None, algorithm=algo)
    want = 8 * (np.arange(n) % 10).astype(np.float32) + 28
    for r in range(8):
        assert np.array_equal(recv[r], want), r


def test_model_gives_the_allgather_closed_form():
    m = M.Model(fixture("allgather4"), [0, 0, 1, 1], 4 * 5, M.ALLGATHER, M.SUM, default_chunks=4)
    assert (m.multi_nic, m.each_nic_per_rank) == (1, 1)
    send = [np.arange(5, dtype=np.float32) + 10 * r for r in range(4)]
    recv = [np.full(20, -1, dtype=np.float32) for _ in range(4)]
    m.execute(send, recv, None)
    for r in range(4):
        assert np.array_equal(recv[r], np.concatenate(send)), r


def alltoallv_case(scale, dtype, seed):
    """Counts / displacements in elements for the fixture's chunk matrix, inputs and the
    closed form: rank i's recv holds, at rDispls[i][r], what rank r keeps at sDispls[r][i]."""
    send_c, sd, recv_c, rd = GEN.alltoallv_layout()
    mul = lambda m: [[x * scale for x in row] for row in m]
    v = tuple(mul(m) for m in (send_c, sd, recv_c, rd))
    n = 8 * scale
    rng = np.random.default_rng(seed)
    hosts = [rng.integers(-2**30, 2**30, n).astype(dtype) for _ in range(4)]
    want = [np.frombuffer(bytes([0x55]) * (n * np.dtype(dtype).itemsize), dtype=dtype).copy() for _ in range(4)]
    for r in range(4):
        for i in range(4):
            c = v[0][r][i]
            want[i][v[3][i][r]:v[3][i][r] + c] = hosts[r][v[1][r][i]:v[1][r][i] + c]
    return n, v, hosts, want


def test_model_gives_the_alltoallv_closed_form():
    n, v, hosts, want = alltoallv_case(7, np.int32, 3)
    m = M.Model(fixture("alltoallv4"), [0, 0, 1, 1], n, M.ALLTOALLV, 5, default_chunks=8)
    recv = [np.full(n, 0x55555555, dtype=np.int32) for _ in range(4)]
    m.execute([h.copy() for h in hosts], recv, None, v_args=v)
    for r in range(4):
        assert np.array_equal(recv[r], want[r]), r


CL4 = [0, 0, 1, 1]


def int_inputs(nr, n, seed, npdt=np.int32):
    rng = np.random.default_rng(seed)
    return [rng.integers(-2**26, 2**26, n).astype(npdt) for _ in range(nr)]


def junk(n, npdt, byte):
    return np.frombuffer(bytes([byte]) * (n * np.dtype(npdt).itemsize), dtype=npdt).copy()


@pytest.mark.parametrize("algo", [M.ALGO_SEQUENTIAL, M.ALGO_INPUT])
def test_model_gives_the_reducescatter_closed_form(algo):
    """2 clusters of 4 as findStrategy lays the sequential reduce-scatter out: every staging
    step in scratch, rank r ends with the sum of everybody's r-th block and nothing else of
    its receive buffer is touched.  Under `sequential` the refreshes run where
    c2c_algo.cc:2205-2208 and 2276-2282 put them, which the closed form needs: without the one
    before the post function every block would come out four times too large."""
    rc = 33
    n = 8 * rc
    hosts = int_inputs(8, n, 21)
    m = M.Model(fixture("reducescatter8"), CL8, n, M.REDUCESCATTER, M.SUM, default_chunks=8)
    recv = [junk(n, np.int32, 0x55) for _ in range(8)]
    m.execute([h.copy() for h in hosts], recv, [junk(n, np.int32, 0x33) for _ in range(8)], algorithm=algo)
    total = sum(hosts)
    for r in range(8):
        assert np.array_equal(recv[r][:rc], total[r * rc:(r + 1) * rc]), r
        assert np.array_equal(recv[r][rc:], junk(n - rc, np.int32, 0x55)), r
    # the reference's own reduce-scatter pattern, floor(i / recvcount) on every rank: shard r = 8 r
    pat = [(np.arange(n) // rc).astype(np.float32) for _ in range(8)]
    recv = [np.full(n, -1, dtype=np.float32) for _ in range(8)]
    m.execute(pat, recv, [np.full(n, -2, dtype=np.float32) for _ in range(8)], algorithm=algo)
    for r in range(8):
        assert np.array_equal(recv[r][:rc], np.full(rc, 8.0 * r, dtype=np.float32)), r


@pytest.mark.parametrize("root", [6, 4])
def test_model_gives_the_reduce_closed_form(root):
    n = 4 * 29
    hosts = int_inputs(8, n, 22)
    m = M.Model(fixture("reduce8"), CL8, n, M.REDUCE, M.SUM, default_chunks=4)
    recv = [junk(n, np.int32, 0x55) for _ in range(8)]
    m.execute([h.copy() for h in hosts], recv, None, root=root, algorithm=M.ALGO_SEQUENTIAL)
    assert np.array_equal(recv[root], sum(hosts))


def test_model_gives_the_gather_closed_form():
    """Root 3 sits in the second cluster and stages its hetero receive in its RECEIVE buffer, the
    other ranks in scratch (c2c_algo.cc:2122-2131): the model, given scratch for every rank, must
    still take recv on the root, or block 1 of the result is not rank 1's."""
    s_ = 17
    n = 4 * s_
    hosts = int_inputs(4, n, 23)
    m = M.Model(fixture("gather4"), CL4, n, M.GATHER, 5, default_chunks=4)
    recv = [junk(n, np.int32, 0x55) for _ in range(4)]
    m.execute([h.copy() for h in hosts], recv, [junk(n, np.int32, 0x33) for _ in range(4)], root=3)
    assert np.array_equal(recv[3], np.concatenate([h[:s_] for h in hosts]))
    for r in range(3):
        assert np.array_equal(recv[r], junk(n, np.int32, 0x55)), r


def uneven4_expected(hosts, c):
    """By hand.  T = sum over the four ranks, halves T0 = T[:2c], T1 = T[2c:].  After hetero
    function 0 and the all-reduce behind it every rank holds T.  Function 1 exists on ranks 0
    and 2 only: they alone refresh again (keep their first half) and swap it into each other's
    second half: [T0, T0].  The post function exists in cluster 0 only: ranks 0 and 1 refresh
    (rank 1 keeps its second half) and rank 1 broadcasts: both end with [0, T1].  Ranks 2 and 3
    are not refreshed again: [T0, T0] and T."""
    t = sum(hosts)
    t0, t1, z = t[:2 * c], t[2 * c:], np.zeros(2 * c, dtype=t.dtype)
    return [np.concatenate([z, t1]), np.concatenate([z, t1]), np.concatenate([t0, t0]), t]


@pytest.mark.parametrize("algo", [M.ALGO_SEQUENTIAL, M.ALGO_PIPELINE, M.ALGO_INPUT])
def test_model_walks_every_ranks_own_tables(algo):
    """Ranks with fewer functions in a step leave its loop earlier (c2c_algo.cc:2204,2277) and are
    not refreshed again; a lock-step replay would wipe rank 3's first half."""
    c = 11
    n = 4 * c
    hosts = int_inputs(4, n, 24)
    m = M.Model(fixture("uneven4"), CL4, n, M.ALLREDUCE, M.SUM, default_chunks=4)
    recv = [junk(n, np.int32, 0x55) for _ in range(4)]
    m.execute([h.copy() for h in hosts], recv, None, algorithm=algo)
    for r, want in enumerate(uneven4_expected(hosts, c)):
        assert np.array_equal(recv[r], want), r


# ------------------------------------------------------------------ GPU: replay

def run_both(prefix, clusters, n, commop, redop, hosts, dt, algo, root=-1, chunks=None, scratch=False, is_inter=None,
             recv_fill=0x55, fused=True):
    """Replays the plan on the GPU and in the numpy model from the same inputs;
    returns (gpu recv arrays, model recv arrays, gpu send arrays after the run)."""
    import torch
    nr = len(clusters)
    npdt = hosts[0].dtype
    ts = npdt.itemsize
    plan = local.Plan(clusters, n, commop, redop, is_inter=is_inter)
    if chunks:
        plan.set_chunks(chunks)
    plan.import_xml(prefix)
    plan.set_algorithm(algo)
    plan.set_fused(fused)
    send = [to_dev(h) for h in hosts]
    recv = [to_dev(np.frombuffer(bytes([recv_fill]) * (n * ts), dtype=npdt)) for _ in range(nr)]     # the byte, repeated
    scr = [to_dev(np.frombuffer(bytes([0x33]) * (n * ts), dtype=npdt)) for _ in range(nr)] if scratch else None
    plan.execute([s.data_ptr() for s in send], [r.data_ptr() for r in recv],
                 [s.data_ptr() for s in scr] if scr else None, dt, root=root)
    torch.cuda.synchronize()
    m = M.Model(prefix, clusters, n, commop, int(redop), is_inter=is_inter, default_chunks=chunks)
    msend = [h.copy() for h in hosts]
    fillv = np.frombuffer(bytes([recv_fill]) * ts, dtype=npdt)[0]
    mrecv = [np.full(n, fillv, dtype=npdt) for _ in range(nr)]
    mscr = [np.frombuffer(bytes([0x33]) * (n * ts), dtype=npdt).copy() for _ in range(nr)] if scratch else None
    m.execute(msend, mrecv, mscr, root=root, algorithm=algo)
    return [from_dev(r, npdt) for r in recv], mrecv, [from_dev(s, npdt) for s in send]


@pytest.mark.gpu
@pytest.mark.parametrize("algo", [0, 1, 2], ids=["sequential", "pipeline", "input"])
@pytest.mark.parametrize("dt", [O.FP32, O.INT32, O.BF16])
def test_allreduce8_fixture_replays_like_the_reference(dt, algo):
    """8 ranks, 2 clusters of 4, set_pipeline(1, 0, 1, 1, 1), refresh per rank: the
    pipelined post step and the refresh placement of c2c_algo.cc:2160-2285.  The result
    equals the model's under every algorithm setting (under `sequential` the refreshes
    before the sequential post functions wipe gathered chunks: no all-reduce, and the
    same bytes in both), and the all-reduce closed form under `pipeline` and `input`."""
    n = 8 * 25001
    rng = np.random.default_rng(7 + dt)
    if dt == O.FP32:
        hosts = [rng.standard_normal(n).astype(np.float32) for _ in range(8)]
        closed = None                                   # rounding depends on the fold: the model is the reference
    elif dt == O.INT32:
        hosts = [rng.integers(-2**27, 2**27, n, dtype=np.int32) for _ in range(8)]
        closed = sum(hosts)
    else:   # small integers are exact in bf16: i % 10 shifted per rank
        vals = [(np.arange(n) % 10 + r).astype(np.float32) for r in range(8)]
        hosts = [(v.view(np.uint32) >> 16).astype(np.uint16) for v in vals]
        closed = (sum(vals).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    if dt == O.BF16:
        # the model folds numpy arrays: give it fp32 values and narrow its result (exact here)
        got, _, sent = run_both(fixture("allreduce8"), CL8, n, 6, local.RedOp.Sum, hosts, dt, algo, chunks=8, recv_fill=0)
        _, want32, _ = run_both(fixture("allreduce8"), CL8, n, 6, local.RedOp.Sum, vals, O.FP32, algo, chunks=8, recv_fill=0)
        want = [(w.view(np.uint32) >> 16).astype(np.uint16) for w in want32]
    else:
        got, want, sent = run_both(fixture("allreduce8"), CL8, n, 6, local.RedOp.Sum, hosts, dt, algo, chunks=8)
    for r in range(8):
        assert same(got[r], want[r]), (algo, r)
        assert same(sent[r], hosts[r])                  # user send buffers untouched
        if algo != 0 and closed is not None:
            assert same(got[r], closed), (algo, r)
    if algo != 0 and dt == O.FP32:
        # every rank holds the same bytes, and they are the all-reduce up to rounding
        exact = sum(h.astype(np.float64) for h in hosts)
        for r in range(8):
            assert same(got[r], got[0])
        assert np.allclose(got[0], exact, rtol=0, atol=1e-5)
    if algo == 0:
        assert not np.array_equal(got[0], got[4])       # not an all-reduce: documented, and equal to the model


@pytest.mark.gpu
def test_allgather4_fixture_sends_from_the_user_buffer():
    """2 clusters of 2, every rank an inter-rank: the hetero sends read the SEND buffer
    (c2c_algo.cc:2132-2137, the all-gather case of sendTmpBuff)."""
    n = 4 * 30001
    rng = np.random.default_rng(11)
    hosts = [rng.integers(-2**30, 2**30, n // 4, dtype=np.int32) for _ in range(4)]
    # recvcount-sized send buffers: a read from recv instead of send would be out of place
    got, want, _ = run_both(fixture("allgather4"), [0, 0, 1, 1], n, 7, local.RedOp.Sum,
                            [np.concatenate([h, np.zeros(n - len(h), np.int32)]) for h in hosts], O.INT32, 2, chunks=4)
    for r in range(4):
        assert same(got[r], np.concatenate(hosts)), r
        assert same(got[r], want[r]), r


@pytest.mark.gpu
@pytest.mark.parametrize("npdt,dt", [(np.int32, O.INT32), (np.float32, O.FP32), (np.int8, O.INT8)])
def test_alltoallv4_fixture_moves_every_piece(npdt, dt):
    """2 clusters of 2: the pieces for the own cluster travel in the AlltoAllv homo function
    with the caller's counts and displacements (c2c_algo.cc:482-508), the others as the
    plan's P2P ops (c2c_algo.cc:1618-1630); ragged counts, two empty pieces."""
    import torch
    scale = 30001
    n, v, hosts, want = alltoallv_case(scale, npdt, 5)
    ts = np.dtype(npdt).itemsize
    plan = local.Plan([0, 0, 1, 1], n, 10, local.RedOp.Sum)
    plan.set_chunks(8)
    plan.import_xml(fixture("alltoallv4"))
    send = [to_dev(h) for h in hosts]
    recv = [to_dev(np.frombuffer(bytes([0x55]) * (n * ts), dtype=npdt)) for _ in range(4)]
    # without the arrays the homo function cannot run (c2c_algo.cc:2083-2089)
    with pytest.raises(local.FlagcxError) as e:
        plan.execute([s.data_ptr() for s in send], [r.data_ptr() for r in recv], None, dt)
    assert e.value.code == int(local.Result.InvalidArgument) and "AlltoAllv" in str(e.value)
    with pytest.raises(local.FlagcxError) as e:
        plan.set_alltoallv(v[0], None, v[2], v[3])
    assert e.value.code == int(local.Result.InvalidArgument)
    plan.set_alltoallv(*v)
    plan.execute([s.data_ptr() for s in send], [r.data_ptr() for r in recv], None, dt)
    torch.cuda.synchronize()
    m = M.Model(fixture("alltoallv4"), [0, 0, 1, 1], n, M.ALLTOALLV, 0, default_chunks=8)
    mrecv = [np.frombuffer(bytes([0x55]) * (n * ts), dtype=npdt).copy() for _ in range(4)]
    m.execute([h.copy() for h in hosts], mrecv, None, v_args=v)
    for r in range(4):
        got = from_dev(recv[r], npdt)
        assert same(got, want[r]), r
        assert same(got, mrecv[r]), r
        assert same(from_dev(send[r], npdt), hosts[r]), r
    # a receive count that no send matches is an error, not a hang
    bad = [[list(row) for row in m_] for m_ in v]
    bad[2][1][0] += 1
    plan.set_alltoallv(*bad)
    with pytest.raises(local.FlagcxError) as e:
        plan.execute([s.data_ptr() for s in send], [r.data_ptr() for r in recv], None, dt)
    assert e.value.code == int(local.Result.InvalidUsage)


def broadcast_two_clusters(prefix, root):
    """8 ranks, 2 clusters of 4, broadcast from `root` (cluster 1): the root cluster
    broadcasts inside itself with rootRank -1 (the collective's root), every rank sends
    the buffer to the rank of the same index in cluster 0."""
    for r in range(8):
        cl, h = r // 4, r % 4
        pre = [[PX.homo(PX.BROADCAST if cl == 1 else 11, 0 if cl == 1 else 1, 1, 0, 0, 4, 0)]]
        het = [[[PX.p2p(r, r - 4, 0, 4, 0)]]] if cl == 1 else [[[PX.p2p(r, r + 4, 0, 4, 1)]]]
        PX.write_rank(prefix, r, 4, (1, 0, 1, 0, 0), PX.NO_REFRESH, pre, het, [[]], [])


@pytest.mark.gpu
@pytest.mark.parametrize("root", [5, 7, 4])
def test_root_in_the_second_cluster_is_mapped_to_its_homo_rank(tmp_path, root):
    """The collective's root is a global rank; homo functions with rootRank -1 get
    globalrank2homorank[root] (c2c_algo.cc:2147,2170)."""
    prefix = str(tmp_path / "bc")
    broadcast_two_clusters(prefix, root)
    n = 4 * 9001
    rng = np.random.default_rng(root)
    hosts = [rng.integers(-2**30, 2**30, n, dtype=np.int32) for _ in range(8)]
    got, want, _ = run_both(prefix, CL8, n, 2, local.RedOp.Sum, hosts, O.INT32, 2, root=root)
    for r in range(8):
        assert same(got[r], hosts[root]), r
        assert same(got[r], want[r]), r


def send_recv_plan(prefix):
    """2 clusters of 2 (ranks 0,1 | 2,3), every rank an inter-rank, 6 chunks.  Cluster 0:
      pre    homoType 0, root 0: rank 0 sends send[0:1) to inter-rank 1, which receives at recv[4:5)
      hetero rank 2 -> rank 1 at recv[2:3), rank 3 -> rank 1 at recv[3:4)
      inter  homoType 1: inter-rank 1 sends what it received to inter-rank 0, piece by piece
      post   homoType 2, root 1: inter-rank 0 sends recv[2:4) to the root, which receives at recv[0:2)
    Cluster 1 only feeds the hetero step."""
    SEND, RECV, NOP = 0, 1, 11
    for r in range(4):
        if r == 0:
            pre, inter = [[PX.homo(SEND, 0, 1, 0, 0, 1, 0, rootRank=0)]], [[PX.homo(RECV, 1, 1, 0, 0, 6, 1)]]
            post = [[PX.homo(SEND, 1, 1, 2, 0, 2, 2, rootRank=1)]]
            het = [[[]]]    # a hetero function without P2P ops, as findStrategy pushes one for every rank
                            # (c2c_algo.cc:1763-1766): with none at all the rank would never reach its inter function
        elif r == 1:
            pre, inter = [[PX.homo(RECV, 0, 1, 0, 4, 1, 0, rootRank=0)]], [[PX.homo(SEND, 1, 1, 0, 0, 6, 1)]]
            post = [[PX.homo(RECV, 1, 1, 0, 0, 2, 2, rootRank=1)]]
            het = [[[PX.p2p(1, 2, 2, 1, 1), PX.p2p(1, 3, 3, 1, 1)]]]
        else:
            pre, inter, post = [[PX.homo(NOP, 0, 1, 0, 0, 6, 0)]], [[PX.homo(NOP, 1, 1, 0, 0, 6, 1)]], [[]]
            het = [[[PX.p2p(r, 1, 0, 1, 0)]]]
        PX.write_rank(prefix, r, 6, (1, 0, 1, 0, 1), PX.NO_REFRESH, pre, het, inter, post)


@pytest.mark.gpu
def test_send_recv_homo_functions_of_all_three_types(tmp_path):
    """Send / Recv homo functions (c2c_algo.cc:364-463).  The collective is a gather to rank 1:
    every other rank stages its hetero functions in scratch (c2c_algo.cc:2122-2137), so ranks 2
    and 3 send what their scratch buffers hold, and the root receives into its receive buffer."""
    import torch
    prefix = str(tmp_path / "sr")
    send_recv_plan(prefix)
    c = 5003
    n = 6 * c
    rng = np.random.default_rng(3)
    hosts = [rng.integers(-2**30, 2**30, n, dtype=np.int32) for _ in range(4)]
    plan = local.Plan([0, 0, 1, 1], n, 3, local.RedOp.Sum)       # gather
    plan.import_xml(prefix)
    send = [to_dev(h) for h in hosts]
    fills = [np.full(n, 1000 + r, dtype=np.int32) for r in range(4)]
    recv = [to_dev(f) for f in fills]
    scr = [to_dev(np.full(n, 2000 + r, dtype=np.int32)) for r in range(4)]
    # without scratch the ranks that stage there cannot run their hetero functions
    with pytest.raises(local.FlagcxError) as e:
        plan.execute([s.data_ptr() for s in send], [r.data_ptr() for r in recv], None, O.INT32, root=1)
    assert e.value.code == int(local.Result.InvalidArgument) and "scratch" in str(e.value)
    recv = [to_dev(f) for f in fills]
    plan.execute([s.data_ptr() for s in send], [r.data_ptr() for r in recv], [s.data_ptr() for s in scr], O.INT32, root=1)
    torch.cuda.synchronize()
    got = [from_dev(r, np.int32) for r in recv]
    # by hand: rank 1 gets send_0's first chunk at chunk 4, the two hetero pieces at chunks 2 and 3
    # (the senders' scratch fill), rank 0 gets those two pieces at the same place, and finally rank 1
    # gets them at chunks 0 and 1
    want0 = fills[0].copy()
    want0[2 * c:3 * c], want0[3 * c:4 * c] = 2002, 2003
    want1 = fills[1].copy()
    want1[4 * c:5 * c] = hosts[0][:c]
    want1[2 * c:3 * c], want1[3 * c:4 * c] = 2002, 2003
    want1[0:c], want1[c:2 * c] = 2002, 2003
    assert same(got[0], want0)
    assert same(got[1], want1)
    assert same(got[2], fills[2]) and same(got[3], fills[3])
    # and the same from the model
    m = M.Model(prefix, [0, 0, 1, 1], n, M.GATHER, M.SUM)
    mrecv = [f.copy() for f in fills]
    m.execute([h.copy() for h in hosts], mrecv, [np.full(n, 2000 + r, dtype=np.int32) for r in range(4)], root=1)
    for r in range(4):
        assert same(got[r], mrecv[r]), r


def case_inputs(dt, nr, n, seed):
    """Random inputs, the numpy carrier type, and whether sums are exact (closed form usable)."""
    rng = np.random.default_rng(seed)
    if dt == O.FP32:
        return [rng.standard_normal(n).astype(np.float32) for _ in range(nr)], False
    if dt == O.INT32:
        return [rng.integers(-2**26, 2**26, n).astype(np.int32) for _ in range(nr)], True
    raise ValueError(dt)


@pytest.mark.gpu
@pytest.mark.parametrize("fused", [True, False], ids=["fused", "literal"])
@pytest.mark.parametrize("algo", [0, 2], ids=["sequential", "input"])
@pytest.mark.parametrize("dt", [O.FP32, O.INT32])
def test_reducescatter8_fixture_with_scratch(dt, algo, fused):
    """The sequential reduce-scatter of findStrategy for 2 clusters of 4, replayed with scratch:
    cluster sums into scratch, quarters across, all-reduce of the scratch buffers (2 of 4 members
    hold data per quarter), refresh, reduce-scatter out of scratch (1 of 4).  Same bytes as the
    numpy model, the closed form for integers, recv beyond the shard untouched."""
    rc = 20011
    n = 8 * rc
    hosts, exact = case_inputs(dt, 8, n, 31 + dt)
    got, want, sent = run_both(fixture("reducescatter8"), CL8, n, 8, local.RedOp.Sum, hosts, dt, algo, chunks=8,
                               scratch=True, fused=fused)
    total = sum(hosts)
    for r in range(8):
        assert same(got[r], want[r]), (algo, r)
        assert same(sent[r], hosts[r])
        assert same(got[r][rc:], junk(n - rc, hosts[0].dtype, 0x55)), r
        if exact:
            assert same(got[r][:rc], total[r * rc:(r + 1) * rc]), r


@pytest.mark.gpu
@pytest.mark.parametrize("fused", [True, False], ids=["fused", "literal"])
@pytest.mark.parametrize("root", [6, 5])
@pytest.mark.parametrize("dt", [O.FP32, O.INT32])
def test_reduce8_fixture_root_in_the_second_cluster(dt, root, fused):
    n = 4 * 15013
    hosts, exact = case_inputs(dt, 8, n, 41 + dt)
    got, want, sent = run_both(fixture("reduce8"), CL8, n, 5, local.RedOp.Sum, hosts, dt, 0, root=root, chunks=4,
                               fused=fused)
    for r in range(8):
        assert same(got[r], want[r]), r
        assert same(sent[r], hosts[r])
    if exact:
        assert same(got[root], sum(hosts))


@pytest.mark.gpu
@pytest.mark.parametrize("fused", [True, False], ids=["fused", "literal"])
def test_gather4_fixture_root_stages_in_its_receive_buffer(fused):
    """Root 3 in the second cluster; scratch handed over for EVERY rank.  The reference gives the
    root no scratch buffer (c2c_algo.cc:2122-2129), so its hetero receive lands in recvbuff, where
    its Send function of homoType 1 then reads it."""
    s_ = 9001
    n = 4 * s_
    hosts = int_inputs(4, n, 51)
    got, want, sent = run_both(fixture("gather4"), CL4, n, 3, 5, hosts, O.INT32, 0, root=3, chunks=4, scratch=True,
                               fused=fused)
    assert same(got[3], np.concatenate([h[:s_] for h in hosts]))
    for r in range(4):
        assert same(got[r], want[r]), r
        assert same(sent[r], hosts[r])
        if r != 3:
            assert same(got[r], junk(n, np.int32, 0x55)), r


@pytest.mark.gpu
@pytest.mark.parametrize("fused", [True, False], ids=["fused", "literal"])
@pytest.mark.parametrize("algo", [0, 1, 2], ids=["sequential", "pipeline", "input"])
def test_uneven4_fixture_every_rank_walks_its_own_tables(algo, fused):
    c = 7001
    n = 4 * c
    hosts = int_inputs(4, n, 61)
    got, want, _ = run_both(fixture("uneven4"), CL4, n, 6, local.RedOp.Sum, hosts, O.INT32, algo, chunks=4, fused=fused)
    for r, by_hand in enumerate(uneven4_expected(hosts, c)):
        assert same(got[r], by_hand), r
        assert same(got[r], want[r]), r


@pytest.mark.gpu
def test_a_collective_that_lacks_a_member_is_refused(tmp_path):
    """Rank 1 has no hetero function in the sequential step, so in the reference it never reaches
    the all-reduce behind it, which its cluster then waits for forever; here: flagcxInvalidUsage."""
    prefix = str(tmp_path / "lack")
    for r in range(4):
        het = [[]] if r == 1 else [[[]]]                  # <Step/> against a step with one empty function
        inter = [[PX.homo(PX.ALLREDUCE, 1, 1, 0, 0, 4, 0)]]
        PX.write_rank(prefix, r, 4, (0, 0, 1, 0, 0), PX.NO_REFRESH, [], het, inter, [])
    n = 4 * 100
    plan = local.Plan(CL4, n, 6, local.RedOp.Sum)
    plan.import_xml(prefix)
    bufs = [dev_empty(n, 4, fill=1) for _ in range(8)]
    with pytest.raises(local.FlagcxError) as e:
        plan.execute([b.data_ptr() for b in bufs[:4]], [b.data_ptr() for b in bufs[4:]], None, O.INT32)
    assert e.value.code == int(local.Result.InvalidUsage) and "rank 1" in str(e.value)
