"""The entry points allocate nothing and never synchronise on a non-NULL stream, so a
launch-bound sequence of them (the 4 MiB chunk steps of a shard) can be captured once
into a HIP graph and replayed.  Replays are checked one by one against the eager
result, with eager work and synchronisation between them."""
import numpy as np
import pytest

from oracle import cpu_oracle as O
from tests.util import from_dev, make_inputs, same, to_dev

pytestmark = pytest.mark.gpu


def test_chunked_reduce_scatter_pipeline_replays_from_a_graph():
    import torch
    from flagcx_amd import local as L
    assert L.lib().flagcxLocalInit() == 0
    dt, op, k = O.BF16, O.SUM, 8
    chunk, nchunks = 64 * 1024, 12                 # elements per chunk, chunks per shard
    n = chunk * nchunks
    ins = make_inputs(dt, k, n, seed=77)
    devs = [to_dev(a) for a in ins]
    staged = torch.zeros(k * n, dtype=torch.int16, device="cuda")      # pack target, rank-major
    out = torch.zeros(n, dtype=torch.int16, device="cuda")
    mirror = torch.zeros(n, dtype=torch.int16, device="cuda")
    scratch = torch.zeros(2 * n, dtype=torch.int16, device="cuda")
    rc, want = O.reduce(ins, dt, op)
    assert rc == 0

    def pipeline():
        # refresh (fill kernel), pack the k inputs, reduce chunk by chunk, copy the shard out
        L.refresh(scratch, 0, n // 2, n, 2 * n, L.RedOp.Sum, dtype=dt)
        L.pack_list(staged.data_ptr(), [d.data_ptr() for d in devs], n * 2)
        for c in range(nchunks):
            srcs = [staged.data_ptr() + (j * n + c * chunk) * 2 for j in range(k)]
            st = L.current_stream()
            L.check(L.lib().flagcxLocalReduce(L._ptr_array(srcs), k, out.data_ptr() + c * chunk * 2, chunk,
                                              int(dt), int(op), L._sref(st)))
        L.memcpy(mirror.data_ptr(), out.data_ptr(), n * 2)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        pipeline()                                  # eager warm-up on the capture stream
    side.synchronize()
    assert same(from_dev(mirror, np.uint16), want, nan_class=True, dtype=dt)

    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=side):
        pipeline()
    for rep in range(4):
        # new inputs every replay: rotate which device buffer holds which input
        perm = np.roll(np.arange(k), rep + 1)
        for j in range(k):
            devs[j].copy_(to_dev(ins[perm[j]]))
        out.zero_()
        mirror.zero_()
        scratch.fill_(0x1234)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        rc, want_rep = O.reduce([ins[perm[j]] for j in range(k)], dt, op)
        assert same(from_dev(out, np.uint16), want_rep, nan_class=True, dtype=dt), rep
        assert same(from_dev(mirror, np.uint16), want_rep, nan_class=True, dtype=dt), rep
        s = from_dev(scratch, np.uint16)
        assert not s[:n // 2].any() and not s[n // 2 + n:].any() and (s[n // 2:n // 2 + n] == 0x1234).all(), rep


@pytest.mark.parametrize("name,commop,scratch", [("allreduce8", 6, False), ("reducescatter8", 8, True)])
@pytest.mark.parametrize("fused", [True, False], ids=["fused", "literal"])
def test_plan_replay_is_captured_once_and_replayed_on_new_inputs(name, commop, scratch, fused):
    """flagcxLocalPlanExecute only launches kernels (a refresh is a fill kernel, copies are the
    batch kernel), and the fused replay decides on the host, from the plan alone, which members a
    sum reads: so one Execute captured into a HIP graph stands for every later one with the same
    buffers.  Four replays on new inputs, the receive and scratch buffers refilled with junk in
    between, each compared with the numpy model of flagcxC2cPlanner::execute."""
    import torch
    from flagcx_amd import local as L
    from oracle import c2c_plan_model as M
    from tests.test_plan_fixtures import CL8, fixture
    assert L.lib().flagcxLocalInit() == 0
    nr, n = 8, 8 * 3001
    plan = L.Plan(CL8, n, commop, L.RedOp.Sum)
    plan.set_chunks(8)
    plan.import_xml(fixture(name))
    plan.set_algorithm(2)
    plan.set_fused(fused)
    send = [torch.zeros(n, dtype=torch.int32, device="cuda") for _ in range(nr)]
    recv = [torch.zeros(n, dtype=torch.int32, device="cuda") for _ in range(nr)]
    scr = [torch.zeros(n, dtype=torch.int32, device="cuda") for _ in range(nr)] if scratch else None
    ptrs = ([s.data_ptr() for s in send], [r.data_ptr() for r in recv], [s.data_ptr() for s in scr] if scr else None)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        plan.execute(*ptrs, O.INT32)                # eager warm-up on the capture stream
    side.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=side, capture_error_mode="global"):
        plan.execute(*ptrs, O.INT32)
    model = M.Model(fixture(name), CL8, n, commop, 0, default_chunks=8)
    for rep in range(4):
        rng = np.random.default_rng(500 + rep)
        hosts = [rng.integers(-2**27, 2**27, n, dtype=np.int32) for _ in range(nr)]
        for r in range(nr):
            send[r].copy_(to_dev(hosts[r]))
            recv[r].fill_(0x55550000 + rep)
            if scr:
                scr[r].fill_(0x33330000 + rep)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        mrecv = [np.full(n, 0x55550000 + rep, dtype=np.int32) for _ in range(nr)]
        mscr = [np.full(n, 0x33330000 + rep, dtype=np.int32) for _ in range(nr)] if scratch else None
        model.execute([h.copy() for h in hosts], mrecv, mscr, algorithm=2)
        for r in range(nr):
            assert same(from_dev(recv[r], np.int32), mrecv[r]), (rep, r)
            assert same(from_dev(send[r], np.int32), hosts[r]), (rep, r)
