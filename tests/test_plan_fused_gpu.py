"""The fused replay of C2C plans against the literal one, and the sparse sum behind it.

The reference assembles sums across a cluster by clearing all but a member's own slice
(flagcxC2cRefreshFunc::run, flagcx/core/c2c_algo.cc:586-608) and all-reducing whole buffers
(c2c_algo.cc:310-336).  The fused replay reads only the members that hold data.  What must
hold: the same bytes in every receive buffer as the literal replay, signed zeros included
(the reference adds +0.0 to every element: -0.0 inputs come out +0.0), NaNs where it has
NaNs, and maxima / minima untouched (the refresh acts for sums only, c2c_algo.cc:596)."""
import os
import random

import numpy as np
import pytest

from flagcx_amd import local
from oracle import c2c_plan_model as M
from oracle import cpu_oracle as O
from tests import plan_xml as PX
from tests.util import dev_empty, f32_to_bf16_bits, from_dev, same, to_dev

PLANS = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "plans")
CL8 = [0, 0, 0, 0, 1, 1, 1, 1]
CL4 = [0, 0, 1, 1]
FLOATS = (O.FP16, O.FP32, O.FP64, O.BF16)


def special_values(dt, n, seed, zero_share=0.3):
    """Random values with many signed zeros and a few NaNs, infinities and denormals."""
    rng = np.random.default_rng(seed)
    if dt in (O.INT32, O.INT8, O.INT64):
        npdt = O.NP_OF[dt]
        hi = 2**20 if dt != O.INT8 else 100
        v = rng.integers(-hi, hi, n).astype(npdt)
        v[rng.random(n) < zero_share] = 0
        return v
    f = rng.standard_normal(n)
    pick = rng.random(n)
    f[pick < zero_share] = -0.0
    f[pick < zero_share / 2] = 0.0
    f[(pick > 0.96) & (pick < 0.97)] = np.nan
    f[(pick > 0.97) & (pick < 0.975)] = np.inf
    f[(pick > 0.975) & (pick < 0.98)] = -np.inf
    f[(pick > 0.98) & (pick < 0.99)] = 1e-41
    if dt == O.FP32:
        return f.astype(np.float32)
    if dt == O.FP64:
        return f.astype(np.float64)
    if dt == O.FP16:
        return f.astype(np.float16)
    bits = f32_to_bf16_bits(np.nan_to_num(f.astype(np.float32), nan=0.0))
    bits[np.isnan(f)] = 0x7fc1                       # a NaN with a payload
    bits[(f == 0) & np.signbit(f)] = 0x8000
    return bits


# ------------------------------------------------------------ the sparse sum itself

@pytest.mark.gpu
@pytest.mark.parametrize("dt", [O.FP32, O.BF16, O.FP16, O.FP64, O.INT32, O.INT8])
def test_sparse_sum_equals_the_sum_over_zero_filled_members(dt):
    """flagcxLocalReduceBatchSparse over the members that hold data == flagcxLocalReduce over the
    full list with zero-filled buffers wherever the other members stand, bit for bit (NaNs by
    class): 1..12 members read, 1..4 left out, ragged counts, buffers inside cache lines and at
    other offsets modulo 16, several descriptors per call."""
    import torch
    rnd = random.Random(1000 + dt)
    npdt = np.dtype(O.NP_OF[dt])
    ts = npdt.itemsize
    for case in range(40):
        nlive = rnd.choice([1, 1, 2, 2, 3, 4, 5, 7, 8, 9, 12])
        nzero = rnd.randint(1, 4)
        ndescs = rnd.choice([1, 1, 2, 5])
        aligned = rnd.random() < 0.7 or nlive > 8
        descs_sparse, descs_full, outs_s, outs_f, keep = [], [], [], [], []
        for d in range(ndescs):
            n = rnd.choice([1, 7, 64, 1000, 4097, rnd.randint(1, 300_000)])
            base = rnd.randrange(0, 64) if not aligned else rnd.choice([0, 0, 16 // ts * rnd.randrange(0, 8)])
            lives = []
            for j in range(nlive):
                off = base if aligned else rnd.randrange(0, 32)
                t = to_dev(np.concatenate([np.zeros(off, npdt), special_values(dt, n, 7 * case + 13 * d + j)]))
                keep.append(t)
                lives.append(t.data_ptr() + off * ts)
            zero = torch.zeros((n + 64) * ts, dtype=torch.uint8, device="cuda")
            keep.append(zero)
            zoff = base if aligned else rnd.randrange(0, 32)
            full = list(lives)
            for _ in range(nzero):
                full.insert(rnd.randrange(0, len(full) + 1), zero.data_ptr() + zoff * ts)
            out_s = dev_empty(n + 64, ts, fill=0x55)
            out_f = dev_empty(n + 64, ts, fill=0x55)
            outs_s.append(out_s)
            outs_f.append(out_f)
            descs_sparse.append((lives, out_s.data_ptr() + base * ts, n))
            descs_full.append((full, out_f.data_ptr() + base * ts, n))
        local.reduce_batch_sparse(descs_sparse, local.RedOp.Sum, dt, nlive, nzero)
        local.reduce_batch(descs_full, local.RedOp.Sum, dt, nlive + nzero)
        torch.cuda.synchronize()
        for d in range(ndescs):
            a, b = from_dev(outs_s[d], npdt), from_dev(outs_f[d], npdt)
            assert same(a, b, nan_class=dt in FLOATS, dtype=dt), (case, d, nlive, nzero, aligned)


@pytest.mark.gpu
def test_sparse_sum_turns_minus_zero_into_plus_zero_and_keeps_everything_else():
    import torch
    for dt, npdt in ((O.FP32, np.float32), (O.FP64, np.float64), (O.FP16, np.float16)):
        x = np.array([-0.0, 0.0, 1.5, -2.25, np.inf, -np.inf, 6e-8, -6e-8], dtype=npdt)
        y = np.array([-0.0, -0.0, -1.5, 2.0, 1.0, 1.0, 0.0, -0.0], dtype=npdt)
        dx, dy = to_dev(x), to_dev(y)
        out = dev_empty(len(x), npdt().itemsize, fill=0x55)
        # one member read: x + (+0.0)
        local.reduce_batch_sparse([([dx.data_ptr()], out.data_ptr(), len(x))], local.RedOp.Sum, dt, 1, 3)
        torch.cuda.synchronize()
        assert same(from_dev(out, npdt), x + npdt(0.0))
        assert not np.signbit(from_dev(out, npdt)[0])
        # two members: (-0) + (-0) is -0 without zero members and +0 with one
        local.reduce_batch_sparse([([dx.data_ptr(), dy.data_ptr()], out.data_ptr(), len(x))], local.RedOp.Sum, dt, 2, 0)
        torch.cuda.synchronize()
        assert same(from_dev(out, npdt), y + x)
        assert np.signbit(from_dev(out, npdt)[0])
        local.reduce_batch_sparse([([dx.data_ptr(), dy.data_ptr()], out.data_ptr(), len(x))], local.RedOp.Sum, dt, 2, 1)
        torch.cuda.synchronize()
        assert same(from_dev(out, npdt), (y + x) + npdt(0.0))
        assert not np.signbit(from_dev(out, npdt)[0])


@pytest.mark.gpu
def test_sparse_sum_argument_checks():
    a = dev_empty(64, 4, fill=0)
    d = [([a.data_ptr()], a.data_ptr(), 64)]
    for op in (local.RedOp.Max, local.RedOp.Min, local.RedOp.Prod, local.RedOp.Avg):
        with pytest.raises(local.FlagcxError) as e:
            local.reduce_batch_sparse(d, op, O.FP32, 1, 1)
        assert e.value.code == int(local.Result.InvalidArgument)
    with pytest.raises(local.FlagcxError):
        local.reduce_batch_sparse(d, local.RedOp.Sum, O.FP32, 1, -1)
    with pytest.raises(local.FlagcxError):
        local.reduce_batch_sparse(d, local.RedOp.Sum, O.FP32, 1, 64)
    local.reduce_batch_sparse(d, local.RedOp.Max, O.FP32, 1, 0)        # nothing left out: any op


# ----------------------------------------------------------------- plans, both ways

def replay(prefix, clusters, n, commop, redop, hosts, dt, algo, fused, chunks=None, scratch=False, root=-1,
           in_place=False):
    """Returns (recv arrays, send arrays after the run, (bytes, launches))."""
    import torch
    nr = len(clusters)
    npdt = hosts[0].dtype
    ts = npdt.itemsize
    plan = local.Plan(clusters, n, commop, redop)
    if chunks:
        plan.set_chunks(chunks)
    plan.import_xml(prefix)
    plan.set_algorithm(algo)
    plan.set_fused(fused)
    send = [to_dev(h) for h in hosts]
    recv = send if in_place else [dev_empty(n, ts, fill=0x55) for _ in range(nr)]
    scr = [dev_empty(n, ts, fill=0x33) for _ in range(nr)] if scratch else None
    plan.execute([s.data_ptr() for s in send], [r.data_ptr() for r in recv],
                 [s.data_ptr() for s in scr] if scr else None, dt, root=root)
    torch.cuda.synchronize()
    return [from_dev(r, npdt) for r in recv], [from_dev(s, npdt) for s in send], plan.traffic()


@pytest.mark.gpu
@pytest.mark.parametrize("algo", [1, 2], ids=["pipeline", "input"])
@pytest.mark.parametrize("dt", [O.FP32, O.BF16, O.INT32])
def test_allreduce8_fused_equals_literal_with_signed_zeros_and_nans(dt, algo):
    """The 8-rank all-reduce fixture over inputs full of -0.0 / +0.0, NaN, infinities and
    denormals: fused == literal bit for bit (NaNs by class), both equal to the numpy model for
    fp32, every rank holds the same bytes, and a column of -0.0 on all ranks comes out +0.0 as
    in the reference (its zero members are +0.0)."""
    n = 8 * 12007
    hosts = [special_values(dt, n, 100 * dt + r) for r in range(8)]
    if dt != O.INT32:
        minus_zero = np.array([-0.0], dtype=np.float32 if dt == O.FP32 else np.float16)
        bits = hosts[0].dtype.type(0x8000) if dt == O.BF16 else None
        for h in hosts:                                  # columns 0..99 of every chunk: -0.0 on all ranks
            for c in range(8):
                h[c * (n // 8):c * (n // 8) + 100] = bits if dt == O.BF16 else minus_zero[0]
    prefix = os.path.join(PLANS, "allreduce8")
    lit, sent_l, tl = replay(prefix, CL8, n, 6, local.RedOp.Sum, hosts, dt, algo, False, chunks=8)
    fus, sent_f, tf = replay(prefix, CL8, n, 6, local.RedOp.Sum, hosts, dt, algo, True, chunks=8)
    isf = dt != O.INT32
    for r in range(8):
        assert same(fus[r], lit[r], nan_class=isf, dtype=dt), r
        assert same(fus[r], fus[0], nan_class=isf, dtype=dt), r
        assert same(sent_f[r], hosts[r]) and same(sent_l[r], hosts[r])
    if isf:
        z = fus[0].view(np.uint16 if dt == O.BF16 else np.uint32)
        for c in range(8):
            assert not z[c * (n // 8):c * (n // 8) + 100].any()      # +0.0, not -0.0
    if dt == O.FP32:
        m = M.Model(prefix, CL8, n, M.ALLREDUCE, M.SUM, default_chunks=8)
        mrecv = [np.full(n, 0x55555555, dtype=np.uint32).view(np.float32) for _ in range(8)]
        with np.errstate(invalid="ignore"):
            m.execute([h.copy() for h in hosts], mrecv, None, algorithm=algo)
        for r in range(8):
            assert same(fus[r], mrecv[r], nan_class=True, dtype=dt), r
    # the fused replay hands the kernels less than the literal one
    assert tf[0] < tl[0]


@pytest.mark.gpu
@pytest.mark.parametrize("dt", [O.FP32, O.BF16, O.INT32])
def test_reducescatter8_fused_equals_literal_and_moves_a_fraction(dt):
    """The sequential reduce-scatter with scratch: three refreshes of 3/4 of every rank's scratch
    buffer and two collectives that read them back in the literal replay; the fused one writes
    no zeros at all (scratch dies with the call) and reads live quarters only.  In algorithmic
    bytes, per chunk: literal 80 (pre) + 144 (refreshes) + 32 (hetero) + 176 (all-reduce and its
    copies to the members) + 40 (post) = 472, fused 80 + 0 + 32 + 144 + 16 = 272."""
    rc = 16411
    n = 8 * rc
    hosts = [special_values(dt, n, 300 * dt + r) for r in range(8)]
    prefix = os.path.join(PLANS, "reducescatter8")
    lit, _, tl = replay(prefix, CL8, n, 8, local.RedOp.Sum, hosts, dt, 0, False, chunks=8, scratch=True)
    fus, _, tf = replay(prefix, CL8, n, 8, local.RedOp.Sum, hosts, dt, 0, True, chunks=8, scratch=True)
    for r in range(8):
        assert same(fus[r], lit[r], nan_class=dt != O.INT32, dtype=dt), r
    assert tf[0] < 0.6 * tl[0] and tf[1] < tl[1], (tf, tl)


@pytest.mark.gpu
@pytest.mark.parametrize("maker,scratch", [(PX.allreduce_2x2_locred, False), (PX.allreduce_2x2_refresh_scratch, True),
                                           (PX.allreduce_2x2_reference_ops_only, False)],
                         ids=lambda v: getattr(v, "__name__", str(v)))
@pytest.mark.parametrize("redop", [local.RedOp.Sum, local.RedOp.Max, local.RedOp.Min])
def test_hand_written_plans_fused_equals_literal(tmp_path, maker, scratch, redop):
    """Plans that clear with an explicit buffType, keep nothing (count 0), or reduce with max /
    min (for which a refresh clears nothing, and, where the plan's refresh is a sum but its
    collective is not, the zeros are values like any other and are written before they are read)."""
    prefix = str(tmp_path / "p")
    maker(prefix)
    n = 4 * 10007
    hosts = [special_values(O.FP32, n, 500 + r) for r in range(4)]
    commop = 8 if scratch else 6        # staging in scratch: only where the reference owns one (c2c_algo.cc:2121-2131)
    lit, _, _ = replay(prefix, CL4, n, commop, redop, hosts, O.FP32, 2, False, scratch=scratch)
    fus, _, _ = replay(prefix, CL4, n, commop, redop, hosts, O.FP32, 2, True, scratch=scratch)
    for r in range(4):
        assert same(fus[r], lit[r], nan_class=True, dtype=O.FP32), r


@pytest.mark.gpu
def test_fused_replay_in_place():
    """sendbuff == recvbuff on every rank (flagcx/include/flagcx.h:340): the ranges a refresh
    clears are then part of what the send side reads."""
    n = 8 * 5003
    hosts = [special_values(O.FP32, n, 700 + r) for r in range(8)]
    prefix = os.path.join(PLANS, "allreduce8")
    lit, _, _ = replay(prefix, CL8, n, 6, local.RedOp.Sum, hosts, O.FP32, 2, False, chunks=8, in_place=True)
    fus, _, _ = replay(prefix, CL8, n, 6, local.RedOp.Sum, hosts, O.FP32, 2, True, chunks=8, in_place=True)
    for r in range(8):
        assert same(fus[r], lit[r], nan_class=True, dtype=O.FP32), r


@pytest.mark.gpu
def test_zeros_still_due_when_the_plan_ends_are_written(tmp_path):
    """A plan whose refresh clears a range that nothing overwrites afterwards: the fused replay
    writes those zeros at the end, and copies out of cleared ranges carry the zeros along."""
    prefix = str(tmp_path / "z")
    for r in range(4):
        h = r % 2
        refresh = dict(buffType=1, start=0, offset=2 * h, count=1, totalCount=4, redOp=0)
        pre = [[PX.homo(PX.ALLREDUCE, 0, 1, 0, 0, 4, 0)]]
        # chunk 2h + 1 was cleared on the sender: the receiver's chunk 2(1 - h) + 1 must end as zeros too
        het = [[[PX.p2p(r, (r + 2) % 4, 2 * h + 1, 1, 0), PX.p2p(r, (r + 2) % 4, 2 * (1 - h) + 1, 1, 1)]]]
        PX.write_rank(prefix, r, 4, (1, 0, 1, 0, 0), refresh, pre, het, [[]], [])
    n = 4 * 3001
    c = n // 4
    hosts = [special_values(O.FP32, n, 900 + r) for r in range(4)]
    lit, _, _ = replay(prefix, CL4, n, 6, local.RedOp.Sum, hosts, O.FP32, 2, False)
    fus, _, tf = replay(prefix, CL4, n, 6, local.RedOp.Sum, hosts, O.FP32, 2, True)
    for r in range(4):
        h = r % 2
        assert same(fus[r], lit[r], nan_class=True, dtype=O.FP32), r
        for chunk in range(4):                           # everything but the chunk the refresh keeps
            if chunk != 2 * h:
                assert not fus[r][chunk * c:(chunk + 1) * c].view(np.uint32).any(), (r, chunk)
