#!/usr/bin/env python3
"""Writes the C2C plan fixtures under tests/golden/plans/ with the reference's own
plan DSL (flagcx/tools/algorithm.py, standard library only), so that the importer
of flagcxLocalPlanImportXml is tested on files its own author did not format.

Run in the build container only (the reference tree is not on the GPU box):

    python tests/golden/gen_plan_fixtures.py [/root/reference]

The fixtures are data: plan documents, no reference code.  Three sets:

  test_{0..7}.xml        the workflow of flagcx/tools/test.py run as it stands.  Its
                         cluster-1 half addresses buffers with `rank - 4` where rank
                         runs 0..3, so those documents hold negative offsets and
                         global ranks as roots: they pin the DSL's layout (tag order,
                         pretty-printer whitespace, no <nChunks>, <Step/> for an empty
                         step) and must be refused at execution, not replayed.
  allreduce8_{0..7}.xml  the same workflow with the cluster-1 half written out as
                         its cluster-0 half reads (offsets rank, rank + 4; homo ranks
                         as roots): an 8-rank all-reduce over 2 clusters of 4,
                         set_pipeline(1, 0, 1, 1, 1), refresh per rank.
  allgather4_{0..3}.xml  the all-gather that flagcxC2cPlanner::findStrategy lays out
                         for 2 clusters of 2 where every rank is an inter-rank
                         (flagcx/core/c2c_algo.cc:1494-1537, 1668-1690, 1824-1866):
                         hetero sends read the user send buffer.
  alltoallv4_{0..3}.xml  the all-to-all-v that findStrategy lays out for 2 clusters of 2
                         (flagcx/core/c2c_algo.cc:1554-1556, 1618-1630, and the NoOp inter
                         and post functions): the pieces for the own cluster travel in the
                         AlltoAllv homo function, whose counts are arguments of execute()
                         and not part of the document; the cross-cluster pieces are P2P ops
                         with their displacements and counts.  ALLTOALLV_UNITS below is the
                         count / displacement matrix in chunks, shared with the test.
  reducescatter8_{0..7}.xml  the reduce-scatter that findStrategy lays out with the sequential
                         algorithm for 2 clusters of 4, every rank an inter-rank
                         (c2c_algo.cc:1125-1201 buffer lists, 1406-1453 refresh, 1494-1503 pre,
                         1227-1394 + 1653-1694 hetero, 1771-1774 inter, 1828-1831 post): every
                         staging buffer is scratch (buffType / sendType / recvType 2), refresh per
                         rank keeps the quarter the rank forwards; 8 chunks of recvcount.
  reduce8_{0..7}.xml     the reduce to a root in cluster 1 for the same 8 ranks
                         (c2c_algo.cc:1142-1150 root cluster scheduled, 1499-1503 pre,
                         1775-1779 inter Reduce on homo_comm with rootRank -1, no post function);
                         4 chunks of count / 4.
  gather4_{0..3}.xml     the gather to rank 3 for 2 clusters of 2 (c2c_algo.cc:1128-1150,
                         1406-1411 buffType 2 off the root, 1475-1486 recvType / sendType per
                         rank, 1533-1536 pre AllGather, 1800-1807 inter Send / Recv of homoType 1,
                         1871-1878 post Send / Recv of homoType 2): the root stages in its
                         receive buffer, everybody else in scratch; 4 chunks of sendcount.
  uneven4_{0..3}.xml     NOT a findStrategy layout: 2 clusters of 2 where ranks 0 and 2 hold two
                         hetero functions in the sequential step, ranks 1 and 3 one, and only
                         cluster 0 holds a post function.  In the reference every rank walks its
                         own tables (c2c_algo.cc:2204,2277), so only the ranks that still have a
                         function refresh again; the expected buffers are derived by hand in the
                         test that replays it.
"""
import os
import runpy
import shutil
import sys
import tempfile

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
TOOLS = os.path.join(REF, "flagcx", "tools")
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "plans")


def reference_example(outdir):
    """flagcx/tools/test.py, unchanged: it writes output/test_<rank>.xml."""
    work = tempfile.mkdtemp()
    os.makedirs(os.path.join(work, "output"))
    cwd = os.getcwd()
    os.chdir(work)
    try:
        runpy.run_path(os.path.join(TOOLS, "test.py"), run_name="__main__")
    finally:
        os.chdir(cwd)
    for r in range(8):
        shutil.copy(os.path.join(work, "output", "test_%d.xml" % r), os.path.join(outdir, "test_%d.xml" % r))
    shutil.rmtree(work)


def allreduce8(outdir):
    from algorithm import (BuffRef, Collective, FlagcxWorkflow, Param, Primitive, RedOp, Stage, add_opr, init_buffer,
                           set_pipeline, set_refresh, to_xml)
    with FlagcxWorkflow("allreduce8", Collective.AllReduce, [], [], 8):
        send, recv = {}, {}
        for rank in range(8):
            send[rank] = init_buffer(rank, 0, 8)
            recv[rank] = init_buffer(rank, 1, 8)
        set_pipeline(1, 0, 1, 1, 1)
        for rank in range(8):
            set_refresh(rank, 1, rank // 4 * 4, rank % 4, 1, 4, RedOp.sum)
        for cl in range(2):
            for h in range(4):
                rank = 4 * cl + h
                other = 4 * (1 - cl)
                mine = 4 * cl
                # pre: the cluster reduce-scatters both halves of the send buffer
                for half in (0, 4):
                    add_opr(rank_=rank, stage_=Stage.PreHomoFunc, step_=0,
                            params_={Param.send_buff: BuffRef(send[rank], half, 4),
                                     Param.recv_buff: BuffRef(recv[rank], half + h, 1),
                                     Param.count: 1, Param.homo_type: 0, Param.comm_op: Primitive.ReduceScatter})
                # hetero step 0: the partial sum of the other cluster's chunk goes over, one of ours comes in
                add_opr(rank_=rank, stage_=Stage.HeteroFunc, step_=0,
                        params_={Param.peer_or_root_rank: other + (h + 1) % 4, Param.send_offset: other + h,
                                 Param.recv_offset: -1, Param.count: 1})
                add_opr(rank_=rank, stage_=Stage.HeteroFunc, step_=0,
                        params_={Param.peer_or_root_rank: other + (h + 3) % 4, Param.send_offset: -1,
                                 Param.recv_offset: mine + (h + 3) % 4, Param.count: 1})
                # hetero step 1: the finished chunks are exchanged pairwise
                add_opr(rank_=rank, stage_=Stage.HeteroFunc, step_=1,
                        params_={Param.peer_or_root_rank: other + h, Param.send_offset: mine + h,
                                 Param.recv_offset: -1, Param.count: 1})
                add_opr(rank_=rank, stage_=Stage.HeteroFunc, step_=1,
                        params_={Param.peer_or_root_rank: other + h, Param.send_offset: -1,
                                 Param.recv_offset: other + h, Param.count: 1})
                # homo inter: own partial + the one received, scattered back to its owner
                add_opr(rank_=rank, stage_=Stage.HomoInterFunc, step_=0,
                        params_={Param.send_buff: BuffRef(recv[rank], mine, 1),
                                 Param.recv_buff: BuffRef(recv[rank], mine + h, 1),
                                 Param.count: 1, Param.homo_type: 2, Param.comm_op: Primitive.ReduceScatter})
                add_opr(rank_=rank, stage_=Stage.HomoInterFunc, step_=1, params_=None)
                # post: broadcast the cluster's own chunks, then the other cluster's
                for step, base in ((0, mine), (1, other)):
                    for root in range(4):
                        add_opr(rank_=rank, stage_=Stage.PostHomoFunc, step_=step,
                                params_={Param.peer_or_root_rank: root,
                                         Param.send_buff: BuffRef(recv[rank], base + root, 1),
                                         Param.recv_buff: BuffRef(recv[rank], base + root, 1),
                                         Param.count: 1, Param.homo_type: 2, Param.comm_op: Primitive.Broadcast})
        for rank in range(8):
            to_xml(rank_=rank, path_=outdir)


def allgather4(outdir):
    from algorithm import (BuffRef, Collective, FlagcxWorkflow, Param, Primitive, RedOp, Stage, add_opr, init_buffer,
                           set_pipeline, set_refresh, to_xml)
    with FlagcxWorkflow("allgather4", Collective.AllGather, [], [], 4):
        send, recv = {}, {}
        for rank in range(4):
            send[rank] = init_buffer(rank, 0, 1)
            recv[rank] = init_buffer(rank, 1, 4)
        set_pipeline(1, 0, 1, 0, 1)
        for rank in range(4):
            # flagcxC2cRefreshFunc(0, 0, totalCount_, redOp_) with redOp nop: nothing is cleared
            set_refresh(rank, -1, 0, 0, 0, 4, RedOp.nop)
        for cl in range(2):
            for h in range(2):
                rank, peer = 2 * cl + h, 2 * (1 - cl) + h
                # pre: all-gather inside the cluster, send[0] -> recv[clusterOffset + homo rank]
                add_opr(rank_=rank, stage_=Stage.PreHomoFunc, step_=0,
                        params_={Param.send_buff: BuffRef(send[rank], 0, 1), Param.recv_buff: BuffRef(recv[rank], 2 * cl, 1),
                                 Param.count: 1, Param.homo_type: 0, Param.comm_op: Primitive.AllGather})
                # hetero: own block, from offset 0 of the SEND buffer, to the rank of the same homo index
                add_opr(rank_=rank, stage_=Stage.HeteroFunc, step_=0,
                        params_={Param.peer_or_root_rank: peer, Param.send_offset: 0, Param.recv_offset: -1, Param.count: 1})
                add_opr(rank_=rank, stage_=Stage.HeteroFunc, step_=0,
                        params_={Param.peer_or_root_rank: peer, Param.send_offset: -1, Param.recv_offset: peer, Param.count: 1})
                add_opr(rank_=rank, stage_=Stage.HomoInterFunc, step_=0,
                        params_={Param.send_type: 0, Param.recv_type: 1, Param.send_offset: 0, Param.recv_offset: 0,
                                 Param.count: 4, Param.homo_type: 1, Param.comm_op: Primitive.Nop})
                # post: every inter-rank broadcasts the block it received
                for root in range(2):
                    blk = 2 * (1 - cl) + root
                    add_opr(rank_=rank, stage_=Stage.PostHomoFunc, step_=0,
                            params_={Param.peer_or_root_rank: root, Param.send_buff: BuffRef(recv[rank], blk, 1),
                                     Param.recv_buff: BuffRef(recv[rank], blk, 1), Param.count: 1, Param.homo_type: 2,
                                     Param.comm_op: Primitive.Broadcast})
        for rank in range(4):
            to_xml(rank_=rank, path_=outdir)


# sendCounts[r][i] in chunks: rank r sends that many chunks to rank i (ragged, one empty piece
# inside a cluster, one across); displacements pack the pieces in peer order
ALLTOALLV_UNITS = [[1, 2, 3, 0],
                   [0, 1, 1, 2],
                   [2, 0, 1, 3],
                   [1, 1, 2, 1]]


def alltoallv_layout(units=ALLTOALLV_UNITS):
    n = len(units)
    send = [list(row) for row in units]
    recv = [[units[r][i] for r in range(n)] for i in range(n)]
    sd = [[sum(send[r][:i]) for i in range(n)] for r in range(n)]
    rd = [[sum(recv[i][:r]) for r in range(n)] for i in range(n)]
    return send, sd, recv, rd


def alltoallv4(outdir):
    from algorithm import (BuffRef, Collective, FlagcxWorkflow, Param, Primitive, RedOp, Stage, add_opr, init_buffer,
                           set_pipeline, set_refresh, to_xml)
    send_c, sd, recv_c, rd = alltoallv_layout()
    with FlagcxWorkflow("alltoallv4", Collective.AlltoAllv, [], [], 4):
        send, recv = {}, {}
        for rank in range(4):
            send[rank] = init_buffer(rank, 0, 8)
            recv[rank] = init_buffer(rank, 1, 8)
        set_pipeline(1, 0, 1, 0, 1)
        for rank in range(4):
            set_refresh(rank, -1, 0, 0, 0, 8, RedOp.nop)
        for rank in range(4):
            cl = rank // 2
            # pre: AlltoAllv inside the cluster; offsets and count stay 0 (c2c_algo.cc:1554-1556)
            add_opr(rank_=rank, stage_=Stage.PreHomoFunc, step_=0,
                    params_={Param.send_buff: BuffRef(send[rank], 0, 0), Param.recv_buff: BuffRef(recv[rank], 0, 0),
                             Param.count: 0, Param.homo_type: 0, Param.comm_op: Primitive.AlltoAllv})
            # hetero: one send and one receive per rank of the other cluster that has something (c2c_algo.cc:1618-1630)
            for i in range(4):
                if i // 2 == cl:
                    continue
                if send_c[rank][i]:
                    add_opr(rank_=rank, stage_=Stage.HeteroFunc, step_=0,
                            params_={Param.peer_or_root_rank: i, Param.send_offset: sd[rank][i], Param.recv_offset: -1,
                                     Param.count: send_c[rank][i]})
                if recv_c[rank][i]:
                    add_opr(rank_=rank, stage_=Stage.HeteroFunc, step_=0,
                            params_={Param.peer_or_root_rank: i, Param.send_offset: -1, Param.recv_offset: rd[rank][i],
                                     Param.count: recv_c[rank][i]})
            add_opr(rank_=rank, stage_=Stage.HomoInterFunc, step_=0,
                    params_={Param.send_type: 0, Param.recv_type: 1, Param.send_offset: 0, Param.recv_offset: 0,
                             Param.count: 8, Param.homo_type: 1, Param.comm_op: Primitive.Nop})
            add_opr(rank_=rank, stage_=Stage.PostHomoFunc, step_=0,
                    params_={Param.send_type: 0, Param.recv_type: 1, Param.send_offset: 0, Param.recv_offset: 0,
                             Param.count: 8, Param.homo_type: 2, Param.comm_op: Primitive.Nop})
        for rank in range(4):
            to_xml(rank_=rank, path_=outdir)


def reducescatter8(outdir):
    from algorithm import (Collective, FlagcxWorkflow, Param, Primitive, RedOp, Stage, add_opr, set_pipeline,
                           set_refresh, to_xml)
    with FlagcxWorkflow("reducescatter8", Collective.ReduceScatter, [], [], 8):
        set_pipeline(1, 0, 1, 0, 1)
        for rank in range(8):
            cl, h = rank // 4, rank % 4
            other = 4 * (1 - cl)
            # the rank's buffer list starts with the quarter it forwards: [2h, 2h + 2) of 8 chunks
            set_refresh(rank, 2, 0, 2 * h, 2, 8, RedOp.sum)
            add_opr(rank_=rank, stage_=Stage.PreHomoFunc, step_=0,
                    params_={Param.send_type: 0, Param.recv_type: 2, Param.send_offset: 0, Param.recv_offset: 2 * h,
                             Param.count: 2, Param.homo_type: 0, Param.comm_op: Primitive.ReduceScatter})
            # inter-rank r1 of one cluster sends to inter-rank (r1 + 1) % 4 of the other, the first whose list is free there
            add_opr(rank_=rank, stage_=Stage.HeteroFunc, step_=0,
                    params_={Param.peer_or_root_rank: other + (h + 1) % 4, Param.send_offset: 2 * h, Param.recv_offset: -1,
                             Param.count: 2})
            add_opr(rank_=rank, stage_=Stage.HeteroFunc, step_=0,
                    params_={Param.peer_or_root_rank: other + (h + 3) % 4, Param.send_offset: -1,
                             Param.recv_offset: 2 * ((h + 3) % 4), Param.count: 2})
            add_opr(rank_=rank, stage_=Stage.HomoInterFunc, step_=0,
                    params_={Param.send_type: 2, Param.recv_type: 2, Param.send_offset: 0, Param.recv_offset: 0,
                             Param.count: 8, Param.homo_type: 1, Param.comm_op: Primitive.AllReduce})
            add_opr(rank_=rank, stage_=Stage.PostHomoFunc, step_=0,
                    params_={Param.send_type: 2, Param.recv_type: 1, Param.send_offset: 4 * cl, Param.recv_offset: 0,
                             Param.count: 1, Param.homo_type: 2, Param.comm_op: Primitive.ReduceScatter})
        for rank in range(8):
            to_xml(rank_=rank, path_=outdir)


def reduce8(outdir):
    from algorithm import (Collective, FlagcxWorkflow, Param, Primitive, RedOp, Stage, add_opr, set_pipeline,
                           set_refresh, to_xml)
    with FlagcxWorkflow("reduce8", Collective.Reduce, [], [], 8):
        set_pipeline(1, 0, 1, 0, 1)
        for rank in range(8):
            cl, h = rank // 4, rank % 4
            set_refresh(rank, 1, 0, h, 1, 4, RedOp.sum)
            add_opr(rank_=rank, stage_=Stage.PreHomoFunc, step_=0,
                    params_={Param.send_type: 0, Param.recv_type: 1, Param.send_offset: 0, Param.recv_offset: h,
                             Param.count: 1, Param.homo_type: 0, Param.comm_op: Primitive.ReduceScatter})
            if cl == 0:     # only the other cluster's quarters travel; the root cluster's are scheduled from the start
                add_opr(rank_=rank, stage_=Stage.HeteroFunc, step_=0,
                        params_={Param.peer_or_root_rank: 4 + (h + 1) % 4, Param.send_offset: h, Param.recv_offset: -1,
                                 Param.count: 1})
                add_opr(rank_=rank, stage_=Stage.HomoInterFunc, step_=0,
                        params_={Param.send_type: 1, Param.recv_type: 1, Param.send_offset: 0, Param.recv_offset: 0,
                                 Param.count: 4, Param.homo_type: 1, Param.comm_op: Primitive.Nop})
            else:
                add_opr(rank_=rank, stage_=Stage.HeteroFunc, step_=0,
                        params_={Param.peer_or_root_rank: (h + 3) % 4, Param.send_offset: -1, Param.recv_offset: (h + 3) % 4,
                                 Param.count: 1})
                add_opr(rank_=rank, stage_=Stage.HomoInterFunc, step_=0,
                        params_={Param.send_type: 1, Param.recv_type: 1, Param.send_offset: 0, Param.recv_offset: 0,
                                 Param.count: 4, Param.homo_type: 0, Param.comm_op: Primitive.Reduce})
            add_opr(rank_=rank, stage_=Stage.PostHomoFunc, step_=0, params_=None)
        for rank in range(8):
            to_xml(rank_=rank, path_=outdir)


def gather4(outdir, root=3):
    from algorithm import (Collective, FlagcxWorkflow, Param, Primitive, RedOp, Stage, add_opr, set_pipeline,
                           set_refresh, to_xml)
    SEND, RECV = Primitive.P2P, Primitive.Custom     # the values 0 and 1: flagcxCommOpSend, flagcxCommOpRecv
    with FlagcxWorkflow("gather4", Collective.Gather, [], [], 4):
        set_pipeline(1, 0, 1, 0, 1)
        for rank in range(4):
            cl, h = rank // 2, rank % 2
            typ = 1 if rank == root else 2          # recvType = sendType: scratch everywhere but on the root
            set_refresh(rank, typ, 0, 2 * cl + h, 1, 4, RedOp.nop)
            add_opr(rank_=rank, stage_=Stage.PreHomoFunc, step_=0,
                    params_={Param.send_type: 0, Param.recv_type: typ, Param.send_offset: 0, Param.recv_offset: 2 * cl,
                             Param.count: 1, Param.homo_type: 0, Param.comm_op: Primitive.AllGather})
            if cl == 0:
                add_opr(rank_=rank, stage_=Stage.HeteroFunc, step_=0,
                        params_={Param.peer_or_root_rank: 2 + h, Param.send_offset: h, Param.recv_offset: -1, Param.count: 1})
                add_opr(rank_=rank, stage_=Stage.HomoInterFunc, step_=0,
                        params_={Param.send_type: typ, Param.recv_type: typ, Param.send_offset: 0, Param.recv_offset: 0,
                                 Param.count: 4, Param.homo_type: 1, Param.comm_op: Primitive.Nop})
                add_opr(rank_=rank, stage_=Stage.PostHomoFunc, step_=0, params_=None)
            else:
                add_opr(rank_=rank, stage_=Stage.HeteroFunc, step_=0,
                        params_={Param.peer_or_root_rank: h, Param.send_offset: -1, Param.recv_offset: h, Param.count: 1})
                # inter-rank 0 of the root cluster collects what the other inter-ranks received, then hands all to the root
                add_opr(rank_=rank, stage_=Stage.HomoInterFunc, step_=0,
                        params_={Param.send_type: typ, Param.recv_type: typ, Param.send_offset: 0, Param.recv_offset: 0,
                                 Param.count: 4, Param.homo_type: 1, Param.comm_op: RECV if h == 0 else SEND})
                add_opr(rank_=rank, stage_=Stage.PostHomoFunc, step_=0,
                        params_={Param.peer_or_root_rank: root - 2, Param.send_type: typ, Param.recv_type: 1,
                                 Param.send_offset: 0, Param.recv_offset: 0, Param.count: 4, Param.homo_type: 2,
                                 Param.comm_op: RECV if rank == root else SEND})
        for rank in range(4):
            to_xml(rank_=rank, path_=outdir)


def uneven4(outdir):
    from algorithm import (Collective, FlagcxWorkflow, Param, Primitive, RedOp, Stage, add_opr, set_pipeline,
                           set_refresh, to_xml)
    with FlagcxWorkflow("uneven4", Collective.AllReduce, [], [], 4):
        set_pipeline(1, 0, 1, 0, 1)
        for rank in range(4):
            cl, h = rank // 2, rank % 2
            set_refresh(rank, 1, 0, 2 * h, 2, 4, RedOp.sum)
            # the cluster's partial sum of half h lands at its own place
            add_opr(rank_=rank, stage_=Stage.PreHomoFunc, step_=0,
                    params_={Param.send_type: 0, Param.recv_type: 1, Param.send_offset: 0, Param.recv_offset: 2 * h,
                             Param.count: 2, Param.homo_type: 0, Param.comm_op: Primitive.ReduceScatter})
            # function 0: the halves cross over to the other cluster's rank that does not own them
            peer = 2 * (1 - cl) + (1 - h)
            add_opr(rank_=rank, stage_=Stage.HeteroFunc, step_=0,
                    params_={Param.peer_or_root_rank: peer, Param.send_offset: 2 * h, Param.recv_offset: -1, Param.count: 2})
            add_opr(rank_=rank, stage_=Stage.HeteroFunc, step_=0,
                    params_={Param.peer_or_root_rank: peer, Param.send_offset: -1, Param.recv_offset: 2 * (1 - h), Param.count: 2})
            add_opr(rank_=rank, stage_=Stage.HomoInterFunc, step_=0,
                    params_={Param.send_type: 1, Param.recv_type: 1, Param.send_offset: 0, Param.recv_offset: 0,
                             Param.count: 4, Param.homo_type: 1, Param.comm_op: Primitive.AllReduce})
            if h == 0:
                # function 1, on ranks 0 and 2 only: they swap their first halves into each other's second half
                add_opr(rank_=rank, stage_=Stage.HeteroFunc, step_=0,
                        params_={Param.peer_or_root_rank: 2 - rank, Param.send_offset: 0, Param.recv_offset: -1, Param.count: 2,
                                 Param.sub_step: 1})
                add_opr(rank_=rank, stage_=Stage.HeteroFunc, step_=0,
                        params_={Param.peer_or_root_rank: 2 - rank, Param.send_offset: -1, Param.recv_offset: 2, Param.count: 2,
                                 Param.sub_step: 1})
            if cl == 0:
                add_opr(rank_=rank, stage_=Stage.PostHomoFunc, step_=0,
                        params_={Param.peer_or_root_rank: 1, Param.send_type: 1, Param.recv_type: 1, Param.send_offset: 0,
                                 Param.recv_offset: 0, Param.count: 4, Param.homo_type: 2, Param.comm_op: Primitive.Broadcast})
            else:
                add_opr(rank_=rank, stage_=Stage.PostHomoFunc, step_=0, params_=None)
        for rank in range(4):
            to_xml(rank_=rank, path_=outdir)


def main():
    if not os.path.isdir(TOOLS):
        sys.exit("reference tree not found at %s" % REF)
    sys.path.insert(0, TOOLS)
    os.makedirs(OUT, exist_ok=True)
    reference_example(OUT)
    allreduce8(OUT)
    allgather4(OUT)
    alltoallv4(OUT)
    reducescatter8(OUT)
    reduce8(OUT)
    gather4(OUT)
    uneven4(OUT)
    print("wrote", sorted(os.listdir(OUT)))


if __name__ == "__main__":
    main()
