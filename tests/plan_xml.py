"""Writes per-rank C2C plan files in the XML layout of the reference's exportXml
(flagcx/core/c2c_algo.cc:1050-1087; element serializers flagcx/core/c2c_ir.h:62-144):
one <prefix>_<rank>.xml per rank.  Offsets and counts are in chunks."""


def homo(commOp, sendType, recvType, sendOffset, recvOffset, count, homoType, rootRank=-1):
    return dict(rootRank=rootRank, sendType=sendType, recvType=recvType, sendOffset=sendOffset,
                recvOffset=recvOffset, count=count, homoType=homoType, commOp=commOp)


def p2p(rank, peerRank, offset, count, isRecv):
    return dict(rank=rank, peerRank=peerRank, offset=offset, count=count, isRecv=isRecv)


def _homo_steps(tag, steps):
    out = ["  <%s>" % tag]
    for step in steps:
        if not step:
            out.append("    <Step/>")
            continue
        out.append("    <Step>")
        for h in step:
            out.append("      <HomoFunc>")
            for k in ("rootRank", "sendType", "recvType", "sendOffset", "recvOffset", "count", "homoType", "commOp"):
                out.append("        <%s>%d</%s>" % (k, h[k], k))
            out.append("      </HomoFunc>")
        out.append("    </Step>")
    out.append("  </%s>" % tag)
    return out


def write_rank(prefix, rank, nchunks, steps, refresh, pre, hetero, inter, post):
    """steps = (nSeqPre, nPipePre, nSeqInter, nPipePost, nSeqPost); refresh = dict(buffType,start,offset,count,
    totalCount,redOp); pre/inter/post = list of steps of homo funcs; hetero = list of steps of lists of p2p lists."""
    out = ["<FlagcxC2cPlanner>", "  <nChunks>%d</nChunks>" % nchunks]
    for k, v in zip(("nSeqPreSteps", "nPipePreSteps", "nSeqInterSteps", "nPipePostSteps", "nSeqPostSteps"), steps):
        out.append("  <%s>%d</%s>" % (k, v, k))
    out.append("  <RefreshFunc>")
    for k in ("buffType", "start", "offset", "count", "totalCount", "redOp"):
        out.append("    <%s>%d</%s>" % (k, refresh[k], k))
    out.append("  </RefreshFunc>")
    out += _homo_steps("PreHomoFuncSteps", pre)
    out.append("  <HeteroFuncSteps>")
    for step in hetero:
        if not step:
            out.append("    <Step/>")
            continue
        out.append("    <Step>")
        for func in step:
            out.append("      <HeteroFunc>")
            for op in func:
                out.append("        <P2pOp>")
                for k in ("rank", "peerRank", "offset", "count", "isRecv"):
                    out.append("          <%s>%d</%s>" % (k, op[k], k))
                out.append("        </P2pOp>")
            out.append("      </HeteroFunc>")
        out.append("    </Step>")
    out.append("  </HeteroFuncSteps>")
    out += _homo_steps("HomoInterFuncSteps", inter)
    out += _homo_steps("PostHomoFuncSteps", post)
    out.append("</FlagcxC2cPlanner>")
    with open("%s_%d.xml" % (prefix, rank), "w") as f:
        f.write("\n".join(out) + "\n")


NO_REFRESH = dict(buffType=1, start=0, offset=0, count=0, totalCount=0, redOp=0)

# flagcxCommOp_t values (flagcx/include/flagcx.h:62-76) and the two reserved local primitives
BROADCAST, GATHER, SCATTER, REDUCE, ALLREDUCE, ALLGATHER, REDUCESCATTER, ALLTOALL = 2, 3, 4, 5, 6, 7, 8, 9
LOCCPY, LOCRED = 12, 13


def allreduce_2x2_locred(prefix):
    """Plan A: 2 clusters x 2 ranks, 4 chunks.  intra-cluster reduce-scatter, exchange of
    the owned half with the partner cluster, rank-local reduce, intra-cluster all-gather."""
    for r in range(4):
        h, partner = r % 2, (r + 2) % 4
        pre = [[homo(REDUCESCATTER, 0, 1, 0, 2 * h, 2, 0)]]
        het = [[[p2p(r, partner, 2 * h, 2, 0), p2p(r, partner, 2 * (1 - h), 2, 1)]]]
        inter = [[homo(LOCRED, 1, 1, 2 * (1 - h), 2 * h, 2, 1)]]
        post = [[homo(ALLGATHER, 1, 1, 2 * h, 0, 2, 2)]]
        write_rank(prefix, r, 4, (1, 0, 1, 0, 1), NO_REFRESH, pre, het, inter, post)


def allreduce_2x2_refresh_scratch(prefix):
    """Plan B: cluster sums into scratch, exchange halves, rank-local reduce, then the
    reference's assembly idiom: zero everything but the own half (refresh) and
    all-reduce the cluster's scratch buffers into recv."""
    for r in range(4):
        h, partner = r % 2, (r + 2) % 4
        refresh = dict(buffType=2, start=0, offset=2 * h, count=2, totalCount=4, redOp=0)
        pre = [[homo(ALLREDUCE, 0, 2, 0, 0, 4, 0)]]
        het = [[[p2p(r, partner, 2 * h, 2, 0), p2p(r, partner, 2 * (1 - h), 2, 1)]]]
        inter = [[homo(LOCRED, 2, 2, 2 * (1 - h), 2 * h, 2, 1)]]
        post = [[homo(ALLREDUCE, 2, 1, 0, 0, 4, 2)]]
        write_rank(prefix, r, 4, (1, 0, 1, 0, 1), refresh, pre, het, inter, post)


def allreduce_2x2_reference_ops_only(prefix):
    """Plan C: only primitives the reference executes.  Cluster sums everywhere; homo
    rank 1 of each cluster zeroes its buffer (refresh with count 0) and receives the
    other cluster's sum; an inter-rank all-reduce then gives the total on all ranks."""
    for r in range(4):
        h = r % 2
        refresh = dict(buffType=1, start=0, offset=0, count=4 if h == 0 else 0, totalCount=4, redOp=0)
        pre = [[homo(ALLREDUCE, 0, 1, 0, 0, 4, 0)]]
        # rank 0 -> rank 3, rank 2 -> rank 1
        if h == 0:
            het = [[[p2p(r, (r + 3) % 4, 0, 4, 0)]]]
        else:
            het = [[[p2p(r, (r + 1) % 4, 0, 4, 1)]]]
        inter = [[homo(ALLREDUCE, 1, 1, 0, 0, 4, 1)]]
        write_rank(prefix, r, 4, (1, 0, 1, 0, 0), refresh, pre, het, inter, [])


def one_cluster_collective(prefix, commop, nranks=4, root=2):
    """One cluster of `nranks`, one homo step from the user send buffer (type 0) into recv
    (type 1): all-gather / gather of one chunk per rank, or all-to-all of one chunk per pair.
    nChunks = nranks, so a chunk is totalCount / nranks elements."""
    for r in range(nranks):
        pre = [[homo(commop, 0, 1, 0, 0, 1, 0, rootRank=root if commop in (GATHER, REDUCE) else -1)]]
        write_rank(prefix, r, nranks, (1, 0, 0, 0, 0), NO_REFRESH, pre, [], [], [])
