"""CPU restatement of how the reference replays C2C plans, for ALL ranks at once.

TEST INFRASTRUCTURE ONLY: the checker of flagcxLocalPlanExecute.  Imported by
tests/ only; the product package never imports this module.

What it follows (paths relative to the reference tree):
  - plan documents: flagcx/core/c2c_algo.cc:973-1048 (importXml), serializers in
    flagcx/core/c2c_ir.h:62-176; documents written by flagcx/tools/algorithm.py
    carry no <nChunks>, the caller then says how many chunks the collective has;
  - stage order and refresh placement: flagcxC2cPlanner::execute,
    flagcx/core/c2c_algo.cc:2121-2298;
  - homo functions: flagcxC2cHomoFunc::run, c2c_algo.cc:286-511, with the vendor
    collective replaced by its definition on numpy arrays (members folded in
    communicator-rank order 0..n-1: acc = s_0, acc = OP(s_j, acc));
  - hetero functions: flagcxC2cHeteroFunc::run / flagcxC2cP2pOp::run,
    c2c_algo.cc:219-236,565-584: a send is matched with the peer's next receive
    from that sender;
  - refresh: flagcxC2cRefreshFunc::run, c2c_algo.cc:586-608;
  - eachNicPerRank_ / multiNic_: the planner's constructor, c2c_algo.cc:636-672.

Pinning: the all-reduce / all-gather closed forms the plans under
tests/golden/plans must produce (every rank ends with the fold, or the
concatenation, of all ranks' inputs) fail if a stage is out of order, a refresh is
misplaced, or an offset is read in the wrong unit; fold order inside the vendor
collectives of the reference is parity unpinned (un-vendored dependency).
"""
import xml.etree.ElementTree as ET

import numpy as np

# flagcxCommOp_t, flagcx/include/flagcx.h:78-88 (+ the DSL's LocCpy / LocRed, flagcx/tools/utils.py:43-44)
SEND, RECV, BROADCAST, GATHER, SCATTER, REDUCE, ALLREDUCE, ALLGATHER, REDUCESCATTER, ALLTOALL, ALLTOALLV, NOOP = range(12)
LOCCPY, LOCRED = 12, 13
SUM, PROD, MAX, MIN = 0, 1, 2, 3
ALGO_SEQUENTIAL, ALGO_PIPELINE, ALGO_INPUT = 0, 1, 2


class Homo:
    def __init__(self, node, cs):
        g = lambda t, d=0: int(node.findtext(t, str(d)))
        self.root = g("rootRank", -1)
        self.send_type, self.recv_type = g("sendType"), g("recvType")
        self.send_off, self.recv_off, self.count = g("sendOffset") * cs, g("recvOffset") * cs, g("count") * cs
        self.homo_type, self.op = g("homoType"), g("commOp")


class P2p:
    def __init__(self, node, cs):
        g = lambda t: int(node.findtext(t, "0"))
        self.rank, self.peer, self.off, self.count, self.is_recv = g("rank"), g("peerRank"), g("offset") * cs, g("count") * cs, g("isRecv")


class RankPlan:
    def __init__(self, path, total_count, default_chunks=None):
        root = ET.parse(path).getroot()
        assert root.tag == "FlagcxC2cPlanner"
        nchunks = root.findtext("nChunks")
        self.nchunks = int(nchunks) if nchunks is not None else default_chunks
        assert self.nchunks and total_count % self.nchunks == 0
        cs = total_count // self.nchunks
        g = lambda t: int(root.findtext(t, "0"))
        self.n_seq_pre, self.n_pipe_pre, self.n_seq_inter = g("nSeqPreSteps"), g("nPipePreSteps"), g("nSeqInterSteps")
        self.n_pipe_post, self.n_seq_post = g("nPipePostSteps"), g("nSeqPostSteps")
        rf = root.find("RefreshFunc")
        r = lambda t, d=0: int(rf.findtext(t, str(d))) if rf is not None else d
        self.rf_type, self.rf_start, self.rf_off = r("buffType", -1), r("start") * cs, r("offset") * cs
        self.rf_count, self.rf_total, self.rf_op = r("count") * cs, r("totalCount") * cs, r("redOp")

        def homo(tag):
            t = root.find(tag)
            return [[Homo(f, cs) for f in step.findall("HomoFunc")] for step in t.findall("Step")] if t is not None else []
        self.pre, self.inter, self.post = homo("PreHomoFuncSteps"), homo("HomoInterFuncSteps"), homo("PostHomoFuncSteps")
        t = root.find("HeteroFuncSteps")
        self.hetero = [[[P2p(o, cs) for o in f.findall("P2pOp")] for f in step.findall("HeteroFunc")]
                       for step in t.findall("Step")] if t is not None else []
        while len(self.inter) < len(self.hetero):
            self.inter.append([])


def _fold(arrs, op):
    acc = arrs[0].copy()
    for a in arrs[1:]:
        if op == SUM:
            acc = a + acc
        elif op == MAX:
            acc = np.where(a < acc, acc, a)      # std::max(a, acc)
        elif op == MIN:
            acc = np.where(acc < a, acc, a)      # std::min(a, acc)
        else:
            raise ValueError(op)
    return acc


class Model:
    """send / recv / scratch: lists of 1-D numpy arrays per rank (scratch entries may be None)."""

    def __init__(self, prefix, cluster_ids, total_count, comm_op, red_op, is_inter=None, default_chunks=None):
        self.n = len(cluster_ids)
        self.cluster_of = list(cluster_ids)
        self.is_inter = [1] * self.n if is_inter is None else [int(bool(x)) for x in is_inter]
        ncl = max(cluster_ids) + 1
        self.members = [[r for r in range(self.n) if cluster_ids[r] == c] for c in range(ncl)]
        self.inters = [[r for r in m if self.is_inter[r]] for m in self.members]
        self.total, self.comm_op, self.red_op = total_count, comm_op, red_op
        self.plans = [RankPlan("%s_%d.xml" % (prefix, r), total_count, default_chunks) for r in range(self.n)]
        self.algorithm = ALGO_INPUT
        # c2c_algo.cc:636-672
        if comm_op in (ALLREDUCE, REDUCESCATTER, REDUCE):
            self.multi_nic = int(all(len(i) != 1 for i in self.inters))
        else:
            self.multi_nic = int(any(len(i) != 1 for i in self.inters))
        if any(len(i) > total_count for i in self.inters):
            self.multi_nic = 0
        self.each_nic_per_rank = int(all(len(i) == len(m) for i, m in zip(self.inters, self.members)))

    # -- buffers
    def _buf(self, r, typ):
        return self.send[r] if typ == 0 else self.recv[r] if typ == 1 else self.scratch[r]

    def _homo_rank(self, r):
        return self.members[self.cluster_of[r]].index(r)

    def _refresh(self, only=None):
        for r, p in enumerate(self.plans):
            if only is not None and r not in only:
                continue
            typ = p.rf_type
            start = p.rf_start
            if typ == -1:                                    # c2c_algo.cc:2156-2164
                typ = 2 if self.owns_scratch[r] else 1
                if self.comm_op in (REDUCESCATTER, ALLREDUCE) and self.algorithm == ALGO_PIPELINE:
                    cl = self.cluster_of[r]
                    start = sum(len(self.members[c]) for c in range(cl)) * self.total // self.n
            if p.rf_op != SUM or p.rf_total == 0:
                continue
            b = self.recv[r] if typ == 1 else self.scratch[r]
            b[start:start + p.rf_off] = 0
            b[start + p.rf_off + p.rf_count:start + p.rf_total] = 0

    def _homo(self, table, s, i, root, only=None):
        """Function i of step s of one table on every rank that has it (only: and is in that set)."""
        fn = {}
        for r, p in enumerate(self.plans):
            t = getattr(p, table)
            if only is not None and r not in only:
                continue
            if s < len(t) and i < len(t[s]):
                f = t[s][i]
                if f.homo_type == 1 and not self.is_inter[r]:
                    continue                                 # c2c_algo.cc:293-295
                fn[r] = f
        writes = []                                          # (array, offset, values): applied after all reads
        for cl, members in enumerate(self.members):
            have = [r for r in members if r in fn]
            if not have:
                continue
            f0 = fn[have[0]]
            op = f0.op
            if op == NOOP:
                continue
            if op in (LOCCPY, LOCRED):
                for r in have:
                    f = fn[r]
                    s_ = self._buf(r, f.send_type)[f.send_off:f.send_off + f.count]
                    d = self._buf(r, 1 if f.recv_type == 1 else 2)
                    v = s_.copy() if op == LOCCPY else _fold([d[f.recv_off:f.recv_off + f.count], s_], self.red_op)
                    writes.append((d, f.recv_off, v))
                continue
            comm = self.inters[cl] if f0.homo_type == 1 else members
            homo_root = lambda f: f.root if f.root != -1 else root
            if op in (SEND, RECV):
                writes += self._send_recv(cl, fn, root)
                continue
            if op == ALLTOALLV:                              # c2c_algo.cc:482-508: peers of the own cluster only
                sc, sd, rc, rd = self.v_args
                for r in have:
                    for i in members:
                        cnt = sc[r][i]
                        assert cnt == (rc[i][r] if i in fn else 0), "unmatched AlltoAllv piece %d -> %d" % (r, i)
                        if cnt:
                            src = self._buf(r, fn[r].send_type)
                            dst = self._buf(i, 1 if fn[i].recv_type == 1 else 2)
                            writes.append((dst, rd[i][r], src[sd[r][i]:sd[r][i] + cnt].copy()))
                continue
            S = [self._buf(r, fn[r].send_type) for r in comm]
            D = [self._buf(r, 1 if fn[r].recv_type == 1 else 2) for r in comm]
            so, ro = [fn[r].send_off for r in comm], [fn[r].recv_off for r in comm]
            c = f0.count
            n = len(comm)
            if op == REDUCE:
                rt = homo_root(f0)
                writes.append((D[rt], ro[rt], _fold([S[j][so[j]:so[j] + c] for j in range(n)], self.red_op)))
            elif op == ALLREDUCE:
                v = _fold([S[j][so[j]:so[j] + c] for j in range(n)], self.red_op)
                writes += [(D[h], ro[h], v) for h in range(n)]
            elif op == REDUCESCATTER:
                for h in range(n):
                    writes.append((D[h], ro[h], _fold([S[j][so[j] + h * c:so[j] + (h + 1) * c] for j in range(n)], self.red_op)))
            elif op == ALLGATHER:
                for h in range(n):
                    writes += [(D[h], ro[h] + j * c, S[j][so[j]:so[j] + c].copy()) for j in range(n)]
            elif op == GATHER:
                rt = homo_root(f0)
                writes += [(D[rt], ro[rt] + j * c, S[j][so[j]:so[j] + c].copy()) for j in range(n)]
            elif op == SCATTER:
                rt = homo_root(f0)
                writes += [(D[h], ro[h], S[rt][so[rt] + h * c:so[rt] + (h + 1) * c].copy()) for h in range(n)]
            elif op == BROADCAST:
                rt = homo_root(f0)
                writes += [(D[h], ro[h], S[rt][so[rt]:so[rt] + c].copy()) for h in range(n)]
            elif op == ALLTOALL:
                for h in range(n):
                    writes += [(D[h], ro[h] + j * c, S[j][so[j] + h * c:so[j] + (h + 1) * c].copy()) for j in range(n)]
            else:
                raise NotImplementedError(op)
        for arr, off, v in writes:
            arr[off:off + len(v)] = v

    def _send_recv(self, cl, fn, root):
        """Send / Recv homo functions, c2c_algo.cc:364-463: homoType 0 root -> inter-ranks,
        1 inter-ranks i > 0 -> inter-rank 0 (what each received from other clusters),
        2 inter-rank 0 -> root.  Roots are homo ranks."""
        members, inters = self.members[cl], self.inters[cl]
        out = []
        for r in members:
            f = fn.get(r)
            if f is None or f.op != SEND:
                continue
            rt = f.root if f.root != -1 else root
            src = self._buf(r, f.send_type)
            if f.homo_type == 0 and self._homo_rank(r) == rt:
                for peer in inters:
                    g = fn.get(peer)
                    if peer != r and g is not None and g.op == RECV and self._homo_rank(peer) != rt:
                        out.append((self._buf(peer, 1 if g.recv_type == 1 else 2), g.recv_off,
                                    src[f.send_off:f.send_off + f.count].copy()))
            elif f.homo_type == 1 and self.is_inter[r] and inters.index(r) > 0:
                g = fn.get(inters[0])
                if g is not None and g.op == RECV:
                    dst = self._buf(inters[0], 1 if g.recv_type == 1 else 2)
                    for off, cnt in self._received(r):
                        out.append((dst, off, src[off:off + cnt].copy()))
            elif f.homo_type == 2 and self.is_inter[r] and inters.index(r) == 0 and self._homo_rank(r) != rt:
                peer = members[rt]
                g = fn.get(peer)
                if g is not None and g.op == RECV:
                    out.append((self._buf(peer, 1 if g.recv_type == 1 else 2), g.recv_off,
                                src[f.send_off:f.send_off + f.count].copy()))
        return out

    def _received(self, r):
        """(offset, count) of every receive of rank r in its hetero functions: the isRecv_
        entries of the planner's inter-rank buffer list (c2c_algo.cc:386-400,434-452)."""
        seen, out = set(), []
        for step in self.plans[r].hetero:
            for f in step:
                for o in f:
                    if o.is_recv and (o.off, o.count) not in seen:
                        seen.add((o.off, o.count))
                        out.append((o.off, o.count))
        return out

    def _hetero(self, s, i, send_tmp, recv_tmp):
        recvs, used, writes = {}, {}, []
        for r, p in enumerate(self.plans):
            if s < len(p.hetero) and i < len(p.hetero[s]):
                for o in p.hetero[s][i]:
                    if o.is_recv:
                        recvs.setdefault((r, o.peer), []).append(o)
        for r, p in enumerate(self.plans):
            if s < len(p.hetero) and i < len(p.hetero[s]):
                for o in p.hetero[s][i]:
                    if o.is_recv:
                        continue
                    key = (o.peer, r)
                    u = used.get(key, 0)
                    rv = recvs[key][u]
                    used[key] = u + 1
                    assert rv.count == o.count
                    writes.append((recv_tmp[o.peer], rv.off, send_tmp[r][o.off:o.off + o.count].copy()))
        for arr, off, v in writes:
            arr[off:off + len(v)] = v

    def _has(self, table, s, i):
        """Ranks whose own table holds a function i in step s (the reference's
        `homoInterFuncSteps_[s].size() > i` is evaluated by every rank for itself)."""
        return {r for r, p in enumerate(self.plans) if s < len(getattr(p, table)) and i < len(getattr(p, table)[s])}

    def _width(self, table, s):
        return max((len(getattr(p, table)[s]) if s < len(getattr(p, table)) else 0) for p in self.plans)

    def execute(self, send, recv, scratch, root=-1, algorithm=ALGO_INPUT, v_args=None):
        """flagcxC2cPlanner::execute, c2c_algo.cc:2121-2298; buffers are modified in place.
        v_args: (sendCounts, sDispls, recvCounts, rDispls) of an AlltoAllv, row r = rank r's arrays.
        Every rank walks its own tables: it runs hetero function i of a step while i is below the
        length of ITS hetero table for that step, homoInter function i behind it if its own table
        holds one, and refreshes where its own loop stands (c2c_algo.cc:2177-2194,2204-2231,
        2247-2267,2276-2288)."""
        self.v_args = v_args
        self.send, self.recv = send, recv
        self.scratch = scratch if scratch is not None else [None] * self.n
        self.algorithm = algorithm
        homo_root = self._homo_rank(root) if 0 <= root < self.n else root     # globalrank2homorank[root]
        # the ranks the reference gives a scratch buffer for the call (c2c_algo.cc:2121-2129); hetero
        # receives land there, and in recvbuff on every other rank (c2c_algo.cc:2131)
        self.owns_scratch = [self.comm_op in (REDUCESCATTER, SCATTER) or (self.comm_op == GATHER and r != root)
                             for r in range(self.n)]
        recv_tmp = [self.scratch[r] if self.owns_scratch[r] else self.recv[r] for r in range(self.n)]
        send_tmp = []
        for r in range(self.n):
            from_send = self.comm_op in (ALLTOALL, ALLTOALLV) or (self.comm_op == SCATTER and r == root) or \
                (self.comm_op == ALLGATHER and self.each_nic_per_rank and self.multi_nic)
            send_tmp.append(self.send[r] if from_send else recv_tmp[r])
        c = self.plans[0]
        any_pipe = c.n_pipe_pre > 0 or c.n_pipe_post > 0
        for s in range(c.n_seq_pre):
            for i in range(self._width("pre", s)):
                self._homo("pre", s, i, homo_root)
        self._refresh()
        for s in range(c.n_pipe_pre):
            for i in range(self._width("pre", c.n_seq_pre + s)):
                self._homo("pre", c.n_seq_pre + s, i, homo_root)
            for i in range(self._width("hetero", s)):
                self._hetero(s, i, send_tmp, recv_tmp)
                has = self._has("hetero", s, i) & self._has("inter", s, i)
                if has:
                    self._homo("inter", s, i, homo_root, has)
                    self._refresh(has)
        for s in range(c.n_seq_inter):
            hs = c.n_pipe_pre + s
            for i in range(self._width("hetero", hs)):
                at = self._has("hetero", hs, i)
                if algorithm == ALGO_SEQUENTIAL or not any_pipe:
                    self._refresh(at)
                self._hetero(hs, i, send_tmp, recv_tmp)
                has = at & self._has("inter", hs, i)
                if has:
                    self._homo("inter", hs, i, homo_root, has)
                    if algorithm == ALGO_PIPELINE and any_pipe:
                        self._refresh(has)
        for s in range(c.n_pipe_post):
            for i in range(self._width("post", s)):
                self._homo("post", s, i, homo_root)
            hs = c.n_pipe_pre + c.n_seq_inter + s
            for i in range(self._width("hetero", hs)):
                self._hetero(hs, i, send_tmp, recv_tmp)
                has = self._has("hetero", hs, i) & self._has("inter", hs, i)
                if has:
                    self._homo("inter", hs, i, homo_root, has)
        for s in range(c.n_seq_post):
            for i in range(self._width("post", c.n_pipe_post + s)):
                if algorithm == ALGO_SEQUENTIAL or not any_pipe:
                    self._refresh(self._has("post", c.n_pipe_post + s, i))
                self._homo("post", c.n_pipe_post + s, i, homo_root)
