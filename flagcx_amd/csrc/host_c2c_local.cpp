// host_c2c_local.cpp - replays C2C plans on ONE GPU that holds the buffers of all
// simulated ranks, using only the library's own C ABI (flagcxLocalReduce*,
// flagcxLocalMemcpy, flagcxLocalRefresh).
//
// A plan is what flagcxC2cPlanner keeps per rank (flagcx/core/c2c_algo.h:205-268):
// step counts, one refresh function and four step tables of homo / hetero
// functions, in the XML format its exportXml / importXml use
// (flagcx/core/c2c_algo.cc:973-1087, serializers in flagcx/core/c2c_ir.h:62-176).
// The field names below are the reference's.  Execution follows
// flagcxC2cPlanner::execute (c2c_algo.cc:2142-2290) stage by stage, with all
// ranks advanced in lock step:
//   - a homo function is the same collective on every member of a cluster
//     (homoType 1: on the cluster's inter-ranks only, c2c_algo.cc:293-295); where
//     the reference calls the vendor CCL (c2c_algo.cc:309-481) the members'
//     buffers are reduced / copied by the local kernels, folding in homo-rank
//     order 0..n-1;
//   - a hetero function's P2P ops (c2c_algo.cc:565-584) are matched send-to-recv
//     between ranks and become device copies;
//   - the refresh function is flagcxLocalRefresh (c2c_algo.cc:586-608).
// Two rank-local primitives the reference's plan DSL reserves but its executor
// lacks (LocCpy = 12, LocRed = 13, flagcx/tools/utils.py:43-44) are accepted as
// commOp values: LocCpy copies send[sendOffset..) to recv[recvOffset..); LocRed
// sets recv[recvOffset..) = OP(send[sendOffset..), recv[recvOffset..)).
//
// Send / Recv homo functions (c2c_algo.cc:364-463) are replayed for all three
// homoTypes; for homoType 1 the planner's inter-rank buffer list, which the plan
// document does not carry, is rebuilt from the rank's hetero receives (the list's
// isRecv_ entries are exactly those, c2c_algo.cc:386-400,434-452).
// AlltoAllv takes its counts and displacements, which are arguments of execute() and not
// part of a plan (c2c_algo.cc:2042-2046), from flagcxLocalPlanSetAlltoAllv.
//
// Two ways to replay, with the same bytes in every receive buffer at the end:
//   - literal: every refresh is a zero-fill and every reduce-type homo function reads all
//     of its members' buffers, zeros included, as the reference does;
//   - fused (the default): a refresh only records the ranges it would clear, and a sum
//     reads the members whose slices hold data (ZeroSet below).  The assembly idiom
//     "clear everything but the own slice, then all-reduce the buffers"
//     (c2c_algo.cc:586-608 + 310-336) then moves the live slices only.
#include "../../include/flagcx_amd.h"

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <iterator>
#include <map>
#include <new>
#include <string>
#include <utility>
#include <vector>

namespace {

enum { kLocCpy = 12, kLocRed = 13 };

struct HomoFunc {
  int rootRank_ = -1, sendType_ = 0, recvType_ = 1;
  size_t sendOffset_ = 0, recvOffset_ = 0, count_ = 0;
  int homoType_ = 0;
  int commOp_ = flagcxCommNoOp;
};
struct P2pOp {
  int rank_ = 0, peerRank_ = 0;
  size_t offset_ = 0, count_ = 0;
  int isRecv_ = 0;
};
struct HeteroFunc {
  std::vector<P2pOp> p2pOps_;
};
struct RefreshFunc {
  int bufftype_ = -1;
  size_t start_ = 0, offset_ = 0, count_ = 0, totalCount_ = 0;
  int redOp_ = flagcxSum;
};
struct RankPlan {
  size_t nchunks_ = 1;
  int nSeqPreSteps_ = 0, nPipePreSteps_ = 0, nSeqInterSteps_ = 0, nPipePostSteps_ = 0, nSeqPostSteps_ = 0;
  RefreshFunc refreshFunc_;
  std::vector<std::vector<HomoFunc>> preHomoFuncSteps_, homoInterFuncSteps_, postHomoFuncSteps_;
  std::vector<std::vector<HeteroFunc>> heteroFuncSteps_;
};

// ------------------------------------------------------------ tiny XML tree
struct Node {
  std::string name, text;
  std::vector<Node> kids;
  const Node *child(const char *n) const {
    for (auto &k : kids) if (k.name == n) return &k;
    return nullptr;
  }
  long long num(const char *n, long long dflt = 0) const {
    const Node *c = child(n);
    return c ? strtoll(c->text.c_str(), nullptr, 10) : dflt;
  }
  size_t size(const char *n) const {
    const Node *c = child(n);
    return c ? (size_t)strtoull(c->text.c_str(), nullptr, 10) : 0;
  }
  // the name of the first child (searched to any depth) among `fields` that holds a
  // negative number: offsets and counts are sizes (readSizeTag, c2c_ir.h:55-60)
  const char *negativeSize(const char *const *fields, int nfields) const {
    for (auto &k : kids) {
      for (int i = 0; i < nfields; i++)
        if (k.name == fields[i] && !k.text.empty() && k.text[0] == '-') return fields[i];
      if (const char *deep = k.negativeSize(fields, nfields)) return deep;
    }
    return nullptr;
  }
};

static bool parseNode(const std::string &s, size_t &pos, Node &out) {
  // expects pos at '<' of an opening (or self-closing) tag
  size_t gt = s.find('>', pos);
  if (gt == std::string::npos) return false;
  std::string tag = s.substr(pos + 1, gt - pos - 1);
  pos = gt + 1;
  if (!tag.empty() && tag.back() == '/') {
    out.name = tag.substr(0, tag.size() - 1);
    return true;
  }
  out.name = tag;
  for (;;) {
    size_t lt = s.find('<', pos);
    if (lt == std::string::npos) return false;
    out.text += s.substr(pos, lt - pos);
    if (s.compare(lt, 2, "</") == 0) {
      size_t end = s.find('>', lt);
      if (end == std::string::npos || s.substr(lt + 2, end - lt - 2) != out.name) return false;
      pos = end + 1;
      // trim
      size_t a = out.text.find_first_not_of(" \t\r\n"), b = out.text.find_last_not_of(" \t\r\n");
      out.text = a == std::string::npos ? "" : out.text.substr(a, b - a + 1);
      return true;
    }
    pos = lt;
    Node kid;
    if (!parseNode(s, pos, kid)) return false;
    out.kids.push_back(kid);
  }
}

static HomoFunc homoFrom(const Node &n, size_t chunksize) {
  HomoFunc f;
  f.rootRank_ = (int)n.num("rootRank", -1);
  f.sendType_ = (int)n.num("sendType");
  f.recvType_ = (int)n.num("recvType");
  f.sendOffset_ = n.size("sendOffset") * chunksize;
  f.recvOffset_ = n.size("recvOffset") * chunksize;
  f.count_ = n.size("count") * chunksize;
  f.homoType_ = (int)n.num("homoType");
  f.commOp_ = (int)n.num("commOp");
  return f;
}

static void homoSteps(const Node *table, size_t chunksize, std::vector<std::vector<HomoFunc>> &out) {
  out.clear();
  if (!table) return;
  for (auto &step : table->kids) {
    if (step.name != "Step") continue;
    std::vector<HomoFunc> fs;
    for (auto &f : step.kids) if (f.name == "HomoFunc") fs.push_back(homoFrom(f, chunksize));
    out.push_back(fs);
  }
}

static void heteroSteps(const Node *table, size_t chunksize, std::vector<std::vector<HeteroFunc>> &out) {
  out.clear();
  if (!table) return;
  for (auto &step : table->kids) {
    if (step.name != "Step") continue;
    std::vector<HeteroFunc> fs;
    for (auto &f : step.kids) {
      if (f.name != "HeteroFunc") continue;
      HeteroFunc h;
      for (auto &o : f.kids) {
        if (o.name != "P2pOp") continue;
        P2pOp p;
        p.rank_ = (int)o.num("rank");
        p.peerRank_ = (int)o.num("peerRank");
        p.offset_ = o.size("offset") * chunksize;
        p.count_ = o.size("count") * chunksize;
        p.isRecv_ = (int)o.num("isRecv");
        h.p2pOps_.push_back(p);
      }
      fs.push_back(h);
    }
    out.push_back(fs);
  }
}

static void writeHomoSteps(FILE *f, const char *tag, const std::vector<std::vector<HomoFunc>> &steps, size_t cs) {
  // layout of serializeFunc2DVector / serializeHomoFunc (c2c_ir.h:76-92,121-144)
  fprintf(f, "  <%s>\n", tag);
  for (auto &step : steps) {
    if (step.empty()) { fprintf(f, "    <Step/>\n"); continue; }
    fprintf(f, "    <Step>\n");
    for (auto &h : step) {
      fprintf(f, "      <HomoFunc>\n");
      fprintf(f, "        <rootRank>%d</rootRank>\n", h.rootRank_);
      fprintf(f, "        <sendType>%d</sendType>\n", h.sendType_);
      fprintf(f, "        <recvType>%d</recvType>\n", h.recvType_);
      fprintf(f, "        <sendOffset>%zu</sendOffset>\n", h.sendOffset_ / cs);
      fprintf(f, "        <recvOffset>%zu</recvOffset>\n", h.recvOffset_ / cs);
      fprintf(f, "        <count>%zu</count>\n", h.count_ / cs);
      fprintf(f, "        <homoType>%d</homoType>\n", h.homoType_);
      fprintf(f, "        <commOp>%d</commOp>\n", h.commOp_);
      fprintf(f, "      </HomoFunc>\n");
    }
    fprintf(f, "    </Step>\n");
  }
  fprintf(f, "  </%s>\n", tag);
}

} // namespace

// Temporaries of one Execute (member lists, pending copies, the record of cleared ranges) come
// from a block that the plan keeps between calls: an allocation is a pointer bump, a release is
// nothing, and everything goes at once when the call ends.  A replay of a small collective is
// bound by the host, and some three hundred heap allocations per call were half of its time.
struct Arena {
  std::vector<char> block;
  size_t used = 0;
  std::vector<void *> overflow; // requests that did not fit: plain heap, freed at reset
  void *alloc(size_t n, size_t align) {
    size_t at = (used + align - 1) & ~(align - 1);
    if (at + n <= block.size()) {
      used = at + n;
      return block.data() + at;
    }
    void *q = ::operator new(n);
    overflow.push_back(q);
    return q;
  }
  void reset() {
    used = 0;
    for (void *q : overflow) ::operator delete(q);
    overflow.clear();
  }
};

struct flagcxLocalPlan {
  int nranks = 0;
  std::vector<int> clusterOf, isInter;
  std::vector<std::vector<int>> clusterRanks, clusterInterRanks; // global ranks, ascending
  std::vector<int> homoRank, homoInterRank;                      // per global rank (-1: none)
  size_t totalCount = 0;
  int commOp = flagcxCommNoOp, redOp = flagcxSum;
  std::vector<RankPlan> ranks;
  int algorithm = 2; // flagcxAlgoInput: what importXml sets (c2c_algo.h:15-19, c2c_algo.cc:974)
  size_t defaultChunks = 0; // nChunks of documents that carry none (flagcxLocalPlanSetChunks)
  int eachNicPerRank = 0, multiNic = 0; // as the planner's constructor sets them (c2c_algo.cc:636-672)
  // AlltoAllv: row r of each matrix is the array rank r hands to execute() (c2c_algo.cc:2042-2046,2083-2094)
  std::vector<size_t> sendCounts, sDispls, recvCounts, rDispls;
  bool loaded = false;
  bool fused = true; // flagcxLocalPlanSetFused
  uint64_t lastBytes = 0, lastLaunches = 0; // flagcxLocalPlanGetTraffic
  Arena arena;                              // temporaries of the Execute in progress
  char err[256] = "";
};

namespace {

static flagcxResult_t planFail(flagcxLocalPlan *p, flagcxResult_t code, const char *fmt, const char *a = "",
                               long long b = 0, long long c = 0) {
  snprintf(p->err, sizeof(p->err), fmt, a, b, c);
  return code;
}

#define LCHECK(call)                                                           \
  do {                                                                         \
    flagcxResult_t r_ = (call);                                                \
    if (r_ != flagcxSuccess) return r_;                                        \
  } while (0)

static thread_local Arena *tlsArena = nullptr; // set for the duration of one flagcxLocalPlanExecute

template <typename T>
struct ArenaAlloc {
  typedef T value_type;
  ArenaAlloc() = default;
  template <typename U>
  ArenaAlloc(const ArenaAlloc<U> &) {}
  // containers with this allocator live inside one flagcxLocalPlanExecute and nowhere else
  T *allocate(size_t n) {
    if (!tlsArena) throw std::bad_alloc();
    return static_cast<T *>(tlsArena->alloc(n * sizeof(T), alignof(T) < 8 ? 8 : alignof(T)));
  }
  void deallocate(T *, size_t) {}
  template <typename U>
  bool operator==(const ArenaAlloc<U> &) const { return true; }
  template <typename U>
  bool operator!=(const ArenaAlloc<U> &) const { return false; }
};
namespace ex {
template <typename T>
using vector = std::vector<T, ArenaAlloc<T>>;
template <typename K, typename V>
using map = std::map<K, V, std::less<K>, ArenaAlloc<std::pair<const K, V>>>;
} // namespace ex

// Byte ranges of device memory that hold zeros by definition but have not been written.
// The reference assembles a sum across a cluster by clearing, in every member's buffer,
// all but the member's own slice (flagcxC2cRefreshFunc::run, c2c_algo.cc:586-608) and
// then all-reducing the whole buffers (c2c_algo.cc:310-336): most of what that collective
// reads are the zeros just written.  The fused replay keeps those ranges here instead:
// a refresh adds ranges, a write removes them, a copy out of them moves them, a sum leaves
// out the members that lie in them, and what is left when the plan ends is written then.
class ZeroSet {
  ex::map<uintptr_t, uintptr_t> r_; // begin -> end: disjoint, never adjacent
 public:
  bool empty() const { return r_.empty(); }
  void add(uintptr_t b, uintptr_t e) {
    if (b >= e) return;
    auto it = r_.upper_bound(b);
    if (it != r_.begin()) {
      auto pv = std::prev(it);
      if (pv->second >= b) {
        b = pv->first;
        if (pv->second > e) e = pv->second;
        it = r_.erase(pv);
      }
    }
    while (it != r_.end() && it->first <= e) {
      if (it->second > e) e = it->second;
      it = r_.erase(it);
    }
    r_[b] = e;
  }
  void remove(uintptr_t b, uintptr_t e) {
    if (b >= e) return;
    auto it = r_.upper_bound(b);
    if (it != r_.begin()) --it;
    while (it != r_.end() && it->first < e) {
      const uintptr_t rb = it->first, re = it->second;
      if (re <= b) {
        ++it;
        continue;
      }
      it = r_.erase(it);
      if (rb < b) r_[rb] = b;
      if (re > e) r_[e] = re;
    }
  }
  bool touches(uintptr_t b, uintptr_t e) const {
    if (b >= e) return false;
    auto it = r_.upper_bound(b);
    if (it != r_.begin() && std::prev(it)->second > b) return true;
    return it != r_.end() && it->first < e;
  }
  bool covers(uintptr_t b, uintptr_t e) const {
    auto it = r_.upper_bound(b);
    if (it == r_.begin()) return false;
    --it;
    return it->second >= e;
  }
  // where zero ranges begin or end strictly inside (b, e), as offsets from b, ascending
  void cuts(uintptr_t b, uintptr_t e, ex::vector<size_t> &out) const {
    auto it = r_.upper_bound(b);
    if (it != r_.begin()) --it;
    for (; it != r_.end() && it->first < e; ++it) {
      if (it->first > b) out.push_back(it->first - b);
      if (it->second > b && it->second < e) out.push_back(it->second - b);
    }
  }
  ex::vector<std::pair<uintptr_t, uintptr_t>> ranges() const {
    return ex::vector<std::pair<uintptr_t, uintptr_t>>(r_.begin(), r_.end());
  }
};

// One reduction of a collective: dst = fold of src[0..n) over `count` elements.
struct Red {
  char *dst;
  ex::vector<const char *> src;
  size_t count;
};

// One flagcxLocalPlanExecute call.
struct Exec {
  flagcxLocalPlan *p;
  const void *const *send;
  void *const *recv;
  void *const *scratch;
  flagcxDataType_t dt;
  size_t ts;
  int homoRoot;
  flagcxStream_t stream;
  bool fused;
  ZeroSet zeros;
  ex::vector<char> ownsScratch; // per rank: the reference allocates a scratch buffer for this call (c2c_algo.cc:2122-2129)
  ex::vector<char *> recvTmp, sendTmp;
  uint64_t bytes = 0, launches = 0; // algorithmic traffic handed to the kernels

  char *pick(int rank, int type) const {
    // sendType_: 0 user send, 1 recv, 2 scratch; recvType_: 1 recv, else scratch (c2c_algo.cc:297-300)
    if (type == 0) return (char *)const_cast<void *>(send[rank]);
    if (type == 1) return (char *)recv[rank];
    return scratch ? (char *)scratch[rank] : nullptr;
  }
  flagcxResult_t needScratch() { return planFail(p, flagcxInvalidArgument, "plan needs a scratch buffer%s", ""); }
  // [offset, offset + blocks * count) in elements lies inside the totalCount elements that the
  // largest buffer of the collective holds
  bool fits(size_t offset, size_t count, size_t blocks) const {
    if (offset > p->totalCount) return false;
    const size_t room = p->totalCount - offset;
    return blocks == 0 || count <= room / blocks;
  }
  flagcxResult_t outside(int r) {
    return planFail(p, flagcxInvalidArgument, "rank %s%lld: a function reaches past totalCount elements", "", r);
  }

  // Copies wait here until something depends on them, and then go out together: the P2P ops of a
  // hetero function run as one group in the reference (flagcxC2cHeteroFunc::run,
  // c2c_algo.cc:554-568), and so do the sends of a homo function; on one GPU a group is one launch
  // of the batch kernel with one input per segment (a sum of one input is a copy) instead of a
  // launch per copy, which for chunk-sized copies runs at the rate of a large launch.
  struct Pending {
    char *dst;
    const char *src;
    size_t n;
  };
  ex::vector<Pending> pending;
  static bool hit(const char *a, size_t an, const char *b, size_t bn) { return a < b + bn && b < a + an; }

  flagcxResult_t flushCopies() {
    if (pending.empty()) return flagcxSuccess;
    flagcxResult_t r;
    if (pending.size() == 1) {
      launches++;
      r = flagcxLocalMemcpy(pending[0].dst, pending[0].src, pending[0].n, stream);
    } else {
      // copies of one source and one length (the sends of a broadcast, a member's block in an
      // all-gather) share one read of it: flagcxLocalCopyFanout; the rest go as one batch
      const size_t np = pending.size();
      ex::vector<int> groupOf(np, -1);
      ex::vector<ex::vector<void *>> dsts;
      ex::vector<size_t> first;
      for (size_t i = 0; i < np; i++) {
        for (size_t g = 0; g < first.size() && groupOf[i] < 0; g++)
          if (pending[first[g]].src == pending[i].src && pending[first[g]].n == pending[i].n) groupOf[i] = (int)g;
        if (groupOf[i] < 0) {
          groupOf[i] = (int)first.size();
          first.push_back(i);
          dsts.emplace_back();
        }
        dsts[groupOf[i]].push_back(pending[i].dst);
      }
      ex::vector<flagcxLocalFanoutDesc> fans;
      ex::vector<const void *> src;
      ex::vector<flagcxLocalReduceDesc> descs;
      src.reserve(np);
      for (size_t g = 0; g < first.size(); g++) {
        const Pending &c = pending[first[g]];
        if (dsts[g].size() >= 2) {
          fans.push_back({c.src, dsts[g].data(), (int)dsts[g].size(), c.n});
          bytes -= (uint64_t)(dsts[g].size() - 1) * c.n; // the source is read once
        } else {
          src.push_back(c.src);
          descs.push_back({&src.back(), c.dst, c.n});
        }
      }
      r = flagcxSuccess;
      if (!fans.empty()) {
        launches += (fans.size() + 15) / 16;
        r = flagcxLocalCopyFanout(fans.data(), (int)fans.size(), stream);
      }
      if (r == flagcxSuccess && descs.size() == 1) {
        launches++;
        r = flagcxLocalMemcpy(descs[0].recvbuff, src[0], descs[0].count, stream);
      } else if (r == flagcxSuccess && !descs.empty()) {
        launches += (descs.size() + 31) / 32;
        r = flagcxLocalReduceBatch(descs.data(), (int)descs.size(), 1, flagcxUint8, flagcxSum, stream);
      }
    }
    pending.clear();
    return r;
  }
  flagcxResult_t memcpyNow(char *dst, const char *src, size_t n) {
    if (hit(dst, n, src, n)) return planFail(p, flagcxInvalidArgument, "a copy's buffers overlap%s", "");
    // a copy that touches what a waiting copy writes, or writes what one reads, must follow it
    for (auto &c : pending)
      if (hit(dst, n, c.dst, c.n) || hit(dst, n, c.src, c.n) || hit(src, n, c.dst, c.n)) {
        LCHECK(flushCopies());
        break;
      }
    bytes += 2 * n;
    pending.push_back({dst, src, n});
    if (pending.size() >= 64) return flushCopies();
    return flagcxSuccess;
  }
  flagcxResult_t memsetNow(char *dst, size_t n) {
    LCHECK(flushCopies());
    bytes += n;
    launches++;
    return flagcxLocalMemset(dst, 0, n, stream);
  }

  // dst[0, n) = src[0, n), zeros that were never written included.
  flagcxResult_t copy(char *dst, const char *src, size_t n) {
    if (!n || dst == src) return flagcxSuccess;
    const uintptr_t s = (uintptr_t)src, d = (uintptr_t)dst;
    if (!fused || zeros.empty()) return memcpyNow(dst, src, n);
    if (!zeros.touches(s, s + n)) {
      zeros.remove(d, d + n);
      return memcpyNow(dst, src, n);
    }
    if (d < s + n && s < d + n) return planFail(p, flagcxInvalidArgument, "a copy's buffers overlap%s", "");
    ex::vector<size_t> cut{0};
    zeros.cuts(s, s + n, cut);
    cut.push_back(n);
    ex::vector<char> isZero(cut.size() - 1);
    for (size_t i = 0; i + 1 < cut.size(); i++) isZero[i] = zeros.covers(s + cut[i], s + cut[i + 1]);
    for (size_t i = 0; i + 1 < cut.size(); i++) {
      const size_t at = cut[i], len = cut[i + 1] - cut[i];
      if (isZero[i]) {
        zeros.add(d + at, d + at + len);
      } else {
        zeros.remove(d + at, d + at + len);
        LCHECK(memcpyNow(dst + at, src + at, len));
      }
    }
    return flagcxSuccess;
  }

  // m blocks of `n` bytes from the pointers in `src` into dst, back to back.  The blocks join
  // the waiting copies: an all-gather hands every block to every member, and copies of one
  // source go out with one read of it (flushCopies); a block that already lies at its place
  // (in-place all-gather, flagcx/include/flagcx.h:373) is a copy onto itself, i.e. nothing.
  flagcxResult_t gather(char *dst, const ex::vector<const void *> &src, size_t n) {
    for (size_t j = 0; j < src.size(); j++) LCHECK(copy(dst + j * n, (const char *)src[j], n));
    return flagcxSuccess;
  }

  // Zeros that are due in [b, e) are written now.
  flagcxResult_t materialize(uintptr_t b, uintptr_t e) {
    if (!fused || !zeros.touches(b, e)) return flagcxSuccess;
    ex::vector<size_t> cut{0};
    zeros.cuts(b, e, cut);
    cut.push_back(e - b);
    for (size_t i = 0; i + 1 < cut.size(); i++)
      if (zeros.covers(b + cut[i], b + cut[i + 1])) LCHECK(memsetNow((char *)b + cut[i], cut[i + 1] - cut[i]));
    zeros.remove(b, e);
    return flagcxSuccess;
  }

  flagcxResult_t reduceNow(const ex::vector<Red> &reds, int nzero) {
    LCHECK(flushCopies());
    const int nlive = (int)reds[0].src.size();
    const flagcxRedOp_t rop = (flagcxRedOp_t)p->redOp;
    ex::vector<flagcxLocalReduceDesc> descs(reds.size());
    for (size_t i = 0; i < reds.size(); i++) {
      descs[i] = {(const void *const *)reds[i].src.data(), reds[i].dst, reds[i].count};
      bytes += (uint64_t)(nlive + 1) * reds[i].count * ts;
    }
    launches += (reds.size() + 31) / 32;
    if (nzero) return flagcxLocalReduceBatchSparse(descs.data(), (int)descs.size(), nlive, nzero, dt, rop, stream);
    if (reds.size() == 1) return flagcxLocalReduce(descs[0].sendbuffs, nlive, descs[0].recvbuff, descs[0].count, dt, rop, stream);
    return flagcxLocalReduceBatch(descs.data(), (int)descs.size(), nlive, dt, rop, stream);
  }

  // The reductions of one collective (same member count; they run concurrently).  Members
  // whose slice lies in zeros that were never written are not read: a sum over the rest,
  // with +0.0 added once, has the bytes of the sum over all of them (the zero members turn
  // a -0.0 result into +0.0 and change nothing else).
  flagcxResult_t reduce(const ex::vector<Red> &reds) {
    if (reds.empty()) return flagcxSuccess;
    for (auto &r : reds)
      if (r.src.size() != reds[0].src.size()) {
        // clusters of different sizes in one slot: one call per member count
        ex::map<size_t, ex::vector<Red>> byCount;
        for (auto &q : reds) byCount[q.src.size()].push_back(q);
        for (auto &g : byCount) LCHECK(reduce(g.second));
        return flagcxSuccess;
      }
    bool plain = !fused || zeros.empty();
    if (!plain) {
      plain = true;
      for (auto &r : reds)
        for (auto s : r.src)
          if (zeros.touches((uintptr_t)s, (uintptr_t)s + r.count * ts)) plain = false;
    }
    if (!plain && p->redOp != flagcxSum) {
      // for a maximum or a minimum a zero is a value like any other
      for (auto &r : reds)
        for (auto s : r.src) LCHECK(materialize((uintptr_t)s, (uintptr_t)s + r.count * ts));
      plain = true;
    }
    if (plain) {
      if (fused)
        for (auto &r : reds) zeros.remove((uintptr_t)r.dst, (uintptr_t)r.dst + r.count * ts);
      return reduceNow(reds, 0);
    }
    const int n = (int)reds[0].src.size();
    ex::map<int, ex::vector<Red>> byLive; // members read -> pieces (n: no member left out)
    ex::vector<std::pair<uintptr_t, uintptr_t>> written, cleared;
    for (auto &r : reds) {
      const size_t len = r.count * ts;
      ex::vector<size_t> cut{0, len};
      for (auto s : r.src) zeros.cuts((uintptr_t)s, (uintptr_t)s + len, cut);
      std::sort(cut.begin(), cut.end());
      cut.erase(std::unique(cut.begin(), cut.end()), cut.end());
      for (size_t i = 0; i + 1 < cut.size(); i++) {
        const size_t a = cut[i], b = cut[i + 1];
        if (a % ts || b % ts) return planFail(p, flagcxInternalError, "a cleared range ends inside an element%s", "");
        Red piece{r.dst + a, {}, (b - a) / ts};
        for (auto s : r.src)
          if (!zeros.covers((uintptr_t)s + a, (uintptr_t)s + b)) piece.src.push_back(s + a);
        if (piece.src.empty()) {
          cleared.push_back({(uintptr_t)r.dst + a, (uintptr_t)r.dst + b}); // 0 + 0 + ... = +0
        } else {
          written.push_back({(uintptr_t)r.dst + a, (uintptr_t)r.dst + b});
          byLive[(int)piece.src.size()].push_back(std::move(piece));
        }
      }
    }
    for (auto &w : written) zeros.remove(w.first, w.second);
    for (auto &c : cleared) zeros.add(c.first, c.second);
    for (auto &g : byLive) LCHECK(reduceNow(g.second, n - g.first));
    return flagcxSuccess;
  }

  // No reduction of one group writes what a reduction of another group reads or writes (the
  // groups are collectives of different clusters, or folds local to different ranks).
  bool independent(const ex::vector<ex::vector<Red>> &groups) const {
    for (size_t a = 0; a < groups.size(); a++)
      for (size_t b = 0; b < groups.size(); b++) {
        if (a == b) continue;
        for (auto &w : groups[a])
          for (auto &r : groups[b]) {
            const size_t wn = w.count * ts, rn = r.count * ts;
            if (hit(w.dst, wn, r.dst, rn)) return false;
            for (auto s : r.src)
              if (hit(w.dst, wn, s, rn)) return false;
          }
      }
    return true;
  }

  flagcxResult_t refresh(const ex::vector<char> *only);
  flagcxResult_t homoSlot(const ex::vector<const HomoFunc *> &fn);
  flagcxResult_t sendRecv(int cl, const ex::vector<const HomoFunc *> &fn);
  flagcxResult_t homoStep(std::vector<std::vector<HomoFunc>> RankPlan::*table, int s, int onlyIndex = -1,
                          const ex::vector<char> *only = nullptr, bool refreshBeforeEach = false);
  flagcxResult_t heteroSlot(int s, int i);
  flagcxResult_t run();
  flagcxResult_t finish();
};

// One homo function slot (step s, index i of one table) across all ranks; fn[r] is rank
// r's function or NULL.  The collective's root reaches the functions as a rank of its
// cluster, globalrank2homorank[root] (c2c_algo.cc:2147,2170).
flagcxResult_t Exec::homoSlot(const ex::vector<const HomoFunc *> &fn) {
  const int ncl = (int)p->clusterRanks.size();
  const int root = homoRoot;
  // The clusters run a slot side by side, each on its own ranks' buffers: their reductions go
  // out together (one batch launch per member count instead of one per cluster), and the copies
  // that hand an all-reduce's result to the other members follow them.
  ex::vector<ex::vector<Red>> groups; // one per collective (or per rank-local fold)
  struct After {
    char *dst;
    const char *src;
    size_t n;
  };
  ex::vector<After> after;
  for (int cl = 0; cl < ncl; cl++) {
    // members that hold a function in this slot; homoType 1 runs on inter-ranks only
    ex::vector<int> mem;
    const HomoFunc *first = nullptr;
    for (int r : p->clusterRanks[cl]) {
      const HomoFunc *f = fn[r];
      if (!f) continue;
      if (f->homoType_ == 1 && p->homoInterRank[r] == -1) continue; // c2c_algo.cc:293-295
      if (!first) first = f;
      mem.push_back(r);
    }
    if (!first) continue;
    const int op = first->commOp_;
    // rank-local primitives need no peers
    if (op == kLocCpy || op == kLocRed) {
      for (int r : mem) {
        const HomoFunc *f = fn[r];
        char *s = pick(r, f->sendType_), *d = pick(r, f->recvType_ == 1 ? 1 : 2);
        if (!s || !d) return needScratch();
        if (!fits(f->sendOffset_, f->count_, 1) || !fits(f->recvOffset_, f->count_, 1)) return outside(r);
        s += f->sendOffset_ * ts;
        d += f->recvOffset_ * ts;
        if (op == kLocCpy) {
          LCHECK(copy(d, s, f->count_ * ts));
        } else {
          groups.push_back({Red{d, {d, s}, f->count_}}); // acc = recv slice; acc = OP(send slice, acc)
        }
      }
      continue;
    }
    if (op == flagcxCommOpSend || op == flagcxCommOpRecv) {
      LCHECK(sendRecv(cl, fn));
      continue;
    }
    if (op == flagcxCommOpAlltoAllv) {
      // every member sends to and receives from the members of its own cluster, counts and
      // displacements from the caller's arrays, buffers without offsets (c2c_algo.cc:482-508)
      const size_t n = (size_t)p->nranks;
      if (p->sendCounts.empty())
        return planFail(p, flagcxInvalidArgument, "AlltoAllv needs counts and displacements (flagcxLocalPlanSetAlltoAllv)%s", "");
      for (int r : mem) {
        const HomoFunc *f = fn[r];
        char *src = pick(r, f->sendType_);
        if (!src) return needScratch();
        for (int i : p->clusterRanks[cl]) {
          const size_t cnt = p->sendCounts[r * n + i];
          const HomoFunc *g = fn[i];
          const bool recvs = g && g->commOp_ == op && !(g->homoType_ == 1 && p->homoInterRank[i] == -1);
          if (cnt != (recvs ? p->recvCounts[i * n + r] : 0))
            return planFail(p, flagcxInvalidUsage, "AlltoAllv: rank %s%lld sends to rank %lld what that rank does not receive", "", r, i);
          if (!cnt) continue;
          char *dst = pick(i, g->recvType_ == 1 ? 1 : 2);
          if (!dst) return needScratch();
          LCHECK(copy(dst + p->rDispls[i * n + r] * ts, src + p->sDispls[r * n + i] * ts, cnt * ts));
        }
      }
      // a receive nobody sends would hang the reference
      for (int i : mem)
        for (int r : p->clusterRanks[cl]) {
          const bool sends = fn[r] && fn[r]->commOp_ == op && !(fn[r]->homoType_ == 1 && p->homoInterRank[r] == -1);
          if (p->recvCounts[i * n + r] && !sends)
            return planFail(p, flagcxInvalidUsage, "AlltoAllv: rank %s%lld receives from rank %lld what that rank does not send", "", i, r);
        }
      continue;
    }
    // the communicator the reference would use: homoInterComm for homoType 1, else homo_comm
    const std::vector<int> &comm = first->homoType_ == 1 ? p->clusterInterRanks[cl] : p->clusterRanks[cl];
    const int n = (int)comm.size();
    ex::vector<char *> S(n, nullptr), D(n, nullptr);
    ex::vector<size_t> cnt(n, 0);
    for (int h = 0; h < n; h++) {
      const int r = comm[h];
      const HomoFunc *f = fn[r];
      if (!f || f->commOp_ != op)
        return planFail(p, flagcxInvalidUsage, "rank %s%lld has no matching homo function (commOp %lld)", "", r, op);
      char *s = pick(r, f->sendType_), *d = pick(r, f->recvType_ == 1 ? 1 : 2);
      if (!s || !d) return needScratch();
      S[h] = s + f->sendOffset_ * ts;
      D[h] = d + f->recvOffset_ * ts;
      cnt[h] = f->count_;
    }
    const size_t count = cnt[0];
    auto homoRootOf = [&](const HomoFunc *f) { return f->rootRank_ == -1 ? root : f->rootRank_; };
    auto badRoot = [&](int rt) { return planFail(p, flagcxInvalidArgument, "root %s%lld outside the communicator", "", rt); };
    {
      // every range a member reads or writes lies inside totalCount elements, the most any
      // buffer of the collective holds (c2c_algo.cc:623,2124): blocks per member, and whether
      // only the root's range is touched
      const bool sBlocks = op == flagcxCommOpReduceScatter || op == flagcxCommOpScatter || op == flagcxCommOpAlltoAll;
      const bool dBlocks = op == flagcxCommOpAllGather || op == flagcxCommOpGather || op == flagcxCommOpAlltoAll;
      const bool sRootOnly = op == flagcxCommOpScatter || op == flagcxCommOpBroadcast;
      const bool dRootOnly = op == flagcxCommOpReduce || op == flagcxCommOpGather;
      const int rt = (sRootOnly || dRootOnly) ? homoRootOf(first) : -1;
      if (op != flagcxCommNoOp)
        for (int h = 0; h < n; h++) {
          const HomoFunc *f = fn[comm[h]];
          if (!(sRootOnly && h != rt) && !fits(f->sendOffset_, count, sBlocks ? (size_t)n : 1)) return outside(comm[h]);
          if (!(dRootOnly && h != rt) && !fits(f->recvOffset_, count, dBlocks ? (size_t)n : 1)) return outside(comm[h]);
        }
    }
    const ex::vector<const char *> members(S.begin(), S.end());
    switch (op) {
      case flagcxCommOpReduce: {
        const int rt = homoRootOf(first);
        if (rt < 0 || rt >= n) return badRoot(rt);
        groups.push_back({Red{D[rt], members, count}});
        break;
      }
      case flagcxCommOpAllReduce: {
        // every member ends with the same bytes: reduce once, then copy
        groups.push_back({Red{D[0], members, count}});
        for (int h = 1; h < n; h++) after.push_back({D[h], D[0], count * ts});
        break;
      }
      case flagcxCommOpReduceScatter: {
        // member h receives the fold of everybody's h-th block; one batch launch
        ex::vector<Red> reds(n);
        for (int h = 0; h < n; h++) {
          reds[h].dst = D[h];
          reds[h].count = count;
          for (int j = 0; j < n; j++) reds[h].src.push_back(S[j] + (size_t)h * count * ts);
        }
        groups.push_back(std::move(reds));
        break;
      }
      case flagcxCommOpAllGather: {
        const ex::vector<const void *> blocks(S.begin(), S.end());
        for (int h = 0; h < n; h++) LCHECK(gather(D[h], blocks, count * ts));
        break;
      }
      case flagcxCommOpGather: {
        const int rt = homoRootOf(first);
        if (rt < 0 || rt >= n) return badRoot(rt);
        LCHECK(gather(D[rt], ex::vector<const void *>(S.begin(), S.end()), count * ts));
        break;
      }
      case flagcxCommOpScatter: {
        const int rt = homoRootOf(first);
        if (rt < 0 || rt >= n) return badRoot(rt);
        for (int h = 0; h < n; h++) LCHECK(copy(D[h], S[rt] + (size_t)h * count * ts, count * ts));
        break;
      }
      case flagcxCommOpBroadcast: {
        const int rt = homoRootOf(first);
        if (rt < 0 || rt >= n) return badRoot(rt);
        for (int h = 0; h < n; h++) LCHECK(copy(D[h], S[rt], count * ts));
        break;
      }
      case flagcxCommOpAlltoAll: {
        ex::vector<const void *> blocks(n);
        for (int h = 0; h < n; h++) {
          for (int j = 0; j < n; j++) blocks[j] = S[j] + (size_t)h * count * ts;
          LCHECK(gather(D[h], blocks, count * ts));
        }
        break;
      }
      case flagcxCommNoOp:
        break;
      default:
        return planFail(p, flagcxNotSupported, "homo function commOp %s%lld is not replayed", "", op);
    }
  }
  if (groups.size() > 1 && independent(groups)) {
    ex::vector<Red> all;
    for (auto &g : groups)
      for (auto &r : g) all.push_back(std::move(r));
    LCHECK(reduce(all));
  } else {
    for (auto &g : groups) LCHECK(reduce(g));
  }
  for (auto &c : after) LCHECK(copy(c.dst, c.src, c.n));
  return flagcxSuccess;
}

// Functions i (all of them, or `onlyIndex`) of step s of one table.  `only`: the ranks that
// take part (a rank leaves a loop of the reference when ITS table runs out); with
// refreshBeforeEach every rank that runs function i refreshes first (c2c_algo.cc:2276-2282).
flagcxResult_t Exec::homoStep(std::vector<std::vector<HomoFunc>> RankPlan::*table, int s, int onlyIndex,
                              const ex::vector<char> *only, bool refreshBeforeEach) {
  size_t width = 0;
  for (auto &rp : p->ranks) {
    auto &t = rp.*table;
    if (s < (int)t.size() && t[s].size() > width) width = t[s].size();
  }
  ex::vector<char> has(p->nranks);
  for (size_t i = 0; i < width; i++) {
    if (onlyIndex >= 0 && (int)i != onlyIndex) continue;
    ex::vector<const HomoFunc *> fn(p->nranks, nullptr);
    bool any = false;
    for (int r = 0; r < p->nranks; r++) {
      auto &t = p->ranks[r].*table;
      has[r] = (!only || (*only)[r]) && s < (int)t.size() && i < t[s].size();
      if (has[r]) fn[r] = &t[s][i];
      any = any || has[r];
    }
    if (!any) continue;
    if (refreshBeforeEach) LCHECK(refresh(&has));
    LCHECK(homoSlot(fn));
  }
  return flagcxSuccess;
}

// Hetero function i of step s on every rank: match each send with the peer's
// next unmatched receive from that sender (order of appearance).
flagcxResult_t Exec::heteroSlot(int s, int i) {
  ex::map<std::pair<int, int>, ex::vector<const P2pOp *>> recvs; // (receiver, sender) -> ops
  for (int r = 0; r < p->nranks; r++) {
    auto &t = p->ranks[r].heteroFuncSteps_;
    if (s >= (int)t.size() || i >= (int)t[s].size()) continue;
    for (auto &op : t[s][i].p2pOps_)
      if (op.isRecv_) recvs[{r, op.peerRank_}].push_back(&op);
  }
  ex::map<std::pair<int, int>, size_t> used;
  for (int r = 0; r < p->nranks; r++) {
    auto &t = p->ranks[r].heteroFuncSteps_;
    if (s >= (int)t.size() || i >= (int)t[s].size()) continue;
    for (auto &op : t[s][i].p2pOps_) {
      if (op.isRecv_) continue;
      const int peer = op.peerRank_;
      if (peer < 0 || peer >= p->nranks) return planFail(p, flagcxInvalidArgument, "P2pOp peer %s%lld out of range", "", peer);
      auto key = std::make_pair(peer, r);
      size_t &u = used[key];
      auto it = recvs.find(key);
      if (it == recvs.end() || u >= it->second.size())
        return planFail(p, flagcxInvalidUsage, "send %s%lld -> %lld has no matching receive", "", r, peer);
      const P2pOp *rv = it->second[u++];
      if (rv->count_ != op.count_)
        return planFail(p, flagcxInvalidUsage, "send/recv count mismatch between ranks %s%lld and %lld", "", r, peer);
      if (!recvTmp[peer] || !sendTmp[r])
        return planFail(p, flagcxInvalidArgument, "rank %s%lld stages its hetero functions in scratch and was given none", "",
                        recvTmp[peer] ? r : peer);
      if (!fits(op.offset_, op.count_, 1)) return outside(r);
      if (!fits(rv->offset_, rv->count_, 1)) return outside(peer);
      LCHECK(copy(recvTmp[peer] + rv->offset_ * ts, sendTmp[r] + op.offset_ * ts, op.count_ * ts));
    }
  }
  for (auto &kv : recvs)
    if (used[kv.first] != kv.second.size())
      return planFail(p, flagcxInvalidUsage, "receive on rank %s%lld from %lld has no matching send", "", kv.first.first, kv.first.second);
  return flagcxSuccess;
}

// The refresh function of every rank (only: of the ranks marked).
flagcxResult_t Exec::refresh(const ex::vector<char> *only) {
  for (int r = 0; r < p->nranks; r++) {
    if (only && !(*only)[r]) continue;
    const RefreshFunc &f = p->ranks[r].refreshFunc_;
    // bufftype -1 resolves to scratch (2) on a rank the reference gives a scratch buffer and to
    // recv (1) on every other, and under the pipeline algorithm a reduce-type collective starts
    // at its cluster's part (c2c_algo.cc:2156-2164)
    int bt = f.bufftype_;
    size_t start = f.start_;
    if (bt == -1) {
      bt = ownsScratch[r] ? 2 : 1;
      if ((p->commOp == flagcxCommOpReduceScatter || p->commOp == flagcxCommOpAllReduce) && p->algorithm == 1) {
        size_t clusterOffset = 0;
        for (int c = 0; c < p->clusterOf[r]; c++) clusterOffset += p->clusterRanks[c].size();
        start = clusterOffset * p->totalCount / (size_t)p->nranks;
      }
    }
    void *buff = bt == 1 ? recv[r] : (scratch ? scratch[r] : nullptr);
    if (f.totalCount_ == 0) continue;
    if (!buff) return planFail(p, flagcxInvalidArgument, "refresh needs a scratch buffer%s", "");
    if (f.redOp_ == flagcxSum && !fits(start, f.totalCount_, 1)) return outside(r);
    if (!fused) {
      LCHECK(flushCopies());
      if (f.redOp_ == flagcxSum && f.count_ < f.totalCount_) {
        bytes += (f.totalCount_ - f.count_) * ts;
        launches++;
      }
      LCHECK(flagcxLocalRefresh(buff, start, f.offset_, f.count_, f.totalCount_, dt, (flagcxRedOp_t)f.redOp_, stream));
      continue;
    }
    if (f.offset_ + f.count_ > f.totalCount_ || f.offset_ + f.count_ < f.offset_)
      return planFail(p, flagcxInvalidArgument, "refresh: offset + count exceeds totalCount%s", "");
    if (f.redOp_ != flagcxSum) continue; // c2c_algo.cc:596
    const uintptr_t base = (uintptr_t)buff + start * ts;
    zeros.add(base, base + f.offset_ * ts);
    zeros.add(base + (f.offset_ + f.count_) * ts, base + f.totalCount_ * ts);
  }
  return flagcxSuccess;
}

// Send / Recv homo functions of one cluster in one slot (c2c_algo.cc:364-463).  A
// send is carried out when the receiving rank holds the matching Recv function:
//   homoType 0: the root sends [sendOffset, +count) to every other inter-rank,
//               which receives at its recvOffset;
//   homoType 1: inter-ranks 1.. send to inter-rank 0 what they received from other
//               clusters, piece by piece at the pieces' own offsets;
//   homoType 2: inter-rank 0 sends to the root unless it is the root itself.
// Roots are ranks inside the cluster.
flagcxResult_t Exec::sendRecv(int cl, const ex::vector<const HomoFunc *> &fn) {
  const std::vector<int> &members = p->clusterRanks[cl], &inters = p->clusterInterRanks[cl];
  const int root = homoRoot;
  auto recvOf = [&](int r) -> const HomoFunc * {
    const HomoFunc *g = fn[r];
    return (g && g->commOp_ == flagcxCommOpRecv) ? g : nullptr;
  };
  for (int r : members) {
    const HomoFunc *f = fn[r];
    if (!f || f->commOp_ != flagcxCommOpSend) continue;
    const int rt = f->rootRank_ == -1 ? root : f->rootRank_;
    if (rt < 0 || rt >= (int)members.size())
      return planFail(p, flagcxInvalidArgument, "root %s%lld outside the communicator", "", rt);
    char *src = pick(r, f->sendType_);
    if (!src) return needScratch();
    if (f->homoType_ == 0) {
      if (p->homoRank[r] != rt) continue;
      for (int peer : inters) {
        const HomoFunc *g = recvOf(peer);
        if (peer == r || !g || p->homoRank[peer] == rt) continue;
        char *dst = pick(peer, g->recvType_ == 1 ? 1 : 2);
        if (!dst) return needScratch();
        if (!fits(f->sendOffset_, f->count_, 1)) return outside(r);
        if (!fits(g->recvOffset_, f->count_, 1)) return outside(peer);
        LCHECK(copy(dst + g->recvOffset_ * ts, src + f->sendOffset_ * ts, f->count_ * ts));
      }
    } else if (f->homoType_ == 1) {
      if (p->homoInterRank[r] <= 0 || inters.empty()) continue;
      const HomoFunc *g = recvOf(inters[0]);
      if (!g) continue;
      char *dst = pick(inters[0], g->recvType_ == 1 ? 1 : 2);
      if (!dst) return needScratch();
      // what rank r received from other clusters: every receive of its hetero functions
      ex::vector<std::pair<size_t, size_t>> pieces;
      for (auto &step : p->ranks[r].heteroFuncSteps_)
        for (auto &h : step)
          for (auto &o : h.p2pOps_) {
            if (!o.isRecv_) continue;
            bool seen = false;
            for (auto &q : pieces) seen = seen || (q.first == o.offset_ && q.second == o.count_);
            if (!seen) pieces.push_back({o.offset_, o.count_});
          }
      for (auto &q : pieces) {
        if (!fits(q.first, q.second, 1)) return outside(r);
        LCHECK(copy(dst + q.first * ts, src + q.first * ts, q.second * ts));
      }
    } else if (f->homoType_ == 2) {
      if (p->homoInterRank[r] != 0 || p->homoRank[r] == rt) continue;
      const int peer = members[rt];
      const HomoFunc *g = recvOf(peer);
      if (!g) continue;
      char *dst = pick(peer, g->recvType_ == 1 ? 1 : 2);
      if (!dst) return needScratch();
      if (!fits(f->sendOffset_, f->count_, 1)) return outside(r);
      if (!fits(g->recvOffset_, f->count_, 1)) return outside(peer);
      LCHECK(copy(dst + g->recvOffset_ * ts, src + f->sendOffset_ * ts, f->count_ * ts));
    }
  }
  return flagcxSuccess;
}

// flagcxC2cPlanner::execute from its first step on (c2c_algo.cc:2142-2290).
flagcxResult_t Exec::run() {
  const RankPlan &c = p->ranks[0];
  const int nr = p->nranks;
  const bool anyPipe = c.nPipePreSteps_ > 0 || c.nPipePostSteps_ > 0;
  // when the reference refreshes around sequential steps (c2c_algo.cc:2205-2208,2226-2229,2276-2279)
  const bool refreshSeq = p->algorithm == 0 || !anyPipe;
  const bool refreshAfterInter = p->algorithm == 1 && anyPipe;
  // Every rank walks ITS OWN tables: it runs hetero function i of a step while
  // i < heteroFuncSteps_[s].size() for itself, and behind it homoInter function i if its own
  // homoInterFuncSteps_[s] holds one (c2c_algo.cc:2177-2194,2204-2231,2247-2267).
  ex::vector<char> in(nr), has(nr);
  auto heteroAt = [&](int hs, size_t i) {
    bool any = false;
    for (int r = 0; r < nr; r++) {
      auto &t = p->ranks[r].heteroFuncSteps_;
      in[r] = hs < (int)t.size() && i < t[hs].size();
      any = any || in[r];
    }
    return any;
  };
  auto interAt = [&](int hs, size_t i) {
    bool any = false;
    for (int r = 0; r < nr; r++) {
      auto &t = p->ranks[r].homoInterFuncSteps_;
      has[r] = in[r] && hs < (int)t.size() && i < t[hs].size();
      any = any || has[r];
    }
    return any;
  };
  auto heteroWidth = [&](int hs) {
    size_t w = 0;
    for (auto &rp : p->ranks)
      if (hs < (int)rp.heteroFuncSteps_.size() && rp.heteroFuncSteps_[hs].size() > w) w = rp.heteroFuncSteps_[hs].size();
    return w;
  };

  // sequential preHomoFunc steps
  for (int s = 0; s < c.nSeqPreSteps_; s++) LCHECK(homoStep(&RankPlan::preHomoFuncSteps_, s));
  LCHECK(refresh(nullptr));
  // pipelined preHomoFunc + heteroFunc steps
  for (int s = 0; s < c.nPipePreSteps_; s++) {
    LCHECK(homoStep(&RankPlan::preHomoFuncSteps_, c.nSeqPreSteps_ + s));
    for (size_t i = 0; i < heteroWidth(s); i++) {
      if (!heteroAt(s, i)) continue;
      LCHECK(heteroSlot(s, (int)i));
      if (interAt(s, i)) {
        LCHECK(homoStep(&RankPlan::homoInterFuncSteps_, s, (int)i, &has));
        LCHECK(refresh(&has));
      }
    }
  }
  // sequential heteroFunc steps
  for (int s = 0; s < c.nSeqInterSteps_; s++) {
    const int hs = c.nPipePreSteps_ + s;
    for (size_t i = 0; i < heteroWidth(hs); i++) {
      if (!heteroAt(hs, i)) continue;
      if (refreshSeq) LCHECK(refresh(&in));
      LCHECK(heteroSlot(hs, (int)i));
      if (interAt(hs, i)) {
        LCHECK(homoStep(&RankPlan::homoInterFuncSteps_, hs, (int)i, &has));
        if (refreshAfterInter) LCHECK(refresh(&has));
      }
    }
  }
  // pipelined heteroFunc + postHomoFunc steps
  for (int s = 0; s < c.nPipePostSteps_; s++) {
    LCHECK(homoStep(&RankPlan::postHomoFuncSteps_, s));
    const int hs = c.nPipePreSteps_ + c.nSeqInterSteps_ + s;
    for (size_t i = 0; i < heteroWidth(hs); i++) {
      if (!heteroAt(hs, i)) continue;
      LCHECK(heteroSlot(hs, (int)i));
      if (interAt(hs, i)) LCHECK(homoStep(&RankPlan::homoInterFuncSteps_, hs, (int)i, &has));
    }
  }
  // sequential postHomoFunc steps
  for (int s = 0; s < c.nSeqPostSteps_; s++)
    LCHECK(homoStep(&RankPlan::postHomoFuncSteps_, c.nPipePostSteps_ + s, -1, nullptr, refreshSeq));
  return finish();
}

// Zeros that are still due are written, except into the scratch buffers that the reference
// allocates for the call and frees when it ends (c2c_algo.cc:2122-2129,2292-2295): nobody
// reads those again.
flagcxResult_t Exec::finish() {
  if (!fused) return flushCopies();
  for (int r = 0; r < p->nranks; r++)
    if (ownsScratch[r] && scratch && scratch[r])
      zeros.remove((uintptr_t)scratch[r], (uintptr_t)scratch[r] + p->totalCount * ts);
  for (auto &z : zeros.ranges()) LCHECK(memsetNow((char *)z.first, z.second - z.first));
  return flushCopies();
}

} // namespace

#pragma GCC visibility push(default)
extern "C" {

flagcxResult_t flagcxLocalPlanCreate(flagcxLocalPlan **plan, int nranks, const int *clusterIds,
                                     const int *isInterRank, size_t totalCount, flagcxCommOp_t commOp,
                                     flagcxRedOp_t redOp) {
  if (!plan || nranks < 1 || nranks > FLAGCX_LOCAL_MAX_RANKS || !clusterIds || totalCount == 0)
    return flagcxInvalidArgument;
  flagcxLocalPlan *p = nullptr;
  try {
  p = new flagcxLocalPlan();
  p->nranks = nranks;
  p->totalCount = totalCount;
  memcpy(&p->commOp, &commOp, sizeof(int)); // enum bits as they came from the caller
  memcpy(&p->redOp, &redOp, sizeof(int));
  int ncl = 0;
  for (int r = 0; r < nranks; r++) {
    if (clusterIds[r] < 0 || clusterIds[r] >= nranks) { delete p; return flagcxInvalidArgument; }
    if (clusterIds[r] + 1 > ncl) ncl = clusterIds[r] + 1;
  }
  p->clusterOf.assign(clusterIds, clusterIds + nranks);
  p->isInter.resize(nranks);
  p->clusterRanks.resize(ncl);
  p->clusterInterRanks.resize(ncl);
  p->homoRank.assign(nranks, -1);
  p->homoInterRank.assign(nranks, -1);
  for (int r = 0; r < nranks; r++) {
    const int cl = clusterIds[r];
    p->isInter[r] = isInterRank ? (isInterRank[r] != 0) : 1;
    p->homoRank[r] = (int)p->clusterRanks[cl].size();
    p->clusterRanks[cl].push_back(r);
    if (p->isInter[r]) {
      p->homoInterRank[r] = (int)p->clusterInterRanks[cl].size();
      p->clusterInterRanks[cl].push_back(r);
    }
  }
  // multiNic_ / eachNicPerRank_ of the planner's constructor (c2c_algo.cc:636-672)
  const bool reduceType = p->commOp == flagcxCommOpAllReduce || p->commOp == flagcxCommOpReduceScatter ||
                          p->commOp == flagcxCommOpReduce;
  p->multiNic = reduceType ? 1 : 0;
  p->eachNicPerRank = 1;
  for (int cl = 0; cl < ncl; cl++) {
    const size_t inter = p->clusterInterRanks[cl].size();
    if (reduceType && inter == 1) p->multiNic = 0;
    if (!reduceType && inter != 1) p->multiNic = 1;
    if (inter != p->clusterRanks[cl].size()) p->eachNicPerRank = 0;
  }
  for (int cl = 0; cl < ncl; cl++)
    if (p->clusterInterRanks[cl].size() > totalCount) p->multiNic = 0;
  p->ranks.resize(nranks);
  *plan = p;
  return flagcxSuccess;
  } catch (...) {
    delete p;
    return flagcxSystemError;
  }
}

// Number of chunks of plan documents that carry no <nChunks> (those written by
// flagcx/tools/algorithm.py); offsets and counts of a document are in units of
// totalCount / nChunks elements (c2c_algo.cc:989).
flagcxResult_t flagcxLocalPlanSetChunks(flagcxLocalPlan *plan, size_t nchunks) {
  if (!plan || nchunks == 0) return flagcxInvalidArgument;
  plan->defaultChunks = nchunks;
  return flagcxSuccess;
}

// Counts and displacements (in elements) of an AlltoAllv: four nranks x nranks matrices,
// row r = the arrays rank r passes to flagcxC2cPlanner::execute (c2c_algo.cc:2042-2046).
// The hetero functions of the plan carry the cross-cluster pieces themselves
// (c2c_algo.cc:1618-1630); the homo function reads these for the pieces inside a cluster.
flagcxResult_t flagcxLocalPlanSetAlltoAllv(flagcxLocalPlan *p, const size_t *sendCounts, const size_t *sDispls,
                                           const size_t *recvCounts, const size_t *rDispls) {
  if (!p) return flagcxInvalidArgument;
  // c2c_algo.cc:2083-2089
  if (!sendCounts || !sDispls || !recvCounts || !rDispls)
    return planFail(p, flagcxInvalidArgument, "sendrecv counts and displacements need to be set for AlltoAllv%s", "");
  const size_t n = (size_t)p->nranks * (size_t)p->nranks;
  try {
    p->sendCounts.assign(sendCounts, sendCounts + n);
    p->sDispls.assign(sDispls, sDispls + n);
    p->recvCounts.assign(recvCounts, recvCounts + n);
    p->rDispls.assign(rDispls, rDispls + n);
  } catch (...) {
    return planFail(p, flagcxSystemError, "out of memory%s", "");
  }
  return flagcxSuccess;
}

flagcxResult_t flagcxLocalPlanDestroy(flagcxLocalPlan *plan) {
  delete plan;
  return flagcxSuccess;
}

const char *flagcxLocalPlanGetLastError(flagcxLocalPlan *plan) { return plan ? plan->err : ""; }

// 0 sequential, 1 pipeline, 2 input (flagcxAlgorithm_t, c2c_algo.h:15-19): selects
// where execute() refreshes, for plans exported by a planner that was not in
// input mode.
flagcxResult_t flagcxLocalPlanSetAlgorithm(flagcxLocalPlan *plan, int algorithm) {
  if (!plan || algorithm < 0 || algorithm > 2) return flagcxInvalidArgument;
  plan->algorithm = algorithm;
  return flagcxSuccess;
}

// 1 (the default): a refresh records the ranges it clears and sums leave out the members
// that lie in them; 0: every refresh is a zero-fill and every collective reads all of its
// members, as the reference does.  The receive buffers end with the same bytes either way.
flagcxResult_t flagcxLocalPlanSetFused(flagcxLocalPlan *plan, int fused) {
  if (!plan || fused < 0 || fused > 1) return flagcxInvalidArgument;
  plan->fused = fused != 0;
  return flagcxSuccess;
}

// What the last flagcxLocalPlanExecute handed to the kernels: algorithmic bytes (2 B per
// copied byte, (k + 1) * n * size per k-input reduction, B per cleared byte) and launches.
flagcxResult_t flagcxLocalPlanGetTraffic(flagcxLocalPlan *plan, uint64_t *bytes, uint64_t *launches) {
  if (!plan) return flagcxInvalidArgument;
  if (bytes) *bytes = plan->lastBytes;
  if (launches) *launches = plan->lastLaunches;
  return flagcxSuccess;
}

static flagcxResult_t importXml(flagcxLocalPlan *p, const char *prefix);
static flagcxResult_t exportXml(flagcxLocalPlan *p, const char *prefix);

// Reads <prefix>_<rank>.xml for every rank (file naming of importXml, c2c_algo.cc:975-976).
flagcxResult_t flagcxLocalPlanImportXml(flagcxLocalPlan *p, const char *prefix) {
  if (!p || !prefix) return flagcxInvalidArgument;
  try {
    return importXml(p, prefix);
  } catch (...) {
    return planFail(p, flagcxSystemError, "out of memory while reading %s", prefix);
  }
}

static flagcxResult_t importXml(flagcxLocalPlan *p, const char *prefix) {
  for (int r = 0; r < p->nranks; r++) {
    char filename[512];
    snprintf(filename, sizeof(filename), "%s_%d.xml", prefix, r);
    FILE *f = fopen(filename, "r");
    if (!f) return planFail(p, flagcxInternalError, "cannot open %s", filename); // same code as the reference
    std::string text;
    char buf[4096];
    size_t got;
    while ((got = fread(buf, 1, sizeof(buf), f)) > 0) text.append(buf, got);
    fclose(f);
    size_t pos = text.find('<');
    Node rootNode;
    if (pos == std::string::npos || !parseNode(text, pos, rootNode) || rootNode.name != "FlagcxC2cPlanner")
      return planFail(p, flagcxInvalidArgument, "%s is not a FlagcxC2cPlanner document", filename);
    RankPlan &rp = p->ranks[r];
    // documents written by the reference's plan DSL carry no <nChunks>
    // (flagcx/tools/algorithm.py:160-181); exportXml always writes it (c2c_algo.cc:1058)
    rp.nchunks_ = rootNode.child("nChunks") ? rootNode.size("nChunks") : p->defaultChunks;
    if (rp.nchunks_ == 0 && !rootNode.child("nChunks"))
      return planFail(p, flagcxInvalidArgument, "%s has no <nChunks>: say how many chunks it counts in (flagcxLocalPlanSetChunks)",
                      filename);
    if (rp.nchunks_ == 0 || p->totalCount % rp.nchunks_)
      return planFail(p, flagcxInvalidArgument, "%s: nChunks must divide the total count", filename);
    static const char *const kSizes[] = {"nChunks", "start", "offset", "count", "totalCount", "sendOffset", "recvOffset"};
    if (const char *neg = rootNode.negativeSize(kSizes, 7)) {
      snprintf(p->err, sizeof(p->err), "%s: negative <%s>: offsets and counts are sizes", filename, neg);
      return flagcxInvalidArgument;
    }
    const size_t cs = p->totalCount / rp.nchunks_; // chunksize = totalCount_ / nchunks_ (c2c_algo.cc:989)
    rp.nSeqPreSteps_ = (int)rootNode.num("nSeqPreSteps");
    rp.nPipePreSteps_ = (int)rootNode.num("nPipePreSteps");
    rp.nSeqInterSteps_ = (int)rootNode.num("nSeqInterSteps");
    rp.nPipePostSteps_ = (int)rootNode.num("nPipePostSteps");
    rp.nSeqPostSteps_ = (int)rootNode.num("nSeqPostSteps");
    if (const Node *rf = rootNode.child("RefreshFunc")) {
      rp.refreshFunc_.bufftype_ = (int)rf->num("buffType", -1);
      rp.refreshFunc_.start_ = rf->size("start") * cs;
      rp.refreshFunc_.offset_ = rf->size("offset") * cs;
      rp.refreshFunc_.count_ = rf->size("count") * cs;
      rp.refreshFunc_.totalCount_ = rf->size("totalCount") * cs;
      rp.refreshFunc_.redOp_ = (int)rf->num("redOp");
    }
    homoSteps(rootNode.child("PreHomoFuncSteps"), cs, rp.preHomoFuncSteps_);
    heteroSteps(rootNode.child("HeteroFuncSteps"), cs, rp.heteroFuncSteps_);
    homoSteps(rootNode.child("HomoInterFuncSteps"), cs, rp.homoInterFuncSteps_);
    homoSteps(rootNode.child("PostHomoFuncSteps"), cs, rp.postHomoFuncSteps_);
    // the executor indexes the tables by these counts
    if ((int)rp.preHomoFuncSteps_.size() < rp.nSeqPreSteps_ + rp.nPipePreSteps_ ||
        (int)rp.heteroFuncSteps_.size() < rp.nPipePreSteps_ + rp.nSeqInterSteps_ + rp.nPipePostSteps_ ||
        (int)rp.postHomoFuncSteps_.size() < rp.nPipePostSteps_ + rp.nSeqPostSteps_)
      return planFail(p, flagcxInvalidArgument, "%s: step tables shorter than the step counts", filename);
    rp.homoInterFuncSteps_.resize(rp.heteroFuncSteps_.size());
  }
  for (int r = 1; r < p->nranks; r++) {
    const RankPlan &a = p->ranks[0], &b = p->ranks[r];
    if (a.nSeqPreSteps_ != b.nSeqPreSteps_ || a.nPipePreSteps_ != b.nPipePreSteps_ ||
        a.nSeqInterSteps_ != b.nSeqInterSteps_ || a.nPipePostSteps_ != b.nPipePostSteps_ ||
        a.nSeqPostSteps_ != b.nSeqPostSteps_)
      return planFail(p, flagcxInvalidUsage, "ranks disagree on the step counts%s", "");
  }
  p->loaded = true;
  return flagcxSuccess;
}

// Writes <prefix>_<rank>.xml in the layout of exportXml (c2c_algo.cc:1050-1087).
flagcxResult_t flagcxLocalPlanExportXml(flagcxLocalPlan *p, const char *prefix) {
  if (!p || !prefix || !p->loaded) return flagcxInvalidArgument;
  try {
    return exportXml(p, prefix);
  } catch (...) {
    return planFail(p, flagcxSystemError, "out of memory while writing %s", prefix);
  }
}

static flagcxResult_t exportXml(flagcxLocalPlan *p, const char *prefix) {
  for (int r = 0; r < p->nranks; r++) {
    char filename[512];
    snprintf(filename, sizeof(filename), "%s_%d.xml", prefix, r);
    FILE *f = fopen(filename, "w");
    if (!f) return planFail(p, flagcxInternalError, "cannot open %s", filename);
    const RankPlan &rp = p->ranks[r];
    const size_t cs = p->totalCount / rp.nchunks_;
    fprintf(f, "<FlagcxC2cPlanner>\n");
    fprintf(f, "  <nChunks>%zu</nChunks>\n", rp.nchunks_);
    fprintf(f, "  <nSeqPreSteps>%d</nSeqPreSteps>\n", rp.nSeqPreSteps_);
    fprintf(f, "  <nPipePreSteps>%d</nPipePreSteps>\n", rp.nPipePreSteps_);
    fprintf(f, "  <nSeqInterSteps>%d</nSeqInterSteps>\n", rp.nSeqInterSteps_);
    fprintf(f, "  <nPipePostSteps>%d</nPipePostSteps>\n", rp.nPipePostSteps_);
    fprintf(f, "  <nSeqPostSteps>%d</nSeqPostSteps>\n", rp.nSeqPostSteps_);
    fprintf(f, "  <RefreshFunc>\n");
    fprintf(f, "    <buffType>%d</buffType>\n", rp.refreshFunc_.bufftype_);
    fprintf(f, "    <start>%zu</start>\n", rp.refreshFunc_.start_ / cs);
    fprintf(f, "    <offset>%zu</offset>\n", rp.refreshFunc_.offset_ / cs);
    fprintf(f, "    <count>%zu</count>\n", rp.refreshFunc_.count_ / cs);
    fprintf(f, "    <totalCount>%zu</totalCount>\n", rp.refreshFunc_.totalCount_ / cs);
    fprintf(f, "    <redOp>%d</redOp>\n", rp.refreshFunc_.redOp_);
    fprintf(f, "  </RefreshFunc>\n");
    writeHomoSteps(f, "PreHomoFuncSteps", rp.preHomoFuncSteps_, cs);
    fprintf(f, "  <HeteroFuncSteps>\n");
    for (auto &step : rp.heteroFuncSteps_) {
      if (step.empty()) { fprintf(f, "    <Step/>\n"); continue; }
      fprintf(f, "    <Step>\n");
      for (auto &h : step) {
        fprintf(f, "      <HeteroFunc>\n");
        for (auto &o : h.p2pOps_) {
          fprintf(f, "        <P2pOp>\n");
          fprintf(f, "          <rank>%d</rank>\n", o.rank_);
          fprintf(f, "          <peerRank>%d</peerRank>\n", o.peerRank_);
          fprintf(f, "          <offset>%zu</offset>\n", o.offset_ / cs);
          fprintf(f, "          <count>%zu</count>\n", o.count_ / cs);
          fprintf(f, "          <isRecv>%d</isRecv>\n", o.isRecv_);
          fprintf(f, "        </P2pOp>\n");
        }
        fprintf(f, "      </HeteroFunc>\n");
      }
      fprintf(f, "    </Step>\n");
    }
    fprintf(f, "  </HeteroFuncSteps>\n");
    writeHomoSteps(f, "HomoInterFuncSteps", rp.homoInterFuncSteps_, cs);
    writeHomoSteps(f, "PostHomoFuncSteps", rp.postHomoFuncSteps_, cs);
    fprintf(f, "</FlagcxC2cPlanner>\n");
    fclose(f);
  }
  return flagcxSuccess;
}

// sendbuffs / recvbuffs / scratchbuffs: host arrays with one device pointer per
// rank (scratchbuffs, or entries of it, may be NULL for ranks that need none).
flagcxResult_t flagcxLocalPlanExecute(flagcxLocalPlan *p, const void *const *sendbuffs, void *const *recvbuffs,
                                      void *const *scratchbuffs, flagcxDataType_t datatype, int root,
                                      flagcxStream_t stream) {
  if (!p || !sendbuffs || !recvbuffs) return flagcxInvalidArgument;
  try {
    if (!p->loaded) return planFail(p, flagcxInvalidUsage, "no plan imported%s", "");
    // redOp validation of flagcxC2cPlanner::execute (c2c_algo.cc:2047-2053)
    if (p->redOp != flagcxRedNoOp && p->redOp != flagcxSum && p->redOp != flagcxMax && p->redOp != flagcxMin)
      return planFail(p, flagcxNotSupported, "Unsupported reduction operation %s%lld", "", p->redOp);
    if (!flagcxLocalGetDataTypeSize(datatype)) return planFail(p, flagcxInvalidArgument, "unsupported data type%s", "");
    for (int r = 0; r < p->nranks; r++)
      if (!sendbuffs[r] || !recvbuffs[r]) return planFail(p, flagcxInvalidArgument, "rank %s%lld has a NULL buffer", "", r);
    // the call's temporaries: one block, kept by the plan, released as a whole when the call ends
    // (declared before the executor, so that the executor's containers go first)
    if (p->arena.block.empty()) p->arena.block.resize(1 << 20);
    struct Scope {
      Arena *a;
      explicit Scope(Arena *arena) : a(arena) { tlsArena = a; }
      ~Scope() {
        tlsArena = nullptr;
        a->reset();
      }
    };
    Scope scope(&p->arena);
    Exec x;
    x.p = p;
    x.send = sendbuffs;
    x.recv = recvbuffs;
    x.scratch = scratchbuffs;
    x.dt = datatype;
    x.ts = flagcxLocalGetDataTypeSize(datatype);
    x.stream = stream;
    x.fused = p->fused;
    // what the homo functions get as root: the root's rank inside its cluster (c2c_algo.cc:2147,2170)
    x.homoRoot = (root >= 0 && root < p->nranks) ? p->homoRank[root] : root;
    // Staging buffers of the hetero functions.  The reference allocates a scratch buffer for a
    // ReduceScatter, a Scatter and on the non-root ranks of a Gather, and nowhere else
    // (c2c_algo.cc:2121-2129); where it does, hetero receives land there, everywhere else in
    // recvbuff (c2c_algo.cc:2131-2137).  A scratch pointer handed over for a rank that has none
    // in the reference is only what functions that name scratch explicitly get.
    x.ownsScratch.assign(p->nranks, 0);
    x.recvTmp.resize(p->nranks);
    x.sendTmp.resize(p->nranks);
    for (int r = 0; r < p->nranks; r++) {
      x.ownsScratch[r] = p->commOp == flagcxCommOpReduceScatter || p->commOp == flagcxCommOpScatter ||
                         (p->commOp == flagcxCommOpGather && r != root);
      char *scratch = scratchbuffs ? (char *)scratchbuffs[r] : nullptr;
      // (a plan that never stages anything there runs without one; what needs it says so when it gets there)
      x.recvTmp[r] = x.ownsScratch[r] ? scratch : (char *)recvbuffs[r];
      const bool fromSend = p->commOp == flagcxCommOpAlltoAll || p->commOp == flagcxCommOpAlltoAllv ||
                            (p->commOp == flagcxCommOpScatter && r == root) ||
                            (p->commOp == flagcxCommOpAllGather && p->eachNicPerRank && p->multiNic);
      x.sendTmp[r] = fromSend ? (char *)const_cast<void *>(sendbuffs[r]) : x.recvTmp[r];
    }
    const flagcxResult_t res = x.run();
    p->lastBytes = x.bytes;
    p->lastLaunches = x.launches;
    return res;
  } catch (...) {
    return planFail(p, flagcxSystemError, "out of memory while replaying the plan%s", "");
  }
}

} // extern "C"
#pragma GCC visibility pop
