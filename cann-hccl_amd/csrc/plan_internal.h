// What the planner's translation units share and nobody else sees: the virtual program the schedules are laid out in
// (plan_schedules.cc), its lowering to the caller's buffers and the symbolic executor that checks both and yields the
// reduction expression of every output range (plan_lower.cc), the fuser that turns those expressions into single-pass
// items (plan_fuse.cc).  plan.cc strings them together (BuildPlan); plan_template.cc derives plans from earlier ones.
#ifndef HCCL_AMD_PLAN_INTERNAL_H
#define HCCL_AMD_PLAN_INTERNAL_H

#include "plan.h"

#include <algorithm>
#include <cstdlib>
#include <map>
#include <sstream>
#include <string>
#include <tuple>
#include <utility>
#include <vector>

namespace hcclamd {
namespace planner {

inline uint64_t RoundUpTo(uint64_t v, uint64_t d) { return d == 0 ? v : (v + d - 1) / d * d; }
inline uint32_t Mod(int64_t v, uint32_t p) { int64_t m = v % static_cast<int64_t>(p); return static_cast<uint32_t>(m < 0 ? m + p : m); }

inline Ref MkRef(uint32_t rank, uint8_t buf, uint64_t off)
{
    Ref r;
    r.rank = rank;
    r.buf = buf;
    r.off = off;
    return r;
}

// ---- virtual program ----------------------------------------------------------------------------
// In the virtual program BUF_SEND names the schedule's input buffer (the reference's CCL-in copy,
// which the schedule may overwrite) and BUF_RECV its output buffer.
struct VProgram {
    std::vector<Phase> phases;
    std::vector<uint64_t> inBytes, outBytes;
    // Library-owned workspace a schedule addresses as input-buffer offsets [inBytes[r], inBytes[r] + workBytes[r])
    // (empty = none): it is only read after it was written, so it lives in scratch.
    std::vector<uint64_t> workBytes;
    // While a schedule is laid out for a sub-communicator: its ranks (local index -> rank of the whole
    // group; empty = identity) and the phase its own phase 0 stands for.
    std::vector<uint32_t> rankMap;
    size_t phaseBase = 0;
    // A schedule that only carries blocks from send buffers to receive buffers may list them here whole, grouped by
    // receiving rank (the phases may move a block in pieces): the planner's short cut for such programs starts here.
    struct Block {
        uint64_t dstOff, srcOff, bytes;
        uint32_t dstRank, srcRank;
    };
    std::vector<Block> blocks;
};

// plan_schedules.cc: lays the request's schedule out as the reference runs it.  0, or 1 with *err set.
int BuildVirtual(const PlanRequest &rq, VProgram *vp, std::string *err);

// plan_lower.cc
// home: where writes to the virtual input buffer go (BUF_RECV or BUF_SCRATCH); stage: copy the send buffers to scratch first.
void Lower(const VProgram &vp, const PlanRequest &rq, uint8_t home, bool stage, std::vector<Phase> *out);

// ---- symbolic execution -----------------------------------------------------------------------------
struct ENode {
    bool red = false;
    int a = -1, b = -1;
    uint64_t da = 0, db = 0;
    Ref leaf;
};
struct Region {
    uint64_t len = 0;
    int expr = -1;
    uint64_t delta = 0;
};
struct Piece {
    uint64_t rel, len;
    int expr;
    uint64_t delta;
};

// Gives equal expressions equal numbers.  The "shape" of an expression is its tree with every leaf
// offset taken relative to the offset of its leftmost leaf, so that one shape number plus that
// leftmost offset identifies the expression at any position.  One interner serves all the symbolic
// runs of a planning pass, which makes shape numbers comparable between them.
struct Interner {
    struct Key {
        int kind, a, b;
        int64_t diff;
        bool operator==(const Key &o) const { return kind == o.kind && a == o.a && b == o.b && diff == o.diff; }
    };
    struct Hash {
        size_t operator()(const Key &k) const
        {
            uint64_t h = 0x9e3779b97f4a7c15ull;
            for (uint64_t v : {uint64_t(k.kind), uint64_t(uint32_t(k.a)), uint64_t(uint32_t(k.b)), uint64_t(k.diff)}) {
                h ^= v + 0x9e3779b97f4a7c15ull + (h << 6) + (h >> 2);
            }
            return size_t(h);
        }
    };
    std::unordered_map<Key, int, Hash> ids;
    int Get(int kind, int a, int b, int64_t diff)
    {
        Key k{kind, a, b, diff};
        auto it = ids.find(k);
        if (it != ids.end()) {
            return it->second;
        }
        int id = int(ids.size());
        ids.emplace(k, id);
        return id;
    }
};

struct Sym {
    Interner *in = nullptr;
    mutable std::vector<int> shapeOf;        // per node, -1 = not computed yet
    mutable std::vector<int64_t> baseOf;     // offset of the node's leftmost leaf at delta 0
    std::vector<ENode> nodes;
    std::vector<std::map<uint64_t, Region>> mem;   // per (rank, buffer): index rank * 3 + buffer, grown on demand
    std::vector<uint8_t> alias;
    std::string err;

    size_t Key(const Ref &r) const
    {
        uint8_t b = r.buf;
        if (b == BUF_SEND && r.rank < alias.size() && alias[r.rank]) {
            b = BUF_RECV;
        }
        return size_t(r.rank) * 3 + b;
    }
    std::map<uint64_t, Region> &Mem(size_t key)
    {
        if (mem.size() <= key) {
            mem.resize(key + 1);
        }
        return mem[key];
    }
    void Init(uint32_t rank, uint64_t bytes)
    {
        if (bytes == 0) {
            return;
        }
        ENode n;
        n.leaf = MkRef(rank, BUF_SEND, 0);
        nodes.push_back(n);
        Region rg;
        rg.len = bytes;
        rg.expr = int(nodes.size()) - 1;
        Mem(Key(MkRef(rank, BUF_SEND, 0)))[0] = rg;
    }
    bool Read(const Ref &ref, uint64_t len, std::vector<Piece> *out)
    {
        const size_t key = Key(ref);
        uint64_t pos = ref.off, end = ref.off + len;
        if (key < mem.size()) {
            auto &m = mem[key];
            auto it = m.upper_bound(pos);
            if (it != m.begin()) {
                --it;
            }
            for (; it != m.end() && it->first < end && pos < end; ++it) {
                uint64_t rb = it->first, re = it->first + it->second.len;
                if (re <= pos) {
                    continue;
                }
                if (rb > pos) {
                    break;
                }
                uint64_t take = std::min(re, end) - pos;
                out->push_back(Piece{pos - ref.off, take, it->second.expr, it->second.delta + (pos - rb)});
                pos += take;
            }
        }
        if (pos < end) {
            std::ostringstream os;
            os << "read of unwritten memory: rank " << ref.rank << " buf " << int(ref.buf) << " offset " << pos;
            err = os.str();
            return false;
        }
        return true;
    }
    void Write(const Ref &ref, const std::vector<Piece> &pieces, uint64_t len)
    {
        auto &m = Mem(Key(ref));
        uint64_t b = ref.off, e = ref.off + len;
        auto it = m.upper_bound(b);
        if (it != m.begin()) {
            --it;
        }
        std::vector<std::pair<uint64_t, Region>> keep;
        while (it != m.end() && it->first < e) {
            uint64_t rb = it->first, re = it->first + it->second.len;
            if (re <= b) {
                ++it;
                continue;
            }
            if (rb < b) {
                Region l = it->second;
                l.len = b - rb;
                keep.emplace_back(rb, l);
            }
            if (re > e) {
                Region r = it->second;
                r.len = re - e;
                r.delta += e - rb;
                keep.emplace_back(e, r);
            }
            it = m.erase(it);
        }
        for (auto &k : keep) {
            m[k.first] = k.second;
        }
        for (const Piece &pc : pieces) {
            Region rg;
            rg.len = pc.len;
            rg.expr = pc.expr;
            rg.delta = pc.delta;
            m[b + pc.rel] = rg;
        }
    }
    bool Run(const std::vector<Phase> &phases)
    {
        for (const Phase &ph : phases) {
            std::vector<std::tuple<Ref, std::vector<Piece>, uint64_t>> writes;
            writes.reserve(ph.steps.size());
            std::vector<Piece> pa, pb, res;    // reused from step to step
            for (const Step &s : ph.steps) {
                pa.clear();
                pb.clear();
                res.clear();
                if (!Read(s.a, s.bytes, &pa)) {
                    return false;
                }
                if (!s.reduce) {
                    res.swap(pa);
                } else {
                    if (!Read(s.b, s.bytes, &pb)) {
                        return false;
                    }
                    size_t i = 0, j = 0;
                    uint64_t pos = 0;
                    while (pos < s.bytes) {
                        const Piece &x = pa[i], &y = pb[j];
                        uint64_t end = std::min(x.rel + x.len, y.rel + y.len);
                        ENode n;
                        n.red = true;
                        n.a = x.expr;
                        n.da = x.delta + (pos - x.rel);
                        n.b = y.expr;
                        n.db = y.delta + (pos - y.rel);
                        nodes.push_back(n);
                        res.push_back(Piece{pos, end - pos, int(nodes.size()) - 1, 0});
                        pos = end;
                        if (x.rel + x.len == end) {
                            i++;
                        }
                        if (y.rel + y.len == end) {
                            j++;
                        }
                    }
                }
                writes.emplace_back(s.dst, res, s.bytes);
            }
            for (auto &w : writes) {
                Write(std::get<0>(w), std::get<1>(w), std::get<2>(w));
            }
        }
        return true;
    }
    // Shape number of expression e and the offset of its leftmost leaf (at delta 0), memoised.
    void Shape(int e, int *shape, int64_t *base) const
    {
        if (shapeOf.size() < nodes.size()) {
            shapeOf.resize(nodes.size(), -1);
            baseOf.resize(nodes.size(), 0);
        }
        if (shapeOf[e] < 0) {
            const ENode &n = nodes[e];
            if (!n.red) {
                shapeOf[e] = in->Get(0, int(n.leaf.rank), int(n.leaf.buf), 0);
                baseOf[e] = int64_t(n.leaf.off);
            } else {
                int sa, sb;
                int64_t ba, bb;
                Shape(n.a, &sa, &ba);
                Shape(n.b, &sb, &bb);
                ba += int64_t(n.da);
                bb += int64_t(n.db);
                shapeOf[e] = in->Get(1, sa, sb, bb - ba);
                baseOf[e] = ba;
            }
        }
        *shape = shapeOf[e];
        *base = baseOf[e];
    }
};

// Final contents of every receive buffer as maximal ranges of one expression each.
struct OutRange {
    uint32_t rank;
    uint64_t start, len;
    int expr;
    uint64_t delta;
    int shape;           // position-independent form: shape number ...
    int64_t rel;         // ... and leftmost source offset minus the range's own start
    int64_t abs;         // leftmost source offset
};
std::vector<OutRange> Outputs(const Sym &sym, uint32_t p);
std::vector<uint64_t> OutputSignature(const Sym &sym, const std::vector<OutRange> &outs, const std::vector<uint8_t> &alias);

// plan_fuse.cc
bool BuildFused(const Sym &sym, const std::vector<OutRange> &outs, const PlanRequest &rq, std::vector<FusedItem> *items);
bool PhaseIsHazardFree(const Phase &ph, const std::vector<uint8_t> &alias, std::string *err);

}  // namespace planner
}  // namespace hcclamd

#endif
