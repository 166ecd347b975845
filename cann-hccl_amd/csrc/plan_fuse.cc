// From the reduction expression of an output range to a fused item (copy, chain, tree, stack program), and the check
// that a phase of steps has no hazard inside it.
#include "plan_internal.h"

namespace hcclamd {
namespace planner {

namespace {

Ref LeafRef(const Sym &sym, int e, uint64_t delta)
{
    Ref r = sym.nodes[e].leaf;
    r.off += delta;
    return r;
}

bool AsChain(const Sym &sym, int e, uint64_t delta, FusedItem *item)
{
    // walk from the outermost combine to the innermost; every level must have a leaf operand
    std::vector<Ref> rev;
    std::vector<uint8_t> revLeft;
    for (;;) {
        const ENode &n = sym.nodes[e];
        if (!n.red) {
            return false;
        }
        bool la = !sym.nodes[n.a].red, lb = !sym.nodes[n.b].red;
        if (la && lb) {
            rev.push_back(LeafRef(sym, n.b, n.db + delta));
            revLeft.push_back(1);                 // acc (+) b with acc = a
            rev.push_back(LeafRef(sym, n.a, n.da + delta));
            revLeft.push_back(0);
            break;
        }
        if (la) {
            rev.push_back(LeafRef(sym, n.a, n.da + delta));
            revLeft.push_back(0);                 // a (+) acc
            uint64_t nd = n.db + delta;
            e = n.b;
            delta = nd;
        } else if (lb) {
            rev.push_back(LeafRef(sym, n.b, n.db + delta));
            revLeft.push_back(1);                 // acc (+) b
            uint64_t nd = n.da + delta;
            e = n.a;
            delta = nd;
        } else {
            return false;
        }
    }
    item->kind = FK_CHAIN;
    item->src.assign(rev.rbegin(), rev.rend());
    item->accLeft.assign(revLeft.rbegin(), revLeft.rend());
    item->srcValid.assign(item->src.size(), 1);
    return true;
}

bool MatchTree(const Sym &sym, int e, uint64_t delta, uint32_t depth, FusedItem *item)
{
    const ENode &n = sym.nodes[e];
    if (depth == 0) {
        if (!n.red) {
            item->src.push_back(LeafRef(sym, e, delta));
            item->srcValid.push_back(1);
            item->src.push_back(Ref());
            item->srcValid.push_back(0);
            return true;
        }
        if (!sym.nodes[n.a].red && !sym.nodes[n.b].red) {
            item->src.push_back(LeafRef(sym, n.a, n.da + delta));
            item->srcValid.push_back(1);
            item->src.push_back(LeafRef(sym, n.b, n.db + delta));
            item->srcValid.push_back(1);
            return true;
        }
        return false;
    }
    if (!n.red) {
        return false;
    }
    return MatchTree(sym, n.a, n.da + delta, depth - 1, item) && MatchTree(sym, n.b, n.db + delta, depth - 1, item);
}

bool AsTree(const Sym &sym, int e, uint64_t delta, FusedItem *item)
{
    for (uint32_t depth = 1; depth <= 5; depth++) {
        FusedItem t;
        if (MatchTree(sym, e, delta, depth, &t)) {
            item->kind = FK_TREE;
            item->src = t.src;
            item->srcValid = t.srcValid;
            item->nleaf = 1u << depth;
            return true;
        }
    }
    return false;
}

// Any expression as a stack program.  Of the two operands of a combine the one that needs the deeper
// stack is evaluated first (the classic register-need numbering), which keeps chains at depth 2 and a
// tree of 2^k equal parts at k + 1 whatever way they lean.
struct StackForm {
    const Sym &sym;
    std::unordered_map<int, uint32_t> need, leaves;
    explicit StackForm(const Sym &s) : sym(s) {}
    void Measure(int e)
    {
        if (need.count(e)) {
            return;
        }
        const ENode &n = sym.nodes[e];
        if (!n.red) {
            need[e] = 1;
            leaves[e] = 1;
            return;
        }
        Measure(n.a);
        Measure(n.b);
        uint32_t na = need[n.a], nb = need[n.b];
        need[e] = na == nb ? na + 1 : std::max(na, nb);
        leaves[e] = std::min<uint32_t>(leaves[n.a] + leaves[n.b], 1u << 20);
    }
    void Emit(int e, uint64_t delta, FusedItem *item)
    {
        const ENode &n = sym.nodes[e];
        if (!n.red) {
            item->src.push_back(LeafRef(sym, e, delta));
            item->srcValid.push_back(1);
            item->ops.push_back(0);
            return;
        }
        const bool leftFirst = need[n.a] >= need[n.b];
        if (leftFirst) {
            Emit(n.a, n.da + delta, item);
            Emit(n.b, n.db + delta, item);
        } else {
            Emit(n.b, n.db + delta, item);
            Emit(n.a, n.da + delta, item);
        }
        uint16_t &op = item->ops.back();
        const uint32_t k = op & 7u;              // at most depth - 1 folds follow one push
        op = uint16_t((op & ~7u) | (k + 1) | (leftFirst ? (1u << (8 + k)) : 0u));
    }
};

bool AsStack(const Sym &sym, int e, uint64_t delta, FusedItem *item)
{
    StackForm f(sym);
    f.Measure(e);
    if (f.need[e] > kStackDepth || f.leaves[e] > kStackMaxSrc) {
        return false;
    }
    item->kind = FK_STACK;
    item->nleaf = f.need[e];          // stack depth the program needs
    item->src.clear();
    item->srcValid.clear();
    item->ops.clear();
    f.Emit(e, delta, item);
    return true;
}

}  // namespace

bool BuildFused(const Sym &sym, const std::vector<OutRange> &outs, const PlanRequest &rq, std::vector<FusedItem> *items)
{
    std::map<std::tuple<uint64_t, int, int64_t>, size_t> index;   // (length, shape, leftmost source offset)
    for (const OutRange &o : outs) {
        auto key = std::make_tuple(o.len, o.shape, o.abs);
        auto it = index.find(key);
        if (it == index.end()) {
            FusedItem item;
            item.bytes = o.len;
            if (!sym.nodes[o.expr].red) {
                item.kind = FK_COPY;
                item.src.push_back(LeafRef(sym, o.expr, o.delta));
                item.srcValid.push_back(1);
            } else if (!AsChain(sym, o.expr, o.delta, &item) && !AsTree(sym, o.expr, o.delta, &item) &&
                       !AsStack(sym, o.expr, o.delta, &item)) {
                return false;
            }
            items->push_back(item);
            it = index.emplace(key, items->size() - 1).first;
        }
        (*items)[it->second].dst.push_back(MkRef(o.rank, BUF_RECV, o.start));
    }
    // A fused launch reads every source and writes every destination in one pass, so a destination
    // may share memory with a source only when it is the same range of the same item (each thread
    // then reads its bytes before it overwrites them).  Only aliased ranks can overlap.
    // Sources are ranges of send buffers and destinations ranges of receive buffers, so only ranks
    // whose two buffers are the same memory need the check.
    if (rq.alias.size() != rq.p) {
        return true;
    }
    struct Span {
        uint64_t off, end;
        size_t item;
    };
    std::vector<std::vector<Span>> srcOf(rq.p);
    for (size_t j = 0; j < items->size(); j++) {
        const FusedItem &it = (*items)[j];
        for (size_t k = 0; k < it.src.size(); k++) {
            const Ref &sr = it.src[k];
            if (it.srcValid[k] && sr.buf == BUF_SEND && rq.alias[sr.rank] && it.bytes) {
                srcOf[sr.rank].push_back(Span{sr.off, sr.off + it.bytes, j});
            }
        }
    }
    std::vector<std::vector<uint64_t>> maxEnd(rq.p);   // running maximum of Span::end in offset order
    for (uint32_t r = 0; r < rq.p; r++) {
        std::sort(srcOf[r].begin(), srcOf[r].end(), [](const Span &x, const Span &y) { return x.off < y.off; });
        maxEnd[r].resize(srcOf[r].size());
        uint64_t m = 0;
        for (size_t i = 0; i < srcOf[r].size(); i++) {
            m = std::max(m, srcOf[r][i].end);
            maxEnd[r][i] = m;
        }
    }
    for (size_t i = 0; i < items->size(); i++) {
        const uint64_t len = (*items)[i].bytes;
        for (const Ref &d : (*items)[i].dst) {
            if (d.buf != BUF_RECV || !rq.alias[d.rank] || len == 0) {
                continue;
            }
            const std::vector<Span> &v = srcOf[d.rank];
            // candidates start below the destination's end; walk down while anything can still reach it
            size_t hi = std::lower_bound(v.begin(), v.end(), d.off + len, [](const Span &x, uint64_t e) { return x.off < e; }) -
                v.begin();
            for (size_t k = hi; k-- > 0 && maxEnd[d.rank][k] > d.off;) {
                if (v[k].end > d.off && !(v[k].item == i && v[k].off == d.off)) {
                    return false;
                }
            }
        }
    }
    return true;
}

// Hazard check of one phase: a destination may not overlap any other step's operands or destination.
bool PhaseIsHazardFree(const Phase &ph, const std::vector<uint8_t> &alias, std::string *err)
{
    struct Acc { uint32_t rank; uint8_t buf; uint64_t off, len; size_t step; bool write; };
    std::vector<Acc> acc;
    acc.reserve(ph.steps.size() * 3);
    auto phys = [&](const Ref &r) { return (r.buf == BUF_SEND && r.rank < alias.size() && alias[r.rank]) ? uint8_t(BUF_RECV) : r.buf; };
    for (size_t i = 0; i < ph.steps.size(); i++) {
        const Step &s = ph.steps[i];
        acc.push_back(Acc{s.dst.rank, phys(s.dst), s.dst.off, s.bytes, i, true});
        acc.push_back(Acc{s.a.rank, phys(s.a), s.a.off, s.bytes, i, false});
        if (s.reduce) {
            acc.push_back(Acc{s.b.rank, phys(s.b), s.b.off, s.bytes, i, false});
        }
    }
    std::sort(acc.begin(), acc.end(), [](const Acc &x, const Acc &y) {
        return std::tie(x.rank, x.buf, x.off) < std::tie(y.rank, y.buf, y.off);
    });
    for (size_t i = 0; i < acc.size(); i++) {
        for (size_t j = i + 1; j < acc.size(); j++) {
            if (acc[j].rank != acc[i].rank || acc[j].buf != acc[i].buf || acc[j].off >= acc[i].off + acc[i].len) {
                break;
            }
            if (!acc[i].write && !acc[j].write) {
                continue;
            }
            if (acc[i].step == acc[j].step && acc[i].off == acc[j].off) {
                continue;   // a step may update its own operand in place
            }
            std::ostringstream os;
            os << "hazard inside a phase at rank " << acc[i].rank << " buf " << int(acc[i].buf) << " offset " << acc[j].off;
            *err = os.str();
            return false;
        }
    }
    return true;
}

}  // namespace planner
}  // namespace hcclamd
