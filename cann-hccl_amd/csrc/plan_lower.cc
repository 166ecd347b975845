// Lowering of a virtual program to the caller's buffers, and the outputs of a symbolic run: which ranges of which
// buffers a program defines, and a signature that tells whether two programs define the same values.
#include "plan_internal.h"

namespace hcclamd {
namespace planner {

namespace {

// ---- interval set ---------------------------------------------------------------------------------
class RangeSet {
public:
    void Add(uint64_t b, uint64_t e)
    {
        if (b >= e) {
            return;
        }
        auto it = m_.upper_bound(b);
        if (it != m_.begin()) {
            auto pv = std::prev(it);
            if (pv->second >= b) {
                b = pv->first;
                e = std::max(e, pv->second);
                it = m_.erase(pv);
            }
        }
        while (it != m_.end() && it->first <= e) {
            e = std::max(e, it->second);
            it = m_.erase(it);
        }
        m_[b] = e;
    }
    // Boundaries of set membership strictly inside (b, e).
    void Cuts(uint64_t b, uint64_t e, std::vector<uint64_t> *out) const
    {
        for (auto it = m_.begin(); it != m_.end(); ++it) {
            if (it->first > b && it->first < e) {
                out->push_back(it->first);
            }
            if (it->second > b && it->second < e) {
                out->push_back(it->second);
            }
        }
    }
    bool Contains(uint64_t x) const
    {
        auto it = m_.upper_bound(x);
        if (it == m_.begin()) {
            return false;
        }
        --it;
        return x < it->second;
    }

private:
    std::map<uint64_t, uint64_t> m_;
};

}  // namespace

// ---- lowering -------------------------------------------------------------------------------------
// home: where writes to the virtual input buffer go (BUF_RECV or BUF_SCRATCH).
void Lower(const VProgram &vp, const PlanRequest &rq, uint8_t home, bool stage, std::vector<Phase> *out)
{
    uint32_t p = rq.p;
    std::vector<RangeSet> written(p);
    out->clear();
    if (stage) {
        Phase ph;
        for (uint32_t r = 0; r < p; r++) {
            if (vp.inBytes[r] == 0) {
                continue;
            }
            Step s;
            s.dst = MkRef(r, BUF_SCRATCH, 0);
            s.a = MkRef(r, BUF_SEND, 0);
            s.bytes = vp.inBytes[r];
            ph.steps.push_back(s);
            written[r].Add(0, vp.inBytes[r]);
        }
        if (!ph.steps.empty()) {
            out->push_back(ph);
        }
        home = BUF_SCRATCH;
    }
    for (const Phase &vph : vp.phases) {
        Phase ph;
        std::vector<std::tuple<uint32_t, uint64_t, uint64_t>> marks;
        for (const Step &vs : vph.steps) {
            std::vector<uint64_t> cuts;   // relative to the step start
            auto addCuts = [&](const Ref &ref) {
                if (ref.buf != BUF_SEND) {
                    return;
                }
                std::vector<uint64_t> abs;
                written[ref.rank].Cuts(ref.off, ref.off + vs.bytes, &abs);
                for (uint64_t c : abs) {
                    cuts.push_back(c - ref.off);
                }
            };
            addCuts(vs.a);
            if (vs.reduce) {
                addCuts(vs.b);
            }
            cuts.push_back(0);
            cuts.push_back(vs.bytes);
            std::sort(cuts.begin(), cuts.end());
            cuts.erase(std::unique(cuts.begin(), cuts.end()), cuts.end());
            for (size_t i = 0; i + 1 < cuts.size(); i++) {
                uint64_t d = cuts[i], n = cuts[i + 1] - cuts[i];
                auto mapRead = [&](const Ref &ref) {
                    if (ref.buf == BUF_RECV) {
                        return MkRef(ref.rank, BUF_RECV, ref.off + d);
                    }
                    bool w = written[ref.rank].Contains(ref.off + d);
                    return MkRef(ref.rank, w ? home : uint8_t(BUF_SEND), ref.off + d);
                };
                Step s;
                s.reduce = vs.reduce;
                s.bytes = n;
                s.a = mapRead(vs.a);
                if (vs.reduce) {
                    s.b = mapRead(vs.b);
                }
                s.dst = MkRef(vs.dst.rank, vs.dst.buf == BUF_SEND ? home : uint8_t(BUF_RECV), vs.dst.off + d);
                bool aliased = rq.alias.size() == p && rq.alias[s.dst.rank];
                auto same = [&](const Ref &x, const Ref &y) {
                    if (x.rank != y.rank || x.off != y.off) {
                        return false;
                    }
                    uint8_t bx = (aliased && x.buf == BUF_SEND) ? uint8_t(BUF_RECV) : x.buf;
                    uint8_t by = (aliased && y.buf == BUF_SEND) ? uint8_t(BUF_RECV) : y.buf;
                    return bx == by;
                };
                if (!s.reduce && same(s.dst, s.a)) {
                    continue;   // the data is already where it has to be
                }
                ph.steps.push_back(s);
            }
            if (vs.dst.buf == BUF_SEND) {
                marks.emplace_back(vs.dst.rank, vs.dst.off, vs.dst.off + vs.bytes);
            }
        }
        for (auto &m : marks) {
            written[std::get<0>(m)].Add(std::get<1>(m), std::get<2>(m));
        }
        if (!ph.steps.empty()) {
            // Order steps by destination offset: the tile that produced a range in one phase and the
            // tile that consumes it in the next then get the same index in both launches.
            std::stable_sort(ph.steps.begin(), ph.steps.end(),
                [](const Step &x, const Step &y) { return x.dst.off < y.dst.off; });
            out->push_back(ph);
        }
    }
}

std::vector<OutRange> Outputs(const Sym &sym, uint32_t p)
{
    std::vector<OutRange> v;
    for (uint32_t r = 0; r < p; r++) {
        const size_t key = size_t(r) * 3 + BUF_RECV;
        if (key >= sym.mem.size()) {
            continue;
        }
        for (auto &kv : sym.mem[key]) {
            OutRange o;
            o.rank = r;
            o.start = kv.first;
            o.len = kv.second.len;
            o.expr = kv.second.expr;
            o.delta = kv.second.delta;
            int64_t base;
            sym.Shape(o.expr, &o.shape, &base);
            o.abs = base + int64_t(o.delta);
            o.rel = o.abs - int64_t(o.start);
            if (!v.empty() && v.back().rank == r && v.back().start + v.back().len == o.start && v.back().shape == o.shape &&
                v.back().rel == o.rel) {
                v.back().len += o.len;   // continuation of the previous range
            } else {
                v.push_back(std::move(o));
            }
        }
    }
    return v;
}

// Numbers that identify the final receive-buffer contents independently of how ranges were split.
// Ranges of an in-place rank that still hold their original bytes (never written) are left out: the
// same memory seen as "send buffer" is not an output.
std::vector<uint64_t> OutputSignature(const Sym &sym, const std::vector<OutRange> &outs, const std::vector<uint8_t> &alias)
{
    std::vector<uint64_t> sig;
    sig.reserve(outs.size() * 5);
    for (const OutRange &o : outs) {
        const ENode &n = sym.nodes[o.expr];
        bool untouched = !n.red && n.leaf.rank == o.rank && n.leaf.buf == BUF_SEND && n.leaf.off + o.delta == o.start &&
            o.rank < alias.size() && alias[o.rank];
        if (untouched) {
            continue;
        }
        sig.push_back(o.rank);
        sig.push_back(o.start);
        sig.push_back(o.len);
        sig.push_back(uint64_t(o.shape));
        sig.push_back(uint64_t(o.rel));
    }
    return sig;
}

}  // namespace planner
}  // namespace hcclamd
