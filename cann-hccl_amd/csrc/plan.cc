// Planner implementation.  See plan.h for the reference interfaces this covers.
//
// Pipeline: (1) emit the schedule on "virtual" buffers the way the reference runs it on its CCL
// staging buffers (partial results accumulate in the input buffer); (2) lower to the caller's
// buffers without touching a send buffer that is not also the receive buffer: partials are homed in
// the receive buffer when it is large enough, else in scratch; (3) run the program symbolically to
// check it (no read of unwritten memory, lowered == virtual) and to derive, per output range, the
// reduction expression over the original inputs; (4) turn those expressions into fused items when
// they are copies, chains or perfect trees.
//
// The pieces: plan_schedules.cc (1), plan_lower.cc (2, 3), plan_fuse.cc (4), plan_template.cc (plans derived from
// earlier plans); this file holds the slice and chunk rules, the short cut for collectives that only move blocks,
// BuildPlan and the plan's JSON form.
#include "plan_internal.h"

namespace hcclamd {

using namespace planner;

namespace {

void JsonRef(std::ostringstream &os, const Ref &r)
{
    os << "[" << r.rank << "," << int(r.buf) << "," << r.off << "]";
}


}  // namespace

std::vector<Slice> RingSlicePlan(uint64_t total, uint32_t n, uint64_t align)
{
    std::vector<Slice> s(n);
    uint64_t per = RoundUpTo((total + n - 1) / n, align);
    uint64_t left = total;
    for (uint32_t i = 0; i < n; i++) {
        uint64_t cur = std::min(per, left);
        s[i].off = total - left;
        s[i].size = cur;
        left -= cur;
    }
    return s;
}

void HalvingDoublingShape(uint32_t p, uint32_t *block, uint32_t *part1)
{
    uint32_t b = 1;
    while (b * 2 <= p) {
        b *= 2;
    }
    *block = b;
    *part1 = 2 * (p - b);
}

std::vector<uint64_t> ChunkCounts(CollKind coll, uint64_t count, uint32_t unit, uint32_t p, uint64_t cclBytes,
    uint64_t align)
{
    std::vector<uint64_t> v;
    uint64_t per = (coll == COLL_ALLREDUCE) ? cclBytes / unit : cclBytes / p / align * align / unit;
    if (per == 0) {
        return v;
    }
    for (uint64_t left = count; left > 0;) {
        uint64_t cur = std::min(left, per);
        v.push_back(cur);
        left -= cur;
    }
    return v;
}

// An all-to-all-v, a scatter or a send / receive only moves blocks from send buffers to receive buffers: nothing is
// combined and nothing rests in a buffer on the way, so the step program is the virtual one and the fused form is one
// copy item per block.  What the general path verifies symbolically reduces to one interval check -- no two blocks
// land on the same bytes of a receive buffer.  This is what an all-to-all-v whose tables change on every call pays
// per call: tens of microseconds at 16 ranks instead of several hundred, and the difference grows with the square of
// the rank count.  HCCL_AMD_PLAN_VERIFY=1 in the environment sends every request the general way.
bool DirectCopyPlan(VProgram &vp, const PlanRequest &rq, const std::vector<uint8_t> &alias, Plan *plan)
{
    static const bool verifyAll = [] {
        const char *e = std::getenv("HCCL_AMD_PLAN_VERIFY");
        return e != nullptr && e[0] != '\0' && e[0] != '0';
    }();
    // A schedule with a workspace qualifies when it lists its whole blocks itself (the staged all-to-all-v: blocks rest
    // in the gathering rank's workspace between the two stages).
    // So does an all-gather that lists its blocks (the variable-count one): its steps pass blocks on from receive buffer
    // to receive buffer, which needs no lowering either, and its fused form is one item per rank's block with every
    // receive buffer as a destination.
    const bool viaWorkspace = !vp.workBytes.empty();
    const bool gathers = rq.coll == COLL_ALLGATHER && !vp.blocks.empty() && !viaWorkspace;
    if (verifyAll || rq.stageInput || (viaWorkspace && vp.blocks.empty()) ||
        (rq.coll != COLL_ALLTOALLV && rq.coll != COLL_SCATTER && rq.coll != COLL_SENDRECV && !gathers)) {
        return false;
    }
    for (uint8_t a : alias) {
        if (a) {
            return false;
        }
    }
    typedef VProgram::Block Block;
    uint64_t stepped = 0;
    auto inWorkspace = [&](const Ref &r) { return viaWorkspace && r.buf == BUF_SEND && r.off >= vp.inBytes[r.rank]; };
    for (const Phase &ph : vp.phases) {
        for (const Step &st : ph.steps) {
            if (st.reduce || !(st.a.buf == BUF_SEND || (gathers && st.a.buf == BUF_RECV)) || st.a.rank >= rq.p || st.dst.rank >= rq.p ||
                !(st.dst.buf == BUF_RECV || inWorkspace(st.dst))) {
                return false;
            }
            stepped += st.bytes;
        }
    }
    std::vector<Block> &blocks = vp.blocks;
    bool grouped = true;
    for (size_t i = 1; i < blocks.size() && grouped; i++) {
        grouped = blocks[i - 1].dstRank <= blocks[i].dstRank;
    }
    if (!grouped) {
        std::stable_sort(blocks.begin(), blocks.end(), [](const Block &x, const Block &y) { return x.dstRank < y.dstRank; });
    }
    if (blocks.empty()) {
        // no list of whole blocks: the steps are the blocks, those that continue one another joined
        for (const Phase &ph : vp.phases) {
            for (const Step &st : ph.steps) {
                blocks.push_back(Block{st.dst.off, st.a.off, st.bytes, st.dst.rank, st.a.rank});
            }
        }
        std::sort(blocks.begin(), blocks.end(), [](const Block &x, const Block &y) {
            return x.dstRank != y.dstRank ? x.dstRank < y.dstRank : x.dstOff < y.dstOff;
        });
        size_t kept = 0;
        for (size_t i = 0; i < blocks.size(); i++) {
            Block &last = blocks[kept ? kept - 1 : 0];
            if (kept && last.dstRank == blocks[i].dstRank && last.srcRank == blocks[i].srcRank &&
                blocks[i].dstOff == last.dstOff + last.bytes && blocks[i].srcOff == last.srcOff + last.bytes) {
                last.bytes += blocks[i].bytes;
            } else {
                blocks[kept++] = blocks[i];
            }
        }
        blocks.resize(kept);
    }
    // No two blocks may land on the same bytes.  Blocks of a rank usually come in rising order (packed receive
    // buffers): one pass; a rank whose blocks do not is sorted first.
    std::vector<std::pair<uint64_t, uint64_t>> spans;
    for (size_t i = 0; i < blocks.size();) {
        size_t j = i;
        bool rising = true;
        uint64_t end = 0;
        for (; j < blocks.size() && blocks[j].dstRank == blocks[i].dstRank; j++) {
            rising = rising && blocks[j].dstOff >= end;
            end = blocks[j].dstOff + blocks[j].bytes;
        }
        if (!rising) {
            spans.clear();
            for (size_t k = i; k < j; k++) {
                spans.emplace_back(blocks[k].dstOff, blocks[k].dstOff + blocks[k].bytes);
            }
            std::sort(spans.begin(), spans.end());
            for (size_t k = 1; k < spans.size(); k++) {
                if (spans[k - 1].second > spans[k].first) {
                    return false;   // overlapping destinations: the general path decides what that means
                }
            }
        }
        i = j;
    }
    if (gathers) {
        // every rank contributes one block, the same wherever it lands (checked before anything is handed over)
        std::vector<uint64_t> size(rq.p, 0);
        for (const Block &b : blocks) {
            if (b.srcOff != 0 || (size[b.srcRank] != 0 && size[b.srcRank] != b.bytes)) {
                return false;
            }
            size[b.srcRank] = b.bytes;
        }
    }
    uint64_t moved = 0;
    for (const Block &b : blocks) {
        moved += b.bytes;
    }
    plan->phases.clear();
    plan->phases.reserve(vp.phases.size());
    plan->scratchBytes = 0;
    for (Phase &vph : vp.phases) {
        if (vph.steps.empty()) {
            continue;
        }
        if (viaWorkspace) {
            // the workspace lies in the library's scratch buffer behind the rank's input, as the general lowering puts it
            for (Step &st : vph.steps) {
                if (inWorkspace(st.a)) {
                    st.a.buf = BUF_SCRATCH;
                }
                if (st.dst.buf == BUF_SEND) {
                    st.dst.buf = BUF_SCRATCH;
                }
            }
        }
        plan->phases.push_back(std::move(vph));
    }
    for (uint32_t r = 0; viaWorkspace && r < rq.p; r++) {
        plan->scratchBytes = std::max(plan->scratchBytes, vp.inBytes[r] + vp.workBytes[r]);
    }
    plan->stepRead = plan->stepWritten = stepped;
    plan->fusedRead = plan->fusedWritten = moved;
    if (gathers) {
        // one item per source block, read once, written to every rank that receives it (ranks in rising order)
        std::vector<int> itemOf(rq.p, -1);
        plan->fused.clear();
        plan->fusedRead = 0;
        for (const Block &b : blocks) {
            if (itemOf[b.srcRank] < 0) {
                itemOf[b.srcRank] = int(plan->fused.size());
                plan->fused.emplace_back();
                FusedItem &item = plan->fused.back();
                item.kind = FK_COPY;
                item.bytes = b.bytes;
                item.src.push_back(MkRef(b.srcRank, BUF_SEND, 0));
                item.srcValid.push_back(1);
                plan->fusedRead += b.bytes;
            }
            FusedItem &item = plan->fused[size_t(itemOf[b.srcRank])];
            item.dst.push_back(MkRef(b.dstRank, BUF_RECV, b.dstOff));
        }
        plan->fusedOk = true;
        return true;
    }
    // fused: a block that the schedule moved in pieces is one item again
    plan->fused.clear();
    plan->fused.reserve(blocks.size());
    for (const Block &b : blocks) {
        plan->fused.emplace_back();
        FusedItem &item = plan->fused.back();
        item.kind = FK_COPY;
        item.bytes = b.bytes;
        item.src.push_back(MkRef(b.srcRank, BUF_SEND, b.srcOff));
        item.srcValid.push_back(1);
        item.dst.push_back(MkRef(b.dstRank, BUF_RECV, b.dstOff));
    }
    plan->fusedOk = true;
    return true;
}

int BuildPlan(const PlanRequest &request, Plan *plan, std::string *err)
{
    if (request.p == 0 || request.unit == 0 || request.align == 0 || request.servers == 0 || request.p % request.servers != 0) {
        *err = "bad plan request";
        return 1;
    }
    if (request.nicMask != 0) {
        const int ports = __builtin_popcount(request.nicMask & 0xffu);
        const bool twoLevel = request.coll == COLL_REDUCESCATTER && request.servers > 1 && request.p == request.servers * 8 &&
            request.level0Rings == 4 && request.algo == ALGO_RING && request.vCounts.empty();
        if ((request.p != 8 && !twoLevel) || (request.nicMask >> 8) != 0 || (ports != 1 && ports != 2 && ports != 4 && ports != 8)) {
            *err = "bad plan request: network ports are given for a ring of 8 ranks, or for a two-level reduce-scatter over "
                   "servers of 8 ranks with four rings inside and the ring between them; 1, 2, 4 or 8 of them";
            return 1;
        }
    }
    if (request.align % request.unit != 0) {
        // a slice boundary inside an element would make the kernels combine across element boundaries
        *err = "bad plan request: the slice alignment must be a multiple of the element size";
        return 1;
    }
    if ((request.level0Rings != 0 && request.level0Rings != 1 && request.level0Rings != 4) ||
        (request.level0Rings == 4 && request.p / request.servers != 8)) {
        *err = "level 0 runs as a mesh, one ring, or the four rings of a group of 8 ranks";
        return 1;
    }
    PlanRequest normalised;
    if (request.algo == ALGO_MESH_ATOMIC) {
        normalised = request;
        normalised.algo = ALGO_MESH;
        normalised.meshAtomic = true;
    }
    const PlanRequest &rq = request.algo == ALGO_MESH_ATOMIC ? normalised : request;
    VProgram vp;
    if (BuildVirtual(rq, &vp, err) != 0) {
        return 1;
    }
    uint32_t p = rq.p;
    std::vector<uint8_t> alias = rq.alias.size() == p ? rq.alias : std::vector<uint8_t>(p, 0);
    plan->p = p;
    plan->sendBytes = vp.inBytes;
    plan->recvBytes = vp.outBytes;
    if (DirectCopyPlan(vp, rq, alias, plan)) {
        return 0;
    }

    // expected outputs: the virtual program with separate input and output buffers
    Interner interner;
    Sym ref;
    ref.in = &interner;
    for (uint32_t r = 0; r < p; r++) {
        ref.Init(r, vp.inBytes[r]);
    }
    if (!ref.Run(vp.phases)) {
        *err = "virtual program: " + ref.err;
        return 2;
    }
    const std::vector<OutRange> refOuts = Outputs(ref, p);   // shared by the comparison below and by the fused form
    const std::vector<uint64_t> want = OutputSignature(ref, refOuts, alias);

    // lowering candidates: partials in the receive buffer (no scratch), else in scratch, else staged
    bool fits = vp.workBytes.empty();
    for (uint32_t r = 0; r < p; r++) {
        fits = fits && vp.inBytes[r] <= vp.outBytes[r];
    }
    struct Cand { uint8_t home; bool stage; };
    std::vector<Cand> cands;
    if (!rq.stageInput) {
        if (fits) {
            cands.push_back(Cand{BUF_RECV, false});
        }
        cands.push_back(Cand{BUF_SCRATCH, false});
    }
    cands.push_back(Cand{BUF_SCRATCH, true});
    bool ok = false;
    std::string why;
    Sym low;
    for (const Cand &c : cands) {
        std::vector<Phase> phases;
        Lower(vp, rq, c.home, c.stage, &phases);
        bool clean = true;
        for (const Phase &ph : phases) {
            if (!PhaseIsHazardFree(ph, alias, &why)) {
                clean = false;
                break;
            }
        }
        if (!clean) {
            continue;
        }
        Sym s;
        s.in = &interner;
        s.alias = alias;
        for (uint32_t r = 0; r < p; r++) {
            s.Init(r, vp.inBytes[r]);
        }
        if (!s.Run(phases)) {
            why = s.err;
            continue;
        }
        if (OutputSignature(s, Outputs(s, p), alias) != want) {
            why = "lowered program computes different outputs";
            continue;
        }
        plan->phases = std::move(phases);
        bool usesScratch = false;
        for (const Phase &ph : plan->phases) {
            for (const Step &st : ph.steps) {
                usesScratch = usesScratch || st.dst.buf == BUF_SCRATCH;
            }
        }
        plan->scratchBytes = 0;
        if (usesScratch) {
            for (uint32_t r = 0; r < p; r++) {
                plan->scratchBytes = std::max(plan->scratchBytes, vp.inBytes[r] + (vp.workBytes.empty() ? 0 : vp.workBytes[r]));
            }
        }
        low = std::move(s);
        ok = true;
        break;
    }
    if (!ok) {
        *err = "no safe lowering: " + why;
        return 2;
    }

    plan->stepRead = plan->stepWritten = 0;
    for (const Phase &ph : plan->phases) {
        for (const Step &s : ph.steps) {
            plan->stepRead += s.bytes * (s.reduce ? 2 : 1);
            plan->stepWritten += s.bytes;
        }
    }

    // fused form, derived from the virtual program's expressions (leaves are send-buffer ranges)
    plan->fused.clear();
    plan->fusedOk = BuildFused(ref, refOuts, rq, &plan->fused);
    plan->fusedRead = plan->fusedWritten = 0;
    if (plan->fusedOk) {
        for (FusedItem &it : plan->fused) {
            uint64_t nsrc = 0;
            for (uint8_t v : it.srcValid) {
                nsrc += v;
            }
            plan->fusedRead += nsrc * it.bytes;
            plan->fusedWritten += it.dst.size() * it.bytes;
        }
        // an aliased copy onto itself moves nothing
        for (FusedItem &it : plan->fused) {
            if (it.kind != FK_COPY) {
                continue;
            }
            std::vector<Ref> keep;
            for (const Ref &d : it.dst) {
                bool self = d.rank == it.src[0].rank && d.off == it.src[0].off && alias[d.rank] && it.src[0].buf == BUF_SEND;
                if (self) {
                    plan->fusedWritten -= it.bytes;
                } else {
                    keep.push_back(d);
                }
            }
            if (keep.empty()) {
                plan->fusedRead -= it.bytes;
            }
            it.dst.assign(keep.begin(), keep.end());
        }
        plan->fused.erase(std::remove_if(plan->fused.begin(), plan->fused.end(),
            [](const FusedItem &it) { return it.dst.empty(); }), plan->fused.end());
    } else {
        plan->fused.clear();
    }
    return 0;
}

std::string DescribePlan(const Plan &plan)
{
    std::ostringstream os;
    os << "{\"p\":" << plan.p << ",\"scratchBytes\":" << plan.scratchBytes << ",\"fusedOk\":" << (plan.fusedOk ? "true" : "false")
       << ",\"stepRead\":" << plan.stepRead << ",\"stepWritten\":" << plan.stepWritten << ",\"fusedRead\":" << plan.fusedRead
       << ",\"fusedWritten\":" << plan.fusedWritten << ",\"phases\":[";
    for (size_t i = 0; i < plan.phases.size(); i++) {
        os << (i ? "," : "") << "[";
        const Phase &ph = plan.phases[i];
        for (size_t j = 0; j < ph.steps.size(); j++) {
            const Step &s = ph.steps[j];
            os << (j ? "," : "") << "{\"r\":" << (s.reduce ? 1 : 0) << ",\"n\":" << s.bytes << ",\"dst\":";
            JsonRef(os, s.dst);
            os << ",\"a\":";
            JsonRef(os, s.a);
            if (s.reduce) {
                os << ",\"b\":";
                JsonRef(os, s.b);
            }
            os << "}";
        }
        os << "]";
    }
    os << "],\"fused\":[";
    for (size_t i = 0; i < plan.fused.size(); i++) {
        const FusedItem &it = plan.fused[i];
        os << (i ? "," : "") << "{\"kind\":" << int(it.kind) << ",\"n\":" << it.bytes << ",\"nleaf\":" << it.nleaf << ",\"src\":[";
        for (size_t k = 0; k < it.src.size(); k++) {
            os << (k ? "," : "");
            if (it.srcValid[k]) {
                JsonRef(os, it.src[k]);
            } else {
                os << "null";
            }
        }
        os << "],\"accLeft\":[";
        for (size_t k = 0; k < it.accLeft.size(); k++) {
            os << (k ? "," : "") << int(it.accLeft[k]);
        }
        os << "],\"ops\":[";
        for (size_t k = 0; k < it.ops.size(); k++) {
            os << (k ? "," : "") << int(it.ops[k]);
        }
        os << "],\"dst\":[";
        for (size_t k = 0; k < it.dst.size(); k++) {
            os << (k ? "," : "");
            JsonRef(os, it.dst[k]);
        }
        os << "]}";
    }
    os << "]}";
    return os.str();
}

}  // namespace hcclamd
