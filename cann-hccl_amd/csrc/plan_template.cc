// Plans derived from earlier plans of the same request: a count's plan from the template of another count (scaled,
// cut off at the last byte), a block table's plan from the template over canonical block sizes.  Nothing is assumed:
// the new request's schedule is laid out and held against the template before a plan is derived.
#include "plan_internal.h"

namespace hcclamd {

using namespace planner;

namespace {

bool Templatable(const PlanRequest &rq)
{
    return rq.count > 0 && rq.coll != COLL_ALLTOALLV && rq.vCounts.empty();
}

PlanRequest Normalised(const PlanRequest &request)
{
    PlanRequest rq = request;
    if (rq.algo == ALGO_MESH_ATOMIC) {
        rq.algo = ALGO_MESH;
        rq.meshAtomic = true;
    }
    return rq;
}

bool SameOffsets(const Step &st) { return st.dst.off == st.a.off && (!st.reduce || st.b.off == st.a.off); }

}  // namespace

namespace {

int BuildCountTemplate(const PlanRequest &request, PlanTemplate *tmpl, std::string *err)
{
    tmpl->count = 0;
    int rc = BuildPlan(request, &tmpl->plan, err);
    if (rc != 0 || !Templatable(request)) {
        return rc;
    }
    VProgram vp;
    std::string ignored;
    if (BuildVirtual(Normalised(request), &vp, &ignored) != 0) {
        return 0;
    }
    tmpl->schedule = std::move(vp.phases);
    tmpl->inBytes = vp.inBytes;
    tmpl->outBytes = vp.outBytes;
    tmpl->workBytes = vp.workBytes;
    tmpl->workspace = !vp.workBytes.empty();
    // position by position: every step, of the schedule and of the plan, touches one offset in all its buffers, every
    // fused item likewise, and every buffer in use is as long as the count
    bool pw = !tmpl->workspace &&
        (request.coll == COLL_ALLREDUCE || request.coll == COLL_BROADCAST || request.coll == COLL_REDUCE);
    const uint64_t extent = request.count * request.unit;
    for (const std::vector<uint64_t> *v : {&tmpl->inBytes, &tmpl->outBytes, &tmpl->plan.sendBytes, &tmpl->plan.recvBytes}) {
        for (uint64_t x : *v) {
            pw = pw && (x == 0 || x == extent);
        }
    }
    pw = pw && (tmpl->plan.scratchBytes == 0 || tmpl->plan.scratchBytes == extent);
    for (const std::vector<Phase> *phases : {&tmpl->schedule, &tmpl->plan.phases}) {
        for (const Phase &ph : *phases) {
            for (const Step &st : ph.steps) {
                pw = pw && SameOffsets(st) && st.dst.off + st.bytes <= extent;
            }
        }
    }
    for (const FusedItem &it : tmpl->plan.fused) {
        for (size_t k = 0; k < it.src.size(); k++) {
            pw = pw && (!it.srcValid[k] || it.src[k].off == it.dst[0].off);
        }
        for (const Ref &d : it.dst) {
            pw = pw && d.off == it.dst[0].off && d.off + it.bytes <= extent;
        }
    }
    tmpl->positionWise = pw;
    tmpl->count = request.count;
    return 0;
}

bool PlanFromCountTemplate(const PlanRequest &request, const PlanTemplate &tmpl, Plan *plan)
{
    if (tmpl.count == 0 || !Templatable(request)) {
        return false;
    }
    VProgram vp;
    std::string ignored;
    if (BuildVirtual(Normalised(request), &vp, &ignored) != 0 || vp.workBytes.empty() == tmpl.workspace) {
        return false;
    }
    typedef unsigned __int128 Wide;
    // The factor: the longest step of the new schedule over the longest of the template's (a whole slice on both
    // sides whenever there is one; if the guess is wrong the comparison below fails and nothing is derived).
    uint64_t num = 0, den = 0;
    for (const Phase &ph : vp.phases) {
        for (const Step &st : ph.steps) {
            num = std::max(num, st.bytes);
        }
    }
    for (const Phase &ph : tmpl.schedule) {
        for (const Step &st : ph.steps) {
            den = std::max(den, st.bytes);
        }
    }
    if (num == 0 || den == 0) {
        return false;
    }
    const bool cut = tmpl.positionWise;
    const uint64_t extent = request.count * request.unit;
    bool whole = true;
    auto scaled = [&](uint64_t x) {
        const Wide y = Wide(x) * num;
        whole = whole && y % den == 0;
        return uint64_t(y / den);
    };
    // length of a range that starts at (scaled) offset `at` and had (scaled) length `len`: cut off at the extent
    auto kept = [&](uint64_t at, uint64_t len) { return !cut ? len : (at >= extent ? 0 : std::min(len, extent - at)); };
    // 1. the new schedule is the template's, scaled and cut off
    if (vp.inBytes.size() != tmpl.inBytes.size() || vp.outBytes.size() != tmpl.outBytes.size() ||
        vp.phases.size() > tmpl.schedule.size()) {
        return false;
    }
    for (size_t r = 0; r < vp.inBytes.size(); r++) {
        if (vp.inBytes[r] != kept(0, scaled(tmpl.inBytes[r])) || vp.outBytes[r] != kept(0, scaled(tmpl.outBytes[r]))) {
            return false;
        }
    }
    if (vp.workBytes.size() != tmpl.workBytes.size()) {
        return false;
    }
    for (size_t r = 0; r < vp.workBytes.size(); r++) {
        if (vp.workBytes[r] != scaled(tmpl.workBytes[r])) {
            return false;
        }
    }
    for (size_t i = 0; i < tmpl.schedule.size(); i++) {
        static const Phase none;
        const Phase &fresh = i < vp.phases.size() ? vp.phases[i] : none;
        size_t at = 0;
        for (const Step &t : tmpl.schedule[i].steps) {
            const uint64_t dst = scaled(t.dst.off), a = scaled(t.a.off), b = t.reduce ? scaled(t.b.off) : 0;
            const uint64_t bytes = kept(dst, scaled(t.bytes));
            if (bytes == 0) {
                continue;
            }
            if (at >= fresh.steps.size()) {
                return false;
            }
            const Step &f = fresh.steps[at++];
            if (f.reduce != t.reduce || f.bytes != bytes || f.dst.rank != t.dst.rank || f.dst.buf != t.dst.buf || f.dst.off != dst ||
                f.a.rank != t.a.rank || f.a.buf != t.a.buf || f.a.off != a ||
                (t.reduce && (f.b.rank != t.b.rank || f.b.buf != t.b.buf || f.b.off != b))) {
                return false;
            }
        }
        if (at != fresh.steps.size()) {
            return false;
        }
    }
    if (!whole) {
        return false;
    }
    // 2. so its plan is the template's plan, scaled and cut off the same way (every number of the plan is a sum or
    // difference of schedule numbers, so it scales with them and comes out whole)
    plan->p = tmpl.plan.p;
    plan->fusedOk = tmpl.plan.fusedOk;
    plan->phases.clear();
    plan->fused.clear();
    plan->stepRead = plan->stepWritten = plan->fusedRead = plan->fusedWritten = 0;
    for (const Phase &tph : tmpl.plan.phases) {
        Phase ph;
        ph.steps.reserve(tph.steps.size());
        for (const Step &t : tph.steps) {
            Step st = t;
            st.dst.off = scaled(t.dst.off);
            st.a.off = scaled(t.a.off);
            st.b.off = scaled(t.b.off);
            st.bytes = kept(st.dst.off, scaled(t.bytes));
            if (st.bytes == 0) {
                continue;
            }
            plan->stepRead += st.bytes * (st.reduce ? 2 : 1);
            plan->stepWritten += st.bytes;
            ph.steps.push_back(st);
        }
        if (!ph.steps.empty()) {
            plan->phases.push_back(std::move(ph));
        }
    }
    for (const FusedItem &t : tmpl.plan.fused) {
        FusedItem it = t;
        for (Ref &r : it.src) {
            r.off = scaled(r.off);
        }
        for (Ref &r : it.dst) {
            r.off = scaled(r.off);
        }
        it.bytes = kept(it.dst.empty() ? 0 : it.dst[0].off, scaled(t.bytes));
        if (it.bytes == 0) {
            continue;
        }
        uint64_t nsrc = 0;
        for (uint8_t v : it.srcValid) {
            nsrc += v;
        }
        plan->fusedRead += nsrc * it.bytes;
        plan->fusedWritten += uint64_t(it.dst.size()) * it.bytes;
        plan->fused.push_back(std::move(it));
    }
    plan->sendBytes = tmpl.plan.sendBytes;
    plan->recvBytes = tmpl.plan.recvBytes;
    for (std::vector<uint64_t> *v : {&plan->sendBytes, &plan->recvBytes}) {
        for (uint64_t &x : *v) {
            x = kept(0, scaled(x));
        }
    }
    plan->scratchBytes = kept(0, scaled(tmpl.plan.scratchBytes));
    return whole;
}

// ---- block-table templates (variable-count reduce-scatter) --------------------------------------------------------
constexpr uint32_t kCanonicalShift = 4;       // canonical block s has 2^(s + 4) elements
constexpr uint32_t kBlockTableMaxRanks = 32;

bool BlockTableRequest(const PlanRequest &rq)
{
    if (rq.coll != COLL_REDUCESCATTER || rq.vCounts.size() != rq.p || rq.vDispls.size() != rq.p || rq.p < 2 ||
        rq.p > kBlockTableMaxRanks || rq.servers > 1) {
        return false;
    }
    if (rq.algo == ALGO_MESH && !rq.meshAtomic) {
        return false;       // the piece cut splits blocks at aligned lengths: its numbers are not runs of blocks
    }
    for (uint8_t shared : rq.alias) {
        if (shared) {
            return false;   // in place, a block's length is held against offsets of the send buffer: an order the sizes decide
        }
    }
    if (rq.stageInput) {
        return false;
    }
    uint64_t at = 0;
    for (uint32_t r = 0; r < rq.p; r++) {
        if (rq.vCounts[r] == 0 || rq.vDispls[r] != at) {
            return false;
        }
        at += rq.vCounts[r];
    }
    return true;
}

// A canonical number (bytes) as the run of blocks [first, last) it measures; false if it is not one.
bool RunOf(uint64_t bytes, uint64_t unit, uint32_t p, uint32_t *first, uint32_t *last)
{
    const uint64_t scale = unit << kCanonicalShift;
    if (bytes % scale != 0) {
        return false;
    }
    const uint64_t m = bytes / scale;      // 2^last - 2^first
    if (m == 0) {
        *first = *last = 0;
        return true;
    }
    const uint32_t a = uint32_t(__builtin_ctzll(m));
    const uint64_t ones = (m >> a) + 1;    // 2^(last - first)
    if ((ones & (ones - 1)) != 0) {
        return false;
    }
    const uint32_t b = a + uint32_t(__builtin_ctzll(ones));
    if (b > p) {
        return false;
    }
    *first = a;
    *last = b;
    return true;
}

bool PlanFromBlockTemplate(const PlanRequest &request, const PlanTemplate &tmpl, Plan *plan)
{
    if (!tmpl.blockTable || !BlockTableRequest(request)) {
        return false;
    }
    VProgram vp;
    std::string ignored;
    if (BuildVirtual(Normalised(request), &vp, &ignored) != 0 || !vp.workBytes.empty()) {
        return false;
    }
    const uint32_t p = request.p;
    std::vector<uint64_t> prefix(p + 1, 0);   // bytes in front of block s
    for (uint32_t s = 0; s < p; s++) {
        prefix[s + 1] = prefix[s] + request.vCounts[s] * request.unit;
    }
    bool ok = true;
    auto measured = [&](uint64_t canonical) -> uint64_t {
        uint32_t a = 0, b = 0;
        if (!RunOf(canonical, request.unit, p, &a, &b)) {
            ok = false;
            return 0;
        }
        return prefix[b] - prefix[a];
    };
    // 1. the new schedule is the canonical one re-measured
    if (vp.phases.size() != tmpl.schedule.size() || vp.inBytes.size() != tmpl.inBytes.size()) {
        return false;
    }
    for (size_t r = 0; r < vp.inBytes.size(); r++) {
        if (vp.inBytes[r] != measured(tmpl.inBytes[r]) || vp.outBytes[r] != measured(tmpl.outBytes[r])) {
            return false;
        }
    }
    for (size_t i = 0; i < vp.phases.size(); i++) {
        if (vp.phases[i].steps.size() != tmpl.schedule[i].steps.size()) {
            return false;
        }
        for (size_t j = 0; j < vp.phases[i].steps.size(); j++) {
            const Step &f = vp.phases[i].steps[j], &t = tmpl.schedule[i].steps[j];
            if (f.reduce != t.reduce || f.dst.rank != t.dst.rank || f.dst.buf != t.dst.buf || f.a.rank != t.a.rank ||
                f.a.buf != t.a.buf || (t.reduce && (f.b.rank != t.b.rank || f.b.buf != t.b.buf)) ||
                f.bytes != measured(t.bytes) || f.dst.off != measured(t.dst.off) || f.a.off != measured(t.a.off) ||
                (t.reduce && f.b.off != measured(t.b.off))) {
                return false;
            }
        }
    }
    if (!ok) {
        return false;
    }
    // 2. so its plan is the canonical plan re-measured
    *plan = tmpl.plan;
    plan->stepRead = plan->stepWritten = plan->fusedRead = plan->fusedWritten = 0;
    for (Phase &ph : plan->phases) {
        for (Step &st : ph.steps) {
            st.dst.off = measured(st.dst.off);
            st.a.off = measured(st.a.off);
            st.b.off = st.reduce ? measured(st.b.off) : 0;
            st.bytes = measured(st.bytes);
            plan->stepRead += st.bytes * (st.reduce ? 2 : 1);
            plan->stepWritten += st.bytes;
        }
    }
    for (FusedItem &it : plan->fused) {
        it.bytes = measured(it.bytes);
        uint64_t nsrc = 0;
        for (size_t k = 0; k < it.src.size(); k++) {
            if (it.srcValid[k]) {
                it.src[k].off = measured(it.src[k].off);
                nsrc++;
            }
        }
        for (Ref &r : it.dst) {
            r.off = measured(r.off);
        }
        plan->fusedRead += nsrc * it.bytes;
        plan->fusedWritten += uint64_t(it.dst.size()) * it.bytes;
    }
    for (std::vector<uint64_t> *v : {&plan->sendBytes, &plan->recvBytes}) {
        for (uint64_t &x : *v) {
            x = measured(x);
        }
    }
    plan->scratchBytes = measured(plan->scratchBytes);
    return ok;
}

int BuildBlockTemplate(const PlanRequest &request, PlanTemplate *tmpl, std::string *err)
{
    PlanRequest canonical = request;
    uint64_t at = 0;
    for (uint32_t s = 0; s < request.p; s++) {
        canonical.vCounts[s] = uint64_t(1) << (s + kCanonicalShift);
        canonical.vDispls[s] = at;
        at += canonical.vCounts[s];
    }
    int rc = BuildPlan(canonical, &tmpl->plan, err);
    if (rc != 0) {
        return rc;
    }
    VProgram vp;
    std::string ignored;
    if (BuildVirtual(Normalised(canonical), &vp, &ignored) != 0 || !vp.workBytes.empty()) {
        return 0;
    }
    tmpl->schedule = std::move(vp.phases);
    tmpl->inBytes = vp.inBytes;
    tmpl->outBytes = vp.outBytes;
    tmpl->blockTable = true;
    return 0;
}

}  // namespace

int BuildPlanTemplate(const PlanRequest &request, PlanTemplate *tmpl, Plan *plan, std::string *err)
{
    tmpl->count = 0;
    tmpl->blockTable = false;
    if (BlockTableRequest(request)) {
        int rc = BuildBlockTemplate(request, tmpl, err);
        if (rc == 0 && tmpl->blockTable && PlanFromBlockTemplate(request, *tmpl, plan)) {
            return 0;
        }
        tmpl->blockTable = false;      // not the canonical schedule re-measured: no template, plan the request itself
        return BuildPlan(request, plan, err);
    }
    int rc = BuildCountTemplate(request, tmpl, err);
    if (rc == 0) {
        *plan = tmpl->plan;
    }
    return rc;
}

bool PlanFromTemplate(const PlanRequest &request, const PlanTemplate &tmpl, Plan *plan)
{
    return tmpl.blockTable ? PlanFromBlockTemplate(request, tmpl, plan) : PlanFromCountTemplate(request, tmpl, plan);
}

}  // namespace hcclamd
