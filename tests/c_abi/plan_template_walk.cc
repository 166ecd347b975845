// A seeded walk over plan requests and, for each request, over a sequence of counts (or block tables): every plan that
// PlanFromTemplate derives from a template of an earlier count of the same request must be the planner's own plan for
// that count, number for number.  Host only (cann-hccl_amd/csrc/plan*.cc alone, no GPU).
//
// The requests: collective, schedule, 2 .. 33 ranks, rank groups ("servers"), rings inside a group, ranks with a network
// port, which ranks run in place, element size, CCL buffer size.  The counts: whole slices, ragged last slices, a few
// elements, several chunks of the CCL buffer.  The tables (variable-count reduce-scatter): non-empty blocks in rank
// order, and tables with gaps or empty blocks, which must not be derived.  Up to four templates are kept per request, as
// the library keeps them.  HCCL_AMD_TEST_SEED_SHIFT moves the walk to other cases; argv[1] = derived plans to reach.
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <string>
#include <vector>

#include "plan.h"

using namespace hcclamd;

namespace {

uint64_t g_state = 0x9E3779B97F4A7C15ull;
uint64_t Next()
{
    g_state = g_state * 6364136223846793005ull + 1442695040888963407ull;
    return g_state >> 29;
}
uint64_t Below(uint64_t n) { return n == 0 ? 0 : Next() % n; }

std::string Show(const PlanRequest &rq)
{
    char buf[320];
    uint32_t mask = 0;
    for (size_t i = 0; i < rq.alias.size() && i < 32; i++) {
        mask |= uint32_t(rq.alias[i] ? 1 : 0) << i;
    }
    std::snprintf(buf, sizeof(buf), "coll %d algo %d p %u servers %u level0 %u nic 0x%x alias 0x%x unit %u ccl %llu count %llu%s root %u",
        int(rq.coll), int(rq.algo), rq.p, rq.servers, rq.level0Rings, rq.nicMask, mask, rq.unit, (unsigned long long)rq.cclBytes,
        (unsigned long long)rq.count, rq.vCounts.empty() ? "" : " (block table)", rq.root);
    return buf;
}

}  // namespace

int main(int argc, char **argv)
{
    const long want = argc > 1 ? std::atol(argv[1]) : 20000;
    if (const char *e = std::getenv("HCCL_AMD_TEST_SEED_SHIFT")) {
        g_state += uint64_t(std::atoll(e)) * 0x2545F4914F6CDD1Dull;
    }
    const auto t0 = std::chrono::steady_clock::now();
    long derived = 0, refused = 0, requests = 0, invalid = 0, ragged = 0, tables = 0, mustRefuse = 0;
    while (derived < want) {
        // ---- a request ----
        PlanRequest base;
        const uint64_t pick = Below(16);
        base.coll = pick < 6 ? COLL_ALLREDUCE : pick < 9 ? COLL_REDUCESCATTER : pick < 11 ? COLL_ALLGATHER
            : pick < 13 ? COLL_BROADCAST : pick < 15 ? COLL_REDUCE : COLL_SCATTER;
        const uint64_t a = Below(8);
        base.algo = a < 3 ? ALGO_RING : a < 4 ? ALGO_MESH : a < 6 ? ALGO_MESH_ATOMIC : ALGO_RHD;
        if (base.coll == COLL_BROADCAST && Below(6) == 0) {
            base.algo = ALGO_STAR;
        } else if (base.coll == COLL_BROADCAST && Below(5) == 0) {
            base.algo = ALGO_HD_BLOCKS;
        }
        if (base.coll == COLL_SCATTER) {
            base.algo = Below(2) ? ALGO_MESH : ALGO_RING;
        }
        // small groups mostly; the piece-cut mesh is expensive to plan for many ranks
        const uint64_t size = Below(50);
        base.p = uint32_t(size < 38 ? 2 + Below(7) : size < 48 ? 9 + Below(8) : 17 + Below(17));
        if (base.algo == ALGO_MESH && base.p > 12) {
            base.p = 2 + uint32_t(Below(11));
        }
        if (Below(4) == 0) {                 // rank groups: a divisor of p that leaves groups of two ranks and more
            std::vector<uint32_t> divisors;
            for (uint32_t s = 2; s * 2 <= base.p; s++) {
                if (base.p % s == 0) {
                    divisors.push_back(s);
                }
            }
            if (!divisors.empty()) {
                base.servers = divisors[Below(divisors.size())];
            }
        }
        const uint32_t perGroup = base.p / base.servers;
        if ((base.coll == COLL_ALLREDUCE || base.coll == COLL_REDUCESCATTER || base.coll == COLL_ALLGATHER || base.coll == COLL_REDUCE ||
                base.coll == COLL_BROADCAST) &&
            Below(4) == 0 && (base.servers > 1 || perGroup == 8)) {
            base.level0Rings = (perGroup == 8 && Below(2)) ? 4 : (base.servers > 1 ? 1 : 0);
        }
        if (base.coll == COLL_ALLREDUCE && base.algo == ALGO_RING && base.p == 8 && base.servers == 1 && base.level0Rings == 0 && Below(3) == 0) {
            const uint32_t masks[] = {0x01, 0x80, 0x11, 0x22, 0x0f, 0x55, 0xaa, 0x04};
            base.nicMask = masks[Below(8)];
        }
        if (base.coll == COLL_REDUCESCATTER && base.algo == ALGO_RING && base.servers > 1 && base.level0Rings == 4 && Below(2) == 0) {
            const uint32_t masks[] = {0x01, 0x80, 0x11, 0x22, 0x0f, 0x55, 0xaa, 0x04};
            base.nicMask = masks[Below(8)];       // servers whose devices do not all have a network port
        }
        const uint32_t units[] = {1, 2, 4, 8};
        base.unit = units[Below(4)];
        const uint64_t ccls[] = {1ull << 20, 16ull << 20, 200ull << 20};
        base.cclBytes = ccls[Below(3)];
        base.root = uint32_t(Below(base.p));
        base.alias.assign(base.p, 0);
        if (base.coll == COLL_ALLREDUCE || base.coll == COLL_BROADCAST) {
            const uint64_t mode = Below(4);       // none, all, a random subset, one rank
            for (uint32_t r = 0; r < base.p; r++) {
                base.alias[r] = mode == 1 ? 1 : mode == 2 ? uint8_t(Below(2)) : (mode == 3 && r == base.root) ? 1 : 0;
            }
            if (base.coll == COLL_BROADCAST && mode >= 2) {
                base.alias.assign(base.p, 0);
            }
        }
        const bool byTable = base.coll == COLL_REDUCESCATTER && base.servers == 1 && base.level0Rings == 0 && Below(3) == 0;
        requests++;

        // ---- a sequence of counts or tables for it ----
        std::vector<PlanTemplate> kept;
        const uint64_t regular = uint64_t(base.p) * base.p * 128 * 12 / base.unit;
        const int steps = base.p <= 8 ? 30 : base.p <= 16 ? 16 : 8;
        bool requestValid = true;
        for (int s = 0; s < steps && requestValid; s++) {
            PlanRequest rq = base;
            bool shouldRefuse = false;
            if (byTable) {
                rq.vCounts.resize(base.p);
                rq.vDispls.resize(base.p);
                const uint64_t kind = s == 0 ? 0 : Below(10);       // mostly non-empty blocks in rank order
                const uint64_t scale = Below(3) == 0 ? 50 : Below(2) ? 100000 : (1u << 22);
                uint64_t at = 0;
                for (uint32_t r = 0; r < base.p; r++) {
                    rq.vCounts[r] = 1 + Below(scale);
                    if (kind == 8 && r == base.p / 2) {
                        rq.vCounts[r] = 0;                          // an empty block
                    }
                    if (kind == 9 && r == base.p - 1) {
                        at += 1 + Below(9);                         // a gap in front of the last block
                    }
                    rq.vDispls[r] = at;
                    at += rq.vCounts[r];
                }
                shouldRefuse = kind >= 8;
            } else {
                const uint64_t kind = Below(10);
                // one chunk of the executor's loop: the CCL buffer holds a count, or one block per rank
                const bool perRank = base.coll == COLL_REDUCESCATTER || base.coll == COLL_ALLGATHER;
                const uint64_t chunk = std::max<uint64_t>(1, base.cclBytes / base.unit / (perRank ? base.p : 1));
                rq.count = kind < 4 ? (1 + Below(9)) * regular                       // whole slices
                    : kind < 7 ? (1 + Below(9)) * regular + 1 + Below(regular - 1)   // a ragged last slice
                    : kind < 8 ? 1 + Below(40)                                        // a few elements
                    : chunk + Below(2 * chunk);                                       // several chunks of the CCL buffer
                if (rq.count > (96ull << 20)) {
                    rq.count = (96ull << 20) + Below(1000);        // keep the plans of many-rank requests small enough to compare
                }
                if (rq.count > 6 * chunk) {
                    rq.count = 6 * chunk - Below(std::min<uint64_t>(chunk, 1000));   // and at most six rounds of the chunk loop
                }
            }
            std::string err;
            Plan direct;
            if (BuildPlan(rq, &direct, &err) != 0) {
                if (s == 0) {
                    invalid++;                                      // a combination the planner does not take: next request
                    requestValid = false;
                    break;
                }
                std::printf("plan failed for a later count of a request that was planned before: %s: %s\n", Show(rq).c_str(), err.c_str());
                return 1;
            }
            bool got = false;
            for (const PlanTemplate &t : kept) {
                Plan fromTemplate;
                if (!PlanFromTemplate(rq, t, &fromTemplate)) {
                    continue;
                }
                got = true;
                if (shouldRefuse) {
                    std::printf("a table with a gap or an empty block was derived: %s\n", Show(rq).c_str());
                    return 1;
                }
                if (DescribePlan(fromTemplate) != DescribePlan(direct) || fromTemplate.sendBytes != direct.sendBytes ||
                    fromTemplate.recvBytes != direct.recvBytes || fromTemplate.scratchBytes != direct.scratchBytes ||
                    fromTemplate.fusedOk != direct.fusedOk) {
                    std::printf("derived plan differs from the planner's own: %s (template count %llu%s)\n", Show(rq).c_str(),
                        (unsigned long long)t.count, t.blockTable ? ", block template" : "");
                    return 1;
                }
                derived++;
                tables += t.blockTable ? 1 : 0;
                ragged += (!t.blockTable && rq.count % regular != 0) ? 1 : 0;
                break;
            }
            if (!got) {
                refused++;
                mustRefuse += shouldRefuse ? 1 : 0;
                PlanTemplate t;
                Plan own;
                if (BuildPlanTemplate(rq, &t, &own, &err) != 0) {
                    std::printf("template failed: %s: %s\n", Show(rq).c_str(), err.c_str());
                    return 1;
                }
                if (DescribePlan(own) != DescribePlan(direct)) {
                    std::printf("the plan returned with a template differs from the planner's own: %s\n", Show(rq).c_str());
                    return 1;
                }
                if (t.count != 0 || t.blockTable) {
                    if (kept.size() == 4) {
                        kept.erase(kept.begin());
                    }
                    kept.push_back(std::move(t));
                }
            }
        }
    }
    const double secs = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
    std::printf("OK %ld derived (%ld of them ragged counts, %ld from block templates), %ld planned from scratch (%ld tables that must be), "
        "%ld requests, %ld not taken by the planner, %.1f s\n", derived, ragged, tables, refused, mustRefuse, requests, invalid, secs);
    return 0;
}
