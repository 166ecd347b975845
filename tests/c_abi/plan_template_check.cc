// Plans derived from a template of another count against plans made from scratch, on the host
// (cann-hccl_amd/csrc/plan*.cc alone, no GPU): wherever PlanFromTemplate says it can derive a plan, the derived plan
// must be the planner's own, number for number; counts that cut into whole slices must be derivable, and so must a
// count with a ragged last slice from a whole-slice template of a ring or uncut-mesh all-reduce or a ring broadcast.
#include <cstdio>
#include <string>
#include <vector>

#include "plan.h"

using namespace hcclamd;

int main()
{
    int derived = 0, refused = 0, cases = 0, ragged = 0;
    struct Shape {
        int coll, algo;
        uint32_t p, servers, level0;
        uint32_t nicMask = 0;
    };
    const std::vector<Shape> shapes = {
        {COLL_ALLREDUCE, ALGO_RING, 8, 1, 0}, {COLL_ALLREDUCE, ALGO_MESH, 4, 1, 0}, {COLL_ALLREDUCE, ALGO_MESH_ATOMIC, 8, 1, 0},
        {COLL_ALLREDUCE, ALGO_RHD, 6, 1, 0}, {COLL_ALLREDUCE, ALGO_RHD, 8, 2, 0}, {COLL_ALLREDUCE, ALGO_RING, 8, 2, 1},
        {COLL_REDUCESCATTER, ALGO_RING, 8, 1, 0}, {COLL_REDUCESCATTER, ALGO_MESH, 5, 1, 0}, {COLL_REDUCESCATTER, ALGO_RHD, 8, 2, 0},
        {COLL_ALLGATHER, ALGO_RING, 8, 1, 0}, {COLL_ALLGATHER, ALGO_MESH, 3, 1, 0}, {COLL_ALLGATHER, ALGO_RHD, 12, 1, 0},
        {COLL_BROADCAST, ALGO_RING, 8, 1, 0}, {COLL_BROADCAST, ALGO_MESH, 8, 2, 0}, {COLL_BROADCAST, ALGO_RHD, 5, 1, 0},
        {COLL_REDUCE, ALGO_RING, 8, 1, 0}, {COLL_REDUCE, ALGO_MESH, 4, 1, 0}, {COLL_REDUCE, ALGO_RHD, 8, 2, 0},
        {COLL_SCATTER, ALGO_MESH, 8, 1, 0}, {COLL_SCATTER, ALGO_RING, 6, 1, 0}, {COLL_SCATTER, ALGO_MESH, 8, 2, 0},
        {COLL_ALLREDUCE, ALGO_RING, 8, 1, 4}, {COLL_ALLREDUCE, ALGO_RHD, 16, 2, 4}, {COLL_ALLREDUCE, ALGO_RING, 8, 1, 0, 0x11},
        {COLL_ALLREDUCE, ALGO_RING, 8, 1, 0, 0x04}, {COLL_BROADCAST, ALGO_STAR, 5, 1, 0}, {COLL_REDUCESCATTER, ALGO_RING, 16, 2, 4},
    };
    for (const Shape &sh : shapes) {
        for (uint32_t unit : {4u, 2u}) {
            for (int inPlace = 0; inPlace < 2; inPlace++) {
                PlanRequest base;
                base.coll = CollKind(sh.coll);
                base.algo = Algo(sh.algo);
                base.p = sh.p;
                base.servers = sh.servers;
                base.level0Rings = sh.level0;
                base.nicMask = sh.nicMask;
                base.unit = unit;
                base.root = sh.p - 1;
                base.cclBytes = 16 << 20;
                const bool aliasable = sh.coll == COLL_ALLREDUCE || sh.coll == COLL_BROADCAST;
                base.alias.assign(sh.p, uint8_t(inPlace && aliasable ? 1 : 0));
                // whole slices: multiples of ranks x alignment (x rank-group sizes); then ragged ones; then several chunks
                const uint64_t regular = uint64_t(sh.p) * sh.p * 128 * 12 / unit;
                const std::vector<uint64_t> counts = {regular, 3 * regular, 7 * regular, regular + 1, 3 * regular + 5, 1, 2,
                    (32u << 20) / unit, (64u << 20) / unit, (64u << 20) / unit + 3};
                for (uint64_t c0 : counts) {
                    PlanRequest r0 = base;
                    r0.count = c0;
                    PlanTemplate tmpl;
                    std::string err;
                    Plan own;
                    if (BuildPlanTemplate(r0, &tmpl, &own, &err) != 0) {
                        printf("template failed: coll %d algo %d p %u count %llu: %s\n", sh.coll, sh.algo, sh.p, (unsigned long long)c0, err.c_str());
                        return 1;
                    }
                    for (uint64_t c1 : counts) {
                        PlanRequest r1 = base;
                        r1.count = c1;
                        Plan direct, scaled;
                        if (BuildPlan(r1, &direct, &err) != 0) {
                            printf("plan failed: %s\n", err.c_str());
                            return 1;
                        }
                        cases++;
                        const bool ok = PlanFromTemplate(r1, tmpl, &scaled);
                        if (ok) {
                            derived++;
                            if (DescribePlan(scaled) != DescribePlan(direct)) {
                                printf("derived plan differs: coll %d algo %d p %u servers %u unit %u in place %d, template %llu, count %llu\n",
                                    sh.coll, sh.algo, sh.p, sh.servers, unit, inPlace, (unsigned long long)c0, (unsigned long long)c1);
                                return 1;
                            }
                            if (scaled.sendBytes != direct.sendBytes || scaled.recvBytes != direct.recvBytes) {
                                printf("derived extents differ\n");
                                return 1;
                            }
                        } else {
                            refused++;
                        }
                        // (one chunk for every collective: the per-rank collectives size their chunks by count x ranks)
                        const bool bothWhole = c0 % regular == 0 && c1 % regular == 0 && c0 * unit * sh.p <= base.cclBytes &&
                            c1 * unit * sh.p <= base.cclBytes;
                        if (bothWhole && !ok) {
                            printf("whole-slice counts not derived: coll %d algo %d p %u servers %u, template %llu, count %llu\n", sh.coll,
                                sh.algo, sh.p, sh.servers, (unsigned long long)c0, (unsigned long long)c1);
                            return 1;
                        }
                        // a ragged count is the whole-slice schedule cut off at its last byte wherever the collective
                        // works position by position and does not cut slices any further: the ring and the uncut mesh
                        const bool cutOff = (sh.coll == COLL_ALLREDUCE && sh.servers == 1 && sh.level0 == 0 && sh.nicMask == 0 &&
                            (sh.algo == ALGO_RING || sh.algo == ALGO_MESH_ATOMIC)) || (sh.coll == COLL_BROADCAST && sh.algo == ALGO_RING);
                        if (c0 == 3 * regular && (c1 == regular + 1 || c1 == 3 * regular + 5) && cutOff && !ok) {
                            printf("a ragged count was not derived from a whole one: coll %d algo %d p %u, count %llu\n", sh.coll, sh.algo,
                                sh.p, (unsigned long long)c1);
                            return 1;
                        }
                        ragged += (ok && c1 % regular != 0 && c0 % regular == 0) ? 1 : 0;
                    }
                }
            }
        }
    }
    // requests without a count have no count template
    PlanRequest v;
    v.coll = COLL_ALLGATHER;
    v.p = 4;
    v.vCounts = {1, 2, 3, 4};
    v.vDispls = {0, 1, 3, 6};
    v.alias.assign(4, 0);
    PlanTemplate tv;
    std::string err;
    Plan out;
    if (BuildPlanTemplate(v, &tv, &out, &err) != 0 || tv.count != 0 || tv.blockTable || PlanFromTemplate(v, tv, &out)) {
        printf("a variable-count all-gather got a template\n");
        return 1;
    }
    // the variable-count reduce-scatter over non-empty blocks in rank order: one template per schedule serves every table
    int tables = 0;
    uint64_t seed = 12345;
    auto next = [&] { seed = seed * 6364136223846793005ull + 1442695040888963407ull; return seed >> 33; };
    for (int algo : {int(ALGO_RING), int(ALGO_MESH_ATOMIC), int(ALGO_RHD), int(ALGO_MESH)}) {
        for (uint32_t p : {2u, 3u, 5u, 8u, 12u, 16u, 32u}) {
            for (uint32_t unit : {4u, 2u}) {
                PlanRequest base;
                base.coll = COLL_REDUCESCATTER;
                base.algo = Algo(algo);
                base.p = p;
                base.unit = unit;
                base.alias.assign(p, 0);
                PlanTemplate bt;
                bool have = false;
                for (int t = 0; t < 12; t++) {
                    PlanRequest rq = base;
                    rq.vCounts.resize(p);
                    rq.vDispls.resize(p);
                    uint64_t at = 0;
                    for (uint32_t r = 0; r < p; r++) {
                        rq.vCounts[r] = t == 0 ? 7 : (t == 1 ? 1 : 1 + next() % (t < 5 ? 50 : (t < 9 ? 100000 : (1u << 26))));   // equal, tiny, mixed
                        rq.vDispls[r] = at;
                        at += rq.vCounts[r];
                    }
                    Plan direct, fromTable;
                    if (BuildPlan(rq, &direct, &err) != 0) {
                        printf("plan failed: %s\n", err.c_str());
                        return 1;
                    }
                    if (!have) {
                        if (BuildPlanTemplate(rq, &bt, &fromTable, &err) != 0) {
                            printf("block template failed: %s\n", err.c_str());
                            return 1;
                        }
                        have = true;
                        if (DescribePlan(fromTable) != DescribePlan(direct)) {
                            printf("plan returned with the block template differs: algo %d p %u\n", algo, p);
                            return 1;
                        }
                        if (bt.blockTable != (algo != int(ALGO_MESH))) {
                            printf("block template %s: algo %d p %u\n", bt.blockTable ? "made for a schedule that cuts blocks" : "missing", algo, p);
                            return 1;
                        }
                        continue;
                    }
                    if (!bt.blockTable) {
                        continue;       // the piece-cut mesh cuts blocks: no template
                    }
                    if (!PlanFromTemplate(rq, bt, &fromTable)) {
                        printf("block table not derived: algo %d p %u table %d\n", algo, p, t);
                        return 1;
                    }
                    if (DescribePlan(fromTable) != DescribePlan(direct)) {
                        printf("plan derived from the block template differs: algo %d p %u unit %u table %d\n", algo, p, unit, t);
                        return 1;
                    }
                    tables++;
                }
                // a gap between blocks or an empty block: not this template's case
                if (bt.blockTable) {
                    PlanRequest gap = base;
                    gap.vCounts.assign(p, 5);
                    gap.vDispls.resize(p);
                    for (uint32_t r = 0; r < p; r++) {
                        gap.vDispls[r] = r * 6;
                    }
                    Plan none;
                    if (PlanFromTemplate(gap, bt, &none)) {
                        printf("a table with gaps was derived\n");
                        return 1;
                    }
                    gap.vCounts[p - 1] = 0;
                    if (PlanFromTemplate(gap, bt, &none)) {
                        printf("a table with an empty block was derived\n");
                        return 1;
                    }
                    PlanRequest inPlace = base;
                    inPlace.vCounts.assign(p, 5);
                    inPlace.vDispls.resize(p);
                    for (uint32_t r = 0; r < p; r++) {
                        inPlace.vDispls[r] = r * 5;
                    }
                    inPlace.alias.assign(p, 1);
                    PlanTemplate ip;
                    if (BuildPlanTemplate(inPlace, &ip, &none, &err) != 0 || ip.blockTable || PlanFromTemplate(inPlace, bt, &none)) {
                        printf("an in-place table got a block template\n");
                        return 1;
                    }
                }
            }
        }
    }
    printf("OK %d cases, %d derived, %d refused, %d ragged counts derived from whole-slice templates, %d block tables derived\n", cases, derived,
        refused, ragged, tables);
    return 0;
}
