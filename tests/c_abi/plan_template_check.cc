// Plans derived from a template of another count against plans made from scratch, on the host
// (cann-hccl_amd/csrc/plan.cc alone, no GPU): wherever PlanFromTemplate says it can derive a plan, the derived plan
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
                    if (BuildPlanTemplate(r0, &tmpl, &err) != 0) {
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
    // requests without a count have no template
    PlanRequest v;
    v.coll = COLL_ALLGATHER;
    v.p = 4;
    v.vCounts = {1, 2, 3, 4};
    v.vDispls = {0, 1, 3, 6};
    v.alias.assign(4, 0);
    PlanTemplate tv;
    std::string err;
    Plan out;
    if (BuildPlanTemplate(v, &tv, &err) != 0 || tv.count != 0 || PlanFromTemplate(v, tv, &out)) {
        printf("a variable-count request got a template\n");
        return 1;
    }
    printf("OK %d cases, %d derived, %d refused, %d ragged counts derived from whole-slice templates\n", cases, derived, refused, ragged);
    return 0;
}
