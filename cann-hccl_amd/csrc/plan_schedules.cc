// The schedules: every collective laid out on "virtual" buffers the way the reference runs it on its CCL staging buffers
// (partial results accumulate in the input buffer), as phases of copy / reduce steps.  One slice plan per chunk of the
// executor-level loop; the same phase of different chunks is merged into one phase.
#include "plan_internal.h"

namespace hcclamd {
namespace planner {

namespace {

void Emit(VProgram &vp, size_t phase, bool reduce, Ref dst, Ref a, Ref b, uint64_t bytes)
{
    if (bytes == 0) {
        return;
    }
    phase += vp.phaseBase;
    if (!vp.rankMap.empty()) {
        dst.rank = vp.rankMap[dst.rank];
        a.rank = vp.rankMap[a.rank];
        if (reduce) {
            b.rank = vp.rankMap[b.rank];
        }
    }
    if (vp.phases.size() <= phase) {
        vp.phases.resize(phase + 1);
    }
    Step s;
    s.reduce = reduce;
    s.dst = dst;
    s.a = a;
    s.b = b;
    s.bytes = bytes;
    vp.phases[phase].steps.push_back(s);
}
void EmitCopy(VProgram &vp, size_t phase, Ref dst, Ref src, uint64_t bytes) { Emit(vp, phase, false, dst, src, Ref(), bytes); }
void EmitReduce(VProgram &vp, size_t phase, Ref dst, Ref own, Ref peer, uint64_t bytes) { Emit(vp, phase, true, dst, own, peer, bytes); }

uint64_t SpanBytes(const std::vector<Slice> &sl, uint32_t first, uint32_t n)
{
    uint64_t s = 0;
    for (uint32_t i = first; i < first + n; i++) {
        s += sl[i].size;
    }
    return s;
}

// Ring reduce-scatter over `in` slices; the last step of each rank writes (outBuf, outSl[rank]).
// Phase k (k = 0..p-2): rank r combines its slice (r-2-k) with the left neighbour's copy of it.
size_t RingReduceScatterPhases(VProgram &vp, size_t phase0, uint32_t p, uint64_t base, const std::vector<Slice> &in,
    uint8_t outBuf, uint64_t outBase, const std::vector<Slice> &out)
{
    for (uint32_t k = 0; k + 1 < p; k++) {
        bool last = (k + 2 == p);
        for (uint32_t r = 0; r < p; r++) {
            uint32_t s = Mod(static_cast<int64_t>(r) - 2 - k, p);
            uint32_t left = Mod(static_cast<int64_t>(r) - 1, p);
            Ref own = MkRef(r, BUF_SEND, base + in[s].off);
            Ref peer = MkRef(left, BUF_SEND, base + in[s].off);
            Ref dst = last ? MkRef(r, outBuf, outBase + out[s].off) : own;
            EmitReduce(vp, phase0 + k, dst, own, peer, in[s].size);
        }
    }
    return phase0 + (p - 1);
}

// Ring all-gather on the output buffer: phase k, rank r takes slice (r-1-k) from its left neighbour.
size_t RingAllGatherPhases(VProgram &vp, size_t phase0, uint32_t p, uint64_t base, const std::vector<Slice> &sl)
{
    for (uint32_t k = 0; k + 1 < p; k++) {
        for (uint32_t r = 0; r < p; r++) {
            uint32_t s = Mod(static_cast<int64_t>(r) - 1 - k, p);
            uint32_t left = Mod(static_cast<int64_t>(r) - 1, p);
            EmitCopy(vp, phase0 + k, MkRef(r, BUF_RECV, base + sl[s].off), MkRef(left, BUF_RECV, base + sl[s].off), sl[s].size);
        }
    }
    return phase0 + (p - 1);
}

// The ring reduce-scatter and all-gather with the slices' chains ending at other ranks than "slice i at rank i":
// slice i is reduced along owner[i] + 1 -> owner[i] + 2 -> ... -> owner[i] and later leaves from owner[i].
// This is the data flow of the port-pruned reduce-scatter of an 8-rank ring (ReduceScatterRing::RunReduceScatterChunk,
// reduce_scatter_ring.cc:299-477 with the send lists of ReduceScatterSlicesPrep, :458-477): with n ranks that own a
// network port the 8 slices form n chunks of 8 / n, chunk j belongs to the j-th port rank, and every rank sends, in
// the order of the ring distance to the port rank behind it, the chunks of the port ranks other than itself.  Hop h
// of a slice's chain is phase h - 1 here, as in the plain ring; a rank combines its own copy (left operand) with
// what its left neighbour sends.
size_t OwnedRingReduceScatterPhases(VProgram &vp, size_t phase0, uint32_t p, uint64_t base, const std::vector<Slice> &sl,
    const std::vector<uint32_t> &owner)
{
    for (uint32_t k = 0; k + 1 < p; k++) {
        for (uint32_t i = 0; i < sl.size(); i++) {
            uint32_t r = (owner[i] + 2 + k) % p, left = (owner[i] + 1 + k) % p;
            Ref own = MkRef(r, BUF_SEND, base + sl[i].off);
            EmitReduce(vp, phase0 + k, own, own, MkRef(left, BUF_SEND, base + sl[i].off), sl[i].size);
        }
    }
    return phase0 + (p - 1);
}

size_t OwnedRingAllGatherPhases(VProgram &vp, size_t phase0, uint32_t p, uint64_t base, const std::vector<Slice> &sl,
    const std::vector<uint32_t> &owner)
{
    for (uint32_t k = 0; k + 1 < p; k++) {
        for (uint32_t i = 0; i < sl.size(); i++) {
            uint32_t r = (owner[i] + 1 + k) % p, left = (owner[i] + k) % p;
            EmitCopy(vp, phase0 + k, MkRef(r, BUF_RECV, base + sl[i].off), MkRef(left, BUF_RECV, base + sl[i].off), sl[i].size);
        }
    }
    return phase0 + (p - 1);
}

// Port ranks of a mask in ascending order (the executor sorts its list, coll_comm_executor.cc:1768), and for every
// slice of an 8-rank ring the rank its chain ends at.  Empty: no pruning.
std::vector<uint32_t> PrunedRingOwners(uint32_t p, uint32_t nicMask)
{
    std::vector<uint32_t> nic, owner;
    for (uint32_t r = 0; r < 8; r++) {
        if ((nicMask >> r) & 1u) {
            nic.push_back(r);
        }
    }
    if (p != 8 || nic.empty() || nic.size() == 8) {
        return owner;
    }
    const uint32_t chunk = 8 / uint32_t(nic.size());
    for (uint32_t i = 0; i < 8; i++) {
        owner.push_back(nic[i / chunk]);
    }
    return owner;
}

// Deterministic mesh reduce-scatter: every rank slice is cut into (p-1) pieces, piece t follows the
// peer order rotated by t, so that in each round the pieces of one rank read p-1 different peers.
// Atomic variant (reduce_scatter_mesh_atomic.cc:82-141): no piece cut; stream j of rank r pulls the
// whole slice r from rank (r+1+j) and accumulates it into the rank's own copy.  The reference lets
// the p-1 streams race (accumulation in arrival order); here they are taken in stream order, one of
// the orders the reference can produce.
size_t MeshReduceScatterPhases(VProgram &vp, size_t phase0, uint32_t p, uint64_t base, const std::vector<Slice> &sl,
    uint64_t align, bool atomic)
{
    uint32_t nstream = (p > 2 && !atomic) ? p - 1 : 1;
    for (uint32_t r = 0; r < p; r++) {
        if (sl[r].size == 0) {
            continue;
        }
        std::vector<Slice> pieces = RingSlicePlan(sl[r].size, nstream, align);
        for (uint32_t t = 0; t < nstream; t++) {
            for (uint32_t round = 1; round < p; round++) {
                uint32_t order = (round + t - 1) % (p - 1);
                uint32_t src = atomic ? (r + round) % p : Mod(static_cast<int64_t>(r) - (order + 1), p);
                uint64_t off = base + sl[r].off + pieces[t].off;
                EmitReduce(vp, phase0 + round - 1, MkRef(r, BUF_SEND, off), MkRef(r, BUF_SEND, off), MkRef(src, BUF_SEND, off),
                    pieces[t].size);
            }
        }
    }
    return phase0 + (p - 1);
}

// Mesh all-gather: every rank pulls slice d from rank d, all peers at once (one phase).
size_t MeshAllGatherPhases(VProgram &vp, size_t phase0, uint32_t p, uint64_t base, const std::vector<Slice> &sl)
{
    for (uint32_t r = 0; r < p; r++) {
        for (uint32_t k = 1; k < p; k++) {
            uint32_t d = (r + k) % p;
            EmitCopy(vp, phase0, MkRef(r, BUF_RECV, base + sl[d].off), MkRef(d, BUF_RECV, base + sl[d].off), sl[d].size);
        }
    }
    return phase0 + 1;
}

// Halving steps of the in-block reduce-scatter (reduce_scatter_halving_doubling.cc:67-91,193-238): in
// step s block rank q keeps the half of its current range that contains its own slice and combines
// it with the same range of block rank q ^ mask.
size_t HalvingSteps(VProgram &vp, size_t ph, uint32_t block, const std::vector<uint32_t> &rankOf, uint64_t base,
    const std::vector<Slice> &sl)
{
    uint32_t steps = 0;
    while ((1u << steps) < block) {
        steps++;
    }
    for (uint32_t s = 0; s < steps; s++) {
        uint32_t mask = 1u << (steps - s - 1);
        for (uint32_t q = 0; q < block; q++) {
            uint32_t first = q & ~(mask - 1);
            uint64_t off = base + sl[first].off;
            EmitReduce(vp, ph, MkRef(rankOf[q], BUF_SEND, off), MkRef(rankOf[q], BUF_SEND, off),
                MkRef(rankOf[q ^ mask], BUF_SEND, off), SpanBytes(sl, first, mask));
        }
        ph++;
    }
    return ph;
}

void AllReduceChunk(VProgram &vp, Algo algo, uint32_t p, uint64_t base, uint64_t bytes, uint64_t align, bool meshAtomic,
    uint32_t nicMask = 0)
{
    if (p == 1) {
        EmitCopy(vp, 0, MkRef(0, BUF_RECV, base), MkRef(0, BUF_SEND, base), bytes);
        return;
    }
    const std::vector<uint32_t> owner = algo == ALGO_RING ? PrunedRingOwners(p, nicMask) : std::vector<uint32_t>();
    if (!owner.empty()) {
        // Port-pruned ring: reduce-scatter on the input buffer with every chunk's chains ending at its port rank;
        // the all-gather hands the finished slices round the ring from there (the reference tree holds no
        // port-pruned form of the all-gather template; this one only moves bytes).
        std::vector<Slice> sl = RingSlicePlan(bytes, p, align);
        size_t ph = OwnedRingReduceScatterPhases(vp, 0, p, base, sl, owner);
        for (uint32_t i = 0; i < p; i++) {
            EmitCopy(vp, ph, MkRef(owner[i], BUF_RECV, base + sl[i].off), MkRef(owner[i], BUF_SEND, base + sl[i].off), sl[i].size);
        }
        OwnedRingAllGatherPhases(vp, ph + 1, p, base, sl, owner);
        return;
    }
    if (algo == ALGO_RING || algo == ALGO_MESH) {
        std::vector<Slice> sl = RingSlicePlan(bytes, p, align);
        size_t ph = 0;
        if (algo == ALGO_RING) {
            // the ring template runs its reduce-scatter with output == input
            ph = RingReduceScatterPhases(vp, ph, p, base, sl, BUF_SEND, base, sl);
        } else {
            ph = MeshReduceScatterPhases(vp, ph, p, base, sl, align, meshAtomic);
        }
        for (uint32_t r = 0; r < p; r++) {
            EmitCopy(vp, ph, MkRef(r, BUF_RECV, base + sl[r].off), MkRef(r, BUF_SEND, base + sl[r].off), sl[r].size);
        }
        ph++;
        if (algo == ALGO_RING) {
            RingAllGatherPhases(vp, ph, p, base, sl);
        } else {
            MeshAllGatherPhases(vp, ph, p, base, sl);
        }
        return;
    }
    // recursive halving-doubling
    uint32_t block, part1;
    HalvingDoublingShape(p, &block, &part1);
    std::vector<Slice> sl = RingSlicePlan(bytes, block, align);
    std::vector<uint32_t> rankOf(block);
    for (uint32_t i = 0; i < p; i++) {
        if (i < part1 && (i & 1)) {
            continue;
        }
        rankOf[i < part1 ? i / 2 : i - part1 / 2] = i;
    }
    uint32_t steps = 0;
    while ((1u << steps) < block) {
        steps++;
    }
    size_t ph = 0;
    if (part1 > 0) {
        for (uint32_t e = 0; e < part1; e += 2) {   // fold the odd rank of each pair into the even one
            EmitReduce(vp, ph, MkRef(e, BUF_SEND, base), MkRef(e, BUF_SEND, base), MkRef(e + 1, BUF_SEND, base), bytes);
        }
        ph++;
    }
    ph = HalvingSteps(vp, ph, block, rankOf, base, sl);
    for (uint32_t q = 0; q < block; q++) {
        EmitCopy(vp, ph, MkRef(rankOf[q], BUF_RECV, base + sl[q].off), MkRef(rankOf[q], BUF_SEND, base + sl[q].off), sl[q].size);
    }
    ph++;
    for (uint32_t s = 0; s < steps; s++) {           // doubling: fetch the peer's gathered range
        uint32_t mask = 1u << s;
        for (uint32_t q = 0; q < block; q++) {
            uint32_t peer = q ^ mask;
            uint32_t first = peer & ~(mask - 1);
            uint64_t off = base + sl[first].off;
            EmitCopy(vp, ph, MkRef(rankOf[q], BUF_RECV, off), MkRef(rankOf[peer], BUF_RECV, off), SpanBytes(sl, first, mask));
        }
        ph++;
    }
    if (part1 > 0) {
        for (uint32_t e = 0; e < part1; e += 2) {   // unfold: the odd rank receives the whole result
            EmitCopy(vp, ph, MkRef(e + 1, BUF_RECV, base), MkRef(e, BUF_RECV, base), bytes);
        }
    }
}

// Device orders of the four rings of the 8-device ring topology (coll_comm_executor.cc:1595-1606).
const uint32_t kRingOrders8[4][8] = {
    {0, 1, 2, 6, 5, 4, 7, 3}, {0, 3, 7, 4, 5, 6, 2, 1}, {0, 2, 3, 1, 5, 7, 6, 4}, {0, 4, 6, 7, 5, 1, 3, 2}};

// Two-level all-reduce of one chunk: `servers` groups of D = p / servers consecutive ranks.
//   level 0  reduce-scatter inside every group over the ring slice plan for D:
//            mesh (CollAllReduceMeshExecutor::KernelRun, coll_all_reduce_mesh_executor.cc:102-118), or ring
//            (CollAllReduceRingExecutor::KernelRun, coll_all_reduce_ring_executor.cc:95-135), the latter over one
//            ring in rank order or over the four rings of the 8-device topology: every slice is cut into one
//            part per ring (MutliSegSlicePrepare, coll_comm_executor.cc:1681-1720) and ring k, whose i-th
//            member is device order[k][i], runs the ring schedule on part k of its members' slices
//            (PrepareMultiRingSlice, :1761-1833), so that every device still ends with its own slice
//   level 1  ranks with the same position d in their groups all-reduce slice d among themselves, ring
//            or recursive halving-doubling, from the input range to the output range
//            (coll_all_reduce_mesh_executor.cc:120-196, coll_all_reduce_ring_executor.cc:137-225)
//   level 0  all-gather of the slices inside every group on the output, mesh or the same rings
//            (coll_all_reduce_mesh_executor.cc:198-236, coll_all_reduce_ring_executor.cc:227-240)
// With one group the middle level is the copy of the own slice and this is the plain one-level all-reduce.
void TwoLevelAllReduceChunk(VProgram &vp, Algo level1, uint32_t p, uint32_t servers, uint32_t level0Rings, uint64_t base,
    uint64_t bytes, uint64_t align, bool meshAtomic)
{
    const uint32_t D = p / servers;
    std::vector<Slice> sl = RingSlicePlan(bytes, D, align);
    const size_t l1 = D > 1 ? D - 1 : 0;
    VProgram shape;   // how many phases the level-1 schedule has (it does not depend on the size)
    AllReduceChunk(shape, level1, servers, 0, uint64_t(servers) * align * 64, align, false);
    const size_t l2 = l1 + shape.phases.size();
    for (uint32_t s = 0; s < servers && D > 1; s++) {
        vp.rankMap.resize(D);
        if (level0Rings == 0) {
            for (uint32_t d = 0; d < D; d++) {
                vp.rankMap[d] = s * D + d;
            }
            vp.phaseBase = 0;
            MeshReduceScatterPhases(vp, 0, D, base, sl, align, meshAtomic);
            vp.phaseBase = l2;
            MeshAllGatherPhases(vp, 0, D, base, sl);
            continue;
        }
        for (uint32_t k = 0; k < level0Rings; k++) {
            std::vector<Slice> part(D);
            for (uint32_t i = 0; i < D; i++) {
                uint32_t dev = level0Rings > 1 ? kRingOrders8[k][i] : i;
                vp.rankMap[i] = s * D + dev;
                std::vector<Slice> cut = RingSlicePlan(sl[dev].size, level0Rings, align);
                part[i] = Slice{sl[dev].off + cut[k].off, cut[k].size};
            }
            vp.phaseBase = 0;
            RingReduceScatterPhases(vp, 0, D, base, part, BUF_SEND, base, part);
            vp.phaseBase = l2;
            RingAllGatherPhases(vp, 0, D, base, part);
        }
    }
    for (uint32_t d = 0; d < D; d++) {
        vp.rankMap.resize(servers);
        for (uint32_t s = 0; s < servers; s++) {
            vp.rankMap[s] = s * D + d;
        }
        vp.phaseBase = l1;
        AllReduceChunk(vp, level1, servers, base + sl[d].off, sl[d].size, align, false);
    }
    vp.rankMap.clear();
    vp.phaseBase = 0;
}

// Halving-doubling shape shared by the standalone reduce-scatter / all-gather variants: block rank b
// below part1/2 stands for the rank pair (2b, 2b+1) and owns both their slices, the others own one.
struct HdShape {
    uint32_t block = 1, part1 = 0, steps = 0;
    std::vector<uint32_t> rankOf;                  // block rank -> real rank
    std::vector<std::vector<uint32_t>> owned;      // block rank -> user slices it ends up with
};

HdShape MakeHdShape(uint32_t p)
{
    HdShape h;
    HalvingDoublingShape(p, &h.block, &h.part1);
    h.rankOf.assign(h.block, 0);
    h.owned.assign(h.block, {});
    for (uint32_t i = 0; i < p; i++) {
        if (i < h.part1 && (i & 1)) {
            continue;
        }
        h.rankOf[i < h.part1 ? i / 2 : i - h.part1 / 2] = i;
    }
    for (uint32_t b = 0; b < h.block; b++) {
        if (2 * b < h.part1) {
            h.owned[b] = {2 * b, 2 * b + 1};
        } else {
            h.owned[b] = {b + h.part1 / 2};
        }
    }
    while ((1u << h.steps) < h.block) {
        h.steps++;
    }
    return h;
}

// Standalone recursive halving-doubling reduce-scatter (reduce_scatter_recursive_hd.cc:33-254) over
// user slices in[i], in place: every rank ends with its reduced slice where the slice lies in its
// input buffer.  Returns the phase after the last one used.
size_t RhdReduceScatterInPlace(VProgram &vp, uint32_t p, const std::vector<Slice> &in)
{
    HdShape h = MakeHdShape(p);
    size_t ph = 0;
    if (h.part1 > 0) {
        for (uint32_t e = 0; e < h.part1; e += 2) {
            for (uint32_t i = 0; i < p; i++) {
                EmitReduce(vp, ph, MkRef(e, BUF_SEND, in[i].off), MkRef(e, BUF_SEND, in[i].off), MkRef(e + 1, BUF_SEND, in[i].off),
                    in[i].size);
            }
        }
        ph++;
    }
    for (uint32_t s = 0; s < h.steps; s++) {
        uint32_t mask = 1u << (h.steps - s - 1);
        for (uint32_t q = 0; q < h.block; q++) {
            uint32_t first = q & ~(mask - 1);
            for (uint32_t b = first; b < first + mask; b++) {
                for (uint32_t u : h.owned[b]) {
                    EmitReduce(vp, ph, MkRef(h.rankOf[q], BUF_SEND, in[u].off), MkRef(h.rankOf[q], BUF_SEND, in[u].off),
                        MkRef(h.rankOf[q ^ mask], BUF_SEND, in[u].off), in[u].size);
                }
            }
        }
        ph++;
    }
    if (h.part1 > 0) {   // the even rank of a pair hands the odd rank its slice
        for (uint32_t e = 0; e < h.part1; e += 2) {
            EmitCopy(vp, ph, MkRef(e + 1, BUF_SEND, in[e + 1].off), MkRef(e, BUF_SEND, in[e + 1].off), in[e + 1].size);
        }
        ph++;
    }
    return ph;
}

// The same with the result copied to (BUF_RECV, outOff).
void RhdReduceScatterChunk(VProgram &vp, uint32_t p, const std::vector<Slice> &in, uint64_t outOff)
{
    size_t ph = RhdReduceScatterInPlace(vp, p, in);
    for (uint32_t r = 0; r < p; r++) {
        EmitCopy(vp, ph, MkRef(r, BUF_RECV, outOff), MkRef(r, BUF_SEND, in[r].off), in[r].size);
    }
}

// Two-level reduce-scatter of one chunk, CollReduceScatterMeshExecutor::KernelRun with several servers
// (coll_reduce_scatter_mesh_executor.cc:128-247): `servers` groups of D = p / servers consecutive ranks;
// block i of the input (the part for rank i) lies at blockOff[i].
//   level 1  ranks with the same position in their groups reduce-scatter the whole input among
//            themselves, ring or recursive halving-doubling, in place: the slice of group s is the D
//            blocks for the ranks of group s (:141-196)
//   level 0  mesh reduce-scatter inside every group over those D blocks, in place (:198-238)
//   then the rank's own block goes to the output (:240-243)
// With rings inside a group (CollReduceScatterRingExecutor::KernelRun, coll_reduce_scatter_ring_executor.cc:132-340;
// slices coll_reduce_scatter_executor.cc:250-287) level 0 is the ring schedule over the same D blocks, one ring in
// rank order or the four rings of the 8-device topology, each on its part of every block.
void TwoLevelReduceScatterChunk(VProgram &vp, Algo level1, uint32_t p, uint32_t servers, uint32_t level0Rings,
    const std::vector<uint64_t> &blockOff, uint64_t bytes, uint64_t outOff, uint64_t align, bool meshAtomic)
{
    const uint32_t D = p / servers;
    size_t l1 = 0;
    for (uint32_t d = 0; d < D && servers > 1; d++) {
        vp.rankMap.resize(servers);
        for (uint32_t s = 0; s < servers; s++) {
            vp.rankMap[s] = s * D + d;
        }
        vp.phaseBase = 0;
        // a group's slice is D separate blocks in the caller's layout: one pass of the schedule per block
        for (uint32_t k = 0; k < D; k++) {
            std::vector<Slice> in(servers);
            for (uint32_t s = 0; s < servers; s++) {
                in[s] = Slice{blockOff[s * D + k], bytes};
            }
            l1 = level1 == ALGO_RING ? RingReduceScatterPhases(vp, 0, servers, 0, in, BUF_SEND, 0, in)
                                     : RhdReduceScatterInPlace(vp, servers, in);
        }
    }
    size_t l0 = l1;
    for (uint32_t s = 0; s < servers && D > 1; s++) {
        vp.rankMap.resize(D);
        std::vector<Slice> sl(D);
        for (uint32_t d = 0; d < D; d++) {
            vp.rankMap[d] = s * D + d;
            sl[d] = Slice{blockOff[s * D + d], bytes};
        }
        vp.phaseBase = l1;
        if (level0Rings == 0) {
            l0 = l1 + MeshReduceScatterPhases(vp, 0, D, 0, sl, align, meshAtomic);
            continue;
        }
        std::vector<Slice> cut = RingSlicePlan(bytes, level0Rings, align);   // every block has the same size
        for (uint32_t k = 0; k < level0Rings; k++) {
            std::vector<Slice> part(D);
            for (uint32_t i = 0; i < D; i++) {
                uint32_t dev = level0Rings > 1 ? kRingOrders8[k][i] : i;
                vp.rankMap[i] = s * D + dev;
                part[i] = Slice{blockOff[s * D + dev] + cut[k].off, cut[k].size};
            }
            l0 = l1 + RingReduceScatterPhases(vp, 0, D, 0, part, BUF_SEND, 0, part);
        }
    }
    vp.rankMap.clear();
    vp.phaseBase = 0;
    for (uint32_t r = 0; r < p; r++) {
        EmitCopy(vp, l0, MkRef(r, BUF_RECV, outOff), MkRef(r, BUF_SEND, blockOff[r]), bytes);
    }
}

// Two-level ring reduce-scatter of one chunk when only some of a server's 8 devices have a network port: the isMultiNic
// branch of CollReduceScatterRingExecutor::KernelRun (coll_reduce_scatter_ring_executor.cc:150-170, 264-300), ring
// between the servers.  Block i of the input lies at blockOff[i]; the reference works on a staged copy in which the
// blocks follow each other, so a range of that copy is taken block by block here.
//   1. all-reduce of the whole input inside every server over the four rings (MultiRingAllReduce, coll_comm_executor.cc:
//      44-170): the p blocks together are cut into 8 slices (PrepareSliceData) and every slice into one part per ring;
//      the reference gathers on its scratch buffer and copies back (:160-168), here the parts go round on the input
//   2. the devices with a port reduce-scatter the whole input among the same devices of all servers (:172-191)
//   3. the port devices hand the blocks of their server's slice on, part k of a block along ring k
//      (MultiRingMultiRootScatter, coll_comm_executor.cc:1312-1415; multi_root_scatter_ring.cc:299-345): with n ports
//      a ring's 8 parts form n runs of 8 / n, run j leaves the ring position of the j-th port (positions ascending),
//      and part i of the order rotated by the first port's position stops at position (i + that position) % 8
//   4. the rank's own block goes to the output (:298-299)
void PrunedTwoLevelReduceScatterChunk(VProgram &vp, uint32_t p, uint32_t servers, uint32_t nicMask,
    const std::vector<uint64_t> &blockOff, uint64_t bytes, uint64_t outOff, uint64_t align)
{
    const uint32_t D = 8, rings = 4;
    VProgram flat;       // step 1 on the staged layout: offsets count through the blocks
    std::vector<Slice> sl = RingSlicePlan(bytes * p, D, align);
    for (uint32_t s = 0; s < servers; s++) {
        flat.rankMap.resize(D);
        for (uint32_t k = 0; k < rings; k++) {
            std::vector<Slice> part(D);
            for (uint32_t i = 0; i < D; i++) {
                const uint32_t dev = kRingOrders8[k][i];
                flat.rankMap[i] = s * D + dev;
                std::vector<Slice> cut = RingSlicePlan(sl[dev].size, rings, align);
                part[i] = Slice{sl[dev].off + cut[k].off, cut[k].size};
            }
            RingReduceScatterPhases(flat, 0, D, 0, part, BUF_SEND, 0, part);
            for (uint32_t h = 0; h + 1 < D; h++) {
                for (uint32_t r = 0; r < D; r++) {
                    const uint32_t i = Mod(int64_t(r) - 1 - h, D), left = Mod(int64_t(r) - 1, D);
                    EmitCopy(flat, D - 1 + h, MkRef(r, BUF_SEND, part[i].off), MkRef(left, BUF_SEND, part[i].off), part[i].size);
                }
            }
        }
    }
    for (size_t ph = 0; ph < flat.phases.size(); ph++) {
        for (const Step &st : flat.phases[ph].steps) {
            uint64_t at = st.a.off, left = st.bytes;
            while (left > 0) {
                const uint64_t block = at / bytes, within = at % bytes, n = std::min(left, bytes - within);
                Step piece = st;
                piece.dst.off = piece.a.off = blockOff[block] + within;
                if (st.reduce) {
                    piece.b.off = piece.a.off;
                }
                Emit(vp, ph, piece.reduce, piece.dst, piece.a, piece.b, n);
                at += n;
                left -= n;
            }
        }
    }
    const size_t l1 = flat.phases.size();
    std::vector<uint32_t> nic;
    for (uint32_t d = 0; d < D; d++) {
        if ((nicMask >> d) & 1u) {
            nic.push_back(d);
        }
    }
    for (uint32_t d : nic) {
        vp.rankMap.resize(servers);
        for (uint32_t s = 0; s < servers; s++) {
            vp.rankMap[s] = s * D + d;
        }
        vp.phaseBase = l1;
        for (uint32_t k = 0; k < D && servers > 1; k++) {
            std::vector<Slice> in(servers);
            for (uint32_t s = 0; s < servers; s++) {
                in[s] = Slice{blockOff[s * D + k], bytes};
            }
            RingReduceScatterPhases(vp, 0, servers, 0, in, BUF_SEND, 0, in);
        }
    }
    vp.rankMap.clear();
    vp.phaseBase = 0;
    const size_t l2 = l1 + (servers - 1);
    const uint32_t run = D / uint32_t(nic.size());
    std::vector<Slice> cut = RingSlicePlan(bytes, rings, align);
    size_t l3 = l2;
    for (uint32_t s = 0; s < servers; s++) {
        for (uint32_t k = 0; k < rings; k++) {
            std::vector<uint32_t> portAt;       // ring positions of the port devices
            for (uint32_t i = 0; i < D; i++) {
                if ((nicMask >> kRingOrders8[k][i]) & 1u) {
                    portAt.push_back(i);
                }
            }
            for (uint32_t j = 0; j < D; j++) {
                const uint32_t from = portAt[j / run], to = (j + portAt[0]) % D, hops = (to + D - from) % D;
                const uint64_t off = blockOff[s * D + kRingOrders8[k][to]] + cut[k].off;
                for (uint32_t h = 0; h < hops; h++) {
                    EmitCopy(vp, l2 + h, MkRef(s * D + kRingOrders8[k][(from + h + 1) % D], BUF_SEND, off),
                        MkRef(s * D + kRingOrders8[k][(from + h) % D], BUF_SEND, off), cut[k].size);
                }
                l3 = std::max(l3, l2 + hops);
            }
        }
    }
    for (uint32_t r = 0; r < p; r++) {
        EmitCopy(vp, l3, MkRef(r, BUF_RECV, outOff), MkRef(r, BUF_SEND, blockOff[r]), bytes);
    }
}

// Standalone recursive halving-doubling all-gather (all_gather_recursive_hd.cc:26-238) on the output
// buffer; phase0 is the first phase after the ranks copied their own block in.
void RhdAllGatherChunk(VProgram &vp, size_t phase0, uint32_t p, const std::vector<Slice> &sl)
{
    HdShape h = MakeHdShape(p);
    size_t ph = phase0;
    if (h.part1 > 0) {
        for (uint32_t e = 0; e < h.part1; e += 2) {
            EmitCopy(vp, ph, MkRef(e, BUF_RECV, sl[e + 1].off), MkRef(e + 1, BUF_RECV, sl[e + 1].off), sl[e + 1].size);
        }
        ph++;
    }
    for (uint32_t s = 0; s < h.steps; s++) {
        uint32_t mask = 1u << s;
        for (uint32_t q = 0; q < h.block; q++) {
            uint32_t peer = q ^ mask;
            uint32_t first = peer & ~(mask - 1);
            for (uint32_t b = first; b < first + mask; b++) {
                for (uint32_t u : h.owned[b]) {
                    EmitCopy(vp, ph, MkRef(h.rankOf[q], BUF_RECV, sl[u].off), MkRef(h.rankOf[peer], BUF_RECV, sl[u].off), sl[u].size);
                }
            }
        }
        ph++;
    }
    if (h.part1 > 0) {
        for (uint32_t e = 0; e < h.part1; e += 2) {
            for (uint32_t i = 0; i < p; i++) {
                EmitCopy(vp, ph, MkRef(e + 1, BUF_RECV, sl[i].off), MkRef(e, BUF_RECV, sl[i].off), sl[i].size);
            }
        }
    }
}

// Two-level all-gather of one chunk (CollAllGatherMeshExecutor::KernelRun, coll_all_gather_mesh_executor.cc:71-175;
// CollAllGatherRingExecutor::KernelRun, coll_all_gather_ring_executor.cc:81-200), after every rank copied its own
// block in (phase 0): the all-gather inside every group of D = p / servers consecutive ranks over the group's D
// blocks (mesh, one ring, or the four rings of the 8-device topology on quarters of every block), then the ranks
// at position d of all groups exchange their groups' D blocks, ring or recursive halving-doubling.
// sl[i] = where block i lies in every output buffer.
void TwoLevelAllGatherChunk(VProgram &vp, Algo level1, uint32_t p, uint32_t servers, uint32_t level0Rings,
    const std::vector<Slice> &sl, uint64_t align)
{
    const uint32_t D = p / servers;
    const size_t l0 = D > 1 ? (level0Rings == 0 ? 1 : D - 1) : 0;
    for (uint32_t s = 0; s < servers && D > 1; s++) {
        std::vector<Slice> own(sl.begin() + size_t(s) * D, sl.begin() + size_t(s + 1) * D);
        vp.rankMap.resize(D);
        vp.phaseBase = 1;
        if (level0Rings == 0) {
            for (uint32_t d = 0; d < D; d++) {
                vp.rankMap[d] = s * D + d;
            }
            MeshAllGatherPhases(vp, 0, D, 0, own);
            continue;
        }
        for (uint32_t k = 0; k < level0Rings; k++) {
            std::vector<Slice> part(D);
            for (uint32_t i = 0; i < D; i++) {
                uint32_t dev = level0Rings > 1 ? kRingOrders8[k][i] : i;
                vp.rankMap[i] = s * D + dev;
                std::vector<Slice> cut = RingSlicePlan(own[dev].size, level0Rings, align);
                part[i] = Slice{own[dev].off + cut[k].off, cut[k].size};
            }
            RingAllGatherPhases(vp, 0, D, 0, part);
        }
    }
    for (uint32_t d = 0; d < D && servers > 1; d++) {
        vp.rankMap.resize(servers);
        for (uint32_t s = 0; s < servers; s++) {
            vp.rankMap[s] = s * D + d;
        }
        vp.phaseBase = 1 + l0;
        for (uint32_t k = 0; k < D; k++) {          // a group's blocks need not be neighbours in the caller's layout
            std::vector<Slice> blk(servers);
            for (uint32_t s = 0; s < servers; s++) {
                blk[s] = sl[size_t(s) * D + k];
            }
            if (level1 == ALGO_RING) {
                RingAllGatherPhases(vp, 0, servers, 0, blk);
            } else {
                RhdAllGatherChunk(vp, 0, servers, blk);
            }
        }
    }
    vp.rankMap.clear();
    vp.phaseBase = 0;
}

// Ring reduce (reduce_ring.cc:29-154) among n ranks of `bytes` bytes at `off` in their input buffers:
// the data walks root+1 -> ... -> root, every rank combining its own with what arrives; the last
// combine writes `result` instead of the root's input.  Returns the phase after the last one used.
size_t RingReducePhases(VProgram &vp, uint32_t n, uint32_t root, uint64_t off, uint64_t bytes, const Ref &result)
{
    for (uint32_t d = 2; d <= n; d++) {
        uint32_t r = (root + d) % n, prev = (root + d - 1) % n;
        Ref own = MkRef(r, BUF_SEND, off);
        EmitReduce(vp, d - 2, d == n ? result : own, own, MkRef(prev, BUF_SEND, off), bytes);
    }
    return n > 1 ? n - 1 : 0;
}

// Recursive halving-doubling reduce (reduce_recursive_hd.cc:31-316) among n ranks: in every rank pair
// of part one the rank with the root's parity folds its neighbour in (:85-148), the block runs the
// halving reduce-scatter (:150-183), and a binomial gather over the output buffers brings the slices
// to the root (:236-313).  The gather only forwards finished slices, so here each slice goes from the
// rank that reduced it straight to `result` (rank and buffer of the destination; its offset is that
// of the start of the data).  Returns the phase after the last one used.
size_t RhdReducePhases(VProgram &vp, uint32_t n, uint32_t root, uint64_t off, uint64_t bytes, uint64_t align, const Ref &result)
{
    uint32_t block, part1;
    HalvingDoublingShape(n, &block, &part1);
    const uint32_t par = (root >= part1 ? 0u : root) % 2;
    std::vector<uint32_t> rankOf(block);
    for (uint32_t b = 0; b < block; b++) {
        rankOf[b] = b < part1 / 2 ? 2 * b + par : b + part1 / 2;
    }
    std::vector<Slice> sl = RingSlicePlan(bytes, block, align);
    size_t ph = 0;
    if (part1 > 0) {
        for (uint32_t b = 0; b < part1 / 2; b++) {
            uint32_t mbr = rankOf[b], other = mbr ^ 1u;
            EmitReduce(vp, ph, MkRef(mbr, BUF_SEND, off), MkRef(mbr, BUF_SEND, off), MkRef(other, BUF_SEND, off), bytes);
        }
        ph++;
    }
    ph = HalvingSteps(vp, ph, block, rankOf, off, sl);
    for (uint32_t b = 0; b < block; b++) {
        Ref dst = result;
        dst.off += sl[b].off;
        EmitCopy(vp, ph, dst, MkRef(rankOf[b], BUF_SEND, off + sl[b].off), sl[b].size);
    }
    return ph + 1;
}

// Two-level reduce of one chunk, CollReduceMeshExecutor::KernelRun with several servers
// (coll_reduce_mesh_executor.cc:75-194): mesh reduce-scatter inside every group of D = p / servers
// consecutive ranks (:95-107), the ranks at position d of all groups reduce slice d towards the one
// in the root's group, ring or recursive halving-doubling (:109-160), and the root gathers the
// slices inside its group (:164-187).  The level-1 results are written straight to the root's
// output, which is where the gather would carry them.
// With rings inside a group (CollReduceRingPlusHdExecutor::KernelRun, coll_reduce_ring_plus_hd_executor.cc:75-168)
// level 0 is the ring reduce-scatter of the two-level all-reduce, one ring or the four rings of the
// 8-device topology on the parts of every slice; the rest is the same.
void TwoLevelReduceChunk(VProgram &vp, Algo level1, uint32_t p, uint32_t servers, uint32_t level0Rings, uint32_t root,
    uint64_t base, uint64_t bytes, uint64_t align, bool meshAtomic)
{
    const uint32_t D = p / servers;
    const uint32_t rootServer = root / D;
    std::vector<Slice> sl = RingSlicePlan(bytes, D, align);
    const size_t l1 = D > 1 ? D - 1 : 0;
    for (uint32_t s = 0; s < servers && D > 1; s++) {
        vp.rankMap.resize(D);
        vp.phaseBase = 0;
        if (level0Rings == 0) {
            for (uint32_t d = 0; d < D; d++) {
                vp.rankMap[d] = s * D + d;
            }
            MeshReduceScatterPhases(vp, 0, D, base, sl, align, meshAtomic);
            continue;
        }
        for (uint32_t k = 0; k < level0Rings; k++) {
            std::vector<Slice> part(D);
            for (uint32_t i = 0; i < D; i++) {
                uint32_t dev = level0Rings > 1 ? kRingOrders8[k][i] : i;
                vp.rankMap[i] = s * D + dev;
                std::vector<Slice> cut = RingSlicePlan(sl[dev].size, level0Rings, align);
                part[i] = Slice{sl[dev].off + cut[k].off, cut[k].size};
            }
            RingReduceScatterPhases(vp, 0, D, base, part, BUF_SEND, base, part);
        }
    }
    for (uint32_t d = 0; d < D; d++) {
        // local ranks 0 .. servers-1 are the groups' ranks at position d; one more entry names the root
        vp.rankMap.resize(servers + 1);
        for (uint32_t s = 0; s < servers; s++) {
            vp.rankMap[s] = s * D + d;
        }
        vp.rankMap[servers] = root;
        vp.phaseBase = l1;
        const Ref result = MkRef(servers, BUF_RECV, base + sl[d].off);
        if (servers == 1) {
            EmitCopy(vp, 0, result, MkRef(0, BUF_SEND, base + sl[d].off), sl[d].size);
        } else if (level1 == ALGO_RING) {
            RingReducePhases(vp, servers, rootServer, base + sl[d].off, sl[d].size, result);
        } else {
            RhdReducePhases(vp, servers, rootServer, base + sl[d].off, sl[d].size, align, result);
        }
    }
    vp.rankMap.clear();
    vp.phaseBase = 0;
}

// Recursive halving-doubling broadcast (bcast_recursive_halvingdoubling.cc:21-290) among n ranks, data(i) naming
// rank i's copy of the chunk: a binomial tree over the block, whole chunk per hop, widest distance first (:162-203);
// the block holds the root and, of every rank pair of part one, the rank with the root's parity (:120-160);
// afterwards that rank hands the chunk to its neighbour (:205-262).  Returns the phase after the last one used.
template <typename F> size_t RhdBroadcastPhases(VProgram &vp, size_t ph, uint32_t n, uint32_t root, F data, uint64_t bytes)
{
    uint32_t block, part1;
    HalvingDoublingShape(n, &block, &part1);
    const uint32_t par = (root < part1 && (root % 2) == 1) ? 1u : 0u;
    std::vector<uint32_t> rankOf(block);
    for (uint32_t b = 0; b < block; b++) {
        rankOf[b] = b < part1 / 2 ? 2 * b + par : b + part1 / 2;
    }
    const uint32_t rootQ = root < part1 ? root / 2 : root - part1 / 2;
    uint32_t rounds = 0;
    while ((1u << rounds) < block) {
        rounds++;
    }
    std::vector<uint8_t> has(block, 0);
    has[rootQ] = 1;
    for (uint32_t i = 0; i < rounds; i++, ph++) {
        const uint32_t mask = 1u << (rounds - i - 1);
        std::vector<uint32_t> got;
        for (uint32_t q = 0; q < block; q++) {
            if (has[q] && (q & (mask - 1)) == (rootQ & (mask - 1)) && !has[q ^ mask]) {
                EmitCopy(vp, ph, data(rankOf[q ^ mask]), data(rankOf[q]), bytes);
                got.push_back(q ^ mask);
            }
        }
        for (uint32_t q : got) {
            has[q] = 1;
        }
    }
    for (uint32_t b = 0; b < part1 / 2; b++) {
        EmitCopy(vp, ph, data(rankOf[b] ^ 1u), data(rankOf[b]), bytes);
    }
    return part1 > 0 ? ph + 1 : ph;
}

// Binary-block halving-doubling broadcast (bcast_halvingdoubling.cc:26-398) among n ranks, whole chunk per hop.  The
// ranks are cut into blocks whose sizes are the powers of two in n, the largest block at rank 0
// (PrepareBlockParams :26-62).  The chunk spreads through the root's block as a binomial tree, widest distance first
// (BcastInRootBlock :165-228), and then from block to block in both directions: into the next smaller block (the one at
// the higher ranks) every (size ratio)-th rank sends to one rank; into the next larger block every rank sends to (size
// ratio) consecutive ranks, one after the other (GatherBetweenBlocksRootBlock :231-281, ...HigherBlock :284-335,
// ...LowerBlock :338-396).  A rank's transfers keep their program order: each takes the phase after the rank's last.
template <typename F> void HdBlocksBroadcastPhases(VProgram &vp, uint32_t n, uint32_t root, F data, uint64_t bytes)
{
    struct Block {
        uint32_t first, size;
    };
    std::vector<Block> blocks;      // from the largest (rank 0) to the smallest
    for (uint32_t bit = 1u << 31, at = 0; bit != 0; bit >>= 1) {
        if ((n & bit) != 0) {
            blocks.push_back(Block{at, bit});
            at += bit;
        }
    }
    size_t home = 0;
    while (root >= blocks[home].first + blocks[home].size) {
        home++;
    }
    std::vector<size_t> free(n, 0);      // the first phase in which a rank holds the chunk and is not sending
    auto hop = [&](uint32_t from, uint32_t to) {
        EmitCopy(vp, free[from], data(to), data(from), bytes);
        free[from]++;
        free[to] = free[from];
    };
    const Block hb = blocks[home];
    const uint32_t rootIn = root - hb.first;
    std::vector<uint8_t> has(hb.size, 0);
    has[rootIn] = 1;
    for (uint32_t mask = hb.size >> 1; mask != 0; mask >>= 1) {
        std::vector<uint32_t> senders;
        for (uint32_t q = 0; q < hb.size; q++) {
            if (has[q] && !has[q ^ mask]) {
                senders.push_back(q);
            }
        }
        for (uint32_t q : senders) {
            hop(hb.first + q, hb.first + (q ^ mask));
            has[q ^ mask] = 1;
        }
    }
    auto intoSmaller = [&](size_t b) {
        const Block from = blocks[b], to = blocks[b + 1];
        const uint32_t ratio = from.size / to.size;
        for (uint32_t q = 0; q < to.size; q++) {
            hop(from.first + q * ratio, to.first + q);
        }
    };
    auto intoLarger = [&](size_t b) {
        const Block from = blocks[b], to = blocks[b - 1];
        const uint32_t ratio = to.size / from.size;
        for (uint32_t i = 0; i < ratio; i++) {
            for (uint32_t q = 0; q < from.size; q++) {
                hop(from.first + q, to.first + q * ratio + i);
            }
        }
    };
    // the root's block serves the smaller block first, then the larger one (:246-279)
    for (size_t b = home; b + 1 < blocks.size(); b++) {
        intoSmaller(b);
    }
    for (size_t b = home; b > 0; b--) {
        intoLarger(b);
    }
}

}  // namespace

int BuildVirtual(const PlanRequest &rq, VProgram *vp, std::string *err)
{
    uint32_t p = rq.p;
    uint64_t u = rq.unit;
    vp->inBytes.assign(p, 0);
    vp->outBytes.assign(p, 0);
    if (rq.coll == COLL_ALLTOALLV) {
        if (rq.sendCounts.size() != size_t(p) * p || rq.sdispls.size() != size_t(p) * p ||
            rq.recvCounts.size() != size_t(p) * p || rq.rdispls.size() != size_t(p) * p) {
            *err = "all-to-all-v tables must be p x p";
            return 1;
        }
        if (rq.servers > 1) {
            // Staged (coll_all_to_all_v_staged_executor.cc:378-470, zero-copy mode): inside a server of m ranks,
            // rank (c, l) collects from its m neighbours everything addressed to the ranks with local index l,
            // laid out by destination, then by source (coll_all_to_all_executor.cc:156-196, :235-265); then the
            // ranks with the same local index exchange those runs pairwise between the servers, each block going
            // to its place in the destination's receive buffer (:300-352; alltoallv_staged_pairwise.cc:65-147).
            if (p % rq.servers != 0) {
                *err = "staged all-to-all-v: the servers must hold the same number of ranks";
                return 1;
            }
            const uint32_t S = rq.servers, m = p / S;
            auto len = [&](uint32_t src, uint32_t dst) { return rq.sendCounts[size_t(src) * p + dst] * u; };
            for (uint32_t r = 0; r < p; r++) {
                for (uint32_t n = 0; n < p; n++) {
                    uint64_t cnt = rq.sendCounts[size_t(r) * p + n];
                    if (cnt) {
                        vp->inBytes[r] = std::max(vp->inBytes[r], (rq.sdispls[size_t(r) * p + n] + cnt) * u);
                        vp->outBytes[n] = std::max(vp->outBytes[n], (rq.rdispls[size_t(n) * p + r] + cnt) * u);
                    }
                }
            }
            // Between the servers a run larger than the CCL buffer goes in batches of the buffer's size: the blocks of
            // a run are packed into a batch in order and the block that does not fit is cut where the batch is full
            // (alltoallv_staged_pairwise.cc:143-244, the BCopy form; a run that fits is one batch, as in the ZCopy
            // form).  Batch t of a step's slowest pair is phase t of that step.  The reference stages a batch
            // through the buffer on both sides; here every part of a block goes direct.
            if (rq.cclBytes == 0) {
                *err = "CCL buffer too small";
                return 1;
            }
            std::vector<uint64_t> batches(S, 1), firstPhase(S, 2);
            for (uint32_t r = 0; r < p; r++) {
                for (uint32_t j = r % m; j < p; j += m) {
                    const uint32_t step = (j / m + S - r / m) % S;
                    uint64_t run = 0;
                    for (uint32_t k = 0; k < m; k++) {
                        run += len(r / m * m + k, j);
                    }
                    if (step > 0) {
                        batches[step] = std::max(batches[step], (run + rq.cclBytes - 1) / rq.cclBytes);
                    }
                }
            }
            for (uint32_t st = 1; st < S; st++) {
                firstPhase[st] = firstPhase[st - 1] + batches[st - 1];
            }
            vp->workBytes.assign(p, 0);
            for (uint32_t r = 0; r < p; r++) {
                const uint32_t c = r / m, l = r % m;
                const uint64_t work = (vp->inBytes[r] + 255) & ~uint64_t(255);
                uint64_t at = work;
                for (uint32_t j = l; j < p; j += m) {
                    const uint32_t step = (j / m + S - c) % S;
                    uint64_t sent = 0;      // bytes of this run handed over so far
                    for (uint32_t k = 0; k < m; k++) {
                        const uint32_t src = c * m + k;
                        const uint64_t n = len(src, j);
                        if (n) {
                            vp->blocks.push_back(VProgram::Block{rq.rdispls[size_t(j) * p + src] * u, rq.sdispls[size_t(src) * p + j] * u, n, j, src});
                        }
                        // stage one: own blocks first (LocalCopy), the neighbours' all at once (alltoallv_staged_mesh.cc:51-130)
                        EmitCopy(*vp, k == l ? 0 : 1, MkRef(r, BUF_SEND, at), MkRef(src, BUF_SEND, rq.sdispls[size_t(src) * p + j] * u), n);
                        // stage two: step i hands the run for server c + i to the rank of that server with local index l
                        const uint64_t to = rq.rdispls[size_t(j) * p + src] * u;
                        if (step == 0) {
                            EmitCopy(*vp, firstPhase[0], MkRef(j, BUF_RECV, to), MkRef(r, BUF_SEND, at), n);
                        }
                        for (uint64_t off = 0; step > 0 && off < n;) {
                            const uint64_t room = rq.cclBytes - sent % rq.cclBytes, part = std::min(room, n - off);
                            EmitCopy(*vp, firstPhase[step] + sent / rq.cclBytes, MkRef(j, BUF_RECV, to + off), MkRef(r, BUF_SEND, at + off), part);
                            off += part;
                            sent += part;
                        }
                        at += n;
                    }
                }
                vp->workBytes[r] = at - vp->inBytes[r];
            }
            return 0;
        }
        // Step i: rank r's block for rank (r+i) goes straight into that rank's receive buffer.  A block larger than
        // the CCL buffer travels in pieces of the buffer's size, one after the other (the BCopy form,
        // alltoallv_pairwise.cc:112-189, which the reference takes when a rank's send or receive extent exceeds the
        // buffer, alltoall_operator.cc:122-145; in its ZCopy form every block fits, so the one rule covers both).
        // The reference stages each piece through the buffer on both sides; here the piece goes direct.
        if (rq.cclBytes == 0) {
            *err = "CCL buffer too small";
            return 1;
        }
        vp->blocks.reserve(size_t(p) * p);
        for (uint32_t n = 0; n < p; n++) {
            for (uint32_t r = 0; r < p; r++) {
                const uint64_t cnt = rq.sendCounts[size_t(r) * p + n];
                if (cnt) {
                    vp->blocks.push_back(VProgram::Block{rq.rdispls[size_t(n) * p + r] * u, rq.sdispls[size_t(r) * p + n] * u, cnt * u, n, r});
                }
            }
        }
        vp->phases.resize(p);
        for (Phase &ph : vp->phases) {
            ph.steps.reserve(p);
        }
        size_t phase = 0;
        for (uint32_t i = 0; i < p; i++) {
            uint64_t pieces = 1;
            for (uint32_t r = 0; r < p && i > 0; r++) {
                const uint64_t bytes = rq.sendCounts[size_t(r) * p + (r + i) % p] * u;
                pieces = std::max(pieces, (bytes + rq.cclBytes - 1) / rq.cclBytes);
            }
            for (uint32_t r = 0; r < p; r++) {
                uint32_t n = (r + i) % p;
                uint64_t cnt = rq.sendCounts[size_t(r) * p + n];
                uint64_t so = rq.sdispls[size_t(r) * p + n] * u, ro = rq.rdispls[size_t(n) * p + r] * u;
                if (i == 0) {
                    EmitCopy(*vp, phase, MkRef(n, BUF_RECV, ro), MkRef(r, BUF_SEND, so), cnt * u);   // LocalCopy (:95-108)
                }
                for (uint64_t t = 0, off = 0; i > 0 && off < cnt * u; t++, off += rq.cclBytes) {
                    EmitCopy(*vp, phase + t, MkRef(n, BUF_RECV, ro + off), MkRef(r, BUF_SEND, so + off),
                        std::min(rq.cclBytes, cnt * u - off));
                }
                if (cnt) {
                    vp->inBytes[r] = std::max(vp->inBytes[r], so + cnt * u);
                    vp->outBytes[n] = std::max(vp->outBytes[n], ro + cnt * u);
                }
            }
            phase += pieces;
        }
        return 0;
    }
    if (rq.coll == COLL_SENDRECV) {
        // one block from the sender's buffer to the receiver's (send_receive.cc: TxAsync / RxAsync pair)
        if (rq.root >= p || rq.peer >= p) {
            *err = "send / receive rank out of range";
            return 1;
        }
        EmitCopy(*vp, 0, MkRef(rq.peer, BUF_RECV, 0), MkRef(rq.root, BUF_SEND, 0), rq.count * u);
        vp->inBytes[rq.root] = rq.count * u;
        vp->outBytes[rq.peer] = rq.count * u;
        return 0;
    }
    if (rq.coll == COLL_BROADCAST || rq.coll == COLL_REDUCE || rq.coll == COLL_SCATTER) {
        if (rq.root >= p) {
            *err = "root out of range";
            return 1;
        }
        const uint32_t R = rq.root;
        uint64_t total = rq.count * u;
        if (rq.coll == COLL_SCATTER && rq.algo == ALGO_RING && p > 1) {
            // ring scatter (scatter_ring.cc:22-135,142-218): the root sends the blocks to its right neighbour one
            // per step, the one with the longest way first (:38-52); every rank keeps the last block it receives
            // and passes the others on (:77-118).  Blocks in transit lie in the rank's workspace (the reference's
            // output staging buffer), at the block's own offset.
            vp->workBytes.assign(p, 0);
            vp->inBytes[R] = total * p;
            EmitCopy(*vp, 0, MkRef(R, BUF_RECV, 0), MkRef(R, BUF_SEND, uint64_t(R) * total), total);
            vp->outBytes[R] = total;
            for (uint32_t j = 1; j < p; j++) {            // j = hops from the root to the block's owner
                const uint32_t dest = (R + j) % p;
                for (uint32_t h = 1; h <= j; h++) {
                    const uint32_t from = (R + h - 1) % p, to = (R + h) % p;
                    // (a rank in transit is never the root: its input buffer is empty and all of it is workspace)
                    const Ref src = MkRef(from, BUF_SEND, uint64_t(dest) * total);
                    const Ref dst = h == j ? MkRef(dest, BUF_RECV, 0) : MkRef(to, BUF_SEND, uint64_t(dest) * total);
                    EmitCopy(*vp, size_t(p - j + h - 2), dst, src, total);
                    if (h != j) {
                        vp->workBytes[to] = std::max(vp->workBytes[to], uint64_t(dest + 1) * total);
                    }
                }
                vp->outBytes[dest] = total;
            }
            return 0;
        }
        if (rq.coll == COLL_SCATTER && rq.servers > 1) {
            // Two levels (coll_scatter_mesh_executor.cc:40-110): S groups of D consecutive ranks.  The rank at the
            // root's position in a group is the group's sub-root (topo_matcher.cc:341-370).  Level 1
            // (coll_scatter_executor.cc:198-241, the ring choice): a group's run of D blocks travels round the ring of
            // sub-roots from the root, the farthest group's first, each run at its own offset of the sub-roots'
            // workspace.  Level 0 (scatter_mesh.cc:46-160): every sub-root hands the ranks of its group their blocks.
            // The reference lands a block in the receiver's staging buffer and copies it out (:103-106); here the
            // hand-over writes the receive buffer itself.
            const uint32_t S = rq.servers, D = p / S, rootGroup = R / D, rootLocal = R % D;
            const uint64_t run = total * D;
            vp->workBytes.assign(p, 0);
            vp->inBytes[R] = total * p;
            for (uint32_t j = 1; j < S; j++) {            // j = hops from the root's group to the run's group
                const uint32_t dest = (rootGroup + j) % S;
                for (uint32_t h = 1; h <= j; h++) {
                    const uint32_t from = ((rootGroup + h - 1) % S) * D + rootLocal, to = ((rootGroup + h) % S) * D + rootLocal;
                    EmitCopy(*vp, size_t(S - j + h - 2), MkRef(to, BUF_SEND, uint64_t(dest) * run),
                        MkRef(from, BUF_SEND, uint64_t(dest) * run), run);
                    vp->workBytes[to] = std::max(vp->workBytes[to], uint64_t(dest + 1) * run);
                }
            }
            for (uint32_t r = 0; r < p && rq.level0Rings == 0; r++) {
                EmitCopy(*vp, size_t(S - 1), MkRef(r, BUF_RECV, 0), MkRef(r / D * D + rootLocal, BUF_SEND, uint64_t(r) * total), total);
                vp->outBytes[r] = total;
            }
            // With rings inside a group (coll_scatter_ring_executor.cc:42-113) level 0 is the ring scatter from the
            // sub-root instead, along the ranks in their order or, for groups of 8 set up as the four-ring topology,
            // in the order of its ring 0 (PrepareScatterRingSliceData, :115-131).
            for (uint32_t g = 0; g < S && rq.level0Rings != 0; g++) {
                auto order = [&](uint32_t i) { return rq.level0Rings == 4 ? kRingOrders8[0][i] : i; };
                uint32_t rootPos = 0;
                for (uint32_t i = 0; i < D; i++) {
                    rootPos = order(i) == rootLocal ? i : rootPos;
                }
                const uint32_t sub = g * D + rootLocal;
                EmitCopy(*vp, size_t(S - 1), MkRef(sub, BUF_RECV, 0), MkRef(sub, BUF_SEND, uint64_t(sub) * total), total);
                vp->outBytes[sub] = total;
                for (uint32_t j = 1; j < D; j++) {            // j = hops from the sub-root to the block's owner
                    const uint32_t dest = g * D + order((rootPos + j) % D);
                    for (uint32_t h = 1; h <= j; h++) {
                        const uint32_t from = g * D + order((rootPos + h - 1) % D), to = g * D + order((rootPos + h) % D);
                        const Ref src = MkRef(from, BUF_SEND, uint64_t(dest) * total);
                        const Ref dst = h == j ? MkRef(dest, BUF_RECV, 0) : MkRef(to, BUF_SEND, uint64_t(dest) * total);
                        EmitCopy(*vp, size_t(S - 1) + size_t(D - j + h - 2), dst, src, total);
                        if (h != j) {
                            vp->workBytes[to] = std::max(vp->workBytes[to], uint64_t(dest + 1) * total);
                        }
                    }
                    vp->outBytes[dest] = total;
                }
            }
            return 0;
        }
        if (rq.coll == COLL_SCATTER) {
            // mesh scatter (scatter_mesh.cc:46-160): the root hands rank i block i, all at once
            for (uint32_t r = 0; r < p; r++) {
                EmitCopy(*vp, 0, MkRef(r, BUF_RECV, 0), MkRef(R, BUF_SEND, uint64_t(r) * total), total);
                vp->outBytes[r] = total;
            }
            vp->inBytes[R] = total * p;
            return 0;
        }
        if (rq.coll == COLL_BROADCAST && rq.algo == ALGO_STAR) {
            // star broadcast (broadcast_star.cc:47-99): the root sends every other rank the whole buffer, in one go
            // (its one caller, broadcast_operator_for_hetero.cc:91-113, runs it without a chunk loop)
            for (uint32_t r = 0; r < p; r++) {
                if (r != R) {
                    EmitCopy(*vp, 0, MkRef(r, BUF_RECV, 0), MkRef(R, BUF_SEND, 0), total);
                }
                vp->inBytes[r] = (r == R) ? total : 0;
                vp->outBytes[r] = (r == R) ? 0 : total;
            }
            return 0;
        }
        uint64_t per = (rq.coll == COLL_BROADCAST || rq.coll == COLL_REDUCE) ? rq.cclBytes / u : 0;
        if (per == 0) {
            *err = "CCL buffer too small";
            return 1;
        }
        uint64_t done = 0;
        for (uint64_t left = rq.count; left > 0;) {
            uint64_t cur = std::min(left, per), bytes = cur * u;
            if (rq.coll == COLL_BROADCAST && rq.level0Rings > 0 && p > 1) {
                // The ring topologies' broadcast (coll_broadcast_ring_executor.cc:64-211): slices over the D ranks of a
                // group, every slice cut into one part per ring.  Step 1, in the root's group only: ring k runs the
                // ring scatter (scatter_ring.cc:22-135) from the root's position over part k of its members' slices --
                // the part with the longest way leaves first, a member keeps the last part it receives and passes the
                // others on.  Step 2: the ranks at position d of all groups pass slice d on by recursive
                // halving-doubling from the root's group.  Step 3: ring all-gather of the parts in every group, ring
                // by ring.  In place; the root keeps its data where it is, so what the all-gather would hand back to
                // it is left out.
                const uint32_t S = rq.servers, D = p / S, rootGroup = R / D, rings = rq.level0Rings;
                std::vector<Slice> sl = RingSlicePlan(bytes, D, rq.align);
                auto at = [&](uint32_t r, uint64_t off) {
                    return r == R ? MkRef(R, BUF_SEND, done + off) : MkRef(r, BUF_RECV, done + off);
                };
                auto device = [&](uint32_t k, uint32_t i) { return rings > 1 ? kRingOrders8[k][i] : i; };
                auto part = [&](uint32_t k, uint32_t i) {
                    const Slice &whole = sl[device(k, i)];
                    std::vector<Slice> cut = RingSlicePlan(whole.size, rings, rq.align);
                    return Slice{whole.off + cut[k].off, cut[k].size};
                };
                const size_t l1 = D > 1 ? D - 1 : 0;
                for (uint32_t k = 0; k < rings && D > 1; k++) {
                    uint32_t rootPos = 0;
                    for (uint32_t i = 0; i < D; i++) {
                        rootPos = device(k, i) == R % D ? i : rootPos;
                    }
                    for (uint32_t j = 1; j < D; j++) {            // j = hops from the root to the part's owner
                        const Slice pt = part(k, (rootPos + j) % D);
                        for (uint32_t h = 1; h <= j; h++) {
                            const uint32_t from = rootGroup * D + device(k, (rootPos + h - 1) % D);
                            const uint32_t to = rootGroup * D + device(k, (rootPos + h) % D);
                            EmitCopy(*vp, size_t(D - j + h - 2), at(to, pt.off), at(from, pt.off), pt.size);
                        }
                    }
                }
                size_t l2 = l1;
                for (uint32_t d = 0; d < D && S > 1; d++) {
                    auto data = [&](uint32_t g) { return at(g * D + d, sl[d].off); };
                    l2 = std::max(l2, RhdBroadcastPhases(*vp, l1, S, rootGroup, data, sl[d].size));
                }
                for (uint32_t g = 0; g < S && D > 1; g++) {
                    for (uint32_t k = 0; k < rings; k++) {
                        for (uint32_t h = 0; h + 1 < D; h++) {
                            for (uint32_t i = 0; i < D; i++) {
                                const uint32_t to = g * D + device(k, i), from = g * D + device(k, Mod(int64_t(i) - 1, D));
                                const Slice pt = part(k, Mod(int64_t(i) - 1 - h, D));
                                if (to != R) {
                                    EmitCopy(*vp, l2 + h, at(to, pt.off), at(from, pt.off), pt.size);
                                }
                            }
                        }
                    }
                }
            } else if (rq.coll == COLL_BROADCAST && rq.servers > 1 && p > 1) {
                // Two levels (coll_broadcast_mesh_executor.cc:59-213 with several servers): the root scatters slice d
                // to position d of its own group (scatter_mesh.cc), the ranks at position d of all groups pass it on by
                // recursive halving-doubling from the root's group, and every group gathers the slices (mesh).
                // The root keeps its data where it is.
                const uint32_t S = rq.servers, D = p / S, rootGroup = R / D;
                uint64_t avg = bytes / D + ((cur % D) > 0 ? 1 : 0);
                uint64_t slice = RoundUpTo(avg, rq.align);
                std::vector<Slice> sl(D);
                uint64_t residue = bytes;
                for (uint32_t i = 0; i < D; i++) {
                    sl[i].size = std::min(slice, residue);
                    sl[i].off = sl[i].size == 0 ? 0 : uint64_t(i) * slice;
                    residue -= sl[i].size;
                }
                auto at = [&](uint32_t r, uint32_t d) {
                    return r == R ? MkRef(R, BUF_SEND, done + sl[d].off) : MkRef(r, BUF_RECV, done + sl[d].off);
                };
                for (uint32_t d = 0; d < D; d++) {
                    const uint32_t holder = rootGroup * D + d;
                    if (holder != R) {
                        EmitCopy(*vp, 0, at(holder, d), at(R, d), sl[d].size);
                    }
                }
                size_t gather = 1;
                for (uint32_t d = 0; d < D; d++) {
                    auto data = [&](uint32_t g) { return at(g * D + d, d); };
                    gather = std::max(gather, RhdBroadcastPhases(*vp, 1, S, rootGroup, data, sl[d].size));
                }
                for (uint32_t r = 0; r < p; r++) {
                    for (uint32_t k = 1; k < D && r != R; k++) {
                        const uint32_t d = (r % D + k) % D, from = r / D * D + d;
                        EmitCopy(*vp, gather, at(r, d), at(from, d), sl[d].size);
                    }
                }
            } else if (rq.coll == COLL_BROADCAST && rq.algo == ALGO_MESH) {
                // mesh broadcast (coll_broadcast_mesh_executor.cc:59-213): the root scatters slice i to
                // rank i (scatter_mesh.cc), then a mesh all-gather; slices from GetRankSliceSize
                // (coll_broadcast_executor.cc:275-306).  The root keeps its data where it is.
                uint64_t avg = bytes / p + ((cur % p) > 0 ? 1 : 0);
                uint64_t slice = RoundUpTo(avg, rq.align);
                std::vector<Slice> sl(p);
                uint64_t residue = bytes;
                for (uint32_t i = 0; i < p; i++) {
                    sl[i].size = std::min(slice, residue);
                    sl[i].off = sl[i].size == 0 ? 0 : uint64_t(i) * slice;
                    residue -= sl[i].size;
                }
                for (uint32_t r = 0; r < p; r++) {
                    if (r != R) {
                        EmitCopy(*vp, 0, MkRef(r, BUF_RECV, done + sl[r].off), MkRef(R, BUF_SEND, done + sl[r].off), sl[r].size);
                    }
                }
                for (uint32_t r = 0; r < p; r++) {
                    for (uint32_t k = 1; k < p && r != R; k++) {
                        uint32_t d = (r + k) % p;
                        Ref src = (d == R) ? MkRef(R, BUF_SEND, done + sl[d].off) : MkRef(d, BUF_RECV, done + sl[d].off);
                        EmitCopy(*vp, 1, MkRef(r, BUF_RECV, done + sl[d].off), src, sl[d].size);
                    }
                }
            } else if (rq.coll == COLL_BROADCAST && rq.algo == ALGO_RHD && p > 1) {
                auto data = [&](uint32_t r) { return r == R ? MkRef(R, BUF_SEND, done) : MkRef(r, BUF_RECV, done); };
                RhdBroadcastPhases(*vp, 0, p, R, data, bytes);
            } else if (rq.coll == COLL_BROADCAST && rq.algo == ALGO_HD_BLOCKS && p > 1) {
                auto data = [&](uint32_t r) { return r == R ? MkRef(R, BUF_SEND, done) : MkRef(r, BUF_RECV, done); };
                HdBlocksBroadcastPhases(*vp, p, R, data, bytes);
            } else if (rq.coll == COLL_REDUCE && rq.servers > 1 && p > 1) {
                TwoLevelReduceChunk(*vp, rq.algo == ALGO_RING ? ALGO_RING : ALGO_RHD, p, rq.servers, rq.level0Rings, R, done, bytes,
                    rq.align, rq.meshAtomic);
            } else if (rq.coll == COLL_REDUCE && rq.algo == ALGO_MESH && p > 1) {
                // mesh reduce (coll_reduce_mesh_executor.cc:75-194): mesh reduce-scatter over the ring
                // slice plan, then the root gathers slice r from rank r (gather_mesh.cc:60-170)
                std::vector<Slice> sl = RingSlicePlan(bytes, p, rq.align);
                size_t ph = MeshReduceScatterPhases(*vp, 0, p, done, sl, rq.align, rq.meshAtomic);
                for (uint32_t r = 0; r < p; r++) {
                    EmitCopy(*vp, ph, MkRef(R, BUF_RECV, done + sl[r].off), MkRef(r, BUF_SEND, done + sl[r].off), sl[r].size);
                }
            } else if (rq.coll == COLL_REDUCE && rq.algo == ALGO_RHD && p > 1) {
                RhdReducePhases(*vp, p, R, done, bytes, rq.align, MkRef(R, BUF_RECV, done));
            } else if (rq.coll == COLL_BROADCAST) {
                // ring broadcast (broadcast_ring.cc:24-160): the chunk is cut into p slices that travel
                // root -> root+1 -> ... -> root-1 as a pipeline; slice j reaches distance d in phase j+d-1
                uint64_t sizeAvg = ((cur + p - 1) / p) * u;
                uint64_t slice = RoundUpTo(sizeAvg, rq.align);
                for (uint32_t j = 0; j < p && p > 1; j++) {
                    uint64_t off = std::min<uint64_t>(uint64_t(j) * slice, bytes);
                    uint64_t n = std::min<uint64_t>(slice, bytes - off);
                    for (uint32_t d = 1; d < p; d++) {
                        uint32_t r = (R + d) % p, prev = (R + d - 1) % p;
                        Ref src = (d == 1) ? MkRef(R, BUF_SEND, done + off) : MkRef(prev, BUF_RECV, done + off);
                        EmitCopy(*vp, j + d - 1, MkRef(r, BUF_RECV, done + off), src, n);
                    }
                }
            } else {
                // ring reduce (reduce_ring.cc:29-154): the whole chunk walks root+1 -> ... -> root, each
                // rank combining its own data with what arrives; the root writes its output
                if (p == 1) {
                    EmitCopy(*vp, 0, MkRef(0, BUF_RECV, done), MkRef(0, BUF_SEND, done), bytes);
                }
                RingReducePhases(*vp, p, R, done, bytes, MkRef(R, BUF_RECV, done));
            }
            done += bytes;
            left -= cur;
        }
        for (uint32_t r = 0; r < p; r++) {
            if (rq.coll == COLL_BROADCAST) {
                vp->inBytes[r] = (r == R) ? total : 0;
                vp->outBytes[r] = (r == R) ? 0 : total;
            } else {
                vp->inBytes[r] = total;
                vp->outBytes[r] = (r == R) ? total : 0;
            }
        }
        return 0;
    }
    if (rq.algo == ALGO_PAIRWISE) {
        *err = "algorithm not available for this collective";
        return 1;
    }
    if (!rq.vCounts.empty()) {
        // variable block sizes: the same schedules over explicit slices, one pass (the slice a rank
        // ends up with is the same whatever the chunking, so no chunk loop is needed)
        if (rq.vCounts.size() != p || rq.vDispls.size() != p || rq.coll == COLL_ALLREDUCE) {
            *err = "variable-count tables must have p entries";
            return 1;
        }
        std::vector<Slice> sl(p);
        uint64_t extent = 0;
        for (uint32_t i = 0; i < p; i++) {
            sl[i] = Slice{rq.vDispls[i] * u, rq.vCounts[i] * u};
            if (sl[i].size) {
                extent = std::max(extent, sl[i].off + sl[i].size);
            }
        }
        if (rq.coll == COLL_REDUCESCATTER) {
            std::vector<Slice> out(p);
            for (uint32_t i = 0; i < p; i++) {
                out[i] = Slice{0, sl[i].size};
            }
            if (p == 1) {
                EmitCopy(*vp, 0, MkRef(0, BUF_RECV, 0), MkRef(0, BUF_SEND, sl[0].off), sl[0].size);
            } else if (rq.algo == ALGO_RING) {
                RingReduceScatterPhases(*vp, 0, p, 0, sl, BUF_RECV, 0, out);
            } else if (rq.algo == ALGO_RHD) {
                RhdReduceScatterChunk(*vp, p, sl, 0);
            } else {
                size_t ph = MeshReduceScatterPhases(*vp, 0, p, 0, sl, rq.align, rq.meshAtomic);
                for (uint32_t r = 0; r < p; r++) {
                    EmitCopy(*vp, ph, MkRef(r, BUF_RECV, 0), MkRef(r, BUF_SEND, sl[r].off), sl[r].size);
                }
            }
            for (uint32_t r = 0; r < p; r++) {
                vp->inBytes[r] = extent;
                vp->outBytes[r] = sl[r].size;
            }
        } else {
            for (uint32_t r = 0; r < p; r++) {
                EmitCopy(*vp, 0, MkRef(r, BUF_RECV, sl[r].off), MkRef(r, BUF_SEND, 0), sl[r].size);
            }
            if (p > 1) {
                if (rq.algo == ALGO_RING) {
                    RingAllGatherPhases(*vp, 1, p, 0, sl);
                } else if (rq.algo == ALGO_RHD) {
                    RhdAllGatherChunk(*vp, 1, p, sl);
                } else {
                    MeshAllGatherPhases(*vp, 1, p, 0, sl);
                }
            }
            for (uint32_t r = 0; r < p; r++) {
                vp->inBytes[r] = sl[r].size;
                vp->outBytes[r] = extent;
            }
            // whole blocks for the planner's short cut: rank r's block lands at its displacement in every receive buffer
            for (uint32_t q = 0; q < p; q++) {
                for (uint32_t r = 0; r < p; r++) {
                    if (sl[r].size) {
                        vp->blocks.push_back(VProgram::Block{sl[r].off, 0, sl[r].size, q, r});
                    }
                }
            }
        }
        return 0;
    }
    // the two-level reduce-scatter sizes its chunks without rounding to the slice alignment
    // (CollReduceScatterMeshExecutor::CalcLoopMaxCount, coll_reduce_scatter_mesh_executor.cc:114-119)
    // and so does the two-level all-gather with rings inside a group (CollAllGatherRingExecutor::CalcLoopMaxCount,
    // coll_all_gather_ring_executor.cc:75-79; with the mesh the rounding stays, coll_all_gather_mesh_executor.cc:64-69)
    const bool twoLevelScatter = (rq.coll == COLL_REDUCESCATTER && rq.servers > 1) ||
        (rq.coll == COLL_ALLGATHER && rq.servers > 1 && rq.level0Rings > 0);
    std::vector<uint64_t> chunks = ChunkCounts(rq.coll, rq.count, rq.unit, p, rq.cclBytes, twoLevelScatter ? 1 : rq.align);
    if (rq.count > 0 && chunks.empty()) {
        *err = "CCL buffer too small for one element per rank";
        return 1;
    }
    uint64_t total = rq.count * u;
    uint64_t done = 0;
    for (uint64_t cur : chunks) {
        uint64_t bytes = cur * u;
        if (rq.coll == COLL_ALLREDUCE && (rq.servers > 1 || rq.level0Rings > 0)) {
            TwoLevelAllReduceChunk(*vp, rq.algo == ALGO_RING ? ALGO_RING : ALGO_RHD, p, rq.servers, rq.level0Rings, done, bytes,
                rq.align, rq.meshAtomic);
        } else if (rq.coll == COLL_ALLREDUCE) {
            AllReduceChunk(*vp, rq.algo, p, done, bytes, rq.align, rq.meshAtomic, rq.nicMask);
        } else if (rq.coll == COLL_REDUCESCATTER) {
            // input slice i of this chunk sits at i * total + done in the caller's layout
            std::vector<Slice> in(p), out(p);
            for (uint32_t i = 0; i < p; i++) {
                in[i] = Slice{uint64_t(i) * total + done, bytes};
                out[i] = Slice{done, bytes};
            }
            if (p == 1) {
                EmitCopy(*vp, 0, MkRef(0, BUF_RECV, done), MkRef(0, BUF_SEND, done), bytes);
            } else if (rq.servers > 1) {
                std::vector<uint64_t> blockOff(p);
                for (uint32_t i = 0; i < p; i++) {
                    blockOff[i] = in[i].off;
                }
                if (rq.nicMask != 0 && (rq.nicMask & 0xffu) != 0xffu) {
                    PrunedTwoLevelReduceScatterChunk(*vp, p, rq.servers, rq.nicMask, blockOff, bytes, done, rq.align);
                } else {
                    TwoLevelReduceScatterChunk(*vp, rq.algo == ALGO_RING ? ALGO_RING : ALGO_RHD, p, rq.servers, rq.level0Rings,
                        blockOff, bytes, done, rq.align, rq.meshAtomic);
                }
            } else if (rq.algo == ALGO_RING) {
                RingReduceScatterPhases(*vp, 0, p, 0, in, BUF_RECV, 0, out);
            } else if (rq.algo == ALGO_RHD) {
                RhdReduceScatterChunk(*vp, p, in, done);
            } else {
                size_t ph = MeshReduceScatterPhases(*vp, 0, p, 0, in, rq.align, rq.meshAtomic);
                for (uint32_t r = 0; r < p; r++) {
                    EmitCopy(*vp, ph, MkRef(r, BUF_RECV, done), MkRef(r, BUF_SEND, in[r].off), bytes);
                }
            }
        } else {
            std::vector<Slice> sl(p);
            for (uint32_t i = 0; i < p; i++) {
                sl[i] = Slice{uint64_t(i) * total + done, bytes};
            }
            for (uint32_t r = 0; r < p; r++) {
                EmitCopy(*vp, 0, MkRef(r, BUF_RECV, sl[r].off), MkRef(r, BUF_SEND, done), bytes);
            }
            if (p > 1 && rq.servers > 1) {
                TwoLevelAllGatherChunk(*vp, rq.algo == ALGO_RING ? ALGO_RING : ALGO_RHD, p, rq.servers, rq.level0Rings, sl, rq.align);
            } else if (p > 1) {
                if (rq.algo == ALGO_RING) {
                    RingAllGatherPhases(*vp, 1, p, 0, sl);
                } else if (rq.algo == ALGO_RHD) {
                    RhdAllGatherChunk(*vp, 1, p, sl);
                } else {
                    MeshAllGatherPhases(*vp, 1, p, 0, sl);
                }
            }
        }
        done += bytes;
    }
    for (uint32_t r = 0; r < p; r++) {
        vp->inBytes[r] = (rq.coll == COLL_REDUCESCATTER) ? total * p : total;
        vp->outBytes[r] = (rq.coll == COLL_ALLGATHER) ? total * p : total;
    }
    return 0;
}

}  // namespace planner
}  // namespace hcclamd
