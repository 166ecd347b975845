// Planner implementation.  See plan.h for the reference interfaces this covers.
//
// Pipeline: (1) emit the schedule on "virtual" buffers the way the reference runs it on its CCL
// staging buffers (partial results accumulate in the input buffer); (2) lower to the caller's
// buffers without touching a send buffer that is not also the receive buffer: partials are homed in
// the receive buffer when it is large enough, else in scratch; (3) run the program symbolically to
// check it (no read of unwritten memory, lowered == virtual) and to derive, per output range, the
// reduction expression over the original inputs; (4) turn those expressions into fused items when
// they are copies, chains or perfect trees.
#include "plan.h"

#include <algorithm>
#include <cstdlib>
#include <map>
#include <sstream>
#include <tuple>
#include <utility>

namespace hcclamd {

namespace {

uint64_t RoundUpTo(uint64_t v, uint64_t d) { return d == 0 ? v : (v + d - 1) / d * d; }
uint32_t Mod(int64_t v, uint32_t p) { int64_t m = v % static_cast<int64_t>(p); return static_cast<uint32_t>(m < 0 ? m + p : m); }

Ref MkRef(uint32_t rank, uint8_t buf, uint64_t off)
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
            for (uint32_t r = 0; r < p; r++) {
                EmitCopy(*vp, size_t(S - 1), MkRef(r, BUF_RECV, 0), MkRef(r / D * D + rootLocal, BUF_SEND, uint64_t(r) * total), total);
                vp->outBytes[r] = total;
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
            if (rq.coll == COLL_BROADCAST && rq.servers > 1 && p > 1) {
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

// ---- expression -> fused item -------------------------------------------------------------------------
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
