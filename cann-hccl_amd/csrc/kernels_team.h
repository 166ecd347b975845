// Team form of the fused kernels, for large launches whose items touch many streams (an all-reduce reads 8 buffers and
// writes 8, an all-gather reads 1 and writes 8).
//
// The plain fused kernels let every workgroup read a tile and write it straight away, so at any moment each XCD of the
// chip has reads and writes of all its workgroups in flight.  This part moves more bytes when an XCD does one thing at
// a time (measured on MI355X, 8 x 256 MiB read and 8 x 256 MiB written: 5.3 - 5.6 TB/s with reads and writes
// interleaved per workgroup, 5.9 - 6.0 TB/s when the 32 workgroups of an XCD read together and then write together;
// 1 read : 8 writes 4.9 against 5.9 TB/s).  So here the workgroups of one XCD form a team:
//   read phase   every workgroup evaluates up to kTeamTiles tiles (every 32nd tile of the team's region, so an XCD
//                works on one contiguous stretch of the tile space) and parks the results in LDS.  A round of whole
//                tiles of one item is read with all its loads issued together (a copy) or source by source with the
//                partial results in LDS (a chain), see Round() below
//   barrier      among the team's workgroups only; the other XCDs run on, in whatever phase they are
//   write phase  every workgroup writes its parked tiles to their destinations, destination by destination
// Workgroup b belongs to XCD b % 8 (workgroups are dealt to the XCDs round robin).  If they are not, or if the team is
// not resident all at once, only the speed changes: nothing passes between workgroups through the barrier, it only
// aligns them in time, every wait is bounded, and after one wait that ran out a team stops waiting for that launch.
//
// The counters live in device memory that starts out zero; the last workgroup of a launch to finish puts them back to
// zero, so the next launch (or a replay of a HIP graph) finds them as the first one did.
#pragma once
#include "kernels_impl.h"

namespace hcclamd {

constexpr uint32_t kTeamVecPerTile = kTileBytes / 16;
constexpr uint64_t kTeamWaitTicks = 20000;                       // 200 us of the 100 MHz clock

// All atomics here are relaxed and at agent scope: they are carried out in memory, beyond the XCDs' separate L2 caches,
// and order nothing else (no data is handed from workgroup to workgroup).
__device__ __forceinline__ uint32_t TeamLoad(const uint32_t *p)
{
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void TeamStore(uint32_t *p, uint32_t v)
{
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint32_t TeamAdd(uint32_t *p, uint32_t v)
{
    return __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The team's region for its next round.  Every workgroup of the team asks on its own; whoever comes first to the
// round's slot claims it (0 -> 1), draws the next region from the launch's ticket counter and leaves the answer
// (region + 2) in the slot.  The others wait for that answer: the claimer is running and needs nobody to get there,
// so the wait ends whether or not the rest of the grid is resident.  `seen` is what an earlier look at the slot showed.
__device__ __forceinline__ uint32_t TeamNextRegion(uint32_t *slot, uint32_t *ticket, uint32_t seen)
{
    uint32_t v = seen;
    for (;;) {
        if (v >= 2u) {
            return v - 2u;
        }
        if (v == 0u) {
            // (also reached when the slot was put back to zero under a waiting workgroup: two launches of one prepared
            // collective running at the same time share this block; each region is then still worked on at least once)
            uint32_t expected = 0u;
            if (__hip_atomic_compare_exchange_strong(slot, &expected, 1u, __ATOMIC_RELAXED, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) {
                v = TeamAdd(ticket, 1u) + kTeamXcds + 2u;      // regions 0 .. kTeamXcds - 1 are the first round's
                TeamStore(slot, v);
            } else {
                v = expected;
            }
            continue;
        }
        __builtin_amdgcn_s_sleep(2);
        v = TeamLoad(slot);
    }
}

// Arrival at the team's barrier, then (thread 0) the question for the next region while the others arrive, then the
// wait: bounded, and given up for the rest of the launch once it has run out (kTeamGaveUpBit in the arrival word).
// Every access here is a trip to memory and back, a few microseconds under load, and whatever the last workgroup to
// arrive does here delays its whole team: it learns from its own arrival that nobody is missing, and it has
// normally seen the next region already (`seen`: a look at the slot taken before its last tile).
__device__ __forceinline__ uint32_t TeamBarrier(uint32_t *c, uint32_t target, uint32_t *slot, uint32_t *ticket, uint32_t seen,
    uint32_t *nextShared)
{
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t v = TeamAdd(c + kTeamArrive, 1u) + 1u;
        *nextShared = TeamNextRegion(slot, ticket, seen);
        if ((v & ~kTeamGaveUpBit) < target && (v & kTeamGaveUpBit) == 0u) {
            const uint64_t t0 = wall_clock64();
            for (;;) {
                v = TeamLoad(c + kTeamArrive);
                if ((v & ~kTeamGaveUpBit) >= target || (v & kTeamGaveUpBit) != 0u) {
                    break;
                }
                if (wall_clock64() - t0 > kTeamWaitTicks) {
                    __hip_atomic_fetch_or(c + kTeamArrive, kTeamGaveUpBit, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    break;
                }
                __builtin_amdgcn_s_sleep(1);
            }
        }
    }
    __syncthreads();
    return *nextShared;
}

// The last workgroup of the launch to finish puts every counter and slot back to zero.  Counted in two levels (the last
// of a team reports for the team): atomics on one address are carried out one after the other, a hundred nanoseconds
// and more each, and a whole grid counting on one word is most of a small launch's time.
__device__ __forceinline__ void TeamLeave(uint32_t *teamCtr, uint32_t *ctr, uint32_t teamSize, uint32_t nregions)
{
    __shared__ uint32_t last;
    __syncthreads();
    if (threadIdx.x == 0) {
        last = 0u;
        if (TeamAdd(ctr + kTeamLeft, 1u) + 1u == teamSize) {
            last = TeamAdd(teamCtr + kTeamFinished, 1u) + 1u == kTeamXcds ? 1u : 0u;
        }
    }
    __syncthreads();
    if (last) {       // everybody else is past every barrier and every slot
        uint32_t *slots = teamCtr + kTeamHeaderWords + 2u * nregions;
        for (uint32_t i = threadIdx.x; i < kTeamXcds * (nregions + 1u); i += kBlockThreads) {
            TeamStore(slots + i, 0u);
        }
        if (threadIdx.x < kTeamXcds) {
            TeamStore(teamCtr + threadIdx.x * kTeamCtrStride + kTeamArrive, 0u);
            TeamStore(teamCtr + threadIdx.x * kTeamCtrStride + kTeamLeft, 0u);
        }
        if (threadIdx.x == 0) {
            TeamStore(teamCtr + kTeamTicket, 0u);
            TeamStore(teamCtr + kTeamFinished, 0u);
        }
    }
}

// One parked tile to one destination.
template <uint32_t MODE, bool ORDINARY>
__device__ __forceinline__ void TeamDrain(const LdsV4 *park, void *o, uint64_t off, uint32_t nvec)
{
    const uint32_t tid = threadIdx.x;
    if (nvec == kTeamVecPerTile) {
        V4 w[kVecPerLane];
#pragma unroll
        for (uint32_t u = 0; u < kVecPerLane; u++) {
            w[u] = park[u * kBlockThreads + tid];
        }
#pragma unroll
        for (uint32_t u = 0; u < kVecPerLane; u++) {
            StoreAny16<MODE, ORDINARY>(o, off + (uint64_t(u) * kBlockThreads + tid) * 16, w[u]);
        }
    } else {
        for (uint32_t i = tid; i < nvec; i += kBlockThreads) {
            StoreAny16<MODE, ORDINARY>(o, off + uint64_t(i) * 16, park[i]);
        }
    }
}

// Eval: SetItem(d, srcPool) is called when the tiles move on to another item, Vec(d, srcPool, extra, off, nvec, park)
// leaves the vectors of one tile in LDS, the static Elem(d, srcPool, extra, dstPool, off, n) handles an element-wise
// piece (a few bytes of head or tail) there and then.
//
// The tile space is cut into regions (first tile, tiles per workgroup), a table the host wrote behind the counters:
// workgroup i of a team of n takes the tiles first + i, first + i + n, ... (per of them) of the team's region.  Team x starts
// with region x; the later ones are drawn from a counter as the teams get there, and the last regions are smaller,
// so that the XCDs, which do not all move data at the same rate, finish together.
template <typename Eval>
__device__ __forceinline__ void TeamBody(const FusedDesc *__restrict__ items, uint32_t nitems, uint32_t ntiles,
    const void *const *__restrict__ srcPool, void *const *__restrict__ dstPool, uint32_t tilesPerItem,
    uint32_t *__restrict__ teamCtr, const void *extra)
{
    extern __shared__ V4 teamLds[];
    __shared__ uint32_t heldItem[kTeamTiles];
    __shared__ uint32_t heldTile[kTeamTiles];
    __shared__ uint32_t heldVec[kTeamTiles];      // vectors parked; 0 = nothing (no tile, or an element-wise piece)
    __shared__ uint32_t nextShared;
    LdsV4 *park = (LdsV4 *)teamLds;

    const uint32_t xcd = blockIdx.x % kTeamXcds, inTeam = blockIdx.x / kTeamXcds, teamSize = gridDim.x / kTeamXcds;
    const uint32_t nregions = teamCtr[kTeamRegionCount];
    const TeamRegion *regions = reinterpret_cast<const TeamRegion *>(teamCtr + kTeamHeaderWords);
    uint32_t *slots = teamCtr + kTeamHeaderWords + 2u * nregions + xcd * (nregions + 1u);
    uint32_t *ctr = teamCtr + xcd * kTeamCtrStride;
    uint32_t target = 0;
    uint32_t region = xcd;
    for (uint32_t round = 0; region < nregions; round++) {
        // A workgroup's tiles are every teamSize-th tile of the region, not a run of consecutive ones: the team then
        // reads, and later writes, one stretch of teamSize tiles of every stream at a time instead of teamSize
        // stretches apart (8 ranks x 256 MiB: 1.5 % faster).
        const TeamRegion reg = regions[region];
        const uint32_t first = reg.first + inTeam;
        const uint32_t fit = first < ntiles ? (ntiles - 1 - first) / teamSize + 1 : 0;
        const uint32_t n = fit < reg.per ? fit : reg.per;
        uint32_t seen = 0;
        uint32_t maxDst = 0;
        uint32_t idx = 0;
        FusedDesc d;
        uint32_t dEnd = 0;
        Eval eval;
        bool bySource = false;
        if constexpr (Eval::kBySource) {
            // All the round's tiles whole, vector-aligned and of one item: the team reads source by source (see
            // TeamChainEval::Round).
            if (n == kTeamTiles || n == kTeamTiles / 2) {
                idx = ItemOfTile(items, nitems, first, tilesPerItem);
                d = items[idx];
                dEnd = d.tile0 + uint32_t((d.bytes + kTileBytes - 1) / kTileBytes);
                const uint32_t lastTile = first + (n - 1) * teamSize;
                bySource = d.mode == ACC_VEC16 && d.nsrc >= Eval::kRoundMinSrc && lastTile < dEnd &&
                    uint64_t(lastTile - d.tile0 + 1) * kTileBytes <= d.bytes;
            }
            if (bySource) {
                const uint64_t off = uint64_t(first - d.tile0) * kTileBytes;
                const uint64_t stride = uint64_t(teamSize) * kTileBytes;
                if (n == kTeamTiles) {
                    Eval::template Round<kTeamTiles>(d, srcPool + d.srcBase, off, stride, park, slots + round, &seen);
                } else {
                    Eval::template Round<kTeamTiles / 2>(d, srcPool + d.srcBase, off, stride, park, slots + round, &seen);
                }
                maxDst = d.ndst;
                if (threadIdx.x < n) {
                    heldItem[threadIdx.x] = idx;
                    heldTile[threadIdx.x] = first + threadIdx.x * teamSize;
                    heldVec[threadIdx.x] = kTeamVecPerTile;
                }
            }
        }
        for (uint32_t q = 0; q < n && !bySource; q++) {
            const uint32_t tile = first + q * teamSize;
            if (q + 1 == n && threadIdx.x == 0) {
                // a look at the slot of the next round, in flight together with the last tile's loads: a workgroup
                // that is behind the others finds the answer there
                seen = TeamLoad(slots + round);
            }
            if (q == 0 || tile >= dEnd) {
                idx = ItemOfTile(items, nitems, tile, tilesPerItem);
                d = items[idx];
                dEnd = d.tile0 + uint32_t((d.bytes + kTileBytes - 1) / kTileBytes);
                eval.SetItem(d, srcPool);
            }
            const uint64_t off = uint64_t(tile - d.tile0) * kTileBytes;
            const uint64_t rest = d.bytes - off;
            const uint32_t bytes = rest < kTileBytes ? uint32_t(rest) : kTileBytes;
            uint32_t nvec = 0;
            if (d.mode == ACC_ELEM) {
                Eval::Elem(d, srcPool, extra, dstPool, off, bytes);
            } else {
                nvec = bytes >> 4;
                eval.Vec(d, srcPool, extra, off, nvec, park + q * kTeamVecPerTile);
                maxDst = d.ndst > maxDst ? d.ndst : maxDst;
            }
            if (threadIdx.x == 0) {
                heldItem[q] = idx;
                heldTile[q] = tile;
                heldVec[q] = nvec;
            }
        }
        target += teamSize;
        region = TeamBarrier(ctr, target, slots + round, teamCtr + kTeamTicket, seen, &nextShared);
        // Every lane reads back the vectors it parked itself.  A workgroup's tiles mostly belong to one item, so its
        // descriptor and the destination pointer are kept from tile to tile.
        for (uint32_t k = 0; k < maxDst; k++) {
            uint32_t cur = ~0u;
            FusedDesc w;
            void *o = nullptr;
            for (uint32_t q = 0; q < n; q++) {
                const uint32_t nvec = heldVec[q];
                if (nvec == 0) {
                    continue;
                }
                if (heldItem[q] != cur) {
                    cur = heldItem[q];
                    w = items[cur];
                    o = k < w.ndst ? dstPool[w.dstBase + k] : nullptr;
                }
                if (o == nullptr) {
                    continue;
                }
                const uint64_t off = uint64_t(heldTile[q] - w.tile0) * kTileBytes;
                const LdsV4 *from = park + q * kTeamVecPerTile;
                if (w.mode == ACC_VEC16) {
                    if (w.flags & kFusedOrdinaryStores) {
                        TeamDrain<ACC_VEC16, true>(from, o, off, nvec);
                    } else {
                        TeamDrain<ACC_VEC16, false>(from, o, off, nvec);
                    }
                } else {
                    TeamDrain<ACC_VEC16_ANY, false>(from, o, off, nvec);
                }
            }
        }
        // the next round's results must not land in LDS before this round's have been read
        __syncthreads();
    }
    TeamLeave(teamCtr, ctr, teamSize, nregions);
}

// ---- what a tile's value is, per kernel family --------------------------------------------------------------------
// A bf16 combine is a dozen instructions per element pair (widen, combine, round); between a set's loads and the next
// request for that set they cost more than the order of the reads gains (8 ranks x 256 MiB, source by source against
// tile by tile: fp32 sum 0.708 / 0.719 ms, int32 0.705 / 0.720, int64 product 0.725 / 0.749, fp16 sum 0.716 / 0.720,
// int8 the same, bf16 sum 0.737 / 0.734, bf16 max 0.762 / 0.753).
template <typename T> struct ReadsBySource { static constexpr bool value = true; };
template <> struct ReadsBySource<Bf16Bits> { static constexpr bool value = false; };

template <typename T, int OP> struct TeamChainEval {
    static constexpr bool kBySource = ReadsBySource<T>::value;
    static constexpr uint32_t kRoundMinSrc = 2;
    // A whole round at once: N whole tiles of one item, `stride` bytes apart from `off` on.  The team reads source by
    // source -- at any moment its loads go to one stretch of N x 32 tiles of one buffer instead of 32 tiles of each of
    // the item's buffers -- and the partial results rest in LDS, folded in the chain's order, so the bits are those of
    // the tile-by-tile evaluation.  Two register sets of N x 4 vectors: while one source is folded, the next one's
    // loads are in flight, and the one after that is requested as soon as the fold has freed its set (8 ranks x
    // 256 MiB, stand-alone: 691 us this way, 770 us with one set, 705 us tile by tile).
    // Straight-line code for a source count fixed at compile time, in which every wait is for exactly the loads it
    // needs, measured the same and takes three times as long to build.
    // `peek` is looked at (thread 0, into *seen) once the last loads are on their way.
    template <uint32_t N>
    static __device__ __forceinline__ void LoadSet(V4 (&v)[N][kVecPerLane], const void *base, uint64_t off, uint64_t stride)
    {
        const char *s = static_cast<const char *>(base) + off;
#pragma unroll
        for (uint32_t q = 0; q < N; q++) {
#pragma unroll
            for (uint32_t u = 0; u < kVecPerLane; u++) {
                v[q][u] = Load16<ACC_VEC16>(s + q * stride + uint64_t(u) * kBlockThreads * 16, threadIdx.x * 16u);
            }
        }
    }
    // Source j into the partial results: source 0 starts them.  A tile's partial results are fetched from LDS together,
    // so that their latencies overlap.
    template <uint32_t N>
    static __device__ __forceinline__ void FoldSet(const V4 (&v)[N][kVecPerLane], const FusedDesc &d, uint32_t j, LdsV4 *park)
    {
        const uint32_t tid = threadIdx.x;
        if (j == 0) {
#pragma unroll
            for (uint32_t q = 0; q < N; q++) {
#pragma unroll
                for (uint32_t u = 0; u < kVecPerLane; u++) {
                    park[q * kTeamVecPerTile + u * kBlockThreads + tid] = v[q][u];
                }
            }
            return;
        }
        const bool accLeft = OrderMatters<T, OP>::value && ((d.accLeftMask >> j) & 1ull);
#pragma unroll
        for (uint32_t q = 0; q < N; q++) {
            V4 a[kVecPerLane];
#pragma unroll
            for (uint32_t u = 0; u < kVecPerLane; u++) {
                a[u] = park[q * kTeamVecPerTile + u * kBlockThreads + tid];
            }
            if (accLeft) {      // the same for the whole wave
#pragma unroll
                for (uint32_t u = 0; u < kVecPerLane; u++) {
                    a[u] = Combine16<T, OP>(a[u], v[q][u]);
                }
            } else {
#pragma unroll
                for (uint32_t u = 0; u < kVecPerLane; u++) {
                    a[u] = Combine16<T, OP>(v[q][u], a[u]);
                }
            }
#pragma unroll
            for (uint32_t u = 0; u < kVecPerLane; u++) {
                park[q * kTeamVecPerTile + u * kBlockThreads + tid] = a[u];
            }
        }
    }
    template <uint32_t N>
    static __device__ __forceinline__ void Round(const FusedDesc &d, const void *const *__restrict__ src, uint64_t off,
        uint64_t stride, LdsV4 *park, const uint32_t *peek, uint32_t *seen)
    {
        const uint32_t nsrc = d.nsrc;
        V4 va[N][kVecPerLane], vb[N][kVecPerLane];
        LoadSet<N>(va, src[0], off, stride);
        LoadSet<N>(vb, src[1], off, stride);
        uint32_t j = 0;
#pragma nounroll
        for (; j + 4 <= nsrc; j += 2) {
            FoldSet<N>(va, d, j, park);
            LoadSet<N>(va, src[j + 2], off, stride);
            FoldSet<N>(vb, d, j + 1, park);
            LoadSet<N>(vb, src[j + 3], off, stride);
        }
        // two or three sources left, the first two of them loaded or on their way
        const bool three = nsrc - j == 3;
        FoldSet<N>(va, d, j, park);
        if (three) {
            LoadSet<N>(va, src[j + 2], off, stride);
        }
        if (threadIdx.x == 0) {
            *seen = TeamLoad(peek);
        }
        FoldSet<N>(vb, d, j + 1, park);
        if (three) {
            FoldSet<N>(va, d, j + 2, park);
        }
    }
    // Up to kChainSrcBatch source pointers are kept in registers from tile to tile: fetched per tile they are a chain
    // of dependent loads in front of the tile's data, with nothing else on the CU to hide it.
    const void *sp[kChainSrcBatch];
    bool few;
    __device__ __forceinline__ void SetItem(const FusedDesc &d, const void *const *__restrict__ srcPool)
    {
        few = d.nsrc <= kChainSrcBatch;
#pragma unroll
        for (uint32_t j = 0; j < kChainSrcBatch; j++) {
            sp[j] = j < d.nsrc ? srcPool[d.srcBase + j] : nullptr;
        }
    }
    template <uint32_t MODE, bool ONE>
    __device__ __forceinline__ void Passes(const FusedDesc &d, const void *const *__restrict__ src, uint64_t off, uint32_t nvec,
        LdsV4 *park) const
    {
        constexpr uint32_t kPass = kChainVec * kBlockThreads;
        uint32_t base = 0;
        for (; base + kPass <= nvec; base += kPass) {
            ChainVecPass<T, OP, MODE, true, false, true, ONE>(d, src, nullptr, off, base, nvec, park);
        }
        if (base < nvec) {
            ChainVecPass<T, OP, MODE, false, false, true, ONE>(d, src, nullptr, off, base, nvec, park);
        }
    }
    __device__ __forceinline__ void Vec(const FusedDesc &d, const void *const *__restrict__ srcPool, const void *,
        uint64_t off, uint32_t nvec, LdsV4 *park) const
    {
        if (few) {
            if (d.mode == ACC_VEC16) {
                Passes<ACC_VEC16, true>(d, sp, off, nvec, park);
            } else {
                Passes<ACC_VEC16_ANY, true>(d, sp, off, nvec, park);
            }
        } else {
            if (d.mode == ACC_VEC16) {
                Passes<ACC_VEC16, false>(d, srcPool + d.srcBase, off, nvec, park);
            } else {
                Passes<ACC_VEC16_ANY, false>(d, srcPool + d.srcBase, off, nvec, park);
            }
        }
    }
    static __device__ __forceinline__ void Elem(const FusedDesc &d, const void *const *__restrict__ srcPool, const void *,
        void *const *__restrict__ dstPool, uint64_t off, uint32_t n)
    {
        ChainElem<T, OP>(d, srcPool + d.srcBase, dstPool + d.dstBase, off, n);
    }
};

struct TeamCopyEval {
    static constexpr bool kBySource = true;
    static constexpr uint32_t kRoundMinSrc = 1;
    // A whole round at once (see TeamChainEval::Round): the loads of all N tiles are issued before the first of them is
    // parked, instead of tile after tile with an LDS write between them.
    template <uint32_t N>
    static __device__ __forceinline__ void Round(const FusedDesc &, const void *const *__restrict__ src, uint64_t off,
        uint64_t stride, LdsV4 *park, const uint32_t *peek, uint32_t *seen)
    {
        const uint32_t tid = threadIdx.x;
        const char *s = static_cast<const char *>(src[0]) + off;
        V4 v[N][kVecPerLane];
#pragma unroll
        for (uint32_t q = 0; q < N; q++) {
#pragma unroll
            for (uint32_t u = 0; u < kVecPerLane; u++) {
                v[q][u] = Load16<ACC_VEC16>(s + q * stride + uint64_t(u) * kBlockThreads * 16, tid * 16u);
            }
        }
        if (tid == 0) {
            *seen = TeamLoad(peek);
        }
#pragma unroll
        for (uint32_t q = 0; q < N; q++) {
#pragma unroll
            for (uint32_t u = 0; u < kVecPerLane; u++) {
                park[q * kTeamVecPerTile + u * kBlockThreads + tid] = v[q][u];
            }
        }
    }
    const void *s;
    __device__ __forceinline__ void SetItem(const FusedDesc &d, const void *const *__restrict__ srcPool) { s = srcPool[d.srcBase]; }
    __device__ __forceinline__ void Vec(const FusedDesc &d, const void *const *__restrict__, const void *, uint64_t off,
        uint32_t nvec, LdsV4 *park) const
    {
        constexpr uint32_t kPass = kChainVec * kBlockThreads;
        uint32_t base = 0;
        if (d.mode == ACC_VEC16) {
            for (; base + kPass <= nvec; base += kPass) {
                CopyVecPass<ACC_VEC16, true, false, true>(s, nullptr, 0, off, base, nvec, park);
            }
            if (base < nvec) {
                CopyVecPass<ACC_VEC16, false, false, true>(s, nullptr, 0, off, base, nvec, park);
            }
        } else {
            for (; base + kPass <= nvec; base += kPass) {
                CopyVecPass<ACC_VEC16_ANY, true, false, true>(s, nullptr, 0, off, base, nvec, park);
            }
            if (base < nvec) {
                CopyVecPass<ACC_VEC16_ANY, false, false, true>(s, nullptr, 0, off, base, nvec, park);
            }
        }
    }
    static __device__ __forceinline__ void Elem(const FusedDesc &d, const void *const *__restrict__ srcPool, const void *,
        void *const *__restrict__ dstPool, uint64_t off, uint32_t n)
    {
        const void *s = srcPool[d.srcBase];
        void *const *dst = dstPool + d.dstBase;
        for (uint32_t i = threadIdx.x; i < n; i += kBlockThreads) {
            const uint8_t b = LoadElem<uint8_t>(s, off + i);
            for (uint32_t k = 0; k < d.ndst; k++) {
                StoreElem<uint8_t>(dst[k], off + i, b);
            }
        }
    }
};

template <typename T, int OP> struct TeamTreeEval {
    static constexpr bool kBySource = false;
    __device__ __forceinline__ void SetItem(const FusedDesc &, const void *const *__restrict__) {}
    __device__ __forceinline__ void Vec(const FusedDesc &d, const void *const *__restrict__ srcPool, const void *,
        uint64_t off, uint32_t nvec, LdsV4 *park) const
    {
        TreeTile<T, OP, true>(d, srcPool + d.srcBase, nullptr, off, nvec, park);
    }
    static __device__ __forceinline__ void Elem(const FusedDesc &d, const void *const *__restrict__ srcPool, const void *,
        void *const *__restrict__ dstPool, uint64_t off, uint32_t n)
    {
        TreeElem<T, OP>(d, srcPool + d.srcBase, dstPool + d.dstBase, off, n);
    }
};

// extra = the launch's op words (they follow the item table)
template <typename T, int OP> struct TeamStackEval {
    static constexpr bool kBySource = false;
    __device__ __forceinline__ void SetItem(const FusedDesc &, const void *const *__restrict__) {}
    __device__ __forceinline__ void Vec(const FusedDesc &d, const void *const *__restrict__ srcPool, const void *extra,
        uint64_t off, uint32_t nvec, LdsV4 *park) const
    {
        const uint32_t *ops = static_cast<const uint32_t *>(extra) + d.srcBase;
        StackTile<T, OP, true>(d, srcPool + d.srcBase, ops, nullptr, off, nvec, park);
    }
    static __device__ __forceinline__ void Elem(const FusedDesc &d, const void *const *__restrict__ srcPool, const void *extra,
        void *const *__restrict__ dstPool, uint64_t off, uint32_t n)
    {
        const uint32_t *ops = static_cast<const uint32_t *>(extra) + d.srcBase;
        StackElem<T, OP>(d, srcPool + d.srcBase, ops, dstPool + d.dstBase, off, n);
    }
};

// Same tables and arguments as the plain fused kernels, plus the team block (counters, region table, slots; layout in
// kernels.h).  Launched with one workgroup per CU
// (a multiple of kTeamXcds workgroups) and kTeamDynamicLds bytes of dynamic LDS.
template <typename T, int OP>
__global__ void __launch_bounds__(kBlockThreads) TeamChainKernel(const FusedDesc *__restrict__ items, uint32_t nitems,
    uint32_t ntiles, const void *const *__restrict__ srcPool, void *const *__restrict__ dstPool, uint32_t tilesPerItem,
    uint32_t *__restrict__ teamCtr)
{
    TeamBody<TeamChainEval<T, OP>>(items, nitems, ntiles, srcPool, dstPool, tilesPerItem, teamCtr, nullptr);
}

template <int Variant>
__global__ void __launch_bounds__(kBlockThreads) TeamCopyKernel(const FusedDesc *__restrict__ items, uint32_t nitems,
    uint32_t ntiles, const void *const *__restrict__ srcPool, void *const *__restrict__ dstPool, uint32_t tilesPerItem,
    uint32_t *__restrict__ teamCtr)
{
    TeamBody<TeamCopyEval>(items, nitems, ntiles, srcPool, dstPool, tilesPerItem, teamCtr, nullptr);
}

template <typename T, int OP>
__global__ void __launch_bounds__(kBlockThreads) TeamTreeKernel(const FusedDesc *__restrict__ items, uint32_t nitems,
    uint32_t ntiles, const void *const *__restrict__ srcPool, void *const *__restrict__ dstPool, uint32_t tilesPerItem,
    uint32_t *__restrict__ teamCtr)
{
    TeamBody<TeamTreeEval<T, OP>>(items, nitems, ntiles, srcPool, dstPool, tilesPerItem, teamCtr, nullptr);
}

template <typename T, int OP>
__global__ void __launch_bounds__(kBlockThreads) TeamStackKernel(const FusedDesc *__restrict__ items, uint32_t nitems,
    uint32_t ntiles, const void *const *__restrict__ srcPool, void *const *__restrict__ dstPool, uint32_t tilesPerItem,
    uint32_t *__restrict__ teamCtr)
{
    TeamBody<TeamStackEval<T, OP>>(items, nitems, ntiles, srcPool, dstPool, tilesPerItem, teamCtr, items + nitems);
}

}  // namespace hcclamd
