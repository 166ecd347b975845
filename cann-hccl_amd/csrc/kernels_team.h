// Team form of the fused kernels, for large launches whose items touch many streams (an all-reduce reads 8 buffers and
// writes 8, an all-gather reads 1 and writes 8).
//
// The plain fused kernels let every workgroup read a tile and write it straight away, so at any moment each XCD of the
// chip has reads and writes of all its workgroups in flight.  This part moves more bytes when an XCD does one thing at
// a time (measured on MI355X, 8 x 256 MiB read and 8 x 256 MiB written: 5.3 - 5.6 TB/s with reads and writes
// interleaved per workgroup, 5.9 - 6.0 TB/s when the 32 workgroups of an XCD read together and then write together;
// 1 read : 8 writes 4.9 against 5.9 TB/s).  So here the workgroups of one XCD form a team:
//   read phase   every workgroup evaluates up to kTeamTiles tiles (a run of consecutive tiles; the team's runs follow
//                each other, so an XCD works on one contiguous stretch of the tile space) and parks the results in LDS
//   barrier      among the team's workgroups only; the other XCDs run on, in whatever phase they are
//   write phase  every workgroup writes its parked tiles to their destinations, destination by destination
// Workgroup b belongs to XCD b % 8 (workgroups are dealt to the XCDs round robin).  If they are not, or if the team is
// not resident all at once, only the speed changes: nothing passes between workgroups through the barrier, it only
// aligns them in time, every wait is bounded, and after one wait that ran out a team stops waiting for that launch.
//
// The barrier counters live in device memory that starts out zero; the last workgroup of a team to finish puts them
// back to zero, so a launch (or a replay of a HIP graph) finds them as the first one did.
#pragma once
#include "kernels_impl.h"

namespace hcclamd {

constexpr uint32_t kTeamVecPerTile = kTileBytes / 16;
constexpr uint64_t kTeamWaitTicks = 20000;                       // 200 us of the 100 MHz clock

__device__ __forceinline__ uint32_t TeamLoad(const uint32_t *p)
{
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// c[0] arrivals, c[1] workgroups that have finished, c[2] set once a wait ran out.  Atomics at agent scope are carried
// out in memory, beyond the XCDs' separate L2 caches; relaxed, because no data is handed over.
__device__ __forceinline__ void TeamBarrier(uint32_t *c, uint32_t target)
{
    __syncthreads();
    if (threadIdx.x == 0) {
        __hip_atomic_fetch_add(c, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (TeamLoad(c + 2) == 0u) {
            const uint64_t t0 = wall_clock64();
            while (TeamLoad(c) < target) {
                if (wall_clock64() - t0 > kTeamWaitTicks) {
                    __hip_atomic_store(c + 2, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    break;
                }
                __builtin_amdgcn_s_sleep(2);
            }
        }
    }
    __syncthreads();
}

__device__ __forceinline__ void TeamLeave(uint32_t *c, uint32_t teamSize)
{
    __syncthreads();
    if (threadIdx.x == 0) {
        const uint32_t before = __hip_atomic_fetch_add(c + 1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (before + 1 == teamSize) {      // everybody else is past every barrier
            __hip_atomic_store(c, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(c + 2, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(c + 1, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
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

// Eval::Vec(d, srcPool, extra, off, nvec, park) leaves the vectors of one tile in LDS; Eval::Elem(d, srcPool, extra,
// dstPool, off, n) handles an element-wise piece (a few bytes of head or tail) there and then.
template <typename Eval>
__device__ __forceinline__ void TeamBody(const FusedDesc *__restrict__ items, uint32_t nitems, uint32_t ntiles,
    const void *const *__restrict__ srcPool, void *const *__restrict__ dstPool, uint32_t tilesPerItem,
    uint32_t *__restrict__ teamCtr, uint32_t roundTiles, const void *extra)
{
    extern __shared__ V4 teamLds[];
    __shared__ uint32_t heldItem[kTeamTiles];
    __shared__ uint32_t heldTile[kTeamTiles];
    __shared__ uint32_t heldVec[kTeamTiles];      // vectors parked; 0 = nothing (no tile, or an element-wise piece)
    LdsV4 *park = (LdsV4 *)teamLds;

    const uint32_t grid = gridDim.x;
    const uint32_t xcd = blockIdx.x % kTeamXcds, inTeam = blockIdx.x / kTeamXcds, teamSize = grid / kTeamXcds;
    uint32_t *ctr = teamCtr + xcd * kTeamCtrStride;
    uint32_t target = 0;
    uint32_t done = 0;                            // tiles of earlier rounds
    while (done < ntiles) {
        // tiles per workgroup this round: roundTiles (at most kTeamTiles), fewer in the last round so that it spreads
        // over all workgroups
        const uint32_t left = ntiles - done;
        const uint32_t per = left >= grid * roundTiles ? roundTiles : (left + grid - 1) / grid;
        const uint32_t first = done + (xcd * teamSize + inTeam) * per;
        const uint32_t n = first < ntiles ? (ntiles - first < per ? ntiles - first : per) : 0;
        uint32_t maxDst = 0;
        uint32_t idx = 0;
        FusedDesc d;
        uint32_t dEnd = 0;
        for (uint32_t q = 0; q < n; q++) {
            const uint32_t tile = first + q;
            if (q == 0 || tile >= dEnd) {
                idx = ItemOfTile(items, nitems, tile, tilesPerItem);
                d = items[idx];
                dEnd = d.tile0 + uint32_t((d.bytes + kTileBytes - 1) / kTileBytes);
            }
            const uint64_t off = uint64_t(tile - d.tile0) * kTileBytes;
            const uint64_t rest = d.bytes - off;
            const uint32_t bytes = rest < kTileBytes ? uint32_t(rest) : kTileBytes;
            uint32_t nvec = 0;
            if (d.mode == ACC_ELEM) {
                Eval::Elem(d, srcPool, extra, dstPool, off, bytes);
            } else {
                nvec = bytes >> 4;
                Eval::Vec(d, srcPool, extra, off, nvec, park + q * kTeamVecPerTile);
                maxDst = d.ndst > maxDst ? d.ndst : maxDst;
            }
            if (threadIdx.x == 0) {
                heldItem[q] = idx;
                heldTile[q] = tile;
                heldVec[q] = nvec;
            }
        }
        target += teamSize;
        TeamBarrier(ctr, target);
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
        done += left >= grid * roundTiles ? grid * roundTiles : left;
    }
    TeamLeave(ctr, teamSize);
}

// ---- what a tile's value is, per kernel family --------------------------------------------------------------------
template <typename T, int OP> struct TeamChainEval {
    static __device__ __forceinline__ void Vec(const FusedDesc &d, const void *const *__restrict__ srcPool, const void *,
        uint64_t off, uint32_t nvec, LdsV4 *park)
    {
        const void *const *src = srcPool + d.srcBase;
        constexpr uint32_t kPass = kChainVec * kBlockThreads;
        uint32_t base = 0;
        if (d.mode == ACC_VEC16) {
            for (; base + kPass <= nvec; base += kPass) {
                ChainVecPass<T, OP, ACC_VEC16, true, false, true>(d, src, nullptr, off, base, nvec, park);
            }
            if (base < nvec) {
                ChainVecPass<T, OP, ACC_VEC16, false, false, true>(d, src, nullptr, off, base, nvec, park);
            }
        } else {
            for (; base + kPass <= nvec; base += kPass) {
                ChainVecPass<T, OP, ACC_VEC16_ANY, true, false, true>(d, src, nullptr, off, base, nvec, park);
            }
            if (base < nvec) {
                ChainVecPass<T, OP, ACC_VEC16_ANY, false, false, true>(d, src, nullptr, off, base, nvec, park);
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
    static __device__ __forceinline__ void Vec(const FusedDesc &d, const void *const *__restrict__ srcPool, const void *,
        uint64_t off, uint32_t nvec, LdsV4 *park)
    {
        const void *s = srcPool[d.srcBase];
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
    static __device__ __forceinline__ void Vec(const FusedDesc &d, const void *const *__restrict__ srcPool, const void *,
        uint64_t off, uint32_t nvec, LdsV4 *park)
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
    static __device__ __forceinline__ void Vec(const FusedDesc &d, const void *const *__restrict__ srcPool, const void *extra,
        uint64_t off, uint32_t nvec, LdsV4 *park)
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

// Same tables and arguments as the plain fused kernels, plus the team counters and the number of tiles a workgroup
// takes per round (1 .. kTeamTiles).  Launched with one workgroup per CU
// (a multiple of kTeamXcds workgroups) and kTeamDynamicLds bytes of dynamic LDS.
template <typename T, int OP>
__global__ void __launch_bounds__(kBlockThreads) TeamChainKernel(const FusedDesc *__restrict__ items, uint32_t nitems,
    uint32_t ntiles, const void *const *__restrict__ srcPool, void *const *__restrict__ dstPool, uint32_t tilesPerItem,
    uint32_t *__restrict__ teamCtr, uint32_t roundTiles)
{
    TeamBody<TeamChainEval<T, OP>>(items, nitems, ntiles, srcPool, dstPool, tilesPerItem, teamCtr, roundTiles, nullptr);
}

template <int Variant>
__global__ void __launch_bounds__(kBlockThreads) TeamCopyKernel(const FusedDesc *__restrict__ items, uint32_t nitems,
    uint32_t ntiles, const void *const *__restrict__ srcPool, void *const *__restrict__ dstPool, uint32_t tilesPerItem,
    uint32_t *__restrict__ teamCtr, uint32_t roundTiles)
{
    TeamBody<TeamCopyEval>(items, nitems, ntiles, srcPool, dstPool, tilesPerItem, teamCtr, roundTiles, nullptr);
}

template <typename T, int OP>
__global__ void __launch_bounds__(kBlockThreads) TeamTreeKernel(const FusedDesc *__restrict__ items, uint32_t nitems,
    uint32_t ntiles, const void *const *__restrict__ srcPool, void *const *__restrict__ dstPool, uint32_t tilesPerItem,
    uint32_t *__restrict__ teamCtr, uint32_t roundTiles)
{
    TeamBody<TeamTreeEval<T, OP>>(items, nitems, ntiles, srcPool, dstPool, tilesPerItem, teamCtr, roundTiles, nullptr);
}

template <typename T, int OP>
__global__ void __launch_bounds__(kBlockThreads) TeamStackKernel(const FusedDesc *__restrict__ items, uint32_t nitems,
    uint32_t ntiles, const void *const *__restrict__ srcPool, void *const *__restrict__ dstPool, uint32_t tilesPerItem,
    uint32_t *__restrict__ teamCtr, uint32_t roundTiles)
{
    TeamBody<TeamStackEval<T, OP>>(items, nitems, ntiles, srcPool, dstPool, tilesPerItem, teamCtr, roundTiles, items + nitems);
}

}  // namespace hcclamd
