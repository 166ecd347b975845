// Device-side contract between the executor and the gfx950 kernels.
//
// These kernels stand where the reference has its closed Reducer / Sender / Transport leaf
// (call sites ALG/base/alg_template/temp_reduce_scatter/reduce_scatter_ring.cc:31-87) and its AIV
// copy / atomic-reduce kernels (ALG/base/alg_aiv_template/aiv_communication_base.h:367-485):
// element-wise dst = a (+) b and plain copies between rank buffers, all in one GPU's HBM.
#pragma once
#include <cstdint>

namespace hcclamd {

// One workgroup iteration handles one tile: 256 lanes x 16 bytes x 4.
constexpr uint32_t kTileBytes = 16384;
constexpr uint32_t kBlockThreads = 256;

// How a step's bytes may be accessed.
enum AccessMode : uint32_t {
    ACC_VEC16 = 0,      // every pointer 16-byte aligned, byte count a multiple of 16
    ACC_VEC16_ANY = 1,  // first destination 16-byte aligned, the other pointers at any element boundary; multiple of 16
    ACC_ELEM = 2        // element by element (heads, tails, unaligned buffers)
};

// dst = a            when b == nullptr
// dst = a (+) b      otherwise (a = the rank's own operand, b = the peer's)
struct StepDesc {
    void *dst;
    const void *a;
    const void *b;
    uint64_t bytes;
    uint32_t tile0;     // index of this step's first tile inside the launch
    uint32_t mode;      // AccessMode
};

// Fused item: read nsrc sources once, combine in the schedule's order, write ndst destinations.
//   chain : acc = src[0]; for j = 1..nsrc-1: acc = bit j of accLeftMask ? acc (+) src[j] : src[j] (+) acc
//   tree  : nleaf leaves, leaf i = src[2i] (+) src[2i+1] (src[2i+1] may be null); then
//           v[i] = v[i] (+) v[i+w] for w = 1, 2, 4, ... ; result v[0]
//   stack : any other expression.  Sources in evaluation order; after pushing src[j] the two topmost
//           values are folded ops[j] & 7 times, bit 8 + i of ops[j] set = the lower value is the left
//           operand of fold i.  The launch's op words (one uint32 per source-pool entry, same index)
//           follow its item table in memory; nleaf holds the stack depth the program needs.
struct FusedDesc {
    uint64_t bytes;
    uint64_t accLeftMask;
    uint32_t tile0;
    uint32_t mode;
    uint32_t nsrc;
    uint32_t ndst;
    uint32_t srcBase;   // index into the source pointer pool
    uint32_t dstBase;   // index into the destination pointer pool
    uint32_t nleaf;
    uint32_t flags;     // kFusedOrdinaryStores
};

// flags of a fused item
constexpr uint32_t kFusedOrdinaryStores = 1u;  // whole passes of the chain kernel store write-back instead of non-temporal

// flags of the step kernel
constexpr uint32_t kStepOrdinaryStores = 1u;   // write-back stores instead of non-temporal ones in the fast loop
constexpr uint32_t kStepReverse = 2u;          // the fast loop walks every step from its last tile to its first

// Small-segment gather (pure data movement, one source and one destination per segment, any byte alignment of
// either): one wave moves one segment through its share of the workgroup's LDS.
struct SegDesc {
    const void *src;
    void *dst;
    uint64_t bytes;     // <= kGatherMaxBytes
    uint64_t pad;
};
constexpr uint32_t kGatherMaxBytes = 8192;

enum KernelKind : int {
    KK_STEP = 0, KK_CHAIN = 1, KK_TREE = 2, KK_STACK = 3,
    KK_TEAM_CHAIN = 4, KK_TEAM_TREE = 5, KK_TEAM_STACK = 6,   // team forms of the fused kernels, see below
    KK_COUNT = 7,
    KK_GATHER = 7                                              // copy kernel table only
};

// Team form of a fused kernel: the workgroups of one XCD read their tiles together, park the results in LDS, and write
// them together (kernels_team.h).  Launched with a multiple of kTeamXcds workgroups (one per CU) and kTeamDynamicLds
// bytes of dynamic LDS; takes one more argument, the launch's team block in device memory, which belongs to this launch
// alone.  Layout, in uint32 words:
//   [x * kTeamCtrStride + kTeamArrive]   x < kTeamXcds: barrier arrivals of team x; kTeamGaveUpBit set once a wait ran out
//   [x * kTeamCtrStride + kTeamLeft]     workgroups of team x that have finished
//   [kTeamTicket]       regions handed out beyond the first kTeamXcds
//   [kTeamFinished]     teams that have finished
//   [kTeamRegionCount]  number of regions n (written by the host, never changed)
//   [kTeamHeaderWords ...]            n x TeamRegion (written by the host, never changed)
//   [kTeamHeaderWords + 2 n ...]      kTeamXcds x (n + 1) slots: the region of team x's round r + 1, plus 2; 1 = being drawn
// Everything but the count and the table starts out zero, and the kernel leaves it zero again.
constexpr uint32_t kTeamTiles = 8;        // tiles a workgroup can park per round
constexpr uint32_t kTeamXcds = 8;
constexpr uint32_t kTeamCtrStride = 32;   // words per XCD (128 bytes, a memory line of its own)
constexpr uint32_t kTeamArrive = 0, kTeamLeft = 1;
constexpr uint32_t kTeamGaveUpBit = 0x80000000u;
constexpr uint32_t kTeamTicket = kTeamXcds * kTeamCtrStride, kTeamFinished = kTeamTicket + 1, kTeamRegionCount = kTeamTicket + 2;
constexpr uint32_t kTeamHeaderWords = kTeamTicket + 4;
constexpr uint32_t kTeamDynamicLds = kTeamTiles * kTileBytes;
struct TeamRegion {
    uint32_t first;   // first tile
    uint32_t per;     // tiles per workgroup, 1 ... kTeamTiles: workgroup i of the team takes [first + i * per, first + (i + 1) * per)
};
inline uint32_t TeamBlockWords(uint32_t nregions) { return kTeamHeaderWords + 2u * nregions + kTeamXcds * (nregions + 1u); }

// Kernel entry for (data type, reduce op, kind); nullptr if the combination is not built.
// Signatures:
//   KK_STEP            (const StepDesc *steps, uint32_t nsteps, uint32_t nwhole, uint32_t ntiles, uint32_t flags)
//                      steps whose tiles are all whole and ACC_VEC16 come first: tiles [0, nwhole)
//   KK_CHAIN / KK_TREE / KK_STACK
//                      (const FusedDesc *items, uint32_t nitems, uint32_t ntiles,
//                       const void *const *srcPool, void *const *dstPool, uint32_t tilesPerItem)
//   KK_TEAM_*          the same and (uint32_t *teamBlock)
const void *LookupKernel(int hcclDataType, int hcclReduceOp, KernelKind kind);

//   KK_GATHER          (const SegDesc *segs, uint32_t nsegs, uint32_t unused, const void *unused, void *unused)
//                      copy kernel table only
// Byte-wise variants for pure data movement (all-gather, all-to-all-v): KK_STEP, KK_CHAIN, KK_TEAM_CHAIN and KK_GATHER.
const void *LookupCopyKernel(KernelKind kind);

}  // namespace hcclamd
