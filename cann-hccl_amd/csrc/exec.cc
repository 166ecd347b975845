// Task issue: plan -> descriptor tables in device memory -> HIP graph of kernel nodes -> replay.
// See runtime.h for the reference interfaces this replaces.
#include <algorithm>
#include <cstdio>
#include <cstring>
#include <sstream>

#include "log.h"
#include "noalloc.h"
#include "runtime.h"

namespace hcclamd {

namespace {

#define HIP_OK(expr)                                                                                  \
    do {                                                                                              \
        hipError_t e_ = (expr);                                                                       \
        if (e_ != hipSuccess) {                                                                       \
            HCCL_LOG_ERROR("%s failed: %s", #expr, hipGetErrorString(e_));                            \
            return HCCL_E_RUNTIME;                                                                    \
        }                                                                                             \
    } while (0)

uint32_t DtypeSize(int dt)
{
    static const uint32_t table[] = {1, 2, 4, 2, 4, 8, 8, 1, 2, 4, 8, 2, 16};
    return (dt >= 0 && dt <= 12) ? table[dt] : 0;
}

}  // namespace

// Descriptor tables too large to ride in kernel arguments pass through a ring of pinned host buffers of this size.
constexpr size_t kStageSlotBytes = size_t(128) << 10;
constexpr uint32_t kStageSlots = 8;

HcclResult EnsureDevice(Group *g, bool quiet)
{
    if (g->deviceReady) {
        return HCCL_SUCCESS;
    }
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || n <= 0) {
        if (!quiet) {
            HCCL_LOG_ERROR("no HIP device available: collectives need a GPU");
        }
        return HCCL_E_RUNTIME;
    }
    HIP_OK(hipGetDevice(&g->device));
    hipDeviceProp_t prop;
    HIP_OK(hipGetDeviceProperties(&prop, g->device));
    g->numCu = prop.multiProcessorCount > 0 ? uint32_t(prop.multiProcessorCount) : 256u;
    // Events that only order streams of this device against each other: no timestamps, and no system-scope fence when
    // they complete (the kernels on either side release and acquire at device scope themselves; a caller that reads
    // results on the host synchronises its own stream, which fences).  One thread per rank, 8 KiB all-reduce: 47 us
    // per collective at 8 ranks against 55 us with the fence, 78 against 95 at 16.
    constexpr unsigned kOrderOnly = hipEventDisableTiming | hipEventDisableSystemFence;
    g->arriveEvents.assign(g->p, nullptr);
    for (uint32_t r = 0; r < g->p; r++) {
        HIP_OK(hipEventCreateWithFlags(&g->arriveEvents[r], kOrderOnly));
    }
    for (hipEvent_t &e : g->doneEvents) {
        HIP_OK(hipEventCreateWithFlags(&e, kOrderOnly));
    }
    HIP_OK(hipEventCreateWithFlags(&g->p2pDoneEvent, kOrderOnly));
    HIP_OK(hipStreamCreateWithFlags(&g->copyStream, hipStreamNonBlocking));
    g->stageSlots.resize(kStageSlots);
    for (StageSlot &slot : g->stageSlots) {
        HIP_OK(hipHostMalloc(&slot.host, kStageSlotBytes, hipHostMallocDefault));
        HIP_OK(hipEventCreateWithFlags(&slot.done, hipEventDisableTiming));
    }
    g->scratch.assign(g->p, nullptr);
    g->arena.allocFn = [](size_t bytes) -> void * {
        void *mem = nullptr;
        if (hipMalloc(&mem, bytes) != hipSuccess) {
            (void)hipGetLastError();
            return nullptr;
        }
        return mem;
    };
    g->arena.freeFn = [](void *mem) { (void)hipFree(mem); };
    // Set-up for the entry point that allocates nothing: the address of the fixed workspace on this
    // device (g->device is the current device), and every kernel's code object loaded now, so that no
    // later launch is the first use of its module.
    HIP_OK(NoAllocWorkspace(g->device, &g->noAllocBase));
    for (int dt = 0; dt <= 11; dt++) {
        const void *f = LookupKernel(dt, 0, KK_STEP);
        hipFuncAttributes attr;
        if (f != nullptr) {
            HIP_OK(hipFuncGetAttributes(&attr, f));
        }
    }
    {
        hipFuncAttributes attr;
        HIP_OK(hipFuncGetAttributes(&attr, LookupCopyKernel(KK_STEP)));
    }
    // the team kernels park their results in more LDS than a kernel gets without asking
    for (int dt = 0; dt <= 11; dt++) {
        for (int op = 0; op <= 3; op++) {
            for (KernelKind kind : {KK_TEAM_CHAIN, KK_TEAM_TREE, KK_TEAM_STACK}) {
                const void *f = LookupKernel(dt, op, kind);
                if (f != nullptr) {
                    HIP_OK(hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, int(kTeamDynamicLds)));
                }
            }
        }
    }
    HIP_OK(hipFuncSetAttribute(LookupCopyKernel(KK_TEAM_CHAIN), hipFuncAttributeMaxDynamicSharedMemorySize, int(kTeamDynamicLds)));
    g->deviceReady = true;
    return HCCL_SUCCESS;
}

namespace {

HcclResult EnsureScratch(Group *g, uint64_t bytes)
{
    if (bytes <= g->scratchBytes) {
        return HCCL_SUCCESS;
    }
    // Collectives issued earlier may still be running out of the old buffers, and a caller's graph may replay
    // some: the buffers are set aside, not freed (freeing waits for the whole device).  Those a graph points at
    // stay until the group goes; the others are freed at the next point where the device is known to be idle.
    // Growing by at least a factor of two keeps what is set aside below the size in use.
    for (uint32_t r = 0; r < g->p; r++) {
        if (g->scratch[r]) {
            (g->pinnedScratchUsers > 0 ? g->retiredScratch : g->idleScratch).push_back(g->scratch[r]);
            g->scratch[r] = nullptr;
        }
    }
    g->pinnedScratchUsers = 0;
    bytes = std::max(bytes, 2 * g->scratchBytes);
    g->scratchBytes = 0;
    g->scratchGen++;
    for (uint32_t r = 0; r < g->p; r++) {
        HIP_OK(hipMalloc(&g->scratch[r], bytes));
    }
    g->scratchBytes = bytes;
    return HCCL_SUCCESS;
}

// With the device idle: frees what earlier calls set aside.
void ReleaseIdle(Group *g)
{
    g->stale.clear();
    for (void *s : g->idleScratch) {
        (void)hipFree(s);
    }
    g->idleScratch.clear();
}

struct Builder {
    Group *g;
    std::vector<void *> scratch;  // per rank: the group's own allocations, or shares of the fixed workspace
    std::vector<uint8_t> host;   // image of the device allocation

    size_t Reserve(size_t bytes)
    {
        size_t at = (host.size() + 255) & ~size_t(255);
        host.resize(at + bytes);
        return at;
    }
    char *Ptr(const Ref &r) const
    {
        char *base = nullptr;
        switch (r.buf) {
            case BUF_SEND: base = static_cast<char *>(g->ctx->send[r.rank]); break;
            case BUF_RECV: base = static_cast<char *>(g->ctx->recv[r.rank]); break;
            default: base = static_cast<char *>(scratch[r.rank]); break;
        }
        return base + r.off;
    }
};

// Cuts [0, bytes) into an element-wise head, a 16-byte vector body and an element-wise tail, given
// the addresses involved (the first one is a destination; all are multiples of the element size).
// The head brings the first destination to a 16-byte boundary; pointers that are then not on one
// too are accessed with unaligned 128-bit loads and stores (ACC_VEC16_ANY).  emit(offset, bytes, mode).
// A long body is cut once more so that its main part starts on a 128-byte boundary of the destination:
// a wave stores 1 KiB at a time, and when those stores straddle memory lines every line is written in
// two pieces (measured, 8-rank fp32 all-reduce of 256 MiB per rank with all buffers 16 bytes off a
// 128-byte boundary: 0.97 ms fused against 0.76 ms aligned).
template <typename F> void SplitByAlignment(const std::vector<uintptr_t> &addrs, uint64_t bytes, F emit)
{
    uintptr_t anchor = addrs[0];
    bool co = true;
    for (uintptr_t a : addrs) {
        co = co && ((a & 15) == (anchor & 15));
    }
    uint64_t head = std::min<uint64_t>(bytes, (16 - (anchor & 15)) & 15);
    uint64_t body = (bytes - head) & ~uint64_t(15);
    uint64_t tail = bytes - head - body;
    if (head) {
        emit(uint64_t(0), head, uint32_t(ACC_ELEM));
    }
    if (body) {
        const uint32_t mode = co ? ACC_VEC16 : ACC_VEC16_ANY;
        const uint64_t lead = (128 - ((anchor + head) & 127)) & 127;     // a multiple of 16
        if (lead != 0 && body >= 4 * uint64_t(kTileBytes)) {
            emit(head, lead, mode);
            emit(head + lead, body - lead, mode);
        } else {
            emit(head, body, mode);
        }
    }
    if (tail) {
        emit(head + body, tail, uint32_t(ACC_ELEM));
    }
}

constexpr size_t kGraphMinLaunches = 12;   // fewer launches go out one by one
constexpr uint32_t kTeamMinRounds = 2;     // the team kernels are chosen for launches of at least this many full rounds
constexpr size_t kAsyncUploadBytes = 4 * kNoAllocUploadBytes;   // tables up to this size are uploaded by launches

uint32_t TilesOf(uint64_t bytes) { return uint32_t((bytes + kTileBytes - 1) / kTileBytes); }

struct PendingLaunch {
    LaunchRec rec;
    size_t tableAt = 0, srcAt = 0, dstAt = 0, ctrAt = 0;
    bool gather = false;     // no pointer pools
};

// Store kind for the step kernel's fast loop.  Ordinary (write-back) stores leave the data in the
// 256 MB memory-side cache, which pays when the next phase reads it back and a phase's output fits
// there; otherwise they only displace useful lines and non-temporal stores are better.  Measured on
// MI355X, 8 ranks, step by step (non-temporal / ordinary, us): ring all-reduce 256 MiB 1478 / 1433,
// ring reduce 886 / 840, ring broadcast 615 / 579 (every phase forwards what the previous one wrote,
// 256 MiB or less per phase); halving-doubling all-reduce 1544 / 1685, mesh broadcast 583 / 638 (phases
// of 1 GiB and more); uniform all-to-all 727 / 785 (nothing is read back).
constexpr uint64_t kMemorySideCacheBytes = 256ull << 20;

bool PreferOrdinaryStores(const Plan &plan, const std::vector<void *> &send, const std::vector<void *> &recv)
{
    typedef std::pair<uint32_t, uint8_t> Where;   // (rank, buffer); a send buffer that is the receive buffer counts as it
    auto where = [&](const Ref &r) {
        uint8_t b = r.buf;
        if (b == BUF_SEND && r.rank < send.size() && send[r.rank] == recv[r.rank]) {
            b = BUF_RECV;
        }
        return Where(r.rank, b);
    };
    std::map<Where, std::vector<std::pair<uint64_t, uint64_t>>> prev;   // what the previous phase wrote, sorted
    uint64_t maxWritten = 0, written = 0, readBack = 0;
    for (const Phase &ph : plan.phases) {
        uint64_t w = 0;
        for (const Step &st : ph.steps) {
            w += st.bytes;
            for (const Ref *src : {&st.a, st.reduce ? &st.b : nullptr}) {
                if (src == nullptr || st.bytes == 0) {
                    continue;
                }
                auto it = prev.find(where(*src));
                if (it == prev.end()) {
                    continue;
                }
                const auto &v = it->second;
                const uint64_t lo = src->off, hi = src->off + st.bytes;
                auto k = std::upper_bound(v.begin(), v.end(), std::make_pair(lo, UINT64_MAX));
                if (k != v.begin()) {
                    --k;
                }
                for (; k != v.end() && k->first < hi; ++k) {
                    uint64_t a = std::max(lo, k->first), e = std::min(hi, k->second);
                    if (e > a) {
                        readBack += e - a;
                    }
                }
            }
        }
        maxWritten = std::max(maxWritten, w);
        written += w;
        prev.clear();
        for (const Step &st : ph.steps) {
            if (st.bytes) {
                prev[where(st.dst)].emplace_back(st.dst.off, st.dst.off + st.bytes);
            }
        }
        for (auto &kv : prev) {
            std::sort(kv.second.begin(), kv.second.end());
        }
    }
    return maxWritten <= kMemorySideCacheBytes && 2 * readBack >= written;
}

// With noAlloc the tables go to the fixed workspace through launches on `stream`, and the schedule's
// scratch is the workspace's data part cut into equal shares, one per rank.
HcclResult BuildTables(Group *g, Prepared *pp, bool reduceColl, int dtype, int op, bool noAlloc, hipStream_t stream)
{
    Builder b;
    b.g = g;
    if (noAlloc) {
        const size_t share = (kNoAllocDataBytes / g->p) & ~size_t(255);
        char *data = static_cast<char *>(g->noAllocBase) + kNoAllocTableBytes;
        for (uint32_t r = 0; r < g->p; r++) {
            b.scratch.push_back(data + size_t(r) * share);
        }
    } else {
        b.scratch = g->scratch;
    }
    std::vector<PendingLaunch> pending;
    // A long launch slows down as it goes when its items move from buffer to buffer (all-to-all, scatter, reduce-
    // scatter: workgroups drift apart and with them the regions of memory in use at one time), and launch boundaries
    // bring them together again.  Measured, 8 ranks: all-to-all of 32 / 64 MiB per pair 774 / 1614 us in one launch,
    // 688 / 1382 us cut at 512 MiB; reduce-scatter to 32 / 64 MiB per rank 408 / 825 us against 393 / 787 us.
    // Collectives that sweep the same buffers from end to end (all-reduce, reduce, broadcast, all-gather) gain
    // nothing or lose (all-reduce of 256 MiB per rank 756 us in one launch, 769 us cut at 512 MiB).
    uint64_t capBytes = g->cfg.launchCapMiB > 0 ? uint64_t(g->cfg.launchCapMiB) << 20 : 0;
    if (g->cfg.launchCapMiB < 0) {
        const int coll = g->ctx->sig.coll;
        // (the two-level reduce-scatter, whose items read their blocks group by group, loses 2 - 4 % and is left whole)
        const bool hops = coll == COLL_ALLTOALLV || coll == COLL_SCATTER || coll == COLL_SENDRECV ||
            (coll == COLL_REDUCESCATTER && g->cfg.servers <= 1);
        capBytes = hops ? uint64_t(512) << 20 : 0;
    }
    // Launch width.  Streaming kernels on this part run best with few, fat workgroups as long as a
    // lane keeps enough memory operations in flight: 1 workgroup per CU when an item touches 8 or
    // more streams (sources + destinations), more when it touches fewer (measured on MI355X: 8 -> 8
    // all-reduce and 1 -> 8 all-gather best at 1 per CU, the 2 -> 1 step kernel at 2 per CU).
    const uint32_t stepGrid = std::max(1u, g->numCu * (g->cfg.blocksPerCu ? g->cfg.blocksPerCu : 2u));
    uint32_t fusedPerCu = g->cfg.blocksPerCu;
    if (fusedPerCu == 0) {
        double streamBytes = 0, storeBytes = 0, bytes = 0;
        for (const FusedItem &it : pp->plan->fused) {
            uint32_t nsrc = 0;
            for (uint8_t v : it.srcValid) {
                nsrc += v;
            }
            streamBytes += double(nsrc + it.dst.size()) * double(it.bytes);
            storeBytes += double(it.dst.size()) * double(it.bytes);
            bytes += double(it.bytes);
        }
        double streams = bytes > 0 ? streamBytes / bytes : 2.0;   // loads + stores per lane and vector
        fusedPerCu = streams >= 8.0 ? 1u : (streams >= 3.0 ? 2u : 4u);
        // That holds for shapes that write as much as they read or more, and for everything much larger than the
        // memory-side cache.  Many sources into one destination (reduce-scatter, reduce) of 8- and 16-bit elements,
        // where a combine costs several instructions, run better wide up to about a gigabyte in all (measured, bf16
        // sum: 8 ranks x 64 MiB 104 us at 1 per CU, 99 at 8; 16 ranks x 64 MiB 196 / 189; a reduce of 8 x 256 MiB in one
        // launch 416 / 423, so not there, but a reduce-scatter of that size, which goes out in launches of 512 MiB, 413 /
        // 396; fp32 within a percent either way at every size).
        const double launchBytes = capBytes != 0 ? std::min(streamBytes, double(capBytes)) : streamBytes;
        if (fusedPerCu == 1 && reduceColl && DtypeSize(dtype) <= 2 && storeBytes * 5.0 <= streamBytes &&
            launchBytes <= 1.25 * 1024.0 * 1024.0 * 1024.0) {
            fusedPerCu = 8;
        }
        // Plain copies (one source, one destination) go through the copy kernel, which really gets the
        // occupancy it is launched with; with non-temporal stores more workgroups only widen the range
        // of addresses written at a time, which this memory system likes less (measured, 8 ranks:
        // uniform all-to-all of 32 MiB per pair 752 us at 1 or 2 per CU, 835 us at 4, 850 us at 8;
        // 16-rank all-to-all-v, 106 MB of ragged segments: 55.6 / 40.5 / 42.5 / 41.3 us at 1 / 2 / 4 / 8).
        if (!reduceColl && streams < 3.0) {
            fusedPerCu = 2u;
        }
        // few tiles per workgroup: a second workgroup per CU evens out the tail (measured: 16-rank
        // ring all-reduce of 32 MiB per rank 241 us at 1 per CU, 220 us at 2)
        if (fusedPerCu == 1 && bytes / kTileBytes < 32.0 * g->numCu) {
            fusedPerCu = 2;
        }
    }
    const uint32_t treeGrid = std::max(1u, g->numCu * fusedPerCu);
    const uint32_t fusedGrid = std::max(1u, g->numCu * fusedPerCu);

    if (!pp->fused) {
        const void *func = reduceColl ? LookupKernel(dtype, op, KK_STEP) : LookupCopyKernel(KK_STEP);
        if (func == nullptr) {
            return HCCL_E_NOT_SUPPORT;
        }
        const bool ordinaryStores = g->cfg.stepStores < 0 ? PreferOrdinaryStores(*pp->plan, g->ctx->send, g->ctx->recv)
                                                          : g->cfg.stepStores == 1;
        uint32_t launchNo = 0;
        for (const Phase &ph : pp->plan->phases) {
            // whole-tile 16-byte-vector pieces first (the kernel's fast loop), everything else after
            std::vector<StepDesc> whole, ragged;
            for (const Step &s : ph.steps) {
                char *dst = b.Ptr(s.dst);
                char *a = b.Ptr(s.a);
                char *bb = s.reduce ? b.Ptr(s.b) : nullptr;
                std::vector<uintptr_t> addrs = {reinterpret_cast<uintptr_t>(dst), reinterpret_cast<uintptr_t>(a)};
                if (bb) {
                    addrs.push_back(reinterpret_cast<uintptr_t>(bb));
                }
                SplitByAlignment(addrs, s.bytes, [&](uint64_t off, uint64_t n, uint32_t mode) {
                    auto add = [&](std::vector<StepDesc> &to, uint64_t at, uint64_t len) {
                        StepDesc d;
                        d.dst = dst + at;
                        d.a = a + at;
                        d.b = bb ? bb + at : nullptr;
                        d.bytes = len;
                        d.tile0 = 0;
                        d.mode = mode;
                        to.push_back(d);
                    };
                    uint64_t body = (mode == ACC_VEC16) ? n / kTileBytes * kTileBytes : 0;
                    if (body) {
                        add(whole, off, body);
                    }
                    if (n > body) {
                        add(ragged, off + body, n - body);
                    }
                });
            }
            // Every other launch walks the data the other way round, so that a phase starts with what the
            // phase before it wrote last (measured, 8-rank fp32 ring all-reduce of 256 MiB per rank: 1.431 ms
            // against 1.437 ms; running all phases on one 16 ... 128 MiB window of offsets at a time, to keep
            // the data between phases in the 256 MB memory-side cache, was slower: 1.44 ... 1.81 ms).
            const bool reverse = g->cfg.stepSweep == 1 && (launchNo & 1u) != 0;
            if (reverse) {
                std::reverse(whole.begin(), whole.end());
            }
            std::vector<StepDesc> descs;
            uint32_t tiles = 0, nwhole = 0;
            for (std::vector<StepDesc> *v : {&whole, &ragged}) {
                for (StepDesc &d : *v) {
                    d.tile0 = tiles;
                    tiles += TilesOf(d.bytes);
                    descs.push_back(d);
                }
                if (v == &whole) {
                    nwhole = tiles;
                }
            }
            if (descs.empty()) {
                continue;
            }
            PendingLaunch pl;
            pl.tableAt = b.Reserve(descs.size() * sizeof(StepDesc));
            std::memcpy(b.host.data() + pl.tableAt, descs.data(), descs.size() * sizeof(StepDesc));
            pl.rec.func = func;
            pl.rec.nitems = uint32_t(descs.size());
            pl.rec.ntiles = tiles;
            pl.rec.nwhole = nwhole;
            // the fast loop hides its descriptor lookups behind its loads and runs best with one
            // workgroup per CU once there are 16 or more tiles per workgroup (measured: 128 MiB per rank
            // 710 us at 1 per CU, 722 us at 2; 32 MiB per rank 207 us against 204 us)
            uint32_t grid = stepGrid;
            if (g->cfg.blocksPerCu == 0 && nwhole >= 16 * g->numCu) {
                grid = g->numCu;
            }
            pl.rec.grid = std::min(tiles, grid);
            pl.rec.flags = (ordinaryStores ? kStepOrdinaryStores : 0u) | (reverse ? kStepReverse : 0u);
            pl.rec.fusedArgs = false;
            pending.push_back(pl);
            launchNo++;
        }
    } else {
        // Fused results are streamed past the caches (non-temporal stores) unless the caller asks for
        // write-back stores.  Measured, 8-rank fp32 all-reduce replayed on the same buffers: write-back is
        // 5 % and 12 % faster at 16 and 32 MiB per rank (the output then stays in the 256 MB memory-side
        // cache), 20 % slower at 4 MiB and 7 % slower from 64 MiB per rank up.
        // Pure data movement with one source and many destinations (all-gather, broadcast) is 4 - 5 % faster with
        // write-back stores once the output is far larger than the memory-side cache (8 ranks: all-gather to
        // 256 MiB per rank 473 us against 501 us, broadcast of 256 MiB 425 us against 447 us); one-to-one copies
        // are not (uniform all-to-all 773 us against 752 us).
        bool fusedOrdinary = g->cfg.fusedStores == 1;
        if (g->cfg.fusedStores < 0 && !reduceColl) {
            double written = 0, read = 0;
            for (const FusedItem &it : pp->plan->fused) {
                written += double(it.dst.size()) * double(it.bytes);
                read += double(it.bytes);
            }
            fusedOrdinary = written >= 4.0 * read && written >= 2.0 * double(kMemorySideCacheBytes);
        }
        // Pure data movement in many short segments (an all-to-all-v of a few hundred bytes per pair): those go to
        // the gather kernel, a wave per segment through LDS, instead of a tile, a table search and up to three
        // descriptors each (measured, 64 ranks, 4096 segments of 430 bytes on average: 32 us with the tile kernel).
        auto movable = [&](const FusedItem &it, uint64_t limit) {
            return !reduceColl && it.kind != FK_TREE && it.kind != FK_STACK && it.dst.size() == 1 && it.src.size() == 1 &&
                it.bytes <= limit;
        };
        size_t nshort = 0;
        for (const FusedItem &it : pp->plan->fused) {
            nshort += movable(it, kGatherMaxBytes) ? 1 : 0;
        }
        // Once the gather kernel runs anyway it also takes the few segments of up to eight times its piece size, cut
        // into pieces, so that they do not cost a launch of their own.
        const bool gather = nshort >= 16;
        auto shortSegment = [&](const FusedItem &it) { return gather && movable(it, 8 * uint64_t(kGatherMaxBytes)); };
        if (gather) {
            std::vector<SegDesc> segs;
            segs.reserve(pp->plan->fused.size());
            for (const FusedItem &it : pp->plan->fused) {
                if (!shortSegment(it)) {
                    continue;
                }
                for (uint64_t at = 0; at < it.bytes; at += kGatherMaxBytes) {
                    SegDesc d;
                    d.src = b.Ptr(it.src[0]) + at;
                    d.dst = b.Ptr(it.dst[0]) + at;
                    d.bytes = std::min<uint64_t>(kGatherMaxBytes, it.bytes - at);
                    d.pad = 0;
                    segs.push_back(d);
                }
            }
            const void *func = LookupCopyKernel(KK_GATHER);
            if (func == nullptr) {
                return HCCL_E_NOT_SUPPORT;
            }
            if (!segs.empty()) {
                PendingLaunch pl;
                pl.tableAt = b.Reserve(segs.size() * sizeof(SegDesc));
                std::memcpy(b.host.data() + pl.tableAt, segs.data(), segs.size() * sizeof(SegDesc));
                pl.rec.func = func;
                pl.rec.nitems = uint32_t(segs.size());
                pl.rec.ntiles = 0;
                // a wave per segment, four waves per workgroup, at most four workgroups per CU (LDS)
                const uint32_t want = uint32_t((segs.size() + 3) / 4);
                pl.rec.grid = std::max(1u, std::min(want, 4u * g->numCu));
                pl.rec.fusedArgs = true;
                pl.gather = true;
                pending.push_back(pl);
            }
        }
        // one launch per kernel kind present, or several under a launch cap: the items in their order, cut where the
        // bytes a launch moves (read and written) reach the cap
        for (int kind : {int(KK_CHAIN), int(KK_TREE), int(KK_STACK)}) {
            std::vector<FusedDesc> descs;
            std::vector<const void *> srcPool;
            std::vector<uint32_t> opPool;      // stack items: one word per source-pool entry
            std::vector<void *> dstPool;
            uint32_t tiles = 0;
            uint64_t traffic = 0;
            std::vector<char *> srcs, dsts;        // reused from item to item: an all-to-all-v has thousands
            std::vector<uintptr_t> addrs;
            const void *func = reduceColl ? LookupKernel(dtype, op, KernelKind(kind)) : LookupCopyKernel(KernelKind(kind));
            auto flush = [&]() {
                if (descs.empty()) {
                    return;
                }
                PendingLaunch pl;
                // the op words of the stack kernel sit right behind its item table
                pl.tableAt = b.Reserve(descs.size() * sizeof(FusedDesc) + opPool.size() * sizeof(uint32_t));
                std::memcpy(b.host.data() + pl.tableAt, descs.data(), descs.size() * sizeof(FusedDesc));
                if (!opPool.empty()) {
                    std::memcpy(b.host.data() + pl.tableAt + descs.size() * sizeof(FusedDesc), opPool.data(),
                        opPool.size() * sizeof(uint32_t));
                }
                pl.srcAt = b.Reserve(srcPool.size() * sizeof(void *));
                std::memcpy(b.host.data() + pl.srcAt, srcPool.data(), srcPool.size() * sizeof(void *));
                pl.dstAt = b.Reserve(dstPool.size() * sizeof(void *));
                std::memcpy(b.host.data() + pl.dstAt, dstPool.data(), dstPool.size() * sizeof(void *));
                pl.rec.func = func;
                pl.rec.nitems = uint32_t(descs.size());
                pl.rec.ntiles = tiles;
                // equal slices (the usual collective): the kernels find a tile's item without searching the table
                pl.rec.tilesPerItem = TilesOf(descs[0].bytes);
                for (size_t i = 0; i < descs.size(); i++) {
                    const uint32_t t = TilesOf(descs[i].bytes);
                    if (i + 1 < descs.size() ? t != pl.rec.tilesPerItem : t > pl.rec.tilesPerItem) {
                        pl.rec.tilesPerItem = 0;
                        break;
                    }
                }
                pl.rec.grid = std::min(tiles, kind == int(KK_TREE) ? treeGrid : fusedGrid);
                pl.rec.fusedArgs = true;
                // Team form (kernels_team.h): pays when every workgroup has much to read or to write per tile and the
                // launch runs for many rounds.  Measured on MI355X with streams of 256 MiB (sources : destinations,
                // plain / team, TB/s): 8 : 8 5.3 / 5.9, 1 : 8 4.9 / 5.9, 1 : 7 4.9 / 5.8, 4 : 4 5.4 / 5.7, 8 : 1
                // 5.8 / 6.0; 2 : 2 5.5 / 5.3, 2 : 1 5.8 / 4.9, 1 : 1 5.8 / 4.2 (a round is then too short for its barrier).
                const KernelKind teamKind = kind == int(KK_TREE) ? KK_TEAM_TREE : (kind == int(KK_STACK) ? KK_TEAM_STACK : KK_TEAM_CHAIN);
                const void *teamFunc = reduceColl ? LookupKernel(dtype, op, teamKind) : LookupCopyKernel(teamKind);
                const bool teamFits = teamFunc != nullptr && g->numCu >= kTeamXcds && g->numCu % kTeamXcds == 0 && g->cfg.blocksPerCu == 0;
                bool team = teamFits && g->cfg.team == 1;
                double storeStreams = 0, allStreams = 0, bytes = 0;
                if (teamFits && g->cfg.team != 0) {
                    for (const FusedDesc &d : descs) {
                        uint32_t nsrc = 0;
                        for (uint32_t k = 0; k < d.nsrc; k++) {
                            nsrc += srcPool[d.srcBase + k] != nullptr ? 1u : 0u;
                        }
                        storeStreams += double(d.ndst) * double(d.bytes);
                        allStreams += double(d.ndst + nsrc) * double(d.bytes);
                        bytes += double(d.bytes);
                    }
                    // A round should keep a workgroup busy for a mebibyte or two per phase (8 tiles of 8 streams): fewer
                    // tiles per round when a tile has many more sources or destinations than that (measured, 32-rank
                    // bf16 all-reduce of 128 MiB per rank: 1650 / 1607 / 1623 us with 2 / 4 / 8 tiles; 8 ranks x 256 MiB
                    // fp32: 892 / 788 / 743 us).
                    const double widest = bytes > 0 ? std::max(storeStreams, allStreams - storeStreams) / bytes : 1.0;
                    pl.rec.roundTiles = g->cfg.teamTiles != 0 ? std::min(g->cfg.teamTiles, kTeamTiles)
                                                              : std::max(1u, std::min(kTeamTiles, uint32_t(128.0 / std::max(1.0, widest))));
                    if (g->cfg.team < 0) {
                        team = bytes > 0 && storeStreams >= 4.0 * bytes && allStreams >= 8.0 * bytes &&
                            tiles >= kTeamMinRounds * pl.rec.roundTiles * g->numCu;
                    }
                }
                if (team) {
                    pl.rec.func = teamFunc;
                    pl.rec.team = true;
                    pl.rec.grid = g->numCu;
                    pl.rec.dynamicLds = kTeamDynamicLds;
                    // The regions the teams draw: roundTiles tiles per workgroup (fewer when that would leave an XCD
                    // without a region); over the last quarter of the tiles the size is halved whenever fewer than 8
                    // regions of the current size are left.  The XCDs do not all move data at the same rate, and with
                    // regions that get smaller towards the end they finish together (measured, 8 x 256 MiB fp32
                    // all-reduce: 727 us with 64 equal regions dealt out in order, 714 us with the shrinking tail
                    // drawn from the counter; shrinking earlier costs more than it brings, small regions run slower --
                    // the more so since rounds of 8 and 4 whole tiles are read in one piece: with "fewer than 16"
                    // all-gather and broadcast took 2 % longer, the all-reduces 1 %).
                    const uint32_t perX = g->numCu / kTeamXcds;
                    std::vector<TeamRegion> regions;
                    uint32_t per = pl.rec.roundTiles;
                    while (per > 1 && uint64_t(per) * perX * kTeamXcds > tiles) {
                        per /= 2;
                    }
                    for (uint32_t at = 0; at < tiles;) {
                        const uint32_t left = tiles - at;
                        if (uint64_t(at) * 4 >= uint64_t(tiles) * 3) {
                            while (per > 1 && uint64_t(per) * perX * 8 > left) {
                                per /= 2;
                            }
                        }
                        regions.push_back(TeamRegion{at, per});
                        at += uint32_t(std::min<uint64_t>(left, uint64_t(per) * perX));
                    }
                    const uint32_t n = uint32_t(regions.size());
                    pl.ctrAt = b.Reserve(size_t(TeamBlockWords(n)) * 4);     // zero in the image, and zero again after every launch
                    uint32_t *block = reinterpret_cast<uint32_t *>(b.host.data() + pl.ctrAt);
                    block[kTeamRegionCount] = n;
                    std::memcpy(block + kTeamHeaderWords, regions.data(), regions.size() * sizeof(TeamRegion));
                }
                pending.push_back(pl);
                descs.clear();
                srcPool.clear();
                opPool.clear();
                dstPool.clear();
                tiles = 0;
                traffic = 0;
            };
            for (const FusedItem &it : pp->plan->fused) {
                int want = it.kind == FK_TREE ? int(KK_TREE) : (it.kind == FK_STACK ? int(KK_STACK) : int(KK_CHAIN));
                if (want != kind || shortSegment(it)) {
                    continue;
                }
                if (func == nullptr) {
                    return HCCL_E_NOT_SUPPORT;
                }
                srcs.clear();
                dsts.clear();
                addrs.clear();
                for (const Ref &d : it.dst) {
                    dsts.push_back(b.Ptr(d));
                    addrs.push_back(reinterpret_cast<uintptr_t>(dsts.back()));
                }
                uint32_t streams = uint32_t(dsts.size());
                for (size_t k = 0; k < it.src.size(); k++) {
                    char *s = it.srcValid[k] ? b.Ptr(it.src[k]) : nullptr;
                    srcs.push_back(s);
                    if (s) {
                        addrs.push_back(reinterpret_cast<uintptr_t>(s));
                        streams++;
                    }
                }
                uint64_t mask = 0;
                for (size_t k = 0; k < it.accLeft.size() && k < 64; k++) {
                    mask |= uint64_t(it.accLeft[k] ? 1 : 0) << k;
                }
                // an item that alone exceeds the cap goes in pieces of whole tiles
                const uint64_t piece = capBytes == 0 ? ~uint64_t(0)
                                                     : std::max<uint64_t>(kTileBytes, capBytes / streams / kTileBytes * kTileBytes);
                SplitByAlignment(addrs, it.bytes, [&](uint64_t off0, uint64_t n0, uint32_t mode) {
                    for (uint64_t at = 0; at < n0; at += piece) {
                        const uint64_t off = off0 + at, n = std::min(piece, n0 - at);
                        FusedDesc d;
                        std::memset(&d, 0, sizeof(d));
                        d.bytes = n;
                        d.accLeftMask = mask;
                        d.tile0 = tiles;
                        d.mode = mode;
                        d.nsrc = uint32_t(srcs.size());
                        d.ndst = uint32_t(dsts.size());
                        d.srcBase = uint32_t(srcPool.size());
                        d.dstBase = uint32_t(dstPool.size());
                        d.nleaf = it.nleaf;
                        d.flags = fusedOrdinary ? kFusedOrdinaryStores : 0u;
                        for (size_t k = 0; k < srcs.size(); k++) {
                            srcPool.push_back(srcs[k] ? srcs[k] + off : nullptr);
                            if (kind == int(KK_STACK)) {
                                opPool.push_back(k < it.ops.size() ? it.ops[k] : 0u);
                            }
                        }
                        for (char *t : dsts) {
                            dstPool.push_back(t + off);
                        }
                        tiles += TilesOf(n);
                        traffic += n * streams;
                        descs.push_back(d);
                        if (capBytes != 0 && traffic >= capBytes) {
                            flush();
                        }
                    }
                });
            }
            flush();
        }
    }
    if (pending.empty()) {
        return HCCL_SUCCESS;   // nothing to move (e.g. one rank, in place)
    }
    if (noAlloc) {
        b.host.resize((b.host.size() + 255) & ~size_t(255));
        if (b.host.size() > kNoAllocTableBytes) {
            HCCL_LOG_ERROR("%s without allocation: the descriptor tables need %zu bytes, the fixed workspace holds %zu",
                CollName(g->ctx->sig.coll), b.host.size(), kNoAllocTableBytes);
            return HCCL_E_PARA;
        }
        pp->devTables = g->noAllocBase;
        HIP_OK(UploadThroughKernelArgs(pp->devTables, b.host.data(), b.host.size(), stream));
    } else {
        b.host.resize((b.host.size() + 255) & ~size_t(255));
        pp->devTables = g->arena.Alloc(b.host.size(), &pp->tableChunk);
        if (pp->devTables == nullptr) {
            HCCL_LOG_ERROR("no device memory for %zu bytes of descriptor tables", b.host.size());
            return HCCL_E_MEMORY;
        }
        if (b.host.size() <= kAsyncUploadBytes && stream != nullptr) {
            // small tables ride on a few upload launches in front of the collective instead of a copy that
            // waits for the device (measured, fused 8-rank all-reduce with fresh buffers every call: 42 us
            // of host time per call with the copy)
            HIP_OK(hipEventCreateWithFlags(&pp->uploaded, hipEventDisableTiming));
            HIP_OK(UploadThroughKernelArgs(pp->devTables, b.host.data(), b.host.size(), stream));
            HIP_OK(hipEventRecord(pp->uploaded, stream));
            pp->uploadStream = stream;
            pp->uploadComplete = false;
            pp->hostTables.swap(b.host);
        } else if (b.host.size() <= kStageSlotBytes && stream != nullptr && !g->stageSlots.empty()) {
            // medium tables (an all-to-all-v between 16 ranks: 40 KiB) go through a ring of pinned host buffers, from
            // where a launch on the caller's stream fetches them: the call does not wait for it, and the stream does
            // not change engines as it would for a copy command.  A slot comes round again after as many collectives
            // as the ring has slots; its previous fetch has normally long finished.
            StageSlot &slot = g->stageSlots[g->stageNext++ % g->stageSlots.size()];
            if (slot.used) {
                HIP_OK(hipEventSynchronize(slot.done));
            }
            std::memcpy(slot.host, b.host.data(), b.host.size());
            HIP_OK(UploadFromPinned(pp->devTables, slot.host, b.host.size(), stream));
            HIP_OK(hipEventRecord(slot.done, stream));
            slot.used = true;
            HIP_OK(hipEventCreateWithFlags(&pp->uploaded, hipEventDisableTiming));
            HIP_OK(hipEventRecord(pp->uploaded, stream));
            pp->uploadStream = stream;
            pp->uploadComplete = false;
            pp->hostTables.swap(b.host);
        } else {
            // over a stream of the library's own, which no caller captures (a plain copy goes through the null
            // stream, which a caller's capture of a blocking stream would not tolerate)
            HIP_OK(hipMemcpyAsync(pp->devTables, b.host.data(), b.host.size(), hipMemcpyHostToDevice, g->copyStream));
            HIP_OK(hipStreamSynchronize(g->copyStream));
        }
    }
    char *base = static_cast<char *>(pp->devTables);
    for (PendingLaunch &pl : pending) {
        pl.rec.table = base + pl.tableAt;
        if (pl.rec.fusedArgs && !pl.gather) {
            pl.rec.srcPool = base + pl.srcAt;
            pl.rec.dstPool = base + pl.dstAt;
        }
        if (pl.rec.team) {
            pl.rec.teamCtr = base + pl.ctrAt;
        }
        pp->launches.push_back(pl.rec);
    }
    return HCCL_SUCCESS;
}

void KernelArgs(LaunchRec &l, void **args)
{
    args[0] = &l.table;
    args[1] = &l.nitems;
    if (l.fusedArgs) {
        args[2] = &l.ntiles;
        args[3] = &l.srcPool;
        args[4] = &l.dstPool;
        args[5] = &l.tilesPerItem;
        args[6] = &l.teamCtr;      // read by the team kernels only
    } else {
        args[2] = &l.nwhole;
        args[3] = &l.ntiles;
        args[4] = &l.flags;
    }
}

HcclResult BuildGraph(Prepared *pp)
{
    HIP_OK(hipGraphCreate(&pp->graph, 0));
    hipGraphNode_t prev = nullptr;
    for (LaunchRec &l : pp->launches) {
        void *args[7];
        KernelArgs(l, args);
        hipKernelNodeParams kp = {};
        kp.func = const_cast<void *>(l.func);
        kp.gridDim = dim3(l.grid, 1, 1);
        kp.blockDim = dim3(kBlockThreads, 1, 1);
        kp.sharedMemBytes = l.dynamicLds;
        kp.kernelParams = args;
        kp.extra = nullptr;
        hipGraphNode_t node = nullptr;
        HIP_OK(hipGraphAddKernelNode(&node, pp->graph, prev ? &prev : nullptr, prev ? 1 : 0, &kp));
        prev = node;
    }
    HIP_OK(hipGraphInstantiate(&pp->exec, pp->graph, nullptr, nullptr, 0));
    return HCCL_SUCCESS;
}

bool RangesOverlap(const char *a, uint64_t al, const char *b, uint64_t bl)
{
    return al && bl && a < b + bl && b < a + al;
}

std::string CacheKey(const Group *g, int algo)
{
    // raw bytes of everything the prepared tables depend on
    std::string key;
    auto put = [&](const void *p, size_t n) { key.append(static_cast<const char *>(p), n); };
    if (g->ctx->sig.variable) {
        put(g->ctx->vCounts.data(), g->ctx->vCounts.size() * 8);
        put(g->ctx->vDispls.data(), g->ctx->vDispls.size() * 8);
        key.push_back('v');
    }
    uint64_t head[11] = {uint64_t(g->cfg.nicMask), uint64_t(g->ctx->sig.coll), uint64_t(algo), uint64_t(g->ctx->sig.dtype), uint64_t(g->ctx->sig.op), g->ctx->sig.count,
        uint64_t(g->cfg.fuse) | (uint64_t(g->cfg.graph) << 1) | (uint64_t(g->ctx->sig.root) << 8) | (uint64_t(g->ctx->sig.peer) << 20), g->cfg.cclBytes, g->cfg.align,
        uint64_t(g->cfg.blocksPerCu) | (uint64_t(uint32_t(g->cfg.stepStores + 1)) << 32) | (uint64_t(g->cfg.servers) << 40) |
            (uint64_t(uint32_t(g->cfg.algo + 1) & 0xfu) << 48) | (uint64_t(g->cfg.deterministic) << 56) | (uint64_t(g->cfg.level0Rings) << 57) |
            (uint64_t(uint32_t(g->cfg.fusedStores + 1)) << 60) | (uint64_t(g->cfg.stepSweep) << 62), g->p};
    put(head, sizeof(head));
    put(&g->cfg.launchCapMiB, sizeof(g->cfg.launchCapMiB));
    put(&g->cfg.team, sizeof(g->cfg.team));
    put(&g->cfg.teamTiles, sizeof(g->cfg.teamTiles));
    put(g->ctx->send.data(), g->ctx->send.size() * sizeof(void *));
    put(g->ctx->recv.data(), g->ctx->recv.size() * sizeof(void *));
    if (g->ctx->sig.coll == COLL_ALLTOALLV) {
        put(g->ctx->sendCounts.data(), g->ctx->sendCounts.size() * 8);
        put(g->ctx->sdispls.data(), g->ctx->sdispls.size() * 8);
        put(g->ctx->recvCounts.data(), g->ctx->recvCounts.size() * 8);
        put(g->ctx->rdispls.data(), g->ctx->rdispls.size() * 8);
    }
    return key;
}

// Planning costs about a millisecond for 8 ranks and tens of milliseconds for 32; a plan depends on
// the request only (sizes, schedule, which ranks run in place), not on addresses, so a caller that
// comes back with other buffers gets the plan from here and pays for the pointer tables only.
int CachedPlan(Group *g, const PlanRequest &rq, std::shared_ptr<const Plan> *out, std::string *err)
{
    if (rq.coll == COLL_ALLTOALLV) {
        // Its plan depends on four p x p tables, which callers like an expert-parallel layer change on every call:
        // a key over the tables and a kept copy of the plan (megabytes at 64 ranks) would cost more than planning,
        // which for this collective is a direct pass over the tables.  A call that does repeat finds the prepared
        // collective in the group's cache before it gets here.
        std::shared_ptr<Plan> fresh = std::make_shared<Plan>();
        int rc = BuildPlan(rq, fresh.get(), err);
        if (rc == 0) {
            *out = fresh;
        }
        return rc;
    }
    std::string key;
    auto put = [&](const void *p, size_t n) { key.append(static_cast<const char *>(p), n); };
    auto putVec = [&](const std::vector<uint64_t> &v) {
        uint64_t n = v.size();
        put(&n, sizeof(n));
        put(v.data(), v.size() * sizeof(uint64_t));
    };
    uint64_t head[11] = {uint64_t(rq.nicMask), uint64_t(rq.coll), uint64_t(rq.algo), rq.p, rq.count, rq.root, rq.peer, rq.unit, rq.cclBytes, rq.align,
        uint64_t(rq.meshAtomic) | (uint64_t(rq.stageInput) << 1) | (uint64_t(rq.servers) << 8) | (uint64_t(rq.level0Rings) << 40)};
    put(head, sizeof(head));
    put(rq.alias.data(), rq.alias.size());
    putVec(rq.sendCounts);
    putVec(rq.sdispls);
    putVec(rq.recvCounts);
    putVec(rq.rdispls);
    putVec(rq.vCounts);
    putVec(rq.vDispls);
    auto it = g->planCache.find(key);
    if (it != g->planCache.end()) {
        *out = it->second;
        return 0;
    }
    if (g->planCache.size() >= 128) {
        g->planCache.clear();   // plans in use stay alive through the prepared collectives that hold them
    }
    // A new count (or, for the variable-count reduce-scatter, a new table of blocks) of a request seen before: its plan
    // is derived from a template of that request where the planner knows how.  Templates are kept per request without
    // its count and tables, a few each.
    std::string shape;
    {
        uint64_t head0[11];
        std::memcpy(head0, head, sizeof(head));
        head0[4] = 0;   // count
        shape.append(reinterpret_cast<const char *>(head0), sizeof(head0));
        shape.append(reinterpret_cast<const char *>(rq.alias.data()), rq.alias.size());
        shape.push_back(rq.vCounts.empty() ? 'c' : 'v');
    }
    std::vector<TemplateSlot> &templates = g->planTemplates[shape];
    std::shared_ptr<Plan> fresh = std::make_shared<Plan>();
    for (TemplateSlot &t : templates) {
        if (PlanFromTemplate(rq, *t.tmpl, fresh.get())) {
            t.hits++;
            g->planCache[key] = fresh;
            *out = fresh;
            return 0;
        }
    }
    std::shared_ptr<PlanTemplate> made = std::make_shared<PlanTemplate>();
    int rc = BuildPlanTemplate(rq, made.get(), fresh.get(), err);
    if (rc != 0) {
        if (templates.empty()) {
            g->planTemplates.erase(shape);
        }
        return rc;
    }
    if (made->count != 0 || made->blockTable) {
        if (g->planTemplates.size() > 64) {
            g->planTemplates.clear();            // (invalidates `templates`)
            g->planTemplates[shape].push_back(TemplateSlot{made, 0});
        } else if (templates.size() < 4) {
            templates.push_back(TemplateSlot{made, 0});
        } else {
            // the one that served least goes (a count with a ragged last slice serves no other count)
            size_t worst = 0;
            for (size_t i = 1; i < templates.size(); i++) {
                worst = templates[i].hits < templates[worst].hits ? i : worst;
            }
            templates[worst] = TemplateSlot{made, 0};
        }
    }
    g->planCache[key] = fresh;
    *out = fresh;
    return 0;
}

// Schedule between the servers of a two-level collective: the one asked for, else the reference's default
// (AlgConfigurator::GetDefaultAlgoLevel1V1, ALG/impl/alg_configurator.cc:226-241): halving-doubling for 8 servers
// and more and for powers of two, ring otherwise.
Algo Level1Algo(const Group *g)
{
    if (g->cfg.algo == ALGO_RING || g->cfg.algo == ALGO_RHD) {
        return Algo(g->cfg.algo);
    }
    const uint32_t n = g->cfg.servers;
    return (n >= 8 || (n > 1 && (n & (n - 1)) == 0)) ? ALGO_RHD : ALGO_RING;
}

HcclResult Prepare(Group *g, int algo, std::unique_ptr<Prepared> *out, bool noAlloc, hipStream_t stream)
{
    std::unique_ptr<Prepared> pp(new Prepared());
    const bool reduceColl = g->ctx->sig.coll == COLL_ALLREDUCE || g->ctx->sig.coll == COLL_REDUCESCATTER || g->ctx->sig.coll == COLL_REDUCE;
    PlanRequest rq;
    rq.coll = CollKind(g->ctx->sig.coll);
    rq.algo = Algo(algo);
    rq.p = g->p;
    rq.count = g->ctx->sig.count;
    rq.root = g->ctx->sig.root;
    rq.peer = g->ctx->sig.peer;
    rq.unit = DtypeSize(g->ctx->sig.dtype);
    rq.cclBytes = g->cfg.cclBytes;
    rq.align = g->cfg.align;
    rq.alias.assign(g->p, 0);
    // only an all-reduce and a broadcast run in place as they are; any other collective whose send buffer is its
    // receive buffer is staged below
    const bool inPlaceKind = rq.coll == COLL_ALLREDUCE || rq.coll == COLL_BROADCAST;
    for (uint32_t r = 0; r < g->p; r++) {
        rq.alias[r] = (inPlaceKind && g->ctx->send[r] == g->ctx->recv[r]) ? 1 : 0;
    }
    const bool fourRings = g->cfg.level0Rings == 4 && g->cfg.servers >= 1 && g->p % g->cfg.servers == 0 && g->p / g->cfg.servers == 8;
    if (rq.coll == COLL_ALLREDUCE && ((g->cfg.servers > 1 && g->p % g->cfg.servers == 0) || fourRings)) {
        // two levels: mesh inside a group of ranks (uncut under the same conditions as the one-level
        // mesh, coll_all_reduce_mesh_executor.cc:108-112) or ring(s) when the group is set up as a ring
        // topology (coll_all_reduce_ring_executor.cc:95-135); ring or halving-doubling between the groups
        rq.servers = g->cfg.servers;
        rq.algo = Level1Algo(g);   // ring or halving-doubling (:185-191)
        rq.level0Rings = g->cfg.level0Rings == 4 ? (fourRings ? 4u : 1u) : g->cfg.level0Rings;
        rq.meshAtomic = rq.level0Rings == 0 && !g->cfg.deterministic && g->ctx->sig.dtype != HCCL_DATA_TYPE_INT64 &&
            g->ctx->sig.op != HCCL_REDUCE_PROD;
    }
    if (rq.coll == COLL_ALLREDUCE && rq.servers <= 1 && rq.level0Rings == 0 && rq.algo == ALGO_RING && g->p == 8) {
        // an 8-rank ring some of whose ranks have no network port: the port-pruned reduce-scatter
        // (reduce_scatter_ring.cc:160-168)
        rq.nicMask = g->cfg.nicMask;
    }
    if (rq.coll == COLL_REDUCESCATTER && !g->ctx->sig.variable && g->cfg.servers > 1 && g->p % g->cfg.servers == 0) {
        // two levels (coll_reduce_scatter_mesh_executor.cc:128-247, coll_reduce_scatter_ring_executor.cc:132-340):
        // ring or halving-doubling between the groups first, then inside a group the mesh (uncut under the
        // conditions of :216-218) or the ring(s)
        rq.servers = g->cfg.servers;
        rq.algo = Level1Algo(g);
        rq.level0Rings = g->cfg.level0Rings == 4 ? (g->p / g->cfg.servers == 8 ? 4u : 1u) : g->cfg.level0Rings;
        rq.meshAtomic = rq.level0Rings == 0 && !g->cfg.deterministic && g->ctx->sig.dtype != HCCL_DATA_TYPE_INT64 &&
            g->ctx->sig.op != HCCL_REDUCE_PROD;
        if (rq.level0Rings == 4 && rq.algo == ALGO_RING) {
            // servers of 8 devices some of which have no network port (:150-170, 264-300); the branch only holds
            // together with the ring between the servers, so the halving-doubling schedule ignores the ports
            rq.nicMask = g->cfg.nicMask;
        }
    }
    if (rq.coll == COLL_ALLGATHER && !g->ctx->sig.variable && g->cfg.servers > 1 && g->p % g->cfg.servers == 0) {
        // two levels (coll_all_gather_mesh_executor.cc:71-175, coll_all_gather_ring_executor.cc:81-200): inside a
        // group first, mesh or ring(s), then ring or halving-doubling between the groups
        rq.servers = g->cfg.servers;
        rq.algo = Level1Algo(g);
        rq.level0Rings = g->cfg.level0Rings == 4 ? (g->p / g->cfg.servers == 8 ? 4u : 1u) : g->cfg.level0Rings;
    }
    if (rq.coll == COLL_BROADCAST && g->cfg.level0Rings > 0 && g->p % g->cfg.servers == 0 && g->cfg.algo != ALGO_RING &&
        g->cfg.algo != ALGO_STAR && g->cfg.algo != ALGO_HD_BLOCKS &&
        (g->cfg.servers > 1 || (g->cfg.level0Rings == 4 && g->p == 8))) {
        // the ring topologies' broadcast (coll_broadcast_ring_executor.cc:64-211): ring scatter in the root's group over
        // one ring or the four rings of a group of 8, halving-doubling between the groups, ring all-gather in every
        // group; also for a single group of 8 with its four rings
        rq.servers = g->cfg.servers;
        rq.level0Rings = g->cfg.level0Rings == 4 ? (g->p / g->cfg.servers == 8 ? 4u : 1u) : g->cfg.level0Rings;
    }
    if (rq.coll == COLL_BROADCAST && g->cfg.servers > 1 && g->p % g->cfg.servers == 0 && g->cfg.algo != ALGO_RING &&
        g->cfg.algo != ALGO_STAR && g->cfg.algo != ALGO_HD_BLOCKS && g->cfg.level0Rings == 0) {
        // two levels (coll_broadcast_mesh_executor.cc:59-213): scatter in the root's group, halving-doubling between
        // the groups, mesh all-gather in every group; the flat ring when the ring is asked for by name
        rq.servers = g->cfg.servers;
    }
    if (rq.coll == COLL_SCATTER && g->cfg.servers > 1 && g->p % g->cfg.servers == 0 && rq.algo != ALGO_RING) {
        // two levels (coll_scatter_mesh_executor.cc:40-110): ring scatter of the groups' runs between the sub-roots,
        // mesh scatter inside every group, or the ring scatter when the groups are set up as rings
        // (coll_scatter_ring_executor.cc:42-113); the flat ring when the ring is asked for by name
        rq.servers = g->cfg.servers;
        rq.level0Rings = g->cfg.level0Rings == 4 ? (g->p / g->cfg.servers == 8 ? 4u : 1u) : g->cfg.level0Rings;
    }
    if (rq.coll == COLL_REDUCE && g->cfg.servers > 1 && g->p % g->cfg.servers == 0) {
        // two levels (coll_reduce_mesh_executor.cc:75-194, coll_reduce_ring_plus_hd_executor.cc:75-168): inside the
        // groups the mesh (uncut under the conditions of :93-97) or the ring(s), then ring or halving-doubling
        // towards the root's group (:133-139)
        rq.servers = g->cfg.servers;
        rq.algo = Level1Algo(g);
        rq.level0Rings = g->cfg.level0Rings == 4 ? (g->p / g->cfg.servers == 8 ? 4u : 1u) : g->cfg.level0Rings;
        rq.meshAtomic = rq.level0Rings == 0 && !g->cfg.deterministic && g->ctx->sig.dtype != HCCL_DATA_TYPE_INT64 &&
            g->ctx->sig.op != HCCL_REDUCE_PROD;
    }
    if (g->ctx->sig.variable) {
        rq.vCounts = g->ctx->vCounts;
        rq.vDispls = g->ctx->vDispls;
    }
    if (rq.coll == COLL_ALLTOALLV) {
        // Several servers: the staged schedule, unless the flat pairwise one is asked for by name
        // (alltoall_operator.cc:225-250).
        if (g->cfg.servers > 1 && g->p % g->cfg.servers == 0 && g->cfg.algo != ALGO_PAIRWISE) {
            rq.servers = g->cfg.servers;
        }
        rq.sendCounts = g->ctx->sendCounts;
        rq.sdispls = g->ctx->sdispls;
        rq.recvCounts = g->ctx->recvCounts;
        rq.rdispls = g->ctx->rdispls;
    }
    std::string err;
    int rc = CachedPlan(g, rq, &pp->plan, &err);
    if (rc != 0) {
        HCCL_LOG_ERROR("%s: planning failed: %s", CollName(g->ctx->sig.coll), err.c_str());
        return rc == 1 ? HCCL_E_PARA : HCCL_E_INTERNAL;
    }
    // Buffers of different ranks must not overlap where one of them is written; a send buffer that
    // overlaps a receive buffer other than as an exact in-place pair is staged through scratch.
    bool needStage = false;
    for (uint32_t i = 0; i < g->p; i++) {
        const char *ri = static_cast<const char *>(g->ctx->recv[i]);
        for (uint32_t j = 0; j < g->p; j++) {
            const char *rj = static_cast<const char *>(g->ctx->recv[j]);
            const char *sj = static_cast<const char *>(g->ctx->send[j]);
            if (i != j && RangesOverlap(ri, pp->plan->recvBytes[i], rj, pp->plan->recvBytes[j])) {
                HCCL_LOG_ERROR("%s: receive buffers of rank %u and rank %u overlap", CollName(g->ctx->sig.coll), i, j);
                return HCCL_E_PARA;
            }
            if (RangesOverlap(ri, pp->plan->recvBytes[i], sj, pp->plan->sendBytes[j])) {
                bool exact = (i == j) && ri == sj && (g->ctx->sig.coll == COLL_ALLREDUCE || g->ctx->sig.coll == COLL_BROADCAST);
                needStage = needStage || !exact;
            }
        }
    }
    if (needStage) {
        rq.stageInput = true;
        rq.alias.assign(g->p, 0);
        rc = CachedPlan(g, rq, &pp->plan, &err);
        if (rc != 0) {
            HCCL_LOG_ERROR("%s: planning (staged) failed: %s", CollName(g->ctx->sig.coll), err.c_str());
            return HCCL_E_INTERNAL;
        }
    }
    pp->fused = g->cfg.fuse && pp->plan->fusedOk && !needStage;
    if (pp->fused) {
        for (const FusedItem &it : pp->plan->fused) {
            if (it.src.size() > 64 || (it.kind == FK_TREE && it.nleaf > 32)) {
                pp->fused = false;   // beyond what the fused kernels encode
            }
        }
    }
    if (!pp->fused && pp->plan->scratchBytes > 0) {
        if (noAlloc) {
            const size_t share = (kNoAllocDataBytes / g->p) & ~size_t(255);
            if (pp->plan->scratchBytes > share) {
                HCCL_LOG_ERROR("%s without allocation: the step-by-step schedule keeps %llu bytes of partial results per rank, "
                    "the fixed workspace has %zu per rank for %u ranks", CollName(g->ctx->sig.coll),
                    (unsigned long long)pp->plan->scratchBytes, share, g->p);
                return HCCL_E_PARA;
            }
        } else {
            HcclResult r = EnsureScratch(g, pp->plan->scratchBytes);
            if (r != HCCL_SUCCESS) {
                return r;
            }
        }
    }
    pp->scratchGen = g->scratchGen;
    HcclResult r = BuildTables(g, pp.get(), reduceColl, g->ctx->sig.dtype, g->ctx->sig.op, noAlloc, stream);
    if (r != HCCL_SUCCESS) {
        return r;
    }
    // The graph of a plan with several launches is built when the collective comes back a second time
    // (IssueCollective): a caller that brings fresh buffers every time pays for tables, not for a graph.
    OpInfo &info = pp->info;
    info.coll = g->ctx->sig.coll;
    info.algo = algo;
    info.fused = pp->fused ? 1 : 0;
    info.graph = 0;
    info.launches = uint32_t(pp->launches.size());
    info.teamLaunches = 0;
    for (const LaunchRec &l : pp->launches) {
        info.teamLaunches += l.team ? 1u : 0u;
    }
    info.bytesRead = pp->fused ? pp->plan->fusedRead : pp->plan->stepRead;
    info.bytesWritten = pp->fused ? pp->plan->fusedWritten : pp->plan->stepWritten;
    info.stepRead = pp->plan->stepRead;
    info.stepWritten = pp->plan->stepWritten;
    info.scratchBytes = pp->fused ? 0 : pp->plan->scratchBytes;
    *out = std::move(pp);
    return HCCL_SUCCESS;
}

}  // namespace

Prepared::~Prepared()
{
    if (uploaded) {
        (void)hipEventDestroy(uploaded);
    }
    if (exec) {
        (void)hipGraphExecDestroy(exec);
    }
    if (graph) {
        (void)hipGraphDestroy(graph);
    }
}

Group::~Group()
{
    if (deviceReady) {
        (void)hipDeviceSynchronize();
    }
    cache.clear();
    pinnedStale.clear();
    stale.clear();
    for (void *s : idleScratch) {
        (void)hipFree(s);
    }
    if (copyStream) {
        (void)hipStreamDestroy(copyStream);
    }
    for (StageSlot &slot : stageSlots) {
        if (slot.done) {
            (void)hipEventDestroy(slot.done);
        }
        if (slot.host) {
            (void)hipHostFree(slot.host);
        }
    }
    if (arena.freeFn != nullptr) {
        arena.FreeAll();
    }
    for (void *s : retiredScratch) {
        (void)hipFree(s);
    }
    for (hipEvent_t e : arriveEvents) {
        if (e) {
            (void)hipEventDestroy(e);
        }
    }
    for (hipEvent_t e : doneEvents) {
        if (e) {
            (void)hipEventDestroy(e);
        }
    }
    if (p2pDoneEvent) {
        (void)hipEventDestroy(p2pDoneEvent);
    }
    for (void *s : scratch) {
        if (s) {
            (void)hipFree(s);
        }
    }
    if (barrierMem) {
        (void)hipFree(barrierMem);
    }
}

const char *CollName(int coll)
{
    switch (coll) {
        case COLL_ALLREDUCE: return "AllReduce";
        case COLL_REDUCESCATTER: return "ReduceScatter";
        case COLL_ALLGATHER: return "AllGather";
        case COLL_ALLTOALLV: return "AlltoAllV";
        case COLL_BROADCAST: return "Broadcast";
        case COLL_REDUCE: return "Reduce";
        case COLL_SCATTER: return "Scatter";
        case COLL_SENDRECV: return "Send/Recv";
        default: return "?";
    }
}

int DefaultAlgo(int coll) { return coll == COLL_ALLTOALLV ? ALGO_PAIRWISE : ALGO_RING; }

HcclResult IssueCollective(Group *g, uint32_t launcher)
{
    HcclResult r = EnsureDevice(g, false);
    if (r != HCCL_SUCCESS) {
        return r;
    }
    int algo = g->cfg.algo >= 0 ? g->cfg.algo : DefaultAlgo(g->ctx->sig.coll);
    if (g->ctx->sig.coll == COLL_ALLTOALLV) {
        algo = ALGO_PAIRWISE;
    } else if (g->ctx->sig.coll == COLL_REDUCE) {
        algo = (algo == ALGO_MESH || algo == ALGO_RHD) ? algo : ALGO_RING;   // ring, mesh or halving-doubling reduce
    } else if (g->ctx->sig.coll == COLL_BROADCAST) {
        algo = (algo == ALGO_MESH || algo == ALGO_RHD || algo == ALGO_STAR || algo == ALGO_HD_BLOCKS) ? algo : ALGO_RING;   // ring, mesh, halving-doubling (either kind) or star
    } else if (g->ctx->sig.coll == COLL_SCATTER) {
        algo = (g->cfg.algo == ALGO_RING) ? ALGO_RING : ALGO_MESH;   // mesh scatter unless the ring is asked for
    } else if (g->ctx->sig.coll >= COLL_SCATTER) {
        algo = ALGO_RING;   // direct send / receive
    } else if (algo == ALGO_PAIRWISE || algo == ALGO_STAR || algo == ALGO_HD_BLOCKS) {
        algo = ALGO_RING;
    }
    // coll_all_reduce_mesh_executor.cc:108-112, coll_reduce_scatter_mesh_executor.cc:227-229,
    // coll_reduce_mesh_executor.cc:93-97: without the
    // deterministic setting the mesh reduce phases run uncut, except for int64 and for products
    if (algo == ALGO_MESH && !g->cfg.deterministic && g->ctx->sig.dtype != HCCL_DATA_TYPE_INT64 &&
        g->ctx->sig.op != HCCL_REDUCE_PROD &&
        (g->ctx->sig.coll == COLL_ALLREDUCE || g->ctx->sig.coll == COLL_REDUCESCATTER || g->ctx->sig.coll == COLL_REDUCE)) {
        algo = ALGO_MESH_ATOMIC;
    }
    Prepared *pp = nullptr;
    std::unique_ptr<Prepared> uncached;   // the collective of a call that allocates nothing: built, launched, dropped
    bool hit = false;
    if (g->ctx->sig.noAlloc) {
        // Tables and partial results live in the fixed workspace, which the next such call overwrites:
        // nothing is kept, and the table upload is queued on the launcher's stream ahead of the kernels.
        if (g->noAllocBase == nullptr) {
            HCCL_LOG_ERROR("%s without allocation: the fixed workspace was not set up", CollName(g->ctx->sig.coll));
            return HCCL_E_INTERNAL;
        }
        // an earlier call's work may still be reading the workspace from another stream
        HIP_OK(NoAllocBegin(g->device, g->ctx->streams[launcher]));
        r = Prepare(g, algo, &uncached, true, g->ctx->streams[launcher]);
        if (r != HCCL_SUCCESS) {
            return r;
        }
        pp = uncached.get();
    }
    std::string key = pp ? std::string() : CacheKey(g, algo);
    auto it = pp ? g->cache.end() : g->cache.find(key);
    if (pp != nullptr) {
        // issued below
    } else if (it != g->cache.end() && (it->second->scratchGen == g->scratchGen || it->second->info.scratchBytes == 0)) {
        // (an entry that points into scratch buffers the group has since outgrown is stale)
        pp = it->second.get();
        hit = true;
    } else {
        // A caller may be recording this stream into a graph of its own and come with a collective for the first
        // time.  Preparing it allocates device memory and copies its tables, which must happen now and not as part
        // of that graph: the thread's capture mode is relaxed for the duration (a capture in the default mode
        // refuses such calls), and the tables go over a stream of the library's own (Prepare without a stream).
        hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
        HIP_OK(hipStreamIsCapturing(g->ctx->streams[launcher], &capture));
        const bool underCapture = capture != hipStreamCaptureStatusNone;
        if (it != g->cache.end()) {
            // stale entry (the scratch buffers moved); earlier launches may still be running out of its tables and
            // a caller's graph may replay it out of the retired buffers, so it is set aside
            (it->second->pinned ? g->pinnedStale : g->stale).push_back(std::move(it->second));
            g->cache.erase(it);
        }
        if (g->cache.size() >= g->cfg.cacheEntries && !underCapture) {
            // Full: wait once for whatever is still in flight and start over.  Dropping one entry at a
            // time would put a device-wide wait on every call of a caller with more buffers than entries
            // (measured with 200 buffer sets against 64 entries: 42 us per small all-reduce instead of 7.5).
            // Collectives recorded into a caller's graph stay, tables and all (the arena keeps their chunks).
            // (Under capture the device may not be waited for: the cache runs over until the next call outside.)
            HIP_OK(hipDeviceSynchronize());
            for (auto e = g->cache.begin(); e != g->cache.end();) {
                e = e->second->pinned ? std::next(e) : g->cache.erase(e);
            }
            ReleaseIdle(g);
            g->arena.Reset();
        }
        std::unique_ptr<Prepared> fresh;
        hipStreamCaptureMode mode = hipStreamCaptureModeRelaxed;
        if (underCapture) {
            HIP_OK(hipThreadExchangeStreamCaptureMode(&mode));
        }
        r = Prepare(g, algo, &fresh, false, underCapture ? nullptr : g->ctx->streams[launcher]);
        if (underCapture) {
            hipError_t back = hipThreadExchangeStreamCaptureMode(&mode);
            if (r == HCCL_SUCCESS) {
                HIP_OK(back);
            }
        }
        if (r != HCCL_SUCCESS) {
            return r;
        }
        pp = fresh.get();
        g->cache[key] = std::move(fresh);
    }
    hipStream_t ls = g->ctx->streams[launcher];
    // A caller may be capturing this stream into a graph of its own.  A graph launched into a
    // capturing stream is not recorded there (the caller's graph came out empty and replays did
    // nothing), so the kernels are then launched one by one and become nodes of the caller's graph.
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    HIP_OK(hipStreamIsCapturing(ls, &capture));
    const bool capturing = capture != hipStreamCaptureStatusNone;
    if (!pp->uploadComplete) {
        // The tables were written by launches on the stream of the call that prepared them, and nothing says yet
        // that those have run.  Outside a capture: ask, and order this stream behind them if need be.  Under
        // capture events of work outside the capture may not be touched and the caller's graph may be replayed
        // on any stream later, so the same upload launches are recorded in front of the collective's kernels:
        // every replay rewrites the same bytes.
        if (capturing) {
            HIP_OK(UploadThroughKernelArgs(pp->devTables, pp->hostTables.data(), pp->hostTables.size(), ls));
        } else if (hipEventQuery(pp->uploaded) == hipSuccess) {
            pp->uploadComplete = true;
            std::vector<uint8_t>().swap(pp->hostTables);
        } else {
            (void)hipGetLastError();
            if (ls != pp->uploadStream) {
                HIP_OK(hipStreamWaitEvent(ls, pp->uploaded, 0));
            }
        }
    }
    if (capturing && !pp->pinned && !g->ctx->sig.noAlloc) {
        // The caller's graph keeps pointers to this collective's tables and, step by step, to the group's
        // scratch buffers: from now on neither is freed or handed out again while the group lives.
        pp->pinned = true;
        g->arena.Pin(pp->tableChunk);
        if (pp->info.scratchBytes > 0) {
            g->pinnedScratchUsers++;
        }
    }
    // A graph launch costs about 33 us of host time plus 2 us per node, a direct launch 3.3 us (measured: 2 launches
    // 38 us through a graph against 16 us, 14 launches 39 against 43, 64 launches 159 against 230): a graph pays
    // from a dozen launches on.
    if (!capturing && !g->ctx->sig.noAlloc && g->cfg.graph && pp->launches.size() >= kGraphMinLaunches && pp->exec == nullptr &&
        pp->uses >= 1) {
        // second use of the same collective on the same buffers: from now on it is replayed from a graph
        r = BuildGraph(pp);
        if (r != HCCL_SUCCESS) {
            return r;
        }
    }
    pp->uses++;
    const bool viaGraph = pp->exec != nullptr && !capturing;
    g->lastInfo = pp->info;
    g->lastInfo.cacheHit = hit ? 1 : 0;
    g->lastInfo.graph = viaGraph ? 1 : 0;

    // Order the launch after everything queued so far on the other ranks' streams, and order those
    // streams after the collective.  Ranks that share the launcher's stream need nothing.
    bool others = false;
    for (uint32_t k = 0; k < g->p; k++) {
        if (k == launcher || g->ctx->streams[k] == ls) {
            continue;
        }
        if (k < g->ctx->recorded.size() && g->ctx->recorded[k]) {
            // the rank put its own marker on its stream when it arrived (it is blocked in its call)
            HIP_OK(hipStreamWaitEvent(ls, g->arriveEvents[k], 0));
            others = true;
            continue;
        }
        bool seen = false;
        for (uint32_t q = 0; q < k; q++) {
            seen = seen || (q != launcher && g->ctx->streams[q] == g->ctx->streams[k] &&
                !(q < g->ctx->recorded.size() && g->ctx->recorded[q]));
        }
        if (!seen) {
            HIP_OK(hipEventRecord(g->arriveEvents[k], g->ctx->streams[k]));
            HIP_OK(hipStreamWaitEvent(ls, g->arriveEvents[k], 0));
        }
        others = true;
    }
    if (viaGraph) {
        HIP_OK(hipGraphLaunch(pp->exec, ls));
    } else {
        for (LaunchRec &l : pp->launches) {
            void *args[7];
            KernelArgs(l, args);
            HIP_OK(hipLaunchKernel(l.func, dim3(l.grid, 1, 1), dim3(kBlockThreads, 1, 1), args, l.dynamicLds, ls));
        }
    }
    if (g->ctx->sig.noAlloc) {
        HIP_OK(NoAllocEnd(g->device, ls));
    }
    // A rank blocked in its call picks up "its" collective's entry and event after it wakes, when later operations may
    // already have been issued: every rendezvous has its own entry and event (by serial number modulo the ring's
    // size), and a matched send / receive, which is not a rendezvous, has an event of its own.
    const bool p2p = g->ctx->sig.coll == COLL_SENDRECV;
    hipEvent_t done = p2p ? g->p2pDoneEvent : g->doneEvents[g->opSerial % 8];
    if (!p2p) {
        g->launchStreams[g->opSerial % 8] = ls;
        g->doneRecorded[g->opSerial % 8] = false;
    }
    if (others) {
        HIP_OK(hipEventRecord(done, ls));
        if (!p2p) {
            g->doneRecorded[g->opSerial % 8] = true;
        }
        // ranks blocked in their calls make their own streams wait when they wake up, each on its own thread
        for (uint32_t k = 0; k < g->p && !g->ctx->ranksWaitThemselves; k++) {
            if (k != launcher && g->ctx->streams[k] != ls) {
                HIP_OK(hipStreamWaitEvent(g->ctx->streams[k], done, 0));
            }
        }
    }
    return HCCL_SUCCESS;
}

}  // namespace hcclamd
