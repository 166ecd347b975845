// Communicator group, rendezvous of the simulated ranks, and task issue.
//
// Stands where the reference has HcclCommunicator::ExecOp / ExecOpAlltoAll
// (FW/communicator/impl/hccl_communicator.cc:3959,4109), the executors' InitTask / LaunchTaskExtend
// bracket (ALG/impl/coll_executor/coll_all_reduce/coll_all_reduce_executor.cc:232-270) and the task
// loader threads (ALG/impl/task/task_loader.cc:102-203): a planned collective becomes a HIP graph of
// kernel nodes, instantiated once per (operation, sizes, buffers) and replayed on later calls.
// (FW = src/domain/collective_communication/framework, ALG = .../algorithm in the reference tree.)
#pragma once
#include <hip/hip_runtime_api.h>

#include <atomic>
#include <condition_variable>
#include <deque>
#include <cstdint>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "arena.h"
#include "hccl/hccl_types.h"
#include "kernels.h"
#include "plan.h"

namespace hcclamd {

constexpr uint32_t kCommMagic = 0x48434c31;   // "HCL1"
constexpr uint32_t kMaxRanks = 64;

struct GroupConfig {
    uint64_t cclBytes = 200ull << 20;     // HCCL_BUFFSIZE / HcclCommConfig.hcclBufferSize (MiB)
    uint64_t align = 128;                 // slice alignment
    int algo = -1;                        // -1 = default per collective, else hcclamd::Algo
    bool fuse = true;                     // run the fused single-pass form when the plan has one
    bool graph = true;                    // issue through a HIP graph
    bool deterministic = false;
    uint32_t servers = 1;            // all-reduce: > 1 = two-level schedule over `servers` groups of consecutive ranks
    uint32_t level0Rings = 0;        // two-level all-reduce inside a group: 0 = mesh, 1 = one ring, 4 = four rings (groups of 8)
    uint32_t nicMask = 0;            // 8-rank ring all-reduce: bit r = rank r has a network port (0: all have one)
    int stepStores = -1;             // step kernel stores: -1 chosen per launch, 0 non-temporal, 1 ordinary
    int fusedStores = -1;            // fused kernels' stores: 0 non-temporal, 1 ordinary, -1 chosen per collective (reductions: non-temporal)
    int stepSweep = 1;               // step kernel: 0 every phase walks its steps forwards, 1 every other phase backwards
    uint32_t cacheEntries = 1024;    // prepared collectives kept (distinct sizes / buffers / settings)
    uint32_t blocksPerCu = 0;             // workgroups per CU; 0 = per-kernel default
    int32_t launchCapMiB = -1;            // fused issue: cut the work into launches that move about this much; 0 = one launch per
                                          // kernel kind, -1 = the library decides per collective
    uint32_t teamTiles = 0;               // team kernels: tiles per workgroup and round, 0 = chosen per launch
    int team = -1;                        // team form of the fused kernels (an XCD's workgroups read together, then write together):
                                          // 1 wherever it can run, 0 never, -1 for large launches whose items touch many streams
    bool blockingArrive = false;          // ranks wait inside the call until the collective is issued
    uint32_t arriveTimeoutMs = 1800 * 1000;
};

// One kernel launch of a prepared collective.
struct LaunchRec {
    const void *func = nullptr;
    uint32_t grid = 0;
    uint32_t dynamicLds = 0;      // bytes of dynamic LDS the launch asks for (team kernels)
    // kernel arguments: step kernels take (table, nitems, nwhole, ntiles, flags), fused kernels
    // (table, nitems, ntiles, srcPool, dstPool, tilesPerItem), their team forms one more: (..., teamCtr)
    const void *table = nullptr;
    uint32_t nitems = 0;
    uint32_t ntiles = 0;
    uint32_t nwhole = 0;
    uint32_t flags = 0;
    const void *srcPool = nullptr;
    const void *dstPool = nullptr;
    uint32_t tilesPerItem = 0;    // fused: every item covers this many tiles (the last at most as many); 0 = they differ
    void *teamCtr = nullptr;      // team kernels: this launch's team block inside the prepared tables (counters, regions, slots)
    uint32_t roundTiles = 0;      // team kernels: tiles per workgroup in a full-size region
    bool fusedArgs = false;
    bool team = false;
};

struct OpInfo {
    int coll = 0, algo = 0, fused = 0, graph = 0, cacheHit = 0;
    uint32_t launches = 0;
    uint32_t teamLaunches = 0;
    uint64_t bytesRead = 0, bytesWritten = 0;     // what the issued kernels move in HBM, all ranks
    uint64_t stepRead = 0, stepWritten = 0;       // the step-by-step schedule's figure
    uint64_t scratchBytes = 0;
};

struct Prepared {
    std::shared_ptr<const Plan> plan;   // shared with the group's plan cache (plans do not depend on addresses)
    bool fused = false;
    void *devTables = nullptr;        // inside the group's table arena
    uint32_t tableChunk = 0;          // the arena chunk they came from
    std::vector<LaunchRec> launches;
    hipGraph_t graph = nullptr;       // built on the second use: a caller that always comes with fresh buffers never pays for it
    hipGraphExec_t exec = nullptr;
    uint64_t scratchGen = 0;
    uint32_t uses = 0;                // times issued
    // Small tables are written by upload launches on the stream of the call that prepared them; until those are
    // known to have finished, a call on another stream orders itself behind them.
    hipEvent_t uploaded = nullptr;
    hipStream_t uploadStream = nullptr;
    bool uploadComplete = true;
    std::vector<uint8_t> hostTables;  // kept until the upload is known to have finished (a capture records it again)
    // Recorded into a caller's HIP graph at least once: that graph's kernel nodes point at the tables (and, for a
    // step-by-step schedule, at the group's scratch buffers), so neither may be freed or reused while the group lives.
    bool pinned = false;
    OpInfo info;
    ~Prepared();
};

struct OpSig {
    int coll = -1;
    uint64_t count = 0;
    int dtype = 0, recvType = 0, op = 0;
    int variable = 0;                // 1: reduce-scatter-v / all-gather-v (block tables instead of a count)
    uint32_t peer = 0;               // send / receive: destination rank (root = source rank)
    uint32_t root = 0;               // broadcast / reduce / scatter
    int noAlloc = 0;                 // 1: issued out of the fixed device workspace, nothing allocated, nothing cached
    bool operator==(const OpSig &o) const
    {
        return coll == o.coll && count == o.count && dtype == o.dtype && recvType == o.recvType && op == o.op &&
            variable == o.variable && root == o.root && peer == o.peer && noAlloc == o.noAlloc;
    }
};

// Everything one collective needs from its callers.
struct OpCtx {
    OpSig sig;
    std::vector<void *> send, recv;
    std::vector<hipStream_t> streams;
    std::vector<uint8_t> recorded;    // per rank: the rank itself put its arrival marker on its stream (it is blocked in its call)
    bool ranksWaitThemselves = false; // the blocked ranks order their streams after the launch when they wake
    std::vector<uint64_t> sendCounts, sdispls, recvCounts, rdispls;   // p x p (all-to-all-v)
    std::vector<uint64_t> vCounts, vDispls;                           // p (reduce-scatter-v / all-gather-v)
};

// A send or receive waiting for its counterpart (matched first-in first-out per (source, destination)).
struct P2PPending {
    bool isSend = false;
    void *buf = nullptr;
    uint64_t count = 0;
    int dtype = 0;
    hipStream_t stream = nullptr;
};

// A plan kept as a template for other counts of the same request, and how often it served as one.
struct TemplateSlot {
    std::shared_ptr<const PlanTemplate> tmpl;
    uint32_t hits = 0;
};

// A pinned host buffer that descriptor tables pass through on their way to the device.
struct StageSlot {
    void *host = nullptr;
    hipEvent_t done = nullptr;      // recorded behind the slot's latest copy
    bool used = false;
};

struct Group;

struct Comm {
    uint32_t magic = kCommMagic;
    Group *group = nullptr;
    uint32_t rank = 0;
    bool inUse = false;
};

struct Group {
    std::mutex m;
    std::condition_variable cv;
    uint32_t p = 0;
    std::vector<std::unique_ptr<Comm>> comms;
    uint32_t liveComms = 0;
    GroupConfig cfg;
    std::string name;
    bool suspended = false;
    HcclResult asyncError = HCCL_SUCCESS;

    // rendezvous of the current collective
    uint32_t arrived = 0;
    uint64_t opSerial = 0;           // bumped whenever a collective is issued or cancelled
    // How the most recent rendezvous ended, by serial number modulo the array size: a rank that blocked in
    // rendezvous n reads entry n even if the other ranks have moved on to n + 1 by the time it wakes.
    HcclResult issueResults[8] = {};
    hipStream_t launchStreams[8] = {};   // same indexing: the stream the collective went to ...
    bool doneRecorded[8] = {};           // ... and whether its done event was recorded after it for the other streams
    std::vector<uint8_t> here;
    OpCtx pend;                      // what the ranks of the current collective passed
    OpCtx *ctx = nullptr;            // the operation being issued (the rendezvous, or a matched send / receive)
    std::map<std::pair<uint32_t, uint32_t>, std::deque<P2PPending>> p2p;

    // device resources
    std::atomic<bool> deviceReady{false};   // set last by EnsureDevice; a rank's early stream marker reads it without the group's lock
    int device = 0;
    uint32_t numCu = 256;
    std::vector<hipEvent_t> arriveEvents;
    hipEvent_t doneEvents[8] = {};        // one per entry of the ring above: recorded behind that collective for the other ranks' streams
    hipEvent_t p2pDoneEvent = nullptr;    // the same for a matched send / receive, which is no rendezvous and has no entry
    std::vector<void *> scratch;
    std::vector<void *> retiredScratch;   // scratch buffers a pinned collective still points at; freed with the group
    uint32_t pinnedScratchUsers = 0;      // pinned collectives that use the current scratch buffers
    std::vector<std::unique_ptr<Prepared>> pinnedStale;   // pinned collectives that left the cache
    std::vector<void *> idleScratch;      // outgrown scratch buffers that work in flight may still use; freed when the device is next known idle
    std::vector<std::unique_ptr<Prepared>> stale;         // collectives that left the cache while work in flight may still use them; same
    hipStream_t copyStream = nullptr;     // the library's own stream for table copies (non-blocking, never captured)
    std::vector<StageSlot> stageSlots;    // ring of pinned buffers for tables too large to ride in kernel arguments
    uint32_t stageNext = 0;
    void *barrierMem = nullptr;       // 2 x p small buffers for HcclBarrier's all-reduce
    void *noAllocBase = nullptr;      // this device's copy of the fixed workspace (noalloc.hip), looked up at set-up
    uint64_t scratchBytes = 0;
    uint64_t scratchGen = 0;
    std::unordered_map<std::string, std::unique_ptr<Prepared>> cache;   // keyed by request, settings and buffer addresses
    TableArena arena;
    std::unordered_map<std::string, std::shared_ptr<const Plan>> planCache;   // keyed by the plan request
    std::unordered_map<std::string, std::vector<TemplateSlot>> planTemplates;   // keyed by the request without its count
    OpInfo lastInfo;

    ~Group();
};

// Creates the group's events on first use of the device.  HCCL_E_RUNTIME when there is no GPU.
HcclResult EnsureDevice(Group *g, bool quiet);

// Called with the group mutex held, by the last rank to arrive.
HcclResult IssueCollective(Group *g, uint32_t launcherRank);

const char *CollName(int coll);
int DefaultAlgo(int coll);

}  // namespace hcclamd
