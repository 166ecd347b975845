// The HCCL C ABI (include/hccl/hccl.h) over the planner and the HIP task issue.
//
// Replaces, for the single-GPU data path, the definitions in the reference's
// src/domain/collective_communication/framework/op_base/src/op_base.cc (cited per function) and the
// argument checks of framework/common/src/param_check.cc.  Check order and return codes follow the
// reference; what differs is stated where it does.
#include <chrono>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <map>
#include <set>
#include <sstream>
#include <string>
#include <vector>

#include "hccl/hccl.h"
#include "hccl/hccl_amd_ext.h"
#include "log.h"
#include "ranktable.h"
#include "runtime.h"

using namespace hcclamd;

namespace {

constexpr uint64_t kSysMaxCount = 0x7FFFFFFFFull;   // largest element count a call may carry

std::mutex g_registryMutex;
std::set<Group *> g_groups;
int g_deterministic = -1;   // -1: not set through HcclSetConfig

#define CHK_PTR(p)                                              \
    do {                                                        \
        if ((p) == nullptr) {                                   \
            HCCL_LOG_ERROR("%s: %s is null", __func__, #p);     \
            return HCCL_E_PTR;                                  \
        }                                                       \
    } while (0)

Comm *AsComm(HcclComm h)
{
    Comm *c = static_cast<Comm *>(h);
    return (c != nullptr && c->magic == kCommMagic && c->group != nullptr) ? c : nullptr;
}

// param_check.cc:22-36,261-269: the supported set; everything else is HCCL_E_NOT_SUPPORT.
bool DataTypeKnown(HcclDataType dt)
{
    return dt >= HCCL_DATA_TYPE_INT8 && dt <= HCCL_DATA_TYPE_INT128;
}

// param_check.cc:375-407: tag, count, data type, stream -- in this order.
HcclResult CheckOpParam(const char *fn, uint64_t count, HcclDataType dt, const void *stream)
{
    if (count > kSysMaxCount) {
        HCCL_LOG_ERROR("%s: count %llu exceeds the maximum %llu", fn, (unsigned long long)count,
            (unsigned long long)kSysMaxCount);
        return HCCL_E_PARA;
    }
    if (!DataTypeKnown(dt)) {
        HCCL_LOG_ERROR("%s: data type %d not supported", fn, int(dt));
        return HCCL_E_NOT_SUPPORT;
    }
    if (stream == nullptr) {
        HCCL_LOG_ERROR("%s: stream is null", fn);
        return HCCL_E_PTR;
    }
    return HCCL_SUCCESS;
}

// param_check.cc:284-294.  The per-SoC restrictions of :296-349 (no int16 / bf16 product on 910B)
// describe Ascend hardware and are not applied here.
HcclResult CheckReduce(const char *fn, HcclDataType dt, HcclReduceOp op)
{
    if (op != HCCL_REDUCE_SUM && op != HCCL_REDUCE_PROD && op != HCCL_REDUCE_MAX && op != HCCL_REDUCE_MIN) {
        HCCL_LOG_ERROR("%s: reduce op %d not supported", fn, int(op));
        return HCCL_E_NOT_SUPPORT;
    }
    if (dt == HCCL_DATA_TYPE_INT128) {
        HCCL_LOG_ERROR("%s: no arithmetic on int128", fn);
        return HCCL_E_NOT_SUPPORT;
    }
    return HCCL_SUCCESS;
}

uint32_t ElemSize(int dt)
{
    static const uint32_t table[] = {1, 2, 4, 2, 4, 8, 8, 1, 2, 4, 8, 2, 16};
    return (dt >= 0 && dt <= 12) ? table[dt] : 0;
}

void ApplyEnv(GroupConfig *cfg)
{
    if (const char *e = std::getenv("HCCL_BUFFSIZE")) {
        long v = std::atol(e);
        if (v >= 1) {
            cfg->cclBytes = uint64_t(v) << 20;
        }
    }
    if (const char *e = std::getenv("HCCL_ALGO")) {
        std::string s(e);
        if (s.find("mesh") != std::string::npos || s.find("fullmesh") != std::string::npos) {
            cfg->algo = ALGO_MESH;
        } else if (s.find("H-D") != std::string::npos || s.find("rhd") != std::string::npos || s.find("HD") != std::string::npos) {
            cfg->algo = ALGO_RHD;
        } else if (s.find("ring") != std::string::npos) {
            cfg->algo = ALGO_RING;
        } else if (s.find("pairwise") != std::string::npos) {
            cfg->algo = ALGO_PAIRWISE;
        }
    }
    if (const char *e = std::getenv("HCCL_DETERMINISTIC")) {
        cfg->deterministic = (std::string(e) == "true" || std::string(e) == "1");
    } else if (g_deterministic >= 0) {
        cfg->deterministic = g_deterministic == 1;
    }
    if (const char *e = std::getenv("HCCL_AMD_FUSE")) {
        cfg->fuse = std::atoi(e) != 0;
    }
    if (const char *e = std::getenv("HCCL_AMD_GRAPH")) {
        cfg->graph = std::atoi(e) != 0;
    }
    if (const char *e = std::getenv("HCCL_AMD_BLOCKS_PER_CU")) {
        int v = std::atoi(e);
        if (v >= 1 && v <= 64) {
            cfg->blocksPerCu = uint32_t(v);
        }
    }
    if (const char *e = std::getenv("HCCL_AMD_TEAM")) {
        const std::string v(e);
        cfg->team = v == "1" ? 1 : (v == "0" ? 0 : -1);
    }
    if (const char *e = std::getenv("HCCL_AMD_BLOCKING_ARRIVE")) {
        cfg->blockingArrive = std::atoi(e) != 0;
    }
    if (const char *e = std::getenv("HCCL_EXEC_TIMEOUT")) {
        long v = std::atol(e);
        if (v > 0) {
            cfg->arriveTimeoutMs = uint32_t(std::min<long>(v, 2000000) * 1000);
        }
    }
    if (const char *e = std::getenv("HCCL_AMD_ARRIVE_TIMEOUT_MS")) {
        long v = std::atol(e);
        if (v > 0) {
            cfg->arriveTimeoutMs = uint32_t(v);
        }
    }
}

// HcclCommConfig loading, as FW/communicator/comm_config.cc:29-178: size-prefixed copy, magic word,
// fields gated by version (>= 1 buffer size and deterministic, >= 2 name).
struct ConfigHeader {
    size_t size;
    uint32_t magicWord;
    uint32_t version;
    uint64_t reserved;
};

HcclResult LoadCommConfig(const HcclCommConfig *user, GroupConfig *cfg, std::string *name)
{
    HcclCommConfig local;
    std::memset(&local, 0, sizeof(local));   // bytes the caller's (older, smaller) struct does not have stay zero
    size_t size = 0;
    std::memcpy(&size, user, sizeof(size));   // the struct is only 4-byte aligned: its leading fields are read by copy
    std::memcpy(&local, user, std::min(size, sizeof(local)));
    ConfigHeader header;
    std::memcpy(&header, &local, sizeof(header));
    const ConfigHeader *h = &header;
    if (h->magicWord != HCCL_COMM_CONFIG_MAGIC_WORD) {
        HCCL_LOG_ERROR("comm config: bad magic word 0x%x; initialise the struct with HcclCommConfigInit()", h->magicWord);
        return HCCL_E_PARA;
    }
    if (h->version >= 1) {
        if (local.hcclBufferSize != HCCL_COMM_BUFFSIZE_CONFIG_NOT_SET) {
            if (local.hcclBufferSize < 1) {
                HCCL_LOG_ERROR("comm config: hcclBufferSize must be at least 1 (MiB)");
                return HCCL_E_PARA;
            }
            cfg->cclBytes = uint64_t(local.hcclBufferSize) << 20;
        }
        if (local.hcclDeterministic != HCCL_COMM_DETERMINISTIC_CONFIG_NOT_SET) {
            if (local.hcclDeterministic > 1) {
                HCCL_LOG_ERROR("comm config: hcclDeterministic must be 0 or 1");
                return HCCL_E_PARA;
            }
            cfg->deterministic = local.hcclDeterministic == 1;
        }
    }
    if (h->version >= 2 && local.hcclCommName[0] != '\0') {
        local.hcclCommName[COMM_NAME_MAX_LENGTH - 1] = '\0';
        *name = local.hcclCommName;
    }
    if (h->version >= 4 && local.hcclOpExpansionMode > 3) {
        HCCL_LOG_WARN("comm config: unknown hcclOpExpansionMode %u, using the default", local.hcclOpExpansionMode);
    }
    return HCCL_SUCCESS;
}

Group *NewGroup(uint32_t nRanks)
{
    Group *g = new Group();
    g->p = nRanks;
    ApplyEnv(&g->cfg);
    g->here.assign(nRanks, 0);
    g->pend.send.assign(nRanks, nullptr);
    g->pend.recv.assign(nRanks, nullptr);
    g->pend.streams.assign(nRanks, nullptr);
    g->pend.recorded.assign(nRanks, 0);
    g->ctx = &g->pend;
    char nm[64];
    std::snprintf(nm, sizeof(nm), "hccl_world_group_%p", static_cast<void *>(g));
    g->name = nm;
    g->comms.resize(nRanks);
    return g;
}

// Groups that are being assembled rank by rank (root-info and sub-communicator creation), by key.
std::map<std::string, Group *> g_forming;
uint64_t g_rootInfoSerial = 0;

// Joins rank `rank` to the group forming under `key` (created on first use).
HcclResult JoinFormingGroup(const std::string &key, uint32_t nRanks, uint32_t rank, const HcclCommConfig *config, HcclComm *out)
{
    std::lock_guard<std::mutex> reg(g_registryMutex);
    Group *g = nullptr;
    auto it = g_forming.find(key);
    if (it == g_forming.end()) {
        if (nRanks > kMaxRanks) {
            HCCL_LOG_ERROR("at most %u ranks per group", kMaxRanks);
            return HCCL_E_PARA;
        }
        g = NewGroup(nRanks);
        g->name = key;
        if (config != nullptr) {
            HcclResult r = LoadCommConfig(config, &g->cfg, &g->name);
            if (r != HCCL_SUCCESS) {
                delete g;
                return r;
            }
        }
        g_forming[key] = g;
        g_groups.insert(g);
    } else {
        g = it->second;
        if (g->p != nRanks) {
            HCCL_LOG_ERROR("rank %u joins with %u ranks, the group was created with %u", rank, nRanks, g->p);
            return HCCL_E_PARA;
        }
    }
    std::lock_guard<std::mutex> lock(g->m);
    if (g->comms[rank]) {
        HCCL_LOG_ERROR("rank %u of this group exists already", rank);
        return HCCL_E_PARA;
    }
    std::unique_ptr<Comm> c(new Comm());
    c->group = g;
    c->rank = rank;
    *out = c.get();
    g->comms[rank] = std::move(c);
    g->liveComms++;
    bool complete = true;
    for (auto &m : g->comms) {
        complete = complete && bool(m);
    }
    if (complete) {
        g_forming.erase(key);
        // Device set-up with the last rank's device current, as HcclCommInitAll does it: no collective call -- in
        // particular not the one that promises to allocate nothing -- is then the first to touch the device.
        // Without a GPU the group exists all the same and its collectives fail with HCCL_E_RUNTIME.
        (void)EnsureDevice(g, true);
    }
    return HCCL_SUCCESS;
}

struct InUse {
    Comm *c;
    explicit InUse(Comm *comm) : c(comm) { c->inUse = true; }
    ~InUse() { c->inUse = false; }
};

// Ends the current rendezvous.  Ranks blocked inside their call wake up and return `result`.
void CancelPending(Group *g, HcclResult result)
{
    g->issueResults[g->opSerial % 8] = result;
    g->arrived = 0;
    std::fill(g->here.begin(), g->here.end(), 0);
    g->opSerial++;
    g->cv.notify_all();
}

// One rank joins the current collective.  The last rank to join issues it.
HcclResult Arrive(Comm *c, const OpSig &sig, void *send, void *recv, hipStream_t stream, const uint64_t *sendCounts,
    const uint64_t *sdispls, const uint64_t *recvCounts, const uint64_t *rdispls, const uint64_t *vCounts = nullptr,
    const uint64_t *vDispls = nullptr)
{
    Group *g = c->group;
    uint32_t r = c->rank;
    // One thread per rank (blocking_arrive): every rank marks its stream before it joins, outside the group's lock, so
    // that the ranks do it side by side (inside the lock the p records of a collective ran one after the other:
    // 12 us of the 63 us a small all-reduce of 8 threaded ranks took).  The two settings read here change only while
    // no collective is under way.  A rank that turns out to be the last to arrive has recorded a marker nobody waits for.
    bool markedEarly = false;
    if (g->cfg.blockingArrive && g->deviceReady && r < g->arriveEvents.size()) {
        if (hipEventRecord(g->arriveEvents[r], stream) == hipSuccess) {
            markedEarly = true;
        } else {
            (void)hipGetLastError();
        }
    }
    std::unique_lock<std::mutex> lock(g->m);
    if (g->suspended) {
        return HCCL_E_SUSPENDING;   // hccl_communicator.cc:2748 (CheckSuspendingStatus)
    }
    if (g->here[r]) {
        HCCL_LOG_ERROR("%s: rank %u called again before the other ranks joined the previous call", CollName(sig.coll), r);
        return HCCL_E_AGAIN;
    }
    bool tablesDiffer = false;
    if (sig.variable && g->arrived > 0 && g->pend.sig.variable) {
        for (uint32_t i = 0; i < g->p; i++) {
            tablesDiffer = tablesDiffer || g->pend.vCounts[i] != vCounts[i] || g->pend.vDispls[i] != vDispls[i];
        }
    }
    if (g->arrived == 0) {
        g->pend.sig = sig;
        if (sig.variable) {
            g->pend.vCounts.assign(vCounts, vCounts + g->p);
            g->pend.vDispls.assign(vDispls, vDispls + g->p);
        }
    } else if (!(g->pend.sig == sig) || tablesDiffer) {
        // every rank must pass the same operation, count, type and op (the reference checks this
        // across processes in RankConsistentcyChecker, hccl_communicator.cc:2803-2805)
        HCCL_LOG_ERROR("%s: rank %u disagrees with the ranks already in the collective (op/count/type)", CollName(sig.coll), r);
        CancelPending(g, HCCL_E_PARA);
        return HCCL_E_PARA;
    }
    g->here[r] = 1;
    g->pend.send[r] = send;
    g->pend.recv[r] = recv;
    g->pend.streams[r] = stream;
    g->pend.recorded[r] = 0;
    // A rank marks its stream when it arrives, so that the rank that issues the collective orders it behind exactly
    // what this stream held at the time of the call: always when the rank is going to wait inside its call (it is on
    // its own thread), otherwise when the ranks are on different streams (ranks that share one stream need no
    // marker, and the common single-stream caller pays nothing).  Not under capture: the marker would become part of
    // the caller's graph for no use.
    if (markedEarly) {
        g->pend.recorded[r] = 1;
    }
    bool mark = !markedEarly && g->deviceReady && g->arrived + 1 < g->p && g->cfg.blockingArrive;
    if (!mark && !markedEarly && g->deviceReady && g->arrived + 1 < g->p && g->arrived > 0) {
        for (uint32_t q = 0; q < g->p && !mark; q++) {
            mark = g->here[q] && q != r && g->pend.streams[q] != stream;
        }
        if (mark) {
            hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
            if (hipStreamIsCapturing(stream, &capture) != hipSuccess || capture != hipStreamCaptureStatusNone) {
                (void)hipGetLastError();
                mark = false;
            }
        }
    }
    if (mark) {
        if (hipEventRecord(g->arriveEvents[r], stream) == hipSuccess) {
            g->pend.recorded[r] = 1;
        } else {
            (void)hipGetLastError();
        }
    }
    if (sig.coll == COLL_ALLTOALLV) {
        size_t p = g->p;
        g->pend.sendCounts.resize(p * p);
        g->pend.sdispls.resize(p * p);
        g->pend.recvCounts.resize(p * p);
        g->pend.rdispls.resize(p * p);
        std::copy(sendCounts, sendCounts + p, g->pend.sendCounts.begin() + r * p);
        std::copy(sdispls, sdispls + p, g->pend.sdispls.begin() + r * p);
        std::copy(recvCounts, recvCounts + p, g->pend.recvCounts.begin() + r * p);
        std::copy(rdispls, rdispls + p, g->pend.rdispls.begin() + r * p);
    }
    g->arrived++;
    if (g->arrived < g->p) {
        if (!g->cfg.blockingArrive) {
            return HCCL_SUCCESS;
        }
        // (Watching the serial number for a while before sleeping was tried: with as many waiting threads as the box has
        // cores it starves the rank that has to issue -- 16 threaded ranks went from 131 us per small all-reduce to 219.)
        uint64_t serial = g->opSerial;
        bool done = g->cv.wait_for(lock, std::chrono::milliseconds(g->cfg.arriveTimeoutMs),
            [&] { return g->opSerial != serial; });
        if (!done) {
            HCCL_LOG_ERROR("%s: rank %u timed out waiting for the other ranks", CollName(sig.coll), r);
            CancelPending(g, HCCL_E_TIMEOUT);
            return HCCL_E_TIMEOUT;
        }
        const HcclResult res = g->issueResults[serial % 8];
        // what follows on this rank's stream comes after the collective
        const bool wait = res == HCCL_SUCCESS && g->doneRecorded[serial % 8] && g->launchStreams[serial % 8] != stream;
        hipEvent_t doneEvent = g->doneEvents[serial % 8];
        lock.unlock();
        if (wait && hipStreamWaitEvent(stream, doneEvent, 0) != hipSuccess) {
            (void)hipGetLastError();
            return HCCL_E_RUNTIME;
        }
        return res;
    }
    // last arrival
    HcclResult res = HCCL_SUCCESS;
    if (sig.coll == COLL_ALLTOALLV) {
        // alltoall_operator.cc:49-72: what i sends to j must be what j expects from i
        for (uint32_t i = 0; i < g->p && res == HCCL_SUCCESS; i++) {
            for (uint32_t j = 0; j < g->p; j++) {
                if (g->pend.sendCounts[size_t(i) * g->p + j] != g->pend.recvCounts[size_t(j) * g->p + i]) {
                    HCCL_LOG_ERROR("AlltoAllV: rank %u sends %llu elements to rank %u, which expects %llu", i,
                        (unsigned long long)g->pend.sendCounts[size_t(i) * g->p + j], j,
                        (unsigned long long)g->pend.recvCounts[size_t(j) * g->p + i]);
                    res = HCCL_E_PARA;
                    break;
                }
            }
        }
    }
    if (res == HCCL_SUCCESS) {
        g->ctx = &g->pend;
        g->pend.ranksWaitThemselves = g->cfg.blockingArrive != 0;   // the other ranks are all blocked in their calls
        res = IssueCollective(g, r);
    }
    if (res != HCCL_SUCCESS && res != HCCL_E_PARA) {
        g->asyncError = res;
    }
    CancelPending(g, res);   // resets the rendezvous and wakes blocked ranks with the result
    return res;
}

// A send meets its receive (or the other way round): the later of the two calls issues the copy on
// its stream, ordered after the earlier caller's stream and before whatever that stream runs next.
HcclResult PointToPoint(Comm *c, bool isSend, void *buf, uint64_t count, HcclDataType dataType, uint32_t other,
    hipStream_t stream)
{
    Group *g = c->group;
    std::unique_lock<std::mutex> lock(g->m);
    if (g->suspended) {
        return HCCL_E_SUSPENDING;
    }
    if (other >= g->p) {
        HCCL_LOG_ERROR("send / receive: rank %u is out of range", other);
        return HCCL_E_PARA;
    }
    uint32_t src = isSend ? c->rank : other, dst = isSend ? other : c->rank;
    auto &queue = g->p2p[std::make_pair(src, dst)];
    if (queue.empty() || queue.front().isSend == isSend) {
        P2PPending pnd;
        pnd.isSend = isSend;
        pnd.buf = buf;
        pnd.count = count;
        pnd.dtype = dataType;
        pnd.stream = stream;
        queue.push_back(pnd);
        return HCCL_SUCCESS;
    }
    P2PPending match = queue.front();
    queue.pop_front();
    if (match.count != count || match.dtype != int(dataType)) {
        HCCL_LOG_ERROR("send / receive between rank %u and rank %u disagree on count or type", src, dst);
        // the call that came first has returned already: its caller learns of the failure through
        // HcclGetCommAsyncError
        g->asyncError = HCCL_E_PARA;
        return HCCL_E_PARA;
    }
    OpCtx ctx;
    ctx.sig.coll = COLL_SENDRECV;
    ctx.sig.count = count;
    ctx.sig.dtype = dataType;
    ctx.sig.recvType = dataType;
    ctx.sig.root = src;
    ctx.sig.peer = dst;
    ctx.send.assign(g->p, nullptr);
    ctx.recv.assign(g->p, nullptr);
    ctx.streams.assign(g->p, stream);
    ctx.send[src] = isSend ? buf : match.buf;
    ctx.recv[dst] = isSend ? match.buf : buf;
    const bool toSelf = other == c->rank;
    if (!toSelf) {
        ctx.streams[other] = match.stream;
    }
    HcclResult res = HCCL_SUCCESS;
    if (toSelf && match.stream != stream) {
        // A rank sending to itself on two streams: the copy runs on this call's stream, after what the earlier
        // call's stream holds so far, and that stream goes on after the copy.
        res = EnsureDevice(g, false);
        if (res == HCCL_SUCCESS && (hipEventRecord(g->arriveEvents[c->rank], match.stream) != hipSuccess ||
            hipStreamWaitEvent(stream, g->arriveEvents[c->rank], 0) != hipSuccess)) {
            (void)hipGetLastError();
            res = HCCL_E_RUNTIME;
        }
    }
    g->ctx = &ctx;
    if (res == HCCL_SUCCESS) {
        res = IssueCollective(g, c->rank);
    }
    g->ctx = &g->pend;
    if (res == HCCL_SUCCESS && toSelf && match.stream != stream) {
        if (hipEventRecord(g->p2pDoneEvent, stream) != hipSuccess || hipStreamWaitEvent(match.stream, g->p2pDoneEvent, 0) != hipSuccess) {
            (void)hipGetLastError();
            res = HCCL_E_RUNTIME;
        }
    }
    if (res != HCCL_SUCCESS && res != HCCL_E_PARA) {
        g->asyncError = res;
    }
    return res;
}

}  // namespace

extern "C" {

// ---- lifecycle ------------------------------------------------------------------------------------

// op_base.cc:244-284.
HcclResult HcclCommInitAll(uint32_t ndev, int32_t *devices, HcclComm *comms)
{
    if (ndev == 0) {
        HCCL_LOG_ERROR("HcclCommInitAll: ndev is 0");
        return HCCL_E_PARA;
    }
    CHK_PTR(comms);
    CHK_PTR(devices);
    std::set<int32_t> distinct(devices, devices + ndev);
    if (distinct.size() != ndev) {
        HCCL_LOG_ERROR("HcclCommInitAll: duplicate device id in the device list");
        return HCCL_E_PARA;
    }
    if (ndev > kMaxRanks) {
        HCCL_LOG_ERROR("HcclCommInitAll: at most %u ranks per group", kMaxRanks);
        return HCCL_E_PARA;
    }
    Group *g = NewGroup(ndev);
    for (uint32_t r = 0; r < ndev; r++) {
        std::unique_ptr<Comm> c(new Comm());
        c->group = g;
        c->rank = r;
        comms[r] = c.get();
        g->comms[r] = std::move(c);
    }
    g->liveComms = ndev;
    // Device set-up (events, the fixed workspace's address, kernel code objects) happens here when a GPU
    // is present, so that no collective call is the first to touch the device; without a GPU the group
    // is still created and its collectives fail with HCCL_E_RUNTIME.
    (void)EnsureDevice(g, true);
    std::lock_guard<std::mutex> reg(g_registryMutex);
    g_groups.insert(g);
    return HCCL_SUCCESS;
}

// op_base.cc:2187-2204: null -> success with a warning; in use -> HCCL_E_AGAIN.
HcclResult HcclCommDestroy(HcclComm comm)
{
    if (comm == nullptr) {
        HCCL_LOG_WARN("HcclCommDestroy: null communicator, nothing to do");
        return HCCL_SUCCESS;
    }
    Comm *c = AsComm(comm);
    if (c == nullptr) {
        return HCCL_E_PARA;
    }
    Group *g = c->group;
    bool last = false;
    {
        std::lock_guard<std::mutex> lock(g->m);
        if (c->inUse) {
            HCCL_LOG_WARN("HcclCommDestroy: communicator is in use, try again later");
            return HCCL_E_AGAIN;
        }
        if (g->here[c->rank]) {
            HCCL_LOG_WARN("HcclCommDestroy: rank %u had joined a collective that was never issued; it is dropped", c->rank);
            CancelPending(g, HCCL_E_PARA);
        }
        for (auto it = g->p2p.begin(); it != g->p2p.end();) {   // unmatched sends / receives of this rank
            it = (it->first.first == c->rank || it->first.second == c->rank) ? g->p2p.erase(it) : std::next(it);
        }
        c->magic = 0;
        c->group = nullptr;
        g->liveComms--;
        last = g->liveComms == 0;
    }
    if (last) {
        {
            std::lock_guard<std::mutex> reg(g_registryMutex);
            g_groups.erase(g);
            for (auto it = g_forming.begin(); it != g_forming.end();) {
                it = (it->second == g) ? g_forming.erase(it) : std::next(it);
            }
        }
        delete g;
    }
    return HCCL_SUCCESS;
}

// op_base.cc:2392-2420.
HcclResult HcclGetRankSize(HcclComm comm, uint32_t *rankSize)
{
    CHK_PTR(comm);
    CHK_PTR(rankSize);
    Comm *c = AsComm(comm);
    if (c == nullptr) {
        return HCCL_E_PARA;
    }
    *rankSize = c->group->p;
    return HCCL_SUCCESS;
}

HcclResult HcclGetRankId(HcclComm comm, uint32_t *rank)
{
    CHK_PTR(comm);
    CHK_PTR(rank);
    Comm *c = AsComm(comm);
    if (c == nullptr) {
        return HCCL_E_PARA;
    }
    *rank = c->rank;
    return HCCL_SUCCESS;
}

// op_base.cc:845-856.
HcclResult HcclGetCommName(HcclComm comm, char *commName)
{
    CHK_PTR(comm);
    CHK_PTR(commName);
    Comm *c = AsComm(comm);
    if (c == nullptr) {
        return HCCL_E_PARA;
    }
    std::strncpy(commName, c->group->name.c_str(), COMM_NAME_MAX_LENGTH - 1);
    commName[COMM_NAME_MAX_LENGTH - 1] = '\0';
    return HCCL_SUCCESS;
}

// op_base.cc:1204-1243: ignored when the environment variable is set; only 0 and 1 are values.
HcclResult HcclSetConfig(HcclConfig config, HcclConfigValue configValue)
{
    if (config != HCCL_DETERMINISTIC) {
        return HCCL_SUCCESS;
    }
    if (std::getenv("HCCL_DETERMINISTIC") != nullptr) {
        HCCL_LOG_WARN("HcclSetConfig: HCCL_DETERMINISTIC is set in the environment and wins");
        return HCCL_SUCCESS;
    }
    if (configValue.value != 0 && configValue.value != 1) {
        HCCL_LOG_ERROR("HcclSetConfig: HCCL_DETERMINISTIC takes 0 or 1");
        return HCCL_E_PARA;
    }
    std::lock_guard<std::mutex> reg(g_registryMutex);
    g_deterministic = configValue.value;
    for (Group *g : g_groups) {
        std::lock_guard<std::mutex> lock(g->m);
        g->cfg.deterministic = configValue.value == 1;
    }
    return HCCL_SUCCESS;
}

// op_base.cc:1245-1253.
HcclResult HcclGetConfig(HcclConfig config, HcclConfigValue *configValue)
{
    CHK_PTR(configValue);
    if (config == HCCL_DETERMINISTIC) {
        const char *e = std::getenv("HCCL_DETERMINISTIC");
        if (e != nullptr) {
            configValue->value = (std::string(e) == "true" || std::string(e) == "1") ? 1 : 0;
        } else {
            std::lock_guard<std::mutex> reg(g_registryMutex);
            configValue->value = g_deterministic == 1 ? 1 : 0;
        }
    }
    return HCCL_SUCCESS;
}

// op_base.cc:3085-3096.  The error is sticky: a failed launch keeps being reported.
HcclResult HcclGetCommAsyncError(HcclComm comm, HcclResult *asyncError)
{
    CHK_PTR(comm);
    CHK_PTR(asyncError);
    Comm *c = AsComm(comm);
    if (c == nullptr) {
        return HCCL_E_PARA;
    }
    std::lock_guard<std::mutex> lock(c->group->m);
    *asyncError = c->group->asyncError;
    return HCCL_SUCCESS;
}

// op_base.cc:3103-3122.  The reference's table has no entry for HCCL_E_SUSPENDING and would throw
// on it; a string is supplied here.
const char *HcclGetErrorString(HcclResult code)
{
    static const char *const names[] = {"no error", "parameter error", "empty pointer", "memory error", "internal error",
        "not support feature", "not found specific resource", "resource unavailable", "call system interface error",
        "timeout", "open file fail", "tcp connect fail", "roce connect fail", "tcp transfer fail", "roce transfer fail",
        "call runtime api fail", "call driver api fail", "call profiling api fail", "call cce api fail",
        "call network api fail", "try again", "error cqe", "communicator suspending"};
    // a caller may hand over any number; it is read as one, not as the enumeration it may not belong to
    int32_t value = 0;
    static_assert(sizeof(value) == sizeof(code), "HcclResult is a 32-bit enumeration");
    std::memcpy(&value, &code, sizeof(value));
    if (value < int32_t(HCCL_SUCCESS) || value >= int32_t(HCCL_E_RESERVED)) {
        return "unknow error";
    }
    return names[value];
}

// op_base.cc:3567-3571.
uint32_t HcclGetCommConfigCapability() { return static_cast<uint32_t>(HCCL_COMM_CONFIG_RESERVED); }

// op_base.cc:3541-3565.  Applies to the whole group: a suspended group refuses collectives.
HcclResult HcclCommSuspend(HcclComm comm)
{
    CHK_PTR(comm);
    Comm *c = AsComm(comm);
    if (c == nullptr) {
        return HCCL_E_PARA;
    }
    std::lock_guard<std::mutex> lock(c->group->m);
    c->group->suspended = true;
    return HCCL_SUCCESS;
}

HcclResult HcclCommResume(HcclComm comm)
{
    CHK_PTR(comm);
    Comm *c = AsComm(comm);
    if (c == nullptr) {
        return HCCL_E_PARA;
    }
    std::lock_guard<std::mutex> lock(c->group->m);
    c->group->suspended = false;
    c->group->asyncError = HCCL_SUCCESS;
    return HCCL_SUCCESS;
}

// ---- the four collectives ---------------------------------------------------------------------------

// op_base.cc:1268-1350.
HcclResult HcclAllReduce(void *sendBuf, void *recvBuf, uint64_t count, HcclDataType dataType, HcclReduceOp op,
    HcclComm comm, aclrtStream stream)
{
    if (count == 0) {
        HCCL_LOG_WARN("HcclAllReduce: count is 0, nothing to do");
        return HCCL_SUCCESS;
    }
    CHK_PTR(comm);
    CHK_PTR(sendBuf);
    CHK_PTR(recvBuf);
    Comm *c = AsComm(comm);
    if (c == nullptr) {
        return HCCL_E_PARA;
    }
    InUse guard(c);
    HcclResult r = CheckOpParam("HcclAllReduce", count, dataType, stream);
    if (r == HCCL_SUCCESS) {
        r = CheckReduce("HcclAllReduce", dataType, op);
    }
    if (r != HCCL_SUCCESS) {
        return r;
    }
    if ((reinterpret_cast<uintptr_t>(sendBuf) | reinterpret_cast<uintptr_t>(recvBuf)) % ElemSize(dataType) != 0) {
        HCCL_LOG_ERROR("HcclAllReduce: buffers must be aligned to the element size");
        return HCCL_E_PARA;
    }
    OpSig sig;
    sig.coll = COLL_ALLREDUCE;
    sig.count = count;
    sig.dtype = dataType;
    sig.recvType = dataType;
    sig.op = op;
    return Arrive(c, sig, sendBuf, recvBuf, static_cast<hipStream_t>(stream), nullptr, nullptr, nullptr, nullptr);
}

// op_base.cc:1506-1583.
HcclResult HcclReduceScatter(void *sendBuf, void *recvBuf, uint64_t recvCount, HcclDataType dataType, HcclReduceOp op,
    HcclComm comm, aclrtStream stream)
{
    if (recvCount == 0) {
        HCCL_LOG_WARN("HcclReduceScatter: recvCount is 0, nothing to do");
        return HCCL_SUCCESS;
    }
    CHK_PTR(comm);
    CHK_PTR(sendBuf);
    CHK_PTR(recvBuf);
    Comm *c = AsComm(comm);
    if (c == nullptr) {
        return HCCL_E_PARA;
    }
    InUse guard(c);
    HcclResult r = CheckOpParam("HcclReduceScatter", recvCount, dataType, stream);
    if (r == HCCL_SUCCESS) {
        r = CheckReduce("HcclReduceScatter", dataType, op);
    }
    if (r != HCCL_SUCCESS) {
        return r;
    }
    if ((reinterpret_cast<uintptr_t>(sendBuf) | reinterpret_cast<uintptr_t>(recvBuf)) % ElemSize(dataType) != 0) {
        HCCL_LOG_ERROR("HcclReduceScatter: buffers must be aligned to the element size");
        return HCCL_E_PARA;
    }
    OpSig sig;
    sig.coll = COLL_REDUCESCATTER;
    sig.count = recvCount;
    sig.dtype = dataType;
    sig.recvType = dataType;
    sig.op = op;
    return Arrive(c, sig, sendBuf, recvBuf, static_cast<hipStream_t>(stream), nullptr, nullptr, nullptr, nullptr);
}

// No counterpart in the reference.  HcclReduceScatter for callers that cannot allocate device memory
// (code under HIP graph capture, tight serving loops, harnesses that forbid it): same arguments and
// checks; descriptor tables and the step-by-step schedule's partial results live in a fixed device
// workspace instead of library allocations, nothing is cached, no graph is instantiated.
HcclResult HcclAmdReduceScatterNoAlloc(void *sendBuf, void *recvBuf, uint64_t recvCount, HcclDataType dataType,
    HcclReduceOp op, HcclComm comm, aclrtStream stream)
{
    if (recvCount == 0) {
        HCCL_LOG_WARN("HcclAmdReduceScatterNoAlloc: recvCount is 0, nothing to do");
        return HCCL_SUCCESS;
    }
    CHK_PTR(comm);
    CHK_PTR(sendBuf);
    CHK_PTR(recvBuf);
    Comm *c = AsComm(comm);
    if (c == nullptr) {
        return HCCL_E_PARA;
    }
    InUse guard(c);
    HcclResult r = CheckOpParam("HcclAmdReduceScatterNoAlloc", recvCount, dataType, stream);
    if (r == HCCL_SUCCESS) {
        r = CheckReduce("HcclAmdReduceScatterNoAlloc", dataType, op);
    }
    if (r != HCCL_SUCCESS) {
        return r;
    }
    if ((reinterpret_cast<uintptr_t>(sendBuf) | reinterpret_cast<uintptr_t>(recvBuf)) % ElemSize(dataType) != 0) {
        HCCL_LOG_ERROR("HcclAmdReduceScatterNoAlloc: buffers must be aligned to the element size");
        return HCCL_E_PARA;
    }
    OpSig sig;
    sig.coll = COLL_REDUCESCATTER;
    sig.count = recvCount;
    sig.dtype = dataType;
    sig.recvType = dataType;
    sig.op = op;
    sig.noAlloc = 1;
    return Arrive(c, sig, sendBuf, recvBuf, static_cast<hipStream_t>(stream), nullptr, nullptr, nullptr, nullptr);
}

// op_base.cc:1796-1861.
HcclResult HcclAllGather(void *sendBuf, void *recvBuf, uint64_t sendCount, HcclDataType dataType, HcclComm comm,
    aclrtStream stream)
{
    if (sendCount == 0) {
        HCCL_LOG_WARN("HcclAllGather: sendCount is 0, nothing to do");
        return HCCL_SUCCESS;
    }
    CHK_PTR(comm);
    CHK_PTR(sendBuf);
    CHK_PTR(recvBuf);
    Comm *c = AsComm(comm);
    if (c == nullptr) {
        return HCCL_E_PARA;
    }
    InUse guard(c);
    HcclResult r = CheckOpParam("HcclAllGather", sendCount, dataType, stream);
    if (r != HCCL_SUCCESS) {
        return r;
    }
    OpSig sig;
    sig.coll = COLL_ALLGATHER;
    sig.count = sendCount;
    sig.dtype = dataType;
    sig.recvType = dataType;
    sig.op = 0;
    return Arrive(c, sig, sendBuf, recvBuf, static_cast<hipStream_t>(stream), nullptr, nullptr, nullptr, nullptr);
}

// op_base.cc:2520-2631, param_check.cc:145-203.
HcclResult HcclAlltoAllV(const void *sendBuf, const void *sendCounts, const void *sdispls, HcclDataType sendType,
    const void *recvBuf, const void *recvCounts, const void *rdispls, HcclDataType recvType, HcclComm comm,
    aclrtStream stream)
{
    CHK_PTR(sendCounts);
    CHK_PTR(sdispls);
    CHK_PTR(recvCounts);
    CHK_PTR(rdispls);
    CHK_PTR(stream);
    CHK_PTR(comm);
    Comm *c = AsComm(comm);
    if (c == nullptr) {
        return HCCL_E_PARA;
    }
    InUse guard(c);
    uint32_t p = c->group->p;
    if (sendBuf != nullptr && recvBuf != nullptr && sendBuf == recvBuf) {
        HCCL_LOG_ERROR("HcclAlltoAllV: sendBuf and recvBuf cannot be the same");
        return HCCL_E_PARA;
    }
    const uint64_t *sc = static_cast<const uint64_t *>(sendCounts);
    const uint64_t *rc = static_cast<const uint64_t *>(recvCounts);
    bool hasSend = false, hasRecv = false;
    for (uint32_t i = 0; i < p; i++) {
        if (sc[i] > kSysMaxCount || rc[i] > kSysMaxCount) {
            HCCL_LOG_ERROR("HcclAlltoAllV: a count exceeds the maximum");
            return HCCL_E_PARA;
        }
        hasSend = hasSend || sc[i] != 0;
        hasRecv = hasRecv || rc[i] != 0;
    }
    if (hasSend) {
        CHK_PTR(sendBuf);
    }
    if (hasRecv) {
        CHK_PTR(recvBuf);
    }
    HcclResult r = CheckOpParam("HcclAlltoAllV", 0, sendType, stream);
    if (r != HCCL_SUCCESS) {
        return r;
    }
    if (!DataTypeKnown(recvType)) {
        return HCCL_E_NOT_SUPPORT;
    }
    if (ElemSize(sendType) != ElemSize(recvType)) {
        HCCL_LOG_ERROR("HcclAlltoAllV: send and receive element sizes differ");
        return HCCL_E_PARA;
    }
    OpSig sig;
    sig.coll = COLL_ALLTOALLV;
    sig.count = 0;
    sig.dtype = sendType;
    sig.recvType = recvType;
    sig.op = 0;
    return Arrive(c, sig, const_cast<void *>(sendBuf), const_cast<void *>(recvBuf), static_cast<hipStream_t>(stream), sc,
        static_cast<const uint64_t *>(sdispls), rc, static_cast<const uint64_t *>(rdispls));
}

// ---- siblings that run through the same schedules and kernels -----------------------------------------

// op_base.cc:1585-1718.  Ring / mesh / halving-doubling reduce-scatter over the caller's block table;
// every rank must pass the same table and recvCount == sendCounts[rank].
HcclResult HcclReduceScatterV(void *sendBuf, const void *sendCounts, const void *sendDispls, void *recvBuf,
    uint64_t recvCount, HcclDataType dataType, HcclReduceOp op, HcclComm comm, aclrtStream stream)
{
    CHK_PTR(sendCounts);
    CHK_PTR(sendDispls);
    CHK_PTR(comm);
    if (recvCount > 0) {
        CHK_PTR(recvBuf);
    }
    Comm *c = AsComm(comm);
    if (c == nullptr) {
        return HCCL_E_PARA;
    }
    InUse guard(c);
    HcclResult r = CheckOpParam("HcclReduceScatterV", recvCount, dataType, stream);
    if (r == HCCL_SUCCESS) {
        r = CheckReduce("HcclReduceScatterV", dataType, op);
    }
    if (r != HCCL_SUCCESS) {
        return r;
    }
    const uint64_t *counts = static_cast<const uint64_t *>(sendCounts);
    uint64_t total = 0;
    for (uint32_t i = 0; i < c->group->p; i++) {
        if (counts[i] > kSysMaxCount) {
            HCCL_LOG_ERROR("HcclReduceScatterV: sendCounts[%u] exceeds the maximum", i);
            return HCCL_E_PARA;
        }
        total += counts[i];
    }
    if (total == 0) {
        HCCL_LOG_WARN("HcclReduceScatterV: nothing to reduce");
        return HCCL_SUCCESS;
    }
    CHK_PTR(sendBuf);
    if (counts[c->rank] != recvCount) {
        HCCL_LOG_ERROR("HcclReduceScatterV: recvCount %llu differs from sendCounts[rank] %llu",
            (unsigned long long)recvCount, (unsigned long long)counts[c->rank]);
        return HCCL_E_PARA;
    }
    uint32_t unit = ElemSize(dataType);
    if (reinterpret_cast<uintptr_t>(sendBuf) % unit != 0 || (recvBuf && reinterpret_cast<uintptr_t>(recvBuf) % unit != 0)) {
        return HCCL_E_PARA;
    }
    OpSig sig;
    sig.coll = COLL_REDUCESCATTER;
    sig.count = 0;
    sig.dtype = dataType;
    sig.recvType = dataType;
    sig.op = op;
    sig.variable = 1;
    return Arrive(c, sig, sendBuf, recvBuf, static_cast<hipStream_t>(stream), nullptr, nullptr, nullptr, nullptr, counts,
        static_cast<const uint64_t *>(sendDispls));
}

// op_base.cc:1863-1972.  sendCount must equal recvCounts[rank]; every rank passes the same table.
HcclResult HcclAllGatherV(void *sendBuf, uint64_t sendCount, void *recvBuf, const void *recvCounts, const void *recvDispls,
    HcclDataType dataType, HcclComm comm, aclrtStream stream)
{
    CHK_PTR(recvCounts);
    CHK_PTR(recvDispls);
    CHK_PTR(comm);
    if (sendCount > 0) {
        CHK_PTR(sendBuf);
    }
    Comm *c = AsComm(comm);
    if (c == nullptr) {
        return HCCL_E_PARA;
    }
    InUse guard(c);
    HcclResult r = CheckOpParam("HcclAllGatherV", sendCount, dataType, stream);
    if (r != HCCL_SUCCESS) {
        return r;
    }
    const uint64_t *counts = static_cast<const uint64_t *>(recvCounts);
    uint64_t total = 0;
    for (uint32_t i = 0; i < c->group->p; i++) {
        if (counts[i] > kSysMaxCount) {
            HCCL_LOG_ERROR("HcclAllGatherV: recvCounts[%u] exceeds the maximum", i);
            return HCCL_E_PARA;
        }
        total += counts[i];
    }
    if (total == 0) {
        HCCL_LOG_WARN("HcclAllGatherV: nothing to gather");
        return HCCL_SUCCESS;
    }
    CHK_PTR(recvBuf);
    if (counts[c->rank] != sendCount) {
        HCCL_LOG_ERROR("HcclAllGatherV: sendCount %llu differs from recvCounts[rank] %llu", (unsigned long long)sendCount,
            (unsigned long long)counts[c->rank]);
        return HCCL_E_PARA;
    }
    OpSig sig;
    sig.coll = COLL_ALLGATHER;
    sig.count = 0;
    sig.dtype = dataType;
    sig.recvType = dataType;
    sig.op = 0;
    sig.variable = 1;
    return Arrive(c, sig, sendBuf, recvBuf, static_cast<hipStream_t>(stream), nullptr, nullptr, nullptr, nullptr, counts,
        static_cast<const uint64_t *>(recvDispls));
}

// op_base.cc:2422-2518: the uniform all-to-all is the pairwise schedule with equal blocks.
HcclResult HcclAlltoAll(const void *sendBuf, uint64_t sendCount, HcclDataType sendType, const void *recvBuf,
    uint64_t recvCount, HcclDataType recvType, HcclComm comm, aclrtStream stream)
{
    if (sendCount == 0 && recvCount == 0) {
        HCCL_LOG_WARN("HcclAlltoAll: both counts are 0, nothing to do");
        return HCCL_SUCCESS;
    }
    CHK_PTR(sendBuf);
    CHK_PTR(recvBuf);
    if (sendCount != recvCount) {
        HCCL_LOG_ERROR("HcclAlltoAll: sendCount and recvCount differ");
        return HCCL_E_PARA;
    }
    if (sendType != recvType) {
        HCCL_LOG_ERROR("HcclAlltoAll: sendType and recvType differ");
        return HCCL_E_PARA;
    }
    CHK_PTR(stream);
    CHK_PTR(comm);
    if (sendBuf == recvBuf) {
        HCCL_LOG_ERROR("HcclAlltoAll: sendBuf and recvBuf cannot be the same");
        return HCCL_E_PARA;
    }
    Comm *c = AsComm(comm);
    if (c == nullptr) {
        return HCCL_E_PARA;
    }
    InUse guard(c);
    HcclResult r = CheckOpParam("HcclAlltoAll", 0, sendType, stream);
    if (r != HCCL_SUCCESS) {
        return r;
    }
    if (sendCount > kSysMaxCount) {
        return HCCL_E_PARA;
    }
    uint32_t p = c->group->p;
    std::vector<uint64_t> counts(p, sendCount), displs(p);
    for (uint32_t i = 0; i < p; i++) {
        displs[i] = uint64_t(i) * sendCount;
    }
    OpSig sig;
    sig.coll = COLL_ALLTOALLV;
    sig.dtype = sendType;
    sig.recvType = recvType;
    return Arrive(c, sig, const_cast<void *>(sendBuf), const_cast<void *>(recvBuf), static_cast<hipStream_t>(stream),
        counts.data(), displs.data(), counts.data(), displs.data());
}

// op_base.cc:2633-2733.  sendCountMatrix is a host array of p x p uint64_t, the same on every rank:
// entry [i * p + j] = elements rank i sends to rank j.  Blocks are packed back to back on both sides
// (displacements are running sums, alltoall_operator.cc:74-120); checks as in param_check.cc:205-242.
HcclResult HcclAlltoAllVC(const void *sendBuf, const void *sendCountMatrix, HcclDataType sendType, const void *recvBuf,
    HcclDataType recvType, HcclComm comm, aclrtStream stream)
{
    CHK_PTR(sendCountMatrix);
    CHK_PTR(comm);
    Comm *c = AsComm(comm);
    if (c == nullptr) {
        return HCCL_E_PARA;
    }
    InUse guard(c);
    const uint32_t p = c->group->p, me = c->rank;
    if (sendBuf != nullptr && recvBuf != nullptr && sendBuf == recvBuf) {
        HCCL_LOG_ERROR("HcclAlltoAllVC: sendBuf and recvBuf cannot be the same");
        return HCCL_E_PARA;
    }
    const uint64_t *m = static_cast<const uint64_t *>(sendCountMatrix);
    std::vector<uint64_t> sc(p), sd(p), rc(p), rd(p);
    bool hasSend = false, hasRecv = false;
    uint64_t sAt = 0, rAt = 0;
    for (uint32_t j = 0; j < p; j++) {
        sc[j] = m[uint64_t(me) * p + j];
        rc[j] = m[uint64_t(j) * p + me];
        if (sc[j] > kSysMaxCount) {
            HCCL_LOG_ERROR("HcclAlltoAllVC: a count exceeds the maximum");
            return HCCL_E_PARA;
        }
        sd[j] = sAt;
        rd[j] = rAt;
        sAt += sc[j];
        rAt += rc[j];
        hasSend = hasSend || sc[j] != 0;
        hasRecv = hasRecv || rc[j] != 0;
    }
    if (hasSend) {
        CHK_PTR(sendBuf);
    }
    if (hasRecv) {
        CHK_PTR(recvBuf);
    }
    HcclResult r = CheckOpParam("HcclAlltoAllVC", 0, sendType, stream);
    if (r != HCCL_SUCCESS) {
        return r;
    }
    if (!DataTypeKnown(recvType)) {
        return HCCL_E_NOT_SUPPORT;
    }
    if (ElemSize(sendType) != ElemSize(recvType)) {
        HCCL_LOG_ERROR("HcclAlltoAllVC: send and receive element sizes differ");
        return HCCL_E_PARA;
    }
    OpSig sig;
    sig.coll = COLL_ALLTOALLV;
    sig.dtype = sendType;
    sig.recvType = recvType;
    // ranks that pass different matrices fail the symmetry check of the rendezvous (HCCL_E_PARA)
    return Arrive(c, sig, const_cast<void *>(sendBuf), const_cast<void *>(recvBuf), static_cast<hipStream_t>(stream),
        sc.data(), sd.data(), rc.data(), rd.data());
}

// op_base.cc:1353-1431: an all-reduce (fp32 sum) of a few elements on buffers the group owns.
HcclResult HcclBarrier(HcclComm comm, aclrtStream stream)
{
    CHK_PTR(comm);
    CHK_PTR(stream);
    Comm *c = AsComm(comm);
    if (c == nullptr) {
        return HCCL_E_PARA;
    }
    InUse guard(c);
    Group *g = c->group;
    constexpr uint64_t kBarrierCount = 8;   // elements per rank; the value is never read back
    constexpr uint64_t kSlot = 256;         // bytes between buffers
    {
        std::lock_guard<std::mutex> lock(g->m);
        HcclResult r = EnsureDevice(g, false);
        if (r != HCCL_SUCCESS) {
            return r;
        }
        if (g->barrierMem == nullptr) {
            if (hipMalloc(&g->barrierMem, 2 * kSlot * g->p) != hipSuccess ||
                hipMemset(g->barrierMem, 0, 2 * kSlot * g->p) != hipSuccess) {
                return HCCL_E_RUNTIME;
            }
        }
    }
    char *base = static_cast<char *>(g->barrierMem);
    OpSig sig;
    sig.coll = COLL_ALLREDUCE;
    sig.count = kBarrierCount;
    sig.dtype = HCCL_DATA_TYPE_FP32;
    sig.recvType = HCCL_DATA_TYPE_FP32;
    sig.op = HCCL_REDUCE_SUM;
    return Arrive(c, sig, base + kSlot * (2 * c->rank), base + kSlot * (2 * c->rank + 1), static_cast<hipStream_t>(stream),
        nullptr, nullptr, nullptr, nullptr);
}

// ---- rooted collectives ---------------------------------------------------------------------------------

// op_base.cc:1433-1504.  Ring broadcast; buf is the source on the root and the destination elsewhere.
HcclResult HcclBroadcast(void *buf, uint64_t count, HcclDataType dataType, uint32_t root, HcclComm comm, aclrtStream stream)
{
    if (count == 0) {
        HCCL_LOG_WARN("HcclBroadcast: count is 0, nothing to do");
        return HCCL_SUCCESS;
    }
    CHK_PTR(comm);
    CHK_PTR(buf);
    Comm *c = AsComm(comm);
    if (c == nullptr) {
        return HCCL_E_PARA;
    }
    InUse guard(c);
    HcclResult r = CheckOpParam("HcclBroadcast", count, dataType, stream);
    if (r != HCCL_SUCCESS) {
        return r;
    }
    if (root >= c->group->p) {   // param_check.cc:351-359
        HCCL_LOG_ERROR("HcclBroadcast: root %u is out of range", root);
        return HCCL_E_PARA;
    }
    OpSig sig;
    sig.coll = COLL_BROADCAST;
    sig.count = count;
    sig.dtype = dataType;
    sig.recvType = dataType;
    sig.root = root;
    return Arrive(c, sig, buf, buf, static_cast<hipStream_t>(stream), nullptr, nullptr, nullptr, nullptr);
}

// op_base.cc:2737-2814.  Ring reduce towards the root; recvBuf is written on the root only.
HcclResult HcclReduce(void *sendBuf, void *recvBuf, uint64_t count, HcclDataType dataType, HcclReduceOp op, uint32_t root,
    HcclComm comm, aclrtStream stream)
{
    if (count == 0) {
        HCCL_LOG_WARN("HcclReduce: count is 0, nothing to do");
        return HCCL_SUCCESS;
    }
    CHK_PTR(comm);
    CHK_PTR(sendBuf);
    CHK_PTR(recvBuf);
    Comm *c = AsComm(comm);
    if (c == nullptr) {
        return HCCL_E_PARA;
    }
    InUse guard(c);
    HcclResult r = CheckOpParam("HcclReduce", count, dataType, stream);
    if (r == HCCL_SUCCESS) {
        r = CheckReduce("HcclReduce", dataType, op);
    }
    if (r != HCCL_SUCCESS) {
        return r;
    }
    if (root >= c->group->p) {
        HCCL_LOG_ERROR("HcclReduce: root %u is out of range", root);
        return HCCL_E_PARA;
    }
    if ((reinterpret_cast<uintptr_t>(sendBuf) | reinterpret_cast<uintptr_t>(recvBuf)) % ElemSize(dataType) != 0) {
        return HCCL_E_PARA;
    }
    OpSig sig;
    sig.coll = COLL_REDUCE;
    sig.count = count;
    sig.dtype = dataType;
    sig.recvType = dataType;
    sig.op = op;
    sig.root = root;
    return Arrive(c, sig, sendBuf, recvBuf, static_cast<hipStream_t>(stream), nullptr, nullptr, nullptr, nullptr);
}

// op_base.cc:1720-1794.  The root's sendBuf holds p blocks of recvCount elements; rank i receives block i.
HcclResult HcclScatter(void *sendBuf, void *recvBuf, uint64_t recvCount, HcclDataType dataType, uint32_t root, HcclComm comm,
    aclrtStream stream)
{
    if (recvCount == 0) {
        HCCL_LOG_WARN("HcclScatter: recvCount is 0, nothing to do");
        return HCCL_SUCCESS;
    }
    CHK_PTR(comm);
    CHK_PTR(recvBuf);
    Comm *c = AsComm(comm);
    if (c == nullptr) {
        return HCCL_E_PARA;
    }
    InUse guard(c);
    if (c->rank == root) {
        CHK_PTR(sendBuf);
    }
    HcclResult r = CheckOpParam("HcclScatter", recvCount, dataType, stream);
    if (r != HCCL_SUCCESS) {
        return r;
    }
    if (root >= c->group->p) {
        HCCL_LOG_ERROR("HcclScatter: root %u is out of range", root);
        return HCCL_E_PARA;
    }
    OpSig sig;
    sig.coll = COLL_SCATTER;
    sig.count = recvCount;
    sig.dtype = dataType;
    sig.recvType = dataType;
    sig.root = root;
    return Arrive(c, sig, sendBuf, recvBuf, static_cast<hipStream_t>(stream), nullptr, nullptr, nullptr, nullptr);
}

// ---- point to point -----------------------------------------------------------------------------------------

// op_base.cc:1974-2054.
HcclResult HcclSend(void *sendBuf, uint64_t count, HcclDataType dataType, uint32_t destRank, HcclComm comm, aclrtStream stream)
{
    if (count == 0) {
        HCCL_LOG_WARN("HcclSend: count is 0, nothing to do");
        return HCCL_SUCCESS;
    }
    CHK_PTR(comm);
    CHK_PTR(sendBuf);
    CHK_PTR(stream);
    if (count > kSysMaxCount) {
        return HCCL_E_PARA;
    }
    if (!DataTypeKnown(dataType)) {
        return HCCL_E_NOT_SUPPORT;
    }
    Comm *c = AsComm(comm);
    if (c == nullptr) {
        return HCCL_E_PARA;
    }
    InUse guard(c);
    return PointToPoint(c, true, sendBuf, count, dataType, destRank, static_cast<hipStream_t>(stream));
}

// op_base.cc:2056-2135.
HcclResult HcclRecv(void *recvBuf, uint64_t count, HcclDataType dataType, uint32_t srcRank, HcclComm comm, aclrtStream stream)
{
    if (count == 0) {
        HCCL_LOG_WARN("HcclRecv: count is 0, nothing to do");
        return HCCL_SUCCESS;
    }
    CHK_PTR(comm);
    CHK_PTR(recvBuf);
    CHK_PTR(stream);
    if (count > kSysMaxCount) {
        return HCCL_E_PARA;
    }
    if (!DataTypeKnown(dataType)) {
        return HCCL_E_NOT_SUPPORT;
    }
    Comm *c = AsComm(comm);
    if (c == nullptr) {
        return HCCL_E_PARA;
    }
    InUse guard(c);
    return PointToPoint(c, false, recvBuf, count, dataType, srcRank, static_cast<hipStream_t>(stream));
}

// op_base.cc:3428-3509: every item is a send or a receive of this rank.
HcclResult HcclBatchSendRecv(HcclSendRecvItem *sendRecvInfo, uint32_t itemNum, HcclComm comm, aclrtStream stream)
{
    CHK_PTR(comm);
    CHK_PTR(stream);
    CHK_PTR(sendRecvInfo);
    if (itemNum == 0) {
        HCCL_LOG_WARN("HcclBatchSendRecv: no items");
        return HCCL_SUCCESS;
    }
    Comm *c = AsComm(comm);
    if (c == nullptr) {
        return HCCL_E_PARA;
    }
    InUse guard(c);
    for (uint32_t i = 0; i < itemNum; i++) {
        const HcclSendRecvItem &it = sendRecvInfo[i];
        CHK_PTR(it.buf);
        if (it.count > kSysMaxCount) {
            return HCCL_E_PARA;
        }
        if (!DataTypeKnown(it.dataType)) {
            return HCCL_E_NOT_SUPPORT;
        }
        if (it.sendRecvType != HCCL_SEND && it.sendRecvType != HCCL_RECV) {
            return HCCL_E_PARA;
        }
    }
    for (uint32_t i = 0; i < itemNum; i++) {
        const HcclSendRecvItem &it = sendRecvInfo[i];
        if (it.count == 0) {
            continue;
        }
        HcclResult r = PointToPoint(c, it.sendRecvType == HCCL_SEND, it.buf, it.count, it.dataType, it.remoteRank,
            static_cast<hipStream_t>(stream));
        if (r != HCCL_SUCCESS) {
            return r;
        }
    }
    return HCCL_SUCCESS;
}

// ---- communicators assembled rank by rank --------------------------------------------------------------------

// op_base.cc:794-843.  The token names a group that HcclCommInitRootInfo calls of this process join.
HcclResult HcclGetRootInfo(HcclRootInfo *rootInfo)
{
    CHK_PTR(rootInfo);
    std::lock_guard<std::mutex> reg(g_registryMutex);
    std::memset(rootInfo->internal, 0, HCCL_ROOT_INFO_BYTES);
    std::snprintf(rootInfo->internal, 128, "hccl_amd_root_%llu", static_cast<unsigned long long>(++g_rootInfoSerial));
    return HCCL_SUCCESS;
}

// op_base.cc:1055-1120.  One call per rank, from any thread of this process; all ranks run on the current GPU.
HcclResult HcclCommInitRootInfo(uint32_t nRanks, const HcclRootInfo *rootInfo, uint32_t rank, HcclComm *comm)
{
    CHK_PTR(rootInfo);
    if (nRanks == 0) {
        HCCL_LOG_ERROR("HcclCommInitRootInfo: nRanks must be greater than 0");
        return HCCL_E_PARA;
    }
    if (rank >= nRanks) {
        HCCL_LOG_ERROR("HcclCommInitRootInfo: rank %u is out of range", rank);
        return HCCL_E_PARA;
    }
    CHK_PTR(comm);
    std::string key(rootInfo->internal, strnlen(rootInfo->internal, 127));
    if (key.compare(0, 14, "hccl_amd_root_") != 0) {
        HCCL_LOG_ERROR("HcclCommInitRootInfo: the root info was not produced by HcclGetRootInfo of this process");
        return HCCL_E_PARA;
    }
    return JoinFormingGroup(key, nRanks, rank, nullptr, comm);
}

// op_base.cc:1122-1202; configuration rules of comm_config.cc (the first rank's configuration applies).
HcclResult HcclCommInitRootInfoConfig(uint32_t nRanks, const HcclRootInfo *rootInfo, uint32_t rank,
    const HcclCommConfig *config, HcclComm *comm)
{
    CHK_PTR(rootInfo);
    if (nRanks == 0 || rank >= nRanks) {
        return HCCL_E_PARA;
    }
    CHK_PTR(comm);
    CHK_PTR(config);
    std::string key(rootInfo->internal, strnlen(rootInfo->internal, 127));
    if (key.compare(0, 14, "hccl_amd_root_") != 0) {
        return HCCL_E_PARA;
    }
    GroupConfig probe;
    std::string name;
    HcclResult r = LoadCommConfig(config, &probe, &name);   // every rank's configuration is validated
    if (r != HCCL_SUCCESS) {
        return r;
    }
    return JoinFormingGroup(key, nRanks, rank, config, comm);
}

// op_base.cc:730-792.  Every member rank calls with the same rankIds and subCommId; a rank outside the
// sub-communicator passes rankIds == nullptr and subCommId == 0xFFFFFFFF and gets nothing.
HcclResult HcclCreateSubCommConfig(HcclComm *comm, uint32_t rankNum, uint32_t *rankIds, uint64_t subCommId,
    uint32_t subCommRankId, HcclCommConfig *config, HcclComm *subComm)
{
    constexpr uint64_t kInvalidSubCommId = 0xFFFFFFFFull;
    CHK_PTR(subComm);
    if (rankIds == nullptr && subCommId == kInvalidSubCommId) {
        return HCCL_SUCCESS;
    }
    if (rankIds == nullptr || subCommId == kInvalidSubCommId) {
        HCCL_LOG_ERROR("HcclCreateSubCommConfig: rankIds and subCommId must both be valid or both be invalid");
        return HCCL_E_PARA;
    }
    if (rankNum == 0 || subCommRankId >= rankNum) {
        return HCCL_E_PARA;
    }
    CHK_PTR(config);
    CHK_PTR(comm);
    Comm *parent = AsComm(*comm);
    if (parent == nullptr) {
        return HCCL_E_PTR;
    }
    if (rankNum > parent->group->p || rankIds[subCommRankId] != parent->rank) {
        HCCL_LOG_ERROR("HcclCreateSubCommConfig: rankIds[subCommRankId] must be the calling rank");
        return HCCL_E_PARA;
    }
    GroupConfig probe;
    std::string name;
    if (LoadCommConfig(config, &probe, &name) != HCCL_SUCCESS) {
        return HCCL_E_PARA;
    }
    std::string key = parent->group->name + "_sub_" + std::to_string(subCommId);
    return JoinFormingGroup(key, rankNum, subCommRankId, config, subComm);
}

// ---- extension ----------------------------------------------------------------------------------------

HcclResult HcclAmdSetParam(HcclComm comm, const char *key, const char *value)
{
    CHK_PTR(comm);
    CHK_PTR(key);
    CHK_PTR(value);
    Comm *c = AsComm(comm);
    if (c == nullptr) {
        return HCCL_E_PARA;
    }
    std::lock_guard<std::mutex> lock(c->group->m);
    GroupConfig &cfg = c->group->cfg;
    std::string k(key), v(value);
    if (k == "algo") {
        if (v == "ring") {
            cfg.algo = ALGO_RING;
        } else if (v == "mesh") {
            cfg.algo = ALGO_MESH;
        } else if (v == "rhd") {
            cfg.algo = ALGO_RHD;
        } else if (v == "pairwise") {
            cfg.algo = ALGO_PAIRWISE;   // all-to-all family: the flat schedule also over several servers; others: ring
        } else if (v == "star") {
            cfg.algo = ALGO_STAR;       // broadcast: the root hands every rank the whole buffer; others: as "auto" would not, ring
        } else if (v == "hd_blocks") {
            cfg.algo = ALGO_HD_BLOCKS;  // broadcast: halving-doubling over blocks of power-of-two sizes; others: ring
        } else if (v == "auto") {
            cfg.algo = -1;
        } else {
            return HCCL_E_PARA;
        }
    } else if (k == "servers") {
        long n = std::atol(value);
        if (n < 1 || uint32_t(n) > c->group->p || c->group->p % uint32_t(n) != 0) {
            return HCCL_E_PARA;
        }
        cfg.servers = uint32_t(n);
    } else if (k == "level0") {
        if (v == "mesh") {
            cfg.level0Rings = 0;
        } else if (v == "ring") {
            cfg.level0Rings = 1;
        } else if (v == "ring4") {
            cfg.level0Rings = 4;
        } else {
            return HCCL_E_PARA;
        }
    } else if (k == "step_sweep") {
        if (v == "forward") {
            cfg.stepSweep = 0;
        } else if (v == "alternate") {
            cfg.stepSweep = 1;
        } else {
            return HCCL_E_PARA;
        }
    } else if (k == "cache_entries") {
        long n = std::atol(value);
        if (n < 1 || n > (1 << 20)) {
            return HCCL_E_PARA;
        }
        cfg.cacheEntries = uint32_t(n);
    } else if (k == "nic_ranks") {
        // the ranks of an 8-rank ring (the devices of every server of 8) that own a network port: "all", or a
        // comma-separated list of 1, 2 or 4 of them
        uint32_t mask = 0;
        if (v != "all" && !v.empty()) {
            if (c->group->p % 8 != 0) {
                return HCCL_E_PARA;
            }
            std::stringstream in(v);
            std::string item;
            while (std::getline(in, item, ',')) {
                char *end = nullptr;
                long r = std::strtol(item.c_str(), &end, 10);
                if (item.empty() || *end != 0 || r < 0 || r > 7 || ((mask >> r) & 1u)) {
                    return HCCL_E_PARA;
                }
                mask |= 1u << r;
            }
            const int ports = __builtin_popcount(mask);
            if (ports != 1 && ports != 2 && ports != 4 && ports != 8) {
                return HCCL_E_PARA;
            }
            if (ports == 8) {
                mask = 0;
            }
        }
        cfg.nicMask = mask;
    } else if (k == "fused_stores") {
        if (v == "auto") {
            cfg.fusedStores = -1;
        } else if (v == "nt") {
            cfg.fusedStores = 0;
        } else if (v == "ordinary") {
            cfg.fusedStores = 1;
        } else {
            return HCCL_E_PARA;
        }
    } else if (k == "team_tiles") {
        long n = std::atol(value);
        if (n < 0 || n > long(kTeamTiles)) {
            return HCCL_E_PARA;
        }
        cfg.teamTiles = uint32_t(n);
    } else if (k == "team") {
        if (v == "auto") {
            cfg.team = -1;
        } else if (v == "0" || v == "1") {
            cfg.team = v == "1" ? 1 : 0;
        } else {
            return HCCL_E_PARA;
        }
    } else if (k == "step_stores") {
        if (v == "auto") {
            cfg.stepStores = -1;
        } else if (v == "nt") {
            cfg.stepStores = 0;
        } else if (v == "ordinary") {
            cfg.stepStores = 1;
        } else {
            return HCCL_E_PARA;
        }
    } else if (k == "deterministic") {
        cfg.deterministic = v != "0";
    } else if (k == "fuse") {
        cfg.fuse = v != "0";
    } else if (k == "graph") {
        cfg.graph = v != "0";
    } else if (k == "buffsize_mib") {
        long n = std::atol(value);
        if (n < 1) {
            return HCCL_E_PARA;
        }
        cfg.cclBytes = uint64_t(n) << 20;
    } else if (k == "buffsize_bytes") {
        long long n = std::atoll(value);
        if (n < 16) {
            return HCCL_E_PARA;
        }
        cfg.cclBytes = uint64_t(n);
    } else if (k == "align") {
        long n = std::atol(value);
        if (n < 1) {
            return HCCL_E_PARA;
        }
        cfg.align = uint64_t(n);
    } else if (k == "blocks_per_cu") {
        long n = std::atol(value);
        if (n < 0 || n > 64) {
            return HCCL_E_PARA;
        }
        cfg.blocksPerCu = uint32_t(n);
    } else if (k == "launch_cap_mib") {
        long n = v == "auto" ? -1 : std::atol(value);
        if (n < -1 || n > (1 << 20)) {
            return HCCL_E_PARA;
        }
        cfg.launchCapMiB = int32_t(n);
    } else if (k == "blocking_arrive") {
        cfg.blockingArrive = v != "0";
    } else if (k == "arrive_timeout_ms") {
        long n = std::atol(value);
        if (n < 1) {
            return HCCL_E_PARA;
        }
        cfg.arriveTimeoutMs = uint32_t(n);
    } else {
        return HCCL_E_PARA;
    }
    return HCCL_SUCCESS;
}

HcclResult HcclAmdGetLastOpInfo(HcclComm comm, HcclAmdOpInfo *info)
{
    CHK_PTR(comm);
    CHK_PTR(info);
    Comm *c = AsComm(comm);
    if (c == nullptr) {
        return HCCL_E_PARA;
    }
    std::lock_guard<std::mutex> lock(c->group->m);
    const OpInfo &o = c->group->lastInfo;
    info->coll = o.coll;
    info->algo = o.algo;
    info->fused = o.fused;
    info->graph = o.graph;
    info->cacheHit = o.cacheHit;
    info->launches = o.launches;
    info->bytesRead = o.bytesRead;
    info->bytesWritten = o.bytesWritten;
    info->schedRead = o.stepRead;
    info->schedWritten = o.stepWritten;
    info->scratchBytes = o.scratchBytes;
    info->teamLaunches = o.teamLaunches;
    info->reserved = 0;
    return HCCL_SUCCESS;
}

HcclResult HcclAmdDescribePlan(int32_t coll, int32_t algo, uint32_t nRanks, uint64_t count, HcclDataType dataType,
    uint64_t cclBytes, uint64_t align, uint64_t inPlaceMask, const uint64_t *tables, char *out, size_t cap, size_t *needed)
{
    CHK_PTR(out);
    if (nRanks == 0 || nRanks > kMaxRanks || !DataTypeKnown(dataType) || coll < 0 || coll > 6) {
        return HCCL_E_PARA;
    }
    PlanRequest rq;
    rq.coll = CollKind(coll);
    if (coll >= COLL_BROADCAST) {
        // rooted collectives: low 16 bits = root rank, bits 16..19 = schedule (0 ring, 1 mesh, 2 rhd, 4 mesh uncut, 5 star, 6 hd over blocks);
        // reduce only: bits 20..27 = number of rank groups of the two-level schedule, bit 28 = its mesh level uncut,
        // bit 29 / bit 30 = one ring / four rings inside a group instead of the mesh
        rq.root = uint32_t(algo) & 0xffffu;
        rq.algo = Algo((uint32_t(algo) >> 16) & 0xfu);
        if (coll == COLL_SCATTER) {
            rq.algo = ((uint32_t(algo) >> 20) & 1u) ? ALGO_RING : ALGO_MESH;   // scatter: bit 20 = the ring schedule
            rq.servers = std::max(1u, (uint32_t(algo) >> 21) & 0xffu);         // bits 21..28 = rank groups (two levels, mesh only)
        }
        if (coll == COLL_BROADCAST) {
            rq.servers = std::max(1u, (uint32_t(algo) >> 20) & 0xffu);   // broadcast: bits 20..27 = rank groups (two levels)
        }
        if (coll == COLL_REDUCE) {
            rq.servers = std::max(1u, (uint32_t(algo) >> 20) & 0xffu);
            rq.meshAtomic = ((uint32_t(algo) >> 28) & 1u) != 0;
            rq.level0Rings = ((uint32_t(algo) >> 29) & 1u) ? 1u : (((uint32_t(algo) >> 30) & 1u) ? 4u : 0u);   // bit 29 one ring, bit 30 four
        }
    } else if (coll == COLL_ALLREDUCE) {
        // all-reduce: low 8 bits = schedule, bits 8..15 = number of rank groups ("servers") of a two-level schedule
        rq.algo = Algo(uint32_t(algo) & 0xffu);
        rq.servers = std::max(1u, (uint32_t(algo) >> 8) & 0xffu);
        rq.meshAtomic = ((uint32_t(algo) >> 16) & 1u) != 0;   // bit 16: mesh level without the piece cut
        rq.level0Rings = (uint32_t(algo) >> 17) & 7u;         // bits 17..19: rings inside a group (0 = mesh, 1, 4)
        rq.nicMask = (uint32_t(algo) >> 20) & 0xffu;          // bits 20..27: ranks with a network port (8-rank ring)
    } else if (coll == COLL_REDUCESCATTER || coll == COLL_ALLGATHER) {
        // reduce-scatter, all-gather: the same fields
        rq.algo = Algo(uint32_t(algo) & 0xffu);
        rq.servers = std::max(1u, (uint32_t(algo) >> 8) & 0xffu);
        rq.meshAtomic = ((uint32_t(algo) >> 16) & 1u) != 0;
        rq.level0Rings = (uint32_t(algo) >> 17) & 7u;
        if (coll == COLL_REDUCESCATTER) {
            rq.nicMask = (uint32_t(algo) >> 20) & 0xffu;      // bits 20..27: devices of every server with a network port
        }
    } else if (coll == COLL_ALLTOALLV) {
        // all-to-all-v: bits 8..15 = number of servers of the staged schedule (0 or 1 = flat pairwise)
        rq.algo = ALGO_PAIRWISE;
        rq.servers = std::max(1u, (uint32_t(algo) >> 8) & 0xffu);
    } else {
        rq.algo = Algo(algo);
    }
    rq.p = nRanks;
    rq.count = count;
    rq.unit = ElemSize(dataType);
    rq.cclBytes = cclBytes;
    rq.align = align;
    rq.alias.assign(nRanks, 0);
    for (uint32_t r = 0; r < nRanks; r++) {
        rq.alias[r] = (inPlaceMask >> r) & 1ull;
    }
    if (coll == COLL_ALLTOALLV) {
        CHK_PTR(tables);
        size_t n = size_t(nRanks) * nRanks;
        rq.sendCounts.assign(tables, tables + n);
        rq.sdispls.assign(tables + n, tables + 2 * n);
        rq.recvCounts.assign(tables + 2 * n, tables + 3 * n);
        rq.rdispls.assign(tables + 3 * n, tables + 4 * n);
    }
    if ((coll == COLL_REDUCESCATTER || coll == COLL_ALLGATHER) && tables != nullptr) {
        rq.vCounts.assign(tables, tables + nRanks);
        rq.vDispls.assign(tables + nRanks, tables + 2 * size_t(nRanks));
    }
    Plan plan;
    std::string err;
    int rc = BuildPlan(rq, &plan, &err);
    if (rc != 0) {
        HCCL_LOG_ERROR("HcclAmdDescribePlan: %s", err.c_str());
        return rc == 1 ? HCCL_E_PARA : HCCL_E_INTERNAL;
    }
    std::string js = DescribePlan(plan);
    if (needed) {
        *needed = js.size() + 1;
    }
    if (js.size() + 1 > cap) {
        return HCCL_E_MEMORY;
    }
    std::memcpy(out, js.c_str(), js.size() + 1);
    return HCCL_SUCCESS;
}

// ---- declared for link compatibility; outside the single-GPU data path -----------------------------------

// op_base.cc:465-503, :567-620 (declarations hccl.h:30, :42).  clusterInfo is the path of a rank table; its ranks are
// the ranks of one group in this process (every one of them makes this call, as for the root-info
// variant), and its servers become the rank groups of the two-level all-reduce.
static HcclResult InitFromRankTable(const char *clusterInfo, uint32_t rank, const HcclCommConfig *config, HcclComm *comm)
{
    std::ifstream file(clusterInfo);
    if (!file) {
        HCCL_LOG_ERROR("HcclCommInitClusterInfo: cannot read the rank table %s", clusterInfo);
        return HCCL_E_PARA;
    }
    std::stringstream text;
    text << file.rdbuf();
    RankTable table;
    std::string err;
    if (ParseRankTable(text.str(), &table, &err) != 0) {
        HCCL_LOG_ERROR("HcclCommInitClusterInfo: %s", err.c_str());
        return HCCL_E_PARA;
    }
    if (rank >= table.rankCount) {
        HCCL_LOG_ERROR("HcclCommInitClusterInfo: rank %u is not in the rank table (%u ranks)", rank, table.rankCount);
        return HCCL_E_PARA;
    }
    // the two-level schedule takes servers of equal size whose ranks are consecutive
    const size_t perServer = table.servers[0].ranks.size();
    bool regular = true;
    for (size_t s = 0; s < table.servers.size(); s++) {
        regular = regular && table.servers[s].ranks.size() == perServer;
        for (size_t d = 0; regular && d < perServer; d++) {
            regular = table.servers[s].ranks[d] == s * perServer + d;
        }
    }
    if (!regular) {
        HCCL_LOG_ERROR("HcclCommInitClusterInfo: servers must hold equally many ranks, numbered consecutively server by server");
        return HCCL_E_NOT_SUPPORT;
    }
    HcclResult r = JoinFormingGroup(std::string("ranktable:") + clusterInfo, table.rankCount, rank, config, comm);
    if (r != HCCL_SUCCESS) {
        return r;
    }
    Group *g = AsComm(*comm)->group;
    std::lock_guard<std::mutex> lock(g->m);
    g->cfg.servers = uint32_t(table.servers.size());
    return HCCL_SUCCESS;
}

HcclResult HcclCommInitClusterInfo(const char *clusterInfo, uint32_t rank, HcclComm *comm)
{
    CHK_PTR(clusterInfo);
    CHK_PTR(comm);
    return InitFromRankTable(clusterInfo, rank, nullptr, comm);
}

HcclResult HcclCommInitClusterInfoConfig(const char *clusterInfo, uint32_t rank, HcclCommConfig *config, HcclComm *comm)
{
    CHK_PTR(clusterInfo);
    CHK_PTR(config);
    CHK_PTR(comm);
    GroupConfig probe;
    std::string name;
    if (LoadCommConfig(config, &probe, &name) != HCCL_SUCCESS) {
        return HCCL_E_PARA;
    }
    return InitFromRankTable(clusterInfo, rank, config, comm);
}

HcclResult HcclCommSetMemoryRange(HcclComm comm, void *, size_t, size_t, uint64_t)
{
    CHK_PTR(comm);
    return HCCL_E_NOT_SUPPORT;
}
HcclResult HcclCommUnsetMemoryRange(HcclComm comm, void *)
{
    CHK_PTR(comm);
    return HCCL_E_NOT_SUPPORT;
}
HcclResult HcclCommActivateCommMemory(HcclComm comm, void *, size_t, size_t, aclrtDrvMemHandle, uint64_t)
{
    CHK_PTR(comm);
    return HCCL_E_NOT_SUPPORT;
}
HcclResult HcclCommDeactivateCommMemory(HcclComm comm, void *)
{
    CHK_PTR(comm);
    return HCCL_E_NOT_SUPPORT;
}

}  // extern "C"
