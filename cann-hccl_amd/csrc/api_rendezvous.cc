// Behind the C ABI: argument checks (framework/common/src/param_check.cc), settings read from the environment and from
// HcclCommConfig, the registry of groups, and the rendezvous of the ranks' calls -- a rank arrives, the last one issues
// the collective; sends meet their receives.
#include <chrono>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <map>
#include <set>
#include <sstream>
#include <string>
#include <vector>

#include "api_internal.h"
#include "ranktable.h"

namespace hcclamd {
namespace api {

std::mutex g_registryMutex;
std::set<Group *> g_groups;
int g_deterministic = -1;

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
    const uint64_t *sdispls, const uint64_t *recvCounts, const uint64_t *rdispls, const uint64_t *vCounts,
    const uint64_t *vDispls)
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

}  // namespace api
}  // namespace hcclamd
