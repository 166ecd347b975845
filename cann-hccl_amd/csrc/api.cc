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

#include "api_internal.h"
#include "ranktable.h"

using namespace hcclamd;
using namespace hcclamd::api;

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

}  // extern "C"
