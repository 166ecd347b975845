// Communicators assembled rank by rank, split, or read from a rank table; and the entry points that exist for link
// compatibility only.
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
