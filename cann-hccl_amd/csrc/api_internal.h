// What the translation units behind the C ABI share: argument checks, the registry of groups, the rendezvous of the
// ranks' calls (api_rendezvous.cc), used by the collectives (api.cc), the communicator calls (api_comm.cc) and the
// extension calls (api_ext.cc).
#ifndef HCCL_AMD_API_INTERNAL_H
#define HCCL_AMD_API_INTERNAL_H

#include <map>
#include <mutex>
#include <set>
#include <string>

#include "hccl/hccl.h"
#include "hccl/hccl_amd_ext.h"
#include "log.h"
#include "runtime.h"

namespace hcclamd {
namespace api {

constexpr uint64_t kSysMaxCount = 0x7FFFFFFFFull;   // largest element count a call may carry

extern std::mutex g_registryMutex;
extern std::set<Group *> g_groups;
extern int g_deterministic;                          // -1: not set through HcclSetConfig
extern std::map<std::string, Group *> g_forming;     // groups that are being assembled rank by rank, by key
extern uint64_t g_rootInfoSerial;

#define CHK_PTR(p)                                              \
    do {                                                        \
        if ((p) == nullptr) {                                   \
            HCCL_LOG_ERROR("%s: %s is null", __func__, #p);     \
            return HCCL_E_PTR;                                  \
        }                                                       \
    } while (0)

struct InUse {
    Comm *c;
    explicit InUse(Comm *comm) : c(comm) { c->inUse = true; }
    ~InUse() { c->inUse = false; }
};

Comm *AsComm(HcclComm h);
bool DataTypeKnown(HcclDataType dt);
HcclResult CheckOpParam(const char *fn, uint64_t count, HcclDataType dt, const void *stream);
HcclResult CheckReduce(const char *fn, HcclDataType dt, HcclReduceOp op);
uint32_t ElemSize(int dt);
void ApplyEnv(GroupConfig *cfg);
HcclResult LoadCommConfig(const HcclCommConfig *user, GroupConfig *cfg, std::string *name);
Group *NewGroup(uint32_t nRanks);
// Joins rank `rank` to the group forming under `key` (created on first use).
HcclResult JoinFormingGroup(const std::string &key, uint32_t nRanks, uint32_t rank, const HcclCommConfig *config, HcclComm *out);
// Ends the current rendezvous.  Ranks blocked inside their call wake up and return `result`.
void CancelPending(Group *g, HcclResult result);
// One rank joins the current collective.  The last rank to join issues it.
HcclResult Arrive(Comm *c, const OpSig &sig, void *send, void *recv, hipStream_t stream, const uint64_t *sendCounts,
    const uint64_t *sdispls, const uint64_t *recvCounts, const uint64_t *rdispls, const uint64_t *vCounts = nullptr,
    const uint64_t *vDispls = nullptr);
HcclResult PointToPoint(Comm *c, bool isSend, void *buf, uint64_t count, HcclDataType dataType, uint32_t other,
    hipStream_t stream);

}  // namespace api
}  // namespace hcclamd

#endif
