/* HCCL C API, as served by the MI355X data-path library (libhccl.so).
 *
 * Every prototype below has the same name, argument list and meaning as the declaration in the
 * reference header inc/hccl/hccl.h (cited per entry as "decl"), and replaces the definition in
 * src/domain/collective_communication/framework/op_base/src/op_base.cc (cited as "impl").
 * Binaries written against the reference header link unchanged; the value passed as aclrtStream
 * is a hipStream_t.
 *
 * Rank model on one GPU: a communicator group created by HcclCommInitAll has p ranks that all
 * live on the same device.  A collective takes effect once every rank of the group has made the
 * matching call; each call returns immediately, the last one to arrive enqueues the work on its
 * stream and orders every other rank's stream after it.
 */
#ifndef HCCL_H_
#define HCCL_H_

#include <hccl/hccl_types.h>
#include <acl/acl.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- hot path: the four collectives --------------------------------------------------------- */

/* recvBuf[i] = reduce over ranks of sendBuf[i], i < count.  In-place (sendBuf == recvBuf) allowed.
 * count == 0 succeeds as a no-op before any pointer check.
 * decl inc/hccl/hccl.h:131, impl op_base.cc:1268. */
extern HcclResult HcclAllReduce(void *sendBuf, void *recvBuf, uint64_t count, HcclDataType dataType,
    HcclReduceOp op, HcclComm comm, aclrtStream stream);

/* sendBuf holds p * recvCount elements; rank r receives the reduction of slice r.
 * decl inc/hccl/hccl.h:162, impl op_base.cc:1506. */
extern HcclResult HcclReduceScatter(void *sendBuf, void *recvBuf, uint64_t recvCount, HcclDataType dataType,
    HcclReduceOp op, HcclComm comm, aclrtStream stream);

/* recvBuf holds p * sendCount elements; block j is rank j's sendBuf.
 * decl inc/hccl/hccl.h:211, impl op_base.cc:1796. */
extern HcclResult HcclAllGather(void *sendBuf, void *recvBuf, uint64_t sendCount, HcclDataType dataType,
    HcclComm comm, aclrtStream stream);

/* sendCounts/sdispls/recvCounts/rdispls are HOST arrays of p uint64_t, in elements, read during
 * the call.  Rank i's sendBuf[sdispls[j] .. +sendCounts[j]) lands in rank j's
 * recvBuf[rdispls_j[i] ..).  sendCounts_i[j] must equal recvCounts_j[i].
 * decl inc/hccl/hccl.h:306, impl op_base.cc:2520. */
extern HcclResult HcclAlltoAllV(const void *sendBuf, const void *sendCounts, const void *sdispls, HcclDataType sendType,
    const void *recvBuf, const void *recvCounts, const void *rdispls, HcclDataType recvType,
    HcclComm comm, aclrtStream stream);

/* ---- siblings that run through the same kernels --------------------------------------------- */

/* decl inc/hccl/hccl.h:325, impl op_base.cc:2422. */
extern HcclResult HcclAlltoAll(const void *sendBuf, uint64_t sendCount, HcclDataType sendType,
    const void *recvBuf, uint64_t recvCount, HcclDataType recvType, HcclComm comm, aclrtStream stream);

/* sendCountMatrix: host array of p x p uint64_t, identical on every rank; entry [i * p + j] is the
 * number of elements rank i sends to rank j.  Blocks lie back to back in both buffers.  Not in the
 * reference's public header: declared in its framework header
 * src/domain/collective_communication/framework/op_base/src/op_base.h:59, impl op_base.cc:2633. */
extern HcclResult HcclAlltoAllVC(const void *sendBuf, const void *sendCountMatrix, HcclDataType sendType,
    const void *recvBuf, HcclDataType recvType, HcclComm comm, aclrtStream stream);

/* decl inc/hccl/hccl.h:181, impl op_base.cc:1585. */
extern HcclResult HcclReduceScatterV(void *sendBuf, const void *sendCounts, const void *sendDispls,
    void *recvBuf, uint64_t recvCount, HcclDataType dataType, HcclReduceOp op, HcclComm comm, aclrtStream stream);

/* decl inc/hccl/hccl.h:229, impl op_base.cc:1863. */
extern HcclResult HcclAllGatherV(void *sendBuf, uint64_t sendCount, void *recvBuf,
    const void *recvCounts, const void *recvDispls, HcclDataType dataType, HcclComm comm, aclrtStream stream);

/* decl inc/hccl/hccl.h:256, impl op_base.cc:1353. */
extern HcclResult HcclBarrier(HcclComm comm, aclrtStream stream);

/* ---- lifecycle and queries ------------------------------------------------------------------ */

/* One process, ndev ranks.  devices[] are distinct labels; every rank runs on the current HIP
 * device.  decl inc/hccl/hccl.h:364, impl op_base.cc:244. */
extern HcclResult HcclCommInitAll(uint32_t ndev, int32_t *devices, HcclComm *comms);

/* decl inc/hccl/hccl.h:353, impl op_base.cc:2187. */
extern HcclResult HcclCommDestroy(HcclComm comm);

/* decl inc/hccl/hccl.h:239 / :248, impl op_base.cc:2392 / :2407. */
extern HcclResult HcclGetRankSize(HcclComm comm, uint32_t *rankSize);
extern HcclResult HcclGetRankId(HcclComm comm, uint32_t *rank);

/* decl inc/hccl/hccl.h:115, impl op_base.cc:845. */
extern HcclResult HcclGetCommName(HcclComm comm, char *commName);

/* decl inc/hccl/hccl.h:103-104, impl op_base.cc:1204 / :1245. */
extern HcclResult HcclSetConfig(HcclConfig config, HcclConfigValue configValue);
extern HcclResult HcclGetConfig(HcclConfig config, HcclConfigValue *configValue);

/* decl inc/hccl/hccl.h:371, impl op_base.cc:3085. */
extern HcclResult HcclGetCommAsyncError(HcclComm comm, HcclResult *asyncError);

/* decl inc/hccl/hccl.h:377, impl op_base.cc:3103. */
extern const char *HcclGetErrorString(HcclResult code);

/* decl inc/hccl/hccl.h:391, impl op_base.cc:3567. */
extern uint32_t HcclGetCommConfigCapability();

/* decl inc/hccl/hccl.h:430 / :436, impl op_base.cc:3541 / :3554. */
extern HcclResult HcclCommSuspend(HcclComm comm);
extern HcclResult HcclCommResume(HcclComm comm);

/* Fills the size/magic/version header and the "not set" defaults
 * (same bytes as the reference inline at inc/hccl/hccl.h:397-424). */
inline void HcclCommConfigInit(HcclCommConfig *config)
{
    if (config == nullptr) {
        return;
    }
    struct Header {
        size_t size;
        uint32_t magicWord;
        uint32_t version;
        uint64_t reserved;
    };
    Header *h = reinterpret_cast<Header *>(config);
    h->size = sizeof(HcclCommConfig);
    h->magicWord = HCCL_COMM_CONFIG_MAGIC_WORD;
    h->version = HCCL_COMM_CONFIG_VERSION;
    h->reserved = 0;
    config->hcclBufferSize = HCCL_COMM_BUFFSIZE_CONFIG_NOT_SET;
    config->hcclDeterministic = HCCL_COMM_DETERMINISTIC_CONFIG_NOT_SET;
    config->hcclCommName[0] = '\0';
    config->hcclUdi[0] = '\0';
    config->hcclOpExpansionMode = HCCL_COMM_DEFAULT_OP_EXPANSION_MODE;
    config->hcclRdmaTrafficClass = HCCL_COMM_TRAFFIC_CLASS_CONFIG_NOT_SET;
    config->hcclRdmaServiceLevel = HCCL_COMM_SERVICE_LEVEL_CONFIG_NOT_SET;
}

/* ---- rooted collectives and point to point --------------------------------------------------------- */

/* Ring broadcast: buf is the source on the root, the destination elsewhere.
 * decl inc/hccl/hccl.h:146, impl op_base.cc:1433. */
extern HcclResult HcclBroadcast(void *buf, uint64_t count, HcclDataType dataType, uint32_t root, HcclComm comm,
    aclrtStream stream);
/* Ring reduce towards the root; recvBuf is written on the root only.
 * decl inc/hccl/hccl.h:343, impl op_base.cc:2737. */
extern HcclResult HcclReduce(void *sendBuf, void *recvBuf, uint64_t count, HcclDataType dataType,
    HcclReduceOp op, uint32_t root, HcclComm comm, aclrtStream stream);
/* The root's sendBuf holds p blocks of recvCount elements; rank i receives block i (sendBuf may be
 * null elsewhere).  decl inc/hccl/hccl.h:196, impl op_base.cc:1720. */
extern HcclResult HcclScatter(void *sendBuf, void *recvBuf, uint64_t recvCount, HcclDataType dataType, uint32_t root,
    HcclComm comm, aclrtStream stream);
/* A send completes with the matching receive of the destination rank (first in, first out per pair
 * of ranks); counts and types must agree.  decl inc/hccl/hccl.h:270 / :284 / :386,
 * impl op_base.cc:1974 / :2056 / :3428. */
extern HcclResult HcclSend(void *sendBuf, uint64_t count, HcclDataType dataType, uint32_t destRank,
    HcclComm comm, aclrtStream stream);
extern HcclResult HcclRecv(void *recvBuf, uint64_t count, HcclDataType dataType, uint32_t srcRank,
    HcclComm comm, aclrtStream stream);
extern HcclResult HcclBatchSendRecv(HcclSendRecvItem *sendRecvInfo, uint32_t itemNum, HcclComm comm,
    aclrtStream stream);

/* ---- communicators assembled rank by rank ---------------------------------------------------------- */

/* HcclGetRootInfo makes a token; nRanks calls of HcclCommInitRootInfo[Config] with that token, one
 * per rank and all from this process, form one group on the current GPU.  The Config variant reads
 * hcclBufferSize (MiB), hcclDeterministic and hcclCommName from a struct prepared with
 * HcclCommConfigInit.  decl inc/hccl/hccl.h:67 / :79 / :92, impl op_base.cc:794 / :1111 / :1192. */
extern HcclResult HcclGetRootInfo(HcclRootInfo *rootInfo);
extern HcclResult HcclCommInitRootInfo(uint32_t nRanks, const HcclRootInfo *rootInfo, uint32_t rank, HcclComm *comm);
extern HcclResult HcclCommInitRootInfoConfig(uint32_t nRanks, const HcclRootInfo *rootInfo, uint32_t rank,
    const HcclCommConfig *config, HcclComm *comm);
/* Sub-communicator over the ranks rankIds[0..rankNum) of an existing one; every member calls with
 * its position subCommRankId.  decl inc/hccl/hccl.h:58, impl op_base.cc:730. */
extern HcclResult HcclCreateSubCommConfig(HcclComm *comm, uint32_t rankNum, uint32_t *rankIds,
    uint64_t subCommId, uint32_t subCommRankId, HcclCommConfig *config, HcclComm *subComm);

/* Communicator from a rank table: clusterInfo is the path of the JSON file ("server_list" of servers with their
 * "device" entries "device_id" / "rank_id"; addresses are ignored).  Every rank of the table makes this call
 * from this process; the group lives on the current GPU.  Servers must hold equally many ranks, numbered
 * consecutively server by server; with more than one server the all-reduce runs the two-level schedule
 * (mesh inside a server, ring or halving-doubling between servers).
 * decl inc/hccl/hccl.h:30 / :42, impl op_base.cc:465 / :567. */
extern HcclResult HcclCommInitClusterInfo(const char *clusterInfo, uint32_t rank, HcclComm *comm);
extern HcclResult HcclCommInitClusterInfoConfig(const char *clusterInfo, uint32_t rank,
    HcclCommConfig *config, HcclComm *comm);

/* ---- declared so existing binaries link; outside the single-GPU data path ------------------- */
/* Virtual-memory registration concerns the Ascend memory manager; each returns HCCL_E_NOT_SUPPORT
 * after the reference's own null-pointer checks.  decl inc/hccl/hccl.h:446-471. */
extern HcclResult HcclCommSetMemoryRange(HcclComm comm, void *baseVirPtr, size_t size, size_t alignment,
    uint64_t flags);
extern HcclResult HcclCommUnsetMemoryRange(HcclComm comm, void *baseVirPtr);
extern HcclResult HcclCommActivateCommMemory(HcclComm comm, void *virPtr, size_t size, size_t offset,
    aclrtDrvMemHandle handle, uint64_t flags);
extern HcclResult HcclCommDeactivateCommMemory(HcclComm comm, void *virPtr);

#ifdef __cplusplus
}
#endif
#endif /* HCCL_H_ */
