/* Value types of the HCCL C API as this library implements it on one MI355X.
 *
 * The binary contract is the reference's inc/hccl/hccl_types.h: same enumerator names and numbers
 * (:23-87), same configuration constants and structure layouts (:99-130, :141-153), so that a caller
 * compiled against either header hands over the same integers and the same bytes.  Only the
 * arrangement and the commentary are this library's own. */
#ifndef HCCL_TYPES_H_
#define HCCL_TYPES_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* A communicator is an opaque handle; the library owns what it points to. */
typedef void *HcclComm;

/* ---- element types and operators (reference :58-87) ------------------------------------------ */
/* Sizes in bytes, in enumerator order: 1 2 4 2 4 8 8 1 2 4 8 2 16 1 1 1.  INT128 is accepted for data
 * movement only.  The three 8-bit float formats are named here and refused by every collective with
 * HCCL_E_NOT_SUPPORT, as by the reference (its accepted set:
 * src/domain/collective_communication/framework/common/src/param_check.cc:22-36). */
typedef enum {
    HCCL_DATA_TYPE_INT8 = 0,    HCCL_DATA_TYPE_INT16 = 1,   HCCL_DATA_TYPE_INT32 = 2,    HCCL_DATA_TYPE_FP16 = 3,
    HCCL_DATA_TYPE_FP32 = 4,    HCCL_DATA_TYPE_INT64 = 5,   HCCL_DATA_TYPE_UINT64 = 6,   HCCL_DATA_TYPE_UINT8 = 7,
    HCCL_DATA_TYPE_UINT16 = 8,  HCCL_DATA_TYPE_UINT32 = 9,  HCCL_DATA_TYPE_FP64 = 10,    HCCL_DATA_TYPE_BFP16 = 11,
    HCCL_DATA_TYPE_INT128 = 12, HCCL_DATA_TYPE_HIF8 = 13,   HCCL_DATA_TYPE_FP8E4M3 = 14, HCCL_DATA_TYPE_FP8E5M2 = 15,
    HCCL_DATA_TYPE_RESERVED = 255
} HcclDataType;

typedef enum {
    HCCL_REDUCE_SUM = 0, HCCL_REDUCE_PROD = 1, HCCL_REDUCE_MAX = 2, HCCL_REDUCE_MIN = 3,
    HCCL_REDUCE_RESERVED = 255
} HcclReduceOp;

/* ---- return codes (reference :23-48) ---------------------------------------------------------- */
/* Used by this library: SUCCESS, PARA (bad value), PTR (null pointer), MEMORY, INTERNAL, NOT_SUPPORT,
 * TIMEOUT, RUNTIME (a HIP call failed), AGAIN, SUSPENDING.  The others exist for callers' switches. */
typedef enum {
    HCCL_SUCCESS = 0,
    HCCL_E_PARA = 1, HCCL_E_PTR = 2, HCCL_E_MEMORY = 3, HCCL_E_INTERNAL = 4, HCCL_E_NOT_SUPPORT = 5,
    HCCL_E_NOT_FOUND = 6, HCCL_E_UNAVAIL = 7, HCCL_E_SYSCALL = 8, HCCL_E_TIMEOUT = 9, HCCL_E_OPEN_FILE_FAILURE = 10,
    HCCL_E_TCP_CONNECT = 11, HCCL_E_ROCE_CONNECT = 12, HCCL_E_TCP_TRANSFER = 13, HCCL_E_ROCE_TRANSFER = 14,
    HCCL_E_RUNTIME = 15, HCCL_E_DRV = 16, HCCL_E_PROFILING = 17, HCCL_E_CCE = 18, HCCL_E_NETWORK = 19,
    HCCL_E_AGAIN = 20, HCCL_E_REMOTE = 21, HCCL_E_SUSPENDING = 22,
    HCCL_E_RESERVED
} HcclResult;

/* ---- point to point (reference :141-153) ------------------------------------------------------ */
typedef enum { HCCL_SEND = 0, HCCL_RECV = 1, HCCL_SEND_RECV_RESERVED } HcclSendRecvType;

/* One entry of HcclBatchSendRecv: count elements of dataType at buf, to or from remoteRank. */
typedef struct HcclSendRecvItemDef {
    HcclSendRecvType sendRecvType;
    void *buf;
    uint64_t count;
    HcclDataType dataType;
    uint32_t remoteRank;
} HcclSendRecvItem;

/* ---- process-wide switches, HcclSetConfig / HcclGetConfig (reference :89-97) ------------------ */
typedef enum { HCCL_DETERMINISTIC = 0, HCCL_CONFIG_RESERVED } HcclConfig;

union HcclConfigValue {
    int32_t value;
};

/* ---- communicator assembly and configuration (reference :99-130) ------------------------------ */
const uint32_t HCCL_ROOT_INFO_BYTES = 4108;   /* size of the token HcclGetRootInfo hands to the other ranks */
const uint32_t COMM_NAME_MAX_LENGTH = 128;
const uint32_t UDI_MAX_LENGTH = 128;

typedef struct HcclRootInfoDef {
    char internal[HCCL_ROOT_INFO_BYTES];
} HcclRootInfo;

/* HcclCommConfig starts with 24 bytes of {size, magic word, version, reserved} that
 * HcclCommConfigInit fills in; the library copies min(size, its own struct size) bytes, so older and
 * newer callers both work.  hcclBufferSize is in MiB; the *_NOT_SET values mean "take the default". */
const uint32_t HCCL_COMM_CONFIG_INFO_BYTES = 24;
const uint32_t HCCL_COMM_CONFIG_MAGIC_WORD = 0xf0f0f0f0;
const uint32_t HCCL_COMM_CONFIG_VERSION = 5;
const uint32_t HCCL_COMM_DEFAULT_BUFFSIZE = 200;
const uint32_t HCCL_COMM_DEFAULT_DETERMINISTIC = 0;
const uint32_t HCCL_COMM_DEFAULT_OP_EXPANSION_MODE = 0;
const uint32_t HCCL_COMM_BUFFSIZE_CONFIG_NOT_SET = 0xffffffff;
const uint32_t HCCL_COMM_DETERMINISTIC_CONFIG_NOT_SET = 0xffffffff;
const uint32_t HCCL_COMM_TRAFFIC_CLASS_CONFIG_NOT_SET = 0xffffffff;
const uint32_t HCCL_COMM_SERVICE_LEVEL_CONFIG_NOT_SET = 0xffffffff;

typedef struct HcclCommConfigDef {
    char reserved[HCCL_COMM_CONFIG_INFO_BYTES];
    uint32_t hcclBufferSize;
    uint32_t hcclDeterministic;
    char hcclCommName[COMM_NAME_MAX_LENGTH];
    char hcclUdi[UDI_MAX_LENGTH];
    uint32_t hcclOpExpansionMode;      /* accepted, not used: there is one execution mode here */
    uint32_t hcclRdmaTrafficClass;     /* accepted, not used: no network */
    uint32_t hcclRdmaServiceLevel;     /* accepted, not used: no network */
} HcclCommConfig;

/* Configuration features; HcclGetCommConfigCapability returns the first value a library does not know. */
typedef enum {
    HCCL_COMM_CONFIG_BUFFER_SIZE = 0, HCCL_COMM_CONFIG_DETERMINISTIC = 1, HCCL_COMM_CONFIG_COMM_NAME = 2,
    HCCL_COMM_CONFIG_OP_EXPANSION_MODE = 3, HCCL_COMM_CONFIG_SUPPORT_INIT_BY_ENV = 4,
    HCCL_COMM_CONFIG_RESERVED
} HcclCommConfigCapability;

#ifdef __cplusplus
}
#endif
#endif /* HCCL_TYPES_H_ */
