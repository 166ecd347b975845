/* Minimal stand-in for the Ascend runtime header that hccl.h pulls in.
 * The HCCL C API only needs two opaque handle types from it
 * (reference: inc/hccl/hccl.h:15 includes <acl/acl.h>; aclrtStream is the last argument of every
 * collective, aclrtDrvMemHandle appears in HcclCommActivateCommMemory, inc/hccl/hccl.h:464).
 * On MI355X the value carried in an aclrtStream is a hipStream_t. */
#ifndef HCCL_AMD_ACL_SHIM_H_
#define HCCL_AMD_ACL_SHIM_H_
#include <stddef.h>
#include <stdint.h>
typedef void *aclrtStream;        /* carries a hipStream_t */
typedef void *aclrtDrvMemHandle;  /* unused on this platform */
#endif
