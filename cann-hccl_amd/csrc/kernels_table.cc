// Lookup of the per-type kernel tables built from kernels_dt.hip.
#include "kernels.h"

namespace hcclamd {

#define HCCL_DECL(name) extern const void *const kKernels_##name[4][KK_COUNT];
HCCL_DECL(int8) HCCL_DECL(int16) HCCL_DECL(int32) HCCL_DECL(fp16) HCCL_DECL(fp32) HCCL_DECL(int64)
HCCL_DECL(uint64) HCCL_DECL(uint8) HCCL_DECL(uint16) HCCL_DECL(uint32) HCCL_DECL(fp64) HCCL_DECL(bf16)
extern const void *const kKernels_bytes[4];

const void *LookupKernel(int dt, int op, KernelKind kind)
{
    if (op < 0 || op > 3 || kind < 0 || kind >= KK_COUNT) {
        return nullptr;
    }
    switch (dt) {
        case 0: return kKernels_int8[op][kind];
        case 1: return kKernels_int16[op][kind];
        case 2: return kKernels_int32[op][kind];
        case 3: return kKernels_fp16[op][kind];
        case 4: return kKernels_fp32[op][kind];
        case 5: return kKernels_int64[op][kind];
        case 6: return kKernels_uint64[op][kind];
        case 7: return kKernels_uint8[op][kind];
        case 8: return kKernels_uint16[op][kind];
        case 9: return kKernels_uint32[op][kind];
        case 10: return kKernels_fp64[op][kind];
        case 11: return kKernels_bf16[op][kind];
        default: return nullptr;
    }
}

const void *LookupCopyKernel(KernelKind kind)
{
    if (kind == KK_STEP) {
        return kKernels_bytes[0];
    }
    if (kind == KK_CHAIN) {
        return kKernels_bytes[1];
    }
    if (kind == KK_GATHER) {
        return kKernels_bytes[2];
    }
    if (kind == KK_TEAM_CHAIN) {
        return kKernels_bytes[3];
    }
    return nullptr;
}

}  // namespace hcclamd
