// Instantiates the kernels for one HcclDataType (selected with -DHCCL_DT=<enum value>), so that the
// twelve element types build in parallel, plus the byte-wise copy variants (-DHCCL_DT=255).
#include "kernels_team.h"

namespace hcclamd {

#if HCCL_DT == 0
using DT = int8_t;
#define HCCL_DT_NAME int8
#elif HCCL_DT == 1
using DT = int16_t;
#define HCCL_DT_NAME int16
#elif HCCL_DT == 2
using DT = int32_t;
#define HCCL_DT_NAME int32
#elif HCCL_DT == 3
using DT = HalfBits;
#define HCCL_DT_NAME fp16
#elif HCCL_DT == 4
using DT = float;
#define HCCL_DT_NAME fp32
#elif HCCL_DT == 5
using DT = int64_t;
#define HCCL_DT_NAME int64
#elif HCCL_DT == 6
using DT = uint64_t;
#define HCCL_DT_NAME uint64
#elif HCCL_DT == 7
using DT = uint8_t;
#define HCCL_DT_NAME uint8
#elif HCCL_DT == 8
using DT = uint16_t;
#define HCCL_DT_NAME uint16
#elif HCCL_DT == 9
using DT = uint32_t;
#define HCCL_DT_NAME uint32
#elif HCCL_DT == 10
using DT = double;
#define HCCL_DT_NAME fp64
#elif HCCL_DT == 11
using DT = Bf16Bits;
#define HCCL_DT_NAME bf16
#elif HCCL_DT == 255
using DT = uint8_t;
#define HCCL_DT_NAME bytes
#else
#error "HCCL_DT must name a supported HcclDataType"
#endif

#define HCCL_CAT2(a, b) a##b
#define HCCL_CAT(a, b) HCCL_CAT2(a, b)

#if HCCL_DT == 255
// pure data movement: the step kernel's copy path and the copy kernel
extern const void *const HCCL_CAT(kKernels_, HCCL_DT_NAME)[4] = {
    reinterpret_cast<const void *>(&StepKernel<DT, ROP_SUM>),
    reinterpret_cast<const void *>(&CopyKernel<0>),
    reinterpret_cast<const void *>(&GatherKernel<0>),
    reinterpret_cast<const void *>(&TeamCopyKernel<0>),
};
#else
#define HCCL_ROW(OP)                                                     \
    {                                                                    \
        reinterpret_cast<const void *>(&StepKernel<DT, OP>),             \
        reinterpret_cast<const void *>(&ChainKernel<DT, OP>),            \
        reinterpret_cast<const void *>(&TreeKernel<DT, OP>),             \
        reinterpret_cast<const void *>(&StackKernel<DT, OP>),            \
        reinterpret_cast<const void *>(&TeamChainKernel<DT, OP>),        \
        reinterpret_cast<const void *>(&TeamTreeKernel<DT, OP>),         \
        reinterpret_cast<const void *>(&TeamStackKernel<DT, OP>),        \
    }
extern const void *const HCCL_CAT(kKernels_, HCCL_DT_NAME)[4][KK_COUNT] = {
    HCCL_ROW(ROP_SUM), HCCL_ROW(ROP_PROD), HCCL_ROW(ROP_MAX), HCCL_ROW(ROP_MIN),
};
#endif

}  // namespace hcclamd
