// A caller written the way an application of the reference library is: it includes <hccl/hccl.h>,
// creates the communicators of one process with HcclCommInitAll, and runs collectives on a stream.
// It is compiled against this repository's include/ (and, where the reference tree is present, against
// the reference's own inc/ with only acl/acl.h taken from here) and linked with libhccl.so.
// Prints ABI_CALLER_OK when every result is right.
#include <hccl/hccl.h>
#include <hip/hip_runtime_api.h>

#include <cstdint>
#include <cstdio>
#include <vector>

#define REQUIRE(cond)                                                             \
    do {                                                                          \
        if (!(cond)) {                                                            \
            std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);         \
            return 1;                                                             \
        }                                                                         \
    } while (0)

int main()
{
    const uint32_t p = 8;
    const uint64_t count = 1000003;
    int32_t devices[p];
    for (uint32_t i = 0; i < p; i++) {
        devices[i] = static_cast<int32_t>(i);
    }
    HcclComm comms[p];
    REQUIRE(HcclCommInitAll(p, devices, comms) == HCCL_SUCCESS);
    uint32_t size = 0, rank = 99;
    REQUIRE(HcclGetRankSize(comms[5], &size) == HCCL_SUCCESS && size == p);
    REQUIRE(HcclGetRankId(comms[5], &rank) == HCCL_SUCCESS && rank == 5);

    hipStream_t stream;
    REQUIRE(hipStreamCreate(&stream) == hipSuccess);
    std::vector<int32_t *> send(p), recv(p);
    std::vector<int32_t> host(count);
    for (uint32_t r = 0; r < p; r++) {
        REQUIRE(hipMalloc(reinterpret_cast<void **>(&send[r]), count * sizeof(int32_t)) == hipSuccess);
        REQUIRE(hipMalloc(reinterpret_cast<void **>(&recv[r]), count * p * sizeof(int32_t)) == hipSuccess);
        for (uint64_t i = 0; i < count; i++) {
            host[i] = static_cast<int32_t>(i * 7 + r * 1000);
        }
        REQUIRE(hipMemcpy(send[r], host.data(), count * sizeof(int32_t), hipMemcpyHostToDevice) == hipSuccess);
    }

    // all-reduce: sum over ranks of (7 i + 1000 r) = 8 * 7 i + 1000 * 28
    for (uint32_t r = 0; r < p; r++) {
        REQUIRE(HcclAllReduce(send[r], recv[r], count, HCCL_DATA_TYPE_INT32, HCCL_REDUCE_SUM, comms[r], stream) == HCCL_SUCCESS);
    }
    REQUIRE(hipStreamSynchronize(stream) == hipSuccess);
    for (uint32_t r = 0; r < p; r++) {
        REQUIRE(hipMemcpy(host.data(), recv[r], count * sizeof(int32_t), hipMemcpyDeviceToHost) == hipSuccess);
        for (uint64_t i = 0; i < count; i++) {
            REQUIRE(host[i] == static_cast<int32_t>(i * 56 + 28000));
        }
    }

    // all-gather: block j of every receive buffer is rank j's send buffer
    for (uint32_t r = 0; r < p; r++) {
        REQUIRE(HcclAllGather(send[r], recv[r], count, HCCL_DATA_TYPE_INT32, comms[r], stream) == HCCL_SUCCESS);
    }
    REQUIRE(hipStreamSynchronize(stream) == hipSuccess);
    std::vector<int32_t> wide(count * p);
    REQUIRE(hipMemcpy(wide.data(), recv[3], count * p * sizeof(int32_t), hipMemcpyDeviceToHost) == hipSuccess);
    for (uint32_t j = 0; j < p; j++) {
        for (uint64_t i = 0; i < count; i += 997) {
            REQUIRE(wide[j * count + i] == static_cast<int32_t>(i * 7 + j * 1000));
        }
    }

    // broadcast from rank 2, in place
    for (uint32_t r = 0; r < p; r++) {
        REQUIRE(HcclBroadcast(send[r], count, HCCL_DATA_TYPE_INT32, 2, comms[r], stream) == HCCL_SUCCESS);
    }
    REQUIRE(hipStreamSynchronize(stream) == hipSuccess);
    REQUIRE(hipMemcpy(host.data(), send[6], count * sizeof(int32_t), hipMemcpyDeviceToHost) == hipSuccess);
    for (uint64_t i = 0; i < count; i += 991) {
        REQUIRE(host[i] == static_cast<int32_t>(i * 7 + 2000));
    }

    // argument checks keep the reference's codes
    REQUIRE(HcclAllReduce(nullptr, recv[0], count, HCCL_DATA_TYPE_INT32, HCCL_REDUCE_SUM, comms[0], stream) == HCCL_E_PTR);
    REQUIRE(HcclAllReduce(nullptr, nullptr, 0, HCCL_DATA_TYPE_INT32, HCCL_REDUCE_SUM, comms[0], stream) == HCCL_SUCCESS);
    HcclCommConfig config;
    HcclCommConfigInit(&config);
    REQUIRE(config.hcclBufferSize == HCCL_COMM_BUFFSIZE_CONFIG_NOT_SET);

    for (uint32_t r = 0; r < p; r++) {
        REQUIRE(HcclCommDestroy(comms[r]) == HCCL_SUCCESS);
        (void)hipFree(send[r]);
        (void)hipFree(recv[r]);
    }
    (void)hipStreamDestroy(stream);
    std::printf("ABI_CALLER_OK\n");
    return 0;
}
