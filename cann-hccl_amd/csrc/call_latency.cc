// What a compiled caller pays for small collectives: 8 simulated ranks, fp32 sum all-reduce of 8 KiB to
// 4 MiB per rank through the C ABI, timed three ways per size:
//   issue    host time per collective to make the 8 calls (the last one launches), nothing waited for
//   device   time per collective with collectives queued back to back (HIP events on the stream)
//   round    one collective issued and waited for with hipStreamSynchronize
//
//     cann-hccl_amd/lib/call_latency [fuse: 1 (default) | 0]
#include <hccl/hccl.h>
#include <hccl/hccl_amd_ext.h>
#include <hip/hip_runtime_api.h>

#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <vector>

#define CHECK(call)                                                                   \
    do {                                                                              \
        if ((call) != 0) {                                                            \
            std::printf("call_latency: %s failed (%s:%d)\n", #call, __FILE__, __LINE__); \
            std::exit(1);                                                             \
        }                                                                             \
    } while (0)

int main(int argc, char **argv)
{
    const uint32_t p = 8;
    int32_t devices[p];
    for (uint32_t i = 0; i < p; i++) {
        devices[i] = static_cast<int32_t>(i);
    }
    HcclComm comms[p];
    CHECK(HcclCommInitAll(p, devices, comms));
    const char *fuse = argc > 1 ? argv[1] : "1";
    CHECK(HcclAmdSetParam(comms[0], "fuse", fuse));
    hipStream_t stream;
    CHECK(hipStreamCreate(&stream));
    const size_t maxCount = size_t(1) << 20;
    std::vector<float *> send(p), recv(p);
    for (uint32_t r = 0; r < p; r++) {
        CHECK(hipMalloc(reinterpret_cast<void **>(&send[r]), maxCount * sizeof(float)));
        CHECK(hipMalloc(reinterpret_cast<void **>(&recv[r]), maxCount * sizeof(float)));
        CHECK(hipMemset(send[r], 0, maxCount * sizeof(float)));
    }
    hipEvent_t a, b;
    CHECK(hipEventCreate(&a));
    CHECK(hipEventCreate(&b));
    auto collective = [&](size_t n) {
        for (uint32_t r = 0; r < p; r++) {
            CHECK(HcclAllReduce(send[r], recv[r], n, HCCL_DATA_TYPE_FP32, HCCL_REDUCE_SUM, comms[r], stream));
        }
    };
    using clock = std::chrono::steady_clock;
    auto us = [](clock::time_point t0, clock::time_point t1) { return std::chrono::duration<double, std::micro>(t1 - t0).count(); };
    std::printf("8-rank fp32 all-reduce through the C ABI, %s; microseconds per collective\n",
        fuse[0] == '0' ? "step by step (graph of 14 kernels)" : "fused (one kernel)");
    std::printf("%12s %10s %10s %10s\n", "bytes/rank", "issue", "device", "round");
    for (size_t n = 2048; n <= maxCount; n *= 8) {
        for (int w = 0; w < 20; w++) {
            collective(n);
        }
        CHECK(hipStreamSynchronize(stream));
        const int iters = 1000;
        clock::time_point t0 = clock::now();
        CHECK(hipEventRecord(a, stream));
        for (int k = 0; k < iters; k++) {
            collective(n);
        }
        CHECK(hipEventRecord(b, stream));
        clock::time_point t1 = clock::now();
        CHECK(hipEventSynchronize(b));
        float ms = 0;
        CHECK(hipEventElapsedTime(&ms, a, b));
        double round = 0;
        const int rounds = 200;
        for (int k = 0; k < rounds; k++) {
            clock::time_point u0 = clock::now();
            collective(n);
            CHECK(hipStreamSynchronize(stream));
            round += us(u0, clock::now());
        }
        std::printf("%12zu %10.2f %10.2f %10.2f\n", n * sizeof(float), us(t0, t1) / iters, ms * 1e3 / iters, round / rounds);
    }
    for (uint32_t r = 0; r < p; r++) {
        (void)hipFree(send[r]);
        (void)hipFree(recv[r]);
    }
    for (uint32_t r = 0; r < p; r++) {
        CHECK(HcclCommDestroy(comms[r]));
    }
    return 0;
}
