// Host cost of a small collective under the reference's calling model: one thread per rank, each rank with a stream of
// its own, every call blocking until the group is complete (HcclAmdSetParam "blocking_arrive" = "1"; the reference runs a
// process per rank, framework/op_base/src/op_base.cc:210-218), against one thread that drives all ranks on one stream.
// Prints one line per case: microseconds per all-reduce of 8 KiB per rank, 2000 back to back.  Exit code 0 unless a call fails.
#include <hip/hip_runtime_api.h>
#include <atomic>
#include <chrono>
#include <cstdio>
#include <thread>
#include <vector>
#include "hccl/hccl.h"
#include "hccl/hccl_amd_ext.h"
#define CK(x) do { auto e_ = (x); if (e_ != 0) { printf("ERR %s = %d line %d\n", #x, int(e_), __LINE__); exit(1); } } while (0)
int main()
{
    for (uint32_t p : {8u, 16u}) {
        for (int blocking = 1; blocking >= 0; blocking--) {
            std::vector<HcclComm> comms(p);
            std::vector<int32_t> devs(p);
            for (uint32_t r = 0; r < p; r++) devs[r] = int32_t(r);
            CK(HcclCommInitAll(p, devs.data(), comms.data()));
            CK(HcclAmdSetParam(comms[0], "blocking_arrive", blocking ? "1" : "0"));
            const uint64_t n = 2048;
            std::vector<void *> send(p), recv(p);
            std::vector<hipStream_t> streams(p);
            for (uint32_t r = 0; r < p; r++) { CK(hipMalloc(&send[r], n * 4)); CK(hipMalloc(&recv[r], n * 4)); CK(hipMemset(send[r], 0, n * 4)); CK(hipStreamCreateWithFlags(&streams[r], hipStreamNonBlocking)); }
            const int iters = 2000;
            double us = 0, hostUs = 0;
            if (blocking) {
                std::vector<std::thread> ts;
                std::atomic<int> ready{0};
                auto t0 = std::chrono::steady_clock::now();
                for (uint32_t r = 0; r < p; r++) {
                    ts.emplace_back([&, r] {
                        for (int it = 0; it < iters; it++) {
                            CK(HcclAllReduce(send[r], recv[r], n, HCCL_DATA_TYPE_FP32, HCCL_REDUCE_SUM, comms[r], streams[r]));
                        }
                        if (r == 0) hostUs = std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count() / iters;
                        CK(hipStreamSynchronize(streams[r]));
                    });
                }
                for (auto &t : ts) t.join();
                us = std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count() / iters;
            } else {
                auto t0 = std::chrono::steady_clock::now();
                for (int it = 0; it < iters; it++) {
                    for (uint32_t r = 0; r < p; r++) {
                        CK(HcclAllReduce(send[r], recv[r], n, HCCL_DATA_TYPE_FP32, HCCL_REDUCE_SUM, comms[r], streams[0]));
                    }
                }
                CK(hipStreamSynchronize(streams[0]));
                us = std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count() / iters;
            }
            printf("p=%2u %s: %.1f us per all-reduce of 8 KiB (host loop alone %.1f)\n", p, blocking ? "one thread per rank, own streams, blocking_arrive" : "one thread, one stream", us, hostUs);
            fflush(stdout);
            for (uint32_t r = 0; r < p; r++) { (void)hipFree(send[r]); (void)hipFree(recv[r]); (void)hipStreamDestroy(streams[r]); }
            for (uint32_t r = 0; r < p; r++) CK(HcclCommDestroy(comms[r]));
        }
    }
    return 0;
}
