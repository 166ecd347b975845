// What this GPU's memory system delivers for the traffic shapes of the collectives: n source streams
// read, m destination streams written, 256 MiB each (far beyond the caches), plain grid-stride loops of
// non-temporal 128-bit accesses -- no descriptors, no arithmetic to speak of.  The numbers bound what
// the library's kernels can reach for the same read : write mix.
//
//     cann-hccl_amd/lib/hbm_probe [MiB per stream, default 256]
//
// Prints one line per shape: the best rate over the launch widths tried, in GB/s of bytes moved.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

typedef uint32_t V4 __attribute__((ext_vector_type(4)));

#define CHECK(call)                                                                           \
    do {                                                                                      \
        hipError_t e_ = (call);                                                               \
        if (e_ != hipSuccess) {                                                               \
            std::printf("hbm_probe: %s failed: %s\n", #call, hipGetErrorString(e_));          \
            std::exit(1);                                                                     \
        }                                                                                     \
    } while (0)

struct Streams {
    const V4 *src[8];
    V4 *dst[8];
};

constexpr int kVec = 4;   // vectors per lane per iteration

// NS sources are read and xor-ed, the result goes to ND destinations.  With ND == 0 the result is
// stored only if it equals a value the zero-filled sources cannot produce, which keeps the loads alive.
template <int NS, int ND>
__global__ void __launch_bounds__(256) Probe(Streams s, uint64_t nvec, uint32_t never)
{
    const uint64_t stride = uint64_t(gridDim.x) * 256 * kVec;
    for (uint64_t base = uint64_t(blockIdx.x) * 256 * kVec; base < nvec; base += stride) {
        V4 acc[kVec];
#pragma unroll
        for (int u = 0; u < kVec; u++) {
            acc[u] = V4{never, 1, 2, 3};
        }
#pragma unroll
        for (int j = 0; j < NS; j++) {
#pragma unroll
            for (int u = 0; u < kVec; u++) {
                acc[u] ^= __builtin_nontemporal_load(s.src[j] + base + u * 256 + threadIdx.x);
            }
        }
        if (ND == 0) {
#pragma unroll
            for (int u = 0; u < kVec; u++) {
                if (acc[u].y == 0x7fffffffu) {
                    s.dst[0][base + u * 256 + threadIdx.x] = acc[u];
                }
            }
        }
#pragma unroll
        for (int k = 0; k < ND; k++) {
#pragma unroll
            for (int u = 0; u < kVec; u++) {
                __builtin_nontemporal_store(acc[u], s.dst[k] + base + u * 256 + threadIdx.x);
            }
        }
    }
}

template <int NS, int ND>
static double BestRate(const Streams &s, uint64_t bytes, int cus)
{
    const uint64_t nvec = bytes / 16;
    hipEvent_t a, b;
    CHECK(hipEventCreate(&a));
    CHECK(hipEventCreate(&b));
    double best = 0;
    for (int perCu : {1, 2, 4, 8}) {
        const int grid = cus * perCu, iters = 10;
        for (int i = 0; i < 2; i++) {
            hipLaunchKernelGGL((Probe<NS, ND>), dim3(grid), dim3(256), 0, 0, s, nvec, 12345u);
        }
        CHECK(hipDeviceSynchronize());
        CHECK(hipEventRecord(a));
        for (int i = 0; i < iters; i++) {
            hipLaunchKernelGGL((Probe<NS, ND>), dim3(grid), dim3(256), 0, 0, s, nvec, 12345u);
        }
        CHECK(hipEventRecord(b));
        CHECK(hipEventSynchronize(b));
        float ms = 0;
        CHECK(hipEventElapsedTime(&ms, a, b));
        double rate = double(NS + ND) * double(bytes) * iters / (ms * 1e-3) / 1e9;
        best = rate > best ? rate : best;
    }
    CHECK(hipEventDestroy(a));
    CHECK(hipEventDestroy(b));
    return best;
}

int main(int argc, char **argv)
{
    const uint64_t mib = argc > 1 ? std::strtoull(argv[1], nullptr, 10) : 256;
    const uint64_t bytes = (mib << 20) / 4096 * 4096;
    if (bytes == 0 || mib > 2048) {
        std::printf("hbm_probe: size must be 1 .. 2048 MiB per stream\n");
        return 1;
    }
    hipDeviceProp_t prop;
    CHECK(hipGetDeviceProperties(&prop, 0));
    const int cus = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
    Streams s;
    std::vector<void *> bufs;
    for (int i = 0; i < 16; i++) {
        void *p = nullptr;
        CHECK(hipMalloc(&p, bytes));
        CHECK(hipMemset(p, 0, bytes));
        bufs.push_back(p);
        if (i < 8) {
            s.src[i] = static_cast<const V4 *>(p);
        } else {
            s.dst[i - 8] = static_cast<V4 *>(p);
        }
    }
    CHECK(hipDeviceSynchronize());
    std::printf("%s, %d CUs, %llu MiB per stream; GB/s of bytes moved (read + written), best of 1/2/4/8 workgroups per CU\n",
        prop.name[0] ? prop.name : prop.gcnArchName, cus, static_cast<unsigned long long>(mib));
    std::printf("  8 read  : 0 written   %8.1f   (what the reduce side of any collective could reach)\n", BestRate<8, 0>(s, bytes, cus));
    std::printf("  8 read  : 1 written   %8.1f   (fused reduce-scatter / reduce)\n", BestRate<8, 1>(s, bytes, cus));
    std::printf("  2 read  : 1 written   %8.1f   (one reduce step)\n", BestRate<2, 1>(s, bytes, cus));
    std::printf("  1 read  : 1 written   %8.1f   (one copy step)\n", BestRate<1, 1>(s, bytes, cus));
    std::printf("  8 read  : 8 written   %8.1f   (fused all-reduce)\n", BestRate<8, 8>(s, bytes, cus));
    std::printf("  1 read  : 8 written   %8.1f   (fused all-gather / broadcast)\n", BestRate<1, 8>(s, bytes, cus));
    std::printf("  0 read  : 8 written   %8.1f\n", BestRate<0, 8>(s, bytes, cus));
    {
        hipEvent_t a, b;
        CHECK(hipEventCreate(&a));
        CHECK(hipEventCreate(&b));
        CHECK(hipMemcpyAsync(bufs[8], bufs[0], bytes, hipMemcpyDeviceToDevice, nullptr));
        CHECK(hipDeviceSynchronize());
        CHECK(hipEventRecord(a));
        for (int i = 0; i < 10; i++) {
            CHECK(hipMemcpyAsync(bufs[8], bufs[0], bytes, hipMemcpyDeviceToDevice, nullptr));
        }
        CHECK(hipEventRecord(b));
        CHECK(hipEventSynchronize(b));
        float ms = 0;
        CHECK(hipEventElapsedTime(&ms, a, b));
        std::printf("  hipMemcpyAsync device to device %8.1f\n", 2.0 * double(bytes) * 10 / (ms * 1e-3) / 1e9);
    }
    for (void *p : bufs) {
        (void)hipFree(p);
    }
    return 0;
}
