// Fixed device workspace for the entry point that allocates nothing (HcclAmdReduceScatterNoAlloc).
//
// The workspace is a file-scope device array: every GPU the library runs on holds one copy of it from
// the moment the code object is loaded until the process ends.  Host code never uses the array's
// name as an address (on the host the name is only a stand-in for the symbol): the address on the
// current device is looked up once with hipGetSymbolAddress and kept per device; everything that
// touches the workspace afterwards -- the upload kernel below, the collective's kernels -- gets that
// pointer as an argument.
#include <hip/hip_runtime.h>

#include <mutex>

#include "noalloc.h"

namespace hcclamd {

namespace {

// [0, kNoAllocTableBytes): descriptor tables of the call in flight; the rest: partial results of the
// step-by-step schedules, one equal share per rank.
static __device__ __align__(256) unsigned char scratch[kNoAllocTableBytes + kNoAllocDataBytes];

constexpr int kMaxDevices = 64;
std::mutex g_lock;
void *g_scratchOnDevice[kMaxDevices] = {};
// the workspace's latest user: an event recorded behind its work, and the stream that work went to
hipEvent_t g_lastUse[kMaxDevices] = {};
hipStream_t g_lastStream[kMaxDevices] = {};
bool g_used[kMaxDevices] = {};

// Table bytes travel as kernel arguments: no host-to-device copy, nothing to stage or allocate, and a
// launch is ordered on the caller's stream like every other kernel of the collective.
typedef uint32_t Word4 __attribute__((ext_vector_type(4)));
struct UploadPiece {
    Word4 words[kNoAllocUploadBytes / 16];
};

__global__ void __launch_bounds__(256) UploadKernel(UploadPiece piece, unsigned char *dst, uint32_t nwords)
{
    typedef Word4 __attribute__((address_space(1))) GlobalWord4;
    for (uint32_t i = threadIdx.x; i < nwords; i += blockDim.x) {
        ((GlobalWord4 *)dst)[i] = piece.words[i];
    }
}

// Table bytes that lie in pinned host memory: the device fetches them itself, as a launch in the stream's order (a copy
// command would hand the stream to a copy engine and back).
__global__ void __launch_bounds__(256) FetchKernel(const unsigned char *__restrict__ pinned, unsigned char *__restrict__ dst,
    uint32_t nwords)
{
    typedef Word4 __attribute__((address_space(1))) GlobalWord4;
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < nwords) {
        ((GlobalWord4 *)dst)[i] = ((const GlobalWord4 *)pinned)[i];
    }
}

}  // namespace

hipError_t UploadFromPinned(void *dst, const void *pinnedHost, size_t bytes, hipStream_t stream)
{
    const uint32_t nwords = uint32_t((bytes + 15) / 16);
    if (nwords == 0) {
        return hipSuccess;
    }
    hipLaunchKernelGGL(FetchKernel, dim3((nwords + 255) / 256), dim3(256), 0, stream,
        static_cast<const unsigned char *>(pinnedHost), static_cast<unsigned char *>(dst), nwords);
    return hipGetLastError();
}

hipError_t NoAllocWorkspace(int device, void **base)
{
    if (device < 0 || device >= kMaxDevices) {
        return hipErrorInvalidDevice;
    }
    std::lock_guard<std::mutex> hold(g_lock);
    if (g_scratchOnDevice[device] == nullptr) {
        int current = -1;
        hipError_t e = hipGetDevice(&current);
        if (e != hipSuccess) {
            return e;
        }
        if (current != device) {
            return hipErrorInvalidDevice;   // the caller makes the device current first: every GPU has its own copy
        }
        void *ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) {
            return e;
        }
        e = hipEventCreateWithFlags(&g_lastUse[device], hipEventDisableTiming);
        if (e != hipSuccess) {
            return e;
        }
        g_scratchOnDevice[device] = ptr;
    }
    *base = g_scratchOnDevice[device];
    return hipSuccess;
}

namespace {

hipError_t Capturing(hipStream_t stream, bool *capturing)
{
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    hipError_t e = hipStreamIsCapturing(stream, &status);
    *capturing = status != hipStreamCaptureStatusNone;
    return e;
}

}  // namespace

hipError_t NoAllocBegin(int device, hipStream_t stream)
{
    if (device < 0 || device >= kMaxDevices) {
        return hipErrorInvalidDevice;
    }
    bool capturing = false;
    hipError_t e = Capturing(stream, &capturing);
    if (e != hipSuccess || capturing) {
        return e;
    }
    std::lock_guard<std::mutex> hold(g_lock);
    if (g_used[device] && g_lastStream[device] != stream) {
        return hipStreamWaitEvent(stream, g_lastUse[device], 0);
    }
    return hipSuccess;
}

hipError_t NoAllocEnd(int device, hipStream_t stream)
{
    if (device < 0 || device >= kMaxDevices) {
        return hipErrorInvalidDevice;
    }
    bool capturing = false;
    hipError_t e = Capturing(stream, &capturing);
    if (e != hipSuccess || capturing) {
        return e;
    }
    std::lock_guard<std::mutex> hold(g_lock);
    e = hipEventRecord(g_lastUse[device], stream);
    if (e == hipSuccess) {
        g_lastStream[device] = stream;
        g_used[device] = true;
    }
    return e;
}

hipError_t UploadThroughKernelArgs(void *dst, const void *hostBytes, size_t bytes, hipStream_t stream)
{
    const unsigned char *from = static_cast<const unsigned char *>(hostBytes);
    unsigned char *to = static_cast<unsigned char *>(dst);
    for (size_t at = 0; at < bytes; at += kNoAllocUploadBytes) {
        const size_t n = bytes - at < kNoAllocUploadBytes ? bytes - at : kNoAllocUploadBytes;
        UploadPiece piece;
        __builtin_memset(&piece, 0, sizeof(piece));
        __builtin_memcpy(&piece, from + at, n);
        hipLaunchKernelGGL(UploadKernel, dim3(1), dim3(256), 0, stream, piece, to + at, uint32_t((n + 15) / 16));
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) {
            return e;
        }
    }
    return hipSuccess;
}

}  // namespace hcclamd
