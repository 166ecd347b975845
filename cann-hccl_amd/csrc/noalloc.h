// Workspace of the entry point that allocates nothing (see noalloc.hip).
#pragma once
#include <hip/hip_runtime_api.h>

#include <cstddef>
#include <cstdint>

namespace hcclamd {

constexpr size_t kNoAllocTableBytes = size_t(256) << 10;   // descriptor tables of one collective
constexpr size_t kNoAllocDataBytes = size_t(32) << 20;     // partial results, shared by all ranks of the group
constexpr size_t kNoAllocUploadBytes = 3072;               // table bytes per upload launch (kernel-argument space)

// Address of the workspace on `device`, which must be the current device.  The first call per device
// looks the symbol up; later calls return the kept pointer.
hipError_t NoAllocWorkspace(int device, void **base);

// Calls on one GPU share that GPU's workspace.  NoAllocBegin, called before a call's first launch on `stream`, makes the
// stream wait for the previous call's work when that went to another stream (an event created with the workspace: nothing
// is allocated here); NoAllocEnd, after the call's last launch, marks the stream as the workspace's latest user.  Both
// do nothing while `stream` is being captured: a graph's replays are the caller's to order.
hipError_t NoAllocBegin(int device, hipStream_t stream);
hipError_t NoAllocEnd(int device, hipStream_t stream);

// Queues on `stream` the launches that write hostBytes[0, bytes) to dst (device memory, 16-byte aligned; the
// copy is rounded up to a multiple of 16 bytes).  The host bytes are consumed before the call returns.
// Also used for the small tables of ordinary collectives: unlike a host-to-device copy it never waits.
hipError_t UploadThroughKernelArgs(void *dst, const void *hostBytes, size_t bytes, hipStream_t stream);
// The same for bytes in pinned host memory (rounded up to 16): one launch that reads them from there.
hipError_t UploadFromPinned(void *dst, const void *pinnedHost, size_t bytes, hipStream_t stream);

}  // namespace hcclamd
