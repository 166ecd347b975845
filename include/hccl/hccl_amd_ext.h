/* Additions of the MI355X library to the HCCL C API.  Nothing here exists in the reference; the
 * entry points let a harness choose the schedule, read back what the last collective moved, and
 * inspect a plan without a GPU.  Plain C ABI, no device types. */
#ifndef HCCL_AMD_EXT_H_
#define HCCL_AMD_EXT_H_

#include <hccl/hccl_types.h>
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Settings of the communicator's whole group.  Keys and values:
 *   "algo"          "ring" | "mesh" | "rhd" | "pairwise" | "star" | "hd_blocks" | "auto"   ("pairwise" only matters to the
 *                                all-to-all family, see "servers"; the other collectives then run their ring schedules;
 *                                the scatter runs the mesh schedule unless "ring" is set; "star" and "hd_blocks" only
 *                                matter to the broadcast, also over several servers: with "star" the root hands every
 *                                rank the whole buffer at once, with "hd_blocks" the buffer spreads by halving-doubling
 *                                over blocks of power-of-two sizes, a binomial tree inside the root's block and then
 *                                from block to block)
 *   "deterministic" "0" | "1"    as HCCL_DETERMINISTIC; with "0" (the default) the mesh reduce phases of
 *                                all-reduce / reduce-scatter run without the piece cut (not for int64, not for products)
 *   "fuse"          "0" | "1"    run the single-pass fused form when the schedule has one
 *   "graph"         "0" | "1"    issue through a HIP graph
 *   "buffsize_mib"  CCL buffer size that sets the chunk plan (default 200, as HCCL_BUFFSIZE);
 *   "buffsize_bytes" the same in bytes (tests of the chunk loop on small inputs)
 *   "align"         slice alignment in bytes (default 128); a collective whose element size does not divide it fails with HCCL_E_PARA
 *   "servers"       number of rank groups for all-reduce, reduce-scatter, all-gather and reduce: with n > 1 the p ranks form n groups of p / n
 *                   consecutive ranks and the two-level schedules run (mesh inside a group, "algo" ring or rhd between;
 *                   with "auto": rhd for 2, 4, 8 or more groups, ring for 3, 5, 6, 7, the reference's default);
 *                   the broadcast then runs scatter / halving-doubling between the groups / all-gather unless "algo" is "ring";
 *                   the scatter then sends a group's blocks round the ring of the ranks at the root's position and hands them out
 *                   inside the group, unless "algo" is "ring";
 *                   the all-to-all family then runs the staged schedule (gather inside a group into a workspace, pairwise
 *                   between the groups) unless "algo" is "pairwise"
 *   "level0"        "mesh" | "ring" | "ring4"   what runs inside a group of the two-level all-reduce / reduce-scatter / all-gather / reduce / broadcast / scatter: the mesh schedule
 *                                (default), one ring in rank order, or -- for groups of 8 ranks, for the all-reduce also with one group --
 *                                the four rings of the 8-device ring topology, each on a quarter of every slice
 *   "nic_ranks"     "all" | list of 1, 2 or 4 ranks, e.g. "0,4"   groups of 8 ranks only: the ranks that own a network port.
 *                                With fewer than 8 the one-level ring all-reduce runs the port-pruned reduce-scatter of the
 *                                reference (the 8 slices form as many chunks as there are ports; all slices of chunk j end
 *                                their ring chain at the j-th listed rank, in ascending rank order), which changes the
 *                                floating-point association of the slices whose chain ends elsewhere.  With several
 *                                groups of 8 ("servers" = ranks / 8, "level0" = "ring4", "algo" = "ring") the list names
 *                                devices of every group, and the reduce-scatter runs the reference's branch for servers
 *                                with fewer ports than devices: all-reduce inside every group, ring reduce-scatter
 *                                between the groups on the listed devices only, then these hand the blocks on inside
 *                                their group; sums are associated inside a group first, then between the groups
 *   "step_stores"   "auto" | "nt" | "ordinary"   store kind of the step-by-step kernels (non-temporal, or write-back
 *                                so that the next phase finds the data in the memory-side cache); "auto" decides per collective
 *   "step_sweep"    "alternate" | "forward"   step-by-step kernels: every other launch walks its data backwards (default),
 *                                or all walk forwards
 *   "fused_stores"  "auto" | "nt" | "ordinary"   store kind of the fused kernels: non-temporal, or write-back, which
 *                                keeps a result of up to 256 MB in the memory-side cache for whoever reads it next; "auto"
 *                                (default): non-temporal, except write-back for pure data movement from one source to four
 *                                or more destinations with more than 512 MB of output (all-gather, broadcast)
 *   "team"          "auto" | "0" | "1"   team form of the fused kernels: the workgroups of one XCD read their tiles together,
 *                                hold the results in LDS and write them together, which this memory system serves faster
 *                                than reads and writes interleaved; "auto" (default): for launches of at least four rounds
 *                                whose items write four or more destinations and touch eight or more buffers (all-reduce,
 *                                all-gather, broadcast); "1": wherever the device allows it; "0": never
 *   "team_tiles"    tiles of 16 KiB a workgroup of a team kernel takes per round, 1 ... 8 ("0", default: 8, fewer when an
 *                                item has more than 8 sources or destinations)
 *   "cache_entries" how many prepared collectives (distinct sizes, buffers, settings) the group keeps (default 1024);
 *                   when full, the library waits for the device once and starts over
 *   "blocks_per_cu" launch width in workgroups per compute unit ("0": chosen per collective)
 *   "launch_cap_mib" fused issue: the items go out in several launches, cut where a launch has moved about this many
 *                                MiB (read and written); "0": one launch per kernel kind; "auto" (default): 512 for the
 *                                collectives whose items hop from buffer to buffer (all-to-all family, scatter, send /
 *                                receive, one-level reduce-scatter), whole for the others
 *   "blocking_arrive" "0" | "1"  a rank's call waits inside the library until the group is complete.  With "0" (default)
 *                                a call returns at once and the last rank's call issues the collective; what a rank's
 *                                stream held when the rank called runs before the collective, but work queued on that
 *                                stream between the rank's call and the last rank's call is NOT ordered after the
 *                                collective (it may read a receive buffer that is not written yet): a caller that drives
 *                                all ranks from one thread queues such work after the last rank's call, or uses one thread
 *                                per rank with "1", which gives every rank the reference's per-stream semantics
 *   "arrive_timeout_ms"          limit of that wait (HCCL_E_TIMEOUT)
 * Unknown key or bad value: HCCL_E_PARA. */
extern HcclResult HcclAmdSetParam(HcclComm comm, const char *key, const char *value);

typedef struct HcclAmdOpInfoDef {
    int32_t coll;            /* 0 all-reduce, 1 reduce-scatter, 2 all-gather, 3 all-to-all-v, 4 broadcast, 5 reduce, 6 scatter */
    int32_t algo;            /* 0 ring, 1 mesh, 2 rhd, 3 pairwise, 4 mesh without the piece cut, 5 star, 6 hd over blocks */
    int32_t fused;           /* 1: issued as fused single-pass kernels */
    int32_t graph;           /* 1: issued as a HIP graph */
    int32_t cacheHit;        /* 1: an instantiated graph / table set was reused */
    uint32_t launches;       /* kernel launches per collective */
    uint64_t bytesRead;      /* bytes the issued kernels read from HBM, all ranks */
    uint64_t bytesWritten;   /* bytes they write */
    uint64_t schedRead;      /* same for the step-by-step schedule (direct peer reads, no staging) */
    uint64_t schedWritten;
    uint64_t scratchBytes;   /* per-rank scratch in use */
    uint32_t teamLaunches;   /* how many of the launches are team kernels (setting "team") */
    uint32_t reserved;
} HcclAmdOpInfo;

/* What the most recent collective of this communicator's group issued. */
extern HcclResult HcclAmdGetLastOpInfo(HcclComm comm, HcclAmdOpInfo *info);

/* Plans a collective without a device and writes the plan as JSON (phases of copy / reduce steps,
 * fused items, byte counts) into out[0..cap).  coll / algo as in HcclAmdOpInfo; for the rooted
 * collectives (coll 4 broadcast, 5 reduce, 6 scatter) the algo argument carries the root rank in its low 16 bits and the
 * schedule in bits 16..19 (0 ring, 1 mesh, 2 rhd, 4 mesh without the piece cut, 5 star, 6 hd over blocks: broadcast only), for the reduce also the number of rank
 * groups of its two-level schedule in bits 20..27, bit 28 for the mesh level without the piece cut and bit 29 / bit 30 for
 * one ring / four rings inside a group, for the broadcast the number of rank groups in bits 20..27 and bit 29 / bit 30 the same way (the scatter takes these two bits too), for the scatter
 * bit 20 for the ring schedule instead of the mesh and the number of rank groups of the two-level mesh schedule in bits 21..28;
 * for the all-reduce (coll 0) bits 8..15 of algo
 * carry the number of rank groups of the two-level schedule (0 or 1: one level), bit 16 asks for its mesh level
 * without the piece cut, bits 17..19 give the rings inside a group (0: mesh, 1, or 4) and bits 20..27 the ranks of an
 * 8-rank ring that own a network port (bit 20 + r for rank r; 0: all of them); the reduce-scatter (coll 1)
 * and the all-gather (coll 2) take bits 8..19 the same way, the reduce-scatter over rank groups of 8 with four rings inside
 * and the ring between them also bits 20..27 (bit 20 + d: device d of every group has a port); for the all-to-all-v (coll 3) bits 8..15 give the number
 * of servers of the staged schedule.  inPlaceMask bit r:
 * rank r's send and receive buffer are the same.  For all-to-all-v, tables points to 4*p*p uint64
 * (sendCounts, sdispls, recvCounts, rdispls, each p x p row-major, row = rank); for the variable-count
 * reduce-scatter / all-gather, tables points to 2*p uint64 (block counts, block displacements); else NULL.
 * Returns HCCL_E_MEMORY and the needed size in *needed when cap is too small. */
extern HcclResult HcclAmdDescribePlan(int32_t coll, int32_t algo, uint32_t nRanks, uint64_t count, HcclDataType dataType,
    uint64_t cclBytes, uint64_t align, uint64_t inPlaceMask, const uint64_t *tables, char *out, size_t cap, size_t *needed);

/* HcclReduceScatter that allocates nothing.  No counterpart in the reference: it is for callers that cannot
 * allocate device memory while they run -- code under HIP graph capture, tight serving loops, harnesses that
 * forbid it.  Arguments, checks and result are HcclReduceScatter's (every rank of the group calls it; the
 * last call issues the work on its stream).  Descriptor tables, and with "fuse" = "0" the schedule's partial
 * results, live in a fixed workspace that every GPU holds from library load to process end:
 * HCCL_AMD_NOALLOC_TABLE_BYTES of tables and HCCL_AMD_NOALLOC_DATA_BYTES of partial results (shared
 * equally by the ranks: nRanks * recvCount * sizeof(type) partial bytes per rank must fit its share).
 * Larger requests fail with HCCL_E_PARA and a message.  Nothing is cached and no graph is built, so a call
 * costs a plan lookup and one small upload launch per 3 KiB of tables on top of the kernels.  All calls on a
 * GPU share that GPU's workspace, whichever group they come from.  The library orders them: a call whose work goes to
 * another stream than the previous call's is queued behind that work (an event created at set-up, nothing allocated),
 * so calls from several groups or streams each get their own result, one after the other.  The exception is a call
 * recorded under stream capture: no event is waited for or recorded there, and replays of the captured graph that may
 * overlap other calls of this kind on another stream are the caller's to order.  The device is set up when a group is
 * complete (HcclCommInitAll, or the last rank's HcclCommInitRootInfo / ...ClusterInfo / HcclCreateSubCommConfig), so
 * this call may be a group's first collective.  Nothing in the workspace has to start at zero: tables are rewritten by
 * every call and partial results are written before they are read. */
#define HCCL_AMD_NOALLOC_TABLE_BYTES (256u << 10)
#define HCCL_AMD_NOALLOC_DATA_BYTES (32u << 20)
extern HcclResult HcclAmdReduceScatterNoAlloc(void *sendBuf, void *recvBuf, uint64_t recvCount, HcclDataType dataType,
    HcclReduceOp op, HcclComm comm, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* HCCL_AMD_EXT_H_ */
