// Schedule planner: turns one collective call into a list of phases of copy / reduce steps over the
// ranks' device buffers, and (when the result can be written as one expression per output range)
// into fused read-reduce-write items.
//
// Reference interfaces this replaces (the host side of the algorithm templates and executors):
//   slice plan   ALG/base/alg_template/temp_all_reduce/all_reduce_ring.cc:119-130
//   chunk loop   ALG/impl/coll_executor/coll_all_reduce/coll_all_reduce_executor.cc:155-203
//   step order   ALG/base/alg_template/temp_reduce_scatter/reduce_scatter_ring.cc:179-297,
//                temp_all_gather/all_gather_ring.cc:120-171, temp_reduce_scatter/reduce_scatter_mesh.cc:57-124,
//                temp_all_gather/all_gather_mesh.cc:91-145, temp_all_reduce/all_reduce_recursive_hd.cc:33-302,
//                temp_reduce_scatter/reduce_scatter_halving_doubling.cc:67-238,
//                temp_all_gather/all_gather_halving_doubling.cc:43-196, temp_alltoallv/alltoallv_pairwise.cc:99-282,
//                temp_broadcast/broadcast_ring.cc:24-160, temp_reduce/reduce_ring.cc:29-154, temp_scatter/scatter_mesh.cc:46-160
// (ALG = src/domain/collective_communication/algorithm in the reference tree.)
//
// Pure C++: no HIP calls, so the planner can be exercised without a GPU.
#pragma once
#include <cstdint>
#include <string>
#include <vector>

namespace hcclamd {

enum CollKind : int {
    COLL_ALLREDUCE = 0, COLL_REDUCESCATTER = 1, COLL_ALLGATHER = 2, COLL_ALLTOALLV = 3,
    COLL_BROADCAST = 4, COLL_REDUCE = 5, COLL_SCATTER = 6, COLL_SENDRECV = 7
};
// ALGO_MESH_ATOMIC: the mesh schedule whose reduce phases skip the piece cut (the reference's
// non-deterministic variant, taken in stream order); BuildPlan turns it into ALGO_MESH + meshAtomic.
// ALGO_STAR: broadcast only, the root hands every rank the whole buffer (broadcast_star.cc).
// ALGO_HD_BLOCKS: broadcast only, halving-doubling over blocks of power-of-two sizes (bcast_halvingdoubling.cc).
enum Algo : int { ALGO_RING = 0, ALGO_MESH = 1, ALGO_RHD = 2, ALGO_PAIRWISE = 3, ALGO_MESH_ATOMIC = 4, ALGO_STAR = 5, ALGO_HD_BLOCKS = 6 };

// Physical buffers of a rank: the caller's send and receive buffers and a library-owned scratch.
enum Buf : uint8_t { BUF_SEND = 0, BUF_RECV = 1, BUF_SCRATCH = 2 };

struct Ref {
    uint32_t rank = 0;
    uint8_t buf = BUF_SEND;
    uint64_t off = 0;
};

// dst = a            (copy,   reduce == false)
// dst = a (+) b      (reduce; a is the rank's own operand, b the one read from the peer)
struct Step {
    bool reduce = false;
    Ref dst, a, b;
    uint64_t bytes = 0;
};

// Steps of one phase have no hazards between them: one kernel launch runs them all.
struct Phase {
    std::vector<Step> steps;
};

enum FusedKind : uint8_t {
    FK_COPY = 0,    // dst[*] = src[0]
    FK_CHAIN = 1,   // acc = src[0]; acc = accLeft[j] ? acc (+) src[j] : src[j] (+) acc, j = 1..n-1
    FK_TREE = 2,    // nleaf = 2^k leaves (leaf i = src[2i] or src[2i] (+) src[2i+1]); pairwise
                    // bottom-up: v[i] = v[i] (+) v[i+w] for w = 1, 2, 4, ...
    FK_STACK = 3    // any other expression, in stack-machine form: for each source in turn push it, then
                    // fold the two topmost values ops[j] & 7 times; bit 8 + i of ops[j] set = in fold i the
                    // lower value is the left operand, clear = the top value is
};

// Limits of the stack form (what its kernel holds in registers).
constexpr uint32_t kStackDepth = 8;
constexpr uint32_t kStackMaxSrc = 64;

// A vector whose first N elements live inside the object.  An all-to-all-v between 64 ranks is 4096 items of one
// source and one destination each, planned anew whenever its tables change: with ordinary vectors the allocations of
// those items were most of the planning time.
template <typename T, uint32_t N> class SmallVec {
public:
    uint32_t size() const { return n_; }
    bool empty() const { return n_ == 0; }
    T *data() { return n_ <= N ? inl_ : heap_.data(); }
    const T *data() const { return n_ <= N ? inl_ : heap_.data(); }
    T *begin() { return data(); }
    T *end() { return data() + n_; }
    const T *begin() const { return data(); }
    const T *end() const { return data() + n_; }
    T &operator[](size_t i) { return data()[i]; }
    const T &operator[](size_t i) const { return data()[i]; }
    T &back() { return data()[n_ - 1]; }
    void clear()
    {
        n_ = 0;
        heap_.clear();
    }
    void push_back(const T &v)
    {
        if (n_ < N) {
            inl_[n_++] = v;
            return;
        }
        if (n_ == N) {
            heap_.assign(inl_, inl_ + N);
        }
        heap_.push_back(v);
        n_++;
    }
    template <typename It> void assign(It first, It last)
    {
        clear();
        for (; first != last; ++first) {
            push_back(*first);
        }
    }
    void assign(size_t count, const T &v)
    {
        clear();
        for (size_t i = 0; i < count; i++) {
            push_back(v);
        }
    }

private:
    T inl_[N] = {};
    uint32_t n_ = 0;
    std::vector<T> heap_;
};

struct FusedItem {
    FusedKind kind = FK_COPY;
    uint64_t bytes = 0;
    SmallVec<Ref, 2> src;
    SmallVec<uint8_t, 4> srcValid;   // FK_TREE: second source of a leaf may be absent
    SmallVec<uint8_t, 4> accLeft;    // FK_CHAIN: one flag per src (index 0 unused)
    SmallVec<uint16_t, 2> ops;       // FK_STACK: one word per src
    uint32_t nleaf = 0;              // FK_TREE: leaves; FK_STACK: stack depth the program needs
    SmallVec<Ref, 2> dst;
};

struct PlanRequest {
    CollKind coll = COLL_ALLREDUCE;
    Algo algo = ALGO_RING;
    uint32_t p = 1;
    uint64_t count = 0;            // all-reduce: elements; reduce-scatter: recvCount; all-gather: sendCount
    uint32_t root = 0;             // broadcast / reduce / scatter; send / receive: the sending rank
    uint32_t peer = 0;             // send / receive: the receiving rank
    uint32_t unit = 4;             // element size in bytes
    uint64_t cclBytes = 200ull << 20;
    uint64_t align = 128;
    std::vector<uint8_t> alias;    // per rank: send buffer and receive buffer are the same memory
    uint32_t servers = 1;          // all-reduce only: > 1 = two levels, `servers` groups of p / servers consecutive ranks
                                   // (mesh inside a group, `algo` ring or halving-doubling between the groups)
    uint32_t level0Rings = 0;      // two-level all-reduce: 0 = mesh inside a group, 1 = one ring, 4 = the four rings of
                                   // the 8-device ring topology (groups of 8 ranks only), each on a quarter of every slice
    uint32_t nicMask = 0;          // one-level ring all-reduce over 8 ranks: bit r set = rank r has a network port.  With 1, 2
                                   // or 4 ports the reduce-scatter runs the port-pruned form (reduce_scatter_ring.cc:160-168,
                                   // 299-477): the slices of chunk j all end their ring chain at the j-th port rank.  0 or all
                                   // 8 bits: the plain ring.  Two-level reduce-scatter over servers of 8 ranks (four rings
                                   // inside, ring between): bit d = device d of every server has a port; with 1, 2 or 4 ports
                                   // the servers all-reduce first, the port devices run the ring between the servers and
                                   // scatter the result inside (coll_reduce_scatter_ring_executor.cc:150-170, 264-300)
    bool meshAtomic = false;       // mesh reduce phases without the piece cut (the reference's non-deterministic variant)
    bool stageInput = false;       // copy the send buffers to scratch first (used when buffers overlap)
    // all-to-all-v only: p x p tables in elements, row r = what rank r passed
    std::vector<uint64_t> sendCounts, sdispls, recvCounts, rdispls;
    // reduce-scatter-v / all-gather-v: per-rank block counts and displacements in elements (p entries
    // each, the same on every rank).  Empty = the uniform collective described by `count`.
    std::vector<uint64_t> vCounts, vDispls;
};

struct Plan {
    uint32_t p = 0;
    std::vector<Phase> phases;          // step-by-step program (always valid)
    uint64_t scratchBytes = 0;          // per-rank scratch the step program needs (0 = none)
    bool fusedOk = false;               // `fused` computes the same outputs from the inputs alone
    std::vector<FusedItem> fused;
    std::vector<uint64_t> sendBytes, recvBytes;   // extent of each rank's buffers the plan touches
    // byte accounting (all ranks): what the step program / the fused items read and write in HBM
    uint64_t stepRead = 0, stepWritten = 0, fusedRead = 0, fusedWritten = 0;
};

// Returns 0 on success; on failure `err` says why (invalid request, or an internal planner check
// failed: hazard inside a phase, read of an unwritten range, fused and stepwise results differ).
int BuildPlan(const PlanRequest &req, Plan *plan, std::string *err);

// A plan together with what is needed to derive from it the plan of the same request with another count.
// Everything the planner does after laying out the schedule compares, adds and subtracts byte offsets and nothing
// else, so when the schedule of a request is the template's with every offset and length multiplied by one factor
// (what happens whenever both counts cut into whole slices: multiples of ranks x alignment inside one chunk; for the
// collectives with one block per rank at any count), its plan is the template's plan multiplied the same way.
// A count with a ragged last slice is covered as well where the collective works position by position (all-reduce,
// broadcast, reduce: every step reads and writes the same offset of every buffer it touches, so what happens below
// an offset does not depend on what lies above it): its schedule then is a whole-slice schedule cut off at the
// count's last byte, and so is its plan.  Either way the new count's schedule is laid out (microseconds) and held
// against the scaled, cut-off template step by step before anything is derived; planning a ring all-reduce of 8
// ranks from scratch costs about a hundred microseconds, a piece-cut mesh of 32 ranks tens of milliseconds --
// which a caller whose sizes change from call to call would otherwise pay on every call.
//
// A reduce-scatter over a table of blocks (the variable-count one) whose blocks are all non-empty and lie one
// behind the other in rank order has a template of another kind: the plan of the same request over blocks of
// 16, 32, 64 ... elements.  Every offset and length of that schedule and of its plan is a run of consecutive blocks,
// and with those sizes the run can be read off the number; the plan for other block sizes is the same plan with every
// run measured in the new sizes (the order of all range ends, which is all the planner looks at, is the same for any
// non-empty blocks laid out that way).  As above, the new schedule is held against the re-measured template first.
struct PlanTemplate {
    uint64_t count = 0;                       // 0: not usable as a count template
    bool blockTable = false;                  // the other kind: canonical block sizes, re-measured per request
    std::vector<Phase> schedule;              // the schedule as laid out, before lowering
    std::vector<uint64_t> inBytes, outBytes, workBytes;
    bool workspace = false;                   // the schedule rests data in a workspace: exact multiples only
    bool positionWise = false;                // may be cut off at a count's last byte
    Plan plan;
};

// BuildPlan that also fills `tmpl` where the request has a template of either kind (tmpl->count != 0 or tmpl->blockTable).
// `plan` receives the plan of `req` itself.
int BuildPlanTemplate(const PlanRequest &req, PlanTemplate *tmpl, Plan *plan, std::string *err);

// The plan of `req` (which must differ from the template's request in nothing but the count), if its schedule is the
// template's multiplied by one factor and, for a position-wise collective, cut off at the count's last byte; false if
// it is not, and the caller plans from scratch.
bool PlanFromTemplate(const PlanRequest &req, const PlanTemplate &tmpl, Plan *plan);

// JSON rendering of a plan (phases, steps, fused items) for tests and debugging.
std::string DescribePlan(const Plan &plan);

// Slice plans (exposed for tests).
struct Slice { uint64_t off, size; };
std::vector<Slice> RingSlicePlan(uint64_t total, uint32_t n, uint64_t align);
void HalvingDoublingShape(uint32_t p, uint32_t *block, uint32_t *part1);
std::vector<uint64_t> ChunkCounts(CollKind coll, uint64_t count, uint32_t unit, uint32_t p, uint64_t cclBytes,
    uint64_t align);

}  // namespace hcclamd
