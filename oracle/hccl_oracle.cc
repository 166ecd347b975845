// TEST INFRASTRUCTURE ONLY -- CPU restatement of the HCCL per-rank data path.
//
// This file is the checker the HIP library is compared against.  It is never linked into, loaded
// by, or called from the product library; only tests, the smoke check and the CPU-baseline leg of
// the benchmark may use it.
//
// What it restates (paths relative to the reference tree; ALG = src/domain/collective_communication/
// algorithm, TPL = ALG/base/alg_template, EXE = ALG/impl/coll_executor):
//   slice plans      TPL/temp_all_reduce/all_reduce_ring.cc:119-130, TPL/recursive_halvingdoubling_base.cc:23-94,
//                    EXE/coll_comm_executor.cc:1681-1721 (piece cut used for the mesh streams)
//   chunk loops      EXE/coll_all_reduce/coll_all_reduce_executor.cc:86-93,155-272,
//                    EXE/coll_reduce_scatter/coll_reduce_scatter_executor.cc:83-90,118-245,
//                    EXE/coll_all_gather/coll_all_gather_executor.cc:79-87,109-193
//   ring             TPL/temp_reduce_scatter/reduce_scatter_ring.cc:89-297 and, for an 8-rank ring with fewer network ports
//                    than ranks, :160-168,299-477 (the port-pruned form); TPL/temp_all_gather/all_gather_ring.cc:51-171,
//                    TPL/temp_all_reduce/all_reduce_ring.cc:32-53,143-191
//   mesh             TPL/temp_reduce_scatter/reduce_scatter_mesh.cc:57-203, TPL/temp_all_gather/all_gather_mesh.cc:91-253,
//                    EXE/coll_all_reduce/coll_all_reduce_mesh_executor.cc:95-240, EXE/coll_comm_executor.cc:1458-1574,
//                    EXE/coll_all_reduce/coll_all_reduce_ring_executor.cc:95-243 with EXE/coll_comm_executor.cc:1595-1606,
//                    1681-1720,1761-1833 (ring or four rings inside a server),
//                    TPL/temp_reduce_scatter/reduce_scatter_mesh_atomic.cc:82-141 (accumulation order of the racing
//                    streams fixed to stream order: for floating point the reference itself has no single answer)
//   two levels       EXE/coll_all_reduce/coll_all_reduce_mesh_executor.cc:95-240 (several servers),
//                    EXE/coll_reduce_scatter/coll_reduce_scatter_mesh_executor.cc:114-119,128-247,
//                    EXE/coll_reduce/coll_reduce_mesh_executor.cc:75-194 (several servers),
//                    EXE/coll_all_gather/coll_all_gather_mesh_executor.cc:64-175, coll_all_gather_ring_executor.cc:75-200
//   halving-doubling TPL/temp_all_reduce/all_reduce_recursive_hd.cc:33-302,
//                    TPL/temp_reduce_scatter/reduce_scatter_recursive_hd.cc:33-254, TPL/temp_all_gather/all_gather_recursive_hd.cc:26-238,
//                    TPL/temp_reduce_scatter/reduce_scatter_halving_doubling.cc:67-238,
//                    TPL/temp_all_gather/all_gather_halving_doubling.cc:43-196
//   pairwise         TPL/temp_alltoallv/alltoallv_pairwise.cc:75-282, ALG/impl/operator/alltoall_operator.cc:49-72
//   staged a2av      TPL/temp_alltoallv/alltoallv_staged_{mesh,pairwise}.cc, ALG/impl/coll_executor/coll_all_to_all/
//                    coll_all_to_all_v_staged_executor.cc:276-470, coll_all_to_all_executor.cc:156-335 (zero-copy mode)
//   rooted           TPL/temp_broadcast/broadcast_ring.cc:24-160, TPL/temp_reduce/reduce_ring.cc:29-154,
//                    TPL/temp_scatter/scatter_mesh.cc:46-160, TPL/temp_gather/gather_mesh.cc:60-170,
//                    EXE/coll_broadcast/coll_broadcast_mesh_executor.cc:59-213 (one server and several: scatter, halving-doubling
//                    between the servers, all-gather), EXE/coll_reduce/coll_reduce_mesh_executor.cc:75-194,
//                    TPL/temp_reduce/reduce_recursive_hd.cc:31-316, TPL/temp_broadcast/bcast_recursive_halvingdoubling.cc:21-290
//
// Method: every template is restated as the per-rank program it issues (send / receive-and-reduce /
// receive-and-copy / local copy), one virtual process per rank (per rank and stream for the mesh),
// and the programs are run by a message-passing machine with FIFO mailboxes.  A message is a
// snapshot of the sender's bytes at send time ("snapshot" mode) or a pointer into the sender's
// buffer ("direct" mode, which is what an inline-reduce link does; it is valid because no template
// rewrites a range after sending it, and the tests check both modes agree).
//
// Parity status.  The reference ships no tests, golden vectors or fixtures for this path, and its
// leaf arithmetic (Reducer / Sender / Transport) is in closed libraries, so every function here is
// pinned by mathematics only: closed-form reduction chains and trees, order-independent integer
// results, permutation closed forms for gather / all-to-all, and hand-derived slice-plan vectors
// (tests/golden).  Assumptions that only a run of the closed reference could confirm -- PARITY
// UNPINNED for these: the slice alignment constant (128 bytes), the element sizes, the direction of
// ForwardRank / BackwardRank (forced by all_gather_ring.cc:130-163), the piece cut of
// PrepareSliceMeshStreams (taken equal to coll_comm_executor.cc:1681-1721), the level-0 slice plan of the
// two-level executors (closed AlgTemplateBase::PrepareSliceData, taken equal to the ring template's
// all_reduce_ring.cc:119-130, as coll_all_reduce_executor.cc:330-360 does in the open), the operand order and
// the NaN / signed-zero behaviour inside the closed Reducer, and the accumulation width for
// fp16 / bf16 (here: fp32, rounded to nearest-even after every stored step).
#include <algorithm>
#include <atomic>
#include <condition_variable>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <functional>
#include <map>
#include <mutex>
#include <thread>
#include <tuple>
#include <vector>

namespace {

// ------------------------------------------------------------------------------------------------
// Types (values follow inc/hccl/hccl_types.h:58-87)
// ------------------------------------------------------------------------------------------------
enum { DT_INT8 = 0, DT_INT16 = 1, DT_INT32 = 2, DT_FP16 = 3, DT_FP32 = 4, DT_INT64 = 5, DT_UINT64 = 6,
       DT_UINT8 = 7, DT_UINT16 = 8, DT_UINT32 = 9, DT_FP64 = 10, DT_BF16 = 11, DT_INT128 = 12 };
enum { OP_SUM = 0, OP_PROD = 1, OP_MAX = 2, OP_MIN = 3 };
enum { ALGO_RING = 0, ALGO_MESH = 1, ALGO_RHD = 2, ALGO_MESH_ATOMIC = 4 };

size_t DtSize(int dt)
{
    static const size_t table[] = {1, 2, 4, 2, 4, 8, 8, 1, 2, 4, 8, 2, 16, 1, 1, 1};
    return (dt >= 0 && dt < 16) ? table[dt] : 0;
}

struct Slice { uint64_t off; uint64_t size; };

// ------------------------------------------------------------------------------------------------
// 16-bit float conversions (round to nearest even; NaN stays NaN, quiet bit set)
// ------------------------------------------------------------------------------------------------
inline uint32_t F2U(float f) { uint32_t u; std::memcpy(&u, &f, 4); return u; }
inline float U2F(uint32_t u) { float f; std::memcpy(&f, &u, 4); return f; }

inline float Bf16ToF32(uint16_t b) { return U2F(static_cast<uint32_t>(b) << 16); }
inline uint16_t F32ToBf16(float f)
{
    uint32_t u = F2U(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) {
        return static_cast<uint16_t>((u >> 16) | 0x0040u);
    }
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return static_cast<uint16_t>(u >> 16);
}

inline float Fp16ToF32(uint16_t h)
{
    uint32_t sign = static_cast<uint32_t>(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    if (exp == 0) {
        if (man == 0) {
            return U2F(sign);
        }
        // subnormal half: value = man * 2^-24
        float v = static_cast<float>(man) * 5.9604644775390625e-08f;
        return U2F(F2U(v) | sign);
    }
    if (exp == 31) {
        return U2F(sign | 0x7f800000u | (man << 13));
    }
    return U2F(sign | ((exp + 112u) << 23) | (man << 13));
}

inline uint16_t F32ToFp16(float f)
{
    uint32_t u = F2U(f);
    uint16_t sign = static_cast<uint16_t>((u >> 16) & 0x8000u);
    uint32_t abs = u & 0x7fffffffu;
    if (abs > 0x7f800000u) {
        return static_cast<uint16_t>(sign | 0x7e00u | ((abs >> 13) & 0x3ffu));
    }
    if (abs >= 0x47800000u) {  // >= 65536 -> inf (65520 rounds to inf below through the normal path)
        return static_cast<uint16_t>(sign | 0x7c00u);
    }
    if (abs < 0x38800000u) {   // below the smallest normal half (2^-14): subnormal or zero
        if (abs < 0x33000000u) {  // < 2^-25 rounds to zero (2^-25 itself ties to even = 0)
            return sign;
        }
        // value = m * 2^-24 with m in [0.5, 1024); round m to nearest even integer
        uint32_t e = abs >> 23;
        uint32_t m = (abs & 0x7fffffu) | 0x800000u;
        uint32_t shift = 126u - e;          // e in [102,112] -> shift in [14,24]
        uint32_t q = m >> shift;
        uint32_t rem = m & ((1u << shift) - 1u);
        uint32_t half = 1u << (shift - 1u);
        if (rem > half || (rem == half && (q & 1u))) {
            q++;
        }
        return static_cast<uint16_t>(sign | q);
    }
    uint32_t lsb = (abs >> 13) & 1u;
    abs += 0xfffu + lsb;
    uint32_t h = (abs - 0x38000000u) >> 13;
    if (h >= 0x7c00u) {
        h = 0x7c00u;
    }
    return static_cast<uint16_t>(sign | h);
}

// ------------------------------------------------------------------------------------------------
// Element reduction: dst = a (+) b, where a is the local operand and b the received one.
//   sum / prod : integers wrap modulo 2^n (computed unsigned); floats use one IEEE operation
//   max        : (b > a) ? b : a          min : (b < a) ? b : a
// fp16 / bf16 operands are widened to fp32, combined, and rounded back (max / min keep the bits of
// the chosen operand).
// ------------------------------------------------------------------------------------------------
template <typename T, typename U> inline T IntOp(int op, T a, T b)
{
    switch (op) {
        case OP_SUM: return static_cast<T>(static_cast<U>(static_cast<U>(a) + static_cast<U>(b)));
        case OP_PROD: return static_cast<T>(static_cast<U>(static_cast<U>(a) * static_cast<U>(b)));
        case OP_MAX: return (b > a) ? b : a;
        default: return (b < a) ? b : a;
    }
}
// 16-bit unsigned products promote to int and could overflow it: multiply in 32-bit unsigned.
template <> inline int16_t IntOp<int16_t, uint16_t>(int op, int16_t a, int16_t b)
{
    switch (op) {
        case OP_SUM: return static_cast<int16_t>(static_cast<uint16_t>(static_cast<uint32_t>(static_cast<uint16_t>(a)) + static_cast<uint16_t>(b)));
        case OP_PROD: return static_cast<int16_t>(static_cast<uint16_t>(static_cast<uint32_t>(static_cast<uint16_t>(a)) * static_cast<uint16_t>(b)));
        case OP_MAX: return (b > a) ? b : a;
        default: return (b < a) ? b : a;
    }
}
template <> inline uint16_t IntOp<uint16_t, uint16_t>(int op, uint16_t a, uint16_t b)
{
    switch (op) {
        case OP_SUM: return static_cast<uint16_t>(static_cast<uint32_t>(a) + b);
        case OP_PROD: return static_cast<uint16_t>(static_cast<uint32_t>(a) * b);
        case OP_MAX: return (b > a) ? b : a;
        default: return (b < a) ? b : a;
    }
}
template <typename T> inline T FloatOp(int op, T a, T b)
{
    switch (op) {
        case OP_SUM: return a + b;
        case OP_PROD: return a * b;
        case OP_MAX: return (b > a) ? b : a;
        default: return (b < a) ? b : a;
    }
}
template <typename T, typename F> void LoopT(void *dst, const void *a, const void *b, size_t n, F f)
{
    T *d = static_cast<T *>(dst);
    const T *x = static_cast<const T *>(a);
    const T *y = static_cast<const T *>(b);
    for (size_t i = 0; i < n; i++) {
        d[i] = f(x[i], y[i]);
    }
}

int ReduceElems(int dt, int op, void *dst, const void *a, const void *b, size_t n)
{
    switch (dt) {
        case DT_INT8: LoopT<int8_t>(dst, a, b, n, [op](int8_t x, int8_t y) { return IntOp<int8_t, uint8_t>(op, x, y); }); return 0;
        case DT_UINT8: LoopT<uint8_t>(dst, a, b, n, [op](uint8_t x, uint8_t y) { return IntOp<uint8_t, uint8_t>(op, x, y); }); return 0;
        case DT_INT16: LoopT<int16_t>(dst, a, b, n, [op](int16_t x, int16_t y) { return IntOp<int16_t, uint16_t>(op, x, y); }); return 0;
        case DT_UINT16: LoopT<uint16_t>(dst, a, b, n, [op](uint16_t x, uint16_t y) { return IntOp<uint16_t, uint16_t>(op, x, y); }); return 0;
        case DT_INT32: LoopT<int32_t>(dst, a, b, n, [op](int32_t x, int32_t y) { return IntOp<int32_t, uint32_t>(op, x, y); }); return 0;
        case DT_UINT32: LoopT<uint32_t>(dst, a, b, n, [op](uint32_t x, uint32_t y) { return IntOp<uint32_t, uint32_t>(op, x, y); }); return 0;
        case DT_INT64: LoopT<int64_t>(dst, a, b, n, [op](int64_t x, int64_t y) { return IntOp<int64_t, uint64_t>(op, x, y); }); return 0;
        case DT_UINT64: LoopT<uint64_t>(dst, a, b, n, [op](uint64_t x, uint64_t y) { return IntOp<uint64_t, uint64_t>(op, x, y); }); return 0;
        case DT_FP32: LoopT<float>(dst, a, b, n, [op](float x, float y) { return FloatOp<float>(op, x, y); }); return 0;
        case DT_FP64: LoopT<double>(dst, a, b, n, [op](double x, double y) { return FloatOp<double>(op, x, y); }); return 0;
        case DT_FP16:
            LoopT<uint16_t>(dst, a, b, n, [op](uint16_t x, uint16_t y) -> uint16_t {
                float fx = Fp16ToF32(x), fy = Fp16ToF32(y);
                if (op == OP_SUM) return F32ToFp16(fx + fy);
                if (op == OP_PROD) return F32ToFp16(fx * fy);
                if (op == OP_MAX) return (fy > fx) ? y : x;
                return (fy < fx) ? y : x;
            });
            return 0;
        case DT_BF16:
            LoopT<uint16_t>(dst, a, b, n, [op](uint16_t x, uint16_t y) -> uint16_t {
                float fx = Bf16ToF32(x), fy = Bf16ToF32(y);
                if (op == OP_SUM) return F32ToBf16(fx + fy);
                if (op == OP_PROD) return F32ToBf16(fx * fy);
                if (op == OP_MAX) return (fy > fx) ? y : x;
                return (fy < fx) ? y : x;
            });
            return 0;
        default: return -1;
    }
}

// ------------------------------------------------------------------------------------------------
// Thread pool: splits one byte range into element-aligned pieces (per-element order unchanged, so
// the result does not depend on the thread count).
// ------------------------------------------------------------------------------------------------
class Pool {
public:
    explicit Pool(int n) : n_(n < 1 ? 1 : n)
    {
        for (int i = 1; i < n_; i++) {
            workers_.emplace_back([this, i] { Work(i); });
        }
    }
    ~Pool()
    {
        {
            std::lock_guard<std::mutex> g(m_);
            stop_ = true;
            gen_++;
        }
        cv_.notify_all();
        for (auto &t : workers_) {
            t.join();
        }
    }
    int Threads() const { return n_; }
    // fn(begin, end) over [0, total) cut into n_ pieces of a multiple of `grain`.
    void Run(uint64_t total, uint64_t grain, const std::function<void(uint64_t, uint64_t)> &fn)
    {
        if (n_ == 1 || total < (1u << 16)) {
            fn(0, total);
            return;
        }
        uint64_t units = (total + grain - 1) / grain;
        uint64_t per = (units + n_ - 1) / n_ * grain;
        {
            std::lock_guard<std::mutex> g(m_);
            fn_ = &fn;
            total_ = total;
            per_ = per;
            pending_ = n_ - 1;
            gen_++;
        }
        cv_.notify_all();
        Piece(0);
        std::unique_lock<std::mutex> g(m_);
        done_.wait(g, [this] { return pending_ == 0; });
    }

private:
    void Piece(int i)
    {
        uint64_t b = std::min<uint64_t>(total_, per_ * i);
        uint64_t e = std::min<uint64_t>(total_, per_ * (i + 1));
        if (e > b) {
            (*fn_)(b, e);
        }
    }
    void Work(int i)
    {
        uint64_t seen = 0;
        for (;;) {
            {
                std::unique_lock<std::mutex> g(m_);
                cv_.wait(g, [&] { return gen_ != seen; });
                seen = gen_;
                if (stop_) {
                    return;
                }
            }
            Piece(i);
            {
                std::lock_guard<std::mutex> g(m_);
                pending_--;
            }
            done_.notify_one();
        }
    }
    int n_;
    std::vector<std::thread> workers_;
    std::mutex m_;
    std::condition_variable cv_, done_;
    const std::function<void(uint64_t, uint64_t)> *fn_ = nullptr;
    uint64_t total_ = 0, per_ = 0, gen_ = 0;
    int pending_ = 0;
    bool stop_ = false;
};

// ------------------------------------------------------------------------------------------------
// Slice and chunk plans
// ------------------------------------------------------------------------------------------------
uint64_t RoundUp(uint64_t v, uint64_t d) { return d == 0 ? v : (v + d - 1) / d * d; }

// all_reduce_ring.cc:119-130 (same rule: coll_all_reduce_executor.cc:330-360).
std::vector<Slice> RingSlices(uint64_t total, uint32_t p, uint64_t align)
{
    std::vector<Slice> s(p);
    uint64_t per = RoundUp((total + (p - 1)) / p, align);
    uint64_t residue = total;
    for (uint32_t i = 0; i < p; i++) {
        s[i].size = (residue > per) ? per : residue;
        s[i].off = total - residue;
        residue -= s[i].size;
    }
    return s;
}

// recursive_halvingdoubling_base.cc:23-37.
void RhdParams(uint32_t p, uint32_t *block, uint32_t *part1)
{
    uint32_t round = 0;
    while ((1u << round) <= p) {
        round++;
    }
    if (round >= 1) {
        round--;
    }
    *block = 1u << round;
    *part1 = (p - *block) * 2;
}

// recursive_halvingdoubling_base.cc:64-94.
std::vector<Slice> RhdSlices(uint64_t bytes, uint32_t block, uint64_t align)
{
    std::vector<Slice> s(block);
    uint64_t per = bytes / block;
    if (bytes % block != 0) {
        per++;
    }
    per = RoundUp(per, align);
    uint64_t left = bytes;
    uint32_t i = 0;
    while (left > 0) {
        s[i].size = per < left ? per : left;
        s[i].off = bytes - left;
        left -= s[i].size;
        i++;
    }
    while (i < block) {
        s[i].off = bytes;
        s[i].size = 0;
        i++;
    }
    return s;
}

// coll_comm_executor.cc:1681-1721: cut every rank slice into n pieces, left to right.
std::vector<std::vector<Slice>> CutPieces(const std::vector<Slice> &slices, uint32_t n, uint64_t align)
{
    // result[piece][rank]
    std::vector<std::vector<Slice>> out(n, std::vector<Slice>(slices.size()));
    for (size_t r = 0; r < slices.size(); r++) {
        uint64_t size = slices[r].size, start = slices[r].off;
        uint32_t k = 0;
        if (size > 0 && n != 0) {
            uint64_t per = RoundUp((size + n - 1) / n, align);
            uint64_t residue = size;
            while (residue > 0) {
                uint64_t cur = per < residue ? per : residue;
                out[k][r] = Slice{start + size - residue, cur};
                residue -= cur;
                k++;
            }
        }
        while (k < n) {
            out[k][r] = Slice{start, 0};
            k++;
        }
    }
    return out;
}

// Elements per loop iteration of the executor-level chunk loops.
//   AllReduce       : cclBytes / unit                                 (coll_all_reduce_executor.cc:86-93)
//   ReduceScatter   : cclBytes / p / ALIGN * ALIGN / unit             (coll_reduce_scatter_executor.cc:83-90)
//   AllGather       : cclBytes / p / ALIGN * ALIGN / unit             (coll_all_gather_executor.cc:79-87)
uint64_t MaxCountPerLoop(int kind, uint64_t cclBytes, uint32_t p, uint64_t unit, uint64_t align)
{
    if (kind == 0) {
        return cclBytes / unit;
    }
    return cclBytes / p / align * align / unit;
}

// ------------------------------------------------------------------------------------------------
// Message-passing machine
// ------------------------------------------------------------------------------------------------
enum ActKind { SEND, RECV_REDUCE, RECV_COPY, LOCAL_COPY, LOCAL_REDUCE };
enum BufId { B_IN = 0, B_OUT = 1 };

struct Action {
    ActKind kind;
    int peer;        // other rank (SEND / RECV_*)
    int chan;        // FIFO channel between the two ranks (stream index for the mesh)
    int dstBuf; uint64_t dstOff;
    int srcBuf; uint64_t srcOff;   // SEND: payload; RECV_REDUCE / LOCAL_*: local operand
    uint64_t len;
};

struct Proc {
    int rank;
    std::vector<Action> prog;
    size_t pc = 0;
};

struct Msg {
    std::vector<uint8_t> snap;
    const uint8_t *ptr = nullptr;
    uint64_t len = 0;
};

struct Machine {
    int p = 0;
    int dt = 0, op = 0;
    bool direct = false;
    Pool *pool = nullptr;
    std::vector<uint8_t *> buf[2];   // buf[B_IN][rank], buf[B_OUT][rank]
    std::vector<Proc> procs;
    std::map<std::tuple<int, int, int>, std::deque<Msg>> box;   // (src, dst, chan)
    uint64_t bytesTouched = 0;

    uint8_t *At(int rank, int b, uint64_t off) { return buf[b][rank] + off; }

    void Copy(uint8_t *dst, const uint8_t *src, uint64_t len)
    {
        if (len == 0 || dst == src) {
            return;
        }
        pool->Run(len, 64, [&](uint64_t b, uint64_t e) { std::memmove(dst + b, src + b, e - b); });
        bytesTouched += 2 * len;
    }
    void Reduce(uint8_t *dst, const uint8_t *a, const uint8_t *b, uint64_t len)
    {
        if (len == 0) {
            return;
        }
        uint64_t u = DtSize(dt);
        pool->Run(len, 64, [&](uint64_t s, uint64_t e) { ReduceElems(dt, op, dst + s, a + s, b + s, (e - s) / u); });
        bytesTouched += 3 * len;
    }

    // Runs every process to completion; returns 0, or -1 on deadlock.
    int Run()
    {
        bool progress = true;
        size_t live = 0;
        for (auto &pr : procs) {
            live += pr.prog.empty() ? 0 : 1;
        }
        while (live > 0 && progress) {
            progress = false;
            for (auto &pr : procs) {
                while (pr.pc < pr.prog.size()) {
                    const Action &a = pr.prog[pr.pc];
                    if (a.kind == SEND) {
                        Msg m;
                        m.len = a.len;
                        if (direct) {
                            m.ptr = At(pr.rank, a.srcBuf, a.srcOff);
                        } else {
                            const uint8_t *s = At(pr.rank, a.srcBuf, a.srcOff);
                            m.snap.assign(s, s + a.len);
                        }
                        box[std::make_tuple(pr.rank, a.peer, a.chan)].push_back(std::move(m));
                    } else if (a.kind == RECV_REDUCE || a.kind == RECV_COPY) {
                        auto &q = box[std::make_tuple(a.peer, pr.rank, a.chan)];
                        if (q.empty()) {
                            break;
                        }
                        Msg m = std::move(q.front());
                        q.pop_front();
                        if (m.len != a.len) {
                            std::fprintf(stderr, "oracle: message length mismatch %llu vs %llu\n",
                                (unsigned long long)m.len, (unsigned long long)a.len);
                            return -2;
                        }
                        const uint8_t *payload = direct ? m.ptr : m.snap.data();
                        if (a.kind == RECV_REDUCE) {
                            Reduce(At(pr.rank, a.dstBuf, a.dstOff), At(pr.rank, a.srcBuf, a.srcOff), payload, a.len);
                        } else {
                            Copy(At(pr.rank, a.dstBuf, a.dstOff), payload, a.len);
                        }
                    } else if (a.kind == LOCAL_COPY) {
                        Copy(At(pr.rank, a.dstBuf, a.dstOff), At(pr.rank, a.srcBuf, a.srcOff), a.len);
                    } else {
                        Reduce(At(pr.rank, a.dstBuf, a.dstOff), At(pr.rank, a.dstBuf, a.dstOff),
                            At(pr.rank, a.srcBuf, a.srcOff), a.len);
                    }
                    pr.pc++;
                    progress = true;
                    if (pr.pc == pr.prog.size()) {
                        live--;
                    }
                }
            }
        }
        procs.clear();
        for (auto &kv : box) {
            if (!kv.second.empty()) {
                return -3;   // undelivered message: the programs do not match up
            }
        }
        box.clear();
        return live == 0 ? 0 : -1;
    }
};

inline Action MkSend(int peer, int chan, int b, uint64_t off, uint64_t len)
{
    return Action{SEND, peer, chan, 0, 0, b, off, len};
}
inline Action MkRecvReduce(int peer, int chan, int dstB, uint64_t dstOff, int srcB, uint64_t srcOff, uint64_t len)
{
    return Action{RECV_REDUCE, peer, chan, dstB, dstOff, srcB, srcOff, len};
}
inline Action MkRecvCopy(int peer, int chan, int dstB, uint64_t dstOff, uint64_t len)
{
    return Action{RECV_COPY, peer, chan, dstB, dstOff, 0, 0, len};
}
inline Action MkLocalCopy(int dstB, uint64_t dstOff, int srcB, uint64_t srcOff, uint64_t len)
{
    return Action{LOCAL_COPY, -1, 0, dstB, dstOff, srcB, srcOff, len};
}

// ------------------------------------------------------------------------------------------------
// Per-rank programs of the templates.  `inB` / `outB` say which machine buffer plays the template's
// inputMem_ / outputMem_.
// ------------------------------------------------------------------------------------------------

// ReduceScatterRing::RunReduceScatter, reduce_scatter_ring.cc:179-297 (one segment per rank).
void ProgReduceScatterRing(std::vector<Action> &pg, uint32_t r, uint32_t p, int inB, int outB,
    const std::vector<Slice> &in, const std::vector<Slice> &out)
{
    if (p == 1) {
        // reduce_scatter_ring.cc:102-107: whole-buffer copy when input and output differ
        if (inB != outB) {
            pg.push_back(MkLocalCopy(outB, out[0].off, inB, in[0].off, in[0].size));
        }
        return;
    }
    uint32_t left = (r + p - 1) % p, right = (r + 1) % p;
    uint32_t rx = (r + p - 2) % p;
    uint32_t tx = (r + p - 1) % p;
    pg.push_back(MkSend(right, 0, inB, in[tx].off, in[tx].size));
    for (uint32_t i = 0; i < p - 2; i++) {
        pg.push_back(MkRecvReduce(left, 0, inB, in[rx].off, inB, in[rx].off, in[rx].size));
        rx = (rx + p - 1) % p;
        tx = (tx + p - 1) % p;
        pg.push_back(MkSend(right, 0, inB, in[tx].off, in[tx].size));
    }
    // last transfer: result goes to the template's output at the output slice of this rank
    pg.push_back(MkRecvReduce(left, 0, outB, out[r].off, inB, in[r].off, in[r].size));
}

// AllGatherRing::RunAsync + RunAllGather, all_gather_ring.cc:51-171.
void ProgAllGatherRing(std::vector<Action> &pg, uint32_t r, uint32_t p, int inB, int outB,
    const std::vector<Slice> &outSl, const std::vector<Slice> &inSl)
{
    if (p == 1) {
        if (inB != outB) {
            pg.push_back(MkLocalCopy(outB, outSl[0].off, inB, inSl[0].off, outSl[0].size));
        }
        return;
    }
    uint32_t left = (r + p - 1) % p, right = (r + 1) % p;
    if (inB != outB) {
        pg.push_back(MkLocalCopy(outB, outSl[r].off, inB, inSl[r].off, outSl[r].size));
    }
    uint32_t rx = (r + p - 1) % p;   // ForwordRank(rank, p, 1)
    uint32_t tx = r;
    for (uint32_t i = 0; i + 1 < p; i++) {
        pg.push_back(MkSend(right, 0, outB, outSl[tx].off, outSl[tx].size));
        pg.push_back(MkRecvCopy(left, 0, outB, outSl[rx].off, outSl[rx].size));
        tx = (tx + p - 1) % p;
        rx = (rx + p - 1) % p;
    }
}

// ReduceScatterMesh::RunReduceScatter for one stream, reduce_scatter_mesh.cc:57-124.
void ProgReduceScatterMeshStream(std::vector<Action> &pg, uint32_t r, uint32_t p, uint32_t stream, int inB,
    const std::vector<Slice> &sl)
{
    for (uint32_t round = 1; round < p; round++) {
        uint32_t order = (round + stream - 1) % (p - 1);
        uint32_t src = (r + p - (order + 1)) % p;   // ForwardRank(r, p, order + 1)
        uint32_t dst = (r + (order + 1)) % p;       // BackwardRank(r, p, order + 1)
        pg.push_back(MkSend(dst, static_cast<int>(stream), inB, sl[dst].off, sl[dst].size));
        pg.push_back(MkRecvReduce(src, static_cast<int>(stream), inB, sl[r].off, inB, sl[r].off, sl[r].size));
    }
}

// ReduceScatterMeshAtomic::RunReduceScatter, reduce_scatter_mesh_atomic.cc:82-141: stream j of rank r
// pulls slice r of rank (r+1+j) and accumulates it into the rank's own slice r.  The reference lets
// the p-1 streams race, so its floating-point result depends on arrival order; this restatement
// takes the streams in index order, which is one of the outcomes the reference can produce.
// The slices a rank hands out are never written during the phase, so all hand-outs come first.
void ProgReduceScatterMeshAtomic(std::vector<Action> &pg, uint32_t r, uint32_t p, int inB, const std::vector<Slice> &sl)
{
    for (uint32_t j = 0; j + 1 < p; j++) {
        uint32_t puller = (r + p - 1 - j) % p;   // the rank whose stream j reads from this rank
        pg.push_back(MkSend(puller, static_cast<int>(j), inB, sl[puller].off, sl[puller].size));
    }
    for (uint32_t j = 0; j + 1 < p; j++) {
        uint32_t remote = (r + 1 + j) % p;
        pg.push_back(MkRecvReduce(remote, static_cast<int>(j), inB, sl[r].off, inB, sl[r].off, sl[r].size));
    }
}

// AllGatherMesh::RunAllGather, all_gather_mesh.cc:91-145 (one channel per round).
void ProgAllGatherMesh(std::vector<Action> &pg, uint32_t r, uint32_t p, int outB, const std::vector<Slice> &sl)
{
    for (uint32_t round = 1; round < p; round++) {
        uint32_t peer = (r + round) % p;
        uint32_t from = (r + p - round) % p;
        // rank r sends its slice to r+round and receives slice (r-round) from r-round on the same round
        pg.push_back(MkSend(peer, static_cast<int>(round), outB, sl[r].off, sl[r].size));
        pg.push_back(MkRecvCopy(from, static_cast<int>(round), outB, sl[from].off, sl[from].size));
    }
}

// ReduceScatterHalvingDoubling::RunReduceScatter, reduce_scatter_halving_doubling.cc:67-91,193-238.
// q = rank inside the block, rankOf[q] = real rank.
void ProgReduceScatterHd(std::vector<Action> &pg, uint32_t q, uint32_t block, const std::vector<uint32_t> &rankOf,
    int inB, int outB, const std::vector<Slice> &sl)
{
    uint32_t steps = 0;
    while ((1u << steps) < block) {
        steps++;
    }
    auto sum = [&](uint32_t first, uint32_t n) {
        uint64_t s = 0;
        for (uint32_t i = first; i < first + n; i++) {
            s += sl[i].size;
        }
        return s;
    };
    Slice lastRx{0, 0};
    for (uint32_t step = 0; step < steps; step++) {
        uint32_t mask = 1u << (steps - step - 1);
        uint32_t peer = q ^ mask;
        uint32_t txId = peer & ~(mask - 1);
        uint32_t rxId = q & ~(mask - 1);
        Slice tx{sl[txId].off, sum(txId, mask)};
        Slice rx{sl[rxId].off, sum(rxId, mask)};
        pg.push_back(MkSend(static_cast<int>(rankOf[peer]), 0, inB, tx.off, tx.size));
        pg.push_back(MkRecvReduce(static_cast<int>(rankOf[peer]), 0, inB, rx.off, inB, rx.off, rx.size));
        lastRx = rx;
    }
    if (steps > 0) {
        pg.push_back(MkLocalCopy(outB, lastRx.off, inB, lastRx.off, lastRx.size));
    }
}

// AllGatherHalvingDoubling::RunAllGather, all_gather_halving_doubling.cc:43-66,158-196.
void ProgAllGatherHd(std::vector<Action> &pg, uint32_t q, uint32_t block, const std::vector<uint32_t> &rankOf,
    int outB, const std::vector<Slice> &sl)
{
    uint32_t steps = 0;
    while ((1u << steps) < block) {
        steps++;
    }
    auto sum = [&](uint32_t first, uint32_t n) {
        uint64_t s = 0;
        for (uint32_t i = first; i < first + n; i++) {
            s += sl[i].size;
        }
        return s;
    };
    for (uint32_t step = 0; step < steps; step++) {
        uint32_t mask = 1u << step;
        uint32_t peer = q ^ mask;
        uint32_t txId = q & ~(mask - 1);
        uint32_t rxId = peer & ~(mask - 1);
        pg.push_back(MkSend(static_cast<int>(rankOf[peer]), 0, outB, sl[txId].off, sum(txId, mask)));
        pg.push_back(MkRecvCopy(static_cast<int>(rankOf[peer]), 0, outB, sl[rxId].off, sum(rxId, mask)));
    }
}

// ------------------------------------------------------------------------------------------------
// Template-level collectives on machine buffers of `bytes` bytes each
// ------------------------------------------------------------------------------------------------

// AllReduceRing::RunAsync, all_reduce_ring.cc:32-53: RS(in, in, scratch=out) then AG(in, out).
int RunAllReduceRing(Machine &m, uint64_t bytes, uint64_t align)
{
    uint32_t p = m.p;
    if (p == 1) {
        m.Copy(m.buf[B_OUT][0], m.buf[B_IN][0], bytes);
        return 0;
    }
    std::vector<Slice> sl = RingSlices(bytes, p, align);
    for (uint32_t r = 0; r < p; r++) {
        Proc pr;
        pr.rank = r;
        ProgReduceScatterRing(pr.prog, r, p, B_IN, B_IN, sl, sl);
        ProgAllGatherRing(pr.prog, r, p, B_IN, B_OUT, sl, sl);
        m.procs.push_back(std::move(pr));
    }
    return m.Run();
}

// Send lists of the port-pruned ring reduce-scatter, ReduceScatterRing::ReduceScatterSlicesPrep
// (TPL/temp_reduce_scatter/reduce_scatter_ring.cc:458-477): rank r sends, for the ranks at ring distance 1, 2, ...
// behind it that own a network port, the chunkSize slices of that port (chunk j = slices j * chunkSize ...).
std::vector<std::vector<uint32_t>> PrunedRingSendLists(uint32_t p, const std::vector<uint32_t> &nic)
{
    const uint32_t chunk = 8 / static_cast<uint32_t>(nic.size());   // HCCL_NIC_MAX_NUM / nicSize
    std::vector<std::vector<uint32_t>> lists;
    for (uint32_t r = 0; r < p; r++) {
        std::vector<uint32_t> one;
        for (uint32_t dis = 1; dis < p; dis++) {
            uint32_t at = (r + p - dis) % p;
            auto it = std::find(nic.begin(), nic.end(), at);
            if (it != nic.end()) {
                uint32_t j = static_cast<uint32_t>(it - nic.begin());
                for (uint32_t c = 0; c < chunk; c++) {
                    one.push_back(chunk * j + c);
                }
            }
        }
        lists.push_back(one);
    }
    return lists;
}

// Per-rank program of ReduceScatterRing::RunReduceScatterChunk (reduce_scatter_ring.cc:299-333) with its parts
// HeadReduceScatterChunk (:335-370), MidReduceScatterChunk (:372-411) and TailReduceScatterChunk (:413-442), taken
// when 8 ranks share fewer than 8 network ports (:160-168).  A receive combines into the input buffer
// (RunDestRducer, :76-87: destination = the rank's own input slice); empty slices are neither sent nor received.
void ProgReduceScatterRingChunk(std::vector<Action> &pg, uint32_t r, uint32_t p, const std::vector<uint32_t> &nic,
    const std::vector<std::vector<uint32_t>> &lists, int inB, const std::vector<Slice> &sl)
{
    const uint32_t left = (r + p - 1) % p, right = (r + 1) % p;
    const std::vector<uint32_t> &mine = lists[r], &prev = lists[left];
    const uint32_t chunk = 8 / static_cast<uint32_t>(nic.size());
    auto inPrev = [&](uint32_t s) { return std::find(prev.begin(), prev.end(), s) != prev.end(); };
    auto send = [&](uint32_t s) {
        if (sl[s].size > 0) {
            pg.push_back(MkSend(static_cast<int>(right), 0, inB, sl[s].off, sl[s].size));
        }
    };
    auto recv = [&](uint32_t s) {
        if (sl[s].size > 0) {
            pg.push_back(MkRecvReduce(static_cast<int>(left), 0, inB, sl[s].off, inB, sl[s].off, sl[s].size));
        }
    };
    auto mid = [&](uint32_t idx) {
        const uint32_t rx = mine[idx + 1], tx = mine[idx];
        send(tx);                       // both branches of :384-408 send; only one of them receives
        if (inPrev(rx)) {
            recv(rx);
        }
    };
    const uint32_t len = static_cast<uint32_t>(mine.size());
    if (len >= chunk && len >= 2) {
        if (inPrev(mine[0])) {          // head, :345-356
            recv(mine[0]);
        }
        if (inPrev(mine[1])) {          // :357-367
            mid(0);
        } else {
            send(mine[0]);
        }
        for (uint32_t idx = 1; idx + 1 < len; idx++) {
            mid(idx);
        }
    }
    if (len > 0) {
        send(mine[len - 1]);            // tail, :433-440
    }
    auto it = std::find(nic.begin(), nic.end(), r);
    if (it != nic.end()) {              // a port rank ends the chains of its own chunk, :316-331
        const uint32_t j = static_cast<uint32_t>(it - nic.begin());
        for (uint32_t c = 0; c < chunk; c++) {
            recv(j * chunk + c);
        }
    }
}

// All-reduce over an 8-rank ring whose network ports are fewer than its ranks: the port-pruned reduce-scatter on
// the input buffer, then the finished slices go round the ring from the port ranks.  The reference tree has no
// port-pruned all-gather template; this one is the reduce-scatter's mirror image and only moves bytes.
int RunAllReduceRingPruned(Machine &m, uint64_t bytes, uint64_t align, const std::vector<uint32_t> &nic)
{
    const uint32_t p = static_cast<uint32_t>(m.p);
    std::vector<Slice> sl = RingSlices(bytes, p, align);
    std::vector<std::vector<uint32_t>> lists = PrunedRingSendLists(p, nic);
    const uint32_t chunk = 8 / static_cast<uint32_t>(nic.size());
    for (uint32_t r = 0; r < p; r++) {
        Proc pr;
        pr.rank = r;
        ProgReduceScatterRingChunk(pr.prog, r, p, nic, lists, B_IN, sl);
        const uint32_t left = (r + p - 1) % p, right = (r + 1) % p;
        for (uint32_t i = 0; i < p; i++) {
            if (nic[i / chunk] == r) {
                pr.prog.push_back(MkLocalCopy(B_OUT, sl[i].off, B_IN, sl[i].off, sl[i].size));
            }
        }
        for (uint32_t k = 0; k + 1 < p; k++) {
            for (uint32_t i = 0; i < p; i++) {
                if ((nic[i / chunk] + k) % p == r) {          // holds slice i after k hops
                    pr.prog.push_back(MkSend(static_cast<int>(right), 1, B_OUT, sl[i].off, sl[i].size));
                }
            }
            for (uint32_t i = 0; i < p; i++) {
                if ((nic[i / chunk] + k) % p == left) {
                    pr.prog.push_back(MkRecvCopy(static_cast<int>(left), 1, B_OUT, sl[i].off, sl[i].size));
                }
            }
        }
        m.procs.push_back(std::move(pr));
    }
    return m.Run();
}

// CollAllReduceMeshExecutor::KernelRun, deterministic branch (coll_all_reduce_mesh_executor.cc:95-240).
int RunAllReduceMesh(Machine &m, uint64_t bytes, uint64_t align, bool atomic)
{
    uint32_t p = m.p;
    if (p == 1) {
        m.Copy(m.buf[B_OUT][0], m.buf[B_IN][0], bytes);
        return 0;
    }
    std::vector<Slice> sl = RingSlices(bytes, p, align);
    if (atomic) {
        // non-deterministic branch, coll_all_reduce_mesh_executor.cc:108-113
        for (uint32_t r = 0; r < p; r++) {
            Proc pr;
            pr.rank = r;
            ProgReduceScatterMeshAtomic(pr.prog, r, p, B_IN, sl);
            m.procs.push_back(std::move(pr));
        }
    } else if (p > 2) {
        std::vector<std::vector<Slice>> pieces = CutPieces(sl, p - 1, align);
        for (uint32_t t = 0; t < p - 1; t++) {
            for (uint32_t r = 0; r < p; r++) {
                Proc pr;
                pr.rank = r;
                ProgReduceScatterMeshStream(pr.prog, r, p, t, B_IN, pieces[t]);
                m.procs.push_back(std::move(pr));
            }
        }
    } else {
        for (uint32_t r = 0; r < p; r++) {
            Proc pr;
            pr.rank = r;
            ProgReduceScatterMeshStream(pr.prog, r, p, 0, B_IN, sl);
            m.procs.push_back(std::move(pr));
        }
    }
    int rc = m.Run();
    if (rc != 0) {
        return rc;
    }
    // one server: the level-1 all-reduce is a copy of the own slice from input to output
    for (uint32_t r = 0; r < p; r++) {
        m.Copy(m.At(r, B_OUT, sl[r].off), m.At(r, B_IN, sl[r].off), sl[r].size);
    }
    for (uint32_t r = 0; r < p; r++) {
        Proc pr;
        pr.rank = r;
        ProgAllGatherMesh(pr.prog, r, p, B_OUT, sl);
        m.procs.push_back(std::move(pr));
    }
    return m.Run();
}

// AllReduceRecursiveHalvingDoubling::RunAsync, all_reduce_recursive_hd.cc:33-302.
int RunAllReduceRhd(Machine &m, uint64_t bytes, uint64_t align)
{
    uint32_t p = m.p;
    if (p == 1) {
        m.Copy(m.buf[B_OUT][0], m.buf[B_IN][0], bytes);
        return 0;
    }
    uint32_t block, part1;
    RhdParams(p, &block, &part1);
    std::vector<Slice> sl = RhdSlices(bytes, block, align);
    std::vector<uint32_t> rankOf(block);
    for (uint32_t i = 0; i < p; i++) {
        if (i < part1 && (i % 2) == 1) {
            continue;
        }
        uint32_t q = (i < part1) ? i / 2 : i - part1 / 2;
        rankOf[q] = i;
    }
    for (uint32_t r = 0; r < p; r++) {
        Proc pr;
        pr.rank = r;
        bool inPart1 = r < part1;
        if (inPart1 && (r % 2) == 1) {
            // fold: send the whole input to the even neighbour; unfold: receive the whole output
            pr.prog.push_back(MkSend(static_cast<int>(r - 1), 1, B_IN, 0, bytes));
            pr.prog.push_back(MkRecvCopy(static_cast<int>(r - 1), 1, B_OUT, 0, bytes));
        } else {
            if (inPart1) {
                pr.prog.push_back(MkRecvReduce(static_cast<int>(r + 1), 1, B_IN, 0, B_IN, 0, bytes));
            }
            uint32_t q = inPart1 ? r / 2 : r - part1 / 2;
            ProgReduceScatterHd(pr.prog, q, block, rankOf, B_IN, B_OUT, sl);
            ProgAllGatherHd(pr.prog, q, block, rankOf, B_OUT, sl);
            if (inPart1) {
                pr.prog.push_back(MkSend(static_cast<int>(r + 1), 1, B_OUT, 0, bytes));
            }
        }
        m.procs.push_back(std::move(pr));
    }
    int rc = m.Run();
    // block == 1 cannot happen for p >= 2 (block >= 2); with block == 2^0 there would be no copy to out.
    return rc;
}

// Block-rank map and block slices of the standalone recursive halving-doubling reduce-scatter /
// all-gather: block ranks below part1/2 own two consecutive rank slices
// (reduce_scatter_recursive_hd.cc:86-110, all_gather_recursive_hd.cc:69-90).
void RhdBlockLayout(uint32_t p, uint64_t bytes, uint32_t *block, uint32_t *part1, std::vector<uint32_t> *rankOf,
    std::vector<Slice> *blockSlices)
{
    RhdParams(p, block, part1);
    rankOf->assign(*block, 0);
    for (uint32_t i = 0; i < p; i++) {
        if (i < *part1 && (i % 2) == 1) {
            continue;
        }
        (*rankOf)[(i < *part1) ? i / 2 : i - *part1 / 2] = i;
    }
    blockSlices->assign(*block, Slice{0, 0});
    uint32_t half = *part1 / 2;
    for (uint32_t b = 0; b < *block; b++) {
        if (b < half) {
            (*blockSlices)[b] = Slice{uint64_t(b) * 2 * bytes, 2 * bytes};
        } else {
            (*blockSlices)[b] = Slice{uint64_t(b) * bytes + uint64_t(half) * bytes, bytes};
        }
    }
}

int RunAllReduceTemplate(Machine &m, int algo, uint64_t bytes, uint64_t align)
{
    switch (algo) {
        case ALGO_RING: return RunAllReduceRing(m, bytes, align);
        case ALGO_MESH: return RunAllReduceMesh(m, bytes, align, false);
        case ALGO_MESH_ATOMIC: return RunAllReduceMesh(m, bytes, align, true);
        case ALGO_RHD: return RunAllReduceRhd(m, bytes, align);
        default: return -10;
    }
}

}  // namespace

// ================================================================================================
// C entry points (ctypes)
// ================================================================================================
extern "C" {

uint64_t orc_dtype_size(int dt) { return DtSize(dt); }

void orc_ring_slices(uint64_t total, uint32_t p, uint64_t align, uint64_t *off, uint64_t *size)
{
    std::vector<Slice> s = RingSlices(total, p, align);
    for (uint32_t i = 0; i < p; i++) {
        off[i] = s[i].off;
        size[i] = s[i].size;
    }
}

void orc_rhd_params(uint32_t p, uint32_t *block, uint32_t *part1) { RhdParams(p, block, part1); }

void orc_rhd_slices(uint64_t bytes, uint32_t block, uint64_t align, uint64_t *off, uint64_t *size)
{
    std::vector<Slice> s = RhdSlices(bytes, block, align);
    for (uint32_t i = 0; i < block; i++) {
        off[i] = s[i].off;
        size[i] = s[i].size;
    }
}

// pieces laid out [piece][rank]
void orc_cut_pieces(uint32_t nslices, const uint64_t *offIn, const uint64_t *sizeIn, uint32_t n, uint64_t align,
    uint64_t *off, uint64_t *size)
{
    std::vector<Slice> s(nslices);
    for (uint32_t i = 0; i < nslices; i++) {
        s[i] = Slice{offIn[i], sizeIn[i]};
    }
    auto out = CutPieces(s, n, align);
    for (uint32_t k = 0; k < n; k++) {
        for (uint32_t r = 0; r < nslices; r++) {
            off[k * nslices + r] = out[k][r].off;
            size[k * nslices + r] = out[k][r].size;
        }
    }
}

// kind: 0 all-reduce, 1 reduce-scatter, 2 all-gather.  Writes up to maxChunks chunk counts.
uint32_t orc_chunk_plan(int kind, uint64_t count, uint64_t unit, uint32_t p, uint64_t cclBytes, uint64_t align,
    uint32_t maxChunks, uint64_t *counts)
{
    uint64_t maxPer = MaxCountPerLoop(kind, cclBytes, p, unit, align);
    if (maxPer == 0) {
        return 0;
    }
    uint32_t n = 0;
    for (uint64_t left = count; left > 0;) {
        uint64_t cur = left > maxPer ? maxPer : left;
        if (n < maxChunks) {
            counts[n] = cur;
        }
        n++;
        left -= cur;
    }
    return n;
}

int orc_reduce(int dt, int op, void *dst, const void *a, const void *b, uint64_t n)
{
    return ReduceElems(dt, op, dst, a, b, n);
}

void orc_f32_to_bf16(const float *src, uint16_t *dst, uint64_t n) { for (uint64_t i = 0; i < n; i++) dst[i] = F32ToBf16(src[i]); }
void orc_bf16_to_f32(const uint16_t *src, float *dst, uint64_t n) { for (uint64_t i = 0; i < n; i++) dst[i] = Bf16ToF32(src[i]); }
void orc_f32_to_fp16(const float *src, uint16_t *dst, uint64_t n) { for (uint64_t i = 0; i < n; i++) dst[i] = F32ToFp16(src[i]); }
void orc_fp16_to_f32(const uint16_t *src, float *dst, uint64_t n) { for (uint64_t i = 0; i < n; i++) dst[i] = Fp16ToF32(src[i]); }

// flags: bit0 = direct (pointer) messages instead of snapshots,
//        bit1 = run the templates on the caller's buffers (no CCL staging copies; `in` is clobbered)
// Returns 0 on success.  `touched` (optional) receives the bytes read + written by all ranks.
int orc_allreduce(int algo, uint32_t p, void **in, void **out, uint64_t count, int dt, int op,
    uint64_t cclBytes, uint64_t align, int flags, int threads, uint64_t *touched)
{
    uint64_t unit = DtSize(dt);
    if (unit == 0 || p == 0 || cclBytes < unit) {
        return -20;
    }
    Pool pool(threads);
    Machine m;
    m.p = static_cast<int>(p);
    m.dt = dt;
    m.op = op;
    m.direct = (flags & 1) != 0;
    m.pool = &pool;
    bool zero = (flags & 2) != 0;
    uint64_t maxPer = MaxCountPerLoop(0, cclBytes, p, unit, align);
    uint64_t stage = std::min<uint64_t>(count, maxPer) * unit;
    std::vector<std::vector<uint8_t>> cclIn, cclOut;
    if (!zero) {
        cclIn.assign(p, std::vector<uint8_t>(stage));
        cclOut.assign(p, std::vector<uint8_t>(stage));
    }
    m.buf[B_IN].resize(p);
    m.buf[B_OUT].resize(p);
    uint64_t offset = 0;
    for (uint64_t left = count; left > 0;) {
        uint64_t cur = left > maxPer ? maxPer : left;
        uint64_t bytes = cur * unit;
        for (uint32_t r = 0; r < p; r++) {
            if (zero) {
                m.buf[B_IN][r] = static_cast<uint8_t *>(in[r]) + offset;
                m.buf[B_OUT][r] = static_cast<uint8_t *>(out[r]) + offset;
            } else {
                m.buf[B_IN][r] = cclIn[r].data();
                m.buf[B_OUT][r] = cclOut[r].data();
                m.Copy(m.buf[B_IN][r], static_cast<uint8_t *>(in[r]) + offset, bytes);
            }
        }
        int rc = RunAllReduceTemplate(m, algo, bytes, align);
        if (rc != 0) {
            return rc;
        }
        if (!zero) {
            for (uint32_t r = 0; r < p; r++) {
                m.Copy(static_cast<uint8_t *>(out[r]) + offset, m.buf[B_OUT][r], bytes);
            }
        }
        offset += bytes;
        left -= cur;
    }
    if (touched) {
        *touched = m.bytesTouched;
    }
    return 0;
}

// Ring all-reduce over 8 ranks of which only nic[0..nnic) (ascending, 1, 2 or 4 of them) own a network port: the
// executor's chunk loop around RunAllReduceRingPruned.  Flags as for orc_allreduce.
int orc_allreduce_ring_pruned(uint32_t p, void **in, void **out, uint64_t count, int dt, int op, const uint32_t *nic,
    uint32_t nnic, uint64_t cclBytes, uint64_t align, int flags, int threads)
{
    uint64_t unit = DtSize(dt);
    if (unit == 0 || p != 8 || cclBytes < unit || (nnic != 1 && nnic != 2 && nnic != 4)) {
        return -20;
    }
    std::vector<uint32_t> ports(nic, nic + nnic);
    for (uint32_t i = 0; i < nnic; i++) {
        if (ports[i] >= p || (i > 0 && ports[i] <= ports[i - 1])) {
            return -20;
        }
    }
    Pool pool(threads);
    Machine m;
    m.p = static_cast<int>(p);
    m.dt = dt;
    m.op = op;
    m.direct = (flags & 1) != 0;
    m.pool = &pool;
    bool zero = (flags & 2) != 0;
    uint64_t maxPer = MaxCountPerLoop(0, cclBytes, p, unit, align);
    uint64_t stage = std::min<uint64_t>(count, maxPer) * unit;
    std::vector<std::vector<uint8_t>> cclIn, cclOut;
    if (!zero) {
        cclIn.assign(p, std::vector<uint8_t>(stage));
        cclOut.assign(p, std::vector<uint8_t>(stage));
    }
    m.buf[B_IN].resize(p);
    m.buf[B_OUT].resize(p);
    uint64_t offset = 0;
    for (uint64_t left = count; left > 0;) {
        uint64_t cur = left > maxPer ? maxPer : left;
        uint64_t bytes = cur * unit;
        for (uint32_t r = 0; r < p; r++) {
            if (zero) {
                m.buf[B_IN][r] = static_cast<uint8_t *>(in[r]) + offset;
                m.buf[B_OUT][r] = static_cast<uint8_t *>(out[r]) + offset;
            } else {
                m.buf[B_IN][r] = cclIn[r].data();
                m.buf[B_OUT][r] = cclOut[r].data();
                m.Copy(m.buf[B_IN][r], static_cast<uint8_t *>(in[r]) + offset, bytes);
            }
        }
        int rc = RunAllReduceRingPruned(m, bytes, align, ports);
        if (rc != 0) {
            return rc;
        }
        if (!zero) {
            for (uint32_t r = 0; r < p; r++) {
                m.Copy(static_cast<uint8_t *>(out[r]) + offset, m.buf[B_OUT][r], bytes);
            }
        }
        offset += bytes;
        left -= cur;
    }
    return 0;
}

// MutliSegSlicePrepare (EXE/coll_comm_executor.cc:1681-1720): every rank slice is cut into ringCount parts of
// RoundUp(ceil(size / ringCount), align) bytes, the last one shorter; parts that are left get size 0.
std::vector<std::vector<Slice>> MultiSegSlices(const std::vector<Slice> &dataSegs, uint32_t ringCount, uint64_t align)
{
    std::vector<std::vector<Slice>> all;
    for (const Slice &seg : dataSegs) {
        std::vector<Slice> one;
        uint32_t ringIndex = 0;
        if (seg.size > 0) {
            uint64_t per = (seg.size + ringCount - 1) / ringCount;
            per = (per + align - 1) / align * align;
            uint64_t residue = seg.size;
            while (residue > 0) {
                uint64_t sz = per < residue ? per : residue;
                one.push_back(Slice{seg.off + seg.size - residue, sz});
                residue -= sz;
                ringIndex++;
            }
        }
        for (; ringIndex < ringCount; ringIndex++) {
            one.push_back(Slice{seg.off, 0});
        }
        all.push_back(one);
    }
    return all;
}

// PrepareMultiRingSlice with every device on the network list (EXE/coll_comm_executor.cc:1761-1833): ring k
// visits the devices in order[k]; its member i works on part k of the slice of device order[k][i].
// Ring orders of the 8-device ring topology: GetRingsOrderByTopoType, :1595-1606.
const uint32_t kEightDeviceRings[4][8] = {
    {0, 1, 2, 6, 5, 4, 7, 3}, {0, 3, 7, 4, 5, 6, 2, 1}, {0, 2, 3, 1, 5, 7, 6, 4}, {0, 4, 6, 7, 5, 1, 3, 2}};

// Two-level all-reduce: `servers` groups of D = p / servers consecutive ranks.
//   level0 = 0 / 1   CollAllReduceMeshExecutor::KernelRun (EXE/coll_all_reduce/coll_all_reduce_mesh_executor.cc:95-240):
//                    mesh reduce-scatter inside every group (piece cut, or uncut when 1), mesh all-gather at the end
//   level0 = 2 / 3   CollAllReduceRingExecutor::KernelRun (EXE/coll_all_reduce/coll_all_reduce_ring_executor.cc:95-243):
//                    ring reduce-scatter inside every group on the input buffer and ring all-gather on the output,
//                    over one ring in rank order (2) or the four rings of the 8-device topology (3, D = 8)
// In between, the ranks with the same position in their groups all-reduce their slice among themselves
// (level1 = ALGO_RING or ALGO_RHD) from the input range to the output range.  Chunk loop and staging as in
// orc_allreduce.
int orc_allreduce_two_level(int level1, int level0, uint32_t servers, uint32_t p, void **in, void **out, uint64_t count, int dt,
    int op, uint64_t cclBytes, uint64_t align, int flags, int threads)
{
    uint64_t unit = DtSize(dt);
    if (unit == 0 || p == 0 || servers == 0 || p % servers != 0 || cclBytes < unit || (level1 != ALGO_RING && level1 != ALGO_RHD) ||
        level0 < 0 || level0 > 3 || (level0 == 3 && p / servers != 8)) {
        return -20;
    }
    const uint32_t D = p / servers;
    const bool atomic = level0 == 1;
    const uint32_t ringCount = level0 == 3 ? 4u : 1u;
    Pool pool(threads);
    auto machine = [&](uint32_t n) {
        Machine m;
        m.p = static_cast<int>(n);
        m.dt = dt;
        m.op = op;
        m.direct = (flags & 1) != 0;
        m.pool = &pool;
        m.buf[B_IN].resize(n);
        m.buf[B_OUT].resize(n);
        return m;
    };
    Machine all = machine(p);
    uint64_t maxPer = MaxCountPerLoop(0, cclBytes, p, unit, align);
    uint64_t stage = std::min<uint64_t>(count, maxPer) * unit;
    std::vector<std::vector<uint8_t>> cclIn(p, std::vector<uint8_t>(stage)), cclOut(p, std::vector<uint8_t>(stage));
    for (uint32_t r = 0; r < p; r++) {
        all.buf[B_IN][r] = cclIn[r].data();
        all.buf[B_OUT][r] = cclOut[r].data();
    }
    uint64_t offset = 0;
    for (uint64_t left = count; left > 0;) {
        uint64_t cur = left > maxPer ? maxPer : left;
        uint64_t bytes = cur * unit;
        for (uint32_t r = 0; r < p; r++) {
            all.Copy(all.buf[B_IN][r], static_cast<uint8_t *>(in[r]) + offset, bytes);
        }
        std::vector<Slice> sl = RingSlices(bytes, D, align);
        // level 0: reduce-scatter inside every group
        for (uint32_t s = 0; s < servers && D > 1; s++) {
            Machine m = machine(D);
            for (uint32_t d = 0; d < D; d++) {
                m.buf[B_IN][d] = all.buf[B_IN][s * D + d];
                m.buf[B_OUT][d] = all.buf[B_OUT][s * D + d];
            }
            if (level0 >= 2) {
                // one sub-machine per ring: member i is device order[k][i]
                std::vector<std::vector<Slice>> segs = MultiSegSlices(sl, ringCount, align);
                for (uint32_t k = 0; k < ringCount; k++) {
                    Machine ring = machine(D);
                    std::vector<Slice> ringSl(D);
                    for (uint32_t i = 0; i < D; i++) {
                        uint32_t dev = ringCount > 1 ? kEightDeviceRings[k][i] : i;
                        ring.buf[B_IN][i] = m.buf[B_IN][dev];
                        ring.buf[B_OUT][i] = m.buf[B_OUT][dev];
                        ringSl[i] = segs[dev][k];
                    }
                    for (uint32_t i = 0; i < D; i++) {
                        Proc pr;
                        pr.rank = i;
                        ProgReduceScatterRing(pr.prog, i, D, B_IN, B_IN, ringSl, ringSl);
                        ring.procs.push_back(std::move(pr));
                    }
                    int rc = ring.Run();
                    if (rc != 0) {
                        return rc;
                    }
                }
                continue;
            }
            if (atomic) {
                for (uint32_t d = 0; d < D; d++) {
                    Proc pr;
                    pr.rank = d;
                    ProgReduceScatterMeshAtomic(pr.prog, d, D, B_IN, sl);
                    m.procs.push_back(std::move(pr));
                }
            } else {
                uint32_t nstream = D > 2 ? D - 1 : 1;
                std::vector<std::vector<Slice>> pieces = CutPieces(sl, nstream, align);
                for (uint32_t t = 0; t < nstream; t++) {
                    for (uint32_t d = 0; d < D; d++) {
                        Proc pr;
                        pr.rank = d;
                        ProgReduceScatterMeshStream(pr.prog, d, D, t, B_IN, pieces[t]);
                        m.procs.push_back(std::move(pr));
                    }
                }
            }
            int rc = m.Run();
            if (rc != 0) {
                return rc;
            }
        }
        // level 1: all-reduce of slice d among the ranks at position d of every group
        for (uint32_t d = 0; d < D; d++) {
            Machine m = machine(servers);
            for (uint32_t s = 0; s < servers; s++) {
                m.buf[B_IN][s] = all.buf[B_IN][s * D + d] + sl[d].off;
                m.buf[B_OUT][s] = all.buf[B_OUT][s * D + d] + sl[d].off;
            }
            if (sl[d].size == 0) {
                continue;
            }
            int rc = RunAllReduceTemplate(m, level1, sl[d].size, align);
            if (rc != 0) {
                return rc;
            }
        }
        // level 0: all-gather inside every group
        for (uint32_t s = 0; s < servers && D > 1; s++) {
            Machine m = machine(D);
            for (uint32_t d = 0; d < D; d++) {
                m.buf[B_IN][d] = all.buf[B_IN][s * D + d];
                m.buf[B_OUT][d] = all.buf[B_OUT][s * D + d];
            }
            if (level0 >= 2) {
                std::vector<std::vector<Slice>> segs = MultiSegSlices(sl, ringCount, align);
                for (uint32_t k = 0; k < ringCount; k++) {
                    Machine ring = machine(D);
                    std::vector<Slice> ringSl(D);
                    for (uint32_t i = 0; i < D; i++) {
                        uint32_t dev = ringCount > 1 ? kEightDeviceRings[k][i] : i;
                        ring.buf[B_IN][i] = m.buf[B_IN][dev];
                        ring.buf[B_OUT][i] = m.buf[B_OUT][dev];
                        ringSl[i] = segs[dev][k];
                    }
                    for (uint32_t i = 0; i < D; i++) {
                        Proc pr;
                        pr.rank = i;
                        ProgAllGatherRing(pr.prog, i, D, B_OUT, B_OUT, ringSl, ringSl);
                        ring.procs.push_back(std::move(pr));
                    }
                    int rc = ring.Run();
                    if (rc != 0) {
                        return rc;
                    }
                }
                continue;
            }
            for (uint32_t d = 0; d < D; d++) {
                Proc pr;
                pr.rank = d;
                ProgAllGatherMesh(pr.prog, d, D, B_OUT, sl);
                m.procs.push_back(std::move(pr));
            }
            int rc = m.Run();
            if (rc != 0) {
                return rc;
            }
        }
        for (uint32_t r = 0; r < p; r++) {
            all.Copy(static_cast<uint8_t *>(out[r]) + offset, all.buf[B_OUT][r], bytes);
        }
        offset += bytes;
        left -= cur;
    }
    return 0;
}


// ReduceScatterRecursiveHalvingDoubling::RunAsync, reduce_scatter_recursive_hd.cc:33-254, on the machine's
// input buffers (m.p slices of `bytes` bytes each), in place.
void AddReduceScatterRhdProcs(Machine &m, uint64_t bytes)
{
    const uint32_t p = static_cast<uint32_t>(m.p);
    uint32_t block, part1;
    std::vector<uint32_t> rankOf;
    std::vector<Slice> bsl;
    RhdBlockLayout(p, bytes, &block, &part1, &rankOf, &bsl);
    for (uint32_t r = 0; r < p; r++) {
        Proc pr;
        pr.rank = r;
        if (r < part1 && (r % 2) == 1) {
            pr.prog.push_back(MkSend(static_cast<int>(r - 1), 1, B_IN, 0, bytes * p));
            pr.prog.push_back(MkRecvCopy(static_cast<int>(r - 1), 1, B_IN, bytes * r, bytes));
        } else {
            if (r < part1) {
                pr.prog.push_back(MkRecvReduce(static_cast<int>(r + 1), 1, B_IN, 0, B_IN, 0, bytes * p));
            }
            uint32_t q = (r < part1) ? r / 2 : r - part1 / 2;
            ProgReduceScatterHd(pr.prog, q, block, rankOf, B_IN, B_IN, bsl);
            if (r < part1) {
                pr.prog.push_back(MkSend(static_cast<int>(r + 1), 1, B_IN, bytes * (r + 1), bytes));
            }
        }
        m.procs.push_back(std::move(pr));
    }
}

// in[r]: p * recvCount elements, out[r]: recvCount elements.  Ring only at this level
// (coll_reduce_scatter_comm_executor.cc:196-209); mesh uses the same slices with the mesh template.
int orc_reducescatter(int algo, uint32_t p, void **in, void **out, uint64_t recvCount, int dt, int op,
    uint64_t cclBytes, uint64_t align, int flags, int threads)
{
    uint64_t unit = DtSize(dt);
    if (unit == 0 || p == 0) {
        return -20;
    }
    uint64_t maxPer = MaxCountPerLoop(1, cclBytes, p, unit, align);
    if (maxPer == 0) {
        return -21;
    }
    Pool pool(threads);
    Machine m;
    m.p = static_cast<int>(p);
    m.dt = dt;
    m.op = op;
    m.direct = (flags & 1) != 0;
    m.pool = &pool;
    uint64_t stage = std::min<uint64_t>(recvCount, maxPer) * unit;
    std::vector<std::vector<uint8_t>> cclIn(p, std::vector<uint8_t>(stage * p)), cclOut(p, std::vector<uint8_t>(stage));
    m.buf[B_IN].resize(p);
    m.buf[B_OUT].resize(p);
    for (uint32_t r = 0; r < p; r++) {
        m.buf[B_IN][r] = cclIn[r].data();
        m.buf[B_OUT][r] = cclOut[r].data();
    }
    uint64_t offset = 0;
    for (uint64_t left = recvCount; left > 0;) {
        uint64_t cur = left > maxPer ? maxPer : left;
        uint64_t bytes = cur * unit;
        for (uint32_t r = 0; r < p; r++) {
            for (uint32_t i = 0; i < p; i++) {
                m.Copy(m.buf[B_IN][r] + bytes * i, static_cast<uint8_t *>(in[r]) + recvCount * unit * i + offset, bytes);
            }
        }
        std::vector<Slice> sl(p);
        for (uint32_t i = 0; i < p; i++) {
            sl[i] = Slice{bytes * i, bytes};
        }
        if (p > 1) {
            if (algo == ALGO_RING) {
                for (uint32_t r = 0; r < p; r++) {
                    Proc pr;
                    pr.rank = r;
                    ProgReduceScatterRing(pr.prog, r, p, B_IN, B_IN, sl, sl);
                    m.procs.push_back(std::move(pr));
                }
            } else if (algo == ALGO_MESH_ATOMIC) {
                // coll_reduce_scatter_mesh_executor.cc:227-232
                for (uint32_t r = 0; r < p; r++) {
                    Proc pr;
                    pr.rank = r;
                    ProgReduceScatterMeshAtomic(pr.prog, r, p, B_IN, sl);
                    m.procs.push_back(std::move(pr));
                }
            } else if (algo == ALGO_MESH) {
                uint32_t nstream = p > 2 ? p - 1 : 1;
                std::vector<std::vector<Slice>> pieces = CutPieces(sl, nstream, align);
                for (uint32_t t = 0; t < nstream; t++) {
                    for (uint32_t r = 0; r < p; r++) {
                        Proc pr;
                        pr.rank = r;
                        ProgReduceScatterMeshStream(pr.prog, r, p, t, B_IN, pieces[t]);
                        m.procs.push_back(std::move(pr));
                    }
                }
            } else if (algo == ALGO_RHD) {
                AddReduceScatterRhdProcs(m, bytes);
            } else {
                return -10;
            }
            int rc = m.Run();
            if (rc != 0) {
                return rc;
            }
        }
        for (uint32_t r = 0; r < p; r++) {
            m.Copy(m.buf[B_OUT][r], m.buf[B_IN][r] + bytes * r, bytes);
            m.Copy(static_cast<uint8_t *>(out[r]) + offset, m.buf[B_OUT][r], bytes);
        }
        offset += bytes;
        left -= cur;
    }
    return 0;
}

// Two-level reduce-scatter, CollReduceScatterMeshExecutor::KernelRun with several servers
// (EXE/coll_reduce_scatter/coll_reduce_scatter_mesh_executor.cc:128-247): `servers` groups of D = p / servers
// consecutive ranks.  First the ranks with the same position in their groups reduce-scatter the whole staged
// input among themselves (level1 = ALGO_RING or ALGO_RHD; a group's slice is the D blocks for its ranks), in
// place; then the reduce-scatter inside every group over that slice: level0 0 / 1 the mesh (piece cut / uncut),
// 2 / 3 one ring in rank order / the four rings of the 8-device topology (the ring executor);
// then the rank's block goes to the output.  Chunks of cclBytes / (p * unit) elements (:114-119).
int orc_reducescatter_two_level(int level1, int level0, uint32_t servers, uint32_t p, void **in, void **out, uint64_t recvCount,
    int dt, int op, uint64_t cclBytes, uint64_t align, int flags, int threads)
{
    uint64_t unit = DtSize(dt);
    if (unit == 0 || p == 0 || servers == 0 || p % servers != 0 || (level1 != ALGO_RING && level1 != ALGO_RHD) || level0 < 0 ||
        level0 > 3 || (level0 == 3 && p / servers != 8)) {
        return -20;
    }
    const uint32_t D = p / servers;
    const bool atomic = level0 == 1;
    const uint32_t ringCount = level0 == 3 ? 4u : 1u;
    uint64_t maxPer = cclBytes / (uint64_t(p) * unit);
    if (maxPer == 0) {
        return -21;
    }
    Pool pool(threads);
    auto machine = [&](uint32_t n) {
        Machine m;
        m.p = static_cast<int>(n);
        m.dt = dt;
        m.op = op;
        m.direct = (flags & 1) != 0;
        m.pool = &pool;
        m.buf[B_IN].resize(n);
        m.buf[B_OUT].resize(n);
        return m;
    };
    Machine all = machine(p);
    uint64_t stage = std::min<uint64_t>(recvCount, maxPer) * unit;
    std::vector<std::vector<uint8_t>> cclIn(p, std::vector<uint8_t>(stage * p)), cclOut(p, std::vector<uint8_t>(stage));
    for (uint32_t r = 0; r < p; r++) {
        all.buf[B_IN][r] = cclIn[r].data();
        all.buf[B_OUT][r] = cclOut[r].data();
    }
    uint64_t offset = 0;
    for (uint64_t left = recvCount; left > 0;) {
        uint64_t cur = left > maxPer ? maxPer : left;
        uint64_t bytes = cur * unit;
        for (uint32_t r = 0; r < p; r++) {
            for (uint32_t i = 0; i < p; i++) {
                all.Copy(all.buf[B_IN][r] + bytes * i, static_cast<uint8_t *>(in[r]) + recvCount * unit * i + offset, bytes);
            }
        }
        const uint64_t serverSlice = bytes * D;          // inputMem.size() / level1RankSize
        // level 1: between the groups, for every position d
        for (uint32_t d = 0; d < D && servers > 1; d++) {
            Machine m = machine(servers);
            for (uint32_t s = 0; s < servers; s++) {
                m.buf[B_IN][s] = all.buf[B_IN][s * D + d];
                m.buf[B_OUT][s] = all.buf[B_OUT][s * D + d];
            }
            if (level1 == ALGO_RING) {
                std::vector<Slice> sl(servers);
                for (uint32_t s = 0; s < servers; s++) {
                    sl[s] = Slice{serverSlice * s, serverSlice};
                }
                for (uint32_t s = 0; s < servers; s++) {
                    Proc pr;
                    pr.rank = s;
                    ProgReduceScatterRing(pr.prog, s, servers, B_IN, B_IN, sl, sl);
                    m.procs.push_back(std::move(pr));
                }
            } else {
                AddReduceScatterRhdProcs(m, serverSlice);
            }
            int rc = m.Run();
            if (rc != 0) {
                return rc;
            }
        }
        // level 0: mesh inside every group, on the group's slice of the input
        for (uint32_t s = 0; s < servers && D > 1; s++) {
            Machine m = machine(D);
            for (uint32_t d = 0; d < D; d++) {
                m.buf[B_IN][d] = all.buf[B_IN][s * D + d] + serverSlice * s;
                m.buf[B_OUT][d] = all.buf[B_OUT][s * D + d];
            }
            std::vector<Slice> sl(D);
            for (uint32_t d = 0; d < D; d++) {
                sl[d] = Slice{bytes * d, bytes};
            }
            if (level0 >= 2) {
                // CollReduceScatterRingExecutor::KernelRun (EXE/coll_reduce_scatter/coll_reduce_scatter_ring_executor.cc:
                // 280-340) with the slices of ReduceScatterRingSlicePrepare (EXE/coll_reduce_scatter/
                // coll_reduce_scatter_executor.cc:250-287): the D blocks, cut into one part per ring
                std::vector<std::vector<Slice>> segs = MultiSegSlices(sl, ringCount, align);
                for (uint32_t k = 0; k < ringCount; k++) {
                    Machine ring = machine(D);
                    std::vector<Slice> ringSl(D);
                    for (uint32_t i = 0; i < D; i++) {
                        uint32_t dev = ringCount > 1 ? kEightDeviceRings[k][i] : i;
                        ring.buf[B_IN][i] = m.buf[B_IN][dev];
                        ring.buf[B_OUT][i] = m.buf[B_OUT][dev];
                        ringSl[i] = segs[dev][k];
                    }
                    for (uint32_t i = 0; i < D; i++) {
                        Proc pr;
                        pr.rank = i;
                        ProgReduceScatterRing(pr.prog, i, D, B_IN, B_IN, ringSl, ringSl);
                        ring.procs.push_back(std::move(pr));
                    }
                    int rc = ring.Run();
                    if (rc != 0) {
                        return rc;
                    }
                }
                continue;
            }
            if (atomic) {
                for (uint32_t d = 0; d < D; d++) {
                    Proc pr;
                    pr.rank = d;
                    ProgReduceScatterMeshAtomic(pr.prog, d, D, B_IN, sl);
                    m.procs.push_back(std::move(pr));
                }
            } else {
                uint32_t nstream = D > 2 ? D - 1 : 1;
                std::vector<std::vector<Slice>> pieces = CutPieces(sl, nstream, align);
                for (uint32_t t = 0; t < nstream; t++) {
                    for (uint32_t d = 0; d < D; d++) {
                        Proc pr;
                        pr.rank = d;
                        ProgReduceScatterMeshStream(pr.prog, d, D, t, B_IN, pieces[t]);
                        m.procs.push_back(std::move(pr));
                    }
                }
            }
            int rc = m.Run();
            if (rc != 0) {
                return rc;
            }
        }
        for (uint32_t r = 0; r < p; r++) {
            all.Copy(all.buf[B_OUT][r], all.buf[B_IN][r] + bytes * r, bytes);
            all.Copy(static_cast<uint8_t *>(out[r]) + offset, all.buf[B_OUT][r], bytes);
        }
        offset += bytes;
        left -= cur;
    }
    return 0;
}

// Send lists of the multi-root ring scatter, MultiRootScatterRing::MultiRootScatterSlicesPrep
// (TPL/temp_scatter/multi_root_scatter_ring.cc:299-345): slice j leaves the ring position of port j / chunk and stops at
// position (j + first port position) % 8; a position forwards the slices that pass through it, the farthest first.
std::vector<std::vector<uint32_t>> MultiRootScatterLists(const std::vector<uint32_t> &nicPos)
{
    const uint32_t n = 8, chunk = n / static_cast<uint32_t>(nicPos.size());
    struct Range {
        uint32_t slice, start, end;
    };
    std::vector<Range> ranges;
    for (uint32_t i = 0; i < nicPos.size(); i++) {
        for (uint32_t c = 0; c < chunk; c++) {
            Range g{i * chunk + c, nicPos[i], (i * chunk + c + nicPos[0]) % n};
            if (g.end < g.start) {
                g.end += n;
            }
            ranges.push_back(g);
        }
    }
    std::vector<std::vector<uint32_t>> lists;
    for (uint32_t pos = 0; pos < n; pos++) {
        std::vector<std::pair<uint32_t, uint32_t>> mine;     // (hops still to go, slice)
        for (size_t i = ranges.size(); i-- > 0;) {
            const Range &g = ranges[i];
            const uint32_t at = pos >= g.start ? pos : pos + n;
            if (at < g.end) {
                mine.emplace_back(g.end - at, g.slice);
            }
        }
        std::sort(mine.begin(), mine.end(), [](const std::pair<uint32_t, uint32_t> &a, const std::pair<uint32_t, uint32_t> &b) {
            return a.first > b.first;
        });
        std::vector<uint32_t> one;
        for (const auto &e : mine) {
            one.push_back(e.second);
        }
        lists.push_back(one);
    }
    return lists;
}

// Per-position program of MultiRootScatterRing::RunMultiRootScatterChunk (multi_root_scatter_ring.cc:100-140) with
// HeadScatterChunk (:142-205), MidScatterChunk (:207-246) and TailScatterChunk (:248-297); the data lies in buffer b at
// base + slice offset on both sides of a transfer.
void ProgMultiRootScatter(std::vector<Action> &pg, uint32_t pos, const std::vector<uint32_t> &nicPos,
    const std::vector<std::vector<uint32_t>> &lists, int b, uint64_t base, const std::vector<Slice> &sl)
{
    const uint32_t n = 8, left = (pos + n - 1) % n, right = (pos + 1) % n;
    const std::vector<uint32_t> &mine = lists[pos], &prev = lists[left];
    auto inPrev = [&](uint32_t s) { return std::find(prev.begin(), prev.end(), s) != prev.end(); };
    auto send = [&](uint32_t s) { pg.push_back(MkSend(static_cast<int>(right), 0, b, base + sl[s].off, sl[s].size)); };
    auto recv = [&](uint32_t s) { pg.push_back(MkRecvCopy(static_cast<int>(left), 0, b, base + sl[s].off, sl[s].size)); };
    const uint32_t own = (pos + n - nicPos[0]) % n;          // the slice this position keeps
    const uint32_t len = static_cast<uint32_t>(mine.size());
    auto mid = [&](uint32_t idx) {
        send(mine[idx]);
        if (inPrev(mine[idx + 1])) {
            recv(mine[idx + 1]);
        }
    };
    if (len == 0) {
        if (inPrev(own)) {
            recv(own);
        }
        return;
    }
    // head
    bool headDone = false;
    if (inPrev(mine[0])) {
        recv(mine[0]);
    }
    if (len >= 2) {
        if (inPrev(mine[1])) {
            mid(0);
            headDone = true;
        }
    } else if (inPrev(mine[0])) {       // the only slice: head and tail at once
        send(mine[0]);
        recv(own);
        headDone = true;
    }
    if (!headDone) {
        send(mine[0]);
    }
    for (uint32_t idx = 1; idx + 1 < len; idx++) {
        mid(idx);
    }
    if (len >= 2) {                     // tail
        send(mine[len - 1]);
        if (inPrev(own)) {
            recv(own);
        }
    }
}

// Two-level ring reduce-scatter over servers of 8 devices of which only some have a network port: the isMultiNic
// branch of CollReduceScatterRingExecutor::KernelRun (EXE/coll_reduce_scatter/coll_reduce_scatter_ring_executor.cc:
// 150-170, 264-300) with the ring between the servers.  Per chunk of the loop:
//   1. all-reduce of the whole staged input inside every server over the four rings of the 8-device topology
//      (MultiRingAllReduce, EXE/coll_comm_executor.cc:44-170; slices PrepareSliceData over the whole input, then one
//      part per ring), into the scratch buffer and back to the input buffer (:160-168)
//   2. the devices with a port reduce-scatter the whole input among the same devices of all servers (:172-191);
//      the others skip this step
//   3. input buffer -> scratch (:288-291), then the port devices hand the blocks of the server's slice to the devices
//      they belong to, part k of every block along ring k (MultiRingMultiRootScatter, EXE/coll_comm_executor.cc:
//      1312-1415 with the slices of ReduceScatterRingSlicePrepare rotated by the first port's ring position, :264-273)
//   4. the device's own block of the scratch buffer goes to the output (:298-299, :343-345)
// nic: device numbers 0..7 with a port, ascending; 1, 2 or 4 of them.
int orc_reducescatter_two_level_pruned(uint32_t servers, uint32_t p, void **in, void **out, uint64_t recvCount, int dt, int op,
    const uint32_t *nic, uint32_t nNic, uint64_t cclBytes, uint64_t align, int flags, int threads)
{
    uint64_t unit = DtSize(dt);
    if (unit == 0 || servers == 0 || p != servers * 8 || (nNic != 1 && nNic != 2 && nNic != 4)) {
        return -20;
    }
    for (uint32_t i = 0; i < nNic; i++) {
        if (nic[i] > 7 || (i > 0 && nic[i] <= nic[i - 1])) {
            return -20;
        }
    }
    const uint32_t D = 8, ringCount = 4;
    uint64_t maxPer = cclBytes / (uint64_t(p) * unit);
    if (maxPer == 0) {
        return -21;
    }
    Pool pool(threads);
    auto machine = [&](uint32_t n) {
        Machine m;
        m.p = static_cast<int>(n);
        m.dt = dt;
        m.op = op;
        m.direct = (flags & 1) != 0;
        m.pool = &pool;
        m.buf[B_IN].resize(n);
        m.buf[B_OUT].resize(n);
        return m;
    };
    Machine all = machine(p);          // B_IN: the staged input, B_OUT: the scratch buffer of the same size
    uint64_t stage = std::min<uint64_t>(recvCount, maxPer) * unit;
    std::vector<std::vector<uint8_t>> cclIn(p, std::vector<uint8_t>(stage * p)), scratch(p, std::vector<uint8_t>(stage * p));
    for (uint32_t r = 0; r < p; r++) {
        all.buf[B_IN][r] = cclIn[r].data();
        all.buf[B_OUT][r] = scratch[r].data();
    }
    uint64_t offset = 0;
    for (uint64_t left = recvCount; left > 0;) {
        uint64_t cur = left > maxPer ? maxPer : left;
        uint64_t bytes = cur * unit, whole = bytes * p;
        for (uint32_t r = 0; r < p; r++) {
            for (uint32_t i = 0; i < p; i++) {
                all.Copy(all.buf[B_IN][r] + bytes * i, static_cast<uint8_t *>(in[r]) + recvCount * unit * i + offset, bytes);
            }
        }
        // 1. all-reduce inside every server
        std::vector<std::vector<Slice>> segs = MultiSegSlices(RingSlices(whole, D, align), ringCount, align);
        for (uint32_t s = 0; s < servers; s++) {
            for (uint32_t k = 0; k < ringCount; k++) {
                Machine ring = machine(D);
                std::vector<Slice> ringSl(D);
                for (uint32_t i = 0; i < D; i++) {
                    const uint32_t dev = kEightDeviceRings[k][i];
                    ring.buf[B_IN][i] = all.buf[B_IN][s * D + dev];
                    ring.buf[B_OUT][i] = all.buf[B_OUT][s * D + dev];
                    ringSl[i] = segs[dev][k];
                }
                for (uint32_t i = 0; i < D; i++) {
                    Proc pr;
                    pr.rank = i;
                    ProgReduceScatterRing(pr.prog, i, D, B_IN, B_IN, ringSl, ringSl);
                    ProgAllGatherRing(pr.prog, i, D, B_IN, B_OUT, ringSl, ringSl);
                    ring.procs.push_back(std::move(pr));
                }
                int rc = ring.Run();
                if (rc != 0) {
                    return rc;
                }
            }
            for (uint32_t d = 0; d < D; d++) {
                all.Copy(all.buf[B_IN][s * D + d], all.buf[B_OUT][s * D + d], whole);
            }
        }
        // 2. between the servers, port devices only
        const uint64_t serverSlice = bytes * D;
        for (uint32_t i = 0; i < nNic && servers > 1; i++) {
            Machine m = machine(servers);
            std::vector<Slice> sl(servers);
            for (uint32_t s = 0; s < servers; s++) {
                m.buf[B_IN][s] = all.buf[B_IN][s * D + nic[i]];
                m.buf[B_OUT][s] = all.buf[B_OUT][s * D + nic[i]];
                sl[s] = Slice{serverSlice * s, serverSlice};
            }
            for (uint32_t s = 0; s < servers; s++) {
                Proc pr;
                pr.rank = s;
                ProgReduceScatterRing(pr.prog, s, servers, B_IN, B_IN, sl, sl);
                m.procs.push_back(std::move(pr));
            }
            int rc = m.Run();
            if (rc != 0) {
                return rc;
            }
        }
        // 3. scatter inside every server from the port devices
        std::vector<Slice> blocks(D);
        for (uint32_t d = 0; d < D; d++) {
            blocks[d] = Slice{bytes * d, bytes};
        }
        std::vector<std::vector<Slice>> parts = MultiSegSlices(blocks, ringCount, align);
        for (uint32_t s = 0; s < servers; s++) {
            for (uint32_t d = 0; d < D; d++) {
                all.Copy(all.buf[B_OUT][s * D + d], all.buf[B_IN][s * D + d], whole);
            }
            for (uint32_t k = 0; k < ringCount; k++) {
                std::vector<uint32_t> nicPos;
                for (uint32_t i = 0; i < D; i++) {
                    if (std::find(nic, nic + nNic, kEightDeviceRings[k][i]) != nic + nNic) {
                        nicPos.push_back(i);
                    }
                }
                Machine ring = machine(D);
                std::vector<Slice> ringSl(D);
                for (uint32_t i = 0; i < D; i++) {
                    const uint32_t dev = kEightDeviceRings[k][i];
                    ring.buf[B_IN][i] = all.buf[B_IN][s * D + dev];
                    ring.buf[B_OUT][i] = all.buf[B_OUT][s * D + dev];
                    ringSl[i] = parts[kEightDeviceRings[k][(i + nicPos[0]) % D]][k];      // rotated by the first port
                }
                std::vector<std::vector<uint32_t>> lists = MultiRootScatterLists(nicPos);
                for (uint32_t i = 0; i < D; i++) {
                    Proc pr;
                    pr.rank = i;
                    ProgMultiRootScatter(pr.prog, i, nicPos, lists, B_OUT, serverSlice * s, ringSl);
                    ring.procs.push_back(std::move(pr));
                }
                int rc = ring.Run();
                if (rc != 0) {
                    return rc;
                }
            }
        }
        // 4. the own block
        for (uint32_t r = 0; r < p; r++) {
            all.Copy(static_cast<uint8_t *>(out[r]) + offset, all.buf[B_OUT][r] + bytes * r, bytes);
        }
        offset += bytes;
        left -= cur;
    }
    return 0;
}

// in[r]: sendCount elements, out[r]: p * sendCount elements.
int orc_allgather(int algo, uint32_t p, void **in, void **out, uint64_t sendCount, int dt,
    uint64_t cclBytes, uint64_t align, int flags, int threads)
{
    uint64_t unit = DtSize(dt);
    if (unit == 0 || p == 0) {
        return -20;
    }
    uint64_t maxPer = MaxCountPerLoop(2, cclBytes, p, unit, align);
    if (maxPer == 0) {
        return -21;
    }
    Pool pool(threads);
    Machine m;
    m.p = static_cast<int>(p);
    m.dt = dt;
    m.op = 0;
    m.direct = (flags & 1) != 0;
    m.pool = &pool;
    uint64_t stage = std::min<uint64_t>(sendCount, maxPer) * unit;
    std::vector<std::vector<uint8_t>> cclIn(p, std::vector<uint8_t>(stage)), cclOut(p, std::vector<uint8_t>(stage * p));
    m.buf[B_IN].resize(p);
    m.buf[B_OUT].resize(p);
    for (uint32_t r = 0; r < p; r++) {
        m.buf[B_IN][r] = cclIn[r].data();
        m.buf[B_OUT][r] = cclOut[r].data();
    }
    uint64_t offset = 0;
    for (uint64_t left = sendCount; left > 0;) {
        uint64_t cur = left > maxPer ? maxPer : left;
        uint64_t bytes = cur * unit;
        std::vector<Slice> outSl(p), inSl(p);
        for (uint32_t i = 0; i < p; i++) {
            outSl[i] = Slice{bytes * i, bytes};
            inSl[i] = Slice{(p > 1) ? 0 : bytes * i, bytes};   // input smaller than output -> offset 0
        }
        for (uint32_t r = 0; r < p; r++) {
            m.Copy(m.buf[B_IN][r], static_cast<uint8_t *>(in[r]) + offset, bytes);
        }
        for (uint32_t r = 0; r < p; r++) {
            Proc pr;
            pr.rank = r;
            if (algo == ALGO_RING || p == 1) {
                ProgAllGatherRing(pr.prog, r, p, B_IN, B_OUT, outSl, inSl);
            } else if (algo == ALGO_MESH) {
                pr.prog.push_back(MkLocalCopy(B_OUT, outSl[r].off, B_IN, inSl[r].off, bytes));
                ProgAllGatherMesh(pr.prog, r, p, B_OUT, outSl);
            } else if (algo == ALGO_RHD) {
                // AllGatherRecursiveHalvingDoubling::RunAsync, all_gather_recursive_hd.cc:26-238
                uint32_t block, part1;
                std::vector<uint32_t> rankOf;
                std::vector<Slice> bsl;
                RhdBlockLayout(p, bytes, &block, &part1, &rankOf, &bsl);
                pr.prog.push_back(MkLocalCopy(B_OUT, outSl[r].off, B_IN, inSl[r].off, bytes));
                if (r < part1 && (r % 2) == 1) {
                    pr.prog.push_back(MkSend(static_cast<int>(r - 1), 1, B_OUT, bytes * r, bytes));
                    pr.prog.push_back(MkRecvCopy(static_cast<int>(r - 1), 1, B_OUT, 0, bytes * p));
                } else {
                    if (r < part1) {
                        pr.prog.push_back(MkRecvCopy(static_cast<int>(r + 1), 1, B_OUT, bytes * (r + 1), bytes));
                    }
                    uint32_t q = (r < part1) ? r / 2 : r - part1 / 2;
                    ProgAllGatherHd(pr.prog, q, block, rankOf, B_OUT, bsl);
                    if (r < part1) {
                        pr.prog.push_back(MkSend(static_cast<int>(r + 1), 1, B_OUT, 0, bytes * p));
                    }
                }
            } else {
                return -10;
            }
            m.procs.push_back(std::move(pr));
        }
        int rc = m.Run();
        if (rc != 0) {
            return rc;
        }
        for (uint32_t r = 0; r < p; r++) {
            for (uint32_t i = 0; i < p; i++) {
                m.Copy(static_cast<uint8_t *>(out[r]) + sendCount * unit * i + offset, m.buf[B_OUT][r] + bytes * i, bytes);
            }
        }
        offset += bytes;
        left -= cur;
    }
    return 0;
}

// Two-level all-gather over `servers` groups of D = p / servers consecutive ranks
// (CollAllGatherMeshExecutor::KernelRun, ALG/impl/coll_executor/coll_all_gather/coll_all_gather_mesh_executor.cc:71-175;
// CollAllGatherRingExecutor::KernelRun, coll_all_gather_ring_executor.cc:81-200): every rank puts its block at its
// place in the output staging buffer, the group gathers its D blocks (level0: 0 mesh, 2 one ring, 3 the four rings of
// the 8-device topology on the parts MultiSegSlices cuts), then the ranks at position d of all groups gather the
// groups' runs of D blocks, ring or recursive halving-doubling.  Chunks of cclBytes / p (rounded down to the
// alignment with the mesh, :64-69; not with the rings, coll_all_gather_ring_executor.cc:75-79) per rank.
int orc_allgather_two_level(int level1, int level0, uint32_t servers, uint32_t p, void **in, void **out, uint64_t sendCount, int dt,
    uint64_t cclBytes, uint64_t align, int flags, int threads)
{
    uint64_t unit = DtSize(dt);
    if (unit == 0 || p == 0 || servers == 0 || p % servers != 0 || (level1 != ALGO_RING && level1 != ALGO_RHD) ||
        (level0 != 0 && level0 != 2 && level0 != 3) || (level0 == 3 && p / servers != 8)) {
        return -20;
    }
    const uint32_t D = p / servers;
    const uint32_t ringCount = level0 == 3 ? 4u : 1u;
    uint64_t maxPer = MaxCountPerLoop(2, cclBytes, p, unit, level0 == 0 ? align : 1);
    if (maxPer == 0) {
        return -21;
    }
    Pool pool(threads);
    auto machine = [&](uint32_t n) {
        Machine m;
        m.p = static_cast<int>(n);
        m.dt = dt;
        m.op = 0;
        m.direct = (flags & 1) != 0;
        m.pool = &pool;
        m.buf[B_IN].resize(n);
        m.buf[B_OUT].resize(n);
        return m;
    };
    Machine all = machine(p);
    uint64_t stage = std::min<uint64_t>(sendCount, maxPer) * unit;
    std::vector<std::vector<uint8_t>> cclIn(p, std::vector<uint8_t>(stage)), cclOut(p, std::vector<uint8_t>(stage * p));
    for (uint32_t r = 0; r < p; r++) {
        all.buf[B_IN][r] = cclIn[r].data();
        all.buf[B_OUT][r] = cclOut[r].data();
    }
    uint64_t offset = 0;
    for (uint64_t left = sendCount; left > 0;) {
        uint64_t cur = left > maxPer ? maxPer : left;
        uint64_t bytes = cur * unit;
        for (uint32_t r = 0; r < p; r++) {
            all.Copy(all.buf[B_IN][r], static_cast<uint8_t *>(in[r]) + offset, bytes);
            all.Copy(all.buf[B_OUT][r] + bytes * r, all.buf[B_IN][r], bytes);    // own block to its place
        }
        // inside every group, on the group's run of D blocks
        std::vector<Slice> segs(D);
        for (uint32_t d = 0; d < D; d++) {
            segs[d] = Slice{bytes * d, bytes};
        }
        for (uint32_t s = 0; s < servers && D > 1; s++) {
            const uint64_t base = bytes * D * s;
            if (level0 == 0) {
                Machine m = machine(D);
                for (uint32_t d = 0; d < D; d++) {
                    m.buf[B_IN][d] = all.buf[B_IN][s * D + d];
                    m.buf[B_OUT][d] = all.buf[B_OUT][s * D + d] + base;
                    Proc pr;
                    pr.rank = d;
                    ProgAllGatherMesh(pr.prog, d, D, B_OUT, segs);
                    m.procs.push_back(std::move(pr));
                }
                int rc = m.Run();
                if (rc != 0) {
                    return rc;
                }
                continue;
            }
            std::vector<std::vector<Slice>> parts = MultiSegSlices(segs, ringCount, align);
            for (uint32_t k = 0; k < ringCount; k++) {
                Machine ring = machine(D);
                std::vector<Slice> ringSl(D);
                for (uint32_t i = 0; i < D; i++) {
                    uint32_t dev = ringCount > 1 ? kEightDeviceRings[k][i] : i;
                    ring.buf[B_IN][i] = all.buf[B_IN][s * D + dev];
                    ring.buf[B_OUT][i] = all.buf[B_OUT][s * D + dev] + base;
                    ringSl[i] = ringCount > 1 ? parts[dev][k] : segs[dev];
                }
                for (uint32_t i = 0; i < D; i++) {
                    Proc pr;
                    pr.rank = i;
                    ProgAllGatherRing(pr.prog, i, D, B_OUT, B_OUT, ringSl, ringSl);
                    ring.procs.push_back(std::move(pr));
                }
                int rc = ring.Run();
                if (rc != 0) {
                    return rc;
                }
            }
        }
        // between the groups: the ranks at position d, on runs of D blocks
        const uint64_t run = bytes * D;
        for (uint32_t d = 0; d < D && servers > 1; d++) {
            Machine m = machine(servers);
            std::vector<Slice> runs(servers);
            for (uint32_t s = 0; s < servers; s++) {
                m.buf[B_IN][s] = all.buf[B_IN][s * D + d];
                m.buf[B_OUT][s] = all.buf[B_OUT][s * D + d];
                runs[s] = Slice{run * s, run};
            }
            for (uint32_t s = 0; s < servers; s++) {
                Proc pr;
                pr.rank = s;
                if (level1 == ALGO_RING) {
                    ProgAllGatherRing(pr.prog, s, servers, B_OUT, B_OUT, runs, runs);
                } else {
                    // AllGatherRecursiveHalvingDoubling::RunAsync, all_gather_recursive_hd.cc:26-238, data already in place
                    uint32_t block, part1;
                    std::vector<uint32_t> rankOf;
                    std::vector<Slice> bsl;
                    RhdBlockLayout(servers, run, &block, &part1, &rankOf, &bsl);
                    if (s < part1 && (s % 2) == 1) {
                        pr.prog.push_back(MkSend(static_cast<int>(s - 1), 1, B_OUT, run * s, run));
                        pr.prog.push_back(MkRecvCopy(static_cast<int>(s - 1), 1, B_OUT, 0, run * servers));
                    } else {
                        if (s < part1) {
                            pr.prog.push_back(MkRecvCopy(static_cast<int>(s + 1), 1, B_OUT, run * (s + 1), run));
                        }
                        uint32_t q = (s < part1) ? s / 2 : s - part1 / 2;
                        ProgAllGatherHd(pr.prog, q, block, rankOf, B_OUT, bsl);
                        if (s < part1) {
                            pr.prog.push_back(MkSend(static_cast<int>(s + 1), 1, B_OUT, 0, run * servers));
                        }
                    }
                }
                m.procs.push_back(std::move(pr));
            }
            int rc = m.Run();
            if (rc != 0) {
                return rc;
            }
        }
        for (uint32_t r = 0; r < p; r++) {
            for (uint32_t i = 0; i < p; i++) {
                all.Copy(static_cast<uint8_t *>(out[r]) + sendCount * unit * i + offset, all.buf[B_OUT][r] + bytes * i, bytes);
            }
        }
        offset += bytes;
        left -= cur;
    }
    return 0;
}

// Variable-count reduce-scatter: every rank's `in` holds the blocks {displs[i], counts[i]} (elements);
// rank r receives the reduction of block r.  The templates run over these explicit slices
// (reduce_scatter_ring.cc:179-297 takes any slice list; mesh and halving-doubling likewise).
int orc_reducescatter_v(int algo, uint32_t p, void **in, void **out, const uint64_t *counts, const uint64_t *displs,
    int dt, int op, uint64_t align, int flags, int threads)
{
    uint64_t unit = DtSize(dt);
    if (unit == 0 || p == 0) {
        return -20;
    }
    std::vector<Slice> sl(p);
    uint64_t extent = 0;
    for (uint32_t i = 0; i < p; i++) {
        sl[i] = Slice{displs[i] * unit, counts[i] * unit};
        if (sl[i].size) {
            extent = std::max(extent, sl[i].off + sl[i].size);
        }
    }
    Pool pool(threads);
    Machine m;
    m.p = static_cast<int>(p);
    m.dt = dt;
    m.op = op;
    m.direct = (flags & 1) != 0;
    m.pool = &pool;
    std::vector<std::vector<uint8_t>> work(p, std::vector<uint8_t>(extent));
    m.buf[B_IN].resize(p);
    m.buf[B_OUT].resize(p);
    for (uint32_t r = 0; r < p; r++) {
        m.buf[B_IN][r] = work[r].data();
        m.buf[B_OUT][r] = static_cast<uint8_t *>(out[r]);
        m.Copy(work[r].data(), static_cast<uint8_t *>(in[r]), extent);
    }
    if (p > 1) {
        if (algo == ALGO_RING) {
            for (uint32_t r = 0; r < p; r++) {
                Proc pr;
                pr.rank = r;
                ProgReduceScatterRing(pr.prog, r, p, B_IN, B_IN, sl, sl);
                m.procs.push_back(std::move(pr));
            }
        } else if (algo == ALGO_MESH_ATOMIC) {
            for (uint32_t r = 0; r < p; r++) {
                Proc pr;
                pr.rank = r;
                ProgReduceScatterMeshAtomic(pr.prog, r, p, B_IN, sl);
                m.procs.push_back(std::move(pr));
            }
        } else if (algo == ALGO_MESH) {
            uint32_t nstream = p > 2 ? p - 1 : 1;
            std::vector<std::vector<Slice>> pieces = CutPieces(sl, nstream, align);
            for (uint32_t t = 0; t < nstream; t++) {
                for (uint32_t r = 0; r < p; r++) {
                    Proc pr;
                    pr.rank = r;
                    ProgReduceScatterMeshStream(pr.prog, r, p, t, B_IN, pieces[t]);
                    m.procs.push_back(std::move(pr));
                }
            }
        } else if (algo == ALGO_RHD) {
            // No counterpart in the reference, which runs the variable-count reduce-scatter on the mesh only: the order of
            // ReduceScatterRecursiveHalvingDoubling (reduce_scatter_recursive_hd.cc:33-254) over the caller's table.  The
            // blocks of a table need not lie one behind the other, so a step's range travels block by block.
            uint32_t block, part1;
            RhdParams(p, &block, &part1);
            const uint32_t half = part1 / 2;
            std::vector<uint32_t> rankOf(block);
            std::vector<std::vector<uint32_t>> owned(block);
            for (uint32_t b = 0; b < block; b++) {
                rankOf[b] = b < half ? 2 * b : b + half;
                owned[b] = b < half ? std::vector<uint32_t>{2 * b, 2 * b + 1} : std::vector<uint32_t>{b + half};
            }
            uint32_t steps = 0;
            while ((1u << steps) < block) {
                steps++;
            }
            for (uint32_t r = 0; r < p; r++) {
                Proc pr;
                pr.rank = r;
                if (r < part1 && (r % 2) == 1) {
                    pr.prog.push_back(MkSend(static_cast<int>(r - 1), 1, B_IN, 0, extent));
                    pr.prog.push_back(MkRecvCopy(static_cast<int>(r - 1), 1, B_IN, sl[r].off, sl[r].size));
                    m.procs.push_back(std::move(pr));
                    continue;
                }
                if (r < part1) {
                    pr.prog.push_back(MkRecvReduce(static_cast<int>(r + 1), 1, B_IN, 0, B_IN, 0, extent));
                }
                const uint32_t q = r < part1 ? r / 2 : r - half;
                for (uint32_t step = 0; step < steps; step++) {
                    const uint32_t mask = 1u << (steps - step - 1);
                    const uint32_t peer = q ^ mask;
                    const uint32_t txId = peer & ~(mask - 1), rxId = q & ~(mask - 1);
                    for (uint32_t b = txId; b < txId + mask; b++) {
                        for (uint32_t u : owned[b]) {
                            pr.prog.push_back(MkSend(static_cast<int>(rankOf[peer]), 0, B_IN, sl[u].off, sl[u].size));
                        }
                    }
                    for (uint32_t b = rxId; b < rxId + mask; b++) {
                        for (uint32_t u : owned[b]) {
                            pr.prog.push_back(MkRecvReduce(static_cast<int>(rankOf[peer]), 0, B_IN, sl[u].off, B_IN, sl[u].off,
                                sl[u].size));
                        }
                    }
                }
                if (r < part1) {
                    pr.prog.push_back(MkSend(static_cast<int>(r + 1), 1, B_IN, sl[r + 1].off, sl[r + 1].size));
                }
                m.procs.push_back(std::move(pr));
            }
        } else {
            return -10;
        }
        int rc = m.Run();
        if (rc != 0) {
            return rc;
        }
    }
    for (uint32_t r = 0; r < p; r++) {
        m.Copy(static_cast<uint8_t *>(out[r]), work[r].data() + sl[r].off, sl[r].size);
    }
    return 0;
}

// Variable-count all-gather: rank r contributes counts[r] elements, every rank's `out` receives block i
// at displs[i].
int orc_allgather_v(int algo, uint32_t p, void **in, void **out, const uint64_t *counts, const uint64_t *displs, int dt,
    int flags, int threads)
{
    uint64_t unit = DtSize(dt);
    if (unit == 0 || p == 0) {
        return -20;
    }
    std::vector<Slice> sl(p), inSl(p);
    for (uint32_t i = 0; i < p; i++) {
        sl[i] = Slice{displs[i] * unit, counts[i] * unit};
        inSl[i] = Slice{0, counts[i] * unit};
    }
    Pool pool(threads);
    Machine m;
    m.p = static_cast<int>(p);
    m.dt = dt;
    m.direct = (flags & 1) != 0;
    m.pool = &pool;
    m.buf[B_IN].resize(p);
    m.buf[B_OUT].resize(p);
    for (uint32_t r = 0; r < p; r++) {
        m.buf[B_IN][r] = static_cast<uint8_t *>(in[r]);
        m.buf[B_OUT][r] = static_cast<uint8_t *>(out[r]);
    }
    for (uint32_t r = 0; r < p; r++) {
        Proc pr;
        pr.rank = r;
        if (algo == ALGO_RING || p == 1) {
            if (p == 1) {
                pr.prog.push_back(MkLocalCopy(B_OUT, sl[0].off, B_IN, 0, sl[0].size));
            } else {
                ProgAllGatherRing(pr.prog, r, p, B_IN, B_OUT, sl, inSl);
            }
        } else if (algo == ALGO_MESH) {
            pr.prog.push_back(MkLocalCopy(B_OUT, sl[r].off, B_IN, 0, sl[r].size));
            ProgAllGatherMesh(pr.prog, r, p, B_OUT, sl);
        } else {
            return -10;
        }
        m.procs.push_back(std::move(pr));
    }
    return m.Run();
}

// Ring broadcast (broadcast_ring.cc:24-160) with the executor's chunk loop: buf[root] is the source,
// every other buf receives it.  Slices of one chunk travel root -> root+1 -> ... -> root-1.
int orc_broadcast(uint32_t p, void **buf, uint64_t count, int dt, uint32_t root, uint64_t cclBytes, uint64_t align,
    int flags, int threads)
{
    uint64_t unit = DtSize(dt);
    if (unit == 0 || p == 0 || root >= p) {
        return -20;
    }
    uint64_t maxPer = cclBytes / unit;
    if (maxPer == 0) {
        return -21;
    }
    Pool pool(threads);
    Machine m;
    m.p = static_cast<int>(p);
    m.dt = dt;
    m.direct = (flags & 1) != 0;
    m.pool = &pool;
    m.buf[B_IN].resize(p);
    m.buf[B_OUT].resize(p);
    uint64_t offset = 0;
    for (uint64_t left = count; left > 0 && p > 1;) {
        uint64_t cur = left > maxPer ? maxPer : left;
        uint64_t bytes = cur * unit;
        for (uint32_t r = 0; r < p; r++) {
            m.buf[B_IN][r] = static_cast<uint8_t *>(buf[r]) + offset;
            m.buf[B_OUT][r] = static_cast<uint8_t *>(buf[r]) + offset;
        }
        uint64_t sizeAvg = ((cur + p - 1) / p) * unit;
        uint64_t per = RoundUp(sizeAvg, align);
        for (uint32_t r = 0; r < p; r++) {
            Proc pr;
            pr.rank = r;
            uint32_t left_ = (r + p - 1) % p, right = (r + 1) % p;
            uint64_t residue = bytes;
            for (uint32_t round = 0; round < p; round++) {
                uint64_t n = residue > per ? per : residue;
                uint64_t at = bytes - residue;
                if (r == root) {
                    pr.prog.push_back(MkSend(static_cast<int>(right), 0, B_IN, at, n));
                } else {
                    pr.prog.push_back(MkRecvCopy(static_cast<int>(left_), 0, B_OUT, at, n));
                    if (right != root) {
                        pr.prog.push_back(MkSend(static_cast<int>(right), 0, B_OUT, at, n));
                    }
                }
                residue -= n;
            }
            m.procs.push_back(std::move(pr));
        }
        int rc = m.Run();
        if (rc != 0) {
            return rc;
        }
        offset += bytes;
        left -= cur;
    }
    return 0;
}

// Star broadcast (TPL/temp_broadcast/broadcast_star.cc:47-99, run by ALG/impl/legacy/operator/
// broadcast_operator_for_hetero.cc:91-113 over the whole buffer, no chunk loop): the root sends every other rank all
// of it (RunSendBroadcast :137-165), every other rank receives it from the root (RunRecvBroadcast :101-135).
// `touched` (optional) receives the bytes read + written by all ranks.
int orc_broadcast_star(uint32_t p, void **buf, uint64_t count, int dt, uint32_t root, int flags, int threads, uint64_t *touched)
{
    const uint64_t unit = DtSize(dt);
    if (unit == 0 || p == 0 || root >= p) {
        return -20;
    }
    const uint64_t bytes = count * unit;
    Pool pool(threads);
    Machine m;
    m.p = static_cast<int>(p);
    m.dt = dt;
    m.direct = (flags & 1) != 0;
    m.pool = &pool;
    m.buf[B_IN].resize(p);
    m.buf[B_OUT].resize(p);
    for (uint32_t r = 0; r < p; r++) {
        m.buf[B_IN][r] = m.buf[B_OUT][r] = static_cast<uint8_t *>(buf[r]);
    }
    for (uint32_t r = 0; r < p && p > 1; r++) {
        Proc pr;
        pr.rank = r;
        if (r == root) {
            for (uint32_t d = 0; d < p; d++) {
                if (d != root && bytes > 0) {
                    pr.prog.push_back(MkSend(static_cast<int>(d), 0, B_IN, 0, bytes));
                }
            }
        } else if (bytes > 0) {
            pr.prog.push_back(MkRecvCopy(static_cast<int>(root), 0, B_OUT, 0, bytes));
        }
        m.procs.push_back(std::move(pr));
    }
    int rc = p > 1 ? m.Run() : 0;
    if (touched != nullptr) {
        *touched = m.bytesTouched;
    }
    return rc;
}

// Mesh broadcast, CollBroadcastMeshExecutor::KernelRun (EXE/coll_broadcast/coll_broadcast_mesh_executor.cc:59-213)
// on one server: the root scatters slice i to rank i (TPL/temp_scatter/scatter_mesh.cc:46-160), then a mesh
// all-gather; slices from GetRankSliceSize (EXE/coll_broadcast/coll_broadcast_executor.cc:275-306).
int orc_broadcast_mesh(uint32_t p, void **buf, uint64_t count, int dt, uint32_t root, uint64_t cclBytes, uint64_t align,
    int flags, int threads)
{
    uint64_t unit = DtSize(dt);
    if (unit == 0 || p == 0 || root >= p) {
        return -20;
    }
    uint64_t maxPer = cclBytes / unit;
    if (maxPer == 0) {
        return -21;
    }
    Pool pool(threads);
    Machine m;
    m.p = static_cast<int>(p);
    m.dt = dt;
    m.direct = (flags & 1) != 0;
    m.pool = &pool;
    m.buf[B_IN].resize(p);
    m.buf[B_OUT].resize(p);
    uint64_t offset = 0;
    for (uint64_t left = count; left > 0 && p > 1;) {
        uint64_t cur = left > maxPer ? maxPer : left;
        uint64_t bytes = cur * unit;
        for (uint32_t r = 0; r < p; r++) {
            m.buf[B_IN][r] = static_cast<uint8_t *>(buf[r]) + offset;
            m.buf[B_OUT][r] = static_cast<uint8_t *>(buf[r]) + offset;
        }
        uint64_t avg = bytes / p + ((cur % p) > 0 ? 1 : 0);
        uint64_t per = RoundUp(avg, align);
        std::vector<Slice> sl(p);
        uint64_t residue = bytes;
        for (uint32_t i = 0; i < p; i++) {
            sl[i].size = per < residue ? per : residue;
            sl[i].off = sl[i].size == 0 ? 0 : i * per;
            residue -= sl[i].size;
        }
        for (uint32_t r = 0; r < p; r++) {          // stage 0: scatter from the root
            Proc pr;
            pr.rank = r;
            if (r == root) {
                for (uint32_t d = 0; d < p; d++) {
                    if (d != root) {
                        pr.prog.push_back(MkSend(static_cast<int>(d), 0, B_IN, sl[d].off, sl[d].size));
                    }
                }
            } else {
                pr.prog.push_back(MkRecvCopy(static_cast<int>(root), 0, B_OUT, sl[r].off, sl[r].size));
            }
            m.procs.push_back(std::move(pr));
        }
        int rc = m.Run();
        if (rc != 0) {
            return rc;
        }
        for (uint32_t r = 0; r < p; r++) {          // stage 2: all-gather of the slices
            Proc pr;
            pr.rank = r;
            ProgAllGatherMesh(pr.prog, r, p, B_OUT, sl);
            m.procs.push_back(std::move(pr));
        }
        rc = m.Run();
        if (rc != 0) {
            return rc;
        }
        offset += bytes;
        left -= cur;
    }
    return 0;
}

// Per-rank programs of BcastRecursiveHalvingDoubling::RunAsync
// (TPL/temp_broadcast/bcast_recursive_halvingdoubling.cc:21-290) on the machine's buffers: the `bytes` bytes at
// offset `off` of the root's buffer reach every rank.  BroadcastInBlock (:162-203) and the hand-over inside the rank
// pairs of part one (:205-262); block membership from GetRankIndexInBlock (:138-160).
void AddBroadcastRhdProcs(Machine &m, uint32_t root, uint64_t off, uint64_t bytes)
{
    const uint32_t p = static_cast<uint32_t>(m.p);
    uint32_t block, part1;
    RhdParams(p, &block, &part1);
    const bool rootEven = (root < part1 && (root % 2) == 0) || root >= part1;
    auto inBlock = [&](uint32_t r) -> int {   // GetRankIndexInBlock
        if (r >= part1) {
            return static_cast<int>(r - part1 / 2);
        }
        if (rootEven) {
            return (r % 2) == 0 ? static_cast<int>(r / 2) : -1;
        }
        return (r % 2) == 1 ? static_cast<int>((r - 1) / 2) : -1;
    };
    auto real = [&](uint32_t q) -> uint32_t {   // GetRankIndexReal
        if (q < part1 / 2) {
            return rootEven ? q * 2 : q * 2 + 1;
        }
        return part1 / 2 + q;
    };
    uint32_t rounds = 0;
    while ((1u << rounds) < block) {
        rounds++;
    }
    for (uint32_t r = 0; r < p; r++) {
        Proc pr;
        pr.rank = r;
        int q = inBlock(r);
        if (q >= 0) {
            const uint32_t rq = static_cast<uint32_t>(q), rootQ = static_cast<uint32_t>(inBlock(root));
            bool hasData = r == root;
            for (uint32_t i = 0; i < rounds; i++) {
                const uint32_t mask = 1u << (rounds - i - 1);
                const uint32_t peer = real(rq ^ mask);
                if ((rq & (mask - 1)) == (rootQ & (mask - 1)) && r != root && !hasData) {
                    pr.prog.push_back(MkRecvCopy(static_cast<int>(peer), 0, B_IN, off, bytes));
                    hasData = true;
                    continue;
                }
                if (hasData) {
                    pr.prog.push_back(MkSend(static_cast<int>(peer), 0, B_IN, off, bytes));
                }
            }
        }
        if (r < part1) {
            const uint32_t pairPeer = (r % 2) == 0 ? r + 1 : r - 1;
            const bool sends = ((r % 2) == 0) == rootEven;   // EvenNumberRankProcess / OddNumberRankProcess
            if (sends) {
                pr.prog.push_back(MkSend(static_cast<int>(pairPeer), 1, B_IN, off, bytes));
            } else {
                pr.prog.push_back(MkRecvCopy(static_cast<int>(pairPeer), 1, B_IN, off, bytes));
            }
        }
        m.procs.push_back(std::move(pr));
    }
}

// Recursive halving-doubling broadcast with the executor's chunk loop.
int orc_broadcast_rhd(uint32_t p, void **buf, uint64_t count, int dt, uint32_t root, uint64_t cclBytes, uint64_t align,
    int flags, int threads)
{
    (void)align;
    uint64_t unit = DtSize(dt);
    if (unit == 0 || p == 0 || root >= p) {
        return -20;
    }
    uint64_t maxPer = cclBytes / unit;
    if (maxPer == 0) {
        return -21;
    }
    Pool pool(threads);
    Machine m;
    m.p = static_cast<int>(p);
    m.dt = dt;
    m.direct = (flags & 1) != 0;
    m.pool = &pool;
    m.buf[B_IN].resize(p);
    m.buf[B_OUT].resize(p);
    uint64_t offset = 0;
    for (uint64_t left = count; left > 0 && p > 1;) {
        uint64_t cur = left > maxPer ? maxPer : left;
        uint64_t bytes = cur * unit;
        for (uint32_t r = 0; r < p; r++) {
            m.buf[B_IN][r] = static_cast<uint8_t *>(buf[r]) + offset;
            m.buf[B_OUT][r] = static_cast<uint8_t *>(buf[r]) + offset;
        }
        AddBroadcastRhdProcs(m, root, 0, bytes);
        int rc = m.Run();
        if (rc != 0) {
            return rc;
        }
        offset += bytes;
        left -= cur;
    }
    return 0;
}

// Binary-block halving-doubling broadcast (TPL/temp_broadcast/bcast_halvingdoubling.cc:26-398).  The ranks are cut into
// blocks whose sizes are the powers of two in the rank count, the smallest block at the highest ranks
// (PrepareBlockParams :26-62, PrepareRootBlockParam :64-90).  Inside the root's block the buffer spreads as a binomial
// tree, widest distance first (BcastInRootBlock :165-228); then it goes from block to block: towards the smaller block
// every `times`-th rank sends to one rank, towards the larger block every rank sends to `rounds` consecutive ranks, one
// after the other (GatherBetweenBlocksRootBlock :231-281, ...HigherBlock :284-335, ...LowerBlock :338-396).  Every
// transfer carries the whole buffer.
namespace {

struct HdBlocks {
    uint32_t myOffset = 0, mySize = 0, lower = 0, higher = 0, rankIn = 0, steps = 0;
};

HdBlocks HdBlockOf(uint32_t rank, uint32_t n)
{
    HdBlocks b;
    uint32_t offset = n, blockSize = 1, current = 0, pre = 0;
    while (offset > 0) {
        if ((n & blockSize) != 0) {
            pre = current;
            current = blockSize;
            offset -= blockSize;
            if (b.mySize != 0) {
                b.higher = current;
                break;
            }
            if (offset <= rank) {
                b.myOffset = offset;
                b.mySize = current;
                b.lower = pre;
            }
        }
        blockSize <<= 1;
    }
    while ((1u << b.steps) < b.mySize) {
        b.steps++;
    }
    b.rankIn = b.mySize != 0 ? rank % b.mySize : 0;
    return b;
}

// the program of one rank: (peer, isSend) in order
std::vector<std::pair<uint32_t, bool>> HdBlocksProgram(uint32_t rank, uint32_t n, uint32_t root)
{
    std::vector<std::pair<uint32_t, bool>> ops;
    const HdBlocks me = HdBlockOf(rank, n), rb = HdBlockOf(root, n);
    auto toLower = [&] {            // :246-258, :372-393
        if (me.lower != 0) {
            const uint32_t times = me.mySize / me.lower;
            if (me.rankIn % times == 0) {
                ops.emplace_back(me.myOffset + me.mySize + me.rankIn / times, true);
            }
        }
    };
    auto toHigher = [&] {           // :261-279, :310-332
        if (me.higher != 0) {
            const uint32_t rounds = me.higher / me.mySize;
            uint32_t dst = (me.myOffset - me.higher) + me.rankIn * rounds;
            for (uint32_t i = 0; i < rounds; i++) {
                ops.emplace_back(dst + i, true);
            }
        }
    };
    if (rank >= rb.myOffset + rb.mySize) {          // my block lies below the root's: from the larger block, on to the smaller
        if (me.higher != 0) {
            ops.emplace_back((me.myOffset - me.higher) + me.rankIn * (me.higher / me.mySize), false);
        }
        toLower();
    } else if (rank < rb.myOffset) {                 // above: from the smaller block, on to the larger
        if (me.lower != 0) {
            ops.emplace_back(me.myOffset + me.mySize + me.rankIn / (me.mySize / me.lower), false);
        }
        toHigher();
    } else {
        if (me.mySize > 1) {
            const uint32_t rootOff = root - rb.myOffset;
            uint32_t mask = 1u << (me.steps - 1);
            bool have = false;
            for (uint32_t round = 1; round <= me.steps; round++, mask >>= 1) {
                const uint32_t peer = rank ^ mask, low = (1u << (me.steps - round)) - 1;
                if ((me.rankIn & low) == (rootOff & low) && rank != root && !have) {
                    ops.emplace_back(peer, false);
                    have = true;
                    continue;
                }
                if (have || rank == root) {
                    ops.emplace_back(peer, true);
                }
            }
        }
        toLower();
        toHigher();
    }
    return ops;
}

}  // namespace

// The transfers of the binary-block broadcast as (sender, receiver) pairs, rank by rank in program order (sends only):
// what tests hold the route against.  Returns the number of pairs (at most cap are written).
int orc_broadcast_hd_blocks_route(uint32_t p, uint32_t root, uint32_t *pairs, uint32_t cap)
{
    uint32_t n = 0;
    for (uint32_t r = 0; r < p; r++) {
        for (const auto &op : HdBlocksProgram(r, p, root)) {
            if (op.second) {
                if (n < cap) {
                    pairs[2 * n] = r;
                    pairs[2 * n + 1] = op.first;
                }
                n++;
            }
        }
    }
    return static_cast<int>(n);
}

// With a chunk loop over the CCL buffer like the other one-level broadcasts (coll_broadcast_executor.cc:83-121).
// `touched` (optional) receives the bytes read + written by all ranks.
int orc_broadcast_hd_blocks(uint32_t p, void **buf, uint64_t count, int dt, uint32_t root, uint64_t cclBytes, int flags,
    int threads, uint64_t *touched)
{
    uint64_t unit = DtSize(dt);
    if (unit == 0 || p == 0 || root >= p) {
        return -20;
    }
    uint64_t maxPer = cclBytes / unit;
    if (maxPer == 0) {
        return -21;
    }
    Pool pool(threads);
    Machine m;
    m.p = static_cast<int>(p);
    m.dt = dt;
    m.direct = (flags & 1) != 0;
    m.pool = &pool;
    m.buf[B_IN].resize(p);
    m.buf[B_OUT].resize(p);
    uint64_t offset = 0;
    for (uint64_t left = count; left > 0 && p > 1;) {
        uint64_t cur = left > maxPer ? maxPer : left;
        uint64_t bytes = cur * unit;
        for (uint32_t r = 0; r < p; r++) {
            m.buf[B_IN][r] = static_cast<uint8_t *>(buf[r]) + offset;
            m.buf[B_OUT][r] = static_cast<uint8_t *>(buf[r]) + offset;
        }
        for (uint32_t r = 0; r < p; r++) {
            Proc pr;
            pr.rank = r;
            for (const auto &op : HdBlocksProgram(r, p, root)) {
                if (op.second) {
                    pr.prog.push_back(MkSend(static_cast<int>(op.first), 0, B_IN, 0, bytes));
                } else {
                    pr.prog.push_back(MkRecvCopy(static_cast<int>(op.first), 0, B_IN, 0, bytes));
                }
            }
            m.procs.push_back(std::move(pr));
        }
        int rc = m.Run();
        if (rc != 0) {
            return rc;
        }
        offset += bytes;
        left -= cur;
    }
    if (touched != nullptr) {
        *touched = m.bytesTouched;
    }
    return 0;
}

// Two-level broadcast, CollBroadcastMeshExecutor::KernelRun with several servers
// (EXE/coll_broadcast/coll_broadcast_mesh_executor.cc:59-213) under the chunk loop of
// CollBroadcastExecutor::RunLoop (coll_broadcast_executor.cc:83-121); `servers` groups of D = p / servers consecutive
// ranks.  Per chunk: slices over the D ranks of a group (GetRankSliceSize, coll_broadcast_executor.cc:275-306);
// stage 0 (:131-147) only in the root's group: the root scatters slice d to the rank at position d
// (TPL/temp_scatter/scatter_mesh.cc:46-160); stage 1 (:148-186): the ranks at position d of all groups broadcast
// slice d from the root's group by recursive halving-doubling (the default level-1 choice of :113-117; count =
// the slice's size, base offset = the slice's offset); stage 2 (:189-207): mesh all-gather of the slices inside
// every group (TPL/temp_all_gather/all_gather_mesh.cc:91-145).
// `touched` (optional) receives the bytes read + written by all ranks (2 x the bytes received).
int orc_broadcast_two_level(uint32_t servers, uint32_t p, void **buf, uint64_t count, int dt, uint32_t root,
    uint64_t cclBytes, uint64_t align, int flags, int threads, uint64_t *touched)
{
    uint64_t moved = 0;
    uint64_t unit = DtSize(dt);
    if (unit == 0 || p == 0 || root >= p || servers == 0 || p % servers != 0) {
        return -20;
    }
    uint64_t maxPer = cclBytes / unit;
    if (maxPer == 0) {
        return -21;
    }
    const uint32_t D = p / servers, rootGroup = root / D, rootLocal = root % D;
    Pool pool(threads);
    auto machine = [&](uint32_t n) {
        Machine m;
        m.p = static_cast<int>(n);
        m.dt = dt;
        m.direct = (flags & 1) != 0;
        m.pool = &pool;
        m.buf[B_IN].resize(n);
        m.buf[B_OUT].resize(n);
        return m;
    };
    uint64_t offset = 0;
    for (uint64_t left = count; left > 0 && p > 1;) {
        uint64_t cur = left > maxPer ? maxPer : left;
        uint64_t bytes = cur * unit;
        uint64_t avg = bytes / D + ((cur % D) > 0 ? 1 : 0);
        uint64_t per = RoundUp(avg, align);
        std::vector<Slice> sl(D);
        uint64_t residue = bytes;
        for (uint32_t i = 0; i < D; i++) {
            sl[i].size = per < residue ? per : residue;
            sl[i].off = sl[i].size == 0 ? 0 : i * per;
            residue -= sl[i].size;
        }
        auto at = [&](uint32_t g, uint32_t d) { return static_cast<uint8_t *>(buf[g * D + d]) + offset; };
        if (D > 1) {                                   // stage 0: scatter inside the root's group
            Machine m = machine(D);
            for (uint32_t d = 0; d < D; d++) {
                m.buf[B_IN][d] = m.buf[B_OUT][d] = at(rootGroup, d);
            }
            for (uint32_t d = 0; d < D; d++) {
                Proc pr;
                pr.rank = d;
                if (d == rootLocal) {
                    for (uint32_t to = 0; to < D; to++) {
                        if (to != rootLocal) {
                            pr.prog.push_back(MkSend(static_cast<int>(to), 0, B_IN, sl[to].off, sl[to].size));
                        }
                    }
                } else {
                    pr.prog.push_back(MkRecvCopy(static_cast<int>(rootLocal), 0, B_OUT, sl[d].off, sl[d].size));
                }
                m.procs.push_back(std::move(pr));
            }
            int rc = m.Run();
            if (rc != 0) {
                return rc;
            }
            moved += m.bytesTouched;
        }
        if (servers > 1) {                             // stage 1: slice d between the groups
            for (uint32_t d = 0; d < D; d++) {
                if (sl[d].size == 0) {
                    continue;
                }
                Machine m = machine(servers);
                for (uint32_t g = 0; g < servers; g++) {
                    m.buf[B_IN][g] = m.buf[B_OUT][g] = at(g, d);
                }
                AddBroadcastRhdProcs(m, rootGroup, sl[d].off, sl[d].size);
                int rc = m.Run();
                if (rc != 0) {
                    return rc;
                }
                moved += m.bytesTouched;
            }
        }
        if (D > 1) {                                   // stage 2: all-gather inside every group
            for (uint32_t g = 0; g < servers; g++) {
                Machine m = machine(D);
                for (uint32_t d = 0; d < D; d++) {
                    m.buf[B_IN][d] = m.buf[B_OUT][d] = at(g, d);
                }
                for (uint32_t d = 0; d < D; d++) {
                    Proc pr;
                    pr.rank = d;
                    ProgAllGatherMesh(pr.prog, d, D, B_OUT, sl);
                    m.procs.push_back(std::move(pr));
                }
                int rc = m.Run();
                if (rc != 0) {
                    return rc;
                }
                moved += m.bytesTouched;
            }
        }
        offset += bytes;
        left -= cur;
    }
    if (touched != nullptr) {
        *touched = moved;
    }
    return 0;
}

// Two-level broadcast of the ring topologies, CollBroadcastRingExecutor::KernelRun
// (EXE/coll_broadcast/coll_broadcast_ring_executor.cc:64-211) under the chunk loop of CollBroadcastExecutor::RunLoop;
// `servers` groups of D = p / servers consecutive ranks, `rings` = 1 (one ring in rank order) or 4 (the four rings of
// the 8-device topology, D = 8).  Per chunk: slices over the D devices (PrepareSliceData, :80), every slice cut into one
// part per ring (PrepareMultiRingSlice with all ports, :86-93).
//   step 1 (:95-102, MultiRingScatter, EXE/coll_comm_executor.cc:1995-2130): only in the root's server, ring k runs the
//          ring scatter (TPL/temp_scatter/scatter_ring.cc:22-135) from the root's position over part k of its members'
//          slices, in place in the input buffer
//   step 2 (:105-187): the devices at position d of all servers broadcast slice d from the root's server by recursive
//          halving-doubling (segment and size from PrepareLevel1CommInfo, EXE/coll_comm_executor.cc:2176-2214)
//   step 3 (:189-207, MultiRingAllGather): ring all-gather of the parts inside every server, ring by ring
// `touched` (optional) receives the bytes read + written by all ranks.
int orc_broadcast_two_level_ring(uint32_t servers, uint32_t rings, uint32_t p, void **buf, uint64_t count, int dt, uint32_t root,
    uint64_t cclBytes, uint64_t align, int flags, int threads, uint64_t *touched)
{
    uint64_t moved = 0;
    uint64_t unit = DtSize(dt);
    if (unit == 0 || p == 0 || root >= p || servers == 0 || p % servers != 0 || (rings != 1 && rings != 4) ||
        (rings == 4 && p / servers != 8)) {
        return -20;
    }
    uint64_t maxPer = cclBytes / unit;
    if (maxPer == 0) {
        return -21;
    }
    const uint32_t D = p / servers, rootGroup = root / D, rootLocal = root % D;
    Pool pool(threads);
    auto machine = [&](uint32_t n) {
        Machine m;
        m.p = static_cast<int>(n);
        m.dt = dt;
        m.direct = (flags & 1) != 0;
        m.pool = &pool;
        m.buf[B_IN].resize(n);
        m.buf[B_OUT].resize(n);
        return m;
    };
    auto device = [&](uint32_t k, uint32_t i) { return rings > 1 ? kEightDeviceRings[k][i] : i; };
    uint64_t offset = 0;
    for (uint64_t left = count; left > 0 && p > 1;) {
        uint64_t cur = left > maxPer ? maxPer : left;
        uint64_t bytes = cur * unit;
        std::vector<Slice> sl = RingSlices(bytes, D, align);
        std::vector<std::vector<Slice>> segs = MultiSegSlices(sl, rings, align);
        auto at = [&](uint32_t g, uint32_t d) { return static_cast<uint8_t *>(buf[g * D + d]) + offset; };
        for (uint32_t k = 0; k < rings && D > 1; k++) {               // step 1
            Machine m = machine(D);
            std::vector<Slice> ringSl(D);
            uint32_t rootPos = 0;
            for (uint32_t i = 0; i < D; i++) {
                m.buf[B_IN][i] = m.buf[B_OUT][i] = at(rootGroup, device(k, i));
                ringSl[i] = segs[device(k, i)][k];
                if (device(k, i) == rootLocal) {
                    rootPos = i;
                }
            }
            for (uint32_t r = 0; r < D; r++) {
                Proc pr;
                pr.rank = r;
                const int lft = static_cast<int>((r + D - 1) % D), rgt = static_cast<int>((r + 1) % D);
                if (r == rootPos) {
                    for (uint32_t i = 1; i < D; i++) {
                        const uint32_t owner = (r + D - i) % D;
                        pr.prog.push_back(MkSend(rgt, 0, B_IN, ringSl[owner].off, ringSl[owner].size));
                    }
                } else {
                    const uint32_t rounds = (rootPos + D - r) % D;     // parts this position receives, its own last
                    for (uint32_t i = 1; i <= rounds; i++) {
                        const uint32_t owner = (r + rounds - i) % D;
                        if (i != 1) {
                            const uint32_t previous = (r + rounds - i + 1) % D;
                            pr.prog.push_back(MkSend(rgt, 0, B_OUT, ringSl[previous].off, ringSl[previous].size));
                        }
                        pr.prog.push_back(MkRecvCopy(lft, 0, B_OUT, ringSl[owner].off, ringSl[owner].size));
                    }
                }
                m.procs.push_back(std::move(pr));
            }
            int rc = m.Run();
            if (rc != 0) {
                return rc;
            }
            moved += m.bytesTouched;
        }
        for (uint32_t d = 0; d < D && servers > 1; d++) {              // step 2
            if (sl[d].size == 0) {
                continue;
            }
            Machine m = machine(servers);
            for (uint32_t g = 0; g < servers; g++) {
                m.buf[B_IN][g] = m.buf[B_OUT][g] = at(g, d);
            }
            AddBroadcastRhdProcs(m, rootGroup, sl[d].off, sl[d].size);
            int rc = m.Run();
            if (rc != 0) {
                return rc;
            }
            moved += m.bytesTouched;
        }
        for (uint32_t g = 0; g < servers && D > 1; g++) {              // step 3
            for (uint32_t k = 0; k < rings; k++) {
                Machine m = machine(D);
                std::vector<Slice> ringSl(D);
                for (uint32_t i = 0; i < D; i++) {
                    m.buf[B_IN][i] = m.buf[B_OUT][i] = at(g, device(k, i));
                    ringSl[i] = segs[device(k, i)][k];
                }
                for (uint32_t i = 0; i < D; i++) {
                    Proc pr;
                    pr.rank = i;
                    ProgAllGatherRing(pr.prog, i, D, B_OUT, B_OUT, ringSl, ringSl);
                    m.procs.push_back(std::move(pr));
                }
                int rc = m.Run();
                if (rc != 0) {
                    return rc;
                }
                moved += m.bytesTouched;
            }
        }
        offset += bytes;
        left -= cur;
    }
    if (touched != nullptr) {
        *touched = moved;
    }
    return 0;
}

// Per-rank programs of ReduceRecursiveHalvingDoubling::RunAsync (TPL/temp_reduce/reduce_recursive_hd.cc:31-316) on the
// machine's buffers of `bytes` bytes: input accumulates in place, the result ends in the root's output buffer.
void AddReduceRhdProcs(Machine &m, uint32_t root, uint64_t bytes, uint64_t align)
{
    const uint32_t p = static_cast<uint32_t>(m.p);
    uint32_t block, part1;
    RhdParams(p, &block, &part1);
    std::vector<Slice> sl = RhdSlices(bytes, block, align);
    const uint32_t rootFlag = root >= part1 ? 0 : root;
    auto member = [&](uint32_t r) { return r >= part1 || (r % 2) == (rootFlag % 2); };
    auto blockRank = [&](uint32_t r) { return r < part1 ? r / 2 : r - part1 / 2; };
    std::vector<uint32_t> rankOf(block);
    for (uint32_t r = 0; r < p; r++) {
        if (member(r)) {
            rankOf[blockRank(r)] = r;
        }
    }
    const uint32_t rootQ = root > part1 ? root - part1 / 2 : root / 2;   // as written at :246
    uint32_t rounds = 0;
    while ((1u << rounds) < block) {
        rounds++;
    }
    auto sum = [&](uint32_t first, uint32_t n) {
        uint64_t t = 0;
        for (uint32_t i = first; i < first + n; i++) {
            t += sl[i].size;
        }
        return t;
    };
    for (uint32_t r = 0; r < p; r++) {
        Proc pr;
        pr.rank = r;
        const uint32_t pairPeer = (r % 2) == 0 ? r + 1 : r - 1;
        if (!member(r)) {
            pr.prog.push_back(MkSend(static_cast<int>(pairPeer), 1, B_IN, 0, bytes));
            m.procs.push_back(std::move(pr));
            continue;
        }
        if (r < part1) {
            pr.prog.push_back(MkRecvReduce(static_cast<int>(pairPeer), 1, B_IN, 0, B_IN, 0, bytes));
        }
        const uint32_t q = blockRank(r);
        ProgReduceScatterHd(pr.prog, q, block, rankOf, B_IN, B_OUT, sl);
        for (uint32_t step = 0; step < rounds; step++) {
            const uint32_t mask = 1u << step;
            if (step != 0 && (q & (mask - 1)) != (rootQ & (mask - 1))) {
                break;
            }
            const uint32_t peer = q ^ mask;
            if ((q & mask) == (rootQ & mask)) {
                const uint32_t rxId = peer & ~(mask - 1);
                pr.prog.push_back(MkRecvCopy(static_cast<int>(rankOf[peer]), 2, B_OUT, sl[rxId].off, sum(rxId, mask)));
            } else {
                const uint32_t txId = q & ~(mask - 1);
                pr.prog.push_back(MkSend(static_cast<int>(rankOf[peer]), 2, B_OUT, sl[txId].off, sum(txId, mask)));
            }
        }
        m.procs.push_back(std::move(pr));
    }
}

// Per-rank programs of ReduceRing::RunAsync (TPL/temp_reduce/reduce_ring.cc:29-154): the data walks root+1 -> ... -> root.
void AddReduceRingProcs(Machine &m, uint32_t root, uint64_t bytes)
{
    const uint32_t p = static_cast<uint32_t>(m.p);
    for (uint32_t r = 0; r < p; r++) {
        Proc pr;
        pr.rank = r;
        uint32_t left_ = (r + p - 1) % p, right = (r + 1) % p;
        if (r == root) {
            pr.prog.push_back(MkRecvReduce(static_cast<int>(left_), 0, B_OUT, 0, B_IN, 0, bytes));
        } else if (left_ == root) {
            pr.prog.push_back(MkSend(static_cast<int>(right), 0, B_IN, 0, bytes));
        } else {
            pr.prog.push_back(MkRecvReduce(static_cast<int>(left_), 0, B_IN, 0, B_IN, 0, bytes));
            pr.prog.push_back(MkSend(static_cast<int>(right), 0, B_IN, 0, bytes));
        }
        m.procs.push_back(std::move(pr));
    }
}

// Recursive halving-doubling reduce, ReduceRecursiveHalvingDoubling::RunAsync
// (TPL/temp_reduce/reduce_recursive_hd.cc:31-316): ReduceInPartOne (:85-148: in each rank pair of part one the
// rank whose parity is the root's receives), ReduceScatterInBlock (:150-183), GatherInBlock (:236-313: a
// binomial gather over the output buffers towards the root's block rank).  Chunk loop as for the ring reduce.
int orc_reduce_to_root_rhd(uint32_t p, void **in, void *outRoot, uint64_t count, int dt, int op, uint32_t root,
    uint64_t cclBytes, uint64_t align, int flags, int threads)
{
    uint64_t unit = DtSize(dt);
    if (unit == 0 || p == 0 || root >= p) {
        return -20;
    }
    uint64_t maxPer = cclBytes / unit;
    if (maxPer == 0) {
        return -21;
    }
    Pool pool(threads);
    Machine m;
    m.p = static_cast<int>(p);
    m.dt = dt;
    m.op = op;
    m.direct = (flags & 1) != 0;
    m.pool = &pool;
    uint64_t stage = std::min<uint64_t>(count, maxPer) * unit;
    std::vector<std::vector<uint8_t>> cclIn(p, std::vector<uint8_t>(stage)), cclOut(p, std::vector<uint8_t>(stage));
    m.buf[B_IN].resize(p);
    m.buf[B_OUT].resize(p);
    for (uint32_t r = 0; r < p; r++) {
        m.buf[B_IN][r] = cclIn[r].data();
        m.buf[B_OUT][r] = cclOut[r].data();
    }
    uint64_t offset = 0;
    for (uint64_t left = count; left > 0;) {
        uint64_t cur = left > maxPer ? maxPer : left;
        uint64_t bytes = cur * unit;
        for (uint32_t r = 0; r < p; r++) {
            m.Copy(m.buf[B_IN][r], static_cast<uint8_t *>(in[r]) + offset, bytes);
        }
        if (p == 1) {
            m.Copy(m.buf[B_OUT][0], m.buf[B_IN][0], bytes);
        } else {
            AddReduceRhdProcs(m, root, bytes, align);
            int rc = m.Run();
            if (rc != 0) {
                return rc;
            }
        }
        m.Copy(static_cast<uint8_t *>(outRoot) + offset, m.buf[B_OUT][root], bytes);
        offset += bytes;
        left -= cur;
    }
    return 0;
}

// Mesh reduce, CollReduceMeshExecutor::KernelRun (EXE/coll_reduce/coll_reduce_mesh_executor.cc:75-194) on one
// server: mesh reduce-scatter (piece cut, or uncut when `atomic`) over the ring slice plan, the own slice
// copied from input to output, then GatherMesh to the root (TPL/temp_gather/gather_mesh.cc:60-170).
int orc_reduce_to_root_mesh(uint32_t p, void **in, void *outRoot, uint64_t count, int dt, int op, uint32_t root,
    uint64_t cclBytes, uint64_t align, int atomic, int flags, int threads)
{
    uint64_t unit = DtSize(dt);
    if (unit == 0 || p == 0 || root >= p) {
        return -20;
    }
    uint64_t maxPer = cclBytes / unit;
    if (maxPer == 0) {
        return -21;
    }
    Pool pool(threads);
    Machine m;
    m.p = static_cast<int>(p);
    m.dt = dt;
    m.op = op;
    m.direct = (flags & 1) != 0;
    m.pool = &pool;
    uint64_t stage = std::min<uint64_t>(count, maxPer) * unit;
    std::vector<std::vector<uint8_t>> cclIn(p, std::vector<uint8_t>(stage)), cclOut(p, std::vector<uint8_t>(stage));
    m.buf[B_IN].resize(p);
    m.buf[B_OUT].resize(p);
    for (uint32_t r = 0; r < p; r++) {
        m.buf[B_IN][r] = cclIn[r].data();
        m.buf[B_OUT][r] = cclOut[r].data();
    }
    uint64_t offset = 0;
    for (uint64_t left = count; left > 0;) {
        uint64_t cur = left > maxPer ? maxPer : left;
        uint64_t bytes = cur * unit;
        for (uint32_t r = 0; r < p; r++) {
            m.Copy(m.buf[B_IN][r], static_cast<uint8_t *>(in[r]) + offset, bytes);
        }
        if (p == 1) {
            m.Copy(m.buf[B_OUT][0], m.buf[B_IN][0], bytes);
        } else {
            std::vector<Slice> sl = RingSlices(bytes, p, align);
            if (atomic) {
                for (uint32_t r = 0; r < p; r++) {
                    Proc pr;
                    pr.rank = r;
                    ProgReduceScatterMeshAtomic(pr.prog, r, p, B_IN, sl);
                    m.procs.push_back(std::move(pr));
                }
            } else {
                uint32_t nstream = p > 2 ? p - 1 : 1;
                std::vector<std::vector<Slice>> pieces = CutPieces(sl, nstream, align);
                for (uint32_t t = 0; t < nstream; t++) {
                    for (uint32_t r = 0; r < p; r++) {
                        Proc pr;
                        pr.rank = r;
                        ProgReduceScatterMeshStream(pr.prog, r, p, t, B_IN, pieces[t]);
                        m.procs.push_back(std::move(pr));
                    }
                }
            }
            int rc = m.Run();
            if (rc != 0) {
                return rc;
            }
            for (uint32_t r = 0; r < p; r++) {      // one server: the level-1 reduce is a copy input -> output
                m.Copy(m.At(r, B_OUT, sl[r].off), m.At(r, B_IN, sl[r].off), sl[r].size);
            }
            for (uint32_t r = 0; r < p; r++) {      // gather to the root
                Proc pr;
                pr.rank = r;
                if (r == root) {
                    for (uint32_t srcRank = 0; srcRank < p; srcRank++) {
                        if (srcRank != root) {
                            pr.prog.push_back(MkRecvCopy(static_cast<int>(srcRank), 0, B_OUT, sl[srcRank].off, sl[srcRank].size));
                        }
                    }
                } else {
                    pr.prog.push_back(MkSend(static_cast<int>(root), 0, B_OUT, sl[r].off, sl[r].size));
                }
                m.procs.push_back(std::move(pr));
            }
            rc = m.Run();
            if (rc != 0) {
                return rc;
            }
        }
        m.Copy(static_cast<uint8_t *>(outRoot) + offset, m.buf[B_OUT][root], bytes);
        offset += bytes;
        left -= cur;
    }
    return 0;
}


// Two-level reduce, CollReduceMeshExecutor::KernelRun with several servers
// (EXE/coll_reduce/coll_reduce_mesh_executor.cc:75-194): `servers` groups of D = p / servers consecutive ranks.
// Reduce-scatter inside every group over the ring slice plan for D (level0 0 / 1: mesh with the piece cut / uncut;
// 2 / 3: one ring / the four rings of the 8-device topology, EXE/coll_reduce/coll_reduce_ring_plus_hd_executor.cc:75-168); the
// ranks at position d of all groups reduce slice d to the one in the root's group (level1 = ALGO_RING or ALGO_RHD,
// input range to output range; a copy when there is one group); GatherMesh to the root inside its group.
int orc_reduce_to_root_two_level(int level1, int level0, uint32_t servers, uint32_t p, void **in, void *outRoot, uint64_t count,
    int dt, int op, uint32_t root, uint64_t cclBytes, uint64_t align, int flags, int threads)
{
    uint64_t unit = DtSize(dt);
    if (unit == 0 || p == 0 || root >= p || servers == 0 || p % servers != 0 || (level1 != ALGO_RING && level1 != ALGO_RHD) ||
        level0 < 0 || level0 > 3 || (level0 == 3 && p / servers != 8)) {
        return -20;
    }
    const bool atomic = level0 == 1;
    const uint32_t ringCount = level0 == 3 ? 4u : 1u;
    uint64_t maxPer = cclBytes / unit;
    if (maxPer == 0) {
        return -21;
    }
    const uint32_t D = p / servers;
    const uint32_t rootServer = root / D, rootPos = root % D;
    Pool pool(threads);
    auto machine = [&](uint32_t n) {
        Machine m;
        m.p = static_cast<int>(n);
        m.dt = dt;
        m.op = op;
        m.direct = (flags & 1) != 0;
        m.pool = &pool;
        m.buf[B_IN].resize(n);
        m.buf[B_OUT].resize(n);
        return m;
    };
    Machine all = machine(p);
    uint64_t stage = std::min<uint64_t>(count, maxPer) * unit;
    std::vector<std::vector<uint8_t>> cclIn(p, std::vector<uint8_t>(stage)), cclOut(p, std::vector<uint8_t>(stage));
    for (uint32_t r = 0; r < p; r++) {
        all.buf[B_IN][r] = cclIn[r].data();
        all.buf[B_OUT][r] = cclOut[r].data();
    }
    uint64_t offset = 0;
    for (uint64_t left = count; left > 0;) {
        uint64_t cur = left > maxPer ? maxPer : left;
        uint64_t bytes = cur * unit;
        for (uint32_t r = 0; r < p; r++) {
            all.Copy(all.buf[B_IN][r], static_cast<uint8_t *>(in[r]) + offset, bytes);
        }
        std::vector<Slice> sl = RingSlices(bytes, D, align);
        for (uint32_t s = 0; s < servers && D > 1; s++) {
            Machine m = machine(D);
            for (uint32_t d = 0; d < D; d++) {
                m.buf[B_IN][d] = all.buf[B_IN][s * D + d];
                m.buf[B_OUT][d] = all.buf[B_OUT][s * D + d];
            }
            if (level0 >= 2) {
                // CollReduceRingPlusHdExecutor::KernelRun (EXE/coll_reduce/coll_reduce_ring_plus_hd_executor.cc:75-105):
                // the ring reduce-scatter of the two-level all-reduce, one sub-machine per ring
                std::vector<std::vector<Slice>> segs = MultiSegSlices(sl, ringCount, align);
                for (uint32_t k = 0; k < ringCount; k++) {
                    Machine ring = machine(D);
                    std::vector<Slice> ringSl(D);
                    for (uint32_t i = 0; i < D; i++) {
                        uint32_t dev = ringCount > 1 ? kEightDeviceRings[k][i] : i;
                        ring.buf[B_IN][i] = m.buf[B_IN][dev];
                        ring.buf[B_OUT][i] = m.buf[B_OUT][dev];
                        ringSl[i] = segs[dev][k];
                    }
                    for (uint32_t i = 0; i < D; i++) {
                        Proc pr;
                        pr.rank = i;
                        ProgReduceScatterRing(pr.prog, i, D, B_IN, B_IN, ringSl, ringSl);
                        ring.procs.push_back(std::move(pr));
                    }
                    int rc = ring.Run();
                    if (rc != 0) {
                        return rc;
                    }
                }
                continue;
            }
            if (atomic) {
                for (uint32_t d = 0; d < D; d++) {
                    Proc pr;
                    pr.rank = d;
                    ProgReduceScatterMeshAtomic(pr.prog, d, D, B_IN, sl);
                    m.procs.push_back(std::move(pr));
                }
            } else {
                uint32_t nstream = D > 2 ? D - 1 : 1;
                std::vector<std::vector<Slice>> pieces = CutPieces(sl, nstream, align);
                for (uint32_t t = 0; t < nstream; t++) {
                    for (uint32_t d = 0; d < D; d++) {
                        Proc pr;
                        pr.rank = d;
                        ProgReduceScatterMeshStream(pr.prog, d, D, t, B_IN, pieces[t]);
                        m.procs.push_back(std::move(pr));
                    }
                }
            }
            int rc = m.Run();
            if (rc != 0) {
                return rc;
            }
        }
        // level 1: slice d, among the ranks at position d, to the one in the root's group
        for (uint32_t d = 0; d < D; d++) {
            if (sl[d].size == 0) {
                continue;
            }
            Machine m = machine(servers);
            for (uint32_t s = 0; s < servers; s++) {
                m.buf[B_IN][s] = all.buf[B_IN][s * D + d] + sl[d].off;
                m.buf[B_OUT][s] = all.buf[B_OUT][s * D + d] + sl[d].off;
            }
            if (servers == 1) {
                m.Copy(m.buf[B_OUT][0], m.buf[B_IN][0], sl[d].size);
                continue;
            }
            if (level1 == ALGO_RING) {
                AddReduceRingProcs(m, rootServer, sl[d].size);
            } else {
                AddReduceRhdProcs(m, rootServer, sl[d].size, align);
            }
            int rc = m.Run();
            if (rc != 0) {
                return rc;
            }
        }
        // gather inside the root's group
        if (D > 1) {
            Machine m = machine(D);
            for (uint32_t d = 0; d < D; d++) {
                m.buf[B_IN][d] = all.buf[B_IN][rootServer * D + d];
                m.buf[B_OUT][d] = all.buf[B_OUT][rootServer * D + d];
            }
            for (uint32_t d = 0; d < D; d++) {
                Proc pr;
                pr.rank = d;
                if (d == rootPos) {
                    for (uint32_t srcRank = 0; srcRank < D; srcRank++) {
                        if (srcRank != rootPos) {
                            pr.prog.push_back(MkRecvCopy(static_cast<int>(srcRank), 0, B_OUT, sl[srcRank].off, sl[srcRank].size));
                        }
                    }
                } else {
                    pr.prog.push_back(MkSend(static_cast<int>(rootPos), 0, B_OUT, sl[d].off, sl[d].size));
                }
                m.procs.push_back(std::move(pr));
            }
            int rc = m.Run();
            if (rc != 0) {
                return rc;
            }
        }
        all.Copy(static_cast<uint8_t *>(outRoot) + offset, all.buf[B_OUT][root], bytes);
        offset += bytes;
        left -= cur;
    }
    return 0;
}

// Ring reduce (reduce_ring.cc:29-154) with the executor's chunk loop; out[root] receives the result.
// Inputs are staged (the schedule accumulates in its input buffer).
int orc_reduce_to_root(uint32_t p, void **in, void *outRoot, uint64_t count, int dt, int op, uint32_t root, uint64_t cclBytes,
    int flags, int threads)
{
    uint64_t unit = DtSize(dt);
    if (unit == 0 || p == 0 || root >= p) {
        return -20;
    }
    uint64_t maxPer = cclBytes / unit;
    if (maxPer == 0) {
        return -21;
    }
    Pool pool(threads);
    Machine m;
    m.p = static_cast<int>(p);
    m.dt = dt;
    m.op = op;
    m.direct = (flags & 1) != 0;
    m.pool = &pool;
    uint64_t stage = std::min<uint64_t>(count, maxPer) * unit;
    std::vector<std::vector<uint8_t>> cclIn(p, std::vector<uint8_t>(stage)), cclOut(p, std::vector<uint8_t>(stage));
    m.buf[B_IN].resize(p);
    m.buf[B_OUT].resize(p);
    for (uint32_t r = 0; r < p; r++) {
        m.buf[B_IN][r] = cclIn[r].data();
        m.buf[B_OUT][r] = cclOut[r].data();
    }
    uint64_t offset = 0;
    for (uint64_t left = count; left > 0;) {
        uint64_t cur = left > maxPer ? maxPer : left;
        uint64_t bytes = cur * unit;
        for (uint32_t r = 0; r < p; r++) {
            m.Copy(m.buf[B_IN][r], static_cast<uint8_t *>(in[r]) + offset, bytes);
        }
        if (p == 1) {
            m.Copy(m.buf[B_OUT][0], m.buf[B_IN][0], bytes);
        } else {
            AddReduceRingProcs(m, root, bytes);
            int rc = m.Run();
            if (rc != 0) {
                return rc;
            }
        }
        m.Copy(static_cast<uint8_t *>(outRoot) + offset, m.buf[B_OUT][root], bytes);
        offset += bytes;
        left -= cur;
    }
    return 0;
}

// Mesh scatter (scatter_mesh.cc:46-160): in (on the root) holds p blocks of `count` elements.
int orc_scatter(uint32_t p, const void *inRoot, void **out, uint64_t count, int dt, uint32_t root, int flags, int threads)
{
    uint64_t unit = DtSize(dt);
    if (unit == 0 || p == 0 || root >= p) {
        return -20;
    }
    uint64_t bytes = count * unit;
    Pool pool(threads);
    Machine m;
    m.p = static_cast<int>(p);
    m.dt = dt;
    m.direct = (flags & 1) != 0;
    m.pool = &pool;
    m.buf[B_IN].assign(p, nullptr);
    m.buf[B_OUT].resize(p);
    m.buf[B_IN][root] = static_cast<uint8_t *>(const_cast<void *>(inRoot));
    for (uint32_t r = 0; r < p; r++) {
        m.buf[B_OUT][r] = static_cast<uint8_t *>(out[r]);
    }
    for (uint32_t r = 0; r < p; r++) {
        Proc pr;
        pr.rank = r;
        if (r == root) {
            for (uint32_t d = 0; d < p; d++) {
                if (d == root) {
                    pr.prog.push_back(MkLocalCopy(B_OUT, 0, B_IN, bytes * d, bytes));
                } else {
                    pr.prog.push_back(MkSend(static_cast<int>(d), 0, B_IN, bytes * d, bytes));
                }
            }
        } else {
            pr.prog.push_back(MkRecvCopy(static_cast<int>(root), 0, B_OUT, 0, bytes));
        }
        m.procs.push_back(std::move(pr));
    }
    return m.Run();
}

// Ring scatter (TPL/temp_scatter/scatter_ring.cc:22-135,142-218): the root sends the blocks to its right neighbour
// one after the other, the block of the rank before it first (:38-52); a rank in between receives the blocks of all
// ranks from the one before the root down to itself, passes each on before taking the next and keeps the last, its
// own (:77-118); the rank before the root only receives (:55-71).  Blocks travel through an output staging buffer
// of p blocks per rank, each at its own offset.
int orc_scatter_ring(uint32_t p, const void *inRoot, void **out, uint64_t count, int dt, uint32_t root, int flags, int threads)
{
    uint64_t unit = DtSize(dt);
    if (unit == 0 || p == 0 || root >= p) {
        return -20;
    }
    uint64_t bytes = count * unit;
    Pool pool(threads);
    Machine m;
    m.p = static_cast<int>(p);
    m.dt = dt;
    m.direct = (flags & 1) != 0;
    m.pool = &pool;
    std::vector<std::vector<uint8_t>> stage(p, std::vector<uint8_t>(bytes * p + 1));
    m.buf[B_IN].assign(p, nullptr);
    m.buf[B_OUT].resize(p);
    m.buf[B_IN][root] = static_cast<uint8_t *>(const_cast<void *>(inRoot));
    for (uint32_t r = 0; r < p; r++) {
        m.buf[B_OUT][r] = stage[r].data();
    }
    for (uint32_t r = 0; r < p; r++) {
        Proc pr;
        pr.rank = r;
        const int left = static_cast<int>((r + p - 1) % p), right = static_cast<int>((r + 1) % p);
        if (p == 1 || r == root) {
            pr.prog.push_back(MkLocalCopy(B_OUT, bytes * r, B_IN, bytes * r, bytes));
            for (uint32_t i = 1; i < p; i++) {
                uint32_t owner = (r + p - i) % p;
                pr.prog.push_back(MkSend(right, 0, B_IN, bytes * owner, bytes));
            }
        } else {
            const uint32_t rounds = (root + p - r) % p;          // blocks this rank receives, its own last
            for (uint32_t i = 1; i <= rounds; i++) {
                uint32_t owner = (r + rounds - i) % p;
                if (i != 1) {
                    uint32_t previous = (r + rounds - i + 1) % p;
                    pr.prog.push_back(MkSend(right, 0, B_OUT, bytes * previous, bytes));
                }
                pr.prog.push_back(MkRecvCopy(left, 0, B_OUT, bytes * owner, bytes));
            }
        }
        m.procs.push_back(std::move(pr));
    }
    int rc = m.Run();
    if (rc != 0) {
        return rc;
    }
    for (uint32_t r = 0; r < p; r++) {
        m.Copy(static_cast<uint8_t *>(out[r]), stage[r].data() + bytes * r, bytes);
    }
    return 0;
}

// Two-level scatter, CollScatterMeshExecutor::KernelRun with several servers
// (EXE/coll_scatter/coll_scatter_mesh_executor.cc:40-110) under the chunk loop of CollScatterExecutor::RunLoop /
// RunLoopInner (coll_scatter_executor.cc:54-175); `servers` groups of D = p / servers consecutive ranks.
// Per chunk of `cur` elements the root packs the p blocks' parts into its staging buffer (:137-145, source stride =
// the whole block, destination stride = the chunk).  Step 1 (KernelRunLevel1, :198-241, the ring choice of :226-229):
// the ranks at the root's position in every group -- each its group's sub-root (topo_matcher.cc:341-370) -- run
// the ring scatter from the root over `servers` runs of D blocks, in place in their staging buffers.  Step 2
// (:72-101): mesh scatter inside every group from the sub-root over the group's run (scatter_mesh.cc:46-160, base
// offset = the run's), again in place in the staging buffers; then every rank copies its block out (:103-106).
// `touched` (optional) receives the bytes read + written by all ranks.
// level0 = 1 / 2: CollScatterRingExecutor::KernelRun (EXE/coll_scatter/coll_scatter_ring_executor.cc:42-113) instead:
// step 1 is the same, step 2 the ring scatter (scatter_ring.cc) inside every group from the sub-root, along the ranks
// in their order (1) or in the order of ring 0 of the 8-device topology (2; PrepareScatterRingSliceData :115-131 puts
// the blocks in that order).
int orc_scatter_two_level(uint32_t servers, uint32_t p, const void *inRoot, void **out, uint64_t count, int dt,
    uint32_t root, uint64_t cclBytes, uint64_t align, int flags, int threads, uint64_t *touched, int level0)
{
    const uint64_t unit = DtSize(dt);
    if (unit == 0 || p == 0 || root >= p || servers == 0 || p % servers != 0 || align == 0 || level0 < 0 || level0 > 2 ||
        (level0 == 2 && p / servers != 8)) {
        return -20;
    }
    const uint64_t maxPer = cclBytes / p / align * align / unit;
    if (maxPer == 0 && count > 0) {
        return -21;
    }
    const uint32_t D = p / servers, rootGroup = root / D, rootLocal = root % D;
    const uint64_t total = count * unit;
    uint64_t moved = 0;
    Pool pool(threads);
    auto machine = [&](uint32_t n) {
        Machine m;
        m.p = static_cast<int>(n);
        m.dt = dt;
        m.direct = (flags & 1) != 0;
        m.pool = &pool;
        m.buf[B_IN].resize(n);
        m.buf[B_OUT].resize(n);
        return m;
    };
    std::vector<std::vector<uint8_t>> stage(p);
    uint64_t offset = 0;
    for (uint64_t left = count; left > 0;) {
        const uint64_t cur = left * unit * p > cclBytes ? maxPer : left;
        const uint64_t cb = cur * unit;
        for (uint32_t r = 0; r < p; r++) {
            stage[r].assign(cb * p + 1, 0);
        }
        {
            Machine m = machine(1);
            for (uint32_t i = 0; i < p; i++) {
                m.Copy(stage[root].data() + cb * i, static_cast<const uint8_t *>(inRoot) + total * i + offset, cb);
                moved += 2 * cb;
            }
        }
        if (servers > 1) {                             // step 1: runs of D blocks round the ring of sub-roots
            const uint64_t run = cb * D;
            Machine m = machine(servers);
            for (uint32_t g = 0; g < servers; g++) {
                m.buf[B_IN][g] = m.buf[B_OUT][g] = stage[g * D + rootLocal].data();
            }
            for (uint32_t g = 0; g < servers; g++) {
                Proc pr;
                pr.rank = g;
                const int lft = static_cast<int>((g + servers - 1) % servers), rgt = static_cast<int>((g + 1) % servers);
                if (g == rootGroup) {
                    for (uint32_t i = 1; i < servers; i++) {
                        const uint32_t owner = (g + servers - i) % servers;
                        pr.prog.push_back(MkSend(rgt, 0, B_IN, run * owner, run));
                    }
                } else {
                    const uint32_t rounds = (rootGroup + servers - g) % servers;
                    for (uint32_t i = 1; i <= rounds; i++) {
                        const uint32_t owner = (g + rounds - i) % servers;
                        if (i != 1) {
                            pr.prog.push_back(MkSend(rgt, 0, B_OUT, run * ((g + rounds - i + 1) % servers), run));
                        }
                        pr.prog.push_back(MkRecvCopy(lft, 0, B_OUT, run * owner, run));
                    }
                }
                m.procs.push_back(std::move(pr));
            }
            int rc = m.Run();
            if (rc != 0) {
                return rc;
            }
            moved += m.bytesTouched;
        }
        for (uint32_t g = 0; g < servers && D > 1; g++) {      // step 2: inside every group, from the sub-root
            Machine m = machine(D);
            for (uint32_t d = 0; d < D; d++) {
                m.buf[B_IN][d] = m.buf[B_OUT][d] = stage[g * D + d].data() + cb * D * g;
            }
            if (level0 != 0) {
                // machine rank i = ring position i = device order(i); block of a device at cb * device
                auto order = [&](uint32_t i) { return level0 == 2 ? kEightDeviceRings[0][i] : i; };
                uint32_t rootPos = 0;
                for (uint32_t i = 0; i < D; i++) {
                    m.buf[B_IN][i] = m.buf[B_OUT][i] = stage[g * D + order(i)].data() + cb * D * g;
                    rootPos = order(i) == rootLocal ? i : rootPos;
                }
                for (uint32_t r = 0; r < D; r++) {
                    Proc pr;
                    pr.rank = r;
                    const int lft = static_cast<int>((r + D - 1) % D), rgt = static_cast<int>((r + 1) % D);
                    if (r == rootPos) {
                        for (uint32_t i = 1; i < D; i++) {
                            pr.prog.push_back(MkSend(rgt, 0, B_IN, cb * order((r + D - i) % D), cb));
                        }
                    } else {
                        const uint32_t rounds = (rootPos + D - r) % D;
                        for (uint32_t i = 1; i <= rounds; i++) {
                            if (i != 1) {
                                pr.prog.push_back(MkSend(rgt, 0, B_OUT, cb * order((r + rounds - i + 1) % D), cb));
                            }
                            pr.prog.push_back(MkRecvCopy(lft, 0, B_OUT, cb * order((r + rounds - i) % D), cb));
                        }
                    }
                    m.procs.push_back(std::move(pr));
                }
            }
            for (uint32_t d = 0; d < D && level0 == 0; d++) {
                Proc pr;
                pr.rank = d;
                if (d == rootLocal) {
                    for (uint32_t to = 0; to < D; to++) {
                        if (to != rootLocal) {
                            pr.prog.push_back(MkSend(static_cast<int>(to), 0, B_IN, cb * to, cb));
                        }
                    }
                } else {
                    pr.prog.push_back(MkRecvCopy(static_cast<int>(rootLocal), 0, B_OUT, cb * d, cb));
                }
                m.procs.push_back(std::move(pr));
            }
            int rc = m.Run();
            if (rc != 0) {
                return rc;
            }
            moved += m.bytesTouched;
        }
        {
            Machine m = machine(1);
            for (uint32_t r = 0; r < p; r++) {
                m.Copy(static_cast<uint8_t *>(out[r]) + offset, stage[r].data() + cb * r, cb);
                moved += 2 * cb;
            }
        }
        offset += cb;
        left -= cur;
    }
    if (touched != nullptr) {
        *touched = moved;
    }
    return 0;
}

// PairWise all-to-all-v.  counts / displs are p x p row-major tables in elements: row r is what
// rank r passed to HcclAlltoAllV.  Returns 1 if the send / receive tables are not symmetric
// (alltoall_operator.cc:49-72), 0 on success.
// scratchBytes > 0 selects the BCopy piecewise transfer (alltoallv_pairwise.cc:112-189); 0 = ZCopy.
int orc_alltoallv(uint32_t p, void **send, const uint64_t *sendCounts, const uint64_t *sdispls,
    void **recv, const uint64_t *recvCounts, const uint64_t *rdispls, int dt, uint64_t scratchBytes, int flags,
    int threads)
{
    uint64_t unit = DtSize(dt);
    if (unit == 0 || p == 0) {
        return -20;
    }
    for (uint32_t i = 0; i < p; i++) {
        for (uint32_t j = 0; j < p; j++) {
            if (sendCounts[i * p + j] != recvCounts[j * p + i]) {
                return 1;
            }
        }
    }
    Pool pool(threads);
    Machine m;
    m.p = static_cast<int>(p);
    m.dt = dt;
    m.direct = (flags & 1) != 0;
    m.pool = &pool;
    m.buf[B_IN].resize(p);
    m.buf[B_OUT].resize(p);
    for (uint32_t r = 0; r < p; r++) {
        m.buf[B_IN][r] = static_cast<uint8_t *>(send[r]);
        m.buf[B_OUT][r] = static_cast<uint8_t *>(recv[r]);
    }
    for (uint32_t r = 0; r < p; r++) {
        Proc pr;
        pr.rank = r;
        // LocalCopy, alltoallv_pairwise.cc:99-110
        pr.prog.push_back(MkLocalCopy(B_OUT, rdispls[r * p + r] * unit, B_IN, sdispls[r * p + r] * unit,
            sendCounts[r * p + r] * unit));
        for (uint32_t i = 1; i < p; i++) {
            uint32_t prev = (r + p - i) % p, next = (r + i) % p;
            uint64_t sendBytes = sendCounts[r * p + next] * unit, recvBytes = recvCounts[r * p + prev] * unit;
            uint64_t sOff = sdispls[r * p + next] * unit, rOff = rdispls[r * p + prev] * unit;
            if (scratchBytes == 0) {
                pr.prog.push_back(MkSend(static_cast<int>(next), 0, B_IN, sOff, sendBytes));
                pr.prog.push_back(MkRecvCopy(static_cast<int>(prev), 0, B_OUT, rOff, recvBytes));
            } else {
                uint64_t sTimes = (sendBytes + scratchBytes - 1) / scratchBytes;
                uint64_t rTimes = (recvBytes + scratchBytes - 1) / scratchBytes;
                for (uint64_t t = 0; t < std::max(sTimes, rTimes); t++) {
                    if (t < sTimes) {
                        uint64_t cur = std::min(scratchBytes, sendBytes - t * scratchBytes);
                        pr.prog.push_back(MkSend(static_cast<int>(next), 0, B_IN, sOff + t * scratchBytes, cur));
                    }
                    if (t < rTimes) {
                        uint64_t cur = std::min(scratchBytes, recvBytes - t * scratchBytes);
                        pr.prog.push_back(MkRecvCopy(static_cast<int>(prev), 0, B_OUT, rOff + t * scratchBytes, cur));
                    }
                }
            }
        }
        m.procs.push_back(std::move(pr));
    }
    return m.Run();
}

// Rounds of the BCopy form per step: the loop of AlltoAllVPairWise::RunBCopyAlltoAll (alltoallv_pairwise.cc:112-171)
// with CalcSendRecvCounts (:173-189) restated literally for every rank.  rounds[i] (i = 1 .. p-1; rounds[0] = 1, the
// local copy) = the SendRecv calls of the rank that makes the most in step i; maxPiece = the largest piece any call
// moves; pieceBytes = the sum over all ranks and calls of the bytes sent.  Returns 0, or -20 on bad arguments.
int orc_alltoallv_rounds(uint32_t p, const uint64_t *sendCounts, const uint64_t *recvCounts, int dt, uint64_t scratchBytes,
    uint64_t *rounds, uint64_t *maxPiece, uint64_t *pieceBytes)
{
    const uint64_t unit = DtSize(dt);
    if (unit == 0 || p == 0 || scratchBytes == 0) {
        return -20;
    }
    auto curBytes = [&](uint64_t times, uint64_t cur, uint64_t total) -> uint64_t {
        if (times == 0) {
            return 0;
        } else if (times == 1 && cur == times - 1) {
            return total;
        } else if (times > 1 && total % scratchBytes == 0 && cur < times) {
            return scratchBytes;
        } else if (times > 1 && total % scratchBytes != 0 && cur < times - 1) {
            return scratchBytes;
        } else if (times > 1 && total % scratchBytes != 0 && cur == times - 1) {
            return total % scratchBytes;
        }
        return 0;
    };
    *maxPiece = 0;
    *pieceBytes = 0;
    rounds[0] = 1;
    for (uint32_t i = 1; i < p; i++) {
        rounds[i] = 0;
        for (uint32_t r = 0; r < p; r++) {
            const uint32_t prev = (r + p - i) % p, next = (r + i) % p;
            const uint64_t sendBytes = sendCounts[r * p + next] * unit, recvBytes = recvCounts[r * p + prev] * unit;
            const uint64_t sendTimes = sendBytes / scratchBytes + (sendBytes % scratchBytes == 0 ? 0 : 1);
            const uint64_t recvTimes = recvBytes / scratchBytes + (recvBytes % scratchBytes == 0 ? 0 : 1);
            uint64_t curSend = 0, curRecv = 0, calls = 0;
            while (sendTimes != 0 || recvTimes != 0) {
                const uint64_t s = curBytes(sendTimes, curSend, sendBytes), v = curBytes(recvTimes, curRecv, recvBytes);
                calls++;
                *maxPiece = std::max(*maxPiece, std::max(s, v));
                *pieceBytes += s;
                curSend = s != 0 ? curSend + 1 : curSend;
                curRecv = v != 0 ? curRecv + 1 : curRecv;
                if (curSend == sendTimes && curRecv == recvTimes) {
                    break;
                }
            }
            rounds[i] = std::max(rounds[i], calls);
        }
    }
    return 0;
}

// Batches of the staged schedule's second stage in its buffer-copy form: CalcSendRecvTimes and LoadPolicies of
// AlltoAllVStagedPairwise (alltoallv_staged_pairwise.cc:185-244) restated literally for the send side of every rank
// (c, l) and step i: the run for server c + i is the list of blocks (source k = 0 .. m-1 of the own server, addressed
// to rank (c + i, l)); blocks are packed into a batch of `scratchBytes` in order, a block that does not fit is cut
// where the batch is full (SplitSendRecvAddrInfo :317-330), an empty block is skipped.  rounds[i] (i = 1 ..
// servers-1; rounds[0] = 1, the local copies) = the batches of the pair with the most in step i; entries = the list
// entries of all batches of all ranks that carry bytes (blocks and parts of blocks; when the rest of a cut block fills
// a batch exactly, the reference closes that batch only at the next block, with an entry of no bytes in front, :226-236:
// restated, not counted); maxBatch = the bytes of the fullest batch.
// Returns 0, -20 on bad arguments, -22 if a batch count disagrees with CalcSendRecvTimes (CheckPolicies :246-265).
int orc_alltoallv_staged_rounds(uint32_t p, uint32_t servers, const uint64_t *sendCounts, int dt, uint64_t scratchBytes,
    uint64_t *rounds, uint64_t *entries, uint64_t *maxBatch)
{
    const uint64_t unit = DtSize(dt);
    if (unit == 0 || p == 0 || servers == 0 || p % servers != 0 || scratchBytes == 0) {
        return -20;
    }
    const uint32_t m = p / servers;
    *entries = 0;
    *maxBatch = 0;
    rounds[0] = 1;
    for (uint32_t i = 1; i < servers; i++) {
        rounds[i] = 0;
        for (uint32_t r = 0; r < p; r++) {
            const uint32_t c = r / m, l = r % m, dest = ((c + i) % servers) * m + l;
            std::vector<uint64_t> blocks;
            uint64_t sendBytes = 0;
            for (uint32_t k = 0; k < m; k++) {
                blocks.push_back(sendCounts[size_t(c * m + k) * p + dest] * unit);
                sendBytes += blocks.back();
            }
            const uint64_t sendTimes = sendBytes / scratchBytes + (sendBytes % scratchBytes == 0 ? 0 : 1);
            std::vector<std::vector<uint64_t>> policies(sendTimes);
            std::vector<uint64_t> temp;
            uint64_t curTime = 0, room = scratchBytes;
            for (uint64_t block : blocks) {
                if (block == 0) {
                    continue;
                }
                if (block <= room) {
                    temp.push_back(block);
                    room -= block;
                    if (room == 0) {
                        room = scratchBytes;
                        if (curTime >= sendTimes) {
                            return -22;
                        }
                        policies[curTime++] = temp;
                        temp.clear();
                    }
                } else {
                    uint64_t rest = block;
                    while (rest > room) {
                        temp.push_back(room);
                        rest -= room;
                        room = scratchBytes;
                        if (curTime >= sendTimes) {
                            return -22;
                        }
                        policies[curTime++] = temp;
                        temp.clear();
                    }
                    if (rest != 0) {
                        temp.push_back(rest);
                        room -= rest;
                    }
                }
            }
            if (room != scratchBytes) {
                if (curTime >= sendTimes) {
                    return -22;
                }
                policies[curTime++] = temp;
            }
            if (curTime != sendTimes) {
                return -22;
            }
            for (const std::vector<uint64_t> &batch : policies) {
                uint64_t sum = 0;
                for (uint64_t part : batch) {
                    sum += part;
                }
                if (sum > scratchBytes) {
                    return -22;
                }
                *maxBatch = std::max(*maxBatch, sum);
                for (uint64_t part : batch) {
                    *entries += part > 0 ? 1 : 0;
                }
            }
            rounds[i] = std::max(rounds[i], sendTimes);
        }
    }
    return 0;
}

// Staged all-to-all-v over `servers` servers of m = p / servers ranks (zero-copy mode), same tables as
// orc_alltoallv.  Stage one, inside a server (ALG/impl/coll_executor/coll_all_to_all/coll_all_to_all_v_staged_executor.cc:
// 378-440; address tables coll_all_to_all_executor.cc:156-335; template TPL/temp_alltoallv/alltoallv_staged_mesh.cc:51-130):
// rank (c, l) gathers into a workspace, from each rank k of its server, the blocks addressed to the ranks with local
// index l, ordered by destination and then by source.  Stage two, between the servers (:300-352, :441-456; template
// alltoallv_staged_pairwise.cc:65-147): the ranks with local index l exchange their runs pairwise, every block
// landing at its displacement in the destination's receive buffer.  Returns 0, 1 for asymmetric tables, 2 when the
// servers are not of one size.
int orc_alltoallv_staged(uint32_t p, uint32_t servers, void **send, const uint64_t *sendCounts, const uint64_t *sdispls,
    void **recv, const uint64_t *recvCounts, const uint64_t *rdispls, int dt, int flags, int threads)
{
    uint64_t unit = DtSize(dt);
    if (unit == 0 || p == 0 || servers == 0) {
        return -20;
    }
    if (p % servers != 0) {
        return 2;
    }
    for (uint32_t i = 0; i < p; i++) {
        for (uint32_t j = 0; j < p; j++) {
            if (sendCounts[i * p + j] != recvCounts[j * p + i]) {
                return 1;
            }
        }
    }
    const uint32_t m = p / servers;
    auto len = [&](uint32_t src, uint32_t dst) { return sendCounts[size_t(src) * p + dst] * unit; };
    // workspace offset of the block (destination j, source local rank k) at rank (c, l), j = l mod m:
    // everything before it in (destination, source) order (coll_all_to_all_executor.cc:171-187)
    auto workOff = [&](uint32_t c, uint32_t j, uint32_t k) {
        uint64_t off = 0;
        for (uint32_t jj = j % m; jj <= j; jj += m) {
            for (uint32_t kk = 0; kk < m; kk++) {
                if (jj == j && kk == k) {
                    return off;
                }
                off += len(c * m + kk, jj);
            }
        }
        return off;
    };
    std::vector<std::vector<uint8_t>> work(p);
    for (uint32_t r = 0; r < p; r++) {
        uint64_t total = 0;
        for (uint32_t j = r % m; j < p; j += m) {
            for (uint32_t k = 0; k < m; k++) {
                total += len(r / m * m + k, j);
            }
        }
        work[r].assign(total + 1, 0);
    }
    Pool pool(threads);
    Machine mc;
    mc.p = static_cast<int>(p);
    mc.dt = dt;
    mc.direct = (flags & 1) != 0;
    mc.pool = &pool;
    mc.buf[B_IN].resize(p);
    mc.buf[B_OUT].resize(p);
    // stage one: send buffer -> workspace
    for (uint32_t r = 0; r < p; r++) {
        mc.buf[B_IN][r] = static_cast<uint8_t *>(send[r]);
        mc.buf[B_OUT][r] = work[r].data();
    }
    for (uint32_t r = 0; r < p; r++) {
        const uint32_t c = r / m, l = r % m;
        Proc pr;
        pr.rank = static_cast<int>(r);
        for (uint32_t j = l; j < p; j += m) {   // LocalCopy (alltoallv_staged_base.cc:36-56)
            pr.prog.push_back(MkLocalCopy(B_OUT, workOff(c, j, l), B_IN, sdispls[size_t(r) * p + j] * unit, len(r, j)));
        }
        for (uint32_t i = 1; i < m; i++) {      // one stream per neighbour (alltoallv_staged_mesh.cc:96-130)
            const uint32_t dl = (l + i) % m, dest = c * m + dl;
            for (uint32_t j = dl; j < p; j += m) {
                pr.prog.push_back(MkSend(static_cast<int>(dest), static_cast<int>(i), B_IN, sdispls[size_t(r) * p + j] * unit, len(r, j)));
            }
        }
        for (uint32_t i = 1; i < m; i++) {
            const uint32_t sl = (l + m - i) % m, src = c * m + sl;
            for (uint32_t j = l; j < p; j += m) {
                pr.prog.push_back(MkRecvCopy(static_cast<int>(src), static_cast<int>(i), B_OUT, workOff(c, j, sl), len(src, j)));
            }
        }
        mc.procs.push_back(std::move(pr));
    }
    int rc = mc.Run();
    if (rc != 0) {
        return rc;
    }
    // stage two: workspace -> receive buffers
    for (uint32_t r = 0; r < p; r++) {
        mc.buf[B_IN][r] = work[r].data();
        mc.buf[B_OUT][r] = static_cast<uint8_t *>(recv[r]);
    }
    for (uint32_t r = 0; r < p; r++) {
        const uint32_t c = r / m, l = r % m;
        Proc pr;
        pr.rank = static_cast<int>(r);
        for (uint32_t k = 0; k < m; k++) {      // LocalCopy: the run addressed to this rank itself
            pr.prog.push_back(MkLocalCopy(B_OUT, rdispls[size_t(r) * p + c * m + k] * unit, B_IN, workOff(c, r, k), len(c * m + k, r)));
        }
        for (uint32_t i = 1; i < servers; i++) {
            const uint32_t nc = (c + i) % servers, pc = (c + servers - i) % servers;
            const uint32_t next = nc * m + l, prev = pc * m + l;
            for (uint32_t k = 0; k < m; k++) {
                pr.prog.push_back(MkSend(static_cast<int>(next), 0, B_IN, workOff(c, next, k), len(c * m + k, next)));
            }
            for (uint32_t k = 0; k < m; k++) {
                pr.prog.push_back(MkRecvCopy(static_cast<int>(prev), 0, B_OUT, rdispls[size_t(r) * p + pc * m + k] * unit, len(pc * m + k, r)));
            }
        }
        mc.procs.push_back(std::move(pr));
    }
    return mc.Run();
}

// ---- synthetic data ------------------------------------------------------------------------------
static inline uint64_t SplitMix(uint64_t x)
{
    x += 0x9e3779b97f4a7c15ull;
    x = (x ^ (x >> 30)) * 0xbf58476d1ce4e5b9ull;
    x = (x ^ (x >> 27)) * 0x94d049bb133111ebull;
    return x ^ (x >> 31);
}

// x[i] = (u32 >> 8) * 2^-23 - 1  in [-1, 1), counter-based on (seed, rank, i).
void orc_fill_uniform_f32(float *dst, uint64_t n, uint64_t seed, uint32_t rank, int threads)
{
    Pool pool(threads);
    uint64_t key = seed ^ (static_cast<uint64_t>(rank) << 32);
    pool.Run(n, 16, [&](uint64_t b, uint64_t e) {
        for (uint64_t i = b; i < e; i++) {
            uint32_t u = static_cast<uint32_t>(SplitMix(key + i * 0x2545f4914f6cdd1dull) >> 32);
            dst[i] = static_cast<float>(u >> 8) * 1.1920928955078125e-07f - 1.0f;
        }
    });
}

}  // extern "C"
