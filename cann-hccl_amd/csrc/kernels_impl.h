// gfx950 kernels for the per-rank data path: element-wise reduce / copy over descriptor tables.
// Bandwidth-bound work: 128-bit coalesced loads and stores, several independent loads in flight per
// lane, no LDS, no matrix cores.  One launch covers every step of a phase (or every fused item) for
// all ranks; a workgroup walks tiles of kTileBytes with a grid stride.
//
// Arithmetic rules (must match bit for bit on every path):
//   integers   sum / prod wrap modulo 2^n; max = (b > a) ? b : a, min = (b < a) ? b : a
//   fp32/fp64  one IEEE operation per combine, same max / min selection rule
//   fp16/bf16  widen to fp32, combine, round to nearest even; max / min keep the chosen operand's bits
#pragma once
#include <hip/hip_runtime.h>
#include <cstdint>

#include "kernels.h"

namespace hcclamd {

typedef uint32_t V4 __attribute__((ext_vector_type(4)));   // 16 bytes, one global_load_dwordx4

struct HalfBits { uint16_t v; };
struct Bf16Bits { uint16_t v; };

enum : int { ROP_SUM = 0, ROP_PROD = 1, ROP_MAX = 2, ROP_MIN = 3 };

// ---- element arithmetic ---------------------------------------------------------------------------
template <typename T> struct UnsignedOf { using type = T; };
template <> struct UnsignedOf<int8_t> { using type = uint8_t; };
template <> struct UnsignedOf<int16_t> { using type = uint16_t; };
template <> struct UnsignedOf<int32_t> { using type = uint32_t; };
template <> struct UnsignedOf<int64_t> { using type = uint64_t; };

template <typename T, int OP> struct Elem {
    // integers
    static __device__ __forceinline__ T Apply(T a, T b)
    {
        using U = typename UnsignedOf<T>::type;
        if (OP == ROP_SUM) {
            return static_cast<T>(static_cast<U>(static_cast<uint32_t>(static_cast<U>(a)) + static_cast<uint32_t>(static_cast<U>(b))));
        } else if (OP == ROP_PROD) {
            return static_cast<T>(static_cast<U>(static_cast<uint32_t>(static_cast<U>(a)) * static_cast<uint32_t>(static_cast<U>(b))));
        } else if (OP == ROP_MAX) {
            return (b > a) ? b : a;
        } else {
            return (b < a) ? b : a;
        }
    }
};
template <typename T, int OP> struct Elem64 {
    static __device__ __forceinline__ T Apply(T a, T b)
    {
        if (OP == ROP_SUM) {
            return static_cast<T>(static_cast<uint64_t>(a) + static_cast<uint64_t>(b));
        } else if (OP == ROP_PROD) {
            return static_cast<T>(static_cast<uint64_t>(a) * static_cast<uint64_t>(b));
        } else if (OP == ROP_MAX) {
            return (b > a) ? b : a;
        } else {
            return (b < a) ? b : a;
        }
    }
};
template <int OP> struct Elem<int64_t, OP> : Elem64<int64_t, OP> {};
template <int OP> struct Elem<uint64_t, OP> : Elem64<uint64_t, OP> {};

template <typename F, int OP> struct ElemFloat {
    static __device__ __forceinline__ F Apply(F a, F b)
    {
        if (OP == ROP_SUM) {
            return a + b;
        } else if (OP == ROP_PROD) {
            return a * b;
        } else if (OP == ROP_MAX) {
            return (b > a) ? b : a;
        } else {
            return (b < a) ? b : a;
        }
    }
};
template <int OP> struct Elem<float, OP> : ElemFloat<float, OP> {};
template <int OP> struct Elem<double, OP> : ElemFloat<double, OP> {};

__device__ __forceinline__ float Bf16ToFloat(uint16_t b) { return __uint_as_float(static_cast<uint32_t>(b) << 16); }
__device__ __forceinline__ uint16_t FloatToBf16(float f)
{
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) {
        return static_cast<uint16_t>((u >> 16) | 0x0040u);
    }
    u += 0x7fffu + ((u >> 16) & 1u);
    return static_cast<uint16_t>(u >> 16);
}
__device__ __forceinline__ float HalfToFloat(uint16_t h)
{
    _Float16 x;
    __builtin_memcpy(&x, &h, 2);
    return static_cast<float>(x);
}
__device__ __forceinline__ uint16_t FloatToHalf(float f)
{
    _Float16 x = static_cast<_Float16>(f);   // v_cvt_f16_f32, round to nearest even
    uint16_t h;
    __builtin_memcpy(&h, &x, 2);
    return h;
}

template <int OP> struct Elem<HalfBits, OP> {
    static __device__ __forceinline__ HalfBits Apply(HalfBits a, HalfBits b)
    {
        float fa = HalfToFloat(a.v), fb = HalfToFloat(b.v);
        HalfBits r;
        if (OP == ROP_SUM) {
            r.v = FloatToHalf(fa + fb);
        } else if (OP == ROP_PROD) {
            r.v = FloatToHalf(fa * fb);
        } else if (OP == ROP_MAX) {
            r.v = (fb > fa) ? b.v : a.v;
        } else {
            r.v = (fb < fa) ? b.v : a.v;
        }
        return r;
    }
};
template <int OP> struct Elem<Bf16Bits, OP> {
    static __device__ __forceinline__ Bf16Bits Apply(Bf16Bits a, Bf16Bits b)
    {
        float fa = Bf16ToFloat(a.v), fb = Bf16ToFloat(b.v);
        Bf16Bits r;
        if (OP == ROP_SUM) {
            r.v = FloatToBf16(fa + fb);
        } else if (OP == ROP_PROD) {
            r.v = FloatToBf16(fa * fb);
        } else if (OP == ROP_MAX) {
            r.v = (fb > fa) ? b.v : a.v;
        } else {
            r.v = (fb < fa) ? b.v : a.v;
        }
        return r;
    }
};

// 16 bytes of T combined lane by lane; a is the rank's own operand, b the peer's.
template <typename T, int OP> struct Combiner {
    static __device__ __forceinline__ V4 Apply(V4 a, V4 b)
    {
        constexpr int N = 16 / sizeof(T);
        union U {
            V4 v;
            T e[N];
            __device__ U() {}
        } ua, ub, ur;
        ua.v = a;
        ub.v = b;
#pragma unroll
        for (int i = 0; i < N; i++) {
            ur.e[i] = Elem<T, OP>::Apply(ua.e[i], ub.e[i]);
        }
        return ur.v;
    }
};

// Narrow types work on whole 32-bit words with packed 16-bit instructions (v_pk_*_u16 / _i16) and the
// hardware bf16 conversion (v_cvt_pk_bf16_f32, round to nearest even), a fraction of the instructions
// that element-by-element extraction costs; the results are the same bits.
typedef short S2 __attribute__((ext_vector_type(2)));
typedef unsigned short U2 __attribute__((ext_vector_type(2)));
typedef float F2 __attribute__((ext_vector_type(2)));
typedef __bf16 B2 __attribute__((ext_vector_type(2)));

template <typename To, typename From> __device__ __forceinline__ To BitCast(From f)
{
    static_assert(sizeof(To) == sizeof(From), "size");
    To t;
    __builtin_memcpy(&t, &f, sizeof(To));
    return t;
}

template <bool SIGNED, int OP> __device__ __forceinline__ uint32_t Pk16(uint32_t a, uint32_t b)
{
    if (OP == ROP_SUM) {
        return BitCast<uint32_t>(U2(BitCast<U2>(a) + BitCast<U2>(b)));
    } else if (OP == ROP_PROD) {
        return BitCast<uint32_t>(U2(BitCast<U2>(a) * BitCast<U2>(b)));
    } else if (SIGNED) {
        S2 x = BitCast<S2>(a), y = BitCast<S2>(b);
        return BitCast<uint32_t>(OP == ROP_MAX ? __builtin_elementwise_max(x, y) : __builtin_elementwise_min(x, y));
    } else {
        U2 x = BitCast<U2>(a), y = BitCast<U2>(b);
        return BitCast<uint32_t>(OP == ROP_MAX ? __builtin_elementwise_max(x, y) : __builtin_elementwise_min(x, y));
    }
}

template <bool SIGNED, int OP> __device__ __forceinline__ uint32_t Pk8(uint32_t a, uint32_t b)
{
    if (OP == ROP_SUM) {
        // add the low 7 bits of every byte, then fix the top bits without carrying across bytes
        return ((a & 0x7f7f7f7fu) + (b & 0x7f7f7f7fu)) ^ ((a ^ b) & 0x80808080u);
    } else if (OP == ROP_PROD) {
        uint32_t even = Pk16<false, ROP_PROD>(a & 0x00ff00ffu, b & 0x00ff00ffu) & 0x00ff00ffu;
        uint32_t odd = Pk16<false, ROP_PROD>((a >> 8) & 0x00ff00ffu, (b >> 8) & 0x00ff00ffu) & 0x00ff00ffu;
        return even | (odd << 8);
    } else {
        // a byte moved to the top of a 16-bit lane compares like the byte itself
        uint32_t even = Pk16<SIGNED, OP>((a << 8) & 0xff00ff00u, (b << 8) & 0xff00ff00u);
        uint32_t odd = Pk16<SIGNED, OP>(a & 0xff00ff00u, b & 0xff00ff00u);
        return ((even >> 8) & 0x00ff00ffu) | odd;
    }
}

template <int OP> __device__ __forceinline__ uint32_t PkBf16(uint32_t a, uint32_t b)
{
    const uint32_t aLo = a << 16, aHi = a & 0xffff0000u, bLo = b << 16, bHi = b & 0xffff0000u;
    const float faLo = __uint_as_float(aLo), faHi = __uint_as_float(aHi);
    const float fbLo = __uint_as_float(bLo), fbHi = __uint_as_float(bHi);
    if (OP == ROP_SUM || OP == ROP_PROD) {
        F2 r;
        r.x = (OP == ROP_SUM) ? faLo + fbLo : faLo * fbLo;
        r.y = (OP == ROP_SUM) ? faHi + fbHi : faHi * fbHi;
        return BitCast<uint32_t>(__builtin_convertvector(r, B2));
    } else {
        const bool pickLo = (OP == ROP_MAX) ? (fbLo > faLo) : (fbLo < faLo);
        const bool pickHi = (OP == ROP_MAX) ? (fbHi > faHi) : (fbHi < faHi);
        return ((pickHi ? bHi : aHi)) | ((pickLo ? bLo : aLo) >> 16);
    }
}

// fp16, two elements per word.  Sum and product use the packed half instructions (v_pk_add_f16 / v_pk_mul_f16), one
// per word instead of four conversions, two operations and a conversion back.  The bits are those of "widen to fp32,
// combine, round to nearest even": an fp32 has 24 significant bits, 2 x 11 + 2, and with that many the second rounding
// of a sum never changes what a single rounding to 11 bits gives (the product of two halves is exact in fp32 to begin
// with); denormal halves are kept by both forms.  Max / min compare the halves as they are (the conversion to fp32 is
// exact and keeps the order) and keep the chosen operand's bits.
typedef _Float16 H2 __attribute__((ext_vector_type(2)));
template <int OP> __device__ __forceinline__ uint32_t PkF16(uint32_t a, uint32_t b)
{
    const H2 x = BitCast<H2>(a), y = BitCast<H2>(b);
    if (OP == ROP_SUM || OP == ROP_PROD) {
        const H2 r = (OP == ROP_SUM) ? x + y : x * y;
        return BitCast<uint32_t>(r);
    } else {
        const bool pickLo = (OP == ROP_MAX) ? (y.x > x.x) : (y.x < x.x);
        const bool pickHi = (OP == ROP_MAX) ? (y.y > x.y) : (y.y < x.y);
        return ((pickHi ? b : a) & 0xffff0000u) | ((pickLo ? b : a) & 0x0000ffffu);
    }
}

#define HCCL_WORDWISE_COMBINER(TYPE, EXPR)                                  \
    template <int OP> struct Combiner<TYPE, OP> {                           \
        static __device__ __forceinline__ V4 Apply(V4 a, V4 b)              \
        {                                                                   \
            V4 r;                                                           \
            r.x = EXPR(a.x, b.x);                                           \
            r.y = EXPR(a.y, b.y);                                           \
            r.z = EXPR(a.z, b.z);                                           \
            r.w = EXPR(a.w, b.w);                                           \
            return r;                                                       \
        }                                                                   \
    };
#define HCCL_EXPR_I16(x, y) Pk16<true, OP>(x, y)
#define HCCL_EXPR_U16(x, y) Pk16<false, OP>(x, y)
#define HCCL_EXPR_I8(x, y) Pk8<true, OP>(x, y)
#define HCCL_EXPR_U8(x, y) Pk8<false, OP>(x, y)
#define HCCL_EXPR_BF16(x, y) PkBf16<OP>(x, y)
#define HCCL_EXPR_F16(x, y) PkF16<OP>(x, y)
HCCL_WORDWISE_COMBINER(int16_t, HCCL_EXPR_I16)
HCCL_WORDWISE_COMBINER(uint16_t, HCCL_EXPR_U16)
HCCL_WORDWISE_COMBINER(int8_t, HCCL_EXPR_I8)
HCCL_WORDWISE_COMBINER(uint8_t, HCCL_EXPR_U8)
HCCL_WORDWISE_COMBINER(Bf16Bits, HCCL_EXPR_BF16)
HCCL_WORDWISE_COMBINER(HalfBits, HCCL_EXPR_F16)

template <typename T, int OP> __device__ __forceinline__ V4 Combine16(V4 a, V4 b) { return Combiner<T, OP>::Apply(a, b); }

// ---- memory access ---------------------------------------------------------------------------------
// 16 bytes at an address of any alignment: the device runs in unaligned-access mode, so this is still
// one 128-bit load or store (one that may touch two memory lines).
typedef uint32_t V4U __attribute__((ext_vector_type(4), aligned(1)));

// Rank buffers are device (global) memory.  The pointers come out of descriptor tables, so the
// compiler cannot know that and would issue flat accesses, whose completion is counted together
// with scalar loads (a wait for the next descriptor pointer then also waits for every load in
// flight).  Casting to the global address space gives global_load / global_store.
#define HCCL_GLOBAL __attribute__((address_space(1)))
typedef V4 HCCL_GLOBAL GlobalV4;
typedef V4U HCCL_GLOBAL GlobalV4U;

// 16 bytes in LDS (the gather kernel's staging area; the tiles a team kernel holds between its read and write phases)
typedef V4 __attribute__((address_space(3))) LdsV4;
typedef V4U __attribute__((address_space(3))) LdsV4U;

template <uint32_t MODE> __device__ __forceinline__ V4 Load16(const void *base, uint64_t byteOff)
{
    const char *p = static_cast<const char *>(base) + byteOff;
    if (MODE == ACC_VEC16) {
        return __builtin_nontemporal_load((const GlobalV4 *)p);
    } else {
        V4U t = __builtin_nontemporal_load((const GlobalV4U *)p);
        return V4{t.x, t.y, t.z, t.w};
    }
}
__device__ __forceinline__ void Store16(void *base, uint64_t byteOff, V4 v)
{
    __builtin_nontemporal_store(v, (GlobalV4 *)(static_cast<char *>(base) + byteOff));
}

// Element-wise access to global memory (heads, tails, unaligned buffers).
template <size_t N> struct ElemCarrier;
template <> struct ElemCarrier<1> { typedef uint8_t type; };
template <> struct ElemCarrier<2> { typedef uint16_t type; };
template <> struct ElemCarrier<4> { typedef uint32_t type; };
template <> struct ElemCarrier<8> { typedef uint64_t type; };
template <typename T> __device__ __forceinline__ T LoadElem(const void *base, uint64_t byteOff)
{
    typedef typename ElemCarrier<sizeof(T)>::type C;
    C c = *(const C HCCL_GLOBAL *)(static_cast<const char *>(base) + byteOff);
    T t;
    __builtin_memcpy(&t, &c, sizeof(T));
    return t;
}
template <typename T> __device__ __forceinline__ void StoreElem(void *base, uint64_t byteOff, T t)
{
    typedef typename ElemCarrier<sizeof(T)>::type C;
    C c;
    __builtin_memcpy(&c, &t, sizeof(T));
    *(C HCCL_GLOBAL *)(static_cast<char *>(base) + byteOff) = c;
}

// Accesses of the step kernel.  Loads are non-temporal; stores are ordinary write-back stores: what
// one phase writes the next phase reads, and part of it is still in the memory-side cache then
// (measured, 8-rank fp32 ring all-reduce of 256 MiB per rank, 14 phases: 1.478 ms with non-temporal
// stores, 1.433 ms with ordinary ones; ordinary loads instead cost 9 %).  The fused kernels write
// results nobody reads back and keep non-temporal stores (ordinary ones cost 7 % at 256 MiB per rank).
__device__ __forceinline__ V4 StepLoad(const void *base, uint64_t byteOff)
{
    return Load16<ACC_VEC16>(base, byteOff);
}
template <bool ORDINARY> __device__ __forceinline__ void StepStore(void *base, uint64_t byteOff, V4 v)
{
    if (ORDINARY) {
        *(GlobalV4 *)(static_cast<char *>(base) + byteOff) = v;
    } else {
        Store16(base, byteOff, v);
    }
}

// Largest i with table[i].tile0 <= tile (tile0 is ascending, table[0].tile0 == 0).
template <typename D> __device__ __forceinline__ uint32_t FindDesc(const D *table, uint32_t n, uint32_t tile)
{
    uint32_t lo = 0, hi = n;
    while (hi - lo > 1) {
        uint32_t mid = (lo + hi) >> 1;
        if (table[mid].tile0 <= tile) {
            lo = mid;
        } else {
            hi = mid;
        }
    }
    return lo;
}

// Item of a tile in a fused launch.  When every item of the launch covers `tilesPerItem` tiles (the last one at most
// as many; 0 = they differ), the index follows from the tile number and the table search, a chain of dependent loads
// that is most of a small collective's time, is not needed.
template <typename D> __device__ __forceinline__ uint32_t ItemOfTile(const D *table, uint32_t n, uint32_t tile, uint32_t tilesPerItem)
{
    if (tilesPerItem != 0) {
        const uint32_t i = tile / tilesPerItem;
        return i < n ? i : n - 1;
    }
    return FindDesc(table, n, tile);
}

constexpr uint32_t kVecPerLane = kTileBytes / (kBlockThreads * 16);   // 4

// ---- one phase of copy / reduce steps -----------------------------------------------------------------
template <typename T, int OP, uint32_t MODE>
__device__ __forceinline__ void StepTileVec(const StepDesc &d, uint64_t off, uint32_t n)
{
    const uint32_t nvec = n >> 4;
    const uint32_t tid = threadIdx.x;
    if (nvec == kTileBytes / 16) {
        V4 va[kVecPerLane], vb[kVecPerLane];
#pragma unroll
        for (uint32_t u = 0; u < kVecPerLane; u++) {
            va[u] = Load16<MODE>(d.a, off + (uint64_t(u) * kBlockThreads + tid) * 16);
        }
        if (d.b != nullptr) {
#pragma unroll
            for (uint32_t u = 0; u < kVecPerLane; u++) {
                vb[u] = Load16<MODE>(d.b, off + (uint64_t(u) * kBlockThreads + tid) * 16);
            }
#pragma unroll
            for (uint32_t u = 0; u < kVecPerLane; u++) {
                va[u] = Combine16<T, OP>(va[u], vb[u]);
            }
        }
#pragma unroll
        for (uint32_t u = 0; u < kVecPerLane; u++) {
            Store16(d.dst, off + (uint64_t(u) * kBlockThreads + tid) * 16, va[u]);
        }
    } else {
        for (uint32_t i = tid; i < nvec; i += kBlockThreads) {
            V4 v = Load16<MODE>(d.a, off + uint64_t(i) * 16);
            if (d.b != nullptr) {
                v = Combine16<T, OP>(v, Load16<MODE>(d.b, off + uint64_t(i) * 16));
            }
            Store16(d.dst, off + uint64_t(i) * 16, v);
        }
    }
}

template <typename T, int OP>
__device__ __forceinline__ void StepTileElem(const StepDesc &d, uint64_t off, uint32_t n)
{
    const uint32_t cnt = n / sizeof(T);
    for (uint32_t i = threadIdx.x; i < cnt; i += kBlockThreads) {
        const uint64_t at = off + uint64_t(i) * sizeof(T);
        T v = LoadElem<T>(d.a, at);
        if (d.b != nullptr) {
            v = Elem<T, OP>::Apply(v, LoadElem<T>(d.b, at));
        }
        StoreElem<T>(d.dst, at, v);
    }
}

// Fast loop of the step kernel over tiles [blockIdx.x, nwhole) with stride gridDim.x: every tile is
// whole and ACC_VEC16.  The descriptor of the next tile is looked up while the loads of the current
// one are in flight (the lookup is a chain of dependent scalar loads), and not at all while the next
// tile still belongs to the current step.  ORDINARY picks the store kind at compile time (a run-time
// choice per store is folded into one store by the compiler).
template <typename T, int OP, bool ORDINARY>
__device__ __forceinline__ void StepWholeTiles(const StepDesc *__restrict__ steps, uint32_t nsteps, uint32_t nwhole, uint32_t ntiles,
    bool reverse)
{
    const uint32_t tid = threadIdx.x;
    uint32_t tile = blockIdx.x;
    uint32_t idx = FindDesc(steps, nsteps, tile);
    StepDesc d = steps[idx];
    uint32_t dEnd = idx + 1 < nsteps ? steps[idx + 1].tile0 : ntiles;   // first tile past this step
    for (;;) {
        // whole tiles only, so walking a step backwards is a matter of the index
        const uint64_t off = uint64_t(reverse ? dEnd - 1 - tile : tile - d.tile0) * kTileBytes;
        const uint32_t next = tile + gridDim.x;
        const bool reduce = d.b != nullptr;
        V4 va[kVecPerLane], vb[kVecPerLane];
#pragma unroll
        for (uint32_t u = 0; u < kVecPerLane; u++) {
            va[u] = StepLoad(d.a, off + (uint64_t(u) * kBlockThreads + tid) * 16);
        }
        if (reduce) {
#pragma unroll
            for (uint32_t u = 0; u < kVecPerLane; u++) {
                vb[u] = StepLoad(d.b, off + (uint64_t(u) * kBlockThreads + tid) * 16);
            }
        }
        // keep the loads above where they are: without this the compiler sinks them below the lookup
        asm volatile("" ::: "memory");
        StepDesc dn = d;
        uint32_t dnEnd = dEnd;
        if (next < nwhole && next >= dEnd) {
            idx = FindDesc(steps, nsteps, next);
            dn = steps[idx];
            dnEnd = idx + 1 < nsteps ? steps[idx + 1].tile0 : ntiles;
        }
        if (reduce) {
#pragma unroll
            for (uint32_t u = 0; u < kVecPerLane; u++) {
                va[u] = Combine16<T, OP>(va[u], vb[u]);
            }
        }
#pragma unroll
        for (uint32_t u = 0; u < kVecPerLane; u++) {
            StepStore<ORDINARY>(d.dst, off + (uint64_t(u) * kBlockThreads + tid) * 16, va[u]);
        }
        if (next >= nwhole) {
            break;
        }
        tile = next;
        d = dn;
        dEnd = dnEnd;
    }
}

// Tiles [0, nwhole) belong to steps that are ACC_VEC16 and a whole number of tiles (the host puts
// those first in the table); tiles [nwhole, ntiles) are everything else: ragged ends, unaligned
// buffers.  The two get separate loops: with the slow paths in the same loop as the fast one, the
// compiler's wait-count bookkeeping (which joins all paths at the loop head) makes every iteration
// wait for the previous iteration's stores before it issues its loads.
template <typename T, int OP>
__global__ void __launch_bounds__(kBlockThreads) StepKernel(const StepDesc *__restrict__ steps, uint32_t nsteps, uint32_t nwhole,
    uint32_t ntiles, uint32_t flags)
{
    if (blockIdx.x < nwhole) {
        if (flags & kStepOrdinaryStores) {
            StepWholeTiles<T, OP, true>(steps, nsteps, nwhole, ntiles, (flags & kStepReverse) != 0);
        } else {
            StepWholeTiles<T, OP, false>(steps, nsteps, nwhole, ntiles, (flags & kStepReverse) != 0);
        }
    }
    for (uint32_t tile = nwhole + blockIdx.x; tile < ntiles; tile += gridDim.x) {
        const StepDesc d = steps[FindDesc(steps, nsteps, tile)];
        const uint64_t off = uint64_t(tile - d.tile0) * kTileBytes;
        const uint64_t left = d.bytes - off;
        const uint32_t n = left < kTileBytes ? uint32_t(left) : kTileBytes;
        if (d.mode == ACC_VEC16) {
            StepTileVec<T, OP, ACC_VEC16>(d, off, n);
        } else if (d.mode == ACC_VEC16_ANY) {
            StepTileVec<T, OP, ACC_VEC16_ANY>(d, off, n);
        } else {
            StepTileElem<T, OP>(d, off, n);
        }
    }
}

// ---- fused chain: read every source once, combine in schedule order, write every destination ----------
constexpr uint32_t kChainVec = 4;      // vectors per lane per pass
constexpr uint32_t kChainSrcBatch = 8; // sources whose loads are issued together

// Operand order changes the bits only where the combine is not commutative bit for bit:
// floating max / min (NaN and signed zero follow the selection rule).
template <typename T, int OP> struct OrderMatters { static constexpr bool value = false; };
template <int OP> struct OrderMatters<float, OP> { static constexpr bool value = (OP == ROP_MAX || OP == ROP_MIN); };
template <int OP> struct OrderMatters<double, OP> { static constexpr bool value = (OP == ROP_MAX || OP == ROP_MIN); };
template <int OP> struct OrderMatters<HalfBits, OP> { static constexpr bool value = (OP == ROP_MAX || OP == ROP_MIN); };
template <int OP> struct OrderMatters<Bf16Bits, OP> { static constexpr bool value = (OP == ROP_MAX || OP == ROP_MIN); };

template <uint32_t MODE, bool ORDINARY = false> __device__ __forceinline__ void StoreAny16(void *base, uint64_t pos, V4 v)
{
    if (MODE == ACC_VEC16) {
        if (ORDINARY) {
            *(GlobalV4 *)(static_cast<char *>(base) + pos) = v;
        } else {
            Store16(base, pos, v);
        }
    } else {
        V4U t = {v.x, v.y, v.z, v.w};
        __builtin_nontemporal_store(t, (GlobalV4U *)(static_cast<char *>(base) + pos));
    }
}

// One pass over kChainVec * 256 vectors starting at vector vecBase of the tile.
// FULL: every lane has all its vectors inside the tile (no per-lane guards).
// PARK: the results are not stored to the destinations but left in LDS, vector i of the tile at park[i] (the team
// kernels write them out later); dst is not used then.
// ONE_BATCH: the item has at most kChainSrcBatch sources (the caller has checked), so `src` is only ever indexed with
// constants: a caller that keeps the pointers in a local array then keeps them in registers from tile to tile.
template <typename T, int OP, uint32_t MODE, bool FULL, bool ORDINARY = false, bool PARK = false, bool ONE_BATCH = false>
__device__ __forceinline__ void ChainVecPass(const FusedDesc &d, const void *const *__restrict__ src,
    void *const *__restrict__ dst, uint64_t off, uint32_t vecBase, uint32_t nvec, LdsV4 *park = nullptr)
{
    const uint32_t tid = threadIdx.x;
    uint64_t pos[kChainVec];
    bool live[kChainVec];
#pragma unroll
    for (uint32_t u = 0; u < kChainVec; u++) {
        uint32_t i = vecBase + u * kBlockThreads + tid;
        live[u] = FULL || i < nvec;
        pos[u] = off + uint64_t(i) * 16;
    }
    V4 acc[kChainVec];
    const uint32_t nsrc = d.nsrc;
    const uint32_t batched = ONE_BATCH ? 1u : nsrc;
    for (uint32_t j = 0; j < batched; j += kChainSrcBatch) {
        V4 v[kChainSrcBatch][kChainVec];
#pragma unroll
        for (uint32_t jj = 0; jj < kChainSrcBatch; jj++) {
            if (j + jj < nsrc) {
                const void *s = src[j + jj];
#pragma unroll
                for (uint32_t u = 0; u < kChainVec; u++) {
                    if (live[u]) {
                        v[jj][u] = Load16<MODE>(s, pos[u]);
                    }
                }
            }
        }
#pragma unroll
        for (uint32_t jj = 0; jj < kChainSrcBatch; jj++) {
            if (j + jj < nsrc) {
                if (j + jj == 0) {
#pragma unroll
                    for (uint32_t u = 0; u < kChainVec; u++) {
                        acc[u] = v[0][u];
                    }
                } else {
                    const bool accLeft = OrderMatters<T, OP>::value && ((d.accLeftMask >> (j + jj)) & 1ull);
                    // the flag is the same for the whole wave: a branch, not both results and a select per element
                    if (accLeft) {
#pragma unroll
                        for (uint32_t u = 0; u < kChainVec; u++) {
                            if (live[u]) {
                                acc[u] = Combine16<T, OP>(acc[u], v[jj][u]);
                            }
                        }
                    } else {
#pragma unroll
                        for (uint32_t u = 0; u < kChainVec; u++) {
                            if (live[u]) {
                                acc[u] = Combine16<T, OP>(v[jj][u], acc[u]);
                            }
                        }
                    }
                }
            }
        }
    }
    if (PARK) {
#pragma unroll
        for (uint32_t u = 0; u < kChainVec; u++) {
            if (live[u]) {
                park[vecBase + u * kBlockThreads + tid] = acc[u];
            }
        }
        return;
    }
    const uint32_t ndst = d.ndst;
    for (uint32_t k = 0; k < ndst; k++) {
        void *o = dst[k];
#pragma unroll
        for (uint32_t u = 0; u < kChainVec; u++) {
            if (live[u]) {
                StoreAny16<MODE, ORDINARY>(o, pos[u], acc[u]);
            }
        }
    }
}

template <typename T, int OP>
__device__ __forceinline__ void ChainElem(const FusedDesc &d, const void *const *__restrict__ src,
    void *const *__restrict__ dst, uint64_t off, uint32_t n)
{
    const uint32_t cnt = n / sizeof(T);
    for (uint32_t i = threadIdx.x; i < cnt; i += kBlockThreads) {
        const uint64_t at = off + uint64_t(i) * sizeof(T);
        T acc = LoadElem<T>(src[0], at);
        for (uint32_t j = 1; j < d.nsrc; j++) {
            T v = LoadElem<T>(src[j], at);
            acc = ((d.accLeftMask >> j) & 1ull) ? Elem<T, OP>::Apply(acc, v) : Elem<T, OP>::Apply(v, acc);
        }
        for (uint32_t k = 0; k < d.ndst; k++) {
            StoreElem<T>(dst[k], at, acc);
        }
    }
}

template <typename T, int OP>
__global__ void __launch_bounds__(kBlockThreads) ChainKernel(const FusedDesc *__restrict__ items, uint32_t nitems,
    uint32_t ntiles, const void *const *__restrict__ srcPool, void *const *__restrict__ dstPool, uint32_t tilesPerItem)
{
    uint32_t tile = blockIdx.x;
    if (tile >= ntiles) {
        return;
    }
    // a workgroup keeps its item while its tiles stay inside it; the next item is looked up ahead of the current
    // tile's loads (see the copy kernel)
    FusedDesc d = items[ItemOfTile(items, nitems, tile, tilesPerItem)];
    uint32_t dEnd = d.tile0 + uint32_t((d.bytes + kTileBytes - 1) / kTileBytes);
    for (;;) {
        const uint32_t next = tile + gridDim.x;
        FusedDesc dn = d;
        uint32_t dnEnd = dEnd;
        if (next < ntiles && next >= dEnd) {
            dn = items[ItemOfTile(items, nitems, next, tilesPerItem)];
            dnEnd = dn.tile0 + uint32_t((dn.bytes + kTileBytes - 1) / kTileBytes);
        }
        const uint64_t off = uint64_t(tile - d.tile0) * kTileBytes;
        const uint64_t left = d.bytes - off;
        const uint32_t n = left < kTileBytes ? uint32_t(left) : kTileBytes;
        const void *const *src = srcPool + d.srcBase;
        void *const *dst = dstPool + d.dstBase;
        if (d.mode == ACC_ELEM) {
            ChainElem<T, OP>(d, src, dst, off, n);
        } else {
            const uint32_t nvec = n >> 4;
            constexpr uint32_t kPass = kChainVec * kBlockThreads;
            uint32_t base = 0;
            if (d.mode == ACC_VEC16) {
                // the store kind is a compile-time property of the pass (a per-store choice at run time
                // is merged by the compiler into one plain store)
                if (d.flags & kFusedOrdinaryStores) {
                    for (; base + kPass <= nvec; base += kPass) {
                        ChainVecPass<T, OP, ACC_VEC16, true, true>(d, src, dst, off, base, nvec);
                    }
                } else {
                    for (; base + kPass <= nvec; base += kPass) {
                        ChainVecPass<T, OP, ACC_VEC16, true, false>(d, src, dst, off, base, nvec);
                    }
                }
                if (base < nvec) {
                    ChainVecPass<T, OP, ACC_VEC16, false>(d, src, dst, off, base, nvec);
                }
            } else {
                for (; base + kPass <= nvec; base += kPass) {
                    ChainVecPass<T, OP, ACC_VEC16_ANY, true>(d, src, dst, off, base, nvec);
                }
                if (base < nvec) {
                    ChainVecPass<T, OP, ACC_VEC16_ANY, false>(d, src, dst, off, base, nvec);
                }
            }
        }
        if (next >= ntiles) {
            break;
        }
        tile = next;
        d = dn;
        dEnd = dnEnd;
    }
}

// ---- pure data movement: one source, m destinations ------------------------------------------------------
// The chain kernel's copy path with nothing else in the kernel: about 40 registers instead of 170+, so eight
// workgroups fit on a CU where the chain kernel fits two.  A copy keeps only 4 loads per lane in flight, and its
// rate comes from how many waves do that at once (measured, 1 GiB copy: 5.1 TB/s through the chain kernel,
// 6.3 TB/s for a plain copy kernel at full occupancy).
template <uint32_t MODE, bool FULL, bool ORDINARY = false, bool PARK = false>
__device__ __forceinline__ void CopyVecPass(const void *s, void *const *__restrict__ dst, uint32_t ndst, uint64_t off,
    uint32_t vecBase, uint32_t nvec, LdsV4 *park = nullptr)
{
    uint64_t pos[kChainVec];
    bool live[kChainVec];
    V4 v[kChainVec];
#pragma unroll
    for (uint32_t u = 0; u < kChainVec; u++) {
        const uint32_t i = vecBase + u * kBlockThreads + threadIdx.x;
        live[u] = FULL || i < nvec;
        pos[u] = off + uint64_t(i) * 16;
        if (live[u]) {
            v[u] = Load16<MODE>(s, pos[u]);
        }
    }
    if (PARK) {
#pragma unroll
        for (uint32_t u = 0; u < kChainVec; u++) {
            if (live[u]) {
                park[vecBase + u * kBlockThreads + threadIdx.x] = v[u];
            }
        }
        return;
    }
    for (uint32_t k = 0; k < ndst; k++) {
        void *o = dst[k];
#pragma unroll
        for (uint32_t u = 0; u < kChainVec; u++) {
            if (live[u]) {
                StoreAny16<MODE, ORDINARY>(o, pos[u], v[u]);
            }
        }
    }
}

// Same arguments and tables as the chain kernel; every item has exactly one source.  (A template only so that the
// definition may sit in this header; Variant is unused.)
template <int Variant>
__global__ void __launch_bounds__(kBlockThreads) CopyKernel(const FusedDesc *__restrict__ items, uint32_t nitems,
    uint32_t ntiles, const void *const *__restrict__ srcPool, void *const *__restrict__ dstPool, uint32_t tilesPerItem)
{
    uint32_t tile = blockIdx.x;
    if (tile >= ntiles) {
        return;
    }
    // The item of a tile costs a chain of dependent loads (table, item, pointer).  A workgroup that stays inside one
    // item from one tile to the next keeps what it has; when the next tile lies in another item, that item is looked
    // up before the current tile's data is loaded, so that the chain completes behind those loads.
    FusedDesc d = items[ItemOfTile(items, nitems, tile, tilesPerItem)];
    const void *s = srcPool[d.srcBase];
    uint32_t dEnd = d.tile0 + uint32_t((d.bytes + kTileBytes - 1) / kTileBytes);
    for (;;) {
        const uint32_t next = tile + gridDim.x;
        FusedDesc dn = d;
        const void *sn = s;
        uint32_t dnEnd = dEnd;
        if (next < ntiles && next >= dEnd) {
            dn = items[ItemOfTile(items, nitems, next, tilesPerItem)];
            sn = srcPool[dn.srcBase];
            dnEnd = dn.tile0 + uint32_t((dn.bytes + kTileBytes - 1) / kTileBytes);
        }
        const uint64_t off = uint64_t(tile - d.tile0) * kTileBytes;
        const uint64_t left = d.bytes - off;
        const uint32_t n = left < kTileBytes ? uint32_t(left) : kTileBytes;
        void *const *dst = dstPool + d.dstBase;
        if (d.mode == ACC_ELEM) {
            for (uint32_t i = threadIdx.x; i < n; i += kBlockThreads) {
                const uint8_t b = LoadElem<uint8_t>(s, off + i);
                for (uint32_t k = 0; k < d.ndst; k++) {
                    StoreElem<uint8_t>(dst[k], off + i, b);
                }
            }
        } else {
            const uint32_t nvec = n >> 4;
            constexpr uint32_t kPass = kChainVec * kBlockThreads;
            uint32_t base = 0;
            if (d.mode == ACC_VEC16) {
                if (d.flags & kFusedOrdinaryStores) {
                    for (; base + kPass <= nvec; base += kPass) {
                        CopyVecPass<ACC_VEC16, true, true>(s, dst, d.ndst, off, base, nvec);
                    }
                } else {
                    for (; base + kPass <= nvec; base += kPass) {
                        CopyVecPass<ACC_VEC16, true>(s, dst, d.ndst, off, base, nvec);
                    }
                }
                if (base < nvec) {
                    CopyVecPass<ACC_VEC16, false>(s, dst, d.ndst, off, base, nvec);
                }
            } else {
                for (; base + kPass <= nvec; base += kPass) {
                    CopyVecPass<ACC_VEC16_ANY, true>(s, dst, d.ndst, off, base, nvec);
                }
                if (base < nvec) {
                    CopyVecPass<ACC_VEC16_ANY, false>(s, dst, d.ndst, off, base, nvec);
                }
            }
        }
        if (next >= ntiles) {
            break;
        }
        tile = next;
        d = dn;
        s = sn;
        dEnd = dnEnd;
    }
}

// ---- small-segment gather: LDS staging ---------------------------------------------------------------------
// An all-to-all-v of many short segments (a few hundred bytes each, at any byte offset in the send and receive
// buffers) is all overhead in the tile kernels: a descriptor search per tile, a head / body / tail split per
// segment, unaligned accesses.  Here a wave takes a whole segment: it reads the aligned 16-byte granules that cover
// the source bytes into its share of LDS (coalesced, aligned loads; the bytes in front of and behind the segment that
// come along lie in the same granules as valid bytes), then every lane picks the 16 bytes of one aligned granule of
// the destination out of LDS at whatever offset they sit and stores them aligned; the two ragged ends go byte by
// byte.  Segments are dealt to waves round robin, no search.
// Stands where the reference's AIV kernel stages small all-to-all-v slices through its unified buffer
// (ALG/base/alg_aiv_template/aiv_all_to_all_v_910b.h:39-222); nothing of it is reused.
constexpr uint32_t kGatherLdsPerWave = kGatherMaxBytes + 32;

template <int Variant>
__global__ void __launch_bounds__(kBlockThreads) GatherKernel(const SegDesc *__restrict__ segs, uint32_t nsegs, uint32_t,
    const void *const *__restrict__, void *const *__restrict__, uint32_t)
{
    __shared__ __attribute__((aligned(16))) uint8_t lds[(kBlockThreads / 64) * kGatherLdsPerWave];
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    uint8_t *mine = lds + wave * kGatherLdsPerWave;
    const uint32_t wavesPerBlock = kBlockThreads / 64;
    for (uint32_t i = blockIdx.x * wavesPerBlock + wave; i < nsegs; i += gridDim.x * wavesPerBlock) {
        const SegDesc d = segs[i];
        const uint32_t n = uint32_t(d.bytes);
        if (n == 0) {
            continue;
        }
        const uintptr_t s = reinterpret_cast<uintptr_t>(d.src), t = reinterpret_cast<uintptr_t>(d.dst);
        const uintptr_t s0 = s & ~uintptr_t(15);
        const uint32_t delta = uint32_t(s - s0);                       // where the segment starts inside LDS
        const uint32_t nin = (delta + n + 15u) >> 4;                   // granules to read
        for (uint32_t v = lane; v < nin; v += 64) {
            const V4 x = __builtin_nontemporal_load((const GlobalV4 *)(s0 + uintptr_t(v) * 16));
            *(LdsV4 *)(mine + v * 16) = x;
        }
        // LDS operations of one wave complete in order; the compiler must keep that order too
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const uintptr_t t0 = (t + 15) & ~uintptr_t(15);               // first aligned granule inside the destination
        const uint32_t head = uint32_t(t0 - t) < n ? uint32_t(t0 - t) : n;
        const uint32_t body = (n - head) >> 4;                         // whole granules
        const uint32_t tail = n - head - body * 16;
        for (uint32_t v = lane; v < body; v += 64) {
            const LdsV4U *from = (const LdsV4U *)(mine + delta + head + v * 16);
            const V4U x = *from;
            __builtin_nontemporal_store(V4{x.x, x.y, x.z, x.w}, (GlobalV4 *)(t0 + uintptr_t(v) * 16));
        }
        if (lane < head) {
            StoreElem<uint8_t>(d.dst, lane, mine[delta + lane]);
        }
        if (lane < tail) {
            const uint32_t at = head + body * 16 + lane;
            StoreElem<uint8_t>(d.dst, at, mine[delta + at]);
        }
        // the next segment's loads into LDS must not overtake this segment's reads
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    }
}

// ---- fused perfect tree (halving-doubling): leaves pairwise bottom-up ----------------------------------
// v[i] = v[i] (+) v[i+w] for w = 1, 2, 4, ... is evaluated group by group: the first three levels
// inside groups of 8 consecutive leaves (8 loads per vector in flight, one result kept per group), the
// remaining levels over the group results.  Same association as the flat loop, a quarter of the
// registers; a lane works on kTreeVec vectors at a time so that 16 loads are outstanding per group
// (measured, 8-rank fp32 all-reduce of 32 MiB per rank: 124 us with one vector, 104 us with two).
constexpr uint32_t kTreeGroup = 8;
constexpr uint32_t kTreeMaxGroups = 4;   // up to 32 leaves

constexpr uint32_t kTreeVecPlain = 2;    // vectors per lane per pass
constexpr uint32_t kTreeVecTeam = 4;     // in the team kernels, which run one workgroup per CU: twice the loads in flight

// Evaluates the tree for kTreeVec vectors of one lane (positions pos[u], skipped where !live[u]).
// kTreeVec is kTreeVecPlain, or kTreeVecTeam when the results are parked (PARK).
// G = leaves per group: 8 when the tree has 8 or more leaves, else the leaf count itself (1, 2, 4),
// so that no group is ever partial and the loads of a group are issued back to back.
template <typename T, int OP, uint32_t MODE, bool FULL, uint32_t G, uint32_t kTreeVec>
__device__ __forceinline__ void TreeValue(const FusedDesc &d, const void *const *__restrict__ src,
    const uint64_t (&pos)[kTreeVec], const bool (&live)[kTreeVec], V4 (&x)[kTreeVec])
{
    const uint32_t ngroups = d.nleaf / G;   // 1, 2 or 4
    // Pending left operands of the upper levels (a binary counter over the groups seen so far).
    V4 l0[kTreeVec], l1[kTreeVec];
#pragma unroll
    for (uint32_t u = 0; u < kTreeVec; u++) {
        l0[u] = l1[u] = x[u] = V4{0, 0, 0, 0};
    }
    // Kept as a loop on purpose: unrolled, the compiler hoists every group's loads to the top and
    // the register count (and with it the number of resident waves) is back to the flat version's.
#pragma nounroll
    for (uint32_t gi = 0; gi < ngroups; gi++) {
        const void *const *gs = src + 2 * gi * G;
        V4 v[G][kTreeVec];
#pragma unroll
        for (uint32_t i = 0; i < G; i++) {
            const void *s = gs[2 * i];
#pragma unroll
            for (uint32_t u = 0; u < kTreeVec; u++) {
                if (FULL || live[u]) {
                    v[i][u] = Load16<MODE>(s, pos[u]);
                }
            }
        }
        // second sources of the leaves (folded rank pairs), four leaves at a time: all loads of a
        // batch first, then the combines
        constexpr uint32_t B = G >= 4 ? 4 : G;
#pragma unroll
        for (uint32_t b0 = 0; b0 < G; b0 += B) {
            V4 w[B][kTreeVec];
            bool has[B];
#pragma unroll
            for (uint32_t i = 0; i < B; i++) {
                const void *s = gs[2 * (b0 + i) + 1];
                has[i] = s != nullptr;
                if (has[i]) {
#pragma unroll
                    for (uint32_t u = 0; u < kTreeVec; u++) {
                        if (FULL || live[u]) {
                            w[i][u] = Load16<MODE>(s, pos[u]);
                        }
                    }
                }
            }
#pragma unroll
            for (uint32_t i = 0; i < B; i++) {
                if (has[i]) {
#pragma unroll
                    for (uint32_t u = 0; u < kTreeVec; u++) {
                        if (FULL || live[u]) {
                            v[b0 + i][u] = Combine16<T, OP>(v[b0 + i][u], w[i][u]);
                        }
                    }
                }
            }
        }
#pragma unroll
        for (uint32_t w = 1; w < G; w <<= 1) {
#pragma unroll
            for (uint32_t i = 0; i + w < G; i += 2 * w) {
#pragma unroll
                for (uint32_t u = 0; u < kTreeVec; u++) {
                    v[i][u] = Combine16<T, OP>(v[i][u], v[i + w][u]);
                }
            }
        }
#pragma unroll
        for (uint32_t u = 0; u < kTreeVec; u++) {
            x[u] = v[0][u];
        }
        if ((gi & 1u) == 0) {
#pragma unroll
            for (uint32_t u = 0; u < kTreeVec; u++) {
                l0[u] = x[u];
            }
        } else {
#pragma unroll
            for (uint32_t u = 0; u < kTreeVec; u++) {
                x[u] = Combine16<T, OP>(l0[u], x[u]);
            }
            if ((gi & 2u) == 0) {
#pragma unroll
                for (uint32_t u = 0; u < kTreeVec; u++) {
                    l1[u] = x[u];
                }
            } else {
#pragma unroll
                for (uint32_t u = 0; u < kTreeVec; u++) {
                    x[u] = Combine16<T, OP>(l1[u], x[u]);
                }
            }
        }
    }
}

// One pass over kTreeVec * 256 vectors starting at vector vecBase of the tile.
template <typename T, int OP, uint32_t MODE, bool FULL, uint32_t G, bool PARK = false>
__device__ __forceinline__ void TreeVecPass(const FusedDesc &d, const void *const *__restrict__ src,
    void *const *__restrict__ dst, uint64_t off, uint32_t vecBase, uint32_t nvec, LdsV4 *park = nullptr)
{
    constexpr uint32_t kTreeVec = PARK ? kTreeVecTeam : kTreeVecPlain;
    uint64_t pos[kTreeVec];
    bool live[kTreeVec];
#pragma unroll
    for (uint32_t u = 0; u < kTreeVec; u++) {
        uint32_t i = vecBase + u * kBlockThreads + threadIdx.x;
        live[u] = FULL || i < nvec;
        pos[u] = off + uint64_t(i) * 16;
    }
    V4 r[kTreeVec];
    TreeValue<T, OP, MODE, FULL, G, kTreeVec>(d, src, pos, live, r);
    if (PARK) {
#pragma unroll
        for (uint32_t u = 0; u < kTreeVec; u++) {
            if (live[u]) {
                park[vecBase + u * kBlockThreads + threadIdx.x] = r[u];
            }
        }
        return;
    }
    const uint32_t ndst = d.ndst;
    for (uint32_t k = 0; k < ndst; k++) {
        void *o = dst[k];
#pragma unroll
        for (uint32_t u = 0; u < kTreeVec; u++) {
            if (live[u]) {
                StoreAny16<MODE>(o, pos[u], r[u]);
            }
        }
    }
}

// All vector passes of one tile.
template <typename T, int OP, uint32_t G, bool PARK = false>
__device__ __forceinline__ void TreeTileVec(const FusedDesc &d, const void *const *__restrict__ src,
    void *const *__restrict__ dst, uint64_t off, uint32_t nvec, LdsV4 *park = nullptr)
{
    constexpr uint32_t kPass = (PARK ? kTreeVecTeam : kTreeVecPlain) * kBlockThreads;
    uint32_t base = 0;
    if (d.mode == ACC_VEC16) {
        for (; base + kPass <= nvec; base += kPass) {
            TreeVecPass<T, OP, ACC_VEC16, true, G, PARK>(d, src, dst, off, base, nvec, park);
        }
        if (base < nvec) {
            TreeVecPass<T, OP, ACC_VEC16, false, G, PARK>(d, src, dst, off, base, nvec, park);
        }
    } else {
        for (; base < nvec; base += kPass) {
            TreeVecPass<T, OP, ACC_VEC16_ANY, false, G, PARK>(d, src, dst, off, base, nvec, park);
        }
    }
}

// All vector passes of one tile, whatever the number of leaves.
template <typename T, int OP, bool PARK = false>
__device__ __forceinline__ void TreeTile(const FusedDesc &d, const void *const *__restrict__ src,
    void *const *__restrict__ dst, uint64_t off, uint32_t nvec, LdsV4 *park = nullptr)
{
    if (d.nleaf >= kTreeGroup) {
        TreeTileVec<T, OP, kTreeGroup, PARK>(d, src, dst, off, nvec, park);
    } else if (d.nleaf == 4) {
        TreeTileVec<T, OP, 4, PARK>(d, src, dst, off, nvec, park);
    } else if (d.nleaf == 2) {
        TreeTileVec<T, OP, 2, PARK>(d, src, dst, off, nvec, park);
    } else {
        TreeTileVec<T, OP, 1, PARK>(d, src, dst, off, nvec, park);
    }
}

template <typename T, int OP>
__device__ __forceinline__ void TreeElem(const FusedDesc &d, const void *const *__restrict__ src,
    void *const *__restrict__ dst, uint64_t off, uint32_t n)
{
    constexpr uint32_t kMax = kTreeGroup * kTreeMaxGroups;
    const uint32_t cnt = n / sizeof(T);
    for (uint32_t e = threadIdx.x; e < cnt; e += kBlockThreads) {
        const uint64_t at = off + uint64_t(e) * sizeof(T);
        T v[kMax];
#pragma unroll
        for (uint32_t i = 0; i < kMax; i++) {
            if (i < d.nleaf) {
                v[i] = LoadElem<T>(src[2 * i], at);
                const void *s = src[2 * i + 1];
                if (s != nullptr) {
                    v[i] = Elem<T, OP>::Apply(v[i], LoadElem<T>(s, at));
                }
            }
        }
#pragma unroll
        for (uint32_t w = 1; w < kMax; w <<= 1) {
            if (w < d.nleaf) {
#pragma unroll
                for (uint32_t i = 0; i + w < kMax; i += 2 * w) {
                    if (i + w < d.nleaf) {
                        v[i] = Elem<T, OP>::Apply(v[i], v[i + w]);
                    }
                }
            }
        }
        for (uint32_t k = 0; k < d.ndst; k++) {
            StoreElem<T>(dst[k], at, v[0]);
        }
    }
}

template <typename T, int OP>
__global__ void __launch_bounds__(kBlockThreads) TreeKernel(const FusedDesc *__restrict__ items, uint32_t nitems,
    uint32_t ntiles, const void *const *__restrict__ srcPool, void *const *__restrict__ dstPool, uint32_t tilesPerItem)
{
    for (uint32_t tile = blockIdx.x; tile < ntiles; tile += gridDim.x) {
        const FusedDesc d = items[ItemOfTile(items, nitems, tile, tilesPerItem)];
        const uint64_t off = uint64_t(tile - d.tile0) * kTileBytes;
        const uint64_t left = d.bytes - off;
        const uint32_t n = left < kTileBytes ? uint32_t(left) : kTileBytes;
        const void *const *src = srcPool + d.srcBase;
        void *const *dst = dstPool + d.dstBase;
        if (d.mode == ACC_ELEM) {
            TreeElem<T, OP>(d, src, dst, off, n);
        } else {
            TreeTile<T, OP>(d, src, dst, off, n >> 4);
        }
    }
}

// ---- fused general expression: a stack machine over registers -----------------------------------------
// Handles what is neither a chain nor a perfect tree (a ring or halving-doubling schedule whose
// operands are themselves mesh chains, for one).  The item's sources come in evaluation order; after
// source j the two topmost values are folded ops[j] & 7 times, bit 8 + i saying which of the two is
// the left operand in fold i.  The op words of a launch follow its item table in memory.
// The stack lives in registers: its depth is a wave-uniform number, so every access goes through a
// switch with constant indices.  Sources are loaded in batches like the chain kernel's.
// Two shapes: expressions that need at most 4 values (a chain of chains, a 4-leaf tree of chains) run
// with 4 vectors per lane like the chain kernel, deeper ones (up to 8 values) with 2.
constexpr uint32_t kStackVecShallow = 4;
constexpr uint32_t kStackVecDeep = 2;
constexpr uint32_t kStackShallowDepth = 4;
constexpr uint32_t kStackSrcBatch = 8;
// The plain kernel issues the loads of 4 sources together: with 8 it needs every register a wave can have, one
// workgroup fits a CU and nothing hides the table look-ups between its tiles (two-level reduce-scatter of 8 x 256 MiB
// 426 -> 417 us, reduce 434 -> 415 us, all-reduce of 8 x 16 MiB 52 -> 47 us).  The team form, one workgroup per CU by
// its LDS, keeps 8.
constexpr uint32_t kStackPlainBatch = 4;

template <uint32_t U> struct StackVal {
    V4 x[U];
};

// The values below the top one are separate variables, not an array or a struct: a switch over
// parts of one object is merged by the compiler into a single access at a computed offset, which
// moves the object to private memory.  DEEP is a compile-time constant of the enclosing function;
// without it only b0..b2 are ever touched and the others cost no registers.
#define HCCL_STACK_PUT(i, v)              \
    if (DEEP) {                           \
        switch (i) {                      \
            case 0: b0 = (v); break;      \
            case 1: b1 = (v); break;      \
            case 2: b2 = (v); break;      \
            case 3: b3 = (v); break;      \
            case 4: b4 = (v); break;      \
            case 5: b5 = (v); break;      \
            default: b6 = (v); break;     \
        }                                 \
    } else {                              \
        switch (i) {                      \
            case 0: b0 = (v); break;      \
            case 1: b1 = (v); break;      \
            default: b2 = (v); break;     \
        }                                 \
    }
#define HCCL_STACK_GET(i, v)              \
    if (DEEP) {                           \
        switch (i) {                      \
            case 0: (v) = b0; break;      \
            case 1: (v) = b1; break;      \
            case 2: (v) = b2; break;      \
            case 3: (v) = b3; break;      \
            case 4: (v) = b4; break;      \
            case 5: (v) = b5; break;      \
            default: (v) = b6; break;     \
        }                                 \
    } else {                              \
        switch (i) {                      \
            case 0: (v) = b0; break;      \
            case 1: (v) = b1; break;      \
            default: (v) = b2; break;     \
        }                                 \
    }

template <typename T, int OP, uint32_t MODE, bool FULL, bool DEEP, bool PARK = false, uint32_t BATCH = kStackSrcBatch>
__device__ __forceinline__ void StackVecPass(const FusedDesc &d, const void *const *__restrict__ src,
    const uint32_t *__restrict__ ops, void *const *__restrict__ dst, uint64_t off, uint32_t vecBase, uint32_t nvec,
    LdsV4 *park = nullptr)
{
    constexpr uint32_t U = DEEP ? kStackVecDeep : kStackVecShallow;
    uint64_t pos[U];
    bool live[U];
#pragma unroll
    for (uint32_t u = 0; u < U; u++) {
        uint32_t i = vecBase + u * kBlockThreads + threadIdx.x;
        live[u] = FULL || i < nvec;
        pos[u] = off + uint64_t(i) * 16;
    }
    StackVal<U> top;
#pragma unroll
    for (uint32_t u = 0; u < U; u++) {
        top.x[u] = V4{0, 0, 0, 0};
    }
    StackVal<U> b0 = top, b1 = top, b2 = top, b3 = top, b4 = top, b5 = top, b6 = top;
    uint32_t depth = 0;                  // values on the stack, the top one included
    const uint32_t nsrc = d.nsrc;
    for (uint32_t j = 0; j < nsrc; j += BATCH) {
        StackVal<U> v[BATCH];
#pragma unroll
        for (uint32_t jj = 0; jj < BATCH; jj++) {
            if (j + jj < nsrc) {
                const void *s = src[j + jj];
#pragma unroll
                for (uint32_t u = 0; u < U; u++) {
                    if (live[u]) {
                        v[jj].x[u] = Load16<MODE>(s, pos[u]);
                    }
                }
            }
        }
#pragma unroll
        for (uint32_t jj = 0; jj < BATCH; jj++) {
            if (j + jj < nsrc) {
                const uint32_t op = ops[j + jj];
                if (depth > 0) {
                    HCCL_STACK_PUT(depth - 1, top)
                }
                top = v[jj];
                depth++;
                const uint32_t nfold = op & 7u;
#pragma nounroll
                for (uint32_t f = 0; f < nfold && depth >= 2; f++) {
                    StackVal<U> under;
                    HCCL_STACK_GET(depth - 2, under)
                    const bool underLeft = !OrderMatters<T, OP>::value || ((op >> (8 + f)) & 1u);
                    if (underLeft) {           // the same for the whole wave
#pragma unroll
                        for (uint32_t u = 0; u < U; u++) {
                            if (live[u]) {
                                top.x[u] = Combine16<T, OP>(under.x[u], top.x[u]);
                            }
                        }
                    } else {
#pragma unroll
                        for (uint32_t u = 0; u < U; u++) {
                            if (live[u]) {
                                top.x[u] = Combine16<T, OP>(top.x[u], under.x[u]);
                            }
                        }
                    }
                    depth--;
                }
            }
        }
    }
    if (PARK) {
#pragma unroll
        for (uint32_t u = 0; u < U; u++) {
            if (live[u]) {
                park[vecBase + u * kBlockThreads + threadIdx.x] = top.x[u];
            }
        }
        return;
    }
    const uint32_t ndst = d.ndst;
    for (uint32_t k = 0; k < ndst; k++) {
        void *o = dst[k];
#pragma unroll
        for (uint32_t u = 0; u < U; u++) {
            if (live[u]) {
                StoreAny16<MODE>(o, pos[u], top.x[u]);
            }
        }
    }
}

// Heads, tails and unaligned buffers: the same machine element by element.
template <typename T, int OP>
__device__ __forceinline__ void StackElem(const FusedDesc &d, const void *const *__restrict__ src,
    const uint32_t *__restrict__ ops, void *const *__restrict__ dst, uint64_t off, uint32_t n)
{
    const uint32_t cnt = n / sizeof(T);
    for (uint32_t e = threadIdx.x; e < cnt; e += kBlockThreads) {
        const uint64_t at = off + uint64_t(e) * sizeof(T);
        constexpr bool DEEP = true;
        T top = T();
        T b0 = top, b1 = top, b2 = top, b3 = top, b4 = top, b5 = top, b6 = top;
        uint32_t depth = 0;
        for (uint32_t j = 0; j < d.nsrc; j++) {
            const uint32_t op = ops[j];
            if (depth > 0) {
                HCCL_STACK_PUT(depth - 1, top)
            }
            top = LoadElem<T>(src[j], at);
            depth++;
            const uint32_t nfold = op & 7u;
            for (uint32_t f = 0; f < nfold && depth >= 2; f++) {
                T under;
                HCCL_STACK_GET(depth - 2, under)
                top = ((op >> (8 + f)) & 1u) ? Elem<T, OP>::Apply(under, top) : Elem<T, OP>::Apply(top, under);
                depth--;
            }
        }
        for (uint32_t k = 0; k < d.ndst; k++) {
            StoreElem<T>(dst[k], at, top);
        }
    }
}

// All vector passes of one tile.
template <typename T, int OP, bool PARK = false, uint32_t BATCH = kStackSrcBatch>
__device__ __forceinline__ void StackTile(const FusedDesc &d, const void *const *__restrict__ src,
    const uint32_t *__restrict__ ops, void *const *__restrict__ dst, uint64_t off, uint32_t nvec, LdsV4 *park = nullptr)
{
    constexpr uint32_t kPassShallow = kStackVecShallow * kBlockThreads, kPassDeep = kStackVecDeep * kBlockThreads;
    uint32_t base = 0;
    if (d.mode == ACC_VEC16) {
        // d.nleaf: the stack depth the item needs
        if (d.nleaf <= kStackShallowDepth) {
            for (; base + kPassShallow <= nvec; base += kPassShallow) {
                StackVecPass<T, OP, ACC_VEC16, true, false, PARK, BATCH>(d, src, ops, dst, off, base, nvec, park);
            }
        }
        for (; base + kPassDeep <= nvec; base += kPassDeep) {
            StackVecPass<T, OP, ACC_VEC16, true, true, PARK, BATCH>(d, src, ops, dst, off, base, nvec, park);
        }
        if (base < nvec) {
            StackVecPass<T, OP, ACC_VEC16, false, true, PARK, BATCH>(d, src, ops, dst, off, base, nvec, park);
        }
    } else {
        for (; base < nvec; base += kPassDeep) {
            StackVecPass<T, OP, ACC_VEC16_ANY, false, true, PARK, BATCH>(d, src, ops, dst, off, base, nvec, park);
        }
    }
}

template <typename T, int OP>
__global__ void __launch_bounds__(kBlockThreads) StackKernel(const FusedDesc *__restrict__ items, uint32_t nitems,
    uint32_t ntiles, const void *const *__restrict__ srcPool, void *const *__restrict__ dstPool, uint32_t tilesPerItem)
{
    const uint32_t *opPool = reinterpret_cast<const uint32_t *>(items + nitems);
    for (uint32_t tile = blockIdx.x; tile < ntiles; tile += gridDim.x) {
        const FusedDesc d = items[ItemOfTile(items, nitems, tile, tilesPerItem)];
        const uint64_t off = uint64_t(tile - d.tile0) * kTileBytes;
        const uint64_t left = d.bytes - off;
        const uint32_t n = left < kTileBytes ? uint32_t(left) : kTileBytes;
        const void *const *src = srcPool + d.srcBase;
        const uint32_t *ops = opPool + d.srcBase;
        void *const *dst = dstPool + d.dstBase;
        if (d.mode == ACC_ELEM) {
            StackElem<T, OP>(d, src, ops, dst, off, n);
        } else {
            StackTile<T, OP, false, kStackPlainBatch>(d, src, ops, dst, off, n >> 4);
        }
    }
}

}  // namespace hcclamd
