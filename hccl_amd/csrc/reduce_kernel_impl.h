// Fused N-rank reduce for gfx950 (MI355X).
//
// One launch performs the local-reduce work of every rank of a loopback world: each lane owns a
// 16-byte vector position, pulls that position from the N rank buffers with 128-bit loads, combines
// them in registers in the order a fold program dictates, and writes the result once per
// destination.  The path is bound by HBM bandwidth (N reads + M writes of the element range, no
// re-reads, no staging passes), so there is no MFMA; LDS only holds the 320-byte program and, for
// tree-shaped orders, the accumulators of enclosing levels.
//
// Operand roles follow the reference's pairwise step  dst[i] = src[i] (+) dst[i]
// (alg_data_trans_wrapper.cc:1319-1358):
//   SUM   src + dst                 integers wrap
//   PROD  src * dst                 integers wrap (computed unsigned)
//   MAX   (src < dst) ? dst : src   ties / unordered keep src
//   MIN   (dst < src) ? dst : src   ties / unordered keep src
// fp16 / bf16 SUM accumulate in fp32 and round to nearest even once at the end; fp16 PROD rounds
// after every step like the reference's host path (:1237-1257); fp16 / bf16 MAX and MIN compare the
// values and carry the original 16-bit pattern.
#pragma once

#include <hip/hip_runtime.h>

#include "dataplane.h"

namespace hccl_amd {
namespace detail {

constexpr int kSum = 0, kProd = 1, kMax = 2, kMin = 3;
constexpr int kThreads = kMaxReduceThreads;   // upper bound; the launch picks args.threads

// ---------------------------------------------------------------------------------------------
// Element semantics.  S = storage type, A = accumulator type.
// ---------------------------------------------------------------------------------------------
template <typename T, typename UT, int OP>
struct IntOps {
    using S = T;
    using A = T;
    static __device__ __forceinline__ A Widen(S x) { return x; }
    static __device__ __forceinline__ S Narrow(A a) { return a; }
    static __device__ __forceinline__ A Fold(A src, A dst)
    {
        if constexpr (OP == kSum) {
            return static_cast<T>(static_cast<UT>(static_cast<UT>(src) + static_cast<UT>(dst)));
        } else if constexpr (OP == kProd) {
            return static_cast<T>(static_cast<UT>(static_cast<UT>(src) * static_cast<UT>(dst)));
        } else if constexpr (OP == kMax) {
            return (src < dst) ? dst : src;
        } else {
            return (dst < src) ? dst : src;
        }
    }
};

template <typename T, int OP>
struct FpOps {
    using S = T;
    using A = T;
    static __device__ __forceinline__ A Widen(S x) { return x; }
    static __device__ __forceinline__ S Narrow(A a) { return a; }
    static __device__ __forceinline__ A Fold(A src, A dst)
    {
        if constexpr (OP == kSum) {
            return src + dst;
        } else if constexpr (OP == kProd) {
            return src * dst;
        } else if constexpr (OP == kMax) {
            return (src < dst) ? dst : src;
        } else {
            return (dst < src) ? dst : src;
        }
    }
};

__device__ __forceinline__ float HalfBitsToFloat(uint16_t h) { return static_cast<float>(__builtin_bit_cast(_Float16, h)); }
__device__ __forceinline__ uint16_t FloatToHalfBits(float f) { return __builtin_bit_cast(uint16_t, static_cast<_Float16>(f)); }
__device__ __forceinline__ float Bf16BitsToFloat(uint16_t h) { return __builtin_bit_cast(float, static_cast<uint32_t>(h) << 16); }
__device__ __forceinline__ uint16_t FloatToBf16Bits(float f)
{
    uint32_t u = __builtin_bit_cast(uint32_t, f);
    uint32_t rounded = (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
    uint32_t hi = u >> 16;
    uint32_t quiet = (hi & 0x7Fu) ? hi : (hi | 1u);   // NaN stays NaN, payload bits kept
    bool isNan = (u & 0x7FFFFFFFu) > 0x7F800000u;
    return static_cast<uint16_t>(isNan ? quiet : rounded);
}

// fp16 / bf16 SUM: fp32 accumulator, one rounding at the end.
template <bool IS_BF16>
struct HalfSumOps {
    using S = uint16_t;
    using A = float;
    static __device__ __forceinline__ A Widen(S x) { return IS_BF16 ? Bf16BitsToFloat(x) : HalfBitsToFloat(x); }
    static __device__ __forceinline__ S Narrow(A a) { return IS_BF16 ? FloatToBf16Bits(a) : FloatToHalfBits(a); }
    static __device__ __forceinline__ A Fold(A src, A dst) { return src + dst; }
};

// fp16 PROD: the product of two fp16 values is exact in fp32, so rounding it to fp16 after every step
// is the IEEE fp16 multiply.
struct HalfProdOps {
    using S = uint16_t;
    using A = _Float16;
    static __device__ __forceinline__ A Widen(S x) { return __builtin_bit_cast(_Float16, x); }
    static __device__ __forceinline__ S Narrow(A a) { return __builtin_bit_cast(uint16_t, a); }
    static __device__ __forceinline__ A Fold(A src, A dst)
    {
        return static_cast<_Float16>(static_cast<float>(src) * static_cast<float>(dst));
    }
};

// fp16 / bf16 MAX, MIN: pure selection, the bit pattern of the chosen operand survives.
template <bool IS_BF16, int OP>
struct HalfSelectOps {
    using S = uint16_t;
    using A = uint16_t;
    static __device__ __forceinline__ A Widen(S x) { return x; }
    static __device__ __forceinline__ S Narrow(A a) { return a; }
    static __device__ __forceinline__ A Fold(A src, A dst)
    {
        float s = IS_BF16 ? Bf16BitsToFloat(src) : HalfBitsToFloat(src);
        float d = IS_BF16 ? Bf16BitsToFloat(dst) : HalfBitsToFloat(dst);
        if constexpr (OP == kMax) {
            return (s < d) ? dst : src;
        } else {
            return (d < s) ? dst : src;
        }
    }
};

// ---------------------------------------------------------------------------------------------
// Packs: W storage elements that travel as one memory transaction.
// ---------------------------------------------------------------------------------------------
typedef uint32_t U32x4 __attribute__((ext_vector_type(4)));

template <typename S, int W>
struct alignas(sizeof(S) * W >= 16 ? 16 : sizeof(S) * W) Pack {
    S e[W];
};

// Every buffer the kernel touches is global memory.  Saying so keeps the accesses off the flat path:
// a flat load also counts as an LDS operation, and waiting for the next LDS read (a leaf pointer)
// would then wait for every load issued before it.
#define HCCL_AMD_GLOBAL __attribute__((address_space(1)))

template <typename S, int W>
__device__ __forceinline__ Pack<S, W> LoadPack(const void* base, uint64_t elemOff)
{
    const S* p = static_cast<const S*>(base) + elemOff;
    if constexpr (sizeof(S) * W == 16) {
        U32x4 raw = __builtin_nontemporal_load((const HCCL_AMD_GLOBAL U32x4*)p);
        return __builtin_bit_cast(Pack<S, W>, raw);
    } else {
        Pack<S, W> r;
        r.e[0] = __builtin_nontemporal_load((const HCCL_AMD_GLOBAL S*)p);
        return r;
    }
}

template <typename S, int W>
__device__ __forceinline__ void StorePack(void* base, uint64_t elemOff, const Pack<S, W>& v, bool writeThrough)
{
    S* p = static_cast<S*>(base) + elemOff;
    if constexpr (sizeof(S) * W == 16) {
        if (writeThrough) {
            StoreStream16(p, __builtin_bit_cast(StreamVec, v));
        } else {
            __builtin_nontemporal_store(__builtin_bit_cast(U32x4, v), (HCCL_AMD_GLOBAL U32x4*)p);
        }
    } else {
        __builtin_nontemporal_store(v.e[0], (HCCL_AMD_GLOBAL S*)p);
    }
}

__device__ __forceinline__ uint32_t Uniform(uint32_t v) { return __builtin_amdgcn_readfirstlane(v); }

// ---------------------------------------------------------------------------------------------
// Program interpreter.  Control flow depends only on the program, so it is uniform across the
// wavefront.  One accumulator lives in registers; when a nested level opens, the enclosing level's
// accumulator waits in an LDS stack laid out word-major ([level][word][thread], so a wavefront's
// accesses hit 64 consecutive banks) and is popped when the level closes.
// ---------------------------------------------------------------------------------------------
template <class E, int W>
struct AccPack {
    typename E::A a[W];
};

template <class E, int W>
struct AccWords {
    static constexpr int kCount = (sizeof(AccPack<E, W>) + 3) / 4;
    uint32_t w[kCount];
};

template <class E, int W>
__device__ __forceinline__ void PushAcc(uint32_t* stack, uint32_t threads, uint32_t level, const AccPack<E, W>& acc)
{
    AccWords<E, W> words = {};
    __builtin_memcpy(&words, &acc, sizeof(acc));
#pragma unroll
    for (int i = 0; i < AccWords<E, W>::kCount; ++i) {
        stack[(level * AccWords<E, W>::kCount + i) * threads + threadIdx.x] = words.w[i];
    }
}

template <class E, int W>
__device__ __forceinline__ void PopAcc(const uint32_t* stack, uint32_t threads, uint32_t level, AccPack<E, W>& acc)
{
    AccWords<E, W> words;
#pragma unroll
    for (int i = 0; i < AccWords<E, W>::kCount; ++i) {
        words.w[i] = stack[(level * AccWords<E, W>::kCount + i) * threads + threadIdx.x];
    }
    __builtin_memcpy(&acc, &words, sizeof(acc));
}

__device__ __forceinline__ uint64_t Uniform64(uint64_t v)
{
    const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v));
    const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v >> 32));
    return (static_cast<uint64_t>(hi) << 32) | lo;
}

// Per-block view of the program: leaf i is read at leafPtr[i] (the rank's buffer already advanced to
// this sub-segment) and carries ctl[i] (see kCtlOpen).
struct BlockProgram {
    uint64_t leafPtr[kMaxRanks];
    uint8_t ctl[kMaxRanks];
    uint32_t nLeaves;
};

// Leaves whose loads are issued together: sixteen for 4- and 8-byte elements, eight for the narrower ones
// (their unpacked accumulators need the registers).
template <typename S, int W>
__device__ constexpr int LoadBatch()
{
    return (sizeof(S) >= 4 && W > 1) ? 16 : 8;
}

// Makes eight loaded vectors opaque to the optimiser at this point of the instruction stream.
template <typename S, int W>
__device__ __forceinline__ void IssueFence8(Pack<S, W>* v)
{
    U32x4 r0 = __builtin_bit_cast(U32x4, v[0]), r1 = __builtin_bit_cast(U32x4, v[1]);
    U32x4 r2 = __builtin_bit_cast(U32x4, v[2]), r3 = __builtin_bit_cast(U32x4, v[3]);
    U32x4 r4 = __builtin_bit_cast(U32x4, v[4]), r5 = __builtin_bit_cast(U32x4, v[5]);
    U32x4 r6 = __builtin_bit_cast(U32x4, v[6]), r7 = __builtin_bit_cast(U32x4, v[7]);
    asm volatile("" : "+v"(r0), "+v"(r1), "+v"(r2), "+v"(r3), "+v"(r4), "+v"(r5), "+v"(r6), "+v"(r7));
    v[0] = __builtin_bit_cast(Pack<S, W>, r0);
    v[1] = __builtin_bit_cast(Pack<S, W>, r1);
    v[2] = __builtin_bit_cast(Pack<S, W>, r2);
    v[3] = __builtin_bit_cast(Pack<S, W>, r3);
    v[4] = __builtin_bit_cast(Pack<S, W>, r4);
    v[5] = __builtin_bit_cast(Pack<S, W>, r5);
    v[6] = __builtin_bit_cast(Pack<S, W>, r6);
    v[7] = __builtin_bit_cast(Pack<S, W>, r7);
}

// Evaluates the whole tree for the W elements at element offset `e` of the sub-segment.  Leaves are
// taken a batch at a time: their loads are all issued before the first fold, whatever the tree shape.
template <class E, int W>
__device__ __forceinline__ void ReduceOne(const BlockProgram& bp, uint32_t* stack, const ReduceArgs& args,
                                          uint64_t e, uint64_t dstOff, uint32_t group)
{
    using S = typename E::S;
    AccPack<E, W> acc;
    uint32_t level = 0;
    bool init = true;   // the next leaf starts a level instead of being folded into it
    const uint32_t nLeaves = bp.nLeaves;
    constexpr int kBatch = LoadBatch<S, W>();
    for (uint32_t b = 0; b < nLeaves; b += kBatch) {
        Pack<S, W> v[kBatch];
#pragma unroll
        for (int i = 0; i < kBatch; ++i) {
            if (b + i < nLeaves) {
                const void* base = reinterpret_cast<const void*>(Uniform64(bp.leafPtr[b + i]));
                v[i] = LoadPack<S, W>(base, e);
            }
        }
        if constexpr (sizeof(S) * W == 16) {
            // Nothing may consume a loaded vector before the whole batch has been issued: without this the
            // compiler sinks the first unpacking instruction of each operand next to its load and waits there.
#pragma unroll
            for (int i = 0; i < kBatch; i += 8) {
                IssueFence8<S, W>(v + i);
            }
        }
#pragma unroll
        for (int i = 0; i < kBatch; ++i) {
            if (b + i < nLeaves) {
                const uint32_t ctl = Uniform(bp.ctl[b + i]);
                if (ctl & kCtlOpen) {
                    PushAcc<E, W>(stack, args.threads, level, acc);
                    ++level;
                    init = true;
                }
                if (init) {
#pragma unroll
                    for (int w = 0; w < W; ++w) {
                        acc.a[w] = E::Widen(v[i].e[w]);
                    }
                    init = false;
                } else {
#pragma unroll
                    for (int w = 0; w < W; ++w) {
                        acc.a[w] = E::Fold(E::Widen(v[i].e[w]), acc.a[w]);
                    }
                }
                for (uint32_t closes = ctl & 0x7Fu; closes != 0; --closes) {
                    AccPack<E, W> outer;
                    --level;
                    PopAcc<E, W>(stack, args.threads, level, outer);
#pragma unroll
                    for (int w = 0; w < W; ++w) {
                        acc.a[w] = E::Fold(acc.a[w], outer.a[w]);   // nested value is src, enclosing level is dst
                    }
                }
            }
        }
    }
    Pack<S, W> out;
#pragma unroll
    for (int w = 0; w < W; ++w) {
        out.e[w] = E::Narrow(acc.a[w]);
    }
    if (args.dstOwn) {
        StorePack<S, W>(args.dst[group], dstOff + e, out, args.writeThrough != 0);
    } else {
        for (uint32_t d = 0; d < args.nDst; ++d) {
            StorePack<S, W>(args.dst[d], dstOff + e, out, args.writeThrough != 0);
        }
    }
}

// Dynamic LDS: the accumulator stack, (plan depth - 1) * accumulator bytes * args.threads.
template <class E>
__global__ __launch_bounds__(kThreads) void ReduceKernel(const ReduceArgs args)
{
    using S = typename E::S;
    constexpr int W = 16 / sizeof(S);
    __shared__ BlockProgram bp;
    extern __shared__ uint32_t accStack[];

    const uint32_t sub = blockIdx.x / args.blocksPerSub;
    const uint32_t blk = blockIdx.x - sub * args.blocksPerSub;
    const uint32_t g = sub / args.nSub;
    const uint32_t c = sub - g * args.nSub;

    uint64_t gLen;
    uint64_t gSrc;
    if (args.varGroups) {
        gLen = args.groupLenV[g];
        gSrc = args.groupOffV[g];
    } else {
        const uint64_t gBeg = static_cast<uint64_t>(g) * args.groupLen;
        if (gBeg >= args.total) {
            return;
        }
        gLen = (args.total - gBeg < args.groupLen) ? args.total - gBeg : args.groupLen;
        gSrc = static_cast<uint64_t>(g) * args.srcGroupStride;
    }
    const uint64_t sBeg = static_cast<uint64_t>(c) * args.subLen;
    uint64_t sEnd = (c == args.nSub - 1) ? gLen : sBeg + args.subLen;
    sEnd = sEnd < gLen ? sEnd : gLen;
    if (sBeg >= sEnd) {
        return;
    }
    const uint64_t len = sEnd - sBeg;
    const uint64_t srcOff = gSrc + sBeg;
    const uint64_t dstOff = args.dstOwn ? sBeg : static_cast<uint64_t>(g) * args.dstGroupStride + sBeg;

    // Resolve the program once per block: leaf -> address of this sub-segment in that rank's buffer.
    const uint8_t* prog = args.prog + static_cast<uint64_t>(g * args.progGroupStride + c * args.progSubStride) * kDevProgBytes;
    const uint32_t nLeaves = prog[0];
    if (threadIdx.x < nLeaves) {
        const uint32_t rank = prog[kDevProgRankOff + threadIdx.x];
        bp.leafPtr[threadIdx.x] = reinterpret_cast<uint64_t>(args.src[rank]) + srcOff * sizeof(S);
        bp.ctl[threadIdx.x] = prog[kDevProgCtlOff + threadIdx.x];
    }
    if (threadIdx.x == 0) {
        bp.nLeaves = nLeaves;
    }
    __syncthreads();

    const uint64_t stride = static_cast<uint64_t>(args.blocksPerSub) * args.threads;
    const uint64_t first = static_cast<uint64_t>(blk) * args.threads + threadIdx.x;

    // When vecOk, every source and destination address of this sub-segment has the same offset from a
    // 16-byte boundary: `head` elements bring them all onto it, a 128-bit body follows, and fewer than
    // W elements remain.  Otherwise everything goes element by element.  The body's vectors are dealt
    // to the lanes shifted by `lead`, so that lane 0 of every wavefront starts a 128-byte line of the
    // first source (a wavefront whose 1 KiB straddles nine lines fetches two of them twice).
    uint64_t head = len;
    uint64_t nVec = 0;
    uint32_t lead = 0;
    // A group that starts at an odd offset into the sources is not congruent with its destination.
    if (args.vecOk && (!args.varGroups || ((gSrc * sizeof(S)) & 15u) == 0)) {
        const uint64_t addr = reinterpret_cast<uint64_t>(args.src[0]) + srcOff * sizeof(S);
        const uint32_t mis = static_cast<uint32_t>(addr & 15u);
        head = mis ? (16u - mis) / sizeof(S) : 0;
        head = head < len ? head : len;
        nVec = (len - head) / W;
        lead = static_cast<uint32_t>(((addr + head * sizeof(S)) >> 4) & 7u);
    }
    for (uint64_t u = first; u < nVec + lead; u += stride) {
        if (u >= lead) {
            ReduceOne<E, W>(bp, accStack, args, head + (u - lead) * W, dstOff, g);
        }
    }
    const uint64_t bodyEnd = head + nVec * W;
    const uint64_t nScalar = head + (len - bodyEnd);
    for (uint64_t i = first; i < nScalar; i += stride) {
        const uint64_t e = i < head ? i : i - head + bodyEnd;
        ReduceOne<E, 1>(bp, accStack, args, e, dstOff, g);
    }
}

using ReduceKernelFn = void (*)(const ReduceArgs);

}  // namespace detail

// One translation unit per data type defines its selector (nullptr = combination not offered).
detail::ReduceKernelFn SelectReduceI8(int op);
detail::ReduceKernelFn SelectReduceI16(int op);
detail::ReduceKernelFn SelectReduceI32(int op);
detail::ReduceKernelFn SelectReduceI64(int op);
detail::ReduceKernelFn SelectReduceU64(int op);
detail::ReduceKernelFn SelectReduceF16(int op);
detail::ReduceKernelFn SelectReduceBf16(int op);
detail::ReduceKernelFn SelectReduceF32(int op);
detail::ReduceKernelFn SelectReduceF64(int op);

#define HCCL_AMD_DEFINE_SELECT4(NAME, SUM_T, PROD_T, MAX_T, MIN_T)                 \
    detail::ReduceKernelFn NAME(int op)                                           \
    {                                                                             \
        switch (op) {                                                             \
            case detail::kSum: return detail::ReduceKernel<SUM_T>;                \
            case detail::kProd: return detail::ReduceKernel<PROD_T>;              \
            case detail::kMax: return detail::ReduceKernel<MAX_T>;                \
            case detail::kMin: return detail::ReduceKernel<MIN_T>;                \
            default: return nullptr;                                              \
        }                                                                         \
    }

#define HCCL_AMD_DEFINE_SELECT3(NAME, SUM_T, MAX_T, MIN_T)                         \
    detail::ReduceKernelFn NAME(int op)                                           \
    {                                                                             \
        switch (op) {                                                             \
            case detail::kSum: return detail::ReduceKernel<SUM_T>;                \
            case detail::kMax: return detail::ReduceKernel<MAX_T>;                \
            case detail::kMin: return detail::ReduceKernel<MIN_T>;                \
            default: return nullptr;                                              \
        }                                                                         \
    }

}  // namespace hccl_amd
