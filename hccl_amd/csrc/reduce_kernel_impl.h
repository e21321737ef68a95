// Fused N-rank reduce for gfx950 (MI355X).
//
// One launch performs the local-reduce work of every rank of a loopback world: each lane owns a
// 16-byte vector position, pulls that position from the N rank buffers with 128-bit loads, combines
// them in registers in the order a fold program dictates, and writes the result once per
// destination.  The path is bound by HBM bandwidth (N reads + M writes of the element range, no
// re-reads, no staging passes), so there is no MFMA; the fold program is read with scalar loads, and LDS only
// holds, for tree-shaped orders, the accumulators of enclosing levels.
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
            // (16-bit operands are widened first: promoted to int, the product of two large ones would overflow)
            using Wide = decltype(UT{} + 0u);
            return static_cast<T>(static_cast<UT>(static_cast<Wide>(static_cast<UT>(src)) * static_cast<Wide>(static_cast<UT>(dst))));
        } else if constexpr (OP == kMax) {
            return (src < dst) ? dst : src;
        } else {
            return (dst < src) ? dst : src;
        }
    }
};

// int8 with a 16-bit accumulator per element: the low byte of a 16-bit sum or product is the 8-bit result
// (alg_data_trans_wrapper.cc:1332-1343), MAX / MIN see the sign-extended value.  `Swar` switches the 16-byte
// vector path to the packed form of PackOps.
template <int OP>
struct Int8Ops {
    using S = int8_t;
    using A = int16_t;
    using Swar = void;
    static constexpr int kOp = OP;
    static __device__ __forceinline__ A Widen(S x) { return x; }
    static __device__ __forceinline__ S Narrow(A a) { return static_cast<S>(static_cast<uint8_t>(a)); }
    static __device__ __forceinline__ A Fold(A src, A dst)
    {
        if constexpr (OP == kSum) {
            return static_cast<A>(static_cast<uint16_t>(static_cast<uint16_t>(src) + static_cast<uint16_t>(dst)));
        } else if constexpr (OP == kProd) {
            // (widened to 32 bits first: promoted to int, the product of two large 16-bit values would overflow)
            return static_cast<A>(static_cast<uint16_t>(static_cast<uint32_t>(static_cast<uint16_t>(src)) *
                                                        static_cast<uint32_t>(static_cast<uint16_t>(dst))));
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

// 1.0f the optimiser cannot see through: multiplying by it keeps a fused multiply-add a fused multiply-add.
__device__ __forceinline__ float OpaqueOne()
{
    float one;
    asm volatile("v_mov_b32 %0, 1.0" : "=v"(one));
    return one;
}

// fp16 / bf16 SUM: fp32 accumulator, one rounding at the end.
//  * fp16 operands are folded with fma(x, 1, acc): x * 1 is exact, so the result is the IEEE sum, and the
//    hardware's mixed-precision fma converts and adds in one instruction.
//  * bf16 results are narrowed by the hardware's round-to-nearest-even conversion.  A NaN result is some
//    NaN (NaNs produced or carried by a sum have no defined payload); MAX / MIN never come here.
template <bool IS_BF16>
struct HalfSumOps {
    using S = uint16_t;
    using A = float;
    static __device__ __forceinline__ A Widen(S x) { return IS_BF16 ? Bf16BitsToFloat(x) : HalfBitsToFloat(x); }
    static __device__ __forceinline__ S Narrow(A a)
    {
        if constexpr (IS_BF16) {
            return __builtin_bit_cast(uint16_t, static_cast<__bf16>(a));
        } else {
            return FloatToHalfBits(a);
        }
    }
    static __device__ __forceinline__ A Fold(A src, A dst) { return src + dst; }
    static __device__ __forceinline__ A Accumulate(S x, A acc, float one)
    {
        if constexpr (IS_BF16) {
            return Bf16BitsToFloat(x) + acc;
        } else {
            return __builtin_fmaf(static_cast<float>(__builtin_bit_cast(_Float16, x)), one, acc);
        }
    }
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
typedef U32x4 U32x4Unaligned __attribute__((aligned(1)));   // a 128-bit load that may start on any element

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
            __builtin_nontemporal_store(__builtin_bit_cast(U32x4, v), (HCCL_AMD_GLOBAL U32x4Unaligned*)p);
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

// The fold program of this workgroup's sub-segment, read with scalar loads only (the image sits in device
// memory, 16-byte aligned; see kDevProgRankOff / kDevProgCtlOff): leaf i folds rank RankOf(i) and carries
// CtlOf(i) (see kCtlOpen).  srcByteOff advances every rank's buffer to the sub-segment.
typedef const uint32_t __attribute__((address_space(4))) * ProgWords;
struct ProgramView {
    ProgWords words;       // the program image as dwords
    uint64_t srcByteOff;
    uint32_t nLeaves;
};

// Byte `i` (static) of the 16 table bytes that start at byte offset `off` (a multiple of 16) of the image.
template <int kBytes>
struct TableBytes {
    uint32_t w[kBytes / 4];
    __device__ __forceinline__ void Load(ProgWords words, uint32_t off)
    {
#pragma unroll
        for (int k = 0; k < kBytes / 4; ++k) {
            w[k] = words[off / 4 + k];
        }
    }
    __device__ __forceinline__ uint32_t operator[](int i) const { return (w[i / 4] >> (8 * (i % 4))) & 0xFFu; }
};

// The rank and control bytes of a program's first batch of leaves, fetched by the kernel together with the
// program's header (one round of scalar loads) and handed to the interpreter.
template <int kBatch>
struct FirstBatch {
    TableBytes<kBatch> ranks, ctls;
    __device__ __forceinline__ void Load(ProgWords words)
    {
        ranks.Load(words, kDevProgRankOff);
        ctls.Load(words, kDevProgCtlOff);
    }
    // every word exists before the first is used
    __device__ __forceinline__ void Fence()
    {
#pragma unroll
        for (int k = 0; k < kBatch / 4; ++k) {
            asm volatile("" : "+s"(ranks.w[k]), "+s"(ctls.w[k]));
        }
    }
};

// The same for eight uniform 64-bit values (leaf addresses): all of them exist before the first is used.
__device__ __forceinline__ void ScalarFence8(uint64_t* r)
{
    asm volatile("" : "+s"(r[0]), "+s"(r[1]), "+s"(r[2]), "+s"(r[3]), "+s"(r[4]), "+s"(r[5]), "+s"(r[6]), "+s"(r[7]));
}

// Makes eight loaded vectors opaque to the optimiser at this point of the instruction stream.
__device__ __forceinline__ void IssueFence8(U32x4* r)
{
    asm volatile("" : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]), "+v"(r[4]), "+v"(r[5]), "+v"(r[6]), "+v"(r[7]));
}

// The launch's scalars, all fetched before anything is done with one of them: the compiler then requests them as a
// few wide scalar loads behind one wait, instead of one load and one wait wherever the code first needs a field.
__device__ __forceinline__ void FenceHot(ReduceHot& h)
{
    uint64_t prog = reinterpret_cast<uint64_t>(h.prog);
    asm volatile(""
                 : "+s"(prog), "+s"(h.total), "+s"(h.groupLen), "+s"(h.subLen), "+s"(h.srcGroupStride),
                   "+s"(h.dstGroupStride), "+s"(h.nGroup), "+s"(h.nSub), "+s"(h.nDst), "+s"(h.dstOwn),
                   "+s"(h.progGroupStride), "+s"(h.progSubStride), "+s"(h.blocksPerSub), "+s"(h.vecOk), "+s"(h.threads),
                   "+s"(h.vecBatch), "+s"(h.writeThrough), "+s"(h.leadFromSrc), "+s"(h.storeWaves), "+s"(h.varGroups));
    h.prog = reinterpret_cast<const uint8_t*>(prog);
}

// acc <- x (+) acc for a stored element x: the traits' fused form where they have one.
template <class E, class = void>
struct HasAccumulate {
    static constexpr bool value = false;
};
template <class E>
struct HasAccumulate<E, decltype(void(E::Accumulate(typename E::S{}, typename E::A{}, 1.0f)))> {
    static constexpr bool value = true;
};

template <class E>
__device__ __forceinline__ typename E::A Accumulate(typename E::S x, typename E::A acc, float one)
{
    if constexpr (HasAccumulate<E>::value) {
        return E::Accumulate(x, acc, one);
    } else {
        return E::Fold(E::Widen(x), acc);
    }
}

// The four things the interpreter does with a loaded vector of W elements.  The default goes element by
// element; a traits class may bring a packed form for its 16-byte vectors (E::Swar).
template <class E, int W, class = void>
struct PackOps {
    using S = typename E::S;
    static __device__ __forceinline__ void Init(AccPack<E, W>& acc, const Pack<S, W>& v)
    {
#pragma unroll
        for (int w = 0; w < W; ++w) {
            acc.a[w] = E::Widen(v.e[w]);
        }
    }
    static __device__ __forceinline__ void Accumulate(AccPack<E, W>& acc, const Pack<S, W>& v, float one)
    {
#pragma unroll
        for (int w = 0; w < W; ++w) {
            acc.a[w] = detail::Accumulate<E>(v.e[w], acc.a[w], one);
        }
    }
    static __device__ __forceinline__ void Merge(AccPack<E, W>& acc, const AccPack<E, W>& outer)
    {
#pragma unroll
        for (int w = 0; w < W; ++w) {
            acc.a[w] = E::Fold(acc.a[w], outer.a[w]);
        }
    }
    static __device__ __forceinline__ Pack<S, W> Narrow(const AccPack<E, W>& acc)
    {
        Pack<S, W> out;
#pragma unroll
        for (int w = 0; w < W; ++w) {
            out.e[w] = E::Narrow(acc.a[w]);
        }
        return out;
    }
};

// int8 vectors, four elements per dword: the accumulator of a dword is two dwords of two 16-bit lanes each,
// `even` for bytes 0 and 2, `odd` for bytes 1 and 3.  SUM and PROD only need the low byte of a lane to be right
// (it never depends on what sits above it), so operands go in unmasked: `x` for the even lanes, `x >> 8` for the
// odd ones.  MAX / MIN compare sign-extended lanes.  The 32 bytes of AccPack<E, 16> hold the eight dwords.
template <class E>
struct PackOps<E, 16, typename E::Swar> {
    using S = typename E::S;
    typedef int16_t S16x2 __attribute__((ext_vector_type(2)));
    typedef uint16_t U16x2 __attribute__((ext_vector_type(2)));
    struct Lanes {
        uint32_t even[4];
        uint32_t odd[4];
    };
    static_assert(sizeof(Lanes) == sizeof(AccPack<E, 16>), "accumulator layout");

    static __device__ __forceinline__ uint32_t EvenOperand(uint32_t x)
    {
        if constexpr (E::kOp == kMax || E::kOp == kMin) {
            return __builtin_bit_cast(uint32_t, (__builtin_bit_cast(S16x2, x) << 8) >> 8);
        } else {
            return x;
        }
    }
    static __device__ __forceinline__ uint32_t OddOperand(uint32_t x)
    {
        if constexpr (E::kOp == kMax || E::kOp == kMin) {
            return __builtin_bit_cast(uint32_t, __builtin_bit_cast(S16x2, x) >> 8);
        } else {
            return x >> 8;
        }
    }
    // dst <- src (+) dst on both lanes of a dword
    static __device__ __forceinline__ uint32_t FoldLanes(uint32_t src, uint32_t dst)
    {
        if constexpr (E::kOp == kSum) {
            return __builtin_bit_cast(uint32_t, __builtin_bit_cast(U16x2, src) + __builtin_bit_cast(U16x2, dst));
        } else if constexpr (E::kOp == kProd) {
            return __builtin_bit_cast(uint32_t, __builtin_bit_cast(U16x2, src) * __builtin_bit_cast(U16x2, dst));
        } else if constexpr (E::kOp == kMax) {
            return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(S16x2, src),
                                                                          __builtin_bit_cast(S16x2, dst)));
        } else {
            return __builtin_bit_cast(uint32_t, __builtin_elementwise_min(__builtin_bit_cast(S16x2, src),
                                                                          __builtin_bit_cast(S16x2, dst)));
        }
    }
    static __device__ __forceinline__ void Init(AccPack<E, 16>& acc, const Pack<S, 16>& v)
    {
        const U32x4 x = __builtin_bit_cast(U32x4, v);
        Lanes l;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            l.even[k] = EvenOperand(x[k]);
            l.odd[k] = OddOperand(x[k]);
        }
        acc = __builtin_bit_cast(AccPack<E, 16>, l);
    }
    static __device__ __forceinline__ void Accumulate(AccPack<E, 16>& acc, const Pack<S, 16>& v, float)
    {
        const U32x4 x = __builtin_bit_cast(U32x4, v);
        Lanes l = __builtin_bit_cast(Lanes, acc);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            l.even[k] = FoldLanes(EvenOperand(x[k]), l.even[k]);
            l.odd[k] = FoldLanes(OddOperand(x[k]), l.odd[k]);
        }
        acc = __builtin_bit_cast(AccPack<E, 16>, l);
    }
    static __device__ __forceinline__ void Merge(AccPack<E, 16>& acc, const AccPack<E, 16>& outer)
    {
        Lanes l = __builtin_bit_cast(Lanes, acc);
        const Lanes o = __builtin_bit_cast(Lanes, outer);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            l.even[k] = FoldLanes(l.even[k], o.even[k]);
            l.odd[k] = FoldLanes(l.odd[k], o.odd[k]);
        }
        acc = __builtin_bit_cast(AccPack<E, 16>, l);
    }
    static __device__ __forceinline__ Pack<S, 16> Narrow(const AccPack<E, 16>& acc)
    {
        const Lanes l = __builtin_bit_cast(Lanes, acc);
        U32x4 x;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            x[k] = (l.even[k] & 0x00FF00FFu) | ((l.odd[k] & 0x00FF00FFu) << 8);
        }
        return __builtin_bit_cast(Pack<S, 16>, x);
    }
};

// Evaluates the whole tree for the W elements at element offset `e` of the sub-segment.  Leaves are
// taken a batch at a time: their loads are all issued before the first fold, whatever the tree shape.
// kBatch leaves are taken at a time (a multiple of 8).
template <class E, int W, int kBatch>
__device__ __forceinline__ Pack<typename E::S, W> ReduceValue(const ProgramView& pv, uint32_t* stack,
                                                              const ReduceArgs& args, const ReduceHot& h, uint64_t e,
                                                              const FirstBatch<kBatch>* first = nullptr)
{
    using S = typename E::S;
    AccPack<E, W> acc;
    float one = 1.0f;
    if constexpr (HasAccumulate<E>::value) {
        one = OpaqueOne();
    }
    uint32_t level = 0;
    bool init = true;   // the next leaf starts a level instead of being folded into it
    const uint32_t nLeaves = pv.nLeaves;
    for (uint32_t b = 0; b < nLeaves; b += kBatch) {
        TableBytes<kBatch> ranks, ctls;
        if (first != nullptr && b == 0) {
            ranks = first->ranks;
            ctls = first->ctls;
        } else {
            ranks.Load(pv.words, kDevProgRankOff + b);
            ctls.Load(pv.words, kDevProgCtlOff + b);
        }
        // Leaf addresses first and unconditionally (table bytes past the last leaf name rank 0), so that their
        // scalar loads go out together instead of one wait per leaf.
        uint64_t leaf[kBatch];
#pragma unroll
        for (int i = 0; i < kBatch; ++i) {
            leaf[i] = reinterpret_cast<uint64_t>(args.src[ranks[i]]);
        }
#pragma unroll
        for (int i = 0; i < kBatch; i += 8) {
            ScalarFence8(leaf + i);
        }
#pragma unroll
        for (int i = 0; i < kBatch; ++i) {
            leaf[i] += pv.srcByteOff;
        }
        Pack<S, W> v[kBatch];
        if constexpr (sizeof(S) * W == 16) {
            // The vectors stay untyped 128-bit values until the whole batch has been issued: nothing may
            // consume one earlier (the compiler would sink the first unpacking instruction of each operand
            // next to its load and wait there), and a load retyped to the element type loses its
            // non-temporal hint.
            U32x4 raw[kBatch];
#pragma unroll
            for (int i = 0; i < kBatch; ++i) {
                if (b + i < nLeaves) {
                    const S* p = reinterpret_cast<const S*>(leaf[i]) + e;
                    raw[i] = __builtin_nontemporal_load((const HCCL_AMD_GLOBAL U32x4Unaligned*)p);
                }
            }
#pragma unroll
            for (int i = 0; i < kBatch; i += 8) {
                IssueFence8(raw + i);
            }
#pragma unroll
            for (int i = 0; i < kBatch; ++i) {
                v[i] = __builtin_bit_cast(Pack<S, W>, raw[i]);
            }
        } else {
#pragma unroll
            for (int i = 0; i < kBatch; ++i) {
                if (b + i < nLeaves) {
                    v[i] = LoadPack<S, W>(reinterpret_cast<const void*>(leaf[i]), e);
                }
            }
        }
#pragma unroll
        for (int i = 0; i < kBatch; ++i) {
            if (b + i < nLeaves) {
                const uint32_t ctl = ctls[i];
                if (ctl & kCtlOpen) {
                    PushAcc<E, W>(stack, h.threads, level, acc);
                    ++level;
                    init = true;
                }
                if (init) {
                    PackOps<E, W>::Init(acc, v[i]);
                    init = false;
                } else {
                    PackOps<E, W>::Accumulate(acc, v[i], one);
                }
                for (uint32_t closes = ctl & 0x7Fu; closes != 0; --closes) {
                    AccPack<E, W> outer;
                    --level;
                    PopAcc<E, W>(stack, h.threads, level, outer);
                    PackOps<E, W>::Merge(acc, outer);   // nested value is src, enclosing level is dst
                }
            }
        }
    }
    return PackOps<E, W>::Narrow(acc);
}

// The value of ReduceValue written to the destinations firstDst, firstDst + dstStep, ... of the launch (all of
// them with 0 and 1), or to the group's own destination.
// `ownOrFirst` is the address the kernel fetched ahead with its second round of scalar loads: the group's own
// destination, or destination 0.  A launch with one destination per result (ReduceScatter(V), Reduce, the fold of
// the two-kernel AllReduce) then stores without another scalar load between the fold and the store.
// kAhead: firstDst and dstStep are uniform (every wavefront stores to every destination), so the remaining
// addresses can be fetched four at a time.
template <class S, int W, bool kAhead>
__device__ __forceinline__ void StoreResult(const ReduceArgs& args, const ReduceHot& h, const Pack<S, W>& out,
                                            uint64_t elemOff, uint64_t ownOrFirst, uint32_t firstDst, uint32_t dstStep)
{
    void* const ahead = reinterpret_cast<void*>(ownOrFirst);
    if (h.dstOwn) {
        StorePack<S, W>(ahead, elemOff, out, h.writeThrough != 0);
    } else {
        uint32_t d = firstDst;
        if (d == 0) {
            StorePack<S, W>(ahead, elemOff, out, h.writeThrough != 0);
            d = dstStep;
        }
        if constexpr (!kAhead) {
            for (; d < h.nDst; d += dstStep) {
                StorePack<S, W>(args.dst[d], elemOff, out, h.writeThrough != 0);
            }
            return;
        }
        // The other destinations four at a time: their addresses are requested together, one round of scalar loads
        // per four stores instead of one per store (indices past the table are never used and read entry 0).
        for (; d < h.nDst; d += 4 * dstStep) {
            uint64_t to[4];
#pragma unroll
            for (uint32_t k = 0; k < 4; ++k) {
                const uint32_t dk = d + k * dstStep;
                to[k] = reinterpret_cast<uint64_t>(args.dst[dk < static_cast<uint32_t>(kMaxRanks) ? dk : 0u]);
            }
            asm volatile("" : "+s"(to[0]), "+s"(to[1]), "+s"(to[2]), "+s"(to[3]));
#pragma unroll
            for (uint32_t k = 0; k < 4; ++k) {
                if (d + k * dstStep < h.nDst) {
                    StorePack<S, W>(reinterpret_cast<void*>(to[k]), elemOff, out, h.writeThrough != 0);
                }
            }
        }
    }
}

template <class E, int W, int kBatch>
__device__ __forceinline__ void ReduceOne(const ProgramView& pv, uint32_t* stack, const ReduceArgs& args,
                                          const ReduceHot& h, uint64_t e, uint64_t dstOff, uint64_t ownOrFirst,
                                          const FirstBatch<kBatch>* first = nullptr)
{
    const Pack<typename E::S, W> out = ReduceValue<E, W, kBatch>(pv, stack, args, h, e, first);
    StoreResult<typename E::S, W, true>(args, h, out, dstOff + e, ownOrFirst, 0, 1);
}

// Two adjacent tiles per wavefront for flat programs (no nested levels) of up to eight leaves (one batch): the sixteen loads of both tiles
// are issued before the first fold and both folds before the first store.
// A launch that is a single generation of wavefronts (a few MiB per rank) otherwise reads, then writes, and pays
// the ramp of each phase in full.  `on0` / `on1`: this lane has a vector in the first / second tile.
template <class E, int W>
__device__ __forceinline__ void ReducePair(const ProgramView& pv, uint32_t* stack, const ReduceArgs& args,
                                           const ReduceHot& h, uint64_t e0, bool on0, bool on1, uint64_t dstOff,
                                           uint64_t ownOrFirst, const FirstBatch<8>& first)
{
    (void)stack;
    using S = typename E::S;
    static_assert(sizeof(S) * W == 16, "the pair form exists for the 128-bit path only");
    constexpr int kBatch = 8;
    const uint64_t e1 = e0 + 64u * W;
    const uint32_t nLeaves = pv.nLeaves;
    float one = 1.0f;
    if constexpr (HasAccumulate<E>::value) {
        one = OpaqueOne();
    }
    uint64_t leaf[kBatch];
#pragma unroll
    for (int i = 0; i < kBatch; ++i) {
        leaf[i] = reinterpret_cast<uint64_t>(args.src[first.ranks[i]]);
    }
    ScalarFence8(leaf);
#pragma unroll
    for (int i = 0; i < kBatch; ++i) {
        leaf[i] += pv.srcByteOff;
    }
    U32x4 raw0[kBatch];
    U32x4 raw1[kBatch];
#pragma unroll
    for (int i = 0; i < kBatch; ++i) {
        if (static_cast<uint32_t>(i) < nLeaves && on0) {
            const S* p = reinterpret_cast<const S*>(leaf[i]) + e0;
            raw0[i] = __builtin_nontemporal_load((const HCCL_AMD_GLOBAL U32x4Unaligned*)p);
        }
    }
#pragma unroll
    for (int i = 0; i < kBatch; ++i) {
        if (static_cast<uint32_t>(i) < nLeaves && on1) {
            const S* p = reinterpret_cast<const S*>(leaf[i]) + e1;
            raw1[i] = __builtin_nontemporal_load((const HCCL_AMD_GLOBAL U32x4Unaligned*)p);
        }
    }
    // (a flat program: leaf 0 starts the value, every other leaf is folded into it)
    const auto fold = [&](U32x4* raw) {
        IssueFence8(raw);
        AccPack<E, W> acc;
        PackOps<E, W>::Init(acc, __builtin_bit_cast(Pack<S, W>, raw[0]));
#pragma unroll
        for (int i = 1; i < kBatch; ++i) {
            if (static_cast<uint32_t>(i) < nLeaves) {
                PackOps<E, W>::Accumulate(acc, __builtin_bit_cast(Pack<S, W>, raw[i]), one);
            }
        }
        return PackOps<E, W>::Narrow(acc);
    };
    // Both folds in front of the first store: whatever waits for the second tile's loads would otherwise also wait
    // for the first tile's stores to be acknowledged (loads and stores leave one counter in issue order).
    Pack<S, W> out0;
    Pack<S, W> out1;
    if (on0) {
        out0 = fold(raw0);
    }
    if (on1) {
        out1 = fold(raw1);
    }
    if (on0) {
        StoreResult<S, W, true>(args, h, out0, dstOff + e0, ownOrFirst, 0, 1);
    }
    if (on1) {
        StoreResult<S, W, true>(args, h, out1, dstOff + e1, ownOrFirst, 0, 1);
    }
}

// Dynamic LDS: the accumulator stack, (plan depth - 1) * accumulator bytes * args.threads.
// VB = leaves per batch of the 128-bit path: 8 keeps the register count low (more wavefronts in flight), 16 has
// every load of up to sixteen ranks in flight at once; the launcher picks per launch.
// kPair: workgroups of 64 lanes take two adjacent tiles each (ReducePair) where the program has at most eight leaves.
template <class E, int VB, bool kPair = false>
__global__ __launch_bounds__(kThreads) void ReduceKernel(const ReduceArgs args)
{
    static_assert(!kPair || VB == 8, "the pair form is built on the eight-leaf batch");
    using S = typename E::S;
    constexpr int W = 16 / sizeof(S);
    extern __shared__ uint32_t accStack[];
    ReduceHot h = args;
    FenceHot(h);

    uint32_t g, c, blk, blocksHere;   // group, sub-segment, this workgroup's index among the blocksHere of it
    uint64_t gLen;
    uint64_t gSrc;
    if (h.varGroups) {
        // Groups of unequal length own unequal shares of the grid: first group whose last block is not before us.
        uint32_t firstBlock = 0;
        uint32_t endBlock = 0xFFFFFFFFu;
        g = 0;
        if (h.nGroup <= 16) {
            // Up to sixteen groups: their ends in one round of scalar loads (the launcher pads the table with
            // 0xFFFFFFFF up to sixteen entries), then a count without branches: the ends do not decrease, so the
            // groups that end at or before this workgroup are the ones in front of it, the last of them ends where
            // this workgroup's group begins, and the first of the others is its own.
            uint32_t ends[16];
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                ends[j] = args.groupBlockEnd[j];
            }
            asm volatile("" : "+s"(ends[0]), "+s"(ends[1]), "+s"(ends[2]), "+s"(ends[3]), "+s"(ends[4]), "+s"(ends[5]),
                              "+s"(ends[6]), "+s"(ends[7]), "+s"(ends[8]), "+s"(ends[9]), "+s"(ends[10]), "+s"(ends[11]),
                              "+s"(ends[12]), "+s"(ends[13]), "+s"(ends[14]), "+s"(ends[15]));
            const uint32_t me = blockIdx.x;
            const int used = h.nGroup <= 8 ? 8 : 16;
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                if (j < used) {
                    const bool before = ends[j] <= me;
                    // 1 when the group ends at or before this workgroup, in scalar arithmetic (a comparison result
                    // added up as a number would travel through a vector register)
                    g += (ends[j] > me + 1u ? ends[j] : me + 1u) - (ends[j] > me ? ends[j] : me);
                    firstBlock = before ? ends[j] : firstBlock;
                    const uint32_t behind = before ? 0xFFFFFFFFu : ends[j];
                    endBlock = behind < endBlock ? behind : endBlock;
                }
            }
        } else {
            uint32_t lo = 0;
            uint32_t hi = h.nGroup - 1;
            while (lo < hi) {
                const uint32_t mid = (lo + hi) >> 1;
                if (blockIdx.x >= args.groupBlockEnd[mid]) {
                    lo = mid + 1;
                } else {
                    hi = mid;
                }
            }
            g = lo;
            firstBlock = g == 0 ? 0u : args.groupBlockEnd[g - 1];
            endBlock = args.groupBlockEnd[g];
        }
        c = 0;
        blk = blockIdx.x - firstBlock;
        blocksHere = endBlock - firstBlock;
        gLen = args.groupLenV[g];
        gSrc = args.groupOffV[g];
    } else {
        // The grid is (workgroups per sub-segment, sub-segments, groups): no division to find one's place.
        blk = blockIdx.x;
        blocksHere = h.blocksPerSub;
        c = blockIdx.y;
        g = blockIdx.z;
        const uint64_t gBeg = static_cast<uint64_t>(g) * h.groupLen;
        if (gBeg >= h.total) {
            return;
        }
        gLen = (h.total - gBeg < h.groupLen) ? h.total - gBeg : h.groupLen;
        gSrc = static_cast<uint64_t>(g) * h.srcGroupStride;
    }
    const uint64_t sBeg = static_cast<uint64_t>(c) * h.subLen;
    uint64_t sEnd = (c == h.nSub - 1) ? gLen : sBeg + h.subLen;
    sEnd = sEnd < gLen ? sEnd : gLen;
    if (sBeg >= sEnd) {
        return;
    }
    const uint64_t len = sEnd - sBeg;
    const uint64_t srcOff = gSrc + sBeg;
    const uint64_t dstOff = h.dstOwn ? sBeg : static_cast<uint64_t>(g) * h.dstGroupStride + sBeg;

    ProgramView pv;
    pv.words = (ProgWords)(uintptr_t)(h.prog + static_cast<uint64_t>(g * h.progGroupStride + c * h.progSubStride) *
                                                      kDevProgBytes);
    pv.srcByteOff = srcOff * sizeof(S);
    // Second round of scalar loads, all requested together: the program's header, and the two buffer addresses the
    // alignment below is taken from.
    uint32_t header = pv.words[0];
    // (The sixteen-leaf batch keeps its tables out of this round: with sixteen leaf addresses live as well, the
    // scalar registers would not hold them.)
    constexpr bool kPreloadBatch = VB == 8;
    FirstBatch<VB> firstBatch;
    if constexpr (kPreloadBatch) {
        firstBatch.Load(pv.words);
    }
    uint64_t firstDstAddr = reinterpret_cast<uint64_t>(h.dstOwn ? args.dst[g] : args.dst[0]);
    uint64_t firstSrcAddr = reinterpret_cast<uint64_t>(args.src[0]);
    asm volatile("" : "+s"(header), "+s"(firstDstAddr), "+s"(firstSrcAddr));
    if constexpr (kPreloadBatch) {
        firstBatch.Fence();
    }
    const FirstBatch<VB>* const preloaded = kPreloadBatch ? &firstBatch : nullptr;
    pv.nLeaves = header & 0xFFu;

    const uint64_t stride = static_cast<uint64_t>(blocksHere) * h.threads;
    const uint64_t first = static_cast<uint64_t>(blk) * h.threads + threadIdx.x;

    // When vecOk, `head` elements bring the stores to the first destination onto a 16-byte boundary, a 128-bit
    // body follows, and fewer than W elements remain.  Sources and further destinations only need element
    // alignment: their 128-bit accesses may be unaligned (full speed when they are congruent with the first
    // destination, up to 15 % less otherwise).  Without vecOk everything goes element by element.  The body's vectors are dealt to the lanes shifted by `lead`, so that lane 0
    // of every wavefront starts a 1 KiB boundary (a wavefront whose 1 KiB straddles nine lines moves two of them
    // twice, and one that starts on a line but off the 1 KiB grid still loads slower): of the destination, or
    // with leadFromSrc of the sources.
    uint64_t head = len;
    uint64_t nVec = 0;
    uint32_t lead = 0;
    if (h.vecOk) {
        const uint64_t addr = firstDstAddr + dstOff * sizeof(S);
        const uint32_t mis = static_cast<uint32_t>(addr & 15u);
        head = mis ? (16u - mis) / sizeof(S) : 0;
        head = head < len ? head : len;
        nVec = (len - head) / W;
        // One result stream fed by many sources: the sources' lines count (those of the first rank stand for all;
        // peers' buffers are usually congruent), otherwise the destination's.
        const uint64_t lineOf = h.leadFromSrc
                                    ? firstSrcAddr + (srcOff + head) * sizeof(S)
                                    : addr + head * sizeof(S);
        lead = static_cast<uint32_t>((lineOf >> 4) & kReduceLeadMask);
    }
    const uint64_t bodyEnd = head + nVec * W;
    const uint64_t nScalar = head + (len - bodyEnd);
    if (!kPair && VB == 8 && (h.storeWaves & kStoreWavesAllFold) != 0) {
        // (Built into the eight-leaf batch only: the sixteen-leaf kernels have no scalar registers to spare.)
        // Every wavefront of the workgroup folds a tile of its own, parks the result in LDS, and after the barrier
        // writes the tiles of all wavefronts to its destinations: wavefront k owns destinations k, k + waves, ...
        // A launch that is a single generation of wavefronts (a few MiB per rank, many destinations) otherwise ends
        // with every wavefront writing 1 KiB to every stream at the same moment; this way a wavefront writes
        // `waves` KiB in a row to one or two of them.  The programs are flat (the launcher's caller has checked), so
        // the dynamic LDS holds no accumulator stack and is the exchange area: two rounds of `waves` tiles, which
        // makes one barrier per round enough.  The trip count is the same for every wavefront.
        const uint32_t waves = h.storeWaves & 0xFFu;
        U32x4* const parked = reinterpret_cast<U32x4*>(accStack);
        const uint32_t wave = threadIdx.x >> 6;
        const uint32_t lane = threadIdx.x & 63u;
        const uint64_t span = static_cast<uint64_t>(waves) * 64;
        uint32_t slot = 0;
        for (uint64_t base = static_cast<uint64_t>(blk) * span; base < nVec + lead; base += static_cast<uint64_t>(blocksHere) * span) {
            const uint64_t u = base + wave * 64 + lane;
            if (u >= lead && u < nVec + lead) {
                const Pack<S, W> out = ReduceValue<E, W, VB>(pv, accStack, args, h, head + (u - lead) * W, preloaded);
                parked[(slot * waves + wave) * 64 + lane] = __builtin_bit_cast(U32x4, out);
            }
            __syncthreads();
            for (uint32_t t = 0; t < waves; ++t) {
                const uint64_t ut = base + t * 64 + lane;
                if (ut >= lead && ut < nVec + lead) {
                    const Pack<S, W> out = __builtin_bit_cast(Pack<S, W>, parked[(slot * waves + t) * 64 + lane]);
                    StoreResult<S, W, false>(args, h, out, dstOff + head + (ut - lead) * W, firstDstAddr, wave, waves);
                }
            }
            slot ^= 1u;
        }
        if (wave == 0) {
            for (uint64_t i = static_cast<uint64_t>(blk) * 64 + lane; i < nScalar; i += static_cast<uint64_t>(blocksHere) * 64) {
                const uint64_t e = i < head ? i : i - head + bodyEnd;
                ReduceOne<E, 1, 8>(pv, accStack, args, h, e, dstOff, firstDstAddr);
            }
        }
        return;
    }
    if (!kPair && h.storeWaves > 1) {
        // Stores split over the wavefronts of the workgroup (h.threads == 64 lanes fold, 64 * storeWaves run):
        // wavefront 0 folds the tile and parks the result in LDS, wavefront k writes it to destinations k,
        // k + storeWaves, ...  A wavefront that stores to many streams one after the other is what bounds the
        // many-destination launches; with two to four destinations per wavefront the same stores leave 5-15 %
        // faster.  The trip count is the same for every wavefront (the barrier sits in the loop), and results
        // alternate between two LDS tiles so that one barrier per tile is enough.
        __shared__ U32x4 parked[2][64];
        const uint32_t wave = threadIdx.x >> 6;
        const uint32_t lane = threadIdx.x & 63u;
        uint32_t slot = 0;
        for (uint64_t base = static_cast<uint64_t>(blk) * 64; base < nVec + lead; base += static_cast<uint64_t>(blocksHere) * 64) {
            const uint64_t u = base + lane;
            const bool active = u >= lead && u < nVec + lead;
            const uint64_t e = head + (u - lead) * W;
            Pack<S, W> out;
            if (wave == 0 && active) {
                out = ReduceValue<E, W, VB>(pv, accStack, args, h, e, preloaded);
                parked[slot][lane] = __builtin_bit_cast(U32x4, out);
            }
            __syncthreads();
            if (active) {
                if (wave != 0) {
                    out = __builtin_bit_cast(Pack<S, W>, parked[slot][lane]);
                }
                StoreResult<S, W, false>(args, h, out, dstOff + e, firstDstAddr, wave, h.storeWaves);
            }
            slot ^= 1u;
        }
        if (wave == 0) {
            for (uint64_t i = static_cast<uint64_t>(blk) * 64 + lane; i < nScalar; i += static_cast<uint64_t>(blocksHere) * 64) {
                const uint64_t e = i < head ? i : i - head + bodyEnd;
                ReduceOne<E, 1, 8>(pv, accStack, args, h, e, dstOff, firstDstAddr);
            }
        }
        return;
    }
    if constexpr (kPair && sizeof(S) * W == 16) {
        // (h.threads == 64, and the launcher's caller has checked that every program is flat and has at most eight leaves)
        // workgroup blk takes tiles 2 blk and 2 blk + 1, then strides on by pairs
        for (uint64_t u = first + static_cast<uint64_t>(blk) * 64; u < nVec + lead; u += 2 * stride) {
            const bool on0 = u >= lead;
            const bool on1 = u + 64 < nVec + lead;
            ReducePair<E, W>(pv, accStack, args, h, head + (u - lead) * W, on0, on1, dstOff, firstDstAddr, firstBatch);
        }
    } else {
        for (uint64_t u = first; u < nVec + lead; u += stride) {
            if (u >= lead) {
                ReduceOne<E, W, VB>(pv, accStack, args, h, head + (u - lead) * W, dstOff, firstDstAddr, preloaded);
            }
        }
    }
    for (uint64_t i = first; i < nScalar; i += stride) {
        const uint64_t e = i < head ? i : i - head + bodyEnd;
        ReduceOne<E, 1, 8>(pv, accStack, args, h, e, dstOff, firstDstAddr);
    }
}

using ReduceKernelFn = void (*)(const ReduceArgs);

// A flat fold of up to eight leaves to up to eight destinations, described by its arguments alone (DirectFoldArgs):
// for the launch that is a single generation of wavefronts (a few MiB per rank), where the time in front of the first
// vector load and the length of the code count.  Workgroup b takes the blockDim.x / 64 tiles from tile
// b * (blockDim.x / 64) on: every wavefront folds one tile (all leaves' loads issued before the first fold, leaves in
// the order of src[]), parks the result in LDS, and behind the barrier wavefront k writes the tiles of all wavefronts
// to destinations k, k + waves, ...: `waves` KiB in a row to one or two streams instead of 1 KiB to each.  The
// elements behind the last whole vector are folded one by one by the first lanes of workgroup 0.  Same folds in the
// same order as ReduceValue on a flat program, hence the same bits.
template <class E>
__global__ __launch_bounds__(64 * kDirectFoldMaxWaves) void DirectFoldKernel(const DirectFoldArgs a)
{
    using S = typename E::S;
    constexpr int W = 16 / sizeof(S);
    constexpr int kLeaves = static_cast<int>(kDirectFoldMaxLeaves);
    constexpr uint32_t kPerWave = kDirectFoldMaxDst / 2;   // destinations of one wavefront at most (two wavefronts or more)
    static_assert(kLeaves == 8, "one batch of eight loads");
    extern __shared__ uint32_t accStack[];
    U32x4* const parked = reinterpret_cast<U32x4*>(accStack);
    const uint32_t wave = Uniform(threadIdx.x >> 6);
    const uint32_t lane = threadIdx.x & 63u;
    // all leaf addresses and the counts exist before the first is used: one block of scalar loads, one wait
    uint64_t leaf[kLeaves];
#pragma unroll
    for (int i = 0; i < kLeaves; ++i) {
        leaf[i] = reinterpret_cast<uint64_t>(a.src[i]);
    }
    uint64_t nVec = a.nVec;
    uint32_t nSrc = a.nSrc;
    uint32_t nDst = a.nDst;
    uint32_t tail = a.tail;
    uint32_t waves = a.waves;   // == blockDim.x / 64, which would be a scalar load of its own in front of these
    ScalarFence8(leaf);
    asm volatile("" : "+s"(nVec), "+s"(nSrc), "+s"(nDst), "+s"(tail), "+s"(waves));
    // this wavefront's destination addresses, requested before the vector loads and first used behind the barrier
    // (indices past the table read entry 0 and are never used)
    uint64_t to[kPerWave];
#pragma unroll
    for (uint32_t k = 0; k < kPerWave; ++k) {
        const uint32_t d = wave + k * waves;
        to[k] = reinterpret_cast<uint64_t>(a.dst[d < kDirectFoldMaxDst ? d : 0u]);
    }
    float one = 1.0f;
    if constexpr (HasAccumulate<E>::value) {
        one = OpaqueOne();
    }
    const uint64_t tile0 = static_cast<uint64_t>(blockIdx.x) * waves;
    const uint64_t u = (tile0 + wave) * 64 + lane;
    if (u < nVec) {
        U32x4 raw[kLeaves];
#pragma unroll
        for (int i = 0; i < kLeaves; ++i) {
            if (static_cast<uint32_t>(i) < nSrc) {
                raw[i] = __builtin_nontemporal_load(reinterpret_cast<const HCCL_AMD_GLOBAL U32x4*>(leaf[i]) + u);
            }
        }
        IssueFence8(raw);
        AccPack<E, W> acc;
        PackOps<E, W>::Init(acc, __builtin_bit_cast(Pack<S, W>, raw[0]));
#pragma unroll
        for (int i = 1; i < kLeaves; ++i) {
            if (static_cast<uint32_t>(i) < nSrc) {
                PackOps<E, W>::Accumulate(acc, __builtin_bit_cast(Pack<S, W>, raw[i]), one);
            }
        }
        parked[wave * 64 + lane] = __builtin_bit_cast(U32x4, PackOps<E, W>::Narrow(acc));
    }
    __syncthreads();
    // (a workgroup whose tiles are all whole, every one but the last, stores without a bounds check per tile)
    const bool whole = (tile0 + waves) * 64 <= nVec;
#pragma unroll
    for (uint32_t k = 0; k < kPerWave; ++k) {
        if (wave + k * waves < nDst) {
            HCCL_AMD_GLOBAL U32x4* const out = reinterpret_cast<HCCL_AMD_GLOBAL U32x4*>(to[k]) + tile0 * 64 + lane;
            if (whole) {
                for (uint32_t t = 0; t < waves; ++t) {
                    __builtin_nontemporal_store(parked[t * 64 + lane], out + t * 64);
                }
            } else {
                for (uint32_t t = 0; t < waves; ++t) {
                    if ((tile0 + t) * 64 + lane < nVec) {
                        __builtin_nontemporal_store(parked[t * 64 + lane], out + t * 64);
                    }
                }
            }
        }
    }
    if (blockIdx.x == 0 && wave == 0 && lane < tail) {
        const uint64_t e = nVec * W + lane;
        AccPack<E, 1> acc;
        PackOps<E, 1>::Init(acc, LoadPack<S, 1>(reinterpret_cast<const void*>(leaf[0]), e));
#pragma unroll
        for (int i = 1; i < kLeaves; ++i) {
            if (static_cast<uint32_t>(i) < nSrc) {
                PackOps<E, 1>::Accumulate(acc, LoadPack<S, 1>(reinterpret_cast<const void*>(leaf[i]), e), one);
            }
        }
        const Pack<S, 1> out = PackOps<E, 1>::Narrow(acc);
        for (uint32_t d = 0; d < nDst; ++d) {
            StorePack<S, 1>(a.dst[d], e, out, false);
        }
    }
}

// The same with two tiles per wavefront, for a vector count that fills every workgroup (a multiple of
// 128 * waves; no elements behind the last vector; no bounds checks): the loads of both tiles are issued before the
// first fold, a workgroup of W wavefronts takes 2 W tiles in a row, and wavefront k writes 2 W KiB in a row to each of
// its destinations.  Half as many workgroups, each with twice the loads in flight.
template <class E>
__global__ __launch_bounds__(64 * kDirectFoldMaxWaves) void DirectFoldTwoTileKernel(const DirectFoldArgs a)
{
    using S = typename E::S;
    constexpr int W = 16 / sizeof(S);
    constexpr int kLeaves = static_cast<int>(kDirectFoldMaxLeaves);
    constexpr uint32_t kPerWave = kDirectFoldMaxDst / 2;
    static_assert(kLeaves == 8, "one batch of eight loads per tile");
    extern __shared__ uint32_t accStack[];
    U32x4* const parked = reinterpret_cast<U32x4*>(accStack);
    const uint32_t wave = Uniform(threadIdx.x >> 6);
    const uint32_t lane = threadIdx.x & 63u;
    uint64_t leaf[kLeaves];
#pragma unroll
    for (int i = 0; i < kLeaves; ++i) {
        leaf[i] = reinterpret_cast<uint64_t>(a.src[i]);
    }
    uint32_t nSrc = a.nSrc;
    uint32_t nDst = a.nDst;
    uint32_t waves = a.waves;
    ScalarFence8(leaf);
    asm volatile("" : "+s"(nSrc), "+s"(nDst), "+s"(waves));
    uint64_t to[kPerWave];
#pragma unroll
    for (uint32_t k = 0; k < kPerWave; ++k) {
        const uint32_t d = wave + k * waves;
        to[k] = reinterpret_cast<uint64_t>(a.dst[d < kDirectFoldMaxDst ? d : 0u]);
    }
    float one = 1.0f;
    if constexpr (HasAccumulate<E>::value) {
        one = OpaqueOne();
    }
    const uint32_t lanes = waves * 64;
    const uint64_t first = static_cast<uint64_t>(blockIdx.x) * (2 * lanes);   // the workgroup's first vector
    U32x4 raw[2][kLeaves];
#pragma unroll
    for (int i = 0; i < kLeaves; ++i) {
        if (static_cast<uint32_t>(i) < nSrc) {
            const HCCL_AMD_GLOBAL U32x4* const p =
                reinterpret_cast<const HCCL_AMD_GLOBAL U32x4*>(leaf[i]) + first + threadIdx.x;
            raw[0][i] = __builtin_nontemporal_load(p);
            raw[1][i] = __builtin_nontemporal_load(p + lanes);
        }
    }
    IssueFence8(raw[0]);
    IssueFence8(raw[1]);
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        AccPack<E, W> acc;
        PackOps<E, W>::Init(acc, __builtin_bit_cast(Pack<S, W>, raw[k][0]));
#pragma unroll
        for (int i = 1; i < kLeaves; ++i) {
            if (static_cast<uint32_t>(i) < nSrc) {
                PackOps<E, W>::Accumulate(acc, __builtin_bit_cast(Pack<S, W>, raw[k][i]), one);
            }
        }
        parked[k * lanes + threadIdx.x] = __builtin_bit_cast(U32x4, PackOps<E, W>::Narrow(acc));
    }
    __syncthreads();
#pragma unroll
    for (uint32_t k = 0; k < kPerWave; ++k) {
        if (wave + k * waves < nDst) {
            HCCL_AMD_GLOBAL U32x4* const out = reinterpret_cast<HCCL_AMD_GLOBAL U32x4*>(to[k]) + first + lane;
            for (uint32_t t = 0; t < 2 * waves; ++t) {
                __builtin_nontemporal_store(parked[t * 64 + lane], out + t * 64);
            }
        }
    }
}

// The same for nine to sixteen leaves or destinations: one tile per wavefront, both batches of eight loads issued
// before the first fold, whole workgroups only (a vector count that is a multiple of 64 * waves, no elements behind
// the last vector; no bounds checks).  With two wavefronts a wavefront stores to up to eight destinations.
template <class E>
__global__ __launch_bounds__(64 * kDirectFoldMaxWaves) void DirectFoldWideKernel(const DirectFoldArgs a)
{
    using S = typename E::S;
    constexpr int W = 16 / sizeof(S);
    constexpr int kLeaves = static_cast<int>(kDirectFoldWideLeaves);
    constexpr uint32_t kPerWave = kDirectFoldWideDst / 2;
    static_assert(kLeaves == 16, "two batches of eight loads");
    extern __shared__ uint32_t accStack[];
    U32x4* const parked = reinterpret_cast<U32x4*>(accStack);
    const uint32_t wave = Uniform(threadIdx.x >> 6);
    const uint32_t lane = threadIdx.x & 63u;
    uint64_t leaf[kLeaves];
#pragma unroll
    for (int i = 0; i < kLeaves; ++i) {
        leaf[i] = reinterpret_cast<uint64_t>(a.src[i]);
    }
    uint32_t nSrc = a.nSrc;
    uint32_t nDst = a.nDst;
    uint32_t waves = a.waves;
    ScalarFence8(leaf);
    ScalarFence8(leaf + 8);
    asm volatile("" : "+s"(nSrc), "+s"(nDst), "+s"(waves));
    uint64_t to[kPerWave];
#pragma unroll
    for (uint32_t k = 0; k < kPerWave; ++k) {
        const uint32_t d = wave + k * waves;
        to[k] = reinterpret_cast<uint64_t>(a.dst[d < kDirectFoldWideDst ? d : 0u]);
    }
    float one = 1.0f;
    if constexpr (HasAccumulate<E>::value) {
        one = OpaqueOne();
    }
    const uint64_t first = static_cast<uint64_t>(blockIdx.x) * (waves * 64);   // the workgroup's first vector
    U32x4 raw[kLeaves];
#pragma unroll
    for (int i = 0; i < kLeaves; ++i) {
        if (static_cast<uint32_t>(i) < nSrc) {
            raw[i] = __builtin_nontemporal_load(reinterpret_cast<const HCCL_AMD_GLOBAL U32x4*>(leaf[i]) + first + threadIdx.x);
        }
    }
    IssueFence8(raw);
    IssueFence8(raw + 8);
    AccPack<E, W> acc;
    PackOps<E, W>::Init(acc, __builtin_bit_cast(Pack<S, W>, raw[0]));
#pragma unroll
    for (int i = 1; i < kLeaves; ++i) {
        if (static_cast<uint32_t>(i) < nSrc) {
            PackOps<E, W>::Accumulate(acc, __builtin_bit_cast(Pack<S, W>, raw[i]), one);
        }
    }
    parked[threadIdx.x] = __builtin_bit_cast(U32x4, PackOps<E, W>::Narrow(acc));
    __syncthreads();
#pragma unroll
    for (uint32_t k = 0; k < kPerWave; ++k) {
        if (wave + k * waves < nDst) {
            HCCL_AMD_GLOBAL U32x4* const out = reinterpret_cast<HCCL_AMD_GLOBAL U32x4*>(to[k]) + first + lane;
            for (uint32_t t = 0; t < waves; ++t) {
                __builtin_nontemporal_store(parked[t * 64 + lane], out + t * 64);
            }
        }
    }
}

// The same for exactly eight leaves, eight destinations, eight wavefronts per workgroup and a vector count that
// fills every workgroup (a multiple of 512, or of 1024 with K = 2 tiles per wavefront; no elements behind the last
// vector): straight-line code without a count or bounds check.  At a few MiB per rank every wavefront of the launch
// is resident at once and shares its SIMD's issue slots with three others, so the instructions between a
// wavefront's start and its first load, and between the barrier and its stores, are latency that nothing hides.
template <class E, int K>
__global__ __launch_bounds__(64 * 8) void DirectFoldExactKernel(const DirectFoldArgs a)
{
    using S = typename E::S;
    constexpr int W = 16 / sizeof(S);
    constexpr int kLeaves = 8;
    constexpr uint32_t kWaves = 8;
    constexpr uint32_t kLanes = kWaves * 64;
    static_assert(kDirectFoldMaxLeaves == 8 && kDirectFoldMaxDst == 8 && kDirectFoldMaxWaves == 8, "eight of each");
    static_assert(K == 1 || K == 2, "one or two tiles per wavefront");
    extern __shared__ uint32_t accStack[];
    U32x4* const parked = reinterpret_cast<U32x4*>(accStack);
    const uint32_t wave = Uniform(threadIdx.x >> 6);
    const uint32_t lane = threadIdx.x & 63u;
    uint64_t leaf[kLeaves];
#pragma unroll
    for (int i = 0; i < kLeaves; ++i) {
        leaf[i] = reinterpret_cast<uint64_t>(a.src[i]);
    }
    ScalarFence8(leaf);
    const uint64_t to = reinterpret_cast<uint64_t>(a.dst[wave]);   // first used behind the barrier
    float one = 1.0f;
    if constexpr (HasAccumulate<E>::value) {
        one = OpaqueOne();
    }
    // the workgroup's first vector; with two tiles per wavefront the second round of eight tiles follows the first
    const uint64_t first = static_cast<uint64_t>(blockIdx.x) * (K * kLanes);
    U32x4 raw[K][kLeaves];
#pragma unroll
    for (int k = 0; k < K; ++k) {
#pragma unroll
        for (int i = 0; i < kLeaves; ++i) {
            raw[k][i] = __builtin_nontemporal_load(reinterpret_cast<const HCCL_AMD_GLOBAL U32x4*>(leaf[i]) + first +
                                                   k * kLanes + threadIdx.x);
        }
    }
#pragma unroll
    for (int k = 0; k < K; ++k) {
        IssueFence8(raw[k]);
    }
#pragma unroll
    for (int k = 0; k < K; ++k) {
        AccPack<E, W> acc;
        PackOps<E, W>::Init(acc, __builtin_bit_cast(Pack<S, W>, raw[k][0]));
#pragma unroll
        for (int i = 1; i < kLeaves; ++i) {
            PackOps<E, W>::Accumulate(acc, __builtin_bit_cast(Pack<S, W>, raw[k][i]), one);
        }
        parked[k * kLanes + threadIdx.x] = __builtin_bit_cast(U32x4, PackOps<E, W>::Narrow(acc));
    }
    __syncthreads();
    HCCL_AMD_GLOBAL U32x4* const out = reinterpret_cast<HCCL_AMD_GLOBAL U32x4*>(to) + first + lane;
#pragma unroll
    for (uint32_t t = 0; t < K * kWaves; ++t) {
        __builtin_nontemporal_store(parked[t * 64 + lane], out + t * 64);
    }
}

using DirectFoldFn = void (*)(const DirectFoldArgs);

}  // namespace detail

// One translation unit per data type defines its selector (nullptr = combination not offered).
detail::ReduceKernelFn SelectReduceI8(int op, int batch);
detail::ReduceKernelFn SelectReduceI16(int op, int batch);
detail::ReduceKernelFn SelectReduceI32(int op, int batch);
detail::ReduceKernelFn SelectReduceI64(int op, int batch);
detail::ReduceKernelFn SelectReduceU64(int op, int batch);
detail::ReduceKernelFn SelectReduceF16(int op, int batch);
detail::ReduceKernelFn SelectReduceBf16(int op, int batch);
detail::ReduceKernelFn SelectReduceF32(int op, int batch);
detail::ReduceKernelFn SelectReduceF64(int op, int batch);
detail::DirectFoldFn SelectReduceI8Direct(int op, int exact);
detail::DirectFoldFn SelectReduceI16Direct(int op, int exact);
detail::DirectFoldFn SelectReduceI32Direct(int op, int exact);
detail::DirectFoldFn SelectReduceI64Direct(int op, int exact);
detail::DirectFoldFn SelectReduceU64Direct(int op, int exact);
detail::DirectFoldFn SelectReduceF16Direct(int op, int exact);
detail::DirectFoldFn SelectReduceBf16Direct(int op, int exact);
detail::DirectFoldFn SelectReduceF32Direct(int op, int exact);
detail::DirectFoldFn SelectReduceF64Direct(int op, int exact);

#define HCCL_AMD_PICK(T, batch)                                                                \
    ((batch) == 8 ? detail::ReduceKernel<T, 8>                                                 \
                  : (batch) == 16 ? detail::ReduceKernel<T, 16> : detail::ReduceKernel<T, 8, true>)

// 0: any counts; 1 / 2: eight of everything, one / two tiles per wavefront; 3: any counts, two tiles per wavefront;
// 4: up to sixteen leaves and destinations
#define HCCL_AMD_PICK_DIRECT(T, exact)                                                              \
    ((exact) == 1 ? detail::DirectFoldExactKernel<T, 1>                                             \
     : (exact) == 2 ? detail::DirectFoldExactKernel<T, 2>                                           \
     : (exact) == 3 ? detail::DirectFoldTwoTileKernel<T>                                            \
     : (exact) == 4 ? detail::DirectFoldWideKernel<T> : detail::DirectFoldKernel<T>)

#define HCCL_AMD_DEFINE_SELECT4(NAME, SUM_T, PROD_T, MAX_T, MIN_T)                 \
    detail::ReduceKernelFn NAME(int op, int batch)                                \
    {                                                                             \
        switch (op) {                                                             \
            case detail::kSum: return HCCL_AMD_PICK(SUM_T, batch);                \
            case detail::kProd: return HCCL_AMD_PICK(PROD_T, batch);              \
            case detail::kMax: return HCCL_AMD_PICK(MAX_T, batch);                \
            case detail::kMin: return HCCL_AMD_PICK(MIN_T, batch);                \
            default: return nullptr;                                              \
        }                                                                         \
    }                                                                             \
    detail::DirectFoldFn NAME##Direct(int op, int exact)                         \
    {                                                                             \
        switch (op) {                                                             \
            case detail::kSum: return HCCL_AMD_PICK_DIRECT(SUM_T, exact);         \
            case detail::kProd: return HCCL_AMD_PICK_DIRECT(PROD_T, exact);       \
            case detail::kMax: return HCCL_AMD_PICK_DIRECT(MAX_T, exact);         \
            case detail::kMin: return HCCL_AMD_PICK_DIRECT(MIN_T, exact);         \
            default: return nullptr;                                              \
        }                                                                         \
    }

#define HCCL_AMD_DEFINE_SELECT3(NAME, SUM_T, MAX_T, MIN_T)                         \
    detail::ReduceKernelFn NAME(int op, int batch)                                \
    {                                                                             \
        switch (op) {                                                             \
            case detail::kSum: return HCCL_AMD_PICK(SUM_T, batch);                \
            case detail::kMax: return HCCL_AMD_PICK(MAX_T, batch);                \
            case detail::kMin: return HCCL_AMD_PICK(MIN_T, batch);                \
            default: return nullptr;                                              \
        }                                                                         \
    }                                                                             \
    detail::DirectFoldFn NAME##Direct(int op, int exact)                         \
    {                                                                             \
        switch (op) {                                                             \
            case detail::kSum: return HCCL_AMD_PICK_DIRECT(SUM_T, exact);         \
            case detail::kMax: return HCCL_AMD_PICK_DIRECT(MAX_T, exact);         \
            case detail::kMin: return HCCL_AMD_PICK_DIRECT(MIN_T, exact);         \
            default: return nullptr;                                              \
        }                                                                         \
    }

}  // namespace hccl_amd
