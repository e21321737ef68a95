// Slice-copy (AllGather / AllGatherV) and displacement-driven pack/unpack (AlltoAllV) for gfx950.
//
// Both are pure HBM streaming: every payload byte is read once with a 128-bit load and written once
// per destination with a 128-bit store.  Work is cut into tiles of one vector per lane and every tile
// is its own workgroup, so that the workgroups in flight at any moment cover a compact window of
// addresses (looping workgroups that stride over the whole range keep many more DRAM pages open and
// measure 15-20 % slower on this part).  Tiles also load-balance segments of wildly different length
// (a Zipf-distributed token routing table) over the whole chip.  The tile -> segment map comes from
// host-built prefix and hint tables that a workgroup searches with a handful of scalar loads: with only
// one vector per lane in flight, anything the lanes have to wait for before their load is issued (vector
// loads of tables, cross-lane scans) shows up directly as lost bandwidth.
//
// Displacements are in elements, so a segment's source and destination generally sit at different
// offsets from a 16-byte boundary.  For such irregular segments the lanes load the aligned 16-byte
// vectors that cover the tile's source bytes, and every lane rebuilds the vector it has to store from
// its own vector and its right-hand neighbour's (a DPP wavefront shift, no LDS, no barrier) with a
// byte funnel shift.  At most 15 bytes at either end of a tile move byte by byte.
//
// Data movement follows the reference's templates:
//   AllGather(V): out_d[displs[r] ...] = in_r   (ins_temp_all_gather_mesh_1D.cc:249-423,
//                                                ins_temp_all_gather_v_mesh_1D.cc:242-310)
//   AlltoAllV   : recv_i[rdispls_i[j] ...] = send_j[sdispls_j[i] ...], sendCounts_j[i] elements
//                 (ins_temp_all_to_all_v_mesh_1D.cc:229-246, 459-611)
#include <hip/hip_runtime.h>

#include <cstdlib>
#include <mutex>

#include "dataplane.h"

// Tables (descriptors, tile prefixes, hints) of the allocation-free AlltoAllV.  Every GPU the library runs on
// holds its own copy of this array at its own address; host code never uses the array's name as an address but
// the pointer hipGetSymbolAddress returns for the current device (A2aScratchOfCurrentDevice).
static __device__ __align__(256) uint8_t scratch[hccl_amd::kA2aScratchBytes];

namespace hccl_amd {
namespace {

typedef uint32_t U32x4 __attribute__((ext_vector_type(4)));

// Payload pointers are rebuilt from integers; telling the compiler they are global memory keeps the
// accesses off the flat path.
//
// Cache policy: a tile is loaded non-temporally and its 16-byte vectors are written through at system scope, the
// fastest pair for one read stream next to one or several write streams.
template <typename V>
__device__ __forceinline__ V LoadVec(const void* p)
{
    return __builtin_nontemporal_load((const __attribute__((address_space(1))) V*)p);
}
template <typename V>
__device__ __forceinline__ void StoreVec(V v, void* p)
{
    if constexpr (sizeof(V) == 16) {
        StoreStream16(p, __builtin_bit_cast(StreamVec, v));
    } else {
        __builtin_nontemporal_store(v, (__attribute__((address_space(1))) V*)p);
    }
}

// Tables are read through the constant address space so that the loads are scalar.
typedef const uint8_t __attribute__((address_space(4))) * K8;
typedef const uint32_t __attribute__((address_space(4))) * K32;
typedef const uint64_t __attribute__((address_space(4))) * K64;

// First segment whose inclusive tile prefix exceeds `tile`; zero-length segments are never returned.
template <class HintPtr, class EndPtr>
__device__ __forceinline__ uint32_t FindSegment(uint32_t tile, uint32_t shift, HintPtr hint, EndPtr tileEnd)
{
    const uint32_t k = tile >> shift;
    uint32_t lo = hint[k];
    uint32_t hi = hint[k + 1];
    while (lo < hi) {
        const uint32_t mid = (lo + hi) >> 1;
        if (tile >= tileEnd[mid]) {
            lo = mid + 1;
        } else {
            hi = mid;
        }
    }
    return lo;
}

// 1 when tileEnd <= tile, else 0, for tile < 2^31: in scalar arithmetic (a comparison result that is added up
// as a number would travel through a vector register and back for every term).
__device__ __forceinline__ uint32_t EndsAtOrBefore(uint32_t tileEnd, uint32_t tile)
{
    const uint32_t above = tile + 1u;
    return (tileEnd > above ? tileEnd : above) - (tileEnd > tile ? tileEnd : tile);
}

// Four output dwords from five input dwords, dropping `shift` (0..3) leading bytes.
__device__ __forceinline__ U32x4 Funnel(uint32_t w0, uint32_t w1, uint32_t w2, uint32_t w3, uint32_t w4, uint32_t shift)
{
    if (shift == 0) {
        return U32x4{w0, w1, w2, w3};
    }
    return U32x4{__builtin_amdgcn_alignbyte(w1, w0, shift), __builtin_amdgcn_alignbyte(w2, w1, shift),
                 __builtin_amdgcn_alignbyte(w3, w2, shift), __builtin_amdgcn_alignbyte(w4, w3, shift)};
}

// Tiles of a segment are cut so that every tile but the first starts on a 128-byte line of the
// destination: tile k covers bytes [k * kTile - lead, (k + 1) * kTile - lead) of the segment, clipped
// to [0, len), where lead is the offset of the segment's first destination byte within its line.  A
// wavefront whose 1 KiB of stores straddles nine lines instead of eight costs write bandwidth.
template <uint32_t kTile>
__device__ __forceinline__ void TileRange(uint32_t k, uint32_t lead, uint64_t len, uint64_t* off, uint32_t* bytes)
{
    const uint64_t begin = k == 0 ? 0 : static_cast<uint64_t>(k) * kTile - lead;
    const uint32_t cap = k == 0 ? kTile - lead : kTile;
    *off = begin;
    *bytes = static_cast<uint32_t>(len - begin < cap ? len - begin : cap);
}

// Lane i gets `v` of lane i + 1; lane 63 keeps `last`.  Must run with the whole wavefront active.
__device__ __forceinline__ U32x4 NextLane(U32x4 v, U32x4 last)
{
    constexpr int kWaveShl1 = 0x130;   // DPP control: wavefront shift left by one lane
    U32x4 r;
    r.x = __builtin_amdgcn_update_dpp(last.x, v.x, kWaveShl1, 0xF, 0xF, false);
    r.y = __builtin_amdgcn_update_dpp(last.y, v.y, kWaveShl1, 0xF, 0xF, false);
    r.z = __builtin_amdgcn_update_dpp(last.z, v.z, kWaveShl1, 0xF, 0xF, false);
    r.w = __builtin_amdgcn_update_dpp(last.w, v.w, kWaveShl1, 0xF, 0xF, false);
    return r;
}

// Calls store(address) for the destinations d < nDst, address = pointer of destination d + dOff.  The pointers
// come in batches: kBatch scalar loads go out together (ptrOf(d) for a run of d, clamped to the last one) and
// the stores follow back to back.  A loop that fetched one pointer per store would put a scalar-load round
// trip between any two stores of a wavefront.  With kStatic the batch is ptrOf(0 .. kBatch - 1) exactly, so
// that ptrOf may index registers.
// Waits until at most `pace` of the wavefront's memory operations are outstanding (3 and above: no wait).
__device__ __forceinline__ void PaceStores(uint32_t pace)
{
    if (pace == 0) {
        __builtin_amdgcn_s_waitcnt(0x0F70);
    } else if (pace == 1) {
        __builtin_amdgcn_s_waitcnt(0x0F71);
    } else if (pace == 2) {
        __builtin_amdgcn_s_waitcnt(0x0F72);
    }
}

template <int kBatch, bool kStatic, class PtrFn, class StoreFn>
__device__ __forceinline__ void ForEachDst(uint32_t nDst, uint64_t dOff, uint32_t pace, PtrFn ptrOf, StoreFn store)
{
    static_assert(kBatch == 1 || kBatch == 4 || kBatch == 8, "the fences below name every pointer of a batch");
    for (uint32_t base = 0; base < nDst; base += kBatch) {
        uint64_t ptr[kBatch];
#pragma unroll
        for (uint32_t k = 0; k < static_cast<uint32_t>(kBatch); ++k) {
            if constexpr (kStatic) {
                ptr[k] = ptrOf(k);
            } else {
                ptr[k] = ptrOf(base + k < nDst ? base + k : nDst - 1);
            }
        }
        if constexpr (kBatch == 4) {
            asm volatile("" : "+s"(ptr[0]), "+s"(ptr[1]), "+s"(ptr[2]), "+s"(ptr[3]));
        } else if constexpr (kBatch == 8) {
            asm volatile("" : "+s"(ptr[0]), "+s"(ptr[1]), "+s"(ptr[2]), "+s"(ptr[3]), "+s"(ptr[4]), "+s"(ptr[5]),
                              "+s"(ptr[6]), "+s"(ptr[7]));
        }
#pragma unroll
        for (uint32_t k = 0; k < static_cast<uint32_t>(kBatch); ++k) {
            if (base + k < nDst) {
                store(reinterpret_cast<uint8_t*>(ptr[k] + dOff));
                PaceStores(pace);
            }
        }
        if constexpr (kStatic) {
            break;
        }
    }
}

// A loaded value is made ready here, once, before the stores that take it: where each store sits in a block of
// its own the compiler would otherwise wait in front of every one of them for all outstanding memory
// operations, the previous store included, and a wavefront's stores would go out one round trip at a time.
__device__ __forceinline__ void Ready(U32x4& v) { asm volatile("" : "+v"(v)); }
__device__ __forceinline__ void Ready(uint32_t& v) { asm volatile("" : "+v"(v)); }

// Copies one tile (bytes <= T * 16) from src to ptrOf(d) + dOff, d < nDst, one 16-byte vector per lane.  The
// stores to destination 0 are 16-byte aligned; those to the other destinations are too when they share its
// offset from a 16-byte boundary (the usual case) and are unaligned 128-bit stores otherwise.  Must be called
// by all T threads of the workgroup.
template <int T, int MODE, int kBatch, bool kStatic, class PtrFn>
__device__ __forceinline__ void CopyTile(const uint8_t* src, uint32_t bytes, uint32_t nDst, uint64_t dOff, uint32_t pace,
                                         PtrFn ptrOf)
{
    const uint32_t idx = threadIdx.x;
    if (MODE == COPY_ALIGNED) {
        if (idx < bytes / 16u) {
            U32x4 v = LoadVec<U32x4>(reinterpret_cast<const U32x4*>(src) + idx);
            Ready(v);
            ForEachDst<kBatch, kStatic>(nDst, dOff, pace, ptrOf, [&](uint8_t* dst) {
                StoreVec<U32x4>(v, reinterpret_cast<U32x4*>(dst) + idx);
            });
        }
        return;
    }
    const uint32_t dMis = static_cast<uint32_t>((ptrOf(0) + dOff) & 15u);
    uint32_t head = (16u - dMis) & 15u;     // bytes before the first aligned destination vector
    head = head < bytes ? head : bytes;
    const uint32_t nVec = (bytes - head) / 16u;   // <= T
    const uint32_t bodyEnd = head + nVec * 16u;
    const uint8_t* sBody = src + head;
    const uint32_t sMis = MODE == COPY_CONGRUENT ? 0u : static_cast<uint32_t>(reinterpret_cast<uint64_t>(sBody) & 15u);

    U32x4 out = {0, 0, 0, 0};
    if (sMis == 0) {
        if (idx < nVec) {
            out = LoadVec<U32x4>(reinterpret_cast<const U32x4*>(sBody) + idx);
        }
    } else if (nVec != 0) {
        // Irregular: lane i loads the aligned vector i that covers the start of its output and takes
        // vector i + 1 from its right-hand neighbour with a wavefront shift; the last lane of a wavefront
        // has no neighbour and loads that vector itself.  A byte funnel shift joins the two.
        const U32x4* s = reinterpret_cast<const U32x4*>(sBody - sMis);
        U32x4 a = {0, 0, 0, 0};
        U32x4 b = {0, 0, 0, 0};
        if (idx <= nVec) {
            a = LoadVec<U32x4>(s + idx);
        }
        if ((idx & 63u) == 63u && idx < nVec) {
            b = LoadVec<U32x4>(s + idx + 1);
        }
        b = NextLane(a, b);
        const uint32_t shift = sMis & 3u;    // bytes to skip inside a dword
        switch (sMis >> 2) {                 // whole dwords to skip (uniform)
            case 0: out = Funnel(a.x, a.y, a.z, a.w, b.x, shift); break;
            case 1: out = Funnel(a.y, a.z, a.w, b.x, b.y, shift); break;
            case 2: out = Funnel(a.z, a.w, b.x, b.y, b.z, shift); break;
            default: out = Funnel(a.w, b.x, b.y, b.z, b.w, shift); break;
        }
    }
    // The edge byte (up to 15 in front of the body and up to 15 behind it) is requested before the body is stored.
    const uint32_t edge = head + (bytes - bodyEnd);
    const uint32_t edgeAt = idx < head ? idx : bodyEnd + (idx - head);
    uint32_t edgeByte = 0;
    if (idx < edge) {
        edgeByte = LoadVec<uint8_t>(src + edgeAt);
    }
    Ready(out);
    Ready(edgeByte);
    if (idx < nVec) {
        ForEachDst<kBatch, kStatic>(nDst, dOff, pace, ptrOf, [&](uint8_t* dst) {
            StoreVec<U32x4>(out, reinterpret_cast<U32x4*>(dst + head) + idx);
        });
    }
    if (idx < edge) {
        ForEachDst<kBatch, kStatic>(nDst, dOff, pace, ptrOf, [&](uint8_t* dst) {
            StoreVec<uint8_t>(static_cast<uint8_t>(edgeByte), dst + edgeAt);
        });
    }
}

// ---- AllGather / AllGatherV --------------------------------------------------------------------
// Workgroup b copies tile b of the segment list held in the kernel arguments to every destination.
//
// A wavefront has one 16-byte vector per lane in flight, so whatever it waits for before that load is issued is
// lost bandwidth.  Everything a wavefront needs therefore comes in with two rounds of scalar loads of the kernel
// arguments: the first brings the tile prefixes (the tile -> segment map is a branch-free count over them), the
// second what the segment index selects.
template <int T, int MODE>
__global__ __launch_bounds__(T) void BcastCopyKernel(const BcastCopyArgs args)
{
    constexpr uint32_t kTile = T * 16u;
    // First round: everything that does not depend on the segment.
    uint32_t nDst = args.nDst;
    uint32_t nSegPadded = args.nSegPadded;
    uint32_t ends[16];
#pragma unroll
    for (uint32_t k = 0; k < 16; ++k) {
        ends[k] = args.tileEnd[k];
    }
    asm volatile("" : "+s"(nDst), "+s"(nSegPadded));
    asm volatile("" : "+s"(ends[0]), "+s"(ends[1]), "+s"(ends[2]), "+s"(ends[3]), "+s"(ends[4]), "+s"(ends[5]),
                      "+s"(ends[6]), "+s"(ends[7]), "+s"(ends[8]), "+s"(ends[9]), "+s"(ends[10]), "+s"(ends[11]),
                      "+s"(ends[12]), "+s"(ends[13]), "+s"(ends[14]), "+s"(ends[15]));
    const uint32_t tile = blockIdx.x;
    // Number of segments that end at or before this tile = index of the tile's segment (prefixes past the last
    // segment hold 0xFFFFFFFF; empty segments repeat their predecessor's prefix and are skipped by the count).
    uint32_t seg = 0;
#pragma unroll
    for (uint32_t k = 0; k < 16; ++k) {
        seg += EndsAtOrBefore(ends[k], tile);
    }
    for (uint32_t i = 16; i < nSegPadded; i += 16) {
#pragma unroll
        for (uint32_t k = 0; k < 16; ++k) {
            seg += EndsAtOrBefore(args.tileEnd[i + k], tile);
        }
    }
    const uint32_t segFirst = seg == 0 ? 0u : args.tileEnd[seg - 1];
    uint64_t len = args.len[seg];
    uint64_t srcBase = reinterpret_cast<uint64_t>(args.src[seg]);
    uint64_t segDstOff = args.dstOff[seg];
    asm volatile("" : "+s"(srcBase), "+s"(len), "+s"(segDstOff));   // second round: all requested together
    const uint32_t lead = TileLead(args.leadBase + segDstOff);
    uint64_t off;
    uint32_t bytes;
    TileRange<kTile>(tile - segFirst, lead, len, &off, &bytes);
    const uint8_t* src = reinterpret_cast<const uint8_t*>(srcBase + off);
    const uint64_t dOff = segDstOff + off;
    CopyTile<T, MODE, 8, false>(src, bytes, nDst, dOff, args.pace,
                                [&](uint32_t d) { return reinterpret_cast<uint64_t>(args.dst[d]); });
}

// ---- AlltoAllV -------------------------------------------------------------------------------------
// Workgroup b copies tile b of the descriptor list in device memory (one source, one destination).
template <int T, int MODE>
__global__ __launch_bounds__(T) void A2aCopyKernel(const A2aArgs args)
{
    constexpr uint32_t kTile = T * 16u;
    // Rounds of scalar loads in front of the tile's vector load: the arguments; the two hints; the search steps
    // (usually none or one); the descriptor.  Each round's values are requested together.
    uint64_t tileEndAddr = reinterpret_cast<uint64_t>(args.tileEnd);
    uint64_t hintAddr = reinterpret_cast<uint64_t>(args.hint);
    uint64_t descAddr = reinterpret_cast<uint64_t>(args.desc);
    uint32_t hintShift = args.hintShift;
    asm volatile("" : "+s"(tileEndAddr), "+s"(hintAddr), "+s"(descAddr), "+s"(hintShift));
    const K32 tileEnd = (K32)(uintptr_t)tileEndAddr;
    const K32 hint = (K32)(uintptr_t)hintAddr;
    const uint32_t tile = blockIdx.x;
    const uint32_t seg = FindSegment(tile, hintShift, hint, tileEnd);
    const K64 desc = (K64)(uintptr_t)descAddr + static_cast<uint64_t>(seg) * kA2aDescWords;
    uint64_t srcBase = desc[0];
    uint64_t dstBase = desc[1];
    uint64_t len = desc[2];
    uint64_t firstTile = desc[3];
    asm volatile("" : "+s"(srcBase), "+s"(dstBase), "+s"(len), "+s"(firstTile));
    uint64_t off;
    uint32_t bytes;
    TileRange<kTile>(tile - static_cast<uint32_t>(firstTile), TileLead(dstBase), len, &off, &bytes);
    const uint8_t* src = reinterpret_cast<const uint8_t*>(srcBase + off);
    CopyTile<T, MODE, 1, true>(src, bytes, 1u, off, 3u, [&](uint32_t) { return dstBase; });
}

template <int T>
hipError_t LaunchBcastT(const BcastCopyArgs& a, uint32_t mode, uint32_t tiles, hipStream_t stream)
{
    switch (mode) {
        case COPY_ALIGNED: hipLaunchKernelGGL((BcastCopyKernel<T, COPY_ALIGNED>), dim3(tiles), dim3(T), 0, stream, a); break;
        case COPY_CONGRUENT: hipLaunchKernelGGL((BcastCopyKernel<T, COPY_CONGRUENT>), dim3(tiles), dim3(T), 0, stream, a); break;
        default: hipLaunchKernelGGL((BcastCopyKernel<T, COPY_GENERAL>), dim3(tiles), dim3(T), 0, stream, a); break;
    }
    return hipGetLastError();
}

template <int T>
hipError_t LaunchA2aT(const A2aArgs& a, uint32_t tiles, hipStream_t stream)
{
    switch (a.mode) {
        case COPY_ALIGNED: hipLaunchKernelGGL((A2aCopyKernel<T, COPY_ALIGNED>), dim3(tiles), dim3(T), 0, stream, a); break;
        case COPY_CONGRUENT: hipLaunchKernelGGL((A2aCopyKernel<T, COPY_CONGRUENT>), dim3(tiles), dim3(T), 0, stream, a); break;
        default: hipLaunchKernelGGL((A2aCopyKernel<T, COPY_GENERAL>), dim3(tiles), dim3(T), 0, stream, a); break;
    }
    return hipGetLastError();
}

// ---- fan-out of a cached range ------------------------------------------------------------------
// Wavefront y of workgroup b copies tile b (64 vectors) of the source to destination y: one plain load (the first
// wavefront of a tile brings it into the caches, the others find it there) and one non-temporal store.  A
// wavefront with a single store stream is the fastest way to write on this part (sixteen streams from sixteen
// wavefronts: 0.89 of the HBM peak, all sixteen from one wavefront: 0.72), and with next to no preamble the extra
// wavefronts cost little.  Source and destinations share their offset from a 16-byte boundary: up to 15 bytes in
// front of the aligned body and up to 15 behind it move byte by byte, and the body's vectors are dealt to the
// lanes shifted by `lead`, so that every wavefront covers whole 128-byte lines.
constexpr uint32_t kFanOutWaves = 16;
static_assert(kFanOutWaves <= static_cast<uint32_t>(kMaxRanks), "a wavefront reads dst[wave] before it knows nDst");
// kStreamLoad: the source is loaded non-temporally (the caller says when, see launch_policy.h); a kernel of its own, since the
// compiler merges the two flavours of the load into a plain one when they sit in the branches of one kernel.
template <bool kStreamLoad>
__global__ __launch_bounds__(64 * kFanOutWaves) void FanOutKernel(const FanOutArgs args)
{
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.y);
    // Everything the wavefront needs, requested in one round of scalar loads (the workgroup has at most sixteen
    // wavefronts, so dst[wave] is an entry of the table whatever nDst is).
    uint32_t nDst = args.nDst;
    uint64_t dstAddr = reinterpret_cast<uint64_t>(args.dst[wave]);
    uint64_t srcAddr = reinterpret_cast<uint64_t>(args.src);
    uint64_t bytes = args.bytes;
    asm volatile("" : "+s"(nDst), "+s"(dstAddr), "+s"(srcAddr), "+s"(bytes));
    if (wave >= nDst) {
        return;
    }
    const uint32_t mis = static_cast<uint32_t>(srcAddr & 15u);
    uint64_t head = mis ? 16u - mis : 0u;
    head = head < bytes ? head : bytes;
    const uint64_t nVec = (bytes - head) >> 4;
    const uint32_t lead = static_cast<uint32_t>(((srcAddr + head) >> 4) & 7u);
    const uint64_t u = static_cast<uint64_t>(blockIdx.x) * 64u + threadIdx.x;
    if (u >= lead && u < nVec + lead) {
        const uint64_t at = head + ((u - lead) << 4);
        U32x4 v;
        if constexpr (kStreamLoad) {
            v = __builtin_nontemporal_load((const __attribute__((address_space(1))) U32x4*)(srcAddr + at));
        } else {
            v = *((const __attribute__((address_space(1))) U32x4*)(srcAddr + at));
        }
        __builtin_nontemporal_store(v, (__attribute__((address_space(1))) U32x4*)(dstAddr + at));
    }
    const uint64_t bodyEnd = head + (nVec << 4);
    const uint32_t edge = static_cast<uint32_t>(head + (bytes - bodyEnd));   // < 32
    if (blockIdx.x == 0 && threadIdx.x < edge) {
        const uint64_t at = threadIdx.x < head ? threadIdx.x : bodyEnd + (threadIdx.x - head);
        const uint8_t byte = *((const __attribute__((address_space(1))) uint8_t*)(srcAddr + at));
        *((__attribute__((address_space(1))) uint8_t*)(dstAddr + at)) = byte;
    }
}

// One argument-borne piece of a table image: words[0 .. nWords) go to table[firstWord ...].
constexpr uint32_t kChunkWords = 448;
struct TableChunk {
    uint32_t firstWord;
    uint32_t nWords;
    uint64_t words[kChunkWords];
};

__global__ __launch_bounds__(64) void TableWriteKernel(uint64_t* table, const TableChunk chunk)
{
    const uint32_t i = blockIdx.x * 64u + threadIdx.x;
    if (i < chunk.nWords) {
        table[chunk.firstWord + i] = chunk.words[i];
    }
}

// Writes one word: the marks in front of and behind a collective's kernels on its launch stream.
__global__ __launch_bounds__(64) void MarkKernel(uint64_t* word, uint64_t value)
{
    if (threadIdx.x == 0) {
        *word = value;
    }
}

// Up to eight equally long segments into one destination, everything on 16-byte boundaries and every segment's place
// in the destination on a 128-byte line, described by the arguments alone: segment blockIdx.y, 1 KiB per wavefront.
// A copy with one read and one write stream moves its kilobyte in two memory instructions; the general kernel's way
// to a tile (tile prefixes, hints, alignment cases) is a few hundred instructions per wavefront, which at 128 MiB is
// a quarter of the launch (128 MiB: 52 us against 40 us; 256 MiB: 95 against 80).
constexpr uint32_t kDirectCopyMaxSeg = 8;
struct DirectCopyArgs {
    const void* src[kDirectCopyMaxSeg];
    void* dst[kDirectCopyMaxSeg];   // the segment's place in the destination
    uint64_t nVec;                  // 16-byte vectors per segment
};

__global__ __launch_bounds__(64) void DirectCopyKernel(const DirectCopyArgs a)
{
    const uint32_t j = blockIdx.y;
    const uint64_t u = static_cast<uint64_t>(blockIdx.x) * 64 + threadIdx.x;
    if (u >= a.nVec) {
        return;
    }
    const U32x4 v = LoadVec<U32x4>(static_cast<const U32x4*>(a.src[j]) + u);
    StoreVec<U32x4>(v, static_cast<U32x4*>(a.dst[j]) + u);
}

constexpr int kMaxDevices = 64;
std::mutex g_scratchMu;
uint8_t* g_scratchPtr[kMaxDevices] = {};

}  // namespace

hipError_t A2aScratchOfCurrentDevice(uint8_t** ptr)
{
    int device = -1;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) {
        return e;
    }
    if (device < 0 || device >= kMaxDevices) {
        return hipErrorInvalidDevice;
    }
    std::lock_guard<std::mutex> lock(g_scratchMu);
    if (g_scratchPtr[device] == nullptr) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) {
            return e;
        }
        g_scratchPtr[device] = static_cast<uint8_t*>(p);
    }
    *ptr = g_scratchPtr[device];
    return hipSuccess;
}

hipError_t LaunchMark(uint64_t* word, uint64_t value, hipStream_t stream)
{
    hipLaunchKernelGGL(MarkKernel, dim3(1), dim3(64), 0, stream, word, value);
    return hipGetLastError();
}

hipError_t LaunchTableWrite(uint8_t* table, const uint64_t* image, uint32_t nWords, hipStream_t stream)
{
    TableChunk chunk = {};
    for (uint32_t first = 0; first < nWords; first += kChunkWords) {
        chunk.firstWord = first;
        chunk.nWords = nWords - first < kChunkWords ? nWords - first : kChunkWords;
        for (uint32_t i = 0; i < chunk.nWords; ++i) {
            chunk.words[i] = image[first + i];
        }
        hipLaunchKernelGGL(TableWriteKernel, dim3((chunk.nWords + 63u) / 64u), dim3(64), 0, stream,
                           reinterpret_cast<uint64_t*>(table), chunk);
        const hipError_t e = hipGetLastError();
        if (e != hipSuccess) {
            return e;
        }
    }
    return hipSuccess;
}

hipError_t LaunchBcastCopy(const BcastCopyArgs& in, uint32_t tileBytes, hipStream_t stream)
{
    BcastCopyArgs a = in;
    if (a.nDst == 0 || a.nDst > static_cast<uint32_t>(kMaxRanks)) {
        return hipErrorInvalidValue;
    }
    uint64_t misfit = 0;      // non-zero low bits: something is not 16-byte aligned
    bool congruent = true;    // every segment's source shares the offset of the first destination
    const uint64_t dst0 = reinterpret_cast<uint64_t>(a.dst[0]);
    for (uint32_t d = 0; d < a.nDst; ++d) {
        misfit |= reinterpret_cast<uint64_t>(a.dst[d]);
    }
    for (uint32_t j = 0; j < a.nSeg; ++j) {
        if (a.len[j] != 0) {
            const uint64_t s = reinterpret_cast<uint64_t>(a.src[j]);
            misfit |= s | a.dstOff[j] | a.len[j];
            congruent = congruent && ((s ^ (dst0 + a.dstOff[j])) & 15u) == 0;
        }
    }
    const uint32_t mode = !congruent ? COPY_GENERAL : ((misfit & 15u) == 0 ? COPY_ALIGNED : COPY_CONGRUENT);
    // One destination, up to eight equally long aligned segments: the kernel that needs nothing but its arguments.
    // HCCL_AMD_COPY_DIRECT=0 keeps the general kernel (read once per process).
    static const bool directEnv = getenv("HCCL_AMD_COPY_DIRECT") == nullptr || atoi(getenv("HCCL_AMD_COPY_DIRECT")) != 0;
    if (directEnv && tileBytes == 0 && mode == COPY_ALIGNED && a.nDst == 1) {
        DirectCopyArgs d{};
        uint32_t nSeg = 0;
        uint64_t len = 0;
        bool fits = true;
        for (uint32_t j = 0; j < a.nSeg && fits; ++j) {
            if (a.len[j] == 0) {
                continue;
            }
            fits = nSeg < kDirectCopyMaxSeg && (len == 0 || a.len[j] == len) && ((dst0 + a.dstOff[j]) & 127u) == 0;
            if (fits) {
                len = a.len[j];
                d.src[nSeg] = a.src[j];
                d.dst[nSeg] = reinterpret_cast<void*>(dst0 + a.dstOff[j]);
                ++nSeg;
            }
        }
        if (fits && nSeg == 0) {
            return hipSuccess;   // nothing but empty segments
        }
        const uint64_t tiles = ((len >> 4) + 63) / 64;
        if (fits && tiles <= 0x7FFFFFFFull) {
            d.nVec = len >> 4;
            hipLaunchKernelGGL(DirectCopyKernel, dim3(static_cast<uint32_t>(tiles), nSeg), dim3(64), 0, stream, d);
            return hipGetLastError();
        }
    }
    if (tileBytes == 0) {
        // One wavefront per tile, except where lanes realign their source for several destinations: there the
        // larger workgroup measured 1-2 % faster.
        tileBytes = (mode == COPY_GENERAL && a.nDst > 1) ? 4096u : 1024u;
    }
    uint64_t tiles = 0;
    for (uint32_t j = 0; j < a.nSeg; ++j) {
        tiles += TilesOf(a.len[j], dst0 + a.dstOff[j], tileBytes);
        if (tiles > 0x7FFFFFF0ull) {
            return hipErrorInvalidValue;
        }
        a.tileEnd[j] = static_cast<uint32_t>(tiles);
    }
    if (tiles == 0) {
        return hipSuccess;
    }
    a.nSegPadded = (a.nSeg + 15u) & ~15u;
    for (uint32_t j = a.nSeg; j < a.nSegPadded; ++j) {
        a.tileEnd[j] = 0xFFFFFFFFu;
    }
    a.nTiles = static_cast<uint32_t>(tiles);
    a.leadBase = dst0;
    // A wavefront issues a store when at most one earlier store is outstanding (measured best: 0.75 of the HBM
    // peak against 0.72-0.74 with none or two outstanding, or without a limit); HCCL_AMD_COPY_PACE = 0..3 overrides.
    static const int paceEnv = getenv("HCCL_AMD_COPY_PACE") ? atoi(getenv("HCCL_AMD_COPY_PACE")) : -1;
    a.pace = paceEnv >= 0 ? static_cast<uint32_t>(paceEnv) : 1u;
    switch (tileBytes) {
        case 1024: return LaunchBcastT<64>(a, mode, a.nTiles, stream);
        case 4096: return LaunchBcastT<256>(a, mode, a.nTiles, stream);
        case 16384: return LaunchBcastT<1024>(a, mode, a.nTiles, stream);
        default: return hipErrorInvalidValue;
    }
}

bool FanOutTakes(const FanOutArgs& args)
{
    if (args.nDst == 0 || args.nDst > static_cast<uint32_t>(kMaxRanks) || args.bytes == 0 ||
        (args.bytes >> 10) + 2 > 0x7FFFFFFFull) {
        return false;
    }
    for (uint32_t d = 0; d < args.nDst; ++d) {
        if (((reinterpret_cast<uint64_t>(args.dst[d]) ^ reinterpret_cast<uint64_t>(args.src)) & 15u) != 0) {
            return false;
        }
    }
    return true;
}

hipError_t LaunchFanOut(const FanOutArgs& in, bool streamLoad, hipStream_t stream)
{
    if (!FanOutTakes(in)) {
        return hipErrorInvalidValue;
    }
    // vectors of the body plus up to seven lanes skipped in front of it; at least one workgroup for the edge bytes
    const uint64_t vecs = (in.bytes >> 4) + 7;
    const uint32_t tiles = static_cast<uint32_t>((vecs + 63) / 64);
    // One destination per wavefront and as many wavefronts per workgroup as there are: more than sixteen
    // destinations take several launches of equal width (the source stays cached).  Measured at 63 destinations:
    // 0.81 of the HBM peak, against 0.69 for one launch with four destinations per wavefront; and at 15
    // destinations 0.82 in one launch against 0.81 / 0.76 in launches of 8 / 4.
    const uint32_t launches = (in.nDst + kFanOutWaves - 1) / kFanOutWaves;
    const uint32_t perLaunch = (in.nDst + launches - 1) / launches;
    for (uint32_t first = 0; first < in.nDst; first += perLaunch) {
        FanOutArgs a{};
        a.src = in.src;
        a.bytes = in.bytes;
        a.nDst = in.nDst - first < perLaunch ? in.nDst - first : perLaunch;
        for (uint32_t d = 0; d < a.nDst; ++d) {
            a.dst[d] = in.dst[first + d];
        }
        if (streamLoad) {
            hipLaunchKernelGGL(FanOutKernel<true>, dim3(tiles), dim3(64, a.nDst), 0, stream, a);
        } else {
            hipLaunchKernelGGL(FanOutKernel<false>, dim3(tiles), dim3(64, a.nDst), 0, stream, a);
        }
        const hipError_t e = hipGetLastError();
        if (e != hipSuccess) {
            return e;
        }
    }
    return hipSuccess;
}

hipError_t LaunchA2aCopy(const A2aArgs& args, uint32_t nTiles, uint32_t tileBytes, hipStream_t stream)
{
    if (nTiles == 0) {
        return hipSuccess;
    }
    switch (tileBytes) {
        case 1024: return LaunchA2aT<64>(args, nTiles, stream);
        case 4096: return LaunchA2aT<256>(args, nTiles, stream);
        case 16384: return LaunchA2aT<1024>(args, nTiles, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace hccl_amd
