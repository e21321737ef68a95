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
template <typename V>
__device__ __forceinline__ V LoadNt(const void* p)
{
    return __builtin_nontemporal_load((const __attribute__((address_space(1))) V*)p);
}
template <typename V>
__device__ __forceinline__ void StoreNt(V v, void* p)
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

// Copies one tile (bytes <= T * 16) from src to dstOf(d), d < nDst, one 16-byte vector per lane.  The stores
// to dstOf(0) are 16-byte aligned; those to the other destinations are too when they share its offset from a
// 16-byte boundary (the usual case) and are unaligned 128-bit stores otherwise.  Must be called by all T
// threads of the workgroup.
template <int T, int MODE, class DstFn>
__device__ __forceinline__ void CopyTile(const uint8_t* src, uint32_t bytes, uint32_t nDst, DstFn dstOf)
{
    const uint32_t idx = threadIdx.x;
    if (MODE == COPY_ALIGNED) {
        if (idx < bytes / 16u) {
            const U32x4 v = LoadNt<U32x4>(reinterpret_cast<const U32x4*>(src) + idx);
            for (uint32_t d = 0; d < nDst; ++d) {
                StoreNt(v, reinterpret_cast<U32x4*>(dstOf(d)) + idx);
            }
        }
        return;
    }
    const uint32_t dMis = static_cast<uint32_t>(reinterpret_cast<uint64_t>(dstOf(0)) & 15u);
    uint32_t head = (16u - dMis) & 15u;     // bytes before the first aligned destination vector
    head = head < bytes ? head : bytes;
    const uint32_t nVec = (bytes - head) / 16u;   // <= T
    const uint32_t bodyEnd = head + nVec * 16u;
    const uint8_t* sBody = src + head;
    const uint32_t sMis = MODE == COPY_CONGRUENT ? 0u : static_cast<uint32_t>(reinterpret_cast<uint64_t>(sBody) & 15u);

    U32x4 out = {0, 0, 0, 0};
    if (sMis == 0) {
        if (idx < nVec) {
            out = LoadNt<U32x4>(reinterpret_cast<const U32x4*>(sBody) + idx);
        }
    } else if (nVec != 0) {
        // Irregular: lane i loads the aligned vector i that covers the start of its output and takes
        // vector i + 1 from its right-hand neighbour with a wavefront shift; the last lane of a wavefront
        // has no neighbour and loads that vector itself.  A byte funnel shift joins the two.
        const U32x4* s = reinterpret_cast<const U32x4*>(sBody - sMis);
        U32x4 a = {0, 0, 0, 0};
        U32x4 b = {0, 0, 0, 0};
        if (idx <= nVec) {
            a = LoadNt<U32x4>(s + idx);
        }
        if ((idx & 63u) == 63u && idx < nVec) {
            b = LoadNt<U32x4>(s + idx + 1);
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
    if (idx < nVec) {
        for (uint32_t d = 0; d < nDst; ++d) {
            StoreNt(out, reinterpret_cast<U32x4*>(dstOf(d) + head) + idx);
        }
    }
    // Up to 15 bytes in front of the body and up to 15 behind it.
    const uint32_t edge = head + (bytes - bodyEnd);
    if (idx < edge) {
        const uint32_t o = idx < head ? idx : bodyEnd + (idx - head);
        const uint8_t b = LoadNt<uint8_t>(src + o);
        for (uint32_t d = 0; d < nDst; ++d) {
            StoreNt(b, dstOf(d) + o);
        }
    }
}

// ---- AllGather / AllGatherV --------------------------------------------------------------------
// Workgroup b copies tile b of the segment list held in the kernel arguments.
template <int T, int MODE>
__global__ __launch_bounds__(T) void BcastCopyKernel(const BcastCopyArgs args)
{
    constexpr uint32_t kTile = T * 16u;
    const uint32_t tile = blockIdx.x;
    const uint32_t seg = FindSegment(tile, args.hintShift, args.hint, args.tileEnd);
    const uint32_t segFirst = seg == 0 ? 0u : args.tileEnd[seg - 1];
    const uint64_t len = args.len[seg];
    const uint32_t lead = TileLead(reinterpret_cast<uint64_t>(args.dst[0]) + args.dstOff[seg]);
    uint64_t off;
    uint32_t bytes;
    TileRange<kTile>(tile - segFirst, lead, len, &off, &bytes);
    const uint8_t* src = static_cast<const uint8_t*>(args.src[seg]) + off;
    const uint64_t dOff = args.dstOff[seg] + off;
    auto dstOf = [&](uint32_t d) { return static_cast<uint8_t*>(args.dst[d]) + dOff; };
    CopyTile<T, MODE>(src, bytes, args.nDst, dstOf);
}

// ---- AlltoAllV -------------------------------------------------------------------------------------
// Workgroup b copies tile b of the descriptor list in device memory (one source, one destination).
template <int T, int MODE>
__global__ __launch_bounds__(T) void A2aCopyKernel(const A2aArgs args)
{
    constexpr uint32_t kTile = T * 16u;
    const K32 tileEnd = (K32)(uintptr_t)args.tileEnd;
    const K32 hint = (K32)(uintptr_t)args.hint;
    const uint32_t tile = blockIdx.x;
    const uint32_t seg = FindSegment(tile, args.hintShift, hint, tileEnd);
    const K64 desc = (K64)(uintptr_t)args.desc + static_cast<uint64_t>(seg) * kA2aDescWords;
    const uint64_t srcBase = desc[0];
    const uint64_t dstBase = desc[1];
    const uint64_t len = desc[2];
    uint64_t off;
    uint32_t bytes;
    TileRange<kTile>(tile - static_cast<uint32_t>(desc[3]), TileLead(dstBase), len, &off, &bytes);
    const uint8_t* src = reinterpret_cast<const uint8_t*>(srcBase + off);
    uint8_t* dst = reinterpret_cast<uint8_t*>(dstBase + off);
    CopyTile<T, MODE>(src, bytes, 1u, [&](uint32_t) { return dst; });
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
    uint64_t misfit = 0;      // non-zero low bits: something is not 16-byte aligned
    bool congruent = true;    // every segment's source shares the offset of its first destination
    for (uint32_t d = 0; d < a.nDst; ++d) {
        misfit |= reinterpret_cast<uint64_t>(a.dst[d]);
    }
    const uint64_t dst0 = reinterpret_cast<uint64_t>(a.dst[0]);
    for (uint32_t j = 0; j < a.nSeg; ++j) {
        if (a.len[j] != 0) {
            const uint64_t s = reinterpret_cast<uint64_t>(a.src[j]);
            misfit |= s | a.dstOff[j] | a.len[j];
            congruent = congruent && ((s ^ (dst0 + a.dstOff[j])) & 15u) == 0;
        }
    }
    const uint32_t mode = !congruent ? COPY_GENERAL : ((misfit & 15u) == 0 ? COPY_ALIGNED : COPY_CONGRUENT);
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
    uint32_t nHint = 0;
    a.hintShift = BuildTileHints(a.tileEnd, a.nSeg, static_cast<uint32_t>(tiles), kBcastHintMax, a.hint, &nHint);
    const uint32_t nTiles = static_cast<uint32_t>(tiles);
    switch (tileBytes) {
        case 1024: return LaunchBcastT<64>(a, mode, nTiles, stream);
        case 4096: return LaunchBcastT<256>(a, mode, nTiles, stream);
        case 16384: return LaunchBcastT<1024>(a, mode, nTiles, stream);
        default: return hipErrorInvalidValue;
    }
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
