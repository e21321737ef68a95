// Launch descriptors shared by the host layer and the gfx950 kernels of the loopback data plane.
//
// Everything here is plain data that travels in the kernel-argument segment: device pointers,
// element counts and small tables.  No kernel takes a pointer to host memory.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "hccl_types.h"

namespace hccl_amd {

constexpr int kMaxRanks = HCCL_AMD_MAX_RANKS;
constexpr uint32_t kMaxReduceThreads = 256;   // lanes of a reduce workgroup (64, 128 or 256), one 16-byte vector each
// The vectors of a sub-segment are dealt to the lanes shifted by up to kReduceLeadMask positions, so that every
// wavefront's 1 KiB starts on a 1 KiB boundary.  Starting on 128-byte lines only (mask 7) keeps the traffic the same
// but measured 2.5 % slower wherever sub-segments begin off that grid (fp16 RHD over six ranks: 0.75 -> 0.77 of the
// HBM peak with 15 / 31 / 63: 0.754 / 0.764 / 0.770).
constexpr uint32_t kReduceLeadMask = 63;

// ---------------------------------------------------------------------------------------------
// Fold programs
//
// A reduction over N ranks is described by a byte program that fixes the association order and
// which operand of every pairwise step is the accumulator ("dst") and which the incoming value
// ("src"): value = src (+) dst, exactly the roles of the reference's LocalReduce(src, dst)
// (alg_data_trans_wrapper.cc:901-928, 1319-1358).
//
//   0x00..0x3F   fold rank r into the current level (the first operand of a level initialises it)
//   0xC0 | n     n in 1..8: the next n bytes are ranks folded in that order (their loads are issued
//                together, before the first fold)
//   0x80         open a nested level
//   0x81         close the nested level: its value is folded, as src, into the enclosing level
//   0xFF         end of program
// ---------------------------------------------------------------------------------------------
constexpr uint8_t kTokOpen = 0x80;
constexpr uint8_t kTokClose = 0x81;
constexpr uint8_t kTokRun = 0xC0;
constexpr uint8_t kTokEnd = 0xFF;
constexpr int kProgStride = 320;   // upper bound on the byte length of one program
constexpr int kMaxFoldDepth = 8;   // deepest nesting a plan may have
constexpr int kMaxRun = 8;

// Device image of one program (what the kernel reads): the same tree flattened to its leaves in
// evaluation order.  Leaf i folds rank[i]; ctl[i] bit 7 says a nested level opens right before it
// (the enclosing accumulator is parked), ctl[i] bits 0..6 count the levels that close right after it.
constexpr int kDevProgBytes = 160;
constexpr int kDevProgRankOff = 16;   // byte 0 holds the leaf count
constexpr int kDevProgCtlOff = 80;
constexpr uint8_t kCtlOpen = 0x80;

// Geometry of one fused reduce launch.
//
// The logical element range [0, total) is cut into `nGroup` groups of `groupLen` elements (the last
// may be short) and every group into `nSub` sub-segments of `subLen` elements (the last sub-segment
// runs to the end of its group).  Sub-segment (g, c) reads, from every rank t,
//     src[t] + g * srcGroupStride + c * subLen + e
// and writes either to every dst[d], d < nDst, at  g * dstGroupStride + c * subLen + e   (dstOwn == 0)
// or only to dst[g] at  c * subLen + e                                                    (dstOwn == 1).
// Its fold program is number  g * progGroupStride + c * progSubStride.
// The scalars of a launch come first and together (ReduceHot): a workgroup fetches them with one block of scalar
// loads before it does anything else.  Fetched one by one, where the code happens to need them, they were a
// dozen round trips in a row in front of the first vector load of every wavefront.
struct ReduceHot {
    const uint8_t* prog;
    uint64_t total;
    uint64_t groupLen;
    uint64_t subLen;
    uint64_t srcGroupStride;
    uint64_t dstGroupStride;
    uint32_t nGroup;
    uint32_t nSub;
    uint32_t nDst;
    uint32_t dstOwn;
    uint32_t progGroupStride;
    uint32_t progSubStride;
    uint32_t blocksPerSub;   // workgroups per sub-segment: the grid is (blocksPerSub, nSub, nGroup), or one-dimensional with varGroups
    uint32_t vecOk;   // take the 128-bit path (0: element by element, for testing)
    uint32_t threads; // workgroup size of the launch
    uint32_t vecBatch;       // leaves per load batch of the 128-bit path: 8 or 16, or kVecBatchPair (picks the kernel instantiation)
    uint32_t writeThrough;   // 16-byte results leave through StoreStream16 instead of a non-temporal store
    uint32_t leadFromSrc;    // wavefronts start on a 1 KiB boundary of the sources instead of the destination's
    uint32_t storeWaves;     // > 1: workgroups of 64 * storeWaves threads, wavefront 0 folds and wavefront k stores to
                             // destinations k, k + storeWaves, ... (threads must be 64, dstOwn 0); 0 or 1: every wavefront
                             // folds and stores its own tile.  With kStoreWavesAllFold added: every wavefront folds a
                             // tile of its own and stores the tiles of all to its destinations (flat programs only)
    uint32_t varGroups;      // groups of unequal length, see below
};

// vecBatch of the form for short launches: eight-leaf batches, two adjacent tiles per wavefront (threads 64, no shared
// stores, uniform groups; blocksPerSub counts pairs of tiles).
constexpr uint32_t kVecBatchPair = 0x108;
// Flag in storeWaves: the workgroup's wavefronts fold one tile each and exchange the results through LDS (2 KiB of
// dynamic LDS per wavefront), so that wavefront k writes storeWaves neighbouring tiles to destinations k,
// k + storeWaves, ...: one or two long store streams per wavefront instead of a short piece of every stream.
constexpr uint32_t kStoreWavesAllFold = 0x100;

struct ReduceArgs : ReduceHot {
    const void* src[kMaxRanks];
    void* dst[kMaxRanks];
    // Groups of unequal length (ReduceScatterV): when varGroups is set, group g spans groupLenV[g]
    // elements starting groupOffV[g] elements into every source, instead of the uniform
    // groupLen / srcGroupStride / total geometry, and owns the workgroups
    // [groupBlockEnd[g-1], groupBlockEnd[g]) of the grid (filled by the launcher's caller).
    uint32_t groupBlockEnd[kMaxRanks];
    uint64_t groupOffV[kMaxRanks];
    uint64_t groupLenV[kMaxRanks];
};

// A fold of a few MiB per rank with everything the kernel needs in its arguments: up to eight leaves in fold order
// (src[i] is leaf i's buffer) and up to eight destinations, all 16-byte aligned, `nVec` whole 16-byte vectors and
// `tail` (< 16 / element size) elements behind them.  No program image, no tables: the one block of scalar loads that
// fetches the arguments is all that stands in front of a wavefront's first vector load.
constexpr uint32_t kDirectFoldMaxLeaves = 8;
constexpr uint32_t kDirectFoldMaxDst = 8;
constexpr uint32_t kDirectFoldMaxWaves = 8;    // wavefronts per workgroup, 1 KiB of dynamic LDS each
// One instantiation takes up to sixteen leaves and destinations (whole workgroups only, one tile per wavefront).
constexpr uint32_t kDirectFoldWideLeaves = 16;
constexpr uint32_t kDirectFoldWideDst = 16;
struct DirectFoldArgs {
    const void* src[kDirectFoldWideLeaves];
    void* dst[kDirectFoldWideDst];
    uint64_t nVec;
    uint32_t nSrc;
    uint32_t nDst;
    uint32_t tail;
    uint32_t waves;      // wavefronts per workgroup (filled by the launcher)
};

#if defined(__HIPCC__)
// 16-byte streaming store to global memory, written through at system scope.  On this part that cache
// policy sustains about 5 % more bandwidth than a non-temporal store when the stores are mixed with a
// larger volume of loads (8 reads + 1 write: 6.4 vs 6.15 TB/s).  The compiler has no such store that it
// does not also fence, hence the instruction is spelled out; it is an ordinary vector store.
typedef uint32_t StreamVec __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void StoreStream16(void* p, StreamVec v)
{
    asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1" : : "v"(p), "v"(v) : "memory");
}
#endif

// ---- copies -------------------------------------------------------------------------------------
// Copy work is a list of segments cut into tiles of `tileBytes`; workgroup t copies tile t.  The host
// numbers the tiles: tileEnd[s] is the inclusive prefix sum of the segments' tile counts, and a hint
// table over buckets of 2^hintShift tiles (hint[k] = first segment with tileEnd > k << hintShift, one
// closing entry) bounds the search of a workgroup to the segments that touch its bucket.  The kernels
// read these tables with scalar loads only.
constexpr uint32_t kA2aHintMax = 4096;      // buckets of the hint table held in device memory

enum CopyMode : uint32_t {
    COPY_GENERAL = 0,     // source and destination of a segment may differ modulo 16: lanes realign the bytes
    COPY_CONGRUENT = 1,   // every segment has source == destination modulo 16
    COPY_ALIGNED = 2,     // all addresses and lengths are multiples of 16
};

// Offset of a destination address within its 128-byte line, and the number of tiles of a segment of
// `len` bytes whose tiles are cut at the destination's line boundaries (all but the first tile start
// on a line).
__host__ __device__ inline uint32_t TileLead(uint64_t dstAddr) { return static_cast<uint32_t>(dstAddr & 127u); }
inline uint64_t TilesOf(uint64_t len, uint64_t dstAddr, uint32_t tileBytes)
{
    return len == 0 ? 0 : (len + TileLead(dstAddr) + tileBytes - 1) / tileBytes;
}

// Fills hint[0 .. nHint] and returns the shift; nHint = ((tiles - 1) >> shift) + 1 <= maxHint.
template <typename HintT>
inline uint32_t BuildTileHints(const uint32_t* tileEnd, uint32_t nSeg, uint32_t tiles, uint32_t maxHint, HintT* hint,
                               uint32_t* nHintOut)
{
    uint32_t shift = 0;
    while (((tiles - 1) >> shift) + 1 > maxHint) {
        ++shift;
    }
    const uint32_t nHint = ((tiles - 1) >> shift) + 1;
    uint32_t s = 0;
    for (uint32_t k = 0; k < nHint; ++k) {
        const uint64_t first = static_cast<uint64_t>(k) << shift;
        while (tileEnd[s] <= first) {
            ++s;
        }
        hint[k] = static_cast<HintT>(s);
    }
    while (s + 1 < nSeg && tileEnd[s] < tiles) {
        ++s;
    }
    hint[nHint] = static_cast<HintT>(s);
    *nHintOut = nHint;
    return shift;
}

// One-to-many copy (AllGather / AllGatherV / Broadcast / single-rank shortcut): segment j is `len[j]` bytes read
// once from src[j] and written to dst[d] + dstOff[j] for every d < nDst.  The caller fills the first six
// members; LaunchBcastCopy derives the rest: tileEnd[j] = inclusive prefix sum of the segments' tile counts,
// padded with 0xFFFFFFFF up to nSegPadded (a multiple of 16) entries.
struct BcastCopyArgs {
    const void* src[kMaxRanks];
    void* dst[kMaxRanks];
    uint64_t len[kMaxRanks];
    uint64_t dstOff[kMaxRanks];
    uint32_t nSeg;
    uint32_t nDst;
    uint32_t nSegPadded;
    uint32_t nTiles;
    uint64_t leadBase;      // address of the first destination: tiles are cut on its 128-byte lines
    uint32_t pace;          // stores of a wavefront that may be outstanding when it issues the next (3: no limit)
    uint32_t tileEnd[kMaxRanks];
};
static_assert(kMaxRanks % 16 == 0, "the tile prefixes are searched sixteen at a time");

// AlltoAllV: one descriptor of four u64 per non-empty segment (i <- j), all tables in device memory:
//   desc[4s] = send_j + sdispls_j[i] * esz, desc[4s+1] = recv_i + rdispls_i[j] * esz,
//   desc[4s+2] = length in bytes, desc[4s+3] = index of the segment's first tile.
constexpr uint32_t kA2aDescWords = 4;
struct A2aArgs {
    const uint64_t* desc;
    const uint32_t* tileEnd;
    const uint32_t* hint;
    uint32_t hintShift;
    uint32_t mode;        // CopyMode
};

// Tables of one AlltoAllV launch (host image == device image): a descriptor and a tile prefix (u32) per
// segment, then the hint table (u32); 256-byte padded.
inline size_t A2aTableBytes(size_t nSeg)
{
    size_t bytes = nSeg * (kA2aDescWords * sizeof(uint64_t) + sizeof(uint32_t)) + (kA2aHintMax + 4) * sizeof(uint32_t);
    return (bytes + 255) & ~static_cast<size_t>(255);
}

// The allocation-free AlltoAllV keeps its tables in a device array that is part of the library's code object
// (one copy per GPU, held until the process ends) instead of allocated memory: room for the tables of the
// largest world, kMaxRanks * kMaxRanks non-empty segments.
constexpr size_t kA2aScratchBytes =
    ((static_cast<size_t>(kMaxRanks) * kMaxRanks * (kA2aDescWords * sizeof(uint64_t) + sizeof(uint32_t)) +
      (kA2aHintMax + 4) * sizeof(uint32_t)) + 255) & ~static_cast<size_t>(255);
// Address of that array on the current device (looked up once per device).
hipError_t A2aScratchOfCurrentDevice(uint8_t** ptr);
// Writes `nWords` 64-bit words of a host image to `table` (device memory) with small kernels that carry the words
// in their arguments: no copy engine, no staging memory, and the launches can be captured in a graph.
hipError_t LaunchTableWrite(uint8_t* table, const uint64_t* image, uint32_t nWords, hipStream_t stream);

// Stores `value` to `*word` (device-visible memory) from a one-wavefront kernel on `stream`.
hipError_t LaunchMark(uint64_t* word, uint64_t value, hipStream_t stream);

// Launchers (defined in the .hip files).  All are asynchronous on `stream`.
// ldsBytes = (plan depth - 1) * ReduceAccBytes(dtype, op) * args.threads: the accumulator stack of nested levels.
hipError_t LaunchReduce(const ReduceArgs& args, HcclDataType dtype, HcclReduceOp op, uint32_t nBlocks,
                        uint32_t ldsBytes, hipStream_t stream);
// Workgroups of `waves` wavefronts (2 .. kDirectFoldMaxWaves), one 1 KiB tile per wavefront; tilesPerWave = 2: two
// where the launch is whole workgroups of 2 * waves tiles.
hipError_t LaunchDirectFold(const DirectFoldArgs& args, HcclDataType dtype, HcclReduceOp op, uint32_t waves,
                            uint32_t tilesPerWave, hipStream_t stream);
inline uint32_t ReduceAccBytes(HcclDataType dtype, HcclReduceOp op)
{
    bool half = dtype == HCCL_DATA_TYPE_FP16 || dtype == HCCL_DATA_TYPE_BFP16;
    // eight fp32 accumulators (half SUM) or sixteen 16-bit ones (int8) vs one 16-byte pack
    return ((half && op == HCCL_REDUCE_SUM) || dtype == HCCL_DATA_TYPE_INT8) ? 32u : 16u;
}
// tileBytes: 1024, 4096 or 16384; 0 lets the launcher choose.
hipError_t LaunchBcastCopy(const BcastCopyArgs& args, uint32_t tileBytes, hipStream_t stream);
hipError_t LaunchA2aCopy(const A2aArgs& args, uint32_t nTiles, uint32_t tileBytes, hipStream_t stream);

// One freshly written source range to nDst destinations that share its offset from a 16-byte boundary, a
// workgroup of up to sixteen wavefronts per 1 KiB tile with a destination each (more destinations: several
// launches).  FanOutTakes says whether the operands fit; the caller uses LaunchBcastCopy for those that do not.
struct FanOutArgs {
    const void* src;
    void* dst[kMaxRanks];
    uint64_t bytes;
    uint32_t nDst;
};
bool FanOutTakes(const FanOutArgs& args);
// streamLoad: the source is read with non-temporal loads, which leave it out of the caches it passes.
hipError_t LaunchFanOut(const FanOutArgs& args, bool streamLoad, hipStream_t stream);

}  // namespace hccl_amd
