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
struct ReduceArgs {
    const void* src[kMaxRanks];
    void* dst[kMaxRanks];
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
    uint32_t blocksPerSub;
    uint32_t vecOk;   // every address the launch touches is 16-byte aligned
};

// One-to-many copy (AllGather / AllGatherV / single-rank shortcut): segment j is `len[j]` bytes read
// once from src[j] and written to dst[d] + dstOff[j] for every d < nDst.
struct BcastCopyArgs {
    const void* src[kMaxRanks];
    void* dst[kMaxRanks];
    uint64_t len[kMaxRanks];
    uint64_t dstOff[kMaxRanks];
    uint32_t nSeg;
    uint32_t nDst;
    uint32_t unit;   // widest power of two (<= 16) dividing every destination base address
};

// AlltoAllV.  Tables live in device memory, n x n row-major, in elements:
//   cnt[j*n + i] = sendCounts_j[i], sdis[j*n + i] = sdispls_j[i], rdis[i*n + j] = rdispls_i[j].
// rowStart[i] (n + 1 entries) and segEnd[i*n + j] are written by the plan kernel: tiles of
// destination rank i start at rowStart[i]; segEnd is the inclusive tile prefix inside row i.
struct A2aArgs {
    const void* send[kMaxRanks];
    void* recv[kMaxRanks];
    const uint64_t* cnt;
    const uint64_t* sdis;
    const uint64_t* rdis;
    uint32_t* rowStart;
    uint32_t* segEnd;
    uint32_t n;
    uint32_t esz;
    uint32_t tileBytes;   // 4096 or 16384: bytes one workgroup copies
};


// Launchers (defined in the .hip files).  All are asynchronous on `stream`.
// ldsBytes = (plan depth - 1) * ReduceAccBytes(dtype, op) * 256: the accumulator stack of nested levels.
hipError_t LaunchReduce(const ReduceArgs& args, HcclDataType dtype, HcclReduceOp op, uint32_t nBlocks,
                        uint32_t ldsBytes, hipStream_t stream);
inline uint32_t ReduceAccBytes(HcclDataType dtype, HcclReduceOp op)
{
    bool half = dtype == HCCL_DATA_TYPE_FP16 || dtype == HCCL_DATA_TYPE_BFP16;
    return (half && op == HCCL_REDUCE_SUM) ? 32u : 16u;   // eight fp32 accumulators vs one 16-byte pack
}
hipError_t LaunchBcastCopy(const BcastCopyArgs& args, uint32_t tileBytes, hipStream_t stream);
hipError_t LaunchA2aPlan(const A2aArgs& args, hipStream_t stream);
hipError_t LaunchA2aCopy(const A2aArgs& args, uint32_t nTiles, hipStream_t stream);

}  // namespace hccl_amd
