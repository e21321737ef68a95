// Host-side construction of fold programs: for an (operation, algorithm, rankSize) triple, the list of
// per-segment byte programs (see dataplane.h) that reproduce the reference executor's association order.
#pragma once

#include <stdint.h>

#include <vector>

#include "hccl.h"

namespace hccl_amd {

struct FoldPlan {
    // programs[s] is the program of segment s; every program ends with kTokEnd.
    std::vector<std::vector<uint8_t>> programs;
    // true when segment s is the s-th sub-segment of one group (AllReduce cut into units);
    // false when segment s is the group of destination rank s (ReduceScatter).
    bool segmentsAreSubs = false;
    uint32_t maxDepth = 1;
};

// Returns HCCL_E_NOT_SUPPORT for combinations that do not exist (e.g. AIV_MESH AllReduce).
// level0 in (1, rankSize): the two-level AllReduce of the reference's sequence executor over groups of level0
// consecutive ranks, `algo` (RHD, NHR, or MESH for the host-reduce fold) being the template between the groups;
// program i * (rankSize / level0) + j is sub-slice j of chunk i; for ReduceScatter the two-level order of the same
// executor family, program r being rank r's output.  level0 of 1 or rankSize: one level.
HcclResult BuildFoldPlan(HcclAmdOpKind op, HcclAmdAlgo algo, uint32_t rankSize, FoldPlan* plan, uint32_t level0 = 1);

// Geometry helpers of the recursive halving-doubling family (reference template_utils.cc:42-168).
uint32_t RhdPairCount(uint32_t p);                    // r = p - 2^floor(log2 p)
uint32_t RhdSlotOfRank(uint32_t p, uint32_t rank);    // sigma: t -> 2t, t+r -> 2t+1, others identity
uint32_t RhdCarrierOfVirtual(uint32_t p, uint32_t v); // physical rank that plays virtual rank v

// Segments of one slice under the mesh-chunk order, as runs of equally long neighbours: segments
// [firstSeg, firstSeg + nSeg) start `first` elements into the slice, hold segLen elements each and lastLen in the
// last one.  With alignTo4K (ReduceScatter, ReduceScatterV) the first N - 2 segments are floor(bytes / (N - 1))
// rounded down to 4 KiB and the last takes the rest; slices too small for that, and AllReduce always, are dealt
// element-wise, the first len mod (N - 1) segments one element longer, possibly leaving empty segments
// (reference ins_temp_reduce_scatter_mesh_1D_meshchunk.cc:233-258,
// ins_temp_reduce_scatter_v_mesh_1D_meshchunk.cc:147-191, ins_temp_all_reduce_mesh_1D_two_shot_mesh_chunk.cc:181-199).
struct SegmentRun {
    uint64_t first;
    uint32_t firstSeg;
    uint32_t nSeg;
    uint64_t segLen;
    uint64_t lastLen;
};
std::vector<SegmentRun> MeshChunkSegments(uint64_t len, uint32_t rankSize, uint32_t elemSize, bool alignTo4K);

// Loop limits of the reference's executors, which stage every AllReduce through a bounded buffer and cut the
// count into loops that are each sliced afresh.  cclBytes is that buffer's size.
// HCCL_BUFFSIZE (MB, digits only, 2 .. UINT32_MAX) less the 1 MiB kept back; nullptr = unset = 200 MB
// (reference src/common/op_graph/hccl_op_utils.cc:204-225).  HCCL_E_PARA for anything else.
HcclResult CclBufferAvailableSize(const char* envValue, uint64_t* bytes);
// Elements per loop of a single-template executor (reference ins_v2_all_reduce_sole_executor.cc:241-262).
uint64_t SoleMaxCountPerLoop(uint64_t cclBytes, uint64_t scratchMultiple, uint64_t elemSize);
// Elements per loop of the RHD sequence executor with one rank per level-0 group: two 128-byte-rounded tiles of
// p elements leave the buffer when count is not a multiple of p, half of the rest receives, floored to 128
// bytes, whole elements and a multiple of p (reference ins_v2_all_reduce_sequence_rhd_tail.h:64-92,
// ins_v2_all_reduce_sequence_executor_aicpu.cc:592-600, 645-675).  HCCL_E_INTERNAL when nothing fits.
HcclResult RhdMaxCountPerLoop(uint64_t cclBytes, uint64_t count, uint32_t p, uint64_t elemSize, uint64_t* maxCount);
// Elements the next RHD loop takes: whole frames of p while they last, then the remainder below p alone
// (reference ins_v2_all_reduce_sequence_rhd_tail.h:94-99).
uint64_t RhdSelectLoopCount(uint64_t remaining, uint64_t maxCountPerLoop, uint64_t p);

}  // namespace hccl_amd
