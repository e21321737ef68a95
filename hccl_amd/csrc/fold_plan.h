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
// level0 in (1, rankSize): the orders of the reference's sequence executors over level-0 groups of level0 consecutive
// ranks, `algo` (RHD, NHR, or MESH for the host-reduce fold) being the template between the groups.  level1 in
// [1, rankSize / level0): level1 consecutive groups form a level-1 group and the template runs a second time between
// those (three levels; 0: all groups are one level-1 group, two levels).  With l1 groups per level-1 group and l2
// level-1 groups, AllReduce and Reduce: program (i * l1 + j) * l2 + k is part k of sub-slice j of chunk i;
// ReduceScatter: program r is rank r's output.  level0 of 1 or rankSize: one level.
HcclResult BuildFoldPlan(HcclAmdOpKind op, HcclAmdAlgo algo, uint32_t rankSize, FoldPlan* plan, uint32_t level0 = 1,
                         uint32_t level1 = 0);

// The sizes of the levels a world of rankSize ranks has under (level0, level1) as above: false when it has one
// level or the sizes do not divide.  l1 * l2 = rankSize / l0; l2 is 1 in a two-level world.
struct Levels {
    uint32_t l0 = 1, l1 = 1, l2 = 1;
};
bool ResolveLevels(uint32_t rankSize, uint32_t level0, uint32_t level1, Levels* out);

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
// Loops of the three-level sequence executors (reference ins_v2_all_reduce_sequence_executor_aicpu_3level.cc:524-534,
// reduce_sequence_executor_aicpu_3level.cc:877-889): the buffer is cut into l0 + 1 slices of whole elements, the
// first receives the level-0 result, the other l0 the peers' data; a loop holds what those l0 slices take, floored
// to `align` bytes (128 for AllReduce, 4096 for Reduce), whole elements and a multiple of `total` ranks.  With
// rhdTail the two tail tiles of RhdMaxCountPerLoop leave the buffer first (count not a multiple of total).
// resultElems: the elements of the first slice.  HCCL_E_INTERNAL when nothing fits.
HcclResult SequenceMaxCountPerLoop(uint64_t cclBytes, uint64_t count, uint32_t l0, uint32_t total, uint64_t elemSize,
                                   uint64_t align, bool rhdTail, uint64_t* maxCount, uint64_t* resultElems);
// Elements the next loop of those executors takes when the chunks are floor(len / l0) with the rest in the last:
// a last loop whose last chunk would not fit the result slice gives some elements up to one more loop
// (reference ins_v2_all_reduce_sequence_executor_aicpu_3level.cc:704-731).  0 when the slice holds no element.
uint64_t SequenceSelectLoopCount(uint64_t remaining, uint64_t maxCountPerLoop, uint32_t l0, uint64_t resultElems);

}  // namespace hccl_amd
