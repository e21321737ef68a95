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
HcclResult BuildFoldPlan(HcclAmdOpKind op, HcclAmdAlgo algo, uint32_t rankSize, FoldPlan* plan);

// Geometry helpers of the recursive halving-doubling family (reference template_utils.cc:42-168).
uint32_t RhdPairCount(uint32_t p);                    // r = p - 2^floor(log2 p)
uint32_t RhdSlotOfRank(uint32_t p, uint32_t rank);    // sigma: t -> 2t, t+r -> 2t+1, others identity
uint32_t RhdCarrierOfVirtual(uint32_t p, uint32_t v); // physical rank that plays virtual rank v

}  // namespace hccl_amd
