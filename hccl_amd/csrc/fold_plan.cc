// Fold-program construction.  Each builder replays, symbolically, the sequence of pairwise
// LocalReduce / write-reduce steps the reference's template issues and records, for the slot that ends
// up holding a segment's result, which rank values were folded into it, in which order and in which role.
#include "fold_plan.h"

#include <algorithm>
#include <cstdlib>
#include <functional>
#include <memory>

#include "dataplane.h"

namespace hccl_amd {
namespace {

// A value under construction: operands folded left to right into the first one.
struct Expr;
using ExprPtr = std::shared_ptr<const Expr>;
struct Operand {
    int rank;      // >= 0: a rank's input value
    ExprPtr sub;   // otherwise a nested value
};
struct Expr {
    std::vector<Operand> ops;
};

ExprPtr Leaf(uint32_t rank)
{
    auto e = std::make_shared<Expr>();
    e->ops.push_back({static_cast<int>(rank), nullptr});
    return e;
}

// dst <- src (+) dst : dst stays the accumulator, src becomes one more operand of its level.
ExprPtr Fold(const ExprPtr& dst, const ExprPtr& src)
{
    auto e = std::make_shared<Expr>(*dst);
    if (src->ops.size() == 1 && src->ops[0].rank >= 0) {
        e->ops.push_back(src->ops[0]);
    } else {
        e->ops.push_back({-1, src});
    }
    return e;
}

uint32_t Depth(const Expr& e)
{
    uint32_t d = 1;
    for (const Operand& o : e.ops) {
        if (o.rank < 0) {
            uint32_t sd = 1 + Depth(*o.sub);
            d = sd > d ? sd : d;
        }
    }
    return d;
}

void Serialize(const Expr& e, std::vector<uint8_t>* out)
{
    size_t i = 0;
    while (i < e.ops.size()) {
        if (e.ops[i].rank < 0) {
            out->push_back(kTokOpen);
            Serialize(*e.ops[i].sub, out);
            out->push_back(kTokClose);
            ++i;
            continue;
        }
        size_t j = i;
        while (j < e.ops.size() && e.ops[j].rank >= 0 && j - i < static_cast<size_t>(kMaxRun)) {
            ++j;
        }
        out->push_back(static_cast<uint8_t>(kTokRun | (j - i)));
        for (size_t k = i; k < j; ++k) {
            out->push_back(static_cast<uint8_t>(e.ops[k].rank));
        }
        i = j;
    }
}

HcclResult Emit(const ExprPtr& e, FoldPlan* plan)
{
    uint32_t d = Depth(*e);
    if (d > static_cast<uint32_t>(kMaxFoldDepth)) {
        return HCCL_E_NOT_SUPPORT;
    }
    std::vector<uint8_t> prog;
    Serialize(*e, &prog);
    prog.push_back(kTokEnd);
    if (prog.size() > static_cast<size_t>(kProgStride)) {
        return HCCL_E_INTERNAL;
    }
    plan->maxDepth = d > plan->maxDepth ? d : plan->maxDepth;
    plan->programs.push_back(std::move(prog));
    return HCCL_SUCCESS;
}

ExprPtr Chain(const std::vector<uint32_t>& order)
{
    ExprPtr e = Leaf(order[0]);
    for (size_t i = 1; i < order.size(); ++i) {
        e = Fold(e, Leaf(order[i]));
    }
    return e;
}

// What stands for participant k of a step-driven template before its first step: rank k's input in a one-level
// world, the value a level-0 group has folded for that participant in a two-level one.
using LeafFn = std::function<ExprPtr(uint32_t)>;
ExprPtr RankLeaf(uint32_t k) { return Leaf(k); }

HcclResult EmitAll(const std::vector<ExprPtr>& values, FoldPlan* plan)
{
    for (const ExprPtr& e : values) {
        HcclResult rc = Emit(e, plan);
        if (rc != HCCL_SUCCESS) {
            return rc;
        }
    }
    return HCCL_SUCCESS;
}

uint32_t CeilLog2(uint32_t n)
{
    uint32_t s = 0;
    for (uint32_t t = n - 1; t != 0; t >>= 1) {
        ++s;
    }
    return s;
}

uint32_t FloorLog2(uint32_t n)
{
    uint32_t s = 0;
    for (uint32_t t = n; t > 1; t >>= 1) {
        ++s;
    }
    return s;
}

// ---- mesh --------------------------------------------------------------------------------------
// AllReduce: slot 0 accumulates slots 1..N-1 ascending (reference
// ins_temp_all_reduce_mesh_1D_one_shot.cc:223-239; two-shot and the host-reduce NHR template fold in
// the same order, ins_temp_all_reduce_mesh_1D_two_shot.cc:341-357,
// ins_temp_all_reduce_aicpu_reduce_nhr.cc:272-285).
HcclResult MeshAllReduce(uint32_t n, FoldPlan* plan)
{
    std::vector<uint32_t> order(n);
    for (uint32_t r = 0; r < n; ++r) {
        order[r] = r;
    }
    plan->segmentsAreSubs = true;
    return Emit(Chain(order), plan);
}

// ReduceScatter: rank k copies its own slice, then folds the other ranks ascending (reference
// ins_temp_reduce_scatter_mesh_1D.cc:203-237).
HcclResult MeshReduceScatter(uint32_t n, FoldPlan* plan)
{
    for (uint32_t k = 0; k < n; ++k) {
        std::vector<uint32_t> order{k};
        for (uint32_t t = 0; t < n; ++t) {
            if (t != k) {
                order.push_back(t);
            }
        }
        HcclResult rc = Emit(Chain(order), plan);
        if (rc != HCCL_SUCCESS) {
            return rc;
        }
    }
    return HCCL_SUCCESS;
}

// Vector-core mesh ReduceScatter: chunk c of an output starts from peer c and folds peers
// c+1, c+2, ... modulo N (reference aiv_reduce_scatter_mesh_1d.h:34-46, 57-71).
HcclResult AivMeshReduceScatter(uint32_t n, FoldPlan* plan)
{
    plan->segmentsAreSubs = true;
    for (uint32_t c = 0; c < n; ++c) {
        std::vector<uint32_t> order(n);
        for (uint32_t i = 0; i < n; ++i) {
            order[i] = (c + i) % n;
        }
        HcclResult rc = Emit(Chain(order), plan);
        if (rc != HCCL_SUCCESS) {
            return rc;
        }
    }
    return HCCL_SUCCESS;
}

// ---- mesh chunk --------------------------------------------------------------------------------
// Every slice is cut into N - 1 segments.  In step s a rank sends, for i = 0 .. N-2, segment i of the slice of
// the rank `num` places below it, num = s + i + 1, one more once that reaches N (which skips the sender itself),
// and the owner write-reduces it into its copy, which began as its own input (reference
// ins_temp_reduce_scatter_mesh_1D_meshchunk.cc:277-375, ins_temp_reduce_scatter_v_mesh_1D_meshchunk.cc:202-265,
// ins_temp_all_reduce_mesh_1D_two_shot_mesh_chunk.cc:220-295).  Program k * (N - 1) + i is segment i of slice k.
HcclResult MeshChunk(uint32_t n, FoldPlan* plan)
{
    if (n == 1) {
        return Emit(Leaf(0), plan);
    }
    const uint32_t segs = n - 1;
    std::vector<std::vector<ExprPtr>> held(n, std::vector<ExprPtr>(segs));
    for (uint32_t k = 0; k < n; ++k) {
        for (uint32_t i = 0; i < segs; ++i) {
            held[k][i] = Leaf(k);
        }
    }
    for (uint32_t step = 0; step < segs; ++step) {
        for (uint32_t i = 0; i < segs; ++i) {
            uint32_t num = step + i + 1;
            if (num >= n) {
                num += 1;
            }
            for (uint32_t sender = 0; sender < n; ++sender) {
                const uint32_t next = (sender + num) % n;
                const uint32_t owner = (2 * sender + n - next) % n;
                held[owner][i] = Fold(held[owner][i], Leaf(sender));
            }
        }
    }
    for (uint32_t k = 0; k < n; ++k) {
        for (uint32_t i = 0; i < segs; ++i) {
            HcclResult rc = Emit(held[k][i], plan);
            if (rc != HCCL_SUCCESS) {
                return rc;
            }
        }
    }
    return HCCL_SUCCESS;
}

// ---- order preserved ---------------------------------------------------------------------------
// while blocks > 1: M = largest power of two below blocks; block src in [M, blocks) folds into block
// src % M; blocks = M (reference ins_temp_reduce_scatter_order_preserved_group.cc:353-398).
HcclResult OrderPreserved(uint32_t n, FoldPlan* plan)
{
    std::vector<ExprPtr> slot(n);
    for (uint32_t v = 0; v < n; ++v) {
        slot[v] = Leaf(v);
    }
    uint32_t remaining = n;
    while (remaining > 1) {
        uint32_t m = 1;
        while (m * 2 < remaining) {
            m *= 2;
        }
        for (uint32_t src = m; src < remaining; ++src) {
            slot[src % m] = Fold(slot[src % m], slot[src]);
        }
        remaining = m;
    }
    return Emit(slot[0], plan);
}

// ---- NHR ---------------------------------------------------------------------------------------
// Step s: rank m write-reduces slices {m - 2^s - i * 2^(s+1)} into the same slices of rank m - 2^s,
// i < (N - 1 + 2^s) / 2^(s+1); the receiver's value is the accumulator (reference
// ins_temp_reduce_scatter_nhr.cc:316-447, 458-506).  Slice k ends at rank k.
std::vector<ExprPtr> NhrValues(uint32_t n, const LeafFn& leaf)
{
    std::vector<std::vector<ExprPtr>> held(n, std::vector<ExprPtr>(n));
    for (uint32_t m = 0; m < n; ++m) {
        for (uint32_t k = 0; k < n; ++k) {
            held[m][k] = leaf(m);
        }
    }
    uint32_t steps = CeilLog2(n);
    for (uint32_t s = 0; s < steps; ++s) {
        const auto before = held;
        uint32_t delta = 1u << s;
        uint32_t nSlices = (n - 1 + delta) / (delta * 2);
        uint32_t stride = (delta * 2) % n;
        for (uint32_t m = 0; m < n; ++m) {
            uint32_t to = (m + n - delta) % n;
            uint32_t slice = to;
            for (uint32_t i = 0; i < nSlices; ++i) {
                held[to][slice] = Fold(before[to][slice], before[m][slice]);
                slice = (slice + n - stride) % n;
            }
        }
    }
    std::vector<ExprPtr> out(n);
    for (uint32_t k = 0; k < n; ++k) {
        out[k] = held[k][k];
    }
    return out;
}

HcclResult Nhr(uint32_t n, FoldPlan* plan) { return EmitAll(NhrValues(n, RankLeaf), plan); }

// ---- RHD ---------------------------------------------------------------------------------------
uint32_t VirtualSlotStart(uint32_t r, uint32_t a) { return a < r ? 2 * a : a + r; }
uint32_t VirtualSlotEnd(uint32_t r, uint32_t b) { return b <= r ? 2 * b : b + r; }

// Mirror: every rank holds p slots, slot sigma(i) = its contribution to share i.
// PRE:  merged rank t + r write-reduces all p slots into representative t.
// MAIN: step k, dist = P >> (k + 1): virtual rank v write-reduces the slots of its partner's aligned
//       half into the partner v ^ dist (the partner's value is the accumulator).
// Share i ends at the carrier of the virtual rank owning slot sigma(i)
// (reference template_utils.cc:117-208, ins_temp_reduce_scatter_rhd.cc:365-564).
std::vector<ExprPtr> RhdValues(uint32_t p, const LeafFn& leaf)
{
    uint32_t r = RhdPairCount(p);
    uint32_t bigP = p - r;
    std::vector<std::vector<ExprPtr>> held(p, std::vector<ExprPtr>(p));
    for (uint32_t j = 0; j < p; ++j) {
        for (uint32_t u = 0; u < p; ++u) {
            held[j][u] = leaf(j);
        }
    }
    for (uint32_t t = 0; t < r; ++t) {
        for (uint32_t u = 0; u < p; ++u) {
            held[t][u] = Fold(held[t][u], held[t + r][u]);
        }
    }
    uint32_t steps = FloorLog2(bigP);
    for (uint32_t k = 0; k < steps; ++k) {
        const auto before = held;
        uint32_t dist = bigP >> (k + 1);
        for (uint32_t v = 0; v < bigP; ++v) {
            uint32_t peer = v ^ dist;
            uint32_t peerBase = peer & ~(dist - 1);
            uint32_t from = RhdCarrierOfVirtual(p, v);
            uint32_t to = RhdCarrierOfVirtual(p, peer);
            for (uint32_t u = VirtualSlotStart(r, peerBase); u < VirtualSlotEnd(r, peerBase + dist); ++u) {
                held[to][u] = Fold(before[to][u], before[from][u]);
            }
        }
    }
    std::vector<ExprPtr> out(p);
    for (uint32_t i = 0; i < p; ++i) {
        uint32_t slot = RhdSlotOfRank(p, i);
        uint32_t v = slot < 2 * r ? slot / 2 : slot - r;
        out[i] = held[RhdCarrierOfVirtual(p, v)][slot];
    }
    return out;
}

HcclResult Rhd(uint32_t p, FoldPlan* plan) { return EmitAll(RhdValues(p, RankLeaf), plan); }

// ---- two and three levels ----------------------------------------------------------------------
// AllReduce over level-0 groups of l0 consecutive ranks ("boxes") and a template between the boxes (reference
// ins_v2_all_reduce_sequence_executor_aicpu.cc:592-852: step 1 mesh ReduceScatter inside the box, step 2 the
// ReduceScatter between the ranks that hold the same chunk, steps 3 and 4 the two AllGathers).  A loop's elements
// are l0 chunks of l1 sub-slices; sub-slice j of chunk i is the template's value for its unit j, in which
// participant b stands for what box b folded for chunk i, the chunk owner's input first and the other ranks of the
// box ascending (reference ins_temp_reduce_scatter_mesh_1D.cc:203-237; the level-0 template ..._Z_axis_detour
// derives from it).  The template: RHD with POST skipped and the merged share bridged (:700-741), NHR (:784-789),
// or for the types the host reduces the own-first fold of ins_temp_reduce_scatter_aicpu_reduce_nhr.cc:214-250
// (`MESH`).
// With three levels (reference ins_v2_all_reduce_sequence_executor_aicpu_3level.cc:536-800) l1 consecutive boxes
// form a level-1 group, the template runs between the boxes of a group on the sub-slices and once more between
// the l2 groups on the parts of a sub-slice: part k of sub-slice j is the template's value for unit k among the
// groups, participant g standing for the value of unit j among the boxes of group g.  Rank (g * l1 + b) * l0 + i
// is member i of box b of group g.
HcclResult TemplateValues(HcclAmdAlgo algo, uint32_t count, const LeafFn& leaf, std::vector<ExprPtr>* out)
{
    out->clear();
    if (algo == HCCL_AMD_ALGO_RHD) {
        *out = RhdValues(count, leaf);
    } else if (algo == HCCL_AMD_ALGO_NHR) {
        *out = NhrValues(count, leaf);
    } else if (algo == HCCL_AMD_ALGO_MESH) {
        for (uint32_t j = 0; j < count; ++j) {
            ExprPtr e = leaf(j);
            for (uint32_t b = 0; b < count; ++b) {
                if (b != j) {
                    e = Fold(e, leaf(b));
                }
            }
            out->push_back(e);
        }
    } else {
        return HCCL_E_NOT_SUPPORT;
    }
    return HCCL_SUCCESS;
}

// The values of level-0 member i: unit j * l2 + k is part k of sub-slice j of its chunk.
HcclResult LevelUnits(const Levels& lv, HcclAmdAlgo algo, uint32_t i, std::vector<ExprPtr>* units)
{
    std::vector<std::vector<ExprPtr>> group(lv.l2);
    for (uint32_t g = 0; g < lv.l2; ++g) {
        const LeafFn box = [&](uint32_t b) {
            const uint32_t first = (g * lv.l1 + b) * lv.l0;
            std::vector<uint32_t> order{first + i};
            for (uint32_t t = 0; t < lv.l0; ++t) {
                if (t != i) {
                    order.push_back(first + t);
                }
            }
            return Chain(order);
        };
        HcclResult rc = TemplateValues(algo, lv.l1, box, &group[g]);
        if (rc != HCCL_SUCCESS) {
            return rc;
        }
    }
    if (lv.l2 == 1) {
        *units = group[0];
        return HCCL_SUCCESS;
    }
    units->assign(static_cast<size_t>(lv.l1) * lv.l2, nullptr);
    for (uint32_t j = 0; j < lv.l1; ++j) {
        std::vector<ExprPtr> parts;
        HcclResult rc = TemplateValues(algo, lv.l2, [&](uint32_t g) { return group[g][j]; }, &parts);
        if (rc != HCCL_SUCCESS) {
            return rc;
        }
        for (uint32_t k = 0; k < lv.l2; ++k) {
            (*units)[static_cast<size_t>(j) * lv.l2 + k] = parts[k];
        }
    }
    return HCCL_SUCCESS;
}

// AllReduce, and Reduce, whose sequence executors run the same steps and hand the result to the root only
// (reference reduce_sequence_executor_aicpu_3level.cc:744-990).
HcclResult LevelsAllReduce(const Levels& lv, HcclAmdAlgo algo, FoldPlan* plan)
{
    plan->segmentsAreSubs = true;
    for (uint32_t i = 0; i < lv.l0; ++i) {
        std::vector<ExprPtr> units;
        HcclResult rc = LevelUnits(lv, algo, i, &units);
        if (rc == HCCL_SUCCESS) {
            rc = EmitAll(units, plan);
        }
        if (rc != HCCL_SUCCESS) {
            return rc;
        }
    }
    return HCCL_SUCCESS;
}

// ReduceScatter over the same boxes (reference ins_v2_reduce_scatter_sequence_executor_aicpu.cc:298-372, 388-500):
// step 1 is the mesh ReduceScatter inside the box once per box of the world (in repeat q member i folds slice
// q * l0 + i of its box, its own input first), step 2 the ReduceScatter between the members i, whose unit q is that
// slice; box j ends with unit j, the output of rank j * l0 + i.  With three levels
// (ins_v2_reduce_scatter_sequence_executor_3level.cc:243-256) the boxes of a group do that for the slices of every
// group, and the groups reduce-scatter what they hold for each other.  Program r is therefore the tree of part
// r / (l0 * l1) of sub-slice r / l0 % l1 of chunk r % l0 of the AllReduce over the same levels.  The template: RHD
// (reduce_scatter_rhd with its POST, which moves shares and folds nothing), NHR, or the own-first fold of
// reduce_scatter_aicpu_reduce_nhr_pcie.cc:212-280 (`MESH`).  A loop covers the same range of every slice, so loop
// boundaries do not show in the result.
HcclResult LevelsReduceScatter(const Levels& lv, HcclAmdAlgo algo, FoldPlan* plan)
{
    plan->segmentsAreSubs = false;
    std::vector<std::vector<ExprPtr>> units(lv.l0);
    for (uint32_t i = 0; i < lv.l0; ++i) {
        HcclResult rc = LevelUnits(lv, algo, i, &units[i]);
        if (rc != HCCL_SUCCESS) {
            return rc;
        }
    }
    const uint32_t n = lv.l0 * lv.l1 * lv.l2;
    for (uint32_t r = 0; r < n; ++r) {
        const uint32_t box = r / lv.l0;
        HcclResult rc = Emit(units[r % lv.l0][static_cast<size_t>(box % lv.l1) * lv.l2 + box / lv.l1], plan);
        if (rc != HCCL_SUCCESS) {
            return rc;
        }
    }
    return HCCL_SUCCESS;
}

}  // namespace

uint32_t RhdPairCount(uint32_t p)
{
    if (p == 0) {
        return 0;
    }
    uint32_t hp = 1;
    while (hp <= p / 2) {
        hp *= 2;
    }
    return p - hp;
}

uint32_t RhdSlotOfRank(uint32_t p, uint32_t rank)
{
    uint32_t r = RhdPairCount(p);
    if (rank < r) {
        return 2 * rank;
    }
    if (rank < 2 * r) {
        return 2 * (rank - r) + 1;
    }
    return rank;
}

uint32_t RhdCarrierOfVirtual(uint32_t p, uint32_t v)
{
    uint32_t r = RhdPairCount(p);
    return v < r ? v : v + r;
}

bool ResolveLevels(uint32_t n, uint32_t level0, uint32_t level1, Levels* out)
{
    if (level0 <= 1 || level0 >= n || n % level0 != 0) {
        return false;
    }
    const uint32_t boxes = n / level0;
    out->l0 = level0;
    if (level1 == 0 || level1 >= boxes) {
        out->l1 = boxes;
        out->l2 = 1;
        return true;
    }
    if (boxes % level1 != 0) {
        return false;
    }
    out->l1 = level1;
    out->l2 = boxes / level1;
    return true;
}

HcclResult BuildFoldPlan(HcclAmdOpKind op, HcclAmdAlgo algo, uint32_t n, FoldPlan* plan, uint32_t level0,
                         uint32_t level1)
{
    *plan = FoldPlan{};
    if (n == 0 || n > static_cast<uint32_t>(kMaxRanks)) {
        return HCCL_E_PARA;
    }
    if (level0 > 1 && level0 < n) {
        Levels lv;
        // the host-reduce fold knows two levels only: every box of the world is its peer
        if (!ResolveLevels(n, level0, algo == HCCL_AMD_ALGO_MESH ? 0 : level1, &lv)) {
            return HCCL_E_PARA;
        }
        if (op == HCCL_AMD_OP_ALL_REDUCE || op == HCCL_AMD_OP_REDUCE) {
            return LevelsAllReduce(lv, algo, plan);
        }
        if (op == HCCL_AMD_OP_REDUCE_SCATTER) {
            return LevelsReduceScatter(lv, algo, plan);
        }
        return HCCL_E_NOT_SUPPORT;
    }
    if (op == HCCL_AMD_OP_REDUCE) {
        // One-shot: rank 0's slot is the base, the others fold ascending (reference reduce_mesh_1D.cc:268-300).
        // Two-shot: slice k is folded at rank k, own input first (reference reduce_mesh_1D_two_shot.cc:228-265).
        // NHR: the step tree of the NHR ReduceScatter on n slices, gathered at the root (reference
        // reduce_nhr.cc:263-339, 481-519).
        if (algo == HCCL_AMD_ALGO_MESH || algo == HCCL_AMD_ALGO_RING) {
            return MeshAllReduce(n, plan);
        }
        if (algo == HCCL_AMD_ALGO_MESH_TWO_SHOT) {
            plan->segmentsAreSubs = true;
            return MeshReduceScatter(n, plan);
        }
        if (algo == HCCL_AMD_ALGO_NHR) {
            plan->segmentsAreSubs = true;
            return Nhr(n, plan);
        }
        return HCCL_E_NOT_SUPPORT;
    }
    bool ar = op == HCCL_AMD_OP_ALL_REDUCE;
    if (!ar && op != HCCL_AMD_OP_REDUCE_SCATTER) {
        return HCCL_E_PARA;
    }
    switch (algo) {
        case HCCL_AMD_ALGO_MESH:
            return ar ? MeshAllReduce(n, plan) : MeshReduceScatter(n, plan);
        case HCCL_AMD_ALGO_RING:
            // AllReduce: the host-reduce "ring family" template gathers and folds in rank order.
            // ReduceScatter: the in-tree ring-family algorithm is the NHR step tree.
            return ar ? MeshAllReduce(n, plan) : Nhr(n, plan);
        case HCCL_AMD_ALGO_RHD:
            plan->segmentsAreSubs = ar;
            return Rhd(n, plan);
        case HCCL_AMD_ALGO_NHR:
            plan->segmentsAreSubs = ar;
            return Nhr(n, plan);
        case HCCL_AMD_ALGO_ORDER_PRESERVED:
            plan->segmentsAreSubs = true;
            return OrderPreserved(n, plan);
        case HCCL_AMD_ALGO_AIV_MESH:
            return ar ? HCCL_E_NOT_SUPPORT : AivMeshReduceScatter(n, plan);
        case HCCL_AMD_ALGO_MESH_SYMMETRIC:
            // Slice k of the AllReduce result is folded like rank k's ReduceScatter output.
            plan->segmentsAreSubs = ar;
            return MeshReduceScatter(n, plan);
        case HCCL_AMD_ALGO_MESH_CHUNK:
            plan->segmentsAreSubs = true;
            return MeshChunk(n, plan);
        case HCCL_AMD_ALGO_MESH_CONCUR:
            // AllReduce only: slice k of a loop is folded like rank k's ReduceScatter output (reference
            // ins_v2_all_reduce_two_shot_sole_executor.cc:395-398: mesh ReduceScatter + AllGather).
            if (!ar) {
                return HCCL_E_NOT_SUPPORT;
            }
            plan->segmentsAreSubs = true;
            return MeshReduceScatter(n, plan);
        case HCCL_AMD_ALGO_MESH_TWO_SHOT:
            return HCCL_E_NOT_SUPPORT;   // Reduce only; AllReduce's two-shot folds in the MESH order
        default:
            return HCCL_E_PARA;
    }
}

HcclResult CclBufferAvailableSize(const char* envValue, uint64_t* bytes)
{
    constexpr uint64_t kMiB = 1024ull * 1024ull;
    uint64_t mb = 200;
    if (envValue != nullptr) {
        char* end = nullptr;
        mb = std::strtoull(envValue, &end, 10);
        if (end == envValue || *end != '\0' || mb < 2 || mb > 0xFFFFFFFFull) {
            return HCCL_E_PARA;
        }
    }
    *bytes = mb * kMiB - kMiB;
    return HCCL_SUCCESS;
}

uint64_t SoleMaxCountPerLoop(uint64_t cclBytes, uint64_t scratchMultiple, uint64_t elemSize)
{
    uint64_t perLoop = cclBytes;
    if (scratchMultiple != 0) {
        perLoop = std::min(cclBytes, cclBytes / scratchMultiple / 128 * 128);
    }
    return elemSize == 0 ? 0 : perLoop / elemSize;
}

HcclResult RhdMaxCountPerLoop(uint64_t cclBytes, uint64_t count, uint32_t p, uint64_t elemSize, uint64_t* maxCount)
{
    if (p == 0 || elemSize == 0) {
        return HCCL_E_PARA;
    }
    uint64_t workspace = cclBytes;
    if (count % p != 0) {
        if (p > workspace / elemSize / 2) {
            return HCCL_E_INTERNAL;
        }
        const uint64_t tile = p * elemSize;
        const uint64_t slot = (tile + 127) / 128 * 128;
        if (slot >= workspace / 2) {
            return HCCL_E_INTERNAL;
        }
        workspace -= 2 * slot;
    }
    *maxCount = workspace / 2 / 128 * 128 / elemSize / p * p;
    return *maxCount == 0 ? HCCL_E_INTERNAL : HCCL_SUCCESS;
}

std::vector<SegmentRun> MeshChunkSegments(uint64_t len, uint32_t n, uint32_t elemSize, bool alignTo4K)
{
    std::vector<SegmentRun> runs;
    if (len == 0 || n < 2 || elemSize == 0) {
        return runs;
    }
    const uint64_t segs = n - 1;
    if (alignTo4K) {
        const uint64_t alignedBytes = (len * elemSize / segs) / 4096 * 4096;
        if (segs >= 2 && alignedBytes > 0) {
            const uint64_t segLen = alignedBytes / elemSize;
            runs.push_back({0, 0, static_cast<uint32_t>(segs), segLen, len - segLen * (segs - 1)});
            return runs;
        }
    }
    const uint64_t small = len / segs;
    const uint32_t nBig = static_cast<uint32_t>(len % segs);
    if (nBig != 0) {
        runs.push_back({0, 0, nBig, small + 1, small + 1});
    }
    if (small != 0) {
        runs.push_back({static_cast<uint64_t>(nBig) * (small + 1), nBig, static_cast<uint32_t>(segs) - nBig, small,
                        small});
    }
    return runs;
}

uint64_t RhdSelectLoopCount(uint64_t remaining, uint64_t maxCountPerLoop, uint64_t p)
{
    const uint64_t count = std::min(remaining, maxCountPerLoop);
    return count >= p ? count / p * p : count;
}

HcclResult SequenceMaxCountPerLoop(uint64_t cclBytes, uint64_t count, uint32_t l0, uint32_t total, uint64_t elemSize,
                                   uint64_t align, bool rhdTail, uint64_t* maxCount, uint64_t* resultElems)
{
    if (l0 == 0 || total == 0 || elemSize == 0 || align == 0) {
        return HCCL_E_PARA;
    }
    uint64_t workspace = cclBytes;
    if (rhdTail && count % total != 0) {
        if (total > workspace / elemSize / 2) {
            return HCCL_E_INTERNAL;
        }
        const uint64_t slot = (total * elemSize + 127) / 128 * 128;
        if (slot >= workspace / 2) {
            return HCCL_E_INTERNAL;
        }
        workspace -= 2 * slot;
    }
    const uint64_t slice = workspace / (l0 + 1ull) / elemSize * elemSize;
    *resultElems = slice / elemSize;
    *maxCount = slice * l0 / align * align / elemSize / total * total;
    return *maxCount == 0 ? HCCL_E_INTERNAL : HCCL_SUCCESS;
}

uint64_t SequenceSelectLoopCount(uint64_t remaining, uint64_t maxCountPerLoop, uint32_t l0, uint64_t resultElems)
{
    if (remaining > maxCountPerLoop) {
        return maxCountPerLoop;
    }
    const uint64_t q = remaining / l0;
    const uint64_t r = remaining % l0;
    if (q + r <= resultElems || q == 0) {
        return remaining;
    }
    if (resultElems == 0) {
        return 0;
    }
    uint64_t newQ = q - 1;
    uint64_t newR = 0;
    if (newQ >= resultElems) {
        newQ = resultElems;
    } else {
        newR = std::min<uint64_t>(l0 - 1, resultElems - newQ);
    }
    return newQ * l0 + newR;
}

}  // namespace hccl_amd
