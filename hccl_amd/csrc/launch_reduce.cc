// Host layer, part 2: what a reduce collective launches.  The fold order comes from fold_plan.cc, the form of the
// launch (one fused kernel, fold + fan-out, wavefronts that share a tile's stores, load batch) from launch_policy.h.
#include <algorithm>
#include <cctype>
#include <chrono>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "algo_config.h"
#include "host.h"
#include "launch_policy.h"

namespace hccl_amd {

// ---------------------------------------------------------------------------------------------
// Launches.  `s` is the stream the fused kernel runs on.
// ---------------------------------------------------------------------------------------------
uint32_t BlocksPerSub(const World* w, uint64_t subLen, uint32_t esz, uint64_t nSubTotal, uint32_t threads)
{
    uint64_t vecs = (subLen * esz + 15) / 16 + kReduceLeadMask;   // lanes the kernel may skip to start on a 1 KiB boundary
    uint64_t maxUseful = (vecs + threads - 1) / threads;
    if (maxUseful == 0) maxUseful = 1;
    uint64_t want = (w->reduceBlocks + nSubTotal - 1) / nSubTotal;
    if (want == 0) want = 1;
    return static_cast<uint32_t>(want < maxUseful ? want : maxUseful);
}

// The launch described by its arguments alone (DirectFoldKernel): one result of one flat program of up to eight
// leaves that goes to two to eight destinations, every operand on a 16-byte boundary.  Returns the wavefronts per
// workgroup and fills `d`, or 0 where the launch is not of that shape or another form is asked for.
static uint32_t DirectFoldWaves(const World* w, const ReduceArgs& a, const DevicePlan& plan, uint32_t esz,
                                DirectFoldArgs* d)
{
    if (w->reduceDirect == 0 || !w->reduceVector || a.varGroups != 0 || a.dstOwn != 0 || a.nGroup != 1 || a.nSub != 1 ||
        a.nDst < 2 || a.nDst > kDirectFoldWideDst || a.total == 0 || plan.host == nullptr || plan.maxDepth != 1) {
        return 0;
    }
    const bool forced = w->reduceDirect > 0;
    if (!forced && (w->reduceThreads != 0 || w->storeWaves != 0 || w->reduceBatch != 0 || w->reducePair == 1 ||
                    w->reduceAllFold > 0 || w->storePolicy == 1 || w->reduceBlocks != kReduceBlocksDefault)) {
        return 0;   // a setting names another form
    }
    const uint64_t progOff = static_cast<uint64_t>(a.prog - plan.dev);
    if (a.prog < plan.dev || progOff % kDevProgBytes != 0 || progOff + kDevProgBytes > plan.host->size()) {
        return 0;
    }
    const uint8_t* img = plan.host->data() + progOff;
    const uint32_t leaves = img[0];
    if (leaves == 0 || leaves > kDirectFoldWideLeaves) {
        return 0;
    }
    const bool wide = leaves > kDirectFoldMaxLeaves || a.nDst > kDirectFoldMaxDst;
    *d = DirectFoldArgs{};
    for (uint32_t i = 0; i < leaves; ++i) {
        const uint32_t rank = img[kDevProgRankOff + i];
        if (img[kDevProgCtlOff + i] != 0 || rank >= w->n || a.src[rank] == nullptr ||
            (reinterpret_cast<uintptr_t>(a.src[rank]) & 15u) != 0) {
            return 0;
        }
        d->src[i] = a.src[rank];
    }
    for (uint32_t k = 0; k < a.nDst; ++k) {
        if (a.dst[k] == nullptr || (reinterpret_cast<uintptr_t>(a.dst[k]) & 15u) != 0) {
            return 0;
        }
        d->dst[k] = a.dst[k];
    }
    const uint32_t perVec = 16 / esz;
    d->nVec = a.total / perVec;
    d->tail = static_cast<uint32_t>(a.total % perVec);
    d->nSrc = leaves;
    d->nDst = a.nDst;
    if (wide) {
        // the kernel for nine to sixteen leaves or destinations takes whole workgroups only
        const uint32_t waves = forced ? static_cast<uint32_t>(w->reduceDirect)
                               : (reinterpret_cast<uintptr_t>(a.dst[0]) & 127u) != 0 ? 0u
                               : policy::DirectFoldWideWaves(leaves, a.nDst, a.total * esz);
        return waves != 0 && d->tail == 0 && d->nVec % (64ull * waves) == 0 ? waves : 0u;
    }
    if (forced) {
        return static_cast<uint32_t>(w->reduceDirect);
    }
    // by itself: where it was measured, and with tiles that are whole 128-byte lines of the first destination (the
    // general kernel deals its vectors to the lanes shifted so that they are; this one starts at the buffer's start)
    if ((reinterpret_cast<uintptr_t>(a.dst[0]) & 127u) != 0) {
        return 0;
    }
    return policy::DirectFoldWaves(leaves, a.nDst, a.total * esz);
}

HcclResult LaunchOneReduce(World* w, ReduceArgs& a, const DevicePlan& plan, HcclDataType dtype, HcclReduceOp op,
                           hipStream_t s)
{
    uint32_t esz = DataTypeSize(dtype);
    if (esz == 0) {
        return HCCL_E_INTERNAL;
    }
    {
        DirectFoldArgs d;
        uint32_t waves = DirectFoldWaves(w, a, plan, esz, &d);
        if (waves != 0) {
            uint32_t tiles = w->reduceDirectTiles != 0 ? static_cast<uint32_t>(w->reduceDirectTiles) : 1u;
            const bool wide = d.nSrc > kDirectFoldMaxLeaves || d.nDst > kDirectFoldMaxDst;
            if (!wide && w->reduceDirectTiles == 0 && w->reduceDirect < 0 && policy::DirectFoldTwoTiles(d.nSrc, d.nDst, a.total * esz)) {
                waves = 8;
                tiles = 2;
            }
            HIP_OK(LaunchDirectFold(d, dtype, op, waves, tiles, s));
            return HCCL_SUCCESS;
        }
    }
    // 128-bit loads and stores may start on any element (the head is peeled for the first destination, which
    // makes every store aligned in the usual case of equally aligned recvBufs).  HCCL_AMD_REDUCE_VECTOR=0
    // forces the element-by-element path.
    a.vecOk = w->reduceVector ? 1u : 0u;
    uint64_t subs = static_cast<uint64_t>(a.nGroup) * a.nSub;
    uint64_t longest = a.groupLen;   // the last sub-segment takes what the others leave
    if (a.nSub > 1) {
        uint64_t before = a.subLen * (a.nSub - 1);
        uint64_t last = a.groupLen > before ? a.groupLen - before : 0;
        longest = last > a.subLen ? last : a.subLen;
    }
    // The form of the launch (workgroup size, store policy, load batch, wavefronts that share a tile's stores):
    // launch_policy.h, with the measurements behind every choice; the world's settings override.
    const bool oneStream = a.dstOwn || a.nDst == 1;
    a.writeThrough = w->storePolicy != 2 ? w->storePolicy : (policy::WriteThrough(oneStream) ? 1u : 0u);
    // Many sources folded into one result stream: the wavefronts start on the sources' 1 KiB boundaries (a
    // ReduceScatterV slice begins wherever its displacement puts it; measured 0.74 -> 0.80 of peak on uneven
    // slices) and the single store stream straddles.  HCCL_AMD_LEAD_FROM_SRC=0 keeps the destination's lines.
    a.leadFromSrc = (oneStream && w->leadFromSrc) ? 1u : 0u;
    a.vecBatch = w->reduceBatch != 0 ? w->reduceBatch : policy::VecBatch(w->n, oneStream, a.varGroups != 0);
    a.threads = w->reduceThreads != 0 ? w->reduceThreads : policy::kReduceThreads;
    a.storeWaves = 1;
    if (!oneStream && a.threads == 64 && a.vecOk) {
        uint32_t waves = policy::StoreWaves(a.nDst, a.total * esz, esz);
        if (w->storeWaves != 0) {
            waves = w->storeWaves < a.nDst ? w->storeWaves : a.nDst;
        }
        a.storeWaves = waves;
        if (waves > 1 && w->reduceBatch == 0) {
            a.vecBatch = policy::VecBatchWithSharedStores(w->n, a.vecBatch);
        }
    }
    a.blocksPerSub = BlocksPerSub(w, longest, a.vecOk ? esz : 16 /* one element per lane */, subs, a.threads);
    uint32_t exchangeLds = 0;
    if (a.vecOk && a.threads == 64 && a.storeWaves <= 1 && !oneStream && !a.varGroups && plan.maxDepth == 1 &&
        w->reduceAllFold != 0 && w->storeWaves == 0) {
        // every wavefront folds a tile and stores the tiles of its workgroup to its own destinations (forced: wherever
        // the form fits; by itself: where it was measured, a result that is one sub-segment)
        const uint32_t waves = w->reduceAllFold > 0 ? static_cast<uint32_t>(w->reduceAllFold)
                               : (subs == 1 && w->reduceBatch == 0 && w->reducePair != 1)
                                     ? policy::AllFoldWaves(a.nDst, a.total * esz) : 0u;
        if (waves > 1) {
            a.vecBatch = 8;   // the form exists in the eight-leaf kernels
            a.storeWaves = waves | kStoreWavesAllFold;
            a.blocksPerSub = (a.blocksPerSub + waves - 1) / waves;   // a workgroup takes `waves` tiles
            exchangeLds = 2u * waves * 1024u;
        }
    }
    if (a.vecOk && a.threads == 64 && a.storeWaves <= 1 && !a.varGroups && plan.maxLeaves <= 8 && plan.maxDepth == 1 &&
        (w->reduceBatch == 0 || w->reducePair == 1) &&
        (w->reducePair != 2 ? w->reducePair == 1 : policy::PairTiles(w->n, oneStream, a.total * esz))) {
        a.vecBatch = kVecBatchPair;
        a.blocksPerSub = (a.blocksPerSub + 1) / 2;   // a workgroup takes two tiles
    }
    uint64_t blocks = subs * a.blocksPerSub;
    if (a.varGroups) {
        // every group gets the workgroups its own length needs (an empty group gets none)
        blocks = 0;
        for (uint32_t g = 0; g < a.nGroup; ++g) {
            if (a.groupLenV[g] != 0) {
                blocks += BlocksPerSub(w, a.groupLenV[g], a.vecOk ? esz : 16, subs, a.threads);
            }
            a.groupBlockEnd[g] = static_cast<uint32_t>(blocks < 0x7FFFFFFFull ? blocks : 0x7FFFFFFFull);
        }
        for (uint32_t g = a.nGroup; g < 16; ++g) {
            a.groupBlockEnd[g] = 0xFFFFFFFFu;   // the kernel reads sixteen entries in one go when there are that few groups
        }
    }
    if (blocks == 0 || blocks > 0x7FFFFFFFull) {
        return HCCL_E_INTERNAL;
    }
    const uint32_t lds = exchangeLds != 0 ? exchangeLds : (plan.maxDepth - 1) * ReduceAccBytes(dtype, op) * a.threads;
    HIP_OK(LaunchReduce(a, dtype, op, static_cast<uint32_t>(blocks), lds, s));
    return HCCL_SUCCESS;
}

// HCCL_DETERMINISTIC=strict moves float SUM / PROD over more than two ranks to the order-preserved fold
// (reference src/common/order_preserved_common.h:104-114).  The reference offers its write-reduce templates
// (NHR, RHD, mesh chunk) and the vector-core mesh neither PROD nor 64-bit types (REGISTER_ALG_ATTRS in
// ins_v2_all_reduce_sole_executor.cc:401-431, ins_v2_reduce_scatter_sole_executor.cc:377-476, filtered by
// op_common/selector/cost_table.cc:104-131) and its selector then lands on the host-reduce mesh templates, so
// those combinations fold in the MESH order here too.  Everything else keeps the configured algorithm.
HcclAmdAlgo EffectiveAlgo(const World* w, HcclAmdOpKind kind, HcclDataType dtype, HcclReduceOp op)
{
    const bool isFloat = dtype == HCCL_DATA_TYPE_FP16 || dtype == HCCL_DATA_TYPE_FP32 ||
                         dtype == HCCL_DATA_TYPE_BFP16 || dtype == HCCL_DATA_TYPE_FP64;
    if (w->deterministic == 2 && isFloat && (op == HCCL_REDUCE_SUM || op == HCCL_REDUCE_PROD) && w->n > 2) {
        return HCCL_AMD_ALGO_ORDER_PRESERVED;
    }
    const HcclAmdAlgo algo = w->algo[kind];
    const bool hostOnly = op == HCCL_REDUCE_PROD || dtype == HCCL_DATA_TYPE_INT64 || dtype == HCCL_DATA_TYPE_UINT64 ||
                          dtype == HCCL_DATA_TYPE_FP64;
    if (hostOnly && (algo == HCCL_AMD_ALGO_NHR || algo == HCCL_AMD_ALGO_RHD || algo == HCCL_AMD_ALGO_MESH_CHUNK ||
                     algo == HCCL_AMD_ALGO_AIV_MESH || algo == HCCL_AMD_ALGO_MESH_CONCUR ||
                     (algo == HCCL_AMD_ALGO_RING && kind == HCCL_AMD_OP_REDUCE_SCATTER))) {
        return HCCL_AMD_ALGO_MESH;
    }
    return algo;
}

// Mesh-chunk order: one launch per run of equally long segments.  `nGroup` slices of `len` elements start
// `sliceStride` elements apart from element `base` of every send buffer; slice g is slice firstSlice + g of the
// plan.  The results go to dst[...] + dstBase (+ g * sliceStride when every destination receives every slice).
HcclResult LaunchMeshChunk(World* w, const DevicePlan& plan, const PendingOp& p, ReduceArgs a, uint32_t firstSlice,
                           uint32_t nGroup, uint64_t len, uint64_t sliceStride, bool alignTo4K, hipStream_t s)
{
    const uint32_t n = w->n;
    const uint32_t esz = DataTypeSize(p.dtype);
    const uint32_t segs = n - 1;
    for (const SegmentRun& run : MeshChunkSegments(len, n, esz, alignTo4K)) {
        ReduceArgs r = a;
        for (uint32_t k = 0; k < n; ++k) {
            r.src[k] = static_cast<const uint8_t*>(a.src[k]) + run.first * esz;
            if (a.dst[k] != nullptr) {
                r.dst[k] = static_cast<uint8_t*>(a.dst[k]) + run.first * esz;
            }
        }
        r.prog = plan.dev + (static_cast<uint64_t>(firstSlice) * segs + run.firstSeg) * kDevProgBytes;
        r.progGroupStride = segs;
        r.progSubStride = 1;
        r.nGroup = nGroup;
        r.nSub = run.nSeg;
        r.subLen = run.segLen;
        r.groupLen = run.segLen * (run.nSeg - 1) + run.lastLen;
        r.total = r.groupLen * nGroup;
        r.srcGroupStride = sliceStride;
        r.dstGroupStride = sliceStride;
        HcclResult rc = LaunchOneReduce(w, r, plan, p.dtype, p.op, s);
        if (rc != HCCL_SUCCESS) {
            return rc;
        }
    }
    return HCCL_SUCCESS;
}

// A result that every rank receives, as two kernels per piece: the fold of all ranks into the first rank's recvBuf
// (N reads and one write, the shape of a ReduceScatter launch), then that range, just written and therefore still in
// the last-level cache, to the other recvBufs with one wavefront per destination stream.  Exactly the algorithmic
// traffic, no memory of the library's own, same fold program and same bits as the fused kernel.  Reads and writes
// each run near what the part gives them alone, where the fused kernel, whose wavefronts store to every destination
// after loading from every source, reaches 0.70-0.78 (launch_policy.h has the table).
bool FoldThenFanOut(const World* w, uint32_t nDst, uint64_t bytes)
{
    if (nDst < 2) {
        return false;
    }
    if (w->twoKernelMode != 2) {
        return w->twoKernelMode == 1;
    }
    return policy::FoldThenFanOut(nDst, bytes);
}

// Second kernel of the two-kernel forms: bytes [off, off + bytes) of dst[0], just written, to the same range of
// dst[1 .. nDst).  Destinations that differ from dst[0] modulo 16 take the general copy.
HcclResult FanOutFromFirst(World* w, void* const* dst, uint32_t nDst, uint64_t off, uint64_t bytes, bool severalPieces,
                           hipStream_t s)
{
    if (nDst < 2 || bytes == 0) {
        return HCCL_SUCCESS;
    }
    FanOutArgs f{};
    f.src = static_cast<const uint8_t*>(dst[0]) + off;
    f.bytes = bytes;
    f.nDst = nDst - 1;
    for (uint32_t k = 1; k < nDst; ++k) {
        f.dst[k - 1] = static_cast<uint8_t*>(dst[k]) + off;
    }
    if (FanOutTakes(f)) {
        HIP_OK(LaunchFanOut(f, w->fanOutLoadMode != 2 ? w->fanOutLoadMode == 1 : policy::FanOutStreamLoad(f.nDst, severalPieces), s));
        return HCCL_SUCCESS;
    }
    BcastCopyArgs b{};
    b.nSeg = 1;
    b.src[0] = f.src;
    b.len[0] = bytes;
    b.dstOff[0] = 0;
    b.nDst = f.nDst;
    for (uint32_t k = 0; k < f.nDst; ++k) {
        b.dst[k] = f.dst[k];
    }
    return RunBcast(w, b, s);
}

// Launch of a fold whose result [0, a.total) goes to all a.nDst destinations (a.nGroup == 1, a.dstOwn == 0): the
// fused kernel, or fold + fan-out per piece.  Pieces are whole sub-segments while those fit (each has its own fold
// program), and parts of a sub-segment that is longer than a piece.
HcclResult LaunchToAll(World* w, const ReduceArgs& a, const DevicePlan& plan, HcclDataType dtype, HcclReduceOp op,
                       hipStream_t s)
{
    const uint32_t esz = DataTypeSize(dtype);
    if (esz == 0) {
        return HCCL_E_INTERNAL;   // the entry points admit known types only
    }
    if (a.nGroup != 1 || a.dstOwn != 0 || a.varGroups != 0 || !FoldThenFanOut(w, a.nDst, a.total * esz)) {
        ReduceArgs fused = a;
        return LaunchOneReduce(w, fused, plan, dtype, op, s);
    }
    const uint64_t pieceEl = std::max<uint64_t>(1, w->pieceBytes / esz);
    auto piece = [&](uint32_t firstSub, uint32_t nSub, uint64_t begin, uint64_t len) -> HcclResult {
        if (len == 0) {
            return HCCL_SUCCESS;
        }
        ReduceArgs r = a;
        for (uint32_t k = 0; k < w->n; ++k) {
            r.src[k] = static_cast<const uint8_t*>(a.src[k]) + begin * esz;
        }
        for (uint32_t k = 0; k < static_cast<uint32_t>(kMaxRanks); ++k) {
            r.dst[k] = nullptr;
        }
        uint8_t* first = static_cast<uint8_t*>(a.dst[0]) + begin * esz;
        r.dst[0] = first;
        r.nDst = 1;
        r.prog = a.prog + static_cast<uint64_t>(firstSub) * a.progSubStride * kDevProgBytes;
        r.nSub = nSub;
        r.total = r.groupLen = len;
        if (nSub == 1) {
            r.subLen = len;
        }
        HcclResult rc = LaunchOneReduce(w, r, plan, dtype, op, s);
        if (rc != HCCL_SUCCESS) {
            return rc;
        }
        return FanOutFromFirst(w, a.dst, a.nDst, begin * esz, len * esz, a.total > pieceEl, s);
    };
    uint32_t heldFirst = 0;     // sub-segments [heldFirst, c) wait for their launch
    uint64_t heldBegin = 0;
    uint64_t heldLen = 0;
    for (uint32_t c = 0; c < a.nSub; ++c) {
        const uint64_t sBeg = static_cast<uint64_t>(c) * a.subLen;
        uint64_t sEnd = (c == a.nSub - 1) ? a.total : sBeg + a.subLen;
        sEnd = sEnd < a.total ? sEnd : a.total;
        const uint64_t len = sEnd > sBeg ? sEnd - sBeg : 0;
        if (heldLen + len > pieceEl && heldLen != 0) {
            HcclResult rc = piece(heldFirst, c - heldFirst, heldBegin, heldLen);
            if (rc != HCCL_SUCCESS) {
                return rc;
            }
            heldLen = 0;
        }
        if (len > pieceEl) {
            for (uint64_t at = 0; at < len; at += pieceEl) {
                HcclResult rc = piece(c, 1, sBeg + at, std::min(pieceEl, len - at));
                if (rc != HCCL_SUCCESS) {
                    return rc;
                }
            }
            continue;
        }
        if (heldLen == 0) {
            heldFirst = c;
            heldBegin = sBeg;
        }
        heldLen += len;
    }
    if (heldLen != 0) {
        return piece(heldFirst, a.nSub - heldFirst, heldBegin, heldLen);
    }
    return HCCL_SUCCESS;
}

// The cut of the sequence executors whose chunks are floor(len / d) elements with the rest in the last one, level
// after level (reference ins_v2_all_reduce_sequence_3level_utils.h:124-126, 150-160,
// ins_v2_all_reduce_sequence_executor_aicpu_3level.cc:361-370): `dims` are the level sizes from level 0 on, program
// progBase + ((i * d1 + j) * d2 + k) belongs to part k of sub-slice j of chunk i.  launch(program, nSub, begin, len,
// subLen) receives runs of nSub neighbouring units of subLen elements, the last one longer by what is left of len.
template <class Launch>
HcclResult CutByLevels(const uint32_t* dims, uint32_t nDims, uint32_t progBase, uint64_t begin, uint64_t len,
                       Launch&& launch)
{
    if (len == 0) {
        return HCCL_SUCCESS;
    }
    const uint32_t d = dims[0];
    if (nDims == 1) {
        const uint64_t sub = len / d;
        // fewer elements than units: all of them belong to the last unit
        return sub == 0 ? launch(progBase + d - 1, 1u, begin, len, len) : launch(progBase, d, begin, len, sub);
    }
    uint32_t below = 1;
    for (uint32_t k = 1; k < nDims; ++k) {
        below *= dims[k];
    }
    const uint64_t chunk = len / d;
    if (chunk != 0 && chunk * d == len && chunk % below == 0) {
        return launch(progBase, d * below, begin, len, chunk / below);   // every unit equally long: one run
    }
    for (uint32_t i = 0; i < d; ++i) {
        const uint64_t cur = i == d - 1 ? len - static_cast<uint64_t>(i) * chunk : chunk;
        HcclResult rc = CutByLevels(dims + 1, nDims - 1, progBase + i * below, begin + static_cast<uint64_t>(i) * chunk, cur,
                                    launch);
        if (rc != HCCL_SUCCESS) {
            return rc;
        }
    }
    return HCCL_SUCCESS;
}

// The levels of a world as CutByLevels takes them (a level of one participant cuts nothing and is left out).
uint32_t LevelDims(const Levels& lv, uint32_t* dims)
{
    uint32_t nDims = 0;
    dims[nDims++] = lv.l0;
    if (lv.l1 > 1) {
        dims[nDims++] = lv.l1;
    }
    if (lv.l2 > 1) {
        dims[nDims++] = lv.l2;
    }
    return nDims;
}

HcclResult RunAllReduce(World* w, PendingOp& p, hipStream_t s)
{
    const uint32_t n = w->n;
    HcclAmdAlgo algo = EffectiveAlgo(w, HCCL_AMD_OP_ALL_REDUCE, p.dtype, p.op);
    // A world with level-0 groups runs the step-driven orders in two levels: a mesh ReduceScatter inside every
    // group, the configured template between the groups (reference
    // ins_v2_all_reduce_sequence_executor_aicpu.cc:592-852), and in three when the groups form level-1 groups
    // (ins_v2_all_reduce_sequence_executor_aicpu_3level.cc).  The types the reference reduces on the host take its
    // host-reduce template between the groups, which folds the own share first (EffectiveAlgo has turned their
    // RHD / NHR into MESH; a configured sequence{mesh, nhr_aicpu_reduce} asks for the same); that executor knows
    // two levels only.
    const HcclAmdAlgo configured = w->algo[HCCL_AMD_OP_ALL_REDUCE];
    const bool stepDriven = configured == HCCL_AMD_ALGO_RHD || configured == HCCL_AMD_ALGO_NHR;
    Levels lv;
    const bool twoLevel = ResolveLevels(n, w->level0, algo == HCCL_AMD_ALGO_MESH ? 0 : w->level1, &lv) &&
                          w->allReduceSequence != 0 &&
                          (algo == HCCL_AMD_ALGO_RHD || algo == HCCL_AMD_ALGO_NHR ||
                           (algo == HCCL_AMD_ALGO_MESH && (stepDriven || w->allReduceSequence == 1)));
    DevicePlan plan;
    HcclResult rc = GetDevicePlan(w, HCCL_AMD_OP_ALL_REDUCE, algo, &plan, twoLevel ? lv.l0 : 1, twoLevel ? w->level1 : 0);
    if (rc != HCCL_SUCCESS) {
        return rc;
    }
    const uint32_t esz = DataTypeSize(p.dtype);
    ReduceArgs a{};
    for (uint32_t r = 0; r < n; ++r) {
        a.src[r] = p.ranks[r].send;
        a.dst[r] = p.ranks[r].recv;
    }
    a.prog = plan.dev;
    a.nDst = n;
    a.dstOwn = 0;
    a.nGroup = 1;
    if (plan.nProg == 1) {
        a.total = a.groupLen = a.subLen = p.count;
        a.nSub = 1;
        return LaunchToAll(w, a, plan, p.dtype, p.op, s);
    }
    if (algo == HCCL_AMD_ALGO_MESH_CHUNK) {
        // Slices of ceil(len / n) elements, short or empty towards the end (reference
        // ins_temp_all_reduce_mesh_1D_two_shot_mesh_chunk.cc:86-112); the executor loops over half of the
        // staging buffer (:55-62, ins_v2_all_reduce_sole_executor.cc:241-300).
        uint64_t maxPerLoop = p.count;
        if (w->cclBytes != 0) {
            maxPerLoop = SoleMaxCountPerLoop(w->cclBytes, 2, esz);
            if (maxPerLoop == 0) {
                return HCCL_E_INTERNAL;
            }
        }
        for (uint64_t done = 0; done < p.count;) {
            const uint64_t len = std::min(p.count - done, maxPerLoop);
            const uint64_t slice = (len + n - 1) / n;
            const uint32_t nFull = static_cast<uint32_t>(len / slice);
            for (uint32_t r = 0; r < n; ++r) {
                a.src[r] = static_cast<const uint8_t*>(p.ranks[r].send) + done * esz;
                a.dst[r] = static_cast<uint8_t*>(p.ranks[r].recv) + done * esz;
            }
            if (FoldThenFanOut(w, n, len * esz) && slice * esz <= w->pieceBytes &&
                (n >= policy::kMeshChunkFanOutMinRanks || w->twoKernelMode == 1)) {
                // Fold + fan-out per piece of whole slices: the launches of a piece write rank 0's recvBuf only,
                // then that range goes to the other recvBufs (fp32, 8 ranks of 256 MiB: 0.74 -> 0.81 of the HBM peak,
                // 16 ranks of 64 MiB: 0.71 -> 0.79; six ranks lose, 0.74 -> 0.71, and keep the fused kernel).
                const uint64_t rest = len - static_cast<uint64_t>(nFull) * slice;
                const uint32_t perPiece = static_cast<uint32_t>(std::max<uint64_t>(1, w->pieceBytes / esz / slice));
                for (uint32_t g0 = 0; g0 < nFull; g0 += perPiece) {   // nFull >= 1: a slice is never longer than the loop
                    const uint32_t g1 = std::min(nFull, g0 + perPiece);
                    const uint64_t begin = static_cast<uint64_t>(g0) * slice;
                    uint64_t pieceLen = static_cast<uint64_t>(g1 - g0) * slice;
                    ReduceArgs f = a;
                    f.nDst = 1;
                    for (uint32_t r = 0; r < n; ++r) {
                        f.src[r] = static_cast<const uint8_t*>(a.src[r]) + begin * esz;
                        f.dst[r] = r == 0 ? static_cast<uint8_t*>(a.dst[0]) + begin * esz : nullptr;
                    }
                    rc = LaunchMeshChunk(w, plan, p, f, g0, g1 - g0, slice, slice, false, s);
                    if (rc != HCCL_SUCCESS) {
                        return rc;
                    }
                    if (g1 == nFull && rest != 0) {   // the short last slice rides with the last piece
                        ReduceArgs t = a;
                        t.nDst = 1;
                        for (uint32_t r = 0; r < n; ++r) {
                            t.src[r] = static_cast<const uint8_t*>(a.src[r]) + static_cast<uint64_t>(nFull) * slice * esz;
                            t.dst[r] = r == 0 ? static_cast<uint8_t*>(a.dst[0]) + static_cast<uint64_t>(nFull) * slice * esz : nullptr;
                        }
                        rc = LaunchMeshChunk(w, plan, p, t, nFull, 1, rest, 0, false, s);
                        if (rc != HCCL_SUCCESS) {
                            return rc;
                        }
                        pieceLen += rest;
                    }
                    rc = FanOutFromFirst(w, a.dst, n, begin * esz, pieceLen * esz, nFull > perPiece, s);
                    if (rc != HCCL_SUCCESS) {
                        return rc;
                    }
                }
                done += len;
                continue;
            }
            if (nFull != 0) {
                rc = LaunchMeshChunk(w, plan, p, a, 0, nFull, slice, slice, false, s);
                if (rc != HCCL_SUCCESS) {
                    return rc;
                }
            }
            const uint64_t rest = len - static_cast<uint64_t>(nFull) * slice;
            if (rest != 0) {
                for (uint32_t r = 0; r < n; ++r) {
                    a.src[r] = static_cast<const uint8_t*>(a.src[r]) + static_cast<uint64_t>(nFull) * slice * esz;
                    a.dst[r] = static_cast<uint8_t*>(a.dst[r]) + static_cast<uint64_t>(nFull) * slice * esz;
                }
                rc = LaunchMeshChunk(w, plan, p, a, nFull, 1, rest, 0, false, s);
                if (rc != HCCL_SUCCESS) {
                    return rc;
                }
            }
            done += len;
        }
        return HCCL_SUCCESS;
    }
    a.nSub = n;
    a.progSubStride = 1;
    // One launch per loop of the reference's executor: elements [done, done + len) cut into n sub-segments of
    // `unit` elements, the last one taking what the others leave.
    auto launchLoop = [&](uint64_t done, uint64_t len, uint64_t unit) {
        for (uint32_t r = 0; r < n; ++r) {
            a.src[r] = static_cast<const uint8_t*>(p.ranks[r].send) + done * esz;
            a.dst[r] = static_cast<uint8_t*>(p.ranks[r].recv) + done * esz;
        }
        a.total = a.groupLen = len;
        a.subLen = unit;
        return LaunchToAll(w, a, plan, p.dtype, p.op, s);
    };
    if (twoLevel && algo != HCCL_AMD_ALGO_RHD) {
        // Between the groups NHR, or the host-reduce fold: every loop is cut into level0 chunks of floor(len / level0)
        // elements, the last chunk taking the rest, every chunk into sub-slices the same way and, with three levels,
        // every sub-slice into parts (reference ins_v2_all_reduce_sequence_executor_aicpu.cc:413-415, 445-455).
        // Two levels: the loops hold what fits half the staging buffer, floored to 128 bytes and to a multiple of n
        // elements (:653-656); three: SequenceMaxCountPerLoop.
        uint64_t maxPerLoop = p.count;
        uint64_t resultElems = ~0ull;
        if (w->cclBytes != 0) {
            if (lv.l2 > 1) {
                rc = SequenceMaxCountPerLoop(w->cclBytes, p.count, lv.l0, n, esz, 128, false, &maxPerLoop, &resultElems);
            } else {
                maxPerLoop = w->cclBytes / 2 / 128 * 128 / esz / n * n;
                rc = maxPerLoop == 0 ? HCCL_E_INTERNAL : HCCL_SUCCESS;
            }
            if (rc != HCCL_SUCCESS) {
                Log(1, "AllReduce: the staging buffer of %llu bytes holds no loop of the %s-level order",
                    static_cast<unsigned long long>(w->cclBytes), lv.l2 > 1 ? "three" : "two");
                return HCCL_E_INTERNAL;
            }
        }
        uint32_t dims[3];
        const uint32_t nDims = LevelDims(lv, dims);
        auto launch = [&](uint32_t prog, uint32_t nSub, uint64_t begin, uint64_t len, uint64_t subLen) {
            for (uint32_t r = 0; r < n; ++r) {
                a.src[r] = static_cast<const uint8_t*>(p.ranks[r].send) + begin * esz;
                a.dst[r] = static_cast<uint8_t*>(p.ranks[r].recv) + begin * esz;
            }
            a.prog = plan.dev + static_cast<uint64_t>(prog) * kDevProgBytes;
            a.nSub = nSub;
            a.total = a.groupLen = len;
            a.subLen = subLen;
            return LaunchToAll(w, a, plan, p.dtype, p.op, s);
        };
        for (uint64_t done = 0; done < p.count;) {
            const uint64_t len = lv.l2 > 1 ? SequenceSelectLoopCount(p.count - done, maxPerLoop, lv.l0, resultElems)
                                           : std::min(p.count - done, maxPerLoop);
            if (len == 0) {
                return HCCL_E_INTERNAL;
            }
            rc = CutByLevels(dims, nDims, 0, done, len, launch);
            if (rc != HCCL_SUCCESS) {
                return rc;
            }
            done += len;
        }
        return HCCL_SUCCESS;
    }
    if (algo == HCCL_AMD_ALGO_RHD) {
        // (With level-0 groups the frame is the same: unit u = i * (n / level0) + j is sub-slice j of chunk i, with
        // three levels unit (i * l1 + j) * l2 + k part k of it, and the remainder shorter than n is padded to one
        // element per unit; only the programs differ, and the share of the buffer a three-level loop may fill.)
        // Whole frames of n uniform units while they last, then a remainder shorter than n with one element per
        // unit (reference ins_v2_all_reduce_sequence_rhd_tail.h:94-113); a bounded staging buffer limits the
        // frames one loop holds.
        uint64_t maxPerLoop = ~0ull / 2 / n * n;
        if (w->cclBytes != 0) {
            uint64_t resultElems = 0;
            rc = twoLevel && lv.l2 > 1
                     ? SequenceMaxCountPerLoop(w->cclBytes, p.count, lv.l0, n, esz, 128, true, &maxPerLoop, &resultElems)
                     : RhdMaxCountPerLoop(w->cclBytes, p.count, n, esz, &maxPerLoop);
            if (rc != HCCL_SUCCESS) {
                Log(1, "AllReduce: the staging buffer of %llu bytes holds no loop of the RHD order",
                    static_cast<unsigned long long>(w->cclBytes));
                return rc;
            }
        }
        for (uint64_t done = 0; done < p.count;) {
            const uint64_t valid = RhdSelectLoopCount(p.count - done, maxPerLoop, n);
            rc = launchLoop(done, valid, valid >= n ? valid / n : 1);
            if (rc != HCCL_SUCCESS) {
                return rc;
            }
            done += valid;
        }
        return HCCL_SUCCESS;
    }
    if (algo == HCCL_AMD_ALGO_NHR) {
        // Slices of floor(len / n) elements, the last slice takes the rest (reference
        // ins_temp_all_reduce_nhr.cc:214-216); the executor loops over the staging buffer, which this template
        // uses once (scratch multiple 1, reference ins_temp_all_reduce_nhr.cc:65-71,
        // ins_v2_all_reduce_sole_executor.cc:241-300).
        uint64_t maxPerLoop = p.count;
        if (w->cclBytes != 0) {
            maxPerLoop = SoleMaxCountPerLoop(w->cclBytes, 1, esz);
            if (maxPerLoop == 0) {
                Log(1, "AllReduce: the staging buffer of %llu bytes holds no element",
                    static_cast<unsigned long long>(w->cclBytes));
                return HCCL_E_INTERNAL;
            }
        }
        for (uint64_t done = 0; done < p.count;) {
            const uint64_t len = std::min(p.count - done, maxPerLoop);
            rc = launchLoop(done, len, len / n);
            if (rc != HCCL_SUCCESS) {
                return rc;
            }
            done += len;
        }
        return HCCL_SUCCESS;
    }
    if (algo == HCCL_AMD_ALGO_MESH_CONCUR) {
        // Slices of floor(len / n) elements, the last slice takes the rest; loops of half the staging buffer,
        // floored to 128 bytes and a multiple of n elements (reference
        // ins_v2_all_reduce_two_shot_sole_executor.cc:236-237, 328-340).
        uint64_t maxPerLoop = p.count;
        if (w->cclBytes != 0) {
            maxPerLoop = w->cclBytes / 2 / 128 * 128 / esz / n * n;
            if (maxPerLoop == 0) {
                Log(1, "AllReduce: the staging buffer of %llu bytes holds no loop of the mesh two-shot executor",
                    static_cast<unsigned long long>(w->cclBytes));
                return HCCL_E_INTERNAL;
            }
        }
        for (uint64_t done = 0; done < p.count;) {
            const uint64_t len = std::min(p.count - done, maxPerLoop);
            rc = launchLoop(done, len, len / n);
            if (rc != HCCL_SUCCESS) {
                return rc;
            }
            done += len;
        }
        return HCCL_SUCCESS;
    }
    // Symmetric two-shot: slices of ceil(count / n) elements (reference two_shot.cc:184), always in one loop
    // (reference ins_v2_all_reduce_sole_executor.cc:273-282).
    return launchLoop(0, p.count, (p.count + n - 1) / n);
}

HcclResult RunReduceScatter(World* w, PendingOp& p, hipStream_t s)
{
    const uint32_t n = w->n;
    HcclAmdAlgo algo = EffectiveAlgo(w, HCCL_AMD_OP_REDUCE_SCATTER, p.dtype, p.op);
    // A world with level-0 groups runs the step-driven orders in two or three levels, as AllReduce does (reference
    // ins_v2_reduce_scatter_sequence_executor_aicpu.cc:298-372, ins_v2_reduce_scatter_sequence_executor_3level.cc):
    // the mesh ReduceScatter inside every group, the configured template between the groups, the own-first host-reduce
    // fold there for the types the reference reduces on the host.  Every rank's output keeps one program, so the
    // launch is the one-level one.
    const HcclAmdAlgo configured = w->algo[HCCL_AMD_OP_REDUCE_SCATTER];
    const bool stepDriven = configured == HCCL_AMD_ALGO_RHD || configured == HCCL_AMD_ALGO_NHR;
    Levels lv;
    const bool twoLevel = ResolveLevels(n, w->level0, algo == HCCL_AMD_ALGO_MESH ? 0 : w->level1, &lv) &&
                          w->reduceScatterSequence != 0 &&
                          (algo == HCCL_AMD_ALGO_RHD || algo == HCCL_AMD_ALGO_NHR ||
                           (algo == HCCL_AMD_ALGO_MESH && (stepDriven || w->reduceScatterSequence == 1)));
    DevicePlan plan;
    HcclResult rc = GetDevicePlan(w, HCCL_AMD_OP_REDUCE_SCATTER, algo, &plan, twoLevel ? lv.l0 : 1,
                                  twoLevel ? w->level1 : 0);
    if (rc != HCCL_SUCCESS) {
        return rc;
    }
    ReduceArgs a{};
    for (uint32_t r = 0; r < n; ++r) {
        a.src[r] = p.ranks[r].send;
        a.dst[r] = p.ranks[r].recv;
    }
    a.prog = plan.dev;
    a.nDst = 1;
    a.dstOwn = 1;
    if (algo == HCCL_AMD_ALGO_MESH_CHUNK) {
        // The executor loops over the staging buffer, of which this template keeps n - 1 slots (reference
        // ins_temp_reduce_scatter_mesh_1D_meshchunk.cc:119-125, ins_v2_reduce_scatter_sole_executor.cc:212-277);
        // every loop cuts its share of each rank's output into segments of its own.
        const uint32_t esz = DataTypeSize(p.dtype);
        uint64_t maxPerLoop = p.count;
        if (w->cclBytes != 0) {
            maxPerLoop = SoleMaxCountPerLoop(w->cclBytes, n - 1, esz);
            if (maxPerLoop == 0) {
                return HCCL_E_INTERNAL;
            }
        }
        for (uint64_t done = 0; done < p.count;) {
            const uint64_t len = std::min(p.count - done, maxPerLoop);
            for (uint32_t r = 0; r < n; ++r) {
                a.src[r] = static_cast<const uint8_t*>(p.ranks[r].send) + done * esz;
                a.dst[r] = static_cast<uint8_t*>(p.ranks[r].recv) + done * esz;
            }
            rc = LaunchMeshChunk(w, plan, p, a, 0, n, len, p.count, true, s);
            if (rc != HCCL_SUCCESS) {
                return rc;
            }
            done += len;
        }
        return HCCL_SUCCESS;
    }
    a.nGroup = n;
    a.groupLen = p.count;                  // input slice stride = recvCount (reference
    a.srcGroupStride = p.count;            // ins_v2_reduce_scatter_sole_executor.cc:260)
    a.total = static_cast<uint64_t>(n) * p.count;
    if (plan.segmentsAreSubs && plan.nProg > 1) {
        a.nSub = n;                        // vector-core mesh: output cut into n chunks
        a.subLen = p.count / n;
        a.progSubStride = 1;
    } else {
        a.nSub = 1;
        a.subLen = p.count;
        a.progGroupStride = plan.nProg > 1 ? 1 : 0;
    }
    return LaunchOneReduce(w, a, plan, p.dtype, p.op, s);
}

// ReduceScatterV, mesh order: rank k's output = in_k[displs[k] ..] first, then the other ranks ascending
// (reference ins_temp_reduce_scatter_v_mesh_1D.cc:109-162).  Every rank must pass the same counts / displs.
HcclResult RunReduceScatterV(World* w, PendingOp& p, hipStream_t s)
{
    const uint32_t n = w->n;
    const std::vector<uint64_t>& ref = p.ranks[0].var;   // counts | displs | recvCount
    uint64_t longest = 0;
    for (uint32_t r = 0; r < n; ++r) {
        const std::vector<uint64_t>& v = p.ranks[r].var;
        if (memcmp(v.data(), ref.data(), 2 * n * sizeof(uint64_t)) != 0) {
            Log(1, "ReduceScatterV: rank %u passed sendCounts / sendDispls that differ from rank 0", r);
            return HCCL_E_PARA;
        }
        if (v[2 * n] != ref[r]) {
            Log(1, "ReduceScatterV: rank %u recvCount %llu != sendCounts[%u] %llu", r, (unsigned long long)v[2 * n], r,
                (unsigned long long)ref[r]);
            return HCCL_E_PARA;
        }
        if (ref[r] != 0 && (p.ranks[r].send == nullptr || p.ranks[r].recv == nullptr)) {
            return HCCL_E_PTR;
        }
        longest = ref[r] > longest ? ref[r] : longest;
    }
    if (longest == 0) {
        return HCCL_SUCCESS;
    }
    const bool meshChunk = EffectiveAlgo(w, HCCL_AMD_OP_REDUCE_SCATTER, p.dtype, p.op) == HCCL_AMD_ALGO_MESH_CHUNK;
    DevicePlan plan;
    HcclResult rc = GetDevicePlan(w, HCCL_AMD_OP_REDUCE_SCATTER, meshChunk ? HCCL_AMD_ALGO_MESH_CHUNK : HCCL_AMD_ALGO_MESH,
                                  &plan);
    if (rc != HCCL_SUCCESS) {
        return rc;
    }
    if (meshChunk) {
        // Always one loop; the reference refuses a count its single accumulation slot cannot hold (reference
        // ins_v2_reduce_scatter_v_sole_executor.cc:158-171, ins_temp_reduce_scatter_v_mesh_1D_meshchunk.cc:49-55).
        const uint32_t esz = DataTypeSize(p.dtype);
        if (w->cclBytes != 0 && longest > SoleMaxCountPerLoop(w->cclBytes, 1, esz)) {
            Log(1, "ReduceScatterV: %llu elements exceed the staging buffer of %llu bytes in the mesh-chunk order",
                static_cast<unsigned long long>(longest), static_cast<unsigned long long>(w->cclBytes));
            return HCCL_E_NOT_SUPPORT;
        }
        for (uint32_t k = 0; k < n; ++k) {
            if (ref[k] == 0) {
                continue;
            }
            ReduceArgs a{};
            for (uint32_t r = 0; r < n; ++r) {
                a.src[r] = static_cast<const uint8_t*>(p.ranks[r].send) + ref[n + k] * esz;
            }
            a.dst[0] = p.ranks[k].recv;
            a.nDst = 1;
            a.dstOwn = 1;
            rc = LaunchMeshChunk(w, plan, p, a, k, 1, ref[k], 0, true, s);
            if (rc != HCCL_SUCCESS) {
                return rc;
            }
        }
        return HCCL_SUCCESS;
    }
    ReduceArgs a{};
    for (uint32_t r = 0; r < n; ++r) {
        a.src[r] = p.ranks[r].send;
        a.dst[r] = p.ranks[r].recv;
        a.groupLenV[r] = ref[r];
        a.groupOffV[r] = ref[n + r];
    }
    a.prog = plan.dev;
    a.varGroups = 1;
    a.nDst = 1;
    a.dstOwn = 1;
    a.nGroup = n;
    a.nSub = 1;
    a.groupLen = a.subLen = longest;
    a.total = static_cast<uint64_t>(n) * longest;
    a.progGroupStride = plan.nProg > 1 ? 1 : 0;
    return LaunchOneReduce(w, a, plan, p.dtype, p.op, s);
}

// Reduce.  MESH: out_root = in_0, then in_1 .. in_{N-1} folded ascending (reference reduce_mesh_1D.cc:268-300):
// the AllReduce rank-order program with the root's recvBuf as only destination.  MESH_TWO_SHOT: every loop of the
// executor deals its elements into N slices, the first len mod N one element longer, and slice k folds rank k's
// input first (reference reduce_mesh_1D_two_shot.cc:138-162, 228-265; N staging slots, :79-84,
// reduce_sole_executor.cc:178-232).  NHR: slices of ceil(len / N) elements, short or empty towards the end, each
// folded along the NHR step tree (reference reduce_nhr.cc:202-226, 263-339; one staging slot, :131-136).  A world
// with level-0 groups runs RHD, NHR and, for the types the reference reduces on the host, the host-reduce fold as the
// AllReduce sequence does, with the root as only destination (reference reduce_sequence_executor_aicpu_3level.cc:
// 744-990): chunks, sub-slices and parts of floor(len / d) elements with the rest in the last, for RHD too.
HcclResult RunReduce(World* w, PendingOp& p, hipStream_t s)
{
    const uint32_t n = w->n;
    if (p.ranks[p.root].recv == nullptr) {
        return HCCL_E_PTR;
    }
    const uint32_t esz = DataTypeSize(p.dtype);
    const HcclAmdAlgo configured = w->algo[HCCL_AMD_OP_REDUCE];
    const bool stepDriven = configured == HCCL_AMD_ALGO_RHD || configured == HCCL_AMD_ALGO_NHR;
    HcclAmdAlgo algo = EffectiveAlgo(w, HCCL_AMD_OP_REDUCE, p.dtype, p.op);
    Levels lv;
    const bool levels = ResolveLevels(n, w->level0, algo == HCCL_AMD_ALGO_MESH ? 0 : w->level1, &lv) &&
                        w->reduceSequence != 0 &&
                        (algo == HCCL_AMD_ALGO_RHD || algo == HCCL_AMD_ALGO_NHR ||
                         (algo == HCCL_AMD_ALGO_MESH && (stepDriven || w->reduceSequence == 1)));
    if (levels) {
        DevicePlan plan;
        HcclResult rc = GetDevicePlan(w, HCCL_AMD_OP_REDUCE, algo, &plan, lv.l0, w->level1);
        if (rc != HCCL_SUCCESS) {
            return rc;
        }
        uint64_t maxPerLoop = p.count;
        uint64_t resultElems = ~0ull;
        if (w->cclBytes != 0) {
            rc = SequenceMaxCountPerLoop(w->cclBytes, p.count, lv.l0, n, esz, 4096, false, &maxPerLoop, &resultElems);
            if (rc != HCCL_SUCCESS) {
                Log(1, "Reduce: the staging buffer of %llu bytes holds no loop of the sequence order",
                    static_cast<unsigned long long>(w->cclBytes));
                return rc;
            }
        }
        ReduceArgs a{};
        a.nDst = 1;
        a.dstOwn = 0;
        a.nGroup = 1;
        a.progSubStride = 1;
        uint32_t dims[3];
        const uint32_t nDims = LevelDims(lv, dims);
        auto launch = [&](uint32_t prog, uint32_t nSub, uint64_t begin, uint64_t len, uint64_t subLen) {
            for (uint32_t r = 0; r < n; ++r) {
                a.src[r] = static_cast<const uint8_t*>(p.ranks[r].send) + begin * esz;
            }
            a.dst[0] = static_cast<uint8_t*>(p.ranks[p.root].recv) + begin * esz;
            a.prog = plan.dev + static_cast<uint64_t>(prog) * kDevProgBytes;
            a.nSub = nSub;
            a.total = a.groupLen = len;
            a.subLen = subLen;
            return LaunchOneReduce(w, a, plan, p.dtype, p.op, s);
        };
        for (uint64_t done = 0; done < p.count;) {
            const uint64_t len = SequenceSelectLoopCount(p.count - done, maxPerLoop, lv.l0, resultElems);
            if (len == 0) {
                return HCCL_E_INTERNAL;
            }
            rc = CutByLevels(dims, nDims, 0, done, len, launch);
            if (rc != HCCL_SUCCESS) {
                return rc;
            }
            done += len;
        }
        return HCCL_SUCCESS;
    }
    if (algo == HCCL_AMD_ALGO_RHD) {
        algo = HCCL_AMD_ALGO_MESH;   // the reference has no single-level RHD Reduce: its selection falls back
    }
    const bool twoShot = algo == HCCL_AMD_ALGO_MESH_TWO_SHOT;
    const bool nhr = algo == HCCL_AMD_ALGO_NHR;
    DevicePlan plan;
    HcclResult rc = GetDevicePlan(w, HCCL_AMD_OP_REDUCE,
                                  twoShot ? HCCL_AMD_ALGO_MESH_TWO_SHOT : nhr ? HCCL_AMD_ALGO_NHR : HCCL_AMD_ALGO_MESH, &plan);
    if (rc != HCCL_SUCCESS) {
        return rc;
    }
    ReduceArgs a{};
    for (uint32_t r = 0; r < n; ++r) {
        a.src[r] = p.ranks[r].send;
    }
    a.dst[0] = p.ranks[p.root].recv;
    a.prog = plan.dev;
    a.nDst = 1;
    a.dstOwn = 0;
    a.nGroup = 1;
    if (!twoShot && !nhr) {
        a.nSub = 1;
        a.total = a.groupLen = a.subLen = p.count;
        return LaunchOneReduce(w, a, plan, p.dtype, p.op, s);
    }
    uint64_t maxPerLoop = p.count;
    if (w->cclBytes != 0) {
        maxPerLoop = SoleMaxCountPerLoop(w->cclBytes, nhr ? 1 : n, esz);
        if (maxPerLoop == 0) {
            return HCCL_E_INTERNAL;
        }
    }
    a.progSubStride = 1;
    for (uint64_t done = 0; done < p.count;) {
        const uint64_t len = std::min(p.count - done, maxPerLoop);
        if (nhr) {
            // nFull slices of ceil(len / n) elements, then one shorter slice if elements are left
            const uint64_t slice = (len + n - 1) / n;
            const uint32_t nFull = static_cast<uint32_t>(len / slice);
            const uint64_t rest = len - static_cast<uint64_t>(nFull) * slice;
            for (int run = 0; run < 2; ++run) {
                const uint32_t slices = run == 0 ? nFull : (rest != 0 ? 1u : 0u);
                if (slices == 0) {
                    continue;
                }
                const uint64_t at = (done + (run == 0 ? 0 : static_cast<uint64_t>(nFull) * slice)) * esz;
                for (uint32_t r = 0; r < n; ++r) {
                    a.src[r] = static_cast<const uint8_t*>(p.ranks[r].send) + at;
                }
                a.dst[0] = static_cast<uint8_t*>(p.ranks[p.root].recv) + at;
                a.prog = plan.dev + static_cast<uint64_t>(run == 0 ? 0 : nFull) * kDevProgBytes;
                a.nSub = slices;
                a.subLen = run == 0 ? slice : rest;
                a.total = a.groupLen = run == 0 ? slice * nFull : rest;
                rc = LaunchOneReduce(w, a, plan, p.dtype, p.op, s);
                if (rc != HCCL_SUCCESS) {
                    return rc;
                }
            }
            done += len;
            continue;
        }
        const uint64_t base = len / n;
        const uint32_t nBig = static_cast<uint32_t>(len % n);
        // two runs of equally long slices: nBig of base + 1 elements, then n - nBig of base
        const uint64_t runFirst[2] = {0, static_cast<uint64_t>(nBig) * (base + 1)};
        const uint32_t runSlices[2] = {nBig, n - nBig};
        const uint64_t runLen[2] = {base + 1, base};
        for (int run = 0; run < 2; ++run) {
            if (runSlices[run] == 0 || runLen[run] == 0) {
                continue;
            }
            const uint64_t at = (done + runFirst[run]) * esz;
            for (uint32_t r = 0; r < n; ++r) {
                a.src[r] = static_cast<const uint8_t*>(p.ranks[r].send) + at;
            }
            a.dst[0] = static_cast<uint8_t*>(p.ranks[p.root].recv) + at;
            a.prog = plan.dev + static_cast<uint64_t>(run == 0 ? 0 : nBig) * kDevProgBytes;
            a.nSub = runSlices[run];
            a.subLen = runLen[run];
            a.total = a.groupLen = runLen[run] * runSlices[run];
            rc = LaunchOneReduce(w, a, plan, p.dtype, p.op, s);
            if (rc != HCCL_SUCCESS) {
                return rc;
            }
        }
        done += len;
    }
    return HCCL_SUCCESS;
}

}  // namespace hccl_amd
