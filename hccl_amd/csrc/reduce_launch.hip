// Dispatch of the fused reduce kernel by (data type, reduce op).
#include "reduce_kernel_impl.h"

namespace hccl_amd {

hipError_t LaunchReduce(const ReduceArgs& args, HcclDataType dtype, HcclReduceOp op, uint32_t nBlocks,
                        uint32_t ldsBytes, hipStream_t stream)
{
    detail::ReduceKernelFn fn = nullptr;
    const int o = static_cast<int>(op);
    const bool pair = args.vecBatch == kVecBatchPair;
    const int batch = pair ? 0 : (args.vecBatch == 8 ? 8 : 16);
    switch (dtype) {
        case HCCL_DATA_TYPE_INT8: fn = SelectReduceI8(o, batch); break;
        case HCCL_DATA_TYPE_INT16: fn = SelectReduceI16(o, batch); break;
        case HCCL_DATA_TYPE_INT32: fn = SelectReduceI32(o, batch); break;
        case HCCL_DATA_TYPE_INT64: fn = SelectReduceI64(o, batch); break;
        case HCCL_DATA_TYPE_UINT64: fn = SelectReduceU64(o, batch); break;
        case HCCL_DATA_TYPE_FP16: fn = SelectReduceF16(o, batch); break;
        case HCCL_DATA_TYPE_BFP16: fn = SelectReduceBf16(o, batch); break;
        case HCCL_DATA_TYPE_FP32: fn = SelectReduceF32(o, batch); break;
        case HCCL_DATA_TYPE_FP64: fn = SelectReduceF64(o, batch); break;
        default: break;
    }
    if (fn == nullptr || nBlocks == 0 || (args.threads != 64 && args.threads != 128 && args.threads != 256)) {
        return hipErrorInvalidValue;
    }
    if (pair && (args.threads != 64 || args.storeWaves > 1 || args.varGroups != 0)) {
        return hipErrorInvalidValue;
    }
    uint32_t threads = args.threads;
    if (args.storeWaves > 1) {
        const uint32_t waves = args.storeWaves & 0xFFu;
        const bool allFold = (args.storeWaves & kStoreWavesAllFold) != 0;
        if ((args.storeWaves & ~(kStoreWavesAllFold | 0xFFu)) != 0 || waves < 2 || args.threads != 64 ||
            args.dstOwn != 0 || waves * 64 > kMaxReduceThreads) {
            return hipErrorInvalidValue;
        }
        // the wavefronts that all fold exchange their tiles through the dynamic LDS: two rounds of `waves` KiB
        if (allFold && (args.varGroups != 0 || batch != 8 || ldsBytes < 2u * waves * 1024u)) {
            return hipErrorInvalidValue;
        }
        threads = 64 * waves;
    }
    // Uniform geometry: (workgroups per sub-segment, sub-segments, groups), consecutive workgroups on consecutive
    // positions of a sub-segment as before; groups of unequal length own runs of a one-dimensional grid.
    dim3 grid(nBlocks);
    if (!args.varGroups) {
        if (args.blocksPerSub == 0 || args.nSub == 0 || args.nGroup == 0 || args.nSub > 65535u || args.nGroup > 65535u ||
            static_cast<uint64_t>(args.blocksPerSub) * args.nSub * args.nGroup != nBlocks) {
            return hipErrorInvalidValue;
        }
        grid = dim3(args.blocksPerSub, args.nSub, args.nGroup);
    }
    hipLaunchKernelGGL(fn, grid, dim3(threads), ldsBytes, stream, args);
    return hipGetLastError();
}

hipError_t LaunchDirectFold(const DirectFoldArgs& args, HcclDataType dtype, HcclReduceOp op, uint32_t waves,
                            uint32_t tilesPerWave, hipStream_t stream)
{
    detail::DirectFoldFn fn = nullptr;
    const int o = static_cast<int>(op);
    // eight of everything and only whole workgroups: the straight-line kernel
    const bool eights = waves == 8 && args.nSrc == 8 && args.nDst == 8 && args.tail == 0 && args.nVec != 0;
    const bool twoTiles = tilesPerWave == 2 && args.tail == 0 && args.nVec != 0 && waves != 0 &&
                          args.nVec % (2 * 64 * static_cast<uint64_t>(waves)) == 0;
    const bool wide = args.nSrc > kDirectFoldMaxLeaves || args.nDst > kDirectFoldMaxDst;
    const int exact = wide ? 4 : eights ? (twoTiles ? 2 : args.nVec % (8 * 64) == 0 ? 1 : 0) : (twoTiles ? 3 : 0);
    switch (dtype) {
        case HCCL_DATA_TYPE_INT8: fn = SelectReduceI8Direct(o, exact); break;
        case HCCL_DATA_TYPE_INT16: fn = SelectReduceI16Direct(o, exact); break;
        case HCCL_DATA_TYPE_INT32: fn = SelectReduceI32Direct(o, exact); break;
        case HCCL_DATA_TYPE_INT64: fn = SelectReduceI64Direct(o, exact); break;
        case HCCL_DATA_TYPE_UINT64: fn = SelectReduceU64Direct(o, exact); break;
        case HCCL_DATA_TYPE_FP16: fn = SelectReduceF16Direct(o, exact); break;
        case HCCL_DATA_TYPE_BFP16: fn = SelectReduceBf16Direct(o, exact); break;
        case HCCL_DATA_TYPE_FP32: fn = SelectReduceF32Direct(o, exact); break;
        case HCCL_DATA_TYPE_FP64: fn = SelectReduceF64Direct(o, exact); break;
        default: break;
    }
    uint32_t esz = 0;
    switch (dtype) {
        case HCCL_DATA_TYPE_INT8: esz = 1; break;
        case HCCL_DATA_TYPE_INT16: case HCCL_DATA_TYPE_FP16: case HCCL_DATA_TYPE_BFP16: esz = 2; break;
        case HCCL_DATA_TYPE_INT32: case HCCL_DATA_TYPE_FP32: esz = 4; break;
        case HCCL_DATA_TYPE_INT64: case HCCL_DATA_TYPE_UINT64: case HCCL_DATA_TYPE_FP64: esz = 8; break;
        default: break;
    }
    if (fn == nullptr || esz == 0 || waves < 2 || waves > kDirectFoldMaxWaves || args.nSrc == 0 ||
        args.nSrc > kDirectFoldWideLeaves || args.nDst == 0 || args.nDst > kDirectFoldWideDst || args.tail >= 16 / esz ||
        (args.nVec == 0 && args.tail == 0)) {
        return hipErrorInvalidValue;
    }
    // the kernel for more than eight leaves or destinations takes whole workgroups only
    if (wide && (args.tail != 0 || args.nVec % (64 * static_cast<uint64_t>(waves)) != 0)) {
        return hipErrorInvalidValue;
    }
    // a wavefront holds the addresses of at most half the destination table
    if ((args.nDst + waves - 1) / waves > (wide ? kDirectFoldWideDst : kDirectFoldMaxDst) / 2) {
        return hipErrorInvalidValue;
    }
    for (uint32_t i = 0; i < args.nSrc; ++i) {
        if (args.src[i] == nullptr || (reinterpret_cast<uintptr_t>(args.src[i]) & 15u) != 0) {
            return hipErrorInvalidValue;
        }
    }
    for (uint32_t d = 0; d < args.nDst; ++d) {
        if (args.dst[d] == nullptr || (reinterpret_cast<uintptr_t>(args.dst[d]) & 15u) != 0) {
            return hipErrorInvalidValue;
        }
    }
    const uint64_t tiles = (args.nVec + 63) / 64;
    const uint32_t perGroup = waves * (exact == 2 || exact == 3 ? 2u : 1u);   // tiles of one workgroup
    const uint64_t blocks = tiles == 0 ? 1 : (tiles + perGroup - 1) / perGroup;
    if (blocks > 0x7FFFFFFFull) {
        return hipErrorInvalidValue;
    }
    DirectFoldArgs a = args;
    a.waves = waves;
    hipLaunchKernelGGL(fn, dim3(static_cast<uint32_t>(blocks)), dim3(64 * waves), perGroup * 1024u, stream, a);
    return hipGetLastError();
}

}  // namespace hccl_amd
