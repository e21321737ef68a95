// Slice-copy (AllGather / AllGatherV) and displacement-driven pack/unpack (AlltoAllV) for gfx950.
//
// Both are pure HBM streaming: every payload byte is read once with 128-bit loads and written once
// per destination with 128-bit stores.  Work is cut into 16 KiB tiles so that segments of wildly
// different length (a Zipf-distributed token routing table) load-balance over the whole chip; the
// tile -> segment map is found with wavefront-level prefix sums (one lane per rank) and ballots, never
// a per-segment launch.
//
// Displacements are in elements, so a segment's source and destination generally sit at different
// offsets from a 16-byte boundary.  Such irregular segments are staged through LDS: the block loads
// the aligned 16-byte vectors that cover the tile's source bytes, and every lane rebuilds the vector it
// has to store from two neighbouring LDS vectors with a byte funnel shift.  Segments whose two sides
// are congruent modulo 16 skip LDS.  At most 15 bytes at either end of a tile move byte by byte.
//
// Data movement follows the reference's templates:
//   AllGather(V): out_d[displs[r] ...] = in_r   (ins_temp_all_gather_mesh_1D.cc:249-423,
//                                                ins_temp_all_gather_v_mesh_1D.cc:242-310)
//   AlltoAllV   : recv_i[rdispls_i[j] ...] = send_j[sdispls_j[i] ...], sendCounts_j[i] elements
//                 (ins_temp_all_to_all_v_mesh_1D.cc:229-246, 459-611)
#include <hip/hip_runtime.h>

#include "dataplane.h"

namespace hccl_amd {
namespace {

constexpr int kThreads = 256;
constexpr int kVecPerTile = kCopyTileBytes / 16;                // 1024
constexpr int kVecPerThread = kVecPerTile / kThreads;           // 4
static_assert(kVecPerThread * kThreads == kVecPerTile, "tile must be a whole number of vector rounds");

typedef uint32_t U32x4 __attribute__((ext_vector_type(4)));

// One staging buffer: the tile's vectors plus the one that completes the last shifted vector.
struct Stage {
    U32x4 v[kVecPerTile + 1];
};

__device__ __forceinline__ uint32_t Uniform(uint32_t v) { return __builtin_amdgcn_readfirstlane(v); }

// Inclusive prefix sum over the 64 lanes of a wavefront.
__device__ __forceinline__ uint32_t WaveInclusiveScan(uint32_t x)
{
    const uint32_t lane = threadIdx.x & 63u;
#pragma unroll
    for (uint32_t d = 1; d < 64; d <<= 1) {
        uint32_t up = __shfl_up(x, d, 64);
        if (lane >= d) {
            x += up;
        }
    }
    return x;
}

// Number of leading lanes whose (non-decreasing) inclusive prefix is <= t: the index of the segment
// that contains item t.  Zero-length segments repeat their predecessor's prefix and are skipped.
__device__ __forceinline__ uint32_t SegmentOf(uint32_t inclusive, uint32_t t)
{
    return static_cast<uint32_t>(__popcll(__ballot(inclusive <= t)));
}

__device__ __forceinline__ uint32_t AlignUnit(uint64_t bits)
{
    // largest power of two <= 16 dividing `bits`
    uint32_t low = static_cast<uint32_t>(bits) | 16u;
    return low & (0u - low);
}

// Copies one tile (bytes <= 16 KiB) from src to dstOf(d), d < nDst.  Every dstOf(d) has the same offset
// from a 16-byte boundary.  Must be called by all threads of the block (it may synchronise).
// Four output dwords from five input dwords, dropping `shift` (0..3) leading bytes.
__device__ __forceinline__ U32x4 Funnel(uint32_t w0, uint32_t w1, uint32_t w2, uint32_t w3, uint32_t w4, uint32_t shift)
{
    if (shift == 0) {
        return U32x4{w0, w1, w2, w3};
    }
    return U32x4{__builtin_amdgcn_alignbyte(w1, w0, shift), __builtin_amdgcn_alignbyte(w2, w1, shift),
                 __builtin_amdgcn_alignbyte(w3, w2, shift), __builtin_amdgcn_alignbyte(w4, w3, shift)};
}

// The two staging buffers alternate between the tiles that use them, so one barrier per tile is enough:
// a buffer is rewritten only after the barrier of the tile that used the other one.
template <class DstFn>
__device__ __forceinline__ void CopyTile(const uint8_t* src, uint32_t bytes, uint32_t nDst, DstFn dstOf, Stage* stages,
                                         uint32_t& parity)
{
    const uint32_t dMis = static_cast<uint32_t>(reinterpret_cast<uint64_t>(dstOf(0)) & 15u);
    uint32_t head = (16u - dMis) & 15u;     // bytes before the first aligned destination vector
    head = head < bytes ? head : bytes;
    const uint32_t nVec = (bytes - head) / 16u;
    const uint32_t bodyEnd = head + nVec * 16u;
    const uint8_t* sBody = src + head;
    const uint32_t sMis = static_cast<uint32_t>(reinterpret_cast<uint64_t>(sBody) & 15u);

    U32x4 out[kVecPerThread];
    if (sMis == 0) {
        const U32x4* s = reinterpret_cast<const U32x4*>(sBody);
#pragma unroll
        for (int k = 0; k < kVecPerThread; ++k) {
            const uint32_t idx = threadIdx.x + k * kThreads;
            if (idx < nVec) {
                out[k] = __builtin_nontemporal_load(s + idx);
            }
        }
    } else if (nVec != 0) {
        // Irregular: stage the covering aligned vectors, then funnel-shift pairs of dwords.
        Stage* st = stages + parity;
        parity ^= 1u;
        const U32x4* s = reinterpret_cast<const U32x4*>(sBody - sMis);
#pragma unroll
        for (int k = 0; k <= kVecPerThread; ++k) {
            const uint32_t idx = threadIdx.x + k * kThreads;
            if (idx <= nVec) {
                st->v[idx] = __builtin_nontemporal_load(s + idx);
            }
        }
        __syncthreads();
        const uint32_t q = sMis >> 2;        // whole dwords to skip
        const uint32_t shift = sMis & 3u;    // bytes to skip inside a dword
#pragma unroll
        for (int k = 0; k < kVecPerThread; ++k) {
            const uint32_t idx = threadIdx.x + k * kThreads;
            if (idx < nVec) {
                const U32x4 a = st->v[idx];
                const U32x4 b = st->v[idx + 1];
                switch (q) {   // uniform: picks the five dwords that straddle the two staged vectors
                    case 0: out[k] = Funnel(a.x, a.y, a.z, a.w, b.x, shift); break;
                    case 1: out[k] = Funnel(a.y, a.z, a.w, b.x, b.y, shift); break;
                    case 2: out[k] = Funnel(a.z, a.w, b.x, b.y, b.z, shift); break;
                    default: out[k] = Funnel(a.w, b.x, b.y, b.z, b.w, shift); break;
                }
            }
        }
    }
    for (uint32_t d = 0; d < nDst; ++d) {
        U32x4* o = reinterpret_cast<U32x4*>(dstOf(d) + head);
#pragma unroll
        for (int k = 0; k < kVecPerThread; ++k) {
            const uint32_t idx = threadIdx.x + k * kThreads;
            if (idx < nVec) {
                __builtin_nontemporal_store(out[k], o + idx);
            }
        }
    }
    // Up to 15 bytes in front of the body and up to 15 behind it.
    const uint32_t edge = head + (bytes - bodyEnd);
    if (threadIdx.x < edge) {
        const uint32_t o = threadIdx.x < head ? threadIdx.x : bodyEnd + (threadIdx.x - head);
        const uint8_t b = src[o];
        for (uint32_t d = 0; d < nDst; ++d) {
            dstOf(d)[o] = b;
        }
    }
}

// Fallback when destinations differ in alignment: lane-per-unit copies of the widest common unit.
template <typename U, class DstFn>
__device__ __forceinline__ void CopyUnits(const uint8_t* src, uint32_t bytes, uint32_t nDst, DstFn dstOf)
{
    const uint32_t n = bytes / sizeof(U);
    const U* s = reinterpret_cast<const U*>(src);
    for (uint32_t i = threadIdx.x; i < n; i += kThreads) {
        U v = __builtin_nontemporal_load(s + i);
        for (uint32_t d = 0; d < nDst; ++d) {
            __builtin_nontemporal_store(v, reinterpret_cast<U*>(dstOf(d)) + i);
        }
    }
}

template <class DstFn>
__device__ __forceinline__ void CopyTileByUnit(const uint8_t* src, uint32_t bytes, uint32_t unit, uint32_t nDst, DstFn dstOf)
{
    if (unit >= 8) {
        CopyUnits<uint64_t>(src, bytes, nDst, dstOf);
    } else if (unit == 4) {
        CopyUnits<uint32_t>(src, bytes, nDst, dstOf);
    } else if (unit == 2) {
        CopyUnits<uint16_t>(src, bytes, nDst, dstOf);
    } else {
        CopyUnits<uint8_t>(src, bytes, nDst, dstOf);
    }
}

// ---- AllGather / AllGatherV --------------------------------------------------------------------
__global__ __launch_bounds__(kThreads) void BcastCopyKernel(const BcastCopyArgs args)
{
    __shared__ Stage stage[2];
    const uint32_t lane = threadIdx.x & 63u;
    const uint64_t myLen = lane < args.nSeg ? args.len[lane] : 0;
    const uint32_t myTiles = static_cast<uint32_t>((myLen + kCopyTileBytes - 1) / kCopyTileBytes);
    const uint32_t incl = WaveInclusiveScan(myTiles);
    const uint32_t total = Uniform(__shfl(incl, 63, 64));

    uint32_t parity = 0;
    for (uint32_t tile = blockIdx.x; tile < total; tile += gridDim.x) {
        const uint32_t seg = Uniform(SegmentOf(incl, tile));
        const uint32_t segFirst = seg == 0 ? 0u : Uniform(__shfl(incl, seg - 1, 64));
        const uint64_t off = static_cast<uint64_t>(tile - segFirst) * kCopyTileBytes;
        const uint64_t len = args.len[seg];
        const uint32_t bytes = static_cast<uint32_t>((len - off < kCopyTileBytes) ? len - off : kCopyTileBytes);
        const uint8_t* src = static_cast<const uint8_t*>(args.src[seg]) + off;
        const uint64_t dOff = args.dstOff[seg] + off;
        auto dstOf = [&](uint32_t d) { return static_cast<uint8_t*>(args.dst[d]) + dOff; };
        if (args.unit == 16) {   // destination bases are all 16-byte aligned, hence congruent
            CopyTile(src, bytes, args.nDst, dstOf, stage, parity);
        } else {
            const uint32_t unit = AlignUnit(reinterpret_cast<uint64_t>(args.src[seg]) | len | args.dstOff[seg] | args.unit);
            CopyTileByUnit(src, bytes, unit, args.nDst, dstOf);
        }
    }
}

// ---- AlltoAllV: tile tables ----------------------------------------------------------------------
// One wavefront per destination rank i: lane j holds the tile count of segment (i <- j); the
// inclusive scan is the per-row table, the row totals are scanned once more by wavefront 0.
__global__ __launch_bounds__(1024) void A2aPlanKernel(const A2aArgs args)
{
    __shared__ uint32_t rowTiles[kMaxRanks];
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t n = args.n;
    for (uint32_t i = wave; i < n; i += 16) {
        const uint64_t cnt = lane < n ? args.cnt[static_cast<uint64_t>(lane) * n + i] : 0;
        const uint32_t tiles = static_cast<uint32_t>((cnt * args.esz + kCopyTileBytes - 1) / kCopyTileBytes);
        const uint32_t incl = WaveInclusiveScan(tiles);
        if (lane < n) {
            args.segEnd[i * n + lane] = incl;
        }
        if (lane == 63) {
            rowTiles[i] = incl;
        }
    }
    __syncthreads();
    if (wave == 0) {
        const uint32_t t = lane < n ? rowTiles[lane] : 0;
        const uint32_t incl = WaveInclusiveScan(t);
        if (lane < n) {
            args.rowStart[lane] = incl - t;
        }
        if (lane == 63) {
            args.rowStart[n] = incl;
        }
    }
}

// ---- AlltoAllV: copy -------------------------------------------------------------------------------
// Each block takes a contiguous run of tiles; it looks the (destination, source) segment up with two
// ballots when it crosses a segment boundary and then streams the tile.
__global__ __launch_bounds__(kThreads) void A2aCopyKernel(const A2aArgs args)
{
    __shared__ Stage stage[2];
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t n = args.n;
    const uint32_t total = args.rowStart[n];
    const uint32_t rowEndLane = lane < n ? args.rowStart[lane + 1] : 0xFFFFFFFFu;
    const uint32_t t0 = static_cast<uint32_t>(static_cast<uint64_t>(total) * blockIdx.x / gridDim.x);
    const uint32_t t1 = static_cast<uint32_t>(static_cast<uint64_t>(total) * (blockIdx.x + 1) / gridDim.x);

    uint32_t rowEnd = 0, rowBase = 0, row = 0;
    uint32_t segBegin = 0, segEnd = 0;   // absolute tile range of the current segment
    uint32_t segEndLane = 0xFFFFFFFFu;
    const uint8_t* src = nullptr;
    uint8_t* dst = nullptr;
    uint64_t len = 0;
    bool haveRow = false;
    uint32_t parity = 0;

    for (uint32_t t = t0; t < t1; ++t) {
        if (!haveRow || t >= rowEnd) {
            row = Uniform(SegmentOf(rowEndLane, t));
            rowBase = args.rowStart[row];
            rowEnd = args.rowStart[row + 1];
            segEndLane = lane < n ? args.segEnd[row * n + lane] : 0xFFFFFFFFu;
            haveRow = true;
            segEnd = 0;
        }
        if (t >= segEnd) {
            const uint32_t rel = t - rowBase;
            const uint32_t seg = Uniform(SegmentOf(segEndLane, rel));
            segBegin = rowBase + (seg == 0 ? 0u : Uniform(__shfl(segEndLane, seg - 1, 64)));
            segEnd = rowBase + Uniform(__shfl(segEndLane, seg, 64));
            const uint64_t cnt = args.cnt[static_cast<uint64_t>(seg) * n + row];
            const uint64_t sd = args.sdis[static_cast<uint64_t>(seg) * n + row];
            const uint64_t rd = args.rdis[static_cast<uint64_t>(row) * n + seg];
            src = static_cast<const uint8_t*>(args.send[seg]) + sd * args.esz;
            dst = static_cast<uint8_t*>(args.recv[row]) + rd * args.esz;
            len = cnt * args.esz;
        }
        const uint64_t off = static_cast<uint64_t>(t - segBegin) * kCopyTileBytes;
        const uint32_t bytes = static_cast<uint32_t>((len - off < kCopyTileBytes) ? len - off : kCopyTileBytes);
        uint8_t* d = dst + off;
        CopyTile(src + off, bytes, 1u, [&](uint32_t) { return d; }, stage, parity);
    }
}

}  // namespace

hipError_t LaunchBcastCopy(const BcastCopyArgs& args, uint32_t maxBlocks, hipStream_t stream)
{
    uint64_t tiles = 0;
    for (uint32_t j = 0; j < args.nSeg; ++j) {
        tiles += (args.len[j] + kCopyTileBytes - 1) / kCopyTileBytes;
    }
    if (tiles == 0) {
        return hipSuccess;
    }
    if (tiles > 0xFFFFFFF0ull) {
        return hipErrorInvalidValue;
    }
    const uint32_t blocks = tiles < maxBlocks ? static_cast<uint32_t>(tiles) : maxBlocks;
    hipLaunchKernelGGL(BcastCopyKernel, dim3(blocks), dim3(kThreads), 0, stream, args);
    return hipGetLastError();
}

hipError_t LaunchA2aPlan(const A2aArgs& args, hipStream_t stream)
{
    hipLaunchKernelGGL(A2aPlanKernel, dim3(1), dim3(1024), 0, stream, args);
    return hipGetLastError();
}

hipError_t LaunchA2aCopy(const A2aArgs& args, uint32_t nBlocks, hipStream_t stream)
{
    if (nBlocks == 0) {
        return hipSuccess;
    }
    hipLaunchKernelGGL(A2aCopyKernel, dim3(nBlocks), dim3(kThreads), 0, stream, args);
    return hipGetLastError();
}

}  // namespace hccl_amd
