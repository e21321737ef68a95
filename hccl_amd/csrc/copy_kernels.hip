// Slice-copy (AllGather / AllGatherV) and displacement-driven pack/unpack (AlltoAllV) for gfx950.
//
// Both are pure HBM streaming: every payload byte is read once with a 128-bit load and written once
// per destination with a 128-bit store.  Work is cut into tiles of one vector per lane and every tile
// is its own workgroup, so that the workgroups in flight at any moment cover a compact window of
// addresses (looping workgroups that stride over the whole range keep many more DRAM pages open and
// measure 15-20 % slower on this part).  Tiles also load-balance segments of wildly different length
// (a Zipf-distributed token routing table) over the whole chip; the tile -> segment map is found with
// wavefront-level prefix sums (one lane per rank) and ballots, never a per-segment launch.
//
// Displacements are in elements, so a segment's source and destination generally sit at different
// offsets from a 16-byte boundary.  Such irregular segments are staged through LDS: the workgroup loads
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

typedef uint32_t U32x4 __attribute__((ext_vector_type(4)));

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

// Four output dwords from five input dwords, dropping `shift` (0..3) leading bytes.
__device__ __forceinline__ U32x4 Funnel(uint32_t w0, uint32_t w1, uint32_t w2, uint32_t w3, uint32_t w4, uint32_t shift)
{
    if (shift == 0) {
        return U32x4{w0, w1, w2, w3};
    }
    return U32x4{__builtin_amdgcn_alignbyte(w1, w0, shift), __builtin_amdgcn_alignbyte(w2, w1, shift),
                 __builtin_amdgcn_alignbyte(w3, w2, shift), __builtin_amdgcn_alignbyte(w4, w3, shift)};
}

// Copies one tile (bytes <= T * 16) from src to dstOf(d), d < nDst, one 16-byte vector per lane.  Every
// dstOf(d) has the same offset from a 16-byte boundary.  `stage` holds T + 1 vectors.  Must be called by
// all T threads of the workgroup (the irregular path synchronises).
template <int T, class DstFn>
__device__ __forceinline__ void CopyTile(const uint8_t* src, uint32_t bytes, uint32_t nDst, DstFn dstOf, U32x4* stage)
{
    const uint32_t dMis = static_cast<uint32_t>(reinterpret_cast<uint64_t>(dstOf(0)) & 15u);
    uint32_t head = (16u - dMis) & 15u;     // bytes before the first aligned destination vector
    head = head < bytes ? head : bytes;
    const uint32_t nVec = (bytes - head) / 16u;   // <= T
    const uint32_t bodyEnd = head + nVec * 16u;
    const uint8_t* sBody = src + head;
    const uint32_t sMis = static_cast<uint32_t>(reinterpret_cast<uint64_t>(sBody) & 15u);
    const uint32_t idx = threadIdx.x;

    U32x4 out = {0, 0, 0, 0};
    if (sMis == 0) {
        if (idx < nVec) {
            out = __builtin_nontemporal_load(reinterpret_cast<const U32x4*>(sBody) + idx);
        }
    } else if (nVec != 0) {
        // Irregular: stage the covering aligned vectors, then funnel-shift across two of them.
        const U32x4* s = reinterpret_cast<const U32x4*>(sBody - sMis);
        if (idx <= nVec) {
            stage[idx] = __builtin_nontemporal_load(s + idx);
        }
        if (idx == 0 && nVec == static_cast<uint32_t>(T)) {
            stage[T] = __builtin_nontemporal_load(s + T);
        }
        __syncthreads();
        const uint32_t q = sMis >> 2;        // whole dwords to skip
        const uint32_t shift = sMis & 3u;    // bytes to skip inside a dword
        if (idx < nVec) {
            const U32x4 a = stage[idx];
            const U32x4 b = stage[idx + 1];
            switch (q) {   // uniform: picks the five dwords that straddle the two staged vectors
                case 0: out = Funnel(a.x, a.y, a.z, a.w, b.x, shift); break;
                case 1: out = Funnel(a.y, a.z, a.w, b.x, b.y, shift); break;
                case 2: out = Funnel(a.z, a.w, b.x, b.y, b.z, shift); break;
                default: out = Funnel(a.w, b.x, b.y, b.z, b.w, shift); break;
            }
        }
    }
    if (idx < nVec) {
        for (uint32_t d = 0; d < nDst; ++d) {
            __builtin_nontemporal_store(out, reinterpret_cast<U32x4*>(dstOf(d) + head) + idx);
        }
    }
    // Up to 15 bytes in front of the body and up to 15 behind it.
    const uint32_t edge = head + (bytes - bodyEnd);
    if (idx < edge) {
        const uint32_t o = idx < head ? idx : bodyEnd + (idx - head);
        const uint8_t b = src[o];
        for (uint32_t d = 0; d < nDst; ++d) {
            dstOf(d)[o] = b;
        }
    }
}

// Fallback when destinations differ in alignment: lane-per-unit copies of the widest common unit.
template <int T, typename U, class DstFn>
__device__ __forceinline__ void CopyUnits(const uint8_t* src, uint32_t bytes, uint32_t nDst, DstFn dstOf)
{
    const uint32_t n = bytes / sizeof(U);
    const U* s = reinterpret_cast<const U*>(src);
    for (uint32_t i = threadIdx.x; i < n; i += T) {
        U v = __builtin_nontemporal_load(s + i);
        for (uint32_t d = 0; d < nDst; ++d) {
            __builtin_nontemporal_store(v, reinterpret_cast<U*>(dstOf(d)) + i);
        }
    }
}

// ---- AllGather / AllGatherV --------------------------------------------------------------------
// Workgroup b copies tile b.  Lane j of every wavefront holds segment j's tile count; the wavefront
// scan turns the counts into the tile -> segment map.
template <int T>
__global__ __launch_bounds__(T) void BcastCopyKernel(const BcastCopyArgs args)
{
    constexpr uint32_t kTile = T * 16u;
    __shared__ U32x4 stage[T + 1];
    const uint32_t lane = threadIdx.x & 63u;
    const uint64_t myLen = lane < args.nSeg ? args.len[lane] : 0;
    const uint32_t myTiles = static_cast<uint32_t>((myLen + kTile - 1) / kTile);
    const uint32_t incl = WaveInclusiveScan(myTiles);
    const uint32_t tile = blockIdx.x;
    if (tile >= Uniform(__shfl(incl, 63, 64))) {
        return;
    }
    const uint32_t seg = Uniform(SegmentOf(incl, tile));
    const uint32_t segFirst = seg == 0 ? 0u : Uniform(__shfl(incl, seg - 1, 64));
    const uint64_t off = static_cast<uint64_t>(tile - segFirst) * kTile;
    const uint64_t len = args.len[seg];
    const uint32_t bytes = static_cast<uint32_t>((len - off < kTile) ? len - off : kTile);
    const uint8_t* src = static_cast<const uint8_t*>(args.src[seg]) + off;
    const uint64_t dOff = args.dstOff[seg] + off;
    auto dstOf = [&](uint32_t d) { return static_cast<uint8_t*>(args.dst[d]) + dOff; };
    if (args.unit == 16) {   // destination bases are all 16-byte aligned, hence congruent
        CopyTile<T>(src, bytes, args.nDst, dstOf, stage);
    } else {
        const uint32_t unit = AlignUnit(reinterpret_cast<uint64_t>(args.src[seg]) | len | args.dstOff[seg] | args.unit);
        if (unit >= 8) {
            CopyUnits<T, uint64_t>(src, bytes, args.nDst, dstOf);
        } else if (unit == 4) {
            CopyUnits<T, uint32_t>(src, bytes, args.nDst, dstOf);
        } else if (unit == 2) {
            CopyUnits<T, uint16_t>(src, bytes, args.nDst, dstOf);
        } else {
            CopyUnits<T, uint8_t>(src, bytes, args.nDst, dstOf);
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
        const uint32_t tiles = static_cast<uint32_t>((cnt * args.esz + args.tileBytes - 1) / args.tileBytes);
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
// Workgroup b copies tile b: one ballot over the row table finds the destination rank, one over that
// row's segment table finds the source rank.
template <int T>
__global__ __launch_bounds__(T) void A2aCopyKernel(const A2aArgs args)
{
    constexpr uint32_t kTile = T * 16u;
    __shared__ U32x4 stage[T + 1];
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t n = args.n;
    const uint32_t t = blockIdx.x;
    const uint32_t rowEndLane = lane < n ? args.rowStart[lane + 1] : 0xFFFFFFFFu;
    const uint32_t row = Uniform(SegmentOf(rowEndLane, t));
    if (row >= n) {
        return;   // beyond the last tile (the grid is sized from host-side counts, so this is defensive)
    }
    const uint32_t rowBase = row == 0 ? 0u : Uniform(__shfl(rowEndLane, row - 1, 64));
    const uint32_t segEndLane = lane < n ? args.segEnd[row * n + lane] : 0xFFFFFFFFu;
    const uint32_t seg = Uniform(SegmentOf(segEndLane, t - rowBase));
    if (seg >= n) {
        return;
    }
    const uint32_t segBegin = rowBase + (seg == 0 ? 0u : Uniform(__shfl(segEndLane, seg - 1, 64)));
    const uint64_t cnt = args.cnt[static_cast<uint64_t>(seg) * n + row];
    const uint64_t sd = args.sdis[static_cast<uint64_t>(seg) * n + row];
    const uint64_t rd = args.rdis[static_cast<uint64_t>(row) * n + seg];
    const uint64_t len = cnt * args.esz;
    const uint64_t off = static_cast<uint64_t>(t - segBegin) * kTile;
    if (off >= len) {
        return;
    }
    const uint32_t bytes = static_cast<uint32_t>((len - off < kTile) ? len - off : kTile);
    const uint8_t* src = static_cast<const uint8_t*>(args.send[seg]) + sd * args.esz + off;
    uint8_t* dst = static_cast<uint8_t*>(args.recv[row]) + rd * args.esz + off;
    CopyTile<T>(src, bytes, 1u, [&](uint32_t) { return dst; }, stage);
}

}  // namespace

hipError_t LaunchBcastCopy(const BcastCopyArgs& args, uint32_t tileBytes, hipStream_t stream)
{
    uint64_t tiles = 0;
    for (uint32_t j = 0; j < args.nSeg; ++j) {
        tiles += (args.len[j] + tileBytes - 1) / tileBytes;
    }
    if (tiles == 0) {
        return hipSuccess;
    }
    if (tiles > 0x7FFFFFF0ull) {
        return hipErrorInvalidValue;
    }
    if (tileBytes == 4096) {
        hipLaunchKernelGGL(BcastCopyKernel<256>, dim3(static_cast<uint32_t>(tiles)), dim3(256), 0, stream, args);
    } else if (tileBytes == 16384) {
        hipLaunchKernelGGL(BcastCopyKernel<1024>, dim3(static_cast<uint32_t>(tiles)), dim3(1024), 0, stream, args);
    } else {
        return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t LaunchA2aPlan(const A2aArgs& args, hipStream_t stream)
{
    hipLaunchKernelGGL(A2aPlanKernel, dim3(1), dim3(1024), 0, stream, args);
    return hipGetLastError();
}

hipError_t LaunchA2aCopy(const A2aArgs& args, uint32_t nTiles, hipStream_t stream)
{
    if (nTiles == 0) {
        return hipSuccess;
    }
    if (args.tileBytes == 4096) {
        hipLaunchKernelGGL(A2aCopyKernel<256>, dim3(nTiles), dim3(256), 0, stream, args);
    } else if (args.tileBytes == 16384) {
        hipLaunchKernelGGL(A2aCopyKernel<1024>, dim3(nTiles), dim3(1024), 0, stream, args);
    } else {
        return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace hccl_amd
