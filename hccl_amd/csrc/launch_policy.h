// The form a collective is launched in: every threshold the launch planners use, in one place, each with the
// measurement it came from.  All figures are fractions of the 8 TB/s HBM peak on one MI355X, timed in one process
// on the same buffers (buffer sets in rotation where a set would fit the 256 MB last-level cache); boxes of the
// pool differ by a few per cent, crossovers move little.  `python -m hccl_amd.tune` times both sides of every
// threshold on the GPU at hand.
//
// Environment overrides (read at world creation) are named with each entry.
#pragma once

#include <stdint.h>

#include <initializer_list>

namespace hccl_amd {
namespace policy {

constexpr uint64_t kMiB = 1ull << 20;

// ---- AllReduce, Reduce, ReduceScatter(V): the fused reduce kernel ----------------------------------------
// Workgroups of one wavefront (64 lanes, one 16-byte vector each): small workgroups retire sooner and keep the
// window of addresses in flight compact; measured best for flat and nested programs alike (128: -9 %, 256: -3 %
// on 8 ranks x 4 MiB).  HCCL_AMD_REDUCE_THREADS.
constexpr uint32_t kReduceThreads = 64;

// Leaves whose loads are issued together.  Up to eight ranks folded into one result stream run best with
// eight-load batches (fewer registers, more wavefronts in flight: +1-2 %); a result that goes to many destinations
// and larger worlds with sixteen (+5 %).  8 ranks x 4 MiB: equal.  HCCL_AMD_REDUCE_BATCH.
inline uint32_t VecBatch(uint32_t ranks, bool oneResultStream, bool unequalGroups)
{
    return (ranks <= 8 && !unequalGroups && oneResultStream) ? 8u : 16u;
}

// Two adjacent tiles per wavefront, all sixteen loads issued before the first fold and both folds before the first
// store (kVecBatchPair; flat programs of up to eight leaves).  A launch of a few thousand tiles is one generation of
// wavefronts: all of them load, then all of them store, and the two phases add up; with pairs the second tile's
// loads travel while the first tile's arrive.  AllReduce fp32 SUM in rank order, us per collective, one tile / two:
//   ranks   1 MiB       2 MiB       3 MiB        4 MiB         6 MiB         8 MiB         12-16 MiB per rank
//     8   6.4 / 6.6   8.4 / 7.4   10.4 / 9.7   15.3 / 14.0   20.0 / 19.6   26.5 / 27.1   37.8 / 39.7, 46.8 / 47.2
//     6               6.4 / 6.3                11.8 / 10.3                 21.0 / 21.6
//     4               5.2 / 5.1                 7.6 / 7.6                  14.9 / 15.0   26.0 / 26.3
//     3                                         6.8 / 6.4                  11.3 / 11.4
//     2                                         5.7 / 4.8                   8.5 / 8.0    13.7 / 14.4
// (kernel time of 8 ranks x 4 MiB under rocprofv3: 15.7 / 14.5 us.)  A result written once does not gain: ReduceScatter
// over 8 ranks, 512 KiB / 1 / 2 / 4 MiB out per rank 9.7 / 9.3, 16.2 / 16.2, 27.6 / 28.6, 50.0 / 52.3.
// HCCL_AMD_REDUCE_PAIR = 0 / 1 forces.
inline bool PairTiles(uint32_t ranks, bool oneResultStream, uint64_t bytesPerRank)
{
    return !oneResultStream && 2 * bytesPerRank >= 3 * kMiB && bytesPerRank <= (ranks <= 3 ? 8 : 6) * kMiB;
}

// A flat fold of up to eight leaves to two to eight destinations launched from its arguments alone
// (DirectFoldKernel; every operand on a 16-byte boundary, the first destination on a 128-byte line): wavefronts per
// workgroup, 0 = not this form.  Nothing but one block of scalar loads stands in front of a wavefront's first vector
// load, the code is a few hundred instructions, and the wavefronts of a workgroup exchange their tiles so that each
// writes `waves` KiB in a row to its own destinations.  AllReduce fp32 SUM in rank order, us per collective: the
// general kernel with one tile per wavefront / two / wavefronts that exchange (kStoreWavesAllFold, 3) / this kernel
// with 2 / 3 / 4 / 6 / 8 wavefronts:
//   ranks   1 MiB                                   2 MiB                                   3 MiB                                    4 MiB                                            6 MiB                                            8 MiB                                            12 MiB per rank
//     8   6.9/6.8/7.1/ 6.3/6.5/6.6/6.6/6.6   8.4/7.4/8.2/ 6.6/6.7/6.5/7.5/6.5   10.1/9.6/10.3/ 9.2/9.1/10.1/8.6/10.2   15.7/14.4/13.6/ 15.0/14.0/14.4/13.7/13.0   20.7/20.0/18.8/ 19.1/18.9/19.9/18.6/18.6   26.6/26.6/28.4/ 26.3/25.2/26.1/26.4/26.0   37.3/39.6/40.0/ 39.2/36.8/38.8/38.3/37.8
//     6   6.2/6.2/6.1/ 5.5/5.8/5.8/5.8/5.8   6.8/6.3/7.0/ 5.8/6.0/6.0/6.0/6.1    7.7/7.9/8.2/ 7.1/6.6/6.9/6.7/7.3      12.1/10.5/10.4/ 11.1/10.7/11.3/11.0/9.5    16.4/15.2/14.4/ 14.6/14.4/14.6/13.8/14.3   20.7/20.9/21.4/ 20.8/19.1/20.5/19.8/18.9   28.7/29.4/30.2/ 29.2/27.7/28.6/28.4/28.3
//     4   5.3/5.3/5.2/ 4.7/5.0/5.0/5.0/5.0   5.4/5.3/5.7/ 4.7/5.0/5.0/5.1/5.0    6.1/6.2/6.3/ 5.5/5.6/5.3/5.6/5.7       7.7/7.6/8.0/ 7.5/7.5/7.3/7.0/6.5         11.7/10.5/9.9/ 10.6/10.5/10.5/9.9/10.1     14.6/14.7/15.4/ 14.0/13.1/13.6/13.5/13.3   20.1/20.6/20.6/ 20.7/18.8/19.3/19.1/19.4
//     2   4.3/4.4/4.5/ 3.8/4.0/4.1/4.0/4.1   4.3/4.4/4.6/ 3.8/4.1/4.0/4.0/4.1                                             5.7/4.8/6.4/ 4.7/4.6/4.4/4.8/4.4          7.4/6.0/7.6/ 5.4/5.3/5.3/5.4/5.4           8.7/7.9/9.0/ 8.0/7.5/7.6/7.6/7.2          (16 MiB: 13.6/14.3/14.4/ 13.7/13.0/13.0/13.0/13.3)
// (8 ranks x 256 / 512 KiB: 6.9 against 6.3 / 6.4; 8 ranks x 2.5 / 3.5 / 5 / 7 / 10 MiB: 8.3 -> 7.3 with 2, 12.5 -> 11.6
// with 8, 15.4 -> 15.6 with 4, 22.4 -> 23.1 with 4, 32.0 -> 31.1 with 3; 5 ranks x 4 MiB 9.1 -> 7.9, 7 ranks x 4 MiB
// 12.0 -> 11.7; 4 ranks x 16 MiB 26.0 -> 24.5 with 3, 3 ranks x 16 MiB 19.7 -> 18.8, 2 ranks x 32 MiB 23.4 -> 23.3; at
// 8 ranks x 16 MiB every form takes 46.6.)  Up to 2 MiB the launch is bound by its latency and two wavefronts are
// ahead; up to 8 MiB the whole launch is one generation of wavefronts and the longer store runs of many wavefronts
// pay, as long as the workgroups deal out evenly over the 256 CUs (8 ranks x 3 MiB = 3072 tiles: 384 workgroups of
// eight wavefronts 10.2, 512 of six 8.6; 5 MiB: 640 of eight 17.1, 1280 of four 15.6); above, three wavefronts.
// HCCL_AMD_REDUCE_DIRECT = 0 / 2 .. 8 forces.
inline uint32_t DirectFoldWaves(uint32_t nLeaves, uint32_t nDst, uint64_t bytesPerRank)
{
    (void)nLeaves;
    if (bytesPerRank > (nDst <= 4 ? 16 : 12) * kMiB) {
        return 0;
    }
    if (bytesPerRank <= 2 * kMiB) {
        return 2;
    }
    if (bytesPerRank > 8 * kMiB) {
        return 3;
    }
    // the most wavefronts whose workgroups fill whole rounds of the CUs to 95 %, else the count that fills them best
    constexpr uint64_t kCus = 256;
    const uint64_t tiles = (bytesPerRank + 1023) / 1024;
    uint32_t best = 2;
    uint64_t bestFill = 0;   // per mille
    for (uint32_t waves : {8u, 6u, 4u, 3u, 2u}) {
        const uint64_t groups = (tiles + waves - 1) / waves;
        const uint64_t rounds = (groups + kCus - 1) / kCus;
        const uint64_t fill = groups * 1000 / (rounds * kCus);
        if (fill >= 950) {
            return waves;
        }
        if (fill > bestFill) {
            bestFill = fill;
            best = waves;
        }
    }
    return best;
}

// That kernel's instantiation for nine to sixteen leaves or destinations (whole workgroups only, one tile per
// wavefront): wavefronts per workgroup, 0 = not this form.  AllReduce fp32 SUM in rank order, us per collective, the
// general kernel's best form (one tile per wavefront or wavefronts that exchange their tiles) / this kernel with
// 2 / 4 / 8 wavefronts:
//   ranks   512 KiB             1 MiB                2 MiB                  3 MiB                  4 MiB                  6 MiB per rank
//    16   9.8 / 9.5 9.8 9.7   10.0 / 9.5 9.6 9.7   13.4 / 11.9 12.5 11.3   18.2 / 18.6 18.7 17.7   24.9 / 27.5 25.7 26.4   36.4 / 37.0 38.1 36.8
//    12                        8.6 / 8.0 8.3 8.3   10.6 /  8.7  9.3  8.9   14.4 / 14.7 14.4 14.4   19.0 / 21.4 19.9 20.3   27.3 / 27.8 28.7 27.7
//    10                                             8.6 /  7.6  8.0  7.9                          16.0 / 16.9 16.9 16.1
//     9                                             8.7 /  7.1  7.2  7.3                          14.9 / 17.0 16.2 14.4
// (16 ranks x 8 MiB, where fold + fan-out takes over: 48.6 for every form.)  The short launches gain what the
// kernels for up to eight ranks gain; from 4 MiB the general kernel's exchange form is level or ahead.
// HCCL_AMD_REDUCE_DIRECT = 0 / 2 .. 8 forces.
inline uint32_t DirectFoldWideWaves(uint32_t nLeaves, uint32_t nDst, uint64_t bytesPerRank)
{
    (void)nLeaves;
    if (bytesPerRank > 3 * kMiB) {
        return 0;
    }
    if (bytesPerRank <= kMiB) {
        return 2;
    }
    return (nDst >= 14 || 2 * bytesPerRank > 5 * kMiB) ? 8 : 2;
}

// That kernel with eight wavefronts and two tiles per wavefront, for a multiple of 16 KiB per rank: sixteen loads in
// flight per lane, half as many workgroups, and 16 KiB in a row to every destination.  True where it is taken, and
// then with eight wavefronts whatever DirectFoldWaves says.  AllReduce fp32 SUM, us per collective, DirectFoldWaves'
// count with one tile per wavefront / eight wavefronts with two:
//   ranks   3 MiB        4 MiB         6 MiB         8 MiB         12 MiB        16 MiB per rank
//     8   8.6 / 8.8   12.9 / 11.2   18.5 / 18.0   25.4 / 23.5   36.6 / 35.5                 (2 MiB 6.6 / 6.8, 7 MiB 22.9 / 20.9)
//     7               11.9 / 10.2   16.8 / 16.2   22.6 / 19.5   32.1 / 29.9
//     6   6.7 / 7.2    9.4 / 9.0    14.3 / 14.6   19.1 / 16.9   27.5 / 25.0
//     5                7.9 / 7.8                  15.9 / 14.5
//     4   5.5 / 5.5    6.6 / 6.6    10.1 / 10.1   13.3 / 12.3   18.7 / 18.4   24.3 / 24.9
//     3                5.7 / 5.4                  10.4 / 8.3                  18.7 / 18.3
//     2                4.4 / 4.4                   7.2 / 6.3                  12.8 / 13.9
// It pays where the workgroups of sixteen tiles come out even over the 256 CUs (4 MiB: 256 of them, 8 MiB: 512) and
// not where they do not (8 ranks x 5 MiB: 320 workgroups, 15.6 / 16.8; 10 MiB: 640, 31.1 / 31.5).
// HCCL_AMD_REDUCE_DIRECT_TILES = 1 / 2 forces.
inline bool DirectFoldTwoTiles(uint32_t nLeaves, uint32_t nDst, uint64_t bytesPerRank)
{
    (void)nLeaves;
    (void)nDst;
    if (bytesPerRank % (16 * 1024) != 0 || 2 * bytesPerRank < 7 * kMiB || bytesPerRank > 12 * kMiB) {
        return false;
    }
    constexpr uint64_t kCus = 256;
    const uint64_t groups = bytesPerRank / (16 * 1024);
    const uint64_t rounds = (groups + kCus - 1) / kCus;
    return groups * 100 >= 70 * rounds * kCus;   // the workgroups fill whole rounds of the CUs to 70 %
}

// Every wavefront of a workgroup folds a tile of its own and, after an exchange through LDS, stores the tiles of all
// to its own destinations (kStoreWavesAllFold; flat programs, one sub-segment): the number of wavefronts per
// workgroup, 0 = not this form.  Between the launch that is one generation of wavefronts and the one that reaches a
// steady state, a fused launch to many destinations ends with every wavefront writing 1 KiB to every stream; with
// three wavefronts exchanging their tiles each writes 3 KiB in a row to a third of the streams.  AllReduce fp32 SUM in
// rank order, us per collective: one tile per wavefront / two / this form with 2 / 3 / 4 wavefronts:
//   ranks    3 MiB                 4 MiB                      5 MiB                 6 MiB                      7 MiB              7.5 - 8 MiB per rank
//     5                   10.4/ 9.3/ 9.8/ 9.3/ 9.5   12.0/10.7/10.5/10.4/10.7   13.9/13.1/12.0/12.1/12.6   15.6/15.5/14.3/16.3/14.5
//     6                   12.1/10.7/11.3/10.5/11.1   13.9/13.3/12.5/11.9/12.7   16.0/15.2/14.4/14.2/15.4   18.0/17.8/16.7/18.7/17.1   19.9/20.1/21.1/20.5/21.4
//     8   9.9/9.6/10.4/10.2/10.7   15.8/14.3/14.2/13.8/14.1   17.3/16.8/15.8/15.4/16.1   20.7/20.0/18.8/19.0/19.5   23.6/23.8/22.2/24.9/22.9   26.3/27.4/30.6/28.4/30.4
//    12   15.3/15.3/14.7/14.3/15.0   21.4/21.3/19.8/19.0/20.3                       31.2/31.3/27.3/27.8/29.4   35.6/35.6/34.6/36.1/35.2
//    16   20.3/20.2/18.2/18.3/19.2   28.8/28.7/26.2/25.1/27.0                       39.5/39.5/36.6/36.9/39.4   47.6/47.5/44.1/48.5/46.0   (8 MiB: two kernels)
//    24   28.0/27.9/26.8/26.8/28.3   42.0/41.8/39.2/38.1/41.3
//    32   37.9/37.7/35.8/35.0/37.6   54.9/54.7/51.8/50.0/58.0          (2 MiB: 25.5/25.3/24.1/25.4/27.1)
// Below the window the form loses (16 ranks x 2 MiB 12.5/12.4/13.5/14.0/14.3, 2.5 MiB 17.5/17.4/15.5/16.2/16.5; 12 ranks x
// 2 MiB 10.0/10.0/10.5/10.9/10.6; 24 ranks x 2 MiB 18.9/18.9/19.0/19.6/20.4; 2 to 4 ranks never gain; 64 ranks x 1 MiB
// 28.6/28.5/34.5/33.5/37.6).  Three wavefronts lose at 7 MiB where two still gain.  As a bare kernel eight wavefronts
// are the best (8 ranks x 4 MiB: 14.8 one tile per wavefront, 12.7 three wavefronts, 12.2 eight); inside the library
// eight measured 13.9 against 13.8 for three, so the workgroup limit stays at 256 lanes.
// HCCL_AMD_REDUCE_ALL_FOLD = 0 / 2 .. 4 forces.
inline uint32_t AllFoldWaves(uint32_t nDst, uint64_t bytesPerRank)
{
    if (nDst < 5 || nDst > 32 || bytesPerRank > 7 * kMiB) {
        return 0;
    }
    const uint64_t from = nDst >= 32 ? 2 * kMiB
                        : nDst >= 24 ? 3 * kMiB
                        : nDst >= 16 ? 5 * kMiB / 2
                        : nDst >= 12 ? 3 * kMiB
                        : nDst >= 8 ? 4 * kMiB : 5 * kMiB;
    if (bytesPerRank < from) {
        return 0;
    }
    return bytesPerRank > 6 * kMiB ? 2u : 3u;
}

// A result written once (ReduceScatter(V), Reduce, the fold of the two-kernel AllReduce) leaves through
// write-through stores, 3-4 % faster than non-temporal ones next to eight read streams; a result written to many
// destinations keeps non-temporal stores, 2-3 % faster there.  HCCL_AMD_STORE_POLICY.
inline bool WriteThrough(bool oneResultStream) { return oneResultStream; }

// Wavefronts that share the stores of a fused tile (wavefront 0 folds, every wavefront stores to its share of the
// destinations): `bytes` per rank, `elemSize` of the type.
//   4-7 destinations, from 48 MiB: two.  fp32 over 4 ranks 0.72 -> 0.74 / 0.75 -> 0.79 / 0.76 -> 0.79 at 64 / 256 /
//     512 MiB; over 6 ranks 0.70 -> 0.75 / 0.74 -> 0.79 / 0.70 -> 0.77; three wavefronts 0.77 / 0.78 / 0.76; at
//     16-32 MiB one wavefront wins by a point; two and three ranks lose at every size (0.83 -> 0.61, 0.80 -> 0.76).
//   8 and more destinations: three from 24 MiB for 4- and 8-byte types (8 ranks 0.70 -> 0.78 at 64 MiB), two from
//     64 MiB for the 1- and 2-byte types, whose folds take longer (the waiting wavefronts hold slots).
// HCCL_AMD_REDUCE_STORE_WAVES.
inline uint32_t StoreWaves(uint32_t nDst, uint64_t bytes, uint32_t elemSize)
{
    const bool longFold = elemSize < 4;
    if (nDst >= 8) {
        return longFold ? (bytes >= 64 * kMiB ? 2u : 1u) : (bytes >= 24 * kMiB ? 3u : 1u);
    }
    if (nDst >= 4) {
        return bytes >= 48 * kMiB ? 2u : 1u;
    }
    return 1u;
}
// With the stores elsewhere the folding wavefront is better off with the eight-load batch where that holds every
// leaf (fp16 RHD over 6 ranks 0.71 -> 0.75, fp16 NHR over 8 ranks 0.71 -> 0.77).
inline uint32_t VecBatchWithSharedStores(uint32_t ranks, uint32_t batch) { return ranks <= 8 ? 8u : batch; }

// ---- AllReduce as fold + fan-out ------------------------------------------------------------------------
// All ranks folded into the first recvBuf, then that range to the other recvBufs with one wavefront per
// destination.  Two kernels / fused, fp32 SUM in rank order:
//   ranks    8 MiB         16 MiB        32 MiB        64 MiB        256 MiB per rank
//     4                  0.63 / 0.62   0.69 / 0.67   0.74 / 0.74   0.77 / 0.79
//     5                  0.65 / 0.62                 0.76 / 0.72   0.79 / 0.78
//     6    0.57 / 0.58   0.66 / 0.63   0.73 / 0.69   0.78 / 0.75   0.82 / 0.79
//     8    0.60 / 0.60   0.67 / 0.62   0.75 / 0.71   0.79 / 0.78   0.82 / 0.76
//    16    0.65 / 0.57   0.74 / 0.58   0.79 / 0.73   0.82 / 0.76   0.83 / 0.74
// (2 and 3 ranks lose: 0.69 / 0.83, 0.74 / 0.80.)  HCCL_AMD_ALLREDUCE_TWO_KERNELS = 0 / 1 forces a form.
inline bool FoldThenFanOut(uint32_t nDst, uint64_t bytes)
{
    return nDst >= 12 ? bytes >= 8 * kMiB : (nDst >= 5 && bytes >= 16 * kMiB);
}
// Mesh-chunk launches write one strip per slice, so their pieces are whole slices, which pays from eight ranks on
// (8 ranks of 256 MiB 0.74 -> 0.81, 16 ranks of 64 MiB 0.71 -> 0.79; six ranks lose, 0.74 -> 0.71).
constexpr uint32_t kMeshChunkFanOutMinRanks = 8;
// A piece must still be cached when it is read back: 1 GiB per rank over 6 ranks 0.76 / 0.78 / 0.78 with pieces of
// 64 / 128 / 256 MiB, 0.64 with 512 MiB; 512 MiB per rank fp16: 0.76 / 0.74 / 0.77 / 0.67 with 96 / 176 / 256 / 352 MiB.
// HCCL_AMD_ALLREDUCE_PIECE_BYTES.
constexpr uint64_t kPieceBytes = 256 * kMiB;

// The fan-out kernel's load of the range the kernel before it wrote.  A plain load lets the wavefronts behind the
// first find the tile cached, but what it leaves in the caches slows the fold of the next piece down; a
// non-temporal load leaves nothing behind and costs where many wavefronts share a tile.  AllReduce fp32, plain /
// non-temporal: 512 MiB per rank (two pieces) over 5 / 6 / 7 / 8 / 10 / 12 ranks 0.77 / 0.79, 0.77 / 0.80, 0.78 / 0.80,
// 0.78 / 0.79, 0.77 / 0.78, 0.76 / 0.77 (fp16 RHD over 6 ranks 0.79 / 0.81); one piece of 256 MiB over 5-7 ranks
// equal, over 8 / 10 / 12 / 16 ranks 0.83 / 0.82, 0.83 / 0.82, 0.82 / 0.80, 0.81 / 0.78; 16 ranks in pieces of
// 128 MiB 0.83 / 0.79; Broadcast to 7 ranks equal.  So: up to six destinations always, up to eleven where another
// piece follows.
inline bool FanOutStreamLoad(uint32_t nDst, bool severalPieces) { return nDst <= 6 || (severalPieces && nDst <= 11); }

// ---- AllGather(V), Broadcast: gather + fan-out ----------------------------------------------------------
// The segments into the first destination with the plain copy, then that range to the other destinations.  Two
// kernels / one, `bytes` per destination: AllGather of 16 x 64 MiB 0.84 / 0.69, 16 x 16 MiB 0.76 / 0.68, 8 x 128 MiB
// 0.77 / 0.71, 8 x 8 MiB 0.76 / 0.69, 6 x 32 MiB 0.72 / 0.74, 6 ranks of 2-64 MiB at odd displacements 0.74 / 0.76,
// 4 x 64 MiB 0.67 / 0.77; Broadcast of 128 MiB to 15 ranks 0.78 / 0.68, to 7 ranks 0.81 / 0.73 (16 MiB: 0.61 / 0.65),
// to 5 ranks 0.72 / 0.77.  Six destinations: from 128 MiB per destination where every source shares its
// destination's offset from a 16-byte boundary (6 x 16 MiB 0.74 / 0.74, 6 x 32 MiB 0.77 / 0.73, 6 x 64 MiB 0.77 / 0.72,
// 6 x 128 MiB 0.76 / 0.73, Broadcast of 64 / 128 / 192 MiB 0.73 / 0.73, 0.76 / 0.72, 0.77 / 0.73; with lanes realigning the bytes the first kernel is the slower one and the one-kernel
// form stays ahead, 0.74 / 0.76); five destinations never (0.72-0.74 / 0.75-0.77 from 16 to 128 MiB per rank).
// Where the forms cross, per destination: 16 ranks 16 MiB 0.74 / 0.60, 32 MiB 0.82 / 0.59; 12 ranks 12 MiB 0.66 / 0.66,
// 24 MiB 0.68 / 0.65, 36 MiB 0.74 / 0.65; 10 ranks 20 MiB 0.69 / 0.67, 30 MiB 0.72 / 0.69, 40 MiB 0.77 / 0.72; 8 ranks
// 16 MiB 0.65 / 0.66, 24 MiB 0.70 / 0.69, 32 MiB 0.71 / 0.69, 40 MiB 0.73 / 0.71; 7 ranks 21-42 MiB 0.65-0.69 / 0.69-0.72,
// 49 MiB 0.72 / 0.71.  Since the gather step runs through the copy kernel that is launched from its arguments alone
// (a quarter faster), with aligned operands: AllGather of 16 x 16 MiB 0.85 / 0.68, 12 x 8 MiB 0.81 / 0.68, 8 x 8 MiB
// 0.81 / 0.72, 8 x 24 MiB 0.85 / 0.70, 7 x 8 MiB 0.79 / 0.74, 7 x 32 MiB 0.84 / 0.74, 6 x 16 MiB 0.80 / 0.76, 6 x 32 MiB
// 0.82 / 0.74, 5 x 16 MiB 0.75 / 0.77, 5 x 64 MiB 0.77 / 0.76, 4 x 64 MiB 0.76 / 0.77; Broadcast to 15 ranks of 16 / 64 MiB
// 0.76 / 0.64, 0.86 / 0.66, to 6 ranks of 32 / 64 / 128 MiB 0.70 / 0.72, 0.75 / 0.73, 0.82 / 0.73, to 5 ranks of 64 /
// 128 MiB 0.74 / 0.76, 0.78 / 0.78, to 4 ranks 0.71-0.73 / 0.76-0.78: six destinations now from 64 MiB.  And per
// destination: 8 ranks 8 MiB 0.61 / 0.67, 16 MiB 0.69 / 0.66, 24 MiB 0.74 / 0.67; 10 ranks 10 MiB 0.63 / 0.65, 20 MiB
// 0.70 / 0.67; 12 ranks 12 MiB 0.67 / 0.66; Broadcast to 8 ranks of 8 / 16 / 24 MiB 0.59 / 0.62, 0.70 / 0.67, 0.74 / 0.67,
// to 11 ranks 0.63 / 0.64, 0.71 / 0.66, 0.75 / 0.68, to 14 ranks of 4 / 8 / 16 MiB 0.36 / 0.40, 0.70 / 0.66, 0.75 / 0.63:
// eight to thirteen destinations from 16 MiB, fourteen and more from 8 MiB.
// HCCL_AMD_COPY_TWO_KERNELS = 0 / 1 forces a form.
inline bool GatherThenFanOut(uint32_t nDst, uint64_t bytes, bool congruent)
{
    if (nDst >= 14) {
        return bytes >= 8 * kMiB;
    }
    if (nDst >= 8) {
        return bytes >= 16 * kMiB;
    }
    return (nDst == 7 && bytes >= 48 * kMiB) || (nDst == 6 && congruent && bytes >= 64 * kMiB);
}

}  // namespace policy
}  // namespace hccl_amd
