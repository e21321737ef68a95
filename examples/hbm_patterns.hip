// What one MI355X gives for the memory access patterns of the loopback collectives, measured with bare kernels
// that do nothing but the loads, one add per operand and the stores: the yardstick the library's kernels are
// held against, and the experiments behind the shapes they have.
//
//   reads alone                   N read streams, one 16-byte vector per lane, one wavefront per 1 KiB tile
//   writes alone                  N write streams from one wavefront per tile, or dealt to the W wavefronts of a
//                                 workgroup (W = N: one stream per wavefront)
//   fused N reads + N writes      the AllReduce pattern in one kernel; with the stores of a tile shared by W
//                                 wavefronts (wavefront 0 folds and hands the result over through LDS)
//   fold + fan-out                the same work as two kernels per piece of P MiB: N reads folded into the first
//                                 destination, then that range (still cached) to the other N - 1 destinations with
//                                 one wavefront per destination; also with the two kernels of neighbouring pieces
//                                 overlapped on two streams
//   one source, N destinations    the AllGather / Broadcast pattern, source read from memory
//
//   placement                     `hbm_patterns place <ranks> <MiB>`: the fused and the fold kernels over buffers carved
//                                 out of one allocation at a stride of the buffer size + D, for a list of D: how much
//                                 the relative position of the peers' buffers is worth
//   small messages                `hbm_patterns small <MiB>`: eight ranks of a few MiB over buffer sets in rotation (no
//                                 pass finds its data cached): an empty launch of the same grid, reads, writes, fused
//   scalar preamble               `hbm_patterns chain <ranks> <MiB>` (and the last rows of `small`): the fused pattern
//                                 behind 0 .. 14 scalar loads that each wait for the one before, with one and with
//                                 three wavefronts per tile: what fetching launch parameters one by one costs
//
// Build: make -C examples      Run: examples/bin/hbm_patterns [ranks=16] [MiB per rank=256]
// Prints one line per pattern: time per pass, bytes moved per second, fraction of the 8 TB/s HBM peak.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>

typedef uint32_t U4 __attribute__((ext_vector_type(4)));
#define CK(x)                                                                      \
    do {                                                                           \
        hipError_t e_ = (x);                                                       \
        if (e_ != hipSuccess) {                                                    \
            printf("%s failed: %s (line %d)\n", #x, hipGetErrorString(e_), __LINE__); \
            exit(1);                                                               \
        }                                                                          \
    } while (0)

constexpr int kMaxStreams = 16;
constexpr double kPeakGBs = 8000.0;
struct Bufs {
    const U4* src[kMaxStreams];
    U4* dst[kMaxStreams];
};

__device__ __forceinline__ U4 LoadNt(const U4* p) { return __builtin_nontemporal_load((const __attribute__((address_space(1))) U4*)p); }
__device__ __forceinline__ U4 LoadPlain(const U4* p) { return *((const __attribute__((address_space(1))) U4*)p); }
// STORE: 0 non-temporal, 1 written through at system scope
template <int STORE>
__device__ __forceinline__ void Store(U4 v, U4* p)
{
    if (STORE == 0) {
        __builtin_nontemporal_store(v, (__attribute__((address_space(1))) U4*)p);
    } else {
        asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1" : : "v"(p), "v"(v) : "memory");
    }
}
template <int N>
__device__ __forceinline__ void AllIssued(U4* v)
{
#pragma unroll
    for (int i = 0; i < N; ++i) {
        asm volatile("" : "+v"(v[i]));
    }
}
template <int N>
__device__ __forceinline__ U4 Fold(const Bufs& b, size_t idx)
{
    U4 v[N];
#pragma unroll
    for (int i = 0; i < N; ++i) {
        v[i] = LoadNt(b.src[i] + idx);
    }
    AllIssued<N>(v);
    U4 acc = v[0];
#pragma unroll
    for (int i = 1; i < N; ++i) {
        acc += v[i];
    }
    return acc;
}

// Every size here is a multiple of 1 KiB, so a workgroup never has lanes without a vector.
//
// W wavefronts per tile.  READ: wavefront 0 folds the tile (and hands the result to the others through LDS when
// W > 1).  WRITE: wavefront w stores to destinations w, w + W, ...
template <int N, int W, bool READ, bool WRITE, int STORE>
__global__ __launch_bounds__(64 * W) void Streams(Bufs b, size_t nVec)
{
    __shared__ U4 parked[64];
    const unsigned lane = threadIdx.x & 63u;
    const unsigned wave = threadIdx.x >> 6;
    const size_t idx = static_cast<size_t>(blockIdx.x) * 64 + lane;
    U4 acc = {1u, 2u, 3u, static_cast<uint32_t>(idx)};
    if (READ) {
        if (wave == 0) {
            acc = Fold<N>(b, idx);
            if (W > 1) {
                parked[lane] = acc;
            }
        }
        if (W > 1) {
            __syncthreads();
            if (wave != 0) {
                acc = parked[lane];
            }
        }
    }
    if (WRITE) {
#pragma unroll
        for (int i = 0; i < (N + W - 1) / W; ++i) {
            if (wave + W * i < N) {
                Store<STORE>(acc, b.dst[wave + W * i] + idx);
            }
        }
    } else if (acc.x == 0x12345678u && acc.y == 0x9ABCDEF0u) {
        Store<STORE>(acc, b.dst[0] + idx);   // keeps the loads alive
    }
}

// The fused pattern behind `rounds` dependent scalar loads (the address of each comes out of the one before): what a
// kernel pays whose wavefronts fetch their launch parameters one after the other before the first vector load.
// Table entries are below 256, so the chain's result adds nothing to the index; the compiler cannot know that.
template <int N, int W>
__global__ __launch_bounds__(64 * W) void StreamsAfterChain(Bufs b, const uint32_t* chain, int rounds, size_t nVec)
{
    typedef const __attribute__((address_space(4))) uint32_t* K32;
    __shared__ U4 parked[64];
    const K32 table = (K32)(uintptr_t)chain;
    uint32_t x = blockIdx.x & 255u;
    for (int r = 0; r < rounds; ++r) {
        x = table[x & 255u];
    }
    const unsigned lane = threadIdx.x & 63u;
    const unsigned wave = threadIdx.x >> 6;
    const size_t idx = static_cast<size_t>(blockIdx.x) * 64 + lane + (x >> 31);
    U4 acc = {1u, 2u, 3u, static_cast<uint32_t>(idx)};
    if (wave == 0) {
        acc = Fold<N>(b, idx);
        if (W > 1) {
            parked[lane] = acc;
        }
    }
    if (W > 1) {
        __syncthreads();
        if (wave != 0) {
            acc = parked[lane];
        }
    }
#pragma unroll
    for (int i = 0; i < (N + W - 1) / W; ++i) {
        if (wave + W * i < N) {
            Store<0>(acc, b.dst[wave + W * i] + idx);
        }
    }
}

// N reads folded into dst[0], from element `first` on
template <int N>
__global__ __launch_bounds__(64) void FoldToFirst(Bufs b, size_t first)
{
    const size_t idx = first + static_cast<size_t>(blockIdx.x) * 64 + threadIdx.x;
    Store<1>(Fold<N>(b, idx), b.dst[0] + idx);
}

// `source` to the destinations firstDst, firstDst + 1, ...: wavefront w of the workgroup takes destinations
// firstDst + w, firstDst + w + W, ... below N.  HOT: the source has just been written (plain load, non-temporal
// stores); otherwise it comes from memory (non-temporal load, stores written through).
template <int N, int W, int HOT>
__global__ __launch_bounds__(64 * W) void FanOut(Bufs b, const U4* source, int firstDst, size_t first)
{
    const unsigned wave = threadIdx.x >> 6;
    const size_t idx = first + static_cast<size_t>(blockIdx.x) * 64 + (threadIdx.x & 63u);
    const U4 v = HOT ? LoadPlain(source + idx) : LoadNt(source + idx);   // HOT == 2: source from memory through the caches
#pragma unroll
    for (int i = 0; i < (N + W - 1) / W; ++i) {
        const int d = firstDst + static_cast<int>(wave) + W * i;
        if (d < N) {
            Store<HOT == 1 ? 0 : 1>(v, b.dst[d] + idx);
        }
    }
}

// One source from memory to N destinations, the loading done once per tile: wavefront 0 loads the tile and hands it
// to the other W - 1 wavefronts through LDS; wavefront w stores to destinations w, w + W, ...
template <int N, int W>
__global__ __launch_bounds__(64 * W) void FanOutShared(Bufs b, const U4* source)
{
    __shared__ U4 parked[64];
    const unsigned lane = threadIdx.x & 63u;
    const unsigned wave = threadIdx.x >> 6;
    const size_t idx = static_cast<size_t>(blockIdx.x) * 64 + lane;
    U4 v = {0u, 0u, 0u, 0u};
    if (wave == 0) {
        v = LoadNt(source + idx);
        parked[lane] = v;
    }
    __syncthreads();
    if (wave != 0) {
        v = parked[lane];
    }
#pragma unroll
    for (int i = 0; i < (N + W - 1) / W; ++i) {
        const int d = static_cast<int>(wave) + W * i;
        if (d < N) {
            Store<1>(v, b.dst[d] + idx);
        }
    }
}

hipEvent_t g_start, g_stop;
template <class F>
float MsPerPass(F pass)
{
    for (int i = 0; i < 2; ++i) {
        pass();
    }
    CK(hipEventRecord(g_start));
    for (int i = 0; i < 6; ++i) {
        pass();
    }
    CK(hipEventRecord(g_stop));
    CK(hipEventSynchronize(g_stop));
    float ms = 0;
    CK(hipEventElapsedTime(&ms, g_start, g_stop));
    return ms / 6;
}

void Report(int n, const char* what, float ms, double bytes)
{
    printf("N=%-2d %-72s %8.4f ms %6.0f GB/s  %.3f\n", n, what, ms, bytes / ms / 1e6, bytes / ms / 1e6 / kPeakGBs);
    fflush(stdout);
}

template <int N, int W>
void SplitRows(const Bufs& b, size_t nVec, double half)
{
    const unsigned blocks = static_cast<unsigned>(nVec / 64);
    char what[128];
    snprintf(what, sizeof what, "writes alone over %d wavefronts per tile, written through", W);
    Report(N, what, MsPerPass([&] { hipLaunchKernelGGL((Streams<N, W, false, true, 1>), dim3(blocks), dim3(64 * W), 0, 0, b, nVec); }), half);
    snprintf(what, sizeof what, "fused, wavefront 0 folds, %d wavefronts store, non-temporal", W);
    Report(N, what, MsPerPass([&] { hipLaunchKernelGGL((Streams<N, W, true, true, 0>), dim3(blocks), dim3(64 * W), 0, 0, b, nVec); }), 2 * half);
}

template <int N>
void FoldFanRow(const Bufs& b, size_t nVec, size_t pieceMiB, bool twoStreams, hipStream_t other, hipEvent_t* folded, hipEvent_t joined)
{
    size_t piece = (pieceMiB << 20) / 16;
    piece = piece < nVec ? piece : nVec;
    constexpr int W = N - 1;
    const float ms = MsPerPass([&] {
        int k = 0;
        for (size_t first = 0; first < nVec; first += piece, ++k) {
            const unsigned blocks = static_cast<unsigned>((first + piece <= nVec ? piece : nVec - first) / 64);
            hipLaunchKernelGGL((FoldToFirst<N>), dim3(blocks), dim3(64), 0, 0, b, first);
            if (twoStreams) {
                CK(hipEventRecord(folded[k % 64], 0));
                CK(hipStreamWaitEvent(other, folded[k % 64], 0));
            }
            hipLaunchKernelGGL((FanOut<N, W, 1>), dim3(blocks), dim3(64 * W), 0, twoStreams ? other : 0, b, b.dst[0], 1, first);
        }
        if (twoStreams) {
            CK(hipEventRecord(joined, other));
            CK(hipStreamWaitEvent(0, joined, 0));
        }
    });
    char what[128];
    snprintf(what, sizeof what, "fold + fan-out, pieces of %3zu MiB%s", pieceMiB, twoStreams ? ", neighbouring pieces overlapped on two streams" : "");
    Report(N, what, ms, 2.0 * N * nVec * 16);
}

template <int N>
void Run(size_t bytesPerRank)
{
    const size_t nVec = bytesPerRank / 16;
    Bufs b{};
    for (int i = 0; i < N; ++i) {
        CK(hipMalloc((void**)&b.src[i], bytesPerRank));
        CK(hipMemset((void*)b.src[i], 1 + i, bytesPerRank));
        CK(hipMalloc((void**)&b.dst[i], bytesPerRank));
    }
    hipStream_t other;
    CK(hipStreamCreateWithFlags(&other, hipStreamNonBlocking));
    hipEvent_t folded[64], joined;
    for (hipEvent_t& ev : folded) {
        CK(hipEventCreateWithFlags(&ev, hipEventDisableTiming));
    }
    CK(hipEventCreateWithFlags(&joined, hipEventDisableTiming));
    const unsigned blocks = static_cast<unsigned>(nVec / 64);
    const double half = static_cast<double>(N) * bytesPerRank;
    Report(N, "reads alone", MsPerPass([&] { hipLaunchKernelGGL((Streams<N, 1, true, false, 0>), dim3(blocks), dim3(64), 0, 0, b, nVec); }), half);
    Report(N, "writes alone, one wavefront per tile, non-temporal", MsPerPass([&] { hipLaunchKernelGGL((Streams<N, 1, false, true, 0>), dim3(blocks), dim3(64), 0, 0, b, nVec); }), half);
    Report(N, "writes alone, one wavefront per tile, written through", MsPerPass([&] { hipLaunchKernelGGL((Streams<N, 1, false, true, 1>), dim3(blocks), dim3(64), 0, 0, b, nVec); }), half);
    Report(N, "fused N reads + N writes, non-temporal stores", MsPerPass([&] { hipLaunchKernelGGL((Streams<N, 1, true, true, 0>), dim3(blocks), dim3(64), 0, 0, b, nVec); }), 2 * half);
    Report(N, "fused N reads + N writes, stores written through", MsPerPass([&] { hipLaunchKernelGGL((Streams<N, 1, true, true, 1>), dim3(blocks), dim3(64), 0, 0, b, nVec); }), 2 * half);
    SplitRows<N, 2>(b, nVec, half);
    SplitRows<N, 3>(b, nVec, half);
    SplitRows<N, 4>(b, nVec, half);
    SplitRows<N, N>(b, nVec, half);
    for (size_t pieceMiB : {16, 64, 256}) {
        FoldFanRow<N>(b, nVec, pieceMiB, false, other, folded, joined);
    }
    FoldFanRow<N>(b, nVec, 64, true, other, folded, joined);
    // one source (src[k], another one every pass) to N destinations
    int pass = 0;
    const double moved = (1.0 + N) * bytesPerRank;
    Report(N, "1 source to N destinations, one wavefront per tile", MsPerPass([&] {
               hipLaunchKernelGGL((FanOut<N, 1, 0>), dim3(blocks), dim3(64), 0, 0, b, b.src[pass++ % N], 0, size_t(0));
           }), moved);
    Report(N, "1 source to N destinations, two wavefronts per tile", MsPerPass([&] {
               hipLaunchKernelGGL((FanOut<N, 2, 0>), dim3(blocks), dim3(128), 0, 0, b, b.src[pass++ % N], 0, size_t(0));
           }), moved);
    Report(N, "1 source to N destinations, three wavefronts per tile, cached loads", MsPerPass([&] {
               hipLaunchKernelGGL((FanOut<N, 3, 2>), dim3(blocks), dim3(192), 0, 0, b, b.src[pass++ % N], 0, size_t(0));
           }), moved);
    Report(N, "1 source to N destinations, one wavefront per destination, cached loads", MsPerPass([&] {
               hipLaunchKernelGGL((FanOut<N, N, 2>), dim3(blocks), dim3(64 * N), 0, 0, b, b.src[pass++ % N], 0, size_t(0));
           }), moved);
    Report(N, "1 source to N destinations, wavefront 0 loads, 2 wavefronts store", MsPerPass([&] {
               hipLaunchKernelGGL((FanOutShared<N, 2>), dim3(blocks), dim3(128), 0, 0, b, b.src[pass++ % N]);
           }), moved);
    Report(N, "1 source to N destinations, wavefront 0 loads, 3 wavefronts store", MsPerPass([&] {
               hipLaunchKernelGGL((FanOutShared<N, 3>), dim3(blocks), dim3(192), 0, 0, b, b.src[pass++ % N]);
           }), moved);
    for (int i = 0; i < N; ++i) {
        CK(hipFree((void*)b.src[i]));
        CK(hipFree(b.dst[i]));
    }
    CK(hipStreamDestroy(other));
}

// Nothing but the launch: what a grid of that many one-wavefront workgroups costs by itself.
__global__ __launch_bounds__(64) void Empty(Bufs b, size_t nVec)
{
    if (static_cast<size_t>(blockIdx.x) * 64 + threadIdx.x == nVec + 1) {   // never true
        b.dst[0][0] = U4{1u, 2u, 3u, 4u};
    }
}

template <int N>
void Placement(size_t bytesPerRank)
{
    const size_t nVec = bytesPerRank / 16;
    const unsigned blocks = static_cast<unsigned>(nVec / 64);
    const size_t gaps[] = {0, 256, 1024, 4096, 65536, 1u << 20, 2u << 20, 4u << 20, 8u << 20, 32u << 20, (32u << 20) + 4096};
    const size_t maxGap = (32u << 20) + 4096;
    const size_t gib = size_t(1) << 30;
    char* raw = nullptr;
    CK(hipMalloc((void**)&raw, 2 * N * (bytesPerRank + maxGap) + gib));
    char* pool = reinterpret_cast<char*>((reinterpret_cast<uintptr_t>(raw) + gib - 1) & ~(uintptr_t)(gib - 1));
    CK(hipMemset(pool, 3, 2 * N * (bytesPerRank + maxGap)));
    const double moved = 2.0 * N * bytesPerRank;
    for (size_t gap : gaps) {
        Bufs b{};
        for (int i = 0; i < N; ++i) {   // source i, destination i, source i + 1, ... at a stride of the size + gap
            b.src[i] = reinterpret_cast<const U4*>(pool + static_cast<size_t>(2 * i) * (bytesPerRank + gap));
            b.dst[i] = reinterpret_cast<U4*>(pool + static_cast<size_t>(2 * i + 1) * (bytesPerRank + gap));
        }
        char what[128];
        snprintf(what, sizeof what, "stride = size + %8zu B: fused, one wavefront per tile", gap);
        Report(N, what, MsPerPass([&] { hipLaunchKernelGGL((Streams<N, 1, true, true, 0>), dim3(blocks), dim3(64), 0, 0, b, nVec); }), moved);
        snprintf(what, sizeof what, "stride = size + %8zu B: fused, stores shared by 3 wavefronts", gap);
        Report(N, what, MsPerPass([&] { hipLaunchKernelGGL((Streams<N, 3, true, true, 0>), dim3(blocks), dim3(192), 0, 0, b, nVec); }), moved);
        snprintf(what, sizeof what, "stride = size + %8zu B: fold into the first destination", gap);
        Report(N, what, MsPerPass([&] { hipLaunchKernelGGL((FoldToFirst<N>), dim3(blocks), dim3(64), 0, 0, b, size_t(0)); }),
               (N + 1.0) * bytesPerRank);
    }
    CK(hipFree(raw));
}

// Rows of the fused pattern behind 0 .. 14 dependent scalar rounds, one and three wavefronts per tile.
template <int N>
void ChainRows(const Bufs* sets, int nSets, size_t nVec)
{
    uint32_t host[256];
    for (uint32_t i = 0; i < 256; ++i) {
        host[i] = (i * 37u + 11u) & 255u;
    }
    uint32_t* chain = nullptr;
    CK(hipMalloc((void**)&chain, sizeof host));
    CK(hipMemcpy(chain, host, sizeof host, hipMemcpyHostToDevice));
    const unsigned blocks = static_cast<unsigned>(nVec / 64);
    const double moved = 2.0 * N * nVec * 16;
    int pass = 0;
    for (int rounds : {0, 2, 4, 8, 14}) {
        char what[128];
        snprintf(what, sizeof what, "fused behind %2d dependent scalar loads, one wavefront per tile", rounds);
        Report(N, what, MsPerPass([&] {
                   hipLaunchKernelGGL((StreamsAfterChain<N, 1>), dim3(blocks), dim3(64), 0, 0, sets[pass++ % nSets], chain, rounds, nVec);
               }), moved);
        snprintf(what, sizeof what, "fused behind %2d dependent scalar loads, stores shared by 3 wavefronts", rounds);
        Report(N, what, MsPerPass([&] {
                   hipLaunchKernelGGL((StreamsAfterChain<N, 3>), dim3(blocks), dim3(192), 0, 0, sets[pass++ % nSets], chain, rounds, nVec);
               }), moved);
    }
    CK(hipFree(chain));
}

template <int N>
void Chain(size_t bytesPerRank)
{
    Bufs b{};
    for (int i = 0; i < N; ++i) {
        CK(hipMalloc((void**)&b.src[i], bytesPerRank));
        CK(hipMemset((void*)b.src[i], 1 + i, bytesPerRank));
        CK(hipMalloc((void**)&b.dst[i], bytesPerRank));
    }
    ChainRows<N>(&b, 1, bytesPerRank / 16);
    for (int i = 0; i < N; ++i) {
        CK(hipFree((void*)b.src[i]));
        CK(hipFree(b.dst[i]));
    }
}

void Small(size_t bytesPerRank)
{
    constexpr int N = 8;
    constexpr int kSets = 6;   // 6 x 16 x 4 MiB = 384 MiB: past the last-level cache
    const size_t nVec = bytesPerRank / 16;
    const unsigned blocks = static_cast<unsigned>(nVec / 64);
    Bufs sets[kSets] = {};
    for (Bufs& b : sets) {
        for (int i = 0; i < N; ++i) {
            CK(hipMalloc((void**)&b.src[i], bytesPerRank));
            CK(hipMemset((void*)b.src[i], 1 + i, bytesPerRank));
            CK(hipMalloc((void**)&b.dst[i], bytesPerRank));
        }
    }
    int pass = 0;
    const double half = static_cast<double>(N) * bytesPerRank;
    Report(N, "empty launch of the same grid", MsPerPass([&] { hipLaunchKernelGGL(Empty, dim3(blocks), dim3(64), 0, 0, sets[pass++ % kSets], nVec); }), 0);
    Report(N, "reads alone", MsPerPass([&] { hipLaunchKernelGGL((Streams<N, 1, true, false, 0>), dim3(blocks), dim3(64), 0, 0, sets[pass++ % kSets], nVec); }), half);
    Report(N, "writes alone, non-temporal", MsPerPass([&] { hipLaunchKernelGGL((Streams<N, 1, false, true, 0>), dim3(blocks), dim3(64), 0, 0, sets[pass++ % kSets], nVec); }), half);
    Report(N, "fused N reads + N writes, non-temporal stores", MsPerPass([&] { hipLaunchKernelGGL((Streams<N, 1, true, true, 0>), dim3(blocks), dim3(64), 0, 0, sets[pass++ % kSets], nVec); }), 2 * half);
    Report(N, "fused, stores shared by 2 wavefronts", MsPerPass([&] { hipLaunchKernelGGL((Streams<N, 2, true, true, 0>), dim3(blocks), dim3(128), 0, 0, sets[pass++ % kSets], nVec); }), 2 * half);
    ChainRows<N>(sets, kSets, nVec);
    for (Bufs& b : sets) {
        for (int i = 0; i < N; ++i) {
            CK(hipFree((void*)b.src[i]));
            CK(hipFree(b.dst[i]));
        }
    }
}

int main(int argc, char** argv)
{
    if (argc > 1 && (strcmp(argv[1], "place") == 0 || strcmp(argv[1], "small") == 0 || strcmp(argv[1], "chain") == 0)) {
        const bool chain = argv[1][0] == 'c';
        const bool place = argv[1][0] == 'p' || chain;   // both take <ranks> <MiB>
        const int ranks = place && argc > 2 ? atoi(argv[2]) : 8;
        const size_t mibArg = static_cast<size_t>(atoi(argc > (place ? 3 : 2) ? argv[place ? 3 : 2] : "4"));
        if (mibArg < 1 || mibArg > 1024 || (ranks != 6 && ranks != 8 && ranks != 16)) {
            printf("usage: hbm_patterns place|chain <ranks: 6, 8 or 16> <MiB per rank: 1 .. 1024> | hbm_patterns small <MiB per rank>\n");
            return 1;
        }
        CK(hipEventCreate(&g_start));
        CK(hipEventCreate(&g_stop));
        printf("pattern%68s time per pass   moved   of 8 TB/s\n", "");
        if (!place) {
            Small(mibArg << 20);
        } else if (chain) {
            if (ranks == 16) {
                Chain<16>(mibArg << 20);
            } else if (ranks == 8) {
                Chain<8>(mibArg << 20);
            } else {
                Chain<6>(mibArg << 20);
            }
        } else if (ranks == 16) {
            Placement<16>(mibArg << 20);
        } else if (ranks == 8) {
            Placement<8>(mibArg << 20);
        } else {
            Placement<6>(mibArg << 20);
        }
        return 0;
    }
    const int n = argc > 1 ? atoi(argv[1]) : 16;
    const size_t mib = argc > 2 ? static_cast<size_t>(atoi(argv[2])) : 256;
    if ((n != 6 && n != 8 && n != 16) || mib < 64 || mib > 2048) {
        printf("usage: hbm_patterns [ranks: 6, 8 or 16] [MiB per rank: 64 .. 2048]\n");
        return 1;
    }
    CK(hipEventCreate(&g_start));
    CK(hipEventCreate(&g_stop));
    printf("pattern%68s time per pass   moved   of 8 TB/s\n", "");
    if (n == 16) {
        Run<16>(mib << 20);
    } else if (n == 8) {
        Run<8>(mib << 20);
    } else {
        Run<6>(mib << 20);
    }
    return 0;
}
