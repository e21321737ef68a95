// What one MI355X gives for the memory access patterns of the loopback collectives, measured with bare kernels
// that do nothing but the loads, one add per operand and the stores: the yardstick the library's kernels are
// held against, and the experiments behind the shapes they have.
//
//   reads / writes alone          N read streams, or N write streams, one 16-byte vector per lane
//   fused N reads + N writes      the AllReduce pattern in one kernel
//   slab                          the same work as two kernels per piece: N reads folded into a slab of P MiB,
//                                 then the slab written to the N destinations (by one wavefront per tile, or by
//                                 wavefronts that take D destinations each)
//   one source, N destinations    the AllGather / Broadcast pattern: one wavefront per tile storing to every
//                                 destination, against D destinations per wavefront with the wavefronts of one
//                                 tile on the same XCD (workgroup indices 8 apart)
//
// Build: make -C examples      Run: examples/bin/hbm_patterns [ranks=16] [MiB per rank=256]
// Prints one line per pattern: time per pass, bytes moved per second, fraction of the 8 TB/s HBM peak.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>

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
    U4* slab;
};

__device__ __forceinline__ U4 LoadNt(const U4* p) { return __builtin_nontemporal_load((const __attribute__((address_space(1))) U4*)p); }
__device__ __forceinline__ U4 LoadPlain(const U4* p) { return *((const __attribute__((address_space(1))) U4*)p); }
// STORE: 0 non-temporal, 1 written through at system scope, 2 plain
template <int STORE>
__device__ __forceinline__ void Store(U4 v, U4* p)
{
    if (STORE == 0) {
        __builtin_nontemporal_store(v, (__attribute__((address_space(1))) U4*)p);
    } else if (STORE == 1) {
        asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1" : : "v"(p), "v"(v) : "memory");
    } else {
        *((__attribute__((address_space(1))) U4*)p) = v;
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

template <int N, bool READ, bool WRITE, int STORE>
__global__ __launch_bounds__(64) void Streams(Bufs b, size_t first, size_t nVec)
{
    const size_t o = static_cast<size_t>(blockIdx.x) * 64 + threadIdx.x;
    if (o >= nVec) {
        return;
    }
    const size_t idx = first + o;
    U4 acc = {1u, 2u, 3u, static_cast<uint32_t>(idx)};
    if (READ) {
        U4 v[N];
#pragma unroll
        for (int i = 0; i < N; ++i) {
            v[i] = LoadNt(b.src[i] + idx);
        }
        AllIssued<N>(v);
        acc = v[0];
#pragma unroll
        for (int i = 1; i < N; ++i) {
            acc += v[i];
        }
    }
    if (WRITE) {
#pragma unroll
        for (int i = 0; i < N; ++i) {
            Store<STORE>(acc, b.dst[i] + idx);
        }
    } else if (acc.x == 0x12345678u && acc.y == 0x9ABCDEF0u) {
        Store<STORE>(acc, b.dst[0] + idx);   // keeps the loads alive
    }
}

// N reads folded into slab[o]
template <int N>
__global__ __launch_bounds__(64) void ToSlab(Bufs b, size_t first, size_t nVec)
{
    const size_t o = static_cast<size_t>(blockIdx.x) * 64 + threadIdx.x;
    if (o >= nVec) {
        return;
    }
    U4 v[N];
#pragma unroll
    for (int i = 0; i < N; ++i) {
        v[i] = LoadNt(b.src[i] + first + o);
    }
    AllIssued<N>(v);
    U4 acc = v[0];
#pragma unroll
    for (int i = 1; i < N; ++i) {
        acc += v[i];
    }
    Store<1>(acc, b.slab + o);
}

// source[o] (the slab, or src[0] + first) to D destinations per wavefront.  XCD: the G = N / D wavefronts of one
// tile have workgroup indices 8 apart (same XCD), and the source is loaded with a plain load so that its L2
// serves all but the first; otherwise group g covers all tiles before group g + 1 starts.
template <int N, int D, int STORE, bool XCD>
__global__ __launch_bounds__(64) void Fan(Bufs b, const U4* source, size_t first, size_t nVec)
{
    constexpr int G = N / D;
    const size_t blk = blockIdx.x;
    size_t tile;
    int g;
    if (XCD) {
        const size_t row = blk / (8 * G);
        const size_t j = blk % (8 * G);
        tile = row * 8 + (j & 7);
        g = static_cast<int>(j >> 3);
    } else {
        const size_t tiles = (nVec + 63) / 64;
        g = static_cast<int>(blk / tiles);
        tile = blk - static_cast<size_t>(g) * tiles;
    }
    const size_t o = tile * 64 + threadIdx.x;
    if (o >= nVec) {
        return;
    }
    const U4 v = XCD ? LoadPlain(source + o) : LoadNt(source + o);
#pragma unroll
    for (int i = 0; i < D; ++i) {
        Store<STORE>(v, b.dst[g * D + i] + first + o);
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
    printf("N=%-2d %-66s %8.3f ms %6.0f GB/s  %.3f\n", n, what, ms, bytes / ms / 1e6, bytes / ms / 1e6 / kPeakGBs);
    fflush(stdout);
}

template <int N, int D>
void SlabRow(const Bufs& b, size_t nVec, size_t pieceMiB, double total)
{
    size_t piece = (pieceMiB << 20) / 16;
    piece = piece < nVec ? piece : nVec;
    const unsigned blocks = static_cast<unsigned>((piece + 63) / 64);
    const unsigned fanBlocks = D == N ? blocks : (blocks + 7) / 8 * 8 * (N / D);
    const float ms = MsPerPass([&] {
        for (size_t first = 0; first < nVec; first += piece) {
            hipLaunchKernelGGL((ToSlab<N>), dim3(blocks), dim3(64), 0, 0, b, first, piece);
            hipLaunchKernelGGL((Fan<N, D, D == N ? 1 : 0, D != N>), dim3(fanBlocks), dim3(64), 0, 0, b, b.slab, first, piece);
        }
    });
    char what[128];
    snprintf(what, sizeof what, "slab of %3zu MiB: fold kernel, then %d destination(s) per wavefront", pieceMiB, D);
    Report(N, what, ms, total);
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
    CK(hipMalloc((void**)&b.slab, 128u << 20));
    const unsigned blocks = static_cast<unsigned>((nVec + 63) / 64);
    const double half = static_cast<double>(N) * bytesPerRank;
    Report(N, "reads alone", MsPerPass([&] { hipLaunchKernelGGL((Streams<N, true, false, 0>), dim3(blocks), dim3(64), 0, 0, b, size_t(0), nVec); }), half);
    Report(N, "writes alone, non-temporal", MsPerPass([&] { hipLaunchKernelGGL((Streams<N, false, true, 0>), dim3(blocks), dim3(64), 0, 0, b, size_t(0), nVec); }), half);
    Report(N, "writes alone, written through", MsPerPass([&] { hipLaunchKernelGGL((Streams<N, false, true, 1>), dim3(blocks), dim3(64), 0, 0, b, size_t(0), nVec); }), half);
    Report(N, "fused N reads + N writes, non-temporal stores", MsPerPass([&] { hipLaunchKernelGGL((Streams<N, true, true, 0>), dim3(blocks), dim3(64), 0, 0, b, size_t(0), nVec); }), 2 * half);
    Report(N, "fused N reads + N writes, stores written through", MsPerPass([&] { hipLaunchKernelGGL((Streams<N, true, true, 1>), dim3(blocks), dim3(64), 0, 0, b, size_t(0), nVec); }), 2 * half);
    for (size_t pieceMiB : {16, 32, 64, 128}) {
        SlabRow<N, N>(b, nVec, pieceMiB, 2 * half);
        SlabRow<N, 2>(b, nVec, pieceMiB, 2 * half);
    }
    // one source (src[0]), N destinations, whole buffers and the first 64 MiB of them
    for (size_t span : {bytesPerRank, static_cast<size_t>(64) << 20}) {
        const size_t vecs = (span < bytesPerRank ? span : bytesPerRank) / 16;
        const unsigned bl = static_cast<unsigned>((vecs + 63) / 64);
        const double moved = (1.0 + N) * vecs * 16;
        char what[128];
        snprintf(what, sizeof what, "1 source of %zu MiB to N destinations, one wavefront per tile", vecs >> 16);
        Report(N, what, MsPerPass([&] { hipLaunchKernelGGL((Fan<N, N, 1, false>), dim3(bl), dim3(64), 0, 0, b, b.src[0], size_t(0), vecs); }), moved);
        snprintf(what, sizeof what, "1 source of %zu MiB to N destinations, 2 per wavefront, tile's wavefronts on one XCD", vecs >> 16);
        Report(N, what, MsPerPass([&] { hipLaunchKernelGGL((Fan<N, 2, 0, true>), dim3((bl + 7) / 8 * 8 * (N / 2)), dim3(64), 0, 0, b, b.src[0], size_t(0), vecs); }), moved);
        snprintf(what, sizeof what, "1 source of %zu MiB to N destinations, 2 per wavefront, group after group", vecs >> 16);
        Report(N, what, MsPerPass([&] { hipLaunchKernelGGL((Fan<N, 2, 0, false>), dim3(bl * (N / 2)), dim3(64), 0, 0, b, b.src[0], size_t(0), vecs); }), moved);
    }
    for (int i = 0; i < N; ++i) {
        CK(hipFree((void*)b.src[i]));
        CK(hipFree(b.dst[i]));
    }
    CK(hipFree(b.slab));
}

int main(int argc, char** argv)
{
    const int n = argc > 1 ? atoi(argv[1]) : 16;
    const size_t mib = argc > 2 ? static_cast<size_t>(atoi(argv[2])) : 256;
    if ((n != 6 && n != 8 && n != 16) || mib < 64 || mib > 2048) {
        printf("usage: hbm_patterns [ranks: 6, 8 or 16] [MiB per rank: 64 .. 2048]\n");
        return 1;
    }
    CK(hipEventCreate(&g_start));
    CK(hipEventCreate(&g_stop));
    printf("pattern%62s time per pass   moved   of 8 TB/s\n", "");
    if (n == 16) {
        Run<16>(mib << 20);
    } else if (n == 8) {
        Run<8>(mib << 20);
    } else {
        Run<6>(mib << 20);
    }
    return 0;
}
