// One host thread per rank, like the reference's examples/02_collectives (01_allreduce/main.cc:46-124 and its
// siblings): every thread joins the world with HcclCommInitRootInfo, owns a stream and two device buffers, and
// issues blocking collectives.  The N "devices" of the reference are N ranks of a loopback world on the one GPU.
// Runs AllReduce, ReduceScatter, AllGather, Broadcast and AlltoAll on closed-form inputs and checks every element;
// prints PASS and exits 0 when all ranks agree.
//
// Build: make -C examples      Run: examples/bin/collectives_threads [ranks] [count]
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <thread>
#include <vector>

#include "hccl.h"

#define HIPCHECK(x)                                                                            \
    do {                                                                                       \
        hipError_t e_ = (x);                                                                   \
        if (e_ != hipSuccess) {                                                                \
            fprintf(stderr, "%s:%d %s: %s\n", __FILE__, __LINE__, #x, hipGetErrorString(e_));  \
            exit(2);                                                                           \
        }                                                                                      \
    } while (0)
#define HCCLCHECK(x)                                                                           \
    do {                                                                                       \
        HcclResult r_ = (x);                                                                   \
        if (r_ != HCCL_SUCCESS) {                                                              \
            fprintf(stderr, "%s:%d %s: %s\n", __FILE__, __LINE__, #x, HcclGetErrorString(r_)); \
            exit(3);                                                                           \
        }                                                                                      \
    } while (0)

namespace {

std::atomic<int> g_failures{0};

void Expect(bool ok, uint32_t rank, const char* what, uint64_t index, double got, double want)
{
    if (!ok && g_failures.fetch_add(1) < 8) {
        fprintf(stderr, "rank %u %s[%llu]: got %.9g want %.9g\n", rank, what, (unsigned long long)index, got, want);
    }
}

// Rank r's element i: small integers, so that every sum is exact in fp32 whatever the order.
float Input(uint32_t rank, uint64_t i) { return static_cast<float>((rank + 1) * 3 + (i % 251)); }

void RankMain(uint32_t nRanks, const HcclRootInfo* rootInfo, uint32_t rank, uint64_t count)
{
    HIPCHECK(hipSetDevice(0));
    HcclComm comm;
    HCCLCHECK(HcclCommInitRootInfo(nRanks, rootInfo, rank, &comm));
    hipStream_t stream;
    HIPCHECK(hipStreamCreate(&stream));

    const uint64_t big = count * nRanks;
    float *send = nullptr, *recv = nullptr;
    HIPCHECK(hipMalloc(reinterpret_cast<void**>(&send), big * sizeof(float)));
    HIPCHECK(hipMalloc(reinterpret_cast<void**>(&recv), big * sizeof(float)));
    std::vector<float> host(big), out(big);
    for (uint64_t i = 0; i < big; ++i) {
        host[i] = Input(rank, i);
    }
    HIPCHECK(hipMemcpyAsync(send, host.data(), big * sizeof(float), hipMemcpyHostToDevice, stream));

    // AllReduce: every element becomes the sum over ranks
    HCCLCHECK(HcclAllReduce(send, recv, count, HCCL_DATA_TYPE_FP32, HCCL_REDUCE_SUM, comm, stream));
    HIPCHECK(hipMemcpyAsync(out.data(), recv, count * sizeof(float), hipMemcpyDeviceToHost, stream));
    HIPCHECK(hipStreamSynchronize(stream));
    for (uint64_t i = 0; i < count; ++i) {
        float want = 0;
        for (uint32_t r = 0; r < nRanks; ++r) want += Input(r, i);
        Expect(out[i] == want, rank, "allreduce", i, out[i], want);
    }

    // ReduceScatter: rank k keeps slice k of the sums
    HCCLCHECK(HcclReduceScatter(send, recv, count, HCCL_DATA_TYPE_FP32, HCCL_REDUCE_SUM, comm, stream));
    HIPCHECK(hipMemcpyAsync(out.data(), recv, count * sizeof(float), hipMemcpyDeviceToHost, stream));
    HIPCHECK(hipStreamSynchronize(stream));
    for (uint64_t i = 0; i < count; ++i) {
        float want = 0;
        for (uint32_t r = 0; r < nRanks; ++r) want += Input(r, rank * count + i);
        Expect(out[i] == want, rank, "reducescatter", i, out[i], want);
    }

    // AllGather: block r of the output is rank r's first `count` elements
    HCCLCHECK(HcclAllGather(send, recv, count, HCCL_DATA_TYPE_FP32, comm, stream));
    HIPCHECK(hipMemcpyAsync(out.data(), recv, big * sizeof(float), hipMemcpyDeviceToHost, stream));
    HIPCHECK(hipStreamSynchronize(stream));
    for (uint64_t i = 0; i < big; ++i) {
        const float want = Input(static_cast<uint32_t>(i / count), i % count);
        Expect(out[i] == want, rank, "allgather", i, out[i], want);
    }

    // AlltoAll: block j of the output is block `rank` of rank j's input
    HCCLCHECK(HcclAlltoAll(send, count, HCCL_DATA_TYPE_FP32, recv, count, HCCL_DATA_TYPE_FP32, comm, stream));
    HIPCHECK(hipMemcpyAsync(out.data(), recv, big * sizeof(float), hipMemcpyDeviceToHost, stream));
    HIPCHECK(hipStreamSynchronize(stream));
    for (uint64_t i = 0; i < big; ++i) {
        const float want = Input(static_cast<uint32_t>(i / count), rank * count + i % count);
        Expect(out[i] == want, rank, "alltoall", i, out[i], want);
    }

    // Broadcast from the last rank
    const uint32_t root = nRanks - 1;
    HCCLCHECK(HcclBroadcast(send, count, HCCL_DATA_TYPE_FP32, root, comm, stream));
    HIPCHECK(hipMemcpyAsync(out.data(), send, count * sizeof(float), hipMemcpyDeviceToHost, stream));
    HIPCHECK(hipStreamSynchronize(stream));
    for (uint64_t i = 0; i < count; ++i) {
        Expect(out[i] == Input(root, i), rank, "broadcast", i, out[i], Input(root, i));
    }

    HCCLCHECK(HcclCommDestroy(comm));
    HIPCHECK(hipFree(send));
    HIPCHECK(hipFree(recv));
    HIPCHECK(hipStreamDestroy(stream));
}

}  // namespace

int main(int argc, char** argv)
{
    const uint32_t nRanks = argc > 1 ? static_cast<uint32_t>(atoi(argv[1])) : 8;
    const uint64_t count = argc > 2 ? static_cast<uint64_t>(atoll(argv[2])) : 100003;
    HIPCHECK(hipSetDevice(0));
    HcclRootInfo rootInfo;
    HCCLCHECK(HcclGetRootInfo(&rootInfo));
    std::vector<std::thread> threads;
    for (uint32_t r = 0; r < nRanks; ++r) {
        threads.emplace_back(RankMain, nRanks, &rootInfo, r, count);
    }
    for (std::thread& t : threads) {
        t.join();
    }
    if (g_failures.load() != 0) {
        printf("FAIL: %d mismatches\n", g_failures.load());
        return 1;
    }
    printf("PASS: %u ranks x %llu elements: allreduce reducescatter allgather alltoall broadcast\n", nRanks,
           (unsigned long long)count);
    return 0;
}
