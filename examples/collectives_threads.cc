// One host thread per rank, like the reference's examples/02_collectives (01_allreduce/main.cc:46-124 and its
// siblings): every thread joins the world with HcclCommInitRootInfo, owns a stream and two device buffers, and
// issues blocking collectives.  The N "devices" of the reference are N ranks of a loopback world on the one GPU.
// Runs the thirteen operators of the reference's examples/01_point_to_point and examples/02_collectives (AllReduce,
// Broadcast, AllGather, ReduceScatter, Reduce, AlltoAll, AlltoAllV, AlltoAllVC, Scatter, AllGatherV, ReduceScatterV,
// Send / Recv, BatchSendRecv) on closed-form inputs and checks every element; prints PASS and exits 0 when all ranks
// agree.
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

    // The broadcast overwrote the first `count` elements of every send buffer: restore the inputs.
    HIPCHECK(hipMemcpyAsync(send, host.data(), big * sizeof(float), hipMemcpyHostToDevice, stream));

    // Reduce to rank 0: only the root's receive buffer changes
    HCCLCHECK(HcclReduce(send, recv, count, HCCL_DATA_TYPE_FP32, HCCL_REDUCE_SUM, 0, comm, stream));
    HIPCHECK(hipMemcpyAsync(out.data(), recv, count * sizeof(float), hipMemcpyDeviceToHost, stream));
    HIPCHECK(hipStreamSynchronize(stream));
    for (uint64_t i = 0; rank == 0 && i < count; ++i) {
        float want = 0;
        for (uint32_t r = 0; r < nRanks; ++r) want += Input(r, i);
        Expect(out[i] == want, rank, "reduce", i, out[i], want);
    }

    // Scatter from rank 1 (rank 0 in a world of one): rank k receives block k of the root's send buffer
    const uint32_t scatterRoot = nRanks > 1 ? 1 : 0;
    HCCLCHECK(HcclScatter(send, recv, count, HCCL_DATA_TYPE_FP32, scatterRoot, comm, stream));
    HIPCHECK(hipMemcpyAsync(out.data(), recv, count * sizeof(float), hipMemcpyDeviceToHost, stream));
    HIPCHECK(hipStreamSynchronize(stream));
    for (uint64_t i = 0; i < count; ++i) {
        const float want = Input(scatterRoot, rank * count + i);
        Expect(out[i] == want, rank, "scatter", i, out[i], want);
    }

    // The V operators: rank r contributes vCount(r) elements, slices packed back to back.
    auto vCount = [&](uint32_t r) { return count - (r % 2) * (count / 2); };
    std::vector<uint64_t> counts(nRanks), displs(nRanks);
    uint64_t packed = 0;
    for (uint32_t r = 0; r < nRanks; ++r) {
        counts[r] = vCount(r);
        displs[r] = packed;
        packed += counts[r];
    }
    HCCLCHECK(HcclAllGatherV(send, counts[rank], recv, counts.data(), displs.data(), HCCL_DATA_TYPE_FP32, comm, stream));
    HIPCHECK(hipMemcpyAsync(out.data(), recv, packed * sizeof(float), hipMemcpyDeviceToHost, stream));
    HIPCHECK(hipStreamSynchronize(stream));
    for (uint32_t r = 0; r < nRanks; ++r) {
        for (uint64_t i = 0; i < counts[r]; ++i) {
            Expect(out[displs[r] + i] == Input(r, i), rank, "allgatherv", displs[r] + i, out[displs[r] + i], Input(r, i));
        }
    }
    HCCLCHECK(HcclReduceScatterV(send, counts.data(), displs.data(), recv, counts[rank], HCCL_DATA_TYPE_FP32,
                                 HCCL_REDUCE_SUM, comm, stream));
    HIPCHECK(hipMemcpyAsync(out.data(), recv, counts[rank] * sizeof(float), hipMemcpyDeviceToHost, stream));
    HIPCHECK(hipStreamSynchronize(stream));
    for (uint64_t i = 0; i < counts[rank]; ++i) {
        float want = 0;
        for (uint32_t r = 0; r < nRanks; ++r) want += Input(r, displs[rank] + i);
        Expect(out[i] == want, rank, "reducescatterv", i, out[i], want);
    }

    // AlltoAllV: ranks i and j trade pairCount(i, j) elements, blocks at multiples of `count` on both sides
    auto pairCount = [&](uint32_t i, uint32_t j) { return count - ((i + j) % 2) * (count / 2); };
    std::vector<uint64_t> sendCounts(nRanks), blockAt(nRanks);
    for (uint32_t j = 0; j < nRanks; ++j) {
        sendCounts[j] = pairCount(rank, j);
        blockAt[j] = j * count;
    }
    HCCLCHECK(HcclAlltoAllV(send, sendCounts.data(), blockAt.data(), HCCL_DATA_TYPE_FP32, recv, sendCounts.data(),
                            blockAt.data(), HCCL_DATA_TYPE_FP32, comm, stream));
    HIPCHECK(hipMemcpyAsync(out.data(), recv, big * sizeof(float), hipMemcpyDeviceToHost, stream));
    HIPCHECK(hipStreamSynchronize(stream));
    for (uint32_t j = 0; j < nRanks; ++j) {
        for (uint64_t i = 0; i < sendCounts[j]; ++i) {
            const float want = Input(j, rank * count + i);
            Expect(out[j * count + i] == want, rank, "alltoallv", j * count + i, out[j * count + i], want);
        }
    }

    // AlltoAllVC: the same amounts as one matrix every rank passes; segments packed back to back on both sides
    std::vector<uint64_t> matrix(static_cast<size_t>(nRanks) * nRanks);
    for (uint32_t i = 0; i < nRanks; ++i) {
        for (uint32_t j = 0; j < nRanks; ++j) {
            matrix[static_cast<size_t>(i) * nRanks + j] = pairCount(i, j);
        }
    }
    HCCLCHECK(HcclAlltoAllVC(send, matrix.data(), HCCL_DATA_TYPE_FP32, recv, HCCL_DATA_TYPE_FP32, comm, stream));
    HIPCHECK(hipMemcpyAsync(out.data(), recv, big * sizeof(float), hipMemcpyDeviceToHost, stream));
    HIPCHECK(hipStreamSynchronize(stream));
    uint64_t recvAt = 0;
    for (uint32_t j = 0; j < nRanks; ++j) {
        uint64_t sentAt = 0;   // where rank j's segment for this rank starts in j's send buffer
        for (uint32_t k = 0; k < rank; ++k) sentAt += pairCount(j, k);
        for (uint64_t i = 0; i < pairCount(j, rank); ++i) {
            const float want = Input(j, sentAt + i);
            Expect(out[recvAt + i] == want, rank, "alltoallvc", recvAt + i, out[recvAt + i], want);
        }
        recvAt += pairCount(j, rank);
    }

    if (nRanks > 1) {
        // Send / Recv in pairs (0, 1), (2, 3), ...: the even rank sends first, then the roles swap
        const uint32_t mate = rank % 2 == 0 ? rank + 1 : rank - 1;
        if (mate < nRanks) {
            if (rank % 2 == 0) {
                HCCLCHECK(HcclSend(send, count, HCCL_DATA_TYPE_FP32, mate, comm, stream));
                HCCLCHECK(HcclRecv(recv, count, HCCL_DATA_TYPE_FP32, mate, comm, stream));
            } else {
                HCCLCHECK(HcclRecv(recv, count, HCCL_DATA_TYPE_FP32, mate, comm, stream));
                HCCLCHECK(HcclSend(send, count, HCCL_DATA_TYPE_FP32, mate, comm, stream));
            }
            HIPCHECK(hipMemcpyAsync(out.data(), recv, count * sizeof(float), hipMemcpyDeviceToHost, stream));
            HIPCHECK(hipStreamSynchronize(stream));
            for (uint64_t i = 0; i < count; ++i) {
                Expect(out[i] == Input(mate, i), rank, "send/recv", i, out[i], Input(mate, i));
            }
        }
        // BatchSendRecv around the ring: to the next rank, from the previous one
        const uint32_t next = (rank + 1) % nRanks;
        const uint32_t prev = (rank + nRanks - 1) % nRanks;
        HcclSendRecvItem items[2] = {{HCCL_SEND, send, count, HCCL_DATA_TYPE_FP32, next},
                                     {HCCL_RECV, recv, count, HCCL_DATA_TYPE_FP32, prev}};
        HCCLCHECK(HcclBatchSendRecv(items, 2, comm, stream));
        HIPCHECK(hipMemcpyAsync(out.data(), recv, count * sizeof(float), hipMemcpyDeviceToHost, stream));
        HIPCHECK(hipStreamSynchronize(stream));
        for (uint64_t i = 0; i < count; ++i) {
            Expect(out[i] == Input(prev, i), rank, "batchsendrecv", i, out[i], Input(prev, i));
        }
    }

    // Destroying one rank ends the world for all of them: nobody leaves before everybody is through.
    HCCLCHECK(HcclBarrier(comm, stream));
    HIPCHECK(hipStreamSynchronize(stream));
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
    printf("PASS: %u ranks x %llu elements: allreduce reducescatter allgather alltoall broadcast reduce scatter allgatherv "
           "reducescatterv alltoallv alltoallvc send/recv batchsendrecv\n", nRanks, (unsigned long long)count);
    return 0;
}
