// Stress of the host layer (rendezvous, groups, point-to-point queues, destroy) under ThreadSanitizer, linked against
// the CPU emulation build of the library: test infrastructure only.
//
// Two worlds at once, one host thread per rank, a few hundred blocking collectives per rank with closed-form
// answers, point-to-point rings in alternating order, a single thread that drives a third world through groups,
// and a world in which one rank leaves early while its peers are parked in a collective.  Prints PASS and exits 0
// when every answer is right and every call returned what it should.
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <thread>
#include <vector>

#include "hccl.h"

namespace {

std::atomic<int> g_failures{0};
hipStream_t const kStream = reinterpret_cast<hipStream_t>(0x1000);   // the emulation runs every launch to completion

void Fail(const char* what, uint32_t world, uint32_t rank, int iteration, int code)
{
    if (g_failures.fetch_add(1) < 10) {
        fprintf(stderr, "world %u rank %u iteration %d: %s (code %d)\n", world, rank, iteration, what, code);
    }
}

void RankMain(uint32_t world, uint32_t n, const HcclRootInfo* info, uint32_t rank, int iterations, uint64_t count)
{
    HcclComm comm;
    if (HcclCommInitRootInfo(n, info, rank, &comm) != HCCL_SUCCESS) {
        Fail("init", world, rank, -1, 0);
        return;
    }
    std::vector<float> x(count, static_cast<float>(rank + 1)), y(count, 0.0f), g(count * n, 0.0f), s(count / n, 0.0f);
    std::vector<float> inbox(count, 0.0f);
    const float total = static_cast<float>(n * (n + 1) / 2);
    for (int it = 0; it < iterations; ++it) {
        HcclResult rc = HCCL_SUCCESS;
        switch (it % 6) {
            case 0:
                rc = HcclAllReduce(x.data(), y.data(), count, HCCL_DATA_TYPE_FP32, HCCL_REDUCE_SUM, comm, kStream);
                if (rc == HCCL_SUCCESS && (y[0] != total || y[count - 1] != total)) Fail("all_reduce value", world, rank, it, 0);
                break;
            case 1:
                rc = HcclAllGather(x.data(), g.data(), count, HCCL_DATA_TYPE_FP32, comm, kStream);
                for (uint32_t r = 0; rc == HCCL_SUCCESS && r < n; ++r) {
                    if (g[r * count] != static_cast<float>(r + 1)) Fail("all_gather value", world, rank, it, 0);
                }
                break;
            case 2:
                rc = HcclReduceScatter(x.data(), s.data(), count / n, HCCL_DATA_TYPE_FP32, HCCL_REDUCE_SUM, comm, kStream);
                if (rc == HCCL_SUCCESS && s[0] != total) Fail("reduce_scatter value", world, rank, it, 0);
                break;
            case 3:
                y[0] = static_cast<float>(rank == static_cast<uint32_t>(it) % n ? 77 : 0);
                rc = HcclBroadcast(y.data(), 1, HCCL_DATA_TYPE_FP32, static_cast<uint32_t>(it) % n, comm, kStream);
                if (rc == HCCL_SUCCESS && y[0] != 77.0f) Fail("broadcast value", world, rank, it, 0);
                break;
            case 4: {   // a ring of blocking sends and receives: even ranks send first (n is even where this runs)
                if (n % 2 != 0) break;
                const uint32_t nxt = (rank + 1) % n, prv = (rank + n - 1) % n;
                if (rank % 2 == 0) {
                    rc = HcclSend(x.data(), count, HCCL_DATA_TYPE_FP32, nxt, comm, kStream);
                    if (rc == HCCL_SUCCESS) rc = HcclRecv(inbox.data(), count, HCCL_DATA_TYPE_FP32, prv, comm, kStream);
                } else {
                    rc = HcclRecv(inbox.data(), count, HCCL_DATA_TYPE_FP32, prv, comm, kStream);
                    if (rc == HCCL_SUCCESS) rc = HcclSend(x.data(), count, HCCL_DATA_TYPE_FP32, nxt, comm, kStream);
                }
                if (rc == HCCL_SUCCESS && inbox[count / 2] != static_cast<float>(prv + 1)) Fail("ring value", world, rank, it, 0);
                break;
            }
            default: {  // the same ring as one batch per rank
                const uint32_t nxt = (rank + 1) % n, prv = (rank + n - 1) % n;
                HcclSendRecvItem items[2] = {{HCCL_SEND, x.data(), count, HCCL_DATA_TYPE_FP32, nxt},
                                             {HCCL_RECV, inbox.data(), count, HCCL_DATA_TYPE_FP32, prv}};
                inbox[0] = 0.0f;
                rc = HcclBatchSendRecv(items, 2, comm, kStream);
                if (rc == HCCL_SUCCESS && inbox[0] != static_cast<float>(prv + 1)) Fail("batch value", world, rank, it, 0);
                break;
            }
        }
        if (rc != HCCL_SUCCESS) {
            Fail("call failed", world, rank, it, rc);
            break;
        }
    }
    // Nobody destroys before everybody is through: destroying one rank ends the world.
    if (HcclBarrier(comm, kStream) != HCCL_SUCCESS) Fail("barrier", world, rank, iterations, 0);
    if (HcclCommDestroy(comm) != HCCL_SUCCESS) Fail("destroy", world, rank, iterations, 0);
}

// One thread, all ranks, groups.
void GroupedWorld(uint32_t n, int iterations, uint64_t count)
{
    std::vector<HcclComm> comms(n);
    if (HcclCommInitAll(n, nullptr, comms.data()) != HCCL_SUCCESS) {
        Fail("init all", 9, 0, -1, 0);
        return;
    }
    std::vector<std::vector<int32_t>> in(n, std::vector<int32_t>(count)), out(n, std::vector<int32_t>(count));
    for (uint32_t r = 0; r < n; ++r) {
        for (uint64_t i = 0; i < count; ++i) in[r][i] = static_cast<int32_t>(r * 1000 + i);
    }
    for (int it = 0; it < iterations; ++it) {
        HcclGroupStart();
        for (uint32_t r = 0; r < n; ++r) {
            HcclResult rc = HcclAllReduce(in[r].data(), out[r].data(), count, HCCL_DATA_TYPE_INT32, HCCL_REDUCE_MAX, comms[r], kStream);
            if (rc != HCCL_SUCCESS) Fail("grouped all_reduce", 9, r, it, rc);
        }
        HcclResult end = HcclGroupEnd();
        if (end != HCCL_SUCCESS) Fail("group end", 9, 0, it, end);
        for (uint32_t r = 0; r < n; ++r) {
            if (out[r][count - 1] != static_cast<int32_t>((n - 1) * 1000 + count - 1)) Fail("grouped value", 9, r, it, 0);
        }
    }
    for (HcclComm c : comms) HcclCommDestroy(c);
}

// Rank 2 never joins the collective and destroys instead: ranks 0 and 1 must come back with HCCL_E_UNAVAIL, and
// what they call afterwards must be refused at once.
void WorldWithALeaver()
{
    constexpr uint32_t n = 3;
    HcclRootInfo info;
    HcclGetRootInfo(&info);
    std::atomic<int> parked{0};
    auto stay = [&](uint32_t rank) {
        HcclComm comm;
        HcclCommInitRootInfo(n, &info, rank, &comm);
        float v = 1.0f, w = 0.0f;
        parked.fetch_add(1);
        HcclResult rc = HcclAllReduce(&v, &w, 1, HCCL_DATA_TYPE_FP32, HCCL_REDUCE_SUM, comm, kStream);
        if (rc != HCCL_E_UNAVAIL) Fail("parked rank was not released with HCCL_E_UNAVAIL", 7, rank, 0, rc);
        rc = HcclSend(&v, 1, HCCL_DATA_TYPE_FP32, (rank + 1) % 2, comm, kStream);
        if (rc != HCCL_E_UNAVAIL) Fail("send after a peer left", 7, rank, 1, rc);
        HcclCommDestroy(comm);
    };
    std::thread a(stay, 0u), b(stay, 1u);
    HcclComm comm;
    HcclCommInitRootInfo(n, &info, 2, &comm);
    while (parked.load() < 2) std::this_thread::yield();
    std::this_thread::sleep_for(std::chrono::milliseconds(50));
    HcclCommDestroy(comm);
    a.join();
    b.join();
}

}  // namespace

int main(int argc, char** argv)
{
    const int iterations = argc > 1 ? atoi(argv[1]) : 240;
    std::vector<std::thread> threads;
    HcclRootInfo infoA, infoB;
    HcclGetRootInfo(&infoA);
    HcclGetRootInfo(&infoB);
    for (uint32_t r = 0; r < 8; ++r) threads.emplace_back(RankMain, 0u, 8u, &infoA, r, iterations, uint64_t(8 * 128));
    for (uint32_t r = 0; r < 3; ++r) threads.emplace_back(RankMain, 1u, 3u, &infoB, r, iterations, uint64_t(3 * 500));
    threads.emplace_back(GroupedWorld, 5u, iterations / 4, uint64_t(1000));
    threads.emplace_back(WorldWithALeaver);
    for (std::thread& t : threads) t.join();
    if (g_failures.load() != 0) {
        fprintf(stderr, "FAIL: %d failures\n", g_failures.load());
        return 1;
    }
    printf("PASS: %d iterations per rank in two threaded worlds, a grouped world and a world with a leaver\n", iterations);
    return 0;
}
