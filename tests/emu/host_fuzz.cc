// Randomised sequences of collectives with deliberate faults, against the CPU emulation build of the library under
// ThreadSanitizer / AddressSanitizer: test infrastructure only.
//
// A seeded script of steps is shared by the ranks of a world (one host thread per rank, blocking calls).  A step is a
// collective (the V operators among them, with counts and displacements that change from step to step); in some
// steps one rank passes a count (for a V operator: a count table) that differs from its peers', a null buffer, a data
// type the operator does not take, or a zero count together with everybody else.  What must hold whatever the interleaving:
// every rank gets the same return code for the step (success, or the code of the fault), the results of the clean
// steps are right, the calls after a fault pair up as if nothing had happened, and nothing hangs.  Prints PASS.
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
hipStream_t const kStream = reinterpret_cast<hipStream_t>(0x1000);

enum Fault { kNone, kWrongCount, kNullBuffer, kBadType, kZeroCount, kFaults };
enum Op { kAllReduce, kAllGather, kReduceScatter, kBroadcast, kReduce, kBarrier, kAllGatherV, kReduceScatterV, kAlltoAllV, kOps };

struct Step {
    Op op;
    Fault fault;
    uint32_t who;    // the rank that misbehaves
    uint32_t root;
    uint64_t count;
};

uint64_t Next(uint64_t& s)
{
    s = s * 6364136223846793005ull + 1442695040888963407ull;
    return s >> 33;
}

std::vector<Step> Script(uint64_t seed, uint32_t n, int steps)
{
    std::vector<Step> script;
    uint64_t s = seed;
    for (int i = 0; i < steps; ++i) {
        Step st;
        st.op = static_cast<Op>(Next(s) % kOps);
        st.fault = (Next(s) % 3 == 0) ? static_cast<Fault>(1 + Next(s) % (kFaults - 1)) : kNone;
        st.who = static_cast<uint32_t>(Next(s) % n);
        st.root = static_cast<uint32_t>(Next(s) % n);
        st.count = 1 + Next(s) % 700;
        if (st.op == kBarrier) {
            st.fault = kNone;
        }
        script.push_back(st);
    }
    return script;
}

void Fail(const char* what, uint32_t rank, int step, int got, int want)
{
    if (g_failures.fetch_add(1) < 12) {
        fprintf(stderr, "rank %u step %d: %s (got %d, want %d)\n", rank, step, what, got, want);
    }
}

void RankMain(uint32_t n, const HcclRootInfo* info, uint32_t rank, const std::vector<Step>* script)
{
    HcclComm comm;
    if (HcclCommInitRootInfo(n, info, rank, &comm) != HCCL_SUCCESS) {
        Fail("init", rank, -1, 0, 0);
        return;
    }
    const uint64_t cap = 701 * n;
    std::vector<int32_t> in(cap), out(cap);
    for (size_t k = 0; k < script->size(); ++k) {
        const Step& st = (*script)[k];
        const bool bad = st.fault != kNone && st.fault != kZeroCount && st.who == rank;
        uint64_t count = st.fault == kZeroCount ? 0 : st.count;
        if (bad && st.fault == kWrongCount) {
            count += 1;
        }
        const HcclDataType dtype = (bad && st.fault == kBadType) ? HCCL_DATA_TYPE_RESERVED : HCCL_DATA_TYPE_INT32;
        void* send = (bad && st.fault == kNullBuffer) ? nullptr : in.data();
        for (uint64_t i = 0; i < cap; ++i) {
            in[i] = static_cast<int32_t>(rank * 100000 + k * 7 + i);
            out[i] = -1;
        }
        // V operators: rank r contributes / receives vcount(r) elements, slices packed back to back; AlltoAllV trades
        // pair(i, j) elements between ranks i and j in blocks of st.count.
        auto vcount = [&](uint32_t r) { return (st.count + r * 13) % 97 + 1; };
        auto pair = [&](uint32_t i, uint32_t j) { return (st.count + (i + j) * 7) % (st.count + 1); };
        std::vector<uint64_t> counts(n), displs(n), sendCounts(n), blockAt(n);
        uint64_t packed = 0;
        for (uint32_t r = 0; r < n; ++r) {
            counts[r] = vcount(r);
            displs[r] = packed;
            packed += counts[r];
            sendCounts[r] = pair(rank, r);
            blockAt[r] = r * (st.count + 1);
        }
        const bool isV = st.op == kAllGatherV || st.op == kReduceScatterV || st.op == kAlltoAllV;
        if (isV && st.fault == kZeroCount) {
            continue;   // the V operators have no single count to zero
        }
        if (isV && bad && st.fault == kWrongCount) {
            counts[(rank + 1) % n] += 1;        // a table that differs from the peers'
            sendCounts[(rank + 1) % n] += 1;    // an amount the receiver does not expect
            if (n == 1) {
                continue;
            }
        }
        HcclResult rc = HCCL_SUCCESS;
        switch (st.op) {
            case kAllGatherV:
                rc = HcclAllGatherV(send, vcount(rank), out.data(), counts.data(), displs.data(), dtype, comm, kStream);
                break;
            case kReduceScatterV:
                rc = HcclReduceScatterV(send, counts.data(), displs.data(), out.data(), vcount(rank), dtype, HCCL_REDUCE_MAX, comm, kStream);
                break;
            case kAlltoAllV: {
                std::vector<uint64_t> recvCounts(n);
                for (uint32_t r = 0; r < n; ++r) recvCounts[r] = pair(r, rank);
                rc = HcclAlltoAllV(send, sendCounts.data(), blockAt.data(), dtype, out.data(), recvCounts.data(), blockAt.data(), dtype, comm, kStream);
                break;
            }
            case kAllReduce: rc = HcclAllReduce(send, out.data(), count, dtype, HCCL_REDUCE_MAX, comm, kStream); break;
            case kAllGather: rc = HcclAllGather(send, out.data(), count, dtype, comm, kStream); break;
            case kReduceScatter: rc = HcclReduceScatter(send, out.data(), count, dtype, HCCL_REDUCE_MAX, comm, kStream); break;
            case kBroadcast: rc = HcclBroadcast(send, count, dtype, st.root, comm, kStream); break;
            case kReduce: rc = HcclReduce(send, out.data(), count, dtype, HCCL_REDUCE_MAX, st.root, comm, kStream); break;
            default: rc = HcclBarrier(comm, kStream); break;
        }
        HcclResult want = HCCL_SUCCESS;
        if (st.fault == kWrongCount) want = HCCL_E_PARA;
        if (st.fault == kNullBuffer) want = HCCL_E_PTR;
        if (st.fault == kBadType) want = HCCL_E_NOT_SUPPORT;
        if (rc != want) {
            Fail("return code", rank, static_cast<int>(k), rc, want);
            continue;
        }
        if (want != HCCL_SUCCESS || count == 0) {
            continue;
        }
        // the maximum over ranks is the last rank's value
        const int32_t top = static_cast<int32_t>((n - 1) * 100000 + k * 7);
        switch (st.op) {
            case kAllReduce:
                if (out[0] != top || out[count - 1] != top + static_cast<int32_t>(count - 1)) Fail("all_reduce value", rank, static_cast<int>(k), out[0], top);
                break;
            case kAllGather:
                for (uint32_t r = 0; r < n; ++r) {
                    const int32_t v = static_cast<int32_t>(r * 100000 + k * 7);
                    if (out[r * count] != v) Fail("all_gather value", rank, static_cast<int>(k), out[r * count], v);
                }
                break;
            case kReduceScatter:
                if (out[0] != top + static_cast<int32_t>(rank * count)) Fail("reduce_scatter value", rank, static_cast<int>(k), out[0], top);
                break;
            case kBroadcast: {
                const int32_t v = static_cast<int32_t>(st.root * 100000 + k * 7);
                if (in[0] != v || in[count - 1] != v + static_cast<int32_t>(count - 1)) Fail("broadcast value", rank, static_cast<int>(k), in[0], v);
                break;
            }
            case kReduce:
                if (rank == st.root && out[0] != top) Fail("reduce value", rank, static_cast<int>(k), out[0], top);
                break;
            case kAllGatherV:
                for (uint32_t r = 0; r < n; ++r) {
                    const int32_t v = static_cast<int32_t>(r * 100000 + k * 7 + counts[r] - 1);
                    if (out[displs[r] + counts[r] - 1] != v) Fail("all_gather_v value", rank, static_cast<int>(k), out[displs[r] + counts[r] - 1], v);
                }
                break;
            case kReduceScatterV:
                if (out[0] != top + static_cast<int32_t>(displs[rank])) Fail("reduce_scatter_v value", rank, static_cast<int>(k), out[0], top);
                break;
            case kAlltoAllV:
                for (uint32_t r = 0; r < n; ++r) {
                    if (pair(r, rank) == 0) continue;
                    const int32_t v = static_cast<int32_t>(r * 100000 + k * 7 + rank * (st.count + 1));
                    if (out[r * (st.count + 1)] != v) Fail("all_to_all_v value", rank, static_cast<int>(k), out[r * (st.count + 1)], v);
                }
                break;
            default: break;
        }
    }
    if (HcclBarrier(comm, kStream) != HCCL_SUCCESS) Fail("closing barrier", rank, -1, 0, 0);
    HcclCommDestroy(comm);
}

// The same script driven by one thread through groups: the calls queue, HcclGroupEnd reports the worst result.
void Grouped(uint32_t n, const std::vector<Step>& script)
{
    std::vector<HcclComm> comms(n);
    HcclCommInitAll(n, nullptr, comms.data());
    const uint64_t cap = 701 * n;
    std::vector<std::vector<int32_t>> in(n, std::vector<int32_t>(cap)), out(n, std::vector<int32_t>(cap));
    for (size_t k = 0; k < script.size(); ++k) {
        const Step& st = script[k];
        if (st.op == kBroadcast || st.op >= kBarrier || st.fault == kZeroCount) {
            continue;
        }
        for (uint32_t r = 0; r < n; ++r) {
            for (uint64_t i = 0; i < cap; ++i) in[r][i] = static_cast<int32_t>(r * 100000 + k * 7 + i);
        }
        HcclResult want = HCCL_SUCCESS;
        if (st.fault == kWrongCount) want = HCCL_E_PARA;
        if (st.fault == kNullBuffer) want = HCCL_E_PTR;
        if (st.fault == kBadType) want = HCCL_E_NOT_SUPPORT;
        HcclGroupStart();
        HcclResult worstCall = HCCL_SUCCESS;
        for (uint32_t r = 0; r < n; ++r) {
            const bool bad = st.fault != kNone && st.who == r;
            const uint64_t count = st.count + ((bad && st.fault == kWrongCount) ? 1 : 0);
            const HcclDataType dtype = (bad && st.fault == kBadType) ? HCCL_DATA_TYPE_RESERVED : HCCL_DATA_TYPE_INT32;
            void* send = (bad && st.fault == kNullBuffer) ? nullptr : in[r].data();
            HcclResult rc;
            switch (st.op) {
                case kAllReduce: rc = HcclAllReduce(send, out[r].data(), count, dtype, HCCL_REDUCE_MAX, comms[r], kStream); break;
                case kAllGather: rc = HcclAllGather(send, out[r].data(), count, dtype, comms[r], kStream); break;
                case kReduceScatter: rc = HcclReduceScatter(send, out[r].data(), count, dtype, HCCL_REDUCE_MAX, comms[r], kStream); break;
                default: rc = HcclReduce(send, out[r].data(), count, dtype, HCCL_REDUCE_MAX, st.root, comms[r], kStream); break;
            }
            if (rc != HCCL_SUCCESS) {
                worstCall = rc;
            }
        }
        const HcclResult end = HcclGroupEnd();
        const HcclResult seen = end != HCCL_SUCCESS ? end : worstCall;
        if (seen != want) {
            Fail("grouped step", 0, static_cast<int>(k), seen, want);
        } else if (want == HCCL_SUCCESS && st.op == kAllReduce) {
            const int32_t top = static_cast<int32_t>((n - 1) * 100000 + k * 7);
            for (uint32_t r = 0; r < n; ++r) {
                if (out[r][0] != top) Fail("grouped all_reduce value", r, static_cast<int>(k), out[r][0], top);
            }
        }
    }
    for (HcclComm c : comms) HcclCommDestroy(c);
}

}  // namespace

int main(int argc, char** argv)
{
    const uint64_t seed = argc > 1 ? strtoull(argv[1], nullptr, 0) : 1;
    const int steps = argc > 2 ? atoi(argv[2]) : 400;
    std::vector<std::thread> threads;
    HcclRootInfo infoA, infoB;
    HcclGetRootInfo(&infoA);
    HcclGetRootInfo(&infoB);
    const std::vector<Step> scriptA = Script(seed, 5, steps), scriptB = Script(seed + 17, 2, steps), scriptC = Script(seed + 99, 4, steps);
    for (uint32_t r = 0; r < 5; ++r) threads.emplace_back(RankMain, 5u, &infoA, r, &scriptA);
    for (uint32_t r = 0; r < 2; ++r) threads.emplace_back(RankMain, 2u, &infoB, r, &scriptB);
    threads.emplace_back([&] { Grouped(4, scriptC); });
    for (std::thread& t : threads) t.join();
    if (g_failures.load() != 0) {
        fprintf(stderr, "FAIL: %d failures (seed %llu)\n", g_failures.load(), (unsigned long long)seed);
        return 1;
    }
    printf("PASS: seed %llu, %d steps per world\n", (unsigned long long)seed, steps);
    return 0;
}
