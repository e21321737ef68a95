// Host layer, part 3: what a copy collective launches (AllGather(V), Broadcast, AlltoAll(V / VC), Scatter, the
// single-rank shortcut), and the tables of the descriptor-driven copy kernel.
#include <algorithm>
#include <cctype>
#include <chrono>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "algo_config.h"
#include "host.h"
#include "launch_policy.h"

namespace hccl_amd {

// Bytes of one slot: the tables of a world whose n * n segments are all non-empty.
size_t A2aSlotBytes(uint32_t n)
{
    return A2aTableBytes(static_cast<size_t>(n) * n);
}

// Calls may be in flight on different streams, so each of the kStagingSlots calls owns its own host
// staging area and device tables until the event recorded behind its copy kernel has fired.
HcclResult EnsureA2aBuffers(World* w)
{
    if (w->a2aDev != nullptr) {
        return HCCL_SUCCESS;
    }
    HIP_OK(hipMalloc(reinterpret_cast<void**>(&w->a2aDev), kStagingSlots * A2aSlotBytes(w->n)));
    for (int s = 0; s < kStagingSlots; ++s) {
        HIP_OK(hipHostMalloc(reinterpret_cast<void**>(&w->a2aHost[s]), A2aSlotBytes(w->n), hipHostMallocDefault));
        HIP_OK(hipEventCreateWithFlags(&w->a2aSlotFree[s], hipEventDisableTiming));
    }
    return HCCL_SUCCESS;
}

// Every world and stream of a GPU shares that GPU's table array.  Its users are put in order: one at a time on
// the host (the mutex is held from the wait to the record), and on the device each call's table writes wait for
// the event recorded behind the copy kernel of the call before it, whichever world or stream that was on.  The
// event is created with the first allocation-free call on the device; waiting and recording allocate nothing.
struct ScratchUsers {
    std::mutex mu;
    hipEvent_t lastUse = nullptr;
    bool used = false;
};
constexpr int kScratchDevices = 64;
ScratchUsers g_scratchUsers[kScratchDevices];

// Set-up of the allocation-free entry point, on its first call in a world (the world's device is current):
// the address of the device-resident table array, and the events a launch over several streams takes from
// the pool, so that later calls create nothing.
HcclResult PrepareNoAlloc(World* w)
{
    if (w->a2aScratch != nullptr) {
        return HCCL_SUCCESS;
    }
    if (w->device < 0 || w->device >= kScratchDevices) {
        return HCCL_E_NOT_SUPPORT;
    }
    {
        ScratchUsers& users = g_scratchUsers[w->device];
        std::lock_guard<std::mutex> lock(users.mu);
        if (users.lastUse == nullptr) {
            HIP_OK(hipEventCreateWithFlags(&users.lastUse, hipEventDisableTiming));
        }
    }
    uint8_t* ptr = nullptr;
    HIP_OK(A2aScratchOfCurrentDevice(&ptr));
    while (w->eventPool.size() < w->n) {
        hipEvent_t ev;
        HIP_OK(hipEventCreateWithFlags(&ev, hipEventDisableTiming));
        w->eventPool.push_back(ev);
    }
    if (w->doneEvent == nullptr) {
        HIP_OK(hipEventCreateWithFlags(&w->doneEvent, hipEventDisableTiming));
    }
    w->a2aImage.assign(kA2aScratchBytes / sizeof(uint64_t), 0);
    w->a2aScratch = ptr;
    return HCCL_SUCCESS;
}

HcclResult RunBcast(World* w, BcastCopyArgs& b, hipStream_t s)
{
    HIP_OK(LaunchBcastCopy(b, w->copyTileBytes, s));   // 0: the launcher picks
    return HCCL_SUCCESS;
}

// One-to-many copy as two kernels per window of at most pieceBytes of every destination: the segments into the first
// destination (one read and one write stream each, the fastest copy there is), then that range, still cached, to
// the other destinations with one wavefront per destination.  A wavefront that stores to many streams one after
// the other is what bounds the one-kernel form.  Taken when the destinations share their offset from a 16-byte
// boundary and the segments' destination ranges do not overlap; runs of adjacent ranges fan out in one launch.
// `bytes` is what every destination receives (launch_policy.h has the measurements).
bool GatherThenFanOut(const World* w, uint32_t nDst, uint64_t bytes, bool congruent)
{
    if (nDst < 3) {
        return false;
    }
    if (w->copyTwoKernelMode != 2) {
        return w->copyTwoKernelMode == 1;
    }
    return policy::GatherThenFanOut(nDst, bytes, congruent);
}

HcclResult RunOneToMany(World* w, BcastCopyArgs& b, hipStream_t s)
{
    uint64_t total = 0;
    std::vector<uint32_t> order;
    for (uint32_t j = 0; j < b.nSeg; ++j) {
        if (b.len[j] != 0) {
            total += b.len[j];
            order.push_back(j);
        }
    }
    bool congruent = true;   // every source shares the offset of its place in the first destination from a 16-byte boundary
    for (uint32_t j : order) {
        congruent = congruent && ((reinterpret_cast<uint64_t>(b.src[j]) ^
                                   (reinterpret_cast<uint64_t>(b.dst[0]) + b.dstOff[j])) & 15u) == 0;
    }
    bool dstCongruent = true;
    for (uint32_t d = 1; d < b.nDst; ++d) {
        dstCongruent = dstCongruent &&
                       ((reinterpret_cast<uint64_t>(b.dst[d]) ^ reinterpret_cast<uint64_t>(b.dst[0])) & 15u) == 0;
    }
    if (!GatherThenFanOut(w, b.nDst, total, congruent)) {
        return RunBcast(w, b, s);
    }
    if (!dstCongruent) {
        return RunBcast(w, b, s);
    }
    std::sort(order.begin(), order.end(), [&](uint32_t x, uint32_t y) { return b.dstOff[x] < b.dstOff[y]; });
    for (size_t i = 1; i < order.size(); ++i) {
        if (b.dstOff[order[i - 1]] + b.len[order[i - 1]] > b.dstOff[order[i]]) {
            return RunBcast(w, b, s);
        }
    }
    size_t next = 0;            // first segment with bytes left
    uint64_t consumed = 0;      // bytes of it already copied
    while (next < order.size()) {
        // one window: [begin, begin + pieceBytes) of every destination
        const uint64_t begin = b.dstOff[order[next]] + consumed;
        const uint64_t end = begin + w->pieceBytes;
        BcastCopyArgs g{};
        g.nDst = 1;
        g.dst[0] = b.dst[0];
        struct Run {
            uint64_t off, len;
        };
        std::vector<Run> runs;
        while (next < order.size() && g.nSeg < static_cast<uint32_t>(kMaxRanks)) {
            const uint32_t j = order[next];
            const uint64_t segBegin = b.dstOff[j] + consumed;
            if (segBegin >= end) {
                break;
            }
            const uint64_t len = std::min(b.len[j] - consumed, end - segBegin);
            g.src[g.nSeg] = static_cast<const uint8_t*>(b.src[j]) + consumed;
            g.dstOff[g.nSeg] = segBegin;
            g.len[g.nSeg] = len;
            ++g.nSeg;
            if (!runs.empty() && runs.back().off + runs.back().len == segBegin) {
                runs.back().len += len;
            } else {
                runs.push_back({segBegin, len});
            }
            consumed += len;
            if (consumed == b.len[j]) {
                ++next;
                consumed = 0;
            }
        }
        HcclResult rc = RunBcast(w, g, s);
        if (rc != HCCL_SUCCESS) {
            return rc;
        }
        for (const Run& run : runs) {
            FanOutArgs f{};
            f.src = static_cast<const uint8_t*>(b.dst[0]) + run.off;
            f.bytes = run.len;
            f.nDst = b.nDst - 1;
            for (uint32_t d = 1; d < b.nDst; ++d) {
                f.dst[d - 1] = static_cast<uint8_t*>(b.dst[d]) + run.off;
            }
            // (a copy in front of it, not a fold: a non-temporal load only loses here, AllGather over 16 ranks
            // 0.84 -> 0.81)
            HIP_OK(LaunchFanOut(f, w->fanOutLoadMode != 2 ? w->fanOutLoadMode == 1 : policy::FanOutStreamLoad(f.nDst, false), s));
        }
    }
    return HCCL_SUCCESS;
}

HcclResult RunAllGather(World* w, PendingOp& p, hipStream_t s)
{
    const uint32_t n = w->n;
    const uint64_t esz = DataTypeSize(p.dtype);
    BcastCopyArgs b{};
    b.nSeg = n;
    b.nDst = n;
    for (uint32_t r = 0; r < n; ++r) {
        b.src[r] = p.ranks[r].send;
        b.dst[r] = p.ranks[r].recv;
        b.len[r] = p.count * esz;
        b.dstOff[r] = static_cast<uint64_t>(r) * p.count * esz;   // reference all_gather_mesh_1D.cc:298-380
    }
    return RunOneToMany(w, b, s);
}

HcclResult RunAllGatherV(World* w, PendingOp& p, hipStream_t s)
{
    const uint32_t n = w->n;
    const uint64_t esz = DataTypeSize(p.dtype);
    const std::vector<uint64_t>& ref = p.ranks[0].var;   // counts | displs | sendCount
    for (uint32_t r = 0; r < n; ++r) {
        const std::vector<uint64_t>& v = p.ranks[r].var;
        if (memcmp(v.data(), ref.data(), 2 * n * sizeof(uint64_t)) != 0) {
            Log(1, "AllGatherV: rank %u passed recvCounts / recvDispls that differ from rank 0", r);
            return HCCL_E_PARA;
        }
        if (v[2 * n] != ref[r]) {
            Log(1, "AllGatherV: rank %u sendCount %llu != recvCounts[%u] %llu", r, (unsigned long long)v[2 * n], r,
                (unsigned long long)ref[r]);
            return HCCL_E_PARA;
        }
    }
    BcastCopyArgs b{};
    b.nSeg = n;
    b.nDst = n;
    for (uint32_t r = 0; r < n; ++r) {
        b.src[r] = p.ranks[r].send;
        b.dst[r] = p.ranks[r].recv;
        b.len[r] = ref[r] * esz;
        b.dstOff[r] = ref[n + r] * esz;   // reference all_gather_v_mesh_1D.cc:242-310
    }
    return RunOneToMany(w, b, s);
}

// Copies a list of at most n * n non-empty segments with one launch of the descriptor-driven copy kernel.
// With `noAlloc` the tables travel in kernel arguments to the library's device-resident array instead of
// through a pinned staging slot into allocated device memory.
HcclResult RunSegmentCopy(World* w, const std::vector<CopySeg>& segs, hipStream_t s, bool noAlloc = false)
{
    const uint32_t n = w->n;
    const uint32_t tileBytes = w->copyTileBytes != 0 ? w->copyTileBytes : 1024u;
    const uint32_t nSeg = static_cast<uint32_t>(segs.size());
    if (nSeg == 0) {
        return HCCL_SUCCESS;
    }
    if (nSeg > n * n) {
        return HCCL_E_INTERNAL;
    }
    uint64_t* hDesc;
    uint8_t* dev;
    uint32_t slot = 0;
    if (noAlloc) {
        if (A2aTableBytes(nSeg) > kA2aScratchBytes) {
            Log(1, "the tables of %u segments (%zu bytes) exceed the %zu bytes of the allocation-free entry point", nSeg,
                A2aTableBytes(nSeg), kA2aScratchBytes);
            return HCCL_E_MEMORY;
        }
        hDesc = w->a2aImage.data();
        dev = w->a2aScratch;
    } else {
        HcclResult rc = EnsureA2aBuffers(w);
        if (rc != HCCL_SUCCESS) {
            return rc;
        }
        slot = w->a2aNext;
        w->a2aNext = (w->a2aNext + 1) % kStagingSlots;
        if (w->a2aSlotUsed[slot] && hipEventQuery(w->a2aSlotFree[slot]) != hipSuccess) {
            // The call that last used this slot is still running: wait for it without the world's lock, so that
            // other ranks can keep depositing their calls (launches stay one at a time: launchBusy is set).
            hipEvent_t busy = w->a2aSlotFree[slot];
            if (w->launchLock != nullptr) {
                w->launchLock->unlock();
            }
            const hipError_t waited = hipEventSynchronize(busy);
            if (w->launchLock != nullptr) {
                w->launchLock->lock();
            }
            HIP_OK(waited);
            if (w->destroyed != 0) {
                // A rank left while the lock was released: its HcclCommDestroy has settled this collective for the
                // peers (who may free their buffers now), so nothing of it is enqueued.
                return HCCL_E_UNAVAIL;
            }
        }
        hDesc = w->a2aHost[slot];
        dev = w->a2aDev + slot * A2aSlotBytes(n);
    }
    uint32_t* hEnd = reinterpret_cast<uint32_t*>(hDesc + static_cast<size_t>(kA2aDescWords) * nSeg);
    uint32_t* hHint = hEnd + ((nSeg + 1u) & ~1u);
    uint64_t tiles = 0;
    uint64_t misfit = 0;
    bool congruent = true;
    for (uint32_t k = 0; k < nSeg; ++k) {
        const CopySeg& seg = segs[k];
        uint64_t* d = hDesc + static_cast<size_t>(kA2aDescWords) * k;
        d[0] = seg.src;
        d[1] = seg.dst;
        d[2] = seg.len;
        d[3] = tiles;
        tiles += TilesOf(seg.len, seg.dst, tileBytes);
        if (tiles > 0x7FFFFFF0ull) {
            return HCCL_E_PARA;
        }
        hEnd[k] = static_cast<uint32_t>(tiles);
        misfit |= seg.src | seg.dst | seg.len;
        congruent = congruent && ((seg.src ^ seg.dst) & 15u) == 0;
    }
    A2aArgs a{};
    uint32_t nHint = 0;
    a.hintShift = BuildTileHints(hEnd, nSeg, static_cast<uint32_t>(tiles), kA2aHintMax, hHint, &nHint);
    a.mode = !congruent ? COPY_GENERAL : ((misfit & 15u) == 0 ? COPY_ALIGNED : COPY_CONGRUENT);
    const size_t used = reinterpret_cast<uint8_t*>(hHint + nHint + 1) - reinterpret_cast<uint8_t*>(hDesc);
    a.desc = reinterpret_cast<const uint64_t*>(dev);
    a.tileEnd = reinterpret_cast<const uint32_t*>(a.desc + static_cast<size_t>(kA2aDescWords) * nSeg);
    a.hint = a.tileEnd + ((nSeg + 1u) & ~1u);
    if (noAlloc) {
        // The array's users on this GPU in order: this call's table writes start when the copy kernel of the call
        // before it, of whichever world and on whichever stream, has read its tables.  A stream under capture
        // records launches for later: the replays of a captured call are ordered by whoever launches the graph.
        ScratchUsers& users = g_scratchUsers[w->device];
        std::lock_guard<std::mutex> order(users.mu);
        hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
        HIP_OK(hipStreamIsCapturing(s, &capture));
        const bool eager = capture == hipStreamCaptureStatusNone;
        if (eager && users.used) {
            HIP_OK(hipStreamWaitEvent(s, users.lastUse, 0));
        }
        HIP_OK(LaunchTableWrite(dev, hDesc, static_cast<uint32_t>((used + 7) / 8), s));
        HIP_OK(LaunchA2aCopy(a, static_cast<uint32_t>(tiles), tileBytes, s));
        if (eager) {
            HIP_OK(hipEventRecord(users.lastUse, s));
            users.used = true;
        }
        return HCCL_SUCCESS;
    }
    HIP_OK(hipMemcpyAsync(dev, hDesc, used, hipMemcpyHostToDevice, s));
    HIP_OK(LaunchA2aCopy(a, static_cast<uint32_t>(tiles), tileBytes, s));
    HIP_OK(hipEventRecord(w->a2aSlotFree[slot], s));
    w->a2aSlotUsed[slot] = true;
    return HCCL_SUCCESS;
}

HcclResult RunAlltoAllV(World* w, PendingOp& p, hipStream_t s)
{
    const uint32_t n = w->n;
    const uint64_t esz = DataTypeSize(p.dtype);
    // rank r's var = sendCounts | recvCounts | sdispls | rdispls (reference all_to_all_v.cc:617-643)
    for (uint32_t i = 0; i < n; ++i) {
        for (uint32_t j = 0; j < n; ++j) {
            uint64_t sent = p.ranks[j].var[i];
            uint64_t expected = p.ranks[i].var[n + j];
            if (sent != expected) {
                Log(1, "AlltoAllV: rank %u recvCounts[%u]=%llu but rank %u sendCounts[%u]=%llu", i, j,
                    (unsigned long long)expected, j, i, (unsigned long long)sent);
                return HCCL_E_PARA;
            }
        }
    }
    // One descriptor per non-empty segment, destination-major so that neighbouring tiles write
    // neighbouring addresses: recv_i[rdispls_i[j] ...] = send_j[sdispls_j[i] ...]
    // (reference ins_temp_all_to_all_v_mesh_1D.cc:229-246).
    std::vector<CopySeg>& segs = w->a2aSegs;   // keeps its capacity from call to call
    segs.clear();
    segs.reserve(static_cast<size_t>(n) * n);
    for (uint32_t i = 0; i < n; ++i) {
        const uint64_t* vi = p.ranks[i].var.data();
        for (uint32_t j = 0; j < n; ++j) {
            const uint64_t* vj = p.ranks[j].var.data();
            const uint64_t len = vj[i] * esz;
            if (len == 0) {
                continue;
            }
            segs.push_back({reinterpret_cast<uint64_t>(p.ranks[j].send) + vj[2 * n + i] * esz,
                            reinterpret_cast<uint64_t>(p.ranks[i].recv) + vi[3 * n + j] * esz, len});
        }
    }
    return RunSegmentCopy(w, segs, s, p.noAlloc);
}

// Broadcast: buf_r = buf_root, one read of the root's buffer and n - 1 writes (reference hccl.h:52-53).
HcclResult RunBroadcast(World* w, PendingOp& p, hipStream_t s)
{
    const uint32_t n = w->n;
    BcastCopyArgs b{};
    b.nSeg = 1;
    b.src[0] = p.ranks[p.root].recv;
    b.len[0] = p.count * DataTypeSize(p.dtype);
    b.dstOff[0] = 0;
    for (uint32_t r = 0; r < n; ++r) {
        if (r != p.root && p.ranks[r].recv != p.ranks[p.root].recv) {
            b.dst[b.nDst++] = p.ranks[r].recv;
        }
    }
    if (b.nDst == 0) {
        return HCCL_SUCCESS;
    }
    return RunOneToMany(w, b, s);
}

// Scatter: recv_r = send_root[r * recvCount ..] (reference hccl.h:107-109).
HcclResult RunScatter(World* w, PendingOp& p, hipStream_t s)
{
    const uint32_t n = w->n;
    const uint64_t len = p.count * DataTypeSize(p.dtype);
    const uint64_t base = reinterpret_cast<uint64_t>(p.ranks[p.root].send);
    if (base == 0) {
        return HCCL_E_PTR;
    }
    std::vector<CopySeg> segs;
    for (uint32_t r = 0; r < n; ++r) {
        segs.push_back({base + r * len, reinterpret_cast<uint64_t>(p.ranks[r].recv), len});
    }
    return RunSegmentCopy(w, segs, s);
}

// rankSize == 1: a plain copy, nothing when in place (reference op_common.cc:4458-4522).
HcclResult RunSingleRank(World* w, PendingOp& p, hipStream_t s)
{
    const RankArgs& r = p.ranks[0];
    if (r.send == r.recv) {
        return HCCL_SUCCESS;
    }
    const uint64_t esz = DataTypeSize(p.dtype);
    uint64_t len = p.count * esz;
    uint64_t dstOff = 0;
    if (p.type == OpType::BROADCAST) {
        return HCCL_SUCCESS;    // the only rank is the root
    }
    if (p.type == OpType::ALL_GATHER_V) {
        len = r.var[0] * esz;
        dstOff = r.var[1] * esz;
    } else if (p.type == OpType::ALL_TO_ALL_V) {
        len = r.var[0] * esz;   // sendCounts[0], copied from the start of sendBuf to the start of recvBuf
    } else if (p.type == OpType::REDUCE_SCATTER_V) {
        len = r.var[0] * esz;   // sendCounts[0], likewise from the start (op_common.cc:4490-4491)
    }
    if (len == 0) {
        return HCCL_SUCCESS;
    }
    BcastCopyArgs b{};
    b.nSeg = 1;
    b.nDst = 1;
    b.src[0] = r.send;
    b.dst[0] = r.recv;
    b.len[0] = len;
    b.dstOff[0] = dstOff;
    return RunBcast(w, b, s);
}

}  // namespace hccl_amd
