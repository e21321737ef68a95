// Host layer, part 4: the rendezvous of the per-rank calls of one collective, the launch by the call that completes
// the set, and the queues of point-to-point transfers.
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

HcclResult Launch(World* w, PendingOp& p, uint32_t launcher)
{
    DeviceScope onWorldDevice(w->device);
    hipStream_t s = p.ranks[launcher].stream;
    if (p.noAlloc) {
        HcclResult prc = PrepareNoAlloc(w);
        if (prc != HCCL_SUCCESS) {
            return prc;
        }
    }
    // Order the fused kernel after everything queued so far on the other ranks' streams (a superset of
    // what each rank had queued when it called).  Ranks that share the launch stream need nothing.
    std::vector<hipEvent_t> used;
    // Events go back to the pool on every path out of here.
    struct Returner {
        World* w;
        std::vector<hipEvent_t>& used;
        ~Returner()
        {
            for (hipEvent_t ev : used) {
                w->eventPool.push_back(ev);
            }
        }
    } returner{w, used};
    for (uint32_t r = 0; r < w->n; ++r) {
        if (p.ranks[r].stream == s) {
            continue;
        }
        bool seen = false;
        for (uint32_t q = 0; q < r; ++q) {
            seen = seen || p.ranks[q].stream == p.ranks[r].stream;
        }
        if (seen) {
            continue;
        }
        hipEvent_t ev;
        HcclResult erc = TakeEvent(w, &ev);
        if (erc != HCCL_SUCCESS) {
            return erc;
        }
        used.push_back(ev);
        HIP_OK(hipEventRecord(ev, p.ranks[r].stream));
        HIP_OK(hipStreamWaitEvent(s, ev, 0));
    }
    if (w->stuckEnabled) {
        if (w->stuck == nullptr) {
            HIP_OK(hipHostMalloc(reinterpret_cast<void**>(&w->stuck), 2 * sizeof(uint64_t), hipHostMallocDefault));
            w->stuck[0] = w->stuck[1] = 0;
        }
        HIP_OK(LaunchMark(w->stuck, ++w->launchSeq, s));
    }
    HcclResult rc;
    if (p.type == OpType::BARRIER) {
        rc = HCCL_SUCCESS;   // the ordering of the streams around this point is the whole operation
    } else if (w->n == 1) {
        rc = RunSingleRank(w, p, s);
    } else {
        switch (p.type) {
            case OpType::ALL_REDUCE: rc = RunAllReduce(w, p, s); break;
            case OpType::REDUCE_SCATTER: rc = RunReduceScatter(w, p, s); break;
            case OpType::ALL_GATHER: rc = RunAllGather(w, p, s); break;
            case OpType::ALL_GATHER_V: rc = RunAllGatherV(w, p, s); break;
            case OpType::REDUCE_SCATTER_V: rc = RunReduceScatterV(w, p, s); break;
            case OpType::REDUCE: rc = RunReduce(w, p, s); break;
            case OpType::BROADCAST: rc = RunBroadcast(w, p, s); break;
            case OpType::SCATTER: rc = RunScatter(w, p, s); break;
            default: rc = RunAlltoAllV(w, p, s); break;
        }
    }
    if (w->stuckEnabled && w->stuck != nullptr) {
        HIP_OK(LaunchMark(w->stuck + 1, w->launchSeq, s));
    }
    // Order every other rank's stream after the fused kernel.
    bool others = false;
    for (uint32_t r = 0; r < w->n; ++r) {
        others = others || p.ranks[r].stream != s;
    }
    if (others && rc == HCCL_SUCCESS) {
        if (w->doneEvent == nullptr) {
            HIP_OK(hipEventCreateWithFlags(&w->doneEvent, hipEventDisableTiming));
        }
        HIP_OK(hipEventRecord(w->doneEvent, s));
        for (uint32_t r = 0; r < w->n; ++r) {
            if (p.ranks[r].stream != s) {
                HIP_OK(hipStreamWaitEvent(p.ranks[r].stream, w->doneEvent, 0));
            }
        }
    }
    return rc;
}

// Drops the collectives at the head of the queue that every rank has been through.
void PopFinished(World* w)
{
    while (!w->pending.empty() && w->pending.front() && w->pending.front()->done &&
           w->pending.front()->arrived == w->n) {
        w->pending.pop_front();
        w->baseSeq++;
    }
}

// The cell of rank `rank`'s next call in the world's sequence of collectives (created by the first rank to get
// there).  Caller holds w->mu.
std::shared_ptr<PendingOp> NextCell(World* w, uint32_t rank, OpType type, HcclDataType dtype, HcclReduceOp op,
                                    uint64_t count, uint32_t root, bool noAlloc, bool* created)
{
    const uint64_t seq = w->nextSeq[rank]++;
    while (w->baseSeq + w->pending.size() <= seq) {
        w->pending.push_back(nullptr);
    }
    std::shared_ptr<PendingOp>& cell = w->pending[seq - w->baseSeq];
    *created = !cell;
    if (!cell) {
        cell = std::make_shared<PendingOp>();
        cell->type = type;
        cell->dtype = dtype;
        cell->op = op;
        cell->count = count;
        cell->root = root;
        cell->noAlloc = noAlloc;
        cell->ranks.resize(w->n);
    }
    return cell;
}

// Deposits one rank's arguments; the call that completes the set launches.
HcclResult Submit(const CommRef& ref, OpType type, HcclDataType dtype, HcclReduceOp op, uint64_t count, const void* send,
                  void* recv, hipStream_t stream, std::vector<uint64_t>&& var, uint32_t root, bool noAlloc)
{
    Comm* c = ref.c;
    World* w = c->world;
    std::unique_lock<std::mutex> lock(w->mu);
    if (w->destroyed != 0) {
        Log(1, "%s on rank %u: a communicator of this world has been destroyed", OpName(type), c->rank);
        return HCCL_E_UNAVAIL;
    }
    bool created = false;
    std::shared_ptr<PendingOp> p = NextCell(w, c->rank, type, dtype, op, count, root, noAlloc, &created);
    p->arrived++;
    if (p->done) {
        // Settled before this rank arrived: a peer's call failed its checks, or timed out.
        const HcclResult rc = p->result;
        PopFinished(w);
        return rc;
    }
    if (p->type != type || p->dtype != dtype || p->op != op || p->count != count || p->root != root ||
        p->noAlloc != noAlloc) {
        Log(1, "%s on rank %u does not match the call of the other ranks (%s, count %llu, type %d, root %u)",
            OpName(type), c->rank, OpName(p->type), (unsigned long long)p->count, static_cast<int>(p->dtype), p->root);
        p->result = HCCL_E_PARA;
    }
    RankArgs& ra = p->ranks[c->rank];
    ra.send = send;
    ra.recv = recv;
    ra.stream = stream;
    ra.var = std::move(var);
    ra.arrived = true;

    if (p->arrived < w->n) {
        if (t_groupDepth > 0) {
            t_groupItems.push_back({ref.hold, p, nullptr});
            return p->result;   // queued; the call that completes the set launches, HcclGroupEnd waits for it
        }
        bool ok = w->cv.wait_for(lock, std::chrono::seconds(w->execTimeout), [&] { return p->done; });
        if (!ok) {
            Log(1, "%s: rank %u waited %u s for the other ranks", OpName(type), c->rank, w->execTimeout);
            p->result = HCCL_E_TIMEOUT;
            return HCCL_E_TIMEOUT;
        }
        return p->result;
    }

    // Last arrival: launch, one launch at a time per world.
    w->cv.wait(lock, [&] { return !w->launchBusy; });
    if (p->result == HCCL_SUCCESS && w->destroyed == 0) {
        w->launchBusy = true;
        w->launchLock = &lock;
        const HcclResult launched = Launch(w, *p, c->rank);
        if (!p->done) {   // (settled meanwhile by a rank that left while a launch waited without the lock: that verdict stands)
            p->result = launched;
        }
        w->launchLock = nullptr;
        w->launchBusy = false;
    } else if (p->result == HCCL_SUCCESS) {
        p->result = HCCL_E_UNAVAIL;
    }
    p->done = true;
    PopFinished(w);
    w->cv.notify_all();
    return p->result;
}

// A call that fails its argument checks after its communicator has been identified still takes its place in
// the rank's sequence of collectives: the peers of that collective wake at once with the same verdict (nothing
// is launched), and the calls that follow pair up as they would have.
HcclResult Reject(const CommRef& ref, OpType type, HcclResult rc)
{
    if (ref.c == nullptr) {
        return rc;
    }
    World* w = ref.c->world;
    std::unique_lock<std::mutex> lock(w->mu);
    if (w->destroyed != 0) {
        return rc;
    }
    bool created = false;
    std::shared_ptr<PendingOp> p = NextCell(w, ref.c->rank, type, HCCL_DATA_TYPE_RESERVED, HCCL_REDUCE_RESERVED, 0, 0,
                                            false, &created);
    p->arrived++;
    if (!p->done) {
        if (p->result == HCCL_SUCCESS) {
            p->result = rc;
        }
        p->done = true;
        Log(1, "%s: the call of rank %u was rejected (%d); the collective is abandoned on every rank", OpName(type),
            ref.c->rank, static_cast<int>(rc));
    }
    PopFinished(w);
    w->cv.notify_all();
    return rc;
}

// Deposits one side of a Send / Recv pair (src -> dst); completes the pair when the other side is waiting.
// Caller holds w->mu.  Returns the op so that the caller can wait for it.
std::shared_ptr<P2pOp> DepositP2p(World* w, bool isSend, uint32_t src, uint32_t dst, void* buf, uint64_t count,
                                  HcclDataType dtype, hipStream_t stream)
{
    std::deque<std::shared_ptr<P2pOp>>& q = w->p2p[{src, dst}];
    std::shared_ptr<P2pOp> op;
    for (const std::shared_ptr<P2pOp>& cand : q) {
        if (isSend ? !cand->haveSend : !cand->haveRecv) {
            op = cand;
            break;
        }
    }
    if (!op) {
        op = std::make_shared<P2pOp>();
        op->count = count;
        op->dtype = dtype;
        q.push_back(op);
    } else if (op->result == HCCL_SUCCESS && (op->count != count || op->dtype != dtype)) {
        Log(1, "%s %u -> %u: count %llu / type %d do not match the other side's %llu / %d", isSend ? "Send" : "Recv", src,
            dst, (unsigned long long)count, static_cast<int>(dtype), (unsigned long long)op->count,
            static_cast<int>(op->dtype));
        op->result = HCCL_E_PARA;
    }
    if (isSend) {
        op->haveSend = true;
        op->src = buf;
        op->sendStream = stream;
    } else {
        op->haveRecv = true;
        op->dst = buf;
        op->recvStream = stream;
    }
    if (op->haveSend && op->haveRecv) {
        if (op->result == HCCL_SUCCESS && op->src != op->dst) {
            BcastCopyArgs b{};
            b.nSeg = 1;
            b.nDst = 1;
            b.src[0] = op->src;
            b.dst[0] = op->dst;
            b.len[0] = op->count * DataTypeSize(op->dtype);
            op->result = RunBetweenStreams(w, stream, isSend ? op->recvStream : op->sendStream,
                                           [&] { return RunBcast(w, b, stream); });
        }
        op->done = true;
        for (auto it = q.begin(); it != q.end(); ++it) {
            if (*it == op) {
                q.erase(it);
                break;
            }
        }
        w->cv.notify_all();
    }
    return op;
}

// Blocks until every op of `ops` is complete (outside a group); the worst result wins.
HcclResult AwaitP2p(const CommRef& ref, std::unique_lock<std::mutex>& lock,
                    const std::vector<std::shared_ptr<P2pOp>>& ops, const char* what, uint32_t rank)
{
    World* w = ref.c->world;
    HcclResult rc = HCCL_SUCCESS;
    if (t_groupDepth > 0) {
        for (const auto& op : ops) {
            if (!op->done) {
                t_groupItems.push_back({ref.hold, nullptr, op});   // HcclGroupEnd waits for the peer
            }
        }
    }
    if (t_groupDepth == 0) {
        bool ok = w->cv.wait_for(lock, std::chrono::seconds(w->execTimeout), [&] {
            for (const auto& op : ops) {
                if (!op->done) {
                    return false;
                }
            }
            return true;
        });
        if (!ok) {
            Log(1, "%s: rank %u waited %u s for its peer", what, rank, w->execTimeout);
            for (const auto& op : ops) {
                if (!op->done) {
                    op->result = HCCL_E_TIMEOUT;   // the late peer finds the verdict and copies nothing
                }
            }
            return HCCL_E_TIMEOUT;
        }
    }
    for (const auto& op : ops) {
        if (op->result != HCCL_SUCCESS) {
            rc = op->result;
        }
    }
    return rc;
}

}  // namespace hccl_amd
