// Shared state of the host layer: worlds, communicators, pending collectives, and the helpers every part of it
// uses.  Internal to the library (nothing here is part of the C ABI).
//
// The host layer in files: host_world.cc (logging, argument checks, environment, world creation, the registry of
// live handles, fold-plan upload), launch_reduce.cc and launch_copy.cc (what one collective launches, and in which
// form: launch_policy.h), rendezvous.cc (pairing the per-rank calls, the launch itself, point-to-point queues),
// api.cc (the extern "C" entry points of include/hccl.h with the reference's argument checks).
#pragma once

#include <hip/hip_runtime.h>

#include <condition_variable>
#include <deque>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "dataplane.h"
#include "fold_plan.h"
#include "hccl.h"

namespace hccl_amd {

// Logging: HCCL_AMD_LOG_LEVEL = 0 (silent), 1 (errors, default), 2 (info).
void Log(int level, const char* fmt, ...);

#define HIP_OK(expr)                                                                          \
    do {                                                                                      \
        hipError_t e_ = (expr);                                                               \
        if (e_ != hipSuccess) {                                                               \
            Log(1, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), __FILE__, __LINE__); \
            return HCCL_E_RUNTIME;                                                            \
        }                                                                                     \
    } while (0)

uint32_t DataTypeSize(HcclDataType t);
HcclResult CheckCount(uint64_t count);
HcclResult CheckDataType(HcclDataType t, bool needReduce);
HcclResult CheckReduceOp(HcclDataType t, HcclReduceOp op);

// ---------------------------------------------------------------------------------------------
// World, communicators, pending collectives
// ---------------------------------------------------------------------------------------------
enum class OpType {
    ALL_REDUCE, REDUCE_SCATTER, ALL_GATHER, ALL_GATHER_V, ALL_TO_ALL_V,
    REDUCE_SCATTER_V, REDUCE, BROADCAST, SCATTER, BARRIER
};
const char* OpName(OpType t);

struct RankArgs {
    const void* send = nullptr;
    void* recv = nullptr;
    hipStream_t stream = nullptr;
    bool arrived = false;
    // AllGatherV: counts | displs | sendCount ; AlltoAllV: sendCounts | recvCounts | sdispls | rdispls ;
    // ReduceScatterV: counts | displs | recvCount
    std::vector<uint64_t> var;
};

struct PendingOp {
    OpType type;
    HcclDataType dtype;
    HcclReduceOp op = HCCL_REDUCE_RESERVED;
    uint64_t count = 0;
    uint32_t root = 0;
    uint32_t arrived = 0;
    bool done = false;
    HcclResult result = HCCL_SUCCESS;
    bool noAlloc = false;   // the allocation-free variant of the entry point was called
    std::vector<RankArgs> ranks;
};

// One Send / Recv pair.  The side that arrives second launches the copy.
struct P2pOp {
    uint64_t count = 0;
    HcclDataType dtype = HCCL_DATA_TYPE_RESERVED;
    const void* src = nullptr;
    void* dst = nullptr;
    hipStream_t sendStream = nullptr;
    hipStream_t recvStream = nullptr;
    bool haveSend = false;
    bool haveRecv = false;
    bool done = false;
    HcclResult result = HCCL_SUCCESS;
};

struct DevicePlan {
    uint8_t* dev = nullptr;
    uint32_t nProg = 0;
    uint32_t maxDepth = 1;
    uint32_t maxLeaves = 0;   // most leaves of any program of the plan
    bool segmentsAreSubs = false;
    std::shared_ptr<const std::vector<uint8_t>> host;   // the image at `dev`, for launches that resolve a program's leaves on the host
};

constexpr uint32_t kMagic = 0x48434C41u;   // "HCLA"
constexpr int kStagingSlots = 4;

// One (source, destination, length in bytes) copy; sources and destinations are arbitrary device addresses.
struct CopySeg {
    uint64_t src;
    uint64_t dst;
    uint64_t len;
};

struct World;
struct Comm {
    uint32_t magic = kMagic;
    World* world = nullptr;
    uint32_t rank = 0;
    bool destroyed = false;
};

constexpr uint32_t kReduceBlocksDefault = 1u << 26;   // HCCL_AMD_REDUCE_BLOCKS unset: as many workgroups as there are tiles

struct World {
    std::mutex mu;
    std::condition_variable cv;
    uint64_t id = 0;
    uint32_t n = 0;
    int device = 0;
    uint32_t joined = 0;
    uint32_t destroyed = 0;
    std::vector<std::unique_ptr<Comm>> comms;
    HcclAmdAlgo algo[HCCL_AMD_OP_COUNT] = {HCCL_AMD_ALGO_MESH, HCCL_AMD_ALGO_MESH};
    std::deque<std::shared_ptr<PendingOp>> pending;
    // Sends and receives that wait for their counterpart, first in first out per (source, destination) pair.
    std::map<std::pair<uint32_t, uint32_t>, std::deque<std::shared_ptr<P2pOp>>> p2p;
    uint64_t baseSeq = 0;
    uint64_t nextSeq[kMaxRanks] = {};
    std::map<uint32_t, DevicePlan> plans;
    std::vector<hipEvent_t> eventPool;
    hipEvent_t doneEvent = nullptr;
    // One launch at a time per world; while it runs, launchLock is the lock its caller holds on `mu`, so that
    // a step that has to wait for the GPU can release it for the duration of the wait.
    bool launchBusy = false;
    std::unique_lock<std::mutex>* launchLock = nullptr;
    // AlltoAllV tables
    uint8_t* a2aDev = nullptr;
    uint64_t* a2aHost[kStagingSlots] = {};
    hipEvent_t a2aSlotFree[kStagingSlots] = {};
    bool a2aSlotUsed[kStagingSlots] = {};
    uint32_t a2aNext = 0;
    // Hang triage (HCCL_AMD_STUCK_COUNTERS=1): two words in pinned host memory, written from the launch stream in
    // front of (head) and behind (tail) the kernels of every collective with the collective's number in this
    // world, like the reference's head / tail counters (aiv_communication_base_v2.h:365-378,
    // stuck_detect_counter_helper.h).  head != tail while the host can still read them = a kernel of collective
    // `head` started and has not finished.
    bool stuckEnabled = false;
    uint64_t* stuck = nullptr;
    uint64_t launchSeq = 0;
    // AllReduce as fold + fan-out (two kernels per piece of at most pieceBytes of results).
    uint64_t pieceBytes = 256ull << 20;   // HCCL_AMD_ALLREDUCE_PIECE_BYTES
    int twoKernelMode = 2;                // HCCL_AMD_ALLREDUCE_TWO_KERNELS: 0 never, 1 always, unset: by rank count and size
    int reducePair = 2;                   // HCCL_AMD_REDUCE_PAIR: 0 never, 1 wherever the form fits, else launch_policy.h decides
    int reduceDirect = -1;                // HCCL_AMD_REDUCE_DIRECT: 0 never, 2 .. 8 wavefronts wherever the form fits, else launch_policy.h decides
    int reduceDirectTiles = 0;            // HCCL_AMD_REDUCE_DIRECT_TILES: 1 / 2 tiles per wavefront of its straight-line instantiation, else launch_policy.h decides
    int reduceAllFold = -1;               // HCCL_AMD_REDUCE_ALL_FOLD: 0 never, 2 .. 4 wavefronts wherever the form fits, else launch_policy.h decides
    int fanOutLoadMode = 2;               // HCCL_AMD_FANOUT_STREAM_LOAD: 0 plain, 1 non-temporal, else launch_policy.h decides
    int copyTwoKernelMode = 2;            // HCCL_AMD_COPY_TWO_KERNELS, likewise for AllGather(V) and Broadcast
    // Allocation-free AlltoAllV: host image of the tables and the device array that receives them.
    std::vector<uint64_t> a2aImage;
    std::vector<CopySeg> a2aSegs;   // the segment list of the AlltoAllV being launched (one launch at a time per world)
    uint8_t* a2aScratch = nullptr;
    uint32_t reduceBlocks = kReduceBlocksDefault;
    uint32_t reduceThreads = 0;   // 0: chosen per launch
    uint32_t storeWaves = 0;      // wavefronts sharing the stores of a many-destination reduce tile; 0: chosen per launch
    uint32_t copyTileBytes = 0;
    bool reduceVector = true;
    uint32_t reduceBatch = 0;     // HCCL_AMD_REDUCE_BATCH: 8 or 16, 0 = per launch
    bool leadFromSrc = true;      // HCCL_AMD_LEAD_FROM_SRC=0: wavefronts always start on the destination's lines
    uint32_t storePolicy = 2;     // HCCL_AMD_STORE_POLICY for the reduce kernel: 0 non-temporal, 1 write-through, 2 per launch
    // HCCL_DETERMINISTIC (reference alg_env_config.cc:1113-1153): 0 false, 1 true, 2 strict, 0xFF unparsable
    uint8_t deterministic = 0;
    // Longest a rank waits on the host for its peers: the reference's CUSTOM_TIMEOUT = 1836 s (alg_param.h:91),
    // overridable by HCCL_EXEC_TIMEOUT (seconds), read when the world is created.
    uint32_t execTimeout = 1836;
    // Size of the staging buffer whose loops the slice-dependent AllReduce orders (NHR, RHD) reproduce; 0 = one
    // loop.  HCCL_BUFFSIZE when set, or HcclAmdSetCclBufferSize.
    uint64_t cclBytes = 0;
    // Ranks per level-0 group of the two-level AllReduce (HcclAmdSetLevel0RankSize, HCCL_AMD_LEVEL0_RANKS); 1 = one level.
    uint32_t level0 = 1;
    // Level-0 groups per level-1 group (HcclAmdSetLevel1GroupSize, HCCL_AMD_LEVEL1_GROUPS); 0 = all of them, two levels.
    uint32_t level1 = 0;
    // HCCL_ALGO asked for a sequence executor (1), a single-level one (0), or said nothing (-1): with level-0
    // groups, AllReduce runs in two levels unless a single-level executor was asked for.
    int allReduceSequence = -1;
    int reduceScatterSequence = -1;       // the same for ReduceScatter (reducescatter:sequence{mesh..., rhd | nhr | nhr_aicpu_reduce})
    int reduceSequence = -1;              // and for Reduce (reduce:sequence{mesh..., rhd | nhr | nhr_aicpu_reduce})
    bool envInvalid = false;      // an environment variable of the reference failed its parser

    ~World()
    {
        for (auto& kv : plans) {
            if (kv.second.dev) (void)hipFree(kv.second.dev);
        }
        for (hipEvent_t e : eventPool) (void)hipEventDestroy(e);
        if (doneEvent) (void)hipEventDestroy(doneEvent);
        if (a2aDev) (void)hipFree(a2aDev);
        if (stuck) (void)hipHostFree(stuck);
        for (int s = 0; s < kStagingSlots; ++s) {
            if (a2aHost[s]) (void)hipHostFree(a2aHost[s]);
            if (a2aSlotFree[s]) (void)hipEventDestroy(a2aSlotFree[s]);
        }
    }
};

// Worlds by id, and the live communicator handles with the world each belongs to.  A handle that is not in
// g_liveComms (never issued, destroyed, or of a world that is gone) is rejected without being dereferenced; a
// call holds its world through the shared pointer until it returns, whatever other threads destroy meanwhile.
extern std::mutex g_registryMu;
extern std::map<uint64_t, std::shared_ptr<World>> g_worlds;
extern std::unordered_map<const void*, std::shared_ptr<World>> g_liveComms;
extern uint64_t g_nextWorldId;
extern thread_local int t_groupDepth;

// What a thread queued since its outermost HcclGroupStart: HcclGroupEnd waits for these and reports their results.
struct GroupItem {
    std::shared_ptr<World> world;
    std::shared_ptr<PendingOp> op;
    std::shared_ptr<P2pOp> p2p;
};
extern thread_local std::vector<GroupItem> t_groupItems;

// A validated handle; keeps the world alive for the duration of the call.
struct CommRef {
    Comm* c = nullptr;
    std::shared_ptr<World> hold;
};

// ---- host_world.cc ------------------------------------------------------------------------------
uint32_t EnvU32(const char* name, uint32_t dflt);
int EnvInt(const char* name, int dflt);
bool AlgoFitsOp(HcclAmdOpKind kind, HcclAmdAlgo algo);
std::unique_ptr<World> NewWorld(uint32_t n);
CommRef AsComm(HcclComm h);
HcclResult CheckUserRank(const Comm* c);
// The fold programs of (kind, algo) for this world's rank size, uploaded on first use; level0 > 1: the two-level
// AllReduce over groups of that many ranks.
HcclResult GetDevicePlan(World* w, HcclAmdOpKind kind, HcclAmdAlgo algo, DevicePlan* out, uint32_t level0 = 1,
                         uint32_t level1 = 0);
HcclResult TakeEvent(World* w, hipEvent_t* ev);

// ---- launch_reduce.cc: `s` is the stream the kernels run on -----------------------------------------
HcclResult RunAllReduce(World* w, PendingOp& p, hipStream_t s);
HcclResult RunReduceScatter(World* w, PendingOp& p, hipStream_t s);
HcclResult RunReduceScatterV(World* w, PendingOp& p, hipStream_t s);
HcclResult RunReduce(World* w, PendingOp& p, hipStream_t s);

// ---- launch_copy.cc ---------------------------------------------------------------------------------
HcclResult PrepareNoAlloc(World* w);
HcclResult RunBcast(World* w, BcastCopyArgs& b, hipStream_t s);
HcclResult RunAllGather(World* w, PendingOp& p, hipStream_t s);
HcclResult RunAllGatherV(World* w, PendingOp& p, hipStream_t s);
HcclResult RunAlltoAllV(World* w, PendingOp& p, hipStream_t s);
HcclResult RunBroadcast(World* w, PendingOp& p, hipStream_t s);
HcclResult RunScatter(World* w, PendingOp& p, hipStream_t s);
HcclResult RunSingleRank(World* w, PendingOp& p, hipStream_t s);

// ---- rendezvous.cc ----------------------------------------------------------------------------------
// Makes the world's device current for the calling thread while the launch is prepared (the last rank to
// arrive may run on a thread that never selected a device) and puts the previous one back afterwards.
struct DeviceScope {
    int previous = -1;
    explicit DeviceScope(int device)
    {
        int current = -1;
        if (hipGetDevice(&current) == hipSuccess && current != device && hipSetDevice(device) == hipSuccess) {
            previous = current;
        }
    }
    ~DeviceScope()
    {
        if (previous >= 0) {
            (void)hipSetDevice(previous);
        }
    }
};

// Deposits one rank's arguments of a collective; the call that completes the set launches.  Blocks until the set
// is complete outside a group (HcclGroupStart / End), returns at once inside one.
HcclResult Submit(const CommRef& ref, OpType type, HcclDataType dtype, HcclReduceOp op, uint64_t count, const void* send,
                  void* recv, hipStream_t stream, std::vector<uint64_t>&& var, uint32_t root = 0, bool noAlloc = false);
// A call that fails its argument checks after its communicator has been identified still takes its place in
// the rank's sequence of collectives: the peers of that collective wake at once with the same verdict (nothing
// is launched), and the calls that follow pair up as they would have.
HcclResult Reject(const CommRef& ref, OpType type, HcclResult rc);
inline HcclResult RejectIfKnown(const CommRef& ref, OpType type, HcclResult rc) { return Reject(ref, type, rc); }
void PopFinished(World* w);

// Runs `run` on stream `s` after everything queued on `other`, and makes `other` wait for it.
template <class F>
HcclResult RunBetweenStreams(World* w, hipStream_t s, hipStream_t other, F run)
{
    DeviceScope onWorldDevice(w->device);
    hipEvent_t ev = nullptr;
    if (other != s) {
        HcclResult rc = TakeEvent(w, &ev);
        if (rc != HCCL_SUCCESS) {
            return rc;
        }
        w->eventPool.push_back(ev);   // reusable as soon as the wait below has been queued
        HIP_OK(hipEventRecord(ev, other));
        HIP_OK(hipStreamWaitEvent(s, ev, 0));
    }
    HcclResult rc = run();
    if (rc == HCCL_SUCCESS && other != s) {
        if (w->doneEvent == nullptr) {
            HIP_OK(hipEventCreateWithFlags(&w->doneEvent, hipEventDisableTiming));
        }
        HIP_OK(hipEventRecord(w->doneEvent, s));
        HIP_OK(hipStreamWaitEvent(other, w->doneEvent, 0));
    }
    return rc;
}

// Deposits one side of a Send / Recv pair (src -> dst); completes the pair when the other side is waiting.
// Caller holds w->mu.  Returns the op so that the caller can wait for it.
std::shared_ptr<P2pOp> DepositP2p(World* w, bool isSend, uint32_t src, uint32_t dst, void* buf, uint64_t count,
                                  HcclDataType dtype, hipStream_t stream);
// Blocks until every op of `ops` is complete (outside a group); the worst result wins.
HcclResult AwaitP2p(const CommRef& ref, std::unique_lock<std::mutex>& lock,
                    const std::vector<std::shared_ptr<P2pOp>>& ops, const char* what, uint32_t rank);

}  // namespace hccl_amd
