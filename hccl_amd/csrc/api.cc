// Host layer of the loopback data plane: the C ABI of include/hccl.h over HIP streams.
//
// What the reference spreads over op entry / selector / executor / template / wrapper
// (src/ops/<op>/<op>.cc -> op_common.cc Selector + HcclExecOp -> executor -> template ->
// alg_data_trans_wrapper.cc) collapses here to: argument checks with the reference's return codes,
// a rendezvous of the N per-rank calls, and one fused kernel launch per collective.
#include <hip/hip_runtime.h>

#include <cctype>
#include <chrono>
#include <condition_variable>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <algorithm>
#include <deque>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "dataplane.h"
#include "algo_config.h"
#include "fold_plan.h"
#include "hccl.h"

namespace hccl_amd {
namespace {

// ---------------------------------------------------------------------------------------------
// Logging: HCCL_AMD_LOG_LEVEL = 0 (silent), 1 (errors, default), 2 (info).
// ---------------------------------------------------------------------------------------------
int LogLevel()
{
    static int level = [] {
        const char* s = getenv("HCCL_AMD_LOG_LEVEL");
        return s ? atoi(s) : 1;
    }();
    return level;
}

void Log(int level, const char* fmt, ...)
{
    if (level > LogLevel()) {
        return;
    }
    va_list ap;
    va_start(ap, fmt);
    fprintf(stderr, level == 1 ? "[hccl_amd][ERROR] " : "[hccl_amd][INFO] ");
    vfprintf(stderr, fmt, ap);
    fputc('\n', stderr);
    va_end(ap);
}

#define HIP_OK(expr)                                                                          \
    do {                                                                                      \
        hipError_t e_ = (expr);                                                               \
        if (e_ != hipSuccess) {                                                               \
            Log(1, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), __FILE__, __LINE__); \
            return HCCL_E_RUNTIME;                                                            \
        }                                                                                     \
    } while (0)

// Element sizes, indexed by HcclDataType (reference src/ops/op_common/inc/alg_param.h:55-73).
uint32_t DataTypeSize(HcclDataType t)
{
    static const uint32_t sizes[18] = {1, 2, 4, 2, 4, 8, 8, 1, 2, 4, 8, 2, 16, 2, 1, 1, 1, 1};
    int v = static_cast<int>(t);
    return (v >= 0 && v < 18) ? sizes[v] : 0;
}

bool IsValidDataType(HcclDataType t)
{
    int v = static_cast<int>(t);
    return v >= 0 && v <= 17 && v != 13;   // 13 is a reserved gap, 255 is RESERVED
}

// Reference op_common.cc:4311-4321.
HcclResult CheckCount(uint64_t count)
{
    if (count > HCCL_SYS_MAX_COUNT) {
        Log(1, "count %llu exceeds the supported maximum %llu", (unsigned long long)count,
            (unsigned long long)HCCL_SYS_MAX_COUNT);
        return HCCL_E_PARA;
    }
    return HCCL_SUCCESS;
}

// Reference op_common.cc:4323-4364.
HcclResult CheckDataType(HcclDataType t, bool needReduce)
{
    bool notValid = !IsValidDataType(t);
    if (needReduce) {
        switch (t) {
            case HCCL_DATA_TYPE_UINT8:
            case HCCL_DATA_TYPE_UINT16:
            case HCCL_DATA_TYPE_UINT32:
            case HCCL_DATA_TYPE_INT128:
            case HCCL_DATA_TYPE_HIF8:
            case HCCL_DATA_TYPE_FP8E4M3:
            case HCCL_DATA_TYPE_FP8E5M2:
            case HCCL_DATA_TYPE_FP8E8M0:
                notValid = true;
                break;
            default:
                break;
        }
    } else if (t == HCCL_DATA_TYPE_INT128) {
        notValid = true;
    }
    if (notValid) {
        Log(1, "data type %d is not supported (%s)", static_cast<int>(t), needReduce ? "reduce" : "copy");
        return HCCL_E_NOT_SUPPORT;
    }
    return HCCL_SUCCESS;
}

// Reference op_common.cc:4392-4413: PROD exists for int8, int32, int64, uint64, fp16, fp32, fp64 only.
HcclResult CheckReduceOp(HcclDataType t, HcclReduceOp op)
{
    if (static_cast<int>(op) < 0 || static_cast<int>(op) >= static_cast<int>(HCCL_REDUCE_RESERVED)) {
        Log(1, "reduce op %d is invalid", static_cast<int>(op));
        return HCCL_E_PARA;
    }
    if (op == HCCL_REDUCE_PROD) {
        switch (t) {
            case HCCL_DATA_TYPE_INT8:
            case HCCL_DATA_TYPE_INT32:
            case HCCL_DATA_TYPE_INT64:
            case HCCL_DATA_TYPE_UINT64:
            case HCCL_DATA_TYPE_FP16:
            case HCCL_DATA_TYPE_FP32:
            case HCCL_DATA_TYPE_FP64:
                break;
            default:
                Log(1, "PROD is not supported for data type %d", static_cast<int>(t));
                return HCCL_E_NOT_SUPPORT;
        }
    }
    return HCCL_SUCCESS;
}

// ---------------------------------------------------------------------------------------------
// World, communicators, pending collectives
// ---------------------------------------------------------------------------------------------
enum class OpType {
    ALL_REDUCE, REDUCE_SCATTER, ALL_GATHER, ALL_GATHER_V, ALL_TO_ALL_V,
    REDUCE_SCATTER_V, REDUCE, BROADCAST, SCATTER, BARRIER
};

const char* OpName(OpType t)
{
    switch (t) {
        case OpType::ALL_REDUCE: return "AllReduce";
        case OpType::REDUCE_SCATTER: return "ReduceScatter";
        case OpType::ALL_GATHER: return "AllGather";
        case OpType::ALL_GATHER_V: return "AllGatherV";
        case OpType::REDUCE_SCATTER_V: return "ReduceScatterV";
        case OpType::REDUCE: return "Reduce";
        case OpType::BROADCAST: return "Broadcast";
        case OpType::SCATTER: return "Scatter";
        case OpType::BARRIER: return "Barrier";
        default: return "AlltoAllV";
    }
}

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
    bool segmentsAreSubs = false;
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
    int copyTwoKernelMode = 2;            // HCCL_AMD_COPY_TWO_KERNELS, likewise for AllGather(V) and Broadcast
    // Allocation-free AlltoAllV: host image of the tables and the device array that receives them.
    std::vector<uint64_t> a2aImage;
    std::vector<CopySeg> a2aSegs;   // the segment list of the AlltoAllV being launched (one launch at a time per world)
    uint8_t* a2aScratch = nullptr;
    uint32_t reduceBlocks = 1u << 26;
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
    // HCCL_ALGO asked for a sequence executor (1), a single-level one (0), or said nothing (-1): with level-0
    // groups, AllReduce runs in two levels unless a single-level executor was asked for.
    int allReduceSequence = -1;
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
std::mutex g_registryMu;
std::map<uint64_t, std::shared_ptr<World>> g_worlds;
std::unordered_map<const void*, std::shared_ptr<World>> g_liveComms;
uint64_t g_nextWorldId = 1;
thread_local int t_groupDepth = 0;

// What a thread queued since its outermost HcclGroupStart: HcclGroupEnd waits for these and reports their results.
struct GroupItem {
    std::shared_ptr<World> world;
    std::shared_ptr<PendingOp> op;
    std::shared_ptr<P2pOp> p2p;
};
thread_local std::vector<GroupItem> t_groupItems;

// A validated handle; keeps the world alive for the duration of the call.
struct CommRef {
    Comm* c = nullptr;
    std::shared_ptr<World> hold;
};

uint32_t EnvU32(const char* name, uint32_t dflt)
{
    const char* s = getenv(name);
    if (!s || !*s) {
        return dflt;
    }
    long v = atol(s);
    return v > 0 ? static_cast<uint32_t>(v) : dflt;
}

// An integer variable that may be 0: `dflt` when it is unset or empty.
int EnvInt(const char* name, int dflt)
{
    const char* s = getenv(name);
    return (s && *s) ? atoi(s) : dflt;
}

bool ParseAlgoName(const std::string& s, HcclAmdAlgo* algo)
{
    static const struct { const char* name; HcclAmdAlgo algo; } table[] = {
        {"mesh", HCCL_AMD_ALGO_MESH}, {"ring", HCCL_AMD_ALGO_RING}, {"rhd", HCCL_AMD_ALGO_RHD},
        {"nhr", HCCL_AMD_ALGO_NHR}, {"order_preserved", HCCL_AMD_ALGO_ORDER_PRESERVED},
        {"aiv_mesh", HCCL_AMD_ALGO_AIV_MESH}, {"mesh_symmetric", HCCL_AMD_ALGO_MESH_SYMMETRIC},
        {"mesh_chunk", HCCL_AMD_ALGO_MESH_CHUNK}, {"mesh_two_shot", HCCL_AMD_ALGO_MESH_TWO_SHOT}};
    for (const auto& e : table) {
        if (s == e.name) {
            *algo = e.algo;
            return true;
        }
    }
    return false;
}

// Which orders exist for which operator.
bool AlgoFitsOp(HcclAmdOpKind kind, HcclAmdAlgo algo)
{
    switch (kind) {
        case HCCL_AMD_OP_ALL_REDUCE:
            return algo != HCCL_AMD_ALGO_AIV_MESH && algo != HCCL_AMD_ALGO_MESH_TWO_SHOT;
        case HCCL_AMD_OP_REDUCE_SCATTER:
            return algo != HCCL_AMD_ALGO_MESH_TWO_SHOT;
        case HCCL_AMD_OP_REDUCE:
            return algo == HCCL_AMD_ALGO_MESH || algo == HCCL_AMD_ALGO_RING || algo == HCCL_AMD_ALGO_MESH_TWO_SHOT;
        default:
            return false;
    }
}

// HCCL_AMD_ALGO="allreduce=rhd;reducescatter=nhr;reduce=mesh_two_shot"
void ApplyAlgoEnv(World* w)
{
    const char* env = getenv("HCCL_AMD_ALGO");
    if (!env) {
        return;
    }
    std::string s(env);
    size_t pos = 0;
    while (pos < s.size()) {
        size_t end = s.find(';', pos);
        if (end == std::string::npos) end = s.size();
        std::string item = s.substr(pos, end - pos);
        size_t eq = item.find('=');
        if (eq != std::string::npos) {
            std::string key = item.substr(0, eq), val = item.substr(eq + 1);
            HcclAmdAlgo a;
            if (ParseAlgoName(val, &a)) {
                HcclAmdOpKind kind = key == "allreduce" ? HCCL_AMD_OP_ALL_REDUCE :
                                     key == "reducescatter" ? HCCL_AMD_OP_REDUCE_SCATTER :
                                     key == "reduce" ? HCCL_AMD_OP_REDUCE : HCCL_AMD_OP_COUNT;
                if (kind != HCCL_AMD_OP_COUNT && AlgoFitsOp(kind, a)) {
                    w->algo[kind] = a;
                } else {
                    Log(1, "HCCL_AMD_ALGO: '%s' does not apply to '%s'", val.c_str(), key.c_str());
                }
            } else {
                Log(1, "HCCL_AMD_ALGO: unknown algorithm '%s'", val.c_str());
            }
        }
        pos = end + 1;
    }
}

// HCCL_ALGO in the reference's own syntax (algo_config.h).  A string its parser rejects is ignored with a warning,
// as there (alg_parse.cc:803-826); clauses that select nothing for the three fold-order operators are ignored too.
void ApplyReferenceAlgoEnv(World* w)
{
    const char* env = getenv("HCCL_ALGO");
    if (!env) {
        return;
    }
    std::vector<AlgoSegment> segments;
    if (ParseHcclAlgo(env, &segments) != HCCL_SUCCESS) {
        Log(1, "HCCL_ALGO [%s] parse failed, the config has not taken effect, standard format: "
               "'opType:executorType{level0=algoType, level1=algoType};...'", env);
        return;
    }
    const AlgoSelection sel = SelectFromHcclAlgo(segments);
    for (int op = 0; op < HCCL_AMD_OP_COUNT; ++op) {
        const HcclAmdOpKind kind = static_cast<HcclAmdOpKind>(op);
        if (sel.set[op] && AlgoFitsOp(kind, sel.algo[op])) {
            w->algo[op] = sel.algo[op];
            if (kind == HCCL_AMD_OP_ALL_REDUCE) {
                w->allReduceSequence = sel.twoLevel[op] ? 1 : 0;
            }
        }
    }
}

std::unique_ptr<World> NewWorld(uint32_t n)
{
    auto w = std::make_unique<World>();
    w->n = n;
    w->comms.resize(n);
    if (hipGetDevice(&w->device) != hipSuccess) {
        w->device = 0;
    }
    w->reduceBlocks = EnvU32("HCCL_AMD_REDUCE_BLOCKS", 1u << 26);
    w->storeWaves = EnvU32("HCCL_AMD_REDUCE_STORE_WAVES", 0);
    if (w->storeWaves > kMaxReduceThreads / 64) {
        w->storeWaves = 0;
    }
    w->reduceThreads = EnvU32("HCCL_AMD_REDUCE_THREADS", 0);
    if (w->reduceThreads != 64 && w->reduceThreads != 128 && w->reduceThreads != 256) {
        w->reduceThreads = 0;
    }
    w->copyTileBytes = EnvU32("HCCL_AMD_COPY_TILE", 0);   // 0: chosen per collective
    if (w->copyTileBytes != 1024 && w->copyTileBytes != 4096 && w->copyTileBytes != 16384) {
        w->copyTileBytes = 0;
    }
    w->execTimeout = EnvU32("HCCL_EXEC_TIMEOUT", 1836);
    w->storePolicy = EnvU32("HCCL_AMD_STORE_POLICY", 2);
    if (w->storePolicy > 2) {
        w->storePolicy = 2;
    }
    w->reduceVector = EnvU32("HCCL_AMD_REDUCE_VECTOR", 1) != 0;
    w->stuckEnabled = EnvU32("HCCL_AMD_STUCK_COUNTERS", 0) != 0;
    w->twoKernelMode = EnvInt("HCCL_AMD_ALLREDUCE_TWO_KERNELS", 2);
    if (w->twoKernelMode < 0 || w->twoKernelMode > 1) {
        w->twoKernelMode = 2;
    }
    w->copyTwoKernelMode = EnvInt("HCCL_AMD_COPY_TWO_KERNELS", 2);
    if (w->copyTwoKernelMode < 0 || w->copyTwoKernelMode > 1) {
        w->copyTwoKernelMode = 2;
    }
    w->pieceBytes = (static_cast<uint64_t>(EnvU32("HCCL_AMD_ALLREDUCE_PIECE_BYTES", 256u << 20)) + 255) & ~255ull;
    if (w->pieceBytes == 0) {
        w->pieceBytes = 256;
    }
    w->leadFromSrc = EnvInt("HCCL_AMD_LEAD_FROM_SRC", 1) != 0;
    w->reduceBatch = EnvU32("HCCL_AMD_REDUCE_BATCH", 0);
    if (w->reduceBatch != 8 && w->reduceBatch != 16) {
        w->reduceBatch = 0;
    }
    ApplyReferenceAlgoEnv(w.get());
    ApplyAlgoEnv(w.get());
    {
        const uint32_t groups = EnvU32("HCCL_AMD_LEVEL0_RANKS", 1);
        if (groups >= 1 && groups <= n && n % groups == 0) {
            w->level0 = groups;
        } else {
            Log(1, "HCCL_AMD_LEVEL0_RANKS=%u does not divide the %u ranks of the world: ignored", groups, n);
        }
    }
    if (const char* det = getenv("HCCL_DETERMINISTIC")) {
        std::string v(det);
        for (char& ch : v) ch = static_cast<char>(toupper(static_cast<unsigned char>(ch)));
        w->deterministic = v == "STRICT" ? 2 : v == "TRUE" ? 1 : v == "FALSE" ? 0 : 0xFF;
        if (w->deterministic == 0xFF) {
            Log(1, "HCCL_DETERMINISTIC is set to [%s], which is incorrect (true, false or strict)", det);
            w->envInvalid = true;
        }
    }
    if (const char* buf = getenv("HCCL_BUFFSIZE")) {
        if (CclBufferAvailableSize(buf, &w->cclBytes) != HCCL_SUCCESS) {
            Log(1, "HCCL_BUFFSIZE is set to [%s], which is not a number of MB between 2 and 4294967295", buf);
            w->envInvalid = true;
        }
    }
    return w;
}

CommRef AsComm(HcclComm h)
{
    CommRef ref;
    if (h == nullptr) {
        return ref;
    }
    std::lock_guard<std::mutex> g(g_registryMu);
    auto it = g_liveComms.find(h);
    if (it != g_liveComms.end()) {
        ref.hold = it->second;
        ref.c = static_cast<Comm*>(h);
    }
    return ref;
}

// Reference src/common/param_check.cc:153-162.
HcclResult CheckUserRank(const Comm* c)
{
    if (c->rank >= c->world->n) {
        Log(1, "rank %u is out of range [0, %u)", c->rank, c->world->n);
        return HCCL_E_PARA;
    }
    return HCCL_SUCCESS;
}

// ---------------------------------------------------------------------------------------------
// Device resources
// ---------------------------------------------------------------------------------------------
HcclResult GetDevicePlan(World* w, HcclAmdOpKind kind, HcclAmdAlgo algo, DevicePlan* out, uint32_t level0 = 1)
{
    uint32_t key = (static_cast<uint32_t>(kind) * 64 + static_cast<uint32_t>(algo)) * 128 + level0;
    auto it = w->plans.find(key);
    if (it != w->plans.end()) {
        *out = it->second;
        return HCCL_SUCCESS;
    }
    FoldPlan plan;
    HcclResult rc = BuildFoldPlan(kind, algo, w->n, &plan, level0);
    if (rc != HCCL_SUCCESS) {
        return rc;
    }
    // Flatten every token program to the kernel's leaf table.
    std::vector<uint8_t> image(plan.programs.size() * kDevProgBytes, 0);
    for (size_t s = 0; s < plan.programs.size(); ++s) {
        uint8_t* img = image.data() + s * kDevProgBytes;
        uint32_t leaves = 0;
        bool open = false;
        const std::vector<uint8_t>& prog = plan.programs[s];
        for (size_t i = 0; i < prog.size() && prog[i] != kTokEnd; ++i) {
            uint8_t tok = prog[i];
            if (tok == kTokOpen) {
                open = true;
            } else if (tok == kTokClose) {
                img[kDevProgCtlOff + leaves - 1]++;
            } else {
                uint32_t n = tok >= kTokRun ? (tok & 0x3Fu) : 1u;
                for (uint32_t k = 0; k < n; ++k) {
                    uint8_t rank = tok >= kTokRun ? prog[++i] : tok;
                    if (leaves >= static_cast<uint32_t>(kMaxRanks)) {
                        return HCCL_E_INTERNAL;
                    }
                    img[kDevProgRankOff + leaves] = rank;
                    img[kDevProgCtlOff + leaves] = open ? kCtlOpen : 0;
                    open = false;
                    ++leaves;
                }
            }
        }
        img[0] = static_cast<uint8_t>(leaves);
    }
    DevicePlan dp;
    dp.nProg = static_cast<uint32_t>(plan.programs.size());
    dp.segmentsAreSubs = plan.segmentsAreSubs;
    dp.maxDepth = plan.maxDepth;
    HIP_OK(hipMalloc(reinterpret_cast<void**>(&dp.dev), image.size()));
    HIP_OK(hipMemcpy(dp.dev, image.data(), image.size(), hipMemcpyHostToDevice));
    w->plans[key] = dp;
    *out = dp;
    return HCCL_SUCCESS;
}

HcclResult TakeEvent(World* w, hipEvent_t* ev)
{
    if (!w->eventPool.empty()) {
        *ev = w->eventPool.back();
        w->eventPool.pop_back();
        return HCCL_SUCCESS;
    }
    HIP_OK(hipEventCreateWithFlags(ev, hipEventDisableTiming));
    return HCCL_SUCCESS;
}

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


// ---------------------------------------------------------------------------------------------
// Launches.  `s` is the stream the fused kernel runs on.
// ---------------------------------------------------------------------------------------------
uint32_t BlocksPerSub(const World* w, uint64_t subLen, uint32_t esz, uint64_t nSubTotal, uint32_t threads)
{
    uint64_t vecs = (subLen * esz + 15) / 16 + kReduceLeadMask;   // lanes the kernel may skip to start on a 1 KiB boundary
    uint64_t maxUseful = (vecs + threads - 1) / threads;
    if (maxUseful == 0) maxUseful = 1;
    uint64_t want = (w->reduceBlocks + nSubTotal - 1) / nSubTotal;
    if (want == 0) want = 1;
    return static_cast<uint32_t>(want < maxUseful ? want : maxUseful);
}

HcclResult LaunchOneReduce(World* w, ReduceArgs& a, const DevicePlan& plan, HcclDataType dtype, HcclReduceOp op,
                           hipStream_t s)
{
    uint32_t esz = DataTypeSize(dtype);
    // 128-bit loads and stores may start on any element (the head is peeled for the first destination, which
    // makes every store aligned in the usual case of equally aligned recvBufs).  HCCL_AMD_REDUCE_VECTOR=0
    // forces the element-by-element path.
    a.vecOk = w->reduceVector ? 1u : 0u;
    uint64_t subs = static_cast<uint64_t>(a.nGroup) * a.nSub;
    uint64_t longest = a.groupLen;   // the last sub-segment takes what the others leave
    if (a.nSub > 1) {
        uint64_t before = a.subLen * (a.nSub - 1);
        uint64_t last = a.groupLen > before ? a.groupLen - before : 0;
        longest = last > a.subLen ? last : a.subLen;
    }
    // One wavefront per workgroup: a wavefront needs nothing from its neighbours (the fold program is read
    // with scalar loads, no barrier), small workgroups retire sooner and keep the window of addresses in
    // flight compact.  Measured best for flat and nested programs alike.
    // A result that is written once (ReduceScatter(V), Reduce) leaves through write-through stores, 3-4 % faster
    // than non-temporal ones next to eight read streams; results written to many destinations (AllReduce)
    // keep non-temporal stores, 2-3 % faster there.  HCCL_AMD_STORE_POLICY = 0 / 1 forces one of them.
    const bool oneStream = a.dstOwn || a.nDst == 1;
    a.writeThrough = w->storePolicy != 2 ? w->storePolicy : (oneStream ? 1u : 0u);
    // Many sources folded into one result stream: the wavefronts start on the sources' 1 KiB boundaries (a
    // ReduceScatterV slice begins wherever its displacement puts it; measured 0.74 -> 0.80 of peak on uneven
    // slices) and the single store stream straddles.  HCCL_AMD_LEAD_FROM_SRC=0 keeps the destination's lines.
    a.leadFromSrc = (oneStream && w->leadFromSrc) ? 1u : 0u;
    // Up to eight ranks folded into one result stream run best with eight-load batches (fewer registers, more
    // wavefronts in flight: +1-2 %); AllReduce's many result streams and larger worlds with sixteen (+5 %).
    a.vecBatch = w->reduceBatch != 0 ? w->reduceBatch : ((w->n <= 8 && !a.varGroups && (a.dstOwn || a.nDst == 1)) ? 8u : 16u);
    a.threads = w->reduceThreads != 0 ? w->reduceThreads : 64u;
    // A result that goes to many destinations: a wavefront that stores to six or more streams one after the other
    // is what bounds the launch, so wavefront 0 of a workgroup folds the tile and two or three wavefronts share its
    // stores.  The extra wavefronts hold slots while they wait, which costs more than it gains on short messages
    // and where folding a tile takes long (8- and 16-bit types with their wide accumulators): measured, fp32 SUM
    // in rank order, 6 ranks 0.72 -> 0.75 / 0.74 -> 0.79 / 0.73 -> 0.78 of the HBM peak at 64 / 128 / 512 MiB per
    // rank with two wavefronts (32 MiB: 0.69 -> 0.67), 8 ranks 0.65 -> 0.72 / 0.70 -> 0.77 / 0.72 -> 0.78 at 32 / 64 /
    // 128 MiB with three (16 MiB: 0.62 -> 0.61).  HCCL_AMD_REDUCE_STORE_WAVES forces a count (1 = one wavefront per
    // tile).
    a.storeWaves = 1;
    if (!oneStream && a.threads == 64 && a.vecOk) {
        const uint64_t bytes = a.total * esz;
        const bool longFold = esz < 4;
        uint32_t waves = 1;
        if (a.nDst >= 8) {
            waves = longFold ? (bytes >= (64ull << 20) ? 2u : 1u) : (bytes >= (24ull << 20) ? 3u : 1u);
        } else if (a.nDst >= 4) {
            // (four and five destinations too, since the launch's scalars come in one round: fp32 over 4 ranks
            // 0.72 -> 0.74 / 0.75 -> 0.79 / 0.76 -> 0.79 at 64 / 256 / 512 MiB per rank, bf16 alike; two and three
            // ranks still lose)
            waves = bytes >= (48ull << 20) ? 2u : 1u;
        }
        if (w->storeWaves != 0) {
            waves = w->storeWaves < a.nDst ? w->storeWaves : a.nDst;
        }
        a.storeWaves = waves;
        // With the stores elsewhere the folding wavefront is better off with the smaller load batch where that
        // holds every leaf (fp16 RHD over 6 ranks: 0.71 -> 0.75, fp16 NHR over 8: 0.71 -> 0.77).
        if (waves > 1 && w->reduceBatch == 0 && w->n <= 8) {
            a.vecBatch = 8;
        }
    }
    a.blocksPerSub = BlocksPerSub(w, longest, a.vecOk ? esz : 16 /* one element per lane */, subs, a.threads);
    uint64_t blocks = subs * a.blocksPerSub;
    if (a.varGroups) {
        // every group gets the workgroups its own length needs (an empty group gets none)
        blocks = 0;
        for (uint32_t g = 0; g < a.nGroup; ++g) {
            if (a.groupLenV[g] != 0) {
                blocks += BlocksPerSub(w, a.groupLenV[g], a.vecOk ? esz : 16, subs, a.threads);
            }
            a.groupBlockEnd[g] = static_cast<uint32_t>(blocks < 0x7FFFFFFFull ? blocks : 0x7FFFFFFFull);
        }
        for (uint32_t g = a.nGroup; g < 16; ++g) {
            a.groupBlockEnd[g] = 0xFFFFFFFFu;   // the kernel reads sixteen entries in one go when there are that few groups
        }
    }
    if (blocks == 0 || blocks > 0x7FFFFFFFull) {
        return HCCL_E_INTERNAL;
    }
    const uint32_t lds = (plan.maxDepth - 1) * ReduceAccBytes(dtype, op) * a.threads;
    HIP_OK(LaunchReduce(a, dtype, op, static_cast<uint32_t>(blocks), lds, s));
    return HCCL_SUCCESS;
}

// HCCL_DETERMINISTIC=strict moves float SUM / PROD over more than two ranks to the order-preserved fold
// (reference src/common/order_preserved_common.h:104-114).  The reference offers its write-reduce templates
// (NHR, RHD, mesh chunk) and the vector-core mesh neither PROD nor 64-bit types (REGISTER_ALG_ATTRS in
// ins_v2_all_reduce_sole_executor.cc:401-431, ins_v2_reduce_scatter_sole_executor.cc:377-476, filtered by
// op_common/selector/cost_table.cc:104-131) and its selector then lands on the host-reduce mesh templates, so
// those combinations fold in the MESH order here too.  Everything else keeps the configured algorithm.
HcclAmdAlgo EffectiveAlgo(const World* w, HcclAmdOpKind kind, HcclDataType dtype, HcclReduceOp op)
{
    const bool isFloat = dtype == HCCL_DATA_TYPE_FP16 || dtype == HCCL_DATA_TYPE_FP32 ||
                         dtype == HCCL_DATA_TYPE_BFP16 || dtype == HCCL_DATA_TYPE_FP64;
    if (w->deterministic == 2 && isFloat && (op == HCCL_REDUCE_SUM || op == HCCL_REDUCE_PROD) && w->n > 2) {
        return HCCL_AMD_ALGO_ORDER_PRESERVED;
    }
    const HcclAmdAlgo algo = w->algo[kind];
    const bool hostOnly = op == HCCL_REDUCE_PROD || dtype == HCCL_DATA_TYPE_INT64 || dtype == HCCL_DATA_TYPE_UINT64 ||
                          dtype == HCCL_DATA_TYPE_FP64;
    if (hostOnly && (algo == HCCL_AMD_ALGO_NHR || algo == HCCL_AMD_ALGO_RHD || algo == HCCL_AMD_ALGO_MESH_CHUNK ||
                     algo == HCCL_AMD_ALGO_AIV_MESH ||
                     (algo == HCCL_AMD_ALGO_RING && kind == HCCL_AMD_OP_REDUCE_SCATTER))) {
        return HCCL_AMD_ALGO_MESH;
    }
    return algo;
}

// Mesh-chunk order: one launch per run of equally long segments.  `nGroup` slices of `len` elements start
// `sliceStride` elements apart from element `base` of every send buffer; slice g is slice firstSlice + g of the
// plan.  The results go to dst[...] + dstBase (+ g * sliceStride when every destination receives every slice).
HcclResult LaunchMeshChunk(World* w, const DevicePlan& plan, const PendingOp& p, ReduceArgs a, uint32_t firstSlice,
                           uint32_t nGroup, uint64_t len, uint64_t sliceStride, bool alignTo4K, hipStream_t s)
{
    const uint32_t n = w->n;
    const uint32_t esz = DataTypeSize(p.dtype);
    const uint32_t segs = n - 1;
    for (const SegmentRun& run : MeshChunkSegments(len, n, esz, alignTo4K)) {
        ReduceArgs r = a;
        for (uint32_t k = 0; k < n; ++k) {
            r.src[k] = static_cast<const uint8_t*>(a.src[k]) + run.first * esz;
            if (a.dst[k] != nullptr) {
                r.dst[k] = static_cast<uint8_t*>(a.dst[k]) + run.first * esz;
            }
        }
        r.prog = plan.dev + (static_cast<uint64_t>(firstSlice) * segs + run.firstSeg) * kDevProgBytes;
        r.progGroupStride = segs;
        r.progSubStride = 1;
        r.nGroup = nGroup;
        r.nSub = run.nSeg;
        r.subLen = run.segLen;
        r.groupLen = run.segLen * (run.nSeg - 1) + run.lastLen;
        r.total = r.groupLen * nGroup;
        r.srcGroupStride = sliceStride;
        r.dstGroupStride = sliceStride;
        HcclResult rc = LaunchOneReduce(w, r, plan, p.dtype, p.op, s);
        if (rc != HCCL_SUCCESS) {
            return rc;
        }
    }
    return HCCL_SUCCESS;
}

HcclResult RunBcast(World* w, BcastCopyArgs& b, hipStream_t s);

// A result that every rank receives, as two kernels per piece: the fold of all ranks into the first rank's recvBuf
// (N reads and one write, the shape of a ReduceScatter launch), then that range, just written and therefore still in
// the last-level cache, to the other recvBufs with one wavefront per destination stream.  Exactly the algorithmic
// traffic, no memory of the library's own, same fold program and same bits as the fused kernel.  Reads and writes
// each run near what the part gives them alone (reads 0.80-0.85 of the HBM peak, writes from one wavefront per
// stream 0.89-0.91), where the fused kernel, whose wavefronts store to every destination after loading from every
// source, reaches 0.70-0.78.  Measured, fp32 SUM in rank order, two kernels / fused:
//   ranks    8 MiB         16 MiB        32 MiB        64 MiB        256 MiB per rank
//     4                  0.62 / 0.62   0.69 / 0.69                 0.78 / 0.78
//     6    0.57 / 0.58   0.66 / 0.63   0.73 / 0.69   0.78 / 0.74   0.82 / 0.79
//     8    0.60 / 0.60   0.68 / 0.62   0.75 / 0.71   0.80 / 0.77   0.82 / 0.76
//    16    0.65 / 0.57   0.74 / 0.58   0.79 / 0.73   0.82 / 0.76   0.83 / 0.74
// (2 and 3 ranks lose: 0.64 / 0.78, 0.76 / 0.77.)  A piece must still be cached when it is read back: 256 MiB pieces
// are the best (1 GiB per rank over 6 ranks: 0.76 / 0.78 / 0.78 with 64 / 128 / 256 MiB, 0.64 with 512 MiB).
bool FoldThenFanOut(const World* w, uint32_t nDst, uint64_t bytes)
{
    if (nDst < 2) {
        return false;
    }
    if (w->twoKernelMode != 2) {
        return w->twoKernelMode == 1;
    }
    return nDst >= 12 ? bytes >= (8ull << 20) : (nDst >= 5 && bytes >= (16ull << 20));
}

// Second kernel of the two-kernel forms: bytes [off, off + bytes) of dst[0], just written, to the same range of
// dst[1 .. nDst).  Destinations that differ from dst[0] modulo 16 take the general copy.
HcclResult FanOutFromFirst(World* w, void* const* dst, uint32_t nDst, uint64_t off, uint64_t bytes, hipStream_t s)
{
    if (nDst < 2 || bytes == 0) {
        return HCCL_SUCCESS;
    }
    FanOutArgs f{};
    f.src = static_cast<const uint8_t*>(dst[0]) + off;
    f.bytes = bytes;
    f.nDst = nDst - 1;
    for (uint32_t k = 1; k < nDst; ++k) {
        f.dst[k - 1] = static_cast<uint8_t*>(dst[k]) + off;
    }
    if (FanOutTakes(f)) {
        HIP_OK(LaunchFanOut(f, s));
        return HCCL_SUCCESS;
    }
    BcastCopyArgs b{};
    b.nSeg = 1;
    b.src[0] = f.src;
    b.len[0] = bytes;
    b.dstOff[0] = 0;
    b.nDst = f.nDst;
    for (uint32_t k = 0; k < f.nDst; ++k) {
        b.dst[k] = f.dst[k];
    }
    return RunBcast(w, b, s);
}

// Launch of a fold whose result [0, a.total) goes to all a.nDst destinations (a.nGroup == 1, a.dstOwn == 0): the
// fused kernel, or fold + fan-out per piece.  Pieces are whole sub-segments while those fit (each has its own fold
// program), and parts of a sub-segment that is longer than a piece.
HcclResult LaunchToAll(World* w, const ReduceArgs& a, const DevicePlan& plan, HcclDataType dtype, HcclReduceOp op,
                       hipStream_t s)
{
    const uint32_t esz = DataTypeSize(dtype);
    if (esz == 0) {
        return HCCL_E_INTERNAL;   // the entry points admit known types only
    }
    if (a.nGroup != 1 || a.dstOwn != 0 || a.varGroups != 0 || !FoldThenFanOut(w, a.nDst, a.total * esz)) {
        ReduceArgs fused = a;
        return LaunchOneReduce(w, fused, plan, dtype, op, s);
    }
    const uint64_t pieceEl = std::max<uint64_t>(1, w->pieceBytes / esz);
    auto piece = [&](uint32_t firstSub, uint32_t nSub, uint64_t begin, uint64_t len) -> HcclResult {
        if (len == 0) {
            return HCCL_SUCCESS;
        }
        ReduceArgs r = a;
        for (uint32_t k = 0; k < w->n; ++k) {
            r.src[k] = static_cast<const uint8_t*>(a.src[k]) + begin * esz;
        }
        for (uint32_t k = 0; k < static_cast<uint32_t>(kMaxRanks); ++k) {
            r.dst[k] = nullptr;
        }
        uint8_t* first = static_cast<uint8_t*>(a.dst[0]) + begin * esz;
        r.dst[0] = first;
        r.nDst = 1;
        r.prog = a.prog + static_cast<uint64_t>(firstSub) * a.progSubStride * kDevProgBytes;
        r.nSub = nSub;
        r.total = r.groupLen = len;
        if (nSub == 1) {
            r.subLen = len;
        }
        HcclResult rc = LaunchOneReduce(w, r, plan, dtype, op, s);
        if (rc != HCCL_SUCCESS) {
            return rc;
        }
        return FanOutFromFirst(w, a.dst, a.nDst, begin * esz, len * esz, s);
    };
    uint32_t heldFirst = 0;     // sub-segments [heldFirst, c) wait for their launch
    uint64_t heldBegin = 0;
    uint64_t heldLen = 0;
    for (uint32_t c = 0; c < a.nSub; ++c) {
        const uint64_t sBeg = static_cast<uint64_t>(c) * a.subLen;
        uint64_t sEnd = (c == a.nSub - 1) ? a.total : sBeg + a.subLen;
        sEnd = sEnd < a.total ? sEnd : a.total;
        const uint64_t len = sEnd > sBeg ? sEnd - sBeg : 0;
        if (heldLen + len > pieceEl && heldLen != 0) {
            HcclResult rc = piece(heldFirst, c - heldFirst, heldBegin, heldLen);
            if (rc != HCCL_SUCCESS) {
                return rc;
            }
            heldLen = 0;
        }
        if (len > pieceEl) {
            for (uint64_t at = 0; at < len; at += pieceEl) {
                HcclResult rc = piece(c, 1, sBeg + at, std::min(pieceEl, len - at));
                if (rc != HCCL_SUCCESS) {
                    return rc;
                }
            }
            continue;
        }
        if (heldLen == 0) {
            heldFirst = c;
            heldBegin = sBeg;
        }
        heldLen += len;
    }
    if (heldLen != 0) {
        return piece(heldFirst, a.nSub - heldFirst, heldBegin, heldLen);
    }
    return HCCL_SUCCESS;
}

HcclResult RunAllReduce(World* w, PendingOp& p, hipStream_t s)
{
    const uint32_t n = w->n;
    HcclAmdAlgo algo = EffectiveAlgo(w, HCCL_AMD_OP_ALL_REDUCE, p.dtype, p.op);
    // A world with level-0 groups runs the step-driven orders in two levels: a mesh ReduceScatter inside every
    // group, the configured template between the groups (reference
    // ins_v2_all_reduce_sequence_executor_aicpu.cc:592-852).  The types the reference reduces on the host take its
    // host-reduce template between the groups, which folds the own share first (EffectiveAlgo has turned their
    // RHD / NHR into MESH; a configured sequence{mesh, nhr_aicpu_reduce} asks for the same).
    const uint32_t level0 = w->level0;
    const HcclAmdAlgo configured = w->algo[HCCL_AMD_OP_ALL_REDUCE];
    const bool stepDriven = configured == HCCL_AMD_ALGO_RHD || configured == HCCL_AMD_ALGO_NHR;
    const bool twoLevel = level0 > 1 && level0 < n && w->allReduceSequence != 0 &&
                          (algo == HCCL_AMD_ALGO_RHD || algo == HCCL_AMD_ALGO_NHR ||
                           (algo == HCCL_AMD_ALGO_MESH && (stepDriven || w->allReduceSequence == 1)));
    DevicePlan plan;
    HcclResult rc = GetDevicePlan(w, HCCL_AMD_OP_ALL_REDUCE, algo, &plan, twoLevel ? level0 : 1);
    if (rc != HCCL_SUCCESS) {
        return rc;
    }
    const uint32_t esz = DataTypeSize(p.dtype);
    ReduceArgs a{};
    for (uint32_t r = 0; r < n; ++r) {
        a.src[r] = p.ranks[r].send;
        a.dst[r] = p.ranks[r].recv;
    }
    a.prog = plan.dev;
    a.nDst = n;
    a.dstOwn = 0;
    a.nGroup = 1;
    if (plan.nProg == 1) {
        a.total = a.groupLen = a.subLen = p.count;
        a.nSub = 1;
        return LaunchToAll(w, a, plan, p.dtype, p.op, s);
    }
    if (algo == HCCL_AMD_ALGO_MESH_CHUNK) {
        // Slices of ceil(len / n) elements, short or empty towards the end (reference
        // ins_temp_all_reduce_mesh_1D_two_shot_mesh_chunk.cc:86-112); the executor loops over half of the
        // staging buffer (:55-62, ins_v2_all_reduce_sole_executor.cc:241-300).
        uint64_t maxPerLoop = p.count;
        if (w->cclBytes != 0) {
            maxPerLoop = SoleMaxCountPerLoop(w->cclBytes, 2, esz);
            if (maxPerLoop == 0) {
                return HCCL_E_INTERNAL;
            }
        }
        for (uint64_t done = 0; done < p.count;) {
            const uint64_t len = std::min(p.count - done, maxPerLoop);
            const uint64_t slice = (len + n - 1) / n;
            const uint32_t nFull = static_cast<uint32_t>(len / slice);
            for (uint32_t r = 0; r < n; ++r) {
                a.src[r] = static_cast<const uint8_t*>(p.ranks[r].send) + done * esz;
                a.dst[r] = static_cast<uint8_t*>(p.ranks[r].recv) + done * esz;
            }
            if (FoldThenFanOut(w, n, len * esz) && slice * esz <= w->pieceBytes && (n >= 8 || w->twoKernelMode == 1)) {
                // Fold + fan-out per piece of whole slices: the launches of a piece write rank 0's recvBuf only,
                // then that range goes to the other recvBufs (fp32, 8 ranks of 256 MiB: 0.74 -> 0.81 of the HBM peak,
                // 16 ranks of 64 MiB: 0.71 -> 0.79; six ranks lose, 0.74 -> 0.71, and keep the fused kernel).
                const uint64_t rest = len - static_cast<uint64_t>(nFull) * slice;
                const uint32_t perPiece = static_cast<uint32_t>(std::max<uint64_t>(1, w->pieceBytes / esz / slice));
                for (uint32_t g0 = 0; g0 < nFull; g0 += perPiece) {   // nFull >= 1: a slice is never longer than the loop
                    const uint32_t g1 = std::min(nFull, g0 + perPiece);
                    const uint64_t begin = static_cast<uint64_t>(g0) * slice;
                    uint64_t pieceLen = static_cast<uint64_t>(g1 - g0) * slice;
                    ReduceArgs f = a;
                    f.nDst = 1;
                    for (uint32_t r = 0; r < n; ++r) {
                        f.src[r] = static_cast<const uint8_t*>(a.src[r]) + begin * esz;
                        f.dst[r] = r == 0 ? static_cast<uint8_t*>(a.dst[0]) + begin * esz : nullptr;
                    }
                    rc = LaunchMeshChunk(w, plan, p, f, g0, g1 - g0, slice, slice, false, s);
                    if (rc != HCCL_SUCCESS) {
                        return rc;
                    }
                    if (g1 == nFull && rest != 0) {   // the short last slice rides with the last piece
                        ReduceArgs t = a;
                        t.nDst = 1;
                        for (uint32_t r = 0; r < n; ++r) {
                            t.src[r] = static_cast<const uint8_t*>(a.src[r]) + static_cast<uint64_t>(nFull) * slice * esz;
                            t.dst[r] = r == 0 ? static_cast<uint8_t*>(a.dst[0]) + static_cast<uint64_t>(nFull) * slice * esz : nullptr;
                        }
                        rc = LaunchMeshChunk(w, plan, p, t, nFull, 1, rest, 0, false, s);
                        if (rc != HCCL_SUCCESS) {
                            return rc;
                        }
                        pieceLen += rest;
                    }
                    rc = FanOutFromFirst(w, a.dst, n, begin * esz, pieceLen * esz, s);
                    if (rc != HCCL_SUCCESS) {
                        return rc;
                    }
                }
                done += len;
                continue;
            }
            if (nFull != 0) {
                rc = LaunchMeshChunk(w, plan, p, a, 0, nFull, slice, slice, false, s);
                if (rc != HCCL_SUCCESS) {
                    return rc;
                }
            }
            const uint64_t rest = len - static_cast<uint64_t>(nFull) * slice;
            if (rest != 0) {
                for (uint32_t r = 0; r < n; ++r) {
                    a.src[r] = static_cast<const uint8_t*>(a.src[r]) + static_cast<uint64_t>(nFull) * slice * esz;
                    a.dst[r] = static_cast<uint8_t*>(a.dst[r]) + static_cast<uint64_t>(nFull) * slice * esz;
                }
                rc = LaunchMeshChunk(w, plan, p, a, nFull, 1, rest, 0, false, s);
                if (rc != HCCL_SUCCESS) {
                    return rc;
                }
            }
            done += len;
        }
        return HCCL_SUCCESS;
    }
    a.nSub = n;
    a.progSubStride = 1;
    // One launch per loop of the reference's executor: elements [done, done + len) cut into n sub-segments of
    // `unit` elements, the last one taking what the others leave.
    auto launchLoop = [&](uint64_t done, uint64_t len, uint64_t unit) {
        for (uint32_t r = 0; r < n; ++r) {
            a.src[r] = static_cast<const uint8_t*>(p.ranks[r].send) + done * esz;
            a.dst[r] = static_cast<uint8_t*>(p.ranks[r].recv) + done * esz;
        }
        a.total = a.groupLen = len;
        a.subLen = unit;
        return LaunchToAll(w, a, plan, p.dtype, p.op, s);
    };
    if (twoLevel && algo != HCCL_AMD_ALGO_RHD) {
        // Between the groups NHR, or the host-reduce fold: every loop is cut into level0 chunks of floor(len / level0)
        // elements, the last chunk taking the rest, and every chunk into n / level0 sub-slices the same way (reference
        // ins_v2_all_reduce_sequence_executor_aicpu.cc:413-415, 445-455).  The loops hold what fits half the staging
        // buffer, floored to 128 bytes and to a multiple of n elements (:653-656).
        const uint32_t level1 = n / level0;
        uint64_t maxPerLoop = p.count;
        if (w->cclBytes != 0) {
            maxPerLoop = w->cclBytes / 2 / 128 * 128 / esz / n * n;
            if (maxPerLoop == 0) {
                Log(1, "AllReduce: the staging buffer of %llu bytes holds no loop of the two-level order",
                    static_cast<unsigned long long>(w->cclBytes));
                return HCCL_E_INTERNAL;
            }
        }
        for (uint64_t done = 0; done < p.count;) {
            const uint64_t len = std::min(p.count - done, maxPerLoop);
            const uint64_t chunk = len / level0;
            if (chunk * level0 == len && chunk % level1 == 0 && chunk != 0) {
                // every sub-slice equally long: one launch over the n units of the loop, unit i * level1 + j being
                // sub-slice j of chunk i
                a.nSub = n;
                a.prog = plan.dev;
                rc = launchLoop(done, len, chunk / level1);
                if (rc != HCCL_SUCCESS) {
                    return rc;
                }
                done += len;
                continue;
            }
            a.nSub = level1;
            for (uint32_t i = 0; i < level0; ++i) {
                const uint64_t begin = done + static_cast<uint64_t>(i) * chunk;
                const uint64_t cur = i == level0 - 1 ? len - static_cast<uint64_t>(i) * chunk : chunk;
                if (cur == 0) {
                    continue;
                }
                for (uint32_t r = 0; r < n; ++r) {
                    a.src[r] = static_cast<const uint8_t*>(p.ranks[r].send) + begin * esz;
                    a.dst[r] = static_cast<uint8_t*>(p.ranks[r].recv) + begin * esz;
                }
                a.prog = plan.dev + static_cast<uint64_t>(i) * level1 * kDevProgBytes;
                a.total = a.groupLen = cur;
                a.subLen = cur / level1;
                if (a.subLen == 0) {
                    // fewer elements than sub-slices: all of them belong to the last sub-slice
                    a.prog = plan.dev + (static_cast<uint64_t>(i) * level1 + level1 - 1) * kDevProgBytes;
                    a.nSub = 1;
                    a.subLen = cur;
                }
                rc = LaunchToAll(w, a, plan, p.dtype, p.op, s);
                a.nSub = level1;
                if (rc != HCCL_SUCCESS) {
                    return rc;
                }
            }
            done += len;
        }
        return HCCL_SUCCESS;
    }
    if (algo == HCCL_AMD_ALGO_RHD) {
        // (With level-0 groups the frame is the same: unit u = i * (n / level0) + j is sub-slice j of chunk i, and
        // the remainder shorter than n is padded to one element per unit; only the programs differ.)
        // Whole frames of n uniform units while they last, then a remainder shorter than n with one element per
        // unit (reference ins_v2_all_reduce_sequence_rhd_tail.h:94-113); a bounded staging buffer limits the
        // frames one loop holds.
        uint64_t maxPerLoop = ~0ull / 2 / n * n;
        if (w->cclBytes != 0) {
            rc = RhdMaxCountPerLoop(w->cclBytes, p.count, n, esz, &maxPerLoop);
            if (rc != HCCL_SUCCESS) {
                Log(1, "AllReduce: the staging buffer of %llu bytes holds no loop of the RHD order",
                    static_cast<unsigned long long>(w->cclBytes));
                return rc;
            }
        }
        for (uint64_t done = 0; done < p.count;) {
            const uint64_t valid = RhdSelectLoopCount(p.count - done, maxPerLoop, n);
            rc = launchLoop(done, valid, valid >= n ? valid / n : 1);
            if (rc != HCCL_SUCCESS) {
                return rc;
            }
            done += valid;
        }
        return HCCL_SUCCESS;
    }
    if (algo == HCCL_AMD_ALGO_NHR) {
        // Slices of floor(len / n) elements, the last slice takes the rest (reference
        // ins_temp_all_reduce_nhr.cc:214-216); the executor loops over the staging buffer, which this template
        // uses once (scratch multiple 1, reference ins_temp_all_reduce_nhr.cc:65-71,
        // ins_v2_all_reduce_sole_executor.cc:241-300).
        uint64_t maxPerLoop = p.count;
        if (w->cclBytes != 0) {
            maxPerLoop = SoleMaxCountPerLoop(w->cclBytes, 1, esz);
            if (maxPerLoop == 0) {
                Log(1, "AllReduce: the staging buffer of %llu bytes holds no element",
                    static_cast<unsigned long long>(w->cclBytes));
                return HCCL_E_INTERNAL;
            }
        }
        for (uint64_t done = 0; done < p.count;) {
            const uint64_t len = std::min(p.count - done, maxPerLoop);
            rc = launchLoop(done, len, len / n);
            if (rc != HCCL_SUCCESS) {
                return rc;
            }
            done += len;
        }
        return HCCL_SUCCESS;
    }
    // Symmetric two-shot: slices of ceil(count / n) elements (reference two_shot.cc:184), always in one loop
    // (reference ins_v2_all_reduce_sole_executor.cc:273-282).
    return launchLoop(0, p.count, (p.count + n - 1) / n);
}

HcclResult RunReduceScatter(World* w, PendingOp& p, hipStream_t s)
{
    const uint32_t n = w->n;
    HcclAmdAlgo algo = EffectiveAlgo(w, HCCL_AMD_OP_REDUCE_SCATTER, p.dtype, p.op);
    DevicePlan plan;
    HcclResult rc = GetDevicePlan(w, HCCL_AMD_OP_REDUCE_SCATTER, algo, &plan);
    if (rc != HCCL_SUCCESS) {
        return rc;
    }
    ReduceArgs a{};
    for (uint32_t r = 0; r < n; ++r) {
        a.src[r] = p.ranks[r].send;
        a.dst[r] = p.ranks[r].recv;
    }
    a.prog = plan.dev;
    a.nDst = 1;
    a.dstOwn = 1;
    if (algo == HCCL_AMD_ALGO_MESH_CHUNK) {
        // The executor loops over the staging buffer, of which this template keeps n - 1 slots (reference
        // ins_temp_reduce_scatter_mesh_1D_meshchunk.cc:119-125, ins_v2_reduce_scatter_sole_executor.cc:212-277);
        // every loop cuts its share of each rank's output into segments of its own.
        const uint32_t esz = DataTypeSize(p.dtype);
        uint64_t maxPerLoop = p.count;
        if (w->cclBytes != 0) {
            maxPerLoop = SoleMaxCountPerLoop(w->cclBytes, n - 1, esz);
            if (maxPerLoop == 0) {
                return HCCL_E_INTERNAL;
            }
        }
        for (uint64_t done = 0; done < p.count;) {
            const uint64_t len = std::min(p.count - done, maxPerLoop);
            for (uint32_t r = 0; r < n; ++r) {
                a.src[r] = static_cast<const uint8_t*>(p.ranks[r].send) + done * esz;
                a.dst[r] = static_cast<uint8_t*>(p.ranks[r].recv) + done * esz;
            }
            rc = LaunchMeshChunk(w, plan, p, a, 0, n, len, p.count, true, s);
            if (rc != HCCL_SUCCESS) {
                return rc;
            }
            done += len;
        }
        return HCCL_SUCCESS;
    }
    a.nGroup = n;
    a.groupLen = p.count;                  // input slice stride = recvCount (reference
    a.srcGroupStride = p.count;            // ins_v2_reduce_scatter_sole_executor.cc:260)
    a.total = static_cast<uint64_t>(n) * p.count;
    if (plan.segmentsAreSubs && plan.nProg > 1) {
        a.nSub = n;                        // vector-core mesh: output cut into n chunks
        a.subLen = p.count / n;
        a.progSubStride = 1;
    } else {
        a.nSub = 1;
        a.subLen = p.count;
        a.progGroupStride = plan.nProg > 1 ? 1 : 0;
    }
    return LaunchOneReduce(w, a, plan, p.dtype, p.op, s);
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
// Measured over rotating buffer sets, two kernels / one, fraction of the HBM peak: AllGather of 16 x 64 MiB
// 0.84 / 0.69, 16 x 16 MiB 0.76 / 0.68, 8 x 128 MiB 0.77 / 0.71, 8 x 8 MiB 0.76 / 0.69, 6 x 32 MiB 0.72 / 0.74,
// 4 x 64 MiB 0.67 / 0.77; Broadcast of 128 MiB to 15 ranks 0.78 / 0.68, to 7 ranks 0.78 / 0.73 (16 MiB: 0.61 /
// 0.65), to 5 ranks 0.72 / 0.77.  `bytes` is what every destination receives.
bool GatherThenFanOut(const World* w, uint32_t nDst, uint64_t bytes)
{
    if (nDst < 3) {
        return false;
    }
    if (w->copyTwoKernelMode != 2) {
        return w->copyTwoKernelMode == 1;
    }
    return nDst >= 7 && bytes >= (48ull << 20);
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
    if (!GatherThenFanOut(w, b.nDst, total)) {
        return RunBcast(w, b, s);
    }
    for (uint32_t d = 1; d < b.nDst; ++d) {
        if (((reinterpret_cast<uint64_t>(b.dst[d]) ^ reinterpret_cast<uint64_t>(b.dst[0])) & 15u) != 0) {
            return RunBcast(w, b, s);
        }
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
            HIP_OK(LaunchFanOut(f, s));
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

// ReduceScatterV, mesh order: rank k's output = in_k[displs[k] ..] first, then the other ranks ascending
// (reference ins_temp_reduce_scatter_v_mesh_1D.cc:109-162).  Every rank must pass the same counts / displs.
HcclResult RunReduceScatterV(World* w, PendingOp& p, hipStream_t s)
{
    const uint32_t n = w->n;
    const std::vector<uint64_t>& ref = p.ranks[0].var;   // counts | displs | recvCount
    uint64_t longest = 0;
    for (uint32_t r = 0; r < n; ++r) {
        const std::vector<uint64_t>& v = p.ranks[r].var;
        if (memcmp(v.data(), ref.data(), 2 * n * sizeof(uint64_t)) != 0) {
            Log(1, "ReduceScatterV: rank %u passed sendCounts / sendDispls that differ from rank 0", r);
            return HCCL_E_PARA;
        }
        if (v[2 * n] != ref[r]) {
            Log(1, "ReduceScatterV: rank %u recvCount %llu != sendCounts[%u] %llu", r, (unsigned long long)v[2 * n], r,
                (unsigned long long)ref[r]);
            return HCCL_E_PARA;
        }
        if (ref[r] != 0 && (p.ranks[r].send == nullptr || p.ranks[r].recv == nullptr)) {
            return HCCL_E_PTR;
        }
        longest = ref[r] > longest ? ref[r] : longest;
    }
    if (longest == 0) {
        return HCCL_SUCCESS;
    }
    const bool meshChunk = EffectiveAlgo(w, HCCL_AMD_OP_REDUCE_SCATTER, p.dtype, p.op) == HCCL_AMD_ALGO_MESH_CHUNK;
    DevicePlan plan;
    HcclResult rc = GetDevicePlan(w, HCCL_AMD_OP_REDUCE_SCATTER, meshChunk ? HCCL_AMD_ALGO_MESH_CHUNK : HCCL_AMD_ALGO_MESH,
                                  &plan);
    if (rc != HCCL_SUCCESS) {
        return rc;
    }
    if (meshChunk) {
        // Always one loop; the reference refuses a count its single accumulation slot cannot hold (reference
        // ins_v2_reduce_scatter_v_sole_executor.cc:158-171, ins_temp_reduce_scatter_v_mesh_1D_meshchunk.cc:49-55).
        const uint32_t esz = DataTypeSize(p.dtype);
        if (w->cclBytes != 0 && longest > SoleMaxCountPerLoop(w->cclBytes, 1, esz)) {
            Log(1, "ReduceScatterV: %llu elements exceed the staging buffer of %llu bytes in the mesh-chunk order",
                static_cast<unsigned long long>(longest), static_cast<unsigned long long>(w->cclBytes));
            return HCCL_E_NOT_SUPPORT;
        }
        for (uint32_t k = 0; k < n; ++k) {
            if (ref[k] == 0) {
                continue;
            }
            ReduceArgs a{};
            for (uint32_t r = 0; r < n; ++r) {
                a.src[r] = static_cast<const uint8_t*>(p.ranks[r].send) + ref[n + k] * esz;
            }
            a.dst[0] = p.ranks[k].recv;
            a.nDst = 1;
            a.dstOwn = 1;
            rc = LaunchMeshChunk(w, plan, p, a, k, 1, ref[k], 0, true, s);
            if (rc != HCCL_SUCCESS) {
                return rc;
            }
        }
        return HCCL_SUCCESS;
    }
    ReduceArgs a{};
    for (uint32_t r = 0; r < n; ++r) {
        a.src[r] = p.ranks[r].send;
        a.dst[r] = p.ranks[r].recv;
        a.groupLenV[r] = ref[r];
        a.groupOffV[r] = ref[n + r];
    }
    a.prog = plan.dev;
    a.varGroups = 1;
    a.nDst = 1;
    a.dstOwn = 1;
    a.nGroup = n;
    a.nSub = 1;
    a.groupLen = a.subLen = longest;
    a.total = static_cast<uint64_t>(n) * longest;
    a.progGroupStride = plan.nProg > 1 ? 1 : 0;
    return LaunchOneReduce(w, a, plan, p.dtype, p.op, s);
}

// Reduce.  MESH: out_root = in_0, then in_1 .. in_{N-1} folded ascending (reference reduce_mesh_1D.cc:268-300):
// the AllReduce rank-order program with the root's recvBuf as only destination.  MESH_TWO_SHOT: every loop of the
// executor deals its elements into N slices, the first len mod N one element longer, and slice k folds rank k's
// input first (reference reduce_mesh_1D_two_shot.cc:138-162, 228-265; N staging slots, :79-84,
// reduce_sole_executor.cc:178-232).
HcclResult RunReduce(World* w, PendingOp& p, hipStream_t s)
{
    const uint32_t n = w->n;
    if (p.ranks[p.root].recv == nullptr) {
        return HCCL_E_PTR;
    }
    const bool twoShot = w->algo[HCCL_AMD_OP_REDUCE] == HCCL_AMD_ALGO_MESH_TWO_SHOT;
    DevicePlan plan;
    HcclResult rc = GetDevicePlan(w, HCCL_AMD_OP_REDUCE, twoShot ? HCCL_AMD_ALGO_MESH_TWO_SHOT : HCCL_AMD_ALGO_MESH,
                                  &plan);
    if (rc != HCCL_SUCCESS) {
        return rc;
    }
    ReduceArgs a{};
    for (uint32_t r = 0; r < n; ++r) {
        a.src[r] = p.ranks[r].send;
    }
    a.dst[0] = p.ranks[p.root].recv;
    a.prog = plan.dev;
    a.nDst = 1;
    a.dstOwn = 0;
    a.nGroup = 1;
    if (!twoShot) {
        a.nSub = 1;
        a.total = a.groupLen = a.subLen = p.count;
        return LaunchOneReduce(w, a, plan, p.dtype, p.op, s);
    }
    const uint32_t esz = DataTypeSize(p.dtype);
    uint64_t maxPerLoop = p.count;
    if (w->cclBytes != 0) {
        maxPerLoop = SoleMaxCountPerLoop(w->cclBytes, n, esz);
        if (maxPerLoop == 0) {
            return HCCL_E_INTERNAL;
        }
    }
    a.progSubStride = 1;
    for (uint64_t done = 0; done < p.count;) {
        const uint64_t len = std::min(p.count - done, maxPerLoop);
        const uint64_t base = len / n;
        const uint32_t nBig = static_cast<uint32_t>(len % n);
        // two runs of equally long slices: nBig of base + 1 elements, then n - nBig of base
        const uint64_t runFirst[2] = {0, static_cast<uint64_t>(nBig) * (base + 1)};
        const uint32_t runSlices[2] = {nBig, n - nBig};
        const uint64_t runLen[2] = {base + 1, base};
        for (int run = 0; run < 2; ++run) {
            if (runSlices[run] == 0 || runLen[run] == 0) {
                continue;
            }
            const uint64_t at = (done + runFirst[run]) * esz;
            for (uint32_t r = 0; r < n; ++r) {
                a.src[r] = static_cast<const uint8_t*>(p.ranks[r].send) + at;
            }
            a.dst[0] = static_cast<uint8_t*>(p.ranks[p.root].recv) + at;
            a.prog = plan.dev + static_cast<uint64_t>(run == 0 ? 0 : nBig) * kDevProgBytes;
            a.nSub = runSlices[run];
            a.subLen = runLen[run];
            a.total = a.groupLen = runLen[run] * runSlices[run];
            rc = LaunchOneReduce(w, a, plan, p.dtype, p.op, s);
            if (rc != HCCL_SUCCESS) {
                return rc;
            }
        }
        done += len;
    }
    return HCCL_SUCCESS;
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
                  void* recv, hipStream_t stream, std::vector<uint64_t>&& var, uint32_t root = 0, bool noAlloc = false)
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

inline HcclResult RejectIfKnown(const CommRef& ref, OpType type, HcclResult rc) { return Reject(ref, type, rc); }

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

}  // namespace
}  // namespace hccl_amd

using namespace hccl_amd;

// ---------------------------------------------------------------------------------------------
// extern "C" surface
// ---------------------------------------------------------------------------------------------
#define CHK_PTR(p, what)                               \
    do {                                               \
        if ((p) == nullptr) {                          \
            Log(1, "%s: %s is nullptr", __func__, what); \
            return HCCL_E_PTR;                         \
        }                                              \
    } while (0)

#define CHK_RET(expr)                 \
    do {                              \
        HcclResult rc_ = (expr);      \
        if (rc_ != HCCL_SUCCESS) {    \
            return rc_;               \
        }                             \
    } while (0)

// The same two checks inside a collective's entry point, where `ref` is the looked-up communicator: a call that
// fails them keeps its place in the rank's sequence of collectives when the communicator is a live one (see
// Reject); the code returned is the same either way.
#define CHK_RET_Q(type, expr)                       \
    do {                                            \
        HcclResult rc_ = (expr);                    \
        if (rc_ != HCCL_SUCCESS) {                  \
            return RejectIfKnown(ref, type, rc_);   \
        }                                           \
    } while (0)

#define CHK_PTR_Q(type, p, what)                          \
    do {                                                  \
        if ((p) == nullptr) {                             \
            Log(1, "%s: %s is nullptr", __func__, what);  \
            return RejectIfKnown(ref, type, HCCL_E_PTR);  \
        }                                                 \
    } while (0)

namespace {

// Common tail of every entry point: the environment verdict, then the rendezvous.
HcclResult SubmitWithReady(const CommRef& ref, OpType type, HcclDataType dtype, HcclReduceOp op, uint64_t count,
                           const void* send, void* recv, aclrtStream stream, std::vector<uint64_t>&& var,
                           uint32_t root = 0, bool noAlloc = false)
{
    if (ref.c->world->envInvalid) {
        return HCCL_E_PARA;   // the reference's environment parsing fails every entry point the same way
    }
    return Submit(ref, type, dtype, op, count, send, recv, static_cast<hipStream_t>(stream), std::move(var), root,
                  noAlloc);
}

// HcclAlltoAllV and its allocation-free variant: reference src/ops/all_to_all_v/all_to_all_v.cc:105-129, 517-598.
// Like the reference, only recvType is consulted for the element size.
HcclResult AlltoAllVEntry(const char* name, const void* sendBuf, const void* sendCounts, const void* sdispls,
                          const void* recvBuf, const void* recvCounts, const void* rdispls, HcclDataType recvType,
                          HcclComm comm, aclrtStream stream, bool noAlloc)
{
    CommRef ref = AsComm(comm);   // looked up first, so that a call that fails any check below keeps its place
#define CHK_ENTRY_PTR(p, what)                                \
    do {                                                      \
        if ((p) == nullptr) {                                 \
            Log(1, "%s: %s is nullptr", name, what);  \
            return RejectIfKnown(ref, OpType::ALL_TO_ALL_V, HCCL_E_PTR); \
        }                                                     \
    } while (0)
    CHK_ENTRY_PTR(comm, "comm");
    CHK_ENTRY_PTR(sendCounts, "sendCounts");
    CHK_ENTRY_PTR(sdispls, "sdispls");
    CHK_ENTRY_PTR(recvCounts, "recvCounts");
    CHK_ENTRY_PTR(rdispls, "rdispls");
    CHK_ENTRY_PTR(stream, "stream");
    if (sendBuf != nullptr && recvBuf != nullptr && sendBuf == recvBuf) {
        Log(1, "%s: sendBuf and recvBuf cannot be the same", name);
        return RejectIfKnown(ref, OpType::ALL_TO_ALL_V, HCCL_E_PARA);
    }
    Comm* c = ref.c;
    if (c == nullptr) {
        Log(1, "%s: comm is not a live communicator", name);
        return RejectIfKnown(ref, OpType::ALL_TO_ALL_V, HCCL_E_PARA);
    }
    const uint32_t n = c->world->n;
    const uint64_t* sc = static_cast<const uint64_t*>(sendCounts);
    const uint64_t* rc = static_cast<const uint64_t*>(recvCounts);
    bool sendZero = true, recvZero = true;
    uint64_t maxCount = 0;
    for (uint32_t i = 0; i < n; ++i) {
        sendZero = sendZero && sc[i] == 0;
        recvZero = recvZero && rc[i] == 0;
        maxCount = sc[i] > maxCount ? sc[i] : maxCount;
        maxCount = rc[i] > maxCount ? rc[i] : maxCount;
    }
    if ((!sendZero && sendBuf == nullptr) || (!recvZero && recvBuf == nullptr)) {
        Log(1, "%s: %s is nullptr", name, (!sendZero && sendBuf == nullptr) ? "sendBuf" : "recvBuf");
        return RejectIfKnown(ref, OpType::ALL_TO_ALL_V, HCCL_E_PTR);
    }
#undef CHK_ENTRY_PTR
    CHK_RET_Q(OpType::ALL_TO_ALL_V, CheckUserRank(c));
    CHK_RET_Q(OpType::ALL_TO_ALL_V, CheckCount(maxCount));
    CHK_RET_Q(OpType::ALL_TO_ALL_V, CheckDataType(recvType, false));
    std::vector<uint64_t> var(4 * n);
    memcpy(var.data(), sc, n * sizeof(uint64_t));
    memcpy(var.data() + n, rc, n * sizeof(uint64_t));
    memcpy(var.data() + 2 * n, sdispls, n * sizeof(uint64_t));
    memcpy(var.data() + 3 * n, rdispls, n * sizeof(uint64_t));
    return SubmitWithReady(ref, OpType::ALL_TO_ALL_V, recvType, HCCL_REDUCE_RESERVED, 0, sendBuf,
                           const_cast<void*>(recvBuf), stream, std::move(var), 0, noAlloc);
}

}  // namespace

extern "C" {

HcclResult HcclAllReduce(void* sendBuf, void* recvBuf, uint64_t count, HcclDataType dataType, HcclReduceOp op,
                         HcclComm comm, aclrtStream stream)
{
    CommRef ref = AsComm(comm);   // looked up first, so that a call that fails any check below keeps its place
    // Order of checks: reference src/ops/all_reduce/all_reduce.cc:41, 111-161.
    if (count == 0) {
        return HCCL_SUCCESS;
    }
    CHK_PTR_Q(OpType::ALL_REDUCE, stream, "stream");
    CHK_PTR_Q(OpType::ALL_REDUCE, comm, "comm");
    CHK_PTR_Q(OpType::ALL_REDUCE, sendBuf, "sendBuf");
    CHK_PTR_Q(OpType::ALL_REDUCE, recvBuf, "recvBuf");
    Comm* c = ref.c;
    if (c == nullptr) {
        Log(1, "HcclAllReduce: comm is not a live communicator");
        return RejectIfKnown(ref, OpType::ALL_REDUCE, HCCL_E_PARA);
    }
    CHK_RET_Q(OpType::ALL_REDUCE, CheckUserRank(c));
    CHK_RET_Q(OpType::ALL_REDUCE, CheckCount(count));
    CHK_RET_Q(OpType::ALL_REDUCE, CheckDataType(dataType, true));
    CHK_RET_Q(OpType::ALL_REDUCE, CheckReduceOp(dataType, op));
    return SubmitWithReady(ref, OpType::ALL_REDUCE, dataType, op, count, sendBuf, recvBuf, stream, {});
}

HcclResult HcclReduceScatter(void* sendBuf, void* recvBuf, uint64_t recvCount, HcclDataType dataType,
                             HcclReduceOp op, HcclComm comm, aclrtStream stream)
{
    CommRef ref = AsComm(comm);   // looked up first, so that a call that fails any check below keeps its place
    // Reference src/ops/reduce_scatter/reduce_scatter.cc:48-62.
    if (recvCount == 0) {
        return HCCL_SUCCESS;
    }
    CHK_PTR_Q(OpType::REDUCE_SCATTER, stream, "stream");
    CHK_PTR_Q(OpType::REDUCE_SCATTER, comm, "comm");
    CHK_PTR_Q(OpType::REDUCE_SCATTER, sendBuf, "sendBuf");
    CHK_PTR_Q(OpType::REDUCE_SCATTER, recvBuf, "recvBuf");
    Comm* c = ref.c;
    if (c == nullptr) {
        Log(1, "HcclReduceScatter: comm is not a live communicator");
        return RejectIfKnown(ref, OpType::REDUCE_SCATTER, HCCL_E_PARA);
    }
    CHK_RET_Q(OpType::REDUCE_SCATTER, CheckUserRank(c));
    CHK_RET_Q(OpType::REDUCE_SCATTER, CheckCount(recvCount));
    CHK_RET_Q(OpType::REDUCE_SCATTER, CheckDataType(dataType, true));
    CHK_RET_Q(OpType::REDUCE_SCATTER, CheckReduceOp(dataType, op));
    return SubmitWithReady(ref, OpType::REDUCE_SCATTER, dataType, op, recvCount, sendBuf, recvBuf, stream, {});
}

HcclResult HcclAllGather(void* sendBuf, void* recvBuf, uint64_t sendCount, HcclDataType dataType, HcclComm comm,
                         aclrtStream stream)
{
    CommRef ref = AsComm(comm);   // looked up first, so that a call that fails any check below keeps its place
    // Reference src/ops/all_gather/all_gather.cc:37, 118-149.
    if (sendCount == 0) {
        return HCCL_SUCCESS;
    }
    CHK_PTR_Q(OpType::ALL_GATHER, stream, "stream");
    CHK_PTR_Q(OpType::ALL_GATHER, comm, "comm");
    CHK_PTR_Q(OpType::ALL_GATHER, sendBuf, "sendBuf");
    CHK_PTR_Q(OpType::ALL_GATHER, recvBuf, "recvBuf");
    Comm* c = ref.c;
    if (c == nullptr) {
        Log(1, "HcclAllGather: comm is not a live communicator");
        return RejectIfKnown(ref, OpType::ALL_GATHER, HCCL_E_PARA);
    }
    CHK_RET_Q(OpType::ALL_GATHER, CheckCount(sendCount));
    CHK_RET_Q(OpType::ALL_GATHER, CheckDataType(dataType, false));
    CHK_RET_Q(OpType::ALL_GATHER, CheckUserRank(c));
    return SubmitWithReady(ref, OpType::ALL_GATHER, dataType, HCCL_REDUCE_RESERVED, sendCount, sendBuf, recvBuf, stream,
                           {});
}

HcclResult HcclAllGatherV(void* sendBuf, uint64_t sendCount, void* recvBuf, const void* recvCounts,
                          const void* recvDispls, HcclDataType dataType, HcclComm comm, aclrtStream stream)
{
    CommRef ref = AsComm(comm);   // looked up first, so that a call that fails any check below keeps its place
    // Reference src/ops/all_gather_v/all_gather_v.cc:41-55, 137-282.
    CHK_PTR_Q(OpType::ALL_GATHER_V, comm, "comm");
    CHK_PTR_Q(OpType::ALL_GATHER_V, recvCounts, "recvCounts");
    CHK_PTR_Q(OpType::ALL_GATHER_V, recvDispls, "recvDispls");
    CHK_PTR_Q(OpType::ALL_GATHER_V, stream, "stream");
    if (sendCount > 0) {
        CHK_PTR_Q(OpType::ALL_GATHER_V, sendBuf, "sendBuf");
    }
    if (sendBuf != nullptr && recvBuf != nullptr && sendBuf == recvBuf) {
        Log(1, "HcclAllGatherV: sendBuf and recvBuf cannot be the same");
        return RejectIfKnown(ref, OpType::ALL_GATHER_V, HCCL_E_PARA);
    }
    Comm* c = ref.c;
    if (c == nullptr) {
        Log(1, "HcclAllGatherV: comm is not a live communicator");
        return RejectIfKnown(ref, OpType::ALL_GATHER_V, HCCL_E_PARA);
    }
    const uint32_t n = c->world->n;
    const uint64_t* counts = static_cast<const uint64_t*>(recvCounts);
    const uint64_t* displs = static_cast<const uint64_t*>(recvDispls);
    bool allZero = true;
    for (uint32_t i = 0; i < n; ++i) {
        allZero = allZero && counts[i] == 0;
    }
    if (allZero) {
        return HCCL_SUCCESS;
    }
    CHK_PTR_Q(OpType::ALL_GATHER_V, recvBuf, "recvBuf");
    CHK_RET_Q(OpType::ALL_GATHER_V, CheckUserRank(c));
    CHK_RET_Q(OpType::ALL_GATHER_V, CheckCount(sendCount));
    CHK_RET_Q(OpType::ALL_GATHER_V, CheckDataType(dataType, false));
    // Non-empty intervals may be unordered and leave holes but must not overlap or overflow.
    const uint64_t esz = DataTypeSize(dataType);
    for (uint32_t a = 0; a < n; ++a) {
        if (counts[a] == 0) {
            continue;
        }
        uint64_t end = displs[a] + counts[a];
        if (end < displs[a] || end > UINT64_MAX / esz) {
            Log(1, "HcclAllGatherV: recvDispls[%u] + recvCounts[%u] overflows", a, a);
            return RejectIfKnown(ref, OpType::ALL_GATHER_V, HCCL_E_PARA);
        }
        for (uint32_t b = a + 1; b < n; ++b) {
            if (counts[b] != 0 && displs[a] < displs[b] + counts[b] && displs[b] < end) {
                Log(1, "HcclAllGatherV: recvDispls intervals of ranks %u and %u overlap", a, b);
                return RejectIfKnown(ref, OpType::ALL_GATHER_V, HCCL_E_PARA);
            }
        }
    }
    std::vector<uint64_t> var(2 * n + 1);
    memcpy(var.data(), counts, n * sizeof(uint64_t));
    memcpy(var.data() + n, displs, n * sizeof(uint64_t));
    var[2 * n] = sendCount;
    // Every rank passes the same count as "count" of the pending op: use 0 so that ranks with different
    // sendCount still meet; per-rank counts are validated at launch.
    return SubmitWithReady(ref, OpType::ALL_GATHER_V, dataType, HCCL_REDUCE_RESERVED, 0, sendBuf, recvBuf, stream,
                           std::move(var));
}

HcclResult HcclAlltoAllV(const void* sendBuf, const void* sendCounts, const void* sdispls, HcclDataType sendType,
                         const void* recvBuf, const void* recvCounts, const void* rdispls, HcclDataType recvType,
                         HcclComm comm, aclrtStream stream)
{
    (void)sendType;
    return AlltoAllVEntry("HcclAlltoAllV", sendBuf, sendCounts, sdispls, recvBuf, recvCounts, rdispls, recvType, comm,
                          stream, false);
}

HcclResult HcclAmdAlltoAllVNoAlloc(const void* sendBuf, const void* sendCounts, const void* sdispls,
                                   HcclDataType sendType, const void* recvBuf, const void* recvCounts,
                                   const void* rdispls, HcclDataType recvType, HcclComm comm, aclrtStream stream)
{
    (void)sendType;
    return AlltoAllVEntry("HcclAmdAlltoAllVNoAlloc", sendBuf, sendCounts, sdispls, recvBuf, recvCounts, rdispls,
                          recvType, comm, stream, true);
}

HcclResult HcclAlltoAll(const void* sendBuf, uint64_t sendCount, HcclDataType sendType, const void* recvBuf,
                        uint64_t recvCount, HcclDataType recvType, HcclComm comm, aclrtStream stream)
{
    CommRef ref = AsComm(comm);   // looked up first, so that a call that fails any check below keeps its place
    // Reference src/ops/all_to_all_v/all_to_all_v.cc:39-82, 475-515.
    if (sendCount == 0 && recvCount == 0) {
        return HCCL_SUCCESS;
    }
    CHK_PTR_Q(OpType::ALL_TO_ALL_V, comm, "comm");
    CHK_PTR_Q(OpType::ALL_TO_ALL_V, sendBuf, "sendBuf");
    CHK_PTR_Q(OpType::ALL_TO_ALL_V, recvBuf, "recvBuf");
    if (sendCount != recvCount) {
        Log(1, "HcclAlltoAll: sendCount %llu and recvCount %llu are not equal", (unsigned long long)sendCount,
            (unsigned long long)recvCount);
        return RejectIfKnown(ref, OpType::ALL_TO_ALL_V, HCCL_E_PARA);
    }
    if (sendType != recvType) {
        Log(1, "HcclAlltoAll: sendType %d and recvType %d are not equal", static_cast<int>(sendType),
            static_cast<int>(recvType));
        return RejectIfKnown(ref, OpType::ALL_TO_ALL_V, HCCL_E_PARA);
    }
    CHK_PTR_Q(OpType::ALL_TO_ALL_V, stream, "stream");
    if (sendBuf == recvBuf) {
        Log(1, "HcclAlltoAll: sendBuf and recvBuf cannot be the same");
        return RejectIfKnown(ref, OpType::ALL_TO_ALL_V, HCCL_E_PARA);
    }
    if (DataTypeSize(sendType) == 0) {
        Log(1, "HcclAlltoAll: sendType %d is not supported", static_cast<int>(sendType));
        return RejectIfKnown(ref, OpType::ALL_TO_ALL_V, HCCL_E_PARA);
    }
    if (sendCount > UINT64_MAX / DataTypeSize(sendType)) {
        Log(1, "HcclAlltoAll: send size overflows");
        return RejectIfKnown(ref, OpType::ALL_TO_ALL_V, HCCL_E_PARA);
    }
    Comm* c = ref.c;
    if (c == nullptr) {
        Log(1, "HcclAlltoAll: comm is not a live communicator");
        return RejectIfKnown(ref, OpType::ALL_TO_ALL_V, HCCL_E_PARA);
    }
    CHK_RET_Q(OpType::ALL_TO_ALL_V, CheckUserRank(c));
    CHK_RET_Q(OpType::ALL_TO_ALL_V, CheckCount(recvCount));
    CHK_RET_Q(OpType::ALL_TO_ALL_V, CheckDataType(recvType, false));
    // Four arrays in AlltoAllV form: counts = recvCount, displacements = i * recvCount (:411-421).
    const uint32_t n = c->world->n;
    std::vector<uint64_t> var(4 * n);
    for (uint32_t i = 0; i < n; ++i) {
        var[i] = recvCount;
        var[n + i] = recvCount;
        var[2 * n + i] = static_cast<uint64_t>(i) * recvCount;
        var[3 * n + i] = static_cast<uint64_t>(i) * recvCount;
    }
    return SubmitWithReady(ref, OpType::ALL_TO_ALL_V, recvType, HCCL_REDUCE_RESERVED, 0, sendBuf,
                           const_cast<void*>(recvBuf), stream, std::move(var));
}

HcclResult HcclAlltoAllVC(const void* sendBuf, const void* sendCountMatrix, HcclDataType sendType, const void* recvBuf,
                          HcclDataType recvType, HcclComm comm, aclrtStream stream)
{
    CommRef ref = AsComm(comm);   // looked up first, so that a call that fails any check below keeps its place
    // Reference src/ops/all_to_all_v/all_to_all_v.cc:153-209, 423-458, 555-598.  Like the reference, only
    // recvType is consulted for the element size.
    (void)sendType;
    CHK_PTR_Q(OpType::ALL_TO_ALL_V, comm, "comm");
    CHK_PTR_Q(OpType::ALL_TO_ALL_V, sendCountMatrix, "sendCountMatrix");
    CHK_PTR_Q(OpType::ALL_TO_ALL_V, stream, "stream");
    if (sendBuf != nullptr && recvBuf != nullptr && sendBuf == recvBuf) {
        Log(1, "HcclAlltoAllVC: sendBuf and recvBuf cannot be the same");
        return RejectIfKnown(ref, OpType::ALL_TO_ALL_V, HCCL_E_PARA);
    }
    Comm* c = ref.c;
    if (c == nullptr) {
        Log(1, "HcclAlltoAllVC: comm is not a live communicator");
        return RejectIfKnown(ref, OpType::ALL_TO_ALL_V, HCCL_E_PARA);
    }
    CHK_RET_Q(OpType::ALL_TO_ALL_V, CheckUserRank(c));
    const uint32_t n = c->world->n;
    const uint32_t me = c->rank;
    const uint64_t* m = static_cast<const uint64_t*>(sendCountMatrix);
    uint64_t maxCount = 0;
    for (uint64_t i = 0; i < static_cast<uint64_t>(n) * n; ++i) {
        maxCount = m[i] > maxCount ? m[i] : maxCount;
    }
    CHK_RET_Q(OpType::ALL_TO_ALL_V, CheckCount(maxCount));
    // sendCounts = row `me`, recvCounts = column `me`, displacements = exclusive prefix sums (:444-455).
    std::vector<uint64_t> var(4 * n);
    uint64_t sOff = 0, rOff = 0;
    bool sendZero = true, recvZero = true;
    for (uint32_t i = 0; i < n; ++i) {
        var[i] = m[static_cast<uint64_t>(me) * n + i];
        var[n + i] = m[static_cast<uint64_t>(i) * n + me];
        var[2 * n + i] = sOff;
        var[3 * n + i] = rOff;
        sOff += var[i];
        rOff += var[n + i];
        sendZero = sendZero && var[i] == 0;
        recvZero = recvZero && var[n + i] == 0;
    }
    if (!sendZero) {
        CHK_PTR_Q(OpType::ALL_TO_ALL_V, sendBuf, "sendBuf");
    }
    if (!recvZero) {
        CHK_PTR_Q(OpType::ALL_TO_ALL_V, recvBuf, "recvBuf");
    }
    CHK_RET_Q(OpType::ALL_TO_ALL_V, CheckDataType(recvType, false));
    return SubmitWithReady(ref, OpType::ALL_TO_ALL_V, recvType, HCCL_REDUCE_RESERVED, 0, sendBuf,
                           const_cast<void*>(recvBuf), stream, std::move(var));
}

HcclResult HcclReduceScatterV(void* sendBuf, const void* sendCounts, const void* sendDispls, void* recvBuf,
                              uint64_t recvCount, HcclDataType dataType, HcclReduceOp op, HcclComm comm,
                              aclrtStream stream)
{
    CommRef ref = AsComm(comm);   // looked up first, so that a call that fails any check below keeps its place
    // Reference src/ops/reduce_scatter_v/reduce_scatter_v.cc:48-79, 180-247.
    CHK_PTR_Q(OpType::REDUCE_SCATTER_V, stream, "stream");
    CHK_PTR_Q(OpType::REDUCE_SCATTER_V, comm, "comm");
    CHK_PTR_Q(OpType::REDUCE_SCATTER_V, sendCounts, "sendCounts");
    CHK_PTR_Q(OpType::REDUCE_SCATTER_V, sendDispls, "sendDispls");
    if (recvCount > 0) {
        CHK_PTR_Q(OpType::REDUCE_SCATTER_V, recvBuf, "recvBuf");
    }
    Comm* c = ref.c;
    if (c == nullptr) {
        Log(1, "HcclReduceScatterV: comm is not a live communicator");
        return RejectIfKnown(ref, OpType::REDUCE_SCATTER_V, HCCL_E_PARA);
    }
    const uint32_t n = c->world->n;
    const uint64_t* counts = static_cast<const uint64_t*>(sendCounts);
    const uint64_t* displs = static_cast<const uint64_t*>(sendDispls);
    bool allZero = true;
    for (uint32_t i = 0; i < n; ++i) {
        allZero = allZero && counts[i] == 0;
    }
    if (allZero) {
        return HCCL_SUCCESS;
    }
    CHK_PTR_Q(OpType::REDUCE_SCATTER_V, sendBuf, "sendBuf");
    CHK_RET_Q(OpType::REDUCE_SCATTER_V, CheckUserRank(c));
    CHK_RET_Q(OpType::REDUCE_SCATTER_V, CheckCount(recvCount));
    // No uint64 / fp64 here, unlike the other reduce ops (:225-247).
    if (dataType == HCCL_DATA_TYPE_UINT64 || dataType == HCCL_DATA_TYPE_FP64) {
        Log(1, "HcclReduceScatterV: data type %d is not supported", static_cast<int>(dataType));
        return RejectIfKnown(ref, OpType::REDUCE_SCATTER_V, HCCL_E_NOT_SUPPORT);
    }
    CHK_RET_Q(OpType::REDUCE_SCATTER_V, CheckDataType(dataType, true));
    CHK_RET_Q(OpType::REDUCE_SCATTER_V, CheckReduceOp(dataType, op));
    std::vector<uint64_t> var(2 * n + 1);
    memcpy(var.data(), counts, n * sizeof(uint64_t));
    memcpy(var.data() + n, displs, n * sizeof(uint64_t));
    var[2 * n] = recvCount;
    // recvCount differs between ranks: 0 is the count the ranks meet on, the per-rank values are checked at launch.
    return SubmitWithReady(ref, OpType::REDUCE_SCATTER_V, dataType, op, 0, sendBuf, recvBuf, stream, std::move(var));
}

HcclResult HcclReduce(void* sendBuf, void* recvBuf, uint64_t count, HcclDataType dataType, HcclReduceOp op,
                      uint32_t root, HcclComm comm, aclrtStream stream)
{
    CommRef ref = AsComm(comm);   // looked up first, so that a call that fails any check below keeps its place
    // Reference src/ops/reduce/reduce.cc:39, 106-153.
    if (count == 0) {
        return HCCL_SUCCESS;
    }
    CHK_PTR_Q(OpType::REDUCE, comm, "comm");
    CHK_PTR_Q(OpType::REDUCE, sendBuf, "sendBuf");
    CHK_PTR_Q(OpType::REDUCE, recvBuf, "recvBuf");
    CHK_PTR_Q(OpType::REDUCE, stream, "stream");
    Comm* c = ref.c;
    if (c == nullptr) {
        Log(1, "HcclReduce: comm is not a live communicator");
        return RejectIfKnown(ref, OpType::REDUCE, HCCL_E_PARA);
    }
    CHK_RET_Q(OpType::REDUCE, CheckCount(count));
    CHK_RET_Q(OpType::REDUCE, CheckDataType(dataType, true));
    CHK_RET_Q(OpType::REDUCE, CheckReduceOp(dataType, op));
    if (root >= c->world->n) {
        Log(1, "HcclReduce: root %u is out of range [0, %u)", root, c->world->n);
        return RejectIfKnown(ref, OpType::REDUCE, HCCL_E_PARA);
    }
    CHK_RET_Q(OpType::REDUCE, CheckUserRank(c));
    return SubmitWithReady(ref, OpType::REDUCE, dataType, op, count, sendBuf, recvBuf, stream, {}, root);
}

HcclResult HcclBroadcast(void* buf, uint64_t count, HcclDataType dataType, uint32_t root, HcclComm comm,
                         aclrtStream stream)
{
    CommRef ref = AsComm(comm);   // looked up first, so that a call that fails any check below keeps its place
    // Reference src/ops/broadcast/broadcast.cc:38, 99-142.
    if (count == 0) {
        return HCCL_SUCCESS;
    }
    CHK_PTR_Q(OpType::BROADCAST, comm, "comm");
    CHK_PTR_Q(OpType::BROADCAST, buf, "buf");
    CHK_PTR_Q(OpType::BROADCAST, stream, "stream");
    Comm* c = ref.c;
    if (c == nullptr) {
        Log(1, "HcclBroadcast: comm is not a live communicator");
        return RejectIfKnown(ref, OpType::BROADCAST, HCCL_E_PARA);
    }
    CHK_RET_Q(OpType::BROADCAST, CheckUserRank(c));
    if (root >= c->world->n) {
        Log(1, "HcclBroadcast: root %u is out of range [0, %u)", root, c->world->n);
        return RejectIfKnown(ref, OpType::BROADCAST, HCCL_E_PARA);
    }
    CHK_RET_Q(OpType::BROADCAST, CheckCount(count));
    CHK_RET_Q(OpType::BROADCAST, CheckDataType(dataType, false));
    return SubmitWithReady(ref, OpType::BROADCAST, dataType, HCCL_REDUCE_RESERVED, count, buf, buf, stream, {}, root);
}

HcclResult HcclScatter(void* sendBuf, void* recvBuf, uint64_t recvCount, HcclDataType dataType, uint32_t root,
                       HcclComm comm, aclrtStream stream)
{
    CommRef ref = AsComm(comm);   // looked up first, so that a call that fails any check below keeps its place
    // Reference src/ops/scatter/scatter.cc:59-73, 115-128.  The reference leaves a null stream to the layers
    // below the entry point; here it is rejected after the reference's own checks.
    if (recvCount == 0) {
        return HCCL_SUCCESS;
    }
    CHK_PTR_Q(OpType::SCATTER, comm, "comm");
    CHK_PTR_Q(OpType::SCATTER, recvBuf, "recvBuf");
    Comm* c = ref.c;
    if (c == nullptr) {
        Log(1, "HcclScatter: comm is not a live communicator");
        return RejectIfKnown(ref, OpType::SCATTER, HCCL_E_PARA);
    }
    if (c->rank == root) {
        CHK_PTR_Q(OpType::SCATTER, sendBuf, "sendBuf");   // only the root's sendBuf is read
    }
    if (root >= c->world->n) {
        Log(1, "HcclScatter: root %u is out of range [0, %u)", root, c->world->n);
        return RejectIfKnown(ref, OpType::SCATTER, HCCL_E_PARA);
    }
    CHK_RET_Q(OpType::SCATTER, CheckCount(recvCount));
    CHK_RET_Q(OpType::SCATTER, CheckDataType(dataType, false));
    CHK_PTR_Q(OpType::SCATTER, stream, "stream");
    return SubmitWithReady(ref, OpType::SCATTER, dataType, HCCL_REDUCE_RESERVED, recvCount, sendBuf, recvBuf, stream, {},
                           root);
}

// ---- lifecycle -------------------------------------------------------------------------------
HcclResult HcclCommInitAll(uint32_t ndev, int32_t* devices, HcclComm* comms)
{
    CHK_PTR(comms, "comms");
    if (ndev == 0 || ndev > static_cast<uint32_t>(kMaxRanks)) {
        Log(1, "HcclCommInitAll: ndev %u outside [1, %d]", ndev, kMaxRanks);
        return HCCL_E_PARA;
    }
    if (devices != nullptr) {
        for (uint32_t i = 1; i < ndev; ++i) {
            if (devices[i] != devices[0]) {
                Log(1, "HcclCommInitAll: a loopback world lives on one GPU; devices[%u]=%d != devices[0]=%d", i,
                    devices[i], devices[0]);
                return HCCL_E_NOT_SUPPORT;
            }
        }
    }
    std::lock_guard<std::mutex> g(g_registryMu);
    auto w = NewWorld(ndev);
    w->id = g_nextWorldId++;
    for (uint32_t r = 0; r < ndev; ++r) {
        w->comms[r] = std::make_unique<Comm>();
        w->comms[r]->world = w.get();
        w->comms[r]->rank = r;
        comms[r] = w->comms[r].get();
    }
    w->joined = ndev;
    std::shared_ptr<World> shared(std::move(w));
    for (uint32_t r = 0; r < ndev; ++r) {
        g_liveComms[comms[r]] = shared;
    }
    g_worlds[shared->id] = shared;
    return HCCL_SUCCESS;
}

HcclResult HcclGetRootInfo(HcclRootInfo* rootInfo)
{
    CHK_PTR(rootInfo, "rootInfo");
    std::lock_guard<std::mutex> g(g_registryMu);
    memset(rootInfo, 0, sizeof(*rootInfo));
    uint64_t id = g_nextWorldId++;
    memcpy(rootInfo->internal, "HCLAROOT", 8);
    memcpy(rootInfo->internal + 8, &id, sizeof(id));
    return HCCL_SUCCESS;
}

HcclResult HcclCommInitRootInfo(uint32_t nRanks, const HcclRootInfo* rootInfo, uint32_t rank, HcclComm* comm)
{
    CHK_PTR(rootInfo, "rootInfo");
    CHK_PTR(comm, "comm");
    if (memcmp(rootInfo->internal, "HCLAROOT", 8) != 0 || nRanks == 0 || nRanks > static_cast<uint32_t>(kMaxRanks) ||
        rank >= nRanks) {
        Log(1, "HcclCommInitRootInfo: invalid rootInfo, nRanks %u or rank %u", nRanks, rank);
        return HCCL_E_PARA;
    }
    uint64_t id;
    memcpy(&id, rootInfo->internal + 8, sizeof(id));
    std::lock_guard<std::mutex> g(g_registryMu);
    auto it = g_worlds.find(id);
    if (it == g_worlds.end()) {
        auto w = NewWorld(nRanks);
        w->id = id;
        it = g_worlds.emplace(id, std::shared_ptr<World>(std::move(w))).first;
    }
    World* w = it->second.get();
    if (w->n != nRanks || w->comms[rank] != nullptr) {
        Log(1, "HcclCommInitRootInfo: rank %u joins a world of %u ranks inconsistently", rank, w->n);
        return HCCL_E_PARA;
    }
    w->comms[rank] = std::make_unique<Comm>();
    w->comms[rank]->world = w;
    w->comms[rank]->rank = rank;
    w->joined++;
    *comm = w->comms[rank].get();
    g_liveComms[*comm] = it->second;
    return HCCL_SUCCESS;
}

HcclResult HcclCommDestroy(HcclComm comm)
{
    CHK_PTR(comm, "comm");
    std::shared_ptr<World> w;
    {
        std::lock_guard<std::mutex> g(g_registryMu);
        auto it = g_liveComms.find(comm);
        if (it == g_liveComms.end()) {
            Log(1, "HcclCommDestroy: comm is not a live communicator");
            return HCCL_E_PARA;   // never issued, or destroyed before: the handle is not dereferenced
        }
        w = it->second;
        g_liveComms.erase(it);
    }
    Comm* c = static_cast<Comm*>(comm);
    bool last;
    {
        std::lock_guard<std::mutex> wl(w->mu);
        c->destroyed = true;
        w->destroyed++;
        last = w->destroyed == w->n;
        // A rank that leaves will not join what its peers are still waiting for: those calls end now, with an
        // error, and nothing more is launched in this world.
        for (std::shared_ptr<PendingOp>& op : w->pending) {
            if (op && !op->done) {
                op->result = HCCL_E_UNAVAIL;
                op->done = true;
            }
        }
        for (auto& kv : w->p2p) {
            for (std::shared_ptr<P2pOp>& op : kv.second) {
                if (!op->done) {
                    op->result = HCCL_E_UNAVAIL;
                    op->done = true;
                }
            }
            kv.second.clear();
        }
        w->cv.notify_all();
    }
    if (last) {
        (void)hipDeviceSynchronize();
        std::lock_guard<std::mutex> g(g_registryMu);
        g_worlds.erase(w->id);   // the world itself goes when the last call that holds it returns
    }
    return HCCL_SUCCESS;
}

HcclResult HcclGetRankSize(HcclComm comm, uint32_t* rankSize)
{
    CHK_PTR(comm, "comm");
    CHK_PTR(rankSize, "rankSize");
    CommRef ref = AsComm(comm);
    Comm* c = ref.c;
    if (c == nullptr) {
        return HCCL_E_PARA;
    }
    *rankSize = c->world->n;
    return HCCL_SUCCESS;
}

HcclResult HcclGetRankId(HcclComm comm, uint32_t* rank)
{
    CHK_PTR(comm, "comm");
    CHK_PTR(rank, "rank");
    CommRef ref = AsComm(comm);
    Comm* c = ref.c;
    if (c == nullptr) {
        return HCCL_E_PARA;
    }
    *rank = c->rank;
    return HCCL_SUCCESS;
}

HcclResult HcclGetCommName(HcclComm comm, char* commName)
{
    CHK_PTR(comm, "comm");
    CHK_PTR(commName, "commName");
    CommRef ref = AsComm(comm);
    if (ref.c == nullptr) {
        return HCCL_E_PARA;
    }
    snprintf(commName, HCCL_AMD_COMM_NAME_LENGTH, "hccl_amd_world_%llu", static_cast<unsigned long long>(ref.c->world->id));
    return HCCL_SUCCESS;
}

const char* HcclGetErrorString(HcclResult code)
{
    switch (code) {
        case HCCL_SUCCESS: return "no error";
        case HCCL_E_PARA: return "parameter error";
        case HCCL_E_PTR: return "empty pointer";
        case HCCL_E_MEMORY: return "memory error";
        case HCCL_E_INTERNAL: return "internal error";
        case HCCL_E_NOT_SUPPORT: return "not support feature";
        case HCCL_E_NOT_FOUND: return "not found specific resource";
        case HCCL_E_UNAVAIL: return "resource unavailable";
        case HCCL_E_TIMEOUT: return "timeout";
        case HCCL_E_RUNTIME: return "call runtime api fail";
        default: return "unknown error";
    }
}

// Every rank's stream waits until all ranks' streams have reached their HcclBarrier.  Reference
// src/ops/barrier/barrier.cc:47-101 (null stream, then null comm, then the rank check).
HcclResult HcclBarrier(HcclComm comm, aclrtStream stream)
{
    CHK_PTR(stream, "stream");
    CHK_PTR(comm, "comm");
    CommRef ref = AsComm(comm);
    Comm* c = ref.c;
    if (c == nullptr) {
        Log(1, "HcclBarrier: comm is not a live communicator");
        return HCCL_E_PARA;
    }
    CHK_RET(CheckUserRank(c));
    return SubmitWithReady(ref, OpType::BARRIER, HCCL_DATA_TYPE_RESERVED, HCCL_REDUCE_RESERVED, 0, nullptr, nullptr, stream,
                           {});
}

// Reference src/ops/send/send.cc:25-49, 136-163.
HcclResult HcclSend(void* sendBuf, uint64_t count, HcclDataType dataType, uint32_t destRank, HcclComm comm,
                    aclrtStream stream)
{
    if (count == 0) {
        return HCCL_SUCCESS;
    }
    CHK_PTR(stream, "stream");
    CHK_PTR(comm, "comm");
    CHK_PTR(sendBuf, "sendBuf");
    CHK_RET(CheckCount(count));
    CHK_RET(CheckDataType(dataType, false));
    CommRef ref = AsComm(comm);
    Comm* c = ref.c;
    if (c == nullptr) {
        Log(1, "HcclSend: comm is not a live communicator");
        return HCCL_E_PARA;
    }
    if (c->rank == destRank) {
        Log(1, "HcclSend: destRank cannot be equal to self");
        return HCCL_E_NOT_SUPPORT;
    }
    CHK_RET(CheckUserRank(c));
    if (destRank >= c->world->n) {
        Log(1, "HcclSend: destRank %u is out of range [0, %u)", destRank, c->world->n);
        return HCCL_E_PARA;
    }
    if (c->world->envInvalid) {
        return HCCL_E_PARA;
    }
    World* w = c->world;
    std::unique_lock<std::mutex> lock(w->mu);
    if (w->destroyed != 0) {
        Log(1, "%s on rank %u: a communicator of this world has been destroyed", "HcclSend", c->rank);
        return HCCL_E_UNAVAIL;   // the peer may be the one that left: nothing would ever complete this transfer
    }
    std::vector<std::shared_ptr<P2pOp>> ops{
        DepositP2p(w, true, c->rank, destRank, sendBuf, count, dataType, static_cast<hipStream_t>(stream))};
    return AwaitP2p(ref, lock, ops, "HcclSend", c->rank);
}

// Reference src/ops/recv/recv.cc:25-49, 134-161.
HcclResult HcclRecv(void* recvBuf, uint64_t count, HcclDataType dataType, uint32_t srcRank, HcclComm comm,
                    aclrtStream stream)
{
    if (count == 0) {
        return HCCL_SUCCESS;
    }
    CHK_PTR(stream, "stream");
    CHK_PTR(comm, "comm");
    CHK_PTR(recvBuf, "recvBuf");
    CHK_RET(CheckCount(count));
    CHK_RET(CheckDataType(dataType, false));
    CommRef ref = AsComm(comm);
    Comm* c = ref.c;
    if (c == nullptr) {
        Log(1, "HcclRecv: comm is not a live communicator");
        return HCCL_E_PARA;
    }
    if (c->rank == srcRank) {
        Log(1, "HcclRecv: srcRank cannot be equal to self");
        return HCCL_E_NOT_SUPPORT;
    }
    CHK_RET(CheckUserRank(c));
    if (srcRank >= c->world->n) {
        Log(1, "HcclRecv: srcRank %u is out of range [0, %u)", srcRank, c->world->n);
        return HCCL_E_PARA;
    }
    if (c->world->envInvalid) {
        return HCCL_E_PARA;
    }
    World* w = c->world;
    std::unique_lock<std::mutex> lock(w->mu);
    if (w->destroyed != 0) {
        Log(1, "%s on rank %u: a communicator of this world has been destroyed", "HcclRecv", c->rank);
        return HCCL_E_UNAVAIL;   // the peer may be the one that left: nothing would ever complete this transfer
    }
    std::vector<std::shared_ptr<P2pOp>> ops{
        DepositP2p(w, false, srcRank, c->rank, recvBuf, count, dataType, static_cast<hipStream_t>(stream))};
    return AwaitP2p(ref, lock, ops, "HcclRecv", c->rank);
}

// Reference src/ops/batch_send_recv/batch_send_recv.cc:22-60, 72-90 and, for which send meets which receive,
// algorithm/executor/ins_v2_batch_send_recv_executor.cc:96-200: items without elements are skipped, several
// transfers between the same two ranks pair up by descending count, then descending data type (stable), and a
// rank may send to itself when the batch holds the matching receive.
HcclResult HcclBatchSendRecv(HcclSendRecvItem* sendRecvInfo, uint32_t itemNum, HcclComm comm, aclrtStream stream)
{
    if (itemNum == 0) {
        return HCCL_SUCCESS;
    }
    CHK_PTR(stream, "stream");
    CHK_PTR(comm, "comm");
    CHK_PTR(sendRecvInfo, "sendRecvInfo");
    for (uint32_t i = 0; i < itemNum; ++i) {
        CHK_RET(CheckCount(sendRecvInfo[i].count));
        CHK_RET(CheckDataType(sendRecvInfo[i].dataType, false));
    }
    CommRef ref = AsComm(comm);
    Comm* c = ref.c;
    if (c == nullptr) {
        Log(1, "HcclBatchSendRecv: comm is not a live communicator");
        return HCCL_E_PARA;
    }
    CHK_RET(CheckUserRank(c));
    World* w = c->world;
    std::vector<const HcclSendRecvItem*> sends, recvs;
    for (uint32_t i = 0; i < itemNum; ++i) {
        const HcclSendRecvItem& it = sendRecvInfo[i];
        if (it.remoteRank >= w->n) {
            Log(1, "HcclBatchSendRecv: item %u names rank %u outside [0, %u)", i, it.remoteRank, w->n);
            return HCCL_E_PARA;
        }
        if (it.count == 0) {
            continue;
        }
        CHK_PTR(it.buf, "item buf");
        if (it.sendRecvType == HCCL_SEND) {
            sends.push_back(&it);
        } else if (it.sendRecvType == HCCL_RECV) {
            recvs.push_back(&it);
        } else {
            Log(1, "HcclBatchSendRecv: item %u has send / recv type %d", i, static_cast<int>(it.sendRecvType));
            return HCCL_E_PARA;
        }
    }
    // Transfers to the own rank must come in pairs (reference ins_v2_batch_send_recv_executor.cc:183-200).
    size_t selfSends = 0, selfRecvs = 0;
    for (const HcclSendRecvItem* it : sends) selfSends += it->remoteRank == c->rank;
    for (const HcclSendRecvItem* it : recvs) selfRecvs += it->remoteRank == c->rank;
    if (selfSends != selfRecvs) {
        Log(1, "HcclBatchSendRecv: %zu sends to the own rank but %zu receives from it", selfSends, selfRecvs);
        return HCCL_E_PARA;
    }
    if (w->envInvalid) {
        return HCCL_E_PARA;
    }
    auto bigFirst = [](const HcclSendRecvItem* a, const HcclSendRecvItem* b) {
        if (a->remoteRank != b->remoteRank) {
            return a->remoteRank < b->remoteRank;   // any fixed order of the peers: pairs are matched per peer
        }
        if (a->count != b->count) {
            return a->count > b->count;
        }
        return static_cast<int>(a->dataType) > static_cast<int>(b->dataType);
    };
    std::stable_sort(sends.begin(), sends.end(), bigFirst);
    std::stable_sort(recvs.begin(), recvs.end(), bigFirst);
    std::unique_lock<std::mutex> lock(w->mu);
    if (w->destroyed != 0) {
        Log(1, "%s on rank %u: a communicator of this world has been destroyed", "HcclBatchSendRecv", c->rank);
        return HCCL_E_UNAVAIL;   // the peer may be the one that left: nothing would ever complete this transfer
    }
    std::vector<std::shared_ptr<P2pOp>> ops;
    for (const HcclSendRecvItem* it : sends) {
        ops.push_back(DepositP2p(w, true, c->rank, it->remoteRank, it->buf, it->count, it->dataType,
                                 static_cast<hipStream_t>(stream)));
    }
    for (const HcclSendRecvItem* it : recvs) {
        ops.push_back(DepositP2p(w, false, it->remoteRank, c->rank, it->buf, it->count, it->dataType,
                                 static_cast<hipStream_t>(stream)));
    }
    return AwaitP2p(ref, lock, ops, "HcclBatchSendRecv", c->rank);
}

HcclResult HcclGroupStart(void)
{
    t_groupDepth++;
    return HCCL_SUCCESS;
}

HcclResult HcclGroupEnd(void)
{
    if (t_groupDepth == 0) {
        Log(1, "HcclGroupEnd without HcclGroupStart");
        return HCCL_E_PARA;
    }
    if (--t_groupDepth != 0) {
        return HCCL_SUCCESS;
    }
    // The outermost end: every call this thread queued since the group began has been launched (by this thread
    // or by the thread that completed its set) or has failed when this returns; the worst result is reported.
    // A set that is never completed ends here after the world's time-out instead of staying pending for ever.
    HcclResult worst = HCCL_SUCCESS;
    std::vector<GroupItem> items;
    items.swap(t_groupItems);
    for (GroupItem& item : items) {
        World* w = item.world.get();
        std::unique_lock<std::mutex> lock(w->mu);
        HcclResult rc;
        if (item.op) {
            const bool ok = w->cv.wait_for(lock, std::chrono::seconds(w->execTimeout), [&] { return item.op->done; });
            if (!ok) {
                Log(1, "HcclGroupEnd: %s waited %u s for the other ranks", OpName(item.op->type), w->execTimeout);
                item.op->result = HCCL_E_TIMEOUT;   // the late ranks find the verdict and launch nothing
            }
            rc = ok ? item.op->result : HCCL_E_TIMEOUT;
        } else {
            const bool ok = w->cv.wait_for(lock, std::chrono::seconds(w->execTimeout), [&] { return item.p2p->done; });
            if (!ok) {
                Log(1, "HcclGroupEnd: a send or receive waited %u s for its peer", w->execTimeout);
                item.p2p->result = HCCL_E_TIMEOUT;
            }
            rc = ok ? item.p2p->result : HCCL_E_TIMEOUT;
        }
        if (rc != HCCL_SUCCESS) {
            worst = rc;
        }
    }
    return worst;
}

HcclResult HcclAmdSetAlgo(HcclComm comm, HcclAmdOpKind op, HcclAmdAlgo algo)
{
    CHK_PTR(comm, "comm");
    CommRef ref = AsComm(comm);
    Comm* c = ref.c;
    if (c == nullptr || static_cast<int>(op) < 0 || op >= HCCL_AMD_OP_COUNT || static_cast<int>(algo) < 0 ||
        algo >= HCCL_AMD_ALGO_COUNT) {
        return HCCL_E_PARA;
    }
    if (!AlgoFitsOp(op, algo)) {
        return HCCL_E_NOT_SUPPORT;
    }
    std::lock_guard<std::mutex> wl(c->world->mu);
    c->world->algo[op] = algo;
    return HCCL_SUCCESS;
}

HcclResult HcclAmdSetCclBufferSize(HcclComm comm, uint64_t bytes)
{
    CHK_PTR(comm, "comm");
    CommRef ref = AsComm(comm);
    Comm* c = ref.c;
    if (c == nullptr) {
        return HCCL_E_PARA;
    }
    std::lock_guard<std::mutex> wl(c->world->mu);
    c->world->cclBytes = bytes;
    return HCCL_SUCCESS;
}

HcclResult HcclAmdGetCclBufferSize(HcclComm comm, uint64_t* bytes)
{
    CHK_PTR(comm, "comm");
    CHK_PTR(bytes, "bytes");
    CommRef ref = AsComm(comm);
    Comm* c = ref.c;
    if (c == nullptr) {
        return HCCL_E_PARA;
    }
    std::lock_guard<std::mutex> wl(c->world->mu);
    *bytes = c->world->cclBytes;
    return HCCL_SUCCESS;
}

HcclResult HcclAmdGetAlgo(HcclComm comm, HcclAmdOpKind op, HcclAmdAlgo* algo)
{
    CHK_PTR(comm, "comm");
    CHK_PTR(algo, "algo");
    CommRef ref = AsComm(comm);
    Comm* c = ref.c;
    if (c == nullptr || static_cast<int>(op) < 0 || op >= HCCL_AMD_OP_COUNT) {
        return HCCL_E_PARA;
    }
    std::lock_guard<std::mutex> wl(c->world->mu);
    *algo = c->world->algo[op];
    return HCCL_SUCCESS;
}

HcclResult HcclAmdGetStuckCounters(HcclComm comm, uint64_t* head, uint64_t* tail)
{
    CHK_PTR(comm, "comm");
    CHK_PTR(head, "head");
    CHK_PTR(tail, "tail");
    CommRef ref = AsComm(comm);
    if (ref.c == nullptr) {
        return HCCL_E_PARA;
    }
    World* w = ref.c->world;
    std::lock_guard<std::mutex> wl(w->mu);
    if (!w->stuckEnabled) {
        return HCCL_E_UNAVAIL;
    }
    // The GPU writes these words; read them as they are now.
    volatile uint64_t* words = w->stuck;
    *head = words != nullptr ? words[0] : 0;
    *tail = words != nullptr ? words[1] : 0;
    return HCCL_SUCCESS;
}

HcclResult HcclAmdSetLevel0RankSize(HcclComm comm, uint32_t ranksPerGroup)
{
    CHK_PTR(comm, "comm");
    CommRef ref = AsComm(comm);
    Comm* c = ref.c;
    if (c == nullptr || ranksPerGroup == 0 || ranksPerGroup > c->world->n || c->world->n % ranksPerGroup != 0) {
        return HCCL_E_PARA;
    }
    std::lock_guard<std::mutex> wl(c->world->mu);
    c->world->level0 = ranksPerGroup;
    return HCCL_SUCCESS;
}

HcclResult HcclAmdGetLevel0RankSize(HcclComm comm, uint32_t* ranksPerGroup)
{
    CHK_PTR(comm, "comm");
    CHK_PTR(ranksPerGroup, "ranksPerGroup");
    CommRef ref = AsComm(comm);
    Comm* c = ref.c;
    if (c == nullptr) {
        return HCCL_E_PARA;
    }
    std::lock_guard<std::mutex> wl(c->world->mu);
    *ranksPerGroup = c->world->level0;
    return HCCL_SUCCESS;
}

HcclResult HcclAmdSelectFromHcclAlgo(const char* config, HcclAmdOpKind op, int32_t* selected, HcclAmdAlgo* algo,
                                     int32_t* twoLevel, char* canonical, uint32_t cap)
{
    CHK_PTR(config, "config");
    if (static_cast<int>(op) < 0 || op >= HCCL_AMD_OP_COUNT) {
        return HCCL_E_PARA;
    }
    std::vector<AlgoSegment> segments;
    HcclResult rc = ParseHcclAlgo(config, &segments);
    if (rc != HCCL_SUCCESS) {
        return rc;
    }
    const AlgoSelection sel = SelectFromHcclAlgo(segments);
    if (selected != nullptr) {
        *selected = sel.set[op] ? 1 : 0;
    }
    if (algo != nullptr) {
        *algo = sel.algo[op];
    }
    if (twoLevel != nullptr) {
        *twoLevel = sel.twoLevel[op] ? 1 : 0;
    }
    if (canonical != nullptr && cap != 0) {
        std::string text;
        for (const AlgoSegment& seg : segments) {
            if (!text.empty()) {
                text += ";";
            }
            std::string unit = seg.executor + "{";
            for (size_t i = 0; i < seg.templates.size(); ++i) {
                unit += (i ? "," : "") + (seg.templates[i].enable ? seg.templates[i].name : "not(" + seg.templates[i].name + ")");
            }
            unit += "}";
            text += (seg.opType.empty() ? "" : seg.opType + ":") + (seg.enable ? unit : "not(" + unit + ")");
        }
        if (text.size() + 1 > cap) {
            return HCCL_E_MEMORY;
        }
        memcpy(canonical, text.c_str(), text.size() + 1);
    }
    return HCCL_SUCCESS;
}

HcclResult HcclAmdGetFoldProgram(HcclAmdOpKind op, HcclAmdAlgo algo, uint32_t rankSize, uint32_t segment,
                                 uint8_t* out, uint32_t cap, uint32_t* len, uint32_t* segmentCount)
{
    return HcclAmdGetFoldProgramTwoLevel(op, algo, rankSize, 1, segment, out, cap, len, segmentCount);
}

HcclResult HcclAmdGetFoldProgramTwoLevel(HcclAmdOpKind op, HcclAmdAlgo algo, uint32_t rankSize, uint32_t level0,
                                         uint32_t segment, uint8_t* out, uint32_t cap, uint32_t* len,
                                         uint32_t* segmentCount)
{
    CHK_PTR(len, "len");
    // Callers walk all segments of one plan: keep the last plan built.
    static std::mutex cacheMu;
    static FoldPlan plan;
    static int cachedOp = -1, cachedAlgo = -1;
    static uint32_t cachedSize = 0, cachedLevel0 = 0;
    std::lock_guard<std::mutex> cacheLock(cacheMu);
    if (cachedOp != static_cast<int>(op) || cachedAlgo != static_cast<int>(algo) || cachedSize != rankSize ||
        cachedLevel0 != level0) {
        cachedOp = -1;
        HcclResult rc = BuildFoldPlan(op, algo, rankSize, &plan, level0);
        if (rc != HCCL_SUCCESS) {
            return rc;
        }
        cachedOp = static_cast<int>(op);
        cachedAlgo = static_cast<int>(algo);
        cachedSize = rankSize;
        cachedLevel0 = level0;
    }
    if (segmentCount != nullptr) {
        *segmentCount = static_cast<uint32_t>(plan.programs.size());
    }
    if (segment >= plan.programs.size()) {
        return HCCL_E_PARA;
    }
    const std::vector<uint8_t>& p = plan.programs[segment];
    *len = static_cast<uint32_t>(p.size());
    if (out != nullptr) {
        if (cap < p.size()) {
            return HCCL_E_MEMORY;
        }
        memcpy(out, p.data(), p.size());
    }
    return HCCL_SUCCESS;
}

}  // extern "C"
