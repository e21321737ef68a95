// Host layer, part 1: logging, the reference's argument checks, environment settings, world creation, the registry
// of live handles and the upload of fold plans.
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

// Worlds by id, and the live communicator handles with the world each belongs to.  A handle that is not in
// g_liveComms (never issued, destroyed, or of a world that is gone) is rejected without being dereferenced; a
// call holds its world through the shared pointer until it returns, whatever other threads destroy meanwhile.
std::mutex g_registryMu;
std::map<uint64_t, std::shared_ptr<World>> g_worlds;
std::unordered_map<const void*, std::shared_ptr<World>> g_liveComms;
uint64_t g_nextWorldId = 1;
thread_local int t_groupDepth = 0;
thread_local std::vector<GroupItem> t_groupItems;

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
        {"mesh_chunk", HCCL_AMD_ALGO_MESH_CHUNK}, {"mesh_two_shot", HCCL_AMD_ALGO_MESH_TWO_SHOT},
        {"mesh_concur", HCCL_AMD_ALGO_MESH_CONCUR}};
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
            return algo != HCCL_AMD_ALGO_MESH_TWO_SHOT && algo != HCCL_AMD_ALGO_MESH_CONCUR;
        case HCCL_AMD_OP_REDUCE:
            return algo == HCCL_AMD_ALGO_MESH || algo == HCCL_AMD_ALGO_RING || algo == HCCL_AMD_ALGO_MESH_TWO_SHOT ||
                   algo == HCCL_AMD_ALGO_NHR || algo == HCCL_AMD_ALGO_RHD;
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
            } else if (kind == HCCL_AMD_OP_REDUCE_SCATTER) {
                w->reduceScatterSequence = sel.twoLevel[op] ? 1 : 0;
            } else if (kind == HCCL_AMD_OP_REDUCE) {
                w->reduceSequence = sel.twoLevel[op] ? 1 : 0;
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
    w->reduceBlocks = EnvU32("HCCL_AMD_REDUCE_BLOCKS", kReduceBlocksDefault);
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
    w->reduceAllFold = EnvInt("HCCL_AMD_REDUCE_ALL_FOLD", -1);
    if (w->reduceAllFold != 0 && (w->reduceAllFold < 2 || w->reduceAllFold > static_cast<int>(kMaxReduceThreads / 64))) {
        w->reduceAllFold = -1;
    }
    w->reduceDirect = EnvInt("HCCL_AMD_REDUCE_DIRECT", -1);
    if (w->reduceDirect != 0 && (w->reduceDirect < 2 || w->reduceDirect > static_cast<int>(kDirectFoldMaxWaves))) {
        w->reduceDirect = -1;
    }
    w->reduceDirectTiles = EnvInt("HCCL_AMD_REDUCE_DIRECT_TILES", 0);
    if (w->reduceDirectTiles < 1 || w->reduceDirectTiles > 2) {
        w->reduceDirectTiles = 0;
    }
    w->reducePair = EnvInt("HCCL_AMD_REDUCE_PAIR", 2);
    if (w->reducePair < 0 || w->reducePair > 1) {
        w->reducePair = 2;
    }
    w->fanOutLoadMode = EnvInt("HCCL_AMD_FANOUT_STREAM_LOAD", 2);
    if (w->fanOutLoadMode < 0 || w->fanOutLoadMode > 1) {
        w->fanOutLoadMode = 2;
    }
    w->copyTwoKernelMode = EnvInt("HCCL_AMD_COPY_TWO_KERNELS", 2);
    if (w->copyTwoKernelMode < 0 || w->copyTwoKernelMode > 1) {
        w->copyTwoKernelMode = 2;
    }
    w->pieceBytes = (static_cast<uint64_t>(EnvU32("HCCL_AMD_ALLREDUCE_PIECE_BYTES", static_cast<uint32_t>(policy::kPieceBytes))) + 255) & ~255ull;
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
        const uint32_t perGroup = EnvU32("HCCL_AMD_LEVEL1_GROUPS", 0);
        if (perGroup == 0 || (n / w->level0) % perGroup == 0) {
            w->level1 = perGroup;
        } else {
            Log(1, "HCCL_AMD_LEVEL1_GROUPS=%u does not divide the %u level-0 groups of the world: ignored", perGroup,
                n / w->level0);
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
HcclResult GetDevicePlan(World* w, HcclAmdOpKind kind, HcclAmdAlgo algo, DevicePlan* out, uint32_t level0,
                         uint32_t level1)
{
    uint32_t key = ((static_cast<uint32_t>(kind) * 64 + static_cast<uint32_t>(algo)) * 128 + level0) * 128 + level1;
    auto it = w->plans.find(key);
    if (it != w->plans.end()) {
        *out = it->second;
        return HCCL_SUCCESS;
    }
    FoldPlan plan;
    HcclResult rc = BuildFoldPlan(kind, algo, w->n, &plan, level0, level1);
    if (rc != HCCL_SUCCESS) {
        return rc;
    }
    // Flatten every token program to the kernel's leaf table.
    std::vector<uint8_t> image(plan.programs.size() * kDevProgBytes, 0);
    uint32_t maxLeaves = 0;
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
        maxLeaves = leaves > maxLeaves ? leaves : maxLeaves;
    }
    DevicePlan dp;
    dp.nProg = static_cast<uint32_t>(plan.programs.size());
    dp.segmentsAreSubs = plan.segmentsAreSubs;
    dp.maxDepth = plan.maxDepth;
    dp.maxLeaves = maxLeaves;
    HIP_OK(hipMalloc(reinterpret_cast<void**>(&dp.dev), image.size()));
    HIP_OK(hipMemcpy(dp.dev, image.data(), image.size(), hipMemcpyHostToDevice));
    dp.host = std::make_shared<const std::vector<uint8_t>>(std::move(image));
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

}  // namespace hccl_amd
