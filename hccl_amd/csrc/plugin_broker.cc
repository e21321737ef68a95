// PluginBroker on top of the loopback data plane: the function table of include/hccl_algo_plugin.h,
// dispatching the fixed-count operators and Send / Recv the reference's plugin manager can describe with one scalar
// count (reference src/algo_plugin/hccl_algo_plugin_mgr.cc: ExtractCountAndDataType, OpTypeToName) to
// the entry points of include/hccl.h.  The V operators have no plugin signature in the reference and
// are answered with "not selected" / HCCL_E_NOT_SUPPORT, like its manager does.
#include <cstdio>
#include <cstring>

#include "hccl.h"
#include "hccl_algo_plugin.h"

namespace {

struct BrokerContext {
    uint32_t magic;
};
constexpr uint32_t kContextMagic = 0x414D4442u;   // "AMDB"
BrokerContext g_context = {kContextMagic};

struct OpEntry {
    const char* opName;
    const char* algName;   // one algorithm per operator: the fused loopback kernel
};
const OpEntry kOps[] = {
    {"AllReduce", "HcclAmdLoopbackAllReduce"},       {"ReduceScatter", "HcclAmdLoopbackReduceScatter"},
    {"AllGather", "HcclAmdLoopbackAllGather"},       {"Reduce", "HcclAmdLoopbackReduce"},
    {"Broadcast", "HcclAmdLoopbackBroadcast"},       {"Scatter", "HcclAmdLoopbackScatter"},
    {"AllToAll", "HcclAmdLoopbackAllToAll"},         {"Send", "HcclAmdLoopbackSend"},
    {"Recv", "HcclAmdLoopbackRecv"},
};

const OpEntry* FindOp(const char* opName)
{
    if (opName == nullptr) {
        return nullptr;
    }
    for (const OpEntry& e : kOps) {
        if (strcmp(e.opName, opName) == 0) {
            return &e;
        }
    }
    return nullptr;
}

bool ParamIsSane(const HcclAlgoPluginParam* p)
{
    return p != nullptr && p->magic == HCCL_ALGO_PLUGIN_PARAM_MAGIC && p->version == HCCL_ALGO_PLUGIN_STRUCT_VERSION &&
           p->structSize == sizeof(HcclAlgoPluginParam);
}

bool IsReady() { return true; }

void* FetchContext() { return &g_context; }

bool SelectAlg(void* ctx, const HcclAlgoPluginParam* param, char* algName, size_t algNameLen)
{
    if (ctx != &g_context || !ParamIsSane(param) || algName == nullptr || algNameLen == 0) {
        return false;
    }
    char name[HCCL_ALGO_PLUGIN_OP_NAME_LEN + 1] = {};
    memcpy(name, param->opName, HCCL_ALGO_PLUGIN_OP_NAME_LEN);
    const OpEntry* e = FindOp(name);
    if (e == nullptr || strlen(e->algName) + 1 > algNameLen) {
        return false;
    }
    memcpy(algName, e->algName, strlen(e->algName) + 1);
    return true;
}

int ExecuteAlg(void* ctx, const char* algName, const char* opName, const HcclAlgoPluginParam* param, void* comm)
{
    if (ctx != &g_context || algName == nullptr || !ParamIsSane(param)) {
        return HCCL_E_PARA;
    }
    const OpEntry* e = FindOp(opName);
    if (e == nullptr) {
        return HCCL_E_NOT_SUPPORT;
    }
    if (strcmp(e->algName, algName) != 0) {
        return HCCL_E_NOT_FOUND;
    }
    const HcclAlgoPluginParam& p = *param;
    if (strcmp(opName, "AllReduce") == 0) {
        return HcclAllReduce(p.sendBuf, p.recvBuf, p.count, p.dataType, p.reduceOp, comm, p.stream);
    }
    if (strcmp(opName, "ReduceScatter") == 0) {
        return HcclReduceScatter(p.sendBuf, p.recvBuf, p.count, p.dataType, p.reduceOp, comm, p.stream);
    }
    if (strcmp(opName, "AllGather") == 0) {
        return HcclAllGather(p.sendBuf, p.recvBuf, p.count, p.dataType, comm, p.stream);
    }
    if (strcmp(opName, "Reduce") == 0) {
        return HcclReduce(p.sendBuf, p.recvBuf, p.count, p.dataType, p.reduceOp, p.root, comm, p.stream);
    }
    if (strcmp(opName, "Broadcast") == 0) {
        // the reference passes the one buffer of Broadcast as inputPtr (sendBuf)
        void* buf = p.sendBuf != nullptr ? p.sendBuf : p.recvBuf;
        return HcclBroadcast(buf, p.count, p.dataType, p.root, comm, p.stream);
    }
    if (strcmp(opName, "Scatter") == 0) {
        return HcclScatter(p.sendBuf, p.recvBuf, p.count, p.dataType, p.root, comm, p.stream);
    }
    // the peer of a point-to-point transfer travels as remoteRank (reference hccl_algo_plugin_mgr.cc:251)
    if (strcmp(opName, "Send") == 0) {
        return HcclSend(p.sendBuf, p.count, p.dataType, p.remoteRank, comm, p.stream);
    }
    if (strcmp(opName, "Recv") == 0) {
        return HcclRecv(p.recvBuf, p.count, p.dataType, p.remoteRank, comm, p.stream);
    }
    return HcclAlltoAll(p.sendBuf, p.count, p.dataType, p.recvBuf, p.count, p.dataType, comm, p.stream);
}

int QueryAlgs(void* ctx, const char* opName, char* buf, size_t bufLen)
{
    if (ctx != &g_context || buf == nullptr || bufLen == 0) {
        return HCCL_E_PARA;
    }
    buf[0] = '\0';
    const OpEntry* e = FindOp(opName);
    if (e == nullptr) {
        return HCCL_SUCCESS;   // no algorithm registered for this operator
    }
    const size_t len = strlen(e->algName);
    if (len + 2 > bufLen) {
        return HCCL_E_MEMORY;
    }
    memcpy(buf, e->algName, len + 1);
    buf[len + 1] = '\0';       // the list ends with an empty name
    return HCCL_SUCCESS;
}

HcclAlgoPlugin_t g_table = {HCCL_PLUGIN_API_VERSION, IsReady, FetchContext, SelectAlg, ExecuteAlg, QueryAlgs};

}  // namespace

extern "C" HcclAlgoPlugin_t* GetHcclAlgoPlugin(void) { return &g_table; }
