// Selector library for the reference's own PluginBroker: compiled once per operator
// (-DHCCL_AMD_SELECTOR_OP=\"AllReduce\" -DHCCL_AMD_SELECTOR_FN=\"HcclAllReduce\") into
// plugin_algs/<Op>/libhccl_plugin_<op>_selector.so.  It registers one algorithm, implemented by the hccl.h entry
// point of libhccl_amd.so, and selects it for every invocation that entry point admits; anything else is left
// to the caller's own algorithms.  The library that implements the algorithm is $HCCL_AMD_LIBRARY if set, else
// libhccl_amd.so two directories above this file (the in-tree layout hccl_amd/plugin_algs/<Op>/).
#include <dlfcn.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>

#include "hccl_algo_plugin.h"

#ifndef HCCL_AMD_SELECTOR_OP
#error "define HCCL_AMD_SELECTOR_OP and HCCL_AMD_SELECTOR_FN"
#endif

namespace {

constexpr const char* kOpName = HCCL_AMD_SELECTOR_OP;
constexpr const char* kFnSymbol = HCCL_AMD_SELECTOR_FN;
constexpr const char* kAlgName = "HcclAmdLoopback" HCCL_AMD_SELECTOR_OP;

bool Fits(char* dst, size_t cap, const std::string& src)
{
    if (src.size() + 1 > cap) {
        return false;
    }
    memcpy(dst, src.c_str(), src.size() + 1);
    return true;
}

std::string ImplementationLibrary()
{
    if (const char* env = getenv("HCCL_AMD_LIBRARY")) {
        if (env[0] != '\0') {
            return env;
        }
    }
    Dl_info info{};
    if (dladdr(reinterpret_cast<const void*>(&ImplementationLibrary), &info) == 0 || info.dli_fname == nullptr) {
        return "libhccl_amd.so";   // left to the loader's search path
    }
    std::string dir(info.dli_fname);
    for (int up = 0; up < 3; ++up) {   // file name, <Op>/, plugin_algs/
        size_t slash = dir.find_last_of('/');
        if (slash == std::string::npos) {
            return "libhccl_amd.so";
        }
        dir.erase(slash);
    }
    return dir + "/libhccl_amd.so";
}

HcclAlgoPluginAlgEntry g_entry;
int g_entryCount = 0;
std::once_flag g_once;

void BuildEntry()
{
    memset(&g_entry, 0, sizeof(g_entry));
    g_entry.version = HCCL_ALGO_PLUGIN_STRUCT_VERSION;
    g_entry.magic = HCCL_ALGO_PLUGIN_ENTRY_MAGIC;
    g_entry.structSize = sizeof(HcclAlgoPluginAlgEntry);
    if (Fits(g_entry.algName, sizeof(g_entry.algName), kAlgName) &&
        Fits(g_entry.soPath, sizeof(g_entry.soPath), ImplementationLibrary()) &&
        Fits(g_entry.fnSymbol, sizeof(g_entry.fnSymbol), kFnSymbol)) {
        g_entryCount = 1;
    } else {
        fprintf(stderr, "[hccl_amd][ERROR] %s selector: the path of the implementation library is too long\n", kOpName);
    }
}

// What the entry points of include/hccl.h accept (reference src/ops/op_common/op_common.cc:4323-4413).
bool Admitted(const HcclAlgoPluginParam* p, bool reduces)
{
    const int t = static_cast<int>(p->dataType);
    if (t < 0 || t > 17 || t == 13 || p->dataType == HCCL_DATA_TYPE_INT128) {
        return false;
    }
    if (!reduces) {
        return true;
    }
    switch (p->dataType) {
        case HCCL_DATA_TYPE_UINT8:
        case HCCL_DATA_TYPE_UINT16:
        case HCCL_DATA_TYPE_UINT32:
        case HCCL_DATA_TYPE_HIF8:
        case HCCL_DATA_TYPE_FP8E4M3:
        case HCCL_DATA_TYPE_FP8E5M2:
        case HCCL_DATA_TYPE_FP8E8M0:
            return false;
        default:
            break;
    }
    if (static_cast<int>(p->reduceOp) < 0 || static_cast<int>(p->reduceOp) >= static_cast<int>(HCCL_REDUCE_RESERVED)) {
        return false;
    }
    if (p->reduceOp == HCCL_REDUCE_PROD) {
        return p->dataType != HCCL_DATA_TYPE_INT16 && p->dataType != HCCL_DATA_TYPE_BFP16;
    }
    return true;
}

}  // namespace

extern "C" {

__attribute__((visibility("default"))) const HcclAlgoPluginAlgEntry* HcclAlgoPluginQueryEntries(int* count)
{
    std::call_once(g_once, BuildEntry);
    if (count != nullptr) {
        *count = g_entryCount;
    }
    return g_entryCount != 0 ? &g_entry : nullptr;
}

__attribute__((visibility("default"))) bool Select(const HcclAlgoPluginParam* param, char* algName, size_t algNameLen)
{
    if (param == nullptr || algName == nullptr || algNameLen == 0 || param->magic != HCCL_ALGO_PLUGIN_PARAM_MAGIC ||
        param->version != HCCL_ALGO_PLUGIN_STRUCT_VERSION || param->structSize != sizeof(HcclAlgoPluginParam)) {
        return false;
    }
    if (strncmp(param->opName, kOpName, HCCL_ALGO_PLUGIN_OP_NAME_LEN) != 0) {
        return false;
    }
    if (const char* off = getenv("HCCL_AMD_PLUGIN_SELECT")) {
        if (strcmp(off, "0") == 0) {
            return false;   // installed but switched off: the caller keeps its own algorithms
        }
    }
    const bool reduces = strcmp(kOpName, "AllReduce") == 0 || strcmp(kOpName, "ReduceScatter") == 0 ||
                         strcmp(kOpName, "Reduce") == 0;
    if (!Admitted(param, reduces) || strlen(kAlgName) + 1 > algNameLen) {
        return false;
    }
    memcpy(algName, kAlgName, strlen(kAlgName) + 1);
    return true;
}

}  // extern "C"
