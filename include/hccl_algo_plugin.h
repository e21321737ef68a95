/*
 * Algorithm-plugin surface: the function table the reference's plugin manager fetches from a
 * "PluginBroker" shared library with dlsym("GetHcclAlgoPlugin") and then uses to let a custom
 * algorithm take over selection and execution of an operator.
 *
 * Layouts, constants and the exported symbol follow the reference's plugin interface so that the
 * table can be handed to its manager unchanged:
 *   HcclAlgoPluginParam  reference src/algo_plugin/inc/hccl_algo_plugin_common.h:74-101
 *   constants            reference src/algo_plugin/inc/hccl_algo_plugin_common.h:53-68
 *   HcclAlgoPlugin_t     reference src/algo_plugin/inc/hccl_algo_plugin_broker_api.h:24-49
 *   GetHcclAlgoPlugin    reference src/algo_plugin/inc/hccl_algo_plugin_broker_api.h:52-55
 *   how it is called     reference src/algo_plugin/hccl_algo_plugin_mgr.cc (load, validate),
 *                        src/ops/op_common/op_common.cc:137 (SelectAlg), :1014 (ExecuteAlg)
 *
 * libhccl_amd_plugin_broker.so implements the table on top of libhccl_amd.so.  The `comm` handed to
 * ExecuteAlg must be a communicator of this library (HcclCommInitAll / HcclCommInitRootInfo).
 */
#ifndef HCCL_AMD_HCCL_ALGO_PLUGIN_H_
#define HCCL_AMD_HCCL_ALGO_PLUGIN_H_

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#include "hccl_types.h"

#ifdef __cplusplus
extern "C" {
#endif

#define HCCL_PLUGIN_API_VERSION 1U
#define HCCL_ALGO_PLUGIN_STRUCT_VERSION 1U
#define HCCL_ALGO_PLUGIN_PARAM_MAGIC 0x48415050U   /* "HAPP" */
#define HCCL_ALGO_PLUGIN_ALG_NAME_LEN 128U
#define HCCL_ALGO_PLUGIN_OP_NAME_LEN 32U
#define HCCL_ALGO_PLUGIN_TOPO_NAME_LEN 32U

/* What the caller knows about one operator invocation.  Field order and widths are the ABI. */
typedef struct {
    uint32_t version;          /* HCCL_ALGO_PLUGIN_STRUCT_VERSION */
    uint32_t magic;            /* HCCL_ALGO_PLUGIN_PARAM_MAGIC */
    uint32_t structSize;       /* sizeof(HcclAlgoPluginParam) */
    int opType;                /* informational */
    char opName[HCCL_ALGO_PLUGIN_OP_NAME_LEN];   /* "AllReduce", "ReduceScatter", ... : selects the operator */
    uint64_t count;            /* elements */
    uint32_t root;             /* Broadcast / Reduce / Scatter */
    int topoType;              /* informational */
    char topoName[HCCL_ALGO_PLUGIN_TOPO_NAME_LEN];
    uint32_t rankNum;
    uint32_t serverNum;
    void* sendBuf;
    void* recvBuf;
    aclrtStream stream;
    HcclDataType dataType;
    HcclReduceOp reduceOp;
    uint32_t remoteRank;
    uint32_t deviceNumPerModule;
    uint32_t moduleNum;
    uint32_t superPodNum;
    uint32_t serverNumPerSuperPod;
    bool isAsymmetricTopo;
    uint32_t reserved[7];
} HcclAlgoPluginParam;

typedef struct HcclAlgoPlugin_t {
    uint32_t version;                   /* must equal HCCL_PLUGIN_API_VERSION */
    bool (*IsReady)(void);
    void* (*FetchContext)(void);        /* ctx argument of the three calls below */
    /* true: algName names the algorithm that takes this invocation; false: the caller keeps its own. */
    bool (*SelectAlg)(void* ctx, const HcclAlgoPluginParam* param, char* algName, size_t algNameLen);
    /* Runs the algorithm; the result is an HcclResult. */
    int (*ExecuteAlg)(void* ctx, const char* algName, const char* opName, const HcclAlgoPluginParam* param,
                      void* comm);
    /* Writes the '\0'-separated algorithm names registered for opName into buf; returns an HcclResult. */
    int (*QueryAlgs)(void* ctx, const char* opName, char* buf, size_t bufLen);
} HcclAlgoPlugin_t;

#define HCCL_ALGO_PLUGIN_GET_TABLE_SYMBOL "GetHcclAlgoPlugin"
HcclAlgoPlugin_t* GetHcclAlgoPlugin(void);

/*
 * Selector libraries.  The reference's own PluginBroker does not implement algorithms: for every operator
 * directory <HCCL_PLUGIN_ALG_DIR>/<OpName>/ it loads libhccl_plugin_<opname>_selector.so, copies the entries
 * HcclAlgoPluginQueryEntries() returns, asks Select() per invocation and then calls the symbol `fnSymbol` of
 * the library `soPath`, which must have the operator's hccl.h signature (reference
 * experimental/eco_system/algo_plugin/hccl_algo_plugin/plugin_broker/src/plugin_broker.cc:140-207, 280-330;
 * entry layout src/algo_plugin/inc/hccl_algo_plugin_common.h:104-115; exported symbols
 * experimental/eco_system/algo_plugin/hccl_algo_plugin/sdk/hccl_algo_plugin_sdk.h:168-181).
 * hccl_amd/plugin_algs/<OpName>/libhccl_plugin_<opname>_selector.so are such libraries: one entry each,
 * naming libhccl_amd.so and its hccl.h entry point.
 */
#define HCCL_ALGO_PLUGIN_ENTRY_MAGIC 0x48415045U   /* "HAPE" */
#define HCCL_ALGO_PLUGIN_SO_PATH_LEN 512U
#define HCCL_ALGO_PLUGIN_FN_SYMBOL_LEN 128U

typedef struct {
    uint32_t version;          /* HCCL_ALGO_PLUGIN_STRUCT_VERSION */
    uint32_t magic;            /* HCCL_ALGO_PLUGIN_ENTRY_MAGIC */
    uint32_t structSize;       /* sizeof(HcclAlgoPluginAlgEntry) */
    char algName[HCCL_ALGO_PLUGIN_ALG_NAME_LEN];
    char soPath[HCCL_ALGO_PLUGIN_SO_PATH_LEN];       /* library that implements the algorithm */
    char fnSymbol[HCCL_ALGO_PLUGIN_FN_SYMBOL_LEN];   /* its entry point, with the operator's hccl.h signature */
} HcclAlgoPluginAlgEntry;

/* Exported by every selector library. */
const HcclAlgoPluginAlgEntry* HcclAlgoPluginQueryEntries(int* count);
bool Select(const HcclAlgoPluginParam* param, char* algName, size_t algNameLen);

#ifdef __cplusplus
}
#endif
#endif /* HCCL_AMD_HCCL_ALGO_PLUGIN_H_ */
