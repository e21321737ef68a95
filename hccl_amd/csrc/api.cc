// Host layer of the loopback data plane: the C ABI of include/hccl.h over HIP streams.
//
// What the reference spreads over op entry / selector / executor / template / wrapper
// (src/ops/<op>/<op>.cc -> op_common.cc Selector + HcclExecOp -> executor -> template ->
// alg_data_trans_wrapper.cc) collapses here to: argument checks with the reference's return codes,
// a rendezvous of the N per-rank calls, and one fused kernel launch per collective.
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
    if (c->world->level1 != 0 && (c->world->n / ranksPerGroup) % c->world->level1 != 0) {
        c->world->level1 = 0;   // the level-1 groups no longer divide the level-0 groups: back to two levels
    }
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

HcclResult HcclAmdSetLevel1GroupSize(HcclComm comm, uint32_t groupsPerLevel1Group)
{
    CHK_PTR(comm, "comm");
    CommRef ref = AsComm(comm);
    Comm* c = ref.c;
    if (c == nullptr) {
        return HCCL_E_PARA;
    }
    std::lock_guard<std::mutex> wl(c->world->mu);
    const uint32_t groups = c->world->n / c->world->level0;
    if (groupsPerLevel1Group != 0 && (groupsPerLevel1Group > groups || groups % groupsPerLevel1Group != 0)) {
        return HCCL_E_PARA;
    }
    c->world->level1 = groupsPerLevel1Group;
    return HCCL_SUCCESS;
}

HcclResult HcclAmdGetLevel1GroupSize(HcclComm comm, uint32_t* groupsPerLevel1Group)
{
    CHK_PTR(comm, "comm");
    CHK_PTR(groupsPerLevel1Group, "groupsPerLevel1Group");
    CommRef ref = AsComm(comm);
    Comm* c = ref.c;
    if (c == nullptr) {
        return HCCL_E_PARA;
    }
    std::lock_guard<std::mutex> wl(c->world->mu);
    *groupsPerLevel1Group = c->world->level1;
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
    return HcclAmdGetFoldProgramLevels(op, algo, rankSize, 1, 0, segment, out, cap, len, segmentCount);
}

HcclResult HcclAmdGetFoldProgramTwoLevel(HcclAmdOpKind op, HcclAmdAlgo algo, uint32_t rankSize, uint32_t level0,
                                         uint32_t segment, uint8_t* out, uint32_t cap, uint32_t* len,
                                         uint32_t* segmentCount)
{
    return HcclAmdGetFoldProgramLevels(op, algo, rankSize, level0, 0, segment, out, cap, len, segmentCount);
}

HcclResult HcclAmdGetFoldProgramLevels(HcclAmdOpKind op, HcclAmdAlgo algo, uint32_t rankSize, uint32_t level0,
                                       uint32_t level1, uint32_t segment, uint8_t* out, uint32_t cap, uint32_t* len,
                                       uint32_t* segmentCount)
{
    CHK_PTR(len, "len");
    // Callers walk all segments of one plan: keep the last plan built.
    static std::mutex cacheMu;
    static FoldPlan plan;
    static int cachedOp = -1, cachedAlgo = -1;
    static uint32_t cachedSize = 0, cachedLevel0 = 0, cachedLevel1 = 0;
    std::lock_guard<std::mutex> cacheLock(cacheMu);
    if (cachedOp != static_cast<int>(op) || cachedAlgo != static_cast<int>(algo) || cachedSize != rankSize ||
        cachedLevel0 != level0 || cachedLevel1 != level1) {
        cachedOp = -1;
        HcclResult rc = BuildFoldPlan(op, algo, rankSize, &plan, level0, level1);
        if (rc != HCCL_SUCCESS) {
            return rc;
        }
        cachedOp = static_cast<int>(op);
        cachedAlgo = static_cast<int>(algo);
        cachedSize = rankSize;
        cachedLevel0 = level0;
        cachedLevel1 = level1;
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
