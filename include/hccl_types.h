/*
 * Scalar types shared by every entry point of the MI355X loopback data plane.
 *
 * The reference gets these from CANN headers that are not part of its tree
 * (reference include/hccl.h:14-16 includes <hccl/hccl_types.h>, <hccl/hccl_comm.h>,
 * <acl/acl.h>).  The numeric values below are the ones the reference's own sources
 * rely on:
 *   - data type order and element sizes: reference
 *     src/ops/op_common/inc/alg_param.h:55-73 (DATATYPE_SIZE_TABLE) and
 *     src/common/hccl_common.h:50-67 (value 13 is a reserved gap, 255 is RESERVED);
 *   - reduce op order SUM/PROD/MAX/MIN: reference
 *     test/ut/all_reduce_aiv/stub/aiv_communication_base_v2.h:49-54;
 *   - HCCL_E_NOT_SUPPORT == 5: reference
 *     experimental/eco_system/python/tests/_platform.py:463-475; the other result
 *     codes follow the public CANN numbering (PARA=1, PTR=2, MEMORY=3, INTERNAL=4 ...).
 */
#ifndef HCCL_AMD_HCCL_TYPES_H_
#define HCCL_AMD_HCCL_TYPES_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
    HCCL_SUCCESS = 0,
    HCCL_E_PARA = 1,
    HCCL_E_PTR = 2,
    HCCL_E_MEMORY = 3,
    HCCL_E_INTERNAL = 4,
    HCCL_E_NOT_SUPPORT = 5,
    HCCL_E_NOT_FOUND = 6,
    HCCL_E_UNAVAIL = 7,
    HCCL_E_SYSCALL = 8,
    HCCL_E_TIMEOUT = 9,
    HCCL_E_OPEN_FILE_FAILURE = 10,
    HCCL_E_TCP_CONNECT = 11,
    HCCL_E_ROCE_CONNECT = 12,
    HCCL_E_TCP_TRANSFER = 13,
    HCCL_E_ROCE_TRANSFER = 14,
    HCCL_E_RUNTIME = 15,
    HCCL_E_DRV = 16,
    HCCL_E_PROFILING = 17,
    HCCL_E_CCE = 18,
    HCCL_E_NETWORK = 19,
    HCCL_E_AGAIN = 20,
    HCCL_E_REMOTE = 21,
    HCCL_E_SUSPENDING = 22,
    HCCL_E_RESERVED
} HcclResult;

typedef enum {
    HCCL_REDUCE_SUM = 0,
    HCCL_REDUCE_PROD = 1,
    HCCL_REDUCE_MAX = 2,
    HCCL_REDUCE_MIN = 3,
    HCCL_REDUCE_RESERVED
} HcclReduceOp;

typedef enum {
    HCCL_DATA_TYPE_INT8 = 0,
    HCCL_DATA_TYPE_INT16 = 1,
    HCCL_DATA_TYPE_INT32 = 2,
    HCCL_DATA_TYPE_FP16 = 3,
    HCCL_DATA_TYPE_FP32 = 4,
    HCCL_DATA_TYPE_INT64 = 5,
    HCCL_DATA_TYPE_UINT64 = 6,
    HCCL_DATA_TYPE_UINT8 = 7,
    HCCL_DATA_TYPE_UINT16 = 8,
    HCCL_DATA_TYPE_UINT32 = 9,
    HCCL_DATA_TYPE_FP64 = 10,
    HCCL_DATA_TYPE_BFP16 = 11,
    HCCL_DATA_TYPE_INT128 = 12,
    /* 13 is a reserved gap */
    HCCL_DATA_TYPE_HIF8 = 14,
    HCCL_DATA_TYPE_FP8E4M3 = 15,
    HCCL_DATA_TYPE_FP8E5M2 = 16,
    HCCL_DATA_TYPE_FP8E8M0 = 17,
    HCCL_DATA_TYPE_RESERVED = 255
} HcclDataType;

/* One transfer of HcclBatchSendRecv.  The type comes from the CANN headers, which are not part of the
 * reference tree; the tree fixes the field names (src/ops/batch_send_recv/algorithm/executor/
 * ins_v2_batch_send_recv_executor.cc:143-160), their order as the Python constructor fills them
 * (experimental/eco_system/python/hccl4py/ops.py:485-498) and "0: send, 1: recv"
 * (src/ops/op_common/algorithm/template/aiv/hccl_aiv_utils.h:111). */
typedef enum {
    HCCL_SEND = 0,
    HCCL_RECV = 1,
    HCCL_SEND_RECV_RESERVED
} HcclSendRecvType;

typedef struct HcclSendRecvItemDef {
    HcclSendRecvType sendRecvType;
    void* buf;
    uint64_t count;        /* elements */
    HcclDataType dataType;
    uint32_t remoteRank;   /* destination of a send, source of a receive */
} HcclSendRecvItem;

/* Opaque communicator handle: one per rank of a loopback world. */
typedef void* HcclComm;

/* Stream handle.  On MI355X this is a hipStream_t passed through unchanged. */
typedef void* aclrtStream;

/* Largest element count one call accepts (reference src/common/hccl_common.h:42). */
#define HCCL_SYS_MAX_COUNT 0x7FFFFFFFFULL

/* Largest rank count of one loopback world. */
#define HCCL_AMD_MAX_RANKS 64

#define HCCL_ROOT_INFO_BYTES 4108
typedef struct HcclRootInfoDef {
    char internal[HCCL_ROOT_INFO_BYTES];
} HcclRootInfo;

#ifdef __cplusplus
}
#endif
#endif /* HCCL_AMD_HCCL_TYPES_H_ */
