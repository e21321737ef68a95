/*
 * CPU oracle for the loopback data plane.  TEST INFRASTRUCTURE ONLY.
 *
 * This is a plain-C restatement of what the reference computes on the path
 * "local reduce / slice copy / displacement pack-unpack" of its ring, mesh and
 * recursive-halving-doubling executors.  Only tests/, __graft_entry__.smoke() and the
 * cpu_baseline leg of bench.py may load it; the shipped library never links or calls it.
 *
 * Every function names the reference lines it follows.  Where the reference's own
 * arithmetic is not in its tree (device DMA reduce for int16 / bf16 / fp16-SUM lives in the
 * separate HCOMM library) the function says "parity unpinned" and states the rule used.
 *
 * Reference build status: the host-reduce arithmetic sits in
 * src/ops/op_common/algorithm/template/wrapper/alg_data_trans_wrapper.cc, a translation
 * unit that includes HCOMM / CANN headers which are not part of the reference tree, so it
 * cannot be compiled from its own sources here (no oracle/_ref).  The restatement is pinned
 * instead by IEEE-754 / two's-complement closed forms, exhaustive numpy float16 tables,
 * brute force on tiny inputs and the step tables held by the reference's unit tests.
 */
#ifndef HCCL_ORACLE_H_
#define HCCL_ORACLE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Same numeric values as HcclDataType / HcclReduceOp / HcclResult. */
enum {
    ORC_INT8 = 0, ORC_INT16 = 1, ORC_INT32 = 2, ORC_FP16 = 3, ORC_FP32 = 4, ORC_INT64 = 5, ORC_UINT64 = 6,
    ORC_UINT8 = 7, ORC_UINT16 = 8, ORC_UINT32 = 9, ORC_FP64 = 10, ORC_BF16 = 11
};
enum { ORC_SUM = 0, ORC_PROD = 1, ORC_MAX = 2, ORC_MIN = 3 };
enum { ORC_OK = 0, ORC_E_PARA = 1, ORC_E_PTR = 2, ORC_E_INTERNAL = 4, ORC_E_NOT_SUPPORT = 5 };

/* How fp16 / bf16 SUM chains accumulate.
 *   ORC_ACC_STEP : every pairwise step widens to fp32, adds, and narrows again -- the
 *                  reference's host pattern (AicpuReduceFp16, wrapper.cc:1237-1257).
 *   ORC_ACC_FP32 : operands are widened once, the whole chain runs in fp32 in the
 *                  algorithm's order, one round-to-nearest-even narrowing at the end.
 *                  This is the rule the GPU kernels implement for fp16 / bf16 SUM (the
 *                  reference's device DMA reduce for these is not in its tree: parity
 *                  unpinned; accepted tolerance is 1 ulp against this mode).
 * PROD / MAX / MIN and every non-half type behave identically in both modes except fp16
 * PROD, which always narrows after every step (it only exists on the host path). */
enum { ORC_ACC_STEP = 0, ORC_ACC_FP32 = 1 };

size_t orc_dtype_size(int dtype);

/* --- a2: half conversions (wrapper.cc:1082-1235) ------------------------------------- */
float orc_fp16_to_fp32(uint16_t h);
uint16_t orc_fp32_to_fp16(float f);
/* bf16 has no host path in the reference (parity unpinned): widen = bits << 16; narrow =
 * round-to-nearest-even on the upper 16 bits; NaN keeps its upper 16 bits, the mantissa forced
 * to 1 if they hold none of it (the rule the reference applies to fp16, wrapper.cc:1201-1206), so
 * that widen followed by narrow is the identity on every bf16 pattern. */
float orc_bf16_to_fp32(uint16_t h);
uint16_t orc_fp32_to_bf16(float f);
/* Array forms of the four conversions (same functions applied element by element). */
void orc_fp16_to_fp32_n(const uint16_t* in, float* out, uint64_t n);
void orc_fp32_to_fp16_n(const float* in, uint16_t* out, uint64_t n);
void orc_bf16_to_fp32_n(const uint16_t* in, float* out, uint64_t n);
void orc_fp32_to_bf16_n(const float* in, uint16_t* out, uint64_t n);

/* --- a1/a3: dst[i] = src[i] (+) dst[i] ------------------------------------------------ */
/* Strict restatement of AicpuReduce (wrapper.cc:1259-1316): byte sizes, E_INTERNAL on a size
 * mismatch or on a type outside {int8,int32,fp16,fp32,int64,uint64,fp64}. */
int orc_aicpu_reduce(void* dst, uint64_t dstBytes, const void* src, uint64_t srcBytes, int dtype, int op);
/* Same plus int16 (modular, like int8/int32) and bf16 (fp16 pattern): "by analogy". */
int orc_pair_reduce(void* dst, const void* src, uint64_t count, int dtype, int op);

/* --- a16 / a10 / a11: step geometry (template_utils.cc:32-362) ------------------------ */
#define ORC_INVALID_RANK 0xFFFFFFFFu
typedef struct {
    uint32_t r, effectiveRankSize, virtualRank, inPart1, isRepresentative, pairedAlgRank, unitStart, unitCount,
        isPowerOfTwo;
} orc_rhd_part1_t;
typedef struct {
    uint32_t step, peer, nSlices, txSegStart, txSegEnd, rxSegStart, rxSegEnd;
} orc_rhd_step_t;

uint64_t orc_round_up(uint64_t dividend, uint64_t divisor);       /* template_utils.h:766 */
uint32_t orc_nhr_step_num(uint32_t rankSize);                      /* template_utils.cc:32 */
uint32_t orc_rhd_step_num(uint32_t rankSize);                      /* :42 */
uint32_t orc_rhd_unit_start_of_rank(uint32_t p, uint32_t algRank); /* :93 (sigma) */
uint32_t orc_rhd_alg_rank_of_virtual(uint32_t p, uint32_t root, uint32_t v); /* :101 */
uint32_t orc_rhd_owner_of_unit(uint32_t p, uint32_t unit); /* ins_temp_all_gather_rhd.cc:355-365 */
int orc_rhd_part1(uint32_t p, uint32_t algRank, uint32_t root, orc_rhd_part1_t* info);     /* :117 */
int orc_rhd_rs_steps(const orc_rhd_part1_t* info, orc_rhd_step_t* steps, uint32_t* nSteps); /* :170 */
int orc_rhd_ag_steps(const orc_rhd_part1_t* info, orc_rhd_step_t* steps, uint32_t* nSteps); /* :211 */
int orc_rhd_prepost(const orc_rhd_part1_t* info, orc_rhd_step_t* pre, orc_rhd_step_t* post, int preFull,
                    int postFull);                                                           /* :251 */
void orc_rhd_seg_bytes_uniform(uint32_t unitStart, uint32_t unitEnd, uint64_t sliceSize, uint64_t tailSize,
                               uint32_t tailUnit, uint64_t* offset, uint64_t* len);          /* :310 */
/* ins_v2_all_reduce_sequence_rhd_tail.h:98-113 */
uint64_t orc_rhd_select_loop_count(uint64_t remaining, uint64_t maxCountPerLoop, uint64_t rankAlign);
/* Staging-buffer ("CCL buffer") loop limits.  hccl_op_utils.cc:204-225; sole_executor.cc:241-262;
 * rhd_tail.h:64-92; sequence_executor_aicpu.cc:592-600, 645-675 (one rank per level-0 group). */
int orc_ccl_buffer_available_size(const char* envValue /* NULL = unset */, uint64_t* bytes);
uint64_t orc_sole_max_count_per_loop(uint64_t cclBytes, uint64_t scratchMultiple, uint64_t elemSize);
int orc_rhd_prepare_tail_workspace(uint64_t count, uint64_t rankAlign, uint64_t elemSize, uint64_t* workspaceBytes,
                                   uint64_t* inputOffset, uint64_t* outputOffset);
int orc_rhd_max_count_per_loop(uint64_t cclBytes, uint64_t count, uint32_t p, uint64_t elemSize, uint64_t* maxCount);
/* ins_temp_reduce_scatter_nhr.cc:458-506; tx/rx arrays need rankSize entries. */
int orc_nhr_step_info(uint32_t rankSize, uint32_t algRank, uint32_t step, uint32_t* toRank, uint32_t* fromRank,
                      uint32_t* nSlices, uint32_t* txSliceIdxs, uint32_t* rxSliceIdxs);

/* --- collectives over N loopback ranks ------------------------------------------------
 * in[r] / out[r] are rank r's send / recv buffers (host memory).  accMode is ORC_ACC_*.  */

/* a6/a7/a8: (((x0+x1)+x2)...): one-shot (one_shot.cc:203-242) / host NHR (aicpu_reduce_nhr.cc:266-288). */
int orc_all_reduce_mesh(uint32_t n, const void* const* in, void* const* out, uint64_t count, int dtype, int op,
                        int accMode);
/* a8: two-shot slicing (two_shot.cc:178-210, 326-360) then gather; same values as one-shot. */
int orc_all_reduce_two_shot(uint32_t n, const void* const* in, void* const* out, uint64_t count, int dtype, int op,
                            int accMode);
/* two-shot over symmetric memory (two_shot.cc:341-357): slice k = x_k first, then ranks ascending skipping k. */
int orc_all_reduce_two_shot_symmetric(uint32_t n, const void* const* in, void* const* out, uint64_t count, int dtype,
                                      int op, int accMode);
/* a11: RS-RHD (skip POST) + bridge + AG-RHD (skip PRE), looped per rhd_tail.h; maxCountPerLoop 0 = unbounded. */
int orc_all_reduce_rhd(uint32_t n, const void* const* in, void* const* out, uint64_t count, int dtype, int op,
                       int accMode, uint64_t maxCountPerLoop);
/* a9: own slice first, then ranks ascending (reduce_scatter_mesh_1D.cc:203-237). */
int orc_reduce_scatter_mesh(uint32_t n, const void* const* in, void* const* out, uint64_t recvCount, int dtype,
                            int op, int accMode);
/* a10: write-reduce steps of reduce_scatter_nhr.cc:316-447. */
int orc_reduce_scatter_nhr(uint32_t n, const void* const* in, void* const* out, uint64_t recvCount, int dtype,
                           int op, int accMode);
/* a11: mirror / PRE / MAIN / POST of reduce_scatter_rhd.cc:192-245. */
int orc_reduce_scatter_rhd(uint32_t n, const void* const* in, void* const* out, uint64_t recvCount, int dtype,
                           int op, int accMode);
/* a12: power-of-two block fold (order_preserved_group.cc:306-409). */
int orc_reduce_scatter_order_preserved(uint32_t n, const void* const* in, void* const* out, uint64_t recvCount,
                                       int dtype, int op, int accMode);
int orc_all_reduce_order_preserved(uint32_t n, const void* const* in, void* const* out, uint64_t count, int dtype,
                                   int op, int accMode);
/* vector-core mesh order (aiv_reduce_scatter_mesh_1d.h:23-71). */
int orc_reduce_scatter_aiv_mesh(uint32_t n, const void* const* in, void* const* out, uint64_t recvCount, int dtype,
                                int op, int accMode);
/* Mesh-chunk order, the mesh variant the reference's selectors pick for large messages: every slice is cut
 * into n - 1 segments, segment i of slice k = x_k, then x_{k+i+1}, x_{k+i+2}, ... wrapping past k.
 * reduce_scatter_mesh_1D_meshchunk.cc:233-375, reduce_scatter_v_mesh_1D_meshchunk.cc:147-265,
 * all_reduce_mesh_1D_two_shot_mesh_chunk.cc:86-112, 177-295.  maxCountPerLoop: elements per executor loop, 0 = one
 * loop; ReduceScatterV always runs one loop (reduce_scatter_v_sole_executor.cc:158-171). */
void orc_mesh_chunk_segments(uint64_t len, uint32_t n, uint32_t elemSize, int align4k, uint64_t* segLen /* n-1 */);
int orc_reduce_scatter_mesh_chunk(uint32_t n, const void* const* in, void* const* out, uint64_t recvCount, int dtype,
                                  int op, int accMode, uint64_t maxCountPerLoop);
int orc_reduce_scatter_v_mesh_chunk(uint32_t n, const void* const* in, void* const* out, const uint64_t* counts,
                                    const uint64_t* displs, int dtype, int op, int accMode);
int orc_all_reduce_mesh_chunk(uint32_t n, const void* const* in, void* const* out, uint64_t count, int dtype, int op,
                              int accMode, uint64_t maxCountPerLoop);
/* One-level NHR AllReduce (ins_temp_all_reduce_nhr.cc:214-216, 646-687): slices of floor(count/n) elements, the
 * last slice takes the rest; every element follows the NHR reduce-scatter tree of its slice, then gather. */
int orc_all_reduce_nhr(uint32_t n, const void* const* in, void* const* out, uint64_t count, int dtype, int op,
                       int accMode);
/* Two-level AllReduce of the reference's sequence executor
 * (ins_v2_all_reduce_sequence_executor_aicpu.cc:592-852): l0 consecutive ranks form a level-0 group; inside
 * it a mesh ReduceScatter (own input first), between the groups l1Algo on every chunk, then the AllGathers.
 * maxCountPerLoop 0 = one loop.  l0 == 1 with ORC_L1_RHD is orc_all_reduce_rhd. */
#define ORC_L1_RHD 0
#define ORC_L1_NHR 1
#define ORC_L1_MESH 2
/* Two-level ReduceScatter of the reference's sequence executor (ins_v2_reduce_scatter_sequence_executor_aicpu.cc):
 * mesh ReduceScatter inside boxes of l0 consecutive ranks, then the level-1 template (ORC_L1_*) between the boxes. */
int orc_reduce_scatter_two_level(uint32_t n, uint32_t l0, int l1Algo, const void* const* in, void* const* out,
                                 uint64_t recvCount, int dtype, int op, int accMode);
int orc_all_reduce_two_level(uint32_t n, uint32_t l0, int l1Algo, const void* const* in, void* const* out,
                             uint64_t count, int dtype, int op, int accMode, uint64_t maxCountPerLoop);
/* Three levels (ins_v2_all_reduce_sequence_executor_aicpu_3level.cc, ins_v2_reduce_scatter_sequence_executor_3level.cc,
 * reduce_sequence_executor_aicpu_3level.cc): l0 consecutive ranks form a box, l1 consecutive boxes a pod; the mesh
 * ReduceScatter inside the boxes, `algo` (ORC_L1_RHD or ORC_L1_NHR) between the boxes of a pod and once more between
 * the pods.  cclBytes: the staging buffer whose loops show in the cuts of AllReduce and Reduce, 0 = one loop.
 * orc_reduce_levels also is the two-level Reduce (l1 = n / l0; ORC_L1_MESH allowed there: the host-reduce fold). */
int orc_all_reduce_three_level(uint32_t n, uint32_t l0, uint32_t l1, int algo, const void* const* in,
                               void* const* out, uint64_t count, int dtype, int op, int accMode, uint64_t cclBytes);
int orc_reduce_scatter_three_level(uint32_t n, uint32_t l0, uint32_t l1, int algo, const void* const* in,
                                   void* const* out, uint64_t recvCount, int dtype, int op, int accMode);
int orc_reduce_levels(uint32_t n, uint32_t l0, uint32_t l1, int algo, const void* const* in, void* const* out,
                      uint64_t count, int dtype, int op, uint32_t root, int accMode, uint64_t cclBytes);
int orc_sequence_max_count_per_loop(uint64_t cclBytes, uint64_t count, uint32_t l0, uint32_t total, uint64_t esz,
                                    uint64_t align, int rhdTail, uint64_t* maxCount, uint64_t* resultElems);
uint64_t orc_sequence_select_loop_count(uint64_t remaining, uint64_t maxCountPerLoop, uint32_t l0,
                                        uint64_t resultElems);
/* AllReduce of the two-shot executor over one mesh (ins_v2_all_reduce_two_shot_sole_executor.cc): slices of
 * floor(len / n) elements, the last taking the rest, slice k folded own input first; maxCountPerLoop 0 = one loop. */
int orc_all_reduce_mesh_concur(uint32_t n, const void* const* in, void* const* out, uint64_t count, int dtype, int op,
                               int accMode, uint64_t maxCountPerLoop);
/* Reduce along the NHR step tree on slices of ceil(len / n) elements (reduce_nhr.cc); only out[root] is written. */
int orc_reduce_nhr(uint32_t n, const void* const* in, void* const* out, uint64_t count, int dtype, int op, int accMode,
                   uint32_t root, uint64_t maxCountPerLoop);

/* The same inside the executor's loop over the staging buffer (ins_v2_all_reduce_sole_executor.cc:266-300):
 * every loop of maxCountPerLoop elements (the last one shorter) is sliced afresh; 0 = one loop. */
int orc_all_reduce_nhr_looped(uint32_t n, const void* const* in, void* const* out, uint64_t count, int dtype, int op,
                              int accMode, uint64_t maxCountPerLoop);

/* a13: all_gather_mesh_1D.cc:249-423. */
int orc_all_gather(uint32_t n, const void* const* in, void* const* out, uint64_t sendCount, int dtype);
/* a14: all_gather_v_mesh_1D.cc:242-310; counts/displs are the (identical) per-rank arrays. */
int orc_all_gather_v(uint32_t n, const void* const* in, void* const* out, const uint64_t* recvCounts,
                     const uint64_t* recvDispls, int dtype);
/* a15: all_to_all_v_mesh_1D.cc:229-246, 459-611.  The four tables are n x n row-major,
 * row r = rank r's argument array. */
int orc_all_to_all_v(uint32_t n, const void* const* in, void* const* out, const uint64_t* sendCounts,
                     const uint64_t* sdispls, const uint64_t* recvCounts, const uint64_t* rdispls, int dtype);

/* AlltoAll (all_to_all_v.cc:24-82, 411-421): every rank sends `count` elements to every rank,
 * sdispls[i] = rdispls[i] = i * count; then orc_all_to_all_v. */
int orc_all_to_all(uint32_t n, const void* const* in, void* const* out, uint64_t count, int dtype);
/* AlltoAllVC parameter conversion for one rank (all_to_all_v.cc:423-458): sendCounts = row `rank` of the
 * n x n matrix, recvCounts = column `rank`, both displacement arrays = exclusive prefix sums. */
void orc_all_to_all_vc_params(uint32_t n, uint32_t rank, const uint64_t* matrix, uint64_t* sendCounts,
                              uint64_t* recvCounts, uint64_t* sdispls, uint64_t* rdispls);
/* AlltoAllVC (all_to_all_v.cc:153-209): convert per rank, then orc_all_to_all_v. */
int orc_all_to_all_vc(uint32_t n, const void* const* in, void* const* out, const uint64_t* matrix, int dtype);

/* ReduceScatterV mesh (ins_temp_reduce_scatter_v_mesh_1D.cc:109-162, executor :117-215): counts / displs
 * are the (identical) per-rank arrays; rank k: out = in_k[displs[k] .. +counts[k]); for t = 0..N-1, t != k:
 * out = in_t[displs[k] ..] (+) out.  Types as the entry point admits (reduce_scatter_v.cc:225-247: no
 * uint64 / fp64). */
int orc_reduce_scatter_v_mesh(uint32_t n, const void* const* in, void* const* out, const uint64_t* counts,
                              const uint64_t* displs, int dtype, int op, int accMode);
/* Reduce mesh (reduce_mesh_1D.cc:268-300): slot r = rank r's input; out_root = slot 0, then
 * out_root = slot_idx (+) out_root for idx = 1..N-1.  Only out[root] is written. */
int orc_reduce_mesh(uint32_t n, const void* const* in, void* const* out, uint64_t count, int dtype, int op,
                    int accMode, uint32_t root);
/* Reduce two-shot (reduce_mesh_1D_two_shot.cc:138-162, 228-265): every executor loop deals its elements into n
 * slices, the first len mod n one longer; slice k = x_k first, then the other ranks ascending; out[root] only. */
int orc_reduce_two_shot(uint32_t n, const void* const* in, void* const* out, uint64_t count, int dtype, int op,
                        int accMode, uint32_t root, uint64_t maxCountPerLoop);
/* Broadcast (hccl.h:52-53): buf_r = buf_root for every r. */
int orc_broadcast(uint32_t n, void* const* buf, uint64_t count, int dtype, uint32_t root);
/* Scatter (hccl.h:107-109): out_r = in_root[r * recvCount .. +recvCount). */
int orc_scatter(uint32_t n, const void* const* in, void* const* out, uint64_t recvCount, int dtype, uint32_t root);

/* a5: LocalCopySlices merge rule (wrapper.cc:930-997): returns how many copies are issued
 * for slices (offset,size) over one base address; copies[] gets (srcOff,dstOff,size) triples. */
uint32_t orc_local_copy_slices(uint32_t nSlices, const uint64_t* srcOff, const uint64_t* dstOff,
                               const uint64_t* sizes, uint64_t* copies);

/* Multi-threaded variants used only for the "all cores" CPU baseline: the element range is
 * split statically over nThreads. */
int orc_reduce_scatter_mesh_mt(uint32_t n, const void* const* in, void* const* out, uint64_t recvCount, int dtype,
                               int op, int accMode, uint32_t nThreads);
int orc_all_reduce_mesh_mt(uint32_t n, const void* const* in, void* const* out, uint64_t count, int dtype, int op,
                           int accMode, uint32_t nThreads);

/* --- point to point ----------------------------------------------------------------------
 * BatchSendRecv over n loopback ranks: items[r] / itemNum[r] are rank r's array.  Every rank sorts its sends and
 * its receives pair-wise (peer order, then count descending, then data type descending, stable;
 * ins_v2_batch_send_recv_executor.cc:105-128, 137-200) and the k-th send of a to b meets the k-th receive from a
 * at b.  A transfer without counterpart or with unequal count / type is E_PARA.  Plain Send / Recv are batches of
 * one item. */
typedef struct {
    int sendRecvType;      /* 0 send, 1 receive */
    void* buf;
    uint64_t count;
    int dataType;
    uint32_t remoteRank;
} orc_send_recv_item_t;
int orc_batch_send_recv(uint32_t n, const orc_send_recv_item_t* const* items, const uint32_t* itemNum);

/* --- a16: AlltoAllV's variable-length argument area --------------------------------------
 * all_to_all_v.cc:600-643 (CalcInputOutputSize, ConstructVarData), template_utils.h:110-159
 * (ParseAlltoAllVarData: out = sendCounts, sendLength, recvCounts, recvLength, sendDispls, sendOffset,
 * recvDispls, recvOffset, n values each). */
void orc_a2a_construct_var_data(uint32_t n, const uint64_t* sendCounts, const uint64_t* recvCounts,
                                const uint64_t* sdispls, const uint64_t* rdispls, uint64_t* varData);
int orc_a2a_parse_var_data(const uint64_t* varData, uint64_t varBytes, uint64_t n, uint64_t elemSize, int isVC,
                           uint64_t* out);
void orc_a2a_io_size(uint32_t n, const uint64_t* sendCounts, const uint64_t* recvCounts, const uint64_t* sdispls,
                     const uint64_t* rdispls, uint64_t elemSize, uint64_t* inputBytes, uint64_t* outputBytes);

/* a4: LocalReduce's routing (wrapper.cc:901-928): 1 = host arithmetic (64-bit types, PROD), 0 = device. */
int orc_local_reduce_runs_on_host(int dtype, int op);

#ifdef __cplusplus
}
#endif
#endif /* HCCL_ORACLE_H_ */
