/*
 * C ABI of the MI355X loopback data plane.
 *
 * The collective entry points have the signatures of the reference's public
 * header (reference include/hccl.h) so that a caller built against that header links
 * against this library unchanged.  `aclrtStream` carries a hipStream_t; every buffer
 * is a device pointer in the HBM of the one GPU; count / displacement arrays are host
 * arrays of uint64_t in elements and are copied during the call.
 *
 * A "world" is a rankSize-N loopback communicator: N HcclComm handles in one process
 * whose send/recv buffers are separate HBM allocations of the same GPU.  One
 * collective is N calls (one per rank, identical count / type / op); the call that
 * completes the set launches ONE fused kernel that performs every rank's share of
 * the work and orders every rank's stream after it.
 *
 * Calling conventions (two are supported):
 *   - one host thread per rank (the reference's examples/02_collectives pattern):
 *     each call blocks on the host until all N ranks have called, then returns with
 *     the work enqueued behind the caller's stream;
 *   - one host thread driving all ranks: bracket the N calls with HcclGroupStart() /
 *     HcclGroupEnd(); calls inside a group never block.
 */
#ifndef HCCL_AMD_HCCL_H_
#define HCCL_AMD_HCCL_H_

#include "hccl_types.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------------------------------
 * Collectives (the drop-in boundary)
 * ---------------------------------------------------------------------------------------- */

/*
 * recvBuf[i] = sendBuf_0[i] (+) sendBuf_1[i] (+) ... over all ranks, for i in [0, count),
 * written to every rank's recvBuf.  Replaces reference include/hccl.h:36-38
 * (implementation src/ops/all_reduce/all_reduce.cc:23).  In-place (sendBuf == recvBuf)
 * is allowed.  count == 0 succeeds without touching anything.
 */
HcclResult HcclAllReduce(void* sendBuf, void* recvBuf, uint64_t count, HcclDataType dataType, HcclReduceOp op,
                         HcclComm comm, aclrtStream stream);

/*
 * Rank k's recvBuf[0, recvCount) = reduction over ranks t of sendBuf_t[k*recvCount + i].
 * Replaces reference include/hccl.h:69-71 (src/ops/reduce_scatter/reduce_scatter.cc:24).
 */
HcclResult HcclReduceScatter(void* sendBuf, void* recvBuf, uint64_t recvCount, HcclDataType dataType,
                             HcclReduceOp op, HcclComm comm, aclrtStream stream);

/*
 * Every rank's recvBuf[r*sendCount + i] = sendBuf_r[i].
 * Replaces reference include/hccl.h:123-124 (src/ops/all_gather/all_gather.cc:23).
 */
HcclResult HcclAllGather(void* sendBuf, void* recvBuf, uint64_t sendCount, HcclDataType dataType, HcclComm comm,
                         aclrtStream stream);

/*
 * Every rank's recvBuf[recvDispls[r] + i] = sendBuf_r[i], i in [0, recvCounts[r]).
 * recvCounts / recvDispls: host uint64_t[rankSize], elements.  Intervals may be unordered
 * and have holes but must not overlap.  Replaces reference include/hccl.h:141-143
 * (src/ops/all_gather_v/all_gather_v.cc:23).
 */
HcclResult HcclAllGatherV(void* sendBuf, uint64_t sendCount, void* recvBuf, const void* recvCounts,
                          const void* recvDispls, HcclDataType dataType, HcclComm comm, aclrtStream stream);

/*
 * Rank i's recvBuf[rdispls_i[j] + e] = sendBuf_j[sdispls_j[i] + e], e in [0, sendCounts_j[i]),
 * with recvCounts_i[j] == sendCounts_j[i].  All four arrays: host uint64_t[rankSize], elements.
 * Replaces reference include/hccl.h:215-217 (src/ops/all_to_all_v/all_to_all_v.cc:85).
 */
HcclResult HcclAlltoAllV(const void* sendBuf, const void* sendCounts, const void* sdispls, HcclDataType sendType,
                         const void* recvBuf, const void* recvCounts, const void* rdispls, HcclDataType recvType,
                         HcclComm comm, aclrtStream stream);

/*
 * HcclAlltoAllV for callers that cannot allocate (code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc).  No counterpart in the reference.  Same arguments, checks and result as
 * HcclAlltoAllV; every rank of a collective must call the same variant (HCCL_E_PARA otherwise).  The
 * segment tables live in a device array that is part of the library (164,096 bytes per GPU, held until the
 * process ends) and reach it inside kernel arguments, so the call performs no hipMalloc / hipFree /
 * hipHostMalloc and no copy from host memory (its bookkeeping on the host uses the process heap like every
 * other entry point's).  The first call in a world looks up the array's address and creates the events later
 * calls use.  HCCL_E_MEMORY if the tables of the call's non-empty segments exceed the array (cannot happen up
 * to HCCL_AMD_MAX_RANKS ranks).  All calls on one GPU share the array and the library puts them in order: a
 * call's table writes wait (hipStreamWaitEvent, no allocation) for the copy kernel of the call before it on that
 * GPU, whichever world or stream that was, so calls from different worlds or streams never see each other's
 * tables; they do not overlap on the GPU either.  A call recorded into a HIP graph is ordered by whoever
 * launches the graph: replays that overlap another user of the array on the same GPU race.
 */
HcclResult HcclAmdAlltoAllVNoAlloc(const void* sendBuf, const void* sendCounts, const void* sdispls,
                                   HcclDataType sendType, const void* recvBuf, const void* recvCounts,
                                   const void* rdispls, HcclDataType recvType, HcclComm comm, aclrtStream stream);

/*
 * AlltoAllV with sendCounts = recvCounts = recvCount for every peer and displacements i * recvCount:
 * rank i's recvBuf[j*recvCount + e] = sendBuf_j[i*recvCount + e].  sendCount must equal recvCount and
 * sendType recvType.  Replaces reference include/hccl.h:234-236 (src/ops/all_to_all_v/all_to_all_v.cc:24).
 */
HcclResult HcclAlltoAll(const void* sendBuf, uint64_t sendCount, HcclDataType sendType, const void* recvBuf,
                        uint64_t recvCount, HcclDataType recvType, HcclComm comm, aclrtStream stream);

/*
 * AlltoAllV whose arrays every rank derives from one host uint64_t[rankSize * rankSize] matrix, row = sender,
 * column = receiver: rank r sends row r, receives column r, both packed without gaps.
 * Replaces reference include/hccl.h:192-194 (src/ops/all_to_all_v/all_to_all_v.cc:153, conversion :423-458).
 */
HcclResult HcclAlltoAllVC(const void* sendBuf, const void* sendCountMatrix, HcclDataType sendType, const void* recvBuf,
                          HcclDataType recvType, HcclComm comm, aclrtStream stream);

/*
 * Rank k's recvBuf[e] = reduction over ranks t of sendBuf_t[sendDispls[k] + e], e in [0, sendCounts[k]),
 * folded own rank first, then the others ascending.  sendCounts / sendDispls: host uint64_t[rankSize],
 * elements, identical on every rank; recvCount must be sendCounts[own rank].  No uint64 / fp64.
 * Replaces reference include/hccl.h:90-92 (src/ops/reduce_scatter_v/reduce_scatter_v.cc:23).
 */
HcclResult HcclReduceScatterV(void* sendBuf, const void* sendCounts, const void* sendDispls, void* recvBuf,
                              uint64_t recvCount, HcclDataType dataType, HcclReduceOp op, HcclComm comm,
                              aclrtStream stream);

/*
 * The root's recvBuf[e] = (((sendBuf_0[e] (+) sendBuf_1[e]) (+) ...) (+) sendBuf_{N-1}[e]); recvBuf of the
 * other ranks is left alone.  Replaces reference include/hccl.h:253-255 (src/ops/reduce/reduce.cc:23).
 */
HcclResult HcclReduce(void* sendBuf, void* recvBuf, uint64_t count, HcclDataType dataType, HcclReduceOp op,
                      uint32_t root, HcclComm comm, aclrtStream stream);

/*
 * Every rank's buf = the root's buf.  Replaces reference include/hccl.h:52-53
 * (src/ops/broadcast/broadcast.cc:23).
 */
HcclResult HcclBroadcast(void* buf, uint64_t count, HcclDataType dataType, uint32_t root, HcclComm comm,
                         aclrtStream stream);

/*
 * Rank r's recvBuf[e] = the root's sendBuf[r*recvCount + e]; sendBuf of the other ranks is ignored.
 * Replaces reference include/hccl.h:107-109 (src/ops/scatter/scatter.cc:30).
 */
HcclResult HcclScatter(void* sendBuf, void* recvBuf, uint64_t recvCount, HcclDataType dataType, uint32_t root,
                       HcclComm comm, aclrtStream stream);

/*
 * Orders the ranks' streams: work queued after the call on any rank's stream starts only when the work queued
 * before the call on every rank's stream has finished.  Replaces the HcclBarrier the reference exports from
 * src/ops/barrier/barrier.cc:47-72 (declared by the CANN header hccl/hccl_comm.h, which is outside its tree).
 */
HcclResult HcclBarrier(HcclComm comm, aclrtStream stream);

/*
 * Point to point.  destRank's HcclRecv(…, srcRank = this rank) receives what this rank sends; sends and receives
 * between the same two ranks pair up in call order.  A rank cannot send to itself (HCCL_E_NOT_SUPPORT).  The side
 * that arrives second launches the copy; the first one blocks until then unless it is inside
 * HcclGroupStart / HcclGroupEnd.  Replace reference include/hccl.h:158-159, 175-176 (src/ops/send/send.cc:25-49,
 * 136-163; src/ops/recv/recv.cc:25-49, 134-161).
 */
HcclResult HcclSend(void* sendBuf, uint64_t count, HcclDataType dataType, uint32_t destRank, HcclComm comm,
                    aclrtStream stream);
HcclResult HcclRecv(void* recvBuf, uint64_t count, HcclDataType dataType, uint32_t srcRank, HcclComm comm,
                    aclrtStream stream);

/*
 * A batch of sends and receives issued together.  Items without elements are skipped; several transfers between
 * the same two ranks pair up by descending count, then descending data type, whatever their order in the array;
 * a send to the own rank is legal when the batch also holds the receive.  Replaces reference
 * include/hccl.h:265-266 (src/ops/batch_send_recv/batch_send_recv.cc:22-90,
 * algorithm/executor/ins_v2_batch_send_recv_executor.cc:96-200).
 */
HcclResult HcclBatchSendRecv(HcclSendRecvItem* sendRecvInfo, uint32_t itemNum, HcclComm comm, aclrtStream stream);

/* ------------------------------------------------------------------------------------------
 * Communicator lifecycle. In the reference these live in the separate HCOMM library and
 * are only called (examples/02_collectives/01_allreduce/main.cc:76,101,123;
 * docs/en/user_guide/api_comm_impl.md:169-190; src/ops/all_reduce/all_reduce.cc:121-125).
 * ---------------------------------------------------------------------------------------- */

/* Creates ndev communicators of one loopback world; comms[r] has rank r.  `devices` may be
 * NULL; when given, every entry must name the same GPU (peer buffers share one HBM). */
HcclResult HcclCommInitAll(uint32_t ndev, int32_t* devices, HcclComm* comms);

/* Fills rootInfo with a fresh world identity to hand to HcclCommInitRootInfo. */
HcclResult HcclGetRootInfo(HcclRootInfo* rootInfo);

/* Joins rank `rank` of the nRanks-rank world named by rootInfo (same process). */
HcclResult HcclCommInitRootInfo(uint32_t nRanks, const HcclRootInfo* rootInfo, uint32_t rank, HcclComm* comm);

HcclResult HcclCommDestroy(HcclComm comm);
HcclResult HcclGetRankSize(HcclComm comm, uint32_t* rankSize);
HcclResult HcclGetRankId(HcclComm comm, uint32_t* rank);
/* Writes the world's name, NUL-terminated, into commName, which holds at least HCCL_AMD_COMM_NAME_LENGTH bytes: the
 * same for every rank of a world, different between worlds.  (HCOMM's call of that name; the reference's entry
 * points and custom-operator examples key their per-communicator state by it: src/ops/all_reduce/all_reduce.cc:124,
 * src/ops/op_common/inc/alg_param.h:75 COMM_INDENTIFIER_MAX_LENGTH = 128.) */
#define HCCL_AMD_COMM_NAME_LENGTH 128
HcclResult HcclGetCommName(HcclComm comm, char* commName);
const char* HcclGetErrorString(HcclResult code);

/* Calls between Start and End on the calling thread are queued without blocking. */
HcclResult HcclGroupStart(void);
HcclResult HcclGroupEnd(void);

/* ------------------------------------------------------------------------------------------
 * Algorithm choice.  The reference picks an algorithm with its selector and the HCCL_ALGO
 * environment variable (src/common/alg_parse.cc); here it is an explicit per-world knob
 * because the algorithm fixes the association order of the reduction.
 * ---------------------------------------------------------------------------------------- */
typedef enum {
    HCCL_AMD_OP_ALL_REDUCE = 0,
    HCCL_AMD_OP_REDUCE_SCATTER = 1,   /* also ReduceScatterV */
    HCCL_AMD_OP_REDUCE = 2,           /* MESH (alias RING), MESH_TWO_SHOT, NHR; RHD in worlds with level-0 groups */
    HCCL_AMD_OP_COUNT
} HcclAmdOpKind;

typedef enum {
    /* AllReduce: (((x0+x1)+x2)...+x_{N-1}), the mesh one-shot / two-shot / host-reduce order
     * (reference ins_temp_all_reduce_mesh_1D_one_shot.cc:223-239,
     * ins_temp_all_reduce_aicpu_reduce_nhr.cc:272-285).
     * ReduceScatter: rank k starts from its own slice then adds ranks ascending, skipping k
     * (reference ins_temp_reduce_scatter_mesh_1D.cc:203-237). */
    HCCL_AMD_ALGO_MESH = 0,
    /* Alias kept for the reference's naming: "ring" AllReduce on the host-reduce path folds
     * in rank order like MESH; "ring" ReduceScatter uses the NHR step tree. */
    HCCL_AMD_ALGO_RING = 1,
    /* Recursive halving-doubling with pre-fold of non-power-of-two ranks
     * (reference template_utils.cc:117-307, ins_temp_reduce_scatter_rhd.cc).  Reduce knows it between level-0
     * groups only (reduce_sequence_executor_aicpu_3level.cc:1024-1048) and folds in the MESH order without them. */
    HCCL_AMD_ALGO_RHD = 2,
    /* Non-uniform hierarchical ring step tree (reference ins_temp_reduce_scatter_nhr.cc:458-506).  AllReduce
     * cuts the count into N slices of floor(count / N) elements, the last slice taking the rest, and folds
     * slice k by rank k's tree (reference ins_temp_all_reduce_nhr.cc:214-216, 646-687).  Reduce cuts slices of
     * ceil(count / N) elements, short or empty towards the end (reference reduce_nhr.cc:202-226). */
    HCCL_AMD_ALGO_NHR = 3,
    /* Power-of-two block fold used when results must not depend on arrival order
     * (reference ins_temp_reduce_scatter_order_preserved_group.cc:306-409). */
    HCCL_AMD_ALGO_ORDER_PRESERVED = 4,
    /* Vector-core mesh order: chunk c of a rank's output starts at peer c and wraps upward
     * (reference aiv_reduce_scatter_mesh_1d.h:23-71). ReduceScatter only. */
    HCCL_AMD_ALGO_AIV_MESH = 5,
    /* AllReduce in the order of the mesh two-shot template over symmetric memory: the result is cut into
     * N slices of ceil(count / N) elements and slice k starts from rank k's input, then adds the other
     * ranks ascending (reference ins_temp_all_reduce_mesh_1D_two_shot.cc:341-357).  ReduceScatter: MESH. */
    HCCL_AMD_ALGO_MESH_SYMMETRIC = 6,
    /* The mesh order the reference's selector picks for large messages: every slice (a rank's ReduceScatter(V)
     * output; for AllReduce one of N slices of ceil(count / N) elements) is cut into N - 1 segments, and segment
     * i of slice k starts from rank k's input, then adds ranks k+i+1, k+i+2, ... wrapping past k
     * (reference ins_temp_reduce_scatter_mesh_1D_meshchunk.cc:233-375,
     * ins_temp_reduce_scatter_v_mesh_1D_meshchunk.cc:147-265,
     * ins_temp_all_reduce_mesh_1D_two_shot_mesh_chunk.cc:177-295).  ReduceScatter(V) segments are
     * floor(bytes / (N - 1)) rounded down to 4 KiB with the last one taking the rest, or dealt element-wise when
     * that is zero; AllReduce segments are always dealt element-wise.  Set for ReduceScatter it also governs
     * ReduceScatterV, which otherwise always uses MESH. */
    HCCL_AMD_ALGO_MESH_CHUNK = 7,
    /* Reduce only, the template the reference's selector picks from 8 MiB on: the count is dealt into N slices,
     * the first count mod N of them one element longer; slice k starts from rank k's input and adds the other
     * ranks ascending; the root gathers the slices (reference reduce_mesh_1D_two_shot.cc:138-162, 228-265,
     * reduce_auto_selector.cc:346-351).  Reduce under MESH folds rank 0's input first and the others ascending
     * (reduce_mesh_1D.cc:268-300). */
    HCCL_AMD_ALGO_MESH_TWO_SHOT = 8,
    /* AllReduce only: the reference's two-shot executor over one mesh (Aicpu AllReduce Sole MeshConcur, reference
     * ins_v2_all_reduce_two_shot_sole_executor.cc:228-250, 328-392): a mesh ReduceScatter, then an AllGather.  Every
     * loop is cut into N slices of floor(len / N) elements, the last slice taking the rest, and slice k starts from
     * rank k's input and adds the other ranks ascending (ins_temp_reduce_scatter_mesh_1D.cc:203-237); loops hold half
     * of the staging buffer, floored to 128 bytes and a multiple of N elements. */
    HCCL_AMD_ALGO_MESH_CONCUR = 9,
    HCCL_AMD_ALGO_COUNT
} HcclAmdAlgo;

/* Sets the algorithm every later call of `op` on comm's world uses.  Also settable before
 * world creation through HCCL_AMD_ALGO="allreduce=rhd;reducescatter=nhr;reduce=mesh_two_shot".  Calls with PROD or a 64-bit type
 * fold in the MESH order under NHR, RHD, MESH_CHUNK, MESH_CONCUR, AIV_MESH and (ReduceScatter) RING: the reference does not
 * offer those templates for them and falls back to its host-reduce mesh templates
 * (op_common/selector/cost_table.cc:104-131). */
HcclResult HcclAmdSetAlgo(HcclComm comm, HcclAmdOpKind op, HcclAmdAlgo algo);
HcclResult HcclAmdGetAlgo(HcclComm comm, HcclAmdOpKind op, HcclAmdAlgo* algo);

/*
 * Staging-buffer loops.  The reference's executors move every AllReduce through a bounded buffer: the count is
 * cut into loops and each loop is sliced afresh (ins_v2_all_reduce_sole_executor.cc:241-300,
 * ins_v2_all_reduce_sequence_executor_aicpu.cc:645-760), so under the orders whose fold depends on the slice
 * (NHR, RHD, MESH_CHUNK, MESH_CONCUR) the association order of an element depends on the loop it falls in.  No staging exists here;
 * `bytes` only tells the library which loop boundaries to reproduce: 0 (default) = one loop.  The environment
 * variable HCCL_BUFFSIZE (MB), when set at world creation, gives MB * 2^20 - 2^20 bytes
 * (src/common/op_graph/hccl_op_utils.cc:204-225); a value its parser rejects makes every collective return
 * HCCL_E_PARA.  Orders that fold every position alike (MESH, RING, ORDER_PRESERVED) and ReduceScatter under the
 * orders whose fold depends on the receiving rank only are not affected; MESH_CHUNK ReduceScatter loops over the
 * buffer's N - 1 slots, MESH_CHUNK ReduceScatterV runs one loop and returns HCCL_E_NOT_SUPPORT for a slice the
 * buffer cannot hold (ins_v2_reduce_scatter_v_sole_executor.cc:158-171); MESH_SYMMETRIC always runs as one loop
 * (ins_v2_all_reduce_sole_executor.cc:273-282).  A buffer too small for one loop returns HCCL_E_INTERNAL from the
 * collective, like the reference.
 */
HcclResult HcclAmdSetCclBufferSize(HcclComm comm, uint64_t bytes);
HcclResult HcclAmdGetCclBufferSize(HcclComm comm, uint64_t* bytes);

/*
 * Hang triage.  With HCCL_AMD_STUCK_COUNTERS=1 in the environment when the communicators are created, every
 * collective of the world is numbered (1, 2, ...) and its launch stream writes that number to a head word in front
 * of the collective's kernels and to a tail word behind them (pinned host memory, readable while the GPU is
 * busy or hung).  head == tail: nothing is running; head == tail + 1: a kernel of collective `head` has started
 * and not finished.  Follows the reference's head / tail counters
 * (src/ops/op_common/algorithm/template/aiv/aiv_communication_base_v2.h:365-378,
 * src/ops/op_common/stuck_detect_counter_helper.h).  HCCL_E_UNAVAIL when the counters are not enabled.
 */
HcclResult HcclAmdGetStuckCounters(HcclComm comm, uint64_t* head, uint64_t* tail);

/*
 * Host-only view of the reduction plan: writes the fold program the kernel would run for
 * segment `segment` of (op, algo, rankSize) into `out` (at most `cap` bytes) and its length
 * into *len.  Program bytes: 0x00-0x3F = fold rank r into the accumulator of the current
 * nesting level (the first operand of a level initialises it); 0x80 = open a nested level;
 * 0x81 = close it and fold its value (as the incoming operand) into the parent level;
 * 0xC0|n (n in 1..8) = the next n bytes are ranks folded in that order.  No GPU needed.
 */
HcclResult HcclAmdGetFoldProgram(HcclAmdOpKind op, HcclAmdAlgo algo, uint32_t rankSize, uint32_t segment,
                                 uint8_t* out, uint32_t cap, uint32_t* len, uint32_t* segmentCount);
/* The same for the two-level orders over groups of `level0` consecutive ranks (see HcclAmdSetLevel0RankSize).
 * AllReduce and Reduce: segment i * (rankSize / level0) + j is sub-slice j of chunk i; ReduceScatter: segment r is
 * rank r's output.  algo is the template between the groups (RHD, NHR, or MESH for the own-first fold of the
 * host-reduce template).  level0 of 1 or rankSize: HcclAmdGetFoldProgram. */
HcclResult HcclAmdGetFoldProgramTwoLevel(HcclAmdOpKind op, HcclAmdAlgo algo, uint32_t rankSize, uint32_t level0,
                                         uint32_t segment, uint8_t* out, uint32_t cap, uint32_t* len,
                                         uint32_t* segmentCount);
/* And for three levels: `level1` consecutive groups form a level-1 group (see HcclAmdSetLevel1GroupSize), l2 =
 * rankSize / level0 / level1 of them.  AllReduce and Reduce: segment (i * level1 + j) * l2 + k is part k of
 * sub-slice j of chunk i; ReduceScatter: segment r is rank r's output.  level1 of 0: the two-level orders. */
HcclResult HcclAmdGetFoldProgramLevels(HcclAmdOpKind op, HcclAmdAlgo algo, uint32_t rankSize, uint32_t level0,
                                       uint32_t level1, uint32_t segment, uint8_t* out, uint32_t cap, uint32_t* len,
                                       uint32_t* segmentCount);

/*
 * Level-0 groups.  The reference runs AllReduce over a two-level topology (servers of several ranks) as a
 * sequence: a mesh ReduceScatter inside every server, the configured template (RHD, NHR, or the host-reduce fold for
 * PROD and the 64-bit types) between the ranks that hold the same chunk, and the two AllGathers back
 * (src/ops/all_reduce/algorithm/executor/ins_v2_all_reduce_sequence_executor_aicpu.cc:592-852, registered as
 * Aicpu AllReduce Sequence MeshConcur RHD / MeshConcur NHR / Mesh NHRAicpuReduce, :974-1023), and ReduceScatter
 * as the first two of those steps (src/ops/reduce_scatter/algorithm/executor/
 * ins_v2_reduce_scatter_sequence_executor_aicpu.cc:298-500, registrations :567-640).  Where its topology
 * comes from a rank table, a loopback world is told: `ranksPerGroup` consecutive ranks form a group (it must
 * divide the rank size; 1, the default, and the rank size itself mean one level).  Also HCCL_AMD_LEVEL0_RANKS at
 * world creation.  With groups, AllReduce, ReduceScatter and Reduce under RHD and NHR fold in the two-level order
 * (Reduce: src/ops/reduce/algorithm/executor/reduce_sequence_executor_aicpu_3level.cc:744-990, registrations
 * :995-1048); the other orders and the other operators (ReduceScatterV included) are not affected.
 */
HcclResult HcclAmdSetLevel0RankSize(HcclComm comm, uint32_t ranksPerGroup);
HcclResult HcclAmdGetLevel0RankSize(HcclComm comm, uint32_t* ranksPerGroup);
/*
 * Level-1 groups.  Over a three-level topology (servers in pods) the reference adds a step: the template runs
 * between the servers of a pod and once more between the pods (ins_v2_all_reduce_sequence_executor_aicpu_3level.cc:
 * 536-800, ins_v2_reduce_scatter_sequence_executor_3level.cc:243-256, reduce_sequence_executor_aicpu_3level.cc;
 * registered as Sequence MeshConcur NHR NHR and ... RHD RHD).  `groupsPerLevel1Group` consecutive level-0 groups
 * form a level-1 group; it must divide the number of level-0 groups; 0, the default, and that number itself mean
 * two levels.  Also HCCL_AMD_LEVEL1_GROUPS at world creation.  The host-reduce fold of PROD and the 64-bit types
 * knows two levels in the reference and keeps them here: every level-0 group of the world is its peer.
 */
HcclResult HcclAmdSetLevel1GroupSize(HcclComm comm, uint32_t groupsPerLevel1Group);
HcclResult HcclAmdGetLevel1GroupSize(HcclComm comm, uint32_t* groupsPerLevel1Group);

/*
 * The reference's HCCL_ALGO setting ("allreduce:sequence{level0=mesh_concur,level1=rhd};reducescatter:nhr;..."; grammar
 * and vocabulary of src/common/alg_parse.cc:27-437) is read at world creation and selects the fold order of
 * AllReduce, ReduceScatter(V) and Reduce: sole{mesh | mesh_one_shot | mesh_two_shot} -> MESH (Reduce: mesh_two_shot ->
 * MESH_TWO_SHOT), sole{mesh_concur} for AllReduce -> MESH_CONCUR, sole{mesh_chunk...} -> MESH_CHUNK, sole{nhr...} -> NHR, sole{nhr_aicpu_reduce} -> the host-reduce
 * order (RING for AllReduce, MESH for ReduceScatter and Reduce), sole{rhd | hd | hd_aicpu_reduce} -> RHD, strictordered{...} ->
 * ORDER_PRESERVED, sequence{<mesh...>, <template>[, <the same template>]} -> that template between level-0 groups
 * and, where the world has them, between level-1 groups (AllReduce, ReduceScatter, Reduce; a mesh-chunk template
 * inside the groups and different templates at the upper levels are other orders and select nothing).  Clauses are
 * taken last to first, negations select nothing, clauses for the copy operators are accepted and ignored, and a
 * string the reference's parser rejects is ignored with a warning, as there.  HCCL_AMD_ALGO and HcclAmdSetAlgo
 * override it.  This call is the host-only view of that reading: HCCL_E_PARA for a rejected string; otherwise
 * *selected says whether `config` selects an order for `op`, *algo and *twoLevel which, and `canonical` (optional,
 * `cap` bytes) receives the parsed clauses in normal form ("allreduce:sequence{meshconcur,rhd};not(sole{nhr})").
 */
HcclResult HcclAmdSelectFromHcclAlgo(const char* config, HcclAmdOpKind op, int32_t* selected, HcclAmdAlgo* algo,
                                     int32_t* twoLevel, char* canonical, uint32_t cap);

#ifdef __cplusplus
}
#endif
#endif /* HCCL_AMD_HCCL_H_ */
