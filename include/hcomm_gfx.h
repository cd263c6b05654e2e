/*
 * hcomm_gfx.h - C ABI of libhcomm_gfx.so: HCOMM's local copy / local reduce data plane and the
 * collective schedules built from it, executed by hand-written HIP kernels on one MI355X (gfx950).
 *
 * Plain C (C99).  Every type and enumerator that also exists in the reference keeps the reference's
 * name and numeric value, so a caller compiled against the reference headers can bind these symbols
 * unchanged.  Citations are paths relative to the reference tree.
 *
 * Four groups of entry points:
 *   1. drop-in primitives      - same names, argument meaning and return codes as the reference;
 *   2. HcommGfx* extensions    - k-way fused reduce, stream sync, launch log (no reference counterpart);
 *   3. HcommGfxPlan*           - build once / run many replay of the templates' schedules (ring, recursive
 *                                halving-doubling, mesh, NHR, NB, doubling, deterministic local reduce, chunk mesh)
 *                                over N simulated ranks (N pairs of HBM buffers), with HcommGfxSchedule* to obtain
 *                                the operation lists and check them symbolically without a GPU;
 *   4. executor-level plans    - HcommGfxOpBase*, HcommGfxHier*, HcommGfxMeshHier*, HcommGfxHierReduceScatter*,
 *                                HcommGfxDoubleRing*, HcommGfxDoubleRingHierReduceScatter*, HcommGfxOrderPreserved*, HcommGfxOrderPreservedSmall*,
 *                                HcommGfxOrderPreservedAllReduce*,
 *                                HcommGfxOrderPreservedHierAllReduce*, HcommGfxOrderPreservedHierReduceScatter*,
 *                                HcommGfxOrderPreservedFused*: what the
 *                                reference's executors do around the templates (chunk loops through the CCL
 *                                buffers, two communicator levels, user memory read and written directly), each
 *                                as PlanCreate / Emit / Check.
 */
#ifndef HCOMM_GFX_H
#define HCOMM_GFX_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---------------------------------------------------------------------------------------------
 * Types shared with the reference
 * ------------------------------------------------------------------------------------------- */

/* include/hcomm_res_defs.h:26 */
typedef int32_t HcommResult;

/* include/hcomm_primitives.h:30,38 */
#ifndef CHANNEL_HANDLE_DEFINED
#define CHANNEL_HANDLE_DEFINED
typedef uint64_t ChannelHandle;
#endif
#ifndef THREAD_HANDLE_DEFINED
#define THREAD_HANDLE_DEFINED
typedef uint64_t ThreadHandle;
#endif

/* include/hccl/hccl_types.h:23-51 (HcclResult); only the codes this library can return */
enum {
    HCCL_SUCCESS = 0,
    HCCL_E_PARA = 1,
    HCCL_E_PTR = 2,
    HCCL_E_MEMORY = 3,
    HCCL_E_INTERNAL = 4,
    HCCL_E_NOT_SUPPORT = 5,
    HCCL_E_NOT_FOUND = 6,
    HCCL_E_UNAVAIL = 7,
    HCCL_E_TIMEOUT = 9,
    HCCL_E_RUNTIME = 15
};

/* include/hcomm_primitives.h:45-51 (identical to HcclReduceOp, include/hccl/hccl_types.h:71-77) */
typedef enum {
    HCOMM_REDUCE_SUM = 0,
    HCOMM_REDUCE_PROD = 1,
    HCOMM_REDUCE_MAX = 2,
    HCOMM_REDUCE_MIN = 3,
    HCOMM_REDUCE_RESERVED = 255
} HcommReduceOp;

/* include/hcomm_primitives.h:53-72 (identical to HcclDataType, include/hccl/hccl_types.h:82-101) */
typedef enum {
    HCOMM_DATA_TYPE_INT8 = 0,
    HCOMM_DATA_TYPE_INT16 = 1,
    HCOMM_DATA_TYPE_INT32 = 2,
    HCOMM_DATA_TYPE_FP16 = 3,
    HCOMM_DATA_TYPE_FP32 = 4,
    HCOMM_DATA_TYPE_INT64 = 5,
    HCOMM_DATA_TYPE_UINT64 = 6,
    HCOMM_DATA_TYPE_UINT8 = 7,
    HCOMM_DATA_TYPE_UINT16 = 8,
    HCOMM_DATA_TYPE_UINT32 = 9,
    HCOMM_DATA_TYPE_FP64 = 10,
    HCOMM_DATA_TYPE_BFP16 = 11,
    HCOMM_DATA_TYPE_INT128 = 12,
    HCOMM_DATA_TYPE_HIF8 = 14,
    HCOMM_DATA_TYPE_FP8E4M3 = 15,
    HCOMM_DATA_TYPE_FP8E5M2 = 16,
    HCOMM_DATA_TYPE_FP8E8M0 = 17,
    HCOMM_DATA_TYPE_RESERVED = 255
} HcommDataType;

/* include/hcomm_res_defs.h:106-114 */
typedef enum {
    COMM_ENGINE_RESERVED = -1,
    COMM_ENGINE_CPU = 0,
    COMM_ENGINE_CPU_TS = 1,
    COMM_ENGINE_AICPU = 2,
    COMM_ENGINE_AICPU_TS = 3,
    COMM_ENGINE_AIV = 4,
    COMM_ENGINE_CCU = 5
} CommEngine;

/* ---------------------------------------------------------------------------------------------
 * 1. Drop-in primitives
 * ------------------------------------------------------------------------------------------- */

/*
 * dst[0..len) = src[0..len) on the thread's stream.  Replaces include/hcomm_primitives.h:152
 * (host adapter src/base_comm/primitives/api_c_adpt/cpu_primitives_c_adpt.cc:58-86).
 * Check order: dst NULL -> HCCL_E_PTR, src NULL -> HCCL_E_PTR, thread 0 -> HCCL_E_PTR.
 * len == 0 or src == dst succeed without doing anything
 * (src/legacy/ascend910/platform/task/dispatcher.cc:495-498).  len may exceed 4 GiB.
 * Asynchronous: returns once the work is enqueued (or, in batch mode, recorded).
 */
int32_t HcommLocalCopyOnThread(ThreadHandle thread, void* dst, const void* src, uint64_t len);

/*
 * dst[i] = dst[i] (op) src[i] for i < count, result stored in the element type.  Replaces
 * include/hcomm_primitives.h:164-165 (host adapter cpu_primitives_c_adpt.cc:88-130).
 * Check order: dst NULL -> HCCL_E_PTR, src NULL -> HCCL_E_PTR, unsupported dataType/reduceOp ->
 * HCCL_E_PARA, thread 0 -> HCCL_E_PTR.  Supported exactly as the reference
 * (cpu_primitives_c_adpt.cc:31-39): {INT8, INT16, INT32, FP16, FP32, BFP16} x {SUM, MAX, MIN};
 * PROD is rejected here (it exists only at collective level in the reference) unless the
 * environment variable HCOMM_GFX_ALLOW_PROD=1 is set when the library is loaded.
 * count == 0 succeeds without doing anything (dispatcher.cc:719-722).  count may exceed 2^32.
 */
int32_t HcommLocalReduceOnThread(
    ThreadHandle thread, void* dst, const void* src, uint64_t count, HcommDataType dataType, HcommReduceOp reduceOp);

/*
 * Thread = one in-order execution queue (a HIP stream) plus notifyNum local notifies.
 * Replaces include/hcomm_res.h:57-60 (src/base_comm/primitives/api_c_adpt/hcomm_thread_c_adpt.cc:38-86,157).
 * threads NULL or notifyNumPerThread NULL -> HCCL_E_PTR; threadNum == 0 -> HCCL_E_PARA.
 * Only notifyNumPerThread[0] is used, as in the reference.  Every engine value maps to the GPU.
 */
HcommResult
HcommThreadAlloc(CommEngine engine, uint32_t threadNum, const uint32_t* notifyNumPerThread, ThreadHandle* threads);
HcommResult HcommThreadFree(const ThreadHandle* threads, uint32_t threadNum);

/*
 * Bind a thread to a caller-owned stream (a hipStream_t passed as void*; NULL = the default stream).
 * Replaces hcomm_thread_c_adpt.cc:164-187 (declared at src/base_comm/primitives/api_c_adpt/hcomm_c_adpt.h:108,113).
 * The stream is never destroyed by the library.
 */
HcommResult HcommThreadAllocWithStream(CommEngine engine, void* stream, uint32_t notifyNum, ThreadHandle* thread);
HcommResult HcommThreadFreeWithStream(const ThreadHandle* threads, uint32_t threadNum);

/*
 * Cross-thread ordering.  Replaces include/hcomm_primitives.h:181,191.  Record marks, on dstThread's
 * notify slot dstNotifyIdx, the point `thread` has reached; Wait makes `thread` wait for the most recent
 * record on its own slot notifyIdx.  A notify is a HIP event, so the Record has to be ISSUED before the stream can
 * be told to wait for it: a Wait that finds no unconsumed Record on its slot sits on the host until another host
 * thread issues one, for at most min(timeOut seconds, HCOMM_GFX_NOTIFY_HOST_WAIT_MS = 100 ms by default), then
 * queues nothing and returns HCCL_E_TIMEOUT - the reference's wait would sit on the device until timeOut ran out.
 * Callers that issue both from one host thread issue the Record first.  Every Record is consumed by one Wait.
 * Between HcommBatchModeStart and HcommBatchModeEnd a Record or Wait is queued on its thread like the copies and
 * reduces around it (slot numbers are still checked at once), and HcommBatchModeEnd resolves them: see there.
 */
int32_t HcommThreadNotifyRecordOnThread(ThreadHandle thread, ThreadHandle dstThread, uint32_t dstNotifyIdx);
int32_t HcommThreadNotifyWaitOnThread(ThreadHandle thread, uint32_t notifyIdx, uint32_t timeOut);

/*
 * The default notify-wait time-out of the calling host thread and the wait that uses it.  Replace
 * include/hcomm_primitives.h:559,585 (host adapter cpu_primitives_c_adpt.cc:41-50,1015-1034): a NaN, negative or
 * larger-than-UINT32_MAX value is HCCL_E_PARA.  HcommThreadResAcquireTimeOut (:567) is not supported on this
 * path either (cpu_primitives_c_adpt.cc:52-56).
 */
int32_t HcommSetNotifyWaitTimeOut(float timeOut);
int32_t HcommThreadNotifyWaitOnThreadWithDefaultTimeout(ThreadHandle thread, uint32_t notifyIdx);
int32_t HcommThreadResAcquireTimeOut(float timeOut);

/*
 * Ordering points.  Replace include/hcomm_primitives.h:534,542,593 (host adapter cpu_primitives_c_adpt.cc:780-808,
 * 818-823).  A thread is an in-order HIP stream and a simulated peer shares its memory, so everything issued
 * before such a call is already ordered before everything issued after it: the calls validate their handles and
 * return.  Inside batch mode the recorded operations keep their order and their dependences anyway.
 */
int32_t HcommFenceOnThread(ThreadHandle thread);
int32_t HcommChannelFenceOnThread(ThreadHandle thread, ChannelHandle channel);
int32_t HcommChannelDrainOnThread(ThreadHandle thread, ChannelHandle channel);

/*
 * Inter-rank twins of the two local primitives.  Replace include/hcomm_primitives.h:231-246,291-306 (host
 * adapter cpu_primitives_c_adpt.cc:284-318,332-384,490-565).  Same arithmetic with one operand on a peer:
 *   Write        peer dst[0..len) = local src          WriteReduce  peer dst[i] = dst[i] (op) local src[i]
 *   Read         local dst[0..len) = peer src          ReadReduce   local dst[i] = dst[i] (op) peer src[i]
 * With every simulated rank in the HBM of one GPU, a peer buffer is directly addressable and the channel is an
 * opaque non-zero token.  Check order as the reference: dst NULL, src NULL -> HCCL_E_PTR; unsupported
 * type / op -> HCCL_E_PARA; thread 0 -> HCCL_E_PTR; then channel 0 -> HCCL_E_PTR.  Batch mode applies.
 */
int32_t HcommWriteOnThread(ThreadHandle thread, ChannelHandle channel, void* dst, const void* src, uint64_t len);
int32_t HcommReadOnThread(ThreadHandle thread, ChannelHandle channel, void* dst, const void* src, uint64_t len);
int32_t HcommWriteReduceOnThread(
    ThreadHandle thread, ChannelHandle channel, void* dst, const void* src, uint64_t count, HcommDataType dataType,
    HcommReduceOp reduceOp);
int32_t HcommReadReduceOnThread(
    ThreadHandle thread, ChannelHandle channel, void* dst, const void* src, uint64_t count, HcommDataType dataType,
    HcommReduceOp reduceOp);

/* The non-blocking spellings of the copy twins (include/hcomm_primitives.h:317-318,370-371): every operation on a
 * thread is asynchronous here, so they are the same calls. */
int32_t HcommWriteNbiOnThread(ThreadHandle thread, ChannelHandle channel, void* dst, const void* src, uint64_t len);
int32_t HcommReadNbiOnThread(ThreadHandle thread, ChannelHandle channel, void* dst, const void* src, uint64_t len);

/* include/hcomm_primitives.h:77-86 */
typedef enum {
    HCOMM_TRANSFER_TYPE_INVALID = -1,
    HCOMM_TRANSFER_TYPE_WRITE = 0,
    HCOMM_TRANSFER_TYPE_WRITE_REDUCE = 1,
    HCOMM_TRANSFER_TYPE_WRITE_WITH_NOTIFY = 2,
    HCOMM_TRANSFER_TYPE_WRITE_REDUCE_WITH_NOTIFY = 3,
    HCOMM_TRANSFER_TYPE_READ = 4,
    HCOMM_TRANSFER_TYPE_READ_REDUCE = 5,
    HCOMM_TRANSFER_TYPE_NOTIFY_RECORD = 6
} HcommTransferType;

/* include/hcomm_primitives.h:91-131: 64 bytes = type, 4 reserved, 56-byte union; identical layout */
typedef struct {
    HcommTransferType transType;
    uint8_t reserved[4];
    union {
        uint8_t raws[56];
        struct {
            uint64_t len;
            void* dst;
            void* src;
        } write;
        struct {
            uint64_t len;
            void* dst;
            void* src;
        } read;
        struct {
            uint64_t count;
            void* dst;
            void* src;
            HcommReduceOp reduceOp;
            HcommDataType dataType;
        } reduce;
        struct {
            uint32_t notifyIdx;
        } notifyRecord;
        struct {
            uint64_t len;
            void* dst;
            void* src;
            uint32_t notifyIdx;
        } writeWithNotify;
        struct {
            uint64_t count;
            void* dst;
            void* src;
            HcommReduceOp reduceOp;
            HcommDataType dataType;
            uint32_t notifyIdx;
        } writeReduceWithNotify;
    } transferInfo;
} HcommBatchTransferDesc;

/*
 * Submit an array of descriptors as one batch.  Replaces include/hcomm_primitives.h:393-394.  The reference's
 * host adapter forwards this call to NIC plugins only and otherwise returns HCCL_E_NOT_SUPPORT
 * (cpu_primitives_c_adpt.cc:320-330); here WRITE / READ / WRITE_REDUCE / READ_REDUCE descriptors are executed,
 * in array order, with the same merging of independent operations into single launches as batch mode.
 * The three notify-carrying types -> HCCL_E_NOT_SUPPORT (nothing is submitted).  transferDescs NULL with a
 * non-zero count -> HCCL_E_PTR.  Every descriptor is validated before anything is enqueued.
 */
int32_t HcommBatchTransferOnThread(
    ThreadHandle thread, ChannelHandle channel, const HcommBatchTransferDesc* transferDescs, uint32_t transferDescNum);

/* Device memory.  Replaces include/hcomm_res.h:69-71.  ptr NULL -> HCCL_E_PTR, size 0 -> HCCL_E_PARA. */
HcommResult HcommMemAlloc(void** ptr, size_t size);
HcommResult HcommMemFree(void* ptr);

/*
 * Batch mode.  Replaces include/hcomm_primitives.h:498,506 (src/base_comm/primitives/launch_context.cc:139-174).
 * Between Start and End, on the calling host thread, primitives only record.  End submits everything
 * recorded, per ThreadHandle in call order, after merging runs of mutually independent operations of the
 * same kind / type / op into single kernel launches (one launch for all N ranks of a collective step).
 * Two operations are independent when neither writes memory the other reads or writes.
 * Start while already batching, or End without Start -> HCCL_E_PARA.  batchTag may be NULL.
 *
 * A BATCH WITH NOTIFIES.  The reference hands a batch to the device as one task graph over ALL the threads it touched,
 * their notify tasks included (CommTaskLaunch(threads, threadNum), launch_context.cc:16-44).  Here, when any Record or
 * Wait was queued, HcommBatchModeEnd works out on the host an order of all queued copies and reduces that respects
 * each thread's own order and every Record -> Wait pair (a Wait may have been called before its Record; a Record
 * issued BEFORE the batch satisfies a Wait inside it), and issues that one list through the coalescer on the stream
 * of the FIRST thread the batch touched: operations that different threads perform in the same step of a schedule
 * share a launch, exactly as if one thread had been given the step between a Start / End pair of its own, and steps
 * that write more than the memory-side cache serves run piece by piece as in a step-wise plan (HcommGfxSetPieceBytes).  The other
 * threads' streams are placed behind the end of the batch when they are next given a call or synchronised (a stream
 * of the caller's, HcommThreadAllocWithStream: at once), and the batch behind whatever they were given before it.
 * A Wait that neither the batch nor an earlier Record satisfies can never be satisfied - the host thread that would
 * issue the Record is the one inside HcommBatchModeEnd - so End returns HCCL_E_TIMEOUT at once and submits NOTHING of
 * the batch; Records the batch took from before it are handed back.  Records that no Wait of the batch consumes
 * remain for a later Wait, as of the end of the batch.
 */
int32_t HcommBatchModeStart(const char* batchTag);
int32_t HcommBatchModeEnd(const char* batchTag);

/* ---------------------------------------------------------------------------------------------
 * 2. Extensions (no reference counterpart)
 * ------------------------------------------------------------------------------------------- */

#define HCOMM_GFX_MAX_RANKS 32u /* most simulated ranks per plan / most inputs of a fused k-way reduce */

/* Block the host until everything enqueued on the thread has finished. */
int32_t HcommGfxThreadSynchronize(ThreadHandle thread);

/*
 * Fused k-way reduce: dst[i] = (..((srcs[0][i] (op) srcs[1][i]) (op) srcs[2][i]) .. (op) srcs[k-1][i]),
 * left to right with the running value in the "dst" role of the op, rounded to the element type after
 * every step - i.e. the result of one copy followed by k-1 HcommLocalReduceOnThread calls
 * (the chain of src/legacy/ascend910/algorithm/base/alg_template/temp_all_reduce/all_reduce_mesh_oneshot.cc:94-119)
 * in a single pass that reads each input once.  1 <= k <= HCOMM_GFX_MAX_RANKS.  dst may alias srcs[0].
 * PROD is allowed for the types the reference allows at collective level
 * (HcomCheckReduceDataType for 910B / 910_93, src/legacy/ascend910/framework/common/src/param_check.cc:327-343):
 * INT8, INT32, FP16, FP32 - not INT16, not BFP16.
 */
int32_t HcommGfxReduceKOnThread(
    ThreadHandle thread, void* dst, const void* const* srcs, uint32_t k, uint64_t count, HcommDataType dataType,
    HcommReduceOp reduceOp);

/*
 * A recorder thread never touches the GPU: every launch it would make is appended to a log instead.
 * It exists so that argument checking, batching and schedule lowering can be tested on a host without a
 * GPU (the reference's unit tests mock the engine the same way,
 * test/ut/framework/communicator/impl/independent_op/data_api/ut_aicpu_ts_HcommLocalReduceOnThread.cc:26-30).
 */
HcommResult HcommGfxRecorderThreadAlloc(ThreadHandle* thread);

typedef struct {
    uint32_t kind;   /* HcommGfxKernelKind */
    uint32_t dtype;  /* HcommDataType, 255 for copies */
    uint32_t op;     /* HcommReduceOp, 255 for copies */
    uint32_t nseg;   /* segments merged into this launch */
    uint64_t bytes;  /* sum of segment output bytes */
    uint64_t blocks; /* grid size */
    uint32_t rows;   /* copy / two-input reduce: > 0 = two-dimensional grid of `rows` tiles by nseg segments, every
                        address read in one round (the k_*_rows kernels); 0 = one-dimensional grid over the table's
                        tiles.  Folds: 1 = small launch whose addresses the host resolves (the k_fold_*_direct kernels) */
    uint32_t streaming; /* copy / two-input reduce: 1 = the variant for output that nothing reads back soon */
    uint32_t backwards; /* copy / two-input reduce: 1 = the launch walked its table from the end (HcommGfxSetAlternateBytes);
                           decided when a launch is submitted, so always 0 in what HcommGfxPlanGetLaunch reports */
    uint32_t reserved;
} HcommGfxLaunchRecord;

typedef enum {
    HCOMM_GFX_KERNEL_COPY = 0,     /* batched vector copy */
    HCOMM_GFX_KERNEL_REDUCE2 = 1,  /* batched dst = dst (op) src */
    HCOMM_GFX_KERNEL_CHAIN = 2,    /* k inputs folded in sequence, optional partial stores, fan-out stores */
    HCOMM_GFX_KERNEL_TREE = 3,     /* k = 2^j inputs folded as a binary tree with partial stores, fan-out */
    HCOMM_GFX_KERNEL_BYTEWISE = 4  /* copy / two-input reduce for pointers off 16-byte boundaries (unaligned 16-byte items) */
} HcommGfxKernelKind;

/* Copy up to `cap` records of the thread's launch log into `out`; *n receives the total logged. */
int32_t HcommGfxLaunchLogRead(ThreadHandle thread, HcommGfxLaunchRecord* out, uint32_t cap, uint32_t* n);
int32_t HcommGfxLaunchLogClear(ThreadHandle thread);

/* ---------------------------------------------------------------------------------------------
 * 3. Collective schedules over N simulated ranks
 * ------------------------------------------------------------------------------------------- */

typedef enum {
    /* AllReduceRing: temp_all_reduce/all_reduce_ring.cc:26-62 = ring reduce-scatter + ring all-gather */
    HCOMM_GFX_ALG_ALLREDUCE_RING = 0,
    /* reduce-scatter stage of AllReduceRing (RunAsyncStaged(RUN_REDUCE_SCATTER), all_reduce_ring.cc:82-92):
       in place in the input buffers, S1 slice table; rank r ends up owning slice r in in[r] */
    HCOMM_GFX_ALG_REDUCE_SCATTER_RING = 1,
    /* AllReduceRecursiveHalvingDoubling: temp_all_reduce/all_reduce_recursive_hd.cc:28-50 */
    HCOMM_GFX_ALG_ALLREDUCE_RHD = 2,
    /* AllReduceMeshDirectOneshot: temp_all_reduce/all_reduce_mesh_oneshot.cc:78-121 */
    HCOMM_GFX_ALG_ALLREDUCE_MESH_ONESHOT = 3,
    /* ReduceScatterMesh: temp_reduce_scatter/reduce_scatter_mesh.cc:51-215; count = per-rank OUTPUT count */
    HCOMM_GFX_ALG_REDUCE_SCATTER_MESH = 4,
    /* stand-alone ReduceScatterRing: temp_reduce_scatter/reduce_scatter_ring.cc:96-180; count = per-rank
       OUTPUT count, input holds N*count, result written to out[r][0..count) */
    HCOMM_GFX_ALG_REDUCE_SCATTER_RING_STANDALONE = 5,
    /* InsTempAllReduceMesh1DOneShot: src/legacy/ascend950/service/collective/alg/coll_alg_factory/alg_template/
       ins_alg_template/ins_temp_all_reduce_mesh_1D_one_shot.cc:86-164 - out = in[r], then the other ranks'
       inputs in ascending rank order (the legacy one-shot folds them in the order r+1, r+2, ...) */
    HCOMM_GFX_ALG_ALLREDUCE_MESH_ONESHOT_ASCENDING = 6,
    /* AllReduceLocalReduce (the deterministic mesh allreduce): src/legacy/ascend910/algorithm/base/alg_template/
       temp_all_reduce/all_reduce_local_reduce.cc:139-436.  Every rank gathers the other ranks' copies of its
       slice into N-1 slots of its communication buffer, folds the slots in a fixed tree order, and the ranks
       then gather the results.  Needs a third buffer per rank (HcommGfxPlanCreateEx, HcommGfxScratchBytes) and a
       power-of-two rank count: the template's slot arithmetic puts the result where the gather reads it only
       when N = 2 * 2^floor(log2(N-1)).  Step-wise lowering only. */
    HCOMM_GFX_ALG_ALLREDUCE_LOCAL_REDUCE = 7,
    /* AllReduceChunkMesh (two-shot mesh, what the legacy one-shot executor instantiates for more than two
       ranks): temp_all_reduce/all_reduce_chunk_mesh.cc:104-345.  Each rank copies its input into its
       communication buffer, reduces its own slice there in N-1 rounds - sub-chunk p-1 of the slice takes peer
       r+p, r+p+1, ..., r+N-1, r+1, ..., r+p-1 in that order (a Latin square over links and rounds) - and the
       ranks gather the slices.  Needs the third buffer (count * unit bytes).  Step-wise lowering only. */
    HCOMM_GFX_ALG_ALLREDUCE_CHUNK_MESH = 8,
    /* AllReduceNHR (nonuniform hierarchical ring, ceil(log2 N) steps for any N): temp_all_reduce/
       all_reduce_nhr.cc:25-77 = ReduceScatterNHR in place on the inputs (temp_reduce_scatter/
       reduce_scatter_nhr.cc:408-488, step table :552-593: step s, rank r folds from rank r + 2^s) over the
       tree-ordered slice map (nonuniform_hierarchical_ring_base.cc:20-75) with touching slices merged (:94-136),
       own slice input -> output, AllGatherNHR on the outputs (temp_all_gather/all_gather_nhr.cc:141-195,228-268) */
    HCOMM_GFX_ALG_ALLREDUCE_NHR = 9,
    /* stand-alone ReduceScatterNHR (reduce_scatter_nhr.cc:27-95): input holds N slices of count elements (slice i
       at i * strideCount), slice order kept, result in out[r][0..count) */
    HCOMM_GFX_ALG_REDUCE_SCATTER_NHR = 10,
    /* AllReduceNB (nonuniform Bruck): temp_all_reduce/all_reduce_nb.cc:26-61 = ReduceScatterNB in place
       (temp_reduce_scatter/reduce_scatter_nb.cc:119-230: step s, rank r folds from rank r - 2^s), own slice
       input -> output, AllGatherNB (temp_all_gather/all_gather_nb.cc:101-188).  Slices are not cut below
       128 KiB (all_reduce_nb.cc:203-219) */
    HCOMM_GFX_ALG_ALLREDUCE_NB = 11,
    /* stand-alone ReduceScatterNB (reduce_scatter_nb.cc:27-86), layout as HCOMM_GFX_ALG_REDUCE_SCATTER_NHR */
    HCOMM_GFX_ALG_REDUCE_SCATTER_NB = 12,
    /* ReduceScatterLocalReduce (the deterministic mesh reduce-scatter, any N): temp_reduce_scatter/
       reduce_scatter_local_reduce.cc:125-160.  Every rank writes its copy of slice d into a slot of rank d's
       communication buffer (:218-243), rank d folds the slots and its own copy pairwise in a fixed order into
       out[d][0..count) (:252-304).  Input holds N dense slices of count elements; needs the third buffer
       (HcommGfxScratchBytes).  Step-wise lowering only. */
    HCOMM_GFX_ALG_REDUCE_SCATTER_LOCAL_REDUCE = 13,
    /* AllReduceDoubling (recursive doubling on the whole message, the intra-server small-message allreduce):
       temp_all_reduce/all_reduce_doubling.cc:91-128.  Power-of-two rank counts; step s copies the running value
       to the buffer the partner reads (input -> output first, output -> input afterwards) and folds the input of
       rank XOR 2^s into the own output.  The inputs are overwritten.  Step-wise lowering only. */
    HCOMM_GFX_ALG_ALLREDUCE_DOUBLING = 14,
    /* AllReduceNHROneshot (the inter-server allreduce of messages up to 256 KiB per device, which are not cut into
       slices): temp_all_reduce/all_reduce_nhr_oneshot.cc:26-69 = ReduceNHROneshot to rank 0
       (temp_reduce/reduce_nhr_oneshot.cc:169-236, a binomial tree folding input into input) followed by
       BroadcastNHROneshot (temp_broadcast/broadcast_nhr_oneshot.cc:24-59,155-205: rank 0 copies input -> output,
       then the tree runs backwards on the outputs).  Any rank count. */
    HCOMM_GFX_ALG_ALLREDUCE_NHR_ONESHOT = 15,
    /* ReduceScatterRecursiveHalvingDoubling (temp_reduce_scatter/reduce_scatter_recursive_hd.cc:29-84), which works in
       place on slices of total / N bytes: accepted only as the level-1 algorithm of
       HcommGfxHierReduceScatterPlanCreate / Emit / Check (the executors' default between servers); the flat plan
       and schedule calls return HCCL_E_PARA for it */
    HCOMM_GFX_ALG_REDUCE_SCATTER_RHD = 16,
    /* The AICPU deterministic reduce-scatter: AicpuReduceScatter::RunDeterministicReduceScatterLocal
       (src/legacy/ascend910/framework/device/aicpu_kfc/algorithm/aicpu_reduce_scatter.cc:64-118), one pass of its
       loop.  Every rank writes slice d of its input into slot `own rank` of rank d's window (the third buffer:
       HcommGfxScratchBytes = N x count x unit), rank d folds its window in place with
       TaskOrchestrator::SelfLocalReduce (.../task_orchestrator.cc:719-755: the slots beyond the largest power of two
       onto the first ones in one reduce, then rounds of window[0, h) (op)= window[h, 2h), one contiguous reduce
       each) and copies window[0, count) to out[d].  count = per-rank OUTPUT count; input slices at i * strideCount
       (displs, aicpu_reduce_scatter.cc:78-80).  Any rank count.  The fused lowering is one tree launch on the
       inputs alone (the rank-order tree: level l folds rank j + K / 2^(l+1) onto rank j). */
    HCOMM_GFX_ALG_REDUCE_SCATTER_WINDOW_HALVING = 17
} HcommGfxAlgorithm;

typedef enum {
    /* one kernel launch per schedule step, all ranks of the step in that launch; every reduce is a
       two-input dst = dst (op) src exactly as the reference emits it */
    HCOMM_GFX_LOWER_STEPWISE = 0,
    /* steps whose data dependences are element-wise are folded into k-way kernels that read every input
       once and store every value the step-wise replay leaves in a buffer (partials included), so the final
       contents of all 2N buffers are identical to HCOMM_GFX_LOWER_STEPWISE.  Available for the ring, mesh,
       recursive halving-doubling, NHR (sliced and one-shot) and NB algorithms.
       The three algorithms that stage through a communication buffer (deterministic local-reduce allreduce and
       reduce-scatter, chunk-mesh allreduce) are lowered onto the in / out buffers alone: every output holds the bits
       the step-wise replay gives it, the inputs are only read, and no scratch buffers are needed (the argument is
       ignored).  Limits of these three: the local-reduce reduce-scatter needs count * unit to be a multiple of 16,
       the local-reduce allreduce needs its slot size (a multiple of 16 KiB, or of 512 bytes for small messages) to
       keep slices on 16-byte boundaries and at most 16 ranks; otherwise HCCL_E_NOT_SUPPORT.  Inside
       HcommGfxOpBasePlanCreate they stay step-wise only.  ALLREDUCE_DOUBLING, whose steps write the inputs, has
       none (see HCOMM_GFX_LOWER_FUSED_KEEP_INPUTS). */
    HCOMM_GFX_LOWER_FUSED = 1,
    /* the launches of HCOMM_GFX_LOWER_FUSED without their stores into the inputs: every out[r] holds the same bits,
       every in[r] is left as the caller filled it (what the collective's caller sees of the reference, which runs
       its templates on CCL buffers and never writes the send buffer).  One read per input element and one write per
       output element.  Accepted by HcommGfxPlanCreate / Strided / Ex only; the in-place ring reduce-scatter stage,
       whose result lives in the input, returns HCCL_E_NOT_SUPPORT.  The only lowering of ALLREDUCE_DOUBLING besides
       the step-wise one: one tree per rank, root to that rank (N outputs, each from N reads). */
    HCOMM_GFX_LOWER_FUSED_KEEP_INPUTS = 2
} HcommGfxLowering;

typedef struct {
    uint64_t offset; /* bytes from the buffer base */
    uint64_t size;   /* bytes */
} HcommGfxSlice;     /* struct Slice, base/alg_template/template_v1_utils.h:50-53 */

/*
 * Slice table of the allreduce templates: total = count * unit; per = roundup(ceil(total / n), 128);
 * slice i takes min(per, what is left) (temp_all_reduce/all_reduce_ring.cc:142-153,
 * alg_template_base.cc:787-820, recursive_halvingdoubling_base.cc:64-94).  Writes n entries.
 * unitSize 0, n 0 or slices NULL -> error; so is a total beyond 2^62 bytes (HCCL_E_PARA).  Every schedule, plan
 * and emit entry below refuses counts (and strides) above 2^48 elements per rank the same way, so that no byte
 * offset derived from a count can wrap.
 */
int32_t HcommGfxCalcSlices(uint64_t count, uint32_t unitSize, uint32_t n, HcommGfxSlice* slices);

/* Element size in bytes (SIZE_TABLE, pkg_inc/legacy/hccl/dtype_common.h:18-36); 0 for unknown values. */
uint32_t HcommGfxDataTypeSize(HcommDataType dataType);

typedef struct HcommGfxPlan HcommGfxPlan;

/*
 * Build the launch list for one collective over nRanks simulated ranks.
 *   in[r], out[r] : rank r's input and output buffer (device pointers, 128-byte aligned, not overlapping
 *                   each other or any other rank's buffers).  Algorithms that run in place ignore out.
 *   count         : elements per rank (see the algorithm's note for its exact meaning).
 * Dtypes: INT8, INT16, INT32, FP16, FP32, BFP16.  Ops: SUM, MAX, MIN, and PROD where the reference allows it
 * at collective level (param_check.cc:327-343: not INT16, not BFP16).
 * Returns HCCL_SUCCESS and *plan, or an error code and *plan = NULL.  nRanks in [1, HCOMM_GFX_MAX_RANKS].
 * Building a plan allocates nothing on the device and launches nothing.
 */
int32_t HcommGfxPlanCreate(
    HcommGfxAlgorithm alg, HcommGfxLowering lowering, uint32_t nRanks, void* const* in, void* const* out,
    uint64_t count, HcommDataType dataType, HcommReduceOp reduceOp, HcommGfxPlan** plan);

/*
 * As HcommGfxPlanCreate, for the two stand-alone reduce-scatter algorithms with a strided input: rank i's
 * slice starts strideCount elements after rank i-1's (displs[i] = strideLen * i * unitSize,
 * src/legacy/ascend910/framework/device/aicpu_kfc/algorithm/aicpu_reduce_scatter.cc:78-80), so the input
 * buffer holds (nRanks-1)*strideCount + count elements.  strideCount 0 means count (dense);
 * strideCount < count, or a stride with any other algorithm -> HCCL_E_PARA.
 */
int32_t HcommGfxPlanCreateStrided(
    HcommGfxAlgorithm alg, HcommGfxLowering lowering, uint32_t nRanks, void* const* in, void* const* out,
    uint64_t count, uint64_t strideCount, HcommDataType dataType, HcommReduceOp reduceOp, HcommGfxPlan** plan);

/*
 * As HcommGfxPlanCreateStrided, with a per-rank communication ("scratch") buffer for the algorithms that stage
 * data in one (the CCL buffer of the reference).  scratch[r] must be 128-byte aligned and hold
 * HcommGfxScratchBytes() bytes; scratch may be NULL for algorithms that need none.
 */
int32_t HcommGfxPlanCreateEx(
    HcommGfxAlgorithm alg, HcommGfxLowering lowering, uint32_t nRanks, void* const* in, void* const* out,
    void* const* scratch, uint64_t count, uint64_t strideCount, HcommDataType dataType, HcommReduceOp reduceOp,
    HcommGfxPlan** plan);

/* Bytes of communication buffer each rank needs for alg (0 for algorithms that stage nothing). */
int32_t HcommGfxScratchBytes(HcommGfxAlgorithm alg, uint32_t nRanks, uint64_t count, HcommDataType dataType,
                             uint64_t* bytes);

/*
 * The deterministic mesh allreduce (HCOMM_GFX_ALG_ALLREDUCE_LOCAL_REDUCE, step-wise) submitted to `thread` in one call
 * that allocates nothing, neither on the device nor on the host.  No counterpart in the reference: it is for callers
 * that cannot allocate - code under HIP graph capture, serving loops, harnesses that forbid hipMalloc - and so cannot
 * supply the communication buffers HcommGfxPlanCreateEx asks for.  The ranks' communication buffers are slices of one
 * array of HCOMM_GFX_NOALLOC_SCRATCH_BYTES bytes that the library keeps on every GPU it is loaded on, from load until
 * the process ends.  in, out, count, dataType, reduceOp as for HcommGfxPlanCreate; out[r] receives the same bits as
 * the plan's, and in[r] is only read.
 *   nRanks      at most HCOMM_GFX_NOALLOC_MAX_RANKS and a rank count the algorithm takes
 *   size limit  nRanks x (HcommGfxScratchBytes(...) rounded up to 256) must fit the array, else HCCL_E_PARA and nothing
 *               is launched: 8 ranks -> 8 MiB of communication buffer per rank, i.e. just under 8 MiB per rank buffer
 * Every call on a GPU uses that GPU's one array: calls that may overlap in time on one GPU (two threads' streams with
 * no order between them) race on it; calls on one thread's stream are ordered by the stream.  The array keeps the
 * last call's contents; the schedule writes every byte of it that it later reads, so nothing needs clearing.
 * The launches are submitted at once: between HcommBatchModeStart and HcommBatchModeEnd of the calling host thread
 * the call returns HCCL_E_NOT_SUPPORT (it would run ahead of what the batch has recorded), and HCCL_E_UNAVAIL while
 * another host thread's open batch holds operations of `thread`.
 */
#define HCOMM_GFX_NOALLOC_SCRATCH_BYTES (64u << 20)
#define HCOMM_GFX_NOALLOC_MAX_RANKS 8u
int32_t HcommGfxAllReduceLocalReduceNoAlloc(
    ThreadHandle thread, uint32_t nRanks, void* const* in, void* const* out, uint64_t count, HcommDataType dataType,
    HcommReduceOp reduceOp);

/*
 * Enqueue every launch of the plan on the thread, in order.  May be called any number of times, from one host
 * thread at a time.  With HCOMM_GFX_GRAPH=1 in the environment a plan of two or more launches is replayed as a
 * HIP graph captured at its first run on the thread's stream (off by default: it measured slower than
 * launching kernel by kernel); when the caller's stream is itself being captured the launches are always
 * issued individually and become part of the caller's graph.  Like every call that submits at once it returns
 * HCCL_E_NOT_SUPPORT inside the calling host thread's own batch and HCCL_E_UNAVAIL while another host thread's open
 * batch holds operations of `thread`.
 */
int32_t HcommGfxPlanRun(const HcommGfxPlan* plan, ThreadHandle thread);

/* Switch graph replay of HcommGfxPlanRun on or off for this plan (default: HCOMM_GFX_GRAPH in the environment). */
int32_t HcommGfxPlanSetGraphReplay(HcommGfxPlan* plan, int32_t enable);

/* Enqueue launches [first, first + n) only (used to time one phase of a plan). */
int32_t HcommGfxPlanRunRange(const HcommGfxPlan* plan, ThreadHandle thread, uint32_t first, uint32_t n);

int32_t HcommGfxPlanDestroy(HcommGfxPlan* plan);

typedef struct {
    uint32_t launches;        /* kernel launches per run */
    uint32_t steps;           /* schedule steps of the reference algorithm */
    uint64_t algorithmicBytes; /* sum over all two-input steps of 3*b (reduce) or 2*b (copy) */
    uint64_t movedBytes;      /* bytes the launches of this lowering actually read + write */
} HcommGfxPlanInfo;

int32_t HcommGfxPlanGetInfo(const HcommGfxPlan* plan, HcommGfxPlanInfo* info);

/* Per-launch description (same record as the launch log), i in [0, launches). */
int32_t HcommGfxPlanGetLaunch(const HcommGfxPlan* plan, uint32_t i, HcommGfxLaunchRecord* rec);

/*
 * The reduction tree launch i (a HCOMM_GFX_KERNEL_TREE launch) evaluates for its segment `segment`, for inspection and
 * for checking a single-launch lowering against the schedule it stands for without a GPU.  The tree has *k = 2^L leaf
 * positions; leaves[q] receives the rank buffer (the in[] pointer the plan was built with) read at position q, or NULL
 * where the tree has a hole; the element at byte *offset + x of every leaf is folded level by level, level l folding
 * position q + 2^l (src role) onto position q (dst role) for every q that is a multiple of 2^(l+1), holes skipped.
 * *outRank receives the rank whose output takes the root, or -1 when every rank's output does.
 * leaves may be NULL to query *k; cap < *k -> HCCL_E_PARA; offset, bytes and outRank may be NULL.  Not reported: the
 * odd neighbours a recursive halving-doubling launch on a non-power-of-two rank count folds into the even block ranks
 * before the tree, and the partials a launch stores back into the inputs.  No counterpart in the reference: its
 * schedules are only ever run step by step.
 */
int32_t HcommGfxPlanGetTreeSegment(const HcommGfxPlan* plan, uint32_t i, uint32_t segment, const void** leaves,
                                   uint32_t cap, uint32_t* k, uint64_t* offset, uint64_t* bytes, int32_t* outRank);

/*
 * The schedule as the reference's templates emit it, one two-input operation per record, for inspection
 * and for checking a plan against an independent replay.
 */
typedef struct {
    uint32_t step;    /* schedule step (ranks act in parallel within a step) */
    uint32_t kind;    /* 0 = copy, 1 = reduce */
    uint32_t rank;    /* rank that executes the operation (owner of dst) */
    uint32_t dstBuf;  /* 0 = in[rank], 1 = out[rank], 2 = scratch[rank] (communication buffer); op-base lists
                         also use HCOMM_GFX_BUF_USER_IN / HCOMM_GFX_BUF_USER_OUT */
    uint32_t srcRank; /* rank whose buffer is read */
    uint32_t srcBuf;  /* as dstBuf, of srcRank */
    uint64_t dstOff;  /* bytes */
    uint64_t srcOff;  /* bytes */
    uint64_t bytes;
} HcommGfxSchedOp;

/* Buffer roles of an op-base op list: the template runs on the CCL buffers (roles 0, 1, 2), the loop around it
   moves chunks between them and the caller's own buffers. */
#define HCOMM_GFX_BUF_USER_IN 3u
#define HCOMM_GFX_BUF_USER_OUT 4u
#define HCOMM_GFX_NUM_BUFS 5u

/*
 * Emit the op list of an algorithm without any pointers.  Writes up to cap records; *n receives the total.
 * Records are ordered by step, then by rank.
 */
int32_t HcommGfxScheduleEmit(
    HcommGfxAlgorithm alg, uint32_t nRanks, uint64_t count, HcommDataType dataType, HcommGfxSchedOp* ops,
    uint64_t cap, uint64_t* n);

int32_t HcommGfxScheduleEmitStrided(
    HcommGfxAlgorithm alg, uint32_t nRanks, uint64_t count, uint64_t strideCount, HcommDataType dataType,
    HcommGfxSchedOp* ops, uint64_t cap, uint64_t* n);

/*
 * Symbolic check of an op list (no data is moved, no GPU needed) - a miniature of the reference's algorithm
 * checker (test/st/algorithm/README_en.md:13-15,202-231;
 * test/st/algorithm/utils/checker/semantics_check/allreduce_semantics_checker.cc:59-96):
 *   conflicts      - operations of one step that write a range another operation of the step reads or writes;
 *   semanticErrors - bytes of the expected result that do not hold exactly one contribution from every rank,
 *                    taken from the matching offset of that rank's input.
 * message describes the first finding.  The call itself returns HCCL_SUCCESS when the check ran.
 */
typedef enum {
    HCOMM_GFX_EXPECT_ALLREDUCE = 0,               /* out[r][0, count*unit) for every r */
    HCOMM_GFX_EXPECT_REDUCE_SCATTER_IN_PLACE = 1, /* in[r][slice r], slices from HcommGfxCalcSlices(count, unit, n) */
    HCOMM_GFX_EXPECT_REDUCE_SCATTER_OUT = 2,      /* out[r][0, count*unit) = sum of in[k][r*stride*unit + ...] */
    /* op-base lists: the data starts in the user inputs and the result is looked for in the user outputs */
    HCOMM_GFX_EXPECT_ALLREDUCE_USER = 3,
    HCOMM_GFX_EXPECT_REDUCE_SCATTER_USER = 4
} HcommGfxExpectation;

typedef struct {
    uint32_t conflicts;
    uint32_t semanticErrors;
    char message[248];
} HcommGfxCheckReport;

int32_t HcommGfxOpListCheck(
    const HcommGfxSchedOp* ops, uint64_t nOps, uint32_t nRanks, HcommGfxExpectation expect, uint64_t count,
    uint64_t strideCount, uint32_t unitSize, HcommGfxCheckReport* report);

/* Generate the op list of alg and check it against the expectation that belongs to the algorithm. */
int32_t HcommGfxScheduleCheck(
    HcommGfxAlgorithm alg, uint32_t nRanks, uint64_t count, uint64_t strideCount, HcommDataType dataType,
    HcommGfxCheckReport* report);

/*
 * The op-base loop around a template - what the reference's executors do with a caller's buffers when the collective
 * runs through the communicator's CCL buffers (src/legacy/ascend910/algorithm/impl/coll_executor/
 * coll_all_reduce/coll_all_reduce_executor.cc:199-339, coll_reduce_scatter/coll_reduce_scatter_executor.cc:149-306):
 * the message is cut into chunks of at most maxCountPerLoop elements (allreduce: cclBytes / unit; reduce-scatter:
 * cclBytes / N rounded down to 128 bytes, / unit), and every chunk is copied user input -> CCL input, run through
 * the template on the CCL buffers, and copied CCL output -> user output.  A reduce-scatter copies one piece per
 * input slice (a single copy when one chunk takes the whole message).  No counterpart for the in-place ring stage.
 *
 * userIn / userOut: the caller's buffers (allreduce: count elements each; reduce-scatter: N * count in, count out).
 * cclIn / cclOut: cclBytes each, 128-byte aligned.  scratch: as HcommGfxPlanCreateEx, sized for
 * min(count, maxCountPerLoop) elements.  FUSED lowers the template part of every chunk as HcommGfxPlanCreate would.
 * (HCCL_E_NOT_SUPPORT for the algorithms that need scratch: the loop's replay defines what those buffers hold).
 */
int32_t HcommGfxOpBasePlanCreate(
    HcommGfxAlgorithm alg, HcommGfxLowering lowering, uint32_t nRanks, void* const* userIn, void* const* userOut,
    void* const* cclIn, void* const* cclOut, void* const* scratch, uint64_t cclBytes, uint64_t count,
    HcommDataType dataType, HcommReduceOp reduceOp, HcommGfxPlan** plan);

/*
 * The three-step allreduce of the reference's ring executor over two communicator levels
 * (src/legacy/ascend910/algorithm/impl/coll_executor/coll_all_reduce/coll_all_reduce_ring_executor.cc:94-231):
 * nServers x nLocal ranks, rank = server * nLocal + local index.  (1) ring reduce-scatter inside every server, in
 * place on the inputs; (2) for every local index i, level1Alg (HCOMM_GFX_ALG_ALLREDUCE_RING, _RHD, _NHR or _NB) over
 * segment i of the ranks with that index, from the input to the output buffers; (3) ring all-gather inside every
 * server on the outputs.  in / out: nServers * nLocal buffers of count elements.  Step-wise lowering.
 */
int32_t HcommGfxHierPlanCreate(
    HcommGfxAlgorithm level1Alg, uint32_t nServers, uint32_t nLocal, void* const* in, void* const* out, uint64_t count,
    HcommDataType dataType, HcommReduceOp reduceOp, HcommGfxPlan** plan);
int32_t HcommGfxHierEmit(
    HcommGfxAlgorithm level1Alg, uint32_t nServers, uint32_t nLocal, uint64_t count, HcommDataType dataType,
    HcommGfxSchedOp* ops, uint64_t cap, uint64_t* n);
int32_t HcommGfxHierCheck(
    HcommGfxAlgorithm level1Alg, uint32_t nServers, uint32_t nLocal, uint64_t count, HcommDataType dataType,
    HcommGfxCheckReport* report);

/*
 * The same three steps with the mesh executor's level 0
 * (coll_executor/coll_all_reduce/coll_all_reduce_mesh_executor.cc:88-231, its branch without atomic adds):
 * (1) MultiStreamReduceScatterMesh inside every server (coll_comm_executor.cc:1754-1860): every segment cut into
 * nLocal - 1 pieces, piece s folded from the peers in the cyclic order r-1, r-2, ... started at place s, in place on the
 * inputs; (2) as above; (3) AllGatherMesh inside every server on the outputs (alg_template/temp_all_gather/
 * all_gather_mesh.cc:66-131), all segments at once.
 */
int32_t HcommGfxMeshHierPlanCreate(
    HcommGfxAlgorithm level1Alg, uint32_t nServers, uint32_t nLocal, void* const* in, void* const* out, uint64_t count,
    HcommDataType dataType, HcommReduceOp reduceOp, HcommGfxPlan** plan);
int32_t HcommGfxMeshHierEmit(
    HcommGfxAlgorithm level1Alg, uint32_t nServers, uint32_t nLocal, uint64_t count, HcommDataType dataType,
    HcommGfxSchedOp* ops, uint64_t cap, uint64_t* n);
int32_t HcommGfxMeshHierCheck(
    HcommGfxAlgorithm level1Alg, uint32_t nServers, uint32_t nLocal, uint64_t count, HcommDataType dataType,
    HcommGfxCheckReport* report);

/*
 * The allreduce of the reference's double-ring executor for two-ring servers in op-base mode, where the user buffers
 * are read and written directly ("DMA reduce") instead of being staged through the CCL buffers
 * (coll_executor/coll_all_reduce/coll_aligned_all_reduce_double_ring_for_910_93_executor.cc, KernelRun of
 * coll_all_reduce_ring_for_910_93_executor.cc:218-524, loop of coll_all_reduce_executor.cc:234-262), per chunk of at
 * most cclBytes / unit elements:
 *   (1) AlignedReduceScatterDoubleRing inside every server
 *       (alg_template/temp_reduce_scatter/aligned_reduce_scatter_double_ring.cc): every segment is cut in two shares,
 *       share 0 reduced around the ring 0 -> 1 -> ... and share 1 around the mirrored ring; the CCL input buffer is
 *       filled slice by slice from the user input just before each slice is needed;
 *   (2) level1Alg (HCOMM_GFX_ALG_ALLREDUCE_RING, _NHR - one-shot for small chunks - or _NB) between the servers on the
 *       own segment, CCL input -> CCL output;
 *   (3) AlignedAllGatherDoubleRing inside every server (alg_template/temp_all_gather/aligned_all_gather_double_ring.cc):
 *       both shares gathered around their rings in the CCL output buffers, every slice copied on to the user output
 *       (the last one received lands there directly).
 * nServers x nLocal ranks, rank = server * nLocal + local index; one super pod.  userIn / userOut: count elements;
 * cclIn / cclOut: cclBytes each; all 128-byte aligned.  Step-wise lowering.
 */
int32_t HcommGfxDoubleRingPlanCreate(
    HcommGfxAlgorithm level1Alg, uint32_t nServers, uint32_t nLocal, void* const* userIn, void* const* userOut,
    void* const* cclIn, void* const* cclOut, uint64_t cclBytes, uint64_t count, HcommDataType dataType,
    HcommReduceOp reduceOp, HcommGfxPlan** plan);
int32_t HcommGfxDoubleRingEmit(
    HcommGfxAlgorithm level1Alg, uint32_t nServers, uint32_t nLocal, uint64_t count, uint64_t cclBytes,
    HcommDataType dataType, HcommGfxSchedOp* ops, uint64_t cap, uint64_t* n);
int32_t HcommGfxDoubleRingCheck(
    HcommGfxAlgorithm level1Alg, uint32_t nServers, uint32_t nLocal, uint64_t count, uint64_t cclBytes,
    HcommDataType dataType, HcommGfxCheckReport* report);

/*
 * The reduce-scatter of the reference's double-ring executor on one server in op-base mode with DMA reduce
 * (coll_executor/coll_reduce_scatter/coll_aligned_reduce_scatter_double_ring_for_910_93_executor.cc:22-86, slices of
 * coll_reduce_scatter_ring_for_910_93_executor.cc:213-316, AlignedReduceScatterDoubleRing with both user addresses):
 * per chunk of at most cclBytes / nRanks (rounded down to 128 bytes) / unit elements per block, every block is cut in
 * two shares that are reduced around two mirrored rings through the CCL input buffers, fetched from the user input just
 * before they are needed; the last fold of a rank's own block lands in its user output, which the step before filled
 * with the rank's own share.  userIn: nRanks * count elements (block b at b * count); userOut: count; cclIn: cclBytes.
 * nRanks >= 3 (the template's two-rank first step, :353-360, leaves the neighbour's share unwritten; the double-ring
 * servers have more).  Several servers and super pods: HcommGfxDoubleRingHierReduceScatter*, below.
 */
int32_t HcommGfxDoubleRingReduceScatterPlanCreate(
    uint32_t nRanks, void* const* userIn, void* const* userOut, void* const* cclIn, uint64_t cclBytes, uint64_t count,
    HcommDataType dataType, HcommReduceOp reduceOp, HcommGfxPlan** plan);
int32_t HcommGfxDoubleRingReduceScatterEmit(
    uint32_t nRanks, uint64_t count, uint64_t cclBytes, HcommDataType dataType, HcommGfxSchedOp* ops, uint64_t cap,
    uint64_t* n);
int32_t HcommGfxDoubleRingReduceScatterCheck(
    uint32_t nRanks, uint64_t count, uint64_t cclBytes, HcommDataType dataType, HcommGfxCheckReport* report);

/*
 * The same executor over nPods super pods of nServers servers (more than one between them) of nLocal >= 3 devices,
 * rank = (pod * nServers + server) * nLocal + local index (KernelRun of its base,
 * coll_executor/coll_reduce_scatter/coll_reduce_scatter_ring_for_910_93_executor.cc:595-812), per chunk of at most
 * cclBytes / ranks (rounded down to 128 bytes) / unit elements per block:
 *   (1) AlignedReduceScatterDoubleRing inside every server with nPods * nServers slices per ring position - the two
 *       shares of the blocks of the ranks with one local index, one per server of every pod (FillMultiRingSlice :213-233,
 *       user-memory slices :297-313; alg_template/temp_reduce_scatter/aligned_reduce_scatter_double_ring.cc:305-332,
 *       366-425) - and only the user input address set (:664-670), so every fold stays in the CCL input buffers;
 *   (2) nServers > 1: level1Alg (HCOMM_GFX_ALG_REDUCE_SCATTER_RING, _NHR or _NB, :689-746) between the servers of a pod,
 *       in place on the CCL input buffers of the ranks with one local index; server i's rank owns one slice per pod, the
 *       block of the rank with its place in that pod (:327-350), and the templates walk the slices of a rank one after
 *       the other (reduce_scatter_ring.cc:221-224, reduce_scatter_nhr.cc:573-579, reduce_scatter_nb.cc:174);
 *   (3) nPods > 1: level2Alg (the same three, :748-797) between the pods, slice i = the block of pod i's rank (:376-382);
 *   (4) the own block from the CCL input to the user output (:800-808).
 * userIn: ranks * count elements (block b at b * count); userOut: count; cclIn: cclBytes.  The AHC branches and the
 * reduce-scatter-v slices are not built.
 */
int32_t HcommGfxDoubleRingHierReduceScatterPlanCreate(
    HcommGfxAlgorithm level1Alg, HcommGfxAlgorithm level2Alg, uint32_t nPods, uint32_t nServers, uint32_t nLocal,
    void* const* userIn, void* const* userOut, void* const* cclIn, uint64_t cclBytes, uint64_t count, HcommDataType dataType,
    HcommReduceOp reduceOp, HcommGfxPlan** plan);
int32_t HcommGfxDoubleRingHierReduceScatterEmit(
    HcommGfxAlgorithm level1Alg, HcommGfxAlgorithm level2Alg, uint32_t nPods, uint32_t nServers, uint32_t nLocal, uint64_t count,
    uint64_t cclBytes, HcommDataType dataType, HcommGfxSchedOp* ops, uint64_t cap, uint64_t* n);
int32_t HcommGfxDoubleRingHierReduceScatterCheck(
    HcommGfxAlgorithm level1Alg, HcommGfxAlgorithm level2Alg, uint32_t nPods, uint32_t nServers, uint32_t nLocal, uint64_t count,
    uint64_t cclBytes, HcommDataType dataType, HcommGfxCheckReport* report);

/*
 * The reduce-scatter of the reference's ring executor (level0Mesh 0: coll_executor/coll_reduce_scatter/
 * coll_reduce_scatter_ring_executor.cc:136-363, one ring per server) or mesh executor (level0Mesh 1:
 * coll_reduce_scatter_mesh_executor.cc:131-259, its branch without atomic adds) over two communicator levels in
 * op-base mode (loop and staging copies of coll_reduce_scatter_executor.cc:149-306, chunks of at most
 * cclBytes / (N * unit) elements per block, N = nServers * nLocal, rank = server * nLocal + local index):
 * user input -> CCL input; level1Alg (HCOMM_GFX_ALG_REDUCE_SCATTER_RING, _NHR, _NB or _RHD, in place) between the servers over
 * the nServers runs of nLocal blocks; ring or multi-stream mesh reduce-scatter inside every server over the blocks of
 * its run; own block -> CCL output -> user output.
 * userIn: N * count elements (block b at b * count belongs to rank b); userOut: count; cclIn / cclOut: cclBytes.
 */
int32_t HcommGfxHierReduceScatterPlanCreate(
    int32_t level0Mesh, HcommGfxAlgorithm level1Alg, uint32_t nServers, uint32_t nLocal, void* const* userIn,
    void* const* userOut, void* const* cclIn, void* const* cclOut, uint64_t cclBytes, uint64_t count,
    HcommDataType dataType, HcommReduceOp reduceOp, HcommGfxPlan** plan);
int32_t HcommGfxHierReduceScatterEmit(
    int32_t level0Mesh, HcommGfxAlgorithm level1Alg, uint32_t nServers, uint32_t nLocal, uint64_t count, uint64_t cclBytes,
    HcommDataType dataType, HcommGfxSchedOp* ops, uint64_t cap, uint64_t* n);
int32_t HcommGfxHierReduceScatterCheck(
    int32_t level0Mesh, HcommGfxAlgorithm level1Alg, uint32_t nServers, uint32_t nLocal, uint64_t count, uint64_t cclBytes,
    HcommDataType dataType, HcommGfxCheckReport* report);

/*
 * The reduce-scatter of the reference's order-preserving executor on one server in op-base mode
 * (coll_executor/coll_reduce_scatter/coll_reduce_scatter_order_preserved_executor.cc:181-216, 260-283, around
 * ReduceScatterPlantLocalReduce, alg_template/temp_reduce_scatter/reduce_scatter_plant_local_reduce.cc): per chunk of
 * at most cclBytes / nRanks (rounded down to 128 bytes) / unit elements, every rank plants block p of its user input
 * into rank p's CCL output buffer, every rank folds the N blocks it received in RANK order along one fixed tree
 * (so the result does not depend on which rank computes it), and copies its slot to its user output.
 * userIn: nRanks * count elements (block p at p * count); userOut: count elements; cclOut: cclBytes; 128-byte
 * aligned.  nRanks >= 2 (a single rank per module relies on the inter-module stage, which is not built); the
 * executor's recursive-halving branch for messages up to 32 KiB on 4 or 8 devices (:33-38) is
 * HcommGfxOrderPreservedSmallPlanCreate below: this entry point always takes the plant branch.  Step-wise lowering.
 */
int32_t HcommGfxOrderPreservedPlanCreate(
    uint32_t nRanks, void* const* userIn, void* const* userOut, void* const* cclOut, uint64_t cclBytes, uint64_t count,
    HcommDataType dataType, HcommReduceOp reduceOp, HcommGfxPlan** plan);
int32_t HcommGfxOrderPreservedEmit(
    uint32_t nRanks, uint64_t count, uint64_t cclBytes, HcommDataType dataType, HcommGfxSchedOp* ops, uint64_t cap,
    uint64_t* n);
int32_t HcommGfxOrderPreservedCheck(
    uint32_t nRanks, uint64_t count, uint64_t cclBytes, HcommDataType dataType, HcommGfxCheckReport* report);

/*
 * The branch the same executor takes for small messages (coll_reduce_scatter_order_preserved_executor.cc:29-38:
 * count * unit <= 32 KiB, one module of 4 or 8 devices, op-base mode): ReduceScatterHDStage
 * (alg_template/temp_reduce_scatter/reduce_scatter_hd_stage.cc) - every rank copies the half of its user input that
 * holds its block to its CCL output buffer, the rank N / 2 away folds its own copy of that half in, then log2(N) - 1
 * halving steps fold the partner's run of blocks, and block p goes to the user output: 2 + log2(N) operations per
 * rank instead of the plant branch's 2 N.  The fold tree over rank order is the plant branch's, seen from rank p
 * (every leaf XOR p: the two operands of a fold swap places from rank to rank).
 * nRanks 4 or 8, count * unit <= 32 KiB, and the message must fit one chunk (count <= cclBytes / nRanks rounded down
 * to 128 bytes / unit): HCCL_E_PARA otherwise.  Buffers as for HcommGfxOrderPreservedPlanCreate.
 */
int32_t HcommGfxOrderPreservedSmallPlanCreate(
    uint32_t nRanks, void* const* userIn, void* const* userOut, void* const* cclOut, uint64_t cclBytes, uint64_t count,
    HcommDataType dataType, HcommReduceOp reduceOp, HcommGfxPlan** plan);
int32_t HcommGfxOrderPreservedSmallEmit(
    uint32_t nRanks, uint64_t count, uint64_t cclBytes, HcommDataType dataType, HcommGfxSchedOp* ops, uint64_t cap,
    uint64_t* n);
int32_t HcommGfxOrderPreservedSmallCheck(
    uint32_t nRanks, uint64_t count, uint64_t cclBytes, HcommDataType dataType, HcommGfxCheckReport* report);

/*
 * The allreduce of the reference's order-preserving executor on one server in op-base mode
 * (coll_executor/coll_all_reduce/coll_all_reduce_order_preserved_executor.cc:131-193, 248-283, 342-380): per chunk of
 * at most cclBytes / unit elements, cut into N blocks of ceil(chunk / N) elements rounded up to 128 bytes (trailing
 * blocks short or empty), every rank plants block p of its user input into rank p's CCL buffers - N - 1 slots of
 * the CCL output buffer plus, on every rank but the last, one slot borrowed from the CCL input buffer
 * (alg_template/temp_reduce_scatter/reduce_scatter_plant_local_reduce.cc:168-188, 221-247) - rank p folds them in
 * RANK order along the fixed tree of the order-preserving reduce-scatter, the blocks are gathered over the mesh
 * inside the CCL output buffers (alg_template/temp_all_gather/all_gather_mesh_atomic.cc:19-69) and the chunk is copied
 * to the user output.  The result is bit-identical on every rank and does not depend on N's factorisation.
 * userIn, userOut: count elements; cclIn, cclOut: cclBytes; 128-byte aligned.  nRanks >= 2; the inter-module stages
 * (:208-246, :285-340) are not built.  HCCL_E_PARA when the N - 1 rounded-up slots of a chunk reach past cclBytes
 * (CCL buffers below about N * N * 128 bytes; the reference's DeviceMem::range refuses them too).  Step-wise lowering.
 */
int32_t HcommGfxOrderPreservedAllReducePlanCreate(
    uint32_t nRanks, void* const* userIn, void* const* userOut, void* const* cclIn, void* const* cclOut,
    uint64_t cclBytes, uint64_t count, HcommDataType dataType, HcommReduceOp reduceOp, HcommGfxPlan** plan);
int32_t HcommGfxOrderPreservedAllReduceEmit(
    uint32_t nRanks, uint64_t count, uint64_t cclBytes, HcommDataType dataType, HcommGfxSchedOp* ops, uint64_t cap,
    uint64_t* n);
int32_t HcommGfxOrderPreservedAllReduceCheck(
    uint32_t nRanks, uint64_t count, uint64_t cclBytes, HcommDataType dataType, HcommGfxCheckReport* report);

/*
 * The same executor over nServers modules of nLocal devices each (rank = server * nLocal + local index;
 * coll_all_reduce_order_preserved_executor.cc:149-193, 208-246, 285-340): inside every server the plant template works
 * on one group of nLocal blocks per server with an all-to-all offset of 1, so that the partial for block b lands one
 * slot beside b's own place; between the servers ReduceScatterPlantLocalReduceCombine
 * (alg_template/temp_reduce_scatter/reduce_scatter_plant_local_reduce_combine.cc, SDMA branch) plants the partials
 * into the blocks' own places and folds them in SERVER order; then the mesh all-gather inside the servers, the
 * all-gather of the servers' runs between them - level1Alg HCOMM_GFX_ALG_ALLREDUCE_RING, _NB or _NHR selects
 * AllGatherRing, AllGatherNB or AllGatherNHR (:293-303) - and the copy to the user output.  Every element is
 * reduced as tree(servers)( tree(devices of server 0), tree(devices of server 1), ... ) with the rank-order tree of
 * the single-server executor at both levels.  nServers >= 2; with nLocal == 1 (one device per module, :195-206) level 0
 * is a copy of the chunk into the CCL input buffer, the stage between the servers reads its blocks from there and
 * nothing is gathered inside the module.  Buffers and errors as above.  Step-wise lowering.
 */
int32_t HcommGfxOrderPreservedHierAllReducePlanCreate(
    HcommGfxAlgorithm level1Alg, uint32_t nServers, uint32_t nLocal, void* const* userIn, void* const* userOut,
    void* const* cclIn, void* const* cclOut, uint64_t cclBytes, uint64_t count, HcommDataType dataType,
    HcommReduceOp reduceOp, HcommGfxPlan** plan);
int32_t HcommGfxOrderPreservedHierAllReduceEmit(
    HcommGfxAlgorithm level1Alg, uint32_t nServers, uint32_t nLocal, uint64_t count, uint64_t cclBytes,
    HcommDataType dataType, HcommGfxSchedOp* ops, uint64_t cap, uint64_t* n);
int32_t HcommGfxOrderPreservedHierAllReduceCheck(
    HcommGfxAlgorithm level1Alg, uint32_t nServers, uint32_t nLocal, uint64_t count, uint64_t cclBytes,
    HcommDataType dataType, HcommGfxCheckReport* report);

/*
 * The order-preserving REDUCE-SCATTER executor over nServers modules of nLocal devices
 * (coll_executor/coll_reduce_scatter/coll_reduce_scatter_order_preserved_executor.cc:171-218, 220-258, 260-283): the
 * two plant levels of the allreduce executor above on blocks of one chunk each (at most cclBytes / N rounded down to
 * 128 bytes per block), without borrowed places, and rank p's block from the CCL output buffer to its user output.
 * userIn: N * count elements per rank (block p at p * count); userOut: count elements; cclOut: cclBytes.  Rank p's
 * result is tree(servers)( tree(devices of server 0), ... ) over the N contributions to block p.
 * nServers >= 2.  nLocal == 1 (one device per module, :123-139, :246-252) stages the N blocks in the CCL input buffer
 * instead of planting inside the server and runs the stage between the servers with the borrowed place: only then is
 * cclIn used (cclBytes each); it may be NULL otherwise.  Step-wise lowering.
 */
int32_t HcommGfxOrderPreservedHierReduceScatterPlanCreate(
    uint32_t nServers, uint32_t nLocal, void* const* userIn, void* const* userOut, void* const* cclIn, void* const* cclOut,
    uint64_t cclBytes, uint64_t count, HcommDataType dataType, HcommReduceOp reduceOp, HcommGfxPlan** plan);
int32_t HcommGfxOrderPreservedHierReduceScatterEmit(
    uint32_t nServers, uint32_t nLocal, uint64_t count, uint64_t cclBytes, HcommDataType dataType, HcommGfxSchedOp* ops,
    uint64_t cap, uint64_t* n);
int32_t HcommGfxOrderPreservedHierReduceScatterCheck(
    uint32_t nServers, uint32_t nLocal, uint64_t count, uint64_t cclBytes, HcommDataType dataType,
    HcommGfxCheckReport* report);

/*
 * The single-launch lowering of the order-preserving executors (no counterpart in the reference, which has no device
 * that can read N ranks' memory in one kernel): every element of the result is folded in registers from the N user
 * inputs along the executors' fixed tree - on one server (nServers == 1) the tree over rank order
 * (reduce_scatter_plant_local_reduce.cc:337-414: contribution h + j onto contribution j for h = 2^(S-1), .., 1); over
 * nServers x nLocal ranks that tree over every server's devices, then the same shape over the servers
 * (reduce_scatter_plant_local_reduce_combine.cc:232-304) - and written straight to the user output(s).
 * allReduce == 0: userIn holds N * count elements per rank and rank p's userOut receives block p (the result of
 * HcommGfxOrderPreservedPlanCreate / HcommGfxOrderPreservedHierReduceScatterPlanCreate); allReduce != 0: count
 * elements in and out on every rank (the result of HcommGfxOrderPreservedAllReducePlanCreate /
 * HcommGfxOrderPreservedHierAllReducePlanCreate).  The user outputs are bit-identical to those plans' for every data
 * type and reduce operation; the user inputs are only read; the CCL buffers are not needed and not touched, so there
 * is no chunk loop.  HCCL_E_NOT_SUPPORT for a reduce-scatter whose block (count * unit bytes) is not a multiple of
 * 16 bytes, and where ceil_pow2(nServers) * ceil_pow2(nLocal) exceeds 32 (5 x 6, 3 x 9 ...): use the step-wise plan.
 * Buffers 128-byte aligned, at least two ranks.
 */
int32_t HcommGfxOrderPreservedFusedPlanCreate(
    int32_t allReduce, uint32_t nServers, uint32_t nLocal, void* const* userIn, void* const* userOut, uint64_t count,
    HcommDataType dataType, HcommReduceOp reduceOp, HcommGfxPlan** plan);

/*
 * A plan from a caller's own op list - any schedule written as the two operations the reference's templates hand
 * to the dispatcher (HcclD2DMemcpyAsync / HcclReduceAsync, src/legacy/ascend910/platform/task/
 * dispatcher_common.cc:114-147), ordered by step.  buffers[role][rank] gives the device buffer behind each of the
 * HCOMM_GFX_NUM_BUFS roles an operation may name (a role no operation names may be NULL).  Operations of a step
 * are merged into single launches exactly as batch mode merges primitive calls (no written range may overlap
 * another range the launch reads or writes); HcommGfxOpListCheck verifies such a list without a GPU.
 */
int32_t HcommGfxPlanCreateFromOps(
    const HcommGfxSchedOp* ops, uint64_t nOps, uint32_t nRanks, void* const* const* buffers, HcommDataType dataType,
    HcommReduceOp reduceOp, HcommGfxPlan** plan);

/*
 * A caller's own op list over the roles 0 (in), 1 (out) and 2 (communication buffer) as tree launches that keep the
 * inputs: the list is replayed on symbols, and what it leaves in the outputs - per byte range a tree of dst (op) src
 * folds over input ranges - is evaluated in registers from the original inputs.  Every out range the list writes
 * receives the bits the list's replay would give it; in[] is only read and no communication buffer is needed, whatever
 * the list does to them.  HCCL_E_NOT_SUPPORT when a range is read with other bounds than it was written with, when a
 * value is read that the list never wrote, when an operation reads or writes a range that an earlier operation of the
 * same step writes (the operations of a step must not observe each other: such a step has no single meaning), as
 * soon as a tree grows deeper than 5 folds, when a tree combines ranges at different offsets or starts off a 16-byte
 * boundary.  ops ordered by step.  No counterpart in the reference.
 */
int32_t HcommGfxPlanCreateFromOpsKeepInputs(
    const HcommGfxSchedOp* ops, uint64_t nOps, uint32_t nRanks, void* const* in, void* const* out, HcommDataType dataType,
    HcommReduceOp reduceOp, HcommGfxPlan** plan);

/* Elements per chunk of the op-base loop. */
int32_t HcommGfxOpBaseMaxCount(HcommGfxAlgorithm alg, uint32_t nRanks, uint64_t cclBytes, HcommDataType dataType,
                               uint64_t* maxCountPerLoop);

/* The op list HcommGfxOpBasePlanCreate replays (buffer roles 0-2 are the CCL buffers, 3 and 4 the caller's). */
int32_t HcommGfxOpBaseEmit(
    HcommGfxAlgorithm alg, uint32_t nRanks, uint64_t count, uint64_t cclBytes, HcommDataType dataType,
    HcommGfxSchedOp* ops, uint64_t cap, uint64_t* n);

/* Generate the op-base op list and check it (HCOMM_GFX_EXPECT_ALLREDUCE_USER / _REDUCE_SCATTER_USER). */
int32_t HcommGfxOpBaseCheck(
    HcommGfxAlgorithm alg, uint32_t nRanks, uint64_t count, uint64_t cclBytes, HcommDataType dataType,
    HcommGfxCheckReport* report);

/* No reference counterpart.  Small launches (a few MiB; a fold of at most 16 inputs) run kernels of their own that
 * read all their arguments at once: addresses resolved on the host, a two-dimensional grid (segment, tile).  Passing
 * 0 keeps every launch shaped after this call (plans: at creation) on the kernels large launches use, which is how
 * the tests run those kernels on small and ragged shapes; 1 restores the default.  Returns the previous setting.
 * HCOMM_GFX_DIRECT=0 in the environment sets the initial value to 0. */
int32_t HcommGfxSetDirectLaunches(int32_t enable);

/* No reference counterpart.  A copy / two-input reduce launch that writes more than `bytes` and reads what one of
 * its thread's last two such launches wrote walks its table the other way than that launch did (it starts on what
 * the memory-side cache still holds of it); 0 = no launch ever does.  Returns the previous value; the initial one is
 * HCOMM_GFX_ALTERNATE_BYTES from the environment, 128 MiB without it.  Results never depend on it; tests lower it
 * to run both directions on small shapes. */
uint64_t HcommGfxSetAlternateBytes(uint64_t bytes);

/* No reference counterpart.  A step-wise plan created after this call whose steps write more than 2.5 x `bytes`, and
 * whose operations are whole slices (any two ranges they touch the same or apart), runs piece by piece: all steps on
 * the first part of every slice, then all steps on the second, ... about `bytes` written per launch and no piece
 * shorter than an eighth of that, so that each step finds what the step before wrote in the memory-side cache.
 * 0 = plans keep one launch per step.  Returns the previous value; the initial one is HCOMM_GFX_PIECE_BYTES from
 * the environment, 128 MiB without it.  Results never depend on it. */
uint64_t HcommGfxSetPieceBytes(uint64_t bytes);

/* Library version string, e.g. "hcomm_gfx 0.1 gfx950". */
const char* HcommGfxVersion(void);

#ifdef __cplusplus
}
#endif
#endif /* HCOMM_GFX_H */
