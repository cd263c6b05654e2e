/*
 * hg_host.h - host-side objects of libhcomm_gfx.so shared by hg_api.c, hg_batch.c, hg_sched.c and hg_plan.c.
 */
#ifndef HG_HOST_H
#define HG_HOST_H

#include "hg_internal.h"

#define HG_THREAD_MAGIC 0x48474654u /* "HGFT" */
#define HG_PLAN_MAGIC 0x4847504cu   /* "HGPL" */

/* One recorded primitive call (also the unit the batch coalescer works on). */
typedef struct {
    uint8_t is_reduce;
    uint8_t dtype; /* HcommDataType (255 for copies) */
    uint8_t op;    /* HcommReduceOp (255 for copies) */
    uint8_t sync;  /* only in a thread's batch queue: 0 = a copy / reduce, HG_SYNC_RECORD (dst = the HgThread notified),
                      HG_SYNC_WAIT; never reaches the coalescer */
    uint32_t idx;  /* notify slot of a record / wait */
    void* dst;
    const void* src;
    uint64_t bytes;
} HgOp;

/* One kernel launch, fully prepared on the host. */
typedef struct {
    uint32_t kind; /* HcommGfxKernelKind */
    uint32_t dtype;
    uint32_t op;
    uint32_t acc_is_dst; /* fold kernels only */
    uint64_t blocks;
    uint64_t bytes;       /* output bytes covered */
    uint64_t moved_bytes; /* bytes read + written */
    uint32_t nseg;
    uint32_t streaming;   /* copy / two-input reduce: nothing it writes is expected in the memory-side cache later */
    uint32_t lds_bytes;   /* dynamic LDS per workgroup: bounds the workgroups per CU, never used as memory */
    union {
        HgSeg2Table seg2;
        HgFoldTable fold;
    } tab;
} HgLaunch;

#define HG_SYNC_RECORD 1u
#define HG_SYNC_WAIT 2u

typedef struct HgThread {
    uint32_t magic;
    int recorder;     /* 1: log launches, never touch the GPU */
    int owns_stream;
    void* stream;     /* hipStream_t */
    uint32_t notify_num;
    void** notifies;  /* hipEvent_t per slot */
    uint64_t* notify_pending; /* per slot: records issued that no wait has consumed yet (atomics: recorded by other threads) */
    /* operations recorded in batch mode, in call order */
    HgOp* pending;
    uint32_t pending_n, pending_cap;
    /* launch log */
    HcommGfxLaunchRecord* log;
    uint32_t log_n, log_cap;
    /* the host thread's launch context that holds recorded operations of this thread between HcommBatchModeStart and
     * End (NULL outside a batch); read and written with atomics: another host thread may ask to free the thread */
    const void* batch_owner;
    int log_enabled;
    int log_fixed; /* set while a call that must not allocate runs: the log takes what fits and drops the rest */
    /* batches that order several threads by notifies run on one of them: */
    void* join_ev;      /* hipEvent_t (created on first use) by which this thread's stream and another's are ordered */
    int own_work;       /* something was submitted on this thread's own stream since it was last joined to another */
    /* what the thread's last two large copy / two-input reduce launches wrote, and which way they walked (hg_submit) */
    struct HgWritten {
        uint32_t n;
        int backwards;
        const void* at[HG_MAX_SEG2];
        uint64_t bytes[HG_MAX_SEG2];
    } written[2]; /* [0] the later one */
    int led_batch;      /* other threads may still be waiting to be put behind join_ev on this thread's stream */
    struct HgThread* after; /* first thread of the batch this thread's stream is still to be put behind (hg_thread_settle) */
    uint32_t batch_cursor; /* next entry of `pending` while HcommBatchModeEnd walks the threads of a batch */
} HgThread;

HgThread* hg_thread_from_handle(ThreadHandle h);
/* Puts the thread's stream behind the batch it last took part in on another thread's stream, if that is still due: to be
 * called before anything is queued on, recorded on or waited for on the thread's stream outside hg_submit. */
int hg_thread_settle(HgThread* t);
/* HCCL_SUCCESS, or HCCL_E_UNAVAIL while a batch of ANOTHER host thread holds recorded operations of the thread */
int hg_thread_free_for_caller(const HgThread* t);
/* whether the calling host thread is between HcommBatchModeStart and HcommBatchModeEnd */
int hg_caller_is_batching(void);

/* Turn a list of operations (stream order) into launches: consecutive independent operations of equal
 * kind / dtype / op share one launch.  Calls emit(launch, ctx) for each; stops at the first error. */
typedef int (*HgEmitFn)(const HgLaunch* launch, void* ctx);
int hg_coalesce(const HgOp* ops, uint64_t n, HgEmitFn emit, void* ctx);
/* the same with the launch under construction in storage of the caller's (no allocation) */
int hg_coalesce_with(const HgOp* ops, uint64_t n, HgEmitFn emit, void* ctx, HgLaunch* work);
uint64_t hg_split_head(const HgOp* o);      /* bytes before the 16-byte boundary both operands reach together, or 0 */
uint64_t hg_alternate_bytes(void);
/* ops[0 .. *m) with the step of each (malloc'ed, steps numbered in order): replaced by the piece-major list when the
 * schedule has a step larger than the memory-side cache serves and is made of whole slices (hg_plan.c) */
int hg_cut_into_pieces(HgOp** ops_io, uint32_t** steps_io, uint64_t* m_io);
uint64_t hg_piece_bytes(void); /* the size such pieces aim at; 0 = nothing is cut */
uint32_t hg_op_launch_key(const HgOp* o);   /* operations with different keys never share a launch */

/* Fill tile_begin / blocks / bytes and the launch shape (streaming, lds_bytes, xcd_run) of a launch whose segment
 * pointers and sizes are set. */
void hg_finish_seg2(HgLaunch* l);
uint32_t hg_launch_rows(const HgLaunch* l);
void hg_shape_seg2(HgLaunch* l, int streaming); /* streaming < 0: decided by the bytes the launch writes */
void hg_finish_fold(HgLaunch* l);

/* Execute (or, on a recorder thread, log) one prepared launch. */
int hg_submit(HgThread* t, const HgLaunch* l);
/* Append one prepared launch to the thread's log without executing it. */
void hg_log_only(HgThread* t, const HgLaunch* l);

int hg_dtype_supported(int dtype);
int hg_reduce_supported(int dtype, int op, int allow_prod);

#endif
