/*
 * hg_api.c - the exported primitives: threads, local copy / reduce, notifies, memory, batch mode.
 *
 * Mirrors the host adapter of the reference (src/base_comm/primitives/api_c_adpt/cpu_primitives_c_adpt.cc,
 * hcomm_thread_c_adpt.cc) in names, argument meaning, check order and return codes.  A ThreadHandle is an
 * opaque pointer to a library-owned object, as in the reference (cpu_primitives_c_adpt.cc:66).
 */
#define _POSIX_C_SOURCE 200809L
#include <pthread.h>
#include <sched.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

#include "hg_host.h"

_Static_assert(sizeof(HcommBatchTransferDesc) == 64, "HcommBatchTransferDesc must keep the reference's 64-byte layout");

#define HG_LOG_MAX (1u << 16)
#define HG_TOUCHED_MAX 64u

static int g_allow_prod = -1;

/* Settings read from the environment on first use: several host threads may get there at once, every one of them
 * computes the same value, and the relaxed atomics keep that a defined program. */
static int allow_prod(void)
{
    int v = __atomic_load_n(&g_allow_prod, __ATOMIC_RELAXED);
    if (v < 0) {
        const char* e = getenv("HCOMM_GFX_ALLOW_PROD");
        v = (e && e[0] == '1') ? 1 : 0;
        __atomic_store_n(&g_allow_prod, v, __ATOMIC_RELAXED);
    }
    return v;
}

/* thread_local launch context of the calling host thread (cpu_primitives_c_adpt.cc:27) */
static _Thread_local struct {
    int batching;
    HgThread* touched[HG_TOUCHED_MAX];
    uint32_t ntouched;
} g_ctx;

const char* HcommGfxVersion(void) { return "hcomm_gfx 0.1 gfx950"; }

uint32_t HcommGfxDataTypeSize(HcommDataType dataType)
{
    /* SIZE_TABLE, pkg_inc/legacy/hccl/dtype_common.h:18-36 */
    switch ((int)dataType) {
        case HCOMM_DATA_TYPE_INT8: return 1;
        case HCOMM_DATA_TYPE_INT16: return 2;
        case HCOMM_DATA_TYPE_INT32: return 4;
        case HCOMM_DATA_TYPE_FP16: return 2;
        case HCOMM_DATA_TYPE_FP32: return 4;
        case HCOMM_DATA_TYPE_INT64: return 8;
        case HCOMM_DATA_TYPE_UINT64: return 8;
        case HCOMM_DATA_TYPE_UINT8: return 1;
        case HCOMM_DATA_TYPE_UINT16: return 2;
        case HCOMM_DATA_TYPE_UINT32: return 4;
        case HCOMM_DATA_TYPE_FP64: return 8;
        case HCOMM_DATA_TYPE_BFP16: return 2;
        case HCOMM_DATA_TYPE_INT128: return 16;
        case 13: return 2;
        case HCOMM_DATA_TYPE_HIF8: return 1;
        case HCOMM_DATA_TYPE_FP8E4M3: return 1;
        case HCOMM_DATA_TYPE_FP8E5M2: return 1;
        case HCOMM_DATA_TYPE_FP8E8M0: return 1;
        default: return 0;
    }
}

int hg_dtype_supported(int dtype)
{
    return dtype == HCOMM_DATA_TYPE_FP32 || dtype == HCOMM_DATA_TYPE_FP16 || dtype == HCOMM_DATA_TYPE_INT8 ||
           dtype == HCOMM_DATA_TYPE_INT16 || dtype == HCOMM_DATA_TYPE_INT32 || dtype == HCOMM_DATA_TYPE_BFP16;
}

int hg_reduce_supported(int dtype, int op, int prod_ok)
{
    if (!hg_dtype_supported(dtype)) return 0;
    if (op == HCOMM_REDUCE_SUM || op == HCOMM_REDUCE_MAX || op == HCOMM_REDUCE_MIN) return 1;
    /* PROD: the collective-level matrix of the reference for 910B / 910_93 excludes int16 and bf16
     * (HcomCheckReduceDataType, framework/common/src/param_check.cc:327-343) */
    if (op == HCOMM_REDUCE_PROD && prod_ok) return dtype != HCOMM_DATA_TYPE_INT16 && dtype != HCOMM_DATA_TYPE_BFP16;
    return 0;
}

/* Live thread objects.  A handle is only dereferenced after it was found here, so a stale or made-up handle
 * is refused instead of followed (the reference keeps the same kind of map, hcomm_thread_c_adpt.cc:31-35). */
#define HG_THREADS_MAX 1024u
static HgThread* g_threads[HG_THREADS_MAX];
static uint32_t g_threads_hi = 0;
static pthread_mutex_t g_threads_mtx = PTHREAD_MUTEX_INITIALIZER;

static int registry_add(HgThread* t)
{
    int ok = 0;
    pthread_mutex_lock(&g_threads_mtx);
    for (uint32_t i = 0; i < HG_THREADS_MAX; ++i) {
        if (!g_threads[i]) {
            __atomic_store_n(&g_threads[i], t, __ATOMIC_RELEASE); /* readers look up without the mutex */
            if (i + 1 > g_threads_hi) __atomic_store_n(&g_threads_hi, i + 1, __ATOMIC_RELEASE);
            ok = 1;
            break;
        }
    }
    pthread_mutex_unlock(&g_threads_mtx);
    return ok;
}

static void registry_remove(HgThread* t)
{
    pthread_mutex_lock(&g_threads_mtx);
    for (uint32_t i = 0; i < g_threads_hi; ++i)
        if (g_threads[i] == t) __atomic_store_n(&g_threads[i], (HgThread*)NULL, __ATOMIC_RELEASE);
    pthread_mutex_unlock(&g_threads_mtx);
}

HgThread* hg_thread_from_handle(ThreadHandle h)
{
    HgThread* t = (HgThread*)(uintptr_t)h;
    if (!t) return NULL;
    const uint32_t hi = __atomic_load_n(&g_threads_hi, __ATOMIC_ACQUIRE);
    for (uint32_t i = 0; i < hi; ++i)
        if (__atomic_load_n(&g_threads[i], __ATOMIC_ACQUIRE) == t) return (t->magic == HG_THREAD_MAGIC) ? t : NULL;
    return NULL;
}

/* ---- threads ---------------------------------------------------------------------------------- */

static HgThread* thread_new(int recorder, void* stream, int owns_stream, uint32_t notify_num)
{
    HgThread* t = (HgThread*)calloc(1, sizeof(HgThread));
    if (!t) return NULL;
    t->magic = HG_THREAD_MAGIC;
    t->recorder = recorder;
    t->stream = stream;
    t->owns_stream = owns_stream;
    t->notify_num = notify_num;
    t->log_enabled = 1;
    if (!recorder) {
        /* set-up is the place to look up where the library's own array lives on this thread's GPU, so that
         * HcommGfxAllReduceLocalReduceNoAlloc finds the address ready; a failure here only postpones the lookup */
        void* unused = NULL;
        (void)hg_rt_scratch(stream, &unused);
    }
    if (notify_num) {
        t->notifies = (void**)calloc(notify_num, sizeof(void*));
        t->notify_pending = (uint64_t*)calloc(notify_num, sizeof(uint64_t));
        if (!t->notifies || !t->notify_pending) {
            free(t->notifies);
            free(t->notify_pending);
            free(t);
            return NULL;
        }
        if (!recorder) {
            for (uint32_t i = 0; i < notify_num; ++i) {
                if (hg_rt_event_create(&t->notifies[i]) != HCCL_SUCCESS) {
                    for (uint32_t j = 0; j < i; ++j) hg_rt_event_destroy(t->notifies[j]);
                    free(t->notifies);
                    free(t->notify_pending);
                    free(t);
                    return NULL;
                }
            }
        }
    }
    if (!registry_add(t)) {
        if (!recorder)
            for (uint32_t i = 0; i < notify_num; ++i) hg_rt_event_destroy(t->notifies[i]);
        free(t->notifies);
        free(t->notify_pending);
        free(t);
        return NULL;
    }
    return t;
}

static void thread_delete(HgThread* t)
{
    if (!t) return;
    registry_remove(t);
    /* a thread freed between HcommBatchModeStart and End takes its recorded operations with it */
    for (uint32_t i = 0; i < g_ctx.ntouched; ++i)
        if (g_ctx.touched[i] == t) g_ctx.touched[i] = NULL;
    if (!t->recorder) {
        /* threads that a batch put behind this one's stream and that have not been used since find it gone: what
         * they were to wait for is finished before it goes */
        if (t->led_batch && t->stream && !t->owns_stream) hg_rt_stream_sync(t->stream);
        if (t->owns_stream && t->stream) {
            hg_rt_stream_sync(t->stream);
            hg_rt_stream_destroy(t->stream);
        }
        for (uint32_t i = 0; i < t->notify_num; ++i)
            if (t->notifies[i]) hg_rt_event_destroy(t->notifies[i]);
        if (t->join_ev) hg_rt_event_destroy(t->join_ev);
    }
    free(t->notifies);
    free(t->notify_pending);
    free(t->pending);
    free(t->log);
    t->magic = 0;
    free(t);
}

HcommResult
HcommThreadAlloc(CommEngine engine, uint32_t threadNum, const uint32_t* notifyNumPerThread, ThreadHandle* threads)
{
    (void)engine;
    if (!threads) return HCCL_E_PTR;
    if (!notifyNumPerThread) return HCCL_E_PTR;
    if (threadNum == 0) return HCCL_E_PARA;
    if (hg_rt_device_count() <= 0) return HCCL_E_UNAVAIL;
    const uint32_t notify_num = notifyNumPerThread[0]; /* only [0] is used (hcomm_thread_c_adpt.cc:44-49) */
    for (uint32_t i = 0; i < threadNum; ++i) {
        void* stream = NULL;
        HgThread* t = NULL;
        if (hg_rt_stream_create(&stream) == HCCL_SUCCESS) t = thread_new(0, stream, 1, notify_num);
        if (!t) {
            if (stream) hg_rt_stream_destroy(stream);
            for (uint32_t j = 0; j < i; ++j) thread_delete(hg_thread_from_handle(threads[j]));
            return HCCL_E_INTERNAL;
        }
        threads[i] = (ThreadHandle)(uintptr_t)t;
    }
    return HCCL_SUCCESS;
}

HcommResult HcommThreadFree(const ThreadHandle* threads, uint32_t threadNum)
{
    if (!threads) return HCCL_E_PTR;
    HcommResult ret = HCCL_SUCCESS;
    for (uint32_t i = 0; i < threadNum; ++i) {
        HgThread* t = hg_thread_from_handle(threads[i]);
        if (!t) {
            ret = HCCL_E_NOT_FOUND;
            continue;
        }
        /* operations recorded on it by a batch of another host thread are still to be submitted by that thread's
         * HcommBatchModeEnd: the thread stays until then */
        const void* owner = __atomic_load_n(&t->batch_owner, __ATOMIC_ACQUIRE);
        if (owner && owner != (const void*)&g_ctx) {
            ret = HCCL_E_UNAVAIL;
            continue;
        }
        thread_delete(t);
    }
    return ret;
}

HcommResult HcommThreadAllocWithStream(CommEngine engine, void* stream, uint32_t notifyNum, ThreadHandle* thread)
{
    (void)engine;
    if (!thread) return HCCL_E_PTR;
    if (hg_rt_device_count() <= 0) return HCCL_E_UNAVAIL;
    HgThread* t = thread_new(0, stream, 0, notifyNum);
    if (!t) return HCCL_E_INTERNAL;
    *thread = (ThreadHandle)(uintptr_t)t;
    return HCCL_SUCCESS;
}

HcommResult HcommThreadFreeWithStream(const ThreadHandle* threads, uint32_t threadNum)
{
    if (!threads) return HCCL_E_PTR;
    if (threadNum == 0) return HCCL_E_PARA; /* hcomm_thread_c_adpt.cc:190-193 */
    return HcommThreadFree(threads, threadNum);
}

HcommResult HcommGfxRecorderThreadAlloc(ThreadHandle* thread)
{
    if (!thread) return HCCL_E_PTR;
    HgThread* t = thread_new(1, NULL, 0, HCOMM_GFX_MAX_RANKS); /* one notify slot per possible peer: their bookkeeping is host logic, no event behind them */
    if (!t) return HCCL_E_MEMORY;
    *thread = (ThreadHandle)(uintptr_t)t;
    return HCCL_SUCCESS;
}

int32_t HcommGfxThreadSynchronize(ThreadHandle thread)
{
    HgThread* t = hg_thread_from_handle(thread);
    if (!t) return HCCL_E_PTR;
    if (t->recorder) return HCCL_SUCCESS;
    const int rc = hg_thread_settle(t);
    if (rc != HCCL_SUCCESS) return rc;
    return hg_rt_stream_sync(t->stream);
}

/* ---- launch log and submission ---------------------------------------------------------------------- */

static void log_launch(HgThread* t, const HgLaunch* l, int backwards)
{
    if (!t->log_enabled || t->log_n >= HG_LOG_MAX) return;
    if (t->log_n == t->log_cap) {
        if (t->log_fixed) return;
        uint32_t cap = t->log_cap ? t->log_cap * 2 : 64;
        HcommGfxLaunchRecord* p = (HcommGfxLaunchRecord*)realloc(t->log, cap * sizeof(*p));
        if (!p) return;
        t->log = p;
        t->log_cap = cap;
    }
    HcommGfxLaunchRecord* r = &t->log[t->log_n++];
    r->kind = l->kind;
    r->dtype = l->dtype;
    r->op = l->op;
    r->nseg = l->nseg;
    r->bytes = l->bytes;
    r->blocks = l->blocks;
    r->rows = hg_launch_rows(l);
    r->streaming = l->streaming;
    r->backwards = (uint32_t)backwards;
    r->reserved = 0;
}

void hg_log_only(HgThread* t, const HgLaunch* l) { log_launch(t, l, 0); }

/*
 * A batch that ordered its threads by notifies ran on the stream of its first thread.  Its other threads are put
 * behind the end of that batch only when they are next given something or synchronised - a wait on every one of
 * their streams at the end of each batch delayed the batch's own launches by a tenth of its run time - and this is
 * that moment.  The first thread's event is recorded anew by every such batch it leads: waiting for a later
 * record than the one meant waits longer, never shorter.  A first thread that is gone by now was synchronised when
 * it was freed.
 */
int hg_thread_settle(HgThread* t)
{
    HgThread* lead = t->after;
    if (!lead) return HCCL_SUCCESS;
    t->after = NULL;
    lead = hg_thread_from_handle((ThreadHandle)(uintptr_t)lead);
    if (!lead || lead == t || t->recorder || lead->recorder || !lead->join_ev) return HCCL_SUCCESS;
    return hg_rt_stream_wait_event(t->stream, lead->join_ev);
}

/*
 * Which way a large copy / two-input reduce launch walks its table.  A step of a schedule reads what a step before
 * it wrote.  When that step wrote more than the memory-side cache keeps, the cache is left with what it wrote LAST -
 * which a launch walking memory in the same direction reaches last, after its own traffic has displaced it.  So a
 * launch that reads what one of the thread's last two large launches wrote walks the other way than that launch
 * did (last segment first, every segment's last tile first: it starts on the bytes still cached); one that reads
 * nothing of theirs (the first step of a collective, a fetch of fresh data between two folds) walks forwards.
 * 16-rank halving-doubling allreduce 1.535 -> 1.506 ms, 7-rank ring reduce-scatter in steps of 400 MB 1.107 -> 1.066,
 * deterministic mesh reduce-scatter 0.737 -> 0.698; the double-ring reduce-scatter over 2 x 8 ranks, whose folds
 * alternate with fetches as large as they are, is the one loser (1.480 -> 1.496: its folds gain, its fetches lose more).
 * Results do not depend on it.  Launches that write no more than HCOMM_GFX_ALTERNATE_BYTES (128 MiB) fit the cache
 * with their operands and are left alone.
 */
static int reads_from(const HgLaunch* l, const struct HgWritten* w)
{
    const HgSeg2Table* t = &l->tab.seg2;
    const int reads_dst = l->op != 255u; /* a reduce reads the operand it overwrites */
    for (uint32_t s = 0; s < t->nseg; ++s) {
        const uintptr_t p0 = (uintptr_t)t->src[s], d0 = (uintptr_t)t->dst[s];
        const uint64_t n = t->bytes[s];
        for (uint32_t q = 0; q < w->n; ++q) {
            const uintptr_t w0 = (uintptr_t)w->at[q];
            if (p0 < w0 + w->bytes[q] && w0 < p0 + n) return 1;
            if (reads_dst && d0 < w0 + w->bytes[q] && w0 < d0 + n) return 1;
        }
    }
    return 0;
}

static int direction_of(HgThread* t, const HgLaunch* l)
{
    if (l->bytes <= hg_alternate_bytes()) return 0;
    int backwards;
    if (reads_from(l, &t->written[0])) backwards = !t->written[0].backwards;
    else if (reads_from(l, &t->written[1])) backwards = !t->written[1].backwards;
    else backwards = 0;
    t->written[1] = t->written[0];
    struct HgWritten* w = &t->written[0];
    const HgSeg2Table* tab = &l->tab.seg2;
    w->n = tab->nseg;
    w->backwards = backwards;
    for (uint32_t s = 0; s < tab->nseg; ++s) {
        w->at[s] = tab->dst[s];
        w->bytes[s] = tab->bytes[s];
    }
    return backwards;
}

int hg_submit(HgThread* t, const HgLaunch* l)
{
    const int backwards = (l->kind == HCOMM_GFX_KERNEL_COPY || l->kind == HCOMM_GFX_KERNEL_REDUCE2 || l->kind == HCOMM_GFX_KERNEL_BYTEWISE)
                              ? direction_of(t, l) : 0;
    log_launch(t, l, backwards);
    if (t->recorder) return HCCL_SUCCESS;
    if (t->after) {
        const int rc = hg_thread_settle(t);
        if (rc != HCCL_SUCCESS) return rc;
    }
    t->own_work = 1;
    switch (l->kind) {
        case HCOMM_GFX_KERNEL_COPY:
            return hg_launch_copy(t->stream, &l->tab.seg2, l->blocks, (int)l->streaming, l->lds_bytes, backwards);
        case HCOMM_GFX_KERNEL_REDUCE2:
            return hg_launch_reduce2(t->stream, (int)l->dtype, (int)l->op, &l->tab.seg2, l->blocks, (int)l->streaming,
                                     l->lds_bytes, backwards);
        case HCOMM_GFX_KERNEL_BYTEWISE:
            return hg_launch_bytewise(t->stream, l->op != 255u, (int)l->dtype, (int)l->op, &l->tab.seg2, l->blocks,
                                      (int)l->streaming, l->lds_bytes, backwards);
        case HCOMM_GFX_KERNEL_CHAIN:
        case HCOMM_GFX_KERNEL_TREE:
            return hg_launch_fold(t->stream, (int)l->dtype, (int)l->op, (int)l->acc_is_dst, &l->tab.fold, l->blocks,
                                  l->lds_bytes);
        default: return HCCL_E_INTERNAL;
    }
}

int32_t HcommGfxLaunchLogRead(ThreadHandle thread, HcommGfxLaunchRecord* out, uint32_t cap, uint32_t* n)
{
    HgThread* t = hg_thread_from_handle(thread);
    if (!t || !n) return HCCL_E_PTR;
    *n = t->log_n;
    if (out) {
        const uint32_t m = t->log_n < cap ? t->log_n : cap;
        if (m) memcpy(out, t->log, m * sizeof(*out));
    }
    return HCCL_SUCCESS;
}

int32_t HcommGfxLaunchLogClear(ThreadHandle thread)
{
    HgThread* t = hg_thread_from_handle(thread);
    if (!t) return HCCL_E_PTR;
    t->log_n = 0;
    return HCCL_SUCCESS;
}

/* ---- eager / batch submission of primitive calls -------------------------------------------------------- */

static int emit_to_thread(const HgLaunch* l, void* ctx) { return hg_submit((HgThread*)ctx, l); }

/* 0 when the calling host thread may submit on `t` now: no batch of another host thread holds operations of it */
int hg_thread_free_for_caller(const HgThread* t)
{
    const void* held = __atomic_load_n(&t->batch_owner, __ATOMIC_ACQUIRE);
    return (held && held != (const void*)&g_ctx) ? HCCL_E_UNAVAIL : HCCL_SUCCESS;
}

int hg_caller_is_batching(void) { return g_ctx.batching; }

static int record_or_run(HgThread* t, const HgOp* o)
{
    /* a thread that holds recorded operations of another host thread's batch takes nothing from this one, batching
     * or not: what this call launched would run ahead of what that batch recorded before it */
    if (hg_thread_free_for_caller(t) != HCCL_SUCCESS) return HCCL_E_UNAVAIL;
    if (!g_ctx.batching) return hg_coalesce(o, 1, emit_to_thread, t);
    /* The thread joins this host thread's batch before anything is queued on it, so that a refusal leaves nothing
     * behind for a later, unrelated batch.  The claim is one compare-and-exchange: of two host threads that find the
     * thread free at the same moment one wins and the other is refused. */
    if (__atomic_load_n(&t->batch_owner, __ATOMIC_ACQUIRE) != (const void*)&g_ctx) {
        if (g_ctx.ntouched == HG_TOUCHED_MAX) return HCCL_E_UNAVAIL;
        const void* expected = NULL;
        if (!__atomic_compare_exchange_n(&t->batch_owner, &expected, (const void*)&g_ctx, 0, __ATOMIC_ACQ_REL,
                                         __ATOMIC_ACQUIRE))
            return HCCL_E_UNAVAIL;
        g_ctx.touched[g_ctx.ntouched++] = t;
    }
    if (t->pending_n == t->pending_cap) {
        uint32_t cap = t->pending_cap ? t->pending_cap * 2 : 64;
        HgOp* p = (HgOp*)realloc(t->pending, cap * sizeof(*p));
        if (!p) return HCCL_E_MEMORY; /* the thread stays in the batch (empty, or with what was recorded before) */
        t->pending = p;
        t->pending_cap = cap;
    }
    t->pending[t->pending_n++] = *o;
    return HCCL_SUCCESS;
}

int32_t HcommLocalCopyOnThread(ThreadHandle thread, void* dst, const void* src, uint64_t len)
{
    if (!dst) return HCCL_E_PTR;
    if (!src) return HCCL_E_PTR;
    HgThread* t = hg_thread_from_handle(thread);
    if (!t) return HCCL_E_PTR;
    HgOp o;
    memset(&o, 0, sizeof(o));
    o.is_reduce = 0;
    o.dtype = 255;
    o.op = 255;
    o.dst = dst;
    o.src = src;
    o.bytes = len;
    return record_or_run(t, &o);
}

int32_t HcommLocalReduceOnThread(
    ThreadHandle thread, void* dst, const void* src, uint64_t count, HcommDataType dataType, HcommReduceOp reduceOp)
{
    if (!dst) return HCCL_E_PTR;
    if (!src) return HCCL_E_PTR;
    if (!hg_reduce_supported((int)dataType, (int)reduceOp, allow_prod())) return HCCL_E_PARA;
    HgThread* t = hg_thread_from_handle(thread);
    if (!t) return HCCL_E_PTR;
    HgOp o;
    memset(&o, 0, sizeof(o));
    o.is_reduce = 1;
    o.dtype = (uint8_t)dataType;
    o.op = (uint8_t)reduceOp;
    o.dst = dst;
    o.src = src;
    o.bytes = count * HcommGfxDataTypeSize(dataType); /* cpu_primitives_c_adpt.cc:109 */
    return record_or_run(t, &o);
}

/* ---- inter-rank twins: the same two operations with one operand in a peer's buffer -------------------- */

static int32_t channel_op(ThreadHandle thread, ChannelHandle channel, int is_reduce, void* dst, const void* src,
                          uint64_t n, HcommDataType dataType, HcommReduceOp reduceOp)
{
    if (!dst) return HCCL_E_PTR;
    if (!src) return HCCL_E_PTR;
    if (is_reduce && !hg_reduce_supported((int)dataType, (int)reduceOp, allow_prod())) return HCCL_E_PARA;
    HgThread* t = hg_thread_from_handle(thread);
    if (!t) return HCCL_E_PTR;
    if (!channel) return HCCL_E_PTR;
    HgOp o;
    memset(&o, 0, sizeof(o));
    o.is_reduce = (uint8_t)is_reduce;
    o.dtype = is_reduce ? (uint8_t)dataType : 255;
    o.op = is_reduce ? (uint8_t)reduceOp : 255;
    o.dst = dst;
    o.src = src;
    o.bytes = is_reduce ? n * HcommGfxDataTypeSize(dataType) : n;
    return record_or_run(t, &o);
}

int32_t HcommWriteOnThread(ThreadHandle thread, ChannelHandle channel, void* dst, const void* src, uint64_t len)
{
    return channel_op(thread, channel, 0, dst, src, len, HCOMM_DATA_TYPE_RESERVED, HCOMM_REDUCE_RESERVED);
}

int32_t HcommReadOnThread(ThreadHandle thread, ChannelHandle channel, void* dst, const void* src, uint64_t len)
{
    return channel_op(thread, channel, 0, dst, src, len, HCOMM_DATA_TYPE_RESERVED, HCOMM_REDUCE_RESERVED);
}

int32_t HcommWriteNbiOnThread(ThreadHandle thread, ChannelHandle channel, void* dst, const void* src, uint64_t len)
{
    return channel_op(thread, channel, 0, dst, src, len, HCOMM_DATA_TYPE_RESERVED, HCOMM_REDUCE_RESERVED);
}

int32_t HcommReadNbiOnThread(ThreadHandle thread, ChannelHandle channel, void* dst, const void* src, uint64_t len)
{
    return channel_op(thread, channel, 0, dst, src, len, HCOMM_DATA_TYPE_RESERVED, HCOMM_REDUCE_RESERVED);
}

int32_t HcommWriteReduceOnThread(
    ThreadHandle thread, ChannelHandle channel, void* dst, const void* src, uint64_t count, HcommDataType dataType,
    HcommReduceOp reduceOp)
{
    return channel_op(thread, channel, 1, dst, src, count, dataType, reduceOp);
}

int32_t HcommReadReduceOnThread(
    ThreadHandle thread, ChannelHandle channel, void* dst, const void* src, uint64_t count, HcommDataType dataType,
    HcommReduceOp reduceOp)
{
    return channel_op(thread, channel, 1, dst, src, count, dataType, reduceOp);
}

int32_t HcommBatchTransferOnThread(
    ThreadHandle thread, ChannelHandle channel, const HcommBatchTransferDesc* transferDescs, uint32_t transferDescNum)
{
    HgThread* t = hg_thread_from_handle(thread);
    if (!t) return HCCL_E_PTR;
    if (!channel) return HCCL_E_PTR;
    if (transferDescNum == 0) return HCCL_SUCCESS;
    if (!transferDescs) return HCCL_E_PTR;
    HgOp* ops = (HgOp*)calloc(transferDescNum, sizeof(HgOp));
    if (!ops) return HCCL_E_MEMORY;
    int32_t ret = HCCL_SUCCESS;
    for (uint32_t i = 0; i < transferDescNum && ret == HCCL_SUCCESS; ++i) {
        const HcommBatchTransferDesc* d = &transferDescs[i];
        HgOp* o = &ops[i];
        switch (d->transType) {
            case HCOMM_TRANSFER_TYPE_WRITE:
            case HCOMM_TRANSFER_TYPE_READ:
                o->dtype = 255;
                o->op = 255;
                o->dst = d->transferInfo.write.dst;
                o->src = d->transferInfo.write.src;
                o->bytes = d->transferInfo.write.len;
                break;
            case HCOMM_TRANSFER_TYPE_WRITE_REDUCE:
            case HCOMM_TRANSFER_TYPE_READ_REDUCE:
                if (!hg_reduce_supported((int)d->transferInfo.reduce.dataType, (int)d->transferInfo.reduce.reduceOp,
                                         allow_prod())) {
                    ret = HCCL_E_PARA;
                    break;
                }
                o->is_reduce = 1;
                o->dtype = (uint8_t)d->transferInfo.reduce.dataType;
                o->op = (uint8_t)d->transferInfo.reduce.reduceOp;
                o->dst = d->transferInfo.reduce.dst;
                o->src = d->transferInfo.reduce.src;
                o->bytes = d->transferInfo.reduce.count * HcommGfxDataTypeSize(d->transferInfo.reduce.dataType);
                break;
            case HCOMM_TRANSFER_TYPE_WRITE_WITH_NOTIFY:
            case HCOMM_TRANSFER_TYPE_WRITE_REDUCE_WITH_NOTIFY:
            case HCOMM_TRANSFER_TYPE_NOTIFY_RECORD: ret = HCCL_E_NOT_SUPPORT; break;
            default: ret = HCCL_E_PARA; break;
        }
        if (ret == HCCL_SUCCESS && (!o->dst || !o->src)) ret = HCCL_E_PTR;
    }
    if (ret == HCCL_SUCCESS) ret = hg_thread_free_for_caller(t);
    if (ret == HCCL_SUCCESS) {
        if (g_ctx.batching) {
            for (uint32_t i = 0; i < transferDescNum && ret == HCCL_SUCCESS; ++i) ret = record_or_run(t, &ops[i]);
        } else {
            ret = hg_coalesce(ops, transferDescNum, emit_to_thread, t);
        }
    }
    free(ops);
    return ret;
}

int32_t HcommBatchModeStart(const char* batchTag)
{
    (void)batchTag;
    if (g_ctx.batching) return HCCL_E_PARA;
    g_ctx.batching = 1;
    g_ctx.ntouched = 0;
    return HCCL_SUCCESS;
}

/*
 * A batch whose threads order one another by notifies - the reference submits such a batch as one task graph over all
 * its threads (CommTaskLaunch(threads, threadNum), launch_context.cc:16-44) - is resolved on the host into one list.
 * Every thread's queue is walked up to its next copy or reduce: records on the way are noted, a wait passes when a
 * record for its slot has been noted (or was issued before the batch), otherwise the thread sits there.  Of the
 * copies and reduces now at the head of their threads - none of them ordered after another by any record - those
 * that can share a launch with the head of the thread that has had the fewest so far are appended to the list, their
 * threads move on, and so forth.  In a schedule whose ranks post to and wait for one another between steps, one
 * such round is one step.  The list respects every thread's own order and every record -> wait edge, and the
 * coalescer keeps apart whatever touches the same memory; it is issued on the stream of the first thread of the
 * batch, the other threads' streams are ordered after it, and it after them where they had work of their own.  All
 * ranks of a step thus share one launch although each was given to a thread of its own.
 * When no thread can move and calls are left, a wait is there that nothing in the batch and no earlier record
 * satisfies, and this host thread can never satisfy it: HCCL_E_TIMEOUT, and nothing of the batch is submitted.
 * Records that no wait of the batch consumes stay pending for a later wait, marking the end of the batch.
 */
typedef struct {
    HgThread* t;
    uint32_t idx;
} HgSlot;

static int32_t batch_end_ordered(HgThread** th, uint32_t nt)
{
    int32_t ret = HCCL_SUCCESS;
    uint64_t total = 0;
    for (uint32_t i = 0; i < nt; ++i) {
        th[i]->batch_cursor = 0;
        total += th[i]->pending_n;
    }
    const uint64_t cap = total ? total : 1;
    HgOp* sorted = (HgOp*)malloc(cap * sizeof(HgOp));
    uint32_t* round_of = (uint32_t*)malloc(cap * sizeof(uint32_t)); /* the round each of them was taken in: a schedule's step */
    uint32_t rounds = 0;
    HgSlot* outside = (HgSlot*)malloc(cap * sizeof(HgSlot)); /* records to threads outside the batch */
    HgSlot* earlier = (HgSlot*)malloc(cap * sizeof(HgSlot)); /* records issued before the batch that its waits consume */
    uint32_t** count = (uint32_t**)calloc(nt, sizeof(uint32_t*)); /* per thread and slot: unconsumed records of the batch */
    uint32_t had[HG_TOUCHED_MAX];                                 /* copies and reduces taken from each thread so far */
    HgThread* main_t = th[0];
    uint64_t n = 0, nearlier = 0, noutside = 0, done = 0;
    if (!sorted || !round_of || !outside || !earlier || !count) ret = HCCL_E_MEMORY;
    for (uint32_t i = 0; i < nt && ret == HCCL_SUCCESS; ++i) {
        had[i] = 0;
        count[i] = (uint32_t*)calloc(th[i]->notify_num ? th[i]->notify_num : 1, sizeof(uint32_t));
        if (!count[i]) ret = HCCL_E_MEMORY;
    }
    while (ret == HCCL_SUCCESS && done < total) {
        /* every thread up to its next copy or reduce, until no record makes another wait pass */
        uint64_t moved;
        do {
            moved = 0;
            for (uint32_t i = 0; i < nt; ++i) {
                HgThread* t = th[i];
                while (t->batch_cursor < t->pending_n && t->pending[t->batch_cursor].sync != 0) {
                    const HgOp* o = &t->pending[t->batch_cursor];
                    if (o->sync == HG_SYNC_RECORD) {
                        HgThread* d = (HgThread*)o->dst;
                        uint32_t j = 0;
                        while (j < nt && th[j] != d) ++j;
                        if (j < nt) ++count[j][o->idx];
                        else outside[noutside++] = (HgSlot){d, o->idx};
                    } else if (count[i][o->idx] > 0) {
                        --count[i][o->idx];
                    } else {
                        /* a record issued before the batch began */
                        uint64_t pending = __atomic_load_n(&t->notify_pending[o->idx], __ATOMIC_ACQUIRE);
                        int took = 0;
                        while (pending != 0 && !took)
                            took = __atomic_compare_exchange_n(&t->notify_pending[o->idx], &pending, pending - 1, 0,
                                                               __ATOMIC_ACQ_REL, __ATOMIC_ACQUIRE);
                        if (!took) break; /* its record is further down another thread's queue, or nowhere */
                        earlier[nearlier++] = (HgSlot){t, o->idx};
                    }
                    ++t->batch_cursor;
                    ++moved;
                }
            }
            done += moved;
        } while (moved != 0);
        /* the thread that is furthest behind names the launch of this round */
        uint32_t lead = nt;
        for (uint32_t i = 0; i < nt; ++i) {
            const HgThread* t = th[i];
            if (t->batch_cursor < t->pending_n && t->pending[t->batch_cursor].sync == 0 && (lead == nt || had[i] < had[lead])) lead = i;
        }
        if (lead == nt) {
            if (done < total) ret = HCCL_E_TIMEOUT; /* every thread with calls left sits at a wait */
            break;
        }
        const uint32_t key = hg_op_launch_key(&th[lead]->pending[th[lead]->batch_cursor]);
        for (uint32_t i = 0; i < nt; ++i) {
            HgThread* t = th[i];
            if (t->batch_cursor < t->pending_n && t->pending[t->batch_cursor].sync == 0 &&
                hg_op_launch_key(&t->pending[t->batch_cursor]) == key) {
                round_of[n] = rounds;
                sorted[n++] = t->pending[t->batch_cursor++];
                ++had[i];
                ++done;
            }
        }
        ++rounds;
    }
    if (ret != HCCL_SUCCESS) {
        /* nothing is submitted; the earlier records that waits of this batch took are handed back */
        for (uint64_t k = 0; k < nearlier; ++k)
            __atomic_add_fetch(&earlier[k].t->notify_pending[earlier[k].idx], 1, __ATOMIC_RELEASE);
    } else {
        if (!main_t->recorder) {
            /* the batch's stream after what the other threads had queued on their own, and after the earlier records */
            ret = hg_thread_settle(main_t);
            for (uint32_t i = 1; i < nt && ret == HCCL_SUCCESS; ++i) {
                HgThread* t = th[i];
                if (t->recorder) continue;
                if (t->after != main_t) ret = hg_thread_settle(t); /* behind another batch's first thread: its own stream says so */
                if (ret != HCCL_SUCCESS || !(t->own_work || !t->owns_stream)) continue;
                if (!t->join_ev) ret = hg_rt_event_create(&t->join_ev);
                if (ret == HCCL_SUCCESS) ret = hg_rt_event_record(t->join_ev, t->stream);
                if (ret == HCCL_SUCCESS) ret = hg_rt_stream_wait_event(main_t->stream, t->join_ev);
                t->own_work = 0;
            }
            for (uint64_t k = 0; k < nearlier && ret == HCCL_SUCCESS; ++k)
                if (!earlier[k].t->recorder) ret = hg_rt_stream_wait_event(main_t->stream, earlier[k].t->notifies[earlier[k].idx]);
        }
        /* rounds are steps: a collective handed over whole gets the lowering a step-wise plan of it gets, steps larger
         * than the memory-side cache serves run piece by piece */
        if (ret == HCCL_SUCCESS) ret = hg_cut_into_pieces(&sorted, &round_of, &n);
        if (ret == HCCL_SUCCESS) ret = hg_coalesce(sorted, n, emit_to_thread, main_t);
        /* what the batch leaves behind: records nobody in it waited for, and the other threads behind its end */
        for (uint32_t i = 0; i < nt && ret == HCCL_SUCCESS; ++i)
            for (uint32_t k = 0; k < th[i]->notify_num && ret == HCCL_SUCCESS; ++k)
                for (; count[i][k] > 0 && ret == HCCL_SUCCESS; --count[i][k]) {
                    if (!(main_t->recorder || th[i]->recorder)) ret = hg_rt_event_record(th[i]->notifies[k], main_t->stream);
                    __atomic_add_fetch(&th[i]->notify_pending[k], 1, __ATOMIC_RELEASE);
                }
        for (uint64_t k = 0; k < noutside && ret == HCCL_SUCCESS; ++k) {
            if (!hg_thread_from_handle((ThreadHandle)(uintptr_t)outside[k].t)) continue; /* freed since the call was recorded */
            if (!(main_t->recorder || outside[k].t->recorder)) ret = hg_rt_event_record(outside[k].t->notifies[outside[k].idx], main_t->stream);
            __atomic_add_fetch(&outside[k].t->notify_pending[outside[k].idx], 1, __ATOMIC_RELEASE);
        }
        if (!main_t->recorder && nt > 1 && ret == HCCL_SUCCESS) {
            /* the other threads' own streams go behind the end of the batch when they are next used (hg_thread_settle) */
            if (!main_t->join_ev) ret = hg_rt_event_create(&main_t->join_ev);
            if (ret == HCCL_SUCCESS) ret = hg_rt_event_record(main_t->join_ev, main_t->stream);
            main_t->led_batch = 1;
            for (uint32_t i = 1; i < nt && ret == HCCL_SUCCESS; ++i) {
                if (th[i]->recorder) continue;
                /* a stream of the caller's may be given work the library never sees: it goes behind the batch now */
                if (th[i]->owns_stream) th[i]->after = main_t;
                else ret = hg_rt_stream_wait_event(th[i]->stream, main_t->join_ev);
            }
        }
    }
    for (uint32_t i = 0; i < nt; ++i) {
        if (count) free(count[i]);
    }
    free(count);
    free(outside);
    free(earlier);
    free(sorted);
    free(round_of);
    return ret;
}

/*
 * A thread's queue of a batch without notifies.  Normally it goes to the coalescer as it is.  When it holds more than
 * one step's worth of large operations - a whole collective recorded in one batch - its steps are told apart the way
 * the coalescer would (a call of another kind, or one that touches what the step so far touches, begins a step) and
 * go through the lowering of a step-wise plan: steps larger than the memory-side cache serves run piece by piece.
 */
static int touches(const HgOp* a, const HgOp* b)
{
    const uintptr_t ad = (uintptr_t)a->dst, as = (uintptr_t)a->src, bd = (uintptr_t)b->dst, bs = (uintptr_t)b->src;
    return (ad < bd + b->bytes && bd < ad + a->bytes) || (ad < bs + b->bytes && bs < ad + a->bytes) ||
           (as < bd + b->bytes && bd < as + a->bytes);
}

static int32_t end_plain(HgThread* t)
{
    const uint64_t aim = hg_piece_bytes();
    uint64_t bytes = 0;
    for (uint32_t k = 0; k < t->pending_n; ++k) bytes += t->pending[k].bytes;
    if (aim == 0 || t->pending_n < 2u || bytes <= aim * 5u) /* fewer than two steps worth cutting */
        return hg_coalesce(t->pending, t->pending_n, emit_to_thread, t);
    uint64_t n = t->pending_n;
    HgOp* ops = (HgOp*)malloc(n * sizeof(HgOp));
    uint32_t* steps = (uint32_t*)malloc(n * sizeof(uint32_t));
    if (!ops || !steps) {
        free(ops);
        free(steps);
        return HCCL_E_MEMORY;
    }
    memcpy(ops, t->pending, n * sizeof(HgOp));
    uint32_t step = 0;
    uint64_t begin = 0;
    for (uint64_t k = 0; k < n; ++k) {
        /* The steps only say how much a step writes, i.e. whether cutting pays: the piece-major order is right
         * whatever they are (two pieces meet only when they are the same piece of the same range, and those keep
         * their order).  So a very long step is compared with its latest part only, which bounds the work. */
        int fresh = k != 0 && hg_op_launch_key(&ops[k]) != hg_op_launch_key(&ops[begin]);
        for (uint64_t q = k - begin > 128u ? k - 128u : begin; q < k && !fresh; ++q) fresh = touches(&ops[k], &ops[q]);
        if (fresh) {
            ++step;
            begin = k;
        }
        steps[k] = step;
    }
    int32_t ret = hg_cut_into_pieces(&ops, &steps, &n);
    if (ret == HCCL_SUCCESS) ret = hg_coalesce(ops, n, emit_to_thread, t);
    free(ops);
    free(steps);
    return ret;
}

int32_t HcommBatchModeEnd(const char* batchTag)
{
    (void)batchTag;
    if (!g_ctx.batching) return HCCL_E_PARA;
    g_ctx.batching = 0;
    int32_t ret = HCCL_SUCCESS;
    /* the threads of the batch that are still alive, and whether any of them recorded a notify call */
    HgThread* th[HG_TOUCHED_MAX];
    uint32_t nt = 0;
    int ordered = 0;
    for (uint32_t i = 0; i < g_ctx.ntouched; ++i) {
        HgThread* t = g_ctx.touched[i];
        if (!t) continue; /* freed inside the batch */
        th[nt++] = t;
        for (uint32_t k = 0; k < t->pending_n && !ordered; ++k) ordered = t->pending[k].sync != 0;
    }
    if (ordered) {
        ret = batch_end_ordered(th, nt);
    } else {
        for (uint32_t i = 0; i < nt; ++i)
            if (ret == HCCL_SUCCESS) ret = end_plain(th[i]);
    }
    for (uint32_t i = 0; i < nt; ++i) {
        th[i]->pending_n = 0;
        __atomic_store_n(&th[i]->batch_owner, NULL, __ATOMIC_RELEASE);
    }
    g_ctx.ntouched = 0;
    return ret;
}

/* ---- k-way fused reduce -------------------------------------------------------------------------- */

int32_t HcommGfxReduceKOnThread(
    ThreadHandle thread, void* dst, const void* const* srcs, uint32_t k, uint64_t count, HcommDataType dataType,
    HcommReduceOp reduceOp)
{
    if (!dst) return HCCL_E_PTR;
    if (!srcs) return HCCL_E_PTR;
    if (k == 0 || k > HCOMM_GFX_MAX_RANKS) return HCCL_E_PARA;
    for (uint32_t j = 0; j < k; ++j)
        if (!srcs[j]) return HCCL_E_PTR;
    if (!hg_reduce_supported((int)dataType, (int)reduceOp, 1)) return HCCL_E_PARA;
    HgThread* t = hg_thread_from_handle(thread);
    if (!t) return HCCL_E_PTR;
    if (g_ctx.batching) return HCCL_E_NOT_SUPPORT;
    if (hg_thread_free_for_caller(t) != HCCL_SUCCESS) return HCCL_E_UNAVAIL;
    const uint64_t bytes = count * HcommGfxDataTypeSize(dataType);
    if (bytes == 0) return HCCL_SUCCESS;
    uintptr_t align = (uintptr_t)dst;
    for (uint32_t j = 0; j < k; ++j) align |= (uintptr_t)srcs[j];
    if (align & (HG_VEC_BYTES - 1)) {
        /* unaligned operands: the same chain as k-1 two-input launches of the kernel for unaligned operands */
        HgOp o;
        memset(&o, 0, sizeof(o));
        o.dst = dst;
        o.src = srcs[0];
        o.bytes = bytes;
        o.dtype = 255;
        o.op = 255;
        int32_t ret = hg_coalesce(&o, 1, emit_to_thread, t);
        for (uint32_t j = 1; j < k && ret == HCCL_SUCCESS; ++j) {
            o.is_reduce = 1;
            o.dtype = (uint8_t)dataType;
            o.op = (uint8_t)reduceOp;
            o.src = srcs[j];
            ret = hg_coalesce(&o, 1, emit_to_thread, t);
        }
        return ret;
    }
    HgLaunch* l = (HgLaunch*)calloc(1, sizeof(HgLaunch));
    if (!l) return HCCL_E_MEMORY;
    l->kind = HCOMM_GFX_KERNEL_CHAIN;
    l->dtype = (uint32_t)dataType;
    l->op = (uint32_t)reduceOp;
    l->acc_is_dst = 1;
    HgFoldTable* f = &l->tab.fold;
    for (uint32_t j = 0; j < k; ++j) f->in[j] = srcs[j];
    f->out[0] = dst;
    f->nseg = 1;
    f->k = k;
    f->nranks = k;
    f->stride = 1;
    f->out_mode = 1;
    f->bytes[0] = bytes;
    hg_finish_fold(l);
    int32_t ret = hg_submit(t, l);
    free(l);
    return ret;
}

/* ---- notifies ------------------------------------------------------------------------------------ */

int32_t HcommThreadNotifyRecordOnThread(ThreadHandle thread, ThreadHandle dstThread, uint32_t dstNotifyIdx)
{
    HgThread* t = hg_thread_from_handle(thread);
    if (!t) return HCCL_E_PTR;
    HgThread* d = hg_thread_from_handle(dstThread);
    if (!d) return HCCL_E_PTR;
    if (dstNotifyIdx >= d->notify_num) return HCCL_E_PARA;
    if (g_ctx.batching) { /* a step of the thread's sequence like any other: resolved by HcommBatchModeEnd */
        HgOp o;
        memset(&o, 0, sizeof(o));
        o.sync = HG_SYNC_RECORD;
        o.idx = dstNotifyIdx;
        o.dst = d;
        return record_or_run(t, &o);
    }
    if (hg_thread_free_for_caller(t) != HCCL_SUCCESS) return HCCL_E_UNAVAIL;
    if (!(t->recorder || d->recorder)) {
        int rc = hg_thread_settle(t);
        if (rc == HCCL_SUCCESS) rc = hg_rt_event_record(d->notifies[dstNotifyIdx], t->stream);
        if (rc != HCCL_SUCCESS) return rc;
    }
    __atomic_add_fetch(&d->notify_pending[dstNotifyIdx], 1, __ATOMIC_RELEASE);
    return HCCL_SUCCESS;
}

/* How long a wait whose record has not been issued yet may sit on the host, milliseconds (HCOMM_GFX_NOTIFY_HOST_WAIT_MS;
 * never longer than the call's own timeOut, which is in seconds). */
static uint64_t notify_host_wait_ms(void)
{
    static uint64_t cached = 0; /* value + 1 */
    uint64_t v = __atomic_load_n(&cached, __ATOMIC_RELAXED);
    if (v == 0) {
        const char* e = getenv("HCOMM_GFX_NOTIFY_HOST_WAIT_MS");
        v = (e && *e ? strtoull(e, NULL, 10) : 100u) + 1u;
        __atomic_store_n(&cached, v, __ATOMIC_RELAXED);
    }
    return v - 1u;
}

int32_t HcommThreadNotifyWaitOnThread(ThreadHandle thread, uint32_t notifyIdx, uint32_t timeOut)
{
    HgThread* t = hg_thread_from_handle(thread);
    if (!t) return HCCL_E_PTR;
    if (notifyIdx >= t->notify_num) return HCCL_E_PARA;
    if (g_ctx.batching) {
        HgOp o;
        memset(&o, 0, sizeof(o));
        o.sync = HG_SYNC_WAIT;
        o.idx = notifyIdx;
        return record_or_run(t, &o);
    }
    if (hg_thread_free_for_caller(t) != HCCL_SUCCESS) return HCCL_E_UNAVAIL;
    /* A wait on a stream can only follow a record that has been issued.  The reference queues the wait and lets the
     * device sit until the record arrives or timeOut runs out (include/hcomm_primitives.h:181-191); here the wait
     * sits on the HOST until another host thread has issued the record - for at most min(timeOut seconds, the bound
     * above), so that callers who drive each thread from a host thread of its own need not order the two calls -
     * and then returns HCCL_E_TIMEOUT with nothing queued. */
    uint64_t budget_ms = (uint64_t)timeOut * 1000u;
    if (budget_ms > notify_host_wait_ms()) budget_ms = notify_host_wait_ms();
    struct timespec t0;
    clock_gettime(CLOCK_MONOTONIC, &t0);
    for (;;) {
        uint64_t pending = __atomic_load_n(&t->notify_pending[notifyIdx], __ATOMIC_ACQUIRE);
        while (pending != 0) {
            if (__atomic_compare_exchange_n(&t->notify_pending[notifyIdx], &pending, pending - 1, 0, __ATOMIC_ACQ_REL,
                                            __ATOMIC_ACQUIRE)) {
                if (t->recorder) return HCCL_SUCCESS;
                t->own_work = 1;
                return hg_rt_stream_wait_event(t->stream, t->notifies[notifyIdx]);
            }
        }
        struct timespec now;
        clock_gettime(CLOCK_MONOTONIC, &now);
        const uint64_t waited_ms = (uint64_t)(now.tv_sec - t0.tv_sec) * 1000u + (uint64_t)((now.tv_nsec - t0.tv_nsec) / 1000000);
        if (waited_ms >= budget_ms) return HCCL_E_TIMEOUT;
        sched_yield();
    }
}

/* default notify-wait time-out of the calling host thread, seconds: NOTIFY_WAIT_TIMEOUT_DEFAULT,
 * src/base_comm/primitives/launch_context.h:24 (kept per host thread there too, cpu_primitives_c_adpt.cc:26) */
static _Thread_local uint32_t g_notify_timeout = 1836u;

int32_t HcommSetNotifyWaitTimeOut(float timeOut)
{
    if (timeOut != timeOut || timeOut < 0.0f || timeOut > (float)UINT32_MAX) return HCCL_E_PARA;
    g_notify_timeout = (uint32_t)timeOut;
    return HCCL_SUCCESS;
}

int32_t HcommThreadNotifyWaitOnThreadWithDefaultTimeout(ThreadHandle thread, uint32_t notifyIdx)
{
    return HcommThreadNotifyWaitOnThread(thread, notifyIdx, g_notify_timeout);
}

int32_t HcommThreadResAcquireTimeOut(float timeOut)
{
    (void)timeOut;
    return HCCL_E_NOT_SUPPORT;
}

/* ---- ordering points ------------------------------------------------------------------------------ */

int32_t HcommFenceOnThread(ThreadHandle thread)
{
    return hg_thread_from_handle(thread) ? HCCL_SUCCESS : HCCL_E_PTR;
}

int32_t HcommChannelFenceOnThread(ThreadHandle thread, ChannelHandle channel)
{
    if (!channel) return HCCL_E_PTR;
    return hg_thread_from_handle(thread) ? HCCL_SUCCESS : HCCL_E_PTR;
}

int32_t HcommChannelDrainOnThread(ThreadHandle thread, ChannelHandle channel)
{
    if (!hg_thread_from_handle(thread)) return HCCL_E_PTR;
    return channel ? HCCL_SUCCESS : HCCL_E_PTR;
}

/* ---- memory -------------------------------------------------------------------------------------- */

HcommResult HcommMemAlloc(void** ptr, size_t size)
{
    if (!ptr) return HCCL_E_PTR;
    if (size == 0) return HCCL_E_PARA;
    *ptr = NULL;
    return hg_rt_malloc(ptr, size);
}

HcommResult HcommMemFree(void* ptr)
{
    if (!ptr) return HCCL_E_PTR;
    return hg_rt_free(ptr);
}
