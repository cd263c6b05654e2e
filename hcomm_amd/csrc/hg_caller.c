/*
 * hg_caller.c - a stand-in for the CALLER of the primitives: what the external HCCL operator library does with them.
 *
 * Not part of libhcomm_gfx.so.  It binds the library the way the operator library binds libhcomm - dlopen + dlsym of
 * the symbol names of include/hcomm_primitives.h (docs/zh/architecture/architecture-brief.md:282) - and uses nothing
 * but those symbols: HcommBatchModeStart / End (:496,504), HcommLocalCopyOnThread (:152), HcommLocalReduceOnThread
 * (:164-165), HcommThreadNotifyRecordOnThread / WaitOnThread (:181,191).  Given a schedule as a list of two-input
 * operations (the records HcommGfxScheduleEmit writes; a template of the reference produces the same calls from its
 * loops) it replays it
 *   - batched: one BatchModeStart / End pair per schedule step on ONE thread, every rank's operation of the step
 *     between them - the task-batching path of the host adapter (cpu_primitives_c_adpt.cc:58-130 record into the
 *     launch context while batching, launch_context.cc:139-174 submits at End);
 *   - on one thread per rank, eagerly: rank r's operations go to thread r as they come, and between steps each thread
 *     posts to and waits for exactly the peers it exchanges data with - the data signal from the rank it reads and
 *     the acknowledgement from the rank that read it (the TxAck / RxAck / DataSignal handshake of the templates,
 *     reduce_scatter_ring.cc:211-217,254-272), with a fork from and a join to thread 0 around the whole schedule (the
 *     main / sub stream pattern of the executors).
 *   - on one thread per rank with one HOST thread per rank as well: the same posts and waits, every rank's calls
 *     issued by a host thread of its own, as the ranks of the reference are processes of their own.  A wait may then
 *     reach the library before the record it is for; the library's wait sits on the host until the record is issued.
 * The benchmark times all three against the library's prepared plans, and the GPU tests compare what they leave in the
 * rank buffers with the CPU oracle.
 */
#define _POSIX_C_SOURCE 200809L
#include <dlfcn.h>
#include <pthread.h>
#include <sched.h>
#include <stdint.h>
#include <string.h>
#include <time.h>

#include "hcomm_gfx.h" /* types only: HcommGfxSchedOp, ThreadHandle, the enums */

#define CALLER_MAX_RANKS 32u

typedef int32_t (*BatchFn)(const char*);
typedef int32_t (*CopyFn)(ThreadHandle, void*, const void*, uint64_t);
typedef int32_t (*ReduceFn)(ThreadHandle, void*, const void*, uint64_t, HcommDataType, HcommReduceOp);
typedef int32_t (*RecordFn)(ThreadHandle, ThreadHandle, uint32_t);
typedef int32_t (*WaitFn)(ThreadHandle, uint32_t, uint32_t);

static struct {
    void* lib;
    BatchFn start, end;
    CopyFn copy;
    ReduceFn reduce;
    RecordFn record;
    WaitFn wait;
} g;

typedef struct {
    uint32_t batches;   /* BatchModeStart / End pairs (batched) or schedule steps (threads) */
    uint32_t calls;     /* HcommLocalCopyOnThread + HcommLocalReduceOnThread calls */
    uint32_t notifies;  /* record + wait pairs */
    uint32_t reserved;
    double host_us;     /* host time of the whole replay call */
    double host_us_end; /* of which inside HcommBatchModeEnd (coalescing and launching) */
    double host_us_end_max;
    double host_us_notify; /* of which inside the notify calls */
} HgCallerStats;

static double now_us(void)
{
    struct timespec t;
    clock_gettime(CLOCK_MONOTONIC, &t);
    return (double)t.tv_sec * 1e6 + (double)t.tv_nsec * 1e-3;
}

/* 0, or -1 when the library or one of the reference's symbols is missing */
int hg_caller_bind(const char* libpath)
{
    if (g.lib) return 0;
    void* lib = dlopen(libpath, RTLD_NOW | RTLD_GLOBAL);
    if (!lib) return -1;
    g.start = (BatchFn)dlsym(lib, "HcommBatchModeStart");
    g.end = (BatchFn)dlsym(lib, "HcommBatchModeEnd");
    g.copy = (CopyFn)dlsym(lib, "HcommLocalCopyOnThread");
    g.reduce = (ReduceFn)dlsym(lib, "HcommLocalReduceOnThread");
    g.record = (RecordFn)dlsym(lib, "HcommThreadNotifyRecordOnThread");
    g.wait = (WaitFn)dlsym(lib, "HcommThreadNotifyWaitOnThread");
    if (!g.start || !g.end || !g.copy || !g.reduce || !g.record || !g.wait) return -1;
    g.lib = lib;
    return 0;
}

static uint32_t unit_of(int dtype)
{
    /* SIZE_TABLE, pkg_inc/legacy/hccl/dtype_common.h:18-36 */
    switch (dtype) {
        case HCOMM_DATA_TYPE_INT8: return 1;
        case HCOMM_DATA_TYPE_INT32:
        case HCOMM_DATA_TYPE_FP32: return 4;
        default: return 2;
    }
}

/* one operation of the list as the primitive call it stands for, on `thread` */
static int32_t issue(ThreadHandle thread, const HcommGfxSchedOp* o, void* const* const* bufs, int dtype, int op, uint32_t unit)
{
    char* dst = (char*)bufs[o->dstBuf][o->rank] + o->dstOff;
    const char* src = (const char*)bufs[o->srcBuf][o->srcRank] + o->srcOff;
    if (o->kind == 0) return g.copy(thread, dst, src, o->bytes);
    return g.reduce(thread, dst, src, o->bytes / unit, (HcommDataType)dtype, (HcommReduceOp)op);
}

/*
 * ops: n records ordered by step; bufs[role][rank] = base address of that rank's buffer of that role (roles a list
 * does not use may be NULL).  Returns the first HcclResult that is not success.
 */
int32_t hg_caller_replay_batched(ThreadHandle thread, const HcommGfxSchedOp* ops, uint64_t n, void* const* const* bufs,
                                 int dtype, int op, HgCallerStats* st)
{
    if (!g.lib || !ops || !bufs || !st) return HCCL_E_PTR;
    memset(st, 0, sizeof(*st));
    const uint32_t unit = unit_of(dtype);
    const double t0 = now_us();
    int32_t rc = HCCL_SUCCESS;
    uint64_t i = 0;
    while (i < n && rc == HCCL_SUCCESS) {
        const uint32_t step = ops[i].step;
        rc = g.start("step");
        for (; i < n && ops[i].step == step && rc == HCCL_SUCCESS; ++i) {
            rc = issue(thread, &ops[i], bufs, dtype, op, unit);
            ++st->calls;
        }
        const double e0 = now_us();
        const int32_t rc_end = g.end("step"); /* always closes the batch, also after a refused call */
        const double e = now_us() - e0;
        st->host_us_end += e;
        if (e > st->host_us_end_max) st->host_us_end_max = e;
        if (rc == HCCL_SUCCESS) rc = rc_end;
        ++st->batches;
    }
    st->host_us = now_us() - t0;
    return rc;
}

/* The whole list between ONE HcommBatchModeStart / End pair on one thread: the collective handed over in one piece. */
int32_t hg_caller_replay_one_batch(ThreadHandle thread, const HcommGfxSchedOp* ops, uint64_t n, void* const* const* bufs,
                                   int dtype, int op, HgCallerStats* st)
{
    if (!g.lib || !ops || !bufs || !st) return HCCL_E_PTR;
    memset(st, 0, sizeof(*st));
    const uint32_t unit = unit_of(dtype);
    const double t0 = now_us();
    int32_t rc = g.start("collective");
    if (rc != HCCL_SUCCESS) return rc;
    for (uint64_t i = 0; i < n && rc == HCCL_SUCCESS; ++i) {
        rc = issue(thread, &ops[i], bufs, dtype, op, unit);
        ++st->calls;
    }
    const double e0 = now_us();
    const int32_t rc_end = g.end("collective");
    st->host_us_end = st->host_us_end_max = now_us() - e0;
    st->batches = 1;
    st->host_us = now_us() - t0;
    return rc != HCCL_SUCCESS ? rc : rc_end;
}

static int32_t post_and_wait(const ThreadHandle* threads, uint32_t from, uint32_t to, uint32_t timeout, HgCallerStats* st)
{
    /* thread `to` keeps one notify slot per peer: slot `from` */
    int32_t rc = g.record(threads[from], threads[to], from);
    if (rc == HCCL_SUCCESS) rc = g.wait(threads[to], from, timeout);
    ++st->notifies;
    return rc;
}

/*
 * The same list with rank r's operations on threads[r] (each allocated with at least nRanks notify slots), nothing
 * batched.  Before the operations of a step are issued, thread r waits for thread q when
 *   - it is about to read rank q's buffers and q has written since r last waited for it (only q's thread writes
 *     rank q's buffers: the executing rank owns dst), or
 *   - q has read rank r's buffers since then (r is about to overwrite what q may still be reading).
 * Work timed on threads[0]'s stream brackets everything: the other threads wait for it first and it waits for them
 * last.
 */
static int32_t replay_threads(const ThreadHandle* threads, uint32_t nRanks, const HcommGfxSchedOp* ops, uint64_t n,
                              void* const* const* bufs, int dtype, int op, uint32_t timeout, HgCallerStats* st);

int32_t hg_caller_replay_threads(const ThreadHandle* threads, uint32_t nRanks, const HcommGfxSchedOp* ops, uint64_t n,
                                 void* const* const* bufs, int dtype, int op, uint32_t timeout, HgCallerStats* st)
{
    if (!g.lib || !threads || !ops || !bufs || !st) return HCCL_E_PTR;
    if (nRanks == 0 || nRanks > CALLER_MAX_RANKS) return HCCL_E_PARA;
    return replay_threads(threads, nRanks, ops, n, bufs, dtype, op, timeout, st);
}

/*
 * The same calls between ONE HcommBatchModeStart / End pair: the whole collective - every rank's operations on its
 * own thread, every post and wait - is handed over as one batch, the way the reference hands a task graph over all
 * its threads to CommTaskLaunch at the end of a batch (launch_context.cc:16-44).
 */
int32_t hg_caller_replay_threads_batched(const ThreadHandle* threads, uint32_t nRanks, const HcommGfxSchedOp* ops, uint64_t n,
                                         void* const* const* bufs, int dtype, int op, uint32_t timeout, HgCallerStats* st)
{
    if (!g.lib || !threads || !ops || !bufs || !st) return HCCL_E_PTR;
    if (nRanks == 0 || nRanks > CALLER_MAX_RANKS) return HCCL_E_PARA;
    const double t0 = now_us();
    int32_t rc = g.start("collective");
    if (rc != HCCL_SUCCESS) return rc;
    rc = replay_threads(threads, nRanks, ops, n, bufs, dtype, op, timeout, st);
    const double e0 = now_us();
    const int32_t rc_end = g.end("collective");
    st->host_us_end = st->host_us_end_max = now_us() - e0;
    st->host_us = now_us() - t0;
    return rc != HCCL_SUCCESS ? rc : rc_end;
}

static int32_t replay_threads(const ThreadHandle* threads, uint32_t nRanks, const HcommGfxSchedOp* ops, uint64_t n,
                              void* const* const* bufs, int dtype, int op, uint32_t timeout, HgCallerStats* st)
{
    memset(st, 0, sizeof(*st));
    const uint32_t unit = unit_of(dtype);
    /* in units of "steps issued so far" (1-based); 0 = never */
    static _Thread_local uint32_t last_op[CALLER_MAX_RANKS];                      /* q's latest operation */
    static _Thread_local uint32_t last_read[CALLER_MAX_RANKS][CALLER_MAX_RANKS];  /* q's latest read of rank r's buffers */
    static _Thread_local uint32_t synced[CALLER_MAX_RANKS][CALLER_MAX_RANKS];     /* what of q thread r has waited for */
    memset(last_op, 0, sizeof(last_op));
    memset(last_read, 0, sizeof(last_read));
    memset(synced, 0, sizeof(synced));
    const double t0 = now_us();
    int32_t rc = HCCL_SUCCESS;
    double tn = now_us();
    for (uint32_t r = 1; r < nRanks && rc == HCCL_SUCCESS; ++r) rc = post_and_wait(threads, 0, r, timeout, st);
    st->host_us_notify += now_us() - tn;
    uint64_t i = 0;
    uint32_t tick = 0;
    while (i < n && rc == HCCL_SUCCESS) {
        const uint32_t step = ops[i].step;
        uint64_t j = i;
        while (j < n && ops[j].step == step) ++j;
        ++tick;
        tn = now_us();
        for (uint64_t k = i; k < j && rc == HCCL_SUCCESS; ++k) {
            const uint32_t r = ops[k].rank, q0 = ops[k].srcRank;
            if (r >= nRanks || q0 >= nRanks) return HCCL_E_PARA;
            for (uint32_t q = 0; q < nRanks && rc == HCCL_SUCCESS; ++q) {
                if (q == r) continue;
                const int raw = (q == q0) && last_op[q] > synced[q][r];
                const int war = last_read[q][r] > synced[q][r];
                if (raw || war) {
                    rc = post_and_wait(threads, q, r, timeout, st);
                    synced[q][r] = tick - 1; /* everything q was given in earlier steps */
                }
            }
        }
        st->host_us_notify += now_us() - tn;
        for (uint64_t k = i; k < j && rc == HCCL_SUCCESS; ++k) {
            rc = issue(threads[ops[k].rank], &ops[k], bufs, dtype, op, unit);
            ++st->calls;
            last_op[ops[k].rank] = tick;
            if (ops[k].srcRank != ops[k].rank) last_read[ops[k].rank][ops[k].srcRank] = tick;
        }
        ++st->batches;
        i = j;
    }
    tn = now_us();
    for (uint32_t r = 1; r < nRanks && rc == HCCL_SUCCESS; ++r) rc = post_and_wait(threads, r, 0, timeout, st);
    st->host_us_notify += now_us() - tn;
    st->host_us = now_us() - t0;
    return rc;
}


/* ---- one host thread per rank ---------------------------------------------------------------------------------
 *
 * Every worker walks the whole list with the same bookkeeping as hg_caller_replay_threads - it is deterministic, so
 * all of them derive the same posts and waits - and issues only what belongs to its rank: the posts it owes (before
 * anything else of the step: they mark what it was given in earlier steps and never block), then its waits, then its
 * operations.  Every post of a step precedes every wait of that step in each worker, so a wait only ever sits for a
 * worker that is still busy with an earlier step.
 */

static struct {
    pthread_mutex_t mtx;
    pthread_cond_t cv;
    pthread_t th[CALLER_MAX_RANKS];
    uint32_t nworkers;
    uint64_t gen;        /* bumped (under mtx) to start a job; read with atomics by workers that are still spinning */
    uint32_t finished;   /* workers done with the current job (atomics) */
    int stop;
    /* the job */
    const ThreadHandle* threads;
    uint32_t nRanks;
    const HcommGfxSchedOp* ops;
    uint64_t n;
    void* const* const* bufs;
    int dtype, op;
    uint32_t timeout;
    int32_t rc[CALLER_MAX_RANKS];
    HgCallerStats st[CALLER_MAX_RANKS];
} pool = {.mtx = PTHREAD_MUTEX_INITIALIZER, .cv = PTHREAD_COND_INITIALIZER};

static int32_t rank_walk(uint32_t me, HgCallerStats* st)
{
    static _Thread_local uint32_t last_op[CALLER_MAX_RANKS];
    static _Thread_local uint32_t last_read[CALLER_MAX_RANKS][CALLER_MAX_RANKS];
    static _Thread_local uint32_t synced[CALLER_MAX_RANKS][CALLER_MAX_RANKS];
    static _Thread_local uint8_t need[CALLER_MAX_RANKS][CALLER_MAX_RANKS]; /* [q][r]: q posts to r before this step */
    memset(last_op, 0, sizeof(last_op));
    memset(last_read, 0, sizeof(last_read));
    memset(synced, 0, sizeof(synced));
    memset(st, 0, sizeof(*st));
    const uint32_t nRanks = pool.nRanks, unit = unit_of(pool.dtype);
    const HcommGfxSchedOp* ops = pool.ops;
    const double t0 = now_us();
    int32_t rc = HCCL_SUCCESS;
    uint64_t i = 0;
    uint32_t tick = 0;
    while (i < pool.n && rc == HCCL_SUCCESS) {
        const uint32_t step = ops[i].step;
        uint64_t j = i;
        while (j < pool.n && ops[j].step == step) ++j;
        ++tick;
        memset(need, 0, sizeof(need));
        for (uint64_t k = i; k < j; ++k) {
            const uint32_t r = ops[k].rank, q0 = ops[k].srcRank;
            if (r >= nRanks || q0 >= nRanks) return HCCL_E_PARA;
            for (uint32_t q = 0; q < nRanks; ++q) {
                if (q == r || need[q][r]) continue;
                if (((q == q0) && last_op[q] > synced[q][r]) || last_read[q][r] > synced[q][r]) need[q][r] = 1;
            }
        }
        const double tn = now_us();
        for (uint32_t r = 0; r < nRanks && rc == HCCL_SUCCESS; ++r) /* what this rank owes its peers */
            if (need[me][r]) rc = g.record(pool.threads[me], pool.threads[r], me);
        for (uint32_t q = 0; q < nRanks && rc == HCCL_SUCCESS; ++q) /* what its peers owe this rank */
            if (need[q][me]) {
                rc = g.wait(pool.threads[me], q, pool.timeout);
                ++st->notifies;
            }
        st->host_us_notify += now_us() - tn;
        for (uint32_t q = 0; q < nRanks; ++q)
            for (uint32_t r = 0; r < nRanks; ++r)
                if (need[q][r]) synced[q][r] = tick - 1;
        for (uint64_t k = i; k < j && rc == HCCL_SUCCESS; ++k) {
            if (ops[k].rank == me) {
                rc = issue(pool.threads[me], &ops[k], pool.bufs, pool.dtype, pool.op, unit);
                ++st->calls;
            }
            last_op[ops[k].rank] = tick;
            if (ops[k].srcRank != ops[k].rank) last_read[ops[k].rank][ops[k].srcRank] = tick;
        }
        ++st->batches;
        i = j;
    }
    st->host_us = now_us() - t0;
    return rc;
}

static void* worker_main(void* arg)
{
    const uint32_t me = (uint32_t)(uintptr_t)arg;
    uint64_t seen = 0;
    for (;;) {
        /* a caller that replays in a loop finds the workers still spinning; an idle pool sleeps */
        uint32_t spins = 0;
        while (__atomic_load_n(&pool.gen, __ATOMIC_ACQUIRE) == seen && !__atomic_load_n(&pool.stop, __ATOMIC_ACQUIRE)) {
            if (++spins < 20000u) {
                sched_yield();
            } else {
                pthread_mutex_lock(&pool.mtx);
                while (pool.gen == seen && !pool.stop) pthread_cond_wait(&pool.cv, &pool.mtx);
                pthread_mutex_unlock(&pool.mtx);
            }
        }
        if (__atomic_load_n(&pool.stop, __ATOMIC_ACQUIRE)) return NULL;
        seen = __atomic_load_n(&pool.gen, __ATOMIC_ACQUIRE);
        if (me < pool.nRanks) pool.rc[me] = rank_walk(me, &pool.st[me]);
        __atomic_add_fetch(&pool.finished, 1, __ATOMIC_ACQ_REL);
    }
}

/* Stop and join the workers (also called before the pool grows). */
void hg_caller_pool_shutdown(void)
{
    if (pool.nworkers == 0) return;
    pthread_mutex_lock(&pool.mtx);
    __atomic_store_n(&pool.stop, 1, __ATOMIC_RELEASE);
    pthread_cond_broadcast(&pool.cv);
    pthread_mutex_unlock(&pool.mtx);
    for (uint32_t w = 0; w < pool.nworkers; ++w) pthread_join(pool.th[w], NULL);
    pool.nworkers = 0;
    pool.stop = 0;
    pool.gen = 0; /* workers start out having seen generation 0 */
}

/*
 * As hg_caller_replay_threads, with rank r's calls issued by worker r of a pool of host threads that lives until
 * hg_caller_pool_shutdown.  The calling host thread forks the rank threads from threads[0] first and joins them to it
 * last, so work timed on threads[0]'s stream brackets everything.  *st: the slowest worker's host time (the
 * critical path), calls and notify pairs summed over the workers.
 */
int32_t hg_caller_replay_host_threads(const ThreadHandle* threads, uint32_t nRanks, const HcommGfxSchedOp* ops, uint64_t n,
                                      void* const* const* bufs, int dtype, int op, uint32_t timeout, HgCallerStats* st)
{
    if (!g.lib || !threads || !ops || !bufs || !st) return HCCL_E_PTR;
    if (nRanks == 0 || nRanks > CALLER_MAX_RANKS) return HCCL_E_PARA;
    memset(st, 0, sizeof(*st));
    if (pool.nworkers < nRanks) {
        hg_caller_pool_shutdown();
        pool.finished = 0;
        for (uint32_t w = 0; w < nRanks; ++w) {
            if (pthread_create(&pool.th[w], NULL, worker_main, (void*)(uintptr_t)w) != 0) {
                pool.nworkers = w;
                hg_caller_pool_shutdown();
                return HCCL_E_INTERNAL;
            }
        }
        pool.nworkers = nRanks;
    }
    const double t0 = now_us();
    int32_t rc = HCCL_SUCCESS;
    HgCallerStats fork_join;
    memset(&fork_join, 0, sizeof(fork_join));
    for (uint32_t r = 1; r < nRanks && rc == HCCL_SUCCESS; ++r) rc = post_and_wait(threads, 0, r, timeout, &fork_join);
    if (rc != HCCL_SUCCESS) return rc;
    pool.threads = threads;
    pool.nRanks = nRanks;
    pool.ops = ops;
    pool.n = n;
    pool.bufs = bufs;
    pool.dtype = dtype;
    pool.op = op;
    pool.timeout = timeout;
    __atomic_store_n(&pool.finished, 0, __ATOMIC_RELEASE);
    pthread_mutex_lock(&pool.mtx);
    __atomic_add_fetch(&pool.gen, 1, __ATOMIC_ACQ_REL);
    pthread_cond_broadcast(&pool.cv);
    pthread_mutex_unlock(&pool.mtx);
    while (__atomic_load_n(&pool.finished, __ATOMIC_ACQUIRE) < pool.nworkers) sched_yield();
    for (uint32_t r = 0; r < nRanks; ++r) {
        if (rc == HCCL_SUCCESS) rc = pool.rc[r];
        st->calls += pool.st[r].calls;
        st->notifies += pool.st[r].notifies;
        if (pool.st[r].host_us > st->host_us_end_max) st->host_us_end_max = pool.st[r].host_us; /* slowest worker */
        st->host_us_notify += pool.st[r].host_us_notify;
        st->batches = pool.st[r].batches;
    }
    /* also after a failure: the ranks that did get work are joined to thread 0 */
    for (uint32_t r = 1; r < nRanks; ++r) {
        const int32_t rj = post_and_wait(threads, r, 0, timeout, &fork_join);
        if (rc == HCCL_SUCCESS) rc = rj;
    }
    st->notifies += fork_join.notifies;
    st->host_us = now_us() - t0;
    return rc;
}
