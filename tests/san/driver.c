/* Exercises every host-side generator, checker and plan builder of libhcomm_gfx on a recorder thread (no GPU): built
 * with -fsanitize=address,undefined by tests/test_host_sanitizers.py together with the library's C files and
 * stubs.c in place of the HIP layer.  Valid, boundary and invalid arguments alike; exit status 0 = every call that
 * reported success produced a consistent plan / list. */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include "hcomm_gfx.h"

static void* bufs[5][32];
static uint64_t plans, emits, checks, bad;

static void run_plan(ThreadHandle th, HcommGfxPlan* p)
{
    if (!p) return;
    ++plans;
    HcommGfxPlanInfo info;
    if (HcommGfxPlanGetInfo(p, &info)) ++bad;
    for (uint32_t i = 0; i < info.launches; ++i) {
        HcommGfxLaunchRecord r;
        if (HcommGfxPlanGetLaunch(p, i, &r)) ++bad;
    }
    if (HcommGfxPlanRun(p, th)) ++bad;
    if (info.launches > 1 && HcommGfxPlanRunRange(p, th, 1, info.launches - 1)) ++bad;
    HcommGfxLaunchLogClear(th);
    HcommGfxPlanDestroy(p);
}

static void emit_twice(int32_t (*f)(void*, HcommGfxSchedOp*, uint64_t, uint64_t*), void* ctx)
{
    uint64_t n = 0;
    if (f(ctx, NULL, 0, &n)) return;
    ++emits;
    HcommGfxSchedOp* ops = (HcommGfxSchedOp*)malloc((n ? n : 1) * sizeof(*ops));
    uint64_t m = 0;
    f(ctx, ops, n / 2, &m); /* a short buffer must not be overrun */
    f(ctx, ops, n, &m);
    if (m != n) ++bad;
    free(ops);
}

typedef struct { int a, b; uint32_t n, s, l; uint64_t count, ccl; int dt; } Ctx;
static int32_t e_sched(void* c, HcommGfxSchedOp* o, uint64_t cap, uint64_t* n) { Ctx* x = c; return HcommGfxScheduleEmitStrided(x->a, x->n, x->count, x->count + 3, x->dt, o, cap, n); }
static int32_t e_opbase(void* c, HcommGfxSchedOp* o, uint64_t cap, uint64_t* n) { Ctx* x = c; return HcommGfxOpBaseEmit(x->a, x->n, x->count, x->ccl, x->dt, o, cap, n); }
static int32_t e_hier(void* c, HcommGfxSchedOp* o, uint64_t cap, uint64_t* n) { Ctx* x = c; return x->b ? HcommGfxMeshHierEmit(x->a, x->s, x->l, x->count, x->dt, o, cap, n) : HcommGfxHierEmit(x->a, x->s, x->l, x->count, x->dt, o, cap, n); }
static int32_t e_dbring(void* c, HcommGfxSchedOp* o, uint64_t cap, uint64_t* n) { Ctx* x = c; return HcommGfxDoubleRingEmit(x->a, x->s, x->l, x->count, x->ccl, x->dt, o, cap, n); }
static int32_t e_dbrs(void* c, HcommGfxSchedOp* o, uint64_t cap, uint64_t* n) { Ctx* x = c; return HcommGfxDoubleRingReduceScatterEmit(x->n, x->count, x->ccl, x->dt, o, cap, n); }
static int32_t e_dbhrs(void* c, HcommGfxSchedOp* o, uint64_t cap, uint64_t* n) { Ctx* x = c; return HcommGfxDoubleRingHierReduceScatterEmit(x->a, x->a, x->b + 1, x->s, x->l, x->count, x->ccl, x->dt, o, cap, n); }
static int32_t e_hrs(void* c, HcommGfxSchedOp* o, uint64_t cap, uint64_t* n) { Ctx* x = c; return HcommGfxHierReduceScatterEmit(x->b, x->a, x->s, x->l, x->count, x->ccl, x->dt, o, cap, n); }
static int32_t e_oph(void* c, HcommGfxSchedOp* o, uint64_t cap, uint64_t* n) { Ctx* x = c; return HcommGfxOrderPreservedHierAllReduceEmit(x->a, x->s, x->l, x->count, x->ccl, x->dt, o, cap, n); }
static int32_t e_ops(void* c, HcommGfxSchedOp* o, uint64_t cap, uint64_t* n) { Ctx* x = c; return HcommGfxOrderPreservedSmallEmit(x->n, x->count, x->ccl, x->dt, o, cap, n); }
static int32_t e_ophrs(void* c, HcommGfxSchedOp* o, uint64_t cap, uint64_t* n) { Ctx* x = c; return HcommGfxOrderPreservedHierReduceScatterEmit(x->s, x->l, x->count, x->ccl, x->dt, o, cap, n); }
static int32_t e_op(void* c, HcommGfxSchedOp* o, uint64_t cap, uint64_t* n) { Ctx* x = c; return HcommGfxOrderPreservedEmit(x->n, x->count, x->ccl, x->dt, o, cap, n); }
static int32_t e_opar(void* c, HcommGfxSchedOp* o, uint64_t cap, uint64_t* n) { Ctx* x = c; return HcommGfxOrderPreservedAllReduceEmit(x->n, x->count, x->ccl, x->dt, o, cap, n); }

/* Batches whose threads order one another by notifies: rank r's operations on thread r with every thread posting to
 * and waiting for every other between the steps, all inside one HcommBatchModeStart / End pair; the same with a wait
 * too many (nothing can satisfy it: HCCL_E_TIMEOUT), with a thread freed in the middle of the batch (likewise: its
 * records went with it), and with records to threads outside the batch, one of them freed before End. */
static void ordered_batches(void)
{
    enum { N = 6 };
    ThreadHandle t[N], out[2];
    for (int r = 0; r < N; ++r) bad += HcommGfxRecorderThreadAlloc(&t[r]) != 0;
    for (int r = 0; r < 2; ++r) bad += HcommGfxRecorderThreadAlloc(&out[r]) != 0;
    for (int variant = 0; variant < 4; ++variant)
        for (int alg = 0; alg <= 17; ++alg) {
            uint64_t n = 0;
            if (HcommGfxScheduleEmit(alg, N, 4099, HCOMM_DATA_TYPE_FP32, NULL, 0, &n)) continue;
            HcommGfxSchedOp* ops = (HcommGfxSchedOp*)malloc((n ? n : 1) * sizeof(*ops));
            bad += HcommGfxScheduleEmit(alg, N, 4099, HCOMM_DATA_TYPE_FP32, ops, n, &n) != 0;
            bad += HcommBatchModeStart("ordered") != 0;
            int freed = 0;
            for (uint64_t i = 0; i < n;) {
                uint64_t j = i;
                while (j < n && ops[j].step == ops[i].step) ++j;
                for (int r = 0; r < N; ++r)
                    for (int q = 0; q < N; ++q)
                        if (q != r && !(freed && (q == N - 1 || r == N - 1))) bad += HcommThreadNotifyRecordOnThread(t[r], t[q], (uint32_t)r) != 0;
                for (int r = 0; r < N; ++r)
                    for (int q = 0; q < N; ++q)
                        if (q != r && !(freed && (q == N - 1 || r == N - 1))) bad += HcommThreadNotifyWaitOnThread(t[r], (uint32_t)q, 10) != 0;
                for (uint64_t k = i; k < j; ++k) {
                    if (freed && ops[k].rank == N - 1) continue;
                    char* d = (char*)bufs[ops[k].dstBuf][ops[k].rank] + ops[k].dstOff;
                    char* sp = (char*)bufs[ops[k].srcBuf][ops[k].srcRank] + ops[k].srcOff;
                    bad += (ops[k].kind ? HcommLocalReduceOnThread(t[ops[k].rank], d, sp, ops[k].bytes / 4, HCOMM_DATA_TYPE_FP32, HCOMM_REDUCE_SUM)
                                        : HcommLocalCopyOnThread(t[ops[k].rank], d, sp, ops[k].bytes)) != 0;
                }
                if (variant == 2 && !freed && j < n) { /* a thread of the batch goes away with records still addressed to it */
                    bad += HcommThreadFree(&t[N - 1], 1) != 0;
                    freed = 1;
                }
                i = j;
            }
            if (variant == 1) bad += HcommThreadNotifyWaitOnThread(t[2], 0, 10) != 0; /* one wait too many */
            if (variant == 3) {
                bad += HcommThreadNotifyRecordOnThread(t[0], out[0], 3) != 0;
                bad += HcommThreadNotifyRecordOnThread(t[1], out[1], 4) != 0;
                bad += HcommThreadFree(&out[1], 1) != 0;
            }
            const int32_t rc = HcommBatchModeEnd("ordered");
            /* a freed thread takes its queued calls with it, records included: the peers' waits for them can never pass */
            bad += rc != (variant == 1 || freed ? HCCL_E_TIMEOUT : HCCL_SUCCESS);
            if (variant == 3) {
                bad += HcommThreadNotifyWaitOnThread(out[0], 3, 0) != 0;
                bad += HcommGfxRecorderThreadAlloc(&out[1]) != 0;
            }
            if (freed) bad += HcommGfxRecorderThreadAlloc(&t[N - 1]) != 0;
            /* whatever the batch left pending is drained, so that the next one starts clean */
            for (int r = 0; r < N; ++r)
                for (uint32_t q = 0; q < N; ++q)
                    while (HcommThreadNotifyWaitOnThread(t[r], q, 0) == 0) {}
            for (int r = 0; r < N; ++r) HcommGfxLaunchLogClear(t[r]);
            free(ops);
            ++checks;
        }
    bad += HcommThreadFree(t, N) != 0;
    bad += HcommThreadFree(out, 2) != 0;
}

int main(void)
{
    for (int k = 0; k < 5; ++k)
        for (int r = 0; r < 32; ++r) bufs[k][r] = (void*)(uintptr_t)(0x7f0000000000ull + ((uint64_t)(k * 32 + r) << 32));
    ThreadHandle th;
    if (HcommGfxRecorderThreadAlloc(&th)) return 2;
    const uint64_t counts[] = {0, 1, 100, 4097};
    const uint32_t ns[] = {0, 1, 2, 3, 4, 5, 8, 17, 32, 33};
    const uint32_t sl[] = {0, 1, 2, 3, 5, 8};
    const uint64_t ccls[] = {128, 4096, 1 << 20};
    const int dts[] = {HCOMM_DATA_TYPE_INT8, HCOMM_DATA_TYPE_BFP16, 99};
    HcommGfxCheckReport rep;
    HcommGfxPlan* p;
    for (unsigned ni = 0; ni < 10; ++ni)
        for (unsigned ci = 0; ci < 4; ++ci)
            for (unsigned di = 0; di < 3; ++di) {
                const uint32_t n = ns[ni];
                Ctx x = {0, 0, n, 0, 0, counts[ci], 0, dts[di]};
                for (int alg = -1; alg <= 17; ++alg) {
                    x.a = alg;
                    emit_twice(e_sched, &x);
                    if (HcommGfxScheduleCheck(alg, n, x.count, 0, x.dt, &rep) == 0) ++checks;
                    for (int low = 0; low < 2; ++low) {
                        p = NULL;
                        HcommGfxPlanCreateEx(alg, low, n, bufs[0], bufs[1], bufs[2], x.count, 0, x.dt, HCOMM_REDUCE_SUM, &p);
                        run_plan(th, p);
                    }
                    for (unsigned cc = 0; cc < 3; ++cc) {
                        x.ccl = ccls[cc];
                        if (n % 4 == 1 || n == 8) {
                            emit_twice(e_opbase, &x);
                            if (HcommGfxOpBaseCheck(alg, n, x.count, x.ccl, x.dt, &rep) == 0) ++checks;
                            for (int low = 0; low < 2; ++low) {
                                p = NULL;
                                HcommGfxOpBasePlanCreate(alg, low, n, bufs[3], bufs[4], bufs[0], bufs[1], bufs[2], x.ccl, x.count, x.dt, HCOMM_REDUCE_MAX, &p);
                                run_plan(th, p);
                            }
                        }
                    }
                }
                for (unsigned cc = 0; cc < 3; ++cc) {
                    x.ccl = ccls[cc];
                    emit_twice(e_dbrs, &x);
                    emit_twice(e_op, &x);
                    emit_twice(e_ops, &x);
                    if (HcommGfxOrderPreservedSmallCheck(n, x.count, x.ccl, x.dt, &rep) == 0) ++checks;
                    p = NULL; HcommGfxOrderPreservedSmallPlanCreate(n, bufs[3], bufs[4], bufs[1], x.ccl, x.count, x.dt, HCOMM_REDUCE_MAX, &p); run_plan(th, p);
                    emit_twice(e_opar, &x);
                    if (HcommGfxDoubleRingReduceScatterCheck(n, x.count, x.ccl, x.dt, &rep) == 0) ++checks;
                    if (HcommGfxOrderPreservedCheck(n, x.count, x.ccl, x.dt, &rep) == 0) ++checks;
                    if (HcommGfxOrderPreservedAllReduceCheck(n, x.count, x.ccl, x.dt, &rep) == 0) ++checks;
                    p = NULL; HcommGfxDoubleRingReduceScatterPlanCreate(n, bufs[3], bufs[4], bufs[0], x.ccl, x.count, x.dt, HCOMM_REDUCE_SUM, &p); run_plan(th, p);
                    p = NULL; HcommGfxOrderPreservedPlanCreate(n, bufs[3], bufs[4], bufs[1], x.ccl, x.count, x.dt, HCOMM_REDUCE_MIN, &p); run_plan(th, p);
                    p = NULL; HcommGfxOrderPreservedAllReducePlanCreate(n, bufs[3], bufs[4], bufs[0], bufs[1], x.ccl, x.count, x.dt, HCOMM_REDUCE_SUM, &p); run_plan(th, p);
                }
                HcommGfxAllReduceLocalReduceNoAlloc(th, n, bufs[0], bufs[1], x.count, x.dt, HCOMM_REDUCE_SUM); /* launches on storage of the call's own */
                for (int ar = 0; ar < 2; ++ar) { p = NULL; HcommGfxOrderPreservedFusedPlanCreate(ar, 1, n, bufs[3], bufs[4], x.count, x.dt, HCOMM_REDUCE_PROD, &p); run_plan(th, p); }
            }
    /* the single-launch lowerings of the three-buffer schedules at sizes that keep their slices on 16-byte
     * boundaries, with the trees read back */
    {
        const uint32_t fn[] = {2, 4, 8, 16, 32};
        const uint64_t fc[] = {1 << 16, (1 << 18) + 40, 3 << 20};
        const int fa[] = {HCOMM_GFX_ALG_ALLREDUCE_LOCAL_REDUCE, HCOMM_GFX_ALG_ALLREDUCE_CHUNK_MESH, HCOMM_GFX_ALG_REDUCE_SCATTER_LOCAL_REDUCE, HCOMM_GFX_ALG_ALLREDUCE_DOUBLING};
        for (unsigned ni = 0; ni < 5; ++ni)
            for (unsigned ci = 0; ci < 3; ++ci)
                for (unsigned ai = 0; ai < 4; ++ai) {
                    p = NULL;
                    HcommGfxPlanCreateEx(fa[ai], ai == 3 ? HCOMM_GFX_LOWER_FUSED_KEEP_INPUTS : HCOMM_GFX_LOWER_FUSED, fn[ni], bufs[0], bufs[1], NULL, fc[ci], 0, HCOMM_DATA_TYPE_FP32, HCOMM_REDUCE_SUM, &p);
                    HcommGfxPlanInfo info;
                    if (p && HcommGfxPlanGetInfo(p, &info) == 0)
                        for (uint32_t i = 0; i < info.launches; ++i)
                            for (uint32_t sgm = 0; sgm < 40; ++sgm) {
                                const void* leaves[32];
                                uint32_t k = 0;
                                uint64_t off = 0, bytes = 0;
                                if (HcommGfxPlanGetTreeSegment(p, i, sgm, leaves, 32, &k, &off, &bytes, NULL) == 0) ++checks;
                                HcommGfxPlanGetTreeSegment(p, i, sgm, leaves, 1, &k, NULL, NULL, NULL);
                            }
                    run_plan(th, p);
                }
    }
    /* any schedule's own list as tree launches that keep the inputs (most are refused: deep or re-cut trees) */
    for (int alg = 0; alg <= 17; ++alg)
        for (uint32_t n = 1; n <= 9; ++n) {
            uint64_t total = 0;
            if (HcommGfxScheduleEmit(alg, n, 40960, HCOMM_DATA_TYPE_FP32, NULL, 0, &total) != 0 || total == 0) continue;
            HcommGfxSchedOp* ops = (HcommGfxSchedOp*)calloc(total, sizeof(*ops));
            if (!ops) return 2;
            if (HcommGfxScheduleEmit(alg, n, 40960, HCOMM_DATA_TYPE_FP32, ops, total, &total) == 0) {
                p = NULL;
                if (HcommGfxPlanCreateFromOpsKeepInputs(ops, total, n, bufs[0], bufs[1], HCOMM_DATA_TYPE_FP32, HCOMM_REDUCE_MAX, &p) == 0) ++checks;
                run_plan(th, p);
                p = NULL;
                HcommGfxPlanCreateFromOpsKeepInputs(ops, total / 2, n, bufs[0], bufs[1], HCOMM_DATA_TYPE_FP32, HCOMM_REDUCE_MAX, &p); /* a truncated list */
                run_plan(th, p);
            }
            free(ops);
        }
    /* lists a caller could write that the tree lowering must refuse at once: a value folded into itself (its tree doubles
     * with every operation), a chain of a million folds, operations of one step that observe each other */
    {
        const uint64_t big = 1000001;
        HcommGfxSchedOp* ops = (HcommGfxSchedOp*)calloc(big, sizeof(*ops));
        if (!ops) return 2;
        for (int variant = 0; variant < 3; ++variant) {
            const uint64_t total = variant == 0 ? 65 : variant == 1 ? big : 3;
            memset(ops, 0, total * sizeof(*ops));
            ops[0].kind = 0; ops[0].dstBuf = 1; ops[0].srcBuf = 0; ops[0].bytes = 4096;       /* out0 = in0 */
            for (uint64_t i = 1; i < total; ++i) {
                ops[i].step = variant == 2 ? 1 : (uint32_t)i;                                   /* variant 2: both in step 1 */
                ops[i].kind = 1; ops[i].dstBuf = 1; ops[i].bytes = 4096;                        /* out0 += ... */
                ops[i].srcBuf = variant == 0 ? 1 : 0;                                           /* ... out0 / in1 / in1, in2 */
                ops[i].srcRank = variant == 0 ? 0 : variant == 1 ? 1 : (uint32_t)i;
            }
            p = NULL;
            if (HcommGfxPlanCreateFromOpsKeepInputs(ops, total, 3, bufs[0], bufs[1], HCOMM_DATA_TYPE_FP32, HCOMM_REDUCE_SUM, &p) == HCCL_E_NOT_SUPPORT && !p) ++checks;
            else return 3;
        }
        free(ops);
    }
    /* two-level executors */
    for (unsigned si = 0; si < 5; ++si)
        for (unsigned li = 0; li < 5; ++li)
            for (unsigned ci = 0; ci < 4; ++ci)
                for (int alg = -1; alg <= 17; ++alg)
                    for (int mesh = 0; mesh < 2; ++mesh) {
                        const uint32_t s = sl[si], l = sl[li];
                        Ctx x = {alg, mesh, s * l, s, l, counts[ci], 0, HCOMM_DATA_TYPE_FP16};
                        emit_twice(e_hier, &x);
                        if ((mesh ? HcommGfxMeshHierCheck : HcommGfxHierCheck)(alg, s, l, x.count, x.dt, &rep) == 0) ++checks;
                        p = NULL;
                        (mesh ? HcommGfxMeshHierPlanCreate : HcommGfxHierPlanCreate)(alg, s, l, bufs[0], bufs[1], x.count, x.dt, HCOMM_REDUCE_SUM, &p);
                        run_plan(th, p);
                        for (unsigned cc = 0; cc < 3; ++cc) {
                            x.ccl = ccls[cc];
                            if (x.ccl < 4096 && x.count > 1000) continue;
                            emit_twice(e_hrs, &x);
                            if (HcommGfxHierReduceScatterCheck(mesh, alg, s, l, x.count, x.ccl, x.dt, &rep) == 0) ++checks;
                            p = NULL;
                            HcommGfxHierReduceScatterPlanCreate(mesh, alg, s, l, bufs[3], bufs[4], bufs[0], bufs[1], x.ccl, x.count, x.dt, HCOMM_REDUCE_SUM, &p);
                            run_plan(th, p);
                            if (!mesh) {
                                emit_twice(e_dbhrs, &x);
                                if (HcommGfxDoubleRingHierReduceScatterCheck(alg, alg, 1, s, l, x.count, x.ccl, x.dt, &rep) == 0) ++checks;
                                p = NULL; HcommGfxDoubleRingHierReduceScatterPlanCreate(alg, alg, 1, s, l, bufs[3], bufs[4], bufs[0], x.ccl, x.count, x.dt, HCOMM_REDUCE_SUM, &p); run_plan(th, p);
                                if (s * l * 2 <= 32) { p = NULL; HcommGfxDoubleRingHierReduceScatterPlanCreate(alg, HCOMM_GFX_ALG_REDUCE_SCATTER_NHR, 2, s, l, bufs[3], bufs[4], bufs[0], x.ccl, x.count, x.dt, HCOMM_REDUCE_SUM, &p); run_plan(th, p); }
                                emit_twice(e_oph, &x);
                                if (alg == 0) {
                                    emit_twice(e_ophrs, &x);
                                    if (HcommGfxOrderPreservedHierReduceScatterCheck(s, l, x.count, x.ccl, x.dt, &rep) == 0) ++checks;
                                    p = NULL; HcommGfxOrderPreservedHierReduceScatterPlanCreate(s, l, bufs[3], bufs[4], bufs[0], bufs[1], x.ccl, x.count, x.dt, HCOMM_REDUCE_SUM, &p); run_plan(th, p);
                                    for (int ar = 0; ar < 2; ++ar) { p = NULL; HcommGfxOrderPreservedFusedPlanCreate(ar, s, l, bufs[3], bufs[4], x.count, x.dt, HCOMM_REDUCE_SUM, &p); run_plan(th, p); }
                                }
                                if (HcommGfxOrderPreservedHierAllReduceCheck(alg, s, l, x.count, x.ccl, x.dt, &rep) == 0) ++checks;
                                p = NULL;
                                HcommGfxOrderPreservedHierAllReducePlanCreate(alg, s, l, bufs[3], bufs[4], bufs[0], bufs[1], x.ccl, x.count, x.dt, HCOMM_REDUCE_SUM, &p);
                                run_plan(th, p);
                                emit_twice(e_dbring, &x);
                                if (HcommGfxDoubleRingCheck(alg, s, l, x.count, x.ccl, x.dt, &rep) == 0) ++checks;
                                p = NULL;
                                HcommGfxDoubleRingPlanCreate(alg, s, l, bufs[3], bufs[4], bufs[0], bufs[1], x.ccl, x.count, x.dt, HCOMM_REDUCE_SUM, &p);
                                run_plan(th, p);
                            }
                        }
                    }
    /* malformed op lists */
    HcommGfxSchedOp ops[4];
    memset(ops, 0, sizeof(ops));
    ops[0].bytes = 16; ops[1].bytes = 16; ops[1].rank = 40; ops[2].dstBuf = 9; ops[3].step = 0;
    void* const* bb[5] = {bufs[0], bufs[1], bufs[2], bufs[3], bufs[4]};
    for (uint64_t k = 0; k <= 4; ++k) {
        p = NULL;
        HcommGfxPlanCreateFromOps(ops, k, 2, bb, HCOMM_DATA_TYPE_FP32, HCOMM_REDUCE_SUM, &p);
        run_plan(th, p);
        HcommGfxOpListCheck(ops, k, 2, HCOMM_GFX_EXPECT_ALLREDUCE, 4, 0, 4, &rep);
    }
    /* the same plans shaped with the one-round kernels switched off, and on again */
    for (int on = 0; on <= 1; ++on) {
        const int32_t before = HcommGfxSetDirectLaunches(on);
        if (before != !on) ++bad;
        for (uint32_t n = 1; n <= 9; ++n)
            for (int alg = 0; alg <= 17; ++alg)
                for (int low = 0; low <= 2; ++low) {
                    p = NULL;
                    HcommGfxPlanCreateEx(alg, low, n, bufs[0], bufs[1], bufs[2], 4099, 0, HCOMM_DATA_TYPE_FP16, HCOMM_REDUCE_SUM, &p);
                    run_plan(th, p);
                }
    }
    ordered_batches();
    HcommGfxSlice slc[32];
    for (uint32_t n = 0; n <= 32; ++n) HcommGfxCalcSlices(100003, 2, n, slc);
    HcommThreadFree(&th, 1);
    printf("plans %llu emits %llu checks %llu bad %llu\n", (unsigned long long)plans, (unsigned long long)emits,
           (unsigned long long)checks, (unsigned long long)bad);
    return bad ? 1 : 0;
}
