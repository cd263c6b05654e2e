/* Eight host threads use the library at once, each with recorder threads of its own: thread registry, batch mode
 * (per host thread), plan building and replay, launch logs.  Built with -fsanitize=thread by
 * tests/test_host_sanitizers.py; exit status 0 = every call returned what a single-threaded run returns. */
#define _POSIX_C_SOURCE 200809L
#include <pthread.h>
#include <stdio.h>
#include <stdint.h>
#include "hcomm_gfx.h"

static void* worker(void* arg)
{
    const uintptr_t id = (uintptr_t)arg;
    uintptr_t bad = 0;
    void* bufs[3][8];
    for (int k = 0; k < 3; ++k)
        for (int r = 0; r < 8; ++r) bufs[k][r] = (void*)(uintptr_t)(0x7f0000000000ull + ((id * 64 + (uint64_t)k * 8 + r) << 32));
    for (int it = 0; it < 1000; ++it) {
        ThreadHandle th[2];
        if (HcommGfxRecorderThreadAlloc(&th[0]) || HcommGfxRecorderThreadAlloc(&th[1])) { ++bad; continue; }
        char tag[32];
        snprintf(tag, sizeof(tag), "w%u_%d", (unsigned)id, it);
        bad += HcommBatchModeStart(tag) != 0;
        for (int r = 0; r < 8; ++r) {
            bad += HcommLocalCopyOnThread(th[0], bufs[1][r], bufs[0][r], 4096) != 0;
            bad += HcommLocalReduceOnThread(th[0], bufs[1][r], bufs[0][(r + 1) % 8], 1024, HCOMM_DATA_TYPE_FP32, HCOMM_REDUCE_SUM) != 0;
        }
        bad += HcommBatchModeEnd(tag) != 0;
        HcommGfxLaunchRecord rec[8];
        uint32_t n = 0;
        bad += HcommGfxLaunchLogRead(th[0], rec, 8, &n) != 0 || n == 0;
        HcommGfxPlan* p = NULL;
        bad += HcommGfxPlanCreate((HcommGfxAlgorithm)(it % 3), HCOMM_GFX_LOWER_STEPWISE, 8, bufs[0], bufs[1], 100003 + it,
                                  HCOMM_DATA_TYPE_BFP16, HCOMM_REDUCE_MAX, &p) != 0;
        if (p) {
            bad += HcommGfxPlanRun(p, th[1]) != 0;
            bad += HcommGfxPlanDestroy(p) != 0;
        }
        bad += HcommGfxLaunchLogRead(th[1], rec, 8, &n) != 0 || n == 0;
        bad += HcommThreadFree(th, 2) != 0;
        bad += HcommLocalCopyOnThread(th[0], bufs[1][0], bufs[0][0], 16) == 0; /* a freed handle is refused */
    }
    return (void*)bad;
}

/* One host thread records into a recorder thread inside a batch while another host thread tries to free it and to
 * record into it: both are refused until the batch has ended, and nothing of the refused calls is left queued. */
static pthread_barrier_t g_bar;
static ThreadHandle g_shared;

static void* batch_owner(void* arg)
{
    (void)arg;
    uintptr_t bad = 0;
    bad += HcommGfxRecorderThreadAlloc(&g_shared) != 0;
    bad += HcommBatchModeStart("owner") != 0;
    bad += HcommLocalCopyOnThread(g_shared, (void*)0x200000, (const void*)0x100000, 4096) != 0;
    pthread_barrier_wait(&g_bar); /* the other thread now tries to free and to record */
    pthread_barrier_wait(&g_bar);
    bad += HcommBatchModeEnd("owner") != 0;
    uint32_t n = 0;
    bad += HcommGfxLaunchLogRead(g_shared, NULL, 0, &n) != 0 || n != 1; /* one launch: the other thread's copy was refused */
    pthread_barrier_wait(&g_bar); /* after End the other thread may free it */
    return (void*)bad;
}

static void* batch_intruder(void* arg)
{
    (void)arg;
    uintptr_t bad = 0;
    pthread_barrier_wait(&g_bar);
    bad += HcommThreadFree(&g_shared, 1) != HCCL_E_UNAVAIL;
    bad += HcommLocalCopyOnThread(g_shared, (void*)0x400000, (const void*)0x300000, 4096) != HCCL_E_UNAVAIL; /* not batching either */
    bad += HcommBatchModeStart("intruder") != 0;
    bad += HcommLocalCopyOnThread(g_shared, (void*)0x400000, (const void*)0x300000, 4096) != HCCL_E_UNAVAIL;
    bad += HcommBatchModeEnd("intruder") != 0;
    pthread_barrier_wait(&g_bar);
    pthread_barrier_wait(&g_bar);
    bad += HcommThreadFree(&g_shared, 1) != 0;
    return (void*)bad;
}

/* Two host threads open a batch and record into the same free thread at the same moment, 2,000 times over: the claim
 * is one compare-and-exchange, so exactly one of them is taken each time, and the launch log holds the winner's
 * operation alone. */
static ThreadHandle g_raced;
static int g_race_result[2];

static void* racer(void* arg)
{
    const uintptr_t id = (uintptr_t)arg;
    uintptr_t bad = 0;
    for (int it = 0; it < 2000; ++it) {
        if (id == 0) bad += HcommGfxRecorderThreadAlloc(&g_raced) != 0;
        pthread_barrier_wait(&g_bar);
        bad += HcommBatchModeStart("race") != 0;
        g_race_result[id] = HcommLocalCopyOnThread(g_raced, (void*)(0x200000 + (id << 24)), (const void*)(0x100000 + (id << 24)), 4096);
        pthread_barrier_wait(&g_bar); /* both have tried before either batch ends */
        bad += HcommBatchModeEnd("race") != 0;
        pthread_barrier_wait(&g_bar);
        if (id == 0) {
            const int won = (g_race_result[0] == 0) + (g_race_result[1] == 0);
            const int lost = (g_race_result[0] == HCCL_E_UNAVAIL) + (g_race_result[1] == HCCL_E_UNAVAIL);
            uint32_t n = 0;
            bad += won != 1 || lost != 1;
            bad += HcommGfxLaunchLogRead(g_raced, NULL, 0, &n) != 0 || n != 1;
            bad += HcommThreadFree(&g_raced, 1) != 0;
        }
        pthread_barrier_wait(&g_bar);
    }
    return (void*)bad;
}

int main(void)
{
    pthread_t t[8];
    uintptr_t bad = 0;
    if (pthread_barrier_init(&g_bar, NULL, 2)) return 2;
    for (uintptr_t i = 0; i < 2; ++i)
        if (pthread_create(&t[i], NULL, racer, (void*)i)) return 2;
    for (int i = 0; i < 2; ++i) {
        void* r = NULL;
        pthread_join(t[i], &r);
        bad += (uintptr_t)r;
    }
    if (bad) {
        printf("racing claims: bad %lu\n", (unsigned long)bad);
        return 1;
    }
    if (pthread_create(&t[0], NULL, batch_owner, NULL) || pthread_create(&t[1], NULL, batch_intruder, NULL)) return 2;
    for (int i = 0; i < 2; ++i) {
        void* r = NULL;
        pthread_join(t[i], &r);
        bad += (uintptr_t)r;
    }
    if (bad) {
        printf("batch ownership: bad %lu\n", (unsigned long)bad);
        return 1;
    }
    for (uintptr_t i = 0; i < 8; ++i)
        if (pthread_create(&t[i], NULL, worker, (void*)i)) return 2;
    for (int i = 0; i < 8; ++i) {
        void* r = NULL;
        pthread_join(t[i], &r);
        bad += (uintptr_t)r;
    }
    printf("threads 8 bad %lu\n", (unsigned long)bad);
    return bad ? 1 : 0;
}
