/*
 * hg_check.c - symbolic checker for schedule op lists.
 *
 * A miniature of the reference's algorithm checker (test/st/algorithm/README_en.md:13-15,202-231): no data is
 * moved; every byte range of every rank buffer carries the set of (rank, origin offset) contributions folded
 * into it.  Each buffer is an ordered map of intervals that is split on demand: an operation first cuts its source
 * and destination ranges at their ends and at each other's inner cuts, so that it maps whole intervals onto whole
 * intervals, and then copies or merges the interval states.  Two verdicts:
 *   memory conflicts - inside one step no operation may write a range another operation of the step reads or
 *                      writes (test/st/algorithm/README_en.md:202-231);
 *   semantics        - at the end, every byte of the expected result ranges holds exactly one contribution from
 *                      every rank, taken from the same offset of that rank's input
 *                      (test/st/algorithm/utils/checker/semantics_check/allreduce_semantics_checker.cc:59-96 and
 *                      its reduce-scatter twin).
 * Used by the tests as a guard on every generated schedule and on deliberately broken ones.
 */
#include <stdlib.h>
#include <string.h>
#include <stdio.h>

#include "hg_host.h"
#include "hg_sched.h"

#define NO_DELTA INT64_MIN
#define NBUF HCOMM_GFX_NUM_BUFS

typedef struct {
    uint8_t cnt[HCOMM_GFX_MAX_RANKS];   /* how many times rank k's data is folded in */
    int64_t delta[HCOMM_GFX_MAX_RANKS]; /* origin offset - current offset of that contribution */
    uint8_t bad;                        /* contributions of one rank from two different origins were mixed */
} Cell;

static void report(HcommGfxCheckReport* r, int is_conflict, const char* fmt, uint64_t a, uint64_t b, uint64_t c)
{
    if (is_conflict) r->conflicts++; else r->semanticErrors++;
    if (r->message[0] == 0) snprintf(r->message, sizeof(r->message), fmt, (unsigned long long)a, (unsigned long long)b, (unsigned long long)c);
}

static int ranges_overlap(uint64_t a, uint64_t an, uint64_t b, uint64_t bn) { return a < b + bn && b < a + an; }

#define MAX_INTERVALS_PER_BUFFER (1u << 20)

/* One rank buffer: intervals [b[i], b[i+1]) with state pool[ix[i]], i < n; b has n + 1 entries.  The states live in a
 * pool and the map orders indices into it, so that cutting an interval moves 4 bytes per interval behind the cut and
 * not a whole state. */
typedef struct {
    uint64_t* b;
    uint32_t* ix;
    Cell* pool;
    size_t n, cap, pool_n, pool_cap;
} IMap;

#define CELL(m, i) ((m)->pool[(m)->ix[i]])

static int imap_init(IMap* m, uint64_t extent, uint32_t nranks, int own_rank)
{
    m->cap = 16;
    m->pool_cap = 16;
    m->b = (uint64_t*)malloc((m->cap + 1) * sizeof(uint64_t));
    m->ix = (uint32_t*)malloc(m->cap * sizeof(uint32_t));
    m->pool = (Cell*)calloc(m->pool_cap, sizeof(Cell));
    if (!m->b || !m->ix || !m->pool) return -1;
    m->n = 1;
    m->pool_n = 1;
    m->ix[0] = 0;
    m->b[0] = 0;
    m->b[1] = extent;
    for (uint32_t k = 0; k < nranks; ++k) m->pool[0].delta[k] = NO_DELTA;
    if (own_rank >= 0) { /* an input holds its own rank's data from the same offset */
        m->pool[0].cnt[own_rank] = 1;
        m->pool[0].delta[own_rank] = 0;
    }
    return 0;
}

/* index of the interval that starts at v, after cutting one in two if v falls inside it; -1 when out of memory */
static long imap_cut(IMap* m, uint64_t v)
{
    size_t lo = 0, hi = m->n; /* first boundary >= v among b[0..n] */
    while (lo < hi) {
        const size_t mid = (lo + hi) / 2;
        if (m->b[mid] < v) lo = mid + 1; else hi = mid;
    }
    if (m->b[lo] == v) return (long)lo;
    /* b[lo-1] < v < b[lo]: interval lo-1 is cut */
    if (m->n >= MAX_INTERVALS_PER_BUFFER) return -1;
    if (m->n == m->cap) {
        const size_t cap = m->cap * 2;
        uint64_t* nb = (uint64_t*)realloc(m->b, (cap + 1) * sizeof(uint64_t));
        if (!nb) return -1;
        m->b = nb;
        uint32_t* ni = (uint32_t*)realloc(m->ix, cap * sizeof(uint32_t));
        if (!ni) return -1;
        m->ix = ni;
        m->cap = cap;
    }
    if (m->pool_n == m->pool_cap) {
        const size_t cap = m->pool_cap * 2;
        Cell* nc = (Cell*)realloc(m->pool, cap * sizeof(Cell));
        if (!nc) return -1;
        m->pool = nc;
        m->pool_cap = cap;
    }
    memmove(&m->b[lo + 1], &m->b[lo], (m->n + 1 - lo) * sizeof(uint64_t));
    memmove(&m->ix[lo], &m->ix[lo - 1], (m->n - (lo - 1)) * sizeof(uint32_t));
    m->pool[m->pool_n] = m->pool[m->ix[lo - 1]]; /* the upper half starts as a copy of the interval that was cut */
    m->ix[lo] = (uint32_t)m->pool_n++;
    m->b[lo] = v;
    m->n++;
    return (long)lo;
}

/* cut `to` wherever `from` is cut strictly inside (lo, lo + len), moved by to_lo - lo */
static int imap_mirror_cuts(const IMap* from, uint64_t lo, uint64_t len, IMap* to, uint64_t to_lo)
{
    size_t k = 0, hi = from->n;
    while (k < hi) { /* first boundary > lo */
        const size_t mid = (k + hi) / 2;
        if (from->b[mid] <= lo) k = mid + 1; else hi = mid;
    }
    size_t m = 0;
    while (k + m <= from->n && from->b[k + m] < lo + len) ++m;
    if (m == 0) return 0;
    uint64_t* v = (uint64_t*)malloc(m * sizeof(uint64_t)); /* `to` may be `from` itself: take a snapshot first */
    if (!v) return -1;
    memcpy(v, &from->b[k], m * sizeof(uint64_t));
    int rc = 0;
    for (size_t i = 0; i < m && rc == 0; ++i)
        if (imap_cut(to, v[i] - lo + to_lo) < 0) rc = -1;
    free(v);
    return rc;
}

int32_t HcommGfxOpListCheck(
    const HcommGfxSchedOp* ops, uint64_t nOps, uint32_t nRanks, HcommGfxExpectation expect, uint64_t count,
    uint64_t strideCount, uint32_t unitSize, HcommGfxCheckReport* rep)
{
    if (!rep) return HCCL_E_PTR;
    memset(rep, 0, sizeof(*rep));
    if (nOps && !ops) return HCCL_E_PTR;
    if (nRanks == 0 || nRanks > HCOMM_GFX_MAX_RANKS || unitSize == 0) return HCCL_E_PARA;
    if ((uint32_t)expect > HCOMM_GFX_EXPECT_REDUCE_SCATTER_USER) return HCCL_E_PARA;
    const int user = (expect == HCOMM_GFX_EXPECT_ALLREDUCE_USER || expect == HCOMM_GFX_EXPECT_REDUCE_SCATTER_USER);
    const uint32_t data_buf = user ? HCOMM_GFX_BUF_USER_IN : 0u; /* where every rank's own data starts */
    if (strideCount == 0) strideCount = count;
    const uint64_t total = count * unitSize;
    for (uint64_t i = 0; i < nOps; ++i)
        if (ops[i].rank >= nRanks || ops[i].srcRank >= nRanks || ops[i].dstBuf >= NBUF || ops[i].srcBuf >= NBUF ||
            ops[i].kind > 1)
            return HCCL_E_PARA;

    /* 1. the expected result ranges, and how far every buffer (input, output, communication buffer, user input,
     *    user output of every rank) is used */
    const uint32_t nbuf = NBUF * nRanks;
    IMap* im = (IMap*)calloc(nbuf, sizeof(IMap));
    uint64_t* extent = (uint64_t*)calloc(nbuf, sizeof(uint64_t));
    Cell* tmp = NULL;
    size_t tmp_cap = 0;
    int rc = (im && extent) ? HCCL_SUCCESS : HCCL_E_MEMORY;
#define IM(rank, buf) im[(size_t)(rank) * NBUF + (buf)]
#define EXT(rank, buf) extent[(size_t)(rank) * NBUF + (buf)]
    HcommGfxSlice sl[HCOMM_GFX_MAX_RANKS];
    HcommGfxCalcSlices(count, unitSize, nRanks, sl);
    uint64_t res_lo[HCOMM_GFX_MAX_RANKS], res_hi[HCOMM_GFX_MAX_RANKS], res_origin[HCOMM_GFX_MAX_RANKS];
    uint32_t res_buf = user ? HCOMM_GFX_BUF_USER_OUT : 1u;
    for (uint32_t r = 0; r < nRanks && rc == HCCL_SUCCESS; ++r) {
        res_lo[r] = 0;
        res_hi[r] = total;
        res_origin[r] = 0;
        if (expect == HCOMM_GFX_EXPECT_REDUCE_SCATTER_IN_PLACE) {
            res_buf = 0;
            res_lo[r] = sl[r].offset;
            res_hi[r] = sl[r].offset + sl[r].size;
        } else if (expect == HCOMM_GFX_EXPECT_REDUCE_SCATTER_OUT || expect == HCOMM_GFX_EXPECT_REDUCE_SCATTER_USER) {
            res_origin[r] = (uint64_t)r * strideCount * unitSize; /* out[r][x] comes from everybody's in[..][origin + x] */
        }
        if (res_hi[r] > EXT(r, res_buf)) EXT(r, res_buf) = res_hi[r];
    }
    for (uint64_t i = 0; i < nOps && rc == HCCL_SUCCESS; ++i) {
        const HcommGfxSchedOp* o = &ops[i];
        if (o->dstOff + o->bytes > EXT(o->rank, o->dstBuf)) EXT(o->rank, o->dstBuf) = o->dstOff + o->bytes;
        if (o->srcOff + o->bytes > EXT(o->srcRank, o->srcBuf)) EXT(o->srcRank, o->srcBuf) = o->srcOff + o->bytes;
    }
    for (uint32_t r = 0; r < nRanks && rc == HCCL_SUCCESS; ++r)
        for (uint32_t buf = 0; buf < NBUF && rc == HCCL_SUCCESS; ++buf)
            if (imap_init(&IM(r, buf), EXT(r, buf) ? EXT(r, buf) : 1, nRanks, buf == data_buf ? (int)r : -1) < 0)
                rc = HCCL_E_MEMORY;

    /* 2. replay step by step */
    for (uint64_t i = 0; i < nOps && rc == HCCL_SUCCESS;) {
        uint64_t j = i;
        while (j < nOps && ops[j].step == ops[i].step) ++j;
        for (uint64_t a = i; a < j; ++a)
            for (uint64_t b = i; b < j; ++b) {
                if (a == b || ops[a].bytes == 0 || ops[b].bytes == 0) continue;
                const HcommGfxSchedOp *x = &ops[a], *y = &ops[b];
                if (x->rank == y->rank && x->dstBuf == y->dstBuf && a < b &&
                    ranges_overlap(x->dstOff, x->bytes, y->dstOff, y->bytes))
                    report(rep, 1, "step %llu: two operations write overlapping ranges of rank %llu (offset %llu)", x->step, x->rank, x->dstOff);
                if (x->rank == y->srcRank && x->dstBuf == y->srcBuf && ranges_overlap(x->dstOff, x->bytes, y->srcOff, y->bytes))
                    report(rep, 1, "step %llu: rank %llu writes a range (offset %llu) another operation of the step reads", x->step, x->rank, x->dstOff);
            }
        for (uint64_t a = i; a < j && rc == HCCL_SUCCESS; ++a) {
            const HcommGfxSchedOp* o = &ops[a];
            if (o->bytes == 0) continue;
            IMap* sm = &IM(o->srcRank, o->srcBuf);
            IMap* dm = &IM(o->rank, o->dstBuf);
            /* cut both ranges at their ends and at each other's inner cuts (twice: a cut mirrored into a map that is
             * both source and destination may itself need mirroring) */
            if (imap_cut(sm, o->srcOff) < 0 || imap_cut(sm, o->srcOff + o->bytes) < 0 || imap_cut(dm, o->dstOff) < 0 ||
                imap_cut(dm, o->dstOff + o->bytes) < 0)
                rc = HCCL_E_MEMORY;
            for (int pass = 0; pass < 2 && rc == HCCL_SUCCESS; ++pass)
                if (imap_mirror_cuts(sm, o->srcOff, o->bytes, dm, o->dstOff) < 0 ||
                    imap_mirror_cuts(dm, o->dstOff, o->bytes, sm, o->srcOff) < 0)
                    rc = HCCL_E_MEMORY;
            if (rc != HCCL_SUCCESS) break;
            const size_t s0 = (size_t)imap_cut(sm, o->srcOff), s1 = (size_t)imap_cut(sm, o->srcOff + o->bytes);
            const size_t d0 = (size_t)imap_cut(dm, o->dstOff), d1 = (size_t)imap_cut(dm, o->dstOff + o->bytes);
            const size_t m = s1 - s0;
            if (d1 - d0 != m) { /* only when the operation's own source and destination overlap */
                report(rep, 1, "step %llu: an operation of rank %llu reads what it writes (offset %llu)", o->step, o->rank, o->dstOff);
                continue;
            }
            if (m > tmp_cap) {
                Cell* q = (Cell*)realloc(tmp, m * sizeof(Cell));
                if (!q) {
                    rc = HCCL_E_MEMORY;
                    break;
                }
                tmp = q;
                tmp_cap = m;
            }
            const int64_t shift = (int64_t)o->srcOff - (int64_t)o->dstOff;
            for (size_t k = 0; k < m; ++k) tmp[k] = CELL(sm, s0 + k); /* the value before this operation */
            for (size_t k = 0; k < m; ++k) {
                Cell* d = &CELL(dm, d0 + k);
                Cell s = tmp[k];
                for (uint32_t q = 0; q < nRanks; ++q)
                    if (s.cnt[q]) s.delta[q] += shift;
                if (o->kind == 0) {
                    *d = s;
                } else {
                    for (uint32_t q = 0; q < nRanks; ++q) {
                        if (!s.cnt[q]) continue;
                        if (d->cnt[q] && d->delta[q] != s.delta[q]) d->bad = 1;
                        if (!d->cnt[q]) d->delta[q] = s.delta[q];
                        d->cnt[q] = (uint8_t)(d->cnt[q] + s.cnt[q] > 255 ? 255 : d->cnt[q] + s.cnt[q]);
                    }
                    d->bad |= s.bad;
                }
            }
        }
        i = j;
    }

    /* 3. the expected result ranges */
    for (uint32_t r = 0; r < nRanks && rc == HCCL_SUCCESS; ++r) {
        if (res_hi[r] <= res_lo[r]) continue;
        IMap* m = &IM(r, res_buf);
        const long i0 = imap_cut(m, res_lo[r]), i1 = imap_cut(m, res_hi[r]);
        if (i0 < 0 || i1 < 0) {
            rc = HCCL_E_MEMORY;
            break;
        }
        for (size_t iv = (size_t)i0; iv < (size_t)i1; ++iv) {
            const Cell* c = &CELL(m, iv);
            if (c->bad) report(rep, 0, "result of rank %llu at offset %llu mixes one rank's data from two different offsets (buffer %llu)", r, m->b[iv], res_buf);
            for (uint32_t q = 0; q < nRanks; ++q) {
                if (c->cnt[q] != 1)
                    report(rep, 0, "result of rank %llu at offset %llu holds rank %llu's data a wrong number of times", r, m->b[iv], q);
                else if (c->delta[q] != (int64_t)res_origin[r])
                    report(rep, 0, "result of rank %llu at offset %llu took rank %llu's data from a different offset", r, m->b[iv], q);
            }
        }
    }
#undef IM
#undef EXT
    free(tmp);
    if (im)
        for (uint32_t q = 0; q < nbuf; ++q) {
            free(im[q].b);
            free(im[q].ix);
            free(im[q].pool);
        }
    free(im);
    free(extent);
    return rc;
}

int32_t HcommGfxScheduleCheck(
    HcommGfxAlgorithm alg, uint32_t nRanks, uint64_t count, uint64_t strideCount, HcommDataType dataType,
    HcommGfxCheckReport* rep)
{
    if (!rep) return HCCL_E_PTR;
    HgOpList l;
    int rc = hg_schedule(&l, (int)alg, nRanks, count, strideCount, (int)dataType);
    if (rc != HCCL_SUCCESS) return rc;
    HcommGfxExpectation e = HCOMM_GFX_EXPECT_ALLREDUCE;
    if (alg == HCOMM_GFX_ALG_REDUCE_SCATTER_RING) e = HCOMM_GFX_EXPECT_REDUCE_SCATTER_IN_PLACE;
    if (alg == HCOMM_GFX_ALG_REDUCE_SCATTER_MESH || alg == HCOMM_GFX_ALG_REDUCE_SCATTER_RING_STANDALONE ||
        alg == HCOMM_GFX_ALG_REDUCE_SCATTER_NHR || alg == HCOMM_GFX_ALG_REDUCE_SCATTER_NB ||
        alg == HCOMM_GFX_ALG_REDUCE_SCATTER_LOCAL_REDUCE || alg == HCOMM_GFX_ALG_REDUCE_SCATTER_WINDOW_HALVING)
        e = HCOMM_GFX_EXPECT_REDUCE_SCATTER_OUT;
    rc = HcommGfxOpListCheck(l.ops, l.n, nRanks, e, count, strideCount, HcommGfxDataTypeSize(dataType), rep);
    hg_oplist_free(&l);
    return rc;
}

int32_t HcommGfxOpBaseCheck(
    HcommGfxAlgorithm alg, uint32_t nRanks, uint64_t count, uint64_t cclBytes, HcommDataType dataType,
    HcommGfxCheckReport* rep)
{
    if (!rep) return HCCL_E_PTR;
    HgOpList l;
    int rc = hg_schedule_opbase(&l, (int)alg, nRanks, count, cclBytes, (int)dataType);
    if (rc != HCCL_SUCCESS) return rc;
    HcommGfxExpectation e = HCOMM_GFX_EXPECT_ALLREDUCE_USER;
    if (alg == HCOMM_GFX_ALG_REDUCE_SCATTER_MESH || alg == HCOMM_GFX_ALG_REDUCE_SCATTER_RING_STANDALONE ||
        alg == HCOMM_GFX_ALG_REDUCE_SCATTER_NHR || alg == HCOMM_GFX_ALG_REDUCE_SCATTER_NB ||
        alg == HCOMM_GFX_ALG_REDUCE_SCATTER_LOCAL_REDUCE)
        e = HCOMM_GFX_EXPECT_REDUCE_SCATTER_USER;
    rc = HcommGfxOpListCheck(l.ops, l.n, nRanks, e, count, 0, HcommGfxDataTypeSize(dataType), rep);
    hg_oplist_free(&l);
    return rc;
}

int32_t HcommGfxHierCheck(
    HcommGfxAlgorithm level1Alg, uint32_t nServers, uint32_t nLocal, uint64_t count, HcommDataType dataType,
    HcommGfxCheckReport* rep)
{
    if (!rep) return HCCL_E_PTR;
    HgOpList l;
    int rc = hg_schedule_hier(&l, 0, (int)level1Alg, nServers, nLocal, count, (int)dataType);
    if (rc != HCCL_SUCCESS) return rc;
    rc = HcommGfxOpListCheck(l.ops, l.n, nServers * nLocal, HCOMM_GFX_EXPECT_ALLREDUCE, count, 0,
                             HcommGfxDataTypeSize(dataType), rep);
    hg_oplist_free(&l);
    return rc;
}

int32_t HcommGfxMeshHierCheck(
    HcommGfxAlgorithm level1Alg, uint32_t nServers, uint32_t nLocal, uint64_t count, HcommDataType dataType,
    HcommGfxCheckReport* rep)
{
    if (!rep) return HCCL_E_PTR;
    HgOpList l;
    int rc = hg_schedule_hier(&l, 1, (int)level1Alg, nServers, nLocal, count, (int)dataType);
    if (rc != HCCL_SUCCESS) return rc;
    rc = HcommGfxOpListCheck(l.ops, l.n, nServers * nLocal, HCOMM_GFX_EXPECT_ALLREDUCE, count, 0,
                             HcommGfxDataTypeSize(dataType), rep);
    hg_oplist_free(&l);
    return rc;
}

int32_t HcommGfxDoubleRingCheck(
    HcommGfxAlgorithm level1Alg, uint32_t nServers, uint32_t nLocal, uint64_t count, uint64_t cclBytes,
    HcommDataType dataType, HcommGfxCheckReport* rep)
{
    if (!rep) return HCCL_E_PTR;
    HgOpList l;
    int rc = hg_schedule_dbring(&l, (int)level1Alg, nServers, nLocal, count, cclBytes, (int)dataType);
    if (rc != HCCL_SUCCESS) return rc;
    rc = HcommGfxOpListCheck(l.ops, l.n, nServers * nLocal, HCOMM_GFX_EXPECT_ALLREDUCE_USER, count, 0,
                             HcommGfxDataTypeSize(dataType), rep);
    hg_oplist_free(&l);
    return rc;
}

int32_t HcommGfxOrderPreservedCheck(
    uint32_t nRanks, uint64_t count, uint64_t cclBytes, HcommDataType dataType, HcommGfxCheckReport* rep)
{
    if (!rep) return HCCL_E_PTR;
    HgOpList l;
    int rc = hg_schedule_order_preserved(&l, nRanks, count, cclBytes, (int)dataType);
    if (rc != HCCL_SUCCESS) return rc;
    rc = HcommGfxOpListCheck(l.ops, l.n, nRanks, HCOMM_GFX_EXPECT_REDUCE_SCATTER_USER, count, 0,
                             HcommGfxDataTypeSize(dataType), rep);
    hg_oplist_free(&l);
    return rc;
}

int32_t HcommGfxOrderPreservedAllReduceCheck(
    uint32_t nRanks, uint64_t count, uint64_t cclBytes, HcommDataType dataType, HcommGfxCheckReport* rep)
{
    if (!rep) return HCCL_E_PTR;
    HgOpList l;
    int rc = hg_schedule_order_preserved_ar(&l, nRanks, count, cclBytes, (int)dataType);
    if (rc != HCCL_SUCCESS) return rc;
    rc = HcommGfxOpListCheck(l.ops, l.n, nRanks, HCOMM_GFX_EXPECT_ALLREDUCE_USER, count, 0,
                             HcommGfxDataTypeSize(dataType), rep);
    hg_oplist_free(&l);
    return rc;
}

int32_t HcommGfxOrderPreservedHierAllReduceCheck(
    HcommGfxAlgorithm level1Alg, uint32_t nServers, uint32_t nLocal, uint64_t count, uint64_t cclBytes,
    HcommDataType dataType, HcommGfxCheckReport* rep)
{
    if (!rep) return HCCL_E_PTR;
    HgOpList l;
    int rc = hg_schedule_order_preserved_ar2(&l, (int)level1Alg, nServers, nLocal, count, cclBytes, (int)dataType);
    if (rc != HCCL_SUCCESS) return rc;
    rc = HcommGfxOpListCheck(l.ops, l.n, nServers * nLocal, HCOMM_GFX_EXPECT_ALLREDUCE_USER, count, 0,
                             HcommGfxDataTypeSize(dataType), rep);
    hg_oplist_free(&l);
    return rc;
}

int32_t HcommGfxOrderPreservedHierReduceScatterCheck(
    uint32_t nServers, uint32_t nLocal, uint64_t count, uint64_t cclBytes, HcommDataType dataType, HcommGfxCheckReport* rep)
{
    if (!rep) return HCCL_E_PTR;
    HgOpList l;
    int rc = hg_schedule_order_preserved_rs2(&l, nServers, nLocal, count, cclBytes, (int)dataType);
    if (rc != HCCL_SUCCESS) return rc;
    rc = HcommGfxOpListCheck(l.ops, l.n, nServers * nLocal, HCOMM_GFX_EXPECT_REDUCE_SCATTER_USER, count, 0,
                             HcommGfxDataTypeSize(dataType), rep);
    hg_oplist_free(&l);
    return rc;
}

int32_t HcommGfxOrderPreservedSmallCheck(
    uint32_t nRanks, uint64_t count, uint64_t cclBytes, HcommDataType dataType, HcommGfxCheckReport* rep)
{
    if (!rep) return HCCL_E_PTR;
    HgOpList l;
    int rc = hg_schedule_order_preserved_small(&l, nRanks, count, cclBytes, (int)dataType);
    if (rc != HCCL_SUCCESS) return rc;
    rc = HcommGfxOpListCheck(l.ops, l.n, nRanks, HCOMM_GFX_EXPECT_REDUCE_SCATTER_USER, count, 0,
                             HcommGfxDataTypeSize(dataType), rep);
    hg_oplist_free(&l);
    return rc;
}

int32_t HcommGfxHierReduceScatterCheck(
    int32_t level0Mesh, HcommGfxAlgorithm level1Alg, uint32_t nServers, uint32_t nLocal, uint64_t count, uint64_t cclBytes,
    HcommDataType dataType, HcommGfxCheckReport* rep)
{
    if (!rep) return HCCL_E_PTR;
    HgOpList l;
    int rc = hg_schedule_hier_rs(&l, level0Mesh != 0, (int)level1Alg, nServers, nLocal, count, cclBytes, (int)dataType);
    if (rc != HCCL_SUCCESS) return rc;
    rc = HcommGfxOpListCheck(l.ops, l.n, nServers * nLocal, HCOMM_GFX_EXPECT_REDUCE_SCATTER_USER, count, 0,
                             HcommGfxDataTypeSize(dataType), rep);
    hg_oplist_free(&l);
    return rc;
}

int32_t HcommGfxDoubleRingHierReduceScatterCheck(
    HcommGfxAlgorithm level1Alg, HcommGfxAlgorithm level2Alg, uint32_t nPods, uint32_t nServers, uint32_t nLocal, uint64_t count,
    uint64_t cclBytes, HcommDataType dataType, HcommGfxCheckReport* rep)
{
    if (!rep) return HCCL_E_PTR;
    HgOpList l;
    int rc = hg_schedule_dbring_rs_servers(&l, (int)level1Alg, (int)level2Alg, nPods, nServers, nLocal, count, cclBytes, (int)dataType);
    if (rc != HCCL_SUCCESS) return rc;
    rc = HcommGfxOpListCheck(l.ops, l.n, nPods * nServers * nLocal, HCOMM_GFX_EXPECT_REDUCE_SCATTER_USER, count, 0,
                             HcommGfxDataTypeSize(dataType), rep);
    hg_oplist_free(&l);
    return rc;
}

int32_t HcommGfxDoubleRingReduceScatterCheck(
    uint32_t nRanks, uint64_t count, uint64_t cclBytes, HcommDataType dataType, HcommGfxCheckReport* rep)
{
    if (!rep) return HCCL_E_PTR;
    HgOpList l;
    int rc = hg_schedule_dbring_rs(&l, nRanks, count, cclBytes, (int)dataType);
    if (rc != HCCL_SUCCESS) return rc;
    rc = HcommGfxOpListCheck(l.ops, l.n, nRanks, HCOMM_GFX_EXPECT_REDUCE_SCATTER_USER, count, 0,
                             HcommGfxDataTypeSize(dataType), rep);
    hg_oplist_free(&l);
    return rc;
}
