/*
 * hg_check.c - symbolic checker for schedule op lists.
 *
 * A miniature of the reference's algorithm checker (test/st/algorithm/README_en.md:13-15,202-231): no data is
 * moved; every byte range of every rank buffer carries the set of (rank, origin offset) contributions folded
 * into it.  Each buffer is cut into intervals at the ends of the ranges operations touch in it, and at the images
 * of those cuts under the operations' source <-> destination translations, so that one operation always maps whole
 * intervals onto whole intervals.  Two verdicts:
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

typedef struct {
    uint8_t cnt[HCOMM_GFX_MAX_RANKS];   /* how many times rank k's data is folded in */
    int64_t delta[HCOMM_GFX_MAX_RANKS]; /* origin offset - current offset of that contribution */
    uint8_t bad;                        /* contributions of one rank from two different origins were mixed */
} Cell;

typedef struct {
    uint64_t* b; /* sorted, unique interval boundaries */
    size_t n, cap;
} Bounds;

static int bounds_add(Bounds* s, uint64_t v)
{
    size_t lo = 0, hi = s->n;
    while (lo < hi) {
        size_t mid = (lo + hi) / 2;
        if (s->b[mid] < v) lo = mid + 1; else hi = mid;
    }
    if (lo < s->n && s->b[lo] == v) return 0;
    if (s->n == s->cap) {
        size_t cap = s->cap ? s->cap * 2 : 64;
        uint64_t* p = (uint64_t*)realloc(s->b, cap * sizeof(uint64_t));
        if (!p) return -1;
        s->b = p;
        s->cap = cap;
    }
    memmove(&s->b[lo + 1], &s->b[lo], (s->n - lo) * sizeof(uint64_t));
    s->b[lo] = v;
    s->n++;
    return 1;
}

static size_t bounds_find(const Bounds* s, uint64_t v)
{
    size_t lo = 0, hi = s->n;
    while (lo < hi) {
        size_t mid = (lo + hi) / 2;
        if (s->b[mid] < v) lo = mid + 1; else hi = mid;
    }
    return lo; /* v is always present when this is called */
}

static void report(HcommGfxCheckReport* r, int is_conflict, const char* fmt, uint64_t a, uint64_t b, uint64_t c)
{
    if (is_conflict) r->conflicts++; else r->semanticErrors++;
    if (r->message[0] == 0) snprintf(r->message, sizeof(r->message), fmt, (unsigned long long)a, (unsigned long long)b, (unsigned long long)c);
}

static int ranges_overlap(uint64_t a, uint64_t an, uint64_t b, uint64_t bn) { return a < b + bn && b < a + an; }

#define MAX_BOUNDS_PER_BUFFER (1u << 20)

/* Copy the boundaries of `from` that lie strictly inside (lo, lo + len) into `to`, moved by to_off - lo.
 * Returns 1 when `to` grew, 0 when not, -1 when out of memory. */
static int translate_bounds(const Bounds* from, uint64_t lo, uint64_t len, Bounds* to, uint64_t to_off)
{
    size_t k0 = bounds_find(from, lo + 1), k1 = bounds_find(from, lo + len);
    if (k1 <= k0) return 0;
    const size_t m = k1 - k0;
    uint64_t* v = (uint64_t*)malloc(m * sizeof(uint64_t)); /* `to` may be `from` itself: take a snapshot first */
    if (!v) return -1;
    memcpy(v, &from->b[k0], m * sizeof(uint64_t));
    int grew = 0;
    for (size_t k = 0; k < m; ++k) {
        const int a = bounds_add(to, v[k] - lo + to_off);
        if (a < 0 || to->n > MAX_BOUNDS_PER_BUFFER) {
            free(v);
            return -1;
        }
        grew |= a;
    }
    free(v);
    return grew;
}

int32_t HcommGfxOpListCheck(
    const HcommGfxSchedOp* ops, uint64_t nOps, uint32_t nRanks, HcommGfxExpectation expect, uint64_t count,
    uint64_t strideCount, uint32_t unitSize, HcommGfxCheckReport* rep)
{
    if (!rep) return HCCL_E_PTR;
    memset(rep, 0, sizeof(*rep));
    if (nOps && !ops) return HCCL_E_PTR;
    if (nRanks == 0 || nRanks > HCOMM_GFX_MAX_RANKS || unitSize == 0) return HCCL_E_PARA;
    if (expect != HCOMM_GFX_EXPECT_ALLREDUCE && expect != HCOMM_GFX_EXPECT_REDUCE_SCATTER_IN_PLACE &&
        expect != HCOMM_GFX_EXPECT_REDUCE_SCATTER_OUT)
        return HCCL_E_PARA;
    if (strideCount == 0) strideCount = count;
    const uint64_t total = count * unitSize;
    for (uint64_t i = 0; i < nOps; ++i)
        if (ops[i].rank >= nRanks || ops[i].srcRank >= nRanks || ops[i].dstBuf > 2 || ops[i].srcBuf > 2 || ops[i].kind > 1)
            return HCCL_E_PARA;

    /* 1. interval boundaries, one set per rank buffer (input, output, communication buffer), closed under the
     *    translations the operations perform between their source and destination buffers */
    const uint32_t nbuf = 3 * nRanks;
    Bounds* bs = (Bounds*)calloc(nbuf, sizeof(Bounds));
    size_t* first = (size_t*)calloc((size_t)nbuf + 1, sizeof(size_t));
    Cell *st = NULL, *tmp = NULL;
    int rc = (bs && first) ? HCCL_SUCCESS : HCCL_E_MEMORY;
#define BS(rank, buf) bs[(size_t)(rank) * 3 + (buf)]
    HcommGfxSlice sl[HCOMM_GFX_MAX_RANKS];
    HcommGfxCalcSlices(count, unitSize, nRanks, sl);
    uint64_t res_lo[HCOMM_GFX_MAX_RANKS], res_hi[HCOMM_GFX_MAX_RANKS], res_origin[HCOMM_GFX_MAX_RANKS];
    uint32_t res_buf = 1;
    for (uint32_t r = 0; r < nRanks && rc == HCCL_SUCCESS; ++r) { /* the expected result ranges */
        res_lo[r] = 0;
        res_hi[r] = total;
        res_origin[r] = 0;
        if (expect == HCOMM_GFX_EXPECT_REDUCE_SCATTER_IN_PLACE) {
            res_buf = 0;
            res_lo[r] = sl[r].offset;
            res_hi[r] = sl[r].offset + sl[r].size;
        } else if (expect == HCOMM_GFX_EXPECT_REDUCE_SCATTER_OUT) {
            res_origin[r] = (uint64_t)r * strideCount * unitSize; /* out[r][x] comes from everybody's in[..][origin + x] */
        }
        if (bounds_add(&BS(r, res_buf), res_lo[r]) < 0 || bounds_add(&BS(r, res_buf), res_hi[r]) < 0) rc = HCCL_E_MEMORY;
    }
    for (uint64_t i = 0; i < nOps && rc == HCCL_SUCCESS; ++i) {
        const HcommGfxSchedOp* o = &ops[i];
        if (bounds_add(&BS(o->rank, o->dstBuf), o->dstOff) < 0 || bounds_add(&BS(o->rank, o->dstBuf), o->dstOff + o->bytes) < 0 ||
            bounds_add(&BS(o->srcRank, o->srcBuf), o->srcOff) < 0 || bounds_add(&BS(o->srcRank, o->srcBuf), o->srcOff + o->bytes) < 0)
            rc = HCCL_E_MEMORY;
    }
    for (int changed = 1; changed && rc == HCCL_SUCCESS;) {
        changed = 0;
        for (uint64_t i = 0; i < nOps && rc == HCCL_SUCCESS; ++i) {
            const HcommGfxSchedOp* o = &ops[i];
            if (o->bytes == 0) continue;
            Bounds* s = &BS(o->srcRank, o->srcBuf);
            Bounds* d = &BS(o->rank, o->dstBuf);
            const int a = translate_bounds(s, o->srcOff, o->bytes, d, o->dstOff);
            const int b = a < 0 ? -1 : translate_bounds(d, o->dstOff, o->bytes, s, o->srcOff);
            if (a < 0 || b < 0) rc = HCCL_E_MEMORY;
            else if (a || b) changed = 1;
        }
    }

    /* 2. state: one cell per interval of every buffer */
    size_t ncell = 0, widest = 1;
    for (uint32_t q = 0; q < nbuf && rc == HCCL_SUCCESS; ++q) {
        first[q] = ncell;
        const size_t ni = bs[q].n ? bs[q].n - 1 : 0;
        ncell += ni;
        if (ni > widest) widest = ni;
    }
    if (rc == HCCL_SUCCESS) {
        first[nbuf] = ncell;
        st = (Cell*)calloc(ncell ? ncell : 1, sizeof(Cell));
        tmp = (Cell*)calloc(widest, sizeof(Cell));
        if (!st || !tmp) rc = HCCL_E_MEMORY;
    }
    if (rc != HCCL_SUCCESS) goto done;
#define CELL(rank, buf, iv) st[first[(size_t)(rank) * 3 + (buf)] + (iv)]
    for (uint32_t r = 0; r < nRanks; ++r)
        for (uint32_t buf = 0; buf < 3; ++buf) {
            const size_t ni = first[(size_t)r * 3 + buf + 1] - first[(size_t)r * 3 + buf];
            for (size_t iv = 0; iv < ni; ++iv) {
                for (uint32_t k = 0; k < nRanks; ++k) CELL(r, buf, iv).delta[k] = NO_DELTA;
                if (buf == 0) { /* an input holds its own rank's data from the same offset */
                    CELL(r, 0, iv).cnt[r] = 1;
                    CELL(r, 0, iv).delta[r] = 0;
                }
            }
        }

    /* 3. replay step by step */
    for (uint64_t i = 0; i < nOps;) {
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
        for (uint64_t a = i; a < j; ++a) {
            const HcommGfxSchedOp* o = &ops[a];
            if (o->bytes == 0) continue;
            const Bounds* sb = &BS(o->srcRank, o->srcBuf);
            const Bounds* db = &BS(o->rank, o->dstBuf);
            const size_t s0 = bounds_find(sb, o->srcOff), s1 = bounds_find(sb, o->srcOff + o->bytes);
            const size_t d0 = bounds_find(db, o->dstOff);
            const int64_t shift = (int64_t)o->srcOff - (int64_t)o->dstOff;
            /* closure makes the two ranges cut at the same relative positions: s1 - s0 intervals on both sides */
            for (size_t k = 0; k < s1 - s0; ++k) tmp[k] = CELL(o->srcRank, o->srcBuf, s0 + k); /* pre-step value */
            for (size_t k = 0; k < s1 - s0; ++k) {
                Cell* d = &CELL(o->rank, o->dstBuf, d0 + k);
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

    /* 4. the expected result ranges */
    for (uint32_t r = 0; r < nRanks; ++r) {
        if (res_hi[r] <= res_lo[r]) continue;
        const Bounds* b = &BS(r, res_buf);
        const size_t i0 = bounds_find(b, res_lo[r]), i1 = bounds_find(b, res_hi[r]);
        for (size_t iv = i0; iv < i1; ++iv) {
            const Cell* c = &CELL(r, res_buf, iv);
            if (c->bad) report(rep, 0, "result of rank %llu at offset %llu mixes one rank's data from two different offsets (buffer %llu)", r, b->b[iv], res_buf);
            for (uint32_t q = 0; q < nRanks; ++q) {
                if (c->cnt[q] != 1)
                    report(rep, 0, "result of rank %llu at offset %llu holds rank %llu's data a wrong number of times", r, b->b[iv], q);
                else if (c->delta[q] != (int64_t)res_origin[r])
                    report(rep, 0, "result of rank %llu at offset %llu took rank %llu's data from a different offset", r, b->b[iv], q);
            }
        }
    }
#undef CELL
#undef BS
done:
    free(st);
    free(tmp);
    if (bs)
        for (uint32_t q = 0; q < nbuf; ++q) free(bs[q].b);
    free(bs);
    free(first);
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
        alg == HCOMM_GFX_ALG_REDUCE_SCATTER_LOCAL_REDUCE)
        e = HCOMM_GFX_EXPECT_REDUCE_SCATTER_OUT;
    rc = HcommGfxOpListCheck(l.ops, l.n, nRanks, e, count, strideCount, HcommGfxDataTypeSize(dataType), rep);
    hg_oplist_free(&l);
    return rc;
}
