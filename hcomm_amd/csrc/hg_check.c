/*
 * hg_check.c - symbolic checker for schedule op lists.
 *
 * A miniature of the reference's algorithm checker (test/st/algorithm/README_en.md:13-15,202-231): no data is
 * moved; every byte range of every rank buffer carries the set of (rank, origin offset) contributions folded
 * into it.  Two verdicts:
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

int32_t HcommGfxOpListCheck(
    const HcommGfxSchedOp* ops, uint64_t nOps, uint32_t nRanks, HcommGfxExpectation expect, uint64_t count,
    uint64_t strideCount, uint32_t unitSize, HcommGfxCheckReport* rep)
{
    if (!rep) return HCCL_E_PTR;
    memset(rep, 0, sizeof(*rep));
    if (nOps && !ops) return HCCL_E_PTR;
    if (nRanks == 0 || nRanks > HCOMM_GFX_MAX_RANKS || unitSize == 0) return HCCL_E_PARA;
    if (strideCount == 0) strideCount = count;
    const uint64_t total = count * unitSize;
    for (uint64_t i = 0; i < nOps; ++i)
        if (ops[i].rank >= nRanks || ops[i].srcRank >= nRanks || ops[i].dstBuf > 2 || ops[i].srcBuf > 2 || ops[i].kind > 1)
            return HCCL_E_PARA;

    /* 1. interval boundaries, closed under the translations the operations perform */
    Bounds bs = {0};
    int rc = HCCL_SUCCESS;
    HcommGfxSlice sl[HCOMM_GFX_MAX_RANKS];
    HcommGfxCalcSlices(count, unitSize, nRanks, sl);
    if (bounds_add(&bs, 0) < 0 || bounds_add(&bs, total) < 0) rc = HCCL_E_MEMORY;
    for (uint32_t r = 0; r < nRanks && rc == HCCL_SUCCESS; ++r) {
        if (bounds_add(&bs, sl[r].offset) < 0 || bounds_add(&bs, sl[r].offset + sl[r].size) < 0) rc = HCCL_E_MEMORY;
        if (bounds_add(&bs, (uint64_t)r * strideCount * unitSize) < 0 ||
            bounds_add(&bs, (uint64_t)r * strideCount * unitSize + total) < 0) rc = HCCL_E_MEMORY;
    }
    for (uint64_t i = 0; i < nOps && rc == HCCL_SUCCESS; ++i) {
        if (bounds_add(&bs, ops[i].dstOff) < 0 || bounds_add(&bs, ops[i].dstOff + ops[i].bytes) < 0 ||
            bounds_add(&bs, ops[i].srcOff) < 0 || bounds_add(&bs, ops[i].srcOff + ops[i].bytes) < 0) rc = HCCL_E_MEMORY;
    }
    for (int changed = 1, guard = 0; changed && rc == HCCL_SUCCESS && guard < 64; ++guard) {
        changed = 0;
        for (uint64_t i = 0; i < nOps && rc == HCCL_SUCCESS; ++i) {
            const HcommGfxSchedOp* o = &ops[i];
            if (o->dstOff == o->srcOff) continue;
            for (size_t k = 0; k < bs.n; ++k) {
                const uint64_t v = bs.b[k];
                int a = 0, b = 0;
                if (v > o->srcOff && v < o->srcOff + o->bytes) a = bounds_add(&bs, v - o->srcOff + o->dstOff);
                if (v > o->dstOff && v < o->dstOff + o->bytes) b = bounds_add(&bs, v - o->dstOff + o->srcOff);
                if (a < 0 || b < 0) { rc = HCCL_E_MEMORY; break; }
                if (a > 0 || b > 0) changed = 1;
            }
        }
    }
    if (rc != HCCL_SUCCESS) { free(bs.b); return rc; }

    /* 2. state: 3 buffers per rank (input, output, communication buffer) x intervals */
    const size_t ni = bs.n - 1;
    Cell* st = (Cell*)calloc((size_t)3 * nRanks * (ni ? ni : 1), sizeof(Cell));
    Cell* tmp = (Cell*)calloc(ni ? ni : 1, sizeof(Cell));
    if (!st || !tmp) { free(st); free(tmp); free(bs.b); return HCCL_E_MEMORY; }
#define CELL(rank, buf, iv) st[((size_t)(rank) * 3 + (buf)) * ni + (iv)]
    for (uint32_t r = 0; r < nRanks; ++r)
        for (size_t iv = 0; iv < ni; ++iv) {
            for (uint32_t k = 0; k < nRanks; ++k) {
                CELL(r, 0, iv).delta[k] = NO_DELTA;
                CELL(r, 1, iv).delta[k] = NO_DELTA;
                CELL(r, 2, iv).delta[k] = NO_DELTA;
            }
            CELL(r, 0, iv).cnt[r] = 1; /* an input holds its own rank's data from the same offset */
            CELL(r, 0, iv).delta[r] = 0;
        }

    /* 3. replay step by step */
    uint64_t i = 0;
    while (i < nOps) {
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
            const size_t s0 = bounds_find(&bs, o->srcOff), s1 = bounds_find(&bs, o->srcOff + o->bytes);
            const size_t d0 = bounds_find(&bs, o->dstOff);
            const int64_t shift = (int64_t)o->srcOff - (int64_t)o->dstOff;
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
        uint64_t lo = 0, hi = total, origin = 0;
        uint32_t buf = 1;
        if (expect == HCOMM_GFX_EXPECT_REDUCE_SCATTER_IN_PLACE) {
            buf = 0;
            lo = sl[r].offset;
            hi = sl[r].offset + sl[r].size;
        } else if (expect == HCOMM_GFX_EXPECT_REDUCE_SCATTER_OUT) {
            origin = (uint64_t)r * strideCount * unitSize; /* out[r][x] comes from everybody's in[..][origin + x] */
        } else if (expect != HCOMM_GFX_EXPECT_ALLREDUCE) {
            rc = HCCL_E_PARA;
            break;
        }
        if (hi <= lo) continue;
        const size_t i0 = bounds_find(&bs, lo), i1 = bounds_find(&bs, hi);
        for (size_t iv = i0; iv < i1; ++iv) {
            const Cell* c = &CELL(r, buf, iv);
            if (c->bad) report(rep, 0, "result of rank %llu at offset %llu mixes one rank's data from two different offsets (buffer %llu)", r, bs.b[iv], buf);
            for (uint32_t q = 0; q < nRanks; ++q) {
                if (c->cnt[q] != 1)
                    report(rep, 0, "result of rank %llu at offset %llu holds rank %llu's data a wrong number of times", r, bs.b[iv], q);
                else if (c->delta[q] != (int64_t)origin)
                    report(rep, 0, "result of rank %llu at offset %llu took rank %llu's data from a different offset", r, bs.b[iv], q);
            }
        }
    }
#undef CELL
    free(st);
    free(tmp);
    free(bs.b);
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
        alg == HCOMM_GFX_ALG_REDUCE_SCATTER_NHR || alg == HCOMM_GFX_ALG_REDUCE_SCATTER_NB)
        e = HCOMM_GFX_EXPECT_REDUCE_SCATTER_OUT;
    rc = HcommGfxOpListCheck(l.ops, l.n, nRanks, e, count, strideCount, HcommGfxDataTypeSize(dataType), rep);
    hg_oplist_free(&l);
    return rc;
}
