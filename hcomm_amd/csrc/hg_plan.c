/*
 * hg_plan.c - lowering a schedule to a fixed list of kernel launches ("prepare once, run many", the
 * Prepare / RunAsync split of the reference's templates,
 * src/legacy/ascend910/algorithm/base/alg_template/alg_template_base_pub.h:237-253).
 *
 * STEPWISE lowering feeds the op list through the same coalescer batch mode uses, so every launch is one
 * schedule step over all ranks.  FUSED lowering uses the k-way fold kernel where the data flow of a whole
 * phase is element-wise (every ring and mesh schedule): each input is read once, and every value the
 * step-wise replay would leave in a buffer is still stored, so both lowerings end in identical memory.
 */
#include <stdlib.h>
#include <string.h>

#include "hg_host.h"
#include "hg_sched.h"

struct HcommGfxPlan {
    uint32_t magic;
    uint32_t nlaunch, cap;
    HgLaunch* launches;
    HcommGfxPlanInfo info;
    /* graph replay of the whole launch list: built at the first full run on a stream, rebuilt when the stream
     * changes, never used when the caller's stream is itself being captured */
    void* graph_exec;
    void* graph_stream;
    int graph_state; /* 0 not built, 1 ready, -1 unavailable */
    int graph_wanted;
};

static int g_use_graph = -1;

static int use_graph(void)
{
    int v = __atomic_load_n(&g_use_graph, __ATOMIC_RELAXED); /* first use may come from several host threads */
    if (v < 0) {
        const char* e = getenv("HCOMM_GFX_GRAPH");
        /* measured on ROCm 7: replaying 15 small kernels as a graph takes 60 us against 54 us launched one by
         * one, so graph replay is opt-in */
        v = (e && e[0] == '1') ? 1 : 0;
        __atomic_store_n(&g_use_graph, v, __ATOMIC_RELAXED);
    }
    return v;
}

static int plan_push(const HgLaunch* l, void* ctx)
{
    HcommGfxPlan* p = (HcommGfxPlan*)ctx;
    if (p->nlaunch == p->cap) {
        uint32_t cap = p->cap ? p->cap * 2 : 16;
        HgLaunch* q = (HgLaunch*)realloc(p->launches, (size_t)cap * sizeof(*q));
        if (!q) return HCCL_E_MEMORY;
        p->launches = q;
        p->cap = cap;
    }
    p->launches[p->nlaunch++] = *l;
    p->info.movedBytes += l->moved_bytes;
    return HCCL_SUCCESS;
}

static int ranges_meet(const void* a, uint64_t an, const void* b, uint64_t bn)
{
    const uintptr_t a0 = (uintptr_t)a, b0 = (uintptr_t)b;
    return an && bn && a0 < b0 + bn && b0 < a0 + an;
}

/* no operation of the group writes what another one reads or writes */
static int step_is_conflict_free(const HgOp* o, uint64_t n)
{
    for (uint64_t a = 0; a < n; ++a)
        for (uint64_t b = 0; b < n; ++b) {
            if (a == b) continue;
            if (ranges_meet(o[a].dst, o[a].bytes, o[b].dst, o[b].bytes) || ranges_meet(o[a].dst, o[a].bytes, o[b].src, o[b].bytes))
                return 0;
        }
    return 1;
}

/* bufs[role][rank]: the buffer behind each role an op list may name (HCOMM_GFX_NUM_BUFS roles) */
/* 3 / 2: reduce on / off 16-byte boundaries, 1 / 0: copy on / off them - the kernels the coalescer tells apart */
static int op_class(const HgOp* o)
{
    const int aligned = (((uintptr_t)o->dst | (uintptr_t)o->src) & (HG_VEC_BYTES - 1u)) == 0;
    return (o->is_reduce ? 2 : 0) + aligned;
}

/* Resolve a schedule's operations into pointers: two entries per operation, because one whose operands are equally far
 * from a 16-byte boundary is cut, as the coalescer would cut it, into the few bytes up to that boundary and an aligned
 * rest - here, so that the grouping below sees the pieces; steps[] carries the step of every entry.  ops and steps hold
 * 2 * n entries; *m receives how many were written. */
static int resolve_ops(const HcommGfxSchedOp* list, uint64_t n, void* const* const* bufs, int dtype, int op, HgOp* ops,
                       uint32_t* steps, uint64_t* m_out)
{
    uint64_t m = 0;
    for (uint64_t i = 0; i < n; ++i) {
        const HcommGfxSchedOp* s = &list[i];
        HgOp* o = &ops[m];
        o->is_reduce = (uint8_t)s->kind;
        o->dtype = s->kind ? (uint8_t)dtype : 255;
        o->op = s->kind ? (uint8_t)op : 255;
        if (s->dstBuf >= HCOMM_GFX_NUM_BUFS || s->srcBuf >= HCOMM_GFX_NUM_BUFS || !bufs[s->dstBuf] || !bufs[s->srcBuf])
            return HCCL_E_PTR;
        o->dst = (char*)bufs[s->dstBuf][s->rank] + s->dstOff;
        o->src = (const char*)bufs[s->srcBuf][s->srcRank] + s->srcOff;
        o->bytes = s->bytes;
        steps[m++] = s->step;
        uint64_t head = hg_split_head(o);
        if (head) {
            ops[m] = *o;
            ops[m].dst = (char*)o->dst + head;
            ops[m].src = (const char*)o->src + head;
            ops[m].bytes = o->bytes - head;
            o->bytes = head;
            steps[m++] = s->step;
        }
    }
    *m_out = m;
    return HCCL_SUCCESS;
}

/* A step that holds both reduces and copies (the double-ring templates pair every reduce with the fetch of the next
 * slice), or operations on 16-byte boundaries beside others that are not (blocks of odd sizes), would change kernel
 * with every operation: when nothing in the step can observe anything else in it, run it class by class - reduces
 * before copies, the aligned kernels before the one for unaligned operands - each class in its original order.
 * tmp holds as many entries as the largest step that is regrouped (at most HG_REGROUP_MAX). */
#define HG_REGROUP_MAX 4096u /* the pairwise test is quadratic: steps larger than any schedule here produces keep their order */
static void regroup_steps(HgOp* ops, const uint32_t* steps, uint64_t n, HgOp* tmp, uint64_t tmp_cap)
{
    for (uint64_t i = 0; i < n;) {
        uint64_t j = i;
        uint32_t seen = 0;
        while (j < n && steps[j] == steps[i]) seen |= 1u << op_class(&ops[j++]);
        if ((seen & (seen - 1u)) != 0 && j - i <= HG_REGROUP_MAX && j - i <= tmp_cap && step_is_conflict_free(ops + i, j - i)) {
            uint64_t k = 0;
            for (int want = 3; want >= 0; --want)
                for (uint64_t q = i; q < j; ++q)
                    if (op_class(&ops[q]) == want) tmp[k++] = ops[q];
            memcpy(ops + i, tmp, (j - i) * sizeof(HgOp));
        }
        i = j;
    }
}

/*
 * Steps that write more than the memory-side cache keeps, cut into pieces that fit it.
 *
 * Element i of a collective only ever meets element i of other buffers, so a schedule restricted to a part of every
 * operation's range is a schedule of its own.  When every two ranges the operations touch are either the same range
 * or apart - ring, mesh and the other schedules whose operations are whole slices - each operation is cut into the
 * same P pieces, and the list becomes: all steps on the first piece of every range, then all steps on the second, ...
 * A step of a piece writes about 128 MiB, so the next step finds the operand it reads in the cache instead of
 * fetching it from HBM again (7-rank ring reduce-scatter in steps of 400 MB: three pieces).  Same operations on the
 * same bytes in the same order per byte, hence the same result; schedules that nest ranges (halving-doubling, NHR's
 * merged runs, the op-base loop's re-cut buffers) stay as they are.  HCOMM_GFX_PIECE_BYTES sets the size aimed at
 * (0 = never cut).
 */
typedef struct {
    uintptr_t at;
    uint64_t bytes;
} HgRange;

static int range_cmp(const void* a, const void* b)
{
    const HgRange* x = (const HgRange*)a;
    const HgRange* y = (const HgRange*)b;
    if (x->at != y->at) return x->at < y->at ? -1 : 1;
    return x->bytes < y->bytes ? -1 : (x->bytes > y->bytes);
}

static uint64_t g_piece_bytes = 0; /* value + 1; 0 = not read yet */

uint64_t hg_piece_bytes(void)
{
    uint64_t v = __atomic_load_n(&g_piece_bytes, __ATOMIC_RELAXED);
    if (v == 0) {
        const char* e = getenv("HCOMM_GFX_PIECE_BYTES");
        v = ((e && *e) ? strtoull(e, NULL, 10) : (128ull << 20));
        if (v > (1ull << 62)) v = 1ull << 62;
        v += 1u;
        __atomic_store_n(&g_piece_bytes, v, __ATOMIC_RELAXED);
    }
    return v - 1u;
}

uint64_t HcommGfxSetPieceBytes(uint64_t bytes)
{
    const uint64_t before = hg_piece_bytes();
    if (bytes > (1ull << 62)) bytes = 1ull << 62;
    __atomic_store_n(&g_piece_bytes, bytes + 1u, __ATOMIC_RELAXED);
    return before;
}

#define HG_PIECES_MAX 16u
#define HG_PIECE_MIN_PART 8u /* no operation is cut into pieces shorter than an eighth of the size aimed at (16 MiB) */
#define HG_SPLIT_HEAD_MAX 16u            /* resolve_ops cuts off fewer bytes than this before a 16-byte boundary */
#define HG_PIECE_ALIGN 128u /* a piece starts as far from a 16-byte (and element) boundary as its operation does */

/* ops[0 .. *m) with steps[]: replaced by the piece-major list when the schedule allows it and has a step large enough
 * to gain; HCCL_SUCCESS either way, HCCL_E_MEMORY when the larger list cannot be allocated */
int hg_cut_into_pieces(HgOp** ops_io, uint32_t** steps_io, uint64_t* m_io)
{
    HgOp* ops = *ops_io;
    const uint32_t* steps = *steps_io;
    const uint64_t m = *m_io, aim = hg_piece_bytes();
    if (aim == 0 || m == 0) return HCCL_SUCCESS;
    uint64_t largest = 0, smallest = UINT64_MAX; /* bytes the largest step writes; the shortest operation of the steps worth cutting */
    for (uint64_t i = 0; i < m;) {
        uint64_t written = 0, shortest = UINT64_MAX, j = i;
        for (; j < m && steps[j] == steps[i]; ++j) {
            written += ops[j].bytes;
            if (ops[j].bytes >= HG_SPLIT_HEAD_MAX && ops[j].bytes < shortest) shortest = ops[j].bytes; /* not the few bytes cut off before a boundary */
        }
        if (written > largest) largest = written;
        if (written > aim * 5u / 2u && shortest < smallest) smallest = shortest;
        i = j;
    }
    /* Up to about twice the size aimed at, a step walked against its producer (direction_of in hg_api.c) finds enough
     * of it in the cache as it is: ring allreduce in steps of 257 MiB 0.905 of the roofline whole, 0.89 in pieces;
     * in steps of 381 MiB 0.845 whole, 0.90 in pieces. */
    if (largest <= aim * 5u / 2u) return HCCL_SUCCESS;
    if (steps[m - 1u] == steps[0]) return HCCL_SUCCESS; /* one step: nobody follows to find its pieces cached */
    uint64_t pieces = (largest + aim - 1u - aim / 16u) / aim; /* a sixteenth over the size aimed at is not worth a piece more */
    if (pieces > HG_PIECES_MAX) pieces = HG_PIECES_MAX;
    /* a launch of many short segments streams worse than it gains from the cache (64 pieces of 2 MiB: 0.75 of the
     * roofline against 0.91 for the whole slices walked against their producer) */
    const uint64_t shortest_piece = aim / HG_PIECE_MIN_PART ? aim / HG_PIECE_MIN_PART : 1u;
    if (pieces > smallest / shortest_piece) pieces = smallest / shortest_piece;
    if (pieces < 2u) return HCCL_SUCCESS;
    /* every two ranges the same or apart */
    HgRange* r = (HgRange*)malloc(2u * m * sizeof(HgRange));
    if (!r) return HCCL_E_MEMORY;
    for (uint64_t i = 0; i < m; ++i) {
        r[2u * i] = (HgRange){(uintptr_t)ops[i].dst, ops[i].bytes};
        r[2u * i + 1u] = (HgRange){(uintptr_t)ops[i].src, ops[i].bytes};
    }
    qsort(r, 2u * m, sizeof(HgRange), range_cmp);
    /* sorted by (start, length): a range that is not a repeat of the one before must start at or behind the furthest
     * end seen so far */
    int apart = 1;
    uintptr_t end = 0;
    for (uint64_t i = 0; i < 2u * m && apart; ++i) {
        if (i && r[i].at == r[i - 1u].at && r[i].bytes == r[i - 1u].bytes) continue;
        if (r[i].at < end) apart = 0;
        if (r[i].at + r[i].bytes > end) end = r[i].at + r[i].bytes;
    }
    free(r);
    if (!apart) return HCCL_SUCCESS;
    HgOp* cut = (HgOp*)calloc(m * pieces, sizeof(HgOp));
    uint32_t* cut_steps = (uint32_t*)calloc(m * pieces, sizeof(uint32_t));
    if (!cut || !cut_steps) {
        free(cut);
        free(cut_steps);
        return HCCL_E_MEMORY;
    }
    const uint32_t nsteps = steps[m - 1u] + 1u; /* steps are numbered in order */
    uint64_t k = 0;
    for (uint64_t q = 0; q < pieces; ++q)
        for (uint64_t i = 0; i < m; ++i) {
            uint64_t each = (ops[i].bytes + pieces - 1u) / pieces;
            each = (each + HG_PIECE_ALIGN - 1u) / HG_PIECE_ALIGN * HG_PIECE_ALIGN;
            const uint64_t from = q * each;
            if (from >= ops[i].bytes) continue;
            cut[k] = ops[i];
            cut[k].dst = (char*)ops[i].dst + from;
            cut[k].src = (const char*)ops[i].src + from;
            cut[k].bytes = ops[i].bytes - from < each ? ops[i].bytes - from : each;
            cut_steps[k++] = (uint32_t)q * nsteps + steps[i];
        }
    free(*ops_io);
    free(*steps_io);
    *ops_io = cut;
    *steps_io = cut_steps;
    *m_io = k;
    return HCCL_SUCCESS;
}

static int lower_ops(HcommGfxPlan* p, const HcommGfxSchedOp* list, uint64_t n, void* const* const* bufs, int dtype,
                     int op)
{
    HgOp* ops = (HgOp*)calloc(n ? 2 * n : 1, sizeof(HgOp));
    uint32_t* steps = (uint32_t*)calloc(n ? 2 * n : 1, sizeof(uint32_t));
    const uint64_t tmp_cap = 2 * n < HG_REGROUP_MAX ? 2 * n : HG_REGROUP_MAX;
    HgOp* tmp = (HgOp*)calloc(tmp_cap ? tmp_cap : 1, sizeof(HgOp));
    int rc = (ops && steps && tmp) ? HCCL_SUCCESS : HCCL_E_MEMORY;
    uint64_t m = 0;
    if (rc == HCCL_SUCCESS) rc = resolve_ops(list, n, bufs, dtype, op, ops, steps, &m);
    if (rc == HCCL_SUCCESS) {
        regroup_steps(ops, steps, m, tmp, tmp_cap);
        rc = hg_cut_into_pieces(&ops, &steps, &m);
    }
    if (rc == HCCL_SUCCESS) rc = hg_coalesce(ops, m, plan_push, p);
    free(ops);
    free(steps);
    free(tmp);
    return rc;
}

static int lower_stepwise(HcommGfxPlan* p, const HgOpList* ol, void* const* in, void* const* out,
                          void* const* scratch, int dtype, int op)
{
    void* const* bufs[HCOMM_GFX_NUM_BUFS] = {in, out, scratch, NULL, NULL};
    return lower_ops(p, ol->ops, ol->n, bufs, dtype, op);
}

static HgLaunch* new_fold(int dtype, int op, int acc_is_dst, uint32_t n, void* const* in, void* const* out)
{
    HgLaunch* l = (HgLaunch*)calloc(1, sizeof(HgLaunch));
    if (!l) return NULL;
    l->kind = HCOMM_GFX_KERNEL_CHAIN;
    l->dtype = (uint32_t)dtype;
    l->op = (uint32_t)op;
    l->acc_is_dst = (uint32_t)acc_is_dst;
    HgFoldTable* f = &l->tab.fold;
    for (uint32_t r = 0; r < n; ++r) {
        f->in[r] = in[r];
        f->out[r] = out ? out[r] : NULL;
    }
    f->k = n;
    f->nranks = n;
    f->stride = 1;
    return l;
}

static int single_copy(HcommGfxPlan* p, void* dst, const void* src, uint64_t bytes)
{
    HgOp o;
    memset(&o, 0, sizeof(o));
    o.dtype = 255;
    o.op = 255;
    o.dst = dst;
    o.src = src;
    o.bytes = bytes;
    return hg_coalesce(&o, 1, plan_push, p);
}

/* ring allreduce / reduce-scatter: slice c travels c+1 -> c+2 -> ... -> c, every hop storing its partial */
static int fused_ring(HcommGfxPlan* p, uint32_t n, void* const* in, void* const* out, uint64_t count,
                      uint64_t stride, int dtype, int op, int out_mode, int standalone)
{
    const uint32_t unit = HcommGfxDataTypeSize((HcommDataType)dtype);
    HcommGfxSlice sl[HCOMM_GFX_MAX_RANKS];
    if (standalone) {
        for (uint32_t i = 0; i < n; ++i) {
            sl[i].offset = (uint64_t)i * stride * unit;
            sl[i].size = count * unit;
        }
    } else {
        int rc = HcommGfxCalcSlices(count, unit, n, sl);
        if (rc != HCCL_SUCCESS) return rc;
    }
    HgLaunch* l = new_fold(dtype, op, 0, n, in, out);
    if (!l) return HCCL_E_MEMORY;
    HgFoldTable* f = &l->tab.fold;
    f->store_partials = 1;
    f->out_mode = (uint32_t)out_mode;
    for (uint32_t c = 0; c < n; ++c) {
        if (sl[c].size == 0) continue;
        const uint32_t s = f->nseg++;
        f->off[s] = sl[c].offset;
        f->bytes[s] = sl[c].size;
        f->first[s] = (uint8_t)((c + 1) % n);
        f->owner[s] = (uint8_t)c;
        f->out_off[s] = 0;
    }
    int rc = HCCL_SUCCESS;
    if (f->nseg) {
        hg_finish_fold(l);
        rc = plan_push(l, p);
    }
    free(l);
    return rc;
}

static int fused_mesh(HcommGfxPlan* p, uint32_t n, void* const* in, void* const* out, uint64_t count,
                      uint64_t stride, int dtype, int op, int scatter, int ascending)
{
    const uint32_t unit = HcommGfxDataTypeSize((HcommDataType)dtype);
    const uint64_t sz = count * unit;
    if (sz == 0) return HCCL_SUCCESS;
    HgLaunch* l = new_fold(dtype, op, 1, n, in, out);
    if (!l) return HCCL_E_MEMORY;
    HgFoldTable* f = &l->tab.fold;
    f->out_mode = 1;
    f->stride = scatter ? -1 : 1;     /* reduce-scatter visits r-1, r-2, ...; one-shot visits r+1, r+2, ... */
    f->store_final_first = scatter ? 1 : 0; /* reduce-scatter accumulates in in[r][slice r] before copying out */
    f->ascending = ascending ? 1u : 0u;
    f->nseg = n;
    for (uint32_t r = 0; r < n; ++r) {
        f->off[r] = scatter ? (uint64_t)r * stride * unit : 0;
        f->bytes[r] = sz;
        f->first[r] = (uint8_t)r;
        f->owner[r] = (uint8_t)r;
        f->out_off[r] = 0;
    }
    hg_finish_fold(l);
    int rc = plan_push(l, p);
    free(l);
    return rc;
}

/* recursive halving-doubling allreduce as one tree launch (block ranks in the table, real ranks as outputs) */
static int fused_rhd(HcommGfxPlan* p, uint32_t n, void* const* in, void* const* out, uint64_t count, int dtype, int op)
{
    const uint32_t unit = HcommGfxDataTypeSize((HcommDataType)dtype);
    uint32_t block = 1;
    while ((block << 1) <= n) block <<= 1;
    const uint32_t part1 = (n - block) * 2;
    HcommGfxSlice sl[HCOMM_GFX_MAX_RANKS];
    int rc = HcommGfxCalcSlices(count, unit, block, sl);
    if (rc != HCCL_SUCCESS) return rc;
    HgLaunch* l = (HgLaunch*)calloc(1, sizeof(HgLaunch));
    if (!l) return HCCL_E_MEMORY;
    l->kind = HCOMM_GFX_KERNEL_TREE;
    l->dtype = (uint32_t)dtype;
    l->op = (uint32_t)op;
    HgFoldTable* f = &l->tab.fold;
    f->tree = 1;
    f->k = block;
    f->nranks = block;
    f->nout = n;
    for (uint32_t b = 0; b < block; ++b) { /* block rank -> rank, recursive_halvingdoubling_base.cc:39-62 */
        const uint32_t real = (b < part1 / 2) ? 2 * b : b + part1 / 2;
        f->in[b] = in[real];
        f->in2[b] = (b < part1 / 2) ? in[real + 1] : NULL;
    }
    for (uint32_t r = 0; r < n; ++r) f->out[r] = out[r];
    for (uint32_t c = 0; c < block; ++c) {
        if (sl[c].size == 0) continue;
        const uint32_t s = f->nseg++;
        f->off[s] = sl[c].offset;
        f->bytes[s] = sl[c].size;
        f->first[s] = (uint8_t)c;
        f->owner[s] = (uint8_t)c;
    }
    if (f->nseg) {
        hg_finish_fold(l);
        rc = plan_push(l, p);
    }
    free(l);
    return rc;
}

/* NHR / NB as one tree launch: slice c is folded over the truncated balanced tree whose position q holds rank
 * c + q (NHR, the tree-ordered slice map decides where slice c lies) or c - q (NB); see k_fold_tree.  scatter: the
 * stand-alone reduce-scatter, whose input slice i lies at i * stride elements and whose result goes to out[c][0..). */
static int fused_rot_tree(HcommGfxPlan* p, int alg, uint32_t n, void* const* in, void* const* out, uint64_t count,
                          uint64_t stride, int dtype, int op)
{
    HgOpList ol;
    /* the slice geometry is whatever the schedule's own-slice copy (allreduce) or final copy (reduce-scatter)
     * says: one copy per rank at step ceil(log2 n), from the input slice that rank owns */
    int rc = hg_schedule(&ol, alg, n, count, stride, dtype);
    if (rc != HCCL_SUCCESS) return rc;
    uint32_t steps = 0;
    while ((1u << steps) < n) ++steps;
    const int scatter = (alg == HCOMM_GFX_ALG_REDUCE_SCATTER_NHR || alg == HCOMM_GFX_ALG_REDUCE_SCATTER_NB);
    const int plus = (alg == HCOMM_GFX_ALG_ALLREDUCE_NHR || alg == HCOMM_GFX_ALG_REDUCE_SCATTER_NHR);
    HgLaunch* l = (HgLaunch*)calloc(1, sizeof(HgLaunch));
    if (!l) {
        hg_oplist_free(&ol);
        return HCCL_E_MEMORY;
    }
    l->kind = HCOMM_GFX_KERNEL_TREE;
    l->dtype = (uint32_t)dtype;
    l->op = (uint32_t)op;
    HgFoldTable* f = &l->tab.fold;
    f->tree = plus ? 2u : 3u;
    f->k = 1u << steps;
    f->nranks = n;
    f->nout = scatter ? 0 : n;
    f->out_mode = scatter ? 1u : 2u;
    for (uint32_t r = 0; r < n; ++r) {
        f->in[r] = in[r];
        f->out[r] = out[r];
    }
    for (uint64_t i = 0; i < ol.n; ++i) {
        const HcommGfxSchedOp* o = &ol.ops[i];
        if (o->step != steps || o->kind != 0 || o->srcBuf != 0 || o->dstBuf != 1 || o->srcRank != o->rank) continue;
        const uint32_t s = f->nseg++;
        f->off[s] = o->srcOff;
        f->out_off[s] = o->dstOff;
        f->bytes[s] = o->bytes;
        f->first[s] = (uint8_t)o->rank;
        f->owner[s] = (uint8_t)o->rank;
    }
    hg_oplist_free(&ol);
    rc = HCCL_SUCCESS;
    if (f->nseg) {
        hg_finish_fold(l);
        rc = plan_push(l, p);
    }
    free(l);
    return rc;
}

/* The one-shot NHR allreduce: one segment, the whole message, on the balanced fold tree rooted at rank 0 - the
 * positions that absorb a neighbour keep their last partial in their input, as the step-wise replay leaves them. */
static int fused_oneshot_tree(HcommGfxPlan* p, uint32_t n, void* const* in, void* const* out, uint64_t total, int dtype,
                              int op)
{
    if (total == 0) return HCCL_SUCCESS;
    HgLaunch* l = (HgLaunch*)calloc(1, sizeof(HgLaunch));
    if (!l) return HCCL_E_MEMORY;
    l->kind = HCOMM_GFX_KERNEL_TREE;
    l->dtype = (uint32_t)dtype;
    l->op = (uint32_t)op;
    HgFoldTable* f = &l->tab.fold;
    f->tree = 2u;
    f->k = 2;
    while (f->k < n) f->k <<= 1;
    f->nranks = n;
    f->nout = n;
    f->out_mode = 2u;
    for (uint32_t r = 0; r < n; ++r) {
        f->in[r] = in[r];
        f->out[r] = out[r];
    }
    f->nseg = 1;
    f->bytes[0] = total;
    hg_finish_fold(l);
    const int rc = plan_push(l, p);
    free(l);
    return rc;
}

/* bit reversal of q inside `bits` bits */
static uint32_t bitrev_n(uint32_t q, uint32_t bits)
{
    uint32_t r = 0;
    for (uint32_t i = 0; i < bits; ++i) r |= ((q >> i) & 1u) << (bits - 1 - i);
    return r;
}

/* ReduceScatterLocalReduce as one tree launch on the user buffers.  Destination d's row is V[j] = rank d - j's copy
 * of slice d; the step-wise replay folds V[a + P] onto V[a] for the tail beyond the largest power of two P <= n and
 * then V[a + h] onto V[a] for h = P/2 .. 1 (temp_reduce_scatter/reduce_scatter_local_reduce.cc:266-301).  With
 * leaf position q holding V[bitrev(q)] (a hole where bitrev(q) >= n) level l of the kernel's tree folds exactly
 * V[j + K / 2^(l+1)] onto V[j].  Only the inputs are read and only out[d] is written: the communication buffers,
 * which the replay uses for the slots, are not touched. */
static int fused_rs_local_reduce(HcommGfxPlan* p, uint32_t n, void* const* in, void* const* out, uint64_t count,
                                 int dtype, int op)
{
    const uint64_t sz = count * HcommGfxDataTypeSize((HcommDataType)dtype);
    if (sz == 0) return HCCL_SUCCESS;
    /* slice d is read at d * sz in every input: 128-bit accesses need 16-byte multiples */
    if (sz & (HG_VEC_BYTES - 1u)) return HCCL_E_NOT_SUPPORT;
    HgLaunch* l = (HgLaunch*)calloc(1, sizeof(HgLaunch));
    if (!l) return HCCL_E_MEMORY;
    l->kind = HCOMM_GFX_KERNEL_TREE;
    l->dtype = (uint32_t)dtype;
    l->op = (uint32_t)op;
    HgFoldTable* f = &l->tab.fold;
    uint32_t bits = 1;
    while ((1u << bits) < n) ++bits;
    f->tree = 5u;
    f->k = 1u << bits;
    f->nranks = n;
    f->out_mode = 1u;
    memset(f->pos, 255, sizeof(f->pos));
    for (uint32_t q = 0; q < f->k; ++q)
        if (bitrev_n(q, bits) < n) f->pos[q] = (uint8_t)bitrev_n(q, bits);
    f->nseg = n;
    for (uint32_t d = 0; d < n; ++d) {
        f->in[d] = in[d];
        f->out[d] = out[d];
        f->off[d] = (uint64_t)d * sz;
        f->bytes[d] = sz;
        f->first[d] = (uint8_t)d;
        f->owner[d] = (uint8_t)d;
        f->out_off[d] = 0;
    }
    hg_finish_fold(l);
    const int rc = plan_push(l, p);
    free(l);
    return rc;
}

/* AllReduceChunkMesh on the user buffers: sub-chunk q of rank r's slice is the chain in[r], then the peers at
 * distances q+1, q+2, .., n-1, 1, .., q (temp_all_reduce/all_reduce_chunk_mesh.cc:234-256), the running value in the
 * dst role; the result goes to every output.  n (n-1) segments, whole ranks' worth per launch.  The communication
 * buffers, where the replay keeps its copies, are not touched and the inputs are only read. */
static int fused_chunk_mesh(HcommGfxPlan* p, uint32_t n, void* const* in, void* const* out, uint64_t count, int dtype,
                            int op)
{
    const uint32_t unit = HcommGfxDataTypeSize((HcommDataType)dtype);
    HcommGfxSlice sl[HCOMM_GFX_MAX_RANKS], sub[HCOMM_GFX_MAX_RANKS];
    int rc = HcommGfxCalcSlices(count, unit, n, sl);
    if (rc != HCCL_SUCCESS) return rc;
    HgLaunch* l = NULL;
    for (uint32_t r = 0; r < n && rc == HCCL_SUCCESS; ++r) {
        if (l && l->tab.fold.nseg + (n - 1) > HG_MAX_SEG) {
            hg_finish_fold(l);
            rc = plan_push(l, p);
            free(l);
            l = NULL;
            if (rc != HCCL_SUCCESS) break;
        }
        if (!l) {
            l = new_fold(dtype, op, 1, n, in, out);
            if (!l) return HCCL_E_MEMORY;
            l->tab.fold.ascending = 2u;
            l->tab.fold.out_mode = 2u;
        }
        HgFoldTable* f = &l->tab.fold;
        rc = HcommGfxCalcSlices(sl[r].size / unit, unit, n - 1, sub);
        for (uint32_t q = 0; q + 1 < n && rc == HCCL_SUCCESS; ++q) {
            if (sub[q].size == 0) continue;
            const uint32_t s = f->nseg++;
            f->off[s] = sl[r].offset + sub[q].offset;
            f->bytes[s] = sub[q].size;
            f->first[s] = (uint8_t)r;
            f->owner[s] = (uint8_t)r;
            f->start[s] = (uint8_t)q;
        }
    }
    if (l) {
        if (rc == HCCL_SUCCESS && l->tab.fold.nseg) {
            hg_finish_fold(l);
            rc = plan_push(l, p);
        }
        free(l);
    }
    return rc;
}

/* ---- a schedule's own expression trees as one tree launch ------------------------------------------------------
 *
 * The operation list is replayed on symbols: a cell is an exact byte range of one buffer, its value a node - a leaf
 * (rank, offset: the range of that rank's input) or a fold (dst node, src node).  What ends up in the output cells
 * are the trees the kernel must evaluate; they are laid out over 2^depth leaf positions so that the kernel's fixed
 * pattern (level l folds position q + 2^l onto q) walks them with every dst operand on the left.  Lists that read a
 * range with other bounds than it was written with are refused (HCCL_E_NOT_SUPPORT), and so are lists that write an
 * input unless the caller asked for the inputs to be left alone (the launch only ever reads the original inputs).
 * Outputs that hold the same trees in every rank become segments written to all ranks, others one segment each. */
typedef struct {
    uint32_t rank, buf;
    uint64_t off, bytes;
    int32_t node;
} SymCell;

typedef struct {
    int32_t left, right; /* -1, -1: a leaf */
    uint32_t rank;
    uint32_t depth;      /* folds between this node and its deepest leaf: 0 for a leaf */
    uint64_t off;
} SymNode;

#define HG_TREE_MAX_DEPTH 6u /* per-segment trees span 64 = 2^6 leaf positions at most (two halves of 32, one after the other) */

typedef struct {
    SymCell* cell;
    SymNode* node;
    uint32_t ncell, nnode, cap;
} SymState;

static int32_t sym_find(const SymState* st, uint32_t rank, uint32_t buf, uint64_t off, uint64_t bytes)
{
    for (uint32_t i = 0; i < st->ncell; ++i) {
        const SymCell* c = &st->cell[i];
        if (c->rank != rank || c->buf != buf) continue;
        if (c->off == off && c->bytes == bytes) return (int32_t)i;
        if (c->off < off + bytes && off < c->off + c->bytes) return -2; /* other bounds */
    }
    return -1;
}

static int32_t sym_node(SymState* st, int32_t left, int32_t right, uint32_t rank, uint64_t off)
{
    SymNode* n = &st->node[st->nnode];
    n->left = left;
    n->right = right;
    n->rank = rank;
    n->off = off;
    n->depth = 0;
    if (left >= 0) {
        const uint32_t a = st->node[left].depth, b = st->node[right].depth;
        n->depth = 1u + (a > b ? a : b);
    }
    return (int32_t)st->nnode++;
}

/* node into the span of 2^h positions that starts at q; 0 when a leaf lies at another offset than the segment.
 * Recursion is as deep as the node, which no caller lets exceed HG_TREE_MAX_DEPTH. */
static int sym_place(const SymState* st, int32_t node, uint8_t* pos, uint32_t q, uint32_t h, uint64_t off)
{
    const SymNode* n = &st->node[node];
    if (n->left < 0) {
        pos[q] = (uint8_t)n->rank;
        return n->off == off;
    }
    return sym_place(st, n->left, pos, q, h - 1, off) && sym_place(st, n->right, pos, q + (1u << (h - 1)), h - 1, off);
}

static int fused_from_trees(HcommGfxPlan* p, const HgOpList* ol, uint32_t n, void* const* in, void* const* out, int dtype,
                            int op, int inputs_may_change)
{
    SymState st;
    memset(&st, 0, sizeof(st));
    st.cap = (uint32_t)(2 * ol->n + 1);
    st.cell = (SymCell*)calloc(st.cap, sizeof(SymCell));                       /* at most two new cells per operation */
    st.node = (SymNode*)calloc((size_t)st.cap + ol->n, sizeof(SymNode));       /* and three new nodes */
    int32_t* pend_cell = (int32_t*)calloc(ol->n + 1, sizeof(int32_t));
    int32_t* pend_node = (int32_t*)calloc(ol->n + 1, sizeof(int32_t));
    uint64_t* written_in = (uint64_t*)calloc(st.cap, sizeof(uint64_t)); /* per cell: 1 + first operation of the step that writes it */
    HgLaunch* l = NULL;
    int rc = (st.cell && st.node && pend_cell && pend_node && written_in) ? HCCL_SUCCESS : HCCL_E_MEMORY;
    /* the operations of a step act in parallel: all of them read the state the step began with */
    for (uint64_t i = 0, j; i < ol->n && rc == HCCL_SUCCESS; i = j) {
        for (j = i; j < ol->n && ol->ops[j].step == ol->ops[i].step && rc == HCCL_SUCCESS; ++j) {
            const HcommGfxSchedOp* o = &ol->ops[j];
            pend_cell[j] = -1;
            if (o->bytes == 0) continue;
            /* a list that writes its inputs can only be lowered for a caller who wants them left alone: the launch
             * reads the original inputs at the leaves and stores nothing into them */
            if (o->dstBuf == 0 && !inputs_may_change) rc = HCCL_E_NOT_SUPPORT;
            int32_t src = sym_find(&st, o->srcRank, o->srcBuf, o->srcOff, o->bytes);
            if (src == -1 && o->srcBuf == 0) { /* first read of an input range: a leaf */
                SymCell* c = &st.cell[st.ncell];
                c->rank = o->srcRank;
                c->buf = 0;
                c->off = o->srcOff;
                c->bytes = o->bytes;
                c->node = sym_node(&st, -1, -1, o->srcRank, o->srcOff);
                src = (int32_t)st.ncell++;
            }
            int32_t dst = sym_find(&st, o->rank, o->dstBuf, o->dstOff, o->bytes);
            if (src < 0 || dst == -2 || st.cell[src].node < 0) rc = HCCL_E_NOT_SUPPORT; /* other bounds, or never written */
            if (rc != HCCL_SUCCESS) break;
            if (dst == -1) {
                SymCell* c = &st.cell[st.ncell];
                c->rank = o->rank;
                c->buf = o->dstBuf;
                c->off = o->dstOff;
                c->bytes = o->bytes;
                /* an input range folded into starts as its own leaf; any other range has no value yet */
                c->node = (o->dstBuf == 0) ? sym_node(&st, -1, -1, o->rank, o->dstOff) : -1;
                dst = (int32_t)st.ncell++;
            }
            if (o->kind && st.cell[dst].node < 0) {
                rc = HCCL_E_NOT_SUPPORT;
                break;
            }
            /* "every operation of a step reads the state the step began with" equals the list's replay only while no
             * operation of the step writes what another one of it reads or writes: refuse the lists where it does not */
            if (written_in[dst] > i || written_in[src] > i) {
                rc = HCCL_E_NOT_SUPPORT;
                break;
            }
            written_in[dst] = i + 1;
            pend_cell[j] = dst;
            pend_node[j] = o->kind ? sym_node(&st, st.cell[dst].node, st.cell[src].node, 0, 0) : st.cell[src].node;
            if (st.node[pend_node[j]].depth > HG_TREE_MAX_DEPTH) { /* deeper than the kernel folds: no point in going on */
                rc = HCCL_E_NOT_SUPPORT;
                break;
            }
        }
        for (uint64_t t = i; t < j && rc == HCCL_SUCCESS; ++t)
            if (pend_cell[t] >= 0) st.cell[pend_cell[t]].node = pend_node[t];
    }
    free(pend_cell);
    free(pend_node);
    free(written_in);
    /* When every rank's output holds the same trees at the same places, the output cells of rank 0 are the segments
     * and the root goes to all outputs; otherwise (whole-message recursive doubling: every rank folds in an order of
     * its own) every output cell is a segment with a single destination. */
    uint32_t nseg = 0, nseg_all = 0, depth = 1;
    int uniform = 1;
    for (uint32_t i = 0; i < st.ncell && rc == HCCL_SUCCESS; ++i) {
        const SymCell* c = &st.cell[i];
        if (c->buf != 1) continue;
        ++nseg_all;
        if (c->node < 0) {
            rc = HCCL_E_NOT_SUPPORT;
            break;
        }
        const uint32_t d = st.node[c->node].depth;
        if (d > depth) depth = d;
        if (c->rank == 0) {
            ++nseg;
            for (uint32_t r = 1; r < n; ++r) {
                const int32_t j = sym_find(&st, r, 1, c->off, c->bytes);
                if (j < 0 || st.cell[j].node != c->node) uniform = 0;
            }
        } else if (sym_find(&st, 0, 1, c->off, c->bytes) < 0) {
            uniform = 0;
        }
    }
    if (!uniform) nseg = nseg_all;
    if (rc == HCCL_SUCCESS && depth > HG_TREE_MAX_DEPTH) rc = HCCL_E_NOT_SUPPORT;
    const uint32_t k = 1u << (depth > HG_TREE_MAX_DEPTH ? HG_TREE_MAX_DEPTH : depth);
    const uint32_t per_launch = HG_POS_BYTES / k < HG_MAX_SEG ? HG_POS_BYTES / k : HG_MAX_SEG;
    for (uint32_t i = 0; i < st.ncell && rc == HCCL_SUCCESS; ++i) {
        const SymCell* c = &st.cell[i];
        if (c->buf != 1 || (uniform && c->rank != 0)) continue;
        if (!l) {
            l = (HgLaunch*)calloc(1, sizeof(HgLaunch));
            if (!l) {
                rc = HCCL_E_MEMORY;
                break;
            }
            l->kind = HCOMM_GFX_KERNEL_TREE;
            l->dtype = (uint32_t)dtype;
            l->op = (uint32_t)op;
            HgFoldTable* f = &l->tab.fold;
            f->tree = 6u;
            f->k = k;
            f->nranks = n;
            f->nout = uniform ? n : 0;
            f->out_mode = uniform ? 2u : 1u;
            memset(f->pos, 255, sizeof(f->pos));
            for (uint32_t r = 0; r < n; ++r) {
                f->in[r] = in[r];
                f->out[r] = out[r];
            }
        }
        HgFoldTable* f = &l->tab.fold;
        const uint32_t s = f->nseg++;
        f->off[s] = c->off;
        f->out_off[s] = c->off;
        f->owner[s] = (uint8_t)c->rank;
        f->bytes[s] = c->bytes;
        /* 128-bit accesses: a segment must start on a 16-byte boundary of every buffer */
        if ((c->off & (HG_VEC_BYTES - 1u)) || !sym_place(&st, c->node, f->pos + s * k, 0, depth, c->off)) rc = HCCL_E_NOT_SUPPORT;
        --nseg;
        if (rc == HCCL_SUCCESS && (f->nseg == per_launch || nseg == 0)) {
            hg_finish_fold(l);
            rc = plan_push(l, p);
            free(l);
            l = NULL;
        }
    }
    free(l);
    free(st.cell);
    free(st.node);
    return rc;
}

/* Leaf table of the rank-order tree over n_servers x n_local ranks: the low position bits walk a server's devices so
 * that level l folds device j + 2^(bits - 1 - l) onto device j, the high bits the servers likewise; 255 = no leaf. */
static uint32_t rank_order_positions(uint32_t n_servers, uint32_t n_local, uint8_t* pos)
{
    uint32_t bits_l = 0, bits_s = 0;
    while ((1u << bits_l) < n_local) ++bits_l;
    while ((1u << bits_s) < n_servers) ++bits_s;
    uint32_t k = 1u << (bits_l + bits_s);
    if (k < 2) k = 2;
    memset(pos, 255, HG_POS_BYTES);
    for (uint32_t q = 0; q < k; ++q) {
        const uint32_t dev = bitrev_n(q & ((1u << bits_l) - 1u), bits_l), srv = bitrev_n(q >> bits_l, bits_s);
        if (dev < n_local && srv < n_servers) pos[q] = (uint8_t)(srv * n_local + dev);
    }
    return k;
}

/* The AICPU deterministic reduce-scatter in one launch: SelfLocalReduce's folds (the slots beyond the largest power of
 * two onto the first ones, then halving rounds) are the rank-order tree over the N inputs, slot s holding rank s's
 * slice; block d of every input at d * stride, root to out[d]. */
static int fused_window_halving(HcommGfxPlan* p, uint32_t n, void* const* in, void* const* out, uint64_t count, uint64_t stride,
                                int dtype, int op)
{
    const uint32_t unit = HcommGfxDataTypeSize((HcommDataType)dtype);
    const uint64_t block = count * unit;
    if (block == 0) return HCCL_SUCCESS;
    if (n > 32u) return HCCL_E_NOT_SUPPORT;
    /* 128-bit accesses: every block of every input must start on a 16-byte boundary */
    if ((stride * unit) & (HG_VEC_BYTES - 1u)) return HCCL_E_NOT_SUPPORT;
    HgLaunch* l = (HgLaunch*)calloc(1, sizeof(HgLaunch));
    if (!l) return HCCL_E_MEMORY;
    l->kind = HCOMM_GFX_KERNEL_TREE;
    l->dtype = (uint32_t)dtype;
    l->op = (uint32_t)op;
    HgFoldTable* f = &l->tab.fold;
    f->tree = 4u;
    f->k = rank_order_positions(1, n, f->pos);
    f->nranks = n;
    f->out_mode = 1u;
    f->nseg = n;
    for (uint32_t r = 0; r < n; ++r) {
        f->in[r] = in[r];
        f->out[r] = out[r];
        f->off[r] = stride * unit * r;
        f->bytes[r] = block;
        f->owner[r] = (uint8_t)r;
    }
    hg_finish_fold(l);
    const int rc = plan_push(l, p);
    free(l);
    return rc;
}

static int lower_fused(HcommGfxPlan* p, int alg, const HgOpList* ol, uint32_t n, void* const* in, void* const* out,
                       uint64_t count, uint64_t stride, int dtype, int op, int keep_inputs)
{
    const uint64_t total = count * HcommGfxDataTypeSize((HcommDataType)dtype);
    switch (alg) {
        case HCOMM_GFX_ALG_ALLREDUCE_RING:
            if (n == 1) return single_copy(p, out[0], in[0], total);
            return fused_ring(p, n, in, out, count, count, dtype, op, 2, 0);
        case HCOMM_GFX_ALG_REDUCE_SCATTER_RING:
            if (n == 1) return HCCL_SUCCESS;
            return fused_ring(p, n, in, out, count, count, dtype, op, 0, 0);
        case HCOMM_GFX_ALG_REDUCE_SCATTER_RING_STANDALONE:
            if (n == 1) return single_copy(p, out[0], in[0], total);
            return fused_ring(p, n, in, out, count, stride, dtype, op, 1, 1);
        case HCOMM_GFX_ALG_ALLREDUCE_RHD:
            if (n == 1) return single_copy(p, out[0], in[0], total);
            return fused_rhd(p, n, in, out, count, dtype, op);
        case HCOMM_GFX_ALG_ALLREDUCE_MESH_ONESHOT: return fused_mesh(p, n, in, out, count, count, dtype, op, 0, 0);
        case HCOMM_GFX_ALG_ALLREDUCE_MESH_ONESHOT_ASCENDING:
            return fused_mesh(p, n, in, out, count, count, dtype, op, 0, 1);
        case HCOMM_GFX_ALG_REDUCE_SCATTER_MESH:
            if (n == 1) return single_copy(p, out[0], in[0], total);
            return fused_mesh(p, n, in, out, count, stride, dtype, op, 1, 0);
        case HCOMM_GFX_ALG_ALLREDUCE_NHR:
        case HCOMM_GFX_ALG_ALLREDUCE_NB:
        case HCOMM_GFX_ALG_REDUCE_SCATTER_NHR:
        case HCOMM_GFX_ALG_REDUCE_SCATTER_NB:
            if (n == 1) return single_copy(p, out[0], in[0], total);
            return fused_rot_tree(p, alg, n, in, out, count, stride, dtype, op);
        case HCOMM_GFX_ALG_ALLREDUCE_NHR_ONESHOT:
            if (n == 1) return single_copy(p, out[0], in[0], total);
            return fused_oneshot_tree(p, n, in, out, total, dtype, op);
        case HCOMM_GFX_ALG_ALLREDUCE_CHUNK_MESH:
            if (n == 1) return single_copy(p, out[0], in[0], total);
            return fused_chunk_mesh(p, n, in, out, count, dtype, op);
        case HCOMM_GFX_ALG_ALLREDUCE_LOCAL_REDUCE:
            if (n == 1) return single_copy(p, out[0], in[0], total);
            return ol ? fused_from_trees(p, ol, n, in, out, dtype, op, 0) : HCCL_E_NOT_SUPPORT;
        case HCOMM_GFX_ALG_ALLREDUCE_DOUBLING:
            /* its steps copy the running value back into the input for the partner to read, so only the lowering
             * that promises to leave the inputs alone has a single launch: one tree per rank, root to that rank */
            if (n == 1) return single_copy(p, out[0], in[0], total);
            return (ol && keep_inputs) ? fused_from_trees(p, ol, n, in, out, dtype, op, 1) : HCCL_E_NOT_SUPPORT;
        case HCOMM_GFX_ALG_REDUCE_SCATTER_LOCAL_REDUCE:
            if (n == 1) return single_copy(p, out[0], in[0], total);
            return fused_rs_local_reduce(p, n, in, out, count, dtype, op);
        case HCOMM_GFX_ALG_REDUCE_SCATTER_WINDOW_HALVING:
            if (n == 1) return single_copy(p, out[0], in[0], total);
            return fused_window_halving(p, n, in, out, count, stride, dtype, op);
        default: return HCCL_E_NOT_SUPPORT;
    }
}

/* HCOMM_GFX_LOWER_FUSED_KEEP_INPUTS: the launches of the fused lowering with every store into an input dropped */
static void drop_input_stores(HcommGfxPlan* p)
{
    p->info.movedBytes = 0;
    for (uint32_t i = 0; i < p->nlaunch; ++i) {
        HgLaunch* l = &p->launches[i];
        HgFoldTable* f = &l->tab.fold;
        if (l->kind == HCOMM_GFX_KERNEL_CHAIN) {
            f->store_partials = 0;
            f->store_final_first = 0;
            hg_finish_fold(l);
        } else if (l->kind == HCOMM_GFX_KERNEL_TREE) {
            f->keep_inputs = 1;
            hg_finish_fold(l);
        }
        p->info.movedBytes += l->moved_bytes;
    }
}

static int in_place(int alg) { return alg == HCOMM_GFX_ALG_REDUCE_SCATTER_RING; }

int32_t HcommGfxPlanCreate(
    HcommGfxAlgorithm alg, HcommGfxLowering lowering, uint32_t nRanks, void* const* in, void* const* out,
    uint64_t count, HcommDataType dataType, HcommReduceOp reduceOp, HcommGfxPlan** plan)
{
    return HcommGfxPlanCreateStrided(alg, lowering, nRanks, in, out, count, 0, dataType, reduceOp, plan);
}

int32_t HcommGfxPlanCreateStrided(
    HcommGfxAlgorithm alg, HcommGfxLowering lowering, uint32_t nRanks, void* const* in, void* const* out,
    uint64_t count, uint64_t strideCount, HcommDataType dataType, HcommReduceOp reduceOp, HcommGfxPlan** plan)
{
    return HcommGfxPlanCreateEx(alg, lowering, nRanks, in, out, NULL, count, strideCount, dataType, reduceOp, plan);
}

int32_t HcommGfxScratchBytes(HcommGfxAlgorithm alg, uint32_t nRanks, uint64_t count, HcommDataType dataType,
                             uint64_t* bytes)
{
    if (!bytes) return HCCL_E_PTR;
    if (nRanks == 0 || nRanks > HCOMM_GFX_MAX_RANKS || HcommGfxDataTypeSize(dataType) == 0) return HCCL_E_PARA;
    if (count > HG_MAX_COUNT) return HCCL_E_PARA;
    *bytes = hg_scratch_bytes((int)alg, nRanks, count, (int)dataType);
    return HCCL_SUCCESS;
}

int32_t HcommGfxPlanCreateEx(
    HcommGfxAlgorithm alg, HcommGfxLowering lowering, uint32_t nRanks, void* const* in, void* const* out,
    void* const* scratch, uint64_t count, uint64_t strideCount, HcommDataType dataType, HcommReduceOp reduceOp,
    HcommGfxPlan** plan)
{
    if (!plan) return HCCL_E_PTR;
    *plan = NULL;
    if (!in) return HCCL_E_PTR;
    if (!out && !in_place((int)alg)) return HCCL_E_PTR;
    if (nRanks == 0 || nRanks > HCOMM_GFX_MAX_RANKS) return HCCL_E_PARA;
    if (!hg_reduce_supported((int)dataType, (int)reduceOp, 1)) return HCCL_E_PARA;
    if (lowering != HCOMM_GFX_LOWER_STEPWISE && lowering != HCOMM_GFX_LOWER_FUSED && lowering != HCOMM_GFX_LOWER_FUSED_KEEP_INPUTS)
        return HCCL_E_PARA;
    /* a result that lives in the input cannot leave the input alone */
    if (lowering == HCOMM_GFX_LOWER_FUSED_KEEP_INPUTS && in_place((int)alg)) return HCCL_E_NOT_SUPPORT;
    for (uint32_t r = 0; r < nRanks; ++r) {
        if (!in[r]) return HCCL_E_PTR;
        if (((uintptr_t)in[r]) & 127u) return HCCL_E_PARA;
        if (!in_place((int)alg)) {
            if (!out[r]) return HCCL_E_PTR;
            if (((uintptr_t)out[r]) & 127u) return HCCL_E_PARA;
        }
    }
    /* the single-launch lowerings work on the user buffers alone */
    if (lowering == HCOMM_GFX_LOWER_STEPWISE && nRanks > 1 && hg_scratch_bytes((int)alg, nRanks, count, (int)dataType) > 0) {
        if (!scratch) return HCCL_E_PTR;
        for (uint32_t r = 0; r < nRanks; ++r) {
            if (!scratch[r]) return HCCL_E_PTR;
            if (((uintptr_t)scratch[r]) & 127u) return HCCL_E_PARA;
        }
    }
    HgOpList ol;
    if (strideCount == 0) strideCount = count;
    int rc = hg_schedule(&ol, (int)alg, nRanks, count, strideCount, (int)dataType);
    if (rc != HCCL_SUCCESS) return rc;
    HcommGfxPlan* p = (HcommGfxPlan*)calloc(1, sizeof(*p));
    if (!p) {
        hg_oplist_free(&ol);
        return HCCL_E_MEMORY;
    }
    p->magic = HG_PLAN_MAGIC;
    p->graph_wanted = use_graph();
    p->info.steps = ol.steps;
    for (uint64_t i = 0; i < ol.n; ++i) p->info.algorithmicBytes += ol.ops[i].bytes * (ol.ops[i].kind ? 3u : 2u);
    if (lowering == HCOMM_GFX_LOWER_STEPWISE)
        rc = lower_stepwise(p, &ol, in, out, scratch, (int)dataType, (int)reduceOp);
    else
        rc = lower_fused(p, (int)alg, &ol, nRanks, in, out, count, strideCount, (int)dataType, (int)reduceOp,
                         lowering == HCOMM_GFX_LOWER_FUSED_KEEP_INPUTS);
    if (rc == HCCL_SUCCESS && lowering == HCOMM_GFX_LOWER_FUSED_KEEP_INPUTS) drop_input_stores(p);
    hg_oplist_free(&ol);
    if (rc != HCCL_SUCCESS) {
        HcommGfxPlanDestroy(p);
        return rc;
    }
    p->info.launches = p->nlaunch;
    *plan = p;
    return HCCL_SUCCESS;
}

/* ---- the deterministic mesh allreduce for callers that cannot allocate ---------------------------------------- */

#define HG_NOALLOC_MAX_RANKS HCOMM_GFX_NOALLOC_MAX_RANKS
#define HG_NOALLOC_MAX_OPS (3u * HG_NOALLOC_MAX_RANKS * HG_NOALLOC_MAX_RANKS) /* the schedule has 3 n^2 - 2 n operations */

static int emit_now(const HgLaunch* l, void* ctx) { return hg_submit((HgThread*)ctx, l); }

int32_t HcommGfxAllReduceLocalReduceNoAlloc(
    ThreadHandle thread, uint32_t nRanks, void* const* in, void* const* out, uint64_t count, HcommDataType dataType,
    HcommReduceOp reduceOp)
{
    if (!in || !out) return HCCL_E_PTR;
    if (nRanks == 0 || nRanks > HG_NOALLOC_MAX_RANKS) return HCCL_E_PARA;
    if (!hg_reduce_supported((int)dataType, (int)reduceOp, 1)) return HCCL_E_PARA;
    if (count > HG_MAX_COUNT) return HCCL_E_PARA;
    for (uint32_t r = 0; r < nRanks; ++r) {
        if (!in[r] || !out[r]) return HCCL_E_PTR;
        if ((((uintptr_t)in[r]) | ((uintptr_t)out[r])) & 127u) return HCCL_E_PARA;
    }
    HgThread* t = hg_thread_from_handle(thread);
    if (!t) return HCCL_E_PTR;
    /* its launches are submitted at once: inside a batch they would run ahead of what the batch has recorded */
    if (hg_caller_is_batching()) return HCCL_E_NOT_SUPPORT;
    if (hg_thread_free_for_caller(t) != HCCL_SUCCESS) return HCCL_E_UNAVAIL;
    /* every rank's communication buffer is a slice of the library's own array on the thread's GPU */
    uint64_t per_rank = hg_scratch_bytes(HCOMM_GFX_ALG_ALLREDUCE_LOCAL_REDUCE, nRanks, count, (int)dataType);
    per_rank = (per_rank + 255u) & ~(uint64_t)255u;
    if (per_rank > HCOMM_GFX_NOALLOC_SCRATCH_BYTES / nRanks) return HCCL_E_PARA; /* larger than the array: see the header */
    void* base = NULL;
    if (t->recorder) {
        base = (void*)((uintptr_t)1 << 40); /* launches are only logged: any aligned address stands for the array */
    } else {
        const int rc = hg_rt_scratch(t->stream, &base);
        if (rc != HCCL_SUCCESS) return rc;
    }
    void* scratch[HG_NOALLOC_MAX_RANKS];
    for (uint32_t r = 0; r < nRanks; ++r) scratch[r] = (char*)base + (uint64_t)r * per_rank;
    HcommGfxSchedOp sched[HG_NOALLOC_MAX_OPS];
    HgOpList ol;
    memset(&ol, 0, sizeof(ol));
    ol.ops = sched;
    ol.cap = HG_NOALLOC_MAX_OPS;
    ol.fixed = 1;
    int rc = hg_schedule_into(&ol, HCOMM_GFX_ALG_ALLREDUCE_LOCAL_REDUCE, nRanks, count, count, (int)dataType);
    if (rc != HCCL_SUCCESS) return rc;
    /* the plan's own lowering on storage of this call: resolve, regroup the steps that mix kernels, then through the
     * coalescer, which merges what the ranks do in a step into one launch and submits each launch as soon as the
     * next operation cannot join it */
    void* const* bufs[HCOMM_GFX_NUM_BUFS] = {in, out, scratch, NULL, NULL};
    HgOp ops[2 * HG_NOALLOC_MAX_OPS], tmp[2 * HG_NOALLOC_MAX_OPS];
    uint32_t steps[2 * HG_NOALLOC_MAX_OPS];
    uint64_t m = 0;
    rc = resolve_ops(sched, ol.n, bufs, (int)dataType, (int)reduceOp, ops, steps, &m);
    if (rc != HCCL_SUCCESS) return rc;
    regroup_steps(ops, steps, m, tmp, 2 * HG_NOALLOC_MAX_OPS);
    HgLaunch work;
    const int log_fixed = t->log_fixed;
    if (!t->recorder) t->log_fixed = 1; /* the launch log grows by reallocation */
    rc = hg_coalesce_with(ops, m, emit_now, t, &work);
    t->log_fixed = log_fixed;
    if (rc != HCCL_SUCCESS) return rc;
    return HCCL_SUCCESS;
}

static int check_bufs(void* const* b, uint32_t n)
{
    if (!b) return HCCL_E_PTR;
    for (uint32_t r = 0; r < n; ++r) {
        if (!b[r]) return HCCL_E_PTR;
        if (((uintptr_t)b[r]) & 127u) return HCCL_E_PARA;
    }
    return HCCL_SUCCESS;
}

int32_t HcommGfxOpBasePlanCreate(
    HcommGfxAlgorithm alg, HcommGfxLowering lowering, uint32_t nRanks, void* const* userIn, void* const* userOut,
    void* const* cclIn, void* const* cclOut, void* const* scratch, uint64_t cclBytes, uint64_t count,
    HcommDataType dataType, HcommReduceOp reduceOp, HcommGfxPlan** plan)
{
    if (!plan) return HCCL_E_PTR;
    *plan = NULL;
    if (!userIn || !userOut || !cclIn || !cclOut) return HCCL_E_PTR;
    if (nRanks == 0 || nRanks > HCOMM_GFX_MAX_RANKS) return HCCL_E_PARA;
    if (!hg_reduce_supported((int)dataType, (int)reduceOp, 1)) return HCCL_E_PARA;
    if (lowering != HCOMM_GFX_LOWER_STEPWISE && lowering != HCOMM_GFX_LOWER_FUSED) return HCCL_E_PARA;
    for (uint32_t r = 0; r < nRanks; ++r)
        if (!userIn[r] || !userOut[r]) return HCCL_E_PTR;
    int rc = check_bufs(cclIn, nRanks);
    if (rc == HCCL_SUCCESS) rc = check_bufs(cclOut, nRanks);
    if (rc != HCCL_SUCCESS) return rc;
    const uint32_t unit = HcommGfxDataTypeSize(dataType);
    const uint64_t maxc = hg_opbase_max_count((int)alg, nRanks, cclBytes, unit);
    const uint64_t chunk = count < maxc ? count : maxc;
    if (nRanks > 1 && chunk > 0 && hg_scratch_bytes((int)alg, nRanks, chunk, (int)dataType) > 0) {
        /* their single-launch lowerings leave the communication buffers alone, the loop's replay does not */
        if (lowering == HCOMM_GFX_LOWER_FUSED) return HCCL_E_NOT_SUPPORT;
        rc = check_bufs(scratch, nRanks);
        if (rc != HCCL_SUCCESS) return rc;
    }
    HgOpList ol;
    rc = hg_schedule_opbase(&ol, (int)alg, nRanks, count, cclBytes, (int)dataType);
    if (rc != HCCL_SUCCESS) return rc;
    HcommGfxPlan* p = (HcommGfxPlan*)calloc(1, sizeof(*p));
    if (!p) {
        hg_oplist_free(&ol);
        return HCCL_E_MEMORY;
    }
    p->magic = HG_PLAN_MAGIC;
    p->graph_wanted = use_graph();
    p->info.steps = ol.steps;
    for (uint64_t i = 0; i < ol.n; ++i) p->info.algorithmicBytes += ol.ops[i].bytes * (ol.ops[i].kind ? 3u : 2u);
    void* const* bufs[HCOMM_GFX_NUM_BUFS] = {cclIn, cclOut, scratch, userIn, userOut};
    if (lowering == HCOMM_GFX_LOWER_STEPWISE) {
        rc = lower_ops(p, ol.ops, ol.n, bufs, (int)dataType, (int)reduceOp);
    } else {
        /* per chunk: the copies in, the template part fused as a stand-alone plan would be, the copies out.  The
         * list is ordered by step, and inside a chunk every op that names a user buffer is one of its copies. */
        uint64_t i = 0, done = 0;
        while (i < ol.n && rc == HCCL_SUCCESS) {
            uint64_t j = i;
            while (j < ol.n && ol.ops[j].srcBuf == HCOMM_GFX_BUF_USER_IN) ++j;
            rc = lower_ops(p, &ol.ops[i], j - i, bufs, (int)dataType, (int)reduceOp);
            uint64_t k = j;
            while (k < ol.n && ol.ops[k].dstBuf != HCOMM_GFX_BUF_USER_OUT) ++k;
            const uint64_t cur = count - done > maxc ? maxc : count - done;
            if (rc == HCCL_SUCCESS) rc = lower_fused(p, (int)alg, NULL, nRanks, cclIn, cclOut, cur, cur, (int)dataType, (int)reduceOp, 0);
            uint64_t m = k;
            while (m < ol.n && ol.ops[m].dstBuf == HCOMM_GFX_BUF_USER_OUT) ++m;
            if (rc == HCCL_SUCCESS) rc = lower_ops(p, &ol.ops[k], m - k, bufs, (int)dataType, (int)reduceOp);
            done += cur;
            i = m;
        }
    }
    hg_oplist_free(&ol);
    if (rc != HCCL_SUCCESS) {
        HcommGfxPlanDestroy(p);
        return rc;
    }
    p->info.launches = p->nlaunch;
    *plan = p;
    return HCCL_SUCCESS;
}

int32_t HcommGfxPlanCreateFromOps(
    const HcommGfxSchedOp* ops, uint64_t nOps, uint32_t nRanks, void* const* const* buffers, HcommDataType dataType,
    HcommReduceOp reduceOp, HcommGfxPlan** plan)
{
    if (!plan) return HCCL_E_PTR;
    *plan = NULL;
    if ((nOps && !ops) || !buffers) return HCCL_E_PTR;
    if (nRanks == 0 || nRanks > HCOMM_GFX_MAX_RANKS) return HCCL_E_PARA;
    if (!hg_reduce_supported((int)dataType, (int)reduceOp, 1)) return HCCL_E_PARA;
    const uint32_t unit = HcommGfxDataTypeSize(dataType);
    uint32_t steps = 0;
    for (uint64_t i = 0; i < nOps; ++i) {
        const HcommGfxSchedOp* o = &ops[i];
        if (o->kind > 1 || o->rank >= nRanks || o->srcRank >= nRanks || o->dstBuf >= HCOMM_GFX_NUM_BUFS ||
            o->srcBuf >= HCOMM_GFX_NUM_BUFS)
            return HCCL_E_PARA;
        if (o->kind == 1 && o->bytes % unit) return HCCL_E_PARA; /* a reduce moves whole elements */
        if (i && o->step < ops[i - 1].step) return HCCL_E_PARA;   /* ordered by step */
        if (!buffers[o->dstBuf] || !buffers[o->srcBuf] || !buffers[o->dstBuf][o->rank] || !buffers[o->srcBuf][o->srcRank])
            return HCCL_E_PTR;
        if (o->step + 1 > steps) steps = o->step + 1;
    }
    HcommGfxPlan* p = (HcommGfxPlan*)calloc(1, sizeof(*p));
    if (!p) return HCCL_E_MEMORY;
    p->magic = HG_PLAN_MAGIC;
    p->graph_wanted = use_graph();
    p->info.steps = steps;
    for (uint64_t i = 0; i < nOps; ++i) p->info.algorithmicBytes += ops[i].bytes * (ops[i].kind ? 3u : 2u);
    const int rc = lower_ops(p, ops, nOps, buffers, (int)dataType, (int)reduceOp);
    if (rc != HCCL_SUCCESS) {
        HcommGfxPlanDestroy(p);
        return rc;
    }
    p->info.launches = p->nlaunch;
    *plan = p;
    return HCCL_SUCCESS;
}

int32_t HcommGfxPlanCreateFromOpsKeepInputs(
    const HcommGfxSchedOp* ops, uint64_t nOps, uint32_t nRanks, void* const* in, void* const* out, HcommDataType dataType,
    HcommReduceOp reduceOp, HcommGfxPlan** plan)
{
    if (!plan) return HCCL_E_PTR;
    *plan = NULL;
    if ((nOps && !ops) || !in || !out) return HCCL_E_PTR;
    if (nRanks == 0 || nRanks > HCOMM_GFX_MAX_RANKS) return HCCL_E_PARA;
    if (!hg_reduce_supported((int)dataType, (int)reduceOp, 1)) return HCCL_E_PARA;
    int rc = check_bufs(in, nRanks);
    if (rc == HCCL_SUCCESS) rc = check_bufs(out, nRanks);
    if (rc != HCCL_SUCCESS) return rc;
    const uint32_t unit = HcommGfxDataTypeSize(dataType);
    uint32_t steps = 0;
    for (uint64_t i = 0; i < nOps; ++i) {
        const HcommGfxSchedOp* o = &ops[i];
        /* roles 0, 1, 2 only: the communication buffers exist in the list but not in the launch */
        if (o->kind > 1 || o->rank >= nRanks || o->srcRank >= nRanks || o->dstBuf > 2u || o->srcBuf > 2u) return HCCL_E_PARA;
        if (o->kind == 1 && o->bytes % unit) return HCCL_E_PARA;
        if (i && o->step < ops[i - 1].step) return HCCL_E_PARA;
        if (o->step + 1 > steps) steps = o->step + 1;
    }
    HcommGfxPlan* p = (HcommGfxPlan*)calloc(1, sizeof(*p));
    if (!p) return HCCL_E_MEMORY;
    p->magic = HG_PLAN_MAGIC;
    p->graph_wanted = use_graph();
    p->info.steps = steps;
    for (uint64_t i = 0; i < nOps; ++i) p->info.algorithmicBytes += ops[i].bytes * (ops[i].kind ? 3u : 2u);
    HgOpList ol;
    memset(&ol, 0, sizeof(ol));
    ol.ops = (HcommGfxSchedOp*)ops; /* only read */
    ol.n = nOps;
    ol.steps = steps;
    rc = fused_from_trees(p, &ol, nRanks, in, out, (int)dataType, (int)reduceOp, 1);
    if (rc != HCCL_SUCCESS) {
        HcommGfxPlanDestroy(p);
        return rc;
    }
    p->info.launches = p->nlaunch;
    *plan = p;
    return HCCL_SUCCESS;
}

int32_t HcommGfxHierPlanCreate(
    HcommGfxAlgorithm level1Alg, uint32_t nServers, uint32_t nLocal, void* const* in, void* const* out, uint64_t count,
    HcommDataType dataType, HcommReduceOp reduceOp, HcommGfxPlan** plan)
{
    if (!plan) return HCCL_E_PTR;
    *plan = NULL;
    if (!in || !out) return HCCL_E_PTR;
    if (nServers == 0 || nLocal == 0 || (uint64_t)nServers * nLocal > HCOMM_GFX_MAX_RANKS) return HCCL_E_PARA;
    if (!hg_reduce_supported((int)dataType, (int)reduceOp, 1)) return HCCL_E_PARA;
    int rc = check_bufs(in, nServers * nLocal);
    if (rc == HCCL_SUCCESS) rc = check_bufs(out, nServers * nLocal);
    if (rc != HCCL_SUCCESS) return rc;
    HgOpList ol;
    rc = hg_schedule_hier(&ol, 0, (int)level1Alg, nServers, nLocal, count, (int)dataType);
    if (rc != HCCL_SUCCESS) return rc;
    void* const* bufs[HCOMM_GFX_NUM_BUFS] = {in, out, NULL, NULL, NULL};
    rc = HcommGfxPlanCreateFromOps(ol.ops, ol.n, nServers * nLocal, bufs, dataType, reduceOp, plan);
    hg_oplist_free(&ol);
    return rc;
}

int32_t HcommGfxMeshHierPlanCreate(
    HcommGfxAlgorithm level1Alg, uint32_t nServers, uint32_t nLocal, void* const* in, void* const* out, uint64_t count,
    HcommDataType dataType, HcommReduceOp reduceOp, HcommGfxPlan** plan)
{
    if (!plan) return HCCL_E_PTR;
    *plan = NULL;
    if (!in || !out) return HCCL_E_PTR;
    if (nServers == 0 || nLocal == 0 || (uint64_t)nServers * nLocal > HCOMM_GFX_MAX_RANKS) return HCCL_E_PARA;
    if (!hg_reduce_supported((int)dataType, (int)reduceOp, 1)) return HCCL_E_PARA;
    int rc = check_bufs(in, nServers * nLocal);
    if (rc == HCCL_SUCCESS) rc = check_bufs(out, nServers * nLocal);
    if (rc != HCCL_SUCCESS) return rc;
    HgOpList ol;
    rc = hg_schedule_hier(&ol, 1, (int)level1Alg, nServers, nLocal, count, (int)dataType);
    if (rc != HCCL_SUCCESS) return rc;
    void* const* bufs[HCOMM_GFX_NUM_BUFS] = {in, out, NULL, NULL, NULL};
    rc = HcommGfxPlanCreateFromOps(ol.ops, ol.n, nServers * nLocal, bufs, dataType, reduceOp, plan);
    hg_oplist_free(&ol);
    return rc;
}

int32_t HcommGfxDoubleRingPlanCreate(
    HcommGfxAlgorithm level1Alg, uint32_t nServers, uint32_t nLocal, void* const* userIn, void* const* userOut,
    void* const* cclIn, void* const* cclOut, uint64_t cclBytes, uint64_t count, HcommDataType dataType,
    HcommReduceOp reduceOp, HcommGfxPlan** plan)
{
    if (!plan) return HCCL_E_PTR;
    *plan = NULL;
    if (!userIn || !userOut || !cclIn || !cclOut) return HCCL_E_PTR;
    if (nServers == 0 || nLocal == 0 || (uint64_t)nServers * nLocal > HCOMM_GFX_MAX_RANKS) return HCCL_E_PARA;
    if (!hg_reduce_supported((int)dataType, (int)reduceOp, 1)) return HCCL_E_PARA;
    const uint32_t n = nServers * nLocal;
    int rc = check_bufs(userIn, n);
    if (rc == HCCL_SUCCESS) rc = check_bufs(userOut, n);
    if (rc == HCCL_SUCCESS) rc = check_bufs(cclIn, n);
    if (rc == HCCL_SUCCESS) rc = check_bufs(cclOut, n);
    if (rc != HCCL_SUCCESS) return rc;
    HgOpList ol;
    rc = hg_schedule_dbring(&ol, (int)level1Alg, nServers, nLocal, count, cclBytes, (int)dataType);
    if (rc != HCCL_SUCCESS) return rc;
    void* const* bufs[HCOMM_GFX_NUM_BUFS] = {cclIn, cclOut, NULL, userIn, userOut};
    rc = HcommGfxPlanCreateFromOps(ol.ops, ol.n, n, bufs, dataType, reduceOp, plan);
    hg_oplist_free(&ol);
    return rc;
}

int32_t HcommGfxOrderPreservedPlanCreate(
    uint32_t nRanks, void* const* userIn, void* const* userOut, void* const* cclOut, uint64_t cclBytes, uint64_t count,
    HcommDataType dataType, HcommReduceOp reduceOp, HcommGfxPlan** plan)
{
    if (!plan) return HCCL_E_PTR;
    *plan = NULL;
    if (!userIn || !userOut || !cclOut) return HCCL_E_PTR;
    if (nRanks < 2 || nRanks > HCOMM_GFX_MAX_RANKS) return HCCL_E_PARA;
    if (!hg_reduce_supported((int)dataType, (int)reduceOp, 1)) return HCCL_E_PARA;
    int rc = check_bufs(userIn, nRanks);
    if (rc == HCCL_SUCCESS) rc = check_bufs(userOut, nRanks);
    if (rc == HCCL_SUCCESS) rc = check_bufs(cclOut, nRanks);
    if (rc != HCCL_SUCCESS) return rc;
    HgOpList ol;
    rc = hg_schedule_order_preserved(&ol, nRanks, count, cclBytes, (int)dataType);
    if (rc != HCCL_SUCCESS) return rc;
    void* const* bufs[HCOMM_GFX_NUM_BUFS] = {NULL, cclOut, NULL, userIn, userOut};
    rc = HcommGfxPlanCreateFromOps(ol.ops, ol.n, nRanks, bufs, dataType, reduceOp, plan);
    hg_oplist_free(&ol);
    return rc;
}

int32_t HcommGfxOrderPreservedAllReducePlanCreate(
    uint32_t nRanks, void* const* userIn, void* const* userOut, void* const* cclIn, void* const* cclOut,
    uint64_t cclBytes, uint64_t count, HcommDataType dataType, HcommReduceOp reduceOp, HcommGfxPlan** plan)
{
    if (!plan) return HCCL_E_PTR;
    *plan = NULL;
    if (!userIn || !userOut || !cclIn || !cclOut) return HCCL_E_PTR;
    if (nRanks < 2 || nRanks > HCOMM_GFX_MAX_RANKS) return HCCL_E_PARA;
    if (!hg_reduce_supported((int)dataType, (int)reduceOp, 1)) return HCCL_E_PARA;
    int rc = check_bufs(userIn, nRanks);
    if (rc == HCCL_SUCCESS) rc = check_bufs(userOut, nRanks);
    if (rc == HCCL_SUCCESS) rc = check_bufs(cclIn, nRanks);
    if (rc == HCCL_SUCCESS) rc = check_bufs(cclOut, nRanks);
    if (rc != HCCL_SUCCESS) return rc;
    HgOpList ol;
    rc = hg_schedule_order_preserved_ar(&ol, nRanks, count, cclBytes, (int)dataType);
    if (rc != HCCL_SUCCESS) return rc;
    void* const* bufs[HCOMM_GFX_NUM_BUFS] = {cclIn, cclOut, NULL, userIn, userOut};
    rc = HcommGfxPlanCreateFromOps(ol.ops, ol.n, nRanks, bufs, dataType, reduceOp, plan);
    hg_oplist_free(&ol);
    return rc;
}

int32_t HcommGfxOrderPreservedHierAllReducePlanCreate(
    HcommGfxAlgorithm level1Alg, uint32_t nServers, uint32_t nLocal, void* const* userIn, void* const* userOut,
    void* const* cclIn, void* const* cclOut, uint64_t cclBytes, uint64_t count, HcommDataType dataType,
    HcommReduceOp reduceOp, HcommGfxPlan** plan)
{
    if (!plan) return HCCL_E_PTR;
    *plan = NULL;
    if (!userIn || !userOut || !cclIn || !cclOut) return HCCL_E_PTR;
    if (nServers < 2 || nLocal < 1 || (uint64_t)nServers * nLocal > HCOMM_GFX_MAX_RANKS) return HCCL_E_PARA;
    if (!hg_reduce_supported((int)dataType, (int)reduceOp, 1)) return HCCL_E_PARA;
    const uint32_t n = nServers * nLocal;
    int rc = check_bufs(userIn, n);
    if (rc == HCCL_SUCCESS) rc = check_bufs(userOut, n);
    if (rc == HCCL_SUCCESS) rc = check_bufs(cclIn, n);
    if (rc == HCCL_SUCCESS) rc = check_bufs(cclOut, n);
    if (rc != HCCL_SUCCESS) return rc;
    HgOpList ol;
    rc = hg_schedule_order_preserved_ar2(&ol, (int)level1Alg, nServers, nLocal, count, cclBytes, (int)dataType);
    if (rc != HCCL_SUCCESS) return rc;
    void* const* bufs[HCOMM_GFX_NUM_BUFS] = {cclIn, cclOut, NULL, userIn, userOut};
    rc = HcommGfxPlanCreateFromOps(ol.ops, ol.n, n, bufs, dataType, reduceOp, plan);
    hg_oplist_free(&ol);
    return rc;
}

int32_t HcommGfxOrderPreservedSmallPlanCreate(
    uint32_t nRanks, void* const* userIn, void* const* userOut, void* const* cclOut, uint64_t cclBytes, uint64_t count,
    HcommDataType dataType, HcommReduceOp reduceOp, HcommGfxPlan** plan)
{
    if (!plan) return HCCL_E_PTR;
    *plan = NULL;
    if (!userIn || !userOut || !cclOut) return HCCL_E_PTR;
    if (nRanks != 4 && nRanks != 8) return HCCL_E_PARA;
    if (!hg_reduce_supported((int)dataType, (int)reduceOp, 1)) return HCCL_E_PARA;
    int rc = check_bufs(userIn, nRanks);
    if (rc == HCCL_SUCCESS) rc = check_bufs(userOut, nRanks);
    if (rc == HCCL_SUCCESS) rc = check_bufs(cclOut, nRanks);
    if (rc != HCCL_SUCCESS) return rc;
    HgOpList ol;
    rc = hg_schedule_order_preserved_small(&ol, nRanks, count, cclBytes, (int)dataType);
    if (rc != HCCL_SUCCESS) return rc;
    void* const* bufs[HCOMM_GFX_NUM_BUFS] = {NULL, cclOut, NULL, userIn, userOut};
    rc = HcommGfxPlanCreateFromOps(ol.ops, ol.n, nRanks, bufs, dataType, reduceOp, plan);
    hg_oplist_free(&ol);
    return rc;
}

int32_t HcommGfxOrderPreservedHierReduceScatterPlanCreate(
    uint32_t nServers, uint32_t nLocal, void* const* userIn, void* const* userOut, void* const* cclIn, void* const* cclOut,
    uint64_t cclBytes, uint64_t count, HcommDataType dataType, HcommReduceOp reduceOp, HcommGfxPlan** plan)
{
    if (!plan) return HCCL_E_PTR;
    *plan = NULL;
    if (!userIn || !userOut || !cclOut) return HCCL_E_PTR;
    if (nServers < 2 || nLocal < 1 || (uint64_t)nServers * nLocal > HCOMM_GFX_MAX_RANKS) return HCCL_E_PARA;
    if (!hg_reduce_supported((int)dataType, (int)reduceOp, 1)) return HCCL_E_PARA;
    const uint32_t n = nServers * nLocal;
    int rc = check_bufs(userIn, n);
    if (rc == HCCL_SUCCESS) rc = check_bufs(userOut, n);
    if (rc == HCCL_SUCCESS) rc = check_bufs(cclOut, n);
    if (rc == HCCL_SUCCESS && nLocal == 1) rc = check_bufs(cclIn, n); /* only one device per module stages there */
    if (rc != HCCL_SUCCESS) return rc;
    HgOpList ol;
    rc = hg_schedule_order_preserved_rs2(&ol, nServers, nLocal, count, cclBytes, (int)dataType);
    if (rc != HCCL_SUCCESS) return rc;
    void* const* bufs[HCOMM_GFX_NUM_BUFS] = {nLocal == 1 ? cclIn : NULL, cclOut, NULL, userIn, userOut};
    rc = HcommGfxPlanCreateFromOps(ol.ops, ol.n, n, bufs, dataType, reduceOp, plan);
    hg_oplist_free(&ol);
    return rc;
}

/* The order-preserving executors in one launch: the N user inputs are folded in registers along the executors' tree
 * and the root is written to the user output(s).  No CCL buffer is read or written.
 * One server: rounds h = 2^(S-1), .., 1 fold contribution h + j onto contribution j
 * (reduce_scatter_plant_local_reduce.cc:337-414) - a balanced tree whose leaf q is rank bitrev(q).
 * Servers x devices: that tree over a server's devices first, then the same shape over the servers
 * (reduce_scatter_plant_local_reduce_combine.cc:232-304) - leaf q = (server bitrev(high bits), device bitrev(low bits)). */
int32_t HcommGfxOrderPreservedFusedPlanCreate(
    int32_t allReduce, uint32_t nServers, uint32_t nLocal, void* const* userIn, void* const* userOut, uint64_t count,
    HcommDataType dataType, HcommReduceOp reduceOp, HcommGfxPlan** plan)
{
    if (!plan) return HCCL_E_PTR;
    *plan = NULL;
    if (nServers == 0 || nLocal == 0 || (uint64_t)nServers * nLocal < 2 || (uint64_t)nServers * nLocal > HCOMM_GFX_MAX_RANKS)
        return HCCL_E_PARA;
    if (!hg_reduce_supported((int)dataType, (int)reduceOp, 1)) return HCCL_E_PARA;
    const uint32_t nRanks = nServers * nLocal;
    int rc = check_bufs(userIn, nRanks);
    if (rc == HCCL_SUCCESS) rc = check_bufs(userOut, nRanks);
    if (rc != HCCL_SUCCESS) return rc;
    uint32_t bits_l = 0, bits_s = 0;
    while ((1u << bits_l) < nLocal) ++bits_l;
    while ((1u << bits_s) < nServers) ++bits_s;
    /* the kernel folds at most 32 leaf positions, holes included (5 x 6 ranks would need 8 x 8) */
    if (bits_l + bits_s > 5u) return HCCL_E_NOT_SUPPORT;
    const uint64_t block = count * HcommGfxDataTypeSize(dataType);
    /* the reduce-scatter reads block p of every input at p * block: 128-bit accesses need 16-byte multiples */
    if (!allReduce && (block & (HG_VEC_BYTES - 1u))) return HCCL_E_NOT_SUPPORT;
    /* steps and algorithmic bytes are those of the step-wise plan with an unbounded CCL buffer (a single chunk) */
    HgOpList ol;
    const uint64_t unbounded = (uint64_t)1 << 62;
    if (nServers == 1)
        rc = allReduce ? hg_schedule_order_preserved_ar(&ol, nRanks, count, unbounded, (int)dataType)
                       : hg_schedule_order_preserved(&ol, nRanks, count, unbounded, (int)dataType);
    else
        rc = allReduce ? hg_schedule_order_preserved_ar2(&ol, HCOMM_GFX_ALG_ALLREDUCE_RING, nServers, nLocal, count, unbounded,
                                                         (int)dataType)
                       : hg_schedule_order_preserved_rs2(&ol, nServers, nLocal, count, unbounded, (int)dataType);
    if (rc != HCCL_SUCCESS) return rc;
    HcommGfxPlan* p = (HcommGfxPlan*)calloc(1, sizeof(*p));
    if (!p) {
        hg_oplist_free(&ol);
        return HCCL_E_MEMORY;
    }
    p->magic = HG_PLAN_MAGIC;
    p->graph_wanted = use_graph();
    p->info.steps = ol.steps;
    for (uint64_t i = 0; i < ol.n; ++i) p->info.algorithmicBytes += ol.ops[i].bytes * (ol.ops[i].kind ? 3u : 2u);
    hg_oplist_free(&ol);
    if (block) {
        HgLaunch* l = (HgLaunch*)calloc(1, sizeof(HgLaunch));
        if (!l) {
            HcommGfxPlanDestroy(p);
            return HCCL_E_MEMORY;
        }
        l->kind = HCOMM_GFX_KERNEL_TREE;
        l->dtype = (uint32_t)dataType;
        l->op = (uint32_t)reduceOp;
        HgFoldTable* f = &l->tab.fold;
        f->tree = 4u;
        f->k = rank_order_positions(nServers, nLocal, f->pos);
        f->nranks = nRanks;
        for (uint32_t r = 0; r < nRanks; ++r) {
            f->in[r] = userIn[r];
            f->out[r] = userOut[r];
        }
        if (allReduce) {
            f->nout = nRanks;
            f->out_mode = 2u;
            f->nseg = 1;
            f->bytes[0] = block;
        } else {
            f->out_mode = 1u;
            f->nseg = nRanks;
            for (uint32_t r = 0; r < nRanks; ++r) {
                f->off[r] = block * r;
                f->bytes[r] = block;
                f->owner[r] = (uint8_t)r;
            }
        }
        hg_finish_fold(l);
        rc = plan_push(l, p);
        free(l);
        if (rc != HCCL_SUCCESS) {
            HcommGfxPlanDestroy(p);
            return rc;
        }
    }
    p->info.launches = p->nlaunch;
    *plan = p;
    return HCCL_SUCCESS;
}

int32_t HcommGfxHierReduceScatterPlanCreate(
    int32_t level0Mesh, HcommGfxAlgorithm level1Alg, uint32_t nServers, uint32_t nLocal, void* const* userIn,
    void* const* userOut, void* const* cclIn, void* const* cclOut, uint64_t cclBytes, uint64_t count,
    HcommDataType dataType, HcommReduceOp reduceOp, HcommGfxPlan** plan)
{
    if (!plan) return HCCL_E_PTR;
    *plan = NULL;
    if (!userIn || !userOut || !cclIn || !cclOut) return HCCL_E_PTR;
    if (nServers == 0 || nLocal == 0 || (uint64_t)nServers * nLocal > HCOMM_GFX_MAX_RANKS) return HCCL_E_PARA;
    if (!hg_reduce_supported((int)dataType, (int)reduceOp, 1)) return HCCL_E_PARA;
    const uint32_t n = nServers * nLocal;
    int rc = check_bufs(userIn, n);
    if (rc == HCCL_SUCCESS) rc = check_bufs(userOut, n);
    if (rc == HCCL_SUCCESS) rc = check_bufs(cclIn, n);
    if (rc == HCCL_SUCCESS) rc = check_bufs(cclOut, n);
    if (rc != HCCL_SUCCESS) return rc;
    HgOpList ol;
    rc = hg_schedule_hier_rs(&ol, level0Mesh != 0, (int)level1Alg, nServers, nLocal, count, cclBytes, (int)dataType);
    if (rc != HCCL_SUCCESS) return rc;
    void* const* bufs[HCOMM_GFX_NUM_BUFS] = {cclIn, cclOut, NULL, userIn, userOut};
    rc = HcommGfxPlanCreateFromOps(ol.ops, ol.n, n, bufs, dataType, reduceOp, plan);
    hg_oplist_free(&ol);
    return rc;
}

int32_t HcommGfxDoubleRingReduceScatterPlanCreate(
    uint32_t nRanks, void* const* userIn, void* const* userOut, void* const* cclIn, uint64_t cclBytes, uint64_t count,
    HcommDataType dataType, HcommReduceOp reduceOp, HcommGfxPlan** plan)
{
    if (!plan) return HCCL_E_PTR;
    *plan = NULL;
    if (!userIn || !userOut || !cclIn) return HCCL_E_PTR;
    if (nRanks < 3 || nRanks > HCOMM_GFX_MAX_RANKS) return HCCL_E_PARA;
    if (!hg_reduce_supported((int)dataType, (int)reduceOp, 1)) return HCCL_E_PARA;
    int rc = check_bufs(userIn, nRanks);
    if (rc == HCCL_SUCCESS) rc = check_bufs(userOut, nRanks);
    if (rc == HCCL_SUCCESS) rc = check_bufs(cclIn, nRanks);
    if (rc != HCCL_SUCCESS) return rc;
    HgOpList ol;
    rc = hg_schedule_dbring_rs(&ol, nRanks, count, cclBytes, (int)dataType);
    if (rc != HCCL_SUCCESS) return rc;
    void* const* bufs[HCOMM_GFX_NUM_BUFS] = {cclIn, NULL, NULL, userIn, userOut};
    rc = HcommGfxPlanCreateFromOps(ol.ops, ol.n, nRanks, bufs, dataType, reduceOp, plan);
    hg_oplist_free(&ol);
    return rc;
}

int32_t HcommGfxDoubleRingHierReduceScatterPlanCreate(
    HcommGfxAlgorithm level1Alg, HcommGfxAlgorithm level2Alg, uint32_t nPods, uint32_t nServers, uint32_t nLocal,
    void* const* userIn, void* const* userOut, void* const* cclIn, uint64_t cclBytes, uint64_t count, HcommDataType dataType,
    HcommReduceOp reduceOp, HcommGfxPlan** plan)
{
    if (!plan) return HCCL_E_PTR;
    *plan = NULL;
    if (!userIn || !userOut || !cclIn) return HCCL_E_PTR;
    if (nPods == 0 || nServers == 0 || (uint64_t)nPods * nServers < 2 || nLocal < 3 ||
        (uint64_t)nPods * nServers * nLocal > HCOMM_GFX_MAX_RANKS)
        return HCCL_E_PARA;
    if (!hg_reduce_supported((int)dataType, (int)reduceOp, 1)) return HCCL_E_PARA;
    const uint32_t n = nPods * nServers * nLocal;
    int rc = check_bufs(userIn, n);
    if (rc == HCCL_SUCCESS) rc = check_bufs(userOut, n);
    if (rc == HCCL_SUCCESS) rc = check_bufs(cclIn, n);
    if (rc != HCCL_SUCCESS) return rc;
    HgOpList ol;
    rc = hg_schedule_dbring_rs_servers(&ol, (int)level1Alg, (int)level2Alg, nPods, nServers, nLocal, count, cclBytes, (int)dataType);
    if (rc != HCCL_SUCCESS) return rc;
    void* const* bufs[HCOMM_GFX_NUM_BUFS] = {cclIn, NULL, NULL, userIn, userOut};
    rc = HcommGfxPlanCreateFromOps(ol.ops, ol.n, n, bufs, dataType, reduceOp, plan);
    hg_oplist_free(&ol);
    return rc;
}

int32_t HcommGfxPlanRunRange(const HcommGfxPlan* plan, ThreadHandle thread, uint32_t first, uint32_t n)
{
    if (!plan || plan->magic != HG_PLAN_MAGIC) return HCCL_E_PTR;
    HgThread* t = hg_thread_from_handle(thread);
    if (!t) return HCCL_E_PTR;
    if (first > plan->nlaunch || n > plan->nlaunch - first) return HCCL_E_PARA;
    /* a plan's launches are submitted at once: inside a batch they would run ahead of what the batch has recorded */
    if (hg_caller_is_batching()) return HCCL_E_NOT_SUPPORT;
    if (hg_thread_free_for_caller(t) != HCCL_SUCCESS) return HCCL_E_UNAVAIL;
    for (uint32_t i = first; i < first + n; ++i) {
        int rc = hg_submit(t, &plan->launches[i]);
        if (rc != HCCL_SUCCESS) return rc;
    }
    return HCCL_SUCCESS;
}

int32_t HcommGfxPlanRun(const HcommGfxPlan* plan, ThreadHandle thread)
{
    if (!plan || plan->magic != HG_PLAN_MAGIC) return HCCL_E_PTR;
    HgThread* t = hg_thread_from_handle(thread);
    if (!t) return HCCL_E_PTR;
    HcommGfxPlan* p = (HcommGfxPlan*)plan; /* the graph is a cache, not part of the plan's meaning */
    if (!t->recorder) { /* before anything is captured on or launched into the stream */
        const int rc = hg_thread_settle(t);
        if (rc != HCCL_SUCCESS) return rc;
    }
    if (t->recorder || p->nlaunch < 2 || !p->graph_wanted || p->graph_state < 0 || hg_rt_stream_is_capturing(t->stream))
        return HcommGfxPlanRunRange(plan, thread, 0, plan->nlaunch);
    if (p->graph_state == 1 && p->graph_stream != t->stream) {
        hg_rt_graph_destroy(p->graph_exec);
        p->graph_exec = NULL;
        p->graph_state = 0;
    }
    if (p->graph_state == 0) {
        if (hg_rt_capture_begin(t->stream) != HCCL_SUCCESS) {
            p->graph_state = -1;
            return HcommGfxPlanRunRange(plan, thread, 0, plan->nlaunch);
        }
        const int saved = t->log_enabled;
        t->log_enabled = 0;
        int rc = HcommGfxPlanRunRange(plan, thread, 0, plan->nlaunch);
        t->log_enabled = saved;
        void* exec = NULL;
        const int rc2 = hg_rt_capture_end(t->stream, &exec);
        if (rc != HCCL_SUCCESS || rc2 != HCCL_SUCCESS) {
            if (exec) hg_rt_graph_destroy(exec);
            p->graph_state = -1;
            return HcommGfxPlanRunRange(plan, thread, 0, plan->nlaunch);
        }
        p->graph_exec = exec;
        p->graph_stream = t->stream;
        p->graph_state = 1;
    }
    for (uint32_t i = 0; i < p->nlaunch; ++i) hg_log_only(t, &p->launches[i]);
    return hg_rt_graph_launch(p->graph_exec, t->stream);
}

int32_t HcommGfxPlanSetGraphReplay(HcommGfxPlan* plan, int32_t enable)
{
    if (!plan || plan->magic != HG_PLAN_MAGIC) return HCCL_E_PTR;
    plan->graph_wanted = enable ? 1 : 0;
    if (plan->graph_state < 0) plan->graph_state = 0;
    return HCCL_SUCCESS;
}

int32_t HcommGfxPlanDestroy(HcommGfxPlan* plan)
{
    if (!plan || plan->magic != HG_PLAN_MAGIC) return HCCL_E_PTR;
    plan->magic = 0;
    if (plan->graph_exec) hg_rt_graph_destroy(plan->graph_exec);
    free(plan->launches);
    free(plan);
    return HCCL_SUCCESS;
}

int32_t HcommGfxPlanGetInfo(const HcommGfxPlan* plan, HcommGfxPlanInfo* info)
{
    if (!plan || plan->magic != HG_PLAN_MAGIC || !info) return HCCL_E_PTR;
    *info = plan->info;
    return HCCL_SUCCESS;
}

int32_t HcommGfxPlanGetLaunch(const HcommGfxPlan* plan, uint32_t i, HcommGfxLaunchRecord* rec)
{
    if (!plan || plan->magic != HG_PLAN_MAGIC || !rec) return HCCL_E_PTR;
    if (i >= plan->nlaunch) return HCCL_E_PARA;
    const HgLaunch* l = &plan->launches[i];
    rec->kind = l->kind;
    rec->dtype = l->dtype;
    rec->op = l->op;
    rec->nseg = l->nseg;
    rec->bytes = l->bytes;
    rec->blocks = l->blocks;
    rec->rows = hg_launch_rows(l);
    rec->streaming = l->streaming;
    rec->backwards = 0;
    rec->reserved = 0;
    return HCCL_SUCCESS;
}

int32_t HcommGfxPlanGetTreeSegment(const HcommGfxPlan* plan, uint32_t i, uint32_t segment, const void** leaves,
                                   uint32_t cap, uint32_t* k, uint64_t* offset, uint64_t* bytes, int32_t* outRank)
{
    if (!plan || plan->magic != HG_PLAN_MAGIC || !k) return HCCL_E_PTR;
    if (i >= plan->nlaunch) return HCCL_E_PARA;
    const HgLaunch* l = &plan->launches[i];
    const HgFoldTable* f = &l->tab.fold;
    if (l->kind != HCOMM_GFX_KERNEL_TREE || segment >= f->nseg) return HCCL_E_PARA;
    *k = f->k;
    if (offset) *offset = f->off[segment];
    if (bytes) *bytes = f->bytes[segment];
    if (outRank) *outRank = f->out_mode == 1u ? (int32_t)f->owner[segment] : -1;
    if (!leaves) return HCCL_SUCCESS;
    if (cap < f->k) return HCCL_E_PARA;
    const uint32_t n = f->nranks, c = f->first[segment];
    uint32_t bits = 0;
    while ((1u << bits) < f->k) ++bits;
    for (uint32_t q = 0; q < f->k; ++q) {
        uint32_t b = 255;
        switch (f->tree) {
            case 1u: b = c ^ bitrev_n(q, bits); break;
            case 2u: b = q < n ? (c + q) % n : 255u; break;
            case 3u: b = q < n ? (c + n - q) % n : 255u; break;
            case 4u: b = f->pos[q]; break;
            case 5u: b = f->pos[q] < n ? (c + n - f->pos[q]) % n : 255u; break;
            default: b = f->pos[segment * f->k + q]; break;
        }
        leaves[q] = b < n ? f->in[b] : NULL;
    }
    return HCCL_SUCCESS;
}
