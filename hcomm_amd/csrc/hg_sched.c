/*
 * hg_sched.c - slice tables and the step lists of the ring, recursive halving-doubling and mesh schedules.
 *
 * Each generator states the schedule in closed form per step t (all ranks act in parallel inside a step)
 * and emits the two-input operations the reference's templates hand to the dispatcher: a copy
 * (HcclD2DMemcpyAsync) or a reduce dst = dst (op) src (HcclReduceAsync) - src/legacy/ascend910/platform/task/
 * dispatcher_common.cc:114-147.  Paths below are relative to
 * src/legacy/ascend910/algorithm/base/alg_template/.  The reduce operand roles follow the inline-reduce branch
 * of Reducer::run (component/reducer.cc:199-222): dst is the local buffer, src the peer's.
 */
#include <stdlib.h>
#include <string.h>

#include "hg_host.h"
#include "hg_sched.h"

#define HG_SLICE_ALIGN 128u /* HCCL_MIN_SLICE_ALIGN, alg_template_base_pub.h:43 */

int32_t HcommGfxCalcSlices(uint64_t count, uint32_t unitSize, uint32_t n, HcommGfxSlice* slices)
{
    if (!slices) return HCCL_E_PTR;
    if (unitSize == 0 || n == 0) return HCCL_E_PARA;
    if (count > ((uint64_t)1 << 62) / unitSize) return HCCL_E_PARA; /* the byte total and its roundings stay in 64 bits */
    /* temp_all_reduce/all_reduce_ring.cc:142-153; RoundUpWithDivisor(0, 128) is 128 (alg_template_base_pub.h:609-616) */
    const uint64_t total = count * unitSize;
    const uint64_t per_raw = (total + (n - 1)) / n;
    const uint64_t per = (per_raw == 0) ? HG_SLICE_ALIGN : ((per_raw + HG_SLICE_ALIGN - 1) / HG_SLICE_ALIGN) * HG_SLICE_ALIGN;
    uint64_t residue = total;
    for (uint32_t i = 0; i < n; ++i) {
        slices[i].size = residue > per ? per : residue;
        slices[i].offset = total - residue;
        residue -= slices[i].size;
    }
    return HCCL_SUCCESS;
}

void hg_oplist_free(HgOpList* l)
{
    if (!l->fixed) free(l->ops);
    memset(l, 0, sizeof(*l));
}

static int push(HgOpList* l, uint32_t step, uint32_t kind, uint32_t rank, uint32_t dst_buf, uint64_t dst_off,
                uint32_t src_rank, uint32_t src_buf, uint64_t src_off, uint64_t bytes)
{
    if (step + 1 > l->steps) l->steps = step + 1;
    if (bytes == 0) return HCCL_SUCCESS; /* zero-size slices produce no work (dispatcher.cc:495-498, 719-722) */
    if (l->n == l->cap) {
        if (l->fixed) return HCCL_E_INTERNAL;
        uint64_t cap = l->cap ? l->cap * 2 : 256;
        HcommGfxSchedOp* p = (HcommGfxSchedOp*)realloc(l->ops, cap * sizeof(*p));
        if (!p) return HCCL_E_MEMORY;
        l->ops = p;
        l->cap = cap;
    }
    HcommGfxSchedOp* o = &l->ops[l->n++];
    o->step = step;
    o->kind = kind;
    o->rank = rank;
    o->dstBuf = dst_buf;
    o->srcRank = src_rank;
    o->srcBuf = src_buf;
    o->dstOff = dst_off;
    o->srcOff = src_off;
    o->bytes = bytes;
    return HCCL_SUCCESS;
}

#define IN 0u
#define OUT 1u
#define COPY 0u
#define REDUCE 1u
#define CHK(x)                                \
    do {                                      \
        int rc_ = (x);                        \
        if (rc_ != HCCL_SUCCESS) return rc_;  \
    } while (0)

static uint32_t modn(int64_t v, uint32_t n)
{
    int64_t r = v % (int64_t)n;
    return (uint32_t)(r < 0 ? r + n : r);
}

/* Ring reduce-scatter over `sl` in the input buffers: step t, rank r reduces slice (r-2-t) from its left
 * neighbour (temp_reduce_scatter/reduce_scatter_ring.cc:207,214,260,268; last step :288-304). */
static int ring_rs(HgOpList* l, uint32_t n, const HcommGfxSlice* sl, uint32_t step0)
{
    for (uint32_t t = 0; t + 1 < n; ++t)
        for (uint32_t r = 0; r < n; ++r) {
            const uint32_t c = modn((int64_t)r - 2 - t, n);
            CHK(push(l, step0 + t, REDUCE, r, IN, sl[c].offset, modn((int64_t)r - 1, n), IN, sl[c].offset, sl[c].size));
        }
    return HCCL_SUCCESS;
}

static int sched_allreduce_ring(HgOpList* l, uint32_t n, uint64_t count, uint32_t unit, int with_gather)
{
    const uint64_t total = count * unit;
    if (n == 1) /* temp_all_reduce/all_reduce_ring.cc:132-140; the staged reduce-scatter does nothing (:73-76) */
        return with_gather ? push(l, 0, COPY, 0, OUT, 0, 0, IN, 0, total) : HCCL_SUCCESS;
    HcommGfxSlice sl[HCOMM_GFX_MAX_RANKS];
    CHK(HcommGfxCalcSlices(count, unit, n, sl));
    CHK(ring_rs(l, n, sl, 0));
    if (!with_gather) return HCCL_SUCCESS;
    /* temp_all_gather/all_gather_ring.cc:116-121: own slice input -> output */
    for (uint32_t r = 0; r < n; ++r) CHK(push(l, n - 1, COPY, r, OUT, sl[r].offset, r, IN, sl[r].offset, sl[r].size));
    /* all_gather_ring.cc:143-206: round i receives slice (r-1-i) from the left neighbour's output */
    for (uint32_t i = 0; i + 1 < n; ++i)
        for (uint32_t r = 0; r < n; ++r) {
            const uint32_t c = modn((int64_t)r - 1 - i, n);
            CHK(push(l, n + i, COPY, r, OUT, sl[c].offset, modn((int64_t)r - 1, n), OUT, sl[c].offset, sl[c].size));
        }
    return HCCL_SUCCESS;
}

/* Input slice i of the scatter algorithms starts stride elements after slice i-1
 * (displs[i] = strideLen * i * unitSize, src/legacy/ascend910/framework/device/aicpu_kfc/algorithm/
 * aicpu_reduce_scatter.cc:78-80); stride == count is the dense layout of reduce_scatter_ring.cc:140-157. */
static int sched_rs_ring_standalone(HgOpList* l, uint32_t n, uint64_t count, uint64_t stride, uint32_t unit)
{
    const uint64_t sz = count * unit;
    if (n == 1) return push(l, 0, COPY, 0, OUT, 0, 0, IN, 0, sz); /* reduce_scatter_ring.cc:103-109 */
    HcommGfxSlice sl[HCOMM_GFX_MAX_RANKS];
    memset(sl, 0, sizeof(sl));
    for (uint32_t i = 0; i < n; ++i) { /* reduce_scatter_ring.cc:140-157; the output holds one slice, so offset 0 */
        sl[i].offset = (uint64_t)i * stride * unit;
        sl[i].size = sz;
    }
    CHK(ring_rs(l, n, sl, 0));
    /* last step reduces into the input slice, then copies it to the output (reducer.cc:209-218) */
    for (uint32_t r = 0; r < n; ++r) CHK(push(l, n - 1, COPY, r, OUT, 0, r, IN, sl[r].offset, sz));
    return HCCL_SUCCESS;
}

static uint32_t floor_pow2(uint32_t n)
{
    uint32_t b = 1;
    while ((b << 1) <= n) b <<= 1;
    return b;
}

static uint64_t sum_sizes(const HcommGfxSlice* sl, uint32_t first, uint32_t m)
{
    uint64_t s = 0;
    for (uint32_t i = 0; i < m; ++i) s += sl[first + i].size;
    return s;
}

static int sched_allreduce_rhd(HgOpList* l, uint32_t n, uint64_t count, uint32_t unit)
{
    const uint64_t total = count * unit;
    if (n == 1) return push(l, 0, COPY, 0, OUT, 0, 0, IN, 0, total); /* all_reduce_recursive_hd.cc:103-108 */
    /* recursive_halvingdoubling_base.cc:23-37 */
    const uint32_t block = floor_pow2(n);
    const uint32_t part1 = (n - block) * 2;
    uint32_t levels = 0;
    while ((1u << (levels + 1)) <= block) ++levels;
    HcommGfxSlice sl[HCOMM_GFX_MAX_RANKS];
    CHK(HcommGfxCalcSlices(count, unit, block, sl)); /* recursive_halvingdoubling_base.cc:64-94 */
    uint32_t real[HCOMM_GFX_MAX_RANKS]; /* block rank -> rank (recursive_halvingdoubling_base.cc:39-62) */
    for (uint32_t b = 0; b < block; ++b) real[b] = (b < part1 / 2) ? 2 * b : b + part1 / 2;
    uint32_t step = 0;
    if (part1 > 0) { /* fold: even ranks of part one absorb their odd neighbour (all_reduce_recursive_hd.cc:133-203) */
        for (uint32_t r = 0; r < part1; r += 2) CHK(push(l, step, REDUCE, r, IN, 0, r + 1, IN, 0, total));
        ++step;
    }
    /* halving reduce-scatter (temp_reduce_scatter/reduce_scatter_halving_doubling.cc:65-92,196-257) */
    for (uint32_t s = 0; s < levels; ++s, ++step) {
        const uint32_t m = 1u << (levels - 1 - s);
        for (uint32_t b = 0; b < block; ++b) {
            const uint32_t p = b ^ m, first = b & ~(m - 1);
            CHK(push(l, step, REDUCE, real[b], IN, sl[first].offset, real[p], IN, sl[first].offset, sum_sizes(sl, first, m)));
        }
    }
    /* reduce_scatter_halving_doubling.cc:251-254: the slice received last goes input -> output */
    for (uint32_t b = 0; b < block; ++b)
        CHK(push(l, step, COPY, real[b], OUT, sl[b].offset, real[b], IN, sl[b].offset, sl[b].size));
    ++step;
    /* doubling all-gather in the outputs (temp_all_gather/all_gather_halving_doubling.cc:42-66,164-206) */
    for (uint32_t s = 0; s < levels; ++s, ++step) {
        const uint32_t m = 1u << s;
        for (uint32_t b = 0; b < block; ++b) {
            const uint32_t p = b ^ m, first = p & ~(m - 1);
            CHK(push(l, step, COPY, real[b], OUT, sl[first].offset, real[p], OUT, sl[first].offset, sum_sizes(sl, first, m)));
        }
    }
    if (part1 > 0) { /* unfold: even -> odd, whole output (all_reduce_recursive_hd.cc:277-343) */
        for (uint32_t r = 1; r < part1; r += 2) CHK(push(l, step, COPY, r, OUT, 0, r - 1, OUT, 0, total));
        ++step;
    }
    return HCCL_SUCCESS;
}

static int sched_allreduce_mesh_oneshot(HgOpList* l, uint32_t n, uint64_t count, uint32_t unit, int ascending)
{
    /* temp_all_reduce/all_reduce_mesh_oneshot.cc:78-121: out = in, then reduce the peers' copies in the
     * order r+1, r+2, ..., r-1.  A peer's communication buffer holds a copy of its input (:96-100), which
     * the simulation reads as in[peer] directly. */
    const uint64_t total = count * unit;
    for (uint32_t r = 0; r < n; ++r) CHK(push(l, 0, COPY, r, OUT, 0, r, IN, 0, total));
    if (ascending) {
        /* src/legacy/ascend950/service/collective/alg/coll_alg_factory/alg_template/ins_alg_template/
         * ins_temp_all_reduce_mesh_1D_one_shot.cc:102,148-161: out = in, then every other rank's input in
         * ascending rank order (the gathered scratch copies are read as in[peer] directly) */
        for (uint32_t k = 1; k < n; ++k)
            for (uint32_t r = 0; r < n; ++r) CHK(push(l, k, REDUCE, r, OUT, 0, (k - 1 < r) ? k - 1 : k, IN, 0, total));
        return HCCL_SUCCESS;
    }
    for (uint32_t k = 1; k < n; ++k)
        for (uint32_t r = 0; r < n; ++r) CHK(push(l, k, REDUCE, r, OUT, 0, (r + k) % n, IN, 0, total));
    return HCCL_SUCCESS;
}

static int sched_rs_mesh(HgOpList* l, uint32_t n, uint64_t count, uint64_t stride, uint32_t unit)
{
    /* temp_reduce_scatter/reduce_scatter_mesh.cc:51-128 (stream 0): round k receives slice r from rank r-k
     * (ForwardRank, base/inc/reduce_scatter_mesh_pub.h:31-37) and reduces it into in[r][slice r]; then
     * :199-211 copies that slice to the output. */
    const uint64_t sz = count * unit;
    if (n == 1) return push(l, 0, COPY, 0, OUT, 0, 0, IN, 0, sz);
    for (uint32_t k = 1; k < n; ++k)
        for (uint32_t r = 0; r < n; ++r)
            CHK(push(l, k - 1, REDUCE, r, IN, (uint64_t)r * stride * unit, modn((int64_t)r - k, n), IN,
                     (uint64_t)r * stride * unit, sz));
    for (uint32_t r = 0; r < n; ++r) CHK(push(l, n - 1, COPY, r, OUT, 0, r, IN, (uint64_t)r * stride * unit, sz));
    return HCCL_SUCCESS;
}

#define SCR 2u

/* Slot size of the deterministic mesh allreduce: ceil(total / n) rounded up to 16 KiB, or to 512 B, or to the
 * element size, whichever is the first to keep n-1 slots within the message
 * (AllReduceLocalReduce::PrepareSlice, temp_all_reduce/all_reduce_local_reduce.cc:69-92, with the communication
 * buffer distinct from the user output so that sizeLimit = totalSize). */
static uint64_t local_reduce_slot(uint64_t total, uint32_t n, uint32_t unit)
{
    const uint64_t ori = (total + n - 1) / n;
    const uint64_t align[3] = {16384, 512, unit};
    uint64_t per = 0;
    for (int a = 0; a < 3; ++a) {
        per = (ori == 0) ? align[a] : ((ori + align[a] - 1) / align[a]) * align[a];
        if (per * (n - 1) <= total) break;
    }
    return per;
}

static void local_reduce_slices(uint64_t total, uint32_t n, uint32_t unit, HcommGfxSlice* sl, uint64_t* per_out)
{
    const uint64_t per = local_reduce_slot(total, n, unit);
    uint64_t residue = total;
    for (uint32_t i = 0; i < n; ++i) {
        sl[i].size = residue > per ? per : residue;
        sl[i].offset = residue ? total - residue : total;
        residue -= sl[i].size;
    }
    *per_out = per;
}

/* ReduceScatterLocalReduce: where rank i's receive window starts inside its communication buffer
 * (temp_reduce_scatter/reduce_scatter_local_reduce.cc:102-123: staggered by the slice's position in the user input
 * modulo 16 KiB once a slice exceeds 32 KiB) and the distance between the N-1 slots of the window (:162-178: the
 * slice size rounded up to 16 KiB; the communication buffer is sized so that this first choice always fits). */
static uint64_t rs_local_reduce_window(uint64_t total, uint32_t i)
{
    return total > 32u * 1024u ? ((uint64_t)i * total) % 16384u : 0;
}

static uint64_t rs_local_reduce_slot(uint64_t total) { return total == 0 ? 16384u : (total + 16383u) / 16384u * 16384u; }

uint64_t hg_scratch_bytes(int alg, uint32_t n, uint64_t count, int dtype)
{
    const uint32_t unit = HcommGfxDataTypeSize((HcommDataType)dtype);
    if (n < 2) return 0;
    if (alg == HCOMM_GFX_ALG_ALLREDUCE_CHUNK_MESH) return count * unit;
    if (alg == HCOMM_GFX_ALG_REDUCE_SCATTER_LOCAL_REDUCE) {
        uint64_t max_off = 0;
        for (uint32_t i = 0; i < n; ++i) {
            const uint64_t o = rs_local_reduce_window(count * unit, i);
            if (o > max_off) max_off = o;
        }
        return max_off + (uint64_t)(n - 1) * rs_local_reduce_slot(count * unit);
    }
    if (alg == HCOMM_GFX_ALG_REDUCE_SCATTER_WINDOW_HALVING) return (uint64_t)n * count * unit; /* one slot per rank */
    if (alg != HCOMM_GFX_ALG_ALLREDUCE_LOCAL_REDUCE) return 0;
    return (uint64_t)n * local_reduce_slot(count * unit, n, unit);
}

/* AllReduceChunkMesh, temp_all_reduce/all_reduce_chunk_mesh.cc (the communication buffer is not the user output:
 * the "single operator" branches).  Stated per sub-chunk: sub-chunk q of rank r's slice folds the peers' copies in
 * the rotation r+q+1, r+q+2, ..., wrapping from r+n-1 back to r+1 (:234-236), one peer per round. */
static int sched_allreduce_chunk_mesh(HgOpList* l, uint32_t n, uint64_t count, uint32_t unit)
{
    const uint64_t total = count * unit;
    if (n == 1) return push(l, 0, COPY, 0, OUT, 0, 0, IN, 0, total); /* :137-146 */
    HcommGfxSlice sl[HCOMM_GFX_MAX_RANKS], sub[HCOMM_GFX_MAX_RANKS];
    CHK(HcommGfxCalcSlices(count, unit, n, sl)); /* PrepareSlice :69-102 = the 128-byte-aligned table */
    uint32_t step = 0;
    for (uint32_t r = 0; r < n; ++r) CHK(push(l, step, COPY, r, SCR, 0, r, IN, 0, total)); /* :188-193 */
    ++step;
    for (uint32_t round = 1; round < n; ++round, ++step)
        for (uint32_t r = 0; r < n; ++r) {
            CHK(HcommGfxCalcSlices(sl[r].size / unit, unit, n - 1, sub)); /* :108-113 */
            for (uint32_t q = 0; q + 1 < n; ++q) {
                const uint32_t hop = (q + round - 1) % (n - 1) + 1; /* 1 .. n-1, starting at q+1 */
                const uint64_t off = sl[r].offset + sub[q].offset;
                CHK(push(l, step, REDUCE, r, SCR, off, (r + hop) % n, SCR, off, sub[q].size));
            }
        }
    for (uint32_t r = 0; r < n; ++r) CHK(push(l, step, COPY, r, OUT, sl[r].offset, r, SCR, sl[r].offset, sl[r].size));
    ++step;
    for (uint32_t k = 1; k < n; ++k, ++step)
        for (uint32_t r = 0; r < n; ++r) {
            const uint32_t p = modn((int64_t)r - k, n);
            CHK(push(l, step, COPY, r, OUT, sl[p].offset, p, SCR, sl[p].offset, sl[p].size));
        }
    return HCCL_SUCCESS;
}

/* AllReduceLocalReduce, temp_all_reduce/all_reduce_local_reduce.cc.  Stated per destination rank d: its window
 * of n-1 slots starts at slot 0 (slot 1 for the last rank), slot w of the window is filled by rank d - k where
 * k is the round that maps to w (:225-229), the neighbour d + 1 reduces straight onto d's own copy (:230-247),
 * the slots are folded towards the slot at d's natural offset (:301-364), and everybody fetches that slot
 * (:417-424). */
/* The block of slots RunLocalReduce halves: 2^floor(log2(n - 1)) of the n - 1 slots (all_reduce_local_reduce.cc:304-305). */
static uint32_t local_reduce_block(uint32_t n)
{
    uint32_t p = 1;
    while (2u * p <= n - 1u) p *= 2u;
    return p;
}

/* Where rank d's folded slice ends up, as a slot index inside d's window: the block starts at slot 0 for the ranks
 * below the block size and n - block - 1 slots further up for the others (:330), and the halving rounds walk towards
 * position min(d, or d - block + 1, block - 1) of the block (:328-329, :333-362). */
static uint32_t local_reduce_result_slot(uint32_t n, uint32_t d)
{
    const uint32_t p = local_reduce_block(n);
    if (d < p) return d;
    const uint32_t target = d - p + 1u < p - 1u ? d - p + 1u : p - 1u;
    return n - p - 1u + target;
}

/* The gather fetches rank d's slice from slot d of d's window, the last rank's from its slot n - 2 (:419-423; the
 * last rank's window starts one slot up, :102-110).  That is where the folds leave it when n is a power of two, and
 * when n is 3; for every other rank count some rank's result sits in another slot and the gather would fetch a partial
 * sum, so those counts are refused (tests/test_local_reduce_any_n.py replays the reference's statements for them). */
int hg_local_reduce_lands(uint32_t n)
{
    for (uint32_t d = 0; d < n; ++d)
        if (local_reduce_result_slot(n, d) != (d == n - 1u ? n - 2u : d)) return 0;
    return 1;
}

static int sched_allreduce_local_reduce(HgOpList* l, uint32_t n, uint64_t count, uint32_t unit)
{
    const uint64_t total = count * unit;
    if (n == 1) return push(l, 0, COPY, 0, OUT, 0, 0, IN, 0, total); /* :154-163 */
    if (!hg_local_reduce_lands(n)) return HCCL_E_PARA;
    HcommGfxSlice sl[HCOMM_GFX_MAX_RANKS];
    uint64_t per;
    local_reduce_slices(total, n, unit, sl, &per);
    const uint32_t half_n = local_reduce_block(n); /* slots in the block that is halved */
    uint32_t step = 0;
    for (uint32_t d = 0; d < n; ++d) CHK(push(l, step, COPY, d, SCR, sl[d].offset, d, IN, sl[d].offset, sl[d].size));
    ++step;
    for (uint32_t k = 1; k < n; ++k, ++step)
        for (uint32_t d = 0; d < n; ++d) {
            const uint64_t base = (d == n - 1) ? per : 0;
            const uint32_t sender = modn((int64_t)d - k, n);
            if (k == n - 1) {
                const uint32_t own = (d == n - 1) ? d - 1 : d;
                CHK(push(l, step, REDUCE, d, SCR, base + (uint64_t)own * per, sender, IN, sl[d].offset, sl[d].size));
            } else {
                uint32_t w = (d + k) % (n - 1);
                if (d == n - 1) w = (w + n - 2) % (n - 1);
                CHK(push(l, step, COPY, d, SCR, base + (uint64_t)w * per, sender, IN, sl[d].offset, sl[d].size));
            }
        }
    /* fold the n-1 slots: first the n - 1 - block slots beyond the block onto (or from) the first ones (:311-327) ... */
    for (uint32_t d = 0; d < n; ++d) {
        const uint64_t base = (d == n - 1) ? per : 0;
        for (uint32_t i = 0; i + half_n + 1 < n; ++i) {
            const uint64_t lo = base + (uint64_t)i * per, hi = base + (uint64_t)(half_n + i) * per;
            if (d < half_n) CHK(push(l, step, REDUCE, d, SCR, lo, d, SCR, hi, sl[d].size));
            else CHK(push(l, step, REDUCE, d, SCR, hi, d, SCR, lo, sl[d].size));
        }
    }
    ++step;
    /* ... then halve the block of half_n slots towards the slot that holds d's natural offset */
    uint32_t levels = 0;
    while ((1u << (levels + 1)) <= half_n) ++levels;
    for (uint32_t q = 0; q < levels; ++q, ++step)
        for (uint32_t d = 0; d < n; ++d) {
            const uint64_t base = (d == n - 1) ? per : 0;
            uint32_t target = (d < half_n) ? d : ((d - half_n + 1 < half_n - 1) ? d - half_n + 1 : half_n - 1);
            uint32_t first = (d < half_n) ? 0 : n - half_n - 1;
            for (uint32_t z = 0; z < q; ++z) { /* replay the earlier rounds' choice of half */
                const uint32_t h = half_n >> (z + 1);
                if (target >= h) {
                    first += h;
                    target -= h;
                }
            }
            const uint32_t h = half_n >> (q + 1);
            for (uint32_t i = 0; i < h; ++i) {
                const uint64_t lo = base + (uint64_t)(first + i) * per, hi = base + (uint64_t)(first + h + i) * per;
                if (target < h) CHK(push(l, step, REDUCE, d, SCR, lo, d, SCR, hi, sl[d].size));
                else CHK(push(l, step, REDUCE, d, SCR, hi, d, SCR, lo, sl[d].size));
            }
        }
    /* gather: own slice from the own window, every other slice from its owner's window (:405-424) */
    for (uint32_t d = 0; d < n; ++d) CHK(push(l, step, COPY, d, OUT, sl[d].offset, d, SCR, sl[d].offset, sl[d].size));
    ++step;
    for (uint32_t k = 1; k < n; ++k, ++step)
        for (uint32_t d = 0; d < n; ++d) {
            const uint32_t p = modn((int64_t)d - k, n);
            CHK(push(l, step, COPY, d, OUT, sl[p].offset, p, SCR, (uint64_t)p * sl[0].size, sl[p].size));
        }
    return HCCL_SUCCESS;
}

/* The AICPU deterministic reduce-scatter (aicpu_kfc/algorithm/aicpu_reduce_scatter.cc:64-118, one pass of its loop):
 * all N x N slot writes at once (task_orchestrator.cc:80-95, :370-386: rank s's slice d into slot s of rank d's
 * window), then SelfLocalReduce (:719-755) in every window - the N - P slots beyond the largest power of two P onto
 * the first ones as one reduce, log2 P rounds that fold the upper half of what is left onto the lower half, one
 * contiguous reduce each - and window[0, count) to the output (:203-218). */
static int sched_rs_window_halving(HgOpList* l, uint32_t n, uint64_t count, uint64_t stride, uint32_t unit)
{
    const uint64_t cur = count * unit;
    if (n == 1) return push(l, 0, COPY, 0, OUT, 0, 0, IN, 0, cur); /* slot 0 is the result: copied straight through */
    uint32_t step = 0;
    for (uint32_t d = 0; d < n; ++d)
        for (uint32_t s = 0; s < n; ++s) CHK(push(l, step, COPY, d, SCR, (uint64_t)s * cur, s, IN, stride * d * unit, cur));
    ++step;
    uint32_t p = 1;
    while (2u * p <= n) p *= 2u;
    if (p < n) {
        for (uint32_t d = 0; d < n; ++d) CHK(push(l, step, REDUCE, d, SCR, 0, d, SCR, (uint64_t)p * cur, (uint64_t)(n - p) * cur));
    }
    ++step;
    for (uint32_t h = p / 2; h >= 1; h /= 2, ++step)
        for (uint32_t d = 0; d < n; ++d) CHK(push(l, step, REDUCE, d, SCR, 0, d, SCR, (uint64_t)h * cur, (uint64_t)h * cur));
    for (uint32_t d = 0; d < n; ++d) CHK(push(l, step, COPY, d, OUT, 0, d, SCR, 0, cur));
    return HCCL_SUCCESS;
}

/* ---- NHR (nonuniform hierarchical ring) and NB (nonuniform Bruck): ceil(log2 N) steps for any N ------------- */

static uint32_t ceil_log2(uint32_t n) /* nonuniform_hierarchical_ring_base.cc:139-147, nonuniform_bruck_base.cc:19-25 */
{
    uint32_t s = 0;
    while ((1u << s) < n) ++s;
    return s;
}

/* Slice order of the NHR tree (nonuniform_hierarchical_ring_base.cc:20-91, temp_reduce_scatter/
 * reduce_scatter_nhr.cc:97-162), stated recursively: a block of logical slices is split into its even and odd
 * positions, evens first; both halves are split again one level down while a rank still exchanges more than
 * one slice at that level and the block length was even.  dst receives the block in tree order. */
static void nhr_tree_order(uint32_t* dst, const uint32_t* src, uint32_t m, uint32_t n, uint32_t level)
{
    if (((n - 1 + (1u << level)) >> (level + 1)) <= 1) {
        memcpy(dst, src, m * sizeof(uint32_t));
        return;
    }
    uint32_t ev[HCOMM_GFX_MAX_RANKS], od[HCOMM_GFX_MAX_RANKS];
    const uint32_t ne = (m + 1) / 2, no = m / 2;
    for (uint32_t i = 0; i < m; ++i) {
        if (i & 1) od[i / 2] = src[i]; else ev[i / 2] = src[i];
    }
    if (m & 1) {
        memcpy(dst, ev, ne * sizeof(uint32_t));
        memcpy(dst + ne, od, no * sizeof(uint32_t));
        return;
    }
    nhr_tree_order(dst, ev, ne, n, level + 1);
    nhr_tree_order(dst + ne, od, no, n, level + 1);
}

/* map[logical slice] = position in the buffer; the identity when the order must be kept (stand-alone
 * reduce-scatter: reduce_scatter_nhr.cc:86-88) */
static void nhr_slice_map(uint32_t n, int keep_order, uint32_t* map)
{
    uint32_t ident[HCOMM_GFX_MAX_RANKS], tree[HCOMM_GFX_MAX_RANKS];
    for (uint32_t i = 0; i < n; ++i) ident[i] = i;
    if (keep_order) {
        memcpy(map, ident, n * sizeof(uint32_t));
        return;
    }
    nhr_tree_order(tree, ident, n, n, 0);
    for (uint32_t i = 0; i < n; ++i) map[tree[i]] = i;
}

/* Ascending by offset, neighbours that touch become one slice (NHRBase::MergeSlices,
 * nonuniform_hierarchical_ring_base.cc:94-136).  Returns the new number of slices. */
static uint32_t merge_touching(HcommGfxSlice* v, uint32_t m)
{
    if (m <= 1) return m;
    for (uint32_t i = 1; i < m; ++i) { /* insertion sort by (offset, size) */
        HcommGfxSlice x = v[i];
        uint32_t j = i;
        while (j > 0 && (v[j - 1].offset > x.offset || (v[j - 1].offset == x.offset && v[j - 1].size > x.size))) {
            v[j] = v[j - 1];
            --j;
        }
        v[j] = x;
    }
    uint32_t w = 0;
    for (uint32_t i = 1; i < m; ++i) {
        if (v[w].offset + v[w].size == v[i].offset) v[w].size += v[i].size;
        else v[++w] = v[i];
    }
    return w + 1;
}

/* NHR reduce-scatter over `sl` in the input buffers (reduce_scatter_nhr.cc:408-488 with the step table of
 * :552-593 and the inline-reduce receive of :197-259): step s, rank r reads rank r + 2^s and folds the logical
 * slices r, r - 2^(s+1), r - 2*2^(s+1), ... ((N-1+2^s) >> (s+1) of them) into its own copies. */
static int nhr_rs(HgOpList* l, uint32_t n, const HcommGfxSlice* sl, const uint32_t* map, int merge)
{
    const uint32_t steps = ceil_log2(n);
    for (uint32_t s = 0; s < steps; ++s) {
        const uint32_t cnt = (n - 1 + (1u << s)) >> (s + 1);
        for (uint32_t r = 0; r < n; ++r) {
            HcommGfxSlice v[HCOMM_GFX_MAX_RANKS];
            for (uint32_t i = 0; i < cnt; ++i) v[i] = sl[map[modn((int64_t)r - ((int64_t)i << (s + 1)), n)]];
            /* the last step handles its single slice unmerged (:239-259) */
            const uint32_t m = (merge && s + 1 < steps) ? merge_touching(v, cnt) : cnt;
            for (uint32_t i = 0; i < m; ++i)
                CHK(push(l, s, REDUCE, r, IN, v[i].offset, (r + (1u << s)) % n, IN, v[i].offset, v[i].size));
        }
    }
    return HCCL_SUCCESS;
}

/* AllReduceNHR (temp_all_reduce/all_reduce_nhr.cc:25-77,133-173): tree-ordered NHR reduce-scatter in place on
 * the inputs, own slice input -> output, NHR all-gather on the outputs (temp_all_gather/all_gather_nhr.cc:
 * 75-81,141-195, step table :228-268): step s (delta = 2^(S-1-s)), rank r reads rank r - delta and fetches the
 * logical slices r - delta, r - delta - 2 delta, ... */
static int sched_allreduce_nhr(HgOpList* l, uint32_t n, uint64_t count, uint32_t unit)
{
    const uint64_t total = count * unit;
    if (n == 1) return push(l, 0, COPY, 0, OUT, 0, 0, IN, 0, total); /* all_reduce_nhr.cc:35-44 */
    HcommGfxSlice sl[HCOMM_GFX_MAX_RANKS];
    uint32_t map[HCOMM_GFX_MAX_RANKS];
    memset(map, 0, sizeof(map));
    CHK(HcommGfxCalcSlices(count, unit, n, sl)); /* all_reduce_nhr.cc:104-121: the ring's slice table */
    nhr_slice_map(n, 0, map);
    CHK(nhr_rs(l, n, sl, map, 1));
    const uint32_t steps = ceil_log2(n);
    for (uint32_t r = 0; r < n; ++r)
        CHK(push(l, steps, COPY, r, OUT, sl[map[r]].offset, r, IN, sl[map[r]].offset, sl[map[r]].size));
    for (uint32_t s = 0; s < steps; ++s) {
        const uint32_t delta = 1u << (steps - 1 - s);
        const uint32_t cnt = (n - 1 + delta) / (2 * delta);
        for (uint32_t r = 0; r < n; ++r) {
            HcommGfxSlice v[HCOMM_GFX_MAX_RANKS];
            for (uint32_t i = 0; i < cnt; ++i)
                v[i] = sl[map[modn((int64_t)r - delta - (int64_t)i * 2 * delta, n)]];
            const uint32_t m = merge_touching(v, cnt);
            for (uint32_t i = 0; i < m; ++i)
                CHK(push(l, steps + 1 + s, COPY, r, OUT, v[i].offset, modn((int64_t)r - delta, n), OUT, v[i].offset, v[i].size));
        }
    }
    return HCCL_SUCCESS;
}

/* Stand-alone ReduceScatterNHR (reduce_scatter_nhr.cc:27-95): slice i of the input at i * stride elements, slice
 * order kept, nothing merged; the last step reduces into the input slice and copies it to the output, which
 * holds one slice (:57-75, :239-259, :208-217). */
static int sched_rs_nhr(HgOpList* l, uint32_t n, uint64_t count, uint64_t stride, uint32_t unit)
{
    const uint64_t sz = count * unit;
    if (n == 1) return push(l, 0, COPY, 0, OUT, 0, 0, IN, 0, sz); /* :41-46 */
    HcommGfxSlice sl[HCOMM_GFX_MAX_RANKS];
    uint32_t map[HCOMM_GFX_MAX_RANKS];
    memset(sl, 0, sizeof(sl));
    for (uint32_t i = 0; i < n; ++i) {
        sl[i].offset = (uint64_t)i * stride * unit;
        sl[i].size = sz;
    }
    nhr_slice_map(n, 1, map);
    CHK(nhr_rs(l, n, sl, map, 0));
    for (uint32_t r = 0; r < n; ++r) CHK(push(l, ceil_log2(n), COPY, r, OUT, 0, r, IN, sl[r].offset, sz));
    return HCCL_SUCCESS;
}

/* NB reduce-scatter over `sl` in the input buffers (temp_reduce_scatter/reduce_scatter_nb.cc:119-230,260-311):
 * step s, rank r reads rank r - 2^s and folds slices r, r + 2^(s+1), r + 2*2^(s+1), ... into its own copies. */
static int nb_rs(HgOpList* l, uint32_t n, const HcommGfxSlice* sl)
{
    const uint32_t steps = ceil_log2(n);
    for (uint32_t s = 0; s < steps; ++s) {
        const uint32_t cnt = (n - 1 + (1u << s)) >> (s + 1);
        for (uint32_t r = 0; r < n; ++r)
            for (uint32_t i = 0; i < cnt; ++i) {
                const uint32_t c = (uint32_t)((r + ((uint64_t)i << (s + 1))) % n);
                CHK(push(l, s, REDUCE, r, IN, sl[c].offset, modn((int64_t)r - (1 << s), n), IN, sl[c].offset, sl[c].size));
            }
    }
    return HCCL_SUCCESS;
}

/* AllReduceNB (temp_all_reduce/all_reduce_nb.cc:26-61,139-150,162-201): slices of ceil(total/N) rounded up to
 * 128 bytes when larger than 128 KiB, else rounded up to 128 KiB (:203-219: small messages are not cut); NB
 * reduce-scatter in place; own slice input -> output; NB all-gather on the outputs (temp_all_gather/
 * all_gather_nb.cc:88-92,101-188): step s, rank r reads rank r - 2^s and fetches slices r - 2^s - i,
 * i < 2^s (the last step only the N - 2^s that are still missing). */
static int sched_allreduce_nb(HgOpList* l, uint32_t n, uint64_t count, uint32_t unit)
{
    const uint64_t total = count * unit;
    if (n == 1) return push(l, 0, COPY, 0, OUT, 0, 0, IN, 0, total); /* all_reduce_nb.cc:130-137 */
    HcommGfxSlice sl[HCOMM_GFX_MAX_RANKS];
    const uint64_t small = 128u * 1024u; /* NB_ALLREDUCE_SMALL_SIZE, nonuniform_bruck_base_pub.h:19 */
    const uint64_t raw = (total + n - 1) / n;
    const uint64_t gran = raw > small ? HG_SLICE_ALIGN : small;
    const uint64_t per = raw == 0 ? gran : (raw + gran - 1) / gran * gran;
    uint64_t residue = total;
    memset(sl, 0, sizeof(sl));
    for (uint32_t i = 0; i < n; ++i) {
        sl[i].size = residue > per ? per : residue;
        sl[i].offset = total - residue;
        residue -= sl[i].size;
    }
    CHK(nb_rs(l, n, sl));
    const uint32_t steps = ceil_log2(n);
    for (uint32_t r = 0; r < n; ++r) CHK(push(l, steps, COPY, r, OUT, sl[r].offset, r, IN, sl[r].offset, sl[r].size));
    for (uint32_t s = 0; s < steps; ++s) {
        const uint32_t cnt = (s + 1 == steps && n != (1u << steps)) ? n - (1u << s) : (1u << s);
        for (uint32_t r = 0; r < n; ++r)
            for (uint32_t i = 0; i < cnt; ++i) {
                const uint32_t c = modn((int64_t)r - (1 << s) - i, n);
                CHK(push(l, steps + 1 + s, COPY, r, OUT, sl[c].offset, modn((int64_t)r - (1 << s), n), OUT, sl[c].offset, sl[c].size));
            }
    }
    return HCCL_SUCCESS;
}

/* Stand-alone ReduceScatterNB (reduce_scatter_nb.cc:27-86): as the stand-alone NHR variant, other direction. */
static int sched_rs_nb(HgOpList* l, uint32_t n, uint64_t count, uint64_t stride, uint32_t unit)
{
    const uint64_t sz = count * unit;
    if (n == 1) return push(l, 0, COPY, 0, OUT, 0, 0, IN, 0, sz); /* :35-40 */
    HcommGfxSlice sl[HCOMM_GFX_MAX_RANKS];
    memset(sl, 0, sizeof(sl));
    for (uint32_t i = 0; i < n; ++i) {
        sl[i].offset = (uint64_t)i * stride * unit;
        sl[i].size = sz;
    }
    CHK(nb_rs(l, n, sl));
    /* last step: reduce into the input slice, then input slice -> output (:267-289, component/reducer.cc:209-218) */
    for (uint32_t r = 0; r < n; ++r) CHK(push(l, ceil_log2(n), COPY, r, OUT, 0, r, IN, sl[r].offset, sz));
    return HCCL_SUCCESS;
}

/* ReduceScatterLocalReduce, the deterministic mesh reduce-scatter (temp_reduce_scatter/
 * reduce_scatter_local_reduce.cc:125-160).  Stated per destination d: think of the row V[0] = d's user output,
 * V[j] = slot j-1 of d's receive window.  Rank d-j writes its copy of slice d into V[j] and d copies its own into
 * V[0], all at once (:218-243); then the tail beyond the largest power of two P <= N is folded onto the front,
 * V[a] (op)= V[a+P] (:266-283), and the front is halved, V[a] (op)= V[a+h] for h = P/2, P/4, ..., 1 (:286-301). */
static int sched_rs_local_reduce(HgOpList* l, uint32_t n, uint64_t count, uint32_t unit)
{
    const uint64_t sz = count * unit;
    const uint64_t slot = rs_local_reduce_slot(sz);
    for (uint32_t d = 0; d < n; ++d)
        for (uint32_t r = 0; r < n; ++r) {
            if (r == d) CHK(push(l, 0, COPY, d, OUT, 0, d, IN, (uint64_t)d * sz, sz));
            else CHK(push(l, 0, COPY, d, SCR, rs_local_reduce_window(sz, d) + slot * (modn((int64_t)d - r, n) - 1), r, IN, (uint64_t)d * sz, sz));
        }
#define V_BUF(j) ((j) == 0 ? OUT : SCR)
#define V_OFF(d, j) ((j) == 0 ? 0 : rs_local_reduce_window(sz, d) + slot * ((j) - 1))
    const uint32_t p2 = floor_pow2(n);
    uint32_t step = 1;
    if (p2 < n) {
        for (uint32_t d = 0; d < n; ++d)
            for (uint32_t a = 0; a < n - p2; ++a)
                CHK(push(l, step, REDUCE, d, V_BUF(a), V_OFF(d, a), d, SCR, V_OFF(d, a + p2), sz));
        ++step;
    }
    for (uint32_t h = p2 / 2; h >= 1; h /= 2, ++step)
        for (uint32_t d = 0; d < n; ++d)
            for (uint32_t a = 0; a < h; ++a)
                CHK(push(l, step, REDUCE, d, V_BUF(a), V_OFF(d, a), d, SCR, V_OFF(d, a + h), sz));
#undef V_BUF
#undef V_OFF
    return HCCL_SUCCESS;
}

/* AllReduceDoubling (temp_all_reduce/all_reduce_doubling.cc:91-128), power-of-two rank counts only (:81-88): the
 * whole message every step.  Step s: first every rank refreshes the buffer its partner will read - input -> output
 * at s = 0 (:105-106), output -> input afterwards (:107-108) - then folds the partner's input (rank XOR 2^s) into its
 * own output (:113-121).  The two halves of a step are separated by the ack exchange, hence two schedule steps. */
static int sched_allreduce_doubling(HgOpList* l, uint32_t n, uint64_t count, uint32_t unit)
{
    const uint64_t total = count * unit;
    if (n == 1) return push(l, 0, COPY, 0, OUT, 0, 0, IN, 0, total); /* :38-41 */
    if (n & (n - 1)) return HCCL_E_PARA;
    uint32_t step = 0;
    for (uint32_t bit = 1; bit < n; bit <<= 1) {
        for (uint32_t r = 0; r < n; ++r) {
            if (bit == 1) CHK(push(l, step, COPY, r, OUT, 0, r, IN, 0, total));
            else CHK(push(l, step, COPY, r, IN, 0, r, OUT, 0, total));
        }
        ++step;
        for (uint32_t r = 0; r < n; ++r) CHK(push(l, step, REDUCE, r, OUT, 0, r ^ bit, IN, 0, total));
        ++step;
    }
    return HCCL_SUCCESS;
}

/* AllReduceNHROneshot (temp_all_reduce/all_reduce_nhr_oneshot.cc:26-69): the whole message climbs a binomial tree
 * to rank 0 and comes back down it.  Up (temp_reduce/reduce_nhr_oneshot.cc:169-236): in round s every rank q that is
 * a multiple of 2^(s+1) and has a rank q + 2^s above it folds that rank's input into its own input.  Then rank 0
 * copies its input to its output (temp_broadcast/broadcast_nhr_oneshot.cc:40-46) and the rounds run backwards on the
 * outputs (:155-205): rank q + 2^s copies rank q's output. */
static int sched_allreduce_nhr_oneshot(HgOpList* l, uint32_t n, uint64_t count, uint32_t unit)
{
    const uint64_t total = count * unit;
    uint32_t step = 0;
    for (uint32_t d = 1; d < n; d <<= 1, ++step)
        for (uint32_t q = 0; q + d < n; q += 2 * d) CHK(push(l, step, REDUCE, q, IN, 0, q + d, IN, 0, total));
    CHK(push(l, step++, COPY, 0, OUT, 0, 0, IN, 0, total));
    uint32_t top = 1;
    while (top < n) top <<= 1;
    for (uint32_t d = top >> 1; d >= 1; d >>= 1, ++step)
        for (uint32_t q = 0; q + d < n; q += 2 * d) CHK(push(l, step, COPY, q + d, OUT, 0, q, OUT, 0, total));
    return HCCL_SUCCESS;
}

int hg_schedule(HgOpList* l, int alg, uint32_t n, uint64_t count, uint64_t stride, int dtype)
{
    memset(l, 0, sizeof(*l));
    return hg_schedule_into(l, alg, n, count, stride, dtype);
}

int hg_schedule_into(HgOpList* l, int alg, uint32_t n, uint64_t count, uint64_t stride, int dtype)
{
    if (n == 0 || n > HCOMM_GFX_MAX_RANKS) return HCCL_E_PARA;
    if (stride == 0) stride = count;
    if (stride < count || stride > HG_MAX_COUNT) return HCCL_E_PARA;
    if (stride != count && alg != HCOMM_GFX_ALG_REDUCE_SCATTER_MESH && alg != HCOMM_GFX_ALG_REDUCE_SCATTER_RING_STANDALONE &&
        alg != HCOMM_GFX_ALG_REDUCE_SCATTER_NHR && alg != HCOMM_GFX_ALG_REDUCE_SCATTER_NB &&
        alg != HCOMM_GFX_ALG_REDUCE_SCATTER_WINDOW_HALVING)
        return HCCL_E_PARA;
    const uint32_t unit = HcommGfxDataTypeSize((HcommDataType)dtype);
    if (unit == 0) return HCCL_E_PARA;
    int rc;
    switch (alg) {
        case HCOMM_GFX_ALG_ALLREDUCE_RING: rc = sched_allreduce_ring(l, n, count, unit, 1); break;
        case HCOMM_GFX_ALG_REDUCE_SCATTER_RING: rc = sched_allreduce_ring(l, n, count, unit, 0); break;
        case HCOMM_GFX_ALG_ALLREDUCE_RHD: rc = sched_allreduce_rhd(l, n, count, unit); break;
        case HCOMM_GFX_ALG_ALLREDUCE_MESH_ONESHOT: rc = sched_allreduce_mesh_oneshot(l, n, count, unit, 0); break;
        case HCOMM_GFX_ALG_ALLREDUCE_MESH_ONESHOT_ASCENDING: rc = sched_allreduce_mesh_oneshot(l, n, count, unit, 1); break;
        case HCOMM_GFX_ALG_REDUCE_SCATTER_MESH: rc = sched_rs_mesh(l, n, count, stride, unit); break;
        case HCOMM_GFX_ALG_REDUCE_SCATTER_RING_STANDALONE: rc = sched_rs_ring_standalone(l, n, count, stride, unit); break;
        case HCOMM_GFX_ALG_ALLREDUCE_LOCAL_REDUCE: rc = sched_allreduce_local_reduce(l, n, count, unit); break;
        case HCOMM_GFX_ALG_ALLREDUCE_CHUNK_MESH: rc = sched_allreduce_chunk_mesh(l, n, count, unit); break;
        case HCOMM_GFX_ALG_ALLREDUCE_NHR: rc = sched_allreduce_nhr(l, n, count, unit); break;
        case HCOMM_GFX_ALG_REDUCE_SCATTER_NHR: rc = sched_rs_nhr(l, n, count, stride, unit); break;
        case HCOMM_GFX_ALG_ALLREDUCE_NB: rc = sched_allreduce_nb(l, n, count, unit); break;
        case HCOMM_GFX_ALG_REDUCE_SCATTER_NB: rc = sched_rs_nb(l, n, count, stride, unit); break;
        case HCOMM_GFX_ALG_REDUCE_SCATTER_LOCAL_REDUCE: rc = sched_rs_local_reduce(l, n, count, unit); break;
        case HCOMM_GFX_ALG_ALLREDUCE_DOUBLING: rc = sched_allreduce_doubling(l, n, count, unit); break;
        case HCOMM_GFX_ALG_ALLREDUCE_NHR_ONESHOT: rc = sched_allreduce_nhr_oneshot(l, n, count, unit); break;
        case HCOMM_GFX_ALG_REDUCE_SCATTER_WINDOW_HALVING: rc = sched_rs_window_halving(l, n, count, stride, unit); break;
        default: rc = HCCL_E_PARA;
    }
    if (rc != HCCL_SUCCESS) hg_oplist_free(l);
    return rc;
}

int32_t HcommGfxScheduleEmit(
    HcommGfxAlgorithm alg, uint32_t nRanks, uint64_t count, HcommDataType dataType, HcommGfxSchedOp* ops,
    uint64_t cap, uint64_t* n)
{
    return HcommGfxScheduleEmitStrided(alg, nRanks, count, 0, dataType, ops, cap, n);
}

int32_t HcommGfxScheduleEmitStrided(
    HcommGfxAlgorithm alg, uint32_t nRanks, uint64_t count, uint64_t strideCount, HcommDataType dataType,
    HcommGfxSchedOp* ops, uint64_t cap, uint64_t* n)
{
    if (!n) return HCCL_E_PTR;
    HgOpList l;
    int rc = hg_schedule(&l, (int)alg, nRanks, count, strideCount, (int)dataType);
    if (rc != HCCL_SUCCESS) return rc;
    *n = l.n;
    if (ops) {
        const uint64_t m = l.n < cap ? l.n : cap;
        if (m) memcpy(ops, l.ops, m * sizeof(*ops));
    }
    hg_oplist_free(&l);
    return HCCL_SUCCESS;
}

/* ---- the op-base loop around a template (the templates' immediate caller) ------------------------------------ */

static int is_scatter_alg(int alg)
{
    return alg == HCOMM_GFX_ALG_REDUCE_SCATTER_MESH || alg == HCOMM_GFX_ALG_REDUCE_SCATTER_RING_STANDALONE ||
           alg == HCOMM_GFX_ALG_REDUCE_SCATTER_NHR || alg == HCOMM_GFX_ALG_REDUCE_SCATTER_NB ||
           alg == HCOMM_GFX_ALG_REDUCE_SCATTER_LOCAL_REDUCE;
}

uint64_t hg_opbase_max_count(int alg, uint32_t n, uint64_t ccl_bytes, uint32_t unit)
{
    if (unit == 0 || n == 0) return 0;
    /* allreduce: CCLBuffSize / unitSize (coll_all_reduce_executor.cc:129-138); reduce-scatter: the input buffer
     * holds N slices, each a multiple of 128 bytes (coll_reduce_scatter_executor.cc:124-134) */
    if (!is_scatter_alg(alg)) return ccl_bytes / unit;
    return ccl_bytes / n / HG_SLICE_ALIGN * HG_SLICE_ALIGN / unit;
}

/* One pass per chunk of at most maxCountPerLoop elements: user input -> CCL input, the template on the CCL
 * buffers, CCL output -> user output.  Paths relative to src/legacy/ascend910/algorithm/impl/coll_executor/:
 * allreduce coll_all_reduce/coll_all_reduce_executor.cc:199-262 (loop), :304-309 and :326-331 (copies);
 * reduce-scatter coll_reduce_scatter/coll_reduce_scatter_executor.cc:149-220 (loop), :257-275 (one copy per input
 * slice, or a single copy when one pass takes everything, :616-620), :292-297 (copy out). */
int hg_schedule_opbase(HgOpList* l, int alg, uint32_t n, uint64_t count, uint64_t ccl_bytes, int dtype)
{
    memset(l, 0, sizeof(*l));
    if (n == 0 || n > HCOMM_GFX_MAX_RANKS) return HCCL_E_PARA;
    const uint32_t unit = HcommGfxDataTypeSize((HcommDataType)dtype);
    if (unit == 0 || count > HG_MAX_COUNT || alg == HCOMM_GFX_ALG_REDUCE_SCATTER_RING) return HCCL_E_PARA;
    const int scatter = is_scatter_alg(alg);
    const uint64_t maxc = hg_opbase_max_count(alg, n, ccl_bytes, unit);
    if (maxc == 0) return scatter ? HCCL_E_INTERNAL : HCCL_E_PARA; /* :213-218 / :163-165 */
    uint32_t step = 0;
    int rc = HCCL_SUCCESS;
    for (uint64_t done = 0; done < count && rc == HCCL_SUCCESS;) {
        const uint64_t cur = count - done > maxc ? maxc : count - done;
        const uint64_t cur_bytes = cur * unit, off = done * unit;
        for (uint32_t r = 0; r < n && rc == HCCL_SUCCESS; ++r) {
            if (!scatter) {
                rc = push(l, step, COPY, r, IN, 0, r, HCOMM_GFX_BUF_USER_IN, off, cur_bytes);
            } else if (cur == count) {
                rc = push(l, step, COPY, r, IN, 0, r, HCOMM_GFX_BUF_USER_IN, 0, count * unit * n);
            } else {
                for (uint32_t i = 0; i < n && rc == HCCL_SUCCESS; ++i)
                    rc = push(l, step, COPY, r, IN, cur_bytes * i, r, HCOMM_GFX_BUF_USER_IN, count * unit * i + off, cur_bytes);
            }
        }
        ++step;
        HgOpList sub;
        if (rc == HCCL_SUCCESS) rc = hg_schedule(&sub, alg, n, cur, cur, dtype);
        if (rc != HCCL_SUCCESS) break;
        uint32_t used = 0; /* steps of the template that do anything */
        for (uint64_t i = 0; i < sub.n && rc == HCCL_SUCCESS; ++i) {
            const HcommGfxSchedOp* o = &sub.ops[i];
            if (o->step + 1 > used) used = o->step + 1;
            rc = push(l, step + o->step, o->kind, o->rank, o->dstBuf, o->dstOff, o->srcRank, o->srcBuf, o->srcOff, o->bytes);
        }
        hg_oplist_free(&sub);
        step += used;
        for (uint32_t r = 0; r < n && rc == HCCL_SUCCESS; ++r)
            rc = push(l, step, COPY, r, HCOMM_GFX_BUF_USER_OUT, off, r, OUT, 0, cur_bytes);
        ++step;
        done += cur;
    }
    if (rc != HCCL_SUCCESS) hg_oplist_free(l);
    return rc;
}

int32_t HcommGfxOpBaseEmit(
    HcommGfxAlgorithm alg, uint32_t nRanks, uint64_t count, uint64_t cclBytes, HcommDataType dataType,
    HcommGfxSchedOp* ops, uint64_t cap, uint64_t* n)
{
    if (!n) return HCCL_E_PTR;
    HgOpList l;
    int rc = hg_schedule_opbase(&l, (int)alg, nRanks, count, cclBytes, (int)dataType);
    if (rc != HCCL_SUCCESS) return rc;
    *n = l.n;
    if (ops) {
        const uint64_t m = l.n < cap ? l.n : cap;
        if (m) memcpy(ops, l.ops, m * sizeof(*ops));
    }
    hg_oplist_free(&l);
    return HCCL_SUCCESS;
}

int32_t HcommGfxOpBaseMaxCount(HcommGfxAlgorithm alg, uint32_t nRanks, uint64_t cclBytes, HcommDataType dataType,
                               uint64_t* maxCountPerLoop)
{
    if (!maxCountPerLoop) return HCCL_E_PTR;
    const uint32_t unit = HcommGfxDataTypeSize(dataType);
    if (unit == 0 || nRanks == 0 || nRanks > HCOMM_GFX_MAX_RANKS) return HCCL_E_PARA;
    *maxCountPerLoop = hg_opbase_max_count((int)alg, nRanks, cclBytes, unit);
    return HCCL_SUCCESS;
}

/* ---- the three-step allreduce of the ring executor (two communicator levels) ------------------------------- */

/* Append `sub` to `l`: ranks through `map`, steps shifted by step0, offsets in the input / output buffers shifted by
 * base (the templates add baseOffset_ to every slice they address, alg_template_base.cc:53-54).  Only the ops for
 * which keep() holds. */
static int append_mapped(HgOpList* l, const HgOpList* sub, const uint32_t* map, uint32_t step0, uint64_t base,
                         int only_out_to_out, uint32_t* used)
{
    for (uint64_t i = 0; i < sub->n; ++i) {
        const HcommGfxSchedOp* o = &sub->ops[i];
        if (only_out_to_out && !(o->dstBuf == OUT && o->srcBuf == OUT)) continue;
        if (o->step + 1 > *used) *used = o->step + 1;
        CHK(push(l, step0 + o->step, o->kind, map[o->rank], o->dstBuf, o->dstOff + base, map[o->srcRank], o->srcBuf,
                 o->srcOff + base, o->bytes));
    }
    return HCCL_SUCCESS;
}

/* Lists built level by level and, inside a level, group by group: order them by step, then by rank, keeping the
 * order of a rank's operations inside a step (bottom-up merge sort, stable). */
static int op_before(const HcommGfxSchedOp* a, const HcommGfxSchedOp* b)
{
    return a->step < b->step || (a->step == b->step && a->rank <= b->rank);
}

static int order_by_step_rank(HgOpList* l)
{
    if (l->n < 2) return HCCL_SUCCESS;
    HcommGfxSchedOp* tmp = (HcommGfxSchedOp*)malloc(l->n * sizeof(*tmp));
    if (!tmp) return HCCL_E_MEMORY;
    HcommGfxSchedOp *src = l->ops, *dst = tmp;
    for (uint64_t w = 1; w < l->n; w *= 2) {
        for (uint64_t lo = 0; lo < l->n; lo += 2 * w) {
            const uint64_t mid = lo + w < l->n ? lo + w : l->n, hi = lo + 2 * w < l->n ? lo + 2 * w : l->n;
            uint64_t a = lo, b = mid, k = lo;
            while (a < mid && b < hi) dst[k++] = op_before(&src[a], &src[b]) ? src[a++] : src[b++];
            while (a < mid) dst[k++] = src[a++];
            while (b < hi) dst[k++] = src[b++];
        }
        HcommGfxSchedOp* t = src;
        src = dst;
        dst = t;
    }
    if (src != l->ops) memcpy(l->ops, src, l->n * sizeof(*tmp));
    free(tmp);
    return HCCL_SUCCESS;
}

/* CollAllReduceRingExecutor::KernelRun (src/legacy/ascend910/algorithm/impl/coll_executor/coll_all_reduce/
 * coll_all_reduce_ring_executor.cc:94-231) for nServers x nLocal ranks, rank = server * nLocal + local index, one
 * ring per server:
 *   1. inside every server, ring reduce-scatter in place on the inputs over the slices of PrepareSliceData
 *      (:109, alg_template_base.cc:787-820 - the 128-byte-aligned table), MultiRingReduceScatter :134-136;
 *   2. between the servers, for every local index i, the level-1 allreduce template over segment i of the ranks
 *      {i, nLocal + i, ...}: input and output ranges of the rank buffers, baseOffset = the segment's offset
 *      (:156-158, :209-211; segment = local rank, coll_comm_executor.cc:2565-2575);
 *   3. inside every server, ring all-gather on the outputs (MultiRingAllGather :228-230; input == output there,
 *      coll_comm_executor.cc:377-379, so the template's own-slice copy does not happen, all_gather_ring.cc:117). */
/* Level 0 of CollAllReduceMeshExecutor::KernelRun (coll_executor/coll_all_reduce/coll_all_reduce_mesh_executor.cc:
 * 116-119, 204-228) for one server whose ranks are g0 .. g0 + n - 1:
 *   reduce-scatter (MultiStreamReduceScatterMesh, coll_comm_executor.cc:1754-1860): segment r is cut into n - 1 pieces
 *   of ceil(size / (n - 1)) bytes rounded up to 128 (PrepareSliceMeshStreams, alg_template_base.cc:823-865), one per
 *   stream; in round k = 1 .. n - 1 stream s folds its piece of rank r - 1 - ((k + s - 1) mod (n - 1))'s input into
 *   rank r's (reduce_scatter_mesh.cc:56-68): every stream meets the peers in the same cyclic order, each starting at
 *   its own place, so that in every round the n - 1 streams read n - 1 different peers;
 *   all-gather (AllGatherMesh, all_gather_mesh.cc:66-131, on the outputs): every rank fetches every other rank's
 *   segment, all at once. */
static int mesh_level0_rs(HgOpList* l, uint32_t g0, uint32_t n, const HcommGfxSlice* seg, uint32_t step)
{
    for (uint32_t k = 1; k < n; ++k)
        for (uint32_t r = 0; r < n; ++r) {
            const uint64_t per = ((seg[r].size + (n - 2)) / (n - 1) + 127u) / 128u * 128u;
            for (uint32_t s = 0; s + 1 < n; ++s) {
                const uint64_t lo = (uint64_t)s * per < seg[r].size ? (uint64_t)s * per : seg[r].size;
                const uint64_t len = seg[r].size - lo < per ? seg[r].size - lo : per;
                const uint32_t src = (r + 2u * n - 1u - ((k + s - 1u) % (n - 1u))) % n;
                CHK(push(l, step + k - 1, REDUCE, g0 + r, IN, seg[r].offset + lo, g0 + src, IN, seg[r].offset + lo, len));
            }
        }
    return HCCL_SUCCESS;
}

static int mesh_level0_ag(HgOpList* l, uint32_t g0, uint32_t n, const HcommGfxSlice* seg, uint32_t step)
{
    for (uint32_t r = 0; r < n; ++r)
        for (uint32_t k = 1; k < n; ++k) {
            const uint32_t peer = (r + n - k) % n;
            CHK(push(l, step, COPY, g0 + r, OUT, seg[peer].offset, g0 + peer, OUT, seg[peer].offset, seg[peer].size));
        }
    return HCCL_SUCCESS;
}

int hg_schedule_hier(HgOpList* l, int level0_mesh, int alg1, uint32_t n_servers, uint32_t n_local, uint64_t count, int dtype)
{
    memset(l, 0, sizeof(*l));
    const uint32_t unit = HcommGfxDataTypeSize((HcommDataType)dtype);
    if (unit == 0 || count > HG_MAX_COUNT || n_servers == 0 || n_local == 0 || (uint64_t)n_servers * n_local > HCOMM_GFX_MAX_RANKS) return HCCL_E_PARA;
    if (alg1 != HCOMM_GFX_ALG_ALLREDUCE_RING && alg1 != HCOMM_GFX_ALG_ALLREDUCE_RHD && alg1 != HCOMM_GFX_ALG_ALLREDUCE_NHR &&
        alg1 != HCOMM_GFX_ALG_ALLREDUCE_NB)
        return HCCL_E_PARA; /* the level-1 choices of :164-204 that are built here */
    if (level0_mesh && n_local < 2) return HCCL_E_PARA; /* PrepareSliceMeshStreams refuses zero streams (alg_template_base.cc:832-835) */
    HcommGfxSlice seg[HCOMM_GFX_MAX_RANKS];
    CHK(HcommGfxCalcSlices(count, unit, n_local, seg));
    uint32_t map[HCOMM_GFX_MAX_RANKS];
    HgOpList sub;
    int rc = HCCL_SUCCESS;
    uint32_t step = 0, used = 0;
    /* 1 */
    if (level0_mesh) {
        for (uint32_t s = 0; s < n_servers && rc == HCCL_SUCCESS; ++s) rc = mesh_level0_rs(l, s * n_local, n_local, seg, step);
        used = n_local - 1;
    } else if ((rc = hg_schedule(&sub, HCOMM_GFX_ALG_REDUCE_SCATTER_RING, n_local, count, count, dtype)) == HCCL_SUCCESS) {
        for (uint32_t s = 0; s < n_servers && rc == HCCL_SUCCESS; ++s) {
            for (uint32_t j = 0; j < n_local; ++j) map[j] = s * n_local + j;
            rc = append_mapped(l, &sub, map, step, 0, 0, &used);
        }
        hg_oplist_free(&sub);
    }
    step += used;
    /* 2 */
    used = 0;
    /* :171-181: NHR between the servers does not slice messages of up to 256 KiB per device of a server
     * (NHR_ALLREDUCE_SMALL_SIZE, pub_inc/op_context.h:18) */
    if (alg1 == HCOMM_GFX_ALG_ALLREDUCE_NHR && count * unit / n_local <= 256u * 1024u) alg1 = HCOMM_GFX_ALG_ALLREDUCE_NHR_ONESHOT;
    for (uint32_t i = 0; i < n_local && rc == HCCL_SUCCESS; ++i) {
        for (uint32_t s = 0; s < n_servers; ++s) map[s] = s * n_local + i;
        rc = hg_schedule(&sub, alg1, n_servers, seg[i].size / unit, seg[i].size / unit, dtype);
        if (rc != HCCL_SUCCESS) break;
        rc = append_mapped(l, &sub, map, step, seg[i].offset, 0, &used);
        hg_oplist_free(&sub);
    }
    step += used;
    /* 3 */
    used = 0;
    if (level0_mesh) {
        for (uint32_t s = 0; s < n_servers && rc == HCCL_SUCCESS; ++s) rc = mesh_level0_ag(l, s * n_local, n_local, seg, step);
    } else if (rc == HCCL_SUCCESS && (rc = hg_schedule(&sub, HCOMM_GFX_ALG_ALLREDUCE_RING, n_local, count, count, dtype)) == HCCL_SUCCESS) {
        /* the gather rounds of the ring allreduce are the ops that move output to output; renumber them from 0 */
        uint32_t first = UINT32_MAX;
        for (uint64_t i = 0; i < sub.n; ++i)
            if (sub.ops[i].dstBuf == OUT && sub.ops[i].srcBuf == OUT && sub.ops[i].step < first) first = sub.ops[i].step;
        for (uint64_t i = 0; i < sub.n; ++i)
            if (sub.ops[i].dstBuf == OUT && sub.ops[i].srcBuf == OUT) sub.ops[i].step -= first;
        for (uint32_t s = 0; s < n_servers && rc == HCCL_SUCCESS; ++s) {
            for (uint32_t j = 0; j < n_local; ++j) map[j] = s * n_local + j;
            rc = append_mapped(l, &sub, map, step, 0, 1, &used);
        }
        hg_oplist_free(&sub);
    }
    if (rc == HCCL_SUCCESS) rc = order_by_step_rank(l);
    if (rc != HCCL_SUCCESS) hg_oplist_free(l);
    return rc;
}

/* ---- the double-ring allreduce executor in op-base mode --------------------------------------------------------- */

#define UIN HCOMM_GFX_BUF_USER_IN
#define UOUT HCOMM_GFX_BUF_USER_OUT

/* CollAlignedAllReduceDoubleRingFor91093Executor (coll_executor/coll_all_reduce/
 * coll_aligned_all_reduce_double_ring_for_910_93_executor.cc; KernelRun of its base,
 * coll_all_reduce_ring_for_910_93_executor.cc:218-524) with DMA reduce, chunked by the op-base loop
 * (coll_all_reduce_executor.cc:234-262, no staging copies :305-311, :326-331).
 *
 * Every segment of PrepareSliceData is cut in two 128-byte-aligned shares (MutliSegSlicePrepare,
 * coll_comm_executor.cc:2011-2052); share 0 travels the ring 0 -> 1 -> ... and share 1 the mirrored ring
 * 0 -> N-1 -> ... (GetRingsOrderByTopoType, :1939-1949).  Written in rank space, with dir = -1 for ring 0 and +1 for
 * ring 1, every rank r
 *   reduce-scatter (alg_template/temp_reduce_scatter/aligned_reduce_scatter_double_ring.cc:379-412, 640-685):
 *     first copies the shares of segments r + dir and r + 2 dir from the user input to the CCL input; in step s folds
 *     the share of segment r + (2 + s) dir of rank r + dir's CCL input into its own and, except in the last step,
 *     fetches the share of segment r + (3 + s) dir from the user input;
 *   level 1: the template between the servers on segment r of the CCL input / output buffers;
 *   all-gather (alg_template/temp_all_gather/aligned_all_gather_double_ring.cc:343-449): in step s copies the share of
 *     segment r + (1 + s) dir from rank r + dir's CCL output to its own, in the last step straight to the user
 *     output, and copies the share of segment r + s dir from its CCL output to the user output. */
static int dbring_build(HgOpList* l, int alg1, uint32_t n_servers, uint32_t n_local, uint64_t count, uint64_t ccl_bytes,
                        int dtype)
{
    const uint32_t unit = HcommGfxDataTypeSize((HcommDataType)dtype);
    if (unit == 0 || count > HG_MAX_COUNT || n_servers == 0 || n_local == 0 || (uint64_t)n_servers * n_local > HCOMM_GFX_MAX_RANKS) return HCCL_E_PARA;
    if (alg1 != HCOMM_GFX_ALG_ALLREDUCE_RING && alg1 != HCOMM_GFX_ALG_ALLREDUCE_NHR && alg1 != HCOMM_GFX_ALG_ALLREDUCE_NB)
        return HCCL_E_PARA; /* the level-1 choices of coll_all_reduce_ring_for_910_93_executor.cc:304-351 built here */
    const uint64_t max_count = ccl_bytes / unit;
    if (max_count == 0) return HCCL_E_PARA;
    const uint32_t N = n_local;
    int rc = HCCL_SUCCESS;
    uint32_t step = 0;
    uint64_t user_off = 0;
    HcommGfxSlice seg[HCOMM_GFX_MAX_RANKS], share[2][HCOMM_GFX_MAX_RANKS];
    uint32_t map[HCOMM_GFX_MAX_RANKS];
    for (uint64_t left = count; left > 0 && rc == HCCL_SUCCESS;) {
        const uint64_t cur = left > max_count ? max_count : left;
        CHK(HcommGfxCalcSlices(cur, unit, N, seg));
        for (uint32_t i = 0; i < N; ++i) {
            uint64_t first = ((seg[i].size + 1) / 2 + 127u) / 128u * 128u;
            if (first > seg[i].size) first = seg[i].size;
            share[0][i].offset = seg[i].offset;
            share[0][i].size = first;
            share[1][i].offset = seg[i].offset + first;
            share[1][i].size = seg[i].size - first;
        }
#define SEG(r, k, dir) (((r) + (uint64_t)N * 4u + (uint64_t)(k) * ((dir) ? 1u : N - 1u)) % N) /* r + k * (+1 | -1) mod N */
        for (uint32_t srv = 0; srv < n_servers && rc == HCCL_SUCCESS; ++srv) {
            const uint32_t g0 = srv * N;
            if (N == 1) { /* OneRankMemcpy of both templates */
                for (uint32_t ring = 0; ring < 2; ++ring)
                    CHK(push(l, step, COPY, g0, IN, share[ring][0].offset, g0, UIN, user_off + share[ring][0].offset, share[ring][0].size));
                continue;
            }
            for (uint32_t r = 0; r < N; ++r)
                for (uint32_t ring = 0; ring < 2; ++ring)
                    for (uint32_t k = 1; k <= 2; ++k) {
                        const HcommGfxSlice* x = &share[ring][SEG(r, k, ring)];
                        CHK(push(l, step, COPY, g0 + r, IN, x->offset, g0 + r, UIN, user_off + x->offset, x->size));
                    }
            for (uint32_t s = 0; s + 1 < N; ++s)
                for (uint32_t r = 0; r < N; ++r)
                    for (uint32_t ring = 0; ring < 2; ++ring) {
                        const HcommGfxSlice* x = &share[ring][SEG(r, 2 + s, ring)];
                        CHK(push(l, step + 1 + s, REDUCE, g0 + r, IN, x->offset, g0 + (uint32_t)SEG(r, 1, ring), IN, x->offset, x->size));
                        if (s + 2 == N) continue;
                        x = &share[ring][SEG(r, 3 + s, ring)];
                        CHK(push(l, step + 1 + s, COPY, g0 + r, IN, x->offset, g0 + r, UIN, user_off + x->offset, x->size));
                    }
        }
        step += N == 1 ? 1 : N;
        /* level 1 */
        int alg = alg1;
        if (alg1 == HCOMM_GFX_ALG_ALLREDUCE_NHR && cur * unit / N <= 256u * 1024u) alg = HCOMM_GFX_ALG_ALLREDUCE_NHR_ONESHOT;
        uint32_t used = 0;
        for (uint32_t i = 0; i < N && rc == HCCL_SUCCESS; ++i) {
            HgOpList sub;
            for (uint32_t srv = 0; srv < n_servers; ++srv) map[srv] = srv * N + i;
            rc = hg_schedule(&sub, alg, n_servers, seg[i].size / unit, seg[i].size / unit, dtype);
            if (rc != HCCL_SUCCESS) break;
            rc = append_mapped(l, &sub, map, step, seg[i].offset, 0, &used);
            hg_oplist_free(&sub);
        }
        step += used;
        /* all-gather */
        for (uint32_t srv = 0; srv < n_servers && rc == HCCL_SUCCESS; ++srv) {
            const uint32_t g0 = srv * N;
            if (N == 1) {
                for (uint32_t ring = 0; ring < 2; ++ring)
                    CHK(push(l, step, COPY, g0, UOUT, user_off + share[ring][0].offset, g0, OUT, share[ring][0].offset, share[ring][0].size));
                continue;
            }
            for (uint32_t s = 0; s + 1 < N; ++s)
                for (uint32_t r = 0; r < N; ++r)
                    for (uint32_t ring = 0; ring < 2; ++ring) {
                        const HcommGfxSlice* x = &share[ring][SEG(r, 1 + s, ring)];
                        const int last = s + 2 == N;
                        CHK(push(l, step + s, COPY, g0 + r, last ? UOUT : OUT, (last ? user_off : 0) + x->offset,
                                 g0 + (uint32_t)SEG(r, 1, ring), OUT, x->offset, x->size));
                        x = &share[ring][SEG(r, s, ring)];
                        CHK(push(l, step + s, COPY, g0 + r, UOUT, user_off + x->offset, g0 + r, OUT, x->offset, x->size));
                    }
        }
#undef SEG
        step += N == 1 ? 1 : N - 1;
        user_off += cur * unit;
        left -= cur;
    }
    if (rc != HCCL_SUCCESS) return rc;
    return order_by_step_rank(l);
}

int hg_schedule_dbring(HgOpList* l, int alg1, uint32_t n_servers, uint32_t n_local, uint64_t count, uint64_t ccl_bytes,
                       int dtype)
{
    memset(l, 0, sizeof(*l));
    const int rc = dbring_build(l, alg1, n_servers, n_local, count, ccl_bytes, dtype);
    if (rc != HCCL_SUCCESS) hg_oplist_free(l);
    return rc;
}

int32_t HcommGfxDoubleRingEmit(
    HcommGfxAlgorithm level1Alg, uint32_t nServers, uint32_t nLocal, uint64_t count, uint64_t cclBytes,
    HcommDataType dataType, HcommGfxSchedOp* ops, uint64_t cap, uint64_t* n)
{
    if (!n) return HCCL_E_PTR;
    HgOpList l;
    int rc = hg_schedule_dbring(&l, (int)level1Alg, nServers, nLocal, count, cclBytes, (int)dataType);
    if (rc != HCCL_SUCCESS) return rc;
    *n = l.n;
    if (ops) {
        const uint64_t m = l.n < cap ? l.n : cap;
        if (m) memcpy(ops, l.ops, m * sizeof(*ops));
    }
    hg_oplist_free(&l);
    return HCCL_SUCCESS;
}

/* Stand-alone ReduceScatterRecursiveHalvingDoubling (temp_reduce_scatter/reduce_scatter_recursive_hd.cc:29-84) in place
 * on `bytes` of every rank's input, slices of bytes / n (:86-110, not aligned): the even ranks below 2 (n - B), B the
 * largest power of two <= n, absorb their odd neighbour's whole input (:112-186); the B survivors halve (block rank b
 * folds, at distance m = B/2, B/4, .., 1, the group of m block slices that contains its own from block rank b ^ m,
 * reduce_scatter_halving_doubling.cc:65-92,196-249; a survivor that absorbed a neighbour owns both slices); finally the
 * absorbed odd ranks fetch their slice from the neighbour (:238-300). */
static int rhd_rs_inplace(HgOpList* l, uint32_t n, uint64_t bytes)
{
    if (n == 1) return HCCL_SUCCESS;
    const uint32_t block = floor_pow2(n);
    const uint32_t folded = n - block; /* pairs (2i, 2i + 1), i < folded */
    const uint64_t per = bytes / n;
    uint32_t step = 0;
    if (folded) {
        for (uint32_t i = 0; i < folded; ++i) CHK(push(l, step, REDUCE, 2 * i, IN, 0, 2 * i + 1, IN, 0, bytes));
        ++step;
    }
    /* block rank b stands for rank real(b) and owns the slices of ranks [first_rank(b), first_rank(b + 1)) */
#define REAL_OF(b) ((b) < folded ? 2u * (b) : (b) + folded)
    for (uint32_t m = block / 2; m >= 1; m /= 2, ++step)
        for (uint32_t b = 0; b < block; ++b) {
            const uint32_t g = b & ~(m - 1);
            const uint64_t lo = (uint64_t)REAL_OF(g) * per, hi = (uint64_t)(g + m < block ? REAL_OF(g + m) : n) * per;
            CHK(push(l, step, REDUCE, REAL_OF(b), IN, lo, REAL_OF(b ^ m), IN, lo, hi - lo));
        }
#undef REAL_OF
    if (folded) {
        for (uint32_t i = 0; i < folded; ++i)
            CHK(push(l, step, COPY, 2 * i + 1, IN, (uint64_t)(2 * i + 1) * per, 2 * i, IN, (uint64_t)(2 * i + 1) * per, per));
        ++step;
    }
    return HCCL_SUCCESS;
}

/* ---- the ring and mesh reduce-scatter executors over two communicator levels (op-base mode) --------------------- */

/* CollReduceScatterRingExecutor::KernelRun (coll_executor/coll_reduce_scatter/coll_reduce_scatter_ring_executor.cc:
 * 136-363, single ring, every device with a NIC) and CollReduceScatterMeshExecutor::KernelRun
 * (coll_reduce_scatter_mesh_executor.cc:131-259, the branch without atomic adds) inside the loop of
 * CollReduceScatterExecutor (coll_reduce_scatter_executor.cc:149-306, buffer-copy mode) with their own chunk size
 * cclBytes / (N * unit) (:116-121 / :116-121).  N = n_servers * n_local, rank = server * n_local + local index, block b
 * of the input belongs to rank b.  Per chunk of c bytes per block:
 *   0. user input -> CCL input, block by block (one copy when a single chunk takes everything, :262-266);
 *   1. between the servers, in place on the CCL inputs: reduce-scatter (ring, NHR in slice order, or NB) over the
 *      n_servers runs of n_local blocks - rank (s, l) ends up with run s summed over the ranks (., l);
 *   2. inside every server, in place, at base offset = the server's run: ring reduce-scatter over the n_local blocks
 *      of the run, or the multi-stream mesh reduce-scatter over their pieces;
 *   3. the rank's own block CCL input -> CCL output (:359 / :255), then CCL output -> user output (:293-298). */
static int hier_rs_build(HgOpList* l, int level0_mesh, int alg1, uint32_t n_servers, uint32_t n_local, uint64_t count,
                         uint64_t ccl_bytes, uint32_t unit, int dtype)
{
    (void)dtype;
    const uint32_t n = n_servers * n_local;
    const uint64_t max_count = ccl_bytes / ((uint64_t)n * unit);
    if (max_count == 0) return HCCL_E_PARA;
    uint32_t step = 0, map[HCOMM_GFX_MAX_RANKS];
    uint64_t user_off = 0;
    HcommGfxSlice sl[HCOMM_GFX_MAX_RANKS];
    for (uint64_t left = count; left > 0;) {
        const uint64_t cur = left > max_count ? max_count : left;
        const uint64_t c = cur * unit;
        /* 0 */
        for (uint32_t r = 0; r < n; ++r) {
            if (cur == count) {
                CHK(push(l, step, COPY, r, IN, 0, r, UIN, 0, c * n));
                continue;
            }
            for (uint32_t b = 0; b < n; ++b) CHK(push(l, step, COPY, r, IN, c * b, r, UIN, user_off + count * unit * b, c));
        }
        ++step;
        /* 1 */
        if (n_servers > 1) {
            HgOpList sub;
            memset(&sub, 0, sizeof(sub));
            for (uint32_t i = 0; i < n_servers; ++i) {
                sl[i].offset = c * n_local * i;
                sl[i].size = c * n_local;
            }
            int rc;
            if (alg1 == HCOMM_GFX_ALG_REDUCE_SCATTER_RING) rc = ring_rs(&sub, n_servers, sl, 0);
            else if (alg1 == HCOMM_GFX_ALG_REDUCE_SCATTER_NHR) {
                uint32_t order[HCOMM_GFX_MAX_RANKS];
                nhr_slice_map(n_servers, 1, order);
                rc = nhr_rs(&sub, n_servers, sl, order, 0);
            } else if (alg1 == HCOMM_GFX_ALG_REDUCE_SCATTER_NB) rc = nb_rs(&sub, n_servers, sl);
            else rc = rhd_rs_inplace(&sub, n_servers, c * n);
            uint32_t used = 0;
            for (uint32_t i = 0; i < n_local && rc == HCCL_SUCCESS; ++i) {
                for (uint32_t srv = 0; srv < n_servers; ++srv) map[srv] = srv * n_local + i;
                rc = append_mapped(l, &sub, map, step, 0, 0, &used);
            }
            hg_oplist_free(&sub);
            CHK(rc);
            step += used;
        }
        /* 2 */
        for (uint32_t i = 0; i < n_local; ++i) {
            sl[i].offset = c * i;
            sl[i].size = c;
        }
        if (n_local > 1) {
            HgOpList sub;
            memset(&sub, 0, sizeof(sub));
            int rc = level0_mesh ? mesh_level0_rs(&sub, 0, n_local, sl, 0) : ring_rs(&sub, n_local, sl, 0);
            uint32_t used = 0;
            for (uint32_t srv = 0; srv < n_servers && rc == HCCL_SUCCESS; ++srv) {
                for (uint32_t i = 0; i < n_local; ++i) map[i] = srv * n_local + i;
                rc = append_mapped(l, &sub, map, step, c * n_local * srv, 0, &used);
            }
            hg_oplist_free(&sub);
            CHK(rc);
            step += n_local - 1;
        }
        /* 3 */
        for (uint32_t r = 0; r < n; ++r) CHK(push(l, step, COPY, r, OUT, 0, r, IN, c * r, c));
        ++step;
        for (uint32_t r = 0; r < n; ++r) CHK(push(l, step, COPY, r, UOUT, user_off, r, OUT, 0, c));
        ++step;
        user_off += c;
        left -= cur;
    }
    return order_by_step_rank(l);
}

int hg_schedule_hier_rs(HgOpList* l, int level0_mesh, int alg1, uint32_t n_servers, uint32_t n_local, uint64_t count,
                        uint64_t ccl_bytes, int dtype)
{
    memset(l, 0, sizeof(*l));
    const uint32_t unit = HcommGfxDataTypeSize((HcommDataType)dtype);
    if (unit == 0 || count > HG_MAX_COUNT || n_servers == 0 || n_local == 0 || (uint64_t)n_servers * n_local > HCOMM_GFX_MAX_RANKS) return HCCL_E_PARA;
    if (level0_mesh && n_local < 2) return HCCL_E_PARA; /* PrepareSliceMeshStreams refuses zero streams */
    if (alg1 != HCOMM_GFX_ALG_REDUCE_SCATTER_RING && alg1 != HCOMM_GFX_ALG_REDUCE_SCATTER_NHR &&
        alg1 != HCOMM_GFX_ALG_REDUCE_SCATTER_NB && alg1 != HCOMM_GFX_ALG_REDUCE_SCATTER_RHD)
        return HCCL_E_PARA;
    const int rc = hier_rs_build(l, level0_mesh, alg1, n_servers, n_local, count, ccl_bytes, unit, dtype);
    if (rc != HCCL_SUCCESS) hg_oplist_free(l);
    return rc;
}

int32_t HcommGfxHierReduceScatterEmit(
    int32_t level0Mesh, HcommGfxAlgorithm level1Alg, uint32_t nServers, uint32_t nLocal, uint64_t count, uint64_t cclBytes,
    HcommDataType dataType, HcommGfxSchedOp* ops, uint64_t cap, uint64_t* n)
{
    if (!n) return HCCL_E_PTR;
    HgOpList l;
    int rc = hg_schedule_hier_rs(&l, level0Mesh != 0, (int)level1Alg, nServers, nLocal, count, cclBytes, (int)dataType);
    if (rc != HCCL_SUCCESS) return rc;
    *n = l.n;
    if (ops) {
        const uint64_t m = l.n < cap ? l.n : cap;
        if (m) memcpy(ops, l.ops, m * sizeof(*ops));
    }
    hg_oplist_free(&l);
    return HCCL_SUCCESS;
}

/* ---- the double-ring reduce-scatter executor on one server (op-base mode, DMA reduce) ------------------------------ */

/* CollAlignedReduceScatterDoubleRingFor91093Executor on a single server (coll_executor/coll_reduce_scatter/
 * coll_aligned_reduce_scatter_double_ring_for_910_93_executor.cc:22-86; slices and user-memory slices of its base,
 * coll_reduce_scatter_ring_for_910_93_executor.cc:213-316; template alg_template/temp_reduce_scatter/
 * aligned_reduce_scatter_double_ring.cc with both user addresses set), chunked by the reduce-scatter loop.  Per chunk of
 * c bytes per block, with dir = -1 for ring 0 (first shares) and +1 for ring 1 (second shares), every rank r
 *   step 0: fetches the shares of blocks r + dir and r + 2 dir from its user input into its CCL input;
 *   step 1 + s, s < N - 2: folds the share of block r + (2 + s) dir of rank r + dir's CCL input into its own and
 *     fetches the share of block r + (3 + s) dir - which for s = N - 3 is its own block and goes to the user output;
 *   last step: folds the share of its own block of rank r + dir's CCL input into its user output. */
static int dbring_rs_build(HgOpList* l, uint32_t n, uint64_t count, uint64_t ccl_bytes, uint32_t unit)
{
    const uint64_t max_count = ccl_bytes / n / 128u * 128u / unit;
    if (max_count == 0) return HCCL_E_PARA;
    const uint64_t stride = count * unit;
    uint32_t step = 0;
    uint64_t user_off = 0;
    for (uint64_t left = count; left > 0;) {
        const uint64_t cur = left > max_count ? max_count : left;
        const uint64_t c = cur * unit;
        uint64_t first = ((c + 1) / 2 + 127u) / 128u * 128u; /* MutliSegSlicePrepare, coll_comm_executor.cc:2011-2052 */
        if (first > c) first = c;
        const uint64_t off[2] = {0, first}, len[2] = {first, c - first};
#define BLK(r, k, ring) (((r) + (uint64_t)n * 4u + (uint64_t)(k) * ((ring) ? 1u : n - 1u)) % n)
        for (uint32_t r = 0; r < n; ++r)
            for (uint32_t ring = 0; ring < 2; ++ring)
                for (uint32_t k = 1; k <= 2; ++k) {
                    const uint64_t b = BLK(r, k, ring);
                    CHK(push(l, step, COPY, r, IN, b * c + off[ring], r, UIN, user_off + b * stride + off[ring], len[ring]));
                }
        for (uint32_t s = 0; s + 1 < n; ++s)
            for (uint32_t r = 0; r < n; ++r)
                for (uint32_t ring = 0; ring < 2; ++ring) {
                    const uint64_t b = BLK(r, 2 + s, ring);
                    const uint32_t peer = (uint32_t)BLK(r, 1, ring);
                    if (s + 2 == n) {
                        CHK(push(l, step + 1 + s, REDUCE, r, UOUT, user_off + off[ring], peer, IN, b * c + off[ring], len[ring]));
                        continue;
                    }
                    CHK(push(l, step + 1 + s, REDUCE, r, IN, b * c + off[ring], peer, IN, b * c + off[ring], len[ring]));
                    const uint64_t nb = BLK(r, 3 + s, ring);
                    if (s + 3 == n)
                        CHK(push(l, step + 1 + s, COPY, r, UOUT, user_off + off[ring], r, UIN, user_off + nb * stride + off[ring], len[ring]));
                    else
                        CHK(push(l, step + 1 + s, COPY, r, IN, nb * c + off[ring], r, UIN, user_off + nb * stride + off[ring], len[ring]));
                }
#undef BLK
        step += n;
        user_off += c;
        left -= cur;
    }
    return HCCL_SUCCESS;
}

int hg_schedule_dbring_rs(HgOpList* l, uint32_t n, uint64_t count, uint64_t ccl_bytes, int dtype)
{
    memset(l, 0, sizeof(*l));
    const uint32_t unit = HcommGfxDataTypeSize((HcommDataType)dtype);
    if (unit == 0 || count > HG_MAX_COUNT || n < 3 || n > HCOMM_GFX_MAX_RANKS) return HCCL_E_PARA;
    const int rc = dbring_rs_build(l, n, count, ccl_bytes, unit);
    if (rc != HCCL_SUCCESS) hg_oplist_free(l);
    return rc;
}

int32_t HcommGfxDoubleRingReduceScatterEmit(
    uint32_t nRanks, uint64_t count, uint64_t cclBytes, HcommDataType dataType, HcommGfxSchedOp* ops, uint64_t cap,
    uint64_t* n)
{
    if (!n) return HCCL_E_PTR;
    HgOpList l;
    int rc = hg_schedule_dbring_rs(&l, nRanks, count, cclBytes, (int)dataType);
    if (rc != HCCL_SUCCESS) return rc;
    *n = l.n;
    if (ops) {
        const uint64_t m = l.n < cap ? l.n : cap;
        if (m) memcpy(ops, l.ops, m * sizeof(*ops));
    }
    hg_oplist_free(&l);
    return HCCL_SUCCESS;
}

/* ---- the double-ring reduce-scatter executor over servers and super pods (op-base mode, DMA reduce) ---------------- */

/* Append `sub`, a list over the ranks of one communicator level, once per `copies`: operation by operation, copy c shifted
 * by c * shift bytes (the templates walk the slices of a slice index one after the other: reduce_scatter_ring.cc:221-224,
 * 242-245, reduce_scatter_nhr.cc:573-579, reduce_scatter_nb.cc:174). */
static int append_mapped_copies(HgOpList* l, const HgOpList* sub, const uint32_t* map, uint32_t step0, uint64_t base,
                                uint32_t copies, uint64_t shift)
{
    for (uint64_t i = 0; i < sub->n; ++i) {
        const HcommGfxSchedOp* o = &sub->ops[i];
        for (uint32_t c = 0; c < copies; ++c)
            CHK(push(l, step0 + o->step, o->kind, map[o->rank], o->dstBuf, o->dstOff + base + c * shift, map[o->srcRank],
                     o->srcBuf, o->srcOff + base + c * shift, o->bytes));
    }
    return HCCL_SUCCESS;
}

static int level_rs(HgOpList* sub, int alg, uint32_t n, const HcommGfxSlice* sl)
{
    if (alg == HCOMM_GFX_ALG_REDUCE_SCATTER_RING) return ring_rs(sub, n, sl, 0);
    if (alg == HCOMM_GFX_ALG_REDUCE_SCATTER_NB) return nb_rs(sub, n, sl);
    uint32_t order[HCOMM_GFX_MAX_RANKS];
    nhr_slice_map(n, 1, order);
    return nhr_rs(sub, n, sl, order, 0);
}

static uint32_t level_rs_steps(int alg, uint32_t n)
{
    return n < 2 ? 0u : (alg == HCOMM_GFX_ALG_REDUCE_SCATTER_RING ? n - 1u : ceil_log2(n));
}

/* CollAlignedReduceScatterDoubleRingFor91093Executor with several servers and super pods (KernelRun of its base,
 * coll_executor/coll_reduce_scatter/coll_reduce_scatter_ring_for_910_93_executor.cc:595-812).  With P pods of S servers of
 * N devices, rank = (pod * S + server) * N + local index, block g = the output of rank g, per chunk of c bytes per block
 * and dir = -1 for ring 0 (first shares), +1 for ring 1 (second shares), every rank (p, s, r):
 *   step 0: fetches the shares of blocks k * N + (r + dir) and k * N + (r + 2 dir), k = 0 .. P * S - 1, from its user
 *     input into its CCL input - every ring position carries one slice per server of every pod (FillMultiRingSlice
 *     :213-233, user offsets :297-313; aligned_reduce_scatter_double_ring.cc:305-332);
 *   step 1 + t, t < N - 1: folds the shares of blocks k * N + (r + (2 + t) dir) of rank (p, s, r + dir)'s CCL input into
 *     its own and, except in the last of these steps, fetches those of blocks k * N + (r + (3 + t) dir) (:366-425; the
 *     user output address is null here, :664-670, so nothing goes to the user output yet);
 *   then (S > 1) the reduce-scatter between the servers of a pod (ring, NHR or NB, :689-746) in place on the CCL input
 *     buffers of the ranks (p, 0, r) .. (p, S - 1, r): server i's rank owns the blocks (q * S + i) * N + r of every pod q
 *     (:327-350), walked one after the other wherever the template touches a slice;
 *   then (P > 1) the one between the pods (:748-797) over the ranks (0, s, r) .. (P - 1, s, r), slice i = block
 *     (i * S + s) * N + r (:376-382);
 *   last: the own block from the CCL input to the user output (:800-808). */
static int dbring_rs_servers_build(HgOpList* l, int alg1, int alg2, uint32_t n_pods, uint32_t n_srv, uint32_t n, uint64_t count,
                                   uint64_t ccl_bytes, uint32_t unit)
{
    const uint32_t groups = n_pods * n_srv, total = groups * n;
    const uint64_t max_count = ccl_bytes / total / 128u * 128u / unit; /* CalcLoopMaxCount, :167-173 */
    if (max_count == 0) return HCCL_E_PARA;
    const uint64_t stride = count * unit;
    uint32_t step = 0, map[HCOMM_GFX_MAX_RANKS];
    uint64_t user_off = 0;
    HcommGfxSlice sl[HCOMM_GFX_MAX_RANKS];
    for (uint64_t left = count; left > 0;) {
        const uint64_t cur = left > max_count ? max_count : left;
        const uint64_t c = cur * unit;
        uint64_t first = ((c + 1) / 2 + 127u) / 128u * 128u; /* MutliSegSlicePrepare, coll_comm_executor.cc:2011-2052 */
        if (first > c) first = c;
        const uint64_t off[2] = {0, first}, len[2] = {first, c - first};
#define BLK(r, k, ring) (((r) + (uint64_t)n * 4u + (uint64_t)(k) * ((ring) ? 1u : n - 1u)) % n)
        for (uint32_t g = 0; g < total; ++g) {
            const uint32_t r = g % n;
            for (uint32_t k = 0; k < groups; ++k)
                for (uint32_t ring = 0; ring < 2; ++ring)
                    for (uint32_t j = 1; j <= 2; ++j) {
                        const uint64_t b = (uint64_t)k * n + BLK(r, j, ring);
                        CHK(push(l, step, COPY, g, IN, b * c + off[ring], g, UIN, user_off + b * stride + off[ring], len[ring]));
                    }
        }
        for (uint32_t t = 0; t + 1 < n; ++t)
            for (uint32_t g = 0; g < total; ++g) {
                const uint32_t r = g % n, grp = g / n;
                for (uint32_t ring = 0; ring < 2; ++ring) {
                    const uint32_t peer = grp * n + (uint32_t)BLK(r, 1, ring);
                    for (uint32_t k = 0; k < groups; ++k) {
                        const uint64_t b = (uint64_t)k * n + BLK(r, 2 + t, ring);
                        CHK(push(l, step + 1 + t, REDUCE, g, IN, b * c + off[ring], peer, IN, b * c + off[ring], len[ring]));
                        if (t + 2 == n) continue;
                        const uint64_t nb = (uint64_t)k * n + BLK(r, 3 + t, ring);
                        CHK(push(l, step + 1 + t, COPY, g, IN, nb * c + off[ring], g, UIN, user_off + nb * stride + off[ring], len[ring]));
                    }
                }
            }
#undef BLK
        step += n;
        if (n_srv > 1) { /* between the servers of every pod: one list over S ranks, once per (pod, local index) */
            HgOpList sub;
            memset(&sub, 0, sizeof(sub));
            for (uint32_t i = 0; i < n_srv; ++i) {
                sl[i].offset = c * n * i;
                sl[i].size = c;
            }
            int rc = level_rs(&sub, alg1, n_srv, sl);
            for (uint32_t p = 0; p < n_pods && rc == HCCL_SUCCESS; ++p)
                for (uint32_t i = 0; i < n && rc == HCCL_SUCCESS; ++i) {
                    for (uint32_t srv = 0; srv < n_srv; ++srv) map[srv] = (p * n_srv + srv) * n + i;
                    rc = append_mapped_copies(l, &sub, map, step, c * i, n_pods, c * n * n_srv);
                }
            hg_oplist_free(&sub);
            CHK(rc);
            step += level_rs_steps(alg1, n_srv);
        }
        if (n_pods > 1) { /* between the pods: one list over P ranks, once per (server, local index) */
            HgOpList sub;
            memset(&sub, 0, sizeof(sub));
            for (uint32_t i = 0; i < n_pods; ++i) {
                sl[i].offset = c * n * n_srv * i;
                sl[i].size = c;
            }
            int rc = level_rs(&sub, alg2, n_pods, sl);
            for (uint32_t srv = 0; srv < n_srv && rc == HCCL_SUCCESS; ++srv)
                for (uint32_t i = 0; i < n && rc == HCCL_SUCCESS; ++i) {
                    for (uint32_t p = 0; p < n_pods; ++p) map[p] = (p * n_srv + srv) * n + i;
                    rc = append_mapped_copies(l, &sub, map, step, c * (srv * n + i), 1, 0);
                }
            hg_oplist_free(&sub);
            CHK(rc);
            step += level_rs_steps(alg2, n_pods);
        }
        for (uint32_t g = 0; g < total; ++g) CHK(push(l, step, COPY, g, UOUT, user_off, g, IN, c * g, c));
        ++step;
        user_off += c;
        left -= cur;
    }
    return order_by_step_rank(l);
}

static int level_alg_ok(int alg)
{
    return alg == HCOMM_GFX_ALG_REDUCE_SCATTER_RING || alg == HCOMM_GFX_ALG_REDUCE_SCATTER_NHR || alg == HCOMM_GFX_ALG_REDUCE_SCATTER_NB;
}

int hg_schedule_dbring_rs_servers(HgOpList* l, int alg1, int alg2, uint32_t n_pods, uint32_t n_servers, uint32_t n_local,
                                  uint64_t count, uint64_t ccl_bytes, int dtype)
{
    memset(l, 0, sizeof(*l));
    const uint32_t unit = HcommGfxDataTypeSize((HcommDataType)dtype);
    if (unit == 0 || count > HG_MAX_COUNT || n_pods == 0 || n_servers == 0 || (uint64_t)n_pods * n_servers < 2 || n_local < 3 ||
        (uint64_t)n_pods * n_servers * n_local > HCOMM_GFX_MAX_RANKS)
        return HCCL_E_PARA;
    if (!level_alg_ok(alg1) || !level_alg_ok(alg2)) return HCCL_E_PARA;
    const int rc = dbring_rs_servers_build(l, alg1, alg2, n_pods, n_servers, n_local, count, ccl_bytes, unit);
    if (rc != HCCL_SUCCESS) hg_oplist_free(l);
    return rc;
}

int32_t HcommGfxDoubleRingHierReduceScatterEmit(
    HcommGfxAlgorithm level1Alg, HcommGfxAlgorithm level2Alg, uint32_t nPods, uint32_t nServers, uint32_t nLocal, uint64_t count,
    uint64_t cclBytes, HcommDataType dataType, HcommGfxSchedOp* ops, uint64_t cap, uint64_t* n)
{
    if (!n) return HCCL_E_PTR;
    HgOpList l;
    int rc = hg_schedule_dbring_rs_servers(&l, (int)level1Alg, (int)level2Alg, nPods, nServers, nLocal, count, cclBytes, (int)dataType);
    if (rc != HCCL_SUCCESS) return rc;
    *n = l.n;
    if (ops) {
        const uint64_t m = l.n < cap ? l.n : cap;
        if (m) memcpy(ops, l.ops, m * sizeof(*ops));
    }
    hg_oplist_free(&l);
    return HCCL_SUCCESS;
}

/* ---- the order-preserving reduce-scatter executor (one server, op-base mode) ------------------------------------- */

/* CollReduceScatterOrderPreservedExecutor (coll_executor/coll_reduce_scatter/
 * coll_reduce_scatter_order_preserved_executor.cc:181-216, 260-283) around ReduceScatterPlantLocalReduce
 * (alg_template/temp_reduce_scatter/reduce_scatter_plant_local_reduce.cc), chunked by the reduce-scatter loop
 * (coll_reduce_scatter_executor.cc:149-220, DMA reduce: no staging copies).  Per chunk of c bytes:
 *   step 0: every rank q plants block p of its user input into slot (p + q) mod N of rank p's CCL output buffer
 *           (:166-185, :211-240) - so on every rank the slots, read from its own rank number on, hold the
 *           contributions of ranks 0, 1, 2, ... in that order;
 *   ceil(log2 N) rounds (:336-407): the contributions h .. min(N, 2h) - 1 are folded onto 0 .. for h = 2^(S-1), .., 1
 *           - the same tree over RANK order on every rank, which is what "order preserving" means;
 *   last step: slot p of rank p to its user output (:273-279). */
static int order_preserved_build(HgOpList* l, uint32_t n, uint64_t count, uint64_t ccl_bytes, uint32_t unit)
{
    const uint64_t max_count = ccl_bytes / n / 128u * 128u / unit;
    if (max_count == 0) return HCCL_E_PARA;
    const uint32_t rounds = ceil_log2(n);
    const uint64_t stride = count * unit;
    uint32_t step = 0;
    uint64_t user_off = 0;
    for (uint64_t left = count; left > 0;) {
        const uint64_t cur = left > max_count ? max_count : left;
        const uint64_t c = cur * unit;
        for (uint32_t p = 0; p < n; ++p) /* destination rank; q == p is the rank's own block */
            for (uint32_t q = 0; q < n; ++q) CHK(push(l, step, COPY, p, OUT, c * ((p + q) % n), q, UIN, user_off + stride * p, c));
        ++step;
        for (uint32_t h = 1u << (rounds ? rounds - 1 : 0); rounds && h >= 1; h >>= 1, ++step)
            for (uint32_t p = 0; p < n; ++p)
                for (uint32_t j = 0; j + h < (n < 2 * h ? n : 2 * h); ++j)
                    CHK(push(l, step, REDUCE, p, OUT, c * ((j + p) % n), p, OUT, c * ((h + j + p) % n), c));
        for (uint32_t p = 0; p < n; ++p) CHK(push(l, step, COPY, p, UOUT, user_off, p, OUT, c * p, c));
        ++step;
        user_off += c;
        left -= cur;
    }
    return HCCL_SUCCESS;
}

int hg_schedule_order_preserved(HgOpList* l, uint32_t n, uint64_t count, uint64_t ccl_bytes, int dtype)
{
    memset(l, 0, sizeof(*l));
    const uint32_t unit = HcommGfxDataTypeSize((HcommDataType)dtype);
    if (unit == 0 || count > HG_MAX_COUNT || n < 2 || n > HCOMM_GFX_MAX_RANKS) return HCCL_E_PARA;
    const int rc = order_preserved_build(l, n, count, ccl_bytes, unit);
    if (rc != HCCL_SUCCESS) hg_oplist_free(l);
    return rc;
}

int32_t HcommGfxOrderPreservedEmit(
    uint32_t nRanks, uint64_t count, uint64_t cclBytes, HcommDataType dataType, HcommGfxSchedOp* ops, uint64_t cap,
    uint64_t* n)
{
    if (!n) return HCCL_E_PTR;
    HgOpList l;
    int rc = hg_schedule_order_preserved(&l, nRanks, count, cclBytes, (int)dataType);
    if (rc != HCCL_SUCCESS) return rc;
    *n = l.n;
    if (ops) {
        const uint64_t m = l.n < cap ? l.n : cap;
        if (m) memcpy(ops, l.ops, m * sizeof(*ops));
    }
    hg_oplist_free(&l);
    return HCCL_SUCCESS;
}

/* ---- the order-preserving reduce-scatter executor's branch for small messages ----------------------------------- */

/* ReduceScatterHDStage (alg_template/temp_reduce_scatter/reduce_scatter_hd_stage.cc:110-140, 154-185, 205-250), the
 * branch CollReduceScatterOrderPreservedExecutor takes for at most 32 KiB per rank on one module of 4 or 8 devices in
 * op-base mode (coll_reduce_scatter_order_preserved_executor.cc:29-38, 141-169).  With T one block in bytes and
 * H = N / 2:
 *   step 0: rank p copies the half of its user input that holds block p (H blocks) to the front of its CCL output;
 *   step 1: rank p ^ H folds the same half of ITS user input into rank p's copy;
 *   steps 2 ..: for w = H / 2, H / 4, .., 1 rank p folds rank p ^ w's run of w blocks - the run that holds block p,
 *           at ((p / w) * w mod H) * T - into its own;
 *   last step: block p, at (p mod H) * T, to the user output.
 * The fold tree over rank order is the plant branch's; the two operands of a fold swap places from rank to rank. */
static int order_preserved_small_build(HgOpList* l, uint32_t n, uint64_t total)
{
    const uint32_t half = n / 2;
    uint32_t step = 0;
    for (uint32_t p = 0; p < n; ++p) CHK(push(l, step, COPY, p, OUT, 0, p, UIN, p >= half ? half * total : 0, half * total));
    ++step;
    for (uint32_t p = 0; p < n; ++p)
        CHK(push(l, step, REDUCE, p, OUT, 0, p ^ half, UIN, p >= half ? half * total : 0, half * total));
    ++step;
    for (uint32_t w = half / 2; w >= 1; w /= 2, ++step)
        for (uint32_t p = 0; p < n; ++p) {
            const uint64_t off = (uint64_t)(p / w * w % half) * total;
            CHK(push(l, step, REDUCE, p, OUT, off, p ^ w, OUT, off, w * total));
        }
    for (uint32_t p = 0; p < n; ++p) CHK(push(l, step, COPY, p, UOUT, 0, p, OUT, (uint64_t)(p % half) * total, total));
    return HCCL_SUCCESS;
}

int hg_schedule_order_preserved_small(HgOpList* l, uint32_t n, uint64_t count, uint64_t ccl_bytes, int dtype)
{
    memset(l, 0, sizeof(*l));
    const uint32_t unit = HcommGfxDataTypeSize((HcommDataType)dtype);
    if (unit == 0 || count > HG_MAX_COUNT || (n != 4 && n != 8)) return HCCL_E_PARA;
    if (count * unit > 32u * 1024u) return HCCL_E_PARA; /* HCCL_SMALL_COUNT_32_KB, alg_template/template_v1_utils.h:64 */
    /* the template takes the user input's block stride from the chunk (reduce_scatter_hd_stage.cc:156-160): the
     * executor's loop must not cut the message */
    if (count > ccl_bytes / n / 128u * 128u / unit) return HCCL_E_PARA;
    if (count == 0) return HCCL_SUCCESS;
    const int rc = order_preserved_small_build(l, n, count * unit);
    if (rc != HCCL_SUCCESS) hg_oplist_free(l);
    return rc;
}

int32_t HcommGfxOrderPreservedSmallEmit(
    uint32_t nRanks, uint64_t count, uint64_t cclBytes, HcommDataType dataType, HcommGfxSchedOp* ops, uint64_t cap,
    uint64_t* n)
{
    if (!n) return HCCL_E_PTR;
    HgOpList l;
    int rc = hg_schedule_order_preserved_small(&l, nRanks, count, cclBytes, (int)dataType);
    if (rc != HCCL_SUCCESS) return rc;
    *n = l.n;
    if (ops) {
        const uint64_t m = l.n < cap ? l.n : cap;
        if (m) memcpy(ops, l.ops, m * sizeof(*ops));
    }
    hg_oplist_free(&l);
    return HCCL_SUCCESS;
}

/* ---- the order-preserving allreduce executor (one server, op-base mode) ------------------------------------------- */

/* CollAllReduceOrderPreservedExecutor (coll_executor/coll_all_reduce/coll_all_reduce_order_preserved_executor.cc:
 * 131-193, 248-283, 342-380), chunked by the allreduce loop (coll_all_reduce_executor.cc:129-138, 212-252, DMA reduce:
 * no staging copies).  Per chunk of c elements: block size B = ceil(c / N) elements rounded up to 128 bytes, block d
 * = bytes [d * B, min((d + 1) * B, chunk bytes)) - the trailing blocks may be short or empty.
 *   step 0: every rank q plants block p of its user input into slot (p + q) mod N of rank p's CCL output buffer; the
 *           last slot of every rank but the last is "borrowed" from the rank's CCL INPUT buffer at p * B, so that the
 *           N slots of B bytes never reach past the chunk's size (reduce_scatter_plant_local_reduce.cc:168-188, 221-247);
 *   ceil(log2 N) rounds: the fold tree over rank order of the order-preserving reduce-scatter (:337-414);
 *   then the mesh all-gather of the N blocks inside the CCL output buffers (all_gather_mesh_atomic.cc:19-69: round r
 *           reads the block of rank p - r), and the whole chunk from there to the user output (:369-376). */
static int order_preserved_ar_build(HgOpList* l, uint32_t n, uint64_t count, uint64_t ccl_bytes, uint32_t unit)
{
    const uint64_t max_count = ccl_bytes / unit;
    if (max_count == 0) return HCCL_E_PARA;
    const uint32_t rounds = ceil_log2(n);
    const uint32_t last = n - 1;
    uint32_t step = 0;
    uint64_t user_off = 0;
    uint64_t size[HCOMM_GFX_MAX_RANKS];
    for (uint64_t left = count; left > 0;) {
        const uint64_t cur = left > max_count ? max_count : left;
        const uint64_t c = cur * unit;
        const uint64_t blk = ((cur + n - 1) / n * unit + 127u) / 128u * 128u;
        for (uint32_t d = 0; d < n; ++d) size[d] = (uint64_t)d * blk >= c ? 0 : (c - d * blk < blk ? c - d * blk : blk);
        /* the slots of rank p sit at multiples of blk: they fit the buffers whenever they fit the chunk; a tiny
         * chunk whose rounded-up blocks reach past the CCL buffer is an error in the reference as well (DeviceMem::range
         * hands back an empty range) */
        for (uint32_t p = 0; p < n; ++p)
            if (size[p] && (uint64_t)(p == last ? last : last - 1) * blk + size[p] > ccl_bytes) return HCCL_E_PARA;
        for (uint32_t p = 0; p < n; ++p)
            for (uint32_t q = 0; q < n; ++q) {
                const uint32_t slot = (p + q) % n;
                if (slot == last && p != last)
                    CHK(push(l, step, COPY, p, IN, blk * p, q, UIN, user_off + blk * p, size[p]));
                else
                    CHK(push(l, step, COPY, p, OUT, blk * slot, q, UIN, user_off + blk * p, size[p]));
            }
        ++step;
        for (uint32_t h = 1u << (rounds - 1); h >= 1; h >>= 1, ++step)
            for (uint32_t p = 0; p < n; ++p)
                for (uint32_t j = 0; j + h < (n < 2 * h ? n : 2 * h); ++j) {
                    const uint32_t to = (j + p) % n, from = (h + j + p) % n;
                    const int to_in = p != last && to == last, from_in = p != last && from == last;
                    CHK(push(l, step, REDUCE, p, to_in ? IN : OUT, to_in ? blk * p : blk * to, p, from_in ? IN : OUT,
                             from_in ? blk * p : blk * from, size[p]));
                }
        for (uint32_t p = 0; p < n; ++p)
            for (uint32_t r = 1; r < n; ++r) {
                const uint32_t src = (p + n - r) % n;
                CHK(push(l, step, COPY, p, OUT, blk * src, src, OUT, blk * src, size[src]));
            }
        ++step;
        for (uint32_t p = 0; p < n; ++p) CHK(push(l, step, COPY, p, UOUT, user_off, p, OUT, 0, c));
        ++step;
        user_off += c;
        left -= cur;
    }
    return HCCL_SUCCESS;
}

/* The same executor over M servers of L devices (rank = server * L + local index; :149-193, 208-246, 285-340 of
 * coll_all_reduce_order_preserved_executor.cc).  Per chunk, with B the rounded-up block size and block b at b * B:
 *   step 0 (level 0, all2allOffset 1): inside every server, for every group g (= the blocks g * L .. g * L + L - 1
 *           that server g will own), rank q plants block g * L + i into rank i's slot (1 + q + i) mod L of the
 *           group's region of the CCL output buffer; slot L - 1 is borrowed from the CCL input buffer at the block's
 *           own offset, except on the last device for the last group;
 *   ceil(log2 L) rounds: every group's contributions folded in device order; the partial lands in slot (1 + i) mod L,
 *           which is the borrowed place on device L - 2;
 *   next step (level 1, ReduceScatterPlantLocalReduceCombine, SDMA branch): device i of server c plants its partial
 *           for block i + d * L into slot (c + d) mod M of device i of server d, slot k being block i + k * L's own
 *           place in the CCL output buffer - free because the level-0 partials sit one slot further on; the last slot
 *           of the last device of every server but the last is borrowed again;
 *   ceil(log2 M) rounds: the partials folded in server order; block i + d * L ends up in its own place;
 *   mesh all-gather of the server's L blocks, then the all-gather of the M runs of L blocks between the servers
 *           (ring: M - 1 steps; NB / NHR with the slice order kept: ceil(log2 M) steps), then the chunk to the user
 *           output. */
static int order_preserved_ar2_build(HgOpList* l, int alg1, uint32_t n_srv, uint32_t n_loc, uint64_t count,
                                     uint64_t ccl_bytes, uint32_t unit)
{
    const uint64_t max_count = ccl_bytes / unit;
    if (max_count == 0) return HCCL_E_PARA;
    const uint32_t n = n_srv * n_loc, r0 = ceil_log2(n_loc), r1 = ceil_log2(n_srv);
    const uint32_t last_loc = n_loc - 1, last_srv = n_srv - 1;
    uint32_t step = 0;
    uint64_t user_off = 0;
    uint64_t size[HCOMM_GFX_MAX_RANKS];
    for (uint64_t left = count; left > 0;) {
        const uint64_t cur = left > max_count ? max_count : left;
        const uint64_t c = cur * unit;
        const uint64_t blk = ((cur + n - 1) / n * unit + 127u) / 128u * 128u;
        for (uint32_t b = 0; b < n; ++b) size[b] = (uint64_t)b * blk >= c ? 0 : (c - b * blk < blk ? c - b * blk : blk);
#define SRV(s, i) ((s) * n_loc + (i))
        const int single = n_loc == 1; /* one device per module: level 0 is a copy of the chunk into the CCL input buffer */
        if (single) {
            for (uint32_t p = 0; p < n; ++p) CHK(push(l, step, COPY, p, IN, 0, p, UIN, user_off, c));
            ++step;
        }
        /* level 0: plants */
        for (uint32_t s = 0; s < n_srv && !single; ++s)
            for (uint32_t i = 0; i < n_loc; ++i)     /* destination device */
                for (uint32_t q = 0; q < n_loc; ++q) /* planting device; per planter the groups in order */
                    for (uint32_t g = 0; g < n_srv; ++g) {
                        const uint32_t b = g * n_loc + i, slot = (1 + q + i) % n_loc;
                        if (slot == last_loc && !(i == last_loc && g == last_srv))
                            CHK(push(l, step, COPY, SRV(s, i), IN, blk * b, SRV(s, q), UIN, user_off + blk * b, size[b]));
                        else
                            CHK(push(l, step, COPY, SRV(s, i), OUT, blk * (g * n_loc + slot), SRV(s, q), UIN,
                                     user_off + blk * b, size[b]));
                    }
        if (!single) ++step;
        /* level 0: folds in device order; contribution k of device i sits in slot (1 + k + i) mod L */
        for (uint32_t h = single ? 0 : 1u << (r0 - 1); h >= 1; h >>= 1, ++step)
            for (uint32_t s = 0; s < n_srv; ++s)
                for (uint32_t i = 0; i < n_loc; ++i)
                    for (uint32_t g = 0; g < n_srv; ++g) {
                        const uint32_t b = g * n_loc + i;
                        const int may = !(i == last_loc && g == last_srv);
                        for (uint32_t j = 0; j + h < (n_loc < 2 * h ? n_loc : 2 * h); ++j) {
                            const uint32_t to = (1 + j + i) % n_loc, from = (1 + h + j + i) % n_loc;
                            const int to_in = may && to == last_loc, from_in = may && from == last_loc;
                            CHK(push(l, step, REDUCE, SRV(s, i), to_in ? IN : OUT, to_in ? blk * b : blk * (g * n_loc + to),
                                     SRV(s, i), from_in ? IN : OUT, from_in ? blk * b : blk * (g * n_loc + from), size[b]));
                        }
                    }
        /* level 1: device i of server c hands its partial for block i + d * L to server d.  With one device per module
         * the partials are the blocks of the chunk in the CCL input buffer, a block that would go to the borrowed place
         * of its own rank is there already, and the peers' plants come a step after the own ones: one of them may land
         * where the own block was read from */
        for (uint32_t d = 0; d < n_srv; ++d)
            for (uint32_t i = 0; i < n_loc; ++i)
                for (uint32_t c0 = 0; c0 < n_srv; ++c0) {
                    const uint32_t b = i + d * n_loc, slot = (c0 + d) % n_srv;
                    const int src_in = single || i + 2 == n_loc; /* the level-0 partial sits in the borrowed place */
                    const uint64_t src_off = src_in ? blk * (i + d * n_loc) : blk * ((1 + i) % n_loc + d * n_loc);
                    const uint32_t at = step + (single && c0 != d ? 1u : 0u);
                    if (i == last_loc && slot == last_srv && d != last_srv) {
                        if (!(single && c0 == d))
                            CHK(push(l, at, COPY, SRV(d, i), IN, blk * b, SRV(c0, i), src_in ? IN : OUT, src_off, size[b]));
                    } else {
                        CHK(push(l, at, COPY, SRV(d, i), OUT, blk * (i + slot * n_loc), SRV(c0, i), src_in ? IN : OUT, src_off,
                                 size[b]));
                    }
                }
        step += single ? 2 : 1;
        /* level 1: folds in server order; contribution k of server d sits in slot (k + d) mod M */
        for (uint32_t h = 1u << (r1 - 1); h >= 1; h >>= 1, ++step)
            for (uint32_t d = 0; d < n_srv; ++d)
                for (uint32_t i = 0; i < n_loc; ++i) {
                    const uint32_t b = i + d * n_loc;
                    const int may = i == last_loc && d != last_srv;
                    for (uint32_t j = 0; j + h < (n_srv < 2 * h ? n_srv : 2 * h); ++j) {
                        const uint32_t to = (j + d) % n_srv, from = (h + j + d) % n_srv;
                        const int to_in = may && to == last_srv, from_in = may && from == last_srv;
                        CHK(push(l, step, REDUCE, SRV(d, i), to_in ? IN : OUT, to_in ? blk * b : blk * (i + to * n_loc), SRV(d, i),
                                 from_in ? IN : OUT, from_in ? blk * b : blk * (i + from * n_loc), size[b]));
                    }
                }
        /* all-gather inside the servers */
        for (uint32_t s = 0; s < n_srv; ++s)
            for (uint32_t i = 0; i < n_loc; ++i)
                for (uint32_t k = 1; k < n_loc; ++k) {
                    const uint32_t peer = (i + n_loc - k) % n_loc, b = peer + s * n_loc;
                    CHK(push(l, step, COPY, SRV(s, i), OUT, blk * b, SRV(s, peer), OUT, blk * b, size[b]));
                }
        if (!single) ++step;
        /* all-gather of the servers' runs between the servers */
        uint64_t run[HCOMM_GFX_MAX_RANKS];
        for (uint32_t d = 0; d < n_srv; ++d) {
            run[d] = 0;
            for (uint32_t j = 0; j < n_loc; ++j) run[d] += size[d * n_loc + j];
        }
        const uint64_t run_stride = blk * n_loc;
        if (alg1 == HCOMM_GFX_ALG_ALLREDUCE_RING) {
            for (uint32_t k = 0; k + 1 < n_srv; ++k, ++step)
                for (uint32_t s = 0; s < n_srv; ++s)
                    for (uint32_t i = 0; i < n_loc; ++i) {
                        const uint32_t d = (s + 2 * n_srv - 1 - k) % n_srv, from = (s + n_srv - 1) % n_srv;
                        CHK(push(l, step, COPY, SRV(s, i), OUT, run_stride * d, SRV(from, i), OUT, run_stride * d, run[d]));
                    }
        } else if (alg1 == HCOMM_GFX_ALG_ALLREDUCE_NB) {
            for (uint32_t k = 0; k < r1; ++k, ++step) {
                const uint32_t cnt = (k + 1 == r1 && n_srv != (1u << r1)) ? n_srv - (1u << k) : (1u << k);
                for (uint32_t s = 0; s < n_srv; ++s)
                    for (uint32_t i = 0; i < n_loc; ++i)
                        for (uint32_t j = 0; j < cnt; ++j) {
                            const uint32_t d = modn((int64_t)s - (1 << k) - j, n_srv), from = modn((int64_t)s - (1 << k), n_srv);
                            CHK(push(l, step, COPY, SRV(s, i), OUT, run_stride * d, SRV(from, i), OUT, run_stride * d, run[d]));
                        }
            }
        } else {
            for (uint32_t k = 0; k < r1; ++k, ++step) {
                const uint32_t delta = 1u << (r1 - 1 - k);
                const uint32_t cnt = (n_srv - 1 + delta) / (2 * delta);
                for (uint32_t s = 0; s < n_srv; ++s)
                    for (uint32_t i = 0; i < n_loc; ++i)
                        for (uint32_t j = 0; j < cnt; ++j) {
                            const uint32_t d = modn((int64_t)s - delta - (int64_t)j * 2 * delta, n_srv);
                            CHK(push(l, step, COPY, SRV(s, i), OUT, run_stride * d, SRV(modn((int64_t)s - delta, n_srv), i), OUT,
                                     run_stride * d, run[d]));
                        }
            }
        }
        for (uint32_t p = 0; p < n; ++p) CHK(push(l, step, COPY, p, UOUT, user_off, p, OUT, 0, c));
        ++step;
#undef SRV
        user_off += c;
        left -= cur;
    }
    for (uint64_t k = 0; k < l->n; ++k) { /* the reference's DeviceMem::range refuses what reaches past a CCL buffer */
        const HcommGfxSchedOp* o = &l->ops[k];
        if ((o->dstBuf <= OUT && o->dstOff + o->bytes > ccl_bytes) || (o->srcBuf <= OUT && o->srcOff + o->bytes > ccl_bytes))
            return HCCL_E_PARA;
    }
    return HCCL_SUCCESS;
}

int hg_schedule_order_preserved_ar2(HgOpList* l, int alg1, uint32_t n_servers, uint32_t n_local, uint64_t count,
                                    uint64_t ccl_bytes, int dtype)
{
    memset(l, 0, sizeof(*l));
    const uint32_t unit = HcommGfxDataTypeSize((HcommDataType)dtype);
    if (unit == 0 || count > HG_MAX_COUNT || n_servers < 2 || n_local < 1 || (uint64_t)n_servers * n_local > HCOMM_GFX_MAX_RANKS) return HCCL_E_PARA;
    if (alg1 != HCOMM_GFX_ALG_ALLREDUCE_RING && alg1 != HCOMM_GFX_ALG_ALLREDUCE_NHR && alg1 != HCOMM_GFX_ALG_ALLREDUCE_NB)
        return HCCL_E_PARA;
    int rc = order_preserved_ar2_build(l, alg1, n_servers, n_local, count, ccl_bytes, unit);
    if (rc == HCCL_SUCCESS) rc = order_by_step_rank(l);
    if (rc != HCCL_SUCCESS) hg_oplist_free(l);
    return rc;
}

int32_t HcommGfxOrderPreservedHierAllReduceEmit(
    HcommGfxAlgorithm level1Alg, uint32_t nServers, uint32_t nLocal, uint64_t count, uint64_t cclBytes,
    HcommDataType dataType, HcommGfxSchedOp* ops, uint64_t cap, uint64_t* n)
{
    if (!n) return HCCL_E_PTR;
    HgOpList l;
    int rc = hg_schedule_order_preserved_ar2(&l, (int)level1Alg, nServers, nLocal, count, cclBytes, (int)dataType);
    if (rc != HCCL_SUCCESS) return rc;
    *n = l.n;
    if (ops) {
        const uint64_t m = l.n < cap ? l.n : cap;
        if (m) memcpy(ops, l.ops, m * sizeof(*ops));
    }
    hg_oplist_free(&l);
    return HCCL_SUCCESS;
}

/* The order-preserving reduce-scatter executor over M servers of L devices (coll_executor/coll_reduce_scatter/
 * coll_reduce_scatter_order_preserved_executor.cc:171-218, 220-258, 260-283): the two levels of the allreduce executor
 * above without any borrowed place - every block is one chunk of c bytes, block b of the CCL output buffer at b * c,
 * of the user input at b * count * unit - and the own block to the user output instead of the all-gathers. */
static int order_preserved_rs2_build(HgOpList* l, uint32_t n_srv, uint32_t n_loc, uint64_t count, uint64_t ccl_bytes,
                                     uint32_t unit)
{
    const uint32_t n = n_srv * n_loc, r0 = ceil_log2(n_loc), r1 = ceil_log2(n_srv);
    const uint64_t max_count = ccl_bytes / n / 128u * 128u / unit;
    if (max_count == 0) return HCCL_E_PARA;
    const uint64_t stride = count * unit;
    uint32_t step = 0;
    uint64_t user_off = 0;
    for (uint64_t left = count; left > 0;) {
        const uint64_t cur = left > max_count ? max_count : left;
        const uint64_t c = cur * unit;
        if (n_loc == 1) {
            /* one device per module (:123-139, :246-252): the N blocks of the chunk to the CCL input buffer; then the
             * plant stage between the servers WITH the borrowed place - block d's last slot on every rank d but the
             * last is where the block already lies in the CCL input buffer, so the own plant is dropped there and
             * the peers' plants follow a step later */
            const uint32_t last = n - 1;
            for (uint32_t p = 0; p < n; ++p)
                for (uint32_t b = 0; b < n; ++b) CHK(push(l, step, COPY, p, IN, c * b, p, UIN, user_off + stride * b, c));
            ++step;
            for (uint32_t d = 0; d < n; ++d)
                for (uint32_t c0 = 0; c0 < n; ++c0) {
                    const uint32_t slot = (c0 + d) % n;
                    if (slot == last && d != last) {
                        if (c0 != d) CHK(push(l, step + 1, COPY, d, IN, c * d, c0, IN, c * d, c));
                    } else {
                        CHK(push(l, step + (c0 != d ? 1u : 0u), COPY, d, OUT, c * slot, c0, IN, c * d, c));
                    }
                }
            step += 2;
            for (uint32_t h = 1u << (r1 - 1); h >= 1; h >>= 1, ++step)
                for (uint32_t d = 0; d < n; ++d)
                    for (uint32_t j = 0; j + h < (n < 2 * h ? n : 2 * h); ++j) {
                        const uint32_t to = (j + d) % n, from = (h + j + d) % n;
                        const int to_in = d != last && to == last, from_in = d != last && from == last;
                        CHK(push(l, step, REDUCE, d, to_in ? IN : OUT, to_in ? c * d : c * to, d, from_in ? IN : OUT,
                                 from_in ? c * d : c * from, c));
                    }
            for (uint32_t p = 0; p < n; ++p) CHK(push(l, step, COPY, p, UOUT, user_off, p, OUT, c * p, c));
            ++step;
            user_off += c;
            left -= cur;
            continue;
        }
#define SRV(s, i) ((s) * n_loc + (i))
        for (uint32_t s = 0; s < n_srv; ++s)
            for (uint32_t i = 0; i < n_loc; ++i)
                for (uint32_t q = 0; q < n_loc; ++q)
                    for (uint32_t g = 0; g < n_srv; ++g)
                        CHK(push(l, step, COPY, SRV(s, i), OUT, c * (g * n_loc + (1 + q + i) % n_loc), SRV(s, q), UIN,
                                 user_off + stride * (g * n_loc + i), c));
        ++step;
        for (uint32_t h = 1u << (r0 - 1); h >= 1; h >>= 1, ++step)
            for (uint32_t s = 0; s < n_srv; ++s)
                for (uint32_t i = 0; i < n_loc; ++i)
                    for (uint32_t g = 0; g < n_srv; ++g)
                        for (uint32_t j = 0; j + h < (n_loc < 2 * h ? n_loc : 2 * h); ++j)
                            CHK(push(l, step, REDUCE, SRV(s, i), OUT, c * (g * n_loc + (1 + j + i) % n_loc), SRV(s, i), OUT,
                                     c * (g * n_loc + (1 + h + j + i) % n_loc), c));
        for (uint32_t d = 0; d < n_srv; ++d)
            for (uint32_t i = 0; i < n_loc; ++i)
                for (uint32_t c0 = 0; c0 < n_srv; ++c0)
                    CHK(push(l, step, COPY, SRV(d, i), OUT, c * (i + (c0 + d) % n_srv * n_loc), SRV(c0, i), OUT,
                             c * ((1 + i) % n_loc + d * n_loc), c));
        ++step;
        for (uint32_t h = 1u << (r1 - 1); h >= 1; h >>= 1, ++step)
            for (uint32_t d = 0; d < n_srv; ++d)
                for (uint32_t i = 0; i < n_loc; ++i)
                    for (uint32_t j = 0; j + h < (n_srv < 2 * h ? n_srv : 2 * h); ++j)
                        CHK(push(l, step, REDUCE, SRV(d, i), OUT, c * (i + (j + d) % n_srv * n_loc), SRV(d, i), OUT,
                                 c * (i + (h + j + d) % n_srv * n_loc), c));
        for (uint32_t p = 0; p < n; ++p) CHK(push(l, step, COPY, p, UOUT, user_off, p, OUT, c * p, c));
        ++step;
#undef SRV
        user_off += c;
        left -= cur;
    }
    return HCCL_SUCCESS;
}

int hg_schedule_order_preserved_rs2(HgOpList* l, uint32_t n_servers, uint32_t n_local, uint64_t count, uint64_t ccl_bytes,
                                    int dtype)
{
    memset(l, 0, sizeof(*l));
    const uint32_t unit = HcommGfxDataTypeSize((HcommDataType)dtype);
    if (unit == 0 || count > HG_MAX_COUNT || n_servers < 2 || n_local < 1 || (uint64_t)n_servers * n_local > HCOMM_GFX_MAX_RANKS) return HCCL_E_PARA;
    int rc = order_preserved_rs2_build(l, n_servers, n_local, count, ccl_bytes, unit);
    if (rc == HCCL_SUCCESS) rc = order_by_step_rank(l);
    if (rc != HCCL_SUCCESS) hg_oplist_free(l);
    return rc;
}

int32_t HcommGfxOrderPreservedHierReduceScatterEmit(
    uint32_t nServers, uint32_t nLocal, uint64_t count, uint64_t cclBytes, HcommDataType dataType, HcommGfxSchedOp* ops,
    uint64_t cap, uint64_t* n)
{
    if (!n) return HCCL_E_PTR;
    HgOpList l;
    int rc = hg_schedule_order_preserved_rs2(&l, nServers, nLocal, count, cclBytes, (int)dataType);
    if (rc != HCCL_SUCCESS) return rc;
    *n = l.n;
    if (ops) {
        const uint64_t m = l.n < cap ? l.n : cap;
        if (m) memcpy(ops, l.ops, m * sizeof(*ops));
    }
    hg_oplist_free(&l);
    return HCCL_SUCCESS;
}

int hg_schedule_order_preserved_ar(HgOpList* l, uint32_t n, uint64_t count, uint64_t ccl_bytes, int dtype)
{
    memset(l, 0, sizeof(*l));
    const uint32_t unit = HcommGfxDataTypeSize((HcommDataType)dtype);
    if (unit == 0 || count > HG_MAX_COUNT || n < 2 || n > HCOMM_GFX_MAX_RANKS) return HCCL_E_PARA;
    const int rc = order_preserved_ar_build(l, n, count, ccl_bytes, unit);
    if (rc != HCCL_SUCCESS) hg_oplist_free(l);
    return rc;
}

int32_t HcommGfxOrderPreservedAllReduceEmit(
    uint32_t nRanks, uint64_t count, uint64_t cclBytes, HcommDataType dataType, HcommGfxSchedOp* ops, uint64_t cap,
    uint64_t* n)
{
    if (!n) return HCCL_E_PTR;
    HgOpList l;
    int rc = hg_schedule_order_preserved_ar(&l, nRanks, count, cclBytes, (int)dataType);
    if (rc != HCCL_SUCCESS) return rc;
    *n = l.n;
    if (ops) {
        const uint64_t m = l.n < cap ? l.n : cap;
        if (m) memcpy(ops, l.ops, m * sizeof(*ops));
    }
    hg_oplist_free(&l);
    return HCCL_SUCCESS;
}

int32_t HcommGfxHierEmit(
    HcommGfxAlgorithm level1Alg, uint32_t nServers, uint32_t nLocal, uint64_t count, HcommDataType dataType,
    HcommGfxSchedOp* ops, uint64_t cap, uint64_t* n)
{
    if (!n) return HCCL_E_PTR;
    HgOpList l;
    int rc = hg_schedule_hier(&l, 0, (int)level1Alg, nServers, nLocal, count, (int)dataType);
    if (rc != HCCL_SUCCESS) return rc;
    *n = l.n;
    if (ops) {
        const uint64_t m = l.n < cap ? l.n : cap;
        if (m) memcpy(ops, l.ops, m * sizeof(*ops));
    }
    hg_oplist_free(&l);
    return HCCL_SUCCESS;
}

int32_t HcommGfxMeshHierEmit(
    HcommGfxAlgorithm level1Alg, uint32_t nServers, uint32_t nLocal, uint64_t count, HcommDataType dataType,
    HcommGfxSchedOp* ops, uint64_t cap, uint64_t* n)
{
    if (!n) return HCCL_E_PTR;
    HgOpList l;
    int rc = hg_schedule_hier(&l, 1, (int)level1Alg, nServers, nLocal, count, (int)dataType);
    if (rc != HCCL_SUCCESS) return rc;
    *n = l.n;
    if (ops) {
        const uint64_t m = l.n < cap ? l.n : cap;
        if (m) memcpy(ops, l.ops, m * sizeof(*ops));
    }
    hg_oplist_free(&l);
    return HCCL_SUCCESS;
}
