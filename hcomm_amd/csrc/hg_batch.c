/*
 * hg_batch.c - turning recorded primitive calls into kernel launches.
 *
 * The reference's batch mode only records between HcommBatchModeStart and HcommBatchModeEnd and submits
 * once at End (src/base_comm/primitives/launch_context.cc:23-43,139-174).  Here "submitting" additionally
 * merges runs of operations that cannot observe each other into one launch, which is how all N simulated
 * ranks of a collective step end up in a single kernel.  The independence test is the memory-conflict rule
 * of the reference's schedule checker (test/st/algorithm/README_en.md:202-231): within one launch no
 * written range may overlap any other range that is read or written.
 */
#include <stdlib.h>
#include <string.h>

#include "hg_host.h"

/* Settings read from the environment on first use, possibly by several host threads at once: each computes the same
 * value; relaxed atomics keep that defined.  0 = not read yet. */
static uint64_t g_grid_cap = 0; /* UINT64_MAX = not set */
static uint64_t g_small_bytes = 0;
static uint64_t g_direct_bytes = 0;
static uint64_t g_direct_tiles = 0;
static uint64_t g_direct_tree_bytes = 0;

static uint64_t env_once(uint64_t* slot, const char* name, uint64_t unset)
{
    uint64_t v = __atomic_load_n(slot, __ATOMIC_RELAXED);
    if (v == 0) {
        const char* e = getenv(name);
        v = e ? strtoull(e, NULL, 10) : 0;
        if (v == 0) v = unset;
        __atomic_store_n(slot, v, __ATOMIC_RELAXED);
    }
    return v;
}

/* Whether launches may take the kernels that read their arguments in one round - the (tile, segment) grids and the
 * fold launches whose addresses the host resolves (HcommGfxSetDirectLaunches; HCOMM_GFX_DIRECT=0 in the environment
 * starts with them off). */
static int g_direct_state = 0; /* 0 not read yet, 1 off, 2 on */

static int direct_on(void)
{
    int v = __atomic_load_n(&g_direct_state, __ATOMIC_RELAXED);
    if (v == 0) {
        const char* e = getenv("HCOMM_GFX_DIRECT");
        v = (e && e[0] == '0') ? 1 : 2;
        __atomic_store_n(&g_direct_state, v, __ATOMIC_RELAXED);
    }
    return v == 2;
}

/* A copy / two-input reduce launch that writes more than this many bytes may walk its table backwards (direction_of
 * in hg_api.c): HCOMM_GFX_ALTERNATE_BYTES, 0 = no launch does. */
static uint64_t g_alternate = 0; /* 0 = not read yet; else the threshold + 1, UINT64_MAX = never */

static uint64_t alternate_encode(uint64_t bytes) { return (bytes == 0 || bytes >= UINT64_MAX - 1u) ? UINT64_MAX : bytes + 1u; }

uint64_t hg_alternate_bytes(void)
{
    uint64_t v = __atomic_load_n(&g_alternate, __ATOMIC_RELAXED);
    if (v == 0) {
        const char* e = getenv("HCOMM_GFX_ALTERNATE_BYTES");
        v = alternate_encode((e && *e) ? strtoull(e, NULL, 10) : (128ull << 20));
        __atomic_store_n(&g_alternate, v, __ATOMIC_RELAXED);
    }
    return v - 1u; /* never: UINT64_MAX - 1, which no launch exceeds */
}

uint64_t HcommGfxSetAlternateBytes(uint64_t bytes)
{
    const uint64_t before = hg_alternate_bytes();
    __atomic_store_n(&g_alternate, alternate_encode(bytes), __ATOMIC_RELAXED);
    return before == UINT64_MAX - 1u ? 0 : before;
}

int32_t HcommGfxSetDirectLaunches(int32_t enable)
{
    const int32_t before = direct_on();
    __atomic_store_n(&g_direct_state, enable ? 2 : 1, __ATOMIC_RELAXED);
    return before;
}

uint64_t hg_grid_blocks(uint64_t total_tiles)
{
    /* One tile per workgroup, however many that makes: measured with the streaming probe, every grid held at a fixed
     * number of workgroups per CU streams slower (16 x 64 MiB two-input reduce: 5.7 TB/s at 32 per CU, 6.4 without a
     * limit; copy 5.8 against 6.4).  HCOMM_GFX_GRID_CAP limits the grid for experiments. */
    const uint64_t forced = env_once(&g_grid_cap, "HCOMM_GFX_GRID_CAP", UINT64_MAX);
    if (forced != UINT64_MAX) return total_tiles < forced ? total_tiles : forced;
    return total_tiles;
}

/*
 * Launch shapes of the copy and the two-input reduce, from a stand-alone streaming probe built on hg_device.hpp (
 * 16 KiB tiles, bf16 SUM, seeded non-zero data, sc1 stores) and confirmed per workload in the library.  Two regimes:
 *   kept      small enough to stay in the caches until the next launch reads it: the overwritten operand loaded plain,
 *             as many workgroups per CU as the registers allow (reduce) or at most three (copy, in runs of 64 tiles:
 *             8 x 16 MiB ring steps on cold operands 45.0 -> 42.7 us, inside a ring 38.0 -> 37.8).
 *   streaming every load non-temporal.  16 x 64 MiB that nothing touched recently: reduce 477 us with at most three
 *             workgroups per CU and runs of 32 tiles (499 with runs of 128, 522 with two workgroups), copy 320 us with
 *             at most two and runs of 64 (331 with three and runs of 128).
 * A copy streams when it writes more than the 256 MB memory-side cache holds.  A reduce streams from 64 MiB on: with the
 * sc1 stores its streaming shape is ahead of the kept one on ring steps too, whether or not the step before left the peer
 * operand in that cache (library, same box: ring allreduce 8 x 128 MiB 0.709 -> 0.705 ms, two-level ring allreduce 2 x 8
 * 1.457 -> 1.436, order-preserving reduce-scatter 0.787 -> 0.775; at 16 MiB the cache-resident 8 x 4 MiB mesh steps lose
 * 2 % with it).
 * The bound on workgroups per CU is a dynamic LDS size nobody uses as memory: 160 KiB of LDS per CU / 52 KiB = 3.
 * Every figure can be overridden from the environment for experiments.
 */
#define HG_TUNE_AUTO (UINT64_MAX - 1u) /* no value from the environment: the launch's own properties decide */
enum {
    TUNE_STREAM_COPY_BYTES, TUNE_STREAM_REDUCE_BYTES, TUNE_LDS_COPY, TUNE_LDS_COPY_STREAM, TUNE_LDS_REDUCE,
    TUNE_LDS_REDUCE_STREAM, TUNE_RUN_COPY, TUNE_RUN_COPY_STREAM, TUNE_RUN_REDUCE, TUNE_RUN_REDUCE_STREAM, TUNE_LDS_CHAIN, TUNE_RUN_CHAIN, TUNE_LDS_TREE,
    TUNE_RUN_TREE, TUNE_LDS_TREE_TABLES, TUNE_N
};
static const struct {
    const char* env;
    uint64_t dflt;
} g_tune_def[TUNE_N] = {
    {"HCOMM_GFX_STREAM_COPY_BYTES", 256ull << 20},   /* the 256 MB memory-side cache */
    {"HCOMM_GFX_STREAM_REDUCE_BYTES", 64ull << 20},
    {"HCOMM_GFX_LDS_COPY", 53248},
    {"HCOMM_GFX_LDS_COPY_STREAM", 65536},
    {"HCOMM_GFX_LDS_REDUCE", 0},
    {"HCOMM_GFX_LDS_REDUCE_STREAM", 53248},
    {"HCOMM_GFX_XCD_RUN_COPY", 64},
    {"HCOMM_GFX_XCD_RUN_COPY_STREAM", 64},
    {"HCOMM_GFX_XCD_RUN_REDUCE", 128},
    {"HCOMM_GFX_XCD_RUN_REDUCE_STREAM", 32},
    /* the k-way folds, measured on their single-launch lowerings.  Tree (16 x 128 MiB int32 recursive halving, 8 x
     * 128 MiB bf16 NHR): 1.005 -> 0.957 ms and 0.519 -> 0.502 ms with the bound and the runs (inputs kept: 0.785 ->
     * 0.720, 0.398 -> 0.377).  Chain: decided per launch (chain_shape below) unless the environment names a value. */
    {"HCOMM_GFX_LDS_CHAIN", HG_TUNE_AUTO},
    {"HCOMM_GFX_XCD_RUN_CHAIN", HG_TUNE_AUTO},
    {"HCOMM_GFX_LDS_TREE", 53248},
    {"HCOMM_GFX_XCD_RUN_TREE", 128},
    /* trees read from per-segment tables (the lowering of operation lists): four workgroups per CU (deterministic mesh
     * allreduce 8 x 128 MiB in one launch 0.383 -> 0.360 ms; the other tree modes lose 1 - 3 % with it) */
    {"HCOMM_GFX_LDS_TREE_TABLES", 40960},
};
static uint64_t g_tune[TUNE_N]; /* value + 1; 0 = not read yet (same relaxed-atomic rule as env_once) */


#define HG_XCD_RUN_MAX 65536u /* tiles per XCD run: the kernels compute 8 * run in 32 bits */

static uint64_t tune(int i)
{
    uint64_t v = __atomic_load_n(&g_tune[i], __ATOMIC_RELAXED);
    if (v == 0) {
        const char* e = getenv(g_tune_def[i].env);
        v = (e && *e ? strtoull(e, NULL, 10) : g_tune_def[i].dflt);
        const int is_run = i == TUNE_RUN_COPY || i == TUNE_RUN_COPY_STREAM || i == TUNE_RUN_REDUCE ||
                           i == TUNE_RUN_REDUCE_STREAM || i == TUNE_RUN_CHAIN || i == TUNE_RUN_TREE;
        if (is_run && v > HG_XCD_RUN_MAX && v != HG_TUNE_AUTO) v = HG_XCD_RUN_MAX;
        v += 1u;
        __atomic_store_n(&g_tune[i], v, __ATOMIC_RELAXED);
    }
    return v - 1u;
}

#define HG_LDS_MAX 65536u /* what a launch may ask for without raising the kernel's limit */

static uint32_t lds_of(int i)
{
    const uint64_t v = tune(i);
    return v > HG_LDS_MAX ? HG_LDS_MAX : (uint32_t)v;
}

/* Shape of a copy / two-input reduce launch from the bytes it writes; `streaming` < 0 lets the size decide. */
void hg_shape_seg2(HgLaunch* l, int streaming)
{
    HgSeg2Table* t = &l->tab.seg2;
    /* the kernel for operands off 16-byte boundaries comes as a copy (op 255) and as a reduce: shaped like them */
    const int copy = l->kind == HCOMM_GFX_KERNEL_COPY || (l->kind == HCOMM_GFX_KERNEL_BYTEWISE && l->op == 255u);
    const int bytewise = l->kind == HCOMM_GFX_KERNEL_BYTEWISE;
    if ((bytewise && copy) || (!bytewise && t->direct == 0u)) {
        /* The copy for unaligned operands and the one-dimensional kernels (ragged tables; a few more rounds of argument
         * reads before the data) want more workgroups per CU than the row-grid kernels the table above was swept with:
         * a ragged 512 MiB copy launch 170 against 187 us; the unaligned copy of 56 blocks of 16,777,214 bytes loses
         * 17 % with two workgroups per CU.  The reduce for unaligned operands reads both operands in aligned vectors
         * and is shaped like the aligned reduce (order-preserving reduce-scatter on such blocks 0.818 -> 0.788 ms). */
        l->streaming = streaming >= 0 ? (uint32_t)streaming : (l->bytes > (256ull << 20));
        l->lds_bytes = l->streaming ? 53248u : (copy ? 32768u : 0u);
        t->xcd_run = (l->streaming && !copy) ? 32u : 128u;
        return;
    }
    if (copy) {
        l->streaming = streaming >= 0 ? (uint32_t)streaming : (l->bytes > tune(TUNE_STREAM_COPY_BYTES));
        l->lds_bytes = lds_of(l->streaming ? TUNE_LDS_COPY_STREAM : TUNE_LDS_COPY);
        t->xcd_run = (uint32_t)tune(l->streaming ? TUNE_RUN_COPY_STREAM : TUNE_RUN_COPY);
    } else {
        l->streaming = streaming >= 0 ? (uint32_t)streaming : (l->bytes > tune(TUNE_STREAM_REDUCE_BYTES));
        l->lds_bytes = lds_of(l->streaming ? TUNE_LDS_REDUCE_STREAM : TUNE_LDS_REDUCE);
        t->xcd_run = (uint32_t)tune(l->streaming ? TUNE_RUN_REDUCE_STREAM : TUNE_RUN_REDUCE);
    }
}

static uint64_t tiles_of(uint64_t bytes) { return (bytes + HG_TILE_BYTES - 1) / HG_TILE_BYTES; }

void hg_finish_seg2(HgLaunch* l)
{
    HgSeg2Table* t = &l->tab.seg2;
    uint64_t tiles = 0, bytes = 0;
    for (uint32_t s = 0; s < t->nseg; ++s) {
        t->tile_begin[s] = (uint32_t)tiles;
        tiles += tiles_of(t->bytes[s]);
        bytes += t->bytes[s];
    }
    t->tile_begin[t->nseg] = (uint32_t)tiles;
    t->flat = 1u;
    for (uint32_t s = 0; s < t->nseg; ++s)
        if (t->tile_begin[s] != s || t->tile_begin[s + 1] != s + 1u) t->flat = 0u;
    l->nseg = t->nseg;
    l->bytes = bytes;
    l->moved_bytes = bytes * ((l->op == 255u) ? 2u : 3u);
    l->blocks = hg_grid_blocks(tiles);
    /* A two-dimensional grid (segment, tile of it: one round of kernel-argument reads instead of four or five) where
     * that wastes few workgroups: segments of nearly equal length at any size (at most an eighth more workgroups than
     * tiles), anything up to HCOMM_GFX_DIRECT_TILES tiles as long as the grid at most doubles.  Launches that small
     * are latency-bound and take neither the occupancy bound nor the XCD runs. */
    t->direct = 0u;
    const int small = tiles <= env_once(&g_direct_tiles, "HCOMM_GFX_DIRECT_TILES", 512u);
    if (direct_on() && tiles != 0 && l->kind != HCOMM_GFX_KERNEL_BYTEWISE) {
        uint32_t w = 0;
        for (uint32_t s = 0; s < t->nseg; ++s) {
            const uint32_t n = t->tile_begin[s + 1] - t->tile_begin[s];
            if (n > w) w = n;
        }
        const uint64_t grid = (uint64_t)w * t->nseg;
        if (grid <= tiles + tiles / 8u || (small && grid <= 2u * tiles)) {
            t->direct = w;
            l->blocks = grid;
        }
    }
    hg_shape_seg2(l, -1);
    if (small && (t->direct || l->kind == HCOMM_GFX_KERNEL_BYTEWISE)) {
        l->streaming = 0;
        l->lds_bytes = 0;
        t->xcd_run = 0;
    }
}

/* what HcommGfxLaunchRecord.rows reports */
uint32_t hg_launch_rows(const HgLaunch* l)
{
    if (l->kind == HCOMM_GFX_KERNEL_COPY || l->kind == HCOMM_GFX_KERNEL_REDUCE2) return l->tab.seg2.direct;
    if (l->kind == HCOMM_GFX_KERNEL_CHAIN || l->kind == HCOMM_GFX_KERNEL_TREE) return l->tab.fold.direct;
    return 0;
}

/* rank whose buffer a chain reads at position j of segment s (the kernels' fold_rank) */
static uint32_t chain_rank(const HgFoldTable* t, uint32_t s, uint32_t j)
{
    if (t->ascending == 1u) return j == 0 ? t->first[s] : ((j - 1 < t->first[s]) ? j - 1 : j);
    if (t->ascending == 2u) {
        if (j == 0) return t->first[s];
        const uint32_t r = t->first[s] + 1u + (t->start[s] + j - 1u) % (t->nranks - 1u);
        return r >= t->nranks ? r - t->nranks : r;
    }
    int32_t r = ((int32_t)t->first[s] + (int32_t)j * t->stride) % (int32_t)t->nranks;
    return (uint32_t)(r < 0 ? r + (int32_t)t->nranks : r);
}

/*
 * Launch shape of a chain fold.  What a chain launch costs is decided by how much it WRITES: eight read streams alone
 * run at 0.86 of the bus, a mix goes as reads / 0.86 + writes / w with w = 0.92 for one stream written by few
 * workgroups per CU in long runs per XCD and 0.65 - 0.78 for eight or fifteen streams written from a full CU, and no
 * arrangement inside the kernel (phases, tile size, load depth, buffer placement) changes the sum by more than 5 %.
 * So a launch that does not fit the memory-side cache takes the shape its writes like: 15 writes per 8 reads (the
 * ring allreduce with its partials) two workgroups per CU in runs of 128 tiles (8 x 128 MiB: 0.566 -> 0.536 ms); 6 per
 * 7 (the ring reduce-scatter stage) three per CU in runs of 128 (7 x 100,000,003 fp32: 0.922 -> 0.844 ms, and 0.907
 * with two); 8 per 8 (the allreduce without partials, chunk-mesh) three per CU in runs of 64 (0.380 -> 0.361, 0.387
 * -> 0.381).  One-byte elements cost four times the arithmetic per byte and want the waves to hide it: four per CU
 * (int8 reduce-scatter 0.223 -> 0.219 ms, 0.264 with two).  Launches whose operands stay in that cache keep tiles as
 * dealt and no bound (8 x 4 MiB one-shot mesh: 37 us, 48 with runs).
 */
static void chain_shape(HgLaunch* l)
{
    HgFoldTable* t = &l->tab.fold;
    const uint64_t lds = tune(TUNE_LDS_CHAIN), run = tune(TUNE_RUN_CHAIN);
    uint64_t footprint = 0;
    for (uint32_t s = 0; s < t->nseg; ++s) {
        for (uint32_t j = 0; j < t->k; ++j) { /* inputs, each range once however many segments read it */
            const uint32_t r = chain_rank(t, s, j);
            int seen = 0;
            for (uint32_t s2 = 0; s2 < s && !seen; ++s2)
                if (t->off[s2] == t->off[s])
                    for (uint32_t j2 = 0; j2 < t->k && !seen; ++j2) seen = chain_rank(t, s2, j2) == r;
            if (!seen) footprint += t->bytes[s];
        }
        footprint += t->bytes[s] * (t->out_mode == 2u ? t->nranks : t->out_mode == 1u ? 1u : 0u);
    }
    const int big = footprint > tune(TUNE_STREAM_COPY_BYTES) && !t->small;
    const uint32_t reads = t->k;
    const uint32_t writes = (t->store_partials ? t->k - 1u : 0u) + (t->store_final_first ? 1u : 0u) +
                            (t->out_mode == 2u ? t->nranks : t->out_mode == 1u ? 1u : 0u);
    const uint32_t bound = HcommGfxDataTypeSize((HcommDataType)l->dtype) == 1u ? 40960u : (2u * writes > 3u * reads ? 65536u : 53248u);
    l->lds_bytes = lds != HG_TUNE_AUTO ? (lds > HG_LDS_MAX ? HG_LDS_MAX : (uint32_t)lds) : (big ? bound : 0u);
    t->xcd_run = run != HG_TUNE_AUTO ? (uint32_t)run : (big ? (t->store_partials ? 128u : 64u) : 0u);
}

void hg_finish_fold(HgLaunch* l)
{
    HgFoldTable* t = &l->tab.fold;
    uint64_t tiles = 0, bytes = 0;
    l->streaming = 0;
    if (t->tree) {
        l->lds_bytes = lds_of(t->tree == 6u ? TUNE_LDS_TREE_TABLES : TUNE_LDS_TREE);
        t->xcd_run = (uint32_t)tune(TUNE_RUN_TREE);
    }
    if (!t->tree) {
        /* small messages are latency-bound: below the threshold the chain runs as the grouped-load variant */
        const uint64_t small_bytes = env_once(&g_small_bytes, "HCOMM_GFX_SMALL_BYTES", 1u << 20);
        uint64_t largest = 0;
        for (uint32_t s = 0; s < t->nseg; ++s)
            if (t->bytes[s] > largest) largest = t->bytes[s];
        /* measured cross-over with 8 ranks: 1 MiB per segment for read-only chains (mesh, k-way reduce), a
         * quarter of that when every position also stores its partial (ring) */
        const uint64_t limit = t->store_partials ? small_bytes / 4 : small_bytes;
        t->small = (largest <= limit) ? 1u : 0u;
        /* a chain of few inputs and segments runs with host-resolved addresses, which pays up to larger sizes
         * (read-only, 8 ranks x 4 MiB, everything cache-resident: 31 us against 37; at 16 MiB it no longer does; a
         * sixteenth of that when every position also stores its partial: 8 ranks x 2 MiB 10 us against 14, while
         * at 4 MiB on operands nothing touched recently the 16 KiB tiles are ahead again) */
        const uint64_t direct_bytes = env_once(&g_direct_bytes, "HCOMM_GFX_DIRECT_BYTES", 4u << 20);
        const uint64_t direct_limit = t->store_partials ? direct_bytes / 16 : direct_bytes;
        t->direct = (direct_on() && largest <= direct_limit && t->nseg <= HG_DIRECT_SEG && t->k >= 1u && t->k <= HG_DIRECT_K &&
                     (t->out_mode <= 1u || (t->out_mode == 2u && t->nranks <= HG_DIRECT_K)))
                        ? 1u
                        : 0u;
        if (t->direct) t->small = 1u;
        chain_shape(l);
    } else {
        /* small trees of up to 16 positions likewise (the launcher still checks what only it can see): up to 4 MiB
         * of output per launch (8 ranks: 16.6 us against 18.1 there, 72 against 68 at 16 MiB) */
        const uint64_t direct_bytes = env_once(&g_direct_tree_bytes, "HCOMM_GFX_DIRECT_TREE_BYTES", 4u << 20);
        uint64_t sum = 0;
        for (uint32_t s = 0; s < t->nseg; ++s) sum += t->bytes[s];
        t->direct = (direct_on() && sum <= direct_bytes && t->nseg <= HG_DIRECT_SEG && t->k <= 16u) ? 1u : 0u;
        /* what the host-resolved table does not carry: a neighbour absorbed before the tree (recursive halving on a
         * rank count that is not a power of two), more receivers than leaf positions */
        if (t->tree == 1u)
            for (uint32_t b = 0; b < HCOMM_GFX_MAX_RANKS; ++b)
                if (t->in2[b]) t->direct = 0u;
        if (!(t->tree != 1u && t->out_mode == 1u) && t->nout > t->k) t->direct = 0u;
    }
    t->nu = 1u;
    if (t->tree && (t->k == 4u || t->k == 8u)) {
        /* 8 KiB tiles unless the launch also stores partials into its inputs (recursive halving and the NHR / NB
         * rotations when the inputs are not kept) */
        const int stores_partials = t->tree <= 3u && !t->keep_inputs;
        t->nu = stores_partials ? 1u : 2u;
    }
    const uint64_t tile_bytes = t->tree ? HG_TREE_TILE_BYTES * t->nu : (t->small ? HG_TREE_TILE_BYTES : HG_CHAIN_TILE_BYTES);
    for (uint32_t s = 0; s < t->nseg; ++s) {
        t->tile_begin[s] = (uint32_t)tiles;
        tiles += (t->bytes[s] + tile_bytes - 1) / tile_bytes;
        bytes += t->bytes[s];
    }
    t->tile_begin[t->nseg] = (uint32_t)tiles;
    t->flat = 1u;
    for (uint32_t s = 0; s < t->nseg; ++s)
        if (t->tile_begin[s] != s || t->tile_begin[s + 1] != s + 1u) t->flat = 0u;
    l->nseg = t->nseg;
    l->bytes = bytes;
    uint64_t per = t->k; /* reads */
    if (t->tree) {
        /* per element: k leaf reads, one read per absorbed neighbour, one store per even position, one per odd
         * position that absorbed a neighbour (which block ranks sit on odd positions depends on the slice), and
         * nout outputs */
        uint64_t moved = 0;
        if (t->tree != 1u) {
            /* truncated rotation trees: nranks leaf reads, one store per even position that has a right neighbour
             * (none for the rank-order trees, which only read their inputs), and the root to one output or to all */
            const uint64_t n = (uint64_t)t->nranks + ((t->tree >= 4u || t->keep_inputs) ? 0u : t->nranks / 2) + (t->out_mode == 1u ? 1u : t->nout);
            l->moved_bytes = n * bytes;
            l->blocks = hg_grid_blocks(tiles);
            return;
        }
        for (uint32_t s = 0; s < t->nseg; ++s) {
            uint64_t n = t->k + (t->keep_inputs ? 0u : t->k / 2) + t->nout;
            for (uint32_t b = 0; b < t->k; ++b)
                if (t->in2[b]) n += 1 + ((!t->keep_inputs && ((b ^ t->first[s]) & (t->k / 2))) ? 1 : 0);
            moved += n * t->bytes[s];
        }
        l->moved_bytes = moved;
        l->blocks = hg_grid_blocks(tiles);
        return;
    } else {
        if (t->store_partials) per += t->k - 1;
        if (t->store_final_first) per += 1;
        if (t->out_mode == 1) per += 1;
        if (t->out_mode == 2) per += t->nranks;
    }
    l->moved_bytes = bytes * per;
    l->blocks = hg_grid_blocks(tiles);
}

static int overlaps(const void* a, uint64_t an, const void* b, uint64_t bn)
{
    const uintptr_t a0 = (uintptr_t)a, b0 = (uintptr_t)b;
    return a0 < b0 + bn && b0 < a0 + an;
}

static int aligned16(const HgOp* o) { return (((uintptr_t)o->dst | (uintptr_t)o->src) & (HG_VEC_BYTES - 1)) == 0; }

static uint32_t kind_of(const HgOp* o)
{
    if (!aligned16(o)) return HCOMM_GFX_KERNEL_BYTEWISE;
    return o->is_reduce ? HCOMM_GFX_KERNEL_REDUCE2 : HCOMM_GFX_KERNEL_COPY;
}

/* Operations with different keys never share a launch. */
uint32_t hg_op_launch_key(const HgOp* o)
{
    return kind_of(o) << 16 | (o->is_reduce ? (uint32_t)o->dtype << 8 | o->op : 0xffffu);
}

static int conflicts(const HgLaunch* l, const HgOp* o)
{
    const HgSeg2Table* t = &l->tab.seg2;
    for (uint32_t s = 0; s < t->nseg; ++s) {
        if (overlaps(o->dst, o->bytes, t->dst[s], t->bytes[s])) return 1;
        if (overlaps(o->dst, o->bytes, t->src[s], t->bytes[s])) return 1;
        if (overlaps(o->src, o->bytes, t->dst[s], t->bytes[s])) return 1;
    }
    return 0;
}

typedef struct {
    HgLaunch* l;
    int open;
    uint64_t bytes; /* written by the open launch so far */
    HgEmitFn emit;
    void* ctx;
} Coalescer;

/* A copy launch stops growing once it writes half a GiB.  Measured on the schedules whose copy steps are larger (the 64
 * plants of the order-preserving reduce-scatter, the gather of the deterministic mesh allreduce: 1 GiB written per
 * step): two launches of 512 MiB run 1 - 2 % faster than one of 1 GiB, while steps of many small segments (the 56
 * pieces of a mesh reduce-scatter round) gain 4 % from sharing one launch. */
#define HG_COPY_LAUNCH_BYTES (512ull << 20)

static uint64_t copy_launch_bytes(void)
{
    static uint64_t cap = 0;
    uint64_t v = __atomic_load_n(&cap, __ATOMIC_RELAXED);
    if (v == 0) {
        const char* e = getenv("HCOMM_GFX_COPY_LAUNCH_MIB"); /* experiments; 0 = no limit */
        v = e ? (strtoull(e, NULL, 10) ? strtoull(e, NULL, 10) << 20 : UINT64_MAX) : HG_COPY_LAUNCH_BYTES;
        __atomic_store_n(&cap, v, __ATOMIC_RELAXED);
    }
    return v;
}

/* segments a copy / two-input reduce launch may carry: the table's size, or less when HCOMM_GFX_MAX_SEGMENTS says so
 * (experiments) */
static uint32_t seg2_cap(void)
{
    static uint32_t cap = 0;
    uint32_t c = __atomic_load_n(&cap, __ATOMIC_RELAXED);
    if (c == 0) {
        const char* e = getenv("HCOMM_GFX_MAX_SEGMENTS");
        const unsigned long v = e ? strtoul(e, NULL, 10) : 0;
        c = (v >= 1 && v <= HG_MAX_SEG2) ? (uint32_t)v : HG_MAX_SEG2;
        __atomic_store_n(&cap, c, __ATOMIC_RELAXED);
    }
    return c;
}

static int coalesce_one(Coalescer* c, const HgOp* o)
{
    HgLaunch* l = c->l;
    const uint32_t kind = kind_of(o);
    const uint32_t dt = o->is_reduce ? o->dtype : 255u, op = o->is_reduce ? o->op : 255u;
    /* the work launch holds nothing defined until the first operation opens it */
    const int full = c->open && (l->tab.seg2.nseg == seg2_cap() ||
                                 (kind == HCOMM_GFX_KERNEL_COPY && c->bytes + o->bytes > copy_launch_bytes()));
    if (c->open && (l->kind != kind || l->dtype != dt || l->op != op || full || conflicts(l, o))) {
        hg_finish_seg2(l);
        c->open = 0;
        const int rc = c->emit(l, c->ctx);
        if (rc != HCCL_SUCCESS) return rc;
    }
    if (!c->open) {
        memset(l, 0, sizeof(*l));
        l->kind = kind;
        l->dtype = dt;
        l->op = op;
        c->open = 1;
        c->bytes = 0;
    }
    c->bytes += o->bytes;
    HgSeg2Table* t = &l->tab.seg2;
    t->dst[t->nseg] = o->dst;
    t->src[t->nseg] = o->src;
    t->bytes[t->nseg] = o->bytes;
    t->nseg++;
    return HCCL_SUCCESS;
}

/* Both operands equally far from a 16-byte boundary (a rank buffer addressed at an odd element offset): the few
 * bytes up to that boundary go to the kernel for unaligned operands and the rest runs on aligned accesses.  Below this size the
 * extra launch costs more than it saves. */
#define HG_SPLIT_MIN_BYTES (64u * 1024u)

/* Bytes of `o` that come before the 16-byte boundary both operands reach together; 0 when it is not to be cut. */
uint64_t hg_split_head(const HgOp* o)
{
    const uintptr_t md = (uintptr_t)o->dst & (HG_VEC_BYTES - 1), ms = (uintptr_t)o->src & (HG_VEC_BYTES - 1);
    const uint32_t es = o->is_reduce ? HcommGfxDataTypeSize((HcommDataType)o->dtype) : 1u;
    if (md != 0 && md == ms && o->bytes >= HG_SPLIT_MIN_BYTES && es != 0 && md % es == 0) return HG_VEC_BYTES - md;
    return 0;
}

/* One operation into the open launch (closing and emitting it first when the operation cannot join it). */
static int coalesce_op(Coalescer* c, const HgOp* o)
{
    if (o->bytes == 0) return HCCL_SUCCESS;                    /* count == 0: nothing to do (dispatcher.cc:719-722) */
    if (!o->is_reduce && o->dst == o->src) return HCCL_SUCCESS; /* copy onto itself (dispatcher.cc:495-498) */
    const uint64_t cut = hg_split_head(o);
    if (!cut) return coalesce_one(c, o);
    HgOp head = *o, body = *o;
    head.bytes = cut;
    body.dst = (char*)o->dst + head.bytes;
    body.src = (const char*)o->src + head.bytes;
    body.bytes = o->bytes - head.bytes;
    const int rc = coalesce_one(c, &head);
    return rc == HCCL_SUCCESS ? coalesce_one(c, &body) : rc;
}

int hg_coalesce_with(const HgOp* ops, uint64_t n, HgEmitFn emit, void* ctx, HgLaunch* work)
{
    Coalescer c;
    c.l = work;
    c.open = 0;
    c.bytes = 0;
    c.emit = emit;
    c.ctx = ctx;
    int rc = HCCL_SUCCESS;
    for (uint64_t i = 0; i < n && rc == HCCL_SUCCESS; ++i) rc = coalesce_op(&c, &ops[i]);
    if (c.open && rc == HCCL_SUCCESS) {
        hg_finish_seg2(c.l);
        rc = emit(c.l, ctx);
    }
    return rc;
}

int hg_coalesce(const HgOp* ops, uint64_t n, HgEmitFn emit, void* ctx)
{
    HgLaunch* work = (HgLaunch*)calloc(1, sizeof(HgLaunch));
    if (!work) return HCCL_E_MEMORY;
    const int rc = hg_coalesce_with(ops, n, emit, ctx, work);
    free(work);
    return rc;
}
