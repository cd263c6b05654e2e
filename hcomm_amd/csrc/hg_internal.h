/*
 * hg_internal.h - interface between the C host code of libhcomm_gfx.so and its HIP launchers.
 * Plain C; included by the .c host files and by hg_kernels.hip.
 */
#ifndef HG_INTERNAL_H
#define HG_INTERNAL_H

#include <stddef.h>
#include <stdint.h>

#include "hcomm_gfx.h"

#ifdef __cplusplus
extern "C" {
#endif

#define HG_POS_BYTES 256u      /* leaf-position bytes of a tree launch */
#define HG_MAX_SEG 32u          /* segments per k-way fold launch */
#define HG_MAX_SEG2 64u         /* segments per copy / two-input reduce launch */
#define HG_DIRECT_SEG 8u        /* segments of a chain launch with host-resolved addresses */
#define HG_DIRECT_K 8u          /* inputs per segment of such a launch */
#define HG_VEC_BYTES 16u        /* one lane moves 128 bits per access */
#ifndef HG_BLOCK
#define HG_BLOCK 256u           /* threads per workgroup = 4 wavefronts of 64 */
#endif
#ifndef HG_UNROLL
#define HG_UNROLL 4u            /* 128-bit accesses in flight per lane and operand */
#endif
#ifndef HG_CHAIN_UNROLL
#define HG_CHAIN_UNROLL 2u      /* the same for the k-way chain fold at bandwidth-bound sizes: 8 KiB tiles (with 8 - 23
                                 * streams per lane the smaller tile is 4 - 5 % ahead of 16 KiB) */
#endif
#define HG_CHAIN_TILE_BYTES ((uint64_t)HG_BLOCK * HG_CHAIN_UNROLL * HG_VEC_BYTES)
#define HG_TILE_VECS (HG_BLOCK * HG_UNROLL)
#define HG_TILE_BYTES ((uint64_t)HG_TILE_VECS * HG_VEC_BYTES) /* 16 KiB of output per tile */
#define HG_TREE_TILE_BYTES ((uint64_t)HG_BLOCK * HG_VEC_BYTES) /* tree / small-message kernels: one access per lane and input */

/* Two-pointer segment table (copy, reduce2, bytewise), passed to the kernel by value. */
typedef struct {
    void* dst[HG_MAX_SEG2];
    const void* src[HG_MAX_SEG2];
    uint64_t bytes[HG_MAX_SEG2];
    uint32_t tile_begin[HG_MAX_SEG2 + 1]; /* prefix sum of tiles per segment */
    uint32_t nseg;
    uint32_t xcd_run; /* > 0: each XCD walks runs of this many consecutive tiles (block_id in hg_device.hpp) */
    uint32_t flat;    /* every segment is exactly one tile: tile t belongs to segment t, no search (small messages) */
    uint32_t direct;  /* > 0: small launch on a two-dimensional grid, y = segment, x = tile of it, this many tiles wide */
} HgSeg2Table;

/*
 * k-way fold table.  Segment s folds K values per element, position j = 0..K-1 being read from
 *   in[(first[s] + j * stride) mod nranks] + off[s]
 * (a rotation of the rank buffers, which is what every ring / mesh schedule uses), or, when
 * tree == 1, from in[first[s] XOR bitrev(j)] + off[s] (recursive halving), or, when tree == 2 / 3, from
 * in[(first[s] + j) mod nranks] / in[(first[s] - j) mod nranks] with only nranks <= k positions present (the
 * truncated trees of the nonuniform hierarchical ring / nonuniform Bruck schedules), or, when tree == 4, from
 * in[pos[j]] where pos[j] names a rank (the rank-order trees of the order-preserving executors, laid out by the host;
 * inputs only read), or, when tree == 5, from in[(first[s] - pos[j]) mod nranks] (the deterministic mesh
 * reduce-scatter's row of receive slots; inputs only read), or, when tree == 6, from in[pos[s * k + j]] (any
 * tree of depth log2 k per segment, laid out by the host from the schedule's own operation list; inputs only read).
 */
typedef struct {
    const void* in[HCOMM_GFX_MAX_RANKS];
    const void* in2[HCOMM_GFX_MAX_RANKS]; /* tree only: buffer folded into in[b] before the tree, or NULL */
    void* out[HCOMM_GFX_MAX_RANKS];
    uint64_t off[HG_MAX_SEG];     /* byte offset applied to every in[] (and out[] in fan-out mode) */
    uint64_t out_off[HG_MAX_SEG]; /* byte offset into out[owner[s]] in single-output mode */
    uint64_t bytes[HG_MAX_SEG];
    uint32_t tile_begin[HG_MAX_SEG + 1];
    uint32_t nseg;
    uint32_t k;              /* values folded per element */
    uint32_t nranks;         /* modulus of the rotation */
    int32_t stride;          /* +1 or -1 */
    uint32_t store_partials; /* store the running value to position j's buffer after fold step j >= 1 */
    uint32_t store_final_first; /* store the final value to position 0's buffer */
    uint32_t out_mode;       /* 0 none, 1 out[owner[s]] + out_off[s], 2 every out[r] + off[s] */
    uint32_t tree;           /* 0 chain; binary tree over k = 2^L positions: 1 recursive halving, 2 / 3 rotation + / -, 4 / 5 / 6 leaves from pos[] */
    uint32_t nout;           /* tree only: number of out[] entries that receive the result */
    uint32_t ascending;      /* chain only: 1 = position 0 is first[s], positions 1.. are ranks 0, 1, ... skipping first[s];
                              * 2 = position 0 is first[s], position j >= 1 is first[s] + 1 + (start[s] + j - 1) mod (nranks - 1):
                              * the other ranks in cyclic order, entered at distance start[s] + 1 */
    uint32_t keep_inputs;    /* tree modes 1 - 3: the partials the step-wise replay leaves in the inputs are not stored */
    uint32_t small;          /* chain only: latency-oriented variant (4 KiB tiles, loads issued 8 inputs at a time) */
    uint32_t nu;             /* tree only: 128-bit vectors per lane, i.e. tiles of 4 or 8 KiB: two for 4 or 8 leaf positions
                              * (the two sizes compiled both ways) in launches that write little beside their result, else one */
    uint32_t direct;         /* small chain that only reads its inputs, <= HG_DIRECT_K of them in <= HG_DIRECT_SEG segments:
                              * the launcher resolves every address on the host (one round of kernel-argument reads) */
    uint32_t xcd_run;        /* > 0: each XCD walks runs of this many consecutive tiles (block_id in hg_device.hpp) */
    uint32_t flat;           /* every segment is exactly one tile: tile t belongs to segment t, no search */
    uint8_t first[HG_MAX_SEG];
    uint8_t owner[HG_MAX_SEG];
    uint8_t start[HG_MAX_SEG]; /* chain with ascending == 2 only */
    /* tree == 4: the rank at leaf position q (tree == 5: how far below the segment's first rank it lies), or 255 where
     * the tree has a hole; tree == 6: a table of k entries per segment, segment s at pos[s * k ..], so that every
     * segment can have a tree of its own shape (nseg * k <= HG_POS_BYTES) */
    uint8_t pos[HG_POS_BYTES];
} HgFoldTable;

/* Launch geometry decided on the host so that recorder threads can report it without a GPU. */
uint64_t hg_grid_blocks(uint64_t total_tiles);

/* Launchers.  stream is a hipStream_t.  Return a HcclResult-compatible code. */
/* streaming: the launch shape for output nothing reads back soon (and, for the reduce, a non-temporal load of the operand it overwrites);
 * lds: bytes of dynamic LDS per workgroup, asked for only to bound the workgroups a CU runs at once */
/* backwards: the launch walks its table from the end - last segment first, every segment's last tile first */
int hg_launch_copy(void* stream, const HgSeg2Table* tab, uint64_t blocks, int streaming, uint32_t lds, int backwards);
int hg_launch_reduce2(void* stream, int dtype, int op, const HgSeg2Table* tab, uint64_t blocks, int streaming, uint32_t lds, int backwards);
int hg_launch_bytewise(void* stream, int is_reduce, int dtype, int op, const HgSeg2Table* tab, uint64_t blocks, int streaming,
                       uint32_t lds, int backwards);
int hg_launch_fold(void* stream, int dtype, int op, int acc_is_dst, const HgFoldTable* tab, uint64_t blocks, uint32_t lds);

/* Thin wrappers over the HIP runtime so that the C files need no HIP headers. */
int hg_rt_device_count(void);
int hg_rt_stream_create(void** stream);
int hg_rt_stream_destroy(void* stream);
int hg_rt_stream_sync(void* stream);
int hg_rt_event_create(void** ev);
int hg_rt_event_destroy(void* ev);
int hg_rt_event_record(void* ev, void* stream);
int hg_rt_stream_wait_event(void* stream, void* ev);
int hg_rt_malloc(void** p, size_t n);
int hg_rt_free(void* p);
int hg_rt_num_cus(void);
/* The library's own per-GPU array of HCOMM_GFX_NOALLOC_SCRATCH_BYTES bytes: its address on the device `stream` belongs to. */
int hg_rt_scratch(void* stream, void** ptr);
/* Graph replay of a fixed launch list: capture between begin/end on `stream`, then launch the executable. */
int hg_rt_stream_is_capturing(void* stream);
int hg_rt_capture_begin(void* stream);
int hg_rt_capture_end(void* stream, void** graph_exec);
int hg_rt_graph_launch(void* graph_exec, void* stream);
int hg_rt_graph_destroy(void* graph_exec);

#ifdef __cplusplus
}
#endif
#endif
