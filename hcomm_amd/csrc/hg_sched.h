/*
 * hg_sched.h - schedule op lists (see hg_sched.c).
 */
#ifndef HG_SCHED_H
#define HG_SCHED_H

#include "hcomm_gfx.h"

typedef struct {
    HcommGfxSchedOp* ops;
    uint64_t n, cap;
    uint32_t steps;
    int fixed; /* ops is storage of the caller's holding cap entries: never grown, never freed */
} HgOpList;

/* Fill `l` with the op list of `alg`; the caller releases it with hg_oplist_free. */
/* stride: elements between consecutive ranks' slices in the input of the scatter algorithms (0 = count). */
int hg_schedule(HgOpList* l, int alg, uint32_t n, uint64_t count, uint64_t stride, int dtype);
/* The same into a list the caller has set up (empty, or fixed storage: HCCL_E_INTERNAL when it does not fit). */
int hg_schedule_into(HgOpList* l, int alg, uint32_t n, uint64_t count, uint64_t stride, int dtype);
/* The op-base loop around alg: chunks of at most hg_opbase_max_count elements, each copied from the user input
 * into the CCL input buffer, run through the template, and copied from the CCL output to the user output. */
int hg_schedule_opbase(HgOpList* l, int alg, uint32_t n, uint64_t count, uint64_t ccl_bytes, int dtype);
uint64_t hg_opbase_max_count(int alg, uint32_t n, uint64_t ccl_bytes, uint32_t unit);
/* The ring executor's (level0_mesh 0) or the mesh executor's (1) three-step allreduce over n_servers x n_local ranks
 * with alg1 between the servers. */
int hg_schedule_hier(HgOpList* l, int level0_mesh, int alg1, uint32_t n_servers, uint32_t n_local, uint64_t count, int dtype);
/* The double-ring allreduce executor in op-base mode with DMA reduce: user buffers read and written directly, CCL
 * buffers of ccl_bytes in between, chunked like the op-base loop. */
int hg_schedule_dbring(HgOpList* l, int alg1, uint32_t n_servers, uint32_t n_local, uint64_t count, uint64_t ccl_bytes,
                       int dtype);
/* The order-preserving reduce-scatter executor on one server: all-to-all into the CCL output buffers, a fold tree in
 * rank order, own slot to the user output; chunked like the reduce-scatter loop. */
int hg_schedule_order_preserved(HgOpList* l, uint32_t n, uint64_t count, uint64_t ccl_bytes, int dtype);
int hg_schedule_order_preserved_ar(HgOpList* l, uint32_t n, uint64_t count, uint64_t ccl_bytes, int dtype);
int hg_schedule_order_preserved_small(HgOpList* l, uint32_t n, uint64_t count, uint64_t ccl_bytes, int dtype);
int hg_schedule_order_preserved_rs2(HgOpList* l, uint32_t n_servers, uint32_t n_local, uint64_t count, uint64_t ccl_bytes,
                                    int dtype);
int hg_schedule_order_preserved_ar2(HgOpList* l, int alg1, uint32_t n_servers, uint32_t n_local, uint64_t count,
                                    uint64_t ccl_bytes, int dtype);
/* The ring (level0_mesh 0) or mesh (1) reduce-scatter executor over n_servers x n_local ranks in op-base mode: alg1
 * (in-place ring, NHR or NB reduce-scatter) between the servers first, then the level-0 reduce-scatter inside. */
int hg_schedule_hier_rs(HgOpList* l, int level0_mesh, int alg1, uint32_t n_servers, uint32_t n_local, uint64_t count,
                        uint64_t ccl_bytes, int dtype);
/* The double-ring reduce-scatter executor on one server in op-base mode with DMA reduce: user input read share by share,
 * the result folded straight into the user output. */
int hg_schedule_dbring_rs(HgOpList* l, uint32_t n, uint64_t count, uint64_t ccl_bytes, int dtype);
int hg_schedule_dbring_rs_servers(HgOpList* l, int alg1, int alg2, uint32_t n_pods, uint32_t n_servers, uint32_t n_local,
                                  uint64_t count, uint64_t ccl_bytes, int dtype);
/* Most elements per rank any schedule accepts: every byte offset a schedule derives from a count (count x unit x
 * ranks, rounded up to slot sizes) then stays far inside 64 bits.  Larger counts are refused with HCCL_E_PARA. */
#define HG_MAX_COUNT ((uint64_t)1 << 48)
void hg_oplist_free(HgOpList* l);
/* 1 when the deterministic mesh allreduce's folds leave every rank's slice where its gather reads it (n a power of two, or 3). */
int hg_local_reduce_lands(uint32_t n);
/* Per-rank communication-buffer bytes alg needs (0 when it stages nothing). */
uint64_t hg_scratch_bytes(int alg, uint32_t n, uint64_t count, int dtype);

#endif
