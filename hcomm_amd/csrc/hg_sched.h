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
} HgOpList;

/* Fill `l` with the op list of `alg`; the caller releases it with hg_oplist_free. */
int hg_schedule(HgOpList* l, int alg, uint32_t n, uint64_t count, int dtype);
void hg_oplist_free(HgOpList* l);

#endif
