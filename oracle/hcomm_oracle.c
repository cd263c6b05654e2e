/*
 * hcomm_oracle.c - CPU restatement of HCOMM's local copy / reduce semantics, of the ring, recursive
 * halving-doubling, mesh, NHR (sliced and one-shot), NB, local-reduce, chunk-mesh and doubling schedules, of the
 * executors' op-base loop around them, of the ring and mesh executors' three-step allreduce and two-level
 * reduce-scatter, of the double-ring executor with DMA reduce and of the order-preserving reduce-scatter and allreduce
 * executors (the latter on one server and over two levels), used ONLY to check libhcomm_gfx.so.
 *
 * THIS IS TEST INFRASTRUCTURE.  Nothing in the product library links, loads or calls it; only the test
 * suite, the smoke check and the CPU-baseline leg of the benchmark do.
 *
 * Every function cites the reference file:line it restates (paths relative to the reference tree; "tpl/"
 * abbreviates src/legacy/ascend910/algorithm/base/alg_template/).  The schedules are written the way the
 * reference writes them - one program per rank, with the running slice indices of the original loops -
 * and then executed in lock step, which is deliberately a different formulation from the closed-form,
 * step-major generator inside the product.
 *
 * Pinning status (what fixes each function besides its own formula; see tests/test_oracle_*.py):
 *   integer SUM/PROD/MAX/MIN ........ exhaustive int8 pairs + numpy wrap-around arithmetic; pinned
 *   fp32 ops ........................ one IEEE-754 operation, checked against numpy float32; pinned
 *   fp16 conversions and ops ........ exhaustive against numpy float16 and against the reference's own
 *                                     FP16 class compiled from its sources (oracle/_ref); pinned
 *   int8/16/32, fp16, fp32 loops .... against the reference's MemReduceSum/Min/Max compiled from its
 *                                     sources (oracle/_ref); pinned
 *   bf16 conversions and ops ........ PARITY UNPINNED against the reference: it has no bf16 arithmetic on
 *                                     any CPU path (hccl_task_reduce_process.cc:57-84 has no BFP16 case).
 *                                     Defined by analogy with fp16 (fp32 operation + round to nearest even)
 *                                     and checked against torch.bfloat16 only.
 *   NaN payloads, int overflow ...... of the real SDMA / vector engines: PARITY UNPINNED (hardware
 *                                     behaviour outside the reference tree); integers wrap as in the
 *                                     reference's CPU witnesses.
 *   slice tables .................... the reference's hand-computable values for the benchmark configs +
 *                                     invariants; pinned
 *   schedules ....................... hand-derived step chains for N = 4 (tests/golden), the reference's
 *                                     own acceptance rule (every output range receives every rank exactly
 *                                     once, allreduce_semantics_checker.cc:59-96), non-associative fp
 *                                     inputs, and agreement with the product's independent generator; pinned
 *   ring, RHD, mesh (both orders) ... hand-derived receive tables and expression trees, N = 2, 3, 4, 6; pinned
 *   local-reduce allreduce, chunk
 *   mesh ............................ hand-derived fold trees / fold orders, N = 2, 4; pinned
 *   NHR ............................. slice maps N = 3..12, merged receive runs N = 5, fold trees N = 3..6, all
 *                                     by hand; bit reversal for powers of two; pinned
 *   NB .............................. slice tables, gather order N = 6, fold trees N = 3, 4, 5 by hand; pinned
 *   local-reduce reduce-scatter ..... window / slot layout and fold trees N = 3..6 by hand; pinned
 *   recursive doubling .............. per-rank trees and final input contents N = 2, 4, 8 by hand; pinned
 *   op-base loop .................... chunk tables (offsets, sizes, per-slice copies, single-copy case) and
 *                                     maxCountPerLoop values by hand; exact integer results; pinned
 *   one-shot NHR .................... binomial-tree receive tables, output tree and final input contents
 *                                     N = 2, 3, 5, 6, 8 by hand; pinned
 *   three-step allreduce ............ the complete operation list of 2 servers x 2 ranks and the reduction trees
 *                                     of 2 x 3 by hand; the one-shot threshold; exact integer results; pinned
 *   mesh level 0 of the three steps . stream pieces of a ragged segment for 3 and 7 streams, one rank's operation
 *                                     list and the trees of all 12 pieces N = 4 by hand; pinned
 *   double-ring allreduce ........... slice / ring-order tables N = 4, one rank's complete operation list N = 3, the
 *                                     reduction trees of both shares N = 4, all by hand; exact integer results over
 *                                     several chunks; pinned
 *   two-level reduce-scatter ........ the complete operation list and the reduction trees of 2 x 2, the trees of the
 *                                     mesh pieces of 1 x 4, the recursive halving-doubling trees between 3 and 6
 *                                     servers, a chunk table, by hand; exact integer results; pinned
 *   double-ring reduce-scatter ...... one rank's complete operation list N = 3, the trees of both shares N = 4 and a
 *                                     chunk / share table by hand; exact integer results over several chunks; pinned
 *   order-preserving reduce-scatter . the complete operation list N = 3, the rank-order fold trees N = 2..8 and a
 *                                     chunk table by hand; exact integer results over several chunks; pinned
 *   order-preserving small-message branch . the complete operation list N = 4 by hand; per-rank trees N = 4, 8 (the
 *                                     rank-order tree, leaves XOR p); exact integer results; pinned
 *   order-preserving allreduce ...... the complete operation list N = 3 (blocks of 256, 144 and 0 bytes, both borrowed
 *                                     slots), a chunk / block table N = 4 by hand; the same rank-order fold trees for
 *                                     every element N = 2..8; slot and borrowed-slot layout from the definition;
 *                                     exact integer results over several chunks; pinned
 *   two-level order-preserving allreduce . the complete operation lists of 2 x 2 (every borrowed place of both levels)
 *                                     and of 3 x 1 (one device per module) by hand; reduction trees 2 x 2 .. 3 x 3 composed by hand from the single-level
 *                                     trees; slot / borrowed-place layout of both levels from the definition; exact
 *                                     integer results over several chunks, ring / NB / NHR all-gather; pinned
 *   two-level order-preserving reduce-scatter . the complete operation lists of 2 x 2 and 3 x 1 by hand; the composed reduction
 *                                     trees per block; layout from the definition; exact integer results; pinned
 *   (every schedule additionally passes the symbolic checker for N = 1..17, 24, 31, 32)
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_MAX_RANKS 32

enum { ORC_SUM = 0, ORC_PROD = 1, ORC_MAX = 2, ORC_MIN = 3 };
enum { ORC_I8 = 0, ORC_I16 = 1, ORC_I32 = 2, ORC_F16 = 3, ORC_F32 = 4, ORC_BF16 = 11 };

static int g_threads = 1;

void orc_set_threads(int n) { g_threads = n > 0 ? n : 1; }
int orc_get_threads(void) { return g_threads; }

/* ---- 16-bit float conversions --------------------------------------------------------------------- */

static uint32_t f2u(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}
static float u2f(uint32_t u)
{
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* binary16 -> binary32, exact (restates half_to_float, ccu_fp16.h:102-111) */
float orc_f16_to_f32(uint16_t h)
{
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1fu, m = h & 0x3ffu;
    if (e == 0x1f) return u2f(sign | 0x7f800000u | (m << 13)); /* inf / NaN */
    if (e == 0) {
        if (m == 0) return u2f(sign);
        /* subnormal: renormalise */
        int shift = 0;
        while (!(m & 0x400u)) {
            m <<= 1;
            ++shift;
        }
        m &= 0x3ffu;
        e = (uint32_t)(1 - shift);
        return u2f(sign | ((e + 112u) << 23) | (m << 13));
    }
    return u2f(sign | ((e + 112u) << 23) | (m << 13));
}

/* binary32 -> binary16, round to nearest even; NaN -> sign | 0x7e00 (restates float_to_half, ccu_fp16.h:114-135) */
uint16_t orc_f32_to_f16(float f)
{
    const uint32_t x = f2u(f);
    const uint32_t sign = (x >> 16) & 0x8000u, ax = x & 0x7fffffffu;
    if (ax > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);
    if (ax >= 0x47800000u) return (uint16_t)(sign | 0x7c00u); /* >= 65536 or inf */
    const int32_t e = (int32_t)(ax >> 23) - 127 + 15;
    uint32_t m = ax & 0x7fffffu;
    if (e <= 0) {
        if (e < -10) return (uint16_t)sign; /* below half of the smallest subnormal */
        m |= 0x800000u;
        const uint32_t shift = (uint32_t)(14 - e);
        uint32_t hm = m >> shift;
        const uint32_t rem = m & ((1u << shift) - 1u), halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (hm & 1u))) ++hm;
        return (uint16_t)(sign | hm);
    }
    uint32_t hv = ((uint32_t)e << 10) | (m >> 13);
    const uint32_t rem = m & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (hv & 1u))) ++hv; /* a carry into the exponent is the right answer */
    return (uint16_t)(sign | hv);
}

/* bfloat16: the upper half of a binary32.  No reference witness; by analogy with fp16. */
float orc_bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

uint16_t orc_f32_to_bf16(float f)
{
    const uint32_t x = f2u(f);
    if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)(((x >> 16) & 0x8000u) | 0x7fc0u);
    return (uint16_t)((x + 0x7fffu + ((x >> 16) & 1u)) >> 16);
}

/* ---- element operation: returns d (op) s with d in the dst role ------------------------------------------
 * SUM a+b, PROD a*b (reduce_op, test/ut/stub/llt_hccl_stub.cc:4077-4101; AicpuReduceTemplate,
 * src/legacy/ascend950/service/collective/instruction/instruction.cc:472-493);
 * MAX (src > dst) ? src : dst, MIN (src < dst) ? src : dst - the stub is called with src1 = src, src2 = dst
 * (llt_hccl_stub.cc:2374), and MemReduceMax/MinTemplate overwrite dst only when the comparison holds
 * (test/hccl_vm/src/plugin/runner/runner_utils/hccl_task_reduce_process.cc:30-55), so dst survives ties
 * and unordered comparisons.  Integers wrap (native C++ arithmetic on the typed value in both witnesses). */

#define INT_OP(T, U)                                                  \
    static T op_##T(T d, T s, int op)                                 \
    {                                                                 \
        switch (op) {                                                 \
            case ORC_SUM: return (T)(U)((U)d + (U)s);                 \
            case ORC_PROD: return (T)(U)((U)d * (U)s);                \
            case ORC_MAX: return (s > d) ? s : d;                     \
            default: return (s < d) ? s : d;                          \
        }                                                             \
    }
INT_OP(int8_t, uint8_t)
INT_OP(int16_t, uint16_t)
INT_OP(int32_t, uint32_t)

static float op_f32(float d, float s, int op)
{
    switch (op) {
        case ORC_SUM: return d + s;
        case ORC_PROD: return d * s;
        case ORC_MAX: return (s > d) ? s : d;
        default: return (s < d) ? s : d;
    }
}

/* fp16: widen both, operate in fp32, round back (FP16::operator+=, ccu_fp16.h:60-66); MAX/MIN compare the
 * widened values and move the raw 16 bits (FP16::operator>, :69-74 with MemReduceMaxTemplate) */
static uint16_t op_f16(uint16_t d, uint16_t s, int op)
{
    const float fd = orc_f16_to_f32(d), fs = orc_f16_to_f32(s);
    switch (op) {
        case ORC_SUM: return orc_f32_to_f16(fd + fs);
        case ORC_PROD: return orc_f32_to_f16(fd * fs);
        case ORC_MAX: return (fs > fd) ? s : d;
        default: return (fs < fd) ? s : d;
    }
}

static uint16_t op_bf16(uint16_t d, uint16_t s, int op)
{
    const float fd = orc_bf16_to_f32(d), fs = orc_bf16_to_f32(s);
    switch (op) {
        case ORC_SUM: return orc_f32_to_bf16(fd + fs);
        case ORC_PROD: return orc_f32_to_bf16(fd * fs);
        case ORC_MAX: return (fs > fd) ? s : d;
        default: return (fs < fd) ? s : d;
    }
}

uint32_t orc_dtype_size(int dtype)
{
    /* SIZE_TABLE, pkg_inc/legacy/hccl/dtype_common.h:18-36 */
    static const uint32_t table[18] = {1, 2, 4, 2, 4, 8, 8, 1, 2, 4, 8, 2, 16, 2, 1, 1, 1, 1};
    return (dtype >= 0 && dtype < 18) ? table[dtype] : 0;
}

/* dst[i] = dst[i] (op) src[i], i < count (HcommLocalReduceOnThread, include/hcomm_primitives.h:164-165;
 * loop shape of vector_reduce, llt_hccl_stub.cc:4159-4201).  Returns 0, or -1 for an unsupported type. */
int orc_reduce(void* dst, const void* src, uint64_t count, int dtype, int op)
{
    if (op < ORC_SUM || op > ORC_MIN) return -1;
    const int nt = (count >= (1u << 16)) ? g_threads : 1;
    (void)nt;
    int64_t i;
    const int64_t n = (int64_t)count;
    switch (dtype) {
        case ORC_I8: {
            int8_t* d = (int8_t*)dst;
            const int8_t* s = (const int8_t*)src;
#pragma omp parallel for num_threads(nt) schedule(static)
            for (i = 0; i < n; ++i) d[i] = op_int8_t(d[i], s[i], op);
            return 0;
        }
        case ORC_I16: {
            int16_t* d = (int16_t*)dst;
            const int16_t* s = (const int16_t*)src;
#pragma omp parallel for num_threads(nt) schedule(static)
            for (i = 0; i < n; ++i) d[i] = op_int16_t(d[i], s[i], op);
            return 0;
        }
        case ORC_I32: {
            int32_t* d = (int32_t*)dst;
            const int32_t* s = (const int32_t*)src;
#pragma omp parallel for num_threads(nt) schedule(static)
            for (i = 0; i < n; ++i) d[i] = op_int32_t(d[i], s[i], op);
            return 0;
        }
        case ORC_F32: {
            float* d = (float*)dst;
            const float* s = (const float*)src;
#pragma omp parallel for num_threads(nt) schedule(static)
            for (i = 0; i < n; ++i) d[i] = op_f32(d[i], s[i], op);
            return 0;
        }
        case ORC_F16: {
            uint16_t* d = (uint16_t*)dst;
            const uint16_t* s = (const uint16_t*)src;
#pragma omp parallel for num_threads(nt) schedule(static)
            for (i = 0; i < n; ++i) d[i] = op_f16(d[i], s[i], op);
            return 0;
        }
        case ORC_BF16: {
            uint16_t* d = (uint16_t*)dst;
            const uint16_t* s = (const uint16_t*)src;
#pragma omp parallel for num_threads(nt) schedule(static)
            for (i = 0; i < n; ++i) d[i] = op_bf16(d[i], s[i], op);
            return 0;
        }
        default: return -1;
    }
}

/* dst[0..len) = src[0..len); nothing when len == 0 or src == dst (HcommLocalCopyOnThread,
 * include/hcomm_primitives.h:152; src/legacy/ascend910/platform/task/dispatcher.cc:495-498) */
void orc_copy(void* dst, const void* src, uint64_t len)
{
    if (len == 0 || dst == src) return;
    const int nt = (len >= (1u << 20)) ? g_threads : 1;
    if (nt == 1) {
        memmove(dst, src, len);
        return;
    }
    const uint64_t chunk = (len + (uint64_t)nt - 1) / (uint64_t)nt;
    int t;
#pragma omp parallel for num_threads(nt) schedule(static)
    for (t = 0; t < nt; ++t) {
        const uint64_t b = (uint64_t)t * chunk;
        if (b < len) memcpy((char*)dst + b, (const char*)src + b, (len - b < chunk) ? len - b : chunk);
    }
}

/* ---- slice tables ----------------------------------------------------------------------------------- */

typedef struct {
    uint64_t offset, size;
} OrcSlice;

/* AllReduceRing::PrepareRunAsync, tpl/temp_all_reduce/all_reduce_ring.cc:142-153 (same arithmetic as
 * ExecutorBase::PrepareSliceData, tpl/alg_template_base.cc:787-820) */
void orc_slices_ring(uint64_t count, uint32_t unit, uint32_t n, OrcSlice* sl)
{
    const uint64_t total = count * unit;
    const uint64_t calc = (total + (n - 1)) / n;
    /* RoundUpWithDivisor(value, 128): value == 0 gives 128 (tpl/alg_template_base_pub.h:609-616) */
    const uint64_t aligned = (calc == 0) ? 128 : ((calc + 127) / 128) * 128;
    uint64_t residue = total;
    for (uint32_t i = 0; i < n; ++i) {
        sl[i].size = (residue > aligned) ? aligned : residue;
        sl[i].offset = total - residue;
        residue -= sl[i].size;
    }
}

/* RecursiveHalvingDoublingBase::CalculateSlices, tpl/recursive_halvingdoubling_base.cc:64-94 */
void orc_slices_rhd(uint64_t data_bytes, uint32_t block, OrcSlice* sl)
{
    uint64_t per = data_bytes / block;
    if (data_bytes % block != 0) per++;
    per = ((per + 127) / 128) * 128;
    uint64_t left = data_bytes;
    uint32_t i = 0;
    while (left > 0) {
        sl[i].size = per < left ? per : left;
        sl[i].offset = data_bytes - left;
        left -= sl[i].size;
        i++;
    }
    while (i < block) {
        sl[i].offset = data_bytes;
        sl[i].size = 0;
        i++;
    }
}

/* ---- schedules as per-rank programs ------------------------------------------------------------------ */

typedef struct {
    uint32_t step;
    uint32_t kind; /* 0 copy, 1 reduce */
    uint32_t rank;
    uint32_t dst_buf; /* 0 in, 1 out */
    uint32_t src_rank;
    uint32_t src_buf;
    uint64_t dst_off, src_off, bytes;
} OrcOp;

typedef struct {
    OrcOp* ops;
    uint64_t n, cap;
    int oom;
} OrcTrace;

static uint32_t g_step_base = 0; /* added to every emitted step: where the current chunk of an op-base loop starts */
/* A template running on a sub-communicator: its ranks are positions in g_rank_map, and it addresses the rank buffers
 * baseOffset_ bytes in (tpl/alg_template_base.cc:53-54). */
#define B_OUT_ROLE 1u /* roles 0 and 1: the template's input and output memory */
static const uint32_t* g_rank_map = NULL;
static uint64_t g_base_off = 0;
static uint64_t g_user_off = 0; /* where the current chunk of an op-base loop starts in the user buffers (roles 3, 4) */

static void emit(OrcTrace* t, uint32_t step, uint32_t kind, uint32_t rank, uint32_t dst_buf, uint64_t dst_off,
                 uint32_t src_rank, uint32_t src_buf, uint64_t src_off, uint64_t bytes)
{
    if (bytes == 0) return; /* a zero-length task does nothing (dispatcher.cc:495-498, 719-722) */
    if (t->n == t->cap) {
        uint64_t cap = t->cap ? t->cap * 2 : 256;
        OrcOp* p = (OrcOp*)realloc(t->ops, cap * sizeof(OrcOp));
        if (!p) {
            t->oom = 1;
            return;
        }
        t->ops = p;
        t->cap = cap;
    }
    OrcOp* o = &t->ops[t->n++];
    o->step = g_step_base + step;
    o->kind = kind;
    o->rank = g_rank_map ? g_rank_map[rank] : rank;
    o->dst_buf = dst_buf;
    o->src_rank = g_rank_map ? g_rank_map[src_rank] : src_rank;
    o->src_buf = src_buf;
    o->dst_off = dst_off + (dst_buf <= B_OUT_ROLE ? g_base_off : (dst_buf >= 3u ? g_user_off : 0));
    o->src_off = src_off + (src_buf <= B_OUT_ROLE ? g_base_off : (src_buf >= 3u ? g_user_off : 0));
    o->bytes = bytes;
}

enum { B_IN = 0, B_OUT = 1, B_SCR = 2, B_UIN = 3, B_UOUT = 4, K_COPY = 0, K_REDUCE = 1 };

/* ReduceScatterRing::RunReduceScatter for one rank, tpl/temp_reduce_scatter/reduce_scatter_ring.cc:182-312.
 * `out_sl` NULL: the allreduce case, where the template's output memory IS the input memory
 * (all_reduce_ring.cc:186-187) so the last step reduces in place; otherwise the stand-alone case, where
 * the inline-reduce branch reduces into the input slice and then copies it to the output
 * (tpl/component/reducer.cc:199-218). */
static void prog_ring_rs(OrcTrace* t, uint32_t rank, uint32_t n, const OrcSlice* sl, const OrcSlice* out_sl)
{
    const uint32_t left = (rank + n - 1) % n;        /* ringPrevRank, :121 */
    uint32_t rx = (rank + n - 2) % n;                /* rxSliceIndex, :207 */
    uint32_t step = 0;
    for (uint32_t i = 0; i < n - 2; i++) {           /* :232 */
        emit(t, step++, K_REDUCE, rank, B_IN, sl[rx].offset, left, B_IN, sl[rx].offset, sl[rx].size); /* :245, RunVectorDestRducer :44-62 */
        rx = (rx + n - 1) % n;                       /* :260 */
    }
    /* final receive: slice index == rank, :288-304 */
    emit(t, step++, K_REDUCE, rank, B_IN, sl[rank].offset, left, B_IN, sl[rank].offset, sl[rank].size);
    if (out_sl) emit(t, step, K_COPY, rank, B_OUT, out_sl[rank].offset, rank, B_IN, sl[rank].offset, sl[rank].size);
}

/* AllGatherRing::RunAsync + RunAllGather for one rank, tpl/temp_all_gather/all_gather_ring.cc:116-121,143-206 */
static void prog_ring_ag_ex(OrcTrace* t, uint32_t rank, uint32_t n, const OrcSlice* sl, uint32_t step, int two_buffers)
{
    const uint32_t left = (rank + n - 1) % n;
    if (two_buffers) /* inputMem_ != outputMem_, :117 */
        emit(t, step++, K_COPY, rank, B_OUT, sl[rank].offset, rank, B_IN, sl[rank].offset, sl[rank].size); /* :116-121 */
    uint32_t rx = (rank + n - 1) % n; /* ForwordRank(rank, n, 1), :152 */
    for (uint32_t i = 0; i < n - 1; i++) {
        emit(t, step++, K_COPY, rank, B_OUT, sl[rx].offset, left, B_OUT, sl[rx].offset, sl[rx].size); /* RxVector :34-45 */
        rx = (rx + n - 1) % n; /* :196 */
    }
}

static void prog_ring_ag(OrcTrace* t, uint32_t rank, uint32_t n, const OrcSlice* sl, uint32_t step)
{
    prog_ring_ag_ex(t, rank, n, sl, step, 1);
}

static void prog_allreduce_ring(OrcTrace* t, uint32_t rank, uint32_t n, uint64_t count, uint32_t unit, int gather)
{
    if (n == 1) { /* all_reduce_ring.cc:132-140; staged reduce-scatter: nothing (:73-76) */
        if (gather) emit(t, 0, K_COPY, 0, B_OUT, 0, 0, B_IN, 0, count * unit);
        return;
    }
    OrcSlice sl[ORC_MAX_RANKS];
    orc_slices_ring(count, unit, n, sl);
    prog_ring_rs(t, rank, n, sl, NULL);
    if (gather) prog_ring_ag(t, rank, n, sl, n - 1);
}

static void prog_rs_ring_standalone(OrcTrace* t, uint32_t rank, uint32_t n, uint64_t count, uint64_t stride, uint32_t unit)
{
    const uint64_t sz = count * unit;
    if (n == 1) { /* reduce_scatter_ring.cc:103-109 */
        emit(t, 0, K_COPY, 0, B_OUT, 0, 0, B_IN, 0, sz);
        return;
    }
    OrcSlice sl[ORC_MAX_RANKS], osl[ORC_MAX_RANKS];
    /* :140-157 (input larger than output -> output offset 0), with the strided input layout of the MC2 path:
     * displs[i] = strideLen * i * unitSize (src/legacy/ascend910/framework/device/aicpu_kfc/algorithm/
     * aicpu_reduce_scatter.cc:78-80); stride == count is the dense default */
    for (uint32_t i = 0; i < n; i++) {
        sl[i].size = sz;
        sl[i].offset = (uint64_t)i * stride * unit;
        osl[i].size = sz;
        osl[i].offset = 0;
    }
    prog_ring_rs(t, rank, n, sl, osl);
}

/* AllReduceRecursiveHalvingDoubling for one rank, tpl/temp_all_reduce/all_reduce_recursive_hd.cc:28-50 */
static void prog_allreduce_rhd(OrcTrace* t, uint32_t rank, uint32_t n, uint64_t count, uint32_t unit)
{
    const uint64_t total = count * unit;
    if (n == 1) { /* :103-108 */
        emit(t, 0, K_COPY, 0, B_OUT, 0, 0, B_IN, 0, total);
        return;
    }
    /* CalcPartOneSizeAndBlockSize, tpl/recursive_halvingdoubling_base.cc:23-37 */
    uint32_t round = 0;
    while ((1u << round) <= n) round++;
    if (round >= 1) round -= 1;
    const uint32_t block = 1u << round;
    const uint32_t part1 = (n - block) * 2;
    OrcSlice sl[ORC_MAX_RANKS];
    orc_slices_rhd(total, block, sl);

    uint32_t step = 0;
    /* ReduceInPartOne, :133-203: even ranks of part one reduce the odd neighbour's whole input into theirs */
    if (part1 > 0) {
        if (rank < part1 && rank % 2 == 0) emit(t, step, K_REDUCE, rank, B_IN, 0, rank + 1, B_IN, 0, total);
        step++;
    }
    const int idle = (rank < part1 && rank % 2 == 1); /* :208-210, :243-245 */
    uint32_t rib = 0;                                 /* rankInBlock */
    if (!idle) rib = (rank < part1) ? rank / 2 : rank - part1 / 2;
    /* block rank -> real rank: inverse of BuildSubLinks, tpl/recursive_halvingdoubling_base.cc:39-62 */
#define REAL(b) (((b) < part1 / 2) ? 2 * (b) : (b) + part1 / 2)
    uint32_t steps = 0; /* GetBlockStep / Log2 */
    while ((block >> (steps + 1)) != 0) steps++;

    /* ReduceScatterHalvingDoubling, tpl/temp_reduce_scatter/reduce_scatter_halving_doubling.cc:65-92,196-257 */
    uint32_t last_rx = 0;
    for (uint32_t s = 0; s < steps; s++) {
        if (!idle) {
            const uint32_t mask = 1u << (steps - s - 1); /* halvingBitmask :72 */
            const uint32_t peer = rib ^ mask;
            const uint32_t id = rib & (~(mask - 1)); /* rx slice id :76-77 */
            uint64_t sz = 0;
            uint32_t num = mask; /* Sum(), tpl/alg_template_base.cc:1079-1096 */
            while (num > 0) {
                num--;
                sz += sl[id + num].size;
            }
            emit(t, step, K_REDUCE, rank, B_IN, sl[id].offset, REAL(peer), B_IN, sl[id].offset, sz);
            last_rx = id;
        }
        step++;
    }
    /* :251-254 copy of the last received range (one slice) input -> output */
    if (!idle) emit(t, step, K_COPY, rank, B_OUT, sl[last_rx].offset, rank, B_IN, sl[last_rx].offset, sl[last_rx].size);
    step++;
    /* AllGatherHalvingDoubling in the outputs, tpl/temp_all_gather/all_gather_halving_doubling.cc:42-66,164-206 */
    for (uint32_t s = 0; s < steps; s++) {
        if (!idle) {
            const uint32_t mask = 1u << s;
            const uint32_t peer = rib ^ mask;
            const uint32_t id = peer & (~(mask - 1)); /* rx: the peer's aligned group */
            uint64_t sz = 0;
            for (uint32_t k = 0; k < mask; k++) sz += sl[id + k].size;
            emit(t, step, K_COPY, rank, B_OUT, sl[id].offset, REAL(peer), B_OUT, sl[id].offset, sz);
        }
        step++;
    }
    /* GatherInPartOne, :277-343: odd ranks of part one receive the even neighbour's whole output */
    if (part1 > 0) {
        if (rank < part1 && rank % 2 == 1) emit(t, step, K_COPY, rank, B_OUT, 0, rank - 1, B_OUT, 0, total);
        step++;
    }
#undef REAL
}

/* AllReduceMeshDirectOneshot::RunAllReduceOne, tpl/temp_all_reduce/all_reduce_mesh_oneshot.cc:78-121.  The
 * remote buffer read at :108-115 is the peer's communication buffer, filled with the peer's input at :96-100;
 * with two buffers per rank that is in[peer]. */
static void prog_allreduce_mesh_oneshot(OrcTrace* t, uint32_t rank, uint32_t n, uint64_t count, uint32_t unit)
{
    const uint64_t total = count * unit;
    emit(t, 0, K_COPY, rank, B_OUT, 0, rank, B_IN, 0, total); /* :92-94 (also the n == 1 path, :53-62) */
    for (uint32_t round = 1; round < n; round++) {
        const uint32_t peer = (round + rank) % n; /* :103 */
        emit(t, round, K_REDUCE, rank, B_OUT, 0, peer, B_IN, 0, total);
    }
}

/* InsTempAllReduceMesh1DOneShot::RunAllReduce, src/legacy/ascend950/service/collective/alg/coll_alg_factory/
 * alg_template/ins_alg_template/ins_temp_all_reduce_mesh_1D_one_shot.cc:86-164: copy input to output (:102), gather
 * every peer's input into scratch slots (:105-141), then reduce the slots into the output in ascending rank
 * order, skipping the own rank (:148-161).  With two buffers per rank slot[peer] is read as in[peer]. */
static void prog_allreduce_mesh_ascending(OrcTrace* t, uint32_t rank, uint32_t n, uint64_t count, uint32_t unit)
{
    const uint64_t total = count * unit;
    emit(t, 0, K_COPY, rank, B_OUT, 0, rank, B_IN, 0, total);
    uint32_t step = 1;
    for (uint32_t cur = 0; cur < n; cur++) {
        if (cur == rank) continue;
        emit(t, step++, K_REDUCE, rank, B_OUT, 0, cur, B_IN, 0, total);
    }
}

/* ReduceScatterMesh, tpl/temp_reduce_scatter/reduce_scatter_mesh.cc:51-128 (stream index 0), :131-215; the
 * input slice of rank i starts at i * stride elements (aicpu_reduce_scatter.cc:78-80), stride == count by default */
static void prog_rs_mesh(OrcTrace* t, uint32_t rank, uint32_t n, uint64_t count, uint64_t stride, uint32_t unit)
{
    const uint64_t sz = count * unit;
    if (n == 1) { /* :152-157 */
        emit(t, 0, K_COPY, 0, B_OUT, 0, 0, B_IN, 0, sz);
        return;
    }
    uint32_t step = 0;
    for (uint32_t round = 1; round < n; round++) {
        const uint32_t src = (rank + n - round) % n; /* ForwardRank, tpl/../inc/reduce_scatter_mesh_pub.h:31-37 */
        /* RunDestRducer :35-49: dst = own input slice `rank`, remote offset = same slice */
        emit(t, step++, K_REDUCE, rank, B_IN, (uint64_t)rank * stride * unit, src, B_IN, (uint64_t)rank * stride * unit, sz);
    }
    emit(t, step, K_COPY, rank, B_OUT, 0, rank, B_IN, (uint64_t)rank * stride * unit, sz); /* :199-211 */
}

/* AllReduceLocalReduce for one rank, tpl/temp_all_reduce/all_reduce_local_reduce.cc:139-436 - the deterministic
 * mesh allreduce.  Three buffers per rank: user input (B_IN), the communication buffer commMemOut (B_SCR) and
 * user output (B_OUT).  An op is recorded under the rank that OWNS the destination; the rank that issues it is
 * the src rank.  Rounds that the reference runs concurrently on sub-streams get one step each.
 * RunLocalReduce leaves rank d's result in slot `center` of the block of 2^floor(log2(n-1)) slots it halves (:328-331),
 * the gather reads slot d, or n - 2 for the last rank (:419 with the last rank's window one slot up, :102-110).  The two
 * agree for every rank only when n is a power of two or 3 (local_reduce_lands; tests/test_local_reduce_any_n.py replays
 * the statements for the other counts and finds the gather reading a partial sum), so other counts are refused -
 * unless as_written is set, which emits the statements as they stand for that test. */
static int local_reduce_lands(uint32_t n)
{
    uint32_t power = 0;
    while ((2u << power) <= n - 1) power++;
    const uint32_t rank_power = 1u << power;
    for (uint32_t d = 0; d < n; ++d) {
        uint32_t center = d < rank_power ? d : d - rank_power + 1; /* :328-329 */
        if (center > rank_power - 1) center = rank_power - 1;
        const uint32_t block = d < rank_power ? 0 : n - rank_power - 1; /* :330 */
        const uint32_t read = d == n - 1 ? n - 2 : d;                   /* :419 */
        if (block + center != read) return 0;
    }
    return 1;
}

static int prog_allreduce_local_reduce(OrcTrace* t, uint32_t rank, uint32_t n, uint64_t count, uint32_t unit, int as_written)
{
    const uint64_t total = count * unit;
    if (n == 1) { /* :154-163 */
        emit(t, 0, K_COPY, 0, B_OUT, 0, 0, B_IN, 0, total);
        return 0;
    }
    if (!as_written && !local_reduce_lands(n)) return -1;
    /* PrepareSlice :69-120; the communication buffer is not the user output, so sizeLimit = totalSize (:84-88) */
    OrcSlice sl[ORC_MAX_RANKS], start[ORC_MAX_RANKS];
    const uint64_t ori = (total + n - 1) / n;
#define ROUNDUP(v, d) (((v) == 0) ? (uint64_t)(d) : ((((v) + (d) - 1) / (d)) * (d))) /* RoundUpWithDivisor */
    uint64_t per = ROUNDUP(ori, 16384);                              /* HCCL_MIN_SLICE_ALIGN_910B */
    if (per * (n - 1) > total) per = ROUNDUP(ori, 512);              /* HCCL_MIN_SLICE_ALIGN_ONCHIP */
    if (per * (n - 1) > total) per = ROUNDUP(ori, unit);
#undef ROUNDUP
    uint64_t residue = total;
    uint32_t i = 0;
    while (residue > 0) {
        const uint64_t sz = per < residue ? per : residue;
        sl[i].size = sz;
        sl[i].offset = total - residue;
        i++;
        residue -= sz;
        start[i - 1].size = per;
        start[i - 1].offset = (i != n) ? 0 : per; /* :102-110: the last rank's window starts one slot later */
    }
    while (i < n) {
        sl[i].size = 0;
        sl[i].offset = total;
        start[i].size = 0;
        start[i].offset = 0;
        i++;
    }
    uint32_t step = 0;
    /* RunReduceScatter :197-199: own slice, user input -> communication buffer at its natural offset */
    emit(t, step++, K_COPY, rank, B_SCR, sl[rank].offset, rank, B_IN, sl[rank].offset, sl[rank].size);
    for (uint32_t round = 1; round < n; round++) { /* :222-266 */
        const uint32_t dst_rank = (rank + round) % n;
        uint32_t dst_slice = (dst_rank + round) % (n - 1);
        if (dst_rank == n - 1) dst_slice = (dst_slice + n - 1 - 1) % (n - 1);
        if (round == n - 1) {
            dst_slice = (dst_rank == n - 1) ? (dst_rank - 1) : dst_rank; /* :233 */
            emit(t, step++, K_REDUCE, dst_rank, B_SCR, start[dst_rank].offset + dst_slice * start[dst_rank].size, rank,
                 B_IN, sl[dst_rank].offset, sl[dst_rank].size);
        } else {
            emit(t, step++, K_COPY, dst_rank, B_SCR, start[dst_rank].offset + dst_slice * start[dst_rank].size, rank,
                 B_IN, sl[dst_rank].offset, sl[dst_rank].size);
        }
    }
    /* RunLocalReduce :301-364 */
    uint32_t power = 0;
    while ((2u << power) <= n - 1) power++; /* floor(log2(n - 1)) */
    const uint32_t rank_power = 1u << power;
    const uint64_t align = start[rank].size;
    const uint64_t size = sl[rank].size;
    for (uint32_t k = 0; k < n - rank_power - 1; ++k) { /* :311-327, all in one step */
        if (rank < rank_power)
            emit(t, step, K_REDUCE, rank, B_SCR, start[rank].offset + k * align, rank, B_SCR,
                 start[rank].offset + (rank_power + k) * align, size);
        else
            emit(t, step, K_REDUCE, rank, B_SCR, start[rank].offset + (rank_power + k) * align, rank, B_SCR,
                 start[rank].offset + k * align, size);
    }
    step++;
    uint32_t center = rank < rank_power ? rank : (rank - rank_power + 1);
    if (center > rank_power - 1) center = rank_power - 1;
    uint64_t offset = rank < rank_power ? 0 : ((n - rank_power - 1) * align);
    offset += start[rank].offset;
    for (uint32_t round = 0; round < power; round++) { /* :333-362 */
        const uint32_t slices_num = rank_power >> (round + 1);
        if (center < slices_num) {
            for (uint32_t k = 0; k < slices_num; ++k)
                emit(t, step, K_REDUCE, rank, B_SCR, offset + k * align, rank, B_SCR, offset + (slices_num + k) * align, size);
        } else {
            for (uint32_t k = 0; k < slices_num; ++k)
                emit(t, step, K_REDUCE, rank, B_SCR, offset + (slices_num + k) * align, rank, B_SCR, offset + k * align, size);
            offset = offset + slices_num * align;
            center -= slices_num;
        }
        step++;
    }
    /* RunAllGather :366-436 */
    emit(t, step++, K_COPY, rank, B_OUT, sl[rank].offset, rank, B_SCR, sl[rank].offset, sl[rank].size); /* :405-409 */
    for (uint32_t round = 1; round < n; round++) {
        const uint32_t peer = (rank + n - round) % n; /* BackwardRank, tpl/inc_all_reduce_deter/all_reduce_local_reduce_pub.h:44-50 */
        emit(t, step++, K_COPY, rank, B_OUT, sl[peer].offset, peer, B_SCR, (uint64_t)peer * sl[0].size, sl[peer].size); /* :419-423 */
    }
    return 0;
}

/* The AICPU deterministic reduce-scatter for one rank: AicpuReduceScatter::RunDeterministicReduceScatterLocal,
 * src/legacy/ascend910/framework/device/aicpu_kfc/algorithm/aicpu_reduce_scatter.cc:64-118, one pass of its loop (the
 * message fits the window: count * unit * n <= windowSize), with TaskOrchestrator's statements
 * (.../algorithm/task_orchestrator.cc): rank r copies slice r of its send buffer into slot r of its own window
 * (SelfCpySnd2Win :80-95 with winOffset = rankId * curSize), writes slice d into slot r of every peer d's window
 * (IpcCpySnd2Win :370-386, one window offset for all peers), folds its window in place (SelfLocalReduce :719-755: the
 * slots beyond the largest power of two onto the first ones in ONE reduce, then rounds of window[0, h) (op)= window[h, 2h),
 * each one reduce) and copies window[0, curSize) to its receive buffer (SelfCpyWin2Rcv :203-218).  Slice d of a send
 * buffer starts at strideLen * d * unit (displs, :78-80).  The window is B_SCR.  An op is recorded under the rank that
 * owns the destination. */
static void prog_rs_window_halving(OrcTrace* t, uint32_t rank, uint32_t n, uint64_t count, uint64_t stride, uint32_t unit)
{
    const uint64_t cur = count * unit;
    if (n == 1) { /* nothing to fold: the round trip through the window leaves the input slice in the receive buffer */
        emit(t, 0, K_COPY, 0, B_OUT, 0, 0, B_IN, 0, cur);
        return;
    }
    uint32_t step = 0;
    emit(t, step, K_COPY, rank, B_SCR, (uint64_t)rank * cur, rank, B_IN, stride * rank * unit, cur); /* 1. :102-104 */
    for (uint32_t index = 0; index < n; index++)                                                       /* 3. :109 */
        if (index != rank) emit(t, step, K_COPY, index, B_SCR, (uint64_t)rank * cur, rank, B_IN, stride * index * unit, cur);
    step++;
    uint32_t power = 0;
    while ((2u << power) <= n) power++; /* floor(log2(rankNum)), :730 */
    const uint32_t rank_power = 1u << power;
    if (rank_power < n) /* :732-740 */
        emit(t, step, K_REDUCE, rank, B_SCR, 0, rank, B_SCR, (uint64_t)rank_power * cur, (uint64_t)(n - rank_power) * cur);
    step++;
    for (uint32_t round = 0; round < power; round++) { /* :742-751 */
        const uint32_t slice_num = rank_power >> (round + 1);
        emit(t, step++, K_REDUCE, rank, B_SCR, 0, rank, B_SCR, (uint64_t)slice_num * cur, (uint64_t)slice_num * cur);
    }
    emit(t, step, K_COPY, rank, B_OUT, 0, rank, B_SCR, 0, cur); /* 6. :115 */
}

/* AllReduceChunkMesh for one rank, tpl/temp_all_reduce/all_reduce_chunk_mesh.cc:104-345, in the configuration
 * where the communication buffer (B_SCR) is not the user output (the "single operator" branches :186-193,
 * :239-243).  Slices: PrepareSlice :69-102 over n ranks, then each slice again over n-1 sub-chunks (:104-116). */
static void prog_allreduce_chunk_mesh(OrcTrace* t, uint32_t rank, uint32_t n, uint64_t count, uint32_t unit)
{
    const uint64_t total = count * unit;
    if (n == 1) { /* :137-146 */
        emit(t, 0, K_COPY, 0, B_OUT, 0, 0, B_IN, 0, total);
        return;
    }
    OrcSlice sl[ORC_MAX_RANKS], sub[ORC_MAX_RANKS];
    orc_slices_ring(count, unit, n, sl);                     /* same arithmetic as PrepareSlice :69-102 */
    orc_slices_ring(sl[rank].size / unit, unit, n - 1, sub); /* sliceMap[rank] :108-113 */
    uint32_t step = 0;
    emit(t, step++, K_COPY, rank, B_SCR, 0, rank, B_IN, 0, total); /* :188-193 whole input -> communication buffer */
    for (uint32_t round = 1; round < n; round++) {                 /* :213-253 */
        for (uint32_t peer = 1; peer < n; peer++) {
            const uint32_t gap = (peer + round) > n ? (peer + round - 1) % (n - 1) : (peer + round - 1); /* :235 */
            const uint32_t dst_rank = (gap + rank) % n;
            const uint32_t dst_slice = peer - 1;
            const uint64_t off = sl[rank].offset + sub[dst_slice].offset;
            emit(t, step, K_REDUCE, rank, B_SCR, off, dst_rank, B_SCR, off, sub[dst_slice].size); /* :245-252 */
        }
        step++;
    }
    emit(t, step++, K_COPY, rank, B_OUT, sl[rank].offset, rank, B_SCR, sl[rank].offset, sl[rank].size); /* :316-320 */
    for (uint32_t round = 1; round < n; round++) { /* :322-333 */
        const uint32_t peer = (rank + n - round) % n; /* BackwardRank, tpl/inc_all_reduce_deter/all_reduce_chunk_mesh_pub.h:45 */
        emit(t, step++, K_COPY, rank, B_OUT, sl[peer].offset, peer, B_SCR, sl[peer].offset, sl[peer].size);
    }
}

/* AllReduceDoubling::RunAllReduce for one rank, tpl/temp_all_reduce/all_reduce_doubling.cc:91-128 (n == 1: :38-41;
 * the power-of-two check is SimpleCheck's, :81-88).  The copy and the reduce of one round are separated by the
 * TxAck / RxAck exchange (:111-112), so they occupy two lock-step steps. */
static int prog_allreduce_doubling(OrcTrace* t, uint32_t rank, uint32_t n, uint64_t count, uint32_t unit)
{
    const uint64_t total = count * unit;
    if (n == 1) {
        emit(t, 0, K_COPY, 0, B_OUT, 0, 0, B_IN, 0, total);
        return 0;
    }
    if ((n & (n - 1)) != 0) return -1;
    uint32_t n_steps = 0;
    while ((1u << (n_steps + 1)) <= n) n_steps++; /* static_cast<u32>(log2(rankSize)), :97 */
    for (uint32_t step = 0; step < n_steps; step++) {
        const uint32_t neighbor = rank ^ (1u << step); /* :100 */
        if (step == 0) emit(t, 2 * step, K_COPY, rank, B_OUT, 0, rank, B_IN, 0, total);  /* :105-106 */
        else emit(t, 2 * step, K_COPY, rank, B_IN, 0, rank, B_OUT, 0, total);            /* :107-108 */
        emit(t, 2 * step + 1, K_REDUCE, rank, B_OUT, 0, neighbor, B_IN, 0, total);       /* :113-121 */
    }
    return 0;
}

/* ReduceNHROneshot::GetStepInfo, tpl/temp_reduce/reduce_nhr_oneshot.cc:195-227, root 0: whom this rank receives
 * from in the step (n = nobody). */
static uint32_t nhr_oneshot_reduce_from(uint32_t step, uint32_t rank, uint32_t n)
{
    uint32_t from = n;
    const uint32_t n_ranks = (n - 1 + (1u << step)) / (1u << (step + 1));
    const uint32_t delta_root = (rank + n - 0) % n;
    const uint32_t delta_pair = 1u << step, delta_group = 1u << (step + 1);
    if (delta_root / delta_group < n_ranks) {
        if (delta_root % delta_group == 0) from = (rank + delta_pair) % n;
    }
    return from;
}

/* BroadcastNHROneshot::GetStepInfo, tpl/temp_broadcast/broadcast_nhr_oneshot.cc:175-203, root 0 */
static uint32_t nhr_oneshot_bcast_from(uint32_t step, uint32_t n_steps, uint32_t rank, uint32_t n)
{
    uint32_t from = n;
    const uint32_t n_ranks = (n - 1 + (1u << (n_steps - 1 - step))) / (1u << (n_steps - step));
    const uint32_t delta_root = (rank + n - 0) % n;
    const uint32_t delta_pair = 1u << (n_steps - 1 - step), delta_group = 1u << (n_steps - step);
    if (delta_root / delta_group < n_ranks) {
        if ((delta_root + delta_pair) % delta_group == 0) from = (rank + n - delta_pair) % n;
    }
    return from;
}

static uint32_t nhr_steps(uint32_t n);

/* AllReduceNHROneshot::RunAsync for one rank, tpl/temp_all_reduce/all_reduce_nhr_oneshot.cc:26-69: the reduce to
 * rank 0 works on (input, input) with the inline-reduce receive of reduce_nhr_oneshot.cc:96-106 (the left
 * neighbour's input folded into the own input); the broadcast copies input -> output on the root
 * (broadcast_nhr_oneshot.cc:40-46) and then output -> output down the tree (:82-104). */
static void prog_allreduce_nhr_oneshot(OrcTrace* t, uint32_t rank, uint32_t n, uint64_t count, uint32_t unit)
{
    const uint64_t total = count * unit;
    if (n == 1) { /* :34-44 */
        emit(t, 0, K_COPY, 0, B_OUT, 0, 0, B_IN, 0, total);
        return;
    }
    const uint32_t n_steps = nhr_steps(n);
    for (uint32_t step = 0; step < n_steps; step++) {
        const uint32_t from = nhr_oneshot_reduce_from(step, rank, n);
        if (from != n) emit(t, step, K_REDUCE, rank, B_IN, 0, from, B_IN, 0, total);
    }
    if (rank == 0) emit(t, n_steps, K_COPY, rank, B_OUT, 0, rank, B_IN, 0, total);
    for (uint32_t step = 0; step < n_steps; step++) {
        const uint32_t from = nhr_oneshot_bcast_from(step, n_steps, rank, n);
        if (from != n) emit(t, n_steps + 1 + step, K_COPY, rank, B_OUT, 0, from, B_OUT, 0, total);
    }
}

/* ---- NHR and NB: per-rank programs --------------------------------------------------------------------- */

/* NHRBase::GetStepNumInterServer, tpl/nonuniform_hierarchical_ring_base.cc:139-147 = NBBase::CalcCeilLog2,
 * tpl/nonuniform_bruck_base.cc:19-25 */
static uint32_t nhr_steps(uint32_t n)
{
    uint32_t s = 0;
    for (uint32_t tmp = n - 1; tmp != 0; tmp >>= 1) s++;
    return s;
}

/* NHRBase::GetRankMapping + ReorderSequence, tpl/nonuniform_hierarchical_ring_base.cc:20-91 (the same loop is
 * ReduceScatterNHR::GetSliceMap + Reorder, tpl/temp_reduce_scatter/reduce_scatter_nhr.cc:97-162), with the
 * reference's tree / tmp arrays and its part loop. */
static void nhr_rank_mapping(uint32_t n, int keep_order, uint32_t* slice_map)
{
    uint32_t tree[ORC_MAX_RANKS], tmp[ORC_MAX_RANKS];
    for (uint32_t i = 0; i < n; i++) tree[i] = i;
    if (keep_order) { /* :27-31 */
        for (uint32_t i = 0; i < n; i++) slice_map[i] = tree[i];
        return;
    }
    const uint32_t n_steps = nhr_steps(n);
    uint32_t len = n;
    for (uint32_t step = 0; step < n_steps; step++) {
        const uint32_t n_slices = (n - 1 + (1u << step)) / (1u << (step + 1)); /* :40 */
        if (n_slices <= 1) break;
        int end_flag = 0;
        for (uint32_t part = 0; part * len < n; part++) {
            const uint32_t start = part * len;
            const uint32_t end = (start + len < n) ? start + len : n;
            for (uint32_t i = start; i < end; i++) { /* ReorderSequence, :79-91 */
                const uint32_t offset = i - start;
                if ((offset & 1) == 0) tmp[start + offset / 2] = tree[i];
                else tmp[start + (offset + len) / 2] = tree[i];
            }
            if (((end - start) & 1) == 1) end_flag = 1;
        }
        for (uint32_t i = 0; i < n; i++) tree[i] = tmp[i];
        if (end_flag) break;
        len >>= 1;
    }
    for (uint32_t i = 0; i < n; i++) slice_map[tree[i]] = i; /* :69-72 */
}

static int cmp_slices(const void* a, const void* b)
{
    const OrcSlice* x = (const OrcSlice*)a;
    const OrcSlice* y = (const OrcSlice*)b;
    if (x->offset != y->offset) return x->offset < y->offset ? -1 : 1;
    if (x->size != y->size) return x->size < y->size ? -1 : 1;
    return 0;
}

/* NHRBase::MergeSlices, tpl/nonuniform_hierarchical_ring_base.cc:94-136 */
static uint32_t nhr_merge_slices(OrcSlice* v, uint32_t m, int need_merge)
{
    if (!need_merge || m <= 1) return m;
    qsort(v, m, sizeof(OrcSlice), cmp_slices);
    uint32_t merged = 0;
    uint64_t off = v[0].offset, size = v[0].size;
    for (uint32_t i = 1; i < m; i++) {
        if (off + size == v[i].offset) {
            size += v[i].size;
        } else {
            v[merged].size = size;
            v[merged].offset = off;
            merged++;
            size = v[i].size;
            off = v[i].offset;
        }
    }
    v[merged].size = size;
    v[merged].offset = off;
    return merged + 1;
}

/* ReduceScatterNHR::RunReduceScatterNHR for one rank on the SDMA / inline-reduce path,
 * tpl/temp_reduce_scatter/reduce_scatter_nhr.cc:408-488 -> SdmaReducer :383-406 -> InlineReduceRx :222-237 /
 * InlineReduceRxLastStep :239-259 -> InlineReducer :197-220; step table GetStepInfo :552-593.
 * out_sl NULL: called from the allreduce, output memory == input memory, so the last step copies nothing. */
static void prog_nhr_rs(OrcTrace* t, uint32_t rank, uint32_t n, const OrcSlice* sl, const OrcSlice* out_sl,
                        const uint32_t* slice_map, int need_merge)
{
    const uint32_t n_steps = nhr_steps(n);
    for (uint32_t step = 0; step < n_steps; step++) {
        const uint32_t delta_rank = 1u << step;                       /* :562 */
        const uint32_t recv_from = (rank + delta_rank) % n;           /* :564 */
        const uint32_t n_slices = (n - 1 + (1u << step)) / (1u << (step + 1)); /* :567 */
        const uint32_t delta_slice = 1u << (step + 1);
        uint32_t rx_idx = rank;                                       /* :570 */
        uint32_t rx_idxs[ORC_MAX_RANKS];
        for (uint32_t i = 0; i < n_slices; i++) {
            rx_idxs[i] = slice_map[rx_idx];                           /* :577-578 */
            rx_idx = (rx_idx + n - delta_slice) % n;                  /* :586, u32 arithmetic as in the original */
        }
        if (step == n_steps - 1) { /* InlineReduceRxLastStep: per slice, unmerged */
            for (uint32_t i = 0; i < n_slices; i++) {
                const OrcSlice s = sl[rx_idxs[i]];
                emit(t, step, K_REDUCE, rank, B_IN, s.offset, recv_from, B_IN, s.offset, s.size); /* :203-207 */
                if (out_sl) /* localsrc != localdst, :208-217 */
                    emit(t, step + 1, K_COPY, rank, B_OUT, out_sl[rx_idxs[i]].offset, rank, B_IN, s.offset, s.size);
            }
        } else { /* GetRxSlices :357-381 + InlineReduceRx */
            OrcSlice rx[ORC_MAX_RANKS];
            for (uint32_t i = 0; i < n_slices; i++) rx[i] = sl[rx_idxs[i]];
            const uint32_t m = nhr_merge_slices(rx, n_slices, need_merge);
            for (uint32_t i = 0; i < m; i++)
                emit(t, step, K_REDUCE, rank, B_IN, rx[i].offset, recv_from, B_IN, rx[i].offset, rx[i].size);
        }
    }
}

/* AllGatherNHR::RunAllGather for one rank on the SDMA path, tpl/temp_all_gather/all_gather_nhr.cc:141-195 ->
 * SdmaRx :90-108; step table GetStepInfo :228-268 */
static void prog_nhr_ag(OrcTrace* t, uint32_t rank, uint32_t n, const OrcSlice* sl, const uint32_t* slice_map,
                        int need_merge, uint32_t step0)
{
    const uint32_t n_steps = nhr_steps(n);
    for (uint32_t step = 0; step < n_steps; step++) {
        const uint32_t delta_rank = 1u << (n_steps - 1 - step);                         /* :237 */
        const uint32_t recv_from = (rank + n - delta_rank) % n;                         /* :238 */
        const uint32_t n_slices = (n - 1 + (1u << (n_steps - 1 - step))) / (1u << (n_steps - step)); /* :242 */
        const uint32_t delta_slice = 1u << (n_steps - step);
        uint32_t rx_idx = (rank - (1u << (n_steps - 1 - step)) + n) % n;                /* :245 */
        OrcSlice rx[ORC_MAX_RANKS];
        for (uint32_t i = 0; i < n_slices; i++) {
            rx[i] = sl[slice_map[rx_idx]];
            rx_idx = (rx_idx + n - delta_slice) % n;                                    /* :265, u32 arithmetic */
        }
        const uint32_t m = nhr_merge_slices(rx, n_slices, need_merge);                  /* :184 */
        for (uint32_t i = 0; i < m; i++)
            emit(t, step0 + step, K_COPY, rank, B_OUT, rx[i].offset, recv_from, B_OUT, rx[i].offset, rx[i].size);
    }
}

/* AllReduceNHR::RunAsync for one rank, tpl/temp_all_reduce/all_reduce_nhr.cc:25-77: slices :104-121 (the ring's
 * table), RunReduceScatter :133-154 (input, input, output-as-scratch; needMerge = true), RunAllGather :156-173
 * (input, output, output; needMerge = true), whose RunAsync first copies the own slice (all_gather_nhr.cc:75-81). */
static void prog_allreduce_nhr(OrcTrace* t, uint32_t rank, uint32_t n, uint64_t count, uint32_t unit)
{
    if (n == 1) { /* :35-44 */
        emit(t, 0, K_COPY, 0, B_OUT, 0, 0, B_IN, 0, count * unit);
        return;
    }
    OrcSlice sl[ORC_MAX_RANKS];
    uint32_t slice_map[ORC_MAX_RANKS];
    orc_slices_ring(count, unit, n, sl);
    nhr_rank_mapping(n, 0, slice_map);
    prog_nhr_rs(t, rank, n, sl, NULL, slice_map, 1);
    const uint32_t n_steps = nhr_steps(n);
    const uint32_t target = slice_map[rank];
    emit(t, n_steps, K_COPY, rank, B_OUT, sl[target].offset, rank, B_IN, sl[target].offset, sl[target].size);
    prog_nhr_ag(t, rank, n, sl, slice_map, 1, n_steps + 1);
}

/* Stand-alone ReduceScatterNHR::RunAsync, tpl/temp_reduce_scatter/reduce_scatter_nhr.cc:27-95: slices :57-75
 * (input larger than output -> output offset 0; input slice i at i * stride elements as in the strided scatter
 * layout), order kept (:86-88), no merging (isNeedMerge defaults to false,
 * tpl/nonuniform_hierarchical_ring_base_pub.h:54). */
static void prog_rs_nhr(OrcTrace* t, uint32_t rank, uint32_t n, uint64_t count, uint64_t stride, uint32_t unit)
{
    const uint64_t sz = count * unit;
    if (n == 1) { /* :41-46 */
        emit(t, 0, K_COPY, 0, B_OUT, 0, 0, B_IN, 0, sz);
        return;
    }
    OrcSlice sl[ORC_MAX_RANKS], osl[ORC_MAX_RANKS];
    uint32_t slice_map[ORC_MAX_RANKS];
    for (uint32_t i = 0; i < n; i++) {
        sl[i].size = sz;
        sl[i].offset = (uint64_t)i * stride * unit;
        osl[i].size = sz;
        osl[i].offset = 0;
    }
    nhr_rank_mapping(n, 1, slice_map);
    prog_nhr_rs(t, rank, n, sl, osl, slice_map, 0);
}

/* ReduceScatterNB::RunReduceScatterNB for one rank, tpl/temp_reduce_scatter/reduce_scatter_nb.cc:119-230 ->
 * RunDestReducerNB :260-311 -> Reducer::run inline branch (tpl/component/reducer.cc:199-222). */
static void prog_nb_rs(OrcTrace* t, uint32_t rank, uint32_t n, const OrcSlice* sl, const OrcSlice* out_sl)
{
    const uint32_t n_steps = nhr_steps(n);
    for (uint32_t step = 0; step < n_steps; step++) {
        const uint32_t delta_rank = 1u << step;                                /* :149 */
        const uint32_t recv_from = (n + rank - delta_rank) % n;                /* :150 */
        const uint32_t n_slices = (n - 1 + (1u << step)) / (1u << (step + 1)); /* :154 */
        const uint32_t delta_slice = 1u << (step + 1);
        uint32_t rx_idx = rank;                                                /* :157 */
        for (uint32_t i = 0; i < n_slices; i++) {
            if (sl[rx_idx].size > 0) {
                emit(t, step, K_REDUCE, rank, B_IN, sl[rx_idx].offset, recv_from, B_IN, sl[rx_idx].offset, sl[rx_idx].size);
                if (step == n_steps - 1 && out_sl) /* :267-289: dst is the output, src the input slice */
                    emit(t, step + 1, K_COPY, rank, B_OUT, out_sl[rx_idx].offset, rank, B_IN, sl[rx_idx].offset, sl[rx_idx].size);
            }
            rx_idx = (rx_idx + delta_slice) % n;
        }
    }
}

/* AllGatherNB::RunAllGather for one rank, tpl/temp_all_gather/all_gather_nb.cc:101-188 */
static void prog_nb_ag(OrcTrace* t, uint32_t rank, uint32_t n, const OrcSlice* sl, uint32_t step0)
{
    const uint32_t n_steps = nhr_steps(n);
    for (uint32_t step = 0; step < n_steps; step++) {
        const uint32_t delta_rank = 1u << step;
        const uint32_t recv_from = (n + rank - delta_rank) % n; /* :119 */
        uint32_t n_slices = 1u << step;                          /* :124-127 */
        if (step == n_steps - 1 && n != (1u << n_steps)) n_slices = n - (1u << step);
        for (uint32_t i = 0; i < n_slices; i++) {
            const uint32_t rx = (rank - (1u << step) + n - i) % n; /* :138 */
            if (sl[rx].size > 0)
                emit(t, step0 + step, K_COPY, rank, B_OUT, sl[rx].offset, recv_from, B_OUT, sl[rx].offset, sl[rx].size);
        }
    }
}

/* GetSliceSizeOfNB, tpl/temp_all_reduce/all_reduce_nb.cc:203-219 + the slice loop of :139-150 */
void orc_slices_nb(uint64_t total, uint32_t n, OrcSlice* sl)
{
    const uint64_t small = 128u * 1024u; /* NB_ALLREDUCE_SMALL_SIZE, tpl/nonuniform_bruck_base_pub.h:19 */
    const uint64_t calc = (total + (n - 1)) / n;
    const uint64_t div = (calc > small) ? 128u : small;
    const uint64_t aligned = (calc == 0) ? div : ((calc + div - 1) / div) * div; /* RoundUpWithDivisor */
    uint64_t residue = total;
    for (uint32_t i = 0; i < n; i++) {
        sl[i].size = (residue > aligned) ? aligned : residue;
        sl[i].offset = total - residue;
        residue -= sl[i].size;
    }
}

/* AllReduceNB::RunAsync for one rank, tpl/temp_all_reduce/all_reduce_nb.cc:26-61 (RunReduceScatter :162-180,
 * RunAllGather :182-201; the own-slice copy is AllGatherNB::RunAsync, tpl/temp_all_gather/all_gather_nb.cc:88-92) */
static void prog_allreduce_nb(OrcTrace* t, uint32_t rank, uint32_t n, uint64_t count, uint32_t unit)
{
    if (n == 1) { /* PrepareRunAsync :130-137 */
        emit(t, 0, K_COPY, 0, B_OUT, 0, 0, B_IN, 0, count * unit);
        return;
    }
    OrcSlice sl[ORC_MAX_RANKS];
    orc_slices_nb(count * unit, n, sl);
    prog_nb_rs(t, rank, n, sl, NULL);
    const uint32_t n_steps = nhr_steps(n);
    emit(t, n_steps, K_COPY, rank, B_OUT, sl[rank].offset, rank, B_IN, sl[rank].offset, sl[rank].size);
    prog_nb_ag(t, rank, n, sl, n_steps + 1);
}

/* Stand-alone ReduceScatterNB::RunAsync, tpl/temp_reduce_scatter/reduce_scatter_nb.cc:27-86 (slices :50-70) */
static void prog_rs_nb(OrcTrace* t, uint32_t rank, uint32_t n, uint64_t count, uint64_t stride, uint32_t unit)
{
    const uint64_t sz = count * unit;
    if (n == 1) { /* :35-40 */
        emit(t, 0, K_COPY, 0, B_OUT, 0, 0, B_IN, 0, sz);
        return;
    }
    OrcSlice sl[ORC_MAX_RANKS], osl[ORC_MAX_RANKS];
    for (uint32_t i = 0; i < n; i++) {
        sl[i].size = sz;
        sl[i].offset = (uint64_t)i * stride * unit;
        osl[i].size = sz;
        osl[i].offset = 0;
    }
    prog_nb_rs(t, rank, n, sl, osl);
}

/* ReduceScatterLocalReduce::RunAsync for one rank, tpl/temp_reduce_scatter/reduce_scatter_local_reduce.cc:125-160,
 * in the single-pass configuration (count_ == opInfo->count; the template's "output memory" is the communication
 * buffer, sized so that CalAlign's first choice fits).  Returns the bytes of communication buffer a rank needs
 * when t is NULL. */
static uint64_t prog_rs_local_reduce(OrcTrace* t, uint32_t rank, uint32_t n, uint64_t count, uint32_t unit)
{
    const uint64_t total = count * unit;            /* totalSize, :187 */
    const uint64_t offset = count * unit;           /* (opInfo_->count) * unitSize, :192 */
    uint64_t sl_off[ORC_MAX_RANKS], max_off = 0;
    for (uint32_t i = 0; i < n; i++) {              /* PrepareOffset, :113-121 */
        sl_off[i] = (total > 32u * 1024u) ? ((uint64_t)i * offset) % 16384u : 0;
        if (sl_off[i] > max_off) max_off = sl_off[i];
    }
    /* CalAlign, :162-178, first choice: RoundUpWithDivisor(totalSize, HCCL_MIN_SLICE_ALIGN_910B), which is the
     * divisor itself for 0 (tpl/alg_template_base_pub.h:609-616) */
    const uint64_t align = (total == 0) ? 16384u : ((total + 16383u) / 16384u) * 16384u;
    const uint64_t need = max_off + align * (n - 1);
    if (!t || n == 0) return n > 1 ? need : 0;
    /* RunReduceScatter, :218-243: all rounds run at once, each on a stream of its own */
    for (uint32_t round = 1; round < n; round++) {
        const uint32_t dst_rank = (round + rank) % n;
        emit(t, 0, K_COPY, dst_rank, B_SCR, align * (round - 1) + sl_off[dst_rank], rank, B_IN, offset * dst_rank, total);
    }
    emit(t, 0, K_COPY, rank, B_OUT, 0, rank, B_IN, offset * rank, total); /* :238-241 */
    /* RunLocalReduce, :252-304; the window starts at slices_[rank].offset (:262) */
    uint32_t power = 0;
    while ((2u << power) <= n) power++;             /* static_cast<u32>(log2(rankSize)) */
    uint32_t rank_power = 1u << power;
    const uint64_t win = sl_off[rank];
    uint32_t step = 1;
    if (rank_power < n) {
        for (uint32_t add = 0; add < n - rank_power; add++) { /* :270-282 */
            const uint64_t src = win + align * (add + rank_power - 1);
            if (add == 0) emit(t, step, K_REDUCE, rank, B_OUT, 0, rank, B_SCR, src, total);
            else emit(t, step, K_REDUCE, rank, B_SCR, win + align * (add - 1), rank, B_SCR, src, total);
        }
        step++;
    }
    for (uint32_t round = 0; round < power; round++) { /* :286-301 */
        rank_power = 1u << (power - round - 1);
        for (uint32_t add = 0; add < rank_power; add++) {
            const uint64_t src = win + align * (add + rank_power - 1);
            if (add == 0) emit(t, step, K_REDUCE, rank, B_OUT, 0, rank, B_SCR, src, total);
            else emit(t, step, K_REDUCE, rank, B_SCR, win + align * (add - 1), rank, B_SCR, src, total);
        }
        step++;
    }
    return need;
}

/* Bytes of communication buffer per rank for the deterministic mesh reduce-scatter. */
uint64_t orc_rs_local_reduce_scratch_bytes(uint32_t n, uint64_t count, int dtype)
{
    const uint32_t unit = orc_dtype_size(dtype);
    if (n == 0 || n > ORC_MAX_RANKS || unit == 0) return 0;
    return prog_rs_local_reduce(NULL, 0, n, count, unit);
}

/* The NHR slice map, exported for the hand-derived fixtures. */
void orc_nhr_slice_map(uint32_t n, uint32_t* slice_map)
{
    if (n == 0 || n > ORC_MAX_RANKS) return;
    nhr_rank_mapping(n, 0, slice_map);
}

enum {
    ORC_ALG_ALLREDUCE_RING = 0,
    ORC_ALG_RS_RING_STAGE = 1,
    ORC_ALG_ALLREDUCE_RHD = 2,
    ORC_ALG_ALLREDUCE_MESH_ONESHOT = 3,
    ORC_ALG_RS_MESH = 4,
    ORC_ALG_RS_RING_STANDALONE = 5,
    ORC_ALG_ALLREDUCE_MESH_ASCENDING = 6,
    ORC_ALG_ALLREDUCE_LOCAL_REDUCE = 7,
    ORC_ALG_ALLREDUCE_CHUNK_MESH = 8,
    ORC_ALG_ALLREDUCE_NHR = 9,
    ORC_ALG_RS_NHR = 10,
    ORC_ALG_ALLREDUCE_NB = 11,
    ORC_ALG_RS_NB = 12,
    ORC_ALG_RS_LOCAL_REDUCE = 13,
    ORC_ALG_ALLREDUCE_DOUBLING = 14,
    ORC_ALG_ALLREDUCE_NHR_ONESHOT = 15,
    ORC_ALG_RS_RHD = 16, /* only between the servers of the two-level reduce-scatter */
    ORC_ALG_RS_WINDOW_HALVING = 17,
    ORC_ALG_ALLREDUCE_LOCAL_REDUCE_AS_WRITTEN = 18 /* traces only: the statements for any rank count, right or wrong */
};

static int cmp_ops(const void* a, const void* b)
{
    const OrcOp* x = (const OrcOp*)a;
    const OrcOp* y = (const OrcOp*)b;
    if (x->step != y->step) return x->step < y->step ? -1 : 1;
    if (x->rank != y->rank) return x->rank < y->rank ? -1 : 1;
    return 0;
}

/* lock step: order by step, then by the rank that owns the destination; emission order is kept among equals */
static int sort_trace(OrcTrace* t)
{
    if (t->n > 1) {
        OrcOp* tmp = (OrcOp*)malloc(t->n * sizeof(OrcOp));
        if (!tmp) {
            free(t->ops);
            return -2;
        }
        for (uint64_t width = 1; width < t->n; width *= 2) { /* bottom-up merge sort: stable */
            for (uint64_t lo = 0; lo < t->n; lo += 2 * width) {
                const uint64_t mid = lo + width < t->n ? lo + width : t->n;
                const uint64_t hi = lo + 2 * width < t->n ? lo + 2 * width : t->n;
                uint64_t a = lo, b = mid, k = lo;
                while (a < mid && b < hi) tmp[k++] = (cmp_ops(&t->ops[b], &t->ops[a]) < 0) ? t->ops[b++] : t->ops[a++];
                while (a < mid) tmp[k++] = t->ops[a++];
                while (b < hi) tmp[k++] = t->ops[b++];
            }
            memcpy(t->ops, tmp, t->n * sizeof(OrcOp));
        }
        free(tmp);
    }
    return 0;
}

static uint64_t g_stride = 0; /* elements between input slices of the scatter algorithms; 0 = dense */

/* Applies to the next orc_trace / orc_run / orc_algorithmic_bytes calls (scatter algorithms only). */
void orc_set_stride(uint64_t stride) { g_stride = stride; }

static int build_trace(OrcTrace* t, int alg, uint32_t n, uint64_t count, int dtype)
{
    memset(t, 0, sizeof(*t));
    const uint32_t unit = orc_dtype_size(dtype);
    if (n == 0 || n > ORC_MAX_RANKS || unit == 0) return -1;
    const uint64_t stride = g_stride ? g_stride : count;
    if (stride < count) return -1;
    for (uint32_t r = 0; r < n; r++) {
        switch (alg) {
            case ORC_ALG_ALLREDUCE_RING: prog_allreduce_ring(t, r, n, count, unit, 1); break;
            case ORC_ALG_RS_RING_STAGE: prog_allreduce_ring(t, r, n, count, unit, 0); break;
            case ORC_ALG_ALLREDUCE_RHD: prog_allreduce_rhd(t, r, n, count, unit); break;
            case ORC_ALG_ALLREDUCE_MESH_ONESHOT: prog_allreduce_mesh_oneshot(t, r, n, count, unit); break;
            case ORC_ALG_RS_MESH: prog_rs_mesh(t, r, n, count, stride, unit); break;
            case ORC_ALG_RS_RING_STANDALONE: prog_rs_ring_standalone(t, r, n, count, stride, unit); break;
            case ORC_ALG_ALLREDUCE_MESH_ASCENDING: prog_allreduce_mesh_ascending(t, r, n, count, unit); break;
            case ORC_ALG_ALLREDUCE_CHUNK_MESH: prog_allreduce_chunk_mesh(t, r, n, count, unit); break;
            case ORC_ALG_ALLREDUCE_NHR: prog_allreduce_nhr(t, r, n, count, unit); break;
            case ORC_ALG_RS_NHR: prog_rs_nhr(t, r, n, count, stride, unit); break;
            case ORC_ALG_ALLREDUCE_NB: prog_allreduce_nb(t, r, n, count, unit); break;
            case ORC_ALG_RS_NB: prog_rs_nb(t, r, n, count, stride, unit); break;
            case ORC_ALG_RS_WINDOW_HALVING: prog_rs_window_halving(t, r, n, count, stride, unit); break;
            case ORC_ALG_ALLREDUCE_NHR_ONESHOT: prog_allreduce_nhr_oneshot(t, r, n, count, unit); break;
            case ORC_ALG_ALLREDUCE_DOUBLING:
                if (prog_allreduce_doubling(t, r, n, count, unit) != 0) {
                    free(t->ops);
                    return -1;
                }
                break;
            case ORC_ALG_RS_LOCAL_REDUCE:
                if (stride != count) {
                    free(t->ops);
                    return -1;
                }
                prog_rs_local_reduce(t, r, n, count, unit);
                break;
            case ORC_ALG_ALLREDUCE_LOCAL_REDUCE:
            case ORC_ALG_ALLREDUCE_LOCAL_REDUCE_AS_WRITTEN:
                if (prog_allreduce_local_reduce(t, r, n, count, unit, alg == ORC_ALG_ALLREDUCE_LOCAL_REDUCE_AS_WRITTEN) != 0) {
                    free(t->ops);
                    return -1;
                }
                break;
            default: free(t->ops); return -1;
        }
    }
    if (t->oom) {
        free(t->ops);
        return -2;
    }
    return sort_trace(t);
}

/* Write the lock-step op list (ordered by step, then rank).  Returns the total number of ops, or < 0. */
int64_t orc_trace(int alg, uint32_t n, uint64_t count, int dtype, OrcOp* out, uint64_t cap)
{
    OrcTrace t;
    int rc = build_trace(&t, alg, n, count, dtype);
    if (rc) return rc;
    const uint64_t m = t.n < cap ? t.n : cap;
    if (out && m) memcpy(out, t.ops, m * sizeof(OrcOp));
    const int64_t total = (int64_t)t.n;
    free(t.ops);
    return total;
}

static int ranges_overlap(uintptr_t a, uint64_t an, uintptr_t b, uint64_t bn) { return a < b + bn && b < a + an; }

/*
 * Execute a collective on host buffers in[r] / out[r].  Ranks act in lock step; inside a step the
 * operations must not observe each other (the memory-conflict rule of the reference's schedule checker,
 * test/st/algorithm/README_en.md:202-231), which is verified before the step runs, so executing them one
 * after another equals executing them concurrently.  Returns 0, -1 bad argument, -2 out of memory,
 * -3 conflict inside a step.
 */
static void* const* g_scratch = NULL; /* per-rank communication buffers for the next orc_run (or NULL) */

void orc_set_scratch(void* const* scratch) { g_scratch = scratch; }

/* Execute a lock-step op list on host memory; bufs[role][rank], roles B_IN .. B_UOUT.  Refuses a step in which
 * one operation writes what another reads or writes (test/st/algorithm/README_en.md:202-231). */
static int exec_trace(OrcTrace* t, void* const* const* bufs, int dtype, int op)
{
#define BUFPTR(buf, rank) (bufs[buf][rank])
    for (uint64_t q = 0; q < t->n; q++)
        if (!bufs[t->ops[q].dst_buf] || !bufs[t->ops[q].src_buf]) return -1;
    const uint32_t unit = orc_dtype_size(dtype);
    uint64_t i = 0;
    while (i < t->n) {
        uint64_t j = i;
        while (j < t->n && t->ops[j].step == t->ops[i].step) j++;
        for (uint64_t a = i; a < j; a++) {
            const OrcOp* x = &t->ops[a];
            const uintptr_t xd = (uintptr_t)BUFPTR(x->dst_buf, x->rank) + x->dst_off;
            for (uint64_t b = i; b < j; b++) {
                if (a == b) continue;
                const OrcOp* y = &t->ops[b];
                const uintptr_t yd = (uintptr_t)BUFPTR(y->dst_buf, y->rank) + y->dst_off;
                const uintptr_t ys = (uintptr_t)BUFPTR(y->src_buf, y->src_rank) + y->src_off;
                if (ranges_overlap(xd, x->bytes, yd, y->bytes) || ranges_overlap(xd, x->bytes, ys, y->bytes)) return -3;
            }
        }
        for (uint64_t a = i; a < j; a++) {
            const OrcOp* x = &t->ops[a];
            char* d = (char*)BUFPTR(x->dst_buf, x->rank) + x->dst_off;
            const char* s = (const char*)BUFPTR(x->src_buf, x->src_rank) + x->src_off;
            if (x->kind == K_COPY)
                orc_copy(d, s, x->bytes);
            else if (orc_reduce(d, s, x->bytes / unit, dtype, op) != 0)
                return -1;
        }
        i = j;
    }
    return 0;
#undef BUFPTR
}

int orc_run(int alg, uint32_t n, void* const* in, void* const* out, uint64_t count, int dtype, int op)
{
    OrcTrace t;
    int rc = build_trace(&t, alg, n, count, dtype);
    if (rc) return rc;
    void* const* bufs[5] = {in, out, g_scratch, NULL, NULL};
    rc = exec_trace(&t, bufs, dtype, op);
    free(t.ops);
    return rc;
}

/* ---- the op-base loop of the executors, per rank ------------------------------------------------------------ */

static int is_scatter(int alg)
{
    return alg == ORC_ALG_RS_MESH || alg == ORC_ALG_RS_RING_STANDALONE || alg == ORC_ALG_RS_NHR || alg == ORC_ALG_RS_NB ||
           alg == ORC_ALG_RS_LOCAL_REDUCE;
}

/* "exec/" abbreviates src/legacy/ascend910/algorithm/impl/coll_executor/.
 * CollAllReduceExecutor::CalcLoopMaxCount, exec/coll_all_reduce/coll_all_reduce_executor.cc:129-138;
 * CollReduceScatterExecutor::CalcLoopMaxCount, exec/coll_reduce_scatter/coll_reduce_scatter_executor.cc:124-134 */
uint64_t orc_opbase_max_count(int alg, uint32_t n, uint64_t ccl_bytes, int dtype)
{
    const uint32_t unit = orc_dtype_size(dtype);
    if (unit == 0 || n == 0) return 0;
    if (!is_scatter(alg)) return ccl_bytes / unit;
    return ccl_bytes / n / 128u * 128u / unit;
}

static void run_template(OrcTrace* t, int alg, uint32_t r, uint32_t n, uint64_t count, uint32_t unit)
{
    switch (alg) {
        case ORC_ALG_ALLREDUCE_RING: prog_allreduce_ring(t, r, n, count, unit, 1); break;
        case ORC_ALG_ALLREDUCE_RHD: prog_allreduce_rhd(t, r, n, count, unit); break;
        case ORC_ALG_ALLREDUCE_MESH_ONESHOT: prog_allreduce_mesh_oneshot(t, r, n, count, unit); break;
        case ORC_ALG_RS_MESH: prog_rs_mesh(t, r, n, count, count, unit); break;
        case ORC_ALG_RS_RING_STANDALONE: prog_rs_ring_standalone(t, r, n, count, count, unit); break;
        case ORC_ALG_ALLREDUCE_MESH_ASCENDING: prog_allreduce_mesh_ascending(t, r, n, count, unit); break;
        case ORC_ALG_ALLREDUCE_CHUNK_MESH: prog_allreduce_chunk_mesh(t, r, n, count, unit); break;
        case ORC_ALG_ALLREDUCE_LOCAL_REDUCE: prog_allreduce_local_reduce(t, r, n, count, unit, 0); break;
        case ORC_ALG_ALLREDUCE_NHR: prog_allreduce_nhr(t, r, n, count, unit); break;
        case ORC_ALG_RS_NHR: prog_rs_nhr(t, r, n, count, count, unit); break;
        case ORC_ALG_ALLREDUCE_NB: prog_allreduce_nb(t, r, n, count, unit); break;
        case ORC_ALG_RS_NB: prog_rs_nb(t, r, n, count, count, unit); break;
        case ORC_ALG_RS_LOCAL_REDUCE: prog_rs_local_reduce(t, r, n, count, unit); break;
        case ORC_ALG_ALLREDUCE_DOUBLING: prog_allreduce_doubling(t, r, n, count, unit); break;
        case ORC_ALG_ALLREDUCE_NHR_ONESHOT: prog_allreduce_nhr_oneshot(t, r, n, count, unit); break;
        default: break;
    }
}

/* Steps of the template that do anything for `count` elements (the ranks run in lock step, so the copy back to
 * the user buffer of a chunk sits one step after the template's last one on every rank). */
static int template_steps(int alg, uint32_t n, uint64_t count, int dtype, uint32_t* steps)
{
    OrcTrace t;
    const uint64_t keep = g_stride;
    const uint32_t keep_base = g_step_base;
    g_stride = 0;
    g_step_base = 0;
    const int rc = build_trace(&t, alg, n, count, dtype);
    g_stride = keep;
    g_step_base = keep_base;
    if (rc) return rc;
    *steps = t.n ? t.ops[t.n - 1].step + 1 : 0;
    free(t.ops);
    return 0;
}

/* CollAllReduceExecutor::RunLoop + RunLoopInner for one rank (exec/coll_all_reduce/coll_all_reduce_executor.cc:
 * 199-262, 264-339) and CollReduceScatterExecutor::RunLoop + RunLoopInner
 * (exec/coll_reduce_scatter/coll_reduce_scatter_executor.cc:149-220, 222-306), both in the buffer-copy mode
 * (DMAReduceFlag_ false): B_IN / B_OUT are the CCL buffers the template runs on. */
static int prog_opbase(OrcTrace* t, int alg, uint32_t rank, uint32_t n, uint64_t total_count, uint64_t max_count,
                       int dtype)
{
    const uint32_t unit = orc_dtype_size(dtype);
    const int scatter = is_scatter(alg);
    uint64_t cur_in = 0, cur_out = 0;             /* curInputPtr, curOutputPtr as offsets */
    uint64_t cur_count = 0, input_offset = 0, output_offset = 0;
    uint32_t step = 0;
    for (uint64_t count_left = total_count; count_left > 0; count_left -= cur_count) {
        cur_in += input_offset;                   /* :236-237 / :172-173 */
        cur_out += output_offset;
        cur_count = (count_left > max_count) ? max_count : count_left;
        const uint64_t cur_size = cur_count * unit;
        g_step_base = step;
        if (!scatter) {
            emit(t, 0, K_COPY, rank, B_IN, 0, rank, B_UIN, cur_in, cur_size);              /* :304-309 */
        } else if (total_count == cur_count) {                                              /* preloadCopyOpt, :616-620 */
            emit(t, 0, K_COPY, rank, B_IN, 0, rank, B_UIN, cur_in, total_count * unit * n); /* :260-265 */
        } else {
            for (uint32_t i = 0; i < n; i++)                                                /* :267-273 */
                emit(t, 0, K_COPY, rank, B_IN, cur_size * i, rank, B_UIN, cur_in + total_count * unit * i, cur_size);
        }
        uint32_t used = 0;
        const int rc = template_steps(alg, n, cur_count, dtype, &used);
        if (rc) {
            g_step_base = 0;
            return rc;
        }
        g_step_base = step + 1;
        run_template(t, alg, rank, n, cur_count, unit);                                     /* KernelRun */
        g_step_base = step + 1 + used;
        emit(t, 0, K_COPY, rank, B_UOUT, cur_out, rank, B_OUT, 0, cur_size);                /* :326-331 / :292-297 */
        g_step_base = 0;
        step += used + 2;
        input_offset = cur_size;
        output_offset = cur_size;
    }
    return 0;
}

static int build_trace_opbase(OrcTrace* t, int alg, uint32_t n, uint64_t count, uint64_t ccl_bytes, int dtype)
{
    memset(t, 0, sizeof(*t));
    const uint32_t unit = orc_dtype_size(dtype);
    if (n == 0 || n > ORC_MAX_RANKS || unit == 0 || alg == ORC_ALG_RS_RING_STAGE) return -1;
    const uint64_t max_count = orc_opbase_max_count(alg, n, ccl_bytes, dtype);
    if (max_count == 0) return -1; /* :213-218 / :163-165 */
    if (alg == ORC_ALG_ALLREDUCE_DOUBLING && (n & (n - 1))) return -1;
    if (alg == ORC_ALG_ALLREDUCE_LOCAL_REDUCE && n > 1 && !local_reduce_lands(n)) return -1;
    for (uint32_t r = 0; r < n; r++) {
        const int rc = prog_opbase(t, alg, r, n, count, max_count, dtype);
        if (rc || t->oom) {
            free(t->ops);
            return rc ? rc : -2;
        }
    }
    return sort_trace(t);
}

int64_t orc_trace_opbase(int alg, uint32_t n, uint64_t count, uint64_t ccl_bytes, int dtype, OrcOp* out, uint64_t cap)
{
    OrcTrace t;
    int rc = build_trace_opbase(&t, alg, n, count, ccl_bytes, dtype);
    if (rc) return rc;
    const uint64_t m = t.n < cap ? t.n : cap;
    if (out && m) memcpy(out, t.ops, m * sizeof(OrcOp));
    const int64_t total = (int64_t)t.n;
    free(t.ops);
    return total;
}

int orc_run_opbase(int alg, uint32_t n, void* const* user_in, void* const* user_out, void* const* ccl_in,
                   void* const* ccl_out, uint64_t count, uint64_t ccl_bytes, int dtype, int op)
{
    OrcTrace t;
    int rc = build_trace_opbase(&t, alg, n, count, ccl_bytes, dtype);
    if (rc) return rc;
    void* const* bufs[5] = {ccl_in, ccl_out, g_scratch, user_in, user_out};
    rc = exec_trace(&t, bufs, dtype, op);
    free(t.ops);
    return rc;
}

/* ---- the ring executor's three-step allreduce over two communicator levels ----------------------------------- */

/* ExecutorBase::PrepareSliceMeshStreams, tpl/alg_template_base.cc:823-865: every segment cut into stream_count pieces of
 * ceil(size / stream_count) bytes rounded up to 128; out[stream][rank] */
static void slices_mesh_streams(const OrcSlice* seg, uint32_t n, uint32_t stream_count, OrcSlice out[][ORC_MAX_RANKS])
{
    uint64_t rank_stream_size[ORC_MAX_RANKS], rank_residue[ORC_MAX_RANKS];
    for (uint32_t rank_id = 0; rank_id < n; rank_id++) {
        const uint64_t size_per_stream = (seg[rank_id].size + stream_count - 1) / stream_count;
        rank_stream_size[rank_id] = (size_per_stream + 127) / 128 * 128;
        rank_residue[rank_id] = seg[rank_id].size;
    }
    for (uint32_t stream = 0; stream < stream_count; stream++)
        for (uint32_t rank_id = 0; rank_id < n; rank_id++) {
            const uint64_t residue = rank_residue[rank_id];
            if (residue > 0) {
                const uint64_t single = rank_stream_size[rank_id] < residue ? rank_stream_size[rank_id] : residue;
                out[stream][rank_id].offset = seg[rank_id].offset + seg[rank_id].size - residue;
                out[stream][rank_id].size = single;
                rank_residue[rank_id] -= single;
            } else {
                out[stream][rank_id].offset = seg[rank_id].offset;
                out[stream][rank_id].size = 0;
            }
        }
}

/* CollCommExecutor::MultiStreamReduceScatterMesh (exec/coll_comm_executor.cc:1754-1860): one ReduceScatterMesh per
 * stream on that stream's pieces, input memory == output memory (no final copy), each starting its walk through the
 * default peer order at its stream index (tpl/temp_reduce_scatter/reduce_scatter_mesh.cc:51-68); the streams run side
 * by side, so round k of all of them is one lock-step step.  Inline reduce (:40-46). */
static void prog_mesh_rs_streams(OrcTrace* t, uint32_t rank, uint32_t n, const OrcSlice* seg)
{
    if (n == 1) return; /* :141-146 with inputMem_ == outputMem_ */
    static OrcSlice stream_slices[ORC_MAX_RANKS][ORC_MAX_RANKS];
    slices_mesh_streams(seg, n, n - 1, stream_slices);
    uint32_t rx_rank_op_order[ORC_MAX_RANKS];
    for (uint32_t round = 1; round < n; round++) rx_rank_op_order[round - 1] = (rank + n - round) % n; /* ForwardRank */
    for (uint32_t stream_index = 0; stream_index < n - 1; stream_index++)
        for (uint32_t round = 1; round < n; round++) {
            const uint32_t order_index = (round + stream_index - 1) % (n - 1);
            const uint32_t src_rank = rx_rank_op_order[order_index];
            const OrcSlice* own = &stream_slices[stream_index][rank];
            emit(t, round - 1, K_REDUCE, rank, B_IN, own->offset, src_rank, B_IN, own->offset, own->size);
        }
}

/* AllGatherMesh::RunAllGather, tpl/temp_all_gather/all_gather_mesh.cc:66-131, prepared with the output memory as both
 * input and output (exec/coll_all_reduce/coll_all_reduce_mesh_executor.cc:219-222): round r fetches the slice of rank
 * BackwardRank(rank, r) = rank - r (base/inc/all_gather_mesh_pub.h:33-39) on a stream of its own, all rounds at once. */
static void prog_mesh_ag(OrcTrace* t, uint32_t rank, uint32_t n, const OrcSlice* seg)
{
    for (uint32_t round = 1; round < n; round++) {
        const uint32_t dst_rank = (rank + n - round) % n;
        emit(t, 0, K_COPY, rank, B_OUT, seg[dst_rank].offset, dst_rank, B_OUT, seg[dst_rank].offset, seg[dst_rank].size);
    }
}

/* coll_all_reduce_ring_executor.cc:171-181: curSize / deviceNumPerAggregation <= NHR_ALLREDUCE_SMALL_SIZE
 * (256 KiB, pub_inc/op_context.h:18) selects the one-shot NHR template; the devices of an aggregation are the
 * n_local ranks of a server here. */
static int hier_level1_template(int alg1, uint64_t count, uint32_t unit, uint32_t n_local)
{
    const uint64_t cur_size = count * unit;
    if (alg1 == ORC_ALG_ALLREDUCE_NHR && cur_size / n_local <= 256u * 1024u) return ORC_ALG_ALLREDUCE_NHR_ONESHOT;
    return alg1;
}

/* CollAllReduceRingExecutor::KernelRun for one rank, exec/coll_all_reduce/coll_all_reduce_ring_executor.cc:94-231,
 * single ring per server (ringNum == 1, :123-125), buffer-copy mode.  rank = server * n_local + local index. */
static int prog_hier_allreduce(OrcTrace* t, int level0_mesh, int alg1, uint32_t rank, uint32_t n_servers, uint32_t n_local,
                               uint64_t count, int dtype, uint32_t level1_steps)
{
    const uint32_t unit = orc_dtype_size(dtype);
    const uint32_t server = rank / n_local, local = rank % n_local;
    uint32_t level0[ORC_MAX_RANKS], level1[ORC_MAX_RANKS];
    for (uint32_t j = 0; j < n_local; j++) level0[j] = server * n_local + j;
    for (uint32_t s = 0; s < n_servers; s++) level1[s] = s * n_local + local;
    OrcSlice seg[ORC_MAX_RANKS];
    orc_slices_ring(count, unit, n_local, seg);          /* PrepareSliceData, :109 (tpl/alg_template_base.cc:787-820) */
    /* step 1, :134-136: ReduceScatterRing on (input, input, output-as-scratch) inside the server */
    g_rank_map = level0;
    g_step_base = 0;
    if (level0_mesh) prog_mesh_rs_streams(t, local, n_local, seg); /* CollAllReduceMeshExecutor::KernelRun, :116-119 */
    else if (n_local > 1) prog_ring_rs(t, local, n_local, seg, NULL);
    /* step 2, :140-218: level-1 allreduce of the own segment; hdSize / segment from PrepareLevel1CommInfo,
     * exec/coll_comm_executor.cc:2565-2575 */
    const uint64_t hd_count = seg[local].size / unit;    /* :146 */
    g_rank_map = level1;
    g_base_off = seg[local].offset;                      /* :211 */
    g_step_base = n_local - 1;
    run_template(t, hier_level1_template(alg1, count, unit, n_local), server, n_servers, hd_count, unit);
    g_base_off = 0;
    /* step 3, :228-230: AllGatherRing on (output, output, input-as-scratch), exec/coll_comm_executor.cc:377-379 */
    g_rank_map = level0;
    g_step_base = n_local - 1 + level1_steps;
    if (level0_mesh) prog_mesh_ag(t, local, n_local, seg);         /* CollAllReduceMeshExecutor::KernelRun, :204-228 */
    else if (n_local > 1) prog_ring_ag_ex(t, local, n_local, seg, 0, 0);
    g_rank_map = NULL;
    g_step_base = 0;
    return 0;
}

static int build_trace_hier(OrcTrace* t, int level0_mesh, int alg1, uint32_t n_servers, uint32_t n_local, uint64_t count,
                            int dtype)
{
    memset(t, 0, sizeof(*t));
    const uint32_t unit = orc_dtype_size(dtype);
    if (unit == 0 || n_servers == 0 || n_local == 0 || n_servers * n_local > ORC_MAX_RANKS) return -1;
    if (level0_mesh && n_local < 2) return -1; /* streamCount == 0, tpl/alg_template_base.cc:832-835 */
    if (alg1 != ORC_ALG_ALLREDUCE_RING && alg1 != ORC_ALG_ALLREDUCE_RHD && alg1 != ORC_ALG_ALLREDUCE_NHR &&
        alg1 != ORC_ALG_ALLREDUCE_NB)
        return -1;
    /* the ranks run in lock step: the gather starts when the longest level-1 allreduce (the largest segment) is over */
    OrcSlice seg[ORC_MAX_RANKS];
    orc_slices_ring(count, unit, n_local, seg);
    uint32_t level1_steps = 0;
    for (uint32_t i = 0; i < n_local; i++) {
        uint32_t st = 0;
        const int rc = template_steps(hier_level1_template(alg1, count, unit, n_local), n_servers, seg[i].size / unit, dtype, &st);
        if (rc) return rc;
        if (st > level1_steps) level1_steps = st;
    }
    for (uint32_t r = 0; r < n_servers * n_local; r++) {
        prog_hier_allreduce(t, level0_mesh, alg1, r, n_servers, n_local, count, dtype, level1_steps);
        if (t->oom) {
            free(t->ops);
            return -2;
        }
    }
    return sort_trace(t);
}

int64_t orc_trace_hier(int level0_mesh, int alg1, uint32_t n_servers, uint32_t n_local, uint64_t count, int dtype, OrcOp* out,
                       uint64_t cap)
{
    OrcTrace t;
    int rc = build_trace_hier(&t, level0_mesh, alg1, n_servers, n_local, count, dtype);
    if (rc) return rc;
    const uint64_t m = t.n < cap ? t.n : cap;
    if (out && m) memcpy(out, t.ops, m * sizeof(OrcOp));
    const int64_t total = (int64_t)t.n;
    free(t.ops);
    return total;
}

int orc_run_hier(int level0_mesh, int alg1, uint32_t n_servers, uint32_t n_local, void* const* in, void* const* out,
                 uint64_t count, int dtype, int op)
{
    OrcTrace t;
    int rc = build_trace_hier(&t, level0_mesh, alg1, n_servers, n_local, count, dtype);
    if (rc) return rc;
    void* const* bufs[5] = {in, out, NULL, NULL, NULL};
    rc = exec_trace(&t, bufs, dtype, op);
    free(t.ops);
    return rc;
}

/* ---- the double-ring allreduce executor in op-base mode (user memory read and written directly) -------------- */

typedef struct {
    OrcSlice slices[2][ORC_MAX_RANKS]; /* multRingsSliceZero: per ring, the slice each ring position owns */
    uint32_t order[2][ORC_MAX_RANKS];  /* multiRingsOrder */
    OrcSlice seg[ORC_MAX_RANKS];       /* dataSegsSlice */
} OrcDoubleRing;

/* The executor's slice preparation for TOPO_TYPE_NP_DOUBLE_RING with every device in the NIC list:
 * PrepareSliceData (tpl/alg_template_base.cc:787-820), MutliSegSlicePrepare (exec/coll_comm_executor.cc:2011-2052),
 * GetRingsOrderByTopoType (:1939-1949), PrepareMultiRingSlice (:2094-2163, chunkSize == 1). */
static void dbring_prepare(OrcDoubleRing* d, uint64_t count, uint32_t unit, uint32_t n)
{
    orc_slices_ring(count, unit, n, d->seg);
    OrcSlice multi_seg[ORC_MAX_RANKS][2];
    for (uint32_t rank_id = 0; rank_id < n; rank_id++) { /* :2016-2050 */
        const uint64_t rank_data_size = d->seg[rank_id].size, offset_start = d->seg[rank_id].offset;
        uint32_t ring_index = 0;
        if (rank_data_size > 0) {
            const uint64_t size_temp = (rank_data_size + 2 - 1) / 2;
            const uint64_t size_per_ring = (size_temp + 127) / 128 * 128;
            uint64_t residue = rank_data_size;
            while (residue > 0) {
                const uint64_t single = size_per_ring < residue ? size_per_ring : residue;
                multi_seg[rank_id][ring_index].size = single;
                multi_seg[rank_id][ring_index].offset = offset_start + rank_data_size - residue;
                ring_index++;
                residue -= single;
            }
        }
        while (ring_index < 2) {
            multi_seg[rank_id][ring_index].size = 0;
            multi_seg[rank_id][ring_index].offset = offset_start;
            ring_index++;
        }
    }
    for (uint32_t i = 0; i < n; i++) d->order[0][i] = i;                 /* tmpLevel00 = nicList */
    d->order[1][0] = 0;                                                   /* tmpLevel01: nicList[0], then ring 0 reversed */
    for (uint32_t i = 1; i < n; i++) d->order[1][i] = d->order[0][n - i];
    for (uint32_t ring = 0; ring < 2; ring++)
        for (uint32_t segs_index = 0; segs_index < n; segs_index++)
            d->slices[ring][segs_index] = multi_seg[d->order[ring][segs_index]][ring]; /* nicPosition == deviceIdx */
}

/* AlignedReduceScatterDoubleRing::RunAsync for one rank, tpl/temp_reduce_scatter/aligned_reduce_scatter_double_ring.cc,
 * as the allreduce executor prepares it (exec/coll_all_reduce/coll_aligned_all_reduce_double_ring_for_910_93_executor.cc:
 * 57-63): input and output memory = the CCL input buffer, opInfo->inputAddr = the user input, opInfo->outputAddr = null,
 * user-memory slices = the ring slices (CalUserMemSlices, exec/coll_comm_executor.cc:2256-2260), one slice per ring
 * position, inline reduce (:468-488).  Ring 0 (the "sub" ring) receives from rank - 1, ring 1 (the "main" ring) from
 * rank + 1 (:433-447).  Step 0 of the trace is the template's step -1. */
static void prog_dbring_rs(OrcTrace* t, uint32_t rank, uint32_t n, const OrcDoubleRing* d)
{
    if (n == 1) { /* OneRankMemcpy, :125-163 */
        for (uint32_t ring = 0; ring < 2; ring++)
            emit(t, 0, K_COPY, 0, B_IN, d->slices[ring][0].offset, 0, B_UIN, d->slices[ring][0].offset, d->slices[ring][0].size);
        return;
    }
    const uint32_t pre[2] = {(rank + n - 1) % n, (rank + 1) % n};
    /* RunInitStep, :379-412: the two slices of the first step come from the user input */
    const uint32_t init0[2] = {(rank + n - 1) % n, (n - rank - 1 + n) % n};
    const uint32_t init1[2] = {(rank + n - 2) % n, (n - rank - 2 + n) % n};
    for (uint32_t ring = 0; ring < 2; ring++) {
        const OrcSlice* s0 = &d->slices[ring][init0[ring]];
        const OrcSlice* s1 = &d->slices[ring][init1[ring]];
        emit(t, 0, K_COPY, rank, B_IN, s0->offset, rank, B_UIN, s0->offset, s0->size);
        emit(t, 0, K_COPY, rank, B_IN, s1->offset, rank, B_UIN, s1->offset, s1->size);
    }
    /* RunReduceScatter, :640-685 */
    uint32_t rx[2] = {(rank + n - 2) % n, (n - rank - 2 + n) % n};
    uint32_t sub[2] = {(rank + n - 3) % n, (n - rank - 3 + n) % n};
    for (uint32_t step = 0; step < n - 1; step++) {
        for (uint32_t ring = 0; ring < 2; ring++) {
            const OrcSlice* rx_slice = &d->slices[ring][rx[ring]];
            const OrcSlice* ccl_slice = &d->slices[ring][sub[ring]];
            /* ReducerRun, inline: the neighbour's input memory folded into the own, :476-480 */
            emit(t, 1 + step, K_REDUCE, rank, B_IN, rx_slice->offset, pre[ring], B_IN, rx_slice->offset, rx_slice->size);
            /* LocalMemcpy: next step's receive slice from the user input, :503-511, :518-522; none in the last step */
            if (step != n - 2)
                emit(t, 1 + step, K_COPY, rank, B_IN, ccl_slice->offset, rank, B_UIN, ccl_slice->offset, ccl_slice->size);
            rx[ring] = (rx[ring] + n - 1) % n;
            sub[ring] = (sub[ring] + n - 1) % n;
        }
    }
}

/* AlignedAllGatherDoubleRing::RunAsync for one rank, tpl/temp_all_gather/aligned_all_gather_double_ring.cc, as the
 * allreduce executor prepares it (coll_aligned_all_reduce_double_ring_for_910_93_executor.cc:112-122): input and output
 * memory = the CCL output buffer (so the init step copies nothing, :235-237), opInfo->outputAddr = the user output. */
static void prog_dbring_ag(OrcTrace* t, uint32_t rank, uint32_t n, const OrcDoubleRing* d)
{
    if (n == 1) { /* OneRankMemcpy, :119-153 */
        for (uint32_t ring = 0; ring < 2; ring++)
            emit(t, 0, K_COPY, 0, B_UOUT, d->slices[ring][0].offset, 0, B_OUT, d->slices[ring][0].offset, d->slices[ring][0].size);
        return;
    }
    const uint32_t pre[2] = {(rank + n - 1) % n, (rank + 1) % n};
    uint32_t tx[2] = {rank, (n - rank) % n};                     /* :411-414 */
    uint32_t rx[2] = {(rank + n - 1) % n, (n - rank - 1 + n) % n};
    for (uint32_t step = 0; step < n - 1; step++) {
        for (uint32_t ring = 0; ring < 2; ring++) {
            const OrcSlice* rx_slice = &d->slices[ring][rx[ring]];
            const OrcSlice* tx_slice = &d->slices[ring][tx[ring]];
            /* the received slice: into the CCL output, in the last step straight into the user output, :360-374 */
            emit(t, step, K_COPY, rank, step == n - 2 ? B_UOUT : B_OUT, rx_slice->offset, pre[ring], B_OUT, rx_slice->offset,
                 rx_slice->size);
            /* the slice sent in this step also goes to the user output, :376-385 */
            emit(t, step, K_COPY, rank, B_UOUT, tx_slice->offset, rank, B_OUT, tx_slice->offset, tx_slice->size);
            tx[ring] = (tx[ring] + n - 1) % n;
            rx[ring] = (rx[ring] + n - 1) % n;
        }
    }
}

/* CollAllReduceRingFor91093Executor::KernelRun (exec/coll_all_reduce/coll_all_reduce_ring_for_910_93_executor.cc:
 * 218-524) for one rank and one chunk, TOPO_TYPE_NP_DOUBLE_RING, DMAReduceFlag_ set (op-base mode,
 * coll_aligned_all_reduce_double_ring_for_910_93_executor.cc:20-24), one super pod (:298). */
static int prog_dbring_allreduce(OrcTrace* t, int alg1, uint32_t rank, uint32_t n_servers, uint32_t n_local, uint64_t count,
                                 int dtype, uint32_t level1_steps, uint32_t step0)
{
    const uint32_t unit = orc_dtype_size(dtype);
    const uint32_t server = rank / n_local, local = rank % n_local;
    uint32_t level0[ORC_MAX_RANKS], level1[ORC_MAX_RANKS];
    for (uint32_t j = 0; j < n_local; j++) level0[j] = server * n_local + j;
    for (uint32_t s = 0; s < n_servers; s++) level1[s] = s * n_local + local;
    OrcDoubleRing d;
    dbring_prepare(&d, count, unit, n_local);                  /* :229, :242 */
    const uint32_t rs_steps = n_local == 1 ? 1 : n_local;      /* the init step and n - 1 ring steps */
    g_rank_map = level0;
    g_step_base = step0;
    prog_dbring_rs(t, local, n_local, &d);                     /* :267-270 */
    /* PrepareLevel1CommInfo on 910_93: segment = local rank, hdSize = both rings' shares of it,
     * exec/coll_comm_executor.cc:2555-2559 */
    const uint64_t hd_count = d.seg[local].size / unit;        /* :296 */
    g_rank_map = level1;
    g_base_off = d.seg[local].offset;                          /* :299-301, :360 */
    g_step_base = step0 + rs_steps;
    run_template(t, hier_level1_template(alg1, count, unit, n_local), server, n_servers, hd_count, unit); /* :338-347 */
    g_base_off = 0;
    g_rank_map = level0;
    g_step_base = step0 + rs_steps + level1_steps;
    prog_dbring_ag(t, local, n_local, &d);                     /* :519-521 */
    g_rank_map = NULL;
    g_step_base = 0;
    return 0;
}

static int build_trace_dbring(OrcTrace* t, int alg1, uint32_t n_servers, uint32_t n_local, uint64_t count,
                              uint64_t ccl_bytes, int dtype)
{
    memset(t, 0, sizeof(*t));
    const uint32_t unit = orc_dtype_size(dtype);
    if (unit == 0 || n_servers == 0 || n_local == 0 || n_servers * n_local > ORC_MAX_RANKS) return -1;
    if (alg1 != ORC_ALG_ALLREDUCE_RING && alg1 != ORC_ALG_ALLREDUCE_NHR && alg1 != ORC_ALG_ALLREDUCE_NB) return -1; /* :304-351 */
    const uint64_t max_count = ccl_bytes / unit;               /* CalcLoopMaxCount, exec/coll_all_reduce/coll_all_reduce_executor.cc:129-138 */
    if (max_count == 0) return -1;
    /* RunLoop, exec/coll_all_reduce/coll_all_reduce_executor.cc:234-262; no staging copies with DMAReduceFlag_, :305-311, :326-331 */
    uint32_t step0 = 0;
    uint64_t cur_count = 0, user_off = 0;
    for (uint64_t count_left = count; count_left > 0; count_left -= cur_count) {
        cur_count = count_left > max_count ? max_count : count_left;
        OrcSlice seg[ORC_MAX_RANKS];
        orc_slices_ring(cur_count, unit, n_local, seg);
        uint32_t level1_steps = 0;
        for (uint32_t i = 0; i < n_local; i++) {
            uint32_t st = 0;
            const int rc = template_steps(hier_level1_template(alg1, cur_count, unit, n_local), n_servers, seg[i].size / unit, dtype, &st);
            if (rc) {
                free(t->ops);
                return rc;
            }
            if (st > level1_steps) level1_steps = st;
        }
        g_user_off = user_off;
        for (uint32_t r = 0; r < n_servers * n_local; r++) prog_dbring_allreduce(t, alg1, r, n_servers, n_local, cur_count, dtype, level1_steps, step0);
        g_user_off = 0;
        if (t->oom) {
            free(t->ops);
            return -2;
        }
        const uint32_t edge = n_local == 1 ? 1 : n_local - 1;
        step0 += (n_local == 1 ? 1 : n_local) + level1_steps + edge;
        user_off += cur_count * unit;
    }
    return sort_trace(t);
}

int64_t orc_trace_dbring(int alg1, uint32_t n_servers, uint32_t n_local, uint64_t count, uint64_t ccl_bytes, int dtype,
                         OrcOp* out, uint64_t cap)
{
    OrcTrace t;
    int rc = build_trace_dbring(&t, alg1, n_servers, n_local, count, ccl_bytes, dtype);
    if (rc) return rc;
    const uint64_t m = t.n < cap ? t.n : cap;
    if (out && m) memcpy(out, t.ops, m * sizeof(OrcOp));
    const int64_t total = (int64_t)t.n;
    free(t.ops);
    return total;
}

int orc_run_dbring(int alg1, uint32_t n_servers, uint32_t n_local, void* const* user_in, void* const* user_out,
                   void* const* ccl_in, void* const* ccl_out, uint64_t count, uint64_t ccl_bytes, int dtype, int op)
{
    OrcTrace t;
    int rc = build_trace_dbring(&t, alg1, n_servers, n_local, count, ccl_bytes, dtype);
    if (rc) return rc;
    void* const* bufs[5] = {ccl_in, ccl_out, NULL, user_in, user_out};
    rc = exec_trace(&t, bufs, dtype, op);
    free(t.ops);
    return rc;
}

/* the double-ring slice tables, for the tests: out[ring * n + position] */
int orc_dbring_slices(uint64_t count, int dtype, uint32_t n, OrcSlice* out, uint32_t* order)
{
    const uint32_t unit = orc_dtype_size(dtype);
    if (unit == 0 || n == 0 || n > ORC_MAX_RANKS) return -1;
    OrcDoubleRing d;
    dbring_prepare(&d, count, unit, n);
    for (uint32_t ring = 0; ring < 2; ring++)
        for (uint32_t i = 0; i < n; i++) {
            out[ring * n + i] = d.slices[ring][i];
            order[ring * n + i] = d.order[ring][i];
        }
    return 0;
}

/* ReduceScatterRecursiveHalvingDoubling::RunAsync for one rank, tpl/temp_reduce_scatter/reduce_scatter_recursive_hd.cc:
 * 29-84, on data_bytes of the input memory (count_ elements = rankSize slices): everything happens in the input memory
 * (the inner template is prepared with it as input and output, :223-225, so its closing copy, tpl/temp_reduce_scatter/
 * reduce_scatter_halving_doubling.cc:251-254, is a copy onto itself, which the dispatcher drops).  Returns the number of
 * lock-step steps. */
static uint32_t prog_rs_recursive_hd(OrcTrace* t, uint32_t rank, uint32_t n, uint64_t data_bytes)
{
    if (n == 1) return 0; /* :45-50 with inputMem_ == outputMem_ */
    /* CalcPartOneSizeAndBlockSize, tpl/recursive_halvingdoubling_base.cc:23-37 */
    uint32_t round = 0;
    while ((1u << round) <= n) round++;
    if (round >= 1) round -= 1;
    const uint32_t block = 1u << round;
    const uint32_t part1 = (n - block) * 2;
    uint32_t step = 0;
    /* ReduceInPartOne, :112-186: an even rank of part one folds the whole input of its odd neighbour into its own */
    if (part1 > 0) {
        if (rank < part1 && rank % 2 == 0) emit(t, step, K_REDUCE, rank, B_IN, 0, rank + 1, B_IN, 0, data_bytes);
        step++;
    }
    /* CalculateSlices, :86-110: per block rank; the first part1 / 2 of them carry two ranks' slices */
    OrcSlice sl[ORC_MAX_RANKS];
    const uint64_t bytes_per_slice = data_bytes / n;
    const uint32_t half_part1 = part1 / 2;
    uint32_t i = 0;
    while (i < half_part1) {
        sl[i].size = 2 * bytes_per_slice;
        sl[i].offset = (uint64_t)i * 2 * bytes_per_slice;
        i++;
    }
    while (i < block) {
        sl[i].size = bytes_per_slice;
        sl[i].offset = (uint64_t)i * bytes_per_slice + (uint64_t)half_part1 * bytes_per_slice;
        i++;
    }
    /* ReduceScatterInBlock, :188-236 */
    const int idle = (rank < part1 && rank % 2 == 1);
    uint32_t rib = 0;
    if (!idle) rib = (rank < part1) ? rank / 2 : rank - part1 / 2;
#define REAL(b) (((b) < part1 / 2) ? 2 * (b) : (b) + part1 / 2) /* BuildSubLinks, tpl/recursive_halvingdoubling_base.cc:39-62 */
    uint32_t steps = 0;
    while ((block >> (steps + 1)) != 0) steps++;
    for (uint32_t s = 0; s < steps; s++) { /* tpl/temp_reduce_scatter/reduce_scatter_halving_doubling.cc:65-92, 196-249 */
        if (!idle) {
            const uint32_t mask = 1u << (steps - s - 1);
            const uint32_t peer = rib ^ mask;
            const uint32_t id = rib & (~(mask - 1));
            uint64_t sz = 0;
            uint32_t num = mask;
            while (num > 0) {
                num--;
                sz += sl[id + num].size;
            }
            emit(t, step, K_REDUCE, rank, B_IN, sl[id].offset, REAL(peer), B_IN, sl[id].offset, sz);
        }
        step++;
    }
#undef REAL
    /* ScatterInPartOne, :238-300: the odd rank of part one receives its slice from the even neighbour's input */
    if (part1 > 0) {
        if (rank < part1 && rank % 2 == 1) {
            const uint64_t offset = (uint64_t)rank * bytes_per_slice;
            emit(t, step, K_COPY, rank, B_IN, offset, rank - 1, B_IN, offset, bytes_per_slice);
        }
        step++;
    }
    return step;
}

/* ---- the double-ring reduce-scatter executor on one server, op-base mode with DMA reduce ------------------------- */

/* CollAlignedReduceScatterDoubleRingFor91093Executor (exec/coll_reduce_scatter/
 * coll_aligned_reduce_scatter_double_ring_for_910_93_executor.cc:22-86; KernelRun of its base, exec/coll_reduce_scatter/
 * coll_reduce_scatter_ring_for_910_93_executor.cc:595-687) for one rank and one chunk on a single server: the slices of
 * ReduceScatterRingSlicePrepare (exec/coll_reduce_scatter/coll_reduce_scatter_executor.cc:491-535: blocks of the output
 * size, each cut in two shares by PrepareMultiRingSlice), the user-memory slices of CalUserMemDataSegsSlice (:297-313:
 * block index * count * unit + the ring's first slice offset), and AlignedReduceScatterDoubleRing with both user
 * addresses set (tpl/temp_reduce_scatter/aligned_reduce_scatter_double_ring.cc): the last reduce lands in the user output
 * at lastStepOffsets_ (:229-238, :452-458), which the step before initialises from the user input (:490-500). */
static void prog_dbring_rs_user_out(OrcTrace* t, uint32_t rank, uint32_t n, uint64_t cur_size, uint64_t stride_bytes)
{
    /* multiStreamSlice / level0DataSegsSlice */
    OrcSlice seg[ORC_MAX_RANKS], multi_seg[ORC_MAX_RANKS][2], slices[2][ORC_MAX_RANKS], user[2][ORC_MAX_RANKS];
    uint32_t order[2][ORC_MAX_RANKS];
    for (uint32_t i = 0; i < n; i++) {
        seg[i].size = cur_size;
        seg[i].offset = cur_size * i;
    }
    for (uint32_t rank_id = 0; rank_id < n; rank_id++) { /* MutliSegSlicePrepare, exec/coll_comm_executor.cc:2011-2052 */
        const uint64_t size_per_ring = ((seg[rank_id].size + 1) / 2 + 127) / 128 * 128;
        uint64_t residue = seg[rank_id].size;
        for (uint32_t ring = 0; ring < 2; ring++) {
            const uint64_t single = size_per_ring < residue ? size_per_ring : residue;
            multi_seg[rank_id][ring].size = single;
            multi_seg[rank_id][ring].offset = single ? seg[rank_id].offset + seg[rank_id].size - residue : seg[rank_id].offset;
            residue -= single;
        }
    }
    for (uint32_t i = 0; i < n; i++) order[0][i] = i;
    order[1][0] = 0;
    for (uint32_t i = 1; i < n; i++) order[1][i] = order[0][n - i];
    for (uint32_t ring = 0; ring < 2; ring++)
        for (uint32_t i = 0; i < n; i++) slices[ring][i] = multi_seg[order[ring][i]][ring];
    for (uint32_t ring = 0; ring < 2; ring++) /* CalUserMemDataSegsSlice, :297-313 */
        for (uint32_t i = 0; i < n; i++) {
            user[ring][i].size = slices[ring][i].size;
            user[ring][i].offset = (slices[ring][i].offset / cur_size) * stride_bytes + slices[ring][0].offset;
        }
    /* SetSlices, :190-240: ringsOrders_ = the positions of each ring's devices in ring 0 = the orders themselves */
    uint64_t last_step_offset[2];
    last_step_offset[0] = slices[0][order[0][0]].offset;
    last_step_offset[1] = slices[1][order[1][rank]].offset - slices[0][order[0][rank]].offset;

    const uint32_t pre[2] = {(rank + n - 1) % n, (rank + 1) % n};
    const uint32_t init0[2] = {(rank + n - 1) % n, (n - rank - 1 + n) % n};
    const uint32_t init1[2] = {(rank + n - 2) % n, (n - rank - 2 + n) % n};
    for (uint32_t ring = 0; ring < 2; ring++) { /* RunInitStep, :379-412 (rankSize > 2) */
        emit(t, 0, K_COPY, rank, B_IN, slices[ring][init0[ring]].offset, rank, B_UIN, user[ring][init0[ring]].offset,
             slices[ring][init0[ring]].size);
        emit(t, 0, K_COPY, rank, B_IN, slices[ring][init1[ring]].offset, rank, B_UIN, user[ring][init1[ring]].offset,
             slices[ring][init1[ring]].size);
    }
    uint32_t rx[2] = {(rank + n - 2) % n, (n - rank - 2 + n) % n};
    uint32_t sub[2] = {(rank + n - 3) % n, (n - rank - 3 + n) % n};
    for (uint32_t step = 0; step < n - 1; step++) {
        for (uint32_t ring = 0; ring < 2; ring++) {
            const OrcSlice* rx_slice = &slices[ring][rx[ring]];
            const OrcSlice* ccl_slice = &slices[ring][sub[ring]];
            const OrcSlice* sub_slice = &user[ring][sub[ring]];
            if (step == n - 2) /* :452-458 */
                emit(t, 1 + step, K_REDUCE, rank, B_UOUT, last_step_offset[ring], pre[ring], B_IN, rx_slice->offset, rx_slice->size);
            else
                emit(t, 1 + step, K_REDUCE, rank, B_IN, rx_slice->offset, pre[ring], B_IN, rx_slice->offset, rx_slice->size);
            if (step == n - 2) {
                /* :487-489 */
            } else if (step == n - 3) { /* :490-500 */
                emit(t, 1 + step, K_COPY, rank, B_UOUT, last_step_offset[ring], rank, B_UIN, sub_slice->offset, sub_slice->size);
            } else { /* :501-511 */
                emit(t, 1 + step, K_COPY, rank, B_IN, ccl_slice->offset, rank, B_UIN, sub_slice->offset, ccl_slice->size);
            }
            rx[ring] = (rx[ring] + n - 1) % n;
            sub[ring] = (sub[ring] + n - 1) % n;
        }
    }
}

static int build_trace_dbring_rs(OrcTrace* t, uint32_t n, uint64_t count, uint64_t ccl_bytes, int dtype)
{
    memset(t, 0, sizeof(*t));
    const uint32_t unit = orc_dtype_size(dtype);
    /* two ranks take a first step of their own in the template (:353-360) that does not hold together; the double-ring
     * topologies have more */
    if (unit == 0 || n < 3 || n > ORC_MAX_RANKS) return -1;
    const uint64_t max_count = ccl_bytes / n / 128u * 128u / unit; /* CalcLoopMaxCount, coll_reduce_scatter_ring_for_910_93_executor.cc:167-173 */
    if (max_count == 0) return -1;
    uint32_t step0 = 0;
    uint64_t cur_count = 0, user_off = 0;
    for (uint64_t count_left = count; count_left > 0; count_left -= cur_count) {
        cur_count = count_left > max_count ? max_count : count_left;
        g_user_off = user_off;
        g_step_base = step0;
        for (uint32_t r = 0; r < n; r++) prog_dbring_rs_user_out(t, r, n, cur_count * unit, count * unit);
        g_user_off = 0;
        g_step_base = 0;
        if (t->oom) {
            free(t->ops);
            return -2;
        }
        step0 += n;
        user_off += cur_count * unit;
    }
    return sort_trace(t);
}

int64_t orc_trace_dbring_rs(uint32_t n, uint64_t count, uint64_t ccl_bytes, int dtype, OrcOp* out, uint64_t cap)
{
    OrcTrace t;
    int rc = build_trace_dbring_rs(&t, n, count, ccl_bytes, dtype);
    if (rc) return rc;
    const uint64_t m = t.n < cap ? t.n : cap;
    if (out && m) memcpy(out, t.ops, m * sizeof(OrcOp));
    const int64_t total = (int64_t)t.n;
    free(t.ops);
    return total;
}

int orc_run_dbring_rs(uint32_t n, void* const* user_in, void* const* user_out, void* const* ccl_in, uint64_t count,
                      uint64_t ccl_bytes, int dtype, int op)
{
    OrcTrace t;
    int rc = build_trace_dbring_rs(&t, n, count, ccl_bytes, dtype);
    if (rc) return rc;
    void* const* bufs[5] = {ccl_in, NULL, NULL, user_in, user_out};
    rc = exec_trace(&t, bufs, dtype, op);
    free(t.ops);
    return rc;
}

/* ---- the double-ring reduce-scatter executor over servers and super pods, op-base mode with DMA reduce ---------- */

/* The level-1 / level-2 templates with `per` slices per rank (the slice vector holds n * per entries, rank i's at
 * i * per ..): ReduceScatterRing (tpl/temp_reduce_scatter/reduce_scatter_ring.cc:204-304), ReduceScatterNHR
 * (reduce_scatter_nhr.cc:408-488 with the step table of :552-593) and ReduceScatterNB (reduce_scatter_nb.cc:143-230)
 * walk the slices of a slice index one after the other wherever the single-slice case touches one slice; input and
 * output memory are the same, inline reduce, nothing merged. */
static void prog_ring_rs_multi(OrcTrace* t, uint32_t rank, uint32_t n, const OrcSlice* sl, uint32_t per)
{
    const uint32_t left = (rank + n - 1) % n;
    uint32_t rx = (rank + n - 2) % n;
    uint32_t step = 0;
    for (uint32_t i = 0; i < n - 2; i++) { /* :232-283 */
        for (uint32_t j = 0; j < per; j++)
            emit(t, step, K_REDUCE, rank, B_IN, sl[rx * per + j].offset, left, B_IN, sl[rx * per + j].offset, sl[rx * per + j].size);
        step++;
        rx = (rx + n - 1) % n;
    }
    for (uint32_t j = 0; j < per; j++) /* :288-304 */
        emit(t, step, K_REDUCE, rank, B_IN, sl[rank * per + j].offset, left, B_IN, sl[rank * per + j].offset, sl[rank * per + j].size);
}

static void prog_nhr_rs_multi(OrcTrace* t, uint32_t rank, uint32_t n, const OrcSlice* sl, uint32_t per, const uint32_t* slice_map)
{
    const uint32_t n_steps = nhr_steps(n);
    for (uint32_t step = 0; step < n_steps; step++) {
        const uint32_t delta_rank = 1u << step;
        const uint32_t recv_from = (rank + delta_rank) % n;
        const uint32_t n_slices = (n - 1 + (1u << step)) / (1u << (step + 1));
        const uint32_t delta_slice = 1u << (step + 1);
        uint32_t rx_idx = rank;
        for (uint32_t i = 0; i < n_slices; i++) { /* :570-587 */
            for (uint32_t j = 0; j < per; j++) {
                const OrcSlice s = sl[slice_map[rx_idx] * per + j];
                emit(t, step, K_REDUCE, rank, B_IN, s.offset, recv_from, B_IN, s.offset, s.size);
            }
            rx_idx = (rx_idx + n - delta_slice) % n;
        }
    }
}

static void prog_nb_rs_multi(OrcTrace* t, uint32_t rank, uint32_t n, const OrcSlice* sl, uint32_t per)
{
    const uint32_t n_steps = nhr_steps(n);
    for (uint32_t step = 0; step < n_steps; step++) {
        const uint32_t delta_rank = 1u << step;
        const uint32_t recv_from = (n + rank - delta_rank) % n;
        const uint32_t n_slices = (n - 1 + (1u << step)) / (1u << (step + 1));
        const uint32_t delta_slice = 1u << (step + 1);
        uint32_t rx_idx = rank;
        for (uint32_t i = 0; i < n_slices; i++) {
            for (uint32_t j = 0; j < per; j++) {
                const OrcSlice s = sl[rx_idx * per + j];
                emit(t, step, K_REDUCE, rank, B_IN, s.offset, recv_from, B_IN, s.offset, s.size);
            }
            rx_idx = (rx_idx + delta_slice) % n;
        }
    }
}

static uint32_t level_steps(int alg, uint32_t n) { return n < 2 ? 0 : (alg == ORC_ALG_RS_RING_STAGE ? n - 1 : nhr_steps(n)); }

static void prog_level_rs(OrcTrace* t, int alg, uint32_t rank, uint32_t n, const OrcSlice* sl, uint32_t per)
{
    if (alg == ORC_ALG_RS_RING_STAGE) {
        prog_ring_rs_multi(t, rank, n, sl, per);
    } else if (alg == ORC_ALG_RS_NB) {
        prog_nb_rs_multi(t, rank, n, sl, per);
    } else {
        uint32_t slice_map[ORC_MAX_RANKS];
        nhr_rank_mapping(n, 1, slice_map);
        prog_nhr_rs_multi(t, rank, n, sl, per, slice_map); /* Prepare(reduceAttr, false) */
    }
}

/* CollAlignedReduceScatterDoubleRingFor91093Executor with level1RankSize = n_servers and level2RankSize = n_pods, more
 * than one rank between them, for one rank and one chunk (KernelRun of its base, exec/coll_reduce_scatter/
 * coll_reduce_scatter_ring_for_910_93_executor.cc:595-812); rank = (pod * n_servers + server) * n_local + local index:
 *   level 0: every ring position carries n_pods * n_servers slices (FillMultiRingSlice :213-233: the position's share
 *     + level1Idx * sliceNum * output size + level2Idx * sliceNum * level1RankSize * output size, level2Idx the outer
 *     loop), their user-memory twins at block index * count * unit + the ring's first slice offset (:297-313), and
 *     AlignedReduceScatterDoubleRing runs with the user input address only (:664-670: outputAddr = nullptr), so every
 *     fold stays in the CCL input buffer (tpl/temp_reduce_scatter/aligned_reduce_scatter_double_ring.cc: the init step
 *     walks the slices of a position, :305-332 and :232-249; so does every step, :366-425, :583-590);
 *   level 1 (n_servers > 1): reduce-scatter between the servers of the pod (ring, NHR or NB, :689-746) in place on the
 *     CCL input buffer; the i-th server's rank owns one slice per pod, the block of the rank with its place in that pod
 *     (CalLevel1DataSegsSlice :327-350);
 *   level 2 (n_pods > 1): reduce-scatter between the pods (:748-797), slice i = the block of the i-th pod's rank with
 *     this place (CalLevel2DataSegsSlice :376-382);
 *   last: the own block from the CCL input to the user output (:800-808).
 * Steps: 0 the init step, 1 .. n_local - 1 the ring steps, then the level-1 steps, the level-2 steps, the copy out. */
static void prog_dbring_rs_servers(OrcTrace* t, int alg1, int alg2, uint32_t rank, uint32_t n_pods, uint32_t n_servers,
                                   uint32_t n_local, uint64_t cur_size, uint64_t stride_bytes, uint32_t step0)
{
    const uint32_t n = n_local, per = n_servers * n_pods;
    const uint32_t local = rank % n_local, server = rank / n_local % n_servers, pod = rank / n_local / n_servers;
    uint32_t level0[ORC_MAX_RANKS], level1[ORC_MAX_RANKS], level2[ORC_MAX_RANKS];
    for (uint32_t j = 0; j < n_local; j++) level0[j] = (pod * n_servers + server) * n_local + j;
    for (uint32_t s = 0; s < n_servers; s++) level1[s] = (pod * n_servers + s) * n_local + local;
    for (uint32_t p = 0; p < n_pods; p++) level2[p] = (p * n_servers + server) * n_local + local;

    /* multiStreamSlice: ReduceScatterRingSlicePrepare with sliceNum = n_local, as on one server */
    OrcSlice seg[ORC_MAX_RANKS], multi_seg[ORC_MAX_RANKS][2], ms[2][ORC_MAX_RANKS];
    uint32_t order[2][ORC_MAX_RANKS];
    for (uint32_t i = 0; i < n; i++) {
        seg[i].size = cur_size;
        seg[i].offset = cur_size * i;
    }
    for (uint32_t rank_id = 0; rank_id < n; rank_id++) { /* MutliSegSlicePrepare, exec/coll_comm_executor.cc:2011-2052 */
        const uint64_t size_per_ring = ((seg[rank_id].size + 1) / 2 + 127) / 128 * 128;
        uint64_t residue = seg[rank_id].size;
        for (uint32_t ring = 0; ring < 2; ring++) {
            const uint64_t single = size_per_ring < residue ? size_per_ring : residue;
            multi_seg[rank_id][ring].size = single;
            multi_seg[rank_id][ring].offset = single ? seg[rank_id].offset + seg[rank_id].size - residue : seg[rank_id].offset;
            residue -= single;
        }
    }
    for (uint32_t i = 0; i < n; i++) order[0][i] = i;
    order[1][0] = 0;
    for (uint32_t i = 1; i < n; i++) order[1][i] = order[0][n - i];
    for (uint32_t ring = 0; ring < 2; ring++)
        for (uint32_t i = 0; i < n; i++) ms[ring][i] = multi_seg[order[ring][i]][ring];
    /* level0DataSegsSlice and multRingsUserMemSlice: index = ring position * per + level2Idx * n_servers + level1Idx */
    OrcSlice* ccl[2] = {NULL, NULL};
    OrcSlice* user[2] = {NULL, NULL};
    for (uint32_t ring = 0; ring < 2; ring++) {
        ccl[ring] = (OrcSlice*)malloc(sizeof(OrcSlice) * n * per);
        user[ring] = (OrcSlice*)malloc(sizeof(OrcSlice) * n * per);
        if (!ccl[ring] || !user[ring]) {
            t->oom = 1;
            for (uint32_t q = 0; q < 2; q++) {
                free(ccl[q]);
                free(user[q]);
            }
            return;
        }
        for (uint32_t level0_idx = 0; level0_idx < n; level0_idx++)
            for (uint32_t level2_idx = 0; level2_idx < n_pods; level2_idx++)
                for (uint32_t level1_idx = 0; level1_idx < n_servers; level1_idx++) {
                    const uint32_t at = level0_idx * per + level2_idx * n_servers + level1_idx;
                    OrcSlice* c = &ccl[ring][at];
                    c->size = ms[ring][level0_idx].size;
                    c->offset = ms[ring][level0_idx].offset + (uint64_t)level1_idx * n * cur_size +
                                (uint64_t)level2_idx * n * n_servers * cur_size;
                    OrcSlice* u = &user[ring][at];
                    u->size = c->size;
                    u->offset = (c->offset / cur_size) * stride_bytes + ms[ring][0].offset;
                }
    }

    g_rank_map = level0;
    g_step_base = step0;
    const uint32_t pre[2] = {(local + n - 1) % n, (local + 1) % n};
    const uint32_t init0[2] = {(local + n - 1) % n, (n - local - 1 + n) % n};
    const uint32_t init1[2] = {(local + n - 2) % n, (n - local - 2 + n) % n};
    for (uint32_t k = 0; k < per; k++)      /* RunInitStep, :305-332 */
        for (uint32_t ring = 0; ring < 2; ring++) {
            const uint32_t a = init0[ring] * per + k, b = init1[ring] * per + k;
            emit(t, 0, K_COPY, local, B_IN, ccl[ring][a].offset, local, B_UIN, user[ring][a].offset, ccl[ring][a].size);
            emit(t, 0, K_COPY, local, B_IN, ccl[ring][b].offset, local, B_UIN, user[ring][b].offset, ccl[ring][b].size);
        }
    uint32_t rx[2] = {(local + n - 2) % n, (n - local - 2 + n) % n};
    uint32_t sub[2] = {(local + n - 3) % n, (n - local - 3 + n) % n};
    for (uint32_t step = 0; step < n - 1; step++) { /* RunReduceScatter, :640-685 */
        for (uint32_t ring = 0; ring < 2; ring++) {
            for (uint32_t k = 0; k < per; k++) { /* PrepareDeviceMems, :371-425, outputAddr == nullptr */
                const OrcSlice* rx_slice = &ccl[ring][rx[ring] * per + k];
                const OrcSlice* ccl_slice = &ccl[ring][sub[ring] * per + k];
                const OrcSlice* sub_slice = &user[ring][sub[ring] * per + k];
                emit(t, 1 + step, K_REDUCE, local, B_IN, rx_slice->offset, pre[ring], B_IN, rx_slice->offset, rx_slice->size);
                if (step != n - 2)
                    emit(t, 1 + step, K_COPY, local, B_IN, ccl_slice->offset, local, B_UIN, sub_slice->offset, ccl_slice->size);
            }
            rx[ring] = (rx[ring] + n - 1) % n;
            sub[ring] = (sub[ring] + n - 1) % n;
        }
    }
    for (uint32_t ring = 0; ring < 2; ring++) {
        free(ccl[ring]);
        free(user[ring]);
    }

    uint32_t step = step0 + n;
    if (n_servers > 1) { /* between the servers, :689-746 */
        OrcSlice sl[ORC_MAX_RANKS];
        const uint32_t ranks_per_pod = n_servers * n_local;
        for (uint32_t i = 0; i < n_servers; i++) /* CalLevel1DataSegsSlice, :327-350 */
            for (uint32_t level2_idx = 0; level2_idx < n_pods; level2_idx++) {
                OrcSlice* x = &sl[i * n_pods + level2_idx];
                x->size = cur_size;
                x->offset = n_pods <= 1 ? (uint64_t)level1[i] * cur_size
                                        : (uint64_t)(level1[i] % ranks_per_pod) * cur_size + (uint64_t)level2_idx * ranks_per_pod * cur_size;
            }
        g_rank_map = level1;
        g_step_base = step;
        prog_level_rs(t, alg1, server, n_servers, sl, n_pods);
        step += level_steps(alg1, n_servers);
    }
    if (n_pods > 1) { /* between the super pods, :748-797 */
        OrcSlice sl[ORC_MAX_RANKS];
        for (uint32_t i = 0; i < n_pods; i++) { /* CalLevel2DataSegsSlice, :376-382 */
            sl[i].size = cur_size;
            sl[i].offset = (uint64_t)level2[i] * cur_size;
        }
        g_rank_map = level2;
        g_step_base = step;
        prog_level_rs(t, alg2, pod, n_pods, sl, 1);
        step += level_steps(alg2, n_pods);
    }
    g_rank_map = NULL;
    /* :800-808: CalcSrcMemOffset = userRank * output size */
    g_step_base = step;
    emit(t, 0, K_COPY, rank, B_UOUT, 0, rank, B_IN, (uint64_t)rank * cur_size, cur_size);
    g_step_base = 0;
}

static int level_alg_ok(int alg) { return alg == ORC_ALG_RS_RING_STAGE || alg == ORC_ALG_RS_NHR || alg == ORC_ALG_RS_NB; }

static int build_trace_dbring_rs_servers(OrcTrace* t, int alg1, int alg2, uint32_t n_pods, uint32_t n_servers, uint32_t n_local,
                                         uint64_t count, uint64_t ccl_bytes, int dtype)
{
    memset(t, 0, sizeof(*t));
    const uint32_t unit = orc_dtype_size(dtype);
    if (unit == 0 || n_pods == 0 || n_servers == 0 || n_pods * n_servers < 2 || n_local < 3 ||
        (uint64_t)n_pods * n_servers * n_local > ORC_MAX_RANKS)
        return -1;
    if (!level_alg_ok(alg1) || !level_alg_ok(alg2)) return -1;
    const uint32_t n = n_pods * n_servers * n_local;
    const uint64_t max_count = ccl_bytes / n / 128u * 128u / unit; /* CalcLoopMaxCount, :167-173 */
    if (max_count == 0) return -1;
    uint32_t step0 = 0;
    uint64_t cur_count = 0, user_off = 0;
    for (uint64_t count_left = count; count_left > 0; count_left -= cur_count) {
        cur_count = count_left > max_count ? max_count : count_left;
        g_user_off = user_off;
        for (uint32_t r = 0; r < n; r++)
            prog_dbring_rs_servers(t, alg1, alg2, r, n_pods, n_servers, n_local, cur_count * unit, count * unit, step0);
        g_user_off = 0;
        if (t->oom) {
            free(t->ops);
            return -2;
        }
        step0 += n_local + level_steps(alg1, n_servers) + level_steps(alg2, n_pods) + 1;
        user_off += cur_count * unit;
    }
    return sort_trace(t);
}

int64_t orc_trace_dbring_rs_servers(int alg1, int alg2, uint32_t n_pods, uint32_t n_servers, uint32_t n_local, uint64_t count,
                                    uint64_t ccl_bytes, int dtype, OrcOp* out, uint64_t cap)
{
    OrcTrace t;
    int rc = build_trace_dbring_rs_servers(&t, alg1, alg2, n_pods, n_servers, n_local, count, ccl_bytes, dtype);
    if (rc) return rc;
    const uint64_t m = t.n < cap ? t.n : cap;
    if (out && m) memcpy(out, t.ops, m * sizeof(OrcOp));
    const int64_t total = (int64_t)t.n;
    free(t.ops);
    return total;
}

int orc_run_dbring_rs_servers(int alg1, int alg2, uint32_t n_pods, uint32_t n_servers, uint32_t n_local, void* const* user_in,
                              void* const* user_out, void* const* ccl_in, uint64_t count, uint64_t ccl_bytes, int dtype, int op)
{
    OrcTrace t;
    int rc = build_trace_dbring_rs_servers(&t, alg1, alg2, n_pods, n_servers, n_local, count, ccl_bytes, dtype);
    if (rc) return rc;
    void* const* bufs[5] = {ccl_in, NULL, NULL, user_in, user_out};
    rc = exec_trace(&t, bufs, dtype, op);
    free(t.ops);
    return rc;
}

/* ---- the ring and mesh reduce-scatter executors over two communicator levels, op-base mode ---------------------- */

/* CollReduceScatterRingExecutor::KernelRun (exec/coll_reduce_scatter/coll_reduce_scatter_ring_executor.cc:136-363, one
 * ring, every device with a NIC) or CollReduceScatterMeshExecutor::KernelRun (exec/coll_reduce_scatter/
 * coll_reduce_scatter_mesh_executor.cc:131-259, without atomic adds) for one rank and one chunk, between the copies of
 * CollReduceScatterExecutor::RunLoopInner (exec/coll_reduce_scatter/coll_reduce_scatter_executor.cc:258-298). */
static void prog_hier_rs(OrcTrace* t, int level0_mesh, int alg1, uint32_t rank, uint32_t n_servers, uint32_t n_local,
                         uint64_t total_count, uint64_t cur_count, uint32_t unit, uint32_t step0)
{
    const uint32_t n = n_servers * n_local;
    const uint32_t server = rank / n_local, local = rank % n_local;
    const uint64_t cur_size = cur_count * unit;
    uint32_t level0[ORC_MAX_RANKS], level1[ORC_MAX_RANKS];
    for (uint32_t j = 0; j < n_local; j++) level0[j] = server * n_local + j;
    for (uint32_t s = 0; s < n_servers; s++) level1[s] = s * n_local + local;
    g_rank_map = NULL;
    g_base_off = 0;
    g_step_base = step0;
    /* user input -> CCL input, coll_reduce_scatter_executor.cc:258-276 */
    if (total_count == cur_count) {
        emit(t, 0, K_COPY, rank, B_IN, 0, rank, B_UIN, 0, total_count * unit * n);
    } else {
        for (uint32_t i = 0; i < n; i++)
            emit(t, 0, K_COPY, rank, B_IN, cur_size * i, rank, B_UIN, total_count * unit * i, cur_size);
    }
    uint32_t step = step0 + 1;
    /* first: between the servers, :183-247 / :146-205; input memory = scratch of nothing, in place; slices default to
     * count * unit at i * count * unit (tpl/temp_reduce_scatter/reduce_scatter_ring.cc:140-157, reduce_scatter_nhr.cc:
     * 57-75, reduce_scatter_nb.cc) with count = inputMem.size() / level1RankSize / unit */
    if (n_servers > 1) {
        OrcSlice sl[ORC_MAX_RANKS];
        const uint64_t ring_size = cur_size * n / n_servers;
        for (uint32_t i = 0; i < n_servers; i++) {
            sl[i].size = ring_size;
            sl[i].offset = (uint64_t)i * ring_size;
        }
        g_rank_map = level1;
        g_step_base = step;
        if (alg1 == ORC_ALG_RS_RING_STAGE) {
            prog_ring_rs(t, server, n_servers, sl, NULL);
            step += n_servers - 1;
        } else if (alg1 == ORC_ALG_RS_NHR) {
            uint32_t slice_map[ORC_MAX_RANKS];
            nhr_rank_mapping(n_servers, 1, slice_map); /* GetRankMapping(rankSize, true), reduce_scatter_nhr.cc:86-88 */
            prog_nhr_rs(t, server, n_servers, sl, NULL, slice_map, 0);
            step += nhr_steps(n_servers);
        } else if (alg1 == ORC_ALG_RS_NB) {
            prog_nb_rs(t, server, n_servers, sl, NULL);
            step += nhr_steps(n_servers);
        } else { /* the default branch: recursive halving-doubling over inputMem.size() / unit elements, :236-246 / :193-203 */
            step += prog_rs_recursive_hd(t, server, n_servers, cur_size * n);
        }
    }
    /* second: inside the server, :249-357 / :207-252, on the server's run of the CCL input at base offset
     * serverSliceOffset, slices of the output size (ReduceScatterRingSlicePrepare, coll_reduce_scatter_executor.cc:
     * 491-503 / PrepareReduceScatterSliceData, exec/coll_comm_executor.cc:1906-1919) */
    const uint64_t server_slice_size = cur_size * n / n_servers;
    OrcSlice seg[ORC_MAX_RANKS];
    for (uint32_t i = 0; i < n_local; i++) {
        seg[i].size = cur_size;
        seg[i].offset = cur_size * i;
    }
    g_rank_map = level0;
    g_base_off = server_slice_size * server;
    g_step_base = step;
    if (level0_mesh) prog_mesh_rs_streams(t, local, n_local, seg);
    else if (n_local > 1) prog_ring_rs(t, local, n_local, seg, NULL);
    step += n_local - 1;
    g_rank_map = NULL;
    g_base_off = 0;
    /* :359 / :255: the own block to the output memory */
    g_step_base = step;
    emit(t, 0, K_COPY, rank, B_OUT, 0, rank, B_IN, server_slice_size * server + seg[local].offset, cur_size);
    /* coll_reduce_scatter_executor.cc:293-298 */
    g_step_base = step + 1;
    emit(t, 0, K_COPY, rank, B_UOUT, 0, rank, B_OUT, 0, cur_size);
    g_step_base = 0;
}

static int build_trace_hier_rs(OrcTrace* t, int level0_mesh, int alg1, uint32_t n_servers, uint32_t n_local, uint64_t count,
                               uint64_t ccl_bytes, int dtype)
{
    memset(t, 0, sizeof(*t));
    const uint32_t unit = orc_dtype_size(dtype);
    if (unit == 0 || n_servers == 0 || n_local == 0 || n_servers * n_local > ORC_MAX_RANKS) return -1;
    if (level0_mesh && n_local < 2) return -1;
    if (alg1 != ORC_ALG_RS_RING_STAGE && alg1 != ORC_ALG_RS_NHR && alg1 != ORC_ALG_RS_NB && alg1 != ORC_ALG_RS_RHD) return -1;
    const uint32_t n = n_servers * n_local;
    const uint64_t max_count = ccl_bytes / ((uint64_t)n * unit); /* CalcLoopMaxCount of both executors, :116-121 */
    if (max_count == 0) return -1;
    uint32_t level1_steps = n_servers == 1 ? 0 : (alg1 == ORC_ALG_RS_RING_STAGE ? n_servers - 1 : nhr_steps(n_servers));
    if (alg1 == ORC_ALG_RS_RHD && n_servers > 1) {
        OrcTrace dry;
        memset(&dry, 0, sizeof(dry));
        level1_steps = prog_rs_recursive_hd(&dry, 0, n_servers, 0); /* zero-sized operations are not recorded */
        free(dry.ops);
    }
    uint32_t step0 = 0;
    uint64_t cur_count = 0, user_off = 0;
    for (uint64_t count_left = count; count_left > 0; count_left -= cur_count) {
        cur_count = count_left > max_count ? max_count : count_left;
        g_user_off = user_off;
        for (uint32_t r = 0; r < n; r++) prog_hier_rs(t, level0_mesh, alg1, r, n_servers, n_local, count, cur_count, unit, step0);
        g_user_off = 0;
        if (t->oom) {
            free(t->ops);
            return -2;
        }
        step0 += 1 + level1_steps + (n_local - 1) + 2;
        user_off += cur_count * unit;
    }
    return sort_trace(t);
}

int64_t orc_trace_hier_rs(int level0_mesh, int alg1, uint32_t n_servers, uint32_t n_local, uint64_t count, uint64_t ccl_bytes,
                          int dtype, OrcOp* out, uint64_t cap)
{
    OrcTrace t;
    int rc = build_trace_hier_rs(&t, level0_mesh, alg1, n_servers, n_local, count, ccl_bytes, dtype);
    if (rc) return rc;
    const uint64_t m = t.n < cap ? t.n : cap;
    if (out && m) memcpy(out, t.ops, m * sizeof(OrcOp));
    const int64_t total = (int64_t)t.n;
    free(t.ops);
    return total;
}

int orc_run_hier_rs(int level0_mesh, int alg1, uint32_t n_servers, uint32_t n_local, void* const* user_in,
                    void* const* user_out, void* const* ccl_in, void* const* ccl_out, uint64_t count, uint64_t ccl_bytes,
                    int dtype, int op)
{
    OrcTrace t;
    int rc = build_trace_hier_rs(&t, level0_mesh, alg1, n_servers, n_local, count, ccl_bytes, dtype);
    if (rc) return rc;
    void* const* bufs[5] = {ccl_in, ccl_out, NULL, user_in, user_out};
    rc = exec_trace(&t, bufs, dtype, op);
    free(t.ops);
    return rc;
}

/* ---- the order-preserving reduce-scatter executor (one server, op-base mode) ----------------------------------- */

/* ReduceScatterPlantLocalReduce::RunAsync for one rank and one group, tpl/temp_reduce_scatter/
 * reduce_scatter_plant_local_reduce.cc:106-164, as CollReduceScatterOrderPreservedExecutor::RunReduceScatterLevel0
 * prepares it for a single module (exec/coll_reduce_scatter/coll_reduce_scatter_order_preserved_executor.cc:181-216):
 * every block cur_size bytes, block d of the user input at d * stride bytes, slot d of the CCL output buffer at
 * d * cur_size, all2allOffset 0, no borrowed space.  Steps: 0 the all-to-all, 1.. the local reduce rounds. */
static void prog_plant_local_reduce(OrcTrace* t, uint32_t local_rank, uint32_t rank_size, uint64_t cur_size, uint64_t stride)
{
    const uint32_t all2all_offset = 0;
#define CALC_OUTPUT_INDEX(round) ((all2all_offset + (round) + local_rank) % rank_size) /* :90-93 */
    /* LocalCopy, :166-185 */
    emit(t, 0, K_COPY, local_rank, B_OUT, cur_size * CALC_OUTPUT_INDEX(local_rank), local_rank, B_UIN, stride * local_rank,
         cur_size);
    /* RunAlltoAll, :211-240: block `round` of the own user input planted into rank `round`'s output memory */
    for (uint32_t round = 0; round < rank_size; round++) {
        if (round == local_rank) continue;
        emit(t, 0, K_COPY, round, B_OUT, cur_size * CALC_OUTPUT_INDEX(round), local_rank, B_UIN, stride * round, cur_size);
    }
    /* RunLocalReduce, :336-407 */
    uint32_t reduce_step = 0;
    while ((1u << reduce_step) < rank_size) reduce_step++; /* ceil(log2(rankSize)) */
    for (uint32_t round = 0; round < reduce_step; round++) {
        const uint32_t full = 1u << (reduce_step - round);
        const uint32_t tail_index = (rank_size < full ? rank_size : full) - 1;
        const uint32_t head_index = 1u << (reduce_step - round - 1);
        for (uint32_t offset = 0; offset <= tail_index - head_index; offset++) {
            const uint32_t input_index = CALC_OUTPUT_INDEX(head_index + offset);
            const uint32_t output_index = CALC_OUTPUT_INDEX(offset);
            emit(t, 1 + round, K_REDUCE, local_rank, B_OUT, cur_size * output_index, local_rank, B_OUT, cur_size * input_index,
                 cur_size);
        }
    }
#undef CALC_OUTPUT_INDEX
}

/* CollReduceScatterOrderPreservedExecutor::KernelRun for one rank inside CollReduceScatterExecutor::RunLoop
 * (exec/coll_reduce_scatter/coll_reduce_scatter_order_preserved_executor.cc:260-283 with DMAReduceFlag_, :19;
 * exec/coll_reduce_scatter/coll_reduce_scatter_executor.cc:149-220): one module, the plant branch. */
static int build_trace_order_preserved(OrcTrace* t, uint32_t n, uint64_t count, uint64_t ccl_bytes, int dtype)
{
    memset(t, 0, sizeof(*t));
    const uint32_t unit = orc_dtype_size(dtype);
    /* one rank per module takes RunReduceScatterLevel0SingleRank (:134-150), which relies on the level-1 stage that a
     * single module does not have: not restated */
    if (unit == 0 || n < 2 || n > ORC_MAX_RANKS) return -1;
    const uint64_t max_count = ccl_bytes / n / 128u * 128u / unit; /* CalcLoopMaxCount, coll_reduce_scatter_executor.cc:124-134 */
    if (max_count == 0) return -1;
    uint32_t reduce_step = 0;
    while ((1u << reduce_step) < n) reduce_step++;
    uint32_t step0 = 0;
    uint64_t cur_count = 0, user_off = 0;
    for (uint64_t count_left = count; count_left > 0; count_left -= cur_count) {
        cur_count = count_left > max_count ? max_count : count_left;
        const uint64_t cur_size = cur_count * unit;
        g_user_off = user_off;
        for (uint32_t r = 0; r < n; r++) {
            g_step_base = step0;
            prog_plant_local_reduce(t, r, n, cur_size, count * unit);
            /* :273-279: the own slot of the scratch (= CCL output) memory to the user output */
            g_step_base = step0 + 1 + reduce_step;
            emit(t, 0, K_COPY, r, B_UOUT, 0, r, B_OUT, cur_size * r, cur_size);
        }
        g_user_off = 0;
        g_step_base = 0;
        if (t->oom) {
            free(t->ops);
            return -2;
        }
        step0 += 2 + reduce_step;
        user_off += cur_size;
    }
    return sort_trace(t);
}

int64_t orc_trace_order_preserved(uint32_t n, uint64_t count, uint64_t ccl_bytes, int dtype, OrcOp* out, uint64_t cap)
{
    OrcTrace t;
    int rc = build_trace_order_preserved(&t, n, count, ccl_bytes, dtype);
    if (rc) return rc;
    const uint64_t m = t.n < cap ? t.n : cap;
    if (out && m) memcpy(out, t.ops, m * sizeof(OrcOp));
    const int64_t total = (int64_t)t.n;
    free(t.ops);
    return total;
}

int orc_run_order_preserved(uint32_t n, void* const* user_in, void* const* user_out, void* const* ccl_in,
                            void* const* ccl_out, uint64_t count, uint64_t ccl_bytes, int dtype, int op)
{
    OrcTrace t;
    int rc = build_trace_order_preserved(&t, n, count, ccl_bytes, dtype);
    if (rc) return rc;
    void* const* bufs[5] = {ccl_in, ccl_out, NULL, user_in, user_out};
    rc = exec_trace(&t, bufs, dtype, op);
    free(t.ops);
    return rc;
}

/* ---- the order-preserving reduce-scatter executor's branch for small messages (ReduceScatterHDStage) -------------- */

/* ReduceScatterHDStage::RunAsync for one rank, tpl/temp_reduce_scatter/reduce_scatter_hd_stage.cc:72-108, as
 * CollReduceScatterOrderPreservedExecutor::RunReduceScatterLevel0HD prepares it (exec/coll_reduce_scatter/
 * coll_reduce_scatter_order_preserved_executor.cc:141-169: input memory = CCL input, output memory = the scratch
 * memory = CCL output in op-base mode, user pointers through opInfo).  total = one block in bytes. */
static void prog_rs_hd_stage(OrcTrace* t, uint32_t rank, uint32_t n, uint64_t total)
{
    uint32_t power = 0;
    while ((1u << (power + 1)) <= n) power++;
    const uint32_t half = 1u << (power - 1);
    /* PrepareSliceData, :110-140 */
    OrcSlice slice_map[5][ORC_MAX_RANKS];
    memset(slice_map, 0, sizeof(slice_map));
    for (uint32_t round = 1; round <= power; round++) {
        const uint32_t slice_num = n >> round;
        uint32_t k = 0;
        for (uint32_t group = 0; group < (1u << round); group++)
            for (uint32_t c = 0; c < slice_num; c++) {
                OrcSlice tmp;
                tmp.size = total * slice_num;
                const uint64_t offset = total * slice_num * group;
                if (group == 0 || round == 1) tmp.offset = offset;
                else tmp.offset = offset >= half * total ? offset - half * total : offset;
                slice_map[round - 1][k++] = tmp;
            }
    }
    const uint32_t n_steps = power;
    /* RunReduceScatterStage1st, :154-185: the own half of the user input to the front of the CCL output buffer, the
     * other half folded into the partner's */
    emit(t, 0, K_COPY, rank, B_OUT, 0, rank, B_UIN, slice_map[0][rank].offset, slice_map[0][rank].size);
    {
        const uint32_t dst_rank = rank ^ (1u << (n_steps - 1));
        emit(t, 1, K_REDUCE, dst_rank, B_OUT, 0, rank, B_UIN, slice_map[0][dst_rank].offset, slice_map[0][dst_rank].size);
    }
    /* RunReduceScatterRead, :205-250 */
    for (uint32_t step = 1; step < n_steps; step++) {
        const uint32_t dst_rank = rank ^ (1u << (n_steps - 1 - step));
        emit(t, 1 + step, K_REDUCE, rank, B_OUT, slice_map[step][rank].offset, dst_rank, B_OUT, slice_map[step][rank].offset,
             slice_map[step][rank].size);
    }
    emit(t, 1 + n_steps, K_COPY, rank, B_UOUT, 0, rank, B_OUT, slice_map[n_steps - 1][rank].offset, total);
}

/* CollReduceScatterOrderPreservedExecutor::KernelRun on its isUseHDAlg_ branch (exec/coll_reduce_scatter/
 * coll_reduce_scatter_order_preserved_executor.cc:29-38, 182-183, 273: at most 32 KiB per rank, one module of 4 or 8
 * devices, op-base mode; the template writes the user output itself).  The template takes the block stride of the
 * user input from the chunk's count (reduce_scatter_hd_stage.cc:156-160), so the loop of
 * coll_reduce_scatter_executor.cc:149-220 must not cut the message: refused otherwise. */
static int build_trace_order_preserved_small(OrcTrace* t, uint32_t n, uint64_t count, uint64_t ccl_bytes, int dtype)
{
    memset(t, 0, sizeof(*t));
    const uint32_t unit = orc_dtype_size(dtype);
    if (unit == 0 || (n != 4 && n != 8)) return -1;
    if (count * unit > 32u * 1024u) return -1;                       /* HCCL_SMALL_COUNT_32_KB, tpl/template_v1_utils.h:64 */
    const uint64_t max_count = ccl_bytes / n / 128u * 128u / unit;
    if (count > max_count) return -1;
    if (count == 0) return 0;
    for (uint32_t r = 0; r < n; r++) prog_rs_hd_stage(t, r, n, count * unit);
    if (t->oom) {
        free(t->ops);
        return -2;
    }
    return sort_trace(t);
}

int64_t orc_trace_order_preserved_small(uint32_t n, uint64_t count, uint64_t ccl_bytes, int dtype, OrcOp* out, uint64_t cap)
{
    OrcTrace t;
    int rc = build_trace_order_preserved_small(&t, n, count, ccl_bytes, dtype);
    if (rc) return rc;
    const uint64_t m = t.n < cap ? t.n : cap;
    if (out && m) memcpy(out, t.ops, m * sizeof(OrcOp));
    const int64_t total = (int64_t)t.n;
    free(t.ops);
    return total;
}

int orc_run_order_preserved_small(uint32_t n, void* const* user_in, void* const* user_out, void* const* ccl_in,
                                  void* const* ccl_out, uint64_t count, uint64_t ccl_bytes, int dtype, int op)
{
    OrcTrace t;
    int rc = build_trace_order_preserved_small(&t, n, count, ccl_bytes, dtype);
    if (rc) return rc;
    void* const* bufs[5] = {ccl_in, ccl_out, NULL, user_in, user_out};
    rc = exec_trace(&t, bufs, dtype, op);
    free(t.ops);
    return rc;
}

/* ---- the order-preserving allreduce executor (one server, op-base mode) ------------------------------------------ */

/* ReduceScatterPlantLocalReduce::RunAsync for one rank and a single (= last) group whose blocks differ in size and
 * that borrows space, tpl/temp_reduce_scatter/reduce_scatter_plant_local_reduce.cc:105-166 as
 * CollAllReduceOrderPreservedExecutor::RunReduceScatterLevel0 prepares it for one module
 * (exec/coll_all_reduce/coll_all_reduce_order_preserved_executor.cc:149-193: block d is size[d] bytes at d * stride of the
 * user input, of the input memory and of the output memory alike; all2allOffset 0; isNeedSpaceBorrow true).
 * A contribution whose slot is the last one goes to the receiving rank's INPUT memory at that rank's own block
 * offset instead, on every receiving rank but the last one (:168-188, :190-254, :337-414). */
static void prog_plant_local_reduce_borrow(OrcTrace* t, uint32_t local_rank, uint32_t rank_size, const uint64_t* size,
                                           uint64_t stride)
{
#define CALC_OUTPUT_INDEX(round) (((round) + local_rank) % rank_size)            /* :94-97, all2allOffset 0 */
#define IS_LAST_BLOCK(index) ((index) == rank_size - 1)                          /* :103 */
#define IS_LAST_RANK(r) ((r) == rank_size - 1)                                   /* :101; the one group is the last, :99 */
    /* LocalCopy, :168-188 */
    {
        const uint32_t output_index = CALC_OUTPUT_INDEX(local_rank);
        if (IS_LAST_BLOCK(output_index) && !IS_LAST_RANK(local_rank))
            emit(t, 0, K_COPY, local_rank, B_IN, stride * local_rank, local_rank, B_UIN, stride * local_rank, size[local_rank]);
        else
            emit(t, 0, K_COPY, local_rank, B_OUT, stride * output_index, local_rank, B_UIN, stride * local_rank,
                 size[local_rank]);
    }
    /* RunAlltoAll, :221-247 */
    for (uint32_t round = 0; round < rank_size; round++) {
        if (round == local_rank) continue;
        const uint32_t output_index = CALC_OUTPUT_INDEX(round);
        if (IS_LAST_BLOCK(output_index) && !IS_LAST_RANK(round))
            emit(t, 0, K_COPY, round, B_IN, stride * round, local_rank, B_UIN, stride * round, size[round]);
        else
            emit(t, 0, K_COPY, round, B_OUT, stride * output_index, local_rank, B_UIN, stride * round, size[round]);
    }
    /* RunLocalReduce, :337-414 */
    uint32_t reduce_step = 0;
    while ((1u << reduce_step) < rank_size) reduce_step++;
    const uint64_t src_offset = stride * local_rank; /* inputOffsets[localRank_], :340 */
    for (uint32_t round = 0; round < reduce_step; round++) {
        const uint32_t full = 1u << (reduce_step - round);
        const uint32_t tail_index = (rank_size < full ? rank_size : full) - 1;
        const uint32_t head_index = 1u << (reduce_step - round - 1);
        for (uint32_t offset = 0; offset <= tail_index - head_index; offset++) {
            const uint32_t input_index = CALC_OUTPUT_INDEX(head_index + offset);
            const uint32_t output_index = CALC_OUTPUT_INDEX(offset);
            const int src_borrowed = !IS_LAST_RANK(local_rank) && IS_LAST_BLOCK(input_index);  /* :376-381 */
            const int dst_borrowed = !IS_LAST_RANK(local_rank) && IS_LAST_BLOCK(output_index); /* :383-388 */
            emit(t, 1 + round, K_REDUCE, local_rank, dst_borrowed ? B_IN : B_OUT,
                 dst_borrowed ? src_offset : stride * output_index, local_rank, src_borrowed ? B_IN : B_OUT,
                 src_borrowed ? src_offset : stride * input_index, size[local_rank]);
        }
    }
#undef CALC_OUTPUT_INDEX
#undef IS_LAST_BLOCK
#undef IS_LAST_RANK
}

/* CollAllReduceOrderPreservedExecutor::KernelRun for every rank inside CollAllReduceExecutor::RunLoop
 * (exec/coll_all_reduce/coll_all_reduce_order_preserved_executor.cc:342-380 with DMAReduceFlag_, :19;
 * exec/coll_all_reduce/coll_all_reduce_executor.cc:129-138, 212-252): one module. */
static int build_trace_order_preserved_ar(OrcTrace* t, uint32_t n, uint64_t count, uint64_t ccl_bytes, int dtype)
{
    memset(t, 0, sizeof(*t));
    const uint32_t unit = orc_dtype_size(dtype);
    /* one rank per module takes RunReduceScatterLevel0SingleRank (:195-206): not restated */
    if (unit == 0 || n < 2 || n > ORC_MAX_RANKS) return -1;
    const uint64_t max_count = ccl_bytes / unit; /* CalcLoopMaxCount, coll_all_reduce_executor.cc:129-138 */
    if (max_count == 0) return -1;
    uint32_t reduce_step = 0;
    while ((1u << reduce_step) < n) reduce_step++;
    uint32_t step0 = 0;
    uint64_t cur_count = 0, user_off = 0;
    for (uint64_t count_left = count; count_left > 0; count_left -= cur_count) {
        cur_count = count_left > max_count ? max_count : count_left;
        const uint64_t cur_size = cur_count * unit;
        /* CalcSizePerBlock, :131-136 */
        uint64_t size_per_block = (cur_count + n - 1) / n * unit;
        size_per_block = (size_per_block + 127u) / 128u * 128u;
        /* CalGroupSlices, :138-147 */
        uint64_t group_size[ORC_MAX_RANKS];
        uint64_t size_remain = cur_size;
        for (uint32_t r = 0; r < n; r++) {
            group_size[r] = size_remain > size_per_block ? size_per_block : size_remain;
            size_remain -= group_size[r];
        }
        /* RunAllGatherLevel0, :256-263 */
        OrcSlice seg[ORC_MAX_RANKS];
        for (uint32_t r = 0; r < n; r++) {
            seg[r].size = group_size[r];
            seg[r].offset = group_size[r] == 0 ? 0 : r * size_per_block;
        }
        g_user_off = user_off;
        for (uint32_t r = 0; r < n; r++) {
            g_step_base = step0;
            prog_plant_local_reduce_borrow(t, r, n, group_size, size_per_block); /* :356 */
            g_step_base = step0 + 1 + reduce_step;
            prog_mesh_ag(t, r, n, seg);                                          /* :363, AllGatherMeshAtomic: all_gather_mesh_atomic.cc:19-69, the data movement of AllGatherMesh */
            g_step_base = step0 + 2 + reduce_step;
            emit(t, 0, K_COPY, r, B_UOUT, 0, r, B_OUT, 0, cur_size);             /* :369-376 */
        }
        g_user_off = 0;
        g_step_base = 0;
        if (t->oom) {
            free(t->ops);
            return -2;
        }
        step0 += 3 + reduce_step;
        user_off += cur_size;
    }
    /* DeviceMem::range refuses a range past the end of the CCL buffer (the rounded-up blocks of a tiny buffer) */
    for (uint64_t i = 0; i < t->n; i++) {
        const OrcOp* o = &t->ops[i];
        if ((o->dst_buf <= B_OUT && o->dst_off + o->bytes > ccl_bytes) || (o->src_buf <= B_OUT && o->src_off + o->bytes > ccl_bytes)) {
            free(t->ops);
            return -1;
        }
    }
    return sort_trace(t);
}

/* ---- the order-preserving allreduce executor over two communicator levels (op-base mode) -------------------------- */

/* ReduceScatterPlantLocalReduce::RunAsync for one rank of a server and ALL groups, as
 * CollAllReduceOrderPreservedExecutor::RunReduceScatterLevel0 prepares it for several modules
 * (exec/coll_all_reduce/coll_all_reduce_order_preserved_executor.cc:159-186): group g = the blocks g * L .. g * L + L - 1
 * (the blocks server g will own), every offset of block b = b * stride, all2allOffset 1 (:176), borrowed space -
 * and as CollReduceScatterOrderPreservedExecutor::RunReduceScatterLevel0 prepares it (exec/coll_reduce_scatter/
 * coll_reduce_scatter_order_preserved_executor.cc:185-211): block b of the user input at b * uin_stride, no borrowed space.
 * The template walks the groups one after the other (tpl/temp_reduce_scatter/reduce_scatter_plant_local_reduce.cc:
 * 132-160: all-to-all of group g on the main and all-to-all streams, its local reduce on the reduce streams); the
 * groups touch disjoint memory, so step 0 holds every group's all-to-all and steps 1.. every group's reduce rounds. */
static void prog_plant_groups(OrcTrace* t, uint32_t local_rank, uint32_t rank_size, uint32_t n_groups, const uint64_t* size,
                              uint64_t stride, uint64_t uin_stride, int need_space_borrow)
{
    const uint32_t all2all_offset = 1;
#define CALC_OUTPUT_INDEX(round) ((all2all_offset + (round) + local_rank) % rank_size) /* :94-97 */
#define IS_LAST_BLOCK(index) ((index) == rank_size - 1)                                 /* :103 */
    uint32_t reduce_step = 0;
    while ((1u << reduce_step) < rank_size) reduce_step++;
    for (uint32_t g = 0; g < n_groups; g++) {
        const uint64_t base = (uint64_t)g * rank_size; /* first block of the group */
        const int last_group = g == n_groups - 1;      /* :99 */
        /* LocalCopy, :168-188 */
        {
            const uint32_t output_index = CALC_OUTPUT_INDEX(local_rank);
            if (need_space_borrow && IS_LAST_BLOCK(output_index) && !(local_rank == rank_size - 1 && last_group))
                emit(t, 0, K_COPY, local_rank, B_IN, stride * (base + local_rank), local_rank, B_UIN,
                     uin_stride * (base + local_rank), size[base + local_rank]);
            else
                emit(t, 0, K_COPY, local_rank, B_OUT, stride * (base + output_index), local_rank, B_UIN,
                     uin_stride * (base + local_rank), size[base + local_rank]);
        }
        /* RunAlltoAll, :221-247 */
        for (uint32_t round = 0; round < rank_size; round++) {
            if (round == local_rank) continue;
            const uint32_t output_index = CALC_OUTPUT_INDEX(round);
            if (need_space_borrow && IS_LAST_BLOCK(output_index) && !(round == rank_size - 1 && last_group))
                emit(t, 0, K_COPY, round, B_IN, stride * (base + round), local_rank, B_UIN, uin_stride * (base + round),
                     size[base + round]);
            else
                emit(t, 0, K_COPY, round, B_OUT, stride * (base + output_index), local_rank, B_UIN,
                     uin_stride * (base + round), size[base + round]);
        }
        /* RunLocalReduce, :337-414 */
        const uint64_t src_offset = stride * (base + local_rank); /* inputOffsets[localRank_], :340 */
        const int may_borrow = need_space_borrow && !(local_rank == rank_size - 1 && last_group);
        for (uint32_t round = 0; round < reduce_step; round++) {
            const uint32_t full = 1u << (reduce_step - round);
            const uint32_t tail_index = (rank_size < full ? rank_size : full) - 1;
            const uint32_t head_index = 1u << (reduce_step - round - 1);
            for (uint32_t offset = 0; offset <= tail_index - head_index; offset++) {
                const uint32_t input_index = CALC_OUTPUT_INDEX(head_index + offset);
                const uint32_t output_index = CALC_OUTPUT_INDEX(offset);
                const int src_borrowed = may_borrow && IS_LAST_BLOCK(input_index);  /* :376-381 */
                const int dst_borrowed = may_borrow && IS_LAST_BLOCK(output_index); /* :383-388 */
                emit(t, 1 + round, K_REDUCE, local_rank, dst_borrowed ? B_IN : B_OUT,
                     dst_borrowed ? src_offset : stride * (base + output_index), local_rank, src_borrowed ? B_IN : B_OUT,
                     src_borrowed ? src_offset : stride * (base + input_index), size[base + local_rank]);
            }
        }
    }
#undef CALC_OUTPUT_INDEX
#undef IS_LAST_BLOCK
}

/* ReduceScatterPlantLocalReduceCombine::RunAsync for one rank between the servers (links that are not RoCE: the SDMA
 * branch), tpl/temp_reduce_scatter/reduce_scatter_plant_local_reduce_combine.cc:89-116, prepared by
 * CollAllReduceOrderPreservedExecutor::RunReduceScatterLevel1 (exec/coll_all_reduce/
 * coll_all_reduce_order_preserved_executor.cc:208-246).  rank / rank_size: the server index and the number of servers;
 * in_off[d]: where the level-0 result for server d's block lies, out_off[d]: block (i + d * L) itself.
 * Step 0: LocalCopy (:118-142) and the all-to-all (:180-209, :211-230); steps 1..: RunLocalReduce (:232-304). */
static void prog_plant_combine(OrcTrace* t, uint32_t rank, uint32_t rank_size, const uint64_t* size, const uint64_t* in_off,
                               const uint64_t* out_off, int use_ccl_in, int level0_last_rank, int need_space_borrow,
                               uint32_t a2a_step)
{
    /* a2a_step 0: LocalCopy and the all-to-all share step 0 (nothing a peer writes is read by a LocalCopy); 1: the
     * peers' writes come a step after the LocalCopies - with one device per module a peer may write the very place
     * the own block was read from, which the handshake after LocalCopy (:211-220) orders */
    use_ccl_in = use_ccl_in && need_space_borrow;             /* every borrowed place is behind isNeedSpaceBorrow_ */
    level0_last_rank = level0_last_rank && need_space_borrow;
#define CALC_OUTPUT_INDEX(round) (((round) + rank) % rank_size) /* :80 */
#define IS_LAST(x) ((x) == rank_size - 1)                       /* :82-87 */
    /* userInputOffsets == outputOffsets in this executor (coll_all_reduce_order_preserved_executor.cc:224-227) */
    for (uint32_t round = 0; round < rank_size; round++) {
        /* the own block first (LocalCopy), then the peers in ascending order */
        const uint32_t peer = round == 0 ? rank : (round <= rank ? round - 1 : round);
        const uint32_t output_index = CALC_OUTPUT_INDEX(peer);
        const uint32_t src_buf = use_ccl_in ? B_IN : B_OUT;                        /* :125-130, :184-189 */
        const uint64_t src_off = use_ccl_in ? out_off[peer] : in_off[peer];
        const uint32_t at = round == 0 ? 0 : a2a_step;
        if (level0_last_rank && IS_LAST(output_index) && !IS_LAST(peer)) {        /* :132-138, :191-199 */
            /* a copy onto itself is dropped by the dispatcher (platform/task/dispatcher.cc:495-498) */
            if (!(peer == rank && src_buf == B_IN && src_off == out_off[peer]))
                emit(t, at, K_COPY, peer, B_IN, out_off[peer], rank, src_buf, src_off, size[peer]);
        } else {
            emit(t, at, K_COPY, peer, B_OUT, out_off[output_index], rank, src_buf, src_off, size[peer]);
        }
    }
    uint32_t reduce_step = 0;
    while ((1u << reduce_step) < rank_size) reduce_step++;
    for (uint32_t round = 0; round < reduce_step; round++) {
        const uint32_t full = 1u << (reduce_step - round);
        const uint32_t tail_index = (rank_size < full ? rank_size : full) - 1;
        const uint32_t head_index = 1u << (reduce_step - round - 1);
        for (uint32_t offset = 0; offset <= tail_index - head_index; offset++) {
            const uint32_t input_index = CALC_OUTPUT_INDEX(head_index + offset);
            const uint32_t output_index = CALC_OUTPUT_INDEX(offset);
            const int src_borrowed = level0_last_rank && !IS_LAST(rank) && IS_LAST(input_index);  /* :273-277 */
            const int dst_borrowed = level0_last_rank && !IS_LAST(rank) && IS_LAST(output_index); /* :279-283 */
            emit(t, 1 + a2a_step + round, K_REDUCE, rank, dst_borrowed ? B_IN : B_OUT, dst_borrowed ? out_off[rank] : out_off[output_index],
                 rank, src_borrowed ? B_IN : B_OUT, src_borrowed ? out_off[rank] : out_off[input_index], size[rank]);
        }
    }
#undef CALC_OUTPUT_INDEX
#undef IS_LAST
}

static uint32_t ceil_log2_u32(uint32_t n)
{
    uint32_t s = 0;
    while ((1u << s) < n) s++;
    return s;
}

/* CollAllReduceOrderPreservedExecutor::KernelRun for every rank of n_servers modules of n_local devices
 * (exec/coll_all_reduce/coll_all_reduce_order_preserved_executor.cc:342-380) inside CollAllReduceExecutor::RunLoop.
 * alg1 selects the all-gather between the servers (:293-303): ring, NB, else NHR. */
static int build_trace_order_preserved_ar2(OrcTrace* t, int alg1, uint32_t n_servers, uint32_t n_local, uint64_t count,
                                           uint64_t ccl_bytes, int dtype)
{
    memset(t, 0, sizeof(*t));
    const uint32_t unit = orc_dtype_size(dtype);
    /* one module is build_trace_order_preserved_ar */
    if (unit == 0 || n_servers < 2 || n_local < 1 || n_servers * n_local > ORC_MAX_RANKS) return -1;
    if (alg1 != ORC_ALG_ALLREDUCE_RING && alg1 != ORC_ALG_ALLREDUCE_NHR && alg1 != ORC_ALG_ALLREDUCE_NB) return -1;
    const uint32_t n = n_servers * n_local;
    const uint64_t max_count = ccl_bytes / unit;
    if (max_count == 0) return -1;
    const uint32_t steps0 = ceil_log2_u32(n_local), steps1 = ceil_log2_u32(n_servers);
    const uint32_t ag1_steps = alg1 == ORC_ALG_ALLREDUCE_RING ? n_servers - 1 : steps1;
    /* one device per module: level 0 is a copy (:151-155), the peers' writes of level 1 come a step after the
     * LocalCopies, and there is nothing to gather inside the module */
    const int single = n_local == 1;
    const uint32_t lvl0_steps = single ? 1 : 1 + steps0, a2a_step = single ? 1 : 0, ag0_steps = single ? 0 : 1;
    uint32_t identity[ORC_MAX_RANKS];
    for (uint32_t i = 0; i < ORC_MAX_RANKS; i++) identity[i] = i;
    uint32_t step0 = 0;
    uint64_t cur_count = 0, user_off = 0;
    for (uint64_t count_left = count; count_left > 0; count_left -= cur_count) {
        cur_count = count_left > max_count ? max_count : count_left;
        const uint64_t cur_size = cur_count * unit;
        uint64_t spb = (cur_count + n - 1) / n * unit; /* CalcSizePerBlock, :131-136 */
        spb = (spb + 127u) / 128u * 128u;
        uint64_t group_size[ORC_MAX_RANKS]; /* CalGroupSlices, :138-147 */
        uint64_t size_remain = cur_size;
        for (uint32_t r = 0; r < n; r++) {
            group_size[r] = size_remain > spb ? spb : size_remain;
            size_remain -= group_size[r];
        }
        g_user_off = user_off;
        for (uint32_t rank = 0; rank < n; rank++) {
            const uint32_t server = rank / n_local, local = rank % n_local;
            uint32_t level0[ORC_MAX_RANKS], level1[ORC_MAX_RANKS];
            for (uint32_t j = 0; j < n_local; j++) level0[j] = server * n_local + j;
            for (uint32_t d = 0; d < n_servers; d++) level1[d] = d * n_local + local;
            /* level 0, :356 */
            g_rank_map = level0;
            g_step_base = step0;
            if (single) /* RunReduceScatterLevel0SingleRank, :195-206: the chunk to the front of the CCL input buffer */
                emit(t, 0, K_COPY, local, B_IN, 0, local, B_UIN, 0, cur_size);
            else
                prog_plant_groups(t, local, n_local, n_servers, group_size, spb, spb, 1);
            /* level 1, :359: RunReduceScatterLevel1 :208-246 */
            uint64_t size1[ORC_MAX_RANKS], in_off[ORC_MAX_RANKS], out_off[ORC_MAX_RANKS];
            const uint32_t input_base_index = (1 + local) % n_local; /* :218 */
            for (uint32_t d = 0; d < n_servers; d++) {
                in_off[d] = (uint64_t)(input_base_index + d * n_local) * spb;
                size1[d] = group_size[local + d * n_local];
                out_off[d] = (uint64_t)(local + d * n_local) * spb;
            }
            g_rank_map = level1;
            g_step_base = step0 + lvl0_steps;
            prog_plant_combine(t, server, n_servers, size1, in_off, out_off, single || local == n_local - 2 /* :234-235 */,
                               local == n_local - 1 /* :239 */, 1, a2a_step);
            /* all-gather inside the server, :363: RunAllGatherLevel0 :248-283 */
            OrcSlice seg[ORC_MAX_RANKS];
            for (uint32_t r = 0; r < n_local; r++) {
                seg[r].size = group_size[r + server * n_local];
                seg[r].offset = seg[r].size == 0 ? 0 : (uint64_t)(r + server * n_local) * spb;
            }
            g_rank_map = level0;
            g_step_base = step0 + lvl0_steps + 1 + a2a_step + steps1;
            prog_mesh_ag(t, local, n_local, seg);
            /* all-gather between the servers, :366: RunAllGatherLevel1 :285-340 */
            for (uint32_t d = 0; d < n_servers; d++) {
                seg[d].size = 0;
                for (uint32_t j = 0; j < n_local; j++) seg[d].size += group_size[d * n_local + j];
                seg[d].offset = (uint64_t)d * n_local * spb;
            }
            g_rank_map = level1;
            g_step_base = step0 + lvl0_steps + 1 + a2a_step + steps1 + ag0_steps;
            if (alg1 == ORC_ALG_ALLREDUCE_RING) prog_ring_ag_ex(t, server, n_servers, seg, 0, 0);
            else if (alg1 == ORC_ALG_ALLREDUCE_NB) prog_nb_ag(t, server, n_servers, seg, 0);
            else prog_nhr_ag(t, server, n_servers, seg, identity, 0, 0); /* stand-alone: order kept, nothing merged */
            g_rank_map = NULL;
            g_step_base = step0 + lvl0_steps + 1 + a2a_step + steps1 + ag0_steps + ag1_steps;
            emit(t, 0, K_COPY, rank, B_UOUT, 0, rank, B_OUT, 0, cur_size); /* :369-376 */
        }
        g_user_off = 0;
        g_step_base = 0;
        if (t->oom) {
            free(t->ops);
            return -2;
        }
        step0 += lvl0_steps + 1 + a2a_step + steps1 + ag0_steps + ag1_steps + 1;
        user_off += cur_size;
    }
    for (uint64_t i = 0; i < t->n; i++) { /* DeviceMem::range refuses a range past the end of the CCL buffer */
        const OrcOp* o = &t->ops[i];
        if ((o->dst_buf <= B_OUT && o->dst_off + o->bytes > ccl_bytes) || (o->src_buf <= B_OUT && o->src_off + o->bytes > ccl_bytes)) {
            free(t->ops);
            return -1;
        }
    }
    return sort_trace(t);
}

/* CollReduceScatterOrderPreservedExecutor::KernelRun for every rank of n_servers modules of n_local devices
 * (exec/coll_reduce_scatter/coll_reduce_scatter_order_preserved_executor.cc:260-283: level 0 :171-218, level 1
 * :220-258 - the Combine template without borrowed space, :248 - own block to the user output :273-279) inside
 * CollReduceScatterExecutor::RunLoop (exec/coll_reduce_scatter/coll_reduce_scatter_executor.cc:124-134, 149-220). */
static int build_trace_order_preserved_rs2(OrcTrace* t, uint32_t n_servers, uint32_t n_local, uint64_t count,
                                           uint64_t ccl_bytes, int dtype)
{
    memset(t, 0, sizeof(*t));
    const uint32_t unit = orc_dtype_size(dtype);
    if (unit == 0 || n_servers < 2 || n_local < 1 || n_servers * n_local > ORC_MAX_RANKS) return -1;
    const uint32_t n = n_servers * n_local;
    const int single = n_local == 1; /* one device per module */
    const uint64_t max_count = ccl_bytes / n / 128u * 128u / unit;
    if (max_count == 0) return -1;
    const uint32_t steps0 = ceil_log2_u32(n_local), steps1 = ceil_log2_u32(n_servers);
    uint32_t step0 = 0;
    uint64_t cur_count = 0, user_off = 0;
    for (uint64_t count_left = count; count_left > 0; count_left -= cur_count) {
        cur_count = count_left > max_count ? max_count : count_left;
        const uint64_t cur_size = cur_count * unit;
        uint64_t size[ORC_MAX_RANKS];
        for (uint32_t r = 0; r < n; r++) size[r] = cur_size;
        g_user_off = user_off;
        for (uint32_t rank = 0; rank < n; rank++) {
            const uint32_t server = rank / n_local, local = rank % n_local;
            uint32_t level0[ORC_MAX_RANKS], level1[ORC_MAX_RANKS];
            for (uint32_t j = 0; j < n_local; j++) level0[j] = server * n_local + j;
            for (uint32_t d = 0; d < n_servers; d++) level1[d] = d * n_local + local;
            g_rank_map = level0;
            g_step_base = step0;
            if (single) { /* RunReduceScatterLevel0SingleRank, :123-139: every block to its place in the CCL input buffer */
                for (uint32_t i = 0; i < n; i++) emit(t, 0, K_COPY, local, B_IN, cur_size * i, local, B_UIN, count * unit * i, cur_size);
            } else {
                prog_plant_groups(t, local, n_local, n_servers, size, cur_size, count * unit, 0); /* :267 */
            }
            uint64_t in_off[ORC_MAX_RANKS], out_off[ORC_MAX_RANKS];
            const uint32_t input_base_index = (1 + local) % n_local; /* :231-232 */
            for (uint32_t d = 0; d < n_servers; d++) {
                in_off[d] = (uint64_t)(input_base_index + d * n_local) * cur_size;
                out_off[d] = (uint64_t)(local + d * n_local) * cur_size;
            }
            g_rank_map = level1;
            g_step_base = step0 + (single ? 1 : 1 + steps0);
            prog_plant_combine(t, server, n_servers, size, in_off, out_off, single || local == n_local - 2 /* :247 */,
                               local == n_local - 1, single /* borrowSpace = level0Ranksize == 1, :248 */, single ? 1 : 0); /* :270 */
            g_rank_map = NULL;
            g_step_base = step0 + (single ? 3 : 2 + steps0) + steps1;
            emit(t, 0, K_COPY, rank, B_UOUT, 0, rank, B_OUT, cur_size * rank, cur_size); /* :273-279 */
        }
        g_user_off = 0;
        g_step_base = 0;
        if (t->oom) {
            free(t->ops);
            return -2;
        }
        step0 += (single ? 4 : 3 + steps0) + steps1;
        user_off += cur_size;
    }
    return sort_trace(t);
}

int64_t orc_trace_order_preserved_rs2(uint32_t n_servers, uint32_t n_local, uint64_t count, uint64_t ccl_bytes, int dtype,
                                      OrcOp* out, uint64_t cap)
{
    OrcTrace t;
    int rc = build_trace_order_preserved_rs2(&t, n_servers, n_local, count, ccl_bytes, dtype);
    if (rc) return rc;
    const uint64_t m = t.n < cap ? t.n : cap;
    if (out && m) memcpy(out, t.ops, m * sizeof(OrcOp));
    const int64_t total = (int64_t)t.n;
    free(t.ops);
    return total;
}

int orc_run_order_preserved_rs2(uint32_t n_servers, uint32_t n_local, void* const* user_in, void* const* user_out,
                                void* const* ccl_in, void* const* ccl_out, uint64_t count, uint64_t ccl_bytes, int dtype,
                                int op)
{
    OrcTrace t;
    int rc = build_trace_order_preserved_rs2(&t, n_servers, n_local, count, ccl_bytes, dtype);
    if (rc) return rc;
    void* const* bufs[5] = {ccl_in, ccl_out, NULL, user_in, user_out};
    rc = exec_trace(&t, bufs, dtype, op);
    free(t.ops);
    return rc;
}

int64_t orc_trace_order_preserved_ar2(int alg1, uint32_t n_servers, uint32_t n_local, uint64_t count, uint64_t ccl_bytes,
                                      int dtype, OrcOp* out, uint64_t cap)
{
    OrcTrace t;
    int rc = build_trace_order_preserved_ar2(&t, alg1, n_servers, n_local, count, ccl_bytes, dtype);
    if (rc) return rc;
    const uint64_t m = t.n < cap ? t.n : cap;
    if (out && m) memcpy(out, t.ops, m * sizeof(OrcOp));
    const int64_t total = (int64_t)t.n;
    free(t.ops);
    return total;
}

int orc_run_order_preserved_ar2(int alg1, uint32_t n_servers, uint32_t n_local, void* const* user_in, void* const* user_out,
                                void* const* ccl_in, void* const* ccl_out, uint64_t count, uint64_t ccl_bytes, int dtype,
                                int op)
{
    OrcTrace t;
    int rc = build_trace_order_preserved_ar2(&t, alg1, n_servers, n_local, count, ccl_bytes, dtype);
    if (rc) return rc;
    void* const* bufs[5] = {ccl_in, ccl_out, NULL, user_in, user_out};
    rc = exec_trace(&t, bufs, dtype, op);
    free(t.ops);
    return rc;
}

int64_t orc_trace_order_preserved_ar(uint32_t n, uint64_t count, uint64_t ccl_bytes, int dtype, OrcOp* out, uint64_t cap)
{
    OrcTrace t;
    int rc = build_trace_order_preserved_ar(&t, n, count, ccl_bytes, dtype);
    if (rc) return rc;
    const uint64_t m = t.n < cap ? t.n : cap;
    if (out && m) memcpy(out, t.ops, m * sizeof(OrcOp));
    const int64_t total = (int64_t)t.n;
    free(t.ops);
    return total;
}

int orc_run_order_preserved_ar(uint32_t n, void* const* user_in, void* const* user_out, void* const* ccl_in,
                               void* const* ccl_out, uint64_t count, uint64_t ccl_bytes, int dtype, int op)
{
    OrcTrace t;
    int rc = build_trace_order_preserved_ar(&t, n, count, ccl_bytes, dtype);
    if (rc) return rc;
    void* const* bufs[5] = {ccl_in, ccl_out, NULL, user_in, user_out};
    rc = exec_trace(&t, bufs, dtype, op);
    free(t.ops);
    return rc;
}

int64_t orc_algorithmic_bytes_opbase(int alg, uint32_t n, uint64_t count, uint64_t ccl_bytes, int dtype)
{
    OrcTrace t;
    int rc = build_trace_opbase(&t, alg, n, count, ccl_bytes, dtype);
    if (rc) return rc;
    int64_t total = 0;
    for (uint64_t i = 0; i < t.n; i++) total += (int64_t)t.ops[i].bytes * (t.ops[i].kind ? 3 : 2);
    free(t.ops);
    return total;
}

/* Bytes moved by the two-input model: 3b per reduce, 2b per copy. */
int64_t orc_algorithmic_bytes(int alg, uint32_t n, uint64_t count, int dtype)
{
    OrcTrace t;
    int rc = build_trace(&t, alg, n, count, dtype);
    if (rc) return rc;
    int64_t total = 0;
    for (uint64_t i = 0; i < t.n; i++) total += (int64_t)t.ops[i].bytes * (t.ops[i].kind ? 3 : 2);
    free(t.ops);
    return total;
}

/* k-way chain on host memory: dst = (((s0 (op) s1) (op) s2) ...), running value in the dst role - the result
 * of one copy and k-1 reduces (tpl/temp_all_reduce/all_reduce_mesh_oneshot.cc:94-119). */
int orc_reduce_k(void* dst, const void* const* srcs, uint32_t k, uint64_t count, int dtype, int op)
{
    const uint32_t unit = orc_dtype_size(dtype);
    if (k == 0 || unit == 0) return -1;
    orc_copy(dst, srcs[0], count * unit);
    for (uint32_t j = 1; j < k; j++)
        if (orc_reduce(dst, srcs[j], count, dtype, op) != 0) return -1;
    return 0;
}
