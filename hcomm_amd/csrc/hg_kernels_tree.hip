// hg_kernels_tree.hip - the k-way tree fold kernel (recursive halving-doubling, NHR and NB schedules in one launch).

#include "hg_device.hpp"

namespace {

// ---- k-way tree fold (recursive halving) ---------------------------------------------------------
//
// K = 2^L block ranks.  For slice c, position q holds block rank c XOR bitrev(q); level l combines position q
// (dst role) with q + 2^l - exactly the reduce every halving step performs (peer = rank XOR mask, mask from K/2
// down to 1); each buffer receives the last value the step-wise replay would leave in it, and the root value
// goes to every output.
// A block rank with in2 != NULL first absorbs in2 (the odd neighbour folded in before the halving steps).

template <int L> __host__ __device__ __forceinline__ constexpr uint32_t bitrev(uint32_t q)
{
    uint32_t r = 0;
    for (int i = 0; i < L; ++i) r |= ((q >> i) & 1u) << (L - 1 - i);
    return r;
}

// NU items (128-bit vectors or single elements) per lane, all loads of a lane issued before any of its stores;
// live[u] guards every access of item u.
template <class Item, int L, uint32_t NU>
__device__ __forceinline__ void fold_tree_items(const HgFoldTable& tab, uint32_t s, const bool (&live)[NU],
                                                const uint64_t (&idx)[NU])
{
    typedef typename Item::V V;
    constexpr uint32_t K = 1u << L;
    const uint64_t off = tab.off[s];
    const uint32_t c = tab.first[s];
    V x[K][NU];
#pragma unroll
    for (uint32_t q = 0; q < K; ++q) {
        const uint8_t* p = (const uint8_t*)tab.in[c ^ bitrev<L>(q)] + off;
#pragma unroll
        for (uint32_t u = 0; u < NU; ++u) x[q][u] = live[u] ? Item::ld(p, idx[u]) : Item::zero();
    }
#pragma unroll
    for (uint32_t q = 0; q < K; ++q) {
        const uint32_t b = c ^ bitrev<L>(q);
        if (tab.in2[b]) {
            const uint8_t* p = (const uint8_t*)tab.in2[b] + off;
#pragma unroll
            for (uint32_t u = 0; u < NU; ++u)
                if (live[u]) x[q][u] = Item::op(x[q][u], Item::ld(p, idx[u]));
        }
    }
#pragma unroll
    for (int l = 0; l < L; ++l) {
#pragma unroll
        for (uint32_t q = 0; q < K; q += (2u << l)) {
#pragma unroll
            for (uint32_t u = 0; u < NU; ++u) x[q][u] = Item::op(x[q][u], x[q + (1u << l)][u]);
        }
    }
    // What the step-wise replay leaves in each input buffer: an even position is overwritten at every level it
    // takes part in and keeps the last result; an odd position only changes when it absorbed a neighbour.
#pragma unroll
    for (uint32_t q = 0; q < K; ++q) {
        const uint32_t b = c ^ bitrev<L>(q);
        if (!tab.keep_inputs && ((q & 1u) == 0u || tab.in2[b])) {
            uint8_t* p = (uint8_t*)tab.in[b] + off;
#pragma unroll
            for (uint32_t u = 0; u < NU; ++u)
                if (live[u]) Item::st(p, idx[u], x[q][u]);
        }
    }
    for (uint32_t r = 0; r < tab.nout; ++r) {
        uint8_t* p = (uint8_t*)tab.out[r] + off;
#pragma unroll
        for (uint32_t u = 0; u < NU; ++u)
            if (live[u]) Item::st(p, idx[u], x[0][u]);
    }
}

// The trees of the nonuniform hierarchical ring and of the nonuniform Bruck schedule: n <= K = 2^L ranks, position
// q of slice c holds rank c + q (tree == 2) or c - q (tree == 3) mod n, and level l combines position q (dst role,
// q a multiple of 2^(l+1)) with q + 2^l wherever that position exists - the fold rank (c +- q) performs at step l
// from rank (c +- q) +- 2^l.  An even position that had a right neighbour keeps the last value it computed; the
// root goes to every output (allreduce) or to the owner's output (reduce-scatter).
// tree == 4 takes the leaves from tab.pos[] (255 = no leaf): the host lays the rank-order trees of the
// order-preserving executors out that way - on one server position q holds rank bitrev(q) where that rank exists, so
// level l folds rank j + K / 2^(l+1) onto rank j (the contributions K/2 .. onto 0 .., then K/4 .. onto 0 .., down to
// 1 onto 0); over servers x devices the low position bits walk a server's devices like that and the high bits the
// servers.  tree == 5 reads tab.pos[] as distances instead: position q of segment s holds rank first[s] - pos[q]
// (mod n), the row of the deterministic mesh reduce-scatter, whose slot j - 1 is filled by rank d - j.
// tree == 6 gives every segment a table of its own (tab.pos[s * K + q]): trees of any shape up to depth L, a subtree
// that is shallower than its span sitting at the span's start with holes behind it.
// A hole's left neighbour always exists; the inputs are only read.
template <class Item, int L, uint32_t NU>
__device__ __forceinline__ void fold_tree_items_rot(const HgFoldTable& tab, uint32_t s, const bool (&live)[NU],
                                                    const uint64_t (&idx)[NU])
{
    typedef typename Item::V V;
    constexpr uint32_t K = 1u << L;
    const uint64_t off = tab.off[s];
    const uint32_t c = tab.first[s];
    const uint32_t n = tab.nranks;
    const bool plus = tab.tree == 2u;
    const bool order = tab.tree >= 4u;
    const bool dist = tab.tree == 5u;
    V x[K][NU];
    uint32_t b[K];
    bool have[K];
#pragma unroll
    for (uint32_t q = 0; q < K; ++q) {
        if (order) {
            b[q] = tab.pos[(tab.tree == 6u ? s * K : 0u) + q];
            have[q] = b[q] < n;
            if (dist && have[q]) {
                b[q] = c + n - b[q];
                if (b[q] >= n) b[q] -= n;
            }
        } else {
            b[q] = plus ? c + q : c + n - q;
            if (b[q] >= n) b[q] -= n;
            have[q] = q < n;
        }
        if (have[q]) {
            const uint8_t* p = (const uint8_t*)tab.in[b[q]] + off;
#pragma unroll
            for (uint32_t u = 0; u < NU; ++u) x[q][u] = live[u] ? Item::ld(p, idx[u]) : Item::zero();
        }
    }
#pragma unroll
    for (int l = 0; l < L; ++l) {
#pragma unroll
        for (uint32_t q = 0; q < K; q += (2u << l))
            if (have[q + (1u << l)]) {
#pragma unroll
                for (uint32_t u = 0; u < NU; ++u) x[q][u] = Item::op(x[q][u], x[q + (1u << l)][u]);
            }
    }
#pragma unroll
    for (uint32_t q = 0; q < K; q += 2)
        if (!order && !tab.keep_inputs && q + 1 < n) {
            uint8_t* p = (uint8_t*)tab.in[b[q]] + off;
#pragma unroll
            for (uint32_t u = 0; u < NU; ++u)
                if (live[u]) Item::st(p, idx[u], x[q][u]);
        }
    if (tab.out_mode == 1u) {
        uint8_t* p = (uint8_t*)tab.out[tab.owner[s]] + tab.out_off[s];
#pragma unroll
        for (uint32_t u = 0; u < NU; ++u)
            if (live[u]) Item::st(p, idx[u], x[0][u]);
    } else {
        for (uint32_t r = 0; r < tab.nout; ++r) {
            uint8_t* p = (uint8_t*)tab.out[r] + off;
#pragma unroll
            for (uint32_t u = 0; u < NU; ++u)
                if (live[u]) Item::st(p, idx[u], x[0][u]);
        }
    }
}

// Per-segment trees (tree == 6) of depth 6: 64 leaf positions are more than a lane holds at once, so the two halves of
// 32 positions are loaded and folded one after the other - levels 0 .. 4 inside a half are the fixed pattern above -
// and the last level folds the second half's root onto the first's.
template <class Item> __device__ __forceinline__ void fold_tree_items_deep(const HgFoldTable& tab, uint32_t s, bool live, uint64_t idx)
{
    typedef typename Item::V V;
    constexpr uint32_t H = 32u;
    const uint64_t off = tab.off[s];
    const uint32_t n = tab.nranks;
    V root[2];
    bool have_root[2];
#pragma unroll
    for (uint32_t half = 0; half < 2u; ++half) {
        V x[H];
        bool have[H];
#pragma unroll
        for (uint32_t q = 0; q < H; ++q) {
            const uint32_t b = tab.pos[s * 2u * H + half * H + q];
            have[q] = b < n;
            x[q] = Item::zero();
            if (have[q] && live) x[q] = Item::ld((const uint8_t*)tab.in[b] + off, idx);
        }
#pragma unroll
        for (int l = 0; l < 5; ++l) {
#pragma unroll
            for (uint32_t q = 0; q < H; q += (2u << l))
                if (have[q + (1u << l)]) x[q] = Item::op(x[q], x[q + (1u << l)]);
        }
        root[half] = x[0];
        have_root[half] = have[0];
    }
    const V r = have_root[1] ? Item::op(root[0], root[1]) : root[0];
    if (!live) return;
    if (tab.out_mode == 1u) {
        Item::st((uint8_t*)tab.out[tab.owner[s]] + tab.out_off[s], idx, r);
    } else {
        for (uint32_t q = 0; q < tab.nout; ++q) Item::st((uint8_t*)tab.out[q] + off, idx, r);
    }
}

template <int DT, int OP> __global__ __launch_bounds__(HG_BLOCK) void k_fold_tree_deep(const HgFoldTable tab)
{
    constexpr uint32_t ES = ElemSize<DT>::v;
    const uint32_t total = tab.tile_begin[tab.nseg];
    const uint32_t tid = threadIdx.x;
    for (uint32_t tile = block_id(tab.xcd_run); tile < total; tile += gridDim.x) {
        const uint32_t s = seg_of(tab, tile);
        const uint64_t v = (uint64_t)(tile - tab.tile_begin[s]) * HG_BLOCK + tid;
        const uint64_t bytes = tab.bytes[s];
        const uint64_t nvec = bytes >> 4;
        fold_tree_items_deep<VecItem<DT, OP>>(tab, s, v < nvec, v);
        if (v - tid + HG_BLOCK > nvec) { // the segment's last tile also owns its element tail
            const uint64_t e = (nvec << 4) / ES + tid;
            fold_tree_items_deep<ElemItem<DT, OP>>(tab, s, (e + 1) * ES <= bytes, e);
        }
    }
}

// A lane handles NU vectors (tab.nu, chosen by the host): two while the 2 x K values fit comfortably in registers
// (K <= 8) and the launch writes little beside its result, else one (a launch that also stores the partials into
// the inputs moves more on 4 KiB tiles: NHR allreduce of 8 x 128 MiB in one launch 0.499 -> 0.463 ms).
template <int DT, int OP, int L, uint32_t NU> __global__ __launch_bounds__(HG_BLOCK) void k_fold_tree(const HgFoldTable tab)
{
    constexpr uint32_t ES = ElemSize<DT>::v;
    const uint32_t total = tab.tile_begin[tab.nseg];
    const uint32_t tid = threadIdx.x;
    for (uint32_t tile = block_id(tab.xcd_run); tile < total; tile += gridDim.x) {
        const uint32_t s = seg_of(tab, tile);
        const uint64_t v0 = (uint64_t)(tile - tab.tile_begin[s]) * (HG_BLOCK * NU) + tid;
        const uint64_t bytes = tab.bytes[s];
        const uint64_t nvec = bytes >> 4;
        uint64_t idx[NU];
        bool live[NU];
#pragma unroll
        for (uint32_t u = 0; u < NU; ++u) {
            idx[u] = v0 + u * HG_BLOCK;
            live[u] = idx[u] < nvec;
        }
        if (tab.tree == 1u) fold_tree_items<VecItem<DT, OP>, L, NU>(tab, s, live, idx);
        else fold_tree_items_rot<VecItem<DT, OP>, L, NU>(tab, s, live, idx);
        if (v0 - tid + HG_BLOCK * NU > nvec) { // the segment's last tile also owns its element tail
            const uint64_t ti[1] = {(nvec << 4) / ES + tid};
            const bool tl[1] = {(ti[0] + 1) * ES <= bytes};
            if (tab.tree == 1u) fold_tree_items<ElemItem<DT, OP>, L, 1>(tab, s, tl, ti);
            else fold_tree_items_rot<ElemItem<DT, OP>, L, 1>(tab, s, tl, ti);
        }
    }
}

// ---- small tree launches with host-resolved addresses --------------------------------------------------------
//
// The kernels above read their arguments in rounds that wait for one another (the table's scalars, the segment's
// row, the leaf table, the rank pointers it selects), a quarter of a microsecond each, which is much of what a small
// launch costs.  For trees of up to 16 positions in up to HG_DIRECT_SEG segments the launcher lays every leaf's
// address out per segment and the grid is two-dimensional (y = segment, x = tile): one round of argument reads.
// A hole carries position 0's address (a load that is always valid) and is left out of the fold by a select, so
// that no branch sits between the loads.  Same tree, same operand roles, same bits.

template <uint32_t K> struct HgTreeDirect {
    const uint8_t* in[HG_DIRECT_SEG][K]; // leaf position q of segment s (position 0's address where q is a hole)
    uint8_t* out[HG_DIRECT_SEG][K];      // receivers of segment s's root
    uint32_t bytes[HG_DIRECT_SEG];
    uint32_t have[HG_DIRECT_SEG];  // bit q: position q holds a leaf
    uint32_t store[HG_DIRECT_SEG]; // bit q: position q's last value is stored back to its buffer
    uint32_t nout;
};

template <class Item, int L>
__device__ __forceinline__ void fold_tree_direct(const uint8_t* const (&in)[1u << L], uint8_t* const (&out)[1u << L], uint32_t have,
                                                 uint32_t store, uint32_t nout, uint32_t idx)
{
    typedef typename Item::V V;
    constexpr uint32_t K = 1u << L;
    V x[K];
#pragma unroll
    for (uint32_t q = 0; q < K; ++q) x[q] = Item::ld(in[q], idx);
#pragma unroll
    for (int l = 0; l < L; ++l) {
#pragma unroll
        for (uint32_t q = 0; q < K; q += (2u << l)) {
            const V f = Item::op(x[q], x[q + (1u << l)]);
            x[q] = ((have >> (q + (1u << l))) & 1u) ? f : x[q];
        }
    }
#pragma unroll
    for (uint32_t q = 0; q < K; q += 2)
        if ((store >> q) & 1u) Item::st((uint8_t*)in[q], idx, x[q]);
#pragma unroll
    for (uint32_t r = 0; r < K; ++r)
        if (r < nout) Item::st(out[r], idx, x[0]);
}

template <int DT, int OP, int L> __global__ __launch_bounds__(HG_BLOCK) void k_fold_tree_direct(const HgTreeDirect<(1u << L)> tab)
{
    constexpr uint32_t ES = ElemSize<DT>::v;
    constexpr uint32_t K = 1u << L;
    const uint32_t s = blockIdx.y, tid = threadIdx.x;
    // every argument this workgroup needs, read before anything depends on any of them
    const uint8_t* in[K];
    uint8_t* out[K];
#pragma unroll
    for (uint32_t q = 0; q < K; ++q) {
        in[q] = tab.in[s][q];
        out[q] = tab.out[s][q];
    }
    const uint32_t bytes = tab.bytes[s], have = tab.have[s], store = tab.store[s], nout = tab.nout;
    const uint32_t nvec = bytes >> 4;
    const uint32_t v = blockIdx.x * HG_BLOCK + tid;
    // the grid is as wide as the longest segment: workgroups beyond this segment's tiles pass both tests untaken
    if (v < nvec) fold_tree_direct<VecItem<DT, OP, HG_ST_FOLD_DIRECT, false>, L>(in, out, have, store, nout, v);
    if (blockIdx.x == nvec / HG_BLOCK) { // the tile the element tail falls into
        const uint32_t e = (nvec << 4) / ES + tid;
        if ((e + 1u) * ES <= bytes) fold_tree_direct<ElemItem<DT, OP>, L>(in, out, have, store, nout, e);
    }
}

// The direct table of a tree launch, or false where the launch has something it does not carry (a neighbour
// absorbed before the tree, more receivers than positions).  Mirrors fold_tree_items / fold_tree_items_rot.
template <int L> bool tree_direct_table(const HgFoldTable& t, HgTreeDirect<(1u << L)>* d, uint32_t* width)
{
    constexpr uint32_t K = 1u << L;
    const uint32_t n = t.nranks;
    const bool order = t.tree >= 4u;
    const uint32_t nout = (t.tree != 1u && t.out_mode == 1u) ? 1u : t.nout;
    if (nout > K) return false;
    *width = 0;
    for (uint32_t s = 0; s < HG_DIRECT_SEG; ++s) {
        d->bytes[s] = d->have[s] = d->store[s] = 0;
        for (uint32_t q = 0; q < K; ++q) {
            d->in[s][q] = nullptr;
            d->out[s][q] = nullptr;
        }
    }
    for (uint32_t s = 0; s < t.nseg; ++s) {
        if (t.bytes[s] >= (1ull << 31)) return false;
        const uint32_t c = t.first[s];
        const uint64_t off = t.off[s];
        for (uint32_t q = 0; q < K; ++q) {
            uint32_t b;
            bool have;
            if (t.tree == 1u) {
                b = c ^ bitrev<L>(q);
                have = true;
                if (b >= HCOMM_GFX_MAX_RANKS || t.in2[b]) return false;
            } else if (order) {
                b = t.pos[(t.tree == 6u ? s * K : 0u) + q];
                have = b < n;
                if (t.tree == 5u && have) {
                    b = c + n - b;
                    if (b >= n) b -= n;
                }
            } else {
                b = (t.tree == 2u) ? c + q : c + n - q;
                if (b >= n) b -= n;
                have = q < n;
            }
            if (have) {
                d->in[s][q] = (const uint8_t*)t.in[b] + off;
                d->have[s] |= 1u << q;
                const bool stored = t.tree == 1u ? !t.keep_inputs : (!order && !t.keep_inputs && q + 1u < n);
                if ((q & 1u) == 0u && stored) d->store[s] |= 1u << q;
            }
        }
        if (!(d->have[s] & 1u)) return false;
        for (uint32_t q = 0; q < K; ++q)
            if (!d->in[s][q]) d->in[s][q] = d->in[s][0];
        if (t.tree != 1u && t.out_mode == 1u) {
            d->out[s][0] = (uint8_t*)t.out[t.owner[s]] + t.out_off[s];
        } else {
            for (uint32_t r = 0; r < nout; ++r) d->out[s][r] = (uint8_t*)t.out[r] + off;
        }
        d->bytes[s] = (uint32_t)t.bytes[s];
        const uint32_t tiles = (uint32_t)((t.bytes[s] + HG_TREE_TILE_BYTES - 1) / HG_TREE_TILE_BYTES);
        if (tiles > *width) *width = tiles;
    }
    d->nout = nout;
    return *width > 0;
}

template <int DT, int L, uint32_t NU>
int launch_tree_dt_l_nu(hipStream_t st, int op, const HgFoldTable* tab, uint32_t blocks, uint32_t lds)
{
    switch (op) {
        case OP_SUM: hipLaunchKernelGGL((k_fold_tree<DT, OP_SUM, L, NU>), dim3(blocks), dim3(HG_BLOCK), lds, st, *tab); break;
        case OP_PROD: hipLaunchKernelGGL((k_fold_tree<DT, OP_PROD, L, NU>), dim3(blocks), dim3(HG_BLOCK), lds, st, *tab); break;
        case OP_MAX: hipLaunchKernelGGL((k_fold_tree<DT, OP_MAX, L, NU>), dim3(blocks), dim3(HG_BLOCK), lds, st, *tab); break;
        case OP_MIN: hipLaunchKernelGGL((k_fold_tree<DT, OP_MIN, L, NU>), dim3(blocks), dim3(HG_BLOCK), lds, st, *tab); break;
        default: return HCCL_E_PARA;
    }
    return rc(hipGetLastError());
}

template <int DT, int L> int launch_tree_dt_l(hipStream_t st, int op, const HgFoldTable* tab, uint32_t blocks, uint32_t lds)
{
    if constexpr (L <= 4) {
        HgTreeDirect<(1u << L)> direct;
        uint32_t width = 0;
        if (tab->direct && tree_direct_table<L>(*tab, &direct, &width)) {
            const dim3 g2(width, tab->nseg), b(HG_BLOCK);
            switch (op) {
                case OP_SUM: hipLaunchKernelGGL((k_fold_tree_direct<DT, OP_SUM, L>), g2, b, 0, st, direct); break;
                case OP_PROD: hipLaunchKernelGGL((k_fold_tree_direct<DT, OP_PROD, L>), g2, b, 0, st, direct); break;
                case OP_MAX: hipLaunchKernelGGL((k_fold_tree_direct<DT, OP_MAX, L>), g2, b, 0, st, direct); break;
                case OP_MIN: hipLaunchKernelGGL((k_fold_tree_direct<DT, OP_MIN, L>), g2, b, 0, st, direct); break;
                default: return HCCL_E_PARA;
            }
            return rc(hipGetLastError());
        }
    }
    if constexpr (L == 2 || L == 3) {
        if (tab->nu == 2u) return launch_tree_dt_l_nu<DT, L, 2>(st, op, tab, blocks, lds);
    }
    if (tab->nu != 1u) return HCCL_E_INTERNAL;
    return launch_tree_dt_l_nu<DT, L, 1>(st, op, tab, blocks, lds);
}

template <int DT> int launch_tree_deep_dt(hipStream_t st, int op, const HgFoldTable* tab, uint32_t blocks, uint32_t lds)
{
    if (tab->tree != 6u) return HCCL_E_PARA; /* the only mode whose trees are laid out over 64 positions */
    switch (op) {
        case OP_SUM: hipLaunchKernelGGL((k_fold_tree_deep<DT, OP_SUM>), dim3(blocks), dim3(HG_BLOCK), lds, st, *tab); break;
        case OP_PROD: hipLaunchKernelGGL((k_fold_tree_deep<DT, OP_PROD>), dim3(blocks), dim3(HG_BLOCK), lds, st, *tab); break;
        case OP_MAX: hipLaunchKernelGGL((k_fold_tree_deep<DT, OP_MAX>), dim3(blocks), dim3(HG_BLOCK), lds, st, *tab); break;
        case OP_MIN: hipLaunchKernelGGL((k_fold_tree_deep<DT, OP_MIN>), dim3(blocks), dim3(HG_BLOCK), lds, st, *tab); break;
        default: return HCCL_E_PARA;
    }
    return rc(hipGetLastError());
}

template <int DT> int launch_tree_dt(hipStream_t st, int op, const HgFoldTable* tab, uint32_t blocks, uint32_t lds)
{
    switch (tab->k) {
        case 64: return launch_tree_deep_dt<DT>(st, op, tab, blocks, lds);
        case 2: return launch_tree_dt_l<DT, 1>(st, op, tab, blocks, lds);
        case 4: return launch_tree_dt_l<DT, 2>(st, op, tab, blocks, lds);
        case 8: return launch_tree_dt_l<DT, 3>(st, op, tab, blocks, lds);
        case 16: return launch_tree_dt_l<DT, 4>(st, op, tab, blocks, lds);
        case 32: return launch_tree_dt_l<DT, 5>(st, op, tab, blocks, lds);
        default: return HCCL_E_PARA;
    }
}

} // namespace

// Compiled twice (HG_TREE_PART 0: integer element types, 1: floating-point ones) so that the 120 instances of the
// kernel build side by side.
#ifndef HG_TREE_PART
#define HG_TREE_PART 0
#endif

#if HG_TREE_PART == 0
extern "C" int hg_launch_tree_float(void* stream, int dtype, int op, const HgFoldTable* tab, uint64_t blocks, uint32_t lds);

extern "C" int hg_launch_tree(void* stream, int dtype, int op, const HgFoldTable* tab, uint64_t blocks, uint32_t lds)
{
    hipStream_t st = (hipStream_t)stream;
    switch (dtype) {
        case DT_I8: return launch_tree_dt<DT_I8>(st, op, tab, (uint32_t)blocks, lds);
        case DT_I16: return launch_tree_dt<DT_I16>(st, op, tab, (uint32_t)blocks, lds);
        case DT_I32: return launch_tree_dt<DT_I32>(st, op, tab, (uint32_t)blocks, lds);
        default: return hg_launch_tree_float(stream, dtype, op, tab, blocks, lds);
    }
}
#else
extern "C" int hg_launch_tree_float(void* stream, int dtype, int op, const HgFoldTable* tab, uint64_t blocks, uint32_t lds)
{
    hipStream_t st = (hipStream_t)stream;
    switch (dtype) {
        case DT_F16: return launch_tree_dt<DT_F16>(st, op, tab, (uint32_t)blocks, lds);
        case DT_F32: return launch_tree_dt<DT_F32>(st, op, tab, (uint32_t)blocks, lds);
        case DT_BF16: return launch_tree_dt<DT_BF16>(st, op, tab, (uint32_t)blocks, lds);
        default: return HCCL_E_PARA;
    }
}
#endif
