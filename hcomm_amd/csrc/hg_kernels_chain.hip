// hg_kernels_chain.hip - the k-way chain fold kernels (ring and mesh schedules in one launch) and the launcher
// of both fold kernels.

#include "hg_device.hpp"

extern "C" int hg_launch_tree(void* stream, int dtype, int op, const HgFoldTable* tab, uint64_t blocks, uint32_t lds);

namespace {

// ---- k-way fold ---------------------------------------------------------------------------------
//
// Chain: acc = x0; for j = 1..k-1: acc = ACC_IS_DST ? acc (op) xj : xj (op) acc, optionally storing acc into
// xj's buffer, which reproduces k-1 successive two-input reduces while reading every input once.

__host__ __device__ __forceinline__ uint32_t fold_rank(const HgFoldTable& t, uint32_t s, uint32_t j)
{
    if (t.ascending == 1u) {
        if (j == 0) return t.first[s];
        return (j - 1 < t.first[s]) ? j - 1 : j;
    }
    if (t.ascending == 2u) { // the other ranks in cyclic order, entered at distance start[s] + 1
        if (j == 0) return t.first[s];
        const uint32_t r = t.first[s] + 1u + (t.start[s] + j - 1u) % (t.nranks - 1u);
        return r >= t.nranks ? r - t.nranks : r;
    }
    int32_t r = (int32_t)t.first[s] + (int32_t)j * t.stride;
    const int32_t n = (int32_t)t.nranks;
    r %= n;
    if (r < 0) r += n;
    return (uint32_t)r;
}

// NU items per lane (item = 128-bit vector or single element); live[u] guards every access of item u.
template <class Item, bool ACC_IS_DST, uint32_t NU>
__device__ __forceinline__ void fold_chain_items(const HgFoldTable& tab, uint32_t s, const bool (&live)[NU],
                                                 const uint64_t (&idx)[NU])
{
    typedef typename Item::V V;
    const uint64_t off = tab.off[s];
    const uint32_t k = tab.k;
    V acc[NU], nxt[NU];
    const uint8_t* p0 = (const uint8_t*)tab.in[fold_rank(tab, s, 0)] + off;
#pragma unroll
    for (uint32_t u = 0; u < NU; ++u) {
        acc[u] = Item::zero();
        nxt[u] = Item::zero();
        if (live[u]) acc[u] = Item::ld(p0, idx[u]);
    }
    if (k > 1) {
        const uint8_t* p1 = (const uint8_t*)tab.in[fold_rank(tab, s, 1)] + off;
#pragma unroll
        for (uint32_t u = 0; u < NU; ++u)
            if (live[u]) nxt[u] = Item::ld(p1, idx[u]);
    }
    for (uint32_t j = 1; j < k; ++j) {
        V cur[NU];
#pragma unroll
        for (uint32_t u = 0; u < NU; ++u) cur[u] = nxt[u];
        if (j + 1 < k) { // issue the next position's loads before this position's stores
            const uint8_t* pn = (const uint8_t*)tab.in[fold_rank(tab, s, j + 1)] + off;
#pragma unroll
            for (uint32_t u = 0; u < NU; ++u)
                if (live[u]) nxt[u] = Item::ld(pn, idx[u]);
        }
#pragma unroll
        for (uint32_t u = 0; u < NU; ++u) acc[u] = ACC_IS_DST ? Item::op(acc[u], cur[u]) : Item::op(cur[u], acc[u]);
        if (tab.store_partials) {
            uint8_t* pj = (uint8_t*)tab.in[fold_rank(tab, s, j)] + off;
#pragma unroll
            for (uint32_t u = 0; u < NU; ++u)
                if (live[u]) Item::st(pj, idx[u], acc[u]);
        }
    }
    if (tab.store_final_first) {
        uint8_t* pf = (uint8_t*)tab.in[fold_rank(tab, s, 0)] + off;
#pragma unroll
        for (uint32_t u = 0; u < NU; ++u)
            if (live[u]) Item::st(pf, idx[u], acc[u]);
    }
    if (tab.out_mode == 1) {
        uint8_t* po = (uint8_t*)tab.out[tab.owner[s]] + tab.out_off[s];
#pragma unroll
        for (uint32_t u = 0; u < NU; ++u)
            if (live[u]) Item::st(po, idx[u], acc[u]);
    } else if (tab.out_mode == 2) {
        for (uint32_t r = 0; r < tab.nranks; ++r) {
            uint8_t* po = (uint8_t*)tab.out[r] + off;
#pragma unroll
            for (uint32_t u = 0; u < NU; ++u)
                if (live[u]) Item::st(po, idx[u], acc[u]);
        }
    }
}

template <int DT, int OP, bool ACC_IS_DST> __global__ __launch_bounds__(HG_BLOCK) void k_fold_chain(const HgFoldTable tab)
{
    constexpr uint32_t ES = ElemSize<DT>::v;
    const uint32_t total = tab.tile_begin[tab.nseg];
    const uint32_t tid = threadIdx.x;
    for (uint32_t tile = block_id(tab.xcd_run); tile < total; tile += gridDim.x) {
        const uint32_t s = seg_of(tab, tile);
        const uint64_t v0 = (uint64_t)(tile - tab.tile_begin[s]) * (HG_BLOCK * HG_CHAIN_UNROLL) + tid;
        const uint64_t bytes = tab.bytes[s];
        const uint64_t nvec = bytes >> 4;
        bool live[HG_CHAIN_UNROLL];
        uint64_t idx[HG_CHAIN_UNROLL];
        const bool full = (v0 - tid + (HG_BLOCK * HG_CHAIN_UNROLL) <= nvec);
#pragma unroll
        for (uint32_t u = 0; u < HG_CHAIN_UNROLL; ++u) {
            idx[u] = v0 + u * HG_BLOCK;
            live[u] = full || idx[u] < nvec;
        }
        fold_chain_items<VecItem<DT, OP>, ACC_IS_DST, HG_CHAIN_UNROLL>(tab, s, live, idx);
        if (!full) { // element tail of the segment, handled by its last tile
            const uint64_t ti[1] = {(nvec << 4) / ES + tid};
            const bool tl[1] = {(ti[0] + 1) * ES <= bytes};
            fold_chain_items<ElemItem<DT, OP>, ACC_IS_DST, 1>(tab, s, tl, ti);
        }
    }
}

// ---- k-way chain fold, small messages ------------------------------------------------------------------
//
// Same result as k_fold_chain, shaped for latency instead of bandwidth: a 4 KiB tile per workgroup (more
// workgroups for the same bytes) and the loads of eight inputs issued together, so that a launch costs about
// one memory round trip per eight inputs instead of one per input.  The rank buffers of a plan never overlap,
// which is what allows a load to be issued ahead of the partial stores of earlier positions.

template <class Item, bool ACC_IS_DST>
__device__ __forceinline__ void fold_chain_grouped(const HgFoldTable& tab, uint32_t s, uint64_t idx)
{
    typedef typename Item::V V;
    constexpr uint32_t G = 8;
    const uint64_t off = tab.off[s];
    const uint32_t k = tab.k;
    V acc = Item::zero();
    for (uint32_t j0 = 0; j0 < k; j0 += G) {
        V buf[G];
#pragma unroll
        for (uint32_t jj = 0; jj < G; ++jj) {
            buf[jj] = Item::zero();
            if (j0 + jj < k) buf[jj] = Item::ld((const uint8_t*)tab.in[fold_rank(tab, s, j0 + jj)] + off, idx);
        }
#pragma unroll
        for (uint32_t jj = 0; jj < G; ++jj) {
            const uint32_t j = j0 + jj;
            if (j < k) {
                if (j == 0) {
                    acc = buf[0];
                } else {
                    acc = ACC_IS_DST ? Item::op(acc, buf[jj]) : Item::op(buf[jj], acc);
                    if (tab.store_partials) Item::st((uint8_t*)tab.in[fold_rank(tab, s, j)] + off, idx, acc);
                }
            }
        }
    }
    if (tab.store_final_first) Item::st((uint8_t*)tab.in[fold_rank(tab, s, 0)] + off, idx, acc);
    if (tab.out_mode == 1) {
        Item::st((uint8_t*)tab.out[tab.owner[s]] + tab.out_off[s], idx, acc);
    } else if (tab.out_mode == 2) {
        for (uint32_t r = 0; r < tab.nranks; ++r) Item::st((uint8_t*)tab.out[r] + off, idx, acc);
    }
}

template <int DT, int OP, bool ACC_IS_DST>
__global__ __launch_bounds__(HG_BLOCK) void k_fold_chain_small(const HgFoldTable tab)
{
    constexpr uint32_t ES = ElemSize<DT>::v;
    const uint32_t total = tab.tile_begin[tab.nseg];
    const uint32_t tid = threadIdx.x;
    for (uint32_t tile = block_id(tab.xcd_run); tile < total; tile += gridDim.x) {
        const uint32_t s = seg_of(tab, tile);
        const uint64_t v = (uint64_t)(tile - tab.tile_begin[s]) * HG_BLOCK + tid;
        const uint64_t bytes = tab.bytes[s];
        const uint64_t nvec = bytes >> 4;
        if (v < nvec) fold_chain_grouped<VecItem<DT, OP>, ACC_IS_DST>(tab, s, v);
        if (v - tid + HG_BLOCK > nvec) { // the segment's last tile also owns its element tail
            const uint64_t e = (nvec << 4) / ES + tid;
            if ((e + 1) * ES <= bytes) fold_chain_grouped<ElemItem<DT, OP>, ACC_IS_DST>(tab, s, e);
        }
    }
}

// ---- k-way chain fold, small messages, addresses resolved by the host ---------------------------------
//
// A launch timed alone is a chain of dependent memory round trips: kernel arguments, then whatever they index,
// then the data, then the stores.  k_fold_chain_small spends three rounds on arguments (the table's scalars, the
// segment's row, the rank pointers that row selects).  For the common small case (a read-only chain of at most
// HG_DIRECT_K inputs, at most HG_DIRECT_SEG segments) the launcher resolves every address on the host and the grid
// is two-dimensional, y = segment, so that everything a workgroup needs sits at an offset it knows from its own
// index: one round of argument reads.  Same arithmetic, same order, same bits.

struct HgDirectTable {
    const uint8_t* in[HG_DIRECT_SEG][HG_DIRECT_K]; // position j of segment s
    uint8_t* out[HG_DIRECT_SEG][HG_DIRECT_K];      // receivers of segment s's result
    uint32_t bytes[HG_DIRECT_SEG];
    uint32_t k, nout;
    uint32_t store; // bit j >= 1: the running value is stored to position j's buffer after fold step j; bit 0: the
                    // final value is stored to position 0's buffer
};

// Positions beyond k repeat position 0's address (a load that is always valid) and are left out of the fold by a
// select, receivers beyond nout are skipped: no branch sits between the loads, so all of them are in flight at once.
template <class Item, bool ACC_IS_DST>
__device__ __forceinline__ void fold_direct(const uint8_t* const (&in)[HG_DIRECT_K], uint8_t* const (&out)[HG_DIRECT_K],
                                            uint32_t k, uint32_t nout, uint32_t store, uint32_t idx)
{
    typedef typename Item::V V;
    V buf[HG_DIRECT_K];
#pragma unroll
    for (uint32_t j = 0; j < HG_DIRECT_K; ++j) buf[j] = Item::ld(in[j], idx);
    V acc = buf[0];
#pragma unroll
    for (uint32_t j = 1; j < HG_DIRECT_K; ++j) {
        const V f = ACC_IS_DST ? Item::op(acc, buf[j]) : Item::op(buf[j], acc);
        acc = (j < k) ? f : acc;
        if ((store >> j) & 1u) Item::st((uint8_t*)in[j], idx, acc); // set for positions below k only
    }
    if (store & 1u) Item::st((uint8_t*)in[0], idx, acc);
#pragma unroll
    for (uint32_t r = 0; r < HG_DIRECT_K; ++r)
        if (r < nout) Item::st(out[r], idx, acc);
}

template <int DT, int OP, bool ACC_IS_DST>
__global__ __launch_bounds__(HG_BLOCK) void k_fold_chain_direct(const HgDirectTable tab)
{
    constexpr uint32_t ES = ElemSize<DT>::v;
    const uint32_t s = blockIdx.y, tid = threadIdx.x;
    // every argument this workgroup needs, read before anything depends on any of them
    const uint8_t* in[HG_DIRECT_K];
    uint8_t* out[HG_DIRECT_K];
#pragma unroll
    for (uint32_t j = 0; j < HG_DIRECT_K; ++j) {
        in[j] = tab.in[s][j];
        out[j] = tab.out[s][j];
    }
    const uint32_t bytes = tab.bytes[s], k = tab.k, nout = tab.nout, store = tab.store;
    const uint32_t tiles = (bytes + (uint32_t)HG_TREE_TILE_BYTES - 1u) / (uint32_t)HG_TREE_TILE_BYTES;
    const uint32_t nvec = bytes >> 4;
    const uint32_t v = blockIdx.x * HG_BLOCK + tid;
    // the grid is as wide as the longest segment: workgroups beyond this segment's tiles pass both tests untaken
    if (v < nvec) fold_direct<VecItem<DT, OP, HG_ST_FOLD_DIRECT, false>, ACC_IS_DST>(in, out, k, nout, store, v);
    if (blockIdx.x + 1u == tiles) { // the segment's last tile also owns its element tail
        const uint32_t e = (nvec << 4) / ES + tid;
        if ((e + 1u) * ES <= bytes) fold_direct<ElemItem<DT, OP>, ACC_IS_DST>(in, out, k, nout, store, e);
    }
}

// whether a small chain launch can take the direct kernel, and its table if so
bool direct_table(const HgFoldTable& t, HgDirectTable* d, uint32_t* width)
{
    if (!t.direct || t.nseg == 0 || t.nseg > HG_DIRECT_SEG || t.k == 0 || t.k > HG_DIRECT_K) return false;
    *width = 0;
    for (uint32_t s = 0; s < t.nseg; ++s) {
        if (t.bytes[s] >= (1ull << 31)) return false;
        const uint32_t tiles = t.tile_begin[s + 1] - t.tile_begin[s];
        if (tiles > *width) *width = tiles;
        d->bytes[s] = (uint32_t)t.bytes[s];
        for (uint32_t j = 0; j < HG_DIRECT_K; ++j) {
            d->in[s][j] = (const uint8_t*)t.in[fold_rank(t, s, j < t.k ? j : 0u)] + t.off[s];
            d->out[s][j] = nullptr;
        }
        if (t.out_mode == 1u) {
            d->out[s][0] = (uint8_t*)t.out[t.owner[s]] + t.out_off[s];
        } else if (t.out_mode == 2u) {
            if (t.nranks > HG_DIRECT_K) return false;
            for (uint32_t r = 0; r < t.nranks; ++r) d->out[s][r] = (uint8_t*)t.out[r] + t.off[s];
        }
    }
    for (uint32_t s = t.nseg; s < HG_DIRECT_SEG; ++s) d->bytes[s] = 0;
    d->k = t.k;
    d->nout = t.out_mode == 0u ? 0u : t.out_mode == 1u ? 1u : t.nranks;
    d->store = (t.store_partials ? ((1u << t.k) - 2u) : 0u) | (t.store_final_first ? 1u : 0u);
    return *width > 0;
}

template <int DT, bool AD> int launch_fold_dt(hipStream_t st, int op, const HgFoldTable* tab, uint32_t blocks, uint32_t lds)
{
    const dim3 g(blocks), b(HG_BLOCK);
    HgDirectTable direct = {};
    uint32_t width = 0;
    if (direct_table(*tab, &direct, &width)) {
        const dim3 g2(width, tab->nseg);
        switch (op) {
            case OP_SUM: hipLaunchKernelGGL((k_fold_chain_direct<DT, OP_SUM, AD>), g2, b, 0, st, direct); break;
            case OP_PROD: hipLaunchKernelGGL((k_fold_chain_direct<DT, OP_PROD, AD>), g2, b, 0, st, direct); break;
            case OP_MAX: hipLaunchKernelGGL((k_fold_chain_direct<DT, OP_MAX, AD>), g2, b, 0, st, direct); break;
            case OP_MIN: hipLaunchKernelGGL((k_fold_chain_direct<DT, OP_MIN, AD>), g2, b, 0, st, direct); break;
            default: return HCCL_E_PARA;
        }
        return rc(hipGetLastError());
    }
    if (tab->small) {
        switch (op) {
            case OP_SUM: hipLaunchKernelGGL((k_fold_chain_small<DT, OP_SUM, AD>), g, b, lds, st, *tab); break;
            case OP_PROD: hipLaunchKernelGGL((k_fold_chain_small<DT, OP_PROD, AD>), g, b, lds, st, *tab); break;
            case OP_MAX: hipLaunchKernelGGL((k_fold_chain_small<DT, OP_MAX, AD>), g, b, lds, st, *tab); break;
            case OP_MIN: hipLaunchKernelGGL((k_fold_chain_small<DT, OP_MIN, AD>), g, b, lds, st, *tab); break;
            default: return HCCL_E_PARA;
        }
        return rc(hipGetLastError());
    }
    switch (op) {
        case OP_SUM: hipLaunchKernelGGL((k_fold_chain<DT, OP_SUM, AD>), g, b, lds, st, *tab); break;
        case OP_PROD: hipLaunchKernelGGL((k_fold_chain<DT, OP_PROD, AD>), g, b, lds, st, *tab); break;
        case OP_MAX: hipLaunchKernelGGL((k_fold_chain<DT, OP_MAX, AD>), g, b, lds, st, *tab); break;
        case OP_MIN: hipLaunchKernelGGL((k_fold_chain<DT, OP_MIN, AD>), g, b, lds, st, *tab); break;
        default: return HCCL_E_PARA;
    }
    return rc(hipGetLastError());
}

} // namespace

extern "C" {

int hg_launch_fold(void* stream, int dtype, int op, int acc_is_dst, const HgFoldTable* tab, uint64_t blocks, uint32_t lds)
{
    if (blocks == 0) return HCCL_SUCCESS;
    if (tab->tree) return hg_launch_tree(stream, dtype, op, tab, blocks, lds);
    if (acc_is_dst) {
#define CALL(DT) launch_fold_dt<DT, true>((hipStream_t)stream, op, tab, (uint32_t)blocks, lds)
        HG_DISPATCH_DT(dtype, CALL)
#undef CALL
    } else {
#define CALL(DT) launch_fold_dt<DT, false>((hipStream_t)stream, op, tab, (uint32_t)blocks, lds)
        HG_DISPATCH_DT(dtype, CALL)
#undef CALL
    }
}

}
