// hg_kernels.hip - gfx950 kernels of libhcomm_gfx.so and their launchers.
//
// Everything here is HBM-bandwidth bound: one lane moves 128 bits per access, a workgroup of 256 lanes
// keeps HG_UNROLL such accesses per operand in flight, and a launch covers a whole table of segments
// (all simulated ranks of one schedule step) with a grid-stride loop over 16 KiB tiles.
//
// Element semantics (the reference's "dst = dst (op) src", src/legacy/ascend910/platform/task/
// dispatcher_common.cc:137-147; CPU witnesses test/ut/stub/llt_hccl_stub.cc:4077-4204 and
// test/hccl_vm/src/plugin/runner/runner_utils/hccl_task_reduce_process.cc:18-55):
//   SUM a+b, PROD a*b, MAX (src > dst) ? src : dst, MIN (src < dst) ? src : dst;
//   integers wrap in two's complement; fp32 is one IEEE operation; fp16 / bf16 widen to fp32, operate,
//   and round to nearest even back to the storage type after every operation
//   (test/hccl_vm/src/plugin/runner/ccu_executor/ccu_fp16.h:39-66,102-135); a NaN result of SUM / PROD on a
//   16-bit type is stored as sign | 0x7e00 (fp16, ccu_fp16.h:121) or sign | 0x7fc0 (bf16, by analogy).

#include <hip/hip_runtime.h>

#include "hg_internal.h"

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef short s16x2 __attribute__((ext_vector_type(2)));
typedef signed char s8x4 __attribute__((ext_vector_type(4)));

enum { OP_SUM = 0, OP_PROD = 1, OP_MAX = 2, OP_MIN = 3 };
enum { DT_I8 = 0, DT_I16 = 1, DT_I32 = 2, DT_F16 = 3, DT_F32 = 4, DT_BF16 = 11 };

template <int DT> struct ElemSize { static constexpr uint32_t v = (DT == DT_I8) ? 1u : (DT == DT_I32 || DT == DT_F32) ? 4u : 2u; };

// ---- scalar element operations ----------------------------------------------------------------

template <int OP, typename T> __device__ __forceinline__ T int_op(T d, T s)
{
    typedef typename std::make_unsigned<T>::type U;
    if (OP == OP_SUM) return (T)((U)d + (U)s);
    if (OP == OP_PROD) return (T)((U)d * (U)s);
    if (OP == OP_MAX) return (s > d) ? s : d;
    return (s < d) ? s : d;
}

__device__ __forceinline__ float bits_f32(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t f32_bits(float f) { return __builtin_bit_cast(uint32_t, f); }

template <int OP> __device__ __forceinline__ uint32_t f32_op(uint32_t d, uint32_t s)
{
    const float fd = bits_f32(d), fs = bits_f32(s);
    if (OP == OP_SUM) return f32_bits(fd + fs);
    if (OP == OP_PROD) return f32_bits(fd * fs);
    if (OP == OP_MAX) return (fs > fd) ? s : d;
    return (fs < fd) ? s : d;
}

__device__ __forceinline__ float f16_to_f32(uint32_t h) { return (float)__builtin_bit_cast(_Float16, (uint16_t)h); }

__device__ __forceinline__ uint32_t f32_to_f16(float f)
{
    if (f != f) return ((f32_bits(f) >> 16) & 0x8000u) | 0x7e00u;
    return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)f);
}

__device__ __forceinline__ float bf16_to_f32(uint32_t h) { return bits_f32(h << 16); }

__device__ __forceinline__ uint32_t f32_to_bf16(float f)
{
    const uint32_t u = f32_bits(f);
    if (f != f) return ((u >> 16) & 0x8000u) | 0x7fc0u;
    return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
}

// one 16-bit float element held in the low half of a word
template <int DT, int OP> __device__ __forceinline__ uint32_t half_op(uint32_t d, uint32_t s)
{
    const float fd = (DT == DT_F16) ? f16_to_f32(d) : bf16_to_f32(d);
    const float fs = (DT == DT_F16) ? f16_to_f32(s) : bf16_to_f32(s);
    if (OP == OP_MAX) return (fs > fd) ? s : d;
    if (OP == OP_MIN) return (fs < fd) ? s : d;
    const float r = (OP == OP_SUM) ? fd + fs : fd * fs;
    return (DT == DT_F16) ? f32_to_f16(r) : f32_to_bf16(r);
}

// ---- one 32-bit word of packed elements: returns d (op) s, d in the dst role ------------------------

template <int DT, int OP> __device__ __forceinline__ uint32_t word_op(uint32_t d, uint32_t s)
{
    if (DT == DT_I32) return (uint32_t)int_op<OP, int32_t>((int32_t)d, (int32_t)s);
    if (DT == DT_F32) return f32_op<OP>(d, s);
    if (DT == DT_I16) {
        const uint32_t lo = (uint16_t)int_op<OP, int16_t>((int16_t)(d & 0xffffu), (int16_t)(s & 0xffffu));
        const uint32_t hi = (uint16_t)int_op<OP, int16_t>((int16_t)(d >> 16), (int16_t)(s >> 16));
        return lo | (hi << 16);
    }
    if (DT == DT_I8) {
        uint32_t r = 0;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const uint32_t e = (uint8_t)int_op<OP, int8_t>((int8_t)(d >> (8 * b)), (int8_t)(s >> (8 * b)));
            r |= e << (8 * b);
        }
        return r;
    }
    // fp16 / bf16
    const uint32_t lo = half_op<DT, OP>(d & 0xffffu, s & 0xffffu);
    const uint32_t hi = half_op<DT, OP>(d >> 16, s >> 16);
    return lo | (hi << 16);
}

template <int DT, int OP> __device__ __forceinline__ u32x4 vec_op(u32x4 d, u32x4 s)
{
    u32x4 r;
    r.x = word_op<DT, OP>(d.x, s.x);
    r.y = word_op<DT, OP>(d.y, s.y);
    r.z = word_op<DT, OP>(d.z, s.z);
    r.w = word_op<DT, OP>(d.w, s.w);
    return r;
}

// one element at byte address p, zero-extended into a word / stored from the low bits of a word
template <uint32_t ES> __device__ __forceinline__ uint32_t ld_elem(const void* p)
{
    if (ES == 1) return *(const uint8_t*)p;
    if (ES == 2) return *(const uint16_t*)p;
    return *(const uint32_t*)p;
}
template <uint32_t ES> __device__ __forceinline__ void st_elem(void* p, uint32_t v)
{
    if (ES == 1) *(uint8_t*)p = (uint8_t)v;
    else if (ES == 2) *(uint16_t*)p = (uint16_t)v;
    else *(uint32_t*)p = v;
}

// Cache hints.  A ring step reads what the neighbouring rank's previous step wrote, so plain stores are left
// to be kept by the memory-side cache while every load is marked non-temporal (each value is read once).
#ifndef HG_NT_LD_DST
#define HG_NT_LD_DST 1 /* the operand that is overwritten */
#endif
#ifndef HG_NT_LD_SRC
#define HG_NT_LD_SRC 1 /* the peer's operand */
#endif
#ifndef HG_NT_ST
#define HG_NT_ST 0
#endif
#ifndef HG_NT_FOLD_ST
#define HG_NT_FOLD_ST 1 /* nothing a fold launch stores is read again by it */
#endif
template <bool NT> __device__ __forceinline__ u32x4 ldv(const void* base, uint64_t vec)
{
    if (NT) return __builtin_nontemporal_load((const u32x4*)base + vec);
    return ((const u32x4*)base)[vec];
}
template <bool NT> __device__ __forceinline__ void stv(void* base, uint64_t vec, u32x4 v)
{
    if (NT) __builtin_nontemporal_store(v, (u32x4*)base + vec);
    else ((u32x4*)base)[vec] = v;
}

// Workgroups are dealt to the 8 XCDs round-robin by their index.  REMAP renumbers them so that each XCD walks runs
// of HG_XCD_RUN consecutive tiles (2 MiB) - or, when the grid does not divide that way, one contiguous eighth of the
// tiles - instead of every eighth tile.  Measured on the 8 x 128 MiB ring steps (TB/s; plain, runs of 2 / 8 / 32 /
// 128 tiles, contiguous eighth): copy 6.68, 6.69, 6.65, 6.84, 6.93, 6.87; two-input reduce 6.47, 6.49, 6.53, 6.35,
// 6.51, 6.17; k-way fold 5.50, 5.44, 5.56, 5.59, 5.15, 4.84.  Only the copy gains beyond run-to-run noise, so only
// k_copy renumbers.
#ifndef HG_STREAM_COPY_BYTES
#define HG_STREAM_COPY_BYTES (256ull << 20) /* the 256 MB memory-side cache */
#endif
#ifndef HG_STREAM_REDUCE_BYTES
#define HG_STREAM_REDUCE_BYTES (256ull << 20)
#endif
#ifndef HG_XCD_REMAP_COPY
#define HG_XCD_REMAP_COPY 1
#endif
#ifndef HG_XCD_REMAP
#define HG_XCD_REMAP 0
#endif
#ifndef HG_XCD_RUN
#define HG_XCD_RUN 128u
#endif
template <bool REMAP> __device__ __forceinline__ uint32_t block_id()
{
    const uint32_t g = gridDim.x, b = blockIdx.x;
    if (!REMAP) return b;
    if ((g % (8u * HG_XCD_RUN)) == 0u) {
        const uint32_t i = b >> 3;
        return (i / HG_XCD_RUN) * 8u * HG_XCD_RUN + (b & 7u) * HG_XCD_RUN + i % HG_XCD_RUN;
    }
    if ((g & 7u) == 0u) return (b & 7u) * (g >> 3) + (b >> 3);
    return b;
}

// segment that owns a tile (uniform across the workgroup; nseg <= 32)
__device__ __forceinline__ uint32_t find_seg(const uint32_t* tile_begin, uint32_t nseg, uint32_t tile)
{
    uint32_t s = 0;
    while (s + 1 < nseg && tile >= tile_begin[s + 1]) ++s;
    return s;
}

// ---- batched copy ------------------------------------------------------------------------------

// STREAM: what the launch writes exceeds the memory-side cache, so nothing of it can be found there by the next
// launch anyway: store with the non-temporal hint (measured on a 2 GiB copy: 6.12 against 5.88 TB/s).
template <bool STREAM> __global__ __launch_bounds__(HG_BLOCK) void k_copy(const HgSeg2Table tab)
{
    const uint32_t total = tab.tile_begin[tab.nseg];
    const uint32_t tid = threadIdx.x;
    for (uint32_t tile = block_id<HG_XCD_REMAP_COPY>(); tile < total; tile += gridDim.x) {
        const uint32_t s = find_seg(tab.tile_begin, tab.nseg, tile);
        const uint64_t v0 = (uint64_t)(tile - tab.tile_begin[s]) * HG_TILE_VECS + tid;
        const uint64_t bytes = tab.bytes[s];
        const uint64_t nvec = bytes >> 4;
        void* d = tab.dst[s];
        const void* p = tab.src[s];
        if (v0 - tid + HG_TILE_VECS <= nvec) {
            u32x4 a[HG_UNROLL];
#pragma unroll
            for (uint32_t u = 0; u < HG_UNROLL; ++u) a[u] = ldv<HG_NT_LD_SRC>(p, v0 + u * HG_BLOCK);
#pragma unroll
            for (uint32_t u = 0; u < HG_UNROLL; ++u) stv<STREAM || HG_NT_ST>(d, v0 + u * HG_BLOCK, a[u]);
        } else {
#pragma unroll
            for (uint32_t u = 0; u < HG_UNROLL; ++u) {
                const uint64_t v = v0 + u * HG_BLOCK;
                if (v < nvec) stv<STREAM || HG_NT_ST>(d, v, ldv<HG_NT_LD_SRC>(p, v));
            }
            const uint64_t b = (nvec << 4) + tid; // this tile is the segment's last one: byte tail
            if (b < bytes) ((uint8_t*)d)[b] = ((const uint8_t*)p)[b];
        }
    }
}

// ---- batched dst = dst (op) src -----------------------------------------------------------------

template <int DT, int OP, bool STREAM> __global__ __launch_bounds__(HG_BLOCK) void k_reduce2(const HgSeg2Table tab)
{
    constexpr uint32_t ES = ElemSize<DT>::v;
    const uint32_t total = tab.tile_begin[tab.nseg];
    const uint32_t tid = threadIdx.x;
    for (uint32_t tile = block_id<HG_XCD_REMAP>(); tile < total; tile += gridDim.x) {
        const uint32_t s = find_seg(tab.tile_begin, tab.nseg, tile);
        const uint64_t v0 = (uint64_t)(tile - tab.tile_begin[s]) * HG_TILE_VECS + tid;
        const uint64_t bytes = tab.bytes[s];
        const uint64_t nvec = bytes >> 4;
        void* d = tab.dst[s];
        const void* p = tab.src[s];
        if (v0 - tid + HG_TILE_VECS <= nvec) {
            u32x4 a[HG_UNROLL], b[HG_UNROLL];
#pragma unroll
            for (uint32_t u = 0; u < HG_UNROLL; ++u) a[u] = ldv<HG_NT_LD_DST>(d, v0 + u * HG_BLOCK);
#pragma unroll
            for (uint32_t u = 0; u < HG_UNROLL; ++u) b[u] = ldv<HG_NT_LD_SRC>(p, v0 + u * HG_BLOCK);
#pragma unroll
            for (uint32_t u = 0; u < HG_UNROLL; ++u) stv<STREAM || HG_NT_ST>(d, v0 + u * HG_BLOCK, vec_op<DT, OP>(a[u], b[u]));
        } else {
#pragma unroll
            for (uint32_t u = 0; u < HG_UNROLL; ++u) {
                const uint64_t v = v0 + u * HG_BLOCK;
                if (v < nvec) stv<STREAM || HG_NT_ST>(d, v, vec_op<DT, OP>(ldv<HG_NT_LD_DST>(d, v), ldv<HG_NT_LD_SRC>(p, v)));
            }
            const uint64_t b = (nvec << 4) + (uint64_t)tid * ES; // element tail, fewer than 16 / ES elements
            if (b + ES <= bytes) {
                uint8_t* de = (uint8_t*)d + b;
                st_elem<ES>(de, word_op<DT, OP>(ld_elem<ES>(de), ld_elem<ES>((const uint8_t*)p + b)));
            }
        }
    }
}

// ---- element-at-a-time fallback for pointers that are not 16-byte aligned --------------------------------

template <int DT, int OP, bool REDUCE> __global__ __launch_bounds__(HG_BLOCK) void k_bytewise(const HgSeg2Table tab)
{
    constexpr uint32_t ES = REDUCE ? ElemSize<DT>::v : 1u;
    const uint32_t total = tab.tile_begin[tab.nseg];
    for (uint32_t tile = block_id<HG_XCD_REMAP>(); tile < total; tile += gridDim.x) {
        const uint32_t s = find_seg(tab.tile_begin, tab.nseg, tile);
        const uint64_t e0 = (uint64_t)(tile - tab.tile_begin[s]) * HG_TILE_VECS + threadIdx.x;
        const uint64_t nelem = tab.bytes[s] / ES;
        uint8_t* d = (uint8_t*)tab.dst[s];
        const uint8_t* p = (const uint8_t*)tab.src[s];
#pragma unroll
        for (uint32_t u = 0; u < HG_UNROLL; ++u) {
            const uint64_t e = e0 + u * HG_BLOCK;
            if (e < nelem) {
                if (REDUCE) st_elem<ES>(d + e * ES, word_op<DT, OP>(ld_elem<ES>(d + e * ES), ld_elem<ES>(p + e * ES)));
                else d[e] = p[e];
            }
        }
    }
}

// ---- k-way fold ---------------------------------------------------------------------------------
//
// Chain: acc = x0; for j = 1..k-1: acc = ACC_IS_DST ? acc (op) xj : xj (op) acc, optionally storing acc into
// xj's buffer, which reproduces k-1 successive two-input reduces while reading every input once.

__device__ __forceinline__ uint32_t fold_rank(const HgFoldTable& t, uint32_t s, uint32_t j)
{
    if (t.ascending) {
        if (j == 0) return t.first[s];
        return (j - 1 < t.first[s]) ? j - 1 : j;
    }
    int32_t r = (int32_t)t.first[s] + (int32_t)j * t.stride;
    const int32_t n = (int32_t)t.nranks;
    r %= n;
    if (r < 0) r += n;
    return (uint32_t)r;
}

template <int DT, int OP> struct VecItem {
    typedef u32x4 V;
    static __device__ __forceinline__ V zero() { return V{0u, 0u, 0u, 0u}; }
    static __device__ __forceinline__ V ld(const uint8_t* p, uint64_t i) { return ldv<HG_NT_LD_SRC>(p, i); }
    static __device__ __forceinline__ void st(uint8_t* p, uint64_t i, V v) { stv<HG_NT_FOLD_ST>(p, i, v); }
    static __device__ __forceinline__ V op(V d, V s) { return vec_op<DT, OP>(d, s); }
};

template <int DT, int OP> struct ElemItem {
    typedef uint32_t V;
    static constexpr uint32_t ES = ElemSize<DT>::v;
    static __device__ __forceinline__ V zero() { return 0u; }
    static __device__ __forceinline__ V ld(const uint8_t* p, uint64_t i) { return ld_elem<ES>(p + i * ES); }
    static __device__ __forceinline__ void st(uint8_t* p, uint64_t i, V v) { st_elem<ES>(p + i * ES, v); }
    static __device__ __forceinline__ V op(V d, V s) { return word_op<DT, OP>(d, s); }
};

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
    for (uint32_t tile = block_id<HG_XCD_REMAP>(); tile < total; tile += gridDim.x) {
        const uint32_t s = find_seg(tab.tile_begin, tab.nseg, tile);
        const uint64_t v0 = (uint64_t)(tile - tab.tile_begin[s]) * HG_TILE_VECS + tid;
        const uint64_t bytes = tab.bytes[s];
        const uint64_t nvec = bytes >> 4;
        bool live[HG_UNROLL];
        uint64_t idx[HG_UNROLL];
        const bool full = (v0 - tid + HG_TILE_VECS <= nvec);
#pragma unroll
        for (uint32_t u = 0; u < HG_UNROLL; ++u) {
            idx[u] = v0 + u * HG_BLOCK;
            live[u] = full || idx[u] < nvec;
        }
        fold_chain_items<VecItem<DT, OP>, ACC_IS_DST, HG_UNROLL>(tab, s, live, idx);
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
    for (uint32_t tile = block_id<HG_XCD_REMAP>(); tile < total; tile += gridDim.x) {
        const uint32_t s = find_seg(tab.tile_begin, tab.nseg, tile);
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

// ---- k-way tree fold (recursive halving) ---------------------------------------------------------
//
// K = 2^L block ranks.  For slice c, position q holds block rank c XOR bitrev(q); level l combines position q
// (dst role) with q + 2^l - exactly the reduce every halving step performs (peer = rank XOR mask, mask from K/2
// down to 1); each buffer receives the last value the step-wise replay would leave in it, and the root value
// goes to every output.
// A block rank with in2 != NULL first absorbs in2 (the odd neighbour folded in before the halving steps).

template <int L> __device__ __forceinline__ constexpr uint32_t bitrev(uint32_t q)
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
        if ((q & 1u) == 0u || tab.in2[b]) {
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
    V x[K][NU];
    uint32_t b[K];
#pragma unroll
    for (uint32_t q = 0; q < K; ++q) {
        b[q] = plus ? c + q : c + n - q;
        if (b[q] >= n) b[q] -= n;
        if (q < n) {
            const uint8_t* p = (const uint8_t*)tab.in[b[q]] + off;
#pragma unroll
            for (uint32_t u = 0; u < NU; ++u) x[q][u] = live[u] ? Item::ld(p, idx[u]) : Item::zero();
        }
    }
#pragma unroll
    for (int l = 0; l < L; ++l) {
#pragma unroll
        for (uint32_t q = 0; q < K; q += (2u << l))
            if (q + (1u << l) < n) {
#pragma unroll
                for (uint32_t u = 0; u < NU; ++u) x[q][u] = Item::op(x[q][u], x[q + (1u << l)][u]);
            }
    }
#pragma unroll
    for (uint32_t q = 0; q < K; q += 2)
        if (q + 1 < n) {
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

// A lane handles HG_TREE_NU(K) vectors: two while the 2 x K values fit comfortably in registers (K <= 8), else one.
template <int DT, int OP, int L> __global__ __launch_bounds__(HG_BLOCK) void k_fold_tree(const HgFoldTable tab)
{
    constexpr uint32_t ES = ElemSize<DT>::v;
    constexpr uint32_t NU = HG_TREE_NU(1u << L);
    const uint32_t total = tab.tile_begin[tab.nseg];
    const uint32_t tid = threadIdx.x;
    for (uint32_t tile = block_id<HG_XCD_REMAP>(); tile < total; tile += gridDim.x) {
        const uint32_t s = find_seg(tab.tile_begin, tab.nseg, tile);
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

// ---- dispatch -----------------------------------------------------------------------------------

int rc(hipError_t e) { return e == hipSuccess ? HCCL_SUCCESS : HCCL_E_RUNTIME; }

template <int DT, bool STREAM> int launch_reduce2_dt_s(hipStream_t st, int op, const HgSeg2Table* tab, uint32_t blocks)
{
    switch (op) {
        case OP_SUM: hipLaunchKernelGGL((k_reduce2<DT, OP_SUM, STREAM>), dim3(blocks), dim3(HG_BLOCK), 0, st, *tab); break;
        case OP_PROD: hipLaunchKernelGGL((k_reduce2<DT, OP_PROD, STREAM>), dim3(blocks), dim3(HG_BLOCK), 0, st, *tab); break;
        case OP_MAX: hipLaunchKernelGGL((k_reduce2<DT, OP_MAX, STREAM>), dim3(blocks), dim3(HG_BLOCK), 0, st, *tab); break;
        case OP_MIN: hipLaunchKernelGGL((k_reduce2<DT, OP_MIN, STREAM>), dim3(blocks), dim3(HG_BLOCK), 0, st, *tab); break;
        default: return HCCL_E_PARA;
    }
    return rc(hipGetLastError());
}

template <int DT> int launch_reduce2_dt(hipStream_t st, int op, const HgSeg2Table* tab, uint32_t blocks)
{
    uint64_t bytes = 0; /* what the launch writes */
    for (uint32_t s = 0; s < tab->nseg; ++s) bytes += tab->bytes[s];
    if (bytes > HG_STREAM_REDUCE_BYTES) return launch_reduce2_dt_s<DT, true>(st, op, tab, blocks);
    return launch_reduce2_dt_s<DT, false>(st, op, tab, blocks);
}

template <int DT> int launch_bytewise_dt(hipStream_t st, int op, const HgSeg2Table* tab, uint32_t blocks)
{
    switch (op) {
        case OP_SUM: hipLaunchKernelGGL((k_bytewise<DT, OP_SUM, true>), dim3(blocks), dim3(HG_BLOCK), 0, st, *tab); break;
        case OP_PROD: hipLaunchKernelGGL((k_bytewise<DT, OP_PROD, true>), dim3(blocks), dim3(HG_BLOCK), 0, st, *tab); break;
        case OP_MAX: hipLaunchKernelGGL((k_bytewise<DT, OP_MAX, true>), dim3(blocks), dim3(HG_BLOCK), 0, st, *tab); break;
        case OP_MIN: hipLaunchKernelGGL((k_bytewise<DT, OP_MIN, true>), dim3(blocks), dim3(HG_BLOCK), 0, st, *tab); break;
        default: return HCCL_E_PARA;
    }
    return rc(hipGetLastError());
}

template <int DT, bool AD> int launch_fold_dt(hipStream_t st, int op, const HgFoldTable* tab, uint32_t blocks)
{
    const dim3 g(blocks), b(HG_BLOCK);
    if (tab->small) {
        switch (op) {
            case OP_SUM: hipLaunchKernelGGL((k_fold_chain_small<DT, OP_SUM, AD>), g, b, 0, st, *tab); break;
            case OP_PROD: hipLaunchKernelGGL((k_fold_chain_small<DT, OP_PROD, AD>), g, b, 0, st, *tab); break;
            case OP_MAX: hipLaunchKernelGGL((k_fold_chain_small<DT, OP_MAX, AD>), g, b, 0, st, *tab); break;
            case OP_MIN: hipLaunchKernelGGL((k_fold_chain_small<DT, OP_MIN, AD>), g, b, 0, st, *tab); break;
            default: return HCCL_E_PARA;
        }
        return rc(hipGetLastError());
    }
    switch (op) {
        case OP_SUM: hipLaunchKernelGGL((k_fold_chain<DT, OP_SUM, AD>), g, b, 0, st, *tab); break;
        case OP_PROD: hipLaunchKernelGGL((k_fold_chain<DT, OP_PROD, AD>), g, b, 0, st, *tab); break;
        case OP_MAX: hipLaunchKernelGGL((k_fold_chain<DT, OP_MAX, AD>), g, b, 0, st, *tab); break;
        case OP_MIN: hipLaunchKernelGGL((k_fold_chain<DT, OP_MIN, AD>), g, b, 0, st, *tab); break;
        default: return HCCL_E_PARA;
    }
    return rc(hipGetLastError());
}

template <int DT, int L> int launch_tree_dt_l(hipStream_t st, int op, const HgFoldTable* tab, uint32_t blocks)
{
    switch (op) {
        case OP_SUM: hipLaunchKernelGGL((k_fold_tree<DT, OP_SUM, L>), dim3(blocks), dim3(HG_BLOCK), 0, st, *tab); break;
        case OP_PROD: hipLaunchKernelGGL((k_fold_tree<DT, OP_PROD, L>), dim3(blocks), dim3(HG_BLOCK), 0, st, *tab); break;
        case OP_MAX: hipLaunchKernelGGL((k_fold_tree<DT, OP_MAX, L>), dim3(blocks), dim3(HG_BLOCK), 0, st, *tab); break;
        case OP_MIN: hipLaunchKernelGGL((k_fold_tree<DT, OP_MIN, L>), dim3(blocks), dim3(HG_BLOCK), 0, st, *tab); break;
        default: return HCCL_E_PARA;
    }
    return rc(hipGetLastError());
}

template <int DT> int launch_tree_dt(hipStream_t st, int op, const HgFoldTable* tab, uint32_t blocks)
{
    switch (tab->k) {
        case 2: return launch_tree_dt_l<DT, 1>(st, op, tab, blocks);
        case 4: return launch_tree_dt_l<DT, 2>(st, op, tab, blocks);
        case 8: return launch_tree_dt_l<DT, 3>(st, op, tab, blocks);
        case 16: return launch_tree_dt_l<DT, 4>(st, op, tab, blocks);
        case 32: return launch_tree_dt_l<DT, 5>(st, op, tab, blocks);
        default: return HCCL_E_PARA;
    }
}

#define HG_DISPATCH_DT(dtype, CALL)                   \
    switch (dtype) {                                  \
        case DT_I8: return CALL(DT_I8);               \
        case DT_I16: return CALL(DT_I16);             \
        case DT_I32: return CALL(DT_I32);             \
        case DT_F16: return CALL(DT_F16);             \
        case DT_F32: return CALL(DT_F32);             \
        case DT_BF16: return CALL(DT_BF16);           \
        default: return HCCL_E_PARA;                  \
    }

} // namespace

extern "C" {

int hg_launch_copy(void* stream, const HgSeg2Table* tab, uint64_t blocks)
{
    if (blocks == 0) return HCCL_SUCCESS;
    uint64_t bytes = 0;
    for (uint32_t s = 0; s < tab->nseg; ++s) bytes += tab->bytes[s];
    if (bytes > HG_STREAM_COPY_BYTES)
        hipLaunchKernelGGL(k_copy<true>, dim3((uint32_t)blocks), dim3(HG_BLOCK), 0, (hipStream_t)stream, *tab);
    else
        hipLaunchKernelGGL(k_copy<false>, dim3((uint32_t)blocks), dim3(HG_BLOCK), 0, (hipStream_t)stream, *tab);
    return rc(hipGetLastError());
}

int hg_launch_reduce2(void* stream, int dtype, int op, const HgSeg2Table* tab, uint64_t blocks)
{
    if (blocks == 0) return HCCL_SUCCESS;
#define CALL(DT) launch_reduce2_dt<DT>((hipStream_t)stream, op, tab, (uint32_t)blocks)
    HG_DISPATCH_DT(dtype, CALL)
#undef CALL
}

int hg_launch_bytewise(void* stream, int is_reduce, int dtype, int op, const HgSeg2Table* tab, uint64_t blocks)
{
    if (blocks == 0) return HCCL_SUCCESS;
    if (!is_reduce) {
        hipLaunchKernelGGL((k_bytewise<DT_I8, OP_SUM, false>), dim3((uint32_t)blocks), dim3(HG_BLOCK), 0,
                           (hipStream_t)stream, *tab);
        return rc(hipGetLastError());
    }
#define CALL(DT) launch_bytewise_dt<DT>((hipStream_t)stream, op, tab, (uint32_t)blocks)
    HG_DISPATCH_DT(dtype, CALL)
#undef CALL
}

int hg_launch_fold(void* stream, int dtype, int op, int acc_is_dst, const HgFoldTable* tab, uint64_t blocks)
{
    if (blocks == 0) return HCCL_SUCCESS;
    if (tab->tree) {
#define CALL(DT) launch_tree_dt<DT>((hipStream_t)stream, op, tab, (uint32_t)blocks)
        HG_DISPATCH_DT(dtype, CALL)
#undef CALL
    }
    if (acc_is_dst) {
#define CALL(DT) launch_fold_dt<DT, true>((hipStream_t)stream, op, tab, (uint32_t)blocks)
        HG_DISPATCH_DT(dtype, CALL)
#undef CALL
    } else {
#define CALL(DT) launch_fold_dt<DT, false>((hipStream_t)stream, op, tab, (uint32_t)blocks)
        HG_DISPATCH_DT(dtype, CALL)
#undef CALL
    }
}

// ---- HIP runtime wrappers for the C host files -----------------------------------------------------------

int hg_rt_device_count(void)
{
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) return 0;
    return n;
}
int hg_rt_stream_create(void** stream) { return rc(hipStreamCreateWithFlags((hipStream_t*)stream, hipStreamNonBlocking)); }
int hg_rt_stream_destroy(void* stream) { return rc(hipStreamDestroy((hipStream_t)stream)); }
int hg_rt_stream_sync(void* stream) { return rc(hipStreamSynchronize((hipStream_t)stream)); }
int hg_rt_event_create(void** ev) { return rc(hipEventCreateWithFlags((hipEvent_t*)ev, hipEventDisableTiming)); }
int hg_rt_event_destroy(void* ev) { return rc(hipEventDestroy((hipEvent_t)ev)); }
int hg_rt_event_record(void* ev, void* stream) { return rc(hipEventRecord((hipEvent_t)ev, (hipStream_t)stream)); }
int hg_rt_stream_wait_event(void* stream, void* ev) { return rc(hipStreamWaitEvent((hipStream_t)stream, (hipEvent_t)ev, 0)); }
int hg_rt_malloc(void** p, size_t n) { return hipMalloc(p, n) == hipSuccess ? HCCL_SUCCESS : HCCL_E_MEMORY; }
int hg_rt_free(void* p) { return rc(hipFree(p)); }
int hg_rt_stream_is_capturing(void* stream)
{
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing((hipStream_t)stream, &st) != hipSuccess) return 1; /* unknown: treat as busy */
    return st != hipStreamCaptureStatusNone;
}
int hg_rt_capture_begin(void* stream) { return rc(hipStreamBeginCapture((hipStream_t)stream, hipStreamCaptureModeThreadLocal)); }
int hg_rt_capture_end(void* stream, void** graph_exec)
{
    hipGraph_t g = nullptr;
    *graph_exec = nullptr;
    if (hipStreamEndCapture((hipStream_t)stream, &g) != hipSuccess || !g) return HCCL_E_RUNTIME;
    hipGraphExec_t e = nullptr;
    const hipError_t err = hipGraphInstantiate(&e, g, nullptr, nullptr, 0);
    (void)hipGraphDestroy(g);
    if (err != hipSuccess) return HCCL_E_RUNTIME;
    *graph_exec = e;
    return HCCL_SUCCESS;
}
int hg_rt_graph_launch(void* graph_exec, void* stream) { return rc(hipGraphLaunch((hipGraphExec_t)graph_exec, (hipStream_t)stream)); }
int hg_rt_graph_destroy(void* graph_exec) { return rc(hipGraphExecDestroy((hipGraphExec_t)graph_exec)); }
int hg_rt_num_cus(void)
{
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
    return n;
}

} // extern "C"
