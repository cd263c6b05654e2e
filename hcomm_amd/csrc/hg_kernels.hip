// hg_kernels.hip - gfx950 kernels of libhcomm_gfx.so and their launchers.
//
// Everything here is HBM-bandwidth bound: one lane moves 128 bits per access, a workgroup of 256 lanes
// keeps HG_UNROLL such accesses per operand in flight (one 16 KiB tile per workgroup), and a launch covers a whole
// table of segments (all simulated ranks of one schedule step).  Two grid shapes: one-dimensional over the table's
// tiles, each workgroup finding its segment in the prefix sums (k_copy, k_reduce2, k_bytewise: any table), and
// (tile, segment) for tables whose segments are about equally long (k_copy_rows, k_reduce2_rows).
//

#include "hg_device.hpp"

namespace {

// Set in a table's xcd_run by the launchers: the launch walks its table from the end - the last segment's last tile
// goes to the first workgroup (see hg_submit for when and why).  The tiles stay what they are.
#define HG_BACKWARDS 0x80000000u

// ---- batched copy ------------------------------------------------------------------------------

// STREAM: the variant for large launches - a copy that writes more than the memory-side cache holds, a reduce that
// writes more than 64 MiB (hg_shape_seg2 in hg_batch.c decides, with the measurements behind both figures).  Every
// store of these kernels carries the sc1 policy (stp<HG_ST_SEG2> / stp<HG_ST_STREAM>, the same policy today), so the
// copy's two variants differ in their launch shape only - occupancy bound and XCD runs - and the reduce's also in how
// the overwritten operand is loaded (non-temporal when streaming).  The launch's dynamic LDS size is not used as
// memory: it bounds the workgroups a CU runs at once.
template <bool STREAM> __global__ __launch_bounds__(HG_BLOCK) void k_copy(const HgSeg2Table tab)
{
    const uint32_t total = tab.tile_begin[tab.nseg];
    const uint32_t tid = threadIdx.x;
    const uint32_t first = (tab.xcd_run & HG_BACKWARDS) ? block_id_backwards(tab.xcd_run & ~HG_BACKWARDS, gridDim.x, blockIdx.x)
                                                         : block_id(tab.xcd_run);
    for (uint32_t tile = first; tile < total; tile += gridDim.x) {
        const uint32_t s = seg_of(tab, tile);
        const uint64_t t0 = (uint64_t)(tile - tab.tile_begin[s]) * HG_TILE_VECS;
        const uint64_t v0 = t0 + tid;
        const uint64_t bytes = tab.bytes[s];
        const uint64_t nvec = bytes >> 4;
        void* d = tab.dst[s];
        const void* p = tab.src[s];
        if (v0 - tid + HG_TILE_VECS <= nvec) {
            u32x4 a[HG_UNROLL];
#pragma unroll
            for (uint32_t u = 0; u < HG_UNROLL; ++u) a[u] = ldv<HG_NT_LD_SRC>(p, v0 + u * HG_BLOCK);
#pragma unroll
            for (uint32_t u = 0; u < HG_UNROLL; ++u) stp_tile<(STREAM ? HG_ST_STREAM : HG_ST_SEG2)>(d, t0, tid + u * HG_BLOCK, a[u]);
        } else {
#pragma unroll
            for (uint32_t u = 0; u < HG_UNROLL; ++u) {
                const uint64_t v = v0 + u * HG_BLOCK;
                if (v < nvec) stp<(STREAM ? HG_ST_STREAM : HG_ST_SEG2)>(d, v, ldv<HG_NT_LD_SRC>(p, v));
            }
            const uint64_t b = (nvec << 4) + tid; // this tile is the segment's last one: byte tail
            if (b < bytes) ((uint8_t*)d)[b] = ((const uint8_t*)p)[b];
        }
    }
}

// ---- batched dst = dst (op) src -----------------------------------------------------------------

// STREAM as for k_copy; it also decides how the operand that is overwritten is loaded: non-temporal when the launch
// streams, plain when a later launch is to find the result in the memory-side cache.
template <int DT, int OP, bool STREAM> __global__ __launch_bounds__(HG_BLOCK) void k_reduce2(const HgSeg2Table tab)
{
    constexpr uint32_t ES = ElemSize<DT>::v;
    const uint32_t total = tab.tile_begin[tab.nseg];
    const uint32_t tid = threadIdx.x;
    const uint32_t first = (tab.xcd_run & HG_BACKWARDS) ? block_id_backwards(tab.xcd_run & ~HG_BACKWARDS, gridDim.x, blockIdx.x)
                                                         : block_id(tab.xcd_run);
    for (uint32_t tile = first; tile < total; tile += gridDim.x) {
        const uint32_t s = seg_of(tab, tile);
        const uint64_t t0 = (uint64_t)(tile - tab.tile_begin[s]) * HG_TILE_VECS;
        const uint64_t v0 = t0 + tid;
        const uint64_t bytes = tab.bytes[s];
        const uint64_t nvec = bytes >> 4;
        void* d = tab.dst[s];
        const void* p = tab.src[s];
        if (v0 - tid + HG_TILE_VECS <= nvec) {
            u32x4 a[HG_UNROLL], b[HG_UNROLL];
#pragma unroll
            for (uint32_t u = 0; u < HG_UNROLL; ++u) a[u] = ldv<STREAM>(d, v0 + u * HG_BLOCK);
#pragma unroll
            for (uint32_t u = 0; u < HG_UNROLL; ++u) b[u] = ldv<HG_NT_LD_SRC>(p, v0 + u * HG_BLOCK);
#pragma unroll
            for (uint32_t u = 0; u < HG_UNROLL; ++u) stp_tile<(STREAM ? HG_ST_STREAM : HG_ST_REDUCE_KEPT)>(d, t0, tid + u * HG_BLOCK, vec_op<DT, OP>(a[u], b[u]));
        } else {
#pragma unroll
            for (uint32_t u = 0; u < HG_UNROLL; ++u) {
                const uint64_t v = v0 + u * HG_BLOCK;
                if (v < nvec) stp<(STREAM ? HG_ST_STREAM : HG_ST_REDUCE_KEPT)>(d, v, vec_op<DT, OP>(ldv<STREAM>(d, v), ldv<HG_NT_LD_SRC>(p, v)));
            }
            const uint64_t b = (nvec << 4) + (uint64_t)tid * ES; // element tail, fewer than 16 / ES elements
            if (b + ES <= bytes) {
                uint8_t* de = (uint8_t*)d + b;
                st_elem<ES>(de, word_op<DT, OP>(ld_elem<ES>(de), ld_elem<ES>((const uint8_t*)p + b)));
            }
        }
    }
}

// ---- operands that are not on 16-byte boundaries ----------------------------------------------------------
//
// The few elements before dst's next 16-byte boundary go one by one; from there on dst is read and written in
// aligned 16-byte items like k_copy / k_reduce2 do.  src - as far from a boundary as it happens to be - is read in
// ALIGNED 16-byte vectors too: vector v of the 16-byte grid src sits in holds the first bytes of item v, the rest
// are in vector v + 1 = what the next lane has loaded (the last lane of a wavefront loads it itself), and the two
// are put together in registers.  (One unaligned 16-byte load per item - global memory takes them in the unaligned
// access mode the HSA ABI runs in - is served from two cache lines wherever it straddles them and ran at 0.72 of the
// HBM roofline where this runs at 0.83; reading the five dwords an item touches one by one was slower still.)  An
// aligned vector that holds one byte of the operand lies inside the operand's pages, so the up to 15 bytes read
// before its first and after its last byte never fault, and they are never used.  An item holds whole elements
// because dst and src are element-aligned and the head is a whole number of elements.  The bytes after the last
// whole item go one by one too; head and tail belong to the tile that holds the end of the items.

// Item v of src, which starts `off` bytes (1 ... 15) behind a 16-byte boundary, out of the two aligned vectors it
// straddles: bytes off ... off+15 of lo:hi.  `off` is the same for every item of a segment.
__device__ __forceinline__ u32x4 straddle(const u32x4 lo, const u32x4 hi, uint32_t off)
{
    const uint32_t c[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    const uint32_t r = off & 3u;
    u32x4 o;
    switch (off >> 2) { // uniform: a scalar branch
        case 0:
            o = u32x4{__builtin_amdgcn_alignbyte(c[1], c[0], r), __builtin_amdgcn_alignbyte(c[2], c[1], r),
                      __builtin_amdgcn_alignbyte(c[3], c[2], r), __builtin_amdgcn_alignbyte(c[4], c[3], r)};
            break;
        case 1:
            o = u32x4{__builtin_amdgcn_alignbyte(c[2], c[1], r), __builtin_amdgcn_alignbyte(c[3], c[2], r),
                      __builtin_amdgcn_alignbyte(c[4], c[3], r), __builtin_amdgcn_alignbyte(c[5], c[4], r)};
            break;
        case 2:
            o = u32x4{__builtin_amdgcn_alignbyte(c[3], c[2], r), __builtin_amdgcn_alignbyte(c[4], c[3], r),
                      __builtin_amdgcn_alignbyte(c[5], c[4], r), __builtin_amdgcn_alignbyte(c[6], c[5], r)};
            break;
        default:
            o = u32x4{__builtin_amdgcn_alignbyte(c[4], c[3], r), __builtin_amdgcn_alignbyte(c[5], c[4], r),
                      __builtin_amdgcn_alignbyte(c[6], c[5], r), __builtin_amdgcn_alignbyte(c[7], c[6], r)};
            break;
    }
    return o;
}

// The value lane + 1 of the wavefront holds (lane 63: its own).
__device__ __forceinline__ u32x4 from_next_lane(const u32x4 v)
{
    return u32x4{(uint32_t)__shfl_down((int)v.x, 1, 64), (uint32_t)__shfl_down((int)v.y, 1, 64),
                 (uint32_t)__shfl_down((int)v.z, 1, 64), (uint32_t)__shfl_down((int)v.w, 1, 64)};
}

// STREAM as for k_copy / k_reduce2.
template <int DT, int OP, bool REDUCE, bool STREAM> __global__ __launch_bounds__(HG_BLOCK) void k_bytewise(const HgSeg2Table tab)
{
    constexpr uint32_t ES = REDUCE ? ElemSize<DT>::v : 1u;
    const uint32_t total = tab.tile_begin[tab.nseg];
    const uint32_t tid = threadIdx.x;
    const uint32_t first = (tab.xcd_run & HG_BACKWARDS) ? block_id_backwards(tab.xcd_run & ~HG_BACKWARDS, gridDim.x, blockIdx.x)
                                                         : block_id(tab.xcd_run);
    for (uint32_t tile = first; tile < total; tile += gridDim.x) {
        const uint32_t s = seg_of(tab, tile);
        const uint64_t bytes = tab.bytes[s];
        uint8_t* d0 = (uint8_t*)tab.dst[s];
        const uint8_t* p0 = (const uint8_t*)tab.src[s];
        uint64_t head = (HG_VEC_BYTES - ((uintptr_t)d0 & (HG_VEC_BYTES - 1))) & (HG_VEC_BYTES - 1);
        if (head > bytes) head = bytes / ES * ES;
        uint8_t* d = d0 + head;      // on a 16-byte boundary (or past the end of a segment shorter than the head)
        const uint8_t* p = p0 + head;
        const uint64_t nvec = (bytes - head) >> 4;
        const uint64_t vb = (uint64_t)(tile - tab.tile_begin[s]) * HG_TILE_VECS;
        u32x4 a[HG_UNROLL], b[HG_UNROLL];
        const uint32_t skew = (uint32_t)((uintptr_t)p & (HG_VEC_BYTES - 1));
        const uint8_t* pa = p - skew;                            // the 16-byte grid src sits in
        const uint64_t nsrc = nvec + (skew != 0 && nvec != 0);  // aligned vectors that hold bytes of the items
        const bool last_lane = (tid & 63u) == 63u;
        u32x4 own[HG_UNROLL];
#pragma unroll
        for (uint32_t u = 0; u < HG_UNROLL; ++u) {
            const uint64_t v = vb + tid + u * HG_BLOCK;
            b[u] = u32x4{0, 0, 0, 0};
            own[u] = u32x4{0, 0, 0, 0};
            if (v < nsrc) b[u] = ldv<true>(pa, v);
            if (last_lane && v + 1 < nsrc) own[u] = ldv<true>(pa, v + 1);
            if (REDUCE && v < nvec) a[u] = ldv<STREAM>(d, v);
        }
#pragma unroll
        for (uint32_t u = 0; u < HG_UNROLL; ++u) {
            const u32x4 next = from_next_lane(b[u]); // every lane takes part, whatever it has to do itself
            if (skew != 0) b[u] = straddle(b[u], last_lane ? own[u] : next, skew);
        }
#pragma unroll
        for (uint32_t u = 0; u < HG_UNROLL; ++u) {
            const uint64_t v = vb + tid + u * HG_BLOCK;
            if (v < nvec) stp<(STREAM ? HG_ST_STREAM : HG_ST_SEG2)>(d, v, REDUCE ? vec_op<DT, OP>(a[u], b[u]) : b[u]);
        }
        if (vb <= nvec && vb + HG_TILE_VECS > nvec) { // the one tile that holds the end of the items
            // fewer than 16 / ES elements before the first item and fewer than that after the last one
            const uint64_t tail0 = head + (nvec << 4);
            const uint64_t off = (uint64_t)tid * ES < head ? (uint64_t)tid * ES : tail0 + ((uint64_t)tid * ES - head);
            if (off + ES <= bytes && (off < head || off >= tail0)) {
                if (REDUCE) st_elem<ES>(d0 + off, word_op<DT, OP>(ld_elem<ES>(d0 + off), ld_elem<ES>(p0 + off)));
                else d0[off] = p0[off];
            }
        }
    }
}

// ---- launches whose segments are (nearly) equally long: one round of argument reads ----------------------------
//
// A launch starts with a chain of dependent memory round trips (a quarter of a microsecond per round of argument
// reads, measured with a kernel that times its own first instructions; more for the data): kernel arguments,
// whatever they index, the data, the stores.  The kernels above find a tile's segment in the table's prefix sums
// and only then know which pointers to read: several rounds of argument reads before the first byte of data is
// asked for, paid by every launch of a schedule because a launch does not start before the one ahead of it has
// ended.  When the segments have (nearly) the same number of tiles - the slices of one step of a ring, halving
// or mesh schedule - the grid is two-dimensional instead, y = segment and x = tile of that segment (as wide as
// the longest segment; workgroups beyond a shorter segment's tiles find nothing to do): every argument a
// workgroup needs sits at an offset it knows from its own index, so all are read at once.  Same tiles, same
// arithmetic, same cache hints; the XCD runs are walked inside a segment's row (the workgroups of a row whose x
// is equal modulo 8 run on one XCD whatever the row's place in the grid).

// Launches of at most HG_DIRECT_SEG segments pass this table instead of the full one: the runtime copies the kernel
// arguments on every launch, and 200 bytes cost less there than 1.8 KB (half a microsecond to a microsecond per queued launch).
struct HgSeg2Few {
    void* dst[HG_DIRECT_SEG];
    const void* src[HG_DIRECT_SEG];
    uint64_t bytes[HG_DIRECT_SEG];
    uint32_t xcd_run;
};

// `backwards`: the rows in reverse order and the mark that makes a row's workgroups take its tiles from the end.
HgSeg2Few few_of(const HgSeg2Table& t, bool backwards)
{
    HgSeg2Few f;
    for (uint32_t s = 0; s < HG_DIRECT_SEG; ++s) {
        const uint32_t q = backwards ? t.nseg - 1u - s : s;
        f.dst[s] = s < t.nseg ? t.dst[q] : nullptr;
        f.src[s] = s < t.nseg ? t.src[q] : nullptr;
        f.bytes[s] = s < t.nseg ? t.bytes[q] : 0;
    }
    f.xcd_run = t.xcd_run | (backwards ? HG_BACKWARDS : 0u);
    return f;
}

HgSeg2Table backwards_of(const HgSeg2Table& t)
{
    HgSeg2Table r = t;
    for (uint32_t s = 0; s < t.nseg; ++s) {
        r.dst[s] = t.dst[t.nseg - 1u - s];
        r.src[s] = t.src[t.nseg - 1u - s];
        r.bytes[s] = t.bytes[t.nseg - 1u - s];
    }
    r.xcd_run = t.xcd_run | HG_BACKWARDS;
    return r;
}

template <bool STREAM, class Tab> __global__ __launch_bounds__(HG_BLOCK) void k_copy_rows(const Tab tab)
{
    const uint32_t s = blockIdx.y, tid = threadIdx.x;
    void* d = tab.dst[s];
    const void* p = tab.src[s];
    uint64_t bytes = tab.bytes[s];
    uint32_t run = tab.xcd_run, width = gridDim.x;
    arrive_together(d, p, bytes, run, width); // one round of argument reads
    // HG_BACKWARDS: the launch walks memory from its end (the host has turned the rows round)
    const uint32_t tile = (run & HG_BACKWARDS) ? block_id_backwards(run & ~HG_BACKWARDS, width, blockIdx.x) : block_id(run, width, blockIdx.x);
    const uint64_t nvec = bytes >> 4;
    const uint64_t t0 = (uint64_t)tile * HG_TILE_VECS;
    const uint64_t v0 = t0 + tid;
    if (v0 - tid + HG_TILE_VECS <= nvec) {
        u32x4 a[HG_UNROLL];
#pragma unroll
        for (uint32_t u = 0; u < HG_UNROLL; ++u) a[u] = ldv<HG_NT_LD_SRC>(p, v0 + u * HG_BLOCK);
#pragma unroll
        for (uint32_t u = 0; u < HG_UNROLL; ++u) stp_tile<(STREAM ? HG_ST_STREAM : HG_ST_SEG2)>(d, t0, tid + u * HG_BLOCK, a[u]);
    } else {
#pragma unroll
        for (uint32_t u = 0; u < HG_UNROLL; ++u) {
            const uint64_t v = v0 + u * HG_BLOCK;
            if (v < nvec) stp<(STREAM ? HG_ST_STREAM : HG_ST_SEG2)>(d, v, ldv<HG_NT_LD_SRC>(p, v));
        }
        if (tile == nvec / HG_TILE_VECS) { // the tile the byte tail falls into
            const uint64_t b = (nvec << 4) + tid;
            if (b < bytes) ((uint8_t*)d)[b] = ((const uint8_t*)p)[b];
        }
    }
}

template <int DT, int OP, bool STREAM, class Tab> __global__ __launch_bounds__(HG_BLOCK) void k_reduce2_rows(const Tab tab)
{
    constexpr uint32_t ES = ElemSize<DT>::v;
    const uint32_t s = blockIdx.y, tid = threadIdx.x;
    void* d = tab.dst[s];
    const void* p = tab.src[s];
    uint64_t bytes = tab.bytes[s];
    uint32_t run = tab.xcd_run, width = gridDim.x;
    arrive_together(d, p, bytes, run, width); // one round of argument reads
    // HG_BACKWARDS: the launch walks memory from its end (the host has turned the rows round)
    const uint32_t tile = (run & HG_BACKWARDS) ? block_id_backwards(run & ~HG_BACKWARDS, width, blockIdx.x) : block_id(run, width, blockIdx.x);
    const uint64_t nvec = bytes >> 4;
    const uint64_t t0 = (uint64_t)tile * HG_TILE_VECS;
    const uint64_t v0 = t0 + tid;
    if (v0 - tid + HG_TILE_VECS <= nvec) {
        u32x4 a[HG_UNROLL], b[HG_UNROLL];
#pragma unroll
        for (uint32_t u = 0; u < HG_UNROLL; ++u) a[u] = ldv<STREAM>(d, v0 + u * HG_BLOCK);
#pragma unroll
        for (uint32_t u = 0; u < HG_UNROLL; ++u) b[u] = ldv<HG_NT_LD_SRC>(p, v0 + u * HG_BLOCK);
#pragma unroll
        for (uint32_t u = 0; u < HG_UNROLL; ++u) stp_tile<(STREAM ? HG_ST_STREAM : HG_ST_REDUCE_KEPT)>(d, t0, tid + u * HG_BLOCK, vec_op<DT, OP>(a[u], b[u]));
    } else {
#pragma unroll
        for (uint32_t u = 0; u < HG_UNROLL; ++u) {
            const uint64_t v = v0 + u * HG_BLOCK;
            if (v < nvec) stp<(STREAM ? HG_ST_STREAM : HG_ST_REDUCE_KEPT)>(d, v, vec_op<DT, OP>(ldv<STREAM>(d, v), ldv<HG_NT_LD_SRC>(p, v)));
        }
        if (tile == nvec / HG_TILE_VECS) { // the tile the element tail falls into
            const uint64_t b = (nvec << 4) + (uint64_t)tid * ES;
            if (b + ES <= bytes) {
                uint8_t* de = (uint8_t*)d + b;
                st_elem<ES>(de, word_op<DT, OP>(ld_elem<ES>(de), ld_elem<ES>((const uint8_t*)p + b)));
            }
        }
    }
}

// ---- dispatch -----------------------------------------------------------------------------------

template <int DT, bool STREAM, class Tab>
int launch_reduce2_rows(hipStream_t st, int op, const Tab& tab, dim3 g, uint32_t lds)
{
    const dim3 b(HG_BLOCK);
    switch (op) {
        case OP_SUM: hipLaunchKernelGGL((k_reduce2_rows<DT, OP_SUM, STREAM, Tab>), g, b, lds, st, tab); break;
        case OP_PROD: hipLaunchKernelGGL((k_reduce2_rows<DT, OP_PROD, STREAM, Tab>), g, b, lds, st, tab); break;
        case OP_MAX: hipLaunchKernelGGL((k_reduce2_rows<DT, OP_MAX, STREAM, Tab>), g, b, lds, st, tab); break;
        case OP_MIN: hipLaunchKernelGGL((k_reduce2_rows<DT, OP_MIN, STREAM, Tab>), g, b, lds, st, tab); break;
        default: return HCCL_E_PARA;
    }
    return rc(hipGetLastError());
}

template <int DT, bool STREAM>
int launch_reduce2_dt_s(hipStream_t st, int op, const HgSeg2Table* tab, uint32_t blocks, uint32_t lds, bool backwards)
{
    const dim3 g(blocks), b(HG_BLOCK);
    if (tab->direct) {
        const dim3 g2(tab->direct, tab->nseg);
        if (tab->nseg <= HG_DIRECT_SEG) return launch_reduce2_rows<DT, STREAM, HgSeg2Few>(st, op, few_of(*tab, backwards), g2, lds);
        if (backwards) return launch_reduce2_rows<DT, STREAM, HgSeg2Table>(st, op, backwards_of(*tab), g2, lds);
        return launch_reduce2_rows<DT, STREAM, HgSeg2Table>(st, op, *tab, g2, lds);
    }
    switch (op) {
        case OP_SUM: hipLaunchKernelGGL((k_reduce2<DT, OP_SUM, STREAM>), g, b, lds, st, *tab); break;
        case OP_PROD: hipLaunchKernelGGL((k_reduce2<DT, OP_PROD, STREAM>), g, b, lds, st, *tab); break;
        case OP_MAX: hipLaunchKernelGGL((k_reduce2<DT, OP_MAX, STREAM>), g, b, lds, st, *tab); break;
        case OP_MIN: hipLaunchKernelGGL((k_reduce2<DT, OP_MIN, STREAM>), g, b, lds, st, *tab); break;
        default: return HCCL_E_PARA;
    }
    return rc(hipGetLastError());
}

template <int DT>
int launch_reduce2_dt(hipStream_t st, int op, const HgSeg2Table* tab, uint32_t blocks, int streaming, uint32_t lds, bool backwards)
{
    if (streaming) return launch_reduce2_dt_s<DT, true>(st, op, tab, blocks, lds, backwards);
    return launch_reduce2_dt_s<DT, false>(st, op, tab, blocks, lds, backwards);
}

template <bool STREAM> int launch_copy_s(hipStream_t st, const HgSeg2Table* tab, uint32_t blocks, uint32_t lds, bool backwards)
{
    const dim3 b(HG_BLOCK);
    if (tab->direct) {
        const dim3 g2(tab->direct, tab->nseg);
        if (tab->nseg <= HG_DIRECT_SEG)
            hipLaunchKernelGGL((k_copy_rows<STREAM, HgSeg2Few>), g2, b, lds, st, few_of(*tab, backwards));
        else if (backwards)
            hipLaunchKernelGGL((k_copy_rows<STREAM, HgSeg2Table>), g2, b, lds, st, backwards_of(*tab));
        else
            hipLaunchKernelGGL((k_copy_rows<STREAM, HgSeg2Table>), g2, b, lds, st, *tab);
    } else {
        hipLaunchKernelGGL(k_copy<STREAM>, dim3(blocks), b, lds, st, *tab);
    }
    return rc(hipGetLastError());
}

template <int DT, bool STREAM> int launch_bytewise_dt_s(hipStream_t st, int op, const HgSeg2Table* tab, uint32_t blocks, uint32_t lds)
{
    const dim3 g(blocks), b(HG_BLOCK);
    switch (op) {
        case OP_SUM: hipLaunchKernelGGL((k_bytewise<DT, OP_SUM, true, STREAM>), g, b, lds, st, *tab); break;
        case OP_PROD: hipLaunchKernelGGL((k_bytewise<DT, OP_PROD, true, STREAM>), g, b, lds, st, *tab); break;
        case OP_MAX: hipLaunchKernelGGL((k_bytewise<DT, OP_MAX, true, STREAM>), g, b, lds, st, *tab); break;
        case OP_MIN: hipLaunchKernelGGL((k_bytewise<DT, OP_MIN, true, STREAM>), g, b, lds, st, *tab); break;
        default: return HCCL_E_PARA;
    }
    return rc(hipGetLastError());
}

template <int DT> int launch_bytewise_dt(hipStream_t st, int op, const HgSeg2Table* tab, uint32_t blocks, int streaming, uint32_t lds)
{
    if (streaming) return launch_bytewise_dt_s<DT, true>(st, op, tab, blocks, lds);
    return launch_bytewise_dt_s<DT, false>(st, op, tab, blocks, lds);
}

} // namespace

extern "C" {


// The one-dimensional kernels walk the whole table from its last tile when the mark is set; the row grids also need
// their rows turned round (launch_*_s).
#define HG_MARK_ONE_DIMENSIONAL(tab, backwards)      \
    HgSeg2Table marked_;                              \
    if ((backwards) && !(tab)->direct) {              \
        marked_ = *(tab);                             \
        marked_.xcd_run |= HG_BACKWARDS;              \
        (tab) = &marked_;                             \
    }

int hg_launch_copy(void* stream, const HgSeg2Table* tab, uint64_t blocks, int streaming, uint32_t lds, int backwards)
{
    if (blocks == 0) return HCCL_SUCCESS;
    HG_MARK_ONE_DIMENSIONAL(tab, backwards)
    if (streaming) return launch_copy_s<true>((hipStream_t)stream, tab, (uint32_t)blocks, lds, backwards != 0);
    return launch_copy_s<false>((hipStream_t)stream, tab, (uint32_t)blocks, lds, backwards != 0);
}

int hg_launch_reduce2(void* stream, int dtype, int op, const HgSeg2Table* tab, uint64_t blocks, int streaming, uint32_t lds, int backwards)
{
    if (blocks == 0) return HCCL_SUCCESS;
    HG_MARK_ONE_DIMENSIONAL(tab, backwards)
#define CALL(DT) launch_reduce2_dt<DT>((hipStream_t)stream, op, tab, (uint32_t)blocks, streaming, lds, backwards != 0)
    HG_DISPATCH_DT(dtype, CALL)
#undef CALL
}

int hg_launch_bytewise(void* stream, int is_reduce, int dtype, int op, const HgSeg2Table* tab, uint64_t blocks, int streaming,
                       uint32_t lds, int backwards)
{
    if (blocks == 0) return HCCL_SUCCESS;
    HgSeg2Table marked;
    if (backwards) {
        marked = *tab;
        marked.xcd_run |= HG_BACKWARDS;
        tab = &marked;
    }
    if (!is_reduce) {
        const dim3 g((uint32_t)blocks), b(HG_BLOCK);
        if (streaming) hipLaunchKernelGGL((k_bytewise<DT_I8, OP_SUM, false, true>), g, b, lds, (hipStream_t)stream, *tab);
        else hipLaunchKernelGGL((k_bytewise<DT_I8, OP_SUM, false, false>), g, b, lds, (hipStream_t)stream, *tab);
        return rc(hipGetLastError());
    }
#define CALL(DT) launch_bytewise_dt<DT>((hipStream_t)stream, op, tab, (uint32_t)blocks, streaming, lds)
    HG_DISPATCH_DT(dtype, CALL)
#undef CALL
}

// ---- device memory of the library's own, for callers that cannot allocate ---------------------------------
//
// One array per GPU, held from the moment the code object is loaded there until the process ends.  In host code the
// array's name is only a handle for hipGetSymbolAddress; kernels get the address that call returns, per device.

} // extern "C"

static __device__ __align__(256) uint8_t scratch[HCOMM_GFX_NOALLOC_SCRATCH_BYTES];

#define HG_MAX_DEVICES 64
static void* g_scratch_ptr[HG_MAX_DEVICES]; // device address of `scratch` on each GPU, once asked for

extern "C" {

// Address of the array's copy on the device `stream` belongs to (looked up once per device, with that device
// current; the calling thread's current device is left as it was).
int hg_rt_scratch(void* stream, void** ptr)
{
    int cur = -1;
    hipDevice_t sd;
    *ptr = nullptr;
    if (hipGetDevice(&cur) != hipSuccess) return HCCL_E_RUNTIME;
    int dev = cur;
    if (stream && hipStreamGetDevice((hipStream_t)stream, &sd) == hipSuccess) dev = (int)sd;
    if (dev < 0 || dev >= HG_MAX_DEVICES) return HCCL_E_RUNTIME;
    void* p = __atomic_load_n(&g_scratch_ptr[dev], __ATOMIC_ACQUIRE);
    if (!p) {
        if (dev != cur && hipSetDevice(dev) != hipSuccess) return HCCL_E_RUNTIME;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (dev != cur) (void)hipSetDevice(cur);
        if (e != hipSuccess || !p) return HCCL_E_RUNTIME;
        __atomic_store_n(&g_scratch_ptr[dev], p, __ATOMIC_RELEASE);
    }
    *ptr = p;
    return HCCL_SUCCESS;
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
