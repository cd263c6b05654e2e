// hg_device.hpp - what the kernel translation units of libhcomm_gfx.so share: element arithmetic, 128-bit
// accesses with cache hints, the workgroup -> tile numbering and the launch helpers.
//
// Element semantics (the reference's "dst = dst (op) src", src/legacy/ascend910/platform/task/
// dispatcher_common.cc:137-147; CPU witnesses test/ut/stub/llt_hccl_stub.cc:4077-4204 and
// test/hccl_vm/src/plugin/runner/runner_utils/hccl_task_reduce_process.cc:18-55):
//   SUM a+b, PROD a*b, MAX (src > dst) ? src : dst, MIN (src < dst) ? src : dst;
//   integers wrap in two's complement; fp32 is one IEEE operation; fp16 / bf16 widen to fp32, operate,
//   and round to nearest even back to the storage type after every operation
//   (test/hccl_vm/src/plugin/runner/ccu_executor/ccu_fp16.h:39-66,102-135); a NaN result of SUM / PROD on a
//   16-bit type is stored as sign | 0x7e00 (fp16, ccu_fp16.h:121) or sign | 0x7fc0 (bf16, by analogy).

#pragma once
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

// A NaN result takes its canonical pattern either by a select (BR = false: both patterns computed, no branch) or by a
// branch (BR = true: the compiler masks the rare path off, and a vector instruction whose lanes are all masked off
// costs an issue slot instead of a pass through the lanes).  Measured both ways: the two-input reduce, which has
// little arithmetic per byte, is faster with the select (ring step 58.6 -> 57.4 us), the k-way folds with the
// branch (8 x 4 MiB fp16 mesh allreduce in one launch 40.1 -> 36.4 us).
template <bool BR> __device__ __forceinline__ uint32_t f32_to_f16(float f)
{
    if (BR) {
        if (f != f) return ((f32_bits(f) >> 16) & 0x8000u) | 0x7e00u;
        return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)f);
    }
    const uint32_t nan = ((f32_bits(f) >> 16) & 0x8000u) | 0x7e00u;
    const uint32_t r = (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)f);
    return (f != f) ? nan : r;
}

__device__ __forceinline__ float bf16_to_f32(uint32_t h) { return bits_f32(h << 16); }

template <bool BR> __device__ __forceinline__ uint32_t f32_to_bf16(float f)
{
    const uint32_t u = f32_bits(f);
    if (BR) {
        if (f != f) return ((u >> 16) & 0x8000u) | 0x7fc0u;
        return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
    }
    const uint32_t nan = ((u >> 16) & 0x8000u) | 0x7fc0u;
    const uint32_t r = (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
    return (f != f) ? nan : r;
}

// one 16-bit float element held in the low half of a word
template <int DT, int OP, bool BR> __device__ __forceinline__ uint32_t half_op(uint32_t d, uint32_t s)
{
    const float fd = (DT == DT_F16) ? f16_to_f32(d) : bf16_to_f32(d);
    const float fs = (DT == DT_F16) ? f16_to_f32(s) : bf16_to_f32(s);
    if (OP == OP_MAX) return (fs > fd) ? s : d;
    if (OP == OP_MIN) return (fs < fd) ? s : d;
    float r = (OP == OP_SUM) ? fd + fs : fd * fs;
    // The fp32 result is made opaque before it is narrowed: seeing widen - multiply - narrow in one expression, the
    // compiler may select a mixed-precision fused multiply-add with an addend of +0 for it, and (-0) * x + (+0) is +0
    // where the product alone is -0 (found by the signed-zero inputs of the parity suite on the element tail).
    if (DT == DT_F16) asm("" : "+v"(r));
    return (DT == DT_F16) ? f32_to_f16<BR>(r) : f32_to_bf16<BR>(r);
}

// ---- one 32-bit word of packed elements: returns d (op) s, d in the dst role ------------------------

template <int DT, int OP, bool BR = false> __device__ __forceinline__ uint32_t word_op(uint32_t d, uint32_t s)
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
    const uint32_t lo = half_op<DT, OP, BR>(d & 0xffffu, s & 0xffffu);
    const uint32_t hi = half_op<DT, OP, BR>(d >> 16, s >> 16);
    return lo | (hi << 16);
}

// ---- SUM / PROD of two packed 16-bit floats per word on the hardware's packed conversions ------------------------
//
// gfx950 narrows two fp32 values to two bf16 (or two fp16) in one instruction, round to nearest even, which is the
// rounding the element semantics ask for; widening is a shift / mask (bf16) or one conversion (fp16).  What the
// instruction does not do is store a NaN as sign | 0x7fc0 (sign | 0x7e00): it keeps the payload.  So a NaN result is
// replaced, still in fp32, by sign | 0x7fc00000, whose narrowing is exactly the canonical pattern of either type:
// three instructions an element, no branch (a branch per vector that only a wavefront with a NaN takes was tried
// and costs the fold kernels up to 45 %: it cuts the straight-line code their load scheduling relies on).  13 vector
// instructions per word of two elements where the element-by-element path needs 17 to 21.
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float canonical_nan_f32(float r)
{
    const float nan = bits_f32((f32_bits(r) & 0x80000000u) | 0x7fc00000u);
    return (r != r) ? nan : r;
}

template <int DT, int OP> __device__ __forceinline__ uint32_t pair_op_fast(uint32_t d, uint32_t s)
{
    float dl, dh, sl, sh;
    if (DT == DT_BF16) {
        dl = bits_f32(d << 16), dh = bits_f32(d & 0xffff0000u);
        sl = bits_f32(s << 16), sh = bits_f32(s & 0xffff0000u);
    } else {
        const f16x2 dv = __builtin_bit_cast(f16x2, d), sv = __builtin_bit_cast(f16x2, s);
        dl = (float)dv.x, dh = (float)dv.y, sl = (float)sv.x, sh = (float)sv.y;
    }
    float rl = (OP == OP_SUM) ? dl + sl : dl * sl, rh = (OP == OP_SUM) ? dh + sh : dh * sh;
    if (DT == DT_F16) asm("" : "+v"(rl), "+v"(rh)); // keeps the compiler from fusing widen - multiply - narrow (see half_op)
    const f32x2 r = {canonical_nan_f32(rl), canonical_nan_f32(rh)};
    if (DT == DT_BF16) return __builtin_bit_cast(uint32_t, __builtin_convertvector(r, bf16x2));
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(r, f16x2));
}

template <int DT, int OP, bool BR> __device__ __forceinline__ u32x4 vec_op_exact(u32x4 d, u32x4 s)
{
    u32x4 r;
    r.x = word_op<DT, OP, BR>(d.x, s.x);
    r.y = word_op<DT, OP, BR>(d.y, s.y);
    r.z = word_op<DT, OP, BR>(d.z, s.z);
    r.w = word_op<DT, OP, BR>(d.w, s.w);
    return r;
}

// BR = false: the packed conversions for the 16-bit floats (the two-input reduce and the small fold launches: ring step
// 57.0 -> 56.5 us, 8 x 4 MiB fp16 mesh allreduce in one launch 36.7 -> 35.3 us); BR = true: element by element with the
// NaN pattern behind a branch, which the large fold launches keep - with the lighter arithmetic they run 1 - 7 % slower
// at the launch shapes fitted to them (NHR 0.458 -> 0.476 ms, deterministic mesh allreduce 0.358 -> 0.383).
template <int DT, int OP, bool BR = false> __device__ __forceinline__ u32x4 vec_op(u32x4 d, u32x4 s)
{
    if (!BR && (DT == DT_BF16 || DT == DT_F16) && (OP == OP_SUM || OP == OP_PROD)) {
        u32x4 r;
        r.x = pair_op_fast<DT, OP>(d.x, s.x);
        r.y = pair_op_fast<DT, OP>(d.y, s.y);
        r.z = pair_op_fast<DT, OP>(d.z, s.z);
        r.w = pair_op_fast<DT, OP>(d.w, s.w);
        return r;
    }
    return vec_op_exact<DT, OP, BR>(d, s);
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

// Cache hints of the loads.  Measured with a stand-alone streaming probe built on this header, on 8 x 16 MiB ring steps and on
// 16 x 64 MiB launches whose operands nothing touched recently:
//   * small launches (a reduce that writes up to 64 MiB): peer operand loaded non-temporal, the operand that is
//     overwritten loaded plain;
//   * large ones: every load non-temporal, and no more than three workgroups per CU in flight - with the sc1
//     stores this is ahead on the ring steps too, although the next step reads their output back.
// The stores' policies follow further down.
#ifndef HG_NT_LD_SRC
#define HG_NT_LD_SRC 1 /* the peer's operand */
#endif
// Every operand of these kernels is device memory (the primitives' contract, include/hcomm_primitives.h:150), so the
// accesses name the global address space outright: a pointer that came out of a by-value table, or through the asm
// of arrive_together, is a generic one to the compiler, and generic 128-bit loads are FLAT instructions, which count
// on both memory counters and are waited for all at once.
typedef __attribute__((address_space(1))) u32x4 gvec;
typedef const __attribute__((address_space(1))) u32x4 cgvec;
template <bool NT> __device__ __forceinline__ u32x4 ldv(const void* base, uint64_t vec)
{
    if (NT) return __builtin_nontemporal_load((cgvec*)base + vec);
    return ((cgvec*)base)[vec];
}
template <bool NT> __device__ __forceinline__ void stv(void* base, uint64_t vec, u32x4 v)
{
    if (NT) __builtin_nontemporal_store(v, (gvec*)base + vec);
    else ((gvec*)base)[vec] = v;
}

// Store policies.  ST_SC1 carries the sc1 cache-policy bit (device scope) and neither of the other two: measured with
// 8 x 16 MiB ring steps and 16 x 64 MiB streams, with every access's policy bits spelled out, it is the best store for
// the copy / two-input reduce kernels in every situation (streaming reduce 0.825 -> 0.839 of peak over the
// non-temporal store, ring-step copy 0.845 -> 0.885 over the plain one).  The language has no 128-bit global store of
// a given scope; the buffer store builtin has: the policy rides in its aux operand, where the compiler sees it and
// schedules around the instruction like around any other store.  (Two 64-bit agent-scope atomic stores also come out
// as sc1 stores and run at half the speed; the instruction written in an asm needs hand-counted wait states behind it
// and ran 2 % slower on ring steps than the builtin, because the compiler cannot move anything across it.)
enum { ST_PLAIN = 0, ST_NT = 1, ST_SC1 = 2, ST_SC1_NT = 3 };
// the aux operand of the buffer store builtins on gfx940 and later: bit 1 = nt, bit 4 = sc1
template <int POL> struct StAux { static constexpr int v = (POL == ST_SC1) ? 16 : (POL == ST_SC1_NT) ? 18 : (POL == ST_NT) ? 2 : 0; };
#define HG_BUFFER_WORD3 0x00020000 /* descriptor word 3 of a raw buffer on gfx9: 32-bit data format, no swizzle */
template <int POL> __device__ __forceinline__ void stp(void* base, uint64_t vec, u32x4 v)
{
    gvec* p = (gvec*)base + vec;
    if (POL == ST_SC1 || POL == ST_SC1_NT) {
        // a buffer descriptor that starts at the address of the wave's first active lane (the lanes of a wave store to
        // ascending addresses), each lane at its distance from there
        const uint64_t a = (uint64_t)(uintptr_t)p;
        const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)a), hi = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32));
        const uint64_t a0 = ((uint64_t)hi << 32) | lo;
        __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc((void*)(uintptr_t)a0, 0, 0x7fffffff, HG_BUFFER_WORD3);
        __builtin_amdgcn_raw_buffer_store_b128(v, r, (int)(uint32_t)(a - a0), 0, StAux<POL>::v);
    } else if (POL == ST_NT) {
        __builtin_nontemporal_store(v, p);
    } else {
        *p = v;
    }
}
// The same store where the caller knows which part of the address the whole workgroup shares: `base` + 16 * `first`
// (kernel arguments and the workgroup's tile: scalar registers) and the lane's own vector `lane` behind it.
template <int POL> __device__ __forceinline__ void stp_tile(void* base, uint64_t first, uint32_t lane, u32x4 v)
{
    if (POL == ST_SC1 || POL == ST_SC1_NT) {
        __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc((u32x4*)base + first, 0, 0x7fffffff, HG_BUFFER_WORD3);
        __builtin_amdgcn_raw_buffer_store_b128(v, r, (int)(lane << 4), 0, StAux<POL>::v);
    } else {
        stp<POL>(base, first + lane, v);
    }
}

#ifndef HG_ST_SEG2
#define HG_ST_SEG2 ST_SC1 /* copy / two-input reduce kernels, kept and streaming variants alike */
#endif
#ifndef HG_ST_STREAM
#define HG_ST_STREAM ST_SC1 /* streaming variants; ST_SC1_NT there: halving-doubling + 0.6 %, the other large workloads - 1 .. - 2 % */
#endif
#ifndef HG_ST_REDUCE_KEPT
#define HG_ST_REDUCE_KEPT ST_SC1 /* the kept variant of the two-input reduce; ST_NT there: ring step 59.3 -> 59.9 us, mesh step 15.4 -> 16.3 us */
#endif
#ifndef HG_ST_FOLD
#define HG_ST_FOLD ST_NT /* the k-way folds at bandwidth-bound sizes (8 - 23 streams a lane): sc1 loses there (tree launches - 8 %) */
#endif
#ifndef HG_ST_FOLD_DIRECT
#define HG_ST_FOLD_DIRECT ST_SC1 /* the small, cache-resident fold launches (mesh allreduce 8 x 4 MiB in one launch: 41.8 -> 37.0 us) */
#endif

// Workgroups are dealt to the 8 XCDs round-robin by their index.  With run > 0 they are renumbered so that each XCD
// walks runs of `run` consecutive tiles instead of every eighth tile; the workgroups beyond the last whole group of
// 8 * run keep their numbers.  run == 0: as dealt.
__device__ __forceinline__ uint32_t block_id(uint32_t run, uint32_t g, uint32_t b)
{
    if (run == 0u) return b;
    const uint32_t span = 8u * run;
    if (b >= g - g % span) return b;
    const uint32_t i = b >> 3;
    return (i / run) * span + (b & 7u) * run + i % run;
}
__device__ __forceinline__ uint32_t block_id(uint32_t run) { return block_id(run, gridDim.x, blockIdx.x); }

// The same deal walked backwards in time: workgroup b gets the tile that the workgroup which its XCD runs at the
// mirrored moment gets above - the k-th workgroup of an XCD takes what the k-th from the end would have taken - so a
// launch starts on the tiles the forward deal ends with, and every tile stays on the XCD the forward deal gives it
// to.  The few workgroups beyond the last whole group of 8 keep their tiles.
__device__ __forceinline__ uint32_t block_id_backwards(uint32_t run, uint32_t g, uint32_t b)
{
    const uint32_t whole = g & ~7u;
    if (b >= whole) return block_id(run, g, b);
    return block_id(run, g, ((whole >> 3) - 1u - (b >> 3)) * 8u + (b & 7u));
}

// The point by which all the given scalar values must have arrived: the loads that fetch them (kernel arguments, the
// grid size) are all issued before it and waited for once, instead of each where the compiler first needs its value.
template <class A, class B, class C, class D, class E>
__device__ __forceinline__ void arrive_together(A& a, B& b, C& c, D& d, E& e)
{
    asm volatile("" : "+s"(a), "+s"(b), "+s"(c), "+s"(d), "+s"(e));
}

// segment that owns a tile: the last s with tile_begin[s] <= tile (uniform across the workgroup, so the bisection
// runs on the scalar unit: at most 6 probes for the largest table).  Every probe is a scalar load that waits for the
// one before it, so launches whose segments are one tile each (small messages) say so and skip the search.
__device__ __forceinline__ uint32_t find_seg(const uint32_t* tile_begin, uint32_t nseg, uint32_t tile)
{
    uint32_t lo = 0, hi = nseg; // tile_begin[lo] <= tile < tile_begin[hi]
    while (hi - lo > 1u) {
        const uint32_t mid = (lo + hi) >> 1;
        if (tile >= tile_begin[mid]) lo = mid;
        else hi = mid;
    }
    return lo;
}

template <class Table> __device__ __forceinline__ uint32_t seg_of(const Table& tab, uint32_t tile)
{
    return tab.flat ? tile : find_seg(tab.tile_begin, tab.nseg, tile);
}

template <int DT, int OP, int ST = HG_ST_FOLD, bool BR = true> struct VecItem {
    typedef u32x4 V;
    static __device__ __forceinline__ V zero() { return V{0u, 0u, 0u, 0u}; }
    static __device__ __forceinline__ V ld(const uint8_t* p, uint64_t i) { return ldv<HG_NT_LD_SRC>(p, i); }
    static __device__ __forceinline__ void st(uint8_t* p, uint64_t i, V v) { stp<ST>(p, i, v); }
    static __device__ __forceinline__ V op(V d, V s) { return vec_op<DT, OP, BR>(d, s); }
};

template <int DT, int OP> struct ElemItem {
    typedef uint32_t V;
    static constexpr uint32_t ES = ElemSize<DT>::v;
    static __device__ __forceinline__ V zero() { return 0u; }
    static __device__ __forceinline__ V ld(const uint8_t* p, uint64_t i) { return ld_elem<ES>(p + i * ES); }
    static __device__ __forceinline__ void st(uint8_t* p, uint64_t i, V v) { st_elem<ES>(p + i * ES, v); }
    static __device__ __forceinline__ V op(V d, V s) { return word_op<DT, OP, true>(d, s); }
};


int rc(hipError_t e) { return e == hipSuccess ? HCCL_SUCCESS : HCCL_E_RUNTIME; }

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
