// ref_shim.cc - C entry points around reference code compiled from where it lies under the reference tree.
//
// TEST INFRASTRUCTURE ONLY.  Built by oracle/Makefile into oracle/_ref/libhcomm_ref.so when the reference
// tree is present; used by the test suite to check oracle/hcomm_oracle.c against the reference's own code:
//   * VirtualRunTime::MemReduceSum / MemReduceMin / MemReduceMax
//     (test/hccl_vm/src/plugin/runner/runner_utils/hccl_task_reduce_process.cc:57-147), and
//   * class FP16 (test/hccl_vm/src/plugin/runner/ccu_executor/ccu_fp16.h:24-148).
// No reference source is copied: the Makefile compiles hccl_task_reduce_process.cc in place and this file
// only includes the reference headers by path.
#include <cstdint>

#include "hccl_task_reduce_process.h"
#include "ccu_fp16.h"

extern "C" {

// length is in BYTES (MemReduceSumTemplate divides by sizeof(T), hccl_task_reduce_process.cc:23).
void ref_mem_reduce_sum(void* src, void* dst, uint32_t length, int dtype)
{
    VirtualRunTime::MemReduceSum(src, dst, length, static_cast<VirtualRunTime::HcclDataType>(dtype));
}
// NOTE: the reference's Min / Max loops start at element 1 (hccl_task_reduce_process.cc:36,50);
// element 0 is left untouched, and callers of this shim must compare from element 1 on.
void ref_mem_reduce_min(void* src, void* dst, uint32_t length, int dtype)
{
    VirtualRunTime::MemReduceMin(src, dst, length, static_cast<VirtualRunTime::HcclDataType>(dtype));
}
void ref_mem_reduce_max(void* src, void* dst, uint32_t length, int dtype)
{
    VirtualRunTime::MemReduceMax(src, dst, length, static_cast<VirtualRunTime::HcclDataType>(dtype));
}

uint16_t ref_fp16_from_float(float x) { return FP16(x).value; }
float ref_fp16_to_float(uint16_t h) { return FP16(static_cast<half>(h)).to_float(); }
uint16_t ref_fp16_add(uint16_t a, uint16_t b) { return (FP16(static_cast<half>(a)) + FP16(static_cast<half>(b))).value; }
uint16_t ref_fp16_mul(uint16_t a, uint16_t b) { return (FP16(static_cast<half>(a)) * FP16(static_cast<half>(b))).value; }
int ref_fp16_gt(uint16_t a, uint16_t b) { return FP16(static_cast<half>(a)) > FP16(static_cast<half>(b)); }
int ref_fp16_lt(uint16_t a, uint16_t b) { return FP16(static_cast<half>(a)) < FP16(static_cast<half>(b)); }

// bulk forms so that exhaustive sweeps do not pay one foreign call per value
void ref_fp16_from_float_n(const float* x, uint16_t* h, uint64_t n)
{
    for (uint64_t i = 0; i < n; ++i) h[i] = FP16(x[i]).value;
}
void ref_fp16_to_float_n(const uint16_t* h, float* x, uint64_t n)
{
    for (uint64_t i = 0; i < n; ++i) x[i] = FP16(static_cast<half>(h[i])).to_float();
}
}
