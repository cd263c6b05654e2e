/* HcommGfxAllReduceLocalReduceNoAlloc must not allocate on the host either: the library's C files are linked with
 * stand-ins for the HIP layer that play one GPU (stubs.c, -DHG_STUB_GPU_PRESENT) and with the linker's --wrap of malloc,
 * calloc, realloc and free, which counts every call the library's code makes while the entry point runs. */
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#include "hcomm_gfx.h"

extern unsigned long hg_stub_launches;
void* __real_malloc(size_t n);
void* __real_calloc(size_t a, size_t b);
void* __real_realloc(void* p, size_t n);
void __real_free(void* p);

static int counting = 0;
static unsigned long n_alloc = 0, n_free = 0;

void* __wrap_malloc(size_t n) { if (counting) ++n_alloc; return __real_malloc(n); }
void* __wrap_calloc(size_t a, size_t b) { if (counting) ++n_alloc; return __real_calloc(a, b); }
void* __wrap_realloc(void* p, size_t n) { if (counting) ++n_alloc; return __real_realloc(p, n); }
void __wrap_free(void* p) { if (counting) ++n_free; __real_free(p); }

int main(void)
{
    ThreadHandle th = 0;
    if (HcommThreadAllocWithStream(COMM_ENGINE_CPU_TS, (void*)(uintptr_t)0x5000, 0, &th) != 0) return 2;
    void* in[8];
    void* out[8];
    for (int r = 0; r < 8; ++r) {
        in[r] = (void*)(uintptr_t)(0x7f0000000000ull + ((uint64_t)r << 32));
        out[r] = (void*)(uintptr_t)(0x7e0000000000ull + ((uint64_t)r << 32));
    }
    int bad = 0;
    unsigned long calls = 0;
    const uint32_t ns[] = {1, 2, 4, 8};
    const uint64_t counts[] = {0, 1, 4099, 1 << 20, (1 << 20) + 37};
    const int dts[] = {HCOMM_DATA_TYPE_BFP16, HCOMM_DATA_TYPE_FP32, HCOMM_DATA_TYPE_INT8};
    for (int pass = 0; pass < 2; ++pass) /* the second pass finds every lazily read setting already read */
        for (unsigned ni = 0; ni < 4; ++ni)
            for (unsigned ci = 0; ci < 5; ++ci)
                for (unsigned di = 0; di < 3; ++di) {
                    const unsigned long before = hg_stub_launches;
                    counting = 1;
                    const int32_t rc = HcommGfxAllReduceLocalReduceNoAlloc(th, ns[ni], in, out, counts[ci], dts[di], HCOMM_REDUCE_SUM);
                    counting = 0;
                    ++calls;
                    if (rc != 0) ++bad;
                    if (counts[ci] != 0 && hg_stub_launches == before) ++bad; /* it did reach the launches */
                }
    /* refusals allocate nothing either */
    counting = 1;
    if (HcommGfxAllReduceLocalReduceNoAlloc(th, 8, in, out, 1ull << 40, HCOMM_DATA_TYPE_BFP16, HCOMM_REDUCE_SUM) == 0) ++bad;
    if (HcommGfxAllReduceLocalReduceNoAlloc(th, 9, in, out, 16, HCOMM_DATA_TYPE_BFP16, HCOMM_REDUCE_SUM) == 0) ++bad;
    counting = 0;
    HcommThreadFreeWithStream(&th, 1);
    printf("calls %lu launches %lu allocations %lu frees %lu bad %d\n", calls, hg_stub_launches, n_alloc, n_free, bad);
    return (bad || n_alloc || n_free) ? 1 : 0;
}
