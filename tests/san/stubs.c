/* CPU stand-ins for the library's own HIP layer (hg_kernels*.hip), so that its C files link into a host-only
 * sanitizer build: launches and runtime calls report failure, nothing they would touch exists.
 * With -DHG_STUB_GPU_PRESENT the stand-ins play a machine with one GPU instead: streams and events are made-up
 * handles, launches succeed and are counted, the library's own device array is a host array - for checks of what the
 * host code does around a launch (tests/san/driver_noalloc.c). */
#include <stddef.h>
#include <stdint.h>
#include "hg_internal.h"
#ifdef HG_STUB_GPU_PRESENT
unsigned long hg_stub_launches = 0;
static char stub_scratch[256] __attribute__((aligned(256)));
int hg_launch_copy(void* s, const HgSeg2Table* t, uint64_t b, int m, uint32_t l, int w) { (void)s; (void)t; (void)b; (void)m; (void)l; (void)w; ++hg_stub_launches; return 0; }
int hg_launch_reduce2(void* s, int d, int o, const HgSeg2Table* t, uint64_t b, int m, uint32_t l, int w) { (void)s; (void)d; (void)o; (void)t; (void)b; (void)m; (void)l; (void)w; ++hg_stub_launches; return 0; }
int hg_launch_bytewise(void* s, int r, int d, int o, const HgSeg2Table* t, uint64_t b, int st, uint32_t l, int w) { (void)s; (void)r; (void)d; (void)o; (void)t; (void)b; (void)st; (void)l; (void)w; ++hg_stub_launches; return 0; }
int hg_launch_fold(void* s, int d, int o, int a, const HgFoldTable* t, uint64_t b, uint32_t l) { (void)s; (void)d; (void)o; (void)a; (void)t; (void)b; (void)l; ++hg_stub_launches; return 0; }
int hg_rt_device_count(void) { return 1; }
int hg_rt_scratch(void* s, void** p) { (void)s; *p = stub_scratch; return 0; } /* an address to do arithmetic on: never dereferenced */
int hg_rt_stream_create(void** s) { *s = (void*)(uintptr_t)0x5000; return 0; }
int hg_rt_stream_destroy(void* s) { (void)s; return 0; }
int hg_rt_stream_sync(void* s) { (void)s; return 0; }
int hg_rt_event_create(void** e) { *e = (void*)(uintptr_t)0x6000; return 0; }
int hg_rt_event_destroy(void* e) { (void)e; return 0; }
int hg_rt_event_record(void* e, void* s) { (void)e; (void)s; return 0; }
int hg_rt_stream_wait_event(void* s, void* e) { (void)e; (void)s; return 0; }
int hg_rt_malloc(void** p, size_t n) { (void)n; *p = NULL; return 4; }
int hg_rt_free(void* p) { (void)p; return 0; }
int hg_rt_num_cus(void) { return 256; }
int hg_rt_stream_is_capturing(void* s) { (void)s; return 0; }
int hg_rt_capture_begin(void* s) { (void)s; return 4; }
int hg_rt_capture_end(void* s, void** g) { (void)s; *g = NULL; return 4; }
int hg_rt_graph_launch(void* g, void* s) { (void)g; (void)s; return 4; }
int hg_rt_graph_destroy(void* g) { (void)g; return 0; }
#else
int hg_launch_copy(void* s, const HgSeg2Table* t, uint64_t b, int m, uint32_t l, int w) { (void)s; (void)t; (void)b; (void)m; (void)l; (void)w; return 4; }
int hg_launch_reduce2(void* s, int d, int o, const HgSeg2Table* t, uint64_t b, int m, uint32_t l, int w) { (void)s; (void)d; (void)o; (void)t; (void)b; (void)m; (void)l; (void)w; return 4; }
int hg_launch_bytewise(void* s, int r, int d, int o, const HgSeg2Table* t, uint64_t b, int st, uint32_t l, int w) { (void)s; (void)r; (void)d; (void)o; (void)t; (void)b; (void)st; (void)l; (void)w; return 4; }
int hg_launch_fold(void* s, int d, int o, int a, const HgFoldTable* t, uint64_t b, uint32_t l) { (void)s; (void)d; (void)o; (void)a; (void)t; (void)b; (void)l; return 4; }
int hg_rt_device_count(void) { return 0; }
int hg_rt_scratch(void* s, void** p) { (void)s; *p = NULL; return 4; }
int hg_rt_stream_create(void** s) { *s = NULL; return 4; }
int hg_rt_stream_destroy(void* s) { (void)s; return 0; }
int hg_rt_stream_sync(void* s) { (void)s; return 0; }
int hg_rt_event_create(void** e) { *e = NULL; return 4; }
int hg_rt_event_destroy(void* e) { (void)e; return 0; }
int hg_rt_event_record(void* e, void* s) { (void)e; (void)s; return 0; }
int hg_rt_stream_wait_event(void* s, void* e) { (void)e; (void)s; return 0; }
int hg_rt_malloc(void** p, size_t n) { (void)n; *p = NULL; return 4; }
int hg_rt_free(void* p) { (void)p; return 0; }
int hg_rt_num_cus(void) { return 256; }
int hg_rt_stream_is_capturing(void* s) { (void)s; return 0; }
int hg_rt_capture_begin(void* s) { (void)s; return 4; }
int hg_rt_capture_end(void* s, void** g) { (void)s; *g = NULL; return 4; }
int hg_rt_graph_launch(void* g, void* s) { (void)g; (void)s; return 4; }
int hg_rt_graph_destroy(void* g) { (void)g; return 0; }
#endif
