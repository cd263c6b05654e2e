/*
 * hg_nic_plugin.c - the NIC-plugin face of libhcomm_gfx.so: the three symbols the reference's plugin manager resolves
 * (src/base_comm/primitives/api_c_adpt/nic_plugin/nic_plugin_manager.cc:113-151) and the two tables they hand out
 * (hcomm_nic_plugin.h:31-85).  The data-plane entries forward to the primitives of hg_api.c - same kernels, same
 * checks - so that a host which routes a channel's HcommWriteReduceOnThread / HcommBatchTransferOnThread through a
 * plugin table (cpu_primitives_c_adpt.cc:320-340) lands on the same code as a caller of the primitives themselves.
 */
#include <stdlib.h>
#include <string.h>

#include "hcomm_gfx_nic_plugin.h"
#include "hg_host.h"

_Static_assert(sizeof(CommAbiHeader) == 16, "CommAbiHeader: 16 bytes in the reference");
_Static_assert(sizeof(HcommNicEndpointOps) == 80, "HcommNicEndpointOps: 80 bytes in the reference");
_Static_assert(sizeof(HcommNicChannelOps) == 208, "HcommNicChannelOps: 208 bytes in the reference");
_Static_assert(sizeof(HcommNicPluginInfo) == 112, "HcommNicPluginInfo: 112 bytes in the reference");
_Static_assert(sizeof(CommMem) == 24, "CommMem: 24 bytes in the reference");
_Static_assert(sizeof(EndpointDesc) == 160, "EndpointDesc: 160 bytes in the reference");
_Static_assert(offsetof(HcommChannelDescHead, notifyNum) == 176, "HcommChannelDesc.notifyNum sits at offset 176");
_Static_assert(offsetof(HcommNicChannelOps, writeOnThread) == 56 && offsetof(HcommNicChannelOps, writeReduceOnThread) == 88 &&
                   offsetof(HcommNicChannelOps, readReduceOnThread) == 128 &&
                   offsetof(HcommNicChannelOps, batchTransferOnThread) == 176 && offsetof(HcommNicChannelOps, drainOnThread) == 200,
               "entry offsets as probed from the reference's header");

#define EP_MAGIC 0x48474550u /* "HGEP" */
#define CH_MAGIC 0x48474348u /* "HGCH" */
#define CH_NOTIFY_MAX 64u

typedef struct {
    uint32_t magic;
} Endpoint;

typedef struct {
    uint32_t magic;
    uint32_t notify_num;
    void* notifies[CH_NOTIFY_MAX];        /* hipEvent_t, created on first use */
    uint64_t notify_pending[CH_NOTIFY_MAX]; /* records issued that no wait has consumed yet */
} Channel;

static Channel* channel_of(void* ctx)
{
    Channel* c = (Channel*)ctx;
    return (c && c->magic == CH_MAGIC) ? c : NULL;
}

/* ---- plugin info ------------------------------------------------------------------------------------------- */

static HcommNicPluginInfo g_info = {
    {HCOMM_NIC_PLUGIN_INFO_VERSION, HCOMM_NIC_PLUGIN_INFO_MAGIC_WORD, sizeof(HcommNicPluginInfo), 0},
    "hcomm_gfx",
    1,
    {HCOMM_GFX_PROTOCOL_LOCAL_HBM, 0, 0, 0},
    {0},
};
static int g_info_ready = 0;

const HcommNicPluginInfo* HcommNicPluginGetInfo(void)
{
    if (!__atomic_load_n(&g_info_ready, __ATOMIC_ACQUIRE)) {
        /* every caller computes the same list; the flag is set after the list is complete */
        const char* e = getenv("HCOMM_GFX_PLUGIN_PROTOCOLS");
        if (e && *e) {
            uint32_t n = 0;
            CommProtocol list[HCOMM_NIC_PLUGIN_MAX_PROTOCOLS];
            while (*e && n < HCOMM_NIC_PLUGIN_MAX_PROTOCOLS) {
                char* end = NULL;
                const long v = strtol(e, &end, 10);
                if (end == e) break;
                list[n++] = (CommProtocol)v;
                e = (*end == ',') ? end + 1 : end;
            }
            if (n) {
                for (uint32_t i = 0; i < n; ++i) g_info.protocols[i] = list[i];
                g_info.protocolCount = n;
            }
        }
        __atomic_store_n(&g_info_ready, 1, __ATOMIC_RELEASE);
    }
    return &g_info;
}

/* ---- endpoint ---------------------------------------------------------------------------------------------- */

static int32_t ep_init(void* ctx) { return (ctx && ((Endpoint*)ctx)->magic == EP_MAGIC) ? HCCL_SUCCESS : HCCL_E_PTR; }

static int32_t ep_destroy(void* ctx)
{
    Endpoint* e = (Endpoint*)ctx;
    if (!e || e->magic != EP_MAGIC) return HCCL_E_PTR;
    e->magic = 0;
    free(e);
    return HCCL_SUCCESS;
}

static int32_t ep_register(void* ctx, const CommMem* mem, const char* tag, void** handle)
{
    (void)ctx; (void)mem; (void)tag; (void)handle;
    return HCCL_E_NOT_SUPPORT;
}
static int32_t ep_unregister(void* ctx, void* handle) { (void)ctx; (void)handle; return HCCL_E_NOT_SUPPORT; }
static int32_t ep_export(void* ctx, void* handle, void** desc, uint32_t* len) { (void)ctx; (void)handle; (void)desc; (void)len; return HCCL_E_NOT_SUPPORT; }
static int32_t ep_import(void* ctx, const void* desc, uint32_t len, CommMem* out) { (void)ctx; (void)desc; (void)len; (void)out; return HCCL_E_NOT_SUPPORT; }
static int32_t ep_unimport(void* ctx, const void* desc, uint32_t len) { (void)ctx; (void)desc; (void)len; return HCCL_E_NOT_SUPPORT; }
static int32_t ep_port(void* ctx, uint32_t* port) { (void)ctx; (void)port; return HCCL_E_NOT_SUPPORT; }

static HcommNicEndpointOps g_ep_ops = {
    {HCOMM_NIC_ENDPOINT_OPS_VERSION, HCOMM_NIC_ENDPOINT_OPS_MAGIC_WORD, sizeof(HcommNicEndpointOps), 0},
    ep_init, ep_destroy, ep_register, ep_unregister, ep_export, ep_import, ep_unimport, ep_port,
};

int32_t HcommNicPluginCreateEndpoint(const EndpointDesc* endpointDesc, void** outCtx, HcommNicEndpointOps** outOps)
{
    if (!endpointDesc || !outCtx || !outOps) return HCCL_E_PTR;
    Endpoint* e = (Endpoint*)calloc(1, sizeof(*e));
    if (!e) return HCCL_E_MEMORY;
    e->magic = EP_MAGIC;
    *outCtx = e;
    *outOps = &g_ep_ops;
    return HCCL_SUCCESS;
}

/* ---- channel: life cycle -------------------------------------------------------------------------------------- */

static int32_t ch_init(void* ctx) { return channel_of(ctx) ? HCCL_SUCCESS : HCCL_E_PTR; }

static int32_t ch_destroy(void* ctx)
{
    Channel* c = channel_of(ctx);
    if (!c) return HCCL_E_PTR;
    for (uint32_t i = 0; i < c->notify_num; ++i)
        if (c->notifies[i]) hg_rt_event_destroy(c->notifies[i]);
    c->magic = 0;
    free(c);
    return HCCL_SUCCESS;
}

static int32_t ch_status(void* ctx, int32_t* status)
{
    if (!channel_of(ctx)) return HCCL_E_PTR;
    if (!status) return HCCL_E_PTR;
    *status = 0; /* HCOMM_CHANNEL_STATUS_READY, src/base_comm/resources/endpoint_pairs/channels/channel_process.h:33 */
    return HCCL_SUCCESS;
}

/* ---- channel: data plane ------------------------------------------------------------------------------------- */

/* the channel handle the primitives take is any non-zero value: the context's address */
#define CH_HANDLE(ctx) ((ChannelHandle)(uintptr_t)(ctx))

static int32_t ch_write(void* ctx, ThreadHandle thread, void* dst, const void* src, uint64_t len)
{
    if (!channel_of(ctx)) return HCCL_E_PTR;
    return HcommWriteOnThread(thread, CH_HANDLE(ctx), dst, src, len);
}
static int32_t ch_write_nbi(void* ctx, ThreadHandle thread, void* dst, const void* src, uint64_t len)
{
    if (!channel_of(ctx)) return HCCL_E_PTR;
    return HcommWriteNbiOnThread(thread, CH_HANDLE(ctx), dst, src, len);
}
static int32_t ch_read(void* ctx, ThreadHandle thread, void* dst, const void* src, uint64_t len)
{
    if (!channel_of(ctx)) return HCCL_E_PTR;
    return HcommReadOnThread(thread, CH_HANDLE(ctx), dst, src, len);
}
static int32_t ch_read_nbi(void* ctx, ThreadHandle thread, void* dst, const void* src, uint64_t len)
{
    if (!channel_of(ctx)) return HCCL_E_PTR;
    return HcommReadNbiOnThread(thread, CH_HANDLE(ctx), dst, src, len);
}
static int32_t ch_write_reduce(void* ctx, ThreadHandle thread, void* dst, const void* src, uint64_t count, HcommDataType dt, HcommReduceOp op)
{
    if (!channel_of(ctx)) return HCCL_E_PTR;
    return HcommWriteReduceOnThread(thread, CH_HANDLE(ctx), dst, src, count, dt, op);
}
static int32_t ch_read_reduce(void* ctx, ThreadHandle thread, void* dst, const void* src, uint64_t count, HcommDataType dt, HcommReduceOp op)
{
    if (!channel_of(ctx)) return HCCL_E_PTR;
    return HcommReadReduceOnThread(thread, CH_HANDLE(ctx), dst, src, count, dt, op);
}
static int32_t ch_batch(void* ctx, ThreadHandle thread, const HcommBatchTransferDesc* descs, uint32_t n)
{
    if (!channel_of(ctx)) return HCCL_E_PTR;
    return HcommBatchTransferOnThread(thread, CH_HANDLE(ctx), descs, n);
}

/* entries that have no thread to run on, or that signal a remote process */
static int32_t ch_no_thread_copy(void* ctx, void* dst, const void* src, uint64_t len) { (void)ctx; (void)dst; (void)src; (void)len; return HCCL_E_NOT_SUPPORT; }
static int32_t ch_wn_nbi(void* ctx, void* dst, const void* src, uint64_t len, uint32_t idx) { (void)ctx; (void)dst; (void)src; (void)len; (void)idx; return HCCL_E_NOT_SUPPORT; }
static int32_t ch_wn_thread(void* ctx, ThreadHandle t, void* dst, const void* src, uint64_t len, uint32_t idx) { (void)ctx; (void)t; (void)dst; (void)src; (void)len; (void)idx; return HCCL_E_NOT_SUPPORT; }
static int32_t ch_wrn_thread(void* ctx, ThreadHandle t, void* dst, const void* src, uint64_t count, HcommDataType dt, HcommReduceOp op, uint32_t idx) { (void)ctx; (void)t; (void)dst; (void)src; (void)count; (void)dt; (void)op; (void)idx; return HCCL_E_NOT_SUPPORT; }
static int32_t ch_notify_record_host(void* ctx, uint32_t idx) { (void)ctx; (void)idx; return HCCL_E_NOT_SUPPORT; }
static int32_t ch_notify_wait_host(void* ctx, uint32_t idx, uint32_t timeOut) { (void)ctx; (void)idx; (void)timeOut; return HCCL_E_NOT_SUPPORT; }

/* ---- channel: its own notifies ---------------------------------------------------------------------------------
 * A notify of the channel is an event the channel owns: record marks the point `thread` has reached, wait makes
 * `thread` wait for the latest record issued before the wait; every record is consumed by one wait.  Both ends of a
 * simulated link use the one channel object. */

static int32_t ch_notify_record(void* ctx, ThreadHandle thread, uint32_t idx)
{
    Channel* c = channel_of(ctx);
    if (!c) return HCCL_E_PTR;
    HgThread* t = hg_thread_from_handle(thread);
    if (!t) return HCCL_E_PTR;
    if (idx >= c->notify_num) return HCCL_E_PARA;
    if (hg_caller_is_batching()) return HCCL_E_NOT_SUPPORT;
    if (!t->recorder) {
        if (!c->notifies[idx]) {
            const int rc = hg_rt_event_create(&c->notifies[idx]);
            if (rc != HCCL_SUCCESS) return rc;
        }
        int rc = hg_thread_settle(t);
        if (rc == HCCL_SUCCESS) rc = hg_rt_event_record(c->notifies[idx], t->stream);
        if (rc != HCCL_SUCCESS) return rc;
    }
    __atomic_add_fetch(&c->notify_pending[idx], 1, __ATOMIC_RELEASE);
    return HCCL_SUCCESS;
}

static int32_t ch_notify_wait(void* ctx, ThreadHandle thread, uint32_t idx, uint32_t timeOut)
{
    (void)timeOut;
    Channel* c = channel_of(ctx);
    if (!c) return HCCL_E_PTR;
    HgThread* t = hg_thread_from_handle(thread);
    if (!t) return HCCL_E_PTR;
    if (idx >= c->notify_num) return HCCL_E_PARA;
    if (hg_caller_is_batching()) return HCCL_E_NOT_SUPPORT;
    uint64_t pending = __atomic_load_n(&c->notify_pending[idx], __ATOMIC_ACQUIRE);
    do {
        if (pending == 0) return HCCL_E_TIMEOUT; /* no record issued: the wait the reference would time out on */
    } while (!__atomic_compare_exchange_n(&c->notify_pending[idx], &pending, pending - 1, 0, __ATOMIC_ACQ_REL, __ATOMIC_ACQUIRE));
    if (t->recorder) return HCCL_SUCCESS;
    return hg_rt_stream_wait_event(t->stream, c->notifies[idx]);
}

static int32_t ch_notify_wait_default(void* ctx, ThreadHandle thread, uint32_t idx) { return ch_notify_wait(ctx, thread, idx, 0); }

/* ---- channel: ordering points ---------------------------------------------------------------------------------- */

static int32_t ch_fence(void* ctx) { return channel_of(ctx) ? HCCL_SUCCESS : HCCL_E_PTR; }
static int32_t ch_fence_thread(void* ctx, ThreadHandle thread)
{
    if (!channel_of(ctx)) return HCCL_E_PTR;
    return HcommChannelFenceOnThread(thread, CH_HANDLE(ctx));
}
static int32_t ch_drain_thread(void* ctx, ThreadHandle thread)
{
    if (!channel_of(ctx)) return HCCL_E_PTR;
    return HcommChannelDrainOnThread(thread, CH_HANDLE(ctx));
}

static HcommNicChannelOps g_ch_ops = {
    {HCOMM_NIC_CHANNEL_OPS_VERSION, HCOMM_NIC_CHANNEL_OPS_MAGIC_WORD, sizeof(HcommNicChannelOps), 0},
    ch_init,
    ch_destroy,
    ch_status,
    ch_no_thread_copy,  /* writeNbi */
    ch_write_nbi,       /* writeNbiOnThread */
    ch_write,           /* writeOnThread */
    ch_wn_nbi,          /* writeWithNotifyNbi */
    ch_wn_thread,       /* writeWithNotifyNbiOnThread */
    ch_wn_thread,       /* writeWithNotifyOnThread */
    ch_write_reduce,    /* writeReduceOnThread */
    ch_wrn_thread,      /* writeReduceWithNotifyOnThread */
    ch_no_thread_copy,  /* readNbi */
    ch_read_nbi,        /* readNbiOnThread */
    ch_read,            /* readOnThread */
    ch_read_reduce,     /* readReduceOnThread */
    ch_notify_record_host,
    ch_notify_record,
    ch_notify_wait_host,
    ch_notify_wait,
    ch_notify_wait_default,
    ch_batch,
    ch_fence,
    ch_fence_thread,
    ch_drain_thread,
};

int32_t HcommNicPluginCreateChannel(void* epCtx, const HcommChannelDescHead* channelDesc, void** outCtx, HcommNicChannelOps** outOps)
{
    if (!epCtx || ((Endpoint*)epCtx)->magic != EP_MAGIC) return HCCL_E_PTR;
    if (!channelDesc || !outCtx || !outOps) return HCCL_E_PTR;
    Channel* c = (Channel*)calloc(1, sizeof(*c));
    if (!c) return HCCL_E_MEMORY;
    c->magic = CH_MAGIC;
    c->notify_num = channelDesc->notifyNum < CH_NOTIFY_MAX ? channelDesc->notifyNum : CH_NOTIFY_MAX;
    *outCtx = c;
    *outOps = &g_ch_ops;
    return HCCL_SUCCESS;
}
