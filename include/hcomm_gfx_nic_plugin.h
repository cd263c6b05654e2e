/*
 * hcomm_gfx_nic_plugin.h - libhcomm_gfx.so as a NIC plugin of the reference's own libhcomm.
 *
 * The reference loads every .so named in HCOMM_NIC_PLUGIN_SO (src/base_comm/primitives/api_c_adpt/nic_plugin/
 * nic_plugin_manager.cc:34,113-151), looks up the three symbols below and, for channels of a protocol the plugin
 * lists, sends the inter-rank data-plane calls through the plugin's table instead of its own transports
 * (cpu_primitives_c_adpt.cc:320-340: HcommBatchTransferOnThread, HcommWriteReduceOnThread, ...).  This header restates
 * in plain C, with identical layouts, what src/base_comm/primitives/api_c_adpt/nic_plugin/hcomm_nic_plugin.h:23-104
 * declares (the reference's headers compile as C++ only).  Sizes probed from the reference's headers: CommAbiHeader
 * 16, HcommNicEndpointOps 80, HcommNicChannelOps 208, HcommNicPluginInfo 112, CommMem 24, EndpointDesc 160,
 * HcommChannelDesc 360 with notifyNum at offset 176.
 *
 * What the table does here: the entries that move or reduce data on a thread forward to the same kernels as
 * HcommLocalCopyOnThread / HcommLocalReduceOnThread (a "peer" is memory of this GPU); the channel's own notifies are
 * HIP events of the channel; everything that needs an endpoint, a socket or a remote notify returns
 * HCCL_E_NOT_SUPPORT.  The ThreadHandle a caller passes must be one of THIS library's (HcommThreadAlloc /
 * HcommThreadAllocWithStream of libhcomm_gfx.so): the table is for a host whose thread layer is this library too.
 */
#ifndef HCOMM_GFX_NIC_PLUGIN_H
#define HCOMM_GFX_NIC_PLUGIN_H

#include "hcomm_gfx.h"

#ifdef __cplusplus
extern "C" {
#endif

/* hcomm_nic_plugin.h:23-29 */
#define HCOMM_NIC_PLUGIN_MAX_PROTOCOLS 4U
#define HCOMM_NIC_PLUGIN_INFO_MAGIC_WORD 0x0fcf0f1fU
#define HCOMM_NIC_PLUGIN_INFO_VERSION 1U
#define HCOMM_NIC_ENDPOINT_OPS_MAGIC_WORD 0x0fcf0f2fU
#define HCOMM_NIC_ENDPOINT_OPS_VERSION 1U
#define HCOMM_NIC_CHANNEL_OPS_MAGIC_WORD 0x0fcf0f3fU
#define HCOMM_NIC_CHANNEL_OPS_VERSION 1U

/* include/hcomm_res_defs.h:65-70 */
typedef struct {
    uint32_t version;
    uint32_t magicWord;
    uint32_t size;
    uint32_t reserved;
} CommAbiHeader;

/* include/hcomm_res_defs.h:119-133 (values only: the plugin lists protocols, it interprets none).  Identifiers from
 * 1000 on are free for plugins (COMM_PROTOCOL_CUSTOM_BASE, nic_plugin_manager.h:30). */
typedef int32_t CommProtocol;
#define HCOMM_GFX_PROTOCOL_LOCAL_HBM 1000 /* a peer whose buffers this GPU addresses directly */

/* include/hcomm_res_defs.h:206-219 */
typedef struct {
    int32_t type; /* CommMemType: 0 device, 1 host */
    void* addr;
    uint64_t size;
} CommMem;

/* include/hcomm_res_defs.h:191-200 (160 bytes) and include/hcomm_channel.h:33-73 (360 bytes): never interpreted here
 * beyond the channel's notifyNum, so only the leading fields are spelled out */
typedef struct {
    uint8_t raws[160];
} EndpointDesc;
typedef struct {
    CommAbiHeader header;
    EndpointDesc remoteEndpoint;
    uint32_t notifyNum; /* notifies the channel owns */
    /* ... the reference's further fields (memory handles, socket, role, port, protocol attributes, qos, name) */
} HcommChannelDescHead;

/* hcomm_nic_plugin.h:31-42 */
typedef struct {
    CommAbiHeader header;
    int32_t (*init)(void* ctx);
    int32_t (*destroy)(void* ctx);
    int32_t (*registerMemory)(void* ctx, const CommMem* mem, const char* tag, void** handle);
    int32_t (*unregisterMemory)(void* ctx, void* handle);
    int32_t (*memoryExport)(void* ctx, void* handle, void** desc, uint32_t* descLen);
    int32_t (*memoryImport)(void* ctx, const void* desc, uint32_t descLen, CommMem* outMem);
    int32_t (*memoryUnimport)(void* ctx, const void* desc, uint32_t descLen);
    int32_t (*getListenPort)(void* ctx, uint32_t* port);
} HcommNicEndpointOps;

/* hcomm_nic_plugin.h:44-85 */
typedef struct {
    CommAbiHeader header;
    int32_t (*init)(void* ctx);
    int32_t (*destroy)(void* ctx);
    int32_t (*getStatus)(void* ctx, int32_t* status);
    int32_t (*writeNbi)(void* ctx, void* dst, const void* src, uint64_t len);
    int32_t (*writeNbiOnThread)(void* ctx, ThreadHandle thread, void* dst, const void* src, uint64_t len);
    int32_t (*writeOnThread)(void* ctx, ThreadHandle thread, void* dst, const void* src, uint64_t len);
    int32_t (*writeWithNotifyNbi)(void* ctx, void* dst, const void* src, uint64_t len, uint32_t remoteNotifyIdx);
    int32_t (*writeWithNotifyNbiOnThread)(
        void* ctx, ThreadHandle thread, void* dst, const void* src, uint64_t len, uint32_t remoteNotifyIdx);
    int32_t (*writeWithNotifyOnThread)(
        void* ctx, ThreadHandle thread, void* dst, const void* src, uint64_t len, uint32_t remoteNotifyIdx);
    int32_t (*writeReduceOnThread)(
        void* ctx, ThreadHandle thread, void* dst, const void* src, uint64_t count, HcommDataType dataType,
        HcommReduceOp reduceOp);
    int32_t (*writeReduceWithNotifyOnThread)(
        void* ctx, ThreadHandle thread, void* dst, const void* src, uint64_t count, HcommDataType dataType,
        HcommReduceOp reduceOp, uint32_t remoteNotifyIdx);
    int32_t (*readNbi)(void* ctx, void* dst, const void* src, uint64_t len);
    int32_t (*readNbiOnThread)(void* ctx, ThreadHandle thread, void* dst, const void* src, uint64_t len);
    int32_t (*readOnThread)(void* ctx, ThreadHandle thread, void* dst, const void* src, uint64_t len);
    int32_t (*readReduceOnThread)(
        void* ctx, ThreadHandle thread, void* dst, const void* src, uint64_t count, HcommDataType dataType,
        HcommReduceOp reduceOp);
    int32_t (*notifyRecord)(void* ctx, uint32_t remoteNotifyIdx);
    int32_t (*notifyRecordOnThread)(void* ctx, ThreadHandle thread, uint32_t remoteNotifyIdx);
    int32_t (*notifyWait)(void* ctx, uint32_t localNotifyIdx, uint32_t timeOut);
    int32_t (*notifyWaitOnThread)(void* ctx, ThreadHandle thread, uint32_t localNotifyIdx, uint32_t timeOut);
    int32_t (*notifyWaitOnThreadWithDefaultTimeout)(void* ctx, ThreadHandle thread, uint32_t localNotifyIdx);
    int32_t (*batchTransferOnThread)(
        void* ctx, ThreadHandle thread, const HcommBatchTransferDesc* transferDescs, uint32_t transferDescNum);
    int32_t (*fence)(void* ctx);
    int32_t (*fenceOnThread)(void* ctx, ThreadHandle thread);
    int32_t (*drainOnThread)(void* ctx, ThreadHandle thread);
} HcommNicChannelOps;

/* hcomm_nic_plugin.h:87-93 */
typedef struct {
    CommAbiHeader header;
    const char* name;
    uint32_t protocolCount;
    CommProtocol protocols[HCOMM_NIC_PLUGIN_MAX_PROTOCOLS];
    uint64_t reserved[8];
} HcommNicPluginInfo;

/*
 * The three symbols the reference's plugin manager resolves (hcomm_nic_plugin.h:101-104, looked up at
 * nic_plugin_manager.cc:124-129).
 *
 * HcommNicPluginGetInfo: name "hcomm_gfx", one protocol, HCOMM_GFX_PROTOCOL_LOCAL_HBM, or the (at most four)
 * identifiers listed in HCOMM_GFX_PLUGIN_PROTOCOLS, separated by commas, when a host wants the table behind one of
 * its own protocols.
 *
 * HcommNicPluginCreateEndpoint: no endpoint exists on this path (no address, no socket, no memory registration:
 * every buffer is memory of the one GPU); the context only carries init / destroy, and every other entry of its
 * table returns HCCL_E_NOT_SUPPORT.
 *
 * HcommNicPluginCreateChannel: a channel context that owns min(channelDesc->notifyNum, 64) notifies.  Table entries:
 *   write / writeNbi / read / readNbi ...OnThread    dst[0..len) = src[0..len) on the thread, as HcommLocalCopyOnThread
 *   writeReduceOnThread / readReduceOnThread          dst = dst (op) src, as HcommLocalReduceOnThread (same type x op
 *                                                     support, same check order)
 *   batchTransferOnThread                             as HcommBatchTransferOnThread: one launch per run of independent
 *                                                     descriptors of equal kind
 *   notifyRecordOnThread / notifyWaitOnThread /       the channel's notify `idx`: record marks the point the thread
 *   notifyWaitOnThreadWithDefaultTimeout              has reached, wait makes the thread wait for the latest record
 *                                                     issued before it (HCCL_E_TIMEOUT when none is pending)
 *   fence / fenceOnThread / drainOnThread             ordering points of an in-order stream: handles are checked
 *   getStatus                                         0 (HCOMM_CHANNEL_STATUS_READY, channel_process.h:33)
 *   the entries without a thread (writeNbi, readNbi, notifyRecord, notifyWait) and the ...WithNotify... entries, which
 *   signal a REMOTE process                           HCCL_E_NOT_SUPPORT
 */
const HcommNicPluginInfo* HcommNicPluginGetInfo(void);
int32_t HcommNicPluginCreateEndpoint(const EndpointDesc* endpointDesc, void** outCtx, HcommNicEndpointOps** outOps);
int32_t HcommNicPluginCreateChannel(
    void* epCtx, const HcommChannelDescHead* channelDesc, void** outCtx, HcommNicChannelOps** outOps);

#ifdef __cplusplus
}
#endif
#endif
