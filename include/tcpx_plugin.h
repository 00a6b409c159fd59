/*
 * tcpx_plugin.h -- C entry points of the plugin library (libnccl-net.so) of the MI355X receive-side unpack path.
 *
 * Three groups:
 *   1. the ncclNet_v7 functions, under the names the reference gives them (src/net_tcpx.h:22-62), which the
 *      exported `ncclNetPlugin_v7` table points to (src/nccl_plugin.cc:22-42);
 *   2. the synthetic devmem socket: this build has no NIC and no sockets, so what the peer's control socket
 *      and the kernel's devmem-TCP receive path would deliver is pushed in through these calls by a test or
 *      benchmark driver;
 *   3. the device-operations table through which the plugin reaches the GPU.  By default it is bound to
 *      libtcpxu_hip.so (include/tcpx_unpack_hip.h) and initialisation fails if that cannot be loaded or no GPU
 *      is present.  A test may install another table BEFORE tcpxInit to exercise the host logic without a GPU;
 *      the plugin never picks a substitute by itself.
 */
#ifndef TCPX_PLUGIN_H_
#define TCPX_PLUGIN_H_

#include <stddef.h>
#include <stdint.h>

#include "nccl_net_v7.h"
#include "tcpx_synth.h"      /* tcpxSynthFrag */
#include "tcpx_unpack_hip.h" /* tcpxuEngine */

#ifdef __cplusplus
extern "C" {
#endif

/* ---- 1. ncclNet_v7 --------------------------------------------------------------------------------------- */

extern volatile ncclNet_v7_t ncclNetPlugin_v7; /* src/nccl_plugin.cc:22-42 */

ncclResult_t tcpxInit(ncclDebugLogger_t logFunction);                  /* src/net_tcpx.cc:454-696 (flags, devices) */
ncclResult_t tcpxDevices(int* ndev);                                   /* src/net_tcpx.cc:698-703 */
ncclResult_t tcpxGetProperties(int dev, ncclNetProperties_v7_t* props); /* src/net_tcpx.cc:725-744 */
ncclResult_t tcpxListen(int dev, void* handle, void** listenComm);     /* src/net_tcpx.cc:746-750 */
ncclResult_t tcpxConnect_v5(int dev, void* handle, void** sendComm, ncclNetDeviceHandle_v7_t** sendDevHandle);
ncclResult_t tcpxAccept_v5(void* listenComm, void** recvComm, ncclNetDeviceHandle_v7_t** recvDevHandle); /* :761-769 */
ncclResult_t tcpxRegMr(void* comm, void* data, int size, int type, void** mhandle); /* src/net_tcpx.cc:771-823 */
ncclResult_t tcpxDeregMr(void* comm, void* mhandle);                               /* src/net_tcpx.cc:825-853 */
ncclResult_t tcpxIsend_v5(void* sendComm, void* data, int size, int tag, void* mhandle, void** request); /* :898-919 */
ncclResult_t tcpxIrecv_v5(void* recvComm, int n, void** data, int* sizes, int* tags, void** mhandles,
                          void** request);                                         /* src/net_tcpx.cc:921-944 */
ncclResult_t tcpxIflush_v5(void* recvComm, int n, void** data, int* sizes, void** mhandles, void** request); /* :946-954 */
ncclResult_t tcpxTest(void* request, int* done, int* size);                        /* src/net_tcpx.cc:1311-1374 */
ncclResult_t tcpxClose(void* comm);                                                /* src/net_tcpx.cc:1376-1436 */
ncclResult_t tcpxCloseListen(void* listenComm);                                    /* src/net_tcpx.cc:1438-1450 */
ncclResult_t tcpxGetDeviceMr(void* comm, void* mhandle, void** dptr_mhandle);      /* src/net_tcpx.cc:1473-1475 */
ncclResult_t tcpxIrecvConsumed(void* recvComm, int n, void* request);              /* src/net_tcpx.cc:1477-1543 */

/* Undoes tcpxInit: stops the engines, frees arenas and cached queue memory.  Comms must be closed first.
 * The reference has no counterpart (NCCL never unloads it); a persistent kernel needs an orderly stop. */
ncclResult_t tcpxFinalize(void);

/* ---- 2. synthetic devmem socket -------------------------------------------------------------------------- */

/* Control-message types of the reference's control socket (enum CtrlType, src/common.h:138-142). */
#define TCPX_CTRL_NORMAL 0
#define TCPX_CTRL_INLINE 1

/* Creates the bounce-page arena of GPU `dev` (`bytes` a multiple of 4096, at most 4 GiB) and returns its device
 * address; stands in for the receive-datapath-manager's NIC page pool (src/gpu/rx_pool.cu:62-121).  Must be
 * called after tcpxInit and before the first tcpxAccept_v5 on that GPU; one arena per GPU. */
ncclResult_t tcpxSynthArenaCreate(int dev, size_t bytes, void** base);

/* What the peer's control socket would carry for the oldest active receive request: one 16-byte packed
 * `struct tcpxCtrl {u16 type, u16 index, u32 size, u32 offset, u32 total}` (src/common.h:127-133) per chunk,
 * where `index` is the data flow (socket) the chunk travels on, `size` its bytes and `total` the message size. */
ncclResult_t tcpxSynthCtrlSend(void* recvComm, uint16_t type, uint16_t flow, uint32_t size, uint32_t offset,
                               uint32_t total);

/* Fragments that the NIC has placed in bounce pages for data flow `flow`, in arrival order, as the kernel would
 * report them one per SCM_DEVMEM_OFFSET control message (src/sock/tcpx.h:130-134,157-181).  The payload itself
 * must already be in the arena. */
ncclResult_t tcpxSynthDeliver(void* recvComm, uint32_t flow, const tcpxSynthFrag* frags, uint32_t n_frags);

/* Limits how many fragments one synthetic recvmsg returns (default: as many as fit, at most 2048), to exercise
 * partial arrival; 0 restores the default. */
ncclResult_t tcpxSynthSetRecvmsgLimit(void* recvComm, uint32_t max_frags_per_recvmsg);

/* Page references handed to the plugin by the synthetic kernel and not yet given back through
 * SO_DEVMEM_DONTNEED (src/sock/tcpx.h:299-326).  Zero when every received request has been consumed. */
ncclResult_t tcpxSynthOutstandingPages(void* recvComm, uint64_t* pages);

/* Inspection for tests: ring positions of the comm's unpack queue (struct tcpxNetDeviceQueue head/tail,
 * src/devcomm/unpack_defs1.h:53-59) and of its request ring (indices of the five states,
 * src/work_queue.h:78-130: [0] free/dequeue cursor ... [4] enqueue cursor). */
ncclResult_t tcpxDebugQueueState(void* recvComm, uint64_t* head, uint64_t* tail, uint32_t request_idx[5]);

/* Descriptors and count currently in slot `slot_idx` of the comm's mapped metadata (host view). */
ncclResult_t tcpxDebugSlot(void* recvComm, uint32_t slot_idx, const union loadMeta** descs, uint64_t* cnt);

/* ---- 3. device operations -------------------------------------------------------------------------------- */

typedef struct tcpxDeviceOps {
  int (*device_count)(int* count);
  int (*arena_create)(int device, size_t bytes, void** base);
  int (*arena_destroy)(int device, void* base);
  int (*mapped_alloc)(int device, size_t bytes, void** host_ptr, void** dev_ptr);
  int (*mapped_free)(int device, void* host_ptr);
  int (*device_alloc)(int device, size_t bytes, void** ptr);
  int (*device_free)(int device, void* ptr);
  int (*copy_to_device)(int device, void* dst_dev, const void* src_host, size_t bytes);
  int (*engine_create)(int device, const tcpxuEngineConfig* config, tcpxuEngine** engine);
  int (*engine_start)(tcpxuEngine* engine);
  int (*engine_stop)(tcpxuEngine* engine, double* elapsed_us);
  int (*engine_destroy)(tcpxuEngine* engine);
  int (*engine_submit)(tcpxuEngine* engine, const void* bounce_base, void* dst_base, const void* descs_dev,
                       uint32_t n_descs, void* done_flag_dev, uint64_t done_value);
  const char* (*last_error)(void);
} tcpxDeviceOps;

/* Installs `ops` in place of the HIP layer (NULL restores the default binding).  For host-logic tests only;
 * refused with ncclInvalidUsage once tcpxInit has run. */
ncclResult_t tcpxSetDeviceOpsForTesting(const tcpxDeviceOps* ops);

/* When 0, conditions on which the reference calls exit(1) (descriptor overflow: src/sock/tcpx.h:183-187,
 * src/net_tcpx.cc:1350-1353) return ncclInternalError instead, so a test can observe them in-process.
 * Default 1 = fail-stop like the reference. */
ncclResult_t tcpxSetFailStopForTesting(int enabled);

#ifdef __cplusplus
}
#endif
#endif /* TCPX_PLUGIN_H_ */
