/*
 * tcpx_plugin.h -- C entry points of the plugin library (libnccl-net.so) of the MI355X receive-side unpack path.
 *
 * Five groups:
 *   1. the ncclNet_v7 functions, under the names the reference gives them (src/net_tcpx.h:22-62), which the
 *      exported `ncclNetPlugin_v7` table points to (src/nccl_plugin.cc:22-42);
 *   2. the synthetic devmem socket: this build has no NIC and no sockets, so what the peer's control socket
 *      and the kernel's devmem-TCP receive path would deliver is pushed in through these calls by a test or
 *      benchmark driver;
 *   3. the device-operations table through which the plugin reaches the GPU.  By default it is bound to
 *      libtcpxu_hip.so (include/tcpx_unpack_hip.h) and initialisation fails if that cannot be loaded or no GPU
 *      is present.  A test may install another table BEFORE tcpxInit to exercise the host logic without a GPU;
 *      the plugin never picks a substitute by itself;
 *   4. observability: slowness watches, counters and state-transition tracepoints (src/timeout.cc, src/stats/);
 *   5. the flow scheduler (src/flow_mapper.h) on its own.
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

/* Who copies is chosen at tcpxInit by NCCL_GPUDIRECTTCPX_AMD_DEVICE_TYPE:
 *   "host" (default)  the plugin's GPU engine unpacks every request; tcpxTest reports done after the copy;
 *                     tcpxGetProperties / tcpxAccept_v5 say NCCL_NET_DEVICE_HOST (version 0, no device handle), so
 *                     that no consumer kernel copies the same bytes a second time;
 *   "unpack"          the reference's division of labour (src/net_tcpx.cc:725-744,1354-1357,1452-1471): they say
 *                     NCCL_NET_DEVICE_UNPACK version 7 and hand out the 24-byte device unpackNetDeviceHandle;
 *                     tcpxTest reports done once the descriptor count is published; the engine is never started
 *                     and whoever holds the handle copies.
 * tcpxListen writes the listener's identity into the 128-byte handle; tcpxConnect_v5 with that handle joins the
 * listener's backlog (ncclSystemError if the listener is closed, ncclInternalError for a handle tcpxListen did not
 * write); tcpxAccept_v5 returns success with *recvComm = NULL until a connection is waiting
 * (src/net_tcpx.cc:761-769).
 *
 * With NCCL_GPUDIRECTTCPX_AMD_HELPER_THREAD=1 a receive comm's sockets are served by a thread of its own (the receive
 * part of persistentSocketThread, src/net_tcpx.cc:252-384).  NCCL_GPUDIRECTTCPX_RX_BINDINGS, in the reference's syntax
 * "name:lo-hi,lo-hi;name:lo-hi" with the device names that tcpxGetProperties reports, names the CPUs that thread may
 * run on (parseCoreRanges, src/common.cc:65-130; sched_setaffinity over all of them, src/net_tcpx.cc:300-307):
 * the two threads hand every task to each other, so how far apart their CPUs are is what that mode costs. */

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

/* Plays NCCL's receive proxy, the peer and the NIC for `n_requests` requests without an interpreter in the loop:
 * irecv at dst_base + request.dst_off, one control message per chunk (a run of consecutive fragments on one
 * flow) and the chunk's fragments, test() until done, irecvConsumed; up to `window` (1..16) requests are kept
 * posted.  `frags` is the whole workload's fragment array (requests index into it), the payload must already be
 * in the arena and requests whose pages are reused must not be in one call.  Writes the wall time to *seconds
 * and, if latency_s is not NULL, each request's fed-to-done time to latency_s[i].  ncclInternalError if a
 * request does not complete within timeout_ms. */
ncclResult_t tcpxSynthRunRequests(void* recvComm, const tcpxSynthFrag* frags, const tcpxSynthRequest* requests,
                                  uint32_t n_requests, void* dst_base, uint64_t dst_bytes, uint32_t window,
                                  uint32_t timeout_ms, double* seconds, double* latency_s);

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
  /* Optional (may be NULL, and the allocation may fail): device memory that the host can write, for a second
   * copy of the descriptors of small requests (tcpxuVisibleAlloc / Free / Flush, include/tcpx_unpack_hip.h). */
  int (*visible_alloc)(int device, size_t bytes, void** host_ptr, void** dev_ptr);
  int (*visible_free)(int device, void* host_ptr);
  void (*visible_flush)(void);
  /* Optional (may be NULL): engine_submit with the request's size as a hint (tcpxuEngineSubmitSized). */
  int (*engine_submit_sized)(tcpxuEngine* engine, const void* bounce_base, void* dst_base, const void* descs_dev,
                             uint32_t n_descs, uint64_t payload_bytes, void* done_flag_dev, uint64_t done_value);
} tcpxDeviceOps;

/* Installs `ops` in place of the HIP layer (NULL restores the default binding).  For host-logic tests only;
 * refused with ncclInvalidUsage once tcpxInit has run. */
ncclResult_t tcpxSetDeviceOpsForTesting(const tcpxDeviceOps* ops);

/* When 0, conditions on which the reference calls exit(1) (descriptor overflow: src/sock/tcpx.h:183-187,
 * src/net_tcpx.cc:1350-1353) return ncclInternalError instead, so a test can observe them in-process.
 * Default 1 = fail-stop like the reference. */
ncclResult_t tcpxSetFailStopForTesting(int enabled);

/* ---- 4. observability ------------------------------------------------------------------------------------ */
/*
 * Flags read by tcpxInit (names and ranges as in the reference, src/net_tcpx.cc:105-116,519-550, src/flags.cc:119-150):
 *   NCCL_GPUDIRECTTCPX_TIMEOUT_THRESHOLD_NS   a watched wait is reported once it has lasted this long (10 s; >= 100 us)
 *   NCCL_GPUDIRECTTCPX_TIMEOUT_FREQUENCY_NS   ... and again at this interval (30 s; >= 100 us)
 *   NCCL_GPUDIRECTTCPX_SLOWNESS_SWITCH        which waits are watched: SENDRECV (recvmsg finds nothing), RX_CTRL (no
 *                                             control message for the active request), UNPACK (the GPU holds a slot;
 *                                             this build's own), TX_COMP (send side: accepted, never armed), ALL
 *   NCCL_GPUDIRECTTCPX_SLOWNESS_REPORT        which of them also print a warning (default: all that are watched)
 *   NCCL_GPUDIRECTTCPX_TELEMETRY_ENABLE_TASK_LEVEL_STATS / ..._REQUEST_LEVEL_STATS   record tracepoint events
 *   NCCL_GPUDIRECTTCPX_TELEMETRY_SAMPLING_FACTOR   keep only objects whose address is a multiple of this
 */

/* Receive-side members of struct tcpxSocketStats (src/stats/monitoring.h:25-39), one per data flow. */
typedef struct tcpxFlowStats {
  uint64_t flow_id;
  uint64_t rx_ctrl_done_cnt; /* control messages that named this flow */
  uint64_t rx_cnt;           /* recvmsg calls, counted while task-level stats are on (src/stats/tracepoint.cc:72-82) */
  uint64_t rx_slow_cnt;      /* slowness reports of recvmsg (src/stats/tracepoint.cc:22-52) */
} tcpxFlowStats;

typedef struct tcpxCommStats {
  uint64_t rx_ctrl_slow_cnt; /* slowness reports while waiting for a control message (src/net_tcpx.cc:1234-1246) */
  uint64_t unpack_cnt;       /* slots handed to the GPU */
  uint64_t unpack_slow_cnt;  /* slowness reports while the GPU held a slot (no counterpart in the reference) */
  uint64_t unpack_ns;        /* publish -> completion word seen by tcpxTest, summed over unpack_cnt slots */
  uint64_t trace_dropped;    /* tracepoint events lost because nobody drained the buffer */
  uint64_t socket_thread_cpus; /* CPUs the comm's socket thread may run on (NCCL_GPUDIRECTTCPX_RX_BINDINGS), 0 = no such thread */
  uint64_t max_slots_at_gpu; /* most slots of this comm that were with the engine at one time (at most 16) */
} tcpxCommStats;

ncclResult_t tcpxGetFlowStats(void* recvComm, uint32_t flow, tcpxFlowStats* stats);
ncclResult_t tcpxGetCommStats(void* recvComm, tcpxCommStats* stats);

/* One tracepoint: a request ('R') or task ('T') entered `state`, numbered as in the exported lines of the
 * reference (src/stats/tracepoint.h:57-75): requests 0 FREE, 1 INACTIVE, 2 TRANSMITTING, 3 ACTIVE, 4 POSTED;
 * tasks 0 FREE, 1 INACTIVE, 2 COMPLETING, 3 ACTIVE.  Fired where the reference fires TCPX_TP
 * (src/work_queue.h:156-211). */
typedef struct tcpxTraceEvent {
  char kind;
  uint8_t passive;
  uint16_t state;
  uint32_t reserved;
  uint64_t object;   /* address of the request or task */
  int64_t timestamp; /* nanoseconds: wall clock since the epoch, or the injected clock */
} tcpxTraceEvent;

/* Takes up to `max` events of the comm, oldest first, waiting up to `wait_ms` for the first
 * (StatsBuffer::dequeue, src/stats/stats_buffer.h:74-93).  *n = 0 if tracing is off. */
ncclResult_t tcpxTraceDrain(void* recvComm, tcpxTraceEvent* events, uint32_t max, uint32_t wait_ms, uint32_t* n);

/* The line the reference's exporter writes for an event: "R 0x... <passive> <state> <timestamp>"
 * (src/stats/stats_buffer.h:52-56).  Returns snprintf's result. */
int tcpxTraceFormat(const tcpxTraceEvent* event, char* line, size_t len);

/* Replaces the clock of the slowness watches and tracepoints (NULL restores CLOCK_MONOTONIC / the wall clock):
 * the injectable `timenow` of struct tcpxTimeoutDetection::Config (src/timeout.h:26-30).  For tests. */
ncclResult_t tcpxSetClockForTesting(uint64_t (*now_ns)(void));

/* ---- 5. The flow scheduler -------------------------------------------------------------------------------------
 * Which flows may take the next chunk of a message: class FlowMapper (src/flow_mapper.h:52-65) with its two
 * policies, FlowMapperRR (:137-157; alg 0) and FlowMapperKaty (:67-135; alg 1), selected per process by
 * NCCL_GPUDIRECTTCPX_SCHED_ALG = "RR" | "KATY" (src/net_tcpx.cc:643-665; anything else means RR).  A receive comm
 * refills its scheduler at every poll with the flows whose task ring has room and takes control messages only
 * while it holds one (src/net_tcpx.cc:1114,1152-1155,1183); Pick is what the sending peer calls per chunk
 * (src/net_tcpx.cc:1216).  These entry points drive one scheduler on its own, for tests and for a synthetic peer.
 * `alg` NULL = the policy the last tcpxInit selected.  Flows are 0..7, priorities 0..5 (task slots in use). */
typedef struct tcpxFlowSched tcpxFlowSched;
ncclResult_t tcpxFlowSchedCreate(const char* alg, tcpxFlowSched** sched);
int tcpxFlowSchedAlg(const tcpxFlowSched* sched);               /* 0 RR, 1 KATY */
void tcpxFlowSchedReset(tcpxFlowSched* sched);                  /* FlowMapper::reset */
int tcpxFlowSchedHasFlow(const tcpxFlowSched* sched);           /* FlowMapper::hasFlow */
void tcpxFlowSchedSchedule(tcpxFlowSched* sched, int flow, int prio); /* FlowMapper::scheduleFlow */
int tcpxFlowSchedPick(tcpxFlowSched* sched);                    /* FlowMapper::pickFlow: a flow, or -1 */
void tcpxFlowSchedDestroy(tcpxFlowSched* sched);

#ifdef __cplusplus
}
#endif
#endif /* TCPX_PLUGIN_H_ */
