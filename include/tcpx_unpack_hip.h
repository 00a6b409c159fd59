/*
 * tcpx_unpack_hip.h -- C-ABI of the HIP layer (libtcpxu_hip.so) of the MI355X receive-side unpack path.
 *
 * Everything the host-side plugin needs from the GPU goes through these entry points: plain pointers and
 * sizes, no C++ types, no torch types.  Each entry point names the interface of the reference
 * (google/nccl-plugin-gpudirecttcpx, paths relative to its root) that it stands in for.
 *
 * Result codes are the numeric values of ncclResult_t that the reference returns through its adapter
 * (src/adapter/nccl/ret.h:22-31): 0 success, 1 unhandled device error, 2 system error, 3 internal error,
 * 4 invalid argument, 5 invalid usage.
 */
#ifndef TCPX_UNPACK_HIP_H_
#define TCPX_UNPACK_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TCPXU_SUCCESS 0
#define TCPXU_DEVICE_ERROR 1
#define TCPXU_SYSTEM_ERROR 2
#define TCPXU_INTERNAL_ERROR 3
#define TCPXU_INVALID_ARGUMENT 4
#define TCPXU_INVALID_USAGE 5
#define TCPXU_IN_PROGRESS 7 /* ncclInProgress: nothing wrong, try again */

/* One unpack descriptor: copy `len` bytes from bounce_base + src_off to dst_base + dst_off.
 * Same 16-byte layout as NCCL's `union loadMeta`, whose fields the reference fills at
 * src/sock/tcpx.h:178-180 and whose 16-byte stride it relies on at src/net_tcpx.cc:1128-1130. */
typedef struct tcpxuLoadMeta {
  uint32_t src_off;
  uint32_t len;
  uint64_t dst_off;
} tcpxuLoadMeta;

/* Ring geometry the reference compiles against (NCCL's NCCL_NET_DEVICE_UNPACK_MAX_QUEUE_DEPTH and
 * NET_UNPACK_MAX_SLICE_PAGES; used at src/devcomm/nccl/unpack_defs1.h:22-23). */
#define TCPXU_QUEUE_DEPTH 16
#define TCPXU_SLOT_PAGES 2048
#define TCPXU_PAGE_SIZE 4096

/* ---- device selection -------------------------------------------------------------------------------- */

/* Number of visible GPUs.  Replaces gpu_n_dev (src/gpu/cuda_wrapper.cu:49-60). */
int tcpxuDeviceCount(int* count);

/* Human-readable name and compute-unit count of a GPU (for bench output). */
int tcpxuDeviceInfo(int device, char* name, size_t name_len, int* compute_units);

/* Last error message of the calling thread ("" if none). */
const char* tcpxuLastError(void);

/* ---- (1) bounce-page arena in HBM -------------------------------------------------------------------- */

/* Allocates `bytes` of device memory as the bounce-page arena (4 KiB-aligned base) and returns its device
 * address.  Replaces gpu_get_rxmem / GpumemImport, which import the receive-datapath-manager's NIC-bound page
 * pool (src/gpu/cuda_wrapper.cu:214-224, src/gpu/rx_pool.cu:62-121): here the pool is a plain hipMalloc. */
int tcpxuArenaCreate(int device, size_t bytes, void** arena_base);
int tcpxuArenaDestroy(int device, void* arena_base);

/* Plain device buffers and copies, so that a host driver needs no other GPU runtime. */
int tcpxuDeviceAlloc(int device, size_t bytes, void** ptr);
int tcpxuDeviceFree(int device, void* ptr);
int tcpxuCopyToDevice(int device, void* dst_dev, const void* src_host, size_t bytes);
int tcpxuCopyToHost(int device, void* dst_host, const void* src_dev, size_t bytes);
int tcpxuFillDevice(int device, void* dst_dev, int byte_value, size_t bytes);
int tcpxuDeviceSynchronize(int device);

/* ---- (2) host-mapped unpack-metadata memory ---------------------------------------------------------- */

/* Allocates `bytes` of pinned host memory that the GPU can read and write (hipHostMalloc, mapped and
 * coherent) and returns both addresses.  Replaces the cuMemHostAlloc(DEVICEMAP|PORTABLE) +
 * cuMemHostGetDevicePointer pair of __tcpxNetDeviceQueueNew (src/devcomm/nccl/unpack1.cu:41-43,54). */
int tcpxuMappedAlloc(int device, size_t bytes, void** host_ptr, void** dev_ptr);
int tcpxuMappedFree(int device, void* host_ptr);

/* Allocates `bytes` (at most 64 MiB) of DEVICE memory that the host can write through the PCIe BAR, for the few
 * bytes per request that the GPU should not have to fetch over PCIe itself: a caller copies the descriptors of a
 * small request here (in addition to the mapped slot above), calls tcpxuVisibleFlush, and only then submits the
 * request with this copy's device address as `descs`.  The copy is a posted write that PCIe delivers before the
 * completion of any later read by the GPU of host memory written after the flush, so a GPU that has seen the
 * submission finds the descriptors in its own memory (a lone request of 1..16 descriptors completes 0.7-1.3 us
 * sooner).  Write-combined for the host: write whole records, never read.  TCPXU_INVALID_USAGE if the device
 * does not expose its memory to the host (no large BAR) or TCPXU_VISIBLE_DEVICE_MEMORY=0; callers then simply go
 * without.  Freed blocks are kept for later allocations and are not returned to the driver.  No counterpart in
 * the reference, whose consumer (NCCL's kernel) always reads the mapped slot. */
int tcpxuVisibleAlloc(int device, size_t bytes, void** host_ptr, void** dev_ptr);
int tcpxuVisibleFree(int device, void* host_ptr);
void tcpxuVisibleFlush(void); /* orders the host's writes to such memory before its later stores (sfence) */

/* ---- (3) launch-per-batch unpack --------------------------------------------------------------------- */

/* Scatter-gathers `n_descs` descriptors with one kernel launch on `stream` (a hipStream_t, NULL = the
 * default stream): for each i, dst_base[dst_off_i .. +len_i) = bounce_base[src_off_i .. +len_i).
 * `descs` must be readable by the GPU (device memory or the device alias of mapped host memory).
 * Asynchronous; zero-length descriptors are skipped; destination ranges must not overlap each other.
 * Stands in for the consumer the reference feeds, NCCL's ncclNetDeviceUnpack (not part of the reference
 * tree; selected at CMakeLists.txt:77-89), for one slot's descriptor list (src/net_tcpx.cc:1128-1130,1354). */
int tcpxuUnpackBatch(int device, const void* bounce_base, void* dst_base, const tcpxuLoadMeta* descs,
                     uint64_t n_descs, void* stream);

/* ---- (4) persistent unpack engine -------------------------------------------------------------------- */

/* One engine per GPU: a persistent kernel that polls a submission ring in mapped host memory, unpacks every
 * submitted slot and writes a completion word back to mapped host memory -- no kernel launch per request.
 * It takes the place of the NCCL collective kernel that runs ncclNetDeviceUnpack and of the head counter in
 * `struct unpackNetDeviceHandle` (src/devcomm/nccl/unpack1.cu:53-63). */
typedef struct tcpxuEngine tcpxuEngine;

typedef struct tcpxuEngineConfig {
  uint32_t ring_entries;    /* submission ring size, power of two >= 16, 0 = default (4096) */
  uint32_t workgroups;      /* persistent grid size, 0 = two worker workgroups per compute unit + the leader */
  uint32_t descs_per_ticket;/* descriptors one workgroup takes at a time (1..64); 0 = chosen per submission from
                               the backlog of descriptors not yet unpacked: 8 when the engine is idle (lowest
                               latency), 12, then 14 while the backlog is there but shallow (below 100 descriptors
                               per workgroup), 16 when it is deep (highest throughput), and with a payload hint that
                               tells of short fragments 32, 48 or 64; a submission of at most 32 descriptors stays
                               whole once 8 or more are in flight (tcpxuEngineTicketPlan gives the same answers) */
  uint32_t spin_limit;      /* the kernel leaves by itself after this many consecutive empty polls of the ring
                               (about 1.2 us each) and is launched again by the next submission, so that a
                               device-wide synchronize never waits on an idle engine; 0 = default (400, about
                               half a millisecond), 0xFFFFFFFF = never leave */
} tcpxuEngineConfig;

int tcpxuEngineCreate(int device, const tcpxuEngineConfig* config, tcpxuEngine** engine);
/* Launches the persistent kernel.  The engine can be started and stopped repeatedly; a submission made while
 * the kernel is away (never started after a stop excepted) brings it back. */
int tcpxuEngineStart(tcpxuEngine* engine);
/* Asks the kernel to drain and exit, waits for it, and reports the duration of that launch in
 * microseconds as measured by HIP events on the engine's stream (elapsed_us may be NULL). */
int tcpxuEngineStop(tcpxuEngine* engine, double* elapsed_us);
int tcpxuEngineDestroy(tcpxuEngine* engine);

/* Publishes one slot: `n_descs` descriptors at `descs_dev` (device-visible address, normally the device
 * alias of a slot of the mapped queue), gathered from `bounce_base` into `dst_base`.  When the GPU has
 * written every byte it stores `done_value` (nonzero) to `*done_flag_dev` (device alias of a mapped 8-byte
 * word that the host poller reads).  Returns TCPXU_IN_PROGRESS if the ring is full (caller retries).
 * This is the publish of src/net_tcpx.cc:1354-1357 made explicit: count, then a release, then the tail. */
int tcpxuEngineSubmit(tcpxuEngine* engine, const void* bounce_base, void* dst_base, const void* descs_dev,
                      uint32_t n_descs, void* done_flag_dev, uint64_t done_value);
/* The same with a hint: `payload_bytes` = the sum of the descriptors' lengths (the size of the request, which the
 * caller of src/net_tcpx.cc:1354-1357 has at hand in tcpxRequest::offset), 0 = unknown.  The engine hands out a
 * slot's descriptors in tickets of 16 fragments of a page; with the hint, a slot of shorter fragments gets tickets
 * of more descriptors (32, 48, up to 64).  Without it fragments are taken to be whole pages. */
int tcpxuEngineSubmitSized(tcpxuEngine* engine, const void* bounce_base, void* dst_base, const void* descs_dev,
                           uint32_t n_descs, uint64_t payload_bytes, void* done_flag_dev, uint64_t done_value);

/* Several slots published under one lock with one store of the ring's tail: what a poller that finds several
 * requests complete in one pass submits together (a storm of small requests is bound by the host's cost per
 * publish).  All `n` submissions are checked first and none is queued if one is refused (TCPXU_INVALID_ARGUMENT).
 * *accepted (may be NULL) receives how many went into the ring, in order from the first: all of them with
 * TCPXU_SUCCESS, fewer (possibly none) with TCPXU_IN_PROGRESS when the ring is full -- the caller submits the rest
 * later.  payload_bytes as in tcpxuEngineSubmitSized (0 = unknown; sizes of 4 GiB and more are passed as 2^32-1). */
typedef struct tcpxuSubmission {
  const void* bounce_base;
  void* dst_base;
  const void* descs_dev;
  void* done_flag_dev;
  uint64_t done_value;
  uint32_t n_descs;
  uint32_t payload_bytes;
} tcpxuSubmission;
int tcpxuEngineSubmitMany(tcpxuEngine* engine, const tcpxuSubmission* submissions, uint32_t n, uint32_t* accepted);

/* Limits: n_descs may not exceed 65536 tickets' worth -- 65536 x descs_per_ticket, or 524288 (65536 x 8) with
 * descs_per_ticket = 0, and never 1048576: TCPXU_INVALID_ARGUMENT otherwise, decided on the host, nothing queued.
 * TCPXU_INTERNAL_ERROR from a submit means the kernel stopped answering while the entry was already queued: the
 * engine then refuses every later submit, so a caller cannot queue the same work twice by retrying. */

/* The ticket arithmetic of the engine, on the host (no GPU needed): for an engine of `workgroups` workgroups and
 * the given descs_per_ticket (0 = by backlog), a submission of n_descs descriptors and payload_bytes (0 = unknown)
 * with `in_flight` submissions not yet completed (itself included) is handed out in *n_tickets tickets of
 * *per_ticket descriptors; *max_descs is the most descriptors a submission may carry.  Outputs may be NULL.
 * (One more rule lives in the kernel alone, because it depends on what the leader finds at run time: while eight or
 * more submissions wait in one of its polls, tickets sized by backlog are at least 16 descriptors.)
 * TCPXU_INVALID_ARGUMENT for an n_descs beyond that limit. */
int tcpxuEngineTicketPlan(uint32_t workgroups, uint32_t descs_per_ticket, uint32_t in_flight, uint32_t n_descs,
                          uint64_t payload_bytes, uint32_t* per_ticket, uint32_t* n_tickets, uint32_t* max_descs);

/* Number of submissions the GPU has fully completed since creation (monotone; read from mapped memory). */
int tcpxuEngineCompleted(tcpxuEngine* engine, uint64_t* completed);

/* Counters since creation.  The leader's are written by the kernel when it leaves (stop or idle exit), so they
 * are current after tcpxuEngineStop: polls of the submission ring, entries those polls consumed, and how many of
 * the polls fetched 64 entries instead of 16 (the leader does that after a poll that found all sixteen there; with
 * hundreds of entries published ahead of it the leader keeps several groups of sixteen in flight instead of
 * polling, and every 64 entries taken that way count as one such poll). */
typedef struct tcpxuEngineStats {
  uint64_t launches;
  uint64_t submissions;
  uint64_t leader_polls;
  uint64_t leader_entries;
  uint64_t leader_deep_polls;
} tcpxuEngineStats;
int tcpxuEngineGetStats(tcpxuEngine* engine, tcpxuEngineStats* stats);

/* Where a submission's time goes inside the GPU, for measurement (no counterpart in the reference).  After
 * tcpxuEngineEnableStamps (engine stopped; *ticks_per_us, may be NULL, receives the rate of the GPU's constant
 * clock) the kernel keeps four readings of that clock per submission: [0] the leader saw its entry, [1] a
 * workgroup had fetched the first of its tickets, [2] that workgroup had the ticket's descriptors staged, [3] the
 * workgroup that completed it had its last store acknowledged.  tcpxuEngineReadStamps (engine stopped) copies the
 * readings of submissions first_submission .. +n (counted from the engine's creation; n at most ring_entries, and
 * only the last ring_entries submissions are kept) into out[4 * n] and clears them.  A reading of all ones means
 * "never taken".  Readings [1] and [2] are kept as minima and only reading clears them: read at least once every
 * ring_entries submissions, or they may be those of the submission that had the same place in the ring before. */
int tcpxuEngineEnableStamps(tcpxuEngine* engine, double* ticks_per_us);
int tcpxuEngineReadStamps(tcpxuEngine* engine, uint64_t first_submission, uint32_t n, uint64_t* out);

/* The configuration in effect (defaults resolved: actual grid size, ring size; ticket size 0 = by backlog). */
int tcpxuEngineGetConfig(tcpxuEngine* engine, tcpxuEngineConfig* config);

/* The GPU the engine was created on. */
int tcpxuEngineDevice(tcpxuEngine* engine, int* device);

/* 1 if the persistent kernel is running, 0 if stopped or away after being idle. */
int tcpxuEngineRunning(tcpxuEngine* engine, int* running);

/* ---- (5) one slot without any allocation ---------------------------------------------------------------- */

/* tcpxuEngineSubmit for callers that cannot allocate and cannot keep a persistent kernel: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.
 * Unpacks one slot -- `n_descs` descriptors (at most TCPXU_SLOT_PAGES = 2048; more is TCPXU_INVALID_ARGUMENT and
 * nothing is launched) at `descs_dev`, from `bounce_base` into `dst_base` -- with ordinary launches on `stream`
 * (a hipStream_t, NULL = the default stream): the engine's worker workgroups over tickets that a small kernel
 * writes first, and the workgroup that finishes the slot's last ticket stores `done_value` to `*done_flag_dev`
 * (device-visible 8-byte word, e.g. the alias of mapped host memory; may be NULL when stream order is all the
 * caller needs).  Asynchronous.  It calls no hipMalloc, hipFree or other allocating routine: ticket records,
 * ticket cursor and done counters live in a fixed array of device memory inside the library (17 KiB, held by
 * every GPU the library runs on until the process ends), which every call on a GPU shares and which each call
 * clears with its own first kernel.  Calls that overlap on one GPU (two streams, two threads) race on that
 * array: issue them on one stream, or order them otherwise.  (A workgroup that finds its ticket overwritten by
 * such a race gives up after 65536 looks and stores the complement of `done_value` to the completion word, so that
 * a poller is not left waiting; the slot's bytes are then not all there.)
 * Under HIP graph capture: make one ordinary call on the device first -- it looks up the array's address and loads
 * the kernels' code, which do not belong under capture -- then capture; a replay launches the same two kernels
 * with the same arguments. */
int tcpxuUnpackSlotNoAlloc(int device, const void* bounce_base, void* dst_base, const void* descs_dev,
                           uint32_t n_descs, void* done_flag_dev, uint64_t done_value, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* TCPX_UNPACK_HIP_H_ */
