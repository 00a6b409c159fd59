/*
 * tcpx_unpack_bench.h -- C-ABI of the measurement helpers (libtcpxu_bench.so).
 *
 * Nothing here is part of the product: libtcpxu_bench.so is a client of libtcpxu_hip.so (it calls only what
 * include/tcpx_unpack_hip.h declares) that drives the unpack engine the way the plugin's proxy loop does, with no
 * Python in the loop, and times kernels with HIP events on the stream they are launched on.  Benchmarks and
 * tests load it; the plugin never does.  None of it has a counterpart in the reference
 * (google/nccl-plugin-gpudirecttcpx), whose consumer kernel lives in NCCL and which ships no benchmark.
 *
 * Result codes as in tcpx_unpack_hip.h.
 */
#ifndef TCPX_UNPACK_BENCH_H_
#define TCPX_UNPACK_BENCH_H_

#include <stddef.h>
#include <stdint.h>

#include "tcpx_unpack_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Last error message of the calling thread from this library ("" if none). */
const char* tcpxuBenchLastError(void);

/* tcpxuUnpackBatch bracketed by HIP events on its stream, repeated `iters` times after `warmup` untimed ones;
 * writes the mean duration of one launch in microseconds. */
int tcpxuUnpackBatchTimed(int device, const void* bounce_base, void* dst_base, const tcpxuLoadMeta* descs,
                          uint64_t n_descs, int warmup, int iters, double* mean_us);

/* Plain device-to-device copy kernel of `bytes` (multiple of 16), timed the same way: the achievable-copy
 * yardstick printed beside the unpack figure, and the known-size kernel used to calibrate HBM counters.
 * With dst == NULL only the loads are issued (a read of `bytes`), with src == NULL only the stores (a fill):
 * what the memory system gives to each half of a copy on its own. */
int tcpxuCopyKernelTimed(int device, void* dst, const void* src, size_t bytes, int warmup, int iters,
                         double* mean_us);

/* A bare gather, timed the same way: the first fragment_bytes (1024, 2048, 3072 or 4096) of page pages_dev[i] (a
 * list of n_fragments 4 KiB page numbers in device memory) of `src` to dst + i * fragment_bytes, one wavefront per
 * fragment with the unpack kernel's loads and stores and nothing else.  The yardstick for workloads of short
 * fragments: what the memory system gives to a gather of that grain. */
int tcpxuGatherKernelTimed(int device, void* dst, const void* src, const uint32_t* pages_dev, uint32_t n_fragments,
                           uint32_t fragment_bytes, int warmup, int iters, double* mean_us);

/* Launches the copy kernel once on `stream` (a hipStream_t) and returns: something else for the GPU to do while
 * the engine runs. */
int tcpxuCopyKernelLaunch(int device, void* dst, const void* src, size_t bytes, void* stream);

/* ---- streaming driver ----------------------------------------------------------------------------------- */

/* One slot's worth of work. */
typedef struct tcpxuStreamItem {
  const void* bounce_base;
  void* dst_base;
  const tcpxuLoadMeta* descs_host; /* descriptors in ordinary host memory */
  uint32_t n_descs;                /* at most TCPXU_SLOT_PAGES */
  uint32_t payload_bytes;          /* sum of the descriptors' lengths, 0 = unknown (see tcpxuEngineSubmitSized) */
} tcpxuStreamItem;

/* Slots the streaming driver can keep in flight: the unpack queues of 128 receive comms (the storm of 2048
 * concurrent small requests) -- with whole slots of TCPXU_SLOT_PAGES descriptors up to the queues of eight comms,
 * beyond that for items of at most 64 descriptors only. */
#define TCPXU_STREAM_MAX_DEPTH (128 * TCPXU_QUEUE_DEPTH)
#define TCPXU_STREAM_FULL_SLOT_DEPTH (8 * TCPXU_QUEUE_DEPTH)

/* Drives a started engine the way the plugin's proxy loop does, from one host thread: a mapped ring of `depth`
 * slots (1..TCPXU_STREAM_MAX_DEPTH; TCPXU_QUEUE_DEPTH is one comm's unpack queue, a multiple of it is that many
 * comms taking turns) of TCPXU_SLOT_PAGES descriptors each (of 64 beyond TCPXU_STREAM_FULL_SLOT_DEPTH); for every item, in order: wait until the slot's
 * previous occupant has completed, copy the item's descriptors into the slot (the memcpy of
 * src/net_tcpx.cc:1128-1130), publish it (src/net_tcpx.cc:1354-1357), and poll completion words in FIFO order
 * (the tcpxTest / tcpxIrecvConsumed cadence).  Writes the wall time from the first publish to the last
 * completion to *wall_us and, if latency_us is not NULL, each item's publish-to-completion-seen time in
 * microseconds to latency_us[0..n_items).  Returns TCPXU_INTERNAL_ERROR if nothing completes for
 * `stall_timeout_ms` milliseconds.  One stream at a time per process. */
int tcpxuEngineStream(tcpxuEngine* engine, const tcpxuStreamItem* items, uint64_t n_items, uint32_t depth,
                      uint32_t stall_timeout_ms, double* wall_us, double* latency_us);

/* Where the host thread's time went in the process's last stream (any of the calls below): nanoseconds inside the
 * publish step (descriptors into the slot where not staged ahead, the batch of submissions, tcpxuEngineSubmitMany),
 * the submissions and calls that made, the passes of the loop and the stream's wall time. */
typedef struct tcpxuStreamSplit {
  double publish_ns;
  double wall_ns;
  uint64_t published;
  uint64_t publish_calls;
  uint64_t passes;
} tcpxuStreamSplit;
int tcpxuStreamLastSplit(tcpxuStreamSplit* split);

/* Same, with the first `warmup_items` items left out of *wall_us: the clock starts at the publish of item
 * `warmup_items` and stops at the last completion. */
int tcpxuEngineStreamWarm(tcpxuEngine* engine, const tcpxuStreamItem* items, uint64_t n_items,
                          uint64_t warmup_items, uint32_t depth, uint32_t stall_timeout_ms, double* wall_us,
                          double* latency_us);

/* tcpxuEngineStart + tcpxuEngineStream + tcpxuEngineStop in one call on a stopped engine, so that the
 * persistent kernel's launch covers exactly these items (warm-up included); *kernel_us is that launch's duration
 * from HIP events on the engine's stream (the figure a kernel trace shows for it), *wall_us as in
 * tcpxuEngineStreamWarm. */
int tcpxuEngineRunTimed(tcpxuEngine* engine, const tcpxuStreamItem* items, uint64_t n_items,
                        uint64_t warmup_items, uint32_t depth, uint32_t stall_timeout_ms, double* wall_us,
                        double* kernel_us, double* latency_us);

/* Like tcpxuEngineRunTimed, but *wall_us covers items [first_timed, first_timed + n_timed) from completion to
 * completion: the clock starts when item first_timed - 1 is seen completed (at the first publish if first_timed
 * is 0) and stops when item first_timed + n_timed - 1 is; items after that keep the queues full while the timed
 * ones finish. */
int tcpxuEngineRunWindow(tcpxuEngine* engine, const tcpxuStreamItem* items, uint64_t n_items, uint64_t first_timed,
                         uint64_t n_timed, uint32_t depth, uint32_t stall_timeout_ms, double* wall_us,
                         double* kernel_us, double* latency_us);

/* One launch over all items, every completion stamped: done_us[i] = the time, in microseconds since the first
 * publish, at which the host poller saw item i completed (FIFO order, so the stamps never decrease).  A caller
 * cuts any number of completion-to-completion windows out of one launch with these.  *kernel_us and latency_us as
 * in tcpxuEngineRunTimed (latency_us may be NULL). */
int tcpxuEngineRunStamped(tcpxuEngine* engine, const tcpxuStreamItem* items, uint64_t n_items, uint32_t depth,
                          uint32_t stall_timeout_ms, double* kernel_us, double* done_us, double* latency_us);

#ifdef __cplusplus
}
#endif
#endif /* TCPX_UNPACK_BENCH_H_ */
