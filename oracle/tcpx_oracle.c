/*
 * tcpx_oracle.c -- CPU restatement of the receive-side unpack, plain C.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only tests/, __graft_entry__.smoke() and the cpu_baseline leg
 * of bench.py may load this library; nothing in the shipped libraries links or calls it.
 *
 * What it restates.  The reference (google/nccl-plugin-gpudirecttcpx) only PRODUCES the descriptor list; the
 * consumer that moves the bytes is NCCL's ncclNetDeviceUnpack, an un-vendored build-time dependency located
 * through -DNCCL_PATH (CMakeLists.txt:77-89, no pinned version; ABI tag 0x7 at src/devcomm/nccl/unpack1.h:24-25).
 * Its published contract, fixed by the reference's call sites, is a byte scatter-gather:
 *   descriptor fields  {u32 src_off, u32 len, u64 dst_off}         src/sock/tcpx.h:178-180
 *   16-byte stride, appended per finished task                       src/net_tcpx.cc:1128-1130
 *   count published per slot                                         src/net_tcpx.cc:1354
 *   src_off is relative to the bounce buffer                         src/devcomm/nccl/unpack1.cu:56-58
 *   dst_off is relative to the request's receive buffer              src/sock/tcpx.h:180, src/net_tcpx.cc:1044,1049
 * i.e.  for every descriptor i in order:  dst[dst_off_i + k] = bounce[src_off_i + k],  0 <= k < len_i.
 *
 * How it is pinned.  The reference holds no test, golden vector or fixture for this path (its only tests are
 * src/stats/stats_buffer_test.cc and src/stats/tracepoint_test.cc, telemetry).  tests/test_oracle.py pins
 * tcpx_oracle_unpack against (a) a byte-at-a-time pure-Python loop on tiny inputs, (b) a numpy fancy-index
 * gather on medium inputs, (c) the committed fixtures under tests/golden/, and (d) invariants that a dropped
 * term, swapped src/dst or off-by-one length would break: untouched guard bytes, zero-length no-ops, an
 * identity descriptor list reducing to memcpy, and order independence for disjoint destinations.
 */
#define _GNU_SOURCE
#include <pthread.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

typedef struct {
  uint32_t src_off;
  uint32_t len;
  uint64_t dst_off;
} tcpx_oracle_desc; /* union loadMeta: src/sock/tcpx.h:178-180 */

/* One memcpy per descriptor, in list order (the memcpy-per-descriptor CPU statement of the path). */
void tcpx_oracle_unpack(uint8_t* dst, const uint8_t* bounce, const tcpx_oracle_desc* descs, uint64_t n) {
  for (uint64_t i = 0; i < n; ++i) {
    if (descs[i].len) memcpy(dst + descs[i].dst_off, bounce + descs[i].src_off, descs[i].len);
  }
}

/* Bounds audit used by tests before any buffer is touched: returns the index of the first descriptor that
 * reads outside [0,bounce_bytes) or writes outside [0,dst_bytes), or -1 if all are inside. */
int64_t tcpx_oracle_first_out_of_bounds(const tcpx_oracle_desc* descs, uint64_t n, uint64_t bounce_bytes,
                                        uint64_t dst_bytes) {
  for (uint64_t i = 0; i < n; ++i) {
    const uint64_t s = descs[i].src_off, l = descs[i].len, d = descs[i].dst_off;
    if (s + l > bounce_bytes || d + l > dst_bytes || d + l < d) return (int64_t)i;
  }
  return -1;
}

/* ---- timed multi-thread variant: the reported CPU baseline ---------------------------------------------- */

typedef struct {
  uint8_t* dst;
  const uint8_t* bounce;
  const tcpx_oracle_desc* descs;
  uint64_t begin, end;
  int iters;
  pthread_barrier_t* barrier;
} worker_arg;

static void* worker_main(void* p) {
  worker_arg* a = (worker_arg*)p;
  for (int it = 0; it < a->iters; ++it) {
    pthread_barrier_wait(a->barrier); /* start of iteration */
    tcpx_oracle_unpack(a->dst, a->bounce, a->descs + a->begin, a->end - a->begin);
    pthread_barrier_wait(a->barrier); /* end of iteration */
  }
  return NULL;
}

static double now_s(void) {
  struct timespec ts;
  clock_gettime(CLOCK_MONOTONIC, &ts);
  return (double)ts.tv_sec + 1e-9 * (double)ts.tv_nsec;
}

/* Runs the descriptor list `warmup + iters` times on `threads` threads (descriptor list range-partitioned,
 * threads created once), and writes the wall time of each timed iteration to seconds[0..iters).
 * Returns 0 on success. */
int tcpx_oracle_unpack_timed(uint8_t* dst, const uint8_t* bounce, const tcpx_oracle_desc* descs, uint64_t n,
                             int threads, int warmup, int iters, double* seconds) {
  if (threads < 1 || iters < 1 || warmup < 0 || !seconds) return 1;
  const int total = warmup + iters;
  pthread_barrier_t barrier;
  if (pthread_barrier_init(&barrier, NULL, (unsigned)threads + 1)) return 2;
  pthread_t* tids = (pthread_t*)calloc((size_t)threads, sizeof *tids);
  worker_arg* args = (worker_arg*)calloc((size_t)threads, sizeof *args);
  if (!tids || !args) return 3;
  for (int t = 0; t < threads; ++t) {
    args[t].dst = dst;
    args[t].bounce = bounce;
    args[t].descs = descs;
    args[t].begin = n * (uint64_t)t / (uint64_t)threads;
    args[t].end = n * (uint64_t)(t + 1) / (uint64_t)threads;
    args[t].iters = total;
    args[t].barrier = &barrier;
    if (pthread_create(&tids[t], NULL, worker_main, &args[t])) return 4;
  }
  for (int it = 0; it < total; ++it) {
    const double t0 = now_s();
    pthread_barrier_wait(&barrier);
    pthread_barrier_wait(&barrier);
    const double t1 = now_s();
    if (it >= warmup) seconds[it - warmup] = t1 - t0;
  }
  for (int t = 0; t < threads; ++t) pthread_join(tids[t], NULL);
  pthread_barrier_destroy(&barrier);
  free(tids);
  free(args);
  return 0;
}
