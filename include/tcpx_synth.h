/*
 * tcpx_synth.h -- C-ABI of the synthetic fragment source (libtcpx_synth.so).
 *
 * There is no NIC, no devmem-TCP socket and no sender in this build.  What the Linux kernel would report for
 * every received fragment -- `struct devmemvec {frag_offset, frag_size, frag_token}` in an SCM_DEVMEM_OFFSET
 * cmsg (reference: src/sock/tcpx.h:130-134,178-181) -- is generated from a seed instead, for the five
 * workloads the benchmark contract names.  The same object also carries the descriptor list that those
 * fragments produce when they arrive in order, so kernels can be driven without the plugin on top.
 *
 * Every workload obeys the devmem contract behind src/sock/tcpx.h:157-181: a fragment is at most one 4 KiB
 * page and never crosses a page boundary.  A message is cut into requests of at most 4 MiB and at most 2048
 * descriptors (NCCL's slice limits, which the reference enforces at src/net_tcpx.cc:1350-1353 and
 * src/sock/tcpx.h:183-187).
 */
#ifndef TCPX_SYNTH_H_
#define TCPX_SYNTH_H_

#include <stddef.h>
#include <stdint.h>

#include "tcpx_unpack_hip.h" /* tcpxuLoadMeta */

#ifdef __cplusplus
extern "C" {
#endif

/* Workload ids (the order of the benchmark contract's configs). */
#define TCPX_SYNTH_ALIGNED_1M 1   /* 1 MiB, 256 page-aligned 4 KiB fragments, 16 MiB pool, permuted pages      */
#define TCPX_SYNTH_CHUNK_8M 2     /* 8 MiB chunk, 4 flows, 90% 4 KiB / 10% U[64,4095], byte-unaligned sources   */
#define TCPX_SYNTH_STORM_64K 3    /* 2048 requests x 16 x 4 KiB, 512 MiB pool                                   */
#define TCPX_SYNTH_BULK_256M 4    /* 256 MiB, 65536 page-aligned fragments permuted over a 1 GiB pool           */
#define TCPX_SYNTH_ADVERSARIAL 5  /* 32 MiB, len U[1,4096], 10% empty, dst base +3, pages reused across windows */

typedef struct tcpxSynthFrag {
  uint32_t frag_offset; /* byte offset of the fragment in the bounce arena      (devmemvec.frag_offset) */
  uint32_t frag_size;   /* bytes                                                (devmemvec.frag_size)   */
  uint32_t frag_token;  /* page token to give back when the data is consumed    (devmemvec.frag_token)  */
  uint32_t flow;        /* data flow (socket index) the fragment arrived on                              */
} tcpxSynthFrag;

typedef struct tcpxSynthRequest {
  uint64_t first_desc; /* index of the request's first descriptor / fragment                          */
  uint64_t dst_off;    /* offset of the request's receive buffer from the message's destination base  */
  uint32_t n_descs;
  uint32_t bytes;      /* sum of its fragment sizes (what irecv is posted with)                       */
  uint32_t window;     /* pool generation its pages hold (0 unless pages are reused between requests) */
  uint32_t reserved;
} tcpxSynthRequest;

typedef struct tcpxSynthInfo {
  uint64_t pool_bytes;    /* size of the bounce arena the offsets refer to                          */
  uint64_t payload_bytes; /* sum of all fragment sizes                                              */
  uint64_t dst_bytes;     /* bytes of destination covered, counted from the destination base        */
  uint64_t n_descs;
  uint32_t n_requests;
  uint32_t n_flows;
  uint32_t n_windows;     /* >1: the pool must be refilled (tcpxSynthFillWindow) between windows    */
  uint32_t dst_misalign;  /* destination base = a 256-byte aligned address + this many bytes        */
} tcpxSynthInfo;

typedef struct tcpxSynthWorkload tcpxSynthWorkload;

/* Generates workload `config` from `seed`.  `shrink` divides the workload's byte sizes and pool by 2^shrink
 * (0 = the full contract size), keeping its structure, for quick tests.  Returns 0 on success. */
int tcpxSynthCreate(int config, uint64_t seed, uint32_t shrink, tcpxSynthWorkload** workload);
void tcpxSynthDestroy(tcpxSynthWorkload* workload);

int tcpxSynthGetInfo(const tcpxSynthWorkload* workload, tcpxSynthInfo* info);
/* Arrays owned by the workload, valid until it is destroyed.  Descriptor i corresponds to fragment i; its
 * dst_off is relative to the message's destination base (subtract the request's dst_off to get the value the
 * plugin writes for a request posted at its own buffer). */
const tcpxuLoadMeta* tcpxSynthDescs(const tcpxSynthWorkload* workload);
const tcpxSynthFrag* tcpxSynthFrags(const tcpxSynthWorkload* workload);
const tcpxSynthRequest* tcpxSynthRequests(const tcpxSynthWorkload* workload);

/* Writes the payload of pool generation `window` into `pool` (host memory, pool_bytes long).  Window 0 fills
 * the whole pool with seeded bytes; a later window overwrites only the pages its requests use, the way a NIC
 * refills recycled pages.  Deterministic in (seed, window, byte position). */
int tcpxSynthFillWindow(const tcpxSynthWorkload* workload, uint32_t window, uint8_t* pool);

/* How far apart two CPUs are: nanoseconds for a cache line to go from `cpu_a` to `cpu_b` and back, averaged over
 * `rounds`, measured by two threads of this call, one pinned to each.  Two threads that hand work to each other (a
 * proxy thread and the plugin's socket thread) cost this per hand-over, and on a host whose CPUs span sockets it
 * varies tenfold between pairs; a measurement says which pair it ran on.  Returns 0; 4 for bad arguments; 2 if a
 * CPU cannot be used. */
int tcpxSynthCpuRoundTripNs(int cpu_a, int cpu_b, uint32_t rounds, double* ns);

#ifdef __cplusplus
}
#endif
#endif /* TCPX_SYNTH_H_ */
