/*
 * emu_device_ops.c -- a tcpxDeviceOps table for host-logic tests on a machine without a GPU.
 *
 * TEST INFRASTRUCTURE.  It lives under tests/ and is installed through tcpxSetDeviceOpsForTesting by the tests
 * only; the plugin never selects it.  "Device" memory is host memory, a mapped block's device alias is its own
 * address, and the "engine" moves bytes with the CPU oracle (oracle/tcpx_oracle.c), either at once or -- when
 * held -- only when the test releases it, so that a test can watch a request stay not-done while its copy is
 * outstanding.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include "tcpx_plugin.h"

typedef struct {
  uint32_t src_off;
  uint32_t len;
  uint64_t dst_off;
} tcpx_oracle_desc;
void tcpx_oracle_unpack(uint8_t* dst, const uint8_t* bounce, const tcpx_oracle_desc* descs, uint64_t n);

#define EMU_MAX_PENDING 4096
typedef struct {
  const void* bounce;
  void* dst;
  const void* descs;
  uint32_t n;
  uint64_t* flag;
  uint64_t value;
} emu_job;

struct tcpxuEngine {
  int started;
};

static struct tcpxuEngine g_engine;
static emu_job g_pending[EMU_MAX_PENDING];
static int g_n_pending = 0;
static int g_hold = 0;
static int g_skip_copy = 0;
static int g_ring_full = 0;
static uint64_t g_submitted = 0, g_mapped_live = 0, g_device_live = 0, g_arenas_live = 0, g_engine_starts = 0;
/* "Device memory that the host can write": host memory here; the blocks are remembered so that a submission whose
 * descriptors lie in one can be counted. */
#define EMU_MAX_VISIBLE 256
static struct { uint8_t* p; size_t bytes; } g_visible[EMU_MAX_VISIBLE];
static uint64_t g_visible_live = 0, g_staged_submits = 0, g_visible_flushes = 0, g_last_payload_bytes = 0;
static int g_visible_off = 0;
static int in_visible(const void* p);

static void run_job(const emu_job* j) {
  if (j->n && !g_skip_copy) tcpx_oracle_unpack((uint8_t*)j->dst, (const uint8_t*)j->bounce, (const tcpx_oracle_desc*)j->descs, j->n);
  __atomic_store_n(j->flag, j->value, __ATOMIC_RELEASE);
}

/* ---- test controls -------------------------------------------------------------------------------------------- */
void emu_set_hold(int hold) { g_hold = hold; }
void emu_set_skip_copy(int skip) { g_skip_copy = skip; } /* completes submissions without moving bytes: for timing the host code alone */
void emu_set_ring_full(int full) { g_ring_full = full; }
void emu_set_visible_off(int off) { g_visible_off = off; } /* allocations of host-visible device memory fail */
int emu_pending(void) { return g_n_pending; }
int emu_release(int n) { /* completes the n oldest held submissions; returns how many were completed */
  int done = 0;
  while (done < n && g_n_pending > 0) {
    run_job(&g_pending[0]);
    memmove(&g_pending[0], &g_pending[1], sizeof(emu_job) * (size_t)(g_n_pending - 1));
    --g_n_pending;
    ++done;
  }
  return done;
}
int emu_release_at(int index) { /* completes the held submission at `index` (0 = oldest) ahead of the others */
  if (index < 0 || index >= g_n_pending) return 0;
  run_job(&g_pending[index]);
  memmove(&g_pending[index], &g_pending[index + 1], sizeof(emu_job) * (size_t)(g_n_pending - index - 1));
  --g_n_pending;
  return 1;
}
uint64_t emu_counter(int which) {
  switch (which) {
    case 0: return g_submitted;
    case 1: return g_mapped_live;
    case 2: return g_device_live;
    case 3: return g_arenas_live;
    case 4: return g_engine_starts;
    case 5: return g_visible_live;
    case 6: return g_staged_submits;
    case 7: return g_visible_flushes;
    case 8: return g_last_payload_bytes;
    default: return 0;
  }
}

/* ---- the table -------------------------------------------------------------------------------------------------- */
static int emu_device_count(int* n) { *n = 1; return 0; }
static int emu_arena_create(int dev, size_t bytes, void** base) {
  (void)dev;
  if (bytes == 0 || bytes % 4096) return 4;
  if (posix_memalign(base, 4096, bytes)) return 2;
  memset(*base, 0, bytes);
  ++g_arenas_live;
  return 0;
}
static int emu_arena_destroy(int dev, void* base) { (void)dev; free(base); --g_arenas_live; return 0; }
static int emu_mapped_alloc(int dev, size_t bytes, void** h, void** d) {
  (void)dev;
  if (posix_memalign(h, 4096, bytes)) return 2;
  memset(*h, 0, bytes);
  *d = *h;
  ++g_mapped_live;
  return 0;
}
static int emu_mapped_free(int dev, void* h) { (void)dev; free(h); --g_mapped_live; return 0; }
static int emu_device_alloc(int dev, size_t bytes, void** p) {
  (void)dev;
  *p = calloc(1, bytes);
  if (!*p) return 2;
  ++g_device_live;
  return 0;
}
static int emu_device_free(int dev, void* p) { (void)dev; free(p); --g_device_live; return 0; }
static int emu_copy_to_device(int dev, void* dst, const void* src, size_t bytes) { (void)dev; memcpy(dst, src, bytes); return 0; }
static int emu_engine_create(int dev, const tcpxuEngineConfig* cfg, tcpxuEngine** e) { (void)dev; (void)cfg; *e = &g_engine; return 0; }
static int emu_engine_start(tcpxuEngine* e) { e->started = 1; ++g_engine_starts; return 0; }
static int emu_engine_stop(tcpxuEngine* e, double* us) { e->started = 0; if (us) *us = 0; return 0; }
static int emu_engine_destroy(tcpxuEngine* e) { (void)e; return 0; }
static int emu_engine_submit(tcpxuEngine* e, const void* bounce, void* dst, const void* descs, uint32_t n, void* flag,
                             uint64_t value) {
  if (!e->started) return 5;
  if (g_ring_full) return TCPXU_IN_PROGRESS;
  ++g_submitted;
  if (in_visible(descs)) ++g_staged_submits;
  emu_job j = {bounce, dst, descs, n, (uint64_t*)flag, value};
  if (g_hold) {
    if (g_n_pending >= EMU_MAX_PENDING) return TCPXU_IN_PROGRESS;
    g_pending[g_n_pending++] = j;
  } else {
    run_job(&j);
  }
  return 0;
}
static int emu_engine_submit_sized(tcpxuEngine* e, const void* bounce, void* dst, const void* descs, uint32_t n,
                                   uint64_t payload_bytes, void* flag, uint64_t value) {
  g_last_payload_bytes = payload_bytes;
  return emu_engine_submit(e, bounce, dst, descs, n, flag, value);
}
static const char* emu_last_error(void) { return "emulated device"; }
static int emu_visible_alloc(int dev, size_t bytes, void** host_ptr, void** dev_ptr) {
  (void)dev;
  if (g_visible_off) return TCPXU_INVALID_USAGE;
  for (int i = 0; i < EMU_MAX_VISIBLE; ++i) {
    if (!g_visible[i].p) {
      g_visible[i].p = (uint8_t*)calloc(1, bytes);
      if (!g_visible[i].p) return TCPXU_SYSTEM_ERROR;
      g_visible[i].bytes = bytes;
      ++g_visible_live;
      *host_ptr = *dev_ptr = g_visible[i].p;
      return 0;
    }
  }
  return TCPXU_SYSTEM_ERROR;
}
static int emu_visible_free(int dev, void* host_ptr) {
  (void)dev;
  for (int i = 0; i < EMU_MAX_VISIBLE; ++i) {
    if (g_visible[i].p && g_visible[i].p == host_ptr) {
      free(g_visible[i].p);
      g_visible[i].p = NULL;
      --g_visible_live;
      return 0;
    }
  }
  return TCPXU_INVALID_ARGUMENT;
}
static void emu_visible_flush(void) { ++g_visible_flushes; }
static int in_visible(const void* p) {
  for (int i = 0; i < EMU_MAX_VISIBLE; ++i)
    if (g_visible[i].p && (const uint8_t*)p >= g_visible[i].p && (const uint8_t*)p < g_visible[i].p + g_visible[i].bytes) return 1;
  return 0;
}

static const tcpxDeviceOps g_ops = {
    emu_device_count, emu_arena_create,  emu_arena_destroy, emu_mapped_alloc,  emu_mapped_free,
    emu_device_alloc, emu_device_free,   emu_copy_to_device, emu_engine_create, emu_engine_start,
    emu_engine_stop,  emu_engine_destroy, emu_engine_submit, emu_last_error,
    emu_visible_alloc, emu_visible_free, emu_visible_flush, emu_engine_submit_sized,
};
const tcpxDeviceOps* emu_ops(void) { return &g_ops; }
