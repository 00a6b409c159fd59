// Measurement helpers of the unpack path (libtcpxu_bench.so, include/tcpx_unpack_bench.h): kernels of known
// traffic, event-timed launches, and a host loop that drives the persistent engine the way the plugin's proxy
// thread does.  A client of libtcpxu_hip.so: everything here goes through the entry points that
// include/tcpx_unpack_hip.h declares, and nothing in the product loads this library.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <chrono>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <vector>

#include "tcpx_unpack_bench.h"
#include "unpack_device.h"

namespace tcpxu_bench {
namespace {

using tcpxu::kVecPerLane;
using tcpxu::kWaveLanes;
using tcpxu::kWgThreads;
using tcpxu::load_vec_sys;
using tcpxu::store_vec_stream;
using tcpxu::u32x4;

thread_local char g_error[512] = "";
__attribute__((format(printf, 1, 2))) void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof g_error, fmt, ap);
  va_end(ap);
}

#define BENCH_HIP(call)                                                                   \
  do {                                                                                    \
    hipError_t e_ = (call);                                                               \
    if (e_ != hipSuccess) {                                                               \
      set_error("%s:%d %s -> %s", __FILE__, __LINE__, #call, hipGetErrorString(e_));      \
      return TCPXU_DEVICE_ERROR;                                                          \
    }                                                                                     \
  } while (0)
#define BENCH_TRY(call)                   \
  do {                                    \
    int rc_ = (call);                     \
    if (rc_ != TCPXU_SUCCESS) return rc_; \
  } while (0)

// Plain copy, 64 bytes per thread per step, with the payload accesses of the unpack kernels: the yardstick for
// what a copy kernel reaches here.
__global__ __launch_bounds__(kWgThreads) void copy_kernel(uint8_t* __restrict__ dst, const uint8_t* __restrict__ src,
                                                          uint64_t n_vec) {
  const uint64_t stride = static_cast<uint64_t>(gridDim.x) * kWgThreads;
  for (uint64_t base = static_cast<uint64_t>(blockIdx.x) * kWgThreads * kVecPerLane; base < n_vec;
       base += stride * kVecPerLane) {
    u32x4 r[kVecPerLane];
#pragma unroll
    for (int k = 0; k < kVecPerLane; ++k) {
      const uint64_t v = base + static_cast<uint64_t>(k) * kWgThreads + threadIdx.x;
      if (v < n_vec) r[k] = load_vec_sys(src + (v << 4));
    }
#pragma unroll
    for (int k = 0; k < kVecPerLane; ++k) {
      const uint64_t v = base + static_cast<uint64_t>(k) * kWgThreads + threadIdx.x;
      if (v < n_vec) store_vec_stream(dst + (v << 4), r[k]);
    }
  }
}

// The two halves of the copy on their own, with the same accesses: what the memory system gives to loads only and
// to stores only.  The loads are folded into one word per lane that is stored only if it has a value it
// practically never has, which keeps them from being optimised away without adding traffic.
__global__ __launch_bounds__(kWgThreads) void read_kernel(const uint8_t* __restrict__ src, uint64_t n_vec,
                                                          uint32_t* __restrict__ sink) {
  const uint64_t stride = static_cast<uint64_t>(gridDim.x) * kWgThreads;
  u32x4 acc = {0u, 0u, 0u, 0u};
  for (uint64_t base = static_cast<uint64_t>(blockIdx.x) * kWgThreads * kVecPerLane; base < n_vec;
       base += stride * kVecPerLane) {
#pragma unroll
    for (int k = 0; k < kVecPerLane; ++k) {
      const uint64_t v = base + static_cast<uint64_t>(k) * kWgThreads + threadIdx.x;
      if (v < n_vec) acc ^= load_vec_sys(src + (v << 4));
    }
  }
  if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x9E3779B9u && (acc[0] + acc[1]) == 0x7F4A7C15u) *sink = acc[2];
}

__global__ __launch_bounds__(kWgThreads) void fill_kernel(uint8_t* __restrict__ dst, uint64_t n_vec) {
  const uint64_t stride = static_cast<uint64_t>(gridDim.x) * kWgThreads;
  const u32x4 x = {threadIdx.x, blockIdx.x, 0xA5A5A5A5u, 0x5A5A5A5Au};
  for (uint64_t base = static_cast<uint64_t>(blockIdx.x) * kWgThreads * kVecPerLane; base < n_vec;
       base += stride * kVecPerLane) {
#pragma unroll
    for (int k = 0; k < kVecPerLane; ++k) {
      const uint64_t v = base + static_cast<uint64_t>(k) * kWgThreads + threadIdx.x;
      if (v < n_vec) store_vec_stream(dst + (v << 4), x);
    }
  }
}

// A bare gather of short fragments: the first `K` KiB of the 4 KiB page pages[i] of `src` go to dst + i * K KiB, one
// wavefront per fragment, one fragment in flight per wavefront, the unpack kernel's load and store instructions and
// its sixteen copy wavefronts per compute unit -- and nothing else: no descriptors, no alignment work, no shared
// lines.  What the memory system gives to a gather of fragments of that length.
template <int K>
__global__ __launch_bounds__(2 * kWgThreads) void gather_kernel(uint8_t* __restrict__ dst, const uint8_t* __restrict__ src,
                                                                const uint32_t* __restrict__ pages, uint32_t n) {
  constexpr uint32_t kWaves = 2 * kWgThreads / kWaveLanes;
  const uint32_t lane = threadIdx.x & (kWaveLanes - 1);
  const uint32_t wave = blockIdx.x * kWaves + threadIdx.x / kWaveLanes, n_waves = gridDim.x * kWaves;
  for (uint32_t i = wave; i < n; i += n_waves) {
    const uint8_t* from = src + (static_cast<uint64_t>(pages[i]) << 12);
    uint8_t* to = dst + static_cast<uint64_t>(i) * (K * 1024);
    u32x4 r[K];
#pragma unroll
    for (int k = 0; k < K; ++k) r[k] = load_vec_sys(from + ((k * kWaveLanes + lane) << 4));
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
    for (int k = 0; k < K; ++k) store_vec_stream(to + ((k * kWaveLanes + lane) << 4), r[k]);
  }
}

// Mean of per-launch durations: every launch sits between its own pair of events on the launch stream, so
// gaps between launches are not counted.
int time_launches(hipStream_t stream, int warmup, int iters, double* mean_us, int (*launch)(void*, hipStream_t),
                  void* ctx) {
  std::vector<hipEvent_t> ev(static_cast<size_t>(iters) * 2, nullptr);
  int rc = TCPXU_SUCCESS;
  for (int i = 0; i < warmup && rc == TCPXU_SUCCESS; ++i) rc = launch(ctx, stream);
  for (auto& e : ev) {
    if (rc == TCPXU_SUCCESS && hipEventCreate(&e) != hipSuccess) {
      set_error("hipEventCreate failed");
      rc = TCPXU_DEVICE_ERROR;
    }
  }
  if (rc == TCPXU_SUCCESS && hipStreamSynchronize(stream) != hipSuccess) rc = TCPXU_DEVICE_ERROR;
  for (int i = 0; i < iters && rc == TCPXU_SUCCESS; ++i) {
    if (hipEventRecord(ev[2 * i], stream) != hipSuccess) rc = TCPXU_DEVICE_ERROR;
    if (rc == TCPXU_SUCCESS) rc = launch(ctx, stream);
    if (rc == TCPXU_SUCCESS && hipEventRecord(ev[2 * i + 1], stream) != hipSuccess) rc = TCPXU_DEVICE_ERROR;
  }
  if (rc == TCPXU_SUCCESS) {
    hipError_t e = hipStreamSynchronize(stream);
    if (e != hipSuccess) {
      set_error("stream synchronize failed: %s", hipGetErrorString(e));
      rc = TCPXU_DEVICE_ERROR;
    }
  }
  if (rc == TCPXU_SUCCESS) {
    double total_ms = 0.0;
    for (int i = 0; i < iters; ++i) {
      float ms = 0.f;
      if (hipEventElapsedTime(&ms, ev[2 * i], ev[2 * i + 1]) != hipSuccess) rc = TCPXU_DEVICE_ERROR;
      total_ms += ms;
    }
    *mean_us = total_ms * 1000.0 / iters;
  }
  for (auto e : ev)
    if (e) (void)hipEventDestroy(e);
  return rc;
}

struct BatchLaunch {
  int device;
  const void* bounce;
  void* dst;
  const tcpxuLoadMeta* descs;
  uint64_t n;
};

struct CopyLaunch {
  uint8_t* dst;
  const uint8_t* src;
  uint64_t n_vec;
  uint32_t grid;
  uint32_t* sink;
};

int launch_copy(const CopyLaunch* c, hipStream_t s) {
  if (!c->dst) {
    hipLaunchKernelGGL(read_kernel, dim3(c->grid), dim3(kWgThreads), 0, s, c->src, c->n_vec, c->sink);
  } else if (!c->src) {
    hipLaunchKernelGGL(fill_kernel, dim3(c->grid), dim3(kWgThreads), 0, s, c->dst, c->n_vec);
  } else {
    hipLaunchKernelGGL(copy_kernel, dim3(c->grid), dim3(kWgThreads), 0, s, c->dst, c->src, c->n_vec);
  }
  if (hipGetLastError() != hipSuccess) {
    set_error("copy kernel launch failed");
    return TCPXU_DEVICE_ERROR;
  }
  return TCPXU_SUCCESS;
}

struct GatherLaunch {
  uint8_t* dst;
  const uint8_t* src;
  const uint32_t* pages;
  uint32_t n, kib, grid;
};

int launch_gather(const GatherLaunch* g, hipStream_t s) {
  const dim3 grid(g->grid), block(2 * kWgThreads);
  switch (g->kib) {
    case 1: hipLaunchKernelGGL(gather_kernel<1>, grid, block, 0, s, g->dst, g->src, g->pages, g->n); break;
    case 2: hipLaunchKernelGGL(gather_kernel<2>, grid, block, 0, s, g->dst, g->src, g->pages, g->n); break;
    case 3: hipLaunchKernelGGL(gather_kernel<3>, grid, block, 0, s, g->dst, g->src, g->pages, g->n); break;
    default: hipLaunchKernelGGL(gather_kernel<4>, grid, block, 0, s, g->dst, g->src, g->pages, g->n); break;
  }
  if (hipGetLastError() != hipSuccess) {
    set_error("gather kernel launch failed");
    return TCPXU_DEVICE_ERROR;
  }
  return TCPXU_SUCCESS;
}

int copy_geometry(int device, void* dst, const void* src, size_t bytes, CopyLaunch* c) {
  if ((!dst && !src) || bytes == 0 || bytes % 16 != 0 || reinterpret_cast<uintptr_t>(dst) % 16 != 0 ||
      reinterpret_cast<uintptr_t>(src) % 16 != 0) {
    set_error("copy kernel needs 16-byte aligned buffers (at least one of them) and a size that is a multiple of 16");
    return TCPXU_INVALID_ARGUMENT;
  }
  int cus = 0;
  BENCH_TRY(tcpxuDeviceInfo(device, nullptr, 0, &cus));  // also makes the device current
  const uint64_t n_vec = bytes / 16;
  const uint64_t per_wg = static_cast<uint64_t>(kWgThreads) * kVecPerLane;
  const uint32_t grid = static_cast<uint32_t>(
      std::min<uint64_t>((n_vec + per_wg - 1) / per_wg, static_cast<uint64_t>(std::max(cus, 1)) * 16));
  *c = CopyLaunch{static_cast<uint8_t*>(dst), static_cast<const uint8_t*>(src), n_vec, grid, nullptr};
  return TCPXU_SUCCESS;
}

// ---- streaming driver ----------------------------------------------------------------------------------------------
// Mapped memory of the driver, one block per device, allocated on first use and kept for the life of the process
// (freeing mapped memory waits for every stream of the device, the engine's included).
//
// A ring of 2 x depth descriptor slots serves `depth` slots in flight: while a slot's occupant is being unpacked,
// the descriptors of the item that will follow it are already written into the slot's twin, so that a completion
// is answered with a publish at once and the copy of up to 32 KiB of descriptors is not part of a slot's
// turn-around.  This is where the plugin has them as well: it builds a request's descriptors while its fragments
// arrive (src/sock/tcpx.h:178-199 into the task's scatter list), long before tcpxTest publishes the count.
//
// Up to TCPXU_STREAM_FULL_SLOT_DEPTH slots in flight each slot holds a whole unpack-queue slot (2048 descriptors);
// beyond that, up to TCPXU_STREAM_MAX_DEPTH, every item must be small (at most kSmallSlotDescs descriptors: the
// storm of 64 KiB requests) and the slots are that size.
constexpr size_t kFlagStride = 64;
constexpr size_t kSlotBytes = sizeof(tcpxuLoadMeta) * TCPXU_SLOT_PAGES;
constexpr uint32_t kSmallSlotDescs = 64;
constexpr size_t kSmallSlotBytes = sizeof(tcpxuLoadMeta) * kSmallSlotDescs;
constexpr uint32_t kPhysSlots = 2 * TCPXU_STREAM_MAX_DEPTH;
constexpr size_t kFlagsBytes = kFlagStride * kPhysSlots;
constexpr size_t kSlotsBytes = std::max(kSlotBytes * 2 * TCPXU_STREAM_FULL_SLOT_DEPTH, kSmallSlotBytes* kPhysSlots);
// Descriptors of a small item that are also copied into host-visible device memory, and the room per slot.
constexpr uint32_t kStageDescs = 16;
constexpr size_t kStageBytes = kStageDescs * sizeof(tcpxuLoadMeta);
constexpr uint32_t kStageMaxDepth = 384;  // slots in flight up to which that is done (see stream_items)
constexpr uint32_t kPublishBatch = 64;  // submissions handed to the engine under one lock

struct Driver {
  void* host = nullptr;
  void* dev = nullptr;
  void* stage_host = nullptr;  // device memory the host can write, or null
  void* stage_dev = nullptr;
  bool stage_tried = false;
};
Driver g_driver[64];
std::mutex g_driver_mu;  // one stream at a time
tcpxuStreamSplit g_last_split = {};

int driver_for(int device, Driver** out) {
  if (device < 0 || device >= 64) return TCPXU_INVALID_ARGUMENT;
  Driver* d = &g_driver[device];
  if (!d->host) BENCH_TRY(tcpxuMappedAlloc(device, kFlagsBytes + kSlotsBytes, &d->host, &d->dev));
  if (!d->stage_tried) {
    // Optional: without it every item's descriptors are read from the mapped slot.
    d->stage_tried = true;
    if (tcpxuVisibleAlloc(device, kStageBytes * 2 * kStageMaxDepth, &d->stage_host, &d->stage_dev) != TCPXU_SUCCESS)
      d->stage_host = d->stage_dev = nullptr;
  }
  *out = d;
  return TCPXU_SUCCESS;
}

// The streaming loop.  pub_us[i] / done_us[i]: when item i was published / seen completed, in microseconds since
// the first publish.  One pass of the loop reaps what has completed, publishes up to `depth` in flight -- the
// items of a pass go to the engine together (tcpxuEngineSubmitMany), as a poller that finds several requests
// complete submits them -- and stages descriptors ahead.  The clock is read per pass, not per item (a read costs
// 20 ns, a third of what a storm of small requests leaves the host per request): an item's publish stamp is taken
// just before its batch is submitted and its completion stamp just after the reap that found it, so a latency is
// never understated.
int stream_items(tcpxuEngine* e, const tcpxuStreamItem* items, uint64_t n_items, uint32_t depth,
                 uint32_t stall_timeout_ms, double* pub_us, double* done_us) {
  if (!e || !items || depth == 0 || depth > TCPXU_STREAM_MAX_DEPTH) {
    set_error("stream needs an engine, items and 1..%d slots in flight", TCPXU_STREAM_MAX_DEPTH);
    return TCPXU_INVALID_ARGUMENT;
  }
  const bool small_slots = depth > TCPXU_STREAM_FULL_SLOT_DEPTH;
  const uint32_t slot_descs = small_slots ? kSmallSlotDescs : static_cast<uint32_t>(TCPXU_SLOT_PAGES);
  const size_t slot_bytes = small_slots ? kSmallSlotBytes : kSlotBytes;
  for (uint64_t i = 0; i < n_items; ++i) {
    if (items[i].n_descs > slot_descs) {
      set_error("stream item %llu has %u descriptors, a slot holds %u with %u in flight",
                static_cast<unsigned long long>(i), items[i].n_descs, slot_descs, depth);
      return TCPXU_INVALID_ARGUMENT;
    }
  }
  if (stall_timeout_ms == 0) stall_timeout_ms = 10000;
  int device = 0;
  BENCH_TRY(tcpxuEngineDevice(e, &device));
  Driver* d = nullptr;
  BENCH_TRY(driver_for(device, &d));
  uint8_t* hb = static_cast<uint8_t*>(d->host);
  uint8_t* db = static_cast<uint8_t*>(d->dev);
  memset(hb, 0, kFlagsBytes);
  const uint32_t phys = 2 * depth;
  const bool small_to_device = d->stage_host != nullptr && depth <= kStageMaxDepth;
  using clock = std::chrono::steady_clock;
  auto us_since = [](clock::time_point a, clock::time_point b) {
    return std::chrono::duration<double, std::micro>(b - a).count();
  };
  std::vector<const void*> descs_dev(phys, nullptr);
  int rc = TCPXU_SUCCESS;
  uint64_t next_stage = 0, next_submit = 0, next_done = 0;
  tcpxuStreamSplit split = {};
  // Writes item i's descriptors where the GPU will read them.  The twin slot i % phys is free once item i - phys
  // has completed.
  bool staged_unflushed = false;  // descriptors written through the BAR since the last flush
  auto stage = [&](uint64_t i) {
    const uint32_t slot = static_cast<uint32_t>(i % phys);
    const tcpxuStreamItem& it = items[i];
    if (it.n_descs) memcpy(hb + kFlagsBytes + slot_bytes * slot, it.descs_host, sizeof(tcpxuLoadMeta) * it.n_descs);
    descs_dev[slot] = db + kFlagsBytes + slot_bytes * slot;
    if (small_to_device && it.n_descs != 0 && it.n_descs <= kStageDescs) {
      // A small request: its descriptors also go into the GPU's own memory, ahead of the submission, as the plugin
      // does for the requests of a comm's sixteen slots, so that the workgroup that takes the request need not fetch
      // them over PCIe (0.9 us of each request's way: 128 requests of 64 KiB in flight 12.4 -> 14.4 M/s, 384 in
      // flight 27.0 -> 30.8).  The write goes through the BAR and is flushed once per batch of submissions.  (Not
      // beyond kStageMaxDepth in flight: the requests then wait in queues anyway, the copy is the bound, and the
      // writes through the BAR only cost the host: 1024 in flight 44.6 -> 41.7-44.0 M/s.)
      memcpy(static_cast<uint8_t*>(d->stage_host) + kStageBytes * slot, it.descs_host, sizeof(tcpxuLoadMeta) * it.n_descs);
      staged_unflushed = true;
      descs_dev[slot] = static_cast<uint8_t*>(d->stage_dev) + kStageBytes * slot;
    }
  };
  tcpxuSubmission batch[kPublishBatch];
  const auto t0 = clock::now();
  auto last_progress = t0;
  auto now = t0;
  while (next_done < n_items) {
    bool progress = false;
    // Reap completions in FIFO order.  The completion words are lines that the GPU has just written, i.e. misses:
    // the ones further on are asked for early.
    const uint64_t done_before = next_done;
    while (next_done < next_submit) {
      const uint32_t slot = static_cast<uint32_t>(next_done % phys);
      __builtin_prefetch(hb + kFlagStride * ((slot + 4) % phys));
      auto* flag = reinterpret_cast<std::atomic<uint64_t>*>(hb + kFlagStride * slot);
      if (flag->load(std::memory_order_acquire) != next_done + 1) break;
      ++next_done;
    }
    if (next_done != done_before) {
      now = clock::now();
      const double at = us_since(t0, now);
      for (uint64_t i = done_before; i < next_done; ++i) done_us[i] = at;
      progress = true;
    }
    // Publish while fewer than `depth` are in flight.
    while (next_submit < n_items && next_submit - next_done < depth) {
      const uint64_t want = std::min<uint64_t>(std::min<uint64_t>(n_items, next_done + depth) - next_submit, kPublishBatch);
      const auto before = next_submit == 0 ? t0 : clock::now();
      for (uint64_t k = 0; k < want; ++k) {
        const uint64_t i = next_submit + k;
        if (next_stage == i) stage(next_stage++);
        const uint32_t slot = static_cast<uint32_t>(i % phys);
        const tcpxuStreamItem& it = items[i];
        batch[k] = tcpxuSubmission{it.bounce_base, it.dst_base, descs_dev[slot], db + kFlagStride * slot, i + 1, it.n_descs, it.payload_bytes};
      }
      // What went through the BAR must have left this CPU before the submissions that point at it are published:
      // once per batch.
      if (staged_unflushed) {
        tcpxuVisibleFlush();
        staged_unflushed = false;
      }
      uint32_t accepted = 0;
      rc = tcpxuEngineSubmitMany(e, batch, static_cast<uint32_t>(want), &accepted);
      now = clock::now();
      const double at = us_since(t0, before);
      for (uint64_t k = 0; k < accepted; ++k) pub_us[next_submit + k] = at;
      next_submit += accepted;
      split.publish_ns += 1e3 * us_since(before, now);
      split.published += accepted;
      split.publish_calls += 1;
      if (accepted != 0) progress = true;
      if (rc == TCPXU_IN_PROGRESS) {
        rc = TCPXU_SUCCESS;
        break;  // engine ring full: reap first
      }
      if (rc != TCPXU_SUCCESS) {
        set_error("submit of item %llu failed: %s", static_cast<unsigned long long>(next_submit), tcpxuLastError());
        break;
      }
    }
    if (rc != TCPXU_SUCCESS) break;
    // Descriptors ahead: one item per pass with few in flight, so that completions are still seen promptly; with
    // many, as many as the last reap made room for.
    for (uint32_t k = 0, most = depth <= 16 ? 1 : 16; k < most && next_stage < n_items && next_stage < next_done + phys; ++k) {
      stage(next_stage++);
      progress = true;
    }
    split.passes += 1;
    if (progress) {
      last_progress = now;
    } else if ((split.passes & 1023) == 0) {
      now = clock::now();
      if (now - last_progress > std::chrono::milliseconds(stall_timeout_ms)) {
        set_error("stream stalled: %llu of %llu items completed, %llu published",
                  static_cast<unsigned long long>(next_done), static_cast<unsigned long long>(n_items),
                  static_cast<unsigned long long>(next_submit));
        rc = TCPXU_INTERNAL_ERROR;
        break;
      }
    }
  }
  split.wall_ns = 1e3 * us_since(t0, clock::now());
  g_last_split = split;
  return rc;
}

struct Stamps {
  std::vector<double> pub, done;
  explicit Stamps(uint64_t n) : pub(n, 0.0), done(n, 0.0) {}
  void latencies(double* out) const {
    if (out)
      for (size_t i = 0; i < pub.size(); ++i) out[i] = done[i] - pub[i];
  }
};

// Start, stream, stop: the launch covers exactly these items.
int run_launch(tcpxuEngine* e, const tcpxuStreamItem* items, uint64_t n_items, uint32_t depth,
               uint32_t stall_timeout_ms, double* kernel_us, Stamps* st) {
  if (!e || !kernel_us) return TCPXU_INVALID_ARGUMENT;
  if (depth == 0 || depth > TCPXU_STREAM_MAX_DEPTH) {
    set_error("stream needs 1..%d slots in flight", TCPXU_STREAM_MAX_DEPTH);
    return TCPXU_INVALID_ARGUMENT;
  }
  // Touch the driver's memory before the launch so that no allocation happens while the kernel is timed.
  int device = 0;
  BENCH_TRY(tcpxuEngineDevice(e, &device));
  Driver* d = nullptr;
  BENCH_TRY(driver_for(device, &d));
  BENCH_TRY(tcpxuEngineStart(e));
  const int rc = stream_items(e, items, n_items, depth, stall_timeout_ms, st->pub.data(), st->done.data());
  const int rc_stop = tcpxuEngineStop(e, kernel_us);
  if (rc == TCPXU_SUCCESS && rc_stop != TCPXU_SUCCESS) set_error("engine stop failed: %s", tcpxuLastError());
  return rc != TCPXU_SUCCESS ? rc : rc_stop;
}

}  // namespace
}  // namespace tcpxu_bench

using namespace tcpxu_bench;

extern "C" {

const char* tcpxuBenchLastError(void) { return g_error; }

int tcpxuUnpackBatchTimed(int device, const void* bounce_base, void* dst_base, const tcpxuLoadMeta* descs,
                          uint64_t n_descs, int warmup, int iters, double* mean_us) {
  if (!mean_us || iters <= 0 || warmup < 0 || n_descs == 0) return TCPXU_INVALID_ARGUMENT;
  BENCH_TRY(tcpxuDeviceInfo(device, nullptr, 0, nullptr));  // makes the device current
  hipStream_t stream;
  BENCH_HIP(hipStreamCreate(&stream));
  BatchLaunch b{device, bounce_base, dst_base, descs, n_descs};
  int rc = time_launches(
      stream, warmup, iters, mean_us,
      [](void* c, hipStream_t s) {
        auto* b = static_cast<BatchLaunch*>(c);
        const int r = tcpxuUnpackBatch(b->device, b->bounce, b->dst, b->descs, b->n, s);
        if (r != TCPXU_SUCCESS) set_error("tcpxuUnpackBatch: %s", tcpxuLastError());
        return r;
      },
      &b);
  (void)hipStreamDestroy(stream);
  return rc;
}

int tcpxuCopyKernelTimed(int device, void* dst, const void* src, size_t bytes, int warmup, int iters,
                         double* mean_us) {
  if (!mean_us || iters <= 0 || warmup < 0) return TCPXU_INVALID_ARGUMENT;
  CopyLaunch c;
  BENCH_TRY(copy_geometry(device, dst, src, bytes, &c));
  if (!dst) BENCH_HIP(hipMalloc(reinterpret_cast<void**>(&c.sink), 64));
  hipStream_t stream;
  if (hipStreamCreate(&stream) != hipSuccess) {
    (void)hipFree(c.sink);
    set_error("hipStreamCreate failed");
    return TCPXU_DEVICE_ERROR;
  }
  int rc = time_launches(
      stream, warmup, iters, mean_us, [](void* p, hipStream_t s) { return launch_copy(static_cast<CopyLaunch*>(p), s); },
      &c);
  (void)hipStreamDestroy(stream);
  (void)hipFree(c.sink);
  return rc;
}

int tcpxuGatherKernelTimed(int device, void* dst, const void* src, const uint32_t* pages_dev, uint32_t n_fragments,
                           uint32_t fragment_bytes, int warmup, int iters, double* mean_us) {
  if (!mean_us || iters <= 0 || warmup < 0 || !dst || !src || !pages_dev || n_fragments == 0 || fragment_bytes == 0 ||
      fragment_bytes > TCPXU_PAGE_SIZE || fragment_bytes % 1024 != 0 || reinterpret_cast<uintptr_t>(dst) % 16 != 0 ||
      reinterpret_cast<uintptr_t>(src) % 16 != 0) {
    set_error("gather kernel needs 16-byte aligned buffers, a page list and fragments of 1, 2, 3 or 4 KiB");
    return TCPXU_INVALID_ARGUMENT;
  }
  int cus = 0;
  BENCH_TRY(tcpxuDeviceInfo(device, nullptr, 0, &cus));  // also makes the device current
  GatherLaunch g{static_cast<uint8_t*>(dst), static_cast<const uint8_t*>(src), pages_dev, n_fragments, fragment_bytes / 1024,
                 static_cast<uint32_t>(std::max(cus, 1)) * 2};
  hipStream_t stream;
  if (hipStreamCreate(&stream) != hipSuccess) {
    set_error("hipStreamCreate failed");
    return TCPXU_DEVICE_ERROR;
  }
  int rc = time_launches(
      stream, warmup, iters, mean_us, [](void* p, hipStream_t s) { return launch_gather(static_cast<GatherLaunch*>(p), s); }, &g);
  (void)hipStreamDestroy(stream);
  return rc;
}

int tcpxuCopyKernelLaunch(int device, void* dst, const void* src, size_t bytes, void* stream) {
  if (!dst || !src) {
    set_error("a copy needs a source and a destination");
    return TCPXU_INVALID_ARGUMENT;
  }
  CopyLaunch c;
  BENCH_TRY(copy_geometry(device, dst, src, bytes, &c));
  return launch_copy(&c, static_cast<hipStream_t>(stream));
}

int tcpxuStreamLastSplit(tcpxuStreamSplit* split) {
  if (!split) return TCPXU_INVALID_ARGUMENT;
  std::lock_guard<std::mutex> lock(g_driver_mu);
  *split = g_last_split;
  return TCPXU_SUCCESS;
}

int tcpxuEngineStreamWarm(tcpxuEngine* e, const tcpxuStreamItem* items, uint64_t n_items, uint64_t warmup_items,
                          uint32_t depth, uint32_t stall_timeout_ms, double* wall_us, double* latency_us) {
  if (!wall_us || warmup_items > n_items) return TCPXU_INVALID_ARGUMENT;
  std::lock_guard<std::mutex> lock(g_driver_mu);
  Stamps st(n_items);
  const int rc = stream_items(e, items, n_items, depth, stall_timeout_ms, st.pub.data(), st.done.data());
  *wall_us = n_items > warmup_items ? st.done[n_items - 1] - st.pub[warmup_items] : 0.0;
  st.latencies(latency_us);
  return rc;
}

int tcpxuEngineStream(tcpxuEngine* e, const tcpxuStreamItem* items, uint64_t n_items, uint32_t depth,
                      uint32_t stall_timeout_ms, double* wall_us, double* latency_us) {
  return tcpxuEngineStreamWarm(e, items, n_items, 0, depth, stall_timeout_ms, wall_us, latency_us);
}

int tcpxuEngineRunTimed(tcpxuEngine* e, const tcpxuStreamItem* items, uint64_t n_items, uint64_t warmup_items,
                        uint32_t depth, uint32_t stall_timeout_ms, double* wall_us, double* kernel_us,
                        double* latency_us) {
  if (!wall_us || warmup_items > n_items) return TCPXU_INVALID_ARGUMENT;
  std::lock_guard<std::mutex> lock(g_driver_mu);
  Stamps st(n_items);
  const int rc = run_launch(e, items, n_items, depth, stall_timeout_ms, kernel_us, &st);
  *wall_us = n_items > warmup_items ? st.done[n_items - 1] - st.pub[warmup_items] : 0.0;
  st.latencies(latency_us);
  return rc;
}

int tcpxuEngineRunWindow(tcpxuEngine* e, const tcpxuStreamItem* items, uint64_t n_items, uint64_t first_timed,
                         uint64_t n_timed, uint32_t depth, uint32_t stall_timeout_ms, double* wall_us,
                         double* kernel_us, double* latency_us) {
  if (!wall_us || n_timed == 0 || first_timed > n_items || n_timed > n_items - first_timed)
    return TCPXU_INVALID_ARGUMENT;
  std::lock_guard<std::mutex> lock(g_driver_mu);
  Stamps st(n_items);
  const int rc = run_launch(e, items, n_items, depth, stall_timeout_ms, kernel_us, &st);
  *wall_us = st.done[first_timed + n_timed - 1] - (first_timed ? st.done[first_timed - 1] : 0.0);
  st.latencies(latency_us);
  return rc;
}

int tcpxuEngineRunStamped(tcpxuEngine* e, const tcpxuStreamItem* items, uint64_t n_items, uint32_t depth,
                          uint32_t stall_timeout_ms, double* kernel_us, double* done_us, double* latency_us) {
  if (!done_us) return TCPXU_INVALID_ARGUMENT;
  std::lock_guard<std::mutex> lock(g_driver_mu);
  Stamps st(n_items);
  const int rc = run_launch(e, items, n_items, depth, stall_timeout_ms, kernel_us, &st);
  for (uint64_t i = 0; i < n_items; ++i) done_us[i] = st.done[i];
  st.latencies(latency_us);
  return rc;
}

}  // extern "C"
