// Persistent unpack engine: one long-running gfx950 kernel per GPU that turns slots published in mapped host
// memory into scatter-gather copies and reports completion into mapped host memory -- no launch per request.
//
// Roles inside the one kernel launch
//   workgroup 0, wavefront 0  "leader": polls the submission ring over PCIe, cuts each submission into tickets of
//                             `descs_per_ticket` consecutive descriptors and publishes them in a device-memory
//                             ticket ring.  It never copies payload.
//   every other workgroup     "worker": claims the next ticket with one atomic, stages the ticket's descriptors
//                             from the mapped slot into LDS, lets its four wavefronts copy fragments, then
//                             retires the ticket.  Whoever retires the last ticket of a submission writes the
//                             completion word that the host poller reads.
//
// Host <-> GPU ordering (fine-grained mapped memory)
//   host:   descriptors, then the 64-byte submission entry (payload words, release, stamps), then tail
//   leader: system-scope loads of the entry; every 16-byte sector carries its own stamp, so a sector whose stamp
//           matches holds current payload even if the 64 bytes arrive as several PCIe reads
//   worker: system-scope loads of descriptors; payload stores; each wavefront waits for its own stores; one
//           system-scope release per ticket; the last ticket's owner release-stores the completion word
//
// Liveness: no workgroup ever waits for another worker.  Workers wait only for the leader (ticket publication)
// and check the stop word on every poll; the leader waits only for workers to retire tickets, which they do
// without waiting.  The host stop word, or the optional spin limit, ends the leader; the leader's device stop
// word ends every worker once the published tickets are claimed.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <chrono>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <new>
#include <thread>
#include <vector>

#include "hip_common.h"
#include "tcpx_unpack_hip.h"
#include "unpack_device.h"

namespace tcpxu {
namespace {

constexpr uint32_t kTicketRing = 1u << 16;       // tickets in flight at most
constexpr uint32_t kMaxDescsPerTicket = 64;
constexpr uint32_t kMaxDescsPerSubmission = 1u << 20;
constexpr int kTcpxuInProgress = 7;               // ncclInProgress: "try again"

// 64-byte submission entry: four 16-byte sectors of three payload words and one stamp word.
struct alignas(64) SubEntry {
  uint32_t w[16];
};
constexpr int kPayloadWords = 12;
__host__ __device__ constexpr int payload_slot(int i) { return (i / 3) * 4 + (i % 3); }

struct HostCtl {  // mapped host memory
  alignas(64) uint64_t tail;       // host -> GPU: submissions published so far
  alignas(64) uint64_t stop;       // host -> GPU: drain and exit
  alignas(64) uint64_t head;       // GPU -> host: submissions the leader has consumed
  alignas(64) uint64_t completed;  // GPU -> host: submissions fully unpacked (mirrored lazily)
  alignas(64) uint64_t exited;     // GPU -> host: 0 running, 1 stopped on request, 2 spin limit reached
  alignas(64) SubEntry ring[1];    // ring_entries follow
};

struct alignas(32) Ticket {
  uint64_t descs;   // device-visible address of the first descriptor of this ticket
  uint64_t bounce;
  uint64_t dst;
  uint32_t n;       // descriptors in this ticket
  uint32_t job;     // index into the job table
};

struct alignas(32) Job {
  uint64_t done_flag;
  uint64_t done_value;
  uint32_t remaining;  // tickets not yet retired; 0 = slot free
  uint32_t n_tickets;
  uint64_t pad;
};

struct DevState {  // device memory
  alignas(64) uint64_t ticket_head;     // next ticket to claim
  alignas(64) uint64_t ticket_tail;     // tickets published
  alignas(64) uint64_t retired;         // tickets of completed submissions
  alignas(64) uint32_t stop;            // 0 run, 1 host asked, 2 spin limit
  uint32_t exited_wgs;
  // Everything above is reset at every start; everything below survives restarts.
  alignas(64) uint64_t sub_head;        // next submission index
  alignas(64) uint64_t jobs_completed;  // submissions completed since creation
  alignas(64) Ticket tickets[kTicketRing];
  // Job jobs[ring_entries] follow
};

// ---- scoped memory operations -------------------------------------------------------------------------------------
#define SYS __HIP_MEMORY_SCOPE_SYSTEM
#define AGENT __HIP_MEMORY_SCOPE_AGENT

template <typename T>
__device__ __forceinline__ T sys_load(const T* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, SYS);
}
template <typename T>
__device__ __forceinline__ void sys_store(T* p, T v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, SYS);
}
template <typename T>
__device__ __forceinline__ T agent_load(const T* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, AGENT);
}

__device__ __forceinline__ uint32_t bcast(uint32_t v, int src_lane) { return __shfl(v, src_lane, kWaveLanes); }

__device__ __forceinline__ uint64_t payload64(uint32_t word, int i) {
  const uint32_t lo = bcast(word, payload_slot(i));
  const uint32_t hi = bcast(word, payload_slot(i + 1));
  return (static_cast<uint64_t>(hi) << 32) | lo;
}

// ---- leader -------------------------------------------------------------------------------------------------------
// Runs on wavefront 0 of workgroup 0.  All control flow is wave-uniform.
__device__ void leader_loop(HostCtl* ctl, DevState* st, Job* jobs, uint32_t ring_mask, uint32_t per_ticket,
                            uint32_t spin_limit) {
  const uint32_t lane = threadIdx.x;
  uint64_t s = agent_load(&st->sub_head);
  uint64_t tickets_out = agent_load(&st->ticket_tail);
  uint64_t mirrored = ~0ull;
  uint64_t idle = 0;
  uint32_t reason = 0;

  for (;;) {
    // One 64-byte read of entry s; lane 16 fetches the stop word in the same round trip.
    const SubEntry* e = &ctl->ring[s & ring_mask];
    uint32_t word = 0;
    if (lane < 16) word = sys_load(&e->w[lane]);
    uint64_t aux = 0;
    if (lane == 16) aux = sys_load(&ctl->stop);
    const uint32_t expect = static_cast<uint32_t>(s + 1);
    const bool stamp_ok = (lane < 16 && (lane & 3) == 3) ? (word == expect) : true;
    if (__all(stamp_ok)) {
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "");
      const uint64_t bounce = payload64(word, 0);
      const uint64_t dst = payload64(word, 2);
      const uint64_t descs = payload64(word, 4);
      const uint64_t done_flag = payload64(word, 6);
      const uint64_t done_value = payload64(word, 8);
      const uint32_t n = bcast(word, payload_slot(10));
      if (n == 0) {
        if (lane == 0) {
          __hip_atomic_store(reinterpret_cast<uint64_t*>(done_flag), done_value, __ATOMIC_RELEASE, SYS);
          __hip_atomic_fetch_add(&st->jobs_completed, 1ull, __ATOMIC_RELAXED, AGENT);
        }
      } else {
        const uint32_t nt = (n + per_ticket - 1) / per_ticket;
        const uint32_t slot = static_cast<uint32_t>(s) & ring_mask;
        // Both waits depend only on workers retiring tickets they already hold.
        while (__hip_atomic_load(&jobs[slot].remaining, __ATOMIC_ACQUIRE, AGENT) != 0) __builtin_amdgcn_s_sleep(2);
        while (tickets_out + nt - __hip_atomic_load(&st->retired, __ATOMIC_ACQUIRE, AGENT) > kTicketRing)
          __builtin_amdgcn_s_sleep(2);
        if (lane == 0) {
          jobs[slot].done_flag = done_flag;
          jobs[slot].done_value = done_value;
          jobs[slot].n_tickets = nt;
          __hip_atomic_store(&jobs[slot].remaining, nt, __ATOMIC_RELAXED, AGENT);
        }
        for (uint32_t i = lane; i < nt; i += kWaveLanes) {
          Ticket t;
          t.descs = descs + static_cast<uint64_t>(i) * per_ticket * sizeof(tcpxuLoadMeta);
          t.bounce = bounce;
          t.dst = dst;
          t.n = std::min(per_ticket, n - i * per_ticket);
          t.job = slot;
          st->tickets[(tickets_out + i) & (kTicketRing - 1)] = t;
        }
        tickets_out += nt;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
        if (lane == 0) __hip_atomic_store(&st->ticket_tail, tickets_out, __ATOMIC_RELEASE, AGENT);
      }
      ++s;
      idle = 0;
      if (lane == 0) sys_store(&ctl->head, s);
      continue;
    }

    // Nothing new at entry s.
    const uint64_t stop = (static_cast<uint64_t>(bcast(static_cast<uint32_t>(aux >> 32), 16)) << 32) |
                          bcast(static_cast<uint32_t>(aux), 16);
    if (stop != 0) {
      // The host wrote its last tail before the stop word: read the tail again, after the stop word.
      uint64_t tail_now = 0;
      if (lane == 0) tail_now = sys_load(&ctl->tail);
      const uint64_t tail = (static_cast<uint64_t>(bcast(static_cast<uint32_t>(tail_now >> 32), 0)) << 32) |
                            bcast(static_cast<uint32_t>(tail_now), 0);
      if (s >= tail) {
        reason = 1;
        break;
      }
      continue;  // entries up to tail are (or are about to become) visible: keep draining
    }
    if (lane == 0) {
      const uint64_t c = agent_load(&st->jobs_completed);
      if (c != mirrored) {
        sys_store(&ctl->completed, c);
        mirrored = c;
      }
    }
    if (spin_limit != 0 && ++idle > spin_limit) {
      reason = 2;
      break;
    }
    __builtin_amdgcn_s_sleep(1);
  }

  if (lane == 0) {
    __hip_atomic_store(&st->sub_head, s, __ATOMIC_RELAXED, AGENT);
    // Publish the stop word after the last ticket_tail: a worker that sees it re-reads the tail.
    __hip_atomic_store(&st->stop, reason, __ATOMIC_RELEASE, AGENT);
  }
}

// ---- worker -------------------------------------------------------------------------------------------------------
__device__ void worker_loop(DevState* st, Job* jobs) {
  __shared__ Ticket s_ticket;
  __shared__ tcpxuLoadMeta s_desc[kMaxDescsPerTicket];
  __shared__ uint32_t s_go;

  const uint32_t tid = threadIdx.x;
  const uint32_t lane = tid & (kWaveLanes - 1);
  const uint32_t wave = tid / kWaveLanes;
  uint64_t my_ticket = 0;  // meaningful in thread 0 only
  if (tid == 0) my_ticket = __hip_atomic_fetch_add(&st->ticket_head, 1ull, __ATOMIC_RELAXED, AGENT);

  for (;;) {
    if (tid == 0) {
      uint32_t go = 0;
      for (;;) {
        if (__hip_atomic_load(&st->ticket_tail, __ATOMIC_ACQUIRE, AGENT) > my_ticket) {
          go = 1;
          break;
        }
        if (__hip_atomic_load(&st->stop, __ATOMIC_ACQUIRE, AGENT) != 0) {
          go = __hip_atomic_load(&st->ticket_tail, __ATOMIC_ACQUIRE, AGENT) > my_ticket ? 1u : 0u;
          break;
        }
        __builtin_amdgcn_s_sleep(1);
      }
      if (go) s_ticket = st->tickets[my_ticket & (kTicketRing - 1)];
      s_go = go;
    }
    __syncthreads();
    if (s_go == 0) break;  // workgroup-uniform
    const Ticket tk = s_ticket;
    if (tid < tk.n) {
      // 16-byte descriptor as two system-scope 8-byte loads straight from the mapped slot.
      const uint64_t* p = reinterpret_cast<const uint64_t*>(tk.descs) + 2 * tid;
      const uint64_t lo = sys_load(p);
      const uint64_t hi = sys_load(p + 1);
      s_desc[tid].src_off = static_cast<uint32_t>(lo);
      s_desc[tid].len = static_cast<uint32_t>(lo >> 32);
      s_desc[tid].dst_off = hi;
    }
    // Claim the next ticket now: the atomic's round trip overlaps this ticket's copy.
    uint64_t next_ticket = 0;
    if (tid == 0) next_ticket = __hip_atomic_fetch_add(&st->ticket_head, 1ull, __ATOMIC_RELAXED, AGENT);
    __syncthreads();

    const uint8_t* bounce = reinterpret_cast<const uint8_t*>(tk.bounce);
    uint8_t* dst = reinterpret_cast<uint8_t*>(tk.dst);
    for (uint32_t j = wave; j < tk.n; j += kWavesPerWg) {
      const tcpxuLoadMeta d = s_desc[j];
      const uint32_t len = __builtin_amdgcn_readfirstlane(d.len);
      const uint32_t so = __builtin_amdgcn_readfirstlane(d.src_off);
      const uint32_t dlo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(d.dst_off));
      const uint32_t dhi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(d.dst_off >> 32));
      wave_copy_fragment(bounce + so, dst + ((static_cast<uint64_t>(dhi) << 32) | dlo), len, lane);
    }
    // Each wavefront waits until its own payload stores have been acknowledged; only then may thread 0 release.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();

    if (tid == 0) {
      Job* job = &jobs[tk.job];
      const uint64_t done_flag = job->done_flag;
      const uint64_t done_value = job->done_value;
      const uint32_t n_tickets = job->n_tickets;
      // System-scope release: this workgroup's payload leaves its XCD's L2 before the count drops.
      const uint32_t before = __hip_atomic_fetch_sub(&job->remaining, 1u, __ATOMIC_RELEASE, SYS);
      if (before == 1) {
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
        __hip_atomic_store(reinterpret_cast<uint64_t*>(done_flag), done_value, __ATOMIC_RELEASE, SYS);
        __hip_atomic_fetch_add(&st->retired, static_cast<uint64_t>(n_tickets), __ATOMIC_RELEASE, AGENT);
        __hip_atomic_fetch_add(&st->jobs_completed, 1ull, __ATOMIC_RELAXED, AGENT);
      }
      my_ticket = next_ticket;
    }
  }
}

__global__ __launch_bounds__(kWgThreads) void unpack_engine_kernel(HostCtl* ctl, DevState* st, Job* jobs,
                                                                   uint32_t ring_mask, uint32_t per_ticket,
                                                                   uint32_t spin_limit) {
  if (blockIdx.x == 0) {
    if (threadIdx.x < kWaveLanes) leader_loop(ctl, st, jobs, ring_mask, per_ticket, spin_limit);
  } else {
    worker_loop(st, jobs);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    const uint32_t before = __hip_atomic_fetch_add(&st->exited_wgs, 1u, __ATOMIC_ACQ_REL, AGENT);
    if (before + 1 == gridDim.x) {
      // Last workgroup out: every submission that was published has completed.
      sys_store(&ctl->completed, agent_load(&st->jobs_completed));
      __hip_atomic_store(&ctl->exited, static_cast<uint64_t>(agent_load(&st->stop)), __ATOMIC_RELEASE, SYS);
    }
  }
}

}  // namespace
}  // namespace tcpxu

using namespace tcpxu;

struct tcpxuEngine {
  int device = 0;
  uint32_t ring_entries = 0;
  uint32_t workgroups = 0;
  uint32_t per_ticket = 0;
  uint32_t spin_limit = 0;
  hipStream_t stream = nullptr;
  hipEvent_t ev_start = nullptr, ev_stop = nullptr;
  HostCtl* ctl = nullptr;      // host address of the mapped control block
  HostCtl* ctl_dev = nullptr;  // its device alias
  DevState* st = nullptr;
  Job* jobs = nullptr;
  uint64_t tail = 0;  // host copy
  bool launched = false;
  // Mapped slot ring of the streaming driver.  Allocated on first use and kept until the engine is destroyed:
  // hipHostFree waits for every stream of the device, so nothing may be freed while the kernel runs.
  void* stream_host = nullptr;
  void* stream_dev = nullptr;
  std::mutex mu;
};

static size_t ctl_bytes(uint32_t ring_entries) { return offsetof(HostCtl, ring) + sizeof(SubEntry) * ring_entries; }

extern "C" {

int tcpxuEngineCreate(int device, const tcpxuEngineConfig* config, tcpxuEngine** engine) {
  if (!engine) return TCPXU_INVALID_ARGUMENT;
  *engine = nullptr;
  tcpxuEngineConfig cfg{};
  if (config) cfg = *config;
  if (cfg.ring_entries == 0) cfg.ring_entries = 1024;
  if ((cfg.ring_entries & (cfg.ring_entries - 1)) != 0 || cfg.ring_entries > (1u << 16)) {
    set_error("ring_entries %u must be a power of two, at most 65536", cfg.ring_entries);
    return TCPXU_INVALID_ARGUMENT;
  }
  if (cfg.descs_per_ticket == 0) {
    const char* v = getenv("TCPXU_DESCS_PER_TICKET");
    cfg.descs_per_ticket = (v && *v) ? static_cast<uint32_t>(atoi(v)) : 8;
  }
  if (cfg.descs_per_ticket == 0 || cfg.descs_per_ticket > kMaxDescsPerTicket) {
    set_error("descs_per_ticket %u must be in [1,%u]", cfg.descs_per_ticket, kMaxDescsPerTicket);
    return TCPXU_INVALID_ARGUMENT;
  }
  TCPXU_TRY(use_device(device));
  const uint32_t cus = static_cast<uint32_t>(std::max(1, device_compute_units(device)));
  if (cfg.workgroups == 0) {
    const char* v = getenv("TCPXU_ENGINE_WGS_PER_CU");
    const uint32_t per_cu = (v && *v) ? static_cast<uint32_t>(atoi(v)) : 6;
    // Leave wavefront slots free on every compute unit so that other kernels (copies, the caller's own work)
    // can still be scheduled while the engine runs.
    int max_active = 0;
    TCPXU_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&max_active, unpack_engine_kernel, kWgThreads, 0));
    const uint32_t cap = max_active > 1 ? static_cast<uint32_t>(max_active) - 1 : 1;
    cfg.workgroups = cus * std::min(std::max(per_cu, 1u), cap) + 1;
  }
  if (cfg.workgroups < 2) {
    set_error("an engine needs the leader workgroup and at least one worker");
    return TCPXU_INVALID_ARGUMENT;
  }

  tcpxuEngine* e = new (std::nothrow) tcpxuEngine;
  if (!e) return TCPXU_SYSTEM_ERROR;
  e->device = device;
  e->ring_entries = cfg.ring_entries;
  e->workgroups = cfg.workgroups;
  e->per_ticket = cfg.descs_per_ticket;
  e->spin_limit = cfg.spin_limit;
  int rc = TCPXU_SUCCESS;
  do {
    void *h = nullptr, *d = nullptr;
    if ((rc = tcpxuMappedAlloc(device, ctl_bytes(cfg.ring_entries), &h, &d)) != TCPXU_SUCCESS) break;
    e->ctl = static_cast<HostCtl*>(h);
    e->ctl_dev = static_cast<HostCtl*>(d);
    const size_t st_bytes = sizeof(DevState) + sizeof(Job) * cfg.ring_entries;
    if (hipMalloc(reinterpret_cast<void**>(&e->st), st_bytes) != hipSuccess ||
        hipMemset(e->st, 0, st_bytes) != hipSuccess ||
        hipStreamCreateWithFlags(&e->stream, hipStreamNonBlocking) != hipSuccess ||
        hipEventCreate(&e->ev_start) != hipSuccess || hipEventCreate(&e->ev_stop) != hipSuccess ||
        hipDeviceSynchronize() != hipSuccess) {
      set_error("engine allocation failed: %s", hipGetErrorString(hipGetLastError()));
      rc = TCPXU_DEVICE_ERROR;
      break;
    }
    e->jobs = reinterpret_cast<Job*>(reinterpret_cast<uint8_t*>(e->st) + sizeof(DevState));
  } while (false);
  if (rc != TCPXU_SUCCESS) {
    tcpxuEngineDestroy(e);
    return rc;
  }
  *engine = e;
  return TCPXU_SUCCESS;
}

int tcpxuEngineStart(tcpxuEngine* e) {
  if (!e) return TCPXU_INVALID_ARGUMENT;
  std::lock_guard<std::mutex> lock(e->mu);
  if (e->launched) {
    set_error("engine already started");
    return TCPXU_INVALID_USAGE;
  }
  TCPXU_TRY(use_device(e->device));
  // Per-launch state: ticket counters and stop words start from zero; the submission position is kept.
  TCPXU_HIP(hipMemsetAsync(e->st, 0, offsetof(DevState, sub_head), e->stream));
  std::atomic_thread_fence(std::memory_order_seq_cst);
  e->ctl->stop = 0;
  e->ctl->exited = 0;
  std::atomic_thread_fence(std::memory_order_seq_cst);
  TCPXU_HIP(hipEventRecord(e->ev_start, e->stream));
  hipLaunchKernelGGL(unpack_engine_kernel, dim3(e->workgroups), dim3(kWgThreads), 0, e->stream, e->ctl_dev, e->st,
                     e->jobs, e->ring_entries - 1, e->per_ticket, e->spin_limit);
  TCPXU_HIP(hipGetLastError());
  TCPXU_HIP(hipEventRecord(e->ev_stop, e->stream));
  e->launched = true;
  return TCPXU_SUCCESS;
}

int tcpxuEngineStop(tcpxuEngine* e, double* elapsed_us) {
  if (!e) return TCPXU_INVALID_ARGUMENT;
  std::lock_guard<std::mutex> lock(e->mu);
  if (!e->launched) {
    set_error("engine is not started");
    return TCPXU_INVALID_USAGE;
  }
  TCPXU_TRY(use_device(e->device));
  std::atomic_thread_fence(std::memory_order_seq_cst);
  reinterpret_cast<std::atomic<uint64_t>*>(&e->ctl->stop)->store(1, std::memory_order_seq_cst);
  // Wait for the kernel's own exit word first, with a deadline: a stuck kernel then surfaces as an error
  // from this call instead of a host thread parked inside the runtime.
  const char* v = getenv("TCPXU_ENGINE_STOP_TIMEOUT_MS");
  const long timeout_ms = (v && *v) ? atol(v) : 20000;
  const auto t0 = std::chrono::steady_clock::now();
  while (reinterpret_cast<std::atomic<uint64_t>*>(&e->ctl->exited)->load(std::memory_order_acquire) == 0) {
    if (std::chrono::steady_clock::now() - t0 > std::chrono::milliseconds(timeout_ms)) {
      set_error("engine kernel did not exit within %ld ms of the stop request", timeout_ms);
      return TCPXU_INTERNAL_ERROR;
    }
    std::this_thread::yield();
  }
  TCPXU_HIP(hipEventSynchronize(e->ev_stop));
  if (elapsed_us) {
    float ms = 0.f;
    TCPXU_HIP(hipEventElapsedTime(&ms, e->ev_start, e->ev_stop));
    *elapsed_us = static_cast<double>(ms) * 1000.0;
  }
  e->launched = false;
  return TCPXU_SUCCESS;
}

int tcpxuEngineDestroy(tcpxuEngine* e) {
  if (!e) return TCPXU_SUCCESS;
  if (e->launched) {
    int rc = tcpxuEngineStop(e, nullptr);
    if (rc != TCPXU_SUCCESS) return rc;  // never free memory under a running kernel
  }
  (void)hipSetDevice(e->device);
  if (e->ev_start) (void)hipEventDestroy(e->ev_start);
  if (e->ev_stop) (void)hipEventDestroy(e->ev_stop);
  if (e->stream) (void)hipStreamDestroy(e->stream);
  if (e->st) (void)hipFree(e->st);
  if (e->ctl) (void)hipHostFree(e->ctl);
  if (e->stream_host) (void)hipHostFree(e->stream_host);
  delete e;
  return TCPXU_SUCCESS;
}

int tcpxuEngineSubmit(tcpxuEngine* e, const void* bounce_base, void* dst_base, const void* descs_dev,
                      uint32_t n_descs, void* done_flag_dev, uint64_t done_value) {
  if (!e || !done_flag_dev || done_value == 0 || reinterpret_cast<uintptr_t>(done_flag_dev) % 8 != 0) {
    set_error("submit needs an 8-byte aligned completion word and a nonzero completion value");
    return TCPXU_INVALID_ARGUMENT;
  }
  if (n_descs > 0 && (!bounce_base || !dst_base || !descs_dev || reinterpret_cast<uintptr_t>(descs_dev) % 16 != 0)) {
    set_error("submit needs bounce, destination and a 16-byte aligned descriptor address");
    return TCPXU_INVALID_ARGUMENT;
  }
  if (n_descs > kMaxDescsPerSubmission) {
    set_error("%u descriptors in one submission exceed the limit of %u", n_descs, kMaxDescsPerSubmission);
    return TCPXU_INVALID_ARGUMENT;
  }
  std::lock_guard<std::mutex> lock(e->mu);
  const uint64_t head = reinterpret_cast<std::atomic<uint64_t>*>(&e->ctl->head)->load(std::memory_order_acquire);
  if (e->tail - head >= e->ring_entries) return kTcpxuInProgress;
  uint32_t p[kPayloadWords] = {};
  const uint64_t v[5] = {reinterpret_cast<uint64_t>(bounce_base), reinterpret_cast<uint64_t>(dst_base),
                         reinterpret_cast<uint64_t>(descs_dev), reinterpret_cast<uint64_t>(done_flag_dev),
                         done_value};
  for (int i = 0; i < 5; ++i) {
    p[2 * i] = static_cast<uint32_t>(v[i]);
    p[2 * i + 1] = static_cast<uint32_t>(v[i] >> 32);
  }
  p[10] = n_descs;
  SubEntry* ent = &e->ctl->ring[e->tail & (e->ring_entries - 1)];
  volatile uint32_t* w = ent->w;
  for (int i = 0; i < kPayloadWords; ++i) w[payload_slot(i)] = p[i];
  std::atomic_thread_fence(std::memory_order_release);
  const uint32_t stamp = static_cast<uint32_t>(e->tail + 1);
  for (int sct = 0; sct < 4; ++sct) w[sct * 4 + 3] = stamp;
  std::atomic_thread_fence(std::memory_order_release);
  e->tail += 1;
  reinterpret_cast<std::atomic<uint64_t>*>(&e->ctl->tail)->store(e->tail, std::memory_order_release);
  return TCPXU_SUCCESS;
}

int tcpxuEngineCompleted(tcpxuEngine* e, uint64_t* completed) {
  if (!e || !completed) return TCPXU_INVALID_ARGUMENT;
  *completed = reinterpret_cast<std::atomic<uint64_t>*>(&e->ctl->completed)->load(std::memory_order_acquire);
  return TCPXU_SUCCESS;
}

int tcpxuEngineRunning(tcpxuEngine* e, int* running) {
  if (!e || !running) return TCPXU_INVALID_ARGUMENT;
  std::lock_guard<std::mutex> lock(e->mu);
  *running = e->launched &&
             reinterpret_cast<std::atomic<uint64_t>*>(&e->ctl->exited)->load(std::memory_order_acquire) == 0;
  return TCPXU_SUCCESS;
}

int tcpxuEngineStream(tcpxuEngine* e, const tcpxuStreamItem* items, uint64_t n_items, uint32_t depth,
                      uint32_t stall_timeout_ms, double* wall_us, double* latency_us) {
  if (!e || !items || !wall_us || depth == 0 || depth > TCPXU_QUEUE_DEPTH) return TCPXU_INVALID_ARGUMENT;
  for (uint64_t i = 0; i < n_items; ++i) {
    if (items[i].n_descs > TCPXU_SLOT_PAGES) {
      set_error("stream item %llu has %u descriptors, a slot holds %d", static_cast<unsigned long long>(i),
                items[i].n_descs, TCPXU_SLOT_PAGES);
      return TCPXU_INVALID_ARGUMENT;
    }
  }
  if (stall_timeout_ms == 0) stall_timeout_ms = 10000;
  // Mapped block: `depth` completion words (one cache line each), then `depth` descriptor slots.
  const size_t flag_stride = 64;
  const size_t slot_bytes = sizeof(tcpxuLoadMeta) * TCPXU_SLOT_PAGES;
  const size_t flags_bytes = flag_stride * TCPXU_QUEUE_DEPTH;
  if (!e->stream_host)
    TCPXU_TRY(tcpxuMappedAlloc(e->device, flags_bytes + slot_bytes * TCPXU_QUEUE_DEPTH, &e->stream_host,
                               &e->stream_dev));
  uint8_t* hb = static_cast<uint8_t*>(e->stream_host);
  uint8_t* db = static_cast<uint8_t*>(e->stream_dev);
  memset(hb, 0, flags_bytes);
  using clock = std::chrono::steady_clock;
  std::vector<clock::time_point> published(depth);
  int rc = TCPXU_SUCCESS;
  uint64_t next_submit = 0, next_done = 0;
  const auto t_begin = clock::now();
  auto last_progress = t_begin;
  auto t_end = t_begin;
  while (next_done < n_items) {
    bool progress = false;
    // Reap completions in FIFO order.
    while (next_done < next_submit) {
      const uint32_t slot = static_cast<uint32_t>(next_done % depth);
      auto* flag = reinterpret_cast<std::atomic<uint64_t>*>(hb + flag_stride * slot);
      if (flag->load(std::memory_order_acquire) != next_done + 1) break;
      const auto now = clock::now();
      if (latency_us)
        latency_us[next_done] = std::chrono::duration<double, std::micro>(now - published[slot]).count();
      t_end = now;
      ++next_done;
      progress = true;
    }
    // Publish while a slot is free.
    while (next_submit < n_items && next_submit - next_done < depth) {
      const uint32_t slot = static_cast<uint32_t>(next_submit % depth);
      const tcpxuStreamItem& it = items[next_submit];
      uint8_t* slot_host = hb + flags_bytes + slot_bytes * slot;
      if (it.n_descs) memcpy(slot_host, it.descs_host, sizeof(tcpxuLoadMeta) * it.n_descs);
      published[slot] = clock::now();
      rc = tcpxuEngineSubmit(e, it.bounce_base, it.dst_base, db + flags_bytes + slot_bytes * slot, it.n_descs,
                             db + flag_stride * slot, next_submit + 1);
      if (rc == kTcpxuInProgress) {
        rc = TCPXU_SUCCESS;
        break;  // engine ring full: reap first
      }
      if (rc != TCPXU_SUCCESS) break;
      ++next_submit;
      progress = true;
    }
    if (rc != TCPXU_SUCCESS) break;
    const auto now = clock::now();
    if (progress) {
      last_progress = now;
    } else if (now - last_progress > std::chrono::milliseconds(stall_timeout_ms)) {
      set_error("stream stalled: %llu of %llu items completed, %llu published",
                static_cast<unsigned long long>(next_done), static_cast<unsigned long long>(n_items),
                static_cast<unsigned long long>(next_submit));
      rc = TCPXU_INTERNAL_ERROR;
      break;
    }
  }
  *wall_us = std::chrono::duration<double, std::micro>(t_end - t_begin).count();
  return rc;
}

int tcpxuEngineRunTimed(tcpxuEngine* e, const tcpxuStreamItem* items, uint64_t n_items, uint32_t depth,
                        uint32_t stall_timeout_ms, double* wall_us, double* kernel_us, double* latency_us) {
  if (!e || !kernel_us) return TCPXU_INVALID_ARGUMENT;
  // Touch the stream block before the launch so that no allocation happens while the kernel is timed.
  if (!e->stream_host) {
    const size_t bytes = 64 * TCPXU_QUEUE_DEPTH + sizeof(tcpxuLoadMeta) * TCPXU_SLOT_PAGES * TCPXU_QUEUE_DEPTH;
    TCPXU_TRY(tcpxuMappedAlloc(e->device, bytes, &e->stream_host, &e->stream_dev));
  }
  TCPXU_TRY(tcpxuEngineStart(e));
  const int rc = tcpxuEngineStream(e, items, n_items, depth, stall_timeout_ms, wall_us, latency_us);
  const int rc_stop = tcpxuEngineStop(e, kernel_us);
  return rc != TCPXU_SUCCESS ? rc : rc_stop;
}

}  // extern "C"
