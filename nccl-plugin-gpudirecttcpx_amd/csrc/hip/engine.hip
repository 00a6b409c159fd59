// Persistent unpack engine: one long-running gfx950 kernel per GPU that turns slots published in mapped host
// memory into scatter-gather copies and reports completion into mapped host memory -- no launch per request.
//
// Roles inside the one kernel launch
//   workgroup 0, wavefront 0  "leader": polls the submission ring over PCIe (four entries per round trip), cuts
//                             each submission into tickets of `descs_per_ticket` consecutive descriptors and
//                             writes them into a device-memory ticket ring.  It never copies payload and never
//                             waits for a store of its own.
//   every other workgroup     "worker": claims the next ticket number with one atomic, polls that ticket's slot
//                             until its stamps match, stages the ticket's descriptors from the mapped slot into
//                             LDS, lets its four wavefronts copy fragments, then counts the ticket done.  Whoever
//                             counts the last ticket of a submission writes the completion word that the host
//                             poller reads.
//
// No cache maintenance.  Nothing here uses an acquire or release fence: on this GPU those become L2 write-back
// and invalidate instructions, and thousands of pollers issuing them stall everybody.  Instead every access
// to shared state carries its own coherence: control words and tickets are read and written with system-scope
// (sc0 sc1) accesses that bypass the per-XCD L2, payload is loaded and stored the same way, and ordering comes
// from s_waitcnt: a wavefront drains its store counter before the workgroup counts a ticket done.
// Records that are written by one side and polled by the other (host submissions, tickets) are 64 bytes in four
// 16-byte sectors, each ending in a stamp derived from the record's sequence number; a reader accepts a record
// only when all four stamps match, so a record is valid even if its sectors arrive as separate transactions,
// and the writer never has to order "payload, then flag".
//
// Liveness: no workgroup ever waits for another worker.  Workers wait only for the leader (their ticket) and
// watch the stop word while they do; the leader waits for nothing (a full ticket ring or job table just defers
// a submission to the next poll).  The host stop word, or the optional spin limit, ends the leader; the leader
// drains its stores, then sets the stop words; a worker that sees one looks at its ticket a last time and leaves.
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

constexpr uint32_t kTicketRing = 1u << 16;  // tickets in flight at most
constexpr uint32_t kMaxDescsPerTicket = 64;
constexpr uint32_t kMaxDescsPerSubmission = 1u << 20;
constexpr uint32_t kStopReplicas = 64;
constexpr uint32_t kPollEntries = 4;  // submission entries fetched per leader poll
constexpr int kTcpxuInProgress = TCPXU_IN_PROGRESS;

// 64-byte record: four 16-byte sectors of three payload words and one stamp word.
struct alignas(64) Record {
  uint32_t w[16];
};
constexpr int kPayloadWords = 12;
__host__ __device__ constexpr int payload_slot(int i) { return (i / 3) * 4 + (i % 3); }
// Submission payload: 0-1 bounce, 2-3 dst, 4-5 descs, 6-7 done_flag, 8-9 done_value, 10 n_descs, 11 unused.
// Ticket payload:     0-1 bounce, 2-3 dst, 4-5 descs, 6-7 done_flag, 8-9 done_value, 10 n | job << 8, 11 target.

struct HostCtl {  // mapped host memory
  alignas(64) uint64_t tail;       // host -> GPU: submissions published so far
  alignas(64) uint64_t stop;       // host -> GPU: drain and exit
  alignas(64) uint64_t head;       // GPU -> host: submissions the leader has consumed
  alignas(64) uint64_t completed;  // GPU -> host: submissions fully unpacked (mirrored when idle and at exit)
  alignas(64) uint64_t exited;     // GPU -> host: 0 running, 1 stopped on request, 2 spin limit reached
  alignas(64) Record ring[1];      // ring_entries follow
};

struct alignas(256) StopWord {
  uint32_t value;
};

struct DevState {  // device memory
  alignas(64) uint64_t ticket_head;     // next ticket number to claim
  alignas(64) uint64_t tickets_done;    // tickets whose payload is written
  alignas(64) uint64_t jobs_completed;  // submissions completed since creation
  alignas(64) uint64_t sub_head;        // leader-private: next submission index
  uint64_t tickets_out;                 // leader-private: tickets written so far
  alignas(64) uint32_t exited_wgs;      // reset at every start, as are the stop words
  uint32_t exit_reason;
  alignas(256) StopWord stop[kStopReplicas];
  alignas(64) Record tickets[kTicketRing];
  // uint32_t jobs_done[ring_entries], then uint32_t job_target[ring_entries] follow
};

// ---- scoped memory operations -------------------------------------------------------------------------------------
#define SYS __HIP_MEMORY_SCOPE_SYSTEM

template <typename T>
__device__ __forceinline__ T sys_load(const T* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, SYS);
}
template <typename T>
__device__ __forceinline__ void sys_store(T* p, T v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, SYS);
}
__device__ __forceinline__ void drain_memory_ops() { asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory"); }

__device__ __forceinline__ uint32_t bcast(uint32_t v, uint32_t src_lane) {
  return __shfl(v, static_cast<int>(src_lane), kWaveLanes);
}
__device__ __forceinline__ uint64_t bcast64(uint64_t v, uint32_t src_lane) {
  return (static_cast<uint64_t>(bcast(static_cast<uint32_t>(v >> 32), src_lane)) << 32) |
         bcast(static_cast<uint32_t>(v), src_lane);
}
// Payload word i of the record held by lanes [first_lane, first_lane + 16).
__device__ __forceinline__ uint32_t payload32(uint32_t word, uint32_t first_lane, int i) {
  return bcast(word, first_lane + payload_slot(i));
}
__device__ __forceinline__ uint64_t payload64(uint32_t word, uint32_t first_lane, int i) {
  return (static_cast<uint64_t>(payload32(word, first_lane, i + 1)) << 32) | payload32(word, first_lane, i);
}

__device__ __forceinline__ void write_record(Record* rec, const uint32_t (&p)[kPayloadWords], uint32_t stamp) {
  uint8_t* base = reinterpret_cast<uint8_t*>(rec);
#pragma unroll
  for (int sct = 0; sct < 4; ++sct) {
    u32x4 v = {p[3 * sct], p[3 * sct + 1], p[3 * sct + 2], stamp};
    store_vec_sys(base + 16 * sct, v);
  }
}

// ---- leader -------------------------------------------------------------------------------------------------------
// Runs on wavefront 0 of workgroup 0.  All control flow is wave-uniform.
__device__ void leader_loop(HostCtl* ctl, DevState* st, uint32_t* jobs_done, uint32_t* job_target,
                            uint32_t ring_mask, uint32_t per_ticket, uint32_t spin_limit) {
  const uint32_t lane = threadIdx.x;
  uint64_t s = sys_load(&st->sub_head);
  uint64_t tickets_out = sys_load(&st->tickets_out);
  uint64_t mirrored = ~0ull;
  uint64_t idle = 0;
  uint32_t reason = 0;

  for (;;) {
    // One round trip fetches entries s .. s+3 (lane 16k+i reads word i of entry s+k) and, alongside, what is
    // needed to act on them: for each entry its job slot's counters, plus tickets_done and the host stop word.
    const uint32_t k_of_lane = lane >> 4;
    const Record* e = &ctl->ring[(s + k_of_lane) & ring_mask];
    const uint32_t word = sys_load(&e->w[lane & 15]);
    uint64_t aux = 0;
    if (lane < kPollEntries) aux = sys_load(&jobs_done[(s + lane) & ring_mask]);
    else if (lane < 2 * kPollEntries) aux = sys_load(&job_target[(s + lane - kPollEntries) & ring_mask]);
    else if (lane == 8) aux = sys_load(&st->tickets_done);
    else if (lane == 9) aux = sys_load(&ctl->stop);
    const uint32_t expect = static_cast<uint32_t>(s + k_of_lane + 1);
    const bool stamp_ok = ((lane & 3) == 3) ? (word == expect) : true;
    const uint64_t ok_mask = __ballot(stamp_ok);
    const uint64_t tickets_done = bcast64(aux, 8);

    uint32_t consumed = 0;
    for (uint32_t k = 0; k < kPollEntries; ++k) {
      if (((ok_mask >> (16 * k)) & 0xFFFFull) != 0xFFFFull) break;
      const uint32_t first_lane = 16 * k;
      const uint32_t n = payload32(word, first_lane, 10);
      if (n == 0) {
        // Lane broadcasts need the whole wavefront: read the fields before narrowing to one lane.
        const uint64_t done_flag = payload64(word, first_lane, 6);
        const uint64_t done_value = payload64(word, first_lane, 8);
        if (lane == 0) {
          sys_store(reinterpret_cast<uint64_t*>(done_flag), done_value);
          __hip_atomic_fetch_add(&st->jobs_completed, 1ull, __ATOMIC_RELAXED, SYS);
        }
      } else {
        const uint32_t nt = (n + per_ticket - 1) / per_ticket;
        const uint32_t slot = static_cast<uint32_t>(s + k) & ring_mask;
        const uint32_t done_now = bcast(static_cast<uint32_t>(aux), k);
        const uint32_t target_prev = bcast(static_cast<uint32_t>(aux), kPollEntries + k);
        // The job slot is free once every ticket ever issued for it has been counted; the ticket ring has room
        // while fewer than its size are outstanding.  Otherwise leave this entry for a later poll.
        if (done_now != target_prev) break;
        if (tickets_out + nt - tickets_done > kTicketRing) break;
        const uint32_t target = target_prev + nt;
        if (lane == 0) sys_store(&job_target[slot], target);
        uint32_t p[kPayloadWords];
#pragma unroll
        for (int i = 0; i < 10; ++i) p[i] = payload32(word, first_lane, i);
        p[11] = target;
        const uint64_t descs = (static_cast<uint64_t>(p[5]) << 32) | p[4];
        for (uint32_t i = lane; i < nt; i += kWaveLanes) {
          const uint64_t d = descs + static_cast<uint64_t>(i) * per_ticket * sizeof(tcpxuLoadMeta);
          p[4] = static_cast<uint32_t>(d);
          p[5] = static_cast<uint32_t>(d >> 32);
          p[10] = std::min(per_ticket, n - i * per_ticket) | (slot << 8);
          const uint64_t t = tickets_out + i;
          write_record(&st->tickets[t & (kTicketRing - 1)], p, static_cast<uint32_t>(t + 1));
        }
        tickets_out += nt;
      }
      ++consumed;
    }
    if (consumed != 0) {
      s += consumed;
      idle = 0;
      if (lane == 0) sys_store(&ctl->head, s);
      continue;
    }

    // Nothing could be consumed this round.
    if (bcast64(aux, 9) != 0 && ((ok_mask & 0xFFFFull) != 0xFFFFull)) {
      // Stop requested and entry s not there.  The host wrote its last tail before the stop word, so a tail
      // read now bounds what is still to come.
      uint64_t tail_now = 0;
      if (lane == 0) tail_now = sys_load(&ctl->tail);
      if (s >= bcast64(tail_now, 0)) {
        reason = 1;
        break;
      }
      continue;
    }
    if (lane == 0) {
      const uint64_t c = sys_load(&st->jobs_completed);
      if (c != mirrored) {
        sys_store(&ctl->completed, c);
        mirrored = c;
      }
    }
    const bool nothing_there = (ok_mask & 0xFFFFull) != 0xFFFFull;
    if (spin_limit != 0 && nothing_there && ++idle > spin_limit) {
      reason = 2;
      break;
    }
    __builtin_amdgcn_s_sleep(1);
  }

  // Every ticket written must be visible before any stop word is.
  drain_memory_ops();
  if (lane == 0) {
    sys_store(&st->sub_head, s);
    sys_store(&st->tickets_out, tickets_out);
    sys_store(&st->exit_reason, reason);
  }
  drain_memory_ops();
  sys_store(&st->stop[lane].value, 1u);
}

// ---- worker -------------------------------------------------------------------------------------------------------
__device__ void worker_loop(DevState* st, uint32_t* jobs_done) {
  __shared__ uint32_t s_payload[kPayloadWords];
  __shared__ tcpxuLoadMeta s_desc[kMaxDescsPerTicket];
  __shared__ uint32_t s_go;

  const uint32_t tid = threadIdx.x;
  const uint32_t lane = tid & (kWaveLanes - 1);
  const uint32_t wave = tid / kWaveLanes;
  const uint32_t* stop_word = &st->stop[blockIdx.x % kStopReplicas].value;
  uint64_t my_ticket = 0;  // valid in wavefront 0
  if (wave == 0) {
    uint64_t t = 0;
    if (lane == 0) t = __hip_atomic_fetch_add(&st->ticket_head, 1ull, __ATOMIC_RELAXED, SYS);
    my_ticket = bcast64(t, 0);
  }

  for (;;) {
    if (wave == 0) {
      // Poll my ticket's slot (one 64-byte read) together with this workgroup's stop word.
      const Record* rec = &st->tickets[my_ticket & (kTicketRing - 1)];
      const uint32_t expect = static_cast<uint32_t>(my_ticket + 1);
      uint32_t go = 0;
      uint32_t word = 0;
      bool stop_seen = false;
      uint32_t backoff = 1;
      for (;;) {
        uint32_t v = 0;
        if (lane < 16) v = sys_load(&rec->w[lane]);
        else if (lane == 16) v = sys_load(stop_word);
        const bool stamp_ok = (lane < 16 && (lane & 3) == 3) ? (v == expect) : true;
        if (__all(stamp_ok)) {
          go = 1;
          word = v;
          break;
        }
        if (stop_seen) break;  // the stop word was already up on the previous look: my ticket will never come
        stop_seen = bcast(v, 16) != 0;
        if (!stop_seen) {
          for (uint32_t i = 0; i < backoff; ++i) __builtin_amdgcn_s_sleep(4);
          if (backoff < 16) backoff <<= 1;
        }
      }
      // Lane broadcasts need the whole wavefront: gather first, then let 12 lanes store.
      const uint32_t pl = lane < kPayloadWords ? lane : 0u;
      const uint32_t gathered = bcast(word, (pl / 3) * 4 + (pl % 3));
      if (go && lane < kPayloadWords) s_payload[lane] = gathered;
      if (lane == 0) s_go = go;
    }
    __syncthreads();
    if (s_go == 0) break;  // workgroup-uniform
    const uint64_t bounce_addr = (static_cast<uint64_t>(s_payload[1]) << 32) | s_payload[0];
    const uint64_t dst_addr = (static_cast<uint64_t>(s_payload[3]) << 32) | s_payload[2];
    const uint64_t descs_addr = (static_cast<uint64_t>(s_payload[5]) << 32) | s_payload[4];
    const uint32_t n = s_payload[10] & 0xFFu;
    if (tid < n) {
      // 16-byte descriptor as two system-scope 8-byte loads straight from the mapped slot.
      const uint64_t* p = reinterpret_cast<const uint64_t*>(descs_addr) + 2 * tid;
      const uint64_t lo = sys_load(p);
      const uint64_t hi = sys_load(p + 1);
      s_desc[tid].src_off = static_cast<uint32_t>(lo);
      s_desc[tid].len = static_cast<uint32_t>(lo >> 32);
      s_desc[tid].dst_off = hi;
    }
    // Claim the next ticket number now: the atomic's round trip overlaps this ticket's copy.
    uint64_t next_ticket = 0;
    if (tid == 0) next_ticket = __hip_atomic_fetch_add(&st->ticket_head, 1ull, __ATOMIC_RELAXED, SYS);
    __syncthreads();

    const uint8_t* bounce = reinterpret_cast<const uint8_t*>(bounce_addr);
    uint8_t* dst = reinterpret_cast<uint8_t*>(dst_addr);
    for (uint32_t j = wave; j < n; j += kWavesPerWg) {
      const tcpxuLoadMeta d = s_desc[j];
      const uint32_t len = __builtin_amdgcn_readfirstlane(d.len);
      const uint32_t so = __builtin_amdgcn_readfirstlane(d.src_off);
      const uint32_t dlo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(d.dst_off));
      const uint32_t dhi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(d.dst_off >> 32));
      wave_copy_fragment_coherent(bounce + so, dst + ((static_cast<uint64_t>(dhi) << 32) | dlo), len, lane);
    }
    // Each wavefront waits until its own write-through payload stores are acknowledged; after the barrier the
    // whole ticket is in memory and may be counted.
    drain_memory_ops();
    __syncthreads();

    if (wave == 0) {
      if (lane == 0) {
        const uint32_t job = s_payload[10] >> 8;
        const uint32_t target = s_payload[11];
        const uint32_t count = __hip_atomic_fetch_add(&jobs_done[job], 1u, __ATOMIC_RELAXED, SYS) + 1u;
        __hip_atomic_fetch_add(&st->tickets_done, 1ull, __ATOMIC_RELAXED, SYS);
        if (count == target) {
          // Last ticket of the submission: every other ticket's payload was in memory before it was counted.
          const uint64_t done_flag = (static_cast<uint64_t>(s_payload[7]) << 32) | s_payload[6];
          const uint64_t done_value = (static_cast<uint64_t>(s_payload[9]) << 32) | s_payload[8];
          sys_store(reinterpret_cast<uint64_t*>(done_flag), done_value);
          __hip_atomic_fetch_add(&st->jobs_completed, 1ull, __ATOMIC_RELAXED, SYS);
        }
      }
      my_ticket = bcast64(next_ticket, 0);
    }
    // s_payload / s_desc are rewritten only after the next barrier pair; wavefront 0 rewrites s_payload before
    // the first barrier of the next iteration, so everybody must be past their reads of it: they are, since
    // the reads above happen before the second barrier of this iteration.
  }
}

__global__ __launch_bounds__(kWgThreads) void unpack_engine_kernel(HostCtl* ctl, DevState* st, uint32_t* jobs_done,
                                                                   uint32_t* job_target, uint32_t ring_mask,
                                                                   uint32_t per_ticket, uint32_t spin_limit) {
  if (blockIdx.x == 0) {
    if (threadIdx.x < kWaveLanes) leader_loop(ctl, st, jobs_done, job_target, ring_mask, per_ticket, spin_limit);
  } else {
    worker_loop(st, jobs_done);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    drain_memory_ops();
    const uint32_t before = __hip_atomic_fetch_add(&st->exited_wgs, 1u, __ATOMIC_RELAXED, SYS);
    if (before + 1 == gridDim.x) {
      // Last workgroup out: every ticket that was written has been counted.  Ticket numbers claimed beyond the
      // last written one are given back, so the next launch starts where this one ended.
      sys_store(&st->ticket_head, sys_load(&st->tickets_out));
      sys_store(&ctl->completed, sys_load(&st->jobs_completed));
      drain_memory_ops();
      sys_store(&ctl->exited, static_cast<uint64_t>(sys_load(&st->exit_reason)));
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
  uint32_t* jobs_done = nullptr;   // [ring_entries], device memory
  uint32_t* job_target = nullptr;  // [ring_entries], device memory, leader-private
  uint64_t tail = 0;  // host copy
  bool launched = false;
  // Mapped slot ring of the streaming driver.  Allocated on first use and kept until the engine is destroyed:
  // hipHostFree waits for every stream of the device, so nothing may be freed while the kernel runs.
  void* stream_host = nullptr;
  void* stream_dev = nullptr;
  std::mutex mu;
};

static size_t ctl_bytes(uint32_t ring_entries) { return offsetof(HostCtl, ring) + sizeof(Record) * ring_entries; }

extern "C" {

int tcpxuEngineCreate(int device, const tcpxuEngineConfig* config, tcpxuEngine** engine) {
  if (!engine) return TCPXU_INVALID_ARGUMENT;
  *engine = nullptr;
  tcpxuEngineConfig cfg{};
  if (config) cfg = *config;
  if (cfg.ring_entries == 0) cfg.ring_entries = 1024;
  if ((cfg.ring_entries & (cfg.ring_entries - 1)) != 0 || cfg.ring_entries > (1u << 16) || cfg.ring_entries < 16) {
    set_error("ring_entries %u must be a power of two in [16, 65536]", cfg.ring_entries);
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
    const size_t st_bytes = sizeof(DevState) + 2 * sizeof(uint32_t) * cfg.ring_entries;
    if (hipMalloc(reinterpret_cast<void**>(&e->st), st_bytes) != hipSuccess ||
        hipMemset(e->st, 0, st_bytes) != hipSuccess ||
        hipStreamCreateWithFlags(&e->stream, hipStreamNonBlocking) != hipSuccess ||
        hipEventCreate(&e->ev_start) != hipSuccess || hipEventCreate(&e->ev_stop) != hipSuccess ||
        hipDeviceSynchronize() != hipSuccess) {
      set_error("engine allocation failed: %s", hipGetErrorString(hipGetLastError()));
      rc = TCPXU_DEVICE_ERROR;
      break;
    }
    e->jobs_done = reinterpret_cast<uint32_t*>(reinterpret_cast<uint8_t*>(e->st) + sizeof(DevState));
    e->job_target = e->jobs_done + cfg.ring_entries;
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
  // Per-launch state: exit bookkeeping and stop words start from zero; positions and counters are kept.
  TCPXU_HIP(hipMemsetAsync(reinterpret_cast<uint8_t*>(e->st) + offsetof(DevState, exited_wgs), 0,
                           offsetof(DevState, tickets) - offsetof(DevState, exited_wgs), e->stream));
  std::atomic_thread_fence(std::memory_order_seq_cst);
  e->ctl->stop = 0;
  e->ctl->exited = 0;
  std::atomic_thread_fence(std::memory_order_seq_cst);
  TCPXU_HIP(hipEventRecord(e->ev_start, e->stream));
  hipLaunchKernelGGL(unpack_engine_kernel, dim3(e->workgroups), dim3(kWgThreads), 0, e->stream, e->ctl_dev, e->st,
                     e->jobs_done, e->job_target, e->ring_entries - 1, e->per_ticket, e->spin_limit);
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
  Record* ent = &e->ctl->ring[e->tail & (e->ring_entries - 1)];
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
