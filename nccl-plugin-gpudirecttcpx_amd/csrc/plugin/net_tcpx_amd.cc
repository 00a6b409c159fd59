// ncclNet_v7 entry points of the receive-side unpack path and the progress engine behind them.
//
// Call pattern (NCCL's receive proxy, or a test driver in its place):
//   irecv -> test* -> [consume the data] -> iflush? -> irecvConsumed
// Who copies is a switch (NCCL_GPUDIRECTTCPX_AMD_DEVICE_TYPE).  "host" (default): the plugin advertises an
// ordinary host-driven network, its GPU engine unpacks every request and a request reports done=1 only after the
// engine has written its completion word, i.e. after the payload is in the receive buffer.  "unpack": the
// reference's division of labour -- done=1 means "descriptor count published" (src/net_tcpx.cc:1354-1357), the
// device handle is advertised and the caller's own kernel does the copy; the engine is never started.
// Everything else (states, order checks, result codes) follows src/net_tcpx.cc.
#include <errno.h>
#include <limits.h>
#include <sched.h>
#include <strings.h>

#include <algorithm>
#include <atomic>
#include <chrono>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <string>

#include "plugin_internal.h"

namespace tcpx {

Global g;

// ---- logging and flags --------------------------------------------------------------------------------------------
void log_line(ncclDebugLogLevel level, unsigned long flags, const char* file, int line, const char* fmt, ...) {
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  if (g.logger) {
    g.logger(level, flags, file, line, "%s", buf);
  } else if (level == NCCL_LOG_WARN) {
    // Without NCCL's logger only warnings are printed (the reference's fallback prints everything,
    // src/adapter/nccl/debug.cc:22-33; INFO is too chatty for a test run).
    fprintf(stderr, "NET/GPUDirectTCPX-AMD WARN %s:%d %s\n", file, line, buf);
  }
}

ncclResult_t fail_stop(const char* what) {
  if (g.fail_stop) {
    WARN("fail-stop: %s", what);
    exit(1);
  }
  return ncclInternalError;
}

namespace {

// NCCL_GPUDIRECTTCPX_<NAME>, kept only if it parses and lies in [lo, hi] (TCPX_GET_INT_FLAG,
// src/net_tcpx.cc:440-452; TCPX_GET_ENV, src/adapter/param1.h:26-29).
void int_flag(int* flag, const char* name, long lo, long hi) {
  char env[128];
  snprintf(env, sizeof env, "NCCL_GPUDIRECTTCPX_%s", name);
  const char* v = getenv(env);
  if (!v || !*v) return;
  char* end = nullptr;
  const long x = strtol(v, &end, 0);
  if (end == v || x < lo || x > hi) {
    WARN("%s=%s ignored: not an integer in [%ld, %ld]", env, v, lo, hi);
    return;
  }
  *flag = static_cast<int>(x);
}

void int64_flag(int64_t* flag, const char* name, long long lo) {  // [lo, LLONG_MAX)
  char env[128];
  snprintf(env, sizeof env, "NCCL_GPUDIRECTTCPX_%s", name);
  const char* v = getenv(env);
  if (!v || !*v) return;
  char* end = nullptr;
  const long long x = strtoll(v, &end, 0);
  if (end == v || x < lo || x == LLONG_MAX) {
    WARN("%s=%s ignored: not an integer in [%lld, LLONG_MAX)", env, v, lo);
    return;
  }
  *flag = x;
}

// parseSlownessSwitchFlags, src/flags.cc:119-150: which waits are watched, and which of those are reported.
void parse_slowness_flags() {
  static const char kDefault[] = "TX_COMP,SENDRECV,RX_CTRL,UNPACK";
  for (int i = 0; i < kSlowKinds; ++i) g.slow_switch[i] = g.slow_report[i] = 0;
  const char* sw = getenv("NCCL_GPUDIRECTTCPX_SLOWNESS_SWITCH");
  parse_slowness_switches(sw ? sw : kDefault, g.slow_switch);
  const char* rp = getenv("NCCL_GPUDIRECTTCPX_SLOWNESS_REPORT");
  parse_slowness_switches(rp ? rp : kDefault, g.slow_report);
  for (int i = 0; i < kSlowKinds; ++i) {
    if (!g.slow_switch[i] && g.slow_report[i]) {
      INFO(NCCL_INIT, "%s slowness: detection is disabled, hence turning report off", kSlownessNames[i]);
      g.slow_report[i] = 0;
    }
    INFO(NCCL_INIT, "%s slowness: detection %d report %d", kSlownessNames[i], g.slow_switch[i], g.slow_report[i]);
  }
}

// NCCL_GPUDIRECTTCPX_SCHED_ALG, src/net_tcpx.cc:643-665: "RR" when unset, and also (with a note) when not a known name.
void parse_sched_alg() {
  const char* v = getenv("NCCL_GPUDIRECTTCPX_SCHED_ALG");
  if (!v) {
    g.sched_alg = kSchedRoundRobin;
    INFO(NCCL_INIT, "NCCL_GPUDIRECTTCPX_SCHED_ALG unset. Using RR by default");
    return;
  }
  bool valid = false;
  g.sched_alg = sched_alg_from_name(v, &valid);
  if (valid) {
    INFO(NCCL_INIT, "NCCL_GPUDIRECTTCPX_SCHED_ALG %s", v);
  } else {
    INFO(NCCL_INIT, "invalid NCCL_GPUDIRECTTCPX_SCHED_ALG %s. Using RR by default", v);
  }
}

// NCCL_GPUDIRECTTCPX_AMD_DEVICE_TYPE: "host" when unset, and also (with a warning) when not a known name.
void parse_device_type() {
  g.device_type = kDeviceHost;
  const char* v = getenv("NCCL_GPUDIRECTTCPX_AMD_DEVICE_TYPE");
  if (!v || !*v) return;
  if (strcasecmp(v, "unpack") == 0) {
    g.device_type = kDeviceUnpack;
  } else if (strcasecmp(v, "host") != 0) {
    WARN("NCCL_GPUDIRECTTCPX_AMD_DEVICE_TYPE=%s ignored: not \"host\" or \"unpack\"; using host", v);
  }
  INFO(NCCL_INIT, "device type %s", g.device_type == kDeviceUnpack ? "unpack (the caller's kernel copies)" : "host (the plugin's engine copies)");
}

// NCCL_GPUDIRECTTCPX_RX_BINDINGS: the CPUs a receive comm's socket thread may run on, per network device, in the
// reference's syntax "name:lo-hi,lo-hi;name:lo-hi" (parseCoreRanges, src/common.cc:65-130; the names are the ones
// getProperties reports).  A device that is not named keeps the CPUs the process may use (the reference's default is
// the NIC's NUMA node, src/net_tcpx.cc:592-611; a synthetic device has none).  A malformed range is reported and
// skipped and the device's other ranges stand, as there (src/common.cc:104-108).  Called once the device names exist.
void parse_rx_bindings() {
  for (int d = 0; d < kMaxDevices; ++d) {
    CPU_ZERO(&g.rx_cpus[d]);
    g.rx_bound[d] = false;
  }
  const char* v = getenv("NCCL_GPUDIRECTTCPX_RX_BINDINGS");
  if (!v || !*v) return;
  INFO(NCCL_INIT, "NCCL_GPUDIRECTTCPX_RX_BINDINGS %s", v);
  const std::string all(v);
  size_t at = 0;
  while (at < all.size()) {
    size_t end = all.find(';', at);
    if (end == std::string::npos) end = all.size();
    const std::string phrase = all.substr(at, end - at);
    at = end + 1;
    const size_t colon = phrase.find(':');
    if (colon == std::string::npos) continue;
    const std::string name = phrase.substr(0, colon);
    int dev = -1;
    for (int d = 0; d < g.n_devices; ++d) {
      if (name == g.dev_names[d]) dev = d;
    }
    if (dev < 0) {
      INFO(NCCL_NET, "%s not a device of this run", name.c_str());
      continue;
    }
    cpu_set_t set;
    CPU_ZERO(&set);
    size_t r = colon + 1;
    while (r <= phrase.size()) {
      size_t comma = phrase.find(',', r);
      if (comma == std::string::npos) comma = phrase.size();
      const std::string range = phrase.substr(r, comma - r);
      r = comma + 1;
      int lo = -1, hi = -1;
      char tail = 0;
      if (sscanf(range.c_str(), "%d-%d%c", &lo, &hi, &tail) != 2 || lo < 0 || hi < lo || hi >= CPU_SETSIZE) {
        WARN("invalid range %s", range.c_str());
        continue;  // this range only
      }
      for (int c = lo; c <= hi; ++c) CPU_SET(c, &set);
    }
    if (CPU_COUNT(&set) == 0) continue;  // nothing valid was named: the device stays unbound
    g.rx_cpus[dev] = set;
    g.rx_bound[dev] = true;
  }
}

// Timestamp of a tracepoint: the wall clock like the reference's exporter lines, or the injected clock.
int64_t trace_timestamp() {
  if (g.clock_injected) return static_cast<int64_t>(g.clock());
  return std::chrono::duration_cast<std::chrono::nanoseconds>(std::chrono::system_clock::now().time_since_epoch()).count();
}
// tcpxTP_REQUEST / tcpxTP_TASK state tracepoints (src/stats/tracepoint.cc:84-103,178-232).
void tp_request(Comm* comm, const Request* r, int state) {
  if (g.request_stats && comm->trace) comm->trace->enqueue('R', r, comm->passive, state, trace_timestamp(), g.sampling_factor);
}
void tp_task(Comm* comm, const Task* t, int state) {
  if (g.task_stats && comm->trace) comm->trace->enqueue('T', t, comm->passive, state, trace_timestamp(), g.sampling_factor);
}
// The ring transitions with their tracepoints, fired on the item that is about to move (src/work_queue.h:156-211).
void request_advance(Comm* comm, int stage) {
  static const int kEntered[kReqStages] = {kReqPostedTs, kReqTransmittingTs, kReqInactiveTs, kReqFreeTs};
  tp_request(comm, comm->rq.first(stage), kEntered[stage]);
  comm->rq.advance(stage);
}
void task_advance(Comm* comm, TaskRing* tasks, int stage) {
  static const int kEntered[kTaskStages] = {kTaskCompletingTs, kTaskInactiveTs, kTaskFreeTs};
  tp_task(comm, tasks->first(stage), kEntered[stage]);
  tasks->advance(stage);
}

inline bool ctrl_done(const Request* r) { return r->next_flow >= 0; }  // CTRL_DONE, src/net_tcpx.cc:956
// REQUEST_DONE, src/net_tcpx.cc:959-960
inline bool request_done(const Request* r) {
  return (r->size == 0 && ctrl_done(r)) || (r->size && r->size_pending == 0);
}

// ---- socket side: one task's progress (taskProgress, src/net_tcpx.cc:148-212) -------------------------------------
ncclResult_t flow_progress(Comm* comm, int flow) {
  FlowData* fd = &comm->flows[flow];
  TaskRing* tasks = &fd->tasks;
  // The flow's tasks in order: a task whose bytes have all arrived makes room for the next one in the same call (the
  // socket delivers in order, so a task that has to wait ends the pass).
  for (int served = 0; served < kMaxTasks; ++served) {
    if (tasks->has(kTaskActive)) {
      Task* t = tasks->first(kTaskActive);
      if (t->offset == 0) {
        // Nothing received for this task yet: its pipe starts empty.  (Done here, by the thread that serves the
        // socket, where the reference has the thread that enqueues do it: the pipe then never leaves this thread.)
        t->pipe->cnt_cache = 0;
        t->pipe->bytes_cnt = 0;
        t->pipe->pgtoks = t->pgtoks;
        t->pipe->pgtok_cnt = t->pgtok_cnt;
      }
      ncclResult_t res = ncclSuccess;
      const ssize_t bytes = devmem_recv(&fd->sock, t->size, t->offset, t->pipe, static_cast<uint64_t>(t->request_offset), &res);
      if (res != ncclSuccess) {
        t->result = res;
        return res;
      }
      // TCPX_TASK_TP_RECVMSG (src/net_tcpx.cc:167, src/stats/tracepoint.cc:72-82): a recvmsg that finds nothing
      // yet is a possible slowness; the call itself is counted while task-level stats are on.
      if (bytes < 0 && g.slow_switch[kSlowSendRecv] && (errno == EAGAIN || errno == EWOULDBLOCK || errno == EINTR || errno == ENOBUFS)) {
        uint64_t nanos = 0;
        if (t->watch.should_warn(g.clock, &nanos)) {
          FlowData::bump(fd->rx_slow_cnt);
          if (g.slow_report[kSlowSendRecv]) {
            WARN("%p:%p, nic %d, %s, flow %d recv timeout error %d, %s: [%d/%d]/%d cnt %u, nanos %lu", static_cast<void*>(t),
                 static_cast<void*>(comm), comm->dev, g.dev_names[comm->dev], flow, errno, strerror(errno), t->offset, t->size,
                 t->r->size, t->watch.same_count, static_cast<unsigned long>(nanos));
          }
        }
      }
      if (g.task_stats) FlowData::bump(fd->rx_cnt);
      if (bytes > 0) {
        t->offset += static_cast<int>(bytes);
        fd->bytes += static_cast<uint64_t>(bytes);
      }
      if (t->offset == t->size) {
        t->cnt = static_cast<uint32_t>(t->pipe->cnt_cache);
        task_advance(comm, tasks, kTaskActive);  // ACTIVE -> COMPLETING
      }
    }
    if (!tasks->has(kTaskCompleting)) break;  // the active task, if any, is still waiting for bytes
    // The reference asks gpu_inline_test here, which always answers "done" (src/devcomm/nccl/inline.cu:55-60).
    task_advance(comm, tasks, kTaskCompleting);  // COMPLETING -> INACTIVE
  }
  return ncclSuccess;
}

// A pass of the socket thread that found nothing to do: wait a moment without leaving the CPU while work may be
// on its way (tasks arrive every few microseconds under load, and a system call per empty pass costs more than
// that on some machines), give the CPU away once the comm has been quiet for a while.
inline void idle_pass(uint32_t* quiet_passes) {
  if (++*quiet_passes < 4096) {
#if defined(__x86_64__) || defined(__i386__)
    __builtin_ia32_pause();
#endif
  } else {
    sched_yield();
  }
}

void helper_main(Comm* comm) {  // persistentSocketThread, src/net_tcpx.cc:252-384 (receive part)
  // The thread runs on the CPUs bound to its device, all of them (src/net_tcpx.cc:300-307); a refusal (a CPU the
  // process may not use) leaves it where it was.  What it ends up with is kept for tcpxGetCommStats.
  if (g.rx_bound[comm->dev] && sched_setaffinity(0, sizeof(cpu_set_t), &g.rx_cpus[comm->dev]) != 0) {
    WARN("Comm %p dev %d: binding the socket thread failed: %s", static_cast<void*>(comm), comm->dev, strerror(errno));
  }
  cpu_set_t now;
  CPU_ZERO(&now);
  if (sched_getaffinity(0, sizeof now, &now) == 0) comm->helper_cpus.store(static_cast<uint64_t>(CPU_COUNT(&now)), std::memory_order_relaxed);
  uint32_t quiet_passes = 0;
  while (!comm->helper_stop.load(std::memory_order_acquire)) {
    bool idle = true;
    // The same from this side: what the proxy thread has enqueued lies in its CPU's cache.
    for (int f = 0; f < comm->num_flows; ++f) __builtin_prefetch(&comm->flows[f].tasks.entered);
    for (int f = 0; f < comm->num_flows; ++f) {
      TaskRing* tasks = &comm->flows[f].tasks;
      for (uint32_t i = tasks->stage_begin(kTaskActive), end = tasks->stage_end(kTaskActive); i != end; ++i)
        __builtin_prefetch(&tasks->items[i % kMaxTasks]);
    }
    for (int f = 0; f < comm->num_flows; ++f) {
      TaskRing* tasks = &comm->flows[f].tasks;
      if (tasks->has(kTaskActive) || tasks->has(kTaskCompleting)) {
        if (flow_progress(comm, f) != ncclSuccess) return;
        idle = false;
      }
    }
    if (idle) idle_pass(&quiet_passes);
    else quiet_passes = 0;
  }
}

// enqueueTask, src/net_tcpx.cc:1037-1097 (receive part)
void enqueue_task(Comm* comm, Request* r) {
  const int flow = r->next_flow;
  r->next_flow = -1;  // RESET_CTRL
  const int sz = r->next_size;
  TaskRing* tasks = &comm->flows[flow].tasks;
  Task* t = tasks->next_free();
  t->op = static_cast<uint16_t>(r->op);
  t->data = static_cast<char*>(r->data) + r->offset;
  t->r = r;
  t->result = ncclSuccess;
  t->offset = 0;
  t->request_offset = r->offset;
  t->size = sz;
  t->flow = static_cast<uint16_t>(flow);
  t->cnt = 0;
  t->watch.configure(static_cast<uint64_t>(g.timeout_threshold_ns), static_cast<uint64_t>(g.timeout_frequency_ns));
  t->pgtoks = nullptr;
  t->pgtok_cnt = nullptr;
  if (comm->passive) {
    UnpackSlot* u = &r->slot;
    u->flows[flow] = flow;
    t->pgtoks = &u->pgtoks[static_cast<size_t>(flow) * kSlotPages];
    t->pgtok_cnt = &u->pgtok_cnts[flow];
    // Unlike the reference, the count is not zeroed here: a request may put several chunks on the same flow, and
    // every chunk's pages must be given back when the request is consumed.  It is zeroed when the slot is taken.
  }
  tp_task(comm, t, kTaskActiveTs);
  tasks->enqueue();  // FREE -> ACTIVE
  r->offset += sz;
  if (r->size == r->offset) request_advance(comm, kReqActive);  // REQUEST_INACTIVE -> finish_active
}

// Reaps finished tasks: their descriptors move into the request's slot (src/net_tcpx.cc:1119-1151), and the flows
// whose task ring has room are offered to the scheduler.
ncclResult_t reap_tasks(Comm* comm) {
  comm->sched->reset();  // src/net_tcpx.cc:1114
  if (comm->use_helper) {
    // What the socket thread has finished lies in its CPU's cache: the counters first, all flows at once, then every
    // finished task's line and its first descriptors, so that the waits overlap instead of following one another.
    for (int f = 0; f < comm->num_flows; ++f) __builtin_prefetch(&comm->flows[f].tasks.left_[kTaskCompleting]);
    for (int f = 0; f < comm->num_flows; ++f) {
      TaskRing* tasks = &comm->flows[f].tasks;
      for (uint32_t i = tasks->stage_begin(kTaskInactive), end = tasks->stage_end(kTaskInactive); i != end; ++i) {
        __builtin_prefetch(&tasks->items[i % kMaxTasks]);
        __builtin_prefetch(tasks->scatter[i % kMaxTasks]);
      }
    }
  }
  for (int i = 0; i < comm->num_flows; ++i) {
    int idx = comm->end_flow_idx - i;
    if (idx < 0) idx += comm->num_flows;
    TaskRing* tasks = &comm->flows[idx].tasks;
    while (tasks->has(kTaskInactive)) {
      Task* t = tasks->first(kTaskInactive);
      if (t->result != ncclSuccess) return t->result;
      t->r->size_pending -= t->size;
      if (t->op == kOpRecv && t->size > 0) {
        UnpackSlot* u = &t->r->slot;
        if (u->cnt_cache + t->cnt > static_cast<uint64_t>(kSlotPages)) {  // src/net_tcpx.cc:1350-1353
          WARN("request too many pages %lu, failstop", static_cast<unsigned long>(u->cnt_cache + t->cnt));
          return fail_stop("request needs more descriptors than a slot holds");
        }
        memcpy(u->mem + u->cnt_cache, tasks->scatter[t - tasks->items], sizeof(union loadMeta) * t->cnt);
        u->cnt_cache += t->cnt;
      }
      task_advance(comm, tasks, kTaskInactive);  // INACTIVE -> FREE
    }
    // Priority = task slots in use: the emptiest flow is served first (src/net_tcpx.cc:1152-1155).
    if (tasks->has_free()) comm->sched->schedule(idx, kMaxTasks - static_cast<int>(tasks->num_free()));
  }
  return ncclSuccess;
}

ncclResult_t take_control_messages(Comm* comm, bool* enqueued);
ncclResult_t submit_ready_requests(Comm* comm);

// tcpxCommProgress, src/net_tcpx.cc:1099-1308 (receive branch)
ncclResult_t comm_progress(Comm* comm) {
  if (comm->rq.empty()) return ncclSuccess;
  // One call makes up to kProgressPasses passes of: sockets, reap, control messages.  The reference makes one and
  // is called again by the next test(); a pass that has just started tasks is followed by another at once here,
  // because the bytes of a chunk whose control message has been read have usually arrived already and the tasks
  // they finish make room for the next control messages.
  constexpr int kProgressPasses = 4;
  for (int pass = 0; pass < kProgressPasses; ++pass) {
    if (!comm->use_helper) {
      for (int f = 0; f < comm->num_flows; ++f) TCPXCHECK(flow_progress(comm, f));
    }
    TCPXCHECK(reap_tasks(comm));
    TCPXCHECK(submit_ready_requests(comm));
    bool enqueued = false;
    TCPXCHECK(take_control_messages(comm, &enqueued));
    if (!enqueued || comm->use_helper) break;
  }
  return ncclSuccess;
}

ncclResult_t take_control_messages(Comm* comm, bool* enqueued) {
  if (comm->rq.has(kReqPosted)) request_advance(comm, kReqPosted);  // POSTED -> ACTIVE (src/net_tcpx.cc:1158-1180)

  if (!comm->rq.has(kReqActive) || !comm->sched->has_flow()) return ncclSuccess;
  Request* ar = comm->rq.first(kReqActive);
  if (ar->op != kOpRecv) return ncclSuccess;

  do {  // src/net_tcpx.cc:1231-1304
    if (!ctrl_done(ar)) {
      CtrlMessage ctrl;
      bool got_ctrl = false;
      if (comm->ctrl_local.empty()) {  // take over everything that has arrived: one lock per burst, not per message
        std::lock_guard<std::mutex> lock(comm->ctrl_mu);
        comm->ctrl_local.swap(comm->ctrl_rx);
      }
      if (!comm->ctrl_local.empty()) {
        ctrl = comm->ctrl_local.front();
        comm->ctrl_local.pop_front();
        got_ctrl = true;
      }
      // Every look at the control socket counts towards its slowness watch; a message resets it
      // (src/net_tcpx.cc:1234-1246).
      // (A look that finds a message as the first look since the last reset would note the time and be reset again
      // just below: it is skipped, clock read and all.)
      if (g.slow_switch[kSlowRxCtrl] && !(got_ctrl && comm->ctrl_watch.same_count == 0)) {
        uint64_t nanos = 0;
        if (comm->ctrl_watch.should_warn(g.clock, &nanos)) {
          comm->rx_ctrl_slow_cnt++;
          if (g.slow_report[kSlowRxCtrl]) {
            WARN("%p:%p, nic %d, %s, rx ctrl timeout cnt %u, nanos %lu", static_cast<void*>(ar), static_cast<void*>(comm),
                 comm->dev, g.dev_names[comm->dev], comm->ctrl_watch.same_count, static_cast<unsigned long>(nanos));
          }
        }
      }
      if (!got_ctrl) break;
      if (g.slow_switch[kSlowRxCtrl]) comm->ctrl_watch.reset();
      if (ctrl.type != TCPX_CTRL_INLINE && ctrl.index >= comm->num_flows) {
        WARN("control message names flow %u, comm has %d", ctrl.index, comm->num_flows);
        return ncclInternalError;
      }
      if (ctrl.type != TCPX_CTRL_INLINE) FlowData::bump(comm->flows[ctrl.index].rx_ctrl_done_cnt);
      // What the peer announces decides which bytes of the receive buffer the GPU will write.  The reference takes
      // both numbers as they come (src/net_tcpx.cc:995-1010) and a wrong one ends in a device error there; here a
      // message longer than the posted receive, or a chunk that runs past the message's end, is refused before any
      // descriptor is built from it.
      if (ar->size_pending < 0 && ctrl.total > static_cast<uint32_t>(ar->posted_size)) {
        WARN("control message announces %u bytes for a receive of %d posted", ctrl.total, ar->posted_size);
        return ncclInternalError;
      }
      const int64_t message = ar->size_pending < 0 ? static_cast<int64_t>(ctrl.total) : ar->size;
      if (ctrl.type != TCPX_CTRL_INLINE && static_cast<int64_t>(ar->offset) + ctrl.size > message) {
        WARN("control message: chunk of %u bytes at %d runs past the message's %ld", ctrl.size, ar->offset, static_cast<long>(message));
        return ncclInternalError;
      }
      ar->next_flow = ctrl.index;  // tcpxCtrlRecv, src/net_tcpx.cc:995-1014
      ar->next_size = static_cast<int>(ctrl.size);
      if (ar->size_pending < 0) ar->size_pending = ar->size = static_cast<int>(ctrl.total);

      if (ctrl.type == TCPX_CTRL_INLINE) {  // src/net_tcpx.cc:1248-1276: an empty message still takes a slot
        unpack_queue_next_free(comm->queue, &ar->slot);
        if (!ar->slot.active) {
          WARN("no more unpack queue slot, head %lu tail %lu", static_cast<unsigned long>(comm->queue->head),
               static_cast<unsigned long>(comm->queue->tail));
          // The control message is consumed and cannot be re-read: put it back so that a later poll retries.
          comm->ctrl_local.push_front(ctrl);
          ar->next_flow = -1;
          break;
        }
        comm->queue->meta->nccl.cnt[ar->slot.idx] = 0;
        comm->queue->record.flow_cnts[ar->slot.idx] = 0;
        if (ar->size) {
          WARN("payload through the control socket is not supported for device memory");
          return ncclInternalError;
        }
        request_advance(comm, kReqActive);  // -> TRANSMITTING
        break;
      }
    }

    if (ar->slot.cnt == nullptr) {  // first chunk of the request: take a slot (src/net_tcpx.cc:1279-1296)
      unpack_queue_next_free(comm->queue, &ar->slot);
      if (!ar->slot.active) {
        WARN("no more unpack queue slot, head %lu tail %lu", static_cast<unsigned long>(comm->queue->head),
             static_cast<unsigned long>(comm->queue->tail));
        break;  // the pending control message stays in the request; retried at the next poll
      }
      *ar->slot.cnt = 0;
      ar->slot.cnt_cache = 0;
      *ar->slot.flow_cnt = static_cast<size_t>(comm->num_flows);
      memset(ar->slot.pgtok_cnts, 0, kMaxFlows * sizeof(size_t));
    }
    TaskRing* tasks = &comm->flows[ar->next_flow].tasks;
    if (!tasks->has_free()) break;  // "No free space for recv task": retried at the next poll
    comm->end_flow_idx = ar->next_flow;
    enqueue_task(comm, ar);
    *enqueued = true;
  } while (ar->offset < ar->size);
  return ncclSuccess;
}

// recyclePages, src/sock/tcpx.h:310-326
ncclResult_t recycle_pages(Comm* comm, uint64_t q_idx) {
  UnpackQueue* q = comm->queue;
  q_idx %= kQueueDepth;
  const size_t n_flows = q->record.flow_cnts[q_idx];
  for (size_t i = 0; i < n_flows; ++i) {
    const size_t n = q->record.pgtok_cnts[q_idx][i];
    if (n > 0) {
      const int flow = q->record.flows[q_idx][i];
      if (comm->flows[flow].sock.dontneed(q->record.pgtoks[q_idx][i], n) != 0) {
        WARN("page recycle failed on flow %d", flow);
        return ncclInternalError;
      }
    }
  }
  return ncclSuccess;
}

ncclResult_t ensure_engine(DeviceState* ds) {
  std::lock_guard<std::mutex> lock(ds->mu);
  if (!ds->engine) {
    tcpxuEngineConfig cfg{};
    TCPXCHECK(device_result(g.ops->engine_create(ds->dev, &cfg, &ds->engine), "engine_create"));
  }
  if (!ds->engine_started) {
    TCPXCHECK(device_result(g.ops->engine_start(ds->engine), "engine_start"));
    ds->engine_started = true;
  }
  return ncclSuccess;
}


// Publishes a completed receive request's descriptor count and hands its slot to the engine (device type "host").
// The count and the release are the reference's publish (src/net_tcpx.cc:1350-1357); the submission is this
// build's doorbell.  *submitted stays false when the engine's submission ring is full: the caller tries again at
// the next poll.
ncclResult_t publish_to_engine(Comm* comm, Request* r, bool* submitted) {
  *submitted = false;
  UnpackQueue* q = comm->queue;
  if (r->slot.cnt_cache > static_cast<uint64_t>(kSlotPages)) {  // src/net_tcpx.cc:1350-1353
    WARN("request too many pages %lu, failstop", static_cast<unsigned long>(r->slot.cnt_cache));
    return fail_stop("request needs more descriptors than a slot holds");
  }
  *r->slot.cnt = r->slot.cnt_cache;
  std::atomic_thread_fence(std::memory_order_release);
  q->meta->done[r->slot.idx].value = 0;
  r->done_value = ++comm->done_seq;
  // The descriptors the engine reads: the mapped slot, or -- for a small request, of which a comm has at
  // most 16 in flight -- a second copy in the GPU's own memory, written through the BAR ahead of the
  // submission, which saves the GPU a PCIe round trip before it can start copying.
  const void* descs_dev = q->meta_dev->nccl.mem[r->slot.idx];
  if (q->stage && r->slot.cnt_cache <= kStagedDescs) {
    union loadMeta* copy = q->stage + r->slot.idx * kStagedDescs;
    memcpy(copy, r->slot.mem, sizeof(union loadMeta) * r->slot.cnt_cache);
    g.ops->visible_flush();
    descs_dev = q->stage_dev + r->slot.idx * kStagedDescs;
  }
  // The request's size goes along as a hint (it sizes the engine's tickets for fragments shorter than a page).
  const uint32_t n_descs = static_cast<uint32_t>(r->slot.cnt_cache);
  void* done_flag = &q->meta_dev->done[r->slot.idx].value;
  const int rc = g.ops->engine_submit_sized
                     ? g.ops->engine_submit_sized(comm->device->engine, comm->device->arena, r->data, descs_dev, n_descs,
                                                  static_cast<uint64_t>(r->offset), done_flag, r->done_value)
                     : g.ops->engine_submit(comm->device->engine, comm->device->arena, r->data, descs_dev, n_descs,
                                            done_flag, r->done_value);
  if (rc == TCPXU_IN_PROGRESS) {  // submission ring full
    --comm->done_seq;
    return ncclSuccess;
  }
  TCPXCHECK(device_result(rc, "engine_submit"));
  r->published = true;
  r->published_ns = g.clock();
  r->unpack_watch.configure(static_cast<uint64_t>(g.timeout_threshold_ns), static_cast<uint64_t>(g.timeout_frequency_ns));
  comm->unpack_cnt++;
  comm->slots_at_gpu++;
  comm->max_slots_at_gpu = std::max(comm->max_slots_at_gpu, comm->slots_at_gpu);
  *submitted = true;
  return ncclSuccess;
}

// Device type "host": every request whose last byte has been accounted for goes to the engine at once, oldest
// first, whether or not the caller has come to test it yet.  The reference reports done=1 at publish
// (src/net_tcpx.cc:1354-1370), so that up to sixteen slots of a comm are with the consumer together
// (src/devcomm/nccl/unpack1.h:30-65); here done=1 waits for the copy, and submitting ahead of the test is what
// keeps that many slots at the GPU.  Completion is still reported strictly in posting order, by tcpxTest.
ncclResult_t submit_ready_requests(Comm* comm) {
  if (g.device_type != kDeviceHost) return ncclSuccess;
  for (uint32_t i = comm->rq.stage_begin(kReqTransmitting), end = comm->rq.stage_end(kReqTransmitting); i != end; ++i) {
    Request* r = &comm->rq.items[i % kMaxRequests];
    if (r->published || r->op != kOpRecv || r->size == 0 || !request_done(r)) continue;
    bool submitted = false;
    TCPXCHECK(publish_to_engine(comm, r, &submitted));
    if (!submitted) break;  // ring full: the younger ones wait behind this one
  }
  return ncclSuccess;
}

}  // namespace

int sched_alg_from_name(const char* name, bool* valid) {
  const bool rr = name && strcmp(name, "RR") == 0, katy = name && strcmp(name, "KATY") == 0;
  if (valid) *valid = rr || katy;
  return katy ? kSchedKaty : kSchedRoundRobin;
}

void ctrl_send_batch(Comm* comm, const CtrlMessage* messages, size_t n) {
  std::lock_guard<std::mutex> lock(comm->ctrl_mu);
  comm->ctrl_rx.insert(comm->ctrl_rx.end(), messages, messages + n);
}

ncclResult_t deliver_fragments(Comm* comm, uint32_t flow, const tcpxSynthFrag* frags, uint32_t n_frags) {
  const size_t arena = comm->device->arena_bytes;
  for (uint32_t i = 0; i < n_frags; ++i) {
    const tcpxSynthFrag& f = frags[i];
    // The devmem contract: a fragment lies inside the arena and inside one 4 KiB page.
    if (static_cast<size_t>(f.frag_offset) + f.frag_size > arena ||
        (f.frag_offset % SLICE_PAGE_SIZE) + f.frag_size > SLICE_PAGE_SIZE) {
      WARN("fragment %u (offset %u, size %u) breaks the devmem contract", i, f.frag_offset, f.frag_size);
      return ncclInvalidArgument;
    }
  }
  comm->flows[flow].sock.push(frags, n_frags);
  return ncclSuccess;
}

FlowScheduler* new_flow_scheduler(int alg) {
  if (alg == kSchedKaty) return new KatyFlows(kMaxFlows, kMaxTasks);
  return new RoundRobinFlows;
}
}  // namespace tcpx

using namespace tcpx;

extern "C" {

ncclResult_t tcpxSetDeviceOpsForTesting(const tcpxDeviceOps* ops) {
  std::lock_guard<std::mutex> lock(g.mu);
  if (g.initialized) return ncclInvalidUsage;
  g.ops = ops;
  g.ops_injected = ops != nullptr;
  return ncclSuccess;
}

ncclResult_t tcpxSetFailStopForTesting(int enabled) {
  g.fail_stop = enabled != 0;
  return ncclSuccess;
}

ncclResult_t tcpxInit(ncclDebugLogger_t logFunction) {
  std::lock_guard<std::mutex> lock(g.mu);
  g.logger = logFunction;
  if (g.initialized) return ncclSuccess;
  // Flags start from their defaults at every initialisation (a process may finalise and initialise again).
  g.flows_per_comm = 4;
  g.use_helper_thread = 0;
  g.timeout_threshold_ns = 10000000000LL;
  g.timeout_frequency_ns = 30000000000LL;
  g.task_stats = g.request_stats = 0;
  g.sampling_factor = 1;
  int_flag(&g.flows_per_comm, "AMD_FLOWS", 1, kMaxFlows);
  int_flag(&g.use_helper_thread, "AMD_HELPER_THREAD", 0, 1);
  int64_flag(&g.timeout_threshold_ns, "TIMEOUT_THRESHOLD_NS", 100 * 1000);  // src/net_tcpx.cc:519-524
  int64_flag(&g.timeout_frequency_ns, "TIMEOUT_FREQUENCY_NS", 100 * 1000);
  int_flag(&g.task_stats, "TELEMETRY_ENABLE_TASK_LEVEL_STATS", 0, 1);
  int_flag(&g.request_stats, "TELEMETRY_ENABLE_REQUEST_LEVEL_STATS", 0, 1);
  int_flag(&g.sampling_factor, "TELEMETRY_SAMPLING_FACTOR", 1, INT_MAX - 1);
  parse_slowness_flags();
  parse_sched_alg();
  parse_device_type();
  if (!g.ops_injected) {
    g.ops = default_device_ops();
    if (!g.ops) {
      WARN("the HIP layer is not available: this plugin has no other way to move data");
      return ncclSystemError;
    }
  }
  int n = 0;
  TCPXCHECK(device_result(g.ops->device_count(&n), "device_count"));
  if (n <= 0) {
    WARN("no GPU visible");
    return ncclSystemError;
  }
  g.n_devices = std::min(n, kMaxDevices);
  for (int d = 0; d < g.n_devices; ++d) {
    g.devices[d].dev = d;
    snprintf(g.dev_names[d], sizeof g.dev_names[d], "tcpx-amd-synth%d", d);
    snprintf(g.pci_paths[d], sizeof g.pci_paths[d], "/sys/class/net/tcpx-amd-synth%d/device", d);
  }
  parse_rx_bindings();
  g.initialized = true;
  INFO(NCCL_INIT | NCCL_NET, "NET/GPUDirectTCPX-AMD initialised: %d device(s), %d flows per comm", g.n_devices,
       g.flows_per_comm);
  return ncclSuccess;
}

ncclResult_t tcpxFinalize(void) {
  std::lock_guard<std::mutex> lock(g.mu);
  if (!g.initialized) return ncclSuccess;
  ncclResult_t rc = ncclSuccess;
  for (int d = 0; d < g.n_devices; ++d) {
    DeviceState* ds = &g.devices[d];
    std::lock_guard<std::mutex> dl(ds->mu);
    if (ds->comms != 0) {
      WARN("device %d still has %d open comm(s)", d, ds->comms);
      rc = ncclInvalidUsage;
      continue;
    }
    // Stop the persistent kernel first: nothing may be freed underneath it.
    if (ds->engine) {
      if (ds->engine_started && g.ops->engine_stop(ds->engine, nullptr) != TCPXU_SUCCESS) rc = ncclInternalError;
      ds->engine_started = false;
      if (g.ops->engine_destroy(ds->engine) != TCPXU_SUCCESS) rc = ncclInternalError;
      ds->engine = nullptr;
    }
    for (QueueBlock& b : ds->free_blocks) {
      g.ops->mapped_free(d, b.meta);
      g.ops->device_free(d, b.dev_handle);
      if (b.stage && g.ops->visible_free) g.ops->visible_free(d, b.stage);
    }
    ds->free_blocks.clear();
    if (ds->arena) g.ops->arena_destroy(d, ds->arena);
    ds->arena = nullptr;
    ds->arena_bytes = 0;
    ds->page_refs.reset();
    ds->n_pages = 0;
    ds->pages_outstanding = 0;
  }
  if (rc == ncclSuccess) g.initialized = false;
  return rc;
}

ncclResult_t tcpxDevices(int* ndev) {
  std::lock_guard<std::mutex> lock(g.mu);
  *ndev = g.n_devices;
  return ncclSuccess;
}

ncclResult_t tcpxGetProperties(int dev, ncclNetProperties_v7_t* props) {
  if (dev < 0 || dev >= g.n_devices || !props) return ncclInternalError;
  props->name = g.dev_names[dev];
  props->pciPath = g.pci_paths[dev];
  props->guid = static_cast<uint64_t>(dev);
  props->ptrSupport = NCCL_PTR_HOST | NCCL_PTR_CUDA;
  props->speed = 10000;  // the reference's fallback when sysfs has no speed (src/net_tcpx.cc:717-721)
  props->port = 0;
  props->maxComms = 65536;
  props->latency = 0;
  props->maxRecvs = 1;
  if (g.device_type == kDeviceUnpack) {  // src/net_tcpx.cc:739-740
    props->netDeviceType = NCCL_NET_DEVICE_UNPACK;
    props->netDeviceVersion = NCCL_NET_DEVICE_UNPACK_VERSION;
  } else {  // the engine owns the copy: nothing for a consumer kernel to do
    props->netDeviceType = NCCL_NET_DEVICE_HOST;
    props->netDeviceVersion = NCCL_NET_DEVICE_INVALID_VERSION;
  }
  return ncclSuccess;
}

ncclResult_t tcpxSynthArenaCreate(int dev, size_t bytes, void** base) {
  if (!g.initialized || dev < 0 || dev >= g.n_devices || !base) return ncclInvalidArgument;
  DeviceState* ds = &g.devices[dev];
  std::lock_guard<std::mutex> lock(ds->mu);
  if (ds->arena) {
    WARN("device %d already has an arena", dev);
    return ncclInvalidUsage;
  }
  TCPXCHECK(device_result(g.ops->arena_create(dev, bytes, &ds->arena), "arena_create"));
  ds->arena_bytes = bytes;
  ds->n_pages = bytes / SLICE_PAGE_SIZE;
  ds->page_refs.reset(new std::atomic<int32_t>[ds->n_pages]);
  for (size_t i = 0; i < ds->n_pages; ++i) ds->page_refs[i] = 0;
  ds->pages_outstanding = 0;
  *base = ds->arena;
  return ncclSuccess;
}

ncclResult_t tcpxListen(int dev, void* handle, void** listenComm) {
  if (!g.initialized || dev < 0 || dev >= g.n_devices || !handle || !listenComm) return ncclInternalError;
  static std::atomic<uint64_t> next_id{1};
  ListenComm* l = new (std::nothrow) ListenComm;
  if (!l) return ncclSystemError;
  l->dev = dev;
  l->id = next_id.fetch_add(1);
  l->backlog.store(0);
  ConnectHandle h{kConnectMagic, l->id, dev};
  memset(handle, 0, NCCL_NET_HANDLE_MAXSIZE);
  memcpy(handle, &h, sizeof h);  // the connect handle: which listener, on which device
  {
    std::lock_guard<std::mutex> lock(g.listen_mu);
    g.listeners.push_back(l);
  }
  *listenComm = l;
  return ncclSuccess;
}

static ncclResult_t new_comm(int dev, bool passive, Comm** out) {
  Comm* c = new (std::nothrow) Comm;
  if (!c) return ncclSystemError;
  c->passive = passive;
  c->dev = dev;
  c->device = &g.devices[dev];
  c->num_flows = g.flows_per_comm;
  c->use_helper = g.use_helper_thread != 0;
  c->sched.reset(new_flow_scheduler(g.sched_alg));  // src/net_tcpx.cc:1101-1112 (there: at the first progress call)
  for (int f = 0; f < kMaxFlows; ++f) c->flows[f].sock.device = c->device;
  c->ctrl_watch.configure(static_cast<uint64_t>(g.timeout_threshold_ns), static_cast<uint64_t>(g.timeout_frequency_ns));
  if (g.task_stats || g.request_stats) c->trace.reset(new TraceBuffer(kTraceEvents));
  *out = c;
  return ncclSuccess;
}

ncclResult_t tcpxConnect_v5(int dev, void* handle, void** sendComm, ncclNetDeviceHandle_v7_t** sendDevHandle) {
  if (!g.initialized || dev < 0 || dev >= g.n_devices || !handle || !sendComm) return ncclInternalError;
  // The sending side is outside this build (no NIC, no sockets): the comm exists so that the call sequence of a
  // real job can be replayed, but tcpxIsend_v5 on it reports an error.  What connect does do is what a TCP
  // connect does to a listening socket: it finds the listener the handle names and joins its backlog, where
  // accept will find it; a handle that names no open listener is "connection refused".
  ConnectHandle h;
  memcpy(&h, handle, sizeof h);
  if (h.magic != kConnectMagic) {
    WARN("connect: the handle was not written by tcpxListen");
    return ncclInternalError;
  }
  Comm* c = nullptr;
  TCPXCHECK(new_comm(dev, false, &c));
  {
    std::lock_guard<std::mutex> lock(g.listen_mu);
    ListenComm* l = nullptr;
    for (ListenComm* x : g.listeners)
      if (x->id == h.id) l = x;
    if (!l) {
      WARN("connect: listener %lu is not open (connection refused)", static_cast<unsigned long>(h.id));
      delete c;
      return ncclSystemError;
    }
    l->backlog.fetch_add(1, std::memory_order_release);
  }
  *sendComm = c;
  (void)sendDevHandle;  // the sending side has no device handle (src/net_tcpx.cc:754-759)
  return ncclSuccess;
}

ncclResult_t tcpxAccept_v5(void* listenComm, void** recvComm, ncclNetDeviceHandle_v7_t** recvDevHandle) {
  if (!g.initialized || !listenComm || !recvComm) return ncclInternalError;
  ListenComm* l = static_cast<ListenComm*>(listenComm);
  DeviceState* ds = &g.devices[l->dev];
  *recvComm = nullptr;
  // Nobody has connected yet: success with no comm, and the caller asks again (the reference's accept is
  // non-blocking in the same way, which is why src/net_tcpx.cc:764 looks at *recvComm before using it).
  uint32_t waiting = l->backlog.load(std::memory_order_acquire);
  do {
    if (waiting == 0) return ncclSuccess;
  } while (!l->backlog.compare_exchange_weak(waiting, waiting - 1, std::memory_order_acq_rel));
  if (!ds->arena) {
    WARN("device %d has no bounce arena: call tcpxSynthArenaCreate first", l->dev);
    l->backlog.fetch_add(1, std::memory_order_release);  // the connection stays in the backlog
    return ncclInternalError;
  }
  Comm* c = nullptr;
  ncclResult_t rc = new_comm(l->dev, true, &c);
  if (rc != ncclSuccess) {
    l->backlog.fetch_add(1, std::memory_order_release);  // the connection stays in the backlog
    return rc;
  }
  rc = g.device_type == kDeviceHost ? ensure_engine(ds) : ncclSuccess;
  if (rc == ncclSuccess) rc = unpack_queue_new(l->dev, true, &c->queue);  // tcpxGetDeviceHandle, src/net_tcpx.cc:1452-1471
  if (rc != ncclSuccess) {
    delete c;
    l->backlog.fetch_add(1, std::memory_order_release);
    return rc;
  }
  {
    std::lock_guard<std::mutex> lock(ds->mu);
    ds->comms++;
  }
  if (c->use_helper) c->helper = std::thread(helper_main, c);
  if (recvDevHandle && *recvDevHandle) {
    ncclNetDeviceHandle_v7_t* h = *recvDevHandle;
    if (g.device_type == kDeviceUnpack) {  // src/net_tcpx.cc:1463-1467
      h->netDeviceType = NCCL_NET_DEVICE_UNPACK;
      h->netDeviceVersion = NCCL_NET_DEVICE_UNPACK_VERSION;
      h->handle = c->queue->dev_handle;
      h->size = sizeof(struct unpackNetDeviceHandle);
      h->needsProxyProgress = 1;
    } else {  // nothing for a device-side consumer: the queue is this plugin's own business
      h->netDeviceType = NCCL_NET_DEVICE_HOST;
      h->netDeviceVersion = NCCL_NET_DEVICE_INVALID_VERSION;
      h->handle = nullptr;
      h->size = 0;
      h->needsProxyProgress = 0;
    }
  }
  *recvComm = c;
  return ncclSuccess;
}

ncclResult_t tcpxRegMr(void* ocomm, void* data, int size, int type, void** mhandle) {
  if (ocomm == nullptr) {
    WARN("regMr called with NULL communicator.");
    return ncclInternalError;
  }
  if (type != NCCL_PTR_HOST && type != NCCL_PTR_CUDA) {
    WARN("unknown mem type %d", type);
    return ncclInternalError;
  }
  MemHandle* m = static_cast<MemHandle*>(calloc(1, sizeof *m));
  if (!m) return ncclSystemError;
  m->ptr = data;
  m->size = size < 0 ? 0 : static_cast<size_t>(size);  // the registered range bounds what a receive may write (get_request)
  m->mem_type = type;
  *mhandle = m;
  return ncclSuccess;
}

ncclResult_t tcpxDeregMr(void* ocomm, void* mhandle) {
  (void)ocomm;
  free(mhandle);  // NULL is fine (src/net_tcpx.cc:828)
  return ncclSuccess;
}

ncclResult_t tcpxGetDeviceMr(void* comm, void* mhandle, void** dptr_mhandle) {
  (void)comm;
  (void)mhandle;
  (void)dptr_mhandle;
  return ncclSuccess;
}

// tcpxGetRequest, src/net_tcpx.cc:862-896
static ncclResult_t get_request(Comm* comm, int op, void* data, int size, MemHandle* mh, Request** req) {
  if (mh == nullptr) {
    WARN("mhandle is null");
    return ncclInternalError;
  }
  // A receive lies inside the memory its handle registered.  (The reference does not look,
  // src/net_tcpx.cc:862-896; here whatever the request names is what the GPU writes.)
  if (op == kOpRecv) {
    const uintptr_t lo = reinterpret_cast<uintptr_t>(mh->ptr), at = reinterpret_cast<uintptr_t>(data);
    if (size < 0 || at < lo || at - lo > mh->size || static_cast<size_t>(size) > mh->size - (at - lo)) {
      WARN("receive of %d bytes at %p lies outside its registration [%p, +%zu)", size, data, mh->ptr, mh->size);
      return ncclInternalError;
    }
  }
  if (!comm->rq.has_free()) {
    WARN("unable to allocate requests");
    return ncclInternalError;
  }
  Request* r = comm->rq.next_free();
  r->op = op;
  r->mem_type = mh->mem_type;
  r->next_flow = -1;
  r->next_size = 0;
  r->data = data;
  r->offset = 0;
  r->size = size;
  r->posted_size = size;
  r->size_pending = op == kOpSend ? size : -1;
  r->comm = comm;
  r->slot = UnpackSlot{};  // cnt == nullptr: no slot yet
  r->published = false;
  r->done_value = 0;
  *req = r;
  tp_request(comm, r, kReqActiveTs);  // the reference names the enqueue tracepoint "active" (src/work_queue.h:189-192)
  comm->rq.enqueue();  // FREE -> POSTED
  return ncclSuccess;
}

ncclResult_t tcpxIsend_v5(void* sendComm, void* data, int size, int tag, void* mhandle, void** request) {
  (void)sendComm, (void)data, (void)size, (void)tag, (void)mhandle;
  if (request) *request = nullptr;
  WARN("isend: the sending side is not part of this build (no NIC, no sockets)");
  return ncclInternalError;
}

ncclResult_t tcpxIrecv_v5(void* recvComm, int n, void** data, int* sizes, int* tags, void** mhandles, void** request) {
  (void)tags;
  Comm* comm = static_cast<Comm*>(recvComm);
  if (n != 1) return ncclInternalError;
  if (!comm || !comm->passive) return ncclInternalError;
  Request* r = nullptr;
  TCPXCHECK(get_request(comm, kOpRecv, data[0], sizes[0], static_cast<MemHandle*>(mhandles[0]), &r));
  *request = r;
  return ncclSuccess;
}

ncclResult_t tcpxIflush_v5(void* recvComm, int n, void** data, int* sizes, void** mhandles, void** request) {
  (void)recvComm, (void)data, (void)mhandles;
  // "Iflush unused for now" (src/net_tcpx.cc:946-954): the slot the caller passes still holds the receive
  // request, whose size is echoed; no flush request is created and no work is done.
  if (n != 1) return ncclInternalError;
  if (request && request[0] && sizes) sizes[0] = static_cast<Request*>(request[0])->size;
  return ncclSuccess;
}

ncclResult_t tcpxTest(void* request, int* done, int* size) {
  (void)size;  // never written, as in the reference
  *done = 0;
  Request* r = static_cast<Request*>(request);
  if (r == nullptr) {
    WARN("test called with NULL request");
    return ncclInternalError;
  }
  Comm* comm = r->comm;
  TCPXCHECK(comm_progress(comm));
  if (!comm->rq.has(kReqTransmitting)) return ncclSuccess;
  Request* ni = comm->rq.first(kReqTransmitting);
  if (r != ni) {  // requests complete in the order they were posted (src/net_tcpx.cc:1322-1328)
    WARN("test called with invalid request, r %p, ni %p", static_cast<void*>(r), static_cast<void*>(ni));
    return ncclInternalError;
  }
  if (!request_done(r)) return ncclSuccess;
  if (r->op == kOpRecv) {
    if (r->size) {
      UnpackQueue* q = comm->queue;
      if (g.device_type == kDeviceUnpack) {
        if (r->slot.cnt_cache > static_cast<uint64_t>(kSlotPages)) {  // src/net_tcpx.cc:1350-1353
          WARN("request too many pages %lu, failstop", static_cast<unsigned long>(r->slot.cnt_cache));
          return fail_stop("request needs more descriptors than a slot holds");
        }
        // The reference's publish and nothing else (src/net_tcpx.cc:1354-1357): the count, a release, and the store
        // fence that pushes it out of the write-combining buffers; whoever holds the device handle copies.  done=1
        // means "published".
        *r->slot.cnt = r->slot.cnt_cache;
        std::atomic_thread_fence(std::memory_order_release);
        __builtin_ia32_sfence();
        comm->unpack_cnt++;
        request_advance(comm, kReqTransmitting);
        *done = 1;
        return ncclSuccess;
      }
      // The progress call above has submitted the slot, unless the engine's submission ring was full.
      if (!r->published) return ncclSuccess;
      const uint64_t seen =
          reinterpret_cast<std::atomic<uint64_t>*>(&q->meta->done[r->slot.idx].value)->load(std::memory_order_acquire);
      if (seen != r->done_value) {  // the GPU is still copying
        uint64_t nanos = 0;
        if (g.slow_switch[kSlowUnpack] && r->unpack_watch.should_warn(g.clock, &nanos)) {
          comm->unpack_slow_cnt++;
          if (g.slow_report[kSlowUnpack]) {
            WARN("%p:%p, gpu %d, unpack timeout: slot %lu (%lu descriptors, %d bytes) submitted, completion word %lu, expected %lu, "
                 "queue head %lu tail %lu, cnt %u, nanos %lu",
                 static_cast<void*>(r), static_cast<void*>(comm), comm->dev, static_cast<unsigned long>(r->slot.idx),
                 static_cast<unsigned long>(r->slot.cnt_cache), r->size, static_cast<unsigned long>(seen),
                 static_cast<unsigned long>(r->done_value), static_cast<unsigned long>(q->head),
                 static_cast<unsigned long>(q->tail), r->unpack_watch.same_count, static_cast<unsigned long>(nanos));
          }
        }
        return ncclSuccess;
      }
      comm->slots_at_gpu--;
      comm->unpack_ns += g.clock() - r->published_ns;
    } else {
      *r->slot.cnt = 0;  // src/net_tcpx.cc:1361
    }
  }
  request_advance(comm, kReqTransmitting);  // -> INACTIVE
  *done = 1;
  return ncclSuccess;
}

ncclResult_t tcpxIrecvConsumed(void* ocomm, int n, void* request) {
  if (request == nullptr) {
    WARN("irecvConsumed with null request");
    return ncclInternalError;
  }
  if (n != 1) return ncclInternalError;
  Comm* comm = static_cast<Comm*>(ocomm);
  UnpackQueue* q = comm->queue;
  Request* r = static_cast<Request*>(request);
  if (r->op == kOpSend) {
    WARN("irecvConsumed called for send request %p", request);
    return ncclSuccess;
  }
  if (!r->size) {  // skip empty (src/net_tcpx.cc:1500-1504)
    request_advance(comm, kReqInactive);
    q->head += 1;
    return ncclSuccess;
  }
  if (!r->slot.active) {
    WARN("irecvConsumed called with r %p ->size %d inactive unpack slot", request, r->size);
    return ncclInternalError;
  }
  if (!comm->rq.has(kReqInactive)) {
    WARN("irecvConsumed called with %p when no inactive request", request);
    return ncclInternalError;
  }
  Request* ir = comm->rq.first(kReqInactive);
  if (ir != r) {
    WARN("irecvConsumed called with invalid request %p vs expected %p", request, static_cast<void*>(ir));
    return ncclInternalError;
  }
  const uint64_t q_idx = ir->slot.idx;
  if (q->head == q->tail) {
    WARN("irecvConsumed shouldn't be called when head == tail == %lu", static_cast<unsigned long>(q->head));
    return ncclInternalError;
  }
  if (q->head % kQueueDepth != q_idx) {
    WARN("irecvConsumed unexpected q_idx %lu vs head %lu", static_cast<unsigned long>(q_idx),
         static_cast<unsigned long>(q->head));
    return ncclInternalError;
  }
  TCPXCHECK(recycle_pages(comm, q_idx));
  request_advance(comm, kReqInactive);  // INACTIVE -> FREE
  q->head += 1;
  return ncclSuccess;
}

ncclResult_t tcpxClose(void* oComm) {
  Comm* comm = static_cast<Comm*>(oComm);
  if (!comm) return ncclSuccess;
  if (comm->helper.joinable()) {
    comm->helper_stop.store(true, std::memory_order_release);
    comm->helper.join();
  }
  if (comm->queue) {
    if (comm->queue->head != comm->queue->tail)  // src/net_tcpx.cc:1385-1390
      WARN("head %lu tail %lu some pages not yet freed?", static_cast<unsigned long>(comm->queue->head),
           static_cast<unsigned long>(comm->queue->tail));
    unpack_queue_free(comm->queue);
    std::lock_guard<std::mutex> lock(comm->device->mu);
    comm->device->comms--;
  }
  delete comm;
  return ncclSuccess;
}

ncclResult_t tcpxCloseListen(void* oComm) {
  ListenComm* l = static_cast<ListenComm*>(oComm);
  if (!l) return ncclSuccess;
  {
    std::lock_guard<std::mutex> lock(g.listen_mu);
    g.listeners.erase(std::remove(g.listeners.begin(), g.listeners.end(), l), g.listeners.end());
  }
  delete l;
  return ncclSuccess;
}

// ---- synthetic socket and inspection ------------------------------------------------------------------------------

ncclResult_t tcpxSynthCtrlSend(void* recvComm, uint16_t type, uint16_t flow, uint32_t size, uint32_t offset,
                               uint32_t total) {
  Comm* comm = static_cast<Comm*>(recvComm);
  if (!comm || !comm->passive || type > TCPX_CTRL_INLINE) return ncclInvalidArgument;
  std::lock_guard<std::mutex> lock(comm->ctrl_mu);
  comm->ctrl_rx.push_back(CtrlMessage{type, flow, size, offset, total});
  return ncclSuccess;
}

ncclResult_t tcpxSynthDeliver(void* recvComm, uint32_t flow, const tcpxSynthFrag* frags, uint32_t n_frags) {
  Comm* comm = static_cast<Comm*>(recvComm);
  if (!comm || !comm->passive || flow >= static_cast<uint32_t>(comm->num_flows) || (!frags && n_frags)) return ncclInvalidArgument;
  return deliver_fragments(comm, flow, frags, n_frags);
}

ncclResult_t tcpxSynthSetRecvmsgLimit(void* recvComm, uint32_t max_frags_per_recvmsg) {
  Comm* comm = static_cast<Comm*>(recvComm);
  if (!comm) return ncclInvalidArgument;
  for (int f = 0; f < kMaxFlows; ++f) comm->flows[f].sock.max_frags_per_recvmsg.store(max_frags_per_recvmsg, std::memory_order_relaxed);
  return ncclSuccess;
}

ncclResult_t tcpxSynthOutstandingPages(void* recvComm, uint64_t* pages) {
  Comm* comm = static_cast<Comm*>(recvComm);
  if (!comm || !pages) return ncclInvalidArgument;
  *pages = comm->device->pages_outstanding.load();
  return ncclSuccess;
}

ncclResult_t tcpxDebugQueueState(void* recvComm, uint64_t* head, uint64_t* tail, uint32_t request_idx[5]) {
  Comm* comm = static_cast<Comm*>(recvComm);
  if (!comm || !comm->queue) return ncclInvalidArgument;
  if (head) *head = comm->queue->head;
  if (tail) *tail = comm->queue->tail;
  if (request_idx) {
    // In the order of the reference's idx[]: [0] dequeue cursor, [1] left TRANSMITTING, [2] left ACTIVE,
    // [3] left POSTED, [4] enqueue cursor.
    request_idx[0] = comm->rq.stage_begin(kReqInactive);
    request_idx[1] = comm->rq.stage_begin(kReqTransmitting);
    request_idx[2] = comm->rq.stage_begin(kReqActive);
    request_idx[3] = comm->rq.stage_begin(kReqPosted);
    request_idx[4] = comm->rq.entered;
  }
  return ncclSuccess;
}

ncclResult_t tcpxDebugSlot(void* recvComm, uint32_t slot_idx, const union loadMeta** descs, uint64_t* cnt) {
  Comm* comm = static_cast<Comm*>(recvComm);
  if (!comm || !comm->queue || slot_idx >= static_cast<uint32_t>(kQueueDepth)) return ncclInvalidArgument;
  if (descs) *descs = comm->queue->meta->nccl.mem[slot_idx];
  if (cnt) *cnt = comm->queue->meta->nccl.cnt[slot_idx];
  return ncclSuccess;
}

ncclResult_t tcpxGetFlowStats(void* recvComm, uint32_t flow, tcpxFlowStats* stats) {
  Comm* comm = static_cast<Comm*>(recvComm);
  if (!comm || !stats || flow >= static_cast<uint32_t>(comm->num_flows)) return ncclInvalidArgument;
  const FlowData* fd = &comm->flows[flow];
  stats->flow_id = flow;
  stats->rx_ctrl_done_cnt = fd->rx_ctrl_done_cnt.load(std::memory_order_relaxed);
  stats->rx_cnt = fd->rx_cnt.load(std::memory_order_relaxed);
  stats->rx_slow_cnt = fd->rx_slow_cnt.load(std::memory_order_relaxed);
  return ncclSuccess;
}

ncclResult_t tcpxGetCommStats(void* recvComm, tcpxCommStats* stats) {
  Comm* comm = static_cast<Comm*>(recvComm);
  if (!comm || !stats) return ncclInvalidArgument;
  stats->rx_ctrl_slow_cnt = comm->rx_ctrl_slow_cnt;
  stats->unpack_cnt = comm->unpack_cnt;
  stats->unpack_slow_cnt = comm->unpack_slow_cnt;
  stats->unpack_ns = comm->unpack_ns;
  stats->trace_dropped = comm->trace ? comm->trace->dropped() : 0;
  stats->socket_thread_cpus = comm->helper_cpus.load(std::memory_order_relaxed);
  stats->max_slots_at_gpu = comm->max_slots_at_gpu;
  return ncclSuccess;
}

ncclResult_t tcpxTraceDrain(void* recvComm, tcpxTraceEvent* events, uint32_t max, uint32_t wait_ms, uint32_t* n) {
  Comm* comm = static_cast<Comm*>(recvComm);
  if (!comm || !n || (max != 0 && !events)) return ncclInvalidArgument;
  *n = comm->trace ? comm->trace->dequeue(events, max, wait_ms) : 0;
  return ncclSuccess;
}

ncclResult_t tcpxSetClockForTesting(uint64_t (*now_ns)(void)) {
  g.clock = now_ns ? now_ns : monotonic_ns;
  g.clock_injected = now_ns != nullptr;
  return ncclSuccess;
}

// ---- the flow scheduler on its own ---------------------------------------------------------------------------------
struct tcpxFlowSched {
  std::unique_ptr<FlowScheduler> impl;
  int alg;
};

ncclResult_t tcpxFlowSchedCreate(const char* alg, tcpxFlowSched** sched) {
  if (!sched) return ncclInvalidArgument;
  tcpxFlowSched* s = new (std::nothrow) tcpxFlowSched;
  if (!s) return ncclSystemError;
  // NULL: the policy of the current initialisation; a name: parsed like the flag.
  s->alg = alg ? sched_alg_from_name(alg, nullptr) : g.sched_alg;
  s->impl.reset(new_flow_scheduler(s->alg));
  s->impl->reset();
  *sched = s;
  return ncclSuccess;
}
int tcpxFlowSchedAlg(const tcpxFlowSched* sched) { return sched ? sched->alg : -1; }
void tcpxFlowSchedReset(tcpxFlowSched* sched) {
  if (sched) sched->impl->reset();
}
int tcpxFlowSchedHasFlow(const tcpxFlowSched* sched) { return sched && sched->impl->has_flow() ? 1 : 0; }
void tcpxFlowSchedSchedule(tcpxFlowSched* sched, int flow, int prio) {
  if (sched) sched->impl->schedule(flow, prio);
}
int tcpxFlowSchedPick(tcpxFlowSched* sched) { return sched ? sched->impl->pick() : -1; }
void tcpxFlowSchedDestroy(tcpxFlowSched* sched) { delete sched; }

}  // extern "C"
