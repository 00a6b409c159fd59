/*
 * trace.h -- observability of the receive path: slowness watches, counters and state-transition tracepoints.
 *
 * Follows the reference's telemetry where the receive path touches it:
 *   slowness detection          struct tcpxTimeoutDetection, src/timeout.h:25-50, src/timeout.cc:32-75
 *   which waits are watched     kSlownessSwitch / kSlownessReport, src/flags.cc:59-150, src/flags.h:64-72
 *   tracepoints                 TCPX_TP at every ring transition, src/work_queue.h:156-211; src/stats/tracepoint.{h,cc}
 *   per-flow counters           struct tcpxSocketStats, src/stats/monitoring.h:25-39
 *   event buffer                struct StatsBuffer, src/stats/stats_buffer.h:33-103
 * and adds one watch the reference cannot have: a slot handed to the GPU whose completion word does not arrive.
 */
#ifndef TCPX_AMD_TRACE_H_
#define TCPX_AMD_TRACE_H_

#include <stdint.h>

#include <condition_variable>
#include <mutex>
#include <vector>

#include "tcpx_plugin.h"

namespace tcpx {

using ClockFn = uint64_t (*)(void);  // nanoseconds on a monotonic clock
uint64_t monotonic_ns();             // defaultTimenow, src/timeout.cc:26-30

// One watched wait.  The first look after a reset only notes the time; later looks report once when the wait has
// lasted `threshold_ns`, and again every `frequency_ns` after that, always with the time since the first look.
struct SlownessWatch {
  uint64_t threshold_ns = 0;
  uint64_t frequency_ns = 0;
  uint64_t first_ns = 0;
  uint64_t prev_ns = 0;
  uint32_t same_count = 0;
  bool past_threshold = false;

  void configure(uint64_t threshold, uint64_t frequency) {
    threshold_ns = threshold;
    frequency_ns = frequency;
    reset();
  }
  void reset() {  // tcpxTimeoutDetectionReset
    past_threshold = false;
    same_count = 0;
  }
  bool should_warn(ClockFn now, uint64_t* nanos);  // tcpxTimeoutDetectionShouldWarn
};

// The waits that can be watched.  The first three keep the reference's positions (src/flags.h:64-69); TX_COMP is
// a wait of the sending side, accepted in the flags and never armed here.
enum SlownessKind { kSlowTxComp = 0, kSlowSendRecv = 1, kSlowRxCtrl = 2, kSlowUnpack = 3, kSlowKinds = 4 };
extern const char* const kSlownessNames[kSlowKinds];
// Comma-separated names or ALL, case-insensitive; unknown names are ignored (parseSlownessSwitchFlagInternal,
// src/flags.cc:91-117).  Switches are only ever turned on.
void parse_slowness_switches(const char* list, int switches[kSlowKinds]);

// Timestamp codes of the exported lines (src/stats/tracepoint.h:57-75).
enum { kReqFreeTs = 0, kReqInactiveTs = 1, kReqTransmittingTs = 2, kReqActiveTs = 3, kReqPostedTs = 4 };
enum { kTaskFreeTs = 0, kTaskInactiveTs = 1, kTaskCompletingTs = 2, kTaskActiveTs = 3, kTaskRecvmsgTs = 7 };

constexpr size_t kTraceEvents = 10000;  // MAX_ITEMS, src/stats/stats_buffer.h:24

// Bounded, best-effort event buffer: producers never wait (an event that finds the buffer full is dropped and
// counted), one consumer may wait for events.
class TraceBuffer {
 public:
  explicit TraceBuffer(size_t capacity);
  void enqueue(char kind, const void* object, bool passive, int state, int64_t timestamp, int sampling_factor);
  // Up to `max` events, oldest first; waits up to wait_ms for the first one.
  uint32_t dequeue(tcpxTraceEvent* out, uint32_t max, uint32_t wait_ms);
  uint64_t dropped();

 private:
  std::mutex mu_;
  std::condition_variable not_empty_;
  std::vector<tcpxTraceEvent> items_;
  size_t head_ = 0, count_ = 0;
  uint64_t dropped_ = 0;
};

}  // namespace tcpx

#endif  // TCPX_AMD_TRACE_H_
