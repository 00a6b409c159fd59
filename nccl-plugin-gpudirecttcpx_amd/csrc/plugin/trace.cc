// Slowness watches, slowness switches and the tracepoint event buffer of the receive path (see trace.h).
#include "trace.h"

#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <strings.h>
#include <time.h>

#include <chrono>

static_assert(sizeof(tcpxTraceEvent) == 24, "tcpxTraceEvent is 24 bytes");
static_assert(sizeof(tcpxFlowStats) == 32 && sizeof(tcpxCommStats) == 56, "stats records are plain 64-bit counters");

namespace tcpx {

uint64_t monotonic_ns() {
  struct timespec ts;
  if (clock_gettime(CLOCK_MONOTONIC, &ts) < 0) return 0;
  return static_cast<uint64_t>(ts.tv_sec) * 1000000000ull + static_cast<uint64_t>(ts.tv_nsec);
}

// src/timeout.cc:52-75, with the clock passed in.
bool SlownessWatch::should_warn(ClockFn now, uint64_t* nanos) {
  if (same_count++ == 0) {
    first_ns = now();
    return false;
  }
  const uint64_t now_ns = now();
  if (!past_threshold) {
    *nanos = now_ns - first_ns;
    if (*nanos < threshold_ns) return false;
    past_threshold = true;
  } else {
    if (now_ns - prev_ns < frequency_ns) return false;
    *nanos = now_ns - first_ns;
  }
  prev_ns = now_ns;
  return true;
}

const char* const kSlownessNames[kSlowKinds] = {"TX_COMP", "SENDRECV", "RX_CTRL", "UNPACK"};

void parse_slowness_switches(const char* list, int switches[kSlowKinds]) {
  if (list == nullptr) return;
  char* copy = strdup(list);
  if (copy == nullptr) return;
  char* save = nullptr;
  for (char* opt = strtok_r(copy, ",", &save); opt != nullptr; opt = strtok_r(nullptr, ",", &save)) {
    if (strcasecmp(opt, "ALL") == 0) {
      for (int i = 0; i < kSlowKinds; ++i) switches[i] = 1;
      continue;
    }
    for (int i = 0; i < kSlowKinds; ++i) {
      if (strcasecmp(opt, kSlownessNames[i]) == 0) switches[i] = 1;
    }
  }
  free(copy);
}

TraceBuffer::TraceBuffer(size_t capacity) : items_(capacity) {}

void TraceBuffer::enqueue(char kind, const void* object, bool passive, int state, int64_t timestamp,
                          int sampling_factor) {
  // Sampling by object address, as the reference does (src/stats/stats_buffer.h:51,61).
  if (sampling_factor > 1 && reinterpret_cast<uintptr_t>(object) % static_cast<uintptr_t>(sampling_factor) != 0) return;
  std::lock_guard<std::mutex> lock(mu_);
  if (count_ == items_.size()) {
    ++dropped_;
    return;
  }
  tcpxTraceEvent& e = items_[(head_ + count_) % items_.size()];
  e.kind = kind;
  e.passive = passive ? 1 : 0;
  e.state = static_cast<uint16_t>(state);
  e.reserved = 0;
  e.object = reinterpret_cast<uint64_t>(object);
  e.timestamp = timestamp;
  ++count_;
  not_empty_.notify_one();
}

uint32_t TraceBuffer::dequeue(tcpxTraceEvent* out, uint32_t max, uint32_t wait_ms) {
  std::unique_lock<std::mutex> lock(mu_);
  if (count_ == 0 && wait_ms != 0) {
    // A deadline on the system clock makes this pthread_cond_timedwait, which thread-checking tools follow;
    // a steady-clock wait becomes pthread_cond_clockwait, which some of them do not.
    not_empty_.wait_until(lock, std::chrono::system_clock::now() + std::chrono::milliseconds(wait_ms),
                          [this] { return count_ != 0; });
  }
  uint32_t n = 0;
  while (n < max && count_ != 0) {
    out[n++] = items_[head_];
    head_ = (head_ + 1) % items_.size();
    --count_;
  }
  return n;
}

uint64_t TraceBuffer::dropped() {
  std::lock_guard<std::mutex> lock(mu_);
  return dropped_;
}

}  // namespace tcpx

extern "C" int tcpxTraceFormat(const tcpxTraceEvent* event, char* line, size_t len) {
  if (event == nullptr || line == nullptr || len == 0) return -1;
  // "R <request> <passive> <state> <timestamp>" / "T <task> ..." (src/stats/stats_buffer.h:52-56, 62-66).
  return snprintf(line, len, "%c %p %d %d %ld", event->kind, reinterpret_cast<void*>(event->object),
                  static_cast<int>(event->passive), static_cast<int>(event->state), static_cast<long>(event->timestamp));
}
