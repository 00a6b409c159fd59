// Drives the plugin's host code natively so that it can run under AddressSanitizer/UBSan and ThreadSanitizer.
//
// TEST INFRASTRUCTURE.  Built by tests/test_sanitizers.py from the plugin's own sources, the workload generator,
// the emulated device operations of tests/emu and the CPU oracle; nothing here ships.  It receives reduced
// versions of the five workloads through tcpxSynthRunRequests, with the per-comm socket thread off and on and
// with tracepoints on while another thread drains them, and checks every destination byte.
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <atomic>
#include <thread>
#include <vector>

#include "tcpx_plugin.h"
#include "tcpx_synth.h"

extern "C" const tcpxDeviceOps* emu_ops(void);

#define CHECK(cond)                                                        \
  do {                                                                     \
    if (!(cond)) {                                                         \
      fprintf(stderr, "FAILED %s at %s:%d\n", #cond, __FILE__, __LINE__);  \
      return 1;                                                            \
    }                                                                      \
  } while (0)

static int run_case(int config, uint32_t shrink, uint8_t* arena, size_t arena_bytes, bool drain_trace) {
  tcpxSynthWorkload* wl = nullptr;
  CHECK(tcpxSynthCreate(config, 0x5A17u + static_cast<uint64_t>(config), shrink, &wl) == 0);
  tcpxSynthInfo info;
  CHECK(tcpxSynthGetInfo(wl, &info) == 0);
  CHECK(info.pool_bytes <= arena_bytes && info.n_windows == 1);
  CHECK(tcpxSynthFillWindow(wl, 0, arena) == 0);
  const tcpxSynthFrag* frags = tcpxSynthFrags(wl);
  const tcpxSynthRequest* reqs = tcpxSynthRequests(wl);

  char handle[NCCL_NET_HANDLE_MAXSIZE];
  void *listen = nullptr, *comm = nullptr, *send_comm = nullptr;
  CHECK(tcpxListen(0, handle, &listen) == ncclSuccess);
  ncclNetDeviceHandle_v7_t dev_handle;
  ncclNetDeviceHandle_v7_t* dh = &dev_handle;
  CHECK(tcpxAccept_v5(listen, &comm, &dh) == ncclSuccess && comm == nullptr);  // nobody has connected yet
  CHECK(tcpxConnect_v5(0, handle, &send_comm, nullptr) == ncclSuccess && send_comm != nullptr);
  CHECK(tcpxAccept_v5(listen, &comm, &dh) == ncclSuccess && comm != nullptr);

  std::atomic<bool> stop{false};
  std::atomic<uint64_t> drained{0};
  std::thread drainer;
  if (drain_trace) {
    drainer = std::thread([&] {
      std::vector<tcpxTraceEvent> ev(256);
      while (!stop.load()) {
        uint32_t n = 0;
        if (tcpxTraceDrain(comm, ev.data(), 256, 5, &n) != ncclSuccess) return;
        drained += n;
      }
    });
  }

  const size_t guard = 64;
  std::vector<uint8_t> dst(guard + info.dst_bytes + guard, 0xA5), want(dst);
  for (uint32_t r = 0; r < info.n_requests; ++r) {
    size_t pos = guard + reqs[r].dst_off;
    for (uint32_t k = 0; k < reqs[r].n_descs; ++k) {
      const tcpxSynthFrag& f = frags[reqs[r].first_desc + k];
      memcpy(&want[pos], arena + f.frag_offset, f.frag_size);
      pos += f.frag_size;
    }
  }
  double seconds = 0;
  std::vector<double> lat(info.n_requests ? info.n_requests : 1);
  CHECK(tcpxSynthRunRequests(comm, frags, reqs, info.n_requests, dst.data() + guard, info.dst_bytes, 8, 60000, &seconds,
                             lat.data()) == ncclSuccess);
  CHECK(dst == want);
  uint64_t pages = 1;
  CHECK(tcpxSynthOutstandingPages(comm, &pages) == ncclSuccess && pages == 0);
  tcpxCommStats cs;
  CHECK(tcpxGetCommStats(comm, &cs) == ncclSuccess && cs.unpack_slow_cnt == 0);
  if (drain_trace) {
    stop = true;
    drainer.join();
    std::vector<tcpxTraceEvent> ev(20000);
    uint32_t n = 0;
    CHECK(tcpxTraceDrain(comm, ev.data(), 20000, 0, &n) == ncclSuccess);
    CHECK(drained + n + cs.trace_dropped >= 5ull * info.n_requests);
  }
  CHECK(tcpxClose(comm) == ncclSuccess);
  CHECK(tcpxClose(send_comm) == ncclSuccess);
  CHECK(tcpxCloseListen(listen) == ncclSuccess);
  tcpxSynthDestroy(wl);
  printf("case config %d shrink %u: %u requests, %llu fragments, %.3f s ok\n", config, shrink, info.n_requests,
         static_cast<unsigned long long>(info.n_descs), seconds);
  return 0;
}

static int run_mode(const char* helper, const char* stats) {
  setenv("NCCL_GPUDIRECTTCPX_AMD_HELPER_THREAD", helper, 1);
  setenv("NCCL_GPUDIRECTTCPX_AMD_FLOWS", helper[0] == '1' ? "8" : "4", 1);
  setenv("NCCL_GPUDIRECTTCPX_TELEMETRY_ENABLE_TASK_LEVEL_STATS", stats, 1);
  setenv("NCCL_GPUDIRECTTCPX_TELEMETRY_ENABLE_REQUEST_LEVEL_STATS", stats, 1);
  CHECK(tcpxSetDeviceOpsForTesting(emu_ops()) == ncclSuccess);
  CHECK(tcpxSetFailStopForTesting(0) == ncclSuccess);
  CHECK(tcpxInit(nullptr) == ncclSuccess);
  const size_t arena_bytes = 64u << 20;
  void* base = nullptr;
  CHECK(tcpxSynthArenaCreate(0, arena_bytes, &base) == ncclSuccess);
  uint8_t* arena = static_cast<uint8_t*>(base);
  const struct {
    int config;
    uint32_t shrink;
  } cases[] = {{1, 0}, {2, 2}, {3, 3}, {4, 5}, {5, 4}};
  for (const auto& c : cases) {
    if (run_case(c.config, c.shrink, arena, arena_bytes, stats[0] == '1') != 0) return 1;
  }
  CHECK(tcpxFinalize() == ncclSuccess);
  CHECK(tcpxSetDeviceOpsForTesting(nullptr) == ncclSuccess);
  printf("mode helper=%s stats=%s ok\n", helper, stats);
  return 0;
}

int main() {
  if (run_mode("0", "0") != 0) return 1;
  if (run_mode("1", "0") != 0) return 1;
  if (run_mode("1", "1") != 0) return 1;
  if (run_mode("0", "1") != 0) return 1;
  printf("plugin sanitize run ok\n");
  return 0;
}
