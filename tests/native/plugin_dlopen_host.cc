// A host that loads the plugin the way NCCL does (src/nccl_plugin.cc:22-42 is what it finds): dlopen, look up
// `ncclNetPlugin_v7`, and from then on call the receive path ONLY through that table's pointers:
//   init -> devices -> getProperties -> listen -> accept (nobody there yet) -> connect -> accept -> regMr ->
//   per request: irecv -> test* -> iflush -> irecvConsumed  -> deregMr -> closeRecv -> closeSend -> closeListen.
// It links against nothing of this repository.  What a real job gets from the peer and from the kernel -- control
// messages and devmem fragments -- has no NIC behind it here, so the host pushes it in through the plugin's
// synthetic-socket entry points, looked up by name in the same library; device memory comes from the HIP layer's
// C entry points (libtcpxu_hip.so), or, with --emu, from a stand-in device whose table is installed before init.
//
//   plugin_dlopen_host <libnccl-net.so> <fixture.bin> [--emu <libemu.so>] [--watch]
//
// The fixture (tests/golden/make_plugin_fixture.py) holds fragments, requests and the expected receive buffer;
// the result must match byte for byte.  With --watch the host also plays the clock: for a request that the GPU is
// copying it moves the injected clock by 11 s between two polls, expects exactly one slowness report for it, and
// prints the state tracepoints it drains afterwards ("event <kind> <object> <state>") for the caller to check.
#include <dlfcn.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <string>
#include <vector>

#include "nccl_net_v7.h"
#include "tcpx_plugin.h"  // types only: every function is looked up at run time

#define REQUIRE(cond, ...)                                  \
  do {                                                      \
    if (!(cond)) {                                          \
      fprintf(stderr, "%s:%d: %s failed: ", __FILE__, __LINE__, #cond); \
      fprintf(stderr, __VA_ARGS__);                         \
      fprintf(stderr, "\n");                                \
      exit(1);                                              \
    }                                                       \
  } while (0)

namespace {

struct Fixture {
  uint32_t pool_bytes = 0, dst_bytes = 0, n_frags = 0, n_requests = 0;
  uint64_t pool_seed = 0;
  std::vector<tcpxSynthFrag> frags;
  std::vector<tcpxSynthRequest> requests;
  std::vector<uint8_t> expect;
};

Fixture read_fixture(const char* path) {
  FILE* f = fopen(path, "rb");
  REQUIRE(f, "cannot open %s", path);
  char magic[8];
  Fixture x;
  REQUIRE(fread(magic, 1, 8, f) == 8 && memcmp(magic, "TCPXFIX1", 8) == 0, "bad magic");
  REQUIRE(fread(&x.pool_bytes, 4, 1, f) == 1 && fread(&x.dst_bytes, 4, 1, f) == 1 && fread(&x.n_frags, 4, 1, f) == 1 &&
              fread(&x.n_requests, 4, 1, f) == 1 && fread(&x.pool_seed, 8, 1, f) == 1, "short header");
  x.frags.resize(x.n_frags);
  x.requests.resize(x.n_requests);
  x.expect.resize(x.dst_bytes);
  REQUIRE(fread(x.frags.data(), sizeof(tcpxSynthFrag), x.n_frags, f) == x.n_frags, "short fragment table");
  REQUIRE(fread(x.requests.data(), sizeof(tcpxSynthRequest), x.n_requests, f) == x.n_requests, "short request table");
  REQUIRE(fread(x.expect.data(), 1, x.dst_bytes, f) == x.dst_bytes, "short expectation");
  fclose(f);
  return x;
}

std::vector<uint8_t> splitmix64_bytes(uint64_t seed, size_t n) {
  std::vector<uint8_t> out((n + 7) / 8 * 8);
  uint64_t x = seed;
  for (size_t i = 0; i < out.size(); i += 8) {
    x += 0x9E3779B97F4A7C15ull;
    uint64_t z = x;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    memcpy(&out[i], &z, 8);  // little endian host
  }
  out.resize(n);
  return out;
}

template <typename Fn>
Fn lookup(void* lib, const char* name) {
  void* p = dlsym(lib, name);
  REQUIRE(p, "%s: %s", name, dlerror());
  return reinterpret_cast<Fn>(p);
}

// Device memory: the HIP layer, or plain host memory when the device is emulated.
struct Memory {
  bool emu = false;
  int (*alloc)(int, size_t, void**) = nullptr;
  int (*release)(int, void*) = nullptr;
  int (*to_device)(int, void*, const void*, size_t) = nullptr;
  int (*to_host)(int, void*, const void*, size_t) = nullptr;
  void* make(size_t n) {
    void* p = nullptr;
    if (emu) return malloc(n);
    REQUIRE(alloc(0, n, &p) == 0, "device allocation of %zu bytes", n);
    return p;
  }
  void put(void* dst, const void* src, size_t n) {
    if (emu) memcpy(dst, src, n);
    else REQUIRE(to_device(0, dst, src, n) == 0, "copy to device");
  }
  void get(void* dst, const void* src, size_t n) {
    if (emu) memcpy(dst, src, n);
    else REQUIRE(to_host(0, dst, src, n) == 0, "copy to host");
  }
  void drop(void* p) {
    if (emu) free(p);
    else REQUIRE(release(0, p) == 0, "device free");
  }
};

uint64_t g_fake_now = 1000000000ull;  // the injected clock, nanoseconds
uint64_t fake_clock() { return g_fake_now; }

int g_unpack_warnings = 0;
void logger(ncclDebugLogLevel level, unsigned long, const char*, int, const char* fmt, ...) {
  if (level != NCCL_LOG_WARN) return;
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  if (strstr(buf, "unpack timeout")) ++g_unpack_warnings;
  fprintf(stderr, "plugin WARN %s\n", buf);
}

}  // namespace

int main(int argc, char** argv) {
  REQUIRE(argc >= 3, "usage: %s <libnccl-net.so> <fixture.bin> [--emu <libemu.so>] [--watch]", argv[0]);
  const char* emu_path = nullptr;
  bool watch = false;
  for (int i = 3; i < argc; ++i) {
    if (strcmp(argv[i], "--emu") == 0 && i + 1 < argc) emu_path = argv[++i];
    else if (strcmp(argv[i], "--watch") == 0) watch = true;
    else REQUIRE(false, "unknown argument %s", argv[i]);
  }
  const Fixture fx = read_fixture(argv[2]);
  const std::vector<uint8_t> pool = splitmix64_bytes(fx.pool_seed, fx.pool_bytes);

  // ---- what NCCL does: dlopen and one dlsym ---------------------------------------------------------------------
  void* lib = dlopen(argv[1], RTLD_NOW | RTLD_LOCAL);
  REQUIRE(lib, "dlopen %s: %s", argv[1], dlerror());
  ncclNet_v7_t* net = static_cast<ncclNet_v7_t*>(dlsym(lib, "ncclNetPlugin_v7"));
  REQUIRE(net, "ncclNetPlugin_v7: %s", dlerror());
  REQUIRE(strcmp(net->name, "GPUDirectTCPX_v7") == 0, "name %s", net->name);
  REQUIRE(net->regMrDmaBuf == nullptr && net->closeSend == net->closeRecv, "table shape");

  // ---- what stands in for the peer and the kernel ------------------------------------------------------------------
  auto arena_create = lookup<ncclResult_t (*)(int, size_t, void**)>(lib, "tcpxSynthArenaCreate");
  auto ctrl_send = lookup<ncclResult_t (*)(void*, uint16_t, uint16_t, uint32_t, uint32_t, uint32_t)>(lib, "tcpxSynthCtrlSend");
  auto deliver = lookup<ncclResult_t (*)(void*, uint32_t, const tcpxSynthFrag*, uint32_t)>(lib, "tcpxSynthDeliver");
  auto outstanding = lookup<ncclResult_t (*)(void*, uint64_t*)>(lib, "tcpxSynthOutstandingPages");
  auto finalize = lookup<ncclResult_t (*)(void)>(lib, "tcpxFinalize");
  auto comm_stats = lookup<ncclResult_t (*)(void*, tcpxCommStats*)>(lib, "tcpxGetCommStats");
  auto trace_drain = lookup<ncclResult_t (*)(void*, tcpxTraceEvent*, uint32_t, uint32_t, uint32_t*)>(lib, "tcpxTraceDrain");
  Memory mem;
  void* emu_lib = nullptr;
  if (emu_path) {
    emu_lib = dlopen(emu_path, RTLD_NOW | RTLD_LOCAL);
    REQUIRE(emu_lib, "dlopen %s: %s", emu_path, dlerror());
    auto emu_ops = lookup<const tcpxDeviceOps* (*)(void)>(emu_lib, "emu_ops");
    auto set_ops = lookup<ncclResult_t (*)(const tcpxDeviceOps*)>(lib, "tcpxSetDeviceOpsForTesting");
    REQUIRE(set_ops(emu_ops()) == ncclSuccess, "installing the emulated device");
    mem.emu = true;
  } else {
    std::string hip_path(argv[1]);
    const size_t slash = hip_path.rfind('/');
    hip_path = (slash == std::string::npos ? std::string() : hip_path.substr(0, slash + 1)) + "libtcpxu_hip.so";
    void* hip = dlopen(hip_path.c_str(), RTLD_NOW | RTLD_GLOBAL);
    REQUIRE(hip, "dlopen %s: %s", hip_path.c_str(), dlerror());
    mem.alloc = lookup<int (*)(int, size_t, void**)>(hip, "tcpxuDeviceAlloc");
    mem.release = lookup<int (*)(int, void*)>(hip, "tcpxuDeviceFree");
    mem.to_device = lookup<int (*)(int, void*, const void*, size_t)>(hip, "tcpxuCopyToDevice");
    mem.to_host = lookup<int (*)(int, void*, const void*, size_t)>(hip, "tcpxuCopyToHost");
  }
  if (watch) {
    auto set_clock = lookup<ncclResult_t (*)(uint64_t (*)(void))>(lib, "tcpxSetClockForTesting");
    REQUIRE(set_clock(fake_clock) == ncclSuccess, "installing the clock");
  }

  // ---- the ncclNet_v7 sequence, through the table only -----------------------------------------------------------
  REQUIRE(net->init(logger) == ncclSuccess, "init");
  int ndev = 0;
  REQUIRE(net->devices(&ndev) == ncclSuccess && ndev >= 1, "devices -> %d", ndev);
  ncclNetProperties_v7_t props;
  memset(&props, 0, sizeof props);
  REQUIRE(net->getProperties(0, &props) == ncclSuccess, "getProperties");
  REQUIRE(props.maxRecvs == 1 && props.maxComms == 65536 && (props.ptrSupport & NCCL_PTR_CUDA), "properties");
  const bool unpack_type = props.netDeviceType == NCCL_NET_DEVICE_UNPACK;
  printf("properties: name %s, netDeviceType %d, version %d\n", props.name, props.netDeviceType, props.netDeviceVersion);
  REQUIRE(!unpack_type, "this host expects the plugin to do the copy (device type host)");

  void* arena = nullptr;
  REQUIRE(arena_create(0, fx.pool_bytes, &arena) == ncclSuccess && arena, "arena");
  mem.put(arena, pool.data(), pool.size());

  char handle[NCCL_NET_HANDLE_MAXSIZE];
  void *listen_comm = nullptr, *recv_comm = reinterpret_cast<void*>(0x1), *send_comm = nullptr;
  REQUIRE(net->listen(0, handle, &listen_comm) == ncclSuccess && listen_comm, "listen");
  ncclNetDeviceHandle_v7_t dev_handle;
  memset(&dev_handle, 0xFF, sizeof dev_handle);
  ncclNetDeviceHandle_v7_t* dh = &dev_handle;
  REQUIRE(net->accept(listen_comm, &recv_comm, &dh) == ncclSuccess && recv_comm == nullptr, "accept before connect");
  REQUIRE(net->connect(0, handle, &send_comm, nullptr) == ncclSuccess && send_comm, "connect");
  REQUIRE(net->accept(listen_comm, &recv_comm, &dh) == ncclSuccess && recv_comm, "accept after connect");
  REQUIRE(dev_handle.netDeviceType == NCCL_NET_DEVICE_HOST && dev_handle.handle == nullptr && dev_handle.size == 0, "device handle");

  const size_t guard = 256;
  std::vector<uint8_t> host_dst(guard + fx.dst_bytes + guard, 0xA5), want(host_dst);
  memcpy(want.data() + guard, fx.expect.data(), fx.dst_bytes);
  uint8_t* dst = static_cast<uint8_t*>(mem.make(host_dst.size()));
  mem.put(dst, host_dst.data(), host_dst.size());
  void* mhandle = nullptr;
  REQUIRE(net->regMr(recv_comm, dst + guard, static_cast<int>(fx.dst_bytes), NCCL_PTR_CUDA, &mhandle) == ncclSuccess && mhandle, "regMr");

  const int rounds = watch ? 20 : 1;  // with --watch the requests are received again until a poll catches the GPU at work
  int caught = 0;
  uint64_t expected_unpacks = 0;
  for (int round = 0; round < rounds && !(watch && caught > 0 && round > 0); ++round) {
    for (uint32_t i = 0; i < fx.n_requests; ++i) {
      const tcpxSynthRequest& r = fx.requests[i];
      void* data = dst + guard + r.dst_off;
      int size = static_cast<int>(r.bytes), tag = 0;
      void* request = nullptr;
      REQUIRE(net->irecv(recv_comm, 1, &data, &size, &tag, &mhandle, &request) == ncclSuccess && request, "irecv %u", i);
      // the peer: one control message per run of fragments on one flow; the kernel: the fragments themselves
      if (r.bytes == 0) {
        REQUIRE(ctrl_send(recv_comm, TCPX_CTRL_INLINE, 0, 0, 0, 0) == ncclSuccess, "inline control message");
      } else {
        uint32_t offset = 0;
        for (uint32_t a = 0; a < r.n_descs;) {
          uint32_t b = a, bytes = 0;
          const uint32_t flow = fx.frags[r.first_desc + a].flow;
          while (b < r.n_descs && fx.frags[r.first_desc + b].flow == flow) bytes += fx.frags[r.first_desc + b++].frag_size;
          REQUIRE(ctrl_send(recv_comm, TCPX_CTRL_NORMAL, static_cast<uint16_t>(flow), bytes, offset, r.bytes) == ncclSuccess, "control message");
          REQUIRE(deliver(recv_comm, flow, &fx.frags[r.first_desc + a], b - a) == ncclSuccess, "fragments");
          offset += bytes;
          a = b;
        }
        ++expected_unpacks;
      }
      tcpxCommStats before, now;
      REQUIRE(comm_stats(recv_comm, &before) == ncclSuccess, "stats");
      int done = 0, test_size = -777;
      bool jumped = false;
      for (long polls = 0; !done; ++polls) {
        REQUIRE(polls < 200000000L, "request %u never completed", i);
        REQUIRE(net->test(request, &done, &test_size) == ncclSuccess, "test %u", i);
        if (watch && !done && !jumped && r.bytes != 0) {
          REQUIRE(comm_stats(recv_comm, &now) == ncclSuccess, "stats");
          if (now.unpack_cnt == before.unpack_cnt + 1) {
            // The slot is with the GPU and the poll that handed it over has already looked at the completion word
            // once.  Eleven seconds pass on the injected clock; the very next poll either finds the copy finished
            // (no report: nothing was slow) or still running -- then it must report, once.
            g_fake_now += 11000000000ull;
            jumped = true;
            REQUIRE(net->test(request, &done, &test_size) == ncclSuccess, "test %u", i);
            REQUIRE(comm_stats(recv_comm, &now) == ncclSuccess, "stats");
            const uint64_t reports = now.unpack_slow_cnt - before.unpack_slow_cnt;
            REQUIRE(reports == (done ? 0u : 1u), "%lu slowness reports for a request that was %s", (unsigned long)reports,
                    done ? "already done" : "still being copied");
            if (!done) ++caught;
          }
        }
      }
      REQUIRE(test_size == -777, "test() wrote *size");
      REQUIRE(comm_stats(recv_comm, &now) == ncclSuccess, "stats");
      REQUIRE(now.unpack_slow_cnt - before.unpack_slow_cnt <= 1, "a request is reported at most once within the frequency interval");
      int flushed = -1;
      void* flush_request = request;
      REQUIRE(net->iflush(recv_comm, 1, &data, &flushed, &mhandle, &flush_request) == ncclSuccess && flushed == size, "iflush %u -> %d", i, flushed);
      REQUIRE(net->irecvConsumed(recv_comm, 1, request) == ncclSuccess, "irecvConsumed %u", i);
    }
  }
  uint64_t pages = 1;
  REQUIRE(outstanding(recv_comm, &pages) == ncclSuccess && pages == 0, "%lu pages not given back", (unsigned long)pages);
  tcpxCommStats st;
  REQUIRE(comm_stats(recv_comm, &st) == ncclSuccess, "stats");
  REQUIRE(st.unpack_cnt == expected_unpacks, "unpack_cnt %lu, expected %lu", (unsigned long)st.unpack_cnt, (unsigned long)expected_unpacks);
  if (watch) {
    REQUIRE(caught >= 1, "no poll ever found the GPU still copying");
    REQUIRE(st.unpack_slow_cnt == static_cast<uint64_t>(caught) && g_unpack_warnings == caught,
            "slow_cnt %lu, warnings %d, caught %d", (unsigned long)st.unpack_slow_cnt, g_unpack_warnings, caught);
    std::vector<tcpxTraceEvent> ev(65536);
    uint32_t n = 0;
    REQUIRE(trace_drain(recv_comm, ev.data(), static_cast<uint32_t>(ev.size()), 0, &n) == ncclSuccess, "drain");
    REQUIRE(st.trace_dropped == 0, "tracepoints dropped");
    for (uint32_t k = 0; k < n; ++k) printf("event %c %lx %u\n", ev[k].kind, (unsigned long)ev[k].object, ev[k].state);
    printf("watch: %d request(s) caught while the GPU was copying, %d report(s)\n", caught, g_unpack_warnings);
  } else {
    REQUIRE(st.unpack_slow_cnt == 0, "slowness reported without cause");
  }

  mem.get(host_dst.data(), dst, host_dst.size());
  size_t bad = 0, first_bad = 0;
  for (size_t k = 0; k < host_dst.size(); ++k)
    if (host_dst[k] != want[k] && bad++ == 0) first_bad = k;
  REQUIRE(bad == 0, "%zu bytes differ, the first at %zu (got %u, want %u)", bad, first_bad, host_dst[first_bad], want[first_bad]);

  REQUIRE(net->deregMr(recv_comm, mhandle) == ncclSuccess, "deregMr");
  REQUIRE(net->closeRecv(recv_comm) == ncclSuccess, "closeRecv");
  REQUIRE(net->closeSend(send_comm) == ncclSuccess, "closeSend");
  REQUIRE(net->closeListen(listen_comm) == ncclSuccess, "closeListen");
  mem.drop(dst);
  REQUIRE(finalize() == ncclSuccess, "finalize");
  printf("dlopen host ok: %u requests, %u fragments, %u bytes byte-exact through ncclNetPlugin_v7 (%s device)\n", fx.n_requests,
         fx.n_frags, fx.dst_bytes, mem.emu ? "emulated" : "HIP");
  return 0;
}
