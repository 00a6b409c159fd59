// Synthetic fragment source: seeded stand-in for NIC + devmem-TCP socket + sender (see include/tcpx_synth.h).
//
// PRNG: splitmix64.  Independent streams for page choice, lengths, in-page offsets and empty-descriptor choice
// are derived from the seed, so changing how one quantity is drawn does not disturb the others.
// Payload bytes are a counter-based function of (seed, window, 8-byte word index): any part of the pool can be
// produced on its own and in any order.
#include <pthread.h>
#include <sched.h>

#include <algorithm>
#include <atomic>
#include <chrono>
#include <cstdint>
#include <cstring>
#include <new>
#include <thread>
#include <vector>

#include "tcpx_synth.h"

namespace {

constexpr uint64_t kGolden = 0x9E3779B97F4A7C15ull;
constexpr uint32_t kPage = TCPXU_PAGE_SIZE;
constexpr uint32_t kMaxRequestBytes = 4u << 20;        // NET_UNPACK_MAX_SLICE_SIZE
constexpr uint32_t kMaxRequestDescs = TCPXU_SLOT_PAGES;  // NET_UNPACK_MAX_SLICE_PAGES

inline uint64_t mix64(uint64_t z) {
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

struct Stream {
  uint64_t s;
  Stream(uint64_t seed, uint64_t id) : s(mix64(seed ^ (kGolden * (id + 1)))) {}
  uint64_t next() {
    s += kGolden;
    return mix64(s);
  }
  // Uniform integer in [0, n), n >= 1, by the multiply-high method.
  uint64_t below(uint64_t n) { return static_cast<uint64_t>((static_cast<unsigned __int128>(next()) * n) >> 64); }
  uint64_t between(uint64_t lo, uint64_t hi) { return lo + below(hi - lo + 1); }  // inclusive
};

enum StreamId : uint64_t { kPages = 1, kLengths = 2, kOffsets = 3, kEmpties = 4, kPayload = 5 };

}  // namespace

struct tcpxSynthWorkload {
  int config = 0;
  uint64_t seed = 0;
  tcpxSynthInfo info{};
  std::vector<tcpxuLoadMeta> descs;
  std::vector<tcpxSynthFrag> frags;
  std::vector<tcpxSynthRequest> requests;

  void add(uint32_t page, uint32_t in_page, uint32_t len, uint32_t flow, uint64_t dst_off) {
    const uint32_t src = page * kPage + in_page;
    descs.push_back(tcpxuLoadMeta{src, len, dst_off});
    frags.push_back(tcpxSynthFrag{src, len, page, flow});
  }
  void close_request(uint64_t first, uint64_t dst_off, uint32_t bytes, uint32_t window) {
    requests.push_back(
        tcpxSynthRequest{first, dst_off, static_cast<uint32_t>(descs.size() - first), bytes, window, 0});
  }
};

namespace {

std::vector<uint32_t> permutation_prefix(Stream& rng, uint32_t n, uint32_t take) {
  // Fisher-Yates, stopped after `take` positions are final.
  std::vector<uint32_t> p(n);
  for (uint32_t i = 0; i < n; ++i) p[i] = i;
  for (uint32_t i = 0; i < take && i + 1 < n; ++i) std::swap(p[i], p[i + rng.below(n - i)]);
  p.resize(take);
  return p;
}

// Page-aligned 4 KiB fragments on permuted pages, cut into requests of `request_bytes`.
void gen_aligned(tcpxSynthWorkload& w, uint64_t total, uint32_t request_bytes, uint32_t n_flows) {
  Stream pages(w.seed, kPages);
  const uint32_t n_pages = static_cast<uint32_t>(w.info.pool_bytes / kPage);
  const uint32_t n_frags = static_cast<uint32_t>(total / kPage);
  const std::vector<uint32_t> perm = permutation_prefix(pages, n_pages, n_frags);
  const uint32_t per_req = request_bytes / kPage;
  for (uint32_t i = 0; i < n_frags; ++i) {
    if (i % per_req == 0 && i) w.close_request(i - per_req, static_cast<uint64_t>(i - per_req) * kPage, request_bytes, 0);
    // Flows carry runs of 128 KiB (32 fragments), round-robin.
    w.add(perm[i], 0, kPage, (i / 32) % n_flows, static_cast<uint64_t>(i) * kPage);
  }
  const uint32_t first = (n_frags - 1) / per_req * per_req;
  w.close_request(first, static_cast<uint64_t>(first) * kPage, (n_frags - first) * kPage, 0);
}

// 8 MiB chunk over 4 flows: 90% full pages, 10% U[64,4095]; byte-unaligned sources; pages with replacement.
void gen_chunk(tcpxSynthWorkload& w, uint64_t total) {
  Stream pages(w.seed, kPages), lengths(w.seed, kLengths), offsets(w.seed, kOffsets);
  const uint32_t n_pages = static_cast<uint32_t>(w.info.pool_bytes / kPage);
  uint64_t done = 0;
  while (done < total) {
    const uint32_t req_bytes = static_cast<uint32_t>(std::min<uint64_t>(kMaxRequestBytes, total - done));
    const uint64_t first = w.descs.size();
    uint32_t in_req = 0;
    while (in_req < req_bytes) {
      uint32_t len = lengths.below(10) < 9 ? kPage : static_cast<uint32_t>(lengths.between(64, kPage - 1));
      len = std::min(len, req_bytes - in_req);  // the last fragment of a request ends the request exactly
      const uint32_t page = static_cast<uint32_t>(pages.below(n_pages));
      const uint32_t in_page = static_cast<uint32_t>(offsets.between(0, kPage - len));
      w.add(page, in_page, len, static_cast<uint32_t>(w.descs.size() % w.info.n_flows), done + in_req);
      in_req += len;
    }
    w.close_request(first, done, req_bytes, 0);
    done += req_bytes;
  }
}

// Many small requests: 16 full pages each, pages with replacement.
void gen_storm(tcpxSynthWorkload& w, uint32_t n_requests) {
  Stream pages(w.seed, kPages);
  const uint32_t n_pages = static_cast<uint32_t>(w.info.pool_bytes / kPage);
  for (uint32_t r = 0; r < n_requests; ++r) {
    const uint64_t first = w.descs.size();
    const uint64_t base = static_cast<uint64_t>(r) * 16 * kPage;
    for (uint32_t k = 0; k < 16; ++k)
      w.add(static_cast<uint32_t>(pages.below(n_pages)), 0, kPage, 0, base + static_cast<uint64_t>(k) * kPage);
    w.close_request(first, base, 16 * kPage, 0);
  }
}

// Lengths U[1,4096] with 10% forced empty, arbitrary in-page offsets, pages distinct inside a request and
// reused between requests: every request is its own pool generation ("window").
void gen_adversarial(tcpxSynthWorkload& w, uint64_t total) {
  Stream pages(w.seed, kPages), lengths(w.seed, kLengths), offsets(w.seed, kOffsets), empties(w.seed, kEmpties);
  const uint32_t n_pages = static_cast<uint32_t>(w.info.pool_bytes / kPage);
  std::vector<uint32_t> used_in(n_pages, ~0u);
  uint64_t done = 0;
  uint32_t window = 0;
  while (done < total) {
    const uint64_t first = w.descs.size();
    uint32_t in_req = 0;
    while (done + in_req < total && in_req < kMaxRequestBytes && w.descs.size() - first < kMaxRequestDescs &&
           w.descs.size() - first < n_pages) {
      uint32_t len = 0;
      if (empties.below(10) != 0) {
        len = static_cast<uint32_t>(lengths.between(1, kPage));
        len = static_cast<uint32_t>(std::min<uint64_t>(len, std::min<uint64_t>(total - done - in_req,
                                                                              kMaxRequestBytes - in_req)));
      }
      uint32_t page;
      do page = static_cast<uint32_t>(pages.below(n_pages)); while (used_in[page] == window);
      used_in[page] = window;
      // An empty fragment still points into its page (offset 0..4095).
      const uint32_t in_page = static_cast<uint32_t>(offsets.between(0, kPage - std::max(len, 1u)));
      w.add(page, in_page, len, static_cast<uint32_t>(w.descs.size() % w.info.n_flows), done + in_req);
      in_req += len;
    }
    w.close_request(first, done, in_req, window);
    done += in_req;
    ++window;
  }
  w.info.n_windows = window;
}

}  // namespace

extern "C" {

int tcpxSynthCreate(int config, uint64_t seed, uint32_t shrink, tcpxSynthWorkload** workload) {
  if (!workload || shrink > 12) return 4;
  *workload = nullptr;
  tcpxSynthWorkload* w = new (std::nothrow) tcpxSynthWorkload;
  if (!w) return 2;
  w->config = config;
  w->seed = seed;
  w->info.n_windows = 1;
  w->info.n_flows = 1;
  auto shrunk = [shrink](uint64_t v, uint64_t floor) { return std::max<uint64_t>(v >> shrink, floor); };
  switch (config) {
    case TCPX_SYNTH_ALIGNED_1M:
      w->info.pool_bytes = shrunk(16ull << 20, 64 * kPage);
      gen_aligned(*w, shrunk(1ull << 20, 4 * kPage), kMaxRequestBytes, 1);
      break;
    case TCPX_SYNTH_CHUNK_8M:
      w->info.pool_bytes = shrunk(256ull << 20, 64 * kPage);
      w->info.n_flows = 4;
      gen_chunk(*w, shrunk(8ull << 20, 16 * kPage));
      break;
    case TCPX_SYNTH_STORM_64K:
      w->info.pool_bytes = shrunk(512ull << 20, 64 * kPage);
      gen_storm(*w, static_cast<uint32_t>(shrunk(2048, 4)));
      break;
    case TCPX_SYNTH_BULK_256M:
      w->info.pool_bytes = shrunk(1ull << 30, 256 * kPage);
      w->info.n_flows = 8;
      gen_aligned(*w, shrunk(256ull << 20, 64 * kPage), kMaxRequestBytes, 8);
      break;
    case TCPX_SYNTH_ADVERSARIAL:
      w->info.pool_bytes = shrunk(256ull << 20, 64 * kPage);
      w->info.n_flows = 2;
      w->info.dst_misalign = 3;
      gen_adversarial(*w, shrunk(32ull << 20, 16 * kPage));
      break;
    default:
      delete w;
      return 4;
  }
  w->info.n_descs = w->descs.size();
  w->info.n_requests = static_cast<uint32_t>(w->requests.size());
  uint64_t payload = 0, extent = 0;
  for (const auto& d : w->descs) {
    payload += d.len;
    extent = std::max<uint64_t>(extent, d.dst_off + d.len);
  }
  w->info.payload_bytes = payload;
  w->info.dst_bytes = extent;
  *workload = w;
  return 0;
}

void tcpxSynthDestroy(tcpxSynthWorkload* workload) { delete workload; }

int tcpxSynthGetInfo(const tcpxSynthWorkload* workload, tcpxSynthInfo* info) {
  if (!workload || !info) return 4;
  *info = workload->info;
  return 0;
}

const tcpxuLoadMeta* tcpxSynthDescs(const tcpxSynthWorkload* workload) { return workload->descs.data(); }
const tcpxSynthFrag* tcpxSynthFrags(const tcpxSynthWorkload* workload) { return workload->frags.data(); }
const tcpxSynthRequest* tcpxSynthRequests(const tcpxSynthWorkload* workload) { return workload->requests.data(); }

int tcpxSynthFillWindow(const tcpxSynthWorkload* w, uint32_t window, uint8_t* pool) {
  if (!w || !pool || window >= w->info.n_windows) return 4;
  const uint64_t base = mix64(w->seed ^ (kGolden * (kPayload + 1))) + static_cast<uint64_t>(window) * 0xD1B54A32D192ED03ull;
  auto fill_words = [&](uint64_t first_word, uint64_t n_words) {
    for (uint64_t k = first_word; k < first_word + n_words; ++k) {
      const uint64_t v = mix64(base + (k + 1) * kGolden);
      memcpy(pool + k * 8, &v, 8);
    }
  };
  if (window == 0) {
    fill_words(0, w->info.pool_bytes / 8);
    return 0;
  }
  for (const auto& r : w->requests) {
    if (r.window != window) continue;
    for (uint64_t i = r.first_desc; i < r.first_desc + r.n_descs; ++i)
      fill_words(static_cast<uint64_t>(w->frags[i].frag_token) * (kPage / 8), kPage / 8);
  }
  return 0;
}

// Two threads, one pinned to each CPU, pass a cache line back and forth.
int tcpxSynthCpuRoundTripNs(int cpu_a, int cpu_b, uint32_t rounds, double* ns) {
  if (!ns || rounds == 0 || cpu_a < 0 || cpu_b < 0 || cpu_a >= CPU_SETSIZE || cpu_b >= CPU_SETSIZE || cpu_a == cpu_b) return 4;
  struct alignas(64) Ball {
    std::atomic<uint64_t> v{0};
  } ball;
  std::atomic<int> failed{0};
  auto pin = [&](int cpu) {
    cpu_set_t set;
    CPU_ZERO(&set);
    CPU_SET(cpu, &set);
    if (pthread_setaffinity_np(pthread_self(), sizeof set, &set) != 0) failed.store(1);
  };
  double seconds = 0;
  std::thread a([&] {
    pin(cpu_a);
    const auto t0 = std::chrono::steady_clock::now();
    for (uint64_t i = 0; i < rounds && !failed.load(std::memory_order_relaxed); ++i) {
      ball.v.store(2 * i + 1, std::memory_order_release);
      while (ball.v.load(std::memory_order_acquire) != 2 * i + 2 && !failed.load(std::memory_order_relaxed)) {
      }
    }
    seconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
  });
  std::thread b([&] {
    pin(cpu_b);
    for (uint64_t i = 0; i < rounds && !failed.load(std::memory_order_relaxed); ++i) {
      while (ball.v.load(std::memory_order_acquire) != 2 * i + 1 && !failed.load(std::memory_order_relaxed)) {
      }
      ball.v.store(2 * i + 2, std::memory_order_release);
    }
  });
  a.join();
  b.join();
  if (failed.load()) return 2;
  *ns = seconds / rounds * 1e9;
  return 0;
}

}  // extern "C"
