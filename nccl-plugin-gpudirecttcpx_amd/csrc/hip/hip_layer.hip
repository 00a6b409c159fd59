// HIP layer of the receive-side unpack path: device selection, the bounce-page arena, mapped queue memory and
// the launch-per-batch unpack kernel, all behind the C-ABI of include/tcpx_unpack_hip.h.
// The persistent engine lives in engine.hip.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <vector>

#include "hip_common.h"
#include "tcpx_unpack_hip.h"
#include "unpack_device.h"

namespace tcpxu {

thread_local char g_last_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof g_last_error, fmt, ap);
  va_end(ap);
}

namespace {

constexpr uint32_t kMaxDescsPerWg = 64;
// Twelve wavefronts to a workgroup, one fragment each: 128 chunks of 8 MiB in one launch move 70.3 % of the HBM
// roofline this way, 69.6 % with eight wavefronts and eight descriptors, 67-68 % with four wavefronts taking two to
// four fragments each in turn, 65-68 % with sixteen.
#ifndef TCPXU_BATCH_THREADS
#define TCPXU_BATCH_THREADS 768
#endif
constexpr int kBatchThreads = TCPXU_BATCH_THREADS;
constexpr int kBatchWaves = kBatchThreads / kWaveLanes;

// Launch-per-batch unpack.  A workgroup takes `descs_per_wg` consecutive descriptors at a time, stages them in
// LDS with one 16-byte load per thread, then its twelve wavefronts take one fragment each (a short list is cut into
// batches of four or eight).  The descriptors of the workgroup's next batch are fetched into registers before the
// current batch is copied and go into the other of two LDS stages, so that a batch costs one barrier and no exposed
// descriptor fetch.
__global__ __launch_bounds__(kBatchThreads) void unpack_batch_kernel(const uint8_t* __restrict__ bounce,
                                                                   uint8_t* __restrict__ dst,
                                                                   const tcpxuLoadMeta* __restrict__ descs,
                                                                   uint64_t n_descs, uint32_t descs_per_wg,
                                                                   uint64_t n_batches) {
  // A stage holds the batch at [1, cnt] and, around it, the last descriptor of the batch before and the first of the
  // batch after (where the list has them): the fragments at the two ends of a batch share destination lines with
  // them like any other neighbours, and the workgroup that copies the neighbouring batch sees the same pairs.
  __shared__ tcpxuLoadMeta staged[2][kMaxDescsPerWg + 2];
  const uint32_t tid = threadIdx.x;
  const uint32_t lane = tid & (kWaveLanes - 1);
  const uint32_t wave = tid / kWaveLanes;
  const uint64_t n_slots = (n_batches + 7) / 8 * 8;  // work-item indices, some of which name no batch

  // Batch number and descriptor count of work item `wg` (count 0: none), and this thread's descriptor of it.
  auto batch_of = [&](uint64_t wg, uint64_t* first) -> uint32_t {
    if (wg >= n_slots) return 0;
    const uint64_t batch = xcd_contiguous_index(wg, n_batches);
    if (batch >= n_batches) return 0;
    *first = batch * descs_per_wg;
    return static_cast<uint32_t>(std::min<uint64_t>(descs_per_wg, n_descs - *first));
  };
  auto fetch = [&](uint64_t first, uint32_t cnt) -> u32x4 {  // thread t: descriptor first - 1 + t
    const uint64_t one_past = first + tid;
    const bool there = cnt != 0 && tid < cnt + 2 && one_past >= 1 && one_past <= n_descs;
    return there ? *reinterpret_cast<const u32x4*>(descs + one_past - 1) : u32x4{0, 0, 0, 0};
  };

  uint64_t wg = blockIdx.x, first = 0;
  uint32_t cnt = batch_of(wg, &first);
  u32x4 raw = fetch(first, cnt);
  for (uint32_t stage = 0; wg < n_slots; stage ^= 1u) {
    if (tid < cnt + 2) *reinterpret_cast<u32x4*>(&staged[stage][tid]) = raw;
    const uint32_t cnt_now = cnt;
    const bool has_before = first > 0, has_after = first + cnt < n_descs;
    wg += gridDim.x;
    cnt = batch_of(wg, &first);
    raw = fetch(first, cnt);  // in flight while this batch is copied
    __syncthreads();          // the stage is complete; every wavefront has left the stage written two batches ago
    wave_copy_descriptors(staged[stage] + 1, cnt_now, wave, kBatchWaves, cnt_now, bounce, dst, lane, [] {}, has_before,
                          has_after);
  }
}

struct DeviceProps {
  bool valid = false;
  int compute_units = 0;
  char name[256] = "";
};
DeviceProps g_props[kMaxDevices];

int env_int(const char* name, int fallback) {
  const char* v = getenv(name);
  if (!v || !*v) return fallback;
  return atoi(v);
}

}  // namespace

int use_device(int device) {
  if (device < 0 || device >= kMaxDevices) {
    set_error("device index %d out of range", device);
    return TCPXU_INVALID_ARGUMENT;
  }
  TCPXU_HIP(hipSetDevice(device));
  if (!g_props[device].valid) {
    hipDeviceProp_t p;
    TCPXU_HIP(hipGetDeviceProperties(&p, device));
    g_props[device].compute_units = p.multiProcessorCount;
    snprintf(g_props[device].name, sizeof g_props[device].name, "%s (%s)", p.name, p.gcnArchName);
    g_props[device].valid = true;
  }
  return TCPXU_SUCCESS;
}

int device_compute_units(int device) { return g_props[device].compute_units; }

// Grid geometry of the launch-per-batch kernel: enough descriptors per workgroup to amortise the staging
// barrier, few enough that a small slot still spreads over the whole GPU.
void batch_geometry(int device, uint64_t n_descs, uint32_t* descs_per_wg, uint64_t* n_batches, uint32_t* grid) {
  const uint64_t cus = static_cast<uint64_t>(std::max(1, g_props[device].compute_units));
  uint32_t dpw = static_cast<uint32_t>(env_int("TCPXU_DESCS_PER_WG", 0));
  if (dpw == 0) {
    // Aim for about 8 workgroups per compute unit, and at most one fragment per wavefront.
    const uint64_t want_wgs = cus * 8;
    const uint64_t d = (n_descs + want_wgs - 1) / want_wgs;
    dpw = d <= 4 ? 4 : d <= 8 ? 8 : static_cast<uint32_t>(kBatchWaves);
  }
  dpw = std::min(std::max(dpw, 1u), kMaxDescsPerWg);
  const uint64_t batches = (n_descs + dpw - 1) / dpw;
  const uint64_t per_xcd = (batches + 7) / 8;
  // One batch per workgroup up to 128 workgroups per compute unit; beyond that workgroups take several batches in
  // turn.  Letting the dispatcher hand out batches balances the compute units better than a grid that just fills
  // them and strides (1 GiB of 4 KiB fragments: 5.34 against 5.09 TB/s r+w with 16 workgroups per compute unit).
  const uint64_t max_grid = cus * static_cast<uint64_t>(std::max(1, env_int("TCPXU_BATCH_WGS_PER_CU", 128)));
  *descs_per_wg = dpw;
  *n_batches = batches;
  *grid = static_cast<uint32_t>(std::min<uint64_t>(per_xcd * 8, std::max<uint64_t>(max_grid, 8)));
}

}  // namespace tcpxu

using namespace tcpxu;

extern "C" {

const char* tcpxuLastError(void) { return g_last_error; }

int tcpxuDeviceCount(int* count) {
  if (!count) return TCPXU_INVALID_ARGUMENT;
  *count = 0;
  TCPXU_HIP(hipGetDeviceCount(count));
  return TCPXU_SUCCESS;
}

int tcpxuDeviceInfo(int device, char* name, size_t name_len, int* compute_units) {
  TCPXU_TRY(use_device(device));
  if (name && name_len) snprintf(name, name_len, "%s", g_props[device].name);
  if (compute_units) *compute_units = g_props[device].compute_units;
  return TCPXU_SUCCESS;
}

int tcpxuArenaCreate(int device, size_t bytes, void** arena_base) {
  if (!arena_base || bytes == 0 || bytes % TCPXU_PAGE_SIZE != 0) {
    set_error("arena size %zu must be a positive multiple of %d", bytes, TCPXU_PAGE_SIZE);
    return TCPXU_INVALID_ARGUMENT;
  }
  if (bytes > (1ull << 32)) {
    set_error("arena size %zu exceeds the 4 GiB reach of a 32-bit src_off", bytes);
    return TCPXU_INVALID_ARGUMENT;
  }
  TCPXU_TRY(use_device(device));
  TCPXU_HIP(hipMalloc(arena_base, bytes));
  if (reinterpret_cast<uintptr_t>(*arena_base) % TCPXU_PAGE_SIZE != 0) {
    (void)hipFree(*arena_base);
    *arena_base = nullptr;
    set_error("arena base is not page aligned");
    return TCPXU_INTERNAL_ERROR;
  }
  return TCPXU_SUCCESS;
}

int tcpxuArenaDestroy(int device, void* arena_base) {
  TCPXU_TRY(use_device(device));
  TCPXU_HIP(hipFree(arena_base));
  return TCPXU_SUCCESS;
}

int tcpxuDeviceAlloc(int device, size_t bytes, void** ptr) {
  if (!ptr || bytes == 0) return TCPXU_INVALID_ARGUMENT;
  TCPXU_TRY(use_device(device));
  TCPXU_HIP(hipMalloc(ptr, bytes));
  return TCPXU_SUCCESS;
}

int tcpxuDeviceFree(int device, void* ptr) {
  TCPXU_TRY(use_device(device));
  TCPXU_HIP(hipFree(ptr));
  return TCPXU_SUCCESS;
}

int tcpxuCopyToDevice(int device, void* dst_dev, const void* src_host, size_t bytes) {
  TCPXU_TRY(use_device(device));
  TCPXU_HIP(hipMemcpy(dst_dev, src_host, bytes, hipMemcpyHostToDevice));
  return TCPXU_SUCCESS;
}

int tcpxuCopyToHost(int device, void* dst_host, const void* src_dev, size_t bytes) {
  TCPXU_TRY(use_device(device));
  TCPXU_HIP(hipMemcpy(dst_host, src_dev, bytes, hipMemcpyDeviceToHost));
  return TCPXU_SUCCESS;
}

int tcpxuFillDevice(int device, void* dst_dev, int byte_value, size_t bytes) {
  TCPXU_TRY(use_device(device));
  TCPXU_HIP(hipMemset(dst_dev, byte_value, bytes));
  TCPXU_HIP(hipDeviceSynchronize());
  return TCPXU_SUCCESS;
}

int tcpxuDeviceSynchronize(int device) {
  TCPXU_TRY(use_device(device));
  TCPXU_HIP(hipDeviceSynchronize());
  return TCPXU_SUCCESS;
}

int tcpxuMappedAlloc(int device, size_t bytes, void** host_ptr, void** dev_ptr) {
  if (!host_ptr || !dev_ptr || bytes == 0) return TCPXU_INVALID_ARGUMENT;
  TCPXU_TRY(use_device(device));
  TCPXU_HIP(hipHostMalloc(host_ptr, bytes, hipHostMallocMapped | hipHostMallocCoherent | hipHostMallocPortable));
  memset(*host_ptr, 0, bytes);
  TCPXU_HIP(hipHostGetDevicePointer(dev_ptr, *host_ptr, 0));
  return TCPXU_SUCCESS;
}

int tcpxuMappedFree(int device, void* host_ptr) {
  TCPXU_TRY(use_device(device));
  TCPXU_HIP(hipHostFree(host_ptr));
  return TCPXU_SUCCESS;
}

// ---- device memory that the host can write ------------------------------------------------------------------------
// Fine-grained device memory is mapped for the host through the PCIe BAR where the whole of device memory is
// exposed (large BAR).  Blocks are small and few, and they are handed back to a pool, never to the driver:
// memory with non-default caching is not returned while the process lives.
namespace {
struct VisibleBlock {
  void* ptr;
  size_t bytes;
  int device;
  bool in_use;
};
std::mutex g_visible_mu;
std::vector<VisibleBlock> g_visible;
}  // namespace

int tcpxuVisibleAlloc(int device, size_t bytes, void** host_ptr, void** dev_ptr) {
  if (!host_ptr || !dev_ptr || bytes == 0 || bytes > (64u << 20)) return TCPXU_INVALID_ARGUMENT;
  const char* sw = getenv("TCPXU_VISIBLE_DEVICE_MEMORY");
  if (sw && *sw == '0') {
    set_error("host-visible device memory is switched off (TCPXU_VISIBLE_DEVICE_MEMORY=0)");
    return TCPXU_INVALID_USAGE;
  }
  TCPXU_TRY(use_device(device));
  int large_bar = 0;
  if (hipDeviceGetAttribute(&large_bar, hipDeviceAttributeIsLargeBar, device) != hipSuccess || !large_bar) {
    set_error("device %d does not expose its memory to the host (no large BAR)", device);
    return TCPXU_INVALID_USAGE;
  }
  bytes = (bytes + 4095) / 4096 * 4096;
  std::lock_guard<std::mutex> lock(g_visible_mu);
  void* p = nullptr;
  for (auto& b : g_visible) {
    if (!b.in_use && b.device == device && b.bytes == bytes) {
      b.in_use = true;
      p = b.ptr;
      break;
    }
  }
  if (!p) {
    TCPXU_HIP(hipExtMallocWithFlags(&p, bytes, hipDeviceMallocFinegrained));
    g_visible.push_back(VisibleBlock{p, bytes, device, true});
  }
  memset(p, 0, bytes);  // the first host access: through the BAR, write-combined
  __builtin_ia32_sfence();
  *host_ptr = p;
  *dev_ptr = p;
  return TCPXU_SUCCESS;
}

int tcpxuVisibleFree(int device, void* host_ptr) {
  std::lock_guard<std::mutex> lock(g_visible_mu);
  for (auto& b : g_visible) {
    if (b.ptr == host_ptr && b.device == device && b.in_use) {
      b.in_use = false;
      return TCPXU_SUCCESS;
    }
  }
  set_error("not a block of tcpxuVisibleAlloc on device %d", device);
  return TCPXU_INVALID_ARGUMENT;
}

void tcpxuVisibleFlush(void) { __builtin_ia32_sfence(); }

static int launch_batch(int device, const void* bounce_base, void* dst_base, const tcpxuLoadMeta* descs,
                        uint64_t n_descs, hipStream_t stream) {
  if (n_descs == 0) return TCPXU_SUCCESS;
  if (!bounce_base || !dst_base || !descs) {
    set_error("null pointer passed to unpack");
    return TCPXU_INVALID_ARGUMENT;
  }
  if (reinterpret_cast<uintptr_t>(descs) % 16 != 0) {
    set_error("descriptor array must be 16-byte aligned");
    return TCPXU_INVALID_ARGUMENT;
  }
  uint32_t dpw, grid;
  uint64_t batches;
  batch_geometry(device, n_descs, &dpw, &batches, &grid);
  hipLaunchKernelGGL(unpack_batch_kernel, dim3(grid), dim3(kBatchThreads), 0, stream,
                     static_cast<const uint8_t*>(bounce_base), static_cast<uint8_t*>(dst_base), descs, n_descs, dpw,
                     batches);
  TCPXU_HIP(hipGetLastError());
  return TCPXU_SUCCESS;
}

int tcpxuUnpackBatch(int device, const void* bounce_base, void* dst_base, const tcpxuLoadMeta* descs,
                     uint64_t n_descs, void* stream) {
  TCPXU_TRY(use_device(device));
  return launch_batch(device, bounce_base, dst_base, descs, n_descs, static_cast<hipStream_t>(stream));
}

}  // extern "C"
