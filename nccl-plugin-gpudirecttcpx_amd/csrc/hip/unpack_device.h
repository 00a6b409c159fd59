// Device-side building blocks of the gfx950 unpack kernels: how one 64-lane wavefront moves one fragment.
//
// A fragment is `len` bytes (at most one 4 KiB bounce page in practice) with arbitrary byte alignment on both
// sides.  The copy is organised around the DESTINATION: a byte-wise head brings the destination to a 16-byte
// boundary, the body is written with aligned 16-byte vector stores, a byte-wise tail finishes.  Source vectors
// are fetched with 16-byte loads at whatever alignment results (gfx950 global loads accept any alignment), so
// no realignment in registers is needed.  This is a pure bandwidth copy: no MFMA, no LDS for payload.
#ifndef TCPXU_UNPACK_DEVICE_H_
#define TCPXU_UNPACK_DEVICE_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "tcpx_unpack_hip.h"

namespace tcpxu {

constexpr int kWaveLanes = 64;
constexpr int kWgThreads = 256;
constexpr int kWavesPerWg = kWgThreads / kWaveLanes;
// Vectors a lane keeps in flight per round: 4 x 16 B x 64 lanes = one 4 KiB page per wavefront per round.
constexpr int kVecPerLane = 4;
constexpr uint32_t kVecPerRound = kVecPerLane * kWaveLanes;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef u32x4 u32x4_any __attribute__((aligned(1)));  // 16-byte vector at any byte alignment

// Payload always lives in global memory (the arena and the caller's receive buffer), so every payload access
// is cast to the global address space: the compiler then emits global_* instead of flat_* instructions even
// where the address arrives as an integer.  Payload is read once and written once, so both sides carry the
// non-temporal hint.
#define TCPXU_GLOBAL __attribute__((address_space(1)))
__device__ __forceinline__ u32x4 load_vec(const uint8_t* p) {
  return __builtin_nontemporal_load((const TCPXU_GLOBAL u32x4_any*)p);
}
__device__ __forceinline__ void store_vec(uint8_t* p, u32x4 v) {
  __builtin_nontemporal_store(v, (TCPXU_GLOBAL u32x4*)p);
}
__device__ __forceinline__ uint8_t load_byte(const uint8_t* p) { return *(const TCPXU_GLOBAL uint8_t*)p; }
__device__ __forceinline__ void store_byte(uint8_t* p, uint8_t v) { *(TCPXU_GLOBAL uint8_t*)p = v; }

// Copies src[0,len) to dst[0,len) with the 64 lanes of the calling wavefront.  `len`, `src` and `dst` must be
// wave-uniform.  Writes exactly [dst, dst+len): bytes on either side are never touched.
__device__ __forceinline__ void wave_copy_fragment(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst,
                                                   uint32_t len, uint32_t lane) {
  if (len == 0) return;
  uint32_t head = static_cast<uint32_t>(-reinterpret_cast<uintptr_t>(dst)) & 15u;
  if (head > len) head = len;
  const uint32_t body = len - head;
  const uint32_t nvec = body >> 4;
  const uint32_t tail = body & 15u;

  // Edge bytes: lanes [0,head) carry the head, lanes [16,16+tail) the tail (both < 16 bytes).
  uint32_t edge_off = 0;
  bool edge = false;
  if (lane < head) {
    edge = true;
    edge_off = lane;
  } else if (lane >= 16u && lane - 16u < tail) {
    edge = true;
    edge_off = head + (nvec << 4) + (lane - 16u);
  }
  uint8_t edge_byte = 0;
  if (edge) edge_byte = load_byte(src + edge_off);

  const uint8_t* sb = src + head;
  uint8_t* db = dst + head;
  uint32_t base = 0;
  // Full rounds: every lane moves four vectors, all four loads in flight before the first store.
  for (; base + kVecPerRound <= nvec; base += kVecPerRound) {
    u32x4 r[kVecPerLane];
#pragma unroll
    for (int k = 0; k < kVecPerLane; ++k)
      r[k] = load_vec(sb + (static_cast<size_t>(base + static_cast<uint32_t>(k) * kWaveLanes + lane) << 4));
#pragma unroll
    for (int k = 0; k < kVecPerLane; ++k)
      store_vec(db + (static_cast<size_t>(base + static_cast<uint32_t>(k) * kWaveLanes + lane) << 4), r[k]);
  }
  // Last, partial round.  Loads are unconditional (lanes past the end re-read the last vector, which is inside
  // the fragment) so that all of them are issued back to back; only the stores are predicated.
  if (base < nvec) {
    u32x4 r[kVecPerLane];
    const uint32_t last = nvec - 1;
#pragma unroll
    for (int k = 0; k < kVecPerLane; ++k) {
      const uint32_t v = base + static_cast<uint32_t>(k) * kWaveLanes + lane;
      r[k] = load_vec(sb + (static_cast<size_t>(v < last ? v : last) << 4));
    }
#pragma unroll
    for (int k = 0; k < kVecPerLane; ++k) {
      const uint32_t v = base + static_cast<uint32_t>(k) * kWaveLanes + lane;
      if (v < nvec) store_vec(db + (static_cast<size_t>(v) << 4), r[k]);
    }
  }
  if (edge) store_byte(dst + edge_off, edge_byte);
}

// The 8 XCDs of an MI355X receive workgroups round-robin by workgroup id and each has its own L2.  This maps a
// workgroup id to a work-item index such that every XCD walks one contiguous eighth of the index space:
// neighbouring descriptor batches (neighbouring destination lines) then meet in the same L2.
__device__ __forceinline__ uint64_t xcd_contiguous_index(uint64_t wg, uint64_t items) {
  constexpr uint64_t kXcds = 8;
  const uint64_t per_xcd = (items + kXcds - 1) / kXcds;
  return (wg % kXcds) * per_xcd + wg / kXcds;  // may be >= items: caller skips
}

}  // namespace tcpxu

#endif  // TCPXU_UNPACK_DEVICE_H_
