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

// ---- coherent variant, for the persistent engine ------------------------------------------------------------------
// A kernel that never ends gets no cache invalidate at launch and no write-back at exit, so its payload accesses
// carry the coherence themselves: loads and stores are issued at system scope (sc0 sc1).  A load then never
// returns a line that an XCD's L2 kept from an earlier use of a recycled bounce page, and a store is written
// through, so that once the wavefront's store counter has drained (s_waitcnt vmcnt(0)) the bytes are where the
// host, a DMA engine or another kernel will read them -- no L2 write-back instruction is ever needed.
// The loads of one round and the wait for them form a single asm block: the compiler does not track counters
// for memory instructions it cannot see.
__device__ __forceinline__ void store_vec_sys(uint8_t* p, u32x4 v) {
  asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1" ::"v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ void store_byte_sys(uint8_t* p, uint32_t v) {
  asm volatile("global_store_byte %0, %1, off sc0 sc1" ::"v"(p), "v"(v) : "memory");
}

// Same contract as wave_copy_fragment.  One round moves up to 4 KiB: every lane issues the edge-byte load and
// one or four vector loads back to back (lanes past the end re-read the fragment's last vector, which is in
// range), waits once, then stores under its predicates.
__device__ __forceinline__ void wave_copy_fragment_coherent(const uint8_t* __restrict__ src,
                                                            uint8_t* __restrict__ dst, uint32_t len,
                                                            uint32_t lane) {
  if (len == 0) return;
  uint32_t head = static_cast<uint32_t>(-reinterpret_cast<uintptr_t>(dst)) & 15u;
  if (head > len) head = len;
  const uint32_t body = len - head;
  const uint32_t nvec = body >> 4;
  const uint32_t tail = body & 15u;

  uint32_t edge_off = 0;
  bool edge = false;
  if (lane < head) {
    edge = true;
    edge_off = lane;
  } else if (lane >= 16u && lane - 16u < tail) {
    edge = true;
    edge_off = head + (nvec << 4) + (lane - 16u);
  }
  const uint8_t* edge_src = src + edge_off;  // offset 0 for lanes without an edge byte: inside the fragment
  uint32_t edge_byte = 0;

  if (nvec == 0) {
    asm volatile(
        "global_load_ubyte %0, %1, off sc0 sc1\n"
        "s_waitcnt vmcnt(0)"
        : "=&v"(edge_byte)
        : "v"(edge_src)
        : "memory");
    if (edge) store_byte_sys(dst + edge_off, edge_byte);
    return;
  }

  const uint8_t* sb = src + head;
  uint8_t* db = dst + head;
  const uint32_t last = nvec - 1;
  for (uint32_t base = 0; base < nvec; base += kVecPerRound) {
    const uint32_t v0 = base + lane;
    const uint32_t v1 = v0 + kWaveLanes, v2 = v0 + 2 * kWaveLanes, v3 = v0 + 3 * kWaveLanes;
    const uint8_t* p0 = sb + (static_cast<size_t>(v0 < last ? v0 : last) << 4);
    u32x4 r0, r1, r2, r3;
    if (nvec - base <= kWaveLanes) {  // wave-uniform
      asm volatile(
          "global_load_ubyte %1, %3, off sc0 sc1\n"
          "global_load_dwordx4 %0, %2, off sc0 sc1\n"
          "s_waitcnt vmcnt(0)"
          : "=&v"(r0), "=&v"(edge_byte)
          : "v"(p0), "v"(edge_src)
          : "memory");
      if (v0 < nvec) store_vec_sys(db + (static_cast<size_t>(v0) << 4), r0);
    } else {
      const uint8_t* p1 = sb + (static_cast<size_t>(v1 < last ? v1 : last) << 4);
      const uint8_t* p2 = sb + (static_cast<size_t>(v2 < last ? v2 : last) << 4);
      const uint8_t* p3 = sb + (static_cast<size_t>(v3 < last ? v3 : last) << 4);
      asm volatile(
          "global_load_ubyte %4, %9, off sc0 sc1\n"
          "global_load_dwordx4 %0, %5, off sc0 sc1\n"
          "global_load_dwordx4 %1, %6, off sc0 sc1\n"
          "global_load_dwordx4 %2, %7, off sc0 sc1\n"
          "global_load_dwordx4 %3, %8, off sc0 sc1\n"
          "s_waitcnt vmcnt(0)"
          : "=&v"(r0), "=&v"(r1), "=&v"(r2), "=&v"(r3), "=&v"(edge_byte)
          : "v"(p0), "v"(p1), "v"(p2), "v"(p3), "v"(edge_src)
          : "memory");
      if (v0 < nvec) store_vec_sys(db + (static_cast<size_t>(v0) << 4), r0);
      if (v1 < nvec) store_vec_sys(db + (static_cast<size_t>(v1) << 4), r1);
      if (v2 < nvec) store_vec_sys(db + (static_cast<size_t>(v2) << 4), r2);
      if (v3 < nvec) store_vec_sys(db + (static_cast<size_t>(v3) << 4), r3);
    }
  }
  if (edge) store_byte_sys(dst + edge_off, edge_byte);
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
