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
// through, so that once the wavefront's memory counter has drained (s_waitcnt vmcnt(0)) the bytes are where the
// host, a DMA engine or another kernel will read them -- no L2 write-back instruction is ever needed.
typedef TCPXU_GLOBAL u32x4* gvec_ptr;
__device__ __forceinline__ u32x4 load_vec_sys(const uint8_t* p) {
  return __builtin_amdgcn_global_load_b128((gvec_ptr)p, "");
}
__device__ __forceinline__ void store_vec_sys(uint8_t* p, u32x4 v) {
  __builtin_amdgcn_global_store_b128((gvec_ptr)p, v, "");
}
__device__ __forceinline__ uint32_t load_byte_sys(const uint8_t* p) {
  return __hip_atomic_load((const TCPXU_GLOBAL uint8_t*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}
__device__ __forceinline__ void store_byte_sys(uint8_t* p, uint8_t v) {
  __hip_atomic_store((TCPXU_GLOBAL uint8_t*)p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// One round of a wavefront's copy work: up to 4 KiB of 16-byte vectors with a 16-byte aligned destination, plus
// the edge bytes of the fragment it belongs to (a fragment's head and tail, carried by its first round).
// Loading and storing are separate steps so that a wavefront can issue the loads of its next round before the
// stores of the current one: the memory counter of gfx9 retires in issue order, so waiting for the older loads
// leaves the younger ones in flight.
//
// Nothing in a round is predicated.  A lane whose vector index is past the round's end is clamped to the last
// vector for the load AND for the store: it re-reads and re-writes that vector with the very same bytes, which
// changes nothing.  A lane without an edge byte copies the fragment's byte 0 onto itself the same way.  Every
// round therefore issues exactly kVecPerLane + 1 loads and as many stores on every path, which lets the
// compiler compute exact wait counts and keep the younger round in flight.
struct CopyRound {
  // Wave-uniform (scalar registers):
  const uint8_t* src_vec;   // source of vector 0 of this round (any alignment)
  uint8_t* dst_vec;         // destination of vector 0 (16-byte aligned)
  const uint8_t* src_frag;  // first byte of the fragment
  uint8_t* dst_frag;
  uint32_t nvec;            // vectors in this round, 1..kVecPerRound
  // Per lane:
  uint32_t edge_off;        // offset of this lane's edge byte in the fragment, 0 if it has none
};
struct CopyRegs {
  u32x4 r[kVecPerLane];
  uint32_t edge_byte;
};

// Byte offset of lane's k-th vector in a round of nvec vectors, clamped to the last one.
__device__ __forceinline__ uint32_t round_vec_offset(uint32_t nvec, int k, uint32_t lane) {
  const uint32_t v = static_cast<uint32_t>(k) * kWaveLanes + lane;
  const uint32_t last = nvec - 1;
  return (v < last ? v : last) << 4;
}

__device__ __forceinline__ void round_load(const CopyRound& c, CopyRegs& x, uint32_t lane) {
  x.edge_byte = load_byte_sys(c.src_frag + c.edge_off);
#pragma unroll
  for (int k = 0; k < kVecPerLane; ++k) x.r[k] = load_vec_sys(c.src_vec + round_vec_offset(c.nvec, k, lane));
}

__device__ __forceinline__ void round_store(const CopyRound& c, const CopyRegs& x, uint32_t lane) {
#pragma unroll
  for (int k = 0; k < kVecPerLane; ++k) store_vec_sys(c.dst_vec + round_vec_offset(c.nvec, k, lane), x.r[k]);
  store_byte_sys(c.dst_frag + c.edge_off, static_cast<uint8_t>(x.edge_byte));
}

// A fragment too short to contain one destination-aligned vector (at most 30 bytes) is copied byte per lane,
// outside the round pipeline.
__device__ __forceinline__ bool fragment_is_tiny(const uint8_t* dst, uint32_t len) {
  const uint32_t head = static_cast<uint32_t>(-reinterpret_cast<uintptr_t>(dst)) & 15u;
  return len < head + 16u;
}
__device__ __forceinline__ void copy_tiny_fragment(const uint8_t* src, uint8_t* dst, uint32_t len, uint32_t lane) {
  if (lane < len) store_byte_sys(dst + lane, static_cast<uint8_t>(load_byte_sys(src + lane)));
}

// Splits a fragment that is not tiny (src, dst, len wave-uniform) into rounds of 1..kVecPerRound vectors.  Fragments of the wire format (at most
// 4 KiB) have exactly one round; later rounds of a longer fragment repeat the edge copy with the same bytes.
struct FragmentRounds {
  uint32_t nvec_left = 0;  // vectors not yet handed out

  __device__ __forceinline__ CopyRound first_round(const uint8_t* src, uint8_t* dst, uint32_t len, uint32_t lane) {
    uint32_t head = static_cast<uint32_t>(-reinterpret_cast<uintptr_t>(dst)) & 15u;
    if (head > len) head = len;
    const uint32_t body = len - head;
    const uint32_t tail = body & 15u;
    const uint32_t nvec = body >> 4;
    CopyRound c;
    c.src_frag = src;
    c.dst_frag = dst;
    c.src_vec = src + head;
    c.dst_vec = dst + head;
    // Lanes [0,head) carry the head, lanes [16,16+tail) the tail (both < 16 bytes); every other lane gets 0.
    c.edge_off = 0;
    if (lane < head) c.edge_off = lane;
    else if (lane >= 16u && lane - 16u < tail) c.edge_off = head + (nvec << 4) + (lane - 16u);
    c.nvec = nvec < kVecPerRound ? nvec : kVecPerRound;
    nvec_left = nvec - c.nvec;
    return c;
  }
  __device__ __forceinline__ bool more() const { return nvec_left != 0; }
  __device__ __forceinline__ CopyRound next_round(const CopyRound& prev) {
    CopyRound c = prev;
    c.src_vec = prev.src_vec + (static_cast<size_t>(prev.nvec) << 4);
    c.dst_vec = prev.dst_vec + (static_cast<size_t>(prev.nvec) << 4);
    c.nvec = nvec_left < kVecPerRound ? nvec_left : kVecPerRound;
    nvec_left -= c.nvec;
    return c;
  }
};

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
