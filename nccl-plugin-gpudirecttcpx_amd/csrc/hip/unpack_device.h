// Device-side building blocks of the gfx950 unpack kernels: how one 64-lane wavefront moves fragments.
//
// A fragment is `len` bytes (at most one 4 KiB bounce page in practice) with arbitrary byte alignment on both
// sides.  The copy is organised around the DESTINATION: the body is written with aligned 16-byte vector stores
// that cover whole 128-byte lines wherever a neighbouring fragment continues the line, and byte-wise heads and
// tails remain only at the ends of a run of fragments.  Source vectors are fetched with 16-byte loads at the
// 4-byte aligned address just below where the destination alignment puts them and shifted into place in
// registers.  This is a pure bandwidth copy: no MFMA, no LDS for payload.
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
// where the address arrives as an integer.
#define TCPXU_GLOBAL __attribute__((address_space(1)))

// ---- the copy path ------------------------------------------------------------------------------------------------
// Scope of the payload accesses.  A kernel that never ends gets no cache invalidate at launch and no write-back
// at exit, so its payload accesses carry the coherence themselves: loads and stores are issued at system scope
// (sc0 sc1).  A load then never returns a line that an XCD's L2 kept from an earlier use of a recycled bounce
// page, and a store is written through, so that once the wavefront's memory counter has drained
// (s_waitcnt vmcnt(0)) the bytes are where the host, a DMA engine or another kernel will read them -- no L2
// write-back instruction is ever needed.  Plain launches use the same accesses: measured here they stream at
// least as fast as cached non-temporal ones.
typedef TCPXU_GLOBAL u32x4* gvec_ptr;
__device__ __forceinline__ u32x4 load_vec_sys(const uint8_t* p) {
  return __builtin_amdgcn_global_load_b128((gvec_ptr)p, "");
}
__device__ __forceinline__ void store_vec_sys(uint8_t* p, u32x4 v) {
  __builtin_amdgcn_global_store_b128((gvec_ptr)p, v, "");
}
// The bulk of the payload is stored with the non-temporal hint on top of the system scope (sc0 sc1 nt): the
// destination is written once and not read again by this kernel, and telling the caches so keeps it from
// displacing other data (at an 8 MiB chunk of 4 KiB fragments, all from HBM: 2.80 against 2.58 TB/s of payload).
// The hint on the loads as well measured no faster.  No builtin combines the hint with a scope, so the store is
// written as an instruction; the s_nop covers the wait state the hardware wants between a store of more than
// 8 bytes and a write to its data registers, which the compiler cannot insert for an instruction it does not see.
#ifndef TCPXU_STORE_NT
#define TCPXU_STORE_NT 1
#endif
__device__ __forceinline__ void store_vec_stream(uint8_t* p, u32x4 v) {
#if TCPXU_STORE_NT
  asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1 nt\n\ts_nop 1" : : "v"((gvec_ptr)p), "v"(v) : "memory");
#else
  store_vec_sys(p, v);
#endif
}
__device__ __forceinline__ uint32_t load_byte_sys(const uint8_t* p) {
  return __hip_atomic_load((const TCPXU_GLOBAL uint8_t*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}
__device__ __forceinline__ void store_byte_sys(uint8_t* p, uint8_t v) {
  __hip_atomic_store((TCPXU_GLOBAL uint8_t*)p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// Destination lines.  HBM with ECC punishes a 128-byte line that arrives as two partial writes, and with
// write-through stores no cache merges them.  Consecutive fragments of a message land back to back in the
// destination at arbitrary byte offsets, so almost every fragment boundary falls inside a line.  Rule: a line
// belongs to the fragment that holds its first byte.  The wavefront that copies fragment A also writes the rest
// of A's last line, taking those bytes from the source of the next fragment B, and the wavefront that copies B
// starts at B's first full line.  Every line inside a run of fragments is then written whole, by one wavefront.
// Both owners decide with the same inputs whether the rule applies to a boundary:
constexpr uint32_t kLineBytes = 128;
// The line must hold nothing but the end of A and the beginning of B -- A reaches back to the line's first byte, B
// on to its last -- and each of the two must be long enough for a 16-byte load of its own bytes and not be one of
// the tiny fragments that are copied bytewise.
__device__ __forceinline__ bool fragment_is_tiny(const uint8_t* dst, uint32_t len);
__device__ __forceinline__ bool shares_line(uint64_t dst_a, uint32_t len_a, uint64_t dst_b, uint32_t len_b) {
  const uint32_t in_line = static_cast<uint32_t>(dst_a + len_a) & (kLineBytes - 1);  // bytes of A in the line
  return dst_a + len_a == dst_b && in_line != 0 && len_a >= in_line && len_a >= 16u && len_b >= kLineBytes - in_line &&
         len_b >= 16u && !fragment_is_tiny(reinterpret_cast<const uint8_t*>(dst_a), len_a) &&
         !fragment_is_tiny(reinterpret_cast<const uint8_t*>(dst_b), len_b);
}

// 16 bytes starting at byte `shift` (0..16) of the 32 bytes a:b.
__device__ __forceinline__ u32x4 extract16(u32x4 a, u32x4 b, uint32_t shift) {
  const uint32_t q = shift >> 2, r = shift & 3u;
  const uint32_t w[9] = {a[0], a[1], a[2], a[3], b[0], b[1], b[2], b[3], 0u};
  uint32_t sel[5];
#pragma unroll
  for (int k = 0; k < 5; ++k)
    sel[k] = q == 0 ? w[k] : q == 1 ? w[k + 1] : q == 2 ? w[k + 2] : q == 3 ? w[k + 3] : w[k + 4];
  u32x4 out;
#pragma unroll
  for (int d = 0; d < 4; ++d) out[d] = __builtin_amdgcn_alignbyte(sel[d + 1], sel[d], r);
  return out;
}

// One round of a wavefront's copy work: up to 4 KiB of 16-byte vectors with a 16-byte aligned destination, the
// edge bytes of the fragment (a head and a tail of fewer than 16 bytes where the fragment keeps its own partial
// lines), and the shared last line (eight vectors, each assembled from up to two sources).
// Loading and storing are separate steps, with an explicit wait for everything in flight between them.
//
// Only the lanes that have something to move take part in a memory instruction, and a part of the round that
// has nothing to move is skipped by the whole wavefront: the edge bytes where the fragment shares its first and
// last line with its neighbours, the shared line where it does not, the extra dword where the source needs no
// shifting.  (An earlier form issued the same eight loads and six stores in every round, with idle lanes
// repeating a neighbour's access; at an 8 MiB chunk of 4 KiB fragments the four main vectors alone ran 5 % faster
// than that.)
constexpr uint32_t kNoEdge = 0xFFFFFFFFu;
struct CopyRound {
  // Wave-uniform (scalar registers):
  const uint8_t* src_vec;   // source of vector 0 of this round (any alignment)
  uint8_t* dst_vec;         // destination of vector 0 (16-byte aligned)
  const uint8_t* src_frag;  // first byte of the fragment
  uint8_t* dst_frag;
  const uint8_t* src_next;  // first byte of the next fragment's source if the last line is shared, else src_frag
  uint32_t nvec;            // vectors in this round, 0..kVecPerRound (0: nothing but a shared line or edge bytes)
  uint32_t frag_len;
  uint32_t line_off;        // offset of the shared last line from dst_frag
  bool share_next;          // this round completes the fragment's last line out of the next fragment
  bool has_edge;            // this round copies edge bytes (some lane has one)
  // Per lane:
  uint32_t edge_off;        // offset of this lane's edge byte in the fragment, kNoEdge if it has none
};
constexpr int kDppWaveShiftLeft1 = 0x130;  // lane i receives lane i+1's value; lane 63 keeps the first operand
struct CopyRegs {
  u32x4 r[kVecPerLane];
  u32x4 line;  // lanes 0..7: the shared line's vectors as loaded; lane 8: the first 16 bytes of the next fragment
  uint32_t tail_dword;
  uint32_t edge_byte;
};
constexpr uint32_t kLineVecs = kLineBytes / 16;  // lanes that take part in the shared line

// The shared last line, lanes 0..7, one 16-byte vector each.  The fragment (A) has `rem` = frag_len - line_off bytes
// in the line (1..127), the next fragment (B) the rest.  Where the boundary falls is the same for the whole
// wavefront, so nothing here is worked out per lane beyond an address:
//   vectors before the boundary are 16 bytes of A, vectors after it 16 bytes of B, each loaded where it lies
//   (any alignment) and stored as loaded;
//   the one vector the boundary cuts (none if rem is a multiple of 16) is the last `cut` bytes of A followed by
//   the first 16 - cut bytes of B: its lane loads A's last 16 bytes, lane 8 of the same instruction loads B's first
//   16 for it, and it takes bytes [16 - cut, 32 - cut) of the two, a shift by a wave-uniform amount.
// shares_line has seen to it that every one of these loads stays inside its fragment.
// (An earlier form gave every lane two loads and a shift of its own, by a per-lane amount: some sixty vector
// instructions a line instead of some twenty, a sixth of the time of a round of a 2 KiB fragment.)
struct LinePlan {
  uint32_t rem;       // bytes of this fragment in the line
  uint32_t cut_lane;  // the vector the boundary falls in
  uint32_t cut;       // bytes of this fragment in that vector, 0 = the boundary falls between two vectors
};
__device__ __forceinline__ LinePlan line_plan(const CopyRound& c) {
  LinePlan p;
  p.rem = c.frag_len - c.line_off;
  p.cut_lane = p.rem >> 4;
  p.cut = p.rem & 15u;
  return p;
}

// Source realignment.  A 16-byte load whose address is not a multiple of 4 is split by the memory pipeline and
// runs at roughly two thirds of the rate of one that is (a multiple of 4 that is not a multiple of 16 costs
// nothing).  Source and destination of a fragment are misaligned against each other by an arbitrary number of
// bytes, and the destination decides where vectors start, so the source address of a vector is arbitrary.  The
// round therefore loads from the 4-byte aligned address just below (`skew` = 0..3 bytes below, the same for
// every vector of the round) and shifts the bytes into place in registers: a vector is bytes [skew, skew+16)
// of its own four dwords plus one more dword, and that fifth dword is the first dword of the next vector --
// which the neighbouring lane holds.  Only the round's last vector has no neighbour; its fifth dword comes
// from one extra 4-byte load by lane 0 (with skew > 0 that dword starts inside the fragment, and an aligned dword
// never leaves the 4 KiB page it starts in; with skew 0 nothing of it is used and it is not loaded).
__device__ __forceinline__ uint32_t load_dword_sys(const uint8_t* p) {
  return __hip_atomic_load((const TCPXU_GLOBAL uint32_t*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

__device__ __forceinline__ void round_load(const CopyRound& c, CopyRegs& x, uint32_t lane) {
  const uint32_t skew = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(c.src_vec)) & 3u;
  const uint8_t* base4 = c.src_vec - skew;
  // No register of the round is cleared first: a lane that loads nothing stores nothing (the same conditions guard
  // the stores), and what the shifts read from such a lane never reaches a stored byte.  The empty statement only
  // tells the compiler that the registers have a value (clearing them was a tenth of a short round's instructions).
  asm volatile("" : "=v"(x.r[0]), "=v"(x.r[1]), "=v"(x.r[2]), "=v"(x.r[3]), "=v"(x.line), "=v"(x.tail_dword), "=v"(x.edge_byte));
  if (c.has_edge) {
    if (c.edge_off != kNoEdge) x.edge_byte = load_byte_sys(c.src_frag + c.edge_off);
  }
#pragma unroll
  for (int k = 0; k < kVecPerLane; ++k) {
    const uint32_t v = static_cast<uint32_t>(k) * kWaveLanes + lane;
    if (v < c.nvec) x.r[k] = load_vec_sys(base4 + (v << 4));
  }
  if (skew != 0 && c.nvec != 0) {
    if (lane == 0) x.tail_dword = load_dword_sys(base4 + (c.nvec << 4));
  }
  if (c.share_next) {
    const LinePlan p = line_plan(c);
    // One load instruction: the line's eight vectors in lanes 0..7 and, where the boundary cuts a vector, the next
    // fragment's first 16 bytes in lane 8 (a load of its own for that one lane was a fifth of a ragged round's loads).
    if (lane < kLineVecs + (p.cut != 0 ? 1u : 0u)) {
      const uint32_t off = lane << 4;
      const uint8_t* from = lane < p.cut_lane ? c.src_frag + c.line_off + off : c.src_next + (off - p.rem);
      if (p.cut != 0 && lane == p.cut_lane) from = c.src_frag + c.frag_len - 16u;
      if (lane == kLineVecs) from = c.src_next;
      x.line = load_vec_sys(from);
    }
  }
}

// Waits for every load of the round (and for whatever else the wavefront has in flight) rather than let each
// vector be stored as soon as its own load has landed (what the compiler would arrange): the round's stores then
// leave back to back, which measured 2-3 % faster end to end.  The registers pass through the statement so that no
// use of them can be scheduled before it.
__device__ __forceinline__ void round_wait(CopyRegs& x) {
  asm volatile("s_waitcnt vmcnt(0)"
               : "+v"(x.r[0]), "+v"(x.r[1]), "+v"(x.r[2]), "+v"(x.r[3]), "+v"(x.line),
                 "+v"(x.tail_dword), "+v"(x.edge_byte)
               :
               : "memory");
  static_assert(kVecPerLane == 4, "the statement above names the four vectors of a round");
}

// Shifts the loaded bytes into place and stores them; the round's loads must have landed (round_wait).
__device__ __forceinline__ void round_store_loaded(const CopyRound& c, CopyRegs& x, uint32_t lane) {
  const uint32_t skew = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(c.src_vec)) & 3u;
  const uint32_t last = c.nvec - 1;
  const uint32_t tail_dword = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(x.tail_dword), 0));
#pragma unroll
  for (int k = 0; k < kVecPerLane; ++k) {
    // First dword of the next vector: lane+1 of this register, or lane 0 of the next register for lane 63.
    // (a DPP wavefront shift: one vector instruction, no trip through the LDS crossbar)
    uint32_t next0 = static_cast<uint32_t>(
        __builtin_amdgcn_update_dpp(0, static_cast<int>(x.r[k][0]), kDppWaveShiftLeft1, 0xF, 0xF, false));
    if (k + 1 < kVecPerLane) {
      const uint32_t wrap = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(x.r[k + 1 < kVecPerLane ? k + 1 : k][0]), 0));
      if (lane == 63u) next0 = wrap;
    }
    const uint32_t v = static_cast<uint32_t>(k) * kWaveLanes + lane;
    const uint32_t w4 = v < last ? next0 : tail_dword;  // the last vector uses the extra dword
    u32x4 out;
    out[0] = __builtin_amdgcn_alignbyte(x.r[k][1], x.r[k][0], skew);
    out[1] = __builtin_amdgcn_alignbyte(x.r[k][2], x.r[k][1], skew);
    out[2] = __builtin_amdgcn_alignbyte(x.r[k][3], x.r[k][2], skew);
    out[3] = __builtin_amdgcn_alignbyte(w4, x.r[k][3], skew);
    if (v < c.nvec) store_vec_stream(c.dst_vec + (v << 4), out);
  }
  if (c.share_next) {
    const LinePlan p = line_plan(c);
    u32x4 line = x.line;
    if (p.cut != 0) {
      // (lane 8's vector, the same for every lane: scalar registers)
      u32x4 next16;
#pragma unroll
      for (int d = 0; d < 4; ++d)
        next16[d] = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(x.line[d]), static_cast<int>(kLineVecs)));
      const u32x4 cut_vector = extract16(x.line, next16, 16u - p.cut);
      if (lane == p.cut_lane) line = cut_vector;
    }
    if (lane < kLineVecs) store_vec_stream(c.dst_frag + c.line_off + (lane << 4), line);
  }
  if (c.has_edge) {
    if (c.edge_off != kNoEdge) store_byte_sys(c.dst_frag + c.edge_off, static_cast<uint8_t>(x.edge_byte));
  }
}

__device__ __forceinline__ void round_store(const CopyRound& c, CopyRegs& x, uint32_t lane) {
  round_wait(x);
  round_store_loaded(c, x, lane);
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

// Where the vectors of a fragment that is not tiny start and end.
//   share_prev  the fragment's first partial line is written by the owner of the previous fragment
//   share_next  this owner completes the fragment's last line from src_next, the next fragment's source
struct FragmentPlan {
  uint32_t start_off;  // offset of vector 0 from the fragment's first byte
  uint32_t end_off;    // offset of the end of the last vector (where the shared last line starts, if there is one)
  uint32_t head, tail; // edge bytes before vector 0 and after the last vector, each fewer than 16
  uint32_t nvec;       // vectors in all; none where a short fragment lies in the shared lines of its two neighbours
};
__device__ __forceinline__ FragmentPlan plan_fragment(uint64_t dst_addr, uint32_t len, bool share_prev, bool share_next) {
  FragmentPlan p;
  p.head = 0;
  if (share_prev) {
    p.start_off = static_cast<uint32_t>(-dst_addr) & (kLineBytes - 1);
  } else {
    p.head = static_cast<uint32_t>(-dst_addr) & 15u;
    p.start_off = p.head;
  }
  p.tail = 0;
  if (share_next) {
    p.end_off = len - (static_cast<uint32_t>(dst_addr + len) & (kLineBytes - 1));
  } else {
    p.end_off = p.start_off + ((len - p.start_off) & ~15u);
    p.tail = len - p.end_off;
  }
  p.nvec = (p.end_off - p.start_off) >> 4;
  return p;
}
// The first round of a planned fragment; *nvec_left receives the vectors that remain for later rounds.
__device__ __forceinline__ CopyRound first_round_of(const uint8_t* src, uint8_t* dst, const uint8_t* src_next,
                                                    uint32_t len, bool share_next, uint32_t start_off,
                                                    uint32_t end_off, uint32_t head, uint32_t tail, uint32_t nvec,
                                                    uint32_t lane, uint32_t* nvec_left) {
  CopyRound c;
  c.src_frag = src;
  c.dst_frag = dst;
  c.src_vec = src + start_off;
  c.dst_vec = dst + start_off;
  c.src_next = share_next ? src_next : src;
  c.frag_len = len;
  c.line_off = end_off;
  c.share_next = share_next;
  // Lanes [0,head) carry the head, lanes [16,16+tail) the tail (both < 16 bytes); the other lanes have none.
  c.has_edge = (head | tail) != 0;
  c.edge_off = kNoEdge;
  if (lane < head) c.edge_off = lane;
  else if (lane >= 16u && lane - 16u < tail) c.edge_off = end_off + (lane - 16u);
  c.nvec = nvec < kVecPerRound ? nvec : kVecPerRound;
  *nvec_left = nvec - c.nvec;
  return c;
}

// Splits a fragment that is not tiny (all arguments wave-uniform) into rounds of 1..kVecPerRound vectors.
// Fragments of the wire format (at most 4 KiB) have exactly one round; the first round of a longer fragment
// copies its edge bytes and its shared line.
struct FragmentRounds {
  uint32_t nvec_left = 0;  // vectors not yet handed out

  __device__ __forceinline__ CopyRound first_round(const uint8_t* src, uint8_t* dst, uint32_t len, bool share_prev,
                                                   bool share_next, const uint8_t* src_next, uint32_t lane) {
    const FragmentPlan p = plan_fragment(reinterpret_cast<uintptr_t>(dst), len, share_prev, share_next);
    return first_round_of(src, dst, src_next, len, share_next, p.start_off, p.end_off, p.head, p.tail, p.nvec, lane,
                          &nvec_left);
  }
  __device__ __forceinline__ bool more() const { return nvec_left != 0; }
  __device__ __forceinline__ CopyRound next_round(const CopyRound& prev) {
    CopyRound c = prev;
    c.has_edge = false;  // the first round has copied the edge bytes and the shared line
    c.share_next = false;
    c.src_vec = prev.src_vec + (static_cast<size_t>(prev.nvec) << 4);
    c.dst_vec = prev.dst_vec + (static_cast<size_t>(prev.nvec) << 4);
    c.nvec = nvec_left < kVecPerRound ? nvec_left : kVecPerRound;
    nvec_left -= c.nvec;
    return c;
  }
};

// A wavefront's position in its share of a descriptor list staged in LDS: descriptors j, j + stride, ... < end of
// a list of n.  Neighbours in the list (whoever copies them) decide which destination lines are shared.
// Everything that describes a fragment is wave-uniform; saying so keeps it in scalar registers and leaves the
// vector registers to the payload in flight.  `bounce` and `dst` must be wave-uniform.
// `before` / `after`: the list has a valid descriptor at index -1 / at index n (the last of the batch before, the
// first of the batch after, staged with it), which the first and the last fragment of the list may share a line with:
// the wavefront that copies the neighbouring batch looks at the same pair from the other side.
struct ShareCursor {
  const tcpxuLoadMeta* descs;
  uint32_t n, j, end, stride;
  bool before, after;
  const uint8_t* bounce;
  uint8_t* dst;
  FragmentRounds fr;

  static __device__ __forceinline__ uint32_t uniform(uint32_t v) {
    return static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(v));
  }
  static __device__ __forceinline__ uint64_t uniform64(uint64_t v) {
    return (static_cast<uint64_t>(uniform(static_cast<uint32_t>(v >> 32))) << 32) | uniform(static_cast<uint32_t>(v));
  }
  __device__ __forceinline__ void open(const tcpxuLoadMeta* list, uint32_t count, uint32_t first, uint32_t step,
                                       uint32_t stop, const uint8_t* bounce_base, uint8_t* dst_base,
                                       bool has_before, bool has_after) {
    descs = list;
    n = count;
    before = has_before;
    after = has_after;
    j = uniform(first);
    end = uniform(stop);
    stride = step;
    bounce = bounce_base;
    dst = dst_base;
    fr.nvec_left = 0;
  }
  // Next round of the share, or false when there is none.  `prev` is the round before it (read only while a
  // fragment longer than one round is being continued).  `on_take()` runs after each descriptor has been taken
  // off the share, with j already advanced.  Fragments too short for a round are copied here, at once.
  template <typename OnTake>
  __device__ __forceinline__ bool produce(CopyRound& out, const CopyRound& prev, uint32_t lane, OnTake&& on_take) {
    if (fr.more()) {
      out = fr.next_round(prev);
      return true;
    }
    const uint64_t dst_addr = reinterpret_cast<uint64_t>(dst);
    while (j < end) {
      const uint32_t cur = j;
      j += stride;
      on_take();
      const tcpxuLoadMeta d = descs[cur];
      const uint32_t len = uniform(d.len);
      if (len == 0) continue;
      const uint32_t so = uniform(d.src_off);
      const uint64_t doff = uniform64(d.dst_off);
      const uint8_t* fsrc = bounce + so;
      uint8_t* fdst = dst + doff;
      if (fragment_is_tiny(fdst, len)) {
        copy_tiny_fragment(fsrc, fdst, len, lane);
        continue;
      }
      bool share_prev = false, share_next = false;
      const uint8_t* src_next = fsrc;
      if (cur > 0 || before) {
        const tcpxuLoadMeta p = descs[static_cast<int32_t>(cur) - 1];
        share_prev = shares_line(dst_addr + uniform64(p.dst_off), uniform(p.len), dst_addr + doff, len);
      }
      if (cur + 1 < n || after) {
        const tcpxuLoadMeta q = descs[cur + 1];
        share_next = shares_line(dst_addr + doff, len, dst_addr + uniform64(q.dst_off), uniform(q.len));
        if (share_next) src_next = bounce + uniform(q.src_off);
      }
      out = fr.first_round(fsrc, fdst, len, share_prev, share_next, src_next, lane);
      return true;
    }
    return false;
  }
};

// Copies descriptors first, first + stride, ... < end of a descriptor list of n staged in LDS with the calling
// wavefront, one round (at most 4 KiB) in flight at a time.
// `on_last_fragment()` is called exactly once, when the wavefront turns to the last descriptor of its share (at
// once if it has none): a caller that feeds the wavefront can use it to start fetching more work.
template <typename OnLastFragment>
__device__ __forceinline__ void wave_copy_descriptors(const tcpxuLoadMeta* descs, uint32_t n, uint32_t first,
                                                      uint32_t stride, uint32_t end, const uint8_t* bounce,
                                                      uint8_t* dst, uint32_t lane,
                                                      OnLastFragment&& on_last_fragment, bool has_before = false,
                                                      bool has_after = false) {
  ShareCursor cursor;
  cursor.open(descs, n, first, stride, end, bounce, dst, has_before, has_after);
  if (cursor.j >= cursor.end) on_last_fragment();
  auto on_take = [&] {
    if (cursor.j >= cursor.end) on_last_fragment();
  };
  CopyRound r;
  CopyRegs x;
  if (!cursor.produce(r, r, lane, on_take)) return;
  for (;;) {
    round_load(r, x, lane);
    // The next round is worked out while this one's loads are on their way.
    CopyRound nxt;
    const bool more = cursor.produce(nxt, r, lane, on_take);
    round_store(r, x, lane);
    if (!more) return;
    r = nxt;
  }
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
