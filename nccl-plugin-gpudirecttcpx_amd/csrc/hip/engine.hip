// Persistent unpack engine: one long-running gfx950 kernel per GPU that turns slots published in mapped host
// memory into scatter-gather copies and reports completion into mapped host memory -- no launch per request.
//
// Roles inside the one kernel launch
//   workgroup 0, wavefront 0  "leader": polls the submission ring over PCIe (sixteen entries per round trip),
//                             cuts each submission into tickets of 8 to 16 consecutive descriptors (by backlog;
//                             up to 64 where the payload says the fragments are short; or of the fixed
//                             `descs_per_ticket`) and writes them into a device-memory ticket ring: several
//                             waiting submissions at once where it can.  It never copies payload.
//   every other workgroup     "worker": one fetcher wavefront claims the next ticket number with one atomic,
//                             polls that ticket's slot until its stamps match, reads the ticket's descriptors
//                             (one per lane) and leaves in LDS, per fragment, a record of what the copy needs
//                             to know about it (which destination lines it shares with its neighbours, in
//                             the ticket and, when the engine is busy, in the tickets before and after);
//                             the copy wavefronts copy the fragments from those records,
//                             and the last of them to finish counts the ticket done.  Whoever counts the last
//                             ticket of a submission writes the completion word that the host poller reads.
//
// No cache maintenance.  Nothing here uses an acquire or release fence: on this GPU those become L2 write-back
// and invalidate instructions, and thousands of pollers issuing them stall everybody.  Instead every access
// to shared state carries its own coherence: control words and tickets are read and written with system-scope
// (sc0 sc1) accesses that bypass the per-XCD L2, payload is loaded and stored the same way, and ordering comes
// from s_waitcnt: a wavefront drains its store counter before the workgroup counts a ticket done.
// Records that are written by one side and polled by the other (host submissions, tickets) are 64 bytes in four
// 16-byte sectors, each ending in a stamp derived from the record's sequence number; a reader accepts a record
// only when all four stamps match, so a record is valid even if its sectors arrive as separate transactions,
// and the writer never has to order "payload, then flag".
//
// Liveness: no workgroup ever waits for another worker.  Workers wait only for the leader (their ticket) and
// watch the stop word while they do; the leader waits for nothing (a full ticket ring or job table just defers
// a submission to the next poll).  The host stop word, or the optional spin limit, ends the leader; the leader
// drains its stores, then sets the stop words; a worker that sees one looks at its ticket a last time and leaves.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <chrono>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <new>
#include <thread>
#include <type_traits>
#include <vector>

#include "hip_common.h"
#include "tcpx_unpack_hip.h"
#include "unpack_device.h"


namespace tcpxu {
namespace {

constexpr uint32_t kTicketRing = 1u << 16;  // tickets in flight at most
constexpr uint32_t kMaxDescsPerTicket = 64;
// Ticket size when the caller does not fix one.  A ticket occupies a workgroup for one pick-up (a claim, the
// ticket record, the descriptors over PCIe: a few microseconds) plus its copy.  While workgroups are waiting for
// work, small tickets finish a submission sooner (more workgroups share it); once tickets queue up behind busy
// workgroups, larger ones spend less of each workgroup's time on pick-ups.  `backlog` estimates the descriptors of
// all submissions not yet completed, counting each in full until it completes (how far the slots in flight have
// got depends on the ticket size itself and would feed back).  The steps are where throughput measured at 1 to
// 64 slots of 4 MiB in flight changed hands between sizes; 8 is one fragment per copy wavefront, 16 two.  Beyond
// 16 nothing is gained for fragments of a page: with every source page coming from HBM, 64 slots in flight move
// 71.0 % of the roofline in tickets of 16, 70.1 % in tickets of 24 and 69.4 % in tickets of 32 (more tickets than
// workgroups keep every workgroup supplied, and a wavefront that has finished its share waits less for the
// slowest one).
// (Descriptors per worker workgroup below 13, 18; written without the division, which the leader would pay for
// on every submission.  backlog <= 2^20 and workers < 2^16 keep the products in 32 bits.)
__host__ __device__ __forceinline__ uint32_t ticket_size_for(uint32_t backlog, uint32_t workers) {
  return backlog < 13u * workers ? 8u : backlog < 18u * workers ? 12u : 16u;
}
// ceil(n / per_ticket) for 1 <= n <= 2^20 and 1 <= per_ticket <= 64 without the forty-odd instructions of a general
// 32-bit division: the quotient estimated in floating point (both operands are exact there) and put right by at most one.
__host__ __device__ __forceinline__ uint32_t tickets_for(uint32_t n, uint32_t per_ticket) {
  const uint32_t x = n + per_ticket - 1;
#if defined(__HIP_DEVICE_COMPILE__)
  uint32_t q = static_cast<uint32_t>(static_cast<float>(x) * __builtin_amdgcn_rcpf(static_cast<float>(per_ticket)));
#else
  uint32_t q = static_cast<uint32_t>(static_cast<float>(x) / static_cast<float>(per_ticket));
#endif
  while (q * per_ticket > x) --q;
  while (x - q * per_ticket >= per_ticket) ++q;
  return q;
}
// Ticket size for one submission of n descriptors when `in_flight` submissions (this one included) are not yet
// completed; each is taken to be as long as this one.  A small submission among many stays whole: with 8 or
// more in flight the parallelism is in the submissions, and a submission that is one ticket costs the leader
// one store instead of a pass of its loop.  (64 KiB requests of 16 fragments, p50 publish -> done: 8.7 -> 9.1 us
// at 8 in flight, 17.5 -> 9.3 us at 32, where the leader's loop had become the queue.)
//
// `bytes` is the submission's payload if the caller said (0 = unknown: whole pages).  The largest step, 16, stands
// for whole pages (14 while the backlog is shallow, see below: seven copy wavefronts then get two fragments each and
// one gets none); a submission of shorter fragments gets more descriptors per ticket, in multiples of 16 so that
// the copy wavefronts' shares come out even, up to 64 (full_ticket_size).  Written as comparisons: the leader runs
// this for every submission and a division costs it forty instructions.
constexpr uint32_t kManyInFlight = 8, kSmallSubmission = 32;
constexpr uint32_t kLaneTickets = 32;  // tickets of one submission that the lanes holding its entry still write themselves
constexpr uint32_t kLeaderBehind = 8;  // entries waiting in one poll from which the leader counts as the bottleneck
constexpr uint32_t kFullTicket = 16;
constexpr uint32_t kDeepBacklog = 100;  // descriptors per worker workgroup from which whole pages go in tickets of 16
__host__ __device__ __forceinline__ uint32_t full_ticket_size(uint32_t bytes, uint32_t n) {
  static_assert(kFullTicket == 16 && kMaxDescsPerTicket == 64, "the steps below");
  const uint64_t b = bytes;  // n <= 2^20: the products need more than 32 bits
  // Whole pages (or no hint): 16.  Shorter fragments: 32 from two thirds of a page down, 48 from half a page down,
  // 64 below a third -- about 96 KiB a ticket rather than 64, because a round of a short fragment costs a wavefront
  // nearly what a whole page costs and only a larger share per pick-up makes up for it (fragments of 1.8 KiB on
  // average, 64 slots in flight: 59.6 % of the roofline in tickets of 32, 60.6 % in 40, 61.1 % in 48, 61.3 % in 64).
  return bytes == 0 || b >= 2731ull * n ? 16u : b >= 2048ull * n ? 32u : b >= 1366ull * n ? 48u : 64u;
}
__host__ __device__ __forceinline__ uint32_t ticket_size_for_submission(uint32_t in_flight, uint32_t n,
                                                                        uint32_t bytes, uint32_t workers) {
  if (in_flight >= kManyInFlight && n <= kSmallSubmission) return kSmallSubmission;
  const uint64_t all = static_cast<uint64_t>(in_flight) * n;
  const uint32_t backlog = all > (1u << 20) ? (1u << 20) : static_cast<uint32_t>(all);
  const uint32_t size = ticket_size_for(backlog, workers);
  if (size < kFullTicket) return size;
  const uint32_t full = full_ticket_size(bytes, n);
  if (full > kFullTicket) return full;
  // Whole pages and a backlog that is there but not deep (one comm's sixteen slots of 4 MiB are 34 descriptors per
  // workgroup: every workgroup holds a ticket and has the next one staged, and hardly any wait unclaimed): tickets
  // of 14 make a seventh more of them, and the workgroups run dry less often -- one comm 71.1 -> 72.2 % of the
  // roofline, two to four comms the same as with 16 (72.4-72.5 %).
  return backlog < kDeepBacklog * workers ? 14u : kFullTicket;
}
constexpr uint32_t kMaxDescsPerSubmission = 1u << 20;
constexpr uint32_t kSmallestAdaptiveTicket = 8;  // the least ticket_size_for_submission returns
// The most descriptors one submission may carry: all its tickets must fit the ticket ring at once, or the leader
// could never hand it out (it defers a submission until the ring has room for all of its tickets).
__host__ __device__ constexpr uint32_t max_descs_for(uint32_t fixed_per_ticket) {
  const uint64_t smallest = fixed_per_ticket != 0 ? fixed_per_ticket : kSmallestAdaptiveTicket;
  const uint64_t fit = smallest * kTicketRing;
  return fit < kMaxDescsPerSubmission ? static_cast<uint32_t>(fit) : kMaxDescsPerSubmission;
}
constexpr uint32_t kStopReplicas = 64;
constexpr uint32_t kPollEntries = 16;  // submission entries fetched per load instruction of a leader poll (16 B per lane)
// A poll that finds all sixteen entries there and turns them into tickets at a stroke is followed by a deep poll:
// four loads in flight together, 64 entries for the one PCIe round trip (about 1.5 us) that sixteen cost -- which
// is what capped a storm of one-ticket requests near 9 M/s.
constexpr uint32_t kDeepGroups = 3;    // groups of kPollEntries beyond the first in a deep poll
constexpr uint32_t kStormBacklog = 128;  // entries published beyond a poll's 64 from which the leader takes them in a rolling loop
constexpr uint32_t kAuxProbe = 35;  // lane of an auxiliary load that reads the stamp of an entry ahead
constexpr uint32_t kAuxTicketsDone = 32, kAuxHostStop = 33, kAuxJobsCompleted = 34;  // lanes of the auxiliary load
constexpr uint32_t kNeverIdleOut = 0xFFFFFFFFu;
constexpr uint32_t kDefaultIdlePolls = 400;  // empty polls (about 1.2 us each) before the kernel leaves by itself
constexpr int kTcpxuInProgress = TCPXU_IN_PROGRESS;

// 64-byte record: four 16-byte sectors of three payload words and one stamp word.
struct alignas(64) Record {
  uint32_t w[16];
};
constexpr int kPayloadWords = 12;
__host__ __device__ constexpr int payload_slot(int i) { return (i / 3) * 4 + (i % 3); }
// Submission payload: 0-1 bounce, 2-3 dst, 4-5 descs, 6-7 done_flag, 8-9 done_value, 10 n_descs, 11 payload bytes
//                     (0 = not given).
// Ticket payload:     0-1 bounce, 2-3 dst, 4-5 descs, 6-7 done_flag, 8-9 done_value,
//                     10 n | job << 8 | before << 29 | after << 30 | only << 31, 11 target.
// `only`: the submission's only ticket (the job slot index is below 2^16); `before` / `after`: the submission has
// descriptors before this ticket's first / after its last (in the same array: the fetcher looks at the nearest one
// to decide whether the destination line at that end of the ticket is shared with the neighbouring ticket).
constexpr uint32_t kOnlyTicket = 1u << 31;
constexpr uint32_t kMoreAfter = 1u << 30, kMoreBefore = 1u << 29;
__host__ __device__ __forceinline__ uint32_t neighbour_bits(uint32_t i, uint32_t nt, bool across) {
  return (nt == 1 ? kOnlyTicket : 0u) | (across && i != 0 ? kMoreBefore : 0u) | (across && i + 1 < nt ? kMoreAfter : 0u);
}
// Whether a submission's tickets share destination lines across their ends.  It saves two partial writes of a line
// per ticket boundary and costs every ticket's pick-up two more descriptors to read and look at: worth it when the
// engine is busy (8 MiB workload +0.3 points of the roofline, fragments of 1.8 KiB +0.4), not for a request that is
// alone (4 MiB: 0.3 us more), and pointless where whole pages land on line boundaries anyway (1 MiB requests of
// whole pages: 0.90 -> 0.84 of the roofline with it).  Decided by the leader for the whole submission, so that the
// two tickets at a boundary always agree.
__host__ __device__ __forceinline__ bool shares_across_tickets(uint32_t in_flight, uint32_t n, uint32_t bytes,
                                                               uint32_t dst_lo) {
  const bool whole_pages_on_lines = bytes == n * TCPXU_PAGE_SIZE && (dst_lo & 127u) == 0;
  return in_flight >= kManyInFlight && !whole_pages_on_lines;
}

struct HostCtl {  // mapped host memory
  alignas(64) uint64_t tail;       // host -> GPU: submissions published so far
  alignas(64) uint64_t stop;       // host -> GPU: drain and exit
  alignas(64) uint64_t head;       // GPU -> host: submissions the leader has consumed
  alignas(64) uint64_t completed;  // GPU -> host: submissions fully unpacked (mirrored when idle and at exit)
  alignas(64) uint64_t exited;     // GPU -> host: 0 running, 1 stopped on request, 2 left after being idle
  alignas(64) uint64_t exiting;    // GPU -> host: the leader is about to leave for idleness (see leader_loop)
  // GPU -> host, written by the leader when it leaves: its polls of the ring, the entries they consumed and the
  // polls that fetched 64 entries instead of 16, since the engine was created.
  alignas(64) uint64_t leader_polls;
  uint64_t leader_entries;
  uint64_t leader_deep_polls;
  alignas(64) Record ring[1];      // ring_entries follow
};

struct alignas(256) StopWord {
  uint32_t value;
};

struct DevState {  // device memory
  static constexpr uint32_t kTickets = kTicketRing;
  static constexpr uint32_t kStops = kStopReplicas;
  alignas(64) uint64_t ticket_head;     // next ticket number to claim
  alignas(64) uint64_t tickets_done;    // tickets whose payload is written
  alignas(64) uint64_t jobs_completed;  // submissions completed since creation
  alignas(64) uint64_t sub_head;        // leader-private: next submission index
  uint64_t tickets_out;                 // leader-private: tickets written so far
  uint64_t leader_polls, leader_entries, leader_deep_polls;  // leader-private: running totals (see HostCtl)
  alignas(64) uint32_t exited_wgs;      // reset at every start, as are the stop words
  uint32_t exit_reason;
  alignas(256) StopWord stop[kStopReplicas];
  alignas(64) Record tickets[kTicketRing];
  // uint32_t jobs_done[ring_entries], then uint32_t job_target[ring_entries] follow
};

// The same roles for one slot handed out by one ordinary launch (tcpxuUnpackSlotNoAlloc): tickets 0 .. n-1 are
// written by a small kernel before the workers start, there is no leader and no stop word is ever raised.
constexpr uint32_t kOneShotTicketSize = 8;  // one fragment per copy wavefront: the most workgroups per slot
constexpr uint32_t kOneShotTickets = TCPXU_SLOT_PAGES / kOneShotTicketSize;
struct OneShotState {
  static constexpr uint32_t kTickets = kOneShotTickets;
  static constexpr uint32_t kStops = 1;
  alignas(64) uint64_t ticket_head;
  alignas(64) uint64_t tickets_done;
  alignas(64) uint64_t jobs_completed;
  alignas(64) uint32_t jobs_done[16];  // [0]: tickets of the slot counted so far
  alignas(64) uint64_t unused_flag;    // completion word of a caller that passed none
  // The call's completion word and value, for a workgroup that gives up (see worker_loop's look limit): it cannot
  // have them from a ticket, because a ticket is what it did not find.
  uint64_t flag_addr, flag_value;
  alignas(256) StopWord stop[kStops];
  alignas(64) Record tickets[kOneShotTickets];
};
static_assert((kOneShotTickets & (kOneShotTickets - 1)) == 0, "ticket numbers are masked");

// ---- scoped memory operations -------------------------------------------------------------------------------------
#define SYS __HIP_MEMORY_SCOPE_SYSTEM

template <typename T>
__device__ __forceinline__ T sys_load(const T* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, SYS);
}
template <typename T>
__device__ __forceinline__ void sys_store(T* p, T v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, SYS);
}
// The same for memory that is known to be global (device memory, mapped host memory), said outright: where the
// compiler cannot see that -- a pointer that arrived as a function's argument -- it would emit a flat_ store, which
// the hardware is free to complete out of turn among a wavefront's memory instructions.
template <typename T>
__device__ __forceinline__ void sys_store_global(T* p, T v) {
  __hip_atomic_store((TCPXU_GLOBAL T*)p, v, __ATOMIC_RELAXED, SYS);  // (only a C-style cast changes the address space)
}
__device__ __forceinline__ void drain_memory_ops() { asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory"); }

__device__ __forceinline__ uint32_t bcast(uint32_t v, uint32_t src_lane) {
  return __shfl(v, static_cast<int>(src_lane), kWaveLanes);
}
__device__ __forceinline__ uint64_t bcast64(uint64_t v, uint32_t src_lane) {
  return (static_cast<uint64_t>(bcast(static_cast<uint32_t>(v >> 32), src_lane)) << 32) |
         bcast(static_cast<uint32_t>(v), src_lane);
}
// ---- leader -------------------------------------------------------------------------------------------------------
// Runs on wavefront 0 of workgroup 0.  All control flow is wave-uniform.
__device__ __forceinline__ uint32_t lane_value(uint32_t v, uint32_t src_lane) {
  return static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(v), static_cast<int>(src_lane)));
}

// Stamps (optional, tcpxuEngineEnableStamps): four 64-bit readings of the GPU's constant-rate clock per job slot, in
// device memory that the host has filled with ones -- [0] the leader saw the submission, [1] the first of its
// tickets was fetched by a workgroup, [2] the first workgroup had its descriptors staged (both kept as minima),
// [3] the workgroup that completed the submission had its last store acknowledged.
constexpr uint32_t kStampsPerJob = 4;
__device__ __forceinline__ uint64_t clock_now() { return wall_clock64(); }

// What the four lanes of an entry know about it, for the sixteen entries of one group at once.
struct EntryView {
  uint32_t n, bytes, per_ticket, target_prev, in_flight, slot;
  bool sane, slot_free;
};

// Every entry of a group fits one ticket (a storm of small requests): the leading run of them becomes tickets in
// one store instruction.  Returns the length of the run; `room` is what the ticket ring still takes.
__device__ __forceinline__ uint32_t write_single_tickets_of_group(DevState* st, uint32_t* job_target, uint64_t* stamps,
                                                                  uint64_t& tickets_out, uint32_t lane, const EntryView& v,
                                                                  const u32x4& sc, uint32_t room) {
  const uint32_t k_of_lane = lane >> 2;
  const uint64_t not_now = ~__ballot(v.sane && v.slot_free);
  uint32_t run = not_now == 0 ? kPollEntries : static_cast<uint32_t>(__builtin_ctzll(not_now)) >> 2;
  run = std::min(run, room);
  if (run != 0) {
    if (k_of_lane < run) {
      const uint64_t t = tickets_out + k_of_lane;
      const uint32_t stamp = static_cast<uint32_t>(t + 1);
      const uint32_t target = v.target_prev + 1u;
      u32x4 out{sc.x, sc.y, sc.z, stamp};
      if ((lane & 3u) == 3) {
        out.y = v.n | (v.slot << 8) | kOnlyTicket;
        out.z = target;
        sys_store_global(&job_target[v.slot], target);
        if (stamps) sys_store_global(&stamps[kStampsPerJob * v.slot], clock_now());
      }
      store_vec_sys(reinterpret_cast<uint8_t*>(&st->tickets[t & (kTicketRing - 1)]) + 16 * (lane & 3u), out);
    }
    tickets_out += run;
  }
  return run;
}

// Every lane takes the value that lane q of its own group of four holds: one move, no trip through the LDS.
template <int q>
__device__ __forceinline__ uint32_t quad_value(uint32_t v) {
  static_assert(q >= 0 && q < 4, "a lane of the quad");
  return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), q * 0x55, 0xF, 0xF, false));
}

__device__ __forceinline__ uint64_t same_in_all_lanes64(uint64_t v) {
  return (static_cast<uint64_t>(static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(v >> 32)))) << 32) |
         static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(v)));
}
template <typename T>
__device__ __forceinline__ T* same_in_all_lanes_ptr(T* p) {
  return reinterpret_cast<T*>(same_in_all_lanes64(reinterpret_cast<uint64_t>(p)));
}

// A storm: a deep poll turned all its 64 entries into tickets and the host has published kStormBacklog entries beyond
// them -- or a poll wrote several tickets for each of its sixteen entries, none of them large, and more of the kind
// may wait.  Takes entries from s on for as long as they are published and are one ticket each; returns where it
// got to, which is where it started if the first group was not for it.
//
// kGroups (five) groups of sixteen entries are in flight at a time, and the registers of a group that has gone through
// take the group 16 x kGroups entries on at once (every group's loads bring the stamp of the last entry of the group
// that would be asked for next: entries are published in order, so if that one is there the whole group is).  The
// leader's time per group is then a fifth of the round trip to the host's ring or what it takes to turn a group into
// tickets, whichever is longer -- not their sum as in a poll (1024 requests of 64 KiB in flight: 21 -> 44 M
// requests/s, where the copy itself becomes the bound).  Every group has registers of its own (moving one that is
// still in flight to another register would wait for it), hence one step unrolled per group, with every index into
// the groups' arrays a constant.  When the host's tail is reached nothing more is asked for and the groups in flight
// go through: the loop ends with nothing in flight.
//
// The compiler would wait for everything in flight at the top of such a loop.  So the loop's loads are written as
// instructions, which it does not track, and each step waits for its own group by count: the memory instructions of
// a wavefront complete in the order issued, and between a group's loads and its turn the other kGroups - 1 groups
// have had theirs, each with two stores (the tickets, their job slots' targets) and, while the loop feeds, two loads:
// 4 x (kGroups - 1) instructions at the least, so "at most that many outstanding" means that the group's own loads
// have landed.  (More are issued when stamps are on, and the head word once a round: counting too few only waits for
// a little more than is needed; fewer would let a group be read before it has landed, so this function must not
// spill registers to memory -- the build checks the compiler's resource report for 0 bytes of scratch.)  Once the
// loop has stopped feeding, a group waits for everything.  The group's registers pass through a statement after the
// wait so that nothing reads them before it.
//
// A function of its own, not inlined, and called from the top of the leader's loop where little is live: with this
// loop inside the leader's, what the compiler did with the registers around it made every poll that never sees a
// storm 0.2 us slower.  The running count of finished tickets is read once: too few counted as done only ends the
// storm early (after at most kTicketRing entries, which is also how long the host's stop word can go unread).
struct StormEnd {
  uint64_t s, tickets_out;
  uint32_t entries;  // taken off the ring
};
__device__ __attribute__((noinline)) StormEnd leader_storm(HostCtl* ctl_in, DevState* st_in, uint32_t* jobs_done_in,
                                                          uint64_t* stamps_in, uint32_t ring_mask_in,
                                                          uint32_t fixed_per_ticket_in, uint64_t s_in, uint64_t tickets_out_in) {
  // Arguments arrive in vector registers.  These are the same in every lane and go back to scalar registers.  (The job
  // slots' targets follow their counts in memory: one pointer for both.)
  HostCtl* ctl = same_in_all_lanes_ptr(ctl_in);
  DevState* st = same_in_all_lanes_ptr(st_in);
  uint32_t* jobs_done = same_in_all_lanes_ptr(jobs_done_in);
  uint64_t* stamps = same_in_all_lanes_ptr(stamps_in);
  const uint32_t ring_mask = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(ring_mask_in)));
  uint32_t* job_target = jobs_done + ring_mask + 1u;
  const uint32_t fixed_per_ticket = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(fixed_per_ticket_in)));
  uint64_t s = same_in_all_lanes64(s_in);
  uint64_t tickets_out = same_in_all_lanes64(tickets_out_in);
  const uint32_t lane = threadIdx.x;
  const uint32_t k_of_lane = lane >> 2;
  uint32_t consumed = 0, entries = 0;
  // Groups in flight: the round trip to the host's ring, 1.55 us, over what a group costs to turn into tickets, 0.36 us,
  // and one more.  (1024 requests of 64 KiB in flight: 40.3 M/s with four, 44.6 with five -- where the copy itself is
  // the bound -- and 45.5 with six, which spills registers; 384 in flight: 29.4, 27.2, 26.4.)
  constexpr uint32_t kGroups = 5;
  // The four lanes that hold an entry's sectors also fetch what is known of its job slot -- tickets counted as done
  // (first lane), tickets ever issued (second) -- so that both reach all four with a move inside the quad; the other two
  // lanes read the stamp of the last entry of the group that would be asked for next (the probe).  What of a lane's two
  // addresses does not change from group to group is worked out once (and hidden from the compiler, which would work
  // it out again with a branch per kind of lane in every step): address = base + (((s_g + add) & ring_mask) << shift).
  const uint32_t kind = lane & 3;
  uint64_t entry_base = reinterpret_cast<uint64_t>(&ctl->ring[0]) + 16 * kind;
  uint64_t aux_base = kind == 0   ? reinterpret_cast<uint64_t>(jobs_done)
                      : kind == 1 ? reinterpret_cast<uint64_t>(job_target)
                                  : reinterpret_cast<uint64_t>(&ctl->ring[0].w[15]);
  uint32_t aux_add = kind < 2 ? k_of_lane : (kGroups + 1) * kPollEntries - 1;
  uint32_t aux_shift = kind < 2 ? 2 : 6;
  static_assert(sizeof(Record) == 64 && sizeof(uint32_t) == 4, "the shifts above");
  asm volatile("" : "+v"(entry_base), "+v"(aux_base), "+v"(aux_add), "+v"(aux_shift));
  auto fetch_group_untracked = [&](u32x4& sc, uint32_t& ax, uint64_t s_g) {
    const uint32_t at_s = static_cast<uint32_t>(s_g);  // (the mask keeps low bits only)
    const uint64_t entry = entry_base + (static_cast<uint64_t>((at_s + k_of_lane) & ring_mask) << 6);
    const uint64_t at = aux_base + (static_cast<uint64_t>((at_s + aux_add) & ring_mask) << aux_shift);
    // (The job slots' words first: loads return in the order issued, so entries that are there whole -- every sector
    // carries its stamp -- vouch for the words that were asked for before them.)
    asm volatile("global_load_dword %0, %1, off sc0 sc1" : "=v"(ax) : "v"(at) : "memory");
    asm volatile("global_load_dwordx4 %0, %1, off sc0 sc1" : "=v"(sc) : "v"(entry) : "memory");
  };
  // kGroups while the loop feeds (that many groups in flight); once it has caught up with the host, the groups still
  // in flight that have not gone through: kGroups - 1, ..., 1, and at 0 the storm is over.
  uint32_t feeding = kGroups;
  u32x4 sc[kGroups];
  uint32_t ax[kGroups], tickets_done;
  bool queue_deep = false;
  // The first groups, from s on, and the running count of finished tickets: one round trip, waited for whole.
  auto arm = [&]() {
    feeding = kGroups;
#pragma unroll
    for (uint32_t g = 0; g < kGroups; ++g) fetch_group_untracked(sc[g], ax[g], s + g * kPollEntries);
    asm volatile("global_load_dword %0, %1, off sc0 sc1" : "=v"(tickets_done) : "v"(reinterpret_cast<const uint32_t*>(&st->tickets_done)) : "memory");
    asm volatile("s_waitcnt vmcnt(0)" : "+v"(tickets_done) : : "memory");
#pragma unroll
    for (uint32_t g = 0; g < kGroups; ++g) asm volatile("" : "+v"(sc[g]), "+v"(ax[g]) : : "memory");
    tickets_done = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(tickets_done)));
    // The first group's probe: the 16 x (kGroups + 1) entries from s on are published, so the queue at the leader is deep.
    queue_deep = lane_value(ax[0], 2) == static_cast<uint32_t>(s + (kGroups + 1) * kPollEntries);
  };
  // One group through; false when the storm is over: nothing more in flight, or the group was not there whole or not
  // all of one ticket each (then whatever is in flight is dropped, and the leader's next poll asks again).
  auto pass = [&](u32x4& sc, uint32_t& ax) {
    // (While the loop feeds, the kGroups - 1 steps before this one all fed: it stops feeding once and for all.  The
    // first groups have landed, whichever wait they get.)
    if (feeding == kGroups) asm volatile("s_waitcnt vmcnt(%0)" : : "n"((kGroups - 1) * 4) : "memory");
    else asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
    asm volatile("" : "+v"(sc), "+v"(ax) : : "memory");
    const uint64_t s_g = s + consumed;
    const uint64_t okm = __ballot(sc.w == static_cast<uint32_t>(s_g + k_of_lane + 1));
    uint32_t run = 0;
    if ((okm & 0xFull) == 0xFull) {
      const uint32_t left = kTicketRing - (static_cast<uint32_t>(tickets_out) - tickets_done);
      // With hundreds of submissions waiting, one of at most 32 descriptors is one ticket (see
      // ticket_size_for_submission; a fixed ticket size says so itself) -- and when the loop was armed with the entry
      // 16 x (kGroups + 1) ahead published, so is one of as many descriptors as a ticket holds: every workgroup has
      // work anyway, and a ticket per entry is what lets the leader keep up (1024 requests of 33 whole pages in
      // flight: 5.8 -> 33 M requests/s).  No sizing here, and a group with a larger one ends the storm and goes the
      // ordinary way.
      EntryView more;
      more.n = quad_value<3>(sc.y);  // payload word 10 sits in .y of sector 3
      more.bytes = 0, more.per_ticket = 0, more.in_flight = 0;  // (not looked at by write_single_tickets_of_group)
      more.target_prev = quad_value<1>(ax);
      more.sane = ((okm >> (4 * k_of_lane)) & 0xFull) == 0xFull && more.n - 1u < kMaxDescsPerSubmission;
      more.slot_free = quad_value<0>(ax) == more.target_prev;
      more.slot = static_cast<uint32_t>(s_g + k_of_lane) & ring_mask;
      const uint32_t one_ticket = fixed_per_ticket != 0 ? fixed_per_ticket : queue_deep ? kMaxDescsPerTicket : kSmallSubmission;
      if (__ballot(more.sane && more.n > one_ticket) == 0) run = write_single_tickets_of_group(st, job_target, stamps, tickets_out, lane, more, sc, left);
    }
    consumed += run;
    if (run != kPollEntries) return false;
    if (feeding == kGroups) {
      const uint64_t next = s_g + kGroups * kPollEntries;
      if (lane_value(ax, 2) == static_cast<uint32_t>(next + kPollEntries)) fetch_group_untracked(sc, ax, next);
      else feeding = kGroups - 1;
    } else {
      --feeding;
    }
    feeding = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(feeding)));
    return feeding != 0;
  };
  auto round = [&]() {
#pragma unroll
    for (uint32_t g = 0; g < kGroups; ++g)
      if (!pass(sc[g], ax[g])) return false;
    return true;
  };
#pragma unroll 1
  for (;;) {
    arm();
#pragma unroll 1
    for (;;) {
      if (!round()) break;
      // a round of entries on: the host learns of it
      s += consumed;
      entries += consumed;
      consumed = 0;
      if (lane == 0) sys_store_global(&ctl->head, s);
    }
    // Whatever is still in flight is waited for, so that the registers it lands in are free.
    asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
#pragma unroll
    for (uint32_t g = 0; g < kGroups; ++g) asm volatile("" : "+v"(sc[g]), "+v"(ax[g]) : : "memory");
    if (consumed != 0) {  // the round that the loop ended in
      s += consumed;
      entries += consumed;
      consumed = 0;
      if (lane == 0) sys_store_global(&ctl->head, s);
    }
    // Caught up with the host, every group in flight gone through whole (16 x kGroups entries at the least since the
    // loop was armed): the host publishes as requests complete, so more is on its way -- ask again from here instead of
    // leaving, waiting for the ordinary loop to find 64 entries and as many again beyond them, and coming back.
    // Anything else -- a group not there whole, entries of more than one ticket, no room in the ticket ring --
    // is for the ordinary loop.
    if (feeding != 0) break;
  }
  return StormEnd{s, tickets_out, entries};
}

__device__ void leader_loop(HostCtl* ctl, DevState* st, uint32_t* jobs_done, uint32_t* job_target,
                            uint32_t ring_mask, uint32_t fixed_per_ticket, uint32_t spin_limit, uint64_t* stamps) {
  // The leader's positions are the same in every lane: said outright, so that they stay in scalar registers (in
  // vector registers the compiler waits for the leader's own stores at the top of every pass).
  auto same_in_all_lanes = [](uint64_t v) {
    return (static_cast<uint64_t>(static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(v >> 32)))) << 32) |
           static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(v)));
  };
  uint64_t s = same_in_all_lanes(sys_load(&st->sub_head));
  uint64_t tickets_out = same_in_all_lanes(sys_load(&st->tickets_out));
  uint64_t mirrored = ~0ull;
  // Read once: the grid's size comes from the dispatch packet, a scalar load with a wait behind it wherever it is asked.
  const uint32_t workers = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(gridDim.x - 1)));
  uint64_t idle = 0;
  uint32_t reason = 0;
  uint32_t polls = 0, entries = 0, deep_polls = 0;  // of this launch; added to the running totals at the end
  // The next poll fetches 64 entries.  (A ring of fewer entries than that never has them.)
  bool deep = false;
  bool storm_next = false;
  uint32_t storm_backoff = 0, storm_backoff_len = 4;  // polls until the rolling loop is next tried from the several-tickets way
  const bool ring_allows_deep = ring_mask + 1u >= (kDeepGroups + 1) * kPollEntries;
  const bool ring_allows_storm = ring_mask + 1u >= 2 * ((kDeepGroups + 1) * kPollEntries + kStormBacklog);
  // Fixed per-lane roles in the auxiliary load (second load of every poll), so that both loads of a poll are
  // issued back to back by all lanes and waited for once:
  //   lanes 0-15  jobs_done of the job slots of entries s..s+15    lanes 16-31  job_target of the same slots
  //   lane 32     low word of tickets_done                         lane 33      low word of the host stop word
  //   lane 34     low word of jobs_completed                       other lanes repeat lane 33.
  const uint32_t* const tickets_done_lo = reinterpret_cast<const uint32_t*>(&st->tickets_done);
  const uint32_t* const host_stop_lo = reinterpret_cast<const uint32_t*>(&ctl->stop);
  const uint32_t* const jobs_completed_lo = reinterpret_cast<const uint32_t*>(&st->jobs_completed);

  for (;;) {
    // (Every 64 entries it takes count as one deep poll in this launch's figures.)
    if (storm_next) {
      storm_next = false;
      const StormEnd end = leader_storm(ctl, st, jobs_done, stamps, ring_mask, fixed_per_ticket, s, tickets_out);
      s = same_in_all_lanes(end.s);
      tickets_out = same_in_all_lanes(end.tickets_out);
      entries += end.entries;
      polls += (end.entries + (kDeepGroups + 1) * kPollEntries - 1) / ((kDeepGroups + 1) * kPollEntries);
      deep_polls += (end.entries + (kDeepGroups + 1) * kPollEntries - 1) / ((kDeepGroups + 1) * kPollEntries);
      deep = ring_allows_deep;
      // Nothing taken: the queue was not deep, or what waits is not for that loop.  Wait longer each time before
      // asking again (an attempt costs a round trip), and start over once it has worked.
      storm_backoff_len = end.entries != 0 ? 4u : std::min(2u * storm_backoff_len, 256u);
      storm_backoff = end.entries != 0 ? 0u : storm_backoff_len;
    } else if (storm_backoff != 0) {
      --storm_backoff;
    }
    // What depends on the lane is worked out afresh in every pass (the empty statement hides from the compiler that
    // the lane is the same each time): a dozen per-lane addresses kept in registers for the life of the loop are
    // what would push the kernel beyond the 80 vector registers that let two workgroups share a compute unit, and a
    // pass waits a microsecond for the host's memory anyway.
    uint32_t lane = threadIdx.x;
    asm volatile("" : "+v"(lane));
    // One round trip fetches entries s .. s+15: lane 4k+j reads sector j (three payload words and the stamp) of
    // entry s+k.
    const uint32_t k_of_lane = lane >> 2;
    const u32x4 sect = load_vec_sys(reinterpret_cast<const uint8_t*>(&ctl->ring[(s + k_of_lane) & ring_mask]) + 16 * (lane & 3));
    const uint32_t* aux_addr = host_stop_lo;
    if (lane < kPollEntries) aux_addr = &jobs_done[(s + lane) & ring_mask];
    else if (lane < 2 * kPollEntries) aux_addr = &job_target[(s + lane - kPollEntries) & ring_mask];
    else if (lane == kAuxTicketsDone) aux_addr = tickets_done_lo;
    else if (lane == kAuxJobsCompleted) aux_addr = jobs_completed_lo;
    const uint32_t aux = sys_load(aux_addr);
    // A deep poll: entries s+16 .. s+63 and their job slots' counters ride along in the same round trip.
    u32x4 sect_more[kDeepGroups];
    uint32_t aux_more[kDeepGroups];
#pragma unroll
    for (uint32_t g = 0; g < kDeepGroups; ++g) {
      sect_more[g] = u32x4{0u, 0u, 0u, 0u};
      aux_more[g] = 0;
    }
    if (deep) {
#pragma unroll
      for (uint32_t g = 0; g < kDeepGroups; ++g) {
        const uint64_t s_g = s + (g + 1) * kPollEntries;
        sect_more[g] = load_vec_sys(reinterpret_cast<const uint8_t*>(&ctl->ring[(s_g + k_of_lane) & ring_mask]) + 16 * (lane & 3));
        // (The upper lanes of the last group's load read the stamp of the entry kStormBacklog beyond the poll's 64.)
        if (lane < 2 * kPollEntries || g == kDeepGroups - 1)
          aux_more[g] = sys_load(lane < kPollEntries       ? &jobs_done[(s_g + lane) & ring_mask]
                                 : lane < 2 * kPollEntries ? &job_target[(s_g + lane - kPollEntries) & ring_mask]
                                                           : &ctl->ring[(s_g + kPollEntries + kStormBacklog - 1) & ring_mask].w[15]);
      }
      ++deep_polls;
    }
    ++polls;

    const uint32_t expect = static_cast<uint32_t>(s + k_of_lane + 1);
    const uint64_t ok_mask = __ballot(sect.w == expect);
    // Entries of this poll that are there, counted from the first: lane 4k tells whether all four sectors of entry
    // k are.  Eight or more mean that submissions queue up at the leader itself.
    const uint64_t whole = ok_mask & (ok_mask >> 1) & (ok_mask >> 2) & (ok_mask >> 3) & 0x1111111111111111ull;
    const uint64_t missing = ~whole & 0x1111111111111111ull;
    const uint32_t ready = missing != 0 ? static_cast<uint32_t>(__builtin_ctzll(missing)) >> 2 : kPollEntries;
    const bool leader_behind = ready >= kLeaderBehind;
    const uint32_t tickets_done = lane_value(aux, kAuxTicketsDone);
    const uint32_t jobs_completed = lane_value(aux, kAuxJobsCompleted);
    // Payload word i of entry k: component i % 3 of sector i / 3, held by lane 4k + i / 3.
    auto payload_of = [&](uint32_t first_lane, int i) {
      const uint32_t src = first_lane + static_cast<uint32_t>(i / 3);
      return lane_value(i % 3 == 0 ? sect.x : i % 3 == 1 ? sect.y : sect.z, src);
    };

    // Sixteen at a stroke.  The four lanes that hold an entry's sectors hold nearly all of its tickets' words
    // already -- the two records share their layout up to the descriptor pointer and the last sector -- so they
    // write the entry's tickets themselves, ticket i of every entry of the leading run in pass i of one short loop:
    // sixteen submissions of sixteen tickets cost sixteen store instructions, where a pass of the loop below for
    // each (it fetches an entry's words from their lanes into scalars first: about half a microsecond) capped a
    // stream of 1 MiB requests at 2 M/s and a storm of 64 KiB requests at 1.6 M/s.  Taken when the run has some
    // width: a lone entry of many tickets is written faster by the loop below, sixteen tickets to the instruction.
    // (Not for a lone entry of more descriptors than a ticket holds, nor for a first entry of more than 32 tickets of
    // the size its payload asks for -- 512 whole pages, up to 2048 short fragments: nothing here would apply to
    // them, and what is worked out per lane first would only add to their latency.)
    uint32_t consumed = 0;
    bool deep_next = false;
    const uint32_t n_first = lane_value(sect.y, 3);
    const uint32_t lane_tickets_hold = kLaneTickets * (fixed_per_ticket != 0 ? fixed_per_ticket : full_ticket_size(lane_value(sect.z, 3), n_first));
    auto view_entries = [&](const u32x4& sc, uint32_t ax, uint64_t s0, uint64_t okm) {
      EntryView v;
      v.n = bcast(sc.y, lane | 3u);      // payload word 10 sits in .y of sector 3
      v.bytes = bcast(sc.z, lane | 3u);  // payload word 11 sits in .z of sector 3
      const bool all_sectors = ((okm >> (4 * k_of_lane)) & 0xFull) == 0xFull;
      const uint32_t done_now = bcast(ax, k_of_lane);
      v.target_prev = bcast(ax, kPollEntries + k_of_lane);
      v.in_flight = static_cast<uint32_t>(s0 + k_of_lane) - jobs_completed + 1u;
      v.per_ticket = fixed_per_ticket != 0 ? fixed_per_ticket : ticket_size_for_submission(v.in_flight, v.n, v.bytes, workers);
      if (fixed_per_ticket == 0 && leader_behind && v.per_ticket < kFullTicket) v.per_ticket = kFullTicket;  // see below
      v.sane = all_sectors && v.n - 1u < kMaxDescsPerSubmission;  // 1 .. 2^20 descriptors
      v.slot_free = done_now == v.target_prev;  // every ticket ever issued for the job slot has been counted
      v.slot = static_cast<uint32_t>(s0 + k_of_lane) & ring_mask;
      return v;
    };
    auto write_single_tickets = [&](const EntryView& v, const u32x4& sc, uint32_t room) {
      return write_single_tickets_of_group(st, job_target, stamps, tickets_out, lane, v, sc, room);
    };
    if ((ok_mask & 0xFull) == 0xFull &&  // entry s is there
        (n_first <= kMaxDescsPerTicket || (ready >= 2 && n_first <= lane_tickets_hold))) {
      const EntryView ev = view_entries(sect, aux, s, ok_mask);
      const uint32_t n = ev.n, bytes = ev.bytes, per_ticket = ev.per_ticket, target_prev = ev.target_prev;
      const uint32_t in_flight = ev.in_flight, slot = ev.slot;
      const bool sane = ev.sane, slot_free = ev.slot_free;
      // The ticket ring has room while fewer than its size are outstanding (32-bit wrapping arithmetic).
      const uint32_t room = kTicketRing - (static_cast<uint32_t>(tickets_out) - tickets_done);
      const uint32_t sector = lane & 3u;
      if (__ballot(sane && n > per_ticket) == 0) {
        consumed = write_single_tickets(ev, sect, room);
        if (deep && consumed == kPollEntries) {
          // The groups that rode along, in order, each as long as the one before it went through whole.  One loop
          // body that the groups pass through in turn (the registers rotate), so that the three are not worked out
          // side by side in three times the registers: the kernel must stay within 80 for two workgroups per
          // compute unit.
          uint32_t left = room - consumed;
          u32x4 sc0 = sect_more[0], sc1 = sect_more[1], sc2 = sect_more[2];
          uint32_t ax0 = aux_more[0], ax1 = aux_more[1], ax2 = aux_more[2];
          static_assert(kDeepGroups == 3, "the rotation below");
#pragma unroll 1
          for (uint32_t g = 0; g < kDeepGroups; ++g) {
            const uint64_t s_g = s + consumed;
            const uint64_t okm = __ballot(sc0.w == static_cast<uint32_t>(s_g + k_of_lane + 1));
            uint32_t run = 0;
            if ((okm & 0xFull) == 0xFull) {
              const EntryView more = view_entries(sc0, ax0, s_g, okm);
              if (__ballot(more.sane && more.n > more.per_ticket) == 0) run = write_single_tickets(more, sc0, left);
            }
            consumed += run;
            left -= run;
            if (run != kPollEntries) break;
            sc0 = sc1, sc1 = sc2;
            ax0 = ax1, ax1 = ax2;
          }
        }
        deep_next = ring_allows_deep && consumed >= kPollEntries;
        // All 64 entries of a deep poll became tickets and the entry kStormBacklog beyond them is published (entries
        // are published in order, so everything up to it is there): a storm, taken from the top of the next pass.  How
        // far the host has got is read off the ring itself: the host's tail word is a line that the host writes with
        // every publish, and a poll that reads it as well waits half a microsecond longer for it.
        storm_next = ring_allows_storm && consumed == (kDeepGroups + 1) * kPollEntries &&
                     lane_value(aux_more[kDeepGroups - 1], kAuxProbe) == static_cast<uint32_t>(s + (kDeepGroups + 1) * kPollEntries + kStormBacklog);
      } else if (ready >= 2 && n_first <= kLaneTickets * lane_value(per_ticket, 0)) {
        // Several entries, some of more than one ticket, the first of them not too many.  (The empty statement keeps
        // the compiler from working this block's division and lane exchanges out ahead of the branch, where every
        // poll would pay for them.)
        uint32_t n_here = n, per_here = per_ticket;
        asm volatile("" : "+v"(n_here), "+v"(per_here));
        const uint32_t nt = sane ? tickets_for(n_here, per_here) : 0u;
        const bool regular = sane && nt <= kLaneTickets && slot_free;
        const uint64_t irregular = ~__ballot(regular);
        const uint32_t run_regular = irregular == 0 ? kPollEntries : static_cast<uint32_t>(__builtin_ctzll(irregular)) >> 2;
        // Tickets of the entries before this one and up to this one (the four lanes of an entry hold the same values).
        const uint32_t mine = k_of_lane < run_regular ? nt : 0u;
        uint32_t upto = mine, most = mine;
#pragma unroll
        for (uint32_t d = 4; d < kWaveLanes; d <<= 1) {
          const uint32_t below = static_cast<uint32_t>(__shfl_up(static_cast<int>(upto), d, kWaveLanes));
          if (lane >= d) upto += below;
          most = std::max(most, static_cast<uint32_t>(__shfl_xor(static_cast<int>(most), static_cast<int>(d), kWaveLanes)));
        }
        const uint64_t no_room = ~__ballot(k_of_lane < run_regular && upto <= room);
        const uint32_t run = no_room == 0 ? kPollEntries : static_cast<uint32_t>(__builtin_ctzll(no_room)) >> 2;
        const uint32_t total = run != 0 ? lane_value(upto, 4 * run - 4) : 0u;
        // Taken when the run has some width (`most` is over the regular run, which the room may have cut: an upper
        // bound, good enough for the choice): a lone entry of many tickets is written faster by the loop below.
        if (run != 0 && total >= 2 * most) {
          const uint32_t target = target_prev + nt;
          const bool across = shares_across_tickets(in_flight, n, bytes, bcast(sect.z, lane & ~3u));  // dst_lo: .z of sector 0
          const uint64_t first_ticket = tickets_out + (upto - mine);
          const bool takes_part = k_of_lane < run;
          for (uint32_t i = 0; __ballot(takes_part && i < nt) != 0; ++i) {
            if (takes_part && i < nt) {
              const uint64_t t = first_ticket + i;
              const uint32_t stamp = static_cast<uint32_t>(t + 1);
              u32x4 v{sect.x, sect.y, sect.z, stamp};
              if (sector == 1) {  // dst_hi, then where this ticket's descriptors start
                const uint64_t d = ((static_cast<uint64_t>(sect.z) << 32) | sect.y) +
                                   static_cast<uint64_t>(i) * per_ticket * sizeof(tcpxuLoadMeta);
                v.y = static_cast<uint32_t>(d);
                v.z = static_cast<uint32_t>(d >> 32);
              }
              if (sector == 3) {  // val_hi, then the ticket's own words
                v.y = std::min(per_ticket, n - i * per_ticket) | (slot << 8) | neighbour_bits(i, nt, across);
                v.z = target;
              }
              store_vec_sys(reinterpret_cast<uint8_t*>(&st->tickets[t & (kTicketRing - 1)]) + 16 * sector, v);
            }
          }
          if (takes_part && sector == 3) {
            sys_store(&job_target[slot], target);
            if (stamps) sys_store(&stamps[kStampsPerJob * slot], clock_now());
          }
          tickets_out += static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(total)));
          consumed = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(run)));
          // Sixteen entries of a few tickets each, the first of them of no more descriptors than one ticket holds: if
          // hundreds more wait, the rolling loop makes one ticket of each such entry (asked once in a while).
          storm_next = consumed == kPollEntries && n_first <= kMaxDescsPerTicket && ring_allows_storm && storm_backoff == 0;
        }
      }
    }
#pragma unroll 1
    for (uint32_t k = consumed; k < kPollEntries; ++k) {
      if (((ok_mask >> (4 * k)) & 0xFull) != 0xFull) break;
      const uint32_t fl = 4 * k;  // first lane of entry k
      const uint32_t n = payload_of(fl, 10);
      if (n == 0) {
        const uint32_t flag_lo = payload_of(fl, 6), flag_hi = payload_of(fl, 7);
        const uint32_t val_lo = payload_of(fl, 8), val_hi = payload_of(fl, 9);
        if (lane == 0) {
          sys_store(reinterpret_cast<uint64_t*>((static_cast<uint64_t>(flag_hi) << 32) | flag_lo),
                    (static_cast<uint64_t>(val_hi) << 32) | val_lo);
          __hip_atomic_fetch_add(&st->jobs_completed, 1ull, __ATOMIC_RELAXED, SYS);
        }
      } else {
        // Submissions not yet completed, this one included, taken to be as long as this one.
        const uint32_t in_flight = static_cast<uint32_t>(s + k) - jobs_completed + 1u;
        uint32_t per_ticket = fixed_per_ticket != 0
                                  ? fixed_per_ticket
                                  : ticket_size_for_submission(in_flight, n, payload_of(fl, 11), workers);
        // Small tickets spread a small backlog over many workgroups, at the price of more tickets to write.  When
        // submissions queue up at the leader, its time per submission is what limits the engine, not the spread:
        // a stream of 1 MiB requests of 256 whole pages, 64 in flight, is served at 1.44 M/s in tickets of 8 (which
        // the backlog alone asks for: the workers empty it as fast as it comes), at 1.96 M/s in tickets of 16, and at
        // 1.64 M/s with this rule, which holds for part of the time.
        if (fixed_per_ticket == 0 && leader_behind && per_ticket < kFullTicket) per_ticket = kFullTicket;
        const uint32_t nt = tickets_for(n, per_ticket);
        const uint32_t slot = static_cast<uint32_t>(s + k) & ring_mask;
        const uint32_t done_now = lane_value(aux, k);
        const uint32_t target_prev = lane_value(aux, kPollEntries + k);
        // The job slot is free once every ticket ever issued for it has been counted; the ticket ring has room
        // while fewer than its size are outstanding (32-bit wrapping arithmetic).  Otherwise leave this entry
        // for a later poll.
        if (done_now != target_prev) break;
        if (static_cast<uint32_t>(tickets_out) + nt - tickets_done > kTicketRing) break;
        const uint32_t target = target_prev + nt;
        if (lane == 0) {
          sys_store(&job_target[slot], target);
          if (stamps) sys_store(&stamps[kStampsPerJob * slot], clock_now());
        }
        // Four neighbouring lanes write the four sectors of one ticket, so that one store instruction of the
        // wavefront fills 16 consecutive tickets (1 KiB of whole lines).  A ticket's sector differs from the entry's
        // in two places only, so every lane fetches the entry's sector of its own kind from the lane that holds it
        // (three lane exchanges, where fetching the twelve words one by one into scalars took twelve).
        // What changes from one pass to the next is kept running, per lane, instead of being worked out from the
        // ticket's index each time (the leader spends three quarters of its time on a stream of 4 MiB requests in
        // this loop and the lines before it).
        const uint32_t sector = lane & 3u;
        const uint32_t first = lane >> 2;
        constexpr uint32_t kPerPass = kWaveLanes / 4;
        // (asked in this order: a request that is alone pays for nothing but the first comparison)
        const bool across = in_flight >= kManyInFlight && shares_across_tickets(in_flight, n, payload_of(fl, 11), payload_of(fl, 2));
        const uint32_t holder = fl + sector;
        u32x4 v{bcast(sect.x, holder), bcast(sect.y, holder), bcast(sect.z, holder), 0u};
        const uint64_t descs = (static_cast<uint64_t>(v.z) << 32) | v.y;  // in the lanes of sector 1: dst_hi, descs
        if (sector == 3) v.z = target;                                     // in the lanes of sector 3: val_hi, n, bytes
        uint64_t d = descs + static_cast<uint64_t>(first) * per_ticket * sizeof(tcpxuLoadMeta);
        const uint64_t d_step = static_cast<uint64_t>(kPerPass) * per_ticket * sizeof(tcpxuLoadMeta);
        uint32_t left = n - first * per_ticket;  // descriptors from this lane's ticket on (meaningless beyond nt)
        uint32_t at = static_cast<uint32_t>(tickets_out) + first;  // low word of the ticket number
        uint8_t* const ring = reinterpret_cast<uint8_t*>(st->tickets) + 16 * sector;
        // The ticket's own word: count | job slot | whether the submission has tickets before and after this one
        // (the last ticket is the one that takes all that is left).
        const uint32_t across_bits = across ? kMoreBefore | kMoreAfter : 0u;
        const uint32_t fixed_bits = (slot << 8) | (nt == 1 ? kOnlyTicket : 0u), after_bit = across_bits & kMoreAfter;
        uint32_t before_bit = first != 0 ? across_bits & kMoreBefore : 0u;
        for (uint32_t i = first; i < nt; i += kPerPass) {
          v.w = at + 1u;  // the stamp
          if (sector == 1) {
            v.y = static_cast<uint32_t>(d);
            v.z = static_cast<uint32_t>(d >> 32);
          }
          if (sector == 3) v.y = std::min(per_ticket, left) | fixed_bits | (left > per_ticket ? after_bit : 0u) | before_bit;
          before_bit = across_bits & kMoreBefore;  // every ticket but the submission's first
          store_vec_sys(ring + static_cast<size_t>(at & (kTicketRing - 1)) * sizeof(Record), v);
          d += d_step;
          left -= kPerPass * per_ticket;
          at += kPerPass;
        }
        tickets_out += nt;
      }
      ++consumed;
    }
    deep = deep_next;
    if (consumed != 0) {
      consumed = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(consumed)));
      s += consumed;
      entries += consumed;
      idle = 0;
      if (lane == 0) sys_store(&ctl->head, s);
      continue;
    }

    // Nothing could be consumed this round.
    const bool nothing_there = (ok_mask & 0xFull) != 0xFull;
    if (lane_value(aux, kAuxHostStop) != 0 && nothing_there) {
      // Stop requested and entry s not there.  The host wrote its last tail before the stop word, so a tail
      // read now bounds what is still to come.
      uint64_t tail_now = 0;
      if (lane == 0) tail_now = sys_load(&ctl->tail);
      if (s >= bcast64(tail_now, 0)) {
        reason = 1;
        break;
      }
      continue;
    }
    if (lane == 0) {
      const uint64_t c = sys_load(&st->jobs_completed);
      if (c != mirrored) {
        sys_store(&ctl->completed, c);
        mirrored = c;
      }
    }
    if (spin_limit != kNeverIdleOut && nothing_there && ++idle > spin_limit) {
      // Idle for long enough: leave, so that a device-wide synchronize by anybody returns.  The host relaunches
      // the kernel with its next submission.  A submission must not fall between "the leader stopped looking"
      // and "the host thinks the kernel is running": the leader announces that it is leaving, then looks once
      // more; the host publishes, then checks the announcement.  Each side stores before it loads (and PCIe
      // keeps a read behind the posted write issued before it), so at least one of them sees the other.
      if (lane == 0) sys_store(&ctl->exiting, static_cast<uint64_t>(1));
      drain_memory_ops();
      const uint32_t again = sys_load(&ctl->ring[s & ring_mask].w[lane & 15]);
      const bool there = ((lane & 3) == 3 && lane < 16) ? (again == static_cast<uint32_t>(s + 1)) : true;
      if (__all(there)) {
        if (lane == 0) sys_store(&ctl->exiting, static_cast<uint64_t>(0));
        idle = 0;
        continue;
      }
      reason = 2;
      break;
    }
    __builtin_amdgcn_s_sleep(1);
  }

  // Every ticket written must be visible before any stop word is.
  const uint32_t lane = threadIdx.x;
  drain_memory_ops();
  if (lane == 0) {
    sys_store(&st->sub_head, s);
    sys_store(&st->tickets_out, tickets_out);
    sys_store(&st->exit_reason, reason);
    const uint64_t totals[3] = {sys_load(&st->leader_polls) + polls, sys_load(&st->leader_entries) + entries,
                                sys_load(&st->leader_deep_polls) + deep_polls};
    sys_store(&st->leader_polls, totals[0]);
    sys_store(&st->leader_entries, totals[1]);
    sys_store(&st->leader_deep_polls, totals[2]);
    sys_store(&ctl->leader_polls, totals[0]);
    sys_store(&ctl->leader_entries, totals[1]);
    sys_store(&ctl->leader_deep_polls, totals[2]);
  }
  drain_memory_ops();
  sys_store(&st->stop[lane].value, 1u);
}

// ---- worker -------------------------------------------------------------------------------------------------------
// A worker workgroup is kCopyWaves copy wavefronts and one fetcher wavefront.  Towards the end of ticket i the
// fetcher claims a number, polls that ticket's slot, pulls the ticket's descriptors over PCIe and writes their
// records into the other LDS stage; between two tickets the copy wavefronts only meet the fetcher at one barrier.  The copy wavefront
// that finishes a ticket last counts it.
#ifndef TCPXU_ENGINE_COPY_WAVES
#define TCPXU_ENGINE_COPY_WAVES 8
#endif
constexpr uint32_t kCopyWaves = TCPXU_ENGINE_COPY_WAVES;
constexpr uint32_t kEngineThreads = (kCopyWaves + 1) * kWaveLanes;

// What a copy wavefront needs to know about one fragment, worked out by the fetcher: one descriptor per lane, all
// descriptors of a ticket at once, instead of by each copy wavefront from three descriptors per fragment.
constexpr uint32_t kRecSkip = 0, kRecTiny = 1, kRecRounds = 2;
struct alignas(16) RoundRec {
  uint32_t src_lo, src_hi;     // the fragment's first byte
  uint32_t dst_lo, dst_hi;
  uint32_t next_lo, next_hi;   // the next fragment's first source byte (read only if the last line is shared)
  uint32_t start_off, end_off; // FragmentPlan
  uint32_t len;
  uint32_t nvec;
  uint32_t bits;               // head | tail << 8 | share_next << 16 | kind << 24
  uint32_t pad;
};
static_assert(sizeof(RoundRec) == 48, "three 16-byte LDS reads");

struct Stage {
  uint32_t payload[kPayloadWords];
  uint32_t go;
  uint32_t pad[3];
  RoundRec rec[kMaxDescsPerTicket];
};

// The stages live in LDS, and every access says so: through a plain pointer the compiler loses track of that and
// reads the records with flat instructions (a 64-bit address in vector registers each, and slower).
#define TCPXU_LDS __attribute__((address_space(3)))
typedef TCPXU_LDS Stage LdsStage;
typedef TCPXU_LDS uint32_t lds_u32;
typedef TCPXU_LDS u32x4 lds_u32x4;

__device__ __forceinline__ uint32_t lane_shift(uint32_t v, uint32_t from_lane) {
  return static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute(static_cast<int>((from_lane & 63u) << 2), static_cast<int>(v)));
}

// Fetcher: look once at the slot of ticket number `ticket` (one 64-byte read, with this workgroup's stop word in
// the same round trip).  Returns 1 and stages the ticket if it is there.  Wave-uniform.
template <typename State>
__device__ uint32_t try_fetch_ticket(State* st, const uint32_t* stop_word, uint64_t ticket, LdsStage* stage,
                                     uint32_t lane, bool* stop_up, uint64_t* stamps) {
  const Record* rec = &st->tickets[ticket & (State::kTickets - 1)];
  const uint32_t expect = static_cast<uint32_t>(ticket + 1);
  uint32_t word = 0;
  if (lane < 16) word = sys_load(&rec->w[lane]);
  else if (lane == 16) word = sys_load(stop_word);
  *stop_up = bcast(word, 16) != 0;
  const bool stamp_ok = (lane < 16 && (lane & 3) == 3) ? (word == expect) : true;
  if (!__all(stamp_ok)) return 0;
  const uint64_t fetched_at = stamps ? clock_now() : 0;
  // Lane broadcasts need the whole wavefront: gather first, then let 12 lanes store.
  const uint32_t pl = lane < kPayloadWords ? lane : 0u;
  const uint32_t gathered = bcast(word, (pl / 3) * 4 + (pl % 3));
  if (lane < kPayloadWords) stage->payload[lane] = gathered;
  if (lane == 0) stage->go = 1;
  auto word64 = [&](int lo) {
    return (static_cast<uint64_t>(bcast(word, payload_slot(lo + 1))) << 32) | bcast(word, payload_slot(lo));
  };
  const uint64_t bounce = word64(0), dst = word64(2), descs_addr = word64(4);
  const uint32_t ticket_bits = bcast(word, payload_slot(10));
  const uint32_t n = ticket_bits & 0xFFu;
  // One 16-byte descriptor per lane straight from where the submission keeps them (system scope: never a cached
  // copy); lanes past the end repeat the last one and write no record.
  const uint32_t mine = lane < n ? lane : (n != 0 ? n - 1u : 0u);  // a ticket has at least one descriptor
  const u32x4 d = load_vec_sys(reinterpret_cast<const uint8_t*>(descs_addr) + 16 * mine);
  const uint32_t so = d[0], len = d[1];
  const uint64_t doff = (static_cast<uint64_t>(d[3]) << 32) | d[2];
  // The descriptor before the ticket's first and the one after its last, where the submission has them (lanes 0
  // and 1, in the same round trip): the neighbouring tickets' fetchers look at the same pairs from the other side.
  const bool more_before = (ticket_bits & kMoreBefore) != 0, more_after = (ticket_bits & kMoreAfter) != 0;
  uint32_t before_len = 0, before_dlo = 0, before_dhi = 0, after_so = 0, after_len = 0, after_dlo = 0, after_dhi = 0;
  if (more_before || more_after) {  // wave-uniform: a ticket without such neighbours pays nothing here
    u32x4 outer = {0u, 0u, 0u, 0u};
    if ((lane == 0 && more_before) || (lane == 1 && more_after)) {
      const uint64_t at = lane == 0 ? descs_addr - sizeof(tcpxuLoadMeta) : descs_addr + sizeof(tcpxuLoadMeta) * n;
      outer = load_vec_sys(reinterpret_cast<const uint8_t*>(at));
    }
    auto from_lane = [](uint32_t v, int src) { return static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(v), src)); };
    before_len = from_lane(outer[1], 0), before_dlo = from_lane(outer[2], 0), before_dhi = from_lane(outer[3], 0);
    after_so = from_lane(outer[0], 1), after_len = from_lane(outer[1], 1);
    after_dlo = from_lane(outer[2], 1), after_dhi = from_lane(outer[3], 1);
  }
  // The neighbours' descriptors decide which destination lines are shared with them.  A fragment's neighbours are
  // the nearest descriptors of the ticket that are not empty: an empty descriptor between two fragments (a
  // zero-length control message's, a fragment cut to nothing) leaves them back to back in the destination.
  const uint64_t live = __ballot(lane < n && len != 0);
  const uint64_t below = live & ((1ull << lane) - 1ull);
  const uint64_t above = lane < 63u ? live & ~((2ull << lane) - 1ull) : 0ull;
  const bool prev_inside = below != 0, next_inside = above != 0;
  // Across a ticket's ends only the very first and the very last descriptor have a neighbour, and only one that
  // is not empty: that is the pair the other ticket sees too.
  const bool prev_outside = !prev_inside && lane == 0 && before_len != 0;
  const bool next_outside = !next_inside && lane + 1 == n && after_len != 0;
  const bool has_prev = prev_inside || prev_outside, has_next = next_inside || next_outside;
  const uint32_t prev_lane = prev_inside ? 63u - static_cast<uint32_t>(__builtin_clzll(below)) : lane;
  const uint32_t next_lane = next_inside ? static_cast<uint32_t>(__builtin_ctzll(above)) : lane;
  uint32_t p_len = lane_shift(len, prev_lane), p_dlo = lane_shift(d[2], prev_lane), p_dhi = lane_shift(d[3], prev_lane);
  uint32_t q_len = lane_shift(len, next_lane), q_dlo = lane_shift(d[2], next_lane), q_dhi = lane_shift(d[3], next_lane);
  uint32_t q_so = lane_shift(so, next_lane);
  if (prev_outside) p_len = before_len, p_dlo = before_dlo, p_dhi = before_dhi;
  if (next_outside) q_len = after_len, q_dlo = after_dlo, q_dhi = after_dhi, q_so = after_so;
  const uint64_t fdst = dst + doff, fsrc = bounce + so;
  const uint64_t p_dst = dst + ((static_cast<uint64_t>(p_dhi) << 32) | p_dlo);
  const uint64_t q_dst = dst + ((static_cast<uint64_t>(q_dhi) << 32) | q_dlo);
  uint32_t kind = kRecRounds;
  if (len == 0) kind = kRecSkip;
  else if (fragment_is_tiny(reinterpret_cast<const uint8_t*>(fdst), len)) kind = kRecTiny;
  const bool share_prev = kind == kRecRounds && has_prev && shares_line(p_dst, p_len, fdst, len);
  const bool share_next = kind == kRecRounds && has_next && shares_line(fdst, len, q_dst, q_len);
  FragmentPlan plan = {0, 0, 0, 0, 1};
  if (kind == kRecRounds) plan = plan_fragment(fdst, len, share_prev, share_next);
  const uint64_t next_src = share_next ? bounce + q_so : fsrc;
  if (lane < n) {
    RoundRec r;
    r.src_lo = static_cast<uint32_t>(fsrc);
    r.src_hi = static_cast<uint32_t>(fsrc >> 32);
    r.dst_lo = static_cast<uint32_t>(fdst);
    r.dst_hi = static_cast<uint32_t>(fdst >> 32);
    r.next_lo = static_cast<uint32_t>(next_src);
    r.next_hi = static_cast<uint32_t>(next_src >> 32);
    r.start_off = plan.start_off;
    r.end_off = plan.end_off;
    r.len = len;
    r.nvec = plan.nvec;
    r.bits = plan.head | (plan.tail << 8) | (share_next ? 1u << 16 : 0u) | (kind << 24);
    r.pad = 0;
    lds_u32x4* out = reinterpret_cast<lds_u32x4*>(&stage->rec[lane]);
    out[0] = u32x4{r.src_lo, r.src_hi, r.dst_lo, r.dst_hi};
    out[1] = u32x4{r.next_lo, r.next_hi, r.start_off, r.end_off};
    out[2] = u32x4{r.len, r.nvec, r.bits, r.pad};
  }
  if (stamps) {
    const uint32_t job = (ticket_bits >> 8) & 0xFFFFu;
    const uint64_t staged_at = clock_now();
    if (lane == 0) {
      __hip_atomic_fetch_min(&stamps[kStampsPerJob * job + 1], fetched_at, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_fetch_min(&stamps[kStampsPerJob * job + 2], staged_at, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  return 1;
}

// Counts a finished ticket (all of its payload is in memory); the last ticket of a submission publishes the
// completion word.
template <typename State>
__device__ void retire_ticket(State* st, uint32_t* jobs_done, const LdsStage* stage, uint32_t lane, uint64_t* stamps) {
  if (lane == 0) {
    const uint32_t job = (stage->payload[10] >> 8) & 0xFFFFu;
    const uint32_t target = stage->payload[11];
    const uint64_t done_flag = (static_cast<uint64_t>(stage->payload[7]) << 32) | stage->payload[6];
    const uint64_t done_value = (static_cast<uint64_t>(stage->payload[9]) << 32) | stage->payload[8];
    if ((stage->payload[10] & kOnlyTicket) != 0) {
      // The submission's only ticket completes it: tell the caller first, count afterwards (nobody waits for the
      // counts' round trips; the leader reads them when it wants the job slot again).
      if (stamps) sys_store(&stamps[kStampsPerJob * job + 3], clock_now());
      sys_store(reinterpret_cast<uint64_t*>(done_flag), done_value);
      __hip_atomic_fetch_add(&jobs_done[job], 1u, __ATOMIC_RELAXED, SYS);
      __hip_atomic_fetch_add(&st->tickets_done, 1ull, __ATOMIC_RELAXED, SYS);
      __hip_atomic_fetch_add(&st->jobs_completed, 1ull, __ATOMIC_RELAXED, SYS);
      return;
    }
    const uint32_t count = __hip_atomic_fetch_add(&jobs_done[job], 1u, __ATOMIC_RELAXED, SYS) + 1u;
    __hip_atomic_fetch_add(&st->tickets_done, 1ull, __ATOMIC_RELAXED, SYS);
    if (count == target) {
      // Every other ticket's payload was in memory before it was counted, and so is this one's.
      if (stamps) sys_store(&stamps[kStampsPerJob * job + 3], clock_now());
      sys_store(reinterpret_cast<uint64_t*>(done_flag), done_value);
      __hip_atomic_fetch_add(&st->jobs_completed, 1ull, __ATOMIC_RELAXED, SYS);
    }
  }
}

// Copy wavefront `wave` of kCopyWaves: its run of consecutive fragments of the staged ticket (an eighth of the
// ticket, rounded up), one round (at most 4 KiB) in flight at a time.  A wavefront that writes one contiguous
// stretch of the destination after another measured about 1 % faster end to end than fragments dealt out in turn
// (wave, wave + kCopyWaves, ...).
__device__ __forceinline__ void copy_ticket(const LdsStage* stage, uint32_t wave, uint32_t lane, lds_u32* waves_on_last) {
  auto uniform = [](uint32_t v) { return static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(v)); };
  wave = uniform(wave);
  const uint32_t n = uniform(stage->payload[10]) & 0xFFu;
  const uint32_t per = (n + kCopyWaves - 1) / kCopyWaves;
  uint32_t j = wave * per < n ? wave * per : n;
  const uint32_t end = j + per < n ? j + per : n;
  // Told once, when the wavefront turns to the last fragment of its share (at once if it has none): the fetcher
  // uses it to start fetching the next ticket.
  auto on_last_fragment = [&] {
    if (lane == 0) __hip_atomic_fetch_add(waves_on_last, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  };
  if (j >= end) on_last_fragment();
  uint32_t nvec_left = 0;
  // The next round of the share into `out`, or false when there is none; `prev` is the round before it (read only
  // while a fragment longer than one round goes on).
  auto produce = [&](CopyRound& out, const CopyRound& prev) -> bool {
    if (nvec_left != 0) {
      out = prev;
      out.has_edge = false;  // the first round has copied the edge bytes and the shared line
      out.share_next = false;
      out.src_vec = prev.src_vec + (static_cast<size_t>(prev.nvec) << 4);
      out.dst_vec = prev.dst_vec + (static_cast<size_t>(prev.nvec) << 4);
      out.nvec = nvec_left < kVecPerRound ? nvec_left : kVecPerRound;
      nvec_left -= out.nvec;
      return true;
    }
    while (j < end) {
      const lds_u32x4* words = reinterpret_cast<const lds_u32x4*>(&stage->rec[j]);
      const u32x4 w0 = words[0], w1 = words[1], w2 = words[2];
      ++j;
      if (j >= end) on_last_fragment();
      const uint32_t bits = uniform(w2[2]);
      const uint32_t kind = bits >> 24;
      if (kind == kRecSkip) continue;
      const uint8_t* src = reinterpret_cast<const uint8_t*>((static_cast<uint64_t>(uniform(w0[1])) << 32) | uniform(w0[0]));
      uint8_t* dst = reinterpret_cast<uint8_t*>((static_cast<uint64_t>(uniform(w0[3])) << 32) | uniform(w0[2]));
      const uint32_t len = uniform(w2[0]);
      if (kind == kRecTiny) {
        copy_tiny_fragment(src, dst, len, lane);
        continue;
      }
      const uint8_t* src_next = reinterpret_cast<const uint8_t*>((static_cast<uint64_t>(uniform(w1[1])) << 32) | uniform(w1[0]));
      out = first_round_of(src, dst, src_next, len, ((bits >> 16) & 1u) != 0, uniform(w1[2]), uniform(w1[3]), bits & 0xFFu,
                           (bits >> 8) & 0xFFu, uniform(w2[1]), lane, &nvec_left);
      return true;
    }
    return false;
  };
  // In a ticket of short fragments (one of more than kFullTicket descriptors: the leader makes those for
  // submissions whose payload says so) the next round is worked out -- its record read from LDS, its scalars set
  // up -- while the loads of the round in flight are on their way, not after its stores: that work is a seventh of
  // a short round's time (fragments of 1.8 KiB on average: 62.5 % -> 63.6 % of the roofline).  In a ticket of whole
  // pages it stays where it was: they move up to 1 % faster with that pause between a round's stores and the next
  // round's loads.
  const bool ahead = n > kFullTicket;
  CopyRound r, next;
  CopyRegs x;
  bool more = produce(r, r);
  while (more) {
    round_load(r, x, lane);
    if (ahead) more = produce(next, r);
    round_store(r, x, lane);
    if (!ahead) more = produce(next, r);
    r = next;
  }
}

// `ticket_limit`: ticket numbers from this one on do not exist and end the workgroup that claims one (the engine
// passes none: its workgroups leave by the stop words); `look_limit`: looks at a ticket that is not there after
// which the workgroup gives up (0 = never, the engine's workers wait for the leader as long as it lives).
template <typename State>
__device__ void worker_loop(State* st, uint32_t* jobs_done, uint32_t flags, uint64_t ticket_limit,
                            uint32_t look_limit, uint64_t* stamps) {
  __shared__ Stage stages[2];
  __shared__ uint32_t s_waves_done;  // copy wavefronts that have finished (and drained) a ticket, running total
  __shared__ uint32_t s_waves_on_last;  // copy wavefronts that have turned to their last fragment of a ticket, ditto
  const uint32_t tid = threadIdx.x;
  const uint32_t lane = tid & (kWaveLanes - 1);
  const uint32_t wave = tid / kWaveLanes;
  if (tid == 0) {
    s_waves_done = 0;
    s_waves_on_last = 0;
  }
  __syncthreads();

  if (wave == kCopyWaves) {
    // ---- fetcher ----
    // Each pass stages this workgroup's next ticket (or the exit marker) into the free LDS stage, then meets the
    // copy wavefronts at the barrier.
    //
    // When to claim the next ticket number.  Numbers are served in order, so a number claimed by a workgroup
    // that is still busy keeps its ticket waiting even if other workgroups are idle; a number claimed only when
    // the workgroup is idle leaves the whole pick-up (claim, ticket record, descriptors over PCIe) exposed.  The
    // fetcher claims when every copy wavefront has turned to its last fragment of the current ticket: what is
    // left of the copy then takes about as long as the pick-up, so neither waits for the other.  (flags bit 1
    // clear: claim only when the copy has finished; bit 0 set: claim right away while tickets are queueing up,
    // i.e. the previous ticket was already there at the first look.)
    const uint32_t* stop_word = &st->stop[blockIdx.x % State::kStops].value;
    uint32_t staged = 0;
    bool eager = false;
    const bool allow_eager = (flags & 1u) != 0;
    const uint32_t* const claim_gate = (flags & 2u) != 0 ? &s_waves_on_last : &s_waves_done;
    const uint32_t backoff_cap = (flags >> 8) & 0xFFu;
    for (;;) {
      LdsStage* next = (LdsStage*)&stages[staged & 1];
      if (!eager) {
        // Wait for the copy of ticket staged-1 to finish (LDS only: no memory traffic while waiting).
        while (__hip_atomic_load(claim_gate, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) != staged * kCopyWaves)
          __builtin_amdgcn_s_sleep(1);
      }
      uint64_t t = 0;
      if (lane == 0) t = __hip_atomic_fetch_add(&st->ticket_head, 1ull, __ATOMIC_RELAXED, SYS);
      const uint64_t ticket = bcast64(t, 0);
      bool give_up = false, stop_before = false, first_look = true;
      uint32_t backoff = 1, looks = 0;
      for (;;) {
        bool stop_up = false;
        if (ticket < ticket_limit && try_fetch_ticket(st, stop_word, ticket, next, lane, &stop_up, stamps)) {
          eager = first_look && allow_eager;
          break;
        }
        if (ticket >= ticket_limit || (look_limit != 0 && ++looks >= look_limit)) {
          if constexpr (std::is_same<State, OneShotState>::value) {
            // A ticket that exists and never shows up: two calls overlapped on one GPU and overwrote each other's
            // tickets.  The slot cannot be completed; whoever polls its completion word is told so with the
            // complement of the value it waits for, rather than left waiting.
            if (ticket < ticket_limit && lane == 0)
              sys_store(reinterpret_cast<uint64_t*>(sys_load(&st->flag_addr)), ~sys_load(&st->flag_value));
          }
          give_up = true;
          if (lane == 0) next->go = 0;
          break;
        }
        if (stop_before) {
          // The stop word was already up at the previous look and the ticket is still not there: the leader
          // publishes every ticket before any stop word, so it never will be.
          give_up = true;
          if (lane == 0) next->go = 0;
          break;
        }
        stop_before = stop_up;
        first_look = false;
        if (!stop_before) {
          // Idle: look again soon at first, then back off a little, so that a thousand idle workgroups do not
          // load the memory system that busy ones are using.  (At most two sleeps between looks: with up to
          // eight a lone 64 KiB request took 0.2 us longer, four in flight 1.2 us, and no workload was faster.)
          for (uint32_t i = 0; i < backoff; ++i) __builtin_amdgcn_s_sleep(4);
          if (backoff < backoff_cap) backoff <<= 1;
        }
      }
      __syncthreads();  // hands `next` to the copy wavefronts, which are waiting here after their ticket
      if (give_up) break;
      ++staged;
    }
  } else {
    // ---- copy wavefronts ----
    for (uint32_t i = 0;; ++i) {
      __syncthreads();  // stage i&1 is ready
      LdsStage* stage = (LdsStage*)&stages[i & 1];
      if (stage->go == 0) break;
      copy_ticket(stage, wave, lane, (lds_u32*)&s_waves_on_last);
      drain_memory_ops();  // this wavefront's write-through stores are acknowledged
      uint32_t arrived = 0;
      if (lane == 0)
        arrived = __hip_atomic_fetch_add(&s_waves_done, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) + 1u;
      // The wavefront that finishes last counts the ticket: every wavefront's payload is in memory by then.
      if (bcast(arrived, 0) == (i + 1) * kCopyWaves) retire_ticket(st, jobs_done, stage, lane, stamps);
    }
  }
}

__global__ __launch_bounds__(kEngineThreads) __attribute__((amdgpu_waves_per_eu(6))) void unpack_engine_kernel(HostCtl* ctl, DevState* st, uint32_t* jobs_done,
                                                                   uint32_t* job_target, uint32_t ring_mask,
                                                                   uint32_t per_ticket, uint32_t spin_limit,
                                                                   uint32_t flags, uint64_t* stamps) {
  if (blockIdx.x == 0) {
    if (threadIdx.x < kWaveLanes) leader_loop(ctl, st, jobs_done, job_target, ring_mask, per_ticket, spin_limit, stamps);
  } else {
    worker_loop(st, jobs_done, flags, ~0ull, 0u, stamps);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    drain_memory_ops();
    const uint32_t before = __hip_atomic_fetch_add(&st->exited_wgs, 1u, __ATOMIC_RELAXED, SYS);
    if (before + 1 == gridDim.x) {
      // Last workgroup out: every ticket that was written has been counted.  Ticket numbers claimed beyond the
      // last written one are given back, so the next launch starts where this one ended.
      sys_store(&st->ticket_head, sys_load(&st->tickets_out));
      sys_store(&ctl->completed, sys_load(&st->jobs_completed));
      drain_memory_ops();
      sys_store(&ctl->exited, static_cast<uint64_t>(sys_load(&st->exit_reason)));
    }
  }
}

// ---- one slot, one ordinary launch, nothing allocated ---------------------------------------------------------------
// Scratch memory of tcpxuUnpackSlotNoAlloc: what the engine keeps in the DevState it allocates (ticket records, the
// ticket cursor, the done counters), for one slot, held by every GPU the library runs on until the process ends.
// In host code this name is only a handle for hipGetSymbolAddress; kernels get the address it returns.
static __device__ __align__(256) unsigned char scratch[sizeof(OneShotState)];

// Writes the slot's tickets (what the leader does for a submission) and clears the counters; with no descriptors
// it completes the slot itself.  One workgroup of kOneShotTickets threads, thread t writes ticket t.
__global__ __launch_bounds__(kOneShotTickets) void oneshot_prepare_kernel(OneShotState* st, uint64_t bounce,
                                                                         uint64_t dst, uint64_t descs,
                                                                         uint32_t n_descs, uint64_t done_flag,
                                                                         uint64_t done_value) {
  const uint32_t t = threadIdx.x;
  if (done_flag == 0) done_flag = reinterpret_cast<uint64_t>(&st->unused_flag);
  if (t == 0) {
    sys_store(&st->ticket_head, static_cast<uint64_t>(0));
    sys_store(&st->tickets_done, static_cast<uint64_t>(0));
    sys_store(&st->jobs_completed, static_cast<uint64_t>(0));
    sys_store(&st->jobs_done[0], 0u);
    sys_store(&st->stop[0].value, 0u);
    sys_store(&st->flag_addr, done_flag);
    sys_store(&st->flag_value, done_value);
    if (n_descs == 0) sys_store(reinterpret_cast<uint64_t*>(done_flag), done_value);
  }
  const uint32_t nt = (n_descs + kOneShotTicketSize - 1) / kOneShotTicketSize;
  if (t >= nt) return;
  const uint64_t d = descs + static_cast<uint64_t>(t) * kOneShotTicketSize * sizeof(tcpxuLoadMeta);
  const uint32_t count = std::min(kOneShotTicketSize, n_descs - t * kOneShotTicketSize);
  const uint32_t payload[kPayloadWords] = {
      static_cast<uint32_t>(bounce),    static_cast<uint32_t>(bounce >> 32),    static_cast<uint32_t>(dst),
      static_cast<uint32_t>(dst >> 32), static_cast<uint32_t>(d),               static_cast<uint32_t>(d >> 32),
      static_cast<uint32_t>(done_flag), static_cast<uint32_t>(done_flag >> 32), static_cast<uint32_t>(done_value),
      static_cast<uint32_t>(done_value >> 32), count | neighbour_bits(t, nt, true) /* job slot 0 */, nt};
  const uint32_t stamp = t + 1u;
  uint8_t* rec = reinterpret_cast<uint8_t*>(&st->tickets[t]);
#pragma unroll
  for (int sector = 0; sector < 4; ++sector)
    store_vec_sys(rec + 16 * sector, u32x4{payload[3 * sector], payload[3 * sector + 1], payload[3 * sector + 2], stamp});
}

// The engine's worker workgroups over tickets 0 .. n_tickets-1 and nothing else: a workgroup that claims a number
// beyond them leaves.  The tickets were written by the launch before this one on the same stream, so the first
// look finds each; the look limit only keeps a misuse (two calls overlapping on one GPU) from spinning for ever.
__global__ __launch_bounds__(kEngineThreads) void unpack_oneshot_kernel(OneShotState* st, uint32_t flags,
                                                                    uint32_t n_tickets) {
  worker_loop(st, st->jobs_done, flags, n_tickets, 1u << 16, nullptr);
}

}  // namespace
}  // namespace tcpxu

using namespace tcpxu;

struct tcpxuEngine {
  int device = 0;
  uint32_t ring_entries = 0;
  uint32_t workgroups = 0;
  uint32_t per_ticket = 0;
  uint32_t spin_limit = 0;
  uint32_t flags = 0;  // bits 0-1: when fetchers claim (see worker_loop); bits 8-15: idle poll backoff cap
  hipStream_t stream = nullptr;
  hipEvent_t ev_start = nullptr, ev_stop = nullptr;
  HostCtl* ctl = nullptr;      // host address of the mapped control block
  HostCtl* ctl_dev = nullptr;  // its device alias
  DevState* st = nullptr;
  uint32_t* jobs_done = nullptr;   // [ring_entries], device memory
  uint32_t* job_target = nullptr;  // [ring_entries], device memory, leader-private
  uint64_t tail = 0;  // host copy
  bool launched = false;  // between a launch and the Stop that reaps it (the kernel may have left by itself)
  bool failed = false;    // the kernel stopped answering (see tcpxuEngineSubmitSized); nothing more is accepted
  uint64_t launches = 0;
  uint64_t submissions = 0;
  uint64_t* stamps = nullptr;  // device memory, kStampsPerJob per ring entry, or null (tcpxuEngineEnableStamps)
  std::mutex mu;
};

// Engine calls arrive on threads that belong to somebody else (NCCL's proxy thread calls tcpxTest, which may have
// to relaunch the kernel): the calling thread's current device is put back when the call returns.
namespace {
class DeviceScope {
 public:
  explicit DeviceScope(int device) {
    if (hipGetDevice(&saved_) != hipSuccess) saved_ = -1;
    rc_ = use_device(device);
    if (saved_ == device) saved_ = -1;  // nothing to put back
  }
  ~DeviceScope() {
    if (saved_ >= 0) (void)hipSetDevice(saved_);
  }
  int rc() const { return rc_; }
  DeviceScope(const DeviceScope&) = delete;
  DeviceScope& operator=(const DeviceScope&) = delete;

 private:
  int saved_ = -1;
  int rc_ = TCPXU_SUCCESS;
};
}  // namespace

static size_t ctl_bytes(uint32_t ring_entries) { return offsetof(HostCtl, ring) + sizeof(Record) * ring_entries; }

extern "C" {

int tcpxuEngineCreate(int device, const tcpxuEngineConfig* config, tcpxuEngine** engine) {
  if (!engine) return TCPXU_INVALID_ARGUMENT;
  *engine = nullptr;
  tcpxuEngineConfig cfg{};
  if (config) cfg = *config;
  if (cfg.ring_entries == 0) cfg.ring_entries = 4096;
  if ((cfg.ring_entries & (cfg.ring_entries - 1)) != 0 || cfg.ring_entries > (1u << 16) || cfg.ring_entries < 16) {
    set_error("ring_entries %u must be a power of two in [16, 65536]", cfg.ring_entries);
    return TCPXU_INVALID_ARGUMENT;
  }
  if (cfg.descs_per_ticket == 0) {
    const char* v = getenv("TCPXU_DESCS_PER_TICKET");  // tuning aid: fixes the size; unset = by backlog
    if (v && *v) cfg.descs_per_ticket = static_cast<uint32_t>(atoi(v));
  }
  if (cfg.descs_per_ticket > kMaxDescsPerTicket) {
    set_error("descs_per_ticket %u must be in [0,%u]", cfg.descs_per_ticket, kMaxDescsPerTicket);
    return TCPXU_INVALID_ARGUMENT;
  }
  DeviceScope scope(device);
  TCPXU_TRY(scope.rc());
  const uint32_t cus = static_cast<uint32_t>(std::max(1, device_compute_units(device)));
  if (cfg.workgroups == 0) {
    // Two worker workgroups per compute unit: 18 of a compute unit's 32 wavefront slots, so that other kernels
    // (copies, the caller's own work) are scheduled beside the engine while it runs.  One is not enough (8 MiB
    // chunks, 64 slots in flight: 59 % of the HBM roofline against 71 %; fragments of 2 KiB: 41 % against 66 %).
    // Two is also all that is ever resident: the nine wavefronts of a workgroup go to the four SIMDs as 3+2+2+2,
    // a third workgroup would need a ninth slot on the first SIMD, and the hardware counters show a grid of
    // three per compute unit running exactly the wavefront-cycles of two.  (Workgroups of twelve wavefronts, two
    // per compute unit, do fit: 22 copy wavefronts instead of 16 move short fragments 1 % faster and whole pages
    // no faster, and leave other kernels 8 slots instead of 14.)  The occupancy query is not asked: it has answered
    // "one" in a process that had launched other kernels before.  A grid larger than what is resident would still
    // be correct -- no workgroup waits for another worker -- only pointless.
    uint32_t per_cu = 2;
    const char* v = getenv("TCPXU_ENGINE_WGS_PER_CU");  // tuning aid: 1 or 2
    if (v && *v) per_cu = std::min(std::max(static_cast<uint32_t>(atoi(v)), 1u), 2u);
    cfg.workgroups = cus * per_cu + 1;
  }
  if (cfg.workgroups < 2 || cfg.workgroups > (1u << 16)) {
    set_error("an engine needs the leader workgroup and 1 to 65535 workers");
    return TCPXU_INVALID_ARGUMENT;
  }

  tcpxuEngine* e = new (std::nothrow) tcpxuEngine;
  if (!e) return TCPXU_SYSTEM_ERROR;
  e->device = device;
  e->ring_entries = cfg.ring_entries;
  e->workgroups = cfg.workgroups;
  e->per_ticket = cfg.descs_per_ticket;
  e->spin_limit = cfg.spin_limit != 0 ? cfg.spin_limit : kDefaultIdlePolls;
  {
    const char* ve = getenv("TCPXU_ENGINE_EAGER");
    const char* vb = getenv("TCPXU_ENGINE_BACKOFF_CAP");
    const uint32_t eager = (ve && *ve) ? static_cast<uint32_t>(atoi(ve)) & 3u : 2u;
    const uint32_t cap = (vb && *vb) ? static_cast<uint32_t>(atoi(vb)) & 0xFFu : 2u;
    e->flags = eager | (cap << 8);
  }
  int rc = TCPXU_SUCCESS;
  do {
    void *h = nullptr, *d = nullptr;
    if ((rc = tcpxuMappedAlloc(device, ctl_bytes(cfg.ring_entries), &h, &d)) != TCPXU_SUCCESS) break;
    e->ctl = static_cast<HostCtl*>(h);
    e->ctl_dev = static_cast<HostCtl*>(d);
    const size_t st_bytes = sizeof(DevState) + 2 * sizeof(uint32_t) * cfg.ring_entries;
    // The state is cleared on the engine's own stream, and an event pair goes through it, so that whatever the
    // runtime sets up at a stream's first use (its hardware queue: half a millisecond) is paid here and not by the
    // first request.
    // Asking for the kernel's attributes makes the runtime load its code now (lazy otherwise: the first launch
    // would spend half a millisecond on it, after the launch's start event has been recorded).
    hipFuncAttributes attr;
    if (hipFuncGetAttributes(&attr, reinterpret_cast<const void*>(unpack_engine_kernel)) != hipSuccess ||
        hipMalloc(reinterpret_cast<void**>(&e->st), st_bytes) != hipSuccess ||
        hipStreamCreateWithFlags(&e->stream, hipStreamNonBlocking) != hipSuccess ||
        hipEventCreate(&e->ev_start) != hipSuccess || hipEventCreate(&e->ev_stop) != hipSuccess ||
        hipEventRecord(e->ev_start, e->stream) != hipSuccess ||
        hipMemsetAsync(e->st, 0, st_bytes, e->stream) != hipSuccess ||
        hipEventRecord(e->ev_stop, e->stream) != hipSuccess || hipStreamSynchronize(e->stream) != hipSuccess ||
        hipDeviceSynchronize() != hipSuccess) {
      set_error("engine allocation failed: %s", hipGetErrorString(hipGetLastError()));
      rc = TCPXU_DEVICE_ERROR;
      break;
    }
    e->jobs_done = reinterpret_cast<uint32_t*>(reinterpret_cast<uint8_t*>(e->st) + sizeof(DevState));
    e->job_target = e->jobs_done + cfg.ring_entries;  // (leader_storm works the second out from the first)
    // Test aid: where the engine's counts of submissions and tickets start.  Records are stamped with the low 32 bits
    // of their sequence number, and a busy engine passes 2^32 submissions within the hour; a test that starts just
    // below sees the crossing in milliseconds.  (Start more than a lap of the ticket ring below: a slot of either ring
    // that was never written reads as stamped for sequence number 2^32-1, which an engine that counts from zero
    // reaches only after every slot has been written many times.)
    const char* vc = getenv("TCPXU_ENGINE_COUNT_FROM");
    if (vc && *vc) {
      const uint64_t from = strtoull(vc, nullptr, 0);
      uint64_t* const counts[] = {&e->st->ticket_head, &e->st->tickets_done, &e->st->jobs_completed, &e->st->sub_head,
                                  &e->st->tickets_out};  // device addresses: only computed here, never read
      for (uint64_t* c : counts) {
        if (hipMemcpy(c, &from, sizeof from, hipMemcpyHostToDevice) != hipSuccess) {
          set_error("engine counters: %s", hipGetErrorString(hipGetLastError()));
          rc = TCPXU_DEVICE_ERROR;
          break;
        }
      }
      e->tail = from;
      e->ctl->tail = e->ctl->head = e->ctl->completed = from;
    }
  } while (false);
  if (rc != TCPXU_SUCCESS) {
    tcpxuEngineDestroy(e);
    return rc;
  }
  *engine = e;
  return TCPXU_SUCCESS;
}

// Launches the kernel.  Caller holds e->mu; any previous launch has ended (its exit word is set).
static int launch_locked(tcpxuEngine* e) {
  DeviceScope scope(e->device);
  TCPXU_TRY(scope.rc());
  // Per-launch state: exit bookkeeping and stop words start from zero; positions and counters are kept.
  TCPXU_HIP(hipMemsetAsync(reinterpret_cast<uint8_t*>(e->st) + offsetof(DevState, exited_wgs), 0,
                           offsetof(DevState, tickets) - offsetof(DevState, exited_wgs), e->stream));
  std::atomic_thread_fence(std::memory_order_seq_cst);
  e->ctl->stop = 0;
  e->ctl->exited = 0;
  e->ctl->exiting = 0;
  std::atomic_thread_fence(std::memory_order_seq_cst);
  TCPXU_HIP(hipEventRecord(e->ev_start, e->stream));
  hipLaunchKernelGGL(unpack_engine_kernel, dim3(e->workgroups), dim3(kEngineThreads), 0, e->stream, e->ctl_dev, e->st,
                     e->jobs_done, e->job_target, e->ring_entries - 1, e->per_ticket, e->spin_limit, e->flags, e->stamps);
  TCPXU_HIP(hipGetLastError());
  TCPXU_HIP(hipEventRecord(e->ev_stop, e->stream));
  e->launched = true;
  e->launches += 1;
  return TCPXU_SUCCESS;
}

static uint64_t host_load(const uint64_t* p) {
  return reinterpret_cast<const std::atomic<uint64_t>*>(p)->load(std::memory_order_acquire);
}

int tcpxuEngineStart(tcpxuEngine* e) {
  if (!e) return TCPXU_INVALID_ARGUMENT;
  std::lock_guard<std::mutex> lock(e->mu);
  if (e->launched && host_load(&e->ctl->exited) == 0) {
    set_error("engine already started");
    return TCPXU_INVALID_USAGE;
  }
  return launch_locked(e);
}

int tcpxuEngineStop(tcpxuEngine* e, double* elapsed_us) {
  if (!e) return TCPXU_INVALID_ARGUMENT;
  std::lock_guard<std::mutex> lock(e->mu);
  if (!e->launched) {
    set_error("engine is not started");
    return TCPXU_INVALID_USAGE;
  }
  DeviceScope scope(e->device);
  TCPXU_TRY(scope.rc());
  std::atomic_thread_fence(std::memory_order_seq_cst);
  reinterpret_cast<std::atomic<uint64_t>*>(&e->ctl->stop)->store(1, std::memory_order_seq_cst);
  // Wait for the kernel's own exit word first, with a deadline: a stuck kernel then surfaces as an error
  // from this call instead of a host thread parked inside the runtime.
  const char* v = getenv("TCPXU_ENGINE_STOP_TIMEOUT_MS");
  const long timeout_ms = (v && *v) ? atol(v) : 20000;
  const auto t0 = std::chrono::steady_clock::now();
  while (reinterpret_cast<std::atomic<uint64_t>*>(&e->ctl->exited)->load(std::memory_order_acquire) == 0) {
    if (std::chrono::steady_clock::now() - t0 > std::chrono::milliseconds(timeout_ms)) {
      set_error("engine kernel did not exit within %ld ms of the stop request", timeout_ms);
      return TCPXU_INTERNAL_ERROR;
    }
    std::this_thread::yield();
  }
  TCPXU_HIP(hipEventSynchronize(e->ev_stop));
  if (elapsed_us) {
    float ms = 0.f;
    TCPXU_HIP(hipEventElapsedTime(&ms, e->ev_start, e->ev_stop));
    *elapsed_us = static_cast<double>(ms) * 1000.0;
  }
  e->launched = false;
  return TCPXU_SUCCESS;
}

int tcpxuEngineDestroy(tcpxuEngine* e) {
  if (!e) return TCPXU_SUCCESS;
  if (e->launched) {
    int rc = tcpxuEngineStop(e, nullptr);
    if (rc != TCPXU_SUCCESS) return rc;  // never free memory under a running kernel
  }
  DeviceScope scope(e->device);
  if (e->ev_start) (void)hipEventDestroy(e->ev_start);
  if (e->ev_stop) (void)hipEventDestroy(e->ev_stop);
  if (e->stream) (void)hipStreamDestroy(e->stream);
  if (e->st) (void)hipFree(e->st);
  if (e->stamps) (void)hipFree(e->stamps);
  if (e->ctl) (void)hipHostFree(e->ctl);
  delete e;
  return TCPXU_SUCCESS;
}

int tcpxuEngineSubmit(tcpxuEngine* e, const void* bounce_base, void* dst_base, const void* descs_dev,
                      uint32_t n_descs, void* done_flag_dev, uint64_t done_value) {
  return tcpxuEngineSubmitSized(e, bounce_base, dst_base, descs_dev, n_descs, 0, done_flag_dev, done_value);
}

int tcpxuEngineSubmitSized(tcpxuEngine* e, const void* bounce_base, void* dst_base, const void* descs_dev,
                           uint32_t n_descs, uint64_t payload_bytes, void* done_flag_dev, uint64_t done_value) {
  const tcpxuSubmission one = {bounce_base, dst_base, descs_dev, done_flag_dev, done_value, n_descs,
                               payload_bytes > 0xFFFFFFFFull ? 0xFFFFFFFFu : static_cast<uint32_t>(payload_bytes)};
  uint32_t accepted = 0;
  return tcpxuEngineSubmitMany(e, &one, 1, &accepted);
}

// What a submission must look like; decided on the host, before anything is queued.
static int check_submission(const tcpxuEngine* e, const tcpxuSubmission& s) {
  if (!s.done_flag_dev || s.done_value == 0 || reinterpret_cast<uintptr_t>(s.done_flag_dev) % 8 != 0) {
    set_error("submit needs an 8-byte aligned completion word and a nonzero completion value");
    return TCPXU_INVALID_ARGUMENT;
  }
  if (s.n_descs > 0 && (!s.bounce_base || !s.dst_base || !s.descs_dev || reinterpret_cast<uintptr_t>(s.descs_dev) % 16 != 0)) {
    set_error("submit needs bounce, destination and a 16-byte aligned descriptor address");
    return TCPXU_INVALID_ARGUMENT;
  }
  // A submission whose tickets can never all fit the ticket ring would sit at the head of the submission ring for
  // ever, and the leader neither stops nor idles out with an entry waiting.
  if (s.n_descs > max_descs_for(e->per_ticket)) {
    set_error("%u descriptors in one submission exceed the limit of %u (tickets of %u at least, %u tickets in flight at most)",
              s.n_descs, max_descs_for(e->per_ticket), e->per_ticket ? e->per_ticket : kSmallestAdaptiveTicket, kTicketRing);
    return TCPXU_INVALID_ARGUMENT;
  }
  return TCPXU_SUCCESS;
}

int tcpxuEngineSubmitMany(tcpxuEngine* e, const tcpxuSubmission* subs, uint32_t n, uint32_t* accepted) {
  if (accepted) *accepted = 0;
  if (!e || (!subs && n != 0)) {
    set_error("submit needs an engine and submissions");
    return TCPXU_INVALID_ARGUMENT;
  }
  for (uint32_t i = 0; i < n; ++i) TCPXU_TRY(check_submission(e, subs[i]));  // all or nothing: none is queued if one is refused
  if (n == 0) return TCPXU_SUCCESS;
  std::lock_guard<std::mutex> lock(e->mu);
  if (e->failed) {
    set_error("the engine stopped answering earlier and accepts nothing more");
    return TCPXU_INTERNAL_ERROR;
  }
  const uint64_t head = reinterpret_cast<std::atomic<uint64_t>*>(&e->ctl->head)->load(std::memory_order_acquire);
  const uint64_t room = e->ring_entries - (e->tail - head);
  const uint32_t take = static_cast<uint32_t>(std::min<uint64_t>(room, n));
  if (take == 0) return kTcpxuInProgress;
  for (uint32_t k = 0; k < take; ++k) {
    const tcpxuSubmission& sub = subs[k];
    const uint64_t v[5] = {reinterpret_cast<uint64_t>(sub.bounce_base), reinterpret_cast<uint64_t>(sub.dst_base),
                           reinterpret_cast<uint64_t>(sub.descs_dev), reinterpret_cast<uint64_t>(sub.done_flag_dev),
                           sub.done_value};
    // The entry's sixteen words in the order they lie (three payload words and the stamp per sector), written as
    // four 16-byte stores: a record is valid for the leader once all four stamps are there, in whatever order the
    // sectors arrive, so nothing has to be ordered within it.
    const uint32_t stamp = static_cast<uint32_t>(e->tail + 1);
    alignas(64) uint32_t w[16];
    uint32_t p[kPayloadWords];
    for (int i = 0; i < 5; ++i) {
      p[2 * i] = static_cast<uint32_t>(v[i]);
      p[2 * i + 1] = static_cast<uint32_t>(v[i] >> 32);
    }
    p[10] = sub.n_descs;
    p[11] = sub.payload_bytes;
    for (int sct = 0; sct < 4; ++sct) {
      w[4 * sct] = p[3 * sct];
      w[4 * sct + 1] = p[3 * sct + 1];
      w[4 * sct + 2] = p[3 * sct + 2];
      w[4 * sct + 3] = stamp;
    }
    Record* ent = &e->ctl->ring[e->tail & (e->ring_entries - 1)];
    // What the descriptors say must be in memory before the entry that points to them can be seen.
    std::atomic_thread_fence(std::memory_order_release);
    typedef uint32_t host_u32x4 __attribute__((ext_vector_type(4)));
    for (int sct = 0; sct < 4; ++sct)
      *reinterpret_cast<volatile host_u32x4*>(&ent->w[4 * sct]) = *reinterpret_cast<const host_u32x4*>(&w[4 * sct]);
    e->tail += 1;
  }
  e->submissions += take;
  std::atomic_thread_fence(std::memory_order_release);
  reinterpret_cast<std::atomic<uint64_t>*>(&e->ctl->tail)->store(e->tail, std::memory_order_release);
  if (accepted) *accepted = take;
  // The kernel may have left for idleness, or be leaving right now (see leader_loop): publish first, then look.
  if (e->launched) {
    std::atomic_thread_fence(std::memory_order_seq_cst);
    if (host_load(&e->ctl->exiting) != 0 && host_load(&e->ctl->exited) == 0) {
      const auto t0 = std::chrono::steady_clock::now();
      while (host_load(&e->ctl->exiting) != 0 && host_load(&e->ctl->exited) == 0) {
        if (std::chrono::steady_clock::now() - t0 > std::chrono::seconds(5)) {
          // The entries are in the ring and stay there: this is not "not submitted, try again".  The engine is
          // marked failed so that the caller cannot queue the same work twice by retrying.
          e->failed = true;
          set_error("engine kernel announced that it is leaving and never did; the submission stays queued and the "
                    "engine accepts nothing more");
          return TCPXU_INTERNAL_ERROR;
        }
      }
    }
    if (host_load(&e->ctl->exited) == 2) TCPXU_TRY(launch_locked(e));  // it left by itself: bring it back
  }
  return take == n ? TCPXU_SUCCESS : kTcpxuInProgress;
}

int tcpxuEngineEnableStamps(tcpxuEngine* e, double* ticks_per_us) {
  if (!e) return TCPXU_INVALID_ARGUMENT;
  std::lock_guard<std::mutex> lock(e->mu);
  if (e->launched) {
    set_error("stamps are switched on while the engine is stopped");
    return TCPXU_INVALID_USAGE;
  }
  DeviceScope scope(e->device);
  TCPXU_TRY(scope.rc());
  const size_t bytes = sizeof(uint64_t) * kStampsPerJob * e->ring_entries;
  if (!e->stamps) TCPXU_HIP(hipMalloc(reinterpret_cast<void**>(&e->stamps), bytes));
  TCPXU_HIP(hipMemset(e->stamps, 0xFF, bytes));
  if (ticks_per_us) {
    int khz = 0;
    TCPXU_HIP(hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, e->device));
    *ticks_per_us = khz / 1000.0;
  }
  return TCPXU_SUCCESS;
}

int tcpxuEngineReadStamps(tcpxuEngine* e, uint64_t first_submission, uint32_t n, uint64_t* out) {
  if (!e || !out || n > e->ring_entries) {
    set_error("stamps: at most ring_entries submissions at a time");
    return TCPXU_INVALID_ARGUMENT;
  }
  std::lock_guard<std::mutex> lock(e->mu);
  if (!e->stamps || e->launched) {
    set_error("stamps are read while the engine is stopped, after tcpxuEngineEnableStamps");
    return TCPXU_INVALID_USAGE;
  }
  DeviceScope scope(e->device);
  TCPXU_TRY(scope.rc());
  std::vector<uint64_t> all(static_cast<size_t>(kStampsPerJob) * e->ring_entries);
  TCPXU_HIP(hipMemcpy(all.data(), e->stamps, all.size() * sizeof(uint64_t), hipMemcpyDeviceToHost));
  for (uint32_t i = 0; i < n; ++i) {
    const size_t slot = (first_submission + i) & (e->ring_entries - 1);
    for (uint32_t k = 0; k < kStampsPerJob; ++k) out[kStampsPerJob * i + k] = all[kStampsPerJob * slot + k];
  }
  TCPXU_HIP(hipMemset(e->stamps, 0xFF, all.size() * sizeof(uint64_t)));  // the minima start from ones again
  return TCPXU_SUCCESS;
}

int tcpxuEngineGetStats(tcpxuEngine* e, tcpxuEngineStats* stats) {
  if (!e || !stats) return TCPXU_INVALID_ARGUMENT;
  std::lock_guard<std::mutex> lock(e->mu);
  stats->launches = e->launches;
  stats->submissions = e->submissions;
  stats->leader_polls = host_load(&e->ctl->leader_polls);
  stats->leader_entries = host_load(&e->ctl->leader_entries);
  stats->leader_deep_polls = host_load(&e->ctl->leader_deep_polls);
  return TCPXU_SUCCESS;
}

int tcpxuEngineCompleted(tcpxuEngine* e, uint64_t* completed) {
  if (!e || !completed) return TCPXU_INVALID_ARGUMENT;
  *completed = reinterpret_cast<std::atomic<uint64_t>*>(&e->ctl->completed)->load(std::memory_order_acquire);
  return TCPXU_SUCCESS;
}

int tcpxuEngineGetConfig(tcpxuEngine* e, tcpxuEngineConfig* config) {
  if (!e || !config) return TCPXU_INVALID_ARGUMENT;
  config->ring_entries = e->ring_entries;
  config->workgroups = e->workgroups;
  config->descs_per_ticket = e->per_ticket;
  config->spin_limit = e->spin_limit;
  return TCPXU_SUCCESS;
}

int tcpxuEngineDevice(tcpxuEngine* e, int* device) {
  if (!e || !device) return TCPXU_INVALID_ARGUMENT;
  *device = e->device;
  return TCPXU_SUCCESS;
}

int tcpxuEngineTicketPlan(uint32_t workgroups, uint32_t descs_per_ticket, uint32_t in_flight, uint32_t n_descs,
                          uint64_t payload_bytes, uint32_t* per_ticket, uint32_t* n_tickets, uint32_t* max_descs) {
  if (workgroups < 2 || workgroups > (1u << 16) || descs_per_ticket > kMaxDescsPerTicket || in_flight == 0) {
    set_error("ticket plan: 2..65536 workgroups, tickets of 0..%u, at least one submission in flight", kMaxDescsPerTicket);
    return TCPXU_INVALID_ARGUMENT;
  }
  const uint32_t limit = max_descs_for(descs_per_ticket);
  if (max_descs) *max_descs = limit;
  if (n_descs > limit) {
    set_error("%u descriptors in one submission exceed the limit of %u", n_descs, limit);
    return TCPXU_INVALID_ARGUMENT;
  }
  const uint32_t bytes = payload_bytes > 0xFFFFFFFFull ? 0xFFFFFFFFu : static_cast<uint32_t>(payload_bytes);
  const uint32_t per = descs_per_ticket != 0 ? descs_per_ticket
                                             : ticket_size_for_submission(in_flight, n_descs, bytes, workgroups - 1);
  if (per_ticket) *per_ticket = per;
  if (n_tickets) *n_tickets = (n_descs + per - 1) / per;
  return TCPXU_SUCCESS;
}

// The address of `scratch` on each device, asked for once per device with that device current.
static OneShotState* g_scratch_ptr[kMaxDevices];
static std::mutex g_scratch_mu;

static int scratch_for(int device, OneShotState** out) {
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (!g_scratch_ptr[device]) {
    void* p = nullptr;
    TCPXU_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p || reinterpret_cast<uintptr_t>(p) % 256 != 0) {
      set_error("scratch symbol resolved to %p on device %d", p, device);
      return TCPXU_INTERNAL_ERROR;
    }
    g_scratch_ptr[device] = static_cast<OneShotState*>(p);
  }
  *out = g_scratch_ptr[device];
  return TCPXU_SUCCESS;
}

int tcpxuUnpackSlotNoAlloc(int device, const void* bounce_base, void* dst_base, const void* descs_dev,
                           uint32_t n_descs, void* done_flag_dev, uint64_t done_value, void* stream) {
  if (n_descs > TCPXU_SLOT_PAGES) {
    set_error("%u descriptors exceed the %d of one slot, the most this entry point's fixed scratch memory serves",
              n_descs, TCPXU_SLOT_PAGES);
    return TCPXU_INVALID_ARGUMENT;
  }
  if (reinterpret_cast<uintptr_t>(done_flag_dev) % 8 != 0 || (done_flag_dev && done_value == 0)) {
    set_error("the completion word must be 8-byte aligned and its value nonzero");
    return TCPXU_INVALID_ARGUMENT;
  }
  if (n_descs > 0 && (!bounce_base || !dst_base || !descs_dev || reinterpret_cast<uintptr_t>(descs_dev) % 16 != 0)) {
    set_error("unpack needs bounce, destination and a 16-byte aligned descriptor address");
    return TCPXU_INVALID_ARGUMENT;
  }
  DeviceScope scope(device);
  TCPXU_TRY(scope.rc());
  OneShotState* st = nullptr;
  TCPXU_TRY(scratch_for(device, &st));
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipLaunchKernelGGL(oneshot_prepare_kernel, dim3(1), dim3(kOneShotTickets), 0, s, st,
                     reinterpret_cast<uint64_t>(bounce_base), reinterpret_cast<uint64_t>(dst_base),
                     reinterpret_cast<uint64_t>(descs_dev), n_descs, reinterpret_cast<uint64_t>(done_flag_dev), done_value);
  TCPXU_HIP(hipGetLastError());
  if (n_descs == 0) return TCPXU_SUCCESS;
  const uint32_t n_tickets = (n_descs + kOneShotTicketSize - 1) / kOneShotTicketSize;
  const uint32_t cus = static_cast<uint32_t>(std::max(1, device_compute_units(device)));
  const uint32_t grid = std::min(n_tickets, 2u * cus);
  // flags: fetchers claim their next ticket when every copy wavefront is on its last fragment; idle backoff cap 2
  hipLaunchKernelGGL(unpack_oneshot_kernel, dim3(grid), dim3(kEngineThreads), 0, s, st, 2u | (2u << 8), n_tickets);
  TCPXU_HIP(hipGetLastError());
  return TCPXU_SUCCESS;
}

int tcpxuEngineRunning(tcpxuEngine* e, int* running) {
  if (!e || !running) return TCPXU_INVALID_ARGUMENT;
  std::lock_guard<std::mutex> lock(e->mu);
  *running = e->launched &&
             reinterpret_cast<std::atomic<uint64_t>*>(&e->ctl->exited)->load(std::memory_order_acquire) == 0;
  return TCPXU_SUCCESS;
}

}  // extern "C"
