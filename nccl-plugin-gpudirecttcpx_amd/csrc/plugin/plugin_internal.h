// Internal types of the plugin library: the receive-side state that sits between the ncclNet_v7 calls and the
// GPU engine.  Everything here is host code; the GPU is reached only through the tcpxDeviceOps table.
//
// Roles (reference file:line in parentheses)
//   StageRing      fixed-capacity ring whose items move through an ordered list of stages
//                  (tcpxItemQueue, src/work_queue.h:78-130)
//   Request        one posted receive (tcpxRequest, src/work_queue.h:63-76) in a 16-deep RequestRing
//                  (tcpxRequestQueue, src/work_queue.h:174-212; states src/work_queue_states.h:30-39)
//   Task           one chunk of a request travelling on one data flow (tcpxTask, src/work_queue.h:38-59) in a
//                  6-deep TaskRing shared with the socket thread (tcpxTaskQueue, src/work_queue.h:132-172)
//   DataPipe       per-task staging of descriptors and page tokens (tcpxDataPipe, src/sock/datapipe.h:25-46)
//   DevmemSocket   synthetic stand-in for one devmem-TCP data socket
//   UnpackQueue    the slot ring in mapped memory (tcpxNetDeviceQueue, src/devcomm/unpack_defs1.h:39-74)
//   Comm           per-connection state (tcpxComm, src/common.h:159-216)
#ifndef TCPX_AMD_PLUGIN_INTERNAL_H_
#define TCPX_AMD_PLUGIN_INTERNAL_H_

#include <sched.h>
#include <sys/socket.h>
#include <sys/uio.h>

#include <atomic>
#include <cstddef>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <memory>
#include <mutex>
#include <thread>
#include <vector>

#include "tcpx_plugin.h"
#include "flow_mapper.h"
#include "trace.h"

namespace tcpx {

constexpr int kMaxRequests = 16;  // MAX_REQUESTS, src/work_queue.h:20
constexpr int kMaxTasks = 6;      // MAX_TASKS, src/work_queue.h:21
constexpr int kMaxFlows = 8;      // MAX_SOCKETS, src/macro.h:36
constexpr int kQueueDepth = NCCL_NET_DEVICE_UNPACK_MAX_QUEUE_DEPTH;
constexpr int kSlotPages = NET_UNPACK_MAX_SLICE_PAGES;
constexpr int kMaxDevices = 64;

constexpr int kOpSend = 0;  // TCPX_SOCKET_SEND
constexpr int kOpRecv = 1;  // TCPX_SOCKET_RECV

// Linux devmem-TCP control-message types the reference parses (src/sock/tcpx.h:30-42).
constexpr int kScmDevmemHeader = 98;
constexpr int kScmDevmemOffset = 99;

// ---- logging ------------------------------------------------------------------------------------------------------
void log_line(ncclDebugLogLevel level, unsigned long flags, const char* file, int line, const char* fmt, ...)
    __attribute__((format(printf, 5, 6)));
#define WARN(...) ::tcpx::log_line(NCCL_LOG_WARN, NCCL_ALL, __FILE__, __LINE__, __VA_ARGS__)
#define INFO(FLAGS, ...) ::tcpx::log_line(NCCL_LOG_INFO, (FLAGS), __FILE__, __LINE__, __VA_ARGS__)

// Propagate errors up (TCPXCHECK, src/misc/checks1.h:53-61).
#define TCPXCHECK(call)                                                    \
  do {                                                                     \
    ncclResult_t res_ = (call);                                            \
    if (res_ != ncclSuccess) {                                             \
      INFO(NCCL_ALL, "TCPXCHECK %s:%d -> %d", __FILE__, __LINE__, res_);   \
      return res_;                                                         \
    }                                                                      \
  } while (0)

// ---- StageRing ----------------------------------------------------------------------------------------------------
// Items enter at stage 0 and leave each stage in FIFO order.  `entered` counts items ever enqueued, `left[k]` items
// that have left stage k; an item leaving the last stage frees its slot.  Counters only grow, so
//   entered >= left[0] >= left[1] >= ... >= left[Stages-1]   and   entered - left[Stages-1] <= Capacity.
// With Counter = std::atomic<uint32_t> one thread may own `entered` and some stages while another owns the rest
// (single producer, single consumer per counter).
// A counter is written by exactly one thread: its new value is published with a release store and read with an
// acquire load (plain moves on x86; the default sequentially consistent store would be a locked exchange on every
// state transition of every task).
inline uint32_t counter_load(const uint32_t& c) { return c; }
inline void counter_store(uint32_t& c, uint32_t v) { c = v; }
inline uint32_t counter_load(const std::atomic<uint32_t>& c) { return c.load(std::memory_order_acquire); }
inline void counter_store(std::atomic<uint32_t>& c, uint32_t v) { c.store(v, std::memory_order_release); }

template <typename Item, int Capacity, int Stages, typename Counter>
struct StageRing {
  // Each counter has one writer and a cache line of its own: the stages of a task ring are advanced by two threads
  // (the socket thread and the proxy thread), and a counter that shared its line with the other thread's would be
  // taken away from its writer at every step of the other.
  struct alignas(64) Line {
    Counter v;
  };
  alignas(64) Counter entered;
  Line left_[Stages];  // left[k] of the description above
  alignas(64) Item items[Capacity];

  StageRing() {
    counter_store(entered, 0);
    for (int k = 0; k < Stages; ++k) counter_store(left_[k].v, 0);
  }
  uint32_t in_flight() const { return counter_load(entered) - counter_load(left_[Stages - 1].v); }
  bool empty() const { return in_flight() == 0; }
  uint32_t num_free() const { return Capacity - in_flight(); }
  bool has_free() const { return num_free() > 0; }
  Item* next_free() { return &items[counter_load(entered) % Capacity]; }
  void enqueue() { counter_store(entered, counter_load(entered) + 1); }

  uint32_t stage_begin(int k) const { return counter_load(left_[k].v); }
  uint32_t stage_end(int k) const { return k == 0 ? counter_load(entered) : counter_load(left_[k - 1].v); }
  bool has(int k) const { return stage_end(k) != stage_begin(k); }
  Item* first(int k) { return &items[stage_begin(k) % Capacity]; }
  void advance(int k) { counter_store(left_[k].v, counter_load(left_[k].v) + 1); }
};

// ---- unpack queue -------------------------------------------------------------------------------------------------
struct PageToken {  // struct devmemtoken / pgtok_t, src/devcomm/unpack_defs1.h:39-44
  uint32_t token_start;
  uint32_t token_count;
};

// Mapped host memory of one comm.  The prefix is NCCL's netUnpackMeta, bit for bit; the completion words that the
// GPU engine writes follow it.
struct QueueMeta {
  struct netUnpackMeta nccl;
  struct alignas(64) DoneWord {
    uint64_t value;
  } done[kQueueDepth];
};

struct QueueRecord {  // struct tcpxRecord, src/devcomm/unpack_defs1.h:46-51
  size_t flow_cnts[kQueueDepth];
  size_t pgtok_cnts[kQueueDepth][kMaxFlows];
  int flows[kQueueDepth][kMaxFlows];
  PageToken pgtoks[kQueueDepth][kMaxFlows][kSlotPages];
};

struct UnpackQueue {  // struct tcpxNetDeviceQueue, src/devcomm/unpack_defs1.h:53-59
  QueueMeta* meta = nullptr;      // host address
  QueueMeta* meta_dev = nullptr;  // device alias
  struct unpackNetDeviceHandle* dev_handle = nullptr;  // device memory
  union loadMeta* stage = nullptr;      // see QueueBlock
  union loadMeta* stage_dev = nullptr;
  uint64_t head = 0, tail = 0;
  int dev = 0;
  QueueRecord record;
};

struct UnpackSlot {  // struct unpackSlot, src/devcomm/unpack_defs1.h:61-74
  bool active = false;
  uint64_t idx = 0;
  union loadMeta* mem = nullptr;
  uint64_t* cnt = nullptr;  // nullptr also marks "no slot allocated yet" (src/net_tcpx.cc:890)
  uint64_t cnt_cache = 0;
  size_t* flow_cnt = nullptr;
  size_t* pgtok_cnts = nullptr;  // [kMaxFlows]
  int* flows = nullptr;          // [kMaxFlows]
  PageToken* pgtoks = nullptr;   // [kMaxFlows][kSlotPages]
};

ncclResult_t unpack_queue_new(int dev, bool passive, UnpackQueue** queue);
void unpack_queue_free(UnpackQueue* queue);
// src/devcomm/nccl/unpack1.h:30-65
void unpack_queue_next_free(UnpackQueue* queue, UnpackSlot* slot);

// ---- synthetic devmem socket --------------------------------------------------------------------------------------
struct DevmemVec {  // struct devmemvec, src/sock/tcpx.h:130-134
  uint32_t frag_offset;
  uint32_t frag_size;
  uint32_t frag_token;
};

struct DataPipe {  // struct tcpxDataPipe, src/sock/datapipe.h:25-46
  std::vector<char> ctrl_data;           // control-message buffer handed to recvmsg
  std::vector<union loadMeta> scatter_list;  // [kSlotPages]
  uint64_t cnt_cache = 0;
  int bytes_cnt = 0;
  size_t* pgtok_cnt = nullptr;
  PageToken* pgtoks = nullptr;
  DataPipe();
};

struct DeviceState;

// One data flow's receive queue: what the kernel has for this socket.  recvmsg() hands out at most `max_bytes`
// and at most the control buffer's worth of fragments, one SCM_DEVMEM_OFFSET control message each, splitting a
// fragment when the byte budget ends inside it (the kernel does the same at the end of a recvmsg).
struct DevmemSocket {
  // Two sides.  Whoever delivers fragments appends to `arrived` under the lock; the one thread that receives on
  // this socket works on `rx`, which nobody else touches, and takes the lock only when `rx` has run empty, to swap
  // the two -- once per burst of deliveries instead of once per recvmsg.
  std::mutex mu;
  std::vector<tcpxSynthFrag> arrived;
  std::vector<tcpxSynthFrag> rx;
  size_t head = 0;                     // read position in rx
  size_t payload_frags = 0;            // fragments in rx[head..] with frag_size != 0
  std::atomic<uint32_t> max_frags_per_recvmsg{0};  // 0 = no extra limit
  DeviceState* device = nullptr;       // page accounting
  void push(const tcpxSynthFrag* frags, size_t n);  // takes the lock
  ssize_t recvmsg(struct msghdr* msg, size_t max_bytes);
  // setsockopt(SO_DEVMEM_DONTNEED): gives page references back (src/sock/tcpx.h:299-307).
  int dontneed(const PageToken* tokens, size_t n);
};

// Walks the control messages of one recvmsg and appends one descriptor per devmem fragment to the pipe, coalescing
// consecutive page tokens (process_recv_cmsg, src/sock/tcpx.h:136-228).  Returns the bytes described, or -1 with
// *result set when the reference would have stopped the process.
ssize_t process_recv_cmsg(struct msghdr* msg, DataPipe* pipe, int offset, uint64_t dst_base_offset,
                          ncclResult_t* result);
// recvmsg + process_recv_cmsg for one task (gpudirectTCPXRecv, src/sock/tcpx.h:230-297).
ssize_t devmem_recv(DevmemSocket* sock, int size, int offset, DataPipe* pipe, uint64_t dst_base_offset,
                    ncclResult_t* result);

// ---- requests and tasks -------------------------------------------------------------------------------------------
struct Comm;
struct Request;

// A task goes from the proxy thread (which fills it in) to the thread that serves its socket and back (descriptor
// count, result), and with a socket thread each direction is a cache line travelling between two CPUs: everything
// that travels is in the task's first line, and neither thread touches the other's bookkeeping (the pipe, the watch)
// on the way.
struct alignas(64) Task {  // struct tcpxTask, src/work_queue.h:38-59 (receive-side fields)
  int size = 0;
  int offset = 0;
  int request_offset = 0;
  uint16_t op = 0;
  uint16_t flow = 0;
  void* data = nullptr;
  Request* r = nullptr;
  ncclResult_t result = ncclSuccess;
  uint32_t cnt = 0;                // descriptors the task produced (the pipe's cnt_cache when its last byte arrived)
  DataPipe* pipe = nullptr;        // the slot's own, for the life of the ring
  PageToken* pgtoks = nullptr;     // passive side: where the task's page tokens go (the request's slot, per flow)
  size_t* pgtok_cnt = nullptr;
  SlownessWatch watch;  // second line; recvmsg finding nothing, over and over (tcpxTask::timeout)
};
static_assert(offsetof(Task, watch) == 64, "what travels between the threads is one cache line");

enum TaskStage { kTaskActive = 0, kTaskCompleting = 1, kTaskInactive = 2, kTaskStages = 3 };
struct TaskRing : StageRing<Task, kMaxTasks, kTaskStages, std::atomic<uint32_t>> {
  // Where each slot's pipe keeps its descriptors, never written after construction: a line both threads can keep.
  alignas(64) const union loadMeta* scatter[kMaxTasks];
  TaskRing();
  ~TaskRing();
};

struct Request {  // struct tcpxRequest, src/work_queue.h:63-76
  Comm* comm = nullptr;
  void* data = nullptr;
  int op = 0;
  int mem_type = 0;
  int next_flow = -1;  // next_sock_id: >= 0 once a control message is pending for this request
  int next_size = 0;
  int offset = 0;
  int size = 0;          // the message's size once its first control message has been read; until then, posted_size
  int posted_size = 0;   // what irecv was given: the most the message may be
  int size_pending = 0;
  UnpackSlot slot;
  // Engine hand-off: the slot has been submitted, and the value its completion word will take.
  bool published = false;
  uint64_t done_value = 0;
  uint64_t published_ns = 0;
  SlownessWatch unpack_watch;  // the GPU holds the slot and the completion word does not come
};

enum RequestStage { kReqPosted = 0, kReqActive = 1, kReqTransmitting = 2, kReqInactive = 3, kReqStages = 4 };
using RequestRing = StageRing<Request, kMaxRequests, kReqStages, uint32_t>;

struct CtrlMessage {  // struct tcpxCtrl, src/common.h:127-133 (16 bytes on the wire)
  uint16_t type;
  uint16_t index;
  uint32_t size;
  uint32_t offset;
  uint32_t total;
} __attribute__((__packed__));
static_assert(sizeof(CtrlMessage) == 16, "control message is 16 bytes");

struct MemHandle {  // struct tcpxMemHandle, src/common.h:90-98
  void* ptr;
  size_t size;  // bytes registered (the reference does not keep it)
  int mem_type;
};

struct FlowData {  // struct tcpxFdData, src/common.h:144-157 (receive-side fields)
  DevmemSocket sock;
  TaskRing tasks;
  uint64_t bytes = 0;
  // struct tcpxSocketStats (receive side); the socket thread counts, the proxy thread reads.
  std::atomic<uint64_t> rx_ctrl_done_cnt{0}, rx_cnt{0}, rx_slow_cnt{0};
  // Each has one writer (the proxy thread, or the thread that runs this flow's socket), so a count is a load and a
  // store, not a locked read-modify-write.
  static void bump(std::atomic<uint64_t>& c) { c.store(c.load(std::memory_order_relaxed) + 1, std::memory_order_relaxed); }
};

struct Comm {  // struct tcpxComm, src/common.h:159-216
  bool passive = false;
  int dev = 0;
  int num_flows = 0;
  int end_flow_idx = 0;
  FlowData flows[kMaxFlows];
  std::unique_ptr<FlowScheduler> sched;  // tcpxComm::flow_mapper: the flows whose task ring has room
  std::mutex ctrl_mu;
  std::deque<CtrlMessage> ctrl_rx;  // the control socket's receive queue: what has arrived (under ctrl_mu)
  std::deque<CtrlMessage> ctrl_local;  // ... and what the proxy thread has taken over from it, to read without the lock
  RequestRing rq;
  UnpackQueue* queue = nullptr;
  DeviceState* device = nullptr;
  uint64_t done_seq = 0;
  uint32_t slots_at_gpu = 0, max_slots_at_gpu = 0;  // slots submitted to the engine and not yet reported done
  SlownessWatch ctrl_watch;  // tcpxComm::ctrl_timeout
  uint64_t rx_ctrl_slow_cnt = 0, unpack_cnt = 0, unpack_slow_cnt = 0, unpack_ns = 0;
  std::unique_ptr<TraceBuffer> trace;  // tcpxComm::statsbuf; allocated when a stats level is on
  // Optional socket thread (persistentSocketThread, src/net_tcpx.cc:252-384).
  std::thread helper;
  std::atomic<bool> helper_stop{false};
  std::atomic<uint64_t> helper_cpus{0};  // CPUs the socket thread may run on, as it found them when it started
  bool use_helper = false;
};

// What tcpxListen writes into the caller's 128-byte handle and tcpxConnect_v5 reads back (the reference puts the
// listening socket's address there, src/connect.cc; with no sockets, the listener's identity does the same job).
struct ConnectHandle {
  uint64_t magic;  // kConnectMagic
  uint64_t id;     // the listener
  int32_t dev;
};
constexpr uint64_t kConnectMagic = 0x7463707861636365ull;  // "tcpxacce"
static_assert(sizeof(ConnectHandle) <= NCCL_NET_HANDLE_MAXSIZE, "the connect handle must fit NCCL's handle");

struct ListenComm {  // struct tcpxListenComm, src/common.h:112-124
  int dev;
  uint64_t id;
  // Connections made to this listener and not yet accepted (the listening socket's backlog).  connect() runs on
  // whichever thread the peer uses, accept() on the owner's.
  std::atomic<uint32_t> backlog;
};

// ---- per-GPU and global state -------------------------------------------------------------------------------------
struct QueueBlock {  // mapped metadata + device handle, recycled between comms (freed only when the engine is stopped)
  QueueMeta* meta;
  QueueMeta* meta_dev;
  struct unpackNetDeviceHandle* dev_handle;
  // Device memory the host can write, kQueueDepth x kStagedDescs descriptors, or null: where the descriptors of a
  // small request are copied to as well, so that the GPU need not fetch them over PCIe.
  union loadMeta* stage;
  union loadMeta* stage_dev;
};
constexpr uint32_t kStagedDescs = 16;

struct DeviceState {
  int dev = 0;
  std::mutex mu;
  void* arena = nullptr;
  size_t arena_bytes = 0;
  std::unique_ptr<std::atomic<int32_t>[]> page_refs;  // references held by the plugin, per arena page
  size_t n_pages = 0;
  // Counted up by whoever receives (every recvmsg) and down by whoever consumes: a cache line of its own, or every
  // count would take the line with the fields around it away from the thread that reads those at every poll.
  alignas(64) std::atomic<uint64_t> pages_outstanding{0};
  alignas(64) tcpxuEngine* engine = nullptr;
  bool engine_started = false;
  int comms = 0;
  std::vector<QueueBlock> free_blocks;
};

// Who copies.  kDeviceHost: this plugin's engine unpacks every request and test() reports done after the copy; the
// plugin advertises an ordinary host-driven network (NCCL_NET_DEVICE_HOST), so no consumer kernel touches the
// queue.  kDeviceUnpack: the reference's division of labour -- the plugin only publishes descriptor counts
// (src/net_tcpx.cc:1354-1357), advertises NCCL_NET_DEVICE_UNPACK with the device handle, and the caller's kernel
// copies; the engine is never started.
constexpr int kDeviceHost = 0, kDeviceUnpack = 1;

struct Global {
  std::mutex mu;
  bool initialized = false;
  int device_type = kDeviceHost;  // NCCL_GPUDIRECTTCPX_AMD_DEVICE_TYPE=host|unpack
  std::mutex listen_mu;
  std::vector<ListenComm*> listeners;  // open listeners, for connect() to find by id
  ncclDebugLogger_t logger = nullptr;
  const tcpxDeviceOps* ops = nullptr;
  bool ops_injected = false;
  int n_devices = 0;
  DeviceState devices[kMaxDevices];
  // Flags (environment, range-checked in tcpxInit like TCPX_GET_INT_FLAG, src/net_tcpx.cc:440-452).
  int flows_per_comm = 4;
  int use_helper_thread = 0;
  int sched_alg = kSchedRoundRobin;  // NCCL_GPUDIRECTTCPX_SCHED_ALG
  bool fail_stop = true;
  // Observability (src/flags.cc:44-70, src/net_tcpx.cc:105-116).
  ClockFn clock = monotonic_ns;
  bool clock_injected = false;
  int64_t timeout_threshold_ns = 10000000000LL;  // 10 s
  int64_t timeout_frequency_ns = 30000000000LL;  // 30 s
  int slow_switch[kSlowKinds] = {0, 0, 0, 0};
  int slow_report[kSlowKinds] = {0, 0, 0, 0};
  int task_stats = 0;
  int request_stats = 0;
  int sampling_factor = 1;
  // NCCL_GPUDIRECTTCPX_RX_BINDINGS (struct tcpxBindings, src/common.h): CPUs for the socket threads of a device's comms.
  cpu_set_t rx_cpus[kMaxDevices];
  bool rx_bound[kMaxDevices] = {};
  char dev_names[kMaxDevices][32];
  char pci_paths[kMaxDevices][64];
};
extern Global g;

FlowScheduler* new_flow_scheduler(int alg);  // kSchedKaty, or round robin for anything else
int sched_alg_from_name(const char* name, bool* valid);  // "RR" / "KATY" (exact); anything else is round robin

// The synthetic peer and kernel, for drivers inside the library: many control messages under one lock, and
// fragments that the caller has already checked against the devmem contract.
void ctrl_send_batch(Comm* comm, const CtrlMessage* messages, size_t n);
ncclResult_t deliver_fragments(Comm* comm, uint32_t flow, const tcpxSynthFrag* frags, uint32_t n_frags);

const tcpxDeviceOps* default_device_ops();  // binds libtcpxu_hip.so, or nullptr (reason logged)
ncclResult_t device_result(int rc, const char* what);
// Called where the reference stops the process; honours tcpxSetFailStopForTesting.
ncclResult_t fail_stop(const char* what);

}  // namespace tcpx

#endif  // TCPX_AMD_PLUGIN_INTERNAL_H_
