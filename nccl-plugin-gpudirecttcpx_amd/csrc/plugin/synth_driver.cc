// tcpxSynthRunRequests: plays NCCL's receive proxy, the peer and the NIC for a list of requests, natively.
//
// The same sequence the reference's callers produce for the receive path -- irecv (src/net_tcpx.cc:921-944), one
// control message per chunk from the peer (struct tcpxCtrl, src/common.h:127-133), the chunk's fragments from
// the kernel (src/sock/tcpx.h:136-228), test() polled until done (src/net_tcpx.cc:1311-1374), iflush
// (src/net_tcpx.cc:946-954), irecvConsumed (src/net_tcpx.cc:1477-1543) -- with up to `window` requests posted at a time, as NCCL keeps several steps in
// flight.  Used by tests and by the benchmark to drive the plugin without an interpreter in the loop.
#include <time.h>

#include <deque>
#include <vector>

#include "plugin_internal.h"

namespace tcpx {
namespace {

struct Chunk {
  uint32_t flow, first, count, bytes;
};

// Runs of consecutive fragments on the same flow.  An empty fragment cannot travel alone (recvmsg reports it
// together with payload), so it joins the run of the payload fragment before it, or after it at the very start.
void chunks_of(const tcpxSynthFrag* frags, uint32_t n, uint32_t n_flows, std::vector<Chunk>* out) {
  out->clear();
  std::vector<uint32_t> flow(n);
  int64_t last_payload = -1;
  uint32_t first_payload_flow = 0;
  bool any = false;
  for (uint32_t i = 0; i < n && !any; ++i) {
    if (frags[i].frag_size > 0) {
      first_payload_flow = frags[i].flow % n_flows;
      any = true;
    }
  }
  if (!any) return;
  for (uint32_t i = 0; i < n; ++i) {
    if (frags[i].frag_size > 0) last_payload = i;
    flow[i] = last_payload >= 0 ? frags[last_payload].flow % n_flows : first_payload_flow;
  }
  for (uint32_t i = 0; i < n;) {
    uint32_t j = i + 1, bytes = frags[i].frag_size;
    while (j < n && flow[j] == flow[i]) bytes += frags[j++].frag_size;
    out->push_back(Chunk{flow[i], i, j - i, bytes});
    i = j;
  }
}

double now_s() {
  struct timespec ts;
  clock_gettime(CLOCK_MONOTONIC, &ts);
  return static_cast<double>(ts.tv_sec) + 1e-9 * static_cast<double>(ts.tv_nsec);
}

}  // namespace
}  // namespace tcpx

using namespace tcpx;

extern "C" ncclResult_t tcpxSynthRunRequests(void* recvComm, const tcpxSynthFrag* frags, const tcpxSynthRequest* requests,
                                             uint32_t n_requests, void* dst_base, uint64_t dst_bytes, uint32_t window,
                                             uint32_t timeout_ms, double* seconds, double* latency_s) {
  Comm* comm = static_cast<Comm*>(recvComm);
  if (!comm || !comm->passive || !frags || !requests || !dst_base || window == 0 || window > static_cast<uint32_t>(kMaxRequests))
    return ncclInvalidArgument;
  if (dst_bytes > static_cast<uint64_t>(INT32_MAX)) dst_bytes = static_cast<uint64_t>(INT32_MAX);
  void* mhandle = nullptr;
  TCPXCHECK(tcpxRegMr(comm, dst_base, static_cast<int>(dst_bytes), NCCL_PTR_CUDA, &mhandle));
  struct Posted {
    void* request;
    uint32_t index;
    double fed;
  };
  std::deque<Posted> posted;
  std::vector<Chunk> chunks;
  std::vector<CtrlMessage> ctrl;
  std::vector<tcpxSynthFrag> by_flow[kMaxFlows];
  uint32_t next = 0;
  ncclResult_t rc = ncclSuccess;
  const double t0 = now_s();
  double deadline = t0 + 1e-3 * timeout_ms;
  const uint32_t n_flows = static_cast<uint32_t>(comm->num_flows);
  while (rc == ncclSuccess && (next < n_requests || !posted.empty())) {
    while (rc == ncclSuccess && next < n_requests && posted.size() < window) {
      const tcpxSynthRequest& r = requests[next];
      void* data = static_cast<char*>(dst_base) + r.dst_off;
      int size = static_cast<int>(r.bytes), tag = 0;
      void* request = nullptr;
      if ((rc = tcpxIrecv_v5(comm, 1, &data, &size, &tag, &mhandle, &request)) != ncclSuccess) break;
      const tcpxSynthFrag* f = frags + r.first_desc;
      if (r.bytes == 0) {
        rc = tcpxSynthCtrlSend(comm, TCPX_CTRL_INLINE, 0, 0, 0, 0);
      } else {
        // The peer's control messages, one per chunk, in chunk order; then what the kernel has for each flow: the
        // flow's fragments in arrival order (a socket keeps order only within itself, so handing each flow its
        // fragments in one piece is what many small deliveries come to).
        chunks_of(f, r.n_descs, n_flows, &chunks);
        ctrl.clear();
        for (uint32_t k = 0; k < n_flows; ++k) by_flow[k].clear();
        uint32_t offset = 0;
        for (const Chunk& c : chunks) {
          ctrl.push_back(CtrlMessage{TCPX_CTRL_NORMAL, static_cast<uint16_t>(c.flow), c.bytes, offset, r.bytes});
          offset += c.bytes;
          by_flow[c.flow].insert(by_flow[c.flow].end(), f + c.first, f + c.first + c.count);
        }
        ctrl_send_batch(comm, ctrl.data(), ctrl.size());
        for (uint32_t k = 0; rc == ncclSuccess && k < n_flows; ++k)
          if (!by_flow[k].empty()) rc = deliver_fragments(comm, k, by_flow[k].data(), static_cast<uint32_t>(by_flow[k].size()));
      }
      posted.push_back(Posted{request, next, now_s()});
      ++next;
    }
    if (rc != ncclSuccess || posted.empty()) break;
    int done = 0, size = 0;
    if ((rc = tcpxTest(posted.front().request, &done, &size)) != ncclSuccess) break;
    if (done) {
      if (latency_s) latency_s[posted.front().index] = now_s() - posted.front().fed;
      // NCCL's proxy flushes a finished receive before it hands the buffer on (iflush takes the request in the
      // request slot and answers with its size, src/net_tcpx.cc:946-954), then reports the slot consumed.
      const tcpxSynthRequest& fr = requests[posted.front().index];
      void* fdata = static_cast<char*>(dst_base) + fr.dst_off;
      int fsize = -1;
      void* freq = posted.front().request;
      if ((rc = tcpxIflush_v5(comm, 1, &fdata, &fsize, &mhandle, &freq)) != ncclSuccess) break;
      if (fsize != static_cast<int>(fr.bytes)) {
        WARN("iflush answered size %d for a request of %u bytes", fsize, fr.bytes);
        rc = ncclInternalError;
        break;
      }
      if ((rc = tcpxIrecvConsumed(comm, 1, posted.front().request)) != ncclSuccess) break;
      posted.pop_front();
      deadline = now_s() + 1e-3 * timeout_ms;
    } else if (now_s() > deadline) {
      WARN("request %u did not complete within %u ms", posted.front().index, timeout_ms);
      rc = ncclInternalError;
    }
  }
  if (seconds) *seconds = now_s() - t0;
  const ncclResult_t rc2 = tcpxDeregMr(comm, mhandle);
  return rc != ncclSuccess ? rc : rc2;
}
