// Synthetic devmem-TCP data socket and the descriptor builder that consumes it.
//
// The socket side produces exactly what the reference's receive path reads from the kernel: a msghdr whose
// control buffer holds one (SOL_SOCKET, SCM_DEVMEM_OFFSET) control message per fragment, each carrying a
// `struct devmemvec {frag_offset, frag_size, frag_token}` (src/sock/tcpx.h:130-134,157-181).  The builder side
// follows process_recv_cmsg (src/sock/tcpx.h:136-228) and gpudirectTCPXRecv (src/sock/tcpx.h:230-297).
#include <algorithm>

#include "plugin_internal.h"

namespace tcpx {

DataPipe::DataPipe()
    // 2048 control messages of CMSG_SPACE(sizeof(struct iovec)) bytes (src/devcomm/unpack_defs1.h:32-36).
    : ctrl_data(static_cast<size_t>(kSlotPages) * CMSG_SPACE(sizeof(struct iovec))), scatter_list(kSlotPages) {}

void DevmemSocket::push(const tcpxSynthFrag* frags, size_t n) {
  std::lock_guard<std::mutex> lock(mu);
  arrived.insert(arrived.end(), frags, frags + n);
}

ssize_t DevmemSocket::recvmsg(struct msghdr* msg, size_t max_bytes) {
  msg->msg_flags = 0;
  if (head == rx.size()) {  // everything taken over earlier has been received: look for new arrivals
    rx.clear();
    head = 0;
    {
      std::lock_guard<std::mutex> lock(mu);
      rx.swap(arrived);
    }
    for (const tcpxSynthFrag& f : rx) payload_frags += f.frag_size != 0;
  }
  // A recvmsg that returns no bytes means "peer closed" to the caller, so empty fragments (which the adversarial
  // workload contains) only ever travel together with a non-empty one.
  if (payload_frags == 0 && head < rx.size()) {
    // Only empty fragments are left on this side: the payload they travel with may have arrived meanwhile.
    std::lock_guard<std::mutex> lock(mu);
    for (const tcpxSynthFrag& f : arrived) payload_frags += f.frag_size != 0;
    rx.insert(rx.end(), arrived.begin(), arrived.end());
    arrived.clear();
  }
  if (payload_frags == 0 || max_bytes == 0) {
    msg->msg_controllen = 0;
    errno = EAGAIN;
    return -1;
  }
  const uint32_t frag_limit = max_frags_per_recvmsg.load(std::memory_order_relaxed);
  const size_t room = msg->msg_controllen;
  const size_t per_cmsg = CMSG_SPACE(sizeof(DevmemVec));
  static_assert(CMSG_SPACE(sizeof(DevmemVec)) == CMSG_LEN(sizeof(DevmemVec)) + 4, "one control message: header, 12 bytes, 4 of padding");
  char* out = static_cast<char*>(msg->msg_control);
  size_t used = 0;
  size_t bytes = 0;
  uint32_t n_payload = 0;
  uint64_t refs = 0;
  while (head < rx.size()) {
    tcpxSynthFrag& f = rx[head];
    if (f.frag_size != 0) {
      if (bytes >= max_bytes) break;
      if (frag_limit != 0 && n_payload >= frag_limit) break;
    }
    if (used + per_cmsg > room) {
      msg->msg_flags |= MSG_CTRUNC;
      break;
    }
    const uint32_t take = static_cast<uint32_t>(std::min<size_t>(f.frag_size, max_bytes - bytes));
    // One control message: the header's three fields, the vector, and the padding that the kernel zeroes too.
    struct cmsghdr* cm = reinterpret_cast<struct cmsghdr*>(out + used);
    cm->cmsg_len = CMSG_LEN(sizeof(DevmemVec));
    cm->cmsg_level = SOL_SOCKET;
    cm->cmsg_type = kScmDevmemOffset;
    const DevmemVec v{f.frag_offset, take, f.frag_token};
    memcpy(CMSG_DATA(cm), &v, sizeof v);
    memset(CMSG_DATA(cm) + sizeof v, 0, 4);
    used += per_cmsg;
    bytes += take;
    if (f.frag_size != 0) ++n_payload;
    // Every control message hands one page reference to the receiver.
    if (device && f.frag_token < device->n_pages) {
      device->page_refs[f.frag_token].fetch_add(1, std::memory_order_relaxed);
      ++refs;
    }
    if (take == f.frag_size) {
      payload_frags -= f.frag_size != 0;
      ++head;
    } else {  // byte budget ended inside the fragment: the rest stays queued
      f.frag_offset += take;
      f.frag_size -= take;
      break;
    }
  }
  if (refs) device->pages_outstanding.fetch_add(refs, std::memory_order_relaxed);
  msg->msg_controllen = used;
  return static_cast<ssize_t>(bytes);
}

int DevmemSocket::dontneed(const PageToken* tokens, size_t n) {
  if (!device) return 0;
  uint64_t given_back = 0;
  int rc = 0;
  for (size_t i = 0; i < n && rc == 0; ++i) {
    for (uint32_t k = 0; k < tokens[i].token_count; ++k) {
      const uint32_t page = tokens[i].token_start + k;
      if (page >= device->n_pages || device->page_refs[page].fetch_sub(1, std::memory_order_relaxed) <= 0) {
        rc = -1;  // no such page, or freed twice
        break;
      }
      ++given_back;
    }
  }
  device->pages_outstanding.fetch_sub(given_back, std::memory_order_relaxed);
  return rc;
}

ssize_t process_recv_cmsg(struct msghdr* msg, DataPipe* p, int offset, uint64_t dst_base_offset,
                          ncclResult_t* result) {
  int num_cm = 0;
  size_t host_bytes = 0;
  ssize_t dst_offset = 0;
  for (struct cmsghdr* cm = CMSG_FIRSTHDR(msg); cm; cm = CMSG_NXTHDR(msg, cm)) {
    if (cm->cmsg_level != SOL_SOCKET || (cm->cmsg_type != kScmDevmemOffset && cm->cmsg_type != kScmDevmemHeader)) {
      INFO(NCCL_NET, "cmsg: unknown %u.%u", cm->cmsg_level, cm->cmsg_type);
      continue;
    }
    ++num_cm;
    DevmemVec v;
    memcpy(&v, CMSG_DATA(cm), sizeof v);
    if (cm->cmsg_type == kScmDevmemHeader) {
      // Payload that landed in host memory instead of a bounce page.  The reference has no working copy for it
      // (its gpu_inline_memcpy is a no-op, src/devcomm/nccl/inline.cu:48-60) and stops; so does this build.
      if (v.frag_size > 0) {
        host_bytes += v.frag_size;
        dst_offset += v.frag_size;
      }
      continue;
    }
    // src/sock/tcpx.h:178-181: where the fragment lies in the bounce buffer, how long it is, and where in the
    // request's buffer it belongs: bytes of this recvmsg so far + bytes of the task so far + the task's offset in
    // the request.
    union loadMeta& d = p->scatter_list[p->cnt_cache];
    d.src_off = v.frag_offset;
    d.len = v.frag_size;
    d.dst_off = static_cast<uint64_t>(dst_offset) + static_cast<uint64_t>(offset) + dst_base_offset;
    p->cnt_cache++;
    if (p->cnt_cache >= static_cast<uint64_t>(kSlotPages)) {  // src/sock/tcpx.h:183-187
      WARN("received %lu/%d segs, failstop", static_cast<unsigned long>(p->cnt_cache), kSlotPages);
      *result = fail_stop("too many fragments in one task");
      return -1;
    }
    dst_offset += v.frag_size;
    // Page tokens, run-length coded (src/sock/tcpx.h:190-199).
    if (*p->pgtok_cnt > 0) {
      PageToken& prev = p->pgtoks[*p->pgtok_cnt - 1];
      if (prev.token_start + prev.token_count == v.frag_token) {
        prev.token_count++;
        continue;
      }
    }
    // The token list is the slot's, one per flow, and a request may put several chunks on one flow: it is full
    // when it holds as many runs as a slot holds descriptors.  (The reference zeroes the count per task and so
    // never gets here; it also forgets the earlier chunks' pages.)
    if (*p->pgtok_cnt >= static_cast<size_t>(kSlotPages)) {
      WARN("flow holds %zu page-token runs for one request, the most a slot records; failstop", *p->pgtok_cnt);
      *result = fail_stop("too many page-token runs on one flow of a request");
      return -1;
    }
    p->pgtoks[*p->pgtok_cnt] = PageToken{v.frag_token, 1};
    (*p->pgtok_cnt)++;
  }
  if (num_cm == 0) {  // src/sock/tcpx.h:202-209
    WARN("fatal, no cmsg");
    *result = fail_stop("recvmsg returned data without control messages");
    return -1;
  }
  if (dst_offset == 0) {  // src/sock/tcpx.h:210-217
    WARN("fatal, no data");
    *result = fail_stop("control messages describe no data");
    return -1;
  }
  if (host_bytes > 0) {  // src/sock/tcpx.h:218-225
    WARN("fatal, data landed on host memory");
    *result = fail_stop("payload landed in host memory");
    return -1;
  }
  return dst_offset;
}

ssize_t devmem_recv(DevmemSocket* sock, int size, int offset, DataPipe* p, uint64_t dst_base_offset,
                    ncclResult_t* result) {
  struct msghdr msg;
  struct iovec iov;
  memset(&msg, 0, sizeof msg);
  msg.msg_control = p->ctrl_data.data();
  msg.msg_controllen = p->ctrl_data.size();
  msg.msg_iov = &iov;
  msg.msg_iovlen = 1;
  iov.iov_base = nullptr;  // payload never lands in host memory here
  iov.iov_len = static_cast<size_t>(size - p->bytes_cnt);
  const ssize_t ret = sock->recvmsg(&msg, iov.iov_len);
  if (ret < 0) return ret;  // EAGAIN: nothing has arrived yet
  if (msg.msg_flags & MSG_CTRUNC) {  // src/sock/tcpx.h:267-274
    WARN("fatal, cmsg truncated, current msg_controllen %zu", p->ctrl_data.size());
    *result = fail_stop("control messages truncated");
    return -1;
  }
  const ssize_t described = process_recv_cmsg(&msg, p, offset, dst_base_offset, result);
  if (described < 0) return -1;
  if (described != ret) {  // src/sock/tcpx.h:276-283
    WARN("fatal, cmsg total bytes %zd, expected %zd", described, ret);
    *result = fail_stop("control messages do not add up to the bytes received");
    return -1;
  }
  p->bytes_cnt += static_cast<int>(ret);
  if (p->bytes_cnt >= size) p->bytes_cnt = 0;
  return ret;
}

TaskRing::TaskRing() {
  for (int i = 0; i < kMaxTasks; ++i) {
    items[i].pipe = new DataPipe;
    scatter[i] = items[i].pipe->scatter_list.data();
  }
}
TaskRing::~TaskRing() {
  for (int i = 0; i < kMaxTasks; ++i) delete items[i].pipe;
}

}  // namespace tcpx
