"""CPU restatement of the reference's host-side bookkeeping on the receive path, in plain Python.

THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only tests/ imports it.

Each function follows the reference file:line it cites (google/nccl-plugin-gpudirecttcpx).  None of this can be
checked against a build of the reference: every translation unit on the path includes NCCL, CUDA, absl or
protobuf headers that are not available (CMakeLists.txt:35-36,77-93), and the reference holds no test or fixture
for any of these functions (its only tests are src/stats/*_test.cc, telemetry).  tests/test_oracle.py pins them
with hand-computed vectors (tests/golden/host_logic_vectors.json) and with the invariants the structures must
keep; tests/test_plugin_host.py then compares the plugin against them on seeded random sequences.
"""

SLOT_PAGES = 2048  # NET_UNPACK_MAX_SLICE_PAGES: src/devcomm/nccl/unpack_defs1.h:23, src/sock/tcpx.h:183
QUEUE_DEPTH = 16   # NCCL_NET_DEVICE_UNPACK_MAX_QUEUE_DEPTH: src/devcomm/nccl/unpack_defs1.h:22
MAX_REQUESTS = 16  # src/work_queue.h:20


class TooManyFragments(Exception):
    """The reference calls exit(1) here (src/sock/tcpx.h:183-187)."""


def process_recv_cmsg(frags, scatter_list, pgtoks, offset, dst_base_offset):
    """One recvmsg worth of devmem control messages -> descriptors and page-token runs.

    frags: iterable of (frag_offset, frag_size, frag_token), one per SCM_DEVMEM_OFFSET control message.
    scatter_list: list of (src_off, len, dst_off), appended to (tcpxDataPipe.scatter_list / cnt_cache).
    pgtoks: list of [token_start, token_count], appended to / coalesced (tcpxDataPipe.pgtoks / *pgtok_cnt).
    Returns the bytes described.  Follows src/sock/tcpx.h:136-228:
      :178-180  src_off = frag_offset; len = frag_size; dst_off = bytes so far in this recvmsg + offset + base
      :183-187  reaching SLOT_PAGES descriptors in one pipe is fatal
      :188      the running byte count advances by frag_size
      :190-199  a token that continues the previous run extends it, otherwise it starts a new run of 1
    """
    dst_offset = 0
    for frag_offset, frag_size, frag_token in frags:
        scatter_list.append((frag_offset, frag_size, dst_offset + offset + dst_base_offset))
        if len(scatter_list) >= SLOT_PAGES:
            raise TooManyFragments(len(scatter_list))
        dst_offset += frag_size
        if pgtoks and pgtoks[-1][0] + pgtoks[-1][1] == frag_token:
            pgtoks[-1][1] += 1
        else:
            pgtoks.append([frag_token, 1])
    return dst_offset


class SlotRing:
    """head/tail of struct tcpxNetDeviceQueue (src/devcomm/unpack_defs1.h:53-59)."""

    def __init__(self):
        self.head = 0
        self.tail = 0

    def next_free(self):
        """__tcpxNetDeviceQueueNextFree (src/devcomm/nccl/unpack1.h:30-65): slot index, or None when full."""
        if self.tail - self.head >= QUEUE_DEPTH:
            return None
        idx = self.tail % QUEUE_DEPTH
        self.tail += 1
        return idx

    def consume(self, slot_idx):
        """The checks of tcpxIrecvConsumed before head advances (src/net_tcpx.cc:1528-1541)."""
        if self.head == self.tail:
            return False
        if self.head % QUEUE_DEPTH != slot_idx:
            return False
        self.head += 1
        return True


class RequestRing:
    """tcpxRequestQueue: five states on monotone cursors (src/work_queue.h:78-130,174-212;
    states src/work_queue_states.h:30-39).  idx[0] <= idx[1] <= ... <= idx[4], idx[4] - idx[0] <= MAX_REQUESTS.
    idx[4] enqueue cursor (FREE->POSTED), idx[3] finish_posted, idx[2] finish_active, idx[1] finish_transmitting,
    idx[0] dequeue (INACTIVE->FREE)."""

    def __init__(self):
        self.idx = [0, 0, 0, 0, 0]

    def has_free(self):
        return MAX_REQUESTS - (self.idx[4] - self.idx[0]) > 0

    def has(self, state):  # state 1..4: INACTIVE, TRANSMITTING, ACTIVE, POSTED
        return self.idx[state] > self.idx[state - 1]

    def first(self, state):  # ring position of the oldest item in `state`
        return self.idx[state - 1] % MAX_REQUESTS

    def enqueue(self):
        self.idx[4] += 1

    def advance(self, state):  # the oldest item of `state` moves to state-1
        self.idx[state - 1] += 1

    def invariant(self):
        return all(self.idx[i] <= self.idx[i + 1] for i in range(4)) and self.idx[4] - self.idx[0] <= MAX_REQUESTS


def request_done(size, size_pending, ctrl_pending):
    """REQUEST_DONE (src/net_tcpx.cc:959-960)."""
    return (size == 0 and ctrl_pending) or (size != 0 and size_pending == 0)
