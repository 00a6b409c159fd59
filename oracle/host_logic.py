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


class SlownessWatch:
    """struct tcpxTimeoutDetection (src/timeout.h:25-44).  Times are integers of one unit (nanoseconds)."""

    def __init__(self, threshold_ns, frequency_ns):
        self.threshold_ns = threshold_ns
        self.frequency_ns = frequency_ns
        self.reset()
        self.first = 0
        self.prev = 0

    def reset(self):
        """tcpxTimeoutDetectionReset (src/timeout.cc:44-47)."""
        self.past_threshold = False
        self.same_count = 0

    def should_warn(self, now):
        """tcpxTimeoutDetectionShouldWarn (src/timeout.cc:52-75): (warn, nanos since the first look).
          :53-56  the first look after a reset notes the time and never warns
          :60-65  until the threshold has been passed: warn once when now - first >= threshold
          :66-71  afterwards: warn when now - previous warning >= frequency
          :73     a warning moves the 'previous warning' time"""
        self.same_count += 1
        if self.same_count == 1:
            self.first = now
            return False, None
        if not self.past_threshold:
            nanos = now - self.first
            if nanos < self.threshold_ns:
                return False, None
            self.past_threshold = True
        else:
            if now - self.prev < self.frequency_ns:
                return False, None
            nanos = now - self.first
        self.prev = now
        return True, nanos


SLOWNESS_NAMES = ("TX_COMP", "SENDRECV", "RX_CTRL", "UNPACK")  # src/flags.cc:84-89, plus this build's UNPACK


def parse_slowness_switches(text, switches):
    """parseSlownessSwitchFlagInternal (src/flags.cc:91-117): comma-separated names, case-insensitive, ALL turns
    every switch on, unknown names are ignored, nothing is ever turned off."""
    if text is None:
        return switches
    for opt in text.split(","):
        if not opt:
            continue  # strtok skips empty fields
        if opt.upper() == "ALL":
            switches = [1] * len(switches)
        for i, name in enumerate(SLOWNESS_NAMES):
            if opt.upper() == name:
                switches[i] = 1
    return switches


# Codes of the exported tracepoint lines (src/stats/tracepoint.h:57-75) and the transition that fires each
# (src/work_queue.h:156-170, 189-211): the tracepoint names the state the item is entering, except that the
# request's enqueue (FREE -> POSTED) is traced as ACTIVE and its finish_posted (POSTED -> ACTIVE) as POSTED.
REQUEST_TRACE_SEQUENCE = (3, 4, 2, 1, 0)  # enqueue, finish_posted, finish_active, finish_transmitting, dequeue
TASK_TRACE_SEQUENCE = (3, 2, 1, 0)  # enqueue, finish_active, finish_completing, dequeue


# ---- flow schedulers (src/flow_mapper.h) ----------------------------------------------------------------------------
MAX_TASKS = 6  # src/work_queue.h:21
MAX_SOCKETS = 8  # src/macro.h:36
SCHED_ALG_RR, SCHED_ALG_KATY = 0, 1  # src/flow_mapper.h:25-29


def sched_alg_from_flag(value):
    """NCCL_GPUDIRECTTCPX_SCHED_ALG (src/net_tcpx.cc:643-665): unset or unknown -> RR; names are case sensitive."""
    return SCHED_ALG_KATY if value == "KATY" else SCHED_ALG_RR


class FlowMapperRR:
    """FlowMapperRR (src/flow_mapper.h:137-157): a stack of the scheduled flows; the priority is ignored."""

    def __init__(self):
        self.flows = []

    def reset(self):
        self.flows = []

    def has_flow(self):
        return len(self.flows) > 0

    def schedule(self, flow, prio):
        self.flows.append(flow)

    def pick(self):
        return self.flows.pop() if self.flows else -1


class FlowMapperKaty:
    """FlowMapperKaty (src/flow_mapper.h:67-135): one bit per (priority, flow), priority-major; the lowest set
    bit is served, moves one priority group up while its priority is below MAX_TASKS - 1, and at most
    NUM_QUANTA_PER_SCHED = 2 flows are served between two resets."""

    QUANTA = 2

    def __init__(self):
        self.reset()

    def reset(self):
        self.bitmap = 0
        self.quanta = self.QUANTA

    def has_flow(self):
        return self.bitmap != 0 and self.quanta > 0

    def schedule(self, flow, prio):
        if prio < 0 or prio >= MAX_TASKS:
            return
        self.bitmap |= 1 << (flow + MAX_SOCKETS * prio)

    def pick(self):
        if not self.has_flow():
            return -1
        bit = (self.bitmap & -self.bitmap).bit_length() - 1
        prio, flow = divmod(bit, MAX_SOCKETS)
        self.bitmap &= ~(1 << bit)
        if prio < MAX_TASKS - 1:
            self.bitmap |= 1 << (bit + MAX_SOCKETS)
        self.quanta -= 1
        return flow


def run_flow_script(mapper, script):
    """Replays [op, args...] steps -- "reset", ["schedule", flow, prio], "pick", "has" -- and returns the answers
    of the pick and has steps in order."""
    out = []
    for step in script:
        op = step[0]
        if op == "reset":
            mapper.reset()
        elif op == "schedule":
            mapper.schedule(step[1], step[2])
        elif op == "pick":
            out.append(mapper.pick())
        elif op == "has":
            out.append(1 if mapper.has_flow() else 0)
        else:
            raise ValueError(op)
    return out
