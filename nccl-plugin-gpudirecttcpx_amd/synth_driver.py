"""Drives one receive comm of the plugin the way NCCL's receive proxy, the peer and the NIC together would.

For every request of a generated workload it posts ``irecv``, then plays the sender and the kernel: one control
message per chunk (a run of consecutive fragments on one flow) and the fragments themselves, then polls ``test``
until the request is done and calls ``irecvConsumed``.  Up to ``window`` requests are kept posted, as NCCL keeps
several steps in flight.  The payload must already be in the bounce arena.
"""
import ctypes
import time

from . import CTRL_INLINE, CTRL_NORMAL, NCCL_PTR_CUDA, CommStats, NetDeviceHandle, SynthFrag, plugin_lib


class PluginError(RuntimeError):
    def __init__(self, fn, rc):
        super().__init__("%s -> ncclResult %d" % (fn, rc))
        self.rc = rc


def ok(rc, fn):
    if rc != 0:
        raise PluginError(fn, rc)


class RecvComm:
    def __init__(self, dev=0):
        self.lib = plugin_lib()
        handle = ctypes.create_string_buffer(128)
        self.listen = ctypes.c_void_p()
        ok(self.lib.tcpxListen(dev, handle, ctypes.byref(self.listen)), "tcpxListen")
        self.comm = ctypes.c_void_p()
        self.dev_handle = NetDeviceHandle()
        ph = ctypes.pointer(self.dev_handle)
        # nobody has connected yet: accept succeeds and hands out no comm
        ok(self.lib.tcpxAccept_v5(self.listen, ctypes.byref(self.comm), ctypes.byref(ph)), "tcpxAccept_v5")
        assert not self.comm.value, "accept handed out a comm before anybody connected"
        # the peer (in a real job another process, holding the 128-byte handle) connects; then accept pairs with it
        self.send_comm = ctypes.c_void_p()
        ok(self.lib.tcpxConnect_v5(dev, handle, ctypes.byref(self.send_comm), None), "tcpxConnect_v5")
        ok(self.lib.tcpxAccept_v5(self.listen, ctypes.byref(self.comm), ctypes.byref(ph)), "tcpxAccept_v5")
        assert self.comm.value, "accept found no connection after connect"
        self.mhandles = {}

    def reg(self, ptr, size, mem_type=NCCL_PTR_CUDA):
        mh = ctypes.c_void_p()
        ok(self.lib.tcpxRegMr(self.comm, ptr, min(size, 2**31 - 1), mem_type, ctypes.byref(mh)), "tcpxRegMr")
        return mh

    def dereg(self, mh):
        ok(self.lib.tcpxDeregMr(self.comm, mh), "tcpxDeregMr")

    def irecv(self, ptr, size, mh):
        data = (ctypes.c_void_p * 1)(ptr)
        sizes = (ctypes.c_int * 1)(size)
        tags = (ctypes.c_int * 1)(0)
        mhs = (ctypes.c_void_p * 1)(mh)
        req = ctypes.c_void_p()
        rc = self.lib.tcpxIrecv_v5(self.comm, 1, data, sizes, tags, mhs, ctypes.byref(req))
        return rc, req

    def test(self, req):
        done = ctypes.c_int(0)
        size = ctypes.c_int(-12345)
        rc = self.lib.tcpxTest(req, ctypes.byref(done), ctypes.byref(size))
        return rc, done.value, size.value

    def iflush(self, ptr, req, mh):
        """(result, size answered): the request goes in through the request slot, as NCCL's proxy passes it."""
        data = (ctypes.c_void_p * 1)(ptr)
        sizes = (ctypes.c_int * 1)(-1)
        mhs = (ctypes.c_void_p * 1)(mh)
        reqs = (ctypes.c_void_p * 1)(req.value if hasattr(req, "value") else req)
        rc = self.lib.tcpxIflush_v5(self.comm, 1, data, sizes, mhs, reqs)
        return rc, sizes[0]

    def consumed(self, req):
        return self.lib.tcpxIrecvConsumed(self.comm, 1, req)

    def ctrl(self, flow, size, offset, total, ctrl_type=CTRL_NORMAL):
        ok(self.lib.tcpxSynthCtrlSend(self.comm, ctrl_type, flow, size, offset, total), "tcpxSynthCtrlSend")

    def deliver(self, flow, frags):
        """frags: numpy structured array with the tcpxSynthFrag layout (16 bytes per row)."""
        assert frags.dtype.itemsize == ctypes.sizeof(SynthFrag)
        ok(self.lib.tcpxSynthDeliver(self.comm, flow, frags.ctypes.data, len(frags)), "tcpxSynthDeliver")

    def outstanding_pages(self):
        n = ctypes.c_uint64()
        ok(self.lib.tcpxSynthOutstandingPages(self.comm, ctypes.byref(n)), "tcpxSynthOutstandingPages")
        return n.value

    def stats(self):
        st = CommStats()
        ok(self.lib.tcpxGetCommStats(self.comm, ctypes.byref(st)), "tcpxGetCommStats")
        return st

    def queue_state(self):
        head, tail = ctypes.c_uint64(), ctypes.c_uint64()
        idx = (ctypes.c_uint32 * 5)()
        ok(self.lib.tcpxDebugQueueState(self.comm, ctypes.byref(head), ctypes.byref(tail), ctypes.byref(idx)), "state")
        return head.value, tail.value, list(idx)

    def slot(self, slot_idx):
        """(descriptor rows as list of (src_off, len, dst_off), published count) of one slot."""
        import numpy as np

        p = ctypes.c_void_p()
        cnt = ctypes.c_uint64()
        ok(self.lib.tcpxDebugSlot(self.comm, slot_idx, ctypes.byref(p), ctypes.byref(cnt)), "tcpxDebugSlot")
        dt = np.dtype([("src_off", "<u4"), ("len", "<u4"), ("dst_off", "<u8")])
        buf = (ctypes.c_uint8 * (2048 * 16)).from_address(p.value)
        return np.frombuffer(buf, dtype=dt), cnt.value

    def close(self):
        ok(self.lib.tcpxClose(self.comm), "tcpxClose")
        ok(self.lib.tcpxClose(self.send_comm), "tcpxClose")
        ok(self.lib.tcpxCloseListen(self.listen), "tcpxCloseListen")


def chunks_of(frags, n_flows):
    """Runs of consecutive fragments on the same flow: (flow, first, count, bytes).  An empty fragment (the
    adversarial workload has them) cannot travel alone, so it joins the run of the payload before it (or, at the
    very start, after it)."""
    import numpy as np

    n = len(frags)
    flows = (frags["flow"] % n_flows).astype(np.int64)
    sizes = frags["frag_size"]
    payload = np.flatnonzero(sizes > 0)
    if payload.size == 0:
        return []
    # index of the nearest payload fragment at or before i, else the first payload fragment
    idx = np.searchsorted(payload, np.arange(n), side="right") - 1
    owner = payload[np.maximum(idx, 0)]
    flows = flows[owner]
    out = []
    i = 0
    while i < n:
        j = i + 1
        while j < n and flows[j] == flows[i]:
            j += 1
        out.append((int(flows[i]), i, j - i, int(sizes[i:j].sum())))
        i = j
    return out


def feed_request(comm, frags, total, n_flows):
    """Plays sender + NIC for one posted request: a control message per chunk, then the chunks' fragments."""
    if total == 0:
        comm.ctrl(0, 0, 0, 0, CTRL_INLINE)
        return
    chunks = chunks_of(frags, n_flows)
    offset = 0
    for flow, first, count, nbytes in chunks:
        comm.ctrl(flow, nbytes, offset, total)
        offset += nbytes
    assert offset == total, (offset, total)
    for flow, first, count, nbytes in chunks:
        comm.deliver(flow, frags[first : first + count])


def run_workload(comm, workload, dst_ptr, n_flows, window=8, timeout_s=60.0, after_request=None):
    """Receives every request of `workload` into dst_ptr + request.dst_off.  Returns per-request latencies (s)
    from the moment the last fragment was delivered to done=1."""
    reqs = workload.requests
    frags_all = workload.frags
    mh = comm.reg(dst_ptr, int(workload.info.dst_bytes))
    posted = []  # (request handle, index, t_fed)
    latencies = []
    next_post = 0
    deadline = time.time() + timeout_s
    while next_post < len(reqs) or posted:
        while next_post < len(reqs) and len(posted) < window:
            r = reqs[next_post]
            first, n, total = int(r["first_desc"]), int(r["n_descs"]), int(r["bytes"])
            rc, req = comm.irecv(dst_ptr + int(r["dst_off"]), total, mh)
            ok(rc, "tcpxIrecv_v5")
            feed_request(comm, frags_all[first : first + n], total, n_flows)
            posted.append((req, next_post, time.perf_counter()))
            next_post += 1
        req, idx, t_fed = posted[0]
        rc, done, _ = comm.test(req)
        ok(rc, "tcpxTest")
        if done:
            latencies.append(time.perf_counter() - t_fed)
            if after_request:
                after_request(idx)
            r = reqs[idx]
            rc, flushed = comm.iflush(dst_ptr + int(r["dst_off"]), req, mh)  # irecv -> test* -> iflush -> irecvConsumed
            ok(rc, "tcpxIflush_v5")
            assert flushed == int(r["bytes"]), (flushed, int(r["bytes"]))
            ok(comm.consumed(req), "tcpxIrecvConsumed")
            posted.pop(0)
            deadline = time.time() + timeout_s
        elif time.time() > deadline:
            raise TimeoutError("request %d did not complete" % idx)
    comm.dereg(mh)
    return latencies


def run_workload_native(comm, workload, dst_ptr, window=8, timeout_ms=30000, first=0, count=None):
    """The same as run_workload for requests [first, first + count), with the loop inside the plugin library
    (tcpxSynthRunRequests): no interpreter between the calls.  Returns (wall seconds, per-request latencies)."""
    import numpy as np

    reqs = workload.requests
    count = len(reqs) - first if count is None else count
    seconds = ctypes.c_double()
    lat = (ctypes.c_double * max(count, 1))()
    frags = np.ascontiguousarray(workload.frags)
    sub = np.ascontiguousarray(reqs[first : first + count])
    rc = comm.lib.tcpxSynthRunRequests(
        comm.comm, frags.ctypes.data, sub.ctypes.data, count, dst_ptr, int(workload.info.dst_bytes), window, timeout_ms,
        ctypes.byref(seconds), lat,
    )  # fmt: skip
    ok(rc, "tcpxSynthRunRequests")
    return seconds.value, list(lat[:count])


def run_chunks_native(comm, workloads, dst_ptr, chunk_stride, window=16, timeout_ms=30000):
    """Several workloads received back to back as ONE list of requests (workload c into dst_ptr + c * chunk_stride),
    so that the request window stays full across them: tcpxSynthRunRequests over the concatenated fragment and
    request arrays.  Returns (wall seconds, per-request latencies)."""
    import numpy as np

    frags, reqs, first = [], [], 0
    for c, wl in enumerate(workloads):
        r = np.array(wl.requests, copy=True)
        r["first_desc"] += first
        r["dst_off"] += c * chunk_stride
        reqs.append(r)
        frags.append(wl.frags)
        first += len(wl.frags)
    frags = np.ascontiguousarray(np.concatenate(frags))
    reqs = np.ascontiguousarray(np.concatenate(reqs))
    seconds = ctypes.c_double()
    lat = (ctypes.c_double * max(len(reqs), 1))()
    rc = comm.lib.tcpxSynthRunRequests(
        comm.comm, frags.ctypes.data, reqs.ctypes.data, len(reqs), dst_ptr, len(workloads) * chunk_stride, window, timeout_ms,
        ctypes.byref(seconds), lat,
    )  # fmt: skip
    ok(rc, "tcpxSynthRunRequests")
    return seconds.value, list(lat[: len(reqs)])
