"""Observability of the receive path (no GPU): slowness watches on the three waits of a request, counters, and
tracepoints at the ring transitions.  The GPU is replaced by tests/emu through the plugin's testing seam.

What the reference does is cited as src/...:line of google/nccl-plugin-gpudirecttcpx.  Its own tests for this
subsystem are src/stats/tracepoint_test.cc (counter semantics of the RECVMSG tracepoint) and
src/stats/stats_buffer_test.cc (three events in, three events out, a consumer that waits): both are mirrored below.
The watch itself (src/timeout.cc) has no test in the reference; it is pinned by hand-computed looks in
tests/golden/host_logic_vectors.json (test_oracle.py) and the plugin is compared with that restatement here.
"""
import ctypes
import os
import re
import sys
import threading

import numpy as np
import pytest

from plugin_common import ROOT, load_emu

sys.path.insert(0, os.path.join(ROOT, "oracle"))
import host_logic  # noqa: E402  (test infrastructure)

ARENA_BYTES = 16 << 20
THRESHOLD_NS, FREQUENCY_NS = 1_000_000, 2_500_000
# The plugin calls the logger as logger(level, flags, file, line, "%s", text): the text is the first variadic
# argument, which the x86-64 calling convention passes like a sixth ordinary one.
LOGGER = ctypes.CFUNCTYPE(None, ctypes.c_int, ctypes.c_ulong, ctypes.c_char_p, ctypes.c_int, ctypes.c_char_p, ctypes.c_char_p)


class Session:
    """One tcpxInit .. tcpxFinalize with the given environment, an injected clock and a log collector."""

    def __init__(self, pkg, flags):
        self.pkg, self.flags = pkg, flags
        self.now = 5_000_000_000
        self.warnings = []

    def __enter__(self):
        self.saved = {k: os.environ.get(k) for k in self.flags}
        for k, v in self.flags.items():
            os.environ[k] = v
        self.emu = load_emu()
        self.lib = self.pkg.plugin_lib()
        self.clock_cb = self.pkg.CLOCK_FN(lambda: self.now)

        def log(level, flags, file, line, fmt, text):
            if level == 2 and fmt == b"%s":
                self.warnings.append(text.decode(errors="replace"))

        self.log_cb = LOGGER(log)
        assert self.lib.tcpxSetDeviceOpsForTesting(self.emu.emu_ops()) == 0
        assert self.lib.tcpxSetClockForTesting(ctypes.cast(self.clock_cb, ctypes.c_void_p)) == 0
        assert self.lib.tcpxInit(ctypes.cast(self.log_cb, ctypes.c_void_p)) == 0
        base = ctypes.c_void_p()
        assert self.lib.tcpxSynthArenaCreate(0, ARENA_BYTES, ctypes.byref(base)) == 0
        from nccl_plugin_gpudirecttcpx_amd import synth_driver

        self.driver = synth_driver
        self.comm = synth_driver.RecvComm(0)
        self.emu.emu_set_hold(0)
        self.emu.emu_set_ring_full(0)
        return self

    def __exit__(self, *exc):
        self.emu.emu_set_hold(0)
        self.emu.emu_release(1 << 20)
        self.comm.close()
        assert self.lib.tcpxFinalize() == 0
        self.lib.tcpxSetClockForTesting(None)
        assert self.lib.tcpxSetDeviceOpsForTesting(None) == 0
        for k, v in self.saved.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v

    # -- helpers ---------------------------------------------------------------------------------------------
    def comm_stats(self):
        s = self.pkg.CommStats()
        assert self.lib.tcpxGetCommStats(self.comm.comm, ctypes.byref(s)) == 0
        return s

    def flow_stats(self, flow):
        s = self.pkg.FlowStats()
        assert self.lib.tcpxGetFlowStats(self.comm.comm, flow, ctypes.byref(s)) == 0
        return s

    def drain(self, max_events=20000, wait_ms=0):
        ev = (self.pkg.TraceEvent * max_events)()
        n = ctypes.c_uint32()
        assert self.lib.tcpxTraceDrain(self.comm.comm, ev, max_events, wait_ms, ctypes.byref(n)) == 0
        return [ev[i] for i in range(n.value)]

    def frags(self, nbytes=8192, page=0, flow=0):
        f = np.zeros(nbytes // 4096, dtype=self.pkg.Workload(1, shrink=6).frag_dtype)
        f["frag_offset"] = (page + np.arange(len(f))) * 4096
        f["frag_size"] = 4096
        f["frag_token"] = page + np.arange(len(f))
        f["flow"] = flow
        return f


def session(pkg, **flags):
    env = {"NCCL_GPUDIRECTTCPX_TIMEOUT_THRESHOLD_NS": str(THRESHOLD_NS), "NCCL_GPUDIRECTTCPX_TIMEOUT_FREQUENCY_NS": str(FREQUENCY_NS)}
    env.update({"NCCL_GPUDIRECTTCPX_" + k: v for k, v in flags.items()})
    return Session(pkg, env)


def host_buffer(nbytes):
    buf = np.full(nbytes, 0xA5, dtype=np.uint8)
    return buf, buf.ctypes.data


def looks_against_the_restatement(s, req, counter, n_looks, seed):
    """Calls test() n_looks times while the request waits, moving the injected clock by seeded steps, and checks
    after every look that `counter()` has grown exactly when the restated watch (oracle) reports."""
    rng = np.random.default_rng(seed)
    watch = host_logic.SlownessWatch(THRESHOLD_NS, FREQUENCY_NS)
    expected = counter()
    reports = 0
    for _ in range(n_looks):
        s.now += int(rng.integers(0, 700_000))
        assert s.comm.test(req)[:2] == (0, 0)
        warn, _ = watch.should_warn(s.now)
        expected += int(warn)
        reports += int(warn)
        assert counter() == expected
    assert reports >= 2, "the sequence must cross the threshold and at least one frequency interval"
    return reports


def test_waiting_for_the_control_message_is_watched(pkg):
    """src/net_tcpx.cc:1234-1246: every look at the control socket feeds comm->ctrl_timeout; a message resets it."""
    with session(pkg) as s:
        buf, ptr = host_buffer(8192)
        mh = s.comm.reg(ptr, 8192)
        rc, req = s.comm.irecv(ptr, 8192, mh)
        n = looks_against_the_restatement(s, req, lambda: s.comm_stats().rx_ctrl_slow_cnt, 40, seed=1)
        assert sum("rx ctrl timeout" in w for w in s.warnings) == n
        # The message arrives: the watch starts over, so the next request's wait is timed from its own first look.
        s.comm.ctrl(0, 8192, 0, 8192)
        s.comm.deliver(0, s.frags())
        while s.comm.test(req)[1] == 0:
            pass
        assert s.comm.consumed(req) == 0
        before = s.comm_stats().rx_ctrl_slow_cnt
        rc, req = s.comm.irecv(ptr, 8192, mh)
        s.now += 10 * FREQUENCY_NS  # a long gap before the first look must not count
        assert s.comm.test(req)[:2] == (0, 0)
        assert s.comm_stats().rx_ctrl_slow_cnt == before
        looks_against_the_restatement_from_second = host_logic.SlownessWatch(THRESHOLD_NS, FREQUENCY_NS)
        looks_against_the_restatement_from_second.should_warn(s.now)
        s.now += THRESHOLD_NS
        assert s.comm.test(req)[:2] == (0, 0)
        assert looks_against_the_restatement_from_second.should_warn(s.now) == (True, THRESHOLD_NS)
        assert s.comm_stats().rx_ctrl_slow_cnt == before + 1
        s.comm.ctrl(0, 8192, 0, 8192)
        s.comm.deliver(0, s.frags())
        while s.comm.test(req)[1] == 0:
            pass
        assert s.comm.consumed(req) == 0
        s.comm.dereg(mh)


def test_recvmsg_finding_nothing_is_watched_and_counted(pkg):
    """TCPX_TASK_TP_RECVMSG (src/net_tcpx.cc:167, src/stats/tracepoint.cc:22-52,72-82): a recvmsg that returns
    EAGAIN feeds the task's watch; rx_cnt counts every call, successful or not
    (src/stats/tracepoint_test.cc:70-84: "Rx cnt alway ++")."""
    with session(pkg, TELEMETRY_ENABLE_TASK_LEVEL_STATS="1") as s:
        buf, ptr = host_buffer(8192)
        mh = s.comm.reg(ptr, 8192)
        rc, req = s.comm.irecv(ptr, 8192, mh)
        s.comm.ctrl(2, 8192, 0, 8192)
        # takes the control message, creates the task and, in the pass that follows at once, looks at the socket for
        # the first time (nothing there yet)
        assert s.comm.test(req)[:2] == (0, 0)
        assert s.flow_stats(2).rx_ctrl_done_cnt == 1 and s.flow_stats(0).rx_ctrl_done_cnt == 0
        calls0 = s.flow_stats(2).rx_cnt
        assert calls0 == 1
        watch_reports = []
        watch = host_logic.SlownessWatch(THRESHOLD_NS, FREQUENCY_NS)
        assert watch.should_warn(s.now) == (False, None)  # the task's first look only notes the time
        rng = np.random.default_rng(2)
        for i in range(40):
            s.now += int(rng.integers(0, 700_000))
            assert s.comm.test(req)[:2] == (0, 0)
            watch_reports.append(watch.should_warn(s.now)[0])
            assert s.flow_stats(2).rx_slow_cnt == sum(watch_reports)
            assert s.flow_stats(2).rx_cnt == calls0 + i + 1
        assert sum(watch_reports) >= 2
        assert sum("recv timeout" in w for w in s.warnings) == sum(watch_reports)
        assert s.flow_stats(1).rx_cnt == 0 and s.flow_stats(1).rx_slow_cnt == 0
        s.comm.deliver(2, s.frags(flow=2))
        before = s.flow_stats(2).rx_cnt
        while s.comm.test(req)[1] == 0:
            pass
        assert s.flow_stats(2).rx_cnt == before + 1, "the successful recvmsg is counted too"
        assert s.comm.consumed(req) == 0
        s.comm.dereg(mh)
    with session(pkg) as s:  # task-level stats off: the watch still works, the call counter stays at zero
        buf, ptr = host_buffer(8192)
        mh = s.comm.reg(ptr, 8192)
        rc, req = s.comm.irecv(ptr, 8192, mh)
        s.comm.ctrl(0, 8192, 0, 8192)
        for _ in range(3):
            s.now += THRESHOLD_NS
            assert s.comm.test(req)[:2] == (0, 0)
        assert s.flow_stats(0).rx_cnt == 0 and s.flow_stats(0).rx_slow_cnt >= 1
        s.comm.deliver(0, s.frags())
        while s.comm.test(req)[1] == 0:
            pass
        assert s.comm.consumed(req) == 0
        s.comm.dereg(mh)


def test_a_slot_held_by_the_gpu_is_watched(pkg):
    """This build's own watch: the slot has been handed to the engine and the completion word does not come."""
    with session(pkg) as s:
        s.emu.emu_set_hold(1)
        buf, ptr = host_buffer(8192)
        mh = s.comm.reg(ptr, 8192)
        rc, req = s.comm.irecv(ptr, 8192, mh)
        s.comm.ctrl(1, 8192, 0, 8192)
        s.comm.deliver(1, s.frags(flow=1))
        while s.emu.emu_pending() == 0:
            assert s.comm.test(req)[:2] == (0, 0)
        published_at = s.now
        assert s.comm_stats().unpack_cnt == 1 and s.comm_stats().unpack_slow_cnt == 0
        # The test() that published also took the watch's first look.
        watch = host_logic.SlownessWatch(THRESHOLD_NS, FREQUENCY_NS)
        watch.should_warn(s.now)
        rng = np.random.default_rng(3)
        reports = 0
        for _ in range(40):
            s.now += int(rng.integers(0, 700_000))
            assert s.comm.test(req)[:2] == (0, 0)
            reports += int(watch.should_warn(s.now)[0])
            assert s.comm_stats().unpack_slow_cnt == reports
        assert reports >= 2 and sum("unpack timeout" in w for w in s.warnings) == reports
        s.emu.emu_release(1)
        s.now += 12345
        assert s.comm.test(req)[:2] == (0, 1)
        assert s.comm_stats().unpack_ns == s.now - published_at
        assert s.comm.consumed(req) == 0
        s.comm.dereg(mh)


@pytest.mark.parametrize(
    "switch,report,watched,reported",
    [
        ("RX_CTRL", None, {"ctrl"}, {"ctrl"}),  # report defaults to every watch; unwatched ones are turned off
        ("ALL", "unpack", {"ctrl", "recv", "unpack"}, {"unpack"}),
        ("", None, set(), set()),
        ("sendrecv,UNPACK", "ALL", {"recv", "unpack"}, {"recv", "unpack"}),
    ],
)
def test_switches_select_what_is_watched_and_what_is_reported(pkg, switch, report, watched, reported):
    """NCCL_GPUDIRECTTCPX_SLOWNESS_SWITCH / _REPORT (src/flags.cc:119-150)."""
    flags = {"SLOWNESS_SWITCH": switch}
    if report is not None:
        flags["SLOWNESS_REPORT"] = report
    with session(pkg, **flags) as s:
        s.emu.emu_set_hold(1)
        buf, ptr = host_buffer(8192)
        mh = s.comm.reg(ptr, 8192)
        rc, req = s.comm.irecv(ptr, 8192, mh)
        for _ in range(3):  # waiting for the control message
            s.now += THRESHOLD_NS
            assert s.comm.test(req)[:2] == (0, 0)
        s.comm.ctrl(0, 8192, 0, 8192)
        for _ in range(3):  # waiting for fragments
            s.now += THRESHOLD_NS
            assert s.comm.test(req)[:2] == (0, 0)
        s.comm.deliver(0, s.frags())
        for _ in range(5):  # waiting for the (held) GPU
            s.now += THRESHOLD_NS
            assert s.comm.test(req)[:2] == (0, 0)
        got = set()
        if s.comm_stats().rx_ctrl_slow_cnt:
            got.add("ctrl")
        if s.flow_stats(0).rx_slow_cnt:
            got.add("recv")
        if s.comm_stats().unpack_slow_cnt:
            got.add("unpack")
        assert got == watched
        said = set()
        for w in s.warnings:
            for key, name in (("rx ctrl timeout", "ctrl"), ("recv timeout", "recv"), ("unpack timeout", "unpack")):
                if key in w:
                    said.add(name)
        assert said == reported
        s.emu.emu_release(1)
        assert s.comm.test(req)[:2] == (0, 1)
        assert s.comm.consumed(req) == 0
        s.comm.dereg(mh)


def test_timeout_flags_are_range_checked(pkg):
    """Below 100 us the flag is refused and the default stays (src/net_tcpx.cc:519-524)."""
    with Session(pkg, {"NCCL_GPUDIRECTTCPX_TIMEOUT_THRESHOLD_NS": "99999"}) as s:
        assert any("ignored" in w for w in s.warnings)
        buf, ptr = host_buffer(4096)
        mh = s.comm.reg(ptr, 4096)
        rc, req = s.comm.irecv(ptr, 4096, mh)
        assert s.comm.test(req)[:2] == (0, 0)
        s.now += 9_999_999_999  # one nanosecond short of the 10 s default
        assert s.comm.test(req)[:2] == (0, 0)
        assert s.comm_stats().rx_ctrl_slow_cnt == 0
        s.now += 1
        assert s.comm.test(req)[:2] == (0, 0)
        assert s.comm_stats().rx_ctrl_slow_cnt == 1
        s.comm.ctrl(0, 0, 0, 0, pkg.CTRL_INLINE)
        assert s.comm.test(req)[:2] == (0, 1)
        assert s.comm.consumed(req) == 0
        s.comm.dereg(mh)


def run_small_workload(s, n_flows=4):
    wl = s.pkg.Workload(2, seed=0xC0FFEE02, shrink=5)
    pool = np.empty(wl.info.pool_bytes, dtype=np.uint8)
    assert pool.nbytes <= ARENA_BYTES
    dst = np.full(wl.info.dst_bytes + 64, 0xA5, dtype=np.uint8)

    def tick(_):
        s.now += 1000

    s.driver.run_workload(s.comm, wl, dst.ctypes.data, n_flows, window=4, after_request=tick)
    return wl


def test_tracepoints_follow_the_ring_transitions(pkg):
    """A tracepoint at every transition of the request and task rings, with the reference's codes
    (src/work_queue.h:156-211, src/stats/tracepoint.h:57-75); the exported line is
    "R <request> <passive> <state> <timestamp>" (src/stats/stats_buffer.h:52-56)."""
    with session(pkg, TELEMETRY_ENABLE_TASK_LEVEL_STATS="1", TELEMETRY_ENABLE_REQUEST_LEVEL_STATS="1") as s:
        wl = run_small_workload(s)
        events = s.drain()
        assert s.comm_stats().trace_dropped == 0
        per_object = {}
        for e in events:
            assert e.passive == 1 and e.kind in (b"R", b"T")
            per_object.setdefault((e.kind, e.object), []).append(e.state)
        timestamps = [e.timestamp for e in events]
        assert timestamps == sorted(timestamps) and timestamps[0] >= 5_000_000_000  # the injected clock
        n_requests = n_tasks = 0
        for (kind, _), states in per_object.items():
            cycle = host_logic.REQUEST_TRACE_SEQUENCE if kind == b"R" else host_logic.TASK_TRACE_SEQUENCE
            assert len(states) % len(cycle) == 0
            assert tuple(states) == cycle * (len(states) // len(cycle)), (kind, states)
            if kind == b"R":
                n_requests += len(states) // len(cycle)
            else:
                n_tasks += len(states) // len(cycle)
        assert n_requests == len(wl.requests)
        chunks = sum(len(s.driver.chunks_of(wl.frags[int(r["first_desc"]) : int(r["first_desc"]) + int(r["n_descs"])], 4)) for r in wl.requests)
        assert n_tasks == chunks, "one task per chunk (control message)"
        line = ctypes.create_string_buffer(256)
        n = s.lib.tcpxTraceFormat(ctypes.byref(events[0]), line, 256)
        assert n > 0 and re.fullmatch(rb"R 0x[0-9a-f]+ 1 3 \d+", line.value), line.value
        assert s.drain() == []


def test_levels_and_sampling_select_the_events(pkg):
    with session(pkg) as s:  # both levels off: nothing is recorded
        run_small_workload(s)
        assert s.drain() == []
    with session(pkg, TELEMETRY_ENABLE_REQUEST_LEVEL_STATS="1") as s:
        run_small_workload(s)
        all_requests = s.drain()
        assert all_requests and all(e.kind == b"R" for e in all_requests)
    with session(pkg, TELEMETRY_ENABLE_TASK_LEVEL_STATS="1", TELEMETRY_SAMPLING_FACTOR="7") as s:
        run_small_workload(s)
        sampled = s.drain()
        # objects are kept when their address is a multiple of the factor (src/stats/stats_buffer.h:51,61)
        assert all(e.kind == b"T" and e.object % 7 == 0 for e in sampled)


def test_a_consumer_can_wait_and_a_full_buffer_drops(pkg):
    """src/stats/stats_buffer_test.cc: three events enqueued while a consumer waits come out as three events;
    the buffer holds 10000 events (src/stats/stats_buffer.h:24) and enqueueing is best effort beyond that."""
    with session(pkg, TELEMETRY_ENABLE_REQUEST_LEVEL_STATS="1") as s:
        got = []

        def consumer():
            while len(got) < 3:
                got.extend(s.drain(max_events=3 - len(got), wait_ms=5000))

        t = threading.Thread(target=consumer)
        t.start()
        buf, ptr = host_buffer(4096)
        mh = s.comm.reg(ptr, 4096)
        reqs = [s.comm.irecv(ptr, 4096, mh)[1] for _ in range(3)]
        t.join(timeout=30)
        assert not t.is_alive() and [e.state for e in got] == [3, 3, 3]
        assert len({e.object for e in got}) == 3
        for req in reqs:
            s.comm.ctrl(0, 0, 0, 0, pkg.CTRL_INLINE)
            assert s.comm.test(req)[:2] == (0, 1)
            assert s.comm.consumed(req) == 0
        s.drain()
        # 2100 empty messages x 5 transitions with nobody draining: 10000 kept, 500 dropped
        for _ in range(2100):
            rc, req = s.comm.irecv(ptr, 4096, mh)
            assert rc == 0
            s.comm.ctrl(0, 0, 0, 0, pkg.CTRL_INLINE)
            assert s.comm.test(req)[:2] == (0, 1)
            assert s.comm.consumed(req) == 0
        assert s.comm_stats().trace_dropped == 500
        assert len(s.drain()) == 10000
        s.comm.dereg(mh)
