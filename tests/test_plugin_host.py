"""Host logic of the plugin (no GPU): ncclNet_v7 surface, request ring, slot ring, descriptor builder, page
recycle, completion semantics.  The GPU is replaced by tests/emu (host memory + the CPU oracle as the copier),
installed through the plugin's testing seam; nothing here measures or ships that path.

Reference behaviour that each test pins is cited as src/...:line of google/nccl-plugin-gpudirecttcpx.
"""
import ctypes
import json
import os
import subprocess
import sys

import numpy as np
import pytest

import __graft_entry__ as graft
from plugin_common import ROOT, expected_bytes, load_emu

sys.path.insert(0, os.path.join(ROOT, "oracle"))
import host_logic  # noqa: E402  (test infrastructure)

VECTORS = json.load(open(os.path.join(ROOT, "tests", "golden", "host_logic_vectors.json")))
ARENA_BYTES = 64 << 20
INTERNAL_ERROR, INVALID_ARGUMENT, INVALID_USAGE = 3, 4, 5


@pytest.fixture(scope="module")
def env(pkg):
    emu = load_emu()
    lib = pkg.plugin_lib()
    assert lib.tcpxSetDeviceOpsForTesting(emu.emu_ops()) == 0
    assert lib.tcpxSetFailStopForTesting(0) == 0
    assert lib.tcpxInit(None) == 0
    base = ctypes.c_void_p()
    assert lib.tcpxSynthArenaCreate(0, ARENA_BYTES, ctypes.byref(base)) == 0
    from nccl_plugin_gpudirecttcpx_amd import synth_driver

    class Env:
        pass

    e = Env()
    e.pkg, e.lib, e.emu, e.driver, e.arena = pkg, lib, emu, synth_driver, base.value
    e.arena_np = np.frombuffer((ctypes.c_uint8 * ARENA_BYTES).from_address(base.value), dtype=np.uint8)
    yield e
    assert lib.tcpxFinalize() == 0
    assert emu.emu_counter(1) == 0 and emu.emu_counter(2) == 0 and emu.emu_counter(3) == 0, "finalize leaked"
    assert emu.emu_counter(5) == 0, "finalize leaked host-visible device memory"
    lib.tcpxSetFailStopForTesting(1)
    assert lib.tcpxSetDeviceOpsForTesting(None) == 0


@pytest.fixture
def comm(env):
    c = env.driver.RecvComm(0)
    env.emu.emu_set_hold(0)
    env.emu.emu_set_ring_full(0)
    yield c
    env.emu.emu_set_hold(0)
    env.emu.emu_release(1 << 20)
    c.close()


def host_buffer(nbytes):
    buf = np.full(nbytes, 0xA5, dtype=np.uint8)
    return buf, buf.ctypes.data


def test_v7_table_matches_reference_layout(env):
    """Name string, 19 members in order, regMrDmaBuf absent, closeSend == closeRecv (src/nccl_plugin.cc:22-42)."""
    lib, t = env.lib, env.lib.table
    assert ctypes.string_at(t.name) == b"GPUDirectTCPX_v7"
    assert ctypes.sizeof(env.pkg.NetV7) == 19 * 8

    def addr(name):
        return ctypes.cast(getattr(lib, name), ctypes.c_void_p).value

    expect = {
        "init": "tcpxInit", "devices": "tcpxDevices", "getProperties": "tcpxGetProperties", "listen": "tcpxListen",
        "connect": "tcpxConnect_v5", "accept": "tcpxAccept_v5", "regMr": "tcpxRegMr", "deregMr": "tcpxDeregMr",
        "isend": "tcpxIsend_v5", "irecv": "tcpxIrecv_v5", "iflush": "tcpxIflush_v5", "test": "tcpxTest",
        "closeSend": "tcpxClose", "closeRecv": "tcpxClose", "closeListen": "tcpxCloseListen",
        "getDeviceMr": "tcpxGetDeviceMr", "irecvConsumed": "tcpxIrecvConsumed",
    }  # fmt: skip
    for member, fn in expect.items():
        assert getattr(t, member) == addr(fn), member
    assert t.regMrDmaBuf is None


def test_properties_and_device_handle(env, comm):
    """src/net_tcpx.cc:725-744 and 1463-1467, in the default device type "host": the plugin's engine owns the
    copy, so it advertises an ordinary host-driven network and hands out no device handle (a consumer kernel that
    saw UNPACK would copy every request a second time).  The "unpack" type is covered in test_device_type.py."""
    n = ctypes.c_int()
    assert env.lib.tcpxDevices(ctypes.byref(n)) == 0 and n.value == 1
    p = env.pkg.NetProperties()
    assert env.lib.tcpxGetProperties(0, ctypes.byref(p)) == 0
    assert (p.guid, p.ptrSupport, p.port, p.maxComms, p.latency, p.maxRecvs) == (0, 3, 0, 65536, 0.0, 1)
    assert (p.netDeviceType, p.netDeviceVersion, p.speed) == (0, 0, 10000)
    assert env.lib.tcpxGetProperties(5, ctypes.byref(p)) == INTERNAL_ERROR
    h = comm.dev_handle
    assert (h.netDeviceType, h.netDeviceVersion, h.handle, h.size, h.needsProxyProgress) == (0, 0, None, 0, 0)


def fill_arena(env, wl):
    assert wl.info.pool_bytes <= ARENA_BYTES
    pool = env.arena_np[: wl.info.pool_bytes]
    wl.fill_window(0, pool)
    return pool


@pytest.mark.parametrize("config,shrink", [(1, 0), (2, 2), (3, 4), (4, 5), (5, 3)])
def test_receive_workloads_byte_exact(env, comm, config, shrink):
    wl = env.pkg.Workload(config, seed=0xAB00 + config, shrink=shrink)
    pool = fill_arena(env, wl)
    buf, ptr = host_buffer(int(wl.info.dst_bytes) + 64)
    env.driver.run_workload(comm, wl, ptr, n_flows=4, window=8)
    want = expected_bytes(pool, wl.frags, wl.requests, int(wl.info.dst_bytes) + 64)
    assert np.array_equal(buf, want)
    assert comm.outstanding_pages() == 0, "pages not recycled (src/sock/tcpx.h:310-326)"
    head, tail, idx = comm.queue_state()
    assert head == tail == len(wl.requests) and len(set(idx)) == 1 and idx[0] == len(wl.requests)


@pytest.mark.parametrize("config,shrink", [(1, 0), (2, 2), (3, 4), (5, 3)])
def test_native_driver_gives_the_same_bytes(env, comm, config, shrink):
    """tcpxSynthRunRequests (the request loop inside the library) against the same expectation as the Python driver."""
    wl = env.pkg.Workload(config, seed=0xAB00 + config, shrink=shrink)
    pool = fill_arena(env, wl)
    buf, ptr = host_buffer(int(wl.info.dst_bytes) + 64)
    seconds, lat = env.driver.run_workload_native(comm, wl, ptr, window=8)
    assert seconds > 0 and len(lat) == len(wl.requests) and min(lat) > 0
    assert np.array_equal(buf, expected_bytes(pool, wl.frags, wl.requests, int(wl.info.dst_bytes) + 64))
    assert comm.outstanding_pages() == 0
    head, tail, idx = comm.queue_state()
    assert head == tail == len(wl.requests)
    assert env.lib.tcpxSynthRunRequests(comm.comm, None, None, 0, ptr, 64, 8, 1000, None, None) == INVALID_ARGUMENT
    assert env.lib.tcpxSynthRunRequests(comm.comm, ptr, ptr, 0, ptr, 64, 17, 1000, None, None) == INVALID_ARGUMENT


def test_small_requests_hand_over_a_second_copy_of_their_descriptors(env, comm):
    """A request of at most 16 descriptors is submitted with its descriptors in host-visible device memory (copied
    there and flushed before the submission); a longer one with the mapped slot.  Either way the bytes are right,
    and a comm whose device offers no such memory works the same."""
    wl = env.pkg.Workload(3, seed=0x57A6, shrink=6)  # requests of 16 fragments
    big = env.pkg.Workload(2, seed=0x57A7, shrink=2)  # requests of hundreds
    for workload, staged in ((wl, True), (big, False)):
        pool = fill_arena(env, workload)
        buf, ptr = host_buffer(int(workload.info.dst_bytes))
        before = [env.emu.emu_counter(i) for i in (0, 6, 7)]
        env.driver.run_workload(comm, workload, ptr, n_flows=4, window=8)
        after = [env.emu.emu_counter(i) for i in (0, 6, 7)]
        assert np.array_equal(buf, expected_bytes(pool, workload.frags, workload.requests, int(workload.info.dst_bytes)))
        submitted, in_visible, flushes = (a - b for a, b in zip(after, before))
        assert submitted == len(workload.requests)
        assert (in_visible, flushes) == ((submitted, submitted) if staged else (0, 0))
    env.emu.emu_set_visible_off(1)
    try:
        c2 = env.driver.RecvComm(0)
        pool = fill_arena(env, wl)
        buf, ptr = host_buffer(int(wl.info.dst_bytes))
        # (a comm that takes a recycled queue block keeps that block's copy area; a new block gets none)
        env.driver.run_workload(c2, wl, ptr, n_flows=4, window=8)
        assert np.array_equal(buf, expected_bytes(pool, wl.frags, wl.requests, int(wl.info.dst_bytes)))
        c2.close()
    finally:
        env.emu.emu_set_visible_off(0)


def test_the_request_size_goes_along_with_the_submission(env, comm):
    """The slot is handed to the engine with the request's byte count as a hint (the sum of its descriptors'
    lengths); one request at a time, so that the last submission seen is the request just completed."""
    wl = env.pkg.Workload(5, seed=0x51ED, shrink=5)  # ragged fragments and empty descriptors
    pool = fill_arena(env, wl)
    buf, ptr = host_buffer(int(wl.info.dst_bytes))
    env.driver.run_workload(comm, wl, ptr, n_flows=4, window=1)
    assert np.array_equal(buf, expected_bytes(pool, wl.frags, wl.requests, int(wl.info.dst_bytes)))
    last = wl.requests[-1]
    first, n = int(last["first_desc"]), int(last["n_descs"])
    assert env.emu.emu_counter(8) == int(wl.descs["len"][first : first + n].sum()) == int(last["bytes"])


def test_partial_recvmsg_and_window_one(env, comm):
    """Fragments trickle in three per recvmsg; one request in flight at a time."""
    wl = env.pkg.Workload(2, seed=77, shrink=3)
    pool = fill_arena(env, wl)
    assert env.lib.tcpxSynthSetRecvmsgLimit(comm.comm, 3) == 0
    buf, ptr = host_buffer(int(wl.info.dst_bytes))
    env.driver.run_workload(comm, wl, ptr, n_flows=4, window=1)
    assert np.array_equal(buf, expected_bytes(pool, wl.frags, wl.requests, int(wl.info.dst_bytes)))
    assert comm.outstanding_pages() == 0


def drive_until_transmitted(comm, req, limit=100000):
    """Polls test() until every fragment of the request has been turned into descriptors (the engine is held)."""
    for _ in range(limit):
        rc, done, _ = comm.test(req)
        assert rc == 0 and done == 0
        if comm.emu.emu_pending() > 0:
            return
    raise AssertionError("request never reached the engine")


@pytest.mark.parametrize("seed", range(6))
def test_descriptors_match_restated_builder(env, comm, seed):
    """The slot's descriptor list equals what process_recv_cmsg (src/sock/tcpx.h:136-228) produces for the same
    control messages: one flow, random chunk sizes, random fragments per recvmsg."""
    rng = np.random.default_rng(seed)
    comm.emu = env.emu
    n = int(rng.integers(5, 300))
    sizes = rng.integers(1, 4097, size=n).astype(np.uint32)
    pages = rng.choice(ARENA_BYTES // 4096, size=n, replace=False).astype(np.uint32)
    in_page = (rng.integers(0, 4097, size=n) % (4097 - sizes)).astype(np.uint32)
    # make some page tokens consecutive so that runs get coalesced
    for i in range(1, n):
        if rng.random() < 0.3:
            pages[i] = (pages[i - 1] + 1) % (ARENA_BYTES // 4096)
    frags = np.zeros(n, dtype=env.pkg.Workload(1, shrink=6).frag_dtype)
    frags["frag_offset"], frags["frag_size"], frags["frag_token"] = pages * 4096 + in_page, sizes, pages
    total = int(sizes.sum())
    per_recvmsg = int(rng.integers(1, 9))
    assert env.lib.tcpxSynthSetRecvmsgLimit(comm.comm, per_recvmsg) == 0
    # chunks: random cut points on fragment boundaries, all on flow 0
    cuts = sorted(set(rng.integers(1, n, size=int(rng.integers(0, 4))).tolist())) if n > 1 else []
    bounds = [0] + cuts + [n]
    env.emu.emu_set_hold(1)
    buf, ptr = host_buffer(total + 16)
    mh = comm.reg(ptr, total)
    rc, req = comm.irecv(ptr, total, mh)
    assert rc == 0
    # restated builder, fed exactly what the synthetic socket will hand out
    want, tokens, off = [], [], 0
    for a, b in zip(bounds[:-1], bounds[1:]):
        chunk_bytes = int(sizes[a:b].sum())
        comm.ctrl(0, chunk_bytes, off, total)
        scatter, task_off = [], 0
        for k in range(a, b, per_recvmsg):
            part = [(int(f["frag_offset"]), int(f["frag_size"]), int(f["frag_token"])) for f in frags[k : min(k + per_recvmsg, b)]]
            task_off += host_logic.process_recv_cmsg(part, scatter, tokens, task_off, off)
        want += scatter
        off += chunk_bytes
    comm.deliver(0, frags)
    drive_until_transmitted(comm, req)
    head, tail, _ = comm.queue_state()
    rows, cnt = comm.slot(head % 16)
    assert cnt == n
    got = [(int(r["src_off"]), int(r["len"]), int(r["dst_off"])) for r in rows[:n]]
    assert got == want
    assert comm.outstanding_pages() == n  # one reference per control message until consumed
    env.emu.emu_release(1)
    rc, done, size = comm.test(req)
    assert (rc, done) == (0, 1) and size == -12345, "test() never writes *size (src/net_tcpx.cc:1311-1374)"
    assert comm.consumed(req) == 0
    assert comm.outstanding_pages() == 0
    comm.dereg(mh)
    want_buf = np.full(total + 16, 0xA5, dtype=np.uint8)
    pos = 0
    for f in frags:
        want_buf[pos : pos + int(f["frag_size"])] = env.arena_np[int(f["frag_offset"]) : int(f["frag_offset"]) + int(f["frag_size"])]
        pos += int(f["frag_size"])
    assert np.array_equal(buf, want_buf)


def simple_request(env, comm, nbytes=8192, page=0):
    frags = np.zeros(nbytes // 4096, dtype=env.pkg.Workload(1, shrink=6).frag_dtype)
    frags["frag_offset"] = (page + np.arange(len(frags))) * 4096
    frags["frag_size"] = 4096
    frags["frag_token"] = page + np.arange(len(frags))
    return frags


def test_done_only_after_the_copy_completed(env, comm):
    """done=1 is reported when the engine's completion word arrives, not when descriptors are published."""
    comm.emu = env.emu
    env.emu.emu_set_hold(1)
    buf, ptr = host_buffer(8192)
    mh = comm.reg(ptr, 8192)
    rc, req = comm.irecv(ptr, 8192, mh)
    comm.ctrl(1, 8192, 0, 8192)
    comm.deliver(1, simple_request(env, comm))
    drive_until_transmitted(comm, req)
    for _ in range(50):
        assert comm.test(req)[:2] == (0, 0)
    assert (buf == 0xA5).all()
    submitted = env.emu.emu_counter(0)
    env.emu.emu_release(1)
    assert comm.test(req)[:2] == (0, 1)
    assert env.emu.emu_counter(0) == submitted, "a request is submitted to the engine exactly once"
    assert np.array_equal(buf, env.arena_np[:8192])
    assert comm.consumed(req) == 0
    comm.dereg(mh)


def post_and_feed(env, comm, ptr, mh, n, nbytes=8192):
    """n receives of nbytes each, every one with its control message and fragments already there."""
    reqs = []
    for i in range(n):
        rc, req = comm.irecv(ptr + i * nbytes, nbytes, mh)
        assert rc == 0
        comm.ctrl(i % 4, nbytes, 0, nbytes)
        comm.deliver(i % 4, simple_request(env, comm, nbytes, page=i * (nbytes // 4096)))
        reqs.append(req)
    return reqs


def test_every_complete_request_is_at_the_engine_before_it_is_tested(env, comm):
    """A comm keeps up to sixteen slots with the consumer (src/devcomm/nccl/unpack1.h:30-65; the reference reports
    done at publish, src/net_tcpx.cc:1354-1370): polling the OLDEST request submits every request whose bytes are
    all there, and completion is still reported in posting order."""
    env.emu.emu_set_hold(1)
    buf, ptr = host_buffer(16 * 8192)
    mh = comm.reg(ptr, 16 * 8192)
    reqs = post_and_feed(env, comm, ptr, mh, 16)
    submitted = env.emu.emu_counter(0)
    for _ in range(40):
        assert comm.test(reqs[0])[:2] == (0, 0)
    assert env.emu.emu_counter(0) - submitted == 16 and env.emu.emu_pending() == 16
    assert comm.stats().max_slots_at_gpu == 16
    assert (buf == 0xA5).all()
    for i, req in enumerate(reqs):
        assert comm.test(req)[:2] == (0, 0)
        if i + 1 < 16:
            assert comm.test(reqs[i + 1])[0] == INTERNAL_ERROR  # src/net_tcpx.cc:1322-1328
        env.emu.emu_release(1)
        assert comm.test(req)[:2] == (0, 1)
        assert np.array_equal(buf[: (i + 1) * 8192], env.arena_np[: (i + 1) * 8192]) and (buf[(i + 1) * 8192 :] == 0xA5).all()
    assert env.emu.emu_counter(0) - submitted == 16, "a request is submitted to the engine exactly once"
    for req in reqs:
        assert comm.consumed(req) == 0
    assert comm.outstanding_pages() == 0
    comm.dereg(mh)


def test_a_younger_slot_that_finishes_first_waits_for_the_older_one(env, comm):
    """Completion words may arrive in any order; done is reported in posting order only."""
    env.emu.emu_set_hold(1)
    buf, ptr = host_buffer(3 * 8192)
    mh = comm.reg(ptr, 3 * 8192)
    r0, r1, r2 = post_and_feed(env, comm, ptr, mh, 3)
    for _ in range(20):
        assert comm.test(r0)[:2] == (0, 0)
    assert env.emu.emu_pending() == 3
    assert env.emu.emu_release_at(2) == 1 and env.emu.emu_release_at(1) == 1  # the two younger copies finish
    assert np.array_equal(buf[8192:], env.arena_np[8192 : 3 * 8192]) and (buf[:8192] == 0xA5).all()
    for _ in range(20):
        assert comm.test(r0)[:2] == (0, 0), "the oldest request's own completion word gates it"
    assert comm.test(r1)[0] == INTERNAL_ERROR and comm.test(r2)[0] == INTERNAL_ERROR
    assert comm.consumed(r1) == INTERNAL_ERROR
    assert env.emu.emu_release(1) == 1
    assert comm.test(r0)[:2] == (0, 1)
    assert comm.test(r2)[0] == INTERNAL_ERROR
    assert comm.test(r1)[:2] == (0, 1) and comm.test(r2)[:2] == (0, 1)  # their words were there already
    for r in (r0, r1, r2):
        assert comm.consumed(r) == 0
    assert np.array_equal(buf, env.arena_np[: 3 * 8192])
    assert comm.stats().max_slots_at_gpu == 3
    comm.dereg(mh)


def test_submissions_behind_a_full_engine_ring_keep_their_order(env, comm):
    buf, ptr = host_buffer(4 * 8192)
    mh = comm.reg(ptr, 4 * 8192)
    env.emu.emu_set_ring_full(1)
    reqs = post_and_feed(env, comm, ptr, mh, 4)
    submitted = env.emu.emu_counter(0)
    for _ in range(20):
        assert comm.test(reqs[0])[:2] == (0, 0)
    assert env.emu.emu_counter(0) == submitted
    env.emu.emu_set_ring_full(0)
    for req in reqs:
        for _ in range(20):
            rc, done, _ = comm.test(req)
            assert rc == 0
            if done:
                break
        assert done == 1
    assert env.emu.emu_counter(0) - submitted == 4
    for req in reqs:
        assert comm.consumed(req) == 0
    assert np.array_equal(buf, env.arena_np[: 4 * 8192])
    comm.dereg(mh)


def test_a_receive_may_only_write_what_it_registered_and_posted(env, comm):
    """Host-side bounds on what the GPU will be told to write (the reference checks none of them,
    src/net_tcpx.cc:771-853, 862-896, 995-1010)."""
    buf, ptr = host_buffer(4 * 8192)
    mh = comm.reg(ptr + 8192, 8192)
    assert comm.irecv(ptr, 8192, mh)[0] == INTERNAL_ERROR  # starts before the registration
    assert comm.irecv(ptr + 8192, 8193, mh)[0] == INTERNAL_ERROR  # ends after it
    assert comm.irecv(ptr + 12288, 8192, mh)[0] == INTERNAL_ERROR
    assert comm.irecv(ptr + 8192, -1, mh)[0] == INTERNAL_ERROR
    assert comm.queue_state()[2] == [0, 0, 0, 0, 0], "a refused receive takes no request"
    # a message longer than the posted receive
    rc, req = comm.irecv(ptr + 8192, 4096, mh)
    assert rc == 0
    comm.ctrl(0, 8192, 0, 8192)
    assert comm.test(req)[0] == INTERNAL_ERROR
    assert (buf == 0xA5).all() and env.emu.emu_pending() == 0


def test_a_chunk_may_not_run_past_its_message(env, comm):
    buf, ptr = host_buffer(8192)
    mh = comm.reg(ptr, 8192)
    rc, req = comm.irecv(ptr, 8192, mh)
    assert rc == 0
    comm.ctrl(0, 4096, 0, 8192)
    comm.ctrl(1, 4097, 4096, 8192)
    for _ in range(4):
        rc = comm.test(req)[0]
        if rc:
            break
    assert rc == INTERNAL_ERROR
    assert (buf == 0xA5).all()


def test_engine_ring_full_is_retried(env, comm):
    buf, ptr = host_buffer(8192)
    mh = comm.reg(ptr, 8192)
    rc, req = comm.irecv(ptr, 8192, mh)
    comm.ctrl(0, 8192, 0, 8192)
    comm.deliver(0, simple_request(env, comm))
    env.emu.emu_set_ring_full(1)
    for _ in range(20):
        assert comm.test(req)[:2] == (0, 0)
    env.emu.emu_set_ring_full(0)
    for _ in range(20):
        rc, done, _ = comm.test(req)
        assert rc == 0
        if done:
            break
    assert done == 1 and np.array_equal(buf, env.arena_np[:8192])
    assert comm.consumed(req) == 0
    comm.dereg(mh)


def test_irecv_argument_errors_and_ring_capacity(env, comm):
    """n != 1, NULL mhandle, 17th request: ncclInternalError (src/net_tcpx.cc:926, 866-873)."""
    buf, ptr = host_buffer(4096)
    mh = comm.reg(ptr, 4096)
    data = (ctypes.c_void_p * 2)(ptr, ptr)
    sizes = (ctypes.c_int * 2)(1, 1)
    tags = (ctypes.c_int * 2)()
    mhs = (ctypes.c_void_p * 2)(mh, mh)
    req = ctypes.c_void_p()
    assert env.lib.tcpxIrecv_v5(comm.comm, 2, data, sizes, tags, mhs, ctypes.byref(req)) == INTERNAL_ERROR
    assert comm.irecv(ptr, 4096, None)[0] == INTERNAL_ERROR
    reqs = []
    for _ in range(16):
        rc, r = comm.irecv(ptr, 4096, mh)
        assert rc == 0
        reqs.append(r)
    assert comm.irecv(ptr, 4096, mh)[0] == INTERNAL_ERROR
    assert comm.queue_state()[2] == [0, 0, 0, 0, 16]
    # drain them as empty messages so that the comm closes clean
    for r in reqs:
        comm.ctrl(0, 0, 0, 0, env.pkg.CTRL_INLINE)
    for r in reqs:
        for _ in range(10):
            rc, done, _ = comm.test(r)
            assert rc == 0
            if done:
                break
        assert done == 1
        assert comm.consumed(r) == 0
    comm.dereg(mh)
    assert env.lib.tcpxRegMr(None, ptr, 10, 1, ctypes.byref(req)) == INTERNAL_ERROR
    assert env.lib.tcpxRegMr(comm.comm, ptr, 10, 99, ctypes.byref(req)) == INTERNAL_ERROR
    assert env.lib.tcpxDeregMr(comm.comm, None) == 0


def test_zero_size_message(env, comm):
    """An empty message takes a slot, completes with cnt = 0 and is consumed through the fast path
    (src/net_tcpx.cc:1248-1276, 1361, 1500-1504)."""
    buf, ptr = host_buffer(64)
    mh = comm.reg(ptr, 64)
    rc, req = comm.irecv(ptr, 64, mh)
    assert comm.test(req)[:2] == (0, 0)  # nothing arrived yet
    comm.ctrl(0, 0, 0, 0, env.pkg.CTRL_INLINE)
    assert comm.test(req)[:2] == (0, 1)
    head, tail, _ = comm.queue_state()
    assert (head, tail) == (0, 1)
    assert comm.slot(0)[1] == 0
    sizes = (ctypes.c_int * 1)(777)
    reqs = (ctypes.c_void_p * 1)(req)
    assert env.lib.tcpxIflush_v5(comm.comm, 1, None, sizes, None, reqs) == 0 and sizes[0] == 0  # src/net_tcpx.cc:946-954
    assert env.lib.tcpxIflush_v5(comm.comm, 2, None, sizes, None, reqs) == INTERNAL_ERROR
    assert comm.consumed(req) == 0
    assert comm.queue_state()[:2] == (1, 1)
    assert (buf == 0xA5).all()
    comm.dereg(mh)


def test_order_and_consume_errors(env, comm):
    """test(NULL); test() out of order; irecvConsumed with NULL / n != 1 / wrong request / before completion
    (src/net_tcpx.cc:1315-1328, 1479-1535)."""
    assert env.lib.tcpxTest(None, ctypes.byref(ctypes.c_int()), None) == INTERNAL_ERROR
    buf, ptr = host_buffer(16384)
    mh = comm.reg(ptr, 16384)
    rc, r0 = comm.irecv(ptr, 8192, mh)
    rc, r1 = comm.irecv(ptr + 8192, 8192, mh)
    assert env.lib.tcpxIrecvConsumed(comm.comm, 1, None) == INTERNAL_ERROR
    assert env.lib.tcpxIrecvConsumed(comm.comm, 2, r0) == INTERNAL_ERROR
    for i, r in enumerate((r0, r1)):
        comm.ctrl(i, 8192, 0, 8192)
        comm.deliver(i, simple_request(env, comm, page=2 * i))
    # both requests have all their data; the second one may not be tested before the first (1322-1328)
    for _ in range(20):
        rc, done, _ = comm.test(r1)
        if rc != 0:
            break
    assert rc == INTERNAL_ERROR
    assert comm.consumed(r0) == INTERNAL_ERROR  # not completed yet: no INACTIVE request (1512-1515)
    for r in (r0, r1):
        for _ in range(20):
            rc, done, _ = comm.test(r)
            assert rc == 0
            if done:
                break
        assert done == 1
    assert comm.consumed(r1) == INTERNAL_ERROR  # not the oldest (1517-1521)
    assert comm.consumed(r0) == 0 and comm.consumed(r1) == 0
    assert np.array_equal(buf, env.arena_np[:16384])
    assert comm.outstanding_pages() == 0
    comm.dereg(mh)


def test_too_many_fragments_is_fatal(env, comm):
    """2048 descriptors in one task stop the reference (src/sock/tcpx.h:183-187); with fail-stop switched off for
    the test the same condition surfaces as ncclInternalError."""
    n = 2100
    frags = np.zeros(n, dtype=env.pkg.Workload(1, shrink=6).frag_dtype)
    frags["frag_offset"] = np.arange(n) * 4096
    frags["frag_size"] = 2
    frags["frag_token"] = np.arange(n)
    buf, ptr = host_buffer(2 * n)
    mh = comm.reg(ptr, 2 * n)
    rc, req = comm.irecv(ptr, 2 * n, mh)
    comm.ctrl(0, 2 * n, 0, 2 * n)
    comm.deliver(0, frags)
    rc = 0
    for _ in range(50):
        rc, done, _ = comm.test(req)
        if rc != 0:
            break
    assert rc == INTERNAL_ERROR
    comm.dereg(mh)


def test_page_token_runs_of_one_flow_are_bounded(env, comm, capfd):
    """A request may put several chunks on one flow, and their page tokens accumulate in the slot's one list for
    that flow (2048 runs).  Two chunks of 1100 fragments with tokens that never coalesce would write run 2049 past
    the end of the list; the builder stops there, like the reference stops on descriptor overflow
    (src/sock/tcpx.h:183-199), instead of after the fact when the chunk is reaped."""
    per_chunk, size = 1100, 8
    n = 2 * per_chunk
    frags = np.zeros(n, dtype=env.pkg.Workload(1, shrink=6).frag_dtype)
    frags["frag_offset"] = np.arange(n) * 2 * 4096  # every other page: no two tokens are neighbours
    frags["frag_size"] = size
    frags["frag_token"] = np.arange(n) * 2
    total = n * size
    buf, ptr = host_buffer(total)
    mh = comm.reg(ptr, total)
    rc, req = comm.irecv(ptr, total, mh)
    assert rc == 0
    comm.ctrl(0, per_chunk * size, 0, total)
    comm.ctrl(0, per_chunk * size, per_chunk * size, total)
    comm.deliver(0, frags)
    rc = 0
    for _ in range(50):
        rc, done, _ = comm.test(req)
        assert not done
        if rc != 0:
            break
    assert rc == INTERNAL_ERROR
    # stopped by the builder at the 2049th run, not later by the count check when the chunk is reaped
    err = capfd.readouterr().err
    assert "page-token runs" in err and "request too many pages" not in err
    comm.dereg(mh)


def test_devmem_contract_is_enforced(env, comm):
    bad = simple_request(env, comm)
    bad["frag_offset"][0] = 4000
    bad["frag_size"][0] = 200  # crosses a page
    assert env.lib.tcpxSynthDeliver(comm.comm, 0, bad.ctypes.data, len(bad)) == INVALID_ARGUMENT
    bad = simple_request(env, comm)
    bad["frag_offset"][0] = ARENA_BYTES  # outside the arena
    assert env.lib.tcpxSynthDeliver(comm.comm, 0, bad.ctypes.data, len(bad)) == INVALID_ARGUMENT
    assert env.lib.tcpxSynthDeliver(comm.comm, 9, bad.ctypes.data, 0) == INVALID_ARGUMENT


def test_send_side_is_absent(env):
    handle = ctypes.create_string_buffer(128)
    lc, sc, req = ctypes.c_void_p(), ctypes.c_void_p(), ctypes.c_void_p()
    assert env.lib.tcpxListen(0, handle, ctypes.byref(lc)) == 0
    assert env.lib.tcpxConnect_v5(0, handle, ctypes.byref(sc), None) == 0
    assert env.lib.tcpxIsend_v5(sc, None, 0, 0, None, ctypes.byref(req)) == INTERNAL_ERROR
    assert env.lib.tcpxClose(sc) == 0 and env.lib.tcpxCloseListen(lc) == 0


def test_device_ops_cannot_be_swapped_after_init(env):
    assert env.lib.tcpxSetDeviceOpsForTesting(None) == INVALID_USAGE


def test_init_fails_loudly_without_the_hip_layer(tmp_path):
    """No GPU library, no fallback: tcpxInit reports ncclSystemError (run in a fresh process, with the plugin copied
    to a directory that holds no libtcpxu_hip.so)."""
    code = (
        "import ctypes,shutil,sys\n"
        "shutil.copy(r'%s/nccl-plugin-gpudirecttcpx_amd/lib/libnccl-net.so', r'%s/libnccl-net.so')\n"
        "lib=ctypes.CDLL(r'%s/libnccl-net.so')\n"
        "rc=lib.tcpxInit(None)\n"
        "print('rc',rc); sys.exit(0 if rc==2 else 1)\n" % (ROOT, tmp_path, tmp_path)
    )
    env = dict(os.environ, LD_LIBRARY_PATH="")
    p = subprocess.run([sys.executable, "-c", code], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env, timeout=120)
    assert p.returncode == 0, p.stdout


def test_socket_thread_mode(tmp_path):
    """The same receive with fragments consumed by a helper thread per comm (src/net_tcpx.cc:252-384) and 8 flows."""
    script = os.path.join(ROOT, "tests", "helper_thread_case.py")
    env = dict(os.environ, NCCL_GPUDIRECTTCPX_AMD_HELPER_THREAD="1", NCCL_GPUDIRECTTCPX_AMD_FLOWS="8")
    p = subprocess.run([sys.executable, script], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env, timeout=300)
    assert p.returncode == 0, p.stdout
    assert "helper-thread case ok" in p.stdout
    assert "sched alg 0" in p.stdout


def test_socket_thread_binding():
    """NCCL_GPUDIRECTTCPX_RX_BINDINGS in the reference's syntax (parseCoreRanges, src/common.cc:65-130) binds a receive
    comm's socket thread to the CPUs named for its device (src/net_tcpx.cc:300-307); entries for other devices and
    malformed ranges leave it on the CPUs of the process."""
    script = os.path.join(ROOT, "tests", "helper_thread_case.py")
    allowed = sorted(os.sched_getaffinity(0))
    one = allowed[-1]

    def cpus(bindings, helper="1"):
        env = dict(os.environ, NCCL_GPUDIRECTTCPX_AMD_HELPER_THREAD=helper, NCCL_GPUDIRECTTCPX_AMD_FLOWS="4")
        env.pop("NCCL_GPUDIRECTTCPX_RX_BINDINGS", None)
        if bindings is not None:
            env["NCCL_GPUDIRECTTCPX_RX_BINDINGS"] = bindings
        p = subprocess.run([sys.executable, script, "2"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env, timeout=300)
        assert p.returncode == 0 and "helper-thread case ok" in p.stdout, p.stdout
        return [int(line.split()[-1]) for line in p.stdout.splitlines() if line.startswith("socket thread cpus")]

    assert cpus(None) == [len(allowed)]
    assert cpus("tcpx-amd-synth0:%d-%d" % (one, one)) == [1]
    assert cpus("eth9:0-1;tcpx-amd-synth0:%d-%d;" % (one, one)) == [1]
    if len(allowed) >= 2:
        lo, hi = allowed[0], allowed[1]
        assert cpus("tcpx-amd-synth0:%d-%d,%d-%d" % (lo, lo, hi, hi)) == [2]
    assert cpus("eth9:0-1") == [len(allowed)]  # another device's
    assert cpus("tcpx-amd-synth0:%d" % one) == [len(allowed)]  # no upper end: invalid, as in the reference
    # an invalid range is skipped on its own and the device's other ranges stand (src/common.cc:104-108); so does a
    # trailing comma
    assert cpus("tcpx-amd-synth0:%d,%d-%d" % (one, one, one)) == [1]
    assert cpus("tcpx-amd-synth0:%d-%d,bogus," % (one, one)) == [1]
    assert cpus("tcpx-amd-synth0:%d-%d" % (one, one), helper="0") == [0]  # no socket thread


# ---- flow scheduler (src/flow_mapper.h) -----------------------------------------------------------------------------
def run_sched_script(lib, alg, script):
    sched = ctypes.c_void_p()
    assert lib.tcpxFlowSchedCreate(alg.encode() if alg is not None else None, ctypes.byref(sched)) == 0
    out = []
    try:
        for step in script:
            if step[0] == "reset":
                lib.tcpxFlowSchedReset(sched)
            elif step[0] == "schedule":
                lib.tcpxFlowSchedSchedule(sched, step[1], step[2])
            elif step[0] == "pick":
                out.append(lib.tcpxFlowSchedPick(sched))
            else:
                out.append(lib.tcpxFlowSchedHasFlow(sched))
    finally:
        lib.tcpxFlowSchedDestroy(sched)
    return out


def test_flow_scheduler_hand_computed(env):
    for case in VECTORS["flow_mapper"]:
        assert run_sched_script(env.lib, case["alg"], case["script"]) == case["expect"], case["ref"]
    for case in VECTORS["sched_alg_flag"]:
        if case["value"] is None:
            continue  # NULL means "what tcpxInit selected"; the unset flag is covered by test_socket_thread_mode
        sched = ctypes.c_void_p()
        assert env.lib.tcpxFlowSchedCreate(case["value"].encode(), ctypes.byref(sched)) == 0
        assert env.lib.tcpxFlowSchedAlg(sched) == case["alg"], case["value"]
        env.lib.tcpxFlowSchedDestroy(sched)
    assert env.lib.tcpxFlowSchedCreate(b"RR", None) == INVALID_ARGUMENT
    assert env.lib.tcpxFlowSchedPick(None) == -1 and env.lib.tcpxFlowSchedHasFlow(None) == 0


@pytest.mark.parametrize("alg", ["RR", "KATY"])
def test_flow_scheduler_matches_restatement_on_random_scripts(env, alg):
    """Random schedule/pick/reset sequences as a comm would issue them: every flow scheduled at most once between
    two resets, at most 8 flows (the RR mapper's stack holds MAX_SOCKETS entries and is not bounds-checked)."""
    rng = np.random.default_rng(0x5CED + len(alg))
    for _ in range(200):
        script = []
        for _ in range(int(rng.integers(1, 6))):
            script.append(["reset"])
            flows = rng.permutation(8)[: int(rng.integers(0, 9))]
            for f in flows:
                script.append(["schedule", int(f), int(rng.integers(-1, 8))])
            for _ in range(int(rng.integers(0, 6))):
                script.append(["pick"] if rng.random() < 0.7 else ["has"])
        mapper = host_logic.FlowMapperKaty() if alg == "KATY" else host_logic.FlowMapperRR()
        assert run_sched_script(env.lib, alg, script) == host_logic.run_flow_script(mapper, script)


def test_katy_scheduler_receives_the_same_bytes():
    """NCCL_GPUDIRECTTCPX_SCHED_ALG=KATY: the comm gates on the other scheduler; the received bytes do not change."""
    script = os.path.join(ROOT, "tests", "helper_thread_case.py")
    env = dict(os.environ, NCCL_GPUDIRECTTCPX_SCHED_ALG="KATY", NCCL_GPUDIRECTTCPX_AMD_FLOWS="8")
    p = subprocess.run([sys.executable, script], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env, timeout=300)
    assert p.returncode == 0, p.stdout
    assert "sched alg 1" in p.stdout and "helper-thread case ok" in p.stdout


def test_unknown_scheduler_name_means_round_robin():
    script = os.path.join(ROOT, "tests", "helper_thread_case.py")
    env = dict(os.environ, NCCL_GPUDIRECTTCPX_SCHED_ALG="katy", NCCL_GPUDIRECTTCPX_AMD_FLOWS="8")
    p = subprocess.run([sys.executable, script], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env, timeout=300)
    assert p.returncode == 0, p.stdout
    assert "sched alg 0" in p.stdout
