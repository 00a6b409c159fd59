"""End-to-end GPU parity of the plugin path: irecv -> synthetic fragments -> descriptor builder -> mapped slot ->
persistent engine -> completion word -> test() -> irecvConsumed, byte-exact against the CPU oracle, on all five
workloads at their full sizes.  Bounce arena, receive buffers and engine are the real HIP ones.
"""
import ctypes

import numpy as np
import pytest

import __graft_entry__ as graft
from conftest import GUARD, SENTINEL, first_difference

pytestmark = pytest.mark.gpu

ARENA_BYTES = 1 << 30


@pytest.fixture(scope="module")
def env(pkg):
    import torch

    lib = pkg.plugin_lib()
    assert lib.tcpxSetDeviceOpsForTesting(None) == 0  # the real HIP layer
    assert lib.tcpxInit(None) == 0, "tcpxInit must succeed on a GPU box"
    base = ctypes.c_void_p()
    assert lib.tcpxSynthArenaCreate(0, ARENA_BYTES, ctypes.byref(base)) == 0
    from nccl_plugin_gpudirecttcpx_amd import synth_driver

    class Env:
        pass

    e = Env()
    e.pkg, e.lib, e.driver, e.arena, e.torch, e.hip = pkg, lib, synth_driver, base.value, torch, pkg.hip_layer()
    yield e
    assert lib.tcpxFinalize() == 0


def upload(env, pool, offset=0):
    pkg = env.pkg
    pkg.check(env.hip.tcpxuCopyToDevice(0, env.arena + offset, pool.ctypes.data, pool.nbytes), "tcpxuCopyToDevice")


@pytest.mark.parametrize("config", [1, 2, 3, 4])
def test_plugin_workloads_full_size(env, oracle, config):
    torch = env.torch
    wl = env.pkg.Workload(config, seed=0xC0FFEE00 + config)
    info = wl.info
    pool = np.empty(info.pool_bytes, dtype=np.uint8)
    wl.fill_window(0, pool)
    upload(env, pool)
    expect = np.full(GUARD + info.dst_bytes + GUARD, SENTINEL, dtype=np.uint8)
    graft.oracle_unpack(oracle, expect[GUARD : GUARD + info.dst_bytes], pool, np.ascontiguousarray(wl.descs))
    dst = torch.full((GUARD + info.dst_bytes + GUARD,), SENTINEL, dtype=torch.uint8, device="cuda:0")
    torch.cuda.synchronize()
    comm = env.driver.RecvComm(0)
    print("plugin case: config %d, %d requests, %d fragments" % (config, info.n_requests, info.n_descs), flush=True)
    env.driver.run_workload(comm, wl, dst.data_ptr() + GUARD, n_flows=4, window=8, timeout_s=30)
    got = dst.cpu().numpy()  # read back while the engine kernel is still running
    assert comm.outstanding_pages() == 0
    head, tail, _ = comm.queue_state()
    assert head == tail == info.n_requests
    # Counters of the hand-off to the GPU: one slot per request, each timed, none slow (threshold 10 s).
    stats = env.pkg.CommStats()
    assert env.lib.tcpxGetCommStats(comm.comm, ctypes.byref(stats)) == 0
    assert stats.unpack_cnt == info.n_requests and stats.unpack_slow_cnt == 0 and stats.rx_ctrl_slow_cnt == 0
    assert 0 < stats.unpack_ns < 30e9
    print("plugin case: mean publish->done %.1f us" % (stats.unpack_ns / stats.unpack_cnt / 1e3), flush=True)
    comm.close()
    assert first_difference(got, expect) is None, "first (index, got, want, count): %r" % (first_difference(got, expect),)


def test_plugin_adversarial_with_page_reuse(env, oracle):
    """32 MiB, lengths 1..4096 with empty fragments, destination base +3, pages refilled between requests:
    a request's pages are recycled by irecvConsumed before the next window's payload overwrites them."""
    torch = env.torch
    wl = env.pkg.Workload(5, seed=0xC0FFEE05)
    info = wl.info
    pool = np.empty(info.pool_bytes, dtype=np.uint8)
    base = GUARD + info.dst_misalign
    expect = np.full(base + info.dst_bytes + GUARD, SENTINEL, dtype=np.uint8)
    dst = torch.full((base + info.dst_bytes + GUARD,), SENTINEL, dtype=torch.uint8, device="cuda:0")
    torch.cuda.synchronize()
    comm = env.driver.RecvComm(0)
    mh = comm.reg(dst.data_ptr() + base, int(info.dst_bytes))
    for i, r in enumerate(wl.requests):
        first, n, total = int(r["first_desc"]), int(r["n_descs"]), int(r["bytes"])
        wl.fill_window(int(r["window"]), pool)
        upload(env, pool)
        graft.oracle_unpack(oracle, expect[base : base + info.dst_bytes], pool, np.ascontiguousarray(wl.descs[first : first + n]))
        rc, req = comm.irecv(dst.data_ptr() + base + int(r["dst_off"]), total, mh)
        assert rc == 0
        env.driver.feed_request(comm, wl.frags[first : first + n], total, 2)
        print("window %d: %d fragments, %d bytes" % (i, n, total), flush=True)
        import time

        deadline = time.time() + 30
        while True:
            rc, done, _ = comm.test(req)
            assert rc == 0
            if done:
                break
            assert time.time() < deadline, "request %d did not complete" % i
        assert comm.outstanding_pages() > 0
        assert comm.consumed(req) == 0
        assert comm.outstanding_pages() == 0
    got = dst.cpu().numpy()
    comm.dereg(mh)
    comm.close()
    assert first_difference(got, expect) is None, repr(first_difference(got, expect))


def test_two_comms_share_one_engine(env, oracle):
    torch = env.torch
    wls = [env.pkg.Workload(2, seed=100 + i, shrink=1) for i in range(2)]
    pool = np.empty(wls[0].info.pool_bytes, dtype=np.uint8)
    wls[0].fill_window(0, pool)
    upload(env, pool)
    comms = [env.driver.RecvComm(0) for _ in wls]
    outs = []
    for c, wl in zip(comms, wls):
        dst = torch.full((int(wl.info.dst_bytes) + 2 * GUARD,), SENTINEL, dtype=torch.uint8, device="cuda:0")
        torch.cuda.synchronize()
        env.driver.run_workload(c, wl, dst.data_ptr() + GUARD, n_flows=4, window=4, timeout_s=30)
        outs.append(dst)
    for c, wl, dst in zip(comms, wls, outs):
        expect = np.full(int(wl.info.dst_bytes) + 2 * GUARD, SENTINEL, dtype=np.uint8)
        graft.oracle_unpack(oracle, expect[GUARD : GUARD + int(wl.info.dst_bytes)], pool, np.ascontiguousarray(wl.descs))
        assert first_difference(dst.cpu().numpy(), expect) is None
        c.close()


def test_a_comm_keeps_many_slots_at_the_gpu(env, oracle):
    """Sixteen requests posted with all their fragments already there: polling the oldest submits every one of them
    to the engine (the reference's consumer may hold all sixteen slots of a comm, src/devcomm/nccl/unpack1.h:30-65,
    because its test() reports done at publish, src/net_tcpx.cc:1354-1370), done is still reported strictly in
    posting order, and the bytes are the oracle's."""
    import time

    torch = env.torch
    wl = env.pkg.Workload(3, seed=0x51075, shrink=5)  # 64 requests of 16 x 4 KiB
    info = wl.info
    pool = np.empty(info.pool_bytes, dtype=np.uint8)
    wl.fill_window(0, pool)
    upload(env, pool)
    expect = np.full(GUARD + info.dst_bytes + GUARD, SENTINEL, dtype=np.uint8)
    graft.oracle_unpack(oracle, expect[GUARD : GUARD + info.dst_bytes], pool, np.ascontiguousarray(wl.descs))
    dst = torch.full((GUARD + info.dst_bytes + GUARD,), SENTINEL, dtype=torch.uint8, device="cuda:0")
    torch.cuda.synchronize()
    comm = env.driver.RecvComm(0)
    base = dst.data_ptr() + GUARD
    mh = comm.reg(base, int(info.dst_bytes))
    order = []
    print("plugin case: 4 bursts of 16 requests of 64 KiB, all fed before the first poll", flush=True)
    for burst in range(4):
        posted = []
        for k in range(16 * burst, 16 * burst + 16):
            r = wl.requests[k]
            first, n, total = int(r["first_desc"]), int(r["n_descs"]), int(r["bytes"])
            rc, req = comm.irecv(base + int(r["dst_off"]), total, mh)
            assert rc == 0
            env.driver.feed_request(comm, wl.frags[first : first + n], total, 4)
            posted.append((k, req))
        assert comm.irecv(base, 4096, mh)[0] == 3, "the request ring holds sixteen (src/work_queue.h:20)"
        deadline = time.time() + 30
        while posted:
            k, req = posted[0]
            rc, done, _ = comm.test(req)
            assert rc == 0
            if done:
                order.append(k)
                assert comm.consumed(req) == 0
                posted.pop(0)
            else:
                if len(posted) > 1:
                    assert comm.test(posted[1][1])[0] == 3, "only the oldest request may be tested (src/net_tcpx.cc:1322-1328)"
                assert time.time() < deadline, "request %d did not complete" % k
    got = dst.cpu().numpy()
    stats = comm.stats()
    print("plugin case: most slots at the GPU at one time: %d" % stats.max_slots_at_gpu, flush=True)
    assert order == list(range(64))
    assert stats.unpack_cnt == 64 and stats.max_slots_at_gpu >= 8
    assert comm.outstanding_pages() == 0
    head, tail, _ = comm.queue_state()
    assert head == tail == 64
    comm.dereg(mh)
    comm.close()
    assert first_difference(got, expect) is None, "first (index, got, want, count): %r" % (first_difference(got, expect),)


def test_native_driver_with_the_whole_request_ring_posted(env, oracle):
    """tcpxSynthRunRequests with sixteen requests posted at a time over four 8 MiB chunks as one request list."""
    torch = env.torch
    wls = [env.pkg.Workload(2, seed=0xC0FFEE02 + 7919 * i) for i in range(4)]
    info = wls[0].info
    pool = np.empty(info.pool_bytes, dtype=np.uint8)
    wls[0].fill_window(0, pool)
    upload(env, pool)
    chunk = int(info.dst_bytes)
    expect = np.full(GUARD + 4 * chunk + GUARD, SENTINEL, dtype=np.uint8)
    for c, wl in enumerate(wls):
        graft.oracle_unpack(oracle, expect[GUARD + c * chunk : GUARD + (c + 1) * chunk], pool, np.ascontiguousarray(wl.descs))
    dst = torch.full((GUARD + 4 * chunk + GUARD,), SENTINEL, dtype=torch.uint8, device="cuda:0")
    torch.cuda.synchronize()
    comm = env.driver.RecvComm(0)
    print("native plugin case: 4 chunks of 8 MiB, 16 requests posted at a time", flush=True)
    seconds, lat = env.driver.run_chunks_native(comm, wls, dst.data_ptr() + GUARD, chunk, window=16)
    got = dst.cpu().numpy()
    stats = comm.stats()
    print("native plugin case: %.1f GB/s, most slots at the GPU at one time: %d" % (4 * chunk / seconds / 1e9, stats.max_slots_at_gpu), flush=True)
    assert comm.outstanding_pages() == 0 and len(lat) == sum(int(wl.info.n_requests) for wl in wls)
    assert stats.unpack_cnt == len(lat) and 1 <= stats.max_slots_at_gpu <= 16
    comm.close()
    assert first_difference(got, expect) is None, "first (index, got, want, count): %r" % (first_difference(got, expect),)


def test_hip_layer_is_what_init_bound(env):
    """The plugin on a GPU box runs on libtcpxu_hip.so: the device count it reports is the HIP layer's."""
    n = ctypes.c_int()
    m = ctypes.c_int()
    assert env.lib.tcpxDevices(ctypes.byref(n)) == 0
    env.pkg.check(env.hip.tcpxuDeviceCount(ctypes.byref(m)), "tcpxuDeviceCount")
    assert n.value == m.value >= 1


def test_native_driver_full_size(env, oracle):
    """The request loop inside the library (tcpxSynthRunRequests) on the 8 MiB chunk and the small-message storm."""
    torch = env.torch
    for config in (2, 3):
        wl = env.pkg.Workload(config, seed=0xC0FFEE00 + config)
        info = wl.info
        pool = np.empty(info.pool_bytes, dtype=np.uint8)
        wl.fill_window(0, pool)
        upload(env, pool)
        expect = np.full(GUARD + info.dst_bytes + GUARD, SENTINEL, dtype=np.uint8)
        graft.oracle_unpack(oracle, expect[GUARD : GUARD + info.dst_bytes], pool, np.ascontiguousarray(wl.descs))
        dst = torch.full((GUARD + info.dst_bytes + GUARD,), SENTINEL, dtype=torch.uint8, device="cuda:0")
        torch.cuda.synchronize()
        comm = env.driver.RecvComm(0)
        print("native plugin case: config %d, %d requests" % (config, info.n_requests), flush=True)
        seconds, lat = env.driver.run_workload_native(comm, wl, dst.data_ptr() + GUARD, window=8)
        got = dst.cpu().numpy()
        assert comm.outstanding_pages() == 0 and len(lat) == info.n_requests
        comm.close()
        assert first_difference(got, expect) is None, "first (index, got, want, count): %r" % (first_difference(got, expect),)


class WithEmptyRequests:
    """A workload with zero-size requests put between its own: (requests, frags, info) as run_workload reads them."""

    def __init__(self, wl, at):
        reqs = list(wl.requests)
        for k in sorted(at, reverse=True):
            empty = np.zeros(1, dtype=wl.requests.dtype)[0]
            empty["first_desc"] = reqs[k]["first_desc"] if k < len(reqs) else 0
            empty["dst_off"] = reqs[k]["dst_off"] if k < len(reqs) else 0
            reqs.insert(k, empty)
        self.requests = np.array(reqs, dtype=wl.requests.dtype)
        self.frags, self.info = wl.frags, wl.info


def test_zero_size_messages_and_iflush_between_real_requests(env, oracle):
    """irecv -> test* -> iflush -> irecvConsumed on the real engine, with the empty message (a TCPX_CTRL_INLINE
    control message: it takes a slot, publishes a count of 0 and is consumed through the fast path,
    src/net_tcpx.cc:1248-1276,1361,1500-1504) at the start, in the middle and at the end of a run of 64 KiB
    requests.  iflush answers each request's size and does no work (src/net_tcpx.cc:946-954); run_workload checks
    the answer for every request, this test checks bytes, slots and pages."""
    torch = env.torch
    wl = env.pkg.Workload(3, seed=0xF1A5, shrink=5)  # 64 requests of 16 x 4 KiB
    info = wl.info
    pool = np.empty(info.pool_bytes, dtype=np.uint8)
    wl.fill_window(0, pool)
    upload(env, pool)
    expect = np.full(GUARD + info.dst_bytes + GUARD, SENTINEL, dtype=np.uint8)
    graft.oracle_unpack(oracle, expect[GUARD : GUARD + info.dst_bytes], pool, np.ascontiguousarray(wl.descs))
    dst = torch.full((GUARD + info.dst_bytes + GUARD,), SENTINEL, dtype=torch.uint8, device="cuda:0")
    torch.cuda.synchronize()
    mixed = WithEmptyRequests(wl, at=[0, 7, 7, 20, 33, info.n_requests])
    n_all = len(mixed.requests)
    assert n_all == info.n_requests + 6 and sum(int(r["bytes"]) == 0 for r in mixed.requests) == 6
    comm = env.driver.RecvComm(0)
    print("plugin case: %d requests, 6 of them empty" % n_all, flush=True)
    for window in (1, 8):
        env.driver.run_workload(comm, mixed, dst.data_ptr() + GUARD, n_flows=4, window=window, timeout_s=30)
    got = dst.cpu().numpy()
    assert comm.outstanding_pages() == 0
    head, tail, idx = comm.queue_state()
    assert head == tail == 2 * n_all and len(set(idx)) == 1  # an empty message takes a slot like any other
    stats = env.pkg.CommStats()
    assert env.lib.tcpxGetCommStats(comm.comm, ctypes.byref(stats)) == 0
    assert stats.unpack_cnt == 2 * info.n_requests  # only requests with payload go to the GPU
    # n != 1 is an error, and a flush never creates a request of its own (src/net_tcpx.cc:949-953)
    one = (ctypes.c_void_p * 1)(dst.data_ptr())
    sizes = (ctypes.c_int * 1)(-5)
    none = (ctypes.c_void_p * 1)(None)
    assert env.lib.tcpxIflush_v5(comm.comm, 2, one, sizes, none, none) == 3
    assert env.lib.tcpxIflush_v5(comm.comm, 1, one, sizes, none, none) == 0 and sizes[0] == -5 and not none[0]
    comm.close()
    assert first_difference(got, expect) is None, "first (index, got, want, count): %r" % (first_difference(got, expect),)
