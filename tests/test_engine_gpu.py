"""GPU parity of the persistent unpack engine against the CPU oracle, byte-exact, through the C-ABI.

Descriptors and completion words live in hipHostMalloc-mapped memory; the destination is read back while the
engine kernel is still running wherever the test says so, which is what a real consumer does.
Every wait in this file has a deadline, so a stuck engine fails a test instead of hanging the run.
"""
import ctypes
import time

import numpy as np
import pytest

from conftest import GUARD, SENTINEL, GpuBuffers, first_difference, make_descs, oracle_expected

pytestmark = pytest.mark.gpu


class Mapped:
    """A block of mapped host memory: [0, 8*n_flags) completion words, then descriptors."""

    def __init__(self, pkg, hip, descs, n_flags):
        self.pkg, self.hip = pkg, hip
        self.flag_bytes = (8 * n_flags + 63) // 64 * 64
        self.host, self.dev = ctypes.c_void_p(), ctypes.c_void_p()
        nbytes = self.flag_bytes + max(descs.nbytes, 16)
        pkg.check(hip.tcpxuMappedAlloc(0, nbytes, ctypes.byref(self.host), ctypes.byref(self.dev)), "tcpxuMappedAlloc")
        if descs.nbytes:
            ctypes.memmove(self.host.value + self.flag_bytes, descs.ctypes.data, descs.nbytes)
        self.flags = (ctypes.c_uint64 * n_flags).from_address(self.host.value)

    def desc_dev(self, index):
        return self.dev.value + self.flag_bytes + 16 * index

    def flag_dev(self, i):
        return self.dev.value + 8 * i

    def wait(self, i, value, seconds=20.0):
        deadline = time.time() + seconds
        while self.flags[i] != value:
            if time.time() > deadline:
                raise TimeoutError("completion word %d did not reach %d (is %d)" % (i, value, self.flags[i]))

    def free(self):
        self.pkg.check(self.hip.tcpxuMappedFree(0, self.host), "tcpxuMappedFree")


class Engine:
    def __init__(self, pkg, hip, **cfg):
        self.pkg, self.hip = pkg, hip
        self.h = ctypes.c_void_p()
        c = pkg.EngineConfig(
            cfg.get("ring_entries", 0), cfg.get("workgroups", 0), cfg.get("descs_per_ticket", 0), cfg.get("spin_limit", 0)
        )
        pkg.check(hip.tcpxuEngineCreate(0, ctypes.byref(c), ctypes.byref(self.h)), "tcpxuEngineCreate")
        self.started = False

    def start(self):
        self.pkg.check(self.hip.tcpxuEngineStart(self.h), "tcpxuEngineStart")
        self.started = True

    def stop(self):
        us = ctypes.c_double()
        self.started = False
        self.pkg.check(self.hip.tcpxuEngineStop(self.h, ctypes.byref(us)), "tcpxuEngineStop")
        return us.value

    def submit(self, bounce, dst, descs_dev, n, flag_dev, value, seconds=20.0):
        deadline = time.time() + seconds
        while True:
            rc = self.hip.tcpxuEngineSubmit(self.h, bounce, dst, descs_dev, n, flag_dev, value)
            if rc != self.pkg.IN_PROGRESS:
                self.pkg.check(rc, "tcpxuEngineSubmit")
                return
            if time.time() > deadline:
                raise TimeoutError("submission ring stayed full")

    def completed(self):
        c = ctypes.c_uint64()
        self.pkg.check(self.hip.tcpxuEngineCompleted(self.h, ctypes.byref(c)), "tcpxuEngineCompleted")
        return c.value

    def running(self):
        r = ctypes.c_int()
        self.pkg.check(self.hip.tcpxuEngineRunning(self.h, ctypes.byref(r)), "tcpxuEngineRunning")
        return bool(r.value)

    def destroy(self):
        if self.started:
            self.stop()
        self.pkg.check(self.hip.tcpxuEngineDestroy(self.h), "tcpxuEngineDestroy")


def run_requests(pkg, hip, oracle, wl, read_back_while_running, **cfg):
    """One submission per request of the workload; returns nothing, asserts byte equality with the oracle."""
    info = wl.info
    pool = np.empty(info.pool_bytes, dtype=np.uint8)
    wl.fill_window(0, pool)
    expect = oracle_expected(oracle, pool, wl.descs, info.dst_bytes, info.dst_misalign)
    g = GpuBuffers(pool, wl.descs, info.dst_bytes, info.dst_misalign)
    m = Mapped(pkg, hip, np.ascontiguousarray(wl.descs), len(wl.requests))
    e = Engine(pkg, hip, **cfg)
    print("engine case: config=%d shrink=%d requests=%d cfg=%r" % (wl.config, wl.shrink, len(wl.requests), cfg), flush=True)
    e.start()
    try:
        for i, r in enumerate(wl.requests):
            e.submit(g.pool.data_ptr(), g.dst_base, m.desc_dev(int(r["first_desc"])), int(r["n_descs"]), m.flag_dev(i), i + 1)
        for i in range(len(wl.requests)):
            m.wait(i, i + 1)
        if read_back_while_running:
            got = g.result()
    finally:
        e.stop()
    if not read_back_while_running:
        got = g.result()
    assert e.completed() == len(wl.requests)
    e.destroy()
    m.free()
    assert first_difference(got, expect) is None, "first (index, got, want, count): %r" % (first_difference(got, expect),)


def test_engine_smallest(pkg, hip, oracle):
    """One submission, read back after the engine has stopped."""
    wl = pkg.Workload(1, seed=11, shrink=4)
    run_requests(pkg, hip, oracle, wl, read_back_while_running=False)


@pytest.mark.parametrize("config", [1, 2, 3, 4, 5])
def test_engine_workloads_reduced(pkg, hip, oracle, config):
    wl = pkg.Workload(config, seed=0xC0FFEE00 + config, shrink=3)
    run_requests(pkg, hip, oracle, wl, read_back_while_running=True)


@pytest.mark.parametrize("config", [2, 4])
def test_engine_workloads_full_size(pkg, hip, oracle, config):
    wl = pkg.Workload(config, seed=0xC0FFEE00 + config, shrink=0)
    run_requests(pkg, hip, oracle, wl, read_back_while_running=True)


@pytest.mark.parametrize("per_ticket", [1, 4, 14, 16, 64])
def test_engine_ticket_sizes(pkg, hip, oracle, per_ticket):
    wl = pkg.Workload(5, seed=5, shrink=3)
    run_requests(pkg, hip, oracle, wl, read_back_while_running=True, descs_per_ticket=per_ticket)


def test_engine_small_ring_backpressure(pkg, hip, oracle):
    """More submissions than ring entries: submit reports 'in progress' and later succeeds."""
    wl = pkg.Workload(3, seed=6, shrink=3)  # 256 requests
    run_requests(pkg, hip, oracle, wl, read_back_while_running=True, ring_entries=16)


def test_engine_restart_and_empty_submission(pkg, hip, oracle):
    pool = np.random.default_rng(7).integers(0, 256, size=1 << 20, dtype=np.uint8)
    rows = [((i * 4096 + 5) % (1 << 20 - 1), 4000 + i % 90, i * 4096 + 9) for i in range(100)]
    descs = make_descs(rows)
    expect = oracle_expected(oracle, pool, descs, 100 * 4096 + 4096)
    g = GpuBuffers(pool, descs, 100 * 4096 + 4096)
    m = Mapped(pkg, hip, descs, 4)
    e = Engine(pkg, hip, spin_limit=0xFFFFFFFF)  # never leaves by itself: running() is then deterministic
    for round_ in range(3):
        g.reset()
        for f in range(4):
            m.flags[f] = 0
        e.start()
        assert e.running()
        e.submit(g.pool.data_ptr(), g.dst_base, m.desc_dev(0), 50, m.flag_dev(0), 100 + round_)
        e.submit(None, None, None, 0, m.flag_dev(1), 200 + round_)  # zero descriptors: completes at once
        e.submit(g.pool.data_ptr(), g.dst_base, m.desc_dev(50), 50, m.flag_dev(2), 300 + round_)
        m.wait(0, 100 + round_)
        m.wait(1, 200 + round_)
        m.wait(2, 300 + round_)
        us = e.stop()
        assert not e.running()
        assert us > 0
        assert e.completed() == 3 * (round_ + 1)
        got = g.result()
        assert first_difference(got, expect) is None, repr(first_difference(got, expect))
    e.destroy()
    m.free()


def test_engine_submissions_queued_while_stopped(pkg, hip, oracle):
    """Submissions made before the kernel is launched are picked up when it starts."""
    pool = np.random.default_rng(8).integers(0, 256, size=1 << 18, dtype=np.uint8)
    descs = make_descs([(i * 1000, 999, i * 1000) for i in range(200)])
    expect = oracle_expected(oracle, pool, descs, 200 * 1000)
    g = GpuBuffers(pool, descs, 200 * 1000)
    m = Mapped(pkg, hip, descs, 2)
    e = Engine(pkg, hip)
    e.submit(g.pool.data_ptr(), g.dst_base, m.desc_dev(0), 120, m.flag_dev(0), 1)
    e.submit(g.pool.data_ptr(), g.dst_base, m.desc_dev(120), 80, m.flag_dev(1), 2)
    e.start()
    m.wait(0, 1)
    m.wait(1, 2)
    e.stop()
    got = g.result()
    e.destroy()
    m.free()
    assert first_difference(got, expect) is None


def test_engine_spin_limit_exits_by_itself(pkg, hip):
    """Bounded wait: with a spin limit the kernel leaves on its own when nothing is submitted."""
    e = Engine(pkg, hip, spin_limit=2000)
    e.start()
    deadline = time.time() + 20
    while e.running():
        assert time.time() < deadline, "engine with a spin limit is still running"
        time.sleep(0.01)
    e.stop()  # reaps the finished launch
    e.destroy()


def test_engine_leaves_when_idle_and_returns_on_submit(pkg, hip, oracle):
    """Default configuration: the kernel leaves after about half a millisecond without work, so a device-wide
    synchronize returns, and the next submission brings it back without any call besides submit."""
    import torch

    pool = np.random.default_rng(9).integers(0, 256, size=1 << 20, dtype=np.uint8)
    descs = make_descs([(i * 4096 + 3, 4000, i * 4000) for i in range(128)])
    expect = oracle_expected(oracle, pool, descs, 128 * 4000)
    g = GpuBuffers(pool, descs, 128 * 4000)
    m = Mapped(pkg, hip, descs, 8)
    e = Engine(pkg, hip)
    e.start()
    for round_ in range(4):
        g.reset()  # contains a device-wide synchronize: returns only because the idle kernel has left
        deadline = time.time() + 20
        while e.running():
            assert time.time() < deadline
            time.sleep(0.001)
        e.submit(g.pool.data_ptr(), g.dst_base, m.desc_dev(0), 64, m.flag_dev(2 * round_), 1)
        e.submit(g.pool.data_ptr(), g.dst_base, m.desc_dev(64), 64, m.flag_dev(2 * round_ + 1), 1)
        m.wait(2 * round_, 1)
        m.wait(2 * round_ + 1, 1)
        torch.cuda.synchronize()
        assert first_difference(g.result(), expect) is None
    e.stop()
    assert e.completed() == 8
    e.destroy()
    m.free()


def test_engine_argument_errors(pkg, hip):
    e = Engine(pkg, hip)
    flag = ctypes.c_void_p(0x1000)
    assert hip.tcpxuEngineSubmit(e.h, None, None, None, 0, None, 1) == pkg.INVALID_ARGUMENT
    assert hip.tcpxuEngineSubmit(e.h, None, None, None, 0, flag, 0) == pkg.INVALID_ARGUMENT
    assert hip.tcpxuEngineSubmit(e.h, None, None, None, 4, flag, 1) == pkg.INVALID_ARGUMENT
    assert hip.tcpxuEngineStop(e.h, None) == pkg.INVALID_USAGE
    bad = pkg.EngineConfig(1000, 0, 0, 0)
    h = ctypes.c_void_p()
    assert hip.tcpxuEngineCreate(0, ctypes.byref(bad), ctypes.byref(h)) == pkg.INVALID_ARGUMENT
    bad = pkg.EngineConfig(0, 0, 65, 0)
    assert hip.tcpxuEngineCreate(0, ctypes.byref(bad), ctypes.byref(h)) == pkg.INVALID_ARGUMENT
    e.destroy()


@pytest.mark.parametrize("depth", [1, 5, 16, 64, 128])
def test_engine_stream_depths(pkg, hip, oracle, depth, benchlib):
    """The streaming driver (mapped slot ring, warm-up + timed items in one launch) at 1 to 64 slots in flight:
    the leader then cuts tickets of 8 to 16 descriptors by backlog, and every size must give the oracle's bytes.
    Eight distinct 8 MiB chunks, each twice, so every destination is written by two passes of the ring."""
    import torch

    chunks = [pkg.Workload(2, seed=0xBEEF00 + 31 * c) for c in range(8)]
    info0 = chunks[0].info
    cb = info0.payload_bytes
    pool = np.empty(info0.pool_bytes, dtype=np.uint8)
    chunks[0].fill_window(0, pool)  # one pool for all chunks: the oracle and the GPU read the same bytes
    expect = np.full(GUARD + len(chunks) * cb + GUARD, SENTINEL, dtype=np.uint8)
    keep, flat = [], []
    for c, wl in enumerate(chunks):
        assert wl.info.pool_bytes == info0.pool_bytes and wl.info.payload_bytes == cb
        lo = GUARD + c * cb
        expect[lo : lo + cb] = oracle_expected(oracle, pool, wl.descs, cb, 0)[GUARD : GUARD + cb]
    pool_d = torch.from_numpy(pool).to("cuda:0")
    dst_d = torch.full((expect.nbytes,), SENTINEL, dtype=torch.uint8, device="cuda:0")
    torch.cuda.synchronize()
    for rep in range(2):
        for c, wl in enumerate(chunks):
            for r in wl.requests:
                d = np.ascontiguousarray(wl.descs[int(r["first_desc"]) : int(r["first_desc"]) + int(r["n_descs"])])
                keep.append(d)
                flat.append((pool_d.data_ptr(), dst_d.data_ptr() + GUARD + c * cb, d.ctypes.data, len(d)))
    items = (pkg.StreamItem * len(flat))()
    for i, (b, d, p, n) in enumerate(flat):
        items[i].bounce_base, items[i].dst_base, items[i].descs_host, items[i].n_descs = b, d, p, n
    e = Engine(pkg, hip)
    print("engine stream case: depth=%d items=%d" % (depth, len(flat)), flush=True)
    wall, kern = ctypes.c_double(), ctypes.c_double()
    lat = (ctypes.c_double * len(flat))()
    rc = benchlib.tcpxuEngineRunTimed(e.h, items, len(flat), 4, depth, 20000, ctypes.byref(wall), ctypes.byref(kern), lat)
    pkg.check(rc, "tcpxuEngineRunTimed")
    assert e.completed() == len(flat) and 0 < wall.value <= kern.value * 1.5 and min(lat) > 0
    e.destroy()
    got = dst_d.cpu().numpy()
    assert first_difference(got, expect) is None, "first (index, got, want, count): %r" % (first_difference(got, expect),)
    # beyond 128 slots in flight a slot holds 64 descriptors, and more than TCPXU_STREAM_MAX_DEPTH slots there are not:
    # both refused before anything is launched
    e = Engine(pkg, hip)
    assert benchlib.tcpxuEngineRunTimed(e.h, items, 4, 0, 129, 1000, ctypes.byref(wall), ctypes.byref(kern), None) == pkg.INVALID_ARGUMENT
    assert benchlib.tcpxuEngineRunTimed(e.h, items, 4, 0, 2049, 1000, ctypes.byref(wall), ctypes.byref(kern), None) == pkg.INVALID_ARGUMENT
    e.destroy()


@pytest.mark.parametrize(
    "depth,per_ticket,ring",
    [(256, 0, 0), (2048, 0, 0), (2048, 16, 0), (1024, 8, 0), (256, 0, 512)],
    ids=["256", "2048", "2048-tickets-of-16", "1024-two-tickets-each", "256-ring-of-512"],
)
def test_engine_storm_of_small_requests_many_in_flight(pkg, hip, oracle, depth, per_ticket, ring, benchlib):
    """The small-message storm with hundreds to 2048 requests in flight (the unpack queues of 128 comms): the
    leader then fetches 64 submission entries per poll and turns runs of sixteen into tickets at a stroke -- with
    hundreds published ahead of it, in its rolling loop -- and the host publishes in batches.  Also with the ticket
    size fixed at the requests' sixteen descriptors (one ticket each, as when sized by the backlog) and at eight (two
    tickets each: none of this applies, the ordinary way with a thousand waiting), and with a submission ring of 512
    entries, the smallest that the rolling loop takes, wrapped every 512 requests.  Every request twice, byte-exact;
    every submission consumed by exactly one poll."""
    import torch

    wl = pkg.Workload(3, seed=0x5708A + depth + per_ticket + ring, shrink=1)  # 1024 requests of 16 x 4 KiB, 256 MiB pool
    info = wl.info
    pool = np.empty(info.pool_bytes, dtype=np.uint8)
    wl.fill_window(0, pool)
    expect = oracle_expected(oracle, pool, wl.descs, int(info.dst_bytes))
    pool_d = torch.from_numpy(pool).to("cuda:0")
    dst_d = torch.full((expect.nbytes,), SENTINEL, dtype=torch.uint8, device="cuda:0")
    torch.cuda.synchronize()
    descs = np.array(wl.descs, copy=True)
    reqs = wl.requests
    n = len(reqs)
    items = (pkg.StreamItem * (2 * n))()
    for i in range(2 * n):
        r = reqs[i % n]
        first, cnt = int(r["first_desc"]), int(r["n_descs"])
        items[i].bounce_base = pool_d.data_ptr()
        items[i].dst_base = dst_d.data_ptr() + GUARD  # descriptor offsets count from the start of the message
        items[i].descs_host = descs.ctypes.data + 16 * first
        items[i].n_descs = cnt
        items[i].payload_bytes = int(r["bytes"])
    e = Engine(pkg, hip, descs_per_ticket=per_ticket, ring_entries=ring)
    print("engine storm case: depth=%d tickets of %d ring %d items=%d" % (depth, per_ticket, ring, 2 * n), flush=True)
    wall, kern = ctypes.c_double(), ctypes.c_double()
    lat = (ctypes.c_double * (2 * n))()
    pkg.check(benchlib.tcpxuEngineRunTimed(e.h, items, 2 * n, 0, depth, 20000, ctypes.byref(wall), ctypes.byref(kern), lat), "tcpxuEngineRunTimed")
    stats, split = pkg.EngineStats(), pkg.StreamSplit()
    pkg.check(hip.tcpxuEngineGetStats(e.h, ctypes.byref(stats)), "tcpxuEngineGetStats")
    pkg.check(benchlib.tcpxuStreamLastSplit(ctypes.byref(split)), "tcpxuStreamLastSplit")
    print("engine storm case: %.2f M requests/s, %d polls of which %d fetched 64 entries, %.0f ns of host time per publish"
          % (2 * n / wall.value, stats.leader_polls, stats.leader_deep_polls, split.publish_ns / split.published), flush=True)  # fmt: skip
    assert e.completed() == 2 * n and min(lat) > 0
    assert stats.submissions == stats.leader_entries == 2 * n and stats.launches == 1
    assert 0 < stats.leader_polls and stats.leader_deep_polls <= stats.leader_polls
    assert split.published == 2 * n and split.publish_calls <= split.published and split.publish_ns < split.wall_ns
    e.destroy()
    got = dst_d.cpu().numpy()
    assert first_difference(got, expect) is None, "first (index, got, want, count): %r" % (first_difference(got, expect),)


def test_engine_submit_many(pkg, hip, oracle):
    """tcpxuEngineSubmitMany: all submissions checked before any is queued; what the ring takes goes in under one
    publish, in order, and the count comes back with "in progress" when that is not all."""
    pool = np.random.default_rng(41).integers(0, 256, size=1 << 20, dtype=np.uint8)
    rows = [((i * 4096 + 7 * i) % ((1 << 20) - 4096), 1 + (i * 997) % 4096, i * 4096) for i in range(160)]
    descs = make_descs(rows)
    expect = oracle_expected(oracle, pool, descs, 160 * 4096)
    g = GpuBuffers(pool, descs, 160 * 4096)
    m = Mapped(pkg, hip, descs, 40)
    e = Engine(pkg, hip, ring_entries=16)
    subs = (pkg.Submission * 40)()
    for i in range(40):  # 40 submissions of 4 descriptors each
        subs[i] = pkg.Submission(g.pool.data_ptr(), g.dst_base, m.desc_dev(4 * i), m.flag_dev(i), i + 1, 4, 0)
    accepted = ctypes.c_uint32(99)
    # one bad submission (no completion word) among good ones: nothing is queued
    good = subs[3].done_flag_dev
    subs[3].done_flag_dev = None
    assert hip.tcpxuEngineSubmitMany(e.h, subs, 40, ctypes.byref(accepted)) == pkg.INVALID_ARGUMENT and accepted.value == 0
    subs[3].done_flag_dev = good
    assert hip.tcpxuEngineSubmitMany(e.h, subs, 0, ctypes.byref(accepted)) == pkg.SUCCESS and accepted.value == 0
    # the engine is not started: a ring of 16 takes the first 16 and says so
    assert hip.tcpxuEngineSubmitMany(e.h, subs, 40, ctypes.byref(accepted)) == pkg.IN_PROGRESS and accepted.value == 16
    assert hip.tcpxuEngineSubmitMany(e.h, ctypes.byref(subs[16]), 24, ctypes.byref(accepted)) == pkg.IN_PROGRESS and accepted.value == 0
    e.start()
    at = 16
    deadline = time.time() + 20
    while at < 40:
        rc = hip.tcpxuEngineSubmitMany(e.h, ctypes.byref(subs[at]), 40 - at, ctypes.byref(accepted))
        assert rc in (pkg.SUCCESS, pkg.IN_PROGRESS), pkg.hip_layer().tcpxuLastError()
        at += accepted.value
        assert (rc == pkg.SUCCESS) == (at == 40)
        assert time.time() < deadline, "the submission ring stayed full"
    for i in range(40):
        m.wait(i, i + 1)
    e.stop()
    stats = pkg.EngineStats()
    pkg.check(hip.tcpxuEngineGetStats(e.h, ctypes.byref(stats)), "tcpxuEngineGetStats")
    assert stats.submissions == stats.leader_entries == 40 and e.completed() == 40
    got = g.result()
    e.destroy()
    m.free()
    assert first_difference(got, expect) is None, repr(first_difference(got, expect))


@pytest.mark.parametrize("hint", ["true", "none", "tiny", "huge"])
def test_engine_ticket_size_follows_the_payload_hint(pkg, hip, oracle, hint, benchlib):
    """Ragged and empty fragments (the adversarial workload, 2 KiB a fragment on average) with 64 slots in flight:
    with the request's byte count given, the leader cuts tickets of up to 64 descriptors, without it tickets of
    16; a hint is only a hint, so a wrong one (far too small, far too large) must give the same bytes."""
    import torch

    wl = pkg.Workload(5, seed=0xAD5E12)
    info = wl.info
    pool = np.empty(info.pool_bytes, dtype=np.uint8)
    wl.fill_window(0, pool)
    size = int(info.dst_bytes) + int(info.dst_misalign)
    passes = 6
    stride = (size + 4095) // 4096 * 4096
    expect = np.full(GUARD + passes * stride + GUARD, SENTINEL, dtype=np.uint8)
    one = oracle_expected(oracle, pool, wl.descs, int(info.dst_bytes), int(info.dst_misalign))
    for ps in range(passes):
        lo = GUARD + ps * stride
        expect[lo : lo + size] = one[GUARD : GUARD + size]
    pool_d = torch.from_numpy(pool).to("cuda:0")
    dst_d = torch.full((expect.nbytes,), SENTINEL, dtype=torch.uint8, device="cuda:0")
    torch.cuda.synchronize()
    descs = np.ascontiguousarray(wl.descs)
    reqs = [(int(r["first_desc"]), int(r["n_descs"])) for r in wl.requests]
    items = (pkg.StreamItem * (passes * len(reqs)))()
    i = 0
    for ps in range(passes):
        for first, n in reqs:
            nbytes = int(descs["len"][first : first + n].sum())
            items[i].bounce_base = pool_d.data_ptr()
            items[i].dst_base = dst_d.data_ptr() + GUARD + ps * stride + int(info.dst_misalign)
            items[i].descs_host = descs.ctypes.data + 16 * first
            items[i].n_descs = n
            items[i].payload_bytes = {"true": nbytes, "none": 0, "tiny": 1, "huge": 0xFFFFFFFF}[hint]
            i += 1
    e = Engine(pkg, hip)
    print("engine hint case: %s, %d items" % (hint, len(items)), flush=True)
    wall, kern = ctypes.c_double(), ctypes.c_double()
    rc = benchlib.tcpxuEngineRunTimed(e.h, items, len(items), 0, 64, 20000, ctypes.byref(wall), ctypes.byref(kern), None)
    pkg.check(rc, "tcpxuEngineRunTimed")
    assert e.completed() == len(items)
    e.destroy()
    got = dst_d.cpu().numpy()
    assert first_difference(got, expect) is None, "first (index, got, want, count): %r" % (first_difference(got, expect),)


def test_engine_bursts_around_the_idle_exit(pkg, hip, oracle):
    """Three host threads submit in bursts separated by pauses of about the engine's idle limit (set to some
    60 us here), so that submissions keep meeting a kernel that is leaving, has left, or is coming back.  Every
    request must complete and every byte must match; seeded, a few hundred relaunches in a couple of seconds."""
    import threading

    wl = pkg.Workload(3, seed=0x51DE, shrink=3)  # 256 requests of 16 x 4 KiB
    info = wl.info
    pool = np.empty(info.pool_bytes, dtype=np.uint8)
    wl.fill_window(0, pool)
    expect = oracle_expected(oracle, pool, wl.descs, info.dst_bytes, info.dst_misalign)
    g = GpuBuffers(pool, wl.descs, info.dst_bytes, info.dst_misalign)
    n = len(wl.requests)
    m = Mapped(pkg, hip, np.ascontiguousarray(wl.descs), n)
    e = Engine(pkg, hip, spin_limit=40)
    e.start()
    errors = []

    def worker(k):
        rng = np.random.default_rng(100 + k)
        try:
            mine = list(range(k, n, 3))
            i = 0
            while i < len(mine):
                burst = int(rng.integers(1, 5))
                batch = mine[i : i + burst]
                for r in batch:
                    req = wl.requests[r]
                    e.submit(g.pool.data_ptr(), g.dst_base, m.desc_dev(int(req["first_desc"])), int(req["n_descs"]), m.flag_dev(r), r + 1)
                for r in batch:
                    m.wait(r, r + 1, seconds=30.0)
                i += burst
                time.sleep(float(rng.uniform(0, 150e-6)))
        except Exception as exc:  # reported by the main thread
            errors.append(repr(exc))

    threads = [threading.Thread(target=worker, args=(k,)) for k in range(3)]
    print("engine burst case: %d requests, 3 threads" % n, flush=True)
    for t in threads:
        t.start()
    away = 0  # times the main thread found the kernel gone while the others were submitting
    deadline = time.time() + 120
    while any(t.is_alive() for t in threads) and time.time() < deadline:
        away += 0 if e.running() else 1
        time.sleep(50e-6)
    for t in threads:
        t.join(timeout=5)
    assert not any(t.is_alive() for t in threads) and not errors, errors
    # How often the poll above saw the kernel gone depends on how the host schedules four threads: reported, not
    # asserted.  That an idle kernel leaves and a submission brings it back is asserted, without any timing, by
    # test_engine_leaves_when_idle_and_returns_on_submit.
    print("engine burst case: kernel found away %d times" % away, flush=True)
    got = g.result()
    e.stop()
    assert e.completed() == n
    e.destroy()
    m.free()
    assert first_difference(got, expect) is None, "first (index, got, want, count): %r" % (first_difference(got, expect),)


STORM_SIZES = [0, 1, 2, 7, 8, 9, 15, 16, 17, 31, 32, 33, 40, 64, 65, 300]
STORM_MIXED = [.05, .1, .05, .05, .1, .05, .05, .2, .05, .05, .1, .03, .03, .03, .03, .03]
# Nearly all of one ticket, so that hundreds in a row are: one in 250 is empty, just over a ticket, or of two.
STORM_MOSTLY_ONE_TICKET = [.001, .1, .05, .05, .1, .05, .05, .3, .05, .05, .196, .001, .001, .001, 0, 0]


# Mostly just over one ticket of the usual size and up to what one ticket can hold (33, 40, 64 descriptors), some of one
# ticket anyway, a few empty.
STORM_UP_TO_64 = [.005, .02, 0, 0, .05, 0, 0, .1, 0, 0, .1, .25, .25, .225, 0, 0]


def storm_workload(pkg, oracle, seed, n_submissions=3000, p=STORM_MIXED):
    """Submissions of 0 to 300 ragged fragments in random order, each owning a stretch of one destination buffer:
    (pool on the device, sentinel-filled destination on the device, stream items, expected bytes, descriptor count)."""
    import torch

    rng = np.random.default_rng(seed)
    pool = np.random.default_rng(0xD00D).integers(0, 256, size=8 << 20, dtype=np.uint8)
    sizes = rng.choice(STORM_SIZES, size=n_submissions, p=p)
    rows, subs, dst_off = [], [], 0
    for n in sizes:
        first = len(rows)
        base = dst_off
        for _ in range(int(n)):
            ln = int(rng.integers(1, 4097)) if rng.random() < 0.5 else 4096
            page = int(rng.integers(0, len(pool) >> 12))
            so = (page << 12) + int(rng.integers(0, 4096 - ln + 1))
            rows.append((so, ln, dst_off - base))
            dst_off += ln
        subs.append((first, int(n), base))
        dst_off += int(rng.integers(0, 40))  # a gap that must keep the sentinel
    descs = make_descs(rows)
    total = dst_off + 64
    expect = np.full(GUARD + total + GUARD, SENTINEL, dtype=np.uint8)
    absolute = descs.copy()
    for first, n, base in subs:
        absolute["dst_off"][first : first + n] += base
    expect[:] = oracle_expected(oracle, pool, absolute, total, 0)
    pool_d = torch.from_numpy(pool).to("cuda:0")
    dst_d = torch.full((expect.nbytes,), SENTINEL, dtype=torch.uint8, device="cuda:0")
    torch.cuda.synchronize()
    items = (pkg.StreamItem * len(subs))()
    for i, (first, n, base) in enumerate(subs):
        items[i].bounce_base = pool_d.data_ptr()
        items[i].dst_base = dst_d.data_ptr() + GUARD + base
        items[i].descs_host = descs.ctypes.data + 16 * first
        items[i].n_descs = n
    return pool_d, dst_d, items, expect, descs


@pytest.mark.parametrize("depth", [3, 16, 128])
def test_engine_storm_of_mixed_small_submissions(pkg, hip, oracle, depth, benchlib):
    """Thousands of submissions of 0 to 300 ragged fragments in random order, `depth` of them in flight: runs of
    submissions that the leader turns into tickets sixteen at a time are broken at every position by empty ones,
    by ones just over the one-ticket limit and by ones that need many tickets; each submission owns a stretch of
    the destination and every byte must be the oracle's."""
    pool_d, dst_d, items, expect, descs = storm_workload(pkg, oracle, 0x570A + depth)
    e = Engine(pkg, hip)
    print("engine storm case: depth=%d submissions=%d descriptors=%d" % (depth, len(items), len(descs)), flush=True)
    wall, kern = ctypes.c_double(), ctypes.c_double()
    lat = (ctypes.c_double * len(items))()
    pkg.check(benchlib.tcpxuEngineRunTimed(e.h, items, len(items), 0, depth, 20000, ctypes.byref(wall), ctypes.byref(kern), lat), "tcpxuEngineRunTimed")
    assert e.completed() == len(items) and min(lat) > 0
    e.destroy()
    got = dst_d.cpu().numpy()
    assert first_difference(got, expect) is None, "first (index, got, want, count): %r" % (first_difference(got, expect),)


@pytest.mark.parametrize("count_from,with_stamps", [(0, False), (0, True), ((1 << 32) - 70000, False)])
def test_engine_long_runs_of_one_ticket_submissions_broken_by_others(pkg, hip, oracle, benchlib, monkeypatch, count_from, with_stamps):
    """1024 in flight (a slot of the stream then holds up to 64 descriptors), nearly all of one ticket: with hundreds
    of entries published ahead of it the leader takes them in its rolling loop, four groups of sixteen in flight, and
    every few hundred entries an empty submission, one just over a ticket or one of two tickets ends that loop and
    goes the ordinary way.  Every byte must be the oracle's, every submission consumed exactly once -- also when the
    32-bit stamps of tickets and entries wrap in the middle of it (an engine that starts 70000 below 2^32: more than a
    lap of the ticket ring, because a ring slot that was never written reads as the stamp of sequence number 2^32-1),
    and with the kernel's clock stamps switched on (the rolling loop then issues one more store per group, which the
    count it waits by must survive; the four stamps of each of the last 2048 submissions must be there and in order)."""
    assert abs(sum(STORM_MOSTLY_ONE_TICKET) - 1) < 1e-9
    # (with stamps: fewer submissions than the ring has entries, so that no place in the ring is stamped twice)
    pool_d, dst_d, items, expect, descs = storm_workload(pkg, oracle, 0x5709 + (count_from & 0xFF), 4000 if with_stamps else 8000, STORM_MOSTLY_ONE_TICKET)
    if count_from:
        monkeypatch.setenv("TCPXU_ENGINE_COUNT_FROM", str(count_from))
    e = Engine(pkg, hip)
    monkeypatch.delenv("TCPXU_ENGINE_COUNT_FROM", raising=False)
    assert e.completed() == count_from
    rate = ctypes.c_double()
    if with_stamps:
        pkg.check(hip.tcpxuEngineEnableStamps(e.h, ctypes.byref(rate)), "tcpxuEngineEnableStamps")
    launches = 70000 // len(items) + 3 if count_from else 1
    print("engine rolling-loop case: count_from=%d launches=%d submissions each=%d descriptors=%d" % (count_from, launches, len(items), len(descs)), flush=True)  # fmt: skip
    wall, kern = ctypes.c_double(), ctypes.c_double()
    lat = (ctypes.c_double * len(items))()
    stats = pkg.EngineStats()
    for launch in range(launches):
        dst_d.fill_(SENTINEL)
        pkg.check(benchlib.tcpxuEngineRunTimed(e.h, items, len(items), 0, 1024, 20000, ctypes.byref(wall), ctypes.byref(kern), lat), "tcpxuEngineRunTimed")
        pkg.check(hip.tcpxuEngineGetStats(e.h, ctypes.byref(stats)), "tcpxuEngineGetStats")
        print("engine rolling-loop case: launch %d, %.2f M submissions/s, %d entries in %d polls of which %d of 64 so far"
              % (launch, len(items) / wall.value, stats.leader_entries, stats.leader_polls, stats.leader_deep_polls), flush=True)  # fmt: skip
        assert e.completed() == count_from + (launch + 1) * len(items) and min(lat) > 0
        assert stats.submissions == stats.leader_entries == (launch + 1) * len(items) and stats.launches >= launch + 1
        assert stats.leader_deep_polls <= stats.leader_polls
        got = dst_d.cpu().numpy()
        assert first_difference(got, expect) is None, "launch %d, first (index, got, want, count): %r" % (launch, first_difference(got, expect))
    assert not count_from or e.completed() > (1 << 32)
    if with_stamps:
        last = 2048
        out = (ctypes.c_uint64 * (4 * last))()
        pkg.check(hip.tcpxuEngineReadStamps(e.h, len(items) - last, last, out), "tcpxuEngineReadStamps")
        for i in range(last):
            t = [out[4 * i + k] for k in range(4)]
            if items[len(items) - last + i].n_descs == 0:
                continue  # completed by the leader itself: no workgroup ever stamps it
            # [0] is the leader's reading and the others a workgroup's, on another compute unit whose clock may differ by
            # a few ticks: a workgroup that was already looking for the ticket can have it within that.
            slack = 0.5 * rate.value
            assert 0xFFFFFFFFFFFFFFFF not in t and t[0] <= t[1] + slack and t[1] <= t[2] <= t[3], (len(items) - last + i, t)
            assert (t[3] - t[0]) / rate.value < 1e6, "microseconds, not a second"
    e.destroy()


@pytest.mark.parametrize("depth", [1024, 96])
def test_engine_deep_queue_of_submissions_of_up_to_64_fragments(pkg, hip, oracle, benchlib, depth):
    """Submissions of 33 to 64 ragged fragments need several tickets of the usual size.  With a thousand in flight the
    leader finds sixteen of them in a poll, asks its rolling loop, and that loop -- seeing more than a hundred
    entries published ahead -- makes one ticket of up to 64 descriptors of each; with 96 in flight the queue is never
    that deep, the loop hands back at once and is asked again only after longer and longer pauses.  Either way every
    byte must be the oracle's and every submission consumed exactly once."""
    assert abs(sum(STORM_UP_TO_64) - 1) < 1e-9
    pool_d, dst_d, items, expect, descs = storm_workload(pkg, oracle, 0x64D + depth, 6000, STORM_UP_TO_64)
    e = Engine(pkg, hip)
    print("engine deep-queue case: depth=%d submissions=%d descriptors=%d" % (depth, len(items), len(descs)), flush=True)
    wall, kern = ctypes.c_double(), ctypes.c_double()
    lat = (ctypes.c_double * len(items))()
    pkg.check(benchlib.tcpxuEngineRunTimed(e.h, items, len(items), 0, depth, 20000, ctypes.byref(wall), ctypes.byref(kern), lat), "tcpxuEngineRunTimed")
    stats = pkg.EngineStats()
    pkg.check(hip.tcpxuEngineGetStats(e.h, ctypes.byref(stats)), "tcpxuEngineGetStats")
    print("engine deep-queue case: %.2f M submissions/s, %d entries in %d polls of which %d of 64"
          % (len(items) / wall.value, stats.leader_entries, stats.leader_polls, stats.leader_deep_polls), flush=True)  # fmt: skip
    assert e.completed() == len(items) and min(lat) > 0
    assert stats.submissions == stats.leader_entries == len(items) and stats.leader_deep_polls <= stats.leader_polls
    if depth >= 1024:
        assert stats.leader_deep_polls > 0, "the rolling loop took part"
    e.destroy()
    got = dst_d.cpu().numpy()
    assert first_difference(got, expect) is None, "first (index, got, want, count): %r" % (first_difference(got, expect),)


def test_engine_sequence_numbers_cross_2_to_the_32(pkg, hip, oracle, benchlib, monkeypatch):
    """Submission entries and tickets are stamped with the low 32 bits of their sequence numbers, and the leader's
    ring arithmetic runs on low words: an engine that starts 70000 below 2^32 (TCPXU_ENGINE_COUNT_FROM) crosses it
    with its tickets first (after more than one lap of the ticket ring) and with its submissions later, under the
    storm of mixed submissions, launch after launch; every launch's bytes must be the oracle's."""
    start = (1 << 32) - 70000
    pool_d, dst_d, items, expect, descs = storm_workload(pkg, oracle, 0xC2055)
    monkeypatch.setenv("TCPXU_ENGINE_COUNT_FROM", str(start))
    e = Engine(pkg, hip)
    monkeypatch.delenv("TCPXU_ENGINE_COUNT_FROM")
    assert e.completed() == start
    launches = 70000 // len(items) + 4
    print("engine sequence case: start=%d launches=%d submissions each=%d" % (start, launches, len(items)), flush=True)
    wall, kern = ctypes.c_double(), ctypes.c_double()
    for launch in range(launches):
        dst_d.fill_(SENTINEL)
        pkg.check(benchlib.tcpxuEngineRunTimed(e.h, items, len(items), 0, 64, 20000, ctypes.byref(wall), ctypes.byref(kern), None), "tcpxuEngineRunTimed")
        assert e.completed() == start + (launch + 1) * len(items), launch
        got = dst_d.cpu().numpy()
        assert first_difference(got, expect) is None, "launch %d, first (index, got, want, count): %r" % (launch, first_difference(got, expect))
    assert e.completed() > (1 << 32)
    e.destroy()


def test_engine_run_window_times_the_middle_of_a_stream(pkg, hip, oracle, benchlib):
    """tcpxuEngineRunWindow: warm-up items, timed items and a tail in one launch; the clock covers the timed ones
    from completion to completion, so it is shorter than the launch, and every item's bytes are the oracle's."""
    import torch

    chunks = [pkg.Workload(2, seed=0xA11 + c, shrink=2) for c in range(4)]
    info0 = chunks[0].info
    cb = int(info0.dst_bytes)
    pool = np.empty(info0.pool_bytes, dtype=np.uint8)
    chunks[0].fill_window(0, pool)
    expect = np.full(GUARD + len(chunks) * cb + GUARD, SENTINEL, dtype=np.uint8)
    for c, wl in enumerate(chunks):
        expect[GUARD + c * cb : GUARD + (c + 1) * cb] = oracle_expected(oracle, pool, wl.descs, cb, 0)[GUARD : GUARD + cb]
    pool_d = torch.from_numpy(pool).to("cuda:0")
    dst_d = torch.full((expect.nbytes,), SENTINEL, dtype=torch.uint8, device="cuda:0")
    torch.cuda.synchronize()
    keep, flat = [], []
    for rep in range(3):
        for c, wl in enumerate(chunks):
            for r in wl.requests:
                d = np.ascontiguousarray(wl.descs[int(r["first_desc"]) : int(r["first_desc"]) + int(r["n_descs"])])
                keep.append(d)
                flat.append((pool_d.data_ptr(), dst_d.data_ptr() + GUARD + c * cb, d.ctypes.data, len(d)))
    items = (pkg.StreamItem * len(flat))()
    for i, (b, d, p, n) in enumerate(flat):
        items[i].bounce_base, items[i].dst_base, items[i].descs_host, items[i].n_descs = b, d, p, n
    n = len(flat)
    e = Engine(pkg, hip)
    print("engine window case: items=%d" % n, flush=True)
    wall, kern = ctypes.c_double(), ctypes.c_double()
    lat = (ctypes.c_double * n)()
    pkg.check(benchlib.tcpxuEngineRunWindow(e.h, items, n, n // 4, n // 2, 8, 20000, ctypes.byref(wall), ctypes.byref(kern), lat), "tcpxuEngineRunWindow")
    assert e.completed() == n and 0 < wall.value < kern.value and min(lat) > 0
    first = ctypes.c_double()
    pkg.check(benchlib.tcpxuEngineRunWindow(e.h, items, n, 0, n, 8, 20000, ctypes.byref(first), ctypes.byref(kern), None), "tcpxuEngineRunWindow")
    assert wall.value < first.value <= kern.value  # the whole stream takes longer than its middle half
    assert benchlib.tcpxuEngineRunWindow(e.h, items, n, n // 2, n, 8, 1000, ctypes.byref(wall), ctypes.byref(kern), None) == pkg.INVALID_ARGUMENT
    assert benchlib.tcpxuEngineRunWindow(e.h, items, n, 0, 0, 8, 1000, ctypes.byref(wall), ctypes.byref(kern), None) == pkg.INVALID_ARGUMENT
    e.destroy()
    got = dst_d.cpu().numpy()
    assert first_difference(got, expect) is None, "first (index, got, want, count): %r" % (first_difference(got, expect),)


def test_other_kernels_run_beside_the_engine(pkg, hip, oracle, benchlib):
    """The engine takes two workgroups of nine wavefronts per compute unit and leaves the rest of each to others:
    while it streams 64 slots of 4 MiB on its own stream, copy kernels launched on other streams must start and
    finish (each within a deadline), their bytes must be right, and the unpack must still be byte-exact.
    Four other streams carry the copies.  Each has run one copy before the engine starts: a stream's first launch
    sets up its hardware queue, and the kernel's first launch loads its code, both of which take milliseconds
    when the device is busy, as long as the whole engine launch measured here.  The runtime spreads a process's
    streams over a few hardware queues (four by default) and a queue starts its kernels in order, so a stream that
    shares the engine's queue gets its turn when the engine kernel leaves; the others must make progress beside
    it, which is what is asserted: copies finish on at least two of the four streams while the engine runs."""
    import threading

    import torch

    chunks = [pkg.Workload(2, seed=0xC0E5 + c) for c in range(4)]
    info0 = chunks[0].info
    cb = int(info0.dst_bytes)
    pool = np.empty(info0.pool_bytes, dtype=np.uint8)
    chunks[0].fill_window(0, pool)
    expect = np.full(GUARD + len(chunks) * cb + GUARD, SENTINEL, dtype=np.uint8)
    for c, wl in enumerate(chunks):
        expect[GUARD + c * cb : GUARD + (c + 1) * cb] = oracle_expected(oracle, pool, wl.descs, cb, 0)[GUARD : GUARD + cb]
    pool_d = torch.from_numpy(pool).to("cuda:0")
    dst_d = torch.full((expect.nbytes,), SENTINEL, dtype=torch.uint8, device="cuda:0")
    per_chunk = [
        [np.ascontiguousarray(wl.descs[int(r["first_desc"]) : int(r["first_desc"]) + int(r["n_descs"])]) for r in wl.requests]
        for wl in chunks
    ]
    flat = []
    for rep in range(400):  # 3200 slots of 4 MiB: about 10 ms of streaming
        for c, lists in enumerate(per_chunk):
            for d in lists:
                flat.append((pool_d.data_ptr(), dst_d.data_ptr() + GUARD + c * cb, d.ctypes.data, len(d)))
    items = (pkg.StreamItem * len(flat))()
    for i, (b, d, p, n) in enumerate(flat):
        items[i].bounce_base, items[i].dst_base, items[i].descs_host, items[i].n_descs = b, d, p, n
    n_copy = 64 << 20
    src = torch.randint(0, 256, (n_copy,), dtype=torch.uint8, device="cuda:0")
    out = torch.zeros(n_copy, dtype=torch.uint8, device="cuda:0")
    sides = [torch.cuda.Stream() for _ in range(4)]
    for side in sides:
        pkg.check(benchlib.tcpxuCopyKernelLaunch(0, out.data_ptr(), src.data_ptr(), n_copy, side.cuda_stream), "tcpxuCopyKernelLaunch")
    torch.cuda.synchronize()
    assert torch.equal(out, src)
    out.zero_()
    torch.cuda.synchronize()
    e = Engine(pkg, hip)
    cfg = pkg.EngineConfig()
    pkg.check(hip.tcpxuEngineGetConfig(e.h, ctypes.byref(cfg)), "tcpxuEngineGetConfig")
    cus = ctypes.c_int()
    pkg.check(hip.tcpxuDeviceInfo(0, None, 0, ctypes.byref(cus)), "tcpxuDeviceInfo")
    assert cfg.workgroups == 2 * cus.value + 1
    result = {}

    def stream_all():
        wall, kern = ctypes.c_double(), ctypes.c_double()
        result["t0"] = time.perf_counter()
        result["rc"] = benchlib.tcpxuEngineRunTimed(e.h, items, len(flat), 0, 64, 20000, ctypes.byref(wall), ctypes.byref(kern), None)
        result["t1"] = time.perf_counter()
        result["kernel_us"] = kern.value

    print("co-residency case: %d slots on the engine, copies of %d MiB beside it" % (len(flat), n_copy >> 20), flush=True)
    t = threading.Thread(target=stream_all)
    t.start()
    while not e.running() and t.is_alive():  # the launch is the thread's first act
        time.sleep(20e-6)
    finished = [[] for _ in sides]  # when each stream's copies were seen finished
    pending = [None] * len(sides)
    while t.is_alive():
        for k, side in enumerate(sides):
            if pending[k] is None:
                pkg.check(benchlib.tcpxuCopyKernelLaunch(0, out.data_ptr(), src.data_ptr(), n_copy, side.cuda_stream), "tcpxuCopyKernelLaunch")
                pending[k] = torch.cuda.Event()
                pending[k].record(side)
            elif pending[k].query():
                pending[k] = None
                finished[k].append(time.perf_counter())
    t.join(timeout=30)
    assert not t.is_alive() and result["rc"] == 0
    deadline = time.time() + 10
    for side in sides:  # a copy that shared the engine's hardware queue runs now
        while not side.query():
            assert time.time() < deadline, "a copy kernel did not finish after the engine had stopped"
    # a copy counts if it was seen finished well before the engine's launch ended (the launch is over 4 ms long)
    beside = [sum(1 for x in f if result["t0"] < x < result["t1"] - 5e-4) for f in finished]
    copies_while_running = sum(beside)
    print("co-residency case: copies finished while the engine streamed, per stream: %r (%.0f us launch)" % (beside, result["kernel_us"]), flush=True)
    assert copies_while_running >= 1 and sum(b > 0 for b in beside) >= 2, "copy kernels on other streams must run while the engine kernel is running"
    assert e.completed() == len(flat)
    e.destroy()
    assert torch.equal(out, src)
    got = dst_d.cpu().numpy()
    assert first_difference(got, expect) is None, "first (index, got, want, count): %r" % (first_difference(got, expect),)


@pytest.mark.parametrize("per_ticket", [0, 3, 16, 64])
def test_engine_alternating_one_byte_whole_page_and_empty_fragments(pkg, hip, oracle, per_ticket):
    """Fragments of 1, 4096 and 0 bytes in turn, contiguous in the destination from an odd byte offset, through the
    engine in slots of 700 descriptors and through the entry point that allocates nothing: destination lines shared
    by fragments of very different kinds, ticket boundaries falling anywhere among them."""
    from test_unpack_gpu import alternating_fragments, seeded_pool

    pool = seeded_pool(1 << 20, 17)
    descs, dst_bytes = alternating_fragments(401, 3, seed=18)
    expect = oracle_expected(oracle, pool, descs, dst_bytes, 0)
    g = GpuBuffers(pool, descs, dst_bytes, 0)
    slots = [(f, min(700, len(descs) - f)) for f in range(0, len(descs), 700)]
    m = Mapped(pkg, hip, np.ascontiguousarray(descs), len(slots))
    e = Engine(pkg, hip, descs_per_ticket=per_ticket)
    print("engine alternating case: %d descriptors, %d slots, tickets of %d" % (len(descs), len(slots), per_ticket), flush=True)
    e.start()
    try:
        for i, (first, n) in enumerate(slots):
            e.submit(g.pool.data_ptr(), g.dst_base, m.desc_dev(first), n, m.flag_dev(i), i + 1)
        for i in range(len(slots)):
            m.wait(i, i + 1)
    finally:
        e.stop()
    got = g.result()
    e.destroy()
    assert first_difference(got, expect) is None, "first (index, got, want, count): %r" % (first_difference(got, expect),)
    if per_ticket == 0:
        g.reset()
        for i, (first, n) in enumerate(slots):
            pkg.check(hip.tcpxuUnpackSlotNoAlloc(0, g.pool.data_ptr(), g.dst_base, m.desc_dev(first), n, None, 0, None), "tcpxuUnpackSlotNoAlloc")
        pkg.check(hip.tcpxuDeviceSynchronize(0), "tcpxuDeviceSynchronize")
        got = g.result()
        assert first_difference(got, expect) is None, "no-alloc: first (index, got, want, count): %r" % (first_difference(got, expect),)
    m.free()


@pytest.mark.parametrize("kind", ["long", "short"])
@pytest.mark.parametrize("per_ticket", [0, 3, 64])
def test_engine_every_boundary_position_inside_a_shared_line(pkg, hip, oracle, per_ticket, kind):
    """Runs of three contiguous fragments with their boundaries at every offset inside a 128-byte line ("long"), and
    runs of short fragments that lie in the lines they share with their neighbours ("short"), through the engine
    (tickets of 3 descriptors, the adaptive size and 64 cut the runs anywhere) and through the entry point that
    allocates nothing."""
    from test_unpack_gpu import boundary_runs, seeded_pool, short_runs

    pool = seeded_pool(1 << 20, 31)
    descs, dst_bytes = boundary_runs(32 + per_ticket) if kind == "long" else short_runs(52 + per_ticket)
    expect = oracle_expected(oracle, pool, descs, dst_bytes, 0)
    g = GpuBuffers(pool, descs, dst_bytes, 0)
    m = Mapped(pkg, hip, np.ascontiguousarray(descs), 1)
    e = Engine(pkg, hip, descs_per_ticket=per_ticket)
    print("engine boundary case: %d descriptors, tickets of %d" % (len(descs), per_ticket), flush=True)
    e.start()
    try:
        e.submit(g.pool.data_ptr(), g.dst_base, m.desc_dev(0), len(descs), m.flag_dev(0), 1)
        m.wait(0, 1)
    finally:
        e.stop()
    got = g.result()
    e.destroy()
    assert first_difference(got, expect) is None, "first (index, got, want, count): %r" % (first_difference(got, expect),)
    if per_ticket == 0:
        g.reset()
        pkg.check(hip.tcpxuUnpackSlotNoAlloc(0, g.pool.data_ptr(), g.dst_base, m.desc_dev(0), len(descs), None, 0, None), "tcpxuUnpackSlotNoAlloc")
        pkg.check(hip.tcpxuDeviceSynchronize(0), "tcpxuDeviceSynchronize")
        got = g.result()
        assert first_difference(got, expect) is None, "no-alloc: first (index, got, want, count): %r" % (first_difference(got, expect),)
    m.free()


@pytest.mark.parametrize("seed", range(200, 212))
def test_engine_random_mixtures_of_fragment_kinds(pkg, hip, oracle, seed):
    """Descriptor lists drawn from a seed (every kind of fragment beside every other, gaps now and then), in slots of
    a random size, through the engine at a ticket size drawn from the seed, and through the entry point that
    allocates nothing."""
    from test_unpack_gpu import random_mixture, seeded_pool

    rng = np.random.default_rng(seed)
    pool = seeded_pool(1 << 20, seed)
    descs, dst_bytes = random_mixture(seed)
    per_ticket = int(rng.choice([0, 0, 1, 5, 16, 33, 64]))
    slot = int(rng.integers(1, 2049))
    expect = oracle_expected(oracle, pool, descs, dst_bytes, 0)
    g = GpuBuffers(pool, descs, dst_bytes, 0)
    slots = [(f, min(slot, len(descs) - f)) for f in range(0, len(descs), slot)]
    m = Mapped(pkg, hip, np.ascontiguousarray(descs), len(slots))
    e = Engine(pkg, hip, descs_per_ticket=per_ticket)
    print("engine mixture case: seed %d, %d descriptors, slots of %d, tickets of %d" % (seed, len(descs), slot, per_ticket), flush=True)
    e.start()
    try:
        for i, (first, n) in enumerate(slots):
            nbytes = int(descs["len"][first : first + n].sum()) if seed % 2 else 0  # with and without the payload hint
            deadline = time.time() + 20
            while True:
                rc = hip.tcpxuEngineSubmitSized(e.h, g.pool.data_ptr(), g.dst_base, m.desc_dev(first), n, min(nbytes, 0xFFFFFFFF), m.flag_dev(i), i + 1)
                if rc != pkg.IN_PROGRESS:
                    break
                assert time.time() < deadline, "submission ring stayed full"
            pkg.check(rc, "tcpxuEngineSubmitSized")
        for i in range(len(slots)):
            m.wait(i, i + 1)
    finally:
        e.stop()
    got = g.result()
    e.destroy()
    assert first_difference(got, expect) is None, "first (index, got, want, count): %r" % (first_difference(got, expect),)
    g.reset()
    for first, n in slots:
        pkg.check(hip.tcpxuUnpackSlotNoAlloc(0, g.pool.data_ptr(), g.dst_base, m.desc_dev(first), n, None, 0, None), "tcpxuUnpackSlotNoAlloc")
    pkg.check(hip.tcpxuDeviceSynchronize(0), "tcpxuDeviceSynchronize")
    got = g.result()
    assert first_difference(got, expect) is None, "no-alloc: first (index, got, want, count): %r" % (first_difference(got, expect),)
    m.free()


@pytest.mark.parametrize("per_ticket", [0, 7, 16])
def test_engine_many_mid_size_submissions_waiting_at_once(pkg, hip, oracle, per_ticket):
    """A backlog the leader finds sixteen entries deep at its first look: 300 submissions of 1 to 520 descriptors (one
    ticket, a few, up to the most the leader's lanes write themselves, and beyond), empty ones in between, queued
    before the kernel is launched.  Every poll then hands out the tickets of several submissions at once."""
    from test_unpack_gpu import seeded_pool

    rng = np.random.default_rng(900 + per_ticket)
    pool = seeded_pool(1 << 20, 901)
    sizes = [int(x) for x in rng.choice([1, 8, 16, 17, 33, 64, 100, 256, 257, 512, 520, 0], size=300)]
    rows, dst = [], 5
    for n in sizes:
        for _ in range(n):
            ln = int(rng.integers(1, 1500))
            rows.append((int(rng.integers(0, 255)) * 4096 + int(rng.integers(0, 4096 - ln + 1)), ln, dst))
            dst += ln
    descs = make_descs(rows)
    expect = oracle_expected(oracle, pool, descs, dst + 64, 0)
    g = GpuBuffers(pool, descs, dst + 64, 0)
    m = Mapped(pkg, hip, np.ascontiguousarray(descs), len(sizes))
    e = Engine(pkg, hip, descs_per_ticket=per_ticket)
    print("engine backlog case: %d submissions, %d descriptors, tickets of %d" % (len(sizes), len(descs), per_ticket), flush=True)
    first = 0
    for i, n in enumerate(sizes):
        e.submit(g.pool.data_ptr(), g.dst_base, m.desc_dev(first), n, m.flag_dev(i), i + 1)
        first += n
    e.start()
    try:
        for i in range(len(sizes)):
            m.wait(i, i + 1)
    finally:
        e.stop()
    assert e.completed() == len(sizes)
    got = g.result()
    e.destroy()
    m.free()
    assert first_difference(got, expect) is None, "first (index, got, want, count): %r" % (first_difference(got, expect),)


@pytest.mark.parametrize("mean_len", [700, 1500, 2300])
def test_engine_queued_submissions_of_short_fragments_with_the_payload_given(pkg, hip, oracle, mean_len):
    """Forty submissions of 600 to 2048 short fragments each, every one with its byte count, all queued before the
    kernel is launched: the payload asks for tickets of 64, 48 or 32 descriptors, so a submission is at most 32
    tickets and the leader's lanes write the tickets of the whole run of entries they hold (up to 2048 descriptors
    each, where without the byte count it is 512)."""
    from test_unpack_gpu import seeded_pool

    rng = np.random.default_rng(4000 + mean_len)
    pool = seeded_pool(1 << 20, 4001)
    sizes = [int(x) for x in rng.choice([600, 1024, 1500, 2047, 2048], size=40)]
    rows, dst = [], 3
    for n in sizes:
        for _ in range(n):
            ln = int(rng.integers(max(1, mean_len - 600), mean_len + 600))
            rows.append((int(rng.integers(0, 255)) * 4096 + int(rng.integers(0, 4096 - ln + 1)), ln, dst))
            dst += ln
    descs = make_descs(rows)
    expect = oracle_expected(oracle, pool, descs, dst + 64, 0)
    g = GpuBuffers(pool, descs, dst + 64, 0)
    m = Mapped(pkg, hip, np.ascontiguousarray(descs), len(sizes))
    e = Engine(pkg, hip)
    print("engine queued short-fragment case: %d submissions, %d descriptors, mean length %d" % (len(sizes), len(descs), mean_len), flush=True)
    first = 0
    for i, n in enumerate(sizes):
        nbytes = int(descs["len"][first : first + n].sum())
        rc = hip.tcpxuEngineSubmitSized(e.h, g.pool.data_ptr(), g.dst_base, m.desc_dev(first), n, nbytes, m.flag_dev(i), i + 1)
        pkg.check(rc, "tcpxuEngineSubmitSized")
        first += n
    e.start()
    try:
        for i in range(len(sizes)):
            m.wait(i, i + 1)
    finally:
        e.stop()
    assert e.completed() == len(sizes)
    got = g.result()
    e.destroy()
    m.free()
    assert first_difference(got, expect) is None, "first (index, got, want, count): %r" % (first_difference(got, expect),)


@pytest.mark.parametrize("per_ticket", [0, 5, 14, 16])
def test_engine_lines_shared_across_the_ends_of_tickets(pkg, hip, oracle, per_ticket):
    """With eight or more submissions in flight the tickets of a submission share destination lines across their
    ends: runs of fragments with boundaries at every offset inside a line, and runs of short fragments, in slots of
    37 descriptors all submitted at once, so that ticket ends fall anywhere in the runs and most slots are handed out
    while many are in flight (the first few are not, and keep their ends to themselves)."""
    from test_unpack_gpu import boundary_runs, seeded_pool, short_runs

    pool = seeded_pool(1 << 20, 61)
    a, a_bytes = boundary_runs(62 + per_ticket)
    b, b_bytes = short_runs(63 + per_ticket)
    b = b.copy()
    b["dst_off"] += a_bytes
    descs = np.concatenate([a, b])
    dst_bytes = a_bytes + b_bytes
    expect = oracle_expected(oracle, pool, descs, dst_bytes, 0)
    g = GpuBuffers(pool, descs, dst_bytes, 0)
    slots = [(f, min(37, len(descs) - f)) for f in range(0, len(descs), 37)]
    m = Mapped(pkg, hip, np.ascontiguousarray(descs), len(slots))
    e = Engine(pkg, hip, descs_per_ticket=per_ticket)
    print("engine ticket-ends case: %d descriptors, %d slots, tickets of %d" % (len(descs), len(slots), per_ticket), flush=True)
    for i, (first, n) in enumerate(slots):  # queued before the kernel starts: all in flight together
        e.submit(g.pool.data_ptr(), g.dst_base, m.desc_dev(first), n, m.flag_dev(i), i + 1)
    e.start()
    try:
        for i in range(len(slots)):
            m.wait(i, i + 1)
    finally:
        e.stop()
    got = g.result()
    e.destroy()
    m.free()
    assert first_difference(got, expect) is None, "first (index, got, want, count): %r" % (first_difference(got, expect),)


def test_engine_stamps_order_the_stages_of_a_submission(pkg, hip, oracle):
    """With stamps switched on the kernel records when the leader saw a submission, when its first ticket was
    fetched, when that ticket's descriptors were staged and when its last store was acknowledged: four readings of
    one clock, in that order, for single-ticket, multi-ticket and empty-descriptor submissions alike; the bytes are
    the oracle's as ever."""
    wl = pkg.Workload(2, seed=0x57A3, shrink=2)  # 2 MiB in two requests of about 270 descriptors
    info = wl.info
    pool = np.empty(info.pool_bytes, dtype=np.uint8)
    wl.fill_window(0, pool)
    expect = oracle_expected(oracle, pool, wl.descs, info.dst_bytes)
    g = GpuBuffers(pool, wl.descs, info.dst_bytes)
    m = Mapped(pkg, hip, np.ascontiguousarray(wl.descs), 8)
    e = Engine(pkg, hip)
    rate = ctypes.c_double()
    pkg.check(hip.tcpxuEngineEnableStamps(e.h, ctypes.byref(rate)), "tcpxuEngineEnableStamps")
    assert 1.0 <= rate.value <= 10000.0
    out = (ctypes.c_uint64 * 32)()
    e.start()
    assert hip.tcpxuEngineReadStamps(e.h, 0, 1, out) == pkg.INVALID_USAGE  # only while stopped
    subs = []
    for i, r in enumerate(wl.requests):  # whole requests: many tickets each
        subs.append((int(r["first_desc"]), int(r["n_descs"])))
    first, n = subs[0]
    subs += [(first, 5), (first + 5, 3)]  # and two that fit one ticket
    for i, (f, cnt) in enumerate(subs):
        e.submit(g.pool.data_ptr(), g.dst_base, m.desc_dev(f), cnt, m.flag_dev(i), i + 1)
        m.wait(i, i + 1)
    e.stop()
    pkg.check(hip.tcpxuEngineReadStamps(e.h, 0, len(subs), out), "tcpxuEngineReadStamps")
    never = 0xFFFFFFFFFFFFFFFF
    for i in range(len(subs)):
        t = [out[4 * i + k] for k in range(4)]
        assert never not in t, (i, t)
        assert t[0] <= t[1] <= t[2] <= t[3], (i, t)
        assert (t[3] - t[0]) / rate.value < 1e6, "a small submission takes microseconds, not a second"
        if i:
            assert t[0] >= out[4 * (i - 1) + 3], "one at a time: a submission is seen after the one before it completed"
    pkg.check(hip.tcpxuEngineReadStamps(e.h, 0, len(subs), out), "tcpxuEngineReadStamps")
    assert all(out[k] == never for k in range(4 * len(subs))), "reading clears the stamps"
    got = g.result()
    e.destroy()
    m.free()
    assert first_difference(got, expect) is None, repr(first_difference(got, expect))
