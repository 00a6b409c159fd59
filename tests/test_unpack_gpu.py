"""GPU parity of the launch-per-batch unpack kernel (tcpxuUnpackBatch) against the CPU oracle, byte-exact.

Tolerance: none -- this path is integer/byte work, every byte of the destination (guard bands included) must be
identical to the oracle's.
"""
import ctypes

import numpy as np
import pytest

from conftest import GUARD, SENTINEL, GpuBuffers, first_difference, make_descs, oracle_expected

pytestmark = pytest.mark.gpu


def run_batch(pkg, hip, oracle, pool, descs, dst_bytes, misalign=0):
    expect = oracle_expected(oracle, pool, descs, dst_bytes, misalign)
    g = GpuBuffers(pool, descs, dst_bytes, misalign)
    print("case: n=%d dst_bytes=%d misalign=%d" % (len(descs), dst_bytes, misalign), flush=True)
    pkg.check(hip.tcpxuUnpackBatch(0, g.pool.data_ptr(), g.dst_base, g.descs.data_ptr(), g.n, None), "tcpxuUnpackBatch")
    pkg.check(hip.tcpxuDeviceSynchronize(0), "sync")
    got = g.result()
    assert first_difference(got, expect) is None, "first (index, got, want, count): %r" % (first_difference(got, expect),)


def seeded_pool(nbytes, seed):
    return np.random.default_rng(seed).integers(0, 256, size=nbytes, dtype=np.uint8)


@pytest.mark.parametrize("config", [1, 2, 3, 4, 5])
def test_workloads_reduced(pkg, hip, oracle, config):
    wl = pkg.Workload(config, seed=0xC0FFEE00 + config, shrink=4)
    pool = np.empty(wl.info.pool_bytes, dtype=np.uint8)
    wl.fill_window(0, pool)
    # window 0 payload everywhere: reuse of pages across windows is exercised in test_windows_refill
    run_batch(pkg, hip, oracle, pool, wl.descs, wl.info.dst_bytes, wl.info.dst_misalign)


@pytest.mark.parametrize("config", [1, 2, 3, 4])
def test_workloads_full_size(pkg, hip, oracle, config):
    wl = pkg.Workload(config, seed=0xC0FFEE00 + config, shrink=0)
    pool = np.empty(wl.info.pool_bytes, dtype=np.uint8)
    wl.fill_window(0, pool)
    run_batch(pkg, hip, oracle, pool, wl.descs, wl.info.dst_bytes, wl.info.dst_misalign)


def test_windows_refill_full_size(pkg, hip, oracle):
    """Adversarial workload at full size: pages are refilled between requests, as recycled pages would be."""
    import torch

    wl = pkg.Workload(5, seed=0xC0FFEE05, shrink=0)
    info = wl.info
    pool = np.empty(info.pool_bytes, dtype=np.uint8)
    expect = np.full(GUARD + info.dst_misalign + info.dst_bytes + GUARD, SENTINEL, dtype=np.uint8)
    base = GUARD + info.dst_misalign
    g = None
    for r in wl.requests:
        w = int(r["window"])
        wl.fill_window(w, pool)
        d = np.ascontiguousarray(wl.descs[int(r["first_desc"]) : int(r["first_desc"]) + int(r["n_descs"])])
        import __graft_entry__ as graft

        graft.oracle_unpack(oracle, expect[base : base + info.dst_bytes], pool, d)
        if g is None:
            g = GpuBuffers(pool, wl.descs, info.dst_bytes, info.dst_misalign)
        else:
            g.pool.copy_(torch.from_numpy(pool))
            torch.cuda.synchronize()
        print("window %d: %d descriptors" % (w, len(d)), flush=True)
        pkg.check(
            hip.tcpxuUnpackBatch(0, g.pool.data_ptr(), g.dst_base, g.descs.data_ptr() + 16 * int(r["first_desc"]), len(d), None),
            "tcpxuUnpackBatch",
        )
        pkg.check(hip.tcpxuDeviceSynchronize(0), "sync")
    got = g.result()
    assert first_difference(got, expect) is None, repr(first_difference(got, expect))


def test_every_alignment_and_short_length(pkg, hip, oracle):
    """All 16x16 (src, dst) alignments times lengths around the vector and round boundaries."""
    pool = seeded_pool(1 << 20, 1)
    lengths = [1, 2, 3, 15, 16, 17, 31, 32, 33, 63, 64, 65, 255, 256, 1023, 1024, 1025, 4079, 4080, 4081, 4095, 4096]
    rows, dst = [], 0
    rng = np.random.default_rng(2)
    for sa in range(16):
        for da in range(16):
            for ln in lengths:
                page = int(rng.integers(0, (1 << 20) // 4096))
                in_page = sa if sa + ln <= 4096 else 0
                dst = (dst + 15) // 16 * 16 + da
                rows.append((page * 4096 + in_page, ln, dst))
                dst += ln + 1  # one sentinel byte between neighbours must survive
    run_batch(pkg, hip, oracle, pool, make_descs(rows), dst + 16)


def test_empty_and_zero_length(pkg, hip, oracle):
    pool = seeded_pool(1 << 16, 3)
    run_batch(pkg, hip, oracle, pool, make_descs([]), 4096)
    run_batch(pkg, hip, oracle, pool, make_descs([(0, 0, 0), (5, 0, 100), (4096, 0, 4095)]), 4096)
    run_batch(pkg, hip, oracle, pool, make_descs([(0, 0, 0), (7, 100, 3), (9, 0, 50), (4096, 1, 200)]), 4096)


def test_single_bytes_and_ragged_tail(pkg, hip, oracle):
    pool = seeded_pool(1 << 16, 4)
    rows = [(i * 37 % 60000, 1, i * 3) for i in range(1000)]
    run_batch(pkg, hip, oracle, pool, make_descs(rows), 3 * 1000 + 8)
    # descriptor count that is not a multiple of any batch size
    rows = [((i * 4096) % 61440, 4096 - (i % 7), i * 4096) for i in range(1021)]
    run_batch(pkg, hip, oracle, pool, make_descs(rows), 1021 * 4096)


def test_long_descriptor_beyond_one_page(pkg, hip, oracle):
    """The wire contract caps a fragment at 4 KiB, but `len` is 32 bits: longer copies must still be exact."""
    pool = seeded_pool(1 << 20, 5)
    rows = [(3, 70001, 5), (100000, 8192, 80000), (200001, 4097, 90001)]
    run_batch(pkg, hip, oracle, pool, make_descs(rows), 100000)
    # Long fragments that continue each other in the destination with boundaries inside 128-byte lines: several
    # rounds each, and the line at every boundary is completed by the owner of the fragment before it.
    rows, dst = [], 7
    for src, ln in [(11, 10001), (300002, 9000), (500003, 4097 + 4096), (700000, 300), (800005, 20000), (900001, 4096)]:
        rows.append((src, ln, dst))
        dst += ln
    run_batch(pkg, hip, oracle, pool, make_descs(rows), dst + 64)


def test_descriptors_in_mapped_host_memory(pkg, hip, oracle):
    """The kernel reads descriptors through the device alias of hipHostMalloc-mapped memory."""
    wl = pkg.Workload(2, seed=77, shrink=3)
    pool = np.empty(wl.info.pool_bytes, dtype=np.uint8)
    wl.fill_window(0, pool)
    expect = oracle_expected(oracle, pool, wl.descs, wl.info.dst_bytes)
    g = GpuBuffers(pool, wl.descs, wl.info.dst_bytes)
    host_p, dev_p = ctypes.c_void_p(), ctypes.c_void_p()
    pkg.check(hip.tcpxuMappedAlloc(0, wl.descs.nbytes, ctypes.byref(host_p), ctypes.byref(dev_p)), "tcpxuMappedAlloc")
    ctypes.memmove(host_p.value, wl.descs.ctypes.data, wl.descs.nbytes)
    pkg.check(hip.tcpxuUnpackBatch(0, g.pool.data_ptr(), g.dst_base, dev_p.value, g.n, None), "tcpxuUnpackBatch")
    pkg.check(hip.tcpxuDeviceSynchronize(0), "sync")
    got = g.result()
    pkg.check(hip.tcpxuMappedFree(0, host_p), "tcpxuMappedFree")
    assert first_difference(got, expect) is None, repr(first_difference(got, expect))


def test_linearity_two_halves_equal_whole(pkg, hip, oracle):
    """Size-independent property: unpacking a list in two launches equals unpacking it in one."""
    wl = pkg.Workload(4, seed=9, shrink=2)
    pool = np.empty(wl.info.pool_bytes, dtype=np.uint8)
    wl.fill_window(0, pool)
    g = GpuBuffers(pool, wl.descs, wl.info.dst_bytes)
    pkg.check(hip.tcpxuUnpackBatch(0, g.pool.data_ptr(), g.dst_base, g.descs.data_ptr(), g.n, None), "whole")
    pkg.check(hip.tcpxuDeviceSynchronize(0), "sync")
    whole = g.result()
    g.reset()
    half = g.n // 2 + 3
    pkg.check(hip.tcpxuUnpackBatch(0, g.pool.data_ptr(), g.dst_base, g.descs.data_ptr() + 16 * half, g.n - half, None), "b")
    pkg.check(hip.tcpxuUnpackBatch(0, g.pool.data_ptr(), g.dst_base, g.descs.data_ptr(), half, None), "a")
    pkg.check(hip.tcpxuDeviceSynchronize(0), "sync")
    assert np.array_equal(whole, g.result())
    assert np.array_equal(whole, oracle_expected(oracle, pool, wl.descs, wl.info.dst_bytes))


def test_argument_errors(pkg, hip):
    assert hip.tcpxuUnpackBatch(0, None, None, None, 5, None) == pkg.INVALID_ARGUMENT
    p = ctypes.c_void_p()
    assert hip.tcpxuArenaCreate(0, 4097, ctypes.byref(p)) == pkg.INVALID_ARGUMENT
    assert hip.tcpxuArenaCreate(0, (1 << 32) + 4096, ctypes.byref(p)) == pkg.INVALID_ARGUMENT
    assert hip.tcpxuArenaCreate(99, 4096, ctypes.byref(p)) == pkg.INVALID_ARGUMENT
    pkg.check(hip.tcpxuArenaCreate(0, 1 << 20, ctypes.byref(p)), "arena")
    assert p.value % 4096 == 0
    pkg.check(hip.tcpxuArenaDestroy(0, p), "arena destroy")


def test_yardstick_kernels_copy_read_fill(pkg, hip, benchlib):
    """The measurement helpers behind the benchmark's copy, read-only and write-only figures: the copy is exact
    (odd size in vectors, so the last workgroup is partial), the read leaves its source alone, the fill writes
    every vector of the range and nothing beyond it."""
    import torch

    n = (3 << 20) + 16 * 37
    src = torch.randint(0, 256, (n,), dtype=torch.uint8, device="cuda:0")
    dst = torch.full((n + 64,), SENTINEL, dtype=torch.uint8, device="cuda:0")
    keep = src.clone()
    us = ctypes.c_double()
    pkg.check(benchlib.tcpxuCopyKernelTimed(0, dst.data_ptr(), src.data_ptr(), n, 1, 3, ctypes.byref(us)), "copy")
    assert us.value > 0 and torch.equal(dst[:n], src) and bool((dst[n:] == SENTINEL).all())
    pkg.check(benchlib.tcpxuCopyKernelTimed(0, None, src.data_ptr(), n, 1, 3, ctypes.byref(us)), "read")
    assert us.value > 0 and torch.equal(src, keep)
    dst.fill_(SENTINEL)
    pkg.check(benchlib.tcpxuCopyKernelTimed(0, dst.data_ptr(), None, n, 1, 3, ctypes.byref(us)), "fill")
    words = dst[:n].view(torch.int32).view(-1, 4)
    assert us.value > 0 and bool((words[:, 2] == -0x5A5A5A5B).all()) and bool((words[:, 3] == 0x5A5A5A5A).all())
    assert bool((dst[n:] == SENTINEL).all())
    assert benchlib.tcpxuCopyKernelTimed(0, None, None, n, 1, 3, ctypes.byref(us)) == pkg.INVALID_ARGUMENT
    assert benchlib.tcpxuCopyKernelTimed(0, dst.data_ptr(), src.data_ptr(), n + 8, 1, 3, ctypes.byref(us)) == pkg.INVALID_ARGUMENT


@pytest.mark.parametrize("kib", [1, 2, 3, 4])
def test_yardstick_gather_kernel_moves_the_fragments_it_says(pkg, hip, benchlib, kib):
    """The bare gather behind the benchmark's short-fragment yardsticks: fragment i of the destination is the first
    kib KiB of page pages[i] of the pool, for every i, and nothing beyond the last fragment is written."""
    import torch

    n_pages, n_frag, frag = 4096, 3001, kib << 10
    pool = torch.randint(0, 256, (n_pages * 4096,), dtype=torch.uint8, device="cuda:0")
    pages = torch.randint(0, n_pages, (n_frag,), dtype=torch.int32, device="cuda:0")
    dst = torch.full((n_frag * frag + 64,), SENTINEL, dtype=torch.uint8, device="cuda:0")
    us = ctypes.c_double()
    print("gather yardstick case: %d fragments of %d bytes" % (n_frag, frag), flush=True)
    pkg.check(benchlib.tcpxuGatherKernelTimed(0, dst.data_ptr(), pool.data_ptr(), pages.data_ptr(), n_frag, frag, 1, 2, ctypes.byref(us)), "gather")
    want = pool.view(n_pages, 4096)[pages.long(), :frag].reshape(-1)
    assert us.value > 0 and torch.equal(dst[: n_frag * frag], want) and bool((dst[n_frag * frag :] == SENTINEL).all())
    assert benchlib.tcpxuGatherKernelTimed(0, dst.data_ptr(), pool.data_ptr(), pages.data_ptr(), n_frag, frag + 512, 1, 2, ctypes.byref(us)) == pkg.INVALID_ARGUMENT
    assert benchlib.tcpxuGatherKernelTimed(0, dst.data_ptr(), pool.data_ptr(), None, n_frag, frag, 1, 2, ctypes.byref(us)) == pkg.INVALID_ARGUMENT


def test_batch_launches_replayed_from_a_hip_graph(pkg, hip, oracle):
    """A launch-bound loop of small batches (32 requests of 16 fragments, one tcpxuUnpackBatch each) captured once
    into a HIP graph on a caller's stream and replayed: every replay, with the pool refilled and the destination
    reset by ordinary eager work in between, must give the oracle's bytes for the pool of that replay."""
    import torch

    wl = pkg.Workload(3, seed=0x6A9, shrink=6)
    info = wl.info
    reqs = [(int(r["first_desc"]), int(r["n_descs"])) for r in wl.requests][:32]
    n_descs = reqs[-1][0] + reqs[-1][1]
    descs = np.ascontiguousarray(wl.descs[:n_descs])
    dst_bytes = int((descs["dst_off"] + descs["len"]).max())
    pool = np.empty(info.pool_bytes, dtype=np.uint8)
    wl.fill_window(0, pool)
    g = GpuBuffers(pool, descs, dst_bytes, 0)
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    print("graph case: %d launches, %d descriptors" % (len(reqs), n_descs), flush=True)
    with torch.cuda.graph(graph, stream=stream):
        s = torch.cuda.current_stream().cuda_stream
        for first, n in reqs:
            pkg.check(hip.tcpxuUnpackBatch(0, g.pool.data_ptr(), g.dst_base, g.descs.data_ptr() + 16 * first, n, ctypes.c_void_p(s)), "tcpxuUnpackBatch")
    for replay in range(3):
        if replay:
            pool = np.roll(pool, 4099 * replay) ^ np.uint8(replay)
            g.pool.copy_(torch.from_numpy(pool))
        g.reset()
        graph.replay()
        torch.cuda.synchronize()
        expect = oracle_expected(oracle, pool, descs, dst_bytes, 0)
        got = g.result()
        assert first_difference(got, expect) is None, "replay %d, first (index, got, want, count): %r" % (replay, first_difference(got, expect))


def test_descriptors_in_host_visible_device_memory(pkg, hip, oracle):
    """tcpxuVisibleAlloc: the host writes descriptors straight into device memory (through the BAR), flushes, and
    a kernel launched afterwards reads them there; a freed block is handed out again; bad arguments are refused."""
    wl = pkg.Workload(5, seed=0x715, shrink=5)
    pool = np.empty(wl.info.pool_bytes, dtype=np.uint8)
    wl.fill_window(0, pool)
    descs = np.ascontiguousarray(wl.descs)
    g = GpuBuffers(pool, descs[:0], wl.info.dst_bytes, wl.info.dst_misalign)
    host, dev = ctypes.c_void_p(), ctypes.c_void_p()
    rc = hip.tcpxuVisibleAlloc(0, descs.nbytes, ctypes.byref(host), ctypes.byref(dev))
    if rc == pkg.INVALID_USAGE:
        pytest.skip("this device does not expose its memory to the host: " + hip.tcpxuLastError().decode())
    pkg.check(rc, "tcpxuVisibleAlloc")
    print("visible-memory case: %d descriptors" % len(descs), flush=True)
    ctypes.memmove(host.value, descs.ctypes.data, descs.nbytes)
    hip.tcpxuVisibleFlush()
    pkg.check(hip.tcpxuUnpackBatch(0, g.pool.data_ptr(), g.dst_base, dev, len(descs), None), "tcpxuUnpackBatch")
    pkg.check(hip.tcpxuDeviceSynchronize(0), "sync")
    expect = oracle_expected(oracle, pool, descs, wl.info.dst_bytes, wl.info.dst_misalign)
    got = g.result()
    assert first_difference(got, expect) is None, "first (index, got, want, count): %r" % (first_difference(got, expect),)
    pkg.check(hip.tcpxuVisibleFree(0, host), "tcpxuVisibleFree")
    assert hip.tcpxuVisibleFree(0, host) == pkg.INVALID_ARGUMENT  # not handed out any more
    again_h, again_d = ctypes.c_void_p(), ctypes.c_void_p()
    pkg.check(hip.tcpxuVisibleAlloc(0, descs.nbytes, ctypes.byref(again_h), ctypes.byref(again_d)), "tcpxuVisibleAlloc")
    assert again_h.value == host.value  # blocks are kept and reused, not returned to the driver
    pkg.check(hip.tcpxuVisibleFree(0, again_h), "tcpxuVisibleFree")
    assert hip.tcpxuVisibleAlloc(0, 0, ctypes.byref(host), ctypes.byref(dev)) == pkg.INVALID_ARGUMENT
    assert hip.tcpxuVisibleAlloc(0, 65 << 20, ctypes.byref(host), ctypes.byref(dev)) == pkg.INVALID_ARGUMENT


def alternating_fragments(n_groups, dst_base_offset, seed):
    """Fragments of 1, 4096 and 0 bytes in turn (and, every fourth group, 300 and 200 bytes: one that may share a
    line with its neighbours and one too short to), contiguous in the destination from an arbitrary byte offset:
    one-byte and empty fragments sit between whole pages, so that destination lines are shared by up to four
    fragments of very different kinds."""
    rng = np.random.default_rng(seed)
    rows, dst = [], dst_base_offset
    for g in range(n_groups):
        lens = [1, 4096, 0] if g % 4 else [1, 4096, 0, 300, 200]
        for ln in lens:
            page = int(rng.integers(0, 250))
            in_page = int(rng.integers(0, 4096 - ln + 1))
            rows.append((page * 4096 + in_page, ln, dst))
            dst += ln
    return make_descs(rows), dst + 64


@pytest.mark.parametrize("offset", [0, 1, 127, 4095])
def test_alternating_one_byte_whole_page_and_empty_fragments(pkg, hip, oracle, offset):
    pool = seeded_pool(1 << 20, 7)
    descs, dst_bytes = alternating_fragments(301, offset, seed=8 + offset)
    run_batch(pkg, hip, oracle, pool, descs, dst_bytes)


def boundary_runs(seed, pool_bytes=1 << 20):
    """Runs of three fragments that continue each other in the destination, every fragment at least 256 bytes (long
    enough to share a line with its neighbour), with the two boundaries of each run at chosen offsets inside a
    128-byte line: all 128 offsets occur as a first boundary, each with a different second one.  Sources have any
    byte alignment; in every fourth run the first fragment ends exactly at the end of its bounce page, in every
    eighth at the end of the pool, with the next fragment at the start of a page.  Runs are separated by a byte
    that must survive; in every third run an empty descriptor sits between the first two fragments."""
    rng = np.random.default_rng(seed)
    pages = pool_bytes // 4096
    rows, dst = [], 0
    for b1 in range(128):
        b2 = (b1 * 7 + 13) % 128
        start = int(rng.integers(0, 128))
        dst = (dst + 127) // 128 * 128 + start
        len_a = 256 + int(rng.integers(0, 12)) * 128 + (b1 - start - 256) % 128
        len_b = 256 + int(rng.integers(0, 12)) * 128 + (b2 - b1 - 256) % 128
        len_c = 256 + int(rng.integers(0, 3000))
        assert (dst + len_a) % 128 == b1 and (dst + len_a + len_b) % 128 == b2
        for i, ln in enumerate((len_a, len_b, len_c)):
            page = int(rng.integers(0, pages))
            in_page = int(rng.integers(0, 4096 - ln + 1))
            if i == 0 and b1 % 4 == 0:
                in_page = 4096 - ln
                if b1 % 8 == 0:
                    page = pages - 1
            if i == 1 and b1 % 4 == 0:
                in_page = 0
            rows.append((page * 4096 + in_page, ln, dst))
            dst += ln
            if i == 0 and b1 % 3 == 0:
                rows.append((page * 4096, 0, dst))  # an empty descriptor between two that continue each other
        dst += 1
    return make_descs(rows), dst + 64


def test_every_boundary_position_inside_a_shared_line(pkg, hip, oracle):
    pool = seeded_pool(1 << 20, 21)
    for seed in (22, 23):
        descs, dst_bytes = boundary_runs(seed)
        run_batch(pkg, hip, oracle, pool, descs, dst_bytes)
        run_batch(pkg, hip, oracle, pool, descs, dst_bytes, misalign=5)


def random_mixture(seed, pool_bytes=1 << 20, max_descs=3000):
    """A descriptor list drawn from a seed: empty, tiny, short, medium, whole-page and longer-than-a-page fragments in
    random order, mostly continuing each other in the destination (so that lines are shared by every kind of
    neighbour) with gaps now and then, sources at any byte offset."""
    rng = np.random.default_rng(seed)
    n = int(rng.integers(1, max_descs + 1))
    kinds = rng.choice(6, size=n, p=[0.10, 0.10, 0.25, 0.30, 0.20, 0.05])
    rows, dst = [], int(rng.integers(0, 256))
    for kind in kinds:
        ln = (0, int(rng.integers(1, 31)), int(rng.integers(31, 601)), int(rng.integers(601, 4096)), 4096, int(rng.integers(4097, 20001)))[kind]
        if ln <= 4096:
            src = int(rng.integers(0, pool_bytes // 4096)) * 4096 + int(rng.integers(0, 4096 - ln + 1))
        else:
            src = int(rng.integers(0, pool_bytes - ln + 1))
        if rng.random() < 0.2:
            dst += int(rng.integers(1, 301))
        rows.append((src, ln, dst))
        dst += ln
    return make_descs(rows), dst + 64


@pytest.mark.parametrize("seed", range(100, 112))
def test_random_mixtures_of_fragment_kinds(pkg, hip, oracle, seed):
    pool = seeded_pool(1 << 20, seed)
    descs, dst_bytes = random_mixture(seed)
    run_batch(pkg, hip, oracle, pool, descs, dst_bytes, misalign=seed % 16)


def short_runs(seed, pool_bytes=1 << 20):
    """Runs of short fragments (16 to 300 bytes, in random order) that continue each other in the destination between
    two longer ones, one run from every offset in a 128-byte line: a short fragment may lie entirely in the lines it
    shares with its two neighbours, or fill a line together with one of them, or be too short to reach the line's
    end, in which case three fragments meet in one line and nothing is shared."""
    rng = np.random.default_rng(seed)
    lengths = [16, 17, 31, 32, 47, 64, 100, 127, 128, 129, 200, 255, 256, 300]
    rows, dst = [], 0
    for start in range(128):
        dst = (dst + 127) // 128 * 128 + start
        run = [1000] + [int(x) for x in rng.permutation(lengths)[: int(rng.integers(3, len(lengths) + 1))]] + [1000]
        for ln in run:
            page = int(rng.integers(0, pool_bytes // 4096))
            rows.append((page * 4096 + int(rng.integers(0, 4096 - ln + 1)), ln, dst))
            dst += ln
        dst += 1
    return make_descs(rows), dst + 64


def test_short_fragments_in_the_shared_lines_of_their_neighbours(pkg, hip, oracle):
    pool = seeded_pool(1 << 20, 41)
    for seed in (42, 43):
        descs, dst_bytes = short_runs(seed)
        run_batch(pkg, hip, oracle, pool, descs, dst_bytes)
        run_batch(pkg, hip, oracle, pool, descs, dst_bytes, misalign=9)
