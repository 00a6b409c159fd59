"""tcpxuUnpackSlotNoAlloc, the entry point that allocates nothing, against tcpxuEngineSubmit on the same slots,
through the C-ABI (GPU).

Two calls in a row share the library's fixed scratch memory, the second with a smaller slot than the first, so
what the first call left there (ticket records with the same stamps, counters at their final values) must not
leak into the second.  Output = the destination bytes with their guard bands and the completion word; the bar is
byte-exact, against the engine's output and against the CPU oracle.
"""
import ctypes

import numpy as np
import pytest

from conftest import GUARD, SENTINEL, GpuBuffers, first_difference, oracle_expected
from test_engine_gpu import Engine, Mapped

pytestmark = pytest.mark.gpu


def slots_of(pkg, config, seed, shrink=0):
    wl = pkg.Workload(config, seed=seed, shrink=shrink)
    pool = np.empty(wl.info.pool_bytes, dtype=np.uint8)
    wl.fill_window(0, pool)
    return wl, pool


def unpack_with_engine(pkg, hip, buf, mapped, slots):
    """The existing entry point: one tcpxuEngineSubmit per slot on a started engine."""
    e = Engine(pkg, hip)
    e.start()
    try:
        for i, (first, n) in enumerate(slots):
            e.submit(buf.pool.data_ptr(), buf.dst_base, mapped.desc_dev(first), n, mapped.flag_dev(i), 1000 + i)
            mapped.wait(i, 1000 + i)
    finally:
        e.stop()
        e.destroy()
    return buf.result(), [int(mapped.flags[i]) for i in range(len(slots))]


def unpack_without_allocating(pkg, hip, buf, mapped, slots, stream):
    import torch

    for i, (first, n) in enumerate(slots):
        print("no-alloc case: slot %d, first descriptor %d, %d descriptors" % (i, first, n), flush=True)
        rc = hip.tcpxuUnpackSlotNoAlloc(0, buf.pool.data_ptr(), buf.dst_base, mapped.desc_dev(first), n, mapped.flag_dev(i), 1000 + i, stream)
        pkg.check(rc, "tcpxuUnpackSlotNoAlloc")
    torch.cuda.synchronize()
    return buf.result(), [int(mapped.flags[i]) for i in range(len(slots))]


@pytest.mark.parametrize("config,seed,shrink", [(2, 0xA110C, 0), (5, 0xA110D, 2)])
def test_two_calls_in_a_row_match_the_engine(pkg, hip, oracle, config, seed, shrink):
    import torch

    wl, pool = slots_of(pkg, config, seed, shrink)
    info = wl.info
    reqs = [(int(r["first_desc"]), int(r["n_descs"])) for r in wl.requests]
    # first the largest slot, then a smaller one: a quarter of another request, so the second call writes fewer
    # tickets than the first left behind
    big = max(reqs, key=lambda r: r[1])
    other = next(r for r in reqs if r != big) if len(reqs) > 1 else big
    small = (other[0], max(1, other[1] // 4))
    slots = [big, small, (small[0] + small[1], 0)]  # and an empty slot, which still completes
    assert slots[0][1] > slots[1][1] > 0 and slots[0][1] <= pkg.SLOT_PAGES
    descs = np.ascontiguousarray(wl.descs)
    used = np.concatenate([descs[f : f + n] for f, n in slots])
    expect = oracle_expected(oracle, pool, used, info.dst_bytes, info.dst_misalign)

    buf = GpuBuffers(pool, descs, info.dst_bytes, info.dst_misalign)
    mapped = Mapped(pkg, hip, descs, len(slots))
    want_bytes, want_flags = unpack_with_engine(pkg, hip, buf, mapped, slots)
    assert first_difference(want_bytes, expect) is None  # the existing entry point agrees with the oracle

    buf.reset()
    for i in range(len(slots)):
        mapped.flags[i] = 0
    stream = torch.cuda.Stream()
    got_bytes, got_flags = unpack_without_allocating(pkg, hip, buf, mapped, slots, stream.cuda_stream)
    assert got_flags == want_flags == [1000, 1001, 1002]
    assert first_difference(got_bytes, want_bytes) is None, "first (index, got, want, count): %r" % (first_difference(got_bytes, want_bytes),)
    assert first_difference(got_bytes, expect) is None
    mapped.free()


def test_two_calls_captured_into_a_hip_graph_and_replayed(pkg, hip, oracle):
    """What the entry point is for: after one ordinary call (which looks up the scratch memory's address and loads the
    kernels' code, neither of which belongs under capture), two calls in a row -- a large slot, then a smaller one --
    are captured into a HIP graph on a caller's stream and replayed; every replay, with the pool refilled, the
    destination reset and the completion words cleared by ordinary eager work in between, must give the oracle's
    bytes for the pool of that replay."""
    import torch

    wl, pool = slots_of(pkg, 2, 0xA110F, shrink=0)
    info = wl.info
    reqs = [(int(r["first_desc"]), int(r["n_descs"])) for r in wl.requests]
    big = max(reqs, key=lambda r: r[1])
    other = next(r for r in reqs if r != big)
    slots = [big, (other[0], max(1, other[1] // 3))]
    descs = np.ascontiguousarray(wl.descs)
    used = np.concatenate([descs[f : f + n] for f, n in slots])
    buf = GpuBuffers(pool, descs, info.dst_bytes, info.dst_misalign)
    mapped = Mapped(pkg, hip, descs, len(slots))
    stream = torch.cuda.Stream()
    # the warm call, not captured
    pkg.check(hip.tcpxuUnpackSlotNoAlloc(0, buf.pool.data_ptr(), buf.dst_base, mapped.desc_dev(slots[1][0]), slots[1][1], mapped.flag_dev(1), 7, stream.cuda_stream), "tcpxuUnpackSlotNoAlloc")
    torch.cuda.synchronize()
    assert int(mapped.flags[1]) == 7
    graph = torch.cuda.CUDAGraph()
    print("no-alloc graph case: slots of %d and %d descriptors captured" % (slots[0][1], slots[1][1]), flush=True)
    with torch.cuda.graph(graph, stream=stream):
        s = torch.cuda.current_stream().cuda_stream
        for i, (first, n) in enumerate(slots):
            pkg.check(hip.tcpxuUnpackSlotNoAlloc(0, buf.pool.data_ptr(), buf.dst_base, mapped.desc_dev(first), n, mapped.flag_dev(i), 1000 + i, ctypes.c_void_p(s)), "tcpxuUnpackSlotNoAlloc")
    for replay in range(3):
        if replay:
            pool = np.roll(pool, 4099 * replay) ^ np.uint8(replay)
            buf.pool.copy_(torch.from_numpy(pool))
        buf.reset()
        for i in range(len(slots)):
            mapped.flags[i] = 0
        graph.replay()
        torch.cuda.synchronize()
        expect = oracle_expected(oracle, pool, used, info.dst_bytes, info.dst_misalign)
        got = buf.result()
        assert [int(mapped.flags[i]) for i in range(len(slots))] == [1000, 1001], "replay %d" % replay
        assert first_difference(got, expect) is None, "replay %d, first (index, got, want, count): %r" % (replay, first_difference(got, expect))
    mapped.free()


def test_no_completion_word_and_the_default_stream(pkg, hip, oracle):
    """Without a completion word stream order is the only signal; the scratch memory then takes the store."""
    wl, pool = slots_of(pkg, 1, 0xA110E, shrink=2)
    info = wl.info
    expect = oracle_expected(oracle, pool, wl.descs, info.dst_bytes, info.dst_misalign)
    buf = GpuBuffers(pool, wl.descs, info.dst_bytes, info.dst_misalign)
    print("no-alloc case: %d descriptors, no completion word, default stream" % info.n_descs, flush=True)
    pkg.check(hip.tcpxuUnpackSlotNoAlloc(0, buf.pool.data_ptr(), buf.dst_base, buf.descs.data_ptr(), info.n_descs, None, 0, None), "tcpxuUnpackSlotNoAlloc")
    pkg.check(hip.tcpxuDeviceSynchronize(0), "tcpxuDeviceSynchronize")
    assert first_difference(buf.result(), expect) is None


def test_sizes_beyond_the_scratch_memory_are_refused(pkg, hip):
    import torch

    d = torch.zeros(64, dtype=torch.uint8, device="cuda:0")
    p = d.data_ptr()
    assert hip.tcpxuUnpackSlotNoAlloc(0, p, p, p, pkg.SLOT_PAGES + 1, None, 0, None) == pkg.INVALID_ARGUMENT
    assert b"2048" in hip.tcpxuLastError()
    assert hip.tcpxuUnpackSlotNoAlloc(0, p, p, p + 8, 4, None, 0, None) == pkg.INVALID_ARGUMENT  # descriptors not 16-byte aligned
    assert hip.tcpxuUnpackSlotNoAlloc(0, p, p, p, 4, p + 4, 1, None) == pkg.INVALID_ARGUMENT  # completion word not 8-byte aligned
    assert hip.tcpxuUnpackSlotNoAlloc(0, p, p, p, 4, p, 0, None) == pkg.INVALID_ARGUMENT  # completion value zero
    assert hip.tcpxuUnpackSlotNoAlloc(0, None, p, p, 4, None, 0, None) == pkg.INVALID_ARGUMENT
    torch.cuda.synchronize()
    assert int(d.sum()) == 0  # nothing was launched
