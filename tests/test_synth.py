"""The synthetic fragment source: every workload obeys the devmem contract and its own description."""
import numpy as np
import pytest

SHRINKS = {1: 0, 2: 0, 3: 2, 4: 2, 5: 0}


@pytest.mark.parametrize("config", [1, 2, 3, 4, 5])
def test_workload_invariants(pkg, config):
    wl = pkg.Workload(config, seed=0xC0FFEE00 + config, shrink=SHRINKS[config])
    info, d, f, r = wl.info, wl.descs, wl.frags, wl.requests
    assert len(d) == len(f) == info.n_descs and len(r) == info.n_requests
    # descriptor i describes fragment i
    assert np.array_equal(d["src_off"], f["frag_offset"]) and np.array_equal(d["len"], f["frag_size"])
    assert np.array_equal(f["frag_token"], f["frag_offset"] // 4096)
    # devmem contract: at most one page, never across a page boundary, inside the pool
    assert (d["len"] <= 4096).all()
    assert ((d["src_off"] % 4096).astype(np.int64) + d["len"] <= 4096).all()
    assert (d["src_off"].astype(np.int64) + d["len"] <= info.pool_bytes).all()
    assert (f["flow"] < info.n_flows).all()
    # destination contiguous in arrival order
    assert int(d["len"].sum()) == info.payload_bytes == info.dst_bytes
    assert np.array_equal(d["dst_off"], np.cumsum(d["len"].astype(np.uint64)) - d["len"])
    # requests tile the descriptor list and respect the slice limits
    assert int(r["first_desc"][0]) == 0 and int(r["n_descs"].sum()) == info.n_descs
    assert np.array_equal(r["first_desc"][1:], np.cumsum(r["n_descs"].astype(np.uint64))[:-1])
    assert (r["bytes"] <= 4 << 20).all() and (r["n_descs"] <= 2048).all()
    for q in r:
        a, n = int(q["first_desc"]), int(q["n_descs"])
        assert int(d["len"][a : a + n].sum()) == int(q["bytes"])
        assert int(d["dst_off"][a]) == int(q["dst_off"]) if n else True


def test_contract_sizes_at_full_scale(pkg):
    spec = {
        1: dict(pool=16 << 20, payload=1 << 20, descs=256, reqs=1, mis=0),
        2: dict(pool=256 << 20, payload=8 << 20, reqs=2, mis=0),
        3: dict(pool=512 << 20, payload=128 << 20, descs=32768, reqs=2048, mis=0),
        4: dict(pool=1 << 30, payload=256 << 20, descs=65536, reqs=64, mis=0),
        5: dict(pool=256 << 20, payload=32 << 20, mis=3),
    }
    for config, s in spec.items():
        wl = pkg.Workload(config, seed=0xC0FFEE00 + config)
        i = wl.info
        assert (i.pool_bytes, i.payload_bytes, i.dst_misalign) == (s["pool"], s["payload"], s["mis"]), config
        if "descs" in s:
            assert i.n_descs == s["descs"]
        if "reqs" in s:
            assert i.n_requests == s["reqs"]
    # 8 MiB chunk: 90% full pages -> about 8 MiB / 3894 B descriptors; short ones between 64 and 4095 bytes
    wl = pkg.Workload(2, seed=1)
    ln = wl.descs["len"]
    assert 2050 <= len(ln) <= 2260
    assert 0.86 <= (ln == 4096).mean() <= 0.94
    inner = np.ones(len(ln), bool)
    inner[wl.requests["first_desc"][1:].astype(int) - 1] = False
    inner[-1] = False  # the last fragment of a request is cut to end the request exactly
    assert ln[inner].min() >= 64
    assert (wl.frags["flow"] == np.arange(len(ln)) % 4).all()
    # adversarial: 10% empty descriptors, pages distinct inside a request and reused between requests
    wl = pkg.Workload(5, seed=2)
    ln = wl.descs["len"]
    assert 0.08 <= (ln == 0).mean() <= 0.12 and ln.max() <= 4096
    assert wl.info.n_windows == wl.info.n_requests > 1
    tokens = wl.frags["frag_token"]
    for q in wl.requests:
        a, n = int(q["first_desc"]), int(q["n_descs"])
        assert len(np.unique(tokens[a : a + n])) == n
    assert len(np.unique(tokens)) < len(tokens)
    # permuted pages: all distinct
    for config in (1, 4):
        wl = pkg.Workload(config, seed=3)
        assert len(np.unique(wl.frags["frag_token"])) == wl.info.n_descs and (wl.descs["src_off"] % 4096 == 0).all()


def test_determinism_and_seed_sensitivity(pkg):
    a, b, c = pkg.Workload(2, seed=5), pkg.Workload(2, seed=5), pkg.Workload(2, seed=6)
    assert np.array_equal(a.descs, b.descs) and not np.array_equal(a.descs["src_off"][:100], c.descs["src_off"][:100])
    pa = np.empty(a.info.pool_bytes >> 6, dtype=np.uint8)
    small = pkg.Workload(2, seed=5, shrink=6)
    p1 = np.empty(small.info.pool_bytes, dtype=np.uint8)
    p2 = np.empty(small.info.pool_bytes, dtype=np.uint8)
    small.fill_window(0, p1)
    pkg.Workload(2, seed=5, shrink=6).fill_window(0, p2)
    assert np.array_equal(p1, p2) and len(np.unique(p1)) == 256
    assert abs(float(p1.mean()) - 127.5) < 2.0


def test_window_refill_touches_only_that_windows_pages(pkg):
    wl = pkg.Workload(5, seed=9, shrink=2)
    assert wl.info.n_windows >= 2
    pool = np.empty(wl.info.pool_bytes, dtype=np.uint8)
    wl.fill_window(0, pool)
    before = pool.copy()
    wl.fill_window(1, pool)
    changed = np.unique(np.flatnonzero(pool != before) // 4096)
    q = wl.requests[1]
    assert int(q["window"]) == 1
    pages = np.unique(wl.frags["frag_token"][int(q["first_desc"]) : int(q["first_desc"]) + int(q["n_descs"])])
    assert set(changed.tolist()) <= set(pages.tolist()) and len(changed) >= 0.9 * len(pages)
    with pytest.raises(ValueError):
        wl.fill_window(wl.info.n_windows, pool)


def test_bad_arguments(pkg):
    with pytest.raises(ValueError):
        pkg.Workload(9)
    with pytest.raises(ValueError):
        pkg.Workload(1, shrink=40)


def test_cpu_round_trip_probe(pkg):
    """The probe that says how far apart two CPUs are (what a hand-over between two threads costs): a plausible
    time for a pair this process may use, errors for a pair it cannot be."""
    import ctypes
    import os

    synth, ns = pkg.synth_lib(), ctypes.c_double(-1.0)
    cpus = sorted(os.sched_getaffinity(0))
    before = os.sched_getaffinity(0)
    if len(cpus) >= 2:
        assert synth.tcpxSynthCpuRoundTripNs(cpus[0], cpus[1], 2000, ctypes.byref(ns)) == 0
        assert 5.0 < ns.value < 1e6  # a cache line there and back: tens of nanoseconds to a few microseconds
    assert os.sched_getaffinity(0) == before  # the probe pins its own two threads, not the caller
    assert synth.tcpxSynthCpuRoundTripNs(cpus[0], cpus[0], 10, ctypes.byref(ns)) == 4
    assert synth.tcpxSynthCpuRoundTripNs(-1, cpus[0], 10, ctypes.byref(ns)) == 4
    assert synth.tcpxSynthCpuRoundTripNs(cpus[0], cpus[-1] + 1 if len(cpus) < 2 else cpus[1], 0, ctypes.byref(ns)) == 4
    assert synth.tcpxSynthCpuRoundTripNs(cpus[0], 100000, 10, ctypes.byref(ns)) == 4
    not_mine = next((c for c in range(1024) if c not in before), None)
    if not_mine is not None and not_mine < (os.cpu_count() or 0) + 64:
        assert synth.tcpxSynthCpuRoundTripNs(cpus[0], not_mine, 10, ctypes.byref(ns)) == 2
