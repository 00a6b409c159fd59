"""Pins the CPU oracle before anything is compared against it.

The reference holds no golden vector or test for this path, so the oracle is pinned by (a) hand-computed known
answers (tests/golden/host_logic_vectors.json), (b) fixtures whose expected bytes come from a byte-at-a-time
Python loop (tests/golden/unpack_vectors.npz, written by tests/golden/make_vectors.py), (c) an independent numpy
gather, and (d) invariants that a swapped operand, a dropped term or an off-by-one length would break.
"""
import json
import os
import sys

import numpy as np
import pytest

import __graft_entry__ as graft
from conftest import make_descs

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(os.path.dirname(HERE), "oracle"))
import host_logic  # noqa: E402

VECTORS = json.load(open(os.path.join(HERE, "golden", "host_logic_vectors.json")))


def run_oracle(oracle, pool, rows, dst_bytes, sentinel=0xA5):
    dst = np.full(dst_bytes, sentinel, dtype=np.uint8)
    graft.oracle_unpack(oracle, dst, pool, make_descs(rows))
    return dst


def test_unpack_hand_computed(oracle):
    for case in VECTORS["unpack"]:
        pool = (np.arange(case["pool_bytes"]) % 256).astype(np.uint8)
        got = run_oracle(oracle, pool, case["descs"], case["dst_bytes"], case["sentinel"])
        assert got.tolist() == case["expect"], case["ref"]


def test_unpack_brute_force_fixtures(oracle):
    z = np.load(os.path.join(HERE, "golden", "unpack_vectors.npz"))
    n_cases = len([k for k in z.files if k.startswith("pool_")])
    assert n_cases == 4
    for i in range(n_cases):
        pool, descs, expect = z["pool_%d" % i], z["descs_%d" % i], z["expect_%d" % i]
        got = run_oracle(oracle, pool, [tuple(int(x) for x in row) for row in descs], len(expect))
        assert np.array_equal(got, expect), i


def test_unpack_equals_numpy_gather(oracle):
    """Disjoint destinations: dst[index] = pool[index_src] built with fancy indexing, no loops over bytes."""
    rng = np.random.default_rng(5)
    pool = rng.integers(0, 256, size=1 << 18, dtype=np.uint8)
    lens = rng.integers(0, 4097, size=500)
    src = rng.integers(0, (1 << 18) - 4096, size=500)
    gaps = rng.integers(0, 9, size=500)
    dst_off = np.cumsum(lens + gaps) - lens
    total = int(dst_off[-1] + lens[-1] + 5)
    want = np.full(total, 0xA5, dtype=np.uint8)
    di = np.concatenate([np.arange(d, d + l) for d, l in zip(dst_off, lens)])
    si = np.concatenate([np.arange(s, s + l) for s, l in zip(src, lens)])
    want[di] = pool[si]
    got = run_oracle(oracle, pool, list(zip(src.tolist(), lens.tolist(), dst_off.tolist())), total)
    assert np.array_equal(got, want)


def test_unpack_invariants(oracle):
    rng = np.random.default_rng(6)
    pool = rng.integers(0, 256, size=1 << 16, dtype=np.uint8)
    # identity list reduces to memcpy
    n = 40000
    got = run_oracle(oracle, pool, [(0, n, 0)], n)
    assert np.array_equal(got, pool[:n])
    # source and destination are not interchangeable: a swap would fail this
    got = run_oracle(oracle, pool, [(100, 10, 0)], 200)
    assert np.array_equal(got[:10], pool[100:110]) and (got[10:] == 0xA5).all()
    # exactly len bytes: the byte before and the byte after keep the sentinel
    for ln in (1, 15, 16, 17, 4095, 4096):
        got = run_oracle(oracle, pool, [(7, ln, 3)], ln + 10)
        assert (got[:3] == 0xA5).all() and (got[3 + ln :] == 0xA5).all() and np.array_equal(got[3 : 3 + ln], pool[7 : 7 + ln])
    # zero-length descriptors are no-ops wherever they point
    got = run_oracle(oracle, pool, [(0, 0, 0), (65535, 0, 99), (5, 0, 50)], 100)
    assert (got == 0xA5).all()
    # disjoint destinations: any order of the list gives the same bytes
    rows = [(int(rng.integers(0, 60000)), 100, 100 * i) for i in range(50)]
    a = run_oracle(oracle, pool, rows, 5000)
    b = run_oracle(oracle, pool, rows[::-1], 5000)
    assert np.array_equal(a, b)
    # linearity: two halves applied one after the other equal the whole
    dst = np.full(5000, 0xA5, dtype=np.uint8)
    graft.oracle_unpack(oracle, dst, pool, make_descs(rows[:20]))
    graft.oracle_unpack(oracle, dst, pool, make_descs(rows[20:]))
    assert np.array_equal(dst, a)


def test_bounds_audit(oracle):
    d = make_descs([(0, 10, 0), (90, 11, 0), (0, 5, 96)])
    assert oracle.tcpx_oracle_first_out_of_bounds(d.ctypes.data, 3, 100, 100) == 1
    assert oracle.tcpx_oracle_first_out_of_bounds(d.ctypes.data, 1, 100, 100) == -1
    d = make_descs([(0, 5, 96)])
    assert oracle.tcpx_oracle_first_out_of_bounds(d.ctypes.data, 1, 100, 100) == 0
    assert oracle.tcpx_oracle_first_out_of_bounds(d.ctypes.data, 1, 100, 101) == -1


def test_timed_variant_moves_the_same_bytes(oracle):
    import ctypes

    rng = np.random.default_rng(8)
    pool = rng.integers(0, 256, size=1 << 16, dtype=np.uint8)
    rows = [(int(rng.integers(0, 60000)), int(rng.integers(0, 300)), 300 * i) for i in range(200)]
    want = run_oracle(oracle, pool, rows, 60000)
    for threads in (1, 3, 8):
        dst = np.full(60000, 0xA5, dtype=np.uint8)
        secs = (ctypes.c_double * 2)()
        d = make_descs(rows)
        assert oracle.tcpx_oracle_unpack_timed(dst.ctypes.data, pool.ctypes.data, d.ctypes.data, len(d), threads, 1, 2, secs) == 0
        assert np.array_equal(dst, want) and secs[0] > 0


def test_process_recv_cmsg_hand_computed():
    for case in VECTORS["process_recv_cmsg"]:
        scatter = [tuple(x) for x in case["scatter_before"]]
        pgtoks = [list(x) for x in case["pgtoks_before"]]
        ret = host_logic.process_recv_cmsg([tuple(f) for f in case["frags"]], scatter, pgtoks, case["offset"], case["dst_base_offset"])
        assert ret == case["returns"], case["ref"]
        assert scatter == [tuple(x) for x in case["scatter_after"]], case["ref"]
        assert pgtoks == case["pgtoks_after"], case["ref"]


def test_process_recv_cmsg_overflow_is_fatal():
    scatter, toks = [], []
    with pytest.raises(host_logic.TooManyFragments):
        host_logic.process_recv_cmsg([(i * 4096, 1, i) for i in range(2048)], scatter, toks, 0, 0)
    scatter, toks = [], []
    assert host_logic.process_recv_cmsg([(i * 4096, 1, i) for i in range(2047)], scatter, toks, 0, 0) == 2047
    assert toks == [[0, 2047]]


def test_slot_ring_hand_computed_and_invariants():
    ring = host_logic.SlotRing()
    for step in VECTORS["slot_ring"]["script"]:
        if step[0] == "next_free":
            assert ring.next_free() == step[1]
        else:
            assert ring.consume(step[1]) is step[2]
    # now head = 2, tail = 2: sixteen allocations succeed with indices 2..15,0,1 and the seventeenth does not
    assert [ring.next_free() for _ in range(16)] == list(range(2, 16)) + [0, 1]
    assert ring.next_free() is None
    assert 0 <= ring.tail - ring.head <= host_logic.QUEUE_DEPTH
    rng = np.random.default_rng(3)
    ring = host_logic.SlotRing()
    live = []
    for _ in range(2000):
        if rng.random() < 0.55:
            idx = ring.next_free()
            assert (idx is None) == (len(live) == 16)
            if idx is not None:
                assert idx == (ring.tail - 1) % 16
                live.append(idx)
        elif live:
            assert not ring.consume((live[0] + 1) % 16) or len(set(live)) == 1
            assert ring.consume(live.pop(0))
        assert 0 <= ring.tail - ring.head <= 16


def test_request_ring_invariants():
    rq = host_logic.RequestRing()
    rng = np.random.default_rng(4)
    for _ in range(5000):
        op = int(rng.integers(0, 5))
        if op == 4:
            if rq.has_free():
                rq.enqueue()
        elif rq.has(op + 1) if op < 4 else False:
            rq.advance(op + 1)
        assert rq.invariant()
    assert host_logic.request_done(0, -1, True) and not host_logic.request_done(0, -1, False)
    assert host_logic.request_done(10, 0, False) and not host_logic.request_done(10, 4, True)


def test_slowness_watch_hand_computed_and_invariants():
    """struct tcpxTimeoutDetection (src/timeout.cc:44-75) against looks worked out on paper, then what must hold
    for any sequence of looks: never on the first look, never before the threshold, reports at least
    `frequency` apart, nanos = time since the first look."""
    for case in VECTORS["slowness_watch"]:
        w = host_logic.SlownessWatch(case["threshold"], case["frequency"])
        for look in case["looks"]:
            if look == "reset":
                w.reset()
                continue
            now, warn, nanos = look
            assert w.should_warn(now) == (warn, nanos), (case["ref"], look)
    rng = np.random.default_rng(11)
    for threshold, frequency in ((1000, 300), (50, 5000), (1, 1)):
        w = host_logic.SlownessWatch(threshold, frequency)
        now, first, last_report, reports = 0, None, None, 0
        for i in range(3000):
            now += int(rng.integers(0, 400))
            if rng.random() < 0.01:
                w.reset()
                first, last_report = None, None
                continue
            warn, nanos = w.should_warn(now)
            if first is None:
                first = now
                assert not warn
                continue
            if warn:
                assert nanos == now - first and nanos >= threshold
                assert last_report is None or now - last_report >= frequency
                last_report = now
                reports += 1
            else:
                assert now - first < threshold or (last_report is not None and now - last_report < frequency)
        assert reports > 0


def test_slowness_switches_hand_computed():
    for case in VECTORS["slowness_switches"]:
        assert host_logic.parse_slowness_switches(case["text"], list(case["before"])) == case["after"], case["ref"]
    assert host_logic.parse_slowness_switches(None, [0, 1, 0, 0]) == [0, 1, 0, 0]


def test_flow_mappers_hand_computed():
    for case in VECTORS["flow_mapper"]:
        mapper = host_logic.FlowMapperKaty() if case["alg"] == "KATY" else host_logic.FlowMapperRR()
        assert host_logic.run_flow_script(mapper, case["script"]) == case["expect"], case["ref"]
    for case in VECTORS["sched_alg_flag"]:
        assert host_logic.sched_alg_from_flag(case["value"]) == case["alg"], case["value"]


def test_katy_serves_the_emptiest_flow_first():
    """What the policy is for, checked without its bitmap: per reset, at most two picks; each pick is a flow whose
    current priority (scheduled priority plus the times it was picked since) is minimal, lowest flow on a tie."""
    rng = np.random.default_rng(0xCA7)
    for _ in range(300):
        mapper = host_logic.FlowMapperKaty()
        prio = {int(f): int(rng.integers(0, host_logic.MAX_TASKS)) for f in rng.permutation(8)[: int(rng.integers(1, 9))]}
        for f, p in prio.items():
            mapper.schedule(f, p)
        for n in range(3):
            live = {f: p for f, p in prio.items() if p < host_logic.MAX_TASKS}
            got = mapper.pick()
            if n == 2 or not live:
                assert got == -1
                break
            best = min(live.values())
            assert got == min(f for f, p in live.items() if p == best)
            prio[got] += 1
