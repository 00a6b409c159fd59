"""The plugin loaded the way NCCL loads it: a separate program (tests/native/plugin_dlopen_host.cc) that links
against nothing of this repository, dlopens libnccl-net.so, looks up `ncclNetPlugin_v7` and drives
init -> devices -> getProperties -> listen -> connect -> accept -> regMr -> irecv -> test -> iflush ->
irecvConsumed -> deregMr -> close* through the table's pointers only, on the committed fixture
tests/golden/plugin_host_fixture.bin, byte-exact (src/nccl_plugin.cc:22-42, src/net_tcpx.cc:746-769,921-954,
1311-1374,1477-1543).  On the CPU the device is tests/emu; on the GPU it is the HIP layer and the engine, and a
second run plays the clock to see the slowness watch and the tracepoints work against the real engine
(src/timeout.cc:52-75, src/work_queue.h:156-211).
"""
import os
import struct
import subprocess
import sys

import numpy as np
import pytest

import __graft_entry__ as graft
from plugin_common import EMU_LIB, ROOT, build_emu

sys.path.insert(0, os.path.join(ROOT, "oracle"))
import host_logic  # noqa: E402  (test infrastructure)

HOST = os.path.join(ROOT, "tests", "native", "bin", "plugin_dlopen_host")
FIXTURE = os.path.join(ROOT, "tests", "golden", "plugin_host_fixture.bin")


def run_host(pkg, extra, env=None):
    cmd = [HOST, os.path.join(pkg.LIB_DIR, "libnccl-net.so"), FIXTURE] + extra
    print("dlopen host case: %s" % " ".join(extra), flush=True)
    full_env = dict(os.environ)
    for k in list(full_env):
        if k.startswith("NCCL_GPUDIRECTTCPX_"):
            del full_env[k]
    full_env.update(env or {})
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=120, env=full_env)
    assert p.returncode == 0, (p.stdout[-2000:], p.stderr[-2000:])
    assert "dlopen host ok: 3 requests, 32 fragments" in p.stdout
    return p


def read_fixture():
    raw = open(FIXTURE, "rb").read()
    assert raw[:8] == b"TCPXFIX1"
    pool_bytes, dst_bytes, n_frags, n_requests, seed = struct.unpack_from("<IIIIQ", raw, 8)
    pos = 32
    frags = np.frombuffer(raw, dtype=np.dtype([("frag_offset", "<u4"), ("frag_size", "<u4"), ("frag_token", "<u4"), ("flow", "<u4")]), count=n_frags, offset=pos)
    pos += 16 * n_frags
    reqs = np.frombuffer(raw, dtype=np.dtype([("first_desc", "<u8"), ("dst_off", "<u8"), ("n_descs", "<u4"), ("bytes", "<u4"), ("window", "<u4"), ("reserved", "<u4")]), count=n_requests, offset=pos)
    pos += 32 * n_requests
    expect = np.frombuffer(raw, dtype=np.uint8, count=dst_bytes, offset=pos)
    assert pos + dst_bytes == len(raw)
    return pool_bytes, seed, frags, reqs, expect


def test_the_oracle_reproduces_the_fixture(pkg, oracle):
    """The fixture's expectation was made byte by byte in plain Python (tests/golden/make_plugin_fixture.py); the
    C oracle, given the descriptors the fixture's fragments stand for, must produce the same bytes."""
    sys.path.insert(0, os.path.join(ROOT, "tests", "golden"))
    import make_plugin_fixture

    pool_bytes, seed, frags, reqs, expect = read_fixture()
    pool = np.frombuffer(make_plugin_fixture.splitmix64_bytes(seed, pool_bytes), dtype=np.uint8)
    rows, pos = [], 0
    for r in reqs:
        pos = int(r["dst_off"])
        for f in frags[int(r["first_desc"]) : int(r["first_desc"]) + int(r["n_descs"])]:
            rows.append((int(f["frag_offset"]), int(f["frag_size"]), pos))
            pos += int(f["frag_size"])
    descs = np.array(rows, dtype=np.dtype([("src_off", "<u4"), ("len", "<u4"), ("dst_off", "<u8")]))
    got = np.full(len(expect), 0xA5, dtype=np.uint8)
    graft.oracle_unpack(oracle, got, pool, descs)
    assert np.array_equal(got, expect)
    assert [int(r["bytes"]) for r in reqs] == [int(frags["frag_size"][:24].sum()), 0, 8 * 4096]


def test_host_drives_the_plugin_through_the_table_on_the_emulated_device(pkg):
    build_emu()
    run_host(pkg, ["--emu", EMU_LIB])


@pytest.mark.gpu
def test_host_drives_the_plugin_through_the_table_on_the_gpu(pkg):
    p = run_host(pkg, [])
    assert "(HIP device)" in p.stdout and "netDeviceType 0" in p.stdout


@pytest.mark.gpu
def test_slowness_watch_and_tracepoints_against_the_real_engine(pkg):
    """The host moves the injected clock by 11 s between two polls of a request whose slot the engine holds
    (threshold 10 s): exactly one UNPACK report for that request, with its warning, and none for requests that a
    poll found finished; the state tracepoints drained afterwards follow the reference's order per object."""
    flags = {
        "NCCL_GPUDIRECTTCPX_TELEMETRY_ENABLE_TASK_LEVEL_STATS": "1",
        "NCCL_GPUDIRECTTCPX_TELEMETRY_ENABLE_REQUEST_LEVEL_STATS": "1",
    }
    p = run_host(pkg, ["--watch"], env=flags)
    caught = [l for l in p.stdout.splitlines() if l.startswith("watch: ")]
    assert len(caught) == 1 and int(caught[0].split()[1]) >= 1, p.stdout[-500:]
    warnings = [l for l in p.stderr.splitlines() if "unpack timeout" in l]
    assert len(warnings) == int(caught[0].split()[1])
    for w in warnings:  # the report names the slot, what the GPU was given and what the host was waiting for
        assert "descriptors" in w and "completion word" in w and "nanos 11000000000" in w, w
    per_object = {}
    for line in p.stdout.splitlines():
        if line.startswith("event "):
            _, kind, obj, state = line.split()
            per_object.setdefault((kind, obj), []).append(int(state))
    n_requests = n_tasks = 0
    for (kind, _), states in per_object.items():
        cycle = host_logic.REQUEST_TRACE_SEQUENCE if kind == "R" else host_logic.TASK_TRACE_SEQUENCE
        assert len(states) % len(cycle) == 0 and tuple(states) == cycle * (len(states) // len(cycle)), (kind, states)
        if kind == "R":
            n_requests += len(states) // len(cycle)
        else:
            n_tasks += len(states) // len(cycle)
    # every round receives the fixture's 3 requests; request 0 is 24 chunks of one fragment, request 2 is 4 chunks
    assert n_requests >= 3 and n_requests % 3 == 0 and n_tasks == (n_requests // 3) * 28
