"""The C-ABI libraries load without a GPU and export every function their headers declare."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"typedef struct \w+ \{.*?\} \w+;", "", text, flags=re.S)  # function-pointer tables
    names = re.findall(r"\b(tcpx\w+)\s*\(", text)
    return sorted(set(n for n in names if not n.endswith("_t")))


@pytest.mark.parametrize(
    "header,lib",
    [
        ("tcpx_unpack_hip.h", "libtcpxu_hip.so"),
        ("tcpx_unpack_bench.h", "libtcpxu_bench.so"),
        ("tcpx_synth.h", "libtcpx_synth.so"),
        ("tcpx_plugin.h", "libnccl-net.so"),
    ],
)
def test_every_declared_symbol_is_exported(pkg, header, lib):
    names = declared_functions(header)
    assert len(names) >= 7, names
    pkg.hip_layer()  # libtcpxu_bench.so depends on it
    handle = ctypes.CDLL(os.path.join(pkg.LIB_DIR, lib))
    missing = [n for n in names if not hasattr(handle, n)]
    assert not missing, "%s does not export %s" % (lib, missing)


def test_plugin_table_symbol(pkg):
    lib = pkg.plugin_lib()
    assert ctypes.string_at(lib.table.name) == b"GPUDirectTCPX_v7"


def test_bindings_cover_the_headers(pkg):
    pkg.hip_layer(), pkg.bench_layer(), pkg.synth_lib(), pkg.plugin_lib()  # _bind raises if a prototype names a missing symbol
    import nccl_plugin_gpudirecttcpx_amd as m

    for header, table in (
        ("tcpx_unpack_hip.h", m._HIP_PROTOTYPES),
        ("tcpx_unpack_bench.h", m._BENCH_PROTOTYPES),
        ("tcpx_synth.h", m._SYNTH_PROTOTYPES),
        ("tcpx_plugin.h", m._PLUGIN_PROTOTYPES),
    ):
        assert set(declared_functions(header)) == set(table), header


def test_the_product_library_exports_no_measurement_helpers(pkg):
    """libtcpxu_hip.so is the product ABI: the timing and streaming helpers live in libtcpxu_bench.so only."""
    product = ctypes.CDLL(os.path.join(pkg.LIB_DIR, "libtcpxu_hip.so"))
    for name in declared_functions("tcpx_unpack_bench.h"):
        assert not hasattr(product, name), name


def test_ticket_plan_arithmetic(pkg):
    """The engine's ticket sizing on the host: sizes by backlog and payload hint, and the bound on a submission's
    descriptors that keeps all of its tickets within the ticket ring (65536 tickets)."""
    hip = pkg.hip_layer()
    per, nt, lim = ctypes.c_uint32(), ctypes.c_uint32(), ctypes.c_uint32()

    def plan(wgs, fixed, in_flight, n, nbytes=0):
        rc = hip.tcpxuEngineTicketPlan(wgs, fixed, in_flight, n, nbytes, ctypes.byref(per), ctypes.byref(nt), ctypes.byref(lim))
        return rc, per.value, nt.value, lim.value

    # by backlog (768 workers): below 13 descriptors per worker 8, below 18 12, below 100 14, then 16
    assert plan(769, 0, 1, 1078) == (0, 8, 135, 524288)
    assert plan(769, 0, 10, 1078)[1:3] == (12, 90)  # 10780 in flight: 14.04 per worker
    assert plan(769, 0, 16, 1078)[1:3] == (14, 77)  # one comm's sixteen slots: 22.5 per worker
    assert plan(769, 0, 64, 1078)[1:3] == (14, 77)  # 89.8 per worker
    assert plan(769, 0, 72, 1078)[1:3] == (16, 68)  # 101.1 per worker
    assert plan(513, 0, 64, 1078)[1:3] == (16, 68)  # the bench's four comms on 512 workers: 134.8 per worker
    # with the payload hint, short fragments get more descriptors per ticket: 32, 48, at most 64
    assert plan(769, 0, 64, 2048, 2048 * 4096)[1] == 16
    assert plan(769, 0, 64, 2048, 2048 * 2731)[1] == 16 and plan(769, 0, 64, 2048, 2048 * 2730)[1] == 32
    assert plan(769, 0, 64, 2048, 2048 * 2048)[1] == 32 and plan(769, 0, 64, 2048, 2048 * 2047)[1] == 48
    assert plan(769, 0, 64, 2048, 2048 * 1366)[1] == 48 and plan(769, 0, 64, 2048, 2048 * 1365)[1] == 64
    assert plan(769, 0, 64, 2048, 2048 * 100)[1:3] == (64, 32)
    # a small submission among many stays one ticket
    assert plan(769, 0, 8, 32)[1:3] == (32, 1) and plan(769, 0, 7, 32)[1:3] == (8, 4)
    # a fixed size is taken as it is
    assert plan(769, 5, 64, 1078)[1:3] == (5, 216)
    # the bound: every ticket of a submission must fit the ring of 65536 at once
    assert plan(769, 1, 1, 65536) == (0, 1, 65536, 65536)
    assert plan(769, 1, 1, 65537)[0] == pkg.INVALID_ARGUMENT
    assert plan(769, 0, 1, 524288)[0:3] == (0, 16, 32768) and plan(769, 0, 1, 524289)[0] == pkg.INVALID_ARGUMENT
    assert plan(65536, 0, 1, 524288)[0:3] == (0, 8, 65536)  # so many workers that the smallest size still applies
    assert plan(769, 16, 1, 1 << 20)[0:4] == (0, 16, 65536, 1 << 20) and plan(769, 64, 1, (1 << 20) + 1)[0] == pkg.INVALID_ARGUMENT
    for fixed in range(0, 65):
        for n in (1, 7, 8, 2048, lim.value):
            rc, p, t, limit = plan(3, fixed, 1, min(n, plan(3, fixed, 1, 1)[3]))
            assert rc == 0 and 1 <= t <= 65536 and p * t >= min(n, limit) > p * (t - 1)
    assert plan(1, 0, 1, 8)[0] == pkg.INVALID_ARGUMENT and plan(769, 65, 1, 8)[0] == pkg.INVALID_ARGUMENT


def test_struct_sizes_match_the_headers(pkg):
    assert ctypes.sizeof(pkg.LoadMeta) == 16 and ctypes.sizeof(pkg.SynthFrag) == 16
    assert ctypes.sizeof(pkg.SynthRequest) == 32 and ctypes.sizeof(pkg.SynthInfo) == 48
    assert ctypes.sizeof(pkg.EngineConfig) == 16 and ctypes.sizeof(pkg.StreamItem) == 32
    assert ctypes.sizeof(pkg.NetDeviceHandle) == 32 and ctypes.sizeof(pkg.NetProperties) == 56
    assert ctypes.sizeof(pkg.FlowStats) == 32 and ctypes.sizeof(pkg.CommStats) == 56 and ctypes.sizeof(pkg.TraceEvent) == 24


def test_missing_library_raises(pkg, monkeypatch, tmp_path):
    monkeypatch.setattr(pkg, "LIB_DIR", str(tmp_path))
    monkeypatch.setattr(pkg, "_cache", {})
    with pytest.raises(pkg.MissingLibrary):
        pkg.hip_layer()
