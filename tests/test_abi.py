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
    [("tcpx_unpack_hip.h", "libtcpxu_hip.so"), ("tcpx_synth.h", "libtcpx_synth.so"), ("tcpx_plugin.h", "libnccl-net.so")],
)
def test_every_declared_symbol_is_exported(pkg, header, lib):
    names = declared_functions(header)
    assert len(names) >= 7, names
    handle = ctypes.CDLL(os.path.join(pkg.LIB_DIR, lib))
    missing = [n for n in names if not hasattr(handle, n)]
    assert not missing, "%s does not export %s" % (lib, missing)


def test_plugin_table_symbol(pkg):
    lib = pkg.plugin_lib()
    assert ctypes.string_at(lib.table.name) == b"GPUDirectTCPX_v7"


def test_bindings_cover_the_headers(pkg):
    pkg.hip_layer(), pkg.synth_lib(), pkg.plugin_lib()  # _bind raises if a prototype names a missing symbol
    import nccl_plugin_gpudirecttcpx_amd as m

    for header, table in (("tcpx_unpack_hip.h", m._HIP_PROTOTYPES), ("tcpx_synth.h", m._SYNTH_PROTOTYPES), ("tcpx_plugin.h", m._PLUGIN_PROTOTYPES)):
        assert set(declared_functions(header)) == set(table), header


def test_struct_sizes_match_the_headers(pkg):
    assert ctypes.sizeof(pkg.LoadMeta) == 16 and ctypes.sizeof(pkg.SynthFrag) == 16
    assert ctypes.sizeof(pkg.SynthRequest) == 32 and ctypes.sizeof(pkg.SynthInfo) == 48
    assert ctypes.sizeof(pkg.EngineConfig) == 16 and ctypes.sizeof(pkg.StreamItem) == 32
    assert ctypes.sizeof(pkg.NetDeviceHandle) == 32 and ctypes.sizeof(pkg.NetProperties) == 56
    assert ctypes.sizeof(pkg.FlowStats) == 32 and ctypes.sizeof(pkg.CommStats) == 40 and ctypes.sizeof(pkg.TraceEvent) == 24


def test_missing_library_raises(pkg, monkeypatch, tmp_path):
    monkeypatch.setattr(pkg, "LIB_DIR", str(tmp_path))
    monkeypatch.setattr(pkg, "_cache", {})
    with pytest.raises(pkg.MissingLibrary):
        pkg.hip_layer()
