"""The plugin's host code under AddressSanitizer + UndefinedBehaviorSanitizer and under ThreadSanitizer (no GPU).

tests/native/plugin_sanitize.cc links the plugin's sources with the emulated device operations and receives the
five workloads (reduced) with the socket thread off and on and with tracepoints drained by a second thread.
Sanitizers run on host code only; the GPU code is not part of these builds.
"""
import os
import subprocess

import pytest

from plugin_common import ROOT

CSRC = os.path.join(ROOT, "nccl-plugin-gpudirecttcpx_amd", "csrc")
SOURCES = [
    os.path.join(ROOT, "tests", "native", "plugin_sanitize.cc"),
    os.path.join(CSRC, "plugin", "net_tcpx_amd.cc"),
    os.path.join(CSRC, "plugin", "trace.cc"),
    os.path.join(CSRC, "plugin", "synth_driver.cc"),
    os.path.join(CSRC, "plugin", "devmem_socket.cc"),
    os.path.join(CSRC, "plugin", "unpack_queue.cc"),
    os.path.join(CSRC, "plugin", "device_ops.cc"),
    os.path.join(CSRC, "plugin", "nccl_plugin.cc"),
    os.path.join(CSRC, "synth", "fraggen.cc"),
]
C_SOURCES = [os.path.join(ROOT, "tests", "emu", "emu_device_ops.c"), os.path.join(ROOT, "oracle", "tcpx_oracle.c")]
OUT_DIR = os.path.join(ROOT, "tests", "native", "build")


def build(name, flags):
    os.makedirs(OUT_DIR, exist_ok=True)
    exe = os.path.join(OUT_DIR, name)
    headers = [os.path.join(CSRC, "plugin", h) for h in ("plugin_internal.h", "trace.h")]
    newest = max(os.path.getmtime(p) for p in SOURCES + C_SOURCES + headers)
    if os.path.exists(exe) and os.path.getmtime(exe) >= newest:
        return exe
    common = ["-O1", "-g", "-fno-omit-frame-pointer", "-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(CSRC, "plugin")] + flags
    objs = []
    for src in C_SOURCES:
        obj = os.path.join(OUT_DIR, name + "_" + os.path.basename(src) + ".o")
        subprocess.check_call(["gcc", "-c", src, "-o", obj] + common)
        objs.append(obj)
    subprocess.check_call(["g++", "-std=c++17", "-o", exe] + SOURCES + objs + common + ["-pthread", "-ldl"])
    return exe


@pytest.mark.parametrize(
    "name,flags,marker",
    [
        ("plugin_asan_ubsan", ["-fsanitize=address,undefined", "-fno-sanitize-recover=undefined"], "AddressSanitizer"),
        ("plugin_tsan", ["-fsanitize=thread"], "ThreadSanitizer"),
    ],
)
def test_plugin_host_code_is_clean(name, flags, marker):
    exe = build(name, flags)
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", TSAN_OPTIONS="halt_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    p = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env, timeout=600)
    assert p.returncode == 0, p.stdout[-4000:]
    assert "plugin sanitize run ok" in p.stdout
    assert marker not in p.stdout and "runtime error" not in p.stdout, p.stdout[-4000:]
