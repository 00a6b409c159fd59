"""Shared pieces of the plugin tests: the emulated device (CPU runs) and expected-bytes helpers."""
import ctypes
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EMU_DIR = os.path.join(ROOT, "tests", "emu")
EMU_LIB = os.path.join(EMU_DIR, "libemu.so")


def build_emu():
    src = os.path.join(EMU_DIR, "emu_device_ops.c")
    oracle_src = os.path.join(ROOT, "oracle", "tcpx_oracle.c")
    inc = os.path.join(ROOT, "include")
    deps = [src, oracle_src] + [os.path.join(inc, f) for f in os.listdir(inc) if f.endswith(".h")]  # the ops table lives in a header
    if os.path.exists(EMU_LIB) and os.path.getmtime(EMU_LIB) >= max(os.path.getmtime(d) for d in deps):
        return
    subprocess.check_call(
        ["gcc", "-O1", "-g", "-fPIC", "-shared", "-Wall", "-I" + os.path.join(ROOT, "include"), "-o", EMU_LIB, src, oracle_src, "-pthread"]
    )


def load_emu():
    build_emu()
    lib = ctypes.CDLL(EMU_LIB)
    lib.emu_ops.restype = ctypes.c_void_p
    lib.emu_release.restype = ctypes.c_int
    lib.emu_release.argtypes = [ctypes.c_int]
    lib.emu_pending.restype = ctypes.c_int
    lib.emu_release_at.restype = ctypes.c_int
    lib.emu_release_at.argtypes = [ctypes.c_int]
    lib.emu_set_hold.argtypes = [ctypes.c_int]
    lib.emu_set_ring_full.argtypes = [ctypes.c_int]
    lib.emu_set_visible_off.argtypes = [ctypes.c_int]
    lib.emu_counter.restype = ctypes.c_uint64
    lib.emu_counter.argtypes = [ctypes.c_int]
    return lib


def expected_bytes(pool, frags, requests, dst_bytes, sentinel=0xA5):
    """What the receive buffers must hold: every request's fragments laid end to end at its dst_off.
    Independent of the plugin and of the C oracle: plain numpy slicing, fragment by fragment."""
    out = np.full(dst_bytes, sentinel, dtype=np.uint8)
    for r in requests:
        pos = int(r["dst_off"])
        first, n = int(r["first_desc"]), int(r["n_descs"])
        for f in frags[first : first + n]:
            off, size = int(f["frag_offset"]), int(f["frag_size"])
            out[pos : pos + size] = pool[off : off + size]
            pos += size
    return out
