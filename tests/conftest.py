import ctypes
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import __graft_entry__ as graft  # noqa: E402


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def _ensure_built():
    """Tests load what is built; they compile only if nothing is there."""
    pkg = graft.load_package()
    needed = [os.path.join(pkg.LIB_DIR, n) for n in ("libtcpxu_hip.so", "libtcpxu_bench.so", "libtcpx_synth.so", "libnccl-net.so")]
    needed.append(os.path.join(ROOT, "oracle", "liboracle.so"))
    needed.append(os.path.join(ROOT, "tests", "native", "bin", "plugin_dlopen_host"))
    if not all(os.path.exists(p) for p in needed):
        graft.build()
    return pkg


@pytest.fixture(scope="session")
def pkg():
    return _ensure_built()


@pytest.fixture(scope="session")
def oracle(pkg):
    return graft.load_oracle()


@pytest.fixture(scope="session")
def hip(pkg):
    return pkg.hip_layer()


@pytest.fixture(scope="session")
def benchlib(pkg):
    return pkg.bench_layer()


SENTINEL = 0xA5
GUARD = 256


def oracle_expected(oracle, pool, descs, dst_bytes, misalign=0):
    """Sentinel-filled destination with guard bands, unpacked by the CPU oracle.  Returns the whole buffer;
    the destination base is at GUARD + misalign."""
    buf = np.full(GUARD + misalign + dst_bytes + GUARD, SENTINEL, dtype=np.uint8)
    graft.oracle_unpack(oracle, buf[GUARD + misalign : GUARD + misalign + dst_bytes], pool, np.ascontiguousarray(descs))
    return buf


def make_descs(rows):
    """rows: iterable of (src_off, len, dst_off) -> structured array with the loadMeta layout."""
    dt = np.dtype([("src_off", "<u4"), ("len", "<u4"), ("dst_off", "<u8")])
    return np.array([tuple(r) for r in rows], dtype=dt).reshape(-1)


class GpuBuffers:
    """Device-side copies of a pool, a descriptor list and a sentinel-filled destination (torch is plumbing)."""

    def __init__(self, pool, descs, dst_bytes, misalign=0):
        import torch

        self.torch = torch
        self.misalign = misalign
        self.dst_bytes = dst_bytes
        self.pool = torch.from_numpy(pool).to("cuda:0")
        d = np.ascontiguousarray(descs)
        self.n = len(d)
        self.descs = torch.from_numpy(d.view(np.uint8).copy() if len(d) else np.zeros(16, np.uint8)).to("cuda:0")
        self.dst = torch.full((GUARD + misalign + dst_bytes + GUARD,), SENTINEL, dtype=torch.uint8, device="cuda:0")
        assert self.dst.data_ptr() % 256 == 0 and self.pool.data_ptr() % 4096 == 0 and self.descs.data_ptr() % 16 == 0
        torch.cuda.synchronize()

    @property
    def dst_base(self):
        return self.dst.data_ptr() + GUARD + self.misalign

    def reset(self):
        self.dst.fill_(SENTINEL)
        self.torch.cuda.synchronize()

    def result(self):
        return self.dst.cpu().numpy()


def first_difference(a, b):
    idx = np.flatnonzero(a != b)
    return None if idx.size == 0 else (int(idx[0]), int(a[idx[0]]), int(b[idx[0]]), int(idx.size))
