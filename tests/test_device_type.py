"""Who copies, and how connections pair up (no GPU; the device is tests/emu).

NCCL_GPUDIRECTTCPX_AMD_DEVICE_TYPE=unpack is the reference's division of labour (src/net_tcpx.cc:725-744,
1354-1357, 1452-1471): properties and device handle say UNPACK version 7, test() reports done once the descriptor
count is published, nothing is submitted to the engine, and whoever holds the device handle copies.  Here the
"consumer kernel" is the CPU oracle reading the published slot.  The default type, host, is what the other plugin
tests run.  listen / connect / accept: accept hands out a comm only for a connection made through the listener's
handle (src/net_tcpx.cc:746-769).
"""
import ctypes

import numpy as np
import pytest

import __graft_entry__ as graft
from plugin_common import expected_bytes
from test_observability import Session

INTERNAL_ERROR, SYSTEM_ERROR = 3, 2


def unpack_session(pkg, value="unpack"):
    return Session(pkg, {"NCCL_GPUDIRECTTCPX_AMD_DEVICE_TYPE": value})


def test_unpack_type_publishes_and_leaves_the_copy_to_the_consumer(pkg, oracle):
    with unpack_session(pkg) as s:
        p = pkg.NetProperties()
        assert s.lib.tcpxGetProperties(0, ctypes.byref(p)) == 0
        assert (p.netDeviceType, p.netDeviceVersion, p.maxRecvs, p.ptrSupport) == (1, 7, 1, 3)
        h = s.comm.dev_handle
        assert (h.netDeviceType, h.netDeviceVersion, h.size, h.needsProxyProgress) == (1, 7, 24, 1)
        # the 24-byte device handle: {meta, bounce_buf, head = -1} (src/devcomm/nccl/unpack1.cu:54-63)
        raw = (ctypes.c_uint64 * 3).from_address(h.handle)
        arena = np.frombuffer((ctypes.c_uint8 * (16 << 20)).from_address(raw[1]), dtype=np.uint8)
        assert raw[0] != 0 and raw[2] == 2**64 - 1
        assert s.emu.emu_counter(4) == 0, "the engine must not be started in the unpack type"

        wl = pkg.Workload(2, seed=0xDE71, shrink=5)
        assert wl.info.pool_bytes <= arena.nbytes
        pool = arena[: wl.info.pool_bytes]
        wl.fill_window(0, pool)
        dst = np.full(int(wl.info.dst_bytes), 0xA5, dtype=np.uint8)
        mh = s.comm.reg(dst.ctypes.data, dst.nbytes)
        submitted_before = s.emu.emu_counter(0)
        for i, r in enumerate(wl.requests):
            first, n, total, off = int(r["first_desc"]), int(r["n_descs"]), int(r["bytes"]), int(r["dst_off"])
            rc, req = s.comm.irecv(dst.ctypes.data + off, total, mh)
            assert rc == 0
            s.driver.feed_request(s.comm, wl.frags[first : first + n], total, 4)
            for _ in range(10000):
                rc, done, _ = s.comm.test(req)
                assert rc == 0
                if done:
                    break
            assert done, "request %d never reported done" % i
            # done means published: the count is in the slot, and not one byte has been copied
            descs, cnt = s.comm.slot(i % 16)
            assert cnt == n and np.all(dst[off : off + total] == 0xA5)
            # the consumer's turn: slot descriptors (relative to the bounce buffer and to this request's buffer)
            graft.oracle_unpack(oracle, dst[off : off + total], pool, np.ascontiguousarray(descs[:cnt]))
            assert s.comm.iflush(dst.ctypes.data + off, req, mh) == (0, total)
            assert s.comm.consumed(req) == 0
        assert s.emu.emu_counter(0) == submitted_before, "nothing may be submitted to the engine"
        assert np.array_equal(dst, expected_bytes(pool, wl.frags, wl.requests, dst.nbytes))
        assert s.comm.outstanding_pages() == 0 and s.comm_stats().unpack_cnt == len(wl.requests)
        s.comm.dereg(mh)


@pytest.mark.parametrize("value,want_type", [("UNPACK", 1), ("host", 0), ("Host", 0), ("gpu", 0), ("", 0)])
def test_device_type_values(pkg, value, want_type):
    with unpack_session(pkg, value) as s:
        p = pkg.NetProperties()
        assert s.lib.tcpxGetProperties(0, ctypes.byref(p)) == 0 and p.netDeviceType == want_type
        assert s.comm.dev_handle.netDeviceType == want_type
        assert any("DEVICE_TYPE=gpu ignored" in w for w in s.warnings) == (value == "gpu")


def test_accept_pairs_with_connect(pkg):
    with unpack_session(pkg, "host") as s:
        lib = s.lib
        handle = ctypes.create_string_buffer(128)
        lc = ctypes.c_void_p()
        assert lib.tcpxListen(0, handle, ctypes.byref(lc)) == 0
        rc_comm, sc1, sc2 = ctypes.c_void_p(), ctypes.c_void_p(), ctypes.c_void_p()
        # not connected: success and no comm, as often as asked (src/net_tcpx.cc:761-769 checks *recvComm)
        for _ in range(3):
            rc_comm.value = 0xDEAD
            assert lib.tcpxAccept_v5(lc, ctypes.byref(rc_comm), None) == 0 and not rc_comm.value
        # two peers connect through copies of the handle; exactly two accepts find them
        copy = ctypes.create_string_buffer(handle.raw, 128)
        assert lib.tcpxConnect_v5(0, handle, ctypes.byref(sc1), None) == 0 and sc1.value
        assert lib.tcpxConnect_v5(0, copy, ctypes.byref(sc2), None) == 0 and sc2.value
        comms = []
        for _ in range(2):
            assert lib.tcpxAccept_v5(lc, ctypes.byref(rc_comm), None) == 0 and rc_comm.value
            comms.append(rc_comm.value)
        assert comms[0] != comms[1]
        assert lib.tcpxAccept_v5(lc, ctypes.byref(rc_comm), None) == 0 and not rc_comm.value
        # a connection to another listener does not show up here
        other = ctypes.create_string_buffer(128)
        lc2, sc3 = ctypes.c_void_p(), ctypes.c_void_p()
        assert lib.tcpxListen(0, other, ctypes.byref(lc2)) == 0 and other.raw != handle.raw
        assert lib.tcpxConnect_v5(0, other, ctypes.byref(sc3), None) == 0
        assert lib.tcpxAccept_v5(lc, ctypes.byref(rc_comm), None) == 0 and not rc_comm.value
        assert lib.tcpxAccept_v5(lc2, ctypes.byref(rc_comm), None) == 0 and rc_comm.value
        comms.append(rc_comm.value)
        # a closed listener refuses; a handle that tcpxListen did not write is an error
        assert lib.tcpxCloseListen(lc2) == 0
        sc4 = ctypes.c_void_p()
        assert lib.tcpxConnect_v5(0, other, ctypes.byref(sc4), None) == SYSTEM_ERROR and not sc4.value
        junk = ctypes.create_string_buffer(b"\x01" * 128, 128)
        assert lib.tcpxConnect_v5(0, junk, ctypes.byref(sc4), None) == INTERNAL_ERROR
        for c in comms + [sc1.value, sc2.value, sc3.value]:
            assert lib.tcpxClose(c) == 0
        assert lib.tcpxCloseListen(lc) == 0
