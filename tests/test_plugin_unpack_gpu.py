"""The reference's division of labour on the GPU (NCCL_GPUDIRECTTCPX_AMD_DEVICE_TYPE=unpack): the plugin publishes
descriptor counts, hands out the 24-byte device handle, and somebody else's kernel copies.  This test is that
somebody: it reads the handle back from device memory, follows handle.meta to the slot's count and descriptors --
what NCCL's consumer does with `struct unpackNetDeviceHandle` (src/devcomm/nccl/unpack1.cu:53-63,
src/net_tcpx.cc:1354-1357,1452-1471) -- and runs tcpxuUnpackBatch over exactly those device addresses.
"""
import ctypes
import os

import numpy as np
import pytest

import __graft_entry__ as graft
from conftest import GUARD, SENTINEL, first_difference

pytestmark = pytest.mark.gpu

SLOT_BYTES = 2048 * 16
CNT_OFFSET = 16 * SLOT_BYTES  # struct netUnpackMeta: mem[16][2048], then cnt[16]


@pytest.fixture(scope="module")
def env(pkg):
    import torch

    lib = pkg.plugin_lib()
    saved = os.environ.get("NCCL_GPUDIRECTTCPX_AMD_DEVICE_TYPE")
    os.environ["NCCL_GPUDIRECTTCPX_AMD_DEVICE_TYPE"] = "unpack"
    assert lib.tcpxSetDeviceOpsForTesting(None) == 0  # the real HIP layer
    assert lib.tcpxInit(None) == 0
    base = ctypes.c_void_p()
    assert lib.tcpxSynthArenaCreate(0, 256 << 20, ctypes.byref(base)) == 0
    from nccl_plugin_gpudirecttcpx_amd import synth_driver

    class Env:
        pass

    e = Env()
    e.pkg, e.lib, e.driver, e.arena, e.torch, e.hip = pkg, lib, synth_driver, base.value, torch, pkg.hip_layer()
    yield e
    assert lib.tcpxFinalize() == 0
    if saved is None:
        os.environ.pop("NCCL_GPUDIRECTTCPX_AMD_DEVICE_TYPE", None)
    else:
        os.environ["NCCL_GPUDIRECTTCPX_AMD_DEVICE_TYPE"] = saved


def test_a_consumer_unpacks_through_the_device_handle(env, oracle):
    pkg, hip, torch = env.pkg, env.hip, env.torch
    p = pkg.NetProperties()
    assert env.lib.tcpxGetProperties(0, ctypes.byref(p)) == 0
    assert (p.netDeviceType, p.netDeviceVersion, p.maxRecvs, p.ptrSupport, p.maxComms) == (1, 7, 1, 3, 65536)
    comm = env.driver.RecvComm(0)
    h = comm.dev_handle
    assert (h.netDeviceType, h.netDeviceVersion, h.size, h.needsProxyProgress) == (1, 7, 24, 1) and h.handle
    # the handle lives in device memory: {netUnpackMeta* meta, void* bounce_buf, u64 head = -1}
    raw = (ctypes.c_uint64 * 3)()
    pkg.check(hip.tcpxuCopyToHost(0, raw, h.handle, 24), "tcpxuCopyToHost")
    meta_dev, bounce, head = raw[0], raw[1], raw[2]
    assert meta_dev != 0 and bounce == env.arena and head == 2**64 - 1

    wl = pkg.Workload(2, seed=0xC0FFEE02)  # the 8 MiB chunk: two requests, 2 x 1078 descriptors or so
    info = wl.info
    pool = np.empty(info.pool_bytes, dtype=np.uint8)
    wl.fill_window(0, pool)
    pkg.check(hip.tcpxuCopyToDevice(0, env.arena, pool.ctypes.data, pool.nbytes), "tcpxuCopyToDevice")
    expect = np.full(GUARD + info.dst_bytes + GUARD, SENTINEL, dtype=np.uint8)
    graft.oracle_unpack(oracle, expect[GUARD : GUARD + info.dst_bytes], pool, np.ascontiguousarray(wl.descs))
    dst = torch.full((GUARD + info.dst_bytes + GUARD,), SENTINEL, dtype=torch.uint8, device="cuda:0")
    torch.cuda.synchronize()
    mh = comm.reg(dst.data_ptr() + GUARD, int(info.dst_bytes))
    for i, r in enumerate(wl.requests):
        first, n, total, off = int(r["first_desc"]), int(r["n_descs"]), int(r["bytes"]), int(r["dst_off"])
        data = dst.data_ptr() + GUARD + off
        rc, req = comm.irecv(data, total, mh)
        assert rc == 0
        env.driver.feed_request(comm, wl.frags[first : first + n], total, 4)
        for _ in range(100000):
            rc, done, _ = comm.test(req)
            assert rc == 0
            if done:
                break
        assert done
        # done = published.  Nothing has been copied: the plugin does not own the copy in this type.
        assert int((dst[GUARD + off : GUARD + off + total] != SENTINEL).sum()) == 0
        slot = i % 16
        cnt = ctypes.c_uint64()
        pkg.check(hip.tcpxuCopyToHost(0, ctypes.byref(cnt), meta_dev + CNT_OFFSET + 8 * slot, 8), "tcpxuCopyToHost")
        assert cnt.value == n, "meta->cnt[%d] read through the handle is %d, the request has %d fragments" % (slot, cnt.value, n)
        print("consumer case: slot %d, %d descriptors through the handle" % (slot, cnt.value), flush=True)
        # the consumer kernel: descriptors at &handle.meta->mem[slot], sources from handle.bounce_buf, destination
        # the request's own buffer (descriptor offsets are relative to it)
        pkg.check(hip.tcpxuUnpackBatch(0, bounce, data, meta_dev + SLOT_BYTES * slot, cnt.value, None), "tcpxuUnpackBatch")
        pkg.check(hip.tcpxuDeviceSynchronize(0), "tcpxuDeviceSynchronize")
        assert comm.iflush(data, req, mh) == (0, total)
        assert comm.consumed(req) == 0
    got = dst.cpu().numpy()
    assert comm.outstanding_pages() == 0
    head_q, tail_q, _ = comm.queue_state()
    assert head_q == tail_q == info.n_requests
    stats = pkg.CommStats()
    assert env.lib.tcpxGetCommStats(comm.comm, ctypes.byref(stats)) == 0 and stats.unpack_cnt == info.n_requests
    comm.dereg(mh)
    comm.close()
    assert first_difference(got, expect) is None, "first (index, got, want, count): %r" % (first_difference(got, expect),)
