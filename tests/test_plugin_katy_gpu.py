"""The plugin on the GPU with the reference's other flow scheduler and its socket thread:
NCCL_GPUDIRECTTCPX_SCHED_ALG=KATY (src/flow_mapper.h:67-135, src/net_tcpx.cc:643-665) decides when the receive
comm has a flow free to take the next chunk, and NCCL_GPUDIRECTTCPX_AMD_HELPER_THREAD=1 moves recvmsg and the
descriptor builder to a thread of the comm's own (persistentSocketThread, src/net_tcpx.cc:252-384).  Bytes, pages
and slots must come out exactly as with the defaults."""
import ctypes
import os

import numpy as np
import pytest

import __graft_entry__ as graft
from conftest import GUARD, SENTINEL, first_difference

pytestmark = pytest.mark.gpu
FLAGS = {"NCCL_GPUDIRECTTCPX_SCHED_ALG": "KATY", "NCCL_GPUDIRECTTCPX_AMD_HELPER_THREAD": "1", "NCCL_GPUDIRECTTCPX_AMD_FLOWS": "8"}


@pytest.fixture(scope="module")
def env(pkg):
    import torch

    lib = pkg.plugin_lib()
    saved = {k: os.environ.get(k) for k in FLAGS}
    os.environ.update(FLAGS)
    assert lib.tcpxSetDeviceOpsForTesting(None) == 0  # the real HIP layer
    assert lib.tcpxInit(None) == 0
    base = ctypes.c_void_p()
    assert lib.tcpxSynthArenaCreate(0, 512 << 20, ctypes.byref(base)) == 0
    from nccl_plugin_gpudirecttcpx_amd import synth_driver

    class Env:
        pass

    e = Env()
    e.pkg, e.lib, e.driver, e.arena, e.torch, e.hip = pkg, lib, synth_driver, base.value, torch, pkg.hip_layer()
    yield e
    assert lib.tcpxFinalize() == 0
    for k, v in saved.items():
        if v is None:
            os.environ.pop(k, None)
        else:
            os.environ[k] = v


@pytest.mark.parametrize("config,native", [(2, False), (3, True), (2, True)])
def test_katy_scheduler_and_socket_thread_full_size(env, oracle, config, native):
    torch = env.torch
    sched = ctypes.c_void_p()
    assert env.lib.tcpxFlowSchedCreate(None, ctypes.byref(sched)) == 0
    assert env.lib.tcpxFlowSchedAlg(sched) == 1, "the comm's policy must be KATY"
    env.lib.tcpxFlowSchedDestroy(sched)
    wl = env.pkg.Workload(config, seed=0xCA71 + config)
    info = wl.info
    pool = np.empty(info.pool_bytes, dtype=np.uint8)
    wl.fill_window(0, pool)
    env.pkg.check(env.hip.tcpxuCopyToDevice(0, env.arena, pool.ctypes.data, pool.nbytes), "tcpxuCopyToDevice")
    expect = np.full(GUARD + info.dst_bytes + GUARD, SENTINEL, dtype=np.uint8)
    graft.oracle_unpack(oracle, expect[GUARD : GUARD + info.dst_bytes], pool, np.ascontiguousarray(wl.descs))
    dst = torch.full((GUARD + info.dst_bytes + GUARD,), SENTINEL, dtype=torch.uint8, device="cuda:0")
    torch.cuda.synchronize()
    comm = env.driver.RecvComm(0)
    print("katy case: config %d, %d requests, %s driver, 8 flows, socket thread" % (config, info.n_requests, "native" if native else "python"), flush=True)
    if native:
        env.driver.run_workload_native(comm, wl, dst.data_ptr() + GUARD, window=8)
    else:
        env.driver.run_workload(comm, wl, dst.data_ptr() + GUARD, n_flows=8, window=8, timeout_s=60)
    got = dst.cpu().numpy()
    assert comm.outstanding_pages() == 0
    head, tail, _ = comm.queue_state()
    assert head == tail == info.n_requests
    comm.close()
    assert first_difference(got, expect) is None, "first (index, got, want, count): %r" % (first_difference(got, expect),)
