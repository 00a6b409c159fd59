"""Run by test_plugin_host.py (test_socket_thread_mode, test_socket_thread_binding,
test_katy_scheduler_receives_the_same_bytes) in its own process: the flags are read at tcpxInit.  Arguments, if any,
name the configs to run."""
import ctypes
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import __graft_entry__ as graft  # noqa: E402
from plugin_common import expected_bytes, load_emu  # noqa: E402

pkg = graft.load_package()
emu = load_emu()
lib = pkg.plugin_lib()
assert lib.tcpxSetDeviceOpsForTesting(emu.emu_ops()) == 0
assert lib.tcpxInit(None) == 0
arena_bytes = 64 << 20
base = ctypes.c_void_p()
assert lib.tcpxSynthArenaCreate(0, arena_bytes, ctypes.byref(base)) == 0
arena = np.frombuffer((ctypes.c_uint8 * arena_bytes).from_address(base.value), dtype=np.uint8)
from nccl_plugin_gpudirecttcpx_amd import synth_driver  # noqa: E402

cases = ((4, 4), (2, 2), (5, 3))
if len(sys.argv) > 1:  # only these configs
    cases = tuple(c for c in cases if str(c[0]) in sys.argv[1:])
for config, shrink in cases:
    wl = pkg.Workload(config, seed=31 + config, shrink=shrink)
    pool = arena[: wl.info.pool_bytes]
    wl.fill_window(0, pool)
    comm = synth_driver.RecvComm(0)
    buf = np.full(int(wl.info.dst_bytes), 0xA5, dtype=np.uint8)
    synth_driver.run_workload(comm, wl, buf.ctypes.data, n_flows=8, window=8)
    assert np.array_equal(buf, expected_bytes(pool, wl.frags, wl.requests, int(wl.info.dst_bytes))), config
    assert comm.outstanding_pages() == 0
    stats = pkg.CommStats()
    assert lib.tcpxGetCommStats(comm.comm, ctypes.byref(stats)) == 0
    print("socket thread cpus", stats.socket_thread_cpus)
    comm.close()
sched = ctypes.c_void_p()
assert lib.tcpxFlowSchedCreate(None, ctypes.byref(sched)) == 0
print("sched alg", lib.tcpxFlowSchedAlg(sched))
lib.tcpxFlowSchedDestroy(sched)
assert lib.tcpxFinalize() == 0
print("helper-thread case ok")
