"""MI355X-native receive-side unpack path of a GPUDirect-TCPX style net plugin: ctypes view of the C-ABI.

This package holds no compute of its own.  It loads the in-tree shared libraries built from ``csrc/`` and
exposes their C entry points (``include/tcpx_unpack_hip.h``, ``include/tcpx_unpack_bench.h``,
``include/tcpx_synth.h``, ``include/tcpx_plugin.h``) with argument types attached, so tests and the benchmark call exactly what a C or
C++ host would call.  There is no CPU fallback: if a library is missing, loading raises.

The directory name carries a hyphen, so it is imported through ``__graft_entry__.load_package()`` under the
module name ``nccl_plugin_gpudirecttcpx_amd``.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_DIR = os.environ.get("TCPX_AMD_LIB_DIR") or os.path.join(_HERE, "lib")  # override: an alternative build
REPO_ROOT = os.path.dirname(_HERE)

SUCCESS, DEVICE_ERROR, SYSTEM_ERROR, INTERNAL_ERROR, INVALID_ARGUMENT, INVALID_USAGE = 0, 1, 2, 3, 4, 5
IN_PROGRESS = 7

QUEUE_DEPTH = 16
SLOT_PAGES = 2048
PAGE_SIZE = 4096

c_u8p = ctypes.POINTER(ctypes.c_uint8)


class LoadMeta(ctypes.Structure):
    """``tcpxuLoadMeta`` / NCCL ``union loadMeta`` (reference fields: src/sock/tcpx.h:178-180)."""

    _fields_ = [("src_off", ctypes.c_uint32), ("len", ctypes.c_uint32), ("dst_off", ctypes.c_uint64)]


class SynthFrag(ctypes.Structure):
    _fields_ = [
        ("frag_offset", ctypes.c_uint32),
        ("frag_size", ctypes.c_uint32),
        ("frag_token", ctypes.c_uint32),
        ("flow", ctypes.c_uint32),
    ]


class SynthRequest(ctypes.Structure):
    _fields_ = [
        ("first_desc", ctypes.c_uint64),
        ("dst_off", ctypes.c_uint64),
        ("n_descs", ctypes.c_uint32),
        ("bytes", ctypes.c_uint32),
        ("window", ctypes.c_uint32),
        ("reserved", ctypes.c_uint32),
    ]


class SynthInfo(ctypes.Structure):
    _fields_ = [
        ("pool_bytes", ctypes.c_uint64),
        ("payload_bytes", ctypes.c_uint64),
        ("dst_bytes", ctypes.c_uint64),
        ("n_descs", ctypes.c_uint64),
        ("n_requests", ctypes.c_uint32),
        ("n_flows", ctypes.c_uint32),
        ("n_windows", ctypes.c_uint32),
        ("dst_misalign", ctypes.c_uint32),
    ]


class EngineConfig(ctypes.Structure):
    _fields_ = [
        ("ring_entries", ctypes.c_uint32),
        ("workgroups", ctypes.c_uint32),
        ("descs_per_ticket", ctypes.c_uint32),
        ("spin_limit", ctypes.c_uint32),
    ]


class StreamItem(ctypes.Structure):
    _fields_ = [
        ("bounce_base", ctypes.c_void_p),
        ("dst_base", ctypes.c_void_p),
        ("descs_host", ctypes.c_void_p),
        ("n_descs", ctypes.c_uint32),
        ("payload_bytes", ctypes.c_uint32),
    ]


class Submission(ctypes.Structure):
    """tcpxuSubmission (include/tcpx_unpack_hip.h)."""

    _fields_ = [
        ("bounce_base", ctypes.c_void_p),
        ("dst_base", ctypes.c_void_p),
        ("descs_dev", ctypes.c_void_p),
        ("done_flag_dev", ctypes.c_void_p),
        ("done_value", ctypes.c_uint64),
        ("n_descs", ctypes.c_uint32),
        ("payload_bytes", ctypes.c_uint32),
    ]


class EngineStats(ctypes.Structure):
    """tcpxuEngineStats (include/tcpx_unpack_hip.h)."""

    _fields_ = [
        ("launches", ctypes.c_uint64),
        ("submissions", ctypes.c_uint64),
        ("leader_polls", ctypes.c_uint64),
        ("leader_entries", ctypes.c_uint64),
        ("leader_deep_polls", ctypes.c_uint64),
    ]


class StreamSplit(ctypes.Structure):
    """tcpxuStreamSplit (include/tcpx_unpack_bench.h)."""

    _fields_ = [
        ("publish_ns", ctypes.c_double),
        ("wall_ns", ctypes.c_double),
        ("published", ctypes.c_uint64),
        ("publish_calls", ctypes.c_uint64),
        ("passes", ctypes.c_uint64),
    ]


class MissingLibrary(RuntimeError):
    pass


def _load(name):
    path = os.path.join(LIB_DIR, name)
    if not os.path.exists(path):
        raise MissingLibrary(
            "%s is not built: run `python -c 'import __graft_entry__ as g; g.build()'` in %s" % (path, REPO_ROOT)
        )
    return ctypes.CDLL(path, mode=ctypes.RTLD_GLOBAL)


_HIP_PROTOTYPES = {
    # name: (restype, argtypes)
    "tcpxuLastError": (ctypes.c_char_p, []),
    "tcpxuDeviceCount": (ctypes.c_int, [ctypes.POINTER(ctypes.c_int)]),
    "tcpxuDeviceInfo": (ctypes.c_int, [ctypes.c_int, ctypes.c_char_p, ctypes.c_size_t, ctypes.POINTER(ctypes.c_int)]),
    "tcpxuArenaCreate": (ctypes.c_int, [ctypes.c_int, ctypes.c_size_t, ctypes.POINTER(ctypes.c_void_p)]),
    "tcpxuArenaDestroy": (ctypes.c_int, [ctypes.c_int, ctypes.c_void_p]),
    "tcpxuDeviceAlloc": (ctypes.c_int, [ctypes.c_int, ctypes.c_size_t, ctypes.POINTER(ctypes.c_void_p)]),
    "tcpxuDeviceFree": (ctypes.c_int, [ctypes.c_int, ctypes.c_void_p]),
    "tcpxuCopyToDevice": (ctypes.c_int, [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t]),
    "tcpxuCopyToHost": (ctypes.c_int, [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t]),
    "tcpxuFillDevice": (ctypes.c_int, [ctypes.c_int, ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t]),
    "tcpxuDeviceSynchronize": (ctypes.c_int, [ctypes.c_int]),
    "tcpxuMappedAlloc": (
        ctypes.c_int,
        [ctypes.c_int, ctypes.c_size_t, ctypes.POINTER(ctypes.c_void_p), ctypes.POINTER(ctypes.c_void_p)],
    ),
    "tcpxuMappedFree": (ctypes.c_int, [ctypes.c_int, ctypes.c_void_p]),
    "tcpxuVisibleAlloc": (
        ctypes.c_int,
        [ctypes.c_int, ctypes.c_size_t, ctypes.POINTER(ctypes.c_void_p), ctypes.POINTER(ctypes.c_void_p)],
    ),
    "tcpxuVisibleFree": (ctypes.c_int, [ctypes.c_int, ctypes.c_void_p]),
    "tcpxuVisibleFlush": (None, []),
    "tcpxuUnpackBatch": (
        ctypes.c_int,
        [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint64, ctypes.c_void_p],
    ),
    "tcpxuEngineCreate": (
        ctypes.c_int,
        [ctypes.c_int, ctypes.POINTER(EngineConfig), ctypes.POINTER(ctypes.c_void_p)],
    ),
    "tcpxuEngineStart": (ctypes.c_int, [ctypes.c_void_p]),
    "tcpxuEngineStop": (ctypes.c_int, [ctypes.c_void_p, ctypes.POINTER(ctypes.c_double)]),
    "tcpxuEngineDestroy": (ctypes.c_int, [ctypes.c_void_p]),
    "tcpxuEngineSubmit": (
        ctypes.c_int,
        [
            ctypes.c_void_p,
            ctypes.c_void_p,
            ctypes.c_void_p,
            ctypes.c_void_p,
            ctypes.c_uint32,
            ctypes.c_void_p,
            ctypes.c_uint64,
        ],
    ),
    "tcpxuEngineSubmitSized": (
        ctypes.c_int,
        [
            ctypes.c_void_p,
            ctypes.c_void_p,
            ctypes.c_void_p,
            ctypes.c_void_p,
            ctypes.c_uint32,
            ctypes.c_uint64,
            ctypes.c_void_p,
            ctypes.c_uint64,
        ],
    ),
    "tcpxuUnpackSlotNoAlloc": (
        ctypes.c_int,
        [
            ctypes.c_int,
            ctypes.c_void_p,
            ctypes.c_void_p,
            ctypes.c_void_p,
            ctypes.c_uint32,
            ctypes.c_void_p,
            ctypes.c_uint64,
            ctypes.c_void_p,
        ],
    ),
    "tcpxuEngineCompleted": (ctypes.c_int, [ctypes.c_void_p, ctypes.POINTER(ctypes.c_uint64)]),
    "tcpxuEngineSubmitMany": (ctypes.c_int, [ctypes.c_void_p, ctypes.POINTER(Submission), ctypes.c_uint32, ctypes.POINTER(ctypes.c_uint32)]),
    "tcpxuEngineEnableStamps": (ctypes.c_int, [ctypes.c_void_p, ctypes.POINTER(ctypes.c_double)]),
    "tcpxuEngineReadStamps": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_uint64, ctypes.c_uint32, ctypes.POINTER(ctypes.c_uint64)]),
    "tcpxuEngineGetStats": (ctypes.c_int, [ctypes.c_void_p, ctypes.POINTER(EngineStats)]),
    "tcpxuEngineRunning": (ctypes.c_int, [ctypes.c_void_p, ctypes.POINTER(ctypes.c_int)]),
    "tcpxuEngineGetConfig": (ctypes.c_int, [ctypes.c_void_p, ctypes.POINTER(EngineConfig)]),
    "tcpxuEngineDevice": (ctypes.c_int, [ctypes.c_void_p, ctypes.POINTER(ctypes.c_int)]),
    "tcpxuEngineTicketPlan": (
        ctypes.c_int,
        [
            ctypes.c_uint32,
            ctypes.c_uint32,
            ctypes.c_uint32,
            ctypes.c_uint32,
            ctypes.c_uint64,
            ctypes.POINTER(ctypes.c_uint32),
            ctypes.POINTER(ctypes.c_uint32),
            ctypes.POINTER(ctypes.c_uint32),
        ],
    ),
}

_BENCH_PROTOTYPES = {
    "tcpxuBenchLastError": (ctypes.c_char_p, []),
    "tcpxuCopyKernelLaunch": (ctypes.c_int, [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]),
    "tcpxuStreamLastSplit": (ctypes.c_int, [ctypes.POINTER(StreamSplit)]),
    "tcpxuEngineRunStamped": (
        ctypes.c_int,
        [
            ctypes.c_void_p,
            ctypes.POINTER(StreamItem),
            ctypes.c_uint64,
            ctypes.c_uint32,
            ctypes.c_uint32,
            ctypes.POINTER(ctypes.c_double),
            ctypes.POINTER(ctypes.c_double),
            ctypes.POINTER(ctypes.c_double),
        ],
    ),
    "tcpxuUnpackBatchTimed": (
        ctypes.c_int,
        [
            ctypes.c_int,
            ctypes.c_void_p,
            ctypes.c_void_p,
            ctypes.c_void_p,
            ctypes.c_uint64,
            ctypes.c_int,
            ctypes.c_int,
            ctypes.POINTER(ctypes.c_double),
        ],
    ),
    "tcpxuGatherKernelTimed": (
        ctypes.c_int,
        [
            ctypes.c_int,
            ctypes.c_void_p,
            ctypes.c_void_p,
            ctypes.c_void_p,
            ctypes.c_uint32,
            ctypes.c_uint32,
            ctypes.c_int,
            ctypes.c_int,
            ctypes.POINTER(ctypes.c_double),
        ],
    ),
    "tcpxuCopyKernelTimed": (
        ctypes.c_int,
        [
            ctypes.c_int,
            ctypes.c_void_p,
            ctypes.c_void_p,
            ctypes.c_size_t,
            ctypes.c_int,
            ctypes.c_int,
            ctypes.POINTER(ctypes.c_double),
        ],
    ),
    "tcpxuEngineStream": (
        ctypes.c_int,
        [
            ctypes.c_void_p,
            ctypes.POINTER(StreamItem),
            ctypes.c_uint64,
            ctypes.c_uint32,
            ctypes.c_uint32,
            ctypes.POINTER(ctypes.c_double),
            ctypes.POINTER(ctypes.c_double),
        ],
    ),
    "tcpxuEngineStreamWarm": (
        ctypes.c_int,
        [
            ctypes.c_void_p,
            ctypes.POINTER(StreamItem),
            ctypes.c_uint64,
            ctypes.c_uint64,
            ctypes.c_uint32,
            ctypes.c_uint32,
            ctypes.POINTER(ctypes.c_double),
            ctypes.POINTER(ctypes.c_double),
        ],
    ),
    "tcpxuEngineRunTimed": (
        ctypes.c_int,
        [
            ctypes.c_void_p,
            ctypes.POINTER(StreamItem),
            ctypes.c_uint64,
            ctypes.c_uint64,
            ctypes.c_uint32,
            ctypes.c_uint32,
            ctypes.POINTER(ctypes.c_double),
            ctypes.POINTER(ctypes.c_double),
            ctypes.POINTER(ctypes.c_double),
        ],
    ),
    "tcpxuEngineRunWindow": (
        ctypes.c_int,
        [
            ctypes.c_void_p,
            ctypes.POINTER(StreamItem),
            ctypes.c_uint64,
            ctypes.c_uint64,
            ctypes.c_uint64,
            ctypes.c_uint32,
            ctypes.c_uint32,
            ctypes.POINTER(ctypes.c_double),
            ctypes.POINTER(ctypes.c_double),
            ctypes.POINTER(ctypes.c_double),
        ],
    ),
}

_SYNTH_PROTOTYPES = {
    "tcpxSynthCreate": (
        ctypes.c_int,
        [ctypes.c_int, ctypes.c_uint64, ctypes.c_uint32, ctypes.POINTER(ctypes.c_void_p)],
    ),
    "tcpxSynthDestroy": (None, [ctypes.c_void_p]),
    "tcpxSynthGetInfo": (ctypes.c_int, [ctypes.c_void_p, ctypes.POINTER(SynthInfo)]),
    "tcpxSynthDescs": (ctypes.POINTER(LoadMeta), [ctypes.c_void_p]),
    "tcpxSynthFrags": (ctypes.POINTER(SynthFrag), [ctypes.c_void_p]),
    "tcpxSynthRequests": (ctypes.POINTER(SynthRequest), [ctypes.c_void_p]),
    "tcpxSynthFillWindow": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_uint32, ctypes.c_void_p]),
    "tcpxSynthCpuRoundTripNs": (ctypes.c_int, [ctypes.c_int, ctypes.c_int, ctypes.c_uint32, ctypes.POINTER(ctypes.c_double)]),
}


def _bind(lib, prototypes):
    for name, (restype, argtypes) in prototypes.items():
        fn = getattr(lib, name)  # AttributeError if the library does not export it
        fn.restype = restype
        fn.argtypes = argtypes
    return lib


class NetProperties(ctypes.Structure):
    """ncclNetProperties_v7_t (include/nccl_net_v7.h)."""

    _fields_ = [
        ("name", ctypes.c_char_p),
        ("pciPath", ctypes.c_char_p),
        ("guid", ctypes.c_uint64),
        ("ptrSupport", ctypes.c_int),
        ("speed", ctypes.c_int),
        ("port", ctypes.c_int),
        ("latency", ctypes.c_float),
        ("maxComms", ctypes.c_int),
        ("maxRecvs", ctypes.c_int),
        ("netDeviceType", ctypes.c_int),
        ("netDeviceVersion", ctypes.c_int),
    ]


class NetDeviceHandle(ctypes.Structure):
    """ncclNetDeviceHandle_v7_t."""

    _fields_ = [
        ("netDeviceType", ctypes.c_int),
        ("netDeviceVersion", ctypes.c_int),
        ("handle", ctypes.c_void_p),
        ("size", ctypes.c_size_t),
        ("needsProxyProgress", ctypes.c_int),
    ]


class FlowStats(ctypes.Structure):
    """tcpxFlowStats (include/tcpx_plugin.h)."""

    _fields_ = [("flow_id", ctypes.c_uint64), ("rx_ctrl_done_cnt", ctypes.c_uint64), ("rx_cnt", ctypes.c_uint64), ("rx_slow_cnt", ctypes.c_uint64)]


class CommStats(ctypes.Structure):
    """tcpxCommStats (include/tcpx_plugin.h)."""

    _fields_ = [
        ("rx_ctrl_slow_cnt", ctypes.c_uint64),
        ("unpack_cnt", ctypes.c_uint64),
        ("unpack_slow_cnt", ctypes.c_uint64),
        ("unpack_ns", ctypes.c_uint64),
        ("trace_dropped", ctypes.c_uint64),
        ("socket_thread_cpus", ctypes.c_uint64),
        ("max_slots_at_gpu", ctypes.c_uint64),
    ]


class TraceEvent(ctypes.Structure):
    """tcpxTraceEvent (include/tcpx_plugin.h)."""

    _fields_ = [
        ("kind", ctypes.c_char),
        ("passive", ctypes.c_uint8),
        ("state", ctypes.c_uint16),
        ("reserved", ctypes.c_uint32),
        ("object", ctypes.c_uint64),
        ("timestamp", ctypes.c_int64),
    ]


CLOCK_FN = ctypes.CFUNCTYPE(ctypes.c_uint64)

_V = ctypes.c_void_p
_VP = ctypes.POINTER(ctypes.c_void_p)
_IP = ctypes.POINTER(ctypes.c_int)
NET_V7_MEMBERS = [
    "name", "init", "devices", "getProperties", "listen", "connect", "accept", "regMr", "regMrDmaBuf", "deregMr",
    "isend", "irecv", "iflush", "test", "closeSend", "closeRecv", "closeListen", "getDeviceMr", "irecvConsumed",
]  # fmt: skip


class NetV7(ctypes.Structure):
    """ncclNet_v7_t as 19 pointer-sized members, in the reference's order (src/nccl_plugin.cc:22-42)."""

    _fields_ = [(m, ctypes.c_void_p) for m in NET_V7_MEMBERS]


_PLUGIN_PROTOTYPES = {
    "tcpxInit": (ctypes.c_int, [_V]),
    "tcpxFinalize": (ctypes.c_int, []),
    "tcpxDevices": (ctypes.c_int, [_IP]),
    "tcpxGetProperties": (ctypes.c_int, [ctypes.c_int, ctypes.POINTER(NetProperties)]),
    "tcpxListen": (ctypes.c_int, [ctypes.c_int, _V, _VP]),
    "tcpxConnect_v5": (ctypes.c_int, [ctypes.c_int, _V, _VP, _V]),
    "tcpxAccept_v5": (ctypes.c_int, [_V, _VP, ctypes.POINTER(ctypes.POINTER(NetDeviceHandle))]),
    "tcpxRegMr": (ctypes.c_int, [_V, _V, ctypes.c_int, ctypes.c_int, _VP]),
    "tcpxDeregMr": (ctypes.c_int, [_V, _V]),
    "tcpxIsend_v5": (ctypes.c_int, [_V, _V, ctypes.c_int, ctypes.c_int, _V, _VP]),
    "tcpxIrecv_v5": (ctypes.c_int, [_V, ctypes.c_int, _VP, _IP, _IP, _VP, _VP]),
    "tcpxIflush_v5": (ctypes.c_int, [_V, ctypes.c_int, _VP, _IP, _VP, _VP]),
    "tcpxTest": (ctypes.c_int, [_V, _IP, _IP]),
    "tcpxClose": (ctypes.c_int, [_V]),
    "tcpxCloseListen": (ctypes.c_int, [_V]),
    "tcpxGetDeviceMr": (ctypes.c_int, [_V, _V, _VP]),
    "tcpxIrecvConsumed": (ctypes.c_int, [_V, ctypes.c_int, _V]),
    "tcpxSynthArenaCreate": (ctypes.c_int, [ctypes.c_int, ctypes.c_size_t, _VP]),
    "tcpxSynthCtrlSend": (
        ctypes.c_int,
        [_V, ctypes.c_uint16, ctypes.c_uint16, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32],
    ),
    "tcpxSynthDeliver": (ctypes.c_int, [_V, ctypes.c_uint32, _V, ctypes.c_uint32]),
    "tcpxSynthSetRecvmsgLimit": (ctypes.c_int, [_V, ctypes.c_uint32]),
    "tcpxSynthRunRequests": (
        ctypes.c_int,
        [_V, _V, _V, ctypes.c_uint32, _V, ctypes.c_uint64, ctypes.c_uint32, ctypes.c_uint32, ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_double)],
    ),
    "tcpxSynthOutstandingPages": (ctypes.c_int, [_V, ctypes.POINTER(ctypes.c_uint64)]),
    "tcpxDebugQueueState": (
        ctypes.c_int,
        [_V, ctypes.POINTER(ctypes.c_uint64), ctypes.POINTER(ctypes.c_uint64), ctypes.POINTER(ctypes.c_uint32 * 5)],
    ),
    "tcpxDebugSlot": (ctypes.c_int, [_V, ctypes.c_uint32, _VP, ctypes.POINTER(ctypes.c_uint64)]),
    "tcpxSetDeviceOpsForTesting": (ctypes.c_int, [_V]),
    "tcpxSetFailStopForTesting": (ctypes.c_int, [ctypes.c_int]),
    "tcpxGetFlowStats": (ctypes.c_int, [_V, ctypes.c_uint32, ctypes.POINTER(FlowStats)]),
    "tcpxGetCommStats": (ctypes.c_int, [_V, ctypes.POINTER(CommStats)]),
    "tcpxTraceDrain": (
        ctypes.c_int,
        [_V, ctypes.POINTER(TraceEvent), ctypes.c_uint32, ctypes.c_uint32, ctypes.POINTER(ctypes.c_uint32)],
    ),
    "tcpxTraceFormat": (ctypes.c_int, [ctypes.POINTER(TraceEvent), ctypes.c_char_p, ctypes.c_size_t]),
    "tcpxSetClockForTesting": (ctypes.c_int, [_V]),
    "tcpxFlowSchedCreate": (ctypes.c_int, [ctypes.c_char_p, ctypes.POINTER(_V)]),
    "tcpxFlowSchedAlg": (ctypes.c_int, [_V]),
    "tcpxFlowSchedReset": (None, [_V]),
    "tcpxFlowSchedHasFlow": (ctypes.c_int, [_V]),
    "tcpxFlowSchedSchedule": (None, [_V, ctypes.c_int, ctypes.c_int]),
    "tcpxFlowSchedPick": (ctypes.c_int, [_V]),
    "tcpxFlowSchedDestroy": (None, [_V]),
}

NCCL_PTR_HOST, NCCL_PTR_CUDA = 1, 2
CTRL_NORMAL, CTRL_INLINE = 0, 1

_cache = {}


def hip_layer():
    """``libtcpxu_hip.so`` with prototypes attached.  Loading does not need a GPU; calling does."""
    if "hip" not in _cache:
        _cache["hip"] = _bind(_load("libtcpxu_hip.so"), _HIP_PROTOTYPES)
    return _cache["hip"]


def bench_layer():
    """``libtcpxu_bench.so``: measurement helpers on top of the HIP layer (include/tcpx_unpack_bench.h)."""
    if "bench" not in _cache:
        hip_layer()  # its dependency, loaded first so that the symbols resolve whatever the search path
        _cache["bench"] = _bind(_load("libtcpxu_bench.so"), _BENCH_PROTOTYPES)
    return _cache["bench"]


def synth_lib():
    if "synth" not in _cache:
        _cache["synth"] = _bind(_load("libtcpx_synth.so"), _SYNTH_PROTOTYPES)
    return _cache["synth"]


def plugin_lib():
    """``libnccl-net.so`` with prototypes attached, plus ``.table``: the exported ``ncclNetPlugin_v7``."""
    if "plugin" not in _cache:
        lib = _bind(_load("libnccl-net.so"), _PLUGIN_PROTOTYPES)
        lib.table = NetV7.in_dll(lib, "ncclNetPlugin_v7")
        _cache["plugin"] = lib
    return _cache["plugin"]


class HipError(RuntimeError):
    def __init__(self, fn, rc, msg):
        super().__init__("%s failed with result %d: %s" % (fn, rc, msg))
        self.rc = rc


def check(rc, fn="call"):
    if rc != SUCCESS:
        msg = hip_layer().tcpxuLastError().decode(errors="replace")
        if "bench" in _cache:
            msg = (_cache["bench"].tcpxuBenchLastError().decode(errors="replace") + " | " + msg).strip(" |")
        raise HipError(fn, rc, msg)


class Workload:
    """A generated workload (numpy views into memory owned by the C object)."""

    def __init__(self, config, seed=0xC0FFEE00, shrink=0):
        import numpy as np

        self._lib = synth_lib()
        handle = ctypes.c_void_p()
        rc = self._lib.tcpxSynthCreate(config, seed, shrink, ctypes.byref(handle))
        if rc != 0:
            raise ValueError("tcpxSynthCreate(config=%r, shrink=%r) -> %d" % (config, shrink, rc))
        self._h = handle
        self.config, self.seed, self.shrink = config, seed, shrink
        self.info = SynthInfo()
        self._lib.tcpxSynthGetInfo(self._h, ctypes.byref(self.info))
        n = self.info.n_descs
        self.desc_dtype = np.dtype([("src_off", "<u4"), ("len", "<u4"), ("dst_off", "<u8")])
        self.frag_dtype = np.dtype([("frag_offset", "<u4"), ("frag_size", "<u4"), ("frag_token", "<u4"), ("flow", "<u4")])
        self.req_dtype = np.dtype(
            [("first_desc", "<u8"), ("dst_off", "<u8"), ("n_descs", "<u4"), ("bytes", "<u4"), ("window", "<u4"), ("reserved", "<u4")]
        )
        self.descs = self._view(self._lib.tcpxSynthDescs(self._h), n, self.desc_dtype)
        self.frags = self._view(self._lib.tcpxSynthFrags(self._h), n, self.frag_dtype)
        self.requests = self._view(self._lib.tcpxSynthRequests(self._h), self.info.n_requests, self.req_dtype)

    @staticmethod
    def _view(ptr, n, dtype):
        import numpy as np

        if n == 0:
            return np.zeros(0, dtype=dtype)
        buf = (ctypes.c_uint8 * (n * dtype.itemsize)).from_address(ctypes.addressof(ptr.contents))
        return np.frombuffer(buf, dtype=dtype)

    def fill_window(self, window, pool):
        """Writes pool generation `window` into the numpy uint8 array `pool` (length pool_bytes)."""
        assert pool.nbytes == self.info.pool_bytes and pool.flags["C_CONTIGUOUS"]
        rc = self._lib.tcpxSynthFillWindow(self._h, window, pool.ctypes.data_as(ctypes.c_void_p))
        if rc != 0:
            raise ValueError("tcpxSynthFillWindow -> %d" % rc)

    def close(self):
        if self._h:
            self.descs = self.frags = self.requests = None
            self._lib.tcpxSynthDestroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
