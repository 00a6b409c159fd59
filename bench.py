#!/usr/bin/env python3
"""Benchmark of the MI355X receive-side unpack path.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One "step" is the unpack of one 8 MiB chunk of the 4-flow workload (about 2155 descriptors of at most 4 KiB,
byte-unaligned sources in a 256 MiB bounce pool, contiguous destination), cut into two 4 MiB requests the way
NCCL slices an 8 MiB chunk.  The chunk goes through the persistent engine by the entry point the plugin calls
for every completed request (tcpxuEngineSubmitSized): descriptors are copied into a slot of a 16-deep mapped
ring, the slot is published, the GPU unpacks it and writes a completion word that the host polls -- no kernel
launch per request.  The descriptor lists are built beforehand here; the plugin builds them from control messages
and fragments as they arrive, one proxy thread per comm, and that whole path through ncclNet_v7 (host-bound: it
keeps as many slots at the GPU as its one thread can build ahead, `plugin_path.max_slots_at_gpu`) is reported
beside the headline as `plugin_path`, the drop-in figure.  One engine serves every receive
comm of the GPU; the headline keeps `--comms` (4) comms busy, each with the reference's queue depth of 16, taking
turns; the same run with a single comm is reported beside it (`single_comm`).  Successive steps use different
descriptor lists, different destinations (a ring of 128 chunks = 1 GiB, four times the 256 MiB Infinity Cache:
with a ring of 384 MiB part of the writes were still absorbed by the cache and the figure came out 3 % higher) and take
turns over `--pools` (64) copies of the 256 MiB bounce pool, so that sources come from HBM as well: a single pool
would sit in the Infinity Cache and be re-read by every chunk, which a pool that the NIC keeps refilling never
is, and with 16 copies a page was still re-read within the cache's reach often enough (about 3 % of the reads) to
show 1.6 points more than with 64 or 128 copies, where the figure no longer moves.  The figure is therefore HBM
traffic, not cache hits.  Bounce pool, descriptor lists and destinations are resident before the
timed region starts; nothing crosses PCIe during it except descriptors and completion words.

How the K steps are timed.  A step is 3 us of GPU work and a request's way through the engine about 10 us, so
K steps on their own would measure the filling and draining of the queues.  One launch of the persistent kernel
therefore carries: an untimed fill of at least two queues' worth of steps (never fewer than `--warmup`), then R
windows of exactly K steps each, back to back, then an untimed tail of one queue's worth that keeps the queues
full while the last window finishes.  Every completion is stamped by the host poller; a window is timed from the
completion of the step before it to the completion of its last step; `ms_per_step` x K is the MEDIAN window and
`value` the payload of K steps over it.  R is at least 50 and large enough that the launch carries 20000 steps or
more (60 ms), so that the launch's own duration (HIP events on the engine's stream: `roofline`) is the rate too,
with launch, ramp and stop well below 1 % of it; an untimed launch of the same length comes first, because the GPU
takes some milliseconds of load to reach the rate it then sustains.

Prints ONE JSON line: payload GB/s (`value`), the HBM roofline of the dominant kernel, p50/p99 request
completion latency, and a memcpy-per-descriptor CPU baseline timed on this machine's host cores.
"""
import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

import __graft_entry__ as graft

# HBM bytes moved per algorithmic byte (2 x fragment bytes) by unpack_engine_kernel on the headline workload, from
# the hardware counters FETCH_SIZE and WRITE_SIZE of one launch of `bench.py --one-launch --steps 20 --warmup 5`
# (two rocprofv3 --pmc runs), each scaled by what the same counter reads for the plain copy kernel of known size
# (`--calibrate-copy 256`); the summary with the counter values is profiles/unpack_engine_kernel_8MiB_chunk_pmc_traffic.txt.
TRAFFIC_PER_ALGORITHMIC_BYTE = 1.0079
HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published peak
# Steps in the untimed launch that precedes the measured one, and the least steps the windows of the measured launch
# add up to (60 ms each way): the rate the engine sustains shows only after some milliseconds of load.
WARM_LAUNCH_STEPS = 20000
MIN_TIMED_STEPS = 20000
CHUNK_CONFIG = 2


def percentile(values, q):
    return float(np.percentile(np.asarray(values, dtype=np.float64), q))


def cpu_baseline(oracle, descs, dst_bytes, pool, threads, budget_s):
    """memcpy-per-descriptor over a descriptor list, pool and destination in host memory: payload GB/s, iterations."""
    dst = np.empty(dst_bytes + 64, dtype=np.uint8)
    descs = np.ascontiguousarray(descs)
    payload = float(descs["len"].sum())
    probe = (ctypes.c_double * 3)()
    rc = oracle.tcpx_oracle_unpack_timed(dst.ctypes.data, pool.ctypes.data, descs.ctypes.data, len(descs), threads, 2, 3, probe)
    assert rc == 0
    per_iter = max(min(probe), 1e-6)
    iters = int(max(20, min(400000, budget_s / per_iter)))
    secs = (ctypes.c_double * iters)()
    rc = oracle.tcpx_oracle_unpack_timed(dst.ctypes.data, pool.ctypes.data, descs.ctypes.data, len(descs), threads, 5, iters, secs)
    assert rc == 0
    med = float(np.median(np.asarray(secs[:])))
    return payload / med / 1e9, iters


def plugin_path(pkg, hip, torch, workloads, pool, helper_thread=False, rx_bindings=None, what="8 MiB chunks"):
    """The same chunks through the whole plugin (libnccl-net.so): irecv -> control messages -> synthetic recvmsg
    with its control messages -> descriptor builder -> slot -> engine -> test() -> iflush -> irecvConsumed, driven by
    the request loop inside the library.  The host builds one descriptor per fragment here, so this is a host-bound
    figure: what the receive path costs per fragment on one proxy thread (or, with `helper_thread`, on the proxy
    thread plus the plugin's socket thread, NCCL_GPUDIRECTTCPX_AMD_HELPER_THREAD=1, which `rx_bindings` binds to
    CPUs: the value of NCCL_GPUDIRECTTCPX_RX_BINDINGS)."""
    from nccl_plugin_gpudirecttcpx_amd import synth_driver

    lib = pkg.plugin_lib()
    flags = {"NCCL_GPUDIRECTTCPX_AMD_HELPER_THREAD": "1" if helper_thread else "0", "NCCL_GPUDIRECTTCPX_RX_BINDINGS": rx_bindings}
    saved = {k: os.environ.get(k) for k in flags}
    for k, v in flags.items():
        if v is None:
            os.environ.pop(k, None)
        else:
            os.environ[k] = v
    try:
        if lib.tcpxInit(None) != 0:
            return {"error": "tcpxInit failed"}
    finally:
        for k, v in saved.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v
    base = ctypes.c_void_p()
    assert lib.tcpxSynthArenaCreate(0, pool.nbytes, ctypes.byref(base)) == 0
    pkg.check(hip.tcpxuCopyToDevice(0, base, pool.ctypes.data, pool.nbytes), "tcpxuCopyToDevice")
    comm = synth_driver.RecvComm(0)
    chunk_bytes = int(workloads[0].info.payload_bytes)
    dst = torch.empty(len(workloads) * chunk_bytes, dtype=torch.uint8, device="cuda:0")
    torch.cuda.synchronize()
    seconds, frags, lat = 0.0, 0, []
    for rep in range(3):  # the first pass warms up; the other two are timed
        # every chunk's requests in one list, sixteen posted at a time (the request ring's depth, src/work_queue.h:20)
        s, l = synth_driver.run_chunks_native(comm, workloads, dst.data_ptr(), chunk_bytes, window=16)
        if rep > 0:
            seconds += s
            frags += sum(int(wl.info.n_descs) for wl in workloads)
            lat.extend(l)
    stats = pkg.CommStats()
    lib.tcpxGetCommStats(comm.comm, ctypes.byref(stats))
    comm.close()
    assert lib.tcpxFinalize() == 0
    payload = 2 * len(workloads) * chunk_bytes
    return {
        "max_slots_at_gpu": int(stats.max_slots_at_gpu),
        "what": what + " through ncclNet_v7 (irecv/test/iflush/irecvConsumed) with the synthetic devmem socket, "
        + ("the proxy thread plus the plugin's socket thread" if helper_thread else "one proxy thread"),
        "payload_GBps": round(payload / seconds / 1e9, 2),
        "host_ns_per_fragment": round(seconds / frags * 1e9, 1),
        "request_fed_to_done_us_p50": round(percentile(lat, 50) * 1e6, 1),
        "publish_to_done_us_mean": round(stats.unpack_ns / max(stats.unpack_cnt, 1) / 1e3, 2),
    }


def batch_kernel_line(pkg, benchlib, torch, dev, chunks=128, pools=15, warmup=3, iters=20):
    """tcpxuUnpackBatch on `chunks` chunks of the headline workload as ONE descriptor list and one launch: chunk c
    reads copy c % pools of the 256 MiB pool (descriptor offsets are 32-bit: 15 copies stay below 4 GiB) and writes
    its own 8 MiB of the destination, so a launch moves chunks x 8 MiB each way with nothing read or written twice."""
    wls = [pkg.Workload(CHUNK_CONFIG, seed=0xC0FFEE02 + 7919 * i) for i in range(chunks)]
    info0 = wls[0].info
    pool_bytes, chunk_bytes = int(info0.pool_bytes), int(info0.payload_bytes)
    parts = []
    for c, wl in enumerate(wls):
        d = np.array(wl.descs, copy=True)
        d["src_off"] += np.uint32((c % pools) * pool_bytes)
        d["dst_off"] += np.uint64(c * chunk_bytes)
        parts.append(d)
    descs = np.ascontiguousarray(np.concatenate(parts))
    assert int(descs["src_off"].astype(np.int64).max()) + 4096 <= pools * pool_bytes <= 1 << 32
    pool_d = torch.empty(pools * pool_bytes, dtype=torch.uint8, device="cuda:0").random_(0, 256)
    dst_d = torch.empty(chunks * chunk_bytes + 512, dtype=torch.uint8, device="cuda:0")
    descs_d = torch.from_numpy(descs.view(np.uint8)).to("cuda:0")
    torch.cuda.synchronize()
    us = ctypes.c_double()
    pkg.check(
        benchlib.tcpxuUnpackBatchTimed(dev, pool_d.data_ptr(), dst_d.data_ptr() + 256, descs_d.data_ptr(), len(descs), warmup, iters, ctypes.byref(us)),
        "tcpxuUnpackBatchTimed",
    )
    payload = float(descs["len"].sum())
    return {
        "kernel": "unpack_batch_kernel",
        "workload": "%d chunks of 8 MiB in one launch, %d descriptors, sources in %d copies of the 256 MiB pool" % (chunks, len(descs), pools),
        "launches": warmup + iters,
        "bytes_per_launch": 2.0 * payload,
        "launch_us": round(us.value, 2),
        "rw_GBps": round(2.0 * payload / us.value / 1e3, 1),
        "frac": round(2.0 * payload / us.value / 1e3 / HBM_PEAK_GBPS, 4),
    }


def other_configs(pkg, torch, run, only=None):
    """The other workloads of the measurement contract through the same engine, 64 slots in flight.  A pass re-reads
    the pages of the pass `pool_copies` before it, so the copies are as many as it takes for 2 GiB of traffic to pass
    in between (eight times the Infinity Cache), except for config 1, which is cache-resident by construction.
    Their bytes are checked by the GPU tests; here they are only timed."""
    out = {}
    for cfg, passes, pool_copies, note in (
        (4, 120, 4, "bulk: one 256 MiB message of 65536 page-aligned 4 KiB fragments from a 1 GiB pool, as 64 requests of 4 MiB"),
        (5, 512, 32, "adversarial: 32 MiB, fragment lengths uniform in 1..4096, 10% empty descriptors, destination offset by 3 bytes"),
        (1, 2048, 1, "one 1 MiB message of 256 page-aligned fragments from a 16 MiB pool: cache-resident by construction"),
    ):
        if only is not None and cfg != only:
            continue
        wl = pkg.Workload(cfg, seed=0xC0FFEE00 + cfg)
        info = wl.info
        pool_bytes, dst_bytes = int(info.pool_bytes), int(info.dst_bytes)
        pool_d = torch.empty(pool_copies * pool_bytes, dtype=torch.uint8, device="cuda:0").random_(0, 256)
        stride = (dst_bytes + int(info.dst_misalign) + 4095) // 4096 * 4096
        n_dst = max(2, min(passes, (1 << 30) // stride))  # a ring of 1 GiB of destinations
        dst_d = torch.empty(n_dst * stride + 512, dtype=torch.uint8, device="cuda:0")
        torch.cuda.synchronize()
        descs = np.ascontiguousarray(wl.descs)
        reqs = [(int(r["first_desc"]), int(r["n_descs"])) for r in wl.requests]
        req_bytes = [int(descs["len"][f : f + n].sum()) for f, n in reqs]
        assert int((descs["dst_off"] + descs["len"]).max()) <= dst_bytes and int((descs["src_off"].astype(np.int64) + descs["len"]).max()) <= pool_bytes
        items = (pkg.StreamItem * (passes * len(reqs)))()
        i = 0
        for ps in range(passes):
            for (first, n), nbytes in zip(reqs, req_bytes):
                items[i].bounce_base = pool_d.data_ptr() + (ps % pool_copies) * pool_bytes
                # descriptor offsets count from the start of the message, whichever request they belong to
                items[i].dst_base = dst_d.data_ptr() + 256 + (ps % n_dst) * stride + int(info.dst_misalign)
                items[i].descs_host = descs.ctypes.data + 16 * first
                items[i].n_descs = n
                items[i].payload_bytes = nbytes
                i += 1
        wall_us, kernel_us, _ = run(items, 64, warmup_items=len(reqs))
        payload = float(info.payload_bytes) * (passes - 1)
        out["config_%d" % cfg] = {
            "what": note,
            "requests_per_pass": len(reqs),
            "descriptors_per_pass": int(info.n_descs),
            "payload_GBps": round(payload / (wall_us * 1e-6) / 1e9, 1),
            "rw_frac_of_hbm_peak": round(2.0 * payload / (wall_us * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
        }
        if only is not None:  # the whole launch, first pass included, as a profiler sees it
            out["config_%d" % cfg].update(passes=passes, bytes_per_launch=2.0 * float(info.payload_bytes) * passes, launch_us=round(kernel_us, 1))
        del pool_d, dst_d
    return out


def fragment_length_sweep(pkg, torch, run):
    """Fragments of one length through the engine, 64 slots in flight: 65536 fragments a pass, each the first `length`
    bytes of a 4 KiB page of a 256 MiB pool (4 copies in turn), laid end to end from a line boundary, in requests of
    2048 descriptors with their byte counts.  Sources and destinations sit on line boundaries, so nothing is shifted
    and no destination line is shared: what remains is the grain, to be read beside hbm_yardsticks' bare gathers."""
    out = {}
    n_frag, per_req, copies, passes = 65536, 2048, 4, 40
    pool_bytes = n_frag * 4096
    pool_d = torch.empty(copies * pool_bytes, dtype=torch.uint8, device="cuda:0").random_(0, 256)
    dst_d = torch.empty((1 << 30) + 8192, dtype=torch.uint8, device="cuda:0")
    torch.cuda.synchronize()
    for length in (1024, 2048, 4096):
        descs = np.zeros(n_frag, dtype=np.dtype([("src_off", "<u4"), ("len", "<u4"), ("dst_off", "<u8")]))
        descs["src_off"] = np.arange(n_frag, dtype=np.int64) * 4096
        descs["len"] = length
        descs["dst_off"] = np.arange(n_frag, dtype=np.int64) * length
        total = n_frag * length
        n_dst = (1 << 30) // total
        n_req = n_frag // per_req
        items = (pkg.StreamItem * (passes * n_req))()
        i = 0
        for ps in range(passes):
            for r in range(n_req):
                items[i].bounce_base = pool_d.data_ptr() + (ps % copies) * pool_bytes
                items[i].dst_base = dst_d.data_ptr() + 256 + (ps % n_dst) * total
                items[i].descs_host = descs.ctypes.data + 16 * r * per_req
                items[i].n_descs = per_req
                items[i].payload_bytes = per_req * length
                i += 1
        wall_us, _, _ = run(items, 64, warmup_items=n_req)
        out["fragments_of_%d" % length] = {
            "payload_GBps": round(float(total) * (passes - 1) / (wall_us * 1e-6) / 1e9, 1),
            "rw_frac_of_hbm_peak": round(2.0 * total * (passes - 1) / (wall_us * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
        }
    del pool_d, dst_d
    return out


def storm_launch(pkg, hip, benchlib, torch, engine, in_flight, reps=64):
    """One launch of the engine over the storm of 64 KiB requests (2048 requests of 16 whole pages from a 512 MiB
    pool, `reps` times over, into a ring of 1 GiB of destinations), `in_flight` of them in flight."""
    wl = pkg.Workload(3, seed=0xC0FFEE03)
    info = wl.info
    pool_d = torch.empty(int(info.pool_bytes), dtype=torch.uint8, device="cuda:0").random_(0, 256)
    dst_d = torch.empty((1 << 30) + 512, dtype=torch.uint8, device="cuda:0")
    torch.cuda.synchronize()
    descs = np.array(wl.descs, copy=True)
    descs["dst_off"] %= 65536
    n = len(wl.requests)
    items = (pkg.StreamItem * (n * reps))()
    for i in range(n * reps):
        r = wl.requests[i % n]
        items[i].bounce_base = pool_d.data_ptr()
        items[i].dst_base = dst_d.data_ptr() + 256 + (i * 65536) % (1 << 30)
        items[i].descs_host = descs.ctypes.data + 16 * int(r["first_desc"])
        items[i].n_descs = int(r["n_descs"])
        items[i].payload_bytes = int(r["bytes"])
    wall, kern = ctypes.c_double(), ctypes.c_double()
    pkg.check(benchlib.tcpxuEngineRunTimed(engine, items, len(items), n, in_flight, 20000, ctypes.byref(wall), ctypes.byref(kern), None), "tcpxuEngineRunTimed")
    stats, split = pkg.EngineStats(), pkg.StreamSplit()
    pkg.check(hip.tcpxuEngineGetStats(engine, ctypes.byref(stats)), "tcpxuEngineGetStats")
    pkg.check(benchlib.tcpxuStreamLastSplit(ctypes.byref(split)), "tcpxuStreamLastSplit")
    timed = n * (reps - 1)
    return {
        "what": "storm: %d requests of 64 KiB (16 whole pages each), %d in flight" % (n * reps, in_flight),
        "requests": n * reps,
        "requests_per_s": round(timed / (wall.value * 1e-6)),
        "payload_GBps": round(timed * 65536 / (wall.value * 1e-6) / 1e9, 1),
        "rw_frac_of_hbm_peak": round(2.0 * timed * 65536 / (wall.value * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
        "bytes_per_launch": 2.0 * 65536 * n * reps,
        "launch_us": round(kern.value, 1),
        "host_ns_per_publish": round(split.publish_ns / max(split.published, 1), 1),
        "leader_entries_per_poll": round(stats.leader_entries / max(stats.leader_polls, 1), 2),
        "leader_polls": int(stats.leader_polls),
        "leader_polls_fetching_64": int(stats.leader_deep_polls),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400, help="K: steps in one timed window")
    ap.add_argument("--warmup", type=int, default=64, help="W: untimed steps before the first window (at least two queues' worth are run whatever W says)")
    ap.add_argument("--windows", type=int, default=0, help="R: timed windows of K steps in the launch; 0 = max(50, ceil(20000 / K))")
    ap.add_argument(
        "--chunks",
        type=int,
        default=128,
        help="distinct chunks (descriptor lists + destinations) cycled through; the destinations form a ring of this "
        "many times 8 MiB, which must be several times the 256 MiB Infinity Cache or part of the writes never reach HBM "
        "(measured with 16 source pools: 256 MiB ring 80 %% of the roofline, 384 MiB 74 %%, 768 MiB and more 71 %%)",
    )
    ap.add_argument("--pools", type=int, default=64, help="copies of the 256 MiB bounce pool the chunks take turns reading from")
    ap.add_argument("--comms", type=int, default=4, help="receive comms kept busy on the one engine (1..4)")
    ap.add_argument("--depth", type=int, default=16, help="slots of one comm's mapped ring in flight (the unpack queue depth)")
    ap.add_argument("--cpu-seconds", type=float, default=5.0, help="CPU time per baseline leg (four legs)")
    ap.add_argument("--skip-extras", action="store_true", help="only the headline measurement")
    ap.add_argument(
        "--one-launch",
        action="store_true",
        help="exactly one launch of the engine kernel in the process (no untimed launch before it, no single-comm run, "
        "no extras): what a kernel trace or a counter run of the headline should see",
    )
    ap.add_argument("--one-config", type=int, default=0, choices=[0, 1, 3, 4, 5], help="exactly one launch of the engine kernel over this other workload of the contract (1, 4 or 5 with 64 slots in flight; 3, the storm of 64 KiB requests, with --in-flight), and exit: for a profiler")
    ap.add_argument("--in-flight", type=int, default=1024, help="requests in flight for --one-config 3 (1..2048)")
    ap.add_argument(
        "--calibrate-copy",
        type=int,
        default=0,
        metavar="MIB",
        help="run only the plain copy kernel on MIB mebibytes (10 launches) and exit: a kernel of known traffic "
        "against which hardware counters (FETCH_SIZE, WRITE_SIZE) are scaled",
    )
    ap.add_argument(
        "--batch-kernel",
        action="store_true",
        help="run only the launch-per-batch kernel on 128 chunks of the headline workload in one launch (1 GiB of "
        "payload, 15 copies of the pool) and exit: what a kernel trace of unpack_batch_kernel should see",
    )
    args = ap.parse_args()
    if not 1 <= args.comms <= 4 or not 1 <= args.depth <= 16 or not 1 <= args.pools <= 256:
        sys.exit("bench.py: --comms must be 1..4, --depth 1..16, --pools 1..256")
    if args.steps < 1 or args.warmup < 0 or args.windows < 0:
        sys.exit("bench.py: --steps must be at least 1, --warmup and --windows not negative")
    if args.gpus != 1:
        sys.exit("bench.py: this path runs on one GPU; --gpus %d is not supported (every GPU would run an independent copy)" % args.gpus)

    import torch

    pkg = graft.load_package()
    hip = pkg.hip_layer()  # raises if the HIP library is missing; there is no fallback
    benchlib = pkg.bench_layer()  # the streaming driver and the event-timed launches
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    dev = 0
    if args.calibrate_copy > 0:
        n = args.calibrate_copy << 20
        a = torch.empty(n, dtype=torch.uint8, device="cuda:0").random_(0, 256)
        b = torch.empty(n, dtype=torch.uint8, device="cuda:0")
        torch.cuda.synchronize()
        us = ctypes.c_double()
        pkg.check(benchlib.tcpxuCopyKernelTimed(dev, b.data_ptr(), a.data_ptr(), n, 0, 10, ctypes.byref(us)), "tcpxuCopyKernelTimed")
        print(json.dumps({"kernel": "copy_kernel", "launches": 10, "bytes_read_per_launch": n, "bytes_written_per_launch": n, "launch_us": round(us.value, 2)}))
        return
    if args.batch_kernel:
        print(json.dumps(batch_kernel_line(pkg, benchlib, torch, dev)))
        return
    if args.one_config:
        # One launch of the engine kernel over one of the other workloads, after 150 launches of the plain copy kernel
        # (60 ms of load, so that the GPU is in the state it sustains).
        n = 512 << 20
        a = torch.empty(n, dtype=torch.uint8, device="cuda:0").random_(0, 256)
        b = torch.empty(n, dtype=torch.uint8, device="cuda:0")
        torch.cuda.synchronize()
        us = ctypes.c_double()
        pkg.check(benchlib.tcpxuCopyKernelTimed(dev, b.data_ptr(), a.data_ptr(), n, 0, 150, ctypes.byref(us)), "tcpxuCopyKernelTimed")
        del a, b
        engine = ctypes.c_void_p()
        cfg = pkg.EngineConfig(0, 0, 0, 0)
        pkg.check(hip.tcpxuEngineCreate(dev, ctypes.byref(cfg), ctypes.byref(engine)), "tcpxuEngineCreate")

        def run_once(items, depth, warmup_items=0):
            wall, kern = ctypes.c_double(), ctypes.c_double()
            rc = benchlib.tcpxuEngineRunTimed(engine, items, len(items), warmup_items, depth, 20000, ctypes.byref(wall), ctypes.byref(kern), None)
            pkg.check(rc, "tcpxuEngineRunTimed")
            return wall.value, kern.value, None

        if args.one_config == 3:
            out = {"config_3": storm_launch(pkg, hip, benchlib, torch, engine, args.in_flight)}
            in_flight = args.in_flight
        else:
            out = other_configs(pkg, torch, run_once, only=args.one_config)
            in_flight = 64
        pkg.check(hip.tcpxuEngineDestroy(engine), "tcpxuEngineDestroy")
        print(json.dumps(dict(out["config_%d" % args.one_config], kernel="unpack_engine_kernel", slots_in_flight=in_flight)))
        return
    name = ctypes.create_string_buffer(256)
    cus = ctypes.c_int()
    pkg.check(hip.tcpxuDeviceInfo(dev, name, 256, ctypes.byref(cus)), "tcpxuDeviceInfo")

    # ---- inputs: one pool, `chunks` descriptor lists, `chunks` destinations ------------------------------
    workloads = [pkg.Workload(CHUNK_CONFIG, seed=0xC0FFEE02 + 7919 * i) for i in range(args.chunks)]
    info0 = workloads[0].info
    chunk_bytes = info0.payload_bytes
    pool = np.empty(info0.pool_bytes, dtype=np.uint8)
    workloads[0].fill_window(0, pool)
    # `--pools` copies of the 256 MiB bounce pool; chunk c reads from copy c % pools.  One pool alone fits the
    # 256 MiB Infinity Cache and is re-read by every chunk, which a bounce pool that the NIC keeps refilling never is.
    pool_d = torch.from_numpy(pool).to("cuda:0").repeat(args.pools)
    dst_d = torch.full((args.chunks * chunk_bytes + 512,), 0xA5, dtype=torch.uint8, device="cuda:0")
    dst_base = dst_d.data_ptr() + 256
    torch.cuda.synchronize()

    per_chunk_items = []
    keep = []
    for c, wl in enumerate(workloads):
        items = []
        for r in wl.requests:
            d = np.ascontiguousarray(wl.descs[int(r["first_desc"]) : int(r["first_desc"]) + int(r["n_descs"])])
            keep.append(d)
            items.append((pool_d.data_ptr() + (c % args.pools) * info0.pool_bytes, dst_base + c * chunk_bytes, d.ctypes.data, len(d), int(d["len"].sum())))
        per_chunk_items.append(items)
    slots_per_step = len(per_chunk_items[0])
    descs_per_step = float(np.mean([wl.info.n_descs for wl in workloads]))

    item_dtype = np.dtype([("bounce", "<u8"), ("dst", "<u8"), ("descs", "<u8"), ("n", "<u4"), ("bytes", "<u4")])
    assert item_dtype.itemsize == ctypes.sizeof(pkg.StreamItem)
    # the request's size (`bytes`) is what a caller of the plugin's test() has at hand
    ring_items = np.array([it for items in per_chunk_items for it in items], dtype=item_dtype).reshape(args.chunks, slots_per_step)

    def item_array(first_step, n_steps):
        rows = np.ascontiguousarray(ring_items[(first_step + np.arange(n_steps)) % args.chunks].reshape(-1))
        arr = (pkg.StreamItem * len(rows)).from_buffer(rows)
        arr._rows = rows  # keeps the memory alive
        return arr

    engine = ctypes.c_void_p()
    cfg = pkg.EngineConfig(0, 0, 0, 0)
    pkg.check(hip.tcpxuEngineCreate(dev, ctypes.byref(cfg), ctypes.byref(engine)), "tcpxuEngineCreate")

    eff = pkg.EngineConfig()
    pkg.check(hip.tcpxuEngineGetConfig(engine, ctypes.byref(eff)), "tcpxuEngineGetConfig")

    def run(items, depth, warmup_items=0, want_latency=False, timed_items=None, engine=engine):
        """One launch of the engine over `items`.  With `timed_items`, the wall time is that of the timed items
        from completion to completion (the items after them only keep the queues full); otherwise from the publish
        of item `warmup_items` to the last completion."""
        wall, kern = ctypes.c_double(), ctypes.c_double()
        lat = (ctypes.c_double * len(items))() if want_latency else None
        if timed_items is None:
            rc = benchlib.tcpxuEngineRunTimed(
                engine, items, len(items), warmup_items, depth, 20000, ctypes.byref(wall), ctypes.byref(kern), lat
            )
        else:
            rc = benchlib.tcpxuEngineRunWindow(
                engine, items, len(items), warmup_items, timed_items, depth, 20000, ctypes.byref(wall), ctypes.byref(kern), lat
            )
        pkg.check(rc, "tcpxuEngineRunTimed")
        return wall.value, kern.value, (np.asarray(lat[:]) if want_latency else None)

    def run_windows(items, depth):
        """One launch over `items` with every completion stamped: the duration of each of the R windows of K steps
        (completion of the step before the window -> completion of its last step) and of the launch, microseconds."""
        kern = ctypes.c_double()
        done = np.zeros(len(items), dtype=np.float64)
        rc = benchlib.tcpxuEngineRunStamped(
            engine, items, len(items), depth, 20000, ctypes.byref(kern), done.ctypes.data_as(ctypes.POINTER(ctypes.c_double)), None
        )
        pkg.check(rc, "tcpxuEngineRunStamped")
        step_done = done[slots_per_step - 1 :: slots_per_step]  # completion of each step's last slot
        edges = step_done[fill_steps - 1 : fill_steps + windows * args.steps : args.steps]
        assert len(edges) == windows + 1
        return np.diff(edges), kern.value

    # ---- fill, R windows of exactly K steps, tail: all inside ONE launch of the persistent kernel ---------------
    queue_steps = (args.comms * args.depth + slots_per_step - 1) // slots_per_step  # steps that fill every queue once
    fill_steps = max(args.warmup, 2 * queue_steps)
    windows = args.windows if args.windows > 0 else max(50, (MIN_TIMED_STEPS + args.steps - 1) // args.steps)
    tail_steps = queue_steps
    steps_per_launch = fill_steps + windows * args.steps + tail_steps
    all_items = item_array(0, steps_per_launch)
    # An untimed launch first: brings the GPU from idle to the state it is in under sustained load (a measured launch
    # of 2096 steps shows 70.2 % of the roofline after 64 untimed steps, 70.8 % after 2000 and 71.4 % after 20000) and
    # loads the library's code onto the GPU.  Where the
    # process may launch the engine kernel only once (--one-launch, for a profiler), other kernels do that instead:
    # the launch-per-batch kernel (the same code object) on one chunk and the plain copy kernel, 150 times over half the
    # destination ring (60 ms).
    if not args.one_launch:
        run(item_array(0, max(fill_steps, WARM_LAUNCH_STEPS)), args.comms * args.depth)
    else:
        us = ctypes.c_double()
        d0 = torch.from_numpy(np.ascontiguousarray(workloads[0].descs).view(np.uint8)).to("cuda:0")
        pkg.check(benchlib.tcpxuUnpackBatchTimed(dev, pool_d.data_ptr(), dst_base, d0.data_ptr(), workloads[0].info.n_descs, 2, 3, ctypes.byref(us)), "batch timed")
        n_warm = min(1 << 30, args.chunks * int(chunk_bytes) // 2 // 16 * 16)
        pkg.check(benchlib.tcpxuCopyKernelTimed(dev, dst_base + n_warm, dst_base, n_warm, 2, 150, ctypes.byref(us)), "copy timed")  # 60 ms of load
        del d0
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    window_us, kernel_us = run_windows(all_items, args.comms * args.depth)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    assert all(int(wl.info.payload_bytes) == int(chunk_bytes) for wl in workloads)  # every step moves the same bytes
    payload = float(chunk_bytes) * args.steps
    launch_payload = float(chunk_bytes) * steps_per_launch
    wall_us = float(np.median(window_us))
    value_gbps = payload / (wall_us * 1e-6) / 1e9
    achieved = 2.0 * launch_payload / (kernel_us * 1e-6) / 1e9

    # ---- parity spot check: the last chunk written must equal the oracle's bytes ---------------------------
    oracle = graft.load_oracle()
    last = (steps_per_launch - 1) % args.chunks
    expect = np.full(chunk_bytes, 0xA5, dtype=np.uint8)
    graft.oracle_unpack(oracle, expect, pool, np.ascontiguousarray(workloads[last].descs))
    got = dst_d[256 + last * chunk_bytes : 256 + (last + 1) * chunk_bytes].cpu().numpy()
    parity_ok = bool(np.array_equal(got, expect))

    result = {
        "metric": "unpack payload GB/s + % HBM r+w roofline at 8 MiB chunk; p50 request us",
        "value": round(value_gbps, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "steps_run": steps_per_launch,  # what the launch carried: fill_steps + windows x steps + the tail
        "fill_steps": fill_steps,
        "windows": windows,
        "ms_per_step": round(wall_us / 1000.0 / args.steps, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u8",
        "data": "synthetic",
        "config": {
            "workload": "8 MiB chunk, 4 interleaved flows, ~2155 fragments (90%% 4096 B, 10%% U[64,4095]), byte-unaligned "
            "sources in a 256 MiB pool (%d such pools taken in turn), 2 x 4 MiB requests per chunk, %d distinct chunks "
            "cycled; %d receive comms on one engine, unpack queue depth %d each" % (args.pools, args.chunks, args.comms, args.depth),
            "pools": args.pools,
            "comms": args.comms,
            "queue_depth_per_comm": args.depth,
            "fill_steps": fill_steps,
            "windows": windows,
            "tail_steps": tail_steps,
            "timing": "one launch = %d untimed fill steps + %d windows of %d steps + %d untimed tail steps; a window runs from the "
            "completion of the step before it to the completion of its last step; ms_per_step x steps = the median window"
            % (fill_steps, windows, args.steps, tail_steps),
            "path": "persistent engine: mapped descriptor ring -> gfx950 unpack kernel -> mapped completion word",
            "descriptors_per_step": round(descs_per_step, 1),
            "slots_per_step": slots_per_step,
            "device": name.value.decode(),
            "compute_units": cus.value,
            "engine_workgroups": eff.workgroups,
            "descs_per_ticket": eff.descs_per_ticket if eff.descs_per_ticket else "8, 12, 14 or 16 by backlog (a submission of at most 32 stays whole; 32, 48 or 64 for short fragments)",
        },
        "roofline": {
            "bound": "hbm",
            "kernel": "unpack_engine_kernel",
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBPS, 4),
            "traffic": round(2.0 * launch_payload * TRAFFIC_PER_ALGORITHMIC_BYTE),
            "traffic_source": "FETCH_SIZE and WRITE_SIZE of this kernel on this workload (two rocprofv3 --pmc runs, scaled by "
            "the same counters on the plain copy kernel: x1.99977 and x1.0) came to %.4f x the algorithmic bytes; "
            "that ratio times bytes_per_launch" % TRAFFIC_PER_ALGORITHMIC_BYTE,
            "bytes_per_launch": 2.0 * launch_payload,
            "steps_per_launch": steps_per_launch,
            "launch_us": round(kernel_us, 1),
        },
        "window_ms": {
            "median": round(wall_us / 1000.0, 6),
            "mean": round(float(np.mean(window_us)) / 1000.0, 6),
            # every timed step over all the timed time: nothing dropped, slow windows included
            "value_over_all_windows_GBps": round(payload * windows / (float(np.sum(window_us)) * 1e-6) / 1e9, 2),
            "p10": round(percentile(window_us, 10) / 1000.0, 6),
            "p90": round(percentile(window_us, 90) / 1000.0, 6),
            "windows": windows,
            "rw_frac_of_hbm_peak_at_median": round(2.0 * value_gbps / HBM_PEAK_GBPS, 4),
        },
        "parity_ok": parity_ok,
        "timed_region_s": round(t1 - t0, 4),
    }
    if args.comms > 1 and not args.one_launch:
        # The same steps with one comm only: 16 slots (at most 64 MiB) in flight, a launch of its own.
        win1, k1 = run_windows(all_items, args.depth)
        w1 = float(np.median(win1))
        result["single_comm"] = {
            "value": round(payload / (w1 * 1e-6) / 1e9, 2),
            "unit": "GB/s",
            "ms_per_step": round(w1 / 1000.0 / args.steps, 6),
            "roofline_achieved": round(2.0 * launch_payload / (k1 * 1e-6) / 1e9, 1),
            "roofline_frac": round(2.0 * launch_payload / (k1 * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
            "launch_us": round(k1, 1),
        }

    if not args.skip_extras and not args.one_launch:
        # Request completion latency, one request in flight: publish -> host poller sees the completion word.
        storm = pkg.Workload(3, seed=0xC0FFEE03)
        sd = np.array(storm.descs, copy=True)
        # The storm's 512 MiB pool is the first two of the bounce pool's copies; with fewer it is folded into one.
        storm_pool_bytes = min(int(storm.info.pool_bytes), args.pools * int(info0.pool_bytes))
        sd["src_off"] %= storm_pool_bytes
        storm_dst_bytes = args.chunks * chunk_bytes
        n_storm = len(storm.requests)
        storm_items = (pkg.StreamItem * n_storm)()
        for i, r in enumerate(storm.requests):
            storm_items[i].bounce_base = pool_d.data_ptr()
            storm_items[i].dst_base = dst_base + (i * 65536) % (storm_dst_bytes - 65536)
            storm_items[i].descs_host = sd.ctypes.data + 16 * int(r["first_desc"])
            storm_items[i].n_descs = int(r["n_descs"])
            storm_items[i].payload_bytes = int(r["bytes"])
        sd["dst_off"] %= 65536
        _, _, lat64k = run(storm_items, 1, want_latency=True)
        lat4m_items = item_array(0, 200)
        _, _, lat4m = run(lat4m_items, 1, want_latency=True)
        result["latency_us"] = {
            "definition": "host publish of a slot -> host poller observes the completion word, one request in flight",
            "request_64KiB_16_descs": {"p50": round(percentile(lat64k, 50), 2), "p99": round(percentile(lat64k, 99), 2)},
            "request_4MiB_1078_descs": {"p50": round(percentile(lat4m, 50), 2), "p99": round(percentile(lat4m, 99), 2)},
        }
        result["p50_request_us"] = result["latency_us"]["request_64KiB_16_descs"]["p50"]
        # Where a lone request's time goes: the same two runs on a second engine that stamps the GPU's constant-rate
        # clock at four points of every submission (the figures above come from the engine that does not).  The GPU's
        # clock and the host's are not tied to each other, so the two crossings of PCIe -- the publish until the
        # leader's poll has it, the completion word until the host's poll has it -- come out as one term: the request's
        # whole time less what lies between the first and the last stamp.
        stamped = ctypes.c_void_p()
        pkg.check(hip.tcpxuEngineCreate(dev, ctypes.byref(cfg), ctypes.byref(stamped)), "tcpxuEngineCreate")
        ticks_per_us = ctypes.c_double()
        pkg.check(hip.tcpxuEngineEnableStamps(stamped, ctypes.byref(ticks_per_us)), "tcpxuEngineEnableStamps")

        def budget(items, first, in_flight=1):
            n = len(items)
            _, _, lat = run(items, in_flight, want_latency=True, engine=stamped)
            raw = np.zeros(4 * n, dtype=np.uint64)
            pkg.check(hip.tcpxuEngineReadStamps(stamped, first, n, raw.ctypes.data_as(ctypes.POINTER(ctypes.c_uint64))), "tcpxuEngineReadStamps")
            t = raw.reshape(n, 4).astype(np.float64) / ticks_per_us.value
            ok = (raw.reshape(n, 4) != np.uint64(0xFFFFFFFFFFFFFFFF)).all(axis=1)
            t, total = t[ok], lat[ok]
            on_gpu = t[:, 3] - t[:, 0]
            med = lambda v: round(float(np.median(v)), 2)  # noqa: E731
            return {
                "p50_with_stamps": med(total),
                "publish_to_leader_plus_completion_word_to_host": med(total - on_gpu),
                "leader_saw_it_to_first_ticket_fetched": med(t[:, 1] - t[:, 0]),
                "ticket_fetched_to_descriptors_staged": med(t[:, 2] - t[:, 1]),
                "descriptors_staged_to_last_store_acknowledged": med(t[:, 3] - t[:, 2]),
                "requests": int(ok.sum()),
            }

        b64k = budget(storm_items, 0)
        b4m = budget(lat4m_items, n_storm)
        empty = (pkg.StreamItem * 500)()  # no descriptors: the leader itself writes the completion word
        for i in range(500):
            empty[i].bounce_base, empty[i].dst_base, empty[i].descs_host, empty[i].n_descs = pool_d.data_ptr(), dst_base, sd.ctypes.data, 0
        _, _, lat0 = run(empty, 1, want_latency=True, engine=stamped)
        # The same 2048 requests of 64 KiB with 256 of them in flight, where a storm's rate is what one request takes:
        # the term outside the kernel then also holds the wait for the leader's next poll.
        b64k_256 = budget(storm_items, n_storm + len(lat4m_items) + len(empty), in_flight=256)
        pkg.check(hip.tcpxuEngineDestroy(stamped), "tcpxuEngineDestroy")
        result["latency_us"]["budget"] = {
            "definition": "medians, microseconds, one request in flight unless the key says otherwise (the first term then also "
            "holds the wait for the leader's next poll); stamps of the GPU's %g MHz clock taken by the kernel" % ticks_per_us.value,
            "request_64KiB_16_descs": b64k,
            "request_4MiB_1078_descs": b4m,
            "request_64KiB_16_descs_with_256_in_flight": b64k_256,
            "empty_submission_round_trip_p50": round(percentile(lat0, 50), 2),
        }
        # The small-message storm: the 2048 requests of 64 KiB (16 fragments of 4 KiB each) sixteen times over, W of
        # them in flight, W x 16 = 64 .. 32768 descriptors with the engine at a time; W = 2048 is the workload's
        # "2048 concurrent requests" (the unpack queues of 128 comms).  The first 2048 are left out of the rate.
        # Beside each rate, where the time went: the host thread's nanoseconds per publish (descriptors into the slot,
        # the submission entry, one tail store per batch) and what the leader's polls of the submission ring found.
        storm_reps = 16
        many = (pkg.StreamItem * (n_storm * storm_reps))()
        for i in range(n_storm * storm_reps):
            src = storm_items[i % n_storm]
            many[i].bounce_base = src.bounce_base
            many[i].dst_base = dst_base + (i * 65536) % (storm_dst_bytes - 65536)
            many[i].descs_host = src.descs_host
            many[i].n_descs = src.n_descs
            many[i].payload_bytes = src.payload_bytes
        sweep = []
        stats0, stats1, split = pkg.EngineStats(), pkg.EngineStats(), pkg.StreamSplit()
        for in_flight in (4, 8, 16, 32, 64, 128, 256, 512, 1024, 2048):
            pkg.check(hip.tcpxuEngineGetStats(engine, ctypes.byref(stats0)), "tcpxuEngineGetStats")
            w, _, lat = run(many, in_flight, warmup_items=n_storm, want_latency=True)
            pkg.check(hip.tcpxuEngineGetStats(engine, ctypes.byref(stats1)), "tcpxuEngineGetStats")
            pkg.check(benchlib.tcpxuStreamLastSplit(ctypes.byref(split)), "tcpxuStreamLastSplit")
            timed = n_storm * (storm_reps - 1)
            polls = stats1.leader_polls - stats0.leader_polls
            sweep.append(
                {
                    "requests_in_flight": in_flight,
                    "descriptors_in_flight": 16 * in_flight,
                    "requests_per_s": round(timed / (w * 1e-6)),
                    "payload_GBps": round(timed * 65536 / (w * 1e-6) / 1e9, 1),
                    "p50_us": round(percentile(lat[n_storm:], 50), 2),
                    "p99_us": round(percentile(lat[n_storm:], 99), 2),
                    "host_ns_per_publish": round(split.publish_ns / max(split.published, 1), 1),
                    "host_publishes_per_call": round(split.published / max(split.publish_calls, 1), 1),
                    "host_share_of_wall_in_publish": round(split.publish_ns / max(split.wall_ns, 1.0), 3),
                    "leader_entries_per_poll": round((stats1.leader_entries - stats0.leader_entries) / max(polls, 1), 2),
                    "leader_polls_per_us": round(polls / max(split.wall_ns * 1e-3, 1e-9), 3),
                    "leader_share_of_polls_fetching_64": round((stats1.leader_deep_polls - stats0.leader_deep_polls) / max(polls, 1), 3),
                }
            )
        best = max(sweep, key=lambda x: x["requests_per_s"])
        result["storm_64KiB"] = {
            "requests": n_storm * storm_reps,
            "requests_timed": n_storm * (storm_reps - 1),
            "latency": "publish of a request's slot -> host poller observes its completion word",
            "leader": "a poll fetches 16 submission entries, 64 after a poll that found all sixteen; with 192 or more published "
            "ahead the leader keeps five groups of sixteen in flight instead, and every 64 entries taken that way count as a poll of 64",
            "best": {k: best[k] for k in ("requests_in_flight", "requests_per_s", "payload_GBps")},
            "sweep": sweep,
        }
        result["storm_64KiB_requests_per_s"] = next(x["requests_per_s"] for x in sweep if x["requests_in_flight"] == 16)

        # Launch-per-batch kernel on the same chunk and on the 256 MiB bulk workload, and a plain copy kernel.
        us = ctypes.c_double()
        d0 = torch.from_numpy(np.ascontiguousarray(workloads[0].descs).view(np.uint8)).to("cuda:0")
        pkg.check(benchlib.tcpxuUnpackBatchTimed(dev, pool_d.data_ptr(), dst_base, d0.data_ptr(), workloads[0].info.n_descs, 20, 200, ctypes.byref(us)), "batch timed")
        result["launch_per_batch_8MiB"] = {
            "kernel": "unpack_batch_kernel",
            "note": "the same chunk every launch: launch-bound and cache-resident, not an HBM figure",
            "launch_us": round(us.value, 2),
            "rw_GBps": round(2 * chunk_bytes / us.value / 1e3, 1),
            "frac": round(2 * chunk_bytes / us.value / 1e3 / HBM_PEAK_GBPS, 4),
        }
        del d0
        # 1 GiB to 1 GiB, four times the Infinity Cache each way: what a plain copy with the same accesses reaches.
        n_copy = 1 << 30
        scratch = torch.empty(2 * n_copy, dtype=torch.uint8, device="cuda:0")
        scratch.zero_()
        torch.cuda.synchronize()
        pkg.check(benchlib.tcpxuCopyKernelTimed(dev, scratch.data_ptr() + n_copy, scratch.data_ptr(), n_copy, 3, 20, ctypes.byref(us)), "copy timed")
        result["plain_copy_kernel"] = {"bytes": n_copy, "launch_us": round(us.value, 2), "rw_GBps": round(2 * n_copy / us.value / 1e3, 1)}
        # Each half of that copy on its own (loads only, stores only, same accesses), over 2 GiB: a copy that spends
        # 1/read + 1/write per byte moves 2 / (1/read + 1/write) bytes of read + write per second.
        pkg.check(benchlib.tcpxuCopyKernelTimed(dev, None, scratch.data_ptr(), 2 * n_copy, 3, 20, ctypes.byref(us)), "read timed")
        read_gbps = 2 * n_copy / us.value / 1e3
        pkg.check(benchlib.tcpxuCopyKernelTimed(dev, scratch.data_ptr(), None, 2 * n_copy, 3, 20, ctypes.byref(us)), "fill timed")
        write_gbps = 2 * n_copy / us.value / 1e3
        # The runtime's own device-to-device copy of the same gigabyte (torch's copy_ of a contiguous tensor is one
        # hipMemcpyDtoDAsync), timed with events on torch's stream.
        lo, hi = scratch[:n_copy], scratch[n_copy:]
        for _ in range(3):
            hi.copy_(lo)
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ev0.record()
        for _ in range(20):
            hi.copy_(lo)
        ev1.record()
        ev1.synchronize()
        runtime_copy_gbps = 2 * n_copy * 20 / (ev0.elapsed_time(ev1) * 1e-3) / 1e9
        del lo, hi
        # A bare gather of short fragments: 1 GiB of them (four times the Infinity Cache each way) from random pages of
        # a 4 GiB pool to a contiguous destination -- the grain of the adversarial workload (2 KiB a fragment on average)
        # without any of the unpack kernel's work on it.
        del scratch
        gather_pool = torch.empty(4 * n_copy, dtype=torch.uint8, device="cuda:0")
        gather_pool.zero_()
        gather_dst = torch.empty(n_copy, dtype=torch.uint8, device="cuda:0")
        gather = {}
        for kib in (1, 2, 4):
            n_frag = n_copy // (kib << 10)
            pages_d = torch.randint(0, (4 * n_copy) // 4096, (n_frag,), dtype=torch.int32, device="cuda:0")
            torch.cuda.synchronize()
            pkg.check(benchlib.tcpxuGatherKernelTimed(dev, gather_dst.data_ptr(), gather_pool.data_ptr(), pages_d.data_ptr(), n_frag, kib << 10, 2, 10, ctypes.byref(us)), "gather timed")
            gather["gather_%dKiB_fragments_rw_GBps" % kib] = round(2 * n_copy / us.value / 1e3, 1)
            del pages_d
        del gather_pool, gather_dst
        result["hbm_yardsticks"] = {
            "read_only_GBps": round(read_gbps, 1),
            "write_only_GBps": round(write_gbps, 1),
            "runtime_device_to_device_copy_rw_GBps": round(runtime_copy_gbps, 1),
            "copy_bound_rw_GBps": round(2.0 / (1.0 / read_gbps + 1.0 / write_gbps), 1),
            **gather,
            "note": "plain kernels over 2 GiB with the unpack kernel's load and store instructions; copy_bound is what a "
            "plain copy made of these two halves comes to (1/read + 1/write per byte), against the roofline's 8000 GB/s; "
            "gather_*: 1 GiB made of the first 1, 2 or 4 KiB of random pages of a 4 GiB pool to a contiguous destination, "
            "one wavefront per fragment, sixteen per compute unit",
        }

        result["other_configs"] = other_configs(pkg, torch, run)
        result["fragment_length_sweep"] = fragment_length_sweep(pkg, torch, run)
        result["launch_per_batch_1GiB"] = batch_kernel_line(pkg, benchlib, torch, dev)

    pkg.check(hip.tcpxuEngineDestroy(engine), "tcpxuEngineDestroy")

    if not args.skip_extras and not args.one_launch:
        result["plugin_path"] = plugin_path(pkg, hip, torch, workloads[: min(8, args.chunks)], pool)
        # Two threads that hand every task to each other through the task rings, and in this workload (four flows
        # interleaved fragment by fragment) every fragment is a chunk of its own, hence a task: the leg costs about one
        # cache line there and back per fragment, and that depends on where the machine puts the two threads (the
        # virtual CPUs of the test boxes lie 60-85 ns apart in some pairs and 400-750 ns in others, and the leg comes
        # out near 46-57 GB/s or near 11 GB/s accordingly).  So it runs three times as the machine places the threads,
        # median beside all three, and once each with the proxy thread on one CPU and the socket thread bound
        # (NCCL_GPUDIRECTTCPX_RX_BINDINGS, the reference's flag for this) to the CPU nearest to it and farthest from it.
        # The same surface fed as the reference's sender feeds it: chunks of 128 KiB, 32 fragments to the control message,
        # the task and the recvmsg (the bulk workload: whole pages, eight flows, runs of 32 fragments per flow).  On the
        # headline workload every fragment is a chunk of its own, because the contract interleaves its flows fragment
        # by fragment, and the host's time per fragment is a time per task.
        bulk = pkg.Workload(4, seed=0xC0FFEE04, shrink=1)  # 128 MiB in 32 requests of 4 MiB from a 512 MiB pool
        bulk_pool = np.empty(int(bulk.info.pool_bytes), dtype=np.uint8)
        bulk.fill_window(0, bulk_pool)
        result["plugin_path"]["in_chunks_of_32_fragments"] = plugin_path(
            pkg, hip, torch, [bulk], bulk_pool, what="a 128 MiB message of whole pages in 4 MiB requests, eight flows, chunks of 128 KiB,")
        del bulk_pool
        some = workloads[: min(8, args.chunks)]
        legs = [plugin_path(pkg, hip, torch, some, pool, helper_thread=True) for _ in range(3)]
        legs.sort(key=lambda leg: leg.get("payload_GBps", 0.0))
        result["plugin_path"]["with_socket_thread"] = dict(legs[1], payload_GBps_of_three_runs=[leg.get("payload_GBps") for leg in legs])
        cpus = sorted(os.sched_getaffinity(0))
        if len(cpus) >= 2:
            synth, ns, apart = pkg.synth_lib(), ctypes.c_double(), {}
            for other in cpus[1:]:
                if synth.tcpxSynthCpuRoundTripNs(cpus[0], other, 5000, ctypes.byref(ns)) == 0:
                    apart[other] = ns.value
            bound = {}
            try:
                os.sched_setaffinity(0, [cpus[0]])  # this thread is the proxy thread
                for which, other in (("nearest", min(apart, key=apart.get)), ("farthest", max(apart, key=apart.get))) if apart else ():
                    leg = plugin_path(pkg, hip, torch, some, pool, helper_thread=True, rx_bindings="tcpx-amd-synth0:%d-%d" % (other, other))
                    bound[which] = {"cpus": [cpus[0], other], "cache_line_round_trip_ns": round(apart[other]), "payload_GBps": leg.get("payload_GBps"), "host_ns_per_fragment": leg.get("host_ns_per_fragment")}
            except OSError as err:  # a machine that does not let the process choose its CPUs: the unbound runs stand alone
                bound["error"] = str(err)
            finally:
                try:
                    os.sched_setaffinity(0, cpus)
                except OSError:
                    pass
            result["plugin_path"]["with_socket_thread"]["socket_thread_bound_to_the_cpu"] = bound

    # ---- CPU baseline on this machine's host cores: rank 0, bounded sample ---------------------------------
    # Threads: the cores this process may run on.  A GPU box shows every core of the host to os.cpu_count() while a
    # one-GPU job is given a share of them (OMP_NUM_THREADS says how many), so that share is the "all cores" leg.
    logical = os.cpu_count() or 1
    try:
        allowed = len(os.sched_getaffinity(0))
    except (AttributeError, OSError):
        allowed = logical
    share = int(os.environ.get("OMP_NUM_THREADS", "0") or 0)
    threads = max(1, min(allowed, share) if share > 0 else allowed)
    gbps_1, it1 = cpu_baseline(oracle, workloads[0].descs, int(chunk_bytes), pool, 1, args.cpu_seconds)
    gbps_t, itt = cpu_baseline(oracle, workloads[0].descs, int(chunk_bytes), pool, threads, args.cpu_seconds)
    # The same from DRAM: 64 chunks in turn (64 descriptor lists, 512 MiB of destinations, pages from four copies of
    # the pool, 1 GiB), so that neither side stays in the host's caches -- the care the GPU leg takes with HBM.
    n_dram = min(64, args.chunks)
    pool_copies = 4
    big_pool = np.tile(pool, pool_copies)
    parts = []
    for c in range(n_dram):
        d = np.array(workloads[c].descs, copy=True)
        d["src_off"] += np.uint32((c % pool_copies) * pool.nbytes)
        d["dst_off"] += np.uint64(c * int(chunk_bytes))
        parts.append(d)
    dram_descs = np.ascontiguousarray(np.concatenate(parts))
    dram_t, it_dt = cpu_baseline(oracle, dram_descs, n_dram * int(chunk_bytes), big_pool, threads, args.cpu_seconds)
    dram_1, it_d1 = cpu_baseline(oracle, dram_descs, n_dram * int(chunk_bytes), big_pool, 1, args.cpu_seconds)
    del big_pool
    result["cpu_baseline"] = {
        "value": round(dram_t, 2),
        "unit": "GB/s",
        "cores": threads,
        "kind": "port",
        "sample": "%d chunks of 8 MiB in turn (%d descriptors, %d MiB of destinations, pages from %d copies of the 256 MiB pool), "
        "all in host DRAM, memcpy per descriptor, descriptor list range-partitioned over %d threads, median of %d passes"
        % (n_dram, len(dram_descs), n_dram * int(chunk_bytes) >> 20, pool_copies, threads, it_dt),
        "host_logical_cpus": logical,
        "cpus_this_process_may_use": allowed,
        "cpu_share_of_the_job": share if share > 0 else None,
        "single_thread": {"value": round(dram_1, 2), "cores": 1, "passes": it_d1},
        "cache_resident": {
            "what": "the same single 8 MiB chunk over and over (descriptor list 0): sources and destination stay in the host's caches",
            "value": round(gbps_t, 2),
            "cores": threads,
            "iterations": itt,
            "single_thread": {"value": round(gbps_1, 2), "cores": 1, "iterations": it1},
        },
    }
    print(json.dumps(result))
    if not parity_ok:
        sys.exit("bench.py: GPU result differs from the oracle")


if __name__ == "__main__":
    main()
