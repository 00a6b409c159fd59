"""bench.py prints exactly one JSON line with the fields its consumers rely on, and the short command that the
round's driver runs measures the engine in steady state (GPU)."""
import json
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

CONTRACT_KEYS = ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling", "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline")  # fmt: skip


def run_bench(flags, timeout=600):
    print("bench case: %s" % " ".join(flags), flush=True)
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py")] + flags, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=timeout, cwd=ROOT)
    assert p.returncode == 0, p.stderr[-2000:]
    lines = [l for l in p.stdout.splitlines() if l.strip()]
    assert len(lines) == 1, p.stdout
    return json.loads(lines[0])


def check_contract(r, steps, warmup):
    for key in CONTRACT_KEYS:
        assert key in r, key
    assert r["n_gpus"] == 1 and r["steps"] == steps and r["warmup"] == warmup and r["unit"] == "GB/s" and r["dtype"] == "u8"
    assert r["vs_baseline"] is None and r["higher_is_better"] is True and r["data"] == "synthetic" and "workload" in r["config"]
    assert "note" not in r
    roof = r["roofline"]
    assert roof["bound"] == "hbm" and roof["peak"] == 8000.0 and roof["unit"] == "GB/s"
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3 and roof["traffic"] >= roof["bytes_per_launch"]
    cfg = r["config"]
    # at least two queues' worth of untimed steps before the first window, at least 50 windows, and a launch long
    # enough (20000 steps, 60 ms) that its start and end do not show in its duration
    assert cfg["fill_steps"] >= max(warmup, 2 * cfg["comms"] * cfg["queue_depth_per_comm"] // cfg["slots_per_step"])
    assert cfg["windows"] >= 50 and cfg["windows"] * steps >= 20000
    assert roof["steps_per_launch"] == cfg["fill_steps"] + cfg["windows"] * steps + cfg["tail_steps"]
    # ms_per_step x steps is the median window, and value its payload over it: 8 MiB a step
    step_bytes = roof["bytes_per_launch"] / 2 / roof["steps_per_launch"]
    assert step_bytes == 8 << 20
    assert abs(r["ms_per_step"] * steps - r["window_ms"]["median"]) < 1e-5 * steps + 1e-6
    assert abs(r["value"] * 1e9 * r["ms_per_step"] * 1e-3 - step_bytes) / step_bytes < 0.01
    assert r["window_ms"]["p10"] <= r["window_ms"]["median"] <= r["window_ms"]["p90"]
    cpu = r["cpu_baseline"]
    assert cpu["kind"] == "port" and cpu["cores"] >= 1 and cpu["value"] > 0 and cpu["unit"] == "GB/s" and cpu["sample"]
    assert cpu["host_logical_cpus"] >= cpu["cores"] and cpu["cache_resident"]["value"] > 0 and cpu["single_thread"]["value"] > 0
    assert r["parity_ok"] is True


def test_the_drivers_command_measures_steady_state():
    """`bench.py --gpus 1 --steps 20 --warmup 5`, as the round's driver runs it (extras left out here: they are
    covered below).  Twenty steps are 60 us of work; the line must still show the engine's sustained rate: the
    launch's roofline fraction, and the median window's, both above 0.6 of the HBM peak and within 0.05 of each
    other."""
    r = run_bench(["--gpus", "1", "--steps", "20", "--warmup", "5", "--skip-extras", "--cpu-seconds", "0.3"])
    check_contract(r, 20, 5)
    assert r["config"]["fill_steps"] >= 64 and r["config"]["windows"] == 1000
    frac, median_frac = r["roofline"]["frac"], r["window_ms"]["rw_frac_of_hbm_peak_at_median"]
    assert frac > 0.6, r["roofline"]
    assert median_frac > 0.6 and abs(median_frac - frac) < 0.05, (frac, median_frac)
    assert r["single_comm"]["roofline_frac"] > 0.55


def test_bench_prints_one_json_line_with_the_contract_fields():
    r = run_bench(["--steps", "200", "--warmup", "20", "--skip-extras", "--cpu-seconds", "0.2", "--chunks", "8", "--pools", "2"], timeout=300)
    check_contract(r, 200, 20)


def test_bench_extras_report_latency_and_the_storm_sweep():
    r = run_bench(["--steps", "200", "--warmup", "20", "--cpu-seconds", "0.2", "--chunks", "8", "--pools", "2"], timeout=300)
    lat = r["latency_us"]["request_64KiB_16_descs"]
    assert 0 < lat["p50"] <= lat["p99"] and r["p50_request_us"] == lat["p50"]
    deep = r["latency_us"]["budget"]["request_64KiB_16_descs_with_256_in_flight"]
    assert deep["requests"] > 1000 and deep["p50_with_stamps"] > r["latency_us"]["budget"]["request_64KiB_16_descs"]["p50_with_stamps"]
    sweep = r["storm_64KiB"]["sweep"]
    assert [x["requests_in_flight"] for x in sweep] == [4, 8, 16, 32, 64, 128, 256, 512, 1024, 2048]  # up to "2048 concurrent"
    assert r["storm_64KiB"]["requests"] == 16 * 2048 and r["storm_64KiB"]["requests_timed"] == 15 * 2048
    assert all(x["requests_per_s"] > 0 and 0 < x["p50_us"] <= x["p99_us"] for x in sweep)
    # where the time went: the host's cost per publish and what the leader's polls found
    assert all(x["host_ns_per_publish"] > 0 and 0 < x["host_share_of_wall_in_publish"] <= 1 for x in sweep)
    assert all(0 < x["leader_entries_per_poll"] <= 64 and x["leader_polls_per_us"] > 0 for x in sweep)
    assert r["storm_64KiB"]["best"]["requests_per_s"] == max(x["requests_per_s"] for x in sweep)
    assert 1 <= r["plugin_path"]["max_slots_at_gpu"] <= 16
    # the same surface with 32 fragments to the chunk, as the reference's sender cuts a message
    bulk = r["plugin_path"]["in_chunks_of_32_fragments"]
    assert bulk["payload_GBps"] > 0 and 0 < bulk["host_ns_per_fragment"] and 1 <= bulk["max_slots_at_gpu"] <= 16
    assert r["single_comm"]["value"] > 0 and r["plugin_path"]["payload_GBps"] > 0 and r["plain_copy_kernel"]["rw_GBps"] > 0
    assert sorted(r["other_configs"]) == ["config_1", "config_4", "config_5"]
    assert all(v["payload_GBps"] > 0 for v in r["other_configs"].values())
    assert r["launch_per_batch_1GiB"]["kernel"] == "unpack_batch_kernel" and r["launch_per_batch_1GiB"]["rw_GBps"] > 0
    yard = r["hbm_yardsticks"]
    assert yard["read_only_GBps"] > 0 and yard["write_only_GBps"] > 0 and yard["copy_bound_rw_GBps"] > 0
    # the grain of short fragments: bare gathers, and the engine on fragments of one length
    assert all(yard["gather_%dKiB_fragments_rw_GBps" % k] > 0 for k in (1, 2, 4))
    assert sorted(r["fragment_length_sweep"]) == ["fragments_of_1024", "fragments_of_2048", "fragments_of_4096"]
    assert all(0 < v["rw_frac_of_hbm_peak"] < 1 for v in r["fragment_length_sweep"].values())


def test_one_config_mode_launches_the_engine_once_over_another_workload():
    r = run_bench(["--one-config", "1"], timeout=300)
    assert r["kernel"] == "unpack_engine_kernel" and r["slots_in_flight"] == 64 and r["requests_per_pass"] == 1
    assert r["bytes_per_launch"] == 2.0 * (1 << 20) * r["passes"] and r["launch_us"] > 0 and r["payload_GBps"] > 0
