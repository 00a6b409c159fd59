"""bench.py prints exactly one JSON line with the fields its consumers rely on (short run, GPU)."""
import json
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_bench_prints_one_json_line_with_the_contract_fields():
    p = subprocess.run(
        [sys.executable, os.path.join(ROOT, "bench.py"), "--steps", "200", "--warmup", "20", "--skip-extras", "--cpu-seconds", "0.2", "--chunks", "8", "--pools", "2"],
        stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=300, cwd=ROOT,
    )  # fmt: skip
    assert p.returncode == 0, p.stderr[-2000:]
    lines = [l for l in p.stdout.splitlines() if l.strip()]
    assert len(lines) == 1, p.stdout
    r = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling", "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in r, key
    assert r["n_gpus"] == 1 and r["steps"] == 200 and r["warmup"] == 20 and r["unit"] == "GB/s" and r["dtype"] == "u8"
    assert r["vs_baseline"] is None and r["higher_is_better"] is True and r["data"] == "synthetic" and "workload" in r["config"]
    roof = r["roofline"]
    assert roof["bound"] == "hbm" and roof["peak"] == 8000.0 and roof["unit"] == "GB/s"
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3 and roof["traffic"] >= roof["bytes_per_launch"]
    # value x time of the timed steps = their payload = the launch's payload x timed steps / steps in the launch
    assert roof["steps_per_launch"] >= 220
    timed_payload = roof["bytes_per_launch"] / 2 * 200 / roof["steps_per_launch"]
    assert abs(r["value"] * 1e9 * r["ms_per_step"] * 1e-3 * r["steps"] - timed_payload) / timed_payload < 0.02
    cpu = r["cpu_baseline"]
    assert cpu["kind"] == "port" and cpu["cores"] >= 1 and cpu["value"] > 0 and cpu["unit"] == "GB/s" and cpu["sample"]
    assert r["parity_ok"] is True


def test_bench_extras_report_latency_and_the_storm_sweep():
    p = subprocess.run(
        [sys.executable, os.path.join(ROOT, "bench.py"), "--steps", "200", "--warmup", "20", "--cpu-seconds", "0.2", "--chunks", "8", "--pools", "2"],
        stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=300, cwd=ROOT,
    )  # fmt: skip
    assert p.returncode == 0, p.stderr[-2000:]
    r = json.loads(p.stdout.strip())
    lat = r["latency_us"]["request_64KiB_16_descs"]
    assert 0 < lat["p50"] <= lat["p99"] and r["p50_request_us"] == lat["p50"]
    sweep = r["storm_64KiB"]["sweep"]
    assert [x["descriptors_in_flight"] for x in sweep] == [64, 128, 256, 512, 1024, 2048] and r["storm_64KiB"]["requests"] == 2048
    assert all(x["requests_per_s"] > 0 and 0 < x["p50_us"] <= x["p99_us"] for x in sweep)
    assert r["single_comm"]["value"] > 0 and r["plugin_path"]["payload_GBps"] > 0 and r["plain_copy_kernel"]["rw_GBps"] > 0
    assert sorted(r["other_configs"]) == ["config_1", "config_4", "config_5"]
    assert all(v["payload_GBps"] > 0 for v in r["other_configs"].values())
    assert r["launch_per_batch_1GiB"]["kernel"] == "unpack_batch_kernel" and r["launch_per_batch_1GiB"]["rw_GBps"] > 0
    yard = r["hbm_yardsticks"]
    assert yard["read_only_GBps"] > 0 and yard["write_only_GBps"] > 0 and yard["copy_bound_rw_GBps"] > 0
