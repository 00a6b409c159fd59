"""What the leader's rolling loop must compile to for its counted waits to be sound (no GPU needed: hipcc cross-compiles).

The loop waits for a group of submission entries by counting the wavefront's vector memory instructions
(`s_waitcnt vmcnt(N)`), which is only right if every such instruction in the function completes in the order issued:
no flat_ instruction (free to complete out of turn) and no scratch_ instruction (a spill the count does not know)."""
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "nccl-plugin-gpudirecttcpx_amd", "csrc")


@pytest.fixture(scope="module")
def engine_asm(tmp_path_factory):
    flags = subprocess.check_output(["make", "-s", "-C", CSRC, "print-hipflags"], text=True).split()
    out = tmp_path_factory.mktemp("isa") / "engine.s"
    subprocess.run(["hipcc", *flags, "-S", "--cuda-device-only", "-o", str(out), "hip/engine.hip"], cwd=CSRC, check=True,
                   stdout=subprocess.PIPE, stderr=subprocess.PIPE)  # fmt: skip
    return out.read_text()


def function_body(asm, name):
    start = re.search(r"^(\S*%s\S*):" % name, asm, re.M)
    assert start, "no function %s in the engine's code" % name
    end = asm.index(".size\t" + start.group(1), start.end())
    return asm[start.end() : end]


def test_rolling_loop_has_only_global_memory_instructions_and_counted_waits(engine_asm):
    body = function_body(engine_asm, "leader_storm")
    assert "flat_" not in body and "scratch_" not in body
    loads = re.findall(r"global_load_dword(?:x4)? ", body)
    stores = re.findall(r"global_store_dword", body)
    assert loads and stores
    counted = re.findall(r"s_waitcnt vmcnt\((\d+)\)", body)
    groups = sum(1 for c in counted if c not in ("0",))
    assert groups >= 4, counted  # one counted wait per group in flight
    assert len(set(c for c in counted if c != "0")) == 1, counted  # all of them the same count
    assert int(next(c for c in counted if c != "0")) == 4 * (groups - 1), counted  # two loads and two stores per other group


def test_engine_kernel_uses_no_scratch(engine_asm):
    meta = re.search(r"\.name:\s+\S*unpack_engine_kernel\S*.*?\.private_segment_fixed_size:\s+(\d+)", engine_asm, re.S)
    if meta is None:  # the metadata lists the size before the name in some releases
        meta = re.search(r"\.private_segment_fixed_size:\s+(\d+)(?:(?!\.name:).)*?\.name:\s+\S*unpack_engine_kernel", engine_asm, re.S)
    assert meta and int(meta.group(1)) == 0
