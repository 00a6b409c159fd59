"""Writes tests/golden/plugin_host_fixture.bin: three receive requests for a host that drives the plugin through
its `ncclNetPlugin_v7` table (tests/native/plugin_dlopen_host.cc), and the bytes their buffers must hold.

Request 0: 24 fragments of ragged length with byte-unaligned sources, on 4 flows in turn.  Request 1: the empty
message.  Request 2: 8 whole pages on 4 flows, two in a row per flow.  The bounce pool is not stored: both sides
make it from `pool_seed` with splitmix64, eight little-endian bytes per step.  The expected receive buffer is
computed here fragment by fragment, byte by byte, in plain Python -- no library routine, no oracle, no product
code.  Run from the repository root:  python tests/golden/make_plugin_fixture.py

Layout (little endian): "TCPXFIX1"; u32 pool_bytes, dst_bytes, n_frags, n_requests; u64 pool_seed;
n_frags x {u32 frag_offset, frag_size, frag_token, flow}; n_requests x {u64 first_desc, dst_off; u32 n_descs,
bytes, window, reserved}; dst_bytes expected bytes (0xA5 where nothing is received).
"""
import os
import struct

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
SENTINEL = 0xA5
MASK = (1 << 64) - 1


def splitmix64_bytes(seed, nbytes):
    out = bytearray()
    x = seed
    while len(out) < nbytes:
        x = (x + 0x9E3779B97F4A7C15) & MASK
        z = x
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & MASK
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & MASK
        z ^= z >> 31
        out += struct.pack("<Q", z)
    return bytes(out[:nbytes])


def main():
    rng = np.random.default_rng(0xF1C5)
    pool_pages, pool_seed = 64, 0x7C9F1D5A
    pool_bytes = pool_pages * 4096
    pool = splitmix64_bytes(pool_seed, pool_bytes)
    pages = [int(p) for p in rng.permutation(pool_pages)]
    frags, requests = [], []
    dst_pos = 0

    def add_request(lengths, flows):
        nonlocal dst_pos
        first = len(frags)
        total = 0
        for length, flow in zip(lengths, flows):
            page = pages.pop()
            in_page = int(rng.integers(0, 4096 - length + 1))
            frags.append((page * 4096 + in_page, length, page, flow))
            total += length
        requests.append((first, dst_pos, len(lengths), total, 0, 0))
        dst_pos += total

    add_request([int(rng.integers(1, 4097)) for _ in range(24)], [i % 4 for i in range(24)])
    add_request([], [])
    add_request([4096] * 8, [(i // 2) % 4 for i in range(8)])
    dst_bytes = dst_pos + 64
    expect = [SENTINEL] * dst_bytes
    for first, dst_off, n, total, _, _ in requests:
        pos = dst_off
        for off, length, _, _ in frags[first : first + n]:
            for k in range(length):
                expect[pos + k] = pool[off + k]
            pos += length
        assert pos - dst_off == total
    with open(os.path.join(HERE, "plugin_host_fixture.bin"), "wb") as f:
        f.write(b"TCPXFIX1")
        f.write(struct.pack("<IIIIQ", pool_bytes, dst_bytes, len(frags), len(requests), pool_seed))
        for fr in frags:
            f.write(struct.pack("<IIII", *fr))
        for rq in requests:
            f.write(struct.pack("<QQIIII", *rq))
        f.write(bytes(expect))
    print("wrote %d fragments, %d requests, %d destination bytes" % (len(frags), len(requests), dst_bytes))


if __name__ == "__main__":
    main()
