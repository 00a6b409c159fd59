"""Writes tests/golden/unpack_vectors.npz: seeded descriptor lists, pools and the destination they must produce.

The expected destinations are computed here by a byte-at-a-time Python loop (no library, no oracle, no product
code), so the fixture is an independent statement of  dst[dst_off + k] = pool[src_off + k].  Run from the
repository root:  python tests/golden/make_vectors.py
"""
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
SENTINEL = 0xA5


def brute_force(pool, descs, dst_bytes):
    dst = [SENTINEL] * dst_bytes
    for src_off, length, dst_off in descs:
        for k in range(length):
            dst[dst_off + k] = int(pool[src_off + k])
    return np.array(dst, dtype=np.uint8)


def case(seed, n, pool_bytes, contiguous, max_len):
    rng = np.random.default_rng(seed)
    pool = rng.integers(0, 256, size=pool_bytes, dtype=np.uint8)
    descs, pos = [], int(rng.integers(0, 40))
    for _ in range(n):
        length = int(rng.integers(0, max_len + 1)) if rng.random() > 0.1 else 0
        page = int(rng.integers(0, pool_bytes // 4096))
        in_page = int(rng.integers(0, 4096 - length + 1)) if length <= 4096 else 0
        if not contiguous:
            pos += int(rng.integers(0, 70))
        descs.append((page * 4096 + in_page, length, pos))
        pos += length
    dst_bytes = pos + int(rng.integers(1, 40))
    return pool, np.array(descs, dtype=np.uint64).reshape(-1, 3), brute_force(pool, descs, dst_bytes)


def main():
    out = {}
    specs = [(1, 40, 1 << 13, True, 300), (2, 60, 1 << 13, False, 100), (3, 25, 1 << 14, True, 4096), (4, 200, 1 << 13, True, 40)]
    for i, spec in enumerate(specs):
        pool, descs, expect = case(*spec)
        out["pool_%d" % i], out["descs_%d" % i], out["expect_%d" % i] = pool, descs, expect
    np.savez_compressed(os.path.join(HERE, "unpack_vectors.npz"), **out)
    print("wrote", len(specs), "cases")


if __name__ == "__main__":
    main()
