#!/usr/bin/env python3
"""Writes tests/golden/vectors.json: known answers for the oracle, produced WITHOUT the oracle.

Every value below comes from pure-Python integer arithmetic, from Python's math module (the Box-Muller draws), from numpy slicing, or from the
expectation the reference's own test programs state (ramp input and exact comparison,
cudaDMA_test_strided_v2.cu:561-563,659-677; the halo checker cudaDMA_test_halo.cu:91-164; the
integer data of the sgemv driver, sgemv_dma.cu:752-771).  The reference itself is neither
imported nor executed.  tests/test_oracle.py compares oracle/liboracle.so with this file.

    python tests/golden/make_vectors.py
"""
import json
import math
import os

import numpy as np

M64 = (1 << 64) - 1


def splitmix64(x):
    z = (x + 0x9E3779B97F4A7C15) & M64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & M64
    return z ^ (z >> 31)


def hash32(seed, i):
    return splitmix64((seed + i) & M64) >> 32


def uniform_bits(seed, n):
    """float32 bit patterns of (h >> 8) * 2^-23 - 1: exact in binary32, so built from integers."""
    out = []
    for i in range(n):
        v = np.float32(hash32(seed, i) >> 8) * np.float32(2.0 ** -23) - np.float32(1.0)
        out.append(int(np.float32(v).view(np.uint32)))
    return out


def indices(seed, n, n_records):
    out = []
    for i in range(n):
        j = i
        r = hash32(seed ^ 0x5bd1e995, i)
        if i > 1024 and r % 10 == 0:
            j = i - 1 - ((r // 10) % 1024)
        out.append(hash32(seed, j) % n_records)
    return out


def permutation_head(log2_n, seed, count):
    """First entries of the seeded permutation of [0, 2^log2_n) in Python integers."""
    mask = (1 << log2_n) - 1
    h = (log2_n + 1) // 2
    k0, k1 = splitmix64(seed), splitmix64((seed + 1) & M64)
    out = []
    for i in range(min(count, 1 << log2_n)):
        x = i
        x = (x * ((k0 & 0xFFFFFFFF) | 1) + (k0 >> 32)) & mask
        x ^= x >> h
        x = (x * ((k1 & 0xFFFFFFFF) | 1) + (k1 >> 32)) & mask
        x ^= x >> h
        x = (x * 0x9E3779B1) & mask
        out.append(x)
    return out


def normal_bf16_bits(seed, count):
    """(index, bf16 bit pattern) of the first `count` draws of the Box-Muller generator whose value does not lie near
    a rounding boundary of bf16: u1 = ((h(2i) >> 8) + 1) / 2^24, u2 = (h(2i+1) >> 8) / 2^24,
    x = sqrt(-2 ln u1) * cos(2 pi u2) with Python's math module in double precision, rounded to binary32 and then to
    bf16 (nearest even).  A draw is kept when the 16 bits that bf16 drops are at least 2^-8 of a bf16 step away from
    the half-way point, so that neither the last bit of a library's log / cos nor the double rounding matters."""
    out = []
    i = 0
    while len(out) < count:
        u1 = ((hash32(seed, 2 * i) >> 8) + 1) / 16777216.0
        u2 = (hash32(seed, 2 * i + 1) >> 8) / 16777216.0
        x = math.sqrt(-2.0 * math.log(u1)) * math.cos(2.0 * math.pi * u2)
        bits = int(np.float32(x).view(np.uint32))
        dropped = bits & 0xFFFF
        if abs(dropped - 0x8000) >= 0x100:
            out.append([i, (bits + 0x7FFF + ((bits >> 16) & 1)) >> 16])
        i += 1
    return out


def strided_ramp(e_floats, n, src_stride_floats, dst_stride_floats):
    """The reference's strided test: source float(i), every moved element compared exactly."""
    src = np.arange(n * src_stride_floats + e_floats, dtype=np.float32)
    dst = np.full(n * dst_stride_floats + e_floats, -1.0, dtype=np.float32)
    for r in range(n):
        dst[r * dst_stride_floats:r * dst_stride_floats + e_floats] = src[r * src_stride_floats:r * src_stride_floats + e_floats]
    return [int(x) for x in dst]


def halo_ring(dimx, dimy, radius, corners, pitch):
    """Ring of a dimx x dimy tile by numpy slicing; source element (y, x) holds y*pitch + x + 1, untouched cells 0."""
    rows = dimy + 2 * radius
    src = (np.arange(rows * pitch, dtype=np.int64) + 1).reshape(rows, pitch)
    w = dimx + 2 * radius
    dst = np.zeros((rows, w), dtype=np.int64)
    x0 = 0 if corners else radius
    x1 = w if corners else radius + dimx
    dst[:radius, x0:x1] = src[:radius, x0:x1]
    dst[radius + dimy:, x0:x1] = src[radius + dimy:rows, x0:x1]
    dst[radius:radius + dimy, :radius] = src[radius:radius + dimy, :radius]
    dst[radius:radius + dimy, radius + dimx:w] = src[radius:radius + dimy, radius + dimx:w]
    return [int(v) for v in dst.ravel()]


def sgemv_reference_driver(n, m, alpha):
    i, j = np.meshgrid(np.arange(n), np.arange(m), indexing="ij")
    return [int(v) for v in alpha * (((i * j) % 11) @ (np.arange(m) % 11))]


def main():
    vectors = {
        "splitmix64": {str(x): str(splitmix64(x)) for x in (0, 1, 1001, 1234567, 0xDEADBEEFCAFEF00D, M64)},
        "uniform_bits": {str(seed): uniform_bits(seed, 64) for seed in (1001, 1002, 1003, 1004)},
        "indices": {"seed": 1003, "n_records": 4 * 1024 * 1024, "n": 4096, "values": indices(1003, 4096, 4 * 1024 * 1024)},
        "permutations": [{"log2_n": b, "seed": seed, "head": permutation_head(b, seed, 256)}
                         for (b, seed) in ((1, 7), (5, 1006), (16, 1006), (22, 1006), (31, 3))],
        "strided_ramp": [
            {"e_floats": e, "n": n, "src_stride_floats": ss, "dst_stride_floats": ds, "dst": strided_ramp(e, n, ss, ds)}
            for (e, n, ss, ds) in ((16, 5, 40, 16), (3, 7, 9, 5), (64, 4, 64, 68))
        ],
        "halo_ring": [
            {"dimx": dx, "dimy": dy, "radius": r, "corners": c, "pitch": p, "dst": halo_ring(dx, dy, r, c, p)}
            for (dx, dy, r, c, p) in ((8, 6, 2, 0, 16), (8, 6, 2, 1, 16), (32, 32, 4, 0, 48), (5, 3, 1, 1, 9))
        ],
        "normal_bf16": {str(seed): normal_bf16_bits(seed, 192) for seed in (1005, 2005, 7)},
        "sgemv_reference_driver": {"n": 896, "m": 896, "alpha": 2, "y": sgemv_reference_driver(896, 896, 2)},
    }
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "vectors.json")
    with open(path, "w") as f:
        json.dump(vectors, f, separators=(",", ":"))
        f.write("\n")
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
