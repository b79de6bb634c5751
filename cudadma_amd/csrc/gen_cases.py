#!/usr/bin/env python3
"""Writes the compile-time case lists of the known-answer harness (cases_*.inc).

The random part follows the parameter distribution of the reference's fuzz
drivers (src/tests/test_strided/param_sweep_v2.py:51-75 and its siblings):
ALIGNMENT in {4,8,16}, BYTES_PER_THREAD = ALIGNMENT * U{1..8}, element size
|N(256,256)| floats, NUM_ELMTS ~ U{1..32}, DMA warps ~ U{1..16}; here it is a
fixed, seeded list instead of an endless loop, wavefronts have 64 lanes, and the
template level and the warp-specialised flag cycle so that every constructor
form is compiled.  A directed part pins the full benchmark shapes and the edge cases
(4/8/12-byte tails, one element, one wavefront, many steps).

Run from this directory:  python3 gen_cases.py
"""
import math
import os
import random

HERE = os.path.dirname(os.path.abspath(__file__))
LDS_CAP = 40 * 1024          # bytes of LDS a case may need (the reference caps at ~41 KB)
MAX_WS_WAVES = 15            # 64 compute threads + 15 DMA wavefronts = 1024 threads


def rnd_align(r):
    return r.choice([4, 8, 16])


def rnd_elmt_bytes(r, cap):
    while True:
        floats = abs(int(math.ceil(r.gauss(256, 256))))
        if floats >= 1 and floats * 4 <= cap:
            return floats * 4


def sequential_cases():
    r = random.Random(20240601)
    out = []
    directed = [
        # ws level A  BPT   E     T
        (1, 3, 16, 128, 16384, 128),   # benchmark config 1 tile: 8 dwordx4 per lane, one step
        (1, 3, 16, 64, 16384, 128),    # same tile in two steps
        (1, 2, 16, 32, 16384, 64),     # one wavefront, many steps
        (1, 1, 16, 16, 4, 64),         # smallest transfer
        (1, 3, 16, 64, 8, 64), (1, 3, 16, 64, 12, 64), (1, 3, 16, 64, 20, 128),
        (1, 2, 16, 64, 1024 + 4, 64), (1, 1, 16, 64, 1024 + 8, 64), (0, 3, 16, 64, 1024 + 12, 64),
        (0, 1, 8, 16, 8 * 64 * 2 + 4, 64), (0, 2, 4, 4, 4 * 64 * 3, 64),
        (1, 3, 4, 32, 36860, 192), (0, 3, 8, 64, 40000, 960),
        (1, 1, 16, 64, 0, 64), (0, 1, 4, 16, 0, 128),            # empty transfer (run-time size 0)
        (1, 3, 16, 128, 64000, 128), (0, 2, 16, 256, 65200, 256),  # as large as the LDS window allows
    ]
    for c in directed:
        out.append(c)
    combos = [(ws, lv) for ws in (1, 0) for lv in (1, 2, 3)]
    for i in range(36):
        ws, lv = combos[i % len(combos)]
        a = rnd_align(r)
        bpt = a * r.randint(1, 8)
        e = rnd_elmt_bytes(r, LDS_CAP - 64)
        t = 64 * r.randint(1, MAX_WS_WAVES)
        out.append((ws, lv, a, bpt, e, t))
    return out


def grid_cases(seed, n_random, with_gather):
    r = random.Random(seed)
    out = []
    combos = [(ws, lv) for ws in (1, 0) for lv in (1, 2, 3, 4)]
    directed = [
        # ws lv  A  BPT   E    T   N
        (1, 4, 16, 128, 256, 128, 64),    # benchmark config 2 tile: 64 rows x 256 B, one step
        (1, 4, 16, 64, 256, 128, 64),     # same in two steps
        (1, 4, 16, 64, 128, 128, 32),     # benchmark config 3 tile: 32 records x 128 B
        (1, 3, 16, 64, 128, 128, 128),    # GEMM A tile: 128 rows x 128 B
        (1, 2, 16, 64, 4, 64, 1), (1, 1, 16, 64, 12, 64, 7), (0, 4, 16, 32, 20, 64, 5),
        (1, 4, 16, 32, 2048, 128, 3),     # rows wider than one wavefront load
        (1, 3, 16, 16, 4096 + 8, 64, 2),  # wide rows with a tail, many steps
        (0, 2, 8, 8, 1000, 128, 9), (0, 1, 4, 4, 132, 192, 31),
        (1, 4, 16, 128, 1040, 256, 16),   # 65 loads per row: two wavefront loads per row, half idle
        (0, 3, 16, 64, 512, 960, 32),     # more threads than slots
        (1, 1, 16, 64, 256, 64, 0), (0, 3, 8, 32, 64, 128, 0),   # no elements (run-time count 0)
        (1, 4, 16, 128, 16000, 256, 4),   # four rows that fill the LDS window
    ]
    for c in directed:
        out.append(c)
    for i in range(n_random):
        ws, lv = combos[i % len(combos)]
        a = rnd_align(r)
        bpt = a * r.randint(1, 8)
        n = r.randint(1, 32)
        e = rnd_elmt_bytes(r, max(4, (LDS_CAP // n) - 16))
        t = 64 * r.randint(1, MAX_WS_WAVES)
        out.append((ws, lv, a, bpt, e, t, n))
    return out


def halo_cases():
    r = random.Random(77)
    out = []
    # ws level A BPT ES T R C DX DY
    directed = [
        (1, 3, 16, 64, 4, 128, 4, 0, 32, 32),   # benchmark config 4 ring
        (1, 3, 16, 16, 4, 64, 4, 0, 32, 32),    # same ring, one load per step
        (1, 2, 16, 64, 4, 128, 4, 1, 32, 32),
        (1, 0, 4, 16, 4, 64, 1, 0, 8, 8), (1, 0, 4, 16, 4, 128, 3, 1, 17, 9),
        (1, 0, 4, 16, 8, 64, 2, 1, 13, 21), (1, 0, 4, 16, 16, 192, 5, 0, 11, 10),
        (0, 3, 8, 32, 4, 64, 2, 1, 16, 8), (0, 1, 4, 8, 4, 256, 8, 1, 63, 20),
    ]
    for c in directed:
        out.append(c)
    combos = [(1, 0), (1, 1), (1, 2), (1, 3), (0, 1), (0, 2), (0, 3)]
    for i in range(28):
        ws, lv = combos[i % len(combos)]
        es = r.choice([4, 4, 8, 16])
        radius = r.randint(1, 8)
        corners = r.randint(0, 1)
        # ALIGNMENT must divide 2*RADIUS*ES (the destination pitch is (dimx+2R)*ES) and dimx*ES
        a = 4 if lv == 0 else r.choice([x for x in (4, 8, 16) if (2 * radius * es) % x == 0])
        unit = max(1, a // es)
        dimx = unit * r.randint(max(1, 8 // unit), max(1, 63 // unit))
        dimy = r.randint(8, 40)
        while (dimx + 2 * radius) * (dimy + 2 * radius) * es > LDS_CAP:
            dimy = max(1, dimy // 2)
            if dimy == 1:
                dimx = max(unit, (dimx // 2 // unit) * unit)
        bpt = 4 * a if lv == 0 else a * r.randint(1, 8)
        t = 64 * r.randint(1, MAX_WS_WAVES)
        out.append((ws, lv, a, bpt, es, t, radius, corners, dimx, dimy))
    return out


def write(name, lines):
    path = os.path.join(HERE, name)
    with open(path, "w") as f:
        f.write("// Generated by gen_cases.py; do not edit.\n")
        f.write("// A harness source is compiled in HARNESS_SHARDS pieces (see the Makefile): piece HARNESS_SHARD\n")
        f.write("// holds the cases whose number leaves that remainder.\n")
        for i, line in enumerate(lines):
            f.write(f"#if ({i} % HARNESS_SHARDS) == HARNESS_SHARD\n{line}\n#endif\n")
    print(f"{name}: {len(lines)} cases")


def main():
    seq = sequential_cases()
    write("cases_sequential.inc",
          [f"SEQ_CASE({i}, {bool_s(ws)}, {lv}, {a}, {bpt}, {e}, {t})" for i, (ws, lv, a, bpt, e, t) in enumerate(seq)])
    strided = grid_cases(4242, 40, False)
    write("cases_strided.inc",
          [f"STRIDED_CASE({i}, {bool_s(ws)}, {lv}, {bool_s(i % 4 == 3)}, {a}, {bpt}, {e}, {t}, {n})"
           for i, (ws, lv, a, bpt, e, t, n) in enumerate(strided)])
    # the sparse side of an indirect transfer holds n + 3 elements in the tests: it has to fit LDS
    ind = [c for c in grid_cases(977, 32, True) if (c[6] + 3) * c[4] <= 60000]
    lines = []
    for i, (ws, lv, a, bpt, e, t, n) in enumerate(ind):
        gather = (i % 3) != 2          # two thirds gather, one third scatter
        # element k of the sparse side starts at k*E: ALIGNMENT has to divide E
        while e % a:
            a //= 2
        bpt = max(a, bpt // a * a)
        lines.append(f"INDIRECT_CASE({i}, {bool_s(gather)}, {bool_s(ws)}, {lv}, {a}, {bpt}, {e}, {t}, {n})")
    write("cases_indirect.inc", lines)
    halo = halo_cases()
    write("cases_halo.inc",
          [f"HALO_CASE({i}, {bool_s(ws)}, {lv}, {a}, {bpt}, {es}, {t}, {rad}, {c}, {dx}, {dy})"
           for i, (ws, lv, a, bpt, es, t, rad, c, dx, dy) in enumerate(halo)])


def bool_s(v):
    return "true" if v else "false"


if __name__ == "__main__":
    main()
