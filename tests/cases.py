"""Inputs, run arguments and oracle-made expectations for the known-answer cases
of the harness.  Shared by the CPU replay tests and the GPU parity tests."""
import numpy as np

import cudadma_amd as cd
from tests import oracle_lib as ol
from tests.oracle_lib import ptr


def _round_up(v, m):
    return (v + m - 1) // m * m


class CaseIO:
    """Everything one run of a case needs, plus what the LDS buffer must hold afterwards."""

    def __init__(self, case, flavour=0, reps=2, data="ramp", reverse=False, dst_pitch=None):
        self.case = case
        self.reps = reps
        self.reverse = reverse
        a = case.alignment
        rng = np.random.default_rng(1000 * case.pattern + 17 * flavour + case.bytes_per_elmt + case.dma_threads)
        self.index = None
        self.src_stride = self.dst_stride = self.pitch = self.dst_pitch = 0
        self.rep_index_elmts = 0
        self.src_offset = a * (flavour % 3)
        self.dst_offset = a * ((flavour + 1) % 2)
        self.rep_src_bytes = a * 3
        pat = case.pattern
        e, n = case.bytes_per_elmt, case.num_elmts
        if pat == cd.PATTERN_SEQUENTIAL:
            footprint_src = footprint_dst = e
        elif pat == cd.PATTERN_STRIDED:
            one_stride = case.dimx == 1
            self.src_stride = _round_up(e, a) + a * (2 + flavour % 2)
            self.dst_stride = self.src_stride if one_stride else _round_up(e, a) + a * (flavour % 2)
            footprint_src = n * self.src_stride
            footprint_dst = n * self.dst_stride
        elif pat == cd.PATTERN_GATHER:
            self.table_elmts = (n + 3) if reverse else (2 * n + 3)   # the table sits in LDS when reversed
            alt = 0 if flavour % 2 == 0 else e + a
            self.dst_stride = alt
            footprint_src = self.table_elmts * e
            footprint_dst = n * max(alt, e)
            self.rep_src_bytes = 0
            self.rep_index_elmts = n
            idx = rng.integers(0, self.table_elmts, size=max(1, reps * n)).astype(np.int32)
            if idx.size:
                idx[1::5] = idx[0]                               # duplicates
            self.index = idx
        elif pat == cd.PATTERN_SCATTER:
            self.table_elmts = n + 3                              # elements the sparse side holds
            alt = 0 if flavour % 2 == 0 else e + a
            self.src_stride = alt
            footprint_src = n * max(alt, e)
            footprint_dst = self.table_elmts * e
            self.rep_index_elmts = n
            self.index = np.concatenate([rng.permutation(self.table_elmts)[:n] for _ in range(reps)]).astype(np.int32)
            if self.index.size == 0:
                self.index = np.zeros(1, dtype=np.int32)         # a valid pointer for an empty index list
        elif pat == cd.PATTERN_HALO:
            r, dimx, dimy = case.radius, case.dimx, case.dimy
            unit = max(1, a // e)
            self.pitch = _round_up(dimx + 2 * r + (flavour % 3), unit)
            # every third flavour of the v2-style classes widens the destination rows (0 = the reference's dimx + 2R)
            if dst_pitch is None:
                dst_pitch = _round_up(dimx + 2 * r + 1 + flavour % 5, unit) if (case.level >= 1 and flavour % 3 == 2) else 0
            self.dst_pitch = dst_pitch
            self.dst_cells = dst_pitch if dst_pitch > 0 else dimx + 2 * r
            src_origin = (r * self.pitch + r) * e
            dst_origin = (r * self.dst_cells + r) * e
            self.src_offset = (-src_origin) % a
            self.dst_offset = (-dst_origin) % a
            self.rep_src_bytes = a
            footprint_src = (dimy + 2 * r) * self.pitch * e
            footprint_dst = self.dst_cells * (dimy + 2 * r) * e
        else:
            raise ValueError(pat)
        if reverse:
            # LDS holds the source image, the destination is a window of global memory
            self.lds_bytes = _round_up(self.src_offset + footprint_src + 16, 16)
            self.out_bytes = _round_up(self.dst_offset + footprint_dst + 16, 16)
            in_bytes = _round_up(self.lds_bytes + reps * self.rep_src_bytes + 64, 16)
        else:
            self.lds_bytes = _round_up(self.dst_offset + footprint_dst + 16, 16)
            self.out_bytes = 0
            in_bytes = _round_up(self.src_offset + footprint_src + reps * self.rep_src_bytes + 64, 16)
        if data == "ramp":
            # the reference tests' input: h_idata[i] = float(i)
            self.input = ol.ramp(in_bytes // 4).view(np.uint8)
        else:
            self.input = ol.uniform(in_bytes // 4, 4242 + flavour).view(np.uint8)

    # -- the closed form, applied by the oracle to byte buffers -------------------------------
    def apply_oracle(self, src, dst, rep, shift_src=True, swizzle=False):
        """Moves what the case's object moves: src/dst are numpy uint8 arrays standing for
        the source and the destination buffer of one transfer."""
        O = ol.load()
        c = self.case
        so = self.src_offset + (rep * self.rep_src_bytes if shift_src else 0)
        do = self.dst_offset
        e, n = c.bytes_per_elmt, c.num_elmts
        idx = self.index[rep * self.rep_index_elmts:] if self.index is not None else None
        if c.pattern == cd.PATTERN_SEQUENTIAL:
            O.oracle_sequential(ptr(src, so), ptr(dst, do), e)
        elif c.pattern == cd.PATTERN_STRIDED and swizzle:
            O.oracle_strided_swizzled(ptr(src, so), ptr(dst, do), e, n, self.src_stride, self.dst_stride, c.alignment)
        elif c.pattern == cd.PATTERN_STRIDED:
            O.oracle_strided(ptr(src, so), ptr(dst, do), e, n, self.src_stride, self.dst_stride)
        elif c.pattern == cd.PATTERN_GATHER:
            O.oracle_gather(ptr(idx), ptr(src, so), ptr(dst, do), e, n, self.dst_stride)
        elif c.pattern == cd.PATTERN_SCATTER:
            O.oracle_scatter(ptr(idx), ptr(src, so), ptr(dst, do), e, n, self.src_stride)
        else:
            r = c.radius
            O.oracle_halo_pitched(ptr(src, so + (r * self.pitch + r) * e), ptr(dst, do + (r * self.dst_cells + r) * e),
                                  e, r, c.corners, c.dimx, c.dimy, self.pitch, self.dst_cells)

    def expected(self, swizzle=False):
        if self.reverse:
            out = np.zeros((self.reps, self.out_bytes), dtype=np.uint8)
            for rep in range(self.reps):
                image = np.ascontiguousarray(self.input[rep * self.rep_src_bytes:rep * self.rep_src_bytes + self.lds_bytes])
                self.apply_oracle(image, out[rep], rep, shift_src=False)
            return out
        out = np.zeros((self.reps, self.lds_bytes), dtype=np.uint8)
        for rep in range(self.reps):
            self.apply_oracle(self.input, out[rep], rep, swizzle=swizzle)
        return out

    def expected_map(self, rep=0):
        """For every LDS byte the input byte that must land there (-1 = untouched), obtained by
        running the oracle on 4-byte ids: all sizes, strides and offsets scaled by four."""
        c = self.case
        O = ol.load()
        ids = np.arange(self.input.size, dtype=np.int32)
        dst = np.full(self.lds_bytes, -1, dtype=np.int32)
        so = 4 * (self.src_offset + rep * self.rep_src_bytes)
        do = 4 * self.dst_offset
        e, n = 4 * c.bytes_per_elmt, c.num_elmts
        idx = self.index[rep * self.rep_index_elmts:] if self.index is not None else None
        if c.pattern == cd.PATTERN_SEQUENTIAL:
            O.oracle_sequential(ptr(ids, so), ptr(dst, do), e)
        elif c.pattern == cd.PATTERN_STRIDED:
            O.oracle_strided(ptr(ids, so), ptr(dst, do), e, n, 4 * self.src_stride, 4 * self.dst_stride)
        elif c.pattern == cd.PATTERN_GATHER:
            O.oracle_gather(ptr(idx), ptr(ids, so), ptr(dst, do), e, n, 4 * self.dst_stride)
        elif c.pattern == cd.PATTERN_SCATTER:
            O.oracle_scatter(ptr(idx), ptr(ids, so), ptr(dst, do), e, n, 4 * self.src_stride)
        else:
            r = c.radius
            O.oracle_halo_pitched(ptr(ids, so + 4 * (r * self.pitch + r) * c.bytes_per_elmt),
                                  ptr(dst, do + 4 * (r * self.dst_cells + r) * c.bytes_per_elmt),
                                  e, r, c.corners, c.dimx, c.dimy, self.pitch, self.dst_cells)
        return dst

    def replay_map(self, rep=0):
        """The same map, from the host replay of the device objects' own index arithmetic."""
        c = self.case
        e = c.bytes_per_elmt
        src_origin = self.src_offset + rep * self.rep_src_bytes
        dst_origin = self.dst_offset
        if c.pattern == cd.PATTERN_HALO:
            src_origin += (c.radius * self.pitch + c.radius) * e
            dst_origin += (c.radius * self.dst_cells + c.radius) * e
        idx = self.index[rep * self.rep_index_elmts:rep * self.rep_index_elmts + c.num_elmts] \
            if self.index is not None else None
        return cd.plan.plan_map(
            c.pattern, alignment=c.alignment, bytes_per_thread=c.bytes_per_thread, bytes_per_elmt=e,
            dma_threads=c.dma_threads, num_elmts=c.num_elmts, src_stride=self.src_stride,
            dst_stride=self.dst_stride, radius=c.radius, corners=c.corners,
            dimx=(c.dimx if c.pattern == cd.PATTERN_HALO else 0), dimy=c.dimy, pitch=self.pitch,
            dst_pitch=self.dst_pitch, index=idx,
            src_origin=src_origin, dst_origin=dst_origin, map_len=self.lds_bytes)


def case_id_str(case_id, case):
    name = cd._lib.PATTERN_NAMES[case.pattern]
    return (f"{case_id}-{name}-{'ws' if case.warp_specialized else 'all'}-L{case.level}-A{case.alignment}"
            f"-bpt{case.bytes_per_thread}-E{case.bytes_per_elmt}-T{case.dma_threads}-N{case.num_elmts}"
            + (f"-R{case.radius}c{case.corners}-{case.dimx}x{case.dimy}" if case.pattern == cd.PATTERN_HALO else ""))
