# SPDX-License-Identifier: Apache-2.0
"""The gather kernel's lane logic on the CPU, every access checked.

``tests/kernel_sim`` compiles ``csrc/fstx_gather_core.h`` -- the source the GPU kernel is
built from -- for the host and runs it lane by lane: a load must lie inside one segment of
one source, a store inside the destination's payload, every payload byte must be written
exactly once, and the result must equal numpy's own gather of the same bytes (the oracle's
``shard_bytes`` rule: ``outer`` segments of ``seg`` bytes read ``pitch`` apart).  Sweeps odd
segment lengths, pitches, source and destination alignments, joins of unequal blocks and
pitched destinations -- the shapes that cannot be tried blindly on a GPU.
"""
import ctypes
import os
import subprocess

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
SIM_DIR = os.path.join(HERE, "kernel_sim")


@pytest.fixture(scope="module")
def sim():
    so = os.path.join(SIM_DIR, "libfstx_kernel_sim.so")
    src = [os.path.join(SIM_DIR, "gather_sim.cpp"), os.path.join(HERE, "..", "fastsafetensors_amd", "csrc", "fstx_gather_core.h")]
    if not os.path.exists(so) or any(os.path.getmtime(s) > os.path.getmtime(so) for s in src):
        subprocess.run(["make", "-s", "-C", SIM_DIR], check=True)
    lib = ctypes.CDLL(so)
    lib.fstx_gather_sim.restype = ctypes.c_int64
    lib.fstx_gather_sim.argtypes = [ctypes.c_void_p, ctypes.c_uint64, ctypes.c_uint64, ctypes.c_uint64, ctypes.c_uint64,
                                    ctypes.POINTER(ctypes.c_void_p), ctypes.POINTER(ctypes.c_uint64),
                                    ctypes.POINTER(ctypes.c_uint64), ctypes.c_uint32, ctypes.c_int]
    lib.fstx_div_magic_sim.restype = ctypes.c_uint32
    lib.fstx_div_magic_sim.argtypes = [ctypes.c_uint32, ctypes.c_uint64]
    lib.fstx_sim_set_dies_log2.argtypes = [ctypes.c_uint32]
    lib.fstx_tile_order_sim.restype = ctypes.c_uint64
    lib.fstx_tile_order_sim.argtypes = [ctypes.c_uint32, ctypes.POINTER(ctypes.c_uint32)]
    return lib


def run_case(sim, rng, rows, segs, pitches, src_mis, dst_mis, gap):
    """One job; returns (violations, result equals numpy's gather)."""
    n = len(segs)
    srcs, views = [], []
    for seg, pitch, mis in zip(segs, pitches, src_mis):
        raw = rng.integers(0, 256, rows * pitch + 64, dtype=np.uint8)
        off = (-raw.ctypes.data) % 16 + mis  # the block's first byte sits `mis` past a 16-byte boundary
        srcs.append(raw)
        views.append((raw.ctypes.data + off, off))
    row_bytes = sum(segs)
    dst_pitch = row_bytes + gap
    span = (rows - 1) * dst_pitch + row_bytes
    guard = 64
    buf = np.full(span + 2 * guard + 32, 0xA5, dtype=np.uint8)
    d_off = guard + (-(buf.ctypes.data + guard)) % 16 + dst_mis
    ptrs = (ctypes.c_void_p * n)(*[v[0] for v in views])
    seg_a = (ctypes.c_uint64 * n)(*segs)
    pitch_a = (ctypes.c_uint64 * n)(*pitches)
    # the variant the library would pick for the job, and the fully general one: same bytes either way
    general = sim.fstx_gather_sim(buf.ctypes.data + d_off, d_off, buf.size - d_off, dst_pitch if gap else 0, rows, ptrs,
                                  seg_a, pitch_a, n, 1)
    first = buf.copy()
    buf[:] = 0xA5
    bad = sim.fstx_gather_sim(buf.ctypes.data + d_off, d_off, buf.size - d_off, dst_pitch if gap else 0, rows, ptrs, seg_a,
                              pitch_a, n, 0)
    if general != bad or not np.array_equal(first, buf):
        bad = bad if bad else 999
    want = np.full_like(buf, 0xA5)
    for r in range(rows):
        col = 0
        for (addr, off), raw, seg, pitch in zip(views, srcs, segs, pitches):
            want[d_off + r * dst_pitch + col : d_off + r * dst_pitch + col + seg] = raw[off + r * pitch : off + r * pitch + seg]
            col += seg
    return bad, np.array_equal(buf, want)


@pytest.mark.parametrize("seg,pitch", [(16, 16 + 1), (17, 40), (31, 31 + 33), (64, 100), (70, 282), (254, 1018), (1022, 4090),
                                       (1024, 4096), (1040, 2081), (2046, 8180), (2048, 8190), (4094, 16376), (6912, 27648)])
def test_one_source_every_alignment(sim, seg, pitch):
    """A rank's block of one tensor: all 16 x 16 combinations of source and destination alignment."""
    rng = np.random.default_rng(seg * 7 + pitch)
    rows = max(3, min(40, 9000 // seg + 2))
    for src_mis in range(16):
        for dst_mis in range(16):
            bad, same = run_case(sim, rng, rows, [seg], [pitch], [src_mis], dst_mis, 0)
            assert bad == 0 and same, (seg, pitch, src_mis, dst_mis, bad)


def test_joins_of_unequal_and_equal_blocks(sim):
    rng = np.random.default_rng(11)
    cases = [
        ([1022, 254, 254], [4090, 1018, 1018]),          # q, k, v blocks of odd widths
        ([2046] * 4, [8190] * 4),                        # fp8 [N, 8190] cut in 4, last rank
        ([6912] * 14, [27648] * 14),                     # 14 down_proj column blocks (16-byte multiples)
        ([16, 17, 16, 33], [100, 50, 16, 99]),           # shortest legal segments, one source dense (pitch == seg)
        ([70, 70, 70], [282, 282, 282]),
        ([1500, 20, 1500], [1500, 4096, 3001]),
        ([24] * 24, [24 * 5] * 24),                      # the most sources one call takes
    ]
    for segs, pitches in cases:
        for trial in range(6):
            mis = [int(x) for x in rng.integers(0, 16, len(segs))]
            bad, same = run_case(sim, rng, int(rng.integers(1, 30)), segs, pitches, mis, int(rng.integers(0, 16)), 0)
            assert bad == 0 and same, (segs, pitches, mis, bad)


def test_pitched_destinations(sim):
    """Rows of the destination further apart than their payload: the gap is never written,
    whatever its size (smaller than a vector, a vector, several)."""
    rng = np.random.default_rng(12)
    for segs, pitches in [([2046], [8180]), ([100, 28], [300, 28]), ([6912] * 3, [27648] * 3), ([16], [16]), ([40, 1000], [77, 1003])]:
        for gap in (1, 2, 7, 15, 16, 17, 31, 32, 100, 1024, 5000):
            mis = [int(x) for x in rng.integers(0, 16, len(segs))]
            bad, same = run_case(sim, rng, int(rng.integers(1, 12)), segs, pitches, mis, int(rng.integers(0, 16)), gap)
            assert bad == 0 and same, (segs, gap, bad)


def test_narrow_blocks_in_wide_rows(sim):
    """Gaps that are a large part of the destination: the job's vectors are counted row by row.  Every
    alignment of the first row, row pitches that change the alignment from row to row, blocks shorter and
    longer than a tile, one source and several."""
    rng = np.random.default_rng(17)
    for segs, pitches in [([48], [200]), ([16], [16]), ([17], [90]), ([1000], [4000]), ([1024], [4096]), ([3000], [3001]),
                          ([6912], [27648]), ([100, 28, 500], [300, 28, 777]), ([254, 254], [1018, 1018])]:
        for gap in (16, 17, 24, 32, 100, 1001, 5000, 89856):
            if gap <= (sum(segs) + gap) // 8:
                continue  # such a gap keeps the position-wise count (covered above)
            for dst_mis in (0, 1, 7, 8, 15):
                mis = [int(x) for x in rng.integers(0, 16, len(segs))]
                bad, same = run_case(sim, rng, int(rng.integers(1, 40)), segs, pitches, mis, dst_mis, gap)
                assert bad == 0 and same, (segs, gap, dst_mis, bad)


def test_tiles_of_many_short_segments(sim):
    """Segments under 512 bytes: a tile holds from three to sixty-four of them and every lane finds
    its own.  One source and joins of up to 24, equal and unequal widths, every destination
    alignment, dense and pitched (gaps below and above a vector, and wide enough for the row-wise
    count), enough rows for tiles that lie wholly inside the job."""
    rng = np.random.default_rng(21)
    cases = [([16], [16]), ([16], [40]), ([17], [90]), ([254], [1016]), ([96], [384]), ([94], [377]), ([511], [2044]),
             ([254] * 24, [1016] * 24), ([16] * 24, [64] * 24), ([30, 16, 200], [100, 16, 801]), ([254, 300, 17, 254], [1016, 300, 99, 255]),
             ([100] * 7, [400] * 7), ([48, 48], [200, 4096]), ([510, 16, 510], [2040, 64, 511])]
    for segs, pitches in cases:
        rows = max(6, 9000 // sum(segs) + 3)
        for gap in (0, 0, 1, 15, 16, 40, 3 * sum(segs)):
            for dst_mis in (0, 1, 9, 15):
                mis = [int(x) for x in rng.integers(0, 16, len(segs))]
                bad, same = run_case(sim, rng, rows + int(rng.integers(0, 5)), segs, pitches, mis, dst_mis, gap)
                assert bad == 0 and same, (segs, pitches, gap, dst_mis, bad)


def test_random_geometries(sim):
    rng = np.random.default_rng(13)
    for trial in range(400):
        n = int(rng.choice([1, 1, 1, 2, 3, 5]))
        segs = [int(rng.integers(16, 3000 if trial % 2 else 300)) for _ in range(n)]
        if rng.random() < 0.3:
            segs = [segs[0]] * n
        pitches = [s + int(rng.integers(0, 2000)) for s in segs]
        rows = int(rng.integers(1, max(2, 20000 // sum(segs))))
        gap = int(rng.choice([0, 0, 0, int(rng.integers(1, 300))]))
        mis = [int(x) for x in rng.integers(0, 16, n)]
        bad, same = run_case(sim, rng, rows, segs, pitches, mis, int(rng.integers(0, 16)), gap)
        assert bad == 0 and same, (trial, segs, pitches, rows, gap, mis, bad)


@pytest.mark.parametrize("dies", [8, 4, 2, 1])
@pytest.mark.parametrize("n_tiles", [1, 7, 8, 9, 255, 2047, 2048, 2049, 2056, 4095, 4096, 6000, 3 * 2048 + 1, 100_003])
def test_tile_order_visits_every_tile_once_and_keeps_neighbours_on_a_die(sim, n_tiles, dies):
    """For a device of 8, 4, 2 dies, and one die (where the order is the dispatch order)."""
    sim.fstx_sim_set_dies_log2(dies.bit_length() - 1)
    try:
        out = np.empty((n_tiles + dies - 1) // dies * dies, dtype=np.uint32)
        groups = sim.fstx_tile_order_sim(n_tiles, out.ctypes.data_as(ctypes.POINTER(ctypes.c_uint32)))
    finally:
        sim.fstx_sim_set_dies_log2(3)
    assert groups == out.size
    live = out[out != 0xFFFFFFFF]
    assert live.size == n_tiles and np.array_equal(np.sort(live), np.arange(n_tiles, dtype=np.uint32))
    # workgroup b runs on die b % dies: a die's tiles come in runs of consecutive tiles (256 long in whole
    # chunks), in ascending order, so a line shared by two neighbouring tiles is used twice by one die
    chunk = 256 * dies
    die_of = np.empty(n_tiles, dtype=np.int64)
    idx = np.nonzero(out != 0xFFFFFFFF)[0]
    die_of[out[idx]] = idx % dies
    changes = int(np.count_nonzero(np.diff(die_of)))
    assert changes <= dies * (n_tiles // chunk + 1)
    for d in range(dies):
        mine = out[d::dies]
        mine = mine[mine != 0xFFFFFFFF].astype(np.int64)
        assert np.all(np.diff(mine) > 0)
    # all dies work inside one window of 256 x dies tiles at a time
    full = n_tiles // chunk * chunk
    assert np.array_equal(out[:full] // chunk, np.arange(full) // chunk)
    if dies == 1:
        assert np.array_equal(out, np.arange(n_tiles, dtype=np.uint32))


@pytest.mark.parametrize("dies_log2", [0, 1, 2])
def test_jobs_on_a_partitioned_device(sim, dies_log2):
    """The same bytes whatever number of dies the launch is dealt out to."""
    sim.fstx_sim_set_dies_log2(dies_log2)
    try:
        rng = np.random.default_rng(30 + dies_log2)
        for segs, pitches, rows, gap in [([2046], [8180], 700, 0), ([254] * 5, [1016] * 5, 60, 0), ([94], [377], 300, 4000),
                                         ([1022, 254, 254], [4090, 1018, 1018], 40, 7)]:
            mis = [int(x) for x in rng.integers(0, 16, len(segs))]
            bad, same = run_case(sim, rng, rows, segs, pitches, mis, int(rng.integers(0, 16)), gap)
            assert bad == 0 and same, (segs, rows, gap, bad)
    finally:
        sim.fstx_sim_set_dies_log2(3)


def test_division_by_multiplication_is_exact(sim):
    """The kernel divides positions by the row pitch and by the segment length with one multiply-high;
    exact for every 32-bit numerator: checked at the multiples of the divisor and either side of them,
    at the ends of the range, for small, odd, even, power-of-two and huge divisors."""
    rng = np.random.default_rng(16)
    ds = [2, 3, 5, 7, 16, 17, 31, 32, 33, 254, 1022, 2046, 2048, 4094, 6912, 8180, 8190, 96768, 65536, 65537,
          (1 << 31) - 1, 1 << 31, (1 << 31) + 1, (1 << 32) - 1] + [int(x) for x in rng.integers(2, 1 << 32, 200)]
    top = (1 << 32) - 1
    for d in ds:
        ns = {0, 1, d - 1, d, d + 1, top, top - 1, top // d * d, top // d * d - 1}
        for m in rng.integers(0, top // d + 1, 40):
            ns.update((int(m) * d - 1, int(m) * d, int(m) * d + 1))
        ns.update(int(x) for x in rng.integers(0, 1 << 32, 40))
        for n in ns:
            if 0 <= n <= top:
                assert sim.fstx_div_magic_sim(n, d) == n // d, (n, d)


def test_a_job_of_several_chunks(sim):
    rng = np.random.default_rng(15)
    # 2046-byte segments, 2700 rows: 5.5 MB = 5395 tiles, two whole chunks and a partial one
    bad, same = run_case(sim, rng, 2700, [2046], [8180], [6], 3, 0)
    assert bad == 0 and same
    bad, same = run_case(sim, rng, 900, [2046, 1022, 3000], [8180, 4090, 3001], [1, 2, 3], 5, 0)
    assert bad == 0 and same


def test_shapes_outside_the_kernels_domain_are_refused(sim):
    rng = np.random.default_rng(14)
    assert run_case(sim, rng, 4, [15], [100], [0], 0, 0)[0] == -1      # a segment shorter than a vector
    assert run_case(sim, rng, 4, [64, 8], [64, 8], [0, 0], 0, 0)[0] == -1
