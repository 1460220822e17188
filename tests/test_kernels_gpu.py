# SPDX-License-Identifier: Apache-2.0
"""GPU parity of the two HBM kernels, called through the C ABI, against the CPU oracle.

Bit-exact is the bar (pure byte movement).  Device memory and streams come from
torch; the kernels are libfstx's.
"""
import itertools

import numpy as np
import pytest
import torch

from fastsafetensors_amd import _native
from oracle import st_oracle as orc

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    assert _native.device_count() > 0
    return torch.device("cuda:0")


def stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def rand_bytes(n: int, seed: int) -> np.ndarray:
    return np.random.default_rng(seed).integers(0, 256, n, dtype=np.uint8)


def to_dev(a: np.ndarray, dev, pad: int = 64) -> torch.Tensor:
    """Device copy of ``a`` with ``pad`` guard bytes on both sides (value 0xA5)."""
    host = np.full(a.size + 2 * pad, 0xA5, dtype=np.uint8)
    host[pad : pad + a.size] = a
    return torch.from_numpy(host).to(dev)


# ---- realign copy -------------------------------------------------------------------------

SIZES = [0, 1, 2, 15, 16, 17, 31, 33, 255, 256, 4095, 4096, 4097, 65536 + 5, (1 << 20) + 3]


def test_realign_all_alignments(dev):
    """Every (src % 16, dst % 16) pair at sizes around the 16-byte and 4 KiB edges;
    guard bytes around the destination must stay untouched."""
    src_host = rand_bytes((1 << 20) + 256, 1)
    src = torch.from_numpy(src_host).to(dev)
    for n in SIZES:
        dst = torch.full((n + 256,), 0xA5, dtype=torch.uint8, device=dev)
        for so, do in itertools.product(range(16), range(16)):
            if n > 70000 and (so * 16 + do) % 37:  # thin out the big sizes
                continue
            dst.fill_(0xA5)
            _native.realign_copy(dst.data_ptr() + 64 + do, src.data_ptr() + so, n, stream())
            got = dst.cpu().numpy()
            assert np.array_equal(got[64 + do : 64 + do + n], src_host[so : so + n]), (n, so, do)
            assert (got[: 64 + do] == 0xA5).all() and (got[64 + do + n :] == 0xA5).all(), (n, so, do)


def test_realign_matches_reference_memmove_semantics(dev):
    """Shifting a window down by header_length % 16, as copier/gds.py:138-159 does
    through a temporary: compare with the oracle's memmove."""
    for header_length in (104, 4096 + 2, 8192 + 10, 12288 + 15):
        lead = header_length % 4096
        window = rand_bytes(lead + 300_001, header_length)
        want = orc.realign(window, header_length, header_length - lead, 300_001)
        w = torch.from_numpy(window).to(dev)
        out = torch.empty(300_001, dtype=torch.uint8, device=dev)
        _native.realign_copy(out.data_ptr(), w.data_ptr() + lead, 300_001, stream())
        assert np.array_equal(out.cpu().numpy(), want)
        # DeviceBuffer.memmove (two copies through tmp) gives the same bytes in place
        buf = _native.DeviceBuffer(w.data_ptr(), w.numel(), True, w)
        tmp_t = torch.empty(300_001, dtype=torch.uint8, device=dev)
        tmp = _native.DeviceBuffer(tmp_t.data_ptr(), tmp_t.numel(), True, tmp_t)
        assert buf.memmove(0, lead, tmp, 300_001) == 0
        assert np.array_equal(w.cpu().numpy()[:300_001], want)


def test_realign_batch_many_jobs(dev):
    rng = np.random.default_rng(5)
    src_host = rand_bytes(3_000_000, 2)
    src = torch.from_numpy(src_host).to(dev)
    jobs, spans, at = [], [], 0
    dst = torch.full((4_000_000,), 0xA5, dtype=torch.uint8, device=dev)
    for i in range(131):  # more than FSTX_BATCH_MAX: split into launches
        n = int(rng.choice([0, 1, 4, 7, 16, 100, 4096, 20000, 70001]))
        so = int(rng.integers(0, src_host.size - n))
        at += int(rng.integers(0, 40))
        jobs.append((dst.data_ptr() + at, src.data_ptr() + so, n))
        spans.append((at, so, n))
        at += n
    _native.realign_copy_batch(jobs, stream())
    got = dst.cpu().numpy()
    want = np.full(4_000_000, 0xA5, dtype=np.uint8)
    for at, so, n in spans:
        want[at : at + n] = src_host[so : so + n]
    assert np.array_equal(got, want)


def test_realign_rejects_bad_arguments(dev):
    a = torch.zeros(1024, dtype=torch.uint8, device=dev)
    with pytest.raises(_native.NativeError):
        _native.realign_copy(a.data_ptr() + 8, a.data_ptr(), 100)  # overlapping ranges
    descs = (_native.FstxCopyDesc * 49)()
    assert _native.lib().fstx_realign_copy_batch(descs, 49, None) == -10008  # FSTX_E_TOO_MANY


def test_realign_full_size_c2_section(dev):
    """Config C2's whole data section (709,646,336 bytes) shifted by 2 and by 10 bytes:
    checked by 64-bit word sums and sampled windows instead of a full host copy."""
    n = 709_646_336
    g = torch.Generator(device=dev).manual_seed(42)
    base = torch.randint(0, 256, (n + 4096,), dtype=torch.uint8, device=dev, generator=g)
    out = torch.empty(n, dtype=torch.uint8, device=dev)
    for m in (2, 10):
        out.zero_()
        _native.realign_copy(out.data_ptr(), base.data_ptr() + m, n, stream())
        want = base[m : m + n]
        assert torch.equal(out, want)


# ---- slice extract ----------------------------------------------------------------------------


def oracle_shard(raw: np.ndarray, dtype: str, shape, dim, rank, world):
    return orc.shard_bytes(raw, dtype, list(shape), dim, rank, world)


def gpu_shard(dev, raw: np.ndarray, itembits: int, shape, dim, rank, world, src_shift: int = 0):
    """Cut rank's block with fstx_slice_copy; returns the shard bytes as numpy."""
    block = -(-shape[dim] // world)
    lo, hi = min(rank * block, shape[dim]), min((rank + 1) * block, shape[dim])
    inner = int(np.prod(shape[dim + 1 :], dtype=np.int64)) * itembits // 8
    outer = int(np.prod(shape[:dim], dtype=np.int64))
    seg, pitch, first = (hi - lo) * inner, shape[dim] * inner, lo * inner
    host = np.full(raw.size + 64 + src_shift, 0x5A, dtype=np.uint8)
    host[src_shift : src_shift + raw.size] = raw
    src = torch.from_numpy(host).to(dev)
    dst = torch.full((outer * seg + 128,), 0xA5, dtype=torch.uint8, device=dev)
    _native.slice_copy(dst.data_ptr() + 64, src.data_ptr() + src_shift + first, outer, seg, pitch, stream())
    got = dst.cpu().numpy()
    assert (got[:64] == 0xA5).all() and (got[64 + outer * seg :] == 0xA5).all()
    return got[64 : 64 + outer * seg]


SHAPES = [
    ((64, 64), "BF16"), ((5, 3), "BF16"), ((7, 250), "BF16"), ((33, 1000), "F16"), ((3, 4, 5), "F32"),
    ((2, 3, 7), "U8"), ((128, 24), "F8_E4M3"), ((1, 9), "I64"), ((6,), "F32"), ((16, 8), "F16"),
    ((40, 1280), "BF16"), ((9, 6, 10), "BF16"),
]


@pytest.mark.parametrize("shape,dtype", SHAPES)
def test_slice_matches_oracle(dev, shape, dtype):
    bits = orc.DTYPE_BITS[dtype]
    raw = rand_bytes(int(np.prod(shape)) * bits // 8, hash(shape) % 1000)
    for dim in range(len(shape)):
        for world in (1, 2, 3, 4, 8):
            for rank in range(world):
                want, _ = oracle_shard(raw, dtype, shape, dim, rank, world)
                for shift in (0, 16) if world != 4 else (0, 1, 2, 4, 8):
                    got = gpu_shard(dev, raw, bits, shape, dim, rank, world, shift)
                    assert np.array_equal(got, want), (shape, dtype, dim, world, rank, shift)


def test_slice_batch_and_round_trip_full_size_c4(dev):
    """Config C4 shapes at full size (Llama-2-13B, TP=4): the four ranks' shards,
    cut in turn, concatenate back to the tensor (round trip), for dim 0 and dim 1."""
    for shape, dim in [((5120, 5120), 0), ((5120, 5120), 1), ((13824, 5120), 0), ((5120, 13824), 1), ((32000, 5120), 0)]:
        g = torch.Generator(device=dev).manual_seed(shape[0] + dim)
        t = torch.randint(-32768, 32767, shape, dtype=torch.int16, device=dev, generator=g).view(torch.bfloat16)
        world = 4
        block = -(-shape[dim] // world)
        inner = int(np.prod(shape[dim + 1 :], dtype=np.int64)) * 2
        outer = int(np.prod(shape[:dim], dtype=np.int64))
        parts, jobs = [], []
        for rank in range(world):
            out_shape = list(shape)
            out_shape[dim] = block
            p = torch.empty(out_shape, dtype=torch.bfloat16, device=dev)
            parts.append(p)
            jobs.append((p.data_ptr(), t.data_ptr() + rank * block * inner, outer, block * inner, shape[dim] * inner))
        _native.slice_copy_batch(jobs, stream())
        assert torch.equal(torch.cat(parts, dim=dim).view(torch.int16), t.view(torch.int16))
        for rank in range(world):  # and each shard equals torch's own slice
            sl = (slice(None),) * dim + (slice(rank * block, (rank + 1) * block),)
            assert torch.equal(parts[rank].view(torch.int16), t[sl].contiguous().view(torch.int16))


def test_slice_odd_shapes(dev):
    """Segments that are not multiples of 16 bytes (odd column counts, 1-byte dtypes,
    shifted sources, destinations at odd addresses): the gather kernel, against torch's own
    slicing on the GPU, and against the small-unit kernels (FSTX_GATHER_MODE=0) and the
    gather kernel forced onto every shape (FSTX_GATHER_MODE=2)."""
    import os

    rng = np.random.default_rng(11)
    cases = [((4096, 1000), torch.int16, 1, 4), ((3000, 999), torch.uint8, 1, 3), ((257, 4094), torch.uint8, 1, 2),
             ((129, 2047), torch.uint8, 1, 1), ((64, 65, 33), torch.int16, 1, 5), ((1000, 250), torch.int32, 1, 2),
             ((31, 8190), torch.int16, 1, 2), ((5, 100_003), torch.uint8, 1, 4), ((2000, 130), torch.uint8, 1, 2)]
    for shape, dtype, dim, world in cases:
        item = torch.empty((), dtype=dtype).element_size()
        hi = 127 if dtype == torch.uint8 else 30000
        for shift in (0, item, 3 * item):
            base = torch.randint(0, hi, (int(np.prod(shape)) + 64,), dtype=dtype, device=dev)
            t = base[shift // item : shift // item + int(np.prod(shape))].view(shape)
            for rank in range(world):
                block = -(-shape[dim] // world)
                lo, hi_ = min(rank * block, shape[dim]), min((rank + 1) * block, shape[dim])
                want = t[(slice(None),) * dim + (slice(lo, hi_),)].contiguous()
                inner = int(np.prod(shape[dim + 1 :], dtype=np.int64)) * item
                outer = int(np.prod(shape[:dim], dtype=np.int64))
                outs = []
                for mode in ("1", "0", "2"):
                    os.environ["FSTX_GATHER_MODE"] = mode
                    for lead in (0, 1, 5):  # the destination's first element: aligned, and off by 1 and 5 elements
                        got = torch.full((want.numel() + 32,), 77, dtype=dtype, device=dev)
                        _native.slice_copy(got.data_ptr() + lead * item, t.data_ptr() + lo * inner, outer,
                                           (hi_ - lo) * inner, shape[dim] * inner, stream())
                        outs.append((got, lead))
                os.environ.pop("FSTX_GATHER_MODE")
                for got, lead in outs:
                    assert torch.equal(got[lead : lead + want.numel()].view(want.shape), want), (shape, dtype, rank, shift, lead)
                    assert (got[:lead] == 77).all() and (got[lead + want.numel() :] == 77).all(), "wrote outside the shard"


def test_segments_under_16_bytes(dev):
    """Cuts whose segments are shorter than a vector go to the unit kernel: into an aligned dense
    destination it packs 16 / unit of them into one store, else it moves one unit per lane.
    Unit sizes 1, 2, 4 and 8 bytes, row counts that leave a ragged last vector, against torch's
    slicing, with guard elements around every destination."""
    for shape, dtype, world in [((100_003, 4), torch.int16, 4), ((65_537, 3), torch.uint8, 3), ((9_999, 6), torch.int16, 2),
                                ((33_333, 2), torch.int64, 2), ((7, 12), torch.uint8, 4), ((50_001, 2, 3), torch.int32, 2),
                                ((1, 8), torch.int16, 4), ((12_345, 15), torch.uint8, 1),
                                # rows close together: staged through LDS (up to the row pitch where the rows of one
                                # tile no longer fit), rows far apart: one unit per load; segment lengths that do and
                                # do not divide a tile; the last tile ragged
                                ((70_001, 8), torch.int16, 8), ((20_011, 24), torch.uint8, 2), ((3_001, 60), torch.uint8, 4),
                                ((5_003, 1000), torch.uint8, 100), ((4_099, 14), torch.int16, 2), ((1_000_003, 4), torch.uint8, 2),
                                ((2, 4), torch.int16, 4), ((600, 5), torch.int32, 5), ((513, 16), torch.int16, 4)]:
        t = torch.randint(0, 120, shape, dtype=dtype, device=dev)
        item = t.element_size()
        block = -(-shape[1] // world)
        inner = int(np.prod(shape[2:], dtype=np.int64)) * item
        for rank in range(world):
            lo, hi = min(rank * block, shape[1]), min((rank + 1) * block, shape[1])
            want = t[:, lo:hi].contiguous()
            for lead in (0, 1, 8 // item if item < 8 else 1):
                got = torch.full((want.numel() + 64,), 99, dtype=dtype, device=dev)
                _native.slice_copy(got.data_ptr() + lead * item, t.data_ptr() + lo * inner, shape[0], (hi - lo) * inner,
                                   shape[1] * inner, stream())
                assert torch.equal(got[lead : lead + want.numel()].view(want.shape), want), (shape, dtype, rank, lead)
                assert (got[:lead] == 99).all() and (got[lead + want.numel() :] == 99).all(), "wrote outside the shard"


def test_gather_random_geometry_in_one_batch(dev):
    """Byte-level sweep of the gather kernel: segment lengths from the shortest it takes (16
    bytes; 9 and 15 go to the small-unit kernel) over the tile size and its fractions, odd
    pitches, every source and destination alignment, jobs of very different segment lengths
    sharing one launch."""
    rng = np.random.default_rng(23)
    segs = [9, 15, 16, 17, 31, 33, 64, 65, 79, 81, 127, 129, 255, 511, 513, 1023, 1025, 2046, 2047, 2049, 2050, 4094, 4095,
            4097, 6001, 8191]
    for _ in range(6):
        jobs, checks = [], []
        for _j in range(24):
            seg = int(rng.choice(segs))
            pitch = seg + int(rng.choice([1, 2, 3, 7, 13, 16, 17, 100, 1001]))
            outer = int(rng.integers(2, 40)) if seg < 3000 else int(rng.integers(2, 6))
            shift = int(rng.integers(0, 16))
            lead = int(rng.integers(0, 16))
            # the source tensor ends with its last segment: a load that strayed past it would leave the allocation's payload
            src = torch.randint(0, 255, (shift + (outer - 1) * pitch + seg,), dtype=torch.uint8, device=dev)
            dst = torch.full((lead + outer * seg + 48,), 201, dtype=torch.uint8, device=dev)
            jobs.append((dst.data_ptr() + lead, src.data_ptr() + shift, outer, seg, pitch))
            checks.append((src, dst, shift, lead, outer, seg, pitch))
        _native.slice_copy_batch(jobs, stream())
        for src, dst, shift, lead, outer, seg, pitch in checks:
            want = torch.stack([src[shift + r * pitch : shift + r * pitch + seg] for r in range(outer)]).reshape(-1)
            assert torch.equal(dst[lead : lead + outer * seg], want), (seg, pitch, outer, shift, lead)
            assert (dst[:lead] == 201).all() and (dst[lead + outer * seg :] == 201).all(), "wrote outside the block"


def test_slice2d_strided_destination(dev):
    """Blocks of several tensors cut straight into one joined tensor along an inner
    dimension: random geometry (every unit size from 1 to 16 bytes), against torch.cat
    of torch's own slices; bytes between the blocks' columns stay untouched."""
    rng = np.random.default_rng(5)
    for trial in range(12):
        item = int(rng.choice([1, 2, 4]))
        dtype = {1: torch.uint8, 2: torch.int16, 4: torch.int32}[item]
        rows = int(rng.integers(1, 300))
        n_src = int(rng.integers(1, 30))  # more than 24 jobs: two launches
        world = int(rng.integers(1, 5))
        rank = int(rng.integers(0, world))
        srcs = [torch.randint(0, 120, (rows, int(rng.integers(1, 200)) * int(rng.choice([1, 1, 4, 8]))), dtype=dtype, device=dev)
                for _ in range(n_src)]
        parts = []
        for t in srcs:
            block = -(-t.shape[1] // world)
            parts.append(t[:, rank * block : (rank + 1) * block])
        want = torch.cat(parts, dim=1)
        out = torch.full((rows, want.shape[1] + 3), 77, dtype=dtype, device=dev)  # 3 guard columns per row
        jobs, at = [], out.data_ptr()
        for t, p in zip(srcs, parts):
            block = -(-t.shape[1] // world)
            jobs.append((at, t.data_ptr() + min(rank * block, t.shape[1]) * item, rows, p.shape[1] * item,
                         t.shape[1] * item, out.shape[1] * item))
            at += p.shape[1] * item
        _native.slice_copy2d_batch(jobs, stream())
        assert torch.equal(out[:, : want.shape[1]], want), trial
        assert (out[:, want.shape[1] :] == 77).all(), "wrote outside the blocks"
    # argument checks
    a = torch.zeros(4096, dtype=torch.uint8, device=dev)
    lib = _native.lib()
    bad = (_native.FstxSlice2dDesc * 1)(_native.FstxSlice2dDesc(a.data_ptr(), a.data_ptr() + 2048, 4, 64, 128, 32))
    assert lib.fstx_slice_copy2d_batch(bad, 1, None) == -10001  # dst_pitch < seg_bytes


def test_join_copy_matches_cat(dev):
    """fstx_join_copy: the blocks of up to 60 tensors side by side in one joined tensor,
    against torch.cat of torch's own slices; every unit size, short and long segments,
    a padded destination, guard bytes."""
    rng = np.random.default_rng(9)
    for trial in range(14):
        item = int(rng.choice([1, 2, 4]))
        dtype = {1: torch.uint8, 2: torch.int16, 4: torch.int32}[item]
        rows = int(rng.integers(1, 400))
        n_src = int(rng.choice([1, 2, 3, 7, 24, 25, 60]))
        world = int(rng.integers(1, 5))
        rank = int(rng.integers(0, world))
        srcs = [torch.randint(0, 120, (rows, int(rng.integers(1, 300)) * int(rng.choice([1, 1, 4, 8, 64]))), dtype=dtype, device=dev)
                for _ in range(n_src)]
        parts = []
        for t in srcs:
            block = -(-t.shape[1] // world)
            parts.append(t[:, min(rank * block, t.shape[1]) : (rank + 1) * block])
        want = torch.cat(parts, dim=1)
        pad = int(rng.choice([0, 3, 16]))
        out = torch.full((rows, want.shape[1] + pad), 77, dtype=dtype, device=dev)
        jobs = [(t.data_ptr() + (p.storage_offset() - t.storage_offset()) * item, p.shape[1] * item, t.shape[1] * item)
                for t, p in zip(srcs, parts)]
        _native.join_copy(out.data_ptr(), rows, jobs, stream(), dst_pitch=out.shape[1] * item)
        assert torch.equal(out[:, : want.shape[1]], want), trial
        assert (out[:, want.shape[1] :] == 77).all(), "wrote outside the joined columns"
    lib = _native.lib()
    a = torch.zeros(4096, dtype=torch.uint8, device=dev)
    one = (_native.FstxJoinSrc * 1)(_native.FstxJoinSrc(a.data_ptr() + 2048, 64, 32))
    assert lib.fstx_join_copy(a.data_ptr(), 0, 4, one, 1, None) == -10001  # pitch shorter than the segment
    one = (_native.FstxJoinSrc * 1)(_native.FstxJoinSrc(a.data_ptr() + 2048, 64, 64))
    assert lib.fstx_join_copy(a.data_ptr(), 32, 4, one, 1, None) == -10001  # destination rows would overlap
    many = (_native.FstxJoinSrc * 25)()
    assert lib.fstx_join_copy(a.data_ptr(), 0, 4, many, 25, None) == -10008


def test_tensors_beyond_4_gib(dev):
    """One tensor of 5.4 GB: byte offsets and unit indices past 2^32 in the realign copy
    (shifted source), a column cut, a row cut and a conversion."""
    rows, cols = 40960, 65536 + 8
    t = torch.randint(-30000, 30000, (rows, cols), dtype=torch.int16, device=dev)
    nbytes = t.numel() * 2
    assert nbytes > 5 * (1 << 30)
    flat = t.view(-1).view(torch.uint8)
    out = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    _native.realign_copy(out.data_ptr(), flat.data_ptr() + 6, nbytes - 6, stream())
    assert torch.equal(out[: nbytes - 6], flat[6:])
    assert torch.equal(out[nbytes - 4096 - 6 : nbytes - 6], flat[nbytes - 4096 :])
    del out
    half = cols // 2
    cut = torch.empty((rows, half), dtype=torch.int16, device=dev)
    _native.slice_copy(cut.data_ptr(), t.data_ptr() + half * 2, rows, half * 2, cols * 2, stream())
    assert torch.equal(cut, t[:, half:])
    del cut
    block = rows // 2
    rowcut = torch.empty((block, cols), dtype=torch.int16, device=dev)
    _native.slice_copy(rowcut.data_ptr(), t.data_ptr() + block * cols * 2, 1, block * cols * 2, rows * cols * 2, stream())
    assert torch.equal(rowcut, t[block:])
    del rowcut, t
    # an odd column count: the gather kernel with more than 4 GiB per tensor (cut into jobs of 32-bit positions)
    rows, cols = 80000, 65537
    t = torch.randint(-30000, 30000, (rows, cols), dtype=torch.int16, device=dev)
    block = -(-cols // 2)
    for rank in (0, 1):
        width = min(block, cols - rank * block)
        cut = torch.empty((rows, width), dtype=torch.int16, device=dev)
        assert cut.numel() * 2 > (1 << 32)
        _native.slice_copy(cut.data_ptr(), t.data_ptr() + rank * block * 2, rows, width * 2, cols * 2, stream())
        assert torch.equal(cut, t[:, rank * block : rank * block + width]), rank
        del cut
    del t
    # one-byte units (odd pitch): more than 2^32 units, so the direct kernels split the tensor
    # into several jobs by rows
    import os

    rows, cols = 80000, 65537
    t = torch.randint(0, 255, (rows, cols), dtype=torch.uint8, device=dev)
    cut = torch.empty((rows, cols - 1), dtype=torch.uint8, device=dev)
    os.environ["FSTX_GATHER_MODE"] = "0"
    try:
        _native.slice_copy(cut.data_ptr(), t.data_ptr(), rows, cols - 1, cols, stream())
    finally:
        os.environ.pop("FSTX_GATHER_MODE")
    assert torch.equal(cut, t[:, :-1])
    cut.zero_()
    wide = torch.zeros((rows, cols + 2), dtype=torch.uint8, device=dev)
    _native.slice_copy2d_batch([(wide.data_ptr() + 1, t.data_ptr(), rows, cols - 1, cols, cols + 2)], stream())
    assert torch.equal(wide[:, 1:cols], t[:, :-1]) and not wide[:, 0].any() and not wide[:, cols:].any()
    del t, cut, wide
    # a span of 56 GiB: more than one job, and more than one launch, may cover
    n = (56 << 30) + 12345
    big = torch.empty(n + 64, dtype=torch.uint8, device=dev)
    for at in range(0, n + 64, 1 << 32):
        big[at : at + (1 << 32)].random_(0, 255)
    out = torch.empty(n, dtype=torch.uint8, device=dev)
    _native.realign_copy(out.data_ptr(), big.data_ptr() + 3, n, stream())
    assert torch.equal(out, big[3 : 3 + n])
    _native.realign_copy_batch([(out.data_ptr(), big.data_ptr() + 16, n), (big.data_ptr() + n + 32, big.data_ptr(), 32)], stream())
    assert torch.equal(out, big[16 : 16 + n]) and torch.equal(big[n + 32 : n + 64], big[:32])
    del big, out
    f = torch.randn(1_200_000_000, dtype=torch.float32, device=dev)  # 4.8 GB in, 2.4 GB out
    o = torch.empty(f.numel(), dtype=torch.bfloat16, device=dev)
    _native.convert_batch([(o.data_ptr(), f.data_ptr(), f.numel(), _native.ELEM_TYPES["F32"], _native.ELEM_TYPES["BF16"])], stream())
    assert torch.equal(o.view(torch.int16), f.to(torch.bfloat16).view(torch.int16))


def test_cutting_into_jobs_and_launches(dev, monkeypatch):
    """With the launch limits shrunk to a few thousand workgroups the same random sweeps go
    through the code that cuts spans, tensors and joins into several jobs and launches."""
    monkeypatch.setenv("FSTX_MAX_BLOCKS_PER_LAUNCH", "4096")
    test_realign_batch_many_jobs(dev)
    test_slice_odd_shapes(dev)
    test_gather_random_geometry_in_one_batch(dev)
    test_slice2d_strided_destination(dev)
    test_join_copy_matches_cat(dev)
    # one span, one strided tensor, one join and one conversion that are each many launches long
    n = 40_000_003
    src = torch.randint(0, 255, (n + 16,), dtype=torch.uint8, device=dev)
    out = torch.zeros(n + 16, dtype=torch.uint8, device=dev)
    _native.realign_copy(out.data_ptr(), src.data_ptr() + 5, n, stream())
    assert torch.equal(out[:n], src[5 : 5 + n]) and not out[n:].any()
    t = src[: 6000 * 6000].view(6000, 6000)
    cut = torch.empty((6000, 3000), dtype=torch.uint8, device=dev)
    _native.slice_copy(cut.data_ptr(), t.data_ptr() + 3000, 6000, 3000, 6000, stream())
    assert torch.equal(cut, t[:, 3000:])
    joined = torch.empty((6000, 4500), dtype=torch.uint8, device=dev)
    _native.join_copy(joined.data_ptr(), 6000, [(t.data_ptr(), 3000, 6000), (t.data_ptr() + 4000, 1500, 6000)], stream())
    assert torch.equal(joined, torch.cat([t[:, :3000], t[:, 4000:5500]], dim=1))
    f = torch.randn(9_000_001, dtype=torch.float32, device=dev)
    o = torch.zeros(f.numel() + 8, dtype=torch.bfloat16, device=dev)
    _native.convert_batch([(o.data_ptr(), f.data_ptr(), f.numel(), _native.ELEM_TYPES["F32"], _native.ELEM_TYPES["BF16"])], stream())
    assert torch.equal(o[: f.numel()].view(torch.int16), f.to(torch.bfloat16).view(torch.int16)) and not o[f.numel() :].view(torch.int16).any()


def test_entry_points_can_be_captured_in_a_graph(dev):
    """The kernel entry points only enqueue work (no allocation, no synchronisation, tables
    passed by value), so a caller may record them into a HIP graph: three replays, each after
    the sources were changed by eager work, each compared with an eager run."""
    rows, cols = 512, 4096
    a = torch.randint(-3000, 3000, (rows, cols), dtype=torch.int16, device=dev)
    b = torch.randint(-3000, 3000, (rows, cols + 6), dtype=torch.int16, device=dev)  # odd pitch: gather kernel
    f = torch.randn(rows * cols, dtype=torch.float32, device=dev)
    cut_a = torch.empty((rows, cols // 4), dtype=torch.int16, device=dev)
    cut_b = torch.empty((rows, 1001), dtype=torch.int16, device=dev)
    moved = torch.empty(rows * cols * 2 - 6, dtype=torch.uint8, device=dev)
    joined = torch.empty((rows, cols // 4 + 1001), dtype=torch.int16, device=dev)
    half = torch.empty(rows * cols, dtype=torch.bfloat16, device=dev)

    def enqueue(st):
        _native.slice_copy_batch([(cut_a.data_ptr(), a.data_ptr() + cols // 4 * 2, rows, cols // 4 * 2, cols * 2),
                                  (cut_b.data_ptr(), b.data_ptr() + 6, rows, 1001 * 2, (cols + 6) * 2)], st)
        _native.realign_copy(moved.data_ptr(), a.data_ptr() + 6, moved.numel(), st)
        _native.join_copy(joined.data_ptr(), rows, [(a.data_ptr() + cols // 4 * 2, cols // 4 * 2, cols * 2),
                                                    (b.data_ptr() + 6, 1001 * 2, (cols + 6) * 2)], st)
        _native.convert_batch([(half.data_ptr(), f.data_ptr(), f.numel(), _native.ELEM_TYPES["F32"], _native.ELEM_TYPES["BF16"])], st)

    def check():
        assert torch.equal(cut_a, a[:, cols // 4 : cols // 2])
        assert torch.equal(cut_b, b[:, 3 : 3 + 1001])
        assert torch.equal(moved, a.view(-1).view(torch.uint8)[6:])
        assert torch.equal(joined, torch.cat([a[:, cols // 4 : cols // 2], b[:, 3 : 3 + 1001]], dim=1))
        assert torch.equal(half.view(torch.int16), f.to(torch.bfloat16).view(torch.int16))

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        enqueue(side.cuda_stream)  # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    check()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        enqueue(torch.cuda.current_stream().cuda_stream)
    for replay in range(3):
        a.add_(replay + 1)  # eager work between the replays
        b.mul_(-1)
        f.mul_(1.5)
        for t in (cut_a, cut_b, moved, joined):
            t.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        check()


def test_slice_zero_sized_and_errors(dev):
    a = torch.zeros(4096, dtype=torch.uint8, device=dev)
    _native.slice_copy(a.data_ptr(), a.data_ptr() + 2048, 0, 16, 32, stream())  # nothing to do
    _native.slice_copy(a.data_ptr(), a.data_ptr() + 2048, 4, 0, 32, stream())
    with pytest.raises(_native.NativeError):
        _native.slice_copy(a.data_ptr(), a.data_ptr() + 2048, 4, 64, 32, stream())  # pitch < segment
    torch.cuda.synchronize()


def test_joins_of_random_geometry_small_and_large(dev):
    """fstx_join_copy on random jobs against torch's own strided copies, whole destination compared
    (payload and every byte around it): 1 to 24 sources, segments from 16 bytes to 9 KB, equal and
    unequal, any alignment of sources and destination, dense and pitched destinations with gaps from
    one byte to more than the payload, a few rows up to several hundred thousand -- jobs of a few
    tiles and jobs of many chunks of tiles, common tiles and the tiles at the ends of blocks."""
    rng = np.random.default_rng(31)
    lib = _native.lib()
    for trial in range(60):
        n = int(rng.choice([1, 1, 2, 3, 5, 7, 14, 24]))
        hi = int(rng.choice([300, 3000, 9000]))
        segs = [int(rng.integers(16, hi)) for _ in range(n)]
        if rng.random() < 0.4:
            segs = [segs[0]] * n
        if rng.random() < 0.3:
            segs = [s // 16 * 16 + 16 for s in segs]
        budget = 150e6 if trial % 10 == 0 else 8e6
        rows = int(rng.integers(1, max(2, int(budget // sum(segs)))))
        rows = min(rows, int(rng.choice([3, 50, 700, 6000, 40000, 300000])))
        pitches = [s + int(rng.choice([0, 1, 2, 16, 100, 3 * s])) for s in segs]
        shifts = [int(rng.integers(0, 16)) for _ in range(n)]
        lead = int(rng.integers(0, 16))
        gap = int(rng.choice([0, 0, 0, 1, 15, 16, 40, 5000]))
        row_bytes = sum(segs)
        dst_pitch = row_bytes + gap
        srcs = [torch.randint(0, 255, (sh + (rows - 1) * p + s,), dtype=torch.uint8, device=dev)
                for s, p, sh in zip(segs, pitches, shifts)]
        dst = torch.full((lead + (rows - 1) * dst_pitch + row_bytes + 64,), 203, dtype=torch.uint8, device=dev)
        parts = (_native.FstxJoinSrc * n)(*[_native.FstxJoinSrc(t.data_ptr() + sh, s, p)
                                            for t, sh, s, p in zip(srcs, shifts, segs, pitches)])
        case = (trial, segs[:4], rows, pitches[:4], gap, lead, shifts[:4])
        assert lib.fstx_join_copy(dst.data_ptr() + lead, dst_pitch if gap else 0, rows, parts, n, None) == 0, case
        want = torch.full_like(dst, 203)
        col = 0
        for t, sh, s, p in zip(srcs, shifts, segs, pitches):
            torch.as_strided(want, (rows, s), (dst_pitch, 1), lead + col).copy_(torch.as_strided(t, (rows, s), (p, 1), sh))
            col += s
        torch.cuda.synchronize()
        assert torch.equal(dst, want), case


_PARTITION_CHECK = r"""
import sys, torch
from fastsafetensors_amd import _native
dev = torch.device("cuda:0")
st = torch.cuda.current_stream().cuda_stream
g = torch.Generator(device=dev).manual_seed(5)
# realign copy, shifted source, a few thousand tiles
src = torch.randint(0, 255, (5_000_011,), dtype=torch.uint8, device=dev, generator=g)
dst = torch.zeros(5_000_000, dtype=torch.uint8, device=dev)
_native.realign_copy(dst.data_ptr(), src.data_ptr() + 7, dst.numel(), st)
assert torch.equal(dst, src[7 : 7 + dst.numel()])
# aligned column cut (slice kernel), odd column cut (gather kernel), short segments, a narrow block in wide rows, a join
t = torch.randint(-30000, 30000, (3000, 4096), dtype=torch.int16, device=dev, generator=g)
for lo, hi in ((1024, 2048), (1001, 2024), (40, 167)):
    out = torch.empty((3000, hi - lo), dtype=torch.int16, device=dev)
    _native.slice_copy(out.data_ptr(), t.data_ptr() + 2 * lo, 3000, 2 * (hi - lo), 8192, st)
    assert torch.equal(out, t[:, lo:hi]), (lo, hi)
wide = torch.zeros((3000, 1500), dtype=torch.int16, device=dev)
_native.slice_copy2d_batch([(wide.data_ptr() + 2 * 33, t.data_ptr() + 2 * 5, 3000, 2 * 47, 8192, 3000)], st)
assert torch.equal(wide[:, 33:80], t[:, 5:52]) and not wide[:, :33].any() and not wide[:, 80:].any()
parts = [torch.randint(0, 255, (2000, 1016), dtype=torch.uint8, device=dev, generator=g) for _ in range(5)]
joined = torch.empty((2000, 5 * 254), dtype=torch.uint8, device=dev)
_native.join_copy(joined.data_ptr(), 2000, [(p.data_ptr() + 254, 254, 1016) for p in parts], st)
assert torch.equal(joined, torch.cat([p[:, 254:508] for p in parts], dim=1))
# down-cast
f = torch.randn(1_000_003, device=dev, generator=g)
h = torch.empty(f.numel(), dtype=torch.bfloat16, device=dev)
_native.convert_batch([(h.data_ptr(), f.data_ptr(), f.numel(), _native.ELEM_TYPES["F32"], _native.ELEM_TYPES["BF16"])], st)
assert torch.equal(h.view(torch.int16), f.to(torch.bfloat16).view(torch.int16))
torch.cuda.synchronize()
print("ok")
"""


@pytest.mark.parametrize("dies", ["1", "2", "4"])
def test_kernels_on_a_device_with_fewer_dies(dies):
    """The tile order follows the number of dies of the device (compute units / 32; a partition of
    the chip has 4, 2 or 1).  FSTX_DIES stands in for such a device: the same bytes must come out.
    The library reads it once per process, hence a process of its own."""
    import os
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, FSTX_DIES=dies, PYTHONPATH=root + os.pathsep + os.environ.get("PYTHONPATH", ""))
    proc = subprocess.run([sys.executable, "-c", _PARTITION_CHECK], env=env, capture_output=True, text=True, timeout=110)
    assert proc.returncode == 0 and proc.stdout.strip().endswith("ok"), proc.stdout + proc.stderr
