# SPDX-License-Identifier: Apache-2.0
"""Pins the CPU oracle (oracle/) before anything is compared with it.

Nothing here retypes the oracle's own formulas: expectations come from the
reference's committed fixtures and closed-form generators, from the independent
``safetensors`` library plus torch slicing (the oracle of the reference's own
tests), from Python list slicing, from brute-force element loops, and from the
reference's C++ reader compiled into oracle/_ref where that build exists.
"""
import itertools
import os

import numpy as np
import pytest
import torch
from safetensors.torch import load_file, save_file

from conftest import GOLDEN_FILES
from oracle import st_oracle as orc


def as_bytes(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().reshape(-1).view(torch.uint8).numpy()


# ---- header parse ---------------------------------------------------------------


def test_reference_fixture_a_known_answers(golden):
    # facts of the reference's examples/a.safetensors (generator examples/gen.py:5-14)
    h = orc.parse_file(golden("a.safetensors"))
    assert h.header_length == 104 and h.size_bytes == 360 and not h.aligned
    assert h.metadata == {"fst": "sample"}
    assert list(h.tensors) == ["a0"]
    assert h.tensors["a0"] == {"dtype": "F16", "shape": [16, 8], "data_offsets": [0, 256]}
    rows = orc.tensor_bytes(golden("a.safetensors"), h, "a0").view(np.float16).reshape(16, 8)
    assert np.array_equal(rows, np.repeat(np.arange(16, dtype=np.float16)[:, None], 8, axis=1))
    assert rows.view(np.uint16)[15, 0] == 0x4B80  # float16(15.0)


def test_tiny_gpt2_closed_form(golden):
    path = golden("tiny_gpt2.safetensors")
    h = orc.parse_file(path)
    assert len(h.tensors) == 48 and h.metadata == {"fst": "tiny-gpt2"}
    for layer in range(12):
        for name, (r, c), off in [("mlp.c_proj.weight", (8, 16), 0), ("mlp.c_fc.weight", (16, 8), 100),
                                  ("attn.c_proj.weight", (8, 8), 200)]:
            got = orc.tensor_bytes(path, h, f"h.{layer}.{name}").view(np.float16).reshape(r, c)
            # fp16 arithmetic as in the recipe: fp16(arange) + fp16(offset), rounded to fp16
            want = np.arange(r * c).astype(np.float16).reshape(r, c) + np.float16(layer * 1000 + off)
            assert np.array_equal(got, want)
        bias = orc.tensor_bytes(path, h, f"h.{layer}.attn.c_proj.bias").view(np.float16)
        assert np.array_equal(bias, np.arange(8).astype(np.float16) + np.float16(layer * 1000 + 300))


@pytest.mark.parametrize("name", GOLDEN_FILES)
def test_tensor_bytes_match_safetensors_library(golden, name):
    path = golden(name)
    h = orc.parse_file(path)
    ref = load_file(path)
    assert set(ref) == set(h.tensors)
    for key, t in ref.items():
        assert np.array_equal(orc.tensor_bytes(path, h, key), as_bytes(t)), key
    # offsets ascend and tile the data section
    ends = [v["data_offsets"] for v in h.tensors.values()]
    assert ends[0][0] == 0 and all(a[1] == b[0] for a, b in zip(ends, ends[1:]))


def test_misaligned_header_fixture_is_misaligned(golden):
    h = orc.parse_file(golden("misaligned_header.safetensors"))
    assert h.header_length % 8 == 2 and h.header_length % 16 in (2, 10) and not h.aligned


def _blob(json_text: str, data: bytes = b"") -> bytes:
    j = json_text.encode()
    return len(j).to_bytes(8, "little") + j + data


def test_header_error_cases():
    with pytest.raises(Exception, match="HeaderTooSmall"):
        orc.parse_header(b"\0\0\0\0")
    with pytest.raises(Exception, match="HeaderTooLarge"):
        orc.parse_header((100_000_001).to_bytes(8, "little") + b"{}", 1024)
    with pytest.raises(Exception, match="InvalidHeaderLength"):
        orc.parse_header((100).to_bytes(8, "little") + b"{}" * 21, 50)
    one = '{"a":{"dtype":"F32","shape":[2],"data_offsets":[%d,%d]}}'
    assert orc.parse_header(_blob(one % (0, 8), b"x" * 8)).tensors["a"]["shape"] == [2]
    assert orc.parse_header(_blob(one % (0, 8), b"x" * 12)).size_bytes > 0  # trailing bytes are fine
    with pytest.raises(Exception, match="InvalidOffset"):
        orc.parse_header(_blob(one % (4, 12), b"x" * 12))  # gap before the first tensor
    with pytest.raises(Exception, match="TensorInvalidInfo"):
        orc.parse_header(_blob(one % (0, 12), b"x" * 12))  # 12 bytes for 2 x F32
    with pytest.raises(Exception, match="MetadataIncompleteBuffer"):
        orc.parse_header(_blob(one % (0, 8), b"x" * 7))  # file ends inside the tensor
    # only __metadata__: accepted (reference test_from_buffer_success)
    assert orc.parse_header(_blob('{"__metadata__": {"data_offsets": [0, 123]}}')).tensors == {}
    # scalars: shape [] holds one element
    assert orc.parse_header(_blob('{"s":{"dtype":"F32","shape":[],"data_offsets":[0,4]}}', b"abcd")).tensors["s"]["shape"] == []
    # F4 packs two values per byte
    assert orc.parse_header(_blob('{"q":{"dtype":"F4","shape":[8,16],"data_offsets":[0,64]}}', b"q" * 64))


# ---- frame algebra -----------------------------------------------------------------


def test_frame_getitem_matches_list_slicing():
    n, m = 5, 6
    ref = list(range(n))
    for i in range(-n, n):
        shape, strides, offsets = orc.frame_getitem([n, m], i)
        assert shape == [1, m] and offsets[0] == ref[i]
    for i in (n, -n - 1):
        with pytest.raises(IndexError):
            orc.frame_getitem([n, m], i)
    bounds = [None, -n - 2, -n, -2, -1, 0, 1, n - 2, n - 1, n, n + 2]
    for start, stop, step in itertools.product(bounds, bounds, [None, 1, 2, 3, -1, -2]):
        got = orc.frame_getitem([n, m], slice(start, stop, step))
        want = ref[slice(start, stop, step)]
        if not want:
            assert got is None
            continue
        shape, strides, offsets = got
        assert shape[1] == m
        assert [offsets[0] + k * (strides[0] // m) for k in range(shape[0])] == want
    with pytest.raises(ValueError):
        orc.frame_getitem([n, m], slice(None, None, 0))
    assert orc.frame_getitem([n, m], ()) == ([n, m], [m, 1], [0, 0])
    # known answer of the reference's own test (test_fastsafetensors.py:845-849)
    assert orc.frame_getitem([n, m], (slice(1, -1), slice(None, None, 2))) == ([n - 2, m // 2], [m, 2], [1, 0])


# ---- shards ---------------------------------------------------------------------------


def torch_shard(t: torch.Tensor, dim: int, rank: int, world: int) -> torch.Tensor:
    """The oracle of the reference's distributed test (tests/unit/test_multi.py:44-64)."""
    block = (t.shape[dim] + world - 1) // world
    sl = (slice(None),) * dim + (slice(rank * block, (rank + 1) * block, 1),)
    return t[sl].clone()


@pytest.mark.parametrize("world", [1, 2, 3, 4, 7])
def test_shard_bytes_match_torch_slicing(golden, world):
    path = golden("tiny_gpt2.safetensors")
    h = orc.parse_file(path)
    ref = load_file(path)
    for key, t in ref.items():
        for dim in range(t.dim()):
            for rank in range(world):
                want = torch_shard(t, dim, rank, world)
                got, shape = orc.shard_bytes(orc.tensor_bytes(path, h, key), "F16", list(t.shape), dim, rank, world)
                assert shape == list(want.shape)
                assert np.array_equal(got, as_bytes(want)), (key, dim, rank)


def test_shard_bytes_brute_force_uneven_and_empty():
    rng = np.random.default_rng(7)
    for shape, dim, world in [((5, 3), 0, 4), ((5, 3), 1, 2), ((3, 4, 5), 1, 3), ((2, 3, 7), 2, 4),
                              ((1, 9), 1, 16), ((6,), 0, 4)]:
        elems = int(np.prod(shape))
        raw = rng.integers(0, 256, elems * 2, dtype=np.uint8)  # 2-byte elements
        block = -(-shape[dim] // world)
        for rank in range(world):
            lo, hi = min(rank * block, shape[dim]), min((rank + 1) * block, shape[dim])
            want = bytearray()
            for idx in itertools.product(*[range(s) for s in shape]):
                if lo <= idx[dim] < hi:
                    flat = int(np.ravel_multi_index(idx, shape))
                    want += bytes(raw[2 * flat : 2 * flat + 2])
            got, out_shape = orc.shard_bytes(raw, "BF16", list(shape), dim, rank, world)
            assert out_shape[dim] == hi - lo and bytes(got) == bytes(want)
            # the C restatement agrees
            outer = int(np.prod(shape[:dim], dtype=np.int64))
            inner = int(np.prod(shape[dim + 1 :], dtype=np.int64)) * 2
            if hi > lo:
                c = orc.slice_c(raw, outer, (hi - lo) * inner, shape[dim] * inner, lo * inner)
                assert bytes(c) == bytes(want)


def test_shard_bytes_f4_packed(golden):
    # [8, 16] fp4 values = [8, 8] bytes; cutting the last dim in 2 gives byte columns 0:4 / 4:8
    path = golden("f4.safetensors")
    h = orc.parse_file(path)
    assert h.tensors["a"]["shape"] == [8, 16]
    raw = orc.tensor_bytes(path, h, "a")
    assert np.array_equal(raw, np.arange(64, dtype=np.uint8))
    got, shape = orc.shard_bytes(raw, "F4", [8, 16], 1, 1, 2)
    assert shape == [8, 8] and np.array_equal(got, np.arange(64, dtype=np.uint8).reshape(8, 8)[:, 4:].reshape(-1))
    with pytest.raises(ValueError):
        orc.shard_bytes(raw, "F4", [8, 16], 1, 0, 16)  # blocks of one fp4 value split a byte


def test_push_outcome_truth_table():
    # reference test (tests/unit/test_multi.py:71-82): pushing to rank 1 yields a tensor on rank 1 only
    assert orc.push_outcome(1, 0, 0, 0) == "view"
    for world in (2, 4):
        for src, dst, me in itertools.product(range(world), repeat=3):
            out = orc.push_outcome(world, me, dst, src)
            assert (out != "none") == (me == dst)
            if me == dst:
                assert out == ("clone" if src == dst else "recv")


# ---- realign ----------------------------------------------------------------------------


def test_realign_and_memmove():
    rng = np.random.default_rng(3)
    for header_length in (104, 4096 + 2, 8192 + 10, 64):
        data = rng.integers(0, 256, 1000, dtype=np.uint8)
        start = header_length - header_length % 4096
        window = np.concatenate([rng.integers(0, 256, header_length - start, dtype=np.uint8), data])
        assert np.array_equal(orc.realign(window, header_length, start, 1000), data)
        buf = window.copy()
        tmp = np.zeros(1000, dtype=np.uint8)
        assert orc.clib().fst_oracle_memmove(buf.ctypes.data, buf.size, 0, header_length - start, tmp.ctypes.data, 1000, 1000) == 0
        assert np.array_equal(buf[:1000], data)
    assert orc.clib().fst_oracle_memmove(buf.ctypes.data, 10, 0, 12, tmp.ctypes.data, 1000, 4) == -1


# ---- the restated threaded reader ---------------------------------------------------------


@pytest.fixture(scope="module")
def big_file(tmp_path_factory):
    path = str(tmp_path_factory.mktemp("orc") / "big.safetensors")
    g = torch.Generator().manual_seed(11)
    tensors = {f"t{i}": torch.randn(257, 129 + i, generator=g) for i in range(9)}
    tensors["s"] = torch.tensor(3.5)
    save_file(tensors, path)
    return path


@pytest.mark.parametrize("bbuf_kb,threads,block", [(16 * 1024, 16, 16 * 1024**3), (64, 4, 100_000), (3, 2, 4097), (1, 1, 1 << 20)])
def test_nogds_reader_restatement(big_file, bbuf_kb, threads, block):
    h = orc.parse_file(big_file)
    r = orc.NogdsReader(bbuf_kb, threads)
    got = r.load_file(big_file, h, block)
    assert got.ctypes.data % 4096 == 0
    assert np.array_equal(got, orc.file_bytes(big_file, h.header_length, h.size_bytes))
    assert r.bounce_bytes() == -(-bbuf_kb // threads) * 1024 * threads
    r.close()


def test_nogds_reader_short_file_fails(big_file, tmp_path):
    h = orc.parse_file(big_file)
    cut = str(tmp_path / "cut.safetensors")
    with open(big_file, "rb") as f, open(cut, "wb") as g:
        g.write(f.read(h.size_bytes - 1000))
    r = orc.NogdsReader(64, 4)
    with pytest.raises(Exception, match="wait_nogds_read failed"):
        r.load_file(cut, h, 1 << 20)  # header still claims the full size
    r.close()


def test_nogds_reader_against_compiled_reference(big_file):
    """Same requests through the reference's own nogds_file_reader (cpp/ext.cpp:648-806)."""
    cpp = orc.load_reference_cpp()
    if cpp is None:
        pytest.skip("oracle/_ref is not built (the reference tree is absent)")
    h = orc.parse_file(big_file)
    total = h.size_bytes - h.header_length
    for bbuf_kb, threads, block in [(16 * 1024, 16, 16 * 1024**3), (64, 4, 100_000), (3, 2, 4097)]:
        base = cpp.cpu_malloc(total)
        gbuf = cpp.gds_device_buffer(base, total, False)
        reader = cpp.nogds_file_reader(False, bbuf_kb, threads, False, 0)
        fd = os.open(big_file, os.O_RDONLY)
        reqs, count = [], 0
        while count < total:
            l = min(block, total - count)
            req = reader.submit_read(fd, gbuf, h.header_length + count, l, count)
            assert req > 0
            reqs.append(req)
            count += l
        for req in reqs:
            assert reader.wait_read(req) > 0
        os.close(fd)
        assert cpp.get_cpp_metrics().bounce_buffer_bytes == -(-bbuf_kb // threads) * 1024 * threads
        theirs = np.frombuffer(cpp.read_buffer(base, total), dtype=np.uint8)
        mine = orc.NogdsReader(bbuf_kb, threads)
        assert np.array_equal(mine.load_file(big_file, h, block), theirs)
        assert mine.bounce_bytes() == cpp.get_cpp_metrics().bounce_buffer_bytes
        mine.close()
        del reader
        cpp.cpu_free(base)
        assert cpp.get_cpp_metrics().bounce_buffer_bytes == 0
    assert cpp.get_alignment_size() == 4096
