# SPDX-License-Identifier: Apache-2.0
"""Header model, frame algebra and device/dtype vocabulary of the package (CPU).

Expectations are the reference's fixtures, the error substrings its own tests
match (tests/unit/test_fastsafetensors.py:106-206), Python list slicing, the
independent safetensors library -- and agreement with the oracle's parse."""
import itertools
import os

import pytest
import torch
from safetensors.torch import load_file

from conftest import GOLDEN_FILES
from fastsafetensors_amd import Device, DeviceType, DType, SafeTensorsMetadata, TensorFrame
from fastsafetensors_amd.frameworks import get_framework_op
from fastsafetensors_amd.st_types import dtype_size
from oracle import st_oracle as orc


def test_device_parsing():
    with pytest.raises(ValueError, match="Unknown device type: aaaa"):
        Device.from_str("aaaa:0")
    with pytest.raises(ValueError, match="Invalid index: -xxx"):
        Device.from_str("cpu:-xxx")
    with pytest.raises(ValueError, match="Unknown device type: aaa"):
        Device.from_str("aaa")
    cuda = Device.from_str("cuda:4")
    assert cuda.type == DeviceType.CUDA and cuda.index == 4 and cuda.as_str() == "cuda:4"
    cpu = Device(DeviceType.CPU, None)
    assert cpu.type == DeviceType.CPU and cpu.index is None and cpu.as_str() == "cpu"
    assert Device.from_str("CUDA:1").type == DeviceType.CUDA


def test_dtype_table_matches_torch():
    fw = get_framework_op("pytorch")
    from fastsafetensors_amd.frameworks._torch import dtype_convert

    for dt, tdt in dtype_convert.items():
        if dt == DType.F4:
            assert fw.get_dtype_size(dt) == 0.5
        else:
            assert fw.get_dtype_size(dt) == float(tdt.itemsize) == dtype_size(dt)
    assert {d.value for d in DType} - {"AUTO"} == set(orc.DTYPE_BITS)
    assert fw.as_workaround_dtype(DType.F8_E4M3) == DType.I8 and fw.as_workaround_dtype(DType.F4) == DType.U8
    assert fw.as_workaround_dtype(DType.BF16) == DType.BF16
    assert fw.get_device_ptr_align() == 16


def test_framework_errors():
    with pytest.raises(Exception, match="Unknown framework name"):
        get_framework_op("aaaaa")
    fw = get_framework_op("pt")
    assert fw is get_framework_op("pytorch") and fw.get_name() == "pytorch"
    t = fw.get_empty_tensor([1], DType.F16, Device.from_str("cpu"))
    with pytest.raises(Exception):
        fw.is_equal(t, [0.0])
    with pytest.raises(Exception):
        fw.get_process_group(0)
    ver = fw.get_cuda_ver()
    assert ver.startswith("hip-") or ver == "0.0"


def test_f4_shape_helpers_known_answers():
    # reference: test_float4_native_shape_and_slices (test_fastsafetensors.py:718-744)
    fw = get_framework_op("pytorch")
    assert fw.get_native_shape(DType.F4, [8, 16]) == [8, 8]
    assert fw.get_native_shape(DType.F4, [16]) == [8]
    assert fw.get_storage_shape(DType.F4, [8, 16], [16, 1]) == ([64], [1])
    assert fw.get_native_slices(DType.F4, [8, 16], (slice(None, None, None), slice(4, 12, 1))) == (
        slice(None, None, None), slice(2, 6, 1))
    assert fw.get_native_slices(DType.F4, [8, 16], (slice(2, 6, 1),)) == (slice(2, 6, 1),)
    with pytest.raises(ValueError):
        fw.get_native_shape(DType.F4, [8, 15])
    with pytest.raises(ValueError):
        fw.get_storage_shape(DType.F4, [8, 15], [15, 1])
    with pytest.raises(ValueError):
        fw.get_native_slices(DType.F4, [8, 16], (slice(None, None, None), slice(3, 12, 1)))
    assert fw.get_native_shape(DType.BF16, [3, 5]) == [3, 5]


@pytest.mark.parametrize("name", GOLDEN_FILES)
def test_metadata_agrees_with_oracle_and_library(golden, name):
    path = golden(name)
    meta = SafeTensorsMetadata.from_file(path, get_framework_op("pytorch"))
    h = orc.parse_file(path)
    assert meta.header_length == h.header_length and meta.size_bytes == h.size_bytes == os.path.getsize(path)
    assert meta.aligned == h.aligned == (meta.header_length % 16 == 0)
    assert list(meta.tensors) == list(h.tensors)
    for key, frame in meta.tensors.items():
        assert frame.dtype.value == h.tensors[key]["dtype"]
        assert frame.shape == h.tensors[key]["shape"] and frame.data_offsets == h.tensors[key]["data_offsets"]
    ref = load_file(path)
    for key, t in ref.items():
        want = list(t.shape)
        if meta.tensors[key].dtype == DType.F4:
            want[-1] *= 2  # the file counts fp4 values, torch counts packed bytes
        assert meta.tensors[key].shape == want


def test_fixture_a_known_header(golden):
    meta = SafeTensorsMetadata.from_file(golden("a.safetensors"))
    assert meta.header_length == 104 and not meta.aligned and meta.metadata == {"fst": "sample"}
    f = meta.tensors["a0"]
    assert (f.dtype, f.shape, f.data_offsets, f.strides, f.offsets, f.sliced) == (DType.F16, [16, 8], [0, 256], [8, 1], [0, 0], False)
    assert "a0" in repr(meta)


def _blob(text: str, data: bytes = b"") -> bytes:
    j = text.encode()
    return len(j).to_bytes(8, "little") + j + data


def test_header_errors(tmp_path):
    def from_bytes(b, total=None):
        return SafeTensorsMetadata.from_bytes(b, len(b) if total is None else total, "testfile")

    with pytest.raises(Exception, match="HeaderTooSmall"):
        SafeTensorsMetadata.from_buffer(0, 4, "testfile")
    with pytest.raises(Exception, match="HeaderTooSmall"):
        from_bytes(b"\0\0\0")
    with pytest.raises(Exception, match="HeaderTooLarge"):
        from_bytes((100_000_001).to_bytes(8, "little") + b"{}", 1024)
    with pytest.raises(Exception, match="InvalidHeaderLength"):
        from_bytes((100).to_bytes(8, "little") + b" " * 42, 50)
    one = '{"a":{"dtype":"F32","shape":[2],"data_offsets":[%d,%d]}}'
    assert from_bytes(_blob(one % (0, 8), b"x" * 8)).tensors["a"].shape == [2]
    assert from_bytes(_blob(one % (0, 8), b"x" * 12)).data_length == 8  # trailing bytes tolerated
    with pytest.raises(Exception, match="InvalidOffset"):
        from_bytes(_blob(one % (4, 12), b"x" * 12))
    with pytest.raises(Exception, match="TensorInvalidInfo"):
        from_bytes(_blob(one % (0, 12), b"x" * 12))
    with pytest.raises(Exception, match="MetadataIncompleteBuffer"):
        from_bytes(_blob(one % (0, 8), b"x" * 7))
    with pytest.raises(ValueError):
        from_bytes(_blob('{"a":{"dtype":"F3","shape":[2],"data_offsets":[0,8]}}', b"x" * 8))  # unknown dtype tag
    only_meta = from_bytes(_blob('{"__metadata__": {"data_offsets": [0, 123]}}'))
    assert only_meta.tensors == {} and isinstance(only_meta, SafeTensorsMetadata)
    # from_buffer parses a header that sits in host memory
    import ctypes

    raw = _blob(one % (0, 8), b"y" * 8)
    buf = ctypes.create_string_buffer(raw, len(raw))
    assert SafeTensorsMetadata.from_buffer(ctypes.addressof(buf), len(raw), "mem").tensors["a"].data_offsets == [0, 8]
    # files: too small, and ENOENT
    tiny = tmp_path / "tiny.safetensors"
    tiny.write_bytes(b"abc")
    with pytest.raises(Exception, match="HeaderTooSmall"):
        SafeTensorsMetadata.from_file(str(tiny))
    with pytest.raises(FileNotFoundError):
        SafeTensorsMetadata.from_file(str(tmp_path / "missing.safetensors"))


def test_from_fd_survives_short_reads(monkeypatch, golden):
    # reference regression: test_from_fd_short_reads (test_fastsafetensors.py:932-955)
    real_read = os.read
    monkeypatch.setattr(os, "read", lambda fd, n: real_read(fd, min(n, 3)))
    fd = os.open(golden("tiny_gpt2.safetensors"), os.O_RDONLY)
    try:
        meta = SafeTensorsMetadata.from_fd(fd, "tiny", None)
    finally:
        os.close(fd)
    assert len(meta.tensors) == 48 and meta.tensors["h.0.mlp.c_proj.weight"].shape == [8, 16]


def test_tensor_frame_getitem_follows_sequences():
    # reference: test_tensor_frame_getitem (test_fastsafetensors.py:799-849), plus the oracle
    n, m = 5, 6

    def frame():
        return TensorFrame(DType.F32, [n, m], [0, n * m * 4], [m, 1], [0, 0], False)

    ref = list(range(n))
    for i in range(-n, n):
        got = frame()[i]
        assert got.shape == [1, m] and got.offsets[0] == ref[i]
    for i in (n, -n - 1):
        with pytest.raises(IndexError):
            frame()[i]
    bounds = [None, -n - 2, -n, -2, -1, 0, 1, n - 2, n - 1, n, n + 2]
    for start, stop, step in itertools.product(bounds, bounds, [None, 1, 2, 3, -1, -2]):
        sl = slice(start, stop, step)
        got, want = frame()[sl], ref[sl]
        theirs = orc.frame_getitem([n, m], sl)
        if not want:
            assert got.shape == [] and theirs is None
            continue
        assert got.shape[1] == m
        assert [got.offsets[0] + k * (got.strides[0] // m) for k in range(got.shape[0])] == want
        assert (got.shape, got.strides, got.offsets) == theirs
    with pytest.raises(ValueError):
        frame()[::0]
    whole = frame()[()]
    assert (whole.shape, whole.offsets, whole.strides) == ([n, m], [0, 0], [m, 1])
    got = frame()[1:-1, ::2]
    assert (got.shape, got.offsets, got.strides) == ([n - 2, m // 2], [1, 0], [m, 2])
    assert got.sliced and got.data_offsets == [0, n * m * 4]
    with pytest.raises(Exception):
        frame()[0, 0, 0]
    with pytest.raises(Exception):
        frame()["x"]
    nested = frame()[1:4][1:]  # offsets accumulate
    assert nested.offsets == [2, 0] and nested.shape == [2, m]


@pytest.mark.parametrize("name", GOLDEN_FILES)
def test_batched_views_equal_the_views_made_one_by_one(golden, name):
    """``view_tensors`` (one typed view of the buffer per dtype + ``as_strided``) against ``view_tensor``
    (slice, view, view) over a host copy of the file: same address, shape, strides, dtype and bytes for
    every tensor -- scalars, packed fp4, empty tensors and tensors at odd offsets included."""
    import numpy as np
    import torch

    from fastsafetensors_amd import _native

    path = golden(name)
    fwk = get_framework_op("pytorch")
    meta = SafeTensorsMetadata.from_file(path, fwk)
    raw = np.fromfile(path, dtype=np.uint8)[meta.header_length:]
    arena = torch.zeros(raw.size + 16, dtype=torch.uint8)
    arena[: raw.size] = torch.from_numpy(raw.copy())
    buf = _native.DeviceBuffer(arena.data_ptr(), arena.numel(), True)
    buf.keepalive = arena
    from fastsafetensors_amd.st_types import Device

    device = Device.from_str("cpu")
    items = [(k, f.data_offsets[0], f) for k, f in meta.tensors.items()]
    one_by_one = {}
    for k, off, f in items:
        try:
            one_by_one[k] = fwk.view_tensor(buf, off, f, device).get_raw()
        except RuntimeError:
            one_by_one[k] = None  # torch refuses a view at an offset that is odd for the dtype (the copier realigns those)
    aligned = [(k, off, f) for k, off, f in items if one_by_one[k] is not None]
    batched = fwk.view_tensors(buf, aligned, device)
    assert list(batched) == [k for k, _, _ in aligned]
    for k, _, f in aligned:
        a, b = one_by_one[k], batched[k].get_raw()
        assert a.dtype == b.dtype and a.shape == b.shape and a.stride() == b.stride() and b.is_contiguous(), k
        assert (a.numel() == 0 and b.numel() == 0) or a.data_ptr() == b.data_ptr(), k
        assert torch.equal(a.reshape(-1).view(torch.uint8), b.reshape(-1).view(torch.uint8)), k
    with pytest.raises(IndexError):
        fwk.view_tensors(buf, [(items[0][0], arena.numel() - 1, items[0][2])], device)
