# SPDX-License-Identifier: Apache-2.0
"""TEST INFRASTRUCTURE -- CPU oracle of the safetensors load path.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this module; the ``fastsafetensors_amd`` package never
does.  It restates, with numpy and plain Python, what the reference
(foundation-model-stack/fastsafetensors 0.3.2) computes on the load path, so
that the HIP path can be compared with it byte for byte:

=====================  ==========================================================
function               follows (paths relative to the reference root)
=====================  ==========================================================
``parse_header``       ``fastsafetensors/common.py:184-243`` (validation) and
                       ``:270-304`` (size checks of ``from_fd``)
``frame_getitem``      ``fastsafetensors/common.py:418-471`` (``TensorFrame.__getitem__``)
``tensor_bytes``       ``fastsafetensors/common.py:319-333`` with the nogds layout of
                       ``copier/nogds.py:42-51``: bytes ``[header+s, header+e)``
``rank_slices``        ``fastsafetensors/tensor_factory.py:145-156`` (block = ceil(S/N))
``shard_bytes``        ``fastsafetensors/tensor_factory.py:168-175`` (slice + contiguous),
                       packed F4 bounds per ``frameworks/_torch.py:353-389``
``push_outcome``       ``fastsafetensors/tensor_factory.py:58-116`` (who gets what)
``realign``            ``fastsafetensors/copier/gds.py:138-159`` (shift by header % 16)
``NogdsReader`` (C)    ``fastsafetensors/cpp/ext.cpp:648-806`` via ``nogds_oracle.c``
=====================  ==========================================================

What pins each function (see ``tests/test_oracle.py``): the reference's
committed fixture ``examples/a.safetensors`` (row ``i`` of ``a0`` is all
``float16(i)``), the closed-form tiny-gpt2 generator of the reference's
``tests/unit/conftest.py:68-115``, the independent ``safetensors`` library
(``load_file``) with torch slicing -- the oracle the reference's own tests use
(``tests/unit/test_fastsafetensors.py:34-55``, ``tests/unit/test_multi.py:44-64``)
-- Python ``list`` slicing for the frame algebra (``test_fastsafetensors.py:799-849``),
and the reference's own C++ reader compiled into ``oracle/_ref`` for the
threaded reader.  No function is left unpinned.
"""

import ctypes
import importlib.util
import json
import os
import sysconfig
from collections import OrderedDict
from typing import Any, Dict, List, Optional, Sequence, Tuple

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))

# bits per element of each safetensors dtype tag (st_types.py:45-63, _torch.py:277-283)
DTYPE_BITS = {
    "BOOL": 8, "I8": 8, "U8": 8, "F8_E5M2": 8, "F8_E4M3": 8, "F8_E8M0": 8, "F4": 4,
    "I16": 16, "U16": 16, "F16": 16, "BF16": 16, "I32": 32, "U32": 32, "F32": 32,
    "I64": 64, "U64": 64, "F64": 64,
}


class Header:
    def __init__(self, header_length: int, size_bytes: int, metadata: Any, tensors: "OrderedDict[str, dict]"):
        self.header_length = header_length
        self.size_bytes = size_bytes
        self.metadata = metadata
        self.tensors = tensors  # name -> {"dtype", "shape", "data_offsets"} in offset order
        self.aligned = header_length % 16 == 0


def parse_header(blob: bytes, size_bytes: Optional[int] = None, src: str = "") -> Header:
    """Parse + validate the first bytes of a file (``blob`` must hold the whole header)."""
    size_bytes = len(blob) if size_bytes is None else size_bytes
    if size_bytes < 8:
        raise Exception(f"{src}: HeaderTooSmall, buffer_len={size_bytes}")
    n = int.from_bytes(blob[:8], "little", signed=False)
    if n > 100000000:
        raise Exception(f"{src}: HeaderTooLarge, n={n}")
    if n > size_bytes - 8:
        raise Exception(f"{src}: InvalidHeaderLength, n={n}")
    ser = json.loads(blob[8 : 8 + n].decode("utf-8"), object_pairs_hook=OrderedDict)
    metadata = ser.get("__metadata__", "")
    if metadata:
        del ser["__metadata__"]
    header_length = n + 8
    start = 0
    tensors: "OrderedDict[str, dict]" = OrderedDict()
    for name, entry in sorted(ser.items(), key=lambda kv: kv[1]["data_offsets"][0]):
        s, e = entry["data_offsets"]
        if s != start or e < s:
            raise Exception(f"validate(tensor {name}): InvalidOffset s={s}, start={start}, e={e}")
        start = e
        nelements = 1
        for sh in entry["shape"]:
            nelements *= sh
        nbytes = nelements * DTYPE_BITS[entry["dtype"]] // 8
        if e - s != nbytes:
            raise Exception(f"validate(tensor {name}): TensorInvalidInfo, e-s={e - s}, nbytes={nbytes}")
        tensors[name] = {"dtype": entry["dtype"], "shape": list(entry["shape"]), "data_offsets": [s, e]}
    if start + header_length > size_bytes:
        raise Exception(f"MetadataIncompleteBuffer, src={src}, start={start}")
    return Header(header_length, size_bytes, metadata, tensors)


def parse_file(path: str) -> Header:
    size = os.path.getsize(path)
    with open(path, "rb") as f:
        head = f.read(8)
        if len(head) < 8:
            raise Exception(f"{path}: HeaderTooSmall, buffer_len={size}")
        n = int.from_bytes(head, "little")
        body = f.read(min(n, 100000001)) if n <= size else b""
    return parse_header(head + body, size, path)


def frame_getitem(shape: Sequence[int], index) -> Optional[Tuple[List[int], List[int], List[int]]]:
    """``(shape, strides, offsets)`` of ``frame[index]`` for a row-major frame of
    ``shape``; ``None`` for an empty selection (the reference then returns a frame
    with ``shape == []``)."""
    strides = [1] * len(shape)
    for i in range(len(shape) - 2, -1, -1):
        strides[i] = strides[i + 1] * shape[i + 1]
    if isinstance(index, (slice, int)):
        index = (index,)
    if len(index) > len(shape):
        raise Exception("too large slice")
    out_shape, out_strides, out_offsets = [], [], []
    for dim, v in enumerate(index):
        if isinstance(v, int):
            if v >= shape[dim] or v < -shape[dim]:
                raise IndexError(v)
            start = v + shape[dim] if v < 0 else v
            step, length = 1, 1
        else:
            if v.step == 0:
                raise ValueError("slice step cannot be zero")
            start, stop, step = v.indices(shape[dim])
            length = stop - start
            if length == 0 or (length < 0 and step > 0) or (length > 0 and step < 0):
                return None
            length = abs(length)
        out_offsets.append(start)
        out_strides.append(strides[dim] * step)
        out_shape.append((length + abs(step) - 1) // abs(step))
    for dim in range(len(index), len(shape)):
        out_offsets.append(0)
        out_strides.append(strides[dim])
        out_shape.append(shape[dim])
    return out_shape, out_strides, out_offsets


def file_bytes(path: str, lo: int, hi: int) -> np.ndarray:
    return np.fromfile(path, dtype=np.uint8, count=hi - lo, offset=lo)


def tensor_bytes(path: str, header: Header, name: str) -> np.ndarray:
    """Raw little-endian bytes of one tensor, straight from the file."""
    s, e = header.tensors[name]["data_offsets"]
    return file_bytes(path, header.header_length + s, header.header_length + e)


def rank_slices(shape: Sequence[int], dim: int, rank: int, world: int) -> Tuple[slice, ...]:
    block = (shape[dim] + world - 1) // world
    return (slice(None),) * dim + (slice(rank * block, (rank + 1) * block, 1),)


def shard_bytes(raw: np.ndarray, dtype: str, shape: Sequence[int], dim: int, rank: int, world: int
                ) -> Tuple[np.ndarray, List[int]]:
    """Bytes and logical shape of rank ``rank``'s contiguous block along ``dim``.

    Works on bytes: the tensor is viewed as ``shape[:-1] + [row_bytes]`` so that
    any dtype, packed F4 included, slices with numpy's own indexing.
    """
    if dim == -1:
        return raw.copy(), list(shape)
    bits = DTYPE_BITS[dtype]
    sl = rank_slices(shape, dim, rank, world)
    lo, hi, _ = sl[dim].indices(shape[dim])
    hi = max(hi, lo)
    out_shape = list(shape)
    out_shape[dim] = hi - lo
    last = len(shape) - 1
    if dim == last:
        if (lo * bits) % 8 or (hi * bits) % 8 or (shape[last] * bits) % 8:
            raise ValueError("packed sub-byte slice bounds must align to storage units")
        byte_shape = list(shape[:-1]) + [shape[last] * bits // 8]
        view = raw.reshape(byte_shape)
        cut = view[(slice(None),) * dim + (slice(lo * bits // 8, hi * bits // 8),)]
    else:
        if (shape[last] * bits) % 8:
            raise ValueError("last dimension must be divisible by the packing ratio")
        byte_shape = list(shape[:-1]) + [shape[last] * bits // 8]
        cut = raw.reshape(byte_shape)[sl]
    return np.ascontiguousarray(cut).reshape(-1), out_shape


def push_outcome(world: int, me: int, dst_rank: int, src_rank: int) -> str:
    """What ``push`` hands back on rank ``me``: "view", "clone", "recv" or "none"."""
    if world == 1:
        return "view"
    if me != dst_rank and me != src_rank:
        return "none"
    if me == dst_rank and src_rank == dst_rank:
        return "clone"
    if me == src_rank:
        return "none"
    return "recv"


def realign(window: np.ndarray, header_length: int, window_start: int, data_length: int) -> np.ndarray:
    """The data section as it sits after shifting it to offset 0 of its buffer."""
    lead = header_length - window_start
    return window[lead : lead + data_length].copy()


# ---- compiled parts -------------------------------------------------------------------


def build(ref: str = "/root/reference") -> None:
    """Compile ``nogds_oracle.c`` (and ``_ref`` when the reference tree is present)."""
    import subprocess

    subprocess.run(["make", "-s", "-C", HERE, f"REF={ref}"], check=True)


_clib: Optional[ctypes.CDLL] = None


def clib() -> ctypes.CDLL:
    global _clib
    if _clib is None:
        path = os.path.join(HERE, "libfst_oracle.so")
        if not os.path.exists(path):
            build()
        lib = ctypes.CDLL(path)
        vp, u64, i64 = ctypes.c_void_p, ctypes.c_uint64, ctypes.c_int64
        lib.fst_oracle_reader_new.restype = vp
        lib.fst_oracle_reader_new.argtypes = [u64, u64]
        lib.fst_oracle_reader_free.argtypes = [vp]
        lib.fst_oracle_bounce_bytes.restype = u64
        lib.fst_oracle_bounce_bytes.argtypes = [vp]
        lib.fst_oracle_submit_read.restype = ctypes.c_int
        lib.fst_oracle_submit_read.argtypes = [vp, ctypes.c_int, vp, u64, i64, i64, u64]
        lib.fst_oracle_wait_read.restype = ctypes.c_int
        lib.fst_oracle_wait_read.argtypes = [vp, ctypes.c_int]
        lib.fst_oracle_load_file.restype = i64
        lib.fst_oracle_load_file.argtypes = [vp, ctypes.c_char_p, u64, u64, vp, u64]
        lib.fst_oracle_alloc.restype = vp
        lib.fst_oracle_alloc.argtypes = [u64]
        lib.fst_oracle_free.argtypes = [vp]
        lib.fst_oracle_memmove.restype = ctypes.c_int
        lib.fst_oracle_memmove.argtypes = [vp, u64, u64, u64, vp, u64, u64]
        lib.fst_oracle_slice.argtypes = [vp, vp, u64, u64, u64]
        _clib = lib
    return _clib


class NogdsReader:
    """The restated thread-per-request reader with its bounce buffer."""

    def __init__(self, bbuf_size_kb: int = 16 * 1024, max_threads: int = 16):
        self._r = clib().fst_oracle_reader_new(bbuf_size_kb, max_threads)

    def load_file(self, path: str, header: Header, max_copy_block_size: int = 16 * 1024**3) -> np.ndarray:
        """Data section of ``path`` in a 4096-aligned host buffer (as a numpy view)."""
        total = header.size_bytes - header.header_length
        out = np.empty(total + 4096, dtype=np.uint8)
        skip = -out.ctypes.data % 4096
        out = out[skip : skip + total]
        got = clib().fst_oracle_load_file(
            self._r, os.fsencode(path), header.header_length, header.size_bytes,
            out.ctypes.data, max_copy_block_size,
        )
        if got != total:
            raise Exception(f"wait_io: wait_nogds_read failed, path={path}")
        return out

    def bounce_bytes(self) -> int:
        return int(clib().fst_oracle_bounce_bytes(self._r))

    def close(self) -> None:
        if self._r:
            clib().fst_oracle_reader_free(self._r)
            self._r = None

    def __del__(self) -> None:
        self.close()


def slice_c(raw: np.ndarray, outer: int, seg: int, pitch: int, first: int) -> np.ndarray:
    out = np.empty(outer * seg, dtype=np.uint8)
    src = np.ascontiguousarray(raw)
    clib().fst_oracle_slice(out.ctypes.data, src.ctypes.data + first, outer, seg, pitch)
    return out


def load_reference_cpp():
    """The reference's own pybind11 module built into ``oracle/_ref`` or ``None``.

    Only the compiled C++ (``cpp/ext.cpp``) is loaded; none of the reference's
    Python is imported."""
    path = os.path.join(HERE, "_ref", "fastsafetensors_cpp" + sysconfig.get_config_var("EXT_SUFFIX"))
    if not os.path.exists(path):
        return None
    spec = importlib.util.spec_from_file_location("fastsafetensors_cpp", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod
