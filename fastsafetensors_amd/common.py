# SPDX-License-Identifier: Apache-2.0
"""Safetensors header model: ``SafeTensorsMetadata`` and ``TensorFrame``.

Behavioural mirror of the reference's ``fastsafetensors/common.py``:

* header parse and validation            -> ``common.py:184-243`` / ``:270-304``
* short-read tolerant header read        -> ``common.py:158-171``
* shape/stride/offset slice algebra      -> ``common.py:383-471``
* tensor instantiation over one buffer   -> ``common.py:319-377``
* ``SingleGroup`` and NUMA node lookup   -> ``common.py:175-180`` / ``:40-51``

On disk a file is ``u64le N | N bytes of JSON | data section``; every tensor's
``data_offsets`` are relative to the data section, which starts at
``header_length = 8 + N``.
"""

import json
import logging
import os
from collections import OrderedDict
from dataclasses import dataclass
from typing import Any, Dict, List, Mapping, Optional, Sequence, Tuple, Union

from .st_types import Device, DType, dtype_bits

MAX_HEADER_JSON_BYTES = 100_000_000


def init_logger(name: str) -> logging.Logger:
    return logging.getLogger(name)


def is_debug(logger: logging.Logger) -> bool:
    return logger.isEnabledFor(logging.DEBUG)


logger = init_logger(__name__)


class SingleGroup:
    """World of one process; kept for callers that pass it as ``pg``."""

    def size(self) -> int:
        return 1

    def rank(self) -> int:
        return 0


def get_device_numa_node(device: Optional[int]) -> Optional[int]:
    """NUMA node of GPU ``device`` from its PCI bus id, or None when unknown."""
    if device is None or not os.path.isdir("/sys/class/pci_bus"):
        return None
    from . import _native

    pci_addr = _native.get_device_pci_bus(device)
    if not pci_addr:
        return None
    domain_bus = ":".join(pci_addr.split(":")[:2]).lower()
    node_file = f"/sys/class/pci_bus/{domain_bus}/device/numa_node"
    try:
        with open(node_file) as f:
            return int(f.read().strip())
    except (OSError, ValueError):
        return None


def _read_exact(fd: int, length: int, filename: str) -> bytes:
    """``length`` bytes from ``fd``; keeps reading after short reads."""
    got = bytearray()
    while len(got) < length:
        piece = os.read(fd, length - len(got))
        if not piece:
            raise Exception(
                f"{filename}: UnexpectedEOF, expected {length} more bytes but got {len(got)}"
            )
        got += piece
    return bytes(got)


def _check_header_size(n: int, buffer_len: int, where: str) -> None:
    if n > MAX_HEADER_JSON_BYTES:
        raise Exception(f"{where}: HeaderTooLarge, n={n}, buffer_len={buffer_len}")
    if n > buffer_len - 8:
        raise Exception(f"{where}: InvalidHeaderLength, n={n}, buffer_len={buffer_len}")


Index = Union[int, slice]
_DTYPE_OF_TAG = {d.value: d for d in DType}
_BITS_OF_TAG = {d.value: dtype_bits(d) for d in DType if d.value != "AUTO"}


@dataclass
class TensorFrame:
    """Shape, element strides and per-dim start offsets of a (sliced) tensor.

    ``data_offsets`` always names the byte range of the *whole* tensor in the
    data section; a slice only changes ``shape``/``strides``/``offsets``.
    """

    dtype: DType
    shape: List[int]
    data_offsets: List[int]
    strides: List[int]
    offsets: List[int]
    sliced: bool

    @classmethod
    def from_buffer(cls, entry: Dict[str, Any]) -> "TensorFrame":
        shape = entry["shape"]
        rank = len(shape)
        if rank == 2:  # most tensors of a checkpoint
            strides = [shape[1], 1]
        else:
            strides = [1] * rank
            for d in range(rank - 2, -1, -1):
                strides[d] = strides[d + 1] * shape[d + 1]
        tag = entry["dtype"]
        dtype = _DTYPE_OF_TAG.get(tag)
        if dtype is None:
            dtype = DType(tag)  # raises for an unknown tag, as the enum does
        return cls(dtype, shape, list(entry["data_offsets"]), strides, [0] * rank, False)

    def __repr__(self) -> str:
        return str({"dtype": self.dtype, "shape": self.shape, "data_offsets": self.data_offsets})

    def _empty(self) -> "TensorFrame":
        # the reference reports an empty selection as a frame without dims
        return TensorFrame(self.dtype, [], self.data_offsets, [], [], False)

    def __getitem__(self, index: Union[Index, Tuple[Index, ...]]) -> "TensorFrame":
        if isinstance(index, (int, slice)):
            index = (index,)
        elif not isinstance(index, tuple):
            raise Exception(f"[BUG] Unsupported index type for DiskTensor: {index}")
        if len(index) > len(self.shape):
            raise Exception(f"[BUG] tried to get too large slice {index} from {self.shape}")

        shape = list(self.shape)
        strides = list(self.strides)
        offsets = list(self.offsets)
        for dim, sel in enumerate(index):
            extent = self.shape[dim]
            if isinstance(sel, int):
                if not -extent <= sel < extent:
                    raise IndexError(
                        f"[BUG] tried to access index {sel} at dim={dim} for shape={self.shape}"
                    )
                first, step, count = sel % extent, 1, 1
            elif isinstance(sel, slice):
                if sel.step == 0:
                    raise ValueError("[BUG] slice step cannot be zero")
                first, stop, step = sel.indices(extent)
                count = len(range(first, stop, step))
                if count == 0:
                    return self._empty()
            else:
                raise Exception(
                    f"[BUG] Unsupported index type for DiskTensor: {index} at dim={dim}"
                )
            offsets[dim] = self.offsets[dim] + first
            strides[dim] = self.strides[dim] * step
            shape[dim] = count
        return TensorFrame(self.dtype, shape, self.data_offsets, strides, offsets, True)

    @property
    def nbytes(self) -> int:
        return self.data_offsets[1] - self.data_offsets[0]


class LazyFrames(Mapping):
    """``name -> TensorFrame`` of one file, in offset order, over the header's own entries.

    The header has been validated by whoever builds this; the frame objects -- hundreds per file --
    are made at the first look at one of them, all at once.  Keys, length and membership need none,
    so registering a file's names costs no frame, and a loader makes them while the file's bytes
    are already on their way."""

    __slots__ = ("_entries", "_frames")

    def __init__(self, entries: Dict[str, Dict[str, Any]]):
        self._entries = entries
        self._frames: Optional[Dict[str, TensorFrame]] = None

    def _all(self) -> Dict[str, TensorFrame]:
        if self._frames is None:
            self._frames = {name: TensorFrame.from_buffer(entry) for name, entry in self._entries.items()}
        return self._frames

    def __getitem__(self, name: str) -> TensorFrame:
        return self._all()[name]

    def __iter__(self):
        return iter(self._entries)

    def __len__(self) -> int:
        return len(self._entries)

    def __contains__(self, name: object) -> bool:
        return name in self._entries

    def keys(self):
        return self._entries.keys()

    def values(self):
        return self._all().values()

    def items(self):
        return self._all().items()

    def spans(self) -> List[Tuple[int, int]]:
        """(first byte in the data section, bytes) of every tensor, without making a frame."""
        return [(e["data_offsets"][0], e["data_offsets"][1] - e["data_offsets"][0]) for e in self._entries.values()]

    def __repr__(self) -> str:
        return repr(dict(self._all()))


class SafeTensorsMetadata:
    """Parsed and validated header of one ``.safetensors`` file."""

    def __init__(
        self,
        string: str,
        header_length: int,
        size_bytes: int,
        framework: Any = None,
        src: str = "",
        keep_orig_dict: bool = False,
    ):
        self.src = src
        self.framework = framework
        self.header_length = header_length
        self.size_bytes = size_bytes
        table = json.loads(string)  # a plain dict keeps the file's key order (and parses in C throughout)
        self.metadata = table.pop("__metadata__", "") or ""
        if keep_orig_dict:
            self.ser = table
        ptr_align = framework.get_device_ptr_align() if framework is not None else 16
        self.aligned = header_length % ptr_align == 0

        cursor = 0
        items = list(table.items())
        spans = [tuple(entry["data_offsets"]) for _, entry in items]
        if any(a > b for a, b in zip(spans, spans[1:])):  # writers emit them in offset order; sort only when not
            # by (begin, end): an empty tensor shares its offset with its successor and must come first
            # (the reference sorts by begin alone and then depends on the order of the JSON for such a pair)
            items.sort(key=lambda kv: tuple(kv[1]["data_offsets"]))
        for name, entry in items:
            begin, end = entry["data_offsets"]
            if begin != cursor or end < begin:
                raise Exception(
                    f"validate(tensor {name}): InvalidOffset s={begin}, start={cursor}, e={end}, src={src}"
                )
            count = 1
            for extent in entry["shape"]:
                count *= extent
            bits = _BITS_OF_TAG.get(entry["dtype"])
            if bits is None:
                bits = dtype_bits(DType(entry["dtype"]))  # raises for an unknown tag, as the enum does
            expect = count * bits // 8
            if end - begin != expect:
                raise Exception(
                    f"validate(tensor {name}): TensorInvalidInfo, e-s={end - begin}, nbytes={expect}, src={src}"
                )
            cursor = end
        # the frames themselves are made when somebody first asks for one
        self.tensors: Mapping = LazyFrames(dict(items))
        self.data_length = cursor
        if header_length + cursor > size_bytes:
            raise Exception(
                f"MetadataIncompleteBuffer, src={src}, start={cursor}, "
                f"header_length={header_length}, size_bytes={size_bytes}"
            )
        if header_length + cursor < size_bytes:
            # bytes after the last tensor are tolerated (padding of sub-byte dtypes)
            logger.debug(
                "trailing %d bytes after tensor data in %s",
                size_bytes - header_length - cursor,
                src,
            )

    # -- constructors -----------------------------------------------------
    @classmethod
    def from_bytes(
        cls, blob: bytes, total_len: int, filename: str, framework: Any = None
    ) -> "SafeTensorsMetadata":
        """Parse from the first ``8 + N`` bytes of a file of ``total_len`` bytes."""
        if total_len < 8 or len(blob) < 8:
            raise Exception(f"{filename}: HeaderTooSmall, buffer_len={total_len}")
        n = int.from_bytes(blob[:8], "little")
        _check_header_size(n, total_len, filename)
        return cls(blob[8 : 8 + n].decode("utf-8"), n + 8, total_len, framework, filename)

    @classmethod
    def from_buffer(
        cls, buf: int, buffer_len: int, filename: str, framework: Any = None
    ) -> "SafeTensorsMetadata":
        """Parse a header that sits in host memory at address ``buf``."""
        if buffer_len < 8:
            raise Exception(
                f"from_buffer: HeaderTooSmall, filename={filename}, buffer_len={buffer_len}"
            )
        from . import _native

        n = int.from_bytes(_native.read_buffer(buf, 8), "little")
        _check_header_size(n, buffer_len, f"from_buffer: filename={filename}")
        text = _native.read_buffer(buf + 8, n).decode("utf-8")
        return cls(text, n + 8, buffer_len, framework)

    @classmethod
    def from_fd(
        cls, fd: int, filename: str, framework: Any = None, keep_orig_dict: bool = False
    ) -> "SafeTensorsMetadata":
        buffer_len = os.fstat(fd).st_size
        if buffer_len < 8:
            raise Exception(f"{filename}: HeaderTooSmall, buffer_len={buffer_len}")
        n = int.from_bytes(_read_exact(fd, 8, filename), "little")
        _check_header_size(n, buffer_len, filename)
        text = _read_exact(fd, n, filename).decode("utf-8")
        return cls(text, n + 8, buffer_len, framework, filename, keep_orig_dict=keep_orig_dict)

    @classmethod
    def from_file(cls, filename: str, framework: Any = None) -> "SafeTensorsMetadata":
        fd = os.open(filename, os.O_RDONLY)
        try:
            return cls.from_fd(fd, filename, framework)
        finally:
            os.close(fd)

    # -- tensor instantiation ---------------------------------------------
    def get_tensors(
        self,
        gbuf: Any,
        device: Device,
        copy_start_offset: int,
        dtype: DType = DType.AUTO,
    ) -> Dict[str, Any]:
        """Zero-copy views of every tensor over ``gbuf``.

        ``gbuf`` byte 0 holds file byte ``copy_start_offset``; the view of a
        tensor therefore starts at ``header_length + s - copy_start_offset``.
        """
        if dtype != DType.AUTO and any(f.dtype != dtype for f in self.tensors.values()):
            raise NotImplementedError(
                "get_tensors builds views only; conversion on load is done by the copier (wait_io)"
            )
        shift = self.header_length - copy_start_offset
        return self.framework.view_tensors(
            gbuf, [(name, shift + frame.data_offsets[0], frame) for name, frame in self.tensors.items()], device
        )

    def __repr__(self) -> str:
        return str({"__metadata__": self.metadata, "tensors": self.tensors})


def shard_slices(shape: Sequence[int], dim: int, rank: int, world: int) -> Tuple[slice, ...]:
    """Index tuple selecting rank ``rank``'s block of ``ceil(shape[dim]/world)``
    along ``dim`` (the partition rule of ``tensor_factory.py:145-156``)."""
    block = -(-shape[dim] // world)
    return (slice(None),) * dim + (slice(rank * block, (rank + 1) * block, 1),)
