# SPDX-License-Identifier: Apache-2.0
"""Device and dtype vocabulary of the safetensors load path.

Mirrors the public names of the reference's ``fastsafetensors/st_types.py:8-63``
(``DeviceType``, ``Device``, ``DType``) so that callers can switch packages
without touching their code.  The per-dtype byte widths that the reference keeps
in its torch backend (``frameworks/_torch.py:277-283``) live here as plain data,
because the header validator needs them without importing torch.
"""

from dataclasses import dataclass
from enum import Enum
from typing import Optional


class DeviceType(Enum):
    CPU = "cpu"
    CUDA = "cuda"
    GPU = "gpu"


def _device_type(text: str) -> DeviceType:
    try:
        return DeviceType(text.lower())
    except ValueError:
        raise ValueError(f"Unknown device type: {text}") from None


@dataclass(frozen=True)
class Device:
    """``"cuda:0"``-style device name split into (type, index)."""

    type: DeviceType = DeviceType.CPU
    index: Optional[int] = None

    @classmethod
    def from_str(cls, s: str) -> "Device":
        kind, sep, idx = s.partition(":")
        dev_type = _device_type(kind)
        if not sep:
            return cls(dev_type, None)
        try:
            return cls(dev_type, int(idx))
        except ValueError:
            raise ValueError(f"Invalid index: {idx}") from None

    def as_str(self) -> str:
        return self.type.value if self.index is None else f"{self.type.value}:{self.index}"

    @property
    def is_gpu(self) -> bool:
        return self.type is not DeviceType.CPU


# safetensors dtype tag -> bits per logical element (F4 packs two values per byte)
_TAG_BITS = {
    "BOOL": 8, "I8": 8, "U8": 8, "F8_E5M2": 8, "F8_E4M3": 8, "F8_E8M0": 8, "F4": 4,
    "I16": 16, "U16": 16, "F16": 16, "BF16": 16,
    "I32": 32, "U32": 32, "F32": 32,
    "I64": 64, "U64": 64, "F64": 64,
}

# One member per tag, valued by the tag itself (``DType("BF16") is DType.BF16``), plus AUTO
# for "as stored in the file".  Same names as ``st_types.py:45-63`` of the reference.
DType = Enum("DType", {tag: tag for tag in (*_TAG_BITS, "AUTO")}, module=__name__)
DType.__doc__ = "Element type tag of a safetensors header; AUTO means: as stored."

_DTYPE_BITS = {DType(tag): bits for tag, bits in _TAG_BITS.items()}


def dtype_bits(dtype: DType) -> int:
    """Bits per logical element of ``dtype`` (4 for packed F4)."""
    return _DTYPE_BITS[dtype]


def dtype_size(dtype: DType) -> float:
    """Bytes per logical element, fractional for sub-byte dtypes (0.5 for F4)."""
    return _DTYPE_BITS[dtype] / 8


def dtype_storage_align(dtype: DType) -> int:
    """Byte alignment a tensor of ``dtype`` needs before torch can view it."""
    return max(1, _DTYPE_BITS[dtype] // 8)
