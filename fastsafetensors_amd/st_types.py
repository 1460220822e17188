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


class DType(Enum):
    BOOL = "BOOL"
    I8 = "I8"
    I16 = "I16"
    I32 = "I32"
    I64 = "I64"
    U8 = "U8"
    U16 = "U16"
    U32 = "U32"
    U64 = "U64"
    F16 = "F16"
    F32 = "F32"
    F64 = "F64"
    BF16 = "BF16"
    F8_E5M2 = "F8_E5M2"
    F8_E4M3 = "F8_E4M3"
    F8_E8M0 = "F8_E8M0"
    F4 = "F4"
    AUTO = "AUTO"


# bits per logical element; F4 packs two values per byte
_DTYPE_BITS = {
    DType.BOOL: 8,
    DType.I8: 8,
    DType.U8: 8,
    DType.F8_E5M2: 8,
    DType.F8_E4M3: 8,
    DType.F8_E8M0: 8,
    DType.F4: 4,
    DType.I16: 16,
    DType.U16: 16,
    DType.F16: 16,
    DType.BF16: 16,
    DType.I32: 32,
    DType.U32: 32,
    DType.F32: 32,
    DType.I64: 64,
    DType.U64: 64,
    DType.F64: 64,
}


def dtype_bits(dtype: DType) -> int:
    """Bits per logical element of ``dtype`` (4 for packed F4)."""
    return _DTYPE_BITS[dtype]


def dtype_size(dtype: DType) -> float:
    """Bytes per logical element, fractional for sub-byte dtypes (0.5 for F4)."""
    return _DTYPE_BITS[dtype] / 8


def dtype_storage_align(dtype: DType) -> int:
    """Byte alignment a tensor of ``dtype`` needs before torch can view it."""
    return max(1, _DTYPE_BITS[dtype] // 8)
