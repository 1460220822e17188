# SPDX-License-Identifier: Apache-2.0
"""Copier plug-in contract (reference: ``fastsafetensors/copier/base.py:11-30``).

A copier moves the data section of ONE file into ONE device buffer.
``submit_io`` starts the transfer and returns the buffer at once; ``wait_io``
blocks until the bytes are in place and returns ``name -> tensor`` views.
"""

from abc import ABC, abstractmethod
from typing import Dict

from .._native import DeviceBuffer
from ..frameworks import TensorBase
from ..st_types import DType


class CopierInterface(ABC):
    @abstractmethod
    def submit_io(self, use_buf_register: bool, max_copy_block_size: int) -> DeviceBuffer: ...

    @abstractmethod
    def wait_io(
        self, gbuf: DeviceBuffer, dtype: DType = DType.AUTO, noalign: bool = False
    ) -> Dict[str, TensorBase]: ...


class DummyDeviceBuffer(DeviceBuffer):
    """Placeholder for copiers that own no device memory."""

    def __init__(self) -> None:
        super().__init__(0, 0, False)
