# SPDX-License-Identifier: Apache-2.0
"""MI355X-native safetensors load path with the fastsafetensors loader API."""

__version__ = "0.1.0"

from ._native import trim_cache as release_cached_memory
from .copier.mi355x import hold_reader
from .common import SafeTensorsMetadata, SingleGroup, TensorFrame, get_device_numa_node
from .file_buffer import FilesBufferOnDevice
from .frameworks._torch import StubProcessGroup
from .loader import BaseSafeTensorsFileLoader, SafeTensorsFileLoader, fastsafe_open
from .parallel_loader import ParallelLoader, PipelineParallel
from .st_types import Device, DeviceType, DType

__all__ = [
    "BaseSafeTensorsFileLoader",
    "Device",
    "DeviceType",
    "DType",
    "FilesBufferOnDevice",
    "ParallelLoader",
    "PipelineParallel",
    "SafeTensorsFileLoader",
    "SafeTensorsMetadata",
    "SingleGroup",
    "StubProcessGroup",
    "TensorFrame",
    "fastsafe_open",
    "get_device_numa_node",
    "hold_reader",
    "release_cached_memory",
]
