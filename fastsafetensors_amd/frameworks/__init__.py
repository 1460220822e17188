# SPDX-License-Identifier: Apache-2.0
"""Framework abstraction of the load path.

Same contract as the reference's ``fastsafetensors/frameworks/__init__.py``:
``TensorBase`` (``:11-62``), ``ProcessGroupBase`` (``:67-105``) and
``FrameworkOpBase`` (``:111-253``).  Only the PyTorch backend exists here; the
two members that are new (``view_tensor`` and ``extract_shard``) are where this
package hands work to its HIP library instead of DLPack capsules and
``Tensor.contiguous()``.
"""

from abc import ABC, abstractmethod
from dataclasses import dataclass
from typing import Dict, Any, List, Optional, Sequence, Tuple

from ..st_types import Device, DType


@dataclass
class TensorBase(ABC):
    device: Device
    dtype: DType

    @abstractmethod
    def get_raw(self) -> Any: ...

    @abstractmethod
    def contiguous(self) -> "TensorBase": ...

    @abstractmethod
    def to(self, device: Optional[Device] = None, dtype: DType = DType.AUTO) -> "TensorBase": ...

    @abstractmethod
    def clone(self) -> "TensorBase": ...

    @abstractmethod
    def detach(self) -> "TensorBase": ...

    @abstractmethod
    def view(self, dtype: DType) -> "TensorBase": ...

    @abstractmethod
    def __getitem__(self, index) -> "TensorBase": ...

    def reshape(self, shape: List[int]) -> "TensorBase":
        raise NotImplementedError(f"{type(self).__name__} does not implement reshape()")

    def data_ptr(self) -> int:
        raise NotImplementedError(f"{type(self).__name__} does not implement data_ptr()")


class ProcessGroupBase(ABC):
    """The six operations the load path needs from a process group."""

    @abstractmethod
    def size(self) -> int: ...

    @abstractmethod
    def rank(self) -> int: ...

    @abstractmethod
    def broadcast(self, dst: TensorBase, rank: int) -> None: ...

    @abstractmethod
    def scatter(self, dst: TensorBase, scatter_list: List[TensorBase], src: int) -> None: ...

    @abstractmethod
    def send(self, t: TensorBase, dst_rank: int, tag: int) -> None: ...

    @abstractmethod
    def recv(self, t: TensorBase, src_rank: int, tag: int) -> None: ...


class FrameworkOpBase(ABC):
    @abstractmethod
    def get_name(self) -> str: ...

    @abstractmethod
    def get_device(self, device: str, pg: ProcessGroupBase) -> Device: ...

    @abstractmethod
    def set_device(self, device: Device) -> None: ...

    @abstractmethod
    def alloc_tensor_memory(self, length: int, dev: Device) -> Any: ...

    @abstractmethod
    def free_tensor_memory(self, gbuf: Any, dev: Device) -> None: ...

    @abstractmethod
    def get_empty_tensor(self, shape: List[int], dtype: DType, device: Device) -> TensorBase: ...

    @abstractmethod
    def concat_tensors(self, tensors: List[TensorBase], dim: int) -> TensorBase: ...

    @abstractmethod
    def copy_tensor(self, dst: TensorBase, src: TensorBase) -> None: ...

    @abstractmethod
    def get_dtype_size(self, dtype: DType) -> float: ...

    @abstractmethod
    def get_cuda_ver(self) -> str: ...

    @abstractmethod
    def get_device_ptr_align(self) -> int: ...

    @abstractmethod
    def as_workaround_dtype(self, dtype: DType) -> DType: ...

    @abstractmethod
    def view_tensor(self, gbuf: Any, byte_offset: int, frame: Any, device: Device) -> TensorBase:
        """Zero-copy tensor over ``gbuf[byte_offset : byte_offset + frame.nbytes]``."""

    def view_tensors(self, gbuf: Any, items: Any, device: Device) -> Dict[str, TensorBase]:
        """``view_tensor`` for many ``(name, byte_offset, frame)`` over one buffer; a framework may do
        it with less work per tensor."""
        return {name: self.view_tensor(gbuf, off, frame, device) for name, off, frame in items}

    @abstractmethod
    def extract_shard(
        self, src: TensorBase, frame: Any, dim: int, rank: int, world: int
    ) -> TensorBase:
        """Dense copy of rank ``rank``'s ``ceil(S/world)`` block of ``src`` along ``dim``."""

    def extract_shards(self, items: List[Tuple[TensorBase, Any, int]], rank: int, world: int) -> List[TensorBase]:
        """Many ``extract_shard`` calls at once; ``dim == -1`` means a copy of the whole tensor."""
        return [
            src.clone().detach() if dim == -1 else self.extract_shard(src, frame, dim, rank, world)
            for src, frame, dim in items
        ]

    def extract_shards_joined(
        self, items: List[Tuple[TensorBase, Any]], dim: int, rank: int, world: int
    ) -> Optional[TensorBase]:
        """The rank's blocks of several tensors, written side by side along ``dim`` into one new
        tensor by a single batched copy; ``None`` when the backend cannot place them directly."""
        return None

    def extract_shards_joined_many(
        self, groups: List[List[Tuple[TensorBase, Any]]], dim: int, rank: int, world: int
    ) -> Optional[List[TensorBase]]:
        """``extract_shards_joined`` for many groups with batched copies; ``None`` when unsupported."""
        return None

    def get_storage_shape(
        self, dtype: DType, shape: List[int], strides: List[int]
    ) -> Tuple[List[int], List[int]]:
        return shape, strides

    def get_native_shape(self, dtype: DType, st_shape: List[int]) -> List[int]:
        return st_shape

    def get_native_slices(self, dtype: DType, st_shape: Sequence[int], slices: Tuple) -> Tuple:
        return slices

    def synchronize(self, device: Device) -> None:
        return None

    def current_stream(self, device: Device) -> int:
        """Handle of the stream the calling thread's GPU work goes to (0: the null stream)."""
        return 0

    def synchronize_stream(self, device: Device) -> None:
        """Wait for the work queued on the calling thread's stream only."""
        return None

    def get_global_rank(self) -> int:
        return 0

    def get_device_name(self, index: int) -> str:
        return ""

    @abstractmethod
    def get_process_group(self, pg: Optional[Any]) -> ProcessGroupBase: ...

    @abstractmethod
    def is_equal(self, wrapped: TensorBase, real: Any) -> bool: ...

    @abstractmethod
    def randn(self, s: tuple, device: Device, dtype: DType) -> TensorBase: ...

    @abstractmethod
    def support_fp8(self) -> bool: ...

    @abstractmethod
    def get_mem_used(self) -> int: ...


def get_framework_op(name: str) -> FrameworkOpBase:
    if name in ("pt", "pytorch", "torch"):
        from ._torch import get_framework_op as make

        return make()
    raise Exception(f"Unknown framework name: {name}")
