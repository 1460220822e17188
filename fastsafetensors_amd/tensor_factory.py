# SPDX-License-Identifier: Apache-2.0
"""Per-file tensor source (reference: ``fastsafetensors/tensor_factory.py:14-268``).

One ``LazyTensorFactory`` owns the device buffer of one file, the tensor views
over it, and knows how to turn a view into what a rank should see:

``shuffle(pg, name, dim)``
    world of one -> the view itself (``dim`` ignored, as in the reference,
    ``tensor_factory.py:119-122``); ``dim == -1`` -> a private copy (what
    ``broadcast`` leaves on every rank); otherwise the rank's
    ``ceil(S / world)`` block along ``dim``, cut out by the slice-extract
    kernel.  The reference materialises all ``world`` blocks on the owner and
    scatters them (``:162-186``); with a single GPU only the block of
    ``pg.rank()`` is ever produced.
``push(pg, name, dst_rank, src_rank)``
    the truth table of ``tensor_factory.py:58-116`` without the transfer.
"""

from typing import Dict, List, Optional, Tuple

from ._native import DeviceBuffer
from .common import SafeTensorsMetadata, TensorFrame, init_logger, is_debug
from .copier.base import CopierInterface, DummyDeviceBuffer
from .frameworks import FrameworkOpBase, ProcessGroupBase, TensorBase
from .st_types import Device, DType

logger = init_logger(__name__)


class LazyTensorFactory:
    def __init__(
        self,
        metadata: SafeTensorsMetadata,
        device: Device,
        rank: int,
        local_rank: bool,
        factory_idx_bits: int,
        lidx: int,
        copier: Optional[CopierInterface],
        framework: FrameworkOpBase,
        disable_cache: bool = True,
    ):
        self.framework = framework
        self.metadata = metadata
        self.device = device
        self.copier: Optional[CopierInterface] = copier if local_rank else None
        self.tensors: Dict[str, TensorBase] = {}
        self.shuffled: Dict[str, TensorBase] = {}
        self.gbuf: Optional[DeviceBuffer] = None
        self.rank = rank
        self.factory_idx_bits = factory_idx_bits
        self.lidx = lidx
        self.next_tag = 1
        self.disable_cache = disable_cache

    # -- I/O --------------------------------------------------------------------
    def submit_io(self, use_buf_register: bool, max_copy_block_size: int) -> None:
        if self.copier is None:
            return
        self.gbuf = self.copier.submit_io(use_buf_register, max_copy_block_size)
        if self.gbuf:
            logger.debug("submit_io: new buf, addr=0x%x", self.gbuf.get_base_address())

    def wait_io(self, dtype: DType = DType.AUTO, noalign: bool = False) -> None:
        if self.copier is None or self.gbuf is None:
            return
        self.tensors = self.copier.wait_io(self.gbuf, dtype=dtype, noalign=noalign)
        if is_debug(logger):
            for name in self.tensors:
                logger.debug("wait_io: tensor=%s", name)
        self.copier = None

    # -- helpers ------------------------------------------------------------------
    def _held(self, tensor_name: str, who: str) -> TensorBase:
        try:
            return self.tensors[tensor_name]
        except KeyError:
            raise Exception(
                f"{who}: tensor {tensor_name} was not found. released? lidx={self.lidx}"
            ) from None

    # -- point to point -------------------------------------------------------------
    def push(
        self, pg: ProcessGroupBase, tensor_name: str, dst_rank: int, src_rank: int
    ) -> Optional[TensorBase]:
        if pg.size() == 1:
            return self.tensors[tensor_name]
        tag = (self.next_tag << self.factory_idx_bits) + self.lidx
        self.next_tag += 1
        me = pg.rank()
        if me not in (dst_rank, src_rank):
            return None
        if dst_rank == src_rank:  # and me == both
            return self._held(tensor_name, "push").clone().detach()
        frame = self.metadata.tensors[tensor_name]
        if me == src_rank:
            pg.send(self._held(tensor_name, "push").clone().detach(), dst_rank, tag=tag)
            return None
        if not self.tensors:
            self._no_peer("push", tensor_name)
        landing = self.framework.get_empty_tensor(frame.shape, frame.dtype, self.device)
        pg.recv(landing, src_rank, tag=tag)
        return landing

    def _no_peer(self, who: str, tensor_name: str) -> None:
        raise NotImplementedError(
            f"{who}: tensor {tensor_name} belongs to rank {self.rank}, which is not this process; "
            "this loader drives one GPU and has no cross-rank exchange (register the files under "
            "the rank the process group reports)"
        )

    # -- broadcast / scatter ------------------------------------------------------------
    def shuffle(self, pg: ProcessGroupBase, tensor_name: str, dim: int) -> TensorBase:
        if pg.size() == 1:
            return self.tensors[tensor_name]
        if tensor_name in self.shuffled:
            return self.shuffled[tensor_name].clone().detach()
        frame = self.metadata.tensors[tensor_name]
        if dim == -1:
            if self.rank != pg.rank():
                self._no_peer("shuffle", tensor_name)
            out = self._held(tensor_name, "shuffle").clone().detach()
            pg.broadcast(out, self.rank)
        else:
            if self.rank != pg.rank():
                self._no_peer("shuffle", tensor_name)
            out = self.framework.extract_shard(
                self._held(tensor_name, "shuffle"), frame, dim, pg.rank(), pg.size()
            )
            pg.scatter(out, scatter_list=[], src=self.rank)
        if not self.disable_cache:
            self.shuffled[tensor_name] = out
        return out

    def shuffle_many(self, pg: ProcessGroupBase, names_dims: List[Tuple[str, int]]) -> Dict[str, TensorBase]:
        """``shuffle`` for many tensors of this file at once: the copies of all of
        them go to the GPU as batched launches instead of one launch per tensor."""
        if pg.size() == 1:
            return {name: self.tensors[name] for name, _ in names_dims}
        out: Dict[str, TensorBase] = {}
        todo: List[Tuple[str, int]] = []
        for name, dim in names_dims:
            if name in self.shuffled:
                out[name] = self.shuffled[name].clone().detach()
            else:
                if self.rank != pg.rank():
                    self._no_peer("shuffle", name)
                todo.append((name, dim))
        made = self.framework.extract_shards(
            [(self._held(name, "shuffle"), self.metadata.tensors[name], dim) for name, dim in todo],
            pg.rank(), pg.size(),
        )
        for (name, dim), t in zip(todo, made):
            if dim == -1:
                pg.broadcast(t, self.rank)
            else:
                pg.scatter(t, scatter_list=[], src=self.rank)
            if not self.disable_cache:
                self.shuffled[name] = t
            out[name] = t
        return out

    def _joinable(self, tensor_names: List[str], dim: int) -> List[TensorFrame]:
        """Frames of tensors that are to be joined along ``dim``: same number of dimensions, same
        extents everywhere else, and one element type -- the blocks are joined as bytes, and
        bytes of two types side by side are not a tensor (``torch.cat``, which the reference
        joins with, would promote them to a common type instead)."""
        frames = [self.metadata.tensors[name] for name in tensor_names]
        ref = frames[0]
        for name, frame in zip(tensor_names, frames):
            if len(frame.shape) != len(ref.shape):
                raise Exception(f"rank mismatch: tensor {name} has {frame.shape} vs. {ref.shape} (dim={dim})")
            for d, extent in enumerate(frame.shape):
                if d != dim and extent != ref.shape[d]:
                    raise Exception(f"dim {d} mismatch: tensor {name} has {frame.shape} vs. {list(ref.shape)} (dim={dim})")
            if frame.dtype != ref.dtype:
                raise Exception(f"dtype mismatch: tensor {name} is {frame.dtype.value} vs. {ref.dtype.value} of {tensor_names[0]}")
        return frames

    def shuffle_multi_cols(self, pg: ProcessGroupBase, tensor_names: List[str], dim: int) -> TensorBase:
        """The rank's blocks of several tensors joined along ``dim``
        (``tensor_factory.py:194-259``).  The blocks are cut straight into their places in
        the joined tensor by one batched launch (a strided destination when ``dim`` is an
        inner dimension); cutting first and concatenating afterwards remains only for
        tensors that are not in GPU memory."""
        frames = self._joinable(tensor_names, dim)
        held = [self._held(name, "shuffle_multi_cols") for name in tensor_names]
        rank, world = (0, 1) if pg.size() == 1 else (pg.rank(), pg.size())
        joined = self.framework.extract_shards_joined(list(zip(held, frames)), dim, rank, world)
        if joined is not None:
            return joined
        if pg.size() == 1:
            return self.framework.concat_tensors(held, dim=dim)
        pieces = self.framework.extract_shards([(h, f, dim) for h, f in zip(held, frames)], rank, world)
        return self.framework.concat_tensors(pieces, dim=dim)

    def shuffle_multi_cols_many(self, pg: ProcessGroupBase, groups: List[List[str]], dim: int) -> List[TensorBase]:
        """``shuffle_multi_cols`` for many groups of this file at once: one allocation and a
        handful of launches for all of them."""
        items = []
        for names in groups:
            frames = self._joinable(names, dim)
            items.append(list(zip([self._held(n, "shuffle_multi_cols") for n in names], frames)))
        rank, world = (0, 1) if pg.size() == 1 else (pg.rank(), pg.size())
        joined = self.framework.extract_shards_joined_many(items, dim, rank, world)
        if joined is not None:
            return joined
        return [self.shuffle_multi_cols(pg, names, dim) for names in groups]

    # -- release -----------------------------------------------------------------------
    def free_dev_ptrs(self) -> None:
        self.tensors = {}
        self.shuffled = {}
        if self.gbuf is not None and not isinstance(self.gbuf, DummyDeviceBuffer):
            self.framework.free_tensor_memory(self.gbuf, self.device)
            self.gbuf = None
