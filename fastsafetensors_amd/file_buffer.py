# SPDX-License-Identifier: Apache-2.0
"""``FilesBufferOnDevice``: name -> tensor access over the loaded files.

Public surface and bookkeeping follow the reference's
``fastsafetensors/file_buffer.py:14-259``: a key -> (rank, file index) map that
rejects duplicate keys (``:47-56``), ``get_tensor`` = ``get_sharded(dim=-1)``
(``:140-167``), automatic release of a file's buffer once each of its keys was
requested when the group is larger than one (``:86-106``), and ``close``
(``:60-69``).  Tensors handed out alias the file buffers and die with them.

``as_dict`` differs in how it gets there: the shards of all requested tensors
of a file are cut by ONE batched kernel launch instead of one strided copy per
tensor.
"""

from collections import OrderedDict
from typing import Any, Dict, List, Optional, Tuple

from .common import init_logger
from .frameworks import FrameworkOpBase, ProcessGroupBase, TensorBase
from .st_types import Device, DType
from .tensor_factory import LazyTensorFactory

logger = init_logger(__name__)


class FilesBufferOnDevice:
    def __init__(
        self,
        rank_loaders: Dict[int, List[LazyTensorFactory]],
        pg: ProcessGroupBase,
        framework: FrameworkOpBase,
        auto_mem_delete: bool = True,
    ):
        self.framework = framework
        self.pg = pg
        self.rank_loaders = rank_loaders
        self.key_to_rank_lidx: Dict[str, Tuple[int, int]] = {}
        self.instantiated: Dict[int, Dict[int, Dict[str, bool]]] = {}
        for rank, factories in rank_loaders.items():
            self.instantiated[rank] = {}
            for lidx, factory in enumerate(factories):
                self.instantiated[rank][lidx] = {}
                for key in factory.metadata.tensors.keys():  # (names only: no frame is made for this)
                    if key in self.key_to_rank_lidx:
                        raise Exception(f"FilesBufferOnDevice: key {key} must be unique among files")
                    self.key_to_rank_lidx[key] = (rank, lidx)
        self.auto_mem_delete = auto_mem_delete and pg.size() > 1

    # -- lifetime -----------------------------------------------------------------
    def close(self) -> None:
        """Free every file buffer; tensors obtained from this object dangle afterwards.

        The memory goes back to the framework's allocator at once.  Work that still reads those
        tensors must be finished by then, or be queued on the stream that is current on the thread
        that loads next: the next load orders its copies after that stream only, not after the
        whole device."""
        for factories in self.rank_loaders.values():
            for factory in factories:
                factory.free_dev_ptrs()
        self.rank_loaders = {}

    def _mark_used(self, rank: int, lidx: int, tensor_name: str) -> None:
        """Count the key as delivered; free its file once all keys were."""
        if not self.auto_mem_delete:
            return
        seen = self.instantiated[rank][lidx]
        seen[tensor_name] = True
        factory = self.rank_loaders[rank][lidx]
        if len(seen) == len(factory.metadata.tensors):
            logger.debug("free_dev_ptrs: rank=%d, lidx=%d, src=%s", rank, lidx, factory.metadata.src)
            factory.free_dev_ptrs()

    # -- lookups --------------------------------------------------------------------
    def _get_rank_lidx(self, tensor_name: str) -> Tuple[int, int]:
        try:
            return self.key_to_rank_lidx[tensor_name]
        except KeyError:
            raise ValueError(f"_get_rank: key {tensor_name} was not found in files") from None

    def _factory(self, tensor_name: str) -> Tuple[int, int, LazyTensorFactory]:
        rank, lidx = self._get_rank_lidx(tensor_name)
        return rank, lidx, self.rank_loaders[rank][lidx]

    def get_filename(self, tensor_name: str) -> str:
        if tensor_name not in self.key_to_rank_lidx:
            return ""
        return self._factory(tensor_name)[2].metadata.src

    def get_shape(self, tensor_name: str) -> List[int]:
        return self._factory(tensor_name)[2].metadata.tensors[tensor_name].shape

    # -- tensors ----------------------------------------------------------------------
    def _get_tensor(
        self, rank: int, lidx: int, tensor_name: str, ret: TensorBase, device: Optional[Device], dtype: DType
    ) -> TensorBase:
        self._mark_used(rank, lidx, tensor_name)
        return ret.to(device=device, dtype=dtype)

    def get_sharded_wrapped(
        self, tensor_name: str, dim: int, device: Optional[Device] = None, dtype: DType = DType.AUTO
    ) -> TensorBase:
        rank, lidx, factory = self._factory(tensor_name)
        t = factory.shuffle(self.pg, tensor_name, dim)
        return self._get_tensor(rank, lidx, tensor_name, t, device, dtype)

    def get_sharded(
        self, tensor_name: str, dim: int, device: Optional[Device] = None, dtype: DType = DType.AUTO
    ) -> Any:
        """This rank's ``ceil(S / world)`` block of the tensor along ``dim``
        (``dim == -1``: the whole tensor)."""
        return self.get_sharded_wrapped(tensor_name, dim, device, dtype).get_raw()

    def get_tensor_wrapped(
        self, tensor_name: str, device: Optional[Device] = None, dtype: DType = DType.AUTO
    ) -> TensorBase:
        return self.get_sharded_wrapped(tensor_name, -1, device, dtype)

    def get_tensor(
        self, tensor_name: str, device: Optional[Device] = None, dtype: DType = DType.AUTO
    ) -> Any:
        """The whole tensor; in a world of one, a zero-copy view of the file buffer."""
        return self.get_tensor_wrapped(tensor_name, device, dtype).get_raw()

    def push_tensor(
        self, tensor_name: str, dst_rank: int, device: Optional[Device] = None, dtype: DType = DType.AUTO
    ) -> Optional[Any]:
        rank, lidx, factory = self._factory(tensor_name)
        t = factory.push(self.pg, tensor_name, dst_rank, rank)
        if t is None:
            return None
        return self._get_tensor(rank, lidx, tensor_name, t, device, dtype).get_raw()

    def get_multi_cols(
        self, tensor_names: List[str], dim: int, device: Optional[Device] = None, dtype: DType = DType.AUTO
    ) -> TensorBase:
        """This rank's blocks of ``tensor_names`` joined along ``dim``."""
        by_file: Dict[Tuple[int, int], List[str]] = {}
        for name in tensor_names:
            by_file.setdefault(self._get_rank_lidx(name), []).append(name)
        parts = [
            self.rank_loaders[rank][lidx].shuffle_multi_cols(self.pg, names, dim)
            for (rank, lidx), names in sorted(by_file.items())
        ]
        out = parts[0] if len(parts) == 1 else self.framework.concat_tensors(parts, dim=dim)
        for name in tensor_names:
            self._mark_used(*self._get_rank_lidx(name), name)
        return out.to(device=device, dtype=dtype)

    def get_multi_cols_many(
        self, groups: List[List[str]], dim: int, device: Optional[Device] = None, dtype: DType = DType.AUTO
    ) -> List[TensorBase]:
        """``get_multi_cols`` for many groups in one call -- the q/k/v and gate/up packing of every
        layer, say -- with the copies of all groups batched into a few launches and the results
        in one allocation per file.  (The reference has one call per group,
        ``file_buffer.py:193-236``; the result of each group is the same.)  The results of one call
        are views into one allocation per element type and file: the memory of all of them stays
        allocated until the last of them is dropped."""
        outs: List[Optional[TensorBase]] = [None] * len(groups)
        by_file: Dict[Tuple[int, int], List[int]] = {}
        for i, names in enumerate(groups):
            where = {self._get_rank_lidx(n) for n in names}
            if len(where) == 1:
                by_file.setdefault(next(iter(where)), []).append(i)
            else:  # a group that spans files: the one-group path joins the parts
                outs[i] = self.get_multi_cols(names, dim, device, dtype)
        for (rank, lidx), idx in sorted(by_file.items()):
            made = self.rank_loaders[rank][lidx].shuffle_multi_cols_many(self.pg, [groups[i] for i in idx], dim)
            for i, t in zip(idx, made):
                outs[i] = t.to(device=device, dtype=dtype)
        for i in (i for idx in by_file.values() for i in idx):
            for name in groups[i]:
                self._mark_used(*self._get_rank_lidx(name), name)
        return outs  # type: ignore[return-value]

    def as_dict(self, tensor_shard_dim: "OrderedDict[str, int]") -> Dict[str, TensorBase]:
        """``{name: dim}`` -> ``{name: tensor}`` with the rule of ``get_sharded``.  The blocks cut for
        consecutive names of one file are views into one allocation per element type: their memory
        stays allocated until the last of them is dropped (the reference allocates each block on its own)."""
        out: Dict[str, TensorBase] = {}
        run: List[Tuple[str, int]] = []  # consecutive names that live in the same file
        run_of: Optional[Tuple[int, int]] = None

        def flush() -> None:
            if not run:
                return
            rank, lidx = run_of
            out.update(self.rank_loaders[rank][lidx].shuffle_many(self.pg, run))
            for name, _ in run:
                self._mark_used(rank, lidx, name)
            run.clear()

        for name, dim in tensor_shard_dim.items():
            where = self._get_rank_lidx(name)
            if where != run_of:
                flush()
                run_of = where
            run.append((name, dim))
        flush()
        return {name: out[name] for name in tensor_shard_dim}
