# SPDX-License-Identifier: Apache-2.0
"""``SafeTensorsFileLoader`` and ``fastsafe_open`` for one MI355X.

Same public surface as the reference's ``fastsafetensors/loader.py``:
``BaseSafeTensorsFileLoader`` (``:28-168``), ``SafeTensorsFileLoader``
(``:171-245``) and ``fastsafe_open`` (``:248-319``).  Kept on purpose:

* ``add_filenames`` registers files rank by rank in round-robin order, so the
  key order is the interleaved file order (``:97-119``);
* ``copy_files_to_device`` walks files in sorted path order, submits the I/O of
  every file first and only then waits (``:144-167``);
* the constructor signature, including ``bbuf_size_kb``/``max_threads``/``nogds``.

Changed on purpose: the copier is always ``"mi355x"`` (``nogds`` is accepted
and ignored, there is no GDS on ROCm), ``device`` must be a HIP device, and
NUMA placement is per I/O thread inside ``libfstx`` rather than a process-wide
``numa_run_on_node``.
"""

import math
from collections import OrderedDict
from typing import Any, Dict, List, Mapping, Optional, Tuple, Union

from . import _native
from .common import SafeTensorsMetadata, TensorFrame, init_logger
from .copier import CopierConstructFunc, CopierType, create_copier_constructor
from .file_buffer import FilesBufferOnDevice
from .frameworks import TensorBase, get_framework_op
from .st_types import Device, DeviceType, DType
from .tensor_factory import LazyTensorFactory

logger = init_logger(__name__)

DEFAULT_COPIER = "mi355x"


class FramesOfFiles(Mapping):
    """``name -> TensorFrame`` over the files registered with a loader, in registration order.
    Holds each file's own (lazy) mapping and an index of the names; a later file's tensor replaces
    an earlier one of the same name, as ``dict.update`` would."""

    def __init__(self) -> None:
        self._files: List[Mapping] = []
        self._where: Dict[str, int] = {}

    def add(self, frames: Mapping) -> None:
        self._where.update(dict.fromkeys(frames.keys(), len(self._files)))
        self._files.append(frames)

    def __getitem__(self, name: str) -> TensorFrame:
        return self._files[self._where[name]][name]

    def __iter__(self):
        return iter(self._where)

    def __len__(self) -> int:
        return len(self._where)

    def __contains__(self, name: object) -> bool:
        return name in self._where

    def keys(self):
        return self._where.keys()


class BaseSafeTensorsFileLoader:
    """Loader over a named copier backend; see ``SafeTensorsFileLoader`` for the usual entry."""

    @classmethod
    def process_extension_config(cls, ext_config: Mapping[str, Any], **kwargs: Any) -> Dict[str, Any]:
        return dict(ext_config)

    def __init__(
        self,
        pg: Optional[Any],
        device: Device,
        copier_type: CopierType,
        set_numa: bool = True,
        disable_cache: bool = True,
        framework: str = "pytorch",
        **kwargs,
    ):
        self.framework = get_framework_op(framework)
        self.pg = self.framework.get_process_group(pg)
        self.device = device
        self.meta: Dict[str, Tuple[SafeTensorsMetadata, int]] = {}
        self.frames = FramesOfFiles()
        self.disable_cache = disable_cache
        # headers parsed ahead of add_filenames (ParallelLoader reads the next batch's while this one loads)
        self.parsed_ahead: Dict[str, SafeTensorsMetadata] = {}
        if not set_numa:
            kwargs.setdefault("numa_node", -1)
        self.copier_constructor: Optional[CopierConstructFunc] = create_copier_constructor(
            copier_type=copier_type, device=device, framework=self.framework, **kwargs
        )

    def reset(self) -> None:
        self.frames = FramesOfFiles()
        self.meta = {}

    def close(self) -> None:
        self.reset()
        ctor, self.copier_constructor = self.copier_constructor, None
        shut = getattr(ctor, "close", None)
        if shut is not None:
            shut()

    def parse_ahead(self, paths: List[str]) -> None:
        """Read and validate the headers of ``paths`` now, for an ``add_filenames`` that comes later.
        Errors are left for that call to raise."""
        for path in paths:
            try:
                self.parsed_ahead[path] = SafeTensorsMetadata.from_file(path, self.framework)
            except Exception:
                self.parsed_ahead.pop(path, None)

    def get_keys(self) -> List[str]:
        return list(self.frames.keys())

    def get_shape(self, tensor_name: str) -> List[int]:
        return self.frames[tensor_name].shape

    def add_filenames(self, filenames: Dict[int, List[str]]) -> None:
        """Register ``{rank: [paths]}``; headers are parsed here."""
        longest = max((len(paths) for paths in filenames.values()), default=0)
        for turn in range(longest):
            for rank, paths in filenames.items():
                if turn >= len(paths):
                    continue
                path = paths[turn]
                metadata = self.parsed_ahead.pop(path, None) or SafeTensorsMetadata.from_file(path, self.framework)
                self.meta[path] = (metadata, rank)
                self.frames.add(metadata.tensors)
                if rank == self.pg.rank():
                    logger.debug("add_filenames %d: path=%s", len(self.meta), path)

    def copy_files_to_device(
        self,
        dtype: DType = DType.AUTO,
        use_buf_register: bool = True,
        max_copy_block_size: int = 16 * 1024 * 1024 * 1024,
    ) -> FilesBufferOnDevice:
        """Start every file's transfer, wait for all of them, and return the buffers.

        The returned object owns the device memory; tensors taken from it must be
        cloned before its ``close()`` if they are to outlive it.
        """
        return self.start_copy(dtype, use_buf_register, max_copy_block_size).finish()

    def start_copy(
        self,
        dtype: DType = DType.AUTO,
        use_buf_register: bool = True,
        max_copy_block_size: int = 16 * 1024 * 1024 * 1024,
    ) -> "PendingCopy":
        """The first half of ``copy_files_to_device``: allocate the registered files' buffers and queue
        their reads; ``finish()`` of the returned object waits for them.  The loader may be ``reset()``
        and given the next files in between, so that their reads queue up behind these without the
        transfer ever pausing (``ParallelLoader`` does)."""
        if self.copier_constructor is None:
            raise Exception("copy_files_to_device: loader is closed")
        self.framework.set_device(self.device)
        pending = PendingCopy(self, dtype)
        idx_bits = math.ceil(math.log2(len(self.meta) + 1))
        try:
            for lidx, (path, (meta, rank)) in enumerate(sorted(self.meta.items()), start=1):
                local = rank == self.pg.rank()
                copier = self.copier_constructor(meta, self.device, self.framework) if local else None
                factory = LazyTensorFactory(
                    meta, self.device, rank, local, idx_bits, lidx, copier, self.framework,
                    disable_cache=self.disable_cache,
                )
                pending.factories.setdefault(rank, []).append(factory)
                factory.submit_io(use_buf_register, max_copy_block_size)
                if local:
                    pending.mine.append(factory)
        except Exception:
            pending.abandon()
            raise
        return pending


class PendingCopy:
    """Files whose reads are queued (``BaseSafeTensorsFileLoader.start_copy``)."""

    def __init__(self, loader: BaseSafeTensorsFileLoader, dtype: DType):
        self.framework = loader.framework
        self.device = loader.device
        self.pg = loader.pg
        self.dtype = dtype
        self.factories: Dict[int, List[LazyTensorFactory]] = {r: [] for r in range(loader.pg.size())}
        self.mine: List[LazyTensorFactory] = []

    def finish(self) -> FilesBufferOnDevice:
        """Wait for the reads and hand the buffers over."""
        try:
            for factory in self.mine:
                factory.wait_io(dtype=self.dtype, noalign=False)
            # wait_io may have queued realign / convert kernels on this thread's stream: the
            # tensors are complete when this call returns, as after the reference's synchronous copies
            self.framework.synchronize_stream(self.device)
            return FilesBufferOnDevice(self.factories, pg=self.pg, framework=self.framework)
        except Exception:
            self.abandon()
            raise

    def abandon(self) -> None:
        """Leave no arena and no in-flight read behind."""
        mine, self.mine = self.mine, []
        for factory in mine:
            try:
                if factory.copier is not None and hasattr(factory.copier, "_drain"):
                    factory.copier._drain()
            finally:
                factory.free_dev_ptrs()


class SafeTensorsFileLoader(BaseSafeTensorsFileLoader):
    """Load ``.safetensors`` files into one MI355X's HBM.

    Args:
        pg: ``None`` / ``SingleGroup()`` for a world of one, or a
            ``StubProcessGroup(rank, size)`` to obtain rank ``rank``'s shards.
        device: a HIP device such as ``"cuda:0"``.
        bbuf_size_kb: accepted for compatibility (the pinned ring is sized from
            ``max_threads`` and the block size instead).
        max_threads: I/O worker threads.
        nogds: accepted for compatibility; there is one copier.
        kwargs: forwarded to the copier factory (``read_mode``, ``layout``,
            ``block_size_kb``, ``n_streams``, ``slots_per_thread``,
            ``max_direct_reads``, ``direct_read_kb``, ``adaptive_depth``, ``numa_node``).

    Example:
        >>> loader = SafeTensorsFileLoader(SingleGroup(), "cuda:0")
        >>> loader.add_filenames({0: ["model-00001-of-00004.safetensors"]})
        >>> bufs = loader.copy_files_to_device()
        >>> w = bufs.get_tensor(loader.get_keys()[0])
        >>> bufs.close(); loader.close()
    """

    @classmethod
    def process_extension_config(cls, ext_config: Mapping[str, Any], **kwargs: Any) -> Dict[str, Any]:
        out = dict(ext_config)
        out["nogds"] = out.pop("copier_type", "gds") != "gds"
        return out

    def __init__(
        self,
        pg: Optional[Any],
        device: str = "cpu",
        bbuf_size_kb: int = 16 * 1024,
        max_threads: int = 16,
        nogds: bool = False,
        set_numa: bool = True,
        disable_cache: bool = True,
        debug_log: bool = False,
        framework: str = "pytorch",
        **kwargs,
    ):
        fw = get_framework_op(framework)
        dev = fw.get_device(device, fw.get_process_group(pg))
        if dev.type == DeviceType.CPU:
            raise Exception(
                f"SafeTensorsFileLoader: device={device!r}; this build loads into HIP devices only "
                "(pass 'cuda:<n>')"
            )
        _native.set_debug_log(debug_log)
        super().__init__(
            pg, dev, kwargs.pop("copier_type", DEFAULT_COPIER), set_numa, disable_cache, framework,
            bbuf_size_kb=bbuf_size_kb, max_threads=max_threads, **kwargs,
        )


class fastsafe_open:
    """``safe_open``-like context manager over one or more files.

    ``filenames`` may be a path, a list of paths or a ``{rank: [paths]}`` map.
    Tensors are valid only inside the ``with`` block.
    """

    def __init__(
        self,
        filenames: Union[str, List[str], Dict[int, List[str]]],
        framework: str = "pt",
        pg: Optional[Any] = None,
        device: str = "cpu",
        nogds: bool = False,
        debug_log: bool = False,
        max_copy_block_size: int = 16 * 1024 * 1024 * 1024,
        **kwargs,
    ):
        self.fb: Optional[FilesBufferOnDevice] = None
        self.loader = SafeTensorsFileLoader(
            pg, device, nogds=nogds, debug_log=debug_log, framework=framework, **kwargs
        )
        if isinstance(filenames, str):
            file_dict: Dict[int, List[str]] = {0: [filenames]}
        elif isinstance(filenames, dict):
            file_dict = filenames
        else:
            file_dict = {0: list(filenames)}
        try:
            self.loader.add_filenames(file_dict)
            self.fb = self.loader.copy_files_to_device(max_copy_block_size=max_copy_block_size)
        except Exception:
            self.loader.close()
            raise

    def metadata(self) -> Dict[str, Dict[str, str]]:
        return {path: meta.metadata for path, (meta, _) in self.loader.meta.items()}

    def keys(self) -> List[str]:
        return list(self.fb.key_to_rank_lidx.keys())

    def get_tensor_wrapped(self, name: str) -> TensorBase:
        return self.fb.get_tensor_wrapped(name)

    def get_tensor(self, name: str) -> Any:
        return self.get_tensor_wrapped(name).get_raw()

    def __enter__(self) -> "fastsafe_open":
        return self

    def __exit__(self, exc_type, exc_value, tb) -> None:
        if self.fb:
            self.fb.close()
            self.fb = None
        if self.loader:
            self.loader.close()
