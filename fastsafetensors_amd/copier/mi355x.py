# SPDX-License-Identifier: Apache-2.0
"""The ``"mi355x"`` copier: safetensors file -> one HBM arena per file.

It sits where the reference's ``NoGdsFileCopier`` sits (``copier/nogds.py:15-118``)
and keeps that copier's contract, but hands the work to ``libfstx``:

* ``submit_io`` allocates the arena and enqueues the file's data section on the
  shared read pipeline (O_DIRECT or page-cache reads into a pinned ring,
  asynchronous copies on several HIP streams);
* ``wait_io`` drains the requests, realigns what needs realigning with the
  realign-copy kernel, and returns zero-copy tensor views.

Arena layouts
-------------
``direct`` (default)
    Arena byte ``lead + i`` holds data-section byte ``i``.  The DMA engine
    places bytes at any address for free, so a header whose length is not a
    multiple of 16 costs nothing.  ``lead`` (0..127) is chosen so that as many
    tensor bytes as possible start on a 16-byte boundary (and, among such choices,
    on a 128-byte cache line, which the copy kernels like best); the few tensors that
    still do not are copied to an aligned side buffer by one batched kernel
    launch.
``window``
    The arena holds the 4 KiB-aligned file window that contains the data
    section, header tail included, exactly as an O_DIRECT or GDS read delivers
    it (reference: ``copier/gds.py:61-78``).  When ``header_length % 16 != 0``
    every tensor is then misaligned and the whole section is shifted into a
    fresh aligned arena by the realign-copy kernel -- the job the reference does
    with ``gds_device_buffer.memmove`` through a 1 GiB temporary
    (``copier/gds.py:138-159``).
"""

import os
from typing import Dict, List, Optional, Tuple

from .. import _native
from ..common import SafeTensorsMetadata, TensorFrame
from ..frameworks import FrameworkOpBase, TensorBase
from ..st_types import Device, DeviceType, DType, dtype_bits, dtype_storage_align
from .base import CopierInterface
from .registry import CopierConstructFunc, register_copier_constructor

PTR_ALIGN = 16
LINE_ALIGN = 128  # tensors placed in side buffers start on cache lines: the copy kernels write whole lines then
WINDOW_ALIGN = 4096
LAYOUTS = ("direct", "window")


def _align_up(v: int, a: int) -> int:
    return -(-v // a) * a


def pick_lead(frames, align: int = PTR_ALIGN, line: int = LINE_ALIGN) -> int:
    """Offset 0..line-1 of the data section inside the arena that puts the most tensor
    bytes on an ``align`` boundary and, among those, the most on a ``line`` boundary
    (ties go to the smallest offset).  The first is what callers are promised; the second
    lets the copy kernels run over whole cache lines.  ``frames``: tensor frames, or
    (first byte, bytes) pairs."""
    on_align = [0] * align
    on_line = [0] * line
    for f in frames:
        begin, nbytes = f if isinstance(f, tuple) else (f.data_offsets[0], f.nbytes)
        on_align[-begin % align] += nbytes
        on_line[-begin % line] += nbytes
    return max(range(line), key=lambda lead: (on_align[lead % align], on_line[lead], -lead))


class MI355XFileCopier(CopierInterface):
    def __init__(
        self,
        metadata: SafeTensorsMetadata,
        device: Device,
        reader: _native.Reader,
        framework: FrameworkOpBase,
        read_mode: str = "auto",
        layout: str = "direct",
    ):
        if device.type == DeviceType.CPU:
            raise Exception("MI355XFileCopier: needs a HIP device; device='cpu' is not served")
        if layout not in LAYOUTS:
            raise ValueError(f"MI355XFileCopier: unknown layout {layout!r}, expected one of {LAYOUTS}")
        if read_mode not in _native.READ_MODES:
            raise ValueError(f"MI355XFileCopier: unknown read_mode {read_mode!r}")
        self.metadata = metadata
        self.device = device
        self.reader = reader
        self.framework = framework
        self.layout = layout
        self.file: Optional[int] = reader.open(metadata.src, _native.READ_MODES[read_mode])
        self.reqs: List[int] = []
        self.data_at = 0  # arena offset of data-section byte 0

    # -- submit -------------------------------------------------------------------
    def submit_io(self, use_buf_register: bool, max_copy_block_size: int) -> _native.DeviceBuffer:
        meta = self.metadata
        if self.layout == "window":
            first = meta.header_length - meta.header_length % WINDOW_ALIGN
            self.data_at = meta.header_length - first
        else:
            first = meta.header_length
            self.data_at = pick_lead(meta.tensors.spans())  # from the header's entries: the frames are made during the transfer
        total = meta.size_bytes - first
        lead = self.data_at if self.layout == "direct" else 0
        gbuf = self.framework.alloc_tensor_memory(lead + total, self.device)
        try:
            # The allocator may hand back memory that kernels already queued on the caller's
            # stream still read (a buffer closed a moment ago).  The copy streams are not
            # ordered after that stream by themselves: make them wait for what it holds now
            # (an event, not a device-wide synchronize: other streams of the caller keep running).
            self.reader.order_after(self.framework.current_stream(self.device))
            done = 0
            while done < total:
                length = min(total - done, max_copy_block_size)
                self.reqs.append(
                    self.reader.submit_read(self.file, gbuf, first + done, length, lead + done)
                )
                done += length
        except Exception:
            self._drain()
            self.framework.free_tensor_memory(gbuf, self.device)
            raise
        return gbuf

    def _drain(self) -> List[Tuple[int, Exception]]:
        failed = []
        for req in self.reqs:
            try:
                self.reader.wait_read(req)
            except _native.NativeError as e:
                failed.append((req, e))
        self.reqs = []
        if self.file is not None:
            self.reader.close_file(self.file)
            self.file = None
        return failed

    # -- wait -----------------------------------------------------------------------
    def wait_io(
        self, gbuf: _native.DeviceBuffer, dtype: DType = DType.AUTO, noalign: bool = False
    ) -> Dict[str, TensorBase]:
        meta, fw = self.metadata, self.framework
        if dtype != DType.AUTO and any(f.dtype != dtype for f in meta.tensors.values()):
            return self._converted(gbuf, dtype)

        # Everything that does not need the bytes happens while they are still on their way: where
        # each tensor will live, the side allocations, and the views (hundreds per file -- as long
        # as the transfer of a small file's last tenth).  The kernels follow the wait.
        arena, data_at = gbuf, self.data_at
        shift_from = None
        if self.layout == "window" and not noalign and data_at % PTR_ALIGN and meta.data_length:
            # the whole data section will be shifted onto a 16-byte boundary, out of place
            lead = pick_lead(list(meta.tensors.values()))
            fresh = fw.alloc_side_memory(gbuf, lead + meta.data_length, self.device)
            shift_from = (gbuf.get_base_address() + data_at, fresh.get_base_address() + lead)
            arena, data_at = fresh, lead

        # tensors that still start off-boundary move to an aligned side buffer
        base = arena.get_base_address()
        need = {}
        for name, frame in meta.tensors.items():
            want = dtype_storage_align(frame.dtype) if noalign else PTR_ALIGN
            if frame.nbytes and (base + data_at + frame.data_offsets[0]) % want:
                need[name] = frame
        side = None
        placed: Dict[str, int] = {}
        if need:
            cursor = 0
            for name, frame in need.items():
                placed[name] = cursor
                cursor += _align_up(frame.nbytes, LINE_ALIGN)
            side = fw.alloc_side_memory(gbuf, cursor, self.device)
        in_arena = [(n, data_at + f.data_offsets[0], f) for n, f in meta.tensors.items() if n not in placed]
        views = fw.view_tensors(arena, in_arena, self.device)
        if placed:
            views.update(fw.view_tensors(side, [(n, placed[n], meta.tensors[n]) for n in placed], self.device))
        tensors = {name: views[name] for name in meta.tensors}  # in the file's order

        self._drain_or_raise()
        if shift_from is not None:
            _native.realign_copy(shift_from[1], shift_from[0], meta.data_length, self._stream())
            # the window goes back to the allocator right away: its reuse is ordered after this
            # kernel on the same stream, and by order_after() for the copy streams
            fw.shrink_tensor_memory(gbuf)
        if need:
            _native.realign_copy_batch(
                [
                    (side.get_base_address() + placed[n], base + data_at + f.data_offsets[0], f.nbytes)
                    for n, f in need.items()
                ],
                self._stream(),
            )
        return tensors

    def _drain_or_raise(self) -> None:
        failed = self._drain()
        if failed:
            raise Exception(
                f"wait_io: read failed, file={self.metadata.src}, "
                + ", ".join(f"req {r}: {e}" for r, e in failed)
            )

    def _converted(self, gbuf: _native.DeviceBuffer, dtype: DType) -> Dict[str, TensorBase]:
        """Tensors down-cast to ``dtype`` on the GPU (``common.py:355-375`` does it with
        ``Tensor.to`` + ``copy_`` per tensor): one batched kernel converts every tensor
        that is not of ``dtype`` yet into a fresh arena; when nothing is left in the
        original arena it goes back to the allocator, so the file ends up occupying
        its converted size."""
        meta, fw = self.metadata, self.framework
        want_bits = dtype_bits(dtype)
        src_at = gbuf.get_base_address() + self.data_at
        placed: Dict[str, int] = {}
        cursor = 0
        for name, frame in meta.tensors.items():
            if frame.dtype != dtype and frame.nbytes:
                if want_bits > dtype_bits(frame.dtype):
                    self._drain()  # nothing may still be writing to the arena when the caller frees it
                    raise Exception(
                        f"Online type conversion to larger sizes is not supported ({frame.dtype} -> {dtype})"
                    )
            if frame.dtype != dtype or (src_at + frame.data_offsets[0]) % PTR_ALIGN:
                placed[name] = cursor
                count = frame.nbytes * 8 // dtype_bits(frame.dtype)
                cursor += _align_up(count * (want_bits if frame.dtype != dtype else dtype_bits(frame.dtype)) // 8, LINE_ALIGN)
        side = fw.alloc_side_memory(gbuf, cursor, self.device)
        # A source that is misaligned for its own element type (a header of odd length, or odd
        # byte counts in front of it) is first moved to an aligned scratch slot: neither the
        # conversion kernel nor the framework can read it in place.
        staged: Dict[str, int] = {}
        scratch_bytes = 0
        for name in placed:
            frame = meta.tensors[name]
            if frame.dtype != dtype and frame.nbytes and (src_at + frame.data_offsets[0]) % dtype_storage_align(frame.dtype):
                staged[name] = scratch_bytes
                scratch_bytes += _align_up(frame.nbytes, LINE_ALIGN)
        scratch = fw.alloc_tensor_memory(scratch_bytes, self.device) if staged else None
        try:
            # Everything up to here and the views below need no byte of the file: it all happens
            # while the bytes are still on their way; the kernels follow the wait.
            convert, copy, by_framework = [], [], []
            for name, at in placed.items():
                frame = meta.tensors[name]
                if not frame.nbytes:
                    continue
                src = scratch.get_base_address() + staged[name] if name in staged else src_at + frame.data_offsets[0]
                if frame.dtype == dtype:
                    copy.append((side.get_base_address() + at, src, frame.nbytes))
                elif _native.convert_supported(frame.dtype.value, dtype.value):
                    count = frame.nbytes * 8 // dtype_bits(frame.dtype)
                    convert.append((side.get_base_address() + at, src, count,
                                    _native.ELEM_TYPES[frame.dtype.value], _native.ELEM_TYPES[dtype.value]))
                else:
                    by_framework.append((name, at))
            tensors: Dict[str, TensorBase] = {}
            for name, frame in meta.tensors.items():
                if name in placed:
                    if frame.dtype != dtype:
                        count = frame.nbytes * 8 // dtype_bits(frame.dtype)
                        # a frame of its own for the view: the header model keeps describing the file
                        frame = TensorFrame(dtype, frame.shape, [placed[name], placed[name] + count * want_bits // 8],
                                            frame.strides, frame.offsets, frame.sliced)
                    tensors[name] = fw.view_tensor(side, placed[name], frame, self.device)
                else:
                    tensors[name] = fw.view_tensor(gbuf, self.data_at + frame.data_offsets[0], frame, self.device)

            self._drain_or_raise()
            if staged:
                _native.realign_copy_batch(
                    [(scratch.get_base_address() + at, src_at + meta.tensors[n].data_offsets[0], meta.tensors[n].nbytes)
                     for n, at in staged.items()],
                    self._stream(),
                )
            _native.convert_batch(convert, self._stream())
            _native.realign_copy_batch(copy, self._stream())
            # Pairs the conversion kernel does not cover (integer and bool tensors, fp8 sources)
            # are converted on the GPU by the framework's own copy, as the reference converts
            # every tensor (common.py:355-375).
            for name, at in by_framework:
                frame = meta.tensors[name]
                if name in staged:
                    src_view = fw.view_tensor(scratch, staged[name], frame, self.device)
                else:
                    src_view = fw.view_tensor(gbuf, self.data_at + frame.data_offsets[0], frame, self.device)
                fw.copy_tensor(tensors[name], src_view)
        finally:
            if scratch is not None:
                fw.free_tensor_memory(scratch, self.device)  # reuse is ordered after the kernels above on this stream
        if len(placed) == len(meta.tensors):
            fw.shrink_tensor_memory(gbuf)  # nothing lives in the original arena any more
        return tensors

    def _stream(self) -> int:
        return self.framework.current_stream(self.device)

    def __del__(self) -> None:
        try:
            if self.reqs or self.file is not None:
                self._drain()
        except Exception:
            pass


def _default_numa_node(device: Device) -> int:
    from ..common import get_device_numa_node

    node = get_device_numa_node(device.index if device.index is not None else 0)
    return -1 if node is None or node < 0 else node


def _reader_settings(
    device: Device,
    max_threads: int = 16,
    block_size_kb: Optional[int] = None,
    n_streams: int = 0,
    slots_per_thread: int = 0,
    max_direct_reads: int = 0,
    direct_read_kb: Optional[int] = None,
    direct_ramp_kb: Optional[int] = None,
    adaptive_depth: bool = False,
    numa_node: Optional[int] = None,
    shared_reader: bool = True,
    pretouch: bool = True,
) -> Dict[str, int]:
    """Arguments of ``_native.Reader`` from the copier's own, defaults and environment resolved."""
    block_kb = block_size_kb or int(os.environ.get("FSTX_BLOCK_KB", "4096"))
    return dict(
        device_id=device.index if device.index is not None else 0,
        numa_node=numa_node,  # None: looked up from the device (a sysfs read) by whoever builds the reader
        n_threads=max_threads,
        n_streams=n_streams,
        block_bytes=block_kb * 1024,
        slots_per_thread=slots_per_thread,
        max_direct_reads=max_direct_reads,
        direct_read_bytes=(direct_read_kb or int(os.environ.get("FSTX_DIRECT_READ_KB", "0"))) * 1024,
        adaptive_depth=adaptive_depth,
        direct_ramp_kb=direct_ramp_kb if direct_ramp_kb is not None else int(os.environ.get("FSTX_DIRECT_RAMP_KB", "0")),
        shared=shared_reader,
        pretouch=pretouch,
    )


def _build_reader(device: Device, settings: Dict[str, int]) -> _native.Reader:
    if settings["numa_node"] is None:
        settings = dict(settings, numa_node=_default_numa_node(device))
    return _native.Reader(**settings)


def _open_reader(device: Device, **kwargs) -> _native.Reader:
    return _build_reader(device, _reader_settings(device, **kwargs))


def hold_reader(device: str = "cuda:0", max_threads: int = 16, **kwargs) -> _native.Reader:
    """Keep the process-wide read pipeline of this configuration alive until the returned
    handle is closed.

    Loaders created meanwhile with the same settings find its threads, streams and pinned
    ring ready instead of building them again, and, above all, find the ring's pages already
    mapped: the first touch of freshly pinned memory costs about 0.3 ms per MiB, which is
    most of the overhead of loading a file of a few hundred MB.  For processes that load
    many small files one after another (adapters, shards on demand).  ``kwargs`` are the
    copier's own (``block_size_kb``, ``n_streams``, ...).
    """
    import torch

    dev = torch.device(device)
    return _open_reader(Device(DeviceType(dev.type), dev.index), max_threads=max_threads, shared_reader=True, **kwargs)


@register_copier_constructor("mi355x")
def new_mi355x_file_copier(
    device: Device,
    bbuf_size_kb: int = 16 * 1024,
    max_threads: int = 16,
    framework: Optional[FrameworkOpBase] = None,
    read_mode: Optional[str] = None,
    layout: Optional[str] = None,
    block_size_kb: Optional[int] = None,
    n_streams: int = 0,
    slots_per_thread: int = 0,
    max_direct_reads: int = 0,
    direct_read_kb: Optional[int] = None,
    direct_ramp_kb: Optional[int] = None,
    adaptive_depth: bool = False,
    numa_node: Optional[int] = None,
    shared_reader: bool = True,
    pretouch: bool = True,
    **kwargs,
) -> CopierConstructFunc:
    """One read pipeline (threads, pinned ring, streams) shared by every file of a
    loader, as the reference shares one ``nogds_file_reader`` (``copier/nogds.py:107-116``)
    -- and, unless ``shared_reader=False``, by every loader of the process that is alive at
    the same time and asks for the same settings; the last one to close frees it.

    ``bbuf_size_kb`` is accepted for signature compatibility; the ring is sized
    ``max_threads * slots_per_thread * block_size_kb`` instead, because 1 MiB
    slots (the reference's default split) cap the host-to-device link well
    below its peak.
    """
    if device.type == DeviceType.CPU:
        raise Exception("copier 'mi355x' needs a HIP device; device='cpu' is not served")
    if _native.device_count() <= 0:
        raise Exception("[FAIL] no HIP device is visible to libfstx")
    read_mode = read_mode or os.environ.get("FSTX_READ_MODE", "auto")
    layout = layout or os.environ.get("FSTX_LAYOUT", "direct")
    settings = _reader_settings(
        device, max_threads=max_threads, block_size_kb=block_size_kb, n_streams=n_streams,
        slots_per_thread=slots_per_thread, max_direct_reads=max_direct_reads, direct_read_kb=direct_read_kb,
        direct_ramp_kb=direct_ramp_kb, adaptive_depth=adaptive_depth, numa_node=numa_node, shared_reader=shared_reader, pretouch=pretouch,
    )
    # the library builds threads, streams and the ring behind this call's back (a millisecond,
    # during which the caller parses headers, opens files and queues reads)
    reader = _build_reader(device, dict(settings, async_create=True))

    def construct(metadata: SafeTensorsMetadata, device: Device, framework: FrameworkOpBase) -> CopierInterface:
        return MI355XFileCopier(metadata, device, reader, framework, read_mode=read_mode, layout=layout)

    construct.reader = reader  # type: ignore[attr-defined]
    construct.close = reader.close  # type: ignore[attr-defined]
    return construct
