# SPDX-License-Identifier: Apache-2.0
"""ctypes binding of ``libfstx.so`` (declared in ``include/fstx.h``).

This is the only module that talks to the native library.  It plays the part of
the reference's pybind11 module ``fastsafetensors.cpp`` (``cpp/ext.cpp:973-1065``,
typed in ``cpp.pyi``): a reader object with ``submit_read``/``wait_read``, a
device-buffer handle, and a handful of free functions.  There is no Python or
CPU substitute for anything in here: if the library is missing, loading raises.
"""

import array
import ctypes
import os
import threading
from typing import Any, List, Optional, Sequence, Tuple

_LIB_NAME = "libfstx.so"
_lib: Optional[ctypes.CDLL] = None
_lib_lock = threading.Lock()

FSTX_ABI_VERSION = 4
FSTX_BATCH_MAX = 48
READ_AUTO, READ_BUFFERED, READ_DIRECT = 0, 1, 2
ADAPTIVE_DEPTH = 1
PROBE_NO_COPY, PROBE_NO_READ = 2, 4
NO_PRETOUCH = 8
CREATE_ASYNC = 16
STORAGE_KNOWN, STORAGE_ROTATIONAL, STORAGE_VIRTIO = 1, 2, 4
READ_MODES = {"auto": READ_AUTO, "buffered": READ_BUFFERED, "direct": READ_DIRECT}


class NativeError(RuntimeError):
    """A libfstx call returned a negative status."""

    def __init__(self, what: str, code: int):
        self.code = code
        super().__init__(f"{what}: {strerror(code)} (code {code})")


class FstxConfig(ctypes.Structure):
    _fields_ = [
        ("struct_size", ctypes.c_uint32),
        ("device_id", ctypes.c_int32),
        ("numa_node", ctypes.c_int32),
        ("n_threads", ctypes.c_uint32),
        ("n_streams", ctypes.c_uint32),
        ("block_bytes", ctypes.c_uint64),
        ("slots_per_thread", ctypes.c_uint32),
        ("max_direct_reads", ctypes.c_uint32),
        ("direct_read_bytes", ctypes.c_uint64),
        ("flags", ctypes.c_uint32),
        ("direct_ramp_kb", ctypes.c_uint32),
    ]


_METRICS_SIGNED = ("numa_node", "ring_node", "first_bind_error")


class FstxMetrics(ctypes.Structure):
    _fields_ = [
        (name, ctypes.c_int64 if name in _METRICS_SIGNED else ctypes.c_uint64)
        for name in (
            "struct_size",
            "bounce_buffer_bytes",
            "bytes_read",
            "bytes_copied",
            "blocks_buffered",
            "blocks_direct",
            "read_ns",
            "stage_ns",
            "slot_wait_ns",
            "direct_fallbacks",
            "direct_depth",
            "direct_reads",
            "create_ns",
            "numa_node",
            "workers_on_node",
            "ring_node",
            "bind_errors",
            "first_bind_error",
            "pretouched_bytes",
            "direct_read_bytes",
            "direct_steered",
            "staging_buffers_max",
            "storage_nr_requests",
            "storage_max_sectors_kb",
            "storage_flags",
            "ring_reused",
        )
    ]

    def __init__(self, *args, **kwargs):
        super().__init__(*args, **kwargs)
        if not self.struct_size:
            self.struct_size = ctypes.sizeof(FstxMetrics)


class FstxCopyDesc(ctypes.Structure):
    _fields_ = [("dst", ctypes.c_void_p), ("src", ctypes.c_void_p), ("nbytes", ctypes.c_uint64)]


class FstxSliceDesc(ctypes.Structure):
    _fields_ = [
        ("dst", ctypes.c_void_p),
        ("src", ctypes.c_void_p),
        ("outer", ctypes.c_uint64),
        ("seg_bytes", ctypes.c_uint64),
        ("src_pitch", ctypes.c_uint64),
    ]


class FstxSlice2dDesc(ctypes.Structure):
    _fields_ = [
        ("dst", ctypes.c_void_p),
        ("src", ctypes.c_void_p),
        ("outer", ctypes.c_uint64),
        ("seg_bytes", ctypes.c_uint64),
        ("src_pitch", ctypes.c_uint64),
        ("dst_pitch", ctypes.c_uint64),
    ]


class FstxJoinSrc(ctypes.Structure):
    _fields_ = [("src", ctypes.c_void_p), ("seg_bytes", ctypes.c_uint64), ("src_pitch", ctypes.c_uint64)]


class FstxJoinDesc(ctypes.Structure):
    _fields_ = [
        ("dst", ctypes.c_void_p),
        ("dst_pitch", ctypes.c_uint64),
        ("rows", ctypes.c_uint64),
        ("srcs", ctypes.POINTER(FstxJoinSrc)),
        ("n_srcs", ctypes.c_uint32),
        ("reserved", ctypes.c_uint32),
    ]


class FstxConvertDesc(ctypes.Structure):
    _fields_ = [
        ("dst", ctypes.c_void_p),
        ("src", ctypes.c_void_p),
        ("n_elems", ctypes.c_uint64),
        ("src_type", ctypes.c_uint32),
        ("dst_type", ctypes.c_uint32),
    ]


ELEM_TYPES = {"F64": 0, "F32": 1, "F16": 2, "BF16": 3, "F8_E4M3": 4, "F8_E5M2": 5}
_ELEM_BYTES = {"F64": 8, "F32": 4, "F16": 2, "BF16": 2, "F8_E4M3": 1, "F8_E5M2": 1}


def convert_supported(src: str, dst: str) -> bool:
    """Whether ``fstx_convert_batch`` has a kernel for this pair of safetensors dtype tags:
    from f64 / f32 / f16 / bf16 towards a different float type that is not wider."""
    return (
        src in ELEM_TYPES and dst in ELEM_TYPES and src != dst and not src.startswith("F8")
        and dst != "F64" and _ELEM_BYTES[dst] <= _ELEM_BYTES[src]
    )

# name -> (restype, argtypes); must list every function include/fstx.h declares
_SIGNATURES = {
    "fstx_abi_version": (ctypes.c_int, []),
    "fstx_device_count": (ctypes.c_int, []),
    "fstx_get_alignment_size": (ctypes.c_int, []),
    "fstx_get_device_pci_bus": (ctypes.c_int, [ctypes.c_int, ctypes.c_char_p, ctypes.c_int]),
    "fstx_set_numa_node": (ctypes.c_int, [ctypes.c_int]),
    "fstx_node_cpus": (ctypes.c_int, [ctypes.c_int, ctypes.POINTER(ctypes.c_int), ctypes.c_int]),
    "fstx_set_debug_log": (None, [ctypes.c_int]),
    "fstx_bounce_buffer_bytes": (ctypes.c_uint64, []),
    "fstx_cached_ring_bytes": (ctypes.c_uint64, []),
    "fstx_trim_cache": (ctypes.c_uint64, []),
    "fstx_strerror": (ctypes.c_char_p, [ctypes.c_int64]),
    "fstx_host_alloc": (ctypes.c_void_p, [ctypes.c_uint64]),
    "fstx_host_free": (None, [ctypes.c_void_p]),
    "fstx_ctx_create": (ctypes.c_int, [ctypes.POINTER(FstxConfig), ctypes.POINTER(ctypes.c_void_p)]),
    "fstx_ctx_destroy": (ctypes.c_int, [ctypes.c_void_p]),
    "fstx_ctx_acquire": (ctypes.c_int, [ctypes.POINTER(FstxConfig), ctypes.POINTER(ctypes.c_void_p)]),
    "fstx_ctx_release": (ctypes.c_int, [ctypes.c_void_p]),
    "fstx_ctx_order_after": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p]),
    "fstx_file_open": (ctypes.c_int64, [ctypes.c_void_p, ctypes.c_char_p, ctypes.c_int]),
    "fstx_file_close": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int64]),
    "fstx_submit_read": (
        ctypes.c_int64,
        [ctypes.c_void_p, ctypes.c_int64, ctypes.c_uint64, ctypes.c_uint64, ctypes.c_void_p,
         ctypes.c_uint64, ctypes.c_uint64],
    ),
    "fstx_wait_read": (ctypes.c_int64, [ctypes.c_void_p, ctypes.c_int64]),
    "fstx_get_metrics": (ctypes.c_int, [ctypes.c_void_p, ctypes.POINTER(FstxMetrics)]),
    "fstx_realign_copy": (
        ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint64, ctypes.c_void_p]),
    "fstx_realign_copy_batch": (
        ctypes.c_int, [ctypes.POINTER(FstxCopyDesc), ctypes.c_uint32, ctypes.c_void_p]),
    "fstx_slice_copy": (
        ctypes.c_int,
        [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint64, ctypes.c_uint64, ctypes.c_uint64,
         ctypes.c_void_p],
    ),
    "fstx_slice_copy_batch": (
        ctypes.c_int, [ctypes.POINTER(FstxSliceDesc), ctypes.c_uint32, ctypes.c_void_p]),
    "fstx_slice_copy2d_batch": (
        ctypes.c_int, [ctypes.POINTER(FstxSlice2dDesc), ctypes.c_uint32, ctypes.c_void_p]),
    "fstx_join_copy": (
        ctypes.c_int, [ctypes.c_void_p, ctypes.c_uint64, ctypes.c_uint64, ctypes.POINTER(FstxJoinSrc), ctypes.c_uint32,
                       ctypes.c_void_p]),
    "fstx_join_copy_batch": (
        ctypes.c_int, [ctypes.POINTER(FstxJoinDesc), ctypes.c_uint32, ctypes.c_void_p]),
    "fstx_convert_batch": (
        ctypes.c_int, [ctypes.POINTER(FstxConvertDesc), ctypes.c_uint32, ctypes.c_void_p]),
}

EXPORTED_SYMBOLS = tuple(_SIGNATURES)


def library_path() -> str:
    """``libfstx.so`` next to this file, or the build named by ``FSTX_LIBRARY``."""
    return os.environ.get("FSTX_LIBRARY") or os.path.join(os.path.dirname(os.path.abspath(__file__)), _LIB_NAME)


def lib() -> ctypes.CDLL:
    """The loaded library; raises when it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    with _lib_lock:
        if _lib is None:
            path = library_path()
            if not os.path.exists(path):
                raise ImportError(
                    f"{path} is missing: build it with `python -m fastsafetensors_amd.build_native` "
                    "(needs hipcc); this package has no fallback without its HIP library"
                )
            handle = ctypes.CDLL(path)
            for name, (restype, argtypes) in _SIGNATURES.items():
                fn = getattr(handle, name)
                fn.restype = restype
                fn.argtypes = argtypes
            got = handle.fstx_abi_version()
            if got != FSTX_ABI_VERSION:
                raise ImportError(f"{path}: ABI version {got}, expected {FSTX_ABI_VERSION}")
            _lib = handle
    return _lib


def strerror(code: int) -> str:
    return lib().fstx_strerror(int(code)).decode()


def _check(what: str, code: int) -> int:
    if code < 0:
        raise NativeError(what, code)
    return code


# ---- free functions (names follow the reference's cpp.pyi) ----------------------


def device_count() -> int:
    n = lib().fstx_device_count()
    return max(n, 0)


def is_hip_found() -> bool:
    return device_count() > 0


def get_alignment_size() -> int:
    return lib().fstx_get_alignment_size()


def set_debug_log(enabled: bool) -> None:
    lib().fstx_set_debug_log(1 if enabled else 0)


def get_device_pci_bus(device_id: int) -> str:
    buf = ctypes.create_string_buffer(64)
    if lib().fstx_get_device_pci_bus(int(device_id), buf, len(buf)) < 0:
        return ""
    return buf.value.decode()


def set_numa_node(node: int) -> int:
    return 0 if lib().fstx_set_numa_node(int(node)) >= 0 else -1


def node_cpus(node: int) -> List[int]:
    """CPUs of a NUMA node as the library reads them from sysfs; empty when the node is unknown."""
    buf = (ctypes.c_int * 4096)()
    n = lib().fstx_node_cpus(int(node), buf, len(buf))
    return list(buf[: min(n, len(buf))]) if n > 0 else []


def bounce_buffer_bytes() -> int:
    return int(lib().fstx_bounce_buffer_bytes())


def cached_ring_bytes() -> int:
    """Bytes of the pinned ring the last closed reader left parked for the next one (0: none)."""
    return int(lib().fstx_cached_ring_bytes())


def trim_cache() -> int:
    """Free the parked ring; returns the bytes freed."""
    return int(lib().fstx_trim_cache())


def read_buffer(addr: int, length: int) -> bytes:
    return ctypes.string_at(addr, length)


def cpu_malloc(length: int) -> int:
    return int(lib().fstx_host_alloc(length) or 0)


def cpu_free(addr: int) -> None:
    lib().fstx_host_free(ctypes.c_void_p(addr))


class cpp_metrics:
    """Process-wide counters (``get_cpp_metrics()`` of the reference)."""

    def __init__(self) -> None:
        self.bounce_buffer_bytes = bounce_buffer_bytes()
        self.cached_ring_bytes = cached_ring_bytes()  # the ring a closed reader left for the next one


def get_cpp_metrics() -> cpp_metrics:
    return cpp_metrics()


# ---- device buffer handle ----------------------------------------------------------


class DeviceBuffer:
    """Address range of one file's arena; the ``gds_device_buffer`` of this package.

    ``keepalive`` holds whatever owns the memory (a ``torch.uint8`` tensor), and
    ``extras`` holds side allocations that must live exactly as long (realigned
    copies of tensors whose place in the arena is not 16-byte aligned).
    """

    def __init__(self, base: int, length: int, use_gpu: bool, keepalive: Any = None):
        self._base = int(base)
        self._length = int(length)
        self.use_gpu = bool(use_gpu)
        self.keepalive = keepalive
        self.extras: List[Any] = []

    def get_base_address(self) -> int:
        return self._base

    def get_length(self) -> int:
        return self._length

    def total_length(self) -> int:
        return self._length + sum(e.get_length() for e in self.extras)

    def memmove(self, dst_off: int, src_off: int, tmp: "DeviceBuffer", length: int) -> int:
        """Move ``length`` bytes inside the buffer through ``tmp`` (two kernel copies)."""
        if max(dst_off, src_off) > self._length or tmp.get_length() < length:
            return -1
        if length == 0:
            return 0
        try:
            realign_copy(tmp.get_base_address(), self._base + src_off, length)
            realign_copy(self._base + dst_off, tmp.get_base_address(), length)
        except NativeError:
            return -1
        return 0


# ---- kernels ---------------------------------------------------------------------------


def realign_copy(dst: int, src: int, nbytes: int, stream: int = 0) -> None:
    _check("fstx_realign_copy", lib().fstx_realign_copy(dst, src, nbytes, stream))


def realign_copy_batch(jobs: Sequence[Tuple[int, int, int]], stream: int = 0) -> None:
    """``jobs`` = (dst, src, nbytes) triples; any count (split into launches)."""
    for i in range(0, len(jobs), FSTX_BATCH_MAX):
        part = jobs[i : i + FSTX_BATCH_MAX]
        arr = (FstxCopyDesc * len(part))(*[FstxCopyDesc(d, s, n) for d, s, n in part])
        _check("fstx_realign_copy_batch", lib().fstx_realign_copy_batch(arr, len(part), stream))


def slice_copy(dst: int, src: int, outer: int, seg_bytes: int, src_pitch: int, stream: int = 0) -> None:
    _check("fstx_slice_copy", lib().fstx_slice_copy(dst, src, outer, seg_bytes, src_pitch, stream))


def slice_copy_batch(jobs: Sequence[Tuple[int, int, int, int, int]], stream: int = 0) -> None:
    """``jobs`` = (dst, src, outer, seg_bytes, src_pitch) tuples; any count.

    The descriptors travel as one flat array of 64-bit words (an ``fstx_slice_desc`` is five of
    them), which costs a fraction of building a ctypes structure per job."""
    n = len(jobs)
    if n == 0:
        return
    flat = array.array("Q", [v for job in jobs for v in job])
    base, _ = flat.buffer_info()
    step = 5 * 8
    fn = lib().fstx_slice_copy_batch
    for i in range(0, n, FSTX_BATCH_MAX):
        count = min(FSTX_BATCH_MAX, n - i)
        _check("fstx_slice_copy_batch", fn(ctypes.cast(base + i * step, ctypes.POINTER(FstxSliceDesc)), count, stream))


def slice_copy2d_batch(jobs: Sequence[Tuple[int, int, int, int, int, int]], stream: int = 0) -> None:
    """``jobs`` = (dst, src, outer, seg_bytes, src_pitch, dst_pitch) tuples; any count."""
    for i in range(0, len(jobs), FSTX_BATCH_MAX):
        part = jobs[i : i + FSTX_BATCH_MAX]
        arr = (FstxSlice2dDesc * len(part))(*[FstxSlice2dDesc(*j) for j in part])
        _check("fstx_slice_copy2d_batch", lib().fstx_slice_copy2d_batch(arr, len(part), stream))


FSTX_JOIN_MAX = 24


def join_copy(dst: int, rows: int, srcs: Sequence[Tuple[int, int, int]], stream: int = 0, dst_pitch: int = 0) -> None:
    """Row r of ``dst`` = the r-th segments of ``srcs`` = (src, seg_bytes, src_pitch) side by
    side; rows ``dst_pitch`` bytes apart (0: dense).  Any number of sources."""
    pitch = dst_pitch or sum(s[1] for s in srcs)
    at = dst
    for i in range(0, len(srcs), FSTX_JOIN_MAX):
        part = srcs[i : i + FSTX_JOIN_MAX]
        arr = (FstxJoinSrc * len(part))(*[FstxJoinSrc(*s) for s in part])
        _check("fstx_join_copy", lib().fstx_join_copy(at, pitch, rows, arr, len(part), stream))
        at += sum(s[1] for s in part)


def join_copy_batch(joins: Sequence[Tuple[int, int, Sequence[Tuple[int, int, int]]]], stream: int = 0) -> None:
    """``joins`` = (dst, rows, [(src, seg_bytes, src_pitch), ...]) with dense destinations and at
    most ``FSTX_JOIN_MAX`` sources each; any count, as few launches as the kernel's tables allow."""
    if not joins:
        return
    flat = array.array("Q", [v for _, _, srcs in joins for s in srcs for v in s])
    base, _ = flat.buffer_info()
    descs = (FstxJoinDesc * len(joins))()
    at = 0
    for d, (dst, rows, srcs) in zip(descs, joins):
        d.dst, d.dst_pitch, d.rows, d.n_srcs = dst, 0, rows, len(srcs)
        d.srcs = ctypes.cast(base + at * 24, ctypes.POINTER(FstxJoinSrc))
        at += len(srcs)
    _check("fstx_join_copy_batch", lib().fstx_join_copy_batch(descs, len(joins), stream))


def convert_batch(jobs: Sequence[Tuple[int, int, int, int, int]], stream: int = 0) -> None:
    """``jobs`` = (dst, src, n_elems, src_type, dst_type) tuples; any count."""
    for i in range(0, len(jobs), FSTX_BATCH_MAX):
        part = jobs[i : i + FSTX_BATCH_MAX]
        arr = (FstxConvertDesc * len(part))(*[FstxConvertDesc(*j) for j in part])
        _check("fstx_convert_batch", lib().fstx_convert_batch(arr, len(part), stream))


# ---- reader ------------------------------------------------------------------------------


class Reader:
    """One copy pipeline: worker threads, pinned ring and copy streams.

    ``shared=True`` asks the library for the process-wide context of this configuration
    (``fstx_ctx_acquire``): readers that are alive at the same time then use one set of
    threads, one ring and one set of streams, and the last ``close`` frees them.
    ``probe`` is ``PROBE_NO_COPY`` or ``PROBE_NO_READ`` for a measurement context;
    ``pretouch=False`` keeps the workers from mapping their ring slots ahead of the first request.
    ``async_create=True``: the constructor returns once the settings are checked and the library
    builds threads, streams and ring meanwhile; ``wait_read`` / ``metrics`` wait for that build
    and report its failure.
    """

    def __init__(
        self,
        device_id: int,
        numa_node: int = -1,
        n_threads: int = 0,
        n_streams: int = 0,
        block_bytes: int = 0,
        slots_per_thread: int = 0,
        max_direct_reads: int = 0,
        direct_read_bytes: int = 0,
        adaptive_depth: bool = False,
        direct_ramp_kb: int = 0,
        probe: int = 0,
        shared: bool = False,
        pretouch: bool = True,
        async_create: bool = False,
    ):
        cfg = FstxConfig(
            ctypes.sizeof(FstxConfig), device_id, numa_node, n_threads, n_streams, block_bytes,
            slots_per_thread, max_direct_reads, direct_read_bytes,
            (ADAPTIVE_DEPTH if adaptive_depth else 0) | probe | (0 if pretouch else NO_PRETOUCH)
            | (CREATE_ASYNC if async_create else 0), direct_ramp_kb,
        )
        handle = ctypes.c_void_p()
        self._shared = shared
        if shared:
            _check("fstx_ctx_acquire", lib().fstx_ctx_acquire(ctypes.byref(cfg), ctypes.byref(handle)))
        else:
            _check("fstx_ctx_create", lib().fstx_ctx_create(ctypes.byref(cfg), ctypes.byref(handle)))
        self._ctx: Optional[ctypes.c_void_p] = handle

    def _h(self) -> ctypes.c_void_p:
        if self._ctx is None:
            raise RuntimeError("reader is closed")
        return self._ctx

    def open(self, path: str, mode: int = READ_AUTO) -> int:
        return _check(f"fstx_file_open({path})", lib().fstx_file_open(self._h(), os.fsencode(path), mode))

    def close_file(self, file: int) -> None:
        _check("fstx_file_close", lib().fstx_file_close(self._h(), file))

    def submit_read(self, file: int, dst: DeviceBuffer, offset: int, length: int, ptr_off: int) -> int:
        return _check(
            "fstx_submit_read",
            lib().fstx_submit_read(
                self._h(), file, offset, length, dst.get_base_address(), dst.get_length(), ptr_off
            ),
        )

    def wait_read(self, request: int) -> int:
        return _check("fstx_wait_read", lib().fstx_wait_read(self._h(), request))

    def metrics(self) -> FstxMetrics:
        m = FstxMetrics()
        _check("fstx_get_metrics", lib().fstx_get_metrics(self._h(), ctypes.byref(m)))
        return m

    def order_after(self, stream: int) -> None:
        """Copies of requests submitted from now on start after the work queued on ``stream``."""
        _check("fstx_ctx_order_after", lib().fstx_ctx_order_after(self._h(), stream))

    def close(self) -> None:
        if self._ctx is not None:
            ctx, self._ctx = self._ctx, None
            (lib().fstx_ctx_release if self._shared else lib().fstx_ctx_destroy)(ctx)

    def __del__(self) -> None:
        try:
            self.close()
        except Exception:
            pass
