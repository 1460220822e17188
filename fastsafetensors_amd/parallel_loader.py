# SPDX-License-Identifier: Apache-2.0
"""``ParallelLoader.iterate_weights``: stream ``(name, tensor)`` pairs while the next
files are still being read.

Public surface of the reference's ``fastsafetensors/parallel_loader.py``
(``PipelineParallel`` ``:126-416``, ``ParallelLoader`` ``:419-505``): files are taken
in batches of ``pg.size()``, a producer thread runs ``add_filenames`` +
``copy_files_to_device`` for batch ``k+1`` while the caller consumes batch ``k``,
each batch's buffers are closed as soon as its last tensor was handed out, and
``queue_size`` bounds how many batches may sit in device memory:

====  =============================================================  ==============
 -1   serial: load, consume, load, ...                                1 batch in HBM
  0   one batch loading while one is being consumed (default)        2 batches
 > 0  the producer may run ``queue_size`` batches ahead              ``queue_size + 1``
====  =============================================================  ==============

In a world of one the tensors of a batch are views of its file buffers, which
are freed when the batch is closed, so every tensor is copied out first
(``parallel_loader.py:183,342-344``).  Here those copies are batched: up to 48
tensors per kernel launch instead of one ``clone()`` each.
"""

import queue
import threading
import time
from typing import Any, Generator, List, Optional, Tuple, Union

from . import _native
from .common import SingleGroup, init_logger
from .file_buffer import FilesBufferOnDevice
from .loader import BaseSafeTensorsFileLoader, SafeTensorsFileLoader

logger = init_logger(__name__)

COPY_CHUNK = _native.FSTX_BATCH_MAX


class FileBatch:
    """One loaded batch of files and how long it took to get there."""

    def __init__(self, fb: FilesBufferOnDevice, keys: List[str], batch_id: int):
        self.fb = fb
        self.keys = keys
        self.batch_id = batch_id
        self.add_filenames_time: Optional[float] = None  # ms
        self.copy_files_time: Optional[float] = None  # ms
        self.load_time: Optional[float] = None  # ms


class PipelineParallel:
    def __init__(
        self,
        pg: Optional[Any],
        loader: BaseSafeTensorsFileLoader,
        hf_weights_files: List[str],
        max_concurrent_producers: int = 1,
        queue_size: int = 0,
        use_tqdm_on_load: bool = True,
        **kwargs,
    ):
        if max_concurrent_producers != 1:
            raise ValueError(
                f"max_concurrent_producers must be 1 (got {max_concurrent_producers}). "
                "Concurrent producers > 1 are not yet supported because broadcast "
                "batches must be processed in strict order across all ranks."
            )
        self.loader = loader
        self.pg = loader.pg if pg is None or isinstance(pg, SingleGroup) else loader.framework.get_process_group(pg)
        self.hf_weights_files = list(hf_weights_files)
        self.max_concurrent_producers = max_concurrent_producers
        self.queue_size = queue_size
        self.use_tqdm_on_load = use_tqdm_on_load
        step = self.pg.size()
        self.weight_files_batches = [
            self.hf_weights_files[i : i + step] for i in range(0, len(self.hf_weights_files), step)
        ]
        if self.pg.size() > 1:
            raise NotImplementedError(
                "iterate_weights over a group larger than one needs a broadcast between ranks; "
                "this loader drives one GPU (use get_sharded / as_dict with a StubProcessGroup instead)"
            )
        # batches that may be resident at once: the one being consumed plus those ahead of it
        self._resident = threading.Semaphore(1 if queue_size < 0 else 2 if queue_size == 0 else queue_size + 1)
        self._ready: "queue.Queue[Union[FileBatch, BaseException, None]]" = queue.Queue()
        self.stop_event = threading.Event()
        self.error_event = threading.Event()
        self.error_info: Optional[str] = None
        # views die with the batch when the world is one process: copy them out
        self.need_clone = self.pg.size() == 1

    # -- producer ---------------------------------------------------------------------
    def _start_batch(self, batch_id: int, files: List[str]) -> Tuple[int, Any, float, float]:
        """Headers, buffers and queued reads of one batch; ``_finish_batch`` waits for them."""
        t0 = time.perf_counter()
        # file i of a batch belongs to rank i; a stub group owns the file of the rank it reports
        self.loader.add_filenames({rank: [f] for rank, f in enumerate(files)})
        t1 = time.perf_counter()
        try:
            pending = self.loader.start_copy()
        finally:
            self.loader.reset()
        return batch_id, pending, t0, t1

    def _finish_batch(self, started: Tuple[int, Any, float, float]) -> FileBatch:
        batch_id, pending, t0, t1 = started
        fb = pending.finish()
        t2 = time.perf_counter()
        batch = FileBatch(fb, list(fb.key_to_rank_lidx.keys()), batch_id)
        batch.add_filenames_time = (t1 - t0) * 1e3
        batch.copy_files_time = (t2 - t1) * 1e3
        batch.load_time = (t2 - t0) * 1e3
        logger.debug("batch %d loaded: %d keys, %.1f ms", batch_id, len(batch.keys), batch.load_time)
        return batch

    def _load_batch(self, batch_id: int, files: List[str]) -> FileBatch:
        return self._finish_batch(self._start_batch(batch_id, files))

    def _acquire_slot(self, patience: Optional[float]) -> bool:
        """A place among the resident batches; gives up after ``patience`` seconds (None: never) or when stopped."""
        if patience is not None and patience <= 0:
            return self._resident.acquire(blocking=False)
        deadline = None if patience is None else time.perf_counter() + patience
        while not self._resident.acquire(timeout=0.005 if patience is not None else 0.05):
            if self.stop_event.is_set() or (deadline is not None and time.perf_counter() >= deadline):
                return False
        if self.stop_event.is_set():
            self._resident.release()
            return False
        return True

    def _producer_worker(self) -> None:
        # The reads of batch k+1 are queued before batch k is waited for whenever a place is free
        # by then (the consumer has usually let go of batch k-1 within a few milliseconds), so the
        # transfer streams on across the batch boundary instead of draining and starting again.
        started: Optional[Tuple[int, Any, float, float]] = None
        try:
            for batch_id, files in enumerate(self.weight_files_batches):
                # (with one resident batch at most there is never a place while a batch is loading)
                ahead_ok = self._acquire_slot(None if started is None else 0.0 if self.queue_size < 0 else 0.02)
                if not ahead_ok and started is not None:
                    # no place yet: hand the loaded batch over first, then wait for one
                    self._ready.put(self._finish_batch(started))
                    started = None
                    ahead_ok = self._acquire_slot(None)
                if not ahead_ok:
                    return
                # the next batch's headers are read while this batch's bytes are on their way
                ahead = None
                if batch_id + 1 < len(self.weight_files_batches):
                    ahead = threading.Thread(target=self.loader.parse_ahead, args=(self.weight_files_batches[batch_id + 1],),
                                             name="fstx-headers", daemon=True)
                    ahead.start()
                try:
                    try:
                        following = self._start_batch(batch_id, files)
                    except BaseException:
                        self._resident.release()
                        if started is not None:
                            # the batch before the failing one is whole: it is handed over first
                            previous, started = started, None
                            self._ready.put(self._finish_batch(previous))
                        raise
                    if started is not None:
                        previous, started = started, following
                        self._ready.put(self._finish_batch(previous))
                    else:
                        started = following
                finally:
                    if ahead is not None:
                        ahead.join()
            if started is not None:
                last, started = started, None
                self._ready.put(self._finish_batch(last))
        except BaseException as e:  # surfaces in the consumer
            if started is not None:
                try:
                    started[1].abandon()
                except Exception:
                    pass
            self.error_info = f"Producer failed: {e}"
            self.error_event.set()
            self._ready.put(e)
            return
        finally:
            if started is not None and self.stop_event.is_set():
                try:
                    started[1].abandon()
                except Exception:
                    pass
        self._ready.put(None)

    # -- consumer ---------------------------------------------------------------------
    def _tensors_of(self, batch: FileBatch) -> Generator[Tuple[str, Any], None, None]:
        fb = batch.fb
        if not self.need_clone:
            for key in batch.keys:
                yield key, fb.get_tensor(key)
            return
        for i in range(0, len(batch.keys), COPY_CHUNK):
            chunk = batch.keys[i : i + COPY_CHUNK]
            views = [fb.get_tensor_wrapped(k) for k in chunk]
            if all(v.get_raw().is_cuda for v in views):
                frames = [fb.rank_loaders[r][l].metadata.tensors[k]
                          for k, (r, l) in ((k, fb.key_to_rank_lidx[k]) for k in chunk)]
                copies = fb.framework.extract_shards([(v, f, -1) for v, f in zip(views, frames)], 0, 1)
            else:
                copies = [v.clone() for v in views]
            for key, t in zip(chunk, copies):
                yield key, t.get_raw()

    def iterate_weights(self) -> Generator[Tuple[str, Any], None, None]:
        """Yield ``(name, tensor)`` for every tensor of every file, files in the given order."""
        producer = threading.Thread(target=self._producer_worker, name="fstx-producer", daemon=True)
        producer.start()
        pending: Optional[FileBatch] = None
        try:
            while True:
                item = self._ready.get()
                if item is None:
                    break
                if isinstance(item, BaseException):
                    raise item
                pending = item
                try:
                    yield from self._tensors_of(item)
                    if item.fb.framework is not None:
                        # the copies out of the batch ran on this thread's stream: they must be done
                        # before the batch's memory goes back to the allocator (the producer thread
                        # allocates from it); other streams of the caller are left alone
                        item.fb.framework.synchronize_stream(self.loader.device)
                finally:
                    item.fb.close()
                    pending = None
                    self._resident.release()
        finally:
            self.stop_event.set()
            producer.join(timeout=30)
            # batches the producer finished after the consumer stopped listening
            while True:
                try:
                    left = self._ready.get_nowait()
                except queue.Empty:
                    break
                if isinstance(left, FileBatch):
                    left.fb.close()
            if pending is not None:
                pending.fb.close()

    def close(self) -> None:
        self.loader.close()


class ParallelLoader(PipelineParallel):
    """``PipelineParallel`` over a ``SafeTensorsFileLoader`` it creates itself.

    Example:
        >>> it = ParallelLoader(None, files, device="cuda:0")
        >>> for name, tensor in it.iterate_weights():
        ...     model_state[name].copy_(tensor)
        >>> it.close()
    """

    def __init__(
        self,
        pg: Optional[Any],
        hf_weights_files: List[str],
        max_concurrent_producers: int = 1,
        queue_size: int = 0,
        use_tqdm_on_load: bool = True,
        device: str = "cpu",
        bbuf_size_kb: int = 16 * 1024,
        max_threads: int = 16,
        nogds: bool = False,
        set_numa: bool = True,
        debug_log: bool = False,
        framework: str = "pytorch",
        **kwargs,
    ):
        loader = SafeTensorsFileLoader(
            pg, device, bbuf_size_kb=bbuf_size_kb, max_threads=max_threads, nogds=nogds, disable_cache=True,
            set_numa=set_numa, debug_log=debug_log, framework=framework, **kwargs,
        )
        super().__init__(pg, loader, hf_weights_files, max_concurrent_producers, queue_size, use_tqdm_on_load)
