# SPDX-License-Identifier: Apache-2.0
"""Benchmark of the MI355X safetensors load path.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config C3] [--dir DIR]

A step is one full load of the Llama-3-8B-shaped bf16 checkpoint (config C3:
4 files, 291 tensors, 16,060,522,496 data bytes, synthetic values written by
``fastsafetensors_amd.checkpoints``): loader construction, ``add_filenames``,
``copy_files_to_device`` and a touch of every tensor, ending with a device
synchronize -- the timing points of the reference's own harness
(``perf/fastsafetensors_perf/perf.py:761-800``).  ``value`` is data-section
bytes / wall time of the *cold* steps (page cache dropped per file with
``posix_fadvise(DONTNEED)`` before each step, as ``perf.py:402-412`` does); the
warm figures (files resident in the page cache) are in ``warm``.

The stdout line carries the summary (under 12 KB); every figure of the run goes to
``--detail-out`` (default ``bench_out/bench_detail.json`` next to this file).  On the line:

``roofline``      the slice-extract kernel on HBM-resident Llama-2-13B-shaped
                  tensors (config C4, TP=4, all four ranks in turn), timed with
                  events on the stream the launches go to.  Inside it:
                  ``pipeline`` -- the cold and warm loads next to their ceilings: the same
                  engine with one stage left out (reads only, measured cold around every cold
                  step; ring -> HBM copies only), and ceilings that owe nothing to the engine
                  (the best plain O_DIRECT reader of a sweep of threads x request sizes,
                  torch's pinned copy); ``kernels`` -- the other kernels (realign on config
                  C2's data section, row cuts, joined column cuts, odd shapes and short
                  segments through the gather kernel, fp32 -> bf16) as GB/s and fraction of peak.
``configs``       C1 and C2 (cold, warm, warm with the reader held, C2 in the window layout),
                  C3, C4 (whole load from tmpfs; ``as_dict`` and ``get_multi_cols`` for the four
                  ranks of a TP=4 stub group) and C5 (72.7 GB from tmpfs, whole load and
                  ``iterate_weights``), each next to the copy-only leg of its own requests.
``placement``     NUMA node of the device, the node's CPUs, I/O threads and what the library
                  read back after binding them.
``inputs``        generator device, seed base and SHA-256 (first 16 hex digits; the whole
                  digests are in the log) of the generated files.
``cpu_baseline``  the reference's device="cpu" nogds path on the host cores, cold and
                  warm: its own C++ reader when ``oracle/_ref`` is built, else the C
                  restatement in ``oracle/``.
"""
import argparse
import ctypes
import json
import mmap
import os
import shutil
import sys
import threading
import time
from typing import Dict, List, Tuple

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "fstx_slice_kernel_c4_column_cuts_hbm_traffic.txt")


def measured_traffic() -> dict:
    """HBM bytes one launch of the roofline workload moved according to rocprofv3's FETCH_SIZE /
    WRITE_SIZE counters, as written next to the counter summary under ``profiles/`` when it was
    last refreshed (``key = value`` lines); empty when the file is missing."""
    out = {}
    try:
        with open(TRAFFIC_FILE) as f:
            for line in f:
                if "=" in line and not line.lstrip().startswith("#"):
                    k, v = line.split("=", 1)
                    out[k.strip()] = v.strip()
    except OSError:
        pass
    return out


def log(*a):
    print(*a, file=sys.stderr, flush=True)


# ---- page cache control ---------------------------------------------------------------------

_libc = ctypes.CDLL(None, use_errno=True)
_libc.mincore.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_char_p]


def drop_cache(paths: List[str]) -> None:
    for p in paths:
        fd = os.open(p, os.O_RDONLY)
        try:
            os.fsync(fd)
            os.posix_fadvise(fd, 0, 0, os.POSIX_FADV_DONTNEED)
        finally:
            os.close(fd)


def resident_fraction(paths: List[str]) -> float:
    """Share of the files' pages that sit in the page cache (mincore over a mapping)."""
    import numpy as np

    pages = res = 0
    for p in paths:
        size = os.path.getsize(p)
        if size == 0:
            continue
        with open(p, "rb") as f:
            m = mmap.mmap(f.fileno(), size, prot=mmap.PROT_READ)
            view = np.frombuffer(m, dtype=np.uint8)  # only for the mapping's address
            n = (size + 4095) // 4096
            vec = ctypes.create_string_buffer(n)
            if _libc.mincore(view.ctypes.data, size, vec) == 0:
                res += int((np.frombuffer(vec.raw, dtype=np.uint8) & 1).sum())
                pages += n
            del view
            m.close()
    return res / pages if pages else 0.0


def warm_cache(paths: List[str], threads: int = 16) -> None:
    """Read every file once through the page cache."""
    parallel_read(paths, direct=False, threads=threads, limit=None)


def parallel_read(paths: List[str], direct: bool, threads: int, limit, block: int = 4 << 20,
                  start: int = 0) -> Tuple[int, float]:
    """Read ``paths`` in ascending order (skipping the first ``start`` bytes, up to
    ``limit`` bytes in total) into ordinary memory with ``threads`` preads in flight;
    returns (bytes, seconds).  The measured ceiling of the storage."""
    jobs = []
    total = 0
    for p in paths:
        size = os.path.getsize(p)
        if start >= size:
            start -= size
            continue
        first, start = start - start % block, 0
        for off in range(first, size - size % 4096 if direct else size, block):
            n = min(block, size - off)
            if direct:
                n -= n % 4096
            if n <= 0 or (limit is not None and total + n > limit):
                break
            jobs.append((p, off, n))
            total += n
    fds = {p: os.open(p, os.O_RDONLY | (os.O_DIRECT if direct else 0)) for p in {j[0] for j in jobs}}
    lock = threading.Lock()
    cursor = [0]

    # page-aligned anonymous memory, mapped before the clock starts (a read into pages that do not
    # exist yet spends most of its time creating them)
    bufs = [mmap.mmap(-1, block, flags=mmap.MAP_PRIVATE | mmap.MAP_ANONYMOUS | getattr(mmap, "MAP_POPULATE", 0))
            for _ in range(threads)]

    def work(buf):
        view = memoryview(buf)
        while True:
            with lock:
                i = cursor[0]
                cursor[0] += 1
            if i >= len(jobs):
                break
            p, off, n = jobs[i]
            got = 0
            while got < n:
                c = os.preadv(fds[p], [view[got:n]], off + got)
                if c <= 0:
                    raise IOError(f"short read in {p} at {off + got}")
                got += c
        view.release()

    t0 = time.perf_counter()
    ts = [threading.Thread(target=work, args=(b,)) for b in bufs]
    for t in ts:
        t.start()
    for t in ts:
        t.join()
    dt = time.perf_counter() - t0
    for fd in fds.values():
        os.close(fd)
    for b in bufs:
        b.close()
    return total, dt


def plain_reader_sweep(files: List[str]) -> Dict[str, float]:
    """What the storage gives to plain sequential O_DIRECT readers that know nothing of this
    engine: {1, 2, 4} threads x {64 MiB, 256 MiB, 1 GiB} requests, each point over one file
    of the checkpoint (dropped from the page cache first), the files taking turns."""
    out = {}
    k = 0
    for threads in (1, 2, 4):
        for block in (64 << 20, 256 << 20, 1 << 30):
            path = files[k % len(files)]
            k += 1
            drop_cache([path])
            nb, dt = parallel_read([path], direct=True, threads=threads, limit=None, block=block)
            out[f"{threads}x{block >> 20}MiB"] = nb / 1e9 / dt
    return out


# ---- ceilings -----------------------------------------------------------------------------------


def measure_h2d_peak(gib: int = 4, chunk: int = 16 << 20, streams: int = 2) -> float:
    import torch

    pinned = torch.empty(256 << 20, dtype=torch.uint8, pin_memory=True)
    dst = torch.empty(gib << 30, dtype=torch.uint8, device="cuda:0")
    ss = [torch.cuda.Stream() for _ in range(streams)]
    best = 0.0
    for _ in range(2):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        done = k = 0
        while done < dst.numel():
            src = pinned[(done % (pinned.numel() - chunk)) // 4096 * 4096 :][:chunk]
            with torch.cuda.stream(ss[k % streams]):
                dst[done : done + chunk].copy_(src, non_blocking=True)
            done += chunk
            k += 1
        torch.cuda.synchronize()
        best = max(best, dst.numel() / 1e9 / (time.perf_counter() - t0))
    return best


def engine_leg(files: List[str], probe: str, threads: int, block_kb: int, read_mode: str = "auto",
               held: bool = False) -> Dict[str, float]:
    """One stage of the load engine alone, through the C ABI: the same worker threads, block
    queue, request sizes, ring and streams as a load of ``files`` (every file's data section
    submitted up front, then waited for), with the other stage left out.

    ``read_only``  reads run (O_DIRECT runs on cold files, page-cache reads on warm ones),
                   nothing is copied: the rate the storage gives to this request pattern;
    ``copy_only``  no read: ring slots are copied to HBM as they are: the rate of the
                   ring -> HBM copies with this engine's slots, streams and threads.
    No load can be faster than either leg; their minimum is the pipeline's ceiling.
    ``held``: the engine exists before the clock starts and has run once (its ring's pages are
    mapped), as for a load under ``hold_reader``."""
    import torch

    from fastsafetensors_amd import _native
    from fastsafetensors_amd.common import SafeTensorsMetadata
    from fastsafetensors_amd.frameworks import get_framework_op

    fw = get_framework_op("pytorch")
    metas = [SafeTensorsMetadata.from_file(p, fw) for p in files]
    flag = {"read_only": _native.PROBE_NO_COPY, "copy_only": _native.PROBE_NO_READ}[probe]
    mode = _native.READ_MODES["buffered" if probe == "copy_only" else read_mode]
    sizes = [m.size_bytes - m.header_length for m in metas]
    if probe == "copy_only":
        arenas = [torch.empty(n, dtype=torch.uint8, device="cuda:0") for n in sizes]
    else:  # nothing is written: one small buffer stands in for every destination
        arenas = [torch.empty(4096, dtype=torch.uint8, device="cuda:0")] * len(sizes)
    reader = None

    def one_pass() -> float:
        nonlocal reader
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        if reader is None:
            reader = _native.Reader(0, n_threads=threads, block_bytes=block_kb * 1024, probe=flag, shared=False,
                                    async_create=True)
        handles, reqs = [], []
        for path, meta, arena, n in zip(files, metas, arenas, sizes):
            h = reader.open(path, mode)
            handles.append(h)
            cap = n if probe == "copy_only" else 1 << 62  # read_only: the destination is never touched
            buf = _native.DeviceBuffer(arena.data_ptr(), cap, True)
            reqs.append(reader.submit_read(h, buf, meta.header_length, n, 0))
        for r in reqs:
            reader.wait_read(r)
        took = time.perf_counter() - t0
        for h in handles:
            reader.close_file(h)
        return took

    if held:
        one_pass()
    dt = one_pass()
    m = reader.metrics()
    reader.close()
    del arenas
    return {"GBps": sum(sizes) / 1e9 / dt, "seconds": dt, "pread_s": m.read_ns / 1e9, "direct_reads": int(m.direct_reads),
            "blocks_direct": int(m.blocks_direct), "blocks_buffered": int(m.blocks_buffered)}


# ---- one load = one step ------------------------------------------------------------------------


def checksum(t) -> Tuple[int, int]:
    from fastsafetensors_amd.checkpoints import tensor_checksum

    return tensor_checksum(t)


def run_load(files: List[str], read_mode: str, threads: int, block_kb: int, verify=None, **loader_kw) -> Dict[str, float]:
    import torch

    from fastsafetensors_amd import SafeTensorsFileLoader, SingleGroup

    torch.cuda.synchronize()
    t0 = time.perf_counter()
    loader = SafeTensorsFileLoader(SingleGroup(), "cuda:0", max_threads=threads, read_mode=read_mode,
                                   block_size_kb=block_kb, **loader_kw)
    t_ctor = time.perf_counter()
    loader.add_filenames({0: files})
    t1 = time.perf_counter()
    bufs = loader.copy_files_to_device()
    torch.cuda.synchronize()
    t2 = time.perf_counter()
    nbytes = 0
    tensors = {}
    for key in loader.get_keys():
        t = bufs.get_tensor(key)
        nbytes += t.numel() * t.element_size()
        tensors[key] = t
    torch.cuda.synchronize()
    t3 = time.perf_counter()
    metrics = loader.copier_constructor.reader.metrics()
    out = {"init_s": t1 - t0, "ctor_s": t_ctor - t0, "reader_create_s": metrics.create_ns / 1e9,
           "io_s": t2 - t1, "get_s": t3 - t2, "elapsed_s": t3 - t0, "bytes": nbytes,
           "blocks_direct": int(metrics.blocks_direct), "blocks_buffered": int(metrics.blocks_buffered),
           "direct_depth": int(metrics.direct_depth), "direct_reads": int(metrics.direct_reads),
           # summed over the I/O workers; with one O_DIRECT read in flight at a time,
           # pread_s / io_s is the share of the load during which the disk was busy
           "pread_s": metrics.read_ns / 1e9, "stage_memcpy_s": metrics.stage_ns / 1e9,
           "slot_wait_s": metrics.slot_wait_ns / 1e9}
    if verify is not None:
        bad = [k for k, t in tensors.items() if checksum(t) != verify[k]]
        if bad:
            raise SystemExit(f"bench: loaded bytes differ from the generated ones: {bad[:5]}")
        out["verified_tensors"] = len(tensors)
    tensors.clear()
    bufs.close()
    loader.close()
    return out


def bench_small_checkpoint(key: str, data_dir: str, threads: int, write=None, with_cpu: bool = False) -> dict:
    """Configs C1 (GPT-2-small fp32, 0.5 GB) and C2 (GPT-2-medium fp16, 0.7 GB, header length
    = 2 mod 8) -- the sizes of the reference's published single-file figures
    (docs/amd-perf.md:72-86) -- cold and warm, loader construction to last tensor.  For a file
    this small the fixed costs show: building the reader, and mapping the pages of the freshly
    pinned ring at their first touch -- which only the first load of a process pays, since a closed
    reader leaves its ring parked for the next one (``warm_fresh_ring``: the same with that switched
    off, for loads and legs alike).  ``warm_held_reader`` is the same load while the process
    keeps its reader (``hold_reader``), as a server that loads many small files would.  C2 also
    runs in the window layout, where every tensor goes through the realign kernel."""
    import torch

    from fastsafetensors_amd import checkpoints as ck, hold_reader

    # values from the CPU generator: these two files are the same bytes on any machine
    if write is not None:
        recs, _ = write(key, data_dir, "cpu", True)
    else:
        recs = ck.write_config(ck.configs(1.0)[key], data_dir, device="cpu", sha256=False)
    files = [recs[0]["path"]]
    nbytes = recs[0]["size"] - recs[0]["header_length"]
    out = {"workload": f"{key}: {ck.configs(1.0)[key].title}, {nbytes} data bytes, one file"}

    def best(fn, reps=3):
        runs = [fn() for _ in range(reps)]
        r = min(runs, key=lambda r: r["elapsed_s"])
        return {"seconds": r["elapsed_s"], "GBps": nbytes / 1e9 / r["elapsed_s"], "io_s": r["io_s"], "init_s": r["init_s"],
                "reader_create_s": r["reader_create_s"], "get_s": r["get_s"], "blocks_direct": r["blocks_direct"],
                "direct_reads": r["direct_reads"], "pread_s": r["pread_s"]}

    def cold_load(**kw):
        drop_cache(files)
        return run_load(files, "auto", threads, 4096, None, **kw)

    def leg(probe, cold, reps=3, **kw):
        rates = []
        for _ in range(reps):
            if cold:
                drop_cache(files)
            rates.append(engine_leg(files, probe, threads, 4096, **kw))
        return max(rates, key=lambda r: r["GBps"])

    # cold: loads and read-only legs take turns, five of each, best of each (the disk's rate moves by
    # several per cent between two reads of the same file)
    cold_loads, cold_legs = [], []
    for _ in range(5):
        cold_legs.append(leg("read_only", True, reps=1))
        cold_loads.append(cold_load())
    ro = max(cold_legs, key=lambda r: r["GBps"])
    out["cold"] = best(lambda it=iter(cold_loads): next(it), reps=len(cold_loads))
    out["cold"]["read_only_leg_seconds"] = ro["seconds"]
    out["cold"]["read_only_leg_GBps"] = ro["GBps"]
    out["cold"]["io_over_read_only_leg"] = out["cold"]["io_s"] / ro["seconds"]
    warm_cache(files)
    # warm: loads and legs take turns (the box's link rate drifts by 10-20 % within seconds), best of each
    variants = {"warm": {}}
    if key == "C2":
        variants["warm_window_layout_realign"] = {"layout": "window"}
    loads = {k: [] for k in variants}
    legs = []
    for _ in range(6):
        legs.append(leg("copy_only", False, reps=2))
        for k, kw in variants.items():
            loads[k] += [run_load(files, "auto", threads, 4096, None, **kw) for _ in range(2)]
    co = max(legs, key=lambda r: r["GBps"])
    for k in variants:
        out[k] = best(lambda it=iter(loads[k]): next(it), reps=len(loads[k]))
    # the same with nothing left behind by an earlier load: every reader allocates its pinned ring and
    # maps its pages at their first touch, as the first load of a process does
    from fastsafetensors_amd import release_cached_memory

    parked_before = os.environ.get("FSTX_RING_CACHE")
    os.environ["FSTX_RING_CACHE"] = "0"
    release_cached_memory()
    try:
        fresh_loads, fresh_legs = [], []
        for _ in range(4):
            fresh_legs.append(leg("copy_only", False, reps=2))
            fresh_loads += [run_load(files, "auto", threads, 4096, None) for _ in range(2)]
        co_fresh = max(fresh_legs, key=lambda r: r["GBps"])
        out["warm_fresh_ring"] = best(lambda it=iter(fresh_loads): next(it), reps=len(fresh_loads))
    finally:
        if parked_before is None:
            os.environ.pop("FSTX_RING_CACHE", None)
        else:
            os.environ["FSTX_RING_CACHE"] = parked_before
    hold = hold_reader("cuda:0", max_threads=threads, block_size_kb=4096)
    try:
        run_load(files, "auto", threads, 4096, None)  # maps the ring's pages
        held_loads, held_legs = [], []
        for _ in range(5):
            held_legs.append(leg("copy_only", False, reps=2, held=True))
            held_loads += [run_load(files, "auto", threads, 4096, None) for _ in range(2)]
        co_held = max(held_legs, key=lambda r: r["GBps"])
        out["warm_held_reader"] = best(lambda it=iter(held_loads): next(it), reps=len(held_loads))
    finally:
        hold.close()
    for k in ("warm", "warm_fresh_ring", "warm_held_reader", "warm_window_layout_realign"):
        if k in out:
            # a load under a held reader is compared with the leg of an engine that existed before, too
            ceiling = {"warm_held_reader": co_held, "warm_fresh_ring": co_fresh}.get(k, co)
            out[k]["copy_only_leg_GBps"] = ceiling["GBps"]
            out[k]["frac_of_copy_only_leg"] = out[k]["GBps"] / ceiling["GBps"]
    if with_cpu:
        # the reference's device="cpu" path on the same file, cold and warm
        drop_cache(files)
        cc = cpu_baseline(files, cold=True)
        warm_cache(files)
        cw = cpu_baseline(files)
        out["cpu_reference"] = {"kind": cw["kind"], "cold_GBps": cc["value"], "warm_GBps": cw["value"], "cores": cw["cores"],
                                "defaults_cold_GBps": cc["settings"]["defaults"]["GBps"], "defaults_warm_GBps": cw["settings"]["defaults"]["GBps"]}
    torch.cuda.empty_cache()
    shutil.rmtree(data_dir, ignore_errors=True)
    return out


# ---- tensor-parallel extraction through the loader API ---------------------------------------------------


def bench_tp_extract(files: List[str], world: int, threads: int, block_kb: int) -> dict:
    """``FilesBufferOnDevice.as_dict`` for every rank of a TP=``world`` group in turn
    (a stub group reports rank r of ``world``): wall time from the call to the device
    synchronize after it, inputs resident in HBM.  Checked by putting the ranks'
    blocks side by side and comparing with the whole tensors."""
    import torch
    from collections import OrderedDict

    from fastsafetensors_amd import SafeTensorsFileLoader, SingleGroup, StubProcessGroup
    from fastsafetensors_amd import checkpoints as ck

    whole_loader = SafeTensorsFileLoader(SingleGroup(), "cuda:0", max_threads=threads, block_size_kb=block_kb)
    whole_loader.add_filenames({0: files})
    whole = whole_loader.copy_files_to_device()
    per_rank, secs, moved = [], [], 0
    for rank in range(world):
        loader = SafeTensorsFileLoader(StubProcessGroup(rank, world), "cuda:0", max_threads=threads,
                                       block_size_kb=block_kb)
        loader.add_filenames({rank: files})
        bufs = loader.copy_files_to_device()
        dims = OrderedDict((k, ck.llama_shard_dim(k)) for k in loader.get_keys())
        if rank == 0:
            # untimed: one tensor of each kind (row cut, column cut, copy), so that the kernels' code is
            # loaded before the clock starts (the runtime loads a kernel at its first launch)
            first = {}
            for k, d in dims.items():
                first.setdefault(d, k)
            bufs.as_dict(OrderedDict((k, d) for d, k in first.items()))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        out = bufs.as_dict(dims)
        torch.cuda.synchronize()
        secs.append(time.perf_counter() - t0)
        moved += sum(2 * t.get_raw().numel() * t.get_raw().element_size() for t in out.values())
        per_rank.append({k: t.get_raw() for k, t in out.items()})
        bufs.close()
        loader.close()
    checked = 0
    for key, dim in dims.items():
        full = whole.get_tensor(key)
        got = per_rank[0][key] if dim < 0 else torch.cat([per_rank[r][key] for r in range(world)], dim=dim)
        if got.shape != full.shape or not torch.equal(got.reshape(-1).view(torch.uint8), full.reshape(-1).view(torch.uint8)):
            raise SystemExit(f"bench: TP blocks of {key} do not reassemble to the tensor")
        checked += 1
    whole.close()
    whole_loader.close()
    total = sum(secs)
    return {"workload": f"as_dict of {len(dims)} tensors for each of {world} ranks (rows of q/k/v/gate/up/embed/lm_head, "
                        f"columns of o/down, copies of the rest)",
            "seconds_per_rank": secs, "algorithmic_bytes": moved, "GBps": moved / 1e9 / total,
            "tensors_reassembled_and_compared": checked}


def bench_multi_cols(files: List[str], world: int, threads: int, block_kb: int) -> dict:
    """``get_multi_cols`` (fused slice + join: QKV and gate/up packing) for every layer and
    every rank of a TP=``world`` stub group over the HBM-resident checkpoint.  Checked
    against torch's slicing + cat of the whole tensors."""
    import torch

    from fastsafetensors_amd import SafeTensorsFileLoader, SingleGroup, StubProcessGroup

    whole_loader = SafeTensorsFileLoader(SingleGroup(), "cuda:0", max_threads=threads, block_size_kb=block_kb)
    whole_loader.add_filenames({0: files})
    whole = whole_loader.copy_files_to_device()
    layers = sorted({int(k.split(".")[2]) for k in whole_loader.get_keys() if k.startswith("model.layers.")})
    groups = []
    for i in layers:
        p = f"model.layers.{i}."
        groups.append([p + f"self_attn.{x}_proj.weight" for x in "qkv"])
        groups.append([p + f"mlp.{x}_proj.weight" for x in ("gate", "up")])
    secs, secs_singly, moved, checked = [], [], 0, 0
    for rank in range(world):
        loader = SafeTensorsFileLoader(StubProcessGroup(rank, world), "cuda:0", max_threads=threads,
                                       block_size_kb=block_kb)
        loader.add_filenames({rank: files})
        bufs = loader.copy_files_to_device()
        bufs.auto_mem_delete = False
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        singly = [bufs.get_multi_cols(names, dim=0) for names in groups]  # one call, one launch per group
        torch.cuda.synchronize()
        secs_singly.append(time.perf_counter() - t0)
        del singly
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        outs = bufs.get_multi_cols_many(groups, dim=0)  # one call: a few launches per file
        torch.cuda.synchronize()
        secs.append(time.perf_counter() - t0)
        moved += sum(2 * t.get_raw().numel() * t.get_raw().element_size() for t in outs)
        for names, t in list(zip(groups, outs))[:: max(1, len(groups) // 8)]:
            parts = []
            for n in names:
                full = whole.get_tensor(n)
                block = -(-full.shape[0] // world)
                parts.append(full[rank * block : (rank + 1) * block])
            if not torch.equal(t.get_raw(), torch.cat(parts, dim=0)):
                raise SystemExit(f"bench: get_multi_cols({names}) differs from slicing + cat")
            checked += 1
        del outs
        bufs.close()
        loader.close()
    whole.close()
    whole_loader.close()
    return {"workload": f"get_multi_cols_many of [q,k,v] and [gate,up] (dim 0) for {len(layers)} layers ({len(groups)} groups in one "
                        f"call), each of {world} ranks",
            "groups_per_rank": len(groups), "seconds_per_rank": secs, "algorithmic_bytes": moved,
            "GBps": moved / 1e9 / sum(secs), "joined_tensors_compared": checked,
            "one_call_per_group": {"seconds_per_rank": secs_singly, "GBps": moved / 1e9 / sum(secs_singly)}}


def bench_iterate_weights(files: List[str], threads: int, verify) -> dict:
    """``ParallelLoader.iterate_weights`` over the checkpoint, warm page cache: the next file
    loads while the tensors of the current one are copied out and handed to the caller."""
    import torch

    from fastsafetensors_amd import ParallelLoader

    out = {}
    for check in (False, True):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        it = ParallelLoader(None, files, device="cuda:0", max_threads=threads)
        nbytes = count = 0
        for name, t in it.iterate_weights():
            nbytes += t.numel() * t.element_size()
            count += 1
            if check and checksum(t) != verify[name]:
                raise SystemExit(f"bench: iterate_weights handed out wrong bytes for {name}")
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        it.close()
        if not check:
            out = {"workload": "ParallelLoader.iterate_weights, queue_size=0, every tensor copied out of its file buffer",
                   "tensors": count, "bytes": nbytes, "seconds": dt, "GBps": nbytes / 1e9 / dt}
    out["tensors_checksum_verified"] = count
    return out


# ---- kernels ------------------------------------------------------------------------------------------


def bench_kernels(steps: int, warmup: int) -> Dict[str, dict]:
    """Event-timed launches of the kernels on HBM-resident data, through the C ABI."""
    import torch

    from fastsafetensors_amd import _native
    from fastsafetensors_amd import checkpoints as ck

    dev = torch.device("cuda:0")
    stream = torch.cuda.current_stream().cuda_stream
    out: Dict[str, dict] = {}

    def timed(launches) -> List[float]:
        """Per-launch milliseconds: an event pair around each launch, all enqueued
        back to back on the launch stream so that no launch waits for the host."""
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in launches]
        for (a, b), launch in zip(evs, launches):
            a.record()
            launch()
            b.record()
        torch.cuda.synchronize()
        return [a.elapsed_time(b) for a, b in evs]

    # -- config C4 (Llama-2-13B, TP=4), the tensors of file 1 of 3 resident in HBM, every rank in turn.
    #    Column cuts (o_proj, down_proj: dim 1) are strided gathers -> slice_kernel, one launch of 28
    #    tensors per rank.  Row cuts (q/k/v/gate/up/embed: dim 0) are contiguous spans -> the same
    #    entry point hands them to realign_kernel as plain copies, two launches of <= 48 per rank.
    world = 4
    specs = [s for s in ck.configs(1.0)["C4"].files()[0] if ck.llama_shard_dim(s.name) >= 0]
    g = torch.Generator(device=dev).manual_seed(1)
    srcs = {s.name: torch.randint(-32768, 32767, s.shape, dtype=torch.int16, device=dev, generator=g) for s in specs}
    keep = {}
    launches = {0: [], 1: []}  # cut dim -> [(jobs, algorithmic bytes)]
    for rank in range(world):
        jobs = {0: [], 1: []}
        for s in specs:
            dim = ck.llama_shard_dim(s.name)
            block = -(-s.shape[dim] // world)
            inner = 2 * (s.shape[1] if dim == 0 else 1)
            outer = 1 if dim == 0 else s.shape[0]
            out_shape = list(s.shape)
            out_shape[dim] = block
            dst = torch.empty(out_shape, dtype=torch.int16, device=dev)
            keep[(s.name, rank)] = dst
            jobs[dim].append((dst.data_ptr(), srcs[s.name].data_ptr() + rank * block * inner, outer, block * inner,
                              s.shape[dim] * inner))
        for dim in (0, 1):
            for i in range(0, len(jobs[dim]), _native.FSTX_BATCH_MAX):
                part = jobs[dim][i : i + _native.FSTX_BATCH_MAX]
                launches[dim].append((part, 2 * sum(j[2] * j[3] for j in part)))

    def measure(group, label):
        for _ in range(max(1, warmup)):
            for part, _b in group:
                _native.slice_copy_batch(part, stream)
        times, nbytes, pass_ms = [], [], []
        for _ in range(max(1, steps)):
            times += timed([lambda p=part: _native.slice_copy_batch(p, stream) for part, _b in group])
            nbytes += [b for _p, b in group]
            # the same launches between ONE pair of events: no marker between kernels
            pass_ms += timed([lambda: [_native.slice_copy_batch(p, stream) for p, _b in group]])
        avg_ms = sum(pass_ms) / len(pass_ms) / len(group)
        avg_b = sum(nbytes) / len(nbytes)
        return {"workload": label, "launches_timed": len(pass_ms) * len(group), "avg_launch_ms": avg_ms,
                "bytes_per_launch": avg_b, "achieved_GBps": avg_b / 1e6 / avg_ms,
                "best_GBps": max(b / 1e6 / t for b, t in zip(nbytes, times)),
                "avg_launch_ms_with_event_markers": sum(times) / len(times)}

    n1 = sum(1 for s in specs if ck.llama_shard_dim(s.name) == 1)
    out["slice_extract"] = measure(
        launches[1], f"C4 Llama-2-13B bf16 TP=4, column cuts of file 1 of 3: {n1} tensors (o_proj 2,560-byte segments at "
                     f"pitch 10,240; down_proj 6,912 at 27,648) per launch, one launch per rank (slice_kernel)")
    out["row_block_copy"] = measure(
        launches[0], f"C4 Llama-2-13B bf16 TP=4, row cuts of file 1 of 3: {len(specs) - n1} tensors per rank in "
                     f"{len(launches[0]) // world} launches (contiguous spans, realign_kernel without shift)")
    # column cuts written straight into a joined tensor (strided destination): the down_proj
    # column blocks of every layer of the file side by side, per rank
    downs = [s for s in specs if s.name.endswith("down_proj.weight")]
    rows, cols = downs[0].shape
    blk = -(-cols // world)
    joined = [torch.empty((rows, blk * len(downs)), dtype=torch.int16, device=dev) for _ in range(world)]
    jsrcs = [[(srcs[s.name].data_ptr() + 2 * r * blk, 2 * blk, 2 * cols) for s in downs] for r in range(world)]
    for r in range(world):
        _native.join_copy(joined[r].data_ptr(), rows, jsrcs[r], stream)
    jt = timed([lambda r=r: _native.join_copy(joined[r].data_ptr(), rows, jsrcs[r], stream) for r in range(world)] * max(1, steps))
    jb = 2 * joined[0].numel() * 2
    for r in range(world):
        if not torch.equal(joined[r], torch.cat([srcs[s.name][:, r * blk : (r + 1) * blk] for s in downs], dim=1)):
            raise SystemExit("bench: joined column blocks differ from slicing + cat")
    out["slice_join_columns"] = {
        "workload": f"C4 down_proj [{rows}, {cols}] column blocks of {len(downs)} layers cut into one joined [{rows}, {blk * len(downs)}] "
                    f"tensor per rank (one launch of gather_kernel per rank)",
        "launches_timed": len(jt), "avg_launch_ms": sum(jt) / len(jt), "bytes_per_launch": jb,
        "achieved_GBps": jb / 1e6 / (sum(jt) / len(jt)),
    }
    del joined
    # parity at full size: the four ranks' blocks put side by side give the tensor back
    for s in specs:
        dim = ck.llama_shard_dim(s.name)
        whole = torch.cat([keep[(s.name, r)] for r in range(world)], dim=dim)
        if not torch.equal(whole, srcs[s.name]):
            raise SystemExit(f"bench: shards of {s.name} do not concatenate back to the tensor")
    del srcs, keep, launches
    torch.cuda.empty_cache()

    # -- slice extract on shapes whose rows are not multiples of 16 bytes: the gather kernel
    #    (16-byte loads at the data's own byte address), and, for the record, the small-unit
    #    kernels such shapes were left to before it existed (FSTX_GATHER_MODE=0)
    odd = {}
    # (inputs of 0.5 GB each: larger than the 256 MB memory-side cache, so that repeated launches
    #  are served by HBM)
    for label, shape, tdt, lead in [
            ("bf16 [65536, 4090] cut in 4 along dim 1 (2046-byte segments, 8180-byte pitch)", (65536, 4090), torch.int16, 0),
            ("fp8 [65536, 8190] cut in 4 along dim 1 (2048-byte segments, 8190-byte pitch)", (65536, 8190), torch.uint8, 0),
            ("bf16 [32768, 8188] cut in 4 along dim 1 (4094-byte segments, 16376-byte pitch)", (32768, 8188), torch.int16, 0),
            ("bf16 [32768, 8188] cut in 4 along dim 1 into destinations 6 bytes off a 16-byte boundary", (32768, 8188), torch.int16, 3)]:
        t = torch.randint(0, 100, shape, dtype=tdt, device=dev)
        item = t.element_size()
        block = -(-shape[1] // world)
        widths = [min(block, shape[1] - r * block) for r in range(world)]
        flats = [torch.empty(shape[0] * w + 64, dtype=tdt, device=dev) for w in widths]
        dsts = [f[lead : lead + shape[0] * w].view(shape[0], w) for f, w in zip(flats, widths)]
        jobs = [(dsts[r].data_ptr(), t.data_ptr() + r * block * item, shape[0], widths[r] * item, shape[1] * item)
                for r in range(world)]
        nb = 2 * sum(d.numel() * item for d in dsts)
        res = {}
        for mode, env in (("gather_kernel", "1"), ("small_unit_kernels", "0")):
            os.environ["FSTX_GATHER_MODE"] = env
            _native.slice_copy_batch(jobs, stream)
            ms = timed([lambda: _native.slice_copy_batch(jobs, stream)] * 5)
            res[mode] = {"avg_launch_ms": sum(ms) / len(ms), "achieved_GBps": nb / 1e6 / (sum(ms) / len(ms))}
            if not all(torch.equal(dsts[r], t[:, r * block : (r + 1) * block]) for r in range(world)):
                raise SystemExit(f"bench: odd-shape slice ({mode}) differs from torch's slice")
        os.environ.pop("FSTX_GATHER_MODE")
        odd[label] = dict(res, bytes_per_launch=nb)
        del t, dsts, flats
    out["slice_extract_odd_shapes"] = odd

    # -- get_multi_cols along dim 1 on odd widths: the rank's column blocks of several tensors cut
    #    straight into one joined tensor (one launch per rank; a destination vector that holds the end
    #    of one block and the start of the next is put together in registers)
    odd_joins = {}
    for label, shape, tdt, count in [("6 x fp8 [32768, 8190], column blocks of a rank joined along dim 1", (32768, 8190), torch.uint8, 6),
                                     ("8 x bf16 [16384, 4090], column blocks of a rank joined along dim 1", (16384, 4090), torch.int16, 8)]:
        ts = [torch.randint(0, 100, shape, dtype=tdt, device=dev) for _ in range(count)]
        item = ts[0].element_size()
        block = -(-shape[1] // world)
        widths = [min(block, shape[1] - r * block) for r in range(world)]
        outs = [torch.empty((shape[0], count * w), dtype=tdt, device=dev) for w in widths]
        jsrc = [[(t.data_ptr() + r * block * item, widths[r] * item, shape[1] * item) for t in ts] for r in range(world)]
        nb = 2 * sum(o.numel() * item for o in outs) / world
        res = {}
        for mode, env in (("gather_kernel", "1"), ("small_unit_kernels", "0")):
            os.environ["FSTX_GATHER_MODE"] = env
            for r in range(world):
                _native.join_copy(outs[r].data_ptr(), shape[0], jsrc[r], stream)
            ms = timed([lambda r=r: _native.join_copy(outs[r].data_ptr(), shape[0], jsrc[r], stream) for r in range(world)] * 3)
            res[mode] = {"avg_launch_ms": sum(ms) / len(ms), "achieved_GBps": nb / 1e6 / (sum(ms) / len(ms))}
            for r in range(world):
                if not torch.equal(outs[r], torch.cat([t[:, r * block : (r + 1) * block] for t in ts], dim=1)):
                    raise SystemExit(f"bench: odd join ({mode}) differs from slicing + cat")
        os.environ.pop("FSTX_GATHER_MODE")
        odd_joins[label] = dict(res, bytes_per_launch=nb)
        del ts, outs
    out["join_odd_columns"] = odd_joins

    # -- short segments: tiles that hold many of them (every lane finds its own segment), a narrow
    #    block written into a wide tensor, and the small-unit fallback for segments under 16 bytes
    short = {}

    def row(label, kernel, nb, launch, check, torch_way=None):
        launch()
        ms = timed([launch] * 5)
        if not check():
            raise SystemExit(f"bench: {label}: result differs from torch's slicing")
        short[label] = {"kernel": kernel, "avg_launch_ms": sum(ms) / len(ms), "bytes_per_launch": nb,
                        "achieved_GBps": nb / 1e6 / (sum(ms) / len(ms))}
        if torch_way is not None:
            # the same bytes moved by torch's own strided copy, for scale (one pair of events around the whole of it)
            torch_way()
            tm = timed([torch_way] * 3)
            short[label]["torch_strided_copy_GBps"] = nb / 1e6 / (sum(tm) / len(tm))

    rows_n, width, count = 88064, 1016, 24
    ts = [torch.randint(0, 255, (rows_n, width), dtype=torch.uint8, device=dev) for _ in range(count)]
    blk = width // world
    outs = [torch.empty((rows_n, count * blk), dtype=torch.uint8, device=dev) for _ in range(world)]
    jsrc = [[(t.data_ptr() + r * blk, blk, width) for t in ts] for r in range(world)]
    for r in range(world):
        _native.join_copy(outs[r].data_ptr(), rows_n, jsrc[r], stream)
    ms = timed([lambda r=r: _native.join_copy(outs[r].data_ptr(), rows_n, jsrc[r], stream) for r in range(world)] * 3)
    for r in range(world):
        if not torch.equal(outs[r], torch.cat([t[:, r * blk : (r + 1) * blk] for t in ts], dim=1)):
            raise SystemExit("bench: join of short segments differs from slicing + cat")
    nb = 2 * outs[0].numel()
    short[f"{count} x u8 [{rows_n}, {width}], column blocks of a rank ({blk}-byte segments) joined along dim 1"] = {
        "kernel": "gather_kernel<multi, keep>", "avg_launch_ms": sum(ms) / len(ms), "bytes_per_launch": nb,
        "achieved_GBps": nb / 1e6 / (sum(ms) / len(ms))}
    del outs, jsrc
    t = ts[0]
    del ts
    big = torch.randint(0, 255, (1 << 20, width), dtype=torch.uint8, device=dev)
    dsts = [torch.empty((big.shape[0], blk), dtype=torch.uint8, device=dev) for _ in range(world)]
    jobs = [(dsts[r].data_ptr(), big.data_ptr() + r * blk, big.shape[0], blk, width) for r in range(world)]
    row(f"u8 [{big.shape[0]}, {width}] cut in 4 along dim 1 ({blk}-byte segments), 4 ranks per launch", "gather_kernel<keep>",
        2 * sum(d.numel() for d in dsts), lambda: _native.slice_copy_batch(jobs, stream),
        lambda: all(torch.equal(dsts[r], big[:, r * blk : (r + 1) * blk]) for r in range(world)),
        lambda: [dsts[r].copy_(big[:, r * blk : (r + 1) * blk]) for r in range(world)])
    del dsts
    # a rank's narrow column block written into its columns of a wide tensor: through the gather kernel
    # (vectors counted row by row from each row's own first byte) and, for scale, through the unit kernel
    for seg, pitch, dpitch, n_rows in [(96, 384, 4096, 1 << 20), (94, 377, 4094, 1 << 20), (1024, 4096, 8192, 1 << 18),
                                       (1000, 4000, 8000, 1 << 18)]:
        src = torch.randint(0, 255, (n_rows, pitch), dtype=torch.uint8, device=dev)
        wide = torch.zeros((n_rows, dpitch), dtype=torch.uint8, device=dev)
        job = [(wide.data_ptr() + 128, src.data_ptr() + seg, n_rows, seg, pitch, dpitch)]
        label = f"[{n_rows}, {seg}]-byte block (pitch {pitch}) into columns 128.. of a tensor with {dpitch}-byte rows"
        row(label, "gather_kernel<pitched>, vectors counted row by row", 2 * n_rows * seg, lambda: _native.slice_copy2d_batch(job, stream),
            lambda: torch.equal(wide[:, 128 : 128 + seg], src[:, seg : 2 * seg]) and not wide[:, :128].any() and not wide[:, 128 + seg :].any(),
            lambda: wide[:, 128 : 128 + seg].copy_(src[:, seg : 2 * seg]))
        os.environ["FSTX_GATHER_MODE"] = "0"
        _native.slice_copy2d_batch(job, stream)
        ms = timed([lambda: _native.slice_copy2d_batch(job, stream)] * 5)
        os.environ.pop("FSTX_GATHER_MODE")
        short[label]["slice2d_kernel_GBps"] = 2 * n_rows * seg / 1e6 / (sum(ms) / len(ms))
        del src, wide
    # segments under 16 bytes: bf16 [N, 4] cut in 4 along dim 1, one 2-byte element per row and rank
    thin = torch.randint(-32768, 32767, (1 << 25, 4), dtype=torch.int16, device=dev)
    douts = [torch.empty((thin.shape[0], 1), dtype=torch.int16, device=dev) for _ in range(world)]
    jobs2 = [(douts[r].data_ptr(), thin.data_ptr() + 2 * r, thin.shape[0], 2, 8) for r in range(world)]
    row(f"bf16 [{thin.shape[0]}, 4] cut in 4 along dim 1 (2-byte segments), 4 ranks per launch", "slice2d_kernel, 2-byte units",
        2 * sum(d.numel() * 2 for d in douts), lambda: _native.slice_copy_batch(jobs2, stream),
        lambda: all(torch.equal(douts[r], thin[:, r : r + 1]) for r in range(world)),
        lambda: [douts[r].copy_(thin[:, r : r + 1]) for r in range(world)])
    del thin, douts, big, t
    out["short_segments"] = short
    torch.cuda.empty_cache()

    # -- realign: config C2's data section shifted by header_length % 16 = 10 bytes
    n = 709_646_336
    cal = 1 << 30
    window = torch.randint(0, 255, (cal + 4096,), dtype=torch.uint8, device=dev)
    dst = torch.empty(cal, dtype=torch.uint8, device=dev)
    for _ in range(max(1, warmup)):
        _native.realign_copy(dst.data_ptr(), window.data_ptr() + 10, n, stream)
    times = timed([lambda: _native.realign_copy(dst.data_ptr(), window.data_ptr() + 10, n, stream)] * max(3, steps))
    if not torch.equal(dst[:n], window[10 : 10 + n]):
        raise SystemExit("bench: realign copy result differs from the source bytes")
    # plain copy of known size (source already aligned): the yardstick that the
    # FETCH_SIZE / WRITE_SIZE counters of the other launches are scaled by
    _native.realign_copy(dst.data_ptr(), window.data_ptr(), cal, stream)
    cal_times = timed([lambda: _native.realign_copy(dst.data_ptr(), window.data_ptr(), cal, stream)] * 3)
    out["calibration_copy"] = {
        "workload": f"aligned copy of {cal} bytes (realign_kernel, shift 0, grid {cal // 16} lanes)",
        "launches_timed": len(cal_times), "avg_launch_ms": sum(cal_times) / len(cal_times),
        "bytes_per_launch": 2 * cal, "achieved_GBps": 2 * cal / 1e6 / (sum(cal_times) / len(cal_times)),
    }
    # -- two more yardsticks for the counters, independent of this library's kernels: a kernel
    #    that only reads 1 GiB (torch's sum) and one that only writes 1 GiB (torch's fill_)
    ones = window[:cal].view(torch.int32)
    for _ in range(3):
        ones.sum()
    rd = timed([lambda: ones.sum()] * 3)
    for _ in range(3):
        dst[:cal].view(torch.int32).fill_(7)
    wr = timed([lambda: dst[:cal].view(torch.int32).fill_(7)] * 3)
    out["counter_yardsticks"] = {
        "read_only": {"workload": f"torch.sum over {cal} bytes of int32 (reduce_kernel: reads {cal} bytes, writes a few)",
                      "avg_launch_ms": sum(rd) / len(rd), "bytes_read": cal},
        "write_only": {"workload": f"torch fill_ of {cal} bytes (vectorized_elementwise_kernel FillFunctor<int>: writes {cal} bytes, reads none)",
                       "avg_launch_ms": sum(wr) / len(wr), "bytes_written": cal},
    }
    # -- down-cast on load: fp32 -> bf16 over 1 GiB of fp32 in 48 tensors per launch
    #    (4 bytes read + 2 written per element)
    per = cal // 4 // 48 // 64 * 64  # whole 256-byte spans, so that no cache line is shared between two jobs
    src32 = window[: cal].view(torch.float32)
    dst16 = dst[: cal // 2].view(torch.int16)
    cjobs = [(dst16.data_ptr() + 2 * i * per, src32.data_ptr() + 4 * i * per, per,
              _native.ELEM_TYPES["F32"], _native.ELEM_TYPES["BF16"]) for i in range(48)]
    _native.convert_batch(cjobs, stream)
    conv_times = timed([lambda: _native.convert_batch(cjobs, stream)] * max(3, steps))
    probe = slice(0, 1 << 22)
    if not torch.equal(dst16[probe], src32[probe].to(torch.bfloat16).view(torch.int16)):
        raise SystemExit("bench: converted values differ from torch's Tensor.to(bfloat16)")
    conv_ms = sum(conv_times) / len(conv_times)
    out["convert_f32_bf16"] = {
        "workload": f"fp32 -> bf16, 48 tensors of {per} elements per launch (convert_kernel)",
        "launches_timed": len(conv_times), "avg_launch_ms": conv_ms, "bytes_per_launch": 6 * per * 48,
        "achieved_GBps": 6 * per * 48 / 1e6 / conv_ms,
    }
    # -- the remaining variants of the kernels, one row each: the realign copy with its source, then its
    #    destination, 16 bytes into a cache line; two more conversions; the gather kernel with a pitched
    #    destination (one source: a column block into a slightly wider tensor; several: a join into one)
    variants = {}

    def vrow(label, kernel, nb, launch, check=None):
        launch()
        ms = timed([launch] * max(3, steps))
        if check is not None and not check():
            raise SystemExit(f"bench: {label}: wrong bytes")
        variants[label] = {"kernel": kernel, "avg_launch_ms": sum(ms) / len(ms), "bytes_per_launch": nb,
                           "achieved_GBps": nb / 1e6 / (sum(ms) / len(ms))}

    half = 1 << 29
    vrow("realign copy of 512 MiB, source 16 bytes into a cache line", "realign_kernel", 2 * half,
         lambda: _native.realign_copy(dst.data_ptr(), window.data_ptr() + 16, half, stream),
         lambda: torch.equal(dst[:half], window[16 : 16 + half]))
    vrow("realign copy of 512 MiB, destination 16 bytes into a cache line", "realign_kernel", 2 * half,
         lambda: _native.realign_copy(dst.data_ptr() + 16, window.data_ptr(), half, stream),
         lambda: torch.equal(dst[16 : 16 + half], window[:half]))
    vrow("realign copy of 512 MiB, source shifted by 3 bytes, destination 16 bytes into a cache line", "realign_kernel", 2 * half,
         lambda: _native.realign_copy(dst.data_ptr() + 16, window.data_ptr() + 3, half, stream),
         lambda: torch.equal(dst[16 : 16 + half], window[3 : 3 + half]))
    n16 = cal // 2 // 48 // 64 * 64
    src16 = window[:cal].view(torch.float16)
    src16.copy_(torch.randn(src16.numel() // 64, device=dev, dtype=torch.float16).repeat(64))  # finite values
    dst8 = dst[: cal // 2]
    cj = [(dst8.data_ptr() + i * n16, src16.data_ptr() + 2 * i * n16, n16, _native.ELEM_TYPES["F16"], _native.ELEM_TYPES["F8_E4M3"])
          for i in range(48)]
    vrow(f"fp16 -> fp8 e4m3, 48 tensors of {n16} elements per launch", "convert_kernel", 3 * n16 * 48,
         lambda: _native.convert_batch(cj, stream),
         lambda: torch.equal(dst8[: 1 << 22].view(torch.int8), src16[: 1 << 22].to(torch.float8_e4m3fn).view(torch.int8)))
    src32b = window[:cal].view(torch.float32)
    src32b.copy_(torch.randn(src32b.numel() // 64, device=dev).repeat(64))
    cj2 = [(dst16.data_ptr() + 2 * i * per, src32b.data_ptr() + 4 * i * per, per, _native.ELEM_TYPES["F32"], _native.ELEM_TYPES["F16"])
           for i in range(48)]
    vrow(f"fp32 -> fp16, 48 tensors of {per} elements per launch", "convert_kernel", 6 * per * 48,
         lambda: _native.convert_batch(cj2, stream),
         lambda: torch.equal(dst16[probe], src32b[probe].to(torch.float16).view(torch.int16)))
    tp = torch.randint(-30000, 30000, (65536, 4090), dtype=torch.int16, device=dev)
    bw = -(-4090 // world)
    widep = [torch.zeros((65536, bw + 40), dtype=torch.int16, device=dev) for _ in range(world)]
    pj = [(widep[r].data_ptr() + 2 * 7, tp.data_ptr() + 2 * r * bw, 65536, 2 * min(bw, 4090 - r * bw), 8180, 2 * (bw + 40)) for r in range(world)]
    vrow("bf16 [65536, 4090] cut in 4 along dim 1 into columns 7.. of tensors 40 columns wider (pitched destination), 4 ranks per launch",
         "gather_kernel<one source, pitched>", 2 * 2 * 65536 * 4090, lambda: _native.slice_copy2d_batch(pj, stream),
         lambda: all(torch.equal(widep[r][:, 7 : 7 + min(bw, 4090 - r * bw)], tp[:, r * bw : (r + 1) * bw]) and not widep[r][:, :7].any()
                     for r in range(world)))
    del widep
    tsj = [torch.randint(0, 100, (32768, 8190), dtype=torch.uint8, device=dev) for _ in range(6)]
    bj = -(-8190 // world)
    outp = torch.zeros((32768, 6 * bj + 256), dtype=torch.uint8, device=dev)
    jp = [(t.data_ptr(), bj, 8190) for t in tsj]
    vrow("6 x fp8 [32768, 8190], column blocks of rank 0 joined along dim 1 into rows 256 bytes wider (pitched destination)",
         "gather_kernel<several sources, pitched>", 2 * 32768 * 6 * bj,
         lambda: _native.join_copy(outp.data_ptr(), 32768, jp, stream, dst_pitch=6 * bj + 256),
         lambda: torch.equal(outp[:, : 6 * bj], torch.cat([t[:, :bj] for t in tsj], dim=1)) and not outp[:, 6 * bj :].any())
    del tsj, outp, tp
    out["variants"] = variants
    avg_ms = sum(times) / len(times)
    out["realign_copy"] = {
        "workload": "C2 GPT-2-medium fp16 data section, 709,646,336 bytes, source shifted by 10 bytes",
        "launches_timed": len(times), "avg_launch_ms": avg_ms, "bytes_per_launch": 2 * n,
        "achieved_GBps": 2 * n / 1e6 / avg_ms, "best_GBps": 2 * n / 1e6 / min(times),
    }
    return out


def bench_downcast(data_dir: str, threads: int) -> dict:
    """GPT-2-small fp32 (config C1, 497,759,232 data bytes) loaded warm as stored and with a
    down-cast to fp16 / bf16 on load -- the case of the reference's published figure
    (docs/amd-perf.md:73,77: 2.07 GB/s as stored, 0.77 GB/s with the F16 cast, MI300X)."""
    import torch

    from fastsafetensors_amd import DType, SafeTensorsFileLoader, SingleGroup
    from fastsafetensors_amd import checkpoints as ck

    recs = ck.write_config(ck.configs(1.0)["C1"], data_dir, device="cpu", sha256=False)
    path = recs[0]["path"]
    nbytes = recs[0]["size"] - recs[0]["header_length"]
    warm_cache([path])
    out = {"workload": f"C1 GPT-2-small fp32, {nbytes} data bytes, warm page cache; GB/s counts the file's bytes"}
    ref = None
    for label, dtype, tdt in [("as_stored", DType.AUTO, None), ("to_f16", DType.F16, torch.float16),
                              ("to_bf16", DType.BF16, torch.bfloat16)]:
        best = None
        for rep in range(3):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            loader = SafeTensorsFileLoader(SingleGroup(), "cuda:0", max_threads=threads)
            loader.add_filenames({0: [path]})
            bufs = loader.copy_files_to_device(dtype=dtype)
            tensors = {k: bufs.get_tensor(k) for k in loader.get_keys()}
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            best = dt if best is None else min(best, dt)
            if rep == 0:
                if ref is None:
                    ref = {k: t.clone() for k, t in tensors.items()}
                elif not all(torch.equal(t.view(torch.int16), ref[k].to(tdt).view(torch.int16)) for k, t in tensors.items()):
                    raise SystemExit(f"bench: tensors loaded with dtype={dtype} differ from Tensor.to()")
            del tensors
            bufs.close()
            loader.close()
        out[label] = {"seconds_best_of_3": best, "GBps": nbytes / 1e9 / best}
    return out


# ---- CPU baseline -------------------------------------------------------------------------------------


def cpu_baseline(files: List[str], budget_s: float = 25.0, cold: bool = False) -> dict:
    """The reference's device="cpu", nogds=True path on this host: thread-per-request
    pread -> bounce -> memcpy into a 4096-aligned host buffer.  Warm page cache (or, with
    ``cold``, every file dropped from it first), whole
    files until the time budget is used; the reference's defaults (16 MiB bounce,
    16 threads, 16 GiB blocks = one thread per file) and its documented tuned
    setting (16 threads, 16 MiB, 160 MB blocks)."""
    from oracle import st_oracle as orc

    cpp = orc.load_reference_cpp()
    kind = "reference" if cpp is not None else "port"
    results = {}
    for label, bbuf_kb, threads, block in [("defaults", 16 * 1024, 16, 16 * 1024**3),
                                           ("tuned_160MB_blocks", 16 * 1024, 16, 160 * 1000 * 1000)]:
        done_bytes, t_total, used, n_threads_live = 0, 0.0, [], 0
        if cold:
            drop_cache(files)
        for path in files:
            if t_total > budget_s / 2:
                break
            h = orc.parse_file(path)
            total = h.size_bytes - h.header_length
            if cpp is not None:
                base = cpp.cpu_malloc(total)
                gbuf = cpp.gds_device_buffer(base, total, False)
                t0 = time.perf_counter()
                reader = cpp.nogds_file_reader(False, bbuf_kb, threads, False, 0)
                fd = os.open(path, os.O_RDONLY)
                reqs, count = [], 0
                while count < total:
                    l = min(block, total - count)
                    reqs.append(reader.submit_read(fd, gbuf, h.header_length + count, l, count))
                    count += l
                ok = all(reader.wait_read(r) > 0 for r in reqs)
                os.close(fd)
                dt = time.perf_counter() - t0
                del reader
                cpp.cpu_free(base)
                n_threads_live = max(n_threads_live, min(len(reqs), threads))
            else:
                t0 = time.perf_counter()
                reader = orc.NogdsReader(bbuf_kb, threads)
                data = reader.load_file(path, h, block)
                ok = data.size == total
                dt = time.perf_counter() - t0
                reader.close()
                n_threads_live = max(n_threads_live, min(-(-total // block), threads))
            if not ok:
                raise SystemExit("bench: the CPU baseline failed to read " + path)
            done_bytes += total
            t_total += dt
            used.append(os.path.basename(path))
        results[label] = {"GBps": done_bytes / 1e9 / t_total, "bytes": done_bytes, "seconds": t_total,
                          "files": used, "threads": n_threads_live}
    best = max(results.values(), key=lambda r: r["GBps"])
    return {
        "value": best["GBps"], "unit": "GB/s", "cores": best["threads"], "kind": kind,
        "sample": f"{'cold' if cold else 'warm'} page cache, {len(best['files'])} of {len(files)} files ({best['bytes']} bytes) into host "
                  f"memory; host has {os.cpu_count()} CPUs",
        "settings": results,
    }


# ---- whole loads of the other configurations -----------------------------------------------------------


def bench_whole_load(files: List[str], data_bytes: int, verify, threads: int, block_kb: int, reps: int = 3,
                     iterate: bool = False, with_cpu: bool = False) -> dict:
    """Warm whole loads (loader construction to last tensor) of a checkpoint whose files sit in
    the page cache or on tmpfs, next to the copy-only leg of the same requests; the first load is
    verified against the generator's checksums.  ``iterate`` adds ``ParallelLoader.iterate_weights``."""
    import torch

    # Loads and legs take turns, best of each, on the device memory the pass before has just returned
    # to the allocator: a leg is a ceiling, and a pass over device memory that was never handed out
    # before runs 10 % slower.  A leg that a load has beaten is no ceiling: up to three more are taken.
    runs = [run_load(files, "auto", threads, block_kb, verify)]
    legs = []
    for _ in range(max(reps - 1, 1)):
        legs.append(engine_leg(files, "copy_only", threads, block_kb))
        runs.append(run_load(files, "auto", threads, block_kb, None))
    best = min(runs, key=lambda r: r["elapsed_s"])
    for _ in range(3):
        if max(r["GBps"] for r in legs) >= data_bytes / 1e9 / best["elapsed_s"]:
            break
        legs.append(engine_leg(files, "copy_only", threads, block_kb))
    leg = max(legs, key=lambda r: r["GBps"])
    torch.cuda.empty_cache()
    out = {"files": len(files), "data_bytes": data_bytes, "seconds_to_load": best["elapsed_s"],
           "seconds_all": [r["elapsed_s"] for r in runs], "GBps": data_bytes / 1e9 / best["elapsed_s"],
           "copy_only_leg_GBps": leg["GBps"], "copy_only_legs_all_GBps": [r["GBps"] for r in legs],
           "frac_of_copy_only_leg": data_bytes / 1e9 / best["elapsed_s"] / leg["GBps"],
           "verified_tensors": runs[0].get("verified_tensors", 0)}
    if iterate:
        out["iterate_weights"] = bench_iterate_weights(files, threads, verify)
        torch.cuda.empty_cache()
    if with_cpu:
        # the reference's device="cpu" path over as many of the files as 12 s allow (page-cache / tmpfs reads)
        cw = cpu_baseline(files, budget_s=12.0)
        out["cpu_reference"] = {"kind": cw["kind"], "warm_GBps": cw["value"], "cores": cw["cores"], "sample": cw["sample"],
                                "defaults_warm_GBps": cw["settings"]["defaults"]["GBps"]}
    return out


def placement_facts(threads: int, block_kb: int) -> dict:
    """Where the I/O side of a loader runs: the node the device hangs off, that node's CPUs, and
    what the library read back after binding its workers and placing the ring."""
    from fastsafetensors_amd import SafeTensorsFileLoader, SingleGroup, _native
    from fastsafetensors_amd.common import get_device_numa_node

    loader = SafeTensorsFileLoader(SingleGroup(), "cuda:0", max_threads=threads, block_size_kb=block_kb)
    m = loader.copier_constructor.reader.metrics()
    loader.close()
    node = get_device_numa_node(0)
    cpus = _native.node_cpus(int(m.numa_node)) if m.numa_node >= 0 else []
    return {"device_numa_node_sysfs": node, "numa_node_bound": int(m.numa_node), "node_cpus": len(cpus),
            "node_cpu_range": f"{cpus[0]}-{cpus[-1]}" if cpus else None, "io_threads": threads,
            "workers_on_node": int(m.workers_on_node), "ring_node": int(m.ring_node), "bind_errors": int(m.bind_errors),
            "host_cpus": os.cpu_count()}


# ---- main -----------------------------------------------------------------------------------------------


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=3)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--config", default="C3", choices=["C1", "C2", "C3", "C4", "C5"])
    ap.add_argument("--dir", default=os.environ.get("FSTX_BENCH_DIR", os.path.join(ROOT, "_bench_data")))
    ap.add_argument("--threads", type=int, default=16)
    ap.add_argument("--block-kb", type=int, default=4096)
    ap.add_argument("--keep", action="store_true", help="keep the generated checkpoint")
    ap.add_argument("--skip-cpu-baseline", action="store_true")
    ap.add_argument("--skip-kernels", action="store_true")
    ap.add_argument("--skip-c5", action="store_true", help="leave out the 72.7 GB whole load of config C5 from tmpfs")
    ap.add_argument("--kernels-only", action="store_true",
                    help="run only the HBM kernel section (short; the command the counter profiles use)")
    ap.add_argument("--detail-out", default=os.path.join(ROOT, "bench_out", "bench_detail.json"),
                    help="file that receives every figure of the run; the stdout line carries the summary")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        raise SystemExit("bench.py: this load path drives ONE GPU; run it with --gpus 1 "
                         "(files shard across GPUs at file granularity, nothing here spans two devices)")

    import torch

    from fastsafetensors_amd import checkpoints as ck

    assert torch.cuda.is_available(), "bench.py needs the MI355X"
    if args.kernels_only:
        print(json.dumps({"kernels": bench_kernels(args.steps, args.warmup)}), flush=True)
        return
    cfg = ck.configs(1.0)[args.config]
    # the checkpoint (and, briefly, the 0.5 GB down-cast file) must fit; a disk that is too
    # small sends the files to /dev/shm, where "cold" cannot be measured (tmpfs has no O_DIRECT)
    need = sum(sp.nbytes for f in cfg.files() for sp in f) + (2 << 30)
    os.makedirs(args.dir, exist_ok=True)
    storage_note = None
    if shutil.disk_usage(args.dir).free < need and os.path.isdir("/dev/shm") and shutil.disk_usage("/dev/shm").free > need:
        storage_note = (f"{args.dir} has less than {need} bytes free: files written to /dev/shm (tmpfs, no O_DIRECT); "
                        "the cold figures are page-cache reads here")
        log("[bench] " + storage_note)
        args.dir = "/dev/shm/fstx_bench"
    data_dir = os.path.join(args.dir, args.config)
    ck.CHUNK_ELEMS = 1 << 62  # whole tensors, so that one checksum covers each
    SEED_BASE = 1234
    inputs: Dict[str, dict] = {}

    def write(key: str, directory: str, device: str, sha256: bool, sums=None):
        """One configuration's files; seed, generator device and (where asked) SHA-256 go to the log."""
        def on_chunk(spec, chunk):
            if spec.name in sums:
                raise SystemExit("bench: a tensor arrived in several chunks; one checksum must cover it")
            sums[spec.name] = checksum(chunk)

        t0 = time.perf_counter()
        recs = ck.write_config(ck.configs(1.0)[key], directory, seed_base=SEED_BASE, device=device, sha256=sha256,
                               on_chunk=on_chunk if sums is not None else None)
        nbytes = sum(r["size"] - r["header_length"] for r in recs)
        log(f"[bench] wrote {key}: {len(recs)} files, {nbytes} data bytes in {time.perf_counter() - t0:.1f}s -> {directory} "
            f"(values: torch.Generator on {device}, seed base {SEED_BASE}, file k tensor i: seed {SEED_BASE} + 100000 k + i)")
        for r in recs:
            if r["sha256"]:
                log(f"[bench]   sha256 {r['sha256']}  {os.path.basename(r['path'])} ({r['size']} bytes)")
        inputs.setdefault(key, {"generator_device": device, "seed_base": SEED_BASE, "files": len(recs), "data_bytes": nbytes,
                                "sha256": [r["sha256"] for r in recs] if sha256 else None})
        return recs, nbytes

    # C3 and larger are generated on the GPU (16-73 GB of normal variates take minutes on the host
    # cores); C1 and C2 come from the CPU generator and are the same bytes on any machine
    sums: Dict[str, Tuple[int, int]] = {}
    recs, data_bytes = write(args.config, data_dir, "cpu" if args.config in ("C1", "C2") else "cuda", True, sums)
    files = [r["path"] for r in recs]
    verify = dict(sums)
    torch.cuda.empty_cache()

    tp_dir = os.path.join(args.dir, "C4_tp")
    c5_dir = "/dev/shm/fstx_bench_C5"
    c4 = c5 = None
    try:
        placement = placement_facts(args.threads, args.block_kb)
        log(f"[bench] I/O placement: {placement}")
        # ---- cold: every load sits between two read-only legs of the same engine
        drop_cache(files)
        cold_frac = resident_fraction(files)
        h2d = max(measure_h2d_peak(chunk=16 << 20), measure_h2d_peak(chunk=64 << 20))
        log(f"[bench] pinned H2D copy probe (torch, 2 streams): {h2d:.2f} GB/s; resident after drop {cold_frac:.3f}")

        def read_only_cold() -> Dict[str, float]:
            drop_cache(files)
            leg = engine_leg(files, "read_only", args.threads, args.block_kb)
            log(f"[bench]   read-only leg (cold): {leg['GBps']:.2f} GB/s in {leg['seconds']:.3f}s, {leg['direct_reads']} O_DIRECT reads")
            return leg

        def steps_of(kind: str, n: int, check: bool, **kw) -> List[Dict[str, float]]:
            runs = []
            for i in range(n):
                if kind == "cold":
                    before = last_leg[0] if last_leg[0] is not None else read_only_cold()
                    drop_cache(files)
                r = run_load(files, "auto", args.threads, args.block_kb, verify if (check and i == 0) else None, **kw)
                if kind == "cold":
                    # the disk is shared and throttled in bursts: its ceiling is taken right
                    # around the step, not once at the start
                    last_leg[0] = read_only_cold()
                    r["read_only_leg_GBps_around_step"] = [before["GBps"], last_leg[0]["GBps"]]
                    # one O_DIRECT read is in flight at a time, so the time inside pread is the
                    # time the disk was busy: what it delivered to this very load while it worked
                    r["disk_GBps_while_reading"] = r["bytes"] / 1e9 / r["pread_s"] if r["pread_s"] else None
                runs.append(r)
                log(f"[bench] {kind} step {i}: elapsed {r['elapsed_s']:.3f}s (init {r['init_s'] * 1e3:.1f} ms, reader create {r['reader_create_s'] * 1e3:.1f} ms) io {r['io_s']:.3f}s "
                    f"-> {r['bytes'] / 1e9 / r['elapsed_s']:.2f} GB/s (direct blocks {r['blocks_direct']} in {r['direct_reads']} reads, buffered {r['blocks_buffered']}, in pread {r['pread_s']:.2f}s, staging memcpy {r['stage_memcpy_s']:.2f}s, slot wait {r['slot_wait_s']:.2f}s)")
            return runs

        last_leg = [None]  # a read-only leg sits between every two cold loads
        steps_of("cold", args.warmup, False)
        cold = steps_of("cold", args.steps, True)
        # The storage's own ceiling, from readers that share nothing with this engine: a plain
        # single-threaded reader with 1 GiB requests over the whole checkpoint (the fastest plain
        # pattern found on the disk this was developed on), and a sweep of threads x request sizes.
        drop_cache(files)
        nb, dt = parallel_read(files, direct=True, threads=1, limit=None, block=1 << 30)
        plain_reader = nb / 1e9 / dt
        sweep = plain_reader_sweep(files) if not storage_note else {}
        log(f"[bench] plain O_DIRECT readers: whole checkpoint 1 thread x 1 GiB {plain_reader:.2f} GB/s; one file each: "
            + ", ".join(f"{k} {v:.2f}" for k, v in sweep.items()))
        drop_cache(files)
        cold_adaptive = run_load(files, "auto", args.threads, args.block_kb, None, adaptive_depth=True,
                                 direct_read_kb=64 << 10, shared_reader=False)
        log(f"[bench] cold load with steered depth and 64 MiB reads "
            f"{cold_adaptive['bytes'] / 1e9 / cold_adaptive['elapsed_s']:.2f} GB/s (depth settled at {cold_adaptive['direct_depth']})")
        cold_cpu = None if args.skip_cpu_baseline else cpu_baseline(files, cold=True)

        # ---- warm: legs before and after the steps
        warm_cache(files)
        warm_frac = resident_fraction(files)
        warm_legs = {"read_only": [], "copy_only": []}

        def warm_legs_once():
            # best of three each: a leg is a ceiling, and its first pass pays for device memory the
            # allocator has not handed out before (the loads around it reuse their arenas)
            for probe in ("read_only", "copy_only"):
                leg = max((engine_leg(files, probe, args.threads, args.block_kb) for _ in range(3)), key=lambda r: r["GBps"])
                warm_legs[probe].append(leg["GBps"])
            log(f"[bench]   warm legs: read-only {warm_legs['read_only'][-1]:.1f} GB/s, copy-only {warm_legs['copy_only'][-1]:.2f} GB/s")

        warm_legs_once()
        steps_of("warm", args.warmup, False)
        warm = steps_of("warm", args.steps, True)
        warm_legs_once()
        h2d = max(h2d, measure_h2d_peak(chunk=16 << 20))
        itw = bench_iterate_weights(files, args.threads, verify)
        log(f"[bench] iterate_weights warm: {itw['GBps']:.1f} GB/s ({itw['seconds']:.3f} s)")
        base = None if args.skip_cpu_baseline else cpu_baseline(files)
        if not args.keep and args.config != "C4":
            shutil.rmtree(data_dir, ignore_errors=True)  # room in the page cache for what follows (C4's files are used again below)

        small = {}
        for k in ("C1", "C2"):
            small[k] = bench_small_checkpoint(k, os.path.join(args.dir, k + "_small"), args.threads, write, with_cpu=not args.skip_cpu_baseline)
            w = small[k]["warm"]
            log(f"[bench] {k}: cold {small[k]['cold']['GBps']:.2f} GB/s (io {small[k]['cold']['io_over_read_only_leg']:.3f} x read-only leg), "
                f"warm {w['GBps']:.1f} GB/s = {w['frac_of_copy_only_leg']:.3f} of the copy-only leg "
                f"(no ring left parked by an earlier load: {small[k]['warm_fresh_ring']['frac_of_copy_only_leg']:.3f}), held "
                f"{small[k]['warm_held_reader']['frac_of_copy_only_leg']:.3f}"
                + (f", window layout {small[k]['warm_window_layout_realign']['frac_of_copy_only_leg']:.3f}" if k == "C2" else ""))
        # ---- C4: whole load from tmpfs, then the tensor-parallel callers over the resident checkpoint
        c4_sums: Dict[str, Tuple[int, int]] = {}
        if args.config == "C4":
            tp_files, c4_bytes, c4_sums = files, data_bytes, verify
        else:
            # where its files come from does not matter to an HBM-resident workload, so they go to
            # tmpfs when it has room (no second checkpoint on the disk, no write-back to wait for)
            c4_need = sum(sp.nbytes for f in ck.configs(1.0)["C4"].files() for sp in f)
            if os.path.isdir("/dev/shm") and shutil.disk_usage("/dev/shm").free > c4_need + (8 << 30):
                tp_dir = "/dev/shm/fstx_bench_C4_tp"
            tp_recs, c4_bytes = write("C4", tp_dir, "cuda", False, c4_sums)
            tp_files = [r["path"] for r in tp_recs]
            warm_cache(tp_files)
        torch.cuda.empty_cache()
        c4 = bench_whole_load(tp_files, c4_bytes, c4_sums, args.threads, args.block_kb, with_cpu=not args.skip_cpu_baseline)
        log(f"[bench] C4 whole load (warm): {c4['GBps']:.1f} GB/s in {c4['seconds_to_load']:.3f}s = {c4['frac_of_copy_only_leg']:.3f} of the copy-only leg")
        tp = bench_tp_extract(tp_files, 4, args.threads, args.block_kb)
        log(f"[bench] TP=4 as_dict over the resident checkpoint: {tp['GBps']:.0f} GB/s, seconds per rank {[round(x, 4) for x in tp['seconds_per_rank']]}")
        mc = bench_multi_cols(tp_files, 4, args.threads, args.block_kb)
        log(f"[bench] TP=4 get_multi_cols (QKV, gate/up) over the resident checkpoint: {mc['GBps']:.0f} GB/s, seconds per rank {[round(x, 4) for x in mc['seconds_per_rank']]}")
        if args.config != "C4":
            shutil.rmtree(tp_dir, ignore_errors=True)
        downcast = bench_downcast(os.path.join(args.dir, "C1_downcast"), args.threads)
        log(f"[bench] C1 fp32 warm load: " + ", ".join(f"{k} {v['GBps']:.1f} GB/s" for k, v in downcast.items() if isinstance(v, dict)))
        torch.cuda.empty_cache()
        # ---- C5: 72.7 GB of fp8 + bf16 + fp32 scalars from tmpfs into one GPU's HBM
        c5_need = sum(sp.nbytes for f in ck.configs(1.0)["C5"].files() for sp in f)
        if args.skip_c5 or args.config == "C5":
            c5 = {"skipped": "--skip-c5" if args.skip_c5 else "C5 is the main configuration of this run"}
        elif not os.path.isdir("/dev/shm") or shutil.disk_usage("/dev/shm").free < c5_need + (16 << 30):
            c5 = {"skipped": f"/dev/shm has less than {c5_need + (16 << 30)} bytes free"}
        else:
            c5_sums: Dict[str, Tuple[int, int]] = {}
            c5_recs, c5_bytes = write("C5", c5_dir, "cuda", False, c5_sums)
            torch.cuda.empty_cache()
            c5 = bench_whole_load([r["path"] for r in c5_recs], c5_bytes, c5_sums, args.threads, args.block_kb, reps=2, iterate=True,
                                  with_cpu=not args.skip_cpu_baseline)
            shutil.rmtree(c5_dir, ignore_errors=True)
            log(f"[bench] C5 whole load (tmpfs): {c5['GBps']:.1f} GB/s in {c5['seconds_to_load']:.3f}s = {c5['frac_of_copy_only_leg']:.3f} of the copy-only leg; "
                f"iterate_weights {c5['iterate_weights']['GBps']:.1f} GB/s")
        kernels = {} if args.skip_kernels else bench_kernels(args.steps, args.warmup)
    finally:
        if not args.keep:
            shutil.rmtree(data_dir, ignore_errors=True)
        shutil.rmtree(os.path.join(args.dir, "C1_downcast"), ignore_errors=True)
        shutil.rmtree(tp_dir, ignore_errors=True)
        shutil.rmtree(c5_dir, ignore_errors=True)
        if storage_note:
            shutil.rmtree(args.dir, ignore_errors=True)

    def summarize(runs, ceiling):
        el = sorted(r["elapsed_s"] for r in runs)
        total_s = sum(el)
        gbps = data_bytes * len(runs) / 1e9 / total_s
        frac = gbps / ceiling
        return {"GBps": gbps, "seconds_to_load_median": el[len(el) // 2], "seconds_to_load_min": el[0],
                "io_GBps_median": data_bytes / 1e9 / sorted(r["io_s"] for r in runs)[len(runs) // 2],
                "init_ms_median": 1e3 * sorted(r["init_s"] for r in runs)[len(runs) // 2],
                "reader_create_ms_median": 1e3 * sorted(r["reader_create_s"] for r in runs)[len(runs) // 2],
                "roofline_GBps": ceiling, "frac_of_roofline": frac,
                # a load faster than its ceiling means the ceiling moved between the leg and the load
                "ceiling_valid": frac <= 1.0}

    copy_only = max(warm_legs["copy_only"])
    # cold ceiling: the faster of the two read-only legs around each step, median over the steps,
    # and never above the ring -> HBM leg
    around = sorted(max(r["read_only_leg_GBps_around_step"]) for r in cold)
    read_only_cold = around[len(around) // 2]
    cold_s = summarize(cold, min(read_only_cold, copy_only))
    fr = sorted(r["bytes"] / 1e9 / r["elapsed_s"] / min(max(r["read_only_leg_GBps_around_step"]), copy_only) for r in cold)
    cold_s["frac_of_roofline_per_step_median"] = fr[len(fr) // 2]
    busy = sorted(r["pread_s"] / r["elapsed_s"] for r in cold)
    cold_s["disk_busy_fraction_median"] = busy[len(busy) // 2]
    insitu = sorted(r["disk_GBps_while_reading"] for r in cold if r.get("disk_GBps_while_reading"))
    if insitu:
        cold_s["disk_GBps_while_reading_median"] = insitu[len(insitu) // 2]
    best_disk = max([x for r in cold for x in r["read_only_leg_GBps_around_step"]] + insitu + [plain_reader] + list(sweep.values()))
    cold_s["frac_of_best_disk_rate_seen_in_run"] = cold_s["GBps"] / min(best_disk, copy_only)
    # ceilings that owe nothing to this engine: the best plain O_DIRECT reader, torch's pinned copy
    independent_disk = max([plain_reader] + list(sweep.values()))
    cold_s["ceiling_independent_GBps"] = min(independent_disk, h2d)
    cold_s["frac_of_independent_ceiling"] = cold_s["GBps"] / cold_s["ceiling_independent_GBps"]
    cold_s["roofline_note"] = (
        "roofline = min(read-only leg, copy-only leg) of the same engine (fstx_config.flags FSTX_PROBE_NO_COPY / NO_READ: same threads, "
        "queue, request sizes, ring and streams with one stage left out); the read-only leg runs cold right before and right after every "
        "cold step and the faster of the two is taken, because the disk is a throttled shared virtual disk whose rate drifts within a run; "
        "ceiling_independent = min(best plain sequential O_DIRECT reader of the run: whole checkpoint at 1 thread x 1 GiB and a sweep of "
        "{1,2,4} threads x {64 MiB, 256 MiB, 1 GiB} over one file each; torch's pinned copy_ on two streams); "
        "disk_busy_fraction = time inside pread / wall time of the load with one read in flight at a time")
    warm_s = summarize(warm, min(max(warm_legs["read_only"]), copy_only))
    warm_s["ceiling_independent_GBps"] = h2d
    warm_s["frac_of_independent_ceiling"] = warm_s["GBps"] / h2d

    detail = {
        "config": {"workload": f"{args.config}: {cfg.title}, {data_bytes} data bytes, read_mode=auto, {args.threads} I/O threads, "
                               f"{args.block_kb} KiB blocks"},
        "inputs": inputs, "placement": placement,
        "cold": cold_s, "warm": warm_s, "cold_steps": cold, "warm_steps": warm,
        "pipeline": {"read_only_leg_cold_GBps_median_of_best_around_steps": read_only_cold,
                     "read_only_leg_warm_GBps": warm_legs["read_only"], "copy_only_leg_GBps": warm_legs["copy_only"],
                     "vs_plain_reader": cold_s["GBps"] / plain_reader, "plain_o_direct_reader_GBps": plain_reader,
                     "plain_o_direct_sweep_GBps": sweep, "torch_pinned_h2d_probe_GBps": h2d,
                     "cold_adaptive": {"GBps": cold_adaptive["bytes"] / 1e9 / cold_adaptive["elapsed_s"],
                                       "direct_depth": cold_adaptive["direct_depth"], "direct_reads": cold_adaptive["direct_reads"],
                                       "setting": "adaptive_depth=True, 64 MiB reads"},
                     "resident_after_drop": cold_frac, "resident_after_warmup": warm_frac,
                     "parity": f"{cold[0].get('verified_tensors', 0)} tensors checksum-verified on the GPU after a cold and a warm load"},
        "small_checkpoints": small, "C4_whole_load": c4, "C5_whole_load": c5,
        "tp_extract": tp, "multi_cols": mc, "iterate_weights": itw, "downcast_on_load": downcast, "kernels": kernels,
    }
    if storage_note:
        detail["pipeline"]["storage_note"] = storage_note

    def r3(x):
        return None if x is None else round(x, 3)

    def pipe(sm, ceiling_name):
        return {"achieved": r3(sm["GBps"]), "ceiling": r3(sm["roofline_GBps"]), "frac": r3(sm["frac_of_roofline"]),
                "ceiling_independent": r3(sm["ceiling_independent_GBps"]), "frac_independent": r3(sm["frac_of_independent_ceiling"]),
                "seconds_to_load": r3(sm["seconds_to_load_median"]), "unit": "GB/s", "ceiling_is": ceiling_name}

    line = {
        "metric": "file->HBM GB/s, cold page cache, " + ("Llama-3-8B bf16" if args.config == "C3" else cfg.title)
                  + " checkpoint (whole load: ctor to last tensor)",
        "value": cold_s["GBps"],
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": 1e3 * sum(r["elapsed_s"] for r in cold) / len(cold),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u8",
        "data": "synthetic",
        "config": detail["config"],
        "seconds_to_load": {"cold": r3(cold_s["seconds_to_load_median"]), "warm": r3(warm_s["seconds_to_load_median"])},
    }
    if kernels:
        k = kernels["slice_extract"]
        tr = measured_traffic()
        # the counters belong to this workload only while its algorithmic bytes are what they were when profiled
        same = tr.get("algorithmic_bytes_per_launch") == str(int(k["bytes_per_launch"]))
        line["roofline"] = {"bound": "hbm", "achieved": k["achieved_GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                            "frac": k["achieved_GBps"] / HBM_PEAK_GBPS,
                            "traffic": int(tr["hbm_traffic_bytes_per_launch"]) if same else None,
                            "traffic_source": os.path.relpath(TRAFFIC_FILE, ROOT) if same else "no counter profile of this workload",
                            "kernel": "slice_kernel",
                            "workload": "C4 Llama-2-13B bf16 TP=4, column cuts of file 1 of 3 (28 tensors per launch, one launch per rank)",
                            "avg_launch_ms": k["avg_launch_ms"], "bytes_per_launch": k["bytes_per_launch"]}
        detail["roofline"] = dict(line["roofline"], workload=k["workload"])
    else:
        line["roofline"] = {"bound": "hbm", "achieved": None, "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": None, "traffic": None,
                            "note": "--skip-kernels"}
    # the load pipeline next to its own ceilings: not an HBM figure, but the fraction the target is stated on
    line["roofline"]["pipeline"] = {
        "cold": pipe(cold_s, "min(read-only leg around the step, copy-only leg) of the same engine"),
        "warm": pipe(warm_s, "min(warm read-only leg, copy-only leg) of the same engine"),
        "independent_is": "cold: min(best plain O_DIRECT reader of the run, torch pinned copy); warm: torch pinned copy",
        "plain_o_direct_GBps": {"whole_checkpoint_1x1024MiB": r3(plain_reader), **{k: r3(v) for k, v in sweep.items()}},
        "torch_pinned_h2d_GBps": r3(h2d), "disk_busy_fraction": r3(cold_s["disk_busy_fraction_median"]),
        "ceiling_valid": bool(cold_s["ceiling_valid"] and warm_s["ceiling_valid"]),
    }
    if kernels:
        def kern(d):
            return {"GBps": round(d["achieved_GBps"]), "frac": r3(d["achieved_GBps"] / HBM_PEAK_GBPS), "avg_launch_ms": r3(d["avg_launch_ms"])}

        rows = {name: kern(kernels[name]) for name in ("slice_extract", "row_block_copy", "slice_join_columns", "realign_copy",
                                                        "convert_f32_bf16", "calibration_copy") if name in kernels}
        for group in ("slice_extract_odd_shapes", "join_odd_columns", "short_segments", "variants"):
            for label, d in kernels.get(group, {}).items():
                if "gather_kernel" in d:
                    rows[f"{group}: {label}"] = kern(d["gather_kernel"])
                elif "achieved_GBps" in d:
                    rows[f"{group}: {label}"] = kern(d)
        line["roofline"]["kernels"] = rows
    line["configs"] = {
        "C3": {"cold_GBps": r3(cold_s["GBps"]), "cold_s": r3(cold_s["seconds_to_load_median"]), "cold_frac": r3(cold_s["frac_of_roofline"]),
               "warm_GBps": r3(warm_s["GBps"]), "warm_s": r3(warm_s["seconds_to_load_median"]), "warm_frac": r3(warm_s["frac_of_roofline"]),
               "iterate_weights_GBps": r3(itw["GBps"]), "verified_tensors": cold[0].get("verified_tensors", 0)},
    }
    for k in ("C1", "C2"):
        sc = small[k]
        row = {"cold_GBps": r3(sc["cold"]["GBps"]), "cold_s": r3(sc["cold"]["seconds"]),
               "cold_io_over_read_only_leg": r3(sc["cold"]["io_over_read_only_leg"]),
               "warm_GBps": r3(sc["warm"]["GBps"]), "warm_s": round(sc["warm"]["seconds"], 4),
               "warm_frac_of_copy_only_leg": r3(sc["warm"]["frac_of_copy_only_leg"]),
               "warm_fresh_ring_GBps": r3(sc["warm_fresh_ring"]["GBps"]),  # FSTX_RING_CACHE=0: as the first load of a process
               "warm_fresh_ring_frac": r3(sc["warm_fresh_ring"]["frac_of_copy_only_leg"]),
               "warm_held_reader_GBps": r3(sc["warm_held_reader"]["GBps"]),
               "warm_held_reader_frac": r3(sc["warm_held_reader"]["frac_of_copy_only_leg"])}
        if "cpu_reference" in sc:
            row["cpu_reference_GBps"] = {k2: r3(v) for k2, v in sc["cpu_reference"].items() if k2.endswith("GBps")}
        if "warm_window_layout_realign" in sc:
            row["warm_window_layout_realign_GBps"] = r3(sc["warm_window_layout_realign"]["GBps"])
            row["warm_window_layout_realign_frac"] = r3(sc["warm_window_layout_realign"]["frac_of_copy_only_leg"])
        line["configs"][k] = row
    line["configs"]["C4"] = {"warm_GBps": r3(c4["GBps"]), "warm_s": r3(c4["seconds_to_load"]), "warm_frac_of_copy_only_leg": r3(c4["frac_of_copy_only_leg"]),
                             "storage": "page cache" if args.config == "C4" else "tmpfs", "verified_tensors": c4["verified_tensors"],
                             "tp4_as_dict_GBps": round(tp["GBps"]), "tp4_as_dict_ms_per_rank": [round(1e3 * x, 2) for x in tp["seconds_per_rank"]],
                             "tp4_multi_cols_GBps": round(mc["GBps"]), "tp4_multi_cols_ms_per_rank": [round(1e3 * x, 2) for x in mc["seconds_per_rank"]],
                             "shards_reassembled": tp["tensors_reassembled_and_compared"]}
    if "cpu_reference" in c4:
        line["configs"]["C4"]["cpu_reference_GBps"] = {k2: r3(v) for k2, v in c4["cpu_reference"].items() if k2.endswith("GBps")}
    if c5 and "skipped" not in c5:
        line["configs"]["C5"] = {"warm_GBps": r3(c5["GBps"]), "warm_s": r3(c5["seconds_to_load"]), "data_bytes": c5["data_bytes"],
                                 "warm_frac_of_copy_only_leg": r3(c5["frac_of_copy_only_leg"]), "storage": "tmpfs",
                                 "verified_tensors": c5["verified_tensors"],
                                 "iterate_weights_GBps": r3(c5["iterate_weights"]["GBps"])}
        if "cpu_reference" in c5:
            line["configs"]["C5"]["cpu_reference_GBps"] = {k2: r3(v) for k2, v in c5["cpu_reference"].items() if k2.endswith("GBps")}
            line["configs"]["C5"]["cpu_reference_sample"] = c5["cpu_reference"]["sample"]
    else:
        line["configs"]["C5"] = c5
    for key, whole in (("C4", c4), ("C5", c5)):
        if whole.get("frac_of_copy_only_leg", 0) > 1.01:
            # (up to 1 % is the scatter of two passes at the link's rate.)  Beyond that the legs fell into
            # a slow stretch of the link (they come and go within seconds) and bound nothing here
            line["configs"][key]["copy_only_leg_valid"] = False
            line["configs"][key]["copy_only_legs_GBps"] = [r3(x) for x in whole["copy_only_legs_all_GBps"]]
    line["downcast_on_load_GBps"] = {k: r3(v["GBps"]) for k, v in downcast.items() if isinstance(v, dict)}
    line["placement"] = placement
    line["inputs"] = {k: {"generator_device": v["generator_device"], "seed_base": v["seed_base"],
                          "sha256_16": [h[:16] for h in v["sha256"]] if v["sha256"] else None} for k, v in inputs.items()}
    if base:
        if cold_cpu:
            # the headline metric is the cold load: the baseline's own value is its cold figure too,
            # the warm ones sit beside it
            warm_cpu = {k: base[k] for k in ("value", "unit", "cores", "sample")}
            for k, v in cold_cpu["settings"].items():
                base["settings"][k]["cold"] = v
            base["cold"] = {k: cold_cpu[k] for k in ("value", "unit", "cores", "sample", "settings")}
            base["warm"] = warm_cpu
            for k in ("value", "cores", "sample"):
                base[k] = cold_cpu[k]
        detail["cpu_baseline"] = base
        line["cpu_baseline"] = {k: base[k] for k in ("value", "unit", "cores", "kind", "sample")}
        line["cpu_baseline"]["warm_GBps"] = r3(base["warm"]["value"]) if "warm" in base else None
        line["cpu_baseline"]["reference_defaults_GBps"] = {
            "cold": r3(base["settings"]["defaults"].get("cold", {}).get("GBps")), "warm": r3(base["settings"]["defaults"]["GBps"])}
    if storage_note:
        line["storage_note"] = storage_note
    try:
        os.makedirs(os.path.dirname(os.path.abspath(args.detail_out)), exist_ok=True)
        with open(args.detail_out, "w") as f:
            json.dump(dict(line, detail=detail), f, indent=1)
        line["detail_file"] = os.path.relpath(args.detail_out, ROOT)
    except OSError as e:
        log(f"[bench] could not write {args.detail_out}: {e}")
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
