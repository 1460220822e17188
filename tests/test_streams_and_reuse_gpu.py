# SPDX-License-Identifier: Apache-2.0
"""GPU tests of how the loader sits next to a caller's other GPU work and other loaders:
stream ordering instead of device-wide synchronization, the process-wide shared reader,
adaptive O_DIRECT depth, and the corners of the header rules that only show on a device
(empty tensors at odd offsets, conversions the kernel has no pair for)."""
import json
import os
import struct
import time

import numpy as np
import pytest
import torch
from safetensors.torch import load_file

from fastsafetensors_amd import DType, SafeTensorsFileLoader, SingleGroup, _native, checkpoints as ck, hold_reader
from fastsafetensors_amd.frameworks import get_framework_op
from oracle import st_oracle as orc

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def dev_bytes(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().reshape(-1).view(torch.uint8).cpu().numpy()


def assert_clean():
    assert get_framework_op("pytorch").get_mem_used() == 0
    assert _native.get_cpp_metrics().bounce_buffer_bytes == 0


def busy_kernel(ms: float) -> None:
    """Queue a kernel that spins for about ``ms`` milliseconds on the current stream and then
    ends by itself (torch's own test helper; calibrated once)."""
    global _CYCLES_PER_MS
    if _CYCLES_PER_MS is None:
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda._sleep(1_000_000)
        torch.cuda.synchronize()
        a.record()
        torch.cuda._sleep(20_000_000)
        b.record()
        torch.cuda.synchronize()
        _CYCLES_PER_MS = 20_000_000 / a.elapsed_time(b)
    torch.cuda._sleep(int(ms * _CYCLES_PER_MS))


_CYCLES_PER_MS = None


def write_raw(path, entries, pad_to=8):
    """A safetensors file written by hand: ``entries`` = [(name, dtype tag, shape, bytes)] in file order."""
    table, at = {}, 0
    for name, tag, shape, raw in entries:
        table[name] = {"dtype": tag, "shape": list(shape), "data_offsets": [at, at + len(raw)]}
        at += len(raw)
    js = json.dumps(table, separators=(",", ":")).encode()
    js += b" " * (-(8 + len(js)) % pad_to)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(js)) + js + b"".join(e[3] for e in entries))


def test_load_does_not_wait_for_other_streams(golden, monkeypatch):
    """A long kernel on a side stream of the caller: the load does not wait for it.  Two
    checks.  (1) No device-wide synchronize is called anywhere on the path, in either layout.
    (2) A load that launches no kernel (direct layout, aligned file) is back while the side
    kernel still runs.  (A load that does launch kernels is ordered by the runtime, not by the
    loader: null-stream work waits for every stream.)  The runtime spreads all streams of the
    process over a few hardware queues, and what shares a queue with the side stream waits for
    its kernel whatever the loader does: (2) is tried with up to four side streams and holds
    if the load of any attempt was back early -- a loader that waited for the device would be
    late in all of them."""
    path = golden("tiny_gpt2.safetensors")
    h = orc.parse_file(path)
    mine = torch.cuda.Stream()
    busy_kernel(1.0)  # calibrate
    torch.cuda.synchronize()

    def refuse():
        raise AssertionError("torch.cuda.synchronize() called on the load path")

    got, late = {}, []
    for attempt in range(4):
        side, done = torch.cuda.Stream(), torch.cuda.Event()
        with torch.cuda.stream(side):
            busy_kernel(1500 if attempt == 0 else 600)  # finishes by itself
            done.record()
        t0 = time.perf_counter()
        early = None
        with torch.cuda.stream(mine), monkeypatch.context() as mp:
            mp.setattr(torch.cuda, "synchronize", refuse)
            for layout in ("direct", "window") if attempt == 0 else ("direct",):
                loader = SafeTensorsFileLoader(SingleGroup(), DEV, max_threads=4, layout=layout)
                loader.add_filenames({0: [path]})
                bufs = loader.copy_files_to_device()
                if layout == "direct":
                    early = not done.query()
                    if not early:
                        late.append(f"attempt {attempt}: back after {time.perf_counter() - t0:.2f} s")
                got[layout] = {name: bufs.get_tensor(name).clone() for name in h.tensors}
                mine.synchronize()
                bufs.close()
                loader.close()
        side.synchronize()
        if early:
            break
    else:
        raise AssertionError("every load came back only after the side stream's kernel: " + "; ".join(late))
    for layout, tensors in got.items():
        for name, t in tensors.items():
            assert np.array_equal(dev_bytes(t), orc.tensor_bytes(path, h, name)), (layout, name)
    got.clear()
    assert_clean()


def test_arena_reuse_is_ordered_after_the_callers_stream(golden, tmp_path):
    """The allocator hands a closed buffer's memory to the next file; the copy streams must not
    write it while a kernel queued earlier on the caller's stream still reads it."""
    path = str(tmp_path / "big.safetensors")
    n = 48 << 20
    payload = torch.arange(n // 8, dtype=torch.int64)
    write_raw(path, [("x", "I64", [n // 8], payload.numpy().tobytes())])
    want_sum = int(payload.sum())
    loader = SafeTensorsFileLoader(SingleGroup(), DEV, max_threads=8)
    for _ in range(4):
        loader.add_filenames({0: [path]})
        bufs = loader.copy_files_to_device()
        x = bufs.get_tensor("x")
        busy_kernel(30)                            # the reduction below starts 30 ms from now ...
        total = x.sum()                            # ... and reads the arena
        bufs.close()                               # arena back to the allocator while that work is queued
        loader.reset()
        loader.add_filenames({0: [golden("tiny_gpt2.safetensors"), path]})
        again = loader.copy_files_to_device()       # very likely reuses the block
        assert int(total.item()) == want_sum
        assert int(again.get_tensor("x").sum().item()) == want_sum
        again.close()
        loader.reset()
    loader.close()
    assert_clean()


def test_shared_reader_lives_as_long_as_someone_holds_it(golden):
    path = golden("a.safetensors")
    ring = 4 * 2 * (4096 * 1024 + 4096)
    a = SafeTensorsFileLoader(SingleGroup(), DEV, max_threads=4)
    a.copier_constructor.reader.metrics()  # a loader's reader is built behind its back; asking for the metrics waits for it
    assert _native.bounce_buffer_bytes() == ring
    b = SafeTensorsFileLoader(SingleGroup(), DEV, max_threads=4)          # same settings: same reader
    c = SafeTensorsFileLoader(SingleGroup(), DEV, max_threads=4, shared_reader=False)
    b.copier_constructor.reader.metrics(), c.copier_constructor.reader.metrics()
    assert _native.bounce_buffer_bytes() == 2 * ring
    for ld in (a, b, c):
        ld.add_filenames({0: [path]})
        bufs = ld.copy_files_to_device()
        assert torch.equal(bufs.get_tensor("a0").cpu()[:, 0], torch.arange(16, dtype=torch.float16))
        bufs.close()
    a.close()
    c.close()
    assert _native.bounce_buffer_bytes() == ring
    b.close()
    assert_clean()
    # a held reader keeps threads and ring for loaders that come and go
    hold = hold_reader(DEV, max_threads=4)
    created = hold.metrics().create_ns
    for _ in range(3):
        ld = SafeTensorsFileLoader(SingleGroup(), DEV, max_threads=4)
        assert ld.copier_constructor.reader.metrics().create_ns == created  # the same context
        ld.add_filenames({0: [path]})
        ld.copy_files_to_device().close()
        ld.close()
        assert _native.bounce_buffer_bytes() == ring
    hold.close()
    assert_clean()


def test_a_closed_readers_ring_serves_the_next_reader(golden):
    """A closed loader leaves its pinned ring parked; the next loader with the same settings takes
    it over (no allocation, pages already mapped), loads the same bytes, and the parked ring is
    no bounce buffer of anybody and is freed on request."""
    import fastsafetensors_amd

    path = golden("tiny_gpt2.safetensors")
    h = orc.parse_file(path)
    fastsafetensors_amd.release_cached_memory()
    reused = []
    for _ in range(3):
        loader = SafeTensorsFileLoader(SingleGroup(), DEV, max_threads=3, block_size_kb=256)
        loader.add_filenames({0: [path]})
        bufs = loader.copy_files_to_device()
        m = loader.copier_constructor.reader.metrics()
        reused.append(int(m.ring_reused))
        for name in h.tensors:
            assert np.array_equal(dev_bytes(bufs.get_tensor(name)), orc.tensor_bytes(path, h, name)), name
        bufs.close()
        loader.close()
        assert_clean()
        assert _native.cached_ring_bytes() == m.bounce_buffer_bytes
    assert reused == [0, 1, 1]
    assert fastsafetensors_amd.release_cached_memory() == m.bounce_buffer_bytes
    assert _native.cached_ring_bytes() == 0 and fastsafetensors_amd.release_cached_memory() == 0


def test_random_settings_load_the_same_bytes(tmp_path, monkeypatch):
    """Sixty loads of one small multi-file checkpoint with settings drawn at random -- threads,
    block size, read mode, layout, private or shared reader, page cache dropped or not, the ring
    of the last reader kept or not, two loaders at once now and then: every tensor has the
    checksum of the first load, whose bytes are compared with the oracle's."""
    import random
    import threading

    import fastsafetensors_amd

    cfg = ck.configs(0.02)["C3"]
    files = [r["path"] for r in ck.write_config(cfg, str(tmp_path / "c3"))]
    loader = SafeTensorsFileLoader(SingleGroup(), DEV, max_threads=4)
    loader.add_filenames({0: files})
    bufs = loader.copy_files_to_device()
    want = {}
    for path in files:
        h = orc.parse_file(path)
        for name in h.tensors:
            t = bufs.get_tensor(name)
            assert np.array_equal(dev_bytes(t), orc.tensor_bytes(path, h, name)), name
            want[name] = ck.tensor_checksum(t)
    bufs.close()
    loader.close()
    rng = random.Random(11)
    bad = []

    def one(kw, subset):
        ld = SafeTensorsFileLoader(SingleGroup(), DEV, **kw)
        ld.add_filenames({0: subset})
        b = ld.copy_files_to_device()
        bad.extend((kw, k) for k in ld.get_keys() if ck.tensor_checksum(b.get_tensor(k)) != want[k])
        b.close()
        ld.close()

    def draw():
        return dict(max_threads=rng.choice([1, 2, 3, 8, 16]), block_size_kb=rng.choice([64, 256, 1024, 4096]),
                    read_mode=rng.choice(["auto", "buffered", "direct"]), layout=rng.choice(["direct", "window"]),
                    shared_reader=rng.choice([True, False])), (files if rng.random() < 0.7 else files[:1])

    for i in range(60):
        monkeypatch.setenv("FSTX_RING_CACHE", rng.choice(["0", "1", "1"]))
        if rng.random() < 0.3:
            for p in files:
                fd = os.open(p, os.O_RDONLY)
                os.fsync(fd)
                os.posix_fadvise(fd, 0, 0, os.POSIX_FADV_DONTNEED)
                os.close(fd)
        if i % 5 == 4:
            pair = [threading.Thread(target=one, args=draw()) for _ in range(2)]
            for t in pair:
                t.start()
            for t in pair:
                t.join()
        else:
            one(*draw())
        assert not bad, bad[:3]
        assert_clean()
        if i % 9 == 8:
            fastsafetensors_amd.release_cached_memory()
    fastsafetensors_amd.release_cached_memory()
    assert _native.cached_ring_bytes() == 0


def test_adaptive_depth_and_small_direct_reads(tmp_path):
    """O_DIRECT with many small reads in flight and the depth steered while reading -- the
    setting for storage that wants a deep queue -- byte-exact against the oracle."""
    cfg = ck.configs(0.08)["C3"]
    files = [r["path"] for r in ck.write_config(cfg, str(tmp_path / "c3"))]
    total = sum(os.path.getsize(f) for f in files)
    loader = SafeTensorsFileLoader(SingleGroup(), DEV, max_threads=8, read_mode="direct", adaptive_depth=True,
                                   direct_read_kb=1024, block_size_kb=512, shared_reader=False)
    loader.add_filenames({0: files})
    bufs = loader.copy_files_to_device()
    m = loader.copier_constructor.reader.metrics()
    for path in files:
        h = orc.parse_file(path)
        for name in h.tensors:
            assert np.array_equal(dev_bytes(bufs.get_tensor(name)), orc.tensor_bytes(path, h, name)), name
    assert m.direct_depth >= 1
    if m.direct_fallbacks == 0:  # the filesystem took O_DIRECT
        assert m.blocks_direct > 0 and m.blocks_buffered == 0
        assert total // (1 << 20) <= m.direct_reads <= m.blocks_direct  # reads of at most 1 MiB
    bufs.close()
    loader.close()
    assert_clean()


def test_empty_wide_tensor_at_an_odd_offset(tmp_path):
    """An empty F32 / I64 tensor that sits after an odd number of bytes: there is nothing to
    view, and a view at that offset would not be legal for the type."""
    path = str(tmp_path / "odd_empty.safetensors")
    write_raw(path, [("u", "U8", [3], bytes([1, 2, 3])), ("e32", "F32", [0, 5], b""), ("e64", "I64", [0], b""),
                     ("h", "F16", [2], np.array([1.5, -2.0], dtype=np.float16).tobytes()),
                     ("tail", "BF16", [4, 0], b"")])
    for layout in ("direct", "window"):
        loader = SafeTensorsFileLoader(SingleGroup(), DEV, max_threads=2, layout=layout)
        loader.add_filenames({0: [path]})
        bufs = loader.copy_files_to_device()
        assert bufs.get_tensor("u").tolist() == [1, 2, 3]
        assert bufs.get_tensor("h").tolist() == [1.5, -2.0] and bufs.get_tensor("h").data_ptr() % 16 == 0
        for name, shape, dt in (("e32", (0, 5), torch.float32), ("e64", (0,), torch.int64), ("tail", (4, 0), torch.bfloat16)):
            t = bufs.get_tensor(name)
            assert tuple(t.shape) == shape and t.dtype == dt and t.is_cuda
        bufs.close()
        loader.close()
    assert_clean()


@pytest.mark.parametrize("layout", ["direct", "window"])
def test_downcast_of_types_the_kernel_has_no_pair_for(tmp_path, layout):
    """Integer tensors next to float weights, and fp8 sources: converted on the GPU by torch's
    own copy, as the reference converts every tensor (common.py:355-375) -- also when the
    tensor sits at an offset that is odd for its type."""
    g = torch.Generator().manual_seed(4)
    ids = torch.randint(-1000, 1000, (37,), generator=g, dtype=torch.int64)
    i32 = torch.randint(-70000, 70000, (5, 9), generator=g, dtype=torch.int32)
    w = torch.randn(33, 17, generator=g) * 3
    d = torch.randn(11, generator=g, dtype=torch.float64)
    path = str(tmp_path / "mixed_ints.safetensors")
    write_raw(path, [("lead", "BF16", [3], torch.ones(3, dtype=torch.bfloat16).view(torch.int16).numpy().tobytes()),
                     ("ids", "I64", [37], ids.numpy().tobytes()), ("i32", "I32", [5, 9], i32.numpy().tobytes()),
                     ("w", "F32", [33, 17], w.numpy().tobytes()), ("d", "F64", [11], d.numpy().tobytes())], pad_to=1)
    ref = {"lead": torch.ones(3, dtype=torch.bfloat16), "ids": ids, "i32": i32, "w": w, "d": d}
    loader = SafeTensorsFileLoader(SingleGroup(), DEV, max_threads=2, layout=layout)
    loader.add_filenames({0: [path]})
    bufs = loader.copy_files_to_device(dtype=DType.BF16)
    for k, t in ref.items():
        got = bufs.get_tensor(k)
        assert got.dtype == torch.bfloat16 and got.shape == t.shape and got.data_ptr() % 16 == 0, k
        assert torch.equal(got.view(torch.int16).cpu(), t.to(DEV).to(torch.bfloat16).view(torch.int16).cpu()), k
    bufs.close()
    # one-byte sources towards fp8: same size, allowed; fp8 -> fp8 and int8 -> fp8 are torch's
    e5 = (torch.randn(50, generator=g) * 4).to(torch.float8_e5m2)
    i8 = torch.randint(-100, 100, (21,), generator=g, dtype=torch.int8)
    h = torch.randn(13, 3, generator=g, dtype=torch.float16)
    path8 = str(tmp_path / "mixed_fp8.safetensors")
    write_raw(path8, [("u", "U8", [3], bytes([7, 8, 9])), ("e5", "F8_E5M2", [50], e5.view(torch.uint8).numpy().tobytes()),
                      ("i8", "I8", [21], i8.numpy().tobytes()), ("h", "F16", [13, 3], h.numpy().tobytes())], pad_to=1)
    ref8 = {"u": torch.tensor([7, 8, 9], dtype=torch.uint8), "e5": e5, "i8": i8, "h": h}
    loader.reset()
    loader.add_filenames({0: [path8]})
    bufs = loader.copy_files_to_device(dtype=DType.F8_E4M3)
    for k, t in ref8.items():
        got = bufs.get_tensor(k)
        assert got.dtype == torch.float8_e4m3fn and got.shape == t.shape, k
        assert torch.equal(got.view(torch.uint8).cpu(), t.to(DEV).to(torch.float8_e4m3fn).view(torch.uint8).cpu()), k
    bufs.close()
    loader.close()
    assert_clean()


def test_two_batches_of_files_in_flight(data_dir):
    """start_copy / finish: the second batch's reads are queued before the first is waited for (what
    ParallelLoader does between batches).  Each batch is complete when its finish() returns -- compared
    byte for byte with the stock loader right then, while the other batch may still be on its way."""
    cfg = ck.configs(0.05)["C3"]
    files = [r["path"] for r in ck.write_config(cfg, os.path.join(data_dir, "two_batches"))]
    assert len(files) >= 4
    loader = SafeTensorsFileLoader(SingleGroup(), DEV, max_threads=8)
    pending = []
    for batch in (files[:2], files[2:4]):
        loader.add_filenames({0: batch})
        pending.append((batch, loader.start_copy()))
        loader.reset()
    for batch, p in pending:
        bufs = p.finish()
        for path in batch:
            for key, want in load_file(path).items():
                got = bufs.get_tensor(key)
                assert np.array_equal(dev_bytes(got), want.reshape(-1).view(torch.uint8).numpy()), key
        bufs.close()
    # an abandoned batch leaves nothing behind
    loader.add_filenames({0: files[:1]})
    loader.start_copy().abandon()
    loader.close()
    assert_clean()
