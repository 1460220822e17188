# SPDX-License-Identifier: Apache-2.0
"""Host-side logic of the copy pipeline, without a GPU.

``tests/hostsim`` links ``fstx_pipeline.cpp`` -- the very source that ships in
libfstx.so -- against an in-memory stand-in for the GPU runtime whose streams
run late and in order.  These tests drive that build through the C ABI: request
splitting, ring reuse, every read mode, error paths, and the same under the
thread and address sanitizers.
"""
import ctypes
import os
import subprocess

import numpy as np
import pytest

from fastsafetensors_amd import _native

HERE = os.path.dirname(os.path.abspath(__file__))
SIM_DIR = os.path.join(HERE, "hostsim")
PIPELINE_SYMBOLS = [
    n for n in _native.EXPORTED_SYMBOLS if not ("realign" in n or "slice" in n or "convert" in n or "join" in n)
]


@pytest.fixture(scope="module")
def sim():
    # the tests count pinned allocations: no ring stays parked between contexts unless a test asks for it
    parked_before = os.environ.get("FSTX_RING_CACHE")
    os.environ["FSTX_RING_CACHE"] = "0"
    if not os.path.exists(os.path.join(SIM_DIR, "libfstx_hostsim.so")):
        subprocess.run(["make", "-s", "-C", SIM_DIR], check=True)
    lib = ctypes.CDLL(os.path.join(SIM_DIR, "libfstx_hostsim.so"))
    for name in PIPELINE_SYMBOLS:
        restype, argtypes = _native._SIGNATURES[name]
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = restype, argtypes
    lib.fstx_sim_set_copy_delay_us.argtypes = [ctypes.c_int]
    lib.fstx_sim_fail_copy_after.argtypes = [ctypes.c_int64]
    lib.fstx_sim_pinned_live.restype = ctypes.c_int64
    lib.fstx_sim_stream_create.restype = ctypes.c_void_p
    lib.fstx_sim_stream_destroy.argtypes = [ctypes.c_void_p]
    lib.fstx_sim_stream_sleep_then_set.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_int]
    lib.fstx_sim_set_host_alloc_delay_us.argtypes = [ctypes.c_int]
    lib.fstx_sim_fail_host_allocs.argtypes = [ctypes.c_int]
    lib.fstx_sim_set_copy_delay_us(30)
    yield lib
    lib.fstx_trim_cache()
    if parked_before is None:
        os.environ.pop("FSTX_RING_CACHE", None)
    else:
        os.environ["FSTX_RING_CACHE"] = parked_before


@pytest.fixture(scope="module")
def blob(tmp_path_factory):
    path = str(tmp_path_factory.mktemp("sim") / "blob.bin")
    data = np.random.default_rng(1).integers(0, 256, 9_000_011, dtype=np.uint8)
    data.tofile(path)
    return path, data


def make_ctx(sim, **kw):
    cfg = make_cfg(**kw)
    ctx = ctypes.c_void_p()
    rc = (sim.fstx_ctx_acquire if kw.get("shared") else sim.fstx_ctx_create)(ctypes.byref(cfg), ctypes.byref(ctx))
    assert rc == 0, rc
    return ctx


def make_cfg(**kw):
    return _native.FstxConfig(ctypes.sizeof(_native.FstxConfig), 0, -1, kw.get("threads", 4), kw.get("streams", 2),
                              kw.get("block", 64 * 1024), kw.get("slots", 2), kw.get("depth", 0),
                              kw.get("direct_bytes", 0), kw.get("flags", 0), kw.get("ramp_kb", 0))


def metrics(sim, ctx):
    m = _native.FstxMetrics()
    assert sim.fstx_get_metrics(ctx, ctypes.byref(m)) == 0
    return m


@pytest.mark.parametrize("mode", [_native.READ_AUTO, _native.READ_BUFFERED, _native.READ_DIRECT])
@pytest.mark.parametrize("block,threads,slots,direct_bytes,flags", [
    (4096, 3, 1, 4096, 0), (64 * 1024, 4, 2, 0, 1), (1 << 20, 8, 2, 3 << 20, 0), (4 << 20, 2, 3, 0, 0), (8192, 5, 1, 1 << 20, 1)])
def test_random_spans_land_byte_exact(sim, blob, mode, block, threads, slots, direct_bytes, flags):
    path, data = blob
    ctx = make_ctx(sim, block=block, threads=threads, slots=slots, direct_bytes=direct_bytes, flags=flags)
    f = sim.fstx_file_open(ctx, path.encode(), mode)
    assert f >= 1
    rng = np.random.default_rng(block + threads)
    dev = np.full(data.size + 100, 0xEE, dtype=np.uint8)
    spans, at = [], 0
    while at < data.size:
        n = int(rng.integers(1, data.size // 7))
        n = min(n, data.size - at)
        spans.append((at, n, sim.fstx_submit_read(ctx, f, at, n, dev.ctypes.data, dev.size, at + 13)))
        at += n
    for _, n, req in spans:
        assert req >= 1
        assert sim.fstx_wait_read(ctx, req) == n
    assert np.array_equal(dev[13 : 13 + data.size], data)
    assert (dev[:13] == 0xEE).all() and (dev[13 + data.size :] == 0xEE).all()
    m = metrics(sim, ctx)
    assert m.bytes_read == data.size and m.bytes_copied == data.size
    if mode == _native.READ_BUFFERED:
        assert m.blocks_direct == 0
    assert m.bounce_buffer_bytes == threads * slots * (block + 4096)
    assert sim.fstx_bounce_buffer_bytes() == m.bounce_buffer_bytes
    assert sim.fstx_file_close(ctx, f) == 0
    assert sim.fstx_ctx_destroy(ctx) == 0
    assert sim.fstx_bounce_buffer_bytes() == 0 and sim.fstx_sim_pinned_live() == 0


def test_unaligned_window_start_and_zero_length(sim, blob):
    path, data = blob
    ctx = make_ctx(sim, block=8192)
    f = sim.fstx_file_open(ctx, path.encode(), _native.READ_DIRECT)
    dev = np.zeros(50_000, dtype=np.uint8)
    for off, n in [(1, 1), (4095, 2), (4097, 8191), (10, 40_000), (data.size - 5, 5), (0, 0)]:
        dev[:] = 0
        req = sim.fstx_submit_read(ctx, f, off, n, dev.ctypes.data, dev.size, 3)
        assert sim.fstx_wait_read(ctx, req) == n
        assert np.array_equal(dev[3 : 3 + n], data[off : off + n])
        assert not dev[3 + n :].any()
    sim.fstx_file_close(ctx, f)
    sim.fstx_ctx_destroy(ctx)


def test_error_paths(sim, blob, tmp_path):
    path, data = blob
    ctx = make_ctx(sim)
    dev = np.zeros(1 << 20, dtype=np.uint8)
    assert sim.fstx_file_open(ctx, b"/nonexistent/file", 0) == -2  # -ENOENT
    assert "No such file" in sim.fstx_strerror(-2).decode()
    f = sim.fstx_file_open(ctx, path.encode(), 0)
    # destination range must fit the device buffer (std::out_of_range in the reference, ext.hpp:139-146)
    assert sim.fstx_submit_read(ctx, f, 0, 2000, dev.ctypes.data, 1000, 0) == -_native_code("RANGE")
    assert sim.fstx_submit_read(ctx, f, 0, 10, dev.ctypes.data, 1000, 995) == -_native_code("RANGE")
    # reading past the end of the file fails at wait, never silently
    req = sim.fstx_submit_read(ctx, f, data.size - 10, 20, dev.ctypes.data, dev.size, 0)
    assert req >= 1 and sim.fstx_wait_read(ctx, req) == -_native_code("SHORT_READ")
    assert sim.fstx_wait_read(ctx, req) == -_native_code("NO_REQ")  # ids are consumed
    assert sim.fstx_submit_read(ctx, 999, 0, 10, dev.ctypes.data, dev.size, 0) == -_native_code("NO_REQ")
    # file shrinks after open: the worker sees the short read
    cut = str(tmp_path / "cut.bin")
    data[:300_000].tofile(cut)
    g = sim.fstx_file_open(ctx, cut.encode(), _native.READ_BUFFERED)
    os.truncate(cut, 100_000)
    req = sim.fstx_submit_read(ctx, g, 0, 300_000, dev.ctypes.data, dev.size, 0)
    assert sim.fstx_wait_read(ctx, req) == -_native_code("SHORT_READ")
    # a close with a request outstanding is refused
    req = sim.fstx_submit_read(ctx, f, 0, 100_000, dev.ctypes.data, dev.size, 0)
    assert sim.fstx_file_close(ctx, f) == -16  # -EBUSY
    assert sim.fstx_wait_read(ctx, req) == 100_000
    assert sim.fstx_file_close(ctx, f) == 0 and sim.fstx_file_close(ctx, f) == -_native_code("NO_REQ")
    # a failing device copy surfaces at wait
    f = sim.fstx_file_open(ctx, path.encode(), _native.READ_BUFFERED)
    sim.fstx_sim_fail_copy_after(3)
    req = sim.fstx_submit_read(ctx, f, 0, 1 << 20, dev.ctypes.data, dev.size, 0)
    assert sim.fstx_wait_read(ctx, req) == -_native_code("HIP")
    sim.fstx_sim_fail_copy_after(-1)
    req = sim.fstx_submit_read(ctx, f, 0, 1 << 20, dev.ctypes.data, dev.size, 0)
    assert sim.fstx_wait_read(ctx, req) == 1 << 20 and np.array_equal(dev, data[: 1 << 20])
    assert sim.fstx_ctx_destroy(ctx) == 0  # also closes the file left open
    assert sim.fstx_bounce_buffer_bytes() == 0
    # bad configurations
    bad = _native.FstxConfig(ctypes.sizeof(_native.FstxConfig), 0, -1, 4, 2, 1000, 2, 0, 0, 0, 0)  # block not a multiple of 4096
    out = ctypes.c_void_p()
    assert sim.fstx_ctx_create(ctypes.byref(bad), ctypes.byref(out)) == -_native_code("INVAL")
    bad = _native.FstxConfig(ctypes.sizeof(_native.FstxConfig), 7, -1, 4, 2, 4096, 2, 0, 0, 0, 0)  # no such device
    assert sim.fstx_ctx_create(ctypes.byref(bad), ctypes.byref(out)) == -_native_code("INVAL")


def _native_code(name: str) -> int:
    return {"INVAL": 10001, "HIP": 10002, "RANGE": 10003, "SHORT_READ": 10004, "NO_REQ": 10005,
            "CLOSED": 10006, "NO_DEVICE": 10007, "TOO_MANY": 10008}[name]


def test_context_built_behind_the_callers_back(sim, blob):
    """FSTX_CREATE_ASYNC: create returns before ring, streams and workers exist (here the pinned
    allocation takes 400 ms); files are opened and reads queued meanwhile, and the wait delivers
    the bytes once the build is through.  The same configuration without the flag names the same
    shared context."""
    path, data = blob
    import time

    sim.fstx_sim_set_host_alloc_delay_us(400_000)
    try:
        t0 = time.perf_counter()
        ctx = make_ctx(sim, block=64 * 1024, flags=_native.CREATE_ASYNC)
        f = sim.fstx_file_open(ctx, path.encode(), _native.READ_BUFFERED)
        dev = np.zeros(data.size, dtype=np.uint8)
        req = sim.fstx_submit_read(ctx, f, 0, data.size, dev.ctypes.data, dev.size, 0)
        queued_after = time.perf_counter() - t0
        assert req >= 1 and queued_after < 0.3, queued_after  # nothing waited for the build
        assert sim.fstx_wait_read(ctx, req) == data.size
        assert time.perf_counter() - t0 >= 0.4
        assert np.array_equal(dev, data)
        m = metrics(sim, ctx)
        assert m.create_ns >= 400_000_000 and m.bytes_copied == data.size
        assert sim.fstx_file_close(ctx, f) == 0
        # destroying a context right after asking for it waits for the build, then takes it apart
        other = make_ctx(sim, block=8192, flags=_native.CREATE_ASYNC)
        assert sim.fstx_ctx_destroy(other) == 0
        assert sim.fstx_ctx_destroy(ctx) == 0
        assert sim.fstx_bounce_buffer_bytes() == 0 and sim.fstx_sim_pinned_live() == 0
    finally:
        sim.fstx_sim_set_host_alloc_delay_us(0)
    a = make_ctx(sim, block=16384, flags=_native.CREATE_ASYNC, shared=True)
    b = make_ctx(sim, block=16384, flags=0, shared=True)
    assert a.value == b.value
    assert sim.fstx_ctx_release(a) == 0 and sim.fstx_ctx_release(b) == 0
    assert sim.fstx_bounce_buffer_bytes() == 0


def test_a_failed_build_is_reported_by_whoever_waits(sim, blob):
    """The pinned allocation fails.  Built by the creator, fstx_ctx_create returns the error and
    leaves nothing behind; built behind the caller's back, the reads that were queued meanwhile
    fail at their wait, later submits are refused with the same status, and destroy cleans up."""
    path, data = blob
    out = ctypes.c_void_p()
    cfg = make_cfg(block=64 * 1024)
    sim.fstx_sim_fail_host_allocs(1)
    assert sim.fstx_ctx_create(ctypes.byref(cfg), ctypes.byref(out)) == -_native_code("HIP")
    assert not out.value and sim.fstx_bounce_buffer_bytes() == 0 and sim.fstx_sim_pinned_live() == 0
    sim.fstx_sim_set_host_alloc_delay_us(50_000)
    sim.fstx_sim_fail_host_allocs(1)
    try:
        ctx = make_ctx(sim, block=64 * 1024, flags=_native.CREATE_ASYNC)
        f = sim.fstx_file_open(ctx, path.encode(), _native.READ_BUFFERED)
        dev = np.zeros(data.size, dtype=np.uint8)
        reqs = [sim.fstx_submit_read(ctx, f, at, 1 << 20, dev.ctypes.data, dev.size, at) for at in (0, 1 << 20, 2 << 20)]
        assert all(r >= 1 for r in reqs)
        assert [sim.fstx_wait_read(ctx, r) for r in reqs] == [-_native_code("HIP")] * 3
        assert not dev.any()
        assert sim.fstx_submit_read(ctx, f, 0, 4096, dev.ctypes.data, dev.size, 0) == -_native_code("HIP")
        stream = sim.fstx_sim_stream_create()
        flag = ctypes.c_int(0)
        sim.fstx_sim_stream_sleep_then_set(stream, 20_000, ctypes.byref(flag), 1)
        assert sim.fstx_ctx_order_after(ctx, stream) == -_native_code("HIP")
        sim.fstx_sim_stream_destroy(stream)
        assert sim.fstx_file_close(ctx, f) == 0
        assert sim.fstx_ctx_destroy(ctx) == 0
        assert sim.fstx_bounce_buffer_bytes() == 0 and sim.fstx_sim_pinned_live() == 0
    finally:
        sim.fstx_sim_set_host_alloc_delay_us(0)
        sim.fstx_sim_fail_host_allocs(0)


_FAKE_ROCTX = r"""
#include <stdio.h>
#include <string.h>
static __thread int depth;
static int pushes, pops, worst;
static char first[8][160];
int roctxRangePushA(const char *m) { int n = __sync_fetch_and_add(&pushes, 1); if (n < 8) strncpy(first[n], m, 159); if (++depth > worst) worst = depth; return depth; }
int roctxRangePop(void) { __sync_fetch_and_add(&pops, 1); return --depth; }
void fake_roctx_report(int *a, int *b, int *c, char *names) { *a = pushes; *b = pops; *c = worst; names[0] = 0; for (int i = 0; i < 8 && i < pushes; ++i) { strcat(names, first[i]); strcat(names, "|"); } }
"""

_ROCTX_CHECK = r"""
import ctypes, os, sys
import numpy as np
sim = ctypes.CDLL(sys.argv[1]); fake = ctypes.CDLL(sys.argv[2], mode=ctypes.RTLD_GLOBAL); path = sys.argv[3]
from fastsafetensors_amd import _native
cfg = _native.FstxConfig(ctypes.sizeof(_native.FstxConfig), 0, -1, 3, 2, 64 * 1024, 2, 0, 0, int(sys.argv[4]), 0)
ctx = ctypes.c_void_p()
assert sim.fstx_ctx_create(ctypes.byref(cfg), ctypes.byref(ctx)) == 0
sim.fstx_file_open.restype = ctypes.c_int64; sim.fstx_submit_read.restype = ctypes.c_int64; sim.fstx_wait_read.restype = ctypes.c_int64
sim.fstx_file_open.argtypes = [ctypes.c_void_p, ctypes.c_char_p, ctypes.c_int]
sim.fstx_submit_read.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_uint64, ctypes.c_uint64, ctypes.c_void_p, ctypes.c_uint64, ctypes.c_uint64]
sim.fstx_wait_read.argtypes = [ctypes.c_void_p, ctypes.c_int64]
f = sim.fstx_file_open(ctx, path.encode(), 2)
size = os.path.getsize(path)
dev = np.zeros(size, dtype=np.uint8)
req = sim.fstx_submit_read(ctx, f, 0, size, dev.ctypes.data, size, 0)
assert sim.fstx_wait_read(ctx, req) == size
assert np.array_equal(dev, np.fromfile(path, dtype=np.uint8))
sim.fstx_ctx_destroy.argtypes = [ctypes.c_void_p]; sim.fstx_ctx_destroy(ctx)
a, b, c = ctypes.c_int(), ctypes.c_int(), ctypes.c_int(); names = ctypes.create_string_buffer(2000)
fake.fake_roctx_report(ctypes.byref(a), ctypes.byref(b), ctypes.byref(c), names)
print(a.value, b.value, c.value, names.value.decode())
"""


def test_profiler_ranges_are_named_and_balanced(sim, blob, tmp_path):
    """FSTX_ROCTX=1: the library loads a roctx library by itself and brackets the build of the reader,
    every submit, every wait and every O_DIRECT read with a named range; pushes and pops balance on
    every thread.  Without the switch nothing is loaded and nothing is called.  (A counting stand-in
    for libroctx64.so, in a process of its own: the switch is read once.)"""
    import sys

    path, _data = blob
    src = tmp_path / "fake_roctx.c"
    src.write_text(_FAKE_ROCTX)
    lib = str(tmp_path / "libfake_roctx.so")
    subprocess.run(["gcc", "-shared", "-fPIC", "-O1", "-o", lib, str(src)], check=True)
    root = os.path.dirname(HERE)
    for flags in (0, _native.CREATE_ASYNC):
        for switch, expect_calls in (("1", True), ("0", False)):
            env = dict(os.environ, FSTX_ROCTX=switch, FSTX_ROCTX_LIB=lib, PYTHONPATH=root)
            out = subprocess.run([sys.executable, "-c", _ROCTX_CHECK, os.path.join(SIM_DIR, "libfstx_hostsim.so"), lib, path, str(flags)],
                                 env=env, capture_output=True, text=True, timeout=120)
            assert out.returncode == 0, out.stderr
            pushes, pops, worst, names = (out.stdout.strip() + " ").split(" ", 3)
            if not expect_calls:
                assert (pushes, pops) == ("0", "0")
                continue
            assert int(pushes) == int(pops) >= 4 and int(worst) >= 1
            assert "fstx build reader: 3 threads, 2 streams" in names and "fstx submit_read file 1" in names
            assert "fstx wait_read request 1" in names or int(pushes) > 8


def test_injected_read_fault(sim, blob):
    path, data = blob
    os.environ["FSTX_FAULT_READ_AFTER"] = "5"
    try:
        ctx = make_ctx(sim, block=64 * 1024)
    finally:
        del os.environ["FSTX_FAULT_READ_AFTER"]
    f = sim.fstx_file_open(ctx, path.encode(), _native.READ_BUFFERED)
    dev = np.zeros(data.size, dtype=np.uint8)
    req = sim.fstx_submit_read(ctx, f, 0, data.size, dev.ctypes.data, dev.size, 0)
    assert sim.fstx_wait_read(ctx, req) == -5  # -EIO from the sixth block
    req = sim.fstx_submit_read(ctx, f, 0, data.size, dev.ctypes.data, dev.size, 0)
    assert sim.fstx_wait_read(ctx, req) == data.size and np.array_equal(dev, data)
    sim.fstx_ctx_destroy(ctx)


def test_direct_reads_fail_cleanly(sim, blob, tmp_path):
    """The same failures on the O_DIRECT path, where one read stages many blocks that other
    workers ship: an injected read error, a failing device copy while staged blocks are in
    flight, a file that ends early, and a destroy with staged work outstanding."""
    path, data = blob
    dev = np.zeros(data.size, dtype=np.uint8)
    # injected read error: the second large read fails, every block of it reports -EIO
    os.environ["FSTX_FAULT_READ_AFTER"] = "1"
    try:
        ctx = make_ctx(sim, block=64 * 1024, threads=4, direct_bytes=16 * 64 * 1024)
    finally:
        del os.environ["FSTX_FAULT_READ_AFTER"]
    f = sim.fstx_file_open(ctx, path.encode(), _native.READ_DIRECT)
    req = sim.fstx_submit_read(ctx, f, 0, data.size, dev.ctypes.data, dev.size, 0)
    assert sim.fstx_wait_read(ctx, req) == -5
    req = sim.fstx_submit_read(ctx, f, 0, data.size, dev.ctypes.data, dev.size, 0)
    assert sim.fstx_wait_read(ctx, req) == data.size and np.array_equal(dev, data)
    m = _native.FstxMetrics()
    assert sim.fstx_get_metrics(ctx, ctypes.byref(m)) == 0
    if m.direct_fallbacks == 0:  # the filesystem took O_DIRECT: the blocks went through the staged queue
        assert m.blocks_direct > 0 and m.stage_ns > 0
    # a failing device copy while staged blocks are being shipped
    dev[:] = 0
    sim.fstx_sim_fail_copy_after(7)
    req = sim.fstx_submit_read(ctx, f, 0, data.size, dev.ctypes.data, dev.size, 0)
    assert sim.fstx_wait_read(ctx, req) == -_native_code("HIP")
    sim.fstx_sim_fail_copy_after(-1)
    req = sim.fstx_submit_read(ctx, f, 4096, 1 << 20, dev.ctypes.data, dev.size, 4096)
    assert sim.fstx_wait_read(ctx, req) == 1 << 20 and np.array_equal(dev[4096 : 4096 + (1 << 20)], data[4096 : 4096 + (1 << 20)])
    # a file that ends inside a large read
    cut = str(tmp_path / "cut.bin")
    data[:600_000].tofile(cut)
    g = sim.fstx_file_open(ctx, cut.encode(), _native.READ_DIRECT)
    os.truncate(cut, 200_000)
    req = sim.fstx_submit_read(ctx, g, 0, 600_000, dev.ctypes.data, dev.size, 0)
    assert sim.fstx_wait_read(ctx, req) == -_native_code("SHORT_READ")
    # destroy with direct requests outstanding: drains, leaves nothing behind
    sim.fstx_sim_set_copy_delay_us(300)
    dev[:] = 0
    for k in range(3):
        assert sim.fstx_submit_read(ctx, f, k * (1 << 20), 1 << 20, dev.ctypes.data, dev.size, k * (1 << 20)) >= 1
    assert sim.fstx_ctx_destroy(ctx) == 0
    sim.fstx_sim_set_copy_delay_us(30)
    assert np.array_equal(dev[: 3 << 20], data[: 3 << 20])
    assert sim.fstx_bounce_buffer_bytes() == 0 and sim.fstx_sim_pinned_live() == 0


def test_destroy_with_requests_in_flight(sim, blob):
    path, data = blob
    sim.fstx_sim_set_copy_delay_us(300)
    ctx = make_ctx(sim, block=4096, threads=2)
    f = sim.fstx_file_open(ctx, path.encode(), _native.READ_BUFFERED)
    dev = np.zeros(data.size, dtype=np.uint8)
    for k in range(4):
        assert sim.fstx_submit_read(ctx, f, k * 100_000, 100_000, dev.ctypes.data, dev.size, k * 100_000) >= 1
    assert sim.fstx_ctx_destroy(ctx) == 0  # drains, never leaves a copy behind
    sim.fstx_sim_set_copy_delay_us(30)
    assert np.array_equal(dev[:400_000], data[:400_000])
    assert sim.fstx_bounce_buffer_bytes() == 0


def test_shared_contexts_are_counted(sim, blob):
    """fstx_ctx_acquire: equal configurations share one context, the last release frees it."""
    path, data = blob
    a = make_ctx(sim, shared=True, threads=3)
    b = make_ctx(sim, shared=True, threads=3)
    c = make_ctx(sim, shared=True, threads=2)
    private = make_ctx(sim, threads=3)
    assert a.value == b.value and c.value != a.value and private.value != a.value
    ring = lambda t: t * 2 * (64 * 1024 + 4096)
    assert sim.fstx_bounce_buffer_bytes() == ring(3) + ring(2) + ring(3)
    # two users at once, from two threads
    import threading
    devs = [np.zeros(data.size, dtype=np.uint8) for _ in range(2)]
    def user(ctx, dev):
        f = sim.fstx_file_open(ctx, path.encode(), _native.READ_BUFFERED)
        req = sim.fstx_submit_read(ctx, f, 0, data.size, dev.ctypes.data, dev.size, 0)
        assert sim.fstx_wait_read(ctx, req) == data.size
        assert sim.fstx_file_close(ctx, f) == 0
    ts = [threading.Thread(target=user, args=(ctx, dev)) for ctx, dev in zip((a, b), devs)]
    [t.start() for t in ts]
    [t.join() for t in ts]
    assert all(np.array_equal(d, data) for d in devs)
    assert sim.fstx_ctx_release(a) == 0
    assert sim.fstx_bounce_buffer_bytes() == ring(3) + ring(2) + ring(3)  # b still holds it
    dev = np.zeros(1000, dtype=np.uint8)
    f = sim.fstx_file_open(b, path.encode(), _native.READ_BUFFERED)
    assert sim.fstx_wait_read(b, sim.fstx_submit_read(b, f, 5, 1000, dev.ctypes.data, 1000, 0)) == 1000
    assert np.array_equal(dev, data[5:1005])
    assert sim.fstx_ctx_release(b) == 0 and sim.fstx_ctx_release(c) == 0
    assert sim.fstx_ctx_release(private) == 0  # a private context: release destroys it
    assert sim.fstx_bounce_buffer_bytes() == 0 and sim.fstx_sim_pinned_live() == 0
    # after the last release the next acquire builds a new context
    d = make_ctx(sim, shared=True, threads=3)
    assert sim.fstx_ctx_release(d) == 0 and sim.fstx_bounce_buffer_bytes() == 0


def test_order_after_holds_the_copies_back(sim, blob):
    """fstx_ctx_order_after: copies of later requests start only when the work that was
    queued on the caller's stream at the call has run."""
    path, data = blob
    ctx = make_ctx(sim, threads=3, streams=3)
    f = sim.fstx_file_open(ctx, path.encode(), _native.READ_BUFFERED)
    theirs = sim.fstx_sim_stream_create()
    flag = ctypes.c_int(0)
    dev = np.zeros(200_000, dtype=np.uint8)
    sim.fstx_sim_stream_sleep_then_set(theirs, 150_000, ctypes.byref(flag), 7)
    assert sim.fstx_ctx_order_after(ctx, theirs) == 0
    req = sim.fstx_submit_read(ctx, f, 0, dev.size, dev.ctypes.data, dev.size, 0)
    import time
    time.sleep(0.05)
    assert flag.value == 0 and not dev.any()  # the reads are done by now, the copies still wait
    assert sim.fstx_wait_read(ctx, req) == dev.size
    assert flag.value == 7 and np.array_equal(dev, data[: dev.size])
    # work queued on their stream after the call does not hold anything back
    sim.fstx_sim_stream_sleep_then_set(theirs, 400_000, ctypes.byref(flag), 9)
    req = sim.fstx_submit_read(ctx, f, 10, 1000, dev.ctypes.data, dev.size, 0)
    assert sim.fstx_wait_read(ctx, req) == 1000 and flag.value == 7
    assert sim.fstx_ctx_order_after(None, theirs) == -_native_code("INVAL")
    sim.fstx_sim_stream_destroy(theirs)  # joins the stream's thread: flag is 9 afterwards
    assert flag.value == 9
    sim.fstx_ctx_destroy(ctx)


def test_wait_covers_its_own_request_while_later_ones_keep_the_streams_busy(sim, blob):
    """A caller may queue the next file's reads before it waits for this one's: the wait returns
    when this request's bytes are in place, neither earlier nor only when the streams run dry."""
    import time
    path, data = blob
    sim.fstx_sim_set_copy_delay_us(400)
    try:
        ctx = make_ctx(sim, threads=4, streams=2, block=64 * 1024)
        f = sim.fstx_file_open(ctx, path.encode(), _native.READ_BUFFERED)
        first = np.zeros(1_000_000, dtype=np.uint8)
        later = np.zeros(8_000_000, dtype=np.uint8)
        a = sim.fstx_submit_read(ctx, f, 0, first.size, first.ctypes.data, first.size, 0)
        b = sim.fstx_submit_read(ctx, f, first.size, later.size, later.ctypes.data, later.size, 0)
        t0 = time.perf_counter()
        assert sim.fstx_wait_read(ctx, a) == first.size
        t_a = time.perf_counter() - t0
        assert np.array_equal(first, data[: first.size])       # complete the moment the wait returns
        assert not np.array_equal(later, data[first.size : first.size + later.size])  # the later request is still on its way
        assert sim.fstx_wait_read(ctx, b) == later.size
        t_b = time.perf_counter() - t0
        assert np.array_equal(later, data[first.size : first.size + later.size])
        assert t_a < 0.6 * t_b, (t_a, t_b)
        assert sim.fstx_file_close(ctx, f) == 0
        assert sim.fstx_ctx_destroy(ctx) == 0
    finally:
        sim.fstx_sim_set_copy_delay_us(30)


def test_direct_reads_ramp_up_and_down(sim, blob):
    """O_DIRECT runs: small first, growing fourfold to the full size, halving towards the end of
    what is queued; a ramp size at or above the full size keeps every read at full size."""
    path, data = blob
    dev = np.zeros(data.size, dtype=np.uint8)
    counts = {}
    for label, ramp_kb in (("ramped", 64), ("fixed", 4096)):
        ctx = make_ctx(sim, block=64 * 1024, threads=4, direct_bytes=4 << 20, ramp_kb=ramp_kb)
        f = sim.fstx_file_open(ctx, path.encode(), _native.READ_DIRECT)
        dev[:] = 0
        req = sim.fstx_submit_read(ctx, f, 0, data.size, dev.ctypes.data, dev.size, 0)
        assert sim.fstx_wait_read(ctx, req) == data.size and np.array_equal(dev, data)
        m = metrics(sim, ctx)
        counts[label] = (m.direct_reads, m.direct_fallbacks)
        sim.fstx_file_close(ctx, f)
        sim.fstx_ctx_destroy(ctx)
    if counts["fixed"][1] == 0:  # the filesystem took O_DIRECT
        # 9,000,011 bytes in runs of 4 MiB: 3 reads; ramped: 64K, 256K, 1M, then halves of the rest down to 64K
        assert counts["fixed"][0] == 3
        assert 8 <= counts["ramped"][0] <= 14, counts


def test_probe_contexts_leave_out_one_stage(sim, blob):
    path, data = blob
    for mode in (_native.READ_BUFFERED, _native.READ_DIRECT):
        # NO_COPY: the reads run, device memory is not written
        ctx = make_ctx(sim, flags=_native.PROBE_NO_COPY, direct_bytes=1 << 20)
        f = sim.fstx_file_open(ctx, path.encode(), mode)
        dev = np.full(data.size, 0xEE, dtype=np.uint8)
        req = sim.fstx_submit_read(ctx, f, 0, data.size, dev.ctypes.data, dev.size, 0)
        assert sim.fstx_wait_read(ctx, req) == data.size
        m = metrics(sim, ctx)
        assert m.bytes_read == data.size and m.bytes_copied == 0 and (dev == 0xEE).all()
        sim.fstx_ctx_destroy(ctx)
        # NO_READ: every block is copied, no byte comes from the file
        ctx = make_ctx(sim, flags=_native.PROBE_NO_READ, direct_bytes=1 << 20)
        f = sim.fstx_file_open(ctx, path.encode(), mode)
        req = sim.fstx_submit_read(ctx, f, 0, data.size, dev.ctypes.data, dev.size, 0)
        assert sim.fstx_wait_read(ctx, req) == data.size
        m = metrics(sim, ctx)
        assert m.bytes_copied == data.size and m.read_ns < 50_000_000
        sim.fstx_ctx_destroy(ctx)
    bad = make_cfg(flags=64)
    out = ctypes.c_void_p()
    assert sim.fstx_ctx_create(ctypes.byref(bad), ctypes.byref(out)) == -_native_code("INVAL")


def test_auto_mode_reads_cached_stretches_from_the_cache(sim, tmp_path):
    """AUTO: an O_DIRECT run stops at the first block that sits in the page cache."""
    path = str(tmp_path / "partly.bin")
    data = np.random.default_rng(5).integers(0, 256, 6 << 20, dtype=np.uint8)
    data.tofile(path)
    fd = os.open(path, os.O_RDONLY)
    os.fsync(fd)
    os.posix_fadvise(fd, 0, 0, os.POSIX_FADV_DONTNEED)
    os.pread(fd, 2 << 20, 2 << 20)  # the middle third becomes resident
    os.close(fd)
    ctx = make_ctx(sim, block=256 * 1024, threads=3, direct_bytes=16 << 20, ramp_kb=16 << 10)
    f = sim.fstx_file_open(ctx, path.encode(), _native.READ_AUTO)
    dev = np.zeros(data.size, dtype=np.uint8)
    req = sim.fstx_submit_read(ctx, f, 0, data.size, dev.ctypes.data, dev.size, 0)
    assert sim.fstx_wait_read(ctx, req) == data.size and np.array_equal(dev, data)
    m = metrics(sim, ctx)
    if m.blocks_direct:  # the filesystem took O_DIRECT and the drop emptied the cache
        # (read-ahead may have pulled in a little more than the 2 MiB that were read)
        assert 8 <= m.blocks_buffered <= 14 and m.blocks_direct + m.blocks_buffered == 24, (m.blocks_direct, m.blocks_buffered)
        assert m.direct_reads == 2
    sim.fstx_ctx_destroy(ctx)


@pytest.mark.parametrize("binary", ["hostsim_tsan.bin", "hostsim_asan.bin"])
def test_pipeline_under_sanitizers(blob, binary):
    exe = os.path.join(SIM_DIR, binary)
    if not os.path.exists(exe):
        subprocess.run(["make", "-s", "-C", SIM_DIR], check=True)
    path, _ = blob
    # every shape twice in a row, so that the second context of a shape takes over the first one's ring
    run = subprocess.run([exe, path, "3"], capture_output=True, text=True, timeout=300, env=dict(os.environ, FSTX_RING_CACHE="1"))
    assert run.returncode == 0, run.stdout + run.stderr
    assert "Sanitizer" not in run.stderr, run.stderr
    assert "hostsim_driver: ok" in run.stdout


def test_ring_is_parked_for_the_next_context(sim, blob, monkeypatch):
    """The ring of the context destroyed last is taken over by the next context of the same shape:
    one allocation fewer, nothing counted as a bounce buffer meanwhile, freed by a trim, replaced by
    the ring of a context of another shape, and never parked when the environment says no."""
    path, data = blob
    monkeypatch.setenv("FSTX_RING_CACHE", "1")
    ring = lambda threads, block=64 * 1024: threads * 2 * (block + 4096)

    def load(ctx):
        f = sim.fstx_file_open(ctx, path.encode(), _native.READ_BUFFERED)
        dev = np.zeros(data.size, dtype=np.uint8)
        req = sim.fstx_submit_read(ctx, f, 0, data.size, dev.ctypes.data, dev.size, 0)
        assert sim.fstx_wait_read(ctx, req) == data.size and np.array_equal(dev, data)
        assert sim.fstx_file_close(ctx, f) == 0

    a = make_ctx(sim, threads=3)
    load(a)
    assert metrics(sim, a).ring_reused == 0 and sim.fstx_cached_ring_bytes() == 0
    assert sim.fstx_ctx_destroy(a) == 0
    assert sim.fstx_bounce_buffer_bytes() == 0 and sim.fstx_sim_pinned_live() == 1
    assert sim.fstx_cached_ring_bytes() == ring(3)
    # same shape: taken over, also by a context that is built behind the caller's back
    b = make_ctx(sim, threads=3, flags=_native.CREATE_ASYNC)
    load(b)
    assert metrics(sim, b).ring_reused == 1 and sim.fstx_cached_ring_bytes() == 0
    assert sim.fstx_bounce_buffer_bytes() == ring(3) and sim.fstx_sim_pinned_live() == 1
    # a second one alive at the same time gets a ring of its own; the one destroyed last stays
    c = make_ctx(sim, threads=3)
    assert metrics(sim, c).ring_reused == 0 and sim.fstx_sim_pinned_live() == 2
    load(c)
    assert sim.fstx_ctx_destroy(b) == 0 and sim.fstx_sim_pinned_live() == 2
    assert sim.fstx_ctx_destroy(c) == 0 and sim.fstx_sim_pinned_live() == 1
    # another shape: not taken over; its ring replaces the parked one
    d = make_ctx(sim, threads=2)
    assert metrics(sim, d).ring_reused == 0 and sim.fstx_sim_pinned_live() == 2
    load(d)
    assert sim.fstx_ctx_destroy(d) == 0
    assert sim.fstx_sim_pinned_live() == 1 and sim.fstx_cached_ring_bytes() == ring(2)
    assert sim.fstx_trim_cache() == ring(2) and sim.fstx_trim_cache() == 0
    assert sim.fstx_sim_pinned_live() == 0 and sim.fstx_bounce_buffer_bytes() == 0
    # switched off: freed with its context
    monkeypatch.setenv("FSTX_RING_CACHE", "0")
    e = make_ctx(sim, threads=3)
    load(e)
    assert sim.fstx_ctx_destroy(e) == 0
    assert sim.fstx_sim_pinned_live() == 0 and sim.fstx_cached_ring_bytes() == 0


def test_a_context_that_failed_parks_nothing(sim, monkeypatch):
    monkeypatch.setenv("FSTX_RING_CACHE", "1")
    sim.fstx_sim_fail_host_allocs(1)
    try:
        out = ctypes.c_void_p()
        cfg = make_cfg(threads=3)
        assert sim.fstx_ctx_create(ctypes.byref(cfg), ctypes.byref(out)) < 0
        assert sim.fstx_cached_ring_bytes() == 0 and sim.fstx_sim_pinned_live() == 0
    finally:
        sim.fstx_sim_fail_host_allocs(0)


def test_only_the_first_bytes_of_a_burst_are_cut_small(sim, blob, monkeypatch):
    """Requests are cut into small blocks while little has been submitted since the reader was
    last found idle; what follows in the same burst gets whole blocks.  Counted in blocks: a
    4 MiB limit, 1 MiB small blocks, 4 MiB blocks, one worker whose first copy takes long enough
    for the other submits to find its blocks still queued."""
    path, data = blob
    monkeypatch.setenv("FSTX_SMALL_BURST_MB", "4")
    monkeypatch.setenv("FSTX_SMALL_BLOCK_KB", "1024")
    sim.fstx_sim_set_copy_delay_us(50_000)
    try:
        ctx = make_ctx(sim, block=4 << 20, threads=1, slots=1)
        f = sim.fstx_file_open(ctx, path.encode(), _native.READ_BUFFERED)
        dev = np.zeros(data.size, dtype=np.uint8)
        three = (2 << 20) + (512 << 10)  # (the file has 8.6 MiB)
        reqs = [sim.fstx_submit_read(ctx, f, k * three, three, dev.ctypes.data, dev.size, k * three) for k in range(3)]
        for r in reqs:
            assert sim.fstx_wait_read(ctx, r) == three
        assert np.array_equal(dev[: 3 * three], data[: 3 * three])
        # 2.5 MiB under the limit: blocks of 1, 1 and 0.5 MiB; then 5 and 7.5 MiB submitted: whole blocks,
        # cut on 4 MiB boundaries counted from the start of each request (one block each)
        assert metrics(sim, ctx).blocks_buffered == 3 + 1 + 1
        # idle again: the count starts over
        r = sim.fstx_submit_read(ctx, f, 0, three, dev.ctypes.data, dev.size, 0)
        assert sim.fstx_wait_read(ctx, r) == three
        assert metrics(sim, ctx).blocks_buffered == 5 + 3
        assert sim.fstx_file_close(ctx, f) == 0
        assert sim.fstx_ctx_destroy(ctx) == 0
    finally:
        sim.fstx_sim_set_copy_delay_us(30)
