# SPDX-License-Identifier: Apache-2.0
"""Where the I/O side runs and how it shapes its O_DIRECT reads, without a GPU.

The reference pins the whole process to the GPU's NUMA node once
(``fastsafetensors/loader.py:75-81`` -> ``set_numa_node``, ``cpp/ext.cpp:525-533``, node
looked up in ``common.py:40-51``).  Here the pipeline binds its own threads and places its
ring; these tests read the binding back from the operating system (the affinity of every
thread of the process, the node of the ring's page), run the ``cpulist`` parser over a sysfs
tree they lay out themselves, and check that a binding that fails is reported, not swallowed.

The second half gives the pipeline block devices of its own making (a sysfs tree again) and a
storage model behind its O_DIRECT reads, and checks the request shape it settles on.

Everything runs against ``tests/hostsim`` (the shipped pipeline source over an in-memory device).
"""
import ctypes
import errno
import os
import subprocess
import threading
import time

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
    # no ring stays parked between the contexts of these tests
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
    lib.fstx_sim_set_storage.argtypes = [ctypes.c_int, ctypes.c_double, ctypes.c_int]
    lib.fstx_sim_set_copy_delay_us(0)
    yield lib
    lib.fstx_sim_set_storage(0, 0.0, 0)
    lib.fstx_sim_set_copy_delay_us(30)
    lib.fstx_trim_cache()
    if parked_before is None:
        os.environ.pop("FSTX_RING_CACHE", None)
    else:
        os.environ["FSTX_RING_CACHE"] = parked_before


class env:
    """Environment variables for the duration of a block (the library reads them per call)."""

    def __init__(self, **kv):
        self.kv = kv

    def __enter__(self):
        self.old = {k: os.environ.get(k) for k in self.kv}
        os.environ.update({k: str(v) for k, v in self.kv.items()})

    def __exit__(self, *exc):
        for k, v in self.old.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v


def make_ctx(sim, node=-1, threads=4, block=64 * 1024, depth=0, direct_bytes=0, flags=0, ramp_kb=0, streams=2):
    cfg = _native.FstxConfig(ctypes.sizeof(_native.FstxConfig), 0, node, threads, streams, block, 2, depth, direct_bytes, flags, ramp_kb)
    ctx = ctypes.c_void_p()
    rc = sim.fstx_ctx_create(ctypes.byref(cfg), ctypes.byref(ctx))
    assert rc == 0, rc
    return ctx


def metrics(sim, ctx):
    m = _native.FstxMetrics()
    assert sim.fstx_get_metrics(ctx, ctypes.byref(m)) == 0
    return m


def node_cpus(sim, node):
    buf = (ctypes.c_int * 1024)()
    n = sim.fstx_node_cpus(node, buf, len(buf))
    return n if n < 0 else list(buf[:n])


def write(path, text):
    os.makedirs(os.path.dirname(path), exist_ok=True)
    with open(path, "w") as f:
        f.write(text)


def thread_affinities():
    out = {}
    for tid in os.listdir("/proc/self/task"):
        try:
            out[int(tid)] = frozenset(os.sched_getaffinity(int(tid)))
        except ProcessLookupError:
            pass
    return out


# ---- the cpulist parser ----------------------------------------------------------------------


@pytest.mark.parametrize("text,want", [
    ("0-3,8,10-11\n", [0, 1, 2, 3, 8, 10, 11]),
    ("5\n", [5]),
    ("0-1", [0, 1]),
    ("2,4,6-6,9-10\n", [2, 4, 6, 9, 10]),
    ("0-15,32-47\n", list(range(16)) + list(range(32, 48))),
    ("\n", -errno.ENODEV),
    ("x\n", -errno.ENODEV),
])
def test_cpulist_parser_through_a_sysfs_root(sim, tmp_path, text, want):
    write(str(tmp_path / "devices/system/node/node3/cpulist"), text)
    with env(FSTX_SYSFS_ROOT=tmp_path):
        assert node_cpus(sim, 3) == want
        assert node_cpus(sim, 4) == -errno.ENODEV  # no such node in this tree
        buf = (ctypes.c_int * 2)()
        if isinstance(want, list):  # a short buffer gets the first CPUs, the count is still the node's
            assert sim.fstx_node_cpus(3, buf, 2) == len(want) and list(buf[: min(2, len(want))]) == want[:2]
    assert sim.fstx_node_cpus(-1, None, 0) == -10001


def test_node_cpus_of_this_machine_match_sysfs(sim):
    with open("/sys/devices/system/node/node0/cpulist") as f:
        text = f.read().strip()
    want = []
    for part in text.split(","):
        lo, _, hi = part.partition("-")
        want += list(range(int(lo), int(hi or lo) + 1))
    assert node_cpus(sim, 0) == want


# ---- binding, read back from the operating system ---------------------------------------------------


def test_workers_and_ring_sit_on_the_node_and_the_caller_is_left_alone(sim, tmp_path):
    """A node made of two of this process's CPUs (so that being bound to it is visible): every
    worker's affinity, read with sched_getaffinity per thread id, is exactly those two; the
    calling thread keeps its own; the ring's first page lies on node 0 (the only memory node
    here, and the policy names it)."""
    allowed = sorted(os.sched_getaffinity(0))
    if len(allowed) < 3:
        pytest.skip("needs three CPUs to tell a bound thread from an unbound one")
    subset = allowed[1:3]
    write(str(tmp_path / "devices/system/node/node0/cpulist"), ",".join(map(str, subset)) + "\n")
    before = thread_affinities()
    mine = frozenset(os.sched_getaffinity(0))
    with env(FSTX_SYSFS_ROOT=tmp_path):
        ctx = make_ctx(sim, node=0, threads=5)
        m = metrics(sim, ctx)
    assert (m.numa_node, m.workers_on_node, m.bind_errors, m.first_bind_error) == (0, 5, 0, 0)
    assert m.ring_node == 0
    after = thread_affinities()
    bound = [tid for tid, cpus in after.items() if tid not in before and cpus == frozenset(subset)]
    assert len(bound) == 5, (len(bound), after)
    assert frozenset(os.sched_getaffinity(0)) == mine  # the caller's own affinity is untouched
    assert all(after[tid] == cpus for tid, cpus in before.items() if tid in after)
    assert sim.fstx_ctx_destroy(ctx) == 0
    # without a node nothing is bound and nothing is claimed
    ctx = make_ctx(sim, node=-1, threads=3)
    m = metrics(sim, ctx)
    assert (m.numa_node, m.workers_on_node, m.bind_errors, m.ring_node) == (-1, 0, 0, -1)
    assert sim.fstx_ctx_destroy(ctx) == 0


def test_a_binding_that_fails_is_reported(sim, tmp_path):
    """Node 7 has CPUs in this tree but no memory in this machine: the affinity takes, the memory
    policy is refused (EINVAL), and the context says so for every thread that tried.  Node 9 has
    no cpulist at all: ENODEV, nobody is bound."""
    allowed = sorted(os.sched_getaffinity(0))
    write(str(tmp_path / "devices/system/node/node7/cpulist"), f"{allowed[0]}\n")
    if os.path.exists("/sys/devices/system/node/node7"):
        pytest.skip("this machine has a node 7")
    with env(FSTX_SYSFS_ROOT=tmp_path):
        ctx = make_ctx(sim, node=7, threads=3)
        m = metrics(sim, ctx)
        assert m.workers_on_node == 3 and m.bind_errors == 4 and m.first_bind_error == -errno.EINVAL  # 3 workers + the ring's thread
        assert sim.fstx_ctx_destroy(ctx) == 0
        ctx = make_ctx(sim, node=9, threads=3)
        m = metrics(sim, ctx)
        assert m.workers_on_node == 0 and m.bind_errors == 4 and m.first_bind_error == -errno.ENODEV
        assert sim.fstx_ctx_destroy(ctx) == 0
        # the free function reports the same, from a thread of its own (it binds its caller)
        got = {}
        for node in (7, 9):
            t = threading.Thread(target=lambda n=node: got.__setitem__(n, sim.fstx_set_numa_node(n)))
            t.start()
            t.join()
        assert got == {7: -errno.EINVAL, 9: -errno.ENODEV}
    got = {}
    t = threading.Thread(target=lambda: got.__setitem__(0, (sim.fstx_set_numa_node(0), sim.fstx_set_numa_node(-1))))
    t.start()
    t.join()
    assert got[0] == (0, 0)


def test_workers_map_their_slots_before_the_first_request(sim):
    ctx = make_ctx(sim, threads=3, block=256 * 1024)
    deadline = time.time() + 5
    ring = 3 * 2 * (256 * 1024 + 4096)
    while metrics(sim, ctx).pretouched_bytes < ring and time.time() < deadline:
        time.sleep(0.005)
    assert metrics(sim, ctx).pretouched_bytes == ring
    assert sim.fstx_ctx_destroy(ctx) == 0
    ctx = make_ctx(sim, threads=3, block=256 * 1024, flags=_native.NO_PRETOUCH)
    time.sleep(0.02)
    assert metrics(sim, ctx).pretouched_bytes == 0
    assert sim.fstx_ctx_destroy(ctx) == 0


# ---- the shape of the O_DIRECT reads follows the block device ------------------------------------------


@pytest.fixture()
def cold_file(tmp_path):
    path = str(tmp_path / "blob.bin")
    data = np.random.default_rng(3).integers(0, 256, 3_000_000, dtype=np.uint8)
    data.tofile(path)
    return path, data


def device_tree(root, dev, name, nr_requests, max_sectors_kb, rotational=0, partition=False):
    """A block device as sysfs shows it: /sys/dev/block/<maj>:<min> is a link into /sys/devices/...;
    a partition has no queue directory of its own, its parent -- the disk -- has."""
    disk = os.path.join(root, "devices", "pci0000:00", "virtio3" if name.startswith("vd") else "0000:00:04.0", "block", name)
    for key, value in (("nr_requests", nr_requests), ("max_sectors_kb", max_sectors_kb), ("rotational", rotational)):
        write(os.path.join(disk, "queue", key), f"{value}\n")
    target = disk
    if partition:
        target = os.path.join(disk, name + "1")
        os.makedirs(target)
    link = os.path.join(root, "dev", "block", f"{os.major(dev)}:{os.minor(dev)}")
    os.makedirs(os.path.dirname(link), exist_ok=True)
    os.symlink(os.path.relpath(target, os.path.dirname(link)), link)


GIB, MIB = 1 << 30, 1 << 20


@pytest.mark.parametrize("name,nr,kb,rot,part,want", [
    # the disk these loads were tuned on: virtio, 256 requests of 4 MiB = 1 GiB in one read, one at a time
    ("vda", 256, 4096, 0, False, dict(bytes=GIB, depth=1, steered=0, flags=1 | 4)),
    ("vdb", 256, 4096, 0, True, dict(bytes=GIB, depth=1, steered=0, flags=1 | 4)),
    # NVMe, 1023 requests of 1280 KiB: budget capped at 1 GiB, several reads of a quarter of it, steered
    ("nvme0n1", 1023, 1280, 0, False, dict(bytes=256 * MIB, depth=2, steered=1, flags=1)),
    ("nvme1n1", 1023, 1280, 0, True, dict(bytes=256 * MIB, depth=2, steered=1, flags=1)),
    # NVMe with small requests: 1023 x 128 KiB is just under 128 MiB; never below 64 MiB per read
    ("nvme2n1", 1023, 128, 0, False, dict(bytes=64 * MIB, depth=2, steered=1, flags=1)),
    # a rotating disk: one read in flight, of one queue's worth (128 x 512 KiB = 64 MiB)
    ("sda", 128, 512, 1, False, dict(bytes=64 * MIB, depth=1, steered=0, flags=1 | 2)),
])
def test_read_shape_follows_the_block_device(sim, tmp_path, cold_file, name, nr, kb, rot, part, want):
    path, data = cold_file
    root = str(tmp_path / "sys")
    device_tree(root, os.stat(path).st_dev, name, nr, kb, rot, part)
    write(str(tmp_path / "proc/meminfo"), "MemTotal:       263780000 kB\nMemAvailable:   201326592 kB\n")
    with env(FSTX_SYSFS_ROOT=root, FSTX_PROCFS_ROOT=tmp_path / "proc"):
        ctx = make_ctx(sim, block=4 * MIB, threads=16)
        assert metrics(sim, ctx).direct_read_bytes == 0  # nothing settled before a file is known
        f = sim.fstx_file_open(ctx, path.encode(), _native.READ_DIRECT)
        m = metrics(sim, ctx)
        if m.direct_read_bytes == 0:
            pytest.skip("this filesystem refuses O_DIRECT")
        assert (m.direct_read_bytes, m.direct_depth, m.direct_steered, m.storage_flags) == (
            want["bytes"], want["depth"], want["steered"], want["flags"])
        assert (m.storage_nr_requests, m.storage_max_sectors_kb) == (nr, kb)
        # the load itself is unaffected by what the tree claims
        dev = np.zeros(data.size, dtype=np.uint8)
        req = sim.fstx_submit_read(ctx, f, 0, data.size, dev.ctypes.data, dev.size, 0)
        assert sim.fstx_wait_read(ctx, req) == data.size and np.array_equal(dev, data)
        assert sim.fstx_ctx_destroy(ctx) == 0


def test_read_shape_without_device_facts_and_with_explicit_settings(sim, tmp_path, cold_file):
    path, _ = cold_file
    empty = str(tmp_path / "sys")
    os.makedirs(empty)
    write(str(tmp_path / "proc/meminfo"), "MemAvailable:   201326592 kB\n")
    with env(FSTX_SYSFS_ROOT=empty, FSTX_PROCFS_ROOT=tmp_path / "proc"):
        # nothing known about the device: one read in flight, 1 GiB
        ctx = make_ctx(sim, block=4 * MIB, threads=16)
        sim.fstx_file_open(ctx, path.encode(), _native.READ_DIRECT)
        m = metrics(sim, ctx)
        if m.direct_read_bytes:
            assert (m.direct_read_bytes, m.direct_depth, m.direct_steered, m.storage_flags) == (GIB, 1, 0, 0)
        assert sim.fstx_ctx_destroy(ctx) == 0
    # what the configuration names is kept whatever the device says, and is settled from the start
    root = str(tmp_path / "sys2")
    device_tree(root, os.stat(path).st_dev, "nvme0n1", 1023, 1280)
    with env(FSTX_SYSFS_ROOT=root, FSTX_PROCFS_ROOT=tmp_path / "proc"):
        ctx = make_ctx(sim, block=MIB, threads=8, depth=3, direct_bytes=8 * MIB)
        m = metrics(sim, ctx)
        assert (m.direct_read_bytes, m.direct_depth, m.direct_steered, m.staging_buffers_max) == (8 * MIB, 3, 0, 4)
        sim.fstx_file_open(ctx, path.encode(), _native.READ_DIRECT)
        m = metrics(sim, ctx)
        assert (m.direct_read_bytes, m.direct_depth, m.direct_steered) == (8 * MIB, 3, 0)
        assert sim.fstx_ctx_destroy(ctx) == 0
        # depth named, size left open: the device's budget in one read, the named depth, not steered
        ctx = make_ctx(sim, block=MIB, threads=8, depth=1)
        sim.fstx_file_open(ctx, path.encode(), _native.READ_DIRECT)
        m = metrics(sim, ctx)
        if m.direct_read_bytes:
            assert (m.direct_read_bytes, m.direct_depth, m.direct_steered) == (GIB, 1, 0)
        assert sim.fstx_ctx_destroy(ctx) == 0


def test_staging_memory_stays_under_a_share_of_available_memory(sim, tmp_path, cold_file):
    """Steered reads may hold up to 17 staging buffers; on a small host their number, then their
    size, shrink until the total is at most MemAvailable / 16."""
    path, _ = cold_file
    root = str(tmp_path / "sys")
    device_tree(root, os.stat(path).st_dev, "nvme0n1", 1023, 1280)
    for avail_kb, want_total_max in ((201326592, 12 * GIB), (16 * 1024 * 1024, GIB), (1024 * 1024, 128 * MIB)):
        write(str(tmp_path / "proc/meminfo"), f"MemAvailable:   {avail_kb} kB\n")
        with env(FSTX_SYSFS_ROOT=root, FSTX_PROCFS_ROOT=tmp_path / "proc"):
            ctx = make_ctx(sim, block=4 * MIB, threads=16)
            sim.fstx_file_open(ctx, path.encode(), _native.READ_DIRECT)
            m = metrics(sim, ctx)
            if m.direct_read_bytes == 0:
                pytest.skip("this filesystem refuses O_DIRECT")
            assert m.staging_buffers_max >= 3 and m.direct_read_bytes % (4 * MIB) == 0
            assert m.staging_buffers_max * m.direct_read_bytes <= max(want_total_max, 128 * MIB)
            assert sim.fstx_ctx_destroy(ctx) == 0


# ---- steering the depth against a storage model ------------------------------------------------------------


def _steered_load(sim, path, size, parallel, lat_us, mbps, start_depth=2):
    sim.fstx_sim_set_storage(lat_us, float(mbps), parallel)
    try:
        ctx = make_ctx(sim, block=16 * 1024, threads=16, depth=start_depth, direct_bytes=64 * 1024,
                       flags=_native.ADAPTIVE_DEPTH, ramp_kb=64, streams=4)
        f = sim.fstx_file_open(ctx, path.encode(), _native.READ_DIRECT)
        dev = np.zeros(size, dtype=np.uint8)
        t0 = time.perf_counter()
        req = sim.fstx_submit_read(ctx, f, 0, size, dev.ctypes.data, dev.size, 0)
        assert sim.fstx_wait_read(ctx, req) == size
        wall = time.perf_counter() - t0
        m = metrics(sim, ctx)
        assert sim.fstx_ctx_destroy(ctx) == 0
        return m, wall, dev
    finally:
        sim.fstx_sim_set_storage(0, 0.0, 0)


@pytest.fixture(scope="module")
def big_file(tmp_path_factory):
    path = str(tmp_path_factory.mktemp("steer") / "big.bin")
    data = np.random.default_rng(9).integers(0, 256, 96 * MIB, dtype=np.uint8)
    data.tofile(path)
    return path, data


def timing_test(attempts=3):
    """A test of a controller that steers by measured rates: on a machine whose CPUs come and go
    (a shared virtual machine) one run can be starved into a wrong reading, so the property must
    hold in one of a few attempts; what fails every time is reported."""
    def wrap(fn):
        import functools

        @functools.wraps(fn)
        def run(*args, **kwargs):
            for attempt in range(attempts):
                try:
                    return fn(*args, **kwargs)
                except AssertionError:
                    if attempt + 1 == attempts:
                        raise
        return run
    return wrap


@timing_test()
def test_depth_climbs_on_parallel_storage_and_stays_low_on_serial_storage(sim, big_file):
    """Model: a request of 64 KiB takes 5 ms + 64 KiB at bandwidth / parallel (another 5 ms); up to
    `parallel` requests are served at once.  (Slow on purpose: the model, not this machine's
    scheduler, must be what the gate measures.)  With 16 channels every further read in flight
    adds rate until the gain drops under 8 % (12 -> 13); with one channel a second read adds
    nothing."""
    path, data = big_file
    m, wall, dev = _steered_load(sim, path, data.size, parallel=16, lat_us=5000, mbps=210)
    if m.direct_fallbacks:
        pytest.skip("this filesystem refuses O_DIRECT")
    assert np.array_equal(dev, data)
    assert m.direct_steered == 1 and 8 <= m.direct_depth <= 16, m.direct_depth
    parallel_rate = data.size / wall
    m, wall, dev = _steered_load(sim, path, 10 * MIB, parallel=1, lat_us=5000, mbps=13.1)
    assert np.array_equal(dev, data[: 10 * MIB])
    assert m.direct_depth <= 2, m.direct_depth
    # and the climb paid
    assert parallel_rate > 3 * (10 * MIB / wall), (parallel_rate, 10 * MIB / wall)


@timing_test()
def test_staging_copies_keep_up_with_fast_storage(sim, big_file):
    """Storage modelled at 8 GB/s over 8 channels, 4 MiB reads, depth 8: moving the bytes from the
    staging buffers into the ring is spread over all workers, and they spend well under half of
    their time in it (this machine's memcpy and thread scheduling set the absolute rate, so only
    the share is asserted)."""
    path, data = big_file
    sim.fstx_sim_set_storage(50, 8000.0, 8)
    try:
        ctx = make_ctx(sim, block=MIB, threads=8, depth=8, direct_bytes=4 * MIB, ramp_kb=4096, streams=4)
        f = sim.fstx_file_open(ctx, path.encode(), _native.READ_DIRECT)
        dev = np.zeros(data.size, dtype=np.uint8)
        best = None
        for _ in range(3):
            m0 = metrics(sim, ctx)
            t0 = time.perf_counter()
            req = sim.fstx_submit_read(ctx, f, 0, data.size, dev.ctypes.data, dev.size, 0)
            assert sim.fstx_wait_read(ctx, req) == data.size
            wall = time.perf_counter() - t0
            m1 = metrics(sim, ctx)
            share = (m1.stage_ns - m0.stage_ns) / 1e9 / (wall * 8)
            if best is None or wall < best[0]:
                best = (wall, share)
        if m1.direct_fallbacks:
            pytest.skip("this filesystem refuses O_DIRECT")
        assert np.array_equal(dev, data)
        wall, share = best
        assert share < 0.5, (share, data.size / wall / 1e9)
        assert sim.fstx_ctx_destroy(ctx) == 0
    finally:
        sim.fstx_sim_set_storage(0, 0.0, 0)
