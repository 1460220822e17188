# SPDX-License-Identifier: Apache-2.0
"""The benchmark checkpoints at their full sizes, on the GPU.

Byte-for-byte comparison with the oracle is kept for sizes it finishes in
seconds (C1, C2 in test_loader_gpu.py).  Here the 16 GB and 26 GB checkpoints
are checked through size-independent properties: order-sensitive checksums taken
from the generator before the bytes ever reached the disk, and the round trip
"the four ranks' blocks, cut in turn, reassemble to the tensor".  The 73 GB
checkpoint (C5) is written to FSTX_TEST_C5_DIR, or to /dev/shm when that has the
room (tmpfs: the reader's O_DIRECT request falls back to page-cache reads there).
"""
import os
from collections import OrderedDict

import pytest
import torch

from fastsafetensors_amd import SafeTensorsFileLoader, SingleGroup, StubProcessGroup, _native
from fastsafetensors_amd import checkpoints as ck
from fastsafetensors_amd.frameworks import get_framework_op

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def write_with_checksums(key, directory):
    sums = {}

    def on_chunk(spec, chunk):
        assert spec.name not in sums
        sums[spec.name] = ck.tensor_checksum(chunk)

    old = ck.CHUNK_ELEMS
    ck.CHUNK_ELEMS = 1 << 62  # whole tensors: one checksum each
    try:
        recs = ck.write_config(ck.configs(1.0)[key], directory, device="cuda", sha256=False, on_chunk=on_chunk)
    finally:
        ck.CHUNK_ELEMS = old
    torch.cuda.empty_cache()
    return [r["path"] for r in recs], sums, sum(r["size"] - r["header_length"] for r in recs)


def assert_clean():
    assert get_framework_op("pytorch").get_mem_used() == 0
    assert _native.get_cpp_metrics().bounce_buffer_bytes == 0


def load_and_check(files, sums, **kw):
    loader = SafeTensorsFileLoader(SingleGroup(), DEV, **kw)
    loader.add_filenames({0: files})
    bufs = loader.copy_files_to_device()
    assert sorted(loader.get_keys()) == sorted(sums)
    for key in loader.get_keys():
        t = bufs.get_tensor(key)
        assert t.data_ptr() % 16 == 0
        assert ck.tensor_checksum(t) == sums[key], key
    return loader, bufs


def need_free(directory: str, nbytes: float) -> None:
    os.makedirs(directory, exist_ok=True)
    st = os.statvfs(directory)
    if st.f_bavail * st.f_frsize < nbytes:
        pytest.skip(f"{directory} has less than {nbytes / 1e9:.0f} GB free (set FSTX_TEST_DIR)")


def test_c3_llama3_8b_full_size(data_dir):
    need_free(data_dir, 18e9)
    files, sums, nbytes = write_with_checksums("C3", os.path.join(data_dir, "full_C3"))
    assert nbytes == 16_060_522_496 and len(sums) == 291
    try:
        for kw in ({"read_mode": "direct"}, {"read_mode": "buffered"}, {"read_mode": "auto", "layout": "window"}):
            loader, bufs = load_and_check(files, sums, **kw)
            bufs.close()
            loader.close()
            assert_clean()
    finally:
        for f in files:
            os.remove(f)


def test_c4_llama2_13b_tp4_full_size(data_dir):
    """All four TP=4 ranks' shards, extracted in turn on one GPU, against torch's own
    slice of the (checksum-verified) whole tensor."""
    need_free(data_dir, 28e9)
    files, sums, nbytes = write_with_checksums("C4", os.path.join(data_dir, "full_C4"))
    assert nbytes == 26_031_728_640 and len(sums) == 363
    try:
        whole_loader, whole = load_and_check(files, sums)
        world = 4
        for rank in range(world):
            loader = SafeTensorsFileLoader(StubProcessGroup(rank, world), DEV)
            loader.add_filenames({rank: files})
            bufs = loader.copy_files_to_device()
            dims = OrderedDict((k, ck.llama_shard_dim(k)) for k in loader.get_keys())
            out = bufs.as_dict(dims)  # batched launches; frees each file once all of its keys were taken
            assert all(f.gbuf is None for f in bufs.rank_loaders[rank])
            for key, dim in dims.items():
                full = whole.get_tensor(key)
                got = out[key].get_raw()
                if dim < 0:
                    want = full
                else:
                    block = -(-full.shape[dim] // world)
                    want = full[(slice(None),) * dim + (slice(rank * block, (rank + 1) * block),)]
                assert got.shape == want.shape and got.data_ptr() != full.data_ptr()
                assert torch.equal(got.view(torch.int16), want.view(torch.int16)), (key, rank)
            # single get_sharded calls agree with the batched path
            loader2 = SafeTensorsFileLoader(StubProcessGroup(rank, world), DEV)
            loader2.add_filenames({rank: files[:1]})
            bufs2 = loader2.copy_files_to_device()
            for key in ("model.layers.0.self_attn.o_proj.weight", "model.layers.3.mlp.down_proj.weight",
                        "model.embed_tokens.weight"):
                assert torch.equal(bufs2.get_sharded(key, dims[key]).view(torch.int16), out[key].get_raw().view(torch.int16))
            del out
            bufs2.close()
            loader2.close()
            bufs.close()
            loader.close()
        whole.close()
        whole_loader.close()
        assert_clean()
    finally:
        for f in files:
            os.remove(f)


def _c5_directory():
    """FSTX_TEST_C5_DIR, else /dev/shm when it (and the RAM behind it) has room for 73 GB."""
    if os.environ.get("FSTX_TEST_C5_DIR"):
        return os.environ["FSTX_TEST_C5_DIR"]
    try:
        st = os.statvfs("/dev/shm")
        free = st.f_bavail * st.f_frsize
        with open("/proc/meminfo") as f:
            avail = next(int(l.split()[1]) * 1024 for l in f if l.startswith("MemAvailable"))
    except (OSError, StopIteration):
        return None
    return "/dev/shm/fstx_test" if free > 90e9 and avail > 170e9 else None


@pytest.mark.skipif(_c5_directory() is None, reason="no directory with 75 GB free (set FSTX_TEST_C5_DIR)")
def test_c5_llama3_70b_fp8_full_size():
    """72.7 GB of fp8 weights, fp32 scalar scales and bf16 vectors in 15 files, whole in HBM."""
    directory = os.path.join(_c5_directory(), "full_C5")
    files, sums, nbytes = write_with_checksums("C5", directory)
    assert len(files) == 15 and len(sums) == 1283 and nbytes == 72_656_373_952
    try:
        loader, bufs = load_and_check(files, sums)
        dtypes = {bufs.get_tensor(k).dtype for k in loader.get_keys()}
        assert dtypes == {torch.float8_e4m3fn, torch.float32, torch.bfloat16}
        assert get_framework_op("pytorch").get_mem_used() >= nbytes
        scale = bufs.get_tensor("model.layers.0.mlp.down_proj.weight_scale")
        assert scale.shape == () and scale.item() == pytest.approx(0.0002)
        bufs.close()
        loader.close()
        assert_clean()
    finally:
        for f in files:
            os.remove(f)
