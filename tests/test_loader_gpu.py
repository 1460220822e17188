# SPDX-License-Identifier: Apache-2.0
"""End-to-end GPU parity of the load path: file -> HBM -> tensors / shards.

The loader API is the reference's; the expectations are the oracle's file bytes
and numpy slices, plus ``safetensors.torch.load_file`` with torch slicing (the
oracle of the reference's own tests).  Everything is compared bit for bit.
"""
import os
from collections import OrderedDict

import numpy as np
import pytest
import torch
from safetensors.torch import load_file

from conftest import GOLDEN_FILES
from fastsafetensors_amd import (
    SafeTensorsFileLoader,
    SingleGroup,
    StubProcessGroup,
    _native,
    checkpoints as ck,
    fastsafe_open,
)
from fastsafetensors_amd.frameworks import get_framework_op
from oracle import st_oracle as orc

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def dev_bytes(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().reshape(-1).view(torch.uint8).cpu().numpy()


def assert_clean():
    fw = get_framework_op("pytorch")
    assert fw.get_mem_used() == 0
    assert _native.get_cpp_metrics().bounce_buffer_bytes == 0


def check_against_oracle(bufs, path, keys=None):
    h = orc.parse_file(path)
    ref = load_file(path)
    for key in keys or h.tensors:
        t = bufs.get_tensor(key)
        assert t.is_cuda and t.data_ptr() % 16 == 0, key
        assert list(t.shape) == list(ref[key].shape) and t.dtype == ref[key].dtype, key
        assert np.array_equal(dev_bytes(t), orc.tensor_bytes(path, h, key)), key
        assert np.array_equal(dev_bytes(t), ref[key].reshape(-1).view(torch.uint8).numpy()), key


@pytest.mark.parametrize("name", GOLDEN_FILES)
@pytest.mark.parametrize("layout", ["direct", "window"])
@pytest.mark.parametrize("read_mode", ["auto", "buffered", "direct"])
def test_golden_files_all_modes(golden, name, layout, read_mode):
    path = golden(name)
    loader = SafeTensorsFileLoader(SingleGroup(), DEV, layout=layout, read_mode=read_mode, max_threads=4)
    loader.add_filenames({0: [path]})
    bufs = loader.copy_files_to_device()
    check_against_oracle(bufs, path)
    assert bufs.get_filename(loader.get_keys()[0]) == path
    assert bufs.get_filename("aaaaaaaaaaaaa") == ""
    with pytest.raises(ValueError):
        bufs.get_tensor("aaaaaaaaaaaaa")
    bufs.close()
    loader.close()
    assert_clean()


def test_reference_fixture_rows(golden):
    # known answer of the reference's fixture: row i of a0 is all float16(i)
    with fastsafe_open([golden("a.safetensors"), golden("b.safetensors")], device=DEV, nogds=True) as f:
        assert sorted(f.keys()) == ["a0", "b0"]
        for k in ("a0", "b0"):
            t = f.get_tensor(k)
            want = torch.arange(16, dtype=torch.float16).reshape(16, 1).expand(16, 8)
            assert torch.equal(t.cpu(), want)
        assert set(f.metadata().keys()) == {golden("a.safetensors"), golden("b.safetensors")}
    assert_clean()


@pytest.fixture(scope="module")
def small_configs(data_dir):
    """Scaled-down files with the structure of the five benchmark checkpoints."""
    out = {}
    for key, scale in [("C1", 0.06), ("C2", 0.06), ("C3", 0.03), ("C4", 0.03), ("C5", 0.02)]:
        cfg = ck.configs(scale)[key]
        out[key] = [r["path"] for r in ck.write_config(cfg, os.path.join(data_dir, "small_" + key))]
    return out


@pytest.mark.parametrize("key", ["C1", "C2", "C3", "C4", "C5"])
@pytest.mark.parametrize("layout", ["direct", "window"])
def test_small_configs_get_tensor(small_configs, key, layout):
    files = small_configs[key]
    loader = SafeTensorsFileLoader(SingleGroup(), DEV, layout=layout)
    loader.add_filenames({0: files})
    bufs = loader.copy_files_to_device(max_copy_block_size=3_000_000)
    n = 0
    for path in files:
        h = orc.parse_file(path)
        for name in h.tensors:
            t = bufs.get_tensor(name)
            assert t.data_ptr() % 16 == 0
            assert np.array_equal(dev_bytes(t), orc.tensor_bytes(path, h, name)), name
            n += 1
    assert n == len(loader.get_keys())
    bufs.close()
    loader.close()
    assert_clean()


def test_c2_window_layout_runs_realign_on_every_tensor(small_configs):
    """Header length = 2 (mod 8): in the window layout no tensor is aligned where it
    lands, so every returned tensor must come out of the realign kernel's arena."""
    path = small_configs["C2"][0]
    h = orc.parse_file(path)
    assert h.header_length % 8 == 2
    loader = SafeTensorsFileLoader(SingleGroup(), DEV, layout="window")
    loader.add_filenames({0: [path]})
    bufs = loader.copy_files_to_device()
    gbuf = bufs.rank_loaders[0][0].gbuf
    assert gbuf.get_length() == 0 and len(gbuf.extras) == 1  # window released, realigned arena kept
    arena = gbuf.extras[0]
    lo, hi = arena.get_base_address(), arena.get_base_address() + arena.get_length()
    for name in h.tensors:
        t = bufs.get_tensor(name)
        assert lo <= t.data_ptr() < hi and t.data_ptr() % 16 == 0
        assert np.array_equal(dev_bytes(t), orc.tensor_bytes(path, h, name))
    bufs.close()
    loader.close()
    assert_clean()


@pytest.mark.parametrize("key", ["C4", "C5", "C1"])
def test_sharded_all_ranks(small_configs, key):
    """TP ranks emulated in turn by a stub group: every shard equals the oracle's
    slice and torch's slice of load_file's tensor (tests/unit/test_multi.py:44-64)."""
    files = small_configs[key]
    world = 4
    refs = {p: load_file(p) for p in files}
    heads = {p: orc.parse_file(p) for p in files}
    for rank in range(world):
        loader = SafeTensorsFileLoader(StubProcessGroup(rank, world), DEV)
        loader.add_filenames({rank: files})
        bufs = loader.copy_files_to_device()
        bufs.auto_mem_delete = False
        for p in files:
            for name, entry in heads[p].tensors.items():
                shape = entry["shape"]
                dim = ck.llama_shard_dim(name) if key != "C1" else (len(shape) - 1 if shape else -1)
                if not shape:
                    dim = -1
                got = bufs.get_sharded(name, dim)
                raw = orc.tensor_bytes(p, heads[p], name)
                want, want_shape = orc.shard_bytes(raw, entry["dtype"], shape, dim, rank, world)
                assert list(got.shape) == want_shape, (name, dim, rank)
                assert np.array_equal(dev_bytes(got), want), (name, dim, rank)
                if dim >= 0:
                    block = -(-shape[dim] // world)
                    sl = (slice(None),) * dim + (slice(rank * block, (rank + 1) * block, 1),)
                    assert torch.equal(got.cpu().view(torch.uint8), refs[p][name][sl].contiguous().view(torch.uint8))
        bufs.close()
        loader.close()
        assert_clean()


def test_uneven_and_empty_shards(golden):
    """16 rows over 3 ranks -> 6, 6, 4; 8 columns over 16 ranks -> ranks 8..15 get nothing."""
    path = golden("a.safetensors")
    full = load_file(path)["a0"]
    for world, dim in [(3, 0), (16, 1), (5, 1)]:
        for rank in range(world):
            loader = SafeTensorsFileLoader(StubProcessGroup(rank, world), DEV, max_threads=2)
            loader.add_filenames({rank: [path]})
            bufs = loader.copy_files_to_device()
            got = bufs.get_sharded("a0", dim)
            block = -(-full.shape[dim] // world)
            sl = (slice(None),) * dim + (slice(rank * block, (rank + 1) * block, 1),)
            want = full[sl]
            assert tuple(got.shape) == tuple(want.shape)
            assert torch.equal(got.cpu(), want)
            bufs.close()
            loader.close()
    assert_clean()


def test_as_dict_multi_cols_push_and_auto_free(small_configs):
    files = small_configs["C4"]
    rank, world = 1, 4
    loader = SafeTensorsFileLoader(StubProcessGroup(rank, world), DEV)
    loader.add_filenames({rank: files})
    bufs = loader.copy_files_to_device()
    assert bufs.auto_mem_delete  # a group larger than one turns the accounting on
    bufs.auto_mem_delete = False  # ... but keep the buffers while keys are asked for twice
    refs = {}
    for p in files:
        refs.update(load_file(p))
    dims = OrderedDict((k, ck.llama_shard_dim(k)) for k in loader.get_keys())
    # multi cols first (q/k/v rows joined), while every buffer is alive
    qkv = [f"model.layers.0.self_attn.{n}_proj.weight" for n in "qkv"]
    joined = bufs.get_multi_cols(qkv, dim=0).get_raw()
    block = -(-refs[qkv[0]].shape[0] // world)
    want = torch.cat([refs[k][rank * block : (rank + 1) * block] for k in qkv], dim=0)
    assert torch.equal(joined.cpu().view(torch.int16), want.view(torch.int16))
    # a join along dim 1 (column blocks side by side): one launch with a strided destination
    o2 = [f"model.layers.{i}.self_attn.o_proj.weight" for i in (0, 1)]
    joined = bufs.get_multi_cols(o2, dim=1).get_raw()
    block = -(-refs[o2[0]].shape[1] // world)
    want = torch.cat([refs[k][:, rank * block : (rank + 1) * block] for k in o2], dim=1)
    assert torch.equal(joined.cpu().view(torch.int16), want.view(torch.int16))
    # push: a stub of rank 1 keeps what is pushed to rank 1, nothing otherwise
    pushed = bufs.push_tensor("model.norm.weight", 1)
    assert pushed is not None and torch.equal(pushed.cpu(), refs["model.norm.weight"])
    assert bufs.push_tensor("model.layers.1.input_layernorm.weight", 0) is None
    bufs.auto_mem_delete = True
    out = bufs.as_dict(dims)
    for k, dim in dims.items():
        t = refs[k]
        if dim >= 0:
            b = -(-t.shape[dim] // world)
            t = t[(slice(None),) * dim + (slice(rank * b, (rank + 1) * b),)]
        assert torch.equal(out[k].get_raw().cpu().view(torch.uint8), t.contiguous().view(torch.uint8)), k
    # every key was requested once: all file buffers are gone without close()
    assert all(f.gbuf is None for f in bufs.rank_loaders[rank])
    assert get_framework_op("pytorch").get_mem_used() == 0
    bufs.close()
    loader.close()
    assert_clean()


def test_multi_cols_many_and_shared_storage(small_configs):
    """``get_multi_cols_many`` gives what one ``get_multi_cols`` per group gives, for joins along
    the outermost and along an inner dimension; the tensors of one ``as_dict`` call are views of
    one allocation, each on a 16-byte boundary, and stay valid after the file buffers are closed."""
    files = small_configs["C4"]
    rank, world = 1, 4
    loader = SafeTensorsFileLoader(StubProcessGroup(rank, world), DEV)
    loader.add_filenames({rank: files})
    bufs = loader.copy_files_to_device()
    bufs.auto_mem_delete = False
    layers = sorted({int(k.split(".")[2]) for k in loader.get_keys() if k.startswith("model.layers.")})
    for dim in (0, 1):
        groups = []
        for i in layers:
            p = f"model.layers.{i}."
            groups.append([p + f"self_attn.{x}_proj.weight" for x in "qkv"])
            groups.append([p + f"mlp.{x}_proj.weight" for x in ("gate", "up")])
        many = bufs.get_multi_cols_many(groups, dim=dim)
        assert len(many) == len(groups)
        for names, t in zip(groups, many):
            one = bufs.get_multi_cols(names, dim=dim).get_raw()
            assert t.get_raw().shape == one.shape and t.get_raw().data_ptr() % 16 == 0
            assert torch.equal(t.get_raw().view(torch.int16), one.view(torch.int16)), (dim, names)
    dims = OrderedDict((k, ck.llama_shard_dim(k)) for k in loader.get_keys())
    out = bufs.as_dict(dims)
    raws = {k: t.get_raw() for k, t in out.items()}
    assert len({t.untyped_storage().data_ptr() for t in raws.values()}) <= len(files)  # one allocation per file
    assert all(t.data_ptr() % 16 == 0 and t.is_contiguous() for t in raws.values())
    want = {}
    for path in files:
        h = orc.parse_file(path)
        for name, entry in h.tensors.items():
            dim = dims[name]
            if dim < 0:
                want[name] = orc.tensor_bytes(path, h, name)
            else:
                want[name] = orc.shard_bytes(orc.tensor_bytes(path, h, name), entry["dtype"], entry["shape"], dim, rank, world)[0]
    bufs.close()  # the shards are copies: they outlive the file buffers
    loader.close()
    for name, t in raws.items():
        assert np.array_equal(dev_bytes(t), want[name]), name
    del out, raws, many, t, one
    assert_clean()


def test_loader_reuse_and_key_order(small_configs, golden):
    loader = SafeTensorsFileLoader(SingleGroup(), DEV)
    for files in (small_configs["C3"], [golden("tiny_gpt2.safetensors")]):
        loader.add_filenames({0: files})
        want = []
        for p in files:  # registration order x in-file offset order
            want += list(orc.parse_file(p).tensors)
        assert loader.get_keys() == want
        bufs = loader.copy_files_to_device()
        check_against_oracle(bufs, files[-1])
        assert loader.get_shape(want[-1]) == bufs.get_shape(want[-1])
        bufs.close()
        loader.reset()
    loader.close()
    assert_clean()


def test_truncated_file_raises(small_configs, tmp_path):
    src = small_configs["C1"][0]
    cut = str(tmp_path / "cut.safetensors")
    size = os.path.getsize(src)
    with open(src, "rb") as f, open(cut, "wb") as g:
        g.write(f.read(size))
    loader = SafeTensorsFileLoader(SingleGroup(), DEV, max_threads=4)
    loader.add_filenames({0: [cut]})
    os.truncate(cut, size - 70_000)  # header parsed, then the file shrinks
    with pytest.raises(Exception, match="read failed"):
        loader.copy_files_to_device()
    loader.close()
    assert_clean()


def test_duplicate_key_across_files(golden, tmp_path):
    twin = str(tmp_path / "a_copy.safetensors")
    with open(golden("a.safetensors"), "rb") as f, open(twin, "wb") as g:
        g.write(f.read())
    loader = SafeTensorsFileLoader(SingleGroup(), DEV, max_threads=2)
    loader.add_filenames({0: [golden("a.safetensors"), twin]})
    with pytest.raises(Exception, match="must be unique"):
        loader.copy_files_to_device()
    loader.close()
    assert_clean()  # the arenas of both files went back although no FilesBufferOnDevice ever owned them


def test_full_size_c1_and_c2(data_dir):
    """Configs C1 (fp32, 0.5 GB) and C2 (fp16, misaligned header, 0.7 GB) at full size,
    every tensor byte-exact against the oracle's file bytes, cold-ish and warm."""
    for key in ("C1", "C2"):
        cfg = ck.configs(1.0)[key]
        recs = ck.write_config(cfg, os.path.join(data_dir, "full_" + key), device="cuda")
        path = recs[0]["path"]
        h = orc.parse_file(path)
        for layout, mode in [("direct", "direct"), ("window", "buffered"), ("direct", "auto")]:
            loader = SafeTensorsFileLoader(SingleGroup(), DEV, layout=layout, read_mode=mode)
            loader.add_filenames({0: [path]})
            bufs = loader.copy_files_to_device()
            data = orc.file_bytes(path, h.header_length, h.size_bytes)
            for name, entry in h.tensors.items():
                s, e = entry["data_offsets"]
                t = bufs.get_tensor(name)
                assert t.data_ptr() % 16 == 0
                assert np.array_equal(dev_bytes(t), data[s:e]), (key, layout, mode, name)
            bufs.close()
            loader.close()
        os.remove(path)
    assert_clean()


@pytest.mark.parametrize("queue_size", [-1, 0, 2])
def test_parallel_loader_iterate_weights(small_configs, queue_size):
    """The vLLM-facing iterator: every tensor of every file once, in file order, as
    copies that outlive their batch; byte-exact against the oracle's file bytes."""
    from fastsafetensors_amd import ParallelLoader

    files = small_configs["C5"]
    it = ParallelLoader(None, files, queue_size=queue_size, device=DEV, max_threads=8)
    got = {}
    for key, t in it.iterate_weights():
        assert key not in got and t.is_cuda and t.data_ptr() % 16 == 0
        got[key] = t
    it.close()
    n = 0
    for path in files:
        h = orc.parse_file(path)
        for name in h.tensors:
            assert np.array_equal(dev_bytes(got[name]), orc.tensor_bytes(path, h, name)), name
            n += 1
    assert n == len(got)
    got.clear()
    assert_clean()


def test_parallel_loader_error_and_early_stop(small_configs, tmp_path):
    from fastsafetensors_amd import ParallelLoader

    files = list(small_configs["C3"])
    files.insert(2, str(tmp_path / "nope.safetensors"))
    it = ParallelLoader(None, files, device=DEV, max_threads=4)
    with pytest.raises(FileNotFoundError):
        for _ in it.iterate_weights():
            pass
    it.close()
    it = ParallelLoader(None, small_configs["C3"], queue_size=3, device=DEV, max_threads=4)
    gen = it.iterate_weights()
    first = next(gen)
    gen.close()  # the consumer walks away after one tensor
    it.close()
    del first
    assert_clean()


def test_c_abi_from_plain_c(data_dir):
    """A C99 program with no Python, torch or C++ in it loads a file through the pipeline
    (three read modes, a destination range check) and runs the realign, slice, join and
    convert entry points, checking every result against host loops."""
    import subprocess

    exe = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cabi_native", "cabi_check.bin")
    if not os.path.exists(exe):
        pytest.skip("tests/cabi_native/cabi_check.bin is not built (run __graft_entry__.build())")
    blob = os.path.join(data_dir, "cabi_blob.bin")
    np.random.default_rng(3).integers(0, 256, 20_000_003, dtype=np.uint8).tofile(blob)
    try:
        run = subprocess.run([exe, blob], capture_output=True, text=True, timeout=120)
    finally:
        os.remove(blob)
    assert run.returncode == 0 and "cabi_check: ok" in run.stdout, run.stdout + run.stderr


def test_empty_tensors_and_files_without_data(tmp_path):
    """Zero-element tensors between real ones, a file whose only tensor is empty, and a file
    with no tensors at all load like any other (the reference's header rules allow them:
    e - s == 0 == prod(shape) * itemsize, common.py:205-231)."""
    from safetensors.torch import save_file

    mixed = str(tmp_path / "mixed.safetensors")
    save_file({"a": torch.arange(12, dtype=torch.float32).reshape(3, 4), "e": torch.empty((0, 7), dtype=torch.float16),
               "z": torch.ones(5, dtype=torch.bfloat16), "e2": torch.empty(0, dtype=torch.int64)}, mixed)
    only_empty = str(tmp_path / "only_empty.safetensors")
    save_file({"only.e": torch.empty((4, 0), dtype=torch.float32)}, only_empty)
    nothing = str(tmp_path / "nothing.safetensors")
    save_file({}, nothing)
    for layout in ("direct", "window"):
        for rank, world in ((0, 1), (1, 2)):
            pg = SingleGroup() if world == 1 else StubProcessGroup(rank, world)
            loader = SafeTensorsFileLoader(pg, DEV, layout=layout, max_threads=2)
            loader.add_filenames({rank: [mixed, only_empty, nothing]} if world > 1 else {0: [mixed, nothing]})
            bufs = loader.copy_files_to_device()
            bufs.auto_mem_delete = False
            ref = load_file(mixed)
            for k, t in ref.items():
                got = bufs.get_tensor(k)
                assert got.shape == t.shape and got.dtype == t.dtype and torch.equal(got.cpu(), t), (layout, k)
                if world > 1 and t.dim() >= 1:
                    sh = bufs.get_sharded(k, 0)
                    b = -(-t.shape[0] // world)
                    assert torch.equal(sh.cpu(), t[rank * b : (rank + 1) * b]), (layout, k)
            if world > 1:
                assert tuple(bufs.get_tensor("only.e").shape) == (4, 0)
            bufs.close()
            loader.close()
            assert_clean()
