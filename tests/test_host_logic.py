# SPDX-License-Identifier: Apache-2.0
"""Loader, file buffer and tensor factory logic on the CPU, above the copier boundary.

A test-only copier (tests/pyread_copier.py) stands where the HIP copier stands,
so that ordering, bookkeeping and lifetimes can be checked without a GPU.  The
cases follow the reference's tests: as_dict / get_tensor round trips against
safetensors.load_file (test_fastsafetensors.py:548-567), the two auto-free
regressions (:852-929), the push truth table (test_multi.py:71-82), leak checks.
"""
from collections import OrderedDict

import os

import pytest
import torch
from safetensors.torch import load_file, save_file

import pyread_copier  # noqa: F401  (registers "pyread_test")
from fastsafetensors_amd import BaseSafeTensorsFileLoader, Device, SingleGroup, StubProcessGroup
from fastsafetensors_amd.copier import create_copier_constructor
from fastsafetensors_amd.copier.mi355x import pick_lead
from fastsafetensors_amd.common import TensorFrame
from fastsafetensors_amd.frameworks import get_framework_op
from fastsafetensors_amd.st_types import DType
from oracle import st_oracle as orc

CPU = Device.from_str("cpu")
FW = get_framework_op("pytorch")


def loader_for(pg=None, **kw):
    return BaseSafeTensorsFileLoader(pg, CPU, "pyread_test", **kw)


def test_round_trip_all_golden_files(golden):
    files = [golden(n) for n in ("a.safetensors", "b.safetensors", "tiny_gpt2.safetensors", "mixed_fp8.safetensors", "f4.safetensors")]
    # f4.safetensors and a.safetensors both... no shared keys: a0, b0, h.*, w*, norm*, "a"
    loader = loader_for(SingleGroup())
    loader.add_filenames({0: files})
    bufs = loader.copy_files_to_device()
    tensors = bufs.as_dict(OrderedDict((k, -1) for k in loader.get_keys()))
    for path in files:
        for key, exp in load_file(path).items():
            assert FW.is_equal(tensors[key], exp), key
            assert bufs.get_filename(key) == path
    assert bufs.get_shape("a") == [8, 16] and list(tensors["a"].get_raw().shape) == [8, 8]
    bufs.close()
    loader.close()
    assert FW.get_mem_used() == 0


def test_registration_and_processing_order(golden, tmp_path):
    paths = {}
    for name in ("zz", "mm", "aa", "kk"):
        p = str(tmp_path / f"{name}.safetensors")
        save_file({f"{name}.w": torch.full((2, 2), float(ord(name[0]))), f"{name}.b": torch.zeros(3)}, p)
        paths[name] = p
    log = []
    loader = loader_for(StubProcessGroup(0, 2), log=log)
    # ranks are visited round-robin: zz (rank 0), mm (rank 1), aa (rank 0), kk (rank 1)
    loader.add_filenames({0: [paths["zz"], paths["aa"]], 1: [paths["mm"], paths["kk"]]})
    assert loader.get_keys() == ["zz.b", "zz.w", "mm.b", "mm.w", "aa.b", "aa.w", "kk.b", "kk.w"]
    assert loader.get_shape("kk.w") == [2, 2]
    bufs = loader.copy_files_to_device()
    # only this rank's files get a copier, in sorted path order, all submits before any wait
    assert log == [("submit", paths["aa"]), ("submit", paths["zz"]), ("wait", paths["aa"]), ("wait", paths["zz"])]
    assert bufs.key_to_rank_lidx["aa.w"] == (0, 0) and bufs.key_to_rank_lidx["zz.w"] == (0, 1)
    assert bufs.key_to_rank_lidx["kk.w"] == (1, 0) and bufs.key_to_rank_lidx["mm.w"] == (1, 1)
    assert [f.lidx for f in bufs.rank_loaders[0]] == [1, 4] and [f.lidx for f in bufs.rank_loaders[1]] == [2, 3]
    assert torch.equal(bufs.get_tensor("zz.w"), torch.full((2, 2), float(ord("z"))))  # broadcast = private copy
    with pytest.raises(NotImplementedError, match="belongs to rank 1"):
        bufs.get_tensor("mm.w")  # no peer to receive it from
    with pytest.raises(ValueError):
        bufs.get_tensor("nope")
    bufs.close()
    loader.close()
    assert FW.get_mem_used() == 0


def test_world_of_one_returns_views_and_ignores_dim(golden):
    loader = loader_for(None)
    loader.add_filenames({0: [golden("tiny_gpt2.safetensors")]})
    bufs = loader.copy_files_to_device()
    assert not bufs.auto_mem_delete
    arena = bufs.rank_loaders[0][0].gbuf
    lo, hi = arena.get_base_address(), arena.get_base_address() + arena.get_length()
    full = bufs.get_tensor("h.3.mlp.c_fc.weight")
    assert lo <= full.data_ptr() < hi  # zero copy
    same = bufs.get_sharded("h.3.mlp.c_fc.weight", 0)  # dim is ignored (tensor_factory.py:119-122)
    assert same.data_ptr() == full.data_ptr() and list(same.shape) == [16, 8]
    assert bufs.push_tensor("h.3.mlp.c_fc.weight", 0).data_ptr() == full.data_ptr()
    joined = bufs.get_multi_cols(["h.0.attn.c_proj.weight", "h.1.attn.c_proj.weight"], dim=0).get_raw()
    ref = load_file(golden("tiny_gpt2.safetensors"))
    assert torch.equal(joined, torch.cat([ref["h.0.attn.c_proj.weight"], ref["h.1.attn.c_proj.weight"]], dim=0))
    with pytest.raises(Exception, match="mismatch"):
        bufs.get_multi_cols(["h.0.attn.c_proj.weight", "h.0.mlp.c_fc.weight"], dim=1)
    bufs.close()
    assert bufs.rank_loaders == {}
    loader.close()
    assert FW.get_mem_used() == 0


def test_groups_that_cannot_be_joined_as_bytes_are_refused(tmp_path):
    """get_multi_cols joins the rank's blocks as bytes: tensors of two element types, or of
    different numbers of dimensions, are refused (the reference's torch.cat would promote the
    former to a common type; silently joining their bytes would hand back garbage)."""
    path = str(tmp_path / "mixed.safetensors")
    save_file({"a.f16": torch.ones(4, 6, dtype=torch.float16), "b.bf16": torch.ones(4, 6, dtype=torch.bfloat16),
               "c.f16": torch.full((4, 6), 2.0, dtype=torch.float16), "d.f16": torch.ones(4, 6, 1, dtype=torch.float16),
               "e.i32": torch.ones(4, 6, dtype=torch.int32), "f.f32": torch.ones(4, 6, dtype=torch.float32)}, path)
    for pg in (SingleGroup(), StubProcessGroup(1, 2)):
        loader = loader_for(pg)
        loader.add_filenames({pg.rank(): [path]})
        bufs = loader.copy_files_to_device()
        bufs.auto_mem_delete = False
        with pytest.raises(Exception, match="dtype mismatch: tensor b.bf16 is BF16 vs. F16"):
            bufs.get_multi_cols(["a.f16", "b.bf16"], dim=0)
        with pytest.raises(Exception, match="dtype mismatch"):
            bufs.get_multi_cols_many([["a.f16", "c.f16"], ["e.i32", "f.f32"]], dim=1)
        with pytest.raises(Exception, match="rank mismatch"):
            bufs.get_multi_cols(["a.f16", "d.f16"], dim=0)
        if pg.size() == 1:  # (cutting a rank's blocks needs the GPU)
            ok = bufs.get_multi_cols(["a.f16", "c.f16"], dim=1).get_raw()
            assert list(ok.shape) == [4, 12] and ok[:, 6:].eq(2).all()
        bufs.close()
        loader.close()
    assert FW.get_mem_used() == 0


def test_push_truth_table(golden):
    path = golden("tiny_gpt2.safetensors")
    ref = load_file(path)
    key = "h.0.attn.c_proj.bias"
    for world in (2, 3):
        for me in range(world):
            loader = loader_for(StubProcessGroup(me, world))
            loader.add_filenames({me: [path]})  # this process owns the file
            bufs = loader.copy_files_to_device()
            bufs.auto_mem_delete = False
            for dst in range(world):
                got = bufs.push_tensor(key, dst)
                want = orc.push_outcome(world, me, dst, me)
                assert (got is not None) == (want != "none")
                if got is not None:
                    assert want == "clone" and torch.equal(got, ref[key])
                    assert got.data_ptr() != bufs.rank_loaders[me][0].tensors[key].data_ptr()
            bufs.close()
            loader.close()
    assert FW.get_mem_used() == 0


def test_get_multi_cols_multi_file_auto_free(tmp_path):
    # reference regression test_get_multi_cols_multi_file_auto_free (test_fastsafetensors.py:852-895)
    file_a, file_b = str(tmp_path / "a.safetensors"), str(tmp_path / "b.safetensors")
    a0, b0, b1 = torch.randn(4, 8), torch.randn(4, 8), torch.randn(4, 8)
    save_file({"a0": a0}, file_a)
    save_file({"b0": b0, "b1": b1}, file_b)
    loader = loader_for(SingleGroup())
    loader.add_filenames({0: [file_a, file_b]})
    fb = loader.copy_files_to_device()
    fb.auto_mem_delete = True
    out = fb.get_multi_cols(["a0", "b0"], dim=0).get_raw()
    assert torch.equal(out[0:4], a0) and torch.equal(out[4:8], b0)
    assert fb.rank_loaders[0][0].gbuf is None and fb.rank_loaders[0][1].gbuf is not None
    out2 = fb.get_multi_cols(["b1"], dim=0).get_raw()
    assert torch.equal(out2[0:4], b1)
    assert fb.rank_loaders[0][1].gbuf is None
    fb.close()
    loader.close()
    assert FW.get_mem_used() == 0


def test_as_dict_partial_request_close_frees_buffers(tmp_path):
    # reference regression test_as_dict_partial_request_close_frees_buffers (:898-929)
    path = str(tmp_path / "p.safetensors")
    a0, a1 = torch.randn(4, 8), torch.randn(4, 8)
    save_file({"a0": a0, "a1": a1}, path)
    loader = loader_for(SingleGroup())
    loader.add_filenames({0: [path]})
    fb = loader.copy_files_to_device()
    fb.auto_mem_delete = True
    tensors = fb.as_dict(OrderedDict([("a0", -1)]))
    assert FW.is_equal(tensors["a0"], a0)
    assert fb.rank_loaders[0][0].gbuf is not None
    fb.close()
    loader.close()
    assert FW.get_mem_used() == 0


def test_duplicate_keys_and_loader_reuse(golden, tmp_path):
    twin = str(tmp_path / "twin.safetensors")
    with open(golden("a.safetensors"), "rb") as f, open(twin, "wb") as g:
        g.write(f.read())
    loader = loader_for(SingleGroup())
    loader.add_filenames({0: [golden("a.safetensors"), twin]})
    with pytest.raises(Exception, match="must be unique among files"):
        loader.copy_files_to_device()
    FW.mem_used = 0  # buffers of the rejected set were never handed to a FilesBufferOnDevice
    loader.reset()
    assert loader.get_keys() == []
    loader.add_filenames({0: [golden("b.safetensors")]})
    fb = loader.copy_files_to_device()
    assert torch.equal(fb.get_tensor("b0"), load_file(golden("b.safetensors"))["b0"])
    fb.close()
    loader.close()
    with pytest.raises(Exception, match="closed"):
        loader.copy_files_to_device()
    assert FW.get_mem_used() == 0


def test_allocator_accounting():
    # reference: test_cpp_metrics (test_fastsafetensors.py:766-796)
    assert FW.get_mem_used() == 0
    g1 = FW.alloc_tensor_memory(128, CPU)
    assert FW.get_mem_used() == 128 and g1.get_base_address() != 0 and g1.get_length() == 128
    FW.free_tensor_memory(g1, CPU)
    g2 = FW.alloc_tensor_memory(1024, CPU)
    g3 = FW.alloc_tensor_memory(128, CPU)
    side = FW.alloc_side_memory(g2, 64, CPU)
    assert FW.get_mem_used() == 1024 + 128 + 64 and side in g2.extras
    FW.shrink_tensor_memory(g2)
    assert FW.get_mem_used() == 128 + 64 and g2.get_length() == 0
    FW.free_tensor_memory(g2, CPU)
    FW.free_tensor_memory(g3, CPU)
    assert FW.get_mem_used() == 0


def test_unknown_copier_and_cpu_device_are_refused():
    with pytest.raises(KeyError, match="not registered"):
        create_copier_constructor("no_such_copier", CPU)
    with pytest.raises(Exception, match="HIP device"):
        create_copier_constructor("mi355x", CPU)


def test_pick_lead_prefers_most_bytes():
    def f(start, n):
        return TensorFrame(DType.U8, [n], [start, start + n], [1], [0], False)

    assert pick_lead([f(0, 64), f(64, 64)]) == 0
    assert pick_lead([f(0, 4), f(4, 4), f(8, 1000), f(1008, 16)]) == 120  # the big one starts at 8 -> on a line at 128
    assert pick_lead([f(0, 4), f(4, 4), f(8, 1000), f(1008, 16)], line=16) == 8
    assert pick_lead([f(0, 48), f(48, 4096)]) == 80  # 16-byte alignment holds for both at 0, 16, ..; 80 puts the big one on a line
    assert pick_lead([f(0, 10), f(10, 10)]) == 0  # tie -> smallest lead
    assert pick_lead([]) == 0


def test_shard_geometry_matches_oracle_shapes():
    for shape, dtype, tag in [([16, 8], DType.F16, "F16"), ([5, 3, 7], DType.F32, "F32"), ([8, 16], DType.F4, "F4")]:
        frame = TensorFrame(dtype, shape, [0, 0], [], [], False)
        for dim in range(len(shape)):
            for world in (1, 2, 3, 4, 16):
                for rank in range(world):
                    try:
                        import numpy as np

                        bits = orc.DTYPE_BITS[tag]
                        raw = np.zeros(int(np.prod(shape)) * bits // 8, dtype=np.uint8)
                        want_shape = orc.shard_bytes(raw, tag, shape, dim, rank, world)[1]
                    except ValueError:
                        with pytest.raises(ValueError):
                            FW.shard_geometry(frame, dim, rank, world)
                        continue
                    out_shape, outer, seg, pitch, first = FW.shard_geometry(frame, dim, rank, world)
                    assert out_shape == want_shape
                    assert outer * seg == int(np.prod(want_shape)) * bits // 8


# ---- iterate_weights (producer / consumer) on the CPU ------------------------------------------


def _tiny_files(tmp_path, n):
    out, want = [], {}
    for i in range(n):
        p = str(tmp_path / f"part{i}.safetensors")
        tensors = {f"f{i}.w{k}": torch.randn(3 + k, 5) for k in range(4)}
        save_file(tensors, p)
        out.append(p)
        want.update(tensors)
    return out, want


@pytest.mark.parametrize("queue_size", [-1, 0, 2])
def test_iterate_weights_streams_every_tensor(tmp_path, queue_size):
    from fastsafetensors_amd import PipelineParallel

    files, want = _tiny_files(tmp_path, 5)
    loader = loader_for(None)
    it = PipelineParallel(None, loader, files, queue_size=queue_size)
    got = {}
    live_after_close = []
    for key, t in it.iterate_weights():
        assert key not in got
        got[key] = t
        live_after_close.append(t)
    assert list(got) == [k for i in range(5) for k in sorted(want) if k.startswith(f"f{i}.")]
    for key, t in got.items():  # tensors outlive their batches: they are copies
        assert torch.equal(t, want[key])
    it.close()
    assert FW.get_mem_used() == 0


def test_iterate_weights_reports_producer_errors_and_cleans_up(tmp_path):
    from fastsafetensors_amd import PipelineParallel

    files, want = _tiny_files(tmp_path, 3)
    files.insert(2, str(tmp_path / "missing.safetensors"))
    it = PipelineParallel(None, loader_for(None), files, queue_size=0)
    seen = []
    with pytest.raises(FileNotFoundError):
        for key, t in it.iterate_weights():
            seen.append(key)
    assert len(seen) == 8  # the two good files in front of the missing one
    it.close()
    assert FW.get_mem_used() == 0
    # stopping early releases what the producer had already loaded
    files, want = _tiny_files(tmp_path, 4)
    it = PipelineParallel(None, loader_for(None), files, queue_size=3)
    gen = it.iterate_weights()
    next(gen)
    gen.close()
    it.close()
    assert FW.get_mem_used() == 0
    with pytest.raises(ValueError, match="max_concurrent_producers"):
        PipelineParallel(None, loader_for(None), files, max_concurrent_producers=2)
    with pytest.raises(NotImplementedError):
        PipelineParallel(StubProcessGroup(0, 2), loader_for(StubProcessGroup(0, 2)), files)


@pytest.mark.parametrize("queue_size,overlapped", [(0, True), (2, True), (-1, False)])
def test_the_producer_queues_the_next_batch_before_it_waits_for_this_one(tmp_path, queue_size, overlapped):
    """With room for a second resident batch the reads of batch k+1 are submitted before batch k is
    waited for (the transfer then never pauses between batches); with room for one batch only
    (queue_size -1) every batch is submitted, waited for and consumed before the next begins.
    Residency never exceeds its bound either way."""
    from fastsafetensors_amd import PipelineParallel

    files, want = _tiny_files(tmp_path, 5)
    log = []
    loader = loader_for(None, log=log)
    it = PipelineParallel(None, loader, files, queue_size=queue_size)
    peak = 0
    n = 0
    for key, t in it.iterate_weights():
        peak = max(peak, FW.get_mem_used())
        assert torch.equal(t, want[key])
        n += 1
    it.close()
    assert n == len(want) and FW.get_mem_used() == 0
    order = [(what, files.index(path)) for what, path in log]
    assert [i for what, i in order if what == "submit"] == [0, 1, 2, 3, 4]
    assert [i for what, i in order if what == "wait"] == [0, 1, 2, 3, 4]
    at = {entry: pos for pos, entry in enumerate(order)}
    ahead = [at[("submit", k + 1)] < at[("wait", k)] for k in range(4)]
    if overlapped:
        assert any(ahead), order  # (a slow consumer may hold a place now and then; never all the time here)
    else:
        assert not any(ahead), order
    one = max(os.path.getsize(f) for f in files)
    bound = {0: 2, 2: 3, -1: 1}[queue_size]
    assert peak <= bound * one
