# SPDX-License-Identifier: Apache-2.0
"""Down-cast on load (copy_files_to_device(dtype=...)): the convert kernel through the
C ABI and the loader, bit for bit against torch's own Tensor.to() on the same device
(the reference converts with exactly that call, common.py:355-375).  Floating point,
but the bar is still bit-exact: rounding mode, overflow and NaN handling are part
of the contract."""
import os

import pytest
import torch
from safetensors.torch import load_file

from fastsafetensors_amd import DType, SafeTensorsFileLoader, SingleGroup, _native
from fastsafetensors_amd import checkpoints as ck
from fastsafetensors_amd.frameworks import get_framework_op

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
T = {"F64": torch.float64, "F32": torch.float32, "F16": torch.float16, "BF16": torch.bfloat16,
     "F8_E4M3": torch.float8_e4m3fn, "F8_E5M2": torch.float8_e5m2}
PAIRS = [("F64", d) for d in ("F32", "F16", "BF16", "F8_E4M3", "F8_E5M2")] + \
        [("F32", d) for d in ("F16", "BF16", "F8_E4M3", "F8_E5M2")] + \
        [("F16", d) for d in ("BF16", "F8_E4M3", "F8_E5M2")] + [("BF16", d) for d in ("F16", "F8_E4M3", "F8_E5M2")]


def stream():
    return torch.cuda.current_stream().cuda_stream


def inputs_for(src: str) -> torch.Tensor:
    """Values that hit every branch: all 16-bit patterns for the half types; for the
    wide types random data at many scales plus ties, thresholds, denormals, infinities."""
    if src in ("F16", "BF16"):
        return torch.arange(65536, dtype=torch.int32).to(torch.int16).view(T[src])
    g = torch.Generator().manual_seed(5)
    parts = [torch.randn(200_000, generator=g, dtype=torch.float64) * s
             for s in (1e-8, 1e-5, 1e-3, 0.02, 1.0, 30.0, 400.0, 5e4, 7e4, 1e9, 1e38)]
    # every fp16 / bf16 / fp8 value, their midpoints (ties) and neighbours of the midpoints
    for tdt in (torch.float16, torch.bfloat16):
        v = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(tdt).to(torch.float64)
        v = v[torch.isfinite(v)].sort().values
        mid = (v[:-1] + v[1:]) / 2
        parts += [v, mid, torch.nextafter(mid, torch.tensor(float("inf"), dtype=torch.float64)),
                  torch.nextafter(mid, torch.tensor(float("-inf"), dtype=torch.float64))]
    for tdt in (torch.float8_e4m3fn, torch.float8_e5m2):
        v = torch.arange(256, dtype=torch.int16).to(torch.uint8).view(tdt).to(torch.float64)
        v = v[torch.isfinite(v)].sort().values
        mid = (v[:-1] + v[1:]) / 2
        parts += [v, mid, mid * (1 + 2**-20), mid * (1 - 2**-20)]
    parts.append(torch.tensor([0.0, -0.0, float("inf"), float("-inf"), 448.0, 464.0, 479.9, 480.0, 57344.0, 61439.9,
                               61440.0, 65504.0, 65519.9, 65520.0, 65536.0, 3.4e38, 1e-45, 6e-8, 2.0**-9, 2.0**-10,
                               2.0**-17, 2.0**-16 * 1.5], dtype=torch.float64))
    x = torch.cat(parts)
    x = torch.cat([x, -x])
    return x if src == "F64" else x.to(torch.float32)


@pytest.mark.parametrize("src,dst", PAIRS)
def test_convert_matches_torch(src, dst):
    x_host = inputs_for(src)
    x = x_host.to(DEV)
    want = x.to(T[dst])
    # torch's CPU conversion is a second, independent implementation of the same contract
    nan = torch.isnan(x_host)
    isz_ = {1: torch.uint8, 2: torch.int16, 4: torch.int32}[T[dst].itemsize]
    assert torch.equal(want.cpu().view(isz_)[~nan], x_host.to(T[dst]).view(isz_)[~nan]), "torch CPU and GPU conversions disagree"
    isz = {1: torch.uint8, 2: torch.int16, 4: torch.int32}[T[dst].itemsize]
    n = x.numel()
    # aligned; element-misaligned source (still 16-byte loads); element-misaligned destination
    for shift, dshift in ((0, 0), (1, 0), (5, 0), (3, 3)):
        xs = torch.empty(n + 8, dtype=x.dtype, device=DEV)
        xs[shift : shift + n] = x
        out = torch.zeros(n + 64, dtype=isz, device=DEV)
        _native.convert_batch([(out.data_ptr() + dshift * out.element_size(), xs.data_ptr() + shift * x.element_size(), n,
                                _native.ELEM_TYPES[src], _native.ELEM_TYPES[dst])], stream())
        g, w = out[dshift : dshift + n], want.view(isz)
        if not torch.equal(g, w):
            bad = (g != w).nonzero().flatten()[:5]
            raise AssertionError(f"{src}->{dst} shift {shift}/{dshift}: {len((g != w).nonzero())} differ, e.g. "
                                 f"{[(x[i].item(), hex(g[i].item() & 0xffffffff), hex(w[i].item() & 0xffffffff)) for i in bad]}")
        assert not out[:dshift].any() and not out[dshift + n :].any(), "wrote outside the destination"


def test_convert_nan_inputs_stay_nan():
    for src in ("F64", "F32", "F16", "BF16"):
        x = torch.tensor([float("nan"), -float("nan")], dtype=T[src], device=DEV)
        for dst in [d for s, d in PAIRS if s == src]:
            out = torch.zeros(2, dtype=torch.float32, device=DEV).to(T[dst])
            _native.convert_batch([(out.data_ptr(), x.data_ptr(), 2, _native.ELEM_TYPES[src], _native.ELEM_TYPES[dst])], stream())
            assert torch.isnan(out.to(torch.float32)).all(), (src, dst)
            assert torch.equal(torch.isnan(out.to(torch.float32)), torch.isnan(x.to(T[dst]).to(torch.float32)))


def test_convert_rejects_bad_requests():
    a = torch.zeros(64, dtype=torch.float32, device=DEV)
    b = torch.zeros(64, dtype=torch.float64, device=DEV)
    lib = _native.lib()
    for s, d in [("F32", "F64"), ("F16", "F32"), ("F8_E4M3", "F8_E5M2"), ("F32", "F32")]:
        desc = (_native.FstxConvertDesc * 1)(_native.FstxConvertDesc(b.data_ptr(), a.data_ptr(), 8, _native.ELEM_TYPES[s], _native.ELEM_TYPES[d]))
        assert lib.fstx_convert_batch(desc, 1, None) == -10001
    desc = (_native.FstxConvertDesc * 1)(_native.FstxConvertDesc(a.data_ptr() + 4, a.data_ptr(), 8, 1, 3))  # overlap
    assert lib.fstx_convert_batch(desc, 1, None) == -10001


@pytest.mark.parametrize("layout", ["direct", "window"])
def test_loader_downcast_matches_torch(data_dir, layout):
    """fp32 checkpoint loaded with dtype=BF16 / F16 (the case of the reference's
    published down-cast figure): every tensor equals load_file(...).to(dtype)."""
    fw = get_framework_op("pytorch")
    recs = ck.write_config(ck.configs(0.06)["C1"], os.path.join(data_dir, "conv_C1"))
    path = recs[0]["path"]
    ref = load_file(path, device=DEV)
    for dtype, tdt in [(DType.BF16, torch.bfloat16), (DType.F16, torch.float16), (DType.F8_E4M3, torch.float8_e4m3fn),
                       (DType.F32, torch.float32)]:
        loader = SafeTensorsFileLoader(SingleGroup(), DEV, layout=layout, max_threads=4)
        loader.add_filenames({0: [path]})
        bufs = loader.copy_files_to_device(dtype=dtype)
        for key, t in ref.items():
            got = bufs.get_tensor(key)
            assert got.dtype == tdt and got.shape == t.shape and got.data_ptr() % 16 == 0
            isz = {1: torch.uint8, 2: torch.int16, 4: torch.int32}[tdt.itemsize]
            assert torch.equal(got.view(isz), t.to(tdt).view(isz)), (dtype, key)
        if dtype != DType.F32:  # the file now occupies its converted size only
            data = recs[0]["size"] - recs[0]["header_length"]
            assert fw.get_mem_used() < data * tdt.itemsize / 4 + 128 * len(ref) + 64
            assert loader.frames[next(iter(ref))].dtype == DType.F32  # the header model still describes the file
        bufs.close()
        loader.close()
        assert fw.get_mem_used() == 0


def test_shards_and_copies_of_a_downcast_load(data_dir):
    """After a converting load the tensors in memory are narrower than the file says:
    rank blocks, whole copies and joins must follow the tensors, not the header."""
    from collections import OrderedDict

    from fastsafetensors_amd import StubProcessGroup

    recs = ck.write_config(ck.configs(0.06)["C1"], os.path.join(data_dir, "conv_C1"))
    path = recs[0]["path"]
    ref = {k: v.to(torch.bfloat16) for k, v in load_file(path, device=DEV).items()}
    rank, world = 1, 3
    loader = SafeTensorsFileLoader(StubProcessGroup(rank, world), DEV, max_threads=4)
    loader.add_filenames({rank: [path]})
    bufs = loader.copy_files_to_device(dtype=DType.BF16)
    bufs.auto_mem_delete = False
    two_d = [k for k, v in ref.items() if v.dim() == 2]
    same_rows = [k for k in two_d if ref[k].shape[0] == ref[two_d[0]].shape[0]][:3]
    joined = bufs.get_multi_cols(same_rows, dim=1).get_raw()
    blocks = []
    for k in same_rows:
        b = -(-ref[k].shape[1] // world)
        blocks.append(ref[k][:, rank * b : (rank + 1) * b])
    assert torch.equal(joined.view(torch.int16), torch.cat(blocks, dim=1).view(torch.int16))
    dims = OrderedDict((k, (-1 if v.dim() < 2 else i % 2)) for i, (k, v) in enumerate(ref.items()))
    out = bufs.as_dict(dims)
    for k, dim in dims.items():
        want = ref[k]
        if dim >= 0:
            b = -(-want.shape[dim] // world)
            want = want[(slice(None),) * dim + (slice(rank * b, (rank + 1) * b),)]
        got = out[k].get_raw()
        assert got.dtype == torch.bfloat16 and got.shape == want.shape, k
        assert torch.equal(got.reshape(-1).view(torch.int16), want.reshape(-1).view(torch.int16)), k
    del out, joined
    bufs.close()
    loader.close()
    assert get_framework_op("pytorch").get_mem_used() == 0


def test_loader_downcast_to_wider_type_is_refused(data_dir):
    recs = ck.write_config(ck.configs(0.02)["C5"], os.path.join(data_dir, "conv_C5"))
    loader = SafeTensorsFileLoader(SingleGroup(), DEV, max_threads=4)
    loader.add_filenames({0: [recs[0]["path"]]})
    with pytest.raises(Exception, match="larger sizes is not supported"):
        loader.copy_files_to_device(dtype=DType.BF16)  # the fp8 weights would have to grow
    assert get_framework_op("pytorch").get_mem_used() == 0  # the failed load left no arena behind
    loader.close()
