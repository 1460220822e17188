# SPDX-License-Identifier: Apache-2.0
"""Writes the small checkpoint fixtures of this directory.

Run from the repository root: ``python tests/golden/make_golden.py``.
Every file is fully determined by closed forms, so the tests recompute the
expected values instead of trusting the files:

``a.safetensors`` / ``b.safetensors``
    Copied byte for byte from the reference's ``examples/`` (they are data files
    its own tests hold; generator: ``examples/gen.py:5-14``).  One F16 ``[16, 8]``
    tensor ``a0`` / ``b0`` whose row ``i`` is all ``float16(i)``; JSON length 96,
    so ``header_length = 104`` and ``104 % 16 == 8``.  Not rewritten here.
``tiny_gpt2.safetensors``
    The closed-form file of the reference's ``tests/unit/conftest.py:68-115``:
    12 layers x {mlp.c_proj.weight 8x16 (+0), mlp.c_fc.weight 16x8 (+100),
    attn.c_proj.weight 8x8 (+200), attn.c_proj.bias 8 (+300)}, fp16,
    ``arange(rows*cols).reshape(rows, cols) + layer*1000 + offset``; written by
    the stock ``safetensors`` writer.
``misaligned_header.safetensors``
    Same tensors, JSON padded to a length = 2 (mod 8): every tensor's file
    offset is odd-word misaligned.
``mixed_fp8.safetensors``
    fp8 (e4m3) matrices with fp32 scalar scales and bf16 vectors: byte ``k`` of
    fp8 tensor ``t`` is ``(k * 7 + t) % 256`` skipping NaN patterns, scales are
    ``0.5 ** t``, bf16 vectors are ``arange``; the 4-byte scalars come first in
    the file, so the later tensors sit at offsets that are not multiples of 16.
``f4.safetensors``
    ``arange(64, uint8).reshape(8, 8)`` viewed as packed fp4 pairs, logical shape
    ``[8, 16]`` (the reference's ``test_float4_e2m1fn_x2`` recipe,
    ``tests/unit/test_fastsafetensors.py:700-702``).
``odd_bytes.safetensors``
    U8 tensors of 3, 5 and 33 bytes in front of I16/F32 tensors, written in that
    order (not the stock order), so that wider tensors start at odd addresses.
``empty_at_odd.safetensors``
    Zero-byte F32 ``[0, 4]``, I64 ``[0]`` and F16 ``[3, 0]`` tensors whose offsets (3, 3 and 20)
    are not multiples of their element sizes, between U8 / F16 tensors that hold data.
"""
import os
import sys

import torch
from safetensors.torch import save_file

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from fastsafetensors_amd.checkpoints import TensorSpec, build_header  # noqa: E402
from fastsafetensors_amd.st_types import DType  # noqa: E402


def tiny_gpt2_tensors():
    def mat(rows, cols, off):
        return torch.arange(rows * cols, dtype=torch.float16).reshape(rows, cols) + off

    out = {}
    for layer in range(12):
        base = layer * 1000
        out[f"h.{layer}.mlp.c_proj.weight"] = mat(8, 16, base)
        out[f"h.{layer}.mlp.c_fc.weight"] = mat(16, 8, base + 100)
        out[f"h.{layer}.attn.c_proj.weight"] = mat(8, 8, base + 200)
        out[f"h.{layer}.attn.c_proj.bias"] = torch.arange(8, dtype=torch.float16) + (base + 300)
    return out


def raw(t: torch.Tensor) -> bytes:
    return t.contiguous().reshape(-1).view(torch.uint8).numpy().tobytes()


def write_raw(path, items, metadata, pad_rem):
    """items: list of (name, DType, shape, bytes) written in the given order."""
    specs = [TensorSpec(n, d, tuple(s)) for n, d, s, _ in items]
    with open(path, "wb") as f:
        f.write(build_header(specs, metadata, 8, pad_rem))
        for _, _, _, b in items:
            f.write(b)


def fp8_bytes(t: int, n: int) -> bytes:
    vals = [(k * 7 + t) % 256 for k in range(n)]
    return bytes(v if v & 0x7F != 0x7F else v - 1 for v in vals)  # 0x7f / 0xff are NaN in e4m3fn


def mixed_fp8_items():
    items = []
    for t in range(5):
        items.append((f"w{t}.weight_scale", DType.F32, [], raw(torch.tensor(0.5**t, dtype=torch.float32))))
    for t in range(3):
        items.append((f"norm{t}.weight", DType.BF16, [24], raw(torch.arange(24, dtype=torch.float32).to(torch.bfloat16) + t)))
    for t in range(5):
        rows, cols = 6 + t, 10 + 3 * t
        items.append((f"w{t}.weight", DType.F8_E4M3, [rows, cols], fp8_bytes(t, rows * cols)))
    return items


def odd_bytes_items():
    return [
        ("u3", DType.U8, [3], bytes(range(3))),
        ("i16", DType.I16, [4, 5], raw(torch.arange(20, dtype=torch.int16) - 7)),
        ("u5", DType.U8, [5], bytes(range(10, 15))),
        ("f32", DType.F32, [3, 7], raw(torch.arange(21, dtype=torch.float32) * 0.25)),
        ("u33", DType.U8, [33], bytes(range(100, 133))),
        ("f64", DType.F64, [2, 2], raw(torch.arange(4, dtype=torch.float64) - 1.5)),
    ]


def empty_at_odd_items():
    return [
        ("u3", DType.U8, [3], bytes(range(3))),
        ("e32", DType.F32, [0, 4], b""),
        ("e64", DType.I64, [0], b""),
        ("h", DType.F16, [2, 4], raw(torch.arange(8, dtype=torch.float16) - 2)),
        ("u1", DType.U8, [1], b"\x7f"),
        ("e16", DType.F16, [3, 0], b""),
        ("tail", DType.U8, [4], bytes(range(200, 204))),
    ]


def main():
    save_file(tiny_gpt2_tensors(), os.path.join(HERE, "tiny_gpt2.safetensors"), metadata={"fst": "tiny-gpt2"})
    tiny = tiny_gpt2_tensors()
    items = [(k, DType.F16, list(v.shape), raw(v)) for k, v in sorted(tiny.items())]
    write_raw(os.path.join(HERE, "misaligned_header.safetensors"), items, {"fst": "misaligned"}, 2)
    write_raw(os.path.join(HERE, "mixed_fp8.safetensors"), mixed_fp8_items(), {"fst": "mixed"}, 0)
    write_raw(os.path.join(HERE, "odd_bytes.safetensors"), odd_bytes_items(), None, 5)
    write_raw(os.path.join(HERE, "empty_at_odd.safetensors"), empty_at_odd_items(), None, 3)
    u8 = torch.arange(64, dtype=torch.uint8).reshape(8, 8)
    save_file({"a": u8.view(torch.float4_e2m1fn_x2)}, os.path.join(HERE, "f4.safetensors"), metadata={"fst": "sample"})
    for name in sorted(os.listdir(HERE)):
        if name.endswith(".safetensors"):
            print(name, os.path.getsize(os.path.join(HERE, name)))


if __name__ == "__main__":
    main()
