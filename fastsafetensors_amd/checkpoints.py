# SPDX-License-Identifier: Apache-2.0
"""Writer for synthetic ``.safetensors`` checkpoints of the benchmark shapes.

The stock ``safetensors`` writer always pads its JSON header so that the data
section starts on an 8-byte boundary.  The load path must also cope with files
whose header length is arbitrary (the reference's committed fixture
``examples/a.safetensors`` has ``header_length % 16 == 8``), so this module
writes the container itself: ``u64le N | JSON padded with spaces to N bytes |
tensor bytes``, tensors ordered like the stock writer does (larger dtype
alignment first, then by name), and ``N`` padded to any residue asked for.

Values follow one recipe everywhere: tensor ``i`` of a file is
``randn(shape, seed = seed_base + i) * 0.02`` cast to the target dtype, norm
weights are ones, fp8 weights are ``clamp(randn * 0.02 / scale, -448, 448)``
next to a scalar fp32 ``weight_scale``.  Large tensors are produced in row
chunks so that a 70B-shaped checkpoint never needs more than a few hundred MiB
of host memory.
"""

import hashlib
import json
import os
from dataclasses import dataclass
from typing import Callable, Dict, Iterable, List, Optional, Sequence, Tuple

import torch

from .st_types import DType, dtype_bits

TORCH_DTYPE = {
    DType.F32: torch.float32,
    DType.F16: torch.float16,
    DType.BF16: torch.bfloat16,
    DType.F8_E4M3: torch.float8_e4m3fn,
    DType.F8_E5M2: torch.float8_e5m2,
    DType.I8: torch.int8,
    DType.U8: torch.uint8,
    DType.I32: torch.int32,
    DType.I64: torch.int64,
    DType.F64: torch.float64,
}

CHUNK_ELEMS = 64 * 1024 * 1024


@dataclass
class TensorSpec:
    name: str
    dtype: DType
    shape: Tuple[int, ...]
    fill: str = "randn"  # "randn" | "ones" | "fp8" | "scale" | "arange"
    scale: float = 1.0   # divisor of the fp8 recipe / value of a "scale" tensor

    @property
    def nbytes(self) -> int:
        n = 1
        for s in self.shape:
            n *= s
        return n * dtype_bits(self.dtype) // 8


def stock_order(specs: Sequence[TensorSpec]) -> List[TensorSpec]:
    """Order of the stock writer: descending dtype alignment, then name."""
    return sorted(specs, key=lambda s: (-max(1, dtype_bits(s.dtype) // 8), s.name))


def build_header(
    specs: Sequence[TensorSpec], metadata: Optional[Dict[str, str]] = None,
    pad_mod: int = 8, pad_rem: int = 0,
) -> bytes:
    """``u64le N`` + JSON, space-padded until ``N % pad_mod == pad_rem``.

    ``pad_mod=8, pad_rem=0`` reproduces the stock writer (``(8 + N) % 8 == 0``).
    """
    table: Dict[str, object] = {}
    if metadata:
        table["__metadata__"] = metadata
    at = 0
    for s in specs:
        table[s.name] = {"dtype": s.dtype.value, "shape": list(s.shape), "data_offsets": [at, at + s.nbytes]}
        at += s.nbytes
    text = json.dumps(table, separators=(",", ":")).encode("utf-8")
    text += b" " * ((pad_rem - len(text)) % pad_mod)
    return len(text).to_bytes(8, "little") + text


def _chunks(spec: TensorSpec) -> Iterable[Tuple[int, ...]]:
    """Shapes of the row chunks a tensor is generated in."""
    if not spec.shape:
        yield ()
        return
    row = 1
    for s in spec.shape[1:]:
        row *= s
    rows_per = max(1, CHUNK_ELEMS // max(row, 1))
    done = 0
    while done < spec.shape[0]:
        take = min(rows_per, spec.shape[0] - done)
        yield (take,) + tuple(spec.shape[1:])
        done += take
    if spec.shape[0] == 0:
        yield tuple(spec.shape)


def tensor_chunks(spec: TensorSpec, seed: int, device: str = "cpu") -> Iterable[torch.Tensor]:
    """The tensor's values, chunk by chunk along dim 0, on ``device``."""
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    tdt = TORCH_DTYPE[spec.dtype]
    for i, shape in enumerate(_chunks(spec)):
        if spec.fill == "ones":
            t = torch.ones(shape, dtype=tdt, device=device)
        elif spec.fill == "scale":
            t = torch.full(shape, spec.scale, dtype=tdt, device=device)
        elif spec.fill == "arange":
            n = 1
            for s in shape:
                n *= s
            t = (torch.arange(n, dtype=torch.int64, device=device) % 251).reshape(shape).to(tdt)
        else:
            x = torch.randn(shape, generator=gen, dtype=torch.float32, device=device) * 0.02
            if spec.fill == "fp8":
                x = (x / spec.scale).clamp_(-448.0, 448.0)
            t = x.to(tdt)
        yield t


def write_checkpoint(
    path: str,
    specs: Sequence[TensorSpec],
    seed_base: int = 0,
    metadata: Optional[Dict[str, str]] = None,
    pad_mod: int = 8,
    pad_rem: int = 0,
    device: str = "cpu",
    reorder: bool = True,
    trailing: int = 0,
    sha256: bool = True,
    on_chunk: Optional[Callable[[TensorSpec, torch.Tensor], None]] = None,
) -> Dict[str, object]:
    """Write one file; returns ``{"path", "size", "header_length", "sha256", "specs"}``.

    ``sha256`` covers the whole file (``None`` when switched off).  ``trailing``
    appends that many zero bytes after the last tensor (the format allows it).
    ``on_chunk(spec, chunk)`` sees every generated chunk on the generating
    device before it is written, e.g. to keep checksums.
    """
    ordered = stock_order(specs) if reorder else list(specs)
    header = build_header(ordered, metadata, pad_mod, pad_rem)
    digest = hashlib.sha256() if sha256 else _NoDigest()
    tmp = f"{path}.{os.getpid()}.tmp"
    with open(tmp, "wb", buffering=0) as f:
        f.write(header)
        digest.update(header)
        for i, spec in enumerate(ordered):
            for t in tensor_chunks(spec, seed_base + i, device):
                if not t.numel():
                    continue
                if on_chunk is not None:
                    on_chunk(spec, t)
                raw = memoryview(t.contiguous().reshape(-1).view(torch.uint8).cpu().numpy())
                f.write(raw)
                digest.update(raw)
        if trailing:
            f.write(b"\0" * trailing)
            digest.update(b"\0" * trailing)
        size = f.tell()
    os.replace(tmp, path)
    return {"path": path, "size": size, "header_length": len(header), "sha256": digest.hexdigest(),
            "specs": ordered}


def tensor_checksum(t: torch.Tensor) -> Tuple[int, int]:
    """Two order-sensitive 64-bit check words of a tensor's bytes, computed on the
    tensor's device: the sum of its 32-bit words and the sum of those words weighted
    by their position (mod 8191).  A shifted, swapped or stale region changes them."""
    b = t.contiguous().reshape(-1).view(torch.uint8)
    n4 = b.numel() // 4 * 4
    w = b[:n4].view(torch.int32).to(torch.int64)
    idx = torch.arange(w.numel(), device=w.device, dtype=torch.int64) % 8191 + 1
    tail = int(b[n4:].to(torch.int64).sum().item()) if n4 < b.numel() else 0
    return int(w.sum().item()) + tail, int((w * idx).sum().item())


class _NoDigest:
    def update(self, _b) -> None:
        pass

    def hexdigest(self) -> None:
        return None


# ---- the benchmark shapes ---------------------------------------------------------


def gpt2_specs(n_layer: int, d: int, vocab: int, ctx: int, dtype: DType) -> List[TensorSpec]:
    out = [TensorSpec("wte.weight", dtype, (vocab, d)), TensorSpec("wpe.weight", dtype, (ctx, d))]
    for i in range(n_layer):
        p = f"h.{i}."
        out += [
            TensorSpec(p + "ln_1.weight", dtype, (d,)), TensorSpec(p + "ln_1.bias", dtype, (d,)),
            TensorSpec(p + "attn.c_attn.weight", dtype, (d, 3 * d)), TensorSpec(p + "attn.c_attn.bias", dtype, (3 * d,)),
            TensorSpec(p + "attn.c_proj.weight", dtype, (d, d)), TensorSpec(p + "attn.c_proj.bias", dtype, (d,)),
            TensorSpec(p + "ln_2.weight", dtype, (d,)), TensorSpec(p + "ln_2.bias", dtype, (d,)),
            TensorSpec(p + "mlp.c_fc.weight", dtype, (d, 4 * d)), TensorSpec(p + "mlp.c_fc.bias", dtype, (4 * d,)),
            TensorSpec(p + "mlp.c_proj.weight", dtype, (4 * d, d)), TensorSpec(p + "mlp.c_proj.bias", dtype, (d,)),
        ]
    out += [TensorSpec("ln_f.weight", dtype, (d,)), TensorSpec("ln_f.bias", dtype, (d,))]
    return out


def llama_layer_specs(i: int, d: int, kv_dim: int, ffn: int, dtype: DType, fp8: bool = False) -> List[TensorSpec]:
    p = f"model.layers.{i}."
    lin = [
        ("self_attn.q_proj", (d, d)), ("self_attn.k_proj", (kv_dim, d)), ("self_attn.v_proj", (kv_dim, d)),
        ("self_attn.o_proj", (d, d)), ("mlp.gate_proj", (ffn, d)), ("mlp.up_proj", (ffn, d)),
        ("mlp.down_proj", (d, ffn)),
    ]
    out: List[TensorSpec] = []
    for name, shape in lin:
        if fp8:
            scale = 0.02 / 100.0
            out.append(TensorSpec(p + name + ".weight", DType.F8_E4M3, shape, "fp8", scale))
            out.append(TensorSpec(p + name + ".weight_scale", DType.F32, (), "scale", scale))
        else:
            out.append(TensorSpec(p + name + ".weight", dtype, shape))
    out.append(TensorSpec(p + "input_layernorm.weight", dtype, (d,), "ones"))
    out.append(TensorSpec(p + "post_attention_layernorm.weight", dtype, (d,), "ones"))
    return out


def llama_files(
    n_layer: int, d: int, kv_dim: int, ffn: int, vocab: int, n_files: int, dtype: DType = DType.BF16,
    fp8: bool = False,
) -> List[List[TensorSpec]]:
    """Per-file tensor lists: layers split evenly, embeddings in the first file,
    final norm and ``lm_head`` in the last."""
    files: List[List[TensorSpec]] = [[] for _ in range(n_files)]
    files[0].append(TensorSpec("model.embed_tokens.weight", dtype, (vocab, d)))
    for i in range(n_layer):
        files[min(i * n_files // n_layer, n_files - 1)] += llama_layer_specs(i, d, kv_dim, ffn, dtype, fp8)
    files[-1].append(TensorSpec("model.norm.weight", dtype, (d,), "ones"))
    files[-1].append(TensorSpec("lm_head.weight", dtype, (vocab, d)))
    return files


@dataclass
class CheckpointConfig:
    key: str
    title: str
    files: Callable[[], List[List[TensorSpec]]]
    pad_rem: int = 0  # residue of the JSON length modulo 8


def _scaled(v: int, s: float, q: int = 16) -> int:
    return max(q, int(v * s) // q * q)


def configs(scale: float = 1.0) -> Dict[str, CheckpointConfig]:
    """The five benchmark checkpoints; ``scale < 1`` shrinks widths and vocabularies
    (layer counts stay) to make test-sized files of the same structure."""
    s = scale
    return {
        "C1": CheckpointConfig("C1", "GPT-2-small fp32, 1 file",
                               lambda: [gpt2_specs(12, _scaled(768, s), _scaled(50257, s, 1), _scaled(1024, s), DType.F32)]),
        "C2": CheckpointConfig("C2", "GPT-2-medium fp16, header length = 2 mod 8, 1 file",
                               lambda: [gpt2_specs(24, _scaled(1024, s), _scaled(50257, s, 1), _scaled(1024, s), DType.F16)],
                               pad_rem=2),
        "C3": CheckpointConfig("C3", "Llama-3-8B bf16, 4 files",
                               lambda: llama_files(32, _scaled(4096, s), _scaled(1024, s), _scaled(14336, s), _scaled(128256, s), 4)),
        "C4": CheckpointConfig("C4", "Llama-2-13B bf16, 3 files",
                               lambda: llama_files(40, _scaled(5120, s), _scaled(5120, s), _scaled(13824, s), _scaled(32000, s), 3)),
        "C5": CheckpointConfig("C5", "Llama-3-70B fp8 + bf16 + fp32 scalars, 15 files",
                               lambda: llama_files(80, _scaled(8192, s), _scaled(1024, s), _scaled(28672, s), _scaled(128256, s), 15, fp8=True)),
    }


def write_config(
    cfg: CheckpointConfig, directory: str, seed_base: int = 1234, device: str = "cpu",
    sha256: bool = True, on_chunk: Optional[Callable[[TensorSpec, torch.Tensor], None]] = None,
) -> List[Dict[str, object]]:
    """Write all files of ``cfg`` into ``directory``; returns ``write_checkpoint`` records."""
    os.makedirs(directory, exist_ok=True)
    file_specs = cfg.files()
    out = []
    for k, specs in enumerate(file_specs):
        name = f"{cfg.key.lower()}-{k + 1:05d}-of-{len(file_specs):05d}.safetensors"
        out.append(
            write_checkpoint(
                os.path.join(directory, name), specs, seed_base + 100_000 * k,
                metadata={"format": "pt"}, pad_mod=8, pad_rem=cfg.pad_rem, device=device,
                sha256=sha256, on_chunk=on_chunk,
            )
        )
    return out


# dims along which a tensor-parallel rank cuts the Llama tensors (q/k/v/gate/up/embed
# by rows, o/down by columns; everything else is replicated)
def llama_shard_dim(name: str) -> int:
    if name.endswith("weight_scale"):
        return -1
    for part in ("q_proj", "k_proj", "v_proj", "gate_proj", "up_proj", "embed_tokens", "lm_head"):
        if part in name:
            return 0
    for part in ("o_proj", "down_proj"):
        if part in name:
            return 1
    return -1
