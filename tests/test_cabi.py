# SPDX-License-Identifier: Apache-2.0
"""The shipped library loads and exports exactly what include/fstx.h declares.
No GPU work is started here: only argument checks and host-side helpers."""
import ctypes
import os
import re

import pytest

from conftest import ROOT
from fastsafetensors_amd import _native


def declared_functions():
    text = open(os.path.join(ROOT, "include", "fstx.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fstx_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_list_the_same_functions():
    assert declared_functions() == sorted(_native.EXPORTED_SYMBOLS)


def test_library_exports_every_declared_symbol():
    assert os.path.exists(_native.library_path()), "libfstx.so is not built"
    raw = ctypes.CDLL(_native.library_path())
    for name in declared_functions():
        assert hasattr(raw, name), name
    assert _native.lib().fstx_abi_version() == _native.FSTX_ABI_VERSION == 4


def test_constants_match_the_header():
    text = open(os.path.join(ROOT, "include", "fstx.h")).read()
    assert int(re.search(r"#define FSTX_BATCH_MAX (\d+)", text).group(1)) == _native.FSTX_BATCH_MAX
    assert int(re.search(r"#define FSTX_ABI_VERSION (\d+)", text).group(1)) == _native.FSTX_ABI_VERSION
    assert ctypes.sizeof(_native.FstxConfig) == 56 and ctypes.sizeof(_native.FstxMetrics) == 208
    assert ctypes.sizeof(_native.FstxCopyDesc) == 24 and ctypes.sizeof(_native.FstxSliceDesc) == 40


def test_header_is_plain_c_and_struct_layouts_match_the_binding(tmp_path):
    """include/fstx.h compiles as C99 on its own, and a C compiler lays the structs out
    exactly as the ctypes binding does (size and the offset of every field)."""
    import shutil
    import subprocess

    cc = shutil.which("gcc") or shutil.which("cc")
    if cc is None:
        pytest.skip("no C compiler")
    pairs = {"fstx_config": _native.FstxConfig, "fstx_metrics": _native.FstxMetrics, "fstx_copy_desc": _native.FstxCopyDesc,
             "fstx_slice_desc": _native.FstxSliceDesc, "fstx_slice2d_desc": _native.FstxSlice2dDesc,
             "fstx_join_src": _native.FstxJoinSrc, "fstx_convert_desc": _native.FstxConvertDesc}
    lines = ['#include <stdio.h>', '#include <stddef.h>', '#include "fstx.h"', "int main(void) {"]
    for cname, ctype in pairs.items():
        lines.append(f'  printf("{cname} %zu\\n", sizeof({cname}));')
        for field, _t in ctype._fields_:
            lines.append(f'  printf("{cname}.{field} %zu\\n", offsetof({cname}, {field}));')
    lines += ['  printf("FSTX_JOIN_MAX %d\\n", FSTX_JOIN_MAX);', "  return 0;", "}"]
    src = tmp_path / "layout.c"
    src.write_text("\n".join(lines))
    exe = tmp_path / "layout"
    subprocess.run([cc, "-std=c99", "-Wall", "-Werror", "-pedantic", f"-I{os.path.join(ROOT, 'include')}", str(src), "-o", str(exe)],
                   check=True)
    got = dict(l.split() for l in subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.splitlines())
    for cname, ctype in pairs.items():
        assert int(got[cname]) == ctypes.sizeof(ctype), cname
        for field, _t in ctype._fields_:
            assert int(got[f"{cname}.{field}"]) == getattr(ctype, field).offset, (cname, field)
    assert int(got["FSTX_JOIN_MAX"]) == _native.FSTX_JOIN_MAX


def test_host_helpers():
    assert _native.get_alignment_size() == 4096  # reference: tests/smoke_import_cpp.py:34-40
    assert _native.get_cpp_metrics().bounce_buffer_bytes == 0
    p = _native.cpu_malloc(10_000)
    assert p and p % 4096 == 0
    ctypes.memset(p, 0x41, 16)
    assert _native.read_buffer(p, 4) == b"AAAA"
    _native.cpu_free(p)
    assert _native.strerror(-10004).startswith("fstx: file ended")
    assert "No such file" in _native.strerror(-2)
    assert _native.strerror(0) == "ok"
    assert _native.set_numa_node(-1) == 0
    _native.set_debug_log(False)


def test_argument_checks_need_no_gpu():
    lib = _native.lib()
    assert lib.fstx_realign_copy_batch(None, 0, None) == 0  # empty batch: nothing launched
    assert lib.fstx_slice_copy_batch(None, 0, None) == 0
    assert lib.fstx_realign_copy_batch(None, 3, None) == -10001
    too_many = (_native.FstxCopyDesc * (_native.FSTX_BATCH_MAX + 1))()
    assert lib.fstx_realign_copy_batch(too_many, len(too_many), None) == -10008
    assert lib.fstx_ctx_create(None, None) == -10001
    assert lib.fstx_ctx_destroy(None) == -10001
    assert lib.fstx_get_device_pci_bus(0, None, 0) == -10001


def test_without_a_gpu_the_product_refuses_loudly():
    import torch

    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    from fastsafetensors_amd import SafeTensorsFileLoader, SingleGroup

    assert _native.device_count() == 0 and not _native.is_hip_found()
    assert _native.get_device_pci_bus(0) == ""
    with pytest.raises(Exception, match="HIP device"):
        SafeTensorsFileLoader(SingleGroup(), "cpu")  # no CPU path behind the loader
    with pytest.raises(Exception, match="no HIP device is visible"):
        SafeTensorsFileLoader(SingleGroup(), "cuda:0")  # and no silent fallback either
    with pytest.raises(_native.NativeError, match="no HIP device"):
        _native.Reader(0)


def test_the_product_never_reaches_for_the_oracle_or_scratch_files():
    """The oracle is test infrastructure: nothing under fastsafetensors_amd/ may import it
    (or anything from the builder's scratch directory), and bench.py may only inside its
    CPU baseline."""
    import ast
    import glob

    def imported(path):
        mods = set()
        for node in ast.walk(ast.parse(open(path).read())):
            if isinstance(node, ast.Import):
                mods |= {a.name.split(".")[0] for a in node.names}
            elif isinstance(node, ast.ImportFrom) and node.module and node.level == 0:
                mods.add(node.module.split(".")[0])
        return mods

    for path in glob.glob(os.path.join(ROOT, "fastsafetensors_amd", "**", "*.py"), recursive=True):
        assert not imported(path) & {"oracle", "_work"}, path
    tree = ast.parse(open(os.path.join(ROOT, "bench.py")).read())
    for fn in [n for n in tree.body if isinstance(n, ast.FunctionDef)]:
        uses = any(isinstance(n, ast.ImportFrom) and n.module == "oracle" for n in ast.walk(fn))
        assert uses == (fn.name == "cpu_baseline"), fn.name
    assert not any(isinstance(n, (ast.Import, ast.ImportFrom)) and "oracle" in ast.dump(n) for n in tree.body)


def test_the_reference_side_stub_matches_the_header():
    """The integration guide at the repository root shows the ctypes stub a maintainer of the reference
    would add.  Its code block must parse, and every ``_lib.fstx_*.argtypes`` / ``.restype`` line and the ``_Config``
    fields in it must say what this package's own binding says (which the test above ties to
    ``include/fstx.h``)."""
    import ast

    text = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    blocks = re.findall(r"```python\n(.*?)```", text, flags=re.S)
    stub = next(b for b in blocks if "fastsafetensors/copier/mi355x.py" in b)
    tree = ast.parse(stub)

    def ctype(node):
        src = ast.unparse(node)
        return eval(src, {"ctypes": ctypes, "_Config": _native.FstxConfig})

    seen = {}
    for node in ast.walk(tree):
        if isinstance(node, ast.Assign) and isinstance(node.targets[0], ast.Attribute):
            target = node.targets[0]
            if (isinstance(target.value, ast.Attribute) and isinstance(target.value.value, ast.Name)
                    and target.value.value.id == "_lib" and target.attr in ("argtypes", "restype")):
                seen.setdefault(target.value.attr, {})[target.attr] = ctype(node.value)
        if isinstance(node, ast.ClassDef) and node.name == "_Config":
            fields = next(n for n in node.body if isinstance(n, ast.Assign) and n.targets[0].id == "_fields_")
            got = [(name, ctype_) for name, ctype_ in ctype(fields.value)]
            assert got == list(_native.FstxConfig._fields_)
    assert len(seen) >= 9
    for name, sig in seen.items():
        restype, argtypes = _native._SIGNATURES[name]
        if "argtypes" in sig:
            assert sig["argtypes"] == argtypes, name
        assert sig.get("restype", ctypes.c_int) == restype, name
    # every library function the stub calls has its signature declared
    called = set(re.findall(r"_lib\.(fstx_\w+)\(", stub))
    assert called <= set(seen), called - set(seen)


def test_the_plain_c_program_calls_every_declared_entry_point():
    """tests/cabi_native/cabi_check.c (run on the GPU by test_loader_gpu) is the C-side user of the
    header: every function include/fstx.h declares appears in it as a call."""
    import re

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    header = open(os.path.join(root, "include", "fstx.h")).read()
    program = open(os.path.join(root, "tests", "cabi_native", "cabi_check.c")).read()
    code = re.sub(r"/\*.*?\*/", "", header, flags=re.S)  # comments mention names followed by a bracket
    declared = set(re.findall(r"\b(fstx_[a-z0-9_]+)\s*\(", code))
    assert declared == set(_native.EXPORTED_SYMBOLS)
    missing = sorted(name for name in declared if not re.search(r"\b%s\s*\(" % name, program))
    assert not missing, missing
