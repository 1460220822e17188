# SPDX-License-Identifier: Apache-2.0
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def golden():
    def path(name: str) -> str:
        return os.path.join(GOLDEN, name)

    return path


@pytest.fixture(scope="session")
def data_dir(tmp_path_factory):
    """Scratch directory for generated checkpoints (on the repo's disk, not tmpfs)."""
    base = os.environ.get("FSTX_TEST_DIR")
    if base:
        os.makedirs(base, exist_ok=True)
        return base
    return str(tmp_path_factory.mktemp("ckpt"))


GOLDEN_FILES = [
    "a.safetensors",
    "b.safetensors",
    "tiny_gpt2.safetensors",
    "misaligned_header.safetensors",
    "mixed_fp8.safetensors",
    "odd_bytes.safetensors",
    "empty_at_odd.safetensors",
    "f4.safetensors",
]
