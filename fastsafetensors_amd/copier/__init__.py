# SPDX-License-Identifier: Apache-2.0
from .base import CopierInterface, DummyDeviceBuffer
from .mi355x import MI355XFileCopier
from .registry import (
    CopierConstructFunc,
    CopierType,
    create_copier_constructor,
    register_copier_constructor,
)

__all__ = [
    "CopierInterface",
    "DummyDeviceBuffer",
    "MI355XFileCopier",
    "CopierConstructFunc",
    "CopierType",
    "create_copier_constructor",
    "register_copier_constructor",
]
