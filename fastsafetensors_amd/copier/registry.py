# SPDX-License-Identifier: Apache-2.0
"""Name -> copier factory table (reference: ``fastsafetensors/copier/registry.py:10-37``).

A *factory* takes ``(device, **kwargs)`` once per loader and returns a
*constructor* ``(metadata, device, framework) -> CopierInterface`` that the
loader calls once per file.
"""

from typing import Callable, Dict

from ..common import SafeTensorsMetadata
from ..frameworks import FrameworkOpBase
from ..st_types import Device
from .base import CopierInterface

CopierType = str
CopierConstructFunc = Callable[[SafeTensorsMetadata, Device, FrameworkOpBase], CopierInterface]
CopierConstructorFactory = Callable[..., CopierConstructFunc]

_factories: Dict[CopierType, CopierConstructorFactory] = {}


def register_copier_constructor(copier_type: CopierType):
    def remember(factory: CopierConstructorFactory) -> CopierConstructorFactory:
        _factories[copier_type] = factory
        return factory

    return remember


def create_copier_constructor(copier_type: CopierType, device: Device, **kwargs) -> CopierConstructFunc:
    try:
        factory = _factories[copier_type]
    except KeyError:
        raise KeyError(
            f"Copier type '{copier_type}' is not registered. Available types: {sorted(_factories)}"
        ) from None
    return factory(device, **kwargs)
