# SPDX-License-Identifier: Apache-2.0
"""TEST INFRASTRUCTURE: a copier plug-in that fills a CPU buffer with Python file
I/O.  It exists so that the loader's host logic above the copier boundary
(ordering, bookkeeping, lifetimes) can run where there is no GPU; it follows
the reference's recipe for third-party copiers (copier/example_copier.py:12-54)
and is registered only by the tests that import this module."""
import numpy as np
import torch

from fastsafetensors_amd.copier import CopierInterface, register_copier_constructor
from fastsafetensors_amd.st_types import DType


class PyReadCopier(CopierInterface):
    def __init__(self, metadata, device, framework, log):
        self.metadata, self.device, self.framework, self.log = metadata, device, framework, log

    def submit_io(self, use_buf_register, max_copy_block_size):
        m = self.metadata
        self.log.append(("submit", m.src))
        gbuf = self.framework.alloc_tensor_memory(m.size_bytes - m.header_length, self.device)
        data = np.fromfile(m.src, dtype=np.uint8, offset=m.header_length)
        gbuf.keepalive[: data.size] = torch.from_numpy(data)
        return gbuf

    def wait_io(self, gbuf, dtype=DType.AUTO, noalign=False):
        self.log.append(("wait", self.metadata.src))
        return self.metadata.get_tensors(gbuf, self.device, self.metadata.header_length, dtype)


@register_copier_constructor("pyread_test")
def new_pyread_copier(device, log=None, **kwargs):
    log = log if log is not None else []

    def construct(metadata, device, framework):
        return PyReadCopier(metadata, device, framework, log)

    construct.log = log
    return construct
