from typing import List, Tuple

import torch

from .. import _C
from ..utils.math import align


class BufferAllocator:
    """Plans aligned tensors as meta placeholders first and binds them to device storage later
    (interface of the reference's deep_ep/buffers/allocator.py)."""

    def __init__(self):
        self.alignment = _C.get_num_allocation_alignment()
        self.allocations: List[Tuple[torch.Tensor, int]] = []
        self.num_bytes = 0
        self.materialized = False

    def allocate(self, shape, dtype: torch.dtype) -> torch.Tensor:
        assert not self.materialized, 'A materialized allocation plan cannot be changed'
        placeholder = torch.empty(shape, dtype=dtype, device='meta')
        offset = align(self.num_bytes, self.alignment)
        self.allocations.append((placeholder, offset))
        self.num_bytes = align(offset + placeholder.nbytes, self.alignment)
        return placeholder

    def materialize(self, storage: torch.Tensor) -> None:
        assert not self.materialized, 'An allocation plan can only be materialized once'
        assert storage.is_cuda and storage.is_contiguous() and storage.dtype == torch.uint8
        assert storage.numel() == self.num_bytes
        for placeholder, offset in self.allocations:
            real = storage.narrow(0, offset, placeholder.nbytes).view(placeholder.dtype).view(placeholder.shape)
            torch.utils.swap_tensors(placeholder, real)
        self.materialized = True
