"""Two-step allocation of the tensors that live in the load-balancing storage of a buffer: sizes are
planned on meta tensors before the buffer exists, and once its storage is there the very same
tensor objects are given real memory (interface of the reference's deep_ep/buffers/allocator.py;
test: tests/buffer/test_allocation.py:42-50)."""
import dataclasses
from typing import List, Tuple

import torch

from .. import _C


@dataclasses.dataclass
class _Planned:
    tensor: torch.Tensor      # meta placeholder handed to the caller
    offset: int               # byte offset inside the storage

    def __iter__(self):       # unpacks as (tensor, offset)
        return iter((self.tensor, self.offset))


class BufferAllocator:
    def __init__(self):
        self.alignment: int = _C.get_num_allocation_alignment()
        self.allocations: List[_Planned] = []
        self.materialized = False

    def _round(self, n: int) -> int:
        return -(-n // self.alignment) * self.alignment

    @property
    def num_bytes(self) -> int:
        """Storage the plan needs: every tensor starts and ends on an allocation boundary."""
        if not self.allocations:
            return 0
        last = self.allocations[-1]
        return self._round(last.offset + last.tensor.nbytes)

    def allocate(self, shape, dtype: torch.dtype) -> torch.Tensor:
        if self.materialized:
            raise AssertionError('A materialized allocation plan cannot be changed')
        planned = _Planned(torch.empty(shape, dtype=dtype, device='meta'), self.num_bytes)
        self.allocations.append(planned)
        return planned.tensor

    def materialize(self, storage: torch.Tensor) -> None:
        if self.materialized:
            raise AssertionError('An allocation plan can only be materialized once')
        assert storage.is_cuda and storage.dtype == torch.uint8 and storage.is_contiguous()
        assert storage.numel() == self.num_bytes, 'the storage must have exactly the planned size'
        for planned in self.allocations:
            meta = planned.tensor
            backing = storage[planned.offset:planned.offset + meta.nbytes].view(meta.dtype).view(meta.shape)
            torch.utils.swap_tensors(meta, backing)          # the caller's object now owns device memory
        self.materialized = True

    def offsets(self) -> Tuple[int, ...]:
        return tuple(p.offset for p in self.allocations)
