"""deep_ep on MI355X: the EPBuffer dispatch/combine path of DeepEP-Ascend, backed by hand-written
gfx950 kernels.  Public names follow the reference's deep_ep/__init__.py for this path."""
from . import _C
from ._C import init_jit as _init_jit

_init_jit()

from . import comm                                                                   # noqa: E402
from .comm import (LocalGroup, LocalNode, destroy_all_managed_hccl_comm, get_logical_domain_size,   # noqa: E402
                   get_physical_domain_size)
from .buffers.allocator import BufferAllocator                                       # noqa: E402
from .buffers.base import BufferBase                                                 # noqa: E402
from .buffers.ep import EPBuffer, EPHandle                                           # noqa: E402
from ._C import (get_num_allocation_alignment, get_num_rdma_alignment,               # noqa: E402
                 get_num_tma_alignment, topk_idx_t)
from .utils.event import EventHandle, EventOverlap                                   # noqa: E402


def init_jit() -> None:
    """Kept for API compatibility: kernels are built ahead of time and loaded on first use."""
    _init_jit()


__version__ = '1.0.0'
