"""Single-GPU stand-ins for the reference's deep_ep/comm package.  There is no transport here:
every "rank" of a group is a partition of the same device's arena."""
from typing import Any, Optional, Tuple

import torch


class LocalGroup:
    """Duck-typed process group (`rank()`, `size()`) describing one of `size` virtual partitions
    that live on this GPU; lets `EPBuffer` run one GPU's share of an EP-`size` layout."""

    def __init__(self, rank: int = 0, size: int = 1, name: str = 'local', node: Optional['LocalNode'] = None):
        assert 0 <= rank < size
        self._rank, self._size, self.name, self.node = rank, size, name, node

    def rank(self) -> int:
        return self._rank

    def size(self) -> int:
        return self._size


class LocalNode:
    """All `size` partitions of an EP group in this process, on this GPU.  Build one `EPBuffer` per
    `node.group(rank)`; once the last one exists they are connected: a dispatch of partition s stores
    its packed rows straight into partition r's arena and a combine stores its partials into the arena
    of the partition the token came from, as ranks do through symmetric memory in the reference.
    Nothing waits across partitions, so drive them phase by phase on one stream, which the deferred
    epilogues of the reference API allow:

        events = [buf[r].dispatch(x[r], ..., async_with_compute_stream=True, defer_epilogue=True) for r in ranks]
        results = [ev.current_stream_wait() for ev in events]      # receive side of every partition
    and the same for combine."""

    def __init__(self, size: int, name: str = 'node'):
        assert size > 1
        self.size, self.name = size, name
        self._groups = [LocalGroup(r, size, f'{name}{r}', node=self) for r in range(size)]
        self._runtimes = [None] * size

    def group(self, rank: int) -> LocalGroup:
        return self._groups[rank]

    def register(self, rank: int, runtime: Any) -> None:
        self._runtimes[rank] = runtime
        if all(r is not None for r in self._runtimes):
            type(runtime).connect(self._runtimes)


class LocalCommHandle:
    """What the reference's HCCLCommHandle is to the native runtime: a name."""

    def __init__(self, name: str, group: Any = None):
        self.name, self.group, self.managed = name, group, False

    def get(self) -> str:
        return self.name


_handles = {}


def get_hccl_comm_handle(group: Any, force_new_comm: bool = False) -> LocalCommHandle:
    key = id(group)
    if force_new_comm or key not in _handles:
        _handles[key] = LocalCommHandle(getattr(group, 'name', None) or f'group{group.rank()}of{group.size()}', group)
    return _handles[key]


def destroy_all_managed_hccl_comm() -> None:
    _handles.clear()


def _domain(group_or_buffer: Any) -> Tuple[int, int]:
    context = getattr(group_or_buffer, 'context', None)
    if context is not None:
        return context.get_physical_domain_size()
    return 1, group_or_buffer.size()


def get_physical_domain_size(group_or_buffer: Any) -> Tuple[int, int]:
    """(scale-out, directly addressable) domain sizes: everything is directly addressable."""
    return _domain(group_or_buffer)


def get_logical_domain_size(group_or_buffer: Any, allow_hybrid_mode: Optional[bool] = None) -> Tuple[int, int]:
    return _domain(group_or_buffer)


def barrier(buffer: Any, wait_comm_stream: bool = True, with_cpu_sync: bool = False, sequential: bool = True,
            context_idx: Optional[int] = None) -> None:
    """All partitions share one stream, so the barrier is stream order itself."""
    if with_cpu_sync:
        torch.cuda.current_stream().synchronize()


def get_comm_stream(buffer: Any = None) -> torch.cuda.Stream:
    """EP work runs on the caller's current stream; that is the "communication" stream."""
    return torch.cuda.current_stream()
