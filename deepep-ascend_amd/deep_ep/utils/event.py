"""`EventOverlap`: a recorded stream event plus a one-shot epilogue that runs when the event is
waited on (interface of the reference's deep_ep/utils/event.py)."""
from typing import Any, Callable, Optional, Tuple

import torch

from .._C import EventHandle


class EventOverlap:
    """Waits for `event` on the current stream, then runs the registered epilogue once.

    Attributes:
        event: the recorded event (None once released).
        extra_tensors: tensors this object keeps alive.
    """

    def __init__(self, event: Optional[EventHandle] = None,
                 extra_tensors: Optional[Tuple[torch.Tensor]] = None) -> None:
        self.event = event
        self.extra_tensors = extra_tensors
        self.hook_after_wait: Optional[Callable] = None
        self._release_on_exit = False

    def register_hook_after_wait(self, hook_after_wait: Callable) -> None:
        assert self.hook_after_wait is None, 'A hook is already registered on this `EventOverlap`'
        self.hook_after_wait = hook_after_wait

    def current_stream_wait(self, release_handle: bool = False) -> Any:
        """Block the current stream on the event; returns what the epilogue returned (None if there
        was none, or if it already ran)."""
        assert self.event is not None
        self.event.current_stream_wait()
        hook, self.hook_after_wait = self.hook_after_wait, None
        result = hook() if hook is not None else None
        if release_handle:
            self.event = None
        return result

    def wait(self) -> Any:
        return self.current_stream_wait()

    def __call__(self, release_handle: bool = False) -> 'EventOverlap':
        """`with event_overlap(release_handle=True): ...` drops the event when the block ends."""
        self._release_on_exit = release_handle
        return self

    def __enter__(self) -> Any:
        return self

    def __exit__(self, exc_type: Any, exc_val: Any, exc_tb: Any) -> None:
        if self.event is not None:
            self.current_stream_wait(release_handle=self._release_on_exit)
        self._release_on_exit = False
