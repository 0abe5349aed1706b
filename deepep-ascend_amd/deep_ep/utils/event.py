"""`EventOverlap` ties two things to one point of a stream: an event recorded after some enqueued
work, and an optional epilogue (a callable) that must run once the current stream has been ordered
behind that event -- the second half of a deferred dispatch or combine.  Same surface as the
reference's deep_ep/utils/event.py."""
from typing import Any, Callable, Optional, Sequence

import torch

from .._C import EventHandle

_NO_RESULT = None


class EventOverlap:
    def __init__(self, event: Optional[EventHandle] = None,
                 extra_tensors: Optional[Sequence[torch.Tensor]] = None) -> None:
        self.event = event                    # dropped when a wait is asked to release it
        self.extra_tensors = extra_tensors    # kept alive for as long as this object lives
        self._epilogue: Optional[Callable[[], Any]] = None
        self._drop_event_at_exit = False

    # -- epilogue ---------------------------------------------------------------------------------
    @property
    def hook_after_wait(self) -> Optional[Callable[[], Any]]:
        return self._epilogue

    def register_hook_after_wait(self, hook_after_wait: Callable[[], Any]) -> None:
        if self._epilogue is not None:
            raise AssertionError('A hook is already registered on this `EventOverlap`')
        self._epilogue = hook_after_wait

    def _run_epilogue_once(self) -> Any:
        epilogue, self._epilogue = self._epilogue, None
        return _NO_RESULT if epilogue is None else epilogue()

    # -- waiting ----------------------------------------------------------------------------------
    def current_stream_wait(self, release_handle: bool = False) -> Any:
        """Orders the current stream behind the event and runs the epilogue (at most once over the
        life of this object); returns whatever the epilogue returned."""
        if self.event is None:
            raise AssertionError('the event of this `EventOverlap` has been released')
        self.event.current_stream_wait()
        outcome = self._run_epilogue_once()
        if release_handle:
            self.event = None
        return outcome

    def wait(self) -> Any:
        return self.current_stream_wait(release_handle=False)

    # -- `with overlap:` / `with overlap(release_handle=True):` --------------------------------------
    def __call__(self, release_handle: bool = False) -> 'EventOverlap':
        self._drop_event_at_exit = bool(release_handle)
        return self                           # no second wrapper: the event keeps a single owner

    def __enter__(self) -> 'EventOverlap':
        return self

    def __exit__(self, exc_type: Any, exc_val: Any, exc_tb: Any) -> None:
        drop, self._drop_event_at_exit = self._drop_event_at_exit, False
        if self.event is not None:
            self.current_stream_wait(release_handle=drop)
