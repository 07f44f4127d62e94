"""`EventOverlap`: what dispatch / combine hand back for stream overlap.  Same public surface as the reference's
deep_ep/utils/event.py:8-96 (`event`, `extra_tensors`, `current_stream_wait`, `register_hook_after_wait`, call and
`with` forms); the state machine below is this package's own."""
from typing import Any, Callable, Optional, Sequence

import torch

from .._binding import EventHandle


class EventOverlap:
    """An event recorded behind the routing kernels of one call.

    `event` is None for calls that already ordered themselves with the caller's stream.  `extra_tensors` keeps the
    tensors of an asynchronous call alive until the object goes away.  One callback can be attached; it fires on the
    first wait (the epilogue of a deterministic call uses it).
    """

    def __init__(self, event: Optional[EventHandle] = None,
                 extra_tensors: Optional[Sequence[torch.Tensor]] = None) -> None:
        self.event, self.extra_tensors = event, extra_tensors
        self.hook_after_wait: Optional[Callable[[], Any]] = None
        self._drop_on_exit = False

    # -- waiting ---------------------------------------------------------------------------------
    def current_stream_wait(self, release_handle: bool = False) -> None:
        """Order torch's current stream behind the event; then fire the callback, once."""
        if self.event is None:
            raise AssertionError("this EventOverlap holds no event")
        self.event.current_stream_wait()
        pending, self.hook_after_wait = self.hook_after_wait, None
        if callable(pending):
            pending()
        if release_handle:
            self.event = None

    def register_hook_after_wait(self, hook_after_wait: Callable[[], Any]) -> None:
        if self.hook_after_wait is not None:
            raise AssertionError("A hook is already registered on this `EventOverlap`")
        self.hook_after_wait = hook_after_wait

    # -- `with overlap:` / `with overlap(release_handle=True):` ----------------------------------
    def __call__(self, release_handle: bool = False) -> "EventOverlap":
        self._drop_on_exit = bool(release_handle)
        return self                      # no second wrapper: the event keeps a single owner

    def __enter__(self) -> "EventOverlap":
        return self

    def __exit__(self, *exc_info: Any) -> None:
        drop, self._drop_on_exit = self._drop_on_exit, False
        if self.event is not None:
            self.current_stream_wait(release_handle=drop)
