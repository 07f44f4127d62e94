"""`EventOverlap`: the stream-event wrapper dispatch / combine hand back
(surface of the reference's deep_ep/utils/event.py:8-96)."""
from typing import Any, Callable, Optional, Tuple

import torch

from .._C import EventHandle


class EventOverlap:
    """Holds the event recorded after the routing kernels, plus an optional hook that must run on
    the waiting stream right after the wait (used by the deterministic epilogue).

    Attributes:
        event: the captured `EventHandle` (None when the call was synchronous with the compute stream).
        extra_tensors: tensors kept alive until the event is released.
    """

    def __init__(self, event: Optional[EventHandle] = None,
                 extra_tensors: Optional[Tuple[torch.Tensor, ...]] = None) -> None:
        self.event = event
        self.extra_tensors = extra_tensors
        self._release_handle_by_call = False
        self.hook_after_wait: Optional[Callable] = None

    def current_stream_wait(self, release_handle: bool = False) -> None:
        """Make `torch.cuda.current_stream()` wait for the event, then run the registered hook once."""
        assert self.event is not None
        self.event.current_stream_wait()
        hook, self.hook_after_wait = self.hook_after_wait, None
        if hook is not None:
            hook()
        if release_handle:
            self.event = None

    def register_hook_after_wait(self, hook_after_wait: Callable) -> None:
        assert self.hook_after_wait is None, "A hook is already registered on this `EventOverlap`"
        self.hook_after_wait = hook_after_wait

    def __call__(self, release_handle: bool = False) -> "EventOverlap":
        """`with event_overlap(release_handle=True): ...` drops the event after the wait."""
        self._release_handle_by_call = release_handle
        return self

    def __enter__(self) -> Any:
        return self

    def __exit__(self, exc_type: Any, exc_val: Any, exc_tb: Any) -> None:
        if self.event is not None:
            self.current_stream_wait(release_handle=self._release_handle_by_call)
        self._release_handle_by_call = False
