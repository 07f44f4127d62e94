"""Which backend this build of the package drives (the role of the reference's
deep_ep/platform.py:9-80, which only knows "cuda" and "ascend")."""
import torch

from . import _C


def get_platform() -> str:
    return _C.get_platform()


def is_hip() -> bool:
    return get_platform() == "hip"


def capture_event() -> "_C.EventHandle":
    return _C.EventHandle()


def unwrap_event(event):
    """EventOverlap or EventHandle or None -> EventHandle or None."""
    return getattr(event, "event", event) if event is not None and not isinstance(event, _C.EventHandle) else event


def synchronize() -> None:
    torch.cuda.synchronize()
