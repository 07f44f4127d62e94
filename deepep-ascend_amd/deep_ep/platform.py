"""Which backend this build of the package drives (the role of the reference's
deep_ep/platform.py:9-80, which only knows "cuda" and "ascend")."""
import torch

from . import _binding


def get_platform() -> str:
    return _binding.get_platform()


def is_hip() -> bool:
    return get_platform() == "hip"


def capture_event():
    return _binding.EventHandle()


def unwrap_event(event):
    """EventOverlap or EventHandle or None -> EventHandle or None."""
    is_handle = isinstance(event, _binding.EventHandle)
    return getattr(event, "event", event) if event is not None and not is_handle else event


def synchronize() -> None:
    torch.cuda.synchronize()
