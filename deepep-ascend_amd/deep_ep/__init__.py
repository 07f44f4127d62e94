"""MI355X-native MoE token routing behind the DeepEP `ElasticBuffer` API (drop-in surface of the
reference's deep_ep/__init__.py:92-109).  The HIP kernel library is loaded at import; without it
the import fails (there is no fallback path)."""
from . import _abi  # noqa: F401  (loads libdeep_ep_hip.so or raises)
from ._binding import Config, EventHandle, topk_idx_t, tuning
from .buffers.elastic import ElasticBuffer, EPHandle, LogicalGroup
from .buffers.legacy import Buffer
from .utils.event import EventOverlap

__version__ = "2.0.0+hip"

__all__ = ["ElasticBuffer", "EPHandle", "EventOverlap", "EventHandle", "Buffer", "Config", "LogicalGroup", "topk_idx_t",
           "tuning", "__version__"]
