"""MI355X-native MoE token routing behind the DeepEP `ElasticBuffer` API (drop-in surface of the
reference's deep_ep/__init__.py:92-109).  The HIP kernel library is loaded at import; without it
the import fails (there is no fallback path)."""
from . import _abi  # noqa: F401  (loads libdeep_ep_hip.so or raises)
from ._binding import Config, EventHandle, topk_idx_t, tuning
from .buffers.elastic import ElasticBuffer, EPHandle, LogicalGroup
from .buffers.legacy import Buffer
from .utils.event import EventOverlap


def get_physical_domain_size(group):
    """(RDMA ranks, scale-up ranks) of a group, deep_ep/utils/envs.py:277-295: every logical rank shares this GPU."""
    return 1, group.size()


def get_logical_domain_size(group, allow_hybrid_mode: bool = True):
    """(scale-out ranks, scale-up ranks), deep_ep/utils/envs.py:298-320: one scale-out domain, whether or not the hybrid
    mode is allowed, as for a single node in the reference."""
    return 1, group.size()


__version__ = "2.0.0+hip"

__all__ = ["ElasticBuffer", "EPHandle", "EventOverlap", "EventHandle", "Buffer", "Config", "LogicalGroup", "topk_idx_t",
           "tuning", "get_physical_domain_size", "get_logical_domain_size", "__version__"]
