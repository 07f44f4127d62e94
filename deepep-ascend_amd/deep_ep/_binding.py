"""Which host runtime the V2 `ElasticBuffer` drives: the compiled `deep_ep._C` extension (csrc/host/, the counterpart of
the reference's pybind module) or the Python runtime over ctypes (`deep_ep._runtime`).  Both sit on the same C ABI and
expose the same names.  DEEP_EP_HIP_BINDING=pybind | ctypes forces one; by default the compiled extension is used when it
has been built."""
import importlib
import os

from . import _abi, _runtime

_choice = os.environ.get("DEEP_EP_HIP_BINDING", "").lower()
if _choice not in ("", "pybind", "ctypes"):
    raise ImportError(f"deep_ep: DEEP_EP_HIP_BINDING must be 'pybind' or 'ctypes', not {_choice!r}")

compiled = None
if _choice != "ctypes":
    try:
        compiled = importlib.import_module("deep_ep._C")
    except ImportError as exc:
        if _choice == "pybind":
            raise ImportError("deep_ep: DEEP_EP_HIP_BINDING=pybind, but the compiled extension deep_ep._C cannot be "
                              "imported; build it with `python deepep-ascend_amd/build.py`") from exc
    if compiled is not None and compiled.abi_version() != _abi.ABI_VERSION:
        raise ImportError(f"deep_ep: deep_ep._C was built against ABI version {compiled.abi_version()}, "
                          f"libdeep_ep_hip.so has {_abi.ABI_VERSION}")

name = "pybind" if compiled is not None else "ctypes"
_impl = compiled if compiled is not None else _runtime

ElasticBuffer = _impl.ElasticBuffer
EventHandle = _impl.EventHandle
calculate_elastic_buffer_size = _impl.calculate_elastic_buffer_size
get_elastic_buffer_alignment = _impl.get_elastic_buffer_alignment
get_platform = _impl.get_platform
topk_idx_t = _impl.topk_idx_t


class _Tuning:
    """Process-wide launch-shape knobs (the `tuning` member of the C argument blocks): attribute writes reach both
    runtimes.  Field names are those of `deep_ep_hip_tuning`; 0 = the library's own choice."""

    def __getattr__(self, field):
        return getattr(_abi.tuning, field)

    def __setattr__(self, field, value):
        if field not in dict(_abi.Tuning._fields_) or field == "reserved":
            raise AttributeError(f"deep_ep.tuning has no field {field!r}")
        setattr(_abi.tuning, field, int(value))
        if compiled is not None:
            compiled.set_tuning(field, int(value))


tuning = _Tuning()
