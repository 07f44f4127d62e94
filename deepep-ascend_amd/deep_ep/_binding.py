"""The host runtime of the package: the compiled `deep_ep._C` extension (csrc/host/, the counterpart of the reference's
pybind module, csrc/python_api.cpp:37-54).  There is no second host path: if the extension cannot be imported the
package import fails and says how to build it."""
import importlib

import torch  # noqa: F401  (the extension's argument converters need torch's Python module loaded first)

from . import _abi

try:
    compiled = importlib.import_module("deep_ep._C")
except ImportError as exc:
    raise ImportError("deep_ep: the compiled host extension deep_ep._C cannot be imported (" + str(exc) + "). Build it with "
                      "`python deepep-ascend_amd/build.py`; there is no fallback path.") from exc
if compiled.abi_version() != _abi.ABI_VERSION:
    raise ImportError(f"deep_ep: deep_ep._C was built against ABI version {compiled.abi_version()}, "
                      f"libdeep_ep_hip.so has {_abi.ABI_VERSION}; rebuild with `python deepep-ascend_amd/build.py`")

name = "pybind"

ElasticBuffer = compiled.ElasticBuffer
Buffer = compiled.Buffer
Config = compiled.Config
EventHandle = compiled.EventHandle
calculate_elastic_buffer_size = compiled.calculate_elastic_buffer_size
get_elastic_buffer_alignment = compiled.get_elastic_buffer_alignment
get_low_latency_rdma_size_hint = compiled.get_low_latency_rdma_size_hint
get_platform = compiled.get_platform
topk_idx_t = compiled.topk_idx_t


class _Tuning:
    """Process-wide launch-shape knobs (the `tuning` member of the C argument blocks) as attributes.  Field names are
    those of `deep_ep_hip_tuning`; 0 = the library's own choice.  A write reaches the compiled runtime and the
    `_abi.tuning` block that callers of the raw C ABI copy into their argument blocks."""

    def __getattr__(self, field):
        return getattr(_abi.tuning, field)

    def __setattr__(self, field, value):
        if field not in dict(_abi.Tuning._fields_) or field == "reserved":
            raise AttributeError(f"deep_ep.tuning has no field {field!r}")
        setattr(_abi.tuning, field, int(value))
        compiled.set_tuning(field, int(value))


tuning = _Tuning()
