// The `deep_ep._C` extension of the HIP backend: module identity, `EventHandle`, `ElasticBuffer`.
// Built with the host compiler alone (no device code lives here) and linked against libdeep_ep_hip.so, whose C ABI
// (include/deep_ep_hip.h) does all GPU work.  Registration follows the reference's templates
// (csrc/elastic/binding.hpp:9-44: register_event / register_common_apis bind *a selected class*) and module layout
// (csrc/python_api.cpp:37-54).
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>
#include <torch/python.h>

#include <c10/hip/HIPFunctions.h>

#include <string>

#include "platform.hpp"
#include "elastic_buffer.hpp"

#ifndef TORCH_EXTENSION_NAME
#define TORCH_EXTENSION_NAME _C
#endif

namespace py = pybind11;

namespace deep_ep::hip::binding {

template <typename EventHandle>
void register_event(py::module_& m) {
    py::class_<EventHandle>(m, "EventHandle")
        .def(py::init<>())
        .def("__copy__", [](const EventHandle& event) { return event; })
        .def("current_stream_wait", [](const EventHandle& event) { event.current_stream_wait(); });
}

template <typename ElasticBuffer>
py::class_<ElasticBuffer> register_common_apis(py::module_& m) {
    py::class_<ElasticBuffer> cls(m, "ElasticBuffer");
    cls.def(py::init<int, int, int64_t, typename ElasticBuffer::cpu_comm_t, int64_t, int64_t, bool, bool, bool, int, int, int,
                     int, bool>());
    cls.def("destroy", &ElasticBuffer::destroy)
        .def("get_comm_stream", &ElasticBuffer::get_comm_stream)
        .def("get_physical_domain_size", &ElasticBuffer::get_physical_domain_size)
        .def("get_logical_domain_size", &ElasticBuffer::get_logical_domain_size)
        .def("barrier", &ElasticBuffer::barrier, py::arg("use_comm_stream") = true, py::arg("with_cpu_sync") = false,
             py::arg("sequential") = true)
        .def("dispatch", &ElasticBuffer::dispatch)
        .def("combine", &ElasticBuffer::combine);
    m.def("calculate_elastic_buffer_size", &ElasticBuffer::calculate_buffer_size);
    return cls;
}

}  // namespace deep_ep::hip::binding

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.doc() = "DeepEP: expert-parallel token routing, HIP (MI355X) backend";
    py::register_exception<deep_ep::hip::EPException>(m, "EPException", PyExc_RuntimeError);

    m.def("get_platform", []() { return std::string(deep_ep::platform::kName); });
    m.attr("topk_idx_t") = py::cast(c10::CppTypeToScalarType<int64_t>::value);      // EP_NUM_TOPK_IDX_BITS default

    deep_ep::hip::binding::register_event<deep_ep::hip::EventHandle>(m);
    auto cls = deep_ep::hip::binding::register_common_apis<deep_ep::hip::ElasticBuffer>(m);

    // Beyond the common contract: what the Ascend build also has (is_destroyed), the V1 layout call kept on this
    // buffer, device-status checks, and the launch-shape knobs.
    cls.def("is_destroyed", &deep_ep::hip::ElasticBuffer::is_destroyed)
        .def("get_dispatch_layout", &deep_ep::hip::ElasticBuffer::get_dispatch_layout)
        .def("check_device_status", &deep_ep::hip::ElasticBuffer::check_device_status, py::arg("what") = "routing")
        .def("queue_status_read", &deep_ep::hip::ElasticBuffer::queue_status_read, py::arg("out"), py::arg("clear") = true)
        .def("poll_device_status", &deep_ep::hip::ElasticBuffer::poll_device_status, py::arg("what") = "routing")
        .def("device_status", &deep_ep::hip::ElasticBuffer::device_status)
        .def("workspace_control_words", &deep_ep::hip::ElasticBuffer::workspace_control_words);
    m.def("get_elastic_buffer_alignment", []() { return deep_ep::hip::kBufferAlignmentBytes; });
    m.def("set_tuning", [](const std::string& name, int value) { *deep_ep::hip::tuning_field(name) = value; });
    m.def("get_tuning", [](const std::string& name) { return *deep_ep::hip::tuning_field(name); });
    m.def("abi_version", []() { return deep_ep_hip_abi_version(); });
}
