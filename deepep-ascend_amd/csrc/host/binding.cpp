// The `deep_ep._C` extension of the HIP backend: module identity, `EventHandle`, `ElasticBuffer` (V2), and `Config` /
// `Buffer` / `get_low_latency_rdma_size_hint` (V1).
// Built with the host compiler alone (no device code lives here) and linked against libdeep_ep_hip.so, whose C ABI
// (include/deep_ep_hip.h) does all GPU work.  Registration follows the reference's templates
// (csrc/elastic/binding.hpp:9-44: register_event / register_common_apis bind *a selected class*;
// csrc/legacy/buffer.hpp:1751-1787 for the V1 names) and module layout (csrc/python_api.cpp:37-54).  Every method takes
// the reference's arguments positionally, in the reference's order; what this backend adds comes after them as
// keyword arguments with defaults.
#include <pybind11/functional.h>
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>
#include <torch/python.h>

#include <c10/hip/HIPFunctions.h>

#include <string>

#include "platform.hpp"
#include "elastic_buffer.hpp"
#include "legacy_buffer.hpp"

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
        .def("dispatch", &ElasticBuffer::dispatch, py::arg("x"), py::arg("sf"), py::arg("topk_idx"), py::arg("topk_weights"),
             py::arg("cumulative_local_expert_recv_stats"), py::arg("cached_num_recv_tokens"), py::arg("cached_num_expanded_tokens"),
             py::arg("cached_num_recv_tokens_per_expert_list"), py::arg("cached_psum_num_recv_tokens_per_scaleup_rank"),
             py::arg("cached_psum_num_recv_tokens_per_expert"), py::arg("cached_num_unaligned_recv_tokens_per_expert"),
             py::arg("cached_dst_buffer_slot_idx"), py::arg("cached_token_metadata_at_forward"), py::arg("cached_recv_src_metadata"),
             py::arg("cached_channel_linked_list"), py::arg("num_max_tokens_per_rank"), py::arg("num_experts"),
             py::arg("expert_alignment"), py::arg("num_sms"), py::arg("num_qps"), py::arg("previous_event"),
             py::arg("previous_event_before_epilogue"), py::arg("async_with_compute_stream"), py::arg("allocate_on_comm_stream"),
             py::arg("do_handle_copy"), py::arg("do_cpu_sync"), py::arg("do_expand"), py::arg("do_zero_padding"),
             py::arg("use_tma_aligned_col_major_sf"), py::arg("cast_to_fp8") = false)
        .def("combine", &ElasticBuffer::combine, py::arg("x"), py::arg("topk_weights"), py::arg("bias_0"), py::arg("bias_1"),
             py::arg("src_metadata"), py::arg("combined_topk_idx"), py::arg("psum_num_recv_tokens_per_scaleup_rank"),
             py::arg("token_metadata_at_forward"), py::arg("channel_linked_list"), py::arg("num_experts"),
             py::arg("num_max_tokens_per_rank"), py::arg("num_sms"), py::arg("num_qps"), py::arg("previous_event"),
             py::arg("previous_event_before_epilogue"), py::arg("async_with_compute_stream"), py::arg("allocate_on_comm_stream"),
             py::arg("use_expanded_layout"), py::arg("dst_buffer_slot_idx") = py::none());
    m.def("calculate_elastic_buffer_size", &ElasticBuffer::calculate_buffer_size);
    return cls;
}

// Status reads and other calls both host classes inherit.
template <typename Runtime>
void register_runtime_extras(py::class_<Runtime>& cls) {
    cls.def("is_destroyed", &Runtime::is_destroyed)
        .def("check_device_status", &Runtime::check_device_status, py::arg("what") = "routing")
        .def("queue_status_read", &Runtime::queue_status_read, py::arg("out"), py::arg("clear") = true)
        .def("poll_device_status", &Runtime::poll_device_status, py::arg("what") = "routing")
        .def("device_status", &Runtime::device_status)
        .def("workspace_control_words", &Runtime::workspace_control_words);
}

// V1: the names of csrc/legacy/buffer.hpp:1751-1787 that exist on one GPU.
void register_legacy_apis(py::module_& m) {
    using deep_ep::hip::Buffer;
    using deep_ep::hip::Config;
    py::class_<Config>(m, "Config")
        .def(py::init<int, int, int, int, int>(), py::arg("num_sms") = 20, py::arg("num_max_nvl_chunked_send_tokens") = 6,
             py::arg("num_max_nvl_chunked_recv_tokens") = 256, py::arg("num_max_rdma_chunked_send_tokens") = 6,
             py::arg("num_max_rdma_chunked_recv_tokens") = 256)
        .def_readonly("num_sms", &Config::num_sms)
        .def("get_nvl_buffer_size_hint", &Config::get_nvl_buffer_size_hint)
        .def("get_rdma_buffer_size_hint", &Config::get_rdma_buffer_size_hint);
    m.def("get_low_latency_rdma_size_hint", &deep_ep::hip::get_low_latency_rdma_size_hint);

    py::class_<Buffer> cls(m, "Buffer");
    cls.def(py::init<int, int, int64_t, int64_t, bool, bool, bool, bool>())
        .def("is_available", &Buffer::is_available)
        .def("get_num_rdma_ranks", &Buffer::get_num_rdma_ranks)
        .def("get_rdma_rank", &Buffer::get_rdma_rank)
        .def("get_root_rdma_rank", &Buffer::get_root_rdma_rank)
        .def("get_local_device_id", &Buffer::get_local_device_id)
        .def("get_comm_stream", &Buffer::get_comm_stream)
        .def("destroy", &Buffer::destroy)
        .def("get_dispatch_layout", &Buffer::get_dispatch_layout)
        .def("intranode_dispatch", &Buffer::intranode_dispatch, py::arg("x"), py::arg("x_scales"), py::arg("topk_idx"),
             py::arg("topk_weights"), py::arg("num_tokens_per_rank"), py::arg("is_token_in_rank"), py::arg("num_tokens_per_expert"),
             py::arg("cached_num_recv_tokens"), py::arg("cached_rank_prefix_matrix"), py::arg("cached_channel_prefix_matrix"),
             py::arg("expert_alignment"), py::arg("num_worst_tokens"), py::arg("config"), py::arg("previous_event"), py::arg("async"),
             py::arg("allocate_on_comm_stream"), py::arg("cached_send_head") = py::none())
        .def("intranode_combine", &Buffer::intranode_combine)
        .def("internode_dispatch", [](const Buffer& b, py::args, py::kwargs) { b.internode_unsupported(); })
        .def("internode_combine", [](const Buffer& b, py::args, py::kwargs) { b.internode_unsupported(); })
        .def("clean_low_latency_buffer", &Buffer::clean_low_latency_buffer)
        .def("low_latency_dispatch", &Buffer::low_latency_dispatch)
        .def("low_latency_combine", &Buffer::low_latency_combine, py::arg("x"), py::arg("topk_idx"), py::arg("topk_weights"),
             py::arg("src_info"), py::arg("layout_range"), py::arg("combine_wait_recv_cost_stats"),
             py::arg("num_max_dispatch_tokens_per_rank"), py::arg("num_experts"), py::arg("use_logfmt"), py::arg("zero_copy"),
             py::arg("async"), py::arg("return_recv_hook"), py::arg("out") = py::none())
        .def("get_next_low_latency_combine_buffer", &Buffer::get_next_low_latency_combine_buffer);
    register_runtime_extras(cls);
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
    cls.def("get_dispatch_layout", &deep_ep::hip::ElasticBuffer::get_dispatch_layout);
    deep_ep::hip::binding::register_runtime_extras(cls);
    deep_ep::hip::binding::register_legacy_apis(m);
    m.def("get_elastic_buffer_alignment", []() { return deep_ep::hip::kBufferAlignmentBytes; });
    m.def("set_tuning", [](const std::string& name, int value) { *deep_ep::hip::tuning_field(name) = value; });
    m.def("get_tuning", [](const std::string& name) { return *deep_ep::hip::tuning_field(name); });
    m.def("abi_version", []() { return deep_ep_hip_abi_version(); });
}
