// An event recorded on a stream at construction, and the stream helpers built on it
// (the role of csrc/utils/event.hpp:10-42 in the reference).
#pragma once

#include <ATen/hip/HIPEvent.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/types.h>

#include <memory>
#include <optional>
#include <vector>

namespace deep_ep::hip {

using Stream = c10::hip::HIPStreamMasqueradingAsCUDA;

inline Stream current_stream() { return c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(); }

struct EventHandle {
    std::shared_ptr<at::cuda::CUDAEvent> event;
    std::vector<std::optional<torch::Tensor>> tensors_to_record;     // kept alive until the event is dropped

    EventHandle() : EventHandle(current_stream()) {}

    explicit EventHandle(const Stream& stream) : event(std::make_shared<at::cuda::CUDAEvent>()) { event->record(stream); }

    EventHandle(const EventHandle&) = default;

    void current_stream_wait() const { event->block(current_stream()); }
};

// `waiter` waits for everything queued on `other` so far.
inline void stream_wait(const Stream& waiter, const Stream& other) {
    at::cuda::CUDAEvent event;
    event.record(other);
    event.block(waiter);
}

inline void stream_wait(const Stream& waiter, const EventHandle& event) { event.event->block(waiter); }

}  // namespace deep_ep::hip
