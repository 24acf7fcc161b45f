#pragma once

#include "coherent_allocator.hpp"

// Loader seen by ath_load.  The framework's loaders fill an Accessor<float>
// over the tensor (include/polarai/core/loader/internal/
// AbstractLoaderInternal.hpp:32-33); the mini-executor only needs the flat
// fp32 view, which is all the framework's MemcpyLoader uses
// (src/loaders/internal/MemcpyLoaderInternal.cpp:24-27).
namespace polarai::core::internal {
class AbstractLoaderInternal {
public:
  virtual ~AbstractLoaderInternal() = default;
  virtual void load(float* dst, size_t count) = 0;
};
} // namespace polarai::core::internal

namespace polar_harness_detail {
extern uint64_t g_deferredReleases;
extern uint64_t g_eventsWaited;
} // namespace polar_harness_detail

extern "C" {
void ath_allocate(GraphHandle*, polarai::backend::generic::Device&, TensorInfo*);
void ath_release(GraphHandle*, polarai::backend::generic::Device&, TensorInfo*,
                 polarai::backend::generic::Event*);
void ath_lock(GraphHandle*, polarai::backend::generic::Device&, TensorInfo*,
              polarai::core::internal::LockType);
polarai::backend::generic::Device* ath_device_select(GraphHandle*, uint64_t nodeId);
void ath_barrier(uint32_t count, polarai::backend::generic::Event** events);
polarai::backend::generic::Event* ath_launch(GraphHandle*, polarai::backend::generic::Device*,
                                             polarai::backend::generic::Event*, LaunchCommand&);
void ath_load(GraphHandle*, uint64_t nodeId, TensorInfo*);
}
