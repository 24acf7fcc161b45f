// polar_rt_support.hpp -- the support library that JIT-compiled graph code
// calls (libpolar_rt_support_static.a): the seven ath_* routines plus the
// host/device coherence allocator they drive.
//
// Replaces, for a framework build that links it, the object library
// `polar_rt_support` (src/backend/generic/runtime/support/CMakeLists.txt:1-11;
// routines in src/backend/generic/runtime/support/routines.cpp:24-102,
// prototypes in src/backend/generic/runtime/support/api.hpp:15-32) and the
// allocator it reaches through GraphHandle::allocator
// (src/backend/generic/lib/allocators/LayerAllocator.cpp).  Differences:
//   * devices are kept in an indexed table, not in maps keyed by the device
//     name string (LayerAllocator.cpp:30-33,60,226-237);
//   * the offload callback of a device layer really moves the evicted tensor
//     to RAM (upstream registers one that is never invoked by its layers);
//   * ath_load hands the loader a flat fp32 view instead of an Accessor
//     object (see AbstractLoaderInternal below).
#pragma once

#include "polar_rt_abi.hpp"

// Loader seen by ath_load.  The framework's loaders fill an Accessor<float>
// over the tensor (include/polarai/core/loader/internal/
// AbstractLoaderInternal.hpp:32-33); this library passes the flat fp32 view,
// which is all the framework's MemcpyLoader uses
// (src/loaders/internal/MemcpyLoaderInternal.cpp:24-27).
namespace polarai::core::internal {
class AbstractLoaderInternal {
public:
  virtual ~AbstractLoaderInternal() = default;
  virtual void load(float* dst, size_t count) = 0;
};
} // namespace polarai::core::internal

extern "C" {
// src/backend/generic/runtime/support/api.hpp:18-32
void ath_allocate(GraphHandle*, polarai::backend::generic::Device&, TensorInfo*);
void ath_release(GraphHandle*, polarai::backend::generic::Device&, TensorInfo*,
                 polarai::backend::generic::Event* blockingEvt);
void ath_lock(GraphHandle*, polarai::backend::generic::Device&, TensorInfo*,
              polarai::core::internal::LockType);
polarai::backend::generic::Device* ath_device_select(GraphHandle*, uint64_t nodeId);
void ath_barrier(uint32_t count, polarai::backend::generic::Event** events);
polarai::backend::generic::Event* ath_launch(GraphHandle*, polarai::backend::generic::Device*,
                                             polarai::backend::generic::Event*, LaunchCommand&);
void ath_load(GraphHandle*, uint64_t nodeId, TensorInfo*);

// Construction of what GraphHandle needs, for callers that cannot name the
// concrete classes (the executor does `std::make_shared<LayerAllocator>()` and
// `allocator->registerDevice(*device)` -- src/backend/generic/lib/
// ExecutorImpl.cpp:99-137).  Objects are owned by the caller and destroyed
// with the matching call.
polarai::backend::generic::BackendAllocator* polar_rt_support_allocator_create();
void polar_rt_support_allocator_destroy(polarai::backend::generic::BackendAllocator*);
void polar_rt_support_register_device(polarai::backend::generic::BackendAllocator*,
                                      polarai::backend::generic::Device*);
// The "host" device input nodes are routed to
// (src/backend/generic/runtime/host/HostDevice.hpp:17-52).
polarai::backend::generic::Device* polar_rt_support_host_device_create();
void polar_rt_support_host_device_destroy(polarai::backend::generic::Device*);
// sizeof(GraphHandle) and the offsets of allocator, devices, mLoaders,
// isHostNode as this library was compiled.
void polar_rt_support_graph_handle_layout(uint64_t out[5]);
}
