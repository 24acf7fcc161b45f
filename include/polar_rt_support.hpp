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
//   * tensors addressed by object (the TensorInternal overloads, which the
//     framework's OutputNodeAccessor uses to read results --
//     include/polarai/core/node/OutputNodeAccessor.hpp:21-31) are turned into
//     records through three member functions of TensorInternal that this
//     library only declares: they resolve against the framework's polar_core
//     when the library is linked into it.
#pragma once

#include "polar_rt_abi.hpp"

#include <initializer_list>

namespace polarai::core {
// include/polarai/core/tensor/Accessor.hpp:20-44 -- what a loader is handed.
// Four virtual functions and no virtual destructor, in this order.
template <typename T> class Accessor {
public:
  virtual auto operator()(std::initializer_list<size_t> idx) -> T& = 0;
  virtual auto operator()(size_t idx) -> T& = 0;
  virtual auto getShape() -> const std::vector<size_t>& = 0;
  virtual auto getRawPtr() -> T* = 0;

protected:
  // first index runs fastest (Accessor.hpp:30-43)
  auto linearIndex(std::initializer_list<size_t> idx, const std::vector<size_t>& shape) -> size_t {
    size_t index = 0, stride = 1, d = 0;
    for (size_t i : idx) {
      if (d == shape.size()) break;
      index += i * stride;
      stride *= shape[d++];
    }
    return index;
  }
};

namespace internal {
// include/polarai/core/loader/internal/AbstractLoaderInternal.hpp:26-38.  The
// framework's class derives from Entity, whose only virtual function is its
// destructor (include/polarai/core/Entity.hpp:24-43), so a loader's vtable is
// {destructor, destructor, load}.  This library calls load through that slot
// and never constructs, destroys, copies or looks inside a loader, so Entity's
// data members are not restated.
class AbstractLoaderInternal {
public:
  virtual ~AbstractLoaderInternal() = default;
  virtual void load(Accessor<float>&) = 0;
};

// include/polarai/core/tensor/internal/TensorInternal.hpp:25-49.  Only these
// three members are used (as LayerAllocator.cpp:21-27 does); they are declared,
// not defined: the definitions are the framework's (src/core/tensor/internal/
// TensorInternal.cpp).  A tensor object is never created or copied here.
class TensorInternal {
public:
  TensorInternal() = delete;
  TensorInternal(const TensorInternal&) = delete;
  DataType getDataType() const;
  size_t getSize() const;            // number of elements
  size_t getVirtualAddress() const;  // utils::Index is size_t (utils/Index.hpp:18)
};
} // namespace internal
} // namespace polarai::core

namespace polarai::backend::generic {
// include/polarai/backend/generic/runtime/BackendAccessor.hpp:23-44 -- the
// accessor ath_load builds over the tensor's RAM copy (routines.cpp:92-96).
template <typename T> class BackendAccessor final : public core::Accessor<T> {
public:
  BackendAccessor(T* data, size_t dims, uint64_t* shape) : mData(data), mShape(shape, shape + dims) {}
  auto operator()(std::initializer_list<size_t> idx) -> T& override {
    return mData[this->linearIndex(idx, mShape)];
  }
  auto operator()(size_t idx) -> T& override { return mData[idx]; }
  auto getShape() -> const std::vector<size_t>& override { return mShape; }
  auto getRawPtr() -> T* override { return mData; }

private:
  T* mData;
  std::vector<size_t> mShape;
};
} // namespace polarai::backend::generic

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
// Optional: where the allocator's RAM-side blocks come from.  With blocks the
// device can address (a runtime plugin's pinned memory), Device::copyToDevice
// and copyToHost need no staging copy.  `quiesce` is called before host code is
// given access to a block (every lock of a record on the host device), so that
// an upload the device still has queued out of the block is complete before the
// host overwrites it; it may be null.  Set before the first tensor is allocated.
// Without this call the blocks come from the heap, as the framework's do.
struct polar_rt_host_memory {
  void* (*allocate)(size_t bytes); // may return null: the heap is used for that block
  void (*release)(void* block);
  void (*quiesce)(void* block);
};
void polar_rt_support_set_host_memory(polarai::backend::generic::BackendAllocator*,
                                      const polar_rt_host_memory* hooks);
// The "host" device input nodes are routed to
// (src/backend/generic/runtime/host/HostDevice.hpp:17-52).
polarai::backend::generic::Device* polar_rt_support_host_device_create();
void polar_rt_support_host_device_destroy(polarai::backend::generic::Device*);
// sizeof(GraphHandle) and the offsets of allocator, devices, mLoaders,
// isHostNode as this library was compiled.
void polar_rt_support_graph_handle_layout(uint64_t out[5]);
}
