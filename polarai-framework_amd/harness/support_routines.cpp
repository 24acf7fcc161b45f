// The seven C symbols that JIT-compiled graph code calls
// (src/backend/generic/runtime/support/api.hpp:15-32, bodies in
// src/backend/generic/runtime/support/routines.cpp:24-102; LLVM prototypes in
// utils/dialects/lib/Passes/DeployDefaultFunctions.cpp:38-108), restated for
// the mini-executor.  "host" nodes go to the RAM side of the allocator, every
// other device to its own layer.
#include "support_routines.hpp"

#include <cstring>

using namespace polar_harness_detail;

namespace {
// src/backend/generic/runtime/utils/utils.hpp:7-17
MemoryRecord toRecord(const TensorInfo* t) {
  size_t bytes = sizeOfDataType(static_cast<polarai::core::DataType>(t->dataType));
  for (uint64_t i = 0; i < t->dims; ++i) bytes *= t->shape[i];
  return MemoryRecord{static_cast<size_t>(t->virtAddr), bytes};
}
// routines.cpp:29,40,55 compare the device's name with "host" on every call;
// the answer is looked up per device object instead (no string is built)
bool isHost(Device& d) { return isHostDevice(d); }
} // namespace

namespace polar_harness_detail {
uint64_t g_deferredReleases = 0;
uint64_t g_eventsWaited = 0;
} // namespace polar_harness_detail

extern "C" {

void ath_allocate(GraphHandle* handle, Device& device, TensorInfo* tensor) {
  const MemoryRecord rec = toRecord(tensor);
  if (isHost(device))
    handle->allocator->allocate(rec);
  else
    handle->allocator->allocate(rec, device);
}

// With an event the release is deferred to the event's callbacks, which run
// when somebody waits on it (the barrier).
void ath_release(GraphHandle* handle, Device& device, TensorInfo* tensor, Event* blockingEvt) {
  const MemoryRecord rec = toRecord(tensor);
  if (isHost(device)) {
    handle->allocator->release(rec);
  } else if (blockingEvt != nullptr) {
    Device* dev = &device;
    blockingEvt->addCallback([handle, dev, rec]() {
      ++g_deferredReleases;
      handle->allocator->release(rec, *dev);
    });
  } else {
    handle->allocator->release(rec, device);
  }
}

void ath_lock(GraphHandle* handle, Device& device, TensorInfo* tensor, LockType type) {
  const MemoryRecord rec = toRecord(tensor);
  if (isHost(device))
    handle->allocator->lock(rec, type);
  else
    handle->allocator->lock(rec, device, type);
}

Device* ath_device_select(GraphHandle* handle, uint64_t nodeId) {
  if (handle->isHostNode.count(nodeId)) return handle->devices.back().get();
  return handle->devices.front().get();
}

void ath_barrier(uint32_t count, Event** events) {
  for (uint32_t i = 0; i < count; ++i) {
    if (events[i] != nullptr) {
      ++g_eventsWaited;
      events[i]->wait();
    }
  }
}

Event* ath_launch(GraphHandle* handle, Device* device, Event* event, LaunchCommand& command) {
  return device->launch(*handle->allocator, command, event);
}

void ath_load(GraphHandle* handle, uint64_t nodeId, TensorInfo* tensor) {
  auto it = handle->mLoaders.find(nodeId);
  if (it == handle->mLoaders.end() || it->second == nullptr)
    fatalError(kFatalOther, "No loader for node %llu", static_cast<unsigned long long>(nodeId));
  const MemoryRecord rec = toRecord(tensor);
  void* ptr = handle->allocator->get(rec);
  const auto type = static_cast<polarai::core::DataType>(tensor->dataType);
  if (type == polarai::core::DataType::FLOAT) {
    // routines.cpp:92-96
    BackendAccessor<float> acc(static_cast<float*>(ptr), tensor->dims, tensor->shape);
    it->second->load(acc);
  } else if (type == polarai::core::DataType::DOUBLE) {
    fatalError(kFatalOther, "Double is not supported.");
  }
}

} // extern "C"
