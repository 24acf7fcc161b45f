// Construction helpers of the support library for callers that cannot name
// its concrete classes.
#include "devices.hpp"
#include "support_routines.hpp"

#include <cstddef>

using namespace polar_harness_detail;

extern "C" {

BackendAllocator* polar_rt_support_allocator_create() { return new CoherentAllocator(); }

void polar_rt_support_allocator_destroy(BackendAllocator* allocator) { delete allocator; }

void polar_rt_support_register_device(BackendAllocator* allocator, Device* device) {
  if (allocator == nullptr || device == nullptr)
    fatalError(kFatalOther, "polar_rt_support_register_device: null argument");
  allocator->registerDevice(*device);
}

void polar_rt_support_set_host_memory(BackendAllocator* allocator, const polar_rt_host_memory* hooks) {
  if (allocator == nullptr) fatalError(kFatalOther, "polar_rt_support_set_host_memory: null allocator");
  auto* mine = static_cast<CoherentAllocator*>(allocator); // created by polar_rt_support_allocator_create
  if (hooks == nullptr) mine->setHostMemory(nullptr, nullptr, nullptr);
  else mine->setHostMemory(hooks->allocate, hooks->release, hooks->quiesce);
}

Device* polar_rt_support_host_device_create() {
  Device* host = new HostDevice();
  rememberDevice(*host, true);
  return host;
}

void polar_rt_support_host_device_destroy(Device* device) {
  if (device != nullptr) forgetDevice(*device);
  delete device;
}

void polar_rt_support_graph_handle_layout(uint64_t out[5]) {
  out[0] = sizeof(GraphHandle);
  out[1] = offsetof(GraphHandle, allocator);
  out[2] = offsetof(GraphHandle, devices);
  out[3] = offsetof(GraphHandle, mLoaders);
  out[4] = offsetof(GraphHandle, isHostNode);
}

} // extern "C"
