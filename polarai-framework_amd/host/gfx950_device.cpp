#include "hip_plugin.hpp"

#include <cstdio>

namespace polarai::backend::generic::mi355x {

HipDevice::HipDevice(int ordinal) {
  checkStatus(polar_hip_device_open(ordinal, &mDev), "polar_hip_device_open");
  polar_hip_device_info info;
  checkStatus(polar_hip_device_get_info(mDev, &info), "polar_hip_device_get_info");
  // The framework keys its per-device tables by this string and compares it
  // with "host" on every call (src/backend/generic/lib/allocators/
  // LayerAllocator.cpp:30,60; src/backend/generic/runtime/support/
  // routines.cpp:29,40,55): it must be unique per GPU and never "host".
  char buf[384];
  std::snprintf(buf, sizeof(buf), "%s (%s) hip:%d pci:%02x",
                info.name[0] ? info.name : "AMD Instinct GPU", info.arch,
                info.ordinal, info.pci_bus_id);
  mName = buf;
  mAllocator = std::make_shared<HipPoolAllocator>(mDev);
}

HipDevice::~HipDevice() {
  if (mDev) polar_hip_device_synchronize(mDev);
  mIdleEvents.clear();
  mEvents.clear();    // returns native events to the device's pool
  mAllocator->detach(); // other owners may keep the layer; its blocks die here
  if (mDev) polar_hip_device_close(mDev);
}

void HipDevice::copyToHost(MemoryRecord record, void* dest) const {
  void* src = mAllocator->getPtr(record);
  if (src == nullptr)
    fatal("copyToHost: tensor %zu has no allocation on %s", record.virtualAddress,
          mName.c_str());
  checkStatus(polar_hip_copy_to_host(mDev, dest, src, record.allocationSize),
              "polar_hip_copy_to_host");
}

void HipDevice::copyToDevice(MemoryRecord record, void* src) const {
  void* dst = mAllocator->getPtr(record);
  if (dst == nullptr)
    fatal("copyToDevice: tensor %zu has no allocation on %s",
          record.virtualAddress, mName.c_str());
  checkStatus(polar_hip_copy_to_device(mDev, dst, src, record.allocationSize),
              "polar_hip_copy_to_device");
}

float* HipDevice::resolve(BackendAllocator& allocator, const MemoryRecord& record) {
  float* p = allocator.get<float>(record, *this);
  if (p == nullptr)
    fatal("tensor %zu has no allocation on %s", record.virtualAddress, mName.c_str());
  return p;
}

HipEvent* HipDevice::newEvent() {
  polar_hip_event* native = nullptr;
  checkStatus(polar_hip_event_record(mDev, &native), "polar_hip_event_record");
  std::lock_guard<std::mutex> g(mEventMutex);
  if (!mIdleEvents.empty()) {
    HipEvent* e = mIdleEvents.back();
    mIdleEvents.pop_back();
    e->rearm(native);
    return e;
  }
  mEvents.push_back(std::make_unique<HipEvent>(this, native));
  return mEvents.back().get();
}

// Enqueues one builtin operation.  A dependency recorded on this device needs
// no wait: the device has one in-order stream, so the new kernel already runs
// after it.  A foreign event is waited for on the host, as the framework's
// SYCL runtime does for every dependency
// (src/backend/generic/runtime/sycl/SYCLDevice.cpp:37-42).
// The returned event is owned by the device; the pointer stays valid until
// consumeEvent() or the end of the context.
Event* HipDevice::launch(BackendAllocator& allocator, LaunchCommand& cmd,
                         Event* blockingEvent) {
  if (blockingEvent != nullptr && blockingEvent->getDevice() != this)
    blockingEvent->wait();
  if (cmd.nativeKernelName == nullptr)
    fatal("launch of '%s' without a native kernel name",
          cmd.kernelName ? cmd.kernelName : "?");
  if (!dispatchNativeKernel(*this, allocator, cmd))
    fatal("no native kernel '%s' (requested by '%s')", cmd.nativeKernelName,
          cmd.kernelName ? cmd.kernelName : "?");
  return newEvent();
}

void HipDevice::consumeEvent(Event* evt) {
  if (evt == nullptr) return;
  if (evt->getDevice() != this) fatal("consumeEvent: event of another device");
  evt->wait();
  auto* mine = static_cast<HipEvent*>(evt);
  std::lock_guard<std::mutex> g(mEventMutex);
  mIdleEvents.push_back(mine);
}

HipContext::HipContext() {
  int n = 0;
  checkStatus(polar_hip_device_count(&n), "polar_hip_device_count");
  for (int i = 0; i < n; ++i) {
    // Only gfx950 parts are usable: the device library holds no other code.
    polar_hip_device* probe = nullptr;
    int st = polar_hip_device_open(i, &probe);
    if (st == POLAR_HIP_ERR_NO_DEVICE) continue;
    checkStatus(st, "polar_hip_device_open");
    polar_hip_device_close(probe);
    mDevices.push_back(std::make_shared<HipDevice>(i));
  }
}

} // namespace polarai::backend::generic::mi355x

extern "C" {

polarai::backend::generic::Context* initContext() {
  return new polarai::backend::generic::mi355x::HipContext();
}

void closeContext(polarai::backend::generic::Context* ctx) { delete ctx; }

}

// Test hook, not part of the framework's interface: caps the capacity of a
// device's memory layer so that the eviction / offload path can be exercised
// without filling 288 GB.  `dev` must be a device returned by this plugin.
extern "C" int polar_rt_hip_set_device_byte_limit(polarai::backend::generic::Device* dev,
                                                  uint64_t bytes) {
  using namespace polarai::backend::generic;
  if (dev == nullptr || dev->getProvider() != DeviceProvider::HIP) return -1;
  auto* mine = static_cast<mi355x::HipDevice*>(dev);
  static_cast<mi355x::HipPoolAllocator*>(mine->getAllocator().get())->setByteLimit(bytes);
  return 0;
}
