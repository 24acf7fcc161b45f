// Classes of the MI355X runtime plugin (libpolar_rt_hip.so): the Context,
// Device, Event and allocator layer the framework's runtime driver receives
// from initContext().  They sit on the C ABI of the device library
// (polar_hip.h); no HIP header is needed here.
//
// Built with -fno-rtti -fno-exceptions like the framework's core
// (CMakeModules/PolarTarget.cmake:8-13): nothing throws across the boundary and
// no dynamic_cast is applied to objects that come from the caller.  Failures
// follow the framework's convention for runtimes -- print and terminate
// (src/backend/generic/runtime/hip/HIPContext.cpp:23-33,
//  src/backend/generic/runtime/cuda/utils.hpp:20-28).
#pragma once

#include "polar_hip.h"
#include "polar_rt_abi.hpp"
#include "record_layer.hpp"

#include <atomic>
#include <deque>
#include <mutex>

namespace polarai::backend::generic::mi355x {

[[noreturn]] void fatal(const char* fmt, ...) __attribute__((format(printf, 1, 2)));
void checkStatus(int status, const char* what);

// Block source of the GPU's allocator layer: the device library's pool.
struct PoolBlocks {
  explicit PoolBlocks(polar_hip_device* dev) : mDev(dev) {}
  void* acquire(size_t bytes);
  void give(void* block);
  bool attached() const { return mDev != nullptr; }
  void detach() { mDev = nullptr; }
  [[noreturn]] void fail(const char* fmt, ...) __attribute__((format(printf, 2, 3)));

private:
  polar_hip_device* mDev;
};

// Device-memory layer of one GPU.  Takes the place of the per-tensor raw
// allocations of the framework's allocator layers
// (src/backend/generic/runtime/cuda/CudaAllocator.hpp:26-91,
//  src/backend/generic/runtime/sycl/USMAllocator.h:30-107): records are keyed
// by virtual address, memory comes from the device library's pool, and the
// out-of-memory hook is live -- released records are handed to the registered
// offload callback and then evicted.
using HipPoolAllocator = RecordLayer<PoolBlocks>;

class HipDevice;

// One point in the stream order of a device: the ordinal of a launch on the
// device's single in-order stream.  No native event is recorded per launch;
// the first wait() that finds its ordinal not yet known to be complete makes
// the device record one marker behind everything launched so far and wait for
// that (HipDevice::waitForLaunch), which completes this event and all earlier
// ones at once.  wait() then runs the callbacks on the calling thread, as the
// framework's events do (src/backend/generic/runtime/cuda/CudaEvent.cpp:21-29).
class HipEvent final : public Event {
public:
  HipEvent(HipDevice* device, uint64_t launchOrdinal)
      : mDevice(device), mOrdinal(launchOrdinal) {}
  ~HipEvent() override = default;
  void wait() override;
  void addCallback(std::function<void()> cb) override;
  auto getDevice() -> Device* override;

  void rearm(uint64_t launchOrdinal);

private:
  HipDevice* mDevice;
  uint64_t mOrdinal;
  std::mutex mMutex;
  std::vector<std::function<void()>> mCallbacks;
};

class HipDevice final : public Device {
public:
  HipDevice(int ordinal);
  ~HipDevice() override;

  DeviceProvider getProvider() const override { return DeviceProvider::HIP; }
  DeviceKind getKind() const override { return DeviceKind::GPU; }
  std::string getDeviceName() const override { return mName; }
  bool isPartitionSupported(PartitionDomain) override { return false; }
  bool hasAllocator() override { return true; }
  std::vector<std::shared_ptr<Device>> partition(PartitionDomain) override {
    return {};
  }
  std::shared_ptr<AllocatorLayerBase> getAllocator() override {
    return mAllocator;
  }
  bool operator==(const Device& other) const override {
    return other.getDeviceName() == mName;
  }
  void copyToHost(MemoryRecord record, void* dest) const override;
  void copyToDevice(MemoryRecord record, void* src) const override;
  Event* launch(BackendAllocator& allocator, LaunchCommand& cmd,
                Event* blockingEvent) override;
  void consumeEvent(Event* evt) override;
  void selectBinary(std::vector<std::shared_ptr<ProgramDesc>>& programs) override;

  polar_hip_device* native() const { return mDev; }
  // Returns once launch number `ordinal` (and with it every earlier one) has
  // completed on the device.
  void waitForLaunch(uint64_t ordinal);
  float* resolve(BackendAllocator& allocator, const MemoryRecord& record);

private:
  HipEvent* newEvent();
  bool launchFromProgram(BackendAllocator& allocator, LaunchCommand& cmd);

  polar_hip_device* mDev = nullptr;
  std::shared_ptr<ProgramDesc> mProgram; // selected code object (kernel geometry lives here)
  polar_hip_module* mModule = nullptr;
  std::string mName;
  std::shared_ptr<HipPoolAllocator> mAllocator;
  std::atomic<uint64_t> mLaunched{0};   // launches enqueued so far
  std::atomic<uint64_t> mCompleted{0};  // all launches up to this ordinal are known complete
  std::mutex mSyncMutex;                // one marker in flight at a time
  std::mutex mEventMutex;
  std::deque<std::unique_ptr<HipEvent>> mEvents; // every event ever returned
  std::vector<HipEvent*> mIdleEvents;            // handed back via consumeEvent
};

class HipContext final : public Context {
public:
  HipContext();
  ~HipContext() override;
  std::vector<std::shared_ptr<Device>>& getDevices() override {
    return mDevices;
  }

private:
  std::vector<std::shared_ptr<Device>> mDevices;
};

// nativeKernelName -> launcher.  Returns false for an unknown name.
bool dispatchNativeKernel(HipDevice& device, BackendAllocator& allocator,
                          LaunchCommand& cmd);

} // namespace polarai::backend::generic::mi355x
