// Devices the mini-executor creates itself: the "host" device that input
// nodes are routed to, a CPU mock device for tests without a GPU, and a
// counting wrapper put around the device under test.
#pragma once

#include "coherent_allocator.hpp"
#include "record_layer.hpp"

#include "polar_harness.h"

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>

namespace polar_harness_detail {

// src/backend/generic/runtime/host/HostDevice.hpp:17-52: not a compute device,
// it only names the memory domain of input nodes.
class HostDevice final : public Device {
public:
  DeviceProvider getProvider() const override { return DeviceProvider::HOST; }
  DeviceKind getKind() const override { return DeviceKind::HOST; }
  std::string getDeviceName() const override { return "host"; }
  std::vector<std::shared_ptr<Device>> partition(PartitionDomain) override { return {}; }
  std::shared_ptr<AllocatorLayerBase> getAllocator() override { return nullptr; }
  bool operator==(const Device& o) const override { return o.getDeviceName() == "host"; }
  void copyToHost(MemoryRecord, void*) const override {}
  void copyToDevice(MemoryRecord, void*) const override {}
  Event* launch(BackendAllocator&, LaunchCommand&, Event*) override { return nullptr; }
  void consumeEvent(Event*) override {}
  void selectBinary(std::vector<std::shared_ptr<ProgramDesc>>&) override {}
};

// Event of the mock device: complete at once; wait() runs the callbacks.
class MockEvent final : public Event {
public:
  explicit MockEvent(Device* d) : mDevice(d) {}
  void wait() override {
    auto run = std::move(mCallbacks);
    mCallbacks.clear();
    for (auto& cb : run) cb();
  }
  void addCallback(std::function<void()> cb) override { mCallbacks.push_back(std::move(cb)); }
  auto getDevice() -> Device* override { return mDevice; }

private:
  Device* mDevice;
  std::vector<std::function<void()>> mCallbacks;
};

// Block source of the mock device's memory layer: the heap.
struct HeapBlocks {
  void* acquire(size_t bytes) {
    void* p = std::aligned_alloc(64, (bytes + 63) / 64 * 64 + 64);
    if (p == nullptr) fatalError(kFatalOther, "Failed to allocate RAM memory!");
    return p;
  }
  void give(void* block) { std::free(block); }
  bool attached() const { return mAttached; }
  void detach() { mAttached = false; }
  [[noreturn]] void fail(const char* fmt, ...) __attribute__((format(printf, 2, 3))) {
    char message[256];
    va_list ap;
    va_start(ap, fmt);
    std::vsnprintf(message, sizeof(message), fmt, ap);
    va_end(ap);
    fatalError(kFatalBadAccess, "%s", message);
  }

private:
  bool mAttached = true;
};

// A device with its own memory layer (heap blocks standing for device memory,
// in the same layer class the GPU plugin uses, so the byte limit and the
// eviction path work without a GPU) whose launch computes nothing: like the MockDevice of the
// framework's allocator unit tests (tests/unit/backend/generic/lib/allocators/
// LayerAllocator.cpp:23-50) it exists so that the coherence protocol and the
// call sequence can be tested on a machine without a GPU.
class MockDevice final : public Device {
public:
  MockDevice() : mLayer(std::make_shared<RecordLayer<HeapBlocks>>()) {}
  DeviceProvider getProvider() const override { return DeviceProvider::HOST; }
  DeviceKind getKind() const override { return DeviceKind::OTHER_ACCELERATOR; }
  std::string getDeviceName() const override { return "mock"; }
  bool hasAllocator() override { return true; }
  std::vector<std::shared_ptr<Device>> partition(PartitionDomain) override { return {}; }
  std::shared_ptr<AllocatorLayerBase> getAllocator() override { return mLayer; }
  bool operator==(const Device& o) const override { return o.getDeviceName() == "mock"; }
  void copyToHost(MemoryRecord r, void* dest) const override {
    std::memcpy(dest, mLayer->getPtr(r), r.allocationSize);
  }
  void copyToDevice(MemoryRecord r, void* src) const override {
    std::memcpy(mLayer->getPtr(r), src, r.allocationSize);
  }
  Event* launch(BackendAllocator&, LaunchCommand& cmd, Event*) override {
    launched.emplace_back(cmd.nativeKernelName);
    mEvents.push_back(std::make_unique<MockEvent>(this));
    return mEvents.back().get();
  }
  void consumeEvent(Event* e) override { e->wait(); }
  void selectBinary(std::vector<std::shared_ptr<ProgramDesc>>&) override {}

  void setByteLimit(uint64_t bytes) { mLayer->setByteLimit(bytes); }
  std::vector<std::string> launched;

private:
  std::shared_ptr<RecordLayer<HeapBlocks>> mLayer;
  std::vector<std::unique_ptr<MockEvent>> mEvents;
};

// Forwards every call to the device under test and counts what crosses the
// boundary.  It reports the inner device's name and allocator layer, so the
// coherence allocator treats the two as one device.
class CountingDevice final : public Device {
public:
  CountingDevice(std::shared_ptr<Device> inner, polar_harness_counters* c)
      : mInner(std::move(inner)), mCounters(c) {}
  DeviceProvider getProvider() const override { return mInner->getProvider(); }
  DeviceKind getKind() const override { return mInner->getKind(); }
  std::string getDeviceName() const override {
    mCounters->device_name_calls++;
    return mInner->getDeviceName();
  }
  bool isPartitionSupported(PartitionDomain d) override { return mInner->isPartitionSupported(d); }
  bool hasAllocator() override { return mInner->hasAllocator(); }
  std::vector<std::shared_ptr<Device>> partition(PartitionDomain d) override { return mInner->partition(d); }
  std::shared_ptr<AllocatorLayerBase> getAllocator() override { return mInner->getAllocator(); }
  bool operator==(const Device& o) const override { return *mInner == o; }
  void copyToHost(MemoryRecord r, void* dest) const override {
    mCounters->copies_to_host++;
    mCounters->bytes_to_host += r.allocationSize;
    mInner->copyToHost(r, dest);
  }
  void copyToDevice(MemoryRecord r, void* src) const override {
    mCounters->copies_to_device++;
    mCounters->bytes_to_device += r.allocationSize;
    mInner->copyToDevice(r, src);
  }
  Event* launch(BackendAllocator& a, LaunchCommand& cmd, Event* dep) override {
    mCounters->launches++;
    return mInner->launch(a, cmd, dep);
  }
  void consumeEvent(Event* e) override { mInner->consumeEvent(e); }
  void selectBinary(std::vector<std::shared_ptr<ProgramDesc>>& p) override { mInner->selectBinary(p); }
  Device& inner() { return *mInner; }

private:
  std::shared_ptr<Device> mInner;
  polar_harness_counters* mCounters;
};

} // namespace polar_harness_detail
