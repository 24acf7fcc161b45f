// Host/device coherence allocator of the mini-executor: the protocol of the
// framework's LayerAllocator (src/backend/generic/lib/allocators/
// LayerAllocator.cpp) restated on an indexed device table instead of maps
// keyed by device-name strings.
//
// Protocol (per tensor record, keyed by virtual address):
//   * a global version counter starts at 1 when the record is first allocated
//     anywhere; every READ_WRITE lock increments it;
//   * every layer (RAM, each device) carries the version of the copy it
//     holds; a lock on a layer whose copy is stale first refreshes RAM from
//     the layer that holds the newest copy (Device::copyToHost) and then, for
//     a device layer, uploads RAM (Device::copyToDevice);
//   * a READ_WRITE lock on a record that is locked anywhere is fatal;
//   * copies happen while the allocator's mutex is held, as upstream.
#pragma once

#include "polar_rt_support.hpp"

#include <list>
#include <mutex>

namespace polar_harness_detail {

using namespace polarai::backend::generic;
using polarai::core::internal::LockType;
using polarai::core::internal::TensorInternal;

[[noreturn]] void fatalError(int code, const char* fmt, ...)
    __attribute__((format(printf, 2, 3)));
constexpr int kFatalOther = 1;     // ATH_FATAL_OTHER (utils/error/FatalError.hpp:32)
constexpr int kFatalBadAccess = 4; // ATH_BAD_ACCESS  (utils/error/FatalError.hpp:35)

// include/polarai/core/tensor/DataType.hpp:22-36
size_t sizeOfDataType(polarai::core::DataType type);

// Is `device` the "host" pseudo-device that input nodes are routed to?  The
// framework asks the device for its name and compares strings on every
// support-routine call (routines.cpp:29,40,55).  Here the answer is kept per
// device object -- keyed by the object's address AND its vtable pointer, so an
// address reused by an object of another class is not mistaken for the old
// one -- and only a device seen for the first time is asked for its name.
bool isHostDevice(Device& device);
void rememberDevice(Device& device, bool isHost);
void forgetDevice(Device& device);

// RAM layer: one heap block per record
// (src/backend/generic/lib/allocators/TrivialAllocator.hpp:23-93).
class RamLayer final : public AllocatorLayerBase {
public:
  ~RamLayer() override;
  void registerMemoryOffloadCallback(MemoryOffloadCallbackT) override {}
  void allocate(MemoryRecord record) override;
  void deallocate(MemoryRecord record) override;
  void lock(MemoryRecord record) override;
  void release(MemoryRecord record) override;
  void* getPtr(MemoryRecord record) override;
  bool isAllocated(const MemoryRecord& record) const override;
  size_t getTag(MemoryRecord record) override;
  void setTag(MemoryRecord record, size_t tag) override;

  // blocks from a provider instead of the heap (see polar_rt_support_set_host_memory)
  void setProvider(void* (*allocate)(size_t), void (*release)(void*), void (*quiesce)(void*)) {
    mAllocate = allocate;
    mRelease = release;
    mQuiesce = quiesce;
  }

private:
  struct Block {
    void* mem = nullptr;
    size_t tag = 0;
    bool locked = false;
    bool provided = false; // from the provider; heap otherwise
  };
  void freeBlock(Block& b);
  std::unordered_map<size_t, Block> mBlocks;
  void* (*mAllocate)(size_t) = nullptr;
  void (*mRelease)(void*) = nullptr;
  void (*mQuiesce)(void*) = nullptr;
};

class CoherentAllocator final : public BackendAllocator {
public:
  CoherentAllocator();
  ~CoherentAllocator() override;

  // TensorAllocator part: tensors addressed by object; each overload derives
  // the record from the object (LayerAllocator.cpp:21-27) and forwards
  void allocate(const TensorInternal&) override;
  void deallocate(const TensorInternal&) override;
  void* get(const TensorInternal&) override;
  void lock(const TensorInternal&, LockType) override;
  void release(const TensorInternal&) override;

  void registerDevice(Device& device) override;
  // RAM-side blocks from a provider (polar_rt_support_set_host_memory)
  void setHostMemory(void* (*allocate)(size_t), void (*release)(void*), void (*quiesce)(void*)) {
    mRam->setProvider(allocate, release, quiesce);
  }
  void allocate(const TensorInternal&, Device&) override;
  void allocate(const MemoryRecord& record, Device& device) override;
  void allocate(const MemoryRecord& record) override;
  void lock(const TensorInternal&, Device&, LockType) override;
  void lock(const MemoryRecord& record, Device& device, LockType type) override;
  void lock(const MemoryRecord& record, LockType type) override;
  void release(const MemoryRecord& record, Device& device) override;
  void release(const MemoryRecord& record) override;
  void* get(const MemoryRecord& record) override;

  // extension (upstream can only deallocate through a tensor object)
  void deallocate(const MemoryRecord& record);
  size_t version(const MemoryRecord& record);
  size_t lockCount(const MemoryRecord& record);

protected:
  void* getImpl(const TensorInternal&, Device&) override;
  void* getImpl(const MemoryRecord& record, Device& device) override;

private:
  struct Slot {
    std::string name;
    Device* device;
    std::shared_ptr<AllocatorLayerBase> layer;
  };
  struct Lock {
    LockType type;
    int slot; // -1 = RAM
  };
  struct State {
    size_t version = 0;
    std::list<Lock> locks;
  };
  int slotOf(Device& device);
  Slot& need(Device& device);
  void refreshHost(const MemoryRecord& record);

  std::mutex mMutex;
  std::unique_ptr<RamLayer> mRam;
  std::vector<Slot> mSlots;
  std::unordered_map<size_t, State> mState; // by virtual address
};

} // namespace polar_harness_detail
