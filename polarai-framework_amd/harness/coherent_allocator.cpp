#include "coherent_allocator.hpp"

#include <cstdarg>
#include <cstdio>
#include <cstdlib>

namespace polar_harness_detail {

// The framework's FatalError prints and exits with the error code in release
// builds (include/polarai/utils/error/FatalError.hpp:88-98).
void fatalError(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  std::vfprintf(stderr, fmt, ap);
  va_end(ap);
  std::fprintf(stderr, "\n");
  std::fflush(stderr);
  std::_Exit(code);
}

// ---- RAM layer ----------------------------------------------------------------

RamLayer::~RamLayer() {
  for (auto& kv : mBlocks) std::free(kv.second.mem);
}

void RamLayer::allocate(MemoryRecord record) {
  if (mBlocks.count(record.virtualAddress)) return;
  Block b;
  b.mem = std::aligned_alloc(64, (record.allocationSize + 63) / 64 * 64 + 64);
  if (b.mem == nullptr) fatalError(kFatalOther, "Failed to allocate RAM memory!");
  b.tag = 1;
  mBlocks.emplace(record.virtualAddress, b);
}

void RamLayer::deallocate(MemoryRecord record) {
  auto it = mBlocks.find(record.virtualAddress);
  if (it == mBlocks.end()) return;
  if (it->second.locked)
    fatalError(kFatalBadAccess, "Double free on vaddr %zu", record.virtualAddress);
  std::free(it->second.mem);
  mBlocks.erase(it);
}

void RamLayer::lock(MemoryRecord record) {
  auto it = mBlocks.find(record.virtualAddress);
  if (it != mBlocks.end()) it->second.locked = true;
}

void RamLayer::release(MemoryRecord record) {
  auto it = mBlocks.find(record.virtualAddress);
  if (it != mBlocks.end()) it->second.locked = false;
}

void* RamLayer::getPtr(MemoryRecord record) {
  auto it = mBlocks.find(record.virtualAddress);
  return it == mBlocks.end() ? nullptr : it->second.mem;
}

bool RamLayer::isAllocated(const MemoryRecord& record) const {
  return mBlocks.count(record.virtualAddress) != 0;
}

size_t RamLayer::getTag(MemoryRecord record) {
  auto it = mBlocks.find(record.virtualAddress);
  return it == mBlocks.end() ? 0 : it->second.tag;
}

void RamLayer::setTag(MemoryRecord record, size_t tag) {
  auto it = mBlocks.find(record.virtualAddress);
  if (it != mBlocks.end()) it->second.tag = tag;
}

// ---- coherence ------------------------------------------------------------------

CoherentAllocator::CoherentAllocator() : mRam(std::make_unique<RamLayer>()) {}

namespace {
[[noreturn]] void noTensorObjects() {
  fatalError(kFatalOther, "the mini-executor addresses tensors by record, not by object");
}
} // namespace

void CoherentAllocator::allocate(const TensorInternal&) { noTensorObjects(); }
void CoherentAllocator::deallocate(const TensorInternal&) { noTensorObjects(); }
void* CoherentAllocator::get(const TensorInternal&) { noTensorObjects(); }
void CoherentAllocator::lock(const TensorInternal&, LockType) { noTensorObjects(); }
void CoherentAllocator::release(const TensorInternal&) { noTensorObjects(); }
void CoherentAllocator::allocate(const TensorInternal&, Device&) { noTensorObjects(); }
void CoherentAllocator::lock(const TensorInternal&, Device&, LockType) { noTensorObjects(); }
void* CoherentAllocator::getImpl(const TensorInternal&, Device&) { noTensorObjects(); }

int CoherentAllocator::slotOf(Device& device) {
  for (size_t i = 0; i < mSlots.size(); ++i)
    if (mSlots[i].device == &device) return static_cast<int>(i);
  // upstream identifies devices by name (LayerAllocator.cpp:30,60,226)
  const std::string name = device.getDeviceName();
  for (size_t i = 0; i < mSlots.size(); ++i)
    if (mSlots[i].name == name) return static_cast<int>(i);
  return -1;
}

CoherentAllocator::Slot& CoherentAllocator::need(Device& device) {
  int s = slotOf(device);
  if (s < 0)
    fatalError(kFatalBadAccess, "Device %s is not registered", device.getDeviceName().c_str());
  return mSlots[s];
}

// LayerAllocator.cpp:224-249
void CoherentAllocator::registerDevice(Device& device) {
  std::scoped_lock g{mMutex};
  if (slotOf(device) >= 0) return;
  Slot s;
  s.name = device.getDeviceName();
  s.device = &device;
  if (device.hasAllocator()) {
    s.layer = device.getAllocator();
  } else { // devices without memory of their own alias RAM
    s.layer = std::shared_ptr<AllocatorLayerBase>(mRam.get(), [](AllocatorLayerBase*) {});
  }
  Device* dev = &device;
  s.layer->registerMemoryOffloadCallback(
      [this, dev](MemoryRecord record, AllocatorLayerBase& layer) {
        // called by a layer that evicts `record`: save it to RAM unless RAM
        // already holds the same version
        if (mRam->getTag(record) == layer.getTag(record)) return;
        if (!mRam->isAllocated(record)) mRam->allocate(record);
        dev->copyToHost(record, mRam->getPtr(record));
        mRam->setTag(record, layer.getTag(record));
      });
  mSlots.push_back(std::move(s));
}

// LayerAllocator.cpp:28-37.  Note that this resets the version to 1 even if
// RAM already holds a newer copy: a result tensor first touched on a device
// through an in-place node would skip its upload.  Kept as upstream.
void CoherentAllocator::allocate(const MemoryRecord& record, Device& device) {
  std::scoped_lock g{mMutex};
  Slot& s = need(device);
  if (s.layer->isAllocated(record)) return;
  s.layer->allocate(record);
  State& st = mState[record.virtualAddress];
  st.version = 1;
}

// LayerAllocator.cpp:95-108
void CoherentAllocator::allocate(const MemoryRecord& record) {
  std::scoped_lock g{mMutex};
  if (mRam->isAllocated(record)) return;
  for (auto& s : mSlots)
    if (s.layer->isAllocated(record)) return;
  mRam->allocate(record);
  mState[record.virtualAddress].version = 1;
}

void CoherentAllocator::deallocate(const MemoryRecord& record) {
  std::scoped_lock g{mMutex};
  auto it = mState.find(record.virtualAddress);
  if (it != mState.end() && !it->second.locks.empty())
    fatalError(kFatalBadAccess, "Attempt to deallocate memory in use: %zu", record.virtualAddress);
  for (auto& s : mSlots)
    if (s.layer.get() != mRam.get() && s.layer->isAllocated(record)) s.layer->deallocate(record);
  if (mRam->isAllocated(record)) mRam->deallocate(record);
  if (it != mState.end()) mState.erase(it);
}

// LayerAllocator.cpp:251-263
void CoherentAllocator::refreshHost(const MemoryRecord& record) {
  const size_t version = mState[record.virtualAddress].version;
  for (auto& s : mSlots) {
    const size_t tag = s.layer->getTag(record);
    if (tag == version && tag > 0) {
      if (!mRam->isAllocated(record)) mRam->allocate(record);
      s.device->copyToHost(record, mRam->getPtr(record));
      break;
    }
  }
}

// LayerAllocator.cpp:46-87
void CoherentAllocator::lock(const MemoryRecord& record, Device& device, LockType type) {
  std::scoped_lock g{mMutex};
  State& st = mState[record.virtualAddress];
  if (type == LockType::READ_WRITE && !st.locks.empty())
    fatalError(kFatalBadAccess,
               "Attempt get READ_WRITE lock for tensor that is already locked: %zu",
               record.virtualAddress);
  const int slot = slotOf(device);
  if (slot < 0)
    fatalError(kFatalBadAccess, "Device %s is not registered", device.getDeviceName().c_str());
  AllocatorLayerBase& layer = *mSlots[slot].layer;
  if (!layer.isAllocated(record)) layer.allocate(record);
  if (layer.getTag(record) != st.version) { // the device copy is stale
    if (st.version != mRam->getTag(record)) refreshHost(record);
    device.copyToDevice(record, mRam->getPtr(record));
  }
  if (type == LockType::READ_WRITE) st.version++;
  layer.setTag(record, st.version);
  st.locks.push_back(Lock{type, slot});
  layer.lock(record);
}

// LayerAllocator.cpp:162-186
void CoherentAllocator::lock(const MemoryRecord& record, LockType type) {
  std::scoped_lock g{mMutex};
  State& st = mState[record.virtualAddress];
  if (type == LockType::READ_WRITE && !st.locks.empty())
    fatalError(kFatalBadAccess,
               "Attempt get READ_WRITE lock for tensor with virtual address %zu that is already locked. ",
               record.virtualAddress);
  if (!mRam->isAllocated(record)) mRam->allocate(record);
  if (st.version != mRam->getTag(record)) refreshHost(record);
  if (type == LockType::READ_WRITE) st.version++;
  mRam->setTag(record, st.version);
  st.locks.push_back(Lock{type, -1});
  mRam->lock(record);
}

// LayerAllocator.cpp:193-204
void CoherentAllocator::release(const MemoryRecord& record) {
  std::scoped_lock g{mMutex};
  auto& locks = mState[record.virtualAddress].locks;
  for (auto it = locks.begin(); it != locks.end(); ++it) {
    if (it->slot == -1) {
      mRam->release(record);
      locks.erase(it);
      return;
    }
  }
}

// LayerAllocator.cpp:271-285
void CoherentAllocator::release(const MemoryRecord& record, Device& device) {
  std::scoped_lock g{mMutex};
  const int slot = slotOf(device);
  auto& locks = mState[record.virtualAddress].locks;
  for (auto it = locks.begin(); it != locks.end(); ++it) {
    if (it->slot >= 0 && it->slot == slot) {
      mSlots[slot].layer->release(record);
      locks.erase(it);
      return;
    }
  }
}

// LayerAllocator.cpp:152-160
void* CoherentAllocator::get(const MemoryRecord& record) {
  if (mRam->isAllocated(record)) return mRam->getPtr(record);
  fatalError(kFatalBadAccess, "No host pointer for vaddr %zu", record.virtualAddress);
}

// LayerAllocator.cpp:213-223
void* CoherentAllocator::getImpl(const MemoryRecord& record, Device& device) {
  std::scoped_lock g{mMutex};
  Slot& s = need(device);
  if (s.layer->isAllocated(record)) return s.layer->getPtr(record);
  fatalError(kFatalBadAccess, "Tensor %zu has no allocation on device %s",
             record.virtualAddress, s.name.c_str());
}

size_t CoherentAllocator::version(const MemoryRecord& record) {
  std::scoped_lock g{mMutex};
  auto it = mState.find(record.virtualAddress);
  return it == mState.end() ? 0 : it->second.version;
}

size_t CoherentAllocator::lockCount(const MemoryRecord& record) {
  std::scoped_lock g{mMutex};
  auto it = mState.find(record.virtualAddress);
  return it == mState.end() ? 0 : it->second.locks.size();
}

} // namespace polar_harness_detail
