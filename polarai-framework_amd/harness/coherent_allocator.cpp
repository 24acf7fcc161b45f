#include "coherent_allocator.hpp"

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>

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

void RamLayer::freeBlock(Block& b) {
  if (b.provided) mRelease(b.mem);
  else std::free(b.mem);
  b.mem = nullptr;
}

RamLayer::~RamLayer() {
  for (auto& kv : mBlocks) freeBlock(kv.second);
}

void RamLayer::allocate(MemoryRecord record) {
  if (mBlocks.count(record.virtualAddress)) return;
  Block b;
  const size_t bytes = (record.allocationSize + 63) / 64 * 64 + 64;
  if (mAllocate != nullptr && mRelease != nullptr) {
    b.mem = mAllocate(bytes);
    b.provided = b.mem != nullptr;
  }
  if (b.mem == nullptr) b.mem = std::aligned_alloc(64, bytes);
  if (b.mem == nullptr) fatalError(kFatalOther, "Failed to allocate RAM memory!");
  b.tag = 1;
  mBlocks.emplace(record.virtualAddress, b);
}

void RamLayer::deallocate(MemoryRecord record) {
  auto it = mBlocks.find(record.virtualAddress);
  if (it == mBlocks.end()) return;
  if (it->second.locked)
    fatalError(kFatalBadAccess, "Double free on vaddr %zu", record.virtualAddress);
  freeBlock(it->second);
  mBlocks.erase(it);
}

void RamLayer::lock(MemoryRecord record) {
  auto it = mBlocks.find(record.virtualAddress);
  if (it == mBlocks.end()) return;
  it->second.locked = true;
  // host code is about to touch the block: nothing the device still has queued
  // out of it may be outstanding
  if (it->second.provided && mQuiesce != nullptr) mQuiesce(it->second.mem);
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

CoherentAllocator::~CoherentAllocator() {
  for (auto& s : mSlots) forgetDevice(*s.device);
}

size_t sizeOfDataType(polarai::core::DataType type) {
  switch (type) {
  case polarai::core::DataType::DOUBLE: return 8;
  case polarai::core::DataType::FLOAT: return 4;
  case polarai::core::DataType::HALF: return 2;
  default: fatalError(kFatalOther, "Size for dataType is not defined");
  }
}

// ---- which devices are "host" -------------------------------------------------

namespace {
struct KnownDevice {
  const Device* object;
  uintptr_t vtable;
  bool isHost;
};
std::mutex g_knownMutex;
std::vector<KnownDevice> g_known;
constexpr size_t kKnownDevicesMax = 64;

uintptr_t vtableOf(const Device& device) {
  uintptr_t v;
  std::memcpy(&v, static_cast<const void*>(&device), sizeof(v));
  return v;
}
} // namespace

void rememberDevice(Device& device, bool isHost) {
  const uintptr_t vt = vtableOf(device);
  std::scoped_lock g{g_knownMutex};
  for (auto& k : g_known)
    if (k.object == &device) {
      k.vtable = vt;
      k.isHost = isHost;
      return;
    }
  if (g_known.size() >= kKnownDevicesMax) g_known.erase(g_known.begin());
  g_known.push_back(KnownDevice{&device, vt, isHost});
}

void forgetDevice(Device& device) {
  std::scoped_lock g{g_knownMutex};
  for (auto it = g_known.begin(); it != g_known.end(); ++it)
    if (it->object == &device) {
      g_known.erase(it);
      return;
    }
}

bool isHostDevice(Device& device) {
  const uintptr_t vt = vtableOf(device);
  {
    std::scoped_lock g{g_knownMutex};
    for (const auto& k : g_known)
      if (k.object == &device && k.vtable == vt) return k.isHost;
  }
  const bool isHost = device.getDeviceName() == "host";
  rememberDevice(device, isHost);
  return isHost;
}

// ---- tensors addressed by object ------------------------------------------------

namespace {
// LayerAllocator.cpp:21-27 (and the same three lines in every other overload)
MemoryRecord recordOf(const TensorInternal& tensor) {
  return MemoryRecord{tensor.getVirtualAddress(),
                      tensor.getSize() * sizeOfDataType(tensor.getDataType())};
}
} // namespace

void CoherentAllocator::allocate(const TensorInternal& t) { allocate(recordOf(t)); }
void CoherentAllocator::deallocate(const TensorInternal& t) { deallocate(recordOf(t)); }
void* CoherentAllocator::get(const TensorInternal& t) { return get(recordOf(t)); }
void CoherentAllocator::lock(const TensorInternal& t, LockType type) { lock(recordOf(t), type); }
void CoherentAllocator::release(const TensorInternal& t) { release(recordOf(t)); }
void CoherentAllocator::allocate(const TensorInternal& t, Device& d) { allocate(recordOf(t), d); }
void CoherentAllocator::lock(const TensorInternal& t, Device& d, LockType type) {
  lock(recordOf(t), d, type);
}
void* CoherentAllocator::getImpl(const TensorInternal& t, Device& d) { return getImpl(recordOf(t), d); }

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
  // Called by a layer that is about to evict `record`, from inside its
  // allocate(), which this allocator only calls with mMutex held -- so mState
  // may be read here.  The device copy is saved only if it is the newest one
  // and RAM does not have it yet; a stale device copy is simply let go (saving
  // it would overwrite newer data in RAM and take RAM's tag back with it).
  s.layer->registerMemoryOffloadCallback(
      [this, dev](MemoryRecord record, AllocatorLayerBase& layer) {
        auto st = mState.find(record.virtualAddress);
        if (st == mState.end()) return;
        const size_t version = st->second.version;
        if (layer.getTag(record) != version || mRam->getTag(record) == version) return;
        if (!mRam->isAllocated(record)) mRam->allocate(record);
        dev->copyToHost(record, mRam->getPtr(record));
        mRam->setTag(record, version);
      });
  rememberDevice(device, s.name == "host");
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
