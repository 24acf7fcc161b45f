#include "hip_plugin.hpp"

#include <cstdarg>
#include <cstdio>
#include <exception>

namespace polarai::backend::generic::mi355x {

void fatal(const char* fmt, ...) {
  std::fprintf(stderr, "polar_rt_hip: fatal: ");
  va_list ap;
  va_start(ap, fmt);
  std::vfprintf(stderr, fmt, ap);
  va_end(ap);
  std::fprintf(stderr, "\n");
  std::fflush(stderr);
  std::terminate();
}

void checkStatus(int status, const char* what) {
  if (status != POLAR_HIP_OK)
    fatal("%s: %s (status %d)", what, polar_hip_last_error(), status);
}

HipPoolAllocator::~HipPoolAllocator() { detach(); }

void HipPoolAllocator::detach() {
  std::lock_guard<std::mutex> g(mMutex);
  if (mDev == nullptr) return;
  for (auto& kv : mEntries)
    if (kv.second.ptr) polar_hip_free(mDev, kv.second.ptr);
  mEntries.clear();
  mBytesHeld = 0;
  mDev = nullptr;
}

void HipPoolAllocator::registerMemoryOffloadCallback(MemoryOffloadCallbackT cb) {
  std::lock_guard<std::mutex> g(mMutex);
  mOffload = std::move(cb);
}

// Evicts one released (unlocked) record: lets the owner of the layers save it
// through the offload callback, then returns its block to the pool.  The
// callback re-enters this layer (getTag, and the device's copyToHost calls
// getPtr), so the mutex is dropped around it.
bool HipPoolAllocator::evictOneLocked(std::unique_lock<std::mutex>& guard) {
  for (auto it = mEntries.begin(); it != mEntries.end(); ++it) {
    if (!it->second.released || it->second.locked) continue;
    const MemoryRecord victim{it->first, it->second.bytes};
    if (mOffload) {
      auto cb = mOffload;
      guard.unlock();
      cb(victim, *this);
      guard.lock();
    }
    auto again = mEntries.find(victim.virtualAddress);
    if (again == mEntries.end()) return true;
    if (again->second.locked) continue; // taken while the mutex was dropped
    checkStatus(polar_hip_free(mDev, again->second.ptr), "polar_hip_free");
    mBytesHeld -= again->second.bytes;
    mEntries.erase(again);
    return true;
  }
  return false;
}

void HipPoolAllocator::allocate(MemoryRecord record) {
  std::unique_lock<std::mutex> g(mMutex);
  if (mDev == nullptr) fatal("allocate on a device that has been closed");
  if (mEntries.count(record.virtualAddress)) return; // double allocation is a no-op
  for (;;) {
    const bool overLimit =
        mByteLimit != 0 && mBytesHeld + record.allocationSize > mByteLimit;
    void* p = nullptr;
    int st = overLimit ? POLAR_HIP_ERR_OOM
                       : polar_hip_alloc(mDev, record.allocationSize, &p);
    if (st == POLAR_HIP_OK) {
      Entry e;
      e.ptr = p;
      e.bytes = record.allocationSize;
      e.tag = 1;
      mEntries.emplace(record.virtualAddress, e);
      mBytesHeld += record.allocationSize;
      return;
    }
    if (st != POLAR_HIP_ERR_OOM) checkStatus(st, "polar_hip_alloc");
    if (!evictOneLocked(g))
      fatal("out of device memory allocating %zu bytes for tensor %zu and "
            "nothing left to evict",
            record.allocationSize, record.virtualAddress);
  }
}

void HipPoolAllocator::deallocate(MemoryRecord record) {
  std::lock_guard<std::mutex> g(mMutex);
  auto it = mEntries.find(record.virtualAddress);
  if (it == mEntries.end()) return;
  if (it->second.locked)
    fatal("deallocate of tensor %zu while it is locked", record.virtualAddress);
  checkStatus(polar_hip_free(mDev, it->second.ptr), "polar_hip_free");
  mBytesHeld -= it->second.bytes;
  mEntries.erase(it);
}

void HipPoolAllocator::lock(MemoryRecord record) {
  std::lock_guard<std::mutex> g(mMutex);
  auto it = mEntries.find(record.virtualAddress);
  if (it == mEntries.end())
    fatal("lock of tensor %zu that has no device allocation", record.virtualAddress);
  it->second.locked = true;
  it->second.released = false;
}

void HipPoolAllocator::release(MemoryRecord record) {
  std::lock_guard<std::mutex> g(mMutex);
  auto it = mEntries.find(record.virtualAddress);
  if (it == mEntries.end()) return;
  it->second.locked = false;
  it->second.released = true;
}

void* HipPoolAllocator::getPtr(MemoryRecord record) {
  std::lock_guard<std::mutex> g(mMutex);
  auto it = mEntries.find(record.virtualAddress);
  return it == mEntries.end() ? nullptr : it->second.ptr;
}

bool HipPoolAllocator::isAllocated(const MemoryRecord& record) const {
  std::lock_guard<std::mutex> g(mMutex);
  return mEntries.count(record.virtualAddress) != 0;
}

size_t HipPoolAllocator::getTag(MemoryRecord record) {
  std::lock_guard<std::mutex> g(mMutex);
  auto it = mEntries.find(record.virtualAddress);
  return it == mEntries.end() ? 0 : it->second.tag;
}

void HipPoolAllocator::setTag(MemoryRecord record, size_t tag) {
  std::lock_guard<std::mutex> g(mMutex);
  auto it = mEntries.find(record.virtualAddress);
  if (it != mEntries.end()) it->second.tag = tag;
}

} // namespace polarai::backend::generic::mi355x
