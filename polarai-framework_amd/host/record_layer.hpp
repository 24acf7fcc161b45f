// An allocator layer (AllocatorLayerBase) over any source of memory blocks:
// the bookkeeping the framework's layers keep per tensor record -- block,
// tag, locked/released state (src/backend/generic/runtime/cuda/
// CudaAllocator.hpp:26-91, sycl/USMAllocator.h:30-107) -- plus what they leave
// out: when the source runs dry, released records are handed to the
// registered offload callback and evicted until the allocation fits.
//
// `Blocks` supplies the memory:
//   void* acquire(size_t bytes)   a block, or nullptr when the source is
//                                 exhausted (any other failure is fatal there)
//   void  give(void* block)       take a block back
//   bool  attached() const        false once the source is gone for good
//   void  fail(const char* fmt, ...)  [[noreturn]] report and terminate
// The plugin's GPU layer uses the device library's pool; the mini-executor's
// CPU mock device uses the heap, so the eviction logic below is the same code
// with and without a GPU.
#pragma once

#include "polar_rt_abi.hpp"

#include <mutex>
#include <utility>

namespace polarai::backend::generic {

template <typename Blocks> class RecordLayer final : public AllocatorLayerBase {
public:
  template <typename... A> explicit RecordLayer(A&&... a) : mBlocks(std::forward<A>(a)...) {}
  ~RecordLayer() override { detach(); }

  void registerMemoryOffloadCallback(MemoryOffloadCallbackT cb) override {
    std::lock_guard<std::mutex> g(mMutex);
    mOffload = std::move(cb);
  }

  void allocate(MemoryRecord record) override {
    std::unique_lock<std::mutex> g(mMutex);
    if (!mBlocks.attached()) mBlocks.fail("allocate on a device that has been closed");
    for (;;) {
      // looked up on every turn: the offload callback runs without the mutex
      if (mEntries.count(record.virtualAddress)) return; // double allocation is a no-op
      const bool overLimit = mByteLimit != 0 && mBytesHeld + record.allocationSize > mByteLimit;
      void* p = overLimit ? nullptr : mBlocks.acquire(record.allocationSize);
      if (p != nullptr) {
        Entry e;
        e.ptr = p;
        e.bytes = record.allocationSize;
        e.tag = 1;
        mEntries.emplace(record.virtualAddress, e);
        mBytesHeld += record.allocationSize;
        return;
      }
      if (!evictOne(g))
        mBlocks.fail("out of device memory allocating %zu bytes for tensor %zu and nothing left "
                     "to evict",
                     record.allocationSize, record.virtualAddress);
    }
  }

  void deallocate(MemoryRecord record) override {
    std::lock_guard<std::mutex> g(mMutex);
    auto it = mEntries.find(record.virtualAddress);
    if (it == mEntries.end()) return;
    if (it->second.locked)
      mBlocks.fail("deallocate of tensor %zu while it is locked", record.virtualAddress);
    drop(it);
  }

  void lock(MemoryRecord record) override {
    std::lock_guard<std::mutex> g(mMutex);
    auto it = mEntries.find(record.virtualAddress);
    if (it == mEntries.end())
      mBlocks.fail("lock of tensor %zu that has no device allocation", record.virtualAddress);
    it->second.locked = true;
    it->second.released = false;
  }

  void release(MemoryRecord record) override {
    std::lock_guard<std::mutex> g(mMutex);
    auto it = mEntries.find(record.virtualAddress);
    if (it == mEntries.end()) return;
    it->second.locked = false;
    it->second.released = true;
  }

  void* getPtr(MemoryRecord record) override {
    std::lock_guard<std::mutex> g(mMutex);
    auto it = mEntries.find(record.virtualAddress);
    return it == mEntries.end() ? nullptr : it->second.ptr;
  }

  bool isAllocated(const MemoryRecord& record) const override {
    std::lock_guard<std::mutex> g(mMutex);
    return mEntries.count(record.virtualAddress) != 0;
  }

  size_t getTag(MemoryRecord record) override {
    std::lock_guard<std::mutex> g(mMutex);
    auto it = mEntries.find(record.virtualAddress);
    return it == mEntries.end() ? 0 : it->second.tag;
  }

  void setTag(MemoryRecord record, size_t tag) override {
    std::lock_guard<std::mutex> g(mMutex);
    auto it = mEntries.find(record.virtualAddress);
    if (it != mEntries.end()) it->second.tag = tag;
  }

  // ---- not part of the interface --------------------------------------------
  // capacity limit for tests of the eviction path (0 = limited by the source)
  void setByteLimit(uint64_t bytes) {
    std::lock_guard<std::mutex> g(mMutex);
    mByteLimit = bytes;
  }
  uint64_t bytesHeld() const {
    std::lock_guard<std::mutex> g(mMutex);
    return mBytesHeld;
  }
  // called by the owning device just before it closes: gives every block back
  // and leaves an empty shell for owners that outlive the device
  void detach() {
    std::lock_guard<std::mutex> g(mMutex);
    if (!mBlocks.attached()) return;
    for (auto& kv : mEntries)
      if (kv.second.ptr) mBlocks.give(kv.second.ptr);
    mEntries.clear();
    mBytesHeld = 0;
    mBlocks.detach();
  }
  Blocks& blocks() { return mBlocks; }

private:
  struct Entry {
    void* ptr = nullptr;
    size_t bytes = 0;
    size_t tag = 0;
    bool locked = false;
    bool released = false;
    uint64_t passedOver = 0; // eviction scan that found it taken again
  };
  using Map = std::unordered_map<size_t, Entry>; // by virtual address

  void drop(typename Map::iterator it) {
    mBlocks.give(it->second.ptr);
    mBytesHeld -= it->second.bytes;
    mEntries.erase(it);
  }

  // Evicts one released, unlocked record: its owner saves it through the
  // offload callback, then the block goes back to the source.  The callback
  // re-enters this layer (getTag; the device's copyToHost calls getPtr) and may
  // allocate, free or lock records, so the mutex is dropped around it and no
  // iterator is kept across it: every turn scans the table afresh, and a record
  // that was locked again meanwhile is not offered a second time in this scan.
  bool evictOne(std::unique_lock<std::mutex>& guard) {
    const uint64_t scan = ++mScans;
    for (;;) {
      auto it = mEntries.begin();
      for (; it != mEntries.end(); ++it)
        if (it->second.released && !it->second.locked && it->second.passedOver != scan) break;
      if (it == mEntries.end()) return false;
      const MemoryRecord victim{it->first, it->second.bytes};
      if (mOffload) {
        auto cb = mOffload;
        guard.unlock();
        cb(victim, *this);
        guard.lock();
      }
      auto again = mEntries.find(victim.virtualAddress);
      if (again == mEntries.end()) return true; // freed by the callback: room was made
      if (again->second.locked || !again->second.released) {
        again->second.passedOver = scan;
        continue;
      }
      drop(again);
      return true;
    }
  }

  Blocks mBlocks;
  mutable std::mutex mMutex;
  Map mEntries;
  MemoryOffloadCallbackT mOffload;
  uint64_t mByteLimit = 0;
  uint64_t mBytesHeld = 0;
  uint64_t mScans = 0;
};

} // namespace polarai::backend::generic
