#include "hip_plugin.hpp"

namespace polarai::backend::generic::mi355x {

void HipEvent::rearm(uint64_t launchOrdinal) {
  std::lock_guard<std::mutex> g(mMutex);
  mOrdinal = launchOrdinal;
  mCallbacks.clear();
}

// Blocks until the device has passed this point, then runs the callbacks here,
// on the waiting thread: they re-enter the framework's allocator (deferred
// releases), which must never happen on a driver thread or under a lock of
// this library.  Later waits only flush callbacks added since.
void HipEvent::wait() {
  uint64_t ordinal;
  {
    std::lock_guard<std::mutex> g(mMutex);
    ordinal = mOrdinal;
  }
  mDevice->waitForLaunch(ordinal);
  std::vector<std::function<void()>> run;
  {
    std::lock_guard<std::mutex> g(mMutex);
    run.swap(mCallbacks);
  }
  for (auto& cb : run) cb();
}

void HipEvent::addCallback(std::function<void()> cb) {
  std::lock_guard<std::mutex> g(mMutex);
  mCallbacks.push_back(std::move(cb));
}

auto HipEvent::getDevice() -> Device* { return mDevice; }

} // namespace polarai::backend::generic::mi355x
