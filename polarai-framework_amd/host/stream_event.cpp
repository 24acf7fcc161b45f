#include "hip_plugin.hpp"

namespace polarai::backend::generic::mi355x {

HipEvent::~HipEvent() {
  if (mNative) polar_hip_event_release(mNative);
}

void HipEvent::rearm(polar_hip_event* native) {
  std::lock_guard<std::mutex> g(mMutex);
  mNative = native;
  mCallbacks.clear();
}

bool HipEvent::idle() {
  std::lock_guard<std::mutex> g(mMutex);
  return mNative == nullptr && mCallbacks.empty();
}

// Blocks until the device has passed this point, then runs the callbacks here,
// on the waiting thread: they re-enter the framework's allocator (deferred
// releases), which must never happen on a driver thread or under a lock of
// this library.  Once passed, the native event goes back to the pool and later
// waits only flush callbacks added since.
void HipEvent::wait() {
  polar_hip_event* native = nullptr;
  {
    std::lock_guard<std::mutex> g(mMutex);
    native = mNative;
  }
  if (native) {
    checkStatus(polar_hip_event_synchronize(native), "polar_hip_event_synchronize");
    std::lock_guard<std::mutex> g(mMutex);
    if (mNative == native) {
      polar_hip_event_release(native);
      mNative = nullptr;
    }
  }
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
