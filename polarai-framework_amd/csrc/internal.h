// Shared definitions of the device library: the device handle (stream, memory
// pool, event pool), error reporting and launch helpers.  Not installed; the
// public surface is include/polar_hip.h.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <cstdarg>
#include <condition_variable>
#include <cstdint>
#include <atomic>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <thread>
#include <unordered_map>
#include <vector>

#include "polar_hip.h"

struct polar_hip_event {
  polar_hip_device* dev;
  hipEvent_t ev;
  // number of the last direct host-block transfer queued on the stream before
  // this event was recorded (see polar_hip_device::directQueued); 0 for events
  // attached to a kernel
  uint64_t directStamp = 0;
};

// Second host thread of large device-to-host copies: the staging slots are
// drained into the caller's memory by two threads, because one thread's copy
// rate (about 22 GB/s) is below what the DMA engine delivers.  It takes one job
// at a time; started on the first copy that uses it, joined when the device is
// closed.
struct DrainThread {
  std::thread thread;
  std::mutex mu;
  std::condition_variable cv;
  char* dst = nullptr;
  const char* src = nullptr;
  size_t bytes = 0;
  bool pending = false; // a job is posted and not yet finished
  bool quit = false;
};

struct polar_hip_device {
  int ordinal = 0;
  hipStream_t stream = nullptr;
  polar_hip_device_info info{};

  std::mutex mu;
  // pool: rounded block size -> cached blocks; live block -> rounded size
  std::map<uint64_t, std::vector<void*>> cached;
  std::unordered_map<void*, uint64_t> live;
  polar_hip_pool_stats stats{};
  std::vector<polar_hip_event*> idleEvents;
  std::vector<polar_hip_event*> allEvents;

  // ring of pinned slots for small and medium host<->device copies; a slot
  // is busy until the event recorded behind its transfer has completed
  std::mutex stagingMu;
  void* staging = nullptr;
  hipEvent_t slotEvent[8] = {};
  bool slotBusy[8] = {};
  // a busy slot either has slotEvent recorded behind its transfer, or (small
  // uploads) only the transfer's number in the directQueued sequence
  bool slotEvented[8] = {};
  uint64_t slotNumber[8] = {};
  int nextSlot = 0;
  DrainThread drain; // used under stagingMu

  // armed by polar_hip_time_next_kernel: the next kernel launch carries these
  // as its start/stop events
  polar_hip_event* timeStart = nullptr;
  polar_hip_event* timeStop = nullptr;

  // this device's copy of the file-scope scratch array that
  // polar_hip_fsoftmax_static works in (resolved once, at open)
  void* softmaxScratch = nullptr;

  // Workspace of the builtins that run more than one kernel per call (softmax
  // partial sums, split-K partial products): one block that grows on demand to
  // the largest request seen so far (workspaceFor), so that a call whose size
  // has been seen before neither allocates nor waits.  workspaceMu is held
  // while a call enqueues the kernels that share it.
  std::mutex workspaceMu;
  void* workspace = nullptr;
  uint64_t workspaceBytes = 0;
  // One arrival counter per C tile of a split contraction whose last-arriving
  // work-group adds the partial products itself (matmul.hip).  Allocated and
  // zeroed when the device is opened; the group that completes a tile sets its
  // counter back to zero, so every launch finds zeros.  Used under workspaceMu.
  uint32_t* tileCounters = nullptr;
  // Transfers queued directly out of or into blocks of polar_hip_host_alloc are
  // numbered per device handle; directDone is the highest number known to be
  // complete, learnt from whatever the caller waits for anyway (an event
  // recorded behind the transfer, the whole stream), so that the blocks need no
  // events of their own.  `serial` names this handle in the blocks' bookkeeping.
  uint64_t serial = 0;
  std::atomic<uint64_t> directQueued{0}, directDone{0};
  // threads waiting for this handle's stream on behalf of a host block, outside
  // the table's mutex; the handle is not destroyed while there are any
  std::atomic<int> waiters{0};
  void noteDirectDone(uint64_t number) {
    uint64_t seen = directDone.load(std::memory_order_relaxed);
    while (seen < number && !directDone.compare_exchange_weak(seen, number)) {
    }
  }
};

struct polar_hip_module {
  polar_hip_device* dev = nullptr;
  hipModule_t module = nullptr;
  std::vector<char> image;
  std::mutex mu;
  std::unordered_map<std::string, hipFunction_t> functions; // null = not in the module
};

namespace polar_hip_detail {

int fail(polar_hip_status st, const char* fmt, ...)
    __attribute__((format(printf, 2, 3)));
int failHip(hipError_t e, const char* what);
int resolveStaticScratch(polar_hip_device* dev); // elementwise.hip

// The matmul planner never asks for more split-K workspace than this, and the
// partial sums of a softmax over 2^31 elements take 256 KiB.
constexpr uint64_t kWorkspaceBytes = 256ull << 20;
// *area: the device's workspace, at least `bytes` long (256-byte aligned,
// contents undefined), grown if it was smaller.  Caller holds dev->workspaceMu.
// Fails for a request above kWorkspaceBytes.
int workspaceFor(polar_hip_device* dev, uint64_t bytes, void** area); // runtime.hip
constexpr uint32_t kTileCounters = 16384;  // entries of polar_hip_device::tileCounters

// Every kernel of the library is launched through here.  Normally a plain
// launch on the device's stream; when a timing pair is armed, the launch
// carries the pair so that the events take the kernel's own begin and end
// timestamps (no host or queue gaps in between).
template <typename... KArgs, typename... Args>
inline hipError_t launchKernelLds(polar_hip_device* dev, void (*kernel)(KArgs...),
                                  dim3 grid, dim3 block, uint32_t dynamicLdsBytes,
                                  Args... args) {
  if (dev->timeStart != nullptr) {
    hipEvent_t e0 = dev->timeStart->ev, e1 = dev->timeStop->ev;
    dev->timeStart = dev->timeStop = nullptr;
    hipExtLaunchKernelGGL(kernel, grid, block, dynamicLdsBytes, dev->stream, e0, e1,
                          0, static_cast<KArgs>(args)...);
  } else {
    hipLaunchKernelGGL(kernel, grid, block, dynamicLdsBytes, dev->stream,
                       static_cast<KArgs>(args)...);
  }
  return hipGetLastError();
}

template <typename... KArgs, typename... Args>
inline hipError_t launchKernel(polar_hip_device* dev, void (*kernel)(KArgs...),
                               dim3 grid, dim3 block, Args... args) {
  return launchKernelLds(dev, kernel, grid, block, 0u, args...);
}

// Streaming stores for output that the kernel does not read again: the
// non-temporal hint plus device-scope write-through (sc1), so the lines leave
// the XCD's L2 as they are written instead of lingering there dirty.  Measured
// on a 2^26-element copy: 84.0 us with the non-temporal hint alone, 81.5 us
// with both (stores without any hint 88 us).
typedef float polar_v4f __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void streamStore(polar_v4f value, polar_v4f* address) {
  // The compiler does not look into the asm text, so it cannot see that a
  // 128-bit store's data registers must not be overwritten by the next
  // instruction or two (the hazard it pads itself for stores it emits): the
  // two wait states are part of the statement.
  asm volatile("global_store_dwordx4 %0, %1, off sc1 nt\n\ts_nop 1"
               : : "v"(address), "v"(value) : "memory");
}
__device__ __forceinline__ void streamStore(float value, float* address) {
  asm volatile("global_store_dword %0, %1, off sc1 nt" : : "v"(address), "v"(value) : "memory");
}
// the same, kByteOffset (0 .. 4095) bytes behind `address`: the offset travels
// in the instruction, so several stores share one address computation
template <int kByteOffset>
__device__ __forceinline__ void streamStoreAt(float value, float* address) {
  static_assert(kByteOffset >= 0 && kByteOffset < 4096, "offset field of the store");
  asm volatile("global_store_dword %0, %1, off offset:%2 sc1 nt"
               : : "v"(address), "v"(value), "n"(kByteOffset) : "memory");
}

inline bool aligned16(const void* p) {
  return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}

} // namespace polar_hip_detail

#define POLAR_HIP_TRY(expr)                                                    \
  do {                                                                         \
    hipError_t e_ = (expr);                                                    \
    if (e_ != hipSuccess) return polar_hip_detail::failHip(e_, #expr);        \
  } while (0)

#define POLAR_HIP_REQUIRE(cond, msg)                                           \
  do {                                                                         \
    if (!(cond))                                                               \
      return polar_hip_detail::fail(POLAR_HIP_ERR_INVALID, "%s: %s", __func__, \
                                    msg);                                      \
  } while (0)
