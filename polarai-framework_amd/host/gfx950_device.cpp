#include "hip_plugin.hpp"

#include <cstdio>

namespace polarai::backend::generic::mi355x {

HipDevice::HipDevice(int ordinal) {
  checkStatus(polar_hip_device_open(ordinal, &mDev), "polar_hip_device_open");
  polar_hip_device_info info;
  checkStatus(polar_hip_device_get_info(mDev, &info), "polar_hip_device_get_info");
  // The framework keys its per-device tables by this string and compares it
  // with "host" on every call (src/backend/generic/lib/allocators/
  // LayerAllocator.cpp:30,60; src/backend/generic/runtime/support/
  // routines.cpp:29,40,55): it must be unique per GPU and never "host".
  char buf[384];
  std::snprintf(buf, sizeof(buf), "%s (%s) hip:%d pci:%02x",
                info.name[0] ? info.name : "AMD Instinct GPU", info.arch,
                info.ordinal, info.pci_bus_id);
  mName = buf;
  mAllocator = std::make_shared<HipPoolAllocator>(mDev);
}

HipDevice::~HipDevice() {
  if (mDev) polar_hip_device_synchronize(mDev);
  if (mModule != nullptr) polar_hip_module_unload(mDev, mModule);
  mIdleEvents.clear();
  mEvents.clear();
  mAllocator->detach(); // other owners may keep the layer; its blocks die here
  if (mDev) polar_hip_device_close(mDev);
}

void HipDevice::copyToHost(MemoryRecord record, void* dest) const {
  void* src = mAllocator->getPtr(record);
  if (src == nullptr)
    fatal("copyToHost: tensor %zu has no allocation on %s", record.virtualAddress,
          mName.c_str());
  checkStatus(polar_hip_copy_to_host(mDev, dest, src, record.allocationSize),
              "polar_hip_copy_to_host");
}

void HipDevice::copyToDevice(MemoryRecord record, void* src) const {
  void* dst = mAllocator->getPtr(record);
  if (dst == nullptr)
    fatal("copyToDevice: tensor %zu has no allocation on %s",
          record.virtualAddress, mName.c_str());
  checkStatus(polar_hip_copy_to_device(mDev, dst, src, record.allocationSize),
              "polar_hip_copy_to_device");
}

float* HipDevice::resolve(BackendAllocator& allocator, const MemoryRecord& record) {
  float* p = allocator.get<float>(record, *this);
  if (p == nullptr)
    fatal("tensor %zu has no allocation on %s", record.virtualAddress, mName.c_str());
  return p;
}

// The event of the launch just enqueued: its ordinal on the stream.
HipEvent* HipDevice::newEvent() {
  const uint64_t ordinal = mLaunched.fetch_add(1, std::memory_order_acq_rel) + 1;
  std::lock_guard<std::mutex> g(mEventMutex);
  if (!mIdleEvents.empty()) {
    HipEvent* e = mIdleEvents.back();
    mIdleEvents.pop_back();
    e->rearm(ordinal);
    return e;
  }
  mEvents.push_back(std::make_unique<HipEvent>(this, ordinal));
  return mEvents.back().get();
}

// One native marker serves every event up to the newest launch: it is
// recorded behind all work enqueued so far (single in-order stream), so its
// completion implies theirs.  A barrier over the N events of a cluster thus
// costs one record and one wait instead of N of each (3 us per record, 7 us
// per wait, measured; polling the stream itself instead of a marker event
// measured 15 us slower per barrier).
void HipDevice::waitForLaunch(uint64_t ordinal) {
  if (mCompleted.load(std::memory_order_acquire) >= ordinal) return;
  std::lock_guard<std::mutex> g(mSyncMutex);
  if (mCompleted.load(std::memory_order_acquire) >= ordinal) return;
  // read before recording: launches enqueued meanwhile only make the marker
  // cover more than it claims
  const uint64_t covered = mLaunched.load(std::memory_order_acquire);
  polar_hip_event* marker = nullptr;
  checkStatus(polar_hip_event_record(mDev, &marker), "polar_hip_event_record");
  checkStatus(polar_hip_event_synchronize(marker), "polar_hip_event_synchronize");
  checkStatus(polar_hip_event_release(marker), "polar_hip_event_release");
  mCompleted.store(covered, std::memory_order_release);
}

// Enqueues one builtin operation.  A dependency recorded on this device needs
// no wait: the device has one in-order stream, so the new kernel already runs
// after it.  A foreign event is waited for on the host, as the framework's
// SYCL runtime does for every dependency
// (src/backend/generic/runtime/sycl/SYCLDevice.cpp:37-42).
// The returned event is owned by the device; the pointer stays valid until
// consumeEvent() or the end of the context.
Event* HipDevice::launch(BackendAllocator& allocator, LaunchCommand& cmd,
                         Event* blockingEvent) {
  if (blockingEvent != nullptr && blockingEvent->getDevice() != this)
    blockingEvent->wait();
  // Hand-written kernels first; a kernel of the selected code object otherwise.
  const bool native = cmd.nativeKernelName != nullptr && cmd.nativeKernelName[0] != 0 &&
                      dispatchNativeKernel(*this, allocator, cmd);
  if (!native && !launchFromProgram(allocator, cmd)) {
    if (cmd.nativeKernelName == nullptr || cmd.nativeKernelName[0] == 0)
      fatal("launch of '%s' without a native kernel name, and no selected program defines it",
            cmd.kernelName ? cmd.kernelName : "?");
    fatal("no native kernel '%s' (requested by '%s')", cmd.nativeKernelName,
          cmd.kernelName ? cmd.kernelName : "?");
  }
  return newEvent();
}

// Keeps the first HSACO program whose target names this device's architecture
// (or no target).  The reference's CUDA runtime does the same with the first
// PTX program (src/backend/generic/runtime/cuda/CudaDevice.cpp:39-61); its SYCL
// runtime ignores programs altogether (sycl/SYCLDevice.h:121-122).
void HipDevice::selectBinary(std::vector<std::shared_ptr<ProgramDesc>>& programs) {
  polar_hip_device_info info;
  checkStatus(polar_hip_device_get_info(mDev, &info), "polar_hip_device_get_info");
  std::string arch = info.arch;
  arch = arch.substr(0, arch.find(':'));
  for (auto& program : programs) {
    if (program == nullptr || program->type != ProgramDesc::Type::HSACO) continue;
    if (!program->target.empty() && program->target.compare(0, arch.size(), arch) != 0) continue;
    if (mModule != nullptr) {
      checkStatus(polar_hip_module_unload(mDev, mModule), "polar_hip_module_unload");
      mModule = nullptr;
    }
    checkStatus(polar_hip_module_load(mDev, program->data.data(), program->data.size(), &mModule),
                "polar_hip_module_load");
    mProgram = program;
    return;
  }
}

// Launch cmd.kernelName from the selected program with the geometry recorded
// for it.  Tensor arguments expand to a memref descriptor -- allocated
// pointer, aligned pointer, offset, sizes, strides -- as the generated code
// expects (cuda/CudaDevice.cpp:75-94; the strides there are zeros, here they
// are the row-major strides of the dense tensor); scalars are passed through.
bool HipDevice::launchFromProgram(BackendAllocator& allocator, LaunchCommand& cmd) {
  if (mModule == nullptr || cmd.kernelName == nullptr) return false;
  auto geometry = mProgram->kernels.find(cmd.kernelName);
  if (geometry == mProgram->kernels.end()) return false;
  int found = 0;
  checkStatus(polar_hip_module_has_kernel(mModule, cmd.kernelName, &found),
              "polar_hip_module_has_kernel");
  if (!found) return false;

  std::vector<void*> pointers;          // device pointers, two slots per tensor
  std::vector<int64_t> integers;        // offsets, sizes, strides
  std::vector<std::pair<int, size_t>> layout; // (0 pointer / 1 integer / 2 scalar, index)
  uint64_t tensors = 0, words = 0;
  for (uint64_t i = 0; i < cmd.argsCount; ++i) {
    // validated before the first use: the sizing pass below reads the tensor's rank
    if (cmd.args[i].arg == nullptr)
      fatal("%s: argument %llu is null", cmd.kernelName, (unsigned long long)i);
    if (cmd.args[i].type == ArgDesc::TENSOR) {
      ++tensors;
      words += 1 + 2 * static_cast<TensorInfo*>(cmd.args[i].arg)->dims;
    }
  }
  pointers.reserve(2 * tensors); // addresses of the elements are taken below
  integers.reserve(words);
  for (uint64_t i = 0; i < cmd.argsCount; ++i) {
    const ArgDesc& a = cmd.args[i];
    if (a.type != ArgDesc::TENSOR) {
      layout.emplace_back(2, i);
      continue;
    }
    auto* t = static_cast<TensorInfo*>(a.arg);
    if (t->dataType != static_cast<int>(core::DataType::FLOAT))
      fatal("%s: tensor %llu has data type %d; this runtime is fp32 only", cmd.kernelName,
            (unsigned long long)t->virtAddr, t->dataType);
    MemoryRecord record{static_cast<size_t>(t->virtAddr), 4};
    for (uint64_t d = 0; d < t->dims; ++d) record.allocationSize *= t->shape[d];
    float* ptr = resolve(allocator, record);
    for (int k = 0; k < 2; ++k) {
      layout.emplace_back(0, pointers.size());
      pointers.push_back(ptr);
    }
    layout.emplace_back(1, integers.size());
    integers.push_back(0); // offset
    for (uint64_t d = 0; d < t->dims; ++d) {
      layout.emplace_back(1, integers.size());
      integers.push_back(static_cast<int64_t>(t->shape[d]));
    }
    const size_t firstStride = integers.size();
    for (uint64_t d = 0; d < t->dims; ++d) {
      layout.emplace_back(1, integers.size());
      integers.push_back(1);
    }
    for (uint64_t d = t->dims; d-- > 1;)
      integers[firstStride + d - 1] =
          integers[firstStride + d] * static_cast<int64_t>(t->shape[d]);
  }
  std::vector<void*> params;
  params.reserve(layout.size());
  for (auto& [kind, index] : layout)
    params.push_back(kind == 0   ? static_cast<void*>(&pointers[index])
                     : kind == 1 ? static_cast<void*>(&integers[index])
                                 : cmd.args[index].arg);
  const KernelDesc& k = geometry->second;
  const uint32_t grid[3] = {static_cast<uint32_t>(k.globalX), static_cast<uint32_t>(k.globalY),
                            static_cast<uint32_t>(k.globalZ)};
  const uint32_t block[3] = {static_cast<uint32_t>(k.localX), static_cast<uint32_t>(k.localY),
                             static_cast<uint32_t>(k.localZ)};
  checkStatus(polar_hip_module_launch(mDev, mModule, cmd.kernelName, grid, block, params.data()),
              "polar_hip_module_launch");
  return true;
}

void HipDevice::consumeEvent(Event* evt) {
  if (evt == nullptr) return;
  if (evt->getDevice() != this) fatal("consumeEvent: event of another device");
  evt->wait();
  auto* mine = static_cast<HipEvent*>(evt);
  std::lock_guard<std::mutex> g(mEventMutex);
  mIdleEvents.push_back(mine);
}

namespace {
// Device through which polarHostMemoryAllocate takes pinned memory: the first
// device of the most recently created context, null when there is none.
std::mutex gHostMemoryMu;
HipDevice* gHostMemoryDevice = nullptr;
} // namespace

HipContext::~HipContext() {
  std::lock_guard<std::mutex> g(gHostMemoryMu);
  for (auto& d : mDevices)
    if (d.get() == gHostMemoryDevice) gHostMemoryDevice = nullptr;
}

HipContext::HipContext() {
  int n = 0;
  checkStatus(polar_hip_device_count(&n), "polar_hip_device_count");
  for (int i = 0; i < n; ++i) {
    // Only gfx950 parts are usable: the device library holds no other code.
    polar_hip_device* probe = nullptr;
    int st = polar_hip_device_open(i, &probe);
    if (st == POLAR_HIP_ERR_NO_DEVICE) continue;
    checkStatus(st, "polar_hip_device_open");
    polar_hip_device_close(probe);
    mDevices.push_back(std::make_shared<HipDevice>(i));
  }
  if (!mDevices.empty()) {
    std::lock_guard<std::mutex> g(gHostMemoryMu);
    gHostMemoryDevice = static_cast<HipDevice*>(mDevices.front().get());
  }
}

} // namespace polarai::backend::generic::mi355x

extern "C" {

polarai::backend::generic::Context* initContext() {
  return new polarai::backend::generic::mi355x::HipContext();
}

void closeContext(polarai::backend::generic::Context* ctx) { delete ctx; }

// Optional extension, not part of the framework's interface: host memory for
// the caller's RAM-side copies of tensors (the framework's TrivialAllocator
// uses new[]: src/backend/generic/lib/allocators/TrivialAllocator.hpp:23-93).
// Blocks from here are pinned; copyToDevice / copyToHost move bytes directly
// between them and device memory instead of staging them.  Because an upload
// out of such a block is only queued when copyToDevice returns, the caller calls
// polarHostMemoryQuiesce(block) before the host writes the block again.
// polarHostMemoryAllocate returns null when no context with a device exists.
void* polarHostMemoryAllocate(size_t bytes) {
  using namespace polarai::backend::generic::mi355x;
  std::lock_guard<std::mutex> g(gHostMemoryMu);
  if (gHostMemoryDevice == nullptr) return nullptr;
  void* p = nullptr;
  checkStatus(polar_hip_host_alloc(gHostMemoryDevice->native(), bytes, &p), "polar_hip_host_alloc");
  return p;
}
void polarHostMemoryRelease(void* block) {
  polarai::backend::generic::mi355x::checkStatus(polar_hip_host_free(block), "polar_hip_host_free");
}
void polarHostMemoryQuiesce(void* block) {
  polarai::backend::generic::mi355x::checkStatus(polar_hip_host_quiesce(block), "polar_hip_host_quiesce");
}

}

// Test hook, not part of the framework's interface: caps the capacity of a
// device's memory layer so that the eviction / offload path can be exercised
// without filling 288 GB.  `dev` must be a device returned by this plugin.
extern "C" int polar_rt_hip_set_device_byte_limit(polarai::backend::generic::Device* dev,
                                                  uint64_t bytes) {
  using namespace polarai::backend::generic;
  if (dev == nullptr || dev->getProvider() != DeviceProvider::HIP) return -1;
  auto* mine = static_cast<mi355x::HipDevice*>(dev);
  static_cast<mi355x::HipPoolAllocator*>(mine->getAllocator().get())->setByteLimit(bytes);
  return 0;
}
