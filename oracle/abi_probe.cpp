// Caller-side probe of the runtime-plugin interface, compiled against the
// REFERENCE's own headers (-I<reference>/include), never against this
// repository's restatement of them.  TEST INFRASTRUCTURE ONLY.
//
// Each function takes objects that were created by code built with
// include/polar_rt_abi.hpp (the plugin's devices, the mini-executor's mock
// device and allocator) and uses them through the reference's class
// declarations.  If the restated vtable order, a by-value parameter type or a
// struct layout differed from the reference's, these calls would land in the
// wrong function or read the wrong field, and the tests that drive this probe
// would fail.
//
// Only headers that compile straight from the reference tree are used
// (Context/Device/Event/AllocatorLayerBase/MemoryRecord/ProgramDesc,
// LaunchCommand.h, TensorInfo.h).  BackendAllocator.hpp is not: it needs the
// cmake-generated polar_core_export.h, so a BackendAllocator only passes
// through here as an opaque reference.
#include <cstddef>
#include <cstdint>
#include <cstring>
#include <map>
#include <memory>
#include <string>
#include <utility>
#include <vector>

#include <polarai/backend/generic/runtime/Context.hpp>
#include <polarai/backend/generic/runtime/Event.hpp>
#include <polarai/backend/generic/runtime/GraphHandle.hpp>
#include <polarai/backend/generic/runtime/LaunchCommand.h>
#include <polarai/backend/generic/runtime/TensorInfo.h>
// header-only in the reference, std headers only: what ath_load hands a loader
#include <polarai/backend/generic/runtime/BackendAccessor.hpp>
#include <polarai/core/tensor/Accessor.hpp>

using namespace polarai::backend::generic;

// The support library under test (libpolar_rt_support_static.a, linked into
// this probe).  The reference declares the seven routines in
// src/backend/generic/runtime/support/api.hpp:18-32, which cannot be included
// here (it needs a cmake-generated export header), so the prototypes are
// written out with the reference's types; LockType is passed as the int the
// lowering emits (READ = 0, READ_WRITE = 1 --
// include/polarai/core/loader/internal/TensorAllocator.hpp:22).
extern "C" {
void ath_allocate(GraphHandle*, Device&, TensorInfo*);
void ath_release(GraphHandle*, Device&, TensorInfo*, Event*);
void ath_lock(GraphHandle*, Device&, TensorInfo*, int lockType);
Device* ath_device_select(GraphHandle*, uint64_t nodeId);
void ath_barrier(uint32_t count, Event** events);
Event* ath_launch(GraphHandle*, Device*, Event*, LaunchCommand&);
void ath_load(GraphHandle*, uint64_t nodeId, TensorInfo*);
BackendAllocator* polar_rt_support_allocator_create();
void polar_rt_support_allocator_destroy(BackendAllocator*);
void polar_rt_support_register_device(BackendAllocator*, Device*);
Device* polar_rt_support_host_device_create();
void polar_rt_support_host_device_destroy(Device*);
void polar_rt_support_graph_handle_layout(uint64_t out[5]);
}

namespace {
// A loader with the vtable of the framework's loaders: the virtual destructor
// inherited from Entity (include/polarai/core/Entity.hpp:29), then
// load(Accessor<float>&) (include/polarai/core/loader/internal/
// AbstractLoaderInternal.hpp:32).  AbstractLoaderInternal.hpp itself cannot be
// included (it needs a cmake-generated export header), but the accessor it is
// handed is the reference's own class template, so every call below goes
// through the reference's declaration of Accessor<float>: if the support
// library built its accessor with another virtual order, these calls would
// land in the wrong function.  `fill` copies data in; `drain` copies the tensor
// out (how this probe reads results: the library hands the loader the RAM copy).
struct ProbeLoader {
  virtual ~ProbeLoader() = default;
  virtual void load(polarai::core::Accessor<float>& acc) {
    const std::vector<size_t>& shape = acc.getShape();
    size_t count = 1;
    for (size_t d : shape) count *= d;
    dims = shape.size();
    float* raw = acc.getRawPtr();
    if (fill != nullptr) {
      std::memcpy(raw, fill, count * sizeof(float));
      acc(size_t(0)) = fill[0];      // element access by flat index
      if (dims == 1) acc({count - 1}) = fill[count - 1]; // and by index list
    }
    if (drain != nullptr) {
      std::memcpy(drain, raw, count * sizeof(float));
      drain[0] = acc(size_t(0));
      if (dims == 1) drain[count - 1] = acc({count - 1});
    }
    ++calls;
  }
  const float* fill = nullptr;
  float* drain = nullptr;
  size_t dims = 0;
  int calls = 0;
};
} // namespace

extern "C" {

// sizeof / offsetof of the plain structs as the reference declares them
void ref_struct_layout(uint64_t* out /* 12 values */) {
  out[0] = sizeof(TensorInfo);
  out[1] = offsetof(TensorInfo, virtAddr);
  out[2] = offsetof(TensorInfo, dataType);
  out[3] = offsetof(TensorInfo, dims);
  out[4] = offsetof(TensorInfo, shape);
  out[5] = sizeof(ArgDesc);
  out[6] = offsetof(ArgDesc, arg);
  out[7] = offsetof(ArgDesc, type);
  out[8] = sizeof(LaunchCommand);
  out[9] = offsetof(LaunchCommand, argsCount);
  out[10] = offsetof(LaunchCommand, nativeKernelName);
  out[11] = sizeof(MemoryRecord);
}

int ref_context_device_count(void* context) {
  return static_cast<int>(static_cast<Context*>(context)->getDevices().size());
}

void* ref_context_device(void* context, int index) {
  return static_cast<Context*>(context)->getDevices().at(index).get();
}

// Device information through the reference's vtable.
// out: provider, kind, hasAllocator, isPartitionSupported(EQUALLY),
//      partition(EQUALLY).size(), (device == device), (device != device)
void ref_device_info(void* device, char* name, size_t nameLen, int* out) {
  auto* d = static_cast<Device*>(device);
  const std::string n = d->getDeviceName();
  std::strncpy(name, n.c_str(), nameLen - 1);
  name[nameLen - 1] = 0;
  out[0] = static_cast<int>(d->getProvider());
  out[1] = static_cast<int>(d->getKind());
  out[2] = d->hasAllocator();
  out[3] = d->isPartitionSupported(Device::PartitionDomain::EQUALLY);
  out[4] = static_cast<int>(d->partition(Device::PartitionDomain::EQUALLY).size());
  out[5] = (*d == *d);
  out[6] = (*d != *d);
  out[7] = static_cast<int>(std::hash<Device>()(*d) == std::hash<std::string>()(n));
  std::vector<std::shared_ptr<ProgramDesc>> none;
  d->selectBinary(none); // must be callable and do nothing harmful
}

// Allocator layer round trip through the reference's vtable, and a host ->
// device -> host copy through Device::copyToDevice / copyToHost.
// Returns 0 if every step behaved, otherwise the number of the failing step.
int ref_allocator_and_copy(void* device, size_t vaddr, const float* src, float* dst,
                           size_t count) {
  auto* d = static_cast<Device*>(device);
  std::shared_ptr<AllocatorLayerBase> layer = d->getAllocator();
  if (!layer) return 1;
  MemoryRecord rec{vaddr, count * sizeof(float)};
  if (layer->isAllocated(rec)) return 2;
  layer->allocate(rec);
  if (!layer->isAllocated(rec)) return 3;
  if (layer->getTag(rec) != 1) return 4;           // allocate sets tag 1
  layer->allocate(rec);                              // double allocation: no-op
  layer->setTag(rec, 7);
  if (layer->getTag(rec) != 7) return 5;
  if (layer->getPtr(rec) == nullptr) return 6;
  layer->lock(rec);
  d->copyToDevice(rec, const_cast<float*>(src));
  d->copyToHost(rec, dst);
  layer->release(rec);
  layer->deallocate(rec);
  if (layer->isAllocated(rec)) return 7;
  int called = 0;
  layer->registerMemoryOffloadCallback([&called](MemoryRecord, AllocatorLayerBase&) { ++called; });
  return 0;
}

// Launch through Device::launch with structs laid out by the reference's
// headers, then Event::addCallback / wait / getDevice and consumeEvent.
// `allocator` is a BackendAllocator built elsewhere (opaque here).  Tensors
// must already be allocated and locked on the device by the caller.
// Returns 0 on success, else the failing step.
int ref_launch_fadd(void* device, void* allocator, uint64_t va, uint64_t vb, uint64_t vc,
                    uint64_t count, float scaleA, float scaleB) {
  auto* d = static_cast<Device*>(device);
  uint64_t shape[1] = {count};
  TensorInfo ta{va, 2, 1, shape}, tb{vb, 2, 1, shape}, tc{vc, 2, 1, shape};
  ArgDesc args[5];
  args[0] = ArgDesc{0, &ta, ArgDesc::TENSOR};
  args[1] = ArgDesc{sizeof(float), &scaleA, ArgDesc::DATA};
  args[2] = ArgDesc{0, &tb, ArgDesc::TENSOR};
  args[3] = ArgDesc{sizeof(float), &scaleB, ArgDesc::DATA};
  args[4] = ArgDesc{0, &tc, ArgDesc::TENSOR};
  LaunchCommand cmd{"probe_fadd", 5, args, "fadd"};
  Event* evt = d->launch(*static_cast<BackendAllocator*>(allocator), cmd, nullptr);
  if (evt == nullptr) return 1;
  int ran = 0;
  evt->addCallback([&ran]() { ++ran; });
  if (ran != 0) return 2;            // callbacks run in wait(), not before
  evt->wait();
  if (ran != 1) return 3;
  evt->wait();                       // callbacks run once
  if (ran != 1) return 4;
  if (evt->getDevice() == nullptr) return 5;
  // a second launch that depends on the first event
  Event* evt2 = d->launch(*static_cast<BackendAllocator*>(allocator), cmd, evt);
  if (evt2 == nullptr) return 6;
  d->consumeEvent(evt2);             // waits and gives the event back
  return 0;
}

// sizeof(GraphHandle) and member offsets as the reference declares it, then
// the same five numbers as the support library was compiled.
void ref_graph_handle_layout(uint64_t* out) {
  out[0] = sizeof(GraphHandle);
  out[1] = offsetof(GraphHandle, allocator);
  out[2] = offsetof(GraphHandle, devices);
  out[3] = offsetof(GraphHandle, mLoaders);
  out[4] = offsetof(GraphHandle, isHostNode);
  polar_rt_support_graph_handle_layout(out + 5);
}

// One graph evaluation as JIT-compiled code performs it
// (src/core/graph/internal/GraphCompiler.cpp:55-108), on a GraphHandle laid
// out by the reference's header, through the support library's ath_*:
// two input nodes (host), one fadd node on `device`, a barrier, then a host
// read of the result (pulled from the device by the host lock) and of the
// first input (whose RAM copy must have survived the device's READ lock).  `device` comes from a runtime plugin or is the mini-executor's mock
// (which computes nothing: sum is then left untouched by the launch).
// Returns 0 on success, else the failing step.
int ref_support_evaluate(void* device, uint64_t count, const float* a, const float* b,
                         float scaleA, float scaleB, float* sum, float* aBack) {
  auto* dev = static_cast<Device*>(device);
  BackendAllocator* rawAllocator = polar_rt_support_allocator_create();
  Device* rawHost = polar_rt_support_host_device_create();
  if (rawAllocator == nullptr || rawHost == nullptr) return 1;
  polar_rt_support_register_device(rawAllocator, dev);

  ProbeLoader loadA, loadB, readSum, readA;
  loadA.fill = a;
  loadB.fill = b;
  readSum.drain = sum;
  readA.drain = aBack;
  using Loader = polarai::core::internal::AbstractLoaderInternal;
  int status = 0;
  {
    GraphHandle handle;
    handle.allocator = std::shared_ptr<BackendAllocator>(
        rawAllocator, [](BackendAllocator* p) { polar_rt_support_allocator_destroy(p); });
    handle.devices.push_back(std::shared_ptr<Device>(dev, [](Device*) {})); // borrowed
    handle.devices.push_back(
        std::shared_ptr<Device>(rawHost, [](Device* p) { polar_rt_support_host_device_destroy(p); }));
    handle.mLoaders[1] = reinterpret_cast<Loader*>(&loadA);
    handle.mLoaders[2] = reinterpret_cast<Loader*>(&loadB);
    handle.mLoaders[4] = reinterpret_cast<Loader*>(&readSum);
    handle.mLoaders[5] = reinterpret_cast<Loader*>(&readA);
    for (uint64_t id : {1, 2, 4, 5}) handle.isHostNode.insert(id);

    uint64_t shape[1] = {count};
    const uint64_t bytes = count * sizeof(float);
    TensorInfo ta{1, 2, 1, shape}, tb{1 + bytes, 2, 1, shape}, tc{1 + 2 * bytes, 2, 1, shape};

    // input nodes
    for (auto [id, t] : {std::pair<uint64_t, TensorInfo*>{1, &ta}, {2, &tb}}) {
      Device* host = ath_device_select(&handle, id);
      if (host != rawHost) { status = 2; break; }
      ath_allocate(&handle, *host, t);
      ath_lock(&handle, *host, t, 1);
      ath_load(&handle, id, t);
      ath_release(&handle, *host, t, nullptr);
    }
    // fadd node
    Event* evt = nullptr;
    if (status == 0) {
      Device* sel = ath_device_select(&handle, 3);
      if (sel != dev) status = 3;
    }
    if (status == 0) {
      ath_allocate(&handle, *dev, &tc);
      ath_lock(&handle, *dev, &ta, 0);
      ath_lock(&handle, *dev, &tb, 0);
      ath_lock(&handle, *dev, &tc, 1);
      ArgDesc args[5];
      args[0] = ArgDesc{0, &ta, ArgDesc::TENSOR};
      args[1] = ArgDesc{sizeof(float), &scaleA, ArgDesc::DATA};
      args[2] = ArgDesc{0, &tb, ArgDesc::TENSOR};
      args[3] = ArgDesc{sizeof(float), &scaleB, ArgDesc::DATA};
      args[4] = ArgDesc{0, &tc, ArgDesc::TENSOR};
      LaunchCommand cmd{"probe_fadd", 5, args, "fadd"};
      evt = ath_launch(&handle, dev, nullptr, cmd);
      if (evt == nullptr) status = 4;
    }
    if (status == 0) {
      ath_release(&handle, *dev, &ta, evt);
      ath_release(&handle, *dev, &tb, evt);
      ath_release(&handle, *dev, &tc, evt);
      Event* events[2] = {evt, nullptr}; // null entries are skipped
      ath_barrier(2, events);
      // output nodes: a host lock pulls the newest copy into RAM
      for (auto [id, t] : {std::pair<uint64_t, TensorInfo*>{4, &tc}, {5, &ta}}) {
        Device* host = ath_device_select(&handle, id);
        ath_lock(&handle, *host, t, 0);
        ath_load(&handle, id, t);
        ath_release(&handle, *host, t, nullptr);
      }
    }
  } // handle (allocator, host device) destroyed
  if (status == 0 && (loadA.calls != 1 || loadB.calls != 1 || readSum.calls != 1 || readA.calls != 1 ||
                      loadA.dims != 1))
    status = 5; // every loader ran exactly once, through the right vtable slot
  return status;
}

} // extern "C"
