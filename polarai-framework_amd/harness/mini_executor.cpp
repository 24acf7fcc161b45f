// The mini-executor: loads a runtime plugin like the framework's runtime
// driver, keeps a program of input and compute nodes grouped in clusters, and
// evaluates it with the call sequence of JIT-compiled graph code.
#include "devices.hpp"
#include "support_routines.hpp"

#include <dlfcn.h>

#include <cstdio>
#include <chrono>
#include <cstring>

using namespace polar_harness_detail;
using polarai::core::internal::AbstractLoaderInternal;

namespace {

// The framework's MemcpyLoader (src/loaders/internal/MemcpyLoaderInternal.cpp:24-27)
// With no data it behaves like the framework's DummyLoader (loads nothing),
// which the gradient graphs use for nodes that only hold an existing tensor.
class MemcpyLoader final : public AbstractLoaderInternal {
public:
  MemcpyLoader(const float* data, size_t count) {
    if (data != nullptr) mData.assign(data, data + count);
  }
  void load(polarai::core::Accessor<float>& acc) override {
    if (mData.empty()) return;
    size_t count = 1;
    for (size_t d : acc.getShape()) count *= d;
    std::memcpy(acc.getRawPtr(), mData.data(),
                (count < mData.size() ? count : mData.size()) * sizeof(float));
  }

private:
  std::vector<float> mData;
};

// What stands for the framework's tensor object in this binary.  The support
// library only calls three member functions of TensorInternal and leaves them
// undefined (in a framework build they are polar_core's); here they read this
// struct, and a HarnessTensor is handed over as a TensorInternal.
struct HarnessTensor {
  size_t virtualAddress;
  polarai::core::DataType type;
  size_t elements;
  const polarai::core::internal::TensorInternal& asTensor() const {
    return *reinterpret_cast<const polarai::core::internal::TensorInternal*>(this);
  }
};

struct TensorDecl {
  uint64_t vaddr;
  std::vector<uint64_t> shape;
  TensorInfo info() { return TensorInfo{vaddr, 2 /* FLOAT */, shape.size(), shape.data()}; }
};

struct NodeDecl {
  uint64_t id;
  bool isInput;
  std::string kernel;   // native kernel name ("" for a kernel of the selected program)
  std::string jitName;  // name of the generated kernel; derived from the node when empty
  std::vector<polar_harness_arg> args;
  uint32_t result;      // index into args (compute) ...
  uint64_t inputVaddr;  // ... or the tensor an input node fills
  std::unique_ptr<MemcpyLoader> loader;
};

} // namespace

namespace polarai::core::internal {
DataType TensorInternal::getDataType() const {
  return reinterpret_cast<const HarnessTensor*>(this)->type;
}
size_t TensorInternal::getSize() const { return reinterpret_cast<const HarnessTensor*>(this)->elements; }
size_t TensorInternal::getVirtualAddress() const {
  return reinterpret_cast<const HarnessTensor*>(this)->virtualAddress;
}
} // namespace polarai::core::internal

struct polar_harness {
  void* lib = nullptr;
  Context* ctx = nullptr;
  void (*closeCtx)(Context*) = nullptr;
  int (*setByteLimit)(Device*, uint64_t) = nullptr;
  MockDevice* mock = nullptr;              // set when the built-in mock device is used
  std::shared_ptr<Device> inner;           // device under test
  std::shared_ptr<CountingDevice> device;  // what the graph code sees
  std::shared_ptr<HostDevice> host;
  std::shared_ptr<CoherentAllocator> allocator;
  polar_harness_counters counters{};
  int deviceCount = 0;
  std::string name;

  uint64_t nextVaddr = 1; // src/core/context/internal/ContextInternal.cpp:24,43-48
  std::unordered_map<uint64_t, TensorDecl> tensors;
  std::vector<std::vector<NodeDecl>> clusters{1};
  uint64_t nextNodeId = 1;

  TensorDecl* find(uint64_t vaddr) {
    auto it = tensors.find(vaddr);
    return it == tensors.end() ? nullptr : &it->second;
  }
};

extern "C" {

// src/backend/generic/runtime/driver/RuntimeDriver.cpp:12-41 and
// DynamicLibrary_posix.cpp:10: dlopen(RTLD_LAZY | RTLD_LOCAL), dlsym of the two
// entry points, devices taken from the context.
int polar_harness_open(const char* plugin_path, int device_index, polar_harness** out) {
  if (out == nullptr) return -1;
  *out = nullptr;
  auto h = std::make_unique<polar_harness>();
  if (plugin_path == nullptr) {
    auto mock = std::make_shared<MockDevice>();
    h->mock = mock.get();
    h->inner = mock;
    h->deviceCount = 1;
  } else {
    h->lib = dlopen(plugin_path, RTLD_LAZY | RTLD_LOCAL);
    if (h->lib == nullptr) {
      std::fprintf(stderr, "Failed to load %s\n%s\n", plugin_path, dlerror());
      return -1;
    }
    auto init = reinterpret_cast<Context* (*)()>(dlsym(h->lib, "initContext"));
    h->closeCtx = reinterpret_cast<void (*)(Context*)>(dlsym(h->lib, "closeContext"));
    h->setByteLimit = reinterpret_cast<int (*)(Device*, uint64_t)>(
        dlsym(h->lib, "polar_rt_hip_set_device_byte_limit"));
    if (init == nullptr || h->closeCtx == nullptr) {
      std::fprintf(stderr, "%s does not export initContext/closeContext\n", plugin_path);
      dlclose(h->lib);
      return -1;
    }
    h->ctx = init();
    auto& devs = h->ctx->getDevices();
    h->deviceCount = static_cast<int>(devs.size());
    if (device_index < 0 || device_index >= h->deviceCount) {
      std::fprintf(stderr, "%s reports %d device(s); index %d requested\n", plugin_path,
                   h->deviceCount, device_index);
      h->closeCtx(h->ctx);
      dlclose(h->lib);
      return -1;
    }
    h->inner = devs[device_index];
  }
  h->device = std::make_shared<CountingDevice>(h->inner, &h->counters);
  h->host = std::make_shared<HostDevice>();
  h->allocator = std::make_shared<CoherentAllocator>();
  h->allocator->registerDevice(*h->device); // src/backend/generic/lib/ExecutorImpl.cpp:130-136
  h->name = h->device->getDeviceName();
  *out = h.release();
  return 0;
}

void polar_harness_close(polar_harness* h) {
  if (h == nullptr) return;
  // allocator first (it points at the devices), then devices, then the context
  h->allocator.reset();
  h->device.reset();
  h->inner.reset();
  if (h->ctx != nullptr) h->closeCtx(h->ctx);
  if (h->lib != nullptr) dlclose(h->lib);
  delete h;
}

int polar_harness_device_count(polar_harness* h) { return h ? h->deviceCount : -1; }
const char* polar_harness_device_name(polar_harness* h) { return h ? h->name.c_str() : nullptr; }
int polar_harness_device_provider(polar_harness* h) {
  return h ? static_cast<int>(h->inner->getProvider()) : -1;
}
int polar_harness_device_kind(polar_harness* h) {
  return h ? static_cast<int>(h->inner->getKind()) : -1;
}

int polar_harness_use_plugin_host_memory(polar_harness* h) {
  if (h == nullptr || h->lib == nullptr) return -1;
  auto allocate = reinterpret_cast<void* (*)(size_t)>(dlsym(h->lib, "polarHostMemoryAllocate"));
  auto release = reinterpret_cast<void (*)(void*)>(dlsym(h->lib, "polarHostMemoryRelease"));
  auto quiesce = reinterpret_cast<void (*)(void*)>(dlsym(h->lib, "polarHostMemoryQuiesce"));
  if (allocate == nullptr || release == nullptr || quiesce == nullptr) return -1;
  h->allocator->setHostMemory(allocate, release, quiesce);
  return 0;
}

uint64_t polar_harness_tensor(polar_harness* h, uint64_t dims, const uint64_t* shape) {
  if (h == nullptr || (dims > 0 && shape == nullptr)) return 0;
  TensorDecl t;
  t.vaddr = h->nextVaddr;
  t.shape.assign(shape, shape + dims);
  uint64_t bytes = 4;
  for (uint64_t d : t.shape) bytes *= d;
  h->nextVaddr += bytes;
  const uint64_t v = t.vaddr;
  h->tensors.emplace(v, std::move(t));
  return v;
}

int polar_harness_input(polar_harness* h, uint64_t vaddr, const float* data) {
  TensorDecl* t = h ? h->find(vaddr) : nullptr;
  if (t == nullptr) return -1;
  size_t count = 1;
  for (uint64_t d : t->shape) count *= d;
  NodeDecl n;
  n.id = h->nextNodeId++;
  n.isInput = true;
  n.result = 0;
  n.inputVaddr = vaddr;
  n.loader = std::make_unique<MemcpyLoader>(data, count);
  h->clusters.back().push_back(std::move(n));
  return 0;
}

int polar_harness_node(polar_harness* h, const char* native_kernel_name, uint32_t nargs,
                       const polar_harness_arg* args, uint32_t result_index) {
  if (h == nullptr || native_kernel_name == nullptr || args == nullptr || result_index >= nargs)
    return -1;
  for (uint32_t i = 0; i < nargs; ++i)
    if (args[i].kind == 0 && h->find(args[i].vaddr) == nullptr) return -1;
  if (args[result_index].kind != 0) return -1;
  NodeDecl n;
  n.id = h->nextNodeId++;
  n.isInput = false;
  n.kernel = native_kernel_name;
  n.args.assign(args, args + nargs);
  n.result = result_index;
  n.inputVaddr = 0;
  h->clusters.back().push_back(std::move(n));
  return 0;
}

int polar_harness_jit_node(polar_harness* h, const char* jit_kernel_name, uint32_t nargs,
                           const polar_harness_arg* args, uint32_t result_index) {
  if (jit_kernel_name == nullptr || jit_kernel_name[0] == 0) return -1;
  if (polar_harness_node(h, "", nargs, args, result_index) != 0) return -1;
  h->clusters.back().back().jitName = jit_kernel_name;
  return 0;
}

// src/backend/generic/lib/ExecutorImpl.cpp:52-64: after a graph is compiled the
// executor passes the generated programs to every device.
int polar_harness_select_binary(polar_harness* h, int program_type, const char* target,
                                const void* image, uint64_t bytes, uint32_t kernel_count,
                                const char* const* kernel_names, const uint64_t* geometry) {
  if (h == nullptr || image == nullptr || (kernel_count != 0 && (!kernel_names || !geometry)))
    return -1;
  auto program = std::make_shared<ProgramDesc>();
  program->type = static_cast<ProgramDesc::Type>(program_type);
  program->target = target ? target : "";
  program->data.assign(static_cast<const char*>(image), static_cast<const char*>(image) + bytes);
  for (uint32_t i = 0; i < kernel_count; ++i) {
    const uint64_t* g = geometry + 6 * i;
    program->kernels[kernel_names[i]] = KernelDesc{g[0], g[1], g[2], g[3], g[4], g[5]};
  }
  std::vector<std::shared_ptr<ProgramDesc>> programs{program};
  h->device->selectBinary(programs);
  return 0;
}

int polar_harness_end_cluster(polar_harness* h) {
  if (h == nullptr) return -1;
  h->clusters.emplace_back();
  return 0;
}

int polar_harness_clear_program(polar_harness* h) {
  if (h == nullptr) return -1;
  h->clusters.clear();
  h->clusters.emplace_back();
  return 0;
}

// Executor::evaluate (src/backend/generic/lib/ExecutorImpl.cpp:66-97) followed
// by what the JIT-compiled graph function does.  Per node
// (src/core/graph/internal/GraphCompiler.cpp:55-70,
//  src/core/operation/internal/OperationInternal.cpp:21-39):
//   device_select; allocate(result);
//   input node:   lock(result, RW); load; release(result)
//   compute node: lock(result, RW); lock(each other tensor arg, READ);
//                 launch; release(args, event); release(result, event)
// and after every cluster a barrier over the events of its launches
// (GraphCompiler.cpp:84-108; utils/dialects/lib/Passes/BarrierLegalizerPass.cpp:33-50).
int polar_harness_run(polar_harness* h) {
  if (h == nullptr) return -1;
  GraphHandle gh;
  gh.allocator = h->allocator;
  gh.devices.push_back(h->device);
  gh.devices.push_back(h->host); // host device goes last (ExecutorImpl.cpp:73-75)
  for (auto& cluster : h->clusters)
    for (auto& n : cluster)
      if (n.isInput) {
        gh.mLoaders[n.id] = n.loader.get();
        gh.isHostNode.insert(n.id);
      }

  const uint64_t deferred0 = g_deferredReleases, waited0 = g_eventsWaited;
  using Clock = std::chrono::steady_clock;
  auto since = [](Clock::time_point t0) {
    return static_cast<uint64_t>(
        std::chrono::duration_cast<std::chrono::nanoseconds>(Clock::now() - t0).count());
  };
  for (auto& cluster : h->clusters) {
    std::vector<Event*> events;
    for (auto& n : cluster) {
      Device* dev = ath_device_select(&gh, n.id);
      if (n.isInput) {
        const auto t0 = Clock::now();
        TensorInfo ti = h->find(n.inputVaddr)->info();
        ath_allocate(&gh, *dev, &ti);
        ath_lock(&gh, *dev, &ti, LockType::READ_WRITE);
        ath_load(&gh, n.id, &ti);
        ath_release(&gh, *dev, &ti, nullptr);
        h->counters.ns_input_nodes += since(t0);
        continue;
      }
      auto t0 = Clock::now();
      std::vector<TensorInfo> infos(n.args.size());
      std::vector<ArgDesc> descs(n.args.size());
      std::vector<float> scalars(n.args.size());
      std::vector<int64_t> integers(n.args.size());
      for (size_t i = 0; i < n.args.size(); ++i) {
        if (n.args[i].kind == 0) {
          infos[i] = h->find(n.args[i].vaddr)->info();
          descs[i] = ArgDesc{0, &infos[i], ArgDesc::TENSOR};
        } else if (n.args[i].kind == 2) {
          integers[i] = static_cast<int64_t>(n.args[i].vaddr);
          descs[i] = ArgDesc{sizeof(int64_t), &integers[i], ArgDesc::DATA};
        } else {
          scalars[i] = n.args[i].scalar;
          descs[i] = ArgDesc{sizeof(float), &scalars[i], ArgDesc::DATA};
        }
      }
      const uint64_t resultVaddr = n.args[n.result].vaddr;
      ath_allocate(&gh, *dev, &infos[n.result]);
      ath_lock(&gh, *dev, &infos[n.result], LockType::READ_WRITE);
      std::vector<size_t> readLocked; // each distinct tensor once, never the result
      for (size_t i = 0; i < n.args.size(); ++i) {
        if (n.args[i].kind != 0 || n.args[i].vaddr == resultVaddr) continue;
        bool seen = false;
        for (size_t j : readLocked) seen |= n.args[j].vaddr == n.args[i].vaddr;
        if (seen) continue;
        ath_lock(&gh, *dev, &infos[i], LockType::READ);
        readLocked.push_back(i);
      }
      const std::string jitName =
          n.jitName.empty() ? "node" + std::to_string(n.id) + "_" + n.kernel : n.jitName;
      LaunchCommand cmd{jitName.c_str(), descs.size(), descs.data(), n.kernel.c_str()};
      h->counters.ns_allocate_and_lock += since(t0);
      t0 = Clock::now();
      Event* evt = ath_launch(&gh, dev, nullptr, cmd);
      h->counters.ns_launch += since(t0);
      t0 = Clock::now();
      for (size_t i : readLocked) ath_release(&gh, *dev, &infos[i], evt);
      ath_release(&gh, *dev, &infos[n.result], evt);
      events.push_back(evt);
      h->counters.ns_release += since(t0);
    }
    if (!events.empty()) {
      const auto t0 = Clock::now();
      ath_barrier(static_cast<uint32_t>(events.size()), events.data());
      h->counters.ns_barrier += since(t0);
    }
  }
  h->counters.deferred_releases += g_deferredReleases - deferred0;
  h->counters.events_waited += g_eventsWaited - waited0;
  return 0;
}

// OutputNode access (include/polarai/core/node/internal/OutputNodeInternal.hpp,
// src/backend/generic/lib/allocators/LayerAllocator.cpp:162-186): a READ_WRITE
// lock on the host side pulls the newest copy down.
int polar_harness_read(polar_harness* h, uint64_t vaddr, float* out, uint64_t count) {
  TensorDecl* t = h ? h->find(vaddr) : nullptr;
  if (t == nullptr || out == nullptr) return -1;
  TensorInfo ti = t->info();
  MemoryRecord rec{static_cast<size_t>(vaddr), 4};
  for (uint64_t d : t->shape) rec.allocationSize *= d;
  if (count * 4 > rec.allocationSize) return -1;
  (void)ti;
  h->allocator->lock(rec, LockType::READ_WRITE);
  std::memcpy(out, h->allocator->get(rec), count * 4);
  h->allocator->release(rec);
  return 0;
}

// include/polarai/core/node/OutputNodeAccessor.hpp:21-31
int polar_harness_read_through_tensor_object(polar_harness* h, uint64_t vaddr, float* out,
                                             uint64_t count) {
  TensorDecl* t = h ? h->find(vaddr) : nullptr;
  if (t == nullptr || out == nullptr) return -1;
  HarnessTensor tensor{static_cast<size_t>(vaddr), polarai::core::DataType::FLOAT, 1};
  for (uint64_t d : t->shape) tensor.elements *= d;
  if (count > tensor.elements) return -1;
  polarai::core::internal::TensorAllocator& allocator = *h->allocator;
  allocator.lock(tensor.asTensor(), LockType::READ_WRITE);
  std::memcpy(out, allocator.get(tensor.asTensor()), count * sizeof(float));
  allocator.release(tensor.asTensor());
  return 0;
}

static bool recordOf(polar_harness* h, uint64_t vaddr, MemoryRecord* rec) {
  TensorDecl* t = h ? h->find(vaddr) : nullptr;
  if (t == nullptr) return false;
  rec->virtualAddress = static_cast<size_t>(vaddr);
  rec->allocationSize = 4;
  for (uint64_t d : t->shape) rec->allocationSize *= d;
  return true;
}

int polar_harness_allocate(polar_harness* h, uint64_t vaddr, int device) {
  MemoryRecord rec;
  if (!recordOf(h, vaddr, &rec)) return -1;
  if (device < 0) h->allocator->allocate(rec);
  else h->allocator->allocate(rec, *h->device);
  return 0;
}

int polar_harness_lock(polar_harness* h, uint64_t vaddr, int device, int lock_type) {
  MemoryRecord rec;
  if (!recordOf(h, vaddr, &rec)) return -1;
  const LockType t = lock_type ? LockType::READ_WRITE : LockType::READ;
  if (device < 0) h->allocator->lock(rec, t);
  else h->allocator->lock(rec, *h->device, t);
  return 0;
}

int polar_harness_release(polar_harness* h, uint64_t vaddr, int device) {
  MemoryRecord rec;
  if (!recordOf(h, vaddr, &rec)) return -1;
  if (device < 0) h->allocator->release(rec);
  else h->allocator->release(rec, *h->device);
  return 0;
}

int polar_harness_host_write(polar_harness* h, uint64_t vaddr, const float* data, uint64_t count) {
  MemoryRecord rec;
  if (!recordOf(h, vaddr, &rec) || data == nullptr || count * 4 > rec.allocationSize) return -1;
  h->allocator->allocate(rec);
  h->allocator->lock(rec, LockType::READ_WRITE);
  std::memcpy(h->allocator->get(rec), data, count * 4);
  h->allocator->release(rec);
  return 0;
}

void* polar_harness_raw_device(polar_harness* h) { return h ? h->inner.get() : nullptr; }
void* polar_harness_raw_allocator(polar_harness* h) {
  return h ? static_cast<BackendAllocator*>(h->allocator.get()) : nullptr;
}
void* polar_harness_raw_context(polar_harness* h) { return h ? h->ctx : nullptr; }

int polar_harness_get_counters(polar_harness* h, polar_harness_counters* out) {
  if (h == nullptr || out == nullptr) return -1;
  *out = h->counters;
  return 0;
}

int polar_harness_set_device_byte_limit(polar_harness* h, uint64_t bytes) {
  if (h == nullptr) return -1;
  if (h->mock != nullptr) {
    h->mock->setByteLimit(bytes);
    return 0;
  }
  if (h->setByteLimit == nullptr) return -1;
  return h->setByteLimit(h->inner.get(), bytes);
}

} // extern "C"
