// polar_rt_abi.hpp -- the runtime-plugin interface of the PolarAI/Athena
// generic backend, restated in one header so that libpolar_rt_hip.so can be
// built without the framework's tree and still be loaded by its runtime
// driver.
//
// This is a C++ ABI, not a C one: the driver calls virtual functions on the
// objects a plugin returns and exchanges libstdc++ types with it.  What must
// match the framework's own headers is therefore
//   * the namespace-qualified class names and the ORDER of virtual functions
//     (Itanium vtable slots),
//   * the by-value parameter types (MemoryRecord is two size_t),
//   * the byte layout of the three plain structs the launch lowering fills
//     (TensorInfo, ArgDesc, LaunchCommand) and of GraphHandle.
// Each declaration names the framework header it mirrors (paths relative to
// the framework's tree).  The static_asserts at the end pin the struct
// layouts to the LLVM types the lowering emits.
#pragma once

#include <cstddef>
#include <cstdint>
#include <functional>
#include <map>
#include <memory>
#include <set>
#include <string>
#include <unordered_map>
#include <vector>

// ---- plain structs filled by the launch lowering (global namespace) ---------

// include/polarai/backend/generic/runtime/TensorInfo.h:17-22
// LLVM type {i64, i32, i64, i64*} (utils/dialects/lib/utils/TensorInfo.h:18-28)
struct TensorInfo {
  uint64_t virtAddr; // byte offset in the context's flat space; 0 = no tensor
  int dataType;      // 1 = f64, 2 = f32, 3 = f16 (core/tensor/DataType.hpp:20)
  uint64_t dims;
  uint64_t* shape;
};

// include/polarai/backend/generic/runtime/LaunchCommand.h:19-24
// LLVM type {i64, i8*, i32} (utils/dialects/lib/utils/LaunchCommand.h:18-29)
struct ArgDesc {
  enum ArgType { TENSOR = 0, DATA = 1 };
  uint64_t size; // DATA: byte width of the scalar; TENSOR: unset
  void* arg;     // TENSOR: TensorInfo*; DATA: pointer to the scalar's bytes
  ArgType type;
};

// include/polarai/backend/generic/runtime/LaunchCommand.h:26-31
// LLVM type {i8*, i64, ArgDesc*, i8*} (utils/dialects/lib/utils/LaunchCommand.h:31-43)
struct LaunchCommand {
  const char* kernelName;       // JIT-outlined symbol "<node>_<builtin>"
  uint64_t argsCount;
  ArgDesc* args;
  const char* nativeKernelName; // builtin name: "fadd", "fmatmul_t_f", ...
};

namespace polarai {
namespace core {
// include/polarai/core/tensor/DataType.hpp:20
enum class DataType : int { UNDEFINED = 0, DOUBLE = 1, FLOAT = 2, HALF = 3 };

namespace internal {
class TensorInternal;         // opaque here: only passed by reference
class AbstractLoaderInternal; // opaque here: only stored by pointer

// include/polarai/core/loader/internal/TensorAllocator.hpp:22
enum class LockType { READ, READ_WRITE };

// include/polarai/core/loader/internal/TensorAllocator.hpp:24-45
class TensorAllocator {
public:
  virtual ~TensorAllocator() = default;
  virtual void allocate(const TensorInternal& tensor) = 0;
  virtual void deallocate(const TensorInternal& tensor) = 0;
  virtual void* get(const TensorInternal& tensor) = 0;
  virtual void lock(const TensorInternal& tensor, LockType type) = 0;
  virtual void release(const TensorInternal& tensor) = 0;
};
} // namespace internal
} // namespace core

namespace backend::generic {

// include/polarai/backend/generic/MemoryRecord.hpp:19-34
struct MemoryRecord {
  size_t virtualAddress;
  size_t allocationSize;
  bool operator==(const MemoryRecord& other) const {
    return virtualAddress == other.virtualAddress;
  }
};

// include/polarai/backend/generic/AllocatorLayerBase.hpp:22-40
class AllocatorLayerBase {
public:
  using MemoryOffloadCallbackT =
      std::function<void(MemoryRecord, AllocatorLayerBase& layer)>;

  virtual ~AllocatorLayerBase() = default;
  // Routine the layer calls when it must evict a record to make room.
  virtual void registerMemoryOffloadCallback(MemoryOffloadCallbackT) = 0;
  virtual void allocate(MemoryRecord record) = 0;
  virtual void deallocate(MemoryRecord record) = 0;
  virtual void lock(MemoryRecord record) = 0;
  virtual void release(MemoryRecord record) = 0;
  virtual void* getPtr(MemoryRecord record) = 0;
  virtual bool isAllocated(const MemoryRecord& record) const = 0;
  virtual size_t getTag(MemoryRecord record) = 0;
  virtual void setTag(MemoryRecord record, size_t tag) = 0;
};

// include/polarai/backend/generic/runtime/ProgramDesc.hpp:20-35
struct KernelDesc {
  size_t globalX, globalY, globalZ;
  size_t localX, localY, localZ;
};
struct ProgramDesc {
  // PTX and SPIRV_SHADER are upstream's; HSACO (an AMDGPU code object, or an
  // offload bundle holding one) is the value a HIP code generator would add --
  // this runtime loads programs of that type in selectBinary.
  enum class Type { PTX, SPIRV_SHADER, HSACO };
  Type type;
  std::string target;
  std::vector<char> data;
  std::map<std::string, KernelDesc> kernels;
};

class Device;
class BackendAllocator;

// include/polarai/backend/generic/runtime/Event.hpp:19-25
class Event {
public:
  virtual ~Event() = default;
  virtual void wait() = 0;
  virtual void addCallback(std::function<void()>) = 0;
  virtual auto getDevice() -> Device* = 0;
};

// include/polarai/backend/generic/runtime/Device.hpp:30-32
enum class DeviceProvider { CUDA, HIP, SYCL, OpenCL, VULKAN, METAL, HOST };
enum class DeviceKind { CPU, GPU, FPGA, OTHER_ACCELERATOR, HOST };

// include/polarai/backend/generic/runtime/Device.hpp:34-63
class Device {
public:
  Device() = default;
  virtual ~Device() = default;

  enum class PartitionDomain { EQUALLY, BY_COUNT, NUMA };

  virtual DeviceProvider getProvider() const = 0;
  virtual DeviceKind getKind() const = 0;
  virtual std::string getDeviceName() const = 0;
  virtual bool isPartitionSupported(PartitionDomain) { return false; }
  virtual bool hasAllocator() { return false; }
  virtual std::vector<std::shared_ptr<Device>> partition(PartitionDomain) = 0;
  virtual std::shared_ptr<AllocatorLayerBase> getAllocator() = 0;

  virtual bool operator==(const Device&) const { return false; }
  bool operator!=(const Device& other) const { return !(*this == other); }

  virtual void copyToHost(MemoryRecord record, void* dest) const = 0;
  virtual void copyToDevice(MemoryRecord record, void* src) const = 0;

  virtual Event* launch(BackendAllocator&, LaunchCommand&, Event*) = 0;
  virtual void consumeEvent(Event*) = 0;
  virtual void selectBinary(std::vector<std::shared_ptr<ProgramDesc>>&) = 0;
};

// include/polarai/backend/generic/runtime/Context.hpp:20-24
class Context {
public:
  virtual ~Context() = default;
  virtual std::vector<std::shared_ptr<Device>>& getDevices() = 0;
};

// include/polarai/backend/generic/BackendAllocator.hpp:22-56
// A plugin only ever calls get<T>(record, device), i.e. the second getImpl.
class BackendAllocator : public core::internal::TensorAllocator {
protected:
  virtual void* getImpl(const core::internal::TensorInternal&, Device&) = 0;
  virtual void* getImpl(const MemoryRecord& record, Device& device) = 0;

public:
  using LockType = core::internal::LockType;
  using TensorInternal = core::internal::TensorInternal;

  virtual void registerDevice(Device& device) = 0;
  virtual void allocate(const TensorInternal&, Device&) = 0;
  virtual void allocate(const MemoryRecord& record, Device& device) = 0;
  virtual void allocate(const MemoryRecord& record) = 0;
  virtual void lock(const TensorInternal&, Device&, LockType) = 0;
  virtual void lock(const MemoryRecord& record, Device& device,
                    LockType type) = 0;
  virtual void lock(const MemoryRecord& record, LockType type) = 0;
  virtual void release(const MemoryRecord& record, Device& device) = 0;
  virtual void release(const MemoryRecord& record) = 0;

  template <typename BufferT>
  BufferT* get(const TensorInternal& tensor, Device& device) {
    return reinterpret_cast<BufferT*>(getImpl(tensor, device));
  }
  template <typename BufferT>
  BufferT* get(const MemoryRecord& record, Device& device) {
    return reinterpret_cast<BufferT*>(getImpl(record, device));
  }
  virtual void* get(const MemoryRecord& record) = 0;

  // the base-class overloads stay visible next to the ones above
  using core::internal::TensorAllocator::allocate;
  using core::internal::TensorAllocator::get;
  using core::internal::TensorAllocator::lock;
  using core::internal::TensorAllocator::release;
};

} // namespace backend::generic
} // namespace polarai

namespace std {
template <> class hash<polarai::backend::generic::MemoryRecord> {
public:
  size_t operator()(const polarai::backend::generic::MemoryRecord& r) const {
    return r.virtualAddress;
  }
};
// include/polarai/backend/generic/runtime/Device.hpp:66-73
template <> class hash<polarai::backend::generic::Device> {
public:
  size_t operator()(const polarai::backend::generic::Device& dev) const {
    return std::hash<std::string>()(dev.getDeviceName());
  }
};
} // namespace std

// include/polarai/backend/generic/runtime/GraphHandle.hpp:31-37
struct GraphHandle {
  std::shared_ptr<polarai::backend::generic::BackendAllocator> allocator;
  std::vector<std::shared_ptr<polarai::backend::generic::Device>> devices;
  std::unordered_map<uint64_t, polarai::core::internal::AbstractLoaderInternal*>
      mLoaders;
  std::set<uint64_t> isHostNode;
};

// include/polarai/backend/generic/runtime/api.h:17-20 -- the two symbols the
// runtime driver resolves with dlsym
// (src/backend/generic/runtime/driver/RuntimeDriver.cpp:28-31).
extern "C" {
polarai::backend::generic::Context* initContext();
void closeContext(polarai::backend::generic::Context*);
}

// Layouts the lowering depends on (x86-64, LP64).
static_assert(sizeof(TensorInfo) == 32 && offsetof(TensorInfo, dataType) == 8 &&
                  offsetof(TensorInfo, dims) == 16 &&
                  offsetof(TensorInfo, shape) == 24,
              "TensorInfo must be {i64,i32,i64,i64*}");
static_assert(sizeof(ArgDesc) == 24 && offsetof(ArgDesc, arg) == 8 &&
                  offsetof(ArgDesc, type) == 16,
              "ArgDesc must be {i64,i8*,i32}");
static_assert(sizeof(LaunchCommand) == 32 &&
                  offsetof(LaunchCommand, argsCount) == 8 &&
                  offsetof(LaunchCommand, args) == 16 &&
                  offsetof(LaunchCommand, nativeKernelName) == 24,
              "LaunchCommand must be {i8*,i64,ArgDesc*,i8*}");
static_assert(sizeof(polarai::backend::generic::MemoryRecord) == 16,
              "MemoryRecord is two size_t, passed in registers");
