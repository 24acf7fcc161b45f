// lspolar_hip -- lists the devices a runtime plugin reports, the way the
// framework's `lspolar` utility does for every runtime it finds
// (utils/lspolar/main.cpp:55-82 on top of RuntimeDriver,
//  src/backend/generic/runtime/driver/RuntimeDriver.cpp:12-41): the plugin is
// opened with dlopen(RTLD_LAZY | RTLD_LOCAL), initContext / closeContext are
// looked up with dlsym, and every device is asked through its vtable.
//
// usage: lspolar_hip [path-of-plugin]   (default: libpolar_rt_hip.so next to
// this program).  Exit status 0 if the plugin loaded, 1 otherwise.  Output is
// the reference tool's: one block per device with the same labels.
#include "polar_rt_abi.hpp"

#include <dlfcn.h>
#include <unistd.h>

#include <climits>
#include <cstdio>
#include <string>

using namespace polarai::backend::generic;

namespace {
const char* providerName(DeviceProvider p) {
  switch (p) {
  case DeviceProvider::CUDA: return "CUDA";
  case DeviceProvider::HIP: return "HIP";
  case DeviceProvider::SYCL: return "SYCL";
  case DeviceProvider::OpenCL: return "OpenCL";
  case DeviceProvider::VULKAN: return "Vulkan";
  case DeviceProvider::METAL: return "Metal";
  case DeviceProvider::HOST: return "Host";
  }
  return "Unknown";
}

const char* kindName(DeviceKind k) {
  switch (k) {
  case DeviceKind::CPU: return "CPU";
  case DeviceKind::GPU: return "GPU";
  case DeviceKind::FPGA: return "FPGA";
  case DeviceKind::OTHER_ACCELERATOR: return "Other";
  case DeviceKind::HOST: return "Host";
  }
  return "Unknown";
}

std::string defaultPlugin() {
  char self[PATH_MAX];
  const ssize_t n = readlink("/proc/self/exe", self, sizeof(self) - 1);
  if (n <= 0) return "libpolar_rt_hip.so";
  std::string dir(self, static_cast<size_t>(n));
  dir.erase(dir.find_last_of('/') + 1);
  return dir + "libpolar_rt_hip.so";
}
} // namespace

int main(int argc, char** argv) {
  const std::string path = argc > 1 ? argv[1] : defaultPlugin();
  void* lib = dlopen(path.c_str(), RTLD_LAZY | RTLD_LOCAL);
  if (lib == nullptr) {
    std::fprintf(stderr, "Failed to load %s\n%s\n", path.c_str(), dlerror());
    return 1;
  }
  auto init = reinterpret_cast<Context* (*)()>(dlsym(lib, "initContext"));
  auto close = reinterpret_cast<void (*)(Context*)>(dlsym(lib, "closeContext"));
  if (init == nullptr || close == nullptr) {
    std::fprintf(stderr, "%s does not export initContext/closeContext\n", path.c_str());
    return 1;
  }
  Context* context = init();
  {
    auto& devices = context->getDevices();
    std::printf("Total device count: %zu\n\n", devices.size());
    for (const auto& device : devices) {
      std::printf("Name       : %s\n", device->getDeviceName().c_str());
      std::printf("Provider   : %s\n", providerName(device->getProvider()));
      std::printf("Kind       : %s\n", kindName(device->getKind()));
      std::printf("Allocator  : %d\n", device->hasAllocator() ? 1 : 0);
      std::printf("Partition\n");
      std::printf("  Equally  : %d\n", device->isPartitionSupported(Device::PartitionDomain::EQUALLY) ? 1 : 0);
      std::printf("  By count : %d\n", device->isPartitionSupported(Device::PartitionDomain::BY_COUNT) ? 1 : 0);
      std::printf("  NUMA     : %d\n\n", device->isPartitionSupported(Device::PartitionDomain::NUMA) ? 1 : 0);
    }
  }
  close(context);
  dlclose(lib);
  return 0;
}
