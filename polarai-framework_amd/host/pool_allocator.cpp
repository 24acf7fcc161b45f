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

void* PoolBlocks::acquire(size_t bytes) {
  void* p = nullptr;
  const int st = polar_hip_alloc(mDev, bytes, &p);
  if (st == POLAR_HIP_ERR_OOM) return nullptr; // the layer evicts and asks again
  checkStatus(st, "polar_hip_alloc");
  return p;
}

void PoolBlocks::give(void* block) { checkStatus(polar_hip_free(mDev, block), "polar_hip_free"); }

void PoolBlocks::fail(const char* fmt, ...) {
  char message[256];
  va_list ap;
  va_start(ap, fmt);
  std::vsnprintf(message, sizeof(message), fmt, ap);
  va_end(ap);
  fatal("%s", message);
}

} // namespace polarai::backend::generic::mi355x
