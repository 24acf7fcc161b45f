// Device handle, memory pool, host<->device copies and events of the device
// library (the non-kernel half of include/polar_hip.h).
#include "internal.h"

#include <chrono>
#include <cstdio>
#include <cstring>

#include <immintrin.h>

namespace {
thread_local char g_lastError[512] = "";

uint64_t roundBlock(uint64_t bytes) {
  // Small blocks: powers of two from 256 B.  Large blocks: multiples of 2 MiB,
  // so that tensors of nearly equal size share cached blocks.
  if (bytes <= 256) return 256;
  if (bytes <= (1ull << 20)) {
    uint64_t r = 256;
    while (r < bytes) r <<= 1;
    return r;
  }
  const uint64_t g = 2ull << 20;
  return (bytes + g - 1) / g * g;
}
} // namespace

namespace polar_hip_detail {
int fail(polar_hip_status st, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_lastError, sizeof(g_lastError), fmt, ap);
  va_end(ap);
  return static_cast<int>(st);
}
int failHip(hipError_t e, const char* what) {
  polar_hip_status st = e == hipErrorOutOfMemory ? POLAR_HIP_ERR_OOM
                        : e == hipErrorNoDevice  ? POLAR_HIP_ERR_NO_DEVICE
                                                 : POLAR_HIP_ERR_RUNTIME;
  return fail(st, "%s failed: %s (%d)", what, hipGetErrorString(e),
              static_cast<int>(e));
}

// ---- workspace ----------------------------------------------------------------

int workspaceFor(polar_hip_device* dev, uint64_t bytes, void** area) {
  if (bytes > kWorkspaceBytes)
    return fail(POLAR_HIP_ERR_INVALID, "workspace request of %llu bytes exceeds the %llu the device holds",
                static_cast<unsigned long long>(bytes), static_cast<unsigned long long>(kWorkspaceBytes));
  *area = dev->workspace;
  return POLAR_HIP_OK;
}

} // namespace polar_hip_detail

using namespace polar_hip_detail;

extern "C" {

const char* polar_hip_last_error(void) { return g_lastError; }
const char* polar_hip_version(void) { return "polar_hip 0.1 (gfx950)"; }

int polar_hip_device_count(int* count) {
  POLAR_HIP_REQUIRE(count != nullptr, "count is null");
  *count = 0;
  int n = 0;
  hipError_t e = hipGetDeviceCount(&n);
  if (e == hipErrorNoDevice) {
    (void)hipGetLastError();
    return POLAR_HIP_OK;
  }
  if (e != hipSuccess) return failHip(e, "hipGetDeviceCount");
  *count = n;
  return POLAR_HIP_OK;
}

int polar_hip_device_open(int ordinal, polar_hip_device** out) {
  POLAR_HIP_REQUIRE(out != nullptr, "out is null");
  *out = nullptr;
  int n = 0;
  int st = polar_hip_device_count(&n);
  if (st) return st;
  if (ordinal < 0 || ordinal >= n)
    return fail(POLAR_HIP_ERR_NO_DEVICE, "device ordinal %d of %d", ordinal, n);
  POLAR_HIP_TRY(hipSetDevice(ordinal));
  hipDeviceProp_t p;
  POLAR_HIP_TRY(hipGetDeviceProperties(&p, ordinal));
  if (strncmp(p.gcnArchName, "gfx950", 6) != 0)
    return fail(POLAR_HIP_ERR_NO_DEVICE,
                "device %d is %s; this library holds gfx950 code only", ordinal,
                p.gcnArchName);
  auto* d = new polar_hip_device();
  d->ordinal = ordinal;
  hipError_t e = hipStreamCreateWithFlags(&d->stream, hipStreamNonBlocking);
  if (e != hipSuccess) {
    delete d;
    return failHip(e, "hipStreamCreateWithFlags");
  }
  snprintf(d->info.name, sizeof(d->info.name), "%s", p.name);
  snprintf(d->info.arch, sizeof(d->info.arch), "%s", p.gcnArchName);
  d->info.ordinal = ordinal;
  d->info.compute_units = p.multiProcessorCount;
  d->info.clock_khz = p.clockRate;
  d->info.memory_clock_khz = p.memoryClockRate;
  d->info.memory_bus_bits = p.memoryBusWidth;
  d->info.lds_bytes_per_block = static_cast<int>(p.sharedMemPerBlock);
  d->info.l2_bytes = p.l2CacheSize;
  d->info.pci_bus_id = p.pciBusID;
  d->info.hbm_bytes = p.totalGlobalMem;
  st = resolveStaticScratch(d);
  if (st == POLAR_HIP_OK) {
    e = hipMalloc(&d->workspace, polar_hip_detail::kWorkspaceBytes);
    if (e != hipSuccess) st = failHip(e, "hipMalloc (workspace)");
  }
  if (st != POLAR_HIP_OK) {
    (void)hipStreamDestroy(d->stream);
    delete d;
    return st;
  }
  *out = d;
  return POLAR_HIP_OK;
}

int polar_hip_device_close(polar_hip_device* dev) {
  POLAR_HIP_REQUIRE(dev != nullptr, "dev is null");
  POLAR_HIP_TRY(hipSetDevice(dev->ordinal));
  POLAR_HIP_TRY(hipStreamSynchronize(dev->stream));
  for (auto& kv : dev->cached)
    for (void* p : kv.second) (void)hipFree(p);
  for (auto& kv : dev->live) (void)hipFree(kv.first);
  if (dev->workspace) (void)hipFree(dev->workspace);
  for (auto* e : dev->allEvents) {
    (void)hipEventDestroy(e->ev);
    delete e;
  }
  if (dev->staging) {
    for (hipEvent_t e : dev->slotEvent) (void)hipEventDestroy(e);
    (void)hipHostFree(dev->staging);
  }
  (void)hipStreamDestroy(dev->stream);
  delete dev;
  return POLAR_HIP_OK;
}

int polar_hip_device_get_info(polar_hip_device* dev,
                              polar_hip_device_info* out) {
  POLAR_HIP_REQUIRE(dev != nullptr && out != nullptr, "null argument");
  *out = dev->info;
  return POLAR_HIP_OK;
}

int polar_hip_device_synchronize(polar_hip_device* dev) {
  POLAR_HIP_REQUIRE(dev != nullptr, "dev is null");
  POLAR_HIP_TRY(hipStreamSynchronize(dev->stream));
  return POLAR_HIP_OK;
}

// ---- pool -------------------------------------------------------------------

static void dropCachedLocked(polar_hip_device* dev) {
  for (auto& kv : dev->cached)
    for (void* p : kv.second) (void)hipFree(p);
  dev->cached.clear();
  dev->stats.bytes_cached = 0;
}

int polar_hip_alloc(polar_hip_device* dev, uint64_t bytes, void** ptr) {
  POLAR_HIP_REQUIRE(dev != nullptr && ptr != nullptr, "null argument");
  *ptr = nullptr;
  const uint64_t sz = roundBlock(bytes);
  std::lock_guard<std::mutex> g(dev->mu);
  auto it = dev->cached.find(sz);
  if (it != dev->cached.end() && !it->second.empty()) {
    void* p = it->second.back();
    it->second.pop_back();
    dev->stats.bytes_cached -= sz;
    dev->stats.bytes_in_use += sz;
    dev->stats.pool_hits++;
    dev->live.emplace(p, sz);
    *ptr = p;
    return POLAR_HIP_OK;
  }
  POLAR_HIP_TRY(hipSetDevice(dev->ordinal));
  void* p = nullptr;
  hipError_t e = hipMalloc(&p, sz);
  if (e == hipErrorOutOfMemory) {
    // Give cached blocks back to the driver and try once more.  Work that
    // still reads them may be in flight, so drain the stream first.
    (void)hipGetLastError();
    (void)hipStreamSynchronize(dev->stream);
    dropCachedLocked(dev);
    e = hipMalloc(&p, sz);
  }
  if (e != hipSuccess) {
    (void)hipGetLastError();
    return failHip(e, "hipMalloc");
  }
  dev->stats.device_allocs++;
  dev->stats.bytes_in_use += sz;
  dev->live.emplace(p, sz);
  *ptr = p;
  return POLAR_HIP_OK;
}

int polar_hip_free(polar_hip_device* dev, void* ptr) {
  POLAR_HIP_REQUIRE(dev != nullptr, "dev is null");
  if (ptr == nullptr) return POLAR_HIP_OK;
  std::lock_guard<std::mutex> g(dev->mu);
  auto it = dev->live.find(ptr);
  if (it == dev->live.end())
    return fail(POLAR_HIP_ERR_INVALID, "polar_hip_free: %p is not a live block",
                ptr);
  const uint64_t sz = it->second;
  dev->live.erase(it);
  dev->cached[sz].push_back(ptr);
  dev->stats.bytes_in_use -= sz;
  dev->stats.bytes_cached += sz;
  return POLAR_HIP_OK;
}

int polar_hip_pool_trim(polar_hip_device* dev) {
  POLAR_HIP_REQUIRE(dev != nullptr, "dev is null");
  POLAR_HIP_TRY(hipSetDevice(dev->ordinal));
  POLAR_HIP_TRY(hipStreamSynchronize(dev->stream));
  std::lock_guard<std::mutex> g(dev->mu);
  dropCachedLocked(dev);
  return POLAR_HIP_OK;
}

int polar_hip_pool_get_stats(polar_hip_device* dev, polar_hip_pool_stats* out) {
  POLAR_HIP_REQUIRE(dev != nullptr && out != nullptr, "null argument");
  std::lock_guard<std::mutex> g(dev->mu);
  *out = dev->stats;
  return POLAR_HIP_OK;
}

// ---- copies -----------------------------------------------------------------
// Host memory handed in by the framework is pageable.  The driver's pageable
// path is fast for large transfers (30 GB/s up, 18 GB/s down, measured) but has
// a high fixed cost for small and medium ones (110 us for 256 KiB), which is
// what graph inputs and read-backs mostly are.  Uploads of up to 4 MiB and all
// downloads go through a ring of pinned 512 KiB slots instead:
//  * upload: the source is copied into a slot and the DMA is enqueued on the
//    device's stream; the call returns without waiting for it (the caller's
//    buffer is already free, and everything that uses the destination is
//    ordered after the DMA on the same stream).  A slot is reused only after
//    the event recorded behind its DMA has completed.
//  * download: up to eight chunk DMAs are kept in flight and each chunk is
//    copied out as soon as its event completes, so the host copy of one chunk
//    overlaps the DMA of the next ones.
namespace {
constexpr uint64_t kSlotBytes = 512ull << 10;
constexpr int kSlots = 8;
constexpr uint64_t kStagingBytes = kSlotBytes * kSlots;

// called with dev->stagingMu held
bool stagingReady(polar_hip_device* dev) {
  if (dev->staging != nullptr) return true;
  void* p = nullptr;
  if (hipHostMalloc(&p, kStagingBytes, hipHostMallocDefault) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  for (int i = 0; i < kSlots; ++i) {
    if (hipEventCreateWithFlags(&dev->slotEvent[i], hipEventDisableTiming) != hipSuccess) {
      (void)hipGetLastError();
      for (int k = 0; k < i; ++k) (void)hipEventDestroy(dev->slotEvent[k]);
      (void)hipHostFree(p);
      return false;
    }
    dev->slotBusy[i] = false;
  }
  dev->staging = p;
  return true;
}

// next slot of the ring, idle (its previous transfer has completed)
hipError_t acquireSlot(polar_hip_device* dev, int* slot) {
  const int s = dev->nextSlot;
  dev->nextSlot = (s + 1) % kSlots;
  if (dev->slotBusy[s]) {
    hipError_t e = hipEventSynchronize(dev->slotEvent[s]);
    if (e != hipSuccess) return e;
    dev->slotBusy[s] = false;
  }
  *slot = s;
  return hipSuccess;
}

char* slotMemory(polar_hip_device* dev, int slot) {
  return static_cast<char*>(dev->staging) + uint64_t(slot) * kSlotBytes;
}

// Host copy out of a staging slot into the caller's memory with streaming
// stores: the destination is written once and not read back by this code, and
// a regular store would first fetch every destination line into the cache
// (twice the memory traffic; the C library's memcpy only switches to streaming
// stores for copies much larger than a slot).
__attribute__((target("avx2"))) void streamCopyAvx2(char* dst, const char* src, size_t n) {
  size_t head = (32 - (reinterpret_cast<uintptr_t>(dst) & 31)) & 31;
  if (head > n) head = n;
  memcpy(dst, src, head);
  dst += head;
  src += head;
  n -= head;
  const size_t body = n & ~size_t(127);
  for (size_t i = 0; i < body; i += 128) {
    const __m256i a = _mm256_loadu_si256(reinterpret_cast<const __m256i*>(src + i));
    const __m256i b = _mm256_loadu_si256(reinterpret_cast<const __m256i*>(src + i + 32));
    const __m256i c = _mm256_loadu_si256(reinterpret_cast<const __m256i*>(src + i + 64));
    const __m256i d = _mm256_loadu_si256(reinterpret_cast<const __m256i*>(src + i + 96));
    _mm256_stream_si256(reinterpret_cast<__m256i*>(dst + i), a);
    _mm256_stream_si256(reinterpret_cast<__m256i*>(dst + i + 32), b);
    _mm256_stream_si256(reinterpret_cast<__m256i*>(dst + i + 64), c);
    _mm256_stream_si256(reinterpret_cast<__m256i*>(dst + i + 96), d);
  }
  _mm_sfence();
  memcpy(dst + body, src + body, n - body);
}

void copyOutOfSlot(void* dst, const void* src, size_t n) {
  static const bool avx2 = __builtin_cpu_supports("avx2");
  if (avx2 && n >= (64u << 10))
    streamCopyAvx2(static_cast<char*>(dst), static_cast<const char*>(src), n);
  else
    memcpy(dst, src, n);
}
} // namespace

int polar_hip_copy_to_device(polar_hip_device* dev, void* dst_device,
                             const void* src_host, uint64_t bytes) {
  POLAR_HIP_REQUIRE(dev != nullptr, "dev is null");
  if (bytes == 0) return POLAR_HIP_OK;
  POLAR_HIP_REQUIRE(dst_device != nullptr && src_host != nullptr,
                    "null buffer");
  POLAR_HIP_TRY(hipSetDevice(dev->ordinal));
  if (bytes <= kStagingBytes) {
    std::lock_guard<std::mutex> g(dev->stagingMu);
    if (stagingReady(dev)) {
      for (uint64_t off = 0; off < bytes; off += kSlotBytes) {
        const uint64_t n = bytes - off < kSlotBytes ? bytes - off : kSlotBytes;
        int slot;
        POLAR_HIP_TRY(acquireSlot(dev, &slot));
        memcpy(slotMemory(dev, slot), static_cast<const char*>(src_host) + off, n);
        POLAR_HIP_TRY(hipMemcpyAsync(static_cast<char*>(dst_device) + off, slotMemory(dev, slot),
                                     n, hipMemcpyHostToDevice, dev->stream));
        POLAR_HIP_TRY(hipEventRecord(dev->slotEvent[slot], dev->stream));
        dev->slotBusy[slot] = true;
      }
      return POLAR_HIP_OK;
    }
  }
  POLAR_HIP_TRY(hipMemcpyAsync(dst_device, src_host, bytes,
                               hipMemcpyHostToDevice, dev->stream));
  POLAR_HIP_TRY(hipStreamSynchronize(dev->stream));
  return POLAR_HIP_OK;
}

int polar_hip_copy_to_host(polar_hip_device* dev, void* dst_host,
                           const void* src_device, uint64_t bytes) {
  POLAR_HIP_REQUIRE(dev != nullptr, "dev is null");
  if (bytes == 0) return POLAR_HIP_OK;
  POLAR_HIP_REQUIRE(dst_host != nullptr && src_device != nullptr,
                    "null buffer");
  POLAR_HIP_TRY(hipSetDevice(dev->ordinal));
  {
    // Any size: at most kSlots chunk DMAs are in flight; a chunk is copied out
    // as soon as its event completes and its slot goes to the chunk kSlots
    // further on.
    std::lock_guard<std::mutex> g(dev->stagingMu);
    if (stagingReady(dev)) {
      int slots[kSlots];
      const uint64_t chunks = (bytes + kSlotBytes - 1) / kSlotBytes;
      auto consume = [&](uint64_t c) -> hipError_t {
        const uint64_t off = c * kSlotBytes;
        const uint64_t n = bytes - off < kSlotBytes ? bytes - off : kSlotBytes;
        const int slot = slots[c % kSlots];
        hipError_t e = hipEventSynchronize(dev->slotEvent[slot]);
        if (e != hipSuccess) return e;
        dev->slotBusy[slot] = false;
        copyOutOfSlot(static_cast<char*>(dst_host) + off, slotMemory(dev, slot), n);
        return hipSuccess;
      };
      for (uint64_t c = 0; c < chunks; ++c) {
        if (c >= kSlots) POLAR_HIP_TRY(consume(c - kSlots));
        const uint64_t off = c * kSlotBytes;
        const uint64_t n = bytes - off < kSlotBytes ? bytes - off : kSlotBytes;
        int slot;
        POLAR_HIP_TRY(acquireSlot(dev, &slot));
        slots[c % kSlots] = slot;
        POLAR_HIP_TRY(hipMemcpyAsync(slotMemory(dev, slot),
                                     static_cast<const char*>(src_device) + off, n,
                                     hipMemcpyDeviceToHost, dev->stream));
        POLAR_HIP_TRY(hipEventRecord(dev->slotEvent[slot], dev->stream));
        dev->slotBusy[slot] = true;
      }
      for (uint64_t c = chunks > kSlots ? chunks - kSlots : 0; c < chunks; ++c)
        POLAR_HIP_TRY(consume(c));
      return POLAR_HIP_OK;
    }
  }
  POLAR_HIP_TRY(hipMemcpyAsync(dst_host, src_device, bytes,
                               hipMemcpyDeviceToHost, dev->stream));
  POLAR_HIP_TRY(hipStreamSynchronize(dev->stream));
  return POLAR_HIP_OK;
}

// ---- events -----------------------------------------------------------------

int polar_hip_event_record(polar_hip_device* dev, polar_hip_event** out) {
  POLAR_HIP_REQUIRE(dev != nullptr && out != nullptr, "null argument");
  *out = nullptr;
  polar_hip_event* e = nullptr;
  {
    std::lock_guard<std::mutex> g(dev->mu);
    if (!dev->idleEvents.empty()) {
      e = dev->idleEvents.back();
      dev->idleEvents.pop_back();
    }
  }
  if (e == nullptr) {
    POLAR_HIP_TRY(hipSetDevice(dev->ordinal));
    hipEvent_t he;
    POLAR_HIP_TRY(hipEventCreate(&he));
    e = new polar_hip_event{dev, he};
    std::lock_guard<std::mutex> g(dev->mu);
    dev->allEvents.push_back(e);
  }
  hipError_t err = hipEventRecord(e->ev, dev->stream);
  if (err != hipSuccess) {
    std::lock_guard<std::mutex> g(dev->mu);
    dev->idleEvents.push_back(e);
    return failHip(err, "hipEventRecord");
  }
  *out = e;
  return POLAR_HIP_OK;
}

// Graph code waits on an event after every cluster, typically for a kernel that
// runs for microseconds, so the wake-up latency of a blocking wait is paid once
// per node.  Poll for a short while first and only then block.
int polar_hip_event_synchronize(polar_hip_event* evt) {
  POLAR_HIP_REQUIRE(evt != nullptr, "evt is null");
  const auto t0 = std::chrono::steady_clock::now();
  for (;;) {
    hipError_t e = hipEventQuery(evt->ev);
    if (e == hipSuccess) return POLAR_HIP_OK;
    if (e != hipErrorNotReady) return failHip(e, "hipEventQuery");
    (void)hipGetLastError();
    if (std::chrono::steady_clock::now() - t0 > std::chrono::microseconds(200)) break;
  }
  POLAR_HIP_TRY(hipEventSynchronize(evt->ev));
  return POLAR_HIP_OK;
}

int polar_hip_event_query(polar_hip_event* evt, int* done) {
  POLAR_HIP_REQUIRE(evt != nullptr && done != nullptr, "null argument");
  hipError_t e = hipEventQuery(evt->ev);
  if (e == hipSuccess) {
    *done = 1;
  } else if (e == hipErrorNotReady) {
    (void)hipGetLastError();
    *done = 0;
  } else {
    return failHip(e, "hipEventQuery");
  }
  return POLAR_HIP_OK;
}

int polar_hip_stream_wait_event(polar_hip_device* dev, polar_hip_event* evt) {
  POLAR_HIP_REQUIRE(dev != nullptr && evt != nullptr, "null argument");
  POLAR_HIP_TRY(hipSetDevice(dev->ordinal));
  POLAR_HIP_TRY(hipStreamWaitEvent(dev->stream, evt->ev, 0));
  return POLAR_HIP_OK;
}

int polar_hip_event_elapsed_ms(polar_hip_event* start, polar_hip_event* stop,
                               float* ms) {
  POLAR_HIP_REQUIRE(start && stop && ms, "null argument");
  POLAR_HIP_TRY(hipEventElapsedTime(ms, start->ev, stop->ev));
  return POLAR_HIP_OK;
}

// Arms a start/stop pair for the next kernel launched on `dev`.
int polar_hip_time_next_kernel(polar_hip_device* dev, polar_hip_event** start,
                               polar_hip_event** stop) {
  POLAR_HIP_REQUIRE(dev && start && stop, "null argument");
  *start = *stop = nullptr;
  polar_hip_event* pair[2] = {nullptr, nullptr};
  POLAR_HIP_TRY(hipSetDevice(dev->ordinal));
  for (auto*& e : pair) {
    {
      std::lock_guard<std::mutex> g(dev->mu);
      if (!dev->idleEvents.empty()) {
        e = dev->idleEvents.back();
        dev->idleEvents.pop_back();
      }
    }
    if (e == nullptr) {
      hipEvent_t he;
      POLAR_HIP_TRY(hipEventCreate(&he));
      e = new polar_hip_event{dev, he};
      std::lock_guard<std::mutex> g(dev->mu);
      dev->allEvents.push_back(e);
    }
  }
  dev->timeStart = *start = pair[0];
  dev->timeStop = *stop = pair[1];
  return POLAR_HIP_OK;
}

int polar_hip_event_release(polar_hip_event* evt) {
  POLAR_HIP_REQUIRE(evt != nullptr, "evt is null");
  std::lock_guard<std::mutex> g(evt->dev->mu);
  evt->dev->idleEvents.push_back(evt);
  return POLAR_HIP_OK;
}

// ---- code objects -------------------------------------------------------------

int polar_hip_module_load(polar_hip_device* dev, const void* image, uint64_t bytes,
                          polar_hip_module** out) {
  POLAR_HIP_REQUIRE(dev && image && out, "null argument");
  POLAR_HIP_REQUIRE(bytes >= 4, "code object is empty");
  *out = nullptr;
  POLAR_HIP_TRY(hipSetDevice(dev->ordinal));
  // the loader parses the image in place: keep a copy alive with the module
  auto m = std::make_unique<polar_hip_module>();
  m->dev = dev;
  m->image.assign(static_cast<const char*>(image), static_cast<const char*>(image) + bytes);
  POLAR_HIP_TRY(hipModuleLoadData(&m->module, m->image.data()));
  *out = m.release();
  return POLAR_HIP_OK;
}

int polar_hip_module_unload(polar_hip_device* dev, polar_hip_module* module) {
  POLAR_HIP_REQUIRE(dev && module && module->dev == dev, "module does not belong to this device");
  POLAR_HIP_TRY(hipSetDevice(dev->ordinal));
  POLAR_HIP_TRY(hipStreamSynchronize(dev->stream)); // its kernels may still run
  hipError_t e = hipModuleUnload(module->module);
  delete module;
  if (e != hipSuccess) return failHip(e, "hipModuleUnload");
  return POLAR_HIP_OK;
}

static hipFunction_t findKernel(polar_hip_module* module, const char* name) {
  std::lock_guard<std::mutex> g(module->mu);
  auto it = module->functions.find(name);
  if (it != module->functions.end()) return it->second;
  hipFunction_t fn = nullptr;
  if (hipModuleGetFunction(&fn, module->module, name) != hipSuccess) {
    (void)hipGetLastError(); // a missing name is an answer, not a sticky error
    fn = nullptr;
  }
  module->functions.emplace(name, fn);
  return fn;
}

int polar_hip_module_has_kernel(polar_hip_module* module, const char* name, int* found) {
  POLAR_HIP_REQUIRE(module && name && found, "null argument");
  POLAR_HIP_TRY(hipSetDevice(module->dev->ordinal));
  *found = findKernel(module, name) != nullptr;
  return POLAR_HIP_OK;
}

int polar_hip_module_launch(polar_hip_device* dev, polar_hip_module* module, const char* name,
                            const uint32_t grid[3], const uint32_t block[3], void** params) {
  POLAR_HIP_REQUIRE(dev && module && name && grid && block, "null argument");
  POLAR_HIP_REQUIRE(module->dev == dev, "module does not belong to this device");
  POLAR_HIP_REQUIRE(grid[0] >= 1 && grid[1] >= 1 && grid[2] >= 1 && block[0] >= 1 &&
                        block[1] >= 1 && block[2] >= 1,
                    "empty launch geometry");
  POLAR_HIP_REQUIRE(uint64_t(block[0]) * block[1] * block[2] <= 1024,
                    "more than 1024 lanes per work-group");
  POLAR_HIP_TRY(hipSetDevice(dev->ordinal));
  hipFunction_t fn = findKernel(module, name);
  if (fn == nullptr)
    return fail(POLAR_HIP_ERR_INVALID, "polar_hip_module_launch: no kernel '%s' in the module", name);
  POLAR_HIP_TRY(hipModuleLaunchKernel(fn, grid[0], grid[1], grid[2], block[0], block[1], block[2],
                                      0, dev->stream, params, nullptr));
  return POLAR_HIP_OK;
}

} // extern "C"
