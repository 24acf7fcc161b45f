// Device handle, memory pool, host<->device copies and events of the device
// library (the non-kernel half of include/polar_hip.h).
#include "internal.h"

#include <chrono>
#include <cstdio>
#include <cstring>

#include <immintrin.h>

namespace {
thread_local char g_lastError[512] = "";
void drainStop(DrainThread& d); // with the copy code below

// Host blocks the GPU can address (polar_hip_host_alloc) and the open device
// handles their queued transfers refer to.
std::mutex g_hostMu;
std::map<uint64_t, polar_hip_device*> g_openDevices; // by serial
uint64_t g_nextSerial = 1;

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

// The block grows on demand, in powers of two from 4 MiB up to kWorkspaceBytes:
// a handle that never splits a contraction or takes a softmax holds nothing,
// and one that does holds what its largest call so far needed.  Growing waits
// for the stream (kernels may still be using the old block) and allocates, so
// the first call of a new size pays for it once; calls after it neither
// allocate nor wait.
int workspaceFor(polar_hip_device* dev, uint64_t bytes, void** area) {
  if (bytes > kWorkspaceBytes)
    return fail(POLAR_HIP_ERR_INVALID, "workspace request of %llu bytes exceeds the cap of %llu",
                static_cast<unsigned long long>(bytes), static_cast<unsigned long long>(kWorkspaceBytes));
  if (bytes > dev->workspaceBytes) {
    uint64_t size = 4ull << 20;
    while (size < bytes) size *= 2;
    hipError_t e = hipSetDevice(dev->ordinal);
    if (e != hipSuccess) return failHip(e, "hipSetDevice");
    if (dev->workspace != nullptr) {
      e = hipStreamSynchronize(dev->stream);
      if (e != hipSuccess) return failHip(e, "hipStreamSynchronize (workspace)");
      (void)hipFree(dev->workspace);
      dev->workspace = nullptr;
      dev->workspaceBytes = 0;
    }
    e = hipMalloc(&dev->workspace, size);
    if (e != hipSuccess) {
      dev->workspace = nullptr;
      return failHip(e, "hipMalloc (workspace)");
    }
    dev->workspaceBytes = size;
  }
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
    e = hipMalloc(reinterpret_cast<void**>(&d->tileCounters), kTileCounters * sizeof(uint32_t));
    if (e == hipSuccess) e = hipMemset(d->tileCounters, 0, kTileCounters * sizeof(uint32_t));
    if (e != hipSuccess) st = failHip(e, "hipMalloc / hipMemset (tile counters)");
  }
  if (st != POLAR_HIP_OK) {
    if (d->tileCounters) (void)hipFree(d->tileCounters);
    (void)hipStreamDestroy(d->stream);
    delete d;
    return st;
  }
  {
    std::lock_guard<std::mutex> g(g_hostMu);
    d->serial = g_nextSerial++;
    g_openDevices.emplace(d->serial, d);
  }
  *out = d;
  return POLAR_HIP_OK;
}

int polar_hip_device_close(polar_hip_device* dev) {
  POLAR_HIP_REQUIRE(dev != nullptr, "dev is null");
  POLAR_HIP_TRY(hipSetDevice(dev->ordinal));
  POLAR_HIP_TRY(hipStreamSynchronize(dev->stream));
  {
    // every transfer this handle queued out of a host block is complete now;
    // a block that still names the handle finds it gone and takes that as done
    std::lock_guard<std::mutex> g(g_hostMu);
    g_openDevices.erase(dev->serial);
  }
  // a thread that found the handle before it left the table may still be waiting
  // for its stream (waitForBlock, outside the mutex): let it finish
  while (dev->waiters.load() != 0) std::this_thread::yield();
  for (auto& kv : dev->cached)
    for (void* p : kv.second) (void)hipFree(p);
  for (auto& kv : dev->live) (void)hipFree(kv.first);
  if (dev->workspace) (void)hipFree(dev->workspace);
  if (dev->tileCounters) (void)hipFree(dev->tileCounters);
  for (auto* e : dev->allEvents) {
    (void)hipEventDestroy(e->ev);
    delete e;
  }
  drainStop(dev->drain);
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
  const uint64_t queued = dev->directQueued.load();
  POLAR_HIP_TRY(hipStreamSynchronize(dev->stream));
  dev->noteDirectDone(queued);
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
// path has a high fixed cost for small and medium transfers (110 us for 256
// KiB), which is what graph inputs and read-backs mostly are, and reaches 30
// GB/s up and 18 GB/s down on large ones.  All copies go through a ring of
// eight pinned slots instead:
//  * upload: the source is copied into a slot and the DMA is enqueued on the
//    device's stream; the call returns without waiting for it (the caller's
//    buffer is already free, and everything that uses the destination is
//    ordered after the DMA on the same stream).  A slot is reused only after
//    the event recorded behind its DMA has completed.
//  * download: chunk DMAs are kept in flight and each chunk is copied out as
//    soon as its event completes, so the host copy of one chunk overlaps the
//    DMA of the next ones.
//  * transfers below 8 MiB move in 512 KiB chunks (the first DMA starts early);
//    larger ones in 2 MiB chunks (about 10 us of driver calls per chunk
//    otherwise cap the rate) with a second host thread taking every second
//    chunk's host-side copy: 256 MiB read back at 40 GB/s instead of 22.
namespace {
constexpr uint64_t kSlotBytes = 512ull << 10;     // chunk of uploads and of small and medium read-backs
constexpr uint64_t kSlotCapacity = 2ull << 20;    // a slot's memory; large read-backs use all of it
constexpr int kSlots = 8;
constexpr uint64_t kTwoThreadBytes = 8ull << 20;  // copies from this size on use whole slots and the drain thread

// called with dev->stagingMu held
bool stagingReady(polar_hip_device* dev) {
  if (dev->staging != nullptr) return true;
  void* p = nullptr;
  if (hipHostMalloc(&p, kSlotCapacity * kSlots, hipHostMallocDefault) != hipSuccess) {
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
    if (dev->slotEvented[s]) {
      hipError_t e = hipEventSynchronize(dev->slotEvent[s]);
      if (e != hipSuccess) return e;
    } else if (dev->directDone.load() < dev->slotNumber[s]) {
      // a small upload left no event, and nothing the caller has waited for
      // since tells that it is over: wait for what the stream holds now
      const uint64_t queued = dev->directQueued.load();
      hipError_t e = hipEventRecord(dev->slotEvent[s], dev->stream);
      if (e == hipSuccess) e = hipEventSynchronize(dev->slotEvent[s]);
      if (e != hipSuccess) return e;
      dev->noteDirectDone(queued);
    }
    dev->slotBusy[s] = false;
  }
  *slot = s;
  return hipSuccess;
}

char* slotMemory(polar_hip_device* dev, int slot) {
  return static_cast<char*>(dev->staging) + uint64_t(slot) * kSlotCapacity;
}

// Host copy between a staging slot and the caller's memory with streaming
// stores: the destination is written once and not read back by this thread, and
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

void copyOutOfSlot(void* dst, const void* src, size_t n);

// Copy between a staging slot and device memory by the compute units instead of
// the DMA engine: the slot is pinned host memory that the GPU can address, so a
// kernel on the device's own queue moves the bytes across the link.  Work that
// follows on the stream then starts as soon as the kernel retires; behind a
// DMA-engine copy it waits for a signal from another engine, which costs
// 10-15 us per transfer in a graph whose kernels run for 2-10 us.
typedef float upload_v4 __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(256) void slotCopyKernel(const upload_v4* src, upload_v4* dst, uint32_t vectors,
                                                    uint32_t tailBytes) {
  const uint32_t i = blockIdx.x * 256 + threadIdx.x;
  if (i < vectors) __builtin_nontemporal_store(__builtin_nontemporal_load(&src[i]), &dst[i]);
  if (blockIdx.x == 0 && threadIdx.x < tailBytes) {
    const char* s = reinterpret_cast<const char*>(src + vectors);
    char* d = reinterpret_cast<char*>(dst + vectors);
    d[threadIdx.x] = s[threadIdx.x];
  }
}

void drainLoop(DrainThread* d) {
  std::unique_lock<std::mutex> lock(d->mu);
  for (;;) {
    d->cv.wait(lock, [&] { return d->pending || d->quit; });
    if (d->quit) return;
    char* dst = d->dst;
    const char* src = d->src;
    const size_t n = d->bytes;
    lock.unlock();
    copyOutOfSlot(dst, src, n);
    lock.lock();
    d->pending = false;
    d->cv.notify_all();
  }
}
// wait until the drain thread has finished the job it holds, if any
void drainWait(DrainThread& d) {
  std::unique_lock<std::mutex> lock(d.mu);
  d.cv.wait(lock, [&] { return !d.pending; });
}
void drainPost(DrainThread& d, char* dst, const char* src, size_t n) {
  std::unique_lock<std::mutex> lock(d.mu);
  d.cv.wait(lock, [&] { return !d.pending; });
  if (!d.thread.joinable()) d.thread = std::thread(drainLoop, &d);
  d.dst = dst;
  d.src = src;
  d.bytes = n;
  d.pending = true;
  d.cv.notify_all();
}
void drainStop(DrainThread& d) {
  {
    std::unique_lock<std::mutex> lock(d.mu);
    d.cv.wait(lock, [&] { return !d.pending; });
    d.quit = true;
    d.cv.notify_all();
  }
  if (d.thread.joinable()) d.thread.join();
}

void copyOutOfSlot(void* dst, const void* src, size_t n) {
  static const bool avx2 = __builtin_cpu_supports("avx2");
  if (avx2 && n >= (64u << 10))
    streamCopyAvx2(static_cast<char*>(dst), static_cast<const char*>(src), n);
  else
    memcpy(dst, src, n);
}
} // namespace

// ---- host blocks the GPU can address -----------------------------------------
namespace {
struct HostBlock {
  uint64_t bytes = 0;
  // the latest transfer queued directly out of or into the block: its number on
  // the device handle `serial` (0: none outstanding)
  uint64_t serial = 0, number = 0;
};
std::map<uintptr_t, HostBlock> g_hostBlocks; // by base address; g_hostMu

// the block that holds [p, p + bytes) and its base address, or null; g_hostMu held
HostBlock* hostBlockOf(const void* p, uint64_t bytes, uintptr_t* base = nullptr) {
  const uintptr_t a = reinterpret_cast<uintptr_t>(p);
  auto it = g_hostBlocks.upper_bound(a);
  if (it == g_hostBlocks.begin()) return nullptr;
  --it;
  if (a + bytes > it->first + it->second.bytes) return nullptr;
  if (base != nullptr) *base = it->first;
  return &it->second;
}

// Returns once every transfer that was queued on the block at `base` when the
// call began is complete.  Usually that is already known: the caller has waited
// for an event recorded behind the transfer (every launch of a graph is followed
// by one), and the device handle has noted how far its stream had got.
// Otherwise the whole stream is waited for.  No event per transfer: a recorded
// event puts a marker packet between the kernels, and waiting for an idle
// stream costs tens of microseconds.
// `lock` holds g_hostMu on entry and on return, but NOT while the stream is
// waited for: the mutex is process-wide (every copy on every device takes it to
// look its buffer up), and a stream may be milliseconds long.  The block may
// have been freed or used again in between, so the caller looks it up afresh;
// the device handle is kept open by its count of waiters (polar_hip_device_close).
hipError_t waitForBlock(std::unique_lock<std::mutex>& lock, uintptr_t base) {
  for (;;) {
    auto bi = g_hostBlocks.find(base);
    if (bi == g_hostBlocks.end() || bi->second.number == 0) return hipSuccess;
    const uint64_t number = bi->second.number, serial = bi->second.serial;
    auto it = g_openDevices.find(serial);
    if (it == g_openDevices.end() || it->second->directDone.load() >= number) {
      bi->second.number = 0;
      return hipSuccess;
    }
    polar_hip_device* dev = it->second;
    const uint64_t queued = dev->directQueued.load();
    dev->waiters.fetch_add(1);
    lock.unlock();
    const hipError_t e = hipStreamSynchronize(dev->stream);
    if (e == hipSuccess) dev->noteDirectDone(queued);
    dev->waiters.fetch_sub(1);
    lock.lock();
    if (e != hipSuccess) return e;
    // look again: the note may be gone, or name a later transfer of another thread
    bi = g_hostBlocks.find(base);
    if (bi == g_hostBlocks.end()) return hipSuccess;
    if (bi->second.number == number && bi->second.serial == serial) {
      bi->second.number = 0;
      return hipSuccess;
    }
    if (bi->second.serial == serial) return hipSuccess;  // a later transfer on the stream we drained: not ours to wait for
  }
}

// Queue a transfer between a host block and device memory on dev's stream and
// note it on the block.  g_hostMu held.
hipError_t queueDirect(std::unique_lock<std::mutex>& lock, polar_hip_device* dev, uintptr_t base, void* dst,
                       const void* src, uint64_t bytes, hipMemcpyKind kind, uint64_t* number = nullptr) {
  // another handle's transfer on the block first: one note per block
  {
    auto bi = g_hostBlocks.find(base);
    if (bi != g_hostBlocks.end() && bi->second.number != 0 && bi->second.serial != dev->serial) {
      const hipError_t w = waitForBlock(lock, base);
      if (w != hipSuccess) return w;
    }
  }
  auto found = g_hostBlocks.find(base);
  if (found == g_hostBlocks.end()) return hipErrorInvalidValue;  // freed by another thread while we waited
  HostBlock& b = found->second;
  hipError_t e;
  if (bytes < kTwoThreadBytes && ((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src)) & 15u) == 0) {
    const uint32_t vectors = static_cast<uint32_t>(bytes / 16), tail = static_cast<uint32_t>(bytes % 16);
    hipLaunchKernelGGL(slotCopyKernel, dim3(vectors / 256 + 1), dim3(256), 0, dev->stream,
                       static_cast<const upload_v4*>(src), static_cast<upload_v4*>(dst), vectors, tail);
    e = hipGetLastError();
  } else {
    e = hipMemcpyAsync(dst, src, bytes, kind, dev->stream);
  }
  if (e != hipSuccess) return e;
  b.serial = dev->serial;
  b.number = dev->directQueued.fetch_add(1) + 1; // after the launch: an event stamped with it is behind the transfer
  if (number != nullptr) *number = b.number;
  return hipSuccess;
}
} // namespace

int polar_hip_host_alloc(polar_hip_device* dev, uint64_t bytes, void** ptr) {
  POLAR_HIP_REQUIRE(dev != nullptr && ptr != nullptr, "null argument");
  *ptr = nullptr;
  POLAR_HIP_TRY(hipSetDevice(dev->ordinal));
  void* p = nullptr;
  POLAR_HIP_TRY(hipHostMalloc(&p, bytes ? bytes : 1, hipHostMallocPortable | hipHostMallocMapped));
  std::lock_guard<std::mutex> g(g_hostMu);
  HostBlock b;
  b.bytes = bytes ? bytes : 1;
  g_hostBlocks.emplace(reinterpret_cast<uintptr_t>(p), b);
  *ptr = p;
  return POLAR_HIP_OK;
}

int polar_hip_host_free(void* ptr) {
  if (ptr == nullptr) return POLAR_HIP_OK;
  {
    std::unique_lock<std::mutex> g(g_hostMu);
    const uintptr_t base = reinterpret_cast<uintptr_t>(ptr);
    if (g_hostBlocks.find(base) == g_hostBlocks.end())
      return fail(POLAR_HIP_ERR_INVALID, "polar_hip_host_free: %p is not a block of polar_hip_host_alloc", ptr);
    // until nothing is outstanding: another thread may queue while the mutex is released
    for (;;) {
      POLAR_HIP_TRY(waitForBlock(g, base));
      auto it = g_hostBlocks.find(base);
      if (it == g_hostBlocks.end())
        return fail(POLAR_HIP_ERR_INVALID, "polar_hip_host_free: %p was freed by another thread", ptr);
      if (it->second.number == 0) {
        g_hostBlocks.erase(it);
        break;
      }
    }
  }
  POLAR_HIP_TRY(hipHostFree(ptr));
  return POLAR_HIP_OK;
}

int polar_hip_host_quiesce(void* ptr) {
  if (ptr == nullptr) return POLAR_HIP_OK;
  std::unique_lock<std::mutex> g(g_hostMu);
  uintptr_t base = 0;
  if (hostBlockOf(ptr, 1, &base) == nullptr)
    return fail(POLAR_HIP_ERR_INVALID, "polar_hip_host_quiesce: %p is not inside a block of polar_hip_host_alloc", ptr);
  POLAR_HIP_TRY(waitForBlock(g, base));
  return POLAR_HIP_OK;
}

int polar_hip_copy_to_device(polar_hip_device* dev, void* dst_device,
                             const void* src_host, uint64_t bytes) {
  POLAR_HIP_REQUIRE(dev != nullptr, "dev is null");
  if (bytes == 0) return POLAR_HIP_OK;
  POLAR_HIP_REQUIRE(dst_device != nullptr && src_host != nullptr,
                    "null buffer");
  POLAR_HIP_TRY(hipSetDevice(dev->ordinal));
  {
    // source inside a block of polar_hip_host_alloc: no staging
    std::unique_lock<std::mutex> g(g_hostMu);
    uintptr_t base = 0;
    if (hostBlockOf(src_host, bytes, &base) != nullptr) {
      POLAR_HIP_TRY(queueDirect(g, dev, base, dst_device, src_host, bytes, hipMemcpyHostToDevice));
      return POLAR_HIP_OK;
    }
  }
  {
    // The data is copied into pinned slots and sent from there, so the call
    // returns once the last DMA is queued and the caller may reuse its memory.
    // From kTwoThreadBytes on, slots are filled whole (2 MiB) and every second
    // one by the drain thread: one thread fills at about 30 GB/s, less than
    // the link takes.
    std::lock_guard<std::mutex> g(dev->stagingMu);
    if (stagingReady(dev)) {
      const bool twoThreads = bytes >= kTwoThreadBytes;
      const uint64_t chunkBytes = twoThreads ? kSlotCapacity : kSlotBytes;
      // Uploads of one or two chunks (graph inputs) record no event behind
      // their slots: a recorded event is a marker packet between the kernels
      // and a few microseconds of host time, and the slot is normally known to
      // be free again from an event the caller waited for in the meantime (see
      // acquireSlot).  Longer uploads reuse slots while they run and need them.
      const bool evented = bytes > 2 * kSlotBytes;
      const char* src = static_cast<const char*>(src_host);
      char* dst = static_cast<char*>(dst_device);
      auto send = [&](int slot, uint64_t off, uint64_t n) -> hipError_t {
        hipError_t e;
        if (!twoThreads && (reinterpret_cast<uintptr_t>(dst + off) & 15u) == 0) {
          const uint32_t vectors = static_cast<uint32_t>(n / 16), tail = static_cast<uint32_t>(n % 16);
          hipLaunchKernelGGL(slotCopyKernel, dim3(vectors / 256 + 1), dim3(256), 0, dev->stream,
                             reinterpret_cast<const upload_v4*>(slotMemory(dev, slot)),
                             reinterpret_cast<upload_v4*>(dst + off), vectors, tail);
          e = hipGetLastError();
        } else {
          e = hipMemcpyAsync(dst + off, slotMemory(dev, slot), n, hipMemcpyHostToDevice, dev->stream);
        }
        if (e != hipSuccess) return e;
        if (evented) e = hipEventRecord(dev->slotEvent[slot], dev->stream);
        else dev->slotNumber[slot] = dev->directQueued.fetch_add(1) + 1;
        if (e == hipSuccess) {
          dev->slotBusy[slot] = true;
          dev->slotEvented[slot] = evented;
        }
        return e;
      };
      hipError_t failed = hipSuccess;
      for (uint64_t off = 0; off < bytes && failed == hipSuccess; off += 2 * chunkBytes) {
        const uint64_t nA = bytes - off < chunkBytes ? bytes - off : chunkBytes;
        const uint64_t offB = off + nA;
        const uint64_t nB = bytes - offB < chunkBytes ? bytes - offB : chunkBytes;
        int slotA, slotB = -1;
        failed = acquireSlot(dev, &slotA);
        if (failed != hipSuccess) break;
        if (twoThreads && nB > 0) {
          failed = acquireSlot(dev, &slotB);
          if (failed != hipSuccess) break;
          drainPost(dev->drain, slotMemory(dev, slotB), src + offB, nB);
        }
        // below the two-thread size a plain memcpy: the source is usually still in
        // the cache, and the GPU's reads of the slot are served from there too
        // (streaming stores measured 5 us slower on an 800 KB graph input)
        if (twoThreads) copyOutOfSlot(slotMemory(dev, slotA), src + off, nA);
        else memcpy(slotMemory(dev, slotA), src + off, nA);
        failed = send(slotA, off, nA);
        if (slotB >= 0) {
          drainWait(dev->drain); // even if the send failed: the thread holds a job
          if (failed == hipSuccess) failed = send(slotB, offB, nB);
        } else if (failed == hipSuccess && nB > 0) {
          failed = acquireSlot(dev, &slotB);
          if (failed != hipSuccess) break;
          memcpy(slotMemory(dev, slotB), src + offB, nB);
          failed = send(slotB, offB, nB);
        }
      }
      if (failed != hipSuccess) return failHip(failed, "host-to-device copy");
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
    // destination inside a block of polar_hip_host_alloc: written directly, and
    // complete when the call returns (this handle's own earlier transfers out
    // of the block are ahead of the new one on its stream)
    uint64_t number = 0;
    {
      std::unique_lock<std::mutex> g(g_hostMu);
      uintptr_t base = 0;
      if (hostBlockOf(dst_host, bytes, &base) != nullptr)
        POLAR_HIP_TRY(queueDirect(g, dev, base, dst_host, src_device, bytes, hipMemcpyDeviceToHost, &number));
    }
    if (number != 0) {
      // wait outside the table's lock (a large read-back takes milliseconds);
      // the block learns that it is idle from the device's count
      POLAR_HIP_TRY(hipStreamSynchronize(dev->stream));
      dev->noteDirectDone(number);
      return POLAR_HIP_OK;
    }
  }
  {
    // Any size: at most kSlots chunk DMAs are in flight; a chunk is copied out
    // as soon as its event completes and its slot goes to the chunk kSlots
    // further on.  In a large transfer every second chunk is copied out by the
    // drain thread while this thread goes on to the next one.  The thread holds
    // one job at a time and posting a job waits for the previous one, so chunks
    // are consumed kSlots - 2 behind the DMAs instead of kSlots: when chunk i is
    // about to take the slot of chunk i - kSlots, chunk i - kSlots + 2 (same
    // parity) has just been posted or copied, which means the copy of chunk
    // i - kSlots has finished, whichever thread made it.
    std::lock_guard<std::mutex> g(dev->stagingMu);
    if (stagingReady(dev)) {
      int slots[kSlots];
      const uint64_t queuedBefore = dev->directQueued.load();
      const bool twoThreads = bytes >= kTwoThreadBytes;
      // per chunk this thread pays about 10 us of driver calls; with 512 KiB
      // chunks that alone capped a 256 MiB read-back at 24 GB/s
      const uint64_t chunkBytes = twoThreads ? kSlotCapacity : kSlotBytes;
      const uint64_t chunks = (bytes + chunkBytes - 1) / chunkBytes;
      auto consume = [&](uint64_t c) -> hipError_t {
        const uint64_t off = c * chunkBytes;
        const uint64_t n = bytes - off < chunkBytes ? bytes - off : chunkBytes;
        const int slot = slots[c % kSlots];
        hipError_t e = hipEventSynchronize(dev->slotEvent[slot]);
        if (e != hipSuccess) return e;
        dev->slotBusy[slot] = false;
        dev->noteDirectDone(queuedBefore); // ahead of this chunk on the stream
        if (twoThreads && (c & 1))
          drainPost(dev->drain, static_cast<char*>(dst_host) + off, slotMemory(dev, slot), n);
        else
          copyOutOfSlot(static_cast<char*>(dst_host) + off, slotMemory(dev, slot), n);
        return hipSuccess;
      };
      const uint64_t lag = twoThreads ? kSlots - 2 : kSlots;
      hipError_t failed = hipSuccess;
      for (uint64_t c = 0; c < chunks && failed == hipSuccess; ++c) {
        if (c >= lag) failed = consume(c - lag);
        if (failed != hipSuccess) break;
        const uint64_t off = c * chunkBytes;
        const uint64_t n = bytes - off < chunkBytes ? bytes - off : chunkBytes;
        int slot;
        failed = acquireSlot(dev, &slot);
        if (failed != hipSuccess) break;
        slots[c % kSlots] = slot;
        const char* from = static_cast<const char*>(src_device) + off;
        if (!twoThreads && (reinterpret_cast<uintptr_t>(from) & 15u) == 0) {
          const uint32_t vectors = static_cast<uint32_t>(n / 16), tail = static_cast<uint32_t>(n % 16);
          hipLaunchKernelGGL(slotCopyKernel, dim3(vectors / 256 + 1), dim3(256), 0, dev->stream,
                             reinterpret_cast<const upload_v4*>(from),
                             reinterpret_cast<upload_v4*>(slotMemory(dev, slot)), vectors, tail);
          failed = hipGetLastError();
        } else {
          failed = hipMemcpyAsync(slotMemory(dev, slot), from, n, hipMemcpyDeviceToHost, dev->stream);
        }
        if (failed != hipSuccess) break;
        failed = hipEventRecord(dev->slotEvent[slot], dev->stream);
        if (failed != hipSuccess) break;
        dev->slotBusy[slot] = true;
        dev->slotEvented[slot] = true;
      }
      for (uint64_t c = chunks > lag ? chunks - lag : 0; c < chunks && failed == hipSuccess; ++c)
        failed = consume(c);
      if (twoThreads) drainWait(dev->drain); // also on failure: the thread may still hold a job
      if (failed != hipSuccess) return failHip(failed, "device-to-host copy");
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
  e->directStamp = dev->directQueued.load();
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
    if (e == hipSuccess) {
      evt->dev->noteDirectDone(evt->directStamp);
      return POLAR_HIP_OK;
    }
    if (e != hipErrorNotReady) return failHip(e, "hipEventQuery");
    (void)hipGetLastError();
    if (std::chrono::steady_clock::now() - t0 > std::chrono::microseconds(200)) break;
  }
  POLAR_HIP_TRY(hipEventSynchronize(evt->ev));
  evt->dev->noteDirectDone(evt->directStamp);
  return POLAR_HIP_OK;
}

int polar_hip_event_query(polar_hip_event* evt, int* done) {
  POLAR_HIP_REQUIRE(evt != nullptr && done != nullptr, "null argument");
  hipError_t e = hipEventQuery(evt->ev);
  if (e == hipSuccess) {
    evt->dev->noteDirectDone(evt->directStamp);
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
  pair[0]->directStamp = pair[1]->directStamp = 0; // attached to a kernel, not recorded behind the stream
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
