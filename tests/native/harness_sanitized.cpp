// Drives the mini-executor on its CPU mock device; built by
// tests/test_native_sanitized.py together with the harness sources under
// -fsanitize=address,undefined so that lifetime or indexing mistakes in the
// host code show up without a GPU.
#include "polar_harness.h"
#include "polar_rt_support.hpp"
#include "devices.hpp"
#include "coherent_allocator.hpp"

#include <cstdio>
#include <cstdlib>
#include <vector>

#define CHECK(cond)                                                        \
  do {                                                                     \
    if (!(cond)) {                                                         \
      std::fprintf(stderr, "%s:%d: check failed: %s\n", __FILE__, __LINE__, #cond); \
      std::exit(1);                                                        \
    }                                                                      \
  } while (0)

// The eviction scan of the allocator layer (the class the GPU plugin's layer is
// made of, here over heap blocks) with an offload callback that mutates the
// layer while the scan has dropped its mutex: it locks the victim again, frees
// other records and adds enough new ones to rehash the table.
static void evictionScanSurvivesMutatingCallback() {
  using namespace polar_harness_detail;
  RecordLayer<HeapBlocks> layer;
  for (size_t v = 1; v <= 8; ++v) {
    const MemoryRecord r{v * 100, 64};
    layer.allocate(r);
    layer.lock(r);
    layer.release(r);
  }
  layer.setByteLimit(8 * 64);
  int calls = 0;
  size_t firstVictim = 0;
  layer.registerMemoryOffloadCallback([&](MemoryRecord victim, AllocatorLayerBase& l) {
    if (++calls != 1) return;
    firstVictim = victim.virtualAddress;
    l.lock(victim); // taken again while the scan waits
    int freed = 0;
    for (size_t v = 1; v <= 8 && freed < 2; ++v)
      if (v * 100 != victim.virtualAddress) {
        l.deallocate(MemoryRecord{v * 100, 64});
        ++freed;
      }
    for (size_t v = 0; v < 100; ++v) l.allocate(MemoryRecord{5000 + v, 1}); // rehash
  });
  layer.allocate(MemoryRecord{999, 64});
  CHECK(calls >= 1 && firstVictim != 0);
  CHECK(layer.isAllocated(MemoryRecord{999, 64}));
  CHECK(layer.isAllocated(MemoryRecord{firstVictim, 64})); // locked: must not have been evicted
  CHECK(layer.bytesHeld() <= 8 * 64);
  // nothing evictable at all: every record locked and the limit reached -> the
  // scan must end (it reports failure through the fatal path, not tested here)
  layer.release(MemoryRecord{firstVictim, 64});
  layer.setByteLimit(0);
  layer.allocate(MemoryRecord{1000, 64});
  CHECK(layer.isAllocated(MemoryRecord{1000, 64}));
}

// RAM-side blocks taken from a provider (polar_rt_support_set_host_memory): the
// provider is asked once per record, a null answer falls back to the heap,
// quiesce runs before every host access to a provided block and never for a
// heap one, and every provided block goes back through release.
namespace provider {
int allocated = 0, released = 0, quiesced = 0, refused = 0;
void* lastQuiesced = nullptr;
void* allocate(size_t bytes) {
  if (bytes > 4096) {
    ++refused;
    return nullptr;
  }
  ++allocated;
  return std::malloc(bytes);
}
void release(void* p) {
  ++released;
  std::free(p);
}
void quiesce(void* p) {
  ++quiesced;
  lastQuiesced = p;
}
} // namespace provider

static void ramBlocksFromAProvider() {
  using polarai::backend::generic::MemoryRecord;
  using LockType = polarai::core::internal::LockType;
  auto* allocator = polar_rt_support_allocator_create();
  auto* host = polar_rt_support_host_device_create();
  const polar_rt_host_memory hooks{provider::allocate, provider::release, provider::quiesce};
  polar_rt_support_set_host_memory(allocator, &hooks);
  polar_rt_support_register_device(allocator, host);
  const MemoryRecord small{1, 256}, other{1000, 512}, big{5000, 1 << 20};
  allocator->allocate(small);
  allocator->allocate(other);
  allocator->allocate(big); // the provider refuses it: heap
  CHECK(provider::allocated == 2 && provider::refused == 1);
  allocator->allocate(small); // already there: the provider is not asked again
  CHECK(provider::allocated == 2);
  CHECK(provider::quiesced == 0);
  allocator->lock(small, *host, LockType::READ_WRITE);
  CHECK(provider::quiesced == 1);
  auto* p = allocator->get<float>(small, *host);
  CHECK(p != nullptr && provider::lastQuiesced == static_cast<void*>(p));
  for (int i = 0; i < 64; ++i) p[i] = float(i);
  allocator->release(small, *host);
  allocator->lock(big, *host, LockType::READ_WRITE);
  CHECK(provider::quiesced == 1); // heap block: nothing to wait for
  allocator->get<float>(big, *host)[(1 << 18) - 1] = 1.0f;
  allocator->release(big, *host);
  allocator->lock(small, *host, LockType::READ);
  CHECK(provider::quiesced == 2 && allocator->get<float>(small, *host)[63] == 63.0f);
  allocator->release(small, *host);
  static_cast<polar_harness_detail::CoherentAllocator*>(allocator)->deallocate(small);
  CHECK(provider::released == 1);
  polar_rt_support_host_device_destroy(host);
  polar_rt_support_allocator_destroy(allocator); // gives back what is left
  CHECK(provider::released == 2);
}

int main() {
  evictionScanSurvivesMutatingCallback();
  ramBlocksFromAProvider();
  for (int round = 0; round < 3; ++round) {
    polar_harness* h = nullptr;
    CHECK(polar_harness_open(nullptr, 0, &h) == 0);
    CHECK(polar_harness_device_count(h) == 1);
    const uint64_t shape[2] = {16, 8};
    const uint64_t a = polar_harness_tensor(h, 2, shape);
    const uint64_t b = polar_harness_tensor(h, 2, shape);
    const uint64_t c = polar_harness_tensor(h, 2, shape);
    const uint64_t d = polar_harness_tensor(h, 2, shape);
    CHECK(a == 1 && b == 1 + 512 && c == 1 + 1024);
    std::vector<float> data(128, 1.5f);
    CHECK(polar_harness_input(h, a, data.data()) == 0);
    CHECK(polar_harness_input(h, b, nullptr) == 0); // holder: loads nothing
    CHECK(polar_harness_end_cluster(h) == 0);
    polar_harness_arg add[5] = {{0, a, 0}, {1, 0, 1.0f}, {0, b, 0}, {1, 0, 2.0f}, {0, c, 0}};
    CHECK(polar_harness_node(h, "fadd", 5, add, 4) == 0);
    CHECK(polar_harness_end_cluster(h) == 0);
    polar_harness_arg inplace[5] = {{0, c, 0}, {1, 0, 1.0f}, {0, a, 0}, {1, 0, 1.0f}, {0, a, 0}};
    CHECK(polar_harness_node(h, "fadd", 5, inplace, 4) == 0); // result aliases an operand
    polar_harness_arg mm[3] = {{0, a, 0}, {0, b, 0}, {0, d, 0}};
    CHECK(polar_harness_node(h, "fmatmul_f_t", 3, mm, 2) == 0);
    CHECK(polar_harness_node(h, "fadd", 5, add, 9) == -1);    // bad result index
    CHECK(polar_harness_end_cluster(h) == 0);
    for (int i = 0; i < 4; ++i) CHECK(polar_harness_run(h) == 0);
    std::vector<float> out(128);
    CHECK(polar_harness_read(h, c, out.data(), 128) == 0);
    CHECK(polar_harness_read(h, a, out.data(), 129) == -1);   // too many elements
    polar_harness_counters k;
    CHECK(polar_harness_get_counters(h, &k) == 0);
    CHECK(k.launches == 12 && k.events_waited == 12);
    CHECK(polar_harness_clear_program(h) == 0);
    // a program handed to the device and a node that names a generated kernel,
    // integer attributes as 64-bit scalars; the support library's helpers
    const char image[] = "not a code object: the mock device ignores programs";
    const char* names[1] = {"gen_kernel"};
    const uint64_t geometry[6] = {4, 1, 1, 64, 1, 1};
    CHECK(polar_harness_select_binary(h, 2, "gfx950", image, sizeof(image), 1, names, geometry) == 0);
    CHECK(polar_harness_select_binary(h, 2, nullptr, nullptr, 0, 0, nullptr, nullptr) == -1);
    polar_harness_arg gen[3] = {{0, a, 0}, {2, 3, 0}, {0, d, 0}};
    CHECK(polar_harness_jit_node(h, "gen_kernel", 3, gen, 2) == 0);
    CHECK(polar_harness_jit_node(h, "", 3, gen, 2) == -1);
    CHECK(polar_harness_end_cluster(h) == 0);
    CHECK(polar_harness_run(h) == 0);
    CHECK(polar_harness_clear_program(h) == 0);
    CHECK(polar_harness_host_write(h, d, data.data(), 128) == 0);
    CHECK(polar_harness_lock(h, d, 0, 0) == 0);
    CHECK(polar_harness_release(h, d, 0) == 0);
    CHECK(polar_harness_read(h, d, out.data(), 128) == 0);
    CHECK(out[5] == 1.5f);
    CHECK(polar_harness_raw_device(h) != nullptr && polar_harness_raw_context(h) == nullptr);
    polar_harness_close(h);
    // construction helpers of the support library
    uint64_t layout[5];
    polar_rt_support_graph_handle_layout(layout);
    CHECK(layout[0] == sizeof(GraphHandle) && layout[1] == 0);
    auto* allocator = polar_rt_support_allocator_create();
    auto* host = polar_rt_support_host_device_create();
    CHECK(allocator != nullptr && host != nullptr && host->getDeviceName() == "host");
    polar_rt_support_host_device_destroy(host);
    polar_rt_support_allocator_destroy(allocator);
  }
  std::puts("ok");
  return 0;
}
