/*
 * polar_harness.h -- C ABI of the mini-executor (libpolar_harness.so).
 *
 * The mini-executor is the caller side of the runtime-plugin boundary, restated
 * so that the plugin can be exercised without the framework's MLIR/LLVM JIT:
 * it loads a plugin the way the framework's runtime driver does
 * (src/backend/generic/runtime/driver/RuntimeDriver.cpp:12-41), owns a
 * host/device coherence allocator with the protocol of
 * src/backend/generic/lib/allocators/LayerAllocator.cpp, and runs a list of
 * nodes with the exact per-node sequence of calls that JIT-compiled graph code
 * makes into the seven ath_* support routines
 * (src/backend/generic/runtime/support/routines.cpp:24-102;
 *  src/core/graph/internal/GraphCompiler.cpp:55-108).
 *
 * Kernels are therefore always reached through
 * initContext() -> Device::launch(LaunchCommand), never called directly.
 *
 * Functions returning int return 0 on success and -1 on a usage error (bad
 * handle or argument).  Runtime failures follow the framework's convention:
 * a message on stderr and process termination.
 */
#ifndef POLAR_HARNESS_H
#define POLAR_HARNESS_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct polar_harness polar_harness;

typedef struct polar_harness_arg {
  int kind;       /* 0 = tensor (vaddr), 1 = fp32 scalar (scalar),
                     2 = 64-bit integer scalar (value in vaddr) */
  uint64_t vaddr; /* virtual address returned by polar_harness_tensor */
  float scalar;
} polar_harness_arg;

typedef struct polar_harness_counters {
  uint64_t launches;        /* Device::launch calls                     */
  uint64_t copies_to_device, bytes_to_device;
  uint64_t copies_to_host, bytes_to_host;
  uint64_t events_waited;   /* Event::wait calls made by barriers       */
  uint64_t deferred_releases; /* releases that ran from event callbacks */
  uint64_t device_name_calls; /* Device::getDeviceName calls on the device
                                 under test (string work the caller causes) */
  /* host wall time of polar_harness_run by phase, nanoseconds, accumulated:
   * input nodes (allocate, lock, load, release in host RAM); per compute node
   * the allocate + lock calls (uploads happen here), the launch call, the
   * release calls; and the barriers that follow the clusters */
  uint64_t ns_input_nodes, ns_allocate_and_lock, ns_launch, ns_release, ns_barrier;
} polar_harness_counters;

/* plugin_path: a runtime plugin to dlopen, or NULL for the built-in CPU mock
 * device (records calls, computes nothing).  device_index selects which of the
 * plugin's devices runs the compute nodes. */
int polar_harness_open(const char* plugin_path, int device_index,
                       polar_harness** out);
void polar_harness_close(polar_harness* h);
int polar_harness_device_count(polar_harness* h);
/* Name / provider / kind of the selected device, through the plugin's vtable. */
const char* polar_harness_device_name(polar_harness* h);
int polar_harness_device_provider(polar_harness* h);
int polar_harness_device_kind(polar_harness* h);

/* Take the RAM-side blocks of tensors from the plugin's pinned host memory
 * (its optional polarHostMemoryAllocate / Release / Quiesce symbols) instead
 * of the heap, so that uploads and read-backs need no staging copy.  Call
 * before the first tensor is allocated.  Returns -1 if the plugin does not
 * export the three symbols (or for the mock device); 0 otherwise.  Off by
 * default: the framework's own RAM layer uses the heap. */
int polar_harness_use_plugin_host_memory(polar_harness* h);

/* Reserve a tensor: returns its virtual address in the context's flat space
 * (first tensor at 1, each next one after the previous one's bytes, as
 * src/core/context/internal/ContextInternal.cpp:43-48). */
uint64_t polar_harness_tensor(polar_harness* h, uint64_t dims,
                              const uint64_t* shape);

/* Append an input node (host node: allocate in RAM, lock RW, load, release).
 * The data is copied; the loader memcpy's it in at run time.  data == NULL
 * gives a loader that loads nothing: a node that only holds a tensor some
 * other node or graph produced (the framework's DummyLoader). */
int polar_harness_input(polar_harness* h, uint64_t vaddr, const float* data);
/* Append a compute node launching one builtin.  args[result_index] is the
 * node's result tensor (allocated on the device, locked READ_WRITE first; the
 * other tensor arguments are locked READ). */
int polar_harness_node(polar_harness* h, const char* native_kernel_name,
                       uint32_t nargs, const polar_harness_arg* args,
                       uint32_t result_index);
/* Append a compute node whose kernel comes from the selected program: it is
 * launched under jit_kernel_name with an empty native kernel name. */
int polar_harness_jit_node(polar_harness* h, const char* jit_kernel_name,
                           uint32_t nargs, const polar_harness_arg* args,
                           uint32_t result_index);
/* Hand the device one compiled program, as the executor does after compiling a
 * graph (Device::selectBinary).  program_type is ProgramDesc::Type (0 PTX,
 * 1 SPIRV_SHADER, 2 HSACO); geometry holds globalX,Y,Z,localX,Y,Z per kernel. */
int polar_harness_select_binary(polar_harness* h, int program_type,
                                const char* target, const void* image,
                                uint64_t bytes, uint32_t kernel_count,
                                const char* const* kernel_names,
                                const uint64_t* geometry);
/* Close the current cluster: a barrier over its launch events follows it. */
int polar_harness_end_cluster(polar_harness* h);
/* Drop all nodes (tensors and their contents stay). */
int polar_harness_clear_program(polar_harness* h);

/* Execute the node list once (the framework's Executor::evaluate). */
int polar_harness_run(polar_harness* h);
/* Read a tensor back the way an output node does: READ_WRITE lock on the
 * host, which pulls the newest copy from the device, then release. */
int polar_harness_read(polar_harness* h, uint64_t vaddr, float* out,
                       uint64_t count);

/* Direct access to the coherence allocator, for protocol tests.
 * device < 0 means host RAM; lock_type 0 = READ, 1 = READ_WRITE. */
int polar_harness_allocate(polar_harness* h, uint64_t vaddr, int device);
int polar_harness_lock(polar_harness* h, uint64_t vaddr, int device, int lock_type);
int polar_harness_release(polar_harness* h, uint64_t vaddr, int device);
int polar_harness_host_write(polar_harness* h, uint64_t vaddr, const float* data,
                             uint64_t count);
/* Read a tensor the way the framework's OutputNodeAccessor does
 * (include/polarai/core/node/OutputNodeAccessor.hpp:21-31): through the
 * allocator's tensor-OBJECT overloads -- lock(tensor, READ_WRITE), get(tensor),
 * release(tensor) -- with a tensor object of this binary standing for the
 * framework's TensorInternal. */
int polar_harness_read_through_tensor_object(polar_harness* h, uint64_t vaddr,
                                             float* out, uint64_t count);

/* Raw object pointers (Device* of the device under test, the BackendAllocator*,
 * the plugin's Context* or NULL for the mock), for code that wants to use them
 * through its own declaration of the interface -- the interface-conformance
 * probe built from the framework's headers does. */
void* polar_harness_raw_device(polar_harness* h);
void* polar_harness_raw_allocator(polar_harness* h);
void* polar_harness_raw_context(polar_harness* h);

int polar_harness_get_counters(polar_harness* h, polar_harness_counters* out);
/* Cap the device layer's capacity (bytes; 0 = no cap) to force the offload
 * path.  Works for the HIP plugin's devices and the built-in mock device;
 * returns -1 for any other plugin. */
int polar_harness_set_device_byte_limit(polar_harness* h, uint64_t bytes);

#ifdef __cplusplus
}
#endif
#endif /* POLAR_HARNESS_H */
