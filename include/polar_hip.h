/*
 * polar_hip.h -- the thin C ABI between the PolarAI/Athena HIP runtime plugin
 * (C++ host library, libpolar_rt_hip.so) and the gfx950 device code
 * (libpolar_hip.so).
 *
 * Everything here is plain C: opaque handles, raw device pointers, 64-bit
 * element counts.  All tensors are dense, row-major fp32, exactly as the
 * reference's runtimes see them (src/backend/generic/runtime/sycl/kernels/
 * common.hpp:35-38).  Kernel entry points enqueue work on the device's stream
 * and return without waiting; ordering is stream order.
 *
 * Return value of every function that returns int: 0 on success, otherwise a
 * polar_hip_status.  A message for the calling thread's last failure is kept
 * and can be read with polar_hip_last_error().  The reference's convention for
 * runtime failures is "print and terminate" (src/backend/generic/runtime/
 * cuda/utils.hpp:20-28, hip/HIPContext.cpp:23-33); the C++ plugin above this
 * layer applies it, this layer only reports.
 *
 * Each entry point names the reference interface it stands in for (paths
 * relative to the reference tree).
 */
#ifndef POLAR_HIP_H
#define POLAR_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum polar_hip_status {
  POLAR_HIP_OK = 0,
  POLAR_HIP_ERR_INVALID = 1,   /* null pointer, bad shape, bad handle         */
  POLAR_HIP_ERR_NO_DEVICE = 2, /* no usable gfx950 device / ordinal too large */
  POLAR_HIP_ERR_OOM = 3,       /* device memory exhausted                     */
  POLAR_HIP_ERR_RUNTIME = 4    /* a HIP call failed; see polar_hip_last_error */
} polar_hip_status;

typedef struct polar_hip_device polar_hip_device; /* one GPU: stream + pool  */
typedef struct polar_hip_event polar_hip_event;   /* a point in stream order */

typedef struct polar_hip_device_info {
  char name[256];          /* marketing name                                  */
  char arch[64];           /* gcnArchName, e.g. "gfx950:sramecc+:xnack-"      */
  int ordinal;             /* HIP device ordinal                              */
  int compute_units;       /* multiProcessorCount                             */
  int clock_khz;           /* max engine clock                                */
  int memory_clock_khz;    /* max memory clock                                */
  int memory_bus_bits;     /* memory bus width                                */
  int lds_bytes_per_block; /* sharedMemPerBlock                               */
  int l2_bytes;            /* l2CacheSize                                     */
  int pci_bus_id;
  uint64_t hbm_bytes;      /* totalGlobalMem                                  */
} polar_hip_device_info;

typedef struct polar_hip_pool_stats {
  uint64_t bytes_in_use;   /* handed out and not yet freed                    */
  uint64_t bytes_cached;   /* held by the pool for reuse                      */
  uint64_t device_allocs;  /* number of hipMalloc calls made so far           */
  uint64_t pool_hits;      /* allocations served from cached blocks           */
} polar_hip_pool_stats;

const char* polar_hip_last_error(void);
const char* polar_hip_version(void);

/* ---- devices ---------------------------------------------------------------
 * Stand in for device enumeration in the reference's contexts
 * (src/backend/generic/runtime/hip/HIPContext.cpp:21-37,
 *  src/backend/generic/runtime/sycl/SYCLContext.cpp:22-39). */
int polar_hip_device_count(int* count);
int polar_hip_device_open(int ordinal, polar_hip_device** out);
int polar_hip_device_close(polar_hip_device* dev);
int polar_hip_device_get_info(polar_hip_device* dev, polar_hip_device_info* out);
/* Block the calling thread until everything enqueued on the device is done. */
int polar_hip_device_synchronize(polar_hip_device* dev);

/* ---- device memory pool -----------------------------------------------------
 * Stand in for the per-tensor raw device allocation of the reference's
 * allocator layers (src/backend/generic/runtime/cuda/CudaAllocator.hpp:54-78,
 * src/backend/generic/runtime/sycl/USMAllocator.h:65-91).  Blocks are at least
 * 256-byte aligned.  Freed blocks are cached and handed out again in stream
 * order: a freed block may be reused by work enqueued later on the same
 * device, never by work already enqueued. */
int polar_hip_alloc(polar_hip_device* dev, uint64_t bytes, void** ptr);
int polar_hip_free(polar_hip_device* dev, void* ptr);
/* Return all cached blocks to the driver (waits for the stream first). */
int polar_hip_pool_trim(polar_hip_device* dev);
int polar_hip_pool_get_stats(polar_hip_device* dev, polar_hip_pool_stats* out);

/* ---- host <-> device copies -------------------------------------------------
 * Stand in for Device::copyToDevice / copyToHost of the reference's runtimes
 * (src/backend/generic/runtime/cuda/CudaDevice.hpp:52-61,
 *  src/backend/generic/runtime/sycl/SYCLDevice.h:81-112): ordered after all
 * work already enqueued on the device.  copy_to_host is complete when the call
 * returns.  copy_to_device has consumed src_host when it returns (the caller
 * may reuse it at once: the bytes were copied into pinned staging memory); the
 * transfer into dst_device may still be in flight on the device's stream,
 * where every later kernel, copy and event of this library is ordered behind
 * it.  Transfers of 8 MiB and more use a second host thread of the library
 * for half of the host-side copying. */
int polar_hip_copy_to_device(polar_hip_device* dev, void* dst_device,
                             const void* src_host, uint64_t bytes);
int polar_hip_copy_to_host(polar_hip_device* dev, void* dst_host,
                           const void* src_device, uint64_t bytes);

/* ---- host memory the GPU can address ----------------------------------------
 * No counterpart in the reference, whose host-side tensor storage is new[]
 * (src/backend/generic/lib/allocators/TrivialAllocator.hpp:23-93).  A caller
 * that keeps its host copies of tensors in blocks from polar_hip_host_alloc
 * (pinned memory) saves the staging copy of every transfer: the two copy
 * calls above recognise a host pointer inside such a block and move the bytes
 * directly between it and device memory.
 * Consequence for copy_to_device from such a block: the call returns with the
 * transfer queued, not with the source consumed.  Before the host WRITES the
 * block again it calls polar_hip_host_quiesce, which returns once every queued
 * transfer out of the block has completed.  That costs nothing when the caller
 * has meanwhile waited for an event recorded behind the transfer
 * (polar_hip_event_synchronize / _query, polar_hip_device_synchronize): the
 * library notes how far the stream has got.  Otherwise it waits for all work
 * the stream holds.  polar_hip_host_free quiesces by itself.  The blocks are process-wide: they
 * outlive the device handle they were allocated through. */
int polar_hip_host_alloc(polar_hip_device* dev, uint64_t bytes, void** ptr);
int polar_hip_host_free(void* ptr);
int polar_hip_host_quiesce(void* ptr);

/* ---- events -------------------------------------------------------------------
 * Stand in for the native event inside the reference's Event objects
 * (src/backend/generic/runtime/cuda/CudaEvent.cpp:18-31,
 *  src/backend/generic/runtime/cuda/CudaDevice.cpp:109-113).  Events come from
 * a per-device pool; release returns one to it. */
int polar_hip_event_record(polar_hip_device* dev, polar_hip_event** out);
int polar_hip_event_synchronize(polar_hip_event* evt);     /* host waits      */
int polar_hip_event_query(polar_hip_event* evt, int* done); /* non-blocking   */
/* Make later work on `dev` wait for `evt` (which may belong to another device)
 * without blocking the host. */
int polar_hip_stream_wait_event(polar_hip_device* dev, polar_hip_event* evt);
/* Milliseconds between two completed events recorded on the same device. */
int polar_hip_event_elapsed_ms(polar_hip_event* start, polar_hip_event* stop,
                               float* ms);
/* Profiling aid with no counterpart in the reference: the next kernel that an
 * entry point below launches on `dev` carries *start and *stop as its own
 * begin and end timestamps, so polar_hip_event_elapsed_ms(*start, *stop) is
 * that kernel's execution time without launch or queue gaps.  Exactly ONE
 * launch is timed: an entry point that runs several kernels (fsoftmax, a
 * matmul that splits the contraction) has only its first one bracketed --
 * time such a call with polar_hip_event_record before and after it instead.
 * Synchronize *stop before reading; release both events afterwards. */
int polar_hip_time_next_kernel(polar_hip_device* dev, polar_hip_event** start,
                               polar_hip_event** stop);
int polar_hip_event_release(polar_hip_event* evt);

/* ---- builtin-operation kernels ---------------------------------------------
 * One entry point per nativeKernelName the launch lowering can emit
 * (utils/dialects/include/PolarGraph/PolarGraphOps.td:237,275,296,317,
 *  343-351,371,393,481,523,542).  n counts elements.  Pointers are device
 * pointers and may have any 4-byte alignment; output may alias an input only
 * where the two are the same pointer (in-place). */

/* fadd: c[i] = scaleA*a[i] + scaleB*b[i]
 * (src/backend/generic/runtime/sycl/kernels/AddNaive.hpp:33-35) */
int polar_hip_fadd(polar_hip_device* dev, const float* a, float scaleA,
                   const float* b, float scaleB, float* c, uint64_t n);
/* fmul: c[i] = a[i]*b[i]  (sycl/kernels/Mul.hpp:32) */
int polar_hip_fmul(polar_hip_device* dev, const float* a, const float* b,
                   float* c, uint64_t n);
/* fdivide: out[i] = numerator[i]/denominator[i], IEEE rounding
 * (sycl/kernels/Divide.hpp:33-35) */
int polar_hip_fdivide(polar_hip_device* dev, const float* numerator,
                      const float* denominator, float* out, uint64_t n);
/* fsigmoid: 1/(1+exp(-x)) clamped into [1e-5, 1-1e-5]
 * (sycl/kernels/Sigmoid.hpp:32-41) */
int polar_hip_fsigmoid(polar_hip_device* dev, const float* in, float* out,
                       uint64_t n);
/* flogloss: -g*log(p+1e-5) - (1-g)*log(1-p+1e-5), elementwise
 * (sycl/kernels/LogLoss.hpp:33-37) */
int polar_hip_flogloss(polar_hip_device* dev, const float* predicted,
                       const float* groundTruth, float* out, uint64_t n);
/* fmulconcat: out[i] = gradient[0]*localDerivative[i]
 * (sycl/kernels/MulConcat.hpp:33-35) */
int polar_hip_fmulconcat(polar_hip_device* dev, const float* gradient,
                         const float* localDerivative, float* out, uint64_t n);
/* fcopy: dst = src (sycl/kernels/Copy.hpp:27-57) */
int polar_hip_fcopy(polar_hip_device* dev, const float* src, float* dst,
                    uint64_t n);
/* ffill: out[i] = pattern (sycl/kernels/Fill.hpp:54-81) */
int polar_hip_ffill(polar_hip_device* dev, float pattern, float* out,
                    uint64_t n);
/* ftranspose: out[j*rows+i] = in[i*cols+j]; in is rows x cols
 * (spec only: include/polarai/core/internal/GenBuiltins.hpp:50,
 *  utils/dialects/include/PolarGraph/PolarGraphOps.td:507-527) */
int polar_hip_ftranspose(polar_hip_device* dev, const float* in, float* out,
                         uint64_t rows, uint64_t cols);
/* fmatmul_{f,t}_{f,t}: C[M x N] = opA(A) * opB(B), C overwritten, fp32.
 * A is stored [M x K] (transA = 0) or [K x M] (transA != 0); B is stored
 * [K x N] (transB = 0) or [N x K] (transB != 0)
 * (sycl/kernels/MatMul.hpp:33-64; shapes as in
 *  tests/integration/operations/MatMulOperation.cpp:203-204,249-250). */
int polar_hip_fmatmul(polar_hip_device* dev, int transA, int transB,
                      const float* a, const float* b, float* c, uint64_t m,
                      uint64_t n, uint64_t k);
/* How polar_hip_fmatmul would compute an M x N x K product (no counterpart in
 * the reference; for tuning and tests): the tile configuration its planner
 * picks (an index into the library's table; -1 for the shapes taken by the
 * short-contraction and long-contraction kernels), the number of parts the
 * contraction is split into, and, if tile is not null, the tile's extent along
 * M, N and K.  The parts' partial products are added in split order, by a
 * second kernel or (up to eight parts, where that is estimated to be cheaper)
 * by the work-group that finishes a tile last: same bits on every run either
 * way. */
int polar_hip_fmatmul_plan(polar_hip_device* dev, uint64_t m, uint64_t n,
                           uint64_t k, int* tile_config, uint32_t* splits,
                           uint32_t tile[3]);
#define POLAR_HIP_MATMUL_TILE_CONFIGS 10
/* polar_hip_fmatmul with the tile configuration (0 .. POLAR_HIP_MATMUL_TILE_
 * CONFIGS - 1) and split count (1 .. 256; reduced to what K can fill) given by
 * the caller instead of the planner.  Same result up to the order of the
 * additions along K. */
int polar_hip_fmatmul_with_plan(polar_hip_device* dev, int transA, int transB,
                                const float* a, const float* b, float* c,
                                uint64_t m, uint64_t n, uint64_t k,
                                int tile_config, uint32_t splits);

/* ---- Code objects compiled elsewhere (the framework's JIT) --------------------
 * Counterpart of the module handling in the reference's CUDA runtime
 * (src/backend/generic/runtime/cuda/CudaDevice.cpp:39-61 link/load,
 *  :98-109 cuModuleGetFunction + cuLaunchKernel): load an AMDGPU code object
 * (HSACO or an offload bundle holding a gfx950 image) and launch a kernel of
 * it by name on the device's stream.  params[i] points at the i-th kernel
 * parameter, as for cuLaunchKernel; grid counts work-groups. */
typedef struct polar_hip_module polar_hip_module;
int polar_hip_module_load(polar_hip_device* dev, const void* image,
                          uint64_t bytes, polar_hip_module** out);
int polar_hip_module_unload(polar_hip_device* dev, polar_hip_module* module);
/* *found = 1 if the module defines a kernel of that name, else 0. */
int polar_hip_module_has_kernel(polar_hip_module* module, const char* name,
                                int* found);
int polar_hip_module_launch(polar_hip_device* dev, polar_hip_module* module,
                            const char* name, const uint32_t grid[3],
                            const uint32_t block[3], void** params);

/* ---- Builtins the reference specifies only as generated (MLIR) kernels ------
 * Their hand-written runtimes have no entry for them; two of them cannot even
 * be named there (ReLU and Softmax both answer "ftranspose" as their builtin
 * name -- utils/dialects/include/PolarGraph/PolarGraphOps.td:462,501), so the
 * plugin takes them under the names frelu / fsoftmax. */
/* frelu: out[i] = in[i] > 0 ? in[i] : 0
 * (utils/dialects/lib/PolarGraph/kernels/ReLUOp.cpp:35-44) */
int polar_hip_frelu(polar_hip_device* dev, const float* in, float* out,
                    uint64_t n);
/* fsoftmax: out[i] = exp(in[i]) / sum_j exp(in[j]), the sum running over the
 * WHOLE tensor, no max subtraction
 * (utils/dialects/lib/PolarGraph/kernels/SoftmaxOp.cpp:38-65).  The sum is
 * accumulated in fp64 in a fixed order and rounded to fp32 once. */
int polar_hip_fsoftmax(polar_hip_device* dev, const float* in, float* out,
                       uint64_t n);
/* fsoftmax that allocates nothing.  No counterpart in the reference: it is for
 * callers that cannot allocate device memory at the call (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  Same kernels
 * and same result, bit for bit, as polar_hip_fsoftmax; the partial sums go to
 * an array in the library's device data segment (256 KiB + 256 B per GPU, held
 * until the process ends) instead of the workspace block that the device
 * allocates when it is opened.  n is limited to 2^31
 * elements; more returns POLAR_HIP_ERR_INVALID.  All calls on one GPU share
 * that array: calls that overlap on one GPU (two host threads, or two devices
 * handles opened on the same ordinal) race on it. */
int polar_hip_fsoftmax_static(polar_hip_device* dev, const float* in,
                              float* out, uint64_t n);
/* fconv2d: single-channel "valid" correlation, in is height x width, kernel
 * kernelHeight x kernelWidth (odd sizes), out is (height-kernelHeight+1) x
 * (width-kernelWidth+1); fp32 accumulation in tap order (a outer, b inner)
 * (utils/dialects/lib/PolarGraph/kernels/Conv2DOp.cpp:35-84;
 *  src/operation/internal/Conv2DOperationInternal.cpp:35-39). */
int polar_hip_fconv2d(polar_hip_device* dev, const float* in,
                      const float* kernel, float* out, uint64_t height,
                      uint64_t width, uint64_t kernelHeight,
                      uint64_t kernelWidth);
/* fpool: max pooling, out[y,x] = max(-10e5, max over the window0 x window1
 * block at (y*stride0, x*stride1)); out is ((height-window0)/stride0+1) x
 * ((width-window1)/stride1+1)
 * (utils/dialects/lib/PolarGraph/kernels/Pool2DOp.cpp:45-82;
 *  src/operation/internal/Pool2DOperationInternal.cpp:37-41). */
int polar_hip_fpool(polar_hip_device* dev, const float* in, float* out,
                    uint64_t height, uint64_t width, uint64_t window0,
                    uint64_t window1, uint64_t stride0, uint64_t stride1);
/* Which kernel polar_hip_fpool takes for a call, without running it (the
 * pooling counterpart of polar_hip_fmatmul_plan; needs no device).
 * input_aligned: the input pointer is 16-byte aligned.  *kernel: 0 = every tap
 * read from memory, 1 = non-overlapping 2x2 / 4x4 windows read by vectors,
 * 2 = the band's input window staged in LDS; then *band_rows output rows per
 * work-group and *lds_bytes of LDS (either may be null), 3 = overlapping square
 * windows of 4 or 5 at stride 1 or 2 over rows that start on 16 bytes: waves
 * march down strips of *band_rows output rows, row folds kept in registers.  No counterpart in the
 * reference, whose pooling is generated code
 * (utils/dialects/lib/PolarGraph/kernels/Pool2DOp.cpp:45-82). */
int polar_hip_fpool_plan(uint64_t height, uint64_t width, uint64_t window0,
                         uint64_t window1, uint64_t stride0, uint64_t stride1,
                         int input_aligned, int* kernel, uint32_t* band_rows,
                         uint32_t* lds_bytes);

/* ---- Extended (fused) builtins -------------------------------------------------
 * The reference's design allows runtimes to offer fused builtins that
 * optimisation passes may emit, never the graph compiler itself
 * (docs/design/llvm/04_builtins.md:12-19); it defines none.  These three fuse
 * the chains its model graphs contain (matmul -> fadd -> fsigmoid, matmul ->
 * fsigmoid, fsigmoid -> flogloss).  Each applies the operations of the
 * builtins it replaces, in their order, so its result is bit-identical to
 * running them one after the other. */
/* out = fsigmoid(opA(A) * opB(B)) */
int polar_hip_fmatmul_fsigmoid(polar_hip_device* dev, int transA, int transB,
                               const float* a, const float* b, float* out,
                               uint64_t m, uint64_t n, uint64_t k);
/* out = fsigmoid(fadd(opA(A) * opB(B), scaleProduct, bias, scaleBias)); bias is
 * M x N (fadd does not broadcast) */
int polar_hip_fmatmul_fadd_fsigmoid(polar_hip_device* dev, int transA,
                                    int transB, const float* a, const float* b,
                                    float scaleProduct, const float* bias,
                                    float scaleBias, float* out, uint64_t m,
                                    uint64_t n, uint64_t k);
/* out = flogloss(fsigmoid(in), groundTruth) */
int polar_hip_fsigmoid_flogloss(polar_hip_device* dev, const float* in,
                                const float* groundTruth, float* out,
                                uint64_t n);

#ifdef __cplusplus
}
#endif
#endif /* POLAR_HIP_H */
