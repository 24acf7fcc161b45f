// Memory-bound builtin operations for gfx950: fadd fmul fdivide fsigmoid
// flogloss fmulconcat fcopy ffill.
//
// One kernel template serves all of them.  A work-group of BLOCK lanes owns a
// tile of BLOCK*UNROLL 16-byte vectors; every lane issues all of its dwordx4
// loads before the first use, then computes and stores.  Measured on MI355X
// with buffers rotated to defeat the Infinity Cache, the best shape for a
// streaming kernel is the smallest one: one vector per lane (UNROLL = 1) and
// work-groups of two waves for kernels that read (one wave-pair per 2 KiB of
// each stream), four waves for the store-only fill (fewer, larger groups keep
// the dispatcher ahead of the stores); grid-stride loops with a fixed grid
// were 3-10 % slower.  Loads and stores are marked non-temporal: every byte
// is touched once, so keeping it in L2 / Infinity Cache only evicts other
// data (6-10 % faster than plain accesses).  Tiles are handed out grid-stride
// only when the element count exceeds what one grid can index.  The n % 4
// trailing elements are done by the first lanes of block 0.  Streams that start
// at the same offset from a 16-byte boundary are peeled by up to 31 leading
// elements so that the output's vector stores cover whole 128-byte lines;
// streams with different offsets take a dword kernel instead.
//
// Arithmetic is written so that it rounds exactly like the host kernels it
// replaces: this file is compiled with -ffp-contract=off (no fused
// multiply-add in `sa*a + sb*b`), `/` is the correctly rounded IEEE division
// and expf/logf are the full-precision library versions.
#include "internal.h"

using namespace polar_hip_detail;

namespace {

typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kScalarBlock = 256;

// ---- per-element operations ---------------------------------------------------
// NIN = number of input streams.  apply(x, y) receives the i-th element of each.

struct AddOp { // src/backend/generic/runtime/sycl/kernels/AddNaive.hpp:33-35
  static constexpr int NIN = 2;
  float sa, sb;
  __device__ __forceinline__ float apply(float a, float b) const {
    return sa * a + sb * b;
  }
};
struct MulOp { // sycl/kernels/Mul.hpp:32
  static constexpr int NIN = 2;
  __device__ __forceinline__ float apply(float a, float b) const {
    return a * b;
  }
};
struct DivOp { // sycl/kernels/Divide.hpp:33-35
  static constexpr int NIN = 2;
  __device__ __forceinline__ float apply(float a, float b) const {
    return a / b;
  }
};
struct LogLossOp { // sycl/kernels/LogLoss.hpp:33-37
  static constexpr int NIN = 2;
  __device__ __forceinline__ float apply(float p, float g) const {
    const float eps = 1e-5f;
    return -g * logf(p + eps) - (1.0f - g) * logf(1.0f - p + eps);
  }
};
struct SigmoidOp { // sycl/kernels/Sigmoid.hpp:32-41
  static constexpr int NIN = 1;
  __device__ __forceinline__ float apply(float x, float) const {
    const float eps = 1e-5f;
    float r = 1.0f / (1.0f + expf(-x));
    if (fabsf(r - 1.0f) < eps) {
      r = 1.0f - eps;
    } else if (fabsf(r) < eps) {
      r = eps;
    }
    return r;
  }
};
// Extended builtin: flogloss(fsigmoid(x), truth) in one pass, the operations of
// the two functors above in the same order (bit-identical to the chain).
struct SigmoidLogLossOp {
  static constexpr int NIN = 2;
  __device__ __forceinline__ float apply(float x, float g) const {
    return LogLossOp{}.apply(SigmoidOp{}.apply(x, 0.0f), g);
  }
};
struct ScaleOp { // sycl/kernels/MulConcat.hpp:33-35 (g = gradient[0])
  static constexpr int NIN = 1;
  float g;
  __device__ __forceinline__ float apply(float d, float) const {
    return g * d;
  }
};
struct ReluOp { // utils/dialects/lib/PolarGraph/kernels/ReLUOp.cpp:35-44
  static constexpr int NIN = 1;
  __device__ __forceinline__ float apply(float x, float) const {
    return x > 0.0f ? x : 0.0f; // ordered compare: NaN -> 0
  }
};
struct SoftmaxScaleOp { // utils/dialects/lib/PolarGraph/kernels/SoftmaxOp.cpp:56-63
  static constexpr int NIN = 1;
  float total;
  __device__ __forceinline__ float apply(float x, float) const {
    return expf(x) / total;
  }
};
struct CopyOp { // sycl/kernels/Copy.hpp:49-53
  static constexpr int NIN = 1;
  __device__ __forceinline__ float apply(float s, float) const { return s; }
};
struct FillOp { // sycl/kernels/Fill.hpp:69-74
  static constexpr int NIN = 0;
  float pattern;
  __device__ __forceinline__ float apply(float, float) const {
    return pattern;
  }
};

template <typename Op>
__device__ __forceinline__ v4f apply4(const Op& op, v4f a, v4f b) {
  v4f r;
  r.x = op.apply(a.x, b.x);
  r.y = op.apply(a.y, b.y);
  r.z = op.apply(a.z, b.z);
  r.w = op.apply(a.w, b.w);
  return r;
}

// fmulconcat reads its scalar from device memory; every lane reads the same
// address, which the compiler turns into one scalar load per wave.
template <typename Op> struct OpLoader {
  __device__ static Op load(const Op& op, const float*) { return op; }
};
template <> struct OpLoader<ScaleOp> {
  __device__ static ScaleOp load(const ScaleOp&, const float* g) {
    return ScaleOp{g[0]};
  }
};

template <> struct OpLoader<SoftmaxScaleOp> {
  __device__ static SoftmaxScaleOp load(const SoftmaxScaleOp&, const float* t) {
    return SoftmaxScaleOp{t[0]};
  }
};

// Output stores.  Kernels with at most one input stream write through at
// device scope as well as non-temporally (fcopy 86.5 -> 80 us, ffill 39.6 ->
// 37.6 us); with two input streams the plain non-temporal store measured
// better (fdivide 120.5 vs 125 us), so those keep it.
template <typename Op>
__device__ __forceinline__ void storeOut(v4f value, v4f* address) {
  if constexpr (Op::NIN >= 2)
    __builtin_nontemporal_store(value, address);
  else
    streamStore(value, address);
}

// as/bs/cs are the tensors themselves; the first `head` (< 32) elements bring
// the output to a 128-byte line boundary (and every stream to a 16-byte one),
// n4 vectors follow, then the tail.
template <typename Op, int kBlock, int UNROLL>
__global__ __launch_bounds__(kBlock) void ewVecKernel(
    Op op0, const float* scalarSrc, const float* as, const float* bs, float* cs,
    uint32_t head, uint64_t n4, uint64_t n, uint64_t numTiles) {
  const Op op = OpLoader<Op>::load(op0, scalarSrc);
  const v4f* a = reinterpret_cast<const v4f*>(as + head);
  const v4f* b = reinterpret_cast<const v4f*>(bs + head);
  v4f* c = reinterpret_cast<v4f*>(cs + head);
  constexpr uint64_t kTile = uint64_t(kBlock) * UNROLL;
  for (uint64_t tile = blockIdx.x; tile < numTiles; tile += gridDim.x) {
    const uint64_t base = tile * kTile + threadIdx.x;
    v4f va[UNROLL], vb[UNROLL];
    if (base - threadIdx.x + kTile <= n4) { // whole tile in range
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        const uint64_t i = base + uint64_t(u) * kBlock;
        va[u] = Op::NIN >= 1 ? __builtin_nontemporal_load(&a[i]) : v4f{0, 0, 0, 0};
        vb[u] = Op::NIN >= 2 ? __builtin_nontemporal_load(&b[i]) : v4f{0, 0, 0, 0};
      }
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        const uint64_t i = base + uint64_t(u) * kBlock;
        storeOut<Op>(apply4(op, va[u], vb[u]), &c[i]);
      }
    } else {
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        const uint64_t i = base + uint64_t(u) * kBlock;
        if (i < n4) {
          va[u] = Op::NIN >= 1 ? __builtin_nontemporal_load(&a[i]) : v4f{0, 0, 0, 0};
          vb[u] = Op::NIN >= 2 ? __builtin_nontemporal_load(&b[i]) : v4f{0, 0, 0, 0};
        }
      }
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        const uint64_t i = base + uint64_t(u) * kBlock;
        if (i < n4) storeOut<Op>(apply4(op, va[u], vb[u]), &c[i]);
      }
    }
  }
  // the elements before the first and after the last whole vector
  if (blockIdx.x == 0 && threadIdx.x < 36) {
    const uint64_t i = threadIdx.x < 32 ? threadIdx.x
                                        : head + n4 * 4 + (threadIdx.x - 32);
    const bool mine = threadIdx.x < 32 ? threadIdx.x < head : i < n;
    if (mine) {
      float x = Op::NIN >= 1 ? as[i] : 0.0f;
      float y = Op::NIN >= 2 ? bs[i] : 0.0f;
      cs[i] = op.apply(x, y);
    }
  }
}

// Streams whose 16-byte phases differ (sub-tensor views, odd offsets): dword
// accesses.  The first `head` (< 32) elements bring the output to a 128-byte
// line boundary, so every wave-wide store of the main part covers whole lines;
// a work-group then takes kScalarUnroll x 256 consecutive elements, all loads
// before the first store.  Stores stream as in the vector kernel; the loads
// stay cacheable, because a wave-wide dword load of a stream that is off the
// output's phase straddles three lines and shares two of them with its
// neighbours (copy of 2^26 elements: 98 us with non-temporal loads, 84 us
// with plain ones, 81 us on the vector path; 117-128 us before this layout).
constexpr int kScalarUnroll = 4;
template <typename Op>
__device__ __forceinline__ void storeOutScalar(float value, float* address) {
  if constexpr (Op::NIN >= 2)
    __builtin_nontemporal_store(value, address);
  else
    streamStore(value, address);
}
template <typename Op>
__global__ __launch_bounds__(kScalarBlock) void ewScalarKernel(
    Op op0, const float* scalarSrc, const float* a, const float* b, float* c,
    uint32_t head, uint64_t n) {
  const Op op = OpLoader<Op>::load(op0, scalarSrc);
  const uint64_t base =
      head + uint64_t(blockIdx.x) * (kScalarBlock * kScalarUnroll) + threadIdx.x;
  float x[kScalarUnroll], y[kScalarUnroll];
#pragma unroll
  for (int u = 0; u < kScalarUnroll; ++u) {
    const uint64_t i = base + uint64_t(u) * kScalarBlock;
    x[u] = (Op::NIN >= 1 && i < n) ? a[i] : 0.0f;
    y[u] = (Op::NIN >= 2 && i < n) ? b[i] : 0.0f;
  }
#pragma unroll
  for (int u = 0; u < kScalarUnroll; ++u) {
    const uint64_t i = base + uint64_t(u) * kScalarBlock;
    if (i < n) storeOutScalar<Op>(op.apply(x[u], y[u]), &c[i]);
  }
  if (blockIdx.x == 0 && threadIdx.x < head) {
    const float hx = Op::NIN >= 1 ? a[threadIdx.x] : 0.0f;
    const float hy = Op::NIN >= 2 ? b[threadIdx.x] : 0.0f;
    c[threadIdx.x] = op.apply(hx, hy);
  }
}

template <typename Op, int kBlock = 128, int UNROLL = 1>
int launchEw(polar_hip_device* dev, const Op& op, const float* scalarSrc,
             const float* a, const float* b, float* c, uint64_t n) {
  if (n == 0) return POLAR_HIP_OK;
  POLAR_HIP_TRY(hipSetDevice(dev->ordinal));
  // The vector path needs all streams to reach a 16-byte boundary after the
  // same number of leading elements (always true for whole pool blocks).
  const uintptr_t phase = reinterpret_cast<uintptr_t>(c) & 15u;
  const bool vec = (Op::NIN < 1 || (reinterpret_cast<uintptr_t>(a) & 15u) == phase) &&
                   (Op::NIN < 2 || (reinterpret_cast<uintptr_t>(b) & 15u) == phase);
  if (vec) {
    // whole wave-wide stores should cover whole 128-byte lines of the output
    uint32_t head = static_cast<uint32_t>(
        ((128u - (reinterpret_cast<uintptr_t>(c) & 127u)) & 127u) / 4u);
    if (head > n) head = static_cast<uint32_t>(n);
    const uint64_t n4 = (n - head) / 4;
    constexpr uint64_t kTile = uint64_t(kBlock) * UNROLL;
    const uint64_t numTiles = (n4 + kTile - 1) / kTile;
    uint64_t grid = numTiles < 1 ? 1 : numTiles;
    if (grid > (1u << 30)) grid = 1u << 30;
    POLAR_HIP_TRY(launchKernel(dev, ewVecKernel<Op, kBlock, UNROLL>,
                               dim3(static_cast<unsigned>(grid)), dim3(kBlock), op,
                               scalarSrc, a, b, c, head, n4, n, numTiles));
  } else {
    uint32_t head = static_cast<uint32_t>(
        ((128u - (reinterpret_cast<uintptr_t>(c) & 127u)) & 127u) / 4u);
    if (head > n) head = static_cast<uint32_t>(n);
    constexpr uint64_t kTile = uint64_t(kScalarBlock) * kScalarUnroll;
    uint64_t grid = (n - head + kTile - 1) / kTile;
    if (grid < 1) grid = 1;
    POLAR_HIP_REQUIRE(grid < (1ull << 31), "tensor too large for one launch");
    POLAR_HIP_TRY(launchKernel(dev, ewScalarKernel<Op>,
                               dim3(static_cast<unsigned>(grid)),
                               dim3(kScalarBlock), op, scalarSrc, a, b, c, head, n));
  }
  return POLAR_HIP_OK;
}

// ---- fsoftmax, first pass: total = sum exp(x) over the whole tensor ----------
// Work-group g sums elements [g*kSumChunk, (g+1)*kSumChunk) into partial[g];
// lanes and partials accumulate in fp64 (groups of four terms in fp32 first)
// and every order is fixed by the index, so the result does not depend on
// scheduling.  A second, single-group launch adds up the partials: letting the
// group that finishes last do it inside the first launch needs a device-wide
// release per group, and the L2 write-back that implements it doubled the
// pass's duration (48 -> 94 us on 2^26 elements).  Plain (temporal) loads: the
// second pass reads the tensor again and should find it in cache if it fits.
constexpr int kSumBlock = 256;
constexpr uint64_t kSumChunk = 65536; // elements per work-group
constexpr int kSumBatch = 8;          // 16-byte loads a lane has in flight while it works on the previous 8
constexpr int kSumRounds = kSumChunk / 4 / kSumBlock / kSumBatch;
static_assert(kSumRounds * kSumBatch * kSumBlock * 4 == kSumChunk, "chunk is whole rounds");

// exp(x) for the terms of the sum: 2^n * 2^r with n = round(x log2 e) and
// r = x log2 e - n in [-0.5, 0.5] computed with two fused multiply-adds (log2 e
// split into a high and a low part), the hardware's exp2 for 2^r and ldexp for
// the scaling.  8 instructions instead of the 13 of the library's expf (which
// spends the difference on range checks); with those the pass was bound by
// instruction issue, not by memory.  The error is below 1.5 units in the last
// place; the total only enters the result through its fp32 rounding.
// Only n is computed from a clamped argument (so that it fits an integer; exp
// overflows above 88.73 and is 0 below -103.98 anyway); r uses x itself, so
// beyond the clamp r is huge and exp2 returns the infinity or the zero that is
// due, +-infinity included, and a NaN stays a NaN.
__device__ __forceinline__ float expTerm(float x) {
  const float kLog2eHi = 1.44269502162933349609375f; // fp32 nearest to log2 e
  const float kLog2eLo = 1.925963033500011e-8f;      // log2 e - kLog2eHi
  const float n = __builtin_rintf(__builtin_amdgcn_fmed3f(x, -104.0f, 89.0f) * kLog2eHi);
  float r = __builtin_fmaf(x, kLog2eHi, -n);
  r = __builtin_fmaf(x, kLog2eLo, r);
  return __builtin_amdgcn_ldexpf(__builtin_amdgcn_exp2f(r), static_cast<int>(n));
}

__device__ __forceinline__ double blockSum(double v, double* lds) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  if (lane == 0) lds[wave] = v;
  __syncthreads();
  double total = 0.0;
  if (threadIdx.x == 0)
    for (int w = 0; w < kSumBlock / 64; ++w) total += lds[w];
  return total; // valid in thread 0
}

__global__ __launch_bounds__(kSumBlock) void expSumKernel(const float* x, uint64_t n,
                                                          double* partial) {
  __shared__ double lds[kSumBlock / 64];
  const uint64_t begin = uint64_t(blockIdx.x) * kSumChunk;
  const uint64_t end = begin + kSumChunk < n ? begin + kSumChunk : n;
  double acc = 0.0;
  if ((reinterpret_cast<uintptr_t>(x) & 15u) == 0 && end - begin == kSumChunk) {
    const v4f* x4 = reinterpret_cast<const v4f*>(x + begin) + threadIdx.x;
    // the loads of round r+1 are issued before the exponentials of round r, so
    // a wave has memory requests in flight while it computes
    v4f v[2][kSumBatch];
#pragma unroll
    for (int u = 0; u < kSumBatch; ++u) v[0][u] = x4[u * kSumBlock];
#pragma unroll
    for (int r = 0; r < kSumRounds; ++r) {
      if (r + 1 < kSumRounds) {
#pragma unroll
        for (int u = 0; u < kSumBatch; ++u)
          v[(r + 1) & 1][u] = x4[((r + 1) * kSumBatch + u) * kSumBlock];
      }
#pragma unroll
      for (int u = 0; u < kSumBatch; ++u) {
        const v4f e = v[r & 1][u];
        // four terms are added in fp32 (two roundings, 1.2e-7 relative at worst),
        // everything above that in fp64
        acc += double((expTerm(e.x) + expTerm(e.y)) + (expTerm(e.z) + expTerm(e.w)));
      }
    }
  } else {
    for (uint64_t i = begin + threadIdx.x; i < end; i += kSumBlock) acc += double(expTerm(x[i]));
  }
  const double total = blockSum(acc, lds);
  if (threadIdx.x == 0) partial[blockIdx.x] = total;
}

// one work-group: total of the partials, rounded to fp32 once
__global__ __launch_bounds__(kSumBlock) void finishSumKernel(const double* partial,
                                                             uint64_t count, float* total) {
  __shared__ double lds[kSumBlock / 64];
  double acc = 0.0;
  for (uint64_t i = threadIdx.x; i < count; i += kSumBlock) acc += partial[i];
  const double t = blockSum(acc, lds);
  if (threadIdx.x == 0) total[0] = static_cast<float>(t);
}

// Both passes of fsoftmax with the caller's workspace: `partial` holds one
// fp64 per work-group of the sum pass, `total` one fp32.  Every slot that is
// read is written first, so the workspace needs no clearing.
int softmaxWithWorkspace(polar_hip_device* dev, const float* in, float* out, uint64_t n,
                         double* partial, float* total) {
  const uint64_t groups = (n + kSumChunk - 1) / kSumChunk;
  POLAR_HIP_TRY(hipSetDevice(dev->ordinal));
  POLAR_HIP_TRY(launchKernel(dev, expSumKernel, dim3(static_cast<unsigned>(groups)),
                             dim3(kSumBlock), in, n, partial));
  POLAR_HIP_TRY(launchKernel(dev, finishSumKernel, dim3(1), dim3(kSumBlock),
                             static_cast<const double*>(partial), groups, total));
  return launchEw<SoftmaxScaleOp>(dev, SoftmaxScaleOp{0.0f}, total, in, nullptr, out, n);
}

// Workspace of polar_hip_fsoftmax_static: lives in the code object's data
// segment, so every device that loads the library holds its own copy for the
// life of the process and no call ever allocates.  32768 partials cover 2^31
// elements (an 8 GiB tensor); 256 KiB + 256 B per device.
constexpr uint64_t kStaticSoftmaxMaxElements = 1ull << 31;
constexpr uint64_t kStaticSoftmaxMaxGroups = kStaticSoftmaxMaxElements / kSumChunk;
static __device__ __align__(256) unsigned char scratch[kStaticSoftmaxMaxGroups * sizeof(double) + 256];

} // namespace

// Called by polar_hip_device_open with the device current: the address of this
// device's copy of the scratch array.  The array's name is only a host-side
// handle for this lookup; kernels and copies use the address kept in the device.
int polar_hip_detail::resolveStaticScratch(polar_hip_device* dev) {
  void* address = nullptr;
  POLAR_HIP_TRY(hipGetSymbolAddress(&address, HIP_SYMBOL(scratch)));
  dev->softmaxScratch = address;
  return POLAR_HIP_OK;
}

extern "C" {

int polar_hip_fadd(polar_hip_device* dev, const float* a, float scaleA,
                   const float* b, float scaleB, float* c, uint64_t n) {
  POLAR_HIP_REQUIRE(dev != nullptr, "dev is null");
  POLAR_HIP_REQUIRE(n == 0 || (a && b && c), "null tensor");
  return launchEw<AddOp>(dev, AddOp{scaleA, scaleB}, nullptr, a, b, c, n);
}

int polar_hip_fmul(polar_hip_device* dev, const float* a, const float* b,
                   float* c, uint64_t n) {
  POLAR_HIP_REQUIRE(dev != nullptr, "dev is null");
  POLAR_HIP_REQUIRE(n == 0 || (a && b && c), "null tensor");
  return launchEw<MulOp>(dev, MulOp{}, nullptr, a, b, c, n);
}

int polar_hip_fdivide(polar_hip_device* dev, const float* numerator,
                      const float* denominator, float* out, uint64_t n) {
  POLAR_HIP_REQUIRE(dev != nullptr, "dev is null");
  POLAR_HIP_REQUIRE(n == 0 || (numerator && denominator && out), "null tensor");
  return launchEw<DivOp>(dev, DivOp{}, nullptr, numerator, denominator, out,
                            n);
}

int polar_hip_fsigmoid(polar_hip_device* dev, const float* in, float* out,
                       uint64_t n) {
  POLAR_HIP_REQUIRE(dev != nullptr, "dev is null");
  POLAR_HIP_REQUIRE(n == 0 || (in && out), "null tensor");
  return launchEw<SigmoidOp>(dev, SigmoidOp{}, nullptr, in, nullptr, out, n);
}

int polar_hip_flogloss(polar_hip_device* dev, const float* predicted,
                       const float* groundTruth, float* out, uint64_t n) {
  POLAR_HIP_REQUIRE(dev != nullptr, "dev is null");
  POLAR_HIP_REQUIRE(n == 0 || (predicted && groundTruth && out), "null tensor");
  return launchEw<LogLossOp>(dev, LogLossOp{}, nullptr, predicted,
                                groundTruth, out, n);
}

int polar_hip_fmulconcat(polar_hip_device* dev, const float* gradient,
                         const float* localDerivative, float* out, uint64_t n) {
  POLAR_HIP_REQUIRE(dev != nullptr, "dev is null");
  POLAR_HIP_REQUIRE(n == 0 || (gradient && localDerivative && out),
                    "null tensor");
  return launchEw<ScaleOp>(dev, ScaleOp{0.0f}, gradient, localDerivative,
                              nullptr, out, n);
}

int polar_hip_fcopy(polar_hip_device* dev, const float* src, float* dst,
                    uint64_t n) {
  POLAR_HIP_REQUIRE(dev != nullptr, "dev is null");
  POLAR_HIP_REQUIRE(n == 0 || (src && dst), "null tensor");
  return launchEw<CopyOp>(dev, CopyOp{}, nullptr, src, nullptr, dst, n);
}

int polar_hip_ffill(polar_hip_device* dev, float pattern, float* out,
                    uint64_t n) {
  POLAR_HIP_REQUIRE(dev != nullptr, "dev is null");
  POLAR_HIP_REQUIRE(n == 0 || out, "null tensor");
  return launchEw<FillOp, 256, 1>(dev, FillOp{pattern}, nullptr, nullptr, nullptr,
                             out, n);
}

int polar_hip_frelu(polar_hip_device* dev, const float* in, float* out, uint64_t n) {
  POLAR_HIP_REQUIRE(dev != nullptr, "dev is null");
  POLAR_HIP_REQUIRE(n == 0 || (in && out), "null tensor");
  return launchEw<ReluOp>(dev, ReluOp{}, nullptr, in, nullptr, out, n);
}

int polar_hip_fsoftmax(polar_hip_device* dev, const float* in, float* out, uint64_t n) {
  POLAR_HIP_REQUIRE(dev != nullptr, "dev is null");
  POLAR_HIP_REQUIRE(n == 0 || (in && out), "null tensor");
  if (n == 0) return POLAR_HIP_OK;
  const uint64_t groups = (n + kSumChunk - 1) / kSumChunk;
  POLAR_HIP_REQUIRE(groups < (1ull << 31), "tensor too large for one launch");
  // one fp64 partial per work-group in the device's workspace, the fp32 total
  // behind them
  std::lock_guard<std::mutex> g(dev->workspaceMu);
  void* area = nullptr;
  const int st = workspaceFor(dev, groups * sizeof(double) + sizeof(float), &area);
  if (st != POLAR_HIP_OK) return st;
  double* partial = static_cast<double*>(area);
  return softmaxWithWorkspace(dev, in, out, n, partial, reinterpret_cast<float*>(partial + groups));
}

int polar_hip_fsoftmax_static(polar_hip_device* dev, const float* in, float* out, uint64_t n) {
  POLAR_HIP_REQUIRE(dev != nullptr, "dev is null");
  POLAR_HIP_REQUIRE(n == 0 || (in && out), "null tensor");
  if (n == 0) return POLAR_HIP_OK;
  if (n > kStaticSoftmaxMaxElements)
    return fail(POLAR_HIP_ERR_INVALID,
                "polar_hip_fsoftmax_static: %llu elements exceed the limit of %llu "
                "(use polar_hip_fsoftmax)",
                static_cast<unsigned long long>(n),
                static_cast<unsigned long long>(kStaticSoftmaxMaxElements));
  POLAR_HIP_REQUIRE(dev->softmaxScratch != nullptr, "the device's scratch array was not resolved");
  // partials at the start of the array, the total at a fixed place behind them
  double* partial = static_cast<double*>(dev->softmaxScratch);
  float* total = reinterpret_cast<float*>(partial + kStaticSoftmaxMaxGroups);
  return softmaxWithWorkspace(dev, in, out, n, partial, total);
}

int polar_hip_fsigmoid_flogloss(polar_hip_device* dev, const float* in,
                                const float* groundTruth, float* out, uint64_t n) {
  POLAR_HIP_REQUIRE(dev != nullptr, "dev is null");
  POLAR_HIP_REQUIRE(n == 0 || (in && groundTruth && out), "null tensor");
  return launchEw<SigmoidLogLossOp>(dev, SigmoidLogLossOp{}, nullptr, in, groundTruth, out, n);
}

} // extern "C"
