// fconv2d and fpool for gfx950: the two builtins with a 2-D neighbourhood.
//
// Both are HBM-bound (a 3x3 correlation is 18 flops per 8 bytes), so what
// matters is that every input line is fetched once and every output line is
// written whole:
//
//  * Output rows are cut into 256-element segments that are aligned IN MEMORY:
//    for output row y the segment boundaries sit where (base + y*OW + x) is a
//    multiple of 32 floats, i.e. the segments of row y are shifted left by
//    s_y = (base + y*OW) mod 32 columns.  A wave-wide store then always covers
//    whole 128-byte lines, whatever OW is; only the first and last segment of
//    a row are partial.  A work-group owns 256 such (skewed) columns of a band
//    of output rows, one column per lane.
//  * fconv2d stages the input window of its band in LDS (band rows + KH-1 halo
//    rows, 256 + 31 skew columns + KW-1 halo columns) and reads the taps from
//    there; the accumulation is the reference's: fp32, a outer / b inner,
//    product rounded before the add (the file is compiled with
//    -ffp-contract=off).  3x3 and 5x5 are compiled with constant bounds.
//  * fpool reads its windows straight from memory: with stride >= window each
//    input element is used once, and the lanes of a wave walk consecutive
//    windows, so the lines they touch are consumed completely by that wave.
#include "internal.h"

using namespace polar_hip_detail;

namespace {

constexpr int kSegment = 256; // output columns per work-group = lanes
constexpr int kLine = 32;     // floats per 128-byte line
constexpr int kConvRows = 32; // output rows per fconv2d work-group
constexpr int kPoolRows = 8;  // output rows per fpool work-group
constexpr uint32_t kMaxConvLds = 64 * 1024;

// columns the segments of output row y are shifted left by
__device__ __forceinline__ uint32_t rowShift(uint32_t y, uint32_t ow, uint32_t basePhase) {
  return ((y % kLine) * (ow % kLine) + basePhase) % kLine;
}

struct ConvArgs {
  const float* in;
  const float* weights;
  float* out;
  uint32_t H, W, KH, KW, OH, OW;
  uint32_t colTiles;
  uint32_t outPhase; // (address of out / 4) mod 32
};

// KH_/KW_ == 0: the kernel size comes from the arguments.
template <int KH_, int KW_>
__global__ __launch_bounds__(kSegment) void conv2dKernel(ConvArgs p) {
  extern __shared__ float tile[];
  const uint32_t KH = KH_ ? KH_ : p.KH, KW = KW_ ? KW_ : p.KW;
  const uint32_t ct = blockIdx.x % p.colTiles, rt = blockIdx.x / p.colTiles;
  const uint32_t y0 = rt * kConvRows;
  const uint32_t rowsOut = p.OH - y0 < uint32_t(kConvRows) ? p.OH - y0 : uint32_t(kConvRows);
  const uint32_t rowsIn = rowsOut + KH - 1; // all inside the input: OH = H - KH + 1
  const uint32_t pitch = kSegment + (kLine - 1) + KW - 1;
  // input column held in tile column 0 (may be negative in the first segment)
  const int64_t x0 = int64_t(ct) * kSegment - (kLine - 1);

  const uint32_t t = threadIdx.x, wave = t / 64, lane = t % 64;
  for (uint32_t row = wave; row < rowsIn; row += kSegment / 64) {
    const float* src = p.in + uint64_t(y0 + row) * p.W;
    for (uint32_t col = lane; col < pitch; col += 64) {
      const int64_t xi = x0 + col;
      tile[row * pitch + col] = (xi >= 0 && xi < int64_t(p.W)) ? src[xi] : 0.0f;
    }
  }
  __syncthreads();

  for (uint32_t r = 0; r < rowsOut; ++r) {
    const uint32_t y = y0 + r;
    const uint32_t shift = rowShift(y, p.OW, p.outPhase);
    const int64_t x = int64_t(ct) * kSegment - shift + t;
    if (x >= 0 && x < int64_t(p.OW)) {
      const float* win = tile + r * pitch + (t + (kLine - 1) - shift);
      float acc = 0.0f;
      for (uint32_t a = 0; a < KH; ++a)
        for (uint32_t b = 0; b < KW; ++b)
          acc = win[a * pitch + b] * p.weights[a * KW + b] + acc;
      __builtin_nontemporal_store(acc, &p.out[uint64_t(y) * p.OW + uint64_t(x)]);
    }
  }
}

// Any kernel size: taps straight from memory (used when the LDS window of the
// tiled kernel would not fit).
__global__ __launch_bounds__(kSegment) void conv2dDirectKernel(ConvArgs p) {
  const uint32_t ct = blockIdx.x % p.colTiles, y = blockIdx.x / p.colTiles;
  const uint32_t shift = rowShift(y, p.OW, p.outPhase);
  const int64_t x = int64_t(ct) * kSegment - shift + threadIdx.x;
  if (x < 0 || x >= int64_t(p.OW)) return;
  float acc = 0.0f;
  for (uint32_t a = 0; a < p.KH; ++a) {
    const float* src = p.in + uint64_t(y + a) * p.W + uint64_t(x);
    for (uint32_t b = 0; b < p.KW; ++b) acc = src[b] * p.weights[a * p.KW + b] + acc;
  }
  __builtin_nontemporal_store(acc, &p.out[uint64_t(y) * p.OW + uint64_t(x)]);
}

struct PoolArgs {
  const float* in;
  float* out;
  uint32_t H, W, win0, win1, stride0, stride1, OH, OW;
  uint32_t colTiles;
  uint32_t outPhase;
};

__global__ __launch_bounds__(kSegment) void poolKernel(PoolArgs p) {
  const uint32_t ct = blockIdx.x % p.colTiles, rt = blockIdx.x / p.colTiles;
  const uint32_t y0 = rt * kPoolRows;
  const uint32_t rows = p.OH - y0 < uint32_t(kPoolRows) ? p.OH - y0 : uint32_t(kPoolRows);
  for (uint32_t r = 0; r < rows; ++r) {
    const uint32_t y = y0 + r;
    const uint32_t shift = rowShift(y, p.OW, p.outPhase);
    const int64_t x = int64_t(ct) * kSegment - shift + threadIdx.x;
    if (x >= 0 && x < int64_t(p.OW)) {
      // utils/dialects/lib/PolarGraph/kernels/Pool2DOp.cpp:50-52,74-76: starts
      // at -10e5, strict ordered greater-than
      float best = -10e5f;
      const float* corner =
          p.in + uint64_t(y) * p.stride0 * p.W + uint64_t(x) * p.stride1;
      for (uint32_t a = 0; a < p.win0; ++a) {
        const float* src = corner + uint64_t(a) * p.W;
        for (uint32_t b = 0; b < p.win1; ++b) {
          const float v = src[b];
          best = v > best ? v : best;
        }
      }
      __builtin_nontemporal_store(best, &p.out[uint64_t(y) * p.OW + uint64_t(x)]);
    }
  }
}

uint32_t phaseOf(const float* out) {
  return static_cast<uint32_t>((reinterpret_cast<uintptr_t>(out) / sizeof(float)) % kLine);
}

} // namespace

extern "C" {

int polar_hip_fconv2d(polar_hip_device* dev, const float* in, const float* kernel,
                      float* out, uint64_t height, uint64_t width,
                      uint64_t kernelHeight, uint64_t kernelWidth) {
  POLAR_HIP_REQUIRE(dev != nullptr, "dev is null");
  POLAR_HIP_REQUIRE(kernelHeight >= 1 && kernelWidth >= 1, "empty convolution kernel");
  // the reference's tap loops run over [-K/2, K/2]: only odd sizes are defined
  POLAR_HIP_REQUIRE(kernelHeight % 2 == 1 && kernelWidth % 2 == 1,
                    "convolution kernel sizes must be odd");
  POLAR_HIP_REQUIRE(height >= kernelHeight && width >= kernelWidth,
                    "convolution kernel larger than the input");
  POLAR_HIP_REQUIRE(in && kernel && out, "null tensor");
  POLAR_HIP_REQUIRE(in != out, "in-place convolution is not supported");
  POLAR_HIP_REQUIRE(height < (1ull << 31) && width < (1ull << 31),
                    "dimension does not fit 31 bits");
  ConvArgs p;
  p.in = in;
  p.weights = kernel;
  p.out = out;
  p.H = static_cast<uint32_t>(height);
  p.W = static_cast<uint32_t>(width);
  p.KH = static_cast<uint32_t>(kernelHeight);
  p.KW = static_cast<uint32_t>(kernelWidth);
  p.OH = p.H - p.KH + 1;
  p.OW = p.W - p.KW + 1;
  p.colTiles = (p.OW + (kLine - 1) + kSegment - 1) / kSegment;
  p.outPhase = phaseOf(out);
  POLAR_HIP_TRY(hipSetDevice(dev->ordinal));
  const uint64_t ldsBytes = uint64_t(kConvRows + p.KH - 1) *
                            (kSegment + (kLine - 1) + p.KW - 1) * sizeof(float);
  if (ldsBytes <= kMaxConvLds) {
    const uint64_t grid = uint64_t(p.colTiles) * ((p.OH + kConvRows - 1) / kConvRows);
    POLAR_HIP_REQUIRE(grid < (1ull << 31), "tensor too large for one launch");
    auto fn = p.KH == 3 && p.KW == 3   ? conv2dKernel<3, 3>
              : p.KH == 5 && p.KW == 5 ? conv2dKernel<5, 5>
                                       : conv2dKernel<0, 0>;
    POLAR_HIP_TRY(launchKernelLds(dev, fn, dim3(static_cast<unsigned>(grid)),
                                  dim3(kSegment), static_cast<uint32_t>(ldsBytes), p));
  } else {
    const uint64_t grid = uint64_t(p.colTiles) * p.OH;
    POLAR_HIP_REQUIRE(grid < (1ull << 31), "tensor too large for one launch");
    POLAR_HIP_TRY(launchKernel(dev, conv2dDirectKernel,
                               dim3(static_cast<unsigned>(grid)), dim3(kSegment), p));
  }
  return POLAR_HIP_OK;
}

int polar_hip_fpool(polar_hip_device* dev, const float* in, float* out,
                    uint64_t height, uint64_t width, uint64_t window0,
                    uint64_t window1, uint64_t stride0, uint64_t stride1) {
  POLAR_HIP_REQUIRE(dev != nullptr, "dev is null");
  POLAR_HIP_REQUIRE(window0 >= 1 && window1 >= 1, "empty pooling window");
  POLAR_HIP_REQUIRE(stride0 >= 1 && stride1 >= 1, "pooling stride must be positive");
  POLAR_HIP_REQUIRE(height >= window0 && width >= window1,
                    "pooling window larger than the input");
  POLAR_HIP_REQUIRE(in && out, "null tensor");
  POLAR_HIP_REQUIRE(in != out, "in-place pooling is not supported");
  POLAR_HIP_REQUIRE(height < (1ull << 31) && width < (1ull << 31),
                    "dimension does not fit 31 bits");
  PoolArgs p;
  p.in = in;
  p.out = out;
  p.H = static_cast<uint32_t>(height);
  p.W = static_cast<uint32_t>(width);
  p.win0 = static_cast<uint32_t>(window0);
  p.win1 = static_cast<uint32_t>(window1);
  p.stride0 = static_cast<uint32_t>(stride0 < height ? stride0 : height);
  p.stride1 = static_cast<uint32_t>(stride1 < width ? stride1 : width);
  // src/operation/internal/Pool2DOperationInternal.cpp:37-41
  p.OH = (p.H - p.win0) / p.stride0 + 1;
  p.OW = (p.W - p.win1) / p.stride1 + 1;
  p.colTiles = (p.OW + (kLine - 1) + kSegment - 1) / kSegment;
  p.outPhase = phaseOf(out);
  const uint64_t grid = uint64_t(p.colTiles) * ((p.OH + kPoolRows - 1) / kPoolRows);
  POLAR_HIP_REQUIRE(grid < (1ull << 31), "tensor too large for one launch");
  POLAR_HIP_TRY(hipSetDevice(dev->ordinal));
  POLAR_HIP_TRY(launchKernel(dev, poolKernel, dim3(static_cast<unsigned>(grid)),
                             dim3(kSegment), p));
  return POLAR_HIP_OK;
}

} // extern "C"
