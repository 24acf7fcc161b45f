// ftranspose for gfx950: out[j*rows + i] = in[i*cols + j].
//
// A work-group of 256 lanes moves one 64x64 tile through LDS.  Each wave reads
// whole 256-byte row segments of the input (lane = column) and, after the
// barrier, writes whole 256-byte row segments of the output (lane = input
// row), so both sides of HBM see full-width coalesced accesses.  The LDS tile
// has a row pitch of 65 words: a column read touches 64 different banks.  All
// 16 loads of a lane are issued before the first LDS store.  Edge tiles are
// predicated per element, so any rows x cols works (neither needs to be a
// multiple of anything).
#include "internal.h"

using namespace polar_hip_detail;

namespace {

constexpr int kTile = 64;
constexpr int kThreads = 256;
constexpr int kRowsPerPass = kThreads / kTile; // 4
constexpr int kPasses = kTile / kRowsPerPass;  // 16

__global__ __launch_bounds__(kThreads) void transposeKernel(
    const float* __restrict__ in, float* __restrict__ out, uint64_t rows,
    uint64_t cols, uint32_t tilesX, uint64_t numTiles) {
  __shared__ float tile[kTile][kTile + 1];
  const int tx = threadIdx.x % kTile;
  const int ty = threadIdx.x / kTile;
  for (uint64_t t = blockIdx.x; t < numTiles; t += gridDim.x) {
    const uint64_t i0 = (t / tilesX) * kTile; // input row of the tile
    const uint64_t j0 = (t % tilesX) * kTile; // input column of the tile
    float v[kPasses];
    const bool inner = i0 + kTile <= rows && j0 + kTile <= cols;
    if (inner) {
#pragma unroll
      for (int p = 0; p < kPasses; ++p) {
        const uint64_t r = i0 + ty + p * kRowsPerPass;
        v[p] = __builtin_nontemporal_load(&in[r * cols + j0 + tx]);
      }
    } else {
#pragma unroll
      for (int p = 0; p < kPasses; ++p) {
        const uint64_t r = i0 + ty + p * kRowsPerPass;
        v[p] = (r < rows && j0 + tx < cols)
                   ? __builtin_nontemporal_load(&in[r * cols + j0 + tx])
                   : 0.0f;
      }
    }
#pragma unroll
    for (int p = 0; p < kPasses; ++p) tile[ty + p * kRowsPerPass][tx] = v[p];
    __syncthreads();
    if (inner) {
#pragma unroll
      for (int p = 0; p < kPasses; ++p) {
        const int c = ty + p * kRowsPerPass; // input column = output row
        __builtin_nontemporal_store(tile[tx][c],
                                    &out[(j0 + c) * rows + i0 + tx]);
      }
    } else {
#pragma unroll
      for (int p = 0; p < kPasses; ++p) {
        const int c = ty + p * kRowsPerPass;
        if (j0 + c < cols && i0 + tx < rows)
          __builtin_nontemporal_store(tile[tx][c],
                                      &out[(j0 + c) * rows + i0 + tx]);
      }
    }
    __syncthreads();
  }
}

} // namespace

extern "C" int polar_hip_ftranspose(polar_hip_device* dev, const float* in,
                                    float* out, uint64_t rows, uint64_t cols) {
  POLAR_HIP_REQUIRE(dev != nullptr, "dev is null");
  if (rows == 0 || cols == 0) return POLAR_HIP_OK;
  POLAR_HIP_REQUIRE(in != nullptr && out != nullptr, "null tensor");
  POLAR_HIP_REQUIRE(in != out, "in-place transpose is not supported");
  const uint64_t tilesX = (cols + kTile - 1) / kTile;
  const uint64_t tilesY = (rows + kTile - 1) / kTile;
  POLAR_HIP_REQUIRE(tilesX < (1ull << 31), "too many columns");
  const uint64_t numTiles = tilesX * tilesY;
  uint64_t grid = numTiles;
  if (grid > (1u << 22)) grid = 1u << 22;
  POLAR_HIP_TRY(hipSetDevice(dev->ordinal));
  POLAR_HIP_TRY(launchKernel(dev, transposeKernel,
                             dim3(static_cast<unsigned>(grid)), dim3(kThreads),
                             in, out, rows, cols, static_cast<uint32_t>(tilesX),
                             numTiles));
  return POLAR_HIP_OK;
}
