// ftranspose for gfx950: out[j*rows + i] = in[i*cols + j].
//
// The operation is pure data movement, so the kernel is shaped by what HBM and
// the L2s like, measured on a 12345 x 6789 matrix (neither pitch is a multiple
// of a cache line):
//
//  * Writes that cover only part of a 128-byte line are expensive (a plain
//    64x64-tile kernel drops from 5.2 TB/s on a line-aligned shape to 2.5 TB/s
//    on this one, and the write side accounts for most of it).  So the output
//    is cut into 128-byte chunks that are aligned IN MEMORY, not in index
//    space: for output row j the chunk boundaries sit at the i for which
//    (j*rows + i) % 32 == 0, i.e. at b_j + 32m with b_j = (-j*rows) mod 32.
//    Every half-wave store then writes one whole line; only the first and last
//    chunk of an output row can be partial.
//  * Because b_j differs from row to row, the output rows of a work-group need
//    input rows from a window that is up to 63 rows tall.  The group therefore
//    walks down a strip of the input, 32 rows per step, keeping the last two
//    32 x 128 tiles in an LDS ring; step m emits, for every output row, the
//    aligned chunk that ends inside tile m.  Each input element is read once
//    per strip (plus one extra tile at the strip's end).
//  * Input row segments are not line-aligned either, so neighbouring column
//    tiles share cache lines.  Work-groups are numbered so that each XCD owns
//    a contiguous range of column tiles and walks them together: the shared
//    lines then mostly hit in that XCD's L2 instead of being fetched twice.
//    For the same reason the loads are plain, not non-temporal (4.7 -> 5.1
//    TB/s); the stores, which never share a line, stay non-temporal.
//  * Shape, measured with rotated buffers on 12345 x 6789 (and seven other
//    shapes from 333 x 777 to 16384^2): column tiles of 128 with 512 lanes and
//    strips of 64 rows, 128-130 us (125.5-126.5 us with the interior path); 256 columns with 1024 lanes and strips of
//    512 rows (fewer, longer-lived groups), 134 us, and 114 instead of 78 us on
//    50000 x 1000; strips of 32 rows 151 us (every tile is then read twice);
//    two tiles in flight per lane instead of one (the tile two steps ahead
//    fetched into a second register set) 150 us, 132-135 us with strips of
//    128-256 rows: more outstanding requests make this pattern slower;
//    numbering the groups strips-first instead of column-tiles-first 131-138
//    us.  Only 16384^2 prefers the long strips (445 against 482 us).  The
//    strip's last tile is read by the next strip as well; that second read
//    is served by the L2 both groups share.
//  * 512 lanes per group (8 waves): 8 loads per lane in flight, and 16 output
//    rows per wave in the store phase, two per wave-wide store.  The ring is
//    33 KB, so four groups share a CU.
//
// The LDS ring has a row pitch of 129 words, so both the row-wise stores of the
// load phase and the column-wise loads of the store phase are conflict-free
// within a half-wave.  All edges are predicated; any rows x cols works.
#include "internal.h"

using namespace polar_hip_detail;

namespace {

constexpr int kTI = 32;   // input rows per step = elements per aligned output chunk
constexpr int kTJ = 128;  // input columns (= output rows) per work-group
constexpr int kThreads = 512;
constexpr int kWaves = kThreads / 64;
constexpr int kLoads = kTI * kTJ / kThreads;    // 8 loads per lane per tile
constexpr int kColsPerStore = 64 / kTI;         // 2 output rows per wave-wide store
constexpr int kStores = kTJ / (kWaves * kColsPerStore); // 8 stores per lane per step
constexpr int kXcds = 8;

struct TransposeArgs {
  const float* in;
  float* out;
  uint32_t rows, cols;
  uint32_t colTiles;        // ceil(cols / kTJ)
  uint32_t colTilesPerXcd;  // colTiles / 8: the column tiles every XCD owns outright
  uint32_t sharedTiles;     // colTiles % 8: the rest, whose strips are dealt out to the XCDs
  uint32_t ownedGroups;     // groups per XCD for the tiles it owns (strips rounded up to whole runs)
  uint32_t stripsPerXcd;    // ceil(strips / 8): an XCD's share of the strips of the shared tiles
  uint32_t strips;          // ceil(rows / stripRows)
  uint32_t stripRows;       // multiple of kTI
  uint32_t fastOffsets;     // rows * cols < 2^31: element offsets fit 32 bits
  uint32_t run;             // strips of one column tile that are numbered consecutively
};

__global__ __launch_bounds__(kThreads) void transposeKernel(TransposeArgs p) {
  __shared__ float ring[2 * kTI][kTJ + 1];

  // XCD x (work-groups with id % 8 == x) owns column tiles
  // [x*perXcd, (x+1)*perXcd) and walks them fastest, in runs of p.run strips
  // per column tile (1: column tiles fastest).  The colTiles % 8 tiles that are
  // left over are shared: every XCD takes an eighth of their strips, so that
  // all XCDs finish together (with 54 column tiles dealt out whole, seven XCDs
  // would hold 7 and the eighth 5, idle for the last 2/7 of the launch).
  const uint32_t xcd = blockIdx.x % kXcds, local = blockIdx.x / kXcds;
  uint32_t colTile, strip;
  if (local < p.ownedGroups) {
    const uint32_t perRun = p.run * p.colTilesPerXcd;
    const uint32_t inRun = local % perRun;
    colTile = xcd * p.colTilesPerXcd + inRun / p.run;
    strip = local / perRun * p.run + inRun % p.run;
    if (strip >= p.strips) return; // the padding of the last run; before any barrier
  } else {
    const uint32_t rest = local - p.ownedGroups; // < sharedTiles * stripsPerXcd
    colTile = kXcds * p.colTilesPerXcd + rest % p.sharedTiles;
    strip = xcd * p.stripsPerXcd + rest / p.sharedTiles;
    if (strip >= p.strips) return;
  }

  const uint32_t R = p.rows, C = p.cols;
  const uint32_t j0 = colTile * kTJ;
  const uint32_t i0 = strip * p.stripRows;
  const uint32_t i1 = i0 + p.stripRows < R ? i0 + p.stripRows : R;
  const bool lastStrip = i1 == R;
  // tiles 0..lastTile are loaded; the final one only feeds the chunks that
  // straddle the end of the strip
  const uint32_t lastTile = lastStrip ? (R - i0 + kTI - 1) / kTI : (i1 - i0) / kTI;

  const int t = threadIdx.x;
  const int wave = t / 64, lane = t % 64;
  const int sub = lane / kTI, l = lane % kTI;

  // Strips and column tiles that lie wholly inside the matrix, away from its
  // first and last rows (nearly all of them), need no bounds checks, and with
  // fewer than 2^31 elements every address is a scalar base plus a 32-bit lane
  // offset that does not change from step to step.  The general code below
  // spends about 30 vector instructions per element on 64-bit addresses and
  // predicates, and the kernel's duration follows that count (8 more per
  // element: +7 us on 12345 x 6789); this path needs 4.
  if (p.fastOffsets && i0 != 0 && uint64_t(i0) + p.stripRows + kTI <= R && j0 + kTJ <= C) {
    float* const flat = &ring[0][0];
    constexpr uint32_t kPitch = kTJ + 1;
    uint32_t loadOff[kLoads], ringWrite[kLoads], storeOff[kStores], ringOdd[kStores], ringEven[kStores];
#pragma unroll
    for (int q = 0; q < kLoads; ++q) {
      const uint32_t e = uint32_t(t) + uint32_t(q) * kThreads;
      const uint32_t row = e / kTJ, col = e % kTJ;
      loadOff[q] = row * C + col;
      ringWrite[q] = row * kPitch + col;
    }
#pragma unroll
    for (int q = 0; q < kStores; ++q) {
      const uint32_t c = uint32_t(wave) * kColsPerStore + uint32_t(sub) + uint32_t(q) * (kWaves * kColsPerStore);
      const uint32_t rowBase = (j0 + c) * R; // < 2^31
      const uint32_t b = (kTI - (rowBase & (kTI - 1))) & (kTI - 1);
      const uint32_t bl = b + uint32_t(l); // 0 .. 62: ring row of the element at odd steps
      storeOff[q] = rowBase + bl;
      ringOdd[q] = bl * kPitch + c;
      ringEven[q] = (bl ^ uint32_t(kTI)) * kPitch + c; // (bl + 32) mod 64
    }
    const uint32_t steps = p.stripRows / kTI; // tiles 0 .. steps are loaded
    const float* src = p.in + uint64_t(i0) * C + j0; // scalar; one tile further per step
    float w[kLoads];
#pragma unroll
    for (int q = 0; q < kLoads; ++q) w[q] = src[loadOff[q]];
    for (uint32_t m = 0; m <= steps; ++m) {
      float* const half = flat + (m & 1) * (kTI * kPitch);
#pragma unroll
      for (int q = 0; q < kLoads; ++q) half[ringWrite[q]] = w[q];
      __syncthreads();
      if (m < steps) {
        src += uint64_t(kTI) * C;
#pragma unroll
        for (int q = 0; q < kLoads; ++q) w[q] = src[loadOff[q]];
      }
      if (m != 0) {
        // chunks [i0 + 32(m-1) + b, i0 + 32m + b) of the group's 128 output rows
        float* const dst = p.out + (uint64_t(i0) + uint64_t(kTI) * (m - 1)); // scalar
        if (m & 1) {
#pragma unroll
          for (int q = 0; q < kStores; ++q) __builtin_nontemporal_store(flat[ringOdd[q]], dst + storeOff[q]);
        } else {
#pragma unroll
          for (int q = 0; q < kStores; ++q) __builtin_nontemporal_store(flat[ringEven[q]], dst + storeOff[q]);
        }
      }
      __syncthreads(); // the older half is overwritten by the next step
    }
    return;
  }

  float v[kLoads];
  auto loadTile = [&](uint32_t m) {
#pragma unroll
    for (int q = 0; q < kLoads; ++q) {
      const int e = t + q * kThreads;
      const int row = e / kTJ, col = e % kTJ;
      const uint64_t r = uint64_t(i0) + uint64_t(m) * kTI + row;
      // plain (temporal) load: the lines shared with the neighbouring column
      // tile must stay in L2 until that tile's group has read them
      v[q] = (r < R && j0 + col < C) ? p.in[r * C + j0 + col] : 0.0f;
    }
  };

  loadTile(0);
  for (uint32_t m = 0; m <= lastTile; ++m) {
    const int half = (m & 1) * kTI;
#pragma unroll
    for (int q = 0; q < kLoads; ++q) {
      const int e = t + q * kThreads;
      ring[half + e / kTJ][e % kTJ] = v[q];
    }
    __syncthreads();
    if (m < lastTile) loadTile(m + 1); // in flight during the store phase

    // Store phase: output row j0+c gets the aligned chunk that ends in tile m,
    // i in [i0 + 32(m-1) + b, i0 + 32m + b), clipped to what this strip owns.
#pragma unroll
    for (int q = 0; q < kStores; ++q) {
      const int c = wave * kColsPerStore + sub + q * (kWaves * kColsPerStore);
      const uint32_t j = j0 + c;
      const uint64_t rowBase = uint64_t(j) * R;
      const uint32_t b = uint32_t((kTI - (rowBase & (kTI - 1))) & (kTI - 1));
      const int64_t first = int64_t(i0) + int64_t(kTI) * (int64_t(m) - 1) + b;
      const int64_t own0 = i0 == 0 ? 0 : int64_t(i0) + b;
      const int64_t own1 = lastStrip ? int64_t(R) : int64_t(i1) + b;
      const int64_t i = first + l;
      if (j < C && i >= own0 && i < own1 && i < int64_t(R)) {
        const float val = ring[uint32_t(i - i0) & (2 * kTI - 1)][c];
        __builtin_nontemporal_store(val, &p.out[rowBase + uint64_t(i)]);
      }
    }
    __syncthreads(); // the older half is overwritten by the next step
  }
}

} // namespace

extern "C" int polar_hip_ftranspose(polar_hip_device* dev, const float* in,
                                    float* out, uint64_t rows, uint64_t cols) {
  POLAR_HIP_REQUIRE(dev != nullptr, "dev is null");
  if (rows == 0 || cols == 0) return POLAR_HIP_OK;
  POLAR_HIP_REQUIRE(in != nullptr && out != nullptr, "null tensor");
  POLAR_HIP_REQUIRE(in != out, "in-place transpose is not supported");
  POLAR_HIP_REQUIRE(rows < (1ull << 31) && cols < (1ull << 31),
                    "dimension does not fit 31 bits");
  TransposeArgs p;
  p.in = in;
  p.out = out;
  p.rows = static_cast<uint32_t>(rows);
  p.cols = static_cast<uint32_t>(cols);
  p.colTiles = (p.cols + kTJ - 1) / kTJ;
  p.colTilesPerXcd = p.colTiles / kXcds;
  p.sharedTiles = p.colTiles % kXcds;
  // Strips of 64 rows, shorter when that is needed to give every CU two groups.
  const uint64_t wanted = 2ull * static_cast<uint64_t>(dev->info.compute_units);
  uint32_t stripRows = 64;
  while (stripRows > kTI &&
         uint64_t(p.colTiles) * ((p.rows + stripRows - 1) / stripRows) < wanted)
    stripRows /= 2;
  p.stripRows = stripRows;
  p.fastOffsets = rows * cols < (1ull << 31) ? 1u : 0u;
  p.strips = (p.rows + stripRows - 1) / stripRows;
  // Column tiles fastest, unless the output's row pitch is a large power-of-two
  // multiple: a group's 128 output rows then map to the same few memory
  // channels, and numbering 16 strips of a column tile consecutively (groups
  // that run together then write neighbouring pieces of the same output rows)
  // measured 16384^2 495 -> 410 us, 8192 x 6789 92 -> 83 us, 12288^2 253 -> 229
  // us; with an odd pitch (12345 x 6789) runs cost 1-3 %.
  p.run = (p.rows % 2048 == 0 && p.rows >= 8192) ? 16 : 1;
  const uint64_t owned = uint64_t(p.colTilesPerXcd) * ((p.strips + p.run - 1) / p.run * p.run);
  p.stripsPerXcd = (p.strips + kXcds - 1) / kXcds;
  const uint64_t grid = uint64_t(kXcds) * (owned + uint64_t(p.sharedTiles) * p.stripsPerXcd);
  POLAR_HIP_REQUIRE(owned < (1ull << 31), "matrix too large for one launch");
  p.ownedGroups = static_cast<uint32_t>(owned);
  POLAR_HIP_REQUIRE(grid < (1ull << 31), "matrix too large for one launch");
  POLAR_HIP_TRY(hipSetDevice(dev->ordinal));
  POLAR_HIP_TRY(launchKernel(dev, transposeKernel,
                             dim3(static_cast<unsigned>(grid)), dim3(kThreads), p));
  return POLAR_HIP_OK;
}
