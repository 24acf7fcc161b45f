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
//    Measured on an 8192^2 image, 3x3, buffers rotated (537 MB per launch; a
//    plain copy of that size takes 80 us): 89 us (93 us before the staging by
//    vectors, the unchecked interior stores, the offset LDS reads and the
//    explicit wait described at those places).  HBM traffic is 1.002 x the
//    algorithmic bytes and the LDS reads are free of bank conflicts; the
//    counters show the waves parked at the barrier, waiting for the window,
//    for most of their life (with the arithmetic removed the kernel still
//    takes 88 us).  Shapes that measured slower than this one: four
//    adjacent outputs per lane with one 16-byte store (115 us with the window
//    row-major, 111 us with the window kept as four interleaved quarters so
//    that the reads stay conflict-free, 16-byte staging loads), no LDS at all
//    (a lane fetching its own KW+3 inputs per tap row: 98-110 us), a resident
//    grid of groups that prefetch their next band into registers while they
//    compute (116 us in row-major band order, 152 us walking down strips; two
//    bands per group, one below the other, the second window on its way into
//    registers while the first is computed: 97 us against 89), a
//    window per wave instead of per group, without any group barrier and with
//    the first output rows computed while the later window rows are still in
//    flight (105-142 us for 2-8 rows per wave), 16 or more rows per band
//    (96-115 us); 8 to 12 rows measured the same then, and with the leaner
//    row loop 8 rows are 2 % ahead of 12 (87.5 against 89.5 us; 6 rows 91.5,
//    4 rows 109).  Also slower: no LDS and no barrier at all — a wave walking
//    down 32-64 rows of 256 columns, each image row fetched once with one
//    16-byte load per lane, the two columns to the right of a lane's four taken
//    from the next lane (wave_shl), three rows of partial sums in registers,
//    three to six rows of fetches in flight with exact vmcnt waits, one 16-byte
//    store per lane and row: bit-exact, 20 vector instructions per output, and
//    118-180 us.  Its fetches alone take 48 us and its stores alone 68-80 us
//    (a plain fill of that size takes 38), and the two add up instead of
//    overlapping: vmcnt counts loads and stores in order, so a wave that waits
//    for a fetch also waits for every store it issued before it.
//  * fpool reads its windows straight from memory: with stride >= window each
//    input element is used once, and the lanes of a wave walk consecutive
//    windows, so the lines they touch are consumed completely by that wave.
//    Non-overlapping 2x2 and 4x4 windows have a kernel of their own that takes
//    a window row per vector load and issues a whole band's loads at once.
//    Short bands are better (8192^2, 2x2, buffers rotated: 61.7 / 55.7 / 57.1 /
//    58.7 / 60.3 us for 1 / 2 / 4 / 8 / 16 rows per group; four input streams
//    merged into one output stream at full vector width take 54 us for the
//    same bytes).  Every other window and stride whose band fits 24 KB of LDS
//    is staged like the convolution (poolStagedKernel; 8192^2, rotated: 3x3
//    stride 2 148 -> 78-83 us, 3x3 stride 1 430 -> 119 us, 2x2 stride 1 281 ->
//    91 us against one vector-memory instruction per tap before), and with
//    16-byte loads where the image rows start on 16 bytes (3x3 stride 2 -> 56
//    us, 3x3 stride 1 -> 106 us, 5x5 stride 2 162 -> 111 us); larger windows
//    fall back to taps from memory.  Bands stay short here too: with LDS for
//    eight output rows where 24 KB hold fewer, 3x3 stride 2 takes 61 us
//    instead of 56, 3x3 stride 3 59-65 instead of 54, 5x5 stride 2 109
//    instead of 106.  Streaming stores with or without the device-scope
//    write-through measure the same in both staged kernels.
#include "internal.h"

#include <type_traits>
#include <utility>

using namespace polar_hip_detail;

namespace {

typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kSegment = 256; // output columns per work-group = lanes
constexpr int kLine = 32;     // floats per 128-byte line
constexpr int kConvRows = 8;  // output rows per fconv2d work-group
constexpr int kPoolRows = 2;  // output rows per fpool work-group
constexpr uint32_t kMaxConvLds = 64 * 1024;
constexpr int kWaitVmcnt0 = 0x0F70; // s_waitcnt vmcnt(0) with the other counters left alone
constexpr uint32_t kMaxPoolLds = 24 * 1024; // window of the staged fpool kernel: six groups per CU
constexpr uint32_t kPoolStagedRows = 12;    // output rows per group of that kernel, at most

// Work-group id -> tile index such that each XCD (ids equal modulo 8 share
// one) works through a contiguous range of tiles: neighbouring tiles, which
// share halo rows and columns, then meet in the same L2.  Returns false for
// the padding groups at the end of the grid.
constexpr uint32_t kXcds = 8;
__device__ __forceinline__ bool tileOfGroup(uint32_t tiles, uint32_t* tile) {
  const uint32_t perXcd = (tiles + kXcds - 1) / kXcds;
  *tile = (blockIdx.x % kXcds) * perXcd + blockIdx.x / kXcds;
  return blockIdx.x / kXcds < perXcd && *tile < tiles;
}
uint64_t paddedGrid(uint64_t tiles) { return (tiles + kXcds - 1) / kXcds * kXcds; }

// columns the segments of output row y are shifted left by
__device__ __forceinline__ uint32_t rowShift(uint32_t y, uint32_t ow, uint32_t basePhase) {
  return ((y % kLine) * (ow % kLine) + basePhase) % kLine;
}

struct ConvArgs {
  const float* in;
  const float* weights;
  float* out;
  uint32_t H, W, KH, KW, OH, OW;
  uint32_t colTiles, tiles;
  uint32_t outPhase; // (address of out / 4) mod 32
};

// Columns of the staged window: the 256 + 31 + KW - 1 the band needs and, when
// the image rows start on 16 bytes (VEC), one more in front and padding to a
// whole number of 16-byte vectors.  The first column a band needs is
// 256 ct - 31; one column earlier is a multiple of 32: the window then starts
// on a line of its image row.
constexpr uint32_t kConvLead = 1;
__host__ __device__ constexpr uint32_t convPitch(uint32_t kw, bool vec) {
  return vec ? (kConvLead + kSegment + (kLine - 1) + kw - 1 + 3) / 4 * 4
             : kSegment + (kLine - 1) + kw - 1;
}

// LDS reads with the distance from a base address in the instruction (up to 64
// KB), for unrolled taps: the three taps of a row of the 3 x 3 kernel for the
// lane's four outputs (64 floats apart), twelve reads, and the wait for them,
// in ONE asm statement.  The compiler does not track what an asm issues, so a
// read whose wait sat in a later statement would leave registers that look
// written but are not until then -- nothing would stop a copy or a spill in
// between from reading them early.  The outputs are early-clobber: the address
// register is read by all twelve instructions.
__device__ __forceinline__ uint32_t ldsAddress(const float* p) {
  return static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
      (const __attribute__((address_space(3))) float*)(p)));
}
template <uint32_t kByteOffset>
__device__ __forceinline__ void ldsReadTapRow(uint32_t address, float (&v)[4][3]) {
  static_assert(kByteOffset + 3 * 256 + 8 < 65536, "offset field of the LDS read");
  asm volatile(
      "ds_read_b32 %0, %12 offset:%13\n\tds_read_b32 %1, %12 offset:%13+4\n\tds_read_b32 %2, %12 offset:%13+8\n\t"
      "ds_read_b32 %3, %12 offset:%13+256\n\tds_read_b32 %4, %12 offset:%13+260\n\tds_read_b32 %5, %12 offset:%13+264\n\t"
      "ds_read_b32 %6, %12 offset:%13+512\n\tds_read_b32 %7, %12 offset:%13+516\n\tds_read_b32 %8, %12 offset:%13+520\n\t"
      "ds_read_b32 %9, %12 offset:%13+768\n\tds_read_b32 %10, %12 offset:%13+772\n\tds_read_b32 %11, %12 offset:%13+776\n\t"
      "s_waitcnt lgkmcnt(0)"
      : "=&v"(v[0][0]), "=&v"(v[0][1]), "=&v"(v[0][2]), "=&v"(v[1][0]), "=&v"(v[1][1]), "=&v"(v[1][2]),
        "=&v"(v[2][0]), "=&v"(v[2][1]), "=&v"(v[2][2]), "=&v"(v[3][0]), "=&v"(v[3][1]), "=&v"(v[3][2])
      : "v"(address), "n"(kByteOffset)
      : "memory");
}

// KH_/KW_ == 0: the kernel size comes from the arguments.  VEC: image rows
// start on 16 bytes (the host checks); full bands inside the image are then
// staged with 16-byte loads.
template <int KH_, int KW_, bool VEC>
__global__ __launch_bounds__(kSegment) void conv2dKernel(ConvArgs p) {
  extern __shared__ float tile[];
  const uint32_t KH = KH_ ? KH_ : p.KH, KW = KW_ ? KW_ : p.KW;
  uint32_t tileIdx;
  if (!tileOfGroup(p.tiles, &tileIdx)) return; // before any barrier
  const uint32_t ct = tileIdx % p.colTiles, rt = tileIdx / p.colTiles;
  const uint32_t y0 = rt * kConvRows;
  const uint32_t rowsOut = p.OH - y0 < uint32_t(kConvRows) ? p.OH - y0 : uint32_t(kConvRows);
  const uint32_t rowsIn = rowsOut + KH - 1; // all inside the input: OH = H - KH + 1
  const uint32_t pitch = convPitch(KW, VEC);
  constexpr uint32_t lead = VEC ? kConvLead : 0;
  // input column held in tile column 0 (may be negative in the first segment);
  // the first column the band needs is `lead` columns further on
  const int64_t x0 = int64_t(ct) * kSegment - (kLine - 1) - lead;

  // Stage the window: lane t takes elements t, t+256, ... of the window in
  // row-major order.  pitch > 256, so stepping by 256 wraps to the next row at
  // most once.
  const uint32_t t = threadIdx.x;
  bool staged = false;
  if constexpr (KH_ != 0 && VEC) {
    // Full band of a constant-size kernel, window inside the image, rows on 16
    // bytes: lane t takes vectors t, t+256, ... of the window in row-major order.
    // Row and column of a vector are those of the lane's first one plus
    // constants and one compare; all loads are issued before the first LDS
    // store.  A quarter of the load instructions of the dword path below, and
    // a third of its address arithmetic.
    constexpr uint32_t P4 = convPitch(KW_ ? KW_ : 1, true) / 4; // vectors per window row
    constexpr uint32_t kRows = kConvRows + KH_ - 1;
    constexpr uint32_t kVectors = kRows * P4;
    constexpr int kRounds = (kVectors + kSegment - 1) / kSegment;
    if (x0 >= 0 && x0 + int64_t(4 * P4) <= int64_t(p.W) && rowsOut == uint32_t(kConvRows) &&
        uint64_t(kRows) * p.W < (1u << 30)) {
      const float* base = p.in + uint64_t(y0) * p.W + x0;
      const uint32_t row0 = t / P4, c0 = t % P4;
      v4f v[kRounds];
#pragma unroll
      for (int u = 0; u < kRounds; ++u) {
        constexpr uint32_t kStep = kSegment; // vectors between a lane's loads
        const uint32_t dq = uint32_t(u) * kStep / P4, dr = uint32_t(u) * kStep % P4; // constants after unrolling
        const bool wrap = c0 + dr >= P4;
        const uint32_t row = row0 + dq + (wrap ? 1u : 0u);
        const uint32_t c = c0 + dr - (wrap ? P4 : 0u);
        if (uint32_t(u + 1) * kStep <= kVectors || uint32_t(u) * kStep + t < kVectors)
          v[u] = *reinterpret_cast<const v4f*>(base + (row * p.W + 4 * c));
      }
#pragma unroll
      for (int u = 0; u < kRounds; ++u) {
        constexpr uint32_t kStep = kSegment;
        if (uint32_t(u + 1) * kStep <= kVectors || uint32_t(u) * kStep + t < kVectors)
          *reinterpret_cast<v4f*>(tile + 4 * (uint32_t(u) * kStep + t)) = v[u];
      }
      staged = true;
    }
  }
  if constexpr (KH_ != 0 && !VEC) {
    // Full band of a constant-size kernel with the whole window inside the
    // image: row and column of every element are compile-time constants plus
    // one compare, nothing is predicated, and all loads are issued before the
    // first LDS store.
    constexpr uint32_t P = kSegment + (kLine - 1) + KW_ - 1;
    constexpr uint32_t kRows = kConvRows + KH_ - 1;
    constexpr uint32_t kTotal = kRows * P;
    constexpr int kRounds = (kTotal + kSegment - 1) / kSegment;
    if (x0 >= 0 && x0 + P <= int64_t(p.W) && rowsOut == uint32_t(kConvRows) &&
        uint64_t(kRows) * p.W < (1u << 30)) {
      const float* base = p.in + uint64_t(y0) * p.W + x0;
      float v[kRounds];
#pragma unroll
      for (int u = 0; u < kRounds; ++u) {
        const uint32_t k = uint32_t(u) * kSegment;
        const uint32_t q = k / P, rem = k % P; // constants after unrolling
        const bool wrap = t + rem >= P;
        const uint32_t off = q * p.W + rem + t + (wrap ? p.W - P : 0u);
        if (k + kSegment <= kTotal || k + t < kTotal) v[u] = base[off];
      }
#pragma unroll
      for (int u = 0; u < kRounds; ++u) {
        const uint32_t k = uint32_t(u) * kSegment;
        if (k + kSegment <= kTotal || k + t < kTotal) tile[k + t] = v[u];
      }
      staged = true;
    }
  }
  if (!staged) {
    const uint32_t total = rowsIn * pitch;
    constexpr int kBatch = 8;
    uint32_t col = t;                                      // column within the window row
    const float* src = p.in + uint64_t(y0) * p.W + x0 + t; // never dereferenced outside the image
    for (uint32_t idx = t; idx < total; idx += kSegment * kBatch) {
      float v[kBatch];
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        const int64_t xi = x0 + col;
        const bool ok = idx + u * kSegment < total && xi >= 0 && xi < int64_t(p.W);
        v[u] = ok ? *src : 0.0f;
        col += kSegment;
        src += kSegment;
        if (col >= pitch) {
          col -= pitch;
          src += int64_t(p.W) - pitch;
        }
      }
#pragma unroll
      for (int u = 0; u < kBatch; ++u)
        if (idx + u * kSegment < total) tile[idx + u * kSegment] = v[u];
    }
  }
  constexpr int kRegWeights = KH_ != 0 ? KH_ * KW_ : 1;
  float wreg[kRegWeights];
  float* const wlds = tile + (kConvRows + KH - 1) * pitch; // generic sizes only
  if constexpr (KH_ != 0) {
#pragma unroll
    for (int i = 0; i < kRegWeights; ++i) wreg[i] = p.weights[i];
  } else {
    for (uint32_t i = t; i < KH * KW; i += kSegment) wlds[i] = p.weights[i];
  }
  // Every load of the staging phase has to be back before the barrier anyway.
  // Saying so here keeps the compiler from putting its own vmcnt(0) into the row
  // loop below (it would protect registers of loads whose lanes were
  // predicated off), where the counter also holds the previous row's stores:
  // each row would then wait for the stores of the row before.
  __builtin_amdgcn_s_waitcnt(kWaitVmcnt0);
  __syncthreads();

  // A wave takes every fourth row of the band; a lane computes the four
  // outputs lane, lane+64, lane+128, lane+192 of the row's segment, so the
  // lanes of a wave read consecutive LDS words for every tap (no bank
  // conflicts: four adjacent outputs per lane would put the lanes 4 words
  // apart, on 8 of the 32 banks) and each of the wave's four stores covers two
  // whole 128-byte lines.  The weights were
  // fetched before the barrier (registers for the constant sizes, LDS behind
  // the window otherwise): read through the pointer inside the loop they would
  // be re-fetched from memory for every row, because the stores may alias them.
  // The wave index is made a scalar so that everything that depends only on
  // the row (row shift, row pointers) is computed on the scalar unit.
  const uint32_t wave = __builtin_amdgcn_readfirstlane(t / 64), lane = t % 64;
  const int32_t xLane = int32_t(ct * kSegment + lane); // before the row's shift
  const int32_t ow = int32_t(p.OW);
  // segments whose 256 columns exist for every shift a row can have (0 .. 31):
  // no lane of the group needs a bounds check
  const bool interior = ct >= 1 && uint64_t(ct) * kSegment + kSegment <= p.OW;
  for (uint32_t r = wave; r < rowsOut; r += kSegment / 64) {
    const uint32_t y = y0 + r;
    const uint32_t shift = rowShift(y, p.OW, p.outPhase);
    const int32_t x = xLane - int32_t(shift); // the lane's first output; the others 64 apart
    const float* win = tile + r * pitch + lead + (kLine - 1) - shift + lane;
    float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if constexpr (KH_ == 3 && KW_ == 3) {
      // The 36 taps of the lane's four outputs, each read with its distance from
      // `win` in the instruction's offset field.  Written in C the compiler
      // pairs the reads (ds_read2, whose offsets reach 1 KB only) and spends a
      // vector add per pair on addresses: 6 of the 24 vector instructions per
      // output, in a kernel whose duration follows its instruction count.
      constexpr uint32_t P = convPitch(3, VEC);
      const uint32_t at = ldsAddress(win);
      float v[3][4][3];
      ldsReadTapRow<0 * P * 4>(at, v[0]);
      ldsReadTapRow<1 * P * 4>(at, v[1]);
      ldsReadTapRow<2 * P * 4>(at, v[2]);
#pragma unroll
      for (int a = 0; a < 3; ++a)
#pragma unroll
        for (int b = 0; b < 3; ++b)
#pragma unroll
          for (int j = 0; j < 4; ++j) acc[j] = v[a][j][b] * wreg[a * 3 + b] + acc[j];
    } else {
      for (uint32_t a = 0; a < KH; ++a)
        for (uint32_t b = 0; b < KW; ++b) {
          float wt;
          if constexpr (KH_ != 0) wt = wreg[a * KW_ + b];
          else wt = wlds[a * KW + b];
#pragma unroll
          for (int j = 0; j < 4; ++j) acc[j] = win[a * pitch + b + 64 * j] * wt + acc[j];
        }
    }
    float* const rowOut = p.out + uint64_t(y) * p.OW; // scalar
    if (interior) {
      // every lane's four outputs exist: one address, the others by offset
      float* const o = rowOut + x;
      streamStoreAt<0>(acc[0], o);
      streamStoreAt<256>(acc[1], o);
      streamStoreAt<512>(acc[2], o);
      streamStoreAt<768>(acc[3], o);
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int32_t xj = x + 64 * j;
        if (xj >= 0 && xj < ow) streamStore(acc[j], rowOut + xj);
      }
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
  streamStore(acc, &p.out[uint64_t(y) * p.OW + uint64_t(x)]);
}

struct PoolArgs {
  const float* in;
  float* out;
  uint32_t H, W, win0, win1, stride0, stride1, OH, OW;
  uint32_t colTiles, tiles;
  uint32_t outPhase;
};

__global__ __launch_bounds__(kSegment) void poolKernel(PoolArgs p) {
  uint32_t tileIdx;
  if (!tileOfGroup(p.tiles, &tileIdx)) return;
  const uint32_t ct = tileIdx % p.colTiles, rt = tileIdx / p.colTiles;
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
      streamStore(best, &p.out[uint64_t(y) * p.OW + uint64_t(x)]);
    }
  }
}

// Non-overlapping WIN x WIN windows (window == stride == WIN, 2 or 4) over an
// input whose rows are 4*WIN-byte aligned: a lane fetches a window row with one
// vector load, and all loads of the group's band (kPoolRows x WIN per lane) are
// issued before the first compare; lanes outside the row read a clamped, valid
// address instead of being branched around.  The loads stay cacheable: the
// skewed segments start anywhere in a line, so neighbouring waves share lines.
template <int WIN>
__global__ __launch_bounds__(kSegment) void poolSquareKernel(PoolArgs p) {
  typedef float vw __attribute__((ext_vector_type(WIN)));
  uint32_t tileIdx;
  if (!tileOfGroup(p.tiles, &tileIdx)) return;
  const uint32_t ct = tileIdx % p.colTiles, rt = tileIdx / p.colTiles;
  const uint32_t y0 = rt * kPoolRows;
  vw v[kPoolRows][WIN];
  int64_t xs[kPoolRows];
#pragma unroll
  for (int r = 0; r < kPoolRows; ++r) {
    const uint32_t y = y0 + r < p.OH ? y0 + r : p.OH - 1;
    const uint32_t shift = rowShift(y, p.OW, p.outPhase);
    const int64_t x = int64_t(ct) * kSegment - shift + threadIdx.x;
    xs[r] = x;
    const uint64_t xc = x < 0 ? 0 : (x >= int64_t(p.OW) ? p.OW - 1 : uint64_t(x));
    const float* corner = p.in + uint64_t(y) * WIN * p.W + xc * WIN;
#pragma unroll
    for (int a = 0; a < WIN; ++a)
      v[r][a] = *reinterpret_cast<const vw*>(corner + uint64_t(a) * p.W);
  }
  // All of the band's loads are waited for here, in one go.  Left to itself the
  // compiler waits for each row's loads just before that row's compares, by
  // count; the streaming stores below are in that count too (and unknown to
  // the compiler, being asm), so the second row's wait would also wait for the
  // first row's store to come back.
  __builtin_amdgcn_s_waitcnt(kWaitVmcnt0);
#pragma unroll
  for (int r = 0; r < kPoolRows; ++r) {
    float best = -10e5f;
#pragma unroll
    for (int a = 0; a < WIN; ++a)
#pragma unroll
      for (int b = 0; b < WIN; ++b) best = v[r][a][b] > best ? v[r][a][b] : best;
    if (y0 + r < p.OH && xs[r] >= 0 && xs[r] < int64_t(p.OW))
      streamStore(best, &p.out[uint64_t(y0 + r) * p.OW + uint64_t(xs[r])]);
  }
}

// Any window and stride, staged: the input window of a band of output rows goes
// through LDS once (as in fconv2d), and the taps are read from there.  Reading
// every tap from memory, as poolKernel does, costs a vector-memory instruction
// per tap and output: 3x3 windows at stride 1 or 2 ran at 16-28 % of the HBM
// rate that way, bound by the address unit, not by memory.
// Window geometry for stride (s0, s1) and bandRows output rows: input rows
// y0*s0 .. y0*s0 + (bandRows-1)*s0 + win0 - 1; input columns from
// (ct*256 - 31)*s1 (the segment's leftmost possible output column) over
// (256 + 31 - 1)*s1 + win1 columns.
struct PoolStagedArgs {
  PoolArgs pool;
  uint32_t bandRows; // output rows per work-group
  uint32_t pitch;    // columns of the staged window (a multiple of 4 when it is staged by vectors)
  uint32_t lead;     // columns the staged window starts before the first one needed (vector staging)
};

// W0_/W1_ == 0: the window size comes from the arguments.  VEC: the window is
// staged with 16-byte loads; it then starts `lead` columns early, on a 16-byte
// boundary of its image row (the host checks that rows start on one).
template <int W0_, int W1_, bool VEC>
__global__ __launch_bounds__(kSegment) void poolStagedKernel(PoolStagedArgs q) {
  extern __shared__ float tile[];
  const PoolArgs& p = q.pool;
  const uint32_t win0 = W0_ ? W0_ : p.win0, win1 = W1_ ? W1_ : p.win1;
  uint32_t tileIdx;
  if (!tileOfGroup(p.tiles, &tileIdx)) return; // before any barrier
  const uint32_t ct = tileIdx % p.colTiles, rt = tileIdx / p.colTiles;
  const uint32_t y0 = rt * q.bandRows;
  const uint32_t rowsOut = p.OH - y0 < q.bandRows ? p.OH - y0 : q.bandRows;
  const uint32_t rowsIn = (rowsOut - 1) * p.stride0 + win0; // all inside the input
  const uint32_t pitch = q.pitch;
  const int64_t x0 = (int64_t(ct) * kSegment - (kLine - 1)) * int64_t(p.stride1); // may be negative
  const uint32_t t = threadIdx.x;

  if constexpr (VEC) {
    // Lane t takes vectors t, t+256, ... of the window in row-major order, up
    // to eight in flight.  Against dword loads (below) this is a quarter of the
    // load instructions for the same bytes: 8192^2, 3x3 stride 2, 82 -> 57 us;
    // 5x5 stride 2, 162 -> 111 us.  (The convolution, which writes as much as
    // it reads, gains nothing from the same change.)
    const uint32_t perRow = pitch / 4, vectors = rowsIn * perRow;
    const int64_t xa = x0 - int64_t(q.lead); // multiple of 4, like W: a vector is inside the image or outside
    const float* const rowBase = p.in + uint64_t(y0) * p.stride0 * p.W;
    constexpr int kVecBatch = 8;
    // row and column of the lane's vector move on by 256 vectors per load: one
    // division per lane instead of one per load
    const uint32_t stepRow = uint32_t(kSegment) / perRow, stepCol = uint32_t(kSegment) % perRow;
    uint32_t row = t / perRow, c = t - row * perRow;
    for (uint32_t first = 0; first < vectors; first += kSegment * kVecBatch) {
      v4f v[kVecBatch];
#pragma unroll
      for (int u = 0; u < kVecBatch; ++u) {
        const uint32_t idx = first + t + u * kSegment;
        const int64_t xi = xa + 4 * int64_t(c);
        v[u] = (idx < vectors && xi >= 0 && xi < int64_t(p.W))
                   ? *reinterpret_cast<const v4f*>(rowBase + uint64_t(row) * p.W + xi)
                   : v4f{0.f, 0.f, 0.f, 0.f};
        row += stepRow;
        c += stepCol;
        if (c >= perRow) {
          c -= perRow;
          ++row;
        }
      }
#pragma unroll
      for (int u = 0; u < kVecBatch; ++u) {
        const uint32_t idx = first + t + u * kSegment;
        if (idx < vectors) *reinterpret_cast<v4f*>(tile + 4 * idx) = v[u];
      }
    }
  }
  // Otherwise: lane t takes window elements t, t+256, ... in row-major order
  // (pitch > 256, so a step of 256 wraps to the next row at most once), eight
  // loads at a time (the whole window's loads at once, up to 24: 10-25 %
  // slower; 4 or 12 at a time: within a few per cent either way).
  const uint32_t total = VEC ? 0 : rowsIn * pitch;
  constexpr int kBatch = 8;
  const bool inside = x0 >= 0 && x0 + pitch <= int64_t(p.W);
  uint32_t col = t;
  const float* src = p.in + uint64_t(y0) * p.stride0 * p.W + x0 + t; // never dereferenced outside the image
  for (uint32_t idx = t; idx < total; idx += kSegment * kBatch) {
    float v[kBatch];
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const int64_t xi = x0 + col;
      const bool ok = idx + u * kSegment < total && (inside || (xi >= 0 && xi < int64_t(p.W)));
      v[u] = ok ? *src : 0.0f;
      col += kSegment;
      src += kSegment;
      if (col >= pitch) {
        col -= pitch;
        src += int64_t(p.W) - pitch;
      }
    }
#pragma unroll
    for (int u = 0; u < kBatch; ++u)
      if (idx + u * kSegment < total) tile[idx + u * kSegment] = v[u];
  }
  __builtin_amdgcn_s_waitcnt(kWaitVmcnt0); // as in conv2dKernel: no vmcnt(0) of the compiler's in the row loop
  __syncthreads();

  const uint32_t wave = __builtin_amdgcn_readfirstlane(t / 64), lane = t % 64;
  const int32_t ow = int32_t(p.OW);
  for (uint32_t r = wave; r < rowsOut; r += kSegment / 64) {
    const uint32_t y = y0 + r;
    const uint32_t shift = rowShift(y, p.OW, p.outPhase);
    float* const rowOut = p.out + uint64_t(y) * p.OW;
    // the lane's first output of the row; its others are 64 outputs further on each
    const float* corner = tile + r * p.stride0 * pitch + (VEC ? q.lead : 0u) +
                          (uint32_t(kLine - 1) - shift + lane) * p.stride1;
    const int32_t x = int32_t(ct * kSegment + lane) - int32_t(shift);
    const uint32_t step = 64 * p.stride1;
    // utils/dialects/lib/PolarGraph/kernels/Pool2DOp.cpp:50-52,74-76: starts
    // at -10e5, strict ordered greater-than, rows outer / columns inner
    float best[4] = {-10e5f, -10e5f, -10e5f, -10e5f};
    if constexpr (W0_ != 0) {
#pragma unroll
      for (int a = 0; a < W0_; ++a)
#pragma unroll
        for (int b = 0; b < W1_; ++b)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float v = corner[a * pitch + b + j * step];
            best[j] = v > best[j] ? v : best[j];
          }
    } else {
      for (uint32_t a = 0; a < win0; ++a)
        for (uint32_t b = 0; b < win1; ++b) {
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float v = corner[a * pitch + b + j * step];
            best[j] = v > best[j] ? v : best[j];
          }
        }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int32_t xj = x + 64 * j;
      if (xj >= 0 && xj < ow) streamStore(best[j], rowOut + xj);
    }
  }
}

// Overlapping square windows of 2..5 at stride 1 or 2 over rows that start on 16
// bytes: a wave marches down a strip of the image.  Every lane holds STRIDE
// 16-byte vectors of each input row (kMarchAhead rows in flight), takes the
// columns its windows reach beyond a vector from the lane that holds the next
// one, and folds the row's taps of each of its four outputs into one value; the
// last WIN rows of those values stay in registers and are folded again when a
// window is complete.  Each input element is loaded once per strip (the WIN -
// stride rows two bands share, twice) and every tap costs a compare and a
// select instead of an LDS read.
//
// Stores decide the rest.  A row of the wave's outputs leaves through 1 KB of
// LDS, so that it can be cut where the 128-byte lines of the output are, not
// where the lanes' columns are: the wave whose nominal piece of the row (220
// columns) holds the start of a line stores that line, whole.  A wave therefore
// computes 252 (stride 2: 254) columns and stores up to 251 of them, the pieces
// of neighbouring waves overlapping by what that takes; only the two ends of an
// output row are stored as parts of lines.  (With every lane storing its own
// four columns, a row left as 1008-byte pieces that shared a line at either
// end: 127 us for 3 x 3 windows at stride 1 over 8192^2, 48 us of it loads.)
//
// The order of the comparisons is the reference's: rows in ascending order,
// columns in ascending order within a row, strictly greater replaces.  Folding
// each row first and the rows' results afterwards picks the same element as
// one pass over the window does -- the first of the largest -- so the result is
// the same bit pattern even where +0 and -0 meet, and NaNs are skipped as
// there, because every fold starts from the floor value, not from an element.
constexpr uint32_t kMarchChunk = 220;   // output columns between the first columns of neighbouring waves
// Rows a wave has in flight, and waves a launch aims for (the bands get shorter
// to reach it, down to kMarchMinBand output rows).  8192^2, stride 1: 125 us
// with 8192 waves, 104 with 16384, 96 with 65536 or more (six rows in flight;
// eight: 1 us less; twelve: more registers, slower again) -- short bands keep
// the rows that many waves read and write at one time close together in
// memory.  Stride 2 has half the stores and prefers long bands, which read
// fewer rows twice: 5 x 5, 66 us with 8192 waves, 67-70 with 16384-65536.
template <int STRIDE> constexpr int kMarchAhead = STRIDE == 1 ? 8 : 6;
constexpr uint32_t marchWaves(uint32_t stride) { return stride == 1 ? 65536 : 8192; }
constexpr uint32_t kMarchMinBand = 8;   // output rows per wave, at least

struct PoolMarchArgs {
  PoolArgs pool;
  uint32_t vecsPerRow;  // W / 4
  uint32_t wavesAcross; // ceil(OW / 220)
  uint32_t bandRows;    // output rows per wave
};

typedef float v2f __attribute__((ext_vector_type(2)));  // (LDS only)

template <int WIN, int STRIDE>
__global__ __launch_bounds__(64) void poolMarchKernel(PoolMarchArgs q) {
  constexpr int VPL = STRIDE;                                  // vectors of a row per lane
  constexpr int NOUT = 4 / STRIDE;                             // outputs per vector and output row
  constexpr int REACH = (NOUT - 1) * STRIDE + WIN;             // columns the windows of a vector span
  constexpr int HALO = REACH > 4 ? REACH - 4 : 0;              // of them, in the next vector
  constexpr int D = kMarchAhead<STRIDE>;
  static_assert(4 % STRIDE == 0 && HALO <= 4, "a vector's windows end within the next vector");
  static_assert(kMarchChunk * STRIDE % 4 == 0, "every wave starts on a vector");
  static_assert(kMarchChunk + 31 <= uint32_t(NOUT) * (64 * VPL - 1), "what a wave may have to store, it computes");
  __shared__ __attribute__((aligned(16))) float stage[64 * VPL * NOUT];
  const PoolArgs& p = q.pool;
  uint32_t task;
  if (!tileOfGroup(p.tiles, &task)) return;
  const uint32_t lane = threadIdx.x;
  const uint32_t across = task % q.wavesAcross, band = task / q.wavesAcross;
  const uint32_t y0 = band * q.bandRows;
  const uint32_t outRows = p.OH - y0 < q.bandRows ? p.OH - y0 : q.bandRows;
  const uint32_t inRows = (outRows - 1) * STRIDE + WIN;
  const uint32_t firstColumn = across * kMarchChunk;  // of the wave's outputs
  // the lane's vectors of a row: 64 j + lane behind the wave's first; beyond the
  // row, some valid address (no output that is stored depends on it)
  const v4f* src[VPL];
#pragma unroll
  for (int j = 0; j < VPL; ++j) {
    uint32_t vec = firstColumn * STRIDE / 4 + 64 * j + lane;
    if (vec >= q.vecsPerRow) vec = q.vecsPerRow - 1;
    src[j] = reinterpret_cast<const v4f*>(p.in + uint64_t(y0) * STRIDE * p.W) + vec;
  }
  const uint64_t pitchVecs = q.vecsPerRow;
  // the output row being completed: where the wave's first column is, in floats from `out`
  uint64_t flat = uint64_t(y0) * p.OW + firstColumn;
  const uint64_t outFloats = reinterpret_cast<uintptr_t>(p.out) / sizeof(float);
  const uint32_t columnsLeft = p.OW - firstColumn;  // of the row, from the wave's first

  const uint32_t lastRow = inRows - 1;
  v4f ahead[D][VPL];
#pragma unroll
  for (int d = 0; d < D; ++d)
#pragma unroll
    for (int j = 0; j < VPL; ++j) ahead[d][j] = src[j][(uint32_t(d) < inRows ? d : lastRow) * pitchVecs];
  float h[WIN][VPL][NOUT];  // the row folds of the last WIN rows, oldest first
#pragma unroll
  for (int a = 0; a < WIN; ++a)
#pragma unroll
    for (int j = 0; j < VPL; ++j)
#pragma unroll
      for (int i = 0; i < NOUT; ++i) h[a][j][i] = -10e5f;

  // one more input row: its folds enter the ring
  auto fold = [&](const v4f (&own)[VPL]) {
#pragma unroll
    for (int a = 0; a + 1 < WIN; ++a)
#pragma unroll
      for (int j = 0; j < VPL; ++j)
#pragma unroll
        for (int i = 0; i < NOUT; ++i) h[a][j][i] = h[a + 1][j][i];
#pragma unroll
    for (int j = 0; j < VPL; ++j) {
      float c[4 + HALO];
#pragma unroll
      for (int e = 0; e < 4; ++e) c[e] = own[j][e];
      // the next vector of the row is the next lane's, and for lane 63 lane 0's
      // next one (the wave's last vector has none: its outputs are never stored)
#pragma unroll
      for (int e = 0; e < HALO; ++e) {
        const float mine = (j + 1 < VPL && lane == 0) ? own[j + 1 < VPL ? j + 1 : j][e] : own[j][e];
        c[4 + e] = __shfl(mine, (lane + 1) & 63);
      }
#pragma unroll
      for (int i = 0; i < NOUT; ++i) {
        // utils/dialects/lib/PolarGraph/kernels/Pool2DOp.cpp:50-52,74-76: starts
        // at -10e5, strict ordered greater-than
        float best = -10e5f;
#pragma unroll
        for (int b = 0; b < WIN; ++b) best = c[i * STRIDE + b] > best ? c[i * STRIDE + b] : best;
        h[WIN - 1][j][i] = best;
      }
    }
  };
  // the ring holds a complete window: one output row
  auto emit = [&]() {
#pragma unroll
    for (int j = 0; j < VPL; ++j) {
      float o[NOUT];
#pragma unroll
      for (int i = 0; i < NOUT; ++i) {
        float best = -10e5f;
#pragma unroll
        for (int a = 0; a < WIN; ++a) best = h[a][j][i] > best ? h[a][j][i] : best;
        o[i] = best;
      }
      // column NOUT (64 j + lane) + i of the wave
      if constexpr (NOUT == 4)
        *reinterpret_cast<v4f*>(stage + 4 * (64 * j + lane)) = v4f{o[0], o[1], o[2], o[3]};
      else
        *reinterpret_cast<v2f*>(stage + 2 * (64 * j + lane)) = v2f{o[0], o[1]};
    }
    // The wave stores columns [from, to) of its own: from the first line that
    // starts in its piece (the row's first wave: from the row's start) up to
    // the first line that starts in the next wave's piece, or the row's end.
    const uint32_t phase = uint32_t(outFloats + flat) & 31u;  // of the wave's first column within its line
    const uint32_t from = across == 0 ? 0 : (32 - phase) & 31u;
    uint32_t to = kMarchChunk + ((32 - ((phase + kMarchChunk) & 31u)) & 31u);
    if (to > columnsLeft) to = columnsLeft;
    // in pieces of 16 bytes, one per lane; only a row's first and last can be
    // partly outside
    const int32_t first = int32_t(from) - int32_t((phase + from) & 3u) + 4 * int32_t(lane);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the row is in LDS (a wave's LDS accesses are served in order)
    float v[4];
    bool inside[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int32_t at = first + e;
      inside[e] = at >= int32_t(from) && at < int32_t(to);
      v[e] = stage[inside[e] ? at : 0];
    }
    float* const dst = p.out + flat + first;  // (only dereferenced where inside)
    // (stores the compiler does not count: its waits for the rows in flight stay exact)
    if (inside[0] && inside[3]) {
      streamStore(v4f{v[0], v[1], v[2], v[3]}, reinterpret_cast<v4f*>(dst));
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (inside[e]) streamStore(v[e], dst + e);
    }
    flat += p.OW;
  };

  // the first WIN - 1 rows complete no window
  constexpr int P = WIN - 1;
  static_assert(P < D && D % STRIDE == 0, "the slots and the output rows repeat with the unrolled loop");
#pragma unroll
  for (int a = 0; a < P; ++a) {
    fold(ahead[a]);
#pragma unroll
    for (int j = 0; j < VPL; ++j) ahead[a][j] = src[j][(uint32_t(a + D) < inRows ? a + D : lastRow) * pitchVecs];
  }
  // From here on row P + n completes a window when n is a multiple of the
  // stride, and sits in slot (P + n) % D.  While 2 D rows remain, every fetch
  // of the loop is of a row of the band: no conditions, so the waits can be
  // exact.
  uint32_t row = P;
  for (; row + 2 * D <= inRows; row += D) {
#pragma unroll
    for (int d = 0; d < D; ++d) {
      const int slot = (P + d) % D;
      fold(ahead[slot]);
#pragma unroll
      for (int j = 0; j < VPL; ++j) ahead[slot][j] = src[j][uint64_t(row + d + D) * pitchVecs];
      if (d % STRIDE == 0) emit();
    }
  }
  // the last rows (fewer than 2 D)
#pragma unroll
  for (int d = 0; d < 2 * D; ++d) {
    if (row + d < inRows) {  // (uniform)
      const int slot = (P + d) % D;
      fold(ahead[slot]);
      if (row + d + D < inRows) {
#pragma unroll
        for (int j = 0; j < VPL; ++j) ahead[slot][j] = src[j][uint64_t(row + d + D) * pitchVecs];
      }
      if (d % STRIDE == 0) emit();
    }
  }
}

// Whether a call goes to the marching kernel, and its geometry
struct MarchPoolPlan {
  bool fits;
  uint32_t vecsPerRow, wavesAcross, bandRows;
  uint64_t tasks;
};
MarchPoolPlan planMarchPool(const PoolArgs& p, bool vec) {
  MarchPoolPlan plan{false, 0, 0, 0, 0};
  const bool square = p.win0 == p.win1 && p.stride0 == p.stride1;
  // Windows of 2 and 3 stay with the staged kernel, which reads fewer input
  // columns twice (8192^2, kernel time, staged / marching: 3 x 3 stride 1 90 /
  // 96 us, stride 2 56 / 66, 2 x 2 stride 1 88 / 95; but 4 x 4 stride 1 138 /
  // 101, stride 2 68 / 66, 5 x 5 stride 1 180 / 108, stride 2 99 / 66).
  if (!vec || !square || p.win0 < 4 || p.win0 > 5 || p.stride0 < 1 || p.stride0 > 2) return plan;
  plan.vecsPerRow = p.W / 4;
  plan.wavesAcross = (p.OW + kMarchChunk - 1) / kMarchChunk;
  const uint32_t bandsWanted = marchWaves(p.stride0) / plan.wavesAcross > 0 ? marchWaves(p.stride0) / plan.wavesAcross : 1;
  uint32_t band = (p.OH + bandsWanted - 1) / bandsWanted;
  if (band < kMarchMinBand) band = kMarchMinBand;
  if (band > p.OH) band = p.OH;
  plan.bandRows = band;
  plan.tasks = uint64_t(plan.wavesAcross) * ((p.OH + band - 1) / band);
  plan.fits = plan.tasks < (1ull << 31) - kXcds;
  return plan;
}

// Geometry of the staged pooling kernel for one call, or fits = false if a band
// of one output row does not fit its LDS budget.  All of it in 64 bits: the
// strides are only bounded by the image (2^31), and a pitch that wrapped in 32
// bits could pass for one that fits.
struct StagedPoolPlan {
  bool fits;
  uint32_t pitch, lead, bandRows, ldsBytes;
};
StagedPoolPlan planStagedPool(const PoolArgs& p, bool vec) {
  StagedPoolPlan plan{false, 0, 0, 0, 0};
  uint64_t pitch = uint64_t(kSegment + kLine - 2) * p.stride1 + p.win1, lead = 0;
  // Image rows that start on 16 bytes: the window is staged by vectors.  Its
  // first needed column is (256 ct - 31) stride1, the same modulo 4 for every
  // column tile; the staged window starts that many columns earlier.
  if (vec) {
    lead = (4 - (uint64_t(kLine - 1) * p.stride1) % 4) % 4;
    pitch = (pitch + lead + 3) / 4 * 4;
  }
  const uint64_t floats = kMaxPoolLds / sizeof(float);
  if (pitch > floats) return plan;
  const uint64_t rowsFit = floats / pitch; // input rows
  if (rowsFit < p.win0 || uint64_t(p.H) * p.W >= (1ull << 40)) return plan;
  uint64_t band = (rowsFit - p.win0) / p.stride0 + 1;
  if (band > kPoolStagedRows) band = kPoolStagedRows;
  plan.fits = true;
  plan.pitch = static_cast<uint32_t>(pitch);
  plan.lead = static_cast<uint32_t>(lead);
  plan.bandRows = static_cast<uint32_t>(band);
  plan.ldsBytes = static_cast<uint32_t>(((band - 1) * p.stride0 + p.win0) * pitch * sizeof(float));
  return plan;
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
  const bool vec = p.W % 4 == 0 && reinterpret_cast<uintptr_t>(in) % 16 == 0;
  const uint64_t ldsBytes = (uint64_t(kConvRows + p.KH - 1) * convPitch(p.KW, vec) +
                             uint64_t(p.KH) * p.KW) * sizeof(float); // window + weights
  if (ldsBytes <= kMaxConvLds) {
    const uint64_t tiles = uint64_t(p.colTiles) * ((p.OH + kConvRows - 1) / kConvRows);
    POLAR_HIP_REQUIRE(tiles < (1ull << 31) - kXcds, "tensor too large for one launch");
    p.tiles = static_cast<uint32_t>(tiles);
    const uint64_t grid = paddedGrid(tiles);
    auto fn = p.KH == 3 && p.KW == 3   ? (vec ? conv2dKernel<3, 3, true> : conv2dKernel<3, 3, false>)
              : p.KH == 5 && p.KW == 5 ? (vec ? conv2dKernel<5, 5, true> : conv2dKernel<5, 5, false>)
                                       : (vec ? conv2dKernel<0, 0, true> : conv2dKernel<0, 0, false>);
    POLAR_HIP_TRY(launchKernelLds(dev, fn, dim3(static_cast<unsigned>(grid)),
                                  dim3(kSegment), static_cast<uint32_t>(ldsBytes), p));
  } else {
    const uint64_t grid = uint64_t(p.colTiles) * p.OH;
    POLAR_HIP_REQUIRE(grid < (1ull << 31), "tensor too large for one launch");
    p.tiles = static_cast<uint32_t>(grid);
    POLAR_HIP_TRY(launchKernel(dev, conv2dDirectKernel,
                               dim3(static_cast<unsigned>(grid)), dim3(kSegment), p));
  }
  return POLAR_HIP_OK;
}

int polar_hip_fpool_plan(uint64_t height, uint64_t width, uint64_t window0, uint64_t window1,
                         uint64_t stride0, uint64_t stride1, int input_aligned, int* kernel,
                         uint32_t* band_rows, uint32_t* lds_bytes) {
  POLAR_HIP_REQUIRE(kernel != nullptr, "null argument");
  POLAR_HIP_REQUIRE(window0 >= 1 && window1 >= 1, "empty pooling window");
  POLAR_HIP_REQUIRE(stride0 >= 1 && stride1 >= 1, "pooling stride must be positive");
  POLAR_HIP_REQUIRE(height >= window0 && width >= window1, "pooling window larger than the input");
  POLAR_HIP_REQUIRE(height < (1ull << 31) && width < (1ull << 31), "dimension does not fit 31 bits");
  PoolArgs p{};
  p.H = static_cast<uint32_t>(height);
  p.W = static_cast<uint32_t>(width);
  p.win0 = static_cast<uint32_t>(window0);
  p.win1 = static_cast<uint32_t>(window1);
  p.stride0 = static_cast<uint32_t>(stride0 < height ? stride0 : height);
  p.stride1 = static_cast<uint32_t>(stride1 < width ? stride1 : width);
  p.OH = (p.H - p.win0) / p.stride0 + 1;
  p.OW = (p.W - p.win1) / p.stride1 + 1;
  const bool aligned = input_aligned != 0;
  auto square = [&](uint32_t w) {
    return p.win0 == w && p.win1 == w && p.stride0 == w && p.stride1 == w && p.W % w == 0 && aligned;
  };
  *kernel = 0;
  if (band_rows) *band_rows = 0;
  if (lds_bytes) *lds_bytes = 0;
  if (square(2) || square(4)) {
    *kernel = 1;
    return POLAR_HIP_OK;
  }
  const MarchPoolPlan march = planMarchPool(p, aligned && p.W % 4 == 0);
  if (march.fits) {
    *kernel = 3;
    if (band_rows) *band_rows = march.bandRows;
    return POLAR_HIP_OK;
  }
  const StagedPoolPlan plan = planStagedPool(p, aligned && p.W % 4 == 0);
  if (plan.fits) {
    *kernel = 2;
    if (band_rows) *band_rows = plan.bandRows;
    if (lds_bytes) *lds_bytes = plan.ldsBytes;
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
  const uint64_t tiles = uint64_t(p.colTiles) * ((p.OH + kPoolRows - 1) / kPoolRows);
  POLAR_HIP_REQUIRE(tiles < (1ull << 31) - kXcds, "tensor too large for one launch");
  p.tiles = static_cast<uint32_t>(tiles);
  const uint64_t grid = paddedGrid(tiles);
  POLAR_HIP_TRY(hipSetDevice(dev->ordinal));
  auto square = [&](uint32_t w) {
    return p.win0 == w && p.win1 == w && p.stride0 == w && p.stride1 == w && p.W % w == 0 &&
           reinterpret_cast<uintptr_t>(in) % (sizeof(float) * w) == 0;
  };
  if (!square(2) && !square(4)) {
    // staged kernel if a band of at least one output row fits the LDS budget
    const bool vec = p.W % 4 == 0 && reinterpret_cast<uintptr_t>(in) % 16 == 0;
    const MarchPoolPlan march = planMarchPool(p, vec);
    if (march.fits) {
      PoolMarchArgs q;
      q.pool = p;
      q.pool.tiles = static_cast<uint32_t>(march.tasks);
      q.vecsPerRow = march.vecsPerRow;
      q.wavesAcross = march.wavesAcross;
      q.bandRows = march.bandRows;
      void (*marching)(PoolMarchArgs) = nullptr;
      switch (p.win0 * 10 + p.stride0) {
      case 41: marching = poolMarchKernel<4, 1>; break;
      case 42: marching = poolMarchKernel<4, 2>; break;
      case 51: marching = poolMarchKernel<5, 1>; break;
      case 52: marching = poolMarchKernel<5, 2>; break;
      }
      POLAR_HIP_REQUIRE(marching != nullptr, "no marching kernel for this window");
      POLAR_HIP_TRY(launchKernel(dev, marching, dim3(static_cast<unsigned>(paddedGrid(march.tasks))), dim3(64), q));
      return POLAR_HIP_OK;
    }
    const StagedPoolPlan plan = planStagedPool(p, vec);
    if (plan.fits) {
      PoolStagedArgs q;
      q.pool = p;
      q.pitch = plan.pitch;
      q.lead = plan.lead;
      q.bandRows = plan.bandRows;
      const uint64_t stagedTiles = uint64_t(p.colTiles) * ((p.OH + q.bandRows - 1) / q.bandRows);
      POLAR_HIP_REQUIRE(stagedTiles < (1ull << 31) - kXcds, "tensor too large for one launch");
      q.pool.tiles = static_cast<uint32_t>(stagedTiles);
      auto staged = p.win0 == 2 && p.win1 == 2   ? (vec ? poolStagedKernel<2, 2, true> : poolStagedKernel<2, 2, false>)
                    : p.win0 == 3 && p.win1 == 3 ? (vec ? poolStagedKernel<3, 3, true> : poolStagedKernel<3, 3, false>)
                    : p.win0 == 5 && p.win1 == 5 ? (vec ? poolStagedKernel<5, 5, true> : poolStagedKernel<5, 5, false>)
                                                 : (vec ? poolStagedKernel<0, 0, true> : poolStagedKernel<0, 0, false>);
      POLAR_HIP_TRY(launchKernelLds(dev, staged, dim3(static_cast<unsigned>(paddedGrid(stagedTiles))),
                                    dim3(kSegment), plan.ldsBytes, q));
      return POLAR_HIP_OK;
    }
  }
  auto fn = square(2) ? poolSquareKernel<2> : square(4) ? poolSquareKernel<4> : poolKernel;
  POLAR_HIP_TRY(launchKernel(dev, fn, dim3(static_cast<unsigned>(grid)), dim3(kSegment), p));
  return POLAR_HIP_OK;
}

} // extern "C"
