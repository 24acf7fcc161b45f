// fmatmul for a short contraction (K <= 128) with one long and one short output
// dimension: C[65536 x 33] = A[65536 x 127] * B[127 x 33] and its mirror image.
//
// Such products stream the long operand and C through HBM once (a few FLOP per
// byte) and keep the matrix cores about as busy as the memory, so the kernel
// is shaped like the streaming kernels of this library rather than like a
// tiled GEMM: many small independent units of work and no barrier on the way.
//   * The short operand (all of it: at most 128 x 128) is put into LDS once per
//     work-group.
//   * Every wave then owns 16 consecutive rows (or columns) of the long
//     dimension with the WHOLE of K: it reads its slice of the long operand
//     straight from HBM into registers, already in the layout the matrix
//     instruction wants (v_mfma_f32_16x16x4_f32: lane l feeds element
//     [l % 16][l / 16] of a 16 x 4 block), 16 values of k per load and two
//     loads ahead of the arithmetic.  No LDS staging and no barrier.
//   * The 16 x 16 x 4 instruction pads the short dimension to a multiple of 16
//     only (33 -> 48, not 64).
//   * A wave stores its accumulators directly; its 16 rows of C are one
//     contiguous piece of memory, written within a few hundred cycles, so the
//     partial lines merge in L2.
// Waves do not wait for each other, so with 16 of them per CU the fetch of
// one overlaps the arithmetic of the others.  Two groups of k in flight per
// wave is what measured best: with four, 65536 x 33 x 127 goes from 18.0 to
// 19.6 us and 65536 x 127 x 33 from 18.6 to 23 us; dropping the two fetches
// that are issued beyond the end of a slice (a peeled last pair) changes
// nothing for those shapes and costs 33 x 65536 x 127 three microseconds.  The result does not depend on
// scheduling: every element is accumulated by one lane in k order.
#include "internal.h"
#include "matmul_epilogue.h"
#include "short_tile.h"

using namespace polar_hip_detail;

namespace {

typedef float v4f __attribute__((ext_vector_type(4)));

constexpr uint32_t kMaxK = 128;
// A work-group has WAVES waves (4 or 8, a template parameter below): 64 WAVES
// lanes, and 16 WAVES values of the long dimension per turn.

struct SmallKArgs {
  const float* A;
  const float* B;
  float* C;
  uint32_t M, N, K;
  uint32_t k4;     // K rounded up to a multiple of 16 (four k steps of the instruction)
  uint32_t pitch;  // LDS pitch of the short operand's tile, in floats
  int epilogue;
  const float* bias;
  float scaleAcc, scaleBias;
};

// The plain product is stored as it is; a fused epilogue is applied on the way
// (a uniform branch, so the plain path carries none of the epilogue's code).
__device__ __forceinline__ void storeResult(const SmallKArgs& p, size_t idx, float value) {
  if (p.epilogue == kEpiNone)
    p.C[idx] = value;
  else
    p.C[idx] = applyEpilogue(p.epilogue, value, p.bias, p.scaleAcc, p.scaleBias, idx);
}

// TS blocks of 16 cover the short dimension.  TALL: M is the long dimension (B
// is the short operand, N <= 16*TS); otherwise N is (A is the short operand,
// M <= 16*TS).
template <int TS, bool TA, bool TB, bool TALL, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void smallKKernel(SmallKArgs p) {
  constexpr int kThreads = WAVES * 64;
  constexpr int kBlock = WAVES * 16; // values of the long dimension per work-group and turn
  extern __shared__ __attribute__((aligned(16))) float shortS[];
  // A is k-contiguous when not transposed ([M x K]); B when transposed ([N x K])
  constexpr bool kShortKContig = TALL ? TB : !TA;
  constexpr bool kLongKContig = TALL ? !TA : TB;
  using Short = ShortTile<kShortKContig>;
  const float* const longX = TALL ? p.A : p.B;
  const uint32_t longDim = TALL ? p.M : p.N, shortDim = TALL ? p.N : p.M;

  const int t = threadIdx.x, lane = t % 64, wave = t / 64;
  const uint32_t fx = lane % 16, fk = lane / 16; // the lane's place in a 16 x 4 fragment
  const uint32_t blocks = (longDim + kBlock - 1) / kBlock;
  const uint32_t groups = p.k4 / 16, pairs = groups / 2, lastGroup = groups - 1;

  // The wave's slice of the long operand comes in groups of four k steps (16
  // values of k), one 16-byte register tuple per lane and group, fetched a pair
  // of groups ahead of the arithmetic.  Which k a lane group feeds at which step
  // is free as long as both operands agree: a k-contiguous operand is read 16
  // bytes per lane, lane group q taking k = 16*g + 4*q + c at step c of group g,
  // so that one load covers 64 contiguous bytes of each of the wave's 16 rows
  // (with 4-byte loads every line would be asked for eight times over); the
  // other kind keeps the plain order k = 16*g + 4*c + q.
  // Every fetch is the same fixed number of loads whatever the lane and the
  // group (addresses are clamped into the operand, what lies beyond it is zeroed
  // afterwards): the compiler can then count the loads in flight and wait for
  // the older pair only, not for the pair it has just issued.
  auto fetchGroup = [&](uint32_t x, uint32_t g) -> v4f {
    const uint32_t xInside = x < longDim ? x : longDim - 1; // its results are never stored
    v4f v;
    if constexpr (kLongKContig) {
      // the four values k .. k+3 of row x; near the end of the row the last
      // four of the row are loaded instead and shifted down by d
      const uint32_t k = 16 * g + 4 * fk;
      const uint32_t from = k + 4 <= p.K ? k : p.K - 4; // K >= 4
      const uint32_t d = k - from;
      const v4f w = *reinterpret_cast<const v4f __attribute__((aligned(4)))*>(longX + size_t(xInside) * p.K + from);
      v[0] = d == 0 ? w[0] : d == 1 ? w[1] : d == 2 ? w[2] : d == 3 ? w[3] : 0.0f;
      v[1] = d == 0 ? w[1] : d == 1 ? w[2] : d == 2 ? w[3] : 0.0f;
      v[2] = d == 0 ? w[2] : d == 1 ? w[3] : 0.0f;
      v[3] = d == 0 ? w[3] : 0.0f;
    } else {
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const uint32_t k = 16 * g + 4 * c + fk;
        const float w = longX[size_t(k < p.K ? k : p.K - 1) * longDim + xInside];
        v[c] = k < p.K ? w : 0.0f;
      }
    }
    return v;
  };

  // the first fetches of the first block go out before the short operand is
  // brought in: they travel while that happens
  const uint32_t firstX = blockIdx.x * kBlock + wave * 16 + fx;
  v4f next0 = fetchGroup(firstX, 0), next1 = fetchGroup(firstX, 1 < groups ? 1 : lastGroup);
  Short::template load<kThreads>(shortS, TALL ? p.B : p.A, shortDim, TS * 16, p.K, p.k4, p.pitch, t);
  __syncthreads();

  for (uint32_t block = blockIdx.x; block < blocks; block += gridDim.x) {
    const uint32_t x0 = block * kBlock + wave * 16; // this wave's 16 rows (columns)
    if (x0 >= longDim) break;
    const uint32_t x = x0 + fx;
    if (block != blockIdx.x) {
      next0 = fetchGroup(x, 0);
      next1 = fetchGroup(x, 1 < groups ? 1 : lastGroup);
    }
    v4f acc[TS];
#pragma unroll
    for (int j = 0; j < TS; ++j) acc[j] = v4f{0.f, 0.f, 0.f, 0.f};
    // one group: 4 k steps, 4*TS matrix instructions, no branch in between (a
    // branch between them would make the compiler move the accumulators about)
    auto multiplyGroup = [&](uint32_t g, v4f longF) {
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const uint32_t k = kLongKContig ? 16 * g + 4 * fk + c : 16 * g + 4 * c + fk;
#pragma unroll
        for (int j = 0; j < TS; ++j) {
          const float other = Short::fragment(shortS, p.pitch, j * 16 + fx, k);
          acc[j] = TALL ? __builtin_amdgcn_mfma_f32_16x16x4f32(longF[c], other, acc[j], 0, 0, 0)
                        : __builtin_amdgcn_mfma_f32_16x16x4f32(other, longF[c], acc[j], 0, 0, 0);
        }
      }
    };
    for (uint32_t pair = 0; pair < pairs; ++pair) {
      const v4f cur0 = next0, cur1 = next1;
      // beyond the end the last group is fetched again (from cache) and not used
      next0 = fetchGroup(x, 2 * pair + 2 < groups ? 2 * pair + 2 : lastGroup);
      next1 = fetchGroup(x, 2 * pair + 3 < groups ? 2 * pair + 3 : lastGroup);
      multiplyGroup(2 * pair, cur0);
      multiplyGroup(2 * pair + 1, cur1);
    }
    if (groups & 1) multiplyGroup(lastGroup, next0);

    // accumulator layout: register r of lane l is row 4*(l/16) + r, column l%16
#pragma unroll
    for (int j = 0; j < TS; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const uint32_t row = (TALL ? x0 : j * 16) + 4 * (lane / 16) + r;
        const uint32_t col = (TALL ? j * 16 : x0) + lane % 16;
        if (row < p.M && col < p.N) storeResult(p, size_t(row) * p.N + col, acc[j][r]);
      }
  }
}

template <int TS, bool TA, bool TB, bool TALL, int WAVES>
int launchWaves(polar_hip_device* dev, SmallKArgs p, uint32_t groupsPerCu) {
  constexpr bool kShortKContig = TALL ? TB : !TA;
  using Short = ShortTile<kShortKContig>;
  constexpr int kBlock = WAVES * 16;
  p.pitch = Short::pitchFor(TS * 16, p.k4);
  const uint32_t bytes = Short::words(TS * 16, p.k4) * sizeof(float);
  auto kernel = smallKKernel<TS, TA, TB, TALL, WAVES>;
  // more dynamic LDS than the default limit has to be asked for, once per
  // kernel and device
  // (asking twice, from two threads at once, is harmless; launching before the
  // first request has returned is not, so the flag is set after it)
  static std::atomic<uint64_t> raised{0};
  const uint64_t bit = 1ull << (dev->ordinal & 63);
  if (bytes > 48 * 1024 && !(raised.load(std::memory_order_acquire) & bit)) {
    POLAR_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
    raised.fetch_or(bit, std::memory_order_release);
  }
  // one turn per group up to groupsPerCu groups per CU; beyond that groups take
  // several turns (and load the short operand once for all of them)
  const uint32_t longDim = TALL ? p.M : p.N;
  const uint32_t blocks = (longDim + kBlock - 1) / kBlock;
  const uint32_t slots = groupsPerCu * static_cast<uint32_t>(dev->info.compute_units);
  const uint32_t turns = (blocks + slots - 1) / slots;
  const uint32_t groups = (blocks + turns - 1) / turns;
  POLAR_HIP_TRY(launchKernelLds(dev, kernel, dim3(groups), dim3(WAVES * 64), bytes, p));
  return POLAR_HIP_OK;
}

// Sixteen waves per CU either way.  Long operands (from 32768 rows or columns)
// take them as two groups of eight, which halves the number of times the short
// operand is loaded: 65536 x 33 x 127 18.0 -> 16.7-17.1 us, 33 x 65536 x 127 16.5 ->
// 15.3-15.8 us.  Shorter ones keep four groups of four (8192 x 128 x 128: 15.8
// against 17.9 us with eight-wave groups).
template <int TS, bool TA, bool TB, bool TALL>
int launchConfig(polar_hip_device* dev, const SmallKArgs& p) {
  const uint32_t longDim = TALL ? p.M : p.N;
  if (longDim >= 32768) return launchWaves<TS, TA, TB, TALL, 8>(dev, p, 2);
  return launchWaves<TS, TA, TB, TALL, 4>(dev, p, 4);
}

template <int TS, bool TALL>
int launchLayouts(polar_hip_device* dev, const SmallKArgs& p, bool ta, bool tb) {
  if (!ta && !tb) return launchConfig<TS, false, false, TALL>(dev, p);
  if (!ta && tb) return launchConfig<TS, false, true, TALL>(dev, p);
  if (ta && !tb) return launchConfig<TS, true, false, TALL>(dev, p);
  return launchConfig<TS, true, true, TALL>(dev, p);
}

template <bool TALL>
int launchShortBlocks(polar_hip_device* dev, const SmallKArgs& p, bool ta, bool tb, uint32_t shortDim) {
  switch ((shortDim + 15) / 16) {
  case 1: return launchLayouts<1, TALL>(dev, p, ta, tb);
  case 2: return launchLayouts<2, TALL>(dev, p, ta, tb);
  case 3: return launchLayouts<3, TALL>(dev, p, ta, tb);
  case 4: return launchLayouts<4, TALL>(dev, p, ta, tb);
  case 5: return launchLayouts<5, TALL>(dev, p, ta, tb);
  case 6: return launchLayouts<6, TALL>(dev, p, ta, tb);
  case 7: return launchLayouts<7, TALL>(dev, p, ta, tb);
  default: return launchLayouts<8, TALL>(dev, p, ta, tb);
  }
}

constexpr uint32_t kShortMax = 128; // the short output dimension, at most 8 blocks of 16
constexpr uint32_t kLongMin = 1024; // below this the general kernel's tiles already fit

} // namespace

namespace polar_hip_detail {

bool smallKMatmulApplies(const MatmulCall& c) {
  if (c.K < 4 || c.K > kMaxK) return false; // a row of a k-contiguous operand is read 4 values at a time
  const bool tall = c.N <= kShortMax && c.M >= kLongMin;
  const bool wide = c.M <= kShortMax && c.N >= kLongMin;
  return tall || wide;
}

int launchSmallKMatmul(polar_hip_device* dev, const MatmulCall& c) {
  SmallKArgs p{};
  p.A = c.A;
  p.B = c.B;
  p.C = c.C;
  p.M = c.M;
  p.N = c.N;
  p.K = c.K;
  p.k4 = (c.K + 15) / 16 * 16; // whole groups of four k steps (see kOf in the kernel)
  p.epilogue = c.epilogue;
  p.bias = c.bias;
  p.scaleAcc = c.scaleAcc;
  p.scaleBias = c.scaleBias;
  POLAR_HIP_TRY(hipSetDevice(dev->ordinal));
  if (c.N <= kShortMax && c.M >= kLongMin) return launchShortBlocks<true>(dev, p, c.transA, c.transB, c.N);
  return launchShortBlocks<false>(dev, p, c.transA, c.transB, c.M);
}

} // namespace polar_hip_detail
