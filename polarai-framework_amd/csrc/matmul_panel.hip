// fmatmul for a short contraction (K <= 128) whose long output dimension is long
// enough to give every SIMD of the GPU a panel of its own: C[65536 x 33] =
// A[65536 x 127] * B[127 x 33], its mirror image, and C[65536 x 127] =
// A[65536 x 33] * B[33 x 127].
//
// Such a product streams the long operand and C through HBM once and gives the
// matrix cores about as much to do as the memory, so what decides its duration
// is whether the two overlap.  With many small waves that each load, multiply
// and store once (matmul_small_k.hip) they do not: the waves of a launch that
// fits the GPU in one round start together and pass through their phases in
// step.  Here one wave per SIMD owns a panel of 64 values of the long dimension
// with the whole of K and pipelines along k inside itself:
//   * all fetches of the panel are issued at once, before anything else waits
//     (up to 32 loads of 16 bytes per lane: 32 KB per wave in flight), in the
//     order of k;
//   * the matrix instructions of a group of 16 values of k start as soon as
//     that group's four loads are back (the hardware returns loads in order, so
//     the wait is a count of the younger loads), while the later groups are
//     still travelling;
//   * the panel is four 16 x 16 x 4 blocks side by side, so a fragment of the
//     short operand read from LDS feeds four matrix instructions, and for an
//     operand whose long dimension is contiguous in memory one 16-byte load
//     brings the four blocks' values of one k: block i holds the values
//     x0 + 4*fx + i of the long dimension (fx = lane % 16);
//   * results leave as 16-byte stores: a wide C (long N) straight from the
//     accumulators, because a lane's four blocks are four neighbouring columns;
//     a tall C (long M) is put together in LDS first, since the panel's 64 rows
//     of C are one contiguous piece of memory whatever N is.
// The short operand goes into LDS once per work-group; its loads are issued
// before the panel's (loads return in order: issued after them, they would
// hold back the first matrix instruction until the whole panel had arrived).
// Every element of C is accumulated by one lane in k order: the result does not
// depend on scheduling.
#include "internal.h"
#include "matmul_epilogue.h"

using namespace polar_hip_detail;

namespace {

typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kWaves = 4;            // one per SIMD
constexpr int kThreads = kWaves * 64;
constexpr uint32_t kSpan = 64;       // values of the long dimension per wave
constexpr uint32_t kGroupSpan = kSpan * kWaves;
constexpr uint32_t kMaxLds = 160 * 1024;

struct PanelArgs {
  const float* A;
  const float* B;
  float* C;
  uint32_t M, N, K;
  uint32_t k4;          // K rounded up to a multiple of 16
  uint32_t shortWords;  // size of that tile, in floats (a multiple of 4)
  uint32_t stageWords;  // per-wave staging area for a tall C, in floats
  int epilogue;
  const float* bias;
  float scaleAcc, scaleBias;
};

// w shifted down by d elements, zeros moving in from the top (d >= 4: all
// zeros).  Written with bit masks: as nested selects the compiler turns it into
// divergent branches.
__device__ __forceinline__ v4f shiftDown(v4f w, uint32_t d) {
  typedef uint32_t v4u __attribute__((ext_vector_type(4)));
  const v4u b = __builtin_bit_cast(v4u, w);
  const uint32_t m0 = d == 0 ? ~0u : 0u, m1 = d == 1 ? ~0u : 0u, m2 = d == 2 ? ~0u : 0u, m3 = d == 3 ? ~0u : 0u;
  v4u r;
  r[0] = (b[0] & m0) | (b[1] & m1) | (b[2] & m2) | (b[3] & m3);
  r[1] = (b[1] & m0) | (b[2] & m1) | (b[3] & m2);
  r[2] = (b[2] & m0) | (b[3] & m1);
  r[3] = b[3] & m0;
  return __builtin_bit_cast(v4f, r);
}

__device__ __forceinline__ v4f loadUnaligned(const float* p) {
  return *reinterpret_cast<const v4f __attribute__((aligned(4)))*>(p);
}

// Size (in floats) of the short operand's tile in LDS: GROUPS x TS blocks of 64
// 16-byte words.
constexpr uint32_t panelTileWords(int ts, int groups) { return uint32_t(groups) * ts * 256; }

// TS blocks of 16 of the short dimension go through the matrix instruction,
// GROUPS groups of 16 cover K.  TALL: M is the long dimension (B is the short
// operand); otherwise N is.  XS: the short dimension is 16 TS + 1, and its last
// row or column is a dot product on the vector ALUs (33 as three blocks would
// spend a third of the matrix instructions on 15 rows of padding); otherwise
// it is at most 16 TS.
template <int TS, int GROUPS, bool TA, bool TB, bool TALL, bool XS>
__global__ __launch_bounds__(kThreads) void panelKernel(PanelArgs p) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  constexpr bool kShortKContig = TALL ? TB : !TA;
  constexpr bool kLongKContig = TALL ? !TA : TB;
  // loads of the short operand per lane: all of it in one go (at most 8192 values)
  constexpr int SU = (TS * 16 + (XS ? 1 : 0)) * GROUPS * 16 < 8192 ? ((TS * 16 + (XS ? 1 : 0)) * GROUPS * 16 + kThreads - 1) / kThreads : 32;
  // groups of k whose loads are in flight ahead of the matrix instructions
#ifndef PANEL_AHEAD
#define PANEL_AHEAD 4
#endif
  constexpr int kAhead = GROUPS < PANEL_AHEAD ? GROUPS : PANEL_AHEAD;

  const float* const longX = TALL ? p.A : p.B;
  const float* const shortX = TALL ? p.B : p.A;
  const uint32_t longDim = TALL ? p.M : p.N, shortDim = TALL ? p.N : p.M;
  const int t = threadIdx.x, lane = t % 64;
  const int wave = __builtin_amdgcn_readfirstlane(t / 64); // uniform, and known to be
  const uint32_t fx = lane % 16, fk = lane / 16;
  const uint32_t x0 = blockIdx.x * kGroupSpan + wave * kSpan; // this wave's panel

  // 1. the short operand: loads only (a fixed number per lane; slots beyond the
  // operand repeat its last value and are not placed)
  const uint32_t shortTotal = shortDim * p.K;
  float sv[SU];
#pragma unroll
  for (int u = 0; u < SU; ++u) {
    const uint32_t e = t + u * kThreads;
    sv[u] = shortX[e < shortTotal ? e : shortTotal - 1];
  }
  // keep the three phases apart: left to itself the compiler interleaves the
  // short operand's loads with their LDS stores, a few at a time with a wait
  // each, and issues the panel's loads after the last of those round trips
  __builtin_amdgcn_sched_barrier(0);

  // 2. the panel: the loads of its first kAhead groups of k.  A fixed number of
  // loads whatever the lane and no arithmetic on what they bring (addresses are
  // clamped into the operand; what was clamped is put right when the group is
  // used), so that the waits below are plain counts.  A wave whose panel lies
  // beyond the operand loads the last panel again and stores nothing.
  const uint32_t xLoad = x0 < longDim ? x0 : (longDim - 1) / kSpan * kSpan;
  v4f buf[GROUPS][4];
  // Byte offsets of all loads, computed here once (the operand is smaller than
  // 4 GiB): between two groups of matrix instructions there is then nothing but
  // the loads themselves, each the operand's base plus a 32-bit lane offset.
  uint32_t at[GROUPS][4];
#pragma unroll
  for (int g = 0; g < GROUPS; ++g) {
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      if constexpr (kLongKContig) {
        // block s: row xLoad + 4 fx + s, the four values k .. k+3, k = 16 g + 4 fk
        // (steps 0..3 of the group for this lane); near the end of the row the
        // last four of the row are loaded instead
        const uint32_t x = xLoad + 4 * fx + s;
        const uint32_t row = x < longDim ? x : longDim - 1;
        const uint32_t k = 16 * g + 4 * fk;
        const uint32_t from = k + 4 <= p.K ? k : p.K - 4; // K >= 4
        at[g][s] = (row * p.K + from) * 4;
      } else {
        // step s: row k = 16 g + 4 s + fk of the operand, the four values
        // xLoad + 4 fx .. + 3 (blocks 0..3 for this lane)
        const uint32_t k = 16 * g + 4 * s + fk;
        const uint32_t x = xLoad + 4 * fx;
        const uint32_t from = x + 4 <= longDim ? x : longDim - 4; // longDim >= 4
        at[g][s] = ((k < p.K ? k : p.K - 1) * longDim + from) * 4;
      }
    }
  }
  auto fetch = [&](int g) {
#pragma unroll
    for (int s = 0; s < 4; ++s)
      buf[g][s] = loadUnaligned(reinterpret_cast<const float*>(reinterpret_cast<const char*>(longX) + at[g][s]));
  };
#pragma unroll
  for (int g = 0; g < kAhead; ++g) fetch(g);

  __builtin_amdgcn_sched_barrier(0);

  // 3. the short operand into LDS (waits for its own loads only: they are
  // older), in the order the matrix instructions want it: the four values of k
  // that a lane multiplies in the four steps of a group are one 16-byte word,
  // the words of a group and block of 16 x are in lane order.  Element (x, k)
  // with x = 16 j + fx and k = 16 g + r goes to word ((g TS + j) 64 + 16 fk + fx),
  // component c, where r = 4 fk + c (long operand read along k) or r = 4 c + fk.
  // The extra row or column follows the blocks, 16 values per group, in the
  // order the lanes multiply them (lane group fk: words 16 g + 4 fk .. + 3).
  constexpr uint32_t kBlockWords = panelTileWords(TS, GROUPS);
  auto tileAt = [&](uint32_t x, uint32_t k) -> uint32_t {
    const uint32_t r = k % 16;
    if (XS && x == TS * 16) return kBlockWords + k / 16 * 16 + (kLongKContig ? r : 4 * (r % 4) + r / 4);
    const uint32_t kLane = kLongKContig ? r / 4 : r % 4, c = kLongKContig ? r % 4 : r / 4;
    return (((k / 16) * TS + x / 16) * 64 + kLane * 16 + x % 16) * 4 + c;
  };
  {
    const uint32_t rowLen = kShortKContig ? p.K : shortDim;
    uint32_t row = uint32_t(t) / rowLen, col = uint32_t(t) % rowLen;
    const uint32_t stepRow = uint32_t(kThreads) / rowLen, stepCol = uint32_t(kThreads) % rowLen;
    // no branch around a store (the compiler would move the load into it, behind
    // the panel's loads): a slot beyond the operand stores the last value again
    const uint32_t lastAt = tileAt(shortDim - 1, p.K - 1);
#pragma unroll
    for (int u = 0; u < SU; ++u) {
      const uint32_t here = kShortKContig ? tileAt(row, col) : tileAt(col, row);
      lds[t + u * kThreads < shortTotal ? here : lastAt] = sv[u];
      col += stepCol;
      row += stepRow;
      if (col >= rowLen) {
        col -= rowLen;
        ++row;
      }
    }
    // k in [K, k4) is multiplied (whole groups only), so it holds zeros
    const uint32_t padK = p.k4 - p.K, xPadded = TS * 16 + (XS ? 1 : 0);
    for (uint32_t e = t; e < padK * xPadded; e += kThreads) lds[tileAt(e % xPadded, p.K + e / xPadded)] = 0.0f;
  }
  __syncthreads();
  if (x0 >= longDim) return;

  // 4. multiply, group by group as the loads come back
  v4f acc[4][TS];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < TS; ++j) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};
  // a clamped load is put right here: values beyond the operand become zeros.
  // Only the last group of K and the last panel of the long dimension have any,
  // and both conditions are uniform.
  const bool lastPanel = xLoad + kSpan > longDim;
  auto settle = [&](int g) {
    if constexpr (kLongKContig) {
      if (16u * (g + 1) > p.K) {
        const uint32_t k = 16 * g + 4 * fk;
        const uint32_t from = k + 4 <= p.K ? k : p.K - 4;
#pragma unroll
        for (int s = 0; s < 4; ++s) buf[g][s] = shiftDown(buf[g][s], k - from);
      }
    } else {
      if (lastPanel) {
        const uint32_t x = xLoad + 4 * fx;
        const uint32_t from = x + 4 <= longDim ? x : longDim - 4;
#pragma unroll
        for (int s = 0; s < 4; ++s) buf[g][s] = shiftDown(buf[g][s], x < longDim ? x - from : 4);
      }
      if (16u * (g + 1) > p.K) {
#pragma unroll
        for (int s = 0; s < 4; ++s)
          if (16 * g + 4 * s + fk >= p.K) buf[g][s] = v4f{0.f, 0.f, 0.f, 0.f};
      }
    }
  };
  // The short operand's fragments of a group are TS 16-byte reads at the lane's
  // base plus a constant, issued a group ahead.  With one wave per SIMD every
  // instruction between two matrix instructions is time the matrix pipe idles
  // (a branch costs about 70 cycles, an LDS read 16), so a group that lies
  // wholly inside K is 48 matrix instructions and nothing else.
  const v4f* const tile = reinterpret_cast<const v4f*>(lds) + lane;
  v4f frag[2][TS];
#pragma unroll
  for (int j = 0; j < TS; ++j) frag[0][j] = tile[j * 64];
  float part[4] = {0.0f, 0.0f, 0.0f, 0.0f};  // XS: the lane's share of the extra row or column, per block
#pragma unroll
  for (int g = 0; g < GROUPS; ++g) {
    if (16u * g < p.K) {
      // The loads of a group leave kAhead groups before it is used, from inside
      // the stream of matrix instructions: a wave that issued them all up front
      // would sit in that queue (the memory pipeline takes them at the rate it
      // delivers) while the matrix pipe waits for its first instruction.
      if (g + kAhead < GROUPS) fetch(g + kAhead);
      if (g + 1 < GROUPS) {
#pragma unroll
        for (int j = 0; j < TS; ++j) frag[(g + 1) & 1][j] = tile[((g + 1) * TS + j) * 64];
      }
      __builtin_amdgcn_sched_barrier(0);
      settle(g);
      v4f ax = {0.f, 0.f, 0.f, 0.f};
      if constexpr (XS) ax = *reinterpret_cast<const v4f*>(lds + kBlockWords + 16 * g + 4 * fk);
      auto step = [&](int c) {
        if constexpr (XS) {
#pragma unroll
          for (int i = 0; i < 4; ++i) part[i] = __builtin_fmaf(kLongKContig ? buf[g][i][c] : buf[g][c][i], ax[c], part[i]);
        }
#pragma unroll
        for (int j = 0; j < TS; ++j) {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float mine = kLongKContig ? buf[g][i][c] : buf[g][c][i];
            const float other = frag[g & 1][j][c];
            acc[i][j] = TALL ? __builtin_amdgcn_mfma_f32_16x16x4f32(mine, other, acc[i][j], 0, 0, 0)
                             : __builtin_amdgcn_mfma_f32_16x16x4f32(other, mine, acc[i][j], 0, 0, 0);
          }
        }
      };
      // the first of the four values of k that a step multiplies tells whether any is inside K
      auto kFirst = [&](int c) -> uint32_t { return kLongKContig ? 16 * g + c : 16 * g + 4 * c; };
      if (kFirst(3) < p.K) {
#pragma unroll
        for (int c = 0; c < 4; ++c) step(c);
      } else {
        step(0);
#pragma unroll
        for (int c = 1; c < 4; ++c)
          if (kFirst(c) < p.K) step(c);
      }
    }
  }

  // 5. store.  Accumulator layout: register r of lane l is row 4*(l/16) + r,
  // column l%16 of the 16 x 16 block.
  const uint32_t q = lane / 16;
  float extra[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  if constexpr (XS) {
    // the four lanes that hold the same four values of the long dimension (one
    // per fk) add their shares, in a fixed order
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float p0 = __shfl(part[i], fx), p1 = __shfl(part[i], fx + 16), p2 = __shfl(part[i], fx + 32),
                  p3 = __shfl(part[i], fx + 48);
      extra[i] = ((p0 + p1) + p2) + p3;
    }
  }
  if constexpr (TALL) {
    // block i, row index m = 4q + r of the block  ->  row x0 + 4m + i of C
    float* const stage = lds + p.shortWords + wave * p.stageWords;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < TS; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const uint32_t local = 4 * (4 * q + r) + i, col = j * 16 + fx;
          if (XS || col < p.N) {
            float v = acc[i][j][r];
            if (p.epilogue != kEpiNone && x0 + local < longDim)
              v = applyEpilogue(p.epilogue, v, p.bias, p.scaleAcc, p.scaleBias, size_t(x0 + local) * p.N + col);
            stage[local * p.N + col] = v;
          }
        }
    if constexpr (XS) {
      // lanes 0..15 hold the extra column of rows x0 + 4 fx + i
      if (fk == 0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float v = extra[i];
          if (p.epilogue != kEpiNone && x0 + 4 * fx + i < longDim)
            v = applyEpilogue(p.epilogue, v, p.bias, p.scaleAcc, p.scaleBias, size_t(x0 + 4 * fx + i) * p.N + TS * 16);
          stage[(4 * fx + i) * p.N + TS * 16] = v;
        }
      }
    }
    // the wave's own writes, read back by other lanes of the same wave: LDS
    // serves a wave's accesses in order
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    const uint32_t rows = longDim - x0 < kSpan ? longDim - x0 : kSpan;
    const uint32_t count = rows * p.N;
    float* const out = p.C + size_t(x0) * p.N;
    if ((reinterpret_cast<uintptr_t>(out) & 15u) == 0) {
      // four 16-byte pieces per lane and turn, read from LDS together
      for (uint32_t base = lane * 4; base < count; base += 1024) {
        v4f piece[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const uint32_t v = base + 256 * u;
          piece[u] = *reinterpret_cast<const v4f*>(stage + (v + 4 <= count ? v : 0));
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const uint32_t v = base + 256 * u;
          if (v + 4 <= count) *reinterpret_cast<v4f*>(out + v) = piece[u];
        }
      }
      const uint32_t tail = count & ~3u;
      if (lane < count - tail) out[tail + lane] = stage[tail + lane];
    } else {
      for (uint32_t v = lane; v < count; v += 64) out[v] = stage[v];
    }
  } else {
    // block i, column index fx of the block  ->  column x0 + 4 fx + i of C
    const uint32_t col = x0 + 4 * fx;
    const bool whole = col + 4 <= p.N;
#pragma unroll
    for (int j = 0; j < TS + (XS ? 1 : 0); ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        // the extra row is held by lanes 0..15, all four columns in one lane
        if (j == TS && r > 0) continue;
        const uint32_t row = j == TS ? TS * 16 : j * 16 + 4 * q + r;
        if (j == TS ? fk == 0 : row < p.M) {
          const size_t idx = size_t(row) * p.N + col;
          v4f v = {extra[0], extra[1], extra[2], extra[3]};
          if (j < TS) v = v4f{acc[0][j < TS ? j : 0][r], acc[1][j < TS ? j : 0][r], acc[2][j < TS ? j : 0][r], acc[3][j < TS ? j : 0][r]};
          if (p.epilogue != kEpiNone) {
#pragma unroll
            for (int i = 0; i < 4; ++i)
              if (col + i < p.N) v[i] = applyEpilogue(p.epilogue, v[i], p.bias, p.scaleAcc, p.scaleBias, idx + i);
          }
          if (whole && (reinterpret_cast<uintptr_t>(p.C + idx) & 15u) == 0) {
            *reinterpret_cast<v4f*>(p.C + idx) = v;
          } else {
#pragma unroll
            for (int i = 0; i < 4; ++i)
              if (col + i < p.N) p.C[idx + i] = v[i];
          }
        }
      }
  }
}

template <int TS, int GROUPS, bool TA, bool TB, bool TALL, bool XS>
int launchPanel(polar_hip_device* dev, PanelArgs p) {
  p.shortWords = panelTileWords(TS, GROUPS) + (XS ? GROUPS * 16 : 0);
  p.stageWords = TALL ? (kSpan * p.N + 3) / 4 * 4 : 0;
  const uint32_t bytes = (p.shortWords + kWaves * p.stageWords) * sizeof(float);
  auto kernel = panelKernel<TS, GROUPS, TA, TB, TALL, XS>;
  // more dynamic LDS than the default limit has to be asked for, once per
  // kernel and device (asking twice is harmless)
  static std::atomic<uint64_t> raised{0};
  const uint64_t bit = 1ull << (dev->ordinal & 63);
  if (bytes > 48 * 1024 && !(raised.load(std::memory_order_acquire) & bit)) {
    POLAR_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, int(kMaxLds)));
    raised.fetch_or(bit, std::memory_order_release);
  }
  const uint32_t longDim = TALL ? p.M : p.N;
  const uint32_t groups = (longDim + kGroupSpan - 1) / kGroupSpan;
  POLAR_HIP_TRY(launchKernelLds(dev, kernel, dim3(groups), dim3(kThreads), bytes, p));
  return POLAR_HIP_OK;
}

template <int TS, int GROUPS, bool TALL, bool XS>
int launchStored(polar_hip_device* dev, const PanelArgs& p, bool ta, bool tb) {
  if (!ta && !tb) return launchPanel<TS, GROUPS, false, false, TALL, XS>(dev, p);
  if (!ta && tb) return launchPanel<TS, GROUPS, false, true, TALL, XS>(dev, p);
  if (ta && !tb) return launchPanel<TS, GROUPS, true, false, TALL, XS>(dev, p);
  return launchPanel<TS, GROUPS, true, true, TALL, XS>(dev, p);
}

template <int TS, int GROUPS, bool TALL>
int launchLayouts(polar_hip_device* dev, const PanelArgs& p, bool ta, bool tb) {
  if constexpr (TS <= 4) {
    if ((TALL ? p.N : p.M) == TS * 16 + 1) return launchStored<TS, GROUPS, TALL, true>(dev, p, ta, tb);
  }
  return launchStored<TS, GROUPS, TALL, false>(dev, p, ta, tb);
}

// blocks of 16 of the short dimension that go through the matrix instruction:
// one row or column beyond up to four whole blocks is computed on the vector ALUs
uint32_t blocksFor(uint32_t n) { return n > 16 && n <= 65 && n % 16 == 1 ? n / 16 : (n + 15) / 16; }

template <bool TALL>
int launchBlocks(polar_hip_device* dev, const PanelArgs& p, bool ta, bool tb, uint32_t shortDim) {
  const bool deep = p.k4 > 64;
  switch (blocksFor(shortDim)) {
  case 1: return deep ? launchLayouts<1, 8, TALL>(dev, p, ta, tb) : launchLayouts<1, 4, TALL>(dev, p, ta, tb);
  case 2: return deep ? launchLayouts<2, 8, TALL>(dev, p, ta, tb) : launchLayouts<2, 4, TALL>(dev, p, ta, tb);
  case 3: return deep ? launchLayouts<3, 8, TALL>(dev, p, ta, tb) : launchLayouts<3, 4, TALL>(dev, p, ta, tb);
  case 4: return deep ? launchLayouts<4, 8, TALL>(dev, p, ta, tb) : launchLayouts<4, 4, TALL>(dev, p, ta, tb);
  case 5: return launchLayouts<5, 4, TALL>(dev, p, ta, tb);
  case 6: return launchLayouts<6, 4, TALL>(dev, p, ta, tb);
  case 7: return launchLayouts<7, 4, TALL>(dev, p, ta, tb);
  default: return launchLayouts<8, 4, TALL>(dev, p, ta, tb);
  }
}

constexpr uint32_t kShortMax = 128;
constexpr uint32_t kShortValuesMax = 8192; // what one round of loads brings into LDS

} // namespace

namespace polar_hip_detail {

bool panelMatmulApplies(const MatmulCall& c, int computeUnits) {
  if (c.K < 4 || c.K > 128) return false;
  const uint32_t longMin = kGroupSpan * uint32_t(computeUnits) * 3 / 4; // most of the SIMDs get a panel
  const bool tall = c.N <= kShortMax && c.M >= longMin;
  const bool wide = c.M <= kShortMax && c.N >= longMin;
  if (!tall && !wide) return false;
  const uint32_t shortDim = tall ? c.N : c.M;
  const uint32_t blocks = blocksFor(shortDim), k4 = (c.K + 15) / 16 * 16;
  if (blocks > 4 && k4 > 64) return false;
  if (shortDim * c.K > kShortValuesMax) return false;
  if (uint64_t(tall ? c.M : c.N) * c.K * sizeof(float) >= (1ull << 32)) return false; // 32-bit load offsets
  // LDS: the short operand's tile (either orientation) and, for a tall C, the staging areas
  const uint32_t tileWords = panelTileWords(int(blocks), k4 > 64 ? 8 : 4);
  const uint32_t stage = tall ? kWaves * (kSpan * c.N + 4) : 0;
  return (tileWords + 128 + stage) * sizeof(float) <= kMaxLds;
}

int launchPanelMatmul(polar_hip_device* dev, const MatmulCall& c) {
  PanelArgs p{};
  p.A = c.A;
  p.B = c.B;
  p.C = c.C;
  p.M = c.M;
  p.N = c.N;
  p.K = c.K;
  p.k4 = (c.K + 15) / 16 * 16;
  p.epilogue = c.epilogue;
  p.bias = c.bias;
  p.scaleAcc = c.scaleAcc;
  p.scaleBias = c.scaleBias;
  POLAR_HIP_TRY(hipSetDevice(dev->ordinal));
  const bool tall = c.N <= kShortMax && c.M >= c.N;
  if (tall) return launchBlocks<true>(dev, p, c.transA, c.transB, c.N);
  return launchBlocks<false>(dev, p, c.transA, c.transB, c.M);
}

} // namespace polar_hip_detail
