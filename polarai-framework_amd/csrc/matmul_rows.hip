// fmatmul for a short contraction (K <= 128), a long M and a short N, A stored
// row by row ([M x K], not transposed): C[65536 x 33] = A[65536 x 127] * B[127 x 33]
// and C[65536 x 127] = A[65536 x 33] * B[33 x 127].
//
// A row of A is a few hundred bytes whose pitch is not a multiple of a cache
// line, and the matrix instruction wants 16 different rows in 16 neighbouring
// lanes.  Loaded straight into that layout (16 bytes per lane, every lane in a
// row of its own: matmul_panel.hip) each load instruction touches 64 cache
// lines, and the address unit, which takes about one line per cycle, becomes
// the bound.  Here a wave owns 32 consecutive rows of A, which are ONE
// contiguous piece of memory, and fetches them as such: 1 KiB per load
// instruction, eight lines.  The piece goes through the wave's own area of LDS
// (written as it was read, 16 bytes per lane and conflict-free) and comes back
// in the matrix instruction's layout, four consecutive k of one row per lane.
//   * All loads of a wave (at most 16 per lane) are issued at once, before
//     anything else waits.  The first 16 rows are multiplied while the second
//     16 are still arriving, and their results leave while the second 16 are
//     multiplied: three stages, eight waves per CU, two per SIMD, so that one
//     wave's waits are the other's matrix instructions.
//   * The short operand B is put into LDS once per work-group, in fragment
//     order, and every wave then holds all of it in registers (TS x GROUPS
//     16-byte words per lane): the loop over k reads nothing but A.
//   * 16 rows of C are one contiguous piece of memory whatever N is; they are
//     put together in LDS and leave as 16-byte stores.
// Every element of C is accumulated by one lane in k order.
#include "internal.h"
#include "matmul_epilogue.h"

using namespace polar_hip_detail;

namespace {

typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kWaves = 8;
constexpr int kThreads = kWaves * 64;
constexpr uint32_t kRows = 32;  // rows of A per wave: two blocks of 16
constexpr uint32_t kGroupRows = kRows * kWaves;
constexpr uint32_t kMaxLds = 160 * 1024;

// w shifted down by d elements (d in 1..3), zeros moving in from the top
__device__ __forceinline__ v4f shiftDown(v4f w, uint32_t d) {
  v4f r;
  r[0] = d == 1 ? w[1] : d == 2 ? w[2] : w[3];
  r[1] = d == 1 ? w[2] : d == 2 ? w[3] : 0.0f;
  r[2] = d == 1 ? w[3] : 0.0f;
  r[3] = 0.0f;
  return r;
}

struct RowsArgs {
  const float* A;
  const float* B;
  float* C;
  uint32_t M, N, K;
  uint32_t k4;          // K rounded up to a multiple of 16
  uint32_t tileWords;   // the short operand's tile in LDS, in floats
  uint32_t areaWords;   // a wave's area of LDS (its rows of A, later rows of C), in floats
  int epilogue;
  const float* bias;
  float scaleAcc, scaleBias;
};

// TS blocks of 16 columns go through the matrix instruction; GROUPS = ceil(K / 16)
// exactly.  TB: B is stored [N x K].  XCOL: N = 16 TS + 1, and the one column
// beyond the blocks is a dot product on the vector ALUs (33 columns as three
// blocks would spend a third of the matrix instructions on 15 columns of
// padding); otherwise N <= 16 TS.
template <int TS, int GROUPS, bool TB, bool XCOL>
__global__ __launch_bounds__(kThreads) void rowsKernel(RowsArgs p) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  constexpr int SU = ((TS * 16 + (XCOL ? 1 : 0)) * GROUPS * 16 + kThreads - 1) / kThreads;  // loads of B per lane
  constexpr int LOADS = 2 * GROUPS;  // 16-byte loads of A per lane: 32 rows x at most 16 GROUPS floats

  const int t = threadIdx.x, lane = t % 64;
  const int wave = __builtin_amdgcn_readfirstlane(t / 64);
  const uint32_t fx = lane % 16, fk = lane / 16;
  const uint32_t x0 = blockIdx.x * kGroupRows + wave * kRows;  // this wave's first row
  const bool active = x0 < p.M;

  // 1. B: loads only (a fixed number per lane; a slot beyond B repeats its last value)
  const uint32_t shortTotal = p.N * p.K;
  float sv[SU];
#pragma unroll
  for (int u = 0; u < SU; ++u) {
    const uint32_t e = t + u * kThreads;
    sv[u] = p.B[e < shortTotal ? e : shortTotal - 1];
  }
  __builtin_amdgcn_sched_barrier(0);

  // 2. the wave's rows of A, as the contiguous piece of memory they are.  The
  // piece starts on a 16-byte boundary (32 K floats per wave, A itself is
  // aligned); past its end the last 16 bytes of A are loaded again.
  const uint32_t rows = active ? (p.M - x0 < kRows ? p.M - x0 : kRows) : 0;
  const uint32_t pieceFloats = rows * p.K;
  const float* const piece = p.A + size_t(active ? x0 : 0) * p.K;
  const uint32_t lastWord = (active ? pieceFloats : p.K) - 4;  // K >= 4
  v4f in[LOADS];
  auto fetchRows = [&](int b) {
#pragma unroll
    for (int u = b * GROUPS; u < (b + 1) * GROUPS; ++u) {
      const uint32_t at = (u * 64 + lane) * 4;
      in[u] = *reinterpret_cast<const v4f __attribute__((aligned(4)))*>(piece + (at + 4 <= pieceFloats ? at : lastWord));
    }
  };
  // The first block's loads go out now, the second block's after B has been
  // placed: the memory pipeline takes loads at the rate it delivers, and B's
  // loads must not sit behind all of A in that queue.
  fetchRows(0);
  __builtin_amdgcn_sched_barrier(0);

  // 3. B into LDS in the order the matrix instructions want it: element (n, k)
  // with n = 16 j + fx, k = 16 g + 4 fk + c goes to 16-byte word
  // ((g TS + j) 64 + 16 fk + fx), component c.
  // The extra column's values follow the blocks in the order of k.
  constexpr uint32_t kBlockWords = uint32_t(GROUPS) * TS * 256;
  auto tileAt = [&](uint32_t n, uint32_t k) -> uint32_t {
    if (XCOL && n == TS * 16) return kBlockWords + k;
    return (((k / 16) * TS + n / 16) * 64 + (k % 16) / 4 * 16 + n % 16) * 4 + k % 4;
  };
  {
    const uint32_t rowLen = TB ? p.K : p.N;
    uint32_t row = uint32_t(t) / rowLen, col = uint32_t(t) % rowLen;
    const uint32_t stepRow = uint32_t(kThreads) / rowLen, stepCol = uint32_t(kThreads) % rowLen;
    // no branch around a store (the compiler would move the load into it, behind
    // the loads of A): a slot beyond B stores the last value again
    const uint32_t lastAt = tileAt(p.N - 1, p.K - 1);
#pragma unroll
    for (int u = 0; u < SU; ++u) {
      const uint32_t here = TB ? tileAt(row, col) : tileAt(col, row);
      lds[t + u * kThreads < shortTotal ? here : lastAt] = sv[u];
      col += stepCol;
      row += stepRow;
      if (col >= rowLen) {
        col -= rowLen;
        ++row;
      }
    }
    // k in [K, 16 GROUPS) is multiplied, so it holds zeros
    const uint32_t padK = GROUPS * 16 - p.K, nPadded = TS * 16 + (XCOL ? 1 : 0);
    for (uint32_t e = t; e < padK * nPadded; e += kThreads) lds[tileAt(e % nPadded, p.K + e / nPadded)] = 0.0f;
  }
  __syncthreads();
  if (!active) return;

  fetchRows(1);
  __builtin_amdgcn_sched_barrier(0);

  // 4. all of B into registers
  v4f bq[GROUPS][TS];
  {
    const v4f* const tile = reinterpret_cast<const v4f*>(lds) + lane;
#pragma unroll
    for (int g = 0; g < GROUPS; ++g)
#pragma unroll
      for (int j = 0; j < TS; ++j) bq[g][j] = tile[(g * TS + j) * 64];
  }
  v4f bx[XCOL ? GROUPS : 1];  // the extra column: the lane's four k of every group
  if constexpr (XCOL) {
#pragma unroll
    for (int g = 0; g < GROUPS; ++g) bx[g] = *reinterpret_cast<const v4f*>(lds + kBlockWords + 16 * g + 4 * fk);
  }

  // 5. block by block: rows into LDS, multiply, rows of C out
  float* const area = lds + p.tileWords + wave * p.areaWords;
  const uint32_t q = lane / 16;

  // the loads that hold block b's rows (16 K floats from 16 b K on; the second
  // block's first row may begin in the first block's last load)
  auto placeRows = [&](int b) {
    if (pieceFloats % 4 != 0) {
      // (only the last wave of a matrix whose size is not a multiple of four
      // floats) the 16 bytes that straddle the end of A were loaded from 4 - d
      // floats earlier: move them down to where they belong
#pragma unroll
      for (int u = b * GROUPS; u < (b + 1) * GROUPS; ++u) {
        const uint32_t at = (u * 64 + lane) * 4;
        if (at < pieceFloats && at + 4 > pieceFloats) in[u] = shiftDown(in[u], at - lastWord);
      }
    }
#pragma unroll
    for (int u = b * GROUPS; u < (b + 1) * GROUPS; ++u)
      *reinterpret_cast<v4f*>(area + (u * 64 + lane) * 4) = in[u];
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // LDS serves a wave's accesses in order
  };

  auto multiply = [&](int b, v4f (&acc)[TS], float& extra) {
    const float* const mine = area + (16 * b + fx) * p.K + 4 * fk;  // row 16 b + fx, k = 4 fk
#pragma unroll
    for (int j = 0; j < TS; ++j) acc[j] = v4f{0.f, 0.f, 0.f, 0.f};
    float part = 0.0f;
    v4f af[2];
    af[0] = *reinterpret_cast<const v4f __attribute__((aligned(4)))*>(mine);
#pragma unroll
    for (int g = 0; g < GROUPS; ++g) {
      if (g + 1 < GROUPS) af[(g + 1) & 1] = *reinterpret_cast<const v4f __attribute__((aligned(4)))*>(mine + 16 * (g + 1));
      v4f a = af[g & 1];
      if (g == GROUPS - 1) {
        // beyond K the area holds the next row (or nothing): zeros instead
#pragma unroll
        for (int c = 0; c < 4; ++c)
          if (16 * g + 4 * fk + c >= p.K) a[c] = 0.0f;
      }
#pragma unroll
      for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int j = 0; j < TS; ++j) acc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[c], bq[g][j][c], acc[j], 0, 0, 0);
      if constexpr (XCOL) {
#pragma unroll
        for (int c = 0; c < 4; ++c) part = __builtin_fmaf(a[c], bx[g][c], part);
      }
    }
    if constexpr (XCOL) {
      // the four lanes that hold row fx (one per fk) add their parts, in a fixed order
      const float p1 = __shfl(part, fx + 16), p2 = __shfl(part, fx + 32), p3 = __shfl(part, fx + 48);
      const float p0 = __shfl(part, fx);
      extra = ((p0 + p1) + p2) + p3;
    }
  };

  // A block's 16 rows of C are put together in LDS -- over the block's rows of A
  // when they fit there (N <= K), behind the wave's rows of A otherwise -- and
  // leave as one contiguous piece.  Accumulator layout: register r of lane l is
  // row 4 (l / 16) + r, column l % 16.
  auto storeBlock = [&](int b, const v4f (&acc)[TS], float extra) {
    float* const stage = p.N <= p.K ? area + 16 * b * p.K : area + LOADS * 256;
    const uint32_t blockRows = rows - 16 * b < 16 ? rows - 16 * b : 16;
    // no branch per element (with two waves per SIMD a branch still costs the
    // wave about 70 cycles): the fused epilogue is one uniform branch around the
    // whole block, and a column beyond N -- only the last block of 16 columns
    // has any -- goes to a spare word behind the wave's area
    float* const spare = area + p.areaWords - 4;
    auto put = [&](auto&& value) {
#pragma unroll
      for (int j = 0; j < TS; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const uint32_t local = 4 * q + r, col = j * 16 + fx;
          float* const to = (XCOL || j < TS - 1 || col < p.N) ? stage + local * p.N + col : spare;
          *to = value(j, r, local, col);
        }
    };
    if constexpr (XCOL) {
      // lanes 0..15 hold the extra column of rows 0..15 of the block
      float v = extra;
      if (p.epilogue != kEpiNone && fx < blockRows)
        v = applyEpilogue(p.epilogue, v, p.bias, p.scaleAcc, p.scaleBias, size_t(x0 + 16 * b + fx) * p.N + TS * 16);
      *(fk == 0 ? stage + fx * p.N + TS * 16 : spare) = v;
    }
    if (p.epilogue == kEpiNone) {
      put([&](int j, int r, uint32_t, uint32_t) { return acc[j][r]; });
    } else {
      put([&](int j, int r, uint32_t local, uint32_t col) {
        const bool inside = local < blockRows && col < p.N;  // bias is read only where C exists
        return inside ? applyEpilogue(p.epilogue, acc[j][r], p.bias, p.scaleAcc, p.scaleBias,
                                      size_t(x0 + 16 * b + local) * p.N + col)
                      : 0.0f;
      });
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    const uint32_t count = blockRows * p.N;
    float* const out = p.C + size_t(x0 + 16 * b) * p.N;
    if ((reinterpret_cast<uintptr_t>(out) & 15u) == 0) {
      for (uint32_t base = lane * 4; base < count; base += 1024) {
        v4f part[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const uint32_t v = base + 256 * u;
          part[u] = *reinterpret_cast<const v4f*>(stage + (v + 4 <= count ? v : 0));
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const uint32_t v = base + 256 * u;
          if (v + 4 <= count) *reinterpret_cast<v4f*>(out + v) = part[u];
        }
      }
      const uint32_t tail = count & ~3u;
      if (lane < count - tail) out[tail + lane] = stage[tail + lane];
    } else {
      for (uint32_t v = lane; v < count; v += 64) out[v] = stage[v];
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the stage may be written again
  };

  // The second block's rows go into LDS before the first block's results leave:
  // the wait for those loads would otherwise also wait for the stores issued
  // in between (loads and stores complete in one order).
  v4f acc0[TS], acc1[TS];
  float extra0 = 0.0f, extra1 = 0.0f;
  placeRows(0);
  multiply(0, acc0, extra0);
  const bool second = rows > 16;
  if (second) placeRows(1);
  storeBlock(0, acc0, extra0);
  if (second) {
    multiply(1, acc1, extra1);
    storeBlock(1, acc1, extra1);
  }
}

uint32_t roundUp4(uint32_t v) { return (v + 3) / 4 * 4; }

// blocks of 16 columns that go through the matrix instruction: one column
// beyond a whole number of blocks is computed on the vector ALUs instead
uint32_t blocksFor(uint32_t n) { return n > 16 && n % 16 == 1 ? n / 16 : (n + 15) / 16; }

// a wave's area: what its loads of A bring (32 rows, rounded up to whole load
// instructions of 64 x 16 bytes), behind that (when a block's rows of C do not
// fit over the block's rows of A) one block of rows of C, and four spare words
// for masked-off stores
uint32_t areaWordsFor(uint32_t n, uint32_t k) {
  const uint32_t groups = (k + 15) / 16;
  return 2 * groups * 256 + (n <= k ? 0 : roundUp4(16 * n)) + 4;
}

template <int TS, int GROUPS, bool TB, bool XCOL>
int launchRows(polar_hip_device* dev, RowsArgs p) {
  p.tileWords = uint32_t(GROUPS) * TS * 256 + (XCOL ? GROUPS * 16 : 0);
  p.areaWords = areaWordsFor(p.N, p.K);
  const uint32_t bytes = (p.tileWords + kWaves * p.areaWords) * sizeof(float);
  auto kernel = rowsKernel<TS, GROUPS, TB, XCOL>;
  // more dynamic LDS than the default limit has to be asked for, once per
  // kernel and device (asking twice is harmless)
  static std::atomic<uint64_t> raised{0};
  const uint64_t bit = 1ull << (dev->ordinal & 63);
  if (bytes > 48 * 1024 && !(raised.load(std::memory_order_acquire) & bit)) {
    POLAR_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, int(kMaxLds)));
    raised.fetch_or(bit, std::memory_order_release);
  }
  const uint32_t groups = (p.M + kGroupRows - 1) / kGroupRows;
  POLAR_HIP_TRY(launchKernelLds(dev, kernel, dim3(groups), dim3(kThreads), bytes, p));
  return POLAR_HIP_OK;
}

template <int TS, int GROUPS>
int launchStored(polar_hip_device* dev, const RowsArgs& p, bool tb) {
  if (p.N == TS * 16 + 1)
    return tb ? launchRows<TS, GROUPS, true, true>(dev, p) : launchRows<TS, GROUPS, false, true>(dev, p);
  return tb ? launchRows<TS, GROUPS, true, false>(dev, p) : launchRows<TS, GROUPS, false, false>(dev, p);
}

// TS x GROUPS 16-byte words of B per lane: at most 32
template <int TS>
int launchGroups(polar_hip_device* dev, const RowsArgs& p, bool tb, uint32_t groups) {
  switch (groups) {
  case 1: return launchStored<TS, 1>(dev, p, tb);
  case 2: return launchStored<TS, 2>(dev, p, tb);
  case 3: return launchStored<TS, 3>(dev, p, tb);
  case 4: return launchStored<TS, 4>(dev, p, tb);
  default: break;
  }
  if constexpr (TS <= 4) {
    switch (groups) {
    case 5: return launchStored<TS, 5>(dev, p, tb);
    case 6: return launchStored<TS, 6>(dev, p, tb);
    case 7: return launchStored<TS, 7>(dev, p, tb);
    default: return launchStored<TS, 8>(dev, p, tb);
    }
  }
  return fail(POLAR_HIP_ERR_INVALID, "rows matmul: no kernel for %d column blocks and %u groups of k", TS, groups);
}

}  // namespace

namespace polar_hip_detail {

bool rowsMatmulApplies(const MatmulCall& c, int computeUnits) {
  if (c.transA || c.K < 4 || c.K > 128 || c.N > 128) return false;
  if (c.M < kGroupRows * uint32_t(computeUnits) * 3 / 4) return false;  // most CUs get a group of waves
  const uint32_t blocks = blocksFor(c.N), groups = (c.K + 15) / 16;
  if (blocks * groups > 32) return false;  // B must fit the registers
  if (blocks > 4 && groups > 4) return false;  // (no kernel is built for those: launchGroups)
  if ((reinterpret_cast<uintptr_t>(c.A) & 15u) != 0) return false;
  const uint32_t words = groups * blocks * 256 + groups * 16 + kWaves * areaWordsFor(c.N, c.K);
  return words * sizeof(float) <= kMaxLds;
}

int launchRowsMatmul(polar_hip_device* dev, const MatmulCall& c) {
  RowsArgs p{};
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
  const uint32_t groups = p.k4 / 16;
  switch (blocksFor(c.N)) {
  case 1: return launchGroups<1>(dev, p, c.transB, groups);
  case 2: return launchGroups<2>(dev, p, c.transB, groups);
  case 3: return launchGroups<3>(dev, p, c.transB, groups);
  case 4: return launchGroups<4>(dev, p, c.transB, groups);
  case 5: return launchGroups<5>(dev, p, c.transB, groups);
  case 6: return launchGroups<6>(dev, p, c.transB, groups);
  case 7: return launchGroups<7>(dev, p, c.transB, groups);
  default: return launchGroups<8>(dev, p, c.transB, groups);
  }
}

}  // namespace polar_hip_detail
