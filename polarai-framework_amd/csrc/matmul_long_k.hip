// fmatmul for a long contraction and a small result: C[33 x 127] =
// A[33 x 65536] * B[65536 x 127], both operands as stored (A [M x K], B [K x N]).
//
// The result is a few kilobytes and the operands are streamed once, so the
// product is cut along K, one slice per work-group (as many groups as CUs), and
// a second kernel adds the groups' partial results in group order: nothing
// depends on scheduling.  Inside a group every wave takes a quarter of the
// slice with the WHOLE of C in its accumulators and reads its operands straight
// into the matrix instruction's layout, no LDS and no barrier on the way:
//   * B's rows are contiguous along n.  A lane loads 16 bytes of row k: the
//     values n = 64 jj + 4 fx + t, t = 0..3 (fx = lane % 16), which belong to four
//     DIFFERENT blocks of 16 columns -- block 4 jj + t is the columns
//     64 jj + 4 fx + t.  One instruction fetches 256 contiguous bytes of each of
//     four rows of B.
//   * A's rows are contiguous along k.  A lane loads 16 bytes of row 16 i + fx:
//     k = 16 g + 4 fk + c, c = 0..3 (fk = lane / 16), the lane's k in the four
//     steps of group g; B's rows are picked in the same order of k.
//   * A 33rd row of A would make a third block of 16 rows out of one row: it
//     is a dot product on the vector ALUs instead.
// The loads of a group of 16 values of k are issued two groups ahead of the
// matrix instructions that use them.  At the end the four waves' accumulators meet in
// LDS (added in wave order) and leave as 16-byte stores into a partial result
// whose rows are padded to a multiple of 64 floats.
#include "internal.h"
#include "matmul_epilogue.h"

using namespace polar_hip_detail;

namespace {

typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kWaves = 4;
constexpr int kThreads = kWaves * 64;
constexpr uint32_t kChunk = 64;  // values of k a wave takes at a time: four groups of 16

struct LongKArgs {
  const float* A;
  const float* B;
  float* partial;      // [groups][rowsPadded][colsPadded]
  uint32_t M, N, K;
  uint32_t kPerGroup;  // multiple of kWaves * kChunk
  uint32_t colsPadded; // 64 * TJ
  uint32_t rowsPadded; // 16 * TM (+ 1 with XROW)
};

__device__ __forceinline__ v4f loadUnaligned(const float* p) {
  return *reinterpret_cast<const v4f __attribute__((aligned(4)))*>(p);
}

// TM blocks of 16 rows and TJ x 4 blocks of 16 columns go through the matrix
// instruction.  XROW: M = 16 TM + 1, the last row on the vector ALUs.
template <int TM, int TJ, bool XROW>
__global__ __launch_bounds__(kThreads) void longKKernel(LongKArgs p) {
  extern __shared__ __attribute__((aligned(16))) float meet[];
  const int t = threadIdx.x, lane = t % 64;
  const int wave = __builtin_amdgcn_readfirstlane(t / 64);
  const uint32_t fx = lane % 16, fk = lane / 16;

  const uint32_t kBegin = blockIdx.x * p.kPerGroup + wave * (p.kPerGroup / kWaves);
  const uint32_t kEnd = kBegin + p.kPerGroup / kWaves < p.K ? kBegin + p.kPerGroup / kWaves : p.K;

  v4f acc[TM][TJ][4];  // [i][jj][t]: rows 16 i + .., columns 64 jj + 4 fx + t
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int jj = 0; jj < TJ; ++jj)
#pragma unroll
      for (int u = 0; u < 4; ++u) acc[i][jj][u] = v4f{0.f, 0.f, 0.f, 0.f};
  v4f part[TJ];  // XROW: the lane's share of the last row, columns 64 jj + 4 fx + t
#pragma unroll
  for (int jj = 0; jj < TJ; ++jj) part[jj] = v4f{0.f, 0.f, 0.f, 0.f};

  // Byte offsets (operands smaller than 4 GiB).  Rows of A beyond M repeat row
  // M - 1 (their results are not stored); columns of B beyond N read on into
  // the next row, or, in the last row, are taken from 16 bytes earlier (their
  // results are not stored either).  k beyond the slice is clamped here and
  // zeroed when used.
  uint32_t rowA[TM + (XROW ? 1 : 0)];
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const uint32_t r = 16 * i + fx;
    rowA[i] = (r < p.M ? r : p.M - 1) * p.K;
  }
  if constexpr (XROW) rowA[TM] = (p.M - 1) * p.K;
  uint32_t colB[TJ];
#pragma unroll
  for (int jj = 0; jj < TJ; ++jj) colB[jj] = 64 * jj + 4 * fx;
  const uint32_t lastB = p.K * p.N - 4;

  for (uint32_t k0 = kBegin; k0 < kEnd; k0 += kChunk) {
    v4f a[4][TM + (XROW ? 1 : 0)], b[4][4][TJ];
    auto fetch = [&](int g) {
      const uint32_t kA = k0 + 16 * g + 4 * fk;
      const uint32_t fromA = kA + 4 <= p.K ? kA : p.K - 4;  // K >= 4
#pragma unroll
      for (int i = 0; i < TM + (XROW ? 1 : 0); ++i) a[g][i] = loadUnaligned(p.A + rowA[i] + fromA);
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const uint32_t k = k0 + 16 * g + 4 * fk + c;
        const uint32_t rowB = (k < p.K ? k : p.K - 1) * p.N;
#pragma unroll
        for (int jj = 0; jj < TJ; ++jj) {
          const uint32_t at = rowB + colB[jj];
          b[g][c][jj] = loadUnaligned(p.B + (at <= lastB ? at : lastB));
        }
      }
    };
    // what was clamped is put right: k at or beyond the end of the slice becomes
    // zeros, and 16 bytes that would have run past the end of an operand were
    // taken from a few floats earlier (the last chunk of the last wave of the
    // last group only)
    auto settle = [&](int g) {
      if (k0 + 16 * (g + 1) >= kEnd) {
        const uint32_t kA = k0 + 16 * g + 4 * fk;
        const uint32_t fromA = kA + 4 <= p.K ? kA : p.K - 4;
        const uint32_t shift = kA - fromA;  // the 16 bytes of A were taken from this many floats earlier
#pragma unroll
        for (int i = 0; i < TM + (XROW ? 1 : 0); ++i) {
          const v4f w = a[g][i];
          v4f s;
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            const uint32_t at = shift + c;
            const float picked = at == 0 ? w[0] : at == 1 ? w[1] : at == 2 ? w[2] : w[3];
            s[c] = (kA + c < kEnd && at < 4) ? picked : 0.0f;
          }
          a[g][i] = s;
        }
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          const bool beyond = kA + c >= kEnd;
          const uint32_t k = kA + c;
          const uint32_t rowB = (k < p.K ? k : p.K - 1) * p.N;
#pragma unroll
          for (int jj = 0; jj < TJ; ++jj) {
            const uint32_t at = rowB + colB[jj];
            const uint32_t d = at > lastB ? at - lastB : 0;  // taken from d floats earlier
            v4f v = b[g][c][jj];
            if (d != 0)
              v = v4f{d == 1 ? v[1] : d == 2 ? v[2] : d == 3 ? v[3] : 0.0f, d == 1 ? v[2] : d == 2 ? v[3] : 0.0f,
                      d == 1 ? v[3] : 0.0f, 0.0f};
            b[g][c][jj] = beyond ? v4f{0.f, 0.f, 0.f, 0.f} : v;
          }
        }
      }
    };
    // two groups ahead: a group's matrix instructions take about a microsecond,
    // a load two to three
    fetch(0);
    fetch(1);
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      if (g + 2 < 4) fetch(g + 2);
      __builtin_amdgcn_sched_barrier(0);
      settle(g);
#pragma unroll
      for (int c = 0; c < 4; ++c) {
#pragma unroll
        for (int jj = 0; jj < TJ; ++jj) {
#pragma unroll
          for (int u = 0; u < 4; ++u) {
#pragma unroll
            for (int i = 0; i < TM; ++i)
              acc[i][jj][u] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[g][i][c], b[g][c][jj][u], acc[i][jj][u], 0, 0, 0);
            if constexpr (XROW) part[jj][u] = __builtin_fmaf(a[g][TM][c], b[g][c][jj][u], part[jj][u]);
          }
        }
      }
    }
  }

  // The four waves' results meet in LDS, one 16-byte word per lane and slot;
  // slot (i, jj, r) is rows 16 i + 4 (lane / 16) + r, columns 64 jj + 4 fx + t of
  // all four blocks (accumulator layout: register r of lane l is row
  // 4 (l / 16) + r, column l % 16 of its block), and TJ more slots hold the
  // extra row.  Wave w then adds the slots s = w, w + 4, ... in wave order and
  // stores them.
  constexpr int kSlots = TM * TJ * 4 + (XROW ? TJ : 0);
  v4f* const mine = reinterpret_cast<v4f*>(meet) + (wave * kSlots) * 64 + lane;
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int jj = 0; jj < TJ; ++jj)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        mine[((i * TJ + jj) * 4 + r) * 64] = v4f{acc[i][jj][0][r], acc[i][jj][1][r], acc[i][jj][2][r], acc[i][jj][3][r]};
  if constexpr (XROW) {
#pragma unroll
    for (int jj = 0; jj < TJ; ++jj) {
      // the four lanes that hold the same columns (one per fk) add their shares
      v4f total;
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const float p0 = __shfl(part[jj][u], fx), p1 = __shfl(part[jj][u], fx + 16), p2 = __shfl(part[jj][u], fx + 32),
                    p3 = __shfl(part[jj][u], fx + 48);
        total[u] = ((p0 + p1) + p2) + p3;
      }
      mine[(TM * TJ * 4 + jj) * 64] = total;  // the same in all four lane groups
    }
  }
  __syncthreads();
  float* const out = p.partial + size_t(blockIdx.x) * p.rowsPadded * p.colsPadded;
  const uint32_t q = lane / 16;
  for (int s = wave; s < kSlots; s += kWaves) {
    const v4f* const from = reinterpret_cast<const v4f*>(meet) + s * 64 + lane;
    v4f sum = from[0];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) {
      const v4f v = from[w * kSlots * 64];
      sum = v4f{sum[0] + v[0], sum[1] + v[1], sum[2] + v[2], sum[3] + v[3]};
    }
    uint32_t row, jj;
    if (s < TM * TJ * 4) {
      const int i = s / (TJ * 4), r = s % 4;
      jj = s / 4 % TJ;
      row = 16 * i + 4 * q + r;
    } else {
      jj = s - TM * TJ * 4;
      row = 16 * TM;
      if (q != 0) continue;  // one lane group stores the extra row
    }
    *reinterpret_cast<v4f*>(out + size_t(row) * p.colsPadded + 64 * jj + 4 * fx) = sum;
  }
}

// C[row][col] = sum over the groups of partial[g][row][col], in a fixed order:
// a work-group owns 64 consecutive elements of C (one per lane); wave w adds
// the groups g = w, w + 16, ... one after the other and the 16 wave sums are
// then added in wave order.
__global__ __launch_bounds__(1024) void longKReduceKernel(const float* __restrict__ partial, float* __restrict__ c,
                                                          uint32_t M, uint32_t N, uint32_t groups,
                                                          uint32_t rowsPadded, uint32_t colsPadded, int epilogue,
                                                          const float* bias, float scaleAcc, float scaleBias) {
  __shared__ float sums[16][64];
  const uint32_t wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const uint32_t e = blockIdx.x * 64 + lane, count = M * N;
  float acc = 0.0f;
  if (e < count) {
    const uint32_t at = e / N * colsPadded + e % N;
    const size_t pitch = size_t(rowsPadded) * colsPadded;
    uint32_t g = wave;
    for (; g + 48 < groups; g += 64) {
      const float v0 = partial[g * pitch + at], v1 = partial[(g + 16) * pitch + at];
      const float v2 = partial[(g + 32) * pitch + at], v3 = partial[(g + 48) * pitch + at];
      acc = (((acc + v0) + v1) + v2) + v3;
    }
    for (; g < groups; g += 16) acc += partial[g * pitch + at];
  }
  sums[wave][lane] = acc;
  __syncthreads();
  if (wave == 0 && e < count) {
    float total = sums[0][lane];
#pragma unroll
    for (int w = 1; w < 16; ++w) total += sums[w][lane];
    c[e] = applyEpilogue(epilogue, total, bias, scaleAcc, scaleBias, e);
  }
}

template <int TM, int TJ, bool XROW>
int launchLongK(polar_hip_device* dev, const MatmulCall& c, LongKArgs p, uint32_t groups) {
  constexpr int kSlots = TM * TJ * 4 + (XROW ? TJ : 0);
  const uint32_t ldsBytes = kWaves * kSlots * 64 * sizeof(v4f);
  auto kernel = longKKernel<TM, TJ, XROW>;
  static std::atomic<uint64_t> raised{0};
  const uint64_t bit = 1ull << (dev->ordinal & 63);
  if (ldsBytes > 48 * 1024 && !(raised.load(std::memory_order_acquire) & bit)) {
    POLAR_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
    raised.fetch_or(bit, std::memory_order_release);
  }
  p.colsPadded = 64 * TJ;
  p.rowsPadded = 16 * TM + (XROW ? 1 : 0);
  // the partial results go to the device's workspace; the lock keeps another
  // thread's call from enqueuing its own user of the workspace between this
  // call's two kernels
  std::lock_guard<std::mutex> workspaceLock(dev->workspaceMu);
  void* workspace = nullptr;
  const int st = workspaceFor(dev, uint64_t(groups) * p.rowsPadded * p.colsPadded * sizeof(float), &workspace);
  if (st != POLAR_HIP_OK) return st;
  p.partial = static_cast<float*>(workspace);
  POLAR_HIP_TRY(launchKernelLds(dev, kernel, dim3(groups), dim3(kThreads), ldsBytes, p));
  POLAR_HIP_TRY(launchKernel(dev, longKReduceKernel, dim3((c.M * c.N + 63) / 64), dim3(1024), p.partial, c.C, c.M, c.N,
                             groups, p.rowsPadded, p.colsPadded, c.epilogue, c.bias, c.scaleAcc, c.scaleBias));
  return POLAR_HIP_OK;
}

template <int TM, bool XROW>
int launchColumns(polar_hip_device* dev, const MatmulCall& c, const LongKArgs& p, uint32_t groups) {
  return c.N <= 64 ? launchLongK<TM, 1, XROW>(dev, c, p, groups) : launchLongK<TM, 2, XROW>(dev, c, p, groups);
}

constexpr uint32_t kLongKMin = 16384;

}  // namespace

namespace polar_hip_detail {

bool longKMatmulApplies(const MatmulCall& c) {
  if (c.transA || c.transB) return false;
  if (c.M > 33 || c.N > 128 || c.N < 4 || c.K < kLongKMin) return false;
  if (c.M > 32 && c.M != 33) return false;
  // 32-bit element offsets into both operands
  return uint64_t(c.M) * c.K < (1ull << 30) && uint64_t(c.K) * c.N < (1ull << 30);
}

int launchLongKMatmul(polar_hip_device* dev, const MatmulCall& c) {
  LongKArgs p{};
  p.A = c.A;
  p.B = c.B;
  p.M = c.M;
  p.N = c.N;
  p.K = c.K;
  POLAR_HIP_TRY(hipSetDevice(dev->ordinal));
  // one slice per CU, a whole number of chunks for each of its four waves
  const uint32_t cus = static_cast<uint32_t>(dev->info.compute_units);
  const uint32_t unit = kWaves * kChunk;
  p.kPerGroup = ((c.K + cus - 1) / cus + unit - 1) / unit * unit;
  const uint32_t groups = (c.K + p.kPerGroup - 1) / p.kPerGroup;
  if (c.M == 33) return launchColumns<2, true>(dev, c, p, groups);
  if (c.M > 16) return launchColumns<2, false>(dev, c, p, groups);
  return launchColumns<1, false>(dev, c, p, groups);
}

}  // namespace polar_hip_detail
