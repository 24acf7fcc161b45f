// fmatmul for a result of at most 16 columns and a moderate number of rows, both
// operands as stored: C[M x N] = A[M x K] B[K x N] with N <= 16, M <= 1024, K a
// multiple of 4 and a small B (the logistic-regression forward product X[256 x 784] W[784 x 10],
// sycl/kernels/MatMul.hpp:33-64).
//
// Such a product is a few MFLOP: what it costs is launches and trips to memory,
// not arithmetic.  The tiled kernel has to cut K into 13-16 parts to occupy the
// chip at all and then needs a second kernel to add them (6.4 + 3.3 us for the
// shape above).  Here one wave computes one row of C in one launch: lane l takes
// the groups of four consecutive k that are congruent to l modulo 64 -- one
// 16-byte load of A and N of B per group (four rows of B, 4 N floats, are
// contiguous and start on 16 bytes) -- with all its loads issued before the
// first multiplication, and the 64 lanes' N partial sums meet in a shuffle
// reduction whose order depends on nothing but the indices.
#include "internal.h"
#include "matmul_epilogue.h"

using namespace polar_hip_detail;

namespace {

typedef float v4f __attribute__((ext_vector_type(4)));

struct SkinnyArgs {
  const float* A;
  const float* B;
  float* C;
  uint32_t M, K;
  int epilogue;
  const float* bias;
  float scaleAcc, scaleBias;
};

// Every wave reads all of B, so the kernel is for a small B and few rows: B up to
// 64 KB and M x B up to 32 MB.  Measured against the tiled plans on a grid of M
// in 16..1024, N in 1..16, K in 64..16384 (stream of calls, settled clock):
// inside these bounds 3.6-5 us against 4.3-8.5 (256 x 10 x 784: 4.3 against 8.4);
// beyond them the tiled kernel's reuse of B wins (1024 x 16 x 4096: 32 us against
// 10, 256 x 16 x 16384: 45 against 10).
constexpr uint32_t kSkinnyMaxRows = 1024;
constexpr uint32_t kSkinnyMaxK = 16384;
constexpr uint32_t kSkinnyMinK = 64;
constexpr uint64_t kSkinnyMaxB = 16384;          // floats of B
constexpr uint64_t kSkinnyMaxWork = 8ull << 20;  // M x floats of B

// U = groups of four k a lane has in flight at a time
template <int N, int U>
__global__ __launch_bounds__(64) void skinnyKernel(SkinnyArgs p) {
  const uint32_t lane = threadIdx.x, m = blockIdx.x;
  const uint32_t quads = p.K / 4;
  const v4f* const a4 = reinterpret_cast<const v4f*>(p.A + size_t(m) * p.K);
  const v4f* const b4 = reinterpret_cast<const v4f*>(p.B);
  float acc[N];
#pragma unroll
  for (int n = 0; n < N; ++n) acc[n] = 0.0f;
  for (uint32_t first = 0; first < quads; first += 64 * U) {
    v4f a[U], b[U][N];
    // all loads of the round first; a group beyond K reads the last one again
    // and multiplies it by zeros
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t q = first + 64 * u + lane, at = q < quads ? q : quads - 1;
      a[u] = a4[at];
#pragma unroll
      for (int i = 0; i < N; ++i) b[u][i] = b4[size_t(at) * N + i];
      if (q >= quads) a[u] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int kk = 0; kk < 4; ++kk)
#pragma unroll
        for (int n = 0; n < N; ++n) {
          // element (kk, n) of the four rows of B: float kk N + n of the 4 N
          const int flat = kk * N + n;
          acc[n] += a[u][kk] * b[u][flat / 4][flat % 4];
        }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1)
#pragma unroll
    for (int n = 0; n < N; ++n) acc[n] += __shfl_down(acc[n], off, 64);
  if (lane == 0) {
#pragma unroll
    for (int n = 0; n < N; ++n) {
      const size_t idx = size_t(m) * N + n;
      p.C[idx] = applyEpilogue(p.epilogue, acc[n], p.bias, p.scaleAcc, p.scaleBias, idx);
    }
  }
}

template <int N>
int launchSkinny(polar_hip_device* dev, const SkinnyArgs& p) {
  constexpr int U = N <= 8 ? 4 : 2;
  POLAR_HIP_TRY(launchKernel(dev, skinnyKernel<N, U>, dim3(p.M), dim3(64), p));
  return POLAR_HIP_OK;
}

}  // namespace

namespace polar_hip_detail {

bool skinnyMatmulApplies(const MatmulCall& c) {
  if (c.transA || c.transB) return false;
  if (c.N > 16 || c.M > kSkinnyMaxRows) return false;
  if (c.K < kSkinnyMinK || c.K > kSkinnyMaxK || c.K % 4 != 0) return false;
  const uint64_t floatsOfB = uint64_t(c.K) * c.N;
  if (floatsOfB > kSkinnyMaxB || c.M * floatsOfB > kSkinnyMaxWork) return false;
  return aligned16(c.A) && aligned16(c.B);
}

int launchSkinnyMatmul(polar_hip_device* dev, const MatmulCall& c) {
  SkinnyArgs p{c.A, c.B, c.C, c.M, c.K, c.epilogue, c.bias, c.scaleAcc, c.scaleBias};
  POLAR_HIP_TRY(hipSetDevice(dev->ordinal));
  switch (c.N) {
  case 1: return launchSkinny<1>(dev, p);
  case 2: return launchSkinny<2>(dev, p);
  case 3: return launchSkinny<3>(dev, p);
  case 4: return launchSkinny<4>(dev, p);
  case 5: return launchSkinny<5>(dev, p);
  case 6: return launchSkinny<6>(dev, p);
  case 7: return launchSkinny<7>(dev, p);
  case 8: return launchSkinny<8>(dev, p);
  case 9: return launchSkinny<9>(dev, p);
  case 10: return launchSkinny<10>(dev, p);
  case 11: return launchSkinny<11>(dev, p);
  case 12: return launchSkinny<12>(dev, p);
  case 13: return launchSkinny<13>(dev, p);
  case 14: return launchSkinny<14>(dev, p);
  case 15: return launchSkinny<15>(dev, p);
  default: return launchSkinny<16>(dev, p);
  }
}

}  // namespace polar_hip_detail
