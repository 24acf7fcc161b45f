// The short operand of a short-contraction matmul, kept whole in LDS; shared by
// the kernels of matmul_small_k.hip and matmul_panel.hip.
#pragma once

#include <cstdint>

namespace polar_hip_detail {

// The short operand X (xdim values of x, a row of C for A and a column of C for
// B) in LDS:
//   KCONTIG:  element (x, k) is X[x*K + k]     -> S[x*pitch + k]   "k-minor"
//   !KCONTIG: element (x, k) is X[k*xdim + x]  -> S[k*pitch + x]   "x-minor"
// Either way it is one contiguous run of HBM made of rows, copied row by row
// into rows of `pitch` words.  A fragment read has 16 lanes on consecutive x and
// 4 groups of lanes on consecutive k: a k-minor pitch with pitch/4 odd, or an
// x-minor pitch of 16 mod 32, spreads them over all banks (two lanes per bank,
// the minimum for 64 lanes) for the plain order of k; in the permuted order (see
// the kernel) the four groups are four rows or words apart instead.  Slots with
// k in [K, k4) are zeroed: the matrix
// instruction multiplies them.
template <bool KCONTIG>
struct ShortTile {
  static uint32_t pitchFor(uint32_t xPadded, uint32_t k4) {
    if (KCONTIG) return (k4 / 4) % 2 == 1 ? k4 : k4 + 4;
    return xPadded % 32 == 16 ? xPadded : xPadded + 16;
  }
  static uint32_t words(uint32_t xPadded, uint32_t k4) {
    return (KCONTIG ? xPadded : k4) * pitchFor(xPadded, k4);
  }

  template <int kThreads>
  static __device__ __forceinline__ void load(float* S, const float* X, uint32_t xdim,
                                              uint32_t xPadded, uint32_t K, uint32_t k4,
                                              uint32_t pitch, int t) {
    const uint32_t rowLen = KCONTIG ? K : xdim, total = xdim * K;
    uint32_t row = uint32_t(t) / rowLen, col = uint32_t(t) % rowLen;
    const uint32_t stepRow = uint32_t(kThreads) / rowLen, stepCol = uint32_t(kThreads) % rowLen;
    constexpr int U = 8; // loads in flight per lane
    for (uint32_t base = t; base < total; base += kThreads * U) {
      float v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint32_t e = base + u * kThreads;
        v[u] = e < total ? X[e] : 0.0f;
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (base + u * kThreads < total) S[row * pitch + col] = v[u];
        col += stepCol;
        row += stepRow;
        if (col >= rowLen) {
          col -= rowLen;
          ++row;
        }
      }
    }
    const uint32_t padK = k4 - K; // 0..15
    if (KCONTIG) {
      for (uint32_t e = t; e < xPadded * padK; e += kThreads) S[(e / padK) * pitch + K + e % padK] = 0.0f;
    } else {
      for (uint32_t e = t; e < padK * xPadded; e += kThreads) S[(K + e / xPadded) * pitch + e % xPadded] = 0.0f;
    }
  }

  static __device__ __forceinline__ float fragment(const float* S, uint32_t pitch, uint32_t x, uint32_t k) {
    return KCONTIG ? S[x * pitch + k] : S[k * pitch + x];
  }
};

} // namespace polar_hip_detail
