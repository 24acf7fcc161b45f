// Epilogue of the extended (fused) matmul builtins, shared by every matmul
// kernel of the library so that a fused call and the chain of builtins it
// replaces round identically whichever kernel the shape selects.
#pragma once

#include <cstddef>

namespace polar_hip_detail {

constexpr int kEpiNone = 0;
constexpr int kEpiSigmoid = 1;     // sigmoid(acc)
constexpr int kEpiAddSigmoid = 2;  // sigmoid(scaleAcc*acc + scaleBias*bias)

// The same operations, in the same order, as the separate fadd and fsigmoid
// kernels apply (sycl/kernels/AddNaive.hpp:33-35, Sigmoid.hpp:32-41), so the
// fused result is bit-identical to the chain of builtins it replaces.
__device__ __forceinline__ float applyEpilogue(int epilogue, float acc, const float* bias,
                                               float scaleAcc, float scaleBias, size_t idx) {
  if (epilogue == kEpiNone) return acc;
  float x = acc;
  if (epilogue == kEpiAddSigmoid) x = scaleAcc * acc + scaleBias * bias[idx];
  const float eps = 1e-5f;
  float r = 1.0f / (1.0f + expf(-x));
  if (fabsf(r - 1.0f) < eps) {
    r = 1.0f - eps;
  } else if (fabsf(r) < eps) {
    r = eps;
  }
  return r;
}

// Operands and fused epilogue of one matmul call, as the entry points hand
// them to a kernel family.
struct MatmulCall {
  const float* A;
  const float* B;
  float* C;
  uint32_t M, N, K;
  bool transA, transB;
  int epilogue;
  const float* bias;  // M x N, dense (the framework's fadd does not broadcast)
  float scaleAcc, scaleBias;
};

// matmul_small_k.hip: kernels for a short contraction (K <= 128) with one long
// and one short output dimension.  Returns false if the shape is not theirs.
bool smallKMatmulApplies(const MatmulCall& call);
int launchSmallKMatmul(polar_hip_device* dev, const MatmulCall& call);

// matmul_panel.hip: the same kind of product when the long dimension gives every
// SIMD of the GPU (computeUnits x 4) a panel of 64 rows or columns of its own.
// A subset of what smallKMatmulApplies accepts.
bool panelMatmulApplies(const MatmulCall& call, int computeUnits);
int launchPanelMatmul(polar_hip_device* dev, const MatmulCall& call);

// matmul_rows.hip: the same again for a long M with A stored row by row, whose
// rows are fetched as the contiguous memory they are.  A subset of what
// smallKMatmulApplies accepts (looks at the alignment of call.A).
bool rowsMatmulApplies(const MatmulCall& call, int computeUnits);
int launchRowsMatmul(polar_hip_device* dev, const MatmulCall& call);


// matmul_long_k.hip: a long contraction with a result of at most 33 x 128, both
// operands as stored: one slice of K per CU, partial results added in a second
// kernel.
bool longKMatmulApplies(const MatmulCall& call);
int launchLongKMatmul(polar_hip_device* dev, const MatmulCall& call);

// matmul_skinny.hip: at most 16 columns and 1024 rows of C, both operands as
// stored, K a multiple of 4 and at most 16384: one wave per row of C, one launch.
bool skinnyMatmulApplies(const MatmulCall& call);
int launchSkinnyMatmul(polar_hip_device* dev, const MatmulCall& call);

} // namespace polar_hip_detail
