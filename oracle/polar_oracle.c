/*
 * CPU oracle for the PolarAI/Athena builtin-operation kernels.
 *
 * TEST INFRASTRUCTURE ONLY.  This file restates, in plain C, the arithmetic of
 * the reference's hand-written host-capable kernels so that the HIP kernels can
 * be checked against it.  Nothing on the product path may call it: only the
 * tests, the smoke check and the benchmark's CPU-baseline leg load this
 * library, and only as the checker / the reported baseline.
 *
 * Every function cites the reference source it follows (paths relative to the
 * reference tree).  All tensors are dense, row-major fp32; counts are 64-bit.
 *
 * Arithmetic rules kept from the reference:
 *   - every operation is a single-precision IEEE operation in source order;
 *     the file must be compiled with -ffp-contract=off and without
 *     -ffast-math so that `sa*a + sb*b` is two roundings of the products
 *     followed by one rounding of the sum, as on a generic x86-64 build of the
 *     reference;
 *   - matmul accumulates sequentially over k in an fp32 scalar.
 *
 * Parity status of each function (what pins it, independent of this file):
 *   fadd, fmul, fdivide, fmulconcat  golden vectors from the reference's
 *                                    integration tests; single IEEE ops.
 *   fmatmul f_f, t_f, f_t            five known-answer cases from the
 *                                    reference's tests (small integers, exact).
 *   fmatmul t_t                      no reference test: pinned by
 *                                    (A^T B^T) = (B A)^T, by equality with
 *                                    f_f on explicitly transposed operands and
 *                                    by an fp64 library matmul.
 *   fsigmoid, flogloss               reference vectors (tests disabled
 *                                    upstream) + closed forms + fp64 libm.
 *   fcopy, ffill                     identity / constant.
 *   ftranspose                       PARITY UNPINNED by the reference (it has no
 *                                    implementation and no test there); pinned
 *                                    only by the textbook definition, the
 *                                    involution T(T(x)) = x and the identity
 *                                    matmul_t_f(A,B) == matmul_f_f(T(A),B).
 *
 *   frelu, fsoftmax, fconv2d, fpool  one golden vector each from the reference's
 *                                    integration tests, plus independent library
 *                                    routines (numpy maximum, scipy softmax in
 *                                    fp64, scipy correlate2d, reshape-max) on
 *                                    random data.  fsoftmax at sizes where the
 *                                    reference's sequential fp32 sum has lost
 *                                    precision is checked against the fp64-
 *                                    accumulated variant instead (see there).
 *
 * Threads: polar_oracle_set_threads(n) selects how many host threads the
 * loops are split over (outermost index, static schedule).  n = 1 is the
 * faithful serial host-device loop; results do not depend on n.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

static int g_threads = 1;

void polar_oracle_set_threads(int n) { g_threads = n < 1 ? 1 : n; }
int polar_oracle_get_threads(void) { return g_threads; }

int polar_oracle_hw_threads(void) {
#ifdef _OPENMP
  return omp_get_num_procs();
#else
  return 1;
#endif
}

/* c[i] = scaleA*a[i] + scaleB*b[i]
 * src/backend/generic/runtime/sycl/kernels/AddNaive.hpp:33-35
 * (same formula, operands commuted: src/backend/generic/runtime/opencl/kernels.h:37) */
void polar_oracle_fadd(const float* a, float scaleA, const float* b,
                       float scaleB, float* c, uint64_t n) {
#pragma omp parallel for num_threads(g_threads) schedule(static)
  for (int64_t i = 0; i < (int64_t)n; ++i) {
    float pa = scaleA * a[i];
    float pb = scaleB * b[i];
    c[i] = pa + pb;
  }
}

/* c[i] = a[i]*b[i]
 * src/backend/generic/runtime/sycl/kernels/Mul.hpp:32 */
void polar_oracle_fmul(const float* a, const float* b, float* c, uint64_t n) {
#pragma omp parallel for num_threads(g_threads) schedule(static)
  for (int64_t i = 0; i < (int64_t)n; ++i) c[i] = a[i] * b[i];
}

/* out[i] = numerator[i]/denominator[i]  (IEEE correctly rounded)
 * src/backend/generic/runtime/sycl/kernels/Divide.hpp:33-35 */
void polar_oracle_fdivide(const float* num, const float* den, float* out,
                          uint64_t n) {
#pragma omp parallel for num_threads(g_threads) schedule(static)
  for (int64_t i = 0; i < (int64_t)n; ++i) out[i] = num[i] / den[i];
}

/* r = 1/(1+exp(-x)); |r-1|<eps -> 1-eps; else |r|<eps -> eps; eps = 1e-5f
 * src/backend/generic/runtime/sycl/kernels/Sigmoid.hpp:32-41
 * (agrees with src/backend/generic/runtime/opencl/kernels.h:143-151 and the
 *  test's own loop tests/integration/operations/SigmoidOperation.cpp:19-32) */
void polar_oracle_fsigmoid(const float* in, float* out, uint64_t n) {
  const float eps = 1e-5f;
#pragma omp parallel for num_threads(g_threads) schedule(static)
  for (int64_t i = 0; i < (int64_t)n; ++i) {
    float e = expf(-in[i]);
    float d = 1.0f + e;
    float r = 1.0f / d;
    if (fabsf(r - 1.0f) < eps) {
      r = 1.0f - eps;
    } else if (fabsf(r) < eps) {
      r = eps;
    }
    out[i] = r;
  }
}

/* out = -g*log(p+eps) - (1-g)*log(1-p+eps), eps = 1e-5f, elementwise, no reduce
 * src/backend/generic/runtime/sycl/kernels/LogLoss.hpp:33-37
 * (agrees with src/backend/generic/runtime/opencl/kernels.h:69-72 and
 *  tests/integration/operations/LogLossOperation.cpp:19-30) */
void polar_oracle_flogloss(const float* predicted, const float* groundTruth,
                           float* out, uint64_t n) {
  const float eps = 1e-5f;
#pragma omp parallel for num_threads(g_threads) schedule(static)
  for (int64_t i = 0; i < (int64_t)n; ++i) {
    float p = predicted[i];
    float g = groundTruth[i];
    float l1 = logf(p + eps);
    float om = 1.0f - p;
    float l2 = logf(om + eps);
    float t1 = (-g) * l1;
    float t2 = (1.0f - g) * l2;
    out[i] = t1 - t2;
  }
}

/* out[i] = gradient[0]*localDerivative[i]  (scalar broadcast of element 0)
 * src/backend/generic/runtime/sycl/kernels/MulConcat.hpp:33-35 */
void polar_oracle_fmulconcat(const float* gradient,
                             const float* localDerivative, float* out,
                             uint64_t n) {
  const float g0 = gradient[0];
#pragma omp parallel for num_threads(g_threads) schedule(static)
  for (int64_t i = 0; i < (int64_t)n; ++i) out[i] = g0 * localDerivative[i];
}

/* dst = src, n elements.
 * src/backend/generic/runtime/sycl/kernels/Copy.hpp:49-53 (whole-buffer copy).
 * The USM variant at Copy.hpp:77 passes an element count where a byte count is
 * expected and so copies a quarter of the tensor; that defect is not restated. */
void polar_oracle_fcopy(const float* src, float* dst, uint64_t n) {
#pragma omp parallel for num_threads(g_threads) schedule(static)
  for (int64_t i = 0; i < (int64_t)n; ++i) dst[i] = src[i];
}

/* out[i] = pattern
 * src/backend/generic/runtime/sycl/kernels/Fill.hpp:69-74 */
void polar_oracle_ffill(float pattern, float* out, uint64_t n) {
#pragma omp parallel for num_threads(g_threads) schedule(static)
  for (int64_t i = 0; i < (int64_t)n; ++i) out[i] = pattern;
}

/* out[j*rows + i] = in[i*cols + j], in is rows x cols, out is cols x rows.
 * The reference only specifies this builtin ("Transpose 2D tensor (matrix)",
 * include/polarai/core/internal/GenBuiltins.hpp:50; operands (a, out),
 * utils/dialects/include/PolarGraph/PolarGraphOps.td:507-527); no runtime
 * implements it.  PARITY UNPINNED by the reference. */
void polar_oracle_ftranspose(const float* in, float* out, uint64_t rows,
                             uint64_t cols) {
  /* blocked so the CPU baseline is not a pure cache-miss measurement */
  const int64_t B = 32;
  const int64_t R = (int64_t)rows, C = (int64_t)cols;
#pragma omp parallel for num_threads(g_threads) schedule(static)
  for (int64_t i0 = 0; i0 < R; i0 += B) {
    int64_t i1 = i0 + B < R ? i0 + B : R;
    for (int64_t j0 = 0; j0 < C; j0 += B) {
      int64_t j1 = j0 + B < C ? j0 + B : C;
      for (int64_t j = j0; j < j1; ++j)
        for (int64_t i = i0; i < i1; ++i) out[j * R + i] = in[i * C + j];
    }
  }
}

/* C[i,j] = sum_k opA(A)[i,k] * opB(B)[k,j], fp32 accumulator, k ascending.
 * src/backend/generic/runtime/sycl/kernels/MatMul.hpp:33-64, with the 2-D
 * row-major indexing of src/backend/generic/runtime/sycl/kernels/common.hpp:35-38.
 *
 * A is stored [a0 x a1], B is stored [b0 x b1] (the TensorInfo shapes), C is
 * [M x N].  K = transA ? a0 : a1 (MatMul.hpp:34-39).  As in the reference, the
 * launch range is C's shape and nothing checks that the operand shapes agree;
 * callers pass consistent shapes.  The same loop appears, with explicit
 * increments, in tests/integration/operations/MatMulOperation.cpp:17-51 and
 * src/backend/generic/runtime/opencl/kernels.h:80-117.
 * Only output rows [rowBegin, rowEnd) are computed (written at their normal
 * place in C), so that full-size parity checks can sample rows. */
void polar_oracle_fmatmul_rows(int transA, int transB, const float* A,
                               uint64_t a0, uint64_t a1, const float* B,
                               uint64_t b0, uint64_t b1, float* C, uint64_t M,
                               uint64_t N, uint64_t rowBegin, uint64_t rowEnd) {
  const int64_t K = (int64_t)(transA ? a0 : a1);
  (void)b0;
  if (rowEnd > M) rowEnd = M;
#pragma omp parallel for num_threads(g_threads) schedule(static)
  for (int64_t i = (int64_t)rowBegin; i < (int64_t)rowEnd; ++i) {
    for (int64_t j = 0; j < (int64_t)N; ++j) {
      float acc = 0.0f;
      for (int64_t k = 0; k < K; ++k) {
        int64_t lrow = transA ? k : i;
        int64_t lcol = transA ? i : k;
        int64_t rrow = transB ? j : k;
        int64_t rcol = transB ? k : j;
        float l = A[lrow * (int64_t)a1 + lcol];
        float r = B[rrow * (int64_t)b1 + rcol];
        float p = l * r;
        acc = acc + p;
      }
      C[i * (int64_t)N + j] = acc;
    }
  }
}

/* Whole output: rows [0, M). */
void polar_oracle_fmatmul(int transA, int transB, const float* A,
                          uint64_t a0, uint64_t a1, const float* B,
                          uint64_t b0, uint64_t b1, float* C, uint64_t M,
                          uint64_t N) {
  polar_oracle_fmatmul_rows(transA, transB, A, a0, a1, B, b0, b1, C, M, N, 0,
                            M);
}

/* Same contraction with an fp64 accumulator: used by the tests to bound the
 * rounding drift of the fp32 sequential-k loop, never as the expected value. */
void polar_oracle_fmatmul_f64acc(int transA, int transB, const float* A,
                                 uint64_t a0, uint64_t a1, const float* B,
                                 uint64_t b0, uint64_t b1, double* C,
                                 uint64_t M, uint64_t N) {
  const int64_t K = (int64_t)(transA ? a0 : a1);
  (void)b0;
#pragma omp parallel for num_threads(g_threads) schedule(static)
  for (int64_t i = 0; i < (int64_t)M; ++i) {
    for (int64_t j = 0; j < (int64_t)N; ++j) {
      double acc = 0.0;
      for (int64_t k = 0; k < K; ++k) {
        double l = transA ? A[k * (int64_t)a1 + i] : A[i * (int64_t)a1 + k];
        double r = transB ? B[j * (int64_t)b1 + k] : B[k * (int64_t)b1 + j];
        acc += l * r;
      }
      C[i * (int64_t)N + j] = acc;
    }
  }
}

/* out[i] = in[i] > 0 ? in[i] : 0  (ordered compare: NaN gives 0)
 * utils/dialects/lib/PolarGraph/kernels/ReLUOp.cpp:35-44 */
void polar_oracle_frelu(const float* in, float* out, uint64_t n) {
#pragma omp parallel for num_threads(g_threads) schedule(static)
  for (int64_t i = 0; i < (int64_t)n; ++i) out[i] = in[i] > 0.0f ? in[i] : 0.0f;
}

/* out[i] = exp(in[i]) / sum_j exp(in[j]) over the WHOLE tensor (any rank, no
 * max subtraction); the sum is an fp32 scalar accumulated in index order.
 * utils/dialects/lib/PolarGraph/kernels/SoftmaxOp.cpp:38-65 (the reference
 * recomputes the sum for every output element; the value is the same).
 * Serial on purpose: the accumulation order is part of the definition. */
void polar_oracle_fsoftmax(const float* in, float* out, uint64_t n) {
  float total = 0.0f;
  for (uint64_t j = 0; j < n; ++j) total = expf(in[j]) + total;
#pragma omp parallel for num_threads(g_threads) schedule(static)
  for (int64_t i = 0; i < (int64_t)n; ++i) out[i] = expf(in[i]) / total;
}

/* Same definition with the sum accumulated in fp64 (then rounded to fp32
 * once): what the reference's loop computes when no precision is lost, used
 * for sizes where the sequential fp32 sum has drifted. */
void polar_oracle_fsoftmax_f64sum(const float* in, float* out, uint64_t n) {
  double total = 0.0;
  for (uint64_t j = 0; j < n; ++j) total += (double)expf(in[j]);
  const float t = (float)total;
#pragma omp parallel for num_threads(g_threads) schedule(static)
  for (int64_t i = 0; i < (int64_t)n; ++i) out[i] = expf(in[i]) / t;
}

/* Single-channel "valid" 2-D correlation: in is H x W, kernel KH x KW, out is
 * (H-KH+1) x (W-KW+1); out[y,x] = sum_a sum_b in[y+a, x+b] * kernel[a,b],
 * fp32 accumulator starting at 0, a outer / b inner, product rounded before
 * the add.
 * utils/dialects/lib/PolarGraph/kernels/Conv2DOp.cpp:35-84 (loops run over
 * [-K/2, K/2], i.e. 2*(K/2)+1 taps: only odd kernel sizes index inside the
 * kernel tensor); output shape src/operation/internal/Conv2DOperationInternal.cpp:35-39. */
void polar_oracle_fconv2d(const float* in, const float* kernel, float* out,
                          uint64_t H, uint64_t W, uint64_t KH, uint64_t KW) {
  const int64_t OH = (int64_t)H - (int64_t)KH + 1, OW = (int64_t)W - (int64_t)KW + 1;
#pragma omp parallel for num_threads(g_threads) schedule(static)
  for (int64_t y = 0; y < OH; ++y) {
    for (int64_t x = 0; x < OW; ++x) {
      float acc = 0.0f;
      for (int64_t a = 0; a < (int64_t)KH; ++a)
        for (int64_t b = 0; b < (int64_t)KW; ++b) {
          float prod = in[(y + a) * (int64_t)W + x + b] * kernel[a * (int64_t)KW + b];
          acc = prod + acc;
        }
      out[y * OW + x] = acc;
    }
  }
}

/* Max pooling: out[y,x] = max(-10e5f, max_{a<win0, b<win1} in[y*s0+a, x*s1+b])
 * (strict ordered greater-than, so NaN inputs are skipped), out is
 * ((H-win0)/s0+1) x ((W-win1)/s1+1).
 * utils/dialects/lib/PolarGraph/kernels/Pool2DOp.cpp:45-82; output shape
 * src/operation/internal/Pool2DOperationInternal.cpp:37-41. */
void polar_oracle_fpool(const float* in, float* out, uint64_t H, uint64_t W,
                        uint64_t win0, uint64_t win1, uint64_t s0, uint64_t s1) {
  const int64_t OH = ((int64_t)H - (int64_t)win0) / (int64_t)s0 + 1;
  const int64_t OW = ((int64_t)W - (int64_t)win1) / (int64_t)s1 + 1;
#pragma omp parallel for num_threads(g_threads) schedule(static)
  for (int64_t y = 0; y < OH; ++y) {
    for (int64_t x = 0; x < OW; ++x) {
      float best = -10e5f;
      for (int64_t a = 0; a < (int64_t)win0; ++a)
        for (int64_t b = 0; b < (int64_t)win1; ++b) {
          float v = in[(y * (int64_t)s0 + a) * (int64_t)W + x * (int64_t)s1 + b];
          best = v > best ? v : best;
        }
      out[y * OW + x] = best;
    }
  }
}

/* Byte size of a tensor record: sizeof(dtype) * prod(shape), dtype codes
 * 1 = f64, 2 = f32, 3 = f16 (include/polarai/core/tensor/DataType.hpp:20-34;
 * src/backend/generic/runtime/utils/utils.hpp:7-17).  Returns 0 for an
 * undefined dtype (the reference aborts there). */
uint64_t polar_oracle_record_bytes(int dataType, uint64_t dims,
                                   const uint64_t* shape) {
  uint64_t sz;
  switch (dataType) {
  case 1: sz = 8; break;
  case 2: sz = 4; break;
  case 3: sz = 2; break;
  default: return 0;
  }
  for (uint64_t i = 0; i < dims; ++i) sz *= shape[i];
  return sz;
}
