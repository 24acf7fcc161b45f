// Stand-ins for kernels the framework's code generator would emit for ops that
// have no hand-written builtin: plain gfx950 kernels whose tensor parameters
// are expanded memref descriptors (allocated pointer, aligned pointer, offset,
// sizes, strides), the convention of the reference's CUDA runtime
// (src/backend/generic/runtime/cuda/CudaDevice.cpp:75-94).  Compiled to a code
// object (tests/native/build/generated_kernels.hsaco) that the plugin loads
// through Device::selectBinary.  TEST INFRASTRUCTURE ONLY.
#include <hip/hip_runtime.h>
#include <stdint.h>

// out[i] = alpha * x[i] + y[i], rank 1
extern "C" __global__ void gen_axpy_1d(const float* xAlloc, const float* x, int64_t xOff,
                                       int64_t xSize, int64_t xStride, float alpha,
                                       const float* yAlloc, const float* y, int64_t yOff,
                                       int64_t ySize, int64_t yStride, float* oAlloc, float* o,
                                       int64_t oOff, int64_t oSize, int64_t oStride) {
  (void)xAlloc; (void)yAlloc; (void)oAlloc; (void)xSize; (void)ySize;
  const int64_t step = int64_t(gridDim.x) * blockDim.x;
  for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < oSize; i += step)
    o[oOff + i * oStride] = alpha * x[xOff + i * xStride] + y[yOff + i * yStride];
}

// out[r, c] = in[r, c] * rowScale[r], rank 2 x rank 1 -> rank 2 (uses sizes and both strides)
extern "C" __global__ void gen_row_scale_2d(const float* inAlloc, const float* in, int64_t inOff,
                                            int64_t inRows, int64_t inCols, int64_t inStride0,
                                            int64_t inStride1, const float* sAlloc, const float* s,
                                            int64_t sOff, int64_t sSize, int64_t sStride,
                                            float* oAlloc, float* o, int64_t oOff, int64_t oRows,
                                            int64_t oCols, int64_t oStride0, int64_t oStride1) {
  (void)inAlloc; (void)sAlloc; (void)oAlloc; (void)inRows; (void)inCols; (void)sSize;
  const int64_t c = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  const int64_t r = int64_t(blockIdx.y) * blockDim.y + threadIdx.y;
  if (r < oRows && c < oCols)
    o[oOff + r * oStride0 + c * oStride1] =
        in[inOff + r * inStride0 + c * inStride1] * s[sOff + r * sStride];
}
