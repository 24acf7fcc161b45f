// nativeKernelName -> device-library entry point, with the argument order the
// launch lowering uses for each builtin.  The orders are those of the
// framework's hand-written runtime (src/backend/generic/runtime/sycl/kernels/)
// and of the IR (utils/dialects/test/ir/operations.mlir:13-168).
#include "hip_plugin.hpp"

#include <cstring>

namespace polarai::backend::generic::mi355x {
namespace {

struct TensorArg {
  TensorInfo* info;
  MemoryRecord record;
  uint64_t count;
};

// src/backend/generic/runtime/utils/utils.hpp:7-17
MemoryRecord recordOf(const TensorInfo* t) {
  if (t->dataType != static_cast<int>(core::DataType::FLOAT))
    fatal("tensor %llu has data type %d; this runtime is fp32 only",
          static_cast<unsigned long long>(t->virtAddr), t->dataType);
  size_t bytes = 4;
  for (uint64_t i = 0; i < t->dims; ++i) bytes *= t->shape[i];
  return MemoryRecord{static_cast<size_t>(t->virtAddr), bytes};
}

TensorArg tensorArg(const LaunchCommand& cmd, uint64_t i) {
  if (i >= cmd.argsCount)
    fatal("%s: argument %llu missing (%llu given)", cmd.nativeKernelName,
          static_cast<unsigned long long>(i),
          static_cast<unsigned long long>(cmd.argsCount));
  const ArgDesc& a = cmd.args[i];
  if (a.type != ArgDesc::TENSOR || a.arg == nullptr)
    fatal("%s: argument %llu must be a tensor", cmd.nativeKernelName,
          static_cast<unsigned long long>(i));
  auto* info = static_cast<TensorInfo*>(a.arg);
  TensorArg t{info, recordOf(info), 0};
  t.count = t.record.allocationSize / 4;
  return t;
}

// Scalars are copied out here: `arg` points at stack memory of the caller.
float scalarArg(const LaunchCommand& cmd, uint64_t i) {
  if (i >= cmd.argsCount)
    fatal("%s: argument %llu missing", cmd.nativeKernelName,
          static_cast<unsigned long long>(i));
  const ArgDesc& a = cmd.args[i];
  if (a.type != ArgDesc::DATA || a.arg == nullptr)
    fatal("%s: argument %llu must be a scalar", cmd.nativeKernelName,
          static_cast<unsigned long long>(i));
  if (a.size == 4) {
    float v;
    std::memcpy(&v, a.arg, 4);
    return v;
  }
  if (a.size == 8) {
    double v;
    std::memcpy(&v, a.arg, 8);
    return static_cast<float>(v);
  }
  fatal("%s: scalar argument %llu has %llu bytes", cmd.nativeKernelName,
        static_cast<unsigned long long>(i), static_cast<unsigned long long>(a.size));
}

void needAtLeast(const LaunchCommand& cmd, const TensorArg& in, uint64_t n) {
  if (in.count < n)
    fatal("%s: operand %zu holds %llu elements, %llu needed", cmd.nativeKernelName,
          in.record.virtualAddress, static_cast<unsigned long long>(in.count),
          static_cast<unsigned long long>(n));
}

// Integer attribute passed as a scalar argument (4 or 8 bytes, signed).
uint64_t countArg(const LaunchCommand& cmd, uint64_t i) {
  if (i >= cmd.argsCount)
    fatal("%s: argument %llu missing", cmd.nativeKernelName,
          static_cast<unsigned long long>(i));
  const ArgDesc& a = cmd.args[i];
  if (a.type != ArgDesc::DATA || a.arg == nullptr)
    fatal("%s: argument %llu must be a scalar", cmd.nativeKernelName,
          static_cast<unsigned long long>(i));
  int64_t v = 0;
  if (a.size == 8) {
    std::memcpy(&v, a.arg, 8);
  } else if (a.size == 4) {
    int32_t w;
    std::memcpy(&w, a.arg, 4);
    v = w;
  } else {
    fatal("%s: integer argument %llu has %llu bytes", cmd.nativeKernelName,
          static_cast<unsigned long long>(i), static_cast<unsigned long long>(a.size));
  }
  if (v <= 0)
    fatal("%s: integer argument %llu must be positive", cmd.nativeKernelName,
          static_cast<unsigned long long>(i));
  return static_cast<uint64_t>(v);
}

void checkMatmulShapes(const LaunchCommand& cmd, bool ta, bool tb, const TensorArg& a,
                       const TensorArg& b, const TensorArg& c, uint64_t* m, uint64_t* n,
                       uint64_t* k) {
  if (a.info->dims != 2 || b.info->dims != 2 || c.info->dims != 2)
    fatal("%s: operands must be 2-D", cmd.nativeKernelName);
  *m = c.info->shape[0];
  *n = c.info->shape[1];
  *k = ta ? a.info->shape[0] : a.info->shape[1];
  const uint64_t am = ta ? a.info->shape[1] : a.info->shape[0];
  const uint64_t bk = tb ? b.info->shape[1] : b.info->shape[0];
  const uint64_t bn = tb ? b.info->shape[0] : b.info->shape[1];
  if (am != *m || bk != *k || bn != *n)
    fatal("%s: shapes do not agree: opA is %llux%llu, opB is %llux%llu, C is %llux%llu",
          cmd.nativeKernelName, (unsigned long long)am, (unsigned long long)*k,
          (unsigned long long)bk, (unsigned long long)bn, (unsigned long long)*m,
          (unsigned long long)*n);
}

using Launcher = void (*)(HipDevice&, BackendAllocator&, LaunchCommand&);

// [0]a T [1]scaleA D [2]b T [3]scaleB D [4]c T; range = c
// (sycl/kernels/AddNaive.hpp:98-125)
void launchAdd(HipDevice& d, BackendAllocator& al, LaunchCommand& cmd) {
  TensorArg a = tensorArg(cmd, 0), b = tensorArg(cmd, 2), c = tensorArg(cmd, 4);
  const float sa = scalarArg(cmd, 1), sb = scalarArg(cmd, 3);
  needAtLeast(cmd, a, c.count);
  needAtLeast(cmd, b, c.count);
  checkStatus(polar_hip_fadd(d.native(), d.resolve(al, a.record), sa,
                             d.resolve(al, b.record), sb, d.resolve(al, c.record),
                             c.count),
              "polar_hip_fadd");
}

// [0] [1] inputs, [2] out; range = out (sycl/kernels/Mul.hpp:50-57,
// Divide.hpp:53-60, LogLoss.hpp:55-62, MulConcat.hpp:53-60)
template <int (*Fn)(polar_hip_device*, const float*, const float*, float*, uint64_t),
          bool FirstIsScalarTensor>
void launchBinary(HipDevice& d, BackendAllocator& al, LaunchCommand& cmd) {
  TensorArg x = tensorArg(cmd, 0), y = tensorArg(cmd, 1), out = tensorArg(cmd, 2);
  needAtLeast(cmd, x, FirstIsScalarTensor ? 1 : out.count);
  needAtLeast(cmd, y, out.count);
  checkStatus(Fn(d.native(), d.resolve(al, x.record), d.resolve(al, y.record),
                 d.resolve(al, out.record), out.count),
              cmd.nativeKernelName);
}

// [0]in T [1]out T (sycl/kernels/Sigmoid.hpp:59-63)
void launchSigmoid(HipDevice& d, BackendAllocator& al, LaunchCommand& cmd) {
  TensorArg in = tensorArg(cmd, 0), out = tensorArg(cmd, 1);
  needAtLeast(cmd, in, out.count);
  checkStatus(polar_hip_fsigmoid(d.native(), d.resolve(al, in.record),
                                 d.resolve(al, out.record), out.count),
              "polar_hip_fsigmoid");
}

// [0]in T [1]out T (utils/dialects/include/PolarGraph/PolarGraphOps.td:447-466,
// 486-505: operands (input, out))
template <int (*Fn)(polar_hip_device*, const float*, float*, uint64_t)>
void launchUnary(HipDevice& d, BackendAllocator& al, LaunchCommand& cmd) {
  TensorArg in = tensorArg(cmd, 0), out = tensorArg(cmd, 1);
  needAtLeast(cmd, in, out.count);
  checkStatus(Fn(d.native(), d.resolve(al, in.record), d.resolve(al, out.record), out.count),
              cmd.nativeKernelName);
}

// [0]input T [1]kernel T [2]out T, all 2-D
// (utils/dialects/include/PolarGraph/PolarGraphOps.td:243-260)
void launchConv2D(HipDevice& d, BackendAllocator& al, LaunchCommand& cmd) {
  TensorArg in = tensorArg(cmd, 0), k = tensorArg(cmd, 1), out = tensorArg(cmd, 2);
  if (in.info->dims != 2 || k.info->dims != 2 || out.info->dims != 2)
    fatal("fconv2d: operands must be 2-D");
  const uint64_t h = in.info->shape[0], w = in.info->shape[1];
  const uint64_t kh = k.info->shape[0], kw = k.info->shape[1];
  if (kh > h || kw > w || out.info->shape[0] != h - kh + 1 || out.info->shape[1] != w - kw + 1)
    fatal("fconv2d: shapes do not agree: input %llux%llu, kernel %llux%llu, out %llux%llu",
          (unsigned long long)h, (unsigned long long)w, (unsigned long long)kh,
          (unsigned long long)kw, (unsigned long long)out.info->shape[0],
          (unsigned long long)out.info->shape[1]);
  checkStatus(polar_hip_fconv2d(d.native(), d.resolve(al, in.record), d.resolve(al, k.record),
                                d.resolve(al, out.record), h, w, kh, kw),
              "polar_hip_fconv2d");
}

// [0]input T [1]out T, then the op's attributes as integer scalars:
// [2]window0 [3]window1 [4]stride0 [5]stride1.  Upstream keeps window and
// stride as attributes of the graph op
// (utils/dialects/include/PolarGraph/PolarGraphOps.td:405-445) and its launch
// lowering forwards operands only, so a native fpool needs them appended.
void launchPool(HipDevice& d, BackendAllocator& al, LaunchCommand& cmd) {
  TensorArg in = tensorArg(cmd, 0), out = tensorArg(cmd, 1);
  if (in.info->dims != 2 || out.info->dims != 2) fatal("fpool: operands must be 2-D");
  if (cmd.argsCount < 6)
    fatal("fpool: window and stride must follow the tensors as four integer scalars");
  const uint64_t w0 = countArg(cmd, 2), w1 = countArg(cmd, 3);
  const uint64_t s0 = countArg(cmd, 4), s1 = countArg(cmd, 5);
  const uint64_t h = in.info->shape[0], w = in.info->shape[1];
  if (w0 > h || w1 > w || out.info->shape[0] != (h - w0) / s0 + 1 ||
      out.info->shape[1] != (w - w1) / s1 + 1)
    fatal("fpool: shapes do not agree: input %llux%llu, window %llux%llu, stride %llux%llu, "
          "out %llux%llu",
          (unsigned long long)h, (unsigned long long)w, (unsigned long long)w0,
          (unsigned long long)w1, (unsigned long long)s0, (unsigned long long)s1,
          (unsigned long long)out.info->shape[0], (unsigned long long)out.info->shape[1]);
  checkStatus(polar_hip_fpool(d.native(), d.resolve(al, in.record), d.resolve(al, out.record),
                              h, w, w0, w1, s0, s1),
              "polar_hip_fpool");
}

// [0]src T [1]dst T; the whole source is copied (sycl/kernels/Copy.hpp:38-53)
void launchCopy(HipDevice& d, BackendAllocator& al, LaunchCommand& cmd) {
  TensorArg src = tensorArg(cmd, 0), dst = tensorArg(cmd, 1);
  needAtLeast(cmd, dst, src.count);
  checkStatus(polar_hip_fcopy(d.native(), d.resolve(al, src.record),
                              d.resolve(al, dst.record), src.count),
              "polar_hip_fcopy");
}

// [0]pattern D [1]out T (sycl/kernels/Fill.hpp:65-74)
void launchFill(HipDevice& d, BackendAllocator& al, LaunchCommand& cmd) {
  const float pattern = scalarArg(cmd, 0);
  TensorArg out = tensorArg(cmd, 1);
  checkStatus(polar_hip_ffill(d.native(), pattern, d.resolve(al, out.record), out.count),
              "polar_hip_ffill");
}

// [0]a T [1]out T, a is 2-D (utils/dialects/include/PolarGraph/PolarGraphOps.td:507-527)
void launchTranspose(HipDevice& d, BackendAllocator& al, LaunchCommand& cmd) {
  TensorArg a = tensorArg(cmd, 0), out = tensorArg(cmd, 1);
  if (a.info->dims != 2) fatal("ftranspose: operand must be 2-D");
  needAtLeast(cmd, out, a.count);
  checkStatus(polar_hip_ftranspose(d.native(), d.resolve(al, a.record),
                                   d.resolve(al, out.record), a.info->shape[0],
                                   a.info->shape[1]),
              "polar_hip_ftranspose");
}

// [0]A T [1]B T [2]C T; M, N = C.shape; K = A.shape[transA ? 0 : 1]
// (sycl/kernels/MatMul.hpp:33-39,130-155).  The framework launches over C's
// shape and never checks the operands against it; a mismatch would read out of
// bounds on a GPU, so it is fatal here.
template <bool TA, bool TB>
void launchMatMul(HipDevice& d, BackendAllocator& al, LaunchCommand& cmd) {
  TensorArg a = tensorArg(cmd, 0), b = tensorArg(cmd, 1), c = tensorArg(cmd, 2);
  uint64_t m, n, k;
  checkMatmulShapes(cmd, TA, TB, a, b, c, &m, &n, &k);
  checkStatus(polar_hip_fmatmul(d.native(), TA, TB, d.resolve(al, a.record),
                                d.resolve(al, b.record), d.resolve(al, c.record), m, n, k),
              cmd.nativeKernelName);
}

// Extended (fused) builtins; none of them is emitted by the graph compiler
// (docs/design/llvm/04_builtins.md:12-19), an optimisation pass would.
// fmatmul_X_Y_fsigmoid: [0]A T [1]B T [2]out T
template <bool TA, bool TB>
void launchMatMulSigmoid(HipDevice& d, BackendAllocator& al, LaunchCommand& cmd) {
  TensorArg a = tensorArg(cmd, 0), b = tensorArg(cmd, 1), c = tensorArg(cmd, 2);
  uint64_t m, n, k;
  checkMatmulShapes(cmd, TA, TB, a, b, c, &m, &n, &k);
  checkStatus(polar_hip_fmatmul_fsigmoid(d.native(), TA, TB, d.resolve(al, a.record),
                                         d.resolve(al, b.record), d.resolve(al, c.record), m,
                                         n, k),
              cmd.nativeKernelName);
}

// fmatmul_X_Y_fadd_fsigmoid: [0]A T [1]B T [2]scaleProduct D [3]bias T [4]scaleBias D [5]out T
// (the matmul's operands followed by fadd's remaining ones)
template <bool TA, bool TB>
void launchMatMulAddSigmoid(HipDevice& d, BackendAllocator& al, LaunchCommand& cmd) {
  TensorArg a = tensorArg(cmd, 0), b = tensorArg(cmd, 1), bias = tensorArg(cmd, 3),
            c = tensorArg(cmd, 5);
  const float sp = scalarArg(cmd, 2), sb = scalarArg(cmd, 4);
  uint64_t m, n, k;
  checkMatmulShapes(cmd, TA, TB, a, b, c, &m, &n, &k);
  needAtLeast(cmd, bias, c.count);
  checkStatus(polar_hip_fmatmul_fadd_fsigmoid(d.native(), TA, TB, d.resolve(al, a.record),
                                              d.resolve(al, b.record), sp,
                                              d.resolve(al, bias.record), sb,
                                              d.resolve(al, c.record), m, n, k),
              cmd.nativeKernelName);
}

struct TableEntry {
  const char* name;
  Launcher fn;
};

// Names: utils/dialects/include/PolarGraph/PolarGraphOps.td:237,275,296,317,
// 343-351,371,393,481,523,542.
const TableEntry kTable[] = {
    {"fadd", launchAdd},
    {"fmul", launchBinary<polar_hip_fmul, false>},
    {"fdivide", launchBinary<polar_hip_fdivide, false>},
    {"flogloss", launchBinary<polar_hip_flogloss, false>},
    {"fmulconcat", launchBinary<polar_hip_fmulconcat, true>},
    {"fsigmoid", launchSigmoid},
    {"fcopy", launchCopy},
    {"ffill", launchFill},
    {"ftranspose", launchTranspose},
    {"frelu", launchUnary<polar_hip_frelu>},
    {"fsoftmax", launchUnary<polar_hip_fsoftmax>},
    {"fconv2d", launchConv2D},
    {"fpool", launchPool},
    {"fmatmul_f_f", launchMatMul<false, false>},
    {"fmatmul_f_t", launchMatMul<false, true>},
    {"fmatmul_t_f", launchMatMul<true, false>},
    {"fmatmul_t_t", launchMatMul<true, true>},
    {"fsigmoid_flogloss", launchBinary<polar_hip_fsigmoid_flogloss, false>},
    {"fmatmul_f_f_fsigmoid", launchMatMulSigmoid<false, false>},
    {"fmatmul_f_t_fsigmoid", launchMatMulSigmoid<false, true>},
    {"fmatmul_t_f_fsigmoid", launchMatMulSigmoid<true, false>},
    {"fmatmul_t_t_fsigmoid", launchMatMulSigmoid<true, true>},
    {"fmatmul_f_f_fadd_fsigmoid", launchMatMulAddSigmoid<false, false>},
    {"fmatmul_f_t_fadd_fsigmoid", launchMatMulAddSigmoid<false, true>},
    {"fmatmul_t_f_fadd_fsigmoid", launchMatMulAddSigmoid<true, false>},
    {"fmatmul_t_t_fadd_fsigmoid", launchMatMulAddSigmoid<true, true>},
};

} // namespace

bool dispatchNativeKernel(HipDevice& device, BackendAllocator& allocator,
                          LaunchCommand& cmd) {
  for (const TableEntry& e : kTable) {
    if (std::strcmp(e.name, cmd.nativeKernelName) == 0) {
      e.fn(device, allocator, cmd);
      return true;
    }
  }
  return false;
}

} // namespace polarai::backend::generic::mi355x
