#!/usr/bin/env python3
"""Writes tests/golden/reference_vectors.json.

Inputs are the literal vectors of the reference's integration tests (cited per
case, paths relative to the reference tree).  The reference computes its
expected values at run time with in-file loops that cannot be built here
(googletest + the framework), so the expected values below are derived
independently of the oracle:
  * single IEEE fp32 operations (add/combine/mul/divide/mulconcat) are
    evaluated with numpy float32 scalars, which round exactly as the
    reference's float arithmetic does;
  * the matmul cases use small integers, so the integer dot products computed
    with Python ints are the exact fp32 results;
  * sigmoid and logloss are evaluated in fp64 with Python's math library and
    carry a tolerance (they go through exp/log whose last bit is
    implementation-defined).
  * relu and pool expectations are the literals of the reference's tests; softmax
    is evaluated in fp64 and checked against the reference's literals; conv2d
    keeps the reference's literal with its 4-ulp comparison.
Nothing here imports the oracle or the device library.
"""
import json
import math
import os

import numpy as np

f32 = np.float32
cases = []


def vec(xs):
    return [float(f32(x)) for x in xs]


# tests/integration/operations/AddOperation.cpp:22-24 (expected is literal there)
cases.append(dict(kernel="fadd", cite="tests/integration/operations/AddOperation.cpp:22-24",
                  a=vec([1, 2, 3, 4]), scaleA=1.0, b=vec([7, 8, 9, 10]), scaleB=1.0,
                  expected=vec([8, 10, 12, 14]), exact=True))

# tests/integration/operations/CombineOperation.cpp:32-34
al, be = f32(0.34), f32(0.21)
a, b = [f32(x) for x in (1, 2, 3, 4)], [f32(x) for x in (7, 8, 9, 10)]
cases.append(dict(kernel="fadd", cite="tests/integration/operations/CombineOperation.cpp:32-34",
                  a=vec(a), scaleA=float(al), b=vec(b), scaleB=float(be),
                  expected=vec([f32(f32(al * x) + f32(be * y)) for x, y in zip(a, b)]), exact=True))

# tests/integration/operations/MulOperation.cpp:32-33
a, b = [f32(x) for x in (8, 2, 5, 6)], [f32(x) for x in (3, 2, 1, 0.34)]
cases.append(dict(kernel="fmul", cite="tests/integration/operations/MulOperation.cpp:32-33",
                  a=vec(a), b=vec(b), expected=vec([f32(x * y) for x, y in zip(a, b)]), exact=True))

# tests/integration/operations/DivideOperation.cpp:32-33
a, b = [f32(x) for x in (1, 2, 3, 4)], [f32(x) for x in (7, 8, 9, 10)]
cases.append(dict(kernel="fdivide", cite="tests/integration/operations/DivideOperation.cpp:32-33",
                  a=vec(a), b=vec(b), expected=vec([f32(x / y) for x, y in zip(a, b)]), exact=True))

# tests/integration/operations/MulConcatOperation.cpp:32-33 (gradient shape {1,1})
loc, g = [f32(x) for x in (-100, 2, 5, 50)], f32(17.5)
cases.append(dict(kernel="fmulconcat", cite="tests/integration/operations/MulConcatOperation.cpp:32-33",
                  gradient=vec([g]), local=vec(loc), expected=vec([f32(g * x) for x in loc]), exact=True))


def matmul_case(cite, ta, tb, m, n, k, left, right):
    # stored shapes: left [k x m] if ta else [m x k]; right [n x k] if tb else [k x n]
    def L(i, kk):
        return left[kk * m + i] if ta else left[i * k + kk]

    def R(kk, j):
        return right[j * k + kk] if tb else right[kk * n + j]
    exp = [sum(L(i, kk) * R(kk, j) for kk in range(k)) for i in range(m) for j in range(n)]
    assert all(abs(v) < 2 ** 24 for v in exp)
    cases.append(dict(kernel="fmatmul", cite=cite, transA=ta, transB=tb, m=m, n=n, k=k,
                      a=vec(left), b=vec(right), expected=vec(exp), exact=True))


T = "tests/integration/operations/MatMulOperation.cpp"
matmul_case(T + ":58-60", False, False, 1, 1, 4, [3, 4, 5, 10], [6, 7, 8, 11])
matmul_case(T + ":105-107", False, False, 2, 2, 2, [3, 4, 5, 10], [6, 7, 8, 11])
matmul_case(T + ":151-153", False, False, 2, 3, 4, [3, 4, 5, 10, 6, 7, 12, 6],
            [6, 7, 8, 11, 7, 8, 9, 1, 3, 2, 5, 6])
matmul_case(T + ":198-204", True, False, 2, 3, 4, [3, 6, 4, 7, 5, 12, 10, 6],
            [6, 7, 8, 11, 7, 8, 9, 1, 3, 2, 5, 6])
matmul_case(T + ":244-250", False, True, 2, 3, 4, [3, 4, 5, 10, 6, 7, 12, 6],
            [6, 11, 9, 2, 7, 7, 1, 5, 8, 8, 3, 6])

# tests/integration/operations/SigmoidOperation.cpp:39 (test DISABLED_ upstream).
# -100 saturates to exactly eps and 50 to exactly 1-eps (fp32 values).
eps = f32(1e-5)
xs = [-100.0, 2.0, 5.0, 50.0]
exp = [float(eps), 1 / (1 + math.exp(-2.0)), 1 / (1 + math.exp(-5.0)), float(f32(1) - eps)]
cases.append(dict(kernel="fsigmoid", cite="tests/integration/operations/SigmoidOperation.cpp:39",
                  x=xs, expected=exp, exact=False, rel_tol=1e-6, exact_indices=[0, 3]))

# tests/integration/operations/LogLossOperation.cpp:37-38 (test DISABLED_ upstream)
p, y = vec([0.6, 0.2, 0.8, 0.3]), [1.0, 0.0, 1.0, 0.0]
e64 = float(eps)
exp = [-(yy * math.log(pp + e64)) - (1 - yy) * math.log(1 - pp + e64) for pp, yy in zip(p, y)]
cases.append(dict(kernel="flogloss", cite="tests/integration/operations/LogLossOperation.cpp:37-38",
                  predicted=p, truth=y, expected=exp, exact=False, rel_tol=1e-6))

# tests/integration/operations/ReLUOperation.cpp:36-37 (expected is literal there)
cases.append(dict(kernel="frelu", cite="tests/integration/operations/ReLUOperation.cpp:36-37",
                  x=vec([-1, 1]), expected=vec([0, 1]), exact=True))

# tests/integration/operations/SoftmaxOperation.cpp:36-39: shape {2,2}, softmax over the whole
# tensor.  The reference compares with EXPECT_FLOAT_EQ (4 ulp) against the literals
# {0.0320586, 0.08714432, 0.23688282, 0.64391426}; the expected values here are the fp64
# evaluation of exp(x)/sum(exp), which those literals round.
xs = [1.0, 2.0, 3.0, 4.0]
den = sum(math.exp(v) for v in xs)
exp = [math.exp(v) / den for v in xs]
lit = [0.0320586, 0.08714432, 0.23688282, 0.64391426]
assert all(abs(e - l) <= 4 * 2.0 ** -24 * l for e, l in zip(exp, lit))
cases.append(dict(kernel="fsoftmax", cite="tests/integration/operations/SoftmaxOperation.cpp:36-39",
                  x=xs, shape=[2, 2], expected=exp, exact=False, rel_tol=4 * 2.0 ** -23))

# tests/integration/operations/Conv2DOperation.cpp:36-40: 4x4 ones, 3x3 kernel of 0.1,
# expected {0.9 x4} under EXPECT_FLOAT_EQ (4 ulp; the nine-term fp32 sum is not exactly 0.9f)
cases.append(dict(kernel="fconv2d", cite="tests/integration/operations/Conv2DOperation.cpp:36-40",
                  x=vec([1] * 16), shape=[4, 4], weights=vec([0.1] * 9), kernel_shape=[3, 3],
                  expected=[0.9] * 4, exact=False, rel_tol=4 * 2.0 ** -23))

# tests/integration/operations/Pool2DOperation.cpp:36-49: 4x4 input, window {2,2}, stride {2,2}
cases.append(dict(kernel="fpool", cite="tests/integration/operations/Pool2DOperation.cpp:36-49",
                  x=vec([1, 0, 2, 3, 4, 6, 6, 8, 3, 1, 1, 0, 1, 2, 2, 4]), shape=[4, 4],
                  window=[2, 2], stride=[2, 2], expected=vec([6, 8, 3, 4]), exact=True))

out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_vectors.json")
with open(out, "w") as fh:
    json.dump(cases, fh, indent=1)
print(f"wrote {len(cases)} cases to {out}")
