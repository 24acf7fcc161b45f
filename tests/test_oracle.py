"""CPU tests that pin the oracle without the device: the reference's golden
vectors, closed forms, identities and an fp64 library matmul.  A plausible
mistake in the oracle (dropped term, wrong sign, transposed operand, wrong
index) fails at least one of these."""
import math

import numpy as np
import pytest

import parity
import polar_oracle as o


@pytest.mark.parametrize("case", parity.golden_cases(), ids=lambda c: c["kernel"] + "@" + c["cite"].split("/")[-1])
def test_golden_vectors(case):
    parity.check_case(case, parity.run_case_oracle(case))


def test_fadd_scales_are_not_swapped():
    a = np.array([1, 0, 2], dtype=np.float32)
    b = np.array([0, 1, 4], dtype=np.float32)
    assert np.array_equal(o.fadd(a, 3.0, b, 5.0), np.array([3, 5, 26], dtype=np.float32))


def test_fadd_is_unfused():
    # sa*a + sb*b with products rounded separately: pick values where an fma
    # would differ in the last bit
    rng = np.random.default_rng(1)
    a = parity.uniform(rng, 4096, -1, 1)
    b = parity.uniform(rng, 4096, -1, 1)
    sa, sb = np.float32(0.34), np.float32(0.21)
    ref = (sa * a).astype(np.float32) + (sb * b).astype(np.float32)
    assert np.array_equal(o.fadd(a, float(sa), b, float(sb)), ref.astype(np.float32))


def test_fdivide_is_ieee_and_ordered():
    rng = np.random.default_rng(2)
    num = parity.uniform(rng, 10000, -1, 1)
    den = parity.uniform(rng, 10000, 0.5, 2)
    assert np.array_equal(o.fdivide(num, den), (num / den).astype(np.float32))
    assert o.fdivide([1.0], [4.0])[0] == np.float32(0.25)  # numerator first


def test_fmulconcat_uses_element_zero_only():
    g = np.array([2.0, 100.0, -7.0], dtype=np.float32)
    d = np.array([1.0, 2.0, 3.0, 4.0], dtype=np.float32)
    assert np.array_equal(o.fmulconcat(g, d), 2.0 * d)


def test_fsigmoid_closed_forms():
    eps = np.float32(1e-5)
    out = o.fsigmoid([0.0, -100.0, 100.0, -11.0, 11.0, -12.0, 12.0])
    assert out[0] == np.float32(0.5)
    assert out[1] == eps and out[2] == np.float32(1) - eps
    # sigma(-11) = 1.67e-5 stays, sigma(-12) = 6.1e-6 < eps is clamped
    assert abs(out[3] - 1 / (1 + math.exp(11.0))) < 1e-11
    assert abs(out[4] - 1 / (1 + math.exp(-11.0))) < 1e-7
    assert out[5] == eps and out[6] == np.float32(1) - eps
    x = np.linspace(-9, 9, 2001).astype(np.float32)
    ref = 1 / (1 + np.exp(-x.astype(np.float64)))
    assert np.max(np.abs(o.fsigmoid(x) - ref) / ref) < 3e-7
    # symmetry sigma(x) + sigma(-x) = 1
    assert np.max(np.abs(o.fsigmoid(x).astype(np.float64) + o.fsigmoid(-x) - 1)) < 2e-7


def test_flogloss_closed_forms():
    e = float(np.float32(1e-5))
    p = np.array([0.25, 0.25, 0.9, 0.9], dtype=np.float32)
    y = np.array([1, 0, 1, 0], dtype=np.float32)
    out = o.flogloss(p, y)
    exp = [-math.log(0.25 + e), -math.log(0.75 + e), -math.log(float(np.float32(0.9)) + e),
           -math.log(1 - float(np.float32(0.9)) + e)]
    assert np.allclose(out, exp, rtol=1e-6, atol=0)
    # argument order: (predicted, groundTruth), not the other way round
    assert not np.allclose(o.flogloss(y, p), exp, rtol=1e-3)
    # soft labels mix the two terms linearly
    ys = np.float32(0.3)
    mix = o.flogloss([0.25], [ys])[0]
    assert abs(mix - (float(ys) * exp[0] + (1 - float(ys)) * exp[1])) < 1e-6


def test_fcopy_ffill():
    x = np.arange(17, dtype=np.float32)
    assert np.array_equal(o.fcopy(x), x)
    assert np.array_equal(o.ffill(3.0, 9), np.full(9, 3.0, dtype=np.float32))


def test_ftranspose_definition_and_involution():
    x = np.arange(3 * 5, dtype=np.float32).reshape(3, 5)
    t = o.ftranspose(x)
    assert t.shape == (5, 3)
    for i in range(3):
        for j in range(5):
            assert t[j, i] == x[i, j]
    rng = np.random.default_rng(3)
    y = parity.normal(rng, (131, 67))
    assert np.array_equal(o.ftranspose(y), y.T)
    assert np.array_equal(o.ftranspose(o.ftranspose(y)), y)


@pytest.mark.parametrize("ta", [False, True])
@pytest.mark.parametrize("tb", [False, True])
def test_fmatmul_against_fp64_library(ta, tb):
    rng = np.random.default_rng(4)
    m, n, k = 13, 7, 29
    sa, sb = parity.stored_shapes(ta, tb, m, n, k)
    a, b = parity.normal(rng, sa), parity.normal(rng, sb)
    A = a.T if ta else a
    B = b.T if tb else b
    ref = A.astype(np.float64) @ B.astype(np.float64)
    got = o.fmatmul(ta, tb, a, b)
    assert got.shape == (m, n)
    assert parity.frobenius_rel_error(got, ref) < 1e-6
    assert parity.frobenius_rel_error(o.fmatmul_f64acc(ta, tb, a, b), ref) < 1e-14


def test_fmatmul_tt_identities():
    # no reference test exists for t_t: (A^T B^T) = (B A)^T and equality with
    # f_f on explicitly transposed operands.  Integer data keeps fp32 exact.
    rng = np.random.default_rng(5)
    m, n, k = 6, 9, 11
    a = rng.integers(-9, 10, (k, m)).astype(np.float32)  # stored [K x M]
    b = rng.integers(-9, 10, (n, k)).astype(np.float32)  # stored [N x K]
    tt = o.fmatmul(True, True, a, b)
    assert np.array_equal(tt, o.fmatmul(False, False, b, a).T)
    assert np.array_equal(tt, o.fmatmul(False, False, np.ascontiguousarray(a.T), np.ascontiguousarray(b.T)))
    assert np.array_equal(tt, o.fmatmul(True, False, a, np.ascontiguousarray(b.T)))
    assert np.array_equal(tt, o.fmatmul(False, True, np.ascontiguousarray(a.T), b))


def test_fmatmul_is_sequential_fp32():
    # sum of 1 + 2^-24 * many: a sequential fp32 accumulator stays at 1.0,
    # pairwise or fp64 accumulation would not
    k = 4096
    a = np.full((1, k), 1.0, dtype=np.float32)
    b = np.full((k, 1), 2.0 ** -25, dtype=np.float32)
    b[0, 0] = 1.0
    assert o.fmatmul(False, False, a, b)[0, 0] == np.float32(1.0)


def test_fmatmul_rows_subset_matches_full():
    rng = np.random.default_rng(6)
    a, b = parity.normal(rng, (20, 33)), parity.normal(rng, (33, 12))
    full = o.fmatmul(False, False, a, b)
    part = o.fmatmul(False, False, a, b, rows=(5, 9))
    assert np.array_equal(part[5:9], full[5:9])
    assert not part[:5].any() and not part[9:].any()


def test_threads_do_not_change_results():
    rng = np.random.default_rng(7)
    a, b = parity.normal(rng, (64, 50)), parity.normal(rng, (50, 40))
    x = parity.uniform(rng, 100003, -1, 1)
    o.set_threads(1)
    r1, s1 = o.fmatmul(False, False, a, b), o.fsigmoid(x)
    o.set_threads(4)
    r4, s4 = o.fmatmul(False, False, a, b), o.fsigmoid(x)
    o.set_threads(1)
    assert np.array_equal(r1, r4) and np.array_equal(s1, s4)


def test_record_bytes():
    # include/polarai/core/tensor/DataType.hpp:20-34 and runtime/utils/utils.hpp:7-17
    assert o.record_bytes(2, [256, 784]) == 256 * 784 * 4
    assert o.record_bytes(1, [3]) == 24
    assert o.record_bytes(3, [2, 2, 2]) == 16
    assert o.record_bytes(2, []) == 4


# ---- relu / softmax / conv2d / pool: independent library routines -------------

def test_frelu_against_numpy_and_special_values():
    rng = np.random.default_rng(31)
    x = parity.normal(rng, 10007)
    assert np.array_equal(o.frelu(x), np.maximum(x, np.float32(0)))
    special = np.array([np.nan, -np.inf, np.inf, -0.0, 0.0, np.float32(1e-45)], dtype=np.float32)
    got = o.frelu(special)
    assert got[0] == 0 and got[1] == 0 and got[2] == np.inf and got[3] == 0 and got[4] == 0
    assert got[5] == np.float32(1e-45)          # ordered greater-than: NaN -> 0, denormals kept


def test_fsoftmax_against_fp64_library():
    from scipy.special import softmax
    rng = np.random.default_rng(32)
    x = parity.normal(rng, (25, 40), std=2.0)
    ref = softmax(x.astype(np.float64), axis=None)       # over the whole tensor, not per row
    assert parity.elementwise_rel_error(o.fsoftmax(x), ref) <= 1e-5
    assert parity.elementwise_rel_error(o.fsoftmax(x, f64sum=True), ref) <= 1e-6
    assert abs(float(o.fsoftmax(x).astype(np.float64).sum()) - 1.0) < 1e-5
    # a per-row softmax would differ grossly
    assert parity.elementwise_rel_error(o.fsoftmax(x), softmax(x.astype(np.float64), axis=1)) > 0.5
    # no max subtraction: large inputs overflow to inf/inf = nan exactly as exp(x)/sum does
    with np.errstate(all="ignore"):
        assert np.isnan(o.fsoftmax(np.array([100.0, 0.0], dtype=np.float32))[0])


def test_fsoftmax_sum_is_sequential_fp32():
    # 2^24 + 1 + 1 ... stagnates in fp32: with x = 0 everywhere the running sum stops at 2^24
    n = (1 << 24) + 1000
    x = np.zeros(n, dtype=np.float32)
    assert o.fsoftmax(x)[0] == np.float32(1.0) / np.float32(1 << 24)
    assert o.fsoftmax(x, f64sum=True)[0] == np.float32(1.0) / np.float32(n)


@pytest.mark.parametrize("shape,kshape", [((4, 4), (3, 3)), ((17, 23), (5, 3)), ((9, 31), (1, 7)), ((12, 12), (11, 11))])
def test_fconv2d_against_scipy_correlate(shape, kshape):
    from scipy.signal import correlate2d
    rng = np.random.default_rng(33)
    # small integers: every product and partial sum is exact in fp32, so the
    # result must EQUAL the library's (a flipped kernel, i.e. a true convolution,
    # or a swapped index would not)
    x = rng.integers(-8, 9, size=shape).astype(np.float32)
    w = rng.integers(-4, 5, size=kshape).astype(np.float32)
    ref = correlate2d(x.astype(np.float64), w.astype(np.float64), mode="valid")
    assert np.array_equal(o.fconv2d(x, w), ref.astype(np.float32))
    assert not np.array_equal(o.fconv2d(x, w[::-1, ::-1].copy()), ref.astype(np.float32)) or w.size == 1
    xr, wr = parity.normal(rng, shape), parity.normal(rng, kshape)
    ref = correlate2d(xr.astype(np.float64), wr.astype(np.float64), mode="valid")
    assert parity.frobenius_rel_error(o.fconv2d(xr, wr), ref) <= 1e-6


def test_fconv2d_accumulates_in_tap_order_unfused():
    # taps chosen so that fp32 order matters: 1e8 + 1 - 1e8 is 0 in tap order, 1 if reordered
    x = np.ones((1, 3), dtype=np.float32)
    w = np.array([[1e8, 1.0, -1e8]], dtype=np.float32)
    assert o.fconv2d(x, w)[0, 0] == 0.0
    w2 = np.array([[1e8, -1e8, 1.0]], dtype=np.float32)
    assert o.fconv2d(x, w2)[0, 0] == 1.0
    # product rounded before the add (no fma): a*b + c with a*b inexact
    a = np.float32(1 + 2 ** -12)
    x3 = np.array([[a, 1.0]], dtype=np.float32)
    w3 = np.array([[a, -(np.float32(a * a))]], dtype=np.float32)
    assert o.fconv2d(x3, w3)[0, 0] == 0.0


@pytest.mark.parametrize("shape,window,stride", [((4, 4), (2, 2), (2, 2)), ((9, 14), (3, 2), (3, 2)),
                                                 ((10, 11), (3, 3), (2, 1)), ((7, 7), (7, 7), (1, 1)),
                                                 ((8, 9), (1, 1), (3, 4))])
def test_fpool_against_sliding_windows(shape, window, stride):
    from numpy.lib.stride_tricks import sliding_window_view
    rng = np.random.default_rng(34)
    x = parity.normal(rng, shape)
    ref = sliding_window_view(x, window)[::stride[0], ::stride[1]].max(axis=(2, 3))
    got = o.fpool(x, window, stride)
    assert got.shape == ref.shape == ((shape[0] - window[0]) // stride[0] + 1, (shape[1] - window[1]) // stride[1] + 1)
    assert np.array_equal(got, ref)


def test_fpool_floor_and_nan():
    # the running maximum starts at -10e5: smaller inputs are clamped to it, NaN is skipped
    x = np.array([[-2e6, -3e6], [np.nan, -5e6]], dtype=np.float32)
    assert o.fpool(x, (2, 2), (2, 2))[0, 0] == np.float32(-10e5)
    x[1, 1] = 7
    assert o.fpool(x, (2, 2), (2, 2))[0, 0] == 7
