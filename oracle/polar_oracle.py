"""ctypes binding of the CPU oracle (oracle/polar_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
bench.py's cpu_baseline leg -- as the checker and the reported baseline, never
by the product path.
"""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libpolar_oracle.so")

_fp = np.ctypeslib.ndpointer(dtype=np.float32, flags="C_CONTIGUOUS")
_dp = np.ctypeslib.ndpointer(dtype=np.float64, flags="C_CONTIGUOUS")
_u64 = C.c_uint64
_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise FileNotFoundError(f"{LIB_PATH} is not built (make -C oracle)")
        l = C.CDLL(LIB_PATH)
        l.polar_oracle_set_threads.argtypes = [C.c_int]
        l.polar_oracle_get_threads.restype = C.c_int
        l.polar_oracle_hw_threads.restype = C.c_int
        l.polar_oracle_fadd.argtypes = [_fp, C.c_float, _fp, C.c_float, _fp, _u64]
        l.polar_oracle_fmul.argtypes = [_fp, _fp, _fp, _u64]
        l.polar_oracle_fdivide.argtypes = [_fp, _fp, _fp, _u64]
        l.polar_oracle_fsigmoid.argtypes = [_fp, _fp, _u64]
        l.polar_oracle_flogloss.argtypes = [_fp, _fp, _fp, _u64]
        l.polar_oracle_fmulconcat.argtypes = [_fp, _fp, _fp, _u64]
        l.polar_oracle_fcopy.argtypes = [_fp, _fp, _u64]
        l.polar_oracle_ffill.argtypes = [C.c_float, _fp, _u64]
        l.polar_oracle_ftranspose.argtypes = [_fp, _fp, _u64, _u64]
        l.polar_oracle_fmatmul.argtypes = [C.c_int, C.c_int, _fp, _u64, _u64, _fp, _u64, _u64, _fp, _u64, _u64]
        l.polar_oracle_fmatmul_rows.argtypes = [C.c_int, C.c_int, _fp, _u64, _u64, _fp, _u64, _u64, _fp, _u64, _u64, _u64, _u64]
        l.polar_oracle_fmatmul_f64acc.argtypes = [C.c_int, C.c_int, _fp, _u64, _u64, _fp, _u64, _u64, _dp, _u64, _u64]
        l.polar_oracle_frelu.argtypes = [_fp, _fp, _u64]
        l.polar_oracle_fsoftmax.argtypes = [_fp, _fp, _u64]
        l.polar_oracle_fsoftmax_f64sum.argtypes = [_fp, _fp, _u64]
        l.polar_oracle_fconv2d.argtypes = [_fp, _fp, _fp, _u64, _u64, _u64, _u64]
        l.polar_oracle_fpool.argtypes = [_fp, _fp, _u64, _u64, _u64, _u64, _u64, _u64]
        l.polar_oracle_record_bytes.argtypes = [C.c_int, _u64, C.POINTER(_u64)]
        l.polar_oracle_record_bytes.restype = _u64
        _lib = l
    return _lib


def set_threads(n):
    lib().polar_oracle_set_threads(int(n))


def hw_threads():
    return lib().polar_oracle_hw_threads()


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def fadd(a, sa, b, sb):
    a, b = _f32(a), _f32(b)
    c = np.empty_like(a)
    lib().polar_oracle_fadd(a.ravel(), sa, b.ravel(), sb, c.ravel(), a.size)
    return c


def fmul(a, b):
    a, b = _f32(a), _f32(b)
    c = np.empty_like(a)
    lib().polar_oracle_fmul(a.ravel(), b.ravel(), c.ravel(), a.size)
    return c


def fdivide(num, den):
    num, den = _f32(num), _f32(den)
    c = np.empty_like(num)
    lib().polar_oracle_fdivide(num.ravel(), den.ravel(), c.ravel(), num.size)
    return c


def fsigmoid(x):
    x = _f32(x)
    c = np.empty_like(x)
    lib().polar_oracle_fsigmoid(x.ravel(), c.ravel(), x.size)
    return c


def flogloss(pred, truth):
    pred, truth = _f32(pred), _f32(truth)
    c = np.empty_like(pred)
    lib().polar_oracle_flogloss(pred.ravel(), truth.ravel(), c.ravel(), pred.size)
    return c


def fmulconcat(grad, local):
    grad, local = _f32(grad), _f32(local)
    c = np.empty_like(local)
    lib().polar_oracle_fmulconcat(grad.ravel(), local.ravel(), c.ravel(), local.size)
    return c


def fcopy(src):
    src = _f32(src)
    c = np.empty_like(src)
    lib().polar_oracle_fcopy(src.ravel(), c.ravel(), src.size)
    return c


def ffill(pattern, n):
    c = np.empty(int(n), dtype=np.float32)
    lib().polar_oracle_ffill(pattern, c, c.size)
    return c


def ftranspose(x):
    x = _f32(x)
    assert x.ndim == 2
    out = np.empty((x.shape[1], x.shape[0]), dtype=np.float32)
    lib().polar_oracle_ftranspose(x.ravel(), out.ravel(), x.shape[0], x.shape[1])
    return out


def frelu(x):
    x = _f32(x)
    c = np.empty_like(x)
    lib().polar_oracle_frelu(x.ravel(), c.ravel(), x.size)
    return c


def fsoftmax(x, f64sum=False):
    """Softmax over the whole tensor; f64sum selects the fp64-accumulated sum."""
    x = _f32(x)
    c = np.empty_like(x)
    fn = lib().polar_oracle_fsoftmax_f64sum if f64sum else lib().polar_oracle_fsoftmax
    fn(x.ravel(), c.ravel(), x.size)
    return c


def fconv2d(x, kernel):
    x, kernel = _f32(x), _f32(kernel)
    assert x.ndim == 2 and kernel.ndim == 2
    out = np.empty((x.shape[0] - kernel.shape[0] + 1, x.shape[1] - kernel.shape[1] + 1), dtype=np.float32)
    lib().polar_oracle_fconv2d(x.ravel(), kernel.ravel(), out.ravel(), x.shape[0], x.shape[1],
                               kernel.shape[0], kernel.shape[1])
    return out


def fpool(x, window, stride):
    x = _f32(x)
    assert x.ndim == 2
    out = np.empty(((x.shape[0] - window[0]) // stride[0] + 1, (x.shape[1] - window[1]) // stride[1] + 1),
                   dtype=np.float32)
    lib().polar_oracle_fpool(x.ravel(), out.ravel(), x.shape[0], x.shape[1], window[0], window[1],
                             stride[0], stride[1])
    return out


def _mn(ta, tb, a, b):
    m = a.shape[1] if ta else a.shape[0]
    n = b.shape[0] if tb else b.shape[1]
    return m, n


def fmatmul(ta, tb, a, b, rows=None):
    """a, b are the STORED 2-D arrays (a is [K x M] when ta, b is [N x K] when
    tb).  rows=(r0, r1) computes only those rows of C (others are left 0)."""
    a, b = _f32(a), _f32(b)
    m, n = _mn(ta, tb, a, b)
    if rows is None:
        c = np.empty((m, n), dtype=np.float32)
        lib().polar_oracle_fmatmul(int(ta), int(tb), a.ravel(), a.shape[0], a.shape[1],
                                   b.ravel(), b.shape[0], b.shape[1], c.ravel(), m, n)
    else:
        c = np.zeros((m, n), dtype=np.float32)
        lib().polar_oracle_fmatmul_rows(int(ta), int(tb), a.ravel(), a.shape[0], a.shape[1],
                                        b.ravel(), b.shape[0], b.shape[1], c.ravel(), m, n,
                                        rows[0], rows[1])
    return c


def fmatmul_f64acc(ta, tb, a, b):
    a, b = _f32(a), _f32(b)
    m, n = _mn(ta, tb, a, b)
    c = np.empty((m, n), dtype=np.float64)
    lib().polar_oracle_fmatmul_f64acc(int(ta), int(tb), a.ravel(), a.shape[0], a.shape[1],
                                      b.ravel(), b.shape[0], b.shape[1], c.ravel(), m, n)
    return c


def record_bytes(dtype_code, shape):
    arr = (_u64 * len(shape))(*shape)
    return lib().polar_oracle_record_bytes(dtype_code, len(shape), arr)
