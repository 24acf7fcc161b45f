"""ctypes binding of include/polar_hip.h (the device library's C ABI).

Every function of the header is bound with its exact signature; a non-zero
status raises ``PolarHipError`` carrying ``polar_hip_last_error()``.  The
``Device`` class is a thin convenience over the raw calls for tests and the
benchmark: it moves numpy arrays in and out of pool memory and enqueues the
builtin-operation kernels.  There is no fallback path: a missing library or a
missing GPU raises.
"""
import ctypes as C
import os

import numpy as np

from . import LIB_DEVICE


class PolarHipError(RuntimeError):
    def __init__(self, status, message):
        super().__init__(f"polar_hip status {status}: {message}")
        self.status = status


class DeviceInfo(C.Structure):
    _fields_ = [
        ("name", C.c_char * 256),
        ("arch", C.c_char * 64),
        ("ordinal", C.c_int),
        ("compute_units", C.c_int),
        ("clock_khz", C.c_int),
        ("memory_clock_khz", C.c_int),
        ("memory_bus_bits", C.c_int),
        ("lds_bytes_per_block", C.c_int),
        ("l2_bytes", C.c_int),
        ("pci_bus_id", C.c_int),
        ("hbm_bytes", C.c_uint64),
    ]


class PoolStats(C.Structure):
    _fields_ = [
        ("bytes_in_use", C.c_uint64),
        ("bytes_cached", C.c_uint64),
        ("device_allocs", C.c_uint64),
        ("pool_hits", C.c_uint64),
    ]


_vp = C.c_void_p
_u64 = C.c_uint64
_f = C.c_float
_i = C.c_int

# name -> (restype, argtypes); one entry per declaration in include/polar_hip.h
SIGNATURES = {
    "polar_hip_last_error": (C.c_char_p, []),
    "polar_hip_version": (C.c_char_p, []),
    "polar_hip_device_count": (_i, [C.POINTER(_i)]),
    "polar_hip_device_open": (_i, [_i, C.POINTER(_vp)]),
    "polar_hip_device_close": (_i, [_vp]),
    "polar_hip_device_get_info": (_i, [_vp, C.POINTER(DeviceInfo)]),
    "polar_hip_device_synchronize": (_i, [_vp]),
    "polar_hip_alloc": (_i, [_vp, _u64, C.POINTER(_vp)]),
    "polar_hip_free": (_i, [_vp, _vp]),
    "polar_hip_pool_trim": (_i, [_vp]),
    "polar_hip_pool_get_stats": (_i, [_vp, C.POINTER(PoolStats)]),
    "polar_hip_copy_to_device": (_i, [_vp, _vp, _vp, _u64]),
    "polar_hip_copy_to_host": (_i, [_vp, _vp, _vp, _u64]),
    "polar_hip_host_alloc": (_i, [_vp, _u64, C.POINTER(_vp)]),
    "polar_hip_host_free": (_i, [_vp]),
    "polar_hip_host_quiesce": (_i, [_vp]),
    "polar_hip_event_record": (_i, [_vp, C.POINTER(_vp)]),
    "polar_hip_event_synchronize": (_i, [_vp]),
    "polar_hip_event_query": (_i, [_vp, C.POINTER(_i)]),
    "polar_hip_stream_wait_event": (_i, [_vp, _vp]),
    "polar_hip_event_elapsed_ms": (_i, [_vp, _vp, C.POINTER(_f)]),
    "polar_hip_time_next_kernel": (_i, [_vp, C.POINTER(_vp), C.POINTER(_vp)]),
    "polar_hip_event_release": (_i, [_vp]),
    "polar_hip_fadd": (_i, [_vp, _vp, _f, _vp, _f, _vp, _u64]),
    "polar_hip_fmul": (_i, [_vp, _vp, _vp, _vp, _u64]),
    "polar_hip_fdivide": (_i, [_vp, _vp, _vp, _vp, _u64]),
    "polar_hip_fsigmoid": (_i, [_vp, _vp, _vp, _u64]),
    "polar_hip_flogloss": (_i, [_vp, _vp, _vp, _vp, _u64]),
    "polar_hip_fmulconcat": (_i, [_vp, _vp, _vp, _vp, _u64]),
    "polar_hip_fcopy": (_i, [_vp, _vp, _vp, _u64]),
    "polar_hip_ffill": (_i, [_vp, _f, _vp, _u64]),
    "polar_hip_ftranspose": (_i, [_vp, _vp, _vp, _u64, _u64]),
    "polar_hip_fmatmul": (_i, [_vp, _i, _i, _vp, _vp, _vp, _u64, _u64, _u64]),
    "polar_hip_fmatmul_plan": (_i, [_vp, _u64, _u64, _u64, C.POINTER(_i), C.POINTER(C.c_uint32),
                                    C.POINTER(C.c_uint32)]),
    "polar_hip_fmatmul_with_plan": (_i, [_vp, _i, _i, _vp, _vp, _vp, _u64, _u64, _u64, _i, C.c_uint32]),
    "polar_hip_module_load": (_i, [_vp, _vp, _u64, C.POINTER(_vp)]),
    "polar_hip_module_unload": (_i, [_vp, _vp]),
    "polar_hip_module_has_kernel": (_i, [_vp, C.c_char_p, C.POINTER(_i)]),
    "polar_hip_module_launch": (_i, [_vp, _vp, C.c_char_p, C.POINTER(C.c_uint32), C.POINTER(C.c_uint32),
                                     C.POINTER(_vp)]),
    "polar_hip_frelu": (_i, [_vp, _vp, _vp, _u64]),
    "polar_hip_fsoftmax": (_i, [_vp, _vp, _vp, _u64]),
    "polar_hip_fsoftmax_static": (_i, [_vp, _vp, _vp, _u64]),
    "polar_hip_fconv2d": (_i, [_vp, _vp, _vp, _vp, _u64, _u64, _u64, _u64]),
    "polar_hip_fpool": (_i, [_vp, _vp, _vp, _u64, _u64, _u64, _u64, _u64, _u64]),
    "polar_hip_fpool_plan": (_i, [_u64, _u64, _u64, _u64, _u64, _u64, _i, C.POINTER(C.c_int), C.POINTER(C.c_uint32),
                                  C.POINTER(C.c_uint32)]),
    "polar_hip_fmatmul_fsigmoid": (_i, [_vp, _i, _i, _vp, _vp, _vp, _u64, _u64, _u64]),
    "polar_hip_fmatmul_fadd_fsigmoid": (_i, [_vp, _i, _i, _vp, _vp, _f, _vp, _f, _vp, _u64, _u64, _u64]),
    "polar_hip_fsigmoid_flogloss": (_i, [_vp, _vp, _vp, _vp, _u64]),
}

_lib = None


def load_library(path=LIB_DEVICE):
    """Load libpolar_hip.so and bind every declared symbol.  Raises if the
    library or any symbol is missing."""
    global _lib
    if _lib is not None and path == LIB_DEVICE:
        return _lib
    if not os.path.exists(path):
        raise FileNotFoundError(
            f"{path} is not built; run __graft_entry__.build() (hipcc, gfx950)")
    lib = C.CDLL(path, mode=C.RTLD_GLOBAL)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is absent
        fn.restype = res
        fn.argtypes = args
    if path == LIB_DEVICE:
        _lib = lib
    return lib


def _check(lib, status):
    if status != 0:
        raise PolarHipError(status, lib.polar_hip_last_error().decode())


def fpool_plan(height, width, window, stride, input_aligned=True):
    """(kernel, band rows, LDS bytes) polar_hip_fpool would use: kernel 0 = taps
    from memory, 1 = non-overlapping square windows, 2 = window staged in LDS,
    3 = waves marching down strips (square windows of 4 and 5).  Needs no GPU."""
    lib = load_library()
    kernel, band, lds = _i(0), C.c_uint32(0), C.c_uint32(0)
    _check(lib, lib.polar_hip_fpool_plan(height, width, window[0], window[1], stride[0], stride[1],
                                         int(bool(input_aligned)), C.byref(kernel), C.byref(band), C.byref(lds)))
    return kernel.value, band.value, lds.value


def device_count():
    lib = load_library()
    n = _i(0)
    _check(lib, lib.polar_hip_device_count(C.byref(n)))
    return n.value


class Buffer:
    """A block of pool memory on one device holding `count` fp32 elements."""

    def __init__(self, dev, count, ptr, offset_bytes=0):
        self.dev = dev
        self.count = int(count)
        self._base = ptr
        self.ptr = ptr + offset_bytes
        self.nbytes = self.count * 4

    def free(self):
        if self._base is not None:
            self.dev._free(self._base)
            self._base = None

    def upload(self, arr):
        arr = np.ascontiguousarray(arr, dtype=np.float32)
        assert arr.size == self.count, (arr.size, self.count)
        self.dev.copy_to_device(self.ptr, arr.ctypes.data, self.nbytes)
        return self

    def download(self, shape=None):
        out = np.empty(self.count, dtype=np.float32)
        self.dev.copy_to_host(out.ctypes.data, self.ptr, self.nbytes)
        return out if shape is None else out.reshape(shape)


class Event:
    def __init__(self, dev, handle):
        self.dev = dev
        self.handle = handle

    def synchronize(self):
        _check(self.dev.lib, self.dev.lib.polar_hip_event_synchronize(self.handle))

    def done(self):
        d = _i(0)
        _check(self.dev.lib, self.dev.lib.polar_hip_event_query(self.handle, C.byref(d)))
        return bool(d.value)

    def elapsed_ms(self, later):
        ms = _f(0)
        _check(self.dev.lib, self.dev.lib.polar_hip_event_elapsed_ms(
            self.handle, later.handle, C.byref(ms)))
        return ms.value

    def release(self):
        _check(self.dev.lib, self.dev.lib.polar_hip_event_release(self.handle))
        self.handle = None


class Device:
    """One opened GPU (stream + memory pool)."""

    def __init__(self, ordinal=0):
        self.lib = load_library()
        h = _vp()
        _check(self.lib, self.lib.polar_hip_device_open(ordinal, C.byref(h)))
        self.handle = h

    # -- lifetime -----------------------------------------------------------
    def close(self):
        if self.handle is not None:
            _check(self.lib, self.lib.polar_hip_device_close(self.handle))
            self.handle = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def info(self):
        inf = DeviceInfo()
        _check(self.lib, self.lib.polar_hip_device_get_info(self.handle, C.byref(inf)))
        return inf

    def synchronize(self):
        _check(self.lib, self.lib.polar_hip_device_synchronize(self.handle))

    # -- memory -------------------------------------------------------------
    def alloc_bytes(self, nbytes):
        p = _vp()
        _check(self.lib, self.lib.polar_hip_alloc(self.handle, nbytes, C.byref(p)))
        return p.value

    def _free(self, ptr):
        _check(self.lib, self.lib.polar_hip_free(self.handle, ptr))

    def empty(self, count, misalign_floats=0):
        """fp32 buffer of `count` elements; `misalign_floats` shifts the
        start by that many elements past the 256-byte aligned block."""
        ptr = self.alloc_bytes((int(count) + misalign_floats) * 4)
        return Buffer(self, count, ptr, misalign_floats * 4)

    def array(self, arr, misalign_floats=0):
        arr = np.ascontiguousarray(arr, dtype=np.float32)
        return self.empty(arr.size, misalign_floats).upload(arr)

    def copy_to_device(self, dst, src_host, nbytes):
        _check(self.lib, self.lib.polar_hip_copy_to_device(self.handle, dst, src_host, nbytes))

    def copy_to_host(self, dst_host, src, nbytes):
        _check(self.lib, self.lib.polar_hip_copy_to_host(self.handle, dst_host, src, nbytes))

    def host_alloc(self, nbytes):
        """Pinned host memory that the copy calls move to and from directly."""
        p = _vp()
        _check(self.lib, self.lib.polar_hip_host_alloc(self.handle, nbytes, C.byref(p)))
        return p.value

    def host_free(self, ptr):
        _check(self.lib, self.lib.polar_hip_host_free(ptr))

    def host_quiesce(self, ptr):
        _check(self.lib, self.lib.polar_hip_host_quiesce(ptr))

    def pool_stats(self):
        st = PoolStats()
        _check(self.lib, self.lib.polar_hip_pool_get_stats(self.handle, C.byref(st)))
        return st

    def pool_trim(self):
        _check(self.lib, self.lib.polar_hip_pool_trim(self.handle))

    # -- events -------------------------------------------------------------
    def record(self):
        h = _vp()
        _check(self.lib, self.lib.polar_hip_event_record(self.handle, C.byref(h)))
        return Event(self, h)

    def time_next_kernel(self):
        """(start, stop) events that take the next kernel's own begin and end."""
        s, e = _vp(), _vp()
        _check(self.lib, self.lib.polar_hip_time_next_kernel(self.handle, C.byref(s), C.byref(e)))
        return Event(self, s), Event(self, e)

    def wait_event(self, evt):
        _check(self.lib, self.lib.polar_hip_stream_wait_event(self.handle, evt.handle))

    # -- builtin operations (asynchronous) ------------------------------------
    def fadd(self, a, scale_a, b, scale_b, c, n=None):
        n = c.count if n is None else n
        _check(self.lib, self.lib.polar_hip_fadd(self.handle, a.ptr, scale_a, b.ptr, scale_b, c.ptr, n))

    def fmul(self, a, b, c, n=None):
        n = c.count if n is None else n
        _check(self.lib, self.lib.polar_hip_fmul(self.handle, a.ptr, b.ptr, c.ptr, n))

    def fdivide(self, num, den, out, n=None):
        n = out.count if n is None else n
        _check(self.lib, self.lib.polar_hip_fdivide(self.handle, num.ptr, den.ptr, out.ptr, n))

    def fsigmoid(self, x, out, n=None):
        n = out.count if n is None else n
        _check(self.lib, self.lib.polar_hip_fsigmoid(self.handle, x.ptr, out.ptr, n))

    def flogloss(self, pred, truth, out, n=None):
        n = out.count if n is None else n
        _check(self.lib, self.lib.polar_hip_flogloss(self.handle, pred.ptr, truth.ptr, out.ptr, n))

    def fmulconcat(self, grad, local, out, n=None):
        n = out.count if n is None else n
        _check(self.lib, self.lib.polar_hip_fmulconcat(self.handle, grad.ptr, local.ptr, out.ptr, n))

    def fcopy(self, src, dst, n=None):
        n = dst.count if n is None else n
        _check(self.lib, self.lib.polar_hip_fcopy(self.handle, src.ptr, dst.ptr, n))

    def ffill(self, pattern, out, n=None):
        n = out.count if n is None else n
        _check(self.lib, self.lib.polar_hip_ffill(self.handle, pattern, out.ptr, n))

    def ftranspose(self, src, dst, rows, cols):
        _check(self.lib, self.lib.polar_hip_ftranspose(self.handle, src.ptr, dst.ptr, rows, cols))

    def frelu(self, x, out, n=None):
        _check(self.lib, self.lib.polar_hip_frelu(self.handle, x.ptr, out.ptr, out.count if n is None else n))

    def fsoftmax(self, x, out, n=None):
        _check(self.lib, self.lib.polar_hip_fsoftmax(self.handle, x.ptr, out.ptr, out.count if n is None else n))

    def fsoftmax_static(self, x, out, n=None):
        _check(self.lib, self.lib.polar_hip_fsoftmax_static(self.handle, x.ptr, out.ptr, out.count if n is None else n))

    def fconv2d(self, x, kernel, out, height, width, kernel_height, kernel_width):
        _check(self.lib, self.lib.polar_hip_fconv2d(self.handle, x.ptr, kernel.ptr, out.ptr, height, width,
                                                    kernel_height, kernel_width))

    def fpool(self, x, out, height, width, window, stride):
        _check(self.lib, self.lib.polar_hip_fpool(self.handle, x.ptr, out.ptr, height, width,
                                                  window[0], window[1], stride[0], stride[1]))

    def fmatmul_fsigmoid(self, trans_a, trans_b, a, b, out, m, n, k):
        _check(self.lib, self.lib.polar_hip_fmatmul_fsigmoid(self.handle, int(trans_a), int(trans_b), a.ptr, b.ptr,
                                                             out.ptr, m, n, k))

    def fmatmul_fadd_fsigmoid(self, trans_a, trans_b, a, b, scale_product, bias, scale_bias, out, m, n, k):
        _check(self.lib, self.lib.polar_hip_fmatmul_fadd_fsigmoid(self.handle, int(trans_a), int(trans_b), a.ptr,
                                                                  b.ptr, scale_product, bias.ptr, scale_bias,
                                                                  out.ptr, m, n, k))

    def fsigmoid_flogloss(self, x, truth, out, n=None):
        _check(self.lib, self.lib.polar_hip_fsigmoid_flogloss(self.handle, x.ptr, truth.ptr, out.ptr,
                                                              out.count if n is None else n))

    def fmatmul_plan(self, m, n, k):
        """(tile configuration or -1, splits, (tile M, tile N, tile K)) the planner picks."""
        cfg, splits, tile = _i(0), C.c_uint32(0), (C.c_uint32 * 3)()
        _check(self.lib, self.lib.polar_hip_fmatmul_plan(self.handle, m, n, k, C.byref(cfg), C.byref(splits), tile))
        return cfg.value, splits.value, tuple(tile)

    def fmatmul_with_plan(self, trans_a, trans_b, a, b, c, m, n, k, tile_config, splits):
        _check(self.lib, self.lib.polar_hip_fmatmul_with_plan(
            self.handle, int(bool(trans_a)), int(bool(trans_b)), a.ptr, b.ptr, c.ptr, m, n, k, tile_config, splits))

    def fmatmul(self, trans_a, trans_b, a, b, c, m, n, k):
        _check(self.lib, self.lib.polar_hip_fmatmul(
            self.handle, int(bool(trans_a)), int(bool(trans_b)), a.ptr, b.ptr, c.ptr, m, n, k))
