"""ctypes binding of include/polar_harness.h (the mini-executor).

`Harness(plugin=LIB_PLUGIN)` opens the HIP runtime plugin through
initContext(); `Harness(plugin=None)` uses the built-in CPU mock device.  A
program is built from input nodes and compute nodes (one builtin each), split
into clusters, and run with the call sequence of the framework's compiled
graph code, so every kernel is reached through Device::launch(LaunchCommand).
"""
import ctypes as C
import os

import numpy as np

from . import LIB_HARNESS, LIB_PLUGIN

READ, READ_WRITE = 0, 1
HOST = -1


class Arg(C.Structure):
    _fields_ = [("kind", C.c_int), ("vaddr", C.c_uint64), ("scalar", C.c_float)]


class Counters(C.Structure):
    _fields_ = [(n, C.c_uint64) for n in (
        "launches", "copies_to_device", "bytes_to_device", "copies_to_host",
        "bytes_to_host", "events_waited", "deferred_releases", "device_name_calls",
        "ns_input_nodes", "ns_allocate_and_lock", "ns_launch", "ns_release", "ns_barrier")]


_vp, _u64, _i = C.c_void_p, C.c_uint64, C.c_int
SIGNATURES = {
    "polar_harness_open": (_i, [C.c_char_p, _i, C.POINTER(_vp)]),
    "polar_harness_close": (None, [_vp]),
    "polar_harness_use_plugin_host_memory": (_i, [_vp]),
    "polar_harness_device_count": (_i, [_vp]),
    "polar_harness_device_name": (C.c_char_p, [_vp]),
    "polar_harness_device_provider": (_i, [_vp]),
    "polar_harness_device_kind": (_i, [_vp]),
    "polar_harness_tensor": (_u64, [_vp, _u64, C.POINTER(_u64)]),
    "polar_harness_input": (_i, [_vp, _u64, _vp]),
    "polar_harness_node": (_i, [_vp, C.c_char_p, C.c_uint32, C.POINTER(Arg), C.c_uint32]),
    "polar_harness_jit_node": (_i, [_vp, C.c_char_p, C.c_uint32, C.POINTER(Arg), C.c_uint32]),
    "polar_harness_select_binary": (_i, [_vp, _i, C.c_char_p, C.c_char_p, _u64, C.c_uint32,
                                         C.POINTER(C.c_char_p), C.POINTER(_u64)]),
    "polar_harness_end_cluster": (_i, [_vp]),
    "polar_harness_clear_program": (_i, [_vp]),
    "polar_harness_run": (_i, [_vp]),
    "polar_harness_read": (_i, [_vp, _u64, _vp, _u64]),
    "polar_harness_allocate": (_i, [_vp, _u64, _i]),
    "polar_harness_lock": (_i, [_vp, _u64, _i, _i]),
    "polar_harness_release": (_i, [_vp, _u64, _i]),
    "polar_harness_host_write": (_i, [_vp, _u64, _vp, _u64]),
    "polar_harness_read_through_tensor_object": (_i, [_vp, _u64, _vp, _u64]),
    "polar_harness_raw_device": (_vp, [_vp]),
    "polar_harness_raw_allocator": (_vp, [_vp]),
    "polar_harness_raw_context": (_vp, [_vp]),
    "polar_harness_get_counters": (_i, [_vp, C.POINTER(Counters)]),
    "polar_harness_set_device_byte_limit": (_i, [_vp, _u64]),
}

_lib = None


def load_library():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_HARNESS):
            raise FileNotFoundError(f"{LIB_HARNESS} is not built; run __graft_entry__.build()")
        lib = C.CDLL(LIB_HARNESS)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


class Tensor:
    def __init__(self, vaddr, shape):
        self.vaddr = vaddr
        self.shape = tuple(int(s) for s in shape)
        self.count = int(np.prod(self.shape, dtype=np.int64)) if self.shape else 1


class Harness:
    def __init__(self, plugin=LIB_PLUGIN, device_index=0, plugin_host_memory=False):
        """plugin_host_memory: keep the RAM side of every tensor in the plugin's pinned host
        memory (polar_harness_use_plugin_host_memory); the default is the heap, as in the
        framework's own RAM layer."""
        self.lib = load_library()
        if plugin is not None and not os.path.exists(plugin):
            raise FileNotFoundError(f"{plugin} is not built; run __graft_entry__.build()")
        h = _vp()
        rc = self.lib.polar_harness_open(None if plugin is None else plugin.encode(),
                                         device_index, C.byref(h))
        if rc != 0:
            raise RuntimeError(f"cannot open runtime plugin {plugin} (device {device_index})")
        self.h = h
        self._keep = []
        if plugin_host_memory and self.lib.polar_harness_use_plugin_host_memory(h) != 0:
            self.close()
            raise RuntimeError(f"{plugin} does not export polarHostMemoryAllocate/Release/Quiesce")

    def close(self):
        if self.h is not None:
            self.lib.polar_harness_close(self.h)
            self.h = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def _ok(self, rc, what):
        if rc != 0:
            raise ValueError(f"polar_harness: {what} rejected its arguments")

    # -- device under test --------------------------------------------------
    @property
    def device_count(self):
        return self.lib.polar_harness_device_count(self.h)

    @property
    def device_name(self):
        return self.lib.polar_harness_device_name(self.h).decode()

    @property
    def device_provider(self):
        return self.lib.polar_harness_device_provider(self.h)

    @property
    def device_kind(self):
        return self.lib.polar_harness_device_kind(self.h)

    # -- program ------------------------------------------------------------
    def tensor(self, *shape):
        arr = (_u64 * len(shape))(*shape)
        v = self.lib.polar_harness_tensor(self.h, len(shape), arr)
        if v == 0:
            raise ValueError("polar_harness_tensor failed")
        return Tensor(v, shape)

    def input(self, data):
        """New tensor shaped like `data`, filled by an input node."""
        data = np.ascontiguousarray(data, dtype=np.float32)
        t = self.tensor(*data.shape)
        self._ok(self.lib.polar_harness_input(self.h, t.vaddr, data.ctypes.data), "input")
        return t

    def input_into(self, t, data):
        """Input node that fills the existing tensor `t`."""
        data = np.ascontiguousarray(data, dtype=np.float32)
        assert data.size == t.count
        self._ok(self.lib.polar_harness_input(self.h, t.vaddr, data.ctypes.data), "input")
        return t

    def holder(self, t):
        """Input node with a loader that loads nothing: it only holds `t`."""
        self._ok(self.lib.polar_harness_input(self.h, t.vaddr, None), "holder")
        return t

    def _args(self, args):
        arr = (Arg * len(args))()
        for i, a in enumerate(args):
            if isinstance(a, Tensor):
                arr[i] = Arg(0, a.vaddr, 0.0)
            elif isinstance(a, (int, np.integer)) and not isinstance(a, bool):
                arr[i] = Arg(2, int(a), 0.0)     # integer attribute, passed as a 64-bit scalar
            else:
                arr[i] = Arg(1, 0, float(a))
        return arr

    def node(self, kernel, args, result_index):
        arr = self._args(args)
        self._ok(self.lib.polar_harness_node(self.h, kernel.encode(), len(args), arr, result_index),
                 f"node {kernel}")

    def jit_node(self, jit_kernel_name, args, result_index):
        """A node whose kernel comes from the selected program (no native kernel name)."""
        arr = self._args(args)
        self._ok(self.lib.polar_harness_jit_node(self.h, jit_kernel_name.encode(), len(args), arr, result_index),
                 f"jit node {jit_kernel_name}")

    def select_binary(self, image, kernels, program_type=2, target="gfx950"):
        """kernels: {name: (globalX, globalY, globalZ, localX, localY, localZ)}"""
        names = (C.c_char_p * len(kernels))(*[k.encode() for k in kernels])
        geo = (C.c_uint64 * (6 * len(kernels)))(*[int(v) for g in kernels.values() for v in g])
        self._ok(self.lib.polar_harness_select_binary(self.h, program_type, target.encode(), image, len(image),
                                                      len(kernels), names, geo), "select_binary")

    def end_cluster(self):
        self._ok(self.lib.polar_harness_end_cluster(self.h), "end_cluster")

    def clear_program(self):
        self._ok(self.lib.polar_harness_clear_program(self.h), "clear_program")

    def run(self):
        self._ok(self.lib.polar_harness_run(self.h), "run")

    def read(self, t):
        out = np.empty(t.count, dtype=np.float32)
        self._ok(self.lib.polar_harness_read(self.h, t.vaddr, out.ctypes.data, t.count), "read")
        return out.reshape(t.shape)

    # builtin operations with the operand order of the launch lowering
    def fadd(self, a, sa, b, sb, out=None):
        out = out or self.tensor(*a.shape)
        self.node("fadd", [a, float(sa), b, float(sb), out], 4)
        return out

    def _binary(self, name, x, y, out=None, shape=None):
        out = out or self.tensor(*(shape or y.shape))
        self.node(name, [x, y, out], 2)
        return out

    def fmul(self, a, b, out=None):
        return self._binary("fmul", a, b, out)

    def fdivide(self, num, den, out=None):
        return self._binary("fdivide", num, den, out)

    def flogloss(self, pred, truth, out=None):
        return self._binary("flogloss", pred, truth, out)

    def fmulconcat(self, grad, local, out=None):
        return self._binary("fmulconcat", grad, local, out)

    def fsigmoid(self, x, out=None):
        out = out or self.tensor(*x.shape)
        self.node("fsigmoid", [x, out], 1)
        return out

    def fcopy(self, src, out=None):
        out = out or self.tensor(*src.shape)
        self.node("fcopy", [src, out], 1)
        return out

    def ffill(self, pattern, out):
        self.node("ffill", [float(pattern), out], 1)
        return out

    def ftranspose(self, a, out=None):
        out = out or self.tensor(a.shape[1], a.shape[0])
        self.node("ftranspose", [a, out], 1)
        return out

    # extended (fused) builtins
    def fsigmoid_flogloss(self, x, truth, out=None):
        return self._binary("fsigmoid_flogloss", x, truth, out)

    def fmatmul_fsigmoid(self, ta, tb, a, b, out=None):
        m = a.shape[1] if ta else a.shape[0]
        n = b.shape[0] if tb else b.shape[1]
        out = out or self.tensor(m, n)
        self.node(f"fmatmul_{'t' if ta else 'f'}_{'t' if tb else 'f'}_fsigmoid", [a, b, out], 2)
        return out

    def fmatmul_fadd_fsigmoid(self, ta, tb, a, b, scale_product, bias, scale_bias, out=None):
        out = out or self.tensor(*bias.shape)
        self.node(f"fmatmul_{'t' if ta else 'f'}_{'t' if tb else 'f'}_fadd_fsigmoid",
                  [a, b, float(scale_product), bias, float(scale_bias), out], 5)
        return out

    def frelu(self, x, out=None):
        out = out or self.tensor(*x.shape)
        self.node("frelu", [x, out], 1)
        return out

    def fsoftmax(self, x, out=None):
        out = out or self.tensor(*x.shape)
        self.node("fsoftmax", [x, out], 1)
        return out

    def fconv2d(self, x, kernel, out=None):
        out = out or self.tensor(x.shape[0] - kernel.shape[0] + 1, x.shape[1] - kernel.shape[1] + 1)
        self.node("fconv2d", [x, kernel, out], 2)
        return out

    def fpool(self, x, window, stride, out=None):
        out = out or self.tensor((x.shape[0] - window[0]) // stride[0] + 1,
                                 (x.shape[1] - window[1]) // stride[1] + 1)
        self.node("fpool", [x, out, int(window[0]), int(window[1]), int(stride[0]), int(stride[1])], 1)
        return out

    def fmatmul(self, ta, tb, a, b, out=None):
        m = a.shape[1] if ta else a.shape[0]
        n = b.shape[0] if tb else b.shape[1]
        out = out or self.tensor(m, n)
        self.node(f"fmatmul_{'t' if ta else 'f'}_{'t' if tb else 'f'}", [a, b, out], 2)
        return out

    # -- allocator access for protocol tests --------------------------------
    def allocate(self, t, device=0):
        self._ok(self.lib.polar_harness_allocate(self.h, t.vaddr, device), "allocate")

    def lock(self, t, device, lock_type):
        self._ok(self.lib.polar_harness_lock(self.h, t.vaddr, device, lock_type), "lock")

    def release(self, t, device):
        self._ok(self.lib.polar_harness_release(self.h, t.vaddr, device), "release")

    def host_write(self, t, data):
        data = np.ascontiguousarray(data, dtype=np.float32)
        self._ok(self.lib.polar_harness_host_write(self.h, t.vaddr, data.ctypes.data, data.size), "host_write")

    def read_through_tensor_object(self, t):
        """Read `t` the way the framework's OutputNodeAccessor does: through the
        allocator's tensor-object overloads."""
        out = np.empty(t.shape, dtype=np.float32)
        self._ok(self.lib.polar_harness_read_through_tensor_object(self.h, t.vaddr, out.ctypes.data, out.size),
                 "read_through_tensor_object")
        return out

    def raw_device(self):
        return self.lib.polar_harness_raw_device(self.h)

    def raw_allocator(self):
        return self.lib.polar_harness_raw_allocator(self.h)

    def raw_context(self):
        return self.lib.polar_harness_raw_context(self.h)

    def counters(self):
        c = Counters()
        self._ok(self.lib.polar_harness_get_counters(self.h, C.byref(c)), "get_counters")
        return c

    def set_device_byte_limit(self, nbytes):
        self._ok(self.lib.polar_harness_set_device_byte_limit(self.h, nbytes), "set_device_byte_limit")
