"""Loader of oracle/_ref/libabi_probe.so: the caller side of the plugin
interface compiled from the reference's own headers (built by `make -C oracle
ref` where the reference tree is present; the built file travels with the
repository to machines that do not have the tree)."""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(os.path.dirname(HERE), "oracle", "_ref", "libabi_probe.so")

# sizeof/offsetof of TensorInfo, ArgDesc, LaunchCommand, MemoryRecord on LP64
EXPECTED_LAYOUT = [32, 0, 8, 16, 24, 24, 8, 16, 32, 8, 24, 16]


def available():
    return os.path.exists(LIB)


def load():
    # The support library inside the probe leaves three member functions of the
    # framework's TensorInternal undefined (in a framework build they come from
    # polar_core); the mini-executor's binary defines them for its own tensor
    # objects, so it is loaded first, with its symbols visible to the probe.
    from polarai_framework_amd import LIB_HARNESS
    C.CDLL(LIB_HARNESS, mode=C.RTLD_GLOBAL)
    lib = C.CDLL(LIB)
    lib.ref_struct_layout.argtypes = [C.POINTER(C.c_uint64)]
    lib.ref_context_device_count.argtypes = [C.c_void_p]
    lib.ref_context_device.argtypes = [C.c_void_p, C.c_int]
    lib.ref_context_device.restype = C.c_void_p
    lib.ref_device_info.argtypes = [C.c_void_p, C.c_char_p, C.c_size_t, C.POINTER(C.c_int)]
    lib.ref_allocator_and_copy.argtypes = [C.c_void_p, C.c_size_t, C.c_void_p, C.c_void_p, C.c_size_t]
    lib.ref_launch_fadd.argtypes = [C.c_void_p, C.c_void_p, C.c_uint64, C.c_uint64, C.c_uint64,
                                    C.c_uint64, C.c_float, C.c_float]
    lib.ref_graph_handle_layout.argtypes = [C.POINTER(C.c_uint64)]
    lib.ref_support_evaluate.argtypes = [C.c_void_p, C.c_uint64, C.c_void_p, C.c_void_p,
                                         C.c_float, C.c_float, C.c_void_p, C.c_void_p]
    return lib


def graph_handle_layouts(lib):
    """(layout per the reference's GraphHandle.hpp, layout the support library was built with)"""
    out = (C.c_uint64 * 10)()
    lib.ref_graph_handle_layout(out)
    return list(out[:5]), list(out[5:])


def support_evaluate(lib, device_ptr, a, b, scale_a, scale_b):
    """Two input nodes, one fadd node, barrier and host reads through the support
    library's ath_* on a reference-declared GraphHandle.  Returns (rc, sum, a_back)."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    b = np.ascontiguousarray(b, dtype=np.float32)
    total = np.full_like(a, np.nan)
    a_back = np.full_like(a, np.nan)
    rc = lib.ref_support_evaluate(device_ptr, a.size, a.ctypes.data, b.ctypes.data, scale_a, scale_b,
                                  total.ctypes.data, a_back.ctypes.data)
    return rc, total, a_back


def struct_layout(lib):
    out = (C.c_uint64 * 12)()
    lib.ref_struct_layout(out)
    return list(out)


def device_info(lib, device_ptr):
    name = C.create_string_buffer(512)
    out = (C.c_int * 8)()
    lib.ref_device_info(device_ptr, name, 512, out)
    keys = ("provider", "kind", "hasAllocator", "partitionSupported", "partitions", "eq", "ne", "hash_ok")
    return name.value.decode(), dict(zip(keys, out))


def allocator_and_copy(lib, device_ptr, vaddr, src):
    src = np.ascontiguousarray(src, dtype=np.float32)
    dst = np.zeros_like(src)
    rc = lib.ref_allocator_and_copy(device_ptr, vaddr, src.ctypes.data, dst.ctypes.data, src.size)
    return rc, dst
