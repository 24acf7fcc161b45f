"""CPU tests of the host side: the libraries load and export what the headers
declare, the coherence protocol and call sequence of the mini-executor (on its
mock device), and the failure conventions.  No compute is called: there is no
GPU here."""
import ctypes as C
import os
import re
import subprocess
import sys

import numpy as np
import pytest

from polarai_framework_amd import LIB_DEVICE, LIB_HARNESS, LIB_PLUGIN, REPO_ROOT, capi, harness


def _declared(header, prefix):
    text = open(os.path.join(REPO_ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(" + prefix + r"\w+)\s*\(", text)))


def test_device_library_exports_every_declared_symbol():
    names = _declared("polar_hip.h", "polar_hip_")
    assert len(names) >= 29
    lib = C.CDLL(LIB_DEVICE)
    for n in names:
        assert hasattr(lib, n), n
    assert sorted(capi.SIGNATURES) == names  # the binding covers the header exactly


def test_pool_plan_stays_off_the_staged_kernel_when_the_stride_overflows_32_bits():
    """The staged pooling kernel's window pitch is 286 x stride1 + window1 floats:
    for strides of tens of millions that product wraps in 32 bits and could pass
    for a pitch that fits LDS.  The planner works in 64 bits."""
    staged = capi.fpool_plan(8192, 8192, (3, 3), (2, 2))
    assert staged[0] == 2 and staged[1] >= 1 and 0 < staged[2] <= 24 * 1024
    assert capi.fpool_plan(8192, 8192, (2, 2), (2, 2))[0] == 1
    assert capi.fpool_plan(8192, 8192, (2, 2), (2, 2), input_aligned=False)[0] == 2
    wide = (1 << 31) - 1
    for stride1 in (15_017_369, 15_017_370, 15_017_372, 30_034_737, 2**24, 2**26 + 5, wide // 2):
        # 286 * stride1 + 3 is 241, 527, 1099 and 193 modulo 2^32 for the first four
        kernel, band, lds = capi.fpool_plan(4, wide, (3, 3), (1, stride1))
        assert (kernel, band, lds) == (0, 0, 0), (stride1, kernel, band, lds)
    assert capi.fpool_plan(64, 100000, (5, 5), (2, 4))[0] == 2      # five input rows of 1152 floats fit 24 KiB
    assert capi.fpool_plan(64, 100000, (5, 5), (2, 5))[0] == 0      # of 1436 floats: only four do


def test_pool_plan_marches_over_square_windows_of_four_and_five():
    """Kernel 3 takes overlapping square windows of 4 and 5 at stride 1 or 2 when the
    image rows start on 16 bytes; everything else stays where it was."""
    for window, stride in (((4, 4), (1, 1)), ((4, 4), (2, 2)), ((5, 5), (1, 1)), ((5, 5), (2, 2))):
        kernel, band, lds = capi.fpool_plan(8192, 8192, window, stride)
        assert kernel == 3 and lds == 0 and 8 <= band <= 8192, (window, stride, kernel, band, lds)
        assert capi.fpool_plan(8192, 8190, window, stride)[0] == 2            # rows off 16 bytes
        assert capi.fpool_plan(8192, 8192, window, stride, input_aligned=False)[0] == 2
    assert capi.fpool_plan(8192, 8192, (4, 4), (4, 4))[0] == 1
    assert capi.fpool_plan(8192, 8192, (5, 5), (3, 3))[0] == 2
    assert capi.fpool_plan(8192, 8192, (5, 4), (1, 1))[0] == 2
    assert capi.fpool_plan(8192, 8192, (3, 3), (1, 1))[0] == 2
    # short images: one band of all the output rows
    assert capi.fpool_plan(9, 8, (5, 5), (1, 1))[:2] == (3, 5)


def test_probe_library_exports_what_the_benchmark_calls():
    import bench
    lib = C.CDLL(bench.LIB_PROBES)
    for name in ("polar_probe_streams", "polar_probe_read", "polar_probe_transpose_pattern", "polar_probe_panels"):
        assert hasattr(lib, name), name


def test_harness_library_exports_every_declared_symbol():
    names = _declared("polar_harness.h", "polar_harness_")
    lib = C.CDLL(LIB_HARNESS)
    for n in names:
        assert hasattr(lib, n), n
    assert sorted(harness.SIGNATURES) == names
    for n in ("ath_allocate", "ath_release", "ath_lock", "ath_device_select", "ath_barrier",
              "ath_launch", "ath_load"):
        assert hasattr(lib, n), n


def test_plugin_exports_driver_entry_points():
    # what the runtime driver resolves: src/backend/generic/runtime/driver/RuntimeDriver.cpp:28-31
    assert os.path.basename(LIB_PLUGIN) == "libpolar_rt_hip.so"
    lib = C.CDLL(LIB_PLUGIN, mode=os.RTLD_LAZY | os.RTLD_LOCAL)
    assert hasattr(lib, "initContext") and hasattr(lib, "closeContext")


def test_plugin_exports_the_optional_host_memory_symbols():
    lib = C.CDLL(LIB_PLUGIN, mode=os.RTLD_LAZY | os.RTLD_LOCAL)
    for name in ("polarHostMemoryAllocate", "polarHostMemoryRelease", "polarHostMemoryQuiesce"):
        assert hasattr(lib, name), name
    # no context has been created in this process: there is no device to pin memory through
    lib.polarHostMemoryAllocate.restype = C.c_void_p
    lib.polarHostMemoryAllocate.argtypes = [C.c_size_t]
    assert lib.polarHostMemoryAllocate(4096) is None


def test_mock_device_has_no_plugin_host_memory():
    with pytest.raises(RuntimeError):
        harness.Harness(plugin=None, plugin_host_memory=True)


def test_device_library_without_gpu_reports_no_device():
    if capi.device_count() != 0:
        pytest.skip("a GPU is present")
    with pytest.raises(capi.PolarHipError) as e:
        capi.Device(0)
    assert e.value.status == 2


def test_null_arguments_are_rejected_not_dereferenced():
    lib = capi.load_library()
    assert lib.polar_hip_fadd(None, None, 1.0, None, 1.0, None, 4) == 1
    assert lib.polar_hip_fmatmul(None, 0, 0, None, None, None, 1, 1, 1) == 1
    assert b"dev is null" in lib.polar_hip_last_error()


def _c(h):
    c = h.counters()
    return {n: getattr(c, n) for n, _ in c._fields_}


def test_virtual_addresses_start_at_one_and_pack_by_bytes():
    # src/core/context/internal/ContextInternal.cpp:24,43-48; e.g. 1, 17, 33 for 2x2 f32
    with harness.Harness(plugin=None) as h:
        assert [h.tensor(2, 2).vaddr for _ in range(3)] == [1, 17, 33]


def test_call_sequence_and_coherence_on_mock():
    with harness.Harness(plugin=None) as h:
        assert h.device_name == "mock"
        a = h.input(np.arange(8, dtype=np.float32))
        b = h.input(np.ones(8, dtype=np.float32))
        h.end_cluster()
        c = h.fadd(a, 1.0, b, 1.0)
        d = h.fmul(c, a)        # c is already on the device: no copy; a already uploaded
        h.end_cluster()
        h.run()
        k = _c(h)
        assert k["launches"] == 2
        assert k["copies_to_device"] == 2 and k["bytes_to_device"] == 64  # a and b once each
        assert k["copies_to_host"] == 0                                  # nothing read yet
        assert k["events_waited"] == 2
        # per node: releases of the READ args and of the result ride on the event
        assert k["deferred_releases"] == 3 + 3
        h.read(d)
        h.read(d)                # RAM now holds the newest version: no second copy
        k = _c(h)
        assert k["copies_to_host"] == 1
        # inputs were never written on the device: reading them needs no copy
        assert np.array_equal(h.read(a), np.arange(8, dtype=np.float32))
        assert _c(h)["copies_to_host"] == 1


def test_host_write_invalidates_device_copy():
    with harness.Harness(plugin=None) as h:
        t = h.tensor(4)
        h.host_write(t, [1, 2, 3, 4])
        h.lock(t, 0, harness.READ); h.release(t, 0)
        assert _c(h)["copies_to_device"] == 1
        h.lock(t, 0, harness.READ); h.release(t, 0)
        assert _c(h)["copies_to_device"] == 1      # still current
        h.host_write(t, [5, 6, 7, 8])
        h.lock(t, 0, harness.READ); h.release(t, 0)
        assert _c(h)["copies_to_device"] == 2      # stale after the host write
        h.lock(t, 0, harness.READ_WRITE); h.release(t, 0)
        assert np.array_equal(h.read(t), [5, 6, 7, 8])  # mock copies real bytes
        assert _c(h)["copies_to_host"] == 1


def test_results_are_readable_through_tensor_objects():
    # what the framework's OutputNodeAccessor does: lock(tensor, READ_WRITE), get(tensor),
    # release(tensor) (include/polarai/core/node/OutputNodeAccessor.hpp:21-31)
    with harness.Harness(plugin=None) as h:
        t = h.tensor(2, 3)
        h.host_write(t, [1, 2, 3, 4, 5, 6])
        h.lock(t, 0, harness.READ_WRITE); h.release(t, 0)   # the device now holds the newest version
        before = _c(h)["copies_to_host"]
        got = h.read_through_tensor_object(t)
        assert np.array_equal(got.ravel(), [1, 2, 3, 4, 5, 6])
        assert _c(h)["copies_to_host"] == before + 1          # pulled from the device by the host lock
        assert np.array_equal(h.read(t).ravel(), got.ravel())
        h.lock(t, 0, harness.READ_WRITE); h.release(t, 0)   # the lock was released again


def test_support_routines_do_no_string_work_after_registration():
    # upstream compares getDeviceName() with "host" on every ath_allocate / ath_lock /
    # ath_release (routines.cpp:29,40,55) and keys its tables by the name
    # (LayerAllocator.cpp:30,60); here a device is asked for its name when it is
    # registered and never again
    with harness.Harness(plugin=None) as h:
        a = h.input(np.arange(8, dtype=np.float32))
        b = h.input(np.ones(8, dtype=np.float32))
        h.end_cluster()
        c = h.fadd(a, 1.0, b, 1.0)
        h.fmul(c, a)
        h.end_cluster()
        h.run()
        first = _c(h)["device_name_calls"]
        for _ in range(3):
            h.run()
        h.read(c)
        assert _c(h)["device_name_calls"] == first
        assert _c(h)["launches"] == 8


def test_eviction_of_a_stale_device_copy_keeps_the_newer_host_data():
    with harness.Harness(plugin=None) as h:
        t, u = h.tensor(4), h.tensor(4)
        h.host_write(t, [1, 2, 3, 4])
        h.lock(t, 0, harness.READ); h.release(t, 0)          # device copy of version 2
        h.host_write(t, [5, 6, 7, 8])                        # RAM has version 3, device copy is stale
        h.host_write(u, [9, 9, 9, 9])
        h.set_device_byte_limit(16)                          # room for one of the two tensors
        h.lock(u, 0, harness.READ); h.release(u, 0)          # evicts t's stale device copy
        to_host = _c(h)["copies_to_host"]
        h.lock(t, 0, harness.READ_WRITE); h.release(t, 0)    # evicts u, uploads RAM's t
        assert np.array_equal(h.read(t), [5, 6, 7, 8])       # read back from the (mock) device
        assert _c(h)["copies_to_host"] == to_host + 1        # only the final read; no stale copy was saved
        assert np.array_equal(h.read(u), [9, 9, 9, 9])


def test_eviction_saves_the_only_copy_of_a_result():
    with harness.Harness(plugin=None) as h:
        t, u = h.tensor(4), h.tensor(4)
        h.host_write(t, [1, 2, 3, 4])
        h.lock(t, 0, harness.READ_WRITE); h.release(t, 0)    # newest version lives on the device only
        h.host_write(u, [9, 9, 9, 9])
        h.set_device_byte_limit(16)
        before = _c(h)["copies_to_host"]
        h.lock(u, 0, harness.READ); h.release(u, 0)          # evicts t: its device copy must be saved
        assert _c(h)["copies_to_host"] == before + 1
        assert np.array_equal(h.read(t), [1, 2, 3, 4])


def test_many_read_locks_are_allowed():
    with harness.Harness(plugin=None) as h:
        t = h.tensor(4)
        h.host_write(t, [1, 2, 3, 4])
        h.lock(t, 0, harness.READ)
        h.lock(t, 0, harness.READ)
        h.lock(t, harness.HOST, harness.READ)
        h.release(t, 0); h.release(t, 0); h.release(t, harness.HOST)
        h.lock(t, 0, harness.READ_WRITE)  # all released: allowed again
        h.release(t, 0)


def test_double_allocate_is_a_noop():
    with harness.Harness(plugin=None) as h:
        t = h.tensor(4)
        h.allocate(t, 0); h.allocate(t, 0); h.allocate(t, harness.HOST)


def test_usage_errors_return_minus_one():
    with harness.Harness(plugin=None) as h:
        t = h.tensor(4)
        with pytest.raises(ValueError):
            h.node("fadd", [t, 1.0, t, 1.0, 2.0], 4)   # result must be a tensor
        with pytest.raises(ValueError):
            h.node("fadd", [harness.Tensor(999, (4,)), 1.0, t, 1.0, t], 4)  # unknown tensor


def _dies(code):
    env = dict(os.environ, PYTHONPATH=REPO_ROOT)
    prog = ("import __graft_entry__ as e; e.load_package();"
            "from polarai_framework_amd import harness; import numpy as np;"
            "h = harness.Harness(plugin=None);" + code)
    return subprocess.run([sys.executable, "-c", prog], env=env, capture_output=True, text=True, timeout=60)


def test_read_write_lock_on_locked_tensor_is_fatal():
    # tests/unit/backend/generic/lib/allocators/LayerAllocator.cpp:99-102 (ASSERT_DEATH)
    r = _dies("t = h.tensor(4); h.host_write(t, [1,2,3,4]); h.lock(t, 0, 0); h.lock(t, 0, 1)")
    assert r.returncode == 4  # ATH_BAD_ACCESS
    assert "Attempt get READ_WRITE lock for tensor that is already locked" in r.stderr


def test_host_read_write_lock_on_locked_tensor_is_fatal():
    r = _dies("t = h.tensor(4); h.host_write(t, [1,2,3,4]); h.lock(t, 0, 0); h.lock(t, -1, 1)")
    assert r.returncode == 4
    assert "already locked" in r.stderr


def test_device_listing_tool_without_gpu():
    import subprocess
    from polarai_framework_amd import TOOL_LSPOLAR
    r = subprocess.run([TOOL_LSPOLAR], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0 and r.stdout.splitlines()[0] == "Total device count: 0"
    r = subprocess.run([TOOL_LSPOLAR, "/nonexistent/libpolar_rt_hip.so"], capture_output=True, text=True, timeout=60)
    assert r.returncode == 1 and "Failed to load" in r.stderr


def test_plugin_without_devices_is_reported():
    if capi.device_count() != 0:
        pytest.skip("a GPU is present")
    with pytest.raises(RuntimeError):
        harness.Harness(plugin=LIB_PLUGIN)
