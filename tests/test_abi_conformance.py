"""Interface conformance against the reference's own headers.

oracle/_ref/libabi_probe.so is compiled from the reference's Device / Context /
Event / AllocatorLayerBase / LaunchCommand / TensorInfo headers.  It is handed
objects built with this repository's restatement (include/polar_rt_abi.hpp) and
uses them through the reference's declarations: a different virtual order,
parameter type or struct layout would make these calls misbehave."""
import numpy as np
import pytest

import abi_probe
from polarai_framework_amd import LIB_PLUGIN, harness

needs_probe = pytest.mark.skipif(not abi_probe.available(),
                                 reason="oracle/_ref/libabi_probe.so not built (needs the reference tree)")


@needs_probe
def test_struct_layouts_match_the_reference_headers():
    assert abi_probe.struct_layout(abi_probe.load()) == abi_probe.EXPECTED_LAYOUT


def _exercise(h, expect_result):
    lib = abi_probe.load()
    dev = h.raw_device()
    name, info = abi_probe.device_info(lib, dev)
    assert name == h.device_name
    assert info["provider"] == h.device_provider and info["kind"] == h.device_kind
    assert info["hasAllocator"] == 1 and info["partitionSupported"] == 0 and info["partitions"] == 0
    assert info["eq"] == 1 and info["ne"] == 0 and info["hash_ok"] == 1
    src = np.arange(1000, dtype=np.float32) * 0.5
    rc, dst = abi_probe.allocator_and_copy(lib, dev, 1 << 40, src)
    assert rc == 0, f"allocator/copy step {rc}"
    assert np.array_equal(dst, src)
    # launch through the reference's Device::launch with reference-laid-out structs
    n = 1003
    a, b, c = h.tensor(n), h.tensor(n), h.tensor(n)
    av, bv = np.arange(n, dtype=np.float32), np.full(n, 2.0, dtype=np.float32)
    h.host_write(a, av); h.host_write(b, bv)
    h.allocate(c, 0)
    h.lock(c, 0, harness.READ_WRITE); h.lock(a, 0, harness.READ); h.lock(b, 0, harness.READ)
    rc = lib.ref_launch_fadd(dev, h.raw_allocator(), a.vaddr, b.vaddr, c.vaddr, n, 0.5, 3.0)
    assert rc == 0, f"launch/event step {rc}"
    for t in (a, b, c):
        h.release(t, 0)
    if expect_result:
        assert np.array_equal(h.read(c), (np.float32(0.5) * av + np.float32(3.0) * bv))


@needs_probe
def test_graph_handle_layout_matches_the_reference_header():
    reference, ours = abi_probe.graph_handle_layouts(abi_probe.load())
    assert reference == ours and reference[1] == 0


def _support_library_evaluate(h, expect_result):
    """The support library (libpolar_rt_support_static.a, linked into the probe) driven
    by a caller that declares GraphHandle, Device, Event and the launch structs from the
    reference's headers."""
    rng = np.random.default_rng(5)
    a = rng.standard_normal(4099).astype(np.float32)
    b = rng.standard_normal(4099).astype(np.float32)
    rc, total, a_back = abi_probe.support_evaluate(abi_probe.load(), h.raw_device(), a, b, 0.25, -1.5)
    assert rc == 0, f"support-library step {rc}"
    assert np.array_equal(a_back, a)           # RAM copy intact after the device's READ lock
    if expect_result:
        assert np.array_equal(total, np.float32(0.25) * a + np.float32(-1.5) * b)


def test_support_library_archive_defines_its_interface():
    """libpolar_rt_support_static.a defines every function include/polar_rt_support.hpp declares."""
    import os, re, subprocess
    from polarai_framework_amd import PACKAGE_DIR as PKG_DIR
    root = os.path.dirname(PKG_DIR)
    header = open(os.path.join(root, "include", "polar_rt_support.hpp")).read()
    declared = set(re.findall(r"\b(ath_\w+|polar_rt_support_\w+)\s*\(", header))
    assert {"ath_allocate", "ath_release", "ath_lock", "ath_device_select", "ath_barrier", "ath_launch",
            "ath_load"} <= declared
    nm = subprocess.run(["nm", "-g", "--defined-only", os.path.join(PKG_DIR, "libpolar_rt_support_static.a")],
                        check=True, capture_output=True, text=True).stdout
    defined = set(re.findall(r" T (\w+)", nm))
    assert declared <= defined, declared - defined


@needs_probe
def test_support_library_with_mock_device_and_reference_graph_handle():
    with harness.Harness(plugin=None) as h:
        _support_library_evaluate(h, expect_result=False)


@needs_probe
@pytest.mark.gpu
def test_support_library_with_hip_plugin_and_reference_graph_handle():
    with harness.Harness(plugin=LIB_PLUGIN) as h:
        _support_library_evaluate(h, expect_result=True)


@needs_probe
def test_mock_device_through_reference_declarations():
    with harness.Harness(plugin=None) as h:
        _exercise(h, expect_result=False)


@needs_probe
@pytest.mark.gpu
def test_hip_plugin_through_reference_declarations():
    with harness.Harness(plugin=LIB_PLUGIN) as h:
        lib = abi_probe.load()
        ctx = h.raw_context()
        assert lib.ref_context_device_count(ctx) == h.device_count >= 1
        assert lib.ref_context_device(ctx, 0) == h.raw_device()
        _exercise(h, expect_result=True)
