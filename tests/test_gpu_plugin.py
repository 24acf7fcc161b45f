"""The runtime plugin end to end: libpolar_rt_hip.so is opened like the
framework's runtime driver opens it, and every kernel is reached through
initContext() -> Device::launch(LaunchCommand) with the call sequence of the
framework's compiled graph code (mini-executor).  Results against the CPU
oracle, per kernel."""
import os
import subprocess
import sys

import numpy as np
import pytest

import parity
import polar_oracle as o
from polarai_framework_amd import LIB_PLUGIN, REPO_ROOT, TOOL_LSPOLAR, graphs, harness

pytestmark = pytest.mark.gpu


def _say(*a):
    print(*a, flush=True)


@pytest.fixture(params=["heap_ram", "plugin_ram"])
def h(request):
    """The caller's RAM-side blocks on the heap (as the framework's allocator keeps them) and in
    the plugin's pinned host memory (its optional polarHostMemory* symbols)."""
    hh = harness.Harness(plugin=LIB_PLUGIN,  # raises if no MI355X is found
                         plugin_host_memory=request.param == "plugin_ram")
    yield hh
    hh.close()


def _counters(h):
    c = h.counters()
    return {n: getattr(c, n) for n, _ in c._fields_}


def test_device_identity(h):
    assert h.device_count >= 1
    assert h.device_provider == 1   # DeviceProvider::HIP (runtime/Device.hpp:30)
    assert h.device_kind == 1       # DeviceKind::GPU
    name = h.device_name
    assert name != "host" and "gfx950" in name and "hip:0" in name


def test_device_listing_tool_reports_what_the_harness_sees(h):
    # the framework's lspolar for this plugin (utils/lspolar/main.cpp:55-82)
    _say("lspolar_hip")
    r = subprocess.run([TOOL_LSPOLAR], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    lines = r.stdout.splitlines()
    assert lines[0] == f"Total device count: {h.device_count}"
    names = [l.split(": ", 1)[1] for l in lines if l.startswith("Name       : ")]
    assert len(names) == h.device_count and h.device_name in names
    assert "Provider   : HIP" in lines and "Kind       : GPU" in lines and "Allocator  : 1" in lines


def _run_case(h, case):
    kn = case["kernel"]
    f32 = lambda x, shape=None: np.asarray(x, dtype=np.float32).reshape(shape or (-1,))
    if kn == "fadd":
        a, b = h.input(f32(case["a"])), h.input(f32(case["b"]))
        h.end_cluster()
        out = h.fadd(a, case["scaleA"], b, case["scaleB"])
    elif kn in ("fmul", "fdivide"):
        a, b = h.input(f32(case["a"])), h.input(f32(case["b"]))
        h.end_cluster()
        out = getattr(h, kn)(a, b)
    elif kn == "fmulconcat":
        g, l = h.input(f32(case["gradient"], (1, 1))), h.input(f32(case["local"], (2, 2)))
        h.end_cluster()
        out = h.fmulconcat(g, l)
    elif kn == "fsigmoid":
        x = h.input(f32(case["x"], (2, 2)))
        h.end_cluster()
        out = h.fsigmoid(x)
    elif kn == "flogloss":
        p, t = h.input(f32(case["predicted"], (2, 2))), h.input(f32(case["truth"], (2, 2)))
        h.end_cluster()
        out = h.flogloss(p, t)
    elif kn == "fmatmul":
        sa, sb = parity.stored_shapes(case["transA"], case["transB"], case["m"], case["n"], case["k"])
        a, b = h.input(f32(case["a"], sa)), h.input(f32(case["b"], sb))
        h.end_cluster()
        out = h.fmatmul(case["transA"], case["transB"], a, b)
    elif kn in ("frelu", "fsoftmax"):
        x = h.input(f32(case["x"], case.get("shape", (len(case["x"]),))))
        h.end_cluster()
        out = getattr(h, kn)(x)
    elif kn == "fconv2d":
        x, w = h.input(f32(case["x"], case["shape"])), h.input(f32(case["weights"], case["kernel_shape"]))
        h.end_cluster()
        out = h.fconv2d(x, w)
    elif kn == "fpool":
        x = h.input(f32(case["x"], case["shape"]))
        h.end_cluster()
        out = h.fpool(x, case["window"], case["stride"])
    h.end_cluster()
    h.run()
    return h.read(out)


@pytest.mark.parametrize("case", parity.golden_cases(), ids=lambda c: c["kernel"] + "@" + c["cite"].split("/")[-1])
def test_golden_vectors_through_plugin(h, case):
    _say("plugin golden", case["cite"])
    parity.check_case(case, _run_case(h, case))


def test_remaining_builtins_through_plugin(h):
    rng = np.random.default_rng(51)
    x = parity.normal(rng, (37, 53))
    X = h.input(x)
    h.end_cluster()
    c = h.fcopy(X)
    t = h.ftranspose(X)
    filled = h.ffill(3.0, h.tensor(1000))
    h.end_cluster()
    tt = h.fmatmul(True, True, X, t)    # X^T (53x37) * t^T (37x53) -> 53x53
    h.end_cluster()
    h.run()
    assert np.array_equal(h.read(c), x)
    assert np.array_equal(h.read(t), o.ftranspose(x))
    assert np.array_equal(h.read(filled), o.ffill(3.0, 1000))
    assert parity.frobenius_rel_error(h.read(tt), o.fmatmul(True, True, x, x.T.copy())) <= parity.MATMUL_FRO_REL


def test_coherence_counts_on_gpu(h):
    a = h.input(np.arange(1024, dtype=np.float32))
    b = h.input(np.ones(1024, dtype=np.float32))
    h.end_cluster()
    c = h.fadd(a, 1.0, b, 1.0)
    d = h.fmul(c, a)
    h.end_cluster()
    h.run()
    k = _counters(h)
    assert k["launches"] == 2 and k["copies_to_device"] == 2 and k["copies_to_host"] == 0
    assert k["events_waited"] == 2 and k["deferred_releases"] == 6
    assert np.array_equal(h.read(d), (np.arange(1024, dtype=np.float32) + 1) * np.arange(1024, dtype=np.float32))
    assert _counters(h)["copies_to_host"] == 1


def test_rewritten_ram_block_reaches_the_device(h):
    """Host code rewrites a tensor between evaluations: every evaluation sees the new values, also
    when the upload out of the RAM block was only queued when the previous evaluation returned."""
    n = 3 << 16
    a = h.tensor(n)
    h.holder(a)
    h.end_cluster()
    c = h.fadd(a, 1.0, a, 2.0)
    h.end_cluster()
    for i in range(6):
        data = np.arange(n, dtype=np.float32) % 977 + i
        h.host_write(a, data)
        h.run()
        if i % 2:                          # read back on some evaluations, rewrite at once on others
            assert np.array_equal(h.read(c), data * 3), i
    assert np.array_equal(h.read(c), data * 3)
    assert np.array_equal(h.read(a), data)


def test_logreg_forward_config(h):
    # X[256x784] U[0,1), W[784x10] N(0,0.01), b zeros, Y Bernoulli(0.1)
    rng = np.random.default_rng(61)
    x = rng.random((256, 784), dtype=np.float32)
    w = parity.normal(rng, (784, 10), 0.01)
    bias = np.zeros((256, 10), dtype=np.float32)
    y = (rng.random((256, 10)) < 0.1).astype(np.float32)
    g, named = graphs.logreg_forward(x, w, bias, y)
    tensors = {}
    graphs.emit(g, h, tensors)
    h.run()
    assert _counters(h)["launches"] == 4
    values = {k: h.read(t) for k, t in tensors.items()}
    report = parity.check_graph_nodes(g, values)
    _say("logreg per-kernel errors", report)
    # end to end against the oracle chain as well (looser: errors compound)
    ref = o.flogloss(o.fsigmoid(o.fadd(o.fmatmul(False, False, x, w), 1.0, bias, 1.0)), y)
    assert parity.elementwise_rel_error(values[named["L"].tensor_key], ref) < 1e-4


def test_mlp_forward_backward_config(h):
    # batch 1024, 1024 -> 4096 -> 1024, weights N(0, 1/sqrt(fan_in)), inputs U[0,1)
    o.set_threads(o.hw_threads())
    try:
        rng = np.random.default_rng(71)
        batch, d_in, d_hid, d_out = 1024, 1024, 4096, 1024
        x = rng.random((batch, d_in), dtype=np.float32)
        w1 = parity.normal(rng, (d_in, d_hid), 1 / np.sqrt(d_in))
        w2 = parity.normal(rng, (d_hid, d_out), 1 / np.sqrt(d_hid))
        y = (rng.random((batch, d_out)) < 0.5).astype(np.float32)
        f, g, u, named = graphs.mlp_graphs(x, w1, w2, y)
        tensors = {}
        for gr in (f, g):
            _say("run", gr.name, len(gr.nodes), "nodes")
            graphs.emit(gr, h, tensors)
            h.run()
            h.clear_program()
        values = {k: h.read(t) for k, t in tensors.items()}
        for gr in (f, g):
            report = parity.check_graph_nodes(gr, values)
            _say(gr.name, "worst", max(report.items(), key=lambda kv: kv[1]))
        assert np.isfinite(values[named["gW1"].tensor_key]).all()
        # weight update in place: W <- grad*lr + W
        graphs.emit(u, h, tensors)
        h.run()
        for wn, gn, w_old in (("W1", "gW1", w1), ("W2", "gW2", w2)):
            new = h.read(tensors[named[wn].tensor_key])
            grad = values[named[gn].tensor_key]
            lr = np.full(grad.shape, -0.01, dtype=np.float32)
            assert np.array_equal(new, o.fadd(o.fmul(grad, lr), 1.0, w_old, 1.0)), wn
    finally:
        o.set_threads(1)


def test_ragged_matmuls_through_plugin(h):
    # both readings of "65536x127x33" / "33x65536x127": (M,K,N) and (M,N,K)
    o.set_threads(o.hw_threads())
    try:
        for (m, n, k) in [(65536, 33, 127), (65536, 127, 33), (33, 127, 65536), (33, 65536, 127)]:
            _say("ragged matmul m,n,k =", m, n, k)
            rng = np.random.default_rng(m + 7 * n + 13 * k)
            a, b = parity.normal(rng, (m, k)), parity.normal(rng, (k, n))
            A, B = h.input(a), h.input(b)
            h.end_cluster()
            c = h.fmatmul(False, False, A, B)
            h.end_cluster()
            h.run()
            h.clear_program()
            got, ref = h.read(c), o.fmatmul(False, False, a, b)
            err = parity.frobenius_rel_error(got, ref)
            _say("  rel. Frobenius", err)
            assert err <= parity.MATMUL_FRO_REL
    finally:
        o.set_threads(1)


def test_offload_path_evicts_released_tensors(h):
    # cap the device layer at 3 MiB; 4 tensors of 1 MiB each cannot all stay
    h.set_device_byte_limit(3 << 20)
    n = 1 << 18
    rng = np.random.default_rng(81)
    data = [parity.normal(rng, n) for _ in range(3)]
    ins = [h.input(d) for d in data]
    h.end_cluster()
    s1 = h.fadd(ins[0], 1.0, ins[1], 1.0)       # device now holds 3 tensors
    h.end_cluster()
    s2 = h.fmul(s1, ins[2])                     # needs 2 more: evicts released ones
    h.end_cluster()
    h.run()
    ref1 = o.fadd(data[0], 1.0, data[1], 1.0)
    assert np.array_equal(h.read(s2), o.fmul(ref1, data[2]))
    assert np.array_equal(h.read(s1), ref1)     # saved by the offload callback or still resident
    h.set_device_byte_limit(0)


def _dies(code):
    env = dict(os.environ, PYTHONPATH=REPO_ROOT)
    prog = ("import __graft_entry__ as e; e.load_package();"
            "from polarai_framework_amd import harness, LIB_PLUGIN; import numpy as np;"
            "h = harness.Harness(plugin=LIB_PLUGIN);" + code)
    return subprocess.run([sys.executable, "-c", prog], env=env, capture_output=True, text=True, timeout=120)


def test_unknown_kernel_name_is_fatal():
    r = _dies("a = h.input(np.ones(4, dtype=np.float32)); h.end_cluster();"
              "h.node('fgelu', [a, h.tensor(4)], 1); h.end_cluster(); h.run()")
    assert r.returncode != 0 and "no native kernel 'fgelu'" in r.stderr


def test_pool_without_window_and_stride_is_fatal():
    # upstream's lowering forwards operands only; a native fpool needs the attributes appended
    r = _dies("a = h.input(np.ones((4, 4), dtype=np.float32)); h.end_cluster();"
              "h.node('fpool', [a, h.tensor(2, 2)], 1); h.end_cluster(); h.run()")
    assert r.returncode != 0 and "window and stride" in r.stderr


def test_next_builtins_through_plugin(h):
    rng = np.random.default_rng(52)
    x = parity.normal(rng, (70, 300))
    k = parity.normal(rng, (3, 3))
    X, K = h.input(x), h.input(k)
    h.end_cluster()
    r = h.frelu(X)
    s = h.fsoftmax(X)
    c = h.fconv2d(X, K)
    pl = h.fpool(X, (2, 3), (2, 2))
    h.end_cluster()
    h.run()
    assert np.array_equal(h.read(r), o.frelu(x))
    assert parity.elementwise_rel_error(h.read(s), o.fsoftmax(x)) <= parity.ELEMENTWISE_REL
    assert np.array_equal(h.read(c), o.fconv2d(x, k))
    assert np.array_equal(h.read(pl), o.fpool(x, (2, 3), (2, 2)))


def test_mismatched_matmul_shapes_are_fatal():
    r = _dies("a = h.input(np.ones((4, 5), dtype=np.float32)); b = h.input(np.ones((6, 3), dtype=np.float32));"
              "h.end_cluster(); h.node('fmatmul_f_f', [a, b, h.tensor(4, 3)], 2); h.end_cluster(); h.run()")
    assert r.returncode != 0 and "shapes do not agree" in r.stderr


# ---- kernels from a selected program (Device::selectBinary) ------------------------

CODE_OBJECT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "native", "build",
                           "generated_kernels.hsaco")


def _code_object():
    assert os.path.exists(CODE_OBJECT), "tests/native/build/generated_kernels.hsaco missing: run __graft_entry__.build()"
    with open(CODE_OBJECT, "rb") as fh:
        return fh.read()


def test_program_kernels_run_when_no_native_kernel_is_named(h):
    """A code object handed over through selectBinary; nodes without a native
    kernel name launch its kernels by their generated name, with tensors
    expanded to memref descriptors and the recorded launch geometry."""
    rng = np.random.default_rng(53)
    n, rows, cols = 5000, 37, 130
    x, y = parity.normal(rng, n), parity.normal(rng, n)
    m, s = parity.normal(rng, (rows, cols)), parity.normal(rng, rows)
    h.select_binary(_code_object(), {
        "gen_axpy_1d": (8, 1, 1, 256, 1, 1),
        "gen_row_scale_2d": ((cols + 63) // 64, (rows + 3) // 4, 1, 64, 4, 1)})
    X, Y, M, S = h.input(x), h.input(y), h.input(m), h.input(s)
    h.end_cluster()
    out1 = h.tensor(n)
    h.jit_node("gen_axpy_1d", [X, 0.5, Y, out1], 3)
    out2 = h.tensor(rows, cols)
    h.jit_node("gen_row_scale_2d", [M, S, out2], 2)
    native = h.fmul(X, Y)                       # hand-written kernels keep working beside it
    h.end_cluster()
    chained = h.frelu(out1)                     # and consume a program kernel's result
    h.end_cluster()
    h.run()
    ref1 = np.float32(0.5) * x + y
    assert np.array_equal(h.read(out1), ref1)
    assert np.array_equal(h.read(out2), m * s[:, None])
    assert np.array_equal(h.read(native), o.fmul(x, y))
    assert np.array_equal(h.read(chained), o.frelu(ref1))


def test_program_of_another_type_or_target_is_not_selected():
    _code_object()
    r = _dies(f"img = open({CODE_OBJECT!r}, 'rb').read();"
              "h.select_binary(img, {'gen_axpy_1d': (8, 1, 1, 256, 1, 1)}, program_type=0);"       # PTX
              "h.select_binary(img, {'gen_axpy_1d': (8, 1, 1, 256, 1, 1)}, target='gfx90a');"
              "a = h.input(np.ones(4, dtype=np.float32)); h.end_cluster();"
              "h.jit_node('gen_axpy_1d', [a, 1.0, a, h.tensor(4)], 3); h.end_cluster(); h.run()")
    assert r.returncode != 0 and "without a native kernel name" in r.stderr


def test_native_kernel_wins_over_a_program_kernel_of_the_same_node(h):
    h.select_binary(_code_object(), {"gen_axpy_1d": (8, 1, 1, 256, 1, 1)})
    a = h.input(np.arange(8, dtype=np.float32))
    h.end_cluster()
    out = h.fadd(a, 2.0, a, 3.0)
    h.end_cluster()
    h.run()
    assert np.array_equal(h.read(out), np.arange(8, dtype=np.float32) * 5)


def test_fused_builtins_through_plugin(h):
    """The logistic-regression forward pass as two fused launches equals the four-kernel graph."""
    rng = np.random.default_rng(54)
    x = rng.random((256, 784), dtype=np.float32)
    w = parity.normal(rng, (784, 10), 0.01)
    bias = parity.normal(rng, (256, 10), 0.1)
    y = (rng.random((256, 10)) < 0.1).astype(np.float32)
    X, W, B, Y = h.input(x), h.input(w), h.input(bias), h.input(y)
    h.end_cluster()
    z = h.fmatmul(False, False, X, W)
    fused_p = h.fmatmul_fadd_fsigmoid(False, False, X, W, 1.0, B, 1.0)
    h.end_cluster()
    s = h.fadd(z, 1.0, B, 1.0)
    h.end_cluster()
    p = h.fsigmoid(s)
    fused_loss = h.fsigmoid_flogloss(s, Y)
    h.end_cluster()
    loss = h.flogloss(p, Y)
    h.end_cluster()
    h.run()
    assert np.array_equal(h.read(fused_p), h.read(p))
    assert np.array_equal(h.read(fused_loss), h.read(loss))
    ref = o.fsigmoid(o.fadd(o.fmatmul(False, False, x, w), 1.0, bias, 1.0))
    assert parity.elementwise_rel_error(h.read(p), ref) <= parity.ELEMENTWISE_REL
