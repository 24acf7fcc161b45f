"""Helpers shared by the parity tests: seeded input generators for the
benchmark configurations, the tolerance rules, and a dispatcher that runs one
golden-vector case on either the oracle or the device."""
import json
import os

import numpy as np

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden",
                      "reference_vectors.json")

# Tolerances of the parity contract
ELEMENTWISE_REL = 1e-5   # per element, relative
MATMUL_FRO_REL = 1e-4    # relative Frobenius


def golden_cases():
    with open(GOLDEN) as fh:
        return json.load(fh)


def uniform(rng, n, lo, hi):
    return (rng.random(n, dtype=np.float32) * np.float32(hi - lo) + np.float32(lo)).astype(np.float32)


def normal(rng, shape, std=1.0):
    return (rng.standard_normal(shape, dtype=np.float32) * np.float32(std)).astype(np.float32)


def elementwise_rel_error(got, ref, scale=None):
    """max |x-r| / max(|r|, 1e-5*scale): relative error with an absolute floor
    where the reference value is ~0 (scale = largest magnitude involved)."""
    got = np.asarray(got, dtype=np.float64).ravel()
    ref = np.asarray(ref, dtype=np.float64).ravel()
    if scale is None:
        scale = float(np.max(np.abs(ref))) if ref.size else 1.0
    floor = max(1e-5 * scale, 1e-30)
    if got.size == 0:
        return 0.0
    return float(np.max(np.abs(got - ref) / np.maximum(np.abs(ref), floor)))


def frobenius_rel_error(got, ref):
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    den = np.linalg.norm(ref)
    return float(np.linalg.norm(got - ref) / (den if den > 0 else 1.0))


def stored_shapes(ta, tb, m, n, k):
    return ((k, m) if ta else (m, k)), ((n, k) if tb else (k, n))


def run_case_oracle(case):
    import polar_oracle as o
    kn = case["kernel"]
    if kn == "fadd":
        return o.fadd(case["a"], case["scaleA"], case["b"], case["scaleB"])
    if kn == "fmul":
        return o.fmul(case["a"], case["b"])
    if kn == "fdivide":
        return o.fdivide(case["a"], case["b"])
    if kn == "fmulconcat":
        return o.fmulconcat(case["gradient"], case["local"])
    if kn == "fsigmoid":
        return o.fsigmoid(case["x"])
    if kn == "flogloss":
        return o.flogloss(case["predicted"], case["truth"])
    if kn == "fmatmul":
        sa, sb = stored_shapes(case["transA"], case["transB"], case["m"], case["n"], case["k"])
        a = np.asarray(case["a"], dtype=np.float32).reshape(sa)
        b = np.asarray(case["b"], dtype=np.float32).reshape(sb)
        return o.fmatmul(case["transA"], case["transB"], a, b).ravel()
    if kn == "frelu":
        return o.frelu(case["x"])
    if kn == "fsoftmax":
        return o.fsoftmax(np.asarray(case["x"], dtype=np.float32).reshape(case["shape"])).ravel()
    if kn == "fconv2d":
        x = np.asarray(case["x"], dtype=np.float32).reshape(case["shape"])
        w = np.asarray(case["weights"], dtype=np.float32).reshape(case["kernel_shape"])
        return o.fconv2d(x, w).ravel()
    if kn == "fpool":
        x = np.asarray(case["x"], dtype=np.float32).reshape(case["shape"])
        return o.fpool(x, case["window"], case["stride"]).ravel()
    raise KeyError(kn)


def run_case_device(dev, case):
    kn = case["kernel"]
    bufs = []

    def up(x):
        b = dev.array(np.asarray(x, dtype=np.float32))
        bufs.append(b)
        return b
    try:
        if kn == "fadd":
            a, b = up(case["a"]), up(case["b"])
            c = dev.empty(a.count); bufs.append(c)
            dev.fadd(a, case["scaleA"], b, case["scaleB"], c)
        elif kn in ("fmul", "fdivide"):
            a, b = up(case["a"]), up(case["b"])
            c = dev.empty(a.count); bufs.append(c)
            getattr(dev, kn)(a, b, c)
        elif kn == "fmulconcat":
            g, l = up(case["gradient"]), up(case["local"])
            c = dev.empty(l.count); bufs.append(c)
            dev.fmulconcat(g, l, c)
        elif kn == "fsigmoid":
            x = up(case["x"])
            c = dev.empty(x.count); bufs.append(c)
            dev.fsigmoid(x, c)
        elif kn == "flogloss":
            p, t = up(case["predicted"]), up(case["truth"])
            c = dev.empty(p.count); bufs.append(c)
            dev.flogloss(p, t, c)
        elif kn == "fmatmul":
            a, b = up(case["a"]), up(case["b"])
            c = dev.empty(case["m"] * case["n"]); bufs.append(c)
            dev.fmatmul(case["transA"], case["transB"], a, b, c, case["m"], case["n"], case["k"])
        elif kn in ("frelu", "fsoftmax"):
            x = up(case["x"])
            c = dev.empty(x.count); bufs.append(c)
            getattr(dev, kn)(x, c)
        elif kn == "fconv2d":
            x, w = up(case["x"]), up(case["weights"])
            (h, wd), (kh, kw) = case["shape"], case["kernel_shape"]
            c = dev.empty((h - kh + 1) * (wd - kw + 1)); bufs.append(c)
            dev.fconv2d(x, w, c, h, wd, kh, kw)
        elif kn == "fpool":
            x = up(case["x"])
            (h, wd), win, st = case["shape"], case["window"], case["stride"]
            c = dev.empty(((h - win[0]) // st[0] + 1) * ((wd - win[1]) // st[1] + 1)); bufs.append(c)
            dev.fpool(x, c, h, wd, win, st)
        else:
            raise KeyError(kn)
        return c.download()
    finally:
        for b in bufs:
            b.free()


def check_case(case, got):
    exp = np.asarray(case["expected"], dtype=np.float64)
    got = np.asarray(got, dtype=np.float64).ravel()
    assert got.shape == exp.shape
    if case["exact"]:
        assert np.array_equal(got.astype(np.float32), exp.astype(np.float32)), (case["cite"], got, exp)
    else:
        rel = np.abs(got - exp) / np.abs(exp)
        assert np.all(rel <= case["rel_tol"]), (case["cite"], got, exp)
        for i in case.get("exact_indices", []):
            assert np.float32(got[i]) == np.float32(exp[i]), (case["cite"], i, got[i], exp[i])


# ---- per-node checking of a kernel DAG run through the mini-executor ---------

BIT_EXACT_KERNELS = {"fadd", "fmul", "fdivide", "fmulconcat", "fcopy", "ffill", "ftranspose", "frelu",
                     "fconv2d", "fpool"}


def oracle_node(node, values):
    """Oracle result of one compute node of polarai_framework_amd.graphs, fed
    with the operand values the device consumed (`values`: tensor key ->
    array)."""
    import polar_oracle as o
    ins = [values[a.tensor_key] if hasattr(a, "tensor_key") else a for a in node.args[:-1]]
    k = node.kernel
    if k == "fadd":
        return o.fadd(ins[0], ins[1], ins[2], ins[3])
    if k == "fmul":
        return o.fmul(ins[0], ins[1])
    if k == "fdivide":
        return o.fdivide(ins[0], ins[1])
    if k == "fsigmoid":
        return o.fsigmoid(ins[0])
    if k == "flogloss":
        return o.flogloss(ins[0], ins[1])
    if k == "fmulconcat":
        return o.fmulconcat(ins[0], ins[1])
    if k.startswith("fmatmul_"):
        return o.fmatmul(k[8] == "t", k[10] == "t", ins[0], ins[1])
    raise KeyError(k)


def check_graph_nodes(graph, values):
    """Every compute node of `graph`: device output (values[result]) against
    the oracle on the same operands.  Returns {node name: error}."""
    report = {}
    for node in graph.nodes:
        if node.kind != "op":
            continue
        got = values[node.tensor_key]
        ref = oracle_node(node, values).reshape(got.shape)
        label = f"{graph.name}:{node.name or node.kernel}"
        if node.kernel in BIT_EXACT_KERNELS:
            assert np.array_equal(got, ref), label
            report[label] = 0.0
        elif node.kernel.startswith("fmatmul"):
            err = frobenius_rel_error(got, ref)
            assert err <= MATMUL_FRO_REL, (label, err)
            report[label] = err
        else:
            err = elementwise_rel_error(got, ref)
            assert err <= ELEMENTWISE_REL, (label, err)
            report[label] = err
    return report
