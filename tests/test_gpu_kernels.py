"""Parity of the gfx950 kernels with the CPU oracle, through the C ABI
(include/polar_hip.h).  Bit-exact for the operations that are single IEEE
operations or pure data movement; 1e-5 relative per element for
sigmoid/logloss; 1e-4 relative Frobenius for matmul."""
import ctypes as C

import numpy as np
import pytest

import parity
import polar_oracle as o

pytestmark = pytest.mark.gpu

SIZES = [1, 2, 3, 4, 5, 63, 64, 255, 256, 1023, 1024, 4099, 65536 + 7, 1000003]


def _say(*a):
    print(*a, flush=True)


@pytest.mark.parametrize("case", parity.golden_cases(), ids=lambda c: c["kernel"] + "@" + c["cite"].split("/")[-1])
def test_golden_vectors_on_device(dev, case):
    _say("golden", case["cite"])
    parity.check_case(case, parity.run_case_device(dev, case))


@pytest.mark.parametrize("n", SIZES)
@pytest.mark.parametrize("misalign", [0, 1, 3, 29])
def test_binary_ops_bit_exact(dev, n, misalign):
    _say("binary ops n=", n, "misalign=", misalign)
    rng = np.random.default_rng(100 + n)
    a = parity.uniform(rng, n, -1, 1)
    b = parity.uniform(rng, n, -1, 1)
    den = parity.uniform(rng, n, 0.5, 2)
    da, db, dden = (dev.array(x, misalign) for x in (a, b, den))
    dc = dev.empty(n, misalign)
    dev.fadd(da, 1.0, db, 1.0, dc)
    assert np.array_equal(dc.download(), o.fadd(a, 1.0, b, 1.0))
    dev.fadd(da, 0.34, db, 0.21, dc)
    assert np.array_equal(dc.download(), o.fadd(a, 0.34, b, 0.21))
    dev.fmul(da, db, dc)
    assert np.array_equal(dc.download(), o.fmul(a, b))
    dev.fdivide(da, dden, dc)
    assert np.array_equal(dc.download(), o.fdivide(a, den))
    for x in (da, db, dden, dc):
        x.free()


@pytest.mark.parametrize("n", SIZES)
def test_mixed_alignment(dev, n):
    # operands at different offsets from a 16-byte boundary: dword path;
    # same offset modulo 16 bytes but different lines: vector path with a head
    _say("mixed alignment n=", n)
    rng = np.random.default_rng(200 + n)
    a, b = parity.uniform(rng, n, -1, 1), parity.uniform(rng, n, -1, 1)
    for ma, mb, mc in ((0, 3, 2), (1, 5, 9), (4, 0, 8), (7, 7, 7)):
        da, db, dc = dev.array(a, ma), dev.array(b, mb), dev.empty(n + 8, mc)
        dev.ffill(-7.0, dc, n + 8)
        dev.fmul(da, db, dc, n)
        got = dc.download()
        assert np.array_equal(got[:n], o.fmul(a, b))
        assert np.all(got[n:] == -7.0)          # nothing written past the end
        for x in (da, db, dc):
            x.free()


@pytest.mark.parametrize("n", SIZES)
@pytest.mark.parametrize("misalign", [0, 1, 2, 31])
def test_unary_and_fill(dev, n, misalign):
    _say("unary n=", n, "misalign=", misalign)
    rng = np.random.default_rng(300 + n)
    x = parity.uniform(rng, n, -1, 1)
    g = np.array([np.float32(-2.5), 9.0], dtype=np.float32)
    dx, dg, dout = dev.array(x, misalign), dev.array(g), dev.empty(n, misalign)
    dev.fcopy(dx, dout)
    assert np.array_equal(dout.download(), x)
    dev.ffill(3.0, dout)
    assert np.array_equal(dout.download(), o.ffill(3.0, n))
    dev.fmulconcat(dg, dx, dout)
    assert np.array_equal(dout.download(), o.fmulconcat(g, x))
    for b in (dx, dg, dout):
        b.free()


@pytest.mark.parametrize("n", SIZES)
def test_sigmoid_logloss(dev, n):
    _say("sigmoid/logloss n=", n)
    rng = np.random.default_rng(400 + n)
    x = parity.uniform(rng, n, -1, 1)
    wide = parity.uniform(rng, n, -30, 30)  # reaches both clamps
    y = (rng.random(n) < 0.1).astype(np.float32)
    dx, dw, dy, dp, dl = dev.array(x), dev.array(wide), dev.array(y), dev.empty(n), dev.empty(n)
    dev.fsigmoid(dx, dp)
    p = dp.download()
    assert parity.elementwise_rel_error(p, o.fsigmoid(x)) <= parity.ELEMENTWISE_REL
    dev.flogloss(dp, dy, dl)
    assert parity.elementwise_rel_error(dl.download(), o.flogloss(p, y)) <= parity.ELEMENTWISE_REL
    dev.fsigmoid(dw, dp)
    pw = dp.download()
    ref = o.fsigmoid(wide)
    assert parity.elementwise_rel_error(pw, ref) <= parity.ELEMENTWISE_REL
    eps = np.float32(1e-5)
    assert pw.min() >= eps and pw.max() <= np.float32(1) - eps
    dev.flogloss(dp, dy, dl)
    assert parity.elementwise_rel_error(dl.download(), o.flogloss(pw, y)) <= parity.ELEMENTWISE_REL
    for b in (dx, dw, dy, dp, dl):
        b.free()


def test_sigmoid_special_values(dev):
    xs = np.array([0.0, -100.0, 100.0, -200.0, 1e30, -1e30, -11.0, 11.0, -12.0, 12.0], dtype=np.float32)
    dx, dp = dev.array(xs), dev.empty(xs.size)
    dev.fsigmoid(dx, dp)
    got, ref = dp.download(), o.fsigmoid(xs)
    assert parity.elementwise_rel_error(got, ref) <= parity.ELEMENTWISE_REL
    eps = np.float32(1e-5)
    assert got[0] == np.float32(0.5)
    assert got[1] == eps and got[3] == eps and got[5] == eps and got[8] == eps
    assert got[2] == np.float32(1) - eps and got[4] == np.float32(1) - eps and got[9] == np.float32(1) - eps
    dx.free(); dp.free()


def test_empty_inputs(dev):
    a = dev.empty(4)
    for fn in (lambda: dev.fadd(a, 1.0, a, 1.0, a, 0), lambda: dev.fmul(a, a, a, 0),
               lambda: dev.fsigmoid(a, a, 0), lambda: dev.ffill(1.0, a, 0),
               lambda: dev.ftranspose(a, a, 0, 5), lambda: dev.fmatmul(0, 0, a, a, a, 0, 4, 4)):
        fn()
    dev.synchronize()
    a.free()


def test_in_place_update(dev):
    # the framework's weight update writes fadd's result into its first operand
    rng = np.random.default_rng(9)
    w, g = parity.normal(rng, 100003), parity.normal(rng, 100003)
    dw, dg = dev.array(w), dev.array(g)
    dev.fadd(dw, 1.0, dg, -0.01, dw)
    assert np.array_equal(dw.download(), o.fadd(w, 1.0, g, -0.01))
    dw.free(); dg.free()


@pytest.mark.parametrize("shape", [(1, 1), (1, 7), (7, 1), (3, 5), (64, 64), (65, 63), (64, 1000),
                                   (1000, 64), (257, 129), (1031, 517), (1, 100003), (100003, 1),
                                   (513, 1025), (2048, 2048), (127, 4099), (4099, 127), (12345, 6789),
                                   # output pitch a large power-of-two multiple (strips numbered in runs),
                                   # with full and ragged column tiles; interior strips on the lean path
                                   (8192, 300), (10240, 257), (16384, 128), (2048, 4100), (300, 8192)])
def test_transpose(dev, shape):
    _say("transpose", shape)
    rng = np.random.default_rng(shape[0] * 7919 + shape[1])
    x = parity.normal(rng, shape)
    dx, dt, dtt = dev.array(x), dev.empty(x.size), dev.empty(x.size)
    dev.ftranspose(dx, dt, shape[0], shape[1])
    assert np.array_equal(dt.download((shape[1], shape[0])), o.ftranspose(x))
    dev.ftranspose(dt, dtt, shape[1], shape[0])  # involution
    assert np.array_equal(dtt.download(shape), x)
    for b in (dx, dt, dtt):
        b.free()


MM_SHAPES = [(1, 1, 4), (2, 2, 2), (2, 3, 4), (1, 1, 1), (5, 7, 3), (32, 32, 32), (64, 64, 64),
             (128, 128, 128), (256, 384, 512), (130, 70, 50), (127, 33, 65), (33, 127, 129),
             (200, 10, 784), (256, 10, 784), (129, 257, 1), (300, 300, 300), (512, 512, 2048)]


def _matmul_device(dev, ta, tb, a, b, m, n, k, misalign=0):
    da, db, dc = dev.array(a, misalign), dev.array(b, misalign), dev.empty(m * n, misalign)
    dev.fmatmul(ta, tb, da, db, dc, m, n, k)
    out = dc.download((m, n))
    for x in (da, db, dc):
        x.free()
    return out


@pytest.mark.parametrize("ta", [False, True])
@pytest.mark.parametrize("tb", [False, True])
@pytest.mark.parametrize("mnk", MM_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_matmul(dev, ta, tb, mnk):
    m, n, k = mnk
    _say("matmul", ta, tb, mnk)
    rng = np.random.default_rng(m * 1000003 + n * 1009 + k + 2 * ta + tb)
    sa, sb = parity.stored_shapes(ta, tb, m, n, k)
    a, b = parity.normal(rng, sa), parity.normal(rng, sb)
    got = _matmul_device(dev, ta, tb, a, b, m, n, k)
    ref = o.fmatmul(ta, tb, a, b)
    assert parity.frobenius_rel_error(got, ref) <= parity.MATMUL_FRO_REL
    # no element is left unwritten or badly off either
    assert np.max(np.abs(got - ref)) <= 1e-3 * max(1.0, np.sqrt(k))


@pytest.mark.parametrize("ta", [False, True])
@pytest.mark.parametrize("tb", [False, True])
def test_matmul_integer_exact_and_tt_identity(dev, ta, tb):
    # small integers: every partial sum is exact in fp32 whatever the order
    rng = np.random.default_rng(11 + 2 * ta + tb)
    m, n, k = 150, 90, 210
    sa, sb = parity.stored_shapes(ta, tb, m, n, k)
    a = rng.integers(-8, 9, sa).astype(np.float32)
    b = rng.integers(-8, 9, sb).astype(np.float32)
    got = _matmul_device(dev, ta, tb, a, b, m, n, k)
    assert np.array_equal(got, o.fmatmul(ta, tb, a, b))
    if ta and tb:  # (A^T B^T) = (B A)^T
        ba = _matmul_device(dev, False, False, b, a, n, m, k)
        assert np.array_equal(got, ba.T)


@pytest.mark.parametrize("ta", [False, True])
@pytest.mark.parametrize("tb", [False, True])
def test_matmul_unaligned_base(dev, ta, tb):
    rng = np.random.default_rng(21 + 2 * ta + tb)
    m, n, k = 132, 68, 100
    sa, sb = parity.stored_shapes(ta, tb, m, n, k)
    a, b = parity.normal(rng, sa), parity.normal(rng, sb)
    got = _matmul_device(dev, ta, tb, a, b, m, n, k, misalign=1)
    assert parity.frobenius_rel_error(got, o.fmatmul(ta, tb, a, b)) <= parity.MATMUL_FRO_REL


# every tile configuration of the tiled kernel, whatever the planner would pick: a shape
# that is a multiple of no tile (edges), one that every tile divides (no edge code), one
# whose leading dimensions are no multiple of 4 (scalar fetches); one part and split
TILE_CASES = [(300, 270, 200), (512, 512, 128), (259, 301, 67)]


@pytest.mark.parametrize("ta", [False, True])
@pytest.mark.parametrize("tb", [False, True])
@pytest.mark.parametrize("config", range(10))
def test_matmul_every_tile_configuration(dev, ta, tb, config):
    for (m, n, k) in TILE_CASES:
        _say("tile configuration", config, ta, tb, (m, n, k))
        rng = np.random.default_rng(config * 131 + m + 2 * ta + tb)
        sa, sb = parity.stored_shapes(ta, tb, m, n, k)
        # small integers: exact in fp32 in any order of the additions
        a = rng.integers(-8, 9, sa).astype(np.float32)
        b = rng.integers(-8, 9, sb).astype(np.float32)
        ref = o.fmatmul(ta, tb, a, b)
        da, db = dev.array(a), dev.array(b)
        for splits in (1, 3):
            dc = dev.array(np.full(m * n, np.nan, dtype=np.float32))
            dev.fmatmul_with_plan(ta, tb, da, db, dc, m, n, k, config, splits)
            assert np.array_equal(dc.download((m, n)), ref), (config, (m, n, k), splits)
            dc.free()
        da.free()
        db.free()


def test_matmul_split_contraction_is_added_by_the_last_group_repeatably(dev):
    """Up to eight parts of K are added by whichever work-group finishes a tile
    last (an arrival counter per tile, set back to zero by that group); more
    parts go through the second kernel.  The sum is taken in split order either
    way: repeated calls give the same bits, calls of other shapes in between find
    the counters at zero, and integer data is exact under every plan."""
    rng = np.random.default_rng(77)
    shapes = [(768, 768, 768), (1536, 1536, 1536), (1000, 515, 2100), (384, 384, 4096)]
    data = {}
    for (m, n, k) in shapes:
        a = rng.integers(-8, 9, (m, k)).astype(np.float32)
        b = rng.integers(-8, 9, (k, n)).astype(np.float32)
        data[(m, n, k)] = (dev.array(a), dev.array(b), o.fmatmul(False, False, a, b))
    for rnd in range(3):                       # the shapes in turn, three times over
        for (m, n, k), (da, db, ref) in data.items():
            _say("split contraction", (m, n, k), "round", rnd)
            dc = dev.array(np.full(m * n, np.nan, dtype=np.float32))
            dev.fmatmul(False, False, da, db, dc, m, n, k)
            assert np.array_equal(dc.download((m, n)), ref)
            for config, splits in ((1, 2), (1, 8), (2, 5), (8, 3), (1, 12), (2, 16)):   # <= 8: last group; more: second kernel
                dev.ffill(float("nan"), dc)
                dev.fmatmul_with_plan(False, False, da, db, dc, m, n, k, config, splits)
                assert np.array_equal(dc.download((m, n)), ref), ((m, n, k), config, splits, rnd)
            dc.free()
    # two operand sets of one shape in turn, back to back with nothing waited for in between: the same plan
    # and the same places in the workspace, different values -- a partial product read from a stale cache
    # line would be the other set's
    m, n, k = 700, 900, 2600
    pair = []
    for i in range(2):
        a = rng.integers(-8, 9, (k, m)).astype(np.float32)
        b = rng.integers(-8, 9, (k, n)).astype(np.float32)
        pair.append((dev.array(a), dev.array(b), dev.empty(m * n), o.fmatmul(True, False, a, b)))
    for config, splits in ((1, 4), (2, 7), (0, 2), (9, 3)):
        for rep in range(4):
            for da, db, dc, ref in pair:
                dev.fmatmul_with_plan(True, False, da, db, dc, m, n, k, config, splits)
        for da, db, dc, ref in pair:
            assert np.array_equal(dc.download((m, n)), ref), (config, splits)
    for st in pair:
        for t in st[:3]:
            t.free()
    # real-valued data: the same bits every time, whichever group arrives last
    m, n, k = 1536, 1536, 1536
    a, b = parity.normal(rng, (m, k)), parity.normal(rng, (k, n))
    da, db = dev.array(a), dev.array(b)
    outs = []
    for i in range(6):
        dc = dev.empty(m * n)
        dev.fmatmul_with_plan(False, False, da, db, dc, m, n, k, 1, 3)
        outs.append(dc.download((m, n)))
        dc.free()
    for other in outs[1:]:
        assert np.array_equal(outs[0].view(np.uint32), other.view(np.uint32))
    assert parity.frobenius_rel_error(outs[0], o.fmatmul(False, False, a, b)) <= parity.MATMUL_FRO_REL
    for t in [da, db] + [x for v in data.values() for x in v[:2]]:
        t.free()


SKINNY_SHAPES = [(256, 10, 784), (1, 1, 64), (1, 1, 16384), (7, 3, 100), (300, 16, 68), (512, 1, 16384),
                 (1000, 5, 260), (64, 8, 1024), (2, 13, 1260), (1024, 1, 64), (1024, 10, 784), (16, 16, 1024),
                 # not this kernel's (K no multiple of 4, K too short, too many rows or columns, too much of B):
                 # passed on
                 (256, 10, 786), (256, 10, 60), (1025, 10, 784), (256, 17, 784), (1024, 16, 784), (513, 9, 4096)]


@pytest.mark.parametrize("mnk", SKINNY_SHAPES)
def test_matmul_with_a_skinny_result(dev, mnk):
    """At most 16 columns and 1024 rows of C, operands as stored: one wave per row of C
    in one launch (the logistic-regression forward product).  Integer data is exact
    under any order of the additions; bases off 16 bytes go to the tiled kernel."""
    m, n, k = mnk
    rng = np.random.default_rng(4100 + m + n + k)
    a = rng.integers(-8, 9, (m, k)).astype(np.float32)
    b = rng.integers(-8, 9, (k, n)).astype(np.float32)
    ref = o.fmatmul(False, False, a, b)
    for mis_a, mis_b, mis_c in ((0, 0, 0), (0, 0, 5), (1, 0, 0), (0, 3, 2)):
        _say("skinny matmul", mnk, "misalign", (mis_a, mis_b, mis_c), "plan", dev.fmatmul_plan(m, n, k))
        da, db, dc = dev.array(a, mis_a), dev.array(b, mis_b), dev.empty(m * n + 32, mis_c)
        dev.ffill(-7.0, dc)
        dev.fmatmul(False, False, da, db, dc, m, n, k)
        got = dc.download()
        assert np.array_equal(got[:m * n].reshape(m, n), ref)
        assert np.all(got[m * n:] == -7.0)
        for t in (da, db, dc):
            t.free()
    # real-valued data against the oracle's sequential sum
    a, b = parity.normal(rng, (m, k)), parity.normal(rng, (k, n))
    da, db, dc = dev.array(a), dev.array(b), dev.empty(m * n)
    dev.fmatmul(False, False, da, db, dc, m, n, k)
    assert parity.frobenius_rel_error(dc.download((m, n)), o.fmatmul(False, False, a, b)) <= parity.MATMUL_FRO_REL
    for t in (da, db, dc):
        t.free()


def test_matmul_plan_is_reported_and_forced_plans_are_checked(dev):
    config, splits, tile = dev.fmatmul_plan(4096, 4096, 4096)
    assert (config, splits, tile) == (0, 1, (256, 256, 32))
    config, splits, tile = dev.fmatmul_plan(300, 257, 3000)
    assert 0 <= config < 10 and splits > 1 and tile[2] == 32
    assert dev.fmatmul_plan(256, 10, 784)[0] == -1            # one wave per row of a skinny result
    assert dev.fmatmul_plan(65536, 33, 127)[0] == -1          # the short-contraction kernels
    x, y, z = dev.empty(64 * 64), dev.empty(64 * 64), dev.empty(64 * 64)
    for bad in ((10, 1), (-1, 1), (2, 0), (2, 257)):
        with pytest.raises(Exception):
            dev.fmatmul_with_plan(False, False, x, y, z, 64, 64, 64, *bad)
    for t in (x, y, z):
        t.free()


# short contraction with one long and one short output dimension: the one-shot
# kernels that keep all of K and of the short dimension in LDS (tall: M long,
# wide: N long), every layout, ragged edges, K and N that are no multiple of 4/16
SHORT_K_SHAPES = [(65536, 33, 127), (65536, 127, 33), (33, 65536, 127), (1024, 1, 1), (1031, 16, 4),
                  (2049, 17, 128), (1, 1024, 5), (128, 3001, 100), (1500, 128, 77), (4096, 48, 64),
                  (100, 1111, 3), (7000, 65, 2)]


@pytest.mark.parametrize("ta", [False, True])
@pytest.mark.parametrize("tb", [False, True])
@pytest.mark.parametrize("mnk", SHORT_K_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_matmul_short_contraction_tall_and_wide(dev, ta, tb, mnk):
    m, n, k = mnk
    _say("short-k matmul", ta, tb, mnk)
    rng = np.random.default_rng(m * 7 + n * 1009 + k + 2 * ta + tb)
    sa, sb = parity.stored_shapes(ta, tb, m, n, k)
    o.set_threads(o.hw_threads())
    try:
        # small integers: exact in fp32 in any order, so a wrong index shows as a wrong value
        a = rng.integers(-8, 9, sa).astype(np.float32)
        b = rng.integers(-8, 9, sb).astype(np.float32)
        da, db, dc = dev.array(a, 1), dev.array(b, 3), dev.empty(m * n + 64, 2)
        dev.ffill(-7.0, dc, m * n + 64)
        dev.fmatmul(ta, tb, da, db, dc, m, n, k)
        got = dc.download()
        assert np.array_equal(got[:m * n].reshape(m, n), o.fmatmul(ta, tb, a, b))
        assert np.all(got[m * n:] == -7.0)                 # nothing written past the end
        for t in (da, db, dc):
            t.free()
        a, b = parity.normal(rng, sa), parity.normal(rng, sb)
        got = _matmul_device(dev, ta, tb, a, b, m, n, k)
        assert parity.frobenius_rel_error(got, o.fmatmul(ta, tb, a, b)) <= parity.MATMUL_FRO_REL
        assert np.array_equal(got, _matmul_device(dev, ta, tb, a, b, m, n, k))   # repeatable
    finally:
        o.set_threads(1)


# One long and one short output dimension with the long one at least 3/4 x 256 x
# the number of CUs: the kernels that give every SIMD a panel of its own
# (matmul_panel.hip; matmul_rows.hip when A is stored row by row and aligned).
LONG_PANEL_SHAPES = [(65536, 33, 127), (65521, 33, 127), (65553, 127, 33), (33, 65536, 127), (65537, 33, 127),
                     (33, 65541, 127), (65599, 64, 128), (49152, 1, 4), (1, 49153, 5), (70001, 17, 63), (16, 70003, 64),
                     (66000, 128, 64), (128, 66001, 33), (65536, 48, 100), (48, 65538, 16), (65536, 65, 17),
                     (100000, 5, 97), (65567, 17, 5), (70000, 128, 16), (65536, 100, 65), (65536, 15, 113),
                     # five or six column blocks with five or six groups of k: too much of B for the kernel that
                     # keeps it in registers, which must pass these on
                     (65536, 70, 90), (50011, 81, 95), (49152, 96, 80), (96, 66000, 80)]


@pytest.mark.parametrize("misalign", [0, 1])
@pytest.mark.parametrize("ta", [False, True])
@pytest.mark.parametrize("tb", [False, True])
@pytest.mark.parametrize("mnk", LONG_PANEL_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_matmul_short_contraction_long_panels(dev, ta, tb, mnk, misalign):
    """Integer data (exact in any summation order, so a wrong index shows as a
    wrong value) with line-aligned and with misaligned operands, a guard region
    on both sides of C; then random data against the oracle."""
    m, n, k = mnk
    _say("long-panel matmul", ta, tb, mnk, misalign)
    rng = np.random.default_rng(m * 13 + n * 1019 + k + 2 * ta + tb)
    sa, sb = parity.stored_shapes(ta, tb, m, n, k)
    o.set_threads(o.hw_threads())
    try:
        a = rng.integers(-4, 5, sa).astype(np.float32)
        b = rng.integers(-4, 5, sb).astype(np.float32)
        da, db = dev.array(a, misalign), dev.array(b, misalign)
        whole = dev.empty(m * n + 128, 0)
        dev.ffill(-7.0, whole, m * n + 128)
        dc = type(whole)(dev, m * n, whole.ptr, (64 + misalign) * 4)   # C inside the guarded block
        dev.fmatmul(ta, tb, da, db, dc, m, n, k)
        got = whole.download()
        lo = 64 + misalign
        assert np.array_equal(got[lo:lo + m * n].reshape(m, n), o.fmatmul(ta, tb, a, b))
        assert np.all(got[:lo] == -7.0) and np.all(got[lo + m * n:] == -7.0)   # nothing written outside C
        for t in (da, db, whole):
            t.free()
        if misalign == 0:
            a, b = parity.normal(rng, sa), parity.normal(rng, sb)
            got = _matmul_device(dev, ta, tb, a, b, m, n, k)
            assert parity.frobenius_rel_error(got, o.fmatmul(ta, tb, a, b)) <= parity.MATMUL_FRO_REL
    finally:
        o.set_threads(1)


# A long contraction with a result of at most 33 x 128, operands as stored: one
# slice of K per CU and a second kernel that adds the partial results
# (matmul_long_k.hip).  K not a multiple of 4, 16 or 64 exercises the clamped
# loads at the end of both operands.
LONG_K_SHAPES = [(33, 127, 65536), (33, 127, 65537), (33, 128, 70001), (32, 100, 16384), (17, 64, 20000), (16, 4, 16385),
                 (1, 65, 33333), (33, 5, 65539), (9, 127, 100003), (16, 4, 16386), (31, 33, 262144)]


@pytest.mark.parametrize("misalign", [0, 1])
@pytest.mark.parametrize("mnk", LONG_K_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_matmul_long_contraction_small_result(dev, mnk, misalign):
    m, n, k = mnk
    _say("long-k matmul", mnk, misalign)
    assert dev.fmatmul_plan(m, n, k)[0] == -1
    rng = np.random.default_rng(m * 17 + n * 1021 + k)
    o.set_threads(o.hw_threads())
    try:
        a = rng.integers(-3, 4, (m, k)).astype(np.float32)
        b = rng.integers(-3, 4, (k, n)).astype(np.float32)
        da, db = dev.array(a, misalign), dev.array(b, misalign)
        whole = dev.empty(m * n + 128, 0)
        dev.ffill(-7.0, whole, m * n + 128)
        lo = 64 + misalign
        dc = type(whole)(dev, m * n, whole.ptr, lo * 4)
        dev.fmatmul(False, False, da, db, dc, m, n, k)
        got = whole.download()
        assert np.array_equal(got[lo:lo + m * n].reshape(m, n), o.fmatmul(False, False, a, b))
        assert np.all(got[:lo] == -7.0) and np.all(got[lo + m * n:] == -7.0)
        first = got.copy()
        dev.fmatmul(False, False, da, db, dc, m, n, k)
        assert np.array_equal(whole.download(), first)                      # repeatable
        for t in (da, db, whole):
            t.free()
        a, b = parity.normal(rng, (m, k)), parity.normal(rng, (k, n))
        got = _matmul_device(dev, False, False, a, b, m, n, k)
        assert parity.frobenius_rel_error(got, o.fmatmul(False, False, a, b)) <= parity.MATMUL_FRO_REL
    finally:
        o.set_threads(1)


NARROW_SHAPES = [(256, 10, 784), (784, 10, 256), (10, 256, 784), (16, 1000, 333), (1000, 16, 16), (64, 1, 5000),
                 (65, 3, 4096), (70, 9, 4097), (5000, 7, 129), (8, 70000, 40), (70000, 5, 200), (300, 16, 17)]


@pytest.mark.parametrize("ta", [False, True])
@pytest.mark.parametrize("tb", [False, True])
@pytest.mark.parametrize("mnk", NARROW_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_matmul_narrow_result(dev, ta, tb, mnk):
    """One output dimension of at most 16 (a classifier's logits), either
    operand in the narrow role, contractions from 16 to 5000: the planner's
    small tiles and split-K plans.  Integer data (exact in any summation order)
    with misaligned bases and a guard region, then random data against the
    oracle."""
    m, n, k = mnk
    _say("narrow matmul", ta, tb, mnk)
    rng = np.random.default_rng(m * 11 + n * 1013 + k + 2 * ta + tb)
    sa, sb = parity.stored_shapes(ta, tb, m, n, k)
    o.set_threads(o.hw_threads())
    try:
        a = rng.integers(-4, 5, sa).astype(np.float32)
        b = rng.integers(-4, 5, sb).astype(np.float32)
        da, db, dc = dev.array(a, 1), dev.array(b, 3), dev.empty(m * n + 64, 2)
        dev.ffill(-7.0, dc, m * n + 64)
        dev.fmatmul(ta, tb, da, db, dc, m, n, k)
        got = dc.download()
        assert np.array_equal(got[:m * n].reshape(m, n), o.fmatmul(ta, tb, a, b))
        assert np.all(got[m * n:] == -7.0)                 # nothing written past the end
        for t in (da, db, dc):
            t.free()
        a, b = parity.normal(rng, sa), parity.normal(rng, sb)
        got = _matmul_device(dev, ta, tb, a, b, m, n, k)
        assert parity.frobenius_rel_error(got, o.fmatmul(ta, tb, a, b)) <= parity.MATMUL_FRO_REL
        assert np.array_equal(got, _matmul_device(dev, ta, tb, a, b, m, n, k))   # repeatable
    finally:
        o.set_threads(1)


SPLIT_K_SHAPES = [(33, 127, 4099), (33, 127, 65536), (256, 10, 784), (10, 256, 2051), (64, 64, 8192),
                  (130, 70, 3000), (1024, 1024, 4096)]


@pytest.mark.parametrize("ta", [False, True])
@pytest.mark.parametrize("tb", [False, True])
@pytest.mark.parametrize("mnk", SPLIT_K_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_matmul_long_k_is_split_and_reduced_in_order(dev, ta, tb, mnk):
    # few output tiles and a long K: the contraction is split along K and the
    # partial products are added in split order
    m, n, k = mnk
    _say("split-k matmul", ta, tb, mnk)
    o.set_threads(o.hw_threads())
    try:
        rng = np.random.default_rng(m + 3 * n + 5 * k + 2 * ta + tb)
        sa, sb = parity.stored_shapes(ta, tb, m, n, k)
        a, b = parity.normal(rng, sa), parity.normal(rng, sb)
        got = _matmul_device(dev, ta, tb, a, b, m, n, k)
        rows = (0, m) if m * n * k < 3e8 else (m // 2 - 4, m // 2 + 4)
        ref = o.fmatmul(ta, tb, a, b, rows=rows)
        assert parity.frobenius_rel_error(got[rows[0]:rows[1]], ref[rows[0]:rows[1]]) <= parity.MATMUL_FRO_REL
        again = _matmul_device(dev, ta, tb, a, b, m, n, k)
        assert np.array_equal(got, again)  # deterministic: no atomics, fixed reduction order
    finally:
        o.set_threads(1)


@pytest.mark.parametrize("ta", [False, True])
@pytest.mark.parametrize("tb", [False, True])
def test_matmul_split_count_never_leaves_an_empty_split(dev, ta, tb):
    """256 x 256 x 16384: the planner asks for 96 splits of 1024 k-steps, i.e. 11
    steps each, which only 94 splits can fill.  The operands are 16 MiB each,
    exactly what the pool hands out, so a split starting beyond K would read
    outside them."""
    m, n, k = 256, 256, 16384
    _say("split-k matmul without empty splits", ta, tb)
    rng = np.random.default_rng(77 + 2 * ta + tb)
    sa, sb = parity.stored_shapes(ta, tb, m, n, k)
    a, b = parity.normal(rng, sa), parity.normal(rng, sb)
    got = _matmul_device(dev, ta, tb, a, b, m, n, k)
    ref = (a.T if ta else a).astype(np.float64) @ (b.T if tb else b).astype(np.float64)
    assert parity.frobenius_rel_error(got, ref) <= 1e-5


def test_matmul_overwrites_output(dev):
    # no beta: C is overwritten, stale contents must not leak
    rng = np.random.default_rng(31)
    a, b = parity.normal(rng, (70, 40)), parity.normal(rng, (40, 50))
    da, db, dc = dev.array(a), dev.array(b), dev.array(np.full(70 * 50, 1e9, dtype=np.float32))
    dev.fmatmul(False, False, da, db, dc, 70, 50, 40)
    assert parity.frobenius_rel_error(dc.download((70, 50)), o.fmatmul(False, False, a, b)) <= parity.MATMUL_FRO_REL
    for x in (da, db, dc):
        x.free()


def test_transpose_matmul_cross_identity(dev):
    # matmul_t_f(A, B) == matmul_f_f(T(A), B) with integer data (exact)
    rng = np.random.default_rng(41)
    k, m, n = 77, 130, 45
    a = rng.integers(-8, 9, (k, m)).astype(np.float32)
    b = rng.integers(-8, 9, (k, n)).astype(np.float32)
    da, db, dat, c1, c2 = dev.array(a), dev.array(b), dev.empty(a.size), dev.empty(m * n), dev.empty(m * n)
    dev.ftranspose(da, dat, k, m)
    dev.fmatmul(True, False, da, db, c1, m, n, k)
    dev.fmatmul(False, False, dat, db, c2, m, n, k)
    assert np.array_equal(c1.download(), c2.download())
    for x in (da, db, dat, c1, c2):
        x.free()


def test_split_contraction_and_softmax_allocate_nothing(dev):
    """Calls that run more than one kernel (a matmul that splits the
    contraction, fsoftmax) work in the block the device holds since it was
    opened: the pool's counters do not move, first call included."""
    rng = np.random.default_rng(51)
    m, n, k = 300, 260, 40000      # 4 tiles of 256 x 256 at most: the contraction is split
    a = rng.integers(-3, 4, (m, k)).astype(np.float32)
    b = rng.integers(-3, 4, (k, n)).astype(np.float32)
    da, db, dc = dev.array(a), dev.array(b), dev.empty(m * n)
    dx, dy = dev.array(parity.normal(rng, 300000)), dev.empty(300000)
    dev.synchronize()
    s0 = dev.pool_stats()
    for _ in range(2):
        dev.fmatmul(False, False, da, db, dc, m, n, k)
        dev.fsoftmax(dx, dy)
    s1 = dev.pool_stats()
    assert (s1.device_allocs, s1.pool_hits, s1.bytes_in_use, s1.bytes_cached) == \
           (s0.device_allocs, s0.pool_hits, s0.bytes_in_use, s0.bytes_cached)
    ref = a.astype(np.float64) @ b.astype(np.float64)     # integers: exact in fp32
    assert np.array_equal(dc.download((m, n)), ref.astype(np.float32))
    for t in (da, db, dc, dx, dy):
        t.free()


@pytest.mark.parametrize("nbytes", [65536, 65536 + 4, 512 * 1024 + 12, 3 * 1024 * 1024 + 100,
                                    8 * 1024 * 1024, 9 * 1024 * 1024 + 20, 41 * 1024 * 1024 + 4])
@pytest.mark.parametrize("offset", [0, 4, 36])
def test_copy_to_host_into_unaligned_memory(dev, nbytes, offset):
    """Large read-backs are drained from the staging ring with streaming stores
    (aligned body, ordinary head and tail), from 8 MiB on by two host threads
    that take alternate chunks: every byte must arrive in place, and nothing
    outside the destination may change."""
    _say("copy_to_host", nbytes, offset)
    count = nbytes // 4
    src = (np.arange(count, dtype=np.int64) % 16000057).astype(np.float32)   # distinct per chunk position
    d = dev.array(src)
    guard = 64
    raw = np.full(nbytes + offset + 2 * guard, 0x5A, dtype=np.uint8)
    dst = raw[guard + offset: guard + offset + nbytes]
    dev.copy_to_host(dst.ctypes.data, d.ptr, nbytes)
    assert np.array_equal(dst.view(np.float32) if offset % 4 == 0 else np.frombuffer(dst.tobytes(), np.float32), src)
    assert np.all(raw[:guard + offset] == 0x5A) and np.all(raw[guard + offset + nbytes:] == 0x5A)
    d.free()


@pytest.mark.parametrize("nbytes", [4 * 1024 * 1024 + 8, 8 * 1024 * 1024, 10 * 1024 * 1024 + 4,
                                    13 * 1024 * 1024 + 36])
def test_copy_to_device_of_large_buffers_round_trips(dev, nbytes):
    """Uploads from 8 MiB on fill whole staging slots with two host threads; the
    source may be reused as soon as the call returns."""
    _say("copy_to_device", nbytes)
    count = nbytes // 4
    src = (np.arange(count, dtype=np.int64) % 16000057).astype(np.float32)
    keep = src.copy()
    d = dev.empty(count)
    dev.copy_to_device(d.ptr, src.ctypes.data, nbytes)
    src[:] = -1.0                      # the call has taken its copy
    assert np.array_equal(d.download(), keep)
    d.free()


@pytest.mark.parametrize("nbytes", [20, 4096 + 4, 3 * 1024 * 1024, 8 * 1024 * 1024, 9 * 1024 * 1024 + 12])
def test_copies_through_pinned_host_blocks(dev, nbytes):
    """A block of polar_hip_host_alloc is moved directly: an upload is queued when the call
    returns (quiesce before rewriting the block), a read-back is complete."""
    _say("host block", nbytes)
    count = nbytes // 4
    block = dev.host_alloc(nbytes + 64)
    try:
        host = np.ctypeslib.as_array(C.cast(block, C.POINTER(C.c_float)), shape=(count + 16,))
        d = dev.empty(count)
        for step in range(3):
            dev.host_quiesce(block)
            host[:count] = (np.arange(count, dtype=np.int64) % 16000057 + step).astype(np.float32)
            expect = host[:count].copy()
            dev.copy_to_device(d.ptr, block, nbytes)
            assert np.array_equal(d.download(), expect)          # pageable destination: staged
            dev.host_quiesce(block + 8)                            # any address inside the block
            host[:] = -1.0
            dev.copy_to_host(block + 16, d.ptr, nbytes)            # into the block, off its base
            assert np.array_equal(host[4:4 + count], expect)
            assert host[4 + count] == -1.0 and host[3] == -1.0
        d.free()
    finally:
        dev.host_free(block)


def test_pinned_host_block_calls_reject_foreign_pointers(dev):
    buf = np.zeros(16, dtype=np.float32)
    with pytest.raises(Exception):
        dev.host_free(buf.ctypes.data)
    with pytest.raises(Exception):
        dev.host_quiesce(buf.ctypes.data)
    dev.host_free(None)
    dev.host_quiesce(None)


@pytest.mark.parametrize("count", [5000, 150000, 262144])
def test_many_small_uploads_without_a_wait_between(dev, count):
    """More one- and two-slot uploads than the staging ring has slots, with no wait in between:
    a slot is only reused once the transfer out of it is over."""
    _say("small uploads", count)
    rng = np.random.default_rng(count)
    src = np.empty(count, dtype=np.float32)
    targets, expect = [], []
    for i in range(40):
        src[:] = rng.random(count, dtype=np.float32) + i
        expect.append(src.copy())
        d = dev.empty(count)
        dev.copy_to_device(d.ptr, src.ctypes.data, count * 4)
        targets.append(d)
        if i == 20:
            dev.record().synchronize()       # tells the library how far the stream has got
    for i, d in enumerate(targets):
        assert np.array_equal(d.download(), expect[i]), i
        d.free()


def test_pool_reuses_blocks(dev):
    dev.synchronize()
    s0 = dev.pool_stats()
    b = dev.empty(1 << 20)
    b.free()
    c = dev.empty(1 << 20)
    s1 = dev.pool_stats()
    c.free()
    assert s1.pool_hits >= s0.pool_hits + 1
    assert s1.device_allocs <= s0.device_allocs + 1


def test_events_order_and_time(dev):
    x = dev.empty(1 << 22)
    e0 = dev.record()
    dev.ffill(1.0, x)
    e1 = dev.record()
    e1.synchronize()
    assert e0.done() and e1.done()
    assert e0.elapsed_ms(e1) > 0
    e0.release(); e1.release(); x.free()


# ---- relu / softmax / conv2d / pool ---------------------------------------------

@pytest.mark.parametrize("n", SIZES)
@pytest.mark.parametrize("misalign", [0, 3])
def test_relu_bit_exact(dev, n, misalign):
    _say("relu n=", n, "misalign=", misalign)
    rng = np.random.default_rng(700 + n)
    x = parity.normal(rng, n)
    x[:: 7] = 0.0
    if n > 5:
        x[1], x[2], x[3] = np.nan, -np.inf, np.inf
    dx, dout = dev.array(x, misalign), dev.empty(n, misalign)
    dev.frelu(dx, dout)
    assert np.array_equal(dout.download(), o.frelu(x))
    dx.free(); dout.free()


@pytest.mark.parametrize("n", [1, 4, 1000, 65536, 65537, 200003])
def test_softmax_against_sequential_oracle(dev, n):
    """Sizes at which the reference's sequential fp32 sum is still accurate:
    1e-5 relative per element against it (tolerance of the parity contract)."""
    _say("softmax n=", n)
    rng = np.random.default_rng(800 + n)
    x = parity.normal(rng, n, std=1.5)
    for mis in (0, 1):
        dx, dout = dev.array(x, mis), dev.empty(n, mis)
        dev.fsoftmax(dx, dout)
        got = dout.download()
        assert parity.elementwise_rel_error(got, o.fsoftmax(x)) <= parity.ELEMENTWISE_REL
        assert parity.elementwise_rel_error(got, o.fsoftmax(x, f64sum=True)) <= 2e-6
        dx.free(); dout.free()


def test_softmax_sum_over_the_exponent_range(dev):
    """The sum pass has an exponential of its own: checked where that could
    differ from the library's -- arguments from deep underflow to just below
    overflow, with the total dominated by few large terms and by many small
    ones -- against the fp64-accumulated oracle."""
    rng = np.random.default_rng(811)
    n = 70001   # one full vector chunk and a ragged tail
    cases = {
        "wide": rng.uniform(-100.0, 80.0, n).astype(np.float32),
        "negative": rng.uniform(-103.0, -60.0, n).astype(np.float32),
        "near overflow": rng.uniform(70.0, 87.0, n).astype(np.float32),
        "small": (rng.standard_normal(n) * 1e-3).astype(np.float32),
    }
    cases["wide"][:5] = [0.0, -103.5, -104.5, 79.99, -0.0]
    for label, x in cases.items():
        _say("softmax range", label)
        dx, dout = dev.array(x), dev.empty(n)
        dev.fsoftmax(dx, dout)
        got = dout.download()
        ref = o.fsoftmax(x, f64sum=True)
        assert np.all(np.isfinite(got)), label
        assert parity.elementwise_rel_error(got, ref) <= 2e-6, label
        dx.free(); dout.free()


@pytest.mark.parametrize("special", [89.0, np.inf, np.nan, -np.inf])
def test_softmax_special_values_follow_the_reference(dev, special):
    """An argument whose exponential overflows makes the total infinite (finite
    terms become 0, the overflowing one inf/inf = NaN); a NaN makes everything
    NaN; -inf contributes 0.  Same pattern as the oracle's loop."""
    _say("softmax special", special)
    n = 65536 + 17
    x = parity.normal(np.random.default_rng(812), n)
    x[n // 2] = special
    x[n - 3] = special
    dx, dout = dev.array(x), dev.empty(n)
    dev.fsoftmax(dx, dout)
    got = dout.download()
    with np.errstate(all="ignore"):
        ref = o.fsoftmax(x, f64sum=True)
    assert np.array_equal(np.isnan(got), np.isnan(ref))
    keep = ~np.isnan(ref)
    assert parity.elementwise_rel_error(got[keep], ref[keep]) <= 2e-6
    dx.free(); dout.free()


def test_softmax_is_repeatable(dev):
    n = 3_000_001
    x = parity.normal(np.random.default_rng(9), n)
    dx, d1, d2 = dev.array(x), dev.empty(n), dev.empty(n)
    dev.fsoftmax(dx, d1)
    dev.fsoftmax(dx, d2)
    assert np.array_equal(d1.download(), d2.download())   # fixed summation order
    for b in (dx, d1, d2):
        b.free()


CONV_SHAPES = [((4, 4), (3, 3)), ((3, 3), (3, 3)), ((37, 53), (3, 3)), ((300, 1000), (5, 5)),
               ((129, 700), (7, 3)), ((64, 64), (1, 1)), ((1, 515), (1, 3)), ((515, 1), (3, 1)),
               ((40, 300), (23, 23)), ((100, 2049), (3, 5)), ((33, 289), (9, 1)),
               # rows on 16 bytes and several column segments: bands staged by vectors, interior segments
               # stored without bounds checks, ragged last band
               ((40, 1024), (3, 3)), ((25, 2052), (3, 3)), ((13, 600), (3, 3)), ((50, 1536), (5, 5))]


@pytest.mark.parametrize("shape,kshape", CONV_SHAPES)
def test_conv2d_bit_exact(dev, shape, kshape):
    _say("conv2d", shape, kshape)
    rng = np.random.default_rng(900 + shape[0] + kshape[1])
    x, w = parity.normal(rng, shape), parity.normal(rng, kshape)
    ref = o.fconv2d(x, w)
    for mis in (0, 5):     # output base at and off a 128-byte line
        dx, dw, dout = dev.array(x), dev.array(w), dev.empty(ref.size + 64, mis)
        dev.ffill(-7.0, dout)
        dev.fconv2d(dx, dw, dout, shape[0], shape[1], kshape[0], kshape[1])
        got = dout.download()
        assert np.array_equal(got[:ref.size].reshape(ref.shape), ref)
        assert np.all(got[ref.size:] == -7.0)          # nothing written past the end
        for b in (dx, dw, dout):
            b.free()


def test_conv2d_rejects_even_kernels_and_oversized(dev):
    from polarai_framework_amd import capi
    dx, dw, dout = dev.empty(64), dev.empty(16), dev.empty(64)
    with pytest.raises(capi.PolarHipError):
        dev.fconv2d(dx, dw, dout, 8, 8, 2, 2)
    with pytest.raises(capi.PolarHipError):
        dev.fconv2d(dx, dw, dout, 2, 2, 3, 3)
    for b in (dx, dw, dout):
        b.free()


POOL_CASES = [((4, 4), (2, 2), (2, 2)), ((100, 257), (2, 2), (2, 2)), ((101, 333), (3, 3), (2, 2)),
              ((50, 50), (3, 2), (1, 3)), ((64, 64), (64, 64), (1, 1)), ((9, 1000), (1, 1), (1, 1)),
              ((257, 1031), (2, 2), (2, 2)), ((16, 4100), (4, 4), (4, 4)), ((30, 30), (5, 5), (7, 7)),
              # even widths: the vector-load kernel for non-overlapping 2x2 / 4x4 windows, ragged edges
              ((101, 334), (2, 2), (2, 2)), ((37, 1030), (2, 2), (2, 2)), ((2, 2), (2, 2), (2, 2)),
              ((19, 6), (2, 2), (2, 2)), ((9, 516), (4, 4), (4, 4)), ((67, 2052), (4, 4), (4, 4)),
              # the staged kernel: overlapping windows, strides beyond the window, several column tiles and
              # bands, a ragged last band, widths around one segment; then windows too large for its LDS budget
              ((300, 1200), (3, 3), (1, 1)), ((133, 777), (2, 2), (1, 1)), ((200, 2100), (3, 3), (2, 2)),
              ((97, 1500), (5, 5), (2, 2)), ((64, 900), (2, 3), (4, 5)), ((41, 290), (3, 3), (3, 3)),
              ((40, 258), (7, 2), (1, 1)), ((300, 40), (3, 5), (2, 1)), ((13, 4000), (13, 1), (1, 2)),
              ((120, 600), (30, 30), (5, 5)), ((60, 700), (3, 200), (2, 100)),
              # the marching kernel (square windows of 4 and 5, stride 1 and 2, widths that are multiples of 4):
              # several waves across and bands down, an output width one past a wave's 220 columns, a ragged
              # last band, images smaller than one wave or one band
              ((300, 1200), (5, 5), (1, 1)), ((133, 776), (4, 4), (1, 1)), ((200, 2100), (4, 4), (2, 2)),
              ((70, 880), (5, 5), (2, 2)), ((31, 224), (4, 4), (1, 1)), ((45, 8), (5, 5), (1, 1)),
              ((1000, 4100), (5, 5), (1, 1)), ((1200, 1764), (5, 5), (2, 2)), ((5, 444), (5, 5), (2, 2)),
              ((9, 8), (4, 4), (2, 2))]


@pytest.mark.parametrize("shape,window,stride", POOL_CASES)
def test_pool_bit_exact(dev, shape, window, stride):
    _say("pool", shape, window, stride)
    rng = np.random.default_rng(1000 + shape[1])
    x = parity.normal(rng, shape)
    x[0, 0] = -3e6                                     # below the -10e5 floor
    ref = o.fpool(x, window, stride)
    # output at and off a line; input rows on 16 bytes (staged by vectors where the width allows) and off them
    for mis, mis_in in ((0, 0), (9, 0), (0, 3)):
        dx, dout = dev.array(x, mis_in), dev.empty(ref.size + 64, mis)
        dev.ffill(-7.0, dout)
        dev.fpool(dx, dout, shape[0], shape[1], window, stride)
        got = dout.download()
        assert np.array_equal(got[:ref.size].reshape(ref.shape), ref)
        assert np.all(got[ref.size:] == -7.0)
        dx.free(); dout.free()


@pytest.mark.parametrize("window,stride", [((2, 2), (2, 2)), ((3, 3), (1, 1)), ((5, 5), (2, 2)), ((4, 4), (1, 1)),
                                           ((3, 2), (1, 3))])
def test_pool_signed_zeros_and_nans_follow_the_reference_order(dev, window, stride):
    """The reference keeps the first of equal maxima (strictly greater replaces) and
    skips NaNs; which of +0 and -0 a window returns shows whether a kernel visits the
    taps in the reference's order.  Compared bit for bit."""
    _say("pool zeros/nans", window, stride)
    rng = np.random.default_rng(1050 + window[0] * 10 + stride[0])
    shape = (150, 1320)
    x = rng.choice(np.array([0.0, -0.0, -1.0, np.nan, -2e6], dtype=np.float32), size=shape,
                   p=[0.3, 0.3, 0.2, 0.1, 0.1]).astype(np.float32)
    ref = o.fpool(x, window, stride)
    dx, dout = dev.array(x), dev.empty(ref.size)
    dev.fpool(dx, dout, shape[0], shape[1], window, stride)
    got = dout.download().reshape(ref.shape)
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))
    assert np.signbit(ref).any() and (~np.signbit(ref)).any()   # both zeros do occur
    dx.free(); dout.free()


# ---- extended (fused) builtins ----------------------------------------------------

FUSED_SHAPES = [(256, 10, 784), (64, 64, 64), (33, 127, 4096), (300, 257, 129), (1024, 1024, 512), (5, 3, 0),
                (2050, 33, 127), (40, 1500, 30), (784, 10, 256), (12, 300, 100),
                # the kernels for a short contraction with one long dimension and for a long contraction with a
                # small result, and a split contraction added by the last group of a tile
                (65536, 33, 127), (65536, 127, 33), (33, 65536, 127), (70001, 17, 63), (33, 127, 65536),
                (16, 100, 20000), (50011, 81, 95), (768, 768, 768)]


@pytest.mark.parametrize("mnk", FUSED_SHAPES)
@pytest.mark.parametrize("ta", [False, True])
@pytest.mark.parametrize("tb", [False, True])
def test_fused_matmul_epilogues_equal_the_unfused_chain(dev, ta, tb, mnk):
    """fmatmul_fsigmoid / fmatmul_fadd_fsigmoid against running fmatmul, fadd and
    fsigmoid one after the other on the device (must be identical bit for bit, for
    plain and for split-K plans), and against the oracle's chain within the
    matmul tolerance."""
    m, n, k = mnk
    _say("fused matmul", ta, tb, mnk)
    rng = np.random.default_rng(1100 + m + k)
    sa, sb = parity.stored_shapes(ta, tb, m, n, max(k, 1))
    a, b = parity.normal(rng, sa, 0.3), parity.normal(rng, sb, 0.3)
    bias = parity.normal(rng, (m, n))
    da, db, dbias = dev.array(a), dev.array(b), dev.array(bias)
    prod, summed, chain, fused = dev.empty(m * n), dev.empty(m * n), dev.empty(m * n), dev.empty(m * n)
    dev.fmatmul(ta, tb, da, db, prod, m, n, k)
    # sigmoid(product)
    dev.fsigmoid(prod, chain)
    dev.fmatmul_fsigmoid(ta, tb, da, db, fused, m, n, k)
    assert np.array_equal(fused.download(), chain.download())
    # sigmoid(0.75 * product - 0.5 * bias)
    dev.fadd(prod, 0.75, dbias, -0.5, summed)
    dev.fsigmoid(summed, chain)
    dev.fmatmul_fadd_fsigmoid(ta, tb, da, db, 0.75, dbias, -0.5, fused, m, n, k)
    got = fused.download()
    assert np.array_equal(got, chain.download())
    if k > 0:
        ref = o.fsigmoid(o.fadd(o.fmatmul(ta, tb, a, b), 0.75, bias, -0.5))
        assert parity.frobenius_rel_error(got.reshape(m, n), ref) <= parity.MATMUL_FRO_REL
    else:
        assert np.array_equal(got.reshape(m, n), o.fsigmoid(o.fadd(np.zeros((m, n), np.float32), 0.75, bias, -0.5)))
    for t in (da, db, dbias, prod, summed, chain, fused):
        t.free()


@pytest.mark.parametrize("n", [1, 5, 1000, 65536 + 7, 1000003])
def test_fused_sigmoid_logloss_equals_the_unfused_chain(dev, n):
    _say("fused sigmoid+logloss n=", n)
    rng = np.random.default_rng(1200 + n)
    x = parity.normal(rng, n, 3.0)
    y = (rng.random(n) < 0.3).astype(np.float32)
    dx, dy, dp, chain, fused = dev.array(x), dev.array(y), dev.empty(n), dev.empty(n), dev.empty(n)
    dev.fsigmoid(dx, dp)
    dev.flogloss(dp, dy, chain)
    dev.fsigmoid_flogloss(dx, dy, fused)
    got = fused.download()
    assert np.array_equal(got, chain.download())
    # per kernel against the oracle, as for the unfused builtins: the sigmoid the
    # device produced, then the oracle's logloss of exactly those values (a chain of
    # two tolerances is not a tolerance: log(1 - p + eps) amplifies the last bit of p
    # where p saturates)
    p = dp.download()
    assert parity.elementwise_rel_error(p, o.fsigmoid(x)) <= parity.ELEMENTWISE_REL
    assert parity.elementwise_rel_error(got, o.flogloss(p, y)) <= parity.ELEMENTWISE_REL
    for t in (dx, dy, dp, chain, fused):
        t.free()
