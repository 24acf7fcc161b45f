"""Seeded random shapes for the kernels with index arithmetic (matmul in its four
layouts -- small shapes, and shapes with one long dimension --, transpose, conv2d,
pool): small enough for the oracle, awkward enough to
hit every edge path (sizes around the tile sizes, odd pitches, bases off a line).
Same bars as the fixed-shape tests: bit-exact for transpose/conv2d/pool, 1e-4
relative Frobenius for matmul."""
import os

import numpy as np
import pytest

import parity
import polar_oracle as o

pytestmark = pytest.mark.gpu

# more seeds for an occasional longer run: POLAR_RANDOM_SEEDS=10 multiplies the counts below
SCALE = int(os.environ.get("POLAR_RANDOM_SEEDS", "1"))


def _say(*a):
    print(*a, flush=True)


def _dims(rng, count, hi):
    """sizes biased towards tile boundaries"""
    special = np.array([1, 2, 3, 4, 5, 15, 16, 17, 31, 32, 33, 63, 64, 65, 127, 128, 129, 255, 256, 257])
    special = special[special <= hi]
    out = []
    for _ in range(count):
        out.append(int(rng.choice(special)) if rng.random() < 0.5 else int(rng.integers(1, hi + 1)))
    return out


@pytest.mark.parametrize("seed", range(40 * SCALE))
def test_random_matmul(dev, seed):
    rng = np.random.default_rng(5000 + seed)
    m, n = _dims(rng, 2, 300)
    k = _dims(rng, 1, 2500 if seed % 4 == 0 else 300)[0]
    ta, tb = bool(rng.integers(2)), bool(rng.integers(2))
    mis = int(rng.choice([0, 0, 1, 3]))
    _say("random matmul", seed, (m, n, k), ta, tb, "misalign", mis)
    sa, sb = parity.stored_shapes(ta, tb, m, n, k)
    a, b = parity.normal(rng, sa), parity.normal(rng, sb)
    da, db, dc = dev.array(a, mis), dev.array(b, mis), dev.empty(m * n + 32, mis)
    dev.ffill(-7.0, dc)
    dev.fmatmul(ta, tb, da, db, dc, m, n, k)
    got = dc.download()
    assert np.all(got[m * n:] == -7.0)
    assert parity.frobenius_rel_error(got[:m * n].reshape(m, n), o.fmatmul(ta, tb, a, b)) <= parity.MATMUL_FRO_REL
    for t in (da, db, dc):
        t.free()


@pytest.mark.parametrize("seed", range(36 * SCALE))
def test_random_matmul_with_one_long_dimension(dev, seed):
    """The kernels for a short contraction with a long M or N and for a long
    contraction with a small result, and whatever the dispatch passes on to the
    tiled kernel when a shape fits none of them.  Integer data: exact under any
    order of the additions."""
    rng = np.random.default_rng(5500 + seed)
    kind = seed % 3
    if kind == 0:
        m, n, k = int(rng.integers(40000, 90000)), _dims(rng, 1, 128)[0], _dims(rng, 1, 140)[0]
    elif kind == 1:
        m, n, k = _dims(rng, 1, 128)[0], int(rng.integers(40000, 90000)), _dims(rng, 1, 140)[0]
    else:
        m, n, k = _dims(rng, 1, 33)[0], _dims(rng, 1, 128)[0], int(rng.integers(16000, 90000))
    ta, tb = bool(rng.integers(2)), bool(rng.integers(2))
    mis_a, mis_b, mis_c = (int(rng.choice([0, 0, 1, 3])) for _ in range(3))
    _say("random long matmul", seed, (m, n, k), ta, tb, "misalign", (mis_a, mis_b, mis_c), "plan", dev.fmatmul_plan(m, n, k))
    sa, sb = parity.stored_shapes(ta, tb, m, n, k)
    a = rng.integers(-4, 5, sa).astype(np.float32)
    b = rng.integers(-4, 5, sb).astype(np.float32)
    da, db, dc = dev.array(a, mis_a), dev.array(b, mis_b), dev.empty(m * n + 32, mis_c)
    dev.ffill(-7.0, dc)
    dev.fmatmul(ta, tb, da, db, dc, m, n, k)
    got = dc.download()
    assert np.all(got[m * n:] == -7.0)
    assert np.array_equal(got[:m * n].reshape(m, n), o.fmatmul(ta, tb, a, b))
    for t in (da, db, dc):
        t.free()


@pytest.mark.parametrize("seed", range(30 * SCALE))
def test_random_transpose(dev, seed):
    rng = np.random.default_rng(6000 + seed)
    rows, cols = _dims(rng, 2, 900)
    mis = int(rng.choice([0, 1, 7]))
    _say("random transpose", seed, (rows, cols), "misalign", mis)
    x = parity.normal(rng, (rows, cols))
    dx, dt = dev.array(x, mis), dev.empty(x.size + 32, mis)
    dev.ffill(-7.0, dt)
    dev.ftranspose(dx, dt, rows, cols)
    got = dt.download()
    assert np.array_equal(got[:x.size].reshape(cols, rows), x.T)
    assert np.all(got[x.size:] == -7.0)
    dx.free(); dt.free()


@pytest.mark.parametrize("seed", range(30 * SCALE))
def test_random_conv2d_and_pool(dev, seed):
    rng = np.random.default_rng(7000 + seed)
    kh, kw = (int(rng.choice([1, 3, 5, 7, 9])) for _ in range(2))
    if seed % 5 == 0:
        kh = kw = int(rng.choice([3, 5]))             # the constant-geometry kernels
    h = kh - 1 + _dims(rng, 1, 120)[0]
    w = kw - 1 + _dims(rng, 1, 700)[0]
    mis = int(rng.choice([0, 5]))
    _say("random conv2d", seed, (h, w), (kh, kw), "misalign", mis)
    x, k = parity.normal(rng, (h, w)), parity.normal(rng, (kh, kw))
    ref = o.fconv2d(x, k)
    dx, dk, dout = dev.array(x), dev.array(k), dev.empty(ref.size + 32, mis)
    dev.ffill(-7.0, dout)
    dev.fconv2d(dx, dk, dout, h, w, kh, kw)
    got = dout.download()
    assert np.array_equal(got[:ref.size].reshape(ref.shape), ref)
    assert np.all(got[ref.size:] == -7.0)
    dout.free(); dk.free()

    win = (int(rng.integers(1, min(h, 5) + 1)), int(rng.integers(1, min(w, 5) + 1)))
    stride = (int(rng.integers(1, 5)), int(rng.integers(1, 5)))
    _say("random pool", seed, (h, w), win, stride)
    ref = o.fpool(x, win, stride)
    dout = dev.empty(ref.size + 32, mis)
    dev.ffill(-7.0, dout)
    dev.fpool(dx, dout, h, w, win, stride)
    got = dout.download()
    assert np.array_equal(got[:ref.size].reshape(ref.shape), ref)
    assert np.all(got[ref.size:] == -7.0)
    dx.free(); dout.free()


@pytest.mark.parametrize("seed", range(16 * SCALE))
def test_random_matmul_medium(dev, seed):
    """Sizes that reach the large tile configurations and the split-K plans; the
    reference is an fp64 library product (the oracle's sequential fp32 sum is within
    1e-5 of it at these sizes, and too slow to run for every case)."""
    rng = np.random.default_rng(8000 + seed)
    m, n = (int(rng.integers(200, 1600)) for _ in range(2))
    k = int(rng.integers(64, 3000))
    if seed % 3 == 0:
        m, n, k = (v // 4 * 4 for v in (m, n, k))        # the vector-fetch variants
    if seed % 5 == 0:
        m, n = (v // 256 * 256 + 256 for v in (m, n)); k = k // 32 * 32 + 32   # edge-free tiles
    ta, tb = bool(rng.integers(2)), bool(rng.integers(2))
    _say("random medium matmul", seed, (m, n, k), ta, tb)
    sa, sb = parity.stored_shapes(ta, tb, m, n, k)
    a, b = parity.normal(rng, sa), parity.normal(rng, sb)
    da, db, dc = dev.array(a), dev.array(b), dev.empty(m * n)
    dev.fmatmul(ta, tb, da, db, dc, m, n, k)
    got = dc.download((m, n))
    ref = (a.T if ta else a).astype(np.float64) @ (b.T if tb else b).astype(np.float64)
    assert parity.frobenius_rel_error(got, ref) <= 1e-5
    for t in (da, db, dc):
        t.free()


@pytest.mark.parametrize("seed", range(12 * SCALE))
def test_random_transpose_large(dev, seed):
    """Shapes with many interior strips and column tiles (the path without bounds checks), column
    tile counts that do not divide by eight (tiles shared between the XCDs), now and then a row
    count that numbers the strips in runs."""
    rng = np.random.default_rng(6500 + seed)
    rows = int(rng.integers(700, 6000)) if seed % 4 else int(rng.choice([8192, 10240]))
    cols = int(rng.integers(130, 2500))
    _say("random large transpose", seed, (rows, cols))
    x = (np.arange(rows * cols, dtype=np.int64) % 16000057).astype(np.float32).reshape(rows, cols)
    dx, dt = dev.array(x), dev.empty(x.size + 32)
    dev.ffill(-7.0, dt)
    dev.ftranspose(dx, dt, rows, cols)
    got = dt.download()
    assert np.array_equal(got[:x.size].reshape(cols, rows), x.T)
    assert np.all(got[x.size:] == -7.0)
    dx.free(); dt.free()


@pytest.mark.parametrize("seed", range(12 * SCALE))
def test_random_conv2d_and_pool_wide_rows_on_16_bytes(dev, seed):
    """Widths that are multiples of 4 and span several column segments: windows staged by vectors,
    interior segments stored without bounds checks, ragged last bands."""
    rng = np.random.default_rng(7500 + seed)
    kh = kw = int(rng.choice([3, 3, 5, 7]))
    h = int(rng.integers(kh, 90))
    w = 4 * int(rng.integers(130, 800))
    mis = int(rng.choice([0, 5]))
    _say("random wide conv2d", seed, (h, w), (kh, kw), "misalign", mis)
    x, k = parity.normal(rng, (h, w)), parity.normal(rng, (kh, kw))
    ref = o.fconv2d(x, k)
    dx, dk, dout = dev.array(x), dev.array(k), dev.empty(ref.size + 32, mis)
    dev.ffill(-7.0, dout)
    dev.fconv2d(dx, dk, dout, h, w, kh, kw)
    got = dout.download()
    assert np.array_equal(got[:ref.size].reshape(ref.shape), ref)
    assert np.all(got[ref.size:] == -7.0)
    dout.free(); dk.free()

    win = (int(rng.integers(2, min(h, 5) + 1)), int(rng.integers(2, 6)))
    stride = (int(rng.integers(1, 4)), int(rng.integers(1, 4)))
    _say("random wide pool", seed, (h, w), win, stride)
    ref = o.fpool(x, win, stride)
    dout = dev.empty(ref.size + 32, mis)
    dev.ffill(-7.0, dout)
    dev.fpool(dx, dout, h, w, win, stride)
    got = dout.download()
    assert np.array_equal(got[:ref.size].reshape(ref.shape), ref)
    assert np.all(got[ref.size:] == -7.0)
    dx.free(); dout.free()

