"""polar_hip_fsoftmax_static: the softmax entry point that allocates nothing.
It must give what polar_hip_fsoftmax gives, bit for bit, on calls in a row that
share the library's scratch array (the second one smaller than the first), must
leave the pool untouched, and must reject sizes beyond its stated limit."""
import numpy as np
import pytest

import parity
import polar_oracle as o

pytestmark = pytest.mark.gpu


def _say(*a):
    print(*a, flush=True)


def test_static_softmax_matches_pool_softmax_on_consecutive_calls(dev):
    rng = np.random.default_rng(77)
    for n in (3 * 65536 + 1234, 65536 + 5, 1000003, 17):     # larger, then smaller, ...
        _say("fsoftmax_static n=", n)
        x = parity.uniform(rng, n, -3, 3)
        dx, want, got = dev.array(x), dev.empty(n), dev.empty(n)
        dev.fsoftmax(dx, want)
        before = dev.pool_stats()
        dev.fsoftmax_static(dx, got)
        after = dev.pool_stats()
        a, b = got.download(), want.download()
        assert np.array_equal(a, b)
        assert (after.device_allocs, after.pool_hits, after.bytes_in_use) == \
               (before.device_allocs, before.pool_hits, before.bytes_in_use)
        if n <= 100000:
            assert parity.elementwise_rel_error(a, o.fsoftmax(x)) <= parity.ELEMENTWISE_REL
        assert parity.elementwise_rel_error(a, o.fsoftmax(x, f64sum=True)) <= 2e-6
        for t in (dx, want, got):
            t.free()


def test_static_softmax_rejects_sizes_beyond_its_scratch(dev):
    _say("fsoftmax_static limit")
    d = dev.empty(16)
    with pytest.raises(Exception, match="exceed the limit"):
        dev.fsoftmax_static(d, d, n=(1 << 31) + 1)
    dev.fsoftmax_static(d, d, n=0)          # empty tensor: nothing to do
    d.free()
