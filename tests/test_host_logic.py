"""Host-side pieces that need no GPU: the seeded generator and the API mirror's
argument handling."""
import numpy as np

from framework_amd import synth


def test_synth_is_deterministic_and_seed_dependent():
    a = synth.normal(1, (64, 64))
    assert np.array_equal(a, synth.normal(1, (64, 64)))
    assert not np.array_equal(a, synth.normal(2, (64, 64)))
    assert not np.array_equal(a, synth.normal(1, (64, 64), stream=1))
    assert a.dtype == np.float32


def test_synth_distributions():
    n = synth.normal(3, (1 << 16,))
    assert abs(float(n.mean())) < 0.02 and abs(float(n.std()) - 1.0) < 0.02
    u = synth.uniform(4, (1 << 16,))
    assert u.min() >= 0.0 and u.max() < 1.0 and abs(float(u.mean()) - 0.5) < 0.01
    k = synth.integers(5, (1 << 12,), 0, 3)
    assert set(np.unique(k)) == {0, 1, 2}
    s = synth.small_ints(6, (1000,), 3)
    assert s.min() >= -3 and s.max() <= 3 and np.array_equal(s, np.round(s))


def test_synth_prefix_property():
    # element i depends only on (seed, stream, i): a larger draw extends a smaller one
    assert np.array_equal(synth.normal(9, (100,)), synth.normal(9, (1000,))[:100])


def test_adam_defaults_and_number_arguments(orc):
    T = orc.Tensor
    x = T.fromFloat32([1, 2], [2])
    assert list(x.mul(3).toFloat32()) == [3, 6]
    assert list(x.sub(1).toFloat32()) == [0, 1]
    opt = orc.Adam([])
    assert (opt.lr, opt.beta2) == (6e-4, 0.95)  # src/optimizer.ts:46-56
