"""Device random numbers (GPU box): ``be.rand()`` inside op-trees, dropout
masks, and generator state handling.  The generator is not the reference's
LFSR pool, so values cannot be compared with it; the checks are the ones the
reference's own tests make (tests/test_backend_randomstate.py:22-73, 150-178):
reproducibility after ``rng_reset`` / with the same seed / after restoring a
saved state, plus distribution statistics."""
import numpy as np
import pytest

from neon_amd.backends.backend import Backend

pytestmark = pytest.mark.gpu


def test_uniform_statistics(hip):
    be = hip
    be.rng_reset()
    out = be.empty((1000, 1024))
    be.rand(out=out)
    u = out.get().astype(np.float64)
    assert u.min() >= 0.0 and u.max() < 1.0
    n = u.size
    assert abs(u.mean() - 0.5) < 5 / np.sqrt(12 * n)
    assert abs(u.var() - 1 / 12.0) < 1e-3
    # no visible structure along either axis and between neighbours
    assert abs(np.corrcoef(u[:, :-1].ravel(), u[:, 1:].ravel())[0, 1]) < 5e-3
    assert abs(np.corrcoef(u[:-1, :].ravel(), u[1:, :].ravel())[0, 1]) < 5e-3
    hist, _ = np.histogram(u, bins=64, range=(0, 1))
    chi2 = ((hist - n / 64.0) ** 2 / (n / 64.0)).sum()
    assert chi2 < 64 + 6 * np.sqrt(2 * 64)          # 63 dof: mean 63, sd ~11


@pytest.mark.parametrize("keep", [0.1, 0.5, 0.8])
def test_binary_mask_fraction(hip, keep):
    be = hip
    out = be.empty((512, 640))
    be.make_binary_mask(out, keepthresh=keep)
    m = out.get()
    assert set(np.unique(m)).issubset({0.0, 1.0})
    assert abs(m.mean() - keep) < 5 * np.sqrt(keep * (1 - keep) / m.size)
    # fp16 destination and a tree that mixes the mask with data
    x = be.ones((512, 640), dtype=np.float16)
    x[:] = x * be.dropout(keep=keep) * (1.0 / keep)
    v = x.get().astype(np.float32)
    assert abs(v.mean() - 1.0) < 0.02 / keep


def test_reproducibility(hip):
    """same seed / rng_reset / restored state give identical streams; successive
    calls differ (reference tests/test_backend_randomstate.py:22-73, 150-178)"""
    be = hip
    a, b, c = be.empty((64, 100)), be.empty((64, 100)), be.empty((64, 100))
    be.rng_reset()
    be.make_binary_mask(a, 0.5)
    be.make_binary_mask(b, 0.5)
    host1 = be.rng.rand(4)
    assert not np.array_equal(a.get(), b.get())
    be.rng_reset()
    be.make_binary_mask(c, 0.5)
    assert np.array_equal(a.get(), c.get())
    assert np.array_equal(host1, be.rng.rand(4))
    state = be.rng_get_state()
    be.rand(out=b)
    first = b.get()
    be.rand(out=b)
    be.rng_set_state(state)
    be.rand(out=c)
    assert np.array_equal(first, c.get())
    # another backend object with the same seed draws the same numbers
    other = Backend.allocate_backend("hip", rng_seed=0)
    o = other.empty((64, 100))
    other.make_binary_mask(o, 0.5)
    assert np.array_equal(o.get(), a.get())
    two = other.empty((64, 100))
    two[:] = other.rand() - other.rand()          # two streams in one kernel are independent
    d = two.get()
    assert abs(d.mean()) < 0.02 and 0.1 < d.var() < 0.25
    be.fill_normal(a, mean=2.0, stdv=0.5)
    assert abs(a.get().mean() - 2.0) < 0.05
