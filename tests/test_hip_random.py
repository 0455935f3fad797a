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


# ---- stochastic rounding of stores (tensor.rounding = mantissa bits) --------------------------

def _on_grid(values, bits):
    """every value has at most `bits` mantissa bits set"""
    b = np.asarray(values, dtype=np.float32).view(np.uint32)
    return bool(np.all((b & np.uint32((1 << (23 - bits)) - 1)) == 0))


def test_sr_one_bit_fp16(hip):
    """reference tests/test_backend_sr.py test_sr: 1 + 0.1 stored with one
    mantissa bit is 1.0 or 1.5, mostly 1.0"""
    n = 10
    A = hip.ones((n, n), dtype=np.float16)
    B = hip.ones((n, n), dtype=np.float16)
    hip.multiply(B, 0.1, out=B)
    C = hip.ones((n, n), dtype=np.float16)
    C.rounding = 1
    C[:] = A + B
    got = C.get().ravel()
    assert np.all((got == 1.0) | (got == 1.5))
    assert (got == 1.5).sum() > .1 * n ** 2
    assert (got == 1.0).sum() > .7 * n ** 2


@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["f32", "f16"])
@pytest.mark.parametrize("bits", [1, 3, 8, True])
def test_sr_unbiased_neighbours(hip, dtype, bits):
    rs = np.random.RandomState(11)
    rows, cols = 64, 8192
    x = ((0.25 + rs.rand(rows, 1)) * np.where(rs.rand(rows, 1) < 0.5, -1, 1)).astype(np.float32)
    X = hip.array(x)
    out = hip.empty((rows, cols), dtype=dtype)
    out.rounding = bits
    out[:] = X + hip.zeros((1, cols))                      # each row: one value, 8192 draws
    got = out.get().astype(np.float32)
    m = 10 if bits is True else bits
    assert _on_grid(got, m)
    ulp = 2.0 ** (np.floor(np.log2(np.abs(x))) - m)
    lo = np.trunc(x / ulp) * ulp                           # neighbour toward zero
    hi = lo + np.sign(x) * ulp
    assert np.all((got == lo) | (got == hi))
    # unbiased: the mean over many draws approaches the value (5 sigma of a
    # two-point distribution with spread ulp)
    err = np.abs(got.astype(np.float64).mean(axis=1, keepdims=True) - x)
    assert np.all(err <= 5 * 0.5 * ulp / np.sqrt(cols) + 1e-7)


@pytest.mark.parametrize("dtype", [np.int32, np.int16, np.int8], ids=["i32", "i16", "i8"])
def test_sr_into_integer_tensors_is_unbiased(hip, dtype):
    """stores into signed integer tensors with ``rounding`` set go to one of the
    two neighbouring whole numbers, the farther one from zero with probability
    equal to the fraction (reference cuda_templates.py:236-286); whole numbers
    stay as they are"""
    rs = np.random.RandomState(12)
    rows, cols = 64, 8192
    x = (rs.rand(rows, 1) * 100.0 * np.where(rs.rand(rows, 1) < 0.5, -1, 1)).astype(np.float32)
    x[:4, 0] = [3.0, -7.0, 0.0, 99.0]
    out = hip.empty((rows, cols), dtype=dtype)
    out.rounding = True
    out[:] = hip.array(x) + hip.zeros((1, cols))           # each row: one value, 8192 draws
    got = out.get().astype(np.float64)
    lo = np.trunc(x)
    hi = lo + np.sign(x) * (x != lo)
    assert np.all((got == lo) | (got == hi))
    assert np.all(got[:4] == x[:4])
    err = np.abs(got.mean(axis=1, keepdims=True) - x)
    assert np.all(err <= 5 * 0.5 / np.sqrt(cols) + 1e-6)
    # without the attribute the store truncates, as the CPU backend's cast does
    plain = hip.empty((rows, cols), dtype=dtype)
    plain[:] = hip.array(x) + hip.zeros((1, cols))
    assert np.array_equal(plain.get(), np.broadcast_to(np.trunc(x), (rows, cols)).astype(dtype))


def test_sr_leaves_representable_values_and_specials(hip):
    x = np.array([[0.0, 1.0, -2.5, 0.75, np.inf, -np.inf, np.nan, 1024.0]], dtype=np.float32)
    out = hip.empty(x.shape, dtype=np.float32)
    out.rounding = 2
    out[:] = hip.array(x) * 1.0
    got = out.get()
    assert np.array_equal(got[:, :4], x[:, :4])
    assert got[0, 4] == np.inf and got[0, 5] == -np.inf and np.isnan(got[0, 6]) and got[0, 7] == 1024.0


def test_sr_fresh_draws_each_time_and_reproducible_state(hip):
    x = hip.array(np.full((64, 256), 1.3, dtype=np.float32))
    out = hip.empty((64, 256), dtype=np.float16)
    out.rounding = 2
    state = hip.rng_get_state()
    out[:] = x * 1.0
    first = out.get()
    out[:] = x * 1.0
    second = out.get()
    assert not np.array_equal(first, second)               # not a replay of the first launch
    hip.rng_set_state(state)
    out[:] = x * 1.0
    assert np.array_equal(out.get(), first)


def test_sr_reduced_output_and_fused_group(hip):
    rs = np.random.RandomState(2)
    x = rs.rand(128, 300).astype(np.float32)
    X = hip.array(x)
    sums = hip.empty((128, 1), dtype=np.float32)
    sums.rounding = 4
    sums[:] = hip.sum(X, axis=1)                           # staged: reduce, then round while copying
    got = sums.get()
    want = x.astype(np.float64).sum(axis=1, keepdims=True)
    assert _on_grid(got, 4)
    assert np.all(np.abs(got - want) <= 2.0 ** (np.floor(np.log2(want)) - 4) * 1.001)
    # inside a fused group: the rounded tensor feeds the next statement rounded
    a = hip.empty((128, 300), dtype=np.float16)
    a.rounding = 3
    b = hip.empty((128, 300), dtype=np.float32)
    with hip.fused():
        a[:] = X * 1.0
        b[:] = a * 2.0
    assert _on_grid(a.get().astype(np.float32), 3)
    assert np.array_equal(b.get(), a.get().astype(np.float32) * 2.0)
