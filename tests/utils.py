"""Helpers shared by the tests (modelled on the reference's tests/utils.py:47-225)."""
import numpy as np


def rel_err(got, want, floor_frac=0.0):
    """max |got-want| / max(|want|, floor_frac*max|want|)"""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    denom = np.abs(want)
    if floor_frac:
        denom = np.maximum(denom, floor_frac * np.abs(want).max())
    denom = np.where(denom == 0, 1.0, denom)
    return float(np.max(np.abs(got - want) / denom)) if got.size else 0.0


def assert_close(got, want, rtol=1e-5, atol=1e-6, what=""):
    got, want = np.asarray(got), np.asarray(want)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    if want.dtype.kind in "iub":
        assert np.array_equal(got, want), what
        return
    bad = ~np.isclose(got.astype(np.float64), want.astype(np.float64), rtol=rtol, atol=atol, equal_nan=True)
    if bad.any():
        i = np.argmax(np.abs(got.astype(np.float64) - want.astype(np.float64)) * bad)
        raise AssertionError("%s: %d/%d mismatches; worst got %r want %r" % (
            what, int(bad.sum()), bad.size, got.reshape(-1)[i], want.reshape(-1)[i]))


def gen_inputs(rs, shape, flag="rand", dtype=np.float32):
    """Same kinds of test tensors as the reference's gen_backend_tensors
    (tests/utils.py:160-225)."""
    if flag == "zeros":
        x = np.zeros(shape)
    elif flag == "pos_ones":
        x = np.ones(shape)
    elif flag == "neg_ones":
        x = -np.ones(shape)
    elif flag == "pos_rand":
        x = rs.rand(*shape)
    elif flag == "neg_rand":
        x = -rs.rand(*shape)
    else:
        x = -1 + 2 * rs.rand(*shape)
    return x.astype(dtype)


def call_func(f, be, arrays, out_dtype=None):
    """Evaluate f(be, *tensors) into a tensor of the tree's shape and fetch it
    (reference tests/utils.py:85-103)."""
    tensors = [be.array(a, dtype=a.dtype) for a in arrays]
    tree = f(be, *tensors)
    out = be.empty(tree.shape, dtype=out_dtype or np.float32)
    out[:] = tree
    return out.get()
