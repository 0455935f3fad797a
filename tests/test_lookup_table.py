"""Lookup table (embedding layer) on the backends: forward gather through
``take``, backward scatter-sum through ``compound_bprop_lut`` (reference
tests/test_lookuptable.py: exact gather, exact counts for all-ones errors,
random errors against explicit sums)."""
import numpy as np
import pytest

from utils import assert_close

def _lut_case(rs, vocab, embed, count, pad_idx=None):
    ids = rs.randint(0, vocab, size=count).astype(np.int32)
    if pad_idx is not None:
        ids[::7] = pad_idx
    W = rs.standard_normal((vocab, embed)).astype(np.float32)
    err = rs.random_sample((embed, count)).astype(np.float32)
    return ids, W, err


def _lut_bprop(be, ids, err, vocab, pad_idx, dtype=np.float32):
    embed, count = err.shape
    inputs = be.array(ids.reshape(1, -1), dtype=np.int32)
    dW = be.zeros((vocab, embed), dtype=dtype)
    dW[:] = 7.0                                  # rows of absent words must keep their contents
    error, error_t = be.array(err.astype(dtype), dtype=dtype), be.empty((count, embed), dtype=dtype)
    be.compound_bprop_lut(count, inputs, error, error_t, dW, pad_idx)
    return dW.get()


def _lut_expected(ids, err, vocab, pad_idx):
    want = np.full((vocab, err.shape[0]), 7.0, dtype=np.float64)
    for w in np.unique(ids):
        if w != pad_idx:
            want[w] = err[:, ids == w].astype(np.float64).sum(axis=1)
    return want


def test_lut_bprop_oracle_matches_brute_force(cpu):
    rs = np.random.RandomState(0)
    ids, W, err = _lut_case(rs, 50, 12, 300, pad_idx=3)
    got = _lut_bprop(cpu, ids, err, 50, 3)
    assert_close(got, _lut_expected(ids, err, 50, 3).astype(np.float32), rtol=1e-5, atol=1e-6)


@pytest.mark.gpu
@pytest.mark.parametrize("vocab,embed,count,pad", [(1000, 50, 128 * 10, None), (20, 64, 5000, 0), (10000, 300, 128 * 128, 5),
                                                   (7, 1, 33, None), (50000, 33, 1, None)])
def test_lookup_table_hip(pair, vocab, embed, count, pad):
    cpu, hip = pair
    rs = np.random.RandomState(vocab + count)
    ids, W, err = _lut_case(rs, vocab, embed, count, pad)
    # forward: outputs = W.take(ids, axis=0).T, exact
    Wd, idsd = hip.array(W), hip.array(ids.reshape(1, -1), dtype=np.int32)
    out_t, out = hip.empty((count, embed)), hip.empty((embed, count))
    out_t[:] = Wd.take(idsd, axis=0)
    out[:] = out_t.T
    assert np.array_equal(out.get(), W[ids].T)
    # backward against float64 sums and against the oracle
    want = _lut_expected(ids, err, vocab, pad)
    got = _lut_bprop(hip, ids, err, vocab, pad)
    assert_close(got, want.astype(np.float32), rtol=1e-5, atol=1e-5)
    assert_close(got, _lut_bprop(cpu, ids, err, vocab, pad), rtol=1e-5, atol=1e-5)
    # ones as errors: exact counts (reference test_lookuptable_ones_error)
    ones = _lut_bprop(hip, ids, np.ones_like(err), vocab, pad)
    counts = np.bincount(ids, minlength=vocab).astype(np.float32)
    for w in np.unique(ids):
        if w != pad:
            assert np.all(ones[w] == counts[w])
    # deterministic: the same bits on a second run
    assert np.array_equal(got, _lut_bprop(hip, ids, err, vocab, pad))


@pytest.mark.gpu
def test_lookup_table_fp16_hip(hip):
    rs = np.random.RandomState(4)
    ids, W, err = _lut_case(rs, 500, 40, 4000)
    got = _lut_bprop(hip, ids, err, 500, None, dtype=np.float16)
    want = _lut_expected(ids, err.astype(np.float16).astype(np.float32), 500, None)
    assert_close(got.astype(np.float32), want.astype(np.float32), rtol=2e-3, atol=1e-3)
