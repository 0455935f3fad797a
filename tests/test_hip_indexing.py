"""Gather / scatter views inside op-trees and the log2 histogram (GPU box).

The reference reaches these through ``tensor.take`` / fancy ``__getitem__``
(nervanagpu.py:230-260, 460-476; argument kinds in1/in2/out1/out2 of
cuda_templates.py:448-483) and ``tensor.hist`` (float_ew.py:1070-1158).
Expected values come from numpy fancy indexing and from the oracle.
"""
import numpy as np
import pytest

from utils import assert_close, gen_inputs

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("shape,n", [((50, 128), 77), ((1000, 64), 4096), ((7, 9), 3)])
def test_gather_rows_and_columns(hip, shape, n):
    rs = np.random.RandomState(n)
    w = gen_inputs(rs, shape)
    be = hip
    tw = be.array(w)
    ri = rs.randint(0, shape[0], n).astype(np.int32)
    ci = rs.randint(0, shape[1], n).astype(np.int32)
    # lookup-table forward: rows of W selected by an index vector
    out = be.empty((n, shape[1]))
    out[:] = tw.take(be.array(ri.reshape(1, n), dtype=np.int32), axis=0)
    assert np.array_equal(out.get(), w[ri, :])
    # the same through __getitem__ with a host index list, inside a larger tree
    out[:] = tw[ri.tolist()] * 2.0 + 1.0
    assert_close(out.get(), w[ri, :] * 2.0 + 1.0, rtol=1e-6)
    # columns
    outc = be.empty((shape[0], n))
    outc[:] = be.take(tw, be.array(ci.reshape(n, 1), dtype=np.int32), axis=1) - 0.5
    assert_close(outc.get(), w[:, ci] - 0.5, rtol=1e-6)
    # gathered operand feeding a reduction
    red = be.empty((1, shape[1]))
    red[:] = be.max(tw[ri.tolist()], axis=0)
    assert np.array_equal(red.get().ravel(), w[ri, :].max(axis=0))


def test_scatter_through_index_view(hip):
    rs = np.random.RandomState(5)
    be = hip
    w = np.zeros((40, 33), dtype=np.float32)
    tw = be.array(w)
    rows = rs.permutation(40)[:12].astype(np.int32)          # distinct targets: no write conflicts
    src = gen_inputs(rs, (12, 33))
    tw[rows.tolist()] = be.array(src) * 3.0
    w[rows, :] = src * 3.0
    assert_close(tw.get(), w, rtol=1e-6)
    cols = rs.permutation(33)[:5].astype(np.int32)
    tw[:, cols.tolist()] = 7.0
    w[:, cols] = 7.0
    assert_close(tw.get(), w, rtol=1e-6)


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("shape", [(1, 1), (64, 327), (2048, 512)])
def test_hist_matches_oracle(pair, shape, dtype):
    cpu, hip = pair
    rs = np.random.RandomState(shape[1])
    a = (rs.standard_normal(shape) * np.exp2(rs.randint(-60, 20, shape))).astype(np.float32)
    a.ravel()[:: 7] = 0.0                       # zeros land in the lowest bin
    a = a.astype(dtype)
    res = []
    for be in (cpu, hip):
        t = be.array(a, dtype=dtype)
        h = t.hist("w")
        res.append(h.get().copy())
    assert res[0].shape == res[1].shape == (1, 64)
    assert np.array_equal(res[1], res[0])
    assert res[1].sum() <= a.size
    # non-contiguous view goes through a packed copy
    if shape[1] > 4:
        v = hip.array(a, dtype=dtype)[:, 1:4]
        hv = v.hist("view").get()
        want = cpu.array(a[:, 1:4].copy(), dtype=dtype).hist("view").get()
        assert np.array_equal(hv, want)
    data, tags = hip.dump_hist_data()
    assert "w" in tags and data.shape[1] == 64



def test_single_index_gather_and_scatter(hip):
    """a gather view of exactly one row / column still goes through its index"""
    rs = np.random.RandomState(12)
    w = rs.standard_normal((40, 9)).astype(np.float32)
    W = hip.array(w)
    one = hip.array(np.array([[17]], dtype=np.int32), dtype=np.int32)
    col = hip.array(np.array([[5]], dtype=np.int32), dtype=np.int32)
    row_out, col_out = hip.empty((1, 9)), hip.empty((40, 1))
    row_out[:] = W.take(one, axis=0) * 2.0
    col_out[:] = W.take(col, axis=1) + 1.0
    assert np.array_equal(row_out.get(), w[17:18] * 2.0)
    assert np.array_equal(col_out.get(), w[:, 5:6] + 1.0)
    W[one] = row_out                                   # scatter into the single indexed row
    w[17] = w[17] * 2.0
    assert np.array_equal(W.get(), w)
