"""Tensors beyond 2^31 elements and 2^32 bytes: element offsets, flattened
extents and grid sizes must not wrap anywhere between the tree and the kernel.
The data is drawn on the device and checked window by window against numpy on
the host (no host array of the full size is ever made).  The file name sorts
behind the other suites: these tests move 5 GB through the device and run
last but for the allocation-free entry point's."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

ROWS, COLS = 70000, 32768           # 2,293,760,000 elements; 4.6 GB as fp16
STEP = 5000                         # rows per window brought to the host


def windows():
    for r0 in range(0, ROWS, STEP):
        yield r0, min(ROWS, r0 + STEP)


@pytest.fixture(scope="module")
def big(hip):
    free = hip.rt.props.hbm_bytes if hasattr(hip.rt.props, "hbm_bytes") else 0
    if free and free < 24 << 30:
        pytest.skip("needs 24 GB of device memory")
    x = hip.empty((ROWS, COLS), dtype=np.float16)
    x[:] = hip.rand() * 8.0 - 4.0
    yield x
    del x


def test_elementwise_over_more_than_2_to_31_elements(hip, big):
    x = big
    assert x.size > 2 ** 31 and x.nbytes > 2 ** 32
    y = hip.empty((ROWS, COLS), dtype=np.float16)
    col = hip.array(np.linspace(-1, 1, ROWS, dtype=np.float32).reshape(ROWS, 1))
    row = hip.array(np.linspace(0, 2, COLS, dtype=np.float32).reshape(1, COLS))
    y[:] = x * 0.5 + 1.0                                  # flattened to one dimension
    for r0, r1 in list(windows())[::3] + [(65530, 65540), (ROWS - 3, ROWS)]:
        want = (x[r0:r1].get().astype(np.float32) * np.float32(0.5) + np.float32(1.0)).astype(np.float16)
        assert np.array_equal(y[r0:r1].get(), want), (r0, r1)
    y[:] = x * col + row                                  # two-dimensional tile, both broadcasts
    ch, rh = col.get(), row.get()
    for r0, r1 in list(windows())[1::3] + [(65530, 65540), (ROWS - 3, ROWS)]:
        want = (x[r0:r1].get().astype(np.float32) * ch[r0:r1] + rh).astype(np.float16)
        assert np.array_equal(y[r0:r1].get(), want), (r0, r1)
    # a window that starts beyond the 4 GiB mark, as operand and as target
    y[:] = 0
    y[66000:66010] = x[69000:69010] * 2.0
    assert np.array_equal(y[66000:66010].get(), (x[69000:69010].get().astype(np.float32) * 2).astype(np.float16))
    assert not y[65990:66000].get().any() and not y[66010:66020].get().any()


def test_reductions_over_more_than_2_to_31_elements(hip, big):
    x = big
    cmax, camax = hip.empty((1, COLS)), hip.empty((1, COLS), dtype=np.int32)
    rsum, rmax = hip.empty((ROWS, 1)), hip.empty((ROWS, 1))
    cmax[:] = hip.max(x, axis=0)
    camax[:] = hip.argmax(x, axis=0)
    rsum[:] = hip.sum(x, axis=1)
    rmax[:] = hip.max(x, axis=1)
    total = hip.empty((1, 1))
    total[:] = hip.sum(x)
    want_cmax = np.full((1, COLS), -np.inf, np.float32)
    want_camax = np.zeros((1, COLS), np.int64)
    want_rsum = np.empty((ROWS, 1), np.float64)
    want_rmax = np.empty((ROWS, 1), np.float32)
    for r0, r1 in windows():
        w = x[r0:r1].get().astype(np.float32)
        m = w.max(axis=0, keepdims=True)
        a = w.argmax(axis=0).reshape(1, COLS) + r0
        better = m > want_cmax                           # first occurrence wins ties
        want_camax = np.where(better, a, want_camax)
        want_cmax = np.where(better, m, want_cmax)
        want_rsum[r0:r1] = w.sum(axis=1, dtype=np.float64, keepdims=True)
        want_rmax[r0:r1] = w.max(axis=1, keepdims=True)
    assert np.array_equal(cmax.get(), want_cmax)
    assert np.array_equal(camax.get(), want_camax.astype(np.int32))
    assert np.array_equal(rmax.get(), want_rmax)
    np.testing.assert_allclose(rsum.get(), want_rsum, rtol=1e-5, atol=0.05)
    np.testing.assert_allclose(total.get()[0, 0], want_rsum.sum(), rtol=1e-4, atol=50.0)


def test_softmax_down_the_columns_of_a_4_gib_matrix(hip, big):
    """axis-0 softmax, staged (reductions in one kernel, then the elementwise rest)"""
    x = big
    y = hip.empty((ROWS, COLS))         # fp32: the values (1e-5 and below) are denormals in fp16
    y[:] = hip.exp(x - hip.max(x, axis=0)) / hip.sum(hip.exp(x - hip.max(x, axis=0)), axis=0)
    m = np.full((1, COLS), -np.inf, np.float64)
    for r0, r1 in windows():
        m = np.maximum(m, x[r0:r1].get().astype(np.float64).max(axis=0, keepdims=True))
    s = np.zeros((1, COLS), np.float64)
    for r0, r1 in windows():
        s += np.exp(x[r0:r1].get().astype(np.float64) - m).sum(axis=0, keepdims=True)
    for r0, r1 in list(windows())[::4] + [(65530, 65540), (ROWS - 3, ROWS)]:
        want = np.exp(x[r0:r1].get().astype(np.float64) - m) / s
        got = y[r0:r1].get().astype(np.float64)
        assert np.max(np.abs(got - want) / np.maximum(want, 1e-3 * want.max())) < 1e-5, (r0, r1)
