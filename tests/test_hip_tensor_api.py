"""Corners of the tensor and backend API on the hip backend that the op-tree
tests do not reach: index forms, host copies of strided views, reshape /
share / set error paths, generator state, event marks, double-buffered input,
statement groups that cannot be one kernel.  Expected values are numpy's."""
import numpy as np
import pytest

from neon_amd.backends.backend import Block, OpTreeNode

pytestmark = pytest.mark.gpu


def test_index_forms_give_numpy_views(hip):
    rs = np.random.RandomState(0)
    a = rs.uniform(-1, 1, (12, 20)).astype(np.float32)
    x = hip.array(a)
    assert np.array_equal(x[-1].get(), a[-1:])                      # an int keeps its axis below three dims
    assert np.array_equal(x[:, -3].get(), a[:, -3:-2])
    assert np.array_equal(x[..., 2:7].get(), a[..., 2:7])
    assert np.array_equal(x[1:5, ...].get(), a[1:5, ...])
    assert np.array_equal(x[...].get(), a)
    assert np.array_equal(x[::2, 1::3].get(), a[::2, 1::3])         # packed on the device before the host copy
    assert np.array_equal(x.T.get(), a.T)
    assert np.array_equal(x[2:9, 3:11].T.get(), a[2:9, 3:11].T)
    assert np.array_equal(x[[3, 1, 7]].get(), a[[3, 1, 7]])
    assert np.array_equal(x[:, np.array([0, 19, 4], dtype=np.int32)].get(), a[:, [0, 19, 4]])
    b = rs.uniform(-1, 1, (3, 4, 5)).astype(np.float32)
    y = hip.array(b)
    assert y[1].shape == (4, 5) and np.array_equal(y[1].get(), b[1])     # three dims: an int drops its axis
    assert np.array_equal(y[..., 2].get(), b[..., 2])
    assert np.array_equal(y[-1, ..., 1:3].get(), b[-1, ..., 1:3])
    assert len(x) == 12 and int(x) == x.gpudata and x.raw() == x.gpudata and "HIPTensor" in str(x)
    for bad in (lambda: x[12], lambda: x[:, -21], lambda: x[..., ...], lambda: x["a"],
                lambda: x[[1, 2], [3, 4]], lambda: x[np.zeros((2, 2), np.int32)],
                lambda: x[hip.zeros((1, 2))], lambda: x[0, 0, 0]):
        with pytest.raises(IndexError):
            bad()
    # writes through a view land in the base
    x[-1] = 7.0
    x[..., 0:1] = -2.0
    a[-1] = 7.0
    a[:, 0:1] = -2.0
    assert np.array_equal(x.get(), a)


def test_reshape_share_set_and_their_errors(hip):
    a = np.arange(24, dtype=np.float32)
    x = hip.array(a.reshape(4, 6))
    assert x.reshape(24).shape == (24, 1) and np.array_equal(x.reshape(24).get()[:, 0], a)
    assert x.reshape(2, -1).shape == (2, 12) and x.reshape((3, 8)).shape == (3, 8)
    assert np.array_equal(x.reshape(2, 3, 4).get(), a.reshape(2, 3, 4))
    with pytest.raises(ValueError):
        x.reshape(5, 5)
    with pytest.raises(ValueError):
        x[:, 1:4].reshape(12, 1)                                    # strided rows cannot be merged
    with pytest.raises(TypeError):
        x[[0, 1]].reshape(12, 1)                                    # nor can a gather view be reshaped
    sh = x.share((2, 6))
    assert sh.gpudata == x.gpudata and np.array_equal(sh.get(), a[:12].reshape(2, 6))
    with pytest.raises(ValueError):
        x.share((5, 6))
    with pytest.raises(TypeError):
        x[:, 1:4].share((2, 2))
    with pytest.raises(TypeError):
        x.set(np.zeros(23, np.float32))
    with pytest.raises(TypeError):
        x[:] = "text"
    x.copy_from(a[::-1].astype(np.float64))                         # cast to the tensor's type on the way in
    assert np.array_equal(x.asnumpyarray().ravel(), a[::-1])
    t = hip.empty((6, 4))
    assert x.transpose().shape == (6, 4)
    x.transpose(out=t)
    assert np.array_equal(t.get(), x.get().T)
    with pytest.raises(TypeError):
        hip.empty((2, "3"))
    with pytest.raises(ValueError):
        type(hip)(default_dtype=np.float64)


def test_array_forms_and_fill_normal(hip):
    v = hip.array([1, 2, 3])                                        # one dim becomes a column
    assert v.shape == (3, 1) and np.array_equal(v.get()[:, 0], [1, 2, 3])
    h = hip.array(np.array([[1.5, -2.5]]), dtype=np.float16)
    assert h.dtype == np.float16 and np.array_equal(h.get(), np.array([[1.5, -2.5]], np.float16))
    big = hip.zeros((64, 300))
    hip.rng_reset()
    hip.fill_normal(big[:, 50:250], mean=3.0, stdv=0.5)             # a view: goes through a kernel, not a host copy
    got = big.get()
    assert not got[:, :50].any() and not got[:, 250:].any()
    assert abs(got[:, 50:250].mean() - 3.0) < 0.02 and abs(got[:, 50:250].std() - 0.5) < 0.02
    hip.rng_reset()
    dense = hip.empty((64, 200))
    hip.fill_normal(dense, mean=3.0, stdv=0.5)
    assert np.array_equal(dense.get(), got[:, 50:250])              # same host stream either way


def test_generator_state_round_trips(hip, cpu):
    out = hip.empty((128, 256))
    hip.rng_reset()
    state = hip.rng_get_state()
    out[:] = hip.rand()
    first, host_first = out.get(), hip.rng.uniform(size=4)
    out[:] = hip.rand()
    assert not np.array_equal(out.get(), first)
    hip.rng_set_state(state)
    out[:] = hip.rand()
    assert np.array_equal(out.get(), first) and np.array_equal(hip.rng.uniform(size=4), host_first)
    # a host-only state, as the CPU backend saves it: the device stream starts over
    cpu.rng_reset()
    hip.rng_set_state(cpu.rng_get_state())
    out[:] = hip.rand()
    assert np.array_equal(out.get(), first)
    assert np.array_equal(hip.rng.uniform(size=4), cpu.rng.uniform(size=4))
    hip.rng_reset()
    cpu.rng_reset()


def test_marks_time_the_work_between_them(hip):
    x = hip.array(np.ones((2048, 2048), np.float32))
    start, end = hip.init_mark(), hip.init_mark()
    hip.record_mark(start)
    for _ in range(20):
        x[:] = x * 1.0001
    hip.record_mark(end)
    hip.synchronize_mark(end)
    ms = hip.get_time(start, end)
    assert 0.0 < ms < 1000.0


def test_consume_double_buffers_host_batches(hip):
    host = [np.arange(12, dtype=np.float32).reshape(3, 4), -np.arange(12, dtype=np.float32).reshape(3, 4)]
    dev = [None, None]
    hip.consume(0, host, dev)
    hip.consume(1, host, dev)
    first = dev[0]
    host[0] = host[0] + 100
    hip.consume(0, host, dev)
    assert dev[0] is first                                          # allocated once, refilled afterwards
    assert np.array_equal(dev[0].get(), host[0]) and np.array_equal(dev[1].get(), host[1])
    with pytest.raises(AssertionError):
        hip.consume(2, host, dev)


def test_group_that_cannot_be_one_kernel_runs_statement_by_statement(hip):
    rs = np.random.RandomState(4)
    a = rs.uniform(-1, 1, (300, 200)).astype(np.float32)
    x = hip.array(a)
    down, across, both = hip.empty((1, 200)), hip.empty((300, 1)), hip.empty((300, 200))
    hip.begin(Block.update, 0)
    down[:] = hip.sum(x, axis=0)
    across[:] = hip.max(x, axis=1)
    both[:] = x - hip.mean(x, axis=1)
    hip.end(Block.update, 0)
    assert np.allclose(down.get(), a.sum(axis=0, keepdims=True), rtol=1e-5, atol=1e-4)
    assert np.array_equal(across.get(), a.max(axis=1, keepdims=True))
    assert np.allclose(both.get(), a - a.mean(axis=1, keepdims=True), rtol=1e-5, atol=1e-6)


def test_dot_of_mixed_storage_types_inside_a_tree(hip):
    rs = np.random.RandomState(5)
    a = rs.uniform(-1, 1, (40, 30)).astype(np.float16)
    b = rs.uniform(-1, 1, (30, 20)).astype(np.float32)
    out = hip.empty((40, 20))
    out[:] = hip.dot(hip.array(a, dtype=np.float16), hip.array(b)) + 1.0
    assert np.allclose(out.get(), a.astype(np.float64) @ b.astype(np.float64) + 1.0, rtol=1e-5, atol=1e-4)


def test_copy_transpose_axes_given_as_a_list(hip):
    rs = np.random.RandomState(6)
    a = rs.uniform(-1, 1, (3, 5, 7)).astype(np.float32)
    x, out = hip.array(a), hip.empty((7, 3, 5))
    hip.copy_transpose(x, out, axes=[2, 0, 1])
    assert np.array_equal(out.get(), a.transpose(2, 0, 1))
    assert isinstance(x[0].T, type(x)) and isinstance((x[0] * 2).T, OpTreeNode)


@pytest.mark.gpu
def test_bench_mode_reports_every_launch(caplog):
    """``bench=True``: events round every launch and one line per launch with
    time, bytes per second, shape, grid, block and the kernel's name
    (reference float_ew.py:917-938 prints `msecs shape blk,thd name`)"""
    import logging
    from neon_amd.backends import NervanaHIP
    from neon_amd.backends import nervanahip
    be = NervanaHIP(rng_seed=0, bench=True)
    try:
        x = be.array(np.arange(64 * 256, dtype=np.float32).reshape(64, 256))
        out, line = be.empty((64, 256)), be.empty((1, 256))
        with caplog.at_level(nervanahip.DISPLAY_LEVEL, logger=nervanahip.logger.name):
            caplog.clear()
            for _ in range(3):                    # repeated statements are timed too: nothing is replayed
                out[:] = x * 2.0 + 1.0
            line[:] = be.max(x, axis=0)
        lines = [r.getMessage() for r in caplog.records if r.levelno == nervanahip.DISPLAY_LEVEL]
        assert len(lines) == 4
        assert all("msecs" in l and "GB/s" in l and "shape(" in l and "grid(" in l and "blk(" in l for l in lines)
        assert "nk_ew_mul_add" in lines[0] and "_max_" in lines[3]
        np.testing.assert_array_equal(out.get(), np.arange(64 * 256, dtype=np.float32).reshape(64, 256) * 2.0 + 1.0)
        assert logging.getLevelName(nervanahip.DISPLAY_LEVEL) == "DISPLAY"
    finally:
        be.cleanup_backend()
