"""The entry point that allocates nothing (``nh_colmax_argmax_f32_static``: its
partials and tickets live in a static device array) against the entry point
that takes a caller's workspace, through the C ABI, on two calls in a row --
the second on a smaller matrix, so that what the first left in the shared
scratch area is still there."""
import numpy as np
import pytest

from neon_amd.backends.hip import runtime as hiprt

pytestmark = pytest.mark.gpu


def _both(rt, x):
    lib = rt.lib
    rows, cols = x.shape
    dx = rt.malloc(x.nbytes)
    rt.memcpy_h2d(dx, np.ascontiguousarray(x))
    outs = [rt.malloc(4 * cols) for _ in range(4)]
    ws = rt.malloc(lib.nh_colreduce_workspace_bytes(rows, cols))
    try:
        rc = lib.nh_colmax_argmax_f32(outs[0], outs[1], dx, rows, cols, cols, ws, None)
        assert rc == 0, lib.nh_last_error()
        rc = lib.nh_colmax_argmax_f32_static(outs[2], outs[3], dx, rows, cols, cols, None)
        assert rc == 0, lib.nh_last_error()
        got = []
        for p, dt in zip(outs, (np.float32, np.int32, np.float32, np.int32)):
            h = np.empty(cols, dt)
            rt.memcpy_d2h(h, p)
            got.append(h)
        return got
    finally:
        rt.synchronize()
        for p in outs + [dx, ws]:
            rt.free(p)


def test_static_scratch_entry_point_matches_the_workspace_one(hip):
    rt = hip.rt
    rs = np.random.RandomState(77)
    # (32000,256): 32 row chunks per strip; then (6000,96): fewer strips and chunks over the same
    # scratch; then a row length that is not a multiple of four (the one-element-per-lane variant)
    for shape in ((32000, 256), (6000, 96), (5000, 131), (3, 5)):
        x = np.round(rs.standard_normal(shape) * 4.0, 1).astype(np.float32)      # rounding makes ties likely
        x[shape[0] // 2, 1] = np.nan
        vmax, imax, vmax_s, imax_s = _both(rt, x)
        assert np.array_equal(imax_s, imax) and np.array_equal(imax, x.argmax(axis=0).astype(np.int32))
        assert np.array_equal(vmax_s, vmax, equal_nan=True) and np.array_equal(vmax, x.max(axis=0), equal_nan=True)


def test_static_scratch_entry_point_refuses_what_does_not_fit(hip):
    rt, lib = hip.rt, hip.rt.lib
    rows, cols = 9000, 8190           # row length not a multiple of four: 16 chunks x 8190 columns x 8 bytes > the 768 KiB behind the tickets
    dx = rt.malloc(rows * cols * 4)
    out = rt.malloc(4 * cols)
    try:
        rc = lib.nh_colmax_argmax_f32_static(out, None, dx, rows, cols, cols, None)
        assert rc == hiprt.NH_EINVAL and b"scratch" in lib.nh_last_error()
        assert lib.nh_colmax_argmax_f32_static(None, None, dx, 10, 10, 10, None) == hiprt.NH_EINVAL
        assert lib.nh_colmax_argmax_f32_static(out, None, dx, 10, 10, 5, None) == hiprt.NH_EINVAL
    finally:
        rt.free(dx)
        rt.free(out)
