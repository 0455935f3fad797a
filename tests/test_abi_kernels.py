"""The prebuilt hand-written kernels, called straight through the C ABI
(ctypes -> libneonhip.so, raw device pointers) and checked against the oracle."""
import ctypes
from ctypes import byref, c_float, c_size_t, c_uint32, c_void_p

import numpy as np
import pytest

from neon_amd import configs
from neon_amd.backends.hip import runtime as hiprt
from utils import assert_close, rel_err

pytestmark = pytest.mark.gpu


class Dev(object):
    """device buffers through nh_malloc / nh_memcpy only"""

    def __init__(self, rt):
        self.rt, self.lib, self.ptrs = rt, rt.lib, []

    def put(self, a):
        a = np.ascontiguousarray(a)
        p = self.rt.malloc(max(a.nbytes, 4))
        self.rt.memcpy_h2d(p, a)
        self.ptrs.append(p)
        return p

    def alloc(self, nbytes):
        p = self.rt.malloc(max(nbytes, 4))
        self.ptrs.append(p)
        return p

    def get(self, p, shape, dtype):
        out = np.empty(shape, dtype)
        self.rt.memcpy_d2h(out, p)
        return out

    def free(self):
        for p in self.ptrs:
            self.rt.free(p)
        self.ptrs = []


@pytest.fixture()
def dev(hip):
    d = Dev(hip.rt)
    yield d
    hip.rt.synchronize()
    d.free()


def ok(lib, rc):
    assert rc == 0, lib.nh_last_error()


@pytest.mark.parametrize("n", [1, 1023, 4096 * 128, 3 * 1000 * 1000 + 1])
def test_ew_entry_points(dev, cpu, n):
    rs = np.random.RandomState(n % 97)
    x = rs.standard_normal(n).astype(np.float32)
    y = rs.standard_normal(n).astype(np.float32)
    dx, dy, do = dev.put(x), dev.put(y), dev.alloc(4 * n)
    ok(dev.lib, dev.lib.nh_ew_axpby_f32(do, dx, dy, 0.5, 2.0, n, None))
    got = dev.get(do, (n,), np.float32)
    tx, ty, out = cpu.array(x.reshape(1, n)), cpu.array(y.reshape(1, n)), cpu.empty((1, n))
    configs.c1a(cpu, out, tx, ty)
    assert_close(got, out.get().ravel(), rtol=1e-6)
    ok(dev.lib, dev.lib.nh_ew_sigmoid_f32(do, do, n, None))
    configs.c1b(cpu, out)
    assert_close(dev.get(do, (n,), np.float32), out.get().ravel(), rtol=1e-5)


@pytest.mark.parametrize("n", [257, 1000 * 1250])
def test_adam_entry_point(dev, cpu, n):
    rs = np.random.RandomState(3)
    g = (rs.standard_normal(n) * 1e-2).astype(np.float32)
    p = (rs.standard_normal(n) * 0.05).astype(np.float32)
    dg, dp = dev.put(g), dev.put(p)
    dm, dv = dev.put(np.zeros(n, np.float32)), dev.put(np.zeros(n, np.float32))
    cpu_bsz, cpu.bsz = cpu.bsz, 1
    tg, tp = cpu.array(g.reshape(1, n)), cpu.array(p.reshape(1, n))
    tm, tv = cpu.zeros((1, n)), cpu.zeros((1, n))
    lr, b1, b2, eps = 1e-3, 0.9, 0.999, 1e-8
    for t in range(1, 4):
        l = lr * np.sqrt(1 - b2 ** t) / (1 - b1 ** t)
        ok(dev.lib, dev.lib.nh_adam_step_f32(dp, dm, dv, dg, l, b1, 1. - b1, b2, 1. - b2, eps, n, None))
        configs.c3_adam_step(cpu, tp, tg, tm, tv, t)
    cpu.bsz = cpu_bsz
    assert_close(dev.get(dp, (n,), np.float32), tp.get().ravel(), rtol=1e-5, atol=1e-12, what="param")
    assert_close(dev.get(dm, (n,), np.float32), tm.get().ravel(), rtol=1e-5, atol=1e-12, what="m")
    assert_close(dev.get(dv, (n,), np.float32), tv.get().ravel(), rtol=1e-5, atol=1e-14, what="v")


@pytest.mark.parametrize("shape", [(5, 8), (7, 8192 + 64), (16, 100352)])
def test_rownorm_entry_point(dev, cpu, shape):
    x, gamma, beta = configs.inputs_c4(shape)
    dx, dgam, dbet = dev.put(x), dev.put(gamma), dev.put(beta)
    do = dev.alloc(2 * x.size)
    ok(dev.lib, dev.lib.nh_rownorm_f16(do, dx, dgam, dbet, 1e-5, shape[0], shape[1], shape[1], None))
    got = dev.get(do, shape, np.float16).astype(np.float64)
    o = cpu.empty(shape, dtype=np.float16)
    configs.c4_rownorm(cpu, o, cpu.array(x.astype(np.float32)), cpu.array(gamma), cpu.array(beta))
    assert rel_err(got, o.get().astype(np.float64), floor_frac=1e-3) <= 1e-3
    # argument validation happens on the host
    assert dev.lib.nh_rownorm_f16(do, dx, dgam, dbet, 1e-5, shape[0], shape[1] - 1, shape[1], None) == hiprt.NH_EINVAL
    assert dev.lib.nh_rownorm_f16(do, dx, dgam, dbet, 1e-5, 1, (1 << 17) + 8, 1 << 18, None) == hiprt.NH_EINVAL


@pytest.mark.parametrize("shape", [(3, 5), (1000, 128), (4000, 256), (32000, 256), (700, 1030)])
def test_colmax_argmax_entry_point(dev, shape):
    rs = np.random.RandomState(shape[0])
    x = np.round(rs.standard_normal(shape) * 4.0, 1).astype(np.float32)      # rounding makes ties likely
    dx = dev.put(x)
    dmax, darg = dev.alloc(4 * shape[1]), dev.alloc(4 * shape[1])
    ws = dev.alloc(dev.lib.nh_colreduce_workspace_bytes(shape[0], shape[1]))
    for _ in range(2):       # twice: the ticket counters must have reset themselves
        ok(dev.lib, dev.lib.nh_colmax_argmax_f32(dmax, darg, dx, shape[0], shape[1], shape[1], ws, None))
        assert np.array_equal(dev.get(dmax, (shape[1],), np.float32), x.max(axis=0))
        assert np.array_equal(dev.get(darg, (shape[1],), np.int32), x.argmax(axis=0))
    assert dev.lib.nh_colmax_argmax_f32(None, None, dx, shape[0], shape[1], shape[1], ws, None) == hiprt.NH_EINVAL


def test_launch_validation(hip):
    lib = hip.rt.lib
    grid = (c_uint32 * 3)(1, 1, 1)
    block = (c_uint32 * 3)(2048, 1, 1)
    assert lib.nh_launch(None, grid, block, 0, None, None, 0) == hiprt.NH_EINVAL
    p = c_void_p()
    assert lib.nh_malloc(byref(p), 0) == hiprt.NH_EINVAL
    assert lib.nh_malloc(byref(p), c_size_t(1 << 60)) != 0          # far beyond device memory
    assert b"exceeds" in lib.nh_last_error()


@pytest.mark.parametrize("nbins,offset", [(64, -48), (100, -60), (256, -130), (7, -3)])
@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["f32", "f16"])
@pytest.mark.parametrize("n,skew", [(1, 0), (4099, 0), (1 << 20, 0), (3 * 1000 * 1000 + 5, 1),
                                    (5 * 1000 * 1000 + 3, 0), (5 * 1000 * 1000 + 3, 1)])
def test_hist_log2_entry_point(dev, n, skew, dtype, nbins, offset):
    """both counting schemes (private counters up to 64 bins, wave-agreed bins
    beyond), vector body and scalar tail, aligned and unaligned start, against
    numpy's histogram of rint(log2|x|) (the binning of nervanacpu.py:424-445)"""
    rs = np.random.RandomState(n % 89 + nbins)
    # magnitudes 2^(k + f), |f| <= 0.4: rint(log2|x|) = k whatever the last bit of log2f
    lo, hi = (-20, 8) if dtype == np.float32 else (-12, 8)
    a = (np.exp2(rs.randint(lo, hi, size=n + skew) + rs.uniform(-0.4, 0.4, size=n + skew)) *
         rs.choice([-1.0, 1.0], size=n + skew)).astype(dtype)
    a[rs.randint(0, n + skew, size=min(n, 5))] = 0
    if n > 16:
        a[3], a[7], a[11] = np.nan, np.inf, -np.inf
    base = dev.put(a)
    x = base + skew * a.dtype.itemsize               # skew: not 16-byte aligned
    hist = dev.alloc(4 * nbins)
    ok(dev.lib, dev.lib.nh_hist_log2(c_void_p(hist), c_void_p(x), a.dtype.itemsize, n, nbins, offset, None))
    got = dev.get(hist, (nbins,), np.int32)
    edges = np.arange(nbins + 1) + float(offset)
    edges[0] = -np.inf
    with np.errstate(divide="ignore", invalid="ignore"):
        want, _ = np.histogram(np.rint(np.log2(np.abs(a[skew:].astype(np.float32)))), bins=edges)
    assert np.array_equal(got, want.astype(np.int32))


@pytest.mark.parametrize("nbins,offset,shift", [(64, -48, 0), (63, -126, 0), (7, -3, 0), (64, 63, 0), (64, -48, 4),
                                                 (5, -2, 4), (64, 64, 0), (40, -127, 0)])
def test_hist_log2_bin_edges(dev, nbins, offset, shift):
    """the values whose bin the last bit decides: the two fp32 neighbours of
    sqrt(2) * 2^k (the lower rounds down, the upper up), exact powers of two,
    the largest and smallest normal numbers, denormals, zeros, infinities and
    NaNs -- against rint(log2|x|) evaluated in float64, which separates the
    neighbours of sqrt(2) by 10^8 of its own roundings.  Covers the kernel that
    bins by exponent and mantissa, the two argument ranges that must fall back
    to the logarithm kernels, an odd number of bins and a result buffer that is
    only 4-byte aligned (no paired adds)."""
    ks = np.arange(-126, 128)
    below = (np.float32(np.sqrt(2.0)) * np.exp2(ks)).astype(np.float32)         # 0x3FB504F3 * 2^k < sqrt(2) * 2^k
    above = np.nextafter(below, np.float32(np.inf)).astype(np.float32)
    assert np.all(below.astype(np.float64) < np.sqrt(2.0) * np.exp2(ks.astype(np.float64)))
    specials = np.array([0.0, -0.0, 1e-45, 1e-40, -1e-39, 1.1754942e-38, 1.17549435e-38, 3.4028235e38, -3.4028235e38,
                         np.inf, -np.inf, np.nan, -np.nan], dtype=np.float32)
    quiet = np.array([0x7fc00000, 0xffc00001, 0x7f800001, 0x7fffffff], dtype=np.uint32).view(np.float32)
    a = np.concatenate([below, -above, np.exp2(ks).astype(np.float32), specials, quiet,
                        np.random.RandomState(3).randn(4096).astype(np.float32)]).astype(np.float32)
    a = np.tile(a, 3)[:-5]                                                       # a scalar tail as well
    x = dev.put(a)
    base = dev.alloc(4 * nbins + 16)
    hist = base + shift
    ok(dev.lib, dev.lib.nh_hist_log2(c_void_p(hist), c_void_p(x), 4, a.size, nbins, offset, None))
    got = dev.get(hist, (nbins,), np.int32)
    with np.errstate(divide="ignore", invalid="ignore"):
        b = np.rint(np.log2(np.abs(a.astype(np.float64)))) - offset
    counted = b <= nbins                                                          # false for NaN
    bins = np.clip(np.where(counted, b, 0), 0, nbins - 1).astype(np.int64)
    want = np.bincount(bins[counted], minlength=nbins)
    assert np.array_equal(got, want.astype(np.int32))
