"""Parity of the hip backend against the CPU oracle (runs on the GPU box).

Every case evaluates the same function on both backends from identical seeded
inputs.  Tolerances: integer / index outputs bit-exact; fp32 1e-5 relative;
fp16 storage 1e-3 relative.
"""
import numpy as np
import pytest

from neon_amd import configs
from utils import assert_close, call_func, gen_inputs, rel_err

pytestmark = pytest.mark.gpu

RTOL32 = 1e-5


def both(pair, f, arrays, out_dtype=None, rtol=RTOL32, atol=1e-6, what=""):
    cpu, hip = pair
    want = call_func(f, cpu, arrays, out_dtype)
    got = call_func(f, hip, arrays, out_dtype)
    assert_close(got, want, rtol=rtol, atol=atol, what=what)
    return got, want


# ---- elementwise ------------------------------------------------------------------------
UNARY = ["neg", "abs", "sgn", "sqr", "exp", "exp2", "sig", "sig2", "tanh", "tanh2", "rint"]
UNARY_POS = ["sqrt", "log", "log2", "safelog"]


@pytest.mark.parametrize("shape", [(64, 327), (4, 3), (1, 1023), (64, 1), (4096, 128)])
def test_unary_ops(pair, shape):
    rs = np.random.RandomState(1)
    x = gen_inputs(rs, shape) * 3
    xp = gen_inputs(rs, shape, "pos_rand") + 0.01
    table = dict(neg="negative", abs="absolute", sgn="sgn", sqr="square", exp="exp", exp2="exp2",
                 sig="sig", sig2="sig2", tanh="tanh", tanh2="tanh2", rint="rint", sqrt="sqrt",
                 log="log", log2="log2", safelog="safelog")
    for op in UNARY:
        both(pair, lambda be, a, op=op: getattr(be, table[op])(a), [x], what=op)
    for op in UNARY_POS:
        both(pair, lambda be, a, op=op: getattr(be, table[op])(a), [xp], what=op)


@pytest.mark.parametrize("shapes", [((64, 327), (64, 327)), ((64, 327), (64, 1)), ((64, 327), (1, 327)),
                                    ((64, 1), (1, 327)), ((4, 3), (1, 1)), ((1, 1023), (1, 1023))])
def test_binary_ops_and_broadcast(pair, shapes):
    rs = np.random.RandomState(2)
    a = gen_inputs(rs, shapes[0])
    b = gen_inputs(rs, shapes[1]) + 1.5
    fns = {
        "add": lambda be, x, y: x + y, "sub": lambda be, x, y: x - y,
        "mul": lambda be, x, y: x * y, "div": lambda be, x, y: x / y,
        "gt": lambda be, x, y: x > y, "ge": lambda be, x, y: x >= y,
        "lt": lambda be, x, y: x < y, "le": lambda be, x, y: x <= y,
        "eq": lambda be, x, y: be.equal(x, y), "ne": lambda be, x, y: be.not_equal(x, y),
        "max": lambda be, x, y: be.maximum(x, y), "min": lambda be, x, y: be.minimum(x, y),
        "pow": lambda be, x, y: be.power(be.absolute(x) + 0.1, y),
        "scalar": lambda be, x, y: 0.5 * x + 2.0 * y - 3 + x / 4.0,
        "clip": lambda be, x, y: be.clip(x, -0.25, 0.5) * y,
    }
    for name, f in fns.items():
        both(pair, f, [a, b], what=name)


def test_numbers_on_either_side_of_an_operator(pair):
    """the same backend evaluates each form right after its mirror image: they
    differ only in the side the number stands on, and must not share a kernel"""
    rs = np.random.RandomState(21)
    a = gen_inputs(rs, (300, 512)) * 0.4 + 0.5
    forms = {
        "x-c": lambda be, x: x - 1.0, "c-x": lambda be, x: 1.0 - x,
        "x/c": lambda be, x: x / 2.0, "c/x": lambda be, x: 2.0 / x,
        "x>c": lambda be, x: x > 0.5, "c>x": lambda be, x: 0.5 > x,
        "x<=c": lambda be, x: x <= 0.5, "c<=x": lambda be, x: 0.5 <= x,
        "x**c": lambda be, x: be.power(be.absolute(x), 2.5), "c**x": lambda be, x: be.power(2.5, x),
        "c/(x-c)": lambda be, x: 1.0 / (x - 3.0), "c/(c-x)": lambda be, x: 1.0 / (3.0 - x),
        "sum(x-c)": lambda be, x: be.sum(x - 1.0, axis=0) + 0 * x, "sum(c-x)": lambda be, x: be.sum(1.0 - x, axis=0) + 0 * x,
        "max(x/c)": lambda be, x: be.max(x / 3.0, axis=1) + 0 * x, "max(c/x)": lambda be, x: be.max(3.0 / x, axis=1) + 0 * x,
    }
    for _ in range(2):              # the second pass runs from the launch cache
        for name, f in forms.items():
            both(pair, f, [a], what=name, atol=1e-5)


def test_onehot_along_rows_in_vector_tiles(pair):
    """onehot(idx, axis=1): one hot column per row, on tiles several elements wide"""
    rs = np.random.RandomState(22)
    R, C = 512, 1024
    x = gen_inputs(rs, (R, C))
    idx = rs.randint(0, C, size=(R, 1)).astype(np.int32)
    res = []
    for be in pair:
        t, out, picked = be.array(x), be.empty((R, C)), be.empty((R, 1))
        hot = be.onehot(be.array(idx, dtype=np.int32), axis=1)
        out[:] = hot * t + 0.5 * t
        picked[:] = be.sum(hot * t, axis=1)
        res.append((out.get(), picked.get()))
    want = x * 0.5
    want[np.arange(R), idx[:, 0]] += x[np.arange(R), idx[:, 0]]
    assert_close(res[1][0], want, what="onehot axis 1")
    assert np.array_equal(res[1][1][:, 0], x[np.arange(R), idx[:, 0]])
    assert_close(res[1][0], res[0][0])
    assert_close(res[1][1], res[0][1])


@pytest.mark.parametrize("shape,axis", [((300, 4096), 1), ((16, 300000), 1), ((2000, 384), 0), ((40000, 64), 0),
                                        ((200000, 16), 0), ((64, 96), 0), ((64, 96), 1)])
def test_index_reductions_broadcast_into_full_tensors(pair, shape, axis):
    """argmax / argmin stored straight into a tensor of the operand's shape
    (every row or column repeats the index), float and int32"""
    rs = np.random.RandomState(23)
    x = gen_inputs(rs, shape)
    res = []
    for be in pair:
        t = be.array(x)
        fo, io = be.empty(shape), be.empty(shape, dtype=np.int32)
        fo[:] = be.argmax(t, axis=axis)
        io[:] = be.argmin(t, axis=axis)
        res.append((fo.get(), io.get()))
    assert np.array_equal(res[1][0], np.broadcast_to(x.argmax(axis=axis, keepdims=True), shape).astype(np.float32))
    assert np.array_equal(res[1][1], np.broadcast_to(x.argmin(axis=axis, keepdims=True), shape).astype(np.int32))
    assert np.array_equal(res[1][0], res[0][0]) and np.array_equal(res[1][1], res[0][1])


def test_reductions_of_operands_that_do_not_vary_along_the_axis(pair):
    """a (1,C) operand reduced down the rows, a (R,1) operand reduced along the
    columns: value reductions return the operand (times the extent for sum),
    index reductions return zero"""
    rs = np.random.RandomState(24)
    R, C = 300, 2000
    x, row, col = gen_inputs(rs, (R, C)), gen_inputs(rs, (1, C)), gen_inputs(rs, (R, 1))
    fns = {
        "argmax row": lambda be, a, r, c: a + be.argmax(r * 2.0, axis=0),
        "argmin col": lambda be, a, r, c: a - be.argmin(c + 1.0, axis=1),
        "max row": lambda be, a, r, c: a * be.max(r, axis=0),
        "min col": lambda be, a, r, c: a * be.min(c, axis=1),
        "argmax alone": lambda be, a, r, c: be.argmax(r, axis=0) + 0 * r,
    }
    for name, f in fns.items():
        both(pair, f, [x, row, col], what=name)


def test_group_with_a_column_shaped_and_a_full_output(pair):
    """one statement of the group writes a (R,1) tensor, the other a (R,C) one:
    the narrow store happens once per row"""
    from neon_amd.backends.backend import Block
    rs = np.random.RandomState(25)
    R, C = 257, 1000
    x, col = gen_inputs(rs, (R, C)), gen_inputs(rs, (R, 1))
    res = []
    for be in pair:
        t, c = be.array(x), be.array(col)
        narrow, full = be.empty((R, 1)), be.empty((R, C))
        be.begin(Block.update, 0)
        narrow[:] = c * 2.0 + 1.0
        full[:] = t + c
        be.end(Block.update, 0)
        res.append((narrow.get(), full.get()))
    assert_close(res[1][0], col * 2.0 + 1.0)
    assert_close(res[1][1], x + col)
    assert_close(res[1][0], res[0][0])
    assert_close(res[1][1], res[0][1])


def test_inplace_and_views(pair):
    rs = np.random.RandomState(3)
    a = gen_inputs(rs, (50, 128))
    b = gen_inputs(rs, (50, 128))
    outs = []
    for be in pair:
        x, y = be.array(a), be.array(b)
        x[:] = be.sig(x)                       # in place
        x[2:7, :] = y[10:15, :] * 2.0          # row-slice views
        x[:, 3:9] = x[:, 3:9] + y[:, 20:26]    # column-slice views, strided
        x[0] = y[1] - 1.0                      # int index keeps the axis
        x[:, 5] = 7.5                          # constant into a strided view
        z = be.empty((128, 50))
        z[:] = x.T + 1.0                       # transposed view as operand
        w = x.reshape((100, 64))
        w[:] = w * 0.5
        outs.append((x.get(), z.get()))
    assert_close(outs[1][0], outs[0][0], what="x")
    assert_close(outs[1][1], outs[0][1], what="z")


@pytest.mark.parametrize("dtype", [np.float16, np.int32, np.uint8, np.int8, np.int16, np.uint16, np.uint32])
def test_storage_dtypes(pair, dtype):
    rs = np.random.RandomState(4)
    if np.dtype(dtype).kind == "f":
        a = (rs.rand(33, 40) * 4 - 2).astype(dtype)
    else:
        a = rs.randint(0, 100, (33, 40)).astype(dtype)
    b = (rs.rand(33, 40) * 3).astype(np.float32)
    outs = []
    for be in pair:
        x = be.array(a, dtype=dtype)
        y = be.array(b)
        if np.dtype(dtype).kind == "f":
            # fp16 storage, fp32 arithmetic: the oracle holds the same values in fp32
            x32 = be.array(a.astype(np.float32)) if be.backend_name == "cpu" else x
            o = be.empty((33, 40), dtype=dtype)
            o[:] = x32 * y + 0.25
        else:
            o = be.empty((33, 40), dtype=dtype)
            o[:] = x + y                       # float -> int store truncates
        outs.append(o.get())
    if np.dtype(dtype).kind == "f":
        assert rel_err(outs[1], outs[0]) <= 1e-3
    else:
        assert np.array_equal(outs[1], outs[0])


# ---- reductions ---------------------------------------------------------------------------
RED_SHAPES = [(2, 2), (10, 32), (50, 50), (50, 128), (1000, 128), (257, 1000), (3, 5000), (5000, 3)]


@pytest.mark.parametrize("shape", RED_SHAPES)
@pytest.mark.parametrize("axis", [0, 1])
def test_reductions(pair, shape, axis):
    rs = np.random.RandomState(5)
    a = gen_inputs(rs, shape)
    # A sum of n terms carries an fp32 rounding error of about eps * sum|x| in
    # either evaluation order (numpy adds rows one after the other along axis
    # 0, the device adds a tree), so near-zero results are compared with that
    # absolute allowance on top of the 1e-5 relative one.
    atol = 2 * np.finfo(np.float32).eps * float(np.abs(a).sum(axis=axis).max())
    for name in ("sum", "max", "min", "mean", "var", "std"):
        both(pair, lambda be, x, n=name: getattr(be, n)(x, axis=axis), [a], rtol=RTOL32, atol=atol,
             what="%s axis%d" % (name, axis))
    for name in ("argmax", "argmin"):
        got, want = both(pair, lambda be, x, n=name: getattr(be, n)(x, axis=axis), [a],
                         out_dtype=np.int32, what=name)


@pytest.mark.parametrize("axis", [0, 1])
def test_argmax_ties_take_first(pair, axis):
    a = np.zeros((37, 41), dtype=np.float32)
    a[5, :] = 1
    a[9, :] = 1
    a[:, 7] = 1
    a[:, 30] = 1
    both(pair, lambda be, x: be.argmax(x, axis=axis), [a], out_dtype=np.int32)
    both(pair, lambda be, x: be.argmin(-x, axis=axis), [a], out_dtype=np.int32)


@pytest.mark.parametrize("shape", [(10, 32), (50, 128), (300, 70)])
def test_reduction_into_slices(pair, shape):
    """reductions written through row / column views (reference
    tests/test_backend_reduction.py:39-43, 59-63)"""
    rs = np.random.RandomState(6)
    a = gen_inputs(rs, shape)
    outs = []
    for be in pair:
        x = be.array(a)
        r = be.zeros((4, shape[1]))
        c = be.zeros((shape[0], 4))
        r[1] = be.sum(x, axis=0)
        r[2, :] = be.max(x, axis=0) + be.min(x, axis=0)
        c[:, 1] = be.mean(x, axis=1)
        c[:, 3] = be.std(x, axis=1)
        outs.append((r.get(), c.get()))
    assert_close(outs[1][0], outs[0][0], rtol=2e-5, what="rows")
    assert_close(outs[1][1], outs[0][1], rtol=2e-5, what="cols")


def test_compound_and_mixed_axes(pair):
    """whole-tensor reductions and nested mixed-axis trees need several kernels"""
    rs = np.random.RandomState(7)
    a = gen_inputs(rs, (50, 128))
    b = gen_inputs(rs, (50, 128))
    both(pair, lambda be, x, y: be.sum(x), [a, b], rtol=2e-5)
    both(pair, lambda be, x, y: be.mean(x * y), [a, b], rtol=2e-5, atol=1e-6)
    both(pair, lambda be, x, y: be.std(be.var(x, axis=0), axis=1), [a, b], rtol=5e-5)
    both(pair, lambda be, x, y: be.max(x) + be.min(y), [a, b])
    # row sums of 128 terms of size ~1 carry ~1e-5 absolute fp32 error in either order
    both(pair, lambda be, x, y: x - be.mean(x) + be.sum(y, axis=1), [a, b], rtol=RTOL32, atol=2e-5)
    both(pair, lambda be, x, y: (x * y).T + 1.0, [a, b])


@pytest.mark.parametrize("axis", [0, 1])
@pytest.mark.parametrize("shape", [(1000, 4096), (333, 130), (32000, 256), (256, 3000)])
def test_values_that_take_the_place_of_a_resident_operand(pair, shape, axis):
    """softmax keeps exp(x - max) in x's registers; variants that read x again
    afterwards, or two operands of which one is reused, must not be disturbed
    by that"""
    rs = np.random.RandomState(shape[0])
    a = (rs.standard_normal(shape) * 2).astype(np.float32)
    b = rs.standard_normal(shape).astype(np.float32)
    cpu, hip = pair

    def softmax(be, x):
        e = be.exp(x - be.max(x, axis=axis))
        return e / be.sum(e, axis=axis)

    cases = [("softmax + x", lambda be, x, y: softmax(be, x) + x),
             ("softmax * y", lambda be, x, y: softmax(be, x) * y),
             ("softmax(x + y) * y", lambda be, x, y: softmax(be, x + y) * y),
             ("log-softmax", lambda be, x, y: be.log(softmax(be, x)) * y),
             ("softmax of softmax", lambda be, x, y: softmax(be, softmax(be, x)))]
    for what, f in cases:
        got = call_func(f, hip, [a, b])
        want = call_func(f, cpu, [a, b])
        assert_close(got, want, rtol=5 * RTOL32 if shape[axis] > 5000 else RTOL32, atol=1e-7, what=what)


@pytest.mark.parametrize("shape", [(32000, 256), (5000, 100), (20000, 1000), (9001, 36)])
def test_tall_multilevel_axis0(pair, shape):
    """deep axis-0 trees over more rows than one workgroup holds: the
    workgroups of a column strip exchange partials between sweeps"""
    rs = np.random.RandomState(shape[1])
    a = (rs.standard_normal(shape) * 3).astype(np.float32)
    cpu, hip = pair
    # With tens of thousands of rows the oracle's own rounding is no longer
    # below 1e-5: numpy adds the rows of an axis-0 sum one after the other in
    # fp32, the device adds a tree.  So both are held against an fp64
    # evaluation: the device to the 1e-5 bound, the oracle to what a
    # sequential fp32 sum of that length can lose.
    a64 = a.astype(np.float64)
    e64 = np.exp(a64 - a64.max(axis=0))
    truth = e64 / e64.sum(axis=0)
    for _ in range(2):          # twice: the arrival counters must have re-armed themselves
        got = call_func(lambda be, x: be.fprop_softmax(x, 0), hip, [a])
        assert_close(got, truth, rtol=RTOL32, atol=1e-12, what="softmax vs fp64")
    want = call_func(lambda be, x: be.fprop_softmax(x, 0), cpu, [a])
    assert_close(want, truth, rtol=shape[0] * 1.2e-7, atol=1e-12, what="oracle softmax vs fp64")
    assert np.allclose(got.astype(np.float64).sum(axis=0), 1.0, atol=1e-5)
    truth = (a64 - a64.mean(axis=0)) / np.sqrt(a64.var(axis=0) + 1e-5)
    f = lambda be, x: (x - be.mean(x, axis=0)) / be.sqrt(be.var(x, axis=0) + 1e-5)   # noqa: E731
    assert_close(call_func(f, hip, [a]), truth, rtol=RTOL32, atol=1e-5, what="colnorm vs fp64")
    assert_close(call_func(f, cpu, [a]), truth, rtol=shape[0] * 1.2e-7, atol=1e-4, what="oracle colnorm vs fp64")
    # an index reduction feeding a later sweep
    both(pair, lambda be, x: be.sum(be.equal(x, be.max(x, axis=0)) * be.argmax(x, axis=0), axis=0), [a],
         what="index in tree")
    if hip.plan_stats is not None and shape == (32000, 256):
        fams = set(p.spec.family for p in hip.plans.values())
        assert "colcoop" in fams


@pytest.mark.parametrize("shape,axis", [((3, 300000), 1), ((2, 150000), 1), ((40000, 33), 0), ((70000, 8), 0),
                                        ((6, 70000), 0), ((70000, 6), 1)])
def test_extreme_aspect_ratios(pair, shape, axis):
    """rows too long to stay in registers (streamed on every sweep), odd
    column counts on the split-row path, very flat and very tall inputs"""
    rs = np.random.RandomState(shape[0] % 91)
    a = gen_inputs(rs, shape)
    atol = 4 * np.finfo(np.float32).eps * float(np.abs(a).sum(axis=axis).max())
    both(pair, lambda be, x: be.sum(x, axis=axis), [a], rtol=RTOL32, atol=atol, what="sum")
    both(pair, lambda be, x: be.max(x, axis=axis) - be.min(x, axis=axis), [a], what="range")
    both(pair, lambda be, x: be.argmax(x, axis=axis), [a], out_dtype=np.int32, what="argmax")
    a64 = a.astype(np.float64)
    truth = (a64 - a64.mean(axis=axis, keepdims=True)) / np.sqrt(a64.var(axis=axis, keepdims=True) + 1e-5)
    got = call_func(lambda be, x: (x - be.mean(x, axis=axis)) / be.sqrt(be.var(x, axis=axis) + 1e-5), pair[1], [a])
    assert_close(got, truth, rtol=RTOL32, atol=1e-5, what="normalise vs fp64")


@pytest.mark.parametrize("dtype", [np.float16, np.int32, np.uint8, np.int16])
@pytest.mark.parametrize("axis", [0, 1])
def test_reductions_over_storage_dtypes(pair, dtype, axis):
    rs = np.random.RandomState(12)
    shape = (96, 160)
    if np.dtype(dtype).kind == "f":
        a = (rs.rand(*shape) * 4 - 2).astype(dtype)
    else:
        a = rs.randint(0, 100, shape).astype(dtype)
    cpu, hip = pair
    res = []
    for be in pair:
        # the oracle holds the same values in fp32 so that it, too, computes in fp32
        x = be.array(a.astype(np.float32)) if be is cpu else be.array(a, dtype=dtype)
        red = (1, shape[1]) if axis == 0 else (shape[0], 1)
        o1, o2, o3 = be.empty(red), be.empty(red, dtype=np.int32), be.empty(shape, dtype=dtype)
        o1[:] = be.max(x, axis=axis) - be.min(x, axis=axis) + be.sum(x, axis=axis)
        o2[:] = be.argmin(x, axis=axis)
        o3[:] = x - be.min(x, axis=axis)
        res.append((o1.get(), o2.get(), o3.get()))
    assert_close(res[1][0], res[0][0], rtol=RTOL32, atol=1e-3, what="stats")
    assert np.array_equal(res[1][1], res[0][1])
    if np.dtype(dtype).kind == "f":
        assert rel_err(res[1][2], res[0][2], floor_frac=1e-3) <= 1e-3
    else:
        assert np.array_equal(res[1][2], res[0][2])


def test_fused_update_rules(pair):
    """optimizer-style statement groups between begin/end(Block.update): same
    results as one kernel per statement (reference optimizer.py: momentum SGD
    :382-426, RMSProp :589-606)"""
    from neon_amd.backends.backend import Block
    rs = np.random.RandomState(13)
    shape = (300, 130)
    g0, p0 = gen_inputs(rs, shape) * 0.1, gen_inputs(rs, shape)
    res = []
    for be in pair:
        for fused in (False, True):
            grad, param = be.array(g0), be.array(p0)
            vel, state = be.zeros(shape), be.zeros(shape)
            for step in range(3):
                if fused:
                    be.begin(Block.update, step)
                vel[:] = vel * 0.9 - 0.01 * (grad + 0.0005 * param)          # momentum + weight decay
                param[:] = param + vel
                state[:] = 0.95 * state + be.square(grad) * (1.0 - 0.95)     # RMSProp state
                param[:] = param - (grad * 0.002) / (be.sqrt(state + 1e-6) + 1e-6)
                if fused:
                    be.end(Block.update, step)
            res.append((param.get(), vel.get(), state.get()))
    for k in range(3):
        assert np.array_equal(res[2][k], res[3][k]), "fused and unfused device results differ"
        assert_close(res[3][k], res[1][k], rtol=RTOL32, atol=1e-7)
        assert_close(res[2][k], res[0][k], rtol=RTOL32, atol=1e-7)


def test_onehot(pair):
    rs = np.random.RandomState(8)
    idx = rs.randint(0, 40, (1, 64)).astype(np.int32)
    y = (rs.rand(40, 64) + 0.1).astype(np.float32)
    outs = []
    for be in pair:
        i = be.array(idx, dtype=np.int32)
        t = be.empty((40, 64))
        t[:] = be.onehot(i, axis=0)              # top-level form
        p = be.array(y)
        ce = be.empty((1, 64))
        ce[:] = be.sum(-be.onehot(i, axis=0) * be.safelog(p), axis=0)   # in-tree form
        outs.append((t.get(), ce.get()))
    assert np.array_equal(outs[1][0], outs[0][0])
    assert_close(outs[1][1], outs[0][1])


# ---- the five benchmark configurations -------------------------------------------------------
def test_config1(pair):
    x, y = configs.inputs_c1()
    res = []
    for be in pair:
        tx, ty, out = be.array(x), be.array(y), be.empty(configs.C1_SHAPE)
        configs.c1a(be, out, tx, ty)
        a = out.get()
        configs.c1b(be, out)
        res.append((a, out.get()))
    assert_close(res[1][0], res[0][0], rtol=RTOL32)
    assert_close(res[1][1], res[0][1], rtol=RTOL32)


def test_config2_softmax(pair):
    (x,) = configs.inputs_c2()
    res = []
    for be in pair:
        tx, out = be.array(x), be.empty(configs.C2_SHAPE)
        configs.c2_softmax(be, out, tx)
        a = out.get()
        configs.c2_softmax_neon(be, out, tx)
        res.append((a, out.get()))
    assert_close(res[1][0], res[0][0], rtol=RTOL32, atol=1e-12)
    assert_close(res[1][1], res[0][1], rtol=RTOL32, atol=1e-12)
    assert np.allclose(res[1][0].sum(axis=0), 1.0, atol=1e-5)


@pytest.mark.parametrize("fused", [False, True])
def test_config3_adam(pair, fused):
    shape = (1000, 1250)       # the oracle needs seconds at this size; the full size is in test_full_size
    grad, param = configs.inputs_c3(shape)
    from neon_amd.backends.backend import Block
    res = []
    for be in pair:
        bsz, be.bsz = be.bsz, 1
        g, p = be.array(grad), be.array(param)
        m, v = be.zeros(shape), be.zeros(shape)
        snap = None
        for t in range(1, 11):
            if fused:
                be.begin(Block.update, t)
            configs.c3_adam_step(be, p, g, m, v, t)
            if fused:
                be.end(Block.update, t)
            if t == 1:
                snap = (p.get(), m.get(), v.get())
        res.append((snap, (p.get(), m.get(), v.get())))
        be.bsz = bsz
    for step in (0, 1):
        for k, name in enumerate(("param", "m", "v")):
            assert_close(res[1][step][k], res[0][step][k], rtol=RTOL32, atol=1e-12, what="%s step %d" % (name, step))


def test_config4_rownorm_fp16(pair):
    shape = (32, 100352)
    x, gamma, beta = configs.inputs_c4(shape)
    cpu, hip = pair
    # oracle: fp16-quantised inputs held in fp32, fp32 arithmetic, fp16 store
    o_cpu = cpu.empty(shape, dtype=np.float16)
    configs.c4_rownorm(cpu, o_cpu, cpu.array(x.astype(np.float32)), cpu.array(gamma), cpu.array(beta))
    o_hip = hip.empty(shape, dtype=np.float16)
    configs.c4_rownorm(hip, o_hip, hip.array(x, dtype=np.float16), hip.array(gamma), hip.array(beta))
    want, got = o_cpu.get().astype(np.float64), o_hip.get().astype(np.float64)
    # relative error against max(|want|, 1e-3 * max|want|): values near the row
    # mean are tiny and one fp16 ulp of the store would dominate otherwise
    assert rel_err(got, want, floor_frac=1e-3) <= 1e-3


def test_config5_argmax_max_ce(pair):
    shape = (4000, 256)
    x, idx = configs.inputs_c5(shape)
    cpu, hip = pair
    res = []
    for be in pair:
        tx = be.array(x)
        ti = be.array(idx, dtype=np.int32)
        am = be.empty((1, shape[1]), dtype=np.int32)
        mx = be.empty((1, shape[1]))
        ce = be.empty((1, shape[1]))
        configs.c5a_argmax(be, am, tx)
        configs.c5b_max(be, mx, tx)
        if be is cpu:
            t = be.empty(shape)
            t[:] = be.onehot(ti, axis=0)
            configs.c5c_cross_entropy(be, ce, tx, t)
        else:
            configs.c5c_cross_entropy(be, ce, tx, be.onehot(ti, axis=0))
        res.append((am.get(), mx.get(), ce.get()))
    assert np.array_equal(res[1][0], res[0][0])
    assert np.array_equal(res[1][1], res[0][1])
    assert_close(res[1][2], res[0][2], rtol=RTOL32)
    assert np.array_equal(res[1][0].ravel(), np.argmax(x, axis=0))


@pytest.mark.parametrize("shape", [(32000, 256), (9001, 36), (20000, 1000)])
def test_tall_trees_with_one_value_per_column_repeat(hip, shape):
    """deep axis-0 trees whose result is one value per column: after the last
    sweep no workgroup waits, the last arrival of each strip folds alone.  Run
    three times on fresh data: the arrival counters must re-arm every time."""
    be = hip
    for rep in range(3):
        rs = np.random.RandomState(rep + shape[1])
        a = (rs.standard_normal(shape) * 3).astype(np.float32)
        idx = rs.randint(0, shape[0], size=(1, shape[1])).astype(np.int32)
        tx, ti = be.array(a), be.array(idx, dtype=np.int32)
        ce, lse = be.empty((1, shape[1])), be.empty((1, shape[1]))
        configs.c5c_cross_entropy(be, ce, tx, be.onehot(ti, axis=0))
        lse[:] = be.log(be.sum(be.exp(tx - be.max(tx, axis=0)), axis=0)) + be.max(tx, axis=0)
        a64 = a.astype(np.float64)
        m = a64.max(axis=0)
        want_lse = np.log(np.exp(a64 - m).sum(axis=0)) + m
        want_ce = want_lse - a64[idx.ravel(), np.arange(shape[1])]
        assert_close(lse.get().ravel(), want_lse, rtol=RTOL32, atol=1e-6, what="log-sum-exp, repetition %d" % rep)
        assert_close(ce.get().ravel(), want_ce, rtol=2e-5, atol=2e-5, what="cross-entropy, repetition %d" % rep)


@pytest.mark.parametrize("shape,dtype", [((600000, 64), np.float16), ((540000, 48), np.float16)])
def test_very_tall_single_strip_reductions_run_in_1024_lane_workgroups(hip, shape, dtype):
    """one strip of columns, long row chunks, fewer workgroups than half the
    compute units: the split column family takes 1024 lanes per workgroup;
    max / argmax bit-exact, sums against float64, two launches on fresh data"""
    for rep in range(2):
        rs = np.random.RandomState(rep + 77)
        x = rs.standard_normal(shape).astype(dtype)
        tx = hip.array(x, dtype=dtype)
        sm, mx, am = hip.empty((1, shape[1])), hip.empty((1, shape[1])), hip.empty((1, shape[1]), dtype=np.int32)
        with hip.capture() as groups:
            sm[:] = hip.sum(tx, axis=0)
        spec = hip.time_group(groups[0], reps=1)[1].spec
        assert spec.family == "colsplit" and spec.block == 1024
        sm[:] = hip.sum(tx, axis=0)
        mx[:] = hip.max(tx, axis=0)
        am[:] = hip.argmax(tx, axis=0)
        x64 = x.astype(np.float64)
        assert_close(sm.get(), x64.sum(axis=0, keepdims=True), rtol=RTOL32, atol=2e-2, what="sum, repetition %d" % rep)
        assert np.array_equal(mx.get(), x.astype(np.float32).max(axis=0, keepdims=True))
        assert np.array_equal(am.get().ravel(), x.argmax(axis=0))


def test_full_size_properties(hip):
    """size-independent checks at the benchmark shapes"""
    be = hip
    x, idx = configs.inputs_c5()
    tx = be.array(x)
    am = be.empty((1, configs.C5_SHAPE[1]), dtype=np.int32)
    mx = be.empty((1, configs.C5_SHAPE[1]))
    configs.c5a_argmax(be, am, tx)
    configs.c5b_max(be, mx, tx)
    assert np.array_equal(am.get().ravel(), np.argmax(x, axis=0))
    assert np.array_equal(mx.get().ravel(), np.max(x, axis=0))
    ce = be.empty((1, configs.C5_SHAPE[1]))
    configs.c5c_cross_entropy(be, ce, tx, be.onehot(be.array(idx, dtype=np.int32), axis=0))
    x64 = x.astype(np.float64)
    lse = np.log(np.exp(x64 - x64.max(0)).sum(0)) + x64.max(0)
    want = lse - x64[idx.ravel(), np.arange(x.shape[1])]
    assert_close(ce.get().ravel(), want, rtol=2e-5)

    x4, gamma, beta = configs.inputs_c4()
    o = be.empty(configs.C4_SHAPE, dtype=np.float16)
    configs.c4_rownorm(be, o, be.array(x4, dtype=np.float16), be.array(gamma), be.array(beta))
    got = o.get().astype(np.float64)
    assert np.allclose(got.mean(axis=1), beta.ravel(), atol=2e-3)
    assert np.allclose(got.std(axis=1), gamma.ravel(), rtol=2e-3)

    grad, param = configs.inputs_c3()
    from neon_amd.backends.backend import Block
    bsz, be.bsz = be.bsz, 1
    g, p, m, v = be.array(grad), be.array(param), be.zeros(configs.C3_SHAPE), be.zeros(configs.C3_SHAPE)
    be.begin(Block.update, 1)
    configs.c3_adam_step(be, p, g, m, v, 1)
    be.end(Block.update, 1)
    be.bsz = bsz
    # after one step from m = v = 0: m = 0.1 g, v = 0.001 g^2, |delta p| ~= lr
    assert_close(m.get(), np.float32(1. - 0.9) * grad, rtol=1e-6, atol=0)
    d = param - p.get()
    nz = np.abs(grad) > 1e-3      # eps / sqrt(v) is below 4e-4 there
    assert np.allclose(np.abs(d[nz]), 1e-3, rtol=2e-3)
    assert np.array_equal(np.sign(d[nz]), np.sign(grad[nz]))


# ---- batch normalisation entry points (fused statement groups) -----------------------------------
@pytest.mark.parametrize("shape,dtype", [((32, 128), np.float32), ((64, 6272), np.float32),
                                         ((16, 100352), np.float16), ((5, 77), np.float32)])
def test_compound_batchnorm(pair, shape, dtype):
    cpu, hip = pair
    rs = np.random.RandomState(shape[1] % 89)
    x0 = (rs.standard_normal(shape) * 2 + 0.5).astype(np.float32).astype(dtype)
    d0 = rs.standard_normal(shape).astype(np.float32).astype(dtype)
    gam0 = rs.uniform(0.5, 1.5, (shape[0], 1)).astype(np.float32)
    bet0 = (rs.standard_normal((shape[0], 1)) * 0.1).astype(np.float32)
    res = []
    for be in pair:
        # the oracle holds fp16 data as fp32 values so that it computes in fp32 as well
        sdt = np.float32 if be is cpu else dtype
        x, din = be.array(x0.astype(sdt), dtype=sdt), be.array(d0.astype(sdt), dtype=sdt)
        y, dout = be.empty(shape, dtype=dtype), be.empty(shape, dtype=dtype)
        vec = lambda: be.zeros((shape[0], 1))     # noqa: E731
        xsum, xvar, gmean, gvar, gg, gb = vec(), vec(), vec(), vec(), vec(), vec()
        gamma, beta = be.array(gam0), be.array(bet0)
        for _ in range(2):                        # running statistics accumulate over two calls
            be.compound_fprop_bn(x, xsum, xvar, gmean, gvar, gamma, beta, y, 1e-3, 0.9, True)
        be.compound_bprop_bn(dout, gg, gb, din, x, xsum, xvar, gamma, 1e-3)
        yi = be.empty(shape, dtype=dtype)
        be.compound_fprop_bn(x, xsum, xvar, gmean, gvar, gamma, beta, yi, 1e-3, 0.9, True, inference=True)
        res.append([t.get().astype(np.float64) for t in (y, xsum, xvar, gmean, gvar, dout, gg, gb, yi)])
    names = ("y", "xmean", "xvar", "gmean", "gvar", "delta", "grad_gamma", "grad_beta", "y_inference")
    tol = 1e-3 if dtype == np.float16 else 2e-5
    for got, want, name in zip(res[1], res[0], names):
        scale = np.abs(want).max() + 1e-30
        assert np.abs(got - want).max() <= tol * scale, (name, np.abs(got - want).max(), scale)
    if hip.plan_stats is not None and shape[1] >= 128:
        # forward ran as one row kernel: x read once
        fams = [p.spec.family for p in hip.plans.values() if len(p.spec.source) and "row" == p.spec.family]
        assert fams


def test_repeated_batchnorm_calls_replay_their_recorded_launches(pair):
    """the second and later calls of compound_fprop_bn / compound_bprop_bn on the
    same tensors take the launches recorded by the first (no trees are built);
    new data, other numbers and other tensors must all still come out right"""
    cpu, hip = pair
    shape = (24, 3000)
    rs = np.random.RandomState(9)
    state = []
    for be in pair:
        vec = lambda: be.zeros((shape[0], 1))     # noqa: E731
        state.append(dict(be=be, x=be.empty(shape), d=be.empty(shape), y=be.empty(shape), dout=be.empty(shape),
                          xsum=vec(), xvar=vec(), gmean=vec(), gvar=vec(), gg=vec(), gb=vec(),
                          gamma=be.array(rs.uniform(0.5, 1.5, (shape[0], 1)).astype(np.float32)),
                          beta=be.array((rs.standard_normal((shape[0], 1)) * 0.1).astype(np.float32))))
        rs = np.random.RandomState(9)             # same gamma / beta on both backends
    before = hip.plan_stats["replayed"]
    for call, rho in enumerate((0.9, 0.9, 0.9, 0.5, 0.5, 0.9)):
        x0 = (rs.standard_normal(shape) * (1 + call) + 0.25 * call).astype(np.float32)
        d0 = rs.standard_normal(shape).astype(np.float32)
        out = []
        for st in state:
            be = st["be"]
            st["x"].set(x0)
            st["d"].set(d0)
            y = st["y"] if call != 4 else be.empty(shape)        # once into another output tensor
            be.compound_fprop_bn(st["x"], st["xsum"], st["xvar"], st["gmean"], st["gvar"], st["gamma"], st["beta"],
                                 y, 1e-3, rho, True)
            be.compound_bprop_bn(st["dout"], st["gg"], st["gb"], st["d"], st["x"], st["xsum"], st["xvar"],
                                 st["gamma"], 1e-3)
            out.append([t.get().astype(np.float64) for t in (y, st["xsum"], st["xvar"], st["gmean"], st["gvar"],
                                                             st["dout"], st["gg"], st["gb"])])
        for got, want, name in zip(out[1], out[0], ("y", "xmean", "xvar", "gmean", "gvar", "delta", "gg", "gb")):
            scale = np.abs(want).max() + 1e-30
            assert np.abs(got - want).max() <= 2e-5 * scale, (call, name)
    # calls 1, 2 and 5 of the forward pass and 1..5 of the backward pass found their recording
    assert hip.plan_stats["replayed"] - before >= 8


def test_more_than_2_31_elements(hip):
    """a tensor of 46341 x 46342 fp16 (2^31 + 83k elements, 4.3 GB): fill,
    elementwise tree and both reduction axes address it with 64-bit offsets;
    checked on the first and the last rows, which hold host data"""
    be = hip
    R, C = 46341, 46342
    x = be.empty((R, C), dtype=np.float16)
    out = be.empty((R, C), dtype=np.float16)
    x[:] = 1.5
    rs = np.random.RandomState(11)
    head = rs.uniform(-2, 2, (3, C)).astype(np.float16)
    tail = rs.uniform(-2, 2, (5, C)).astype(np.float16)
    x[0:3, :].set(head)
    x[R - 5:R, :].set(tail)
    out[:] = x * 2.0 + 1.0
    assert np.array_equal(out[0:3, :].get(), (head.astype(np.float32) * 2 + 1).astype(np.float16))
    assert np.array_equal(out[R - 5:R, :].get(), (tail.astype(np.float32) * 2 + 1).astype(np.float16))
    assert np.all(out[R // 2:R // 2 + 2, :].get() == 4.0)
    rows = be.empty((R, 1))
    rows[:] = be.sum(x, axis=1)
    got = rows.get().ravel()
    assert_close(got[R - 5:], tail.astype(np.float64).sum(axis=1), rtol=1e-5, atol=1e-2)
    assert np.all(got[3:R - 5] == 1.5 * C)
    cols = be.empty((1, C))
    cols[:] = be.max(x, axis=0)
    want = np.maximum(np.maximum(head.max(axis=0), tail.max(axis=0)), np.float16(1.5)).astype(np.float32)
    assert np.array_equal(cols.get().ravel(), want)
    del x, out


@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["f32", "f16"])
@pytest.mark.parametrize("shape", [(37, 1032), (130, 264), (1000, 4096), (16, 8)])
def test_row_vectors_fetched_once_per_workgroup(pair, shape, dtype):
    """(1, C) operands of a two-dimensional elementwise kernel are loaded ahead
    of the row loop and shared by the rows a lane handles"""
    R, C = shape
    rs = np.random.RandomState(R + C)
    x = rs.standard_normal(shape).astype(dtype)
    row = rs.standard_normal((1, C)).astype(np.float32)
    row2 = rs.standard_normal((1, C)).astype(dtype)
    col = rs.standard_normal((R, 1)).astype(np.float32)
    cases = [lambda be, a, r, r2, c: a * r,
             lambda be, a, r, r2, c: a * r + c,
             lambda be, a, r, r2, c: (a - r2) * r + r2 * c,
             lambda be, a, r, r2, c: be.maximum(a, r) - be.minimum(r2, c)]
    cpu, hip = pair
    for f in cases:
        got = call_func(f, hip, [x, row, row2, col])
        want = call_func(f, cpu, [x.astype(np.float32), row, row2.astype(np.float32), col])
        assert_close(got, want, rtol=RTOL32, atol=1e-6)


@pytest.mark.parametrize("dtype", [np.float32, np.float16, np.uint8, np.int32], ids=["f32", "f16", "u8", "i32"])
@pytest.mark.parametrize("shape,lo,hi", [((67, 1001), 3, 2), ((300, 519), 1, 0), ((5, 40), 7, 9), ((1, 4099), 1, 1)])
def test_views_that_start_mid_row_and_odd_row_lengths(pair, shape, lo, hi, dtype):
    """16-byte accesses at addresses that are only element-aligned, with a
    partial last tile in every row: bit-exact against the oracle"""
    R, C = shape
    rs = np.random.RandomState(C)
    if np.dtype(dtype).kind == "f":
        x = rs.uniform(-4, 4, shape).astype(dtype)
        y = rs.uniform(-4, 4, shape).astype(dtype)
    else:
        x = rs.randint(0, 100, shape).astype(dtype)
        y = rs.randint(0, 100, shape).astype(dtype)
    res = []
    for be in pair:
        tx, ty = be.array(x, dtype=dtype), be.array(y, dtype=dtype)
        out = be.zeros(shape, dtype=dtype)
        out[:, lo:C - hi] = tx[:, lo:C - hi] * 2 + ty[:, lo:C - hi]
        whole = be.empty(shape, dtype=np.float32)
        if be is pair[0] and dtype == np.float16:
            # the oracle would do this arithmetic in fp16; the device computes in fp32
            tx, ty = be.array(x.astype(np.float32)), be.array(y.astype(np.float32))
        whole[:] = tx * 0.5 - ty
        res.append((out.get(), whole.get()))
    assert np.array_equal(res[1][0], res[0][0])
    assert_close(res[1][1], res[0][1], rtol=RTOL32, atol=1e-6)


@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["f32", "f16"])
@pytest.mark.parametrize("shape", [(8, 70000), (3, 200003 * 8), (64, 131072), (1, 1 << 20)])
def test_few_very_long_rows(pair, shape, dtype):
    """axis-1 trees over few, very long rows: each row is spread over several
    workgroups that exchange partials after every sweep.  Twice each: the
    arrival counters must re-arm."""
    R, C = shape
    rs = np.random.RandomState(R)
    x = (rs.standard_normal(shape) * 2 + 0.5).astype(dtype)
    x32 = x.astype(np.float32)
    cpu, hip = pair
    x64 = x.astype(np.float64)
    e64 = np.exp(x64 - x64.max(axis=1, keepdims=True))
    cases = [("x - mean", lambda be, a: a - be.mean(a, axis=1), x64 - x64.mean(axis=1, keepdims=True), 2e-5),
             ("softmax", lambda be, a: be.fprop_softmax(a, 1), e64 / e64.sum(axis=1, keepdims=True), 2e-5),
             ("std", lambda be, a: be.sqrt(be.var(a, axis=1)), x64.std(axis=1, keepdims=True), 2e-5),
             ("sum", lambda be, a: be.sum(a, axis=1), x64.sum(axis=1, keepdims=True), 1e-5)]
    for what, f, truth, rtol in cases:
        for rep in range(2):
            got = call_func(f, hip, [x])
            scale = np.abs(truth).max()
            assert np.abs(got - truth).max() <= rtol * scale + 1e-6 * np.sqrt(C), (what, rep)
    got = call_func(lambda be, a: be.argmax(a, axis=1), hip, [x], out_dtype=np.int32)
    assert np.array_equal(got.ravel(), np.argmax(x32, axis=1))
    got = call_func(lambda be, a: be.max(a, axis=1) - be.min(a, axis=1), hip, [x])
    assert np.array_equal(got.ravel(), x32.max(axis=1) - x32.min(axis=1))


@pytest.mark.parametrize("dtype", [np.uint8, np.int8, np.float16, np.int16], ids=["u8", "i8", "f16", "i16"])
@pytest.mark.parametrize("shape", [(5, 6), (9, 2), (4, 3), (33, 10), (7, 12)])
def test_narrow_elements_with_short_rows(pair, shape, dtype):
    """row lengths that leave no whole 32-bit word of 1- or 2-byte elements per
    lane: element-wise tiles, in every family"""
    rs = np.random.RandomState(shape[1])
    x = rs.randint(0, 50, shape).astype(dtype)
    res = []
    for be in pair:
        t = be.array(x if be is pair[1] else x.astype(np.float32), dtype=(dtype if be is pair[1] else np.float32))
        e, c, r = be.empty(shape), be.empty((1, shape[1])), be.empty((shape[0], 1))
        e[:] = t * 2 + 1
        c[:] = be.sum(t, axis=0)
        r[:] = be.max(t, axis=1) - be.min(t, axis=1)
        res.append((e.get(), c.get(), r.get()))
    for want, got in zip(*res):
        assert np.array_equal(got, want)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("shape", [(300, 1000), (40, 16384), (2000, 64), (77, 1003), (5, 40000)])
def test_expensive_values_of_16bit_rows_are_kept_between_sweeps(pair, shape, dtype):
    """softmax and friends over rows of 16-bit elements: the exponentials of the
    summing sweep are kept in float32 registers for the sweep that stores --
    same arithmetic as the oracle's on the widened values"""
    from neon_amd.backends import bfloat16
    cpu, hip = pair
    rs = np.random.RandomState(shape[1] % 1000)
    x32 = (rs.standard_normal(shape) * 3).astype(np.float32)
    if dtype == "f16":
        x16, store = x32.astype(np.float16), np.float16
        x32 = x16.astype(np.float32)
    else:
        store = bfloat16
        x32 = (x32.view(np.uint32) & np.uint32(0xFFFF0000)).view(np.float32)
        x16 = x32
    trees = [lambda be, t: be.exp(t - be.max(t, axis=1)) / be.sum(be.exp(t - be.max(t, axis=1)), axis=1),
             lambda be, t: be.sig(t) / be.sum(be.sig(t), axis=1),
             lambda be, t: be.exp(t - be.max(t, axis=1)) / be.sum(be.exp(t - be.max(t, axis=1)), axis=1)
             + be.tanh(t) * be.max(be.tanh(t), axis=1)]
    for k, f in enumerate(trees):
        want = call_func(f, cpu, [x32])
        th = hip.array(x16, dtype=store)
        out = hip.empty(shape)
        out[:] = f(hip, th)
        assert_close(out.get(), want, rtol=RTOL32, atol=1e-7, what="tree %d" % k)
        narrow = hip.empty(shape, dtype=store)
        narrow[:] = f(hip, th)
        assert_close(narrow.get().astype(np.float32), want, rtol=1e-3 if dtype == "f16" else 8e-3, atol=1e-7,
                     what="tree %d, 16-bit result" % k)


# ---- several reductions of one operand in one launch -----------------------------------------
@pytest.mark.gpu
def test_argmax_and_max_of_one_operand_fuse_into_one_launch(pair):
    cpu, hip = pair
    rs = np.random.RandomState(31)
    x = (rs.standard_normal((5000, 200)) * 4).astype(np.float32)
    x[17, 3] = x[900, 3] = x[:, 3].max() + 1.0          # a tie: the first row wins
    X = hip.array(x)
    am, mx, sm = hip.empty((1, 200), dtype=np.int32), hip.empty((1, 200)), hip.empty((1, 200))
    before = hip.plan_stats["launches"]
    with hip.fused():
        am[:] = hip.argmax(X, axis=0)
        mx[:] = hip.max(X, axis=0)
        sm[:] = hip.sum(X, axis=0)
    assert hip.plan_stats["launches"] - before == 1
    assert np.array_equal(am.get(), x.argmax(axis=0).reshape(1, -1).astype(np.int32)) and am.get()[0, 3] == 17
    assert np.array_equal(mx.get(), x.max(axis=0, keepdims=True))
    assert_close(sm.get(), x.astype(np.float64).sum(axis=0, keepdims=True), rtol=1e-5, atol=1e-3)
    # along the other axis, and a result that lives inside the operand stays out of the group
    rm, rmin = hip.empty((5000, 1)), hip.empty((5000, 1))
    before = hip.plan_stats["launches"]
    with hip.fused():
        rm[:] = hip.max(X, axis=1)
        rmin[:] = hip.min(X, axis=1)
    assert hip.plan_stats["launches"] - before == 1
    assert np.array_equal(rm.get(), x.max(axis=1, keepdims=True)) and np.array_equal(rmin.get(), x.min(axis=1, keepdims=True))
    before = hip.plan_stats["launches"]
    with hip.fused():
        mx[:] = hip.max(X, axis=0)
        X[0:1, :] = hip.min(X, axis=0)
    assert hip.plan_stats["launches"] - before == 2
    want = x.copy()
    want[0, :] = x.min(axis=0)
    assert np.array_equal(X.get(), want) and np.array_equal(mx.get(), x.max(axis=0, keepdims=True))


@pytest.mark.gpu
def test_argmax_argmin_follow_numpy_on_nan(pair):
    """np.argmax / np.argmin return the position of the first NaN
    (reference nervanacpu.py:453-473 calls them directly)"""
    cpu, hip = pair
    rs = np.random.RandomState(32)
    for shape in ((300, 40), (6000, 64), (40000, 16)):
        x = rs.standard_normal(shape).astype(np.float32)
        x[shape[0] // 2, 1] = np.nan
        x[5, 2] = x[shape[0] - 3, 2] = np.nan
        x[0, 3] = np.nan
        x[shape[0] - 1, 4] = np.nan
        x[:, 5] = -np.inf
        x[7, 6] = np.inf
        for name in ("argmax", "argmin"):
            for axis in (0, 1):
                def f(be):
                    out = be.empty((1, shape[1]) if axis == 0 else (shape[0], 1), dtype=np.int32)
                    out[:] = getattr(be, name)(be.array(x), axis=axis)
                    return out.get()
                want = getattr(np, name)(x, axis=axis).reshape(f(cpu).shape).astype(np.int32)
                assert np.array_equal(f(cpu), want)
                assert np.array_equal(f(hip), want), (name, axis, shape)
    # and the values: max / min give NaN for those lines
    x = rs.standard_normal((6000, 64)).astype(np.float32)
    x[100, 1] = np.nan
    mx = hip.empty((1, 64))
    mx[:] = hip.max(hip.array(x), axis=0)
    assert np.array_equal(mx.get(), x.max(axis=0, keepdims=True), equal_nan=True)


@pytest.mark.gpu
def test_derived_builders_against_numpy_directly(hip):
    """mean / var / std / clip / reciprocal / fprop_softmax / whole-tensor
    reductions are compositions made by the API's base class, which the oracle
    backend shares: here the hip results are compared with numpy itself
    (float64), not with the oracle (formulas: reference backend.py:860, 1311,
    1331-1334, 1446-1502; nervanacpu.py:1916-1919)"""
    rs = np.random.RandomState(41)
    x = (rs.standard_normal((700, 260)) * 2 + 0.3).astype(np.float32)
    x64 = x.astype(np.float64)
    X = hip.array(x)

    def ev(tree, shape):
        out = hip.empty(shape)
        out[:] = tree
        return out.get()

    for axis in (0, 1):
        line = (1, 260) if axis == 0 else (700, 1)
        assert_close(ev(hip.mean(X, axis=axis), line), x64.mean(axis=axis, keepdims=True), rtol=1e-5, atol=1e-6)
        assert_close(ev(hip.var(X, axis=axis), line), x64.var(axis=axis, keepdims=True), rtol=1e-5, atol=1e-6)
        assert_close(ev(hip.std(X, axis=axis), line), x64.std(axis=axis, keepdims=True), rtol=1e-5, atol=1e-6)
        e = np.exp(x64 - x64.max(axis=axis, keepdims=True))
        assert_close(ev(hip.fprop_softmax(X, axis), x.shape), e / e.sum(axis=axis, keepdims=True), rtol=1e-5, atol=1e-9)
    assert_close(ev(hip.mean(X), (1, 1)), x64.mean().reshape(1, 1), rtol=1e-5, atol=1e-6)
    assert_close(ev(hip.var(X), (1, 1)), x64.var().reshape(1, 1), rtol=1e-5, atol=1e-6)
    assert_close(ev(hip.sum(X), (1, 1)), x64.sum().reshape(1, 1), rtol=1e-5, atol=1e-3)
    assert np.array_equal(ev(hip.max(X), (1, 1)), x.max().reshape(1, 1))
    assert np.array_equal(ev(hip.min(X), (1, 1)), x.min().reshape(1, 1))
    assert np.array_equal(ev(hip.clip(X, -1.0, 0.5), x.shape), np.clip(x, -1.0, 0.5))
    assert_close(ev(hip.reciprocal(X), x.shape), 1.0 / x64, rtol=1e-6, atol=0)
    assert_close(ev(hip.absolute(X) ** 1.5, x.shape), np.abs(x64) ** 1.5, rtol=1e-5, atol=1e-7)


@pytest.mark.gpu
def test_division_by_a_line_value_with_extreme_divisors(pair):
    """x / d with d constant along the row is computed as x * (1/d) only while
    1/d is a normal number; zero, denormal, huge, infinite and NaN divisors
    give the quotient as written"""
    cpu, hip = pair
    rs = np.random.RandomState(43)
    x = rs.standard_normal((9, 300)).astype(np.float32)
    x[:, 0] = 0.0
    x[:, 1] = np.float32(1e-38)
    d = np.array([[0.0], [1e-42], [3e38], [np.inf], [np.nan], [2.5], [-1e-39], [1.0e-30], [-0.0]], dtype=np.float32)
    res = []
    for be in pair:
        out = be.empty(x.shape)
        with np.errstate(all="ignore"):
            out[:] = be.array(x) / be.array(d)
        res.append(out.get())
    assert np.array_equal(np.isnan(res[1]), np.isnan(res[0]))
    ok = ~np.isnan(res[0])
    assert np.array_equal(np.isinf(res[1][ok]), np.isinf(res[0][ok]))
    fin = ok & np.isfinite(res[0])
    assert_close(res[1][fin], res[0][fin], rtol=1e-6, atol=0)
    assert np.array_equal(np.sign(res[1][ok]), np.sign(res[0][ok]))


@pytest.mark.gpu
def test_gather_views_clamp_indices_outside_the_table(hip):
    """numpy raises IndexError for an index outside the tensor; a kernel cannot,
    so gather / scatter views keep every access inside the indexed tensor"""
    table = np.arange(40 * 6, dtype=np.float32).reshape(40, 6)
    T = hip.array(table)
    idx = np.array([[3], [39], [40], [1000000], [-1], [-7]], dtype=np.int32)
    rows = hip.empty((6, 6))
    rows[:] = T[hip.array(idx, dtype=np.int32)]
    want = table[np.clip(idx.ravel(), 0, 39)]
    assert np.array_equal(rows.get(), want)
    cols = hip.empty((40, 3))
    cols[:] = T.take(hip.array(np.array([[5], [6], [-2]], dtype=np.int32), dtype=np.int32), 1)
    assert np.array_equal(cols.get(), table[:, [5, 5, 0]])


def test_exponential_of_values_below_their_maximum_is_good_to_the_last_place(hip):
    """exp(x - max(x)) runs a shorter exponential (its argument is never
    positive): against float64 over the whole range that yields normal
    numbers, and the edge cases -- equal to the maximum, -inf, NaN columns"""
    rs = np.random.RandomState(21)
    cols = 512
    d = -np.abs(rs.uniform(0, 87.0, (400, cols))).astype(np.float32)
    d[0, :] = 0.0                                           # every column's maximum
    d[1, :] = -np.logspace(-8, 1.9, cols).astype(np.float32)
    x = d + rs.uniform(-50, 50, (1, cols)).astype(np.float32)
    # (the difference is taken in fp32, as any fp32 evaluation takes it; the exponential of
    # that difference is what is being checked)
    want = np.exp((x - x.max(axis=0)).astype(np.float64))
    out = hip.empty(x.shape)
    out[:] = hip.exp(hip.array(x) - hip.max(hip.array(x), axis=0))
    got = out.get().astype(np.float64)
    normal = want > 1.2e-38
    assert np.max(np.abs(got[normal] - want[normal]) / want[normal]) < 2.5e-7        # two units in the last place
    assert np.all(got[~normal] <= 1.2e-38)
    assert np.all(got[0] == 1.0)
    # along rows, with -inf entries and a NaN row
    y = rs.uniform(-30, 30, (64, 300)).astype(np.float32)
    y[3, 5] = -np.inf
    y[7, :] = -np.inf                                      # (all -inf: -inf - -inf = NaN, as in numpy)
    y[9, 11] = np.nan
    outy = hip.empty(y.shape)
    outy[:] = hip.exp(hip.array(y) - hip.max(hip.array(y), axis=1))
    with np.errstate(invalid="ignore"):
        wy = np.exp((y - y.max(axis=1, keepdims=True)).astype(np.float64))
    gy = outy.get()
    assert np.array_equal(np.isnan(gy), np.isnan(wy))
    ok = ~np.isnan(wy)
    np.testing.assert_allclose(gy[ok], wy[ok], rtol=2.5e-7, atol=1e-38)
    assert gy[3, 5] == 0.0


def test_logistic_function_is_good_to_a_few_units_on_both_tails(hip):
    """sig / sig2 are computed from e^-|x| with a Newton-refined reciprocal
    instead of expf and a division: against float64 over the range that
    yields normal numbers, at the edges (0, -0, +-inf, NaN, huge) and on the
    far negative tail, where the true result is below the normal range"""
    rs = np.random.RandomState(33)
    x = np.concatenate([rs.uniform(-87, 87, 200000), rs.normal(0, 2, 200000), np.logspace(-30, 1.9, 20000),
                        -np.logspace(-30, 1.9, 20000)]).astype(np.float32).reshape(-1, 1000)
    out = hip.empty(x.shape)
    for name, base in (("sig", np.e), ("sig2", 2.0)):
        out[:] = getattr(hip, name)(hip.array(x))
        want = 1.0 / (1.0 + np.power(base, -x.astype(np.float64)))
        got = out.get().astype(np.float64)
        assert np.max(np.abs(got - want) / want) < 4e-7, name               # three units in the last place
    edge = np.array([[0.0, -0.0, np.inf, -np.inf, np.nan, 3e38, -3e38, 100.0, -100.0, -95.0, 17.0, -17.0]], np.float32)
    oe = hip.empty(edge.shape)
    oe[:] = hip.sig(hip.array(edge))
    g = oe.get()[0]
    assert g[0] == 0.5 and g[1] == 0.5 and g[2] == 1.0 and g[3] == 0.0 and np.isnan(g[4])
    assert g[5] == 1.0 and g[6] == 0.0 and g[7] == 1.0
    assert 0.0 <= g[8] <= 4e-44 and 0.0 <= g[9] <= 6e-42                     # true values are denormal
    np.testing.assert_allclose(g[10:], 1.0 / (1.0 + np.exp(-edge[0, 10:].astype(np.float64))), rtol=4e-7)


@pytest.mark.parametrize("shape,axis,dtype", [((40, 262144), 1, np.float32), ((24, 393216), 1, np.float16),
                                               ((3, 1 << 21), 1, np.float32)])
def test_lone_reductions_over_few_very_long_rows(hip, shape, axis, dtype):
    """few very long rows reduced along the rows: run over a reshaped view
    plus a small second reduction (two launches); sums against float64,
    max / min exactly"""
    rs = np.random.RandomState(shape[0] % 13)
    xh = rs.standard_normal(shape).astype(np.float32).astype(dtype)
    x = hip.array(xh, dtype=dtype)
    x64 = xh.astype(np.float64)
    line = (shape[0], 1) if axis == 1 else (1, shape[1])
    out = hip.empty(line)

    def launches(issue):
        before = hip.plan_stats["launches"]
        issue()
        return hip.plan_stats["launches"] - before

    n = shape[axis]
    assert launches(lambda: out.__setitem__(slice(None), hip.sum(x, axis=axis))) == 2
    np.testing.assert_allclose(out.get(), x64.sum(axis=axis, keepdims=True), rtol=1e-5, atol=1e-5 * np.sqrt(n))
    assert launches(lambda: out.__setitem__(slice(None), hip.max(x, axis=axis))) == 2
    assert np.array_equal(out.get(), xh.max(axis=axis, keepdims=True).astype(np.float32))
    assert launches(lambda: out.__setitem__(slice(None), hip.min(x, axis=axis))) == 2
    assert np.array_equal(out.get(), xh.min(axis=axis, keepdims=True).astype(np.float32))
    # an expression below the reduction and arithmetic above it (a mean of squares, shifted)
    assert launches(lambda: out.__setitem__(slice(None), hip.sum(x * x + 1.0, axis=axis) * (1.0 / n) - 1.0)) == 2
    np.testing.assert_allclose(out.get(), (x64 * x64).mean(axis=axis, keepdims=True), rtol=2e-5, atol=1e-6)
    # again: replayed from the recording
    out.fill(0)
    assert launches(lambda: out.__setitem__(slice(None), hip.sum(x * x + 1.0, axis=axis) * (1.0 / n) - 1.0)) == 2
    np.testing.assert_allclose(out.get(), (x64 * x64).mean(axis=axis, keepdims=True), rtol=2e-5, atol=1e-6)
    # an index reduction keeps its own kernel
    idx = hip.empty(line, dtype=np.int32)
    assert launches(lambda: idx.__setitem__(slice(None), hip.argmax(x, axis=axis))) == 1
    assert np.array_equal(idx.get(), xh.argmax(axis=axis).reshape(line))


def test_sum_of_exponentials_in_one_sweep_stays_within_a_few_units_of_float64(hip):
    """the one-sweep (max, sum of exponentials) pair adds terms computed with a
    plain product by log2(e): each term's error is weighted by the term, so
    the SUM stays within a few 1e-7 of float64 however many terms there are
    -- checked where the weights are worst (every term near e^-1) and over a
    wide spread"""
    rs = np.random.RandomState(33)
    for rows, lo, hi in ((65536, -1.2, -0.8), (200000, -30.0, 0.0), (40000, -87.0, 0.0)):
        x = rs.uniform(lo, hi, (rows, 64)).astype(np.float32)
        x[rs.randint(0, rows, 64), np.arange(64)] = 0.0                 # the maximum of every column
        out = hip.empty((1, 64))
        dx = hip.array(x)
        out[:] = hip.sum(hip.exp(dx - hip.max(dx, axis=0)), axis=0)
        want = np.exp(x.astype(np.float64)).sum(axis=0)
        got = out.get().ravel().astype(np.float64)
        assert np.max(np.abs(got - want) / want) < 4e-7, (rows, lo, hi)


@pytest.mark.parametrize("shape,dtype", [((9000, 2100), np.float32), ((20000, 2040), np.float16), ((5000, 4110), np.float32), ((60000, 1000), np.float32), ((3000, 9000), np.float32)])
def test_split_column_reductions_with_strips_dealt_to_xcds_in_runs(hip, shape, dtype):
    """rows that are no whole number of cache lines: the split column family
    runs on a one-dimensional grid in which every XCD owns a run of strips
    (surplus workgroups leave at once; the ticket of a strip still counts its
    chunks).  sum / max / argmax / cross-entropy style log-sum-exp against
    numpy, twice on fresh data."""
    for rep in range(2):
        rs = np.random.RandomState(rep + 31)
        x = rs.standard_normal(shape).astype(dtype)
        x[rs.randint(0, shape[0], 50), rs.randint(0, shape[1], 50)] = 3.5         # ties for argmax
        tx = hip.array(x, dtype=dtype)
        sm, mx, lse = (hip.empty((1, shape[1])) for _ in range(3))
        am = hip.empty((1, shape[1]), dtype=np.int32)
        with hip.capture() as groups:
            sm[:] = hip.sum(tx, axis=0)
        spec = hip.time_group(groups[0], reps=1)[1].spec
        assert spec.family == "colsplit" and spec.params["runs"], spec.params
        sm[:] = hip.sum(tx, axis=0)
        mx[:] = hip.max(tx, axis=0)
        am[:] = hip.argmax(tx, axis=0)
        lse[:] = hip.log(hip.sum(hip.exp(tx - hip.max(tx, axis=0)), axis=0)) + hip.max(tx, axis=0)
        x64 = x.astype(np.float64)
        assert_close(sm.get(), x64.sum(axis=0, keepdims=True), rtol=RTOL32, atol=2e-3 * np.sqrt(shape[0]), what="sum")
        assert np.array_equal(mx.get(), x.astype(np.float32).max(axis=0, keepdims=True))
        assert np.array_equal(am.get().ravel(), x.argmax(axis=0))
        m = x64.max(axis=0)
        assert_close(lse.get().ravel(), np.log(np.exp(x64 - m).sum(axis=0)) + m, rtol=RTOL32, atol=1e-5, what="log-sum-exp")


@pytest.mark.parametrize("shape,dtype", [((32000, 256), np.float32), ((16000, 250), np.float32), ((30000, 264), np.float16),
                                         ((8192, 1024), np.float32), ((40000, 96), np.float32), ((6000, 509), np.float16),
                                         ((131072, 64), np.float32), ((100000, 64), np.float16), ((400000, 16), np.float32),
                                         ((50000, 250), np.float16), ((64000, 300), np.float32)])
def test_split_column_reductions_finished_by_the_last_workgroups_of_a_strip(hip, shape, dtype):
    """the split column family where the strip's last workgroups wait for the
    others' tagged partials (a tag bit inside each 8-byte record, flipped every
    launch): sum / max / argmax / min with NaNs / log-sum-exp against numpy on
    fresh data, four launches in a row of every kernel so that both tag values
    are met, widths with a ragged last strip and a ragged last vector included."""
    tagged = 0
    for rep in range(4):
        rs = np.random.RandomState(rep + 77)
        x = rs.standard_normal(shape).astype(dtype)
        x[rs.randint(0, shape[0], 50), rs.randint(0, shape[1], 50)] = 3.5         # ties for argmax
        xn = x.copy()
        xn[rs.randint(0, shape[0], 3), rs.randint(0, shape[1], 3)] = np.nan
        tx, tn = hip.array(x, dtype=dtype), hip.array(xn, dtype=dtype)
        sm, mx, mn, lse = (hip.empty((1, shape[1])) for _ in range(4))
        am = hip.empty((1, shape[1]), dtype=np.int32)
        if rep == 0:
            for issue in (lambda: sm.__setitem__(slice(None), hip.sum(tx, axis=0)),
                          lambda: am.__setitem__(slice(None), hip.argmax(tx, axis=0))):
                with hip.capture() as groups:
                    issue()
                spec = hip.time_group(groups[0], reps=1)[1].spec
                assert spec.family == "colsplit"
                tagged += bool(spec.params["lookback"])
        sm[:] = hip.sum(tx, axis=0)
        mx[:] = hip.max(tx, axis=0)
        am[:] = hip.argmax(tx, axis=0)
        mn[:] = hip.min(tn, axis=0)
        lse[:] = hip.log(hip.sum(hip.exp(tx - hip.max(tx, axis=0)), axis=0)) + hip.max(tx, axis=0)
        x64 = x.astype(np.float64)
        assert_close(sm.get(), x64.sum(axis=0, keepdims=True), rtol=RTOL32, atol=2e-3 * np.sqrt(shape[0]), what="sum")
        assert np.array_equal(mx.get(), x.astype(np.float32).max(axis=0, keepdims=True))
        assert np.array_equal(am.get().ravel(), x.argmax(axis=0))
        assert np.array_equal(mn.get(), xn.astype(np.float32).min(axis=0, keepdims=True), equal_nan=True)
        m = x64.max(axis=0)
        assert_close(lse.get().ravel(), np.log(np.exp(x64 - m).sum(axis=0)) + m, rtol=RTOL32, atol=1e-5, what="log-sum-exp")
    # ((131072,64), (100000,64), (400000,16): several records per polling lane; (50000,250), (64000,300): grids
    # that deal chunks to the XCDs in runs)
    if shape in ((32000, 256), (131072, 64), (100000, 64), (400000, 16), (50000, 250), (64000, 300)):
        assert tagged == 2, "this shape should take the tagged form"
