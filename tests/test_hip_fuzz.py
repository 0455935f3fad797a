"""Random op-trees on the hip backend against the numpy oracle (GPU box).

Seeded, so every run sees the same trees: shapes from a list that mixes
vector-friendly and odd extents, operands that are full, row, column or 1x1
tensors (a third of the full ones views into larger tensors, offset in both
directions), fp32 and fp16 storage, up to three levels of unary / binary
operators with reductions along one axis nested up to three deep.  A second set
uses extents up to 150000 so that the cooperative and split families run, a
third one few and very long lines."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

SMALL = [1, 2, 3, 7, 16, 33, 64, 100, 257, 1000, 1031, 4099]
LARGE = [1, 2, 5, 16, 40, 128, 256, 1000, 8192, 20000, 40003, 150000]
# few to a few hundred lines of 70 thousand to a million elements (and their transposes): rows
# partly resident in LDS, cooperative workgroups with long shares, reductions over reshaped
# views, staged column trees
LONG = [1, 3, 17, 64, 130, 300, 70001, 100352, 150528, 200704, 262144, 1000000]


def _case(rs, dims, limit):
    R, C = int(rs.choice(dims)), int(rs.choice(dims))
    if R * C > limit:
        if rs.rand() < 0.5:
            C = max(1, limit // R)
        else:
            R = max(1, limit // C)
    dtype = rs.choice([np.float32, np.float32, np.float32, np.float16])
    leaves = []
    for k in range(rs.randint(1, 4)):
        kind = "full" if k == 0 else rs.choice(["full", "full", "col", "row", "one"])
        shp = {"full": (R, C), "col": (R, 1), "row": (1, C), "one": (1, 1)}[kind]
        leaves.append(rs.uniform(-2, 2, shp).astype(dtype if shp == (R, C) else np.float32))
    axis = int(rs.randint(0, 2))

    def expr(be, ts, depth, allow_red):
        r = rs.rand()
        if depth == 0 or r < 0.25:
            if rs.rand() < 0.15:
                return float(np.round(rs.uniform(-2, 2), 3))
            return ts[rs.randint(len(ts))]
        if r < 0.5:
            a = expr(be, ts, depth - 1, allow_red)
            op = rs.choice(["neg", "abs", "sqrtabs", "tanh", "sig", "square", "expclip"])
            if isinstance(a, float):
                a = ts[0] * a
            return {"neg": lambda: -a, "abs": lambda: be.absolute(a), "sqrtabs": lambda: be.sqrt(be.absolute(a)),
                    "tanh": lambda: be.tanh(a), "sig": lambda: be.sig(a), "square": lambda: be.square(a),
                    "expclip": lambda: be.exp(be.minimum(a, 3.0))}[op]()
        if r < 0.85 or not allow_red:
            a, b = expr(be, ts, depth - 1, allow_red), expr(be, ts, depth - 1, allow_red)
            if isinstance(a, float) and isinstance(b, float):
                a = ts[0]
            op = rs.choice(["add", "sub", "mul", "max", "min", "div", "gt", "le"])
            if op == "div":
                return a / ((be.absolute(b) if not isinstance(b, float) else abs(b)) + 1.0)
            return {"add": lambda: a + b, "sub": lambda: a - b, "mul": lambda: a * b,
                    "max": lambda: be.maximum(a, b), "min": lambda: be.minimum(a, b),
                    "gt": lambda: be.greater(a, b) * 1.0, "le": lambda: be.less_equal(a, b) * 1.0}[op]()
        a = expr(be, ts, depth - 1, True)
        if isinstance(a, float):
            a = ts[0] * a
        return getattr(be, rs.choice(["sum", "max", "min", "mean"]))(a, axis=axis)
    return R, C, leaves, axis, expr


def _run(be, seed, dims, limit, oracle):
    rs = np.random.RandomState(seed)
    R, C, leaves, axis, expr = _case(rs, dims, limit)
    ts = []
    for leaf in leaves:
        host = leaf.astype(np.float32) if oracle else leaf          # the oracle computes in fp32 on exact copies
        if leaf.shape == (R, C) and rs.rand() < 0.3 and R > 1 and C > 1:
            pr, pc = int(rs.randint(0, 3)), int(rs.randint(0, 4))
            big = np.zeros((R + pr + 1, C + pc + 2), host.dtype)
            big[pr:pr + R, pc:pc + C] = host
            ts.append(be.array(big, dtype=big.dtype)[pr:pr + R, pc:pc + C])
        else:
            ts.append(be.array(host, dtype=host.dtype))
    tree = expr(be, ts, 3, True)
    if isinstance(tree, float):
        tree = ts[0] + tree
    out = be.empty(tree.shape, dtype=np.float32)
    out[:] = tree
    return (R, C, axis), out.get()


@pytest.mark.parametrize("first,count,dims,limit", [(1000, 120, SMALL, 2000000), (5000, 40, LARGE, 30000000),
                                                    (9000, 72, LONG, 40000000)],
                         ids=["small", "large", "long"])
def test_random_trees_match_the_oracle(pair, first, count, dims, limit):
    cpu, hip = pair
    for seed in range(first, first + count):
        (R, C, axis), want = _run(cpu, seed, dims, limit, True)
        _, got = _run(hip, seed, dims, limit, False)
        assert got.shape == want.shape, seed
        w64 = want.astype(np.float64)
        finite = np.isfinite(w64)
        assert np.array_equal(finite, np.isfinite(got)), seed
        scale = max(1.0, np.abs(w64[finite]).max() if finite.any() else 1.0)
        err = np.abs(got.astype(np.float64) - w64)
        err[~finite] = 0
        # the reductions add up to R or C terms in a different order on the device
        tol = 3e-6 * max(8, R if axis == 0 else C)
        # (a comparison operator turns a last-place difference between two exponentials into a
        # 0 / 1 flip: among tens of millions of elements a few such flips are expected, one
        # in a million is allowed)
        over = int((err / scale > tol).sum())
        assert over <= err.size // 1000000, (seed, R, C, axis, err.max() / scale, over)


def _flat_expr(be, rs, ts, depth):
    r = rs.rand()
    if depth == 0 or r < 0.3:
        return ts[rs.randint(len(ts))] if rs.rand() < 0.85 else float(np.round(rs.uniform(-1, 1), 2))
    a, b = _flat_expr(be, rs, ts, depth - 1), _flat_expr(be, rs, ts, depth - 1)
    if isinstance(a, float) and isinstance(b, float):
        a = ts[0]
    op = rs.choice(["add", "sub", "mul", "max", "root", "div"])
    if op == "root":
        return be.sqrt(be.absolute(b if isinstance(a, float) else a))
    if op == "div":
        return a / ((be.absolute(b) if not isinstance(b, float) else abs(b)) + 1.0)
    return {"add": lambda: a + b, "sub": lambda: a - b, "mul": lambda: a * b,
            "max": lambda: be.maximum(a, b)}[op]()


def test_random_fused_statement_groups_match_the_oracle(pair):
    """two to four assigns into four tensors between begin / end: one kernel on
    the device, statement after statement on the oracle; later statements read
    what earlier ones wrote"""
    from neon_amd.backends.backend import Block
    cpu, hip = pair
    for seed in range(100):
        res = []
        for be in (cpu, hip):
            rs = np.random.RandomState(seed)
            shape = [(64, 100), (1000, 33), (1, 5000), (257, 257), (4096, 128)][rs.randint(5)]
            ts = [be.array(rs.uniform(-2, 2, shape).astype(np.float32)) for _ in range(4)]
            be.begin(Block.update, 0)
            for _ in range(rs.randint(2, 5)):
                target = ts[rs.randint(len(ts))]
                e = _flat_expr(be, rs, ts, 2)
                target[:] = ts[0] * e if isinstance(e, float) else e
            be.end(Block.update, 0)
            res.append([t.get() for t in ts])
        for want, got in zip(*res):
            assert np.allclose(got, want, rtol=2e-5, atol=2e-5), seed


def _near_twin(be, rs, ts, idx, depth, axis):
    """small trees from a small vocabulary (five numbers, four tensors): many
    of them differ from an earlier one only in a number, in the side a number
    stands on or in one operator"""
    r = rs.rand()
    if depth == 0 or r < 0.3:
        return float(rs.choice([0.5, 1.0, 2.0, -1.5, 3.0])) if rs.rand() < 0.35 else ts[rs.randint(len(ts))]
    if r < 0.45:
        a = _near_twin(be, rs, ts, idx, depth - 1, axis)
        op = rs.choice(["neg", "sqrtabs", "expclip", "tanh", "sq"])
        return {"neg": lambda: -a, "sqrtabs": lambda: be.sqrt(be.absolute(a)),
                "expclip": lambda: be.exp(be.minimum(a, 3.0)), "tanh": lambda: be.tanh(a),
                "sq": lambda: be.square(a)}[op]()
    if r < 0.9:
        a, b = _near_twin(be, rs, ts, idx, depth - 1, axis), _near_twin(be, rs, ts, idx, depth - 1, axis)
        op = rs.choice(["add", "sub", "mul", "div", "gt", "le", "max", "min", "pow"])
        if op == "div":
            return be.divide(a, be.absolute(b) + 1.0)
        if op == "pow":
            return be.power(be.absolute(a) + 0.5, be.minimum(be.maximum(b, -2.0), 2.0))
        if op in ("gt", "le"):          # as numbers: numpy would add two boolean arrays as a logical or
            return {"gt": be.greater, "le": be.less_equal}[op](a, b) * 1.0
        return {"add": be.add, "sub": be.subtract, "mul": be.multiply, "max": be.maximum, "min": be.minimum}[op](a, b)
    if rs.rand() < 0.2:
        return be.onehot(idx, axis=0)
    a = _near_twin(be, rs, ts, idx, depth - 1, axis)
    return getattr(be, rs.choice(["sum", "max", "min", "mean"]))(ts[0] * a if isinstance(a, float) else a, axis=axis)


def test_many_near_twin_trees_on_the_same_tensors(pair):
    """one backend instance, one set of tensors, several hundred small trees in
    a row: plans are found again by key, recorded launches are replayed and
    re-bound to other numbers -- every result still has to be the tree's own"""
    from neon_amd.backends.backend import Block
    cpu, hip = pair
    R, C = 64, 96
    rs0 = np.random.RandomState(7)
    host = [rs0.uniform(-2, 2, shp).astype(np.float32) for shp in ((R, C), (R, C), (R, 1), (1, C))]
    hidx = rs0.randint(0, R, (1, C)).astype(np.int32)
    env = {be: ([be.array(h) for h in host], be.array(hidx, dtype=np.int32), be.empty((R, C)), be.empty((R, C)))
           for be in pair}
    before = dict(hip.plan_stats)
    for seed in range(500):
        res = []
        for be in (cpu, hip):
            ts, idx, out, out2 = env[be]
            rs = np.random.RandomState(seed)
            axis = int(rs.randint(0, 2))
            targets = [out] if rs.rand() < 0.7 else [out, out2]
            fuse = be is hip and len(targets) == 2 and seed % 2 == 0
            if fuse:
                be.begin(Block.update, 0)
            for target in targets:
                t = _near_twin(be, rs, ts, idx, int(rs.randint(1, 4)), axis)
                target[:] = ts[0] + t if isinstance(t, float) else t
            if fuse:
                be.end(Block.update, 0)
            res.append([t.get() for t in targets])
        for want, got in zip(*res):
            w64 = want.astype(np.float64)
            finite = np.isfinite(w64)
            assert np.array_equal(finite, np.isfinite(got)), seed
            scale = max(1.0, np.abs(w64[finite]).max() if finite.any() else 1.0)
            err = np.abs(got.astype(np.float64) - w64)
            err[~finite] = 0
            assert err.max() / scale <= 3e-6 * C, (seed, err.max() / scale)
    assert hip.plan_stats["replayed"] > before["replayed"] + 100 and hip.plan_stats["hit"] > before["hit"] + 10


def test_near_twin_trees_over_operands_in_many_layouts(pair):
    """operands: dense, window of a larger tensor, transposed view, fp16, column,
    row, 1x1 and a one-column window; results into a dense tensor, a window, a
    transposed view or an fp16 tensor -- 300 trees in a row on one instance"""
    cpu, hip = pair
    R, C = 40, 56
    rs0 = np.random.RandomState(11)
    u = lambda *shp: rs0.uniform(-2, 2, shp).astype(np.float32)
    host = dict(x=u(R, C), big=u(R + 3, C + 5), zt=u(C, R), h=u(R, C).astype(np.float16), col=u(R, 1), row=u(1, C),
                one=u(1, 1), bigcol=u(R + 2, 3))
    hidx = rs0.randint(0, R, (1, C)).astype(np.int32)
    env = {}
    for be in pair:
        # the oracle computes in fp32 on exact copies of the fp16 operand
        put = (lambda a: be.array(a.astype(np.float32))) if be is cpu else (lambda a: be.array(a, dtype=a.dtype))
        t = {k: put(v) for k, v in host.items()}
        leaves = [t["x"], t["big"][1:R + 1, 2:C + 2], t["zt"].T, t["h"], t["col"], t["row"], t["one"],
                  t["bigcol"][1:R + 1, 1:2]]
        outs = dict(dense=be.empty((R, C)), big=be.zeros((R + 2, C + 4)), t=be.zeros((C, R)),
                    half=be.empty((R, C), dtype=np.float32 if be is cpu else np.float16))
        env[be] = (leaves, be.array(hidx, dtype=np.int32), outs)
    for seed in range(300):
        res = []
        for be in pair:
            leaves, idx, outs = env[be]
            rs = np.random.RandomState(seed)
            axis = int(rs.randint(0, 2))
            tree = _near_twin(be, rs, leaves, idx, int(rs.randint(1, 4)), axis)
            tree = (leaves[0] + tree if isinstance(tree, float) else tree) + 0.0 * leaves[0]       # full shape
            kind = rs.choice(["dense", "big", "t", "half"])
            if kind == "big":
                outs["big"][1:R + 1, 3:C + 3] = tree
            elif kind == "t":
                outs["t"].T[:] = tree
            else:
                outs[kind][:] = tree
            res.append(outs[kind].get().astype(np.float32))
        want, got = res
        w64 = want.astype(np.float64)
        finite = np.isfinite(w64)
        assert np.array_equal(finite, np.isfinite(got)), (seed, kind)
        scale = max(1.0, np.abs(w64[finite]).max() if finite.any() else 1.0)
        err = np.abs(got.astype(np.float64) - w64)
        err[~finite] = 0
        assert err.max() / scale <= (1.5e-3 if kind == "half" else 3e-6 * C), (seed, kind, err.max() / scale)


def test_random_storage_types_and_small_extents(pair):
    """every storage type on either operand, extents from 1 to 5000 (many of
    them shorter than a vector): elementwise, both reduction axes, float and
    int32 results"""
    cpu, hip = pair
    types = [np.uint8, np.int8, np.int16, np.uint16, np.int32, np.uint32, np.float16, np.float32]
    dims = [1, 2, 3, 4, 5, 6, 7, 8, 9, 12, 15, 16, 17, 31, 33, 64, 100, 129, 1000, 1031, 5000]
    for seed in range(160):
        rs = np.random.RandomState(seed)
        R, C = int(rs.choice(dims)), int(rs.choice(dims))
        da, db = types[rs.randint(len(types))], types[rs.randint(len(types))]
        a = rs.randint(0, 100, (R, C)).astype(da)
        b = rs.randint(1, 50, (R, C)).astype(db)
        kind = rs.randint(6)
        res = []
        for be in (cpu, hip):
            if be is cpu:       # exact fp32 copies: numpy would do integer arithmetic on integer arrays
                ta, tb = be.array(a.astype(np.float32)), be.array(b.astype(np.float32))
            else:
                ta, tb = be.array(a, dtype=da), be.array(b, dtype=db)
            tree = [lambda: ta * 2 + tb, lambda: be.sum(ta * tb, axis=0), lambda: be.max(ta - tb, axis=1),
                    lambda: ta - be.mean(ta, axis=1) + tb, lambda: be.maximum(ta, tb) - be.min(tb, axis=0),
                    lambda: be.sum(ta, axis=1) + be.sum(tb, axis=1)][kind]()
            out = be.empty(tree.shape)
            out[:] = tree
            ints = None
            if kind != 3:       # integer-valued results also go into an int32 tensor
                oi = be.empty(tree.shape, dtype=np.int32)
                oi[:] = tree
                ints = oi.get()
            res.append((out.get(), ints))
        (want, want_i), (got, got_i) = res
        assert np.allclose(got, want, rtol=1e-5, atol=1e-3), (seed, R, C, da, db, kind)
        assert want_i is None or np.array_equal(got_i, want_i), (seed, R, C, da, db, kind)
