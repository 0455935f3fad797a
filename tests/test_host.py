"""Host-side logic that needs no GPU: the tensor API, the C ABI surface, the
DAG builder, shape-class selection, code generation and hiprtc compilation for
gfx950, the kernel cache, and the error behaviour callers rely on."""
import ctypes
import os
import re

import numpy as np
import pytest

from neon_amd.backends import bfloat16
from neon_amd.backends.backend import Backend, Block, OpCollection, OpTreeNode
from neon_amd.backends.hip import codegen, planner, prebuild
from neon_amd.backends.hip import runtime as hiprt
from neon_amd.backends.hip.optree_ir import MixedAxes, Program

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture()
def pb(tmp_path):
    return prebuild.PlanBackend(cache_dir=str(tmp_path / "kc"), compile_kernels=False)


def plan_of(pb, issue):
    n = len(pb.choices)
    issue()
    assert len(pb.choices) == n + 1
    return pb.choices[-1]


# ---- API --------------------------------------------------------------------------------
def test_backend_registry_and_factory():
    import neon_amd.backends as nb
    assert "hip" in Backend.backend_choices()
    with pytest.raises(ValueError):
        Backend.allocate_backend("no-such-backend")
    assert nb.gen_backend.__defaults__[0] == "hip"


def test_optree_build_rules(pb):
    a, b = pb.empty((4, 3)), pb.empty((4, 1))
    f = a + b * 2.0
    assert f.shape == (4, 3) and f[0]["op"] == "add"
    assert (a > b).shape == (4, 3)
    assert pb.sum(a, axis=0).shape == (1, 3) and pb.sum(a, axis=1).shape == (4, 1)
    assert pb.sum(a).shape == (1, 1)
    assert pb.mean(a, axis=1)[0]["op"] == "mul"                # sum * (1/N)
    assert (2.0 - a)[1] == 2.0 and (2.0 - a)[0]["op"] == "sub"
    assert (-a)[0]["op"] == "neg" and abs(a)[0]["op"] == "abs"
    stack = (a * b + a).traverse([])
    assert [s["op"] if isinstance(s, dict) else "t" for s in stack] == ["t", "t", "mul", "t", "add"]
    k1, t2i, i2t = (a * b + a).intrinsic_key_maps()
    assert k1 == ((0, (4, 3)), (1, (4, 1)), "mul", (0, (4, 3)), "add") and i2t[0] is a
    with pytest.raises(TypeError):
        OpTreeNode.build("bogus", a, b)
    assert OpTreeNode.build("add", a, "x") is NotImplemented
    with pytest.raises(ValueError):
        pb.onehot(pb.empty((1, 4), dtype=np.int32), axis=2)
    assert OpCollection.reduction_ops == {"sum", "max", "min", "argmax", "argmin"}
    assert (a + b).pp().startswith("(")


# ---- C ABI ------------------------------------------------------------------------------
def _declared_symbols():
    with open(os.path.join(ROOT, "include", "neonhip.h")) as f:
        text = f.read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(nh_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = hiprt.load_library()
    names = _declared_symbols()
    assert len(names) >= 35
    for n in names:
        assert hasattr(lib, n), "libneonhip.so does not export %s" % n
    assert sorted(hiprt.SIGNATURES) == names, "runtime.py binds a different set than the header declares"
    assert lib.nh_abi_version() == 1


def test_abi_errors_without_device():
    lib = hiprt.load_library()
    if hiprt.device_count() > 0:
        pytest.skip("device present")
    p = ctypes.c_void_p()
    assert lib.nh_malloc(ctypes.byref(p), 1024) == hiprt.NH_ENOTINIT
    assert b"nh_init" in lib.nh_last_error()
    assert lib.nh_init(0, None) != 0
    with pytest.raises(hiprt.HipError):
        hiprt.Runtime(0)
    from neon_amd.backends import gen_backend
    with pytest.raises(hiprt.HipError):
        gen_backend("hip")          # no silent CPU fallback


def test_rtc_compile_and_error_log():
    code, _ = hiprt.rtc_compile('extern "C" __global__ void k(float* a){ a[threadIdx.x] *= 2.f; }', "k.hip", "gfx950")
    assert code[:4] == b"\x7fELF"
    with pytest.raises(hiprt.HipError) as e:
        hiprt.rtc_compile('extern "C" __global__ void k(float* a){ a[0] = undefined_symbol; }', "bad.hip", "gfx950")
    assert "undefined_symbol" in str(e.value) and e.value.code >= hiprt.NH_RTC_ERROR_BASE


# ---- DAG --------------------------------------------------------------------------------
def _prog(pb, issue):
    got = []
    pb_exec, pb.execute = pb.execute, lambda t: got.append(t) or t[1]
    try:
        issue()
    finally:
        pb.execute = pb_exec
    p = Program()
    for t in got:
        p.add_statement(t)
    return p.finalize()


def test_cse_and_levels(pb):
    x, out = pb.empty((1000, 128)), pb.empty((1000, 128))
    p = _prog(pb, lambda: out.__setitem__(slice(None), pb.exp(x - pb.max(x, axis=0)) /
                                          pb.sum(pb.exp(x - pb.max(x, axis=0)), axis=0)))
    ops = [n.op for n in p.nodes if n.kind in ("E", "R")]
    assert ops.count("max") == 1 and ops.count("exp") == 1 and ops.count("sub") == 1   # duplicates merged
    assert p.axis == 0 and p.domain == (1000, 128)
    assert len(p.tensors) == 2 and p.tensors[0].written and p.tensors[1].read
    # sum(exp(x - max)) shares the sweep that finds the maximum (running pair): one level;
    # taking the pairing back restores one sweep each
    assert p.lse_pairs == 1 and p.nlevels == 1
    sm = [n for n in p.nodes if n.kind == "R" and n.op == "sum"][0]
    assert sm.lse_max.op == "max" and sm.lse_max.lse_sum is sm and sm.level == sm.lse_max.level == 1
    p.unpair_lse()
    assert p.lse_pairs == 0 and p.nlevels == 2 and sm.lse_max is None and sm.level == 2
    # ... and the planner may take it up again (twice is once)
    p.pair_lse()
    p.pair_lse()
    assert p.lse_pairs == 1 and p.nlevels == 1 and sm.lse_max.op == "max"
    # the same along rows; the row planner decides by residence whether to keep it
    y, outy = pb.empty((64, 4096)), pb.empty((64, 4096))
    q = _prog(pb, lambda: outy.__setitem__(slice(None), pb.exp(y - pb.max(y, axis=1)) /
                                           pb.sum(pb.exp(y - pb.max(y, axis=1)), axis=1)))
    assert q.axis == 1 and q.lse_pairs == 1 and q.nlevels == 1
    # a sum of exponentials around something else than the maximum of the same operand is no pair
    r = _prog(pb, lambda: outy.__setitem__(slice(None), pb.exp(y - pb.max(y * 2.0, axis=1)) /
                                           pb.sum(pb.exp(y - pb.max(y * 2.0, axis=1)), axis=1)))
    assert r.lse_pairs == 0 and r.nlevels == 2


def test_sum_over_a_one_hot_becomes_a_gather(pb):
    x, ce = pb.empty((4000, 256)), pb.empty((1, 256))
    idx = pb.empty((1, 256), dtype=np.int32)
    full = pb.empty((4000, 256))

    def cross_entropy():
        sm = pb.exp(x - pb.max(x, axis=0)) / pb.sum(pb.exp(x - pb.max(x, axis=0)), axis=0)
        ce[:] = -pb.sum(pb.onehot(idx, axis=0) * pb.log(sm), axis=0)
    p = _prog(pb, cross_entropy)
    assert p.gathers == 1 and p.lse_pairs == 1 and p.nlevels == 1
    g = [n for n in p.nodes if n.kind == "G"][0]
    assert g.args[1].kind == "H" and g.args[0].op == "log" and not g.vr and g.vc and g.level == 1
    # a column-sum that is broadcast back over the rows stays a sum
    p2 = _prog(pb, lambda: full.__setitem__(slice(None), x - pb.sum(pb.onehot(idx, axis=0) * x, axis=0)))
    assert p2.gathers == 0 and p2.nlevels == 1
    # ... as does one along the other axis of the one-hot
    rows = pb.empty((4000, 1))
    p3 = _prog(pb, lambda: rows.__setitem__(slice(None), pb.sum(pb.onehot(idx, axis=0) * x, axis=1)))
    assert p3.gathers == 0


def test_constant_folding_and_key(pb):
    x, out = pb.empty((8, 8)), pb.empty((8, 8))

    def adam_like(t):
        l = 1e-3 * pb.sqrt(1 - 0.999 ** t) / (1 - 0.9 ** t)
        out[:] = x - l * x

    p1, p2 = _prog(pb, lambda: adam_like(1)), _prog(pb, lambda: adam_like(7))
    assert len(p1.consts) == 1 and np.isclose(p1.consts[0], 1e-3 * np.sqrt(1 - 0.999) / 0.1)
    assert p1.key() == p2.key() and p1.consts != p2.consts          # same kernel, other argument
    p3 = _prog(pb, lambda: out.__setitem__(slice(None), 0.5 * x + 0.5 * x))
    p4 = _prog(pb, lambda: out.__setitem__(slice(None), 0.5 * x + 2.0 * x))
    assert len(p3.consts) == 1 and len(p4.consts) == 2 and p3.key() != p4.key()


def test_key_tells_which_side_a_number_stands_on(pb):
    """a number turns into a node only when its operator is applied, after the
    tensor beside it: ``x - 1`` and ``1 - x`` must still get different keys
    (equal keys share one compiled kernel)"""
    x, out = pb.empty((8, 8)), pb.empty((8, 8))
    forms = [lambda: x - 1.0, lambda: 1.0 - x, lambda: x / 2.0, lambda: 2.0 / x, lambda: x > 0.5, lambda: 0.5 > x,
             lambda: pb.power(x, 2.0), lambda: pb.power(2.0, x), lambda: 1.0 / (x - 1.0), lambda: 1.0 / (1.0 - x),
             lambda: (x - 1.0) - x, lambda: x - (1.0 - x), lambda: pb.sqrt(4.0) - x, lambda: x - pb.sqrt(4.0)]
    progs = [_prog(pb, lambda f=f: out.__setitem__(slice(None), f())) for f in forms]
    keys = [p.key() for p in progs]
    assert len(set(keys)) == len(keys)
    # the same form with another number keeps its key (the number is an argument)
    again = _prog(pb, lambda: out.__setitem__(slice(None), 3.0 - x))
    assert again.key() == keys[1] and again.consts != progs[1].consts


def test_equal_keys_mean_equal_programs(pb):
    """random small statement groups over a fixed set of tensors: whenever two
    of them get the same key they must be the same DAG up to the values of the
    numbers, since the key decides which compiled kernel runs"""
    R, C = 8, 16
    x, y, out, out2 = pb.empty((R, C)), pb.empty((R, C)), pb.empty((R, C)), pb.empty((R, C))
    leaves = [x, y, pb.empty((R, 1)), pb.empty((1, C))]
    idx = pb.empty((1, C), dtype=np.int32)
    rs = np.random.RandomState(0)
    unary = {"neg": pb.negative, "sqrt": pb.sqrt, "exp": pb.exp}
    binary = {"add": pb.add, "sub": pb.subtract, "mul": pb.multiply, "div": pb.divide, "gt": pb.greater,
              "pow": pb.power, "max": pb.maximum}

    def expr(depth, axis):
        r = rs.rand()
        if depth == 0 or r < 0.3:
            return float(rs.choice([0.5, 1.0, 2.0])) if rs.rand() < 0.35 else leaves[rs.randint(len(leaves))]
        if r < 0.45:
            return unary[rs.choice(sorted(unary))](expr(depth - 1, axis))
        if r < 0.9:
            return binary[rs.choice(sorted(binary))](expr(depth - 1, axis), expr(depth - 1, axis))
        if rs.rand() < 0.2:
            return pb.onehot(idx, axis=0)
        a = expr(depth - 1, axis)
        return getattr(pb, rs.choice(["sum", "max"]))(x * a if isinstance(a, float) else a, axis=axis)

    def group():
        axis = int(rs.randint(0, 2))
        for k in range(1 if rs.rand() < 0.7 else 2):
            t = expr(int(rs.randint(1, 4)), axis)
            (out if k == 0 else (out2 if rs.rand() < 0.5 else x))[:] = (x + t if isinstance(t, float) else t)

    seen, built = {}, 0
    for _ in range(6000):
        try:
            p = _prog(pb, group)
        except (TypeError, ValueError, NotImplementedError, planner.NeedsSplit, MixedAxes):
            continue            # mixed axes and the like: never reach a kernel as one program
        built += 1
        dag = (tuple((n.kind, n.op, tuple(a.nid for a in n.args), n.slot, n.axis) for n in p.nodes),
               tuple((st.out.index, st.root.nid) for st in p.statements))
        assert seen.setdefault(p.key(), dag) == dag, p.key()[0]
    assert built > 3000 and len(seen) > 1000


def test_identity_reduction_of_broadcast_operand(pb):
    row, out = pb.empty((1, 16)), pb.empty((1, 16))
    p = _prog(pb, lambda: out.__setitem__(slice(None), pb.sum(row, axis=0) + pb.argmax(row, axis=0)))
    assert p.axis is None and not any(n.kind == "R" for n in p.nodes)


def test_errors_raised_before_any_launch(pb):
    a, b = pb.empty((4, 3)), pb.empty((5, 3))
    with pytest.raises(TypeError):
        _prog(pb, lambda: a.__setitem__(slice(None), a + b))                  # shapes do not broadcast
    with pytest.raises(ValueError):
        _prog(pb, lambda: a.__setitem__(slice(None), OpTreeNode({"op": "sum", "shape": (4, 1), "axis": 2}, a, None)))
    with pytest.raises(MixedAxes):
        _prog(pb, lambda: pb.empty((1, 1)).__setitem__(slice(None), pb.sum(pb.sum(a, axis=0), axis=1)))
    with pytest.raises(TypeError):
        _prog(pb, lambda: pb.empty((1, 3)).__setitem__(slice(None), a * 2.0))  # result larger than target
    with pytest.raises(TypeError):
        a[:] = "text"


def test_fusion_forwards_written_values(pb):
    g, m, p_ = pb.empty((64, 64)), pb.empty((64, 64)), pb.empty((64, 64))

    def stmts():
        m[:] = m * 0.9 + 0.1 * g
        p_[:] = p_ - m

    prog = _prog(pb, stmts)
    assert len(prog.statements) == 2
    # the second statement reads the value written by the first, not memory
    sub = prog.statements[1].root
    assert sub.op == "sub" and sub.args[1] is prog.statements[0].root
    reads = [t.index for t in prog.tensors if t.read]
    assert len(reads) == 3                      # g, old m, old p


# ---- shape classes --------------------------------------------------------------------
def test_shape_class_selection(pb):
    f32, f16 = np.float32, np.float16
    x, y, o = pb.empty((4096, 128)), pb.empty((4096, 128)), pb.empty((4096, 128))
    ch = plan_of(pb, lambda: o.__setitem__(slice(None), 0.5 * x + 2.0 * y))
    assert ch.spec.family == "ew" and ch.spec.params["V"] == 4 and ch.grid[0] == 256 and ch.spec.block == 512
    col, row = pb.empty((4096, 1)), pb.empty((1, 128))
    ch = plan_of(pb, lambda: o.__setitem__(slice(None), x * col + row))
    assert ch.spec.family == "ew" and ch.spec.params["LY"] > 1            # 2-d tiling for broadcasts
    xs = pb.empty((1000, 128))
    ch = plan_of(pb, lambda: pb.empty((1000, 128)).__setitem__(slice(None), pb.fprop_softmax(xs, 0)))
    assert ch.spec.family == "col" and ch.spec.params["NR"] * ch.spec.params["LY"] >= 1000
    # tiny inputs: one 32-bit word per lane, the 16-byte strip made of adjacent lanes
    assert (ch.spec.params["V"], ch.spec.params["LX"]) == (1, 4)
    xh = pb.empty((1000, 128), np.float16)
    ch = plan_of(pb, lambda: pb.empty((1000, 128), np.float16).__setitem__(slice(None), pb.fprop_softmax(xh, 0)))
    assert ch.spec.family == "col" and ch.spec.params["V"] == 2
    xm = pb.empty((2000, 2048))
    ch = plan_of(pb, lambda: pb.empty((2000, 2048)).__setitem__(slice(None), pb.fprop_softmax(xm, 0)))
    assert ch.spec.family == "col" and ch.spec.params["V"] == 4
    x4, o4 = pb.empty((256, 100352), f16), pb.empty((256, 100352), f16)
    ch = plan_of(pb, lambda: o4.__setitem__(slice(None), (x4 - pb.mean(x4, axis=1)) / pb.sqrt(pb.var(x4, axis=1) + 1e-5)))
    assert ch.spec.family == "row" and ch.spec.params["V"] == 8 and ch.spec.params["NCH"] == 13
    assert ch.spec.params["stream"] and ch.grid == (256, 1, 1)
    x5 = pb.empty((32000, 256))
    ch = plan_of(pb, lambda: pb.empty((1, 256), np.int32).__setitem__(slice(None), pb.argmax(x5, axis=0)))
    assert ch.spec.family == "colsplit" and ch.workspace is not None
    assert ch.grid[0] * ch.grid[1] <= 2 * 256 and ch.grid[1] <= codegen.COLSPLIT_MAX_CHUNKS
    # several sweeps over 32000 rows do not fit one workgroup: the workgroups of a strip cooperate;
    # maximum and sum of exponentials travel together, so they meet once, not twice
    ch = plan_of(pb, lambda: pb.empty((32000, 256)).__setitem__(slice(None), pb.fprop_softmax(x5, 0)))
    assert ch.spec.family == "colcoop" and ch.grid[0] * ch.grid[1] <= 256 and ch.workspace is not None
    assert ch.spec.source.count("nh_part_store") == 1 and "NH_SPIN_LIMIT" in ch.spec.source
    assert "nh_op_lse" in ch.spec.source and ch.status_offset is not None
    # cross-entropy with the one-hot made in the kernel: one pass; only the strip's last workgroups wait,
    # for tagged partials, and a program whose wait once expired gets the form that never waits
    i5 = pb.empty((1, 256), np.int32)
    xent = lambda: pb.empty((1, 256)).__setitem__(slice(None), -pb.sum(
        pb.onehot(i5, axis=0) * pb.log(pb.fprop_softmax(x5, 0)), axis=0))
    ch = plan_of(pb, xent)
    assert ch.spec.family == "colsplit" and "nh_op_lse" in ch.spec.source
    assert ch.spec.params["lookback"] and ch.status_offset is not None and "nh_ticket_take" not in ch.spec.source
    assert ch.spec.source.count("NH_SPIN_LIMIT") == 1 and "nh_tag_put" in ch.spec.source
    pb.coop = False
    ch = plan_of(pb, xent)
    pb.coop = True
    assert ch.spec.family == "colsplit" and not ch.spec.params["lookback"] and ch.status_offset is None
    assert "NH_SPIN_LIMIT" not in ch.spec.source and "nh_ticket_take" in ch.spec.source
    huge = pb.empty((4000000, 256))
    with pytest.raises(planner.NeedsSplit):        # too many rows to keep on chip: evaluated stage by stage
        pb.empty((4000000, 256)).__setitem__(slice(None), pb.fprop_softmax(huge, 0))
    odd = pb.empty((64, 327))
    ch = plan_of(pb, lambda: pb.empty((64, 1)).__setitem__(slice(None), pb.sum(odd, axis=1)))
    # 327 columns: vector accesses, the last tile of a row element by element
    assert ch.spec.family == "row" and ch.spec.params["V"] == 4 and ch.spec.params["tail"]
    assert "load_partial" in ch.spec.source
    xt = pb.empty((128, 4096)).T
    ch = plan_of(pb, lambda: o.__setitem__(slice(None), xt + 1.0))
    assert ch.spec.params["V"] == 1                                          # strided operand


def test_adam_fuses_into_one_streaming_kernel(pb):
    from neon_amd import configs
    p, g, m, v = (pb.empty(configs.C3_SHAPE) for _ in range(4))
    n = len(pb.choices)
    pb.begin(Block.update, 0)
    configs.c3_adam_step(pb, p, g, m, v, 3)
    pb.end(Block.update, 0)
    assert len(pb.choices) == n + 1
    spec = pb.choices[-1].spec
    assert spec.family == "ew" and spec.params["stream"] and spec.params["V"] == 4
    # 4 tensors read once (non-temporal), 3 written once (ordinary stores)
    assert spec.source.count(".load_stream(") == 4 and spec.source.count(".store(") == 3
    assert ".store_stream(" not in spec.source


# ---- compile + cache --------------------------------------------------------------------
def test_benchmark_kernels_compile_for_gfx950_and_cache(tmp_path):
    be = prebuild.PlanBackend(cache_dir=str(tmp_path / "kc"))
    prebuild.benchmark_statements(be)
    assert be.cache.stats["compiled"] >= 8 and be.cache.stats["hit_disk"] == 0
    files = os.listdir(str(tmp_path / "kc"))
    assert len(files) == be.cache.stats["compiled"] and all(f.endswith(".hsaco") for f in files)
    be2 = prebuild.PlanBackend(cache_dir=str(tmp_path / "kc"))
    prebuild.benchmark_statements(be2)
    assert be2.cache.stats["compiled"] == 0 and be2.cache.stats["hit_disk"] >= 8
    names = [c.spec.name for c in be.choices]
    assert names == [c.spec.name for c in be2.choices]       # generation is deterministic


@pytest.mark.parametrize("dtype", [np.float16, np.int32, np.uint8, np.int16])
@pytest.mark.parametrize("axis", [0, 1])
def test_generated_kernels_compile_for_every_dtype(tmp_path, dtype, axis):
    be = prebuild.PlanBackend(cache_dir=str(tmp_path / "kc"))
    x = be.empty((96, 160), dtype)
    be.empty((96, 160), dtype)[:] = x * 2.0 + x
    shape = (1, 160) if axis == 0 else (96, 1)
    be.empty(shape)[:] = be.max(x, axis=axis) - be.min(x, axis=axis)
    be.empty(shape, np.int32)[:] = be.argmin(x, axis=axis)
    be.empty((96, 160), dtype)[:] = x - be.mean(x, axis=axis)
    assert be.cache.stats["compiled"] == 4


SHAPES_TO_GENERATE = [(1, 1), (3, 1), (1, 3), (2, 2), (7, 5), (1000, 1), (1, 1000), (1000, 2), (1000, 128),
                      (33, 130), (513, 4), (20000, 1), (20000, 64), (64, 20000), (3, 100003), (100003, 3)]


@pytest.mark.parametrize("shape", SHAPES_TO_GENERATE, ids=lambda s: "%dx%d" % s)
def test_every_family_generates_for_degenerate_and_odd_shapes(pb, shape):
    """planning and code generation (no compilation) of the trees every family
    serves, down to single rows, single columns and 1x1: a planner or generator
    that assumes "some operand has more than one column" fails here, not on the
    device"""
    x = pb.empty(shape)

    def plan(out, tree):
        try:
            out[:] = tree
        except planner.NeedsSplit:
            pass            # no single kernel: the backend evaluates such a tree in stages

    for axis in (0, 1):
        line = (1, shape[1]) if axis == 0 else (shape[0], 1)
        plan(pb.empty(shape), pb.exp(x - pb.max(x, axis=axis)) / pb.sum(pb.exp(x - pb.max(x, axis=axis)), axis=axis))
        pb.empty(line, np.int32)[:] = pb.argmax(x, axis=axis)
        pb.empty(line)[:] = pb.sum(x * x, axis=axis)
        plan(pb.empty(shape, np.float16), (x - pb.mean(x, axis=axis)) / pb.sqrt(pb.var(x, axis=axis) + 1e-3))
    pb.empty(shape)[:] = 1.0 / (1.0 + pb.exp(-x))
    for c in pb.choices:
        assert "@NAME@" not in c.spec.source and c.spec.source.count("{") == c.spec.source.count("}")


def test_stochastic_rounding_store_compiles_and_changes_the_plan(tmp_path):
    be = prebuild.PlanBackend(cache_dir=str(tmp_path / "kc"))
    x = be.empty((96, 160))
    plain = be.empty((96, 160), np.float16)
    rounded = be.empty((96, 160), np.float16)
    rounded.rounding = 3
    plain[:] = x * 2.0
    rounded[:] = x * 2.0
    soft = be.empty((96, 160), np.float16)
    soft.rounding = 3
    soft[:] = x - be.max(x, axis=1)               # full-size output of a reduction tree
    assert be.cache.stats["compiled"] == 3
    narrow = be.empty((96, 1))
    narrow.rounding = 3
    with pytest.raises(NotImplementedError):      # the hip backend stages this one through a temporary
        narrow[:] = be.sum(x, axis=1)
    with pytest.raises(NotImplementedError):
        bad = be.empty((4, 4), np.int32)
        bad.rounding = 2
        bad[:] = x[:4, :4] * 1.0


def test_long_rows_of_two_tensors_keep_one_resident(pb):
    """batch-norm backward shape: x and the deltas, 100352 fp16 columns each --
    one row fits the registers of a 1024-lane workgroup, two do not"""
    K, N = 256, 100352
    x, d, out = (pb.empty((K, N), np.float16) for _ in range(3))
    mean, scale = pb.empty((K, 1)), pb.empty((K, 1))
    gg, gb = pb.empty((K, 1)), pb.empty((K, 1))
    n = len(pb.choices)
    pb.begin(Block.update, 0)
    xhat = (x - mean) * scale
    gg[:] = pb.sum(xhat * d, axis=1)
    gb[:] = pb.sum(d, axis=1)
    out[:] = (d - (xhat * gg + gb) / float(N)) * scale
    pb.end(Block.update, 0)
    assert len(pb.choices) == n + 1
    spec = pb.choices[-1].spec
    assert spec.family == "row" and spec.params["NCH"] == 13 and spec.params["passing"] == 1
    # x is loaded once, the deltas once per sweep
    assert spec.source.count(".load_stream(") == 3


def test_softmax_reuses_the_registers_of_x_for_the_exponentials(pb):
    """exp(x - max) is needed by the sum and by the quotient; x by nothing after
    the sum's sweep: the exponentials take x's registers (one exp per element).
    Not when x is read again later, and not for fp16 storage (two elements per
    register)."""
    x, out = pb.empty((1000, 4096)), pb.empty((1000, 4096))

    def softmax(t):
        e = pb.exp(t - pb.max(t, axis=0))
        return e / pb.sum(e, axis=0)

    spec = plan_of(pb, lambda: out.__setitem__(slice(None), softmax(x))).spec
    assert spec.family == "col" and spec.params["over"] == 1
    assert spec.source.count("nh_exp_nonpos(") == 1 and "expf(" not in spec.source and ".put(j, " in spec.source

    spec = plan_of(pb, lambda: out.__setitem__(slice(None), softmax(x) + x)).spec
    assert spec.params["over"] == 0 and ".put(j, " not in spec.source

    xh = pb.empty((1000, 4096), np.float16)
    spec = plan_of(pb, lambda: out.__setitem__(slice(None), softmax(xh))).spec
    assert spec.params["over"] == 0 and ".put(j, " not in spec.source


def test_row_softmax_reuses_registers_when_the_row_is_resident(pb):
    x, out = pb.empty((4096, 1000)), pb.empty((4096, 1000))

    def softmax(t):
        e = pb.exp(t - pb.max(t, axis=1))
        return e / pb.sum(e, axis=1)

    spec = plan_of(pb, lambda: out.__setitem__(slice(None), softmax(x))).spec
    assert spec.family == "row" and spec.params["NCH"] > 0 and spec.params["over"] == 1
    assert spec.source.count("nh_exp_nonpos(") == 1 and "expf(" not in spec.source
    # 16-bit rows leave registers free: the exponentials get float32 registers of their own
    for dt in (np.float16, bfloat16):
        xh, outh = pb.empty((4096, 1000), dt), pb.empty((4096, 1000), dt)
        spec = plan_of(pb, lambda: outh.__setitem__(slice(None), softmax(xh))).spec
        assert spec.params["over"] == 0 and spec.params["kept"] == 1
        assert spec.source.count("nh_exp_nonpos(") == 1 and "float val" in spec.source
    # ... unless the row itself fills them ((64, 131072) fp16: 16 tiles of 1024 lanes)
    xh, outh = pb.empty((512, 131072), np.float16), pb.empty((512, 131072), np.float16)
    spec = plan_of(pb, lambda: outh.__setitem__(slice(None), softmax(xh))).spec
    # (then maximum and sum share a sweep as a running pair instead: two sweeps, not three)
    assert spec.params["NCH"] == 16 and spec.params["kept"] == 0
    assert spec.source.count("nh_op_lse::stepn<8>(") == 1 and spec.source.count("nh_exp_nonpos(") == 1
    # few rows too long for one workgroup's registers are spread over several
    # workgroups and stay resident
    xl, outl = pb.empty((16, 1 << 20)), pb.empty((16, 1 << 20))
    ch = plan_of(pb, lambda: outl.__setitem__(slice(None), softmax(xl)))
    assert ch.spec.family == "rowcoop" and ch.grid == (16, 16, 1) and ch.spec.params["over"] == 1
    assert ch.spec.source.count("nh_exp_nonpos(") == 1
    # many such rows: a workgroup per row keeps the first tiles in LDS and registers and streams
    # the rest in every sweep, as a loop proper -- nothing to lend registers.  Maximum and sum
    # of exponentials share the first sweep (a running pair), one pass over memory less
    xl, outl = pb.empty((512, 1 << 20)), pb.empty((512, 1 << 20))
    spec = plan_of(pb, lambda: outl.__setitem__(slice(None), softmax(xl))).spec
    assert spec.family == "row" and spec.params["over"] == 0
    assert (spec.params["NCH"], spec.params["parked"], spec.params["held"]) == (256, 9, 16)
    assert spec.source.count("for (int kb = 0; kb < 28; kb += 4)") == 2
    assert spec.source.count("#pragma unroll 1\n    for (int kb = 28; kb < 256; kb += 4)") == 2
    assert spec.source.count("nh_op_lse::stepn<4>(") == 2 and spec.source.count("nh_exp_nonpos(") == 2
    saved = Program.__init__

    def two_sweeps(self, *a, **k):
        saved(self, *a, **k)
        self.online_lse = False
    try:
        Program.__init__ = two_sweeps
        spec = plan_of(pb, lambda: outl.__setitem__(slice(None), softmax(xl))).spec
    finally:
        Program.__init__ = saved
    assert spec.source.count("for (int kb = 0; kb < 28; kb += 4)") == 3 and "stepn" not in spec.source


def test_more_than_2_31_elements_stay_two_dimensional(pb):
    """extents travel as 32-bit kernel arguments: a contiguous elementwise
    program is flattened to one long row only while that row fits"""
    big, small = (60000, 50000), (6000, 5000)
    x, y, out = (pb.empty(big) for _ in range(3))
    spec = plan_of(pb, lambda: out.__setitem__(slice(None), x * 0.5 + y)).spec
    assert spec.family == "ew" and spec.params["LY"] * spec.params["LX"] == 256
    assert pb.choices[-1].grid[0] * spec.params["LX"] * spec.params["V"] >= big[1]
    assert pb.choices[-1].grid[0] * spec.params["LX"] * spec.params["V"] < 2 * big[1]      # a row, not the whole tensor
    x, y, out = (pb.empty(small) for _ in range(3))
    ch = plan_of(pb, lambda: out.__setitem__(slice(None), x * 0.5 + y))
    assert ch.grid[0] * ch.spec.block * ch.spec.params["V"] >= small[0] * small[1] and ch.grid[1] == 1   # flattened


# ---- row family: LDS as a second tier of residence -------------------------------------------
def _bn_backward_group(pb, shape, dtype=np.float16):
    """the statements of batch-norm backward as one fused group (no device needed)"""
    x, d, o = pb.empty(shape, dtype), pb.empty(shape, dtype), pb.empty(shape, dtype)
    xsum, xvar, gamma, gg, gb = (pb.empty((shape[0], 1)) for _ in range(5))
    inv_v = 1.0 / pb.sqrt(xvar + 1e-5)
    xhat = (x - xsum) * inv_v
    pb.begin(Block.update, 0)
    gg[:] = pb.sum(xhat * d, axis=1)
    gb[:] = pb.sum(d, axis=1)
    o[:] = ((d - (xhat * gg + gb) / float(shape[1])) * gamma) * inv_v
    pb.end(Block.update, 0)
    return pb.choices[-1]


def test_row_operands_without_registers_go_to_lds(tmp_path):
    pb = prebuild.PlanBackend(cache_dir=str(tmp_path / "kc"), compile_kernels=True)      # hiprtc takes 144 KB of LDS
    ch = _bn_backward_group(pb, (256, 100352))
    p = ch.spec.params
    assert ch.spec.family == "row" and (p["NCH"], p["passing"], p["parked"], p["held"]) == (13, 1, 9, 3)
    assert "__shared__ __attribute__((aligned(16))) nh_raw<nh_f16, 8> park" in ch.spec.source
    pb = prebuild.PlanBackend(cache_dir=str(tmp_path / "kc"), compile_kernels=False)
    # rows of 25 tiles: one operand split between LDS and registers, the other fetched per sweep
    p = _bn_backward_group(pb, (256, 200704)).spec.params
    assert (p["NCH"], p["passing"], p["parked"], p["held"]) == (25, 2, 9, 16)
    # a single sweep has nothing to come back for: streamed, no LDS
    x, col = pb.empty((1000, 131072)), pb.empty((1000, 1))
    p = plan_of(pb, lambda: col.__setitem__(slice(None), pb.sum(x, axis=1))).spec.params
    assert (p["NCH"], p["parked"], p["held"]) == (0, 0, 0)
    # few very long rows swept twice: workgroups of a row cooperate on shares beyond 16 tiles
    ch = _bn_backward_group(pb, (64, 1605632))
    assert ch.spec.family == "rowcoop" and ch.spec.params["NCH"] == 49 and ch.spec.params["parked"] == 9
    # a device with 64 KB of LDS per workgroup gets 48 KB worth of parked tiles
    saved = planner.ROW_PARK_BYTES
    try:
        planner.limit_lds(64 << 10)
        p = _bn_backward_group(pb, (256, 100352)).spec.params
        assert (p["parked"], p["held"]) == (3, 3)
        planner.limit_lds(8 << 10)
        p = _bn_backward_group(pb, (256, 100352)).spec.params
        assert (p["parked"], p["held"], p["passing"]) == (0, 0, 1)
    finally:
        planner.ROW_PARK_BYTES = saved


def test_cooperating_workgroups_take_mean_and_variance_with_one_exchange(pb, monkeypatch):
    """sum((x - mean)^2) over a row that several workgroups share: each takes the
    squares around the mean of its own part, the parts are combined after the one
    exchange that also carries the sums; other second sweeps still wait twice"""
    x, out = pb.empty((16, 1 << 20)), pb.empty((16, 1 << 20))

    def norm():
        out[:] = (x - pb.mean(x, axis=1)) / pb.sqrt(pb.var(x, axis=1) + 1e-5)

    ch = plan_of(pb, norm)
    # (float partials of cooperating rows travel tagged: an exchange is one polling loop, no ticket)
    waits = lambda spec: spec.source.count("nh_ticket_take(ctr)") + spec.source.count("s_x is free again")
    assert ch.spec.family == "rowcoop" and waits(ch.spec) == 1 and ch.spec.params["tagged"]
    assert "nh_ticket_take" not in ch.spec.source and "ctr + 1" not in ch.spec.source
    assert "const float mu" in ch.spec.source and "n_loc" in ch.spec.source
    monkeypatch.setattr(codegen, "MERGED_MOMENTS", False)
    assert waits(plan_of(pb, norm).spec) == 2
    monkeypatch.setattr(codegen, "MERGED_MOMENTS", True)
    monkeypatch.setattr(codegen, "TAGGED_EXCHANGE", False)
    assert plan_of(pb, norm).spec.source.count("nh_ticket_take(ctr)") == 1
    monkeypatch.setattr(codegen, "TAGGED_EXCHANGE", True)
    # a row maximum with its position travels as a (value, index) pair: no room for a tag
    am = pb.empty((16, 1), dtype=np.int32)
    ch = plan_of(pb, lambda: am.__setitem__(slice(None), pb.argmax(x, axis=1)))
    if ch.spec.family == "rowcoop":
        assert not ch.spec.params["tagged"] and "nh_ticket_take(ctr)" in ch.spec.source
    # the same down columns that several workgroups share
    xc, outc = pb.empty((32000, 256)), pb.empty((32000, 256))

    def colnorm():
        outc[:] = (xc - pb.mean(xc, axis=0)) / pb.sqrt(pb.var(xc, axis=0) + 1e-5)

    ch = plan_of(pb, colnorm)
    assert ch.spec.family == "colcoop" and ch.spec.source.count("nh_ticket_take(ctr)") == 1
    monkeypatch.setattr(codegen, "MERGED_MOMENTS", False)
    assert plan_of(pb, colnorm).spec.source.count("nh_ticket_take(ctr)") == 2
    monkeypatch.setattr(codegen, "MERGED_MOMENTS", True)
    # a second sweep of another form (absolute deviations) needs the finished mean everywhere
    ch = plan_of(pb, lambda: out.__setitem__(slice(None), x / pb.sum(pb.absolute(x - pb.mean(x, axis=1)), axis=1)))
    assert ch.spec.family == "rowcoop" and waits(ch.spec) == 2


def test_the_cheaper_exponential_is_for_arguments_below_their_own_maximum_only(pb):
    x, y, out = pb.empty((1000, 256)), pb.empty((1000, 256)), pb.empty((1000, 256))
    for axis in (0, 1):
        src = plan_of(pb, lambda: out.__setitem__(slice(None), pb.exp(x - pb.max(x, axis=axis)))).spec.source
        assert "nh_exp_nonpos(" in src and "expf(" not in src
        src = plan_of(pb, lambda: out.__setitem__(slice(None), pb.exp(x * 2.0 - pb.max(x * 2.0, axis=axis)))).spec.source
        assert "nh_exp_nonpos(" in src and "expf(" not in src
        # the maximum of something else, a minimum, the difference the other way round: expf
        for tree in (lambda: pb.exp(x - pb.max(y, axis=axis)), lambda: pb.exp(x - pb.min(x, axis=axis)),
                     lambda: pb.exp(pb.max(x, axis=axis) - x), lambda: pb.exp(x + pb.max(x, axis=axis))):
            src = plan_of(pb, lambda: out.__setitem__(slice(None), tree())).spec.source
            assert "expf(" in src and "nh_exp_nonpos(" not in src


# ---- launch shapes away from the benchmark configurations ---------------------------------
def _softmax(pb, x, axis):
    e = pb.exp(x - pb.max(x, axis=axis))
    return e / pb.sum(e, axis=axis)


def _norm(pb, x, axis):
    return (x - pb.mean(x, axis=axis)) / pb.sqrt(pb.var(x, axis=axis) + 1e-5)


def test_short_rows_get_teams_that_fetch_whole_cache_lines(pb):
    """four tiles per lane, but never fewer lanes per row than fetch 128 bytes per load"""
    for shape, dtype, want in (((100000, 64), np.float32, (8, 2)), ((100000, 64), np.float16, (8, 1)),
                               ((50000, 32), np.float32, (8, 1)), ((20000, 256), np.float32, (16, 4)),
                               ((20000, 1000), np.float32, (64, 4))):
        x, out = pb.empty(shape, dtype), pb.empty(shape, dtype)
        p = plan_of(pb, lambda: out.__setitem__(slice(None), _softmax(pb, x, 1))).spec.params
        assert (p["LX"], p["NCH"]) == want, (shape, dtype, p)


def test_column_strips_narrow_until_every_compute_unit_has_one(pb):
    """the widest strip whose rows fit in registers, then narrower ones -- down to 32-byte
    row pieces -- while there are fewer strips than compute units"""
    for shape, dtype, strips, lx in (((512, 4096), np.float32, 256, 4), ((256, 8192), np.float32, 256, 8),
                                     ((1000, 4096), np.float16, 256, 2), ((1000, 65536), np.float32, 2048, 8)):
        x, out = pb.empty(shape, dtype), pb.empty(shape, dtype)
        ch = plan_of(pb, lambda: out.__setitem__(slice(None), _softmax(pb, x, 0)))
        assert ch.spec.family == "col" and ch.grid[0] == strips and ch.spec.params["LX"] == lx, (shape, ch.grid, ch.spec.params)
    # up to 2048 rows narrow strips are preferred to workgroups that wait for each other
    x, out = pb.empty((2000, 2048), np.float16), pb.empty((2000, 2048), np.float16)
    assert plan_of(pb, lambda: out.__setitem__(slice(None), _norm(pb, x, 0))).spec.family == "col"


def test_the_cooperative_column_family_is_for_matrices_of_20_to_48_megabytes(pb):
    x, out = pb.empty((32000, 256)), pb.empty((32000, 256))                  # 32 MB
    assert plan_of(pb, lambda: out.__setitem__(slice(None), _softmax(pb, x, 0))).spec.family == "colcoop"
    for shape in ((4096, 1000), (30000, 1000)):                              # 16 MB, 120 MB: in stages
        x, out = pb.empty(shape), pb.empty(shape)
        with pytest.raises(planner.NeedsSplit):
            out[:] = _softmax(pb, x, 0)
    # 16-bit matrices whose rows per lane would overflow the registers of a cooperating workgroup
    x, out = pb.empty((5000, 5000), np.float16), pb.empty((5000, 5000), np.float16)
    with pytest.raises(planner.NeedsSplit):
        out[:] = _softmax(pb, x, 0)


def test_one_tall_strip_of_long_chunks_takes_1024_lanes(pb):
    x, line = pb.empty((600000, 64), np.float16), pb.empty((1, 64))
    ch = plan_of(pb, lambda: line.__setitem__(slice(None), pb.sum(x, axis=0)))
    assert ch.spec.family == "colsplit" and ch.spec.block == 1024 and ch.grid[0] == 1
    x = pb.empty((32000, 256))
    ch = plan_of(pb, lambda: pb.empty((1, 256)).__setitem__(slice(None), pb.max(x, axis=0)))
    assert ch.spec.family == "colsplit" and ch.spec.block == 512


def test_the_join_of_the_waves_reads_lds_in_batches(pb):
    """(waves - 1) x V reads issued all at once took a 1024-lane kernel with eight values
    per lane to over 200 registers; plain values are joined like pairs, a column shared by
    adjacent lanes"""
    x, out = pb.empty((32000, 256)), pb.empty((32000, 256))
    src = plan_of(pb, lambda: out.__setitem__(slice(None), _norm(pb, x, 0))).spec.source
    assert "const int fcol = threadIdx.x / " in src and "for (int y = 1; y < 16; ++y)" not in src


def test_rows_pair_maximum_and_sum_only_where_it_saves_a_pass_or_an_exchange(pb):
    def paired(shape, dtype):
        x, out = pb.empty(shape, dtype), pb.empty(shape, dtype)
        ch = plan_of(pb, lambda: out.__setitem__(slice(None), _softmax(pb, x, 1)))
        return ch.spec.family, "nh_op_lse::stepn" in ch.spec.source

    assert paired((4096, 1000), np.float32) == ("row", False)          # resident: three sweeps over registers
    assert paired((4096, 4096), np.float16) == ("row", False)          # resident, exponentials kept in spare registers
    assert paired((512, 131072), np.float16) == ("row", True)          # resident but no register left to keep them
    assert paired((1000, 262144), np.float32) == ("row", True)         # partly streamed
    assert paired((64, 1048576), np.float32) == ("rowcoop", True)      # shares that do not fit
    assert paired((16, 1048576), np.float32) == ("rowcoop", False)     # resident fp32 shares: exponentials take x's registers
    assert paired((16, 1605632), np.float16) == ("rowcoop", True)      # resident 16-bit shares of 13 tiles: one exchange less
    assert paired((64, 131072), np.float16) == ("rowcoop", False)      # ... but not shares of 4 tiles


# ---- outputs that overlap operands through another view ---------------------------------
def test_output_hazards_are_found_by_byte_range(pb):
    """a written slot that shares memory with another slot of the program
    through a different view (reference semantics: nervanacpu.py:476-477, the
    right-hand side is finished before the store)"""
    base = 1 << 32
    x = prebuild.ShapeTensor(pb, (12, 8), ptr=base)
    y = prebuild.ShapeTensor(pb, (12, 8), ptr=base + (1 << 20))
    row = prebuild.ShapeTensor(pb, (1, 8), ptr=base + 2 * 8 * 4, base=x)             # x[2:3, :]
    col = prebuild.ShapeTensor(pb, (12, 1), ptr=base + 4, strides=(8, 1), base=x)    # x[:, 1:2]
    shifted = prebuild.ShapeTensor(pb, (10, 8), ptr=base + 8 * 4, base=x)            # x[1:11]
    head = prebuild.ShapeTensor(pb, (10, 8), ptr=base, base=x)                       # x[0:10]
    tree = lambda out, value: OpTreeNode({"op": "assign"}, out, value)

    def hazards(*stmts):
        prog = Program()
        for st in stmts:
            prog.add_statement(st)
        return [t.index for t in prog.finalize().output_hazards()]

    assert hazards(tree(x, y + x)) == []                      # same elements: fine
    assert hazards(tree(x, y * 2.0)) == []
    assert hazards(tree(x, y + row)) == [0]                   # x[:] = y + x[2:3, :]
    assert hazards(tree(x, y * col)) == [0]                   # x[:] = y * x[:, 1:2]
    assert hazards(tree(col, pb.sum(x, axis=1))) == []        # a line's result stored inside that very line: fine
    assert hazards(tree(row, pb.max(x, axis=0))) == []
    assert hazards(tree(col, pb.sum(x * y, axis=1) * 2.0)) == []
    assert hazards(tree(x, x - pb.max(x, axis=0) + row)) == [0]       # ... but not a full-shape result
    assert hazards(tree(shifted, head)) == [0]                # x[1:11] = x[0:10]
    assert hazards(tree(y, x + row)) == []                    # overlapping READS are no hazard


def test_fusion_group_refuses_statements_that_overlap_through_other_views():
    """_can_join on stub tensors (no device): the lanes of a fused elementwise
    kernel only ever touch their own elements, so a tensor the group writes
    may not meet another tensor of the group through a different view"""
    from neon_amd.backends import NervanaHIP
    be = object.__new__(NervanaHIP)
    be._pending, be._pending_post, be._pending_sig = [], [], None
    be._pending_vectors, be._sig_vectors = [], ()
    T = be.tensor_cls
    base = 1 << 32
    x = T(be, (12, 8), gpudata=base)
    y = T(be, (10, 8), gpudata=base + (1 << 20))
    z = T(be, (10, 8), gpudata=base + (2 << 20))
    w = T(be, (10, 8), gpudata=base + (3 << 20))
    tree = lambda out, value: OpTreeNode({"op": "assign"}, out, value)

    def offer(t):
        post = t.traverse([])
        ok = be._can_join(t, post)
        if ok:
            be._pending.append(t)
            be._pending_post.append(post)
        return ok

    assert offer(tree(x[1:11], y * 2.0))                      # opens the group
    assert offer(tree(w, x[1:11] + 1.0))                      # the same view of x: the same elements
    assert not offer(tree(z, x[0:10] + 1.0))                  # x shifted by a row: other lanes' elements
    assert not offer(tree(x[0:10], z * 1.0))                  # writing over what the group has written, shifted
    be._pending, be._pending_post = [], []
    assert offer(tree(z, y * 2.0))
    inside_z = T(be, (1, 1), gpudata=z.gpudata + 29 * 4)      # one element in the interior of a written tensor
    inside_y = T(be, (1, 1), gpudata=y.gpudata + 29 * 4)      # ... of a tensor that is only read: fine
    assert not offer(tree(w, w + inside_z))
    assert offer(tree(w, w + inside_y))
    be._pending, be._pending_post = [], []
    assert not offer(tree(x[1:11], x[0:10] * 2.0))            # overlaps within itself: never fused
