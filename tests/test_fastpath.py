"""The C replayer of repeated statements (neon_amd/csrc/fastpath.c) against the
Python walk it stands in for, without a GPU: the launch function is a ctypes
callback that only counts."""
import ctypes

import numpy as np
import pytest

from neon_amd.backends.hip import fastpath
from neon_amd.backends.hip.prebuild import PlanBackend, ShapeTensor
from neon_amd.backends.nervanahip import NervanaHIPBase


class GeomTensor(ShapeTensor):
    """shape-only tensor carrying the layout tuple the launch key is made of"""
    def __init__(self, *args, **kw):
        super(GeomTensor, self).__init__(*args, **kw)
        self._geom = (self.ptr, self.shape, self.strides, self.dtype.char, 0)


class _Walker(object):
    _walk_key = NervanaHIPBase._walk_key


def python_key(out, value):
    parts, raw = [], []
    node = ({"op": "assign"}, out, value)
    _Walker()._walk_key(node, parts.append, raw.append, GeomTensor)
    parts.append("|")
    return tuple(parts), raw


class Entry(object):
    def __init__(self, fast):
        self.fast = fast


@pytest.fixture()
def rig():
    mod = fastpath.load()
    be = PlanBackend(compile_kernels=False)
    calls = []
    verdict = [0]

    @ctypes.CFUNCTYPE(ctypes.c_int, ctypes.c_void_p)
    def launch(rec):
        calls.append(rec)
        return verdict[0]

    cache = {}
    rp = mod.Replayer(cache, GeomTensor, ctypes.cast(launch, ctypes.c_void_p).value)
    t = lambda shape, dtype=np.float32: GeomTensor(be, shape, dtype)
    return mod, be, rp, cache, calls, verdict, t, launch


def trees(be, t):
    x, y, o = t((64, 32)), t((64, 32)), t((64, 32))
    col, row = t((64, 1)), t((1, 32))
    idx = t((1, 32), np.int32)
    return [
        (o, be.sig(0.5 * x + 2.0 * y)),
        (o, x),
        (o, 3),
        (o, x * 2 - 1 / y + col * row),
        (row, be.sum(x, axis=0)),
        (col, be.max(x - be.max(x, axis=1), axis=1)),
        (row, be.argmax(x, axis=0)),
        (o, be.exp(x - be.max(x, axis=0)) / be.sum(be.exp(x - be.max(x, axis=0)), axis=0)),
        (row, be.sum(be.onehot(idx, axis=0) * be.safelog(x), axis=0)),
        (o, -x + abs(y) ** 2.5),
        (o, be.sqrt(be.var(x, axis=1) + 1e-6)),
        (o, x * np.float64(0.25) + True),            # subclasses of float and int
    ]


def test_c_key_is_the_python_key(rig):
    mod, be, rp, cache, calls, verdict, t, _ = rig
    for out, value in trees(be, t):
        want_key, want_raw = python_key(out, value)
        key, raw = rp.key(out, value)
        assert key == want_key and hash(key) == hash(want_key)
        assert raw == want_raw


def test_c_group_key_is_the_python_group_key(rig):
    from neon_amd.backends.backend import OpTreeNode
    mod, be, rp, cache, calls, verdict, t, _ = rig

    class Keyer(object):
        tensor_cls = GeomTensor
        _launch_key = NervanaHIPBase._launch_key

    pairs = trees(be, t)
    for out, _ in pairs:
        out.rounding = 0
    for group in (pairs[:1], pairs[:3], pairs[3:8], pairs):
        assigns = [OpTreeNode({"op": "assign", "shape": out.shape}, out, value) for out, value in group]
        want_key, want_raw = Keyer()._launch_key(assigns)
        key, raw = rp.key_group(assigns)
        assert key == want_key and hash(key) == hash(want_key) and raw == want_raw
    # one statement: the key replay() looks up
    out, value = pairs[0]
    assert rp.key_group([OpTreeNode({"op": "assign"}, out, value)]) == rp.key(out, value)
    with pytest.raises(TypeError):
        rp.key_group([OpTreeNode({"op": "assign"}, out, OpTreeNode.build("rand", None, None) * value)])
    with pytest.raises(TypeError):
        rp.key_group([(1, 2)])
    assert rp.key_group([]) == ((), [])


def test_what_the_replayer_leaves_to_python(rig):
    mod, be, rp, cache, calls, verdict, t, _ = rig
    x, o = t((8, 8)), t((8, 8))
    assert rp.replay(o, x + 1.0) == 0                        # never seen
    assert rp.replay(o, "text") == 0 and rp.replay(o, [1, 2]) == 0
    from neon_amd.backends.backend import OpTreeNode
    assert rp.replay(o, OpTreeNode.build("rand", None, None) * x) == 0                  # random trees are never replayed
    plain = ShapeTensor(be, (8, 8))
    assert rp.replay(o, plain + 1.0) == 0                    # a tensor of another class
    deep = x
    for _ in range(300):
        deep = deep + 1.0
    assert rp.replay(o, deep) == 0                           # deeper than the C walk goes
    with pytest.raises(TypeError):
        rp.key(o, "text")
    assert calls == [] and rp.replayed == 0


def test_replay_issues_the_records_in_order(rig):
    mod, be, rp, cache, calls, verdict, t, _ = rig
    x, o = t((8, 8)), t((8, 8))
    key, raw = python_key(o, 0.5 * x + 2.0)
    keep = object()
    recs = mod.Records([0x1000, 0x2000, 0x3000], raw, keep)
    assert recs.launches == 3
    cache[key] = Entry(recs)
    assert rp.replay(o, 0.5 * x + 2.0) == 1
    assert calls == [0x1000, 0x2000, 0x3000]
    assert (rp.replayed, rp.launches) == (1, 3)
    # other numbers: the Python path re-binds the constants, then tells the records
    del calls[:]
    assert rp.replay(o, 0.25 * x + 2.0) == 0 and calls == []
    recs.set_numbers([0.25, 2.0])
    assert rp.replay(o, 0.25 * x + 2.0) == 1 and len(calls) == 3
    assert rp.replay(o, 0.5 * x + 2.0) == 0
    # an entry that has no records yet, or something else in their place
    cache[key] = Entry(None)
    assert rp.replay(o, 0.25 * x + 2.0) == 0
    cache[key] = Entry([1, 2])
    assert rp.replay(o, 0.25 * x + 2.0) == 0
    # the same tree over another tensor is another statement
    cache[key] = Entry(recs)
    assert rp.replay(t((8, 8)), 0.25 * x + 2.0) == 0
    # a cleared cache forgets
    cache.clear()
    assert rp.replay(o, 0.25 * x + 2.0) == 0


def test_replay_notes_the_cooperative_plans_it_launched(rig):
    """records may carry (key, plan) pairs of kernels whose workgroups wait
    for one another: every replay enters them in the dict the replayer was
    given, where the backend finds them at its next synchronisation"""
    mod, be, rp, cache, calls, verdict, t, launch = rig
    x, o = t((8, 8)), t((8, 8))
    key, raw = python_key(o, x * x)
    plan_a, plan_b = object(), object()
    recs = mod.Records([0x10, 0x20], raw, None, (("a", plan_a), ("b", plan_b)))
    cache[key] = Entry(recs)
    assert rp.replay(o, x * x) == 0 and calls == []          # this replayer has nowhere to note them
    pending = {}
    rp2 = mod.Replayer(cache, GeomTensor, ctypes.cast(launch, ctypes.c_void_p).value, pending)
    assert rp2.replay(o, x * x) == 1 and calls == [0x10, 0x20]
    assert pending == {"a": plan_a, "b": plan_b}
    pending.clear()                                          # (the backend empties it in place)
    assert rp2.replay(o, x * x) == 1 and pending == {"a": plan_a, "b": plan_b}
    verdict[0] = 3
    pending.clear()
    assert rp2.replay(o, x * x) == -3 and pending == {}       # nothing noted for a launch that failed
    verdict[0] = 0
    cache[key] = Entry(mod.Records([0x10], raw, None, None)) # no cooperative plans: as without the argument
    assert rp.replay(o, x * x) == 1
    for bad in ([("a", plan_a)], (("a",),), ("ab",), 5):
        with pytest.raises(TypeError):
            mod.Records([0x10], raw, None, bad)
    with pytest.raises(TypeError):
        mod.Replayer(cache, GeomTensor, ctypes.cast(launch, ctypes.c_void_p).value, [])


def test_launch_errors_come_back_negated(rig):
    mod, be, rp, cache, calls, verdict, t, _ = rig
    x, o = t((8, 8)), t((8, 8))
    key, raw = python_key(o, x * x)
    cache[key] = Entry(mod.Records([0x10, 0x20], raw, None))
    verdict[0] = 7
    assert rp.replay(o, x * x) == -7
    assert calls == [0x10] and rp.replayed == 0              # stopped at the failing launch
    with pytest.raises(ValueError):
        mod.Records([0], [], None)                           # a null record is refused at construction
    with pytest.raises(TypeError):
        mod.Records([1], ["a"], None)


def test_records_keep_their_owner_alive(rig):
    import gc
    import weakref
    mod = rig[0]

    class Owner(object):
        pass
    owner = Owner()
    ref = weakref.ref(owner)
    recs = mod.Records([0x10], [], owner)
    del owner
    gc.collect()
    assert ref() is not None
    del recs
    gc.collect()
    assert ref() is None


def test_cycles_through_the_replayer_are_collected(rig):
    """backend -> replayer -> launch cache -> entry -> ... -> backend: the
    collector has to see through the C objects"""
    import gc
    import weakref
    mod, be, rp, cache, calls, verdict, t, launch = rig

    class Holder(object):
        pass
    holder = Holder()
    own_cache = {}
    holder.replayer = mod.Replayer(own_cache, GeomTensor, ctypes.cast(launch, ctypes.c_void_p).value)
    holder.records = mod.Records([0x10], [], holder)
    own_cache["entry"] = holder
    ref = weakref.ref(holder)
    del holder, own_cache
    gc.collect()
    assert ref() is None


def test_random_trees_have_no_key(rig):
    from neon_amd.backends.backend import OpTreeNode
    mod, be, rp, cache, calls, verdict, t, _ = rig
    x, o = t((8, 8)), t((8, 8))
    with pytest.raises(TypeError):
        rp.key(o, OpTreeNode.build("rand", None, None) * x)


# ---- on the device: the third and later calls of a statement go through the C replayer -------
@pytest.mark.gpu
def test_replayed_statements_match_the_oracle(hip, cpu):
    assert hip._replayer is not None, "the C replayer is the default path"
    rs = np.random.RandomState(5)
    a, b = rs.randn(300, 70).astype(np.float32), rs.randn(300, 70).astype(np.float32)
    hx, hy, ho = hip.array(a), hip.array(b), hip.empty((300, 70))
    hred = hip.empty((1, 70))
    cx, cy, co = cpu.array(a), cpu.array(b), cpu.empty((300, 70))
    cred = cpu.empty((1, 70))
    before = hip._replayer.replayed
    stats = hip.plan_stats
    for k in range(8):
        scale = 0.5 if k < 5 else 0.125 * k            # the numbers change at the sixth call
        if k == 3:                                     # the data changes, the statement does not
            a2 = rs.randn(300, 70).astype(np.float32)
            hx.set(a2)
            cx.set(a2)
        for be, x, y, o, red in ((hip, hx, hy, ho, hred), (cpu, cx, cy, co, cred)):
            o[:] = be.sig(scale * x + 2.0 * y)
            red[:] = be.sum(o * x, axis=0)
        np.testing.assert_allclose(ho.get(), co.get(), rtol=1e-5, atol=1e-6)
        np.testing.assert_allclose(hred.get(), cred.get(), rtol=1e-4, atol=1e-4)
    # calls 0 record, 1 replay in Python and hand over the records, 2..4 run in C; the changed
    # numbers go back through Python once (6, 7 differ from each other too)
    assert hip._replayer.replayed - before >= 6
    after = hip.plan_stats
    assert after["launches"] - stats["launches"] == 16 and after["replayed"] - stats["replayed"] >= 12


@pytest.mark.gpu
def test_replayer_steps_aside_for_groups_rounding_and_capture(hip, cpu):
    from neon_amd.backends.backend import Block
    rs = np.random.RandomState(6)
    a = rs.randn(64, 48).astype(np.float32)
    hx, ho, hp = hip.array(a), hip.empty((64, 48)), hip.empty((64, 48))
    for _ in range(4):
        ho[:] = hx * 3.0
    np.testing.assert_array_equal(ho.get(), a * np.float32(3.0))
    # the same statement inside a fused group must join the group, not be replayed on its own
    before = hip.plan_stats["launches"]
    hip.begin(Block.update, 0)
    ho[:] = hx * 3.0
    hp[:] = ho + 1.0
    hip.end(Block.update, 0)
    assert hip.plan_stats["launches"] - before == 1
    np.testing.assert_array_equal(hp.get(), a * np.float32(3.0) + np.float32(1.0))
    # captured statements are not launched at all
    ho.fill(0)
    with hip.capture() as groups:
        ho[:] = hx * 3.0
    assert len(groups) == 1 and not ho.get().any()
    # a stochastically rounded target never takes a recorded launch
    h16 = hip.empty((64, 48), dtype=np.float16)
    for _ in range(3):
        h16[:] = hx * 3.0
    exact = h16.get().copy()
    h16.rounding = 4
    h16[:] = hx * 3.0
    got = h16.get()
    assert np.all((got.view(np.uint16) & 0x3f) == 0) and not np.array_equal(got, exact)
    h16.rounding = 0
    h16[:] = hx * 3.0
    np.testing.assert_array_equal(h16.get(), exact)


@pytest.mark.gpu
def test_fusion_groups_are_keyed_by_one_walk_and_still_behave(hip):
    rs = np.random.RandomState(12)
    x0, y0 = rs.randn(96, 40).astype(np.float32), rs.randn(96, 40).astype(np.float32)
    x, y = hip.array(x0), hip.array(y0)
    a, b, s = hip.empty((96, 40)), hip.empty((96, 40)), hip.empty((1, 40))
    # the same group again and again, with other numbers and other data in between
    for k, scale in enumerate((2.0, 2.0, 2.0, 0.5, 0.5)):
        if k == 2:
            x0 = rs.randn(96, 40).astype(np.float32)
            x.set(x0)
        before = hip.plan_stats["launches"]
        with hip.fused():
            a[:] = x * scale
            b[:] = a + y
        assert hip.plan_stats["launches"] - before == 1
        np.testing.assert_array_equal(a.get(), x0 * np.float32(scale))
        np.testing.assert_array_equal(b.get(), x0 * np.float32(scale) + y0)
    # a statement that cannot join (a reduction among elementwise assigns) splits the group
    for _ in range(3):
        with hip.fused():
            a[:] = x * 3.0
            s[:] = hip.sum(a, axis=0)
            b[:] = a - 1.0
        np.testing.assert_array_equal(a.get(), x0 * np.float32(3.0))
        np.testing.assert_allclose(s.get(), (x0 * np.float32(3.0)).sum(axis=0, keepdims=True), rtol=1e-5, atol=1e-5)
        np.testing.assert_array_equal(b.get(), x0 * np.float32(3.0) - np.float32(1.0))
    # reading a tensor inside the group sees everything written before
    with hip.fused():
        a[:] = x + 7.0
        seen = a.get()
        b[:] = a * 2.0
    np.testing.assert_array_equal(seen, x0 + np.float32(7.0))
    np.testing.assert_array_equal(b.get(), (x0 + np.float32(7.0)) * np.float32(2.0))
    # an exception inside the block drops what was queued
    a.fill(0)
    with pytest.raises(RuntimeError):
        with hip.fused():
            a[:] = x + 1.0
            raise RuntimeError("caller's")
    assert not a.get().any()
    a[:] = x + 1.0
    np.testing.assert_array_equal(a.get(), x0 + np.float32(1.0))


def test_c_node_builder_builds_the_nodes_python_builds():
    """every elementwise op over every kind of operand pair: same node class,
    same op dict (same key order), same operands -- or the same refusal"""
    import neon_amd.backends  # noqa: F401  (installs the C builder on this package's API copy)
    from neon_amd.backends import backend as api
    from neon_amd.backends.backend import OpCollection, OpTreeNode
    assert api._c_ew_node is not None
    be = PlanBackend(compile_kernels=False)
    full, col, row, one = be.empty((5, 7)), be.empty((5, 1)), be.empty((1, 7)), be.empty((1, 1))
    vec = ShapeTensor(be, (9,))
    vec.shape = (9,)                                     # a 1-d shape is padded
    cube = be.empty((5, 1))
    cube.shape = (2, 3, 4)                               # more than two axes: left to Python
    listy = be.empty((5, 1))
    listy.shape = [5, 7]                                 # a list, not a tuple: left to Python
    node = full * col
    operands = [full, col, row, one, vec, cube, listy, node, node + 1.0, 2.5, 3, True, np.float64(0.5), None, "text", [1, 2]]
    ops = sorted(set(OpCollection.ew_ops) - {"assign"}) + ["assign", "sum", "bogus"]
    c_builder = api._c_ew_node

    def build_both(op, a, b):
        results = []
        for use_c in (True, False):
            api._c_ew_node = c_builder if use_c else None
            try:
                results.append(OpTreeNode.build(op, a, b) if op not in ("assign", "sum") else
                               (c_builder(op, a, b) if use_c else None))
            except Exception as e:                       # noqa: BLE001  (compared, not handled)
                results.append(type(e))
        api._c_ew_node = c_builder
        return results

    checked = 0
    for op in ops:
        for a in operands:
            for b in operands:
                got, want = build_both(op, a, b)
                if op in ("assign", "sum", "bogus"):
                    if op != "bogus":
                        assert got is None               # never the C builder's business
                    else:
                        assert got is want               # the same refusal, whichever it is
                    continue
                if isinstance(want, tuple):
                    assert type(got) is type(want) is OpTreeNode, (op, a, b)
                    assert got[0] == want[0] and list(got[0]) == list(want[0]), (op, a, b, got[0], want[0])
                    assert type(got[0]["shape"]) is tuple
                    assert got[1] is a and got[2] is b
                    checked += 1
                else:
                    assert got is want, (op, a, b, got, want)
    assert checked > 2000


def test_c_node_builder_builds_the_reductions_python_builds():
    """every reduction over every kind of operand and axis through the
    backend's builders, with the C builder and without: same node class, same
    op dict (same key order), same operand -- or the same refusal; and the
    operators and elementwise builders that go to the C builder first give
    what ``OpTreeNode.build`` gives"""
    import neon_amd.backends  # noqa: F401
    from neon_amd.backends import backend as api
    from neon_amd.backends.backend import OpCollection, OpTreeNode
    assert api._c_red_node is not None
    be = PlanBackend(compile_kernels=False)
    full, col, row, one = be.empty((5, 7)), be.empty((5, 1)), be.empty((1, 7)), be.empty((1, 1))
    vec = ShapeTensor(be, (9,))
    vec.shape = (9,)
    cube = be.empty((5, 1))
    cube.shape = (2, 3, 4)
    node = full * col
    operands = [full, col, row, one, vec, cube, node, be.sum(full, axis=0), 2.5, 3, None, "text"]
    axes = [0, 1, None, -1, 2, True, 1.0, "0"]
    c_ew, c_red = api._c_ew_node, api._c_red_node

    def both(make):
        results = []
        for use_c in (True, False):
            api._c_ew_node, api._c_red_node = (c_ew, c_red) if use_c else (None, None)
            try:
                results.append(make())
            except Exception as e:                       # noqa: BLE001  (compared, not handled)
                results.append(type(e))
        api._c_ew_node, api._c_red_node = c_ew, c_red
        return results

    def same(got, want, what):
        if isinstance(want, tuple):
            assert type(got) is type(want) is OpTreeNode, what
            assert got[0] == want[0] and list(got[0]) == list(want[0]), (what, got[0], want[0])
            assert type(got[0]["shape"]) is tuple
            for g, w in zip(got[1:], want[1:]):
                if isinstance(w, tuple):
                    same(g, w, what)                     # (sum over everything: a reduction of a reduction)
                else:
                    assert g is w, what
        else:
            assert got is want, (what, got, want)

    built = 0
    for name in sorted(OpCollection.reduction_ops):
        for a in operands:
            for axis in axes:
                got, want = both(lambda: getattr(be, name)(a, axis=axis))
                same(got, want, (name, a, axis))
                built += isinstance(want, tuple)
                direct = c_red(name, a, axis)
                assert direct is None or (axis in (0, 1) and type(axis) is int and isinstance(want, tuple))
    assert built > 150
    assert c_red("add", full, 0) is None and c_red("bogus", full, 0) is None
    with pytest.raises(TypeError):
        c_red("sum", full)
    # operators and elementwise builders
    pairs = [(full, col), (col, full), (full, 2.5), (3, row), (node, one), (full, "text"), (None, full)]
    for a, b in pairs:
        for make in (lambda: a + b, lambda: a - b, lambda: a * b, lambda: a / b, lambda: a ** b, lambda: a == b,
                     lambda: a != b, lambda: a < b, lambda: a <= b, lambda: a > b, lambda: a >= b,
                     lambda: be.add(a, b), lambda: be.subtract(a, b), lambda: be.multiply(a, b), lambda: be.divide(a, b),
                     lambda: be.maximum(a, b), lambda: be.minimum(a, b), lambda: be.power(a, b), lambda: be.less(a, b),
                     lambda: be.exp(a), lambda: be.log(b), lambda: be.sqrt(a), lambda: be.sig(a), lambda: be.tanh(b),
                     lambda: be.square(a), lambda: be.absolute(a), lambda: be.negative(b), lambda: be.rint(a)):
            got, want = both(make)
            same(got, want, (a, b))
    assert be.true_divide.__func__ is be.divide.__func__ and be.fabs.__func__ is be.absolute.__func__
    assert type(full).__div__ is type(full).__truediv__


def test_the_extension_is_clean_under_address_and_undefined_behaviour_sanitizers(tmp_path):
    """fastpath.c built with -fsanitize=address,undefined and this file's CPU
    tests (key walks, node builder, records, error paths) run against that
    build in a child process with the sanitizer runtime preloaded: no report"""
    import os
    import shutil
    import subprocess
    import sys
    import sysconfig
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no gcc")
    runtime = subprocess.run([gcc, "-print-file-name=libasan.so"], capture_output=True, text=True).stdout.strip()
    if not os.path.isabs(runtime) or not os.path.exists(runtime):
        pytest.skip("no address sanitizer runtime")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    lib = str(tmp_path / "_fastpath.so")
    build = subprocess.run([gcc, "-O1", "-g", "-fPIC", "-shared", "-fsanitize=address,undefined",
                            "-fno-omit-frame-pointer", "-I" + sysconfig.get_paths()["include"],
                            os.path.join(root, "neon_amd", "csrc", "fastpath.c"), "-o", lib],
                           capture_output=True, text=True)
    assert build.returncode == 0, build.stderr[-2000:]
    env = dict(os.environ)
    env["NEON_HIP_FASTPATH_LIB"] = lib
    env["LD_PRELOAD"] = runtime + (":" + env["LD_PRELOAD"] if env.get("LD_PRELOAD") else "")
    env["ASAN_OPTIONS"] = "detect_leaks=0:verify_asan_link_order=0:abort_on_error=0"
    env["UBSAN_OPTIONS"] = "print_stacktrace=1"
    run = subprocess.run([sys.executable, "-m", "pytest", os.path.abspath(__file__), "-q", "-m", "not gpu",
                          "-p", "no:cacheprovider", "-k", "not sanitizers"], cwd=root, env=env,
                         capture_output=True, text=True, timeout=600)
    report = run.stdout[-3000:] + run.stderr[-3000:]
    assert run.returncode == 0, report
    assert "AddressSanitizer" not in report and "runtime error:" not in report, report
    assert " passed" in run.stdout
