"""The plug-in boundary: ``nervanahip.bind`` derives the backend from a HOST
package's ``Backend`` / ``OpTreeNode`` / ``Tensor`` classes (stand-ins in
tests/foreign_api.py, shaped like neon's abstract_backend.py:23-36 and
backend.py:465-472, 1852-1890), registers it there as ``'hip'`` and executes
trees made of that package's node objects."""
import numpy as np
import pytest

import foreign_api as F
from neon_amd.backends import backend as own
from neon_amd.backends import nervanahip
from neon_amd.backends.hip import planner, prebuild
from neon_amd.backends.hip import runtime as hiprt
from neon_amd.backends.hip.optree_ir import Program
from utils import assert_close


def _bound():
    return nervanahip.bind(F.Backend, F.Node, F.Tensor, F.Block)


def test_bind_registers_hip_in_the_host_registry():
    NervanaHIP, HIPTensor = _bound()
    assert F.Backend.backends["hip"] is NervanaHIP
    assert issubclass(NervanaHIP, F.Backend) and issubclass(NervanaHIP, nervanahip.NervanaHIPBase)
    assert issubclass(HIPTensor, F.Tensor) and issubclass(HIPTensor, nervanahip.HIPTensorBase)
    assert not issubclass(NervanaHIP, own.Backend) and not issubclass(HIPTensor, own.Tensor)
    assert NervanaHIP.tensor_cls is HIPTensor
    assert NervanaHIP.__mro__[1] is nervanahip.NervanaHIPBase and NervanaHIP.__mro__[2] is F.Backend
    assert type(NervanaHIP) is F.Registry
    # every method the host declares abstract is supplied
    assert NervanaHIP.__abstractmethods__ == frozenset()
    # one class pair per host package; this package's own binding is another pair
    assert _bound() == (NervanaHIP, HIPTensor)
    own_pair = nervanahip.bind()
    assert own_pair[0] is own.Backend.backends["hip"] and own_pair[0] is not NervanaHIP
    assert nervanahip.NervanaHIP is own_pair[0] and nervanahip.HIPTensor is own_pair[1]
    assert "hip" not in [k for k, v in F.Backend.backends.items() if v is own_pair[0]]
    assert NervanaHIP._api.OpTreeNode is F.Node and NervanaHIP._api.Block is F.Block


def test_bind_finds_block_next_to_the_backend_class():
    class Other(F.Backend):
        __module__ = F.__name__          # as if defined in the host package
    first = _bound()[0]
    try:
        pair = nervanahip.bind(Other, F.Node, F.Tensor)
        assert pair[0]._api.Block is F.Block
        assert Other.backends["hip"] is pair[0]     # the registry is shared by the host's class tree
    finally:
        F.Backend.backends["hip"] = first


def test_bind_needs_the_three_classes():
    with pytest.raises(TypeError):
        nervanahip.bind(F.Backend)


@pytest.mark.skipif(hiprt.device_count() > 0, reason="needs a machine without a device")
def test_host_side_instantiation_reaches_the_device_probe():
    """abstract-method checks pass (they run before __init__); what stops the
    constructor on a machine without a GPU is the device probe"""
    _bound()
    with pytest.raises(hiprt.HipError):
        F.Backend.allocate_backend("hip", rng_seed=0)


class _ShapeTensor(F.Tensor):
    """host-package tensor with geometry only (device-free planning)"""

    def __init__(self, backend, shape, dtype=np.float32, ptr=1 << 32):
        super(_ShapeTensor, self).__init__(backend, shape, dtype)
        self.shape, self.dtype = tuple(shape), np.dtype(dtype)
        self.strides = (shape[1], 1)
        self.size = shape[0] * shape[1]
        self.is_contiguous, self.take_array, self.base, self.ptr = True, None, None, ptr


def test_foreign_nodes_plan_to_the_same_kernel_as_native_ones():
    """the DAG builder reads only node[0]['op'|'axis'|'idx'], node[1], node[2]
    and traverse(): a tree of host-package nodes gives the same program key
    and the same generated kernel as the tree built with this package's API"""
    fb = F.Backend.__new__(_bound()[0])          # builders only; no device behind it
    x = _ShapeTensor(fb, (1000, 128), ptr=1 << 32)
    out = _ShapeTensor(fb, (1000, 128), ptr=2 << 32)
    tree = fb.exp(x - fb.max(x, axis=0)) / fb.sum(fb.exp(x - fb.max(x, axis=0)), axis=0)
    assert type(tree) is F.Node
    prog = Program()
    prog.add_statement(F.Node(dict(op="assign"), out, tree))
    prog.finalize()

    pb = prebuild.PlanBackend(compile_kernels=False)
    nx = prebuild.ShapeTensor(pb, (1000, 128), ptr=1 << 32)
    nout = prebuild.ShapeTensor(pb, (1000, 128), ptr=2 << 32)
    nprog = Program()
    nprog.add_statement(own.OpTreeNode({"op": "assign"}, nout, pb.exp(nx - pb.max(nx, axis=0)) /
                                       pb.sum(pb.exp(nx - pb.max(nx, axis=0)), axis=0)))
    nprog.finalize()
    assert prog.key() == nprog.key()
    assert planner.choose(prog).spec.name == planner.choose(nprog).spec.name


# ---- GPU ----------------------------------------------------------------------------------
@pytest.fixture(scope="module")
def fhip():
    _bound()
    be = F.Backend.allocate_backend("hip", rng_seed=0)
    be.bsz = 1
    yield be
    be.synchronize()


@pytest.mark.gpu
def test_trees_of_foreign_nodes_execute_and_match_the_oracle(fhip, cpu):
    rs = np.random.RandomState(3)
    x = (rs.standard_normal((500, 96)) * 3).astype(np.float32)
    idx = rs.randint(0, 500, size=(1, 96)).astype(np.int32)
    X, I = fhip.array(x), fhip.array(idx, dtype=np.int32)
    assert isinstance(X, F.Tensor) and not isinstance(X, own.Tensor)
    sm = fhip.empty((500, 96))
    tree = fhip.exp(X - fhip.max(X, axis=0)) / fhip.sum(fhip.exp(X - fhip.max(X, axis=0)), axis=0)
    assert type(tree) is F.Node
    sm[:] = tree
    am = fhip.empty((1, 96), dtype=np.int32)
    fhip.argmax(X, axis=0, out=am)
    ce = fhip.empty((1, 96))
    ce[:] = -fhip.sum(fhip.onehot(I, axis=0) * fhip.log(tree), axis=0)
    rowsum = fhip.empty((500, 1))
    rowsum[:] = fhip.sum(X * X, axis=1) + 1.0

    # the same trees on the oracle, built with this package's API
    CX, CI = cpu.array(x), cpu.array(idx, dtype=np.int32)
    csm = cpu.empty((500, 96))
    ctree = cpu.exp(CX - cpu.max(CX, axis=0)) / cpu.sum(cpu.exp(CX - cpu.max(CX, axis=0)), axis=0)
    csm[:] = ctree
    cam = cpu.empty((1, 96), dtype=np.int32)
    cpu.argmax(CX, axis=0, out=cam)
    ct = cpu.empty((500, 96))
    ct[:] = cpu.onehot(CI, axis=0)
    cce = cpu.empty((1, 96))
    cce[:] = -cpu.sum(ct * cpu.log(ctree), axis=0)
    assert_close(sm.get(), csm.get(), rtol=1e-5, atol=1e-9, what="softmax")
    assert np.array_equal(am.get(), cam.get())
    assert_close(ce.get(), cce.get(), rtol=1e-5, atol=1e-6, what="cross-entropy")
    assert_close(rowsum.get(), (x.astype(np.float64) ** 2).sum(axis=1, keepdims=True) + 1.0, rtol=1e-5, what="rows")


@pytest.mark.gpu
def test_foreign_update_block_fuses(fhip):
    rs = np.random.RandomState(4)
    p0, g0 = rs.standard_normal((64, 200)).astype(np.float32), rs.standard_normal((64, 200)).astype(np.float32)
    p, g, v = fhip.array(p0), fhip.array(g0), fhip.zeros((64, 200))
    before = fhip.plan_stats["launches"]
    fhip.begin(F.Block.update, 0)
    v[:] = 0.9 * v - 0.1 * g
    p[:] = p + v
    fhip.end(F.Block.update, 0)
    assert fhip.plan_stats["launches"] - before == 1
    assert_close(p.get(), p0 - np.float32(0.1) * g0, rtol=1e-6, atol=1e-7)
    for layer_kernel in ("conv_layer", "fprop_pool"):
        with pytest.raises(NotImplementedError):
            getattr(fhip, layer_kernel)()


def test_every_name_of_the_reference_surface_is_supplied():
    """tests/golden/api_surface.json holds the names read off the reference
    (abstract_backend.py:40-1428: 68 abstract methods; backend.py:45-435: the
    Tensor class; backend.py:437-1680: what its Backend class itself defines).
    A host laid out the same way -- an abstract class declaring all 68, a
    Backend below it defining what the reference's Backend defines -- is bound,
    and nothing may be left abstract; the tensor class answers every Tensor
    method, and overrides every one that the reference's base class only
    raises from."""
    import abc
    import json
    import os
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "api_surface.json")) as f:
        surface = json.load(f)
    assert len(surface["abstract_methods"]) == 68

    def stub():
        def method(self, *args, **kwargs):
            raise NotImplementedError()
        return method                     # (abc.abstractmethod marks the function object itself)

    declared = dict((name, abc.abstractmethod(stub())) for name in surface["abstract_methods"])
    AbstractHost = F.Registry("AbstractHost", (F.Backend,), dict(declared, __module__=F.__name__))
    in_backend_py = dict((name, stub()) for name in surface["backend_methods"] if name in declared)
    HostBackend = F.Registry("HostBackend", (AbstractHost,), dict(in_backend_py, __module__=F.__name__))
    left_to_the_concrete_backend = set(surface["abstract_methods"]) - set(in_backend_py)
    assert {"empty", "array", "zeros", "ones", "empty_like", "zeros_like", "compound_dot", "gen_rng",
            "rng_reset", "fprop_conv", "make_binary_mask"} <= left_to_the_concrete_backend
    first = F.Backend.backends.get("hip")
    try:
        NervanaHIP, HIPTensor = nervanahip.bind(HostBackend, F.Node, F.Tensor, F.Block)
        assert NervanaHIP.__abstractmethods__ == frozenset(), sorted(NervanaHIP.__abstractmethods__)
        for name in left_to_the_concrete_backend:
            assert name in vars(nervanahip.NervanaHIPBase), name
    finally:
        if first is not None:
            F.Backend.backends["hip"] = first
    missing = [name for name in surface["tensor_methods"] if not hasattr(nervanahip.HIPTensorBase, name)
               and not hasattr(own.Tensor, name)]
    assert missing == [], missing
    own_tensor = nervanahip.bind()[1]
    for name in surface["tensor_abstract"]:
        if name == "_assign" or not name.startswith("_") or name in ("__getitem__", "__setitem__", "__len__",
                                                                      "__str__", "__repr__"):
            assert name in vars(nervanahip.HIPTensorBase), "%s is only a stub in the base class" % name
    assert callable(getattr(own_tensor, "dimension_reorder", None)) or "dimension_reorder" not in surface["tensor_methods"]
