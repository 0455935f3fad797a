"""
Tensor-library API of the op-tree path: ``Tensor``, ``Backend``, ``OpTreeNode``,
``OpCollection`` and ``Block``.

This is the plugin contract of the reference (neon/backends/backend.py and
neon/backends/abstract_backend.py): operators and ``be.<op>()`` builders do no
arithmetic, they grow an op-tree; ``tensor[:] = tree`` (or ``out=``) wraps the
tree in an ``assign`` node and hands it to ``backend.execute``.  A concrete
backend registers itself by defining ``backend_name`` on a ``Backend`` subclass
(abstract_backend.py:23-36) and is instantiated by ``Backend.allocate_backend``
(backend.py:465-472).

Everything in this module is host-side bookkeeping; nothing here touches data.
"""
import logging
from math import ceil

import numpy as np

logger = logging.getLogger(__name__)


class OpCollection(object):
    """Operation-name sets (reference backend.py:30-42)."""
    zero_operand_ops = {"rand", "onehot"}
    unary_ops = {"finite", "neg", "abs", "sgn", "sqrt", "sqr", "exp", "log",
                 "exp2", "log2", "sig", "sig2", "tanh", "tanh2", "transpose",
                 "safelog", "rint", "binarize"}
    binary_ops = {"assign", "add", "sub", "mul", "div", "eq", "ne", "lt", "le",
                  "gt", "ge", "pow", "minimum", "maximum", "dot", "shift"}
    reduction_ops = {"sum", "max", "min", "argmax", "argmin"}
    float_ops = zero_operand_ops | unary_ops | binary_ops
    ew_ops = float_ops - {"dot", "transpose"}


_EW_NOT_ASSIGN = frozenset(OpCollection.ew_ops) - {"assign"}


class Block(object):
    """Kinds of repeated computation announced through ``Backend.begin/end``
    (reference backend.py:2076-2088)."""
    epoch, minibatch, fprop, bprop, update = list(range(5))


_NO_OPERAND, _SCALAR_SHAPE = (0, 0), (1, 1)

# builder of elementwise nodes in C (neon_amd/csrc/fastpath.c), installed by
# ``use_c_node_builder``; None: nodes are built by ``OpTreeNode.build`` alone
_c_ew_node = None
_c_red_node = None


def use_c_node_builder(module):
    """Let ``OpTreeNode.build`` hand elementwise nodes without keyword
    arguments to ``module.ew_node``, and the reduction builders theirs
    (one axis, no ``out=``) to ``module.red_node`` (same nodes, a third of
    the time); ``None`` switches back to Python."""
    global _c_ew_node, _c_red_node
    if module is None:
        _c_ew_node = _c_red_node = None
        return
    module.configure_builder(OpTreeNode, Tensor, sorted(_EW_NOT_ASSIGN), sorted(OpCollection.reduction_ops))
    _c_ew_node = module.ew_node
    _c_red_node = getattr(module, "red_node", None)


def _shape_of_operand(x):
    """2-d shape an operand contributes to shape inference, None for a type
    that cannot be an operand"""
    if x is None:
        return _NO_OPERAND
    tx = type(x)
    if tx is float or tx is int:
        return _SCALAR_SHAPE
    if tx is OpTreeNode:
        shp = x[0]["shape"]
    elif isinstance(x, Tensor):
        shp = x.shape
    elif isinstance(x, (int, float)):
        return _SCALAR_SHAPE
    elif isinstance(x, OpTreeNode):
        shp = x[0]["shape"]
    else:
        return None
    if len(shp) == 1:
        return (shp[0], 1)
    return shp if type(shp) is tuple else tuple(shp)


class _LazyOperators(object):
    """Python operators that build op-tree nodes instead of computing.

    Shared by ``Tensor`` (reference backend.py:365-435) and ``OpTreeNode``
    (backend.py:2015-2073).  ``==`` is overloaded too, so hashing is by
    identity.
    """
    __slots__ = ()

    def __add__(self, other):
        return OpTreeNode.build("add", self, other)

    def __radd__(self, other):
        return OpTreeNode.build("add", other, self)

    def __sub__(self, other):
        return OpTreeNode.build("sub", self, other)

    def __rsub__(self, other):
        return OpTreeNode.build("sub", other, self)

    def __mul__(self, other):
        return OpTreeNode.build("mul", self, other)

    def __rmul__(self, other):
        return OpTreeNode.build("mul", other, self)

    def __truediv__(self, other):
        return OpTreeNode.build("div", self, other)

    def __rtruediv__(self, other):
        return OpTreeNode.build("div", other, self)

    __div__ = __truediv__
    __rdiv__ = __rtruediv__

    def __pow__(self, other):
        return OpTreeNode.build("pow", self, other)

    def __rpow__(self, other):
        return OpTreeNode.build("pow", other, self)

    def __eq__(self, other):
        return OpTreeNode.build("eq", self, other)

    def __ne__(self, other):
        return OpTreeNode.build("ne", self, other)

    def __lt__(self, other):
        return OpTreeNode.build("lt", self, other)

    def __le__(self, other):
        return OpTreeNode.build("le", self, other)

    def __gt__(self, other):
        return OpTreeNode.build("gt", self, other)

    def __ge__(self, other):
        return OpTreeNode.build("ge", self, other)

    def __abs__(self):
        return OpTreeNode.build("abs", self, None)

    def __neg__(self):
        return OpTreeNode.build("neg", self, None)


class Tensor(_LazyOperators):
    """Abstract n-d array handle (reference backend.py:45-435).

    Concrete backends subclass it and supply storage, views, ``get``/``set``.
    Dimensions are never collapsed below ``_min_dims`` (a scalar is 1x1).
    """
    _min_dims = 2

    def __init__(self, backend, shape=None, dtype=np.float32, name=None,
                     persist_values=True):
        self.backend = backend
        self.shape = shape
        self.dtype = dtype
        self.name = name
        self.persist_values = persist_values

    def __hash__(self):
        return id(self)

    def __str__(self):
        raise NotImplementedError()

    def __repr__(self):
        raise NotImplementedError()

    def __len__(self):
        raise NotImplementedError()

    def __setitem__(self, index, value):
        raise NotImplementedError()

    def __getitem__(self, index):
        raise NotImplementedError()

    def _assign(self, value):
        raise NotImplementedError()

    def set(self, ary):
        raise NotImplementedError()

    def get(self):
        raise NotImplementedError()

    def raw(self):
        raise NotImplementedError()

    def asnumpyarray(self):
        raise NotImplementedError()

    def take(self, indices, axis, out=None):
        raise NotImplementedError()

    def fill(self, value):
        raise NotImplementedError()

    def copy(self, a):
        raise NotImplementedError()

    def copy_from(self, a):
        raise NotImplementedError()

    def reshape(self, *shape):
        raise NotImplementedError()

    @property
    def T(self):
        raise NotImplementedError()

    def transpose(self, out=None):
        raise NotImplementedError()

    def hist(self, tag):
        raise NotImplementedError()

    def dimension_reorder(self, new_order):
        raise NotImplementedError()

    def backend_tensor(self):  # convenience used by a few callers
        return self

    def get_original_base(self):
        """Walk the chain of views back to the tensor that owns the memory."""
        t = self
        while t.base is not None:
            t = t.base
        return t


class OpTreeNode(_LazyOperators, tuple):
    """3-tuple ``(op_dict, left, right)`` (reference backend.py:1682-2073).

    ``op_dict`` carries ``"op"``, the inferred ``"shape"`` and any keyword
    arguments (``axis`` for reductions, ``idx``/``axis`` for onehot).  Operands
    are tensors, numbers, other nodes or ``None``.
    """
    __slots__ = ()

    def __new__(cls, *args):
        return tuple.__new__(cls, args)

    __hash__ = object.__hash__

    # -- printing -----------------------------------------------------------
    @staticmethod
    def _operand_str(x):
        if isinstance(x, Tensor):
            return x.name if x.name else "tensor-" + hex(id(x))
        return str(x)

    def __str__(self):
        return "(%s, %s, %s)" % (str(self[0]), self._operand_str(self[1]),
                                 self._operand_str(self[2]))

    __repr__ = __str__

    _infix = {"add": "+", "sub": "-", "mul": "*", "div": "/", "pow": "**"}

    @staticmethod
    def _pretty_print(node):
        if isinstance(node, Tensor):
            return OpTreeNode._operand_str(node)
        if isinstance(node, OpTreeNode):
            op = node[0]["op"]
            if node[2]:
                body = "%s %s %s" % (OpTreeNode._pretty_print(node[1]),
                                     OpTreeNode._infix.get(op, op),
                                     OpTreeNode._pretty_print(node[2]))
            else:
                body = "%s %s" % (op, OpTreeNode._pretty_print(node[1]))
            return "(" + body + ")"
        return "(" + str(node) + ")"

    def pp(self):
        """Infix rendering of the tree (reference backend.py:1981-1991)."""
        return OpTreeNode._pretty_print(self)

    # -- identity -----------------------------------------------------------
    @staticmethod
    def _strip(entry):
        if type(entry) is dict:
            if "axis" in entry:
                return (entry["op"], entry["axis"])
            return entry["op"]
        return entry

    def key(self):
        """Postfix tuple with op dicts reduced to names; tensors stay objects
        (hashed by id).  Reference backend.py:1717-1734."""
        return tuple(self._strip(e) for e in self.traverse(list()))

    def intrinsic_key_maps(self):
        """Key in which tensors are replaced by (first-occurrence index,
        shape), plus both index maps (reference backend.py:1736-1774)."""
        t2i, i2t, key = {}, {}, []
        for e in self.traverse(list()):
            if isinstance(e, Tensor):
                if e not in t2i:
                    t2i[e] = len(t2i)
                    i2t[t2i[e]] = e
                key.append((t2i[e], e.shape))
            else:
                key.append(self._strip(e))
        return tuple(key), t2i, i2t

    # -- construction ---------------------------------------------------------
    @staticmethod
    def build(op, a, b, out=None, **kwargs):
        """Make a node, inferring its shape; ``assign`` (or ``out=``) executes.

        Shape rules (reference backend.py:1776-1850): elementwise = per-axis
        maximum of the operand shapes (no compatibility check here; a mismatch
        surfaces in ``execute``); reduction with ``axis`` = operand shape with
        that axis set to 1; numbers are 1x1; 1-d shapes are padded to 2-d.
        """
        if _c_ew_node is not None and out is None and not kwargs:
            # (the common case -- an elementwise operator between tensors, nodes and numbers --
            # built in C; None means "not mine")
            node = _c_ew_node(op, a, b)
            if node is not None:
                return node
        sa, sb = _shape_of_operand(a), _shape_of_operand(b)
        if sa is None or sb is None:
            return NotImplemented
        if op in _EW_NOT_ASSIGN:
            # (this branch runs for every arithmetic operator a caller writes: kept short)
            if sa == sb:
                shape = sa
            else:
                shape = (sa[0] if sa[0] > sb[0] else sb[0], sa[1] if sa[1] > sb[1] else sb[1])
            if not kwargs and out is None:
                return OpTreeNode({"op": op, "shape": shape}, a, b)
        elif op in OpCollection.reduction_ops:
            if "axis" in kwargs:
                shape = list(sa)
                shape[kwargs["axis"]] = 1
                shape = tuple(shape)
            else:
                shape = (1, 1)
        elif op == "assign":
            shape = tuple(sa)
        elif op == "dot":
            assert len(sa) == len(sb) == 2 and sa[1] == sb[0]
            shape = (sa[0], sb[1])
        elif op == "transpose":
            assert b is None
            shape = tuple(reversed(sa))
        else:
            raise TypeError("%s is not a valid operation" % op)
        op_dict = {"op": op, "shape": shape}
        op_dict.update(kwargs)
        node = OpTreeNode(op_dict, a, b)
        if op == "assign":
            return node.execute()
        if out is not None:
            return OpTreeNode({"op": "assign"}, out, node).execute()
        return node

    def execute(self):
        """Run a tree whose root is ``assign`` on the backend of its target
        (reference backend.py:1852-1866)."""
        assert self[0]["op"] == "assign"
        backend = self[1].backend
        if isinstance(backend, Backend):
            return backend.execute(self)
        raise NotImplementedError()

    def traverse(self, stack):
        """Post-order walk appending operands then the op dict
        (reference backend.py:1868-1890)."""
        for child in (self[1], self[2]):
            if isinstance(child, OpTreeNode):
                child.traverse(stack)
            elif child is not None:
                stack.append(child)
        stack.append(self[0])
        return stack

    @property
    def shape(self):
        return self[0]["shape"]

    @property
    def T(self):
        return OpTreeNode.build("transpose", self, None)

    def transpose(self, out=None):
        if out:
            return OpTreeNode.build("assign", out, self.T)
        return self.T

    @staticmethod
    def optree_to_list(optree):
        if isinstance(optree, OpTreeNode):
            return [OpTreeNode.optree_to_list(x) for x in optree]
        return optree

    @staticmethod
    def list_to_optree(lst):
        if isinstance(lst, list):
            return OpTreeNode(*[OpTreeNode.list_to_optree(x) for x in lst])
        return lst

    def astensor(self):
        """Evaluate into a freshly allocated tensor of the tree's shape
        (reference backend.py:1993-2013)."""
        be = None
        for s in self.traverse(list()):
            if isinstance(s, Tensor):
                be = s.backend
                break
        if be is None:
            raise ValueError("No tensor object in op_tree")
        buf = be.empty(self.shape)
        buf[:] = self
        return buf

    def asnumpyarray(self):
        return self.astensor().get()


class _BackendRegistry(type):
    """Registers every named ``Backend`` subclass under ``backend_name``
    (reference abstract_backend.py:23-36), which is how ``-b hip`` becomes a
    valid choice."""

    def __init__(cls, name, bases, ns):
        if not hasattr(cls, "backends"):
            cls.backends = {}
        else:
            key = getattr(cls, "backend_name", name)
            if key != "Backend":
                cls.backends[key] = cls
        super(_BackendRegistry, cls).__init__(name, bases, ns)


class Backend(metaclass=_BackendRegistry):
    """Base class of concrete backends (reference backend.py:437-1680).

    Supplies the lazy op builders and derived ops; a subclass supplies
    allocation (``empty/array/zeros/ones/*_like``), the tensor class and
    ``execute``.  Layer-level entry points outside the op-tree path
    (``compound_dot``, convolution, pooling, lookup tables ...) are not part of
    this package and raise ``NotImplementedError``.
    """

    def __init__(self, rng_seed=None, default_dtype=np.float32,
                 compat_mode=None, deterministic=None):
        self.default_dtype = default_dtype
        self.rng_seed = rng_seed
        self.rng = self.gen_rng(rng_seed)
        self.bsz = None
        self._min_dims = 2
        if compat_mode is not None:
            if compat_mode != "caffe":
                raise ValueError("%s mode not supported currently" % compat_mode)
            self.compat_mode = "caffe"
        else:
            self.compat_mode = None
        if deterministic is not None:
            logger.warning("deterministic arg is deprecated in favor of "
                           "specifying random seed")
        self.deterministic = self.rng_seed is not None

    # -- factory --------------------------------------------------------------
    @staticmethod
    def backend_choices():
        return sorted(Backend.backends.keys())

    @staticmethod
    def allocate_backend(name, **kargs):
        try:
            cls = Backend.backends[name]
        except KeyError:
            names = ", ".join("'%s'" % n for n in Backend.backend_choices())
            raise ValueError("backend must be one of (%s)" % names)
        return cls(**kargs)

    def cleanup_backend(self):
        pass

    # -- host RNG (reference nervanacpu.py:583-627) ---------------------------
    def gen_rng(self, seed=None):
        self.rng = np.random.RandomState(seed)
        self.init_rng_state = self.rng.get_state()
        return self.rng

    def rng_reset(self):
        self.rng.set_state(self.init_rng_state)

    def rng_get_state(self):
        return self.rng.get_state()

    def rng_set_state(self, state):
        self.rng.set_state(state)

    # -- misc helpers -----------------------------------------------------------
    def set_caffe_compat(self):
        self.compat_mode = "caffe"

    def check_caffe_compat(self):
        return self.compat_mode == "caffe"

    def output_dim(self, X, S, padding, strides, pooling=False, dilation=1):
        """Output extent of a 1-d sliding window (reference backend.py:506-532)."""
        S = dilation * (S - 1) + 1
        if self.check_caffe_compat() and pooling:
            size = int(ceil(float(X - S + 2 * padding) / strides)) + 1
            if padding > 0 and (size - 1) * strides >= X + padding:
                size -= 1
        else:
            size = (X - S + 2 * padding) // strides + 1
        if pooling and padding >= S:
            raise ValueError("Padding dim %d incompatible with filter size %d"
                             % (padding, S))
        return size

    def iobuf(self, dim0, x=None, dtype=None, name=None, persist_values=True,
              shared=None, parallelism=None):
        """Allocate (or reuse) a zeroed ``(features, batch)`` buffer
        (reference backend.py:546-594)."""
        if x is not None:
            return x
        if isinstance(dim0, tuple):
            if len(dim0) == 2:
                bufshape = (dim0[0], dim0[1] * self.bsz)
            else:
                bufshape = (int(np.prod(dim0)), self.bsz)
        else:
            bufshape = (dim0, self.bsz)
        if shared is not None:
            out = shared if shared.shape == bufshape else shared.share(bufshape)
        else:
            out = self.empty(bufshape, dtype=dtype, name=name,
                             persist_values=persist_values)
        out[:] = 0
        return out

    def shared_iobuf_size(self, shape, parallelism):
        num_dev = 1 if parallelism in ("Data", "Model") else getattr(self, "num_dev", 1)
        return num_dev * int(np.prod(shape))

    def distribute_data(self, tensor, layer_parallelism):
        return None

    def revert_tensor(self, tensor):
        pass

    def execute(self, node):
        raise NotImplementedError()

    def begin(self, block, identifier):
        """Start of a block of repeated computation (reference
        backend.py:671-689): a hint, no effect on results."""
        pass

    def end(self, block, identifier):
        pass

    # -- allocation: supplied by the concrete backend -------------------------
    def empty(self, shape, dtype=None, name=None, persist_values=True,
              parallel=False, distributed=False):
        raise NotImplementedError()

    def array(self, ary, dtype=None, name=None, persist_values=True,
              parallel=False, distributed=False):
        raise NotImplementedError()

    def zeros(self, shape, dtype=None, name=None, persist_values=True,
              parallel=False, distributed=False):
        raise NotImplementedError()

    def ones(self, shape, dtype=None, name=None, persist_values=True,
             parallel=False, distributed=False):
        raise NotImplementedError()

    def empty_like(self, other_ary, name=None, persist_values=True):
        raise NotImplementedError()

    def zeros_like(self, other_ary, name=None, persist_values=True):
        raise NotImplementedError()

    # -- lazy builders (reference backend.py:711-1275) ------------------------
    def dot(self, a, b, out=None):
        return OpTreeNode.build("dot", a, b, out=out)

    def add(self, a, b, out=None):
        return OpTreeNode.build("add", a, b, out=out)

    def subtract(self, a, b, out=None):
        return OpTreeNode.build("sub", a, b, out=out)

    def multiply(self, a, b, out=None):
        return OpTreeNode.build("mul", a, b, out=out)

    def divide(self, a, b, out=None):
        return OpTreeNode.build("div", a, b, out=out)

    true_divide = divide

    def power(self, a, b, out=None):
        return OpTreeNode.build("pow", a, b, out=out)

    def reciprocal(self, a, out=None):
        return OpTreeNode.build("div", 1., a, out=out)

    def negative(self, a, out=None):
        return OpTreeNode.build("neg", a, None, out=out)

    def sgn(self, a, out=None):
        return OpTreeNode.build("sgn", a, None, out=out)

    def absolute(self, a, out=None):
        return OpTreeNode.build("abs", a, None, out=out)

    fabs = absolute

    def sqrt(self, a, out=None):
        return OpTreeNode.build("sqrt", a, None, out=out)

    def square(self, a, out=None):
        return OpTreeNode.build("sqr", a, None, out=out)

    def exp(self, a, out=None):
        return OpTreeNode.build("exp", a, None, out=out)

    def exp2(self, a, out=None):
        return OpTreeNode.build("exp2", a, None, out=out)

    def safelog(self, a, out=None):
        return OpTreeNode.build("safelog", a, None, out=out)

    def log(self, a, out=None):
        return OpTreeNode.build("log", a, None, out=out)

    def log2(self, a, out=None):
        return OpTreeNode.build("log2", a, None, out=out)

    def sig(self, a, out=None):
        return OpTreeNode.build("sig", a, None, out=out)

    def sig2(self, a, out=None):
        return OpTreeNode.build("sig2", a, None, out=out)

    def tanh(self, a, out=None):
        return OpTreeNode.build("tanh", a, None, out=out)

    def tanh2(self, a, out=None):
        return OpTreeNode.build("tanh2", a, None, out=out)

    def finite(self, a, out=None):
        return OpTreeNode.build("finite", a, None, out=out)

    def rint(self, a, out=None):
        return OpTreeNode.build("rint", a, None, out=out)

    def equal(self, a, b, out=None):
        return OpTreeNode.build("eq", a, b, out=out)

    def not_equal(self, a, b, out=None):
        return OpTreeNode.build("ne", a, b, out=out)

    def less(self, a, b, out=None):
        return OpTreeNode.build("lt", a, b, out=out)

    def less_equal(self, a, b, out=None):
        return OpTreeNode.build("le", a, b, out=out)

    def greater(self, a, b, out=None):
        return OpTreeNode.build("gt", a, b, out=out)

    def greater_equal(self, a, b, out=None):
        return OpTreeNode.build("ge", a, b, out=out)

    def maximum(self, a, b, out=None):
        return OpTreeNode.build("maximum", a, b, out=out)

    def minimum(self, a, b, out=None):
        return OpTreeNode.build("minimum", a, b, out=out)

    def clip(self, a, a_min, a_max, out=None):
        return self.minimum(self.maximum(a, a_min), a_max, out=out)

    # -- reductions and derived statistics (reference backend.py:1313-1502) ---
    def _reduce(self, op, a, axis, out):
        if out is None and _c_red_node is not None:
            node = _c_red_node(op, a, axis)          # (None: not an axis-0/1 reduction of a tensor or node)
            if node is not None:
                return node
        if axis is None:
            # whole-tensor reduction = axis 0 then axis 1
            inner = OpTreeNode.build(op, a, None, axis=0)
            return OpTreeNode.build(op, inner, None, axis=1, out=out)
        return OpTreeNode.build(op, a, None, axis=axis, out=out)

    def sum(self, a, axis=None, out=None, keepdims=True):
        return self._reduce("sum", a, axis, out)

    def max(self, a, axis=None, out=None, keepdims=True):
        return self._reduce("max", a, axis, out)

    def min(self, a, axis=None, out=None, keepdims=True):
        return self._reduce("min", a, axis, out)

    def argmax(self, a, axis=1, out=None, keepdims=True):
        if out is None and _c_red_node is not None:
            node = _c_red_node("argmax", a, axis)
            if node is not None:
                return node
        return OpTreeNode.build("argmax", a, None, axis=axis, out=out)

    def argmin(self, a, axis=1, out=None, keepdims=True):
        if out is None and _c_red_node is not None:
            node = _c_red_node("argmin", a, axis)
            if node is not None:
                return node
        return OpTreeNode.build("argmin", a, None, axis=axis, out=out)

    def mean(self, a, axis=None, partial=None, out=None, keepdims=True):
        shape = a.shape
        if axis is None:
            return self.multiply(self.sum(a), 1.0 / (shape[0] * shape[1]), out=out)
        return self.multiply(self.sum(a, axis=axis), 1.0 / shape[axis], out=out)

    def var(self, a, axis=None, partial=None, out=None, keepdims=True,
            binary=False):
        """Biased two-pass variance: mean of squared deviations from the mean
        (reference backend.py:1451-1480)."""
        if binary:
            raise NotImplementedError("shift-based variance is outside the op-tree path")
        if axis is None:
            return self.mean(self.square(a - self.mean(a)), out=out)
        return self.mean(self.square(a - self.mean(a, axis=axis)), axis=axis, out=out)

    def std(self, a, axis=None, partial=None, out=None, keepdims=True):
        return self.sqrt(self.var(a, axis=axis, partial=partial, out=out))

    def take(self, a, indices, axis, out=None):
        return a.take(indices, axis, out)

    def onehot(self, indices, axis, out=None):
        """One-hot expansion of an int32/uint32 index vector along ``axis``
        (reference backend.py:1519-1537)."""
        if axis not in (0, 1):
            raise ValueError("bad axis for onehot")
        assert indices.dtype in (np.dtype(np.int32), np.dtype(np.uint32)), \
            "onehot indices should be int32 or uint32, got " + str(indices.dtype)
        return OpTreeNode.build("onehot", None, None, idx=indices, axis=axis, out=out)

    # -- layer helpers that are plain op-trees (reference nervanacpu.py:1907-1959;
    #    nervanagpu.py:3179-3231) ------------------------------------------------
    def fprop_softmax(self, x, axis):
        return (self.reciprocal(self.sum(self.exp(x - self.max(x, axis=axis)), axis=axis)) *
                self.exp(x - self.max(x, axis=axis)))

    def fprop_relu(self, layer, x, slope):
        return self.maximum(x, 0) + slope * self.minimum(0, x)

    def bprop_relu(self, layer, x, error, deltas, slope):
        return self.greater(x, 0) + slope * self.less(x, 0)

    def fprop_transform(self, ngLayer, transform, inputs, outputs, relu=False):
        outputs[:] = transform(inputs)

    def bprop_transform(self, ngLayer, transform, outputs, error, deltas, relu):
        deltas[:] = transform.bprop(outputs) * error

    def fprop_skipnode(self, x, y, beta):
        y[:] = y * beta + x

    def bprop_skipnode(self, error, deltas, alpha, beta):
        deltas[:] = deltas * beta + alpha * error

    # -- small aliases and hooks of the reference's base class (backend.py:627-650,
    #    808-823, 907-921, 1539-1557) ---------------------------------------------
    def true_divide(self, a, b, out=None):
        return OpTreeNode.build("div", a, b, out=out)

    def fabs(self, a, out=None):
        return OpTreeNode.build("abs", a, None, out=out)

    def update_fc_bias(self, err, out):
        """bias gradient of a fully connected layer: row sums of the error"""
        self.sum(err, axis=1, out=out)

    def add_fc_bias(self, inputs, bias):
        """add one bias value per row, in place"""
        self.add(inputs, bias, out=inputs)

    def compound_rnn_unroll_fprop(self, W_recur, h_prev_s, h_ff_s, h_s, bias, nout, num_steps,
                                  num_used_steps, activation, reverse=False):
        """The time loop of a plain recurrent layer (reference
        backend.py:1559-1601): h[t] = activation(W_recur h[t-1] + h_ff[t] +
        bias) over lists of per-step views; ``h_ff_s`` may be ``h_s`` itself
        when the input projection was written into the outputs."""
        used = num_steps if num_used_steps is None else min(num_used_steps, num_steps)
        order = range(used - 1, -1, -1) if reverse else range(used)
        for t in order:
            h, h_prev, h_ff = h_s[t], h_prev_s[t], h_ff_s[t]
            if h_ff is h:
                self.compound_dot(W_recur, h_prev, h, beta=1.0)
                h[:] = activation(h + bias)
            else:
                self.compound_dot(W_recur, h_prev, h)
                h[:] = activation(h + h_ff + bias)

    def compound_rnn_unroll_bprop(self, W_recur, delta_prev_s, delta_s, h_s, nout, num_steps,
                                  num_used_steps, activation, reverse=True):
        """The time loop of a plain recurrent layer's backward pass (reference
        backend.py:1603-1638); ``W_recur`` arrives already transposed."""
        used = num_steps if num_used_steps is None else min(num_used_steps, num_steps)
        n = min(used, len(delta_s), len(delta_prev_s))
        order = range(n - 1, -1, -1) if reverse else range(n)
        for t in order:
            delta_s[t][:] = activation.bprop(h_s[t]) * delta_s[t]
            self.compound_dot(W_recur, delta_s[t], delta_prev_s[t], beta=1.0)

    def is_mkl(self):
        return False

    def convert_data(self, tensor, layer_mkl):
        return None

    def clean_data(self, tensor, layer_mkl):
        return None

    def allocate_new_deltas(self, delta, in_shape, parallelism):
        return delta

    def allocate_new_outputs(self, layer, share_output):
        layer.allocate(shared_outputs=share_output)

    # -- layer bookkeeping the reference's containers call on any backend: no
    #    backend-side state here, the merges just drive their branches with the
    #    right accumulate flags (reference nervanagpu.py:3179-3231) ---------------
    def relu_layer(self):
        return None

    def batchnorm_layer(self, in_shape):
        return None

    def mergesum_layer(self, layer_num):
        return None

    def mergebroadcast_layer(self, layer_num):
        return None

    def fprop_mergesum(self, ngLayer, inputs, inference, layers, outputs, out_shape):
        """every branch adds into the shared output; the first one overwrites it"""
        for k, layer in enumerate(layers):
            layer.fprop(inputs, inference, beta=0 if k == 0 else 1)

    def bprop_mergesum(self, ngLayer, alpha, beta, layers, error, deltas):
        """branches in reverse; the one that runs first applies the caller's
        ``beta``, the others accumulate"""
        last = len(layers) - 1
        for k in range(last, -1, -1):
            layers[k].bprop(error, alpha=alpha, beta=beta if k == last else 1)

    def fprop_mergebroadcast(self, ngLayer, inputs, inference, outputs, layers, out_shape):
        for layer in layers:
            layer.fprop(inputs, inference)

    def bprop_mergebroadcast(self, ngLayer, layers, error_views, error, delta, out_shape, alpha, beta,
                             alphas, betas):
        betas[-1] = beta
        for k in range(len(layers) - 1, -1, -1):
            layers[k].bprop(error_views[k], alpha=alphas[k] * alpha, beta=betas[k])

    # -- outside the op-tree path ----------------------------------------------
    def compound_dot(self, A, B, C, alpha=1.0, beta=0.0, relu=False, bsum=None):
        raise NotImplementedError("dense contraction is outside the op-tree path")

    def batched_dot(self, A, B, C, alpha=1.0, beta=0.0, relu=False):
        raise NotImplementedError("dense contraction is outside the op-tree path")

    def make_binary_mask(self, out, keepthresh=0.5):
        raise NotImplementedError()

    # -- binary-network helpers: compositions of ordinary ops (reference
    #    nervanacpu.py:1823-1863) ------------------------------------------------
    def _uniform_like(self, ary):
        """uniform [0, 1) values of ``ary``'s shape, as a tensor or an op-tree"""
        raise NotImplementedError()

    def binarize(self, ary, out, stochastic=True):
        """``out`` = +1 / -1: the sign of ``ary`` (zero counts as positive), or,
        with ``stochastic``, +1 with probability clip((ary + 1) / 2, 0, 1)"""
        if stochastic:
            out[:] = (ary + 1) / 2.0
            self.clip(out, 0, 1, out)
            self.less_equal(self._uniform_like(ary), out, out)
        else:
            self.greater_equal(ary, 0, out)
        out[:] = 2 * out - 1
        return out

    def shift(self, ary, shift_ary, value=True, out=None):
        """``ary`` times a power of two: 2 ** shift_ary, or (``value``) the power
        of two nearest to ``shift_ary`` in the log domain, with its sign"""
        if value:
            exponent = self.rint(self.safelog(self.absolute(shift_ary)) / self.log(2))
            ap2 = self.multiply(self.sgn(shift_ary), self.exp2(exponent))
        else:
            ap2 = self.exp2(shift_ary)
        if out is None:
            out = self.empty_like(ary) if hasattr(ary, "shape") else self.empty((1, 1))
        out[:] = self.multiply(ary, ap2)
        return out


# -- the operators and builders above, entered through the C node builder ----------------------
# Every arithmetic operator and elementwise builder is a Python call into ``OpTreeNode.build``,
# which (for the common case) is a call into ``ew_node``: the wrappers below go to ``ew_node``
# first and to the definition above whenever it says "not mine" (or is not installed), which
# saves a Python frame and a keyword dictionary per node -- a quarter of a microsecond each.
def _operator_via_c(op, slow, swap):
    if swap:
        def method(self, other):
            f = _c_ew_node
            if f is not None:
                node = f(op, other, self)
                if node is not None:
                    return node
            return slow(self, other)
    else:
        def method(self, other):
            f = _c_ew_node
            if f is not None:
                node = f(op, self, other)
                if node is not None:
                    return node
            return slow(self, other)
    method.__name__, method.__qualname__, method.__doc__ = slow.__name__, slow.__qualname__, slow.__doc__
    return method


def _builder_via_c(op, slow, operands):
    if operands == 1:
        def method(self, a, out=None):
            if out is None:
                f = _c_ew_node
                if f is not None:
                    node = f(op, a, None)
                    if node is not None:
                        return node
            return slow(self, a, out)
    else:
        def method(self, a, b, out=None):
            if out is None:
                f = _c_ew_node
                if f is not None:
                    node = f(op, a, b)
                    if node is not None:
                        return node
            return slow(self, a, b, out)
    method.__name__, method.__qualname__, method.__doc__ = slow.__name__, slow.__qualname__, slow.__doc__
    return method


for _name, _op, _swap in (("__add__", "add", False), ("__radd__", "add", True), ("__sub__", "sub", False),
                          ("__rsub__", "sub", True), ("__mul__", "mul", False), ("__rmul__", "mul", True),
                          ("__truediv__", "div", False), ("__rtruediv__", "div", True), ("__pow__", "pow", False),
                          ("__rpow__", "pow", True), ("__eq__", "eq", False), ("__ne__", "ne", False),
                          ("__lt__", "lt", False), ("__le__", "le", False), ("__gt__", "gt", False),
                          ("__ge__", "ge", False)):
    setattr(_LazyOperators, _name, _operator_via_c(_op, getattr(_LazyOperators, _name), _swap))
_LazyOperators.__div__, _LazyOperators.__rdiv__ = _LazyOperators.__truediv__, _LazyOperators.__rtruediv__
for _name, _op, _n in (("add", "add", 2), ("subtract", "sub", 2), ("multiply", "mul", 2), ("divide", "div", 2),
                       ("power", "pow", 2), ("negative", "neg", 1), ("sgn", "sgn", 1), ("absolute", "abs", 1),
                       ("sqrt", "sqrt", 1), ("square", "sqr", 1), ("exp", "exp", 1), ("exp2", "exp2", 1),
                       ("safelog", "safelog", 1), ("log", "log", 1), ("log2", "log2", 1), ("sig", "sig", 1),
                       ("sig2", "sig2", 1), ("tanh", "tanh", 1), ("tanh2", "tanh2", 1), ("finite", "finite", 1),
                       ("rint", "rint", 1), ("equal", "eq", 2), ("not_equal", "ne", 2), ("less", "lt", 2),
                       ("less_equal", "le", 2), ("greater", "gt", 2), ("greater_equal", "ge", 2),
                       ("maximum", "maximum", 2), ("minimum", "minimum", 2)):
    setattr(Backend, _name, _builder_via_c(_op, getattr(Backend, _name), _n))
Backend.true_divide, Backend.fabs = Backend.divide, Backend.absolute
del _name, _op, _swap, _n
