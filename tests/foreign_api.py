"""A stand-in for the package that hosts the backend: its OWN ``Backend`` base
with a registering ABC metaclass and abstract layer methods, its own ``Tensor``
and its own tuple-based ``OpTreeNode`` -- the plug-in shape of neon's
neon/backends/abstract_backend.py:23-36 and backend.py:45-435, 465-472,
1682-1890, written independently of ``neon_amd.backends.backend`` and sharing
no class with it.  The binding tests build op-trees from THESE classes and
hand them to the hip backend bound to them."""
import abc

import numpy as np

_EW = {"add", "sub", "mul", "div", "neg", "exp", "log", "sqrt", "sqr", "maximum", "eq", "safelog", "onehot"}
_RED = {"sum", "max", "argmax"}


def _shape(x):
    if x is None:
        return (0, 0)
    if isinstance(x, (int, float)):
        return (1, 1)
    s = x.shape if isinstance(x, Tensor) else x[0]["shape"]
    return tuple(s) if len(s) > 1 else (s[0], 1)


class Node(tuple):
    """(op_dict, left, right)"""

    def __new__(cls, *parts):
        return tuple.__new__(cls, parts)

    __hash__ = object.__hash__

    @staticmethod
    def build(op, a, b, out=None, **kw):
        sa, sb = _shape(a), _shape(b)
        if op in _EW:
            shape = (max(sa[0], sb[0]), max(sa[1], sb[1]))
        elif op in _RED:
            shape = tuple(1 if i == kw["axis"] else d for i, d in enumerate(sa))
        elif op == "assign":
            shape = sa
        else:
            raise TypeError(op)
        d = dict(op=op, shape=shape)
        d.update(kw)
        node = Node(d, a, b)
        if op == "assign":
            return node.execute()
        if out is not None:
            return Node(dict(op="assign"), out, node).execute()
        return node

    def execute(self):
        be = self[1].backend
        if not isinstance(be, Backend):
            raise NotImplementedError()
        return be.execute(self)

    def traverse(self, stack):
        for side in (self[1], self[2]):
            if isinstance(side, Node):
                side.traverse(stack)
            elif side is not None:
                stack.append(side)
        stack.append(self[0])
        return stack

    @property
    def shape(self):
        return self[0]["shape"]

    def __add__(self, o): return Node.build("add", self, o)
    def __radd__(self, o): return Node.build("add", o, self)
    def __sub__(self, o): return Node.build("sub", self, o)
    def __rsub__(self, o): return Node.build("sub", o, self)
    def __mul__(self, o): return Node.build("mul", self, o)
    def __rmul__(self, o): return Node.build("mul", o, self)
    def __truediv__(self, o): return Node.build("div", self, o)
    def __rtruediv__(self, o): return Node.build("div", o, self)
    def __neg__(self): return Node.build("neg", self, None)


class Tensor(object):
    def __init__(self, backend, shape=None, dtype=np.float32, name=None, persist_values=True):
        self.backend, self.shape, self.dtype, self.name = backend, shape, dtype, name
        self.persist_values = persist_values

    __add__, __radd__, __sub__, __rsub__ = Node.__add__, Node.__radd__, Node.__sub__, Node.__rsub__
    __mul__, __rmul__, __truediv__, __rtruediv__ = Node.__mul__, Node.__rmul__, Node.__truediv__, Node.__rtruediv__
    __neg__ = Node.__neg__

    def __setitem__(self, index, value):
        raise NotImplementedError()

    def get(self):
        raise NotImplementedError()


class Block(object):
    epoch, minibatch, fprop, bprop, update = range(5)


class Registry(abc.ABCMeta):
    def __init__(cls, name, bases, ns):
        if not hasattr(cls, "backends"):
            cls.backends = {}
        else:
            name = getattr(cls, "backend_name", name)
            if name != "Backend":
                cls.backends[name] = cls
        super(Registry, cls).__init__(name, bases, ns)


class AbstractBackend(metaclass=Registry):
    @abc.abstractmethod
    def cleanup_backend(self): ...
    @abc.abstractmethod
    def gen_rng(self, seed=None): ...
    @abc.abstractmethod
    def rng_get_state(self): ...
    @abc.abstractmethod
    def rng_reset(self): ...
    @abc.abstractmethod
    def rng_set_state(self, state): ...
    @abc.abstractmethod
    def empty(self, shape, dtype=None, name=None, persist_values=True, parallel=False, distributed=False): ...
    @abc.abstractmethod
    def array(self, ary, dtype=None, name=None, persist_values=True, parallel=False, distributed=False): ...
    @abc.abstractmethod
    def zeros(self, shape, dtype=None, name=None, persist_values=True, parallel=False, distributed=False): ...
    @abc.abstractmethod
    def ones(self, shape, dtype=None, name=None, persist_values=True, parallel=False, distributed=False): ...
    @abc.abstractmethod
    def empty_like(self, other_ary, name=None, persist_values=True): ...
    @abc.abstractmethod
    def zeros_like(self, other_ary, name=None, persist_values=True): ...
    @abc.abstractmethod
    def compound_dot(self, A, B, C, alpha=1.0, beta=0.0, relu=False, bsum=None): ...
    @abc.abstractmethod
    def batched_dot(self, A, B, C, alpha=1.0, beta=0.0, relu=False): ...
    @abc.abstractmethod
    def make_binary_mask(self, out, keepthresh=0.5): ...
    @abc.abstractmethod
    def conv_layer(self, *a, **k): ...
    @abc.abstractmethod
    def fprop_conv(self, *a, **k): ...
    @abc.abstractmethod
    def bprop_conv(self, *a, **k): ...
    @abc.abstractmethod
    def update_conv(self, *a, **k): ...
    @abc.abstractmethod
    def deconv_layer(self, *a, **k): ...
    @abc.abstractmethod
    def pool_layer(self, *a, **k): ...
    @abc.abstractmethod
    def fprop_pool(self, *a, **k): ...
    @abc.abstractmethod
    def bprop_pool(self, *a, **k): ...
    @abc.abstractmethod
    def compound_bprop_lut(self, *a, **k): ...


class Backend(AbstractBackend):
    def __init__(self, rng_seed=None, default_dtype=np.float32, compat_mode=None, deterministic=None):
        self.default_dtype, self.rng_seed, self.bsz = default_dtype, rng_seed, None
        self.rng = self.gen_rng(rng_seed)
        self.compat_mode = compat_mode

    @staticmethod
    def allocate_backend(name, **kw):
        return Backend.backends[name](**kw)

    def begin(self, block, identifier):
        pass

    def end(self, block, identifier):
        pass

    def execute(self, node):
        raise NotImplementedError()

    # op builders, the host package's own
    def exp(self, a, out=None): return Node.build("exp", a, None, out=out)
    def log(self, a, out=None): return Node.build("log", a, None, out=out)
    def safelog(self, a, out=None): return Node.build("safelog", a, None, out=out)
    def sqrt(self, a, out=None): return Node.build("sqrt", a, None, out=out)
    def square(self, a, out=None): return Node.build("sqr", a, None, out=out)
    def maximum(self, a, b, out=None): return Node.build("maximum", a, b, out=out)
    def sum(self, a, axis, out=None): return Node.build("sum", a, None, axis=axis, out=out)
    def max(self, a, axis, out=None): return Node.build("max", a, None, axis=axis, out=out)
    def argmax(self, a, axis, out=None): return Node.build("argmax", a, None, axis=axis, out=out)
    def onehot(self, idx, axis, out=None): return Node.build("onehot", None, None, idx=idx, axis=axis, out=out)
