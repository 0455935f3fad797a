"""
Op-tree -> typed DAG.

Takes the postfix stacks of one or more ``assign`` trees (a *program*; several
statements are fused when the backend was asked to, one otherwise) and builds a
DAG in which

  * every distinct tensor (same object, or same memory + geometry) and every
    distinct constant gets one kernel-argument *slot*;
  * identical sub-expressions are one node (structural hashing over the whole
    tree -- the reference only merges duplicates at reduction boundaries,
    float_ew.py:147-190, so softmax's repeated ``exp(x - max)`` was evaluated
    twice per element there);
  * sub-trees made of numbers only (Adam's ``lr*sqrt(1-b2**t)/(1-b1**t)``) are
    folded on the host in double precision -- what the CPU backend's numpy
    calls do with Python floats -- and become a single constant slot;
  * each node knows along which axes it varies (``vr``, ``vc``) and its
    reduction *level*: how many nested reductions must have completed before
    it can be evaluated.

The same walk yields the cache key: two programs with equal keys generate
byte-identical kernels and bind arguments in the same order.

Host-side checks raise before anything is generated, with the exception types
of the reference launcher (float_ew.py:682-690, 724-726, 821-825, 900-906):
reduction axis outside {0,1} or two different axes -> ValueError; operand
shapes that do not broadcast -> TypeError; unknown op or operand -> TypeError.
"""
import math
import os

import numpy as np

from neon_amd.backends.hip.bf16 import bfloat16


UNARY = {"neg", "abs", "sgn", "sqrt", "sqr", "exp", "log", "exp2", "log2", "sig",
         "sig2", "tanh", "tanh2", "safelog", "rint", "finite",
         # internal: exp of an argument known not to be positive (what staged evaluation makes
         # of exp(x - max(x)) once the maximum sits in a temporary)
         "exp_nonpos"}
BINARY = {"add", "sub", "mul", "div", "eq", "ne", "lt", "le", "gt", "ge", "pow",
          "minimum", "maximum"}
REDUCE = {"sum", "max", "min", "argmax", "argmin"}

# storage dtype -> short code used in keys and kernel names
DTYPE_CODE = {np.dtype(np.float32): "f4", np.dtype(np.float16): "f2",
              np.dtype(np.int32): "i4", np.dtype(np.uint32): "u4",
              np.dtype(np.int16): "i2", np.dtype(np.uint16): "u2",
              np.dtype(np.int8): "i1", np.dtype(np.uint8): "u1",
              bfloat16: "b2"}


def _fold_unary(op, x):
    """Host evaluation of a unary op on a number, numpy semantics in double."""
    x = float(x)
    with np.errstate(all="ignore"):
        if op == "neg":
            return -x
        if op == "abs":
            return abs(x)
        if op == "sgn":
            return float(np.sign(x))
        if op == "sqrt":
            return float(np.sqrt(x))
        if op == "sqr":
            return x * x
        if op == "exp" or op == "exp_nonpos":
            return float(np.exp(x))
        if op == "log":
            return float(np.log(x))
        if op == "safelog":
            return float(np.log(np.maximum(x, np.exp(-50.))))
        if op == "exp2":
            return float(np.exp2(x))
        if op == "log2":
            return float(np.log2(x))
        if op == "sig":
            return float(1. / (1. + np.exp(-x)))
        if op == "sig2":
            return float(1. / (1. + np.exp2(-x)))
        if op == "tanh":
            return float(np.tanh(x))
        if op == "tanh2":
            return float((np.exp2(2. * x) - 1.) / (np.exp2(2. * x) + 1.))
        if op == "rint":
            return float(np.rint(x))
        if op == "finite":
            return float(np.isfinite(x))
    raise TypeError("unknown unary op %s" % op)


def _fold_binary(op, a, b):
    a, b = float(a), float(b)
    with np.errstate(all="ignore"):
        if op == "add":
            return a + b
        if op == "sub":
            return a - b
        if op == "mul":
            return a * b
        if op == "div":
            return float(np.float64(a) / np.float64(b))
        if op == "pow":
            return float(np.power(np.float64(a), np.float64(b)))
        if op == "minimum":
            return float(np.minimum(a, b))
        if op == "maximum":
            return float(np.maximum(a, b))
        if op == "eq":
            return float(a == b)
        if op == "ne":
            return float(a != b)
        if op == "lt":
            return float(a < b)
        if op == "le":
            return float(a <= b)
        if op == "gt":
            return float(a > b)
        if op == "ge":
            return float(a >= b)
    raise TypeError("unknown binary op %s" % op)


class Num(object):
    """A number on the build stack: its value and how it derives from the raw
    numbers of the trees (``('r', i)`` = i-th number in postfix order,
    ``('1', op, e)`` / ``('2', op, a, b)`` = folded on the host), so that a
    recorded launch can be re-bound to new constants without rebuilding."""
    __slots__ = ("value", "expr")

    def __init__(self, value, expr):
        self.value = value
        self.expr = expr


def eval_const(expr, raw):
    """value of a constant-slot expression for the raw numbers ``raw``"""
    tag = expr[0]
    if tag == "r":
        return raw[expr[1]]
    if tag == "1":
        return _fold_unary(expr[1], eval_const(expr[2], raw))
    return _fold_binary(expr[1], eval_const(expr[2], raw), eval_const(expr[3], raw))


def is_tensor(x):
    """a tensor operand, of whatever package's ``Tensor`` class the backend was
    bound to: anything that carries a device address and element strides"""
    return hasattr(x, "ptr") and hasattr(x, "strides")


ONLINE_LSE = os.environ.get("NEON_HIP_ONLINE_LSE", "1") != "0"
ONEHOT_GATHER = os.environ.get("NEON_HIP_ONEHOT_GATHER", "1") != "0"


class MixedAxes(ValueError):
    """Reductions along both axes in one tree: needs more than one kernel."""


def stochastic_bits(tensor):
    """Mantissa bits a store into ``tensor`` rounds to stochastically, 0 for
    the ordinary round-to-nearest store (reference float_ew.py:832-844: True
    means 10, at most 15 for float32 and 10 for float16 targets); ``"int"``
    for signed integer targets, which round to whole numbers."""
    rounding = getattr(tensor, "rounding", 0)
    if not rounding:
        return 0
    dtype = np.dtype(tensor.dtype)
    if dtype == np.float32:
        cap = 15
    elif dtype == np.float16:
        cap = 10
    elif dtype == bfloat16:
        cap = 7
    elif dtype.kind == "i":
        # signed integer targets round to whole numbers, whatever number of bits is asked for
        # (reference cuda_templates.py:236-286: fp32_to_int32_rand / int16 / int8)
        return "int"
    else:
        raise NotImplementedError("stochastic rounding into %s tensors" % dtype)
    return 10 if rounding is True else max(1, min(int(rounding), cap))


class Node(object):
    """DAG node.  kind: 'T' tensor leaf, 'C' constant slot, 'E' elementwise op,
    'R' reduction, 'H' one-hot of an index tensor, 'G' an expression evaluated
    at the hot row of a one-hot (``args = (expression, one-hot)``; what
    ``sum(onehot * expression, axis=0)`` is rewritten to)."""
    __slots__ = ("kind", "op", "args", "slot", "axis", "vr", "vc", "level",
                 "nid", "is_index", "shape", "lse_max", "lse_sum")

    def __init__(self, kind, op=None, args=(), slot=None, axis=None):
        self.kind = kind
        self.op = op
        self.args = tuple(args)
        self.slot = slot
        self.axis = axis
        self.vr = self.vc = False
        self.level = 0
        self.nid = -1
        self.is_index = False
        self.shape = (1, 1)
        self.lse_max = None     # on sum(exp(x - max(x))): the max node it shares a sweep with
        self.lse_sum = None     # on that max node: the sum

    def __repr__(self):
        return "N%d<%s %s %s>" % (self.nid, self.kind, self.op or "", self.slot if self.slot is not None else "")


class TensorSlot(object):
    """One kernel pointer argument: a distinct (memory, geometry, dtype)."""
    __slots__ = ("index", "tensor", "dtype", "shape", "strides", "ptr", "written",
                 "read", "geom", "take_axis", "take_slot", "take_extent")

    def __init__(self, index, tensor, shape, strides):
        self.take_axis = None      # gather / scatter view: indexed axis ...
        self.take_slot = None      # ... the slot of its int32 index vector ...
        self.take_extent = None    # ... and the extent of the indexed axis in the underlying tensor
        self.index = index
        self.tensor = tensor
        self.dtype = np.dtype(tensor.dtype)
        self.shape = shape
        self.strides = strides
        self.ptr = tensor.ptr
        self.written = False
        self.read = False
        self.geom = (tensor.ptr, shape, strides, self.dtype)


class Statement(object):
    __slots__ = ("out", "root")

    def __init__(self, out, root):
        self.out = out      # TensorSlot
        self.root = root    # Node


def view_2d(tensor):
    """(shape, element strides) of a tensor as the 2-d object the kernels see.
    Tensors with more than two dims are accepted only when contiguous and are
    flattened to (dim0, rest)."""
    shape, strides = tuple(tensor.shape), tuple(tensor.strides)
    if len(shape) == 2:
        return shape, strides
    if len(shape) == 1:
        return (shape[0], 1), (strides[0], 1)
    if not tensor.is_contiguous:
        raise ValueError("op-trees on non-contiguous tensors with more than 2 "
                         "dimensions are not supported")
    rest = 1
    for d in shape[1:]:
        rest *= d
    return (shape[0], rest), (rest, 1)


class Program(object):
    """DAG of one fused group of assign statements."""

    def __init__(self):
        self.tensors = []          # TensorSlot list, in first-use order
        self.consts = []           # python floats, in first-use order
        self.statements = []
        self.nodes = []            # topological order
        self._tensor_by_geom = {}
        self._tensor_by_id = {}
        self._cse = {}
        self._const_slot = {}
        self._current = {}         # tensor slot index -> node holding its newest value
        self.key_parts = []
        self.index_slots = set()   # slots used only as index vectors of gather views
        self.rand_count = 0        # number of rand nodes (each draws its own stream)
        # ids of tensor objects whose reads mean "the value before this group
        # ran" even after a statement of the group has assigned that memory
        self.originals = frozenset()
        self.rng_args = (0, 0)     # (seed, first counter) bound by the backend before a launch
        self.raw_count = 0         # numbers seen so far, in postfix order
        self.const_exprs = []      # per constant slot: expressions that produced its value
        self.axis = None           # the one reduction axis, if any
        self.domain = None
        self.nlevels = 0
        # rewrites applied by finalize (module switches, read when the program is made)
        self.online_lse = ONLINE_LSE
        self.onehot_gather = ONEHOT_GATHER

    # -- slots -----------------------------------------------------------------
    def tensor_slot(self, t):
        slot = self._tensor_by_id.get(id(t))
        if slot is not None:
            return slot
        take = getattr(t, "take_array", None)
        take_slot = take_axis = None
        if take:
            # a view through an index vector (the reference's in1/in2/out1/out2
            # argument kinds, cuda_templates.py:448-483): position i along the
            # indexed axis addresses element idx[i] of the base
            idx, take_axis = take
            if len(t.shape) != 2 or take_axis not in (0, 1):
                raise NotImplementedError("fancy-indexed views with more than 2 dimensions")
            if idx.dtype != np.dtype(np.int32) or not idx.is_contiguous:
                raise TypeError("index vector of a fancy-indexed view must be contiguous int32")
            take_slot = self.tensor_slot(idx)
            self.index_slots.add(take_slot.index)
        shape, strides = view_2d(t)
        take_extent = getattr(t, "take_extent", None) if take else None
        geom = (t.ptr, shape, strides, np.dtype(t.dtype),
                take_axis, take_slot.index if take_slot else None, take_extent)
        slot = self._tensor_by_geom.get(geom)
        if slot is None:
            if np.dtype(t.dtype) not in DTYPE_CODE:
                raise TypeError("unsupported tensor dtype %s" % t.dtype)
            slot = TensorSlot(len(self.tensors), t, shape, strides)
            slot.take_axis = take_axis
            slot.take_slot = take_slot.index if take_slot else None
            slot.take_extent = take_extent
            slot.geom = geom
            self.tensors.append(slot)
            self._tensor_by_geom[geom] = slot
        self._tensor_by_id[id(t)] = slot
        return slot

    def const_node(self, num):
        value = float(num.value)
        # every occurrence of an equal number shares a slot; the *value* is a
        # run-time argument, so the key records only the slot pattern
        slot = self._const_slot.get(value)
        if slot is None:
            slot = len(self.consts)
            self.consts.append(value)
            self.const_exprs.append([])
            self._const_slot[value] = slot
        self.const_exprs[slot].append(num.expr)
        self.key_parts.append(("C", slot))
        return self._intern(("C", slot), lambda: Node("C", slot=slot))

    def _intern(self, key, make):
        n = self._cse.get(key)
        if n is None:
            n = make()
            n.nid = len(self.nodes)
            self.nodes.append(n)
            self._cse[key] = n
        return n

    # -- building ------------------------------------------------------------------
    def add_statement(self, optree):
        """Append ``assign(out, expr)`` given as an OpTreeNode."""
        assert optree[0]["op"] == "assign"
        out_t, value = optree[1], optree[2]
        if not is_tensor(out_t):
            raise TypeError("assignment target must be a tensor")
        out_slot = self.tensor_slot(out_t)
        stack = []
        postfix = []
        if isinstance(value, (int, float)):
            postfix = [value]
        elif is_tensor(value):
            postfix = [value]
        else:
            value.traverse(postfix)
        for p in postfix:
            if isinstance(p, dict):
                self._apply(p, stack)
            elif is_tensor(p):
                stack.append(self._read_tensor(p))
            elif isinstance(p, (int, float)):
                stack.append(Num(float(p), ("r", self.raw_count)))      # folded lazily
                self.raw_count += 1
            else:
                raise TypeError("args must be instance of Tensor, int, float, or dict (for operators)")
        if len(stack) != 1:
            raise TypeError("malformed op-tree")
        root = stack[0]
        if not isinstance(root, Node):
            root = self.const_node(root)
        bits = stochastic_bits(out_t)
        if bits:
            # the store rounds stochastically: one more random stream, applied
            # to the value before it is converted to the storage type
            ordinal = self.rand_count
            self.rand_count += 1
            self.key_parts.append(("sround", bits))
            value_node = root
            root = self._intern(("sround", ordinal),
                                lambda: Node("E", op="sround:%s" % bits, args=(value_node,), slot=ordinal,
                                             axis=out_slot.index))     # axis field: the slot stored to
        out_slot.written = True
        st = Statement(out_slot, root)
        self.statements.append(st)
        self.key_parts.append(("=", out_slot.index))
        self._current[out_slot.index] = root
        return st

    def _read_tensor(self, t):
        slot = self.tensor_slot(t)
        original = id(t) in self.originals
        self.key_parts.append(("T0" if original else "T", slot.index))
        cur = None if original else self._current.get(slot.index)
        if cur is not None:
            # value written by an earlier statement of this program: forward it,
            # rounded the way the store rounds it
            if slot.dtype == np.dtype(np.float32):
                return cur
            return self._intern(("Q", cur.nid, DTYPE_CODE[slot.dtype]),
                                lambda: Node("E", op="quant:" + DTYPE_CODE[slot.dtype], args=(cur,)))
        slot.read = True
        return self._intern(("T", slot.index), lambda: Node("T", slot=slot.index))

    def _as_node(self, x):
        return x if isinstance(x, Node) else self.const_node(x)

    def _apply(self, d, stack):
        op = d["op"]
        if op in UNARY:
            x = stack.pop()
            if not isinstance(x, Node):
                self.key_parts.append(("fold1", op))
                stack.append(Num(_fold_unary(op, x.value), ("1", op, x.expr)))
                return
            self.key_parts.append(op)
            stack.append(self._intern(("E", op, x.nid), lambda: Node("E", op=op, args=(x,))))
        elif op in BINARY:
            b = stack.pop()
            a = stack.pop()
            if not isinstance(a, Node) and not isinstance(b, Node):
                self.key_parts.append(("fold2", op))
                stack.append(Num(_fold_binary(op, a.value, b.value), ("2", op, a.expr, b.expr)))
                return
            # a number becomes a node (and a key part) only here, after the
            # operator's own part: say on which side it stands, or ``x - 1``
            # and ``1 - x`` would share a key and therefore a kernel
            self.key_parts.append((op, isinstance(a, Node), isinstance(b, Node)))
            a, b = self._as_node(a), self._as_node(b)
            stack.append(self._intern(("E", op, a.nid, b.nid), lambda: Node("E", op=op, args=(a, b))))
        elif op in REDUCE:
            x = stack.pop()
            axis = d.get("axis", None)
            if axis not in (0, 1):
                raise ValueError("Only reduction along an axis currently supported")
            self.key_parts.append((op, axis))
            x = self._as_node(x)
            n = self._intern(("R", op, axis, x.nid), lambda: Node("R", op=op, args=(x,), axis=axis))
            n.is_index = op in ("argmax", "argmin")
            stack.append(n)
        elif op == "onehot":
            idx = d["idx"]
            slot = self.tensor_slot(idx)
            slot.read = True
            axis = d["axis"]
            self.key_parts.append(("onehot", slot.index, axis))
            stack.append(self._intern(("H", slot.index, axis),
                                      lambda: Node("H", op="onehot", slot=slot.index, axis=axis)))
        elif op == "rand":
            # uniform [0, 1): every occurrence is its own stream (never merged)
            ordinal = self.rand_count
            self.rand_count += 1
            self.key_parts.append("rand")
            stack.append(self._intern(("rand", ordinal), lambda: Node("E", op="rand", slot=ordinal)))
        elif op in ("dot", "transpose", "binarize", "shift", "assign"):
            raise NotImplementedError("op '%s' cannot be part of a fused op-tree kernel" % op)
        else:
            raise TypeError("%s is not a valid operation" % op)

    # -- analysis --------------------------------------------------------------------
    def finalize(self):
        """Infer the iteration domain, per-node variance and reduction levels;
        verify broadcast compatibility."""
        # a tensor assigned more than once in the group is stored once, with its
        # final value; readers in between were given the value in registers
        last = {}
        for st in self.statements:
            last[st.out.index] = st
        self.statements = [st for st in self.statements if last[st.out.index] is st]
        index_only = set(n.slot for n in self.nodes if n.kind == "H") | set(self.index_slots)
        index_only -= set(n.slot for n in self.nodes if n.kind == "T")
        index_only -= set(st.out.index for st in self.statements)
        shaped = [t for t in self.tensors if t.index not in index_only]
        R = C = 1
        for t in shaped:
            R, C = max(R, t.shape[0]), max(C, t.shape[1])
        axes = set(n.axis for n in self.nodes if n.kind == "R")
        if len(axes) > 1:
            raise MixedAxes("Reduction along only one axis is supported per kernel")
        self.axis = axes.pop() if axes else None
        self.domain = (R, C)
        for t in shaped:
            if t.shape[0] not in (1, R) or t.shape[1] not in (1, C):
                raise TypeError("Input shape:%s not compatible with %s" % (t.shape, (R, C)))
        self._analyse()
        self.lse_pairs = 0
        self.gathers = 0
        if self.axis is not None and self.online_lse:
            self._pair_max_with_sum_of_exp()
        if self.axis == 0 and self.onehot_gather:
            self._gather_at_hot_rows()
        if self.lse_pairs or self.gathers:
            self._analyse()
        for st in self.statements:
            rs, os_ = st.root.shape, st.out.shape
            if (rs[0] not in (1, os_[0])) or (rs[1] not in (1, os_[1])):
                raise TypeError("Input shape:%s not compatible with %s" % (rs, os_))
        return self

    def _analyse(self):
        """per node: along which axes it varies, its reduction level, its shape"""
        R, C = self.domain
        for n in self.nodes:
            if n.kind == "T":
                shp = self.tensors[n.slot].shape
                n.vr, n.vc, n.level = shp[0] > 1, shp[1] > 1, 0
            elif n.kind == "C":
                n.vr = n.vc = False
                n.level = 0
            elif n.kind == "H":
                # one-hot of a vector of indices: full variance wherever the
                # index vector and the hot axis have extent
                n.vr, n.vc, n.level = R > 1, C > 1, 0
            elif n.kind == "E" and not n.args:       # rand: varies wherever the domain has extent
                n.vr, n.vc, n.level = R > 1, C > 1, 0
            elif n.kind == "E" and n.op.startswith("sround:"):
                # every stored element draws its own random number
                if self.tensors[n.axis].shape != (R, C):
                    raise NotImplementedError("stochastic rounding of an output narrower than the kernel's domain")
                n.vr, n.vc, n.level = R > 1, C > 1, n.args[0].level
            elif n.kind == "E":
                n.vr = any(a.vr for a in n.args)
                n.vc = any(a.vc for a in n.args)
                n.level = max(a.level for a in n.args)
            elif n.kind == "G":
                # one value per column, computable once the reductions inside the expression are
                n.vr, n.vc, n.level = False, C > 1, n.args[0].level
            elif n.kind == "R":
                a = n.args[0]
                varies = a.vr if n.axis == 0 else a.vc
                if not varies:
                    # extent 1 along the reduced axis: the reduction is the
                    # identity (index reductions give 0), as numpy has it
                    n.kind = "E"
                    n.op = "zero_index" if n.is_index else "ident"
                    n.is_index = False
                    n.vr, n.vc, n.level = a.vr, a.vc, a.level
                else:
                    n.vr = a.vr and n.axis != 0
                    n.vc = a.vc and n.axis != 1
                    n.level = a.level + 1
                    if n.lse_max is not None:
                        n.level = n.lse_max.level        # accumulated in the sweep that finds the maximum
            n.shape = (R if n.vr else 1, C if n.vc else 1)
        if not any(n.kind == "R" for n in self.nodes):
            self.axis = None
        self.nlevels = max([n.level for n in self.nodes] + [0])

    def _pair_max_with_sum_of_exp(self):
        """``sum(exp(x - max(x, 0)), 0)``: the sum joins the sweep that finds the
        maximum, as a running (max, sum) pair that is rescaled whenever the
        maximum grows -- softmax and cross-entropy trees need one pass (and, when
        the rows are spread over several workgroups, one exchange) less.  The
        sum's terms are added in another order and rescaled by exp(m - M)
        factors: equal to the two-sweep result within a few units in the last
        place, not bit for bit (``NEON_HIP_ONLINE_LSE=0`` keeps two sweeps)."""
        for sm in self.nodes:
            if sm.kind != "R" or sm.op != "sum":
                continue
            e = sm.args[0]
            if e.kind != "E" or e.op != "exp":
                continue
            d = e.args[0]
            if d.kind != "E" or d.op != "sub":
                continue
            x, mx = d.args
            if (mx.kind == "R" and mx.op == "max" and mx.axis == sm.axis and mx.args[0] is x
                    and mx.lse_sum is None):
                mx.lse_sum, sm.lse_max = sm, mx
                self.lse_pairs += 1

    def unpair_lse(self):
        """back to one sweep for the maximum and one for the sum"""
        for n in self.nodes:
            n.lse_max = n.lse_sum = None
        self.lse_pairs = 0
        self._analyse()

    def pair_lse(self):
        """(again) one sweep for both, where the tree has the pattern"""
        if not self.lse_pairs and self.online_lse:
            self._pair_max_with_sum_of_exp()
            if self.lse_pairs:
                self._analyse()

    def _gather_at_hot_rows(self):
        """``sum(onehot(idx, 0) * expr, 0)`` adds one term of ``expr`` per column
        and zeros: it becomes ``expr`` evaluated at row ``idx[c]`` only (0 when
        the index is out of range) -- for a cross-entropy tree the second pass
        over the matrix disappears.  Exact as long as ``expr`` is finite in the
        other rows (0 * inf would be NaN in the sum).  Applied when the value is
        only used for one-value-per-column results (``NEON_HIP_ONEHOT_GATHER=0``
        keeps the sum)."""
        roots = [st.root for st in self.statements]
        live = used_nodes(roots)
        users = {}
        for n in live:
            for a in n.args:
                users.setdefault(a.nid, []).append(n)
        line_roots = set(st.root.nid for st in self.statements if st.out.shape[0] == 1)
        other_roots = set(st.root.nid for st in self.statements) - line_roots

        def only_feeds_column_values(n):
            todo, seen = [n], set()
            while todo:
                m = todo.pop()
                if m.nid in seen:
                    continue
                seen.add(m.nid)
                if m.nid in other_roots:
                    return False
                for u in users.get(m.nid, ()):
                    if u.kind != "E" or u.vr or u.op.startswith("sround:"):
                        return False
                    todo.append(u)
            return True

        def plain(expr):
            for m in used_nodes([expr]):
                if m.kind == "G" or (m.kind == "H" and m.axis != 0):
                    return False
                if m.kind == "E" and (not m.args or m.op.startswith("sround:")):
                    return False
                if m.kind == "T" and self.tensors[m.slot].take_axis is not None:
                    return False
            return True

        for n in live:
            if n.kind != "R" or n.op != "sum" or n.axis != 0:
                continue
            p = n.args[0]
            if p.kind != "E" or p.op != "mul":
                continue
            a, b = p.args
            hot, expr = (a, b) if a.kind == "H" else (b, a)
            if hot.kind != "H" or hot.axis != 0 or expr.kind == "H":
                continue
            if not plain(expr) or not only_feeds_column_values(n):
                continue
            n.kind, n.op, n.args = "G", "gather0", (expr, hot)
            self.gathers += 1

    def key(self):
        """Hashable identity of the program's structure and operand geometry."""
        geo = tuple((DTYPE_CODE[t.dtype], t.shape, t.strides, t.ptr % 16 == 0, t.written,
                     t.take_axis, t.take_slot, t.take_extent) for t in self.tensors)
        return (tuple(self.key_parts), geo, self._alias_signature(), self.online_lse, self.onehot_gather)

    def _alias_signature(self):
        """Which slots overlap in memory (matters for what may be declared
        non-aliasing in the generated kernel)."""
        spans = []
        for t in self.tensors:
            isz = t.dtype.itemsize
            extent = 1 + sum((s - 1) * abs(st) for s, st in zip(t.shape, t.strides) if s > 0)
            spans.append((t.ptr, t.ptr + extent * isz))
        sig = []
        if any(t.take_axis is not None for t in self.tensors):
            sig.append(("gather",))      # extent of a gather view is data dependent: assume overlap
        for i in range(len(spans)):
            for j in range(i + 1, len(spans)):
                if spans[i][0] < spans[j][1] and spans[j][0] < spans[i][1]:
                    sig.append((i, j))
        return tuple(sig)

    def overlapping_slots(self):
        return self._alias_signature()

    def output_hazards(self):
        """Written slots whose memory overlaps that of ANOTHER slot of the
        program (one that is read or written through a different view:
        different start, shape or strides -- the same view is the same slot).
        A kernel gives no order between the lanes that write such an output
        and the lanes that read or write the overlapping elements, whereas the
        reference's CPU backend finishes the right-hand side before it stores
        (nervanacpu.py:476-477: ``left[:] = right`` on a finished array).
        Gather / scatter views count by the whole axis they index."""
        spans = []
        for t in self.tensors:
            isz = t.dtype.itemsize
            lo = hi = 0
            for axis, (n, st) in enumerate(zip(t.shape, t.strides)):
                if t.take_axis == axis and t.take_extent:
                    n = t.take_extent
                if n > 1:
                    if st >= 0:
                        hi += (n - 1) * st
                    else:
                        lo += (n - 1) * st
            spans.append((t.ptr + lo * isz, t.ptr + (hi + 1) * isz))
        def line_of_its_operand(w, o):
            """``w`` holds one value per line of the reduction axis and sits INSIDE the
            full-shape operand ``o``, each value in the very line it is computed from
            (``x[0:1, :] = max(x, axis=0)``, ``x[:, 0:1] = sum(x, axis=1)``): every family
            stores a line's results after the last read of that line, and no lane of
            another line ever touches it"""
            ax = self.axis
            if ax is None or w.take_axis is not None or o.take_axis is not None or o.written:
                return False
            if w.shape[ax] != 1 or w.shape[1 - ax] != o.shape[1 - ax] or o.shape != tuple(self.domain):
                return False
            if w.strides[1 - ax] != o.strides[1 - ax] or w.dtype != o.dtype:
                return False
            step = o.strides[ax] * o.dtype.itemsize
            off = w.ptr - o.ptr
            return step > 0 and off % step == 0 and 0 <= off // step < o.shape[ax]

        hazards = []
        for w in self.tensors:
            if not w.written:
                continue
            a = spans[w.index]
            for o in self.tensors:
                if o is w or not (o.read or o.written or o.index in self.index_slots):
                    continue
                b = spans[o.index]
                if a[0] < b[1] and b[0] < a[1] and not line_of_its_operand(w, o):
                    hazards.append(w)
                    break
        return hazards


def build_program(optrees):
    prog = Program()
    for tree in optrees:
        prog.add_statement(tree)
    return prog.finalize()


def used_nodes(roots):
    """Nodes reachable from ``roots`` in topological (id) order."""
    seen = {}
    todo = list(roots)
    while todo:
        n = todo.pop()
        if n.nid in seen:
            continue
        seen[n.nid] = n
        todo.extend(n.args)
    return [seen[k] for k in sorted(seen)]
