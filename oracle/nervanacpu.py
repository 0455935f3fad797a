"""
CPU ORACLE -- test infrastructure, not product code.

A numpy restatement of the reference's CPU backend for the op-tree path
(neon/backends/nervanacpu.py): ``CPUTensor`` wraps a ``numpy.ndarray`` and
``NervanaCPU.execute`` is a postfix-stack interpreter over a table of numpy
calls.  Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline``
leg of ``bench.py`` may import this module; the ``hip`` backend never does.

Importing it registers backend ``'cpu'`` with the factory, as the reference's
``neon/backends/__init__.py:30`` does.

What pins each function (nothing here was produced by running the reference):
  * every entry of ``NUMPY_CALLS`` is the numpy call named in
    nervanacpu.py:480-522, checked in tests/test_oracle.py against pure-Python
    scalar loops on tiny inputs and against closed forms;
  * ``execute`` is checked against direct numpy evaluation of the same
    function (the reference's own test idiom, tests/utils.py:85-103) and the
    known answers the reference's tests hold: softmax of [0,1,-2]
    (tests/test_activations.py:144-147), cross-entropy incl. the exp(-50)
    clamp (tests/test_costs.py:105-122), misclassification 1/3
    (tests/test_costs.py:200-208), the Adam step restated in numpy
    (tests/test_optimizer.py:280-299), reduction shapes
    (tests/test_backend_autodiff_extra.py:250-261);
  * view semantics are checked against numpy basic indexing
    (tests/test_backend_tensor.py:252-315).

Deliberate differences from the reference text, both forced by numpy >= 2:
  * results of scalar-only ops (e.g. ``np.sqrt(python_float)``) are turned back
    into Python floats.  numpy 1.13, which the reference pins, used value-based
    casting so such a scalar never widened an fp32 array; under NEP 50 an
    ``np.float64`` scalar would.  Keeping them weak reproduces the pinned
    behaviour.
  * the top-level one-hot scatter indexes with a tuple of index arrays; the
    reference's list-of-lists index (nervanacpu.py:681) meant the same thing
    under numpy 1.13.

Extension (flagged, pinned by equivalence with the top-level form in
tests/test_oracle.py): ``onehot`` may appear inside a tree, evaluated as the
dense 0/1 matrix the reference's accelerator backend forms on the fly
(cuda_templates.py:484-494, 573).  ``finite`` is evaluated as ``np.isfinite``
(accelerator semantics, cuda_templates.py:531-538); the reference CPU backend
has no entry for either.
"""
import time

import numpy as np

from neon_amd.backends.backend import Backend, OpCollection, OpTreeNode, Tensor

_none_slice = slice(None, None, None)

_SUPPORTED = (np.float16, np.float32, np.float64, np.uint8, np.int8,
              np.uint16, np.int16, np.uint32, np.int32)


class CPUTensor(Tensor):
    """numpy-backed tensor (reference nervanacpu.py:39-445)."""

    def __init__(self, backend, shape=None, dtype=np.float32, ary=None,
                 name=None, persist_values=True, base=None):
        super(CPUTensor, self).__init__(backend, shape, dtype, name, persist_values)
        assert dtype in _SUPPORTED or np.dtype(dtype).type in _SUPPORTED
        dtype = np.dtype(dtype)
        if type(ary) is not np.ndarray:
            data = np.array(ary, dtype)
        elif ary.dtype != dtype:
            data = ary.astype(dtype)
        else:
            data = ary
        while data.ndim < self._min_dims:
            data = data.reshape(data.shape + (1,))
        self._tensor = data
        if shape is not None and len(shape) < self._min_dims:
            shp = tuple(shape) + (1,) * (self._min_dims - len(shape))
        else:
            shp = data.shape
        dims = []
        for d in shp:
            if int(d) != d:
                raise TypeError("shape dims must be integer values [%s]" % str(d))
            dims.append(int(d))
        self.shape = tuple(dims)
        self.size = int(np.prod(dims)) if dims else 1
        self.base = base
        self.dtype = dtype
        self.is_contiguous = data.flags.c_contiguous

    def __str__(self):
        root = self._tensor.base if self._tensor.base is not None else self._tensor
        return ("CPUTensor(base 0x%x) name:%s shape:%s dtype:%s strides:%s"
                " is_c_contiguous:%s" % (id(root), self.name, self.shape, self.dtype,
                                         self._tensor.strides,
                                         self._tensor.flags.c_contiguous))

    __repr__ = __str__

    def __len__(self):
        return self.shape[0] if len(self.shape) else 0

    def __setitem__(self, key, value):
        self.__getitem__(key)._assign(value)
        return self

    def __getitem__(self, key):
        """numpy basic indexing, except that an int index keeps its axis as a
        size-1 dimension while the result has < 3 dims
        (reference nervanacpu.py:166-213)."""
        if not isinstance(key, tuple):
            if isinstance(key, slice) and key == _none_slice:
                return self
            key = (key,)
        fixed = []
        for axis, k in enumerate(key):
            if type(k) is int:
                k = self.shape[axis] + k if k < 0 else k
                k = slice(k, k + 1, None)
            fixed.append(k)
        sub = self._tensor[tuple(fixed)]
        new_shape = list(sub.shape)
        while len(new_shape) > 2 and 1 in new_shape:
            new_shape.remove(1)
        return self.__class__(backend=self.backend, ary=sub.reshape(new_shape),
                              dtype=self._tensor.dtype, base=self)

    def _assign(self, value):
        if isinstance(value, (CPUTensor, OpTreeNode)):
            OpTreeNode.build("assign", self, value)
        elif isinstance(value, (int, float, np.ndarray)):
            self.set(value)
        else:
            raise TypeError("Invalid type for assignment: %s" % type(value))
        return self

    def set(self, value):
        if isinstance(value, np.ndarray):
            if value.dtype != self.dtype:
                value = value.astype(self.dtype)
            assert value.size == self.size
            if value.ndim < self._min_dims:
                value = value.reshape(self.shape)
        self._tensor[:] = value
        return self

    def get(self):
        return self._tensor.copy()

    def raw(self):
        return self._tensor.ctypes.data

    def asnumpyarray(self):
        return self._tensor

    def take(self, indices, axis=None, out=None):
        if type(indices) is self.__class__:
            indices = indices._tensor
        if type(indices) is np.ndarray:
            indices = indices.squeeze()
        new_shape = list(self.shape)
        new_shape[axis] = np.size(indices)
        view = self.__class__(backend=self.backend,
                              ary=self._tensor.take(indices, axis).reshape(new_shape),
                              dtype=self._tensor.dtype, base=self)
        if out is not None:
            return out._assign(view)
        return view

    def fill(self, value):
        self._tensor.fill(value)
        return self

    def copy(self, a):
        return self._assign(a)

    def copy_from(self, a):
        return self._assign(a)

    def reshape(self, *shape):
        if isinstance(shape[0], (tuple, list)):
            shape = tuple(shape[0])
        if shape == self.shape:
            return self
        try:
            ary = self._tensor.reshape(shape)
        except ValueError:
            raise ValueError("The total size of a reshaped tensor must be the same "
                             "as its existing size. Tensor is currently shape %s; "
                             "attempted to reshape to %s." % (self._tensor.shape, shape))
        return self.__class__(backend=self.backend, ary=ary,
                              dtype=self._tensor.dtype, base=self)

    @property
    def T(self):
        if len(self.shape) <= 2:
            ary = self._tensor.transpose()
        else:
            ary = self._tensor.swapaxes(1, 2)
        return self.__class__(backend=self.backend, ary=ary,
                              dtype=self._tensor.dtype, base=self)

    def transpose(self, out=None):
        if out:
            return OpTreeNode.build("assign", out, self.T)
        return self.T

    def share(self, shape, dtype=None, name=None):
        size = int(np.prod(shape))
        if size > self.size:
            raise ValueError("total size of new array must <= size of parent")
        ary = self._tensor.ravel()[:size].reshape(shape)
        return self.__class__(backend=self.backend, ary=ary,
                              dtype=self._tensor.dtype, base=self)


def _cpu_hist(self, tag):
    """log2-magnitude histogram (reference nervanacpu.py:424-445): log2 is taken
    in fp32 whatever the dtype; the lowest bin reaches down to -inf"""
    nbins, offset = self.backend.hist_bins, self.backend.hist_offset
    bins = np.arange(nbins + 1) + float(offset)
    bins[0] = -float("Inf")
    with np.errstate(divide="ignore"):
        log_abs = np.rint(np.log2(np.abs(self._tensor.astype(np.float32))))
    counts, _ = np.histogram(log_abs, density=False, bins=bins)
    return self.backend._hist_tensor(tag)._assign(counts.astype(np.int32).reshape(1, nbins))


CPUTensor.hist = _cpu_hist


def _arg_keepdims(fn):
    """np.argmax/np.argmin with the reduced axis kept
    (reference nervanacpu.py:453-473): first occurrence, int64."""
    def call(op_dict, x):
        axis = op_dict["axis"]
        shape = list(x.shape)
        shape[axis] = 1
        return fn(x, axis=axis).reshape(tuple(shape))
    return call


def _assign_right_to_left(left, right):
    left[:] = right


# Operation table (reference nervanacpu.py:480-522).
NUMPY_CALLS = {
    "assign": _assign_right_to_left,
    # unary
    "neg": lambda x: -x,
    "abs": lambda x: np.abs(x),
    "sgn": lambda x: np.sign(x),
    "sqrt": lambda x: np.sqrt(x),
    "sqr": lambda x: np.square(x),
    "exp": lambda x: np.exp(x),
    "log": lambda x: np.log(x),
    "safelog": lambda x: np.log(np.maximum(x, np.exp(-50.))),
    "exp2": lambda x: np.exp2(x),
    "log2": lambda x: np.log2(x),
    "sig": lambda x: 1. / (1. + np.exp(-x)),
    "sig2": lambda x: 1. / (1. + np.exp2(-x)),
    "tanh": lambda x: np.tanh(x),
    "tanh2": lambda x: (np.exp2(2. * x) - 1.) / (np.exp2(2. * x) + 1.),
    "transpose": lambda x: np.transpose(x),
    "rint": lambda x: np.rint(x),
    "finite": lambda x: np.isfinite(x),      # accelerator-only op, see module docstring
    # binary
    "add": lambda a, b: a + b,
    "sub": lambda a, b: a - b,
    "mul": lambda a, b: a * b,
    "div": lambda a, b: a / b,
    "eq": lambda a, b: a == b,
    "ne": lambda a, b: a != b,
    "lt": lambda a, b: a < b,
    "le": lambda a, b: a <= b,
    "gt": lambda a, b: a > b,
    "ge": lambda a, b: a >= b,
    "pow": lambda a, b: np.power(a, b),
    "minimum": lambda a, b: np.minimum(a, b),
    "maximum": lambda a, b: np.maximum(a, b),
    "dot": lambda a, b: np.dot(a, b),
    # reductions
    "sum": lambda d, x: np.sum(x, axis=d["axis"], keepdims=True),
    "max": lambda d, x: np.max(x, axis=d["axis"], keepdims=True),
    "min": lambda d, x: np.min(x, axis=d["axis"], keepdims=True),
    "argmax": _arg_keepdims(np.argmax),
    "argmin": _arg_keepdims(np.argmin),
}


def _weaken(value):
    """0-d numpy results of scalar-only arithmetic become Python scalars again
    (see the module docstring on value-based casting)."""
    if isinstance(value, np.generic):
        return value.item()
    if isinstance(value, np.ndarray) and value.ndim == 0:
        return value.item()
    return value


def _dense_onehot(op_dict, full_shape):
    """0/1 matrix of ``full_shape`` with ones where the index along ``axis``
    equals ``idx`` (accelerator semantics, cuda_templates.py:484-494)."""
    axis = op_dict["axis"]
    idx = op_dict["idx"]._tensor.reshape(-1).astype(np.int64)
    ar = np.arange(full_shape[axis], dtype=np.int64)
    if axis == 0:
        return (ar[:, None] == idx[None, :]).astype(np.float32)
    return (idx[:, None] == ar[None, :]).astype(np.float32)


class NervanaCPU(Backend):
    """numpy backend for the op-tree path (reference nervanacpu.py:530-904)."""
    backend_name = "cpu"

    def __init__(self, rng_seed=None, default_dtype=np.float32, hist_bins=64,
                 hist_offset=-48, compat_mode=None, num_devices=None,
                 stochastic_round=None, device_id=None, deterministic=None):
        if default_dtype not in (np.float16, np.float32, np.float64):
            raise ValueError("Default data type for nervanacpu backend must be "
                             "float16, 32 or 64")
        super(NervanaCPU, self).__init__(rng_seed, default_dtype, compat_mode=compat_mode)
        self.tensor_cls = CPUTensor
        self.device_type = 0
        self.device_id = 0
        self.hist_bins, self.hist_offset = hist_bins, hist_offset
        self.use_pinned_mem = False
        self.time_marks = {}

    def consume(self, buf_index, hostlist, devlist):
        assert 0 <= buf_index < 2, "Can only double buffer"
        if devlist[buf_index] is None:
            devlist[buf_index] = self.empty_like(hostlist[buf_index].T,
                                                 dtype=hostlist[buf_index].dtype)
        devlist[buf_index][:] = hostlist[buf_index].T

    # -- the interpreter (reference nervanacpu.py:652-715) ---------------------
    def execute(self, optree, numpy_call_dict=NUMPY_CALLS):
        # whole tree is assign(out, onehot): zero-fill + scatter ones
        if (len(optree) == 3 and isinstance(optree[2], OpTreeNode) and
                optree[2][0]["op"] == "onehot"):
            assert optree[0]["op"] == "assign"
            assert isinstance(optree[1], Tensor)
            out = optree[1]._tensor
            axis = optree[2][0]["axis"]
            hot = optree[2][0]["idx"]._tensor.squeeze()
            n = hot.size
            index = [None, None]
            index[axis] = np.asarray(hot, dtype=np.int64).reshape(n)
            index[1 - axis] = np.arange(n)
            out[:] = 0
            out[tuple(index)] = 1
            return out

        postfix = optree.traverse(list())
        full_shape = _full_shape(postfix)
        stack = []
        for p in postfix:
            if isinstance(p, dict):
                op = p["op"]
                if op == "onehot":
                    stack.append(_dense_onehot(p, full_shape))
                elif op in OpCollection.unary_ops:
                    x = stack.pop()
                    stack.append(_weaken(numpy_call_dict[op](x)))
                elif op in OpCollection.binary_ops:
                    right = stack.pop()
                    left = stack.pop()
                    stack.append(_weaken(numpy_call_dict[op](left, right)))
                elif op in OpCollection.reduction_ops:
                    x = stack.pop()
                    stack.append(numpy_call_dict[op](p, x))
                else:
                    raise NotImplementedError(op)
            elif isinstance(p, CPUTensor):
                stack.append(p._tensor)
            else:
                stack.append(p)
        assert len(stack) == 1
        return postfix[0]

    # -- allocation (reference nervanacpu.py:717-904) -----------------------------
    def _dtype(self, dtype):
        return self.default_dtype if dtype is None else dtype

    def empty(self, shape, dtype=None, name=None, persist_values=True,
              parallel=False, distributed=False):
        dtype = self._dtype(dtype)
        return self.tensor_cls(backend=self, ary=np.zeros(shape, dtype), dtype=dtype,
                               name=name, persist_values=persist_values)

    def array(self, ary, dtype=None, name=None, persist_values=True,
              parallel=False, distributed=False):
        dtype = self._dtype(dtype)
        return self.tensor_cls(backend=self, ary=np.array(ary, dtype), dtype=dtype,
                               name=name, persist_values=persist_values)

    def zeros(self, shape, dtype=None, name=None, persist_values=True,
              parallel=False, distributed=False):
        return self.empty(shape, dtype, name, persist_values)

    def ones(self, shape, dtype=None, name=None, persist_values=True,
             parallel=False, distributed=False):
        dtype = self._dtype(dtype)
        return self.tensor_cls(backend=self, ary=np.ones(shape, dtype), dtype=dtype,
                               name=name, persist_values=persist_values)

    def empty_like(self, ary, dtype=None, name=None, persist_values=True):
        dtype = self._dtype(dtype)
        return self.tensor_cls(backend=self, ary=np.zeros(ary.shape, dtype), dtype=dtype,
                               name=name, persist_values=persist_values)

    def zeros_like(self, ary, dtype=None, name=None, persist_values=True):
        return self.empty_like(ary, dtype, name, persist_values)

    # -- dense contraction (reference nervanacpu.py:906-960) ------------------------
    def compound_dot(self, A, B, C, alpha=1.0, beta=0.0, relu=False, bsum=None):
        """C = alpha * A.B + beta * C, ReLU (if asked) on the product term before
        the beta term is added, ``bsum`` = row sums of the final C.

        One deliberate difference from nervanacpu.py:939-948: with beta == 0 that
        code stores the bare product and drops ``alpha``; its own docstring
        (:915-916) and the GPU backend (nervanagpu.py:1441-1470) apply it, and so
        does this."""
        assert A.dtype == B.dtype == C.dtype
        assert A.shape[0] == C.shape[0]
        assert B.shape[1] == C.shape[1]
        assert A.shape[1] == B.shape[0]
        prod = np.dot(A._tensor, B._tensor)
        if alpha != 1.0:
            prod = np.multiply(prod, np.asarray(alpha, dtype=prod.dtype))
        if relu:
            prod = np.maximum(prod, 0)
        if beta == 0:
            C._tensor[:] = prod
        else:
            np.multiply(C._tensor, np.asarray(beta, dtype=C._tensor.dtype), C._tensor)
            np.add(C._tensor, prod, C._tensor)
        if bsum is not None:
            bsum[:] = self.sum(C, 1)
        return C

    def make_binary_mask(self, out, keepthresh=0.5):
        # ones where a host uniform draw falls below the threshold (reference
        # nervanacpu.py:1052-1063)
        out._tensor[:] = (self.rng.uniform(size=out._tensor.shape) < keepthresh).astype(out._tensor.dtype)

    def _uniform_like(self, ary):
        # host draws, as in the reference's binarize (nervanacpu.py:1835)
        return self.array(self.rng.uniform(0, 1, size=ary.shape))

    # -- products over a batch dimension (reference nervanacpu.py:962-1017) ----------
    def batched_dot(self, A, B, C, alpha=1.0, beta=0.0, relu=False):
        assert A.dtype == B.dtype == C.dtype
        dima, dimb, dimc = int(len(A.shape) == 3), int(len(B.shape) == 3), int(len(C.shape) == 3)
        assert dima or dimb, "Tensor A or B must have 3 dims to use batched_dot"
        if dimc:
            assert not dima or A.shape[0] == C.shape[0]
            assert not dimb or B.shape[0] == C.shape[0]
        loops = A.shape[0] if dima else B.shape[0]
        assert not (dima and dimb) or A.shape[0] == B.shape[0]
        assert A.shape[0 + dima] == C.shape[0 + dimc]
        assert B.shape[1 + dimb] == C.shape[1 + dimc]
        assert A.shape[1 + dima] == B.shape[0 + dimb]
        tmp = np.zeros(C.shape)
        for i in range(loops):
            a = A._tensor[i] if dima else A._tensor
            b = B._tensor[i] if dimb else B._tensor
            if dimc:
                tmp[i] = np.dot(a, b)
            else:
                tmp += np.dot(a, b)
        np.multiply(tmp, alpha, tmp)
        if relu:
            np.maximum(tmp, 0, tmp)
        C._tensor[:] = C._tensor * beta + tmp
        return C

    # -- lookup table backward (reference nervanacpu.py:1762-1782) -------------------
    def compound_bprop_lut(self, nin, inputs, error, error_t, dW, pad_idx, alpha=1.0, beta=0):
        wrd_ids = inputs._tensor.reshape(-1)
        unqidx, inv = np.unique(wrd_ids, return_inverse=True)
        for k, wrd_id in enumerate(unqidx):
            if wrd_id != pad_idx:
                group = np.where(inv == k)[0]
                # (the reference assigns self.sum(error.take(group, axis=1), axis=1) through a
                # row view; the same numpy sum, written into the row directly)
                dW._tensor[int(wrd_id), :] = np.sum(error._tensor.take(group, axis=1), axis=1)

    # -- dimension shuffle (reference nervanacpu.py:1046-1051) ------------------------
    def copy_transpose(self, a, out, axes=None, repeat=1):
        out._tensor[:] = np.transpose(a._tensor, axes).copy()

    # -- compensated accumulation ---------------------------------------------------
    def compensated_sum(self, sum_tensor, cmp_tensor, add_tensor, cmp_scale=1.0, add_scale=1.0):
        """The reference's CPU backend has no such method; this restates, in
        numpy float32 arithmetic, the element loop of the accelerator kernel
        (neon/backends/float_ew.py:966-992, round-to-nearest stores) with the
        host-side reset logic of nervanagpu.py:1896-1905.  Pinned in
        tests/test_oracle.py by the defining property of compensated summation
        (many small addends into a float16 accumulator stay within one unit in
        the last place of the exact sum, where plain accumulation stalls)."""
        reset = getattr(cmp_tensor, "kahan_reset", 0)
        count = getattr(cmp_tensor, "kahan_count", 0)
        if reset and count > reset:
            cmp_scale = 0
            count = 0
        assert sum_tensor.dtype.type == cmp_tensor.dtype.type == add_tensor.dtype.type
        cmp_tensor.kahan_count = count + 1
        store = sum_tensor.dtype.type
        s32 = sum_tensor._tensor.astype(np.float32)
        c32 = cmp_tensor._tensor.astype(np.float32)
        a32 = add_tensor._tensor.astype(np.float32)
        y32 = a32 * np.float32(add_scale) - c32 * np.float32(cmp_scale)
        t = (s32 + y32).astype(store)
        c = ((t.astype(np.float32) - s32) - y32).astype(store)
        sum_tensor._tensor[:] = t
        cmp_tensor._tensor[:] = c

    # -- batch normalisation (reference nervanacpu.py:1688-1760), non-binary path ---
    def compound_fprop_bn(self, x, xsum, xvar, gmean, gvar, gamma, beta, y, eps, rho,
                          compute_batch_sum, accumbeta=0.0, relu=False, binary=False,
                          inference=False, outputs=None, layer=None):
        assert not binary
        if inference:
            xhat = (x - gmean) / self.sqrt(gvar + eps)
            y[:] = y * accumbeta + xhat * gamma + beta
            return
        if compute_batch_sum:
            xsum[:] = self.sum(x, axis=1)
        xvar[:] = self.var(x, axis=1)
        xsum[:] = xsum / x.shape[1]
        gmean[:] = gmean * rho + (1.0 - rho) * xsum
        gvar[:] = gvar * rho + (1.0 - rho) * xvar
        xhat = (x - xsum) / self.sqrt(xvar + eps)
        outputs = y.reshape(xhat.shape)
        outputs[:] = xhat * gamma + beta + accumbeta * outputs

    def compound_bprop_bn(self, delta_out, grad_gamma, grad_beta, delta_in, x, xsum, xvar,
                          gamma, eps, binary=False, layer=None):
        assert not binary
        inv_v = 1.0 / self.sqrt(xvar + eps)
        xhat = (x - xsum) * inv_v
        grad_gamma[:] = self.sum(xhat * delta_in, axis=1)
        grad_beta[:] = self.sum(delta_in, axis=1)
        xtmp = (xhat * grad_gamma + grad_beta) / float(x.shape[1])
        delta_out.reshape(delta_in.shape)[:] = ((delta_in - xtmp) * gamma) * inv_v

    # -- histogram buffers (reference nervanacpu.py:1767-1800) ------------------------
    def set_hist_buffers(self, hist_bins, hist_offset):
        self.hist_bins, self.hist_offset = hist_bins, hist_offset
        self.hist_max = 4 * 4096
        self.hist_buf = self.empty((self.hist_max, hist_bins), dtype=np.int32)
        self.hist_idx = 0
        self.hist_map = dict()

    def _hist_tensor(self, tag):
        if getattr(self, "hist_buf", None) is None:
            self.set_hist_buffers(self.hist_bins, self.hist_offset)
        assert self.hist_idx < self.hist_max
        self.hist_map[tag] = self.hist_idx
        row = self.hist_buf[self.hist_idx]
        self.hist_idx += 1
        return row

    # -- timing marks (reference nervanacpu.py:1865-1905) -------------------------
    def init_mark(self):
        return {"time": 0}

    def record_mark(self, marker):
        marker["time"] = time.time()

    def synchronize_mark(self, marker):
        return

    def get_time(self, start, end):
        return (end["time"] - start["time"]) * 1000.0


def _full_shape(postfix):
    """Largest extent per axis over the tensors of a postfix stack; only used
    to size an in-tree one-hot matrix."""
    r, c = 1, 1
    for p in postfix:
        if isinstance(p, Tensor):
            r, c = max(r, p.shape[0]), max(c, p.shape[1])
    return (r, c)
