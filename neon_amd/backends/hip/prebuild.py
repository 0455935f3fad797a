"""
Device-free planning: shape-only tensors and a recording backend.

Generating and compiling a kernel needs the op-tree and the operand geometry
but no device (hiprtc takes the target arch as an option).  This module lets
the build step, the CPU tests and ``kernel_report`` run the very code path the
hip backend runs -- DAG, shape-class choice, code generation, hiprtc -- on a
machine without a GPU, and pre-populates the on-disk kernel cache for the
benchmark trees.
"""
import numpy as np

from neon_amd import configs
from neon_amd.backends.backend import Backend, Block, OpTreeNode, Tensor
from neon_amd.backends.hip import planner
from neon_amd.backends.hip.optree_ir import Program


class ShapeTensor(Tensor):
    """Tensor with geometry and a made-up, 256-byte aligned address."""
    _next_addr = [1 << 32]

    def __init__(self, backend, shape, dtype=np.float32, name=None, strides=None,
                 ptr=None, base=None):
        super(ShapeTensor, self).__init__(backend, shape, dtype, name)
        if len(shape) < 2:
            shape = tuple(shape) + (1,)
        self.shape = tuple(int(d) for d in shape)
        self.dtype = np.dtype(dtype)
        self.size = int(np.prod(self.shape))
        contiguous = []
        acc = 1
        for d in reversed(self.shape):
            contiguous.append(acc)
            acc *= d
        contiguous = tuple(reversed(contiguous))
        self.strides = tuple(strides) if strides is not None else contiguous
        self.is_contiguous = self.strides == contiguous
        self.take_array = None
        self.base = base
        if ptr is None:
            ptr = ShapeTensor._next_addr[0]
            ShapeTensor._next_addr[0] += (self.size * self.dtype.itemsize + 511) // 256 * 256
        self.ptr = ptr

    def __setitem__(self, key, value):
        assert key == slice(None, None, None)
        if isinstance(value, (Tensor, OpTreeNode, int, float)):
            OpTreeNode.build("assign", self, value)
        else:
            raise TypeError("Invalid type for assignment: %s" % type(value))

    def __len__(self):
        return self.shape[0]

    def __repr__(self):
        return "ShapeTensor(%s, %s, strides=%s)" % (self.shape, self.dtype, self.strides)

    __str__ = __repr__

    @property
    def T(self):
        return ShapeTensor(self.backend, self.shape[::-1], self.dtype, self.name,
                           strides=self.strides[::-1], ptr=self.ptr, base=self)


class PlanBackend(Backend):
    """Records assign trees and plans them; never launches."""
    backend_name = "hip-plan"

    def __init__(self, rng_seed=None, default_dtype=np.float32, arch="gfx950",
                 cu_count=256, cache_dir=None, compile_kernels=True, **_ignored):
        super(PlanBackend, self).__init__(rng_seed, default_dtype)
        self.arch = arch
        self.cu_count = cu_count
        self.cache = planner.KernelCache(arch, cache_dir)
        self.compile_kernels = compile_kernels
        self.choices = []          # Choice per executed statement group
        self.coop = True           # False: plan as for a program whose inter-workgroup wait once expired
        self._pending = []
        self._fusing = False

    def empty(self, shape, dtype=None, name=None, **kw):
        return ShapeTensor(self, shape, dtype or self.default_dtype, name)

    zeros = ones = empty

    def empty_like(self, other, name=None, **kw):
        return ShapeTensor(self, other.shape, other.dtype, name)

    zeros_like = empty_like

    def begin(self, block, identifier):
        if block == Block.update:
            self._fusing = True

    def end(self, block, identifier):
        if block == Block.update:
            self._fusing = False
            self._plan(self._pending)
            self._pending = []

    def execute(self, optree):
        if self._fusing:
            self._pending.append(optree)
        else:
            self._plan([optree])
        return optree[1]

    def _plan(self, trees):
        if not trees:
            return
        prog = Program()
        for t in trees:
            prog.add_statement(t)
        prog.finalize()
        ch = planner.choose(prog, self.cu_count, self.coop)
        if self.compile_kernels:
            self.cache.code_object(ch.spec)
        self.choices.append(ch)
        return ch


def benchmark_statements(be):
    """Issue every benchmark tree once on ``be`` (any backend)."""
    f32, f16, i32 = np.float32, np.float16, np.int32
    x, y, out = (be.empty(configs.C1_SHAPE, f32) for _ in range(3))
    configs.c1a(be, out, x, y)
    configs.c1b(be, out)
    configs.c1_fused(be, out, x, y)
    x2, o2 = be.empty(configs.C2_SHAPE, f32), be.empty(configs.C2_SHAPE, f32)
    configs.c2_softmax(be, o2, x2)
    configs.c2_softmax_neon(be, o2, x2)
    p, g, m, v = (be.empty(configs.C3_SHAPE, f32) for _ in range(4))
    configs.c3_adam_step(be, p, g, m, v, 1)              # three kernels, as the reference issues them
    be.begin(Block.update, 0)
    configs.c3_adam_step(be, p, g, m, v, 1)              # fused into one
    be.end(Block.update, 0)
    x4, o4 = be.empty(configs.C4_SHAPE, f16), be.empty(configs.C4_SHAPE, f16)
    gam, bet = be.empty((configs.C4_SHAPE[0], 1), f32), be.empty((configs.C4_SHAPE[0], 1), f32)
    configs.c4_rownorm(be, o4, x4, gam, bet)
    x5 = be.empty(configs.C5_SHAPE, f32)
    am, mx, ce = (be.empty((1, configs.C5_SHAPE[1]), dt) for dt in (i32, f32, f32))
    configs.c5a_argmax(be, am, x5)
    configs.c5b_max(be, mx, x5)


def compile_benchmark_kernels(arch="gfx950", cache_dir=None, verbose=False):
    be = PlanBackend(arch=arch, cache_dir=cache_dir)
    benchmark_statements(be)
    if verbose:
        for ch in be.choices:
            print("  %-9s %-26s grid=%s block=%d %s" % (ch.spec.family, ch.spec.name, ch.grid,
                                                       ch.spec.block, ch.spec.params), flush=True)
    return len(be.choices)
