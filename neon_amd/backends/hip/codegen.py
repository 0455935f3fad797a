"""
Typed DAG -> HIP C++ for gfx950.

The generated text is appended to ``neon_device.h`` and compiled with hiprtc.
It replaces the reference's string templates (cuda_templates.py:45-135 filled
in by float_ew.py:268-617) but is organised around how CDNA4 wants to be fed
rather than around one-thread-block-per-line:

  * every global access is one ``nh_raw<T,V>`` / ``nh_out<T,V>`` tile per lane:
    V consecutive elements, 16 bytes wherever layout and alignment allow;
  * lanes always run along the contiguous (column) axis, for axis-0 reductions
    too, where the reference walked down a strided column per thread
    (float_ew.py:709-711);
  * a line that has to be swept more than once (softmax, variance,
    normalisation) is loaded once and kept in registers in storage format;
  * reductions are wave64 DPP all-reduces; LDS only joins waves; workgroups
    that share a long column strip combine through a ticket, never by waiting.

Kernel families
  ``ew``       no reduction; one or several assign statements per launch
  ``row``      reductions along axis 1; a team of LX lanes owns a row
  ``col``      reductions along axis 0; a workgroup owns a strip of columns
               and all rows, which stay in registers
  ``colsplit`` one level of axis-0 reductions over many rows; (strip x row
               chunk) workgroups, partials folded by the last one to finish

Arithmetic is fp32 whatever the storage type.  Parameters, in order: per
tensor slot ``(pointer, row stride, column stride)`` in elements, one float per
constant slot, ``R``, ``C``, then family-specific extras.
"""
import hashlib
import os
import re

from neon_amd.backends.hip.optree_ir import DTYPE_CODE, used_nodes

CTYPE = {"f4": "float", "f2": "nh_f16", "b2": "nh_bf16", "i4": "nh_i32", "u4": "nh_u32",
         "i2": "nh_i16", "u2": "nh_u16", "i1": "nh_i8", "u1": "nh_u8"}

_BIN = {"add": "({0} + {1})", "sub": "({0} - {1})", "mul": "({0} * {1})",
        "div": "({0} / {1})",
        "eq": "(({0} == {1}) ? 1.0f : 0.0f)", "ne": "(({0} != {1}) ? 1.0f : 0.0f)",
        "lt": "(({0} < {1}) ? 1.0f : 0.0f)", "le": "(({0} <= {1}) ? 1.0f : 0.0f)",
        "gt": "(({0} > {1}) ? 1.0f : 0.0f)", "ge": "(({0} >= {1}) ? 1.0f : 0.0f)",
        "pow": "powf({0}, {1})", "minimum": "nh_min({0}, {1})",
        "maximum": "nh_max({0}, {1})"}
_UN = {"neg": "(-{0})", "abs": "__builtin_fabsf({0})", "sgn": "nh_sgn({0})",
       "sqrt": "sqrtf({0})", "sqr": "nh_sqr({0})", "exp": "expf({0})",
       "log": "logf({0})", "exp2": "exp2f({0})", "log2": "log2f({0})",
       "sig": "nh_sig({0})", "sig2": "nh_sig2({0})", "tanh": "tanhf({0})",
       "tanh2": "nh_tanh2({0})", "safelog": "nh_safelog({0})",
       "rint": "rintf({0})", "finite": "nh_finite({0})", "ident": "({0})",
       "exp_nonpos": "nh_exp_nonpos({0})"}
_RED_OP = {"sum": "nh_op_sum", "max": "nh_op_max", "min": "nh_op_min",
           "argmax": "nh_op_argmax", "argmin": "nh_op_argmin"}


# The ticket counters of neighbouring strips (rows, for the cooperating row family) sit this many 32-bit words apart.  Atomics on one
# cache line are served one after the other, whichever words of it they address: with the
# counters of all strips in one line, the 256 workgroups of an (8 strips x 32 chunks) grid queued
# behind each other for 2 us (max over (32000,256): 7.3 -> 5.1 us with a line per strip).
LOCAL_EXP_REUSE = os.environ.get("NEON_HIP_LOCAL_EXP_REUSE", "1") != "0"
TAGGED_EXCHANGE = os.environ.get("NEON_HIP_TAGGED_EXCHANGE", "1") != "0"
TICKET_STRIDE_WORDS = 64


# Streaming kernels (working set far beyond the caches) read with non-temporal
# loads.  Their stores are ordinary ones, except in the row family: measured
# on the 7-stream fused Adam update, non-temporal loads with ordinary stores
# run at 6.5-6.7 TB/s against 5.9-6.2 TB/s with both non-temporal (axpby,
# in-place sigmoid and the column softmax gain 3-7 % the same way), whereas the
# row kernels, whose workgroups all read, then all write, lose 20 % without
# non-temporal stores.
STREAM_STORES = {"ew": False, "row": True, "col": False, "colsplit": False}


class Spec(object):
    """Everything the launcher needs for one generated kernel."""

    def __init__(self, family, name, source, fmt, block, lds_bytes, params):
        self.family = family
        self.name = name
        self.source = source
        self.fmt = fmt                # struct format of the packed arguments
        self.block = block            # threads per workgroup
        self.lds_bytes = lds_bytes    # static LDS is declared in the source; kept for reports
        self.params = params          # tiling parameters (dict) used to size the grid


class _Lines(object):
    def __init__(self):
        self.out = []
        self.ind = 0

    def __call__(self, text=""):
        self.out.append(("    " * self.ind + text) if text else "")

    def open(self, text):
        self(text + " {")
        self.ind += 1

    def close(self, tail=""):
        self.ind -= 1
        self("}" + tail)

    def text(self):
        return "\n".join(self.out) + "\n"


class _Gen(object):
    """State shared by the family emitters for one program."""

    def __init__(self, prog, V, stream=False, family="ew"):
        self.prog = prog
        self.V = V
        self.R, self.C = prog.domain
        self.axis = prog.axis
        self.L = _Lines()
        # streaming kernels (working set far beyond the caches) mark their
        # global accesses non-temporal
        self.pos = ("0", "0")      # (row, column) expressions of the element being emitted
        self.pos_v = 1             # ... the column expression is a multiple of this
        self.ld = "load_stream" if stream else "load"
        self.st = "store_stream" if (stream and STREAM_STORES[family]) else "store"
        self.prefetched = set()    # gather nodes whose operands were fetched ahead of the sweep
        self.one_declared = False  # the kernel holds ``nh_one`` (see declare_one)

    def is_half_leaf(self, n):
        return n.kind == "T" and DTYPE_CODE[self.prog.tensors[n.slot].dtype] == "f2"

    def declare_one(self):
        """kernels that read fp16 tensors keep an opaque 1.0f for mixed-precision fma forms"""
        if any(t.read and DTYPE_CODE[t.dtype] == "f2" for t in self.prog.tensors):
            self.L("const float nh_one = nh_opaque_one();")
            self.one_declared = True

    # -- parameters -----------------------------------------------------------------
    def slot_ctype(self, slot):
        return CTYPE[DTYPE_CODE[slot.dtype]]

    def col_unit(self, slot):
        """True when the slot's column stride is the literal 1."""
        return slot.shape[1] > 1 and slot.strides[1] == 1

    def param_list(self, extras):
        ps, fmt = [], ""
        no_alias = not self.prog.overlapping_slots()
        for t in self.prog.tensors:
            qual = "" if t.written else "const "
            restrict = " __restrict__" if no_alias else ""
            ps.append("%s%s*%s a%d" % (qual, self.slot_ctype(t), restrict, t.index))
            ps.append("long long sr%d" % t.index)
            ps.append("long long sc%d" % t.index)
            fmt += "Pqq"
        for i in range(len(self.prog.consts)):
            ps.append("float k%d" % i)
            fmt += "f"
        ps += ["int R", "int C"]
        fmt += "ii"
        if self.prog.rand_count:
            ps += ["unsigned int rng_seed", "unsigned long long rng_base"]
            fmt += "IQ"
        for decl, f in extras:
            ps.append(decl)
            fmt += f
        return ", ".join(ps), "@" + fmt

    # -- addresses ------------------------------------------------------------------
    def addr(self, slot, r, c):
        """Element address of (r, c) in a slot, honouring broadcast dims and
        index vectors of gather / scatter views."""
        parts = ["a%d" % slot.index]

        def looked_up(pos):
            # an index outside the indexed tensor is clamped into it (numpy raises
            # IndexError; a kernel can only stay inside the allocation)
            idx = "a%d[(long long)(%s)]" % (slot.take_slot, pos)
            if slot.take_extent:
                return "(long long)nh_clamp_index(%s, %d)" % (idx, slot.take_extent)
            return "(long long)" + idx
        if slot.take_axis == 0:
            # (a view of a single gathered row still has to look its index up)
            parts.append("%s * sr%d" % (looked_up(r if slot.shape[0] > 1 else "0"), slot.index))
        elif slot.shape[0] > 1:
            parts.append("(long long)(%s) * sr%d" % (r, slot.index))
        if slot.take_axis == 1:
            parts.append("%s * sc%d" % (looked_up(c if slot.shape[1] > 1 else "0"), slot.index))
        elif slot.shape[1] > 1:
            if self.col_unit(slot):
                if self.split_columns and c == "c":
                    # the part of the column that is the same for every lane joins the base
                    # (scalar registers); the lane's own part comes last and is 32 bits wide, so
                    # that the access takes a scalar base and a one-register offset
                    parts.append("cu")
                    parts.append("cl")
                else:
                    parts.append("(long long)(%s)" % c)
            else:
                parts.append("(long long)(%s) * sc%d" % (c, slot.index))
        return " + ".join(parts)

    # set by families whose column position is in scope as ``cu`` (long long, uniform over the
    # workgroup) + ``cl`` (unsigned int, the lane's share) besides ``c``
    split_columns = False

    # -- loads -------------------------------------------------------------------------
    def leaf_nodes(self, nodes):
        return [n for n in nodes if n.kind in ("T", "H")]

    def tile_name(self, n, sfx):
        return ("x%d%s" % (n.slot, sfx)) if n.kind == "T" else ("h%d_%d%s" % (n.slot, n.axis, sfx))

    def tile_width(self, n, V):
        if n.kind == "T":
            return V if self.prog.tensors[n.slot].shape[1] > 1 else 1
        return V if n.axis == 0 else 1

    def tile_type(self, n, V):
        slot = self.prog.tensors[n.slot]
        return "nh_raw<%s, %d>" % (self.slot_ctype(slot), self.tile_width(n, V))

    def tile_addr(self, n, r, c):
        slot = self.prog.tensors[n.slot]
        if n.kind == "T":
            return self.addr(slot, r, c)
        # one-hot index vector: flat, contiguous; indexed by the position along
        # the axis that is *not* hot
        return "a%d + (long long)(%s)" % (slot.index, c if n.axis == 0 else r)

    col_tail = False     # column families: the last column tile is partial (`cfull`, `clim` in scope)

    def emit_load(self, n, r, c, V, sfx, declare=True, target=None):
        name = target or self.tile_name(n, sfx)
        if declare:
            self.L("%s %s;" % (self.tile_type(n, V), name))
        self.L(self.load_stmt(name, n, r, c, V))

    def load_stmt(self, name, n, r, c, V, op=None):
        addr = self.tile_addr(n, r, c)
        op = op or self.load_op(n)
        if self.col_tail and self.tile_width(n, V) > 1:
            return "if (cfull) %s.%s(%s); else %s.load_partial(%s, clim);" % (name, op, addr, name, addr)
        return "%s.%s(%s);" % (name, op, addr)

    def store_stmt(self, name, op, addr, width):
        if self.col_tail and width > 1:
            return "if (cfull) %s.%s(%s); else %s.store_partial(%s, clim);" % (name, op, addr, name, addr)
        return "%s.%s(%s);" % (name, op, addr)

    def load_op(self, n):
        """streaming (non-temporal) loads are for data touched once: operands
        that are broadcast along an axis are re-read by many workgroups and
        stay on ordinary loads"""
        t = self.prog.tensors[n.slot]
        if self.ld == "load_stream" and n.kind == "T" and (
                (t.shape[0] == 1 and self.R > 1) or (t.shape[1] == 1 and self.C > 1)):
            return "load"
        return self.ld

    # -- expressions -----------------------------------------------------------------
    def leaf_value(self, n, tile, r, c, V):
        w = self.tile_width(n, V)
        j = "j" if w > 1 else "0"
        if n.kind == "T":
            return "%s.get(%s)" % (tile, j)
        if n.axis == 0:
            return "((%s.geti(%s) == (int)(%s)) ? 1.0f : 0.0f)" % (tile, j, r)
        return "((%s.geti(0) == (int)((%s) + j)) ? 1.0f : 0.0f)" % (tile, c)

    def expr_text(self, n, a, in_loop=True):
        """C expression of elementwise node ``n`` over the operand expressions
        ``a``; ``in_loop``: the expression sits in a loop over the elements of a
        line (not a one-off evaluation)"""
        if n.op.startswith("quant:"):
            return "nh_quant<%s>(%s)" % (CTYPE[n.op.split(":")[1]], a[0])
        if n.op == "zero_index":
            return "0.0f"
        if n.op == "rand" or n.op.startswith("sround:"):
            # random word number = launch base + element index * streams + this node's stream
            r, c = self.pos
            streams = self.prog.rand_count
            # the launch base is even; the words of a lane's tile pair up
            # on shared evaluations when its first word is even as well
            aligned = streams % 2 == 0 or (self.pos_v % 2 == 0 and (self.C % 2 == 0 or self.R == 1))
            word = ("nh_rand_word<%d, %d, %s>(rng_seed, rng_base + ((unsigned long long)(%s) * "
                    "(unsigned long long)C + (unsigned long long)(%s)) * %dull, j)"
                    % (streams, n.slot, "true" if aligned else "false", r, c, streams))
            if n.op == "rand":
                return "nh_rand01(%s)" % word
            if n.op == "sround:int":
                return "nh_sround_int(%s, %s)" % (a[0], word)
            return "nh_sround(%s, %s, %s)" % (a[0], n.op.split(":")[1], word)
        if len(a) == 1:
            if n.op == "exp" and EXP_OF_NONPOSITIVE and _below_its_maximum(n.args[0]):
                # exp(x - max(x)): the argument cannot be positive, which is all nh_exp_nonpos
                # asks for (softmax and log-sum-exp trees; 7 instructions against expf's 13)
                return "nh_exp_nonpos({0})".format(*a)
            return _UN[n.op].format(*a)
        if n.op in ("add", "sub") and self.one_declared and any(self.is_half_leaf(x) for x in n.args):
            # widening of the fp16 operand and the addition in one instruction
            # (v_fma_mix_f32); bit-identical to the plain sum / difference
            if self.is_half_leaf(n.args[0]):
                return "__builtin_fmaf({0}, nh_one, {2}{1})".format(a[0], a[1], "-" if n.op == "sub" else "")
            return "__builtin_fmaf({1}, {2}nh_one, {0})".format(a[0], a[1], "-" if n.op == "sub" else "")
        if n.op == "div" and in_loop and RECIPROCAL_OF_BROADCAST and _broadcast_under(n.args[1], n.args[0]):
            # the divisor is constant along an axis the dividend varies on
            return "nh_div_by_line({0}, {1})".format(*a)
        return _BIN[n.op].format(*a)

    def emit_exprs(self, nodes, ref, skip):
        """Emit ``const float t<id> = ...;`` for E (and G) nodes of ``nodes``
        not in ``skip``; ``ref(node)`` names the value of any operand."""
        for n in nodes:
            if n.nid in skip:
                continue
            if n.kind == "G":
                self.emit_gather(n, ref)
            elif n.kind == "E":
                self.L("const float t%d = %s;" % (n.nid, self.expr_text(n, [ref(x) for x in n.args])))

    def gather_operands(self, n):
        """the nodes of a gather's expression, reductions (finished, taken from
        the caller) excluded, in evaluation order"""
        expr = n.args[0]
        return _needed([expr], set(m.nid for m in used_nodes([expr]) if m.kind == "R"))

    def emit_gather_prefetch(self, nodes, V, guard):
        """Fetch, ahead of the sweep, what the gathers among ``nodes`` will read
        (the hot row's index and the operands at that row, for the V columns
        of the lane's tile): two dependent memory round trips that otherwise
        sit at the very end of the kernel, after the last fold."""
        L = self.L
        for n in nodes:
            if n.kind != "G":
                continue
            hot_slot = self.prog.tensors[n.args[1].slot]
            leaves = [m for m in self.gather_operands(n) if m.kind == "T"]
            L("int gi%d[%d];" % (n.nid, V))
            for m in leaves:
                L("float gp%d_%d[%d];" % (n.nid, m.nid, V))
            L("#pragma unroll")
            L.open("for (int j = 0; j < %d; ++j)" % V)
            L("gi%d[j] = -1;" % n.nid)
            for m in leaves:
                L("gp%d_%d[j] = 0.0f;" % (n.nid, m.nid))
            col = "(%s) + j" % self.pos[1]
            L.open("if ((%s) && %s < C)" % (guard, col))
            L("gi%d[j] = (int)a%d[%s];" % (n.nid, hot_slot.index, col))
            L.open("if (gi%d[j] >= 0 && gi%d[j] < R)" % (n.nid, n.nid))
            for m in leaves:
                slot = self.prog.tensors[m.slot]
                L("gp%d_%d[j] = nh_load_cvt(*(%s));" % (n.nid, m.nid, self.addr(slot, "gi%d[j]" % n.nid, col)))
            L.close()
            L.close()
            L.close()
            self.prefetched.add(n.nid)

    def emit_gather(self, n, ref):
        """``t<id>`` = the expression ``n.args[0]`` at row ``idx[column]`` of the
        one-hot ``n.args[1]`` (0 for an index outside the rows).  Emitted inside
        a loop over ``j`` at a one-value-per-column position; reductions inside
        the expression are finished by then and come from ``ref``."""
        expr, hot = n.args
        L = self.L
        col = "(%s) + j" % self.pos[1]
        hot_slot = self.prog.tensors[hot.slot]
        sub = self.gather_operands(n)
        early = n.nid in self.prefetched
        L("float t%d = 0.0f;" % n.nid)
        L.open("if (%s < C)" % col)
        if early:
            L("const int gi%d_ = gi%d[j];" % (n.nid, n.nid))
        else:
            L("const int gi%d_ = (int)a%d[%s];" % (n.nid, hot_slot.index, col))
        L.open("if (gi%d_ >= 0 && gi%d_ < R)" % (n.nid, n.nid))
        name = lambda m: "u%d_%d" % (n.nid, m.nid)

        def at_row(m):
            if m.kind == "R":
                return ref(m)
            if m.kind == "C":
                return "k%d" % m.slot
            return name(m)

        for m in sub:
            if m.kind == "T":
                slot = self.prog.tensors[m.slot]
                if early:
                    L("const float %s = gp%d_%d[j];" % (name(m), n.nid, m.nid))
                else:
                    L("const float %s = nh_load_cvt(*(%s));" % (name(m), self.addr(slot, "gi%d_" % n.nid, col)))
            elif m.kind == "H":
                L("const float %s = ((int)a%d[%s] == gi%d_) ? 1.0f : 0.0f;"
                  % (name(m), self.prog.tensors[m.slot].index, col, n.nid))
            elif m.kind == "E":
                L("const float %s = %s;" % (name(m), self.expr_text(m, [at_row(x) for x in m.args], in_loop=False)))
        L("t%d = %s;" % (n.nid, at_row(expr)))
        L.close()
        L.close()


RECIPROCAL_OF_BROADCAST = os.environ.get("NEON_HIP_RCP", "1") != "0"
FMA_IN_SUMS = os.environ.get("NEON_HIP_FMA_SUMS", "1") != "0"
# results stored as 16-bit floats: a chain of multiplications / divisions by
# per-line values and a final per-line addend collapse into one multiply-add
EXP_OF_NONPOSITIVE = os.environ.get("NEON_HIP_EXP_NONPOS", "1") != "0"
AFFINE_16BIT_OUTPUTS = os.environ.get("NEON_HIP_AFFINE16", "1") != "0"


def _broadcast_under(b, a):
    """b is constant along at least one axis on which a varies, and varies on none that a does not"""
    return (b.vr <= a.vr and b.vc <= a.vc) and (b.vr < a.vr or b.vc < a.vc)


def _affine_in_line(root, constant):
    """``root`` as ``atom * A + B``: walks down from ``root`` through additions of
    and multiplications / divisions by values that are constant along the line
    (``constant(node)``), never distributing a product over a sum -- the
    subtraction that centres the data stays as written inside ``atom``.
    Returns (atom, [('mul'|'div', node)...], [('add'|'sub', node)...]) with the
    factors in evaluation order, or None when nothing can be peeled off.
    Addends are only taken from the outside (before any factor), so that
    ``root == atom * prod(factors) + sum(addends)`` holds term for term."""
    addends, mults = [], []
    n = root
    # outer additive terms
    while n.kind == "E" and n.op in ("add", "sub") and len(n.args) == 2:
        a, b = n.args
        if constant(b) and not constant(a):
            addends.append(("add" if n.op == "add" else "sub", b))
            n = a
        elif constant(a) and not constant(b) and n.op == "add":
            addends.append(("add", a))
            n = b
        else:
            break
    # multiplicative chain below them
    while n.kind == "E" and n.op in ("mul", "div") and len(n.args) == 2:
        a, b = n.args
        if constant(b) and not constant(a):
            mults.append((n.op, b))
            n = a
        elif constant(a) and not constant(b) and n.op == "mul":
            mults.append(("mul", a))
            n = b
        else:
            break
    if constant(n) or n is root:
        return None
    return n, mults, addends


def _below_its_maximum(n):
    """n is ``v - max(v)`` along some axis: never positive (NaN aside)"""
    if n.kind != "E" or n.op != "sub" or len(n.args) != 2:
        return False
    v, m = n.args
    return m.kind == "R" and m.op == "max" and m.args[0] is v


def _needed(targets, available):
    """Nodes to evaluate for ``targets`` given already-available reductions."""
    seen = {}
    todo = list(targets)
    while todo:
        n = todo.pop()
        if n.nid in seen or n.nid in available:
            continue
        seen[n.nid] = n
        if n.kind != "G":           # an expression evaluated at one row only is emitted by its gather node
            todo.extend(n.args)
    return [seen[k] for k in sorted(seen)]


KERNEL_NAME_OPS = 10      # operators spelled out in a kernel's name (the reference: 15, float_ew.py:478-479)


def _kernel_name(family, source_body, prog=None):
    """``nk_<family>_<operators>_<hash>``: the tree's operators in evaluation
    order, so that a profiler row can be read without a side table (the
    reference joins its op names the same way, float_ew.py:478-479, 590), then
    a hash of the generated text."""
    ops = []
    if prog is not None:
        for n in used_nodes([st.root for st in prog.statements]):
            if n.kind in ("E", "R", "G", "H") and n.op:
                ops.append(re.sub(r"\W", "", n.op))
    if len(ops) > KERNEL_NAME_OPS:
        ops = ops[:KERNEL_NAME_OPS] + ["etc"]
    if not ops:
        ops = ["copy"]
    return "nk_%s_%s_%s" % (family, "_".join(ops), hashlib.sha1(source_body.encode()).hexdigest()[:12])


def _finish(family, g, head, fmt, block, lds, params):
    body = g.L.text()
    name = _kernel_name(family, head + body + repr(sorted(params.items())), g.prog)
    src = head.replace("@NAME@", name) + body
    return Spec(family, name, src, fmt, block, lds, params)


# =====================================================================================
# family: ew
# =====================================================================================
def gen_ew(prog, V, LX, LY, UC, UR, tail, stream=False):
    """Elementwise kernel.  Workgroup = LX column-lanes x LY row-lanes; a lane
    handles UC column tiles x UR rows per step, all loads issued before the
    first store.  ``tail``: emit a scalar path for a last partial tile
    (only needed when C % V != 0, which the planner allows for single-row
    domains)."""
    g = _Gen(prog, V, stream)
    L = g.L
    T = LX * LY
    params, fmt = g.param_list([("int row_tiles", "i")])
    head = ('extern "C" __global__ __launch_bounds__(%d) void @NAME@(%s)\n' % (T, params))
    roots = [st.root for st in prog.statements]
    nodes = _needed(roots, {})
    leaves = g.leaf_nodes(nodes)

    # operands that are one row for every row of the domain ((1, C) vectors):
    # a lane's column position does not change while it walks down the rows,
    # so their tiles are fetched once, ahead of the row loop, instead of once
    # per row (fp16 x * fp32 row vector over (4096,65536): 272 -> 186 us; letting
    # a workgroup walk several row tiles on top of that was slower)
    def row_invariant(n):
        if n.kind != "T" or g.R == 1 or tail:
            return False
        t = prog.tensors[n.slot]
        return t.shape[0] == 1 and t.shape[1] > 1 and t.take_axis is None
    hoisted = set(n.nid for n in leaves if row_invariant(n))

    def tile_of(n, sfx):
        if n.nid in hoisted:
            return g.tile_name(n, "_%s_h" % sfx.split("_")[1])
        return g.tile_name(n, sfx)

    def ref_for(sfx, r, c, Vv):
        g.pos = (r, c)
        g.pos_v = Vv

        def ref(n):
            if n.kind == "C":
                return "k%d" % n.slot
            if n.kind in ("T", "H"):
                return g.leaf_value(n, tile_of(n, sfx), r, c, Vv)
            return "t%d" % n.nid
        return ref

    def body(sfx, r, c, Vv, loads_only=False, compute_only=False):
        if not compute_only:
            for n in leaves:
                if n.nid not in hoisted:
                    g.emit_load(n, r, c, Vv, sfx, declare=False)
        if loads_only:
            return
        for st in prog.statements:
            w = Vv if st.out.shape[1] > 1 else 1
            L("nh_out<%s, %d> o%d%s; o%d%s.clear();" % (g.slot_ctype(st.out), w, st.out.index, sfx,
                                                       st.out.index, sfx))
        if Vv > 1:
            L("#pragma unroll")
        L.open("for (int j = 0; j < %d; ++j)" % Vv)
        g.emit_exprs(nodes, ref_for(sfx, r, c, Vv), {})
        for st in prog.statements:
            w = Vv if st.out.shape[1] > 1 else 1
            jj = "j" if w > 1 else "0"
            val = ref_for(sfx, r, c, Vv)(st.root)
            if w == 1 and Vv > 1:
                L("if (j == 0) o%d%s.set(0, %s);" % (st.out.index, sfx, val))
            else:
                L("o%d%s.set(%s, %s);" % (st.out.index, sfx, jj, val))
        L.close()
        for st in prog.statements:
            L("o%d%s.%s(%s);" % (st.out.index, sfx, g.st, g.addr(st.out, r, c)))

    L.open("")
    g.declare_one()
    L("const int tx = threadIdx.x %% %d, ty = threadIdx.x / %d;" % (LX, LX))
    if hoisted:
        for uc in range(UC):
            L("const long long ch_%d = ((long long)(blockIdx.x * %d + %d) * %d + tx) * %d;" % (uc, UC, uc, LX, V))
            for n in leaves:
                if n.nid in hoisted:
                    name = g.tile_name(n, "_%d_h" % uc)
                    L("%s %s; %s.zero();" % (g.tile_type(n, V), name, name))
                    L("if (ch_%d + %d <= C) %s.load(%s);" % (uc, V, name, g.tile_addr(n, "0", "ch_%d" % uc)))
    L.open("for (int rt = blockIdx.y; rt < row_tiles; rt += gridDim.y)")
    units = [(uc, ur) for uc in range(UC) for ur in range(UR)]
    for (uc, ur) in units:
        s = "_%d_%d" % (uc, ur)
        L("const long long c%s = ((long long)(blockIdx.x * %d + %d) * %d + tx) * %d;" % (s, UC, uc, LX, V))
        L("const long long r%s = ((long long)rt * %d + %d) * %d + ty;" % (s, UR, ur, LY))
        L("const bool ok%s = (r%s < R) && (c%s + %d <= C);" % (s, s, s, V))
        for n in leaves:
            if n.nid not in hoisted:
                L("%s %s; %s.zero();" % (g.tile_type(n, V), g.tile_name(n, s), g.tile_name(n, s)))
    for (uc, ur) in units:
        s = "_%d_%d" % (uc, ur)
        L.open("if (ok%s)" % s)
        body(s, "r" + s, "c" + s, V, loads_only=True)
        L.close()
    for (uc, ur) in units:
        s = "_%d_%d" % (uc, ur)
        L.open("if (ok%s)" % s)
        body(s, "r" + s, "c" + s, V, compute_only=True)
        L.close()
        if tail and V > 1:
            L.open("else if (r%s < R && c%s < C)" % (s, s))
            L.open("for (long long e = c%s; e < C; ++e)" % s)
            for n in leaves:
                L("%s %s;" % (g.tile_type(n, 1), g.tile_name(n, "_e")))
            body("_e", "r" + s, "e", 1)
            L.close()
            L.close()
    L.close()
    L.close()
    return _finish("ew", g, head, fmt, T, 0,
                   dict(V=V, LX=LX, LY=LY, UC=UC, UR=UR, tail=bool(tail), stream=bool(stream),
                        hoisted=len(hoisted)))


# =====================================================================================
# shared pieces of the reduction families
# =====================================================================================
def _levels(prog):
    """reductions grouped by the sweep that produces them: sweep s yields the
    reductions of level s+1."""
    per = {}
    for n in prog.nodes:
        if n.kind == "R":
            per.setdefault(n.level - 1, []).append(n)
    return per


def _live_reductions(prog):
    roots = [st.root for st in prog.statements]
    return [n for n in used_nodes(roots) if n.kind == "R"]


_EXPENSIVE = {"exp", "log", "exp2", "log2", "tanh", "tanh2", "sig", "sig2", "pow", "sqrt",
              "div", "safelog"}


def _costly_nodes(prog):
    costly = {}
    for n in prog.nodes:            # topological order
        if n.kind == "E":
            costly[n.nid] = (n.op in _EXPENSIVE) or any(costly.get(a.nid, False) for a in n.args)
    return costly


def _overwriting_values(prog, stages, resident_ok):
    """Kept values that cost no registers: (node, leaf) pairs where ``node`` is
    an expensive elementwise result that two or more sweeps need and ``leaf``
    is a resident float32 operand that nothing after the node's first sweep
    reads except through the node (softmax: once the maximum is known
    exp(x - max) can take x's place).  The node's value is written over the
    leaf's registers at the end of the sweep that first computes it.
    ``resident_ok(leaf)`` says whether the leaf's tile is one 32-bit word per
    element."""
    reductions = set(n.nid for n in prog.nodes if n.kind == "R")
    costly = _costly_nodes(prog)
    pairs = []                      # (node, leaf, first sweep that computes node)

    def avail_at(t, extra=()):
        # a kept value exists from the sweep after the one that computes it
        return reductions | set(n.nid for n, _, f in list(pairs) + list(extra) if f < t)

    while True:
        taken = set(leaf.nid for _, leaf, _ in pairs)
        first, count, by_id = {}, {}, {}
        for s, targets in enumerate(stages):
            for n in _needed(targets, avail_at(s)):
                if n.kind == "E" and n.vr and n.vc and costly.get(n.nid):
                    first.setdefault(n.nid, s)
                    count[n.nid] = count.get(n.nid, 0) + 1
                    by_id[n.nid] = n
        found = None
        for nid in sorted((k for k, c in count.items() if c >= 2), reverse=True):
            n, f = by_id[nid], first[nid]
            later = set()
            for t in range(f + 1, len(stages)):
                later.update(m.nid for m in _needed(stages[t], avail_at(t, [(n, None, f)])))
            for leaf in _needed([n], avail_at(f)):
                if (leaf.kind == "T" and leaf.nid not in taken and leaf.nid not in later
                        and resident_ok(leaf)):
                    found = (n, leaf, f)
                    break
            if found:
                break
        if not found:
            return [(n, leaf) for n, leaf, _ in pairs]
        pairs.append(found)


def _kept_values(prog, stages, limit, already=()):
    """Elementwise results worth keeping in registers between sweeps: nodes
    that two or more sweeps need and that cost a transcendental or a division
    to recompute (softmax's exp(x - max)).  ``stages`` lists the targets of
    each sweep in order; at most ``limit`` nodes are returned, outermost
    first.  ``already``: nodes kept by other means."""
    reductions = set(n.nid for n in prog.nodes if n.kind == "R")
    costly = _costly_nodes(prog)
    kept = []
    while len(kept) < limit:
        avail = reductions | set(k.nid for k in kept) | set(n.nid for n in already)
        count, by_id = {}, {}
        for targets in stages:
            for n in _needed(targets, avail):
                if n.kind == "E" and n.vr and n.vc and costly.get(n.nid):
                    count[n.nid] = count.get(n.nid, 0) + 1
                    by_id[n.nid] = n
        cands = [nid for nid, c in count.items() if c >= 2]
        if not cands:
            break
        kept.append(by_id[max(cands)])
    return kept


class _RedGen(_Gen):
    """Common machinery of row / col / colsplit."""

    def __init__(self, prog, V, stream=False, family="row"):
        super(_RedGen, self).__init__(prog, V, stream, family)
        self.col_axis = (prog.axis == 0)   # reductions leave one value per column

    # sum(exp(x - max(x))) accumulated together with the maximum as a running
    # (max, sum) pair: the max node stands for both, the sum node is skipped
    @staticmethod
    def fused_sum(n):
        return n.kind == "R" and n.lse_max is not None

    @staticmethod
    def fused_max(n):
        return n.kind == "R" and n.lse_sum is not None

    def is_pair(self, n):
        return n.is_index or self.fused_max(n)

    def red_op(self, n):
        return "nh_op_lse" if self.fused_max(n) else _RED_OP[n.op]

    def own_reductions(self, nodes):
        return [n for n in nodes if not self.fused_sum(n)]

    # value of a finished reduction at element j of the lane's tile
    def red_ref(self, n):
        if self.col_axis:
            return ("(float)ri%d[j]" % n.nid) if n.is_index else ("rv%d[j]" % n.nid)
        return ("(float)ri%d" % n.nid) if n.is_index else ("rv%d" % n.nid)

    def make_ref(self, sfx, r, c, Vv, tiles=None, vals=None):
        self.pos = (r, c)
        self.pos_v = Vv

        def ref(n):
            if vals and n.nid in vals:
                return vals[n.nid]
            if n.kind == "C":
                return "k%d" % n.slot
            if n.kind in ("T", "H"):
                tile = tiles[n.nid] if tiles and n.nid in tiles else self.tile_name(n, sfx)
                return self.leaf_value(n, tile, r, c, Vv)
            if n.kind == "R":
                return self.red_ref(n)
            return "t%d" % n.nid
        return ref

    def declare_acc(self, n):
        L = self.L
        op = self.red_op(n)
        if self.col_axis:
            if self.is_pair(n):
                L("nh_pair acc%d[%d];" % (n.nid, self.V))
            else:
                L("float acc%d[%d];" % (n.nid, self.V))
            L("#pragma unroll")
            L("for (int j = 0; j < %d; ++j) acc%d[j] = %s::init();" % (self.V, n.nid, op))
        else:
            L("%s acc%d = %s::init();" % ("nh_pair" if self.is_pair(n) else "float", n.nid, op))

    def accumulate(self, n, val, index, ref=None):
        """fold one element into the lane's accumulator (inside the j loop)"""
        op = self.red_op(n)
        acc = ("acc%d[j]" % n.nid) if self.col_axis else ("acc%d" % n.nid)
        arg = n.args[0]
        if (ref is not None and n.op == "sum" and not self.fused_sum(n) and arg.kind == "E"
                and arg.op in ("sqr", "mul") and FMA_IN_SUMS):
            # sum of products: multiply-add with one rounding per term (the
            # sum's order already differs from the CPU's; this only makes each
            # term a little more accurate)
            a, b = (arg.args[0], arg.args[0]) if arg.op == "sqr" else arg.args
            self.L("%s = __builtin_fmaf(%s, %s, %s);" % (acc, ref(a), ref(b), acc))
            return
        if self.fused_max(n):
            self.L("%s::step(%s, %s);" % (op, acc, val))
        elif n.is_index:
            self.L("%s::step(%s, %s, (int)(%s));" % (op, acc, val, index))
        else:
            self.L("%s = %s::f(%s, %s);" % (acc, op, acc, val))


# =====================================================================================
# family: row  (axis 1)
# =====================================================================================
MERGED_MOMENTS = os.environ.get("NEON_HIP_MERGED_MOMENTS", "1") != "0"
SHARED_FLOAT_JOIN = os.environ.get("NEON_HIP_FLOAT_JOIN", "1") != "0"   # 0: every lane joins its own columns' pieces


def _shifted_square_sum(n2, firsts):
    """``n2`` = sum(sqr(x - a)) along the reduced axis, with ``x`` free of reductions, ``a``
    constant along that axis and ``sum(x)`` among the first sweep's reductions
    ``firsts`` (the variance around a mean): (n2, sum(x), x, a), else None."""
    if n2.op != "sum" or n2.is_index or n2.lse_max is not None:
        return None
    e = n2.args[0]
    if e.kind != "E" or e.op != "sqr":
        return None
    d = e.args[0]
    if d.kind != "E" or d.op != "sub" or len(d.args) != 2:
        return None
    x, a = d.args
    along_x, along_a = (x.vc, a.vc) if n2.axis == 1 else (x.vr, a.vr)
    if not along_x or x.level != 0 or along_a or a.level > 1 or a.kind == "R" and a.is_index:
        return None
    for r1 in firsts:
        if r1.op == "sum" and not r1.is_index and r1.args[0] is x:
            return (n2, r1, x, a)
    return None


BATCH_FENCE_TILES = int(os.environ.get("NEON_HIP_BATCH_FENCE", "16"))
# rows of more tiles than this: the tiles that are streamed in every sweep run as a loop, not unrolled
ROLLED_TAIL_FROM = int(os.environ.get("NEON_HIP_ROLLED_TAIL", "32"))


def gen_row(prog, V, LX, LY, NCH, stream=False, keep_words=None, chunks=1, tail=False, park_bytes=0,
            max_vals=0):
    """Axis-1 reductions.  A team of LX lanes (a power of two up to 64, or the
    whole workgroup) owns one row; the workgroup holds LY rows.  A lane visits
    column tiles tx, tx+LX, ...; with ``NCH`` > 0 that loop has a fixed trip
    count and the tiles loaded in the first sweep stay in registers for the
    later ones; with ``NCH`` == 0 every sweep streams the row again.

    ``keep_words`` (with ``NCH`` > 0) limits the 32-bit registers per lane that
    resident tiles may take: operands are made resident in order of first use
    while they fit, the others are fetched again, a few tiles at a time, in
    every sweep that reads them (batch-norm backward keeps ``x`` and re-reads
    the deltas: four passes over HBM instead of five).

    ``park_bytes`` (whole-workgroup rows): LDS the workgroup may use as a second
    tier of residence.  An operand that found no registers for all of its tiles
    and is read by more than one sweep leaves the first tiles it fetched in its
    first sweep there -- every lane its own, 16 bytes apart from its
    neighbour's, no barrier needed --, holds the next ones in whatever registers
    are left, and later sweeps take both back instead of going to memory; only
    tiles beyond that are fetched again.

    ``max_vals`` (with ``NCH`` > 0): how many expensive elementwise results
    that two sweeps need may be kept in float32 registers of their own, NCH*V
    words each (softmax over 16-bit rows: exp(x - max) once per element).

    ``chunks`` > 1 (family ``rowcoop``; whole-workgroup rows with ``NCH`` > 0
    only): few, very long rows.  grid = (rows, chunks); workgroup (r, q) owns
    tiles q*NCH ... q*NCH+NCH-1 of row r, and the ``chunks`` workgroups of a row
    -- all resident at once, the planner keeps the grid within one workgroup
    per compute unit -- exchange their partial results after every sweep
    through device-coherent memory: publish, count arrivals on the row's
    counter, wait (bounded), gather and fold.  Extra parameters: workspace
    pointer and the byte offset of the counters (two per row: arrivals,
    departures; zero before the first launch, reset by the last workgroup to
    leave).

    ``tail``: the row length is not a multiple of V; the last tile of a row is
    loaded and stored element by element and only its valid elements enter
    the reductions."""
    g = _RedGen(prog, V, stream, "row")
    L = g.L
    T = LX * LY
    assert LX <= 64 or LY == 1
    resident = NCH > 0
    coop = chunks > 1
    assert not coop or (resident and LY == 1 and T % 64 == 0 and chunks <= T)
    words_left = [keep_words]       # None: everything is kept
    transient = set()               # nids of row operands that are not kept
    park_left = [int(park_bytes) if (LY == 1 and NCH > 0) else 0]
    park = {}                       # nid of a transient operand -> tiles it parks in LDS
    hold = {}                       # ... -> tiles (the next ones) it holds in registers left over
    parked = set()                  # ... whose parked / held tiles have been filled by now
    params, fmt = g.param_list([("char* ws", "P"), ("long long ctr_offset", "q")] if coop else [])
    head = ('extern "C" __global__ __launch_bounds__(%d) void @NAME@(%s)\n' % (T, params))
    per_level = _levels(prog)
    nsweeps = prog.nlevels
    full_out = [st for st in prog.statements if st.out.shape[1] > 1 or g.C == 1]
    line_out = [st for st in prog.statements if st not in full_out]
    done = {}      # nid -> node of reductions already finished
    cached = {}    # leaf nid -> resident tile array name

    L.open("")
    if LX > 64:
        L("__shared__ float s_f[%d];" % (T // 64))
        L("__shared__ nh_pair s_p[%d];" % (T // 64))
    L("const int tx = threadIdx.x %% %d, ty = threadIdx.x / %d;" % (LX, LX))
    g.declare_one()
    L("const long long r = (long long)blockIdx.x * %d + ty;" % LY)
    L("const bool row_ok = r < R;")
    L("const long long rr = row_ok ? r : 0;")   # address clamp for idle teams
    if not resident:
        L("const int nch = (C + %d - 1) / %d;" % (LX * V, LX * V))
    all_reds = g.own_reductions([n for lv in sorted(per_level) for n in per_level[lv]])
    red_slot = dict((n.nid, k) for k, n in enumerate(all_reds))
    exchanges = [0]
    # Exchanges of plain float partials carry a tag in the pair's unused index word: a workgroup's
    # (value, tag) is ONE 8-byte atomic store, so whoever sees the tag has the value -- no wait for the
    # store's acknowledgement, no counter, no separate fetch.  The tag is the one the workgroup's own
    # slot held at kernel start plus one: every launch writes every slot exactly once, so all slots of
    # a plan carry the same tag between launches (the plan's workspace starts zeroed), and nothing has
    # to be re-armed at the end.  One round trip instead of three.
    tagged = bool(coop and TAGGED_EXCHANGE and all_reds and not any(g.is_pair(n) for n in all_reds)
                  and chunks <= 64 and len(all_reds) <= 8)
    if coop:
        L("__shared__ int s_abort;")
        # (the counters of neighbouring lines a cache line apart, see TICKET_STRIDE_WORDS)
        L("unsigned int* ctr = reinterpret_cast<unsigned int*>(ws + ctr_offset) + %d * blockIdx.x;" % TICKET_STRIDE_WORDS)
        L("unsigned int* status = reinterpret_cast<unsigned int*>(ws + ctr_offset) + %d * gridDim.x;" % TICKET_STRIDE_WORDS)
        L("nh_pair* part = reinterpret_cast<nh_pair*>(ws) + (long long)blockIdx.x * %d;" % (len(all_reds) * chunks))
    if tagged:
        L("__shared__ float s_x[8];")
        L("int tag = 0;")
        L("if (threadIdx.x < 64) tag = nh_part_load(&part[blockIdx.y]).i + 1;     // (in flight while the row is fetched)")
        L("if (threadIdx.x == 0) s_abort = 0;     // (the workgroup meets at a barrier before it is read)")

    SU = 4      # column tiles in flight per lane when the row is streamed
    NCHP = -(-NCH // SU) * SU

    # A whole workgroup per row: row and tile number are the same for every lane.  Used where
    # registers are short (not every operand resident): the compiler then recomputes tile
    # addresses from the scalar base instead of keeping a 64-bit address per tile and operand
    # alive across the sweeps (the long-row batch-norm kernels spilled 40 to 115 registers
    # without it).  Where everything is resident the kept addresses are the cheaper form
    # (fp16 row normalisation: 17.0 us against 17.9 us).
    g.split_columns = LX > 64 and keep_words is not None

    def chunk_position(k):
        if coop:
            # (batch loops may run k past NCH: those tiles belong to the next workgroup)
            L("const long long cu = ((long long)blockIdx.y * %d + (%s)) * %d;" % (NCH, k, LX * V))
            L("const unsigned int cl = (unsigned int)tx * %du;" % V)
            L("const long long c = cu + cl;")
            L("const bool ok = row_ok && (c < C) && ((%s) < %d);" % (k, NCH))
        elif g.split_columns:
            L("const long long cu = (long long)(%s) * %d;" % (k, LX * V))
            L("const unsigned int cl = (unsigned int)tx * %du;" % V)
            L("const long long c = cu + cl;")
            L("const bool ok = row_ok && (c < C);")
        else:
            L("const long long c = ((long long)(%s) * %d + tx) * %d;" % (k, LX, V))
            L("const bool ok = row_ok && (c < C);")
        if tail:
            L("const bool full = c + %d <= C;" % V)
            L("const int lim = full ? %d : (int)(C - c);" % V)

    def tile_load(name, n):
        addr = g.tile_addr(n, "rr", "c")
        if tail and g.tile_width(n, V) > 1:
            return ("if (ok && full) %s.%s(%s); else if (ok) %s.load_partial(%s, lim); else %s.zero();"
                    % (name, g.ld, addr, name, addr, name))
        return "if (ok) %s.%s(%s); else %s.zero();" % (name, g.ld, addr, name)

    def exchange(reds, riders=()):
        """join the workgroups of a row: red<id> of every reduction of this
        sweep becomes the result over the whole row, in every lane of every
        workgroup.  ``riders``: reductions whose per-workgroup values travel
        along and are only fetched (g<id>), for the caller to combine"""
        exchanges[0] += 1
        if tagged:
            both = list(reds) + list(riders)
            L.open("if (threadIdx.x == 0)")
            for n in both:
                L("nh_part_store(&part[%d + blockIdx.y], nh_pair{red%d, tag});" % (red_slot[n.nid] * chunks, n.nid))
            L.close()
            for n in both:
                L("nh_pair g%d = nh_pair{%s::init(), 0};" % (n.nid, g.red_op(n)))
            L.open("if (threadIdx.x < %d)" % chunks)
            L("unsigned int spins = 0;")
            L.open("for (;;)")
            for n in both:
                L("g%d = nh_part_load(&part[%d + threadIdx.x]);" % (n.nid, red_slot[n.nid] * chunks))
            L("if (%s) break;" % " && ".join("g%d.i == tag" % n.nid for n in both))
            L("__builtin_amdgcn_s_sleep(2);")
            L("if (++spins > NH_SPIN_LIMIT) { s_abort = 1; break; }")
            L.close()
            L.close()
            L.open("if (threadIdx.x < 64)")
            for k, n in enumerate(reds):
                L("const float w%d = nh_wave_allreduce<%s, 64, float>((threadIdx.x < %d) ? g%d.v : %s::init());"
                  % (n.nid, g.red_op(n), chunks, n.nid, g.red_op(n)))
                L("if (threadIdx.x == 0) s_x[%d] = w%d;" % (k, n.nid))
            L.close()
            L("__syncthreads();")
            L.open("if (s_abort)")
            L("// the other workgroups never showed up: leave word for the host and give up rather than hang")
            L("if (threadIdx.x == 0) __hip_atomic_store(status, NH_COOP_ABORTED, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);")
            L("return;")
            L.close()
            for k, n in enumerate(reds):
                L("red%d = s_x[%d];" % (n.nid, k))
            L("__syncthreads();     // s_x is free again")
            return
        L.open("if (threadIdx.x == 0)")
        for n in list(reds) + list(riders):
            val = ("red%d" % n.nid) if g.is_pair(n) else ("nh_pair{red%d, 0}" % n.nid)
            L("nh_part_store(&part[%d + blockIdx.y], %s);" % (red_slot[n.nid] * chunks, val))
        L.close()
        L("nh_publish_barrier();     // the partial stores have been performed")
        L.open("if (threadIdx.x == 0)")
        L("nh_ticket_take(ctr);")
        L("unsigned int spins = 0; int bad = 0;")
        L.open("while (nh_arrivals(ctr) < %du)" % (chunks * exchanges[0]))
        L("__builtin_amdgcn_s_sleep(4);")
        L("if (++spins > NH_SPIN_LIMIT) { bad = 1; break; }")
        L.close()
        L("s_abort = bad;")
        L.close()
        L("__syncthreads();")
        L.open("if (s_abort)")
        L("// the other workgroups never showed up: leave word for the host and give up rather than hang")
        L("if (threadIdx.x == 0) __hip_atomic_store(status, NH_COOP_ABORTED, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);")
        L("return;")
        L.close()
        for n in list(reds) + list(riders):
            op = g.red_op(n)
            init = ("%s::init()" % op) if g.is_pair(n) else ("nh_pair{%s::init(), 0}" % op)
            L("const nh_pair g%d = (threadIdx.x < %d) ? nh_part_load(&part[%d + threadIdx.x]) : %s;"
              % (n.nid, chunks, red_slot[n.nid] * chunks, init))
        for n in reds:
            op = g.red_op(n)
            if g.is_pair(n):
                L("red%d = nh_block_allreduce<%s, %d, nh_pair>(g%d, s_p);" % (n.nid, op, T // 64, n.nid))
            else:
                L("red%d = nh_block_allreduce<%s, %d, float>(g%d.v, s_f);" % (n.nid, op, T // 64, n.nid))

    def sweep(leaves, emit_body):
        """Loop over the lane's column tiles.  All loads of a batch of tiles
        are issued before the first use (a load directly followed by its use
        would serialise the round trips): resident rows are fetched by a loop
        of their own ahead of the first sweep, streamed rows SU tiles at a
        time.  ``emit_body(tiles)`` writes the per-tile work; ``k``, ``c`` and
        ``ok`` are in scope."""
        moving = [n for n in leaves if varies_in_loop(n)]
        tiles = dict((n.nid, line_tiles[n.nid]) for n in leaves if not varies_in_loop(n))
        if resident:
            fresh = [n for n in moving if n.nid not in cached and n.nid not in transient]
            if fresh:
                L("#pragma unroll")
                L.open("for (int k = 0; k < %d; ++k)" % NCH)
                chunk_position("k")
                for n in fresh:
                    cached[n.nid] = "keep%d" % n.nid
                    L(tile_load("keep%d[k]" % n.nid, n))
                L.close()
            passing = [n for n in moving if n.nid in transient]
            for n in moving:
                if n.nid not in transient:
                    tiles[n.nid] = "%s[k]" % cached[n.nid]
            if not passing:
                L("#pragma unroll")
                L.open("for (int k = 0; k < %d; ++k)" % NCH)
                chunk_position("k")
                emit_body(tiles)
                L.close()
                return
            # kept tiles come from registers, the others SU tiles at a time
            def batches(lo, hi, unrolled):
                """tiles lo ... hi-1, SU at a time; ``unrolled``: k is a compile-time number
                (needed to address registers and LDS slots by tile)"""
                L("#pragma unroll" if unrolled else "#pragma unroll 1")
                L.open("for (int kb = %d; kb < %d; kb += %d)" % (lo, hi, SU))
                for n in passing:
                    L("%s %s[%d];" % (g.tile_type(n, V), g.tile_name(n, "_s"), SU))
                    tiles[n.nid] = "%s[u]" % g.tile_name(n, "_s")
                L("#pragma unroll")
                L.open("for (int u = 0; u < %d; ++u)" % SU)
                L("const int k = kb + u;")
                chunk_position("k")         # k beyond the row: c >= C, so ok is false
                for n in passing:
                    name = "%s[u]" % g.tile_name(n, "_s")
                    pk, hk = park.get(n.nid, 0), hold.get(n.nid, 0)
                    if n.nid in parked and unrolled:
                        L("if (k < %d) %s = park%d[k][threadIdx.x];" % (pk, name, n.nid))
                        if hk:
                            L("else if (k < %d) %s = hold%d[k - %d];" % (pk + hk, name, n.nid, pk))
                        L("else { %s }" % tile_load(name, n))
                    else:
                        L(tile_load(name, n))
                L.close()
                L("#pragma unroll")
                L.open("for (int u = 0; u < %d; ++u)" % SU)
                L("const int k = kb + u;")
                chunk_position("k")
                # (after the batch's loads have all been issued: a store into LDS waits for its tile)
                for n in passing:
                    if n.nid not in parked and n.nid in park and unrolled:
                        name, pk, hk = "%s[u]" % g.tile_name(n, "_s"), park[n.nid], hold.get(n.nid, 0)
                        L("if (k < %d) park%d[k][threadIdx.x] = %s;" % (pk, n.nid, name))
                        if hk:
                            L("else if (k < %d) hold%d[k - %d] = %s;" % (pk + hk, n.nid, pk, name))
                emit_body(tiles)
                L.close()
                if NCH > BATCH_FENCE_TILES and unrolled:
                    # long rows: without this the scheduler starts the loads of every batch of
                    # the unrolled loop at once and spills what they bring
                    L("__builtin_amdgcn_sched_barrier(0);")
                L.close()

            # Tiles beyond what LDS and registers hold are only ever streamed: where nothing
            # else is addressed by tile number they run as a loop proper (64 tiles unrolled
            # three times over made a kernel that spilled 224 registers).
            split_at = NCH
            if len(passing) == len(moving) and NCH > ROLLED_TAIL_FROM and not max_vals:
                kept_tiles = max(park.get(n.nid, 0) + hold.get(n.nid, 0) for n in passing)
                split_at = min(NCH, -(-kept_tiles // SU) * SU)
            if split_at:
                batches(0, split_at, True)
            if split_at < NCH:
                batches(split_at, NCH, False)
            parked.update(n.nid for n in passing if n.nid in park)
            return
        L.open("for (int kb = 0; kb < nch; kb += %d)" % SU)
        for n in moving:
            L("%s %s[%d];" % (g.tile_type(n, V), g.tile_name(n, "_s"), SU))
            tiles[n.nid] = "%s[u]" % g.tile_name(n, "_s")
        L("#pragma unroll")
        L.open("for (int u = 0; u < %d; ++u)" % SU)
        chunk_position("kb + u")
        for n in moving:
            L(tile_load("%s[u]" % g.tile_name(n, "_s"), n))
        L.close()
        L("#pragma unroll")
        L.open("for (int u = 0; u < %d; ++u)" % SU)
        chunk_position("kb + u")
        emit_body(tiles)
        L.close()
        L.close()

    line_tiles = {}   # leaf nid -> tile that does not change along the row

    def varies_in_loop(n):
        return g.tile_width(n, 2) == 2      # tile spans columns

    # how many sweeps (the final, storing one included) read each operand
    sweeps_reading = {}
    if park_left[0]:
        earlier = set()
        rounds = [g.own_reductions(per_level.get(s_, [])) for s_ in range(nsweeps)]
        for reds_ in rounds:
            if reds_:
                for leaf in g.leaf_nodes(_needed([n.args[0] for n in reds_], earlier)):
                    sweeps_reading[leaf.nid] = sweeps_reading.get(leaf.nid, 0) + 1
                earlier.update(n.nid for n in reds_)
        if full_out:
            for leaf in g.leaf_nodes(_needed([st.root for st in full_out], earlier)):
                sweeps_reading[leaf.nid] = sweeps_reading.get(leaf.nid, 0) + 1

    def declare_tiles(leaves):
        """function-scope declarations needed before a sweep's loop"""
        for n in leaves:
            if not varies_in_loop(n):
                if n.nid not in line_tiles:
                    name = "line%d" % n.nid
                    line_tiles[n.nid] = name
                    L("%s %s;" % (g.tile_type(n, V), name))
                    L("%s.load(%s);" % (name, g.tile_addr(n, "rr", "0")))
            elif resident and n.nid not in cached and n.nid not in transient:
                need = NCH * max(1, (g.tile_width(n, V) * prog.tensors[n.slot].dtype.itemsize + 3) // 4)
                if words_left[0] is not None and need > words_left[0]:
                    transient.add(n.nid)
                    tile_words = max(1, (g.tile_width(n, V) * prog.tensors[n.slot].dtype.itemsize + 3) // 4)
                    fit = min(NCH, park_left[0] // (4 * T * tile_words))
                    if fit > 0 and sweeps_reading.get(n.nid, 0) > 1:
                        park[n.nid] = fit
                        park_left[0] -= fit * 4 * T * tile_words
                        L("__shared__ __attribute__((aligned(16))) %s park%d[%d][%d];" % (g.tile_type(n, V), n.nid, fit, T))
                        more = min(NCH - fit, words_left[0] // tile_words)
                        if more > 0:
                            hold[n.nid] = more
                            words_left[0] -= more * tile_words
                            L("%s hold%d[%d];" % (g.tile_type(n, V), n.nid, more))
                    continue
                if words_left[0] is not None:
                    words_left[0] -= need
                # (rounded up to whole batches so that batch loops index within bounds)
                L("%s keep%d[%d];" % (g.tile_type(n, V), n.nid, NCHP))
        if resident:
            for nid, name in cached.items():
                L("#pragma unroll")
                L("for (int k = 0; k < %d; ++k) %s[k].keep();" % (NCH, name))
            for nid in sorted(parked):
                if nid in hold:
                    L("#pragma unroll")
                    L("for (int k = 0; k < %d; ++k) hold%d[k].keep();" % (hold[nid], nid))

    # operands that do not change along the row are fetched once, up front, so
    # their latency overlaps the first sweep
    declare_tiles([n for n in g.leaf_nodes(used_nodes([st.root for st in prog.statements]))
                   if not varies_in_loop(n)])

    # expensive values that later sweeps need again take over the registers of
    # a resident float32 operand nothing else reads afterwards
    over, vals, own = {}, {}, set()
    if resident:
        stages = [[n.args[0] for n in g.own_reductions(per_level.get(s, []))] for s in range(nsweeps)]
        stages = [t for t in stages if t]
        if full_out:
            stages.append([st.root for st in full_out])

        def one_word_per_element(leaf):
            return varies_in_loop(leaf) and DTYPE_CODE[prog.tensors[leaf.slot].dtype] == "f4"

        over = dict((n.nid, leaf) for n, leaf in _overwriting_values(prog, stages, one_word_per_element))
        if max_vals:
            by_nid = dict((n.nid, n) for n in prog.nodes)
            own = set(n.nid for n in _kept_values(prog, stages, max_vals, already=[by_nid[k] for k in over]))

    def stops():
        d = set(done)
        d.update(vals)
        return d

    # Variance around a mean over a row that several workgroups share: instead of a second
    # exchange for sum((x - a)^2), every workgroup takes the squares around the mean of ITS OWN
    # part (known without waiting), and the parts combine exactly afterwards:
    #   sum_i sum_{x in i} (x - a)^2 = sum_i [ M2_i + n_i (mean_i - a)^2 ],  M2_i = sum (x - mean_i)^2
    # -- one exchange for both sweeps, terms that are all non-negative, and the rounding of a
    # two-pass variance (the pairwise form of Chan, Golub and LeVeque).
    merged = []
    if coop and MERGED_MOMENTS and not over and not own and per_level.get(0) and per_level.get(1):
        merged = [_shifted_square_sum(n2, per_level[0]) for n2 in per_level[1]]
        if not all(merged):
            merged = []
    span = NCH * LX * V      # elements of a row that one workgroup owns
    # The same identity with the LANES of one workgroup as the parts, for rows that sit in
    # registers whole: every lane accumulates sum(x - s) and sum((x - s)^2) around a value s of
    # its own (the first element it holds) WHILE ITS TILES ARRIVE, in the sweep that adds up x;
    # once the row's sum is known a lane's share of sum((x - a)^2) is M2 + n (mean - a)^2 from
    # those two numbers, and the second pass over the registers -- a microsecond and a half
    # between the last load and the first store of a (256, 100352) fp16 normalisation, during
    # which the memory system idles -- is gone.  Rounding: that of a two-pass variance inside
    # every lane's share (its s is one of its own values), exact combination across lanes.
    # (the workgroups of a shared row take their OWN part's second moment the same way)
    coop_lane = []
    if (merged and resident and keep_words is None
            and all(m[2].kind == "T" and varies_in_loop(m[2]) for m in merged)):
        coop_lane = merged
    lane_merged = []
    if (not coop and MERGED_MOMENTS and resident and LX > 64 and keep_words is None and not over and not own
            and per_level.get(0) and per_level.get(1)):
        lane_merged = [_shifted_square_sum(n2, per_level[0]) for n2 in per_level[1]]
        if not all(lane_merged) or any(m[2].kind != "T" or not varies_in_loop(m[2]) for m in lane_merged):
            lane_merged = []

    def derived(x):
        # 16-bit operands (eight elements per load: the sweep is bound by instruction issue):
        # sum(x - s) is taken from the lane's plain sum, sum(x) - n s, instead of being added up
        # element by element.  What the subtraction cancels is bounded by what 11-bit inputs
        # can hold (|mean| / spread below 2^11, or the spread is quantisation noise anyway).
        return prog.tensors[x.slot].dtype.itemsize == 2

    def lane_share(n2, r1, x, about):
        """``term_`` = this lane's share of sum((x - about)^2) from what it gathered while its
        tiles arrived (sh: its reference value, sa: sum(x - sh), sb: sum((x - sh)^2), cnt):
        M2 + n (mean - about)^2; nothing for a lane without elements"""
        L("const float a_ = %s;" % about)
        if derived(x):
            L("sa%d = __builtin_fmaf(-cnt%d, sh%d, acc%d);" % (n2.nid, n2.nid, n2.nid, r1.nid))
        L("const float inv_ = (cnt%d > 0.0f) ? 1.0f / cnt%d : 0.0f;" % (n2.nid, n2.nid))
        L("const float mu_ = sa%d * inv_;" % n2.nid)
        L("const float m2_ = nh_max(sb%d - sa%d * mu_, 0.0f);" % (n2.nid, n2.nid))
        L("const float e_ = (sh%d + mu_) - a_;" % n2.nid)
        L("const float term_ = (cnt%d > 0.0f) ? __builtin_fmaf(cnt%d * e_, e_, m2_) : 0.0f;" % (n2.nid, n2.nid))

    def local_second_moments():
        """after the first sweep's fold inside the workgroup (red<sum> = this part's sum):
        red<n2> = sum over this part of (x - this part's mean)^2"""
        L("const long long left_ = (long long)C - (long long)blockIdx.y * %dll;" % span)
        L("const float n_loc = (float)(left_ < %dll ? left_ : %dll);" % (span, span))
        if coop_lane:
            # from what every lane gathered during the first sweep: no second pass over the registers
            for n2, r1, x, a in merged:
                L("float red%d;" % n2.nid)
                L.open("")
                lane_share(n2, r1, x, "red%d / n_loc" % r1.nid)
                L("red%d = nh_block_allreduce<nh_op_sum, %d, float>(term_, s_f);" % (n2.nid, T // 64))
                L.close()
            return
        for n2, r1, x, a in merged:
            L("const float mu%d = red%d / n_loc;" % (n2.nid, r1.nid))
            vals[a.nid] = "mu%d" % n2.nid
        seconds = [m[0] for m in merged]
        nodes = _needed([n.args[0] for n in seconds], stops())
        leaves = g.leaf_nodes(nodes)
        declare_tiles(leaves)
        for n in seconds:
            g.declare_acc(n)

        def body(tiles):
            L.open("if (ok)")
            if V > 1:
                L("#pragma unroll")
            L.open("for (int j = 0; j < %d; ++j)" % V)
            if tail:
                L.open("if (j < lim)")
            ref = g.make_ref("_s", "rr", "c", V, tiles, vals)
            g.emit_exprs(nodes, ref, stops())
            for n in seconds:
                g.accumulate(n, ref(n.args[0]), "c + j", ref)
            if tail:
                L.close()
            L.close()
            L.close()

        sweep(leaves, body)
        for n in seconds:
            L("float red%d = nh_block_allreduce<nh_op_sum, %d, float>(acc%d, s_f);" % (n.nid, T // 64, n.nid))
        for n2, r1, x, a in merged:
            del vals[a.nid]

    def combine_second_moments():
        """after the exchange (g<id> = the parts' sums and second moments, rv<sum> final)"""
        line_ref = g.make_ref("_s", "rr", "0", 1, dict((nid, name) for nid, name in line_tiles.items()), vals)
        for n2, r1, x, a in merged:
            L("float shift%d;" % n2.nid)
            L.open("")
            L("const int j = 0; (void)j;")
            g.emit_exprs(_needed([a], stops()), line_ref, stops())
            L("shift%d = %s;" % (n2.nid, line_ref(a)))
            L.close()
            L("float term%d = 0.0f;" % n2.nid)
            L.open("if (threadIdx.x < %d)" % chunks)
            L("const long long lq = (long long)C - (long long)threadIdx.x * %dll;" % span)
            L("const float nq = (float)(lq < %dll ? lq : %dll);" % (span, span))
            L("const float dq = g%d.v / nq - shift%d;" % (r1.nid, n2.nid))
            L("term%d = __builtin_fmaf(nq * dq, dq, g%d.v);" % (n2.nid, n2.nid))
            L.close()
            L("red%d = nh_block_allreduce<nh_op_sum, %d, float>(term%d, s_f);" % (n2.nid, T // 64, n2.nid))
            L("const float rv%d = red%d;" % (n2.nid, n2.nid))
            done[n2.nid] = n2

    for s in range(nsweeps):
        if (merged or lane_merged) and s == 1:
            continue            # done together with the first sweep
        reds = g.own_reductions(per_level.get(s, []))
        if not reds:
            continue
        args = [n.args[0] for n in reds]
        nodes = _needed(args, stops())
        leaves = g.leaf_nodes(nodes)
        declare_tiles(leaves)
        for n in reds:
            g.declare_acc(n)
        # (an operand that did not get registers cannot lend them)
        fresh = [n for n in nodes if n.nid in over and n.nid not in vals and over[n.nid].nid not in transient]
        fresh_own = [n for n in nodes if n.nid in own and n.nid not in vals and n.nid not in over]
        for n in fresh_own:
            L("float val%d[%d][%d];" % (n.nid, NCH, V))
        riding = (lane_merged or coop_lane) if s == 0 else []

        for n2, r1, x, a in riding:
            L("float sh%d = 0.0f, sa%d = 0.0f, sb%d = 0.0f, cnt%d = 0.0f;" % (n2.nid, n2.nid, n2.nid, n2.nid))

        def reduce_body(tiles, nodes=nodes, reds=reds, fresh=fresh, fresh_own=fresh_own, riding=riding):
            L.open("if (ok)")
            for n2, r1, x, a in riding:
                # the lane's own reference value: the first element it holds
                L("if (k == 0) sh%d = %s.get(0);" % (n2.nid, tiles[x.nid]))
                L("cnt%d += %s;" % (n2.nid, ("(float)lim" if tail else "%d.0f" % V)))
                if V > 1:
                    L("#pragma unroll")
                L.open("for (int j = 0; j < %d; ++j)" % V)
                if tail:
                    L.open("if (j < lim)")
                xv = "%s.get(j)" % tiles[x.nid]
                if g.is_half_leaf(x) and g.one_declared:
                    L("const float d_ = __builtin_fmaf(%s, nh_one, -sh%d);" % (xv, n2.nid))
                else:
                    L("const float d_ = %s - sh%d;" % (xv, n2.nid))
                if not derived(x):
                    L("sa%d += d_;" % n2.nid)
                L("sb%d = __builtin_fmaf(d_, d_, sb%d);" % (n2.nid, n2.nid))
                if tail:
                    L.close()
                L.close()
            # plain sums of a packed fp16 operand: two elements per instruction, straight
            # from the tile (a partial last tile is zero-filled, so it needs no guard)
            pairwise = [n for n in reds if n.op == "sum" and g.is_half_leaf(n.args[0]) and V % 2 == 0
                        and n.args[0].nid not in vals and g.tile_width(n.args[0], V) == V]
            for n in pairwise:
                L("acc%d = %s.sum_into(acc%d);" % (n.nid, tiles[n.args[0].nid], n.nid))
            reds = [n for n in reds if n not in pairwise]
            if not reds and not fresh and not fresh_own:
                L.close()
                return
            # a running (max, sum of exponentials) pair takes the tile's V values at once:
            # one rescaling of the sum per tile instead of one per element
            running = [n for n in reds if g.fused_max(n)]
            for n in running:
                L("float lv%d[%d];" % (n.nid, V))
                if tail:
                    L("#pragma unroll")
                    L("for (int j = 0; j < %d; ++j) lv%d[j] = -NH_INF;" % (V, n.nid))
            if V > 1:
                L("#pragma unroll")
            L.open("for (int j = 0; j < %d; ++j)" % V)
            if tail:
                L.open("if (j < lim)")
            ref = g.make_ref("_s", "rr", "c", V, tiles, vals)
            g.emit_exprs(nodes, ref, stops())
            for n in reds:
                if n in running:
                    L("lv%d[j] = %s;" % (n.nid, ref(n.args[0])))
                else:
                    g.accumulate(n, ref(n.args[0]), "c + j", ref)
            for n in fresh:
                L("keep%d[k].put(j, t%d);" % (over[n.nid].nid, n.nid))
            for n in fresh_own:
                L("val%d[k][j] = t%d;" % (n.nid, n.nid))
            if tail:
                L.close()
            L.close()
            for n in running:
                L("nh_op_lse::stepn<%d>(acc%d, lv%d);" % (V, n.nid, n.nid))
            L.close()

        sweep(leaves, reduce_body)
        for n in fresh:
            vals[n.nid] = "keep%d[k].get(j)" % over[n.nid].nid
        for n in fresh_own:
            vals[n.nid] = "val%d[k][j]" % n.nid
        for n in reds:
            op = g.red_op(n)
            ty_ = "nh_pair" if g.is_pair(n) else "float"
            const = "" if coop else "const "
            if LX <= 64:
                L("%s%s red%d = nh_wave_allreduce<%s, %d, %s>(acc%d);" % (const, ty_, n.nid, op, LX, ty_, n.nid))
            else:
                L("%s%s red%d = nh_block_allreduce<%s, %d, %s>(acc%d, %s);"
                  % (const, ty_, n.nid, op, T // 64, ty_, n.nid, "s_p" if g.is_pair(n) else "s_f"))
        if coop and merged and s == 0:
            local_second_moments()
            exchange(reds, riders=[m[0] for m in merged])
        elif coop:
            exchange(reds)
        for n in reds:
            if n.is_index:
                L("const int ri%d = red%d.i;" % (n.nid, n.nid))
            elif g.fused_max(n):
                L("const float rv%d = red%d.v;" % (n.nid, n.nid))
                L("const float rv%d = nh_lse_total(red%d);" % (n.lse_sum.nid, n.nid))
                done[n.lse_sum.nid] = n.lse_sum
            else:
                L("const float rv%d = red%d;" % (n.nid, n.nid))
            done[n.nid] = n
        if coop and merged and s == 0:
            combine_second_moments()
        if riding and not coop:
            line_ref = g.make_ref("_s", "rr", "0", 1, dict((nid, name) for nid, name in line_tiles.items()), vals)
            for n2, r1, x, a in riding:
                L("float rv%d;" % n2.nid)
                L.open("")
                L("const int j = 0; (void)j;")
                g.emit_exprs(_needed([a], stops()), line_ref, stops())
                lane_share(n2, r1, x, line_ref(a))
                L("rv%d = nh_block_allreduce<nh_op_sum, %d, float>(term_, s_f);" % (n2.nid, T // 64))
                L.close()
                done[n2.nid] = n2

    # outputs that have one value per row
    if line_out:
        roots = [st.root for st in line_out]
        nodes = _needed(roots, done)
        leaves = g.leaf_nodes(nodes)
        L.open("if (row_ok && tx == 0%s)" % (" && blockIdx.y == 0" if coop else ""))
        for n in leaves:
            g.emit_load(n, "r", "0", 1, "_l")
        L.open("")
        L("const int j = 0; (void)j;")
        ref = g.make_ref("_l", "r", "0", 1)
        g.emit_exprs(nodes, ref, done)
        for st in line_out:
            L("nh_out<%s, 1> o%d; o%d.clear();" % (g.slot_ctype(st.out), st.out.index, st.out.index))
            if st.root.kind == "R" and st.root.is_index:
                L("o%d.seti(0, ri%d);" % (st.out.index, st.root.nid))
            else:
                L("o%d.set(0, %s);" % (st.out.index, ref(st.root)))
            L("o%d.store(%s);" % (st.out.index, g.addr(st.out, "r", "0")))
        L.close()
        L.close()

    # outputs with the full shape: one more sweep
    if full_out:
        roots = [st.root for st in full_out]
        nodes = _needed(roots, stops())
        leaves = g.leaf_nodes(nodes)
        declare_tiles(leaves)

        # Results stored as 16-bit floats: root = atom * A + B with A, B constant along the row
        # (a chain of multiplications / divisions by per-row values and a last per-row addend)
        # is evaluated as ONE multiply-add per element, A and B once per row.
        collapsed = {}
        if AFFINE_16BIT_OUTPUTS:
            line_ref = g.make_ref("_s", "rr", "0", 1, dict((nid, name) for nid, name in line_tiles.items()), vals)
            for st in full_out:
                if DTYPE_CODE[st.out.dtype] not in ("f2", "b2") or st.root.kind != "E":
                    continue
                aff = _affine_in_line(st.root, lambda m: not m.vc)
                if aff is None:
                    continue
                atom, mults, addends = aff
                if not mults and not addends:
                    continue
                consts = _needed([m for _, m in mults] + [m for _, m in addends], stops())
                L("float fa%d = 1.0f, fb%d = 0.0f;" % (st.out.index, st.out.index))
                L.open("")
                L("const int j = 0; (void)j;")
                g.emit_exprs(consts, line_ref, stops())
                for kind, m in mults:
                    L("fa%d = fa%d %s %s;" % (st.out.index, st.out.index, "*" if kind == "mul" else "/", line_ref(m)))
                for kind, m in addends:
                    L("fb%d = fb%d %s %s;" % (st.out.index, st.out.index, "+" if kind == "add" else "-", line_ref(m)))
                L.close()
                collapsed[st.out.index] = atom
            if collapsed:
                nodes = _needed([collapsed.get(st.out.index, st.root) for st in full_out], stops())
                leaves = g.leaf_nodes(nodes)

        def store_body(tiles):
            L.open("if (ok)")
            for st in full_out:
                L("nh_out<%s, %d> o%d; o%d.clear();" % (g.slot_ctype(st.out), V, st.out.index, st.out.index))
            if V > 1:
                L("#pragma unroll")
            L.open("for (int j = 0; j < %d; ++j)" % V)
            ref = g.make_ref("_s", "rr", "c", V, tiles, vals)
            g.emit_exprs(nodes, ref, stops())
            for st in full_out:
                if st.root.kind == "R" and st.root.is_index:
                    L("o%d.seti(j, ri%d);" % (st.out.index, st.root.nid))
                elif st.out.index in collapsed:
                    L("o%d.set(j, __builtin_fmaf(%s, fa%d, fb%d));"
                      % (st.out.index, ref(collapsed[st.out.index]), st.out.index, st.out.index))
                else:
                    L("o%d.set(j, %s);" % (st.out.index, ref(st.root)))
            L.close()
            for st in full_out:
                if tail:
                    L("if (full) o%d.%s(%s); else o%d.store_partial(%s, lim);"
                      % (st.out.index, g.st, g.addr(st.out, "r", "c"), st.out.index, g.addr(st.out, "r", "c")))
                else:
                    L("o%d.%s(%s);" % (st.out.index, g.st, g.addr(st.out, "r", "c")))
            L.close()

        sweep(leaves, store_body)
    if coop and not tagged:
        # the last workgroup of the row to get here has seen everyone pass the
        # final wait: it re-arms both counters for the next launch
        L.open("if (threadIdx.x == 0)")
        L("const unsigned int t = __hip_atomic_fetch_add(ctr + 1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);")
        L.open("if (t == %du)" % (chunks - 1))
        L("__hip_atomic_store(ctr, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);")
        L("__hip_atomic_store(ctr + 1, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);")
        L.close()
        L.close()
    L.close()
    return _finish("rowcoop" if coop else "row", g, head, fmt, T, 0,
                   dict(V=V, LX=LX, LY=LY, NCH=NCH, stream=bool(stream), passing=len(transient),
                        over=len([k for k in vals if k in over]), kept=len([k for k in vals if k in own]), chunks=chunks, NRED=len(all_reds), tail=bool(tail),
                        parked=sum(park.values()), held=sum(hold.values()), lane_moments=len(lane_merged),
                        tagged=tagged))


# =====================================================================================
# families: col / colsplit  (axis 0)
# =====================================================================================
def _emit_col_fold(g, L, n, LX, LY, T, V, src, dst_decl=True):
    """Join the row-lanes of every column of the workgroup.  ``src`` is the
    per-lane accumulator array; afterwards every lane holds the result in
    rv<id>[] / ri<id>[].  Lanes of one wave that share a column tile are
    folded with lane-xor exchanges first; LDS then joins the wave groups in
    row order."""
    op = g.red_op(n)
    pair = g.is_pair(n)
    VK = V            # values a lane contributes to the LDS stage
    assert T > 64, "workgroups of the column families span several waves"
    if LX < 64:
        # the wave's row-lanes are folded with lane exchanges that split the V
        # values among the lanes; LDS collects the pieces
        steps = (64 // LX).bit_length() - 1
        VK = max(1, V >> steps)
        WY = T // 64
        wy = "(threadIdx.x >> 6)"
        writer = "((threadIdx.x & 63) < %d)" % (LX * (V // VK))
    else:
        WY = LY
        wy = "ty"
        writer = "true"
    if dst_decl:
        if n.is_index:
            L("int ri%d[%d];" % (n.nid, V))
        else:
            L("float rv%d[%d];" % (n.nid, V))
        if g.fused_max(n):
            L("float rv%d[%d];" % (n.lse_sum.nid, V))
    buf = "s_p" if pair else "s_f"

    def unpack():
        L("#pragma unroll")
        if n.is_index:
            L("for (int j = 0; j < %d; ++j) ri%d[j] = %s[j].i;" % (V, n.nid, src))
        elif g.fused_max(n):
            L("for (int j = 0; j < %d; ++j) { rv%d[j] = %s[j].v; rv%d[j] = nh_lse_total(%s[j]); }"
              % (V, n.nid, src, n.lse_sum.nid, src))
        else:
            L("for (int j = 0; j < %d; ++j) rv%d[j] = %s[j];" % (V, n.nid, src))

    if WY == 1:
        unpack()
        return
    if LX < 64:
        L.open("")
        L("const int j0 = nh_col_wave_fold<%s, %d, %d>(%s);" % (op, V, LX, src))
        L.open("if (%s)" % writer)
        L("#pragma unroll")
        L("for (int j = 0; j < %d; ++j) %s[%s][tx * %d + j0 + j] = %s[j];" % (VK, buf, wy, V, src))
        L.close()
        L.close()
    else:
        L.open("if (%s)" % writer)
        L("#pragma unroll")
        L("for (int j = 0; j < %d; ++j) %s[%s][tx * %d + j] = %s[j];" % (V, buf, wy, V, src))
        L.close()
    L("__syncthreads();")
    S = LX * V
    if S <= T and (pair or SHARED_FLOAT_JOIN):
        # Instead of every lane joining all V columns of its tile over all wave groups, P
        # adjacent lanes share ONE column, each takes every P-th group, a DPP all-reduce
        # over the P lanes finishes, and the results go round through LDS.  (value, index)
        # and (max, sum) pairs cost ten to twenty instructions to combine; for plain values
        # it is the LDS traffic that counts -- 16 waves x 4 values read by each of 1024
        # lanes took a fifth of a softmax over (1000,4096): 9.4 -> 8.6 us, fp16 9.6 -> 7.9 us
        P = 1
        while P * 2 <= min(T // S, 64) and P < WY:
            P *= 2
        L.open("")
        L("const int fcol = threadIdx.x / %d, fk = threadIdx.x %% %d;" % (P, P))
        L("%s one = %s::init();" % ("nh_pair" if pair else "float", op))
        L.open("if (fcol < %d)" % S)
        L("for (int y = fk; y < %d; y += %d) one = %s::f(one, %s[y][fcol]);" % (WY, P, op, buf))
        L.close()
        if P > 1:
            L("one = nh_wave_allreduce<%s, %d, %s>(one);" % (op, P, "nh_pair" if pair else "float"))
        L("__syncthreads();     // every piece has been read: the first row of the buffer takes the results")
        L("if (fk == 0 && fcol < %d) %s[0][fcol] = one;" % (S, buf))
        L.close()
        L("__syncthreads();")
        L("#pragma unroll")
        L("for (int j = 0; j < %d; ++j) %s[j] = %s[0][tx * %d + j];" % (V, src, buf, V))
        unpack()
        L("__syncthreads();")
        return
    # a lane's V partials of one wave group are adjacent and 16-byte aligned:
    # walking the groups in the outer loop lets them come in as one LDS read
    L("#pragma unroll")
    L("for (int j = 0; j < %d; ++j) %s[j] = %s[0][tx * %d + j];" % (V, src, buf, V))
    # (at most 32 LDS reads in flight: unrolled as a whole, the 15 x 8 reads of a 1024-lane
    # workgroup with 8 values per lane were all issued ahead of the first addition and took
    # the kernel from 56 to over 200 registers -- spilled, three times slower)
    L("#pragma unroll %d" % max(1, 32 // V) if (WY - 1) * V > 32 else "#pragma unroll")
    L.open("for (int y = 1; y < %d; ++y)" % WY)
    L("#pragma unroll")
    L("for (int j = 0; j < %d; ++j) %s[j] = %s::f(%s[j], %s[y][tx * %d + j]);" % (V, src, op, src, buf, V))
    L.close()
    unpack()
    L("__syncthreads();")


def _col_lds(L, LX, LY, T, V, any_index):
    WY = (T // 64) if LX < 64 else LY
    pitch = -(-(LX * V) // 4) * 4       # rows stay 16-byte aligned
    L("__shared__ __attribute__((aligned(16))) float s_f[%d][%d];" % (WY, pitch))
    if any_index:
        L("__shared__ __attribute__((aligned(16))) nh_pair s_p[%d][%d];" % (WY, pitch))
    return WY * pitch * (4 + (8 if any_index else 0))


def gen_col(prog, V, LX, LY, NR, stream=False, chunks=1, max_vals=0, tail=False, runs=False):
    """Axis-0 reductions with the rows resident in registers (LX column-lanes x
    LY row-lanes per workgroup, NR rows per lane).

    ``chunks`` == 1: one workgroup owns a column strip and all its rows.

    ``chunks`` > 1 (family ``colcoop``): the rows of a strip are spread over
    ``chunks`` workgroups that are all resident at once (the planner keeps the
    grid within one workgroup per compute unit).  After every sweep they
    exchange their partial results through device-coherent memory: publish,
    count arrivals on a per-strip counter, wait (bounded) for the others,
    gather and fold.  The matrix is still read from HBM exactly once however
    many sweeps the tree needs.  Extra parameters: workspace pointer and the
    byte offset of the counters (two per strip: arrivals, departures; zero
    before the first launch, reset by the last workgroup to leave)."""
    coop = chunks > 1
    g = _RedGen(prog, V, stream, "col")
    g.col_tail = bool(tail)     # C is not a multiple of V: the last column tile is loaded and stored
    #                             element by element; its surplus columns compute on zeros and are dropped
    L = g.L
    T = LX * LY
    params, fmt = g.param_list([("char* ws", "P"), ("long long ctr_offset", "q")] if coop else [])
    head = ('extern "C" __global__ __launch_bounds__(%d) void @NAME@(%s)\n' % (T, params))
    per_level = _levels(prog)
    nsweeps = prog.nlevels
    full_out = [st for st in prog.statements if st.out.shape[0] > 1 or g.R == 1]
    line_out = [st for st in prog.statements if st not in full_out]
    any_index = any(g.is_pair(n) for n in prog.nodes if n.kind == "R")
    done, cached = {}, {}

    L.open("")
    lds = _col_lds(L, LX, LY, T, V, any_index or coop)
    g.declare_one()
    L("const int tx = threadIdx.x %% %d, ty = threadIdx.x / %d;" % (LX, LX))
    wide = [t.dtype.itemsize for t in prog.tensors if t.shape[1] > 1]
    xcd_runs = bool(not coop and wide and (runs or LX * V * max(wide) < 128))
    if xcd_runs:
        # Strips narrower than a cache line: neighbouring strips read the same lines.  Workgroups
        # are handed to the 8 XCDs (each with its own L2) round-robin, so consecutive strips
        # would each pull those lines into a different L2.  Every XCD gets a contiguous run of
        # strips instead, and a run is whole 128-byte lines: with fewer strips than that needs,
        # fewer XCDs take part and the grid carries workgroups that leave at once (col_grid;
        # softmax over (1000,128), memory traffic over the matrix's bytes: 5.1 with strips dealt
        # round-robin, 1.6 with runs of half a line, 1.0 with whole lines on 4 of the 8 XCDs).
        # ``runs``: the same for strips of whole lines when the rows are not a multiple of 128
        # bytes long -- every second row piece then straddles two lines and shares each with
        # the neighbouring strip (softmax down (1000,30000) fp32 read 1.5 times its bytes).
        L("const unsigned int nstrips = (unsigned int)((C + %d) / %d);" % (LX * V - 1, LX * V))
        L("unsigned int nx = nstrips / %du;" % max(1, 128 // (LX * V * max(wide))))
        L("nx = nx < 1u ? 1u : (nx > NH_XCDS ? NH_XCDS : nx);")
        L("const unsigned int per_xcd = (nstrips + nx - 1u) / nx;")
        L("if (blockIdx.x % NH_XCDS >= nx || blockIdx.x / NH_XCDS >= per_xcd) return;")
        L("const unsigned int strip = (blockIdx.x % NH_XCDS) * per_xcd + blockIdx.x / NH_XCDS;")
        L("if (strip >= nstrips) return;")
    else:
        L("const unsigned int strip = blockIdx.x;")
    L("const long long c = ((long long)strip * %d + tx) * %d;" % (LX, V))
    L("const bool col_ok = c < C;")
    L("const long long cc = col_ok ? c : 0;")
    if tail:
        L("const bool cfull = c + %d <= C;" % V)
        L("const int clim = cfull ? %d : (col_ok ? (int)(C - c) : 0);" % V)
    if coop:
        L("__shared__ int s_abort;")
        # (the counters of neighbouring lines a cache line apart, see TICKET_STRIDE_WORDS)
        L("unsigned int* ctr = reinterpret_cast<unsigned int*>(ws + ctr_offset) + %d * blockIdx.x;" % TICKET_STRIDE_WORDS)
        L("unsigned int* status = reinterpret_cast<unsigned int*>(ws + ctr_offset) + %d * gridDim.x;" % TICKET_STRIDE_WORDS)
    all_reds = g.own_reductions([n for lv in sorted(per_level) for n in per_level[lv]])
    red_slot = dict((n.nid, k) for k, n in enumerate(all_reds))
    exchanges = [0]

    def row_loop_open():
        L("#pragma unroll")
        L.open("for (int i = 0; i < %d; ++i)" % NR)
        if coop:
            L("const long long r = ((long long)blockIdx.y * %d + i) * %d + ty;" % (NR, LY))
            L("const bool ok = col_ok && (r < R);")
        else:
            # Only a lane's last row can lie past the end (the planner takes NR = ceil(R / LY)), so
            # after unrolling the other rows carry no test and no branch.  Lanes past the last column
            # compute on the first columns' values (cc) and are kept from storing.  Measured, softmax
            # down the columns: (64,1048576) fp32 93 -> 88 us, (512,65536) 55 -> 52 us.
            L("const long long r = (long long)i * %d + ty;" % LY)
            L("const bool ok = (i < %d) || (r < R);" % (NR - 1))

    def exchange(reds, last_one_folds=False, riders=()):
        """fold the workgroups of a strip: afterwards acc/rv/ri hold the
        result over all rows in every lane of every workgroup.  ``riders``:
        reductions whose per-workgroup values travel along and are only
        fetched (q<id>[][]), for the caller to combine.

        ``last_one_folds``: nothing but one value per column remains to be
        written, so nobody waits: the workgroup whose arrival completes the
        count gathers, folds and goes on alone, the others are done."""
        exchanges[0] += 1
        for n in list(reds) + list(riders):
            L("nh_pair* part%d = reinterpret_cast<nh_pair*>(ws) + (long long)%d * C;"
              % (n.nid, red_slot[n.nid] * chunks))
        L.open("if (col_ok && ty == 0)")
        L("#pragma unroll")
        L.open("for (int j = 0; j < %d; ++j)" % V)
        if tail:
            L.open("if (j < clim)")
        for n in list(reds) + list(riders):
            if g.is_pair(n):
                L("nh_part_store(&part%d[(long long)blockIdx.y * C + c + j], acc%d[j]);" % (n.nid, n.nid))
            else:
                L("nh_part_store(&part%d[(long long)blockIdx.y * C + c + j], nh_pair{rv%d[j], 0});" % (n.nid, n.nid))
        if tail:
            L.close()
        L.close()
        L.close()
        L("nh_publish_barrier();     // every lane's partial stores have been performed")
        if last_one_folds:
            L.open("if (threadIdx.x == 0)")
            L("const unsigned int before = nh_ticket_take(ctr);")
            L("s_abort = before != %du;" % (chunks * exchanges[0] - 1))
            L.close()
            L("__syncthreads();")
            L("if (s_abort) return;     // not the last to arrive: the last one finishes the strip")
        else:
            exchange_wait()
        exchange_gather(reds, riders)

    def exchange_wait():
        L.open("if (threadIdx.x == 0)")
        L("nh_ticket_take(ctr);")
        L("unsigned int spins = 0; int bad = 0;")
        L.open("while (nh_arrivals(ctr) < %du)" % (chunks * exchanges[0]))
        L("__builtin_amdgcn_s_sleep(4);")
        L("if (++spins > NH_SPIN_LIMIT) { bad = 1; break; }")
        L.close()
        L("s_abort = bad;")
        L.close()
        L("__syncthreads();")
        L.open("if (s_abort)")
        L("// the other workgroups never showed up: leave word for the host and give up rather than hang")
        L("if (threadIdx.x == 0) __hip_atomic_store(status, NH_COOP_ABORTED, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);")
        L("return;")
        L.close()

    def exchange_gather(reds, riders=()):
        QMAX = -(-chunks // LY)
        for n in list(reds) + list(riders):
            L("nh_pair q%d[%d][%d];" % (n.nid, QMAX, V))
        L("#pragma unroll")
        L.open("for (int k = 0; k < %d; ++k)" % QMAX)
        L("const int q = ty + k * %d;" % LY)
        L("const bool live = col_ok && (q < %d);" % chunks)
        L("#pragma unroll")
        L.open("for (int j = 0; j < %d; ++j)" % V)
        for n in list(reds) + list(riders):
            op = g.red_op(n)
            init = ("%s::init()" % op) if g.is_pair(n) else ("nh_pair{%s::init(), 0}" % op)
            L("q%d[k][j] = (live%s) ? nh_part_load(&part%d[(long long)q * C + c + j]) : %s;"
              % (n.nid, " && j < clim" if tail else "", n.nid, init))
        L.close()
        L.close()
        for n in reds:
            op = g.red_op(n)
            L("#pragma unroll")
            L("for (int j = 0; j < %d; ++j) acc%d[j] = %s::init();" % (V, n.nid, op))
        L("#pragma unroll")
        L.open("for (int k = 0; k < %d; ++k)" % QMAX)
        L("#pragma unroll")
        L.open("for (int j = 0; j < %d; ++j)" % V)
        for n in reds:
            op = g.red_op(n)
            if g.is_pair(n):
                L("acc%d[j] = %s::f(acc%d[j], q%d[k][j]);" % (n.nid, op, n.nid, n.nid))
            else:
                L("acc%d[j] = %s::f(acc%d[j], q%d[k][j].v);" % (n.nid, op, n.nid, n.nid))
        L.close()
        L.close()
        for n in reds:
            _emit_col_fold(g, L, n, LX, LY, T, V, "acc%d" % n.nid, dst_decl=False)

    def keep_all():
        for nid, name in cached.items():
            L("#pragma unroll")
            L("for (int i = 0; i < %d; ++i) %s[i].keep();" % (NR, name))

    line_tiles = {}   # leaf nid -> tile that does not change down the column

    def varies_in_loop(n):
        if n.kind == "T":
            return prog.tensors[n.slot].shape[0] > 1
        return n.axis == 1           # one-hot along axis 1 reads idx[r]

    def load_leaves(leaves):
        """names of the tiles inside the row loop; rows not yet resident are
        fetched by a loop of their own first, so that all loads are in flight
        before the first use"""
        tiles = {}
        fresh = [n for n in leaves if varies_in_loop(n) and n.nid not in cached]
        if fresh:
            row_loop_open()
            for n in fresh:
                cached[n.nid] = "keep%d" % n.nid
                L("if (ok) { %s } else keep%d[i].zero();" % (g.load_stmt("keep%d[i]" % n.nid, n, "r", "cc", V, op=g.ld), n.nid))
            L.close()
        for n in leaves:
            tiles[n.nid] = ("keep%d[i]" % n.nid) if varies_in_loop(n) else line_tiles[n.nid]
        return tiles

    def declare_tiles(leaves):
        keep_all()
        for n in leaves:
            if not varies_in_loop(n):
                if n.nid not in line_tiles:
                    name = "line%d" % n.nid
                    line_tiles[n.nid] = name
                    L("%s %s;" % (g.tile_type(n, V), name))
                    L(g.load_stmt(name, n, "0", "cc", V, op="load"))
            elif n.nid not in cached:
                L("%s keep%d[%d];" % (g.tile_type(n, V), n.nid, NR))

    declare_tiles([n for n in g.leaf_nodes(used_nodes([st.root for st in prog.statements]))
                   if not varies_in_loop(n)])

    stages = [[n.args[0] for n in g.own_reductions(per_level.get(s, []))] for s in range(nsweeps)]
    stages = [t for t in stages if t]
    if full_out:
        stages.append([st.root for st in full_out])
    def one_word_per_element(leaf):
        t = prog.tensors[leaf.slot]
        return varies_in_loop(leaf) and t.shape[1] > 1 and DTYPE_CODE[t.dtype] == "f4"

    over = dict((n.nid, leaf) for n, leaf in _overwriting_values(prog, stages, one_word_per_element))
    by_nid = dict((n.nid, n) for n in prog.nodes)
    kept = _kept_values(prog, stages, max_vals, already=[by_nid[k] for k in over])
    kept_ids = set(n.nid for n in kept) | set(over)
    vals = {}          # nid -> expression of a value kept from an earlier sweep

    def stops():
        d = set(done)
        d.update(vals)
        return d

    def stash_new_values(nodes):
        """inside the j loop: keep the values later sweeps will want"""
        fresh = [n for n in nodes if n.nid in kept_ids and n.nid not in vals]
        for n in fresh:
            if n.nid in over:
                L("keep%d[i].put(j, t%d);" % (over[n.nid].nid, n.nid))
            else:
                L("val%d[i][j] = t%d;" % (n.nid, n.nid))
        return fresh

    def declare_values(nodes):
        for n in nodes:
            if n.nid in kept_ids and n.nid not in vals and n.nid not in over:
                L("float val%d[%d][%d];" % (n.nid, NR, V))

    # Variance around a mean down columns that several workgroups share: as in the row family,
    # every workgroup takes the squares around the mean of its own rows, and one exchange
    # carries sums and second moments; sum_i [ M2_i + n_i (mean_i - a)^2 ] afterwards.
    merged = []
    if coop and MERGED_MOMENTS and not over and not kept and per_level.get(0) and per_level.get(1):
        merged = [_shifted_square_sum(n2, g.own_reductions(per_level[0])) for n2 in g.own_reductions(per_level[1])]
        if not merged or not all(merged):
            merged = []
    share = NR * LY      # rows of a strip that one workgroup owns

    def local_second_moments():
        L("const long long left_ = (long long)R - (long long)blockIdx.y * %dll;" % share)
        L("const float n_loc = (float)(left_ < %dll ? left_ : %dll);" % (share, share))
        for n2, r1, x, a in merged:
            L("float mu%d[%d];" % (n2.nid, V))
            L("#pragma unroll")
            L("for (int j = 0; j < %d; ++j) mu%d[j] = rv%d[j] / n_loc;" % (V, n2.nid, r1.nid))
            vals[a.nid] = "mu%d[j]" % n2.nid
        seconds = [m[0] for m in merged]
        nodes = _needed([n.args[0] for n in seconds], stops())
        leaves = g.leaf_nodes(nodes)
        declare_tiles(leaves)
        for n in seconds:
            g.declare_acc(n)
        tiles = load_leaves(leaves)
        row_loop_open()
        L.open("if (ok)")
        if V > 1:
            L("#pragma unroll")
        L.open("for (int j = 0; j < %d; ++j)" % V)
        ref = g.make_ref("_s", "r", "cc", V, tiles, vals)
        g.emit_exprs(nodes, ref, stops())
        for n in seconds:
            g.accumulate(n, ref(n.args[0]), "r", ref)
        L.close()
        L.close()
        L.close()
        for n in seconds:
            _emit_col_fold(g, L, n, LX, LY, T, V, "acc%d" % n.nid)
        for n2, r1, x, a in merged:
            del vals[a.nid]

    def combine_second_moments():
        QMAX = -(-chunks // LY)
        for n2, r1, x, a in merged:
            L("float shift%d[%d];" % (n2.nid, V))
            if V > 1:
                L("#pragma unroll")
            L.open("for (int j = 0; j < %d; ++j)" % V)
            ref = g.make_ref("_s", "0", "cc", V, dict(line_tiles), vals)
            g.emit_exprs(_needed([a], stops()), ref, stops())
            L("shift%d[j] = %s;" % (n2.nid, ref(a)))
            L.close()
            L("#pragma unroll")
            L("for (int j = 0; j < %d; ++j) acc%d[j] = 0.0f;" % (V, n2.nid))
            L("#pragma unroll")
            L.open("for (int k = 0; k < %d; ++k)" % QMAX)
            L("const int q = ty + k * %d;" % LY)
            L.open("if (col_ok && q < %d)" % chunks)
            L("const long long lq = (long long)R - (long long)q * %dll;" % share)
            L("const float nq = (float)(lq < %dll ? lq : %dll);" % (share, share))
            L("#pragma unroll")
            L.open("for (int j = 0; j < %d; ++j)" % V)
            if tail:
                L.open("if (j < clim)")
            L("const float dq = q%d[k][j].v / nq - shift%d[j];" % (r1.nid, n2.nid))
            L("acc%d[j] += __builtin_fmaf(nq * dq, dq, q%d[k][j].v);" % (n2.nid, n2.nid))
            if tail:
                L.close()
            L.close()
            L.close()
            L.close()
            _emit_col_fold(g, L, n2, LX, LY, T, V, "acc%d" % n2.nid, dst_decl=False)
            done[n2.nid] = n2

    ticket_finish = False
    for s in range(nsweeps):
        if merged and s == 1:
            continue            # done together with the first sweep
        reds = g.own_reductions(per_level.get(s, []))
        if not reds:
            continue
        args = [n.args[0] for n in reds]
        nodes = _needed(args, stops())
        leaves = g.leaf_nodes(nodes)
        declare_tiles(leaves)
        declare_values(nodes)
        for n in reds:
            g.declare_acc(n)
        tiles = load_leaves(leaves)
        # a running (max, sum of exponentials) pair over rows that sit in registers: the
        # lane first takes the maximum of its own rows, then adds exp(x - that maximum) --
        # one exponential per element; the pairs of different lanes merge in the folds
        local = [n for n in reds if g.fused_max(n) and n.args[0].kind == "T"]
        if local:
            for n in local:
                L("float lm%d[%d], ls%d[%d];" % (n.nid, V, n.nid, V))
                L("#pragma unroll")
                L("for (int j = 0; j < %d; ++j) { lm%d[j] = -NH_INF; ls%d[j] = 0.0f; }" % (V, n.nid, n.nid))
            row_loop_open()
            L.open("if (ok)")
            if V > 1:
                L("#pragma unroll")
            L.open("for (int j = 0; j < %d; ++j)" % V)
            ref = g.make_ref("_s", "r", "cc", V, tiles, vals)
            for n in local:
                L("lm%d[j] = nh_max(lm%d[j], %s);" % (n.nid, n.nid, ref(n.args[0])))
            L.close()
            L.close()
            L.close()
            for n in local:
                # (a lane that saw nothing, or only -inf, shifts by 0: its terms are exp(-inf) = 0)
                L("float lz%d[%d];" % (n.nid, V))
                L("#pragma unroll")
                L("for (int j = 0; j < %d; ++j) lz%d[j] = (lm%d[j] == -NH_INF) ? 0.0f : lm%d[j];"
                  % (V, n.nid, n.nid, n.nid))
        # Where later stages want exp(x - max) itself (softmax) and x only through it, the lane's
        # exponentials exp(x - its own maximum) take x's place in the registers; once the strip's
        # maximum M is known, exp(x - M) is such a value times exp(own maximum - M), one factor per
        # lane and column: a multiplication behind the exchange instead of another exponential
        # per element (softmax down (32000,256), 31 elements a lane: 20.9 -> 19.7 us, (3000,2000) 18.3 -> 17.3).
        reuse = {}
        for n in local:
            e, x = n.lse_sum.args[0], n.args[0]
            if not LOCAL_EXP_REUSE or not one_word_per_element(x) or x.nid in over.values() or e.nid in kept_ids:
                continue
            rest = [t for k, t in enumerate(stages) if k > s] + [[st.root for st in line_out]]
            avail = set(r.nid for r in prog.nodes if r.kind == "R") | set([e.nid]) | set(vals)
            wanted = [m.nid for t in rest for m in _needed(t, avail)]
            later_all = [m.nid for t in rest for m in _needed(t, avail - set([e.nid]))]
            if x.nid not in wanted and e.nid in later_all:
                reuse[n.nid] = (e, x)
        row_loop_open()
        L.open("if (ok)")
        if V > 1:
            L("#pragma unroll")
        L.open("for (int j = 0; j < %d; ++j)" % V)
        ref = g.make_ref("_s", "r", "cc", V, tiles, vals)
        g.emit_exprs(nodes, ref, stops())
        for n in reds:
            if n.nid in reuse:
                L("const float le%d = nh_exp_nonpos(%s - lz%d[j]);" % (n.nid, ref(n.args[0]), n.nid))
                L("ls%d[j] += le%d;" % (n.nid, n.nid))
                L("keep%d[i].put(j, le%d);" % (reuse[n.nid][1].nid, n.nid))
            elif n in local:
                L("ls%d[j] += nh_exp_nonpos(%s - lz%d[j]);" % (n.nid, ref(n.args[0]), n.nid))
            else:
                g.accumulate(n, ref(n.args[0]), "r", ref)
        fresh = stash_new_values(nodes)
        L.close()
        L.close()
        L.close()
        for n in local:
            L("#pragma unroll")
            L("for (int j = 0; j < %d; ++j) { acc%d[j].v = lm%d[j]; acc%d[j].i = __builtin_bit_cast(int, ls%d[j]); }"
              % (V, n.nid, n.nid, n.nid, n.nid))
        for n in fresh:
            vals[n.nid] = ("keep%d[i].get(j)" % over[n.nid].nid) if n.nid in over else ("val%d[i][j]" % n.nid)
        for n in reds:
            _emit_col_fold(g, L, n, LX, LY, T, V, "acc%d" % n.nid)
            done[n.nid] = n
            if g.fused_max(n):
                done[n.lse_sum.nid] = n.lse_sum
        if coop:
            later = [k for k in range(s + 1, nsweeps) if per_level.get(k) and not (merged and k == 1)]
            ticket_finish = not full_out and not later
            if merged and s == 0:
                local_second_moments()
                exchange(reds, last_one_folds=ticket_finish, riders=[m[0] for m in merged])
                combine_second_moments()
            else:
                exchange(reds, last_one_folds=ticket_finish)
        for n in reds:
            if n.nid in reuse:
                e, x = reuse[n.nid]
                L("float corr%d[%d];" % (n.nid, V))
                L("#pragma unroll")
                L("for (int j = 0; j < %d; ++j) corr%d[j] = nh_exp_nonpos(lz%d[j] - rv%d[j]);" % (V, n.nid, n.nid, n.nid))
                vals[e.nid] = "(keep%d[i].get(j) * corr%d[j])" % (x.nid, n.nid)

    if line_out:
        roots = [st.root for st in line_out]
        nodes = _needed(roots, done)
        leaves = g.leaf_nodes(nodes)
        # (cooperative strips: after a waiting exchange every workgroup has the
        # values and the first one writes; after a ticket only the last arrival is left)
        L.open("if (col_ok && ty == 0%s)" % (" && blockIdx.y == 0" if coop and not ticket_finish else ""))
        for n in leaves:
            g.emit_load(n, "0", "c", V, "_l")
        for st in line_out:
            L("nh_out<%s, %d> o%d; o%d.clear();" % (g.slot_ctype(st.out), V, st.out.index, st.out.index))
        if V > 1:
            L("#pragma unroll")
        L.open("for (int j = 0; j < %d; ++j)" % V)
        ref = g.make_ref("_l", "0", "c", V)
        g.emit_exprs(nodes, ref, done)
        for st in line_out:
            if st.root.kind == "R" and st.root.is_index:
                L("o%d.seti(j, ri%d[j]);" % (st.out.index, st.root.nid))
            else:
                L("o%d.set(j, %s);" % (st.out.index, ref(st.root)))
        L.close()
        for st in line_out:
            L(g.store_stmt("o%d" % st.out.index, "store", g.addr(st.out, "0", "c"), V))
        L.close()

    if full_out:
        roots = [st.root for st in full_out]
        nodes = _needed(roots, stops())
        leaves = g.leaf_nodes(nodes)
        declare_tiles(leaves)
        tiles = load_leaves(leaves)
        row_loop_open()
        L.open("if (ok)")
        for st in full_out:
            L("nh_out<%s, %d> o%d; o%d.clear();" % (g.slot_ctype(st.out), V, st.out.index, st.out.index))
        if V > 1:
            L("#pragma unroll")
        L.open("for (int j = 0; j < %d; ++j)" % V)
        ref = g.make_ref("_s", "r", "cc", V, tiles, vals)
        g.emit_exprs(nodes, ref, stops())
        for st in full_out:
            if st.root.kind == "R" and st.root.is_index:
                L("o%d.seti(j, ri%d[j]);" % (st.out.index, st.root.nid))
            else:
                L("o%d.set(j, %s);" % (st.out.index, ref(st.root)))
        L.close()
        for st in full_out:
            stmt = g.store_stmt("o%d" % st.out.index, g.st, g.addr(st.out, "r", "c"), V if st.out.shape[1] > 1 else 1)
            L(stmt if coop else "if (col_ok) { %s }" % stmt)
        L.close()
        L.close()
    if coop and ticket_finish:
        # everyone has arrived for the last time: re-arm the counter for the next launch
        L("if (threadIdx.x == 0) __hip_atomic_store(ctr, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);")
    elif coop:
        # the last workgroup of the strip to get here has seen everyone pass
        # the final wait: it re-arms both counters for the next launch
        L.open("if (threadIdx.x == 0)")
        L("const unsigned int t = __hip_atomic_fetch_add(ctr + 1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);")
        L.open("if (t == %du)" % (chunks - 1))
        L("__hip_atomic_store(ctr, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);")
        L("__hip_atomic_store(ctr + 1, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);")
        L.close()
        L.close()
    L.close()
    return _finish("colcoop" if coop else "col", g, head, fmt, T, lds,
                   dict(V=V, LX=LX, LY=LY, NR=NR, stream=bool(stream), chunks=chunks,
                        NRED=len(all_reds), kept=len(kept), over=len(over), tail=bool(tail),
                        line_strips=(max(1, 128 // (LX * V * max(wide))) if xcd_runs else 0)))


def colsplit_grid(spec, strips, chunks, xcds=8):
    """launch grid of a ``colsplit`` kernel: (strips, chunks), or -- built with ``runs`` -- one
    dimension of XCDs x strips per XCD x chunks"""
    ls = int(spec.params.get("runs") or 0)
    if not ls:
        return (strips, chunks, 1)
    if ls < 0:
        return (xcds * strips * _ceil(chunks, xcds), 1, 1)
    lines = _ceil(strips, ls)
    nx = min(lines, xcds)
    return (xcds * _ceil(lines, nx) * ls * chunks, 1, 1)


def col_grid(spec, strips, xcds=8):
    """workgroups a ``col`` kernel is launched with: one per strip, or -- strips narrower than
    a cache line, dealt to the XCDs in runs of whole lines -- eight times the longest run"""
    spl = spec.params.get("line_strips", 0)
    if not spl:
        return strips
    nx = max(1, min(xcds, strips // spl))
    return xcds * _ceil(strips, nx)


def _ceil(a, b):
    return -(-a // b)


# (more chunks do not help tall narrow matrices: the one workgroup per strip that
# folds the partials becomes the bottleneck -- (200704,128) fp32 with 384 chunks
# 28 us, with 128 chunks 24 us)
COLSPLIT_MAX_CHUNKS = 128


COLSPLIT_FOLD_BATCH = 4
# fewest rows a lane of the split column family takes from its chunk
COLSPLIT_ROWS_IN_FLIGHT = 4
# Rows a lane of the split column family loads at once (all issued before the first is used), and
# rows of such a batch that a pair reduction takes at a time; the former times the words a row
# position costs bounds the registers held.  Measured on (32000,256) fp32, max / argmax /
# cross-entropy in microseconds: 4 rows 5.2 / 6.9 / 8.3, 8 rows 5.2 / 6.5 / 7.8, 16 rows (pairs
# 16 at a time) 5.6 / 6.7 / 8.2, 16 rows (pairs 4 at a time) 5.6 / 7.3 / 8.5.
COLSPLIT_BATCH_ROWS = 8
COLSPLIT_SUBBATCH_ROWS = 8
COLSPLIT_BATCH_WORDS = 64


def gen_colsplit(prog, V, LX, LY, stream=False, tail=False, fold_batch=1, NR=4, NB=4, multi=True, runs=False,
                 lookback=False):
    """One level of axis-0 reductions over a tall matrix.  grid = (column
    strips, row chunks); a workgroup is LX column-lanes x LY row-lanes.
    ``multi``: more than one chunk per strip.

    ``runs`` (rows that are no whole number of cache lines, where the row
    pieces of neighbouring strips share lines; or strips narrower than a
    line, ``runs`` of them per line): a one-dimensional grid (see
    colsplit_grid) in which the strips that share lines run side by side
    behind one L2.  Negative: every XCD takes whole row chunks with all their
    strips (eight chunks and more); positive: every XCD owns a contiguous run
    of strips -- whole lines -- and takes them chunk by chunk.  Surplus
    workgroups leave at once.

    Sweep.  A lane takes its rows NR at a time: all NR loads are issued before
    the first value is used (a chunk of at most NR * LY rows is fetched in ONE
    round of requests).  Pair reductions then take the rows NB at a time: a
    maximum per element and one scan for its first position for
    arg-reductions, one local maximum and one exponential per element for the
    running (max, sum) pair.  Only a batch that reaches beyond the chunk takes
    the row-by-row form.

    The part after the sweep is a chain of dependent steps on a few values, so
    it is kept short rather than wide: the row-lanes of a wave fold by lane
    exchanges (arg-reductions as 64-bit keys, nh_arg_key: a merge is an
    integer maximum), LDS joins the waves with ONE lane per column doing the
    join and -- with several chunks per strip -- publishing that column's
    partial; then the workgroup takes a ticket, and the one that draws the
    strip's last ticket folds the partials: P adjacent lanes share a column,
    each takes every P-th chunk (``fold_batch`` loads in flight), a DPP
    all-reduce over the P lanes finishes.  Results reach the lanes that
    evaluate the statements through LDS.

    Extra parameters: ``rows_per_chunk``, workspace pointer (partials first,
    then one ticket per strip, TICKET_STRIDE_WORDS words apart, after
    ``ticket_offset`` bytes; tickets start at zero and are reset by their
    last user)."""
    assert prog.nlevels == 1
    g = _RedGen(prog, V, stream, "colsplit")
    g.col_tail = bool(tail)     # partial last column tile, as in gen_col
    L = g.L
    T = LX * LY
    S = LX * V                  # columns of a strip
    assert LX < 64 and T % 64 == 0 and S <= T
    WY = T // 64
    P = min(T // S, 64)         # lanes per column in the folding workgroup
    NB = max(1, min(NB, NR))
    params, fmt = g.param_list([("int rows_per_chunk", "i"), ("char* ws", "P"),
                                ("long long ticket_offset", "q")])
    head = ('extern "C" __global__ __launch_bounds__(%d) void @NAME@(%s)\n' % (T, params))
    reds = g.own_reductions(_live_reductions(prog))
    for st in prog.statements:
        assert st.out.shape[0] == 1
    done = {}
    # what the stages after a lane's own sweep merge with: arg-reductions travel as keys
    fold_op = dict((n.nid, "nh_op_key" if n.is_index else g.red_op(n)) for n in reds)
    L.open("")
    lds = 16
    for n in reds:
        ty_ = "nh_pair" if g.is_pair(n) else "float"
        L("__shared__ __attribute__((aligned(16))) %s s_w%d[%d][%d];" % (ty_, n.nid, WY, S))
        lds += WY * S * (8 if g.is_pair(n) else 4)
        L("__shared__ __attribute__((aligned(16))) %s s_r%d[%d];" % (ty_, n.nid, S))
        lds += S * (8 if g.is_pair(n) else 4)
    L("__shared__ int s_last;")
    g.declare_one()
    lookback = int(lookback) if (lookback and multi and V * 64 <= T) else 0
    if lookback:
        L("__shared__ unsigned int s_tag;")
        L("__shared__ int s_abort;")
    if runs < 0:
        # every XCD takes whole row chunks (chunk = 8 * round + XCD), all strips of a chunk side by side
        L("const int nchunks = (int)(((long long)R + rows_per_chunk - 1) / rows_per_chunk);")
        L("const unsigned int nstrips = (unsigned int)((C + %d) / %d);" % (S - 1, S))
        L("const unsigned int slot = blockIdx.x / NH_XCDS;")
        L("const unsigned int strip = slot % nstrips, chunk = (slot / nstrips) * NH_XCDS + blockIdx.x % NH_XCDS;")
        L("if (chunk >= (unsigned int)nchunks) return;")
    elif runs:
        L("const int nchunks = (int)(((long long)R + rows_per_chunk - 1) / rows_per_chunk);")
        L("const unsigned int nstrips = (unsigned int)((C + %d) / %d);" % (S - 1, S))
        ls = int(runs)                # strips that share a cache line (1: strips of whole lines)
        L("const unsigned int nlines = (nstrips + %du) / %du;" % (ls - 1, ls))
        L("const unsigned int nx = nlines < NH_XCDS ? nlines : NH_XCDS;")
        L("const unsigned int per_xcd = ((nlines + nx - 1u) / nx) * %du;" % ls)
        L("const unsigned int slot = blockIdx.x / NH_XCDS;")
        L("const unsigned int strip = (blockIdx.x % NH_XCDS) * per_xcd + slot % per_xcd, chunk = slot / per_xcd;")
        L("if (blockIdx.x % NH_XCDS >= nx || strip >= nstrips || chunk >= (unsigned int)nchunks) return;")
    else:
        L("const int nchunks = gridDim.y;")
        L("const unsigned int nstrips = gridDim.x;")
        L("const unsigned int strip = blockIdx.x, chunk = blockIdx.y;")
    L("const int tx = threadIdx.x %% %d, ty = threadIdx.x / %d;" % (LX, LX))
    L("const long long c0 = (long long)strip * %d;" % S)
    L("const long long c = c0 + tx * %d;" % V)
    L("const bool col_ok = c < C;")
    L("const long long cc = col_ok ? c : 0;")
    if tail:
        L("const bool cfull = c + %d <= C;" % V)
        L("const int clim = cfull ? %d : (col_ok ? (int)(C - c) : 0);" % V)
    L("const long long r0 = (long long)chunk * rows_per_chunk;")
    L("const long long r1 = (r0 + rows_per_chunk < R) ? (r0 + rows_per_chunk) : (long long)R;")
    if lookback:
        # the tag of this launch: what this workgroup's own first record carried, flipped (every launch
        # writes every record once; the workspace starts zeroed).  Loaded now, needed after the sweep.
        L("nh_pair own_ = nh_pair{0.0f, 0};")
        L("if (threadIdx.x == 0) own_ = nh_part_load(reinterpret_cast<const nh_pair*>(ws) + (long long)chunk * C + c0);")
    g.pos = ("0", "c")
    g.emit_gather_prefetch(_needed([st.root for st in prog.statements], set(n.nid for n in prog.nodes if n.kind == "R")),
                           V, "col_ok && ty == 0")
    args = [n.args[0] for n in reds]
    nodes = _needed(args, {})
    leaves = g.leaf_nodes(nodes)
    for n in reds:
        g.declare_acc(n)
    # reductions that take several rows as a whole
    batched = [n for n in reds if g.is_pair(n) and NB > 1]
    L.open("if (col_ok)")
    L.open("for (long long rb = r0 + ty; rb < r1; rb += %d)" % (NR * LY))
    # -- a whole batch inside the chunk: every load first
    L.open("if (rb + %d < r1)" % ((NR - 1) * LY))
    for u in range(NR):
        for n in leaves:
            g.emit_load(n, "rb + %d" % (u * LY), "c", V, "_%d" % u)
    for b0 in range(0, NR, NB):
        nb = min(NB, NR - b0)
        if V > 1:
            L("#pragma unroll")
        L.open("for (int j = 0; j < %d; ++j)" % V)
        for n in batched:
            L("float lv%d[%d];" % (n.nid, nb))
        for u in range(b0, b0 + nb):
            L.open("")
            ref = g.make_ref("_%d" % u, "rb + %d" % (u * LY), "c", V)
            g.emit_exprs(nodes, ref, {})
            for n in reds:
                if n in batched:
                    L("lv%d[%d] = %s;" % (n.nid, u - b0, ref(n.args[0])))
                else:
                    g.accumulate(n, ref(n.args[0]), "rb + %d" % (u * LY), ref)
            L.close()
        for n in batched:
            if g.fused_max(n):
                L("nh_op_lse::stepn<%d>(acc%d[j], lv%d);" % (nb, n.nid, n.nid))
            else:
                L("%s::stepn<%d>(acc%d[j], lv%d, (int)rb + %d, %d);" % (g.red_op(n), nb, n.nid, n.nid, b0 * LY, LY))
        L.close()
    L.close()
    # -- a batch that reaches beyond the chunk: the rows that exist, one by one (loads first all the same)
    L.open("else")
    for u in range(NR):
        for n in leaves:
            L("%s %s;" % (g.tile_type(n, V), g.tile_name(n, "_%d" % u)))
            L.open("if (rb + %d < r1)" % (u * LY))
            L(g.load_stmt(g.tile_name(n, "_%d" % u), n, "rb + %d" % (u * LY), "c", V))
            L.close()
            L("else %s.zero();" % g.tile_name(n, "_%d" % u))
    for u in range(NR):
        L.open("if (rb + %d < r1)" % (u * LY))
        if V > 1:
            L("#pragma unroll")
        L.open("for (int j = 0; j < %d; ++j)" % V)
        ref = g.make_ref("_%d" % u, "rb + %d" % (u * LY), "c", V)
        g.emit_exprs(nodes, ref, {})
        for n in reds:
            g.accumulate(n, ref(n.args[0]), "rb + %d" % (u * LY), ref)
        L.close()
        L.close()
    L.close()
    L.close()
    L.close()
    # -- after the sweep ---------------------------------------------------------------
    for n in reds:
        if n.is_index:
            L("#pragma unroll")
            L("for (int j = 0; j < %d; ++j) acc%d[j] = nh_arg_key<%s>(acc%d[j]);" % (V, n.nid, g.red_op(n), n.nid))
    steps = (64 // LX).bit_length() - 1
    VK = max(1, V >> steps)             # values a lane still holds after the wave's row-lanes have folded
    holders = LX * (V // VK)            # ... and the lanes of a wave that hold distinct columns
    L("int j0[%d];" % len(reds))
    for k, n in enumerate(reds):
        L("j0[%d] = nh_col_wave_fold<%s, %d, %d>(acc%d);" % (k, fold_op[n.nid], V, LX, n.nid))
    # the waves join through LDS, one lane per column
    L.open("if ((threadIdx.x & 63) < %d)" % holders)
    for k, n in enumerate(reds):
        L("#pragma unroll")
        L("for (int j = 0; j < %d; ++j) s_w%d[threadIdx.x >> 6][tx * %d + j0[%d] + j] = acc%d[j];" % (VK, n.nid, V, k, n.nid))
    L.close()
    if lookback:
        L("if (threadIdx.x == 0) { s_tag = ((nh_u32)own_.i >> 31) ^ 1u; s_abort = 0; }")
    L("__syncthreads();")
    for n in reds:
        L("%s one%d = %s::init();" % ("nh_pair" if g.is_pair(n) else "float", n.nid, fold_op[n.nid]))
    # WY adjacent lanes share a column, each brings one wave's piece, a DPP all-reduce joins
    # them: log2(WY) dependent merges instead of WY - 1 (pair merges are long chains)
    spread = 1 < WY <= 16 and S * WY <= T and WY & (WY - 1) == 0
    if spread:
        L("const int jcol = threadIdx.x / %d;" % WY)
        L("const bool joins = (threadIdx.x %% %d) == 0 && jcol < %d;" % (WY, S))
        for n in reds:
            ty_ = "nh_pair" if g.is_pair(n) else "float"
            L("if (jcol < %d) one%d = s_w%d[threadIdx.x %% %d][jcol];" % (S, n.nid, n.nid, WY))
            L("one%d = nh_wave_allreduce<%s, %d, %s>(one%d);" % (n.nid, fold_op[n.nid], WY, ty_, n.nid))
    else:
        L("const int jcol = threadIdx.x;")
        L("const bool joins = threadIdx.x < %d;" % S)
        L.open("if (joins)")
        for n in reds:
            L("one%d = s_w%d[0][threadIdx.x];" % (n.nid, n.nid))
            if WY > 1:
                L("#pragma unroll")
                L("for (int y = 1; y < %d; ++y) one%d = %s::f(one%d, s_w%d[y][threadIdx.x]);"
                  % (WY, n.nid, fold_op[n.nid], n.nid, n.nid))
        L.close()
    if multi:
        # partial buffers: reduction k occupies [k*nchunks*C, (k+1)*nchunks*C) entries of 8 bytes
        for k, n in enumerate(reds):
            L("nh_pair* part%d = reinterpret_cast<nh_pair*>(ws) + (long long)%d * nchunks * C;" % (n.nid, k))
        L("unsigned int* const ticket = reinterpret_cast<unsigned int*>(ws + ticket_offset) + %d * strip;" % TICKET_STRIDE_WORDS)
        if lookback:
            L("const nh_u32 tag = s_tag;")
        L.open("if (joins && c0 + jcol < C)")
        for n in reds:
            val = ("one%d" % n.nid) if g.is_pair(n) else ("nh_pair{one%d, 0}" % n.nid)
            if lookback:
                val = "nh_tag_put(%s, tag)" % val
            L("nh_part_store(&part%d[(long long)chunk * C + c0 + jcol], %s);" % (n.nid, val))
        L.close()
    if multi and lookback:
        # Tagged records instead of a ticket: (value, tag) is one 8-byte atomic store, so whoever sees the
        # tag has the value.  The strip's LAST %d chunks each finish one tile of V columns: a wave per
        # column polls the records of all chunks, a wave-wide fold, and the lane that owns the tile
        # evaluates the statements.  Everybody else is done after its stores.  The finishing workgroups
        # are the last of their XCD to start: block numbers are dealt to the XCDs in turn, every XCD
        # starts its share in order, and in all three block-to-(strip, chunk) mappings above the chunk
        # grows with the block number within an XCD.  So a workgroup that is still to start only ever
        # queues behind workgroups that store and leave, never behind one that waits -- the finishers
        # cannot keep a producer from running.
        G = S // V
        L("const int grp = (int)chunk - (nchunks - %d);" % G)
        L("if (grp < 0) return;")
        L("const int pw = threadIdx.x >> 6, pq = threadIdx.x & 63;")
        L("const long long pc = c0 + grp * %d + pw;" % V)
        # (lane q takes the records of chunks q, q + 64, ...: PK of them)
        PK = max(1, int(lookback))
        L("const bool owns = (pw < %d) && (pc < C);" % V)
        for n in reds:
            L("nh_pair rec%d[%d];" % (n.nid, PK))
            L("#pragma unroll")
            L("for (int k = 0; k < %d; ++k) rec%d[k] = nh_pair{0.0f, 0};" % (PK, n.nid))
        L.open("if (owns && pq < nchunks)")
        L("unsigned int spins = 0;")
        L.open("for (;;)")
        L("bool seen = true;")
        L("#pragma unroll")
        L.open("for (int k = 0; k < %d; ++k)" % PK)
        L.open("if (pq + 64 * k < nchunks)")
        for n in reds:
            L("rec%d[k] = nh_part_load(&part%d[(long long)(pq + 64 * k) * C + pc]);" % (n.nid, n.nid))
            L("seen = seen && nh_tag_is(rec%d[k], tag);" % n.nid)
        L.close()
        L.close()
        L("if (seen) break;")
        L("__builtin_amdgcn_s_sleep(1);")
        L("if (++spins > NH_SPIN_LIMIT) { s_abort = 1; break; }")
        L.close()
        L.close()
        for n in reds:
            op = fold_op[n.nid]
            ty_ = "nh_pair" if g.is_pair(n) else "float"
            L("one%d = %s::init();" % (n.nid, op))
            L("#pragma unroll")
            L.open("for (int k = 0; k < %d; ++k)" % PK)
            L.open("if (owns && pq + 64 * k < nchunks)")
            if n.is_index:
                L("rec%d[k].i = (int)((nh_u32)rec%d[k].i | 0x80000000u);" % (n.nid, n.nid))
            elif g.is_pair(n):
                L("rec%d[k].i = (int)((nh_u32)rec%d[k].i & 0x7fffffffu);" % (n.nid, n.nid))
            L("one%d = %s::f(one%d, rec%d[k]%s);" % (n.nid, op, n.nid, n.nid, "" if g.is_pair(n) else ".v"))
            L.close()
            L.close()
            L("one%d = nh_wave_allreduce<%s, 64, %s>(one%d);" % (n.nid, op, ty_, n.nid))
        L.open("if (pq == 0 && pw < %d)" % V)
        for n in reds:
            L("s_r%d[grp * %d + pw] = one%d;" % (n.nid, V, n.nid))
        L.close()
    elif multi:
        # The partials were written through to device-coherent memory (nh_part_store); every
        # lane waits for its own stores before the barrier (nh_publish_barrier), lane 0 then
        # takes the ticket, and the last workgroup reads the partials past its L2 (nh_part_load).
        L("nh_publish_barrier();")
        L("if (threadIdx.x == 0) s_last = (nh_ticket_take(ticket) == (unsigned int)(nchunks - 1));")
        L("__syncthreads();")
        L("if (!s_last) return;")
        # the last workgroup: P adjacent lanes per column, lane i of them takes chunks
        # i, i + P, ..., QB of them in flight at a time
        QB = max(1, int(fold_batch))
        L("const int fcol = threadIdx.x / %d, flane = threadIdx.x %% %d;" % (P, P))
        L("const bool fold_ok = (fcol < %d) && (c0 + fcol < C);" % S)
        for n in reds:
            L("one%d = %s::init();" % (n.nid, fold_op[n.nid]))
        L.open("for (int kb = flane; kb < nchunks; kb += %d)" % (P * QB))
        for n in reds:
            L("nh_pair q%d[%d];" % (n.nid, QB))
        L("#pragma unroll")
        L.open("for (int k = 0; k < %d; ++k)" % QB)
        L("const int q = kb + k * %d;" % P)
        for n in reds:
            op = fold_op[n.nid]
            init = ("%s::init()" % op) if g.is_pair(n) else ("nh_pair{%s::init(), 0}" % op)
            L("q%d[k] = (fold_ok && q < nchunks) ? nh_part_load(&part%d[(long long)q * C + c0 + fcol]) : %s;"
              % (n.nid, n.nid, init))
        L.close()
        L("#pragma unroll")
        L.open("for (int k = 0; k < %d; ++k)" % QB)
        for n in reds:
            L("one%d = %s::f(one%d, q%d[k]%s);" % (n.nid, fold_op[n.nid], n.nid, n.nid, "" if g.is_pair(n) else ".v"))
        L.close()
        L.close()
        for n in reds:
            ty_ = "nh_pair" if g.is_pair(n) else "float"
            L("one%d = nh_wave_allreduce<%s, %d, %s>(one%d);" % (n.nid, fold_op[n.nid], P, ty_, n.nid))
        L("if (threadIdx.x == 0) nh_ticket_reset(ticket);")
        L.open("if (flane == 0 && fcol < %d)" % S)
        for n in reds:
            L("s_r%d[fcol] = one%d;" % (n.nid, n.nid))
        L.close()
    else:
        L.open("if (joins)")
        for n in reds:
            L("s_r%d[jcol] = one%d;" % (n.nid, n.nid))
        L.close()
    L("__syncthreads();")
    if multi and lookback:
        # a record never came (its workgroup was not running within the wait's bound): no result for
        # this tile, and the host is told through the plan's status word
        L.open("if (s_abort)")
        L("unsigned int* status = reinterpret_cast<unsigned int*>(ws + ticket_offset) + %d * nstrips;" % TICKET_STRIDE_WORDS)
        L("if (threadIdx.x == 0) __hip_atomic_store(status, NH_COOP_ABORTED, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);")
        L("return;")
        L.close()
    # the lanes that evaluate the statements pick up the V columns of their tile
    for n in reds:
        if n.is_index:
            L("int ri%d[%d];" % (n.nid, V))
        else:
            L("float rv%d[%d];" % (n.nid, V))
        if g.fused_max(n):
            L("float rv%d[%d];" % (n.lse_sum.nid, V))
        L("#pragma unroll")
        if n.is_index:
            L("for (int j = 0; j < %d; ++j) ri%d[j] = nh_key_index(s_r%d[tx * %d + j]);" % (V, n.nid, n.nid, V))
        elif g.fused_max(n):
            L("for (int j = 0; j < %d; ++j) { rv%d[j] = s_r%d[tx * %d + j].v; rv%d[j] = nh_lse_total(s_r%d[tx * %d + j]); }"
              % (V, n.nid, n.nid, V, n.lse_sum.nid, n.nid, V))
        else:
            L("for (int j = 0; j < %d; ++j) rv%d[j] = s_r%d[tx * %d + j];" % (V, n.nid, n.nid, V))
        done[n.nid] = n
        if g.fused_max(n):
            done[n.lse_sum.nid] = n.lse_sum

    roots = [st.root for st in prog.statements]
    nodes = _needed(roots, done)
    leaves = g.leaf_nodes(nodes)
    L.open("if (col_ok && ty == 0%s)" % (" && tx == grp" if (multi and lookback) else ""))
    for n in leaves:
        g.emit_load(n, "0", "c", V, "_l")
    for st in prog.statements:
        L("nh_out<%s, %d> o%d; o%d.clear();" % (g.slot_ctype(st.out), V, st.out.index, st.out.index))
    if V > 1:
        L("#pragma unroll")
    L.open("for (int j = 0; j < %d; ++j)" % V)
    ref = g.make_ref("_l", "0", "c", V)
    g.emit_exprs(nodes, ref, done)
    for st in prog.statements:
        if st.root.kind == "R" and st.root.is_index:
            L("o%d.seti(j, ri%d[j]);" % (st.out.index, st.root.nid))
        else:
            L("o%d.set(j, %s);" % (st.out.index, ref(st.root)))
    L.close()
    for st in prog.statements:
        L(g.store_stmt("o%d" % st.out.index, "store", g.addr(st.out, "0", "c"), V))
    L.close()
    L.close()
    return _finish("colsplit", g, head, fmt, T, lds,
                   dict(V=V, LX=LX, LY=LY, NR=NR, NB=NB, NRED=len(reds), multi=bool(multi),
                        stream=bool(stream), tail=bool(tail), runs=int(runs), lookback=int(lookback)))
