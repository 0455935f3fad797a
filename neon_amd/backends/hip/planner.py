"""
Shape-class selection, kernel cache and launch plans.

``make_plan(prog, rt, cache)`` looks at a finalized program (optree_ir) and
picks a kernel family and its tiling from the actual geometry, generates the
source, compiles it (or finds it in the cache) and returns a ``Plan`` whose
``launch`` packs arguments and enqueues.  The reference did the equivalent in
``call_compound_kernel`` (float_ew.py:644-940) with three hard-wired block
sizes tuned for a 24-SM part; here the choice is driven by what fills 256
compute units and keeps every access a 16-byte vector.

``NeedsSplit`` tells the backend that the tree must be broken into several
programs through temporaries (the job of ``_split_to_stacks`` in the
reference, nervanagpu.py:1099-1237).
"""
import hashlib
import os
import tempfile

import numpy as np

from neon_amd.backends.hip import codegen
from neon_amd.backends.hip import runtime as hiprt
from neon_amd.backends.hip.optree_ir import used_nodes


# Kernels that touch at least this much (the eight L2 slices hold 32 MiB
# together) mark their global accesses non-temporal: measured +10% on the
# 7-stream Adam update and +20% on the fp16 row normalisation.
STREAM_BYTES = 32 << 20


def _streams(prog):
    touched = sum(t.dtype.itemsize * t.shape[0] * t.shape[1] for t in prog.tensors)
    return touched >= STREAM_BYTES


class NeedsSplit(Exception):
    """The program cannot run as one kernel; evaluate reductions separately."""


def _pow2ceil(x):
    p = 1
    while p < x:
        p *= 2
    return p


def _pow2floor(x):
    p = 1
    while p * 2 <= x:
        p *= 2
    return p


def _ceil_div(a, b):
    return -(-a // b)


# ---------------------------------------------------------------------------------------
# kernel cache: in-process dict in front of an on-disk store of code objects
# (the role of neon/backends/util/source_module.py:16-22 for the reference)
# ---------------------------------------------------------------------------------------
class KernelCache(object):
    def __init__(self, arch, cache_dir=None, formal_fences=None):
        self.arch = arch
        with open(hiprt.DEVICE_HEADER) as f:
            self.header = f.read()
        if formal_fences is None:
            # The default hand-off between workgroups leans on how gfx950 acknowledges write-through
            # stores (see neon_device.h); on any other part the kernels are built with the
            # device-scope release / acquire fences the language's memory model asks for.
            formal_fences = (os.environ.get("NEON_HIP_FORMAL_FENCES", "0") != "0"
                             or not arch.startswith("gfx950"))
        self.formal_fences = bool(formal_fences)
        if self.formal_fences:
            self.header = "#define NH_FORMAL_FENCES 1\n" + self.header
        if os.environ.get("NEON_HIP_EXACT_LSE_TERMS", "0") != "0":
            # the terms of a running sum of exponentials each rounded like expf (see nh_exp_term)
            self.header = "#define NH_EXACT_LSE_TERMS 1\n" + self.header
        if cache_dir is None:
            cache_dir = os.environ.get("NEON_HIP_CACHE_DIR")
        if cache_dir is None and os.environ.get("NEON_CACHE_DIR"):
            cache_dir = os.path.join(os.environ["NEON_CACHE_DIR"], "hip")
        if cache_dir is None:
            # next to the prebuilt library, so kernels compiled at build time are
            # found at run time; a read-only install falls back to the home dir
            local = os.path.join(os.path.dirname(hiprt.LIB_PATH), "kcache")
            try:
                os.makedirs(local, exist_ok=True)
                cache_dir = local if os.access(local, os.W_OK) else None
            except OSError:
                cache_dir = None
        if cache_dir is None:
            cache_dir = os.path.join(os.path.expanduser("~"), ".cache", "neon_amd", "hip")
        self.cache_dir = cache_dir
        self.loaded = {}      # kernel name -> runtime.Kernel
        self.stats = {"hit_mem": 0, "hit_disk": 0, "compiled": 0}
        self.dump_dir = os.environ.get("NEON_HIP_DUMP")

    def _digest(self, source):
        h = hashlib.sha256()
        h.update(self.arch.encode())
        h.update(" ".join(hiprt.RTC_OPTIONS).encode())
        h.update(self.header.encode())
        h.update(source.encode())
        return h.hexdigest()

    def code_object(self, spec):
        """code-object bytes for a Spec, compiling on a miss"""
        full = self.header + "\n" + spec.source
        path = os.path.join(self.cache_dir, self._digest(spec.source) + ".hsaco")
        if self.dump_dir:
            os.makedirs(self.dump_dir, exist_ok=True)
            with open(os.path.join(self.dump_dir, spec.name + ".hip"), "w") as f:
                f.write(spec.source)
        try:
            with open(path, "rb") as f:
                self.stats["hit_disk"] += 1
                return f.read()
        except (IOError, OSError):
            pass
        code, _log = hiprt.rtc_compile(full, spec.name + ".hip", self.arch)
        self.stats["compiled"] += 1
        try:
            os.makedirs(self.cache_dir, exist_ok=True)
            fd, tmp = tempfile.mkstemp(dir=self.cache_dir)
            with os.fdopen(fd, "wb") as f:
                f.write(code)
            os.replace(tmp, path)
        except (IOError, OSError):
            pass       # a read-only cache directory only costs recompiles
        return code

    def kernel(self, rt, spec):
        k = self.loaded.get(spec.name)
        if k is not None:
            self.stats["hit_mem"] += 1
            return k
        code = self.code_object(spec)
        k = rt.load_kernel(code, spec.name, spec.fmt)
        self.loaded[spec.name] = k
        return k


# ---------------------------------------------------------------------------------------
# vector width
# ---------------------------------------------------------------------------------------
def _vector_width(prog, tail_ok):
    """V (elements per lane access): 16 bytes of the narrowest column-varying
    operand, at most 8 elements.  Addresses need no alignment beyond the
    element's (the device's vector accesses are typed byte-aligned), so views
    that start mid-row and odd row lengths keep full-width accesses; what V
    must do is divide the row length, unless the family handles a partial last
    tile (``tail_ok``)."""
    C = prog.domain[1]
    cols = [t for t in prog.tensors if t.shape[1] > 1]
    used = used_nodes([st.root for st in prog.statements])
    hot0 = [prog.tensors[n.slot] for n in used if n.kind == "H" and n.axis == 0]
    if not cols and not hot0:
        return 1
    if any(t.strides[1] != 1 or t.take_axis == 1 for t in cols):
        return 1
    isz_min = min([t.dtype.itemsize for t in cols] + [4 for _ in hot0])
    V = min(8, 16 // isz_min)
    while V > 1 and C % V and not tail_ok:
        V //= 2
    if C < V:
        V = 1 if not tail_ok else max(1, _pow2floor(C))
    # a lane's tile is held in whole 32-bit words: narrower vectors of 1- and
    # 2-byte elements do not exist
    while V > 1 and any((V * t.dtype.itemsize) % 4 for t in cols):
        V //= 2
    return V


def _check_onehot(prog):
    R, C = prog.domain
    for n in used_nodes([st.root for st in prog.statements]):
        if n.kind == "H":
            t = prog.tensors[n.slot]
            want = C if n.axis == 0 else R
            size = t.shape[0] * t.shape[1]
            contiguous = t.strides == (t.shape[1], 1) or 1 in t.shape and (
                t.strides[0 if t.shape[1] == 1 else 1] == 1)
            if size != want or not contiguous:
                raise TypeError("onehot index vector of size %d does not match extent %d" % (size, want))


def _try_flatten(prog):
    """A reduction-free program whose tensors all have the domain's shape and
    are contiguous (or are 1x1) is a 1-d problem: view it as one long row."""
    R, C = prog.domain
    if R == 1:
        return
    for t in prog.tensors:
        if t.take_axis is not None or t.index in prog.index_slots:
            return
        if t.shape == (1, 1):
            continue
        if t.shape != (R, C) or t.strides != (C, 1):
            return
    for n in prog.nodes:
        if n.kind == "H":
            return
    N = R * C
    if N > 0x7FFFFFFF:
        return                  # extents are 32-bit kernel arguments: stay two-dimensional
    for t in prog.tensors:
        if t.shape != (1, 1):
            t.shape, t.strides = (1, N), (N, 1)
    prog.domain = (1, N)


# ---------------------------------------------------------------------------------------
# plans
# ---------------------------------------------------------------------------------------
class Plan(object):
    """A compiled kernel + grid; ``launch(prog)`` binds the argument values of
    any program with the same key."""

    def __init__(self, rt, kernel, spec, grid, extras_fn=None, workspace=None, status_ptr=None, counters=None):
        self.rt = rt
        # cooperative families: device address of the word an aborting workgroup
        # marks, and (address, count) of the arrival counters -- for the host's check
        self.status_ptr = status_ptr
        self.counters = counters
        self.kernel = kernel
        self.spec = spec
        self.grid = grid
        self.block = (spec.block, 1, 1)
        self.extras_fn = extras_fn
        self.workspace = workspace     # device allocation owned by the plan
        self.key = None                # program key the backend filed the plan under
        self.domain = None             # set by make_plan: the (R, C) the kernel iterates

    def _values(self, prog):
        vals = []
        for t in prog.tensors:
            vals.append(t.ptr)
            vals.append(t.strides[0])
            vals.append(t.strides[1])
        nconst0 = len(vals)
        vals.extend(prog.consts)
        vals.append(self.domain[0])
        vals.append(self.domain[1])
        if prog.rand_count:
            vals.extend(prog.rng_args)
        if self.extras_fn is not None:
            vals.extend(self.extras_fn())
        try:
            self.kernel.packer.pack(*vals)
        except OverflowError:
            # a constant beyond the fp32 range becomes +-inf, as a numpy cast would
            for i in range(nconst0, nconst0 + len(prog.consts)):
                with np.errstate(over="ignore"):
                    vals[i] = float(np.float32(vals[i]))
        return vals

    def pack(self, prog):
        """argument buffer for ``prog`` (any program with this plan's key)"""
        return self.kernel.packer.pack(*self._values(prog))

    def const_offsets(self, prog):
        """byte offset of every constant slot inside the packed arguments"""
        import struct
        head = "@" + "Pqq" * len(prog.tensors)
        return [struct.calcsize(head + "f" * (k + 1)) - 4 for k in range(len(prog.consts))]

    def launch(self, prog):
        self.rt.launch_packed(self.kernel, self.grid, self.block, self.pack(prog))

    def launch_timed(self, prog, reps):
        """mean ms per launch of ``reps`` back-to-back launches (bench mode)"""
        return self.rt.launch_timed(self.kernel, self.grid, self.block, 0, reps, *self._values(prog))

    def launch_timed_sets(self, progs, reps):
        """the same over several programs of this plan's shape (identical
        structure, different tensors), launched in rotation"""
        return self.rt.launch_timed_sets(self.kernel, self.grid, self.block, 0, reps,
                                         [self._values(prog) for prog in progs])

    def release(self):
        if self.workspace:
            self.rt.free(self.workspace)
            self.workspace = None


def _words_per_tile(prog, V, axis):
    """registers one resident tile position costs, summed over the tensor
    leaves that vary along the reduced axis (the others are loaded once)"""
    total = 0
    for t in prog.tensors:
        if not t.read or t.shape[axis] == 1:
            continue
        w = V if t.shape[1] > 1 else 1
        total += max(1, (w * t.dtype.itemsize + 3) // 4)
    return max(total, 1)


class Choice(object):
    """Outcome of shape-class selection: generated kernel, grid and what the
    extra kernel parameters are.  Needs no device."""

    def __init__(self, spec, grid, extras=(), workspace=None, status_offset=None):
        self.spec = spec
        self.grid = grid
        self.extras = tuple(extras)          # literal values appended after R, C
        self.workspace = workspace           # None or (bytes, ticket_offset, n_tickets)
        self.status_offset = status_offset   # cooperative families: byte offset of the status word


def choose(prog, cu_count=256, coop=True):
    """Pick family + tiling for a finalized program and generate its source.
    ``coop=False`` keeps to the families whose workgroups never wait for one
    another (what the backend falls back to once a cooperative plan's bounded
    wait has expired, e.g. on a device it does not have to itself)."""
    R, C = prog.domain
    if R > 0x7FFFFFFF or C > 0x7FFFFFFF:
        raise ValueError("tensor dimension too large")
    _check_onehot(prog)
    if prog.axis is None:
        return _plan_ew(prog, cu_count)
    if prog.axis == 1:
        return _plan_row(prog, cu_count, coop)
    return _plan_col(prog, cu_count, coop)


def make_plan(prog, rt, cache, cu_count, coop=True):
    ch = choose(prog, cu_count, coop)
    kernel = cache.kernel(rt, ch.spec)
    extras = ch.extras
    ws = status = counters = None
    if ch.workspace is not None:
        ws_bytes, ticket_off, n_tickets = ch.workspace
        ws = rt.malloc(ws_bytes)
        rt.memset(ws + ticket_off, 0, n_tickets, 4)   # tickets start at zero and reset themselves
        if ch.spec.params.get("tagged") or ch.spec.params.get("lookback"):
            rt.memset(ws, 0, ticket_off // 4, 4)      # tagged partials: every slot's tag starts at zero
        extras = extras + (ws, ticket_off)
        if ch.status_offset is not None:
            status, counters = ws + ch.status_offset, (ws + ticket_off, n_tickets)
    plan = Plan(rt, kernel, ch.spec, ch.grid, extras_fn=(lambda e=extras: e) if extras else None,
                workspace=ws, status_ptr=status, counters=counters)
    plan.domain = tuple(prog.domain)
    return plan


EW_FLAT_LANES = int(os.environ.get("NEON_HIP_EW_T", "512"))       # tuning aid


def _plan_ew(prog, cu_count):
    _try_flatten(prog)
    R, C = prog.domain
    V = _vector_width(prog, tail_ok=True)
    nvec = _ceil_div(C, V)
    if R == 1:
        # (flattened programs: 512 lanes.  Fused Adam over 25 M parameters, by workgroup size: 64 lanes 105.4 us,
        # 128 104.6, 256 106.4, 512 104.6 / 103.6 in a second run, 1024 105.8; two vectors per lane 105.0; the
        # three-kernel form 155 -> 151 us, the 2 MB sigmoid 2.4 -> 2.2 us)
        LX, LY, UR, UC = EW_FLAT_LANES, 1, 1, 1
    else:
        LX = min(256, _pow2ceil(nvec))
        LY = 256 // LX
        UC = 1
        # rows per lane: several for cache-resident inputs (fewer workgroups to
        # start), one when streaming from HBM (bias add over (4096,65536): 357 us
        # with four rows per lane, 334 us with one -- as for the flat kernels,
        # more loads in flight per lane only add read/write turnarounds)
        UR = 1 if _streams(prog) else max(1, min(4, R // (LY * 8)))
        if UR == 1 and R >= LY * 16:
            # two rows per lane where a workgroup fetches a piece of a row vector for every
            # row tile it handles (x * row over (4096,30000): 190 -> 173 us), and for very many
            # short rows ((131072,1000) bias add: 195 -> 189 us)
            row_vectors = any(t.read and t.shape[0] == 1 and t.shape[1] > 1 for t in prog.tensors)
            if row_vectors or (nvec <= 256 and R > 65535 * LY):
                UR = 2
    # one pass over far more data than the caches hold: streaming accesses
    stream = _streams(prog)
    tail = (C % V) != 0
    spec = codegen.gen_ew(prog, V, LX, LY, UC, UR, tail, stream)
    gx = _ceil_div(nvec, LX * UC)
    row_tiles = _ceil_div(R, LY * UR)
    gy = min(row_tiles, 65535)
    if gx > 0x7FFFFFFF:
        raise ValueError("tensor too large for one launch")
    return Choice(spec, (gx, gy, 1), extras=(row_tiles,))


# LDS a 1024-lane workgroup may use as a second tier of residence (gfx950: 160 KB per compute
# unit; the rest is left to the reduction slots).  A compute unit then holds one such workgroup
# instead of two, which costs less than fetching the tiles again -- also with more rows than
# compute units (batch-norm backward over (512,100352) fp16: 71 -> 57 us; forward over
# (512,200704): 136 -> 80 us; half the LDS and two workgroups per unit: 64 / 87 us).
ROW_PARK_BYTES = int(os.environ.get("NEON_HIP_ROW_PARK_KB", "144")) << 10


def limit_lds(bytes_per_workgroup):
    """tell the planner how much LDS a workgroup may have on the device in use
    (160 KB on gfx950, which the defaults assume); called by the backend with
    the figure the runtime reports"""
    global ROW_PARK_BYTES
    ROW_PARK_BYTES = max(0, min(ROW_PARK_BYTES, int(bytes_per_workgroup) - (16 << 10)))


ROW_SPLIT_WORDS = int(os.environ.get("NEON_HIP_SPLIT_WORDS", "64"))
ROWCOOP_MAX_TILES = int(os.environ.get('NEON_HIP_ROWCOOP_TILES', str(1 << 20)))
ROW_SPLIT_MAX_TILES = int(os.environ.get('NEON_HIP_ROW_SPLIT_TILES', str(1 << 20)))   # tiles of 1024 lanes per row that the split-residence form takes


ROW_KEPT_VALUES = os.environ.get("NEON_HIP_ROW_VALS", "1") != "0"


def _plan_row(prog, cu_count, coop=True):
    # The tiling is chosen for the tree as written.  A maximum and the sum of exponentials
    # around it then share a sweep (a running pair) only where that saves a pass over memory
    # or an exchange: rows that are streamed, wholly or in part; rows resident in registers
    # are swept three times at no cost and keep the exponentials for the last sweep.
    paired = prog.lse_pairs > 0
    if paired:
        prog.unpair_lse()
    R, C = prog.domain
    V = _vector_width(prog, tail_ok=True)
    tail = (C % V) != 0
    nvec = _ceil_div(C, V)
    words = _words_per_tile(prog, V, 1)
    options = []
    if nvec <= 64 * 8:
        # four tiles per lane, but a row's lanes together fetch at least
        # one 128-byte line per load: with fewer, every load of a wave
        # touches a line per row and uses a fraction of it
        line = max(8, 32 // V)
        options.append((max(min(line, _pow2ceil(nvec)), min(64, _pow2ceil(_ceil_div(nvec, 4)))), 256))
    options += [(256, 256), (512, 512), (1024, 1024)]
    LX, T, NCH = 1024, 1024, 0          # fallback: stream the row on every sweep
    for lx, t in options:
        nch = _ceil_div(nvec, lx)
        budget = 64 if t == 1024 else 128
        if nch <= 16 and nch * words <= budget:
            LX, T, NCH = lx, t, nch
            break
    # (rows too long for that are streamed again on every sweep: keeping the
    # two fp16 rows of batch-norm backward resident in 512-lane workgroups, 200
    # registers per lane, measured 53 us against 45 us for streaming twice)
    keep_words = None
    # passes over the row: one per level of reductions, one more when full-shape results are stored
    sweeps = prog.nlevels + (1 if any(st.out.shape[1] > 1 for st in prog.statements) else 0)
    if NCH == 0 and prog.nlevels + 1 >= 2:
        # the row does not fit as a whole: keep what fits of it (in order of
        # first use) in a 1024-lane workgroup and fetch the rest again per sweep
        nch = _ceil_div(nvec, 1024)
        smallest = min([max(1, (V * t.dtype.itemsize + 3) // 4)
                        for t in prog.tensors if t.read and t.shape[1] > 1] or [1 << 30])
        if nch <= 16 and nch * smallest <= 64:
            LX, T, NCH, keep_words = 1024, 1024, nch, 64
        elif nch <= ROW_SPLIT_MAX_TILES and ROW_PARK_BYTES and sweeps >= 2:
            # longer still: registers and LDS together hold (most of) one operand
            # ((256,200704) fp16: 16 tiles in registers + 9 in LDS = the whole row)
            LX, T, NCH, keep_words = 1024, 1024, nch, ROW_SPLIT_WORDS
    # Few, very long rows (batch norm over the 64 feature maps of an early
    # convolution): one workgroup per row would leave most compute units idle
    # and the row may not fit its registers.  Spread every row over several
    # workgroups that exchange their partial results; all of them must be
    # resident at once, so rows x chunks stays within the compute units.
    tiles = _ceil_div(nvec, 1024)
    if coop and R * 2 <= cu_count and tiles >= 8 and prog.nlevels >= 1:
        chunks = min(cu_count // R, tiles // 4, 64)
        per = _ceil_div(tiles, chunks)
        chunks = _ceil_div(tiles, per)
        smallest = min([max(1, (V * t.dtype.itemsize + 3) // 4)
                        for t in prog.tensors if t.read and t.shape[1] > 1] or [1 << 30])
        # (longer shares, where the row is swept more than once: what registers and LDS do not
        # hold of a workgroup's share is fetched again in every sweep -- still all compute units
        # at work instead of one per row.  Batch norm over (64,1605632) fp16: forward 304 ->
        # 147 us, backward 372 -> 169 us; a single sweep gains nothing from it)
        if chunks >= 2 and ((per <= 16 and per * smallest <= 64) or
                            (per <= ROWCOOP_MAX_TILES and ROW_PARK_BYTES and sweeps >= 2)):
            kw = None if (per <= 16 and per * words <= 64) else (64 if per <= 16 else ROW_SPLIT_WORDS)
            # (resident shares of 16-bit rows too: their exponentials cannot take over the
            # operand's registers, so the pair costs no extra exponential and saves an exchange --
            # (16,1605632) fp16 35.8 -> 32.3 us; fp32 shares lose 1-3 us with it)
            narrow = any(t.read and t.shape[1] > 1 and t.dtype.itemsize < 4 for t in prog.tensors)
            # (short shares excepted: folding pairs through the workgroup costs two exponentials a
            # step, more than the exchange saved -- (64,131072) fp16, 4 tiles each: 13.8 vs 16.2 us)
            if paired and (kw is not None or (narrow and per >= 8)):
                prog.pair_lse()
            spec = codegen.gen_row(prog, V, 1024, 1, per, _streams(prog), keep_words=kw, chunks=chunks, tail=tail,
                                   park_bytes=ROW_PARK_BYTES if kw else 0)
            part_bytes = R * spec.params["NRED"] * chunks * 8
            ctr_off = _ceil_div(part_bytes, 256) * 256
            stride = codegen.TICKET_STRIDE_WORDS      # arrivals and departures of a row; rows a cache line apart
            return Choice(spec, (R, chunks, 1), workspace=(ctr_off + (R * stride + 1) * 4, ctr_off, R * stride + 1),
                          status_offset=ctr_off + R * stride * 4)
    LY = T // LX
    gx = _ceil_div(R, LY)
    park = ROW_PARK_BYTES if (keep_words and LY == 1) else 0
    # registers left over next to a fully resident row may hold expensive
    # values that a later sweep needs again
    max_vals = 0
    if NCH and keep_words is None and sweeps >= 2 and ROW_KEPT_VALUES:
        budget = 64 if T == 1024 else 96
        max_vals = min(2, max(0, (budget - NCH * words) // (NCH * V)))
    # (also 16-bit rows that fill the registers: with no room to keep the exponentials, the pair's
    # one sweep is cheaper than the two it replaces -- (4096,131072) fp16 521 -> 482 us)
    narrow = any(t.read and t.shape[1] > 1 and t.dtype.itemsize < 4 for t in prog.tensors)
    if paired and (NCH == 0 or keep_words is not None or (max_vals == 0 and narrow)):
        prog.pair_lse()
    spec = codegen.gen_row(prog, V, LX, LY, NCH, _streams(prog), keep_words=keep_words, tail=tail, park_bytes=park,
                           max_vals=max_vals)
    return Choice(spec, (gx, 1, 1))


# 32-bit registers per lane that resident tiles (and kept values) may occupy,
# by workgroup size: what is left of the 512 / (waves per SIMD) budget after
# the temporaries that full unrolling keeps live (measured: beyond these the
# compiler spills)
_COL_BUDGET = {1024: 40, 512: 120, 256: 300}


COLSPLIT_THREADS = int(os.environ.get("NEON_HIP_CS_T", "256"))

COLSPLIT_RUNS = os.environ.get("NEON_HIP_COLSPLIT_RUNS", "1") != "0"
# split column reductions: the last workgroups of a strip wait for the others' tagged partials
# instead of the last ticket holder folding them all (see gen_colsplit)
COLSPLIT_LOOKBACK = os.environ.get("NEON_HIP_CS_LOOKBACK", "1") != "0"
COLCOOP = os.environ.get("NEON_HIP_COLCOOP", "1") != "0"       # 0: axis-0 trees never wait between workgroups
# Beyond this size the cooperative family (rows resident in registers, one workgroup per compute
# unit, a waiting exchange per level) loses to stage-by-stage evaluation, whose reduction kernels
# stream at full occupancy.  Softmax, measured: (32000,256) 28 us either way; (64000,256) 60 us
# cooperative, 44 us in two kernels; (6000,2304) 54 against 40 us.
COLCOOP_MAX_BYTES = int(os.environ.get("NEON_HIP_COLCOOP_MAX_MB", "48")) << 20
COLCOOP_MAX_BYTES_512 = max(COLCOOP_MAX_BYTES, int(os.environ.get("NEON_HIP_COLCOOP_MAX_MB_512", "72")) << 20)
# ... and below this one its exchanges (some 8 us each, whatever the size) cost more than the extra pass
# over a small matrix.  Softmax, cooperative / staged: (8192,1024) fp16, 16 MB: 26 / 20 us; (4096,1000)
# fp32, 16 MB: 18.3 / 16.6; (3000,2000) fp32, 24 MB: 20.5 / 22.0; (16384,512) fp32, 32 MB: 24.3 / 26.4.
COLCOOP_MIN_BYTES = int(os.environ.get("NEON_HIP_COLCOOP_MIN_MB", "20")) << 20
COL_TINY_ONE_WORD = os.environ.get("NEON_HIP_COL_TINY_ONE_WORD", "1") != "0"
ONLINE_LSE_IN_ONE_WORKGROUP = os.environ.get("NEON_HIP_ONLINE_LSE_COL", "0") != "0"


def _plan_col(prog, cu_count, coop=True, one_word_lanes=None):
    R, C = prog.domain
    V = _vector_width(prog, tail_ok=True)
    isz = max([t.dtype.itemsize for t in prog.tensors if t.shape[1] > 1] + [1])
    if (one_word_lanes is None and COL_TINY_ONE_WORD and V > 4 // isz and isz in (2, 4)
            and R * C * isz <= (4 << 20)):
        # Tiny inputs whose rows stay in registers: one 32-bit word per lane and the strip's width made of
        # adjacent lanes, instead of one 16-byte vector per lane -- a quarter of the registers, and the wave
        # fold has one value (two 16-bit ones) to pass round instead of four (eight).  Softmax down the
        # columns, 16 bytes / 4 bytes per lane: (1000,128) fp32 4.5 -> 4.0 us, (2000,128) 6.3 -> 5.3, (512,512)
        # 4.2 -> 4.0, (300,1024) 4.1 -> 3.6, (100,4096) 3.9 -> 3.6, (64,2048) 3.4 -> 3.2, (1000,256) 4.8 -> 4.8;
        # fp16 (1000,128) 4.9 -> 4.5, (2000,256) 7.1 -> 5.9.  Mean / variance normalisation (1000,128) fp32
        # 4.7 -> 3.9, fp16 5.2 -> 3.9; argmax fp32 3.6 -> 3.2, fp16 4.1 -> 3.2; sum 2.6 -> 2.5.  From 8 MB on
        # there is nothing in it ((2000,2048) fp32 softmax 11.8 / 12.0 us, (1000,4096) 9.1 / 9.2).
        try:
            ch = _plan_col(prog, cu_count, coop, one_word_lanes=True)
            if ch.spec.family == "col":
                return ch
        except NeedsSplit:
            pass
    if one_word_lanes:
        V = 4 // isz
    tail = (C % V) != 0
    nvec = _ceil_div(C, V)
    words = _words_per_tile(prog, V, 0)
    line_only = all(st.out.shape[0] == 1 and R > 1 for st in prog.statements)

    # (a) whole column strip inside one workgroup, rows resident in registers.
    # Wider strips coalesce better (>= 128 B per row segment wanted), narrower
    # ones leave more row-lanes, i.e. fewer rows per lane: take the widest
    # strip for which all rows fit in registers.
    lx_min = max(1, min(64, 128 // (V * isz)))
    tiny = R * C * isz <= (4 << 20)
    if tiny:
        lx_min = 1                       # tiny inputs are latency-bound: favour more workgroups
    lx_pref = max(lx_min, min(64, _pow2floor(max(1, nvec // 32))))
    lx_pref = min(lx_pref, _pow2ceil(nvec))
    lx_min = min(lx_min, lx_pref)
    def lanes_for(lx):
        """workgroup size, row-lanes and rows per lane for strips of ``lx``
        column-lanes, or None where the rows do not fit in registers"""
        strips = _ceil_div(nvec, lx)
        # many strips: small workgroups, several per compute unit; few: spend more lanes on
        # each so that the rows-per-lane count drops and a unit has waves to switch between
        # (tiny inputs: joining 16 waves costs more than a second row per lane -- softmax
        # over (1000,128): 1024 lanes 5.3 us, 512 lanes 4.4 us)
        if strips >= 4 * cu_count:
            order = (256, 512, 1024)
        elif strips >= 2 * cu_count:
            order = (512, 1024, 256)
        elif tiny:
            order = (512, 1024, 256)
        else:
            order = (1024, 512, 256)
        for T in order:
            LY = T // lx
            NR = _ceil_div(R, LY)
            if LY >= 1 and NR <= 16 and NR * words <= _COL_BUDGET[T]:
                return (T, LY, NR)
        return None

    fit = None
    LX = lx_pref
    if R <= 2048:
        # rather strips of 32-byte row pieces than workgroups that have to wait for each other:
        # softmax / normalisation down the columns of (2000,2048) fp16 14.6 / 14.7 us against
        # 18.4 / 21.9 us cooperating, (1500,1024) fp32 7.6 / 7.9 against 11.0 / 13.0, (2048,8192)
        # fp32 38 / 42 against 43 / 53 us in stages; from 3000 rows on the narrow strips lose
        lx_min = min(lx_min, max(1, 32 // (V * isz)))
    while fit is None and LX >= lx_min:
        fit = lanes_for(LX)
        if fit is None:
            LX //= 2
    if fit is None:
        LX = lx_pref
    # Fewer strips than compute units: narrower strips, down to 32-byte row pieces, while the
    # rows still fit -- a strip is one workgroup, and an idle unit costs more than half-used
    # cache lines (whose other half a neighbouring strip on the same XCD reads).  Softmax down
    # the columns, before -> after: (512,4096) fp32 10.6 -> 6.2 us, (256,8192) 10.4 -> 6.1,
    # (1000,1024) 10.3 -> 6.0, (1000,4096) 11.8 -> 9.5, fp16 21.3 -> 9.6, (1000,8192) fp16 23.1 -> 15.9.
    while fit is not None and _ceil_div(nvec, LX) < cu_count and (LX // 2) * V * isz >= 32:
        narrower = lanes_for(LX // 2)
        if narrower is None:
            break
        LX, fit = LX // 2, narrower
    single_level = prog.nlevels == 1
    big = R * C >= (1 << 18)
    if fit and not (single_level and line_only and big and R >= 512):
        T, LY, NR = fit
        if prog.lse_pairs and not ONLINE_LSE_IN_ONE_WORKGROUP:
            # no exchange between workgroups to save here, and the running pair
            # costs two more exponentials per element than a sweep of its own
            prog.unpair_lse()
        budget = _COL_BUDGET[T]
        spare = max(0, (budget - NR * words) // (NR * V))
        assert (NR - 1) * LY < R <= NR * LY      # the kernels test only a lane's last row against R
        # rows that are no whole number of cache lines: neighbouring strips share lines, keep them on one XCD
        runs = (C * isz) % 128 != 0 and LX * V * isz >= 128 and _ceil_div(nvec, LX) >= 64
        spec = codegen.gen_col(prog, V, LX, LY, NR, _streams(prog), max_vals=min(2, spare), tail=tail, runs=runs)
        return Choice(spec, (codegen.col_grid(spec, _ceil_div(nvec, LX)), 1, 1))

    # (c) deeper trees (or full-shape results) over many rows: the workgroups of a
    # strip keep their rows in registers and exchange partials between sweeps.
    # Everything must be resident at once, so the grid stays within one
    # workgroup per compute unit.
    if coop and COLCOOP and not (single_level and line_only) and COLCOOP_MIN_BYTES <= R * C * isz <= COLCOOP_MAX_BYTES_512:
        # narrow strips keep the partials each workgroup has to gather small
        # (measured on (32000,256): 8 column-lanes 37 us, 16 lanes 43 us, 4 lanes
        # 41 us).  More strips than half the compute units leave no second
        # workgroup per strip: such widths go to the families below
        lxc = max(1, min(8, _pow2ceil(nvec)))
        strips_c = _ceil_div(nvec, lxc)
        if strips_c <= cu_count:
            chunks = max(1, min(128, cu_count // strips_c))
            rpc0 = _ceil_div(R, chunks)
            # (eight values per lane: the folds' temporaries take twice the registers, and many
            # rows per lane then spill -- (5000,5000) fp16 softmax with 27 rows per lane in 512
            # lanes 64 us, with 53 in 256 lanes 88 us, in stages 43 us; (10000,2000) 46 / 38 us)
            options = ((1024, 40), (512, 120), (256, 300)) if V < 8 else ((1024, 32), (512, 64))
            if os.environ.get("NEON_HIP_COOP_T"):          # tuning aid
                options = tuple(o for o in options if o[0] == int(os.environ["NEON_HIP_COOP_T"]))
            if R * C * isz > COLCOOP_MAX_BYTES:
                # beyond that size only while the rows still fit workgroups of 512 lanes and more: with 256
                # lanes (60+ rows a lane) the cooperative form loses to stages again -- softmax, cooperative /
                # staged: (60000,256) 34.6 / 40.8 us, (14000,1024) 31.9 / 37.6, (3500,4096) 32.6 / 37.4,
                # (28000,512) 32.5 / 38.5, but (6000,2304) 43.9 / 35.6 and (4096,4096) 46.7 / 42.1 in 256 lanes
                options = tuple(o for o in options if o[0] >= 512)
            for T, budget in options:
                LY = T // lxc
                NR = _ceil_div(rpc0, LY)
                if NR <= 64 and NR * words <= budget:
                    chunks = _ceil_div(R, NR * LY)
                    if chunks < 2:
                        break
                    spare = max(0, (budget - NR * words) // (NR * V))
                    spec = codegen.gen_col(prog, V, lxc, LY, NR, _streams(prog), chunks=chunks,
                                           max_vals=min(2, spare), tail=tail)
                    part_bytes = spec.params["NRED"] * chunks * C * 8
                    ctr_off = _ceil_div(part_bytes, 256) * 256
                    return Choice(spec, (strips_c, chunks, 1),
                                  workspace=(ctr_off + (strips_c * codegen.TICKET_STRIDE_WORDS + 1) * 4, ctr_off,
                                             strips_c * codegen.TICKET_STRIDE_WORDS + 1),
                                  status_offset=ctr_off + strips_c * codegen.TICKET_STRIDE_WORDS * 4)

    # (b) one level, one value per column, many rows: split rows over workgroups
    if single_level and line_only:
        # Workgroups are cheap to run but not free to start: give each one at
        # least ~128 KiB to stream, one per compute unit for small inputs and
        # up to eight for large ones.
        bytes_total = R * C * isz
        per_cu = max(1, min(8, bytes_total // (cu_count * (128 << 10))))
        target = per_cu * cu_count
        # 16 column-lanes per strip; 8 when the chunk limit would leave fewer than
        # two workgroups per compute unit, or when the input is small enough that
        # the last workgroup's fold of the partials shows (fewer, longer chunks).
        # Measured: (200704,128) fp32 23 -> 21 us, fp16 26 -> 18 us, (32000,256)
        # fp32 10.1 -> 9.3 us; (200704,256) fp32 already has 512 workgroups with
        # 16 lanes and loses with 8 (36 us against 44 us).
        # (wide matrices: 32 column-lanes, 512-byte row pieces -- (4096,30000) fp32 97 -> 90 us,
        # (32000,2048) 47 -> 43 us, (30000,4096) fp16 46 -> 41 us, (4096,131072) fp16 183 -> 166 us;
        # 64 lanes gain nothing more)
        LX = max(lx_min, min(32 if nvec >= 256 else 16, _pow2ceil(nvec)))
        if LX == 16 and (per_cu == 1 or
                         _ceil_div(nvec, LX) * codegen.COLSPLIT_MAX_CHUNKS < min(target, 2 * cu_count)):
            LX = max(lx_min, 8)
        if os.environ.get("NEON_HIP_CS_LX"):               # tuning aid
            LX = int(os.environ["NEON_HIP_CS_LX"])
        # one workgroup per compute unit (small inputs): twice the lanes, so that a SIMD has a
        # second wave to run while the first waits for its rows ((32000,256): argmax 11.0 ->
        # 10.7 us, max 8.1 -> 7.3 us); larger inputs already get several workgroups per unit
        strips = _ceil_div(nvec, LX)
        # (the limit bounds what the last workgroup of a strip has to fold; strips
        # under 64 columns may take more chunks, as far as it takes to get two
        # workgroups per compute unit: (802816,32) fp32 34 -> 23 us)
        cap = codegen.COLSPLIT_MAX_CHUNKS
        wide_cap = cap * max(1, 64 // (LX * V))
        cap = max(cap, min(wide_cap, _ceil_div(2 * cu_count, strips)))
        # Row chunks per strip: enough for one workgroup per compute unit, and beyond that no
        # more than 32 -- every further chunk is another ticket on the strip's counter and
        # another partial for its last workgroup to fold, which costs more than the extra
        # workgroups bring.  Measured (max over axis 0): (30000,1000) fp16 94 chunks 27 us, 32
        # chunks 17 us; (131072,1000) fp16 128: 69 us, 32: 60 us; (128000,1024) fp32 127: 94 us,
        # 32: 91 us; (200704,128) fp32, four strips: 126: 22 us, 64: 18 us, 32: 23 us.
        chunks = max(1, min(cap, max(cu_count // strips, min(32, target // strips))))
        # few workgroups: twice the lanes each, so that a SIMD has a second wave to run while the
        # first waits for its rows ((32000,256): max 8.1 -> 7.3 us; (802816,32) fp32 29 -> 22 us;
        # (1000000,64) fp16 52 -> 35 us); many workgroups already overlap
        if os.environ.get("NEON_HIP_CS_T"):
            threads = COLSPLIT_THREADS
        else:
            threads = 512 if strips * chunks <= 2 * cu_count else 256
            if strips * chunks <= cu_count // 2 and R >= 4096 * chunks:
                # half the compute units idle and long chunks: all the lanes a workgroup can have
                # ((1048576,64) fp16, one strip of 128 chunks: sum 31.3 -> 27.4 us, argmax 47.7 -> 36.4)
                threads = 1024
        LY = threads // LX
        # rows a lane fetches at once and reduces as one batch: as many as the registers take
        # (COLSPLIT_BATCH_WORDS words of resident tiles), at most what a chunk gives a lane.
        # A chunk is a whole number of such batches, so that only the matrix's last chunk
        # meets its end inside one.
        per_lane = max(codegen.COLSPLIT_ROWS_IN_FLIGHT, _ceil_div(max(1, _ceil_div(R, chunks)), LY))
        NR = max(1, min(codegen.COLSPLIT_BATCH_ROWS, codegen.COLSPLIT_BATCH_WORDS // words, per_lane))
        rpc = _ceil_div(per_lane, NR) * NR * LY
        chunks = _ceil_div(R, rpc)
        if chunks > 65535:
            raise ValueError("tensor too large for one launch")
        # partials a lane of the last workgroup has in flight: P = lanes per column there
        lanes_per_column = min(threads // (LX * V), 64)
        fold_batch = max(1, min(codegen.COLSPLIT_FOLD_BATCH, _ceil_div(chunks, lanes_per_column)))
        # rows that are no whole number of cache lines: the row pieces of neighbouring strips share lines
        # Rows that are no whole number of cache lines: the row pieces of neighbouring strips share lines.
        # Many strips: every XCD a contiguous run of them; few strips and eight chunks or more: every XCD
        # whole chunks.  Sum over axis 0, (strips, chunks) grid / runs of strips / whole chunks:
        # (4096,30000) fp32 86 / 80 / 83 us, (131072,1000) fp32 111 / 104 / 97 us, fp16 60 / 60 / 50 us.
        runs = 0
        if COLSPLIT_RUNS and chunks > 1 and strips > 1:
            narrow = LX * V * isz < 128                # (strips narrower than a cache line: tuning aid only)
            if (narrow or (C * isz) % 128 != 0) and chunks >= 8 and strips < 64:
                runs = -1
            elif narrow:
                runs = 128 // (LX * V * isz)
            elif (C * isz) % 128 != 0 and strips >= 16:
                runs = 1
        # The strip's last LX workgroups each finish one tile of V columns, the lanes of a wave polling the
        # chunks' tagged partials (up to four each): needs a wave per column of the tile, at least twice as
        # many chunks as tiles, and block numbers that grow with the chunk (so that on every XCD whoever
        # waits starts after everybody else).  (32000,256) fp32 on one box, ticket / tagged: max 5.6 -> 5.1
        # us, argmax 6.9 -> 6.2 us, cross-entropy 8.3 -> 7.8 us; the more chunks the last ticket holder had
        # to fold alone the more it brings: (131072,64) fp16, 128 chunks, sum 9.8 -> 6.0 us, argmax 13.0 ->
        # 8.5; (802816,32) fp32, 224 chunks, 19.7 -> 16.3 / 21.5 -> 17.6; (400000,16) fp32 7.9 -> 5.9 /
        # 9.5 -> 7.1; on the grids dealt to the XCDs in runs (rows that are no whole cache lines) (50000,250)
        # fp16 11.4 -> 9.7 / 13.9 -> 12.0, (64000,300) fp32 23.5 -> 21.7 / 25.1 -> 23.0, (131072,1000) fp16
        # 46.3 -> 44.4 / 56.5 -> 54.0.  Like the other waiting families it is dropped for a program whose
        # wait once expired (coop=False).
        lookback = (coop and COLSPLIT_LOOKBACK and 2 * LX <= chunks <= 256
                    and strips * chunks <= 2 * cu_count and V * 64 <= threads)
        lookback = _ceil_div(chunks, 64) if lookback else 0      # records a polling lane takes
        spec = codegen.gen_colsplit(prog, V, LX, LY, _streams(prog), tail=tail, fold_batch=fold_batch, NR=NR,
                                    NB=codegen.COLSPLIT_SUBBATCH_ROWS, multi=chunks > 1, runs=runs, lookback=lookback)
        part_bytes = spec.params["NRED"] * chunks * C * 8
        ticket_off = _ceil_div(part_bytes, 256) * 256
        n_tickets = strips * codegen.TICKET_STRIDE_WORDS
        if spec.params["lookback"]:
            # (the ticket words go unused; the status word sits behind them, where the kernel looks for it)
            return Choice(spec, codegen.colsplit_grid(spec, strips, chunks), extras=(rpc,),
                          workspace=(ticket_off + (n_tickets + 1) * 4, ticket_off, n_tickets + 1),
                          status_offset=ticket_off + n_tickets * 4)
        return Choice(spec, codegen.colsplit_grid(spec, strips, chunks), extras=(rpc,),
                      workspace=(ticket_off + n_tickets * 4, ticket_off, n_tickets))

    raise NeedsSplit()
