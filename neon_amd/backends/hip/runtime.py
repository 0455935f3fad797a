"""
ctypes binding of libneonhip.so -- the only module that crosses the C ABI.

It stands where PyCUDA stands in the reference (``pycuda.driver`` /
``pycuda.compiler`` as used by neon/backends/nervanagpu.py and float_ew.py):
device memory, copies, fills, events, run-time compilation, module loading and
kernel launch.  Failures surface as ``HipError`` carrying the library's
message (hipGetErrorString text or the hiprtc log).
"""
import ctypes
import os
import struct
from ctypes import (POINTER, byref, c_char, c_char_p, c_float, c_int, c_int32,
                    c_size_t, c_uint8, c_uint16, c_uint32, c_uint64, c_void_p)

_HERE = os.path.dirname(os.path.abspath(__file__))
_PKG = os.path.dirname(os.path.dirname(_HERE))
LIB_PATH = os.path.join(_PKG, "lib", "libneonhip.so")
DEVICE_HEADER = os.path.join(_PKG, "csrc", "device", "neon_device.h")

NH_RTC_ERROR_BASE = 10000
NH_EINVAL = 20001
NH_ENOTINIT = 20002
NH_ECOOP = 20003        # raised by the backend, never returned by the library: a cooperative kernel gave up

# Options every device compilation uses, prebuilt or run-time: no contraction of
# a*b+c into fma (results then follow the expression as written, like numpy's
# separate ufunc calls) and no packed-fp32 instruction selection.
RTC_OPTIONS = ("-O3", "-std=c++17", "-ffp-contract=off",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops")


class HipError(RuntimeError):
    def __init__(self, code, message):
        super(HipError, self).__init__("[%d] %s" % (code, message))
        self.code = code


class Props(ctypes.Structure):
    _fields_ = [("arch", c_char * 64), ("name", c_char * 128),
                ("compute_units", c_int32), ("wave_size", c_int32),
                ("max_threads_per_block", c_int32), ("lds_bytes_per_block", c_int32),
                ("l2_bytes", c_int32), ("clock_khz", c_int32),
                ("mem_clock_khz", c_int32), ("mem_bus_bits", c_int32),
                ("hbm_bytes", c_uint64)]


class LaunchRec(ctypes.Structure):
    """nh_launch_rec: one prepared launch"""
    _fields_ = [("function", c_void_p), ("grid", c_uint32 * 3), ("block", c_uint32 * 3),
                ("lds_bytes", c_uint32), ("arg_bytes", c_uint32), ("stream", c_void_p), ("args", c_void_p)]


# name -> (restype, argtypes); must list every symbol include/neonhip.h declares
SIGNATURES = {
    "nh_abi_version": (c_int, []),
    "nh_device_count": (c_int, [POINTER(c_int)]),
    "nh_init": (c_int, [c_int, POINTER(Props)]),
    "nh_shutdown": (c_int, []),
    "nh_device_sync": (c_int, []),
    "nh_last_error": (c_char_p, []),
    "nh_malloc": (c_int, [POINTER(c_void_p), c_size_t]),
    "nh_free": (c_int, [c_void_p]),
    "nh_mem_info": (c_int, [POINTER(c_size_t), POINTER(c_size_t)]),
    "nh_memcpy_h2d": (c_int, [c_void_p, c_void_p, c_size_t, c_void_p]),
    "nh_memcpy_d2h": (c_int, [c_void_p, c_void_p, c_size_t, c_void_p]),
    "nh_memcpy_d2d": (c_int, [c_void_p, c_void_p, c_size_t, c_void_p]),
    "nh_memset_d8": (c_int, [c_void_p, c_uint8, c_size_t, c_void_p]),
    "nh_memset_d16": (c_int, [c_void_p, c_uint16, c_size_t, c_void_p]),
    "nh_memset_d32": (c_int, [c_void_p, c_uint32, c_size_t, c_void_p]),
    "nh_host_alloc": (c_int, [POINTER(c_void_p), c_size_t]),
    "nh_host_free": (c_int, [c_void_p]),
    "nh_stream_create": (c_int, [POINTER(c_void_p)]),
    "nh_stream_destroy": (c_int, [c_void_p]),
    "nh_stream_sync": (c_int, [c_void_p]),
    "nh_event_create": (c_int, [POINTER(c_void_p)]),
    "nh_event_destroy": (c_int, [c_void_p]),
    "nh_event_record": (c_int, [c_void_p, c_void_p]),
    "nh_event_sync": (c_int, [c_void_p]),
    "nh_event_elapsed_ms": (c_int, [c_void_p, c_void_p, POINTER(c_float)]),
    "nh_rtc_compile": (c_int, [c_char_p, c_char_p, c_char_p, POINTER(c_char_p), c_int,
                               POINTER(c_void_p), POINTER(c_size_t), POINTER(c_void_p)]),
    "nh_buf_free": (c_int, [c_void_p]),
    "nh_module_load": (c_int, [c_void_p, c_size_t, POINTER(c_void_p)]),
    "nh_module_unload": (c_int, [c_void_p]),
    "nh_module_get_function": (c_int, [c_void_p, c_char_p, POINTER(c_void_p)]),
    "nh_launch": (c_int, [c_void_p, POINTER(c_uint32), POINTER(c_uint32), c_uint32,
                          c_void_p, c_void_p, c_size_t]),
    "nh_launch_prepared": (c_int, [c_void_p]),
    "nh_launch_timed": (c_int, [c_void_p, POINTER(c_uint32), POINTER(c_uint32), c_uint32,
                                c_void_p, c_void_p, c_size_t, c_uint32, POINTER(c_float)]),
    "nh_launch_timed_sets": (c_int, [c_void_p, POINTER(c_uint32), POINTER(c_uint32), c_uint32,
                                     c_void_p, POINTER(c_void_p), c_size_t, c_uint32, c_uint32,
                                     POINTER(c_float)]),
    "nh_ew_axpby_f32": (c_int, [c_void_p, c_void_p, c_void_p, c_float, c_float, c_size_t, c_void_p]),
    "nh_ew_sigmoid_f32": (c_int, [c_void_p, c_void_p, c_size_t, c_void_p]),
    "nh_adam_step_f32": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_float, c_float,
                                 c_float, c_float, c_float, c_float, c_size_t, c_void_p]),
    "nh_rownorm_f16": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_float, c_uint32,
                               c_uint32, c_size_t, c_void_p]),
    "nh_hist_log2": (c_int, [c_void_p, c_void_p, c_int, c_size_t, c_int, c_int, c_void_p]),
    "nh_gemm": (c_int, [c_int, c_int, c_int, c_uint32, c_uint32, c_uint32, c_float, c_void_p, c_size_t,
                        c_void_p, c_size_t, c_float, c_void_p, c_size_t, c_void_p]),
    "nh_gemm_batched": (c_int, [c_int, c_int, c_int, c_uint32, c_uint32, c_uint32, c_float, c_void_p, c_size_t,
                                ctypes.c_longlong, c_void_p, c_size_t, ctypes.c_longlong, c_float, c_void_p,
                                c_size_t, ctypes.c_longlong, c_uint32, c_void_p]),
    "nh_copy_transpose": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
    "nh_lut_workspace_bytes": (c_size_t, [c_uint32, c_uint32]),
    "nh_lut_bprop": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_uint32, c_uint32, c_uint32, c_size_t,
                             c_size_t, c_int32, c_void_p, c_size_t, c_void_p]),
    "nh_colreduce_workspace_bytes": (c_size_t, [c_uint32, c_uint32]),
    "nh_colmax_argmax_f32": (c_int, [c_void_p, c_void_p, c_void_p, c_uint32, c_uint32,
                                     c_size_t, c_void_p, c_void_p]),
    "nh_colmax_argmax_f32_static": (c_int, [c_void_p, c_void_p, c_void_p, c_uint32, c_uint32,
                                            c_size_t, c_void_p]),
}

_lib = None


def load_library(path=None):
    """Load libneonhip.so and type every entry point.  There is no fallback:
    a missing library is an ImportError-grade failure for the hip backend."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    path = path or LIB_PATH
    if not os.path.exists(path):
        raise OSError("%s not found: build it with `python -c 'import __graft_entry__ as g; "
                      "g.build()'` (hipcc, gfx950)" % path)
    lib = ctypes.CDLL(path)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def _check(rc):
    if rc != 0:
        msg = _lib.nh_last_error()
        raise HipError(rc, msg.decode("utf-8", "replace") if msg else "unknown error")


def device_count():
    lib = load_library()
    n = c_int(0)
    rc = lib.nh_device_count(byref(n))
    return 0 if rc else n.value


class Kernel(object):
    """A loaded device function plus the struct layout of its parameters."""
    __slots__ = ("module", "function", "name", "packer", "arg_bytes")

    def __init__(self, module, function, name, fmt):
        self.module = module
        self.function = function
        self.name = name
        self.packer = struct.Struct(fmt)
        self.arg_bytes = self.packer.size


class Runtime(object):
    """One initialised device + one stream (the reference backend likewise
    drives a single stream, nervanagpu.py:780)."""

    def __init__(self, device_id=0):
        self.lib = load_library()
        self.props = Props()
        _check(self.lib.nh_init(device_id, byref(self.props)))
        self.device_id = device_id
        self.arch = self.props.arch.decode()
        self.stream = c_void_p(None)      # null stream
        self._grid = (c_uint32 * 3)()
        self._block = (c_uint32 * 3)()
        self._launch_prepared = self.lib.nh_launch_prepared
        # the same entry point as a plain address, for callers that launch from C
        self.launch_prepared_address = ctypes.cast(self.lib.nh_launch_prepared, c_void_p).value

    # -- memory ------------------------------------------------------------------
    def malloc(self, nbytes):
        p = c_void_p()
        _check(self.lib.nh_malloc(byref(p), nbytes))
        return p.value

    def free(self, ptr):
        if ptr:
            _check(self.lib.nh_free(c_void_p(ptr)))

    def mem_info(self):
        f, t = c_size_t(), c_size_t()
        _check(self.lib.nh_mem_info(byref(f), byref(t)))
        return f.value, t.value

    def memcpy_h2d(self, dst, host_array):
        _check(self.lib.nh_memcpy_h2d(c_void_p(dst), c_void_p(host_array.ctypes.data),
                                      host_array.nbytes, self.stream))

    def memcpy_d2h(self, host_array, src):
        _check(self.lib.nh_memcpy_d2h(c_void_p(host_array.ctypes.data), c_void_p(src),
                                      host_array.nbytes, self.stream))

    def memcpy_d2d(self, dst, src, nbytes):
        _check(self.lib.nh_memcpy_d2d(c_void_p(dst), c_void_p(src), nbytes, self.stream))

    def memset(self, dst, pattern, count, itemsize):
        if itemsize == 1:
            _check(self.lib.nh_memset_d8(c_void_p(dst), pattern, count, self.stream))
        elif itemsize == 2:
            _check(self.lib.nh_memset_d16(c_void_p(dst), pattern, count, self.stream))
        elif itemsize == 4:
            _check(self.lib.nh_memset_d32(c_void_p(dst), pattern, count, self.stream))
        else:
            raise ValueError("memset itemsize %d" % itemsize)

    # -- sync / timing -------------------------------------------------------------
    def synchronize(self):
        _check(self.lib.nh_stream_sync(self.stream))

    def event(self):
        e = c_void_p()
        _check(self.lib.nh_event_create(byref(e)))
        return e

    def event_destroy(self, e):
        _check(self.lib.nh_event_destroy(e))

    def event_record(self, e):
        _check(self.lib.nh_event_record(e, self.stream))

    def event_sync(self, e):
        _check(self.lib.nh_event_sync(e))

    def event_elapsed_ms(self, start, stop):
        ms = c_float()
        _check(self.lib.nh_event_elapsed_ms(start, stop, byref(ms)))
        return ms.value

    # -- modules -------------------------------------------------------------------
    def load_kernel(self, code, name, fmt):
        mod = c_void_p()
        buf = ctypes.create_string_buffer(code, len(code))
        _check(self.lib.nh_module_load(buf, len(code), byref(mod)))
        fn = c_void_p()
        _check(self.lib.nh_module_get_function(mod, name.encode(), byref(fn)))
        return Kernel(mod, fn, name, fmt)

    def launch(self, kernel, grid, block, lds_bytes, *values):
        g, b = self._grid, self._block
        g[0], g[1], g[2] = grid
        b[0], b[1], b[2] = block
        args = kernel.packer.pack(*values)
        _check(self.lib.nh_launch(kernel.function, g, b, lds_bytes, self.stream,
                                  args, kernel.arg_bytes))

    def launch_packed(self, kernel, grid, block, args):
        """launch with an already packed argument buffer"""
        g, b = self._grid, self._block
        g[0], g[1], g[2] = grid
        b[0], b[1], b[2] = block
        rc = self.lib.nh_launch(kernel.function, g, b, 0, self.stream, args, kernel.arg_bytes)
        if rc:
            _check(rc)

    def prepare(self, kernel, grid, block, args):
        """a launch record for ``launch_prepared``: (pointer to the record, the
        record, the argument buffer -- a mutable copy that may be patched in
        place between launches)"""
        buf = ctypes.create_string_buffer(bytes(args), len(args))
        rec = LaunchRec()
        rec.function = kernel.function
        rec.grid[0], rec.grid[1], rec.grid[2] = grid
        rec.block[0], rec.block[1], rec.block[2] = block
        rec.lds_bytes, rec.arg_bytes = 0, kernel.arg_bytes
        rec.stream = self.stream
        rec.args = ctypes.addressof(buf)
        return (c_void_p(ctypes.addressof(rec)), rec, buf)

    def launch_prepared(self, prepared):
        rc = self._launch_prepared(prepared[0])
        if rc:
            _check(rc)

    def launch_timed(self, kernel, grid, block, lds_bytes, reps, *values):
        """mean milliseconds per launch over ``reps`` back-to-back launches"""
        g, b = self._grid, self._block
        g[0], g[1], g[2] = grid
        b[0], b[1], b[2] = block
        args = kernel.packer.pack(*values)
        ms = c_float()
        _check(self.lib.nh_launch_timed(kernel.function, g, b, lds_bytes, self.stream,
                                        args, kernel.arg_bytes, reps, byref(ms)))
        return ms.value

    def launch_timed_sets(self, kernel, grid, block, lds_bytes, reps, value_sets):
        """mean milliseconds per launch over ``reps`` launches that cycle
        through the argument tuples in ``value_sets``"""
        g, b = self._grid, self._block
        g[0], g[1], g[2] = grid
        b[0], b[1], b[2] = block
        bufs = [ctypes.create_string_buffer(bytes(kernel.packer.pack(*values)), kernel.arg_bytes)
                for values in value_sets]
        ptrs = (c_void_p * len(bufs))(*[ctypes.addressof(buf) for buf in bufs])
        ms = c_float()
        _check(self.lib.nh_launch_timed_sets(kernel.function, g, b, lds_bytes, self.stream, ptrs,
                                             kernel.arg_bytes, len(bufs), reps, byref(ms)))
        return ms.value

    def hist_log2(self, hist_ptr, x_ptr, itemsize, n, nbins, offset):
        _check(self.lib.nh_hist_log2(c_void_p(hist_ptr), c_void_p(x_ptr), itemsize, n, nbins, offset,
                                     self.stream))

    def gemm(self, itemsize, trans_a, trans_b, m, n, k, alpha, a_ptr, lda, b_ptr, ldb, beta, c_ptr, ldc):
        _check(self.lib.nh_gemm(itemsize, int(trans_a), int(trans_b), m, n, k, alpha, c_void_p(a_ptr), lda,
                                c_void_p(b_ptr), ldb, beta, c_void_p(c_ptr), ldc, self.stream))

    def copy_transpose(self, out_ptr, in_ptr, itemsize, shape, out_strides, in_strides):
        n = len(shape)
        c_shape = (c_uint32 * n)(*shape)
        c_os = (ctypes.c_int64 * n)(*out_strides)
        c_is = (ctypes.c_int64 * n)(*in_strides)
        _check(self.lib.nh_copy_transpose(c_void_p(out_ptr), c_void_p(in_ptr), itemsize, n, c_shape, c_os, c_is,
                                          self.stream))

    def gemm_batched(self, itemsize, trans_a, trans_b, m, n, k, alpha, a_ptr, lda, stride_a, b_ptr, ldb, stride_b,
                     beta, c_ptr, ldc, stride_c, batch):
        _check(self.lib.nh_gemm_batched(itemsize, int(trans_a), int(trans_b), m, n, k, alpha, c_void_p(a_ptr), lda,
                                        stride_a, c_void_p(b_ptr), ldb, stride_b, beta, c_void_p(c_ptr), ldc,
                                        stride_c, batch, self.stream))

    def lut_workspace_bytes(self, nin, vocab):
        return self.lib.nh_lut_workspace_bytes(nin, vocab)

    def lut_bprop(self, dw_ptr, err_t_ptr, ids_ptr, itemsize, nin, embed, vocab, ld_dw, ld_err, pad_idx,
                  ws_ptr, ws_bytes):
        _check(self.lib.nh_lut_bprop(c_void_p(dw_ptr), c_void_p(err_t_ptr), c_void_p(ids_ptr), itemsize, nin, embed,
                                     vocab, ld_dw, ld_err, pad_idx, c_void_p(ws_ptr), ws_bytes, self.stream))

    def shutdown(self):
        self.lib.nh_shutdown()


def rtc_compile(source, name, arch, options=RTC_OPTIONS):
    """HIP C++ text -> code object bytes for ``arch`` (works without a device
    when ``arch`` is given).  Raises ``HipError`` with the compiler log."""
    lib = load_library()
    opts = (c_char_p * len(options))(*[o.encode() for o in options])
    code, size, log = c_void_p(), c_size_t(), c_void_p()
    rc = lib.nh_rtc_compile(source.encode(), name.encode(),
                            arch.encode() if arch else None, opts, len(options),
                            byref(code), byref(size), byref(log))
    log_text = ""
    if log.value:
        log_text = ctypes.string_at(log.value).decode("utf-8", "replace")
        lib.nh_buf_free(log)
    if rc != 0:
        msg = lib.nh_last_error().decode("utf-8", "replace")
        raise HipError(rc, msg if msg else log_text)
    try:
        return ctypes.string_at(code.value, size.value), log_text
    finally:
        lib.nh_buf_free(code)
