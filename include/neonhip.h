/*
 * neonhip.h -- C ABI of libneonhip.so, the device boundary of the `hip` backend.
 *
 * The reference reaches its device through PyCUDA's driver-API wrappers; each
 * entry point below names the reference call it stands in for (paths relative
 * to the reference tree).  The only caller in this package is the ctypes
 * binding neon_amd/backends/hip/runtime.py.
 *
 * Conventions
 *   - every function returns 0 on success, otherwise a positive hipError_t, or
 *     a hiprtcResult offset by NH_RTC_ERROR_BASE, or one of the NH_E* codes;
 *     nh_last_error() returns the message for the calling thread.
 *   - no C++ type, exception or torch object crosses the boundary: device
 *     pointers are void*, streams/events/modules/functions are opaque void*.
 *   - a stream argument of NULL means the null stream.
 *   - the library is re-entrant; the caller serialises use of one stream.
 */
#ifndef NEONHIP_H
#define NEONHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NH_ABI_VERSION 1
#define NH_RTC_ERROR_BASE 10000
#define NH_EINVAL 20001   /* bad argument caught on the host before any launch */
#define NH_ENOTINIT 20002 /* nh_init has not succeeded in this process */

typedef struct nh_props {
    char arch[64];            /* gcnArchName, e.g. "gfx950:sramecc+:xnack-" */
    char name[128];           /* marketing name */
    int32_t compute_units;
    int32_t wave_size;
    int32_t max_threads_per_block;
    int32_t lds_bytes_per_block;
    int32_t l2_bytes;
    int32_t clock_khz;
    int32_t mem_clock_khz;
    int32_t mem_bus_bits;
    uint64_t hbm_bytes;
} nh_props;

/* ---- device / context -----------------------------------------------------
 * replaces: drv.init / Device(id).make_context / ctx.detach
 *           (neon/backends/nervanagpu.py:748-752, 844-850) and the device probe
 *           neon/backends/util/check_gpu.py:21-105.                           */
int nh_abi_version(void);
int nh_device_count(int* count);
int nh_init(int device, nh_props* props);
int nh_shutdown(void);
int nh_device_sync(void);
const char* nh_last_error(void);

/* ---- memory ---------------------------------------------------------------
 * replaces: drv.mem_alloc (nervanagpu.py:87,147), DeviceAllocation.free (GC),
 *           drv.memcpy_htod_async / dtoh_async / dtod_async
 *           (nervanagpu.py:414, 428, 367), drv.memset_d8/d16/d32_async
 *           (nervanagpu.py:351-358), drv.mem_get_info.                        */
int nh_malloc(void** dptr, size_t bytes);
int nh_free(void* dptr);
int nh_mem_info(size_t* free_bytes, size_t* total_bytes);
int nh_memcpy_h2d(void* dst, const void* src, size_t bytes, void* stream);
int nh_memcpy_d2h(void* dst, const void* src, size_t bytes, void* stream);
int nh_memcpy_d2d(void* dst, const void* src, size_t bytes, void* stream);
int nh_memset_d8(void* dst, uint8_t value, size_t count, void* stream);
int nh_memset_d16(void* dst, uint16_t value, size_t count, void* stream);
int nh_memset_d32(void* dst, uint32_t value, size_t count, void* stream);
/* pinned host staging (the reference's use_pinned_mem path, nervanagpu.py:813-824) */
int nh_host_alloc(void** hptr, size_t bytes);
int nh_host_free(void* hptr);

/* ---- streams and events ---------------------------------------------------
 * replaces: the backend's single stream (nervanagpu.py:780) and drv.Event
 *           record / synchronize / time_since (nervanagpu.py:3138-3177).      */
int nh_stream_create(void** stream);
int nh_stream_destroy(void* stream);
int nh_stream_sync(void* stream);
int nh_event_create(void** event);
int nh_event_destroy(void* event);
int nh_event_record(void* event, void* stream);
int nh_event_sync(void* event);
int nh_event_elapsed_ms(void* start, void* stop, float* ms);

/* ---- run-time compilation ---------------------------------------------------
 * replaces: pycuda.compiler.SourceModule(code, options=...) and
 *           module.get_function(name) (neon/backends/float_ew.py:611-615;
 *           neon/backends/util/source_module.py:16-22).
 * nh_rtc_compile builds HIP C++ text for `arch` (NULL = the initialised
 * device's arch; an explicit arch needs no device at all).  On success *code
 * holds a code object of *code_bytes; *log (may be NULL) receives the compiler
 * log on success and failure.  Both buffers are released with nh_buf_free.    */
int nh_rtc_compile(const char* source, const char* name, const char* arch,
                   const char* const* options, int n_options,
                   void** code, size_t* code_bytes, char** log);
int nh_buf_free(void* buf);
int nh_module_load(const void* code, size_t code_bytes, void** module);
int nh_module_unload(void* module);
int nh_module_get_function(void* module, const char* name, void** function);

/* ---- launch -----------------------------------------------------------------
 * replaces: kernel.prepare(...) / kernel.prepared_async_call(grid, block,
 *           stream, *args, shared_size=) (float_ew.py:929-931).
 * `args` is the packed argument buffer laid out exactly as the kernel's
 * parameter list (natural alignment), `arg_bytes` its size.  Grid is in
 * blocks.  Dimensions are validated on the host (non-zero, block <= 1024
 * threads, LDS within the device limit) before anything is enqueued.          */
int nh_launch(void* function, const uint32_t grid[3], const uint32_t block[3],
              uint32_t lds_bytes, void* stream, const void* args, size_t arg_bytes);

/* The same launch from a record filled in once: a statement that is issued
 * again and again (an optimizer step, a layer's forward pass) re-uses its
 * record, and the call crosses the boundary with a single pointer.  The fields
 * are validated like nh_launch's arguments on every call (a handful of integer
 * compares).  `args` must stay valid and unchanged until the call returns.
 * replaces: kernel.prepare(signature) once + kernel.prepared_async_call(...)
 *           per launch (float_ew.py:612-615, 929-931).                          */
typedef struct nh_launch_rec {
    void* function;
    uint32_t grid[3];
    uint32_t block[3];
    uint32_t lds_bytes;
    uint32_t arg_bytes;
    void* stream;
    const void* args;
} nh_launch_rec;
int nh_launch_prepared(const nh_launch_rec* rec);

/* Launch the same kernel `reps` times back to back between two events on
 * `stream`, wait, and return the mean time per launch in milliseconds.
 * replaces: the event bracket of the reference's bench mode
 *           (float_ew.py:917-938: start.record / kernel / end.record /
 *           end.time_since(start)).                                            */
int nh_launch_timed(void* function, const uint32_t grid[3], const uint32_t block[3],
                    uint32_t lds_bytes, void* stream, const void* args, size_t arg_bytes,
                    uint32_t reps, float* mean_ms);

/* The same, cycling through `nsets` argument buffers (launch i uses
 * arg_sets[i % nsets]): with enough distinct tensors behind the sets every
 * launch finds its operands in HBM rather than in a cache.  The reference has
 * no counterpart; it is the cold-cache companion of the bench-mode bracket
 * above.                                                                       */
int nh_launch_timed_sets(void* function, const uint32_t grid[3], const uint32_t block[3],
                         uint32_t lds_bytes, void* stream, const void* const* arg_sets, size_t arg_bytes,
                         uint32_t nsets, uint32_t reps, float* mean_ms);

/* ---- prebuilt hand-written gfx950 kernels ------------------------------------
 * Direct entry points for fixed, hot op-trees; the same trees also run through
 * the generated-code path.  All pointers are device pointers; tensors are
 * row-major and contiguous unless a leading dimension is given.               */

/* out = alpha*x + beta*y over n fp32 elements; the tree `a*x + b*y`
 * (first assign of the elementwise configuration).                             */
int nh_ew_axpby_f32(float* out, const float* x, const float* y, float alpha,
                    float beta, size_t n, void* stream);
/* x = 1/(1+exp(-x)) in place over n fp32 elements (the `sig` op,
 * neon/backends/nervanacpu.py:493).                                            */
int nh_ew_sigmoid_f32(float* out, const float* x, size_t n, void* stream);

/* One fused Adam step over n fp32 elements, the three assigns of
 * Adam.optimize (neon/optimizers/optimizer.py:925-930) in one pass:
 *   m = m*beta1 + (1-beta1)*g ; v = v*beta2 + (1-beta2)*g*g ;
 *   p = p - (lr_t*m)/(sqrt(v)+eps)        with lr_t folded by the caller.
 * `one_minus_beta1/2` are passed separately so the caller decides how the
 * constants are rounded (the CPU path rounds 1-beta in double, then to fp32).  */
int nh_adam_step_f32(float* param, float* m, float* v, const float* grad,
                     float lr_t, float beta1, float one_minus_beta1,
                     float beta2, float one_minus_beta2, float eps,
                     size_t n, void* stream);

/* Row-wise normalisation of an fp16 matrix with fp32 statistics, the op-tree
 *   out = gamma*(x-mean)/sqrt(var+eps)+beta, mean/var over axis 1 (biased,
 *   two-pass) -- BatchNormAutodiff.get_forward_optree
 *   (neon/layers/layer.py:2592-2600).  x/out are (rows, cols) fp16 with row
 *   pitch `ld` elements; gamma/beta are fp32 (rows).  x is read once.
 *   cols must be <= NH_ROWNORM_MAX_COLS.                                       */
#define NH_ROWNORM_MAX_COLS (1024 * 8 * 16)
int nh_rownorm_f16(uint16_t* out, const uint16_t* x, const float* gamma,
                   const float* beta, float eps, uint32_t rows, uint32_t cols,
                   size_t ld, void* stream);

/* Column reductions of an fp32 (rows, cols) matrix along axis 0:
 *   maxval[c] = max_r x[r,c] (may be NULL), argmax[c] = first r attaining it
 *   (may be NULL) -- the `max` / `argmax` reduction ops
 *   (neon/backends/nervanacpu.py:517-521; Misclassification,
 *   neon/transforms/cost.py:421-423).
 * `workspace` is device memory of nh_colreduce_workspace_bytes(rows, cols)
 * bytes; it is scratch, need not be initialised.                               */
size_t nh_colreduce_workspace_bytes(uint32_t rows, uint32_t cols);
int nh_colmax_argmax_f32(float* maxval, int32_t* argmax, const float* x,
                         uint32_t rows, uint32_t cols, size_t ld,
                         void* workspace, void* stream);

/* The same reduction for callers that cannot allocate device memory (code
 * under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc): no workspace argument and no allocation of any kind -- the
 * partials and tickets live in a static device array of
 * NH_STATIC_SCRATCH_BYTES that every device holds from library load until the
 * process ends.  There is no counterpart in the reference (PyCUDA allocates
 * freely; neon/backends/nervanagpu.py:87,147).  Shapes whose partials do not
 * fit (256 KiB of tickets, a 64-byte line per column strip, + row chunks *
 * cols * 8 bytes; the launch geometry keeps that within the array for every
 * matrix whose row length is a multiple of four, and for other row lengths
 * up to about 6000 columns) are refused
 * with NH_EINVAL before anything is launched.  All calls on one device
 * share the array: calls that overlap in time on one device (different
 * streams or threads) race; calls on one stream are safe back to back (the
 * tickets are cleared by a small kernel ahead of the reduction, so the call
 * can be recorded into a graph).                                             */
#define NH_STATIC_SCRATCH_BYTES (1u << 20)
int nh_colmax_argmax_f32_static(float* maxval, int32_t* argmax, const float* x,
                                uint32_t rows, uint32_t cols, size_t ld, void* stream);

/* 64-bin (nbins <= 256) histogram of rint(log2|x|) over n contiguous fp32
 * (itemsize 4) or fp16 (itemsize 2) elements into hist[nbins] (cleared
 * first): bin 0 reaches down to -inf, bin k >= 1 holds offset+k, the last bin
 * also offset+nbins, larger magnitudes and NaN are not counted -- the binning
 * of Tensor.hist on the CPU backend (neon/backends/nervanacpu.py:424-445);
 * replaces kernel_histo / _compute_hist (neon/backends/float_ew.py:1070-1158).
 * rint(log2|x|) is taken from the exponent and mantissa bits, i.e. correctly
 * rounded: for the two fp32 neighbours of sqrt(2) * 2^k a log2f-based binning
 * decides by the last bit of its logarithm.                                  */
int nh_hist_log2(int32_t* hist, const void* x, int itemsize, size_t n, int nbins,
                 int offset, void* stream);

/* Dense contraction hand-off: C[m,n] = alpha * op(A) * op(B) + beta * C on
 * row-major operands; op(X) = X^T when trans_x != 0; lda/ldb/ldc = elements
 * between consecutive stored rows; itemsize 4 = fp32, 2 = fp16 storage with
 * fp32 accumulation.  Forwards to rocBLAS (opened on first use).  Replaces the
 * library GEMM behind NervanaGPU.compound_dot / cublas_dot
 * (neon/backends/nervanagpu.py:1441-1470, 3012-3044), which `dot` nodes inside
 * op-trees are staged through (nervanagpu.py:1099-1237).                      */
int nh_gemm(int itemsize, int trans_a, int trans_b, uint32_t m, uint32_t n, uint32_t k,
            float alpha, const void* a, size_t lda, const void* b, size_t ldb,
            float beta, void* c, size_t ldc, void* stream);

/* `batch` such products in one call: product i reads a + i * stride_a and
 * b + i * stride_b and updates c + i * stride_c (strides in elements; 0 for an
 * operand shared by the whole batch; the outputs must not overlap).  Replaces
 * the batched sgemm/hgemm kernels behind NervanaGPU.batched_dot
 * (neon/backends/nervanagpu.py:1623-1760).                                      */
int nh_gemm_batched(int itemsize, int trans_a, int trans_b, uint32_t m, uint32_t n, uint32_t k,
                    float alpha, const void* a, size_t lda, long long stride_a, const void* b, size_t ldb,
                    long long stride_b, float beta, void* c, size_t ldc, long long stride_c,
                    uint32_t batch, void* stream);

/* Dimension shuffle, numpy.transpose(in, axes) written into `out`: `ndim`
 * dimensions listed in OUTPUT order -- shape[i] is the extent of output
 * dimension i, out_strides[i] its stride in `out` and in_strides[i] the stride
 * of the input dimension it comes from (axes[i]), all in elements and
 * non-negative.  Elements are moved as opaque `itemsize`-byte values (1, 2, 4
 * or 8).  `out` and `in` must not overlap.  Replaces
 * NervanaGPU.copy_transpose / _get_copy_transpose_kernel
 * (neon/backends/nervanagpu.py:3077-3118).                                      */
#define NH_TRANSPOSE_MAX_DIMS 8
int nh_copy_transpose(void* out, const void* in, int itemsize, int ndim, const uint32_t* shape,
                      const int64_t* out_strides, const int64_t* in_strides, void* stream);

/* Lookup-table (embedding) backward pass: dW[w, 0:embed] = sum over the
 * positions j with ids[j] == w of error_t[j, 0:embed], positions in ascending
 * order (deterministic); rows of words that do not occur, of `pad_idx` and of
 * ids >= vocab are left untouched.  `ids` holds nin int32 word ids, error_t is
 * the (nin, embed) transposed error, dW the (vocab, embed) gradient, both of
 * `itemsize` 4 (fp32) or 2 (fp16, fp32 accumulation) with leading dimensions
 * in elements.  `workspace` is device scratch of nh_lut_workspace_bytes(nin,
 * vocab) bytes (0 from that call means the size query failed).  Replaces the
 * sorting + _get_lut_bprop_kernel sequence of NervanaGPU.compound_bprop_lut
 * (neon/backends/nervanagpu.py:2591-2660); semantics of the CPU backend
 * (neon/backends/nervanacpu.py:1762-1782).                                     */
size_t nh_lut_workspace_bytes(uint32_t nin, uint32_t vocab);
int nh_lut_bprop(void* dW, const void* error_t, const int32_t* ids, int itemsize, uint32_t nin, uint32_t embed,
                 uint32_t vocab, size_t ld_dw, size_t ld_err, int32_t pad_idx, void* workspace, size_t workspace_bytes,
                 void* stream);

#ifdef __cplusplus
}
#endif
#endif /* NEONHIP_H */
