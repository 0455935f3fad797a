// Dense contraction hand-off of libneonhip.so: nh_gemm forwards one row-major
// GEMM to rocBLAS, nh_gemm_batched a strided batch of them.  The library is
// opened on the first call, so processes that only run op-trees never load it.
#include "neonhip.h"

#include <hip/hip_runtime.h>
#include <rocblas/rocblas.h>

#include <dlfcn.h>

#include <mutex>
#include <string>

bool nh_internal_ready();
int nh_internal_fail(int code, const char* msg);

namespace {

struct Blas {
    void* lib = nullptr;
    rocblas_handle handle = nullptr;
    decltype(&rocblas_create_handle) create = nullptr;
    decltype(&rocblas_destroy_handle) destroy = nullptr;
    decltype(&rocblas_set_stream) set_stream = nullptr;
    decltype(&rocblas_set_pointer_mode) set_pointer_mode = nullptr;
    decltype(&rocblas_gemm_ex) gemm_ex = nullptr;
    decltype(&rocblas_gemm_strided_batched_ex) gemm_batched_ex = nullptr;
    std::string error;
    bool tried = false;
};

Blas g_blas;
std::mutex g_blas_mutex;

template <typename F>
bool bind(F& fn, const char* name) {
    fn = reinterpret_cast<F>(dlsym(g_blas.lib, name));
    if (!fn) g_blas.error = std::string("librocblas lacks ") + name;
    return fn != nullptr;
}

// caller holds g_blas_mutex
bool blas_ready() {
    if (g_blas.handle) return true;
    if (g_blas.tried) return false;
    g_blas.tried = true;
    if (g_blas.lib && g_blas.create) {            // library already bound: only the handle was released
        if (g_blas.create(&g_blas.handle) != rocblas_status_success) {
            g_blas.handle = nullptr;
            g_blas.error = "rocblas_create_handle failed";
            return false;
        }
        g_blas.set_pointer_mode(g_blas.handle, rocblas_pointer_mode_host);
        return true;
    }
    for (const char* name : {"librocblas.so.5", "librocblas.so", "/opt/rocm/lib/librocblas.so"}) {
        g_blas.lib = dlopen(name, RTLD_NOW | RTLD_LOCAL);
        if (g_blas.lib) break;
    }
    if (!g_blas.lib) {
        const char* why = dlerror();
        g_blas.error = std::string("cannot open librocblas: ") + (why ? why : "unknown");
        return false;
    }
    if (!bind(g_blas.create, "rocblas_create_handle") || !bind(g_blas.destroy, "rocblas_destroy_handle") ||
        !bind(g_blas.set_stream, "rocblas_set_stream") ||
        !bind(g_blas.set_pointer_mode, "rocblas_set_pointer_mode") || !bind(g_blas.gemm_ex, "rocblas_gemm_ex") ||
        !bind(g_blas.gemm_batched_ex, "rocblas_gemm_strided_batched_ex"))
        return false;
    rocblas_status st = g_blas.create(&g_blas.handle);
    if (st != rocblas_status_success) {
        g_blas.handle = nullptr;
        g_blas.error = "rocblas_create_handle failed with status " + std::to_string((int)st);
        return false;
    }
    g_blas.set_pointer_mode(g_blas.handle, rocblas_pointer_mode_host);
    return true;
}

}  // namespace

// called by nh_shutdown: the handle belongs to the device context being left
void nh_internal_blas_release() {
    std::lock_guard<std::mutex> hold(g_blas_mutex);
    if (g_blas.handle && g_blas.destroy) g_blas.destroy(g_blas.handle);
    g_blas.handle = nullptr;
    g_blas.tried = false;
}

namespace {

// batch == 0: one product through gemm_ex; otherwise `batch` products whose
// operands lie stride_x elements apart (0 = the same matrix every time)
int gemm_impl(const char* who, int itemsize, int trans_a, int trans_b, uint32_t m, uint32_t n, uint32_t k, float alpha,
              const void* a, size_t lda, long long stride_a, const void* b, size_t ldb, long long stride_b, float beta,
              void* c, size_t ldc, long long stride_c, uint32_t batch, void* stream) {
    const std::string tag = std::string(who) + ": ";
    if (!nh_internal_ready()) return nh_internal_fail(NH_ENOTINIT, "nh_init has not been called");
    if (itemsize != 4 && itemsize != 2)
        return nh_internal_fail(NH_EINVAL, (tag + "itemsize must be 4 (fp32) or 2 (fp16)").c_str());
    if (m == 0 || n == 0) return 0;
    if (!a || !b || !c) return nh_internal_fail(NH_EINVAL, (tag + "null operand").c_str());
    const size_t int_max = 0x7fffffff;
    if (m > int_max || n > int_max || k > int_max || lda > int_max || ldb > int_max || ldc > int_max || batch > int_max)
        return nh_internal_fail(NH_EINVAL, (tag + "extent beyond 2^31-1").c_str());
    if (stride_a < 0 || stride_b < 0 || stride_c < 0) return nh_internal_fail(NH_EINVAL, (tag + "negative stride").c_str());
    // leading dimensions are elements per stored row
    const size_t need_a = trans_a ? m : k, need_b = trans_b ? k : n;
    if (lda < (need_a ? need_a : 1) || ldb < (need_b ? need_b : 1) || ldc < n)
        return nh_internal_fail(NH_EINVAL, (tag + "leading dimension shorter than a stored row").c_str());
    if (batch > 1 && (size_t)stride_c < (size_t)(m - 1) * ldc + n)
        return nh_internal_fail(NH_EINVAL, (tag + "outputs of the batch overlap").c_str());

    std::lock_guard<std::mutex> hold(g_blas_mutex);
    if (!blas_ready()) return nh_internal_fail(NH_EINVAL, (tag + g_blas.error).c_str());
    rocblas_status st = g_blas.set_stream(g_blas.handle, (hipStream_t)stream);
    if (st != rocblas_status_success) return nh_internal_fail(NH_EINVAL, (tag + "rocblas_set_stream failed").c_str());
    // A row-major matrix is its transpose in column-major storage, so
    // C = op(A) op(B) becomes C^T = op(B)^T op(A)^T: operands swap places and
    // keep their flags.
    const rocblas_datatype t = itemsize == 4 ? rocblas_datatype_f32_r : rocblas_datatype_f16_r;
    const rocblas_operation op_b = trans_b ? rocblas_operation_transpose : rocblas_operation_none;
    const rocblas_operation op_a = trans_a ? rocblas_operation_transpose : rocblas_operation_none;
    if (batch == 0)
        st = g_blas.gemm_ex(g_blas.handle, op_b, op_a, (rocblas_int)n, (rocblas_int)m, (rocblas_int)k, &alpha,
                            b, t, (rocblas_int)ldb, a, t, (rocblas_int)lda, &beta,
                            c, t, (rocblas_int)ldc, c, t, (rocblas_int)ldc,
                            rocblas_datatype_f32_r, rocblas_gemm_algo_standard, 0, 0);
    else
        st = g_blas.gemm_batched_ex(g_blas.handle, op_b, op_a, (rocblas_int)n, (rocblas_int)m, (rocblas_int)k, &alpha,
                                    b, t, (rocblas_int)ldb, (rocblas_stride)stride_b,
                                    a, t, (rocblas_int)lda, (rocblas_stride)stride_a, &beta,
                                    c, t, (rocblas_int)ldc, (rocblas_stride)stride_c,
                                    c, t, (rocblas_int)ldc, (rocblas_stride)stride_c, (rocblas_int)batch,
                                    rocblas_datatype_f32_r, rocblas_gemm_algo_standard, 0, 0);
    if (st != rocblas_status_success)
        return nh_internal_fail(NH_EINVAL, (tag + "rocBLAS failed with status " + std::to_string((int)st)).c_str());
    return 0;
}

}  // namespace

extern "C" int nh_gemm(int itemsize, int trans_a, int trans_b, uint32_t m, uint32_t n, uint32_t k,
                       float alpha, const void* a, size_t lda, const void* b, size_t ldb,
                       float beta, void* c, size_t ldc, void* stream) {
    return gemm_impl("nh_gemm", itemsize, trans_a, trans_b, m, n, k, alpha, a, lda, 0, b, ldb, 0, beta, c, ldc, 0, 0,
                     stream);
}

extern "C" int nh_gemm_batched(int itemsize, int trans_a, int trans_b, uint32_t m, uint32_t n, uint32_t k,
                               float alpha, const void* a, size_t lda, long long stride_a, const void* b, size_t ldb,
                               long long stride_b, float beta, void* c, size_t ldc, long long stride_c,
                               uint32_t batch, void* stream) {
    if (batch == 0) return 0;
    return gemm_impl("nh_gemm_batched", itemsize, trans_a, trans_b, m, n, k, alpha, a, lda, stride_a, b, ldb, stride_b,
                     beta, c, ldc, stride_c, batch, stream);
}
