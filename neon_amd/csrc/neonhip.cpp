// libneonhip.so -- C-ABI device shim of the `hip` backend (see include/neonhip.h).
//
// Thin, stateless wrappers over the HIP runtime, hiprtc and the module API.
// Every entry point validates its arguments on the host, converts any failure
// into an error code plus a thread-local message, and never throws.
#include "neonhip.h"

#include <hip/hip_runtime.h>
#include <hip/hiprtc.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

void nh_internal_blas_release();      // gemm.cpp: drops the rocBLAS handle, if one was created
int nh_internal_scratch_setup(int device);   // kernels.hip: per-device address of the static scratch area

namespace {

thread_local std::string g_err;
bool g_init = false;
int g_device = -1;
hipDeviceProp_t g_prop;

int fail(int code, const std::string& msg) {
    g_err = msg;
    return code;
}

int hip_fail(hipError_t e, const char* what) {
    // clear the sticky "last error" so that it is not reported again by an
    // unrelated later call
    (void)hipGetLastError();
    return fail((int)e, std::string(what) + ": " + hipGetErrorString(e));
}

#define NH_HIP(call)                                   \
    do {                                               \
        hipError_t e_ = (call);                        \
        if (e_ != hipSuccess) return hip_fail(e_, #call); \
    } while (0)

#define NH_NEED_INIT()                                                     \
    do {                                                                   \
        if (!g_init) return fail(NH_ENOTINIT, "nh_init has not been called"); \
    } while (0)

}  // namespace

extern "C" {

int nh_abi_version(void) { return NH_ABI_VERSION; }

const char* nh_last_error(void) { return g_err.c_str(); }

int nh_device_count(int* count) {
    if (!count) return fail(NH_EINVAL, "nh_device_count: null output");
    *count = 0;
    hipError_t e = hipGetDeviceCount(count);
    if (e != hipSuccess) {
        *count = 0;
        return hip_fail(e, "hipGetDeviceCount");
    }
    return 0;
}

int nh_init(int device, nh_props* props) {
    int n = 0;
    int rc = nh_device_count(&n);
    if (rc) return rc;
    if (device < 0 || device >= n)
        return fail(NH_EINVAL, "nh_init: device " + std::to_string(device) + " out of range (" +
                                   std::to_string(n) + " visible)");
    NH_HIP(hipSetDevice(device));
    NH_HIP(hipGetDeviceProperties(&g_prop, device));
    NH_HIP(hipFree(nullptr));  // force context creation now, not inside a timed region
    g_device = device;
    g_init = true;
    if (int rc = nh_internal_scratch_setup(device)) {
        g_init = false;
        return rc;
    }
    if (props) {
        std::memset(props, 0, sizeof(*props));
        std::snprintf(props->arch, sizeof(props->arch), "%s", g_prop.gcnArchName);
        std::snprintf(props->name, sizeof(props->name), "%s", g_prop.name);
        props->compute_units = g_prop.multiProcessorCount;
        props->wave_size = g_prop.warpSize;
        props->max_threads_per_block = g_prop.maxThreadsPerBlock;
        props->lds_bytes_per_block = (int32_t)g_prop.sharedMemPerBlock;
        props->l2_bytes = g_prop.l2CacheSize;
        props->clock_khz = g_prop.clockRate;
        props->mem_clock_khz = g_prop.memoryClockRate;
        props->mem_bus_bits = g_prop.memoryBusWidth;
        props->hbm_bytes = g_prop.totalGlobalMem;
    }
    return 0;
}

int nh_shutdown(void) {
    if (!g_init) return 0;
    NH_HIP(hipDeviceSynchronize());
    nh_internal_blas_release();
    g_init = false;
    return 0;
}

int nh_device_sync(void) {
    NH_NEED_INIT();
    NH_HIP(hipDeviceSynchronize());
    return 0;
}

// ---- memory -----------------------------------------------------------------

int nh_malloc(void** dptr, size_t bytes) {
    NH_NEED_INIT();
    if (!dptr) return fail(NH_EINVAL, "nh_malloc: null output");
    *dptr = nullptr;
    if (bytes == 0) return fail(NH_EINVAL, "nh_malloc: zero bytes");
    if (bytes > g_prop.totalGlobalMem)
        return fail((int)hipErrorOutOfMemory, "nh_malloc: " + std::to_string(bytes) +
                                                  " bytes exceeds device memory");
    NH_HIP(hipMalloc(dptr, bytes));
    return 0;
}

int nh_free(void* dptr) {
    if (!dptr) return 0;
    NH_NEED_INIT();
    NH_HIP(hipFree(dptr));
    return 0;
}

int nh_mem_info(size_t* free_bytes, size_t* total_bytes) {
    NH_NEED_INIT();
    size_t f = 0, t = 0;
    NH_HIP(hipMemGetInfo(&f, &t));
    if (free_bytes) *free_bytes = f;
    if (total_bytes) *total_bytes = t;
    return 0;
}

static int copy(void* dst, const void* src, size_t bytes, void* stream, hipMemcpyKind kind, bool wait) {
    NH_NEED_INIT();
    if (bytes == 0) return 0;
    if (!dst || !src) return fail(NH_EINVAL, "nh_memcpy: null pointer");
    hipStream_t s = (hipStream_t)stream;
    NH_HIP(hipMemcpyAsync(dst, src, bytes, kind, s));
    // Host buffers handed over by the caller are pageable: the call returns
    // only when the bytes have left (or reached) them.
    if (wait) NH_HIP(hipStreamSynchronize(s));
    return 0;
}

int nh_memcpy_h2d(void* dst, const void* src, size_t bytes, void* stream) {
    return copy(dst, src, bytes, stream, hipMemcpyHostToDevice, true);
}
int nh_memcpy_d2h(void* dst, const void* src, size_t bytes, void* stream) {
    return copy(dst, src, bytes, stream, hipMemcpyDeviceToHost, true);
}
int nh_memcpy_d2d(void* dst, const void* src, size_t bytes, void* stream) {
    return copy(dst, src, bytes, stream, hipMemcpyDeviceToDevice, false);
}

int nh_memset_d8(void* dst, uint8_t value, size_t count, void* stream) {
    NH_NEED_INIT();
    if (count == 0) return 0;
    if (!dst) return fail(NH_EINVAL, "nh_memset_d8: null pointer");
    NH_HIP(hipMemsetD8Async((hipDeviceptr_t)dst, value, count, (hipStream_t)stream));
    return 0;
}
int nh_memset_d16(void* dst, uint16_t value, size_t count, void* stream) {
    NH_NEED_INIT();
    if (count == 0) return 0;
    if (!dst) return fail(NH_EINVAL, "nh_memset_d16: null pointer");
    NH_HIP(hipMemsetD16Async((hipDeviceptr_t)dst, value, count, (hipStream_t)stream));
    return 0;
}
int nh_memset_d32(void* dst, uint32_t value, size_t count, void* stream) {
    NH_NEED_INIT();
    if (count == 0) return 0;
    if (!dst) return fail(NH_EINVAL, "nh_memset_d32: null pointer");
    NH_HIP(hipMemsetD32Async((hipDeviceptr_t)dst, (int)value, count, (hipStream_t)stream));
    return 0;
}

int nh_host_alloc(void** hptr, size_t bytes) {
    NH_NEED_INIT();
    if (!hptr || bytes == 0) return fail(NH_EINVAL, "nh_host_alloc: bad argument");
    NH_HIP(hipHostMalloc(hptr, bytes, hipHostMallocDefault));
    return 0;
}
int nh_host_free(void* hptr) {
    if (!hptr) return 0;
    NH_NEED_INIT();
    NH_HIP(hipHostFree(hptr));
    return 0;
}

// ---- streams and events -------------------------------------------------------

int nh_stream_create(void** stream) {
    NH_NEED_INIT();
    if (!stream) return fail(NH_EINVAL, "nh_stream_create: null output");
    hipStream_t s;
    NH_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));  // default priority
    *stream = (void*)s;
    return 0;
}
int nh_stream_destroy(void* stream) {
    if (!stream) return 0;
    NH_NEED_INIT();
    NH_HIP(hipStreamDestroy((hipStream_t)stream));
    return 0;
}
int nh_stream_sync(void* stream) {
    NH_NEED_INIT();
    NH_HIP(hipStreamSynchronize((hipStream_t)stream));
    return 0;
}
int nh_event_create(void** event) {
    NH_NEED_INIT();
    if (!event) return fail(NH_EINVAL, "nh_event_create: null output");
    hipEvent_t e;
    NH_HIP(hipEventCreate(&e));
    *event = (void*)e;
    return 0;
}
int nh_event_destroy(void* event) {
    if (!event) return 0;
    NH_NEED_INIT();
    NH_HIP(hipEventDestroy((hipEvent_t)event));
    return 0;
}
int nh_event_record(void* event, void* stream) {
    NH_NEED_INIT();
    if (!event) return fail(NH_EINVAL, "nh_event_record: null event");
    NH_HIP(hipEventRecord((hipEvent_t)event, (hipStream_t)stream));
    return 0;
}
int nh_event_sync(void* event) {
    NH_NEED_INIT();
    if (!event) return fail(NH_EINVAL, "nh_event_sync: null event");
    NH_HIP(hipEventSynchronize((hipEvent_t)event));
    return 0;
}
int nh_event_elapsed_ms(void* start, void* stop, float* ms) {
    NH_NEED_INIT();
    if (!start || !stop || !ms) return fail(NH_EINVAL, "nh_event_elapsed_ms: null argument");
    NH_HIP(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
    return 0;
}

// ---- run-time compilation -------------------------------------------------------

static int rtc_fail(hiprtcResult r, const char* what) {
    return fail(NH_RTC_ERROR_BASE + (int)r, std::string(what) + ": " + hiprtcGetErrorString(r));
}

int nh_rtc_compile(const char* source, const char* name, const char* arch,
                   const char* const* options, int n_options,
                   void** code, size_t* code_bytes, char** log) {
    if (!source || !code || !code_bytes) return fail(NH_EINVAL, "nh_rtc_compile: null argument");
    if (n_options < 0 || (n_options > 0 && !options)) return fail(NH_EINVAL, "nh_rtc_compile: bad options");
    *code = nullptr;
    *code_bytes = 0;
    if (log) *log = nullptr;

    std::string arch_opt = "--offload-arch=";
    if (arch && arch[0]) {
        arch_opt += arch;
    } else {
        if (!g_init) return fail(NH_ENOTINIT, "nh_rtc_compile: no arch given and no device initialised");
        arch_opt += g_prop.gcnArchName;
    }
    std::vector<const char*> opts;
    opts.push_back(arch_opt.c_str());
    for (int i = 0; i < n_options; ++i) opts.push_back(options[i]);

    hiprtcProgram prog;
    hiprtcResult r = hiprtcCreateProgram(&prog, source, name ? name : "optree.hip", 0, nullptr, nullptr);
    if (r != HIPRTC_SUCCESS) return rtc_fail(r, "hiprtcCreateProgram");

    hiprtcResult cr = hiprtcCompileProgram(prog, (int)opts.size(), opts.data());
    size_t log_size = 0;
    std::string log_text;
    if (hiprtcGetProgramLogSize(prog, &log_size) == HIPRTC_SUCCESS && log_size > 1) {
        log_text.resize(log_size);
        if (hiprtcGetProgramLog(prog, &log_text[0]) != HIPRTC_SUCCESS) log_text.clear();
    }
    if (log && !log_text.empty()) {
        *log = (char*)std::malloc(log_text.size() + 1);
        if (*log) std::memcpy(*log, log_text.c_str(), log_text.size() + 1);
    }
    if (cr != HIPRTC_SUCCESS) {
        hiprtcDestroyProgram(&prog);
        return fail(NH_RTC_ERROR_BASE + (int)cr,
                    std::string("hiprtcCompileProgram: ") + hiprtcGetErrorString(cr) + "\n" + log_text);
    }
    size_t sz = 0;
    r = hiprtcGetCodeSize(prog, &sz);
    if (r != HIPRTC_SUCCESS || sz == 0) {
        hiprtcDestroyProgram(&prog);
        return rtc_fail(r, "hiprtcGetCodeSize");
    }
    void* buf = std::malloc(sz);
    if (!buf) {
        hiprtcDestroyProgram(&prog);
        return fail((int)hipErrorOutOfMemory, "nh_rtc_compile: host allocation failed");
    }
    r = hiprtcGetCode(prog, (char*)buf);
    hiprtcDestroyProgram(&prog);
    if (r != HIPRTC_SUCCESS) {
        std::free(buf);
        return rtc_fail(r, "hiprtcGetCode");
    }
    *code = buf;
    *code_bytes = sz;
    return 0;
}

int nh_buf_free(void* buf) {
    std::free(buf);
    return 0;
}

int nh_module_load(const void* code, size_t code_bytes, void** module) {
    NH_NEED_INIT();
    if (!code || code_bytes == 0 || !module) return fail(NH_EINVAL, "nh_module_load: bad argument");
    hipModule_t m;
    NH_HIP(hipModuleLoadData(&m, code));
    *module = (void*)m;
    return 0;
}
int nh_module_unload(void* module) {
    if (!module) return 0;
    NH_NEED_INIT();
    NH_HIP(hipModuleUnload((hipModule_t)module));
    return 0;
}
int nh_module_get_function(void* module, const char* name, void** function) {
    NH_NEED_INIT();
    if (!module || !name || !function) return fail(NH_EINVAL, "nh_module_get_function: null argument");
    hipFunction_t f;
    NH_HIP(hipModuleGetFunction(&f, (hipModule_t)module, name));
    *function = (void*)f;
    return 0;
}

// ---- launch -------------------------------------------------------------------------

int nh_launch(void* function, const uint32_t grid[3], const uint32_t block[3],
              uint32_t lds_bytes, void* stream, const void* args, size_t arg_bytes) {
    NH_NEED_INIT();
    if (!function) return fail(NH_EINVAL, "nh_launch: null function");
    if (!grid || !block) return fail(NH_EINVAL, "nh_launch: null dimensions");
    for (int i = 0; i < 3; ++i)
        if (grid[i] == 0 || block[i] == 0) return fail(NH_EINVAL, "nh_launch: zero dimension");
    const uint64_t threads = (uint64_t)block[0] * block[1] * block[2];
    if (threads > (uint64_t)g_prop.maxThreadsPerBlock)
        return fail(NH_EINVAL, "nh_launch: " + std::to_string(threads) + " threads per block exceeds " +
                                   std::to_string(g_prop.maxThreadsPerBlock));
    if (grid[1] > 65535u || grid[2] > 65535u || (uint64_t)grid[0] * block[0] > 0xFFFFFFFFull)
        return fail(NH_EINVAL, "nh_launch: grid too large");
    if (lds_bytes > (uint32_t)g_prop.sharedMemPerBlock)
        return fail(NH_EINVAL, "nh_launch: LDS request exceeds the per-block limit");
    if (arg_bytes > 4096 || (arg_bytes > 0 && !args)) return fail(NH_EINVAL, "nh_launch: bad argument buffer");
    size_t sz = arg_bytes;
    void* config[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, const_cast<void*>(args),
                      HIP_LAUNCH_PARAM_BUFFER_SIZE, &sz, HIP_LAUNCH_PARAM_END};
    NH_HIP(hipModuleLaunchKernel((hipFunction_t)function, grid[0], grid[1], grid[2], block[0], block[1],
                                 block[2], lds_bytes, (hipStream_t)stream, nullptr, config));
    return 0;
}

int nh_launch_prepared(const nh_launch_rec* rec) {
    if (!rec) return fail(NH_EINVAL, "nh_launch_prepared: null record");
    return nh_launch(rec->function, rec->grid, rec->block, rec->lds_bytes, rec->stream, rec->args, rec->arg_bytes);
}

int nh_launch_timed_sets(void* function, const uint32_t grid[3], const uint32_t block[3],
                         uint32_t lds_bytes, void* stream, const void* const* arg_sets, size_t arg_bytes,
                         uint32_t nsets, uint32_t reps, float* mean_ms) {
    NH_NEED_INIT();
    if (!mean_ms || reps == 0 || nsets == 0 || !arg_sets) return fail(NH_EINVAL, "nh_launch_timed_sets: bad argument");
    *mean_ms = 0.0f;
    hipEvent_t e0, e1;
    NH_HIP(hipEventCreate(&e0));
    hipError_t err = hipEventCreate(&e1);
    if (err != hipSuccess) {
        (void)hipEventDestroy(e0);
        return hip_fail(err, "hipEventCreate");
    }
    int rc = 0;
    hipStream_t s = (hipStream_t)stream;
    err = hipEventRecord(e0, s);
    if (err != hipSuccess) rc = hip_fail(err, "hipEventRecord");
    for (uint32_t i = 0; rc == 0 && i < reps; ++i)
        rc = nh_launch(function, grid, block, lds_bytes, stream, arg_sets[i % nsets], arg_bytes);
    if (rc == 0) {
        err = hipEventRecord(e1, s);
        if (err == hipSuccess) err = hipEventSynchronize(e1);
        float ms = 0.0f;
        if (err == hipSuccess) err = hipEventElapsedTime(&ms, e0, e1);
        if (err != hipSuccess) rc = hip_fail(err, "nh_launch_timed_sets: event timing");
        else *mean_ms = ms / (float)reps;
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    return rc;
}

int nh_launch_timed(void* function, const uint32_t grid[3], const uint32_t block[3],
                    uint32_t lds_bytes, void* stream, const void* args, size_t arg_bytes,
                    uint32_t reps, float* mean_ms) {
    const void* one[1] = {args};
    return nh_launch_timed_sets(function, grid, block, lds_bytes, stream, one, arg_bytes, 1, reps, mean_ms);
}

}  // extern "C"

// Shared with kernels.hip (same library, not part of the ABI).
bool nh_internal_ready() { return g_init; }
int nh_internal_fail(int code, const char* msg) { return fail(code, msg); }
int nh_internal_cu_count() { return g_init ? g_prop.multiProcessorCount : 0; }
int nh_internal_device() { return g_init ? g_device : -1; }
