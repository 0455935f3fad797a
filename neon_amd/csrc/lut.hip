// Lookup-table (embedding) backward pass: dW[w, :] = sum of the error rows of
// all positions whose word id is w.  Deterministic: positions are sorted by
// word id with a stable device radix sort (rocPRIM), then every run of equal
// ids is summed in position order by one wave -- no floating-point atomics.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstring>

#include <rocprim/device/device_radix_sort.hpp>
#include <rocprim/iterator/counting_iterator.hpp>

#include "neonhip.h"
#include "device/neon_device.h"

bool nh_internal_ready();
int nh_internal_fail(int code, const char* msg);

namespace {

constexpr int LUT_T = 256;
constexpr int LUT_WAVES = LUT_T / 64;

size_t align256(size_t x) { return (x + 255) / 256 * 256; }

int key_bits(uint32_t vocab) {
    int bits = 1;
    while (bits < 32 && (1ull << bits) < (unsigned long long)vocab) ++bits;
    return bits;
}

hipError_t sort_positions(void* temp, size_t& temp_bytes, const uint32_t* ids, uint32_t* keys, uint32_t* pos,
                          uint32_t nin, uint32_t vocab, hipStream_t s) {
    return rocprim::radix_sort_pairs(temp, temp_bytes, ids, keys, rocprim::counting_iterator<uint32_t>(0), pos, nin, 0,
                                     key_bits(vocab), s);
}

// wave `i` of the grid looks at sorted slot i; if a run of equal ids starts
// there it sums the run's error rows, lanes across the embedding columns
template <typename T>
__global__ __launch_bounds__(LUT_T) void lut_bprop_kernel(T* __restrict__ dW, const T* __restrict__ err_t,
                                                          const uint32_t* __restrict__ keys,
                                                          const uint32_t* __restrict__ pos, uint32_t nin, uint32_t embed,
                                                          uint32_t vocab, size_t ld_dw, size_t ld_err, int32_t pad_idx) {
    const uint32_t i = blockIdx.x * LUT_WAVES + threadIdx.x / 64;
    const uint32_t lane = threadIdx.x & 63;
    if (i >= nin) return;
    const uint32_t key = keys[i];
    if (i > 0 && keys[i - 1] == key) return;
    if ((int32_t)key == pad_idx || key >= vocab) return;
    for (uint32_t c = lane; c < embed; c += 64) {
        float acc = 0.0f;
        for (uint32_t k = i; k < nin && keys[k] == key; ++k) acc += (float)err_t[(size_t)pos[k] * ld_err + c];
        dW[(size_t)key * ld_dw + c] = (T)acc;
    }
}

}  // namespace

extern "C" {

size_t nh_lut_workspace_bytes(uint32_t nin, uint32_t vocab) {
    if (nin == 0) return 0;
    size_t temp = 0;
    if (sort_positions(nullptr, temp, nullptr, nullptr, nullptr, nin, vocab, nullptr) != hipSuccess) return 0;
    return 2 * align256(sizeof(uint32_t) * (size_t)nin) + align256(temp) + 256;
}

int nh_lut_bprop(void* dW, const void* error_t, const int32_t* ids, int itemsize, uint32_t nin, uint32_t embed,
                 uint32_t vocab, size_t ld_dw, size_t ld_err, int32_t pad_idx, void* workspace, size_t workspace_bytes,
                 void* stream) {
    if (!nh_internal_ready()) return nh_internal_fail(NH_ENOTINIT, "nh_init has not been called");
    if (nin == 0 || embed == 0 || vocab == 0) return 0;
    if (!dW || !error_t || !ids || !workspace) return nh_internal_fail(NH_EINVAL, "nh_lut_bprop: null pointer");
    if (itemsize != 4 && itemsize != 2) return nh_internal_fail(NH_EINVAL, "nh_lut_bprop: fp32 or fp16 tensors only");
    if (ld_dw < embed || ld_err < embed) return nh_internal_fail(NH_EINVAL, "nh_lut_bprop: leading dimension < embed");
    if (workspace_bytes < nh_lut_workspace_bytes(nin, vocab))
        return nh_internal_fail(NH_EINVAL, "nh_lut_bprop: workspace smaller than nh_lut_workspace_bytes");
    hipStream_t s = (hipStream_t)stream;
    char* ws = (char*)workspace;
    uint32_t* keys = (uint32_t*)ws;
    uint32_t* pos = (uint32_t*)(ws + align256(sizeof(uint32_t) * (size_t)nin));
    void* temp = ws + 2 * align256(sizeof(uint32_t) * (size_t)nin);
    size_t temp_bytes = workspace_bytes - 2 * align256(sizeof(uint32_t) * (size_t)nin);
    hipError_t e = sort_positions(temp, temp_bytes, (const uint32_t*)ids, keys, pos, nin, vocab, s);
    if (e != hipSuccess) return nh_internal_fail((int)e, "nh_lut_bprop: sorting the word ids failed");
    const unsigned blocks = (nin + LUT_WAVES - 1) / LUT_WAVES;
    if (itemsize == 4)
        hipLaunchKernelGGL((lut_bprop_kernel<float>), dim3(blocks), dim3(LUT_T), 0, s, (float*)dW, (const float*)error_t,
                           keys, pos, nin, embed, vocab, ld_dw, ld_err, pad_idx);
    else
        hipLaunchKernelGGL((lut_bprop_kernel<nh_f16>), dim3(blocks), dim3(LUT_T), 0, s, (nh_f16*)dW,
                           (const nh_f16*)error_t, keys, pos, nin, embed, vocab, ld_dw, ld_err, pad_idx);
    e = hipGetLastError();
    if (e != hipSuccess) return nh_internal_fail((int)e, "nh_lut_bprop");
    return 0;
}

}  // extern "C"
