// Prebuilt hand-written gfx950 kernels behind the direct entry points of
// include/neonhip.h.  All of them are HBM-bound streaming kernels: every
// global access is a 16-byte vector per lane, arithmetic is fp32, and nothing
// is read twice.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <string>

#include "neonhip.h"
#include "device/neon_device.h"

bool nh_internal_ready();
int nh_internal_fail(int code, const char* msg);
int nh_internal_cu_count();
int nh_internal_device();

namespace {

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

int launch_status(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return nh_internal_fail((int)e, what);
    return 0;
}

// ---------------------------------------------------------------------------
// Streaming elementwise kernels: 512 threads (the Adam update over 25 M
// parameters: 105.2 us with 256, 103.6 us with 512), one vector of V floats per lane
// and tensor (every wave touches 1 KiB contiguous per instruction), all loads
// issued before the first use.  One vector per lane measured fastest for the
// 7-stream Adam update (more in flight per lane only adds read/write
// turnarounds); inputs far larger than the caches are read with non-temporal
// loads and written with ordinary stores (measured: 6.7 TB/s on the Adam
// update against 5.9 TB/s with non-temporal stores as well).
// ---------------------------------------------------------------------------
constexpr int EW_T = 512;
constexpr size_t EW_STREAM_BYTES = (size_t)256 << 20;

template <int V, bool NT> __device__ __forceinline__ void ew_ld(const float* p, float (&r)[V]) {
    nh_u32 w[V];
    nh_load_words<V, NT>(reinterpret_cast<const nh_u32*>(p), w);
#pragma unroll
    for (int j = 0; j < V; ++j) r[j] = __builtin_bit_cast(float, w[j]);
}
template <int V, bool NT> __device__ __forceinline__ void ew_st(float* p, const float (&r)[V]) {
    nh_u32 w[V];
#pragma unroll
    for (int j = 0; j < V; ++j) w[j] = __builtin_bit_cast(nh_u32, r[j]);
    nh_store_words<V, NT>(reinterpret_cast<nh_u32*>(p), w);
}

template <int V, bool NT, class F>
__global__ __launch_bounds__(EW_T) void ew_stream_kernel(F f, size_t n) {
    const size_t i = ((size_t)blockIdx.x * EW_T + threadIdx.x) * V;
    if (i + V <= n) {
        typename F::template regs<V> r;
        f.template load<V, NT>(r, i);
        f.template compute<V>(r);
        f.template store<V, NT>(r, i);
    } else {
        for (size_t e = i; e < n; ++e) {
            typename F::template regs<1> r;
            f.template load<1, false>(r, e);
            f.template compute<1>(r);
            f.template store<1, false>(r, e);
        }
    }
}

struct AxpbyF {
    float* out; const float* x; const float* y; float a, b;
    static constexpr int TENSORS = 3;
    template <int V> struct regs { float x[V], y[V]; };
    template <int V, bool NT> __device__ void load(regs<V>& r, size_t i) const { ew_ld<V, NT>(x + i, r.x); ew_ld<V, NT>(y + i, r.y); }
    template <int V> __device__ void compute(regs<V>& r) const {
#pragma unroll
        for (int j = 0; j < V; ++j) r.x[j] = a * r.x[j] + b * r.y[j];
    }
    template <int V, bool NT> __device__ void store(const regs<V>& r, size_t i) const { ew_st<V, false>(out + i, r.x); }
};

struct SigmoidF {
    float* out; const float* x;
    static constexpr int TENSORS = 2;
    template <int V> struct regs { float x[V]; };
    template <int V, bool NT> __device__ void load(regs<V>& r, size_t i) const { ew_ld<V, NT>(x + i, r.x); }
    template <int V> __device__ void compute(regs<V>& r) const {
#pragma unroll
        for (int j = 0; j < V; ++j) r.x[j] = nh_sig(r.x[j]);
    }
    template <int V, bool NT> __device__ void store(const regs<V>& r, size_t i) const { ew_st<V, false>(out + i, r.x); }
};

// The three assigns of the reference's Adam.optimize
// (neon/optimizers/optimizer.py:925-930) fused: 4 tensors read, 3 written.
// Operation order follows the Python expressions so that, with contraction
// off, the result is the one numpy computes in fp32.
struct AdamF {
    float* p; float* m; float* v; const float* g;
    float lr, b1, omb1, b2, omb2, eps;
    static constexpr int TENSORS = 7;
    template <int V> struct regs { float p[V], m[V], v[V], g[V]; };
    template <int V, bool NT> __device__ void load(regs<V>& r, size_t i) const {
        ew_ld<V, NT>(g + i, r.g); ew_ld<V, NT>(m + i, r.m); ew_ld<V, NT>(v + i, r.v); ew_ld<V, NT>(p + i, r.p);
    }
    template <int V> __device__ void compute(regs<V>& r) const {
#pragma unroll
        for (int j = 0; j < V; ++j) {
            const float gj = r.g[j];
            const float mj = r.m[j] * b1 + omb1 * gj;
            const float vj = r.v[j] * b2 + (omb2 * gj) * gj;
            r.m[j] = mj;
            r.v[j] = vj;
            r.p[j] = r.p[j] - (lr * mj) / (sqrtf(vj) + eps);
        }
    }
    template <int V, bool NT> __device__ void store(const regs<V>& r, size_t i) const {
        ew_st<V, false>(m + i, r.m); ew_st<V, false>(v + i, r.v); ew_st<V, false>(p + i, r.p);
    }
};

template <class F> int launch_ew(const F& f, size_t n, bool vec_ok, void* stream, const char* what) {
    if (!nh_internal_ready()) return nh_internal_fail(NH_ENOTINIT, "nh_init has not been called");
    if (n == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const int v = vec_ok ? 4 : 1;
    const size_t per_block = (size_t)EW_T * v;
    const size_t blocks = (n + per_block - 1) / per_block;
    if (blocks > 0x7FFFFFFFull) return nh_internal_fail(NH_EINVAL, "tensor too large for one launch");
    const bool nt = n * sizeof(float) * F::TENSORS >= EW_STREAM_BYTES;
    if (vec_ok && nt) hipLaunchKernelGGL((ew_stream_kernel<4, true, F>), dim3((unsigned)blocks), dim3(EW_T), 0, s, f, n);
    else if (vec_ok) hipLaunchKernelGGL((ew_stream_kernel<4, false, F>), dim3((unsigned)blocks), dim3(EW_T), 0, s, f, n);
    else hipLaunchKernelGGL((ew_stream_kernel<1, false, F>), dim3((unsigned)blocks), dim3(EW_T), 0, s, f, n);
    return launch_status(what);
}

// ---------------------------------------------------------------------------
// Row normalisation, fp16 storage / fp32 statistics.  One workgroup of 1024
// threads owns one row and keeps it in registers as raw fp16 vectors (NCH
// chunks of 8 halves per thread), so the row is read from HBM exactly once:
// sweep 1 takes sum and second moment per lane while the tiles arrive, sweep 2
// normalises and stores.  Cross-lane sums use DPP; LDS only joins the 16 waves.
// ---------------------------------------------------------------------------
constexpr int RN_T = 1024;
constexpr int RN_V = 8;

template <int NCH, bool NT>
__global__ __launch_bounds__(RN_T) void rownorm_f16_kernel(nh_f16* out, const nh_f16* x,
                                                           const float* __restrict__ gamma,
                                                           const float* __restrict__ beta, float eps, uint32_t cols,
                                                           size_t ld, float inv_n) {
    __shared__ float slots[RN_T / 64];
    const uint32_t row = blockIdx.x;
    const int tid = threadIdx.x;
    const nh_f16* xr = x + (size_t)row * ld;
    nh_f16* orow = out + (size_t)row * ld;

    // The row stays packed (two halves per register) for the whole kernel;
    // nh_keep_packed() between sweeps stops the compiler from widening it to
    // one fp32 register per element, which would not fit the register file.
    nh_u32 raw[NCH][RN_V / 2];
#pragma unroll
    for (int k = 0; k < NCH; ++k) {
        const uint32_t c = (uint32_t)(k * RN_T + tid) * RN_V;
        if (c < cols) {
            nh_load_words<RN_V / 2, NT>(reinterpret_cast<const nh_u32*>(xr + c), raw[k]);
        } else {
#pragma unroll
            for (int j = 0; j < RN_V / 2; ++j) raw[k][j] = 0u;  // +0.0 pairs
        }
    }
    const float g = gamma[row];
    const float b = beta[row];

    // One pass over the tiles as they arrive takes the lane's sum and its squared deviations from a
    // shift (the lane's first element: deviations stay small, nothing cancels); once the row's mean is
    // known each lane's share of the row's squared deviations follows in closed form
    //   sum (x - mean)^2 = M2_lane + n_lane * (mean_lane - mean)^2,
    // so the second block-wide sum needs no second sweep over the registers.
    const float one = nh_opaque_one();
    float s = 0.0f, sq = 0.0f, cnt = 0.0f;
    const float shift = nh_f16_lo(raw[0][0]);           // (a lane without elements holds zeros and counts none)
#pragma unroll
    for (int k = 0; k < NCH; ++k) {
        const uint32_t c = (uint32_t)(k * RN_T + tid) * RN_V;
        if (c < cols) {
            cnt += (float)RN_V;
#pragma unroll
            for (int j = 0; j < RN_V / 2; ++j) {
                // widening and subtraction in one v_fma_mix_f32 each; the squares are
                // accumulated with one rounding per term
                const float d0 = __builtin_fmaf(nh_f16_lo(raw[k][j]), one, -shift);
                const float d1 = __builtin_fmaf(nh_f16_hi(raw[k][j]), one, -shift);
                sq = __builtin_fmaf(d0, d0, sq);
                sq = __builtin_fmaf(d1, d1, sq);
                s = nh_sum2_f16(raw[k][j], s);
            }
        }
    }
    const float mean = nh_block_allreduce<nh_op_sum, RN_T / 64>(s, slots) * inv_n;
    float q = 0.0f;
    if (cnt > 0.0f) {
        const float sa = __builtin_fmaf(-cnt, shift, s);         // sum of (x - shift)
        const float mu = sa / cnt;                               // lane mean - shift
        const float m2 = nh_max(sq - sa * mu, 0.0f);             // squared deviations from the lane mean
        const float e = (shift + mu) - mean;
        q = __builtin_fmaf(cnt * e, e, m2);
    }
    const float var = nh_block_allreduce<nh_op_sum, RN_T / 64>(q, slots) * inv_n;
    // gamma * (x - mean) / sqrt(var + eps) + beta as (x - mean) * A + beta with A once
    // per row: the output is rounded to fp16 anyway, and the kernel is bound by
    // instruction issue (8 fp16 elements per 16 bytes)
    const float scale = g / sqrtf(var + eps);

#pragma unroll
    for (int k = 0; k < NCH; ++k) nh_keep_packed(raw[k]);
#pragma unroll
    for (int k = 0; k < NCH; ++k) {
        const uint32_t c = (uint32_t)(k * RN_T + tid) * RN_V;
        if (c < cols) {
            nh_u32 o[RN_V / 2];
#pragma unroll
            for (int j = 0; j < RN_V / 2; ++j) {
                const float d0 = __builtin_fmaf(nh_f16_lo(raw[k][j]), one, -mean);
                const float d1 = __builtin_fmaf(nh_f16_hi(raw[k][j]), one, -mean);
                o[j] = nh_f16_pack(__builtin_fmaf(d0, scale, b), __builtin_fmaf(d1, scale, b));
            }
            nh_store_words<RN_V / 2, NT>(reinterpret_cast<nh_u32*>(orow + c), o);
        }
    }
}

template <int NCH>
void launch_rownorm(uint16_t* out, const uint16_t* x, const float* gamma, const float* beta, float eps,
                    uint32_t rows, uint32_t cols, size_t ld, hipStream_t s) {
    // beyond what the L2 slices hold, the row is touched once: stream it
    const bool nt = (size_t)rows * cols * 2 * sizeof(uint16_t) >= ((size_t)32 << 20);
    if (nt)
        hipLaunchKernelGGL((rownorm_f16_kernel<NCH, true>), dim3(rows), dim3(RN_T), 0, s, (nh_f16*)out,
                           (const nh_f16*)x, gamma, beta, eps, cols, ld, 1.0f / (float)cols);
    else
        hipLaunchKernelGGL((rownorm_f16_kernel<NCH, false>), dim3(rows), dim3(RN_T), 0, s, (nh_f16*)out,
                           (const nh_f16*)x, gamma, beta, eps, cols, ld, 1.0f / (float)cols);
}

// ---------------------------------------------------------------------------
// Column (axis-0) max / argmax.  Lanes run across columns so every load is
// coalesced; a workgroup is LX column-lanes x (CR_T / LX) row-lanes and owns a
// (rows_per_chunk x LX*V) tile: 8 lanes x 16 bytes = one 128-byte segment per
// row, 32 rows per step and four steps in flight per lane.  The row-lanes of a
// wave fold with lane exchanges that split the V values between the partners
// (nh_col_wave_fold), LDS joins the four waves.  Tiles of one column strip
// leave (value, index) partials in the scratch area; the last workgroup of the
// strip to finish (ticket counter) folds them and writes the result.  No
// workgroup ever waits for another.
// Partials cross XCDs as write-through stores / L2-bypassing loads; each lane
// waits for its own stores before the barrier that precedes the ticket.
// ---------------------------------------------------------------------------
constexpr int CR_T = 256;                 // lanes per workgroup; twice that for small inputs (one workgroup per
                                          // compute unit), where a second wave per SIMD hides the first one's waits
constexpr int CR_U = 4;                   // rows in flight per lane
constexpr int CR_FOLD_BATCH = 4;          // partials in flight per lane in the final fold
constexpr int CR_MAX_STRIPS = 4096;
constexpr int CR_MAX_CHUNKS = 128;
// The tickets of neighbouring strips sit a 64-byte line apart: atomics on one line are served
// one after the other whichever words of it they address, and with the tickets of all strips in
// one line the workgroups of a (32000 x 256) launch queued behind each other for two microseconds.
constexpr int CR_TICKET_STRIDE = 16;

__device__ unsigned int g_cr_tickets[CR_MAX_STRIPS * CR_TICKET_STRIDE];  // zero at load; each strip's last workgroup resets its ticket

// Scratch of the entry point that allocates nothing: tickets first, partials
// after them.  One copy per device, alive until the process ends; host code
// reaches it through the address hipGetSymbolAddress returns for the device.
constexpr size_t CR_STATIC_TICKET_BYTES = (size_t)CR_MAX_STRIPS * CR_TICKET_STRIDE * sizeof(unsigned int);
static __device__ __align__(256) unsigned char scratch[NH_STATIC_SCRATCH_BYTES];

// Join the row-lanes of the workgroup: the row-lanes of a wave fold with lane
// exchanges, the waves leave their pieces in LDS and ONE lane per column
// (threads 0 .. LX*V-1) joins them.  The steps after the sweep are a chain of
// dependent operations on a few values, so that chain is kept short rather
// than wide.
template <int V, int LX, int T>
__device__ __forceinline__ nh_pair cr_join_rows(nh_pair (&acc)[V], nh_pair (*sp)[LX * V]) {
    constexpr int S = LX * V;
    constexpr int CR_WAVES = T / 64;
    const int tx = threadIdx.x % LX;
    const int wave = threadIdx.x >> 6;
    if constexpr (LX < 64) {
        constexpr int STEPS = __builtin_ctz(64 / LX);
        constexpr int VK = (V >> STEPS) > 0 ? (V >> STEPS) : 1;     // values a lane still holds after the wave fold
        const int j0 = nh_col_wave_fold<nh_op_argmax, V, LX>(acc);
        if ((int)(threadIdx.x & 63) < LX * (V / VK)) {
#pragma unroll
            for (int j = 0; j < VK; ++j) sp[wave][tx * V + j0 + j] = acc[j];
        }
    } else {
#pragma unroll
        for (int j = 0; j < V; ++j) sp[wave][tx * V + j] = acc[j];
    }
    __syncthreads();
    nh_pair one = nh_op_argmax::init();
    if ((int)threadIdx.x < S) {
        one = sp[0][threadIdx.x];
#pragma unroll
        for (int y = 1; y < CR_WAVES; ++y) one = nh_op_argmax::f(one, sp[y][threadIdx.x]);
    }
    return one;
}

template <int V, int LX, int T>
__global__ __launch_bounds__(T) void colmax_kernel(const float* __restrict__ x, uint32_t rows, uint32_t cols,
                                                   size_t ld, uint32_t rows_per_chunk, nh_pair* part,
                                                   float* __restrict__ outv, int* __restrict__ outi,
                                                   unsigned int* tickets) {
    constexpr int CR_WAVES = T / 64;
    constexpr int LY = T / LX;
    constexpr int S = LX * V;                       // columns of a strip
    constexpr int P = T / S;                        // lanes per column in the last workgroup's fold
    static_assert(S <= T && P <= 64, "strip geometry");
    __shared__ __attribute__((aligned(16))) nh_pair sp[CR_WAVES][S];
    __shared__ int s_last;
    const int tid = threadIdx.x;
    const int tx = tid % LX, ty = tid / LX;
    const uint32_t c0 = blockIdx.x * S;
    const uint32_t c = c0 + tx * V;
    const uint32_t r0 = blockIdx.y * rows_per_chunk;
    const uint32_t r1 = (r0 + rows_per_chunk < rows) ? r0 + rows_per_chunk : rows;
    const bool live = c < cols;  // cols % V == 0 is checked on the host

    nh_pair acc[V];
#pragma unroll
    for (int j = 0; j < V; ++j) acc[j] = nh_op_argmax::init();
    if (live) {
        const float* xp = x + c;
        uint32_t r = r0 + ty;
        for (; r + (CR_U - 1) * LY < r1; r += CR_U * LY) {
            float a[CR_U][V];
#pragma unroll
            for (int u = 0; u < CR_U; ++u) nh_load_vec<float, V>(xp + (size_t)(r + u * LY) * ld, a[u]);
#pragma unroll
            for (int u = 0; u < CR_U; ++u)
#pragma unroll
                for (int j = 0; j < V; ++j) nh_op_argmax::step(acc[j], a[u][j], (int)(r + u * LY));
        }
        for (; r < r1; r += LY) {
            float a0[V];
            nh_load_vec<float, V>(xp + (size_t)r * ld, a0);
#pragma unroll
            for (int j = 0; j < V; ++j) nh_op_argmax::step(acc[j], a0[j], (int)r);
        }
    }
    nh_pair one = cr_join_rows<V, LX, T>(acc, sp);     // threads 0 .. S-1: the strip's column c0 + tid

    const uint32_t nchunks = gridDim.y;
    uint32_t col = tid;
    bool writer = tid < S && c0 + tid < cols;
    if (nchunks > 1) {
        if (writer) nh_part_store(&part[(size_t)blockIdx.y * cols + c0 + tid], one);
        nh_publish_barrier();     // every lane's partial stores have been performed before the ticket is taken
        if (tid == 0) {
            const unsigned int t = nh_ticket_take(&tickets[blockIdx.x * CR_TICKET_STRIDE]);
            s_last = (t == nchunks - 1);
        }
        __syncthreads();
        if (!s_last) return;

        // P adjacent lanes share a column; lane k0 of them takes chunks k0, k0 + P, ...
        col = tid / P;
        const uint32_t k0 = tid % P;
        const bool fold_ok = c0 + col < cols;
        one = nh_op_argmax::init();
        for (uint32_t kb = k0; kb < nchunks; kb += P * CR_FOLD_BATCH) {
            nh_pair q[CR_FOLD_BATCH];
#pragma unroll
            for (int k = 0; k < CR_FOLD_BATCH; ++k) {
                const uint32_t chunk = kb + k * P;
                q[k] = (fold_ok && chunk < nchunks) ? nh_part_load(&part[(size_t)chunk * cols + c0 + col])
                                                    : nh_op_argmax::init();
            }
#pragma unroll
            for (int k = 0; k < CR_FOLD_BATCH; ++k) one = nh_op_argmax::f(one, q[k]);
        }
        one = nh_wave_allreduce<nh_op_argmax, P, nh_pair>(one);
        if (tid == 0) nh_ticket_reset(&tickets[blockIdx.x * CR_TICKET_STRIDE]);  // ready for the next launch on this stream
        writer = k0 == 0 && fold_ok;
    }
    if (writer) {
        if (outv) outv[c0 + col] = one.v;
        if (outi) outi[c0 + col] = one.i;
    }
}

// clears the tickets of the static scratch area (a kernel rather than a
// memset so that the call can be recorded into a graph)
__global__ void cr_clear_tickets_kernel(unsigned int* tickets, uint32_t n) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) tickets[i] = 0u;
}

// ---------------------------------------------------------------------------
// log2-magnitude histogram (the reference's kernel_histo, float_ew.py:1070-1131,
// with the binning of its CPU backend, nervanacpu.py:424-445): value v lands in
// bin clamp(rint(log2|v|) - offset, 0, ...); bin 0 extends to -inf (zeros), the
// last bin is closed at offset+nbins, anything larger is not counted.
// Integer counts, LDS atomics per workgroup, one global atomic per bin and
// workgroup: the result does not depend on scheduling.
// ---------------------------------------------------------------------------
constexpr int HIST_T = 256;
constexpr int HIST_MAX_BINS = 256;

// Bin of one value: rint(log2|v|) - offset, clamped below into bin 0 and (one
// past the end only) above into the last bin; -1 = not counted (larger
// magnitudes, infinities, NaN).  rint(log2|v|) is taken from the bits, which
// gives the correctly rounded bin: the exponent, plus one when the mantissa
// lies above sqrt(2) (0x3504F3 is the last fp32 mantissa below it; a tie cannot
// occur, sqrt(2) * 2^k is no fp32 number).  log2f would decide the neighbours
// of sqrt(2) * 2^k by the last bit of its own rounding.
__device__ __forceinline__ int hist_bin(float v, int nbins, int offset) {
    const nh_u32 mag = __builtin_bit_cast(nh_u32, v) & 0x7fffffffu;
    if (mag >= 0x7f800000u) return -1;
    if (mag == 0u) return 0;                                              // log2 0 = -inf
    int k;
    if (mag < 0x00800000u) {
        // denormal m * 2^-149: its leading bit gives the exponent, the bits below it the mantissa
        const int top = 31 - __builtin_clz(mag);
        const nh_u32 mant = (mag << (23 - top)) & 0x007fffffu;
        k = top - 149 + (mant >= 0x003504F4u ? 1 : 0);
    } else {
        k = (int)((mag + 0x004AFB0Cu) >> 23) - 127;                       // carries when the mantissa is above sqrt(2)
    }
    const long long b = (long long)k - offset;
    if (b > nbins) return -1;
    return b < 0 ? 0 : (b > nbins - 1 ? nbins - 1 : (int)b);
}

// Magnitudes of real tensors fall into a handful of bins, so LDS atomics on a
// shared histogram serialise (64 lanes, a few addresses).  Two ways round it:
//
// PRIVATE (nbins <= 64): every lane counts into its own 16-bit counters --
// word [bin][tid % 128] holds lane tid's count in its low half and lane
// tid + 128's in its high half, so the lanes of a wave always hit distinct
// banks whatever the data; the host sizes the grid so that no lane sees more
// than 65535 elements.  32 KiB of LDS per workgroup.
//
// otherwise: the wave agrees on one bin at a time (ballot) and a single lane
// adds the number of lanes that hold it to the wave's own histogram.
constexpr int HIST_PRIVATE_BINS = 64;

template <typename T, bool PRIVATE>
__global__ __launch_bounds__(HIST_T) void hist_log2_kernel(const T* __restrict__ x, size_t n, int nbins, int offset,
                                                           int* __restrict__ hist) {
    constexpr int V = 16 / (int)sizeof(T);                 // elements per 16-byte load
    constexpr int WAVES = HIST_T / 64;
    constexpr int WORDS = PRIVATE ? HIST_PRIVATE_BINS * (HIST_T / 2) : WAVES * HIST_MAX_BINS;
    __shared__ int bins[WORDS];
    for (int b = threadIdx.x; b < WORDS; b += HIST_T) bins[b] = 0;
    __syncthreads();
    const int lane = threadIdx.x & 63;
    int* mine = PRIVATE ? bins + (threadIdx.x & (HIST_T / 2 - 1)) : bins + (threadIdx.x / 64) * HIST_MAX_BINS;
    const int one = (PRIVATE && threadIdx.x >= HIST_T / 2) ? 0x10000 : 1;
    const size_t stride = (size_t)gridDim.x * HIST_T * V;
    // same trip count for every lane of the grid: the wave-wide counting needs all lanes
    const size_t trips = (n + stride - 1) / stride;
    const bool vec_ok = (reinterpret_cast<uintptr_t>(x) & 15u) == 0;
    size_t i0 = ((size_t)blockIdx.x * HIST_T + threadIdx.x) * V;
    constexpr int U = 4;                                   // loads in flight per lane
    for (size_t t = 0; t < trips; t += U, i0 += U * stride) {
        nh_u32 w[U][4];
        bool whole[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const size_t i = i0 + u * stride;
            whole[u] = vec_ok && t + u < trips && i + V <= n;
            if (whole[u]) nh_load_words<4, true>(reinterpret_cast<const nh_u32*>(x + i), w[u]);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const size_t i = i0 + u * stride;
            float v[V];
            int live = 0;
            if (whole[u]) {
#pragma unroll
                for (int j = 0; j < V; ++j) {
                    if constexpr (sizeof(T) == 4) v[j] = __builtin_bit_cast(float, w[u][j]);
                    else v[j] = (j & 1) ? nh_f16_hi(w[u][j / 2]) : nh_f16_lo(w[u][j / 2]);
                }
                live = V;
            } else if (t + u < trips) {
#pragma unroll
                for (int j = 0; j < V; ++j)
                    if (i + j < n) { v[j] = (float)x[i + j]; live = j + 1; }
            }
#pragma unroll
            for (int j = 0; j < V; ++j) {
                const int bin = j < live ? hist_bin(v[j], nbins, offset) : -1;
                if constexpr (PRIVATE) {
                    if (bin >= 0) atomicAdd(&mine[bin * (HIST_T / 2)], one);     // LDS; only lane tid +- 128 shares the word
                } else {
                    unsigned long long todo = __ballot(bin >= 0);
                    while (todo) {
                        const int leader = __ffsll((long long)todo) - 1;
                        const int b = __builtin_amdgcn_readlane(bin, leader);
                        const unsigned long long same = __ballot(bin == b);
                        if (lane == leader) mine[b] += __popcll(same);
                        todo &= ~same;
                    }
                }
            }
        }
    }
    __syncthreads();
    if constexpr (PRIVATE) {
        // four lanes per bin, 32 words each, both halves of every word
        const int b = threadIdx.x / 4, part = threadIdx.x % 4;
        int total = 0;
        if (b < nbins) {
            const int* row = bins + b * (HIST_T / 2) + part * (HIST_T / 8);
            for (int k = 0; k < HIST_T / 8; ++k) {
                const unsigned int w = (unsigned int)row[(k + lane) % (HIST_T / 8)];
                total += (int)(w & 0xffffu) + (int)(w >> 16);
            }
        }
        total += __shfl_xor(total, 1);
        total += __shfl_xor(total, 2);
        if (part == 0 && b < nbins && total) atomicAdd(&hist[b], total);
    } else {
        for (int b = threadIdx.x; b < nbins; b += HIST_T) {
            int total = 0;
#pragma unroll
            for (int w = 0; w < WAVES; ++w) total += bins[w * HIST_MAX_BINS + b];
            if (total) atomicAdd(&hist[b], total);
        }
    }
}

// EXPONENT (what real calls take: nbins <= 64, offset >= -126, offset + nbins
// < 128): rint(log2|v|) of a normal fp32 value is its exponent, plus one when
// the mantissa lies above sqrt(2) -- adding 0x4AFB0C (2^23 minus the first
// mantissa above sqrt 2) to the magnitude bits carries exactly then, so the
// bin row comes out of an add, a clamp and a shift with no logarithm and no
// branch: magnitudes below the first bin's upper edge (zeros and denormals
// included: offset >= -126) clamp into row 0, row nbins collects b == nbins
// (counted into the last bin), row nbins + 1 everything beyond (larger
// magnitudes, infinities and NaNs: offset + nbins < 128), which is dropped.
// Same private 16-bit counters as PRIVATE.  The kernel is bound by instruction
// issue and by its fixed parts, not by LDS or HBM (measured: the logarithm
// version spends 15 us of VALU issue on 25 M values), hence the
// five-instruction binning; loads are double-buffered and never sit inside a
// branch.  ONE workgroup per compute unit: with several, the oldest takes the
// issue slots and the youngest finishes late (25 M values: the last of four
// left its loop at 25 us, a single one at 13 us), and every workgroup pays the
// clearing, the fold and a global atomic per bin.
constexpr int HIST_ROWS = HIST_PRIVATE_BINS + 2;
constexpr int HIST_STAGE = 8;                             // vectors per lane and stage (two stages in flight)
constexpr int HIST_WIDE_T = 256;                          // 512 (two waves per SIMD) leaves its loop sooner but measured 3.7 us slower overall

template <typename T, int THREADS>
__global__ __launch_bounds__(THREADS) void hist_exponent_kernel(const T* __restrict__ x, size_t n, int nbins, int offset,
                                                               int* __restrict__ hist) {
    constexpr int V = 16 / (int)sizeof(T);
    constexpr int HALF = THREADS / 2;                      // words per row: lanes t and t + HALF share one
    constexpr int ROW_SHIFT = 23 - (HALF == 128 ? 9 : 10);  // row << 23  ->  byte offset of the row
    static_assert(HALF == 128 || HALF == 256, "rows of 512 or 1024 bytes");
    constexpr int U = HIST_STAGE;
    __shared__ __attribute__((aligned(16))) int bins[HIST_ROWS * HALF];
    // elements before the first 16-byte boundary and after the last whole vector: first workgroup, one per lane
    const size_t lead = ((16u - (reinterpret_cast<uintptr_t>(x) & 15u)) & 15u) / sizeof(T);
    const size_t head = lead < n ? lead : n;
    const size_t nvec = (n - head) / V;
    const size_t rest = head + nvec * V;
    const nh_u32* xv = reinterpret_cast<const nh_u32*>(x + head);
    const size_t gs = (size_t)gridDim.x * THREADS;
    const size_t last = nvec ? nvec - 1 : 0;
    nh_u32 a[U][4], b[U][4];
    auto load = [&](nh_u32 (&d)[U][4], size_t j) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const size_t jj = j + u * gs;
            nh_load_words<4, true>(xv + (jj < last ? jj : last) * 4, d[u]);          // past the end: the last vector again
        }
    };
    size_t j = (size_t)blockIdx.x * THREADS + threadIdx.x;
    if (j < nvec) load(a, j);                              // in flight while the counters are cleared
    for (int w = threadIdx.x * 4; w < HIST_ROWS * HALF; w += THREADS * 4)
        *reinterpret_cast<int4*>(bins + w) = make_int4(0, 0, 0, 0);
    __syncthreads();
    const nh_u32 lane_byte = (nh_u32)(threadIdx.x & (HALF - 1)) * 4u;
    const int one = threadIdx.x >= HALF ? 0x10000 : 1;
    // (magnitude bits + 0x4AFB0C) - (first row's exponent << 23), saturating at 0 and at row nbins + 1
    const nh_u32 below = ((nh_u32)(127 + offset) << 23) - 0x004AFB0Cu, top = (nh_u32)(nbins + 1) << 23;
    auto count = [&](float v) {
        const nh_u32 mag = __builtin_bit_cast(nh_u32, v) & 0x7fffffffu;
        const nh_u32 r = __builtin_elementwise_min(__builtin_elementwise_sub_sat(mag, below), top);   // row << 23
        atomicAdd(reinterpret_cast<int*>(reinterpret_cast<char*>(bins) + (((r >> ROW_SHIFT) & ~(nh_u32)(HALF * 4 - 1)) | lane_byte)), one);
    };
    auto tally = [&](const nh_u32 (&d)[U][4], size_t jj, bool all) {
#pragma unroll
        for (int u = 0; u < U; ++u)
            if (all || jj + u * gs < nvec) {
#pragma unroll
                for (int e = 0; e < V; ++e) {
                    if constexpr (sizeof(T) == 4) count(__builtin_bit_cast(float, d[u][e]));
                    else count((e & 1) ? nh_f16_hi(d[u][e / 2]) : nh_f16_lo(d[u][e / 2]));
                }
            }
    };
    if (blockIdx.x == 0) {
        if (threadIdx.x < head) count((float)x[threadIdx.x]);
        if (rest + threadIdx.x < n) count((float)x[rest + threadIdx.x]);
    }
    // while both stages are whole for this lane nothing is checked per vector
    for (; j + (2 * U - 1) * gs < nvec; j += 2 * U * gs) {
        load(b, j + U * gs);
        tally(a, j, true);
        load(a, j + 2 * U * gs);
        tally(b, j + U * gs, true);
    }
    if (j < nvec) {
        load(b, j + U * gs);
        tally(a, j, false);
        tally(b, j + U * gs, false);
    }
    __syncthreads();
    const bool wide = (reinterpret_cast<uintptr_t>(hist) & 7u) == 0;      // 64-bit adds need the alignment
    // PER lanes per bin, 32 words each, both halves of every word; row nbins belongs to the last bin
    constexpr int PER = THREADS / HIST_PRIVATE_BINS, WORDS = HALF / PER;
    const int bin = threadIdx.x / PER, part = threadIdx.x % PER;
    auto row_sum = [&](int row) {
        const int4* p = reinterpret_cast<const int4*>(bins + row * HALF + part * WORDS);
        unsigned int sum = 0;
#pragma unroll
        for (int k = 0; k < WORDS / 4; ++k) {
            const int4 w = p[(k + bin) % (WORDS / 4)];
            const unsigned int c[4] = {(unsigned int)w.x, (unsigned int)w.y, (unsigned int)w.z, (unsigned int)w.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) sum += (c[e] & 0xffffu) + (c[e] >> 16);
        }
        return (int)sum;
    };
    int total = 0;
    if (bin < nbins) {
        total = row_sum(bin);
        if (bin == nbins - 1) total += row_sum(nbins);
    }
#pragma unroll
    for (int m = 1; m < PER; m *= 2) total += __shfl_xor(total, m);
    // The adds of all workgroups land on one or two cache lines and are taken one after the other there
    // (about a nanosecond each: with 256 workgroups and 14 occupied bins the last acknowledgement came 3.5 us
    // after the average workgroup was done), so two neighbouring bins travel in one 64-bit add: a workgroup's
    // count of one bin stays far below 2^32, the low half cannot carry into the high one before the int32
    // result itself would overflow.
    const int next = __shfl_down(total, PER);
    if (part == 0 && bin < nbins) {
        const bool paired = wide && bin + 1 < nbins;
        if (paired && (bin & 1) == 0) {
            if (total | next)
                atomicAdd(reinterpret_cast<unsigned long long*>(hist + bin),
                          (unsigned long long)(unsigned int)total | ((unsigned long long)(unsigned int)next << 32));
        } else if (!(wide && (bin & 1)) && total) {
            atomicAdd(&hist[bin], total);
        }
    }
}

struct CrPlan { uint32_t strips, chunks, rows_per_chunk; int v, lx, threads; };

CrPlan cr_plan(uint32_t rows, uint32_t cols, bool vec) {
    CrPlan p;
    // 16-byte accesses, 8 column-lanes (128 bytes per row segment); matrices
    // whose row length is not a multiple of four: one element per lane, 64 lanes
    p.v = vec ? 4 : 1;
    p.lx = vec ? 8 : 64;
    const uint64_t small = (uint64_t)(nh_internal_cu_count() > 0 ? nh_internal_cu_count() : 256) * (256u << 10);
    p.threads = (vec && (uint64_t)rows * cols * sizeof(float) < small) ? 2 * CR_T : CR_T;
    const uint32_t ly = p.threads / p.lx;
    const uint32_t strip_cols = p.lx * p.v;
    p.strips = (cols + strip_cols - 1) / strip_cols;
    // one workgroup per compute unit for small inputs, up to eight for large
    // ones, each with at least ~128 KiB to stream
    const uint64_t bytes = (uint64_t)rows * cols * sizeof(float);
    const uint32_t cus = nh_internal_cu_count() > 0 ? (uint32_t)nh_internal_cu_count() : 256u;
    uint64_t per_cu = bytes / ((uint64_t)cus * (128u << 10));
    if (per_cu < 1) per_cu = 1;
    if (per_cu > 8) per_cu = 8;
    uint32_t chunks = (uint32_t)(per_cu * cus) / (p.strips ? p.strips : 1);
    if (chunks < 1) chunks = 1;
    if (chunks > CR_MAX_CHUNKS) chunks = CR_MAX_CHUNKS;
    uint32_t rpc = (rows + chunks - 1) / chunks;
    const uint32_t min_rpc = CR_U * ly;
    if (rpc < min_rpc) rpc = min_rpc;
    rpc = (rpc + ly - 1) / ly * ly;
    p.rows_per_chunk = rpc;
    p.chunks = (rows + rpc - 1) / rpc;
    if (p.chunks < 1) p.chunks = 1;
    return p;
}

// per device: address of this file's `scratch` array on that device (the
// array's name is only a host-side handle), looked up once by nh_init
constexpr int CR_MAX_DEVICES = 64;
void* g_scratch_ptr[CR_MAX_DEVICES];

// ---------------------------------------------------------------------------
// Dimension shuffle (numpy.transpose into a destination tensor).  Dimensions
// are given in OUTPUT order, each with its output and its input stride.  A
// workgroup moves one 64 x 64 tile spanned by axis `ax` (the output's
// fastest-moving dimension) and axis `ay`; all other dimensions are decoded
// once per workgroup from the block index.
//   SWAP = true:  `ay` is the dimension that moves fastest in the INPUT: the
//     tile is read with lanes along `ay`, turned in LDS (row pitch 65 words:
//     conflict-free for 4- and 8-byte elements) and written with lanes along
//     `ax`, so both sides see 64-element contiguous runs.
//   SWAP = false: the fastest dimension is the same on both sides; lanes run
//     along it for the read and the write and LDS is not used.
// Tiles are handed out along diagonals (tile row q, column c -> ty = (q + c)
// mod tiles_y): the workgroups in flight at one time then differ in both tile
// coordinates, so neither the reads (64 runs a whole input row apart) nor the
// writes pile onto the memory channels a power-of-two row pitch maps to.
// Measured on an 8192 x 8192 fp32 transpose: 81 us against 92 us row by row.
// ---------------------------------------------------------------------------
constexpr int TR_TILE = 64;
constexpr int TR_T = 256;

__device__ __forceinline__ void tr_tile_of(unsigned long long& b, uint32_t tiles_x, uint32_t tiles_y, uint32_t& tx,
                                           uint32_t& ty) {
    tx = (uint32_t)(b % tiles_x);
    b /= tiles_x;
    ty = (uint32_t)((b + tx) % tiles_y);
    b /= tiles_y;
}

struct TrGeom {
    uint32_t n[NH_TRANSPOSE_MAX_DIMS];
    long long os[NH_TRANSPOSE_MAX_DIMS];
    long long is[NH_TRANSPOSE_MAX_DIMS];
    int nd, ax, ay;
    uint32_t tiles_x, tiles_y;
};

template <typename T, bool SWAP>
__global__ __launch_bounds__(TR_T) void transpose_tile_kernel(T* __restrict__ out, const T* __restrict__ in, TrGeom g) {
    __shared__ T tile[SWAP ? TR_TILE : 1][TR_TILE + 1];
    unsigned long long b = blockIdx.x;
    uint32_t tx, ty;
    tr_tile_of(b, g.tiles_x, g.tiles_y, tx, ty);
    long long ibase = 0, obase = 0;
    for (int k = g.nd - 1; k >= 0; --k) {
        if (k == g.ax || k == g.ay) continue;
        const unsigned long long idx = b % g.n[k];
        b /= g.n[k];
        ibase += (long long)idx * g.is[k];
        obase += (long long)idx * g.os[k];
    }
    const uint32_t nx = g.n[g.ax], ny = g.ay >= 0 ? g.n[g.ay] : 1u;
    const long long isx = g.is[g.ax], osx = g.os[g.ax];
    const long long isy = g.ay >= 0 ? g.is[g.ay] : 0, osy = g.ay >= 0 ? g.os[g.ay] : 0;
    const uint32_t x0 = tx * TR_TILE, y0 = ty * TR_TILE;
    const uint32_t lane = threadIdx.x & (TR_TILE - 1), row = threadIdx.x / TR_TILE;
    constexpr uint32_t ROWS = TR_T / TR_TILE;
    if constexpr (SWAP) {
        for (uint32_t i = row; i < TR_TILE; i += ROWS) {
            const uint32_t x = x0 + i, y = y0 + lane;
            if (x < nx && y < ny) tile[i][lane] = in[ibase + (long long)x * isx + (long long)y * isy];
        }
        __syncthreads();
        for (uint32_t i = row; i < TR_TILE; i += ROWS) {
            const uint32_t x = x0 + lane, y = y0 + i;
            if (x < nx && y < ny) out[obase + (long long)x * osx + (long long)y * osy] = tile[lane][i];
        }
    } else {
        const uint32_t x = x0 + lane;
        if (x < nx) {
            for (uint32_t i = row; i < TR_TILE; i += ROWS) {
                const uint32_t y = y0 + i;
                if (y < ny)
                    out[obase + (long long)x * osx + (long long)y * osy] =
                        in[ibase + (long long)x * isx + (long long)y * isy];
            }
        }
    }
}

// The same tile walk for 2- and 4-byte elements with 16-byte global accesses:
// VE = 16 / sizeof(T) elements per lane, 64 / VE lanes cover a 64-element run.
// Needs both tile extents, the strides of every other dimension and the base
// addresses to be multiples of VE elements.  LDS is still accessed element by
// element (the VE elements a lane turns into an output vector come from VE
// tile rows; odd row pitch in 32-bit words), two-way bank conflicts at worst.
template <typename T, bool SWAP>
__global__ __launch_bounds__(TR_T) void transpose_tile_vec_kernel(T* __restrict__ out, const T* __restrict__ in,
                                                                  TrGeom g) {
    constexpr int VE = 16 / (int)sizeof(T);
    constexpr int PITCH = TR_TILE + 4 / (int)sizeof(T);          // 65 words (4-byte) or 33 words (2-byte) per row
    constexpr uint32_t LANES = TR_TILE / VE, RUNS = TR_T / LANES;
    __shared__ T tile[SWAP ? TR_TILE : 1][PITCH];
    unsigned long long b = blockIdx.x;
    uint32_t tx, ty;
    tr_tile_of(b, g.tiles_x, g.tiles_y, tx, ty);
    long long ibase = 0, obase = 0;
    for (int k = g.nd - 1; k >= 0; --k) {
        if (k == g.ax || k == g.ay) continue;
        const unsigned long long idx = b % g.n[k];
        b /= g.n[k];
        ibase += (long long)idx * g.is[k];
        obase += (long long)idx * g.os[k];
    }
    const uint32_t nx = g.n[g.ax], ny = g.ay >= 0 ? g.n[g.ay] : 1u;
    const long long isx = g.is[g.ax];
    const long long isy = g.ay >= 0 ? g.is[g.ay] : 0, osy = g.ay >= 0 ? g.os[g.ay] : 0;
    const uint32_t x0 = tx * TR_TILE, y0 = ty * TR_TILE;
    const uint32_t first = (threadIdx.x % LANES) * VE, run = threadIdx.x / LANES;
    union Vec { nh_u32 w[4]; T e[VE]; };
    if constexpr (SWAP) {
        if (x0 + TR_TILE <= nx && y0 + TR_TILE <= ny) {
            // a whole tile: every load is issued before the first LDS store
            constexpr uint32_t K = TR_TILE / RUNS;
            Vec v[K];
#pragma unroll
            for (uint32_t k = 0; k < K; ++k)
                nh_load_words<4, true>(reinterpret_cast<const nh_u32*>(in + ibase + (long long)(x0 + run + k * RUNS) * isx +
                                                                       (long long)(y0 + first)), v[k].w);
#pragma unroll
            for (uint32_t k = 0; k < K; ++k)
#pragma unroll
                for (int j = 0; j < VE; ++j) tile[run + k * RUNS][first + j] = v[k].e[j];
            __syncthreads();
#pragma unroll
            for (uint32_t k = 0; k < K; ++k) {
                const uint32_t i = run + k * RUNS;
                Vec o;
#pragma unroll
                for (int j = 0; j < VE; ++j) o.e[j] = tile[first + j][i];
                nh_store_words<4, false>(reinterpret_cast<nh_u32*>(out + obase + (long long)(x0 + first) + (long long)(y0 + i) * osy),
                                         o.w);
            }
            return;
        }
        // input runs along y (isy == 1): run index = x
        for (uint32_t i = run; i < TR_TILE; i += RUNS) {
            const uint32_t x = x0 + i, y = y0 + first;
            if (x < nx && y < ny) {
                Vec v;
                nh_load_words<4, true>(reinterpret_cast<const nh_u32*>(in + ibase + (long long)x * isx + (long long)y), v.w);
#pragma unroll
                for (int j = 0; j < VE; ++j) tile[i][first + j] = v.e[j];
            }
        }
        __syncthreads();
        // output runs along x (stride 1): run index = y
        for (uint32_t i = run; i < TR_TILE; i += RUNS) {
            const uint32_t x = x0 + first, y = y0 + i;
            if (x < nx && y < ny) {
                Vec v;
#pragma unroll
                for (int j = 0; j < VE; ++j) v.e[j] = tile[first + j][i];
                nh_store_words<4, false>(reinterpret_cast<nh_u32*>(out + obase + (long long)x + (long long)y * osy), v.w);
            }
        }
    } else {
        for (uint32_t i = run; i < TR_TILE; i += RUNS) {
            const uint32_t x = x0 + first, y = y0 + i;
            if (x < nx && y < ny) {
                Vec v;
                nh_load_words<4, true>(reinterpret_cast<const nh_u32*>(in + ibase + (long long)x + (long long)y * isy), v.w);
                nh_store_words<4, false>(reinterpret_cast<nh_u32*>(out + obase + (long long)x + (long long)y * osy), v.w);
            }
        }
    }
}

template <typename T>
void launch_transpose_vec(void* out, const void* in, const TrGeom& g, bool swap, unsigned blocks, hipStream_t s) {
    if (swap)
        hipLaunchKernelGGL((transpose_tile_vec_kernel<T, true>), dim3(blocks), dim3(TR_T), 0, s, (T*)out, (const T*)in, g);
    else
        hipLaunchKernelGGL((transpose_tile_vec_kernel<T, false>), dim3(blocks), dim3(TR_T), 0, s, (T*)out, (const T*)in, g);
}

template <typename T>
void launch_transpose(void* out, const void* in, const TrGeom& g, bool swap, unsigned blocks, hipStream_t s) {
    if (swap)
        hipLaunchKernelGGL((transpose_tile_kernel<T, true>), dim3(blocks), dim3(TR_T), 0, s, (T*)out, (const T*)in, g);
    else
        hipLaunchKernelGGL((transpose_tile_kernel<T, false>), dim3(blocks), dim3(TR_T), 0, s, (T*)out, (const T*)in, g);
}


}  // namespace

// Called by nh_init with `device` current: every device holds its own copy of
// `scratch` at its own address.
int nh_internal_scratch_setup(int device) {
    if (device < 0 || device >= CR_MAX_DEVICES) return 0;      // such a device simply has no static entry point
    if (g_scratch_ptr[device]) return 0;
    void* ptr = nullptr;
    hipError_t e = hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return nh_internal_fail((int)e, "nh_init: address lookup of the static scratch area failed");
    }
    g_scratch_ptr[device] = ptr;
    return 0;
}

extern "C" {

int nh_ew_axpby_f32(float* out, const float* x, const float* y, float alpha, float beta, size_t n, void* stream) {
    if (n && (!out || !x || !y)) return nh_internal_fail(NH_EINVAL, "nh_ew_axpby_f32: null pointer");
    AxpbyF f{out, x, y, alpha, beta};
    return launch_ew(f, n, aligned16(out) && aligned16(x) && aligned16(y), stream, "nh_ew_axpby_f32");
}

int nh_ew_sigmoid_f32(float* out, const float* x, size_t n, void* stream) {
    if (n && (!out || !x)) return nh_internal_fail(NH_EINVAL, "nh_ew_sigmoid_f32: null pointer");
    SigmoidF f{out, x};
    return launch_ew(f, n, aligned16(out) && aligned16(x), stream, "nh_ew_sigmoid_f32");
}

int nh_adam_step_f32(float* param, float* m, float* v, const float* grad, float lr_t, float beta1,
                     float one_minus_beta1, float beta2, float one_minus_beta2, float eps, size_t n,
                     void* stream) {
    if (n && (!param || !m || !v || !grad)) return nh_internal_fail(NH_EINVAL, "nh_adam_step_f32: null pointer");
    AdamF f{param, m, v, grad, lr_t, beta1, one_minus_beta1, beta2, one_minus_beta2, eps};
    return launch_ew(f, n, aligned16(param) && aligned16(m) && aligned16(v) && aligned16(grad), stream,
                     "nh_adam_step_f32");
}

int nh_rownorm_f16(uint16_t* out, const uint16_t* x, const float* gamma, const float* beta, float eps,
                   uint32_t rows, uint32_t cols, size_t ld, void* stream) {
    if (!nh_internal_ready()) return nh_internal_fail(NH_ENOTINIT, "nh_init has not been called");
    if (rows == 0 || cols == 0) return 0;
    if (!out || !x || !gamma || !beta) return nh_internal_fail(NH_EINVAL, "nh_rownorm_f16: null pointer");
    if (cols > NH_ROWNORM_MAX_COLS) return nh_internal_fail(NH_EINVAL, "nh_rownorm_f16: row longer than NH_ROWNORM_MAX_COLS");
    if (cols % RN_V || ld % RN_V || ld < cols || !aligned16(out) || !aligned16(x))
        return nh_internal_fail(NH_EINVAL, "nh_rownorm_f16: cols and ld must be multiples of 8 and pointers 16-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    const uint32_t per_pass = RN_T * RN_V;
    const uint32_t nch = (cols + per_pass - 1) / per_pass;
    switch (nch) {
        case 1: launch_rownorm<1>(out, x, gamma, beta, eps, rows, cols, ld, s); break;
        case 2: launch_rownorm<2>(out, x, gamma, beta, eps, rows, cols, ld, s); break;
        case 3: case 4: launch_rownorm<4>(out, x, gamma, beta, eps, rows, cols, ld, s); break;
        case 5: case 6: launch_rownorm<6>(out, x, gamma, beta, eps, rows, cols, ld, s); break;
        case 7: case 8: launch_rownorm<8>(out, x, gamma, beta, eps, rows, cols, ld, s); break;
        case 9: case 10: launch_rownorm<10>(out, x, gamma, beta, eps, rows, cols, ld, s); break;
        case 11: case 12: case 13: launch_rownorm<13>(out, x, gamma, beta, eps, rows, cols, ld, s); break;
        default: launch_rownorm<16>(out, x, gamma, beta, eps, rows, cols, ld, s); break;
    }
    return launch_status("nh_rownorm_f16");
}

int nh_hist_log2(int32_t* hist, const void* x, int itemsize, size_t n, int nbins, int offset, void* stream) {
    if (!nh_internal_ready()) return nh_internal_fail(NH_ENOTINIT, "nh_init has not been called");
    if (!hist || (n && !x)) return nh_internal_fail(NH_EINVAL, "nh_hist_log2: null pointer");
    if (nbins < 1 || nbins > HIST_MAX_BINS) return nh_internal_fail(NH_EINVAL, "nh_hist_log2: nbins out of range");
    if (itemsize != 4 && itemsize != 2) return nh_internal_fail(NH_EINVAL, "nh_hist_log2: fp32 or fp16 input only");
    hipStream_t s = (hipStream_t)stream;
    hipError_t e = hipMemsetAsync(hist, 0, sizeof(int32_t) * (size_t)nbins, s);
    if (e != hipSuccess) return nh_internal_fail((int)e, "nh_hist_log2: clearing the bins failed");
    if (n == 0) return 0;
    size_t blocks = (n + HIST_T * 16 - 1) / ((size_t)HIST_T * 16);
    const size_t cap = (size_t)(nh_internal_cu_count() > 0 ? nh_internal_cu_count() : 256) * 4;
    if (blocks > cap) blocks = cap;
    if (blocks < 1) blocks = 1;
    // private 16-bit counters: at most 65535 elements per lane
    const bool priv = nbins <= HIST_PRIVATE_BINS && n / (blocks * HIST_T) < 60000;
    const dim3 grid((unsigned)blocks), block(HIST_T);
    const size_t cus = cap / 4;
    if (nbins <= HIST_PRIVATE_BINS && offset >= -126 && offset + nbins < 128 && n / (cus * HIST_WIDE_T) < 60000) {
        // one workgroup per compute unit, fewer while each would hold less than a stage of vectors per lane
        const size_t stage = (size_t)HIST_WIDE_T * 4 * HIST_STAGE, want = (n + stage - 1) / stage;
        const dim3 wgrid((unsigned)(want < cus ? want : cus)), wblock(HIST_WIDE_T);
        if (itemsize == 4) hipLaunchKernelGGL((hist_exponent_kernel<float, HIST_WIDE_T>), wgrid, wblock, 0, s, (const float*)x, n, nbins, offset, (int*)hist);
        else hipLaunchKernelGGL((hist_exponent_kernel<nh_f16, HIST_WIDE_T>), wgrid, wblock, 0, s, (const nh_f16*)x, n, nbins, offset, (int*)hist);
        return launch_status("nh_hist_log2");
    }
    if (itemsize == 4) {
        if (priv) hipLaunchKernelGGL((hist_log2_kernel<float, true>), grid, block, 0, s, (const float*)x, n, nbins, offset, (int*)hist);
        else hipLaunchKernelGGL((hist_log2_kernel<float, false>), grid, block, 0, s, (const float*)x, n, nbins, offset, (int*)hist);
    } else {
        if (priv) hipLaunchKernelGGL((hist_log2_kernel<nh_f16, true>), grid, block, 0, s, (const nh_f16*)x, n, nbins, offset, (int*)hist);
        else hipLaunchKernelGGL((hist_log2_kernel<nh_f16, false>), grid, block, 0, s, (const nh_f16*)x, n, nbins, offset, (int*)hist);
    }
    return launch_status("nh_hist_log2");
}

int nh_copy_transpose(void* out, const void* in, int itemsize, int ndim, const uint32_t* shape,
                      const int64_t* out_strides, const int64_t* in_strides, void* stream) {
    if (!nh_internal_ready()) return nh_internal_fail(NH_ENOTINIT, "nh_init has not been called");
    if (ndim < 1 || ndim > NH_TRANSPOSE_MAX_DIMS)
        return nh_internal_fail(NH_EINVAL, "nh_copy_transpose: ndim must be 1..NH_TRANSPOSE_MAX_DIMS");
    if (!shape || !out_strides || !in_strides) return nh_internal_fail(NH_EINVAL, "nh_copy_transpose: null geometry");
    if (itemsize != 1 && itemsize != 2 && itemsize != 4 && itemsize != 8)
        return nh_internal_fail(NH_EINVAL, "nh_copy_transpose: itemsize must be 1, 2, 4 or 8");
    TrGeom g;
    unsigned long long total = 1;
    for (int k = 0; k < ndim; ++k) {
        if (out_strides[k] < 0 || in_strides[k] < 0)
            return nh_internal_fail(NH_EINVAL, "nh_copy_transpose: negative stride");
        g.n[k] = shape[k];
        g.os[k] = out_strides[k];
        g.is[k] = in_strides[k];
        total *= shape[k];
    }
    if (total == 0) return 0;
    if (!out || !in) return nh_internal_fail(NH_EINVAL, "nh_copy_transpose: null pointer");
    g.nd = ndim;
    // ax: the dimension the output walks fastest; ay: the one the input walks
    // fastest (extent-1 dimensions never matter)
    int ax = -1, ay = -1;
    for (int k = 0; k < ndim; ++k) {
        if (g.n[k] == 1) continue;
        if (ax < 0 || g.os[k] < g.os[ax]) ax = k;
        if (ay < 0 || g.is[k] < g.is[ay]) ay = k;
    }
    if (ax < 0) ax = ay = ndim - 1;             // a single element
    bool swap = ax != ay;
    if (!swap) {
        // same fastest dimension on both sides: pair it with the next-fastest output dimension
        ay = -1;
        for (int k = 0; k < ndim; ++k) {
            if (k == ax || g.n[k] == 1) continue;
            if (ay < 0 || g.os[k] < g.os[ay]) ay = k;
        }
    }
    g.ax = ax;
    g.ay = ay;
    g.tiles_x = (g.n[ax] + TR_TILE - 1) / TR_TILE;
    g.tiles_y = ay >= 0 ? (g.n[ay] + TR_TILE - 1) / TR_TILE : 1u;
    unsigned long long blocks = (unsigned long long)g.tiles_x * g.tiles_y;
    for (int k = 0; k < ndim; ++k)
        if (k != ax && k != ay) blocks *= g.n[k];
    if (blocks > 0x7fffffffull) return nh_internal_fail(NH_EINVAL, "nh_copy_transpose: too many tiles for one launch");
    hipStream_t s = (hipStream_t)stream;
    if ((itemsize == 4 || itemsize == 2) && ay >= 0) {
        // 16-byte accesses when every run of VE elements is aligned on both sides
        const uint32_t ve = 16u / (uint32_t)itemsize;
        bool vec = aligned16(out) && aligned16(in) && g.n[ax] % ve == 0 && g.os[ax] == 1 &&
                   (swap ? (g.n[ay] % ve == 0 && g.is[ay] == 1) : g.is[ax] == 1);
        for (int k = 0; k < ndim && vec; ++k) {
            if (g.n[k] == 1) continue;
            if (k != ax && g.os[k] % ve) vec = false;
            if (k != (swap ? ay : ax) && g.is[k] % ve) vec = false;
        }
        if (vec) {
            if (itemsize == 4) launch_transpose_vec<uint32_t>(out, in, g, swap, (unsigned)blocks, s);
            else launch_transpose_vec<uint16_t>(out, in, g, swap, (unsigned)blocks, s);
            return launch_status("nh_copy_transpose");
        }
    }
    switch (itemsize) {
        case 1: launch_transpose<uint8_t>(out, in, g, swap, (unsigned)blocks, s); break;
        case 2: launch_transpose<uint16_t>(out, in, g, swap, (unsigned)blocks, s); break;
        case 4: launch_transpose<uint32_t>(out, in, g, swap, (unsigned)blocks, s); break;
        default: launch_transpose<unsigned long long>(out, in, g, swap, (unsigned)blocks, s); break;
    }
    return launch_status("nh_copy_transpose");
}

size_t nh_colreduce_workspace_bytes(uint32_t rows, uint32_t cols) {
    if (rows == 0 || cols == 0) return 0;
    // independent of the device and of which variant runs: the most chunks a launch may use
    return (size_t)CR_MAX_CHUNKS * (size_t)cols * sizeof(nh_pair) + 256;
}

static int colmax_launch(const char* who, float* maxval, int32_t* argmax, const float* x, uint32_t rows, uint32_t cols,
                         size_t ld, const CrPlan& p, nh_pair* part, unsigned int* tickets, hipStream_t s) {
    dim3 grid(p.strips, p.chunks);
    if (p.v == 4 && p.threads == 2 * CR_T)
        hipLaunchKernelGGL((colmax_kernel<4, 8, 2 * CR_T>), grid, dim3(2 * CR_T), 0, s, x, rows, cols, ld,
                           p.rows_per_chunk, part, maxval, (int*)argmax, tickets);
    else if (p.v == 4)
        hipLaunchKernelGGL((colmax_kernel<4, 8, CR_T>), grid, dim3(CR_T), 0, s, x, rows, cols, ld, p.rows_per_chunk, part,
                           maxval, (int*)argmax, tickets);
    else
        hipLaunchKernelGGL((colmax_kernel<1, 64, CR_T>), grid, dim3(CR_T), 0, s, x, rows, cols, ld, p.rows_per_chunk,
                           part, maxval, (int*)argmax, tickets);
    return launch_status(who);
}

static int colmax_check(const char* who, const float* maxval, const int32_t* argmax, const float* x, uint32_t rows,
                        uint32_t cols, size_t ld, CrPlan* plan) {
    if (!x || (!maxval && !argmax)) return nh_internal_fail(NH_EINVAL, (std::string(who) + ": null pointer").c_str());
    if (ld < cols) return nh_internal_fail(NH_EINVAL, (std::string(who) + ": ld < cols").c_str());
    if (rows > 0x7FFFFFFFu)
        return nh_internal_fail(NH_EINVAL, (std::string(who) + ": too many rows for an int32 index").c_str());
    const bool vec = (cols % 4 == 0) && (ld % 4 == 0);
    *plan = cr_plan(rows, cols, vec);
    if (plan->strips > CR_MAX_STRIPS) return nh_internal_fail(NH_EINVAL, (std::string(who) + ": too many columns").c_str());
    if (plan->chunks > 65535u) return nh_internal_fail(NH_EINVAL, (std::string(who) + ": grid too large").c_str());
    return 0;
}

int nh_colmax_argmax_f32(float* maxval, int32_t* argmax, const float* x, uint32_t rows, uint32_t cols, size_t ld,
                         void* workspace, void* stream) {
    if (!nh_internal_ready()) return nh_internal_fail(NH_ENOTINIT, "nh_init has not been called");
    if (rows == 0 || cols == 0) return 0;
    CrPlan p;
    if (int rc = colmax_check("nh_colmax_argmax_f32", maxval, argmax, x, rows, cols, ld, &p)) return rc;
    if (p.chunks > 1 && !workspace) return nh_internal_fail(NH_EINVAL, "nh_colmax_argmax_f32: workspace required");
    if (p.chunks > 1 && (reinterpret_cast<uintptr_t>(workspace) & 7u))
        return nh_internal_fail(NH_EINVAL, "nh_colmax_argmax_f32: workspace must be 8-byte aligned");
    unsigned int* tickets = nullptr;
    hipError_t e = hipGetSymbolAddress((void**)&tickets, HIP_SYMBOL(g_cr_tickets));
    if (e != hipSuccess) return nh_internal_fail((int)e, "nh_colmax_argmax_f32: ticket symbol lookup failed");
    return colmax_launch("nh_colmax_argmax_f32", maxval, argmax, x, rows, cols, ld, p, (nh_pair*)workspace, tickets,
                         (hipStream_t)stream);
}

int nh_colmax_argmax_f32_static(float* maxval, int32_t* argmax, const float* x, uint32_t rows, uint32_t cols,
                                size_t ld, void* stream) {
    if (!nh_internal_ready()) return nh_internal_fail(NH_ENOTINIT, "nh_init has not been called");
    if (rows == 0 || cols == 0) return 0;
    CrPlan p;
    if (int rc = colmax_check("nh_colmax_argmax_f32_static", maxval, argmax, x, rows, cols, ld, &p)) return rc;
    const int dev = nh_internal_device();
    if (dev < 0 || dev >= CR_MAX_DEVICES || !g_scratch_ptr[dev])
        return nh_internal_fail(NH_ENOTINIT, "nh_colmax_argmax_f32_static: no scratch area for this device");
    const size_t need = CR_STATIC_TICKET_BYTES + (p.chunks > 1 ? (size_t)p.chunks * cols * sizeof(nh_pair) : 0);
    if (need > (size_t)NH_STATIC_SCRATCH_BYTES)
        return nh_internal_fail(NH_EINVAL,
                                ("nh_colmax_argmax_f32_static: needs " + std::to_string(need) +
                                 " bytes of scratch, the static area holds " + std::to_string((size_t)NH_STATIC_SCRATCH_BYTES) +
                                 " (use nh_colmax_argmax_f32 with a workspace)").c_str());
    unsigned char* base = (unsigned char*)g_scratch_ptr[dev];
    unsigned int* tickets = (unsigned int*)base;
    nh_pair* part = (nh_pair*)(base + CR_STATIC_TICKET_BYTES);
    hipStream_t s = (hipStream_t)stream;
    if (p.chunks > 1) {
        // the area keeps whatever the last call left: tickets have to start at zero
        const uint32_t words = p.strips * CR_TICKET_STRIDE;
        hipLaunchKernelGGL(cr_clear_tickets_kernel, dim3((words + 255) / 256), dim3(256), 0, s, tickets, words);
        if (int rc = launch_status("nh_colmax_argmax_f32_static: clearing the tickets")) return rc;
    }
    return colmax_launch("nh_colmax_argmax_f32_static", maxval, argmax, x, rows, cols, ld, p, part, tickets, s);
}

}  // extern "C"
