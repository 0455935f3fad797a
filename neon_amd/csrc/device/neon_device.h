// neon_device.h -- device-side building blocks for gfx950 (CDNA4, wave64).
//
// Shared by the prebuilt kernels (compiled with hipcc) and by every kernel the
// op-tree code generator emits (this text is prepended to the generated source
// and compiled with hiprtc).  Nothing here includes a system header so the
// same text works in both places.
//
// Contents
//   * storage types and conversions: fp32 compute, fp16 / bf16 / integer storage
//   * 16-byte vector loads and stores
//   * per-op scalar semantics matching the numpy CPU backend of the reference
//     (neon/backends/nervanacpu.py:480-522)
//   * wave64 cross-lane reductions built on DPP, and the LDS step that
//     combines the waves of a workgroup
#ifndef NEON_DEVICE_H
#define NEON_DEVICE_H

#define NEON_WAVE 64
// accelerator complex dies of an MI355X: workgroups go to them round-robin in
// dispatch order, and each has an L2 of its own
#define NH_XCDS 8
#define NEON_DEV __device__ __forceinline__

typedef _Float16 nh_f16;
typedef __bf16 nh_bf16;
typedef signed char nh_i8;
typedef unsigned char nh_u8;
typedef short nh_i16;
typedef unsigned short nh_u16;
typedef int nh_i32;
typedef unsigned int nh_u32;

// Upper bound on the polls of a bounded wait for other workgroups (each poll
// is a device-scope load plus a short sleep, roughly a microsecond).
#define NH_SPIN_LIMIT (1u << 22)
// Left in a cooperative plan's status word by a workgroup whose bounded wait
// expired (it returns without results); the host looks for it at the next
// synchronisation.
#define NH_COOP_ABORTED 0xDEADu

#define NH_INF __builtin_inff()
#define NH_FLT_MAX 3.402823466e+38f

// ---------------------------------------------------------------------------
// storage <-> fp32
// Loads widen exactly.  Stores follow numpy's unsafe cast, which is what the
// CPU backend's `left[:] = right` does (nervanacpu.py:476-477): floating
// targets round to nearest even, integer targets truncate toward zero.
// ---------------------------------------------------------------------------
template <typename T> NEON_DEV float nh_load_cvt(T x) { return (float)x; }

template <typename T> struct nh_store_cvt;
template <> struct nh_store_cvt<float>   { static NEON_DEV float   f(float x) { return x; } };
template <> struct nh_store_cvt<nh_f16>  { static NEON_DEV nh_f16  f(float x) { return (nh_f16)x; } };
template <> struct nh_store_cvt<nh_bf16> { static NEON_DEV nh_bf16 f(float x) { return (nh_bf16)x; } };
template <> struct nh_store_cvt<nh_i32>  { static NEON_DEV nh_i32  f(float x) { return (nh_i32)x; } };
template <> struct nh_store_cvt<nh_u32>  { static NEON_DEV nh_u32  f(float x) { return (nh_u32)(long long)x; } };
template <> struct nh_store_cvt<nh_i16>  { static NEON_DEV nh_i16  f(float x) { return (nh_i16)(nh_i32)x; } };
template <> struct nh_store_cvt<nh_u16>  { static NEON_DEV nh_u16  f(float x) { return (nh_u16)(nh_i32)x; } };
template <> struct nh_store_cvt<nh_i8>   { static NEON_DEV nh_i8   f(float x) { return (nh_i8)(nh_i32)x; } };
template <> struct nh_store_cvt<nh_u8>   { static NEON_DEV nh_u8   f(float x) { return (nh_u8)(nh_i32)x; } };

// Index of a gather / scatter view, kept inside the indexed tensor.
NEON_DEV int nh_clamp_index(int i, int extent) { return i < 0 ? 0 : (i >= extent ? extent - 1 : i); }

// An index produced by argmax/argmin goes to an integer target unchanged and
// to a floating target as its value.
template <typename T> NEON_DEV T nh_store_index(int i) { return (T)i; }

// ---------------------------------------------------------------------------
// vector access: V consecutive elements, at most 16 bytes per instruction
// ---------------------------------------------------------------------------
template <typename T, int V> struct __attribute__((aligned(sizeof(T) * V > 16 ? 16 : sizeof(T) * V))) nh_vec {
    T v[V];
};

// NW consecutive 32-bit words, 16 bytes per instruction; NT = streaming access
// (non-temporal: the line is not kept in cache, for data touched once).
// The access types claim byte alignment only: global memory takes 16-byte
// instructions at any address (a tensor view that starts mid-row, rows whose
// length is not a multiple of the vector), at the same speed as aligned ones
// when the address happens to be aligned -- and 1.7x (fp32) to 2.9x (fp16) the
// speed of element-wise accesses when it is not.
typedef nh_u32 nh_u32x2 __attribute__((ext_vector_type(2)));
typedef nh_u32 nh_u32x4 __attribute__((ext_vector_type(4)));
typedef nh_u32 nh_u32_any __attribute__((aligned(1)));
typedef nh_u32x2 nh_u32x2_any __attribute__((aligned(1)));
typedef nh_u32x4 nh_u32x4_any __attribute__((aligned(1)));

// (elements of a vector value are copied to scalars before any bit cast: a
// bit cast applied directly to ``t.y`` reads ``t.x`` with this compiler)
template <typename T, int V> NEON_DEV void nh_load_vec(const T* __restrict__ p, T (&raw)[V]) {
    static_assert(sizeof(T) == 4, "word vectors only");
    nh_u32 w[V];
    if constexpr (V == 1) {
        w[0] = *reinterpret_cast<const nh_u32_any*>(p);
    } else if constexpr (V == 2) {
        const nh_u32x2 t = *reinterpret_cast<const nh_u32x2_any*>(p);
        w[0] = t.x; w[1] = t.y;
    } else {
#pragma unroll
        for (int i = 0; i < V; i += 4) {
            const nh_u32x4 t = *reinterpret_cast<const nh_u32x4_any*>(p + i);
            w[i] = t.x; w[i + 1] = t.y; w[i + 2] = t.z; w[i + 3] = t.w;
        }
    }
#pragma unroll
    for (int j = 0; j < V; ++j) raw[j] = __builtin_bit_cast(T, w[j]);
}

template <typename T, int V> NEON_DEV void nh_store_vec(T* p, const T (&raw)[V]) {
    static_assert(sizeof(T) == 4, "word vectors only");
    nh_u32 w[V];
#pragma unroll
    for (int j = 0; j < V; ++j) w[j] = __builtin_bit_cast(nh_u32, raw[j]);
    if constexpr (V == 1) {
        *reinterpret_cast<nh_u32_any*>(p) = w[0];
    } else if constexpr (V == 2) {
        nh_u32x2 t; t.x = w[0]; t.y = w[1];
        *reinterpret_cast<nh_u32x2_any*>(p) = t;
    } else {
#pragma unroll
        for (int i = 0; i < V; i += 4) {
            nh_u32x4 t; t.x = w[i]; t.y = w[i + 1]; t.z = w[i + 2]; t.w = w[i + 3];
            *reinterpret_cast<nh_u32x4_any*>(p + i) = t;
        }
    }
}

template <int NW, bool NT> NEON_DEV void nh_load_words(const nh_u32* p, nh_u32 (&w)[NW]) {
    if constexpr (!NT) {
        nh_load_vec<nh_u32, NW>(p, w);
    } else if constexpr (NW == 1) {
        w[0] = __builtin_nontemporal_load(reinterpret_cast<const nh_u32_any*>(p));
    } else if constexpr (NW == 2) {
        const nh_u32x2 t = __builtin_nontemporal_load(reinterpret_cast<const nh_u32x2_any*>(p));
        w[0] = t.x; w[1] = t.y;
    } else {
#pragma unroll
        for (int i = 0; i < NW; i += 4) {
            const nh_u32x4 t = __builtin_nontemporal_load(reinterpret_cast<const nh_u32x4_any*>(p + i));
            w[i] = t.x; w[i + 1] = t.y; w[i + 2] = t.z; w[i + 3] = t.w;
        }
    }
}
template <int NW, bool NT> NEON_DEV void nh_store_words(nh_u32* p, const nh_u32 (&w)[NW]) {
    if constexpr (!NT) {
        nh_store_vec<nh_u32, NW>(p, w);
    } else if constexpr (NW == 1) {
        __builtin_nontemporal_store(w[0], reinterpret_cast<nh_u32_any*>(p));
    } else if constexpr (NW == 2) {
        nh_u32x2 t; t.x = w[0]; t.y = w[1];
        __builtin_nontemporal_store(t, reinterpret_cast<nh_u32x2_any*>(p));
    } else {
#pragma unroll
        for (int i = 0; i < NW; i += 4) {
            nh_u32x4 t; t.x = w[i]; t.y = w[i + 1]; t.z = w[i + 2]; t.w = w[i + 3];
            __builtin_nontemporal_store(t, reinterpret_cast<nh_u32x4_any*>(p + i));
        }
    }
}

// Packed 16-bit storage kept in 32-bit registers (two elements per register).
typedef nh_f16 nh_f16x2 __attribute__((ext_vector_type(2)));
NEON_DEV float nh_f16_lo(nh_u32 w) { return (float)__builtin_bit_cast(nh_f16x2, w).x; }
NEON_DEV float nh_f16_hi(nh_u32 w) { return (float)__builtin_bit_cast(nh_f16x2, w).y; }
NEON_DEV nh_u32 nh_f16_pack(float lo, float hi) {
    nh_f16x2 h; h.x = (nh_f16)lo; h.y = (nh_f16)hi;
    return __builtin_bit_cast(nh_u32, h);
}
// acc + lo + hi of a packed fp16 pair in one instruction (v_dot2c_f32_f16 with
// a pair of ones; fp32 accumulation)
NEON_DEV float nh_sum2_f16(nh_u32 w, float acc) {
    nh_f16x2 ones; ones.x = (nh_f16)1.0f; ones.y = (nh_f16)1.0f;
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(nh_f16x2, w), ones, acc, false);
}
// 1.0f the compiler cannot see through.  fma(x, one, y) with x widened from
// fp16 selects v_fma_mix_f32 -- widening and the addition in ONE instruction,
// same result as (float)x + y -- where a plain x + y would be folded back into
// a conversion followed by an add.
NEON_DEV float nh_opaque_one() { float one; asm volatile("v_mov_b32 %0, 1.0" : "=v"(one)); return one; }
NEON_DEV float nh_bf16_lo(nh_u32 w) { return __builtin_bit_cast(float, w << 16); }
NEON_DEV float nh_bf16_hi(nh_u32 w) { return __builtin_bit_cast(float, w & 0xFFFF0000u); }
// Compiler barrier on register-resident data: the values are unchanged but
// treated as new, so work derived from them before the call (e.g. widened
// copies) is not kept alive across it.
template <int N> NEON_DEV void nh_keep_packed(nh_u32 (&w)[N]) {
#pragma unroll
    for (int j = 0; j < N; ++j) asm volatile("" : "+v"(w[j]));
}

// ---------------------------------------------------------------------------
// Register tiles.  nh_raw<T,V> holds V consecutive elements of storage type T
// exactly as they sit in memory (32-bit words, 16-bit types two per word), so
// a tile that stays resident across several sweeps costs V*sizeof(T)/4
// registers; get(j) widens one element to fp32 on use.  nh_out<T,V> is the
// store-side mirror: set(j, x) narrows, store() writes the words.
// When V*sizeof(T) is not a multiple of 4 (V == 1 with a narrow type) the
// single element lives in word 0.
// ---------------------------------------------------------------------------
template <typename T> struct nh_is_float { static constexpr bool value = false; };
template <> struct nh_is_float<float> { static constexpr bool value = true; };
template <> struct nh_is_float<nh_f16> { static constexpr bool value = true; };
template <> struct nh_is_float<nh_bf16> { static constexpr bool value = true; };

template <typename T> NEON_DEV nh_u32 nh_bits_of(T x) {
    if constexpr (sizeof(T) == 4) return __builtin_bit_cast(nh_u32, x);
    else if constexpr (sizeof(T) == 2) return (nh_u32)__builtin_bit_cast(nh_u16, x);
    else return (nh_u32)__builtin_bit_cast(nh_u8, x);
}
template <typename T> NEON_DEV T nh_from_bits(nh_u32 b) {
    if constexpr (sizeof(T) == 4) return __builtin_bit_cast(T, b);
    else if constexpr (sizeof(T) == 2) return __builtin_bit_cast(T, (nh_u16)b);
    else return __builtin_bit_cast(T, (nh_u8)b);
}

template <typename T, int V> struct nh_raw {
    static constexpr int BYTES = (int)sizeof(T) * V;
    static constexpr bool PACKED = (BYTES % 4) == 0;
    static constexpr int NW = PACKED ? BYTES / 4 : 1;
    static constexpr int PER = 4 / (int)sizeof(T);  // elements per word
    nh_u32 w[NW];

    NEON_DEV void load(const T* p) {
        if constexpr (PACKED) nh_load_vec<nh_u32, NW>(reinterpret_cast<const nh_u32*>(p), w);
        else w[0] = nh_bits_of<T>(*p);
    }
    NEON_DEV void load_stream(const T* p) {      // touched once: do not keep in cache
        if constexpr (PACKED) nh_load_words<NW, true>(reinterpret_cast<const nh_u32*>(p), w);
        else w[0] = nh_bits_of<T>(__builtin_nontemporal_load(p));
    }
    NEON_DEV void zero() {
#pragma unroll
        for (int i = 0; i < NW; ++i) w[i] = 0u;
    }
    NEON_DEV float get(int j) const {
        const nh_u32 word = w[PACKED ? j / PER : 0];
        const int sub = PACKED ? j % PER : 0;
        const nh_u32 bits = (sizeof(T) == 4) ? word : (word >> (8 * (int)sizeof(T) * sub));
        return (float)nh_from_bits<T>(bits);
    }
    NEON_DEV int geti(int j) const {  // integer view, for index tensors
        const nh_u32 word = w[PACKED ? j / PER : 0];
        const int sub = PACKED ? j % PER : 0;
        const nh_u32 bits = (sizeof(T) == 4) ? word : (word >> (8 * (int)sizeof(T) * sub));
        return (int)nh_from_bits<T>(bits);
    }
    NEON_DEV void keep() {
#pragma unroll
        for (int i = 0; i < NW; ++i) asm volatile("" : "+v"(w[i]));
    }
    // acc + all V elements of a packed fp16 tile, two elements per instruction
    NEON_DEV float sum_into(float acc) const {
        static_assert(sizeof(T) == 2 && PACKED, "packed 16-bit tiles only");
#pragma unroll
        for (int i = 0; i < NW; ++i) acc = nh_sum2_f16(w[i], acc);
        return acc;
    }
    // the first n (< V) elements, one at a time; the rest of the tile is zero
    NEON_DEV void load_partial(const T* p, int n) {
        zero();
#pragma unroll
        for (int j = 0; j < V; ++j) {
            if (j < n) {
                const nh_u32 bits = nh_bits_of<T>(p[j]);
                if constexpr (sizeof(T) == 4) w[PACKED ? j : 0] = bits;
                else w[PACKED ? j / PER : 0] |= bits << (8 * (int)sizeof(T) * (PACKED ? j % PER : 0));
            }
        }
    }
    // reuse the registers of a float tile for a value derived from it
    NEON_DEV void put(int j, float v) {
        static_assert(sizeof(T) == 4, "one word per element only");
        w[j] = nh_bits_of<float>(v);
    }
};

template <typename T, int V> struct nh_out {
    static constexpr int BYTES = (int)sizeof(T) * V;
    static constexpr bool PACKED = (BYTES % 4) == 0;
    static constexpr int NW = PACKED ? BYTES / 4 : 1;
    static constexpr int PER = 4 / (int)sizeof(T);
    nh_u32 w[NW];

    NEON_DEV void clear() {
#pragma unroll
        for (int i = 0; i < NW; ++i) w[i] = 0u;
    }
    NEON_DEV void put_bits(int j, nh_u32 bits) {
        if constexpr (sizeof(T) == 4) w[PACKED ? j : 0] = bits;
        else w[PACKED ? j / PER : 0] |= bits << (8 * (int)sizeof(T) * (PACKED ? j % PER : 0));
    }
    NEON_DEV void set(int j, float x) {
        if constexpr (sizeof(T) == 2 && PACKED && nh_is_float<T>::value) {
            // element insert into the pair (with a compile-time j, a conversion that
            // writes its half of the register directly)
            typedef T pair_t __attribute__((ext_vector_type(2)));
            pair_t v = __builtin_bit_cast(pair_t, w[j / 2]);
            if (j & 1) v.y = nh_store_cvt<T>::f(x); else v.x = nh_store_cvt<T>::f(x);
            w[j / 2] = __builtin_bit_cast(nh_u32, v);
        } else {
            put_bits(j, nh_bits_of<T>(nh_store_cvt<T>::f(x)));
        }
    }
    NEON_DEV void seti(int j, int i) { put_bits(j, nh_bits_of<T>(nh_store_index<T>(i))); }
    NEON_DEV void store(T* p) const {
        if constexpr (PACKED) nh_store_vec<nh_u32, NW>(reinterpret_cast<nh_u32*>(p), w);
        else *p = nh_from_bits<T>(w[0]);
    }
    NEON_DEV void store_stream(T* p) const {
        if constexpr (PACKED) nh_store_words<NW, true>(reinterpret_cast<nh_u32*>(p), w);
        else __builtin_nontemporal_store(nh_from_bits<T>(w[0]), p);
    }
    // the first n (< V) elements, one at a time
    NEON_DEV void store_partial(T* p, int n) const {
#pragma unroll
        for (int j = 0; j < V; ++j) {
            if (j < n) {
                const nh_u32 word = w[PACKED ? j / PER : 0];
                const nh_u32 bits = (sizeof(T) == 4) ? word : (word >> (8 * (int)sizeof(T) * (PACKED ? j % PER : 0)));
                p[j] = nh_from_bits<T>(bits);
            }
        }
    }
};

// value after a round trip through storage type T (what a later read of a
// just-written tensor would see)
template <typename T> NEON_DEV float nh_quant(float x) { return (float)nh_store_cvt<T>::f(x); }

// ---------------------------------------------------------------------------
// scalar op semantics (CPU-backend flavour where the two backends of the
// reference differ: safelog clamps its argument, sign(nan) is nan,
// minimum/maximum and max/min reductions propagate nan like numpy)
// ---------------------------------------------------------------------------
// IEEE-754-2019 maximum / minimum: NaN if either operand is NaN, which is what
// numpy's maximum / max do; one v_maximum3_f32 / v_minimum3_f32 on gfx950.
NEON_DEV float nh_max(float a, float b) { return __builtin_elementwise_maximum(a, b); }
NEON_DEV float nh_min(float a, float b) { return __builtin_elementwise_minimum(a, b); }
NEON_DEV float nh_sgn(float x) { return (x != x) ? x : (float)((x > 0.0f) - (x < 0.0f)); }
NEON_DEV float nh_sqr(float x) { return x * x; }
NEON_DEV float nh_safelog(float x) { return logf(nh_max(x, 1.9287498479639178e-22f)); }  // exp(-50)
NEON_DEV float nh_tanh2(float x) { const float e = exp2f(2.0f * x); return (e - 1.0f) / (e + 1.0f); }
NEON_DEV float nh_finite(float x) { return (__builtin_fabsf(x) <= NH_FLT_MAX) ? 1.0f : 0.0f; }
// x / d for a divisor that is constant along the loop the quotient varies in (a
// row's standard deviation, a column's softmax sum): the reciprocal and the
// test are loop invariants, leaving a multiply per element instead of an IEEE
// division (about ten instructions); at most 1.5 units in the last place from
// the quotient.  Where 1/d is not a normal number (d zero, denormal, huge,
// infinite or NaN) the quotient is computed as written.
NEON_DEV float nh_div_by_line(float x, float d) {
    const float r = 1.0f / d;
    const float ar = __builtin_fabsf(r);
    float q = x * r;
    if (__builtin_expect(!(ar <= NH_FLT_MAX) || ar < 1.17549435e-38f, 0)) {
        // (the empty statement keeps this a branch: as a select the compiler evaluated the
        // division for every element -- 64 of them per lane in a softmax down 1000 rows, more
        // than a third of the kernel's vector instructions)
        asm volatile("");
        q = x / d;
    }
    return q;
}

// Counter-based random numbers.  Word `w` of the stream `seed` is one half of
// splitmix64(w >> 1): stateless, so a tensor filled twice from the same
// (seed, counter) gets the same values whatever the kernel's tiling, and no
// generator state lives on the device (the reference kept a pool of LFSR
// states, cuda_templates.py:138-186).  The two 64-bit multiplies dominate the
// cost of a dropout mask, hence two words per evaluation.
NEON_DEV unsigned long long nh_splitmix64(nh_u32 seed, unsigned long long index) {
    unsigned long long z = index + ((unsigned long long)seed + 1ull) * 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
// Word w0 + j * STRIDE + OFF.  With ALIGNED the caller guarantees that w0 is
// even: the pair index then is (w0 >> 1) plus a compile-time constant once j
// is unrolled, and neighbouring words share one evaluation.
template <int STRIDE, int OFF, bool ALIGNED>
NEON_DEV nh_u32 nh_rand_word(nh_u32 seed, unsigned long long w0, int j) {
    const int rel = j * STRIDE + OFF;
    unsigned long long z;
    bool high;
    if constexpr (ALIGNED) {
        z = nh_splitmix64(seed, (w0 >> 1) + (unsigned long long)(rel >> 1));
        high = (rel & 1) != 0;
    } else {
        const unsigned long long w = w0 + (unsigned long long)rel;
        z = nh_splitmix64(seed, w >> 1);
        high = (w & 1ull) != 0;
    }
    return high ? (nh_u32)(z >> 32) : (nh_u32)z;
}
// uniform in [0, 1) from the top 24 bits of a random word
NEON_DEV float nh_rand01(nh_u32 word) { return (float)(word >> 8) * 5.9604644775390625e-8f; }      // 2^-24

// Stochastic rounding to `bits` (1..22) mantissa bits with the random word
// `rnd`: the value moves to the neighbour of larger magnitude with probability
// equal to the fraction of the spacing it sits above the neighbour of smaller
// magnitude, so the result is unbiased (the reference adds a uniform fraction
// of the spacing with round-toward-zero and masks, cuda_templates.py:148-152,
// 193-235).  Done on the bit pattern: random bits added below the kept
// mantissa bits carry into them (and on into the exponent) with exactly that
// probability.  Infinities and NaN pass through.
NEON_DEV float nh_sround(float x, int bits, nh_u32 rnd) {
    const nh_u32 b = __builtin_bit_cast(nh_u32, x);
    if ((b & 0x7f800000u) == 0x7f800000u) return x;
    const int drop = 23 - bits;
    const nh_u32 noise = rnd >> (32 - drop);
    return __builtin_bit_cast(float, (b + noise) & (0xffffffffu << drop));
}

// Stochastic rounding to a whole number (stores into signed integer tensors;
// the reference adds a uniform fraction with the value's sign, rounding toward
// zero, and truncates: cuda_templates.py:236-286).  x = n + f with n = trunc(x):
// the result is n, or the next whole number away from zero with probability
// |f| -- decided by comparing |f| with a uniform 24-bit fraction, every step
// exact, so the expectation is x.  The store then converts an integral value.
NEON_DEV float nh_sround_int(float x, nh_u32 rnd) {
    const float n = __builtin_truncf(x);
    const float f = __builtin_fabsf(x - n);
    return (nh_rand01(rnd) < f) ? n + __builtin_copysignf(1.0f, x) : n;
}

// ---------------------------------------------------------------------------
// DPP lane permutations.  Every lane of the wave must be active at the call.
// ---------------------------------------------------------------------------
#define NH_DPP_XOR1 0xB1        // quad_perm:[1,0,3,2]
#define NH_DPP_XOR2 0x4E        // quad_perm:[2,3,0,1]
#define NH_DPP_HALF_MIRROR 0x141  // lane i <-> 7-i inside each group of 8
#define NH_DPP_MIRROR 0x140     // lane i <-> 15-i inside each row of 16
#define NH_SWIZZLE_XOR16 0x401F // ds_swizzle bit mode: and 0x1f, or 0, xor 0x10

template <int CTRL> NEON_DEV float nh_dpp(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}
template <int CTRL> NEON_DEV int nh_dpp(int v) {
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, false);
}
NEON_DEV float nh_swz16(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), NH_SWIZZLE_XOR16));
}
NEON_DEV int nh_swz16(int v) { return __builtin_amdgcn_ds_swizzle(v, NH_SWIZZLE_XOR16); }
template <int LANE> NEON_DEV float nh_readlane(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), LANE));
}
template <int LANE> NEON_DEV int nh_readlane(int v) { return __builtin_amdgcn_readlane(v, LANE); }

// ---------------------------------------------------------------------------
// reduction operators.  A value-reduction carries one float; an arg-reduction
// carries (value, index) and breaks ties toward the lower index, which is what
// np.argmax / np.argmin return (first occurrence).
// ---------------------------------------------------------------------------
struct nh_op_sum { static NEON_DEV float init() { return 0.0f; }      static NEON_DEV float f(float a, float b) { return a + b; } };
struct nh_op_max { static NEON_DEV float init() { return -NH_INF; }   static NEON_DEV float f(float a, float b) { return nh_max(a, b); } };
struct nh_op_min { static NEON_DEV float init() { return NH_INF; }    static NEON_DEV float f(float a, float b) { return nh_min(a, b); } };

struct __attribute__((aligned(8))) nh_pair { float v; int i; };
// NaN follows numpy (np.argmax / np.argmin return the position of the first
// NaN when there is one, as np.max / np.min return NaN): a NaN beats every
// number and an earlier NaN beats a later one.
struct nh_op_argmax {
    static NEON_DEV nh_pair init() { nh_pair p; p.v = -NH_INF; p.i = 0; return p; }
    static NEON_DEV nh_pair f(nh_pair a, nh_pair b) {
        const bool an = a.v != a.v, bn = b.v != b.v;
        const bool take_b = bn ? (!an || b.i < a.i) : (!an && ((b.v > a.v) || (b.v == a.v && b.i < a.i)));
        nh_pair r; r.v = take_b ? b.v : a.v; r.i = take_b ? b.i : a.i; return r;
    }
    // sequential update with strictly increasing indices keeps the first hit:
    // !(v <= a.v) holds for a larger value and for a NaN on either side; a NaN
    // already held (a.v != a.v) stays
    static NEON_DEV void step(nh_pair& a, float v, int i) { if (!(v <= a.v) && (a.v == a.v)) { a.v = v; a.i = i; } }
    // N elements at once, x[k] sitting at index i0 + k * stride (increasing): one maximum per
    // element, then -- only when the batch beats what is held -- a scan for the first
    // position of that maximum (of the first NaN when there is one)
    template <int N> static NEON_DEV void stepn(nh_pair& a, const float (&x)[N], int i0, int stride) {
        float m = x[0];
#pragma unroll
        for (int k = 1; k < N; ++k) m = nh_max(m, x[k]);
        if (!(m <= a.v) && (a.v == a.v)) {
            int k0 = N - 1;
            if (__builtin_expect(m != m, 0)) {
#pragma unroll
                for (int k = N - 2; k >= 0; --k) k0 = (x[k] != x[k]) ? k : k0;
            } else {
#pragma unroll
                for (int k = N - 2; k >= 0; --k) k0 = (x[k] == m) ? k : k0;
            }
            a.v = m; a.i = i0 + k0 * stride;
        }
    }
};
struct nh_op_argmin {
    static NEON_DEV nh_pair init() { nh_pair p; p.v = NH_INF; p.i = 0; return p; }
    static NEON_DEV nh_pair f(nh_pair a, nh_pair b) {
        const bool an = a.v != a.v, bn = b.v != b.v;
        const bool take_b = bn ? (!an || b.i < a.i) : (!an && ((b.v < a.v) || (b.v == a.v && b.i < a.i)));
        nh_pair r; r.v = take_b ? b.v : a.v; r.i = take_b ? b.i : a.i; return r;
    }
    static NEON_DEV void step(nh_pair& a, float v, int i) { if (!(v >= a.v) && (a.v == a.v)) { a.v = v; a.i = i; } }
    template <int N> static NEON_DEV void stepn(nh_pair& a, const float (&x)[N], int i0, int stride) {
        float m = x[0];
#pragma unroll
        for (int k = 1; k < N; ++k) m = nh_min(m, x[k]);
        if (!(m >= a.v) && (a.v == a.v)) {
            int k0 = N - 1;
            if (__builtin_expect(m != m, 0)) {
#pragma unroll
                for (int k = N - 2; k >= 0; --k) k0 = (x[k] != x[k]) ? k : k0;
            } else {
#pragma unroll
                for (int k = N - 2; k >= 0; --k) k0 = (x[k] == m) ? k : k0;
            }
            a.v = m; a.i = i0 + k0 * stride;
        }
    }
};

// An arg-reduction's (value, index) as ONE 64-bit key whose unsigned order is the
// reduction's preference -- high word: the value mapped to an unsigned integer that
// grows with it (argmax) or shrinks with it (argmin), -0 taken as +0, any NaN as
// the largest key; low word: ~index, so that among equal values the lower index
// wins.  Merging two keys is a 64-bit maximum (three instructions, no branches),
// which is what every stage after a lane's own sweep uses: lane exchanges, the
// join of the waves, the partials between workgroups.  Carried in an nh_pair
// (v = bits of the high word, i = low word).
NEON_DEV nh_u32 nh_ordered_bits(float v) {
    const nh_u32 u = __builtin_bit_cast(nh_u32, v + 0.0f);
    return u ^ ((nh_u32)((int)u >> 31) | 0x80000000u);
}
template <class OP> NEON_DEV nh_pair nh_arg_key(nh_pair p);
template <> NEON_DEV nh_pair nh_arg_key<nh_op_argmax>(nh_pair p) {
    const nh_u32 k = (p.v != p.v) ? 0xFFFFFFFFu : nh_ordered_bits(p.v);
    nh_pair r; r.v = __builtin_bit_cast(float, k); r.i = ~p.i; return r;
}
template <> NEON_DEV nh_pair nh_arg_key<nh_op_argmin>(nh_pair p) {
    const nh_u32 k = (p.v != p.v) ? 0xFFFFFFFFu : ~nh_ordered_bits(p.v);
    nh_pair r; r.v = __builtin_bit_cast(float, k); r.i = ~p.i; return r;
}
NEON_DEV int nh_key_index(nh_pair k) { return ~k.i; }
struct nh_op_key {
    static NEON_DEV nh_pair init() { nh_pair p; p.v = __builtin_bit_cast(float, 0u); p.i = 0; return p; }
    static NEON_DEV nh_pair f(nh_pair a, nh_pair b) {
        const unsigned long long ka = ((unsigned long long)__builtin_bit_cast(nh_u32, a.v) << 32) | (nh_u32)a.i;
        const unsigned long long kb = ((unsigned long long)__builtin_bit_cast(nh_u32, b.v) << 32) | (nh_u32)b.i;
        return (kb > ka) ? b : a;
    }
};

// Running log-sum-exp state of a column: v = maximum so far, i = the bits of
// s = sum of exp(x - v) over the elements seen.  Carried as an nh_pair so that
// it travels through the same lane exchanges, LDS slots and partial buffers
// as an arg-reduction.  Merging two states rescales both sums to the larger
// maximum: (m, s) + (m', s') = (M, s e^(m-M) + s' e^(m'-M)), M = max(m, m').
// A state that has seen nothing (or only -inf) has v = -inf: its sum is then
// taken as 0 instead of evaluating exp(-inf + inf).  NaN and +inf propagate
// as in the two-sweep form (the sum becomes NaN).
NEON_DEV float nh_lse_sum(nh_pair p) { return __builtin_bit_cast(float, p.i); }
// The finished sum, as the two-sweep evaluation has it: where every element was
// -inf that one adds up exp(-inf - -inf) = NaN terms.
NEON_DEV float nh_lse_total(nh_pair p) { return (p.v == -NH_INF) ? __builtin_nanf("") : nh_lse_sum(p); }
// exp(d) for d <= 0 (a term of a sum whose largest term is 1): the product
// d * log2(e) is carried in two pieces so that the result is good to about a
// unit in the last place, like expf, at half its instruction count; what
// expf spends on results below the normal range is left out -- such terms
// vanish next to the 1.  NaN comes back as NaN, -inf as 0.
NEON_DEV float nh_exp_nonpos(float d) {
    d = nh_max(d, -150.0f);
    const float t = d * 1.44269502e+00f;
    float e = __builtin_fmaf(d, 1.44269502e+00f, -t);
    e = __builtin_fmaf(d, 1.92596299e-08f, e);
    const float r = __builtin_amdgcn_exp2f(t);
    return __builtin_fmaf(r, e * 6.93147182e-01f, r);
}
// 1 / d for d in [1, 2]: the hardware's estimate and one Newton step, within
// a unit in the last place, in place of the ten instructions of a division.
NEON_DEV float nh_rcp_1to2(float d) {
    const float r = __builtin_amdgcn_rcpf(d);
    return __builtin_fmaf(__builtin_fmaf(-d, r, 1.0f), r, r);
}
// Logistic function 1 / (1 + e^-x), from e = e^-|x| in (0, 1]: 1 / (1 + e) for
// x >= 0 and e / (1 + e) below -- no overflow on either side, and about half
// the instructions of expf followed by a division (which bound fused gate
// expressions on 16-bit tensors).  Within 3 units in the last place; results
// below the normal range (x < -87) are flushed towards zero.  NaN stays NaN.
NEON_DEV float nh_sig(float x) {
    const float e = nh_exp_nonpos(-__builtin_fabsf(x));
    const float r = nh_rcp_1to2(1.0f + e);
    return (x >= 0.0f) ? r : e * r;
}
// the same on base 2: 1 / (1 + 2^-x)
NEON_DEV float nh_sig2(float x) {
    const float e = __builtin_amdgcn_exp2f(nh_max(-__builtin_fabsf(x), -150.0f));
    const float r = nh_rcp_1to2(1.0f + e);
    return (x >= 0.0f) ? r : e * r;
}
// exp(d), d <= 0, as one TERM of a sum of such exponentials: the plain product with
// log2(e) (off by up to |d| * 9e-8 relative).  In the sum every term's error is weighted
// by the term itself, e^d * |d| <= 1/e, so the sum stays within 1e-7 relative of the sum
// of exactly rounded terms whatever the number of terms -- at a third of the instructions.
NEON_DEV float nh_exp_term(float d) {
#ifdef NH_EXACT_LSE_TERMS
    return nh_exp_nonpos(d);
#else
    return __builtin_amdgcn_exp2f(d * 1.44269502e+00f);
#endif
}
struct nh_op_lse {
    static NEON_DEV nh_pair init() { nh_pair p; p.v = -NH_INF; p.i = 0; return p; }    // bits of +0.0f
    // the state with the larger maximum keeps its sum, the other one's is scaled by
    // e^(smaller - larger): one exponential per merge, a term of the sum like any other
    static NEON_DEV nh_pair f(nh_pair a, nh_pair b) {
        const float m = nh_max(a.v, b.v);
        const float lo = nh_min(a.v, b.v);
        const float mz = (m == -NH_INF) ? 0.0f : m;
        const bool a_top = a.v >= b.v;
        const float s_top = a_top ? nh_lse_sum(a) : nh_lse_sum(b);
        const float s_low = a_top ? nh_lse_sum(b) : nh_lse_sum(a);
        const float s = __builtin_fmaf(s_low, nh_exp_term(lo - mz), s_top);
        nh_pair r; r.v = m; r.i = __builtin_bit_cast(int, s); return r;
    }
    static NEON_DEV void step(nh_pair& a, float x) {
        const float m = nh_max(a.v, x);
        const float mz = (m == -NH_INF) ? 0.0f : m;
        const float s = nh_lse_sum(a) * nh_exp_nonpos(a.v - mz) + nh_exp_nonpos(x - mz);
        a.v = m; a.i = __builtin_bit_cast(int, s);
    }
    // N elements at once: one rescaling of the running sum for all of them
    template <int N> static NEON_DEV void stepn(nh_pair& a, const float (&x)[N]) {
        float m = a.v;
#pragma unroll
        for (int k = 0; k < N; ++k) m = nh_max(m, x[k]);
        const float mz = (m == -NH_INF) ? 0.0f : m;
        float s = nh_lse_sum(a) * nh_exp_nonpos(a.v - mz);
#pragma unroll
        for (int k = 0; k < N; ++k) s += nh_exp_term(x[k] - mz);
        a.v = m; a.i = __builtin_bit_cast(int, s);
    }
};

// ---------------------------------------------------------------------------
// Hand-off of partial results between workgroups (possibly on another XCD,
// behind another L2).
//
// Producer: nh_part_store (8-byte relaxed device-scope atomic store: written
// through to device-coherent memory), then nh_publish_barrier, then one lane
// bumps the strip's counter with nh_ticket_take / nh_arrive.
// Consumer: reads the counter (its own nh_ticket_take result, or nh_arrivals in
// a bounded wait), a workgroup barrier, then nh_part_load (relaxed device-scope
// atomic load: served from device-coherent memory, never from a stale line).
//
// Ordering.  The partial stores must be performed at device scope before the
// counter update is.  Default build: every storing lane waits for its own
// outstanding vector-memory operations (s_waitcnt vmcnt(0): on this part a
// device-scope write-through store is acknowledged only once performed at
// device scope), then the workgroup barrier, then the counter atomic -- so the
// counter cannot be seen ahead of a partial.  This leans on that hardware
// behaviour rather than on the language's memory model, which would want a
// device-scope release before the counter update and an acquire after reading
// it; those compile to a write-back and an invalidate of the whole L2, and
// cost more than the kernels they sit in.  Defining NH_FORMAL_FENCES builds
// exactly that variant (for comparison and for parts where the assumption
// does not hold).
// ---------------------------------------------------------------------------
#ifndef NH_FORMAL_FENCES
#define NH_FORMAL_FENCES 0
#endif
NEON_DEV void nh_part_store(nh_pair* p, nh_pair v) {
    __hip_atomic_store(reinterpret_cast<unsigned long long*>(p), __builtin_bit_cast(unsigned long long, v),
                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
NEON_DEV nh_pair nh_part_load(const nh_pair* p) {
    return __builtin_bit_cast(nh_pair, __hip_atomic_load(reinterpret_cast<const unsigned long long*>(p),
                                                         __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
}
// A tag in bit 31 of a record's second word: free for float partials (the word is unused), for
// arg-reduction keys (the word is ~index with index < 2^31, so the bit is always 1 and is put back)
// and for (max, sum) pairs (the word holds the bits of a sum >= 0; a NaN loses its sign).
NEON_DEV nh_pair nh_tag_put(nh_pair p, nh_u32 tag) { p.i = (int)(((nh_u32)p.i & 0x7fffffffu) | (tag << 31)); return p; }
NEON_DEV bool nh_tag_is(nh_pair p, nh_u32 tag) { return ((nh_u32)p.i >> 31) == tag; }
// All threads of the workgroup call it, after the last nh_part_store.
NEON_DEV void nh_publish_barrier() {
#if NH_FORMAL_FENCES
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
#else
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#endif
    __syncthreads();
}
// Counter update after nh_publish_barrier; returns the count before.
NEON_DEV nh_u32 nh_ticket_take(nh_u32* ctr) {
#if NH_FORMAL_FENCES
    return __hip_atomic_fetch_add(ctr, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
#else
    return __hip_atomic_fetch_add(ctr, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#endif
}
NEON_DEV nh_u32 nh_arrivals(const nh_u32* ctr) {
#if NH_FORMAL_FENCES
    return __hip_atomic_load(ctr, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT);
#else
    return __hip_atomic_load(ctr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#endif
}
NEON_DEV void nh_ticket_reset(nh_u32* ctr) {
    __hip_atomic_store(ctr, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <int CTRL> NEON_DEV nh_pair nh_dpp(nh_pair p) { nh_pair r; r.v = nh_dpp<CTRL>(p.v); r.i = nh_dpp<CTRL>(p.i); return r; }
NEON_DEV nh_pair nh_swz16(nh_pair p) { nh_pair r; r.v = nh_swz16(p.v); r.i = nh_swz16(p.i); return r; }
template <int LANE> NEON_DEV nh_pair nh_readlane(nh_pair p) { nh_pair r; r.v = nh_readlane<LANE>(p.v); r.i = nh_readlane<LANE>(p.i); return r; }

// Exchange with the lane whose index differs in bit log2(S).  Strides below 32
// use ds_swizzle in bit mode (crossbar only, no LDS memory); 32 crosses the two
// halves of the wave with ds_bpermute.
template <int S> NEON_DEV int nh_lane_xor(int v) {
    if constexpr (S < 32) return __builtin_amdgcn_ds_swizzle(v, 0x1F | (S << 10));
    else return __builtin_amdgcn_ds_bpermute((int)((__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)) ^ 32u) << 2), v);
}
template <int S> NEON_DEV float nh_lane_xor(float v) {
    return __builtin_bit_cast(float, nh_lane_xor<S>(__builtin_bit_cast(int, v)));
}
template <int S> NEON_DEV nh_pair nh_lane_xor(nh_pair p) {
    nh_pair r; r.v = nh_lane_xor<S>(p.v); r.i = nh_lane_xor<S>(p.i); return r;
}

// Fold, over the lanes of a wave that share (lane % LX), LEN values per lane.
// While a lane carries more than one value each step halves them: partners
// (lane ^ S) split the values between them, each sends the half the other
// keeps.  V values cost V - 1 + (steps - log2 V) exchanges instead of
// V * steps; afterwards a lane holds a[0 .. V >> halvings) for elements
// j0, j0 + 1, ... of its column tile, j0 (returned through `j0`) given by the
// lane's bits at the halving strides.
template <class OP, int LEN, int S, typename T> NEON_DEV void nh_fold_step(T* a, int lane, int& j0) {
    if constexpr (S < 64) {
        if constexpr (LEN > 1) {
            constexpr int H = LEN / 2;
            const bool up = (lane & S) != 0;
#pragma unroll
            for (int m = 0; m < H; ++m) {
                const T send = up ? a[m] : a[m + H];
                const T keep = up ? a[m + H] : a[m];
                a[m] = OP::f(keep, nh_lane_xor<S>(send));
            }
            j0 += up ? H : 0;
            nh_fold_step<OP, H, S * 2, T>(a, lane, j0);
        } else {
            a[0] = OP::f(a[0], nh_lane_xor<S>(a[0]));
            nh_fold_step<OP, 1, S * 2, T>(a, lane, j0);
        }
    }
}
template <class OP, int V, int LX, typename T> NEON_DEV int nh_col_wave_fold(T (&a)[V]) {
    int j0 = 0;
    nh_fold_step<OP, V, LX, T>(a, (int)(threadIdx.x & 63u), j0);
    return j0;
}

// All-reduce over aligned groups of WIDTH lanes (WIDTH in 1,2,4,...,64): every
// lane of a group ends with the group's result.  Steps 1-2 are quad
// permutes; steps 4 and 8 use the mirror patterns, valid because the previous
// steps made each group of 4 / 8 lanes uniform; 16 uses ds_swizzle (no LDS
// memory is touched); 64 finishes through four scalar lane reads.
template <class OP, int WIDTH, typename T> NEON_DEV T nh_wave_allreduce(T v) {
    if (WIDTH >= 2) v = OP::f(v, nh_dpp<NH_DPP_XOR1>(v));
    if (WIDTH >= 4) v = OP::f(v, nh_dpp<NH_DPP_XOR2>(v));
    if (WIDTH >= 8) v = OP::f(v, nh_dpp<NH_DPP_HALF_MIRROR>(v));
    if (WIDTH >= 16) v = OP::f(v, nh_dpp<NH_DPP_MIRROR>(v));
    if (WIDTH == 32) v = OP::f(v, nh_swz16(v));
    if (WIDTH == 64) {
        const T a = nh_readlane<0>(v), b = nh_readlane<16>(v), c = nh_readlane<32>(v), d = nh_readlane<48>(v);
        v = OP::f(OP::f(a, b), OP::f(c, d));
    }
    return v;
}

// Workgroup all-reduce: DPP inside each wave, then one LDS slot per wave.
// `slots` must hold NWAVES entries of T; the two barriers make the buffer
// reusable by the next call.  All threads of the workgroup must call it.
template <class OP, int NWAVES, typename T> NEON_DEV T nh_block_allreduce(T v, T* slots) {
    v = nh_wave_allreduce<OP, 64>(v);
    if (NWAVES == 1) return v;
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) slots[wave] = v;
    __syncthreads();
    T r = slots[0];
#pragma unroll
    for (int w = 1; w < NWAVES; ++w) r = OP::f(r, slots[w]);
    __syncthreads();
    return r;
}

#endif  // NEON_DEVICE_H
