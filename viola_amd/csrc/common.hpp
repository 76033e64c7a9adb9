// Device helpers shared by every kernel file: storage-type loads/stores, OCP FP8
// codecs, Philox4x32-10, wavefront reductions. gfx950 only (64-wide wavefronts).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/viola_hip.h"

#define VIOLA_CHECK_ARG(cond) \
    do {                      \
        if (!(cond)) return VIOLA_EINVAL; \
    } while (0)

// Launches go through hipLaunchKernel, whose return value is the launch's own status; the first failure of an
// entry point's launches is kept per thread and handed out (and cleared) by viola_launch_status(). The runtime's
// last-error slot is never read or cleared: it may hold another library's error, and reading it is a call an
// entry point has no need to make while a stream is being captured.
inline thread_local int viola_first_launch_error = 0;

template <typename... Params, typename... Args>
static inline void viola_launch(void (*kernel)(Params...), dim3 grid, dim3 block, unsigned lds_bytes, hipStream_t stream,
                                Args&&... args) {
    static_assert(sizeof...(Params) == sizeof...(Args), "one argument per kernel parameter");
    [&](Params... values) {
        void* slots[] = {const_cast<void*>(static_cast<const void*>(&values))...};
        const hipError_t e = hipLaunchKernel(reinterpret_cast<const void*>(kernel), grid, block, slots, lds_bytes, stream);
        if (e != hipSuccess && viola_first_launch_error == 0) viola_first_launch_error = (int)e;
    }(static_cast<Params>(args)...);
}
#define VIOLA_LAUNCH(kernel, grid, block, lds_bytes, stream, ...) viola_launch(kernel, grid, block, lds_bytes, stream, __VA_ARGS__)

static inline int viola_launch_status() {
    const int e = viola_first_launch_error;
    viola_first_launch_error = 0;
    return e;
}

// First statement of an entry point: the caller's stream, and a clean launch status. A call that launched and then
// left through an argument check never collected its status; the next call on that thread must not inherit it.
static inline hipStream_t viola_enter(viola_stream_t stream) {
    viola_first_launch_error = 0;
    return static_cast<hipStream_t>(stream);
}

static inline bool viola_is_fp8(int dtype) { return dtype == VIOLA_E4M3 || dtype == VIOLA_E5M2; }
static inline bool viola_is_float(int dtype) { return dtype == VIOLA_F32 || dtype == VIOLA_BF16 || dtype == VIOLA_F16; }
static inline int viola_dtype_size(int dtype) { return dtype == VIOLA_F32 ? 4 : (dtype == VIOLA_BF16 || dtype == VIOLA_F16) ? 2 : 1; }

namespace viola {

constexpr int WAVE = 64;

// ------------------------------------------------------------------ storage types
struct bf16_t { uint16_t bits; };
struct f16_t { _Float16 value; };
struct e4m3_t { uint8_t bits; };
struct e5m2_t { uint8_t bits; };

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t bits) { return __uint_as_float(bits << 16); }

// Round-to-nearest-even, NaN -> quiet NaN with the sign dropped (the rule of PyTorch's cast).
// v_cvt_pk_bf16_f32: round to nearest even, identical to the usual add-0x7fff arithmetic on every input
// that is not NaN (checked over all 2^32 patterns); a NaN keeps its sign and top payload bits.
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float x) { return __builtin_bit_cast(uint16_t, (__bf16)x); }
__device__ __forceinline__ uint32_t f32_to_bf16x2_bits(float lo, float hi) {
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    const f32x2_t pair = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(pair, bf16x2_t));
}

// ------------------------------------------------------------------ FP8 (OCP) codecs
// Software encoders: exact RNE onto the grid. e4m3fn has no Inf: anything that
// rounds above 448 becomes NaN (0x7f), as in PyTorch's cast; callers clamp first
// where the reference clamps.
__device__ __forceinline__ uint8_t f32_to_e4m3(float x) {
    uint32_t u = __float_as_uint(x);
    const uint32_t sign = (u >> 24) & 0x80u;
    u &= 0x7fffffffu;
    uint32_t r;
    if (u >= 0x43f00000u) {                       // >= 480, Inf, NaN
        r = 0x7f;
    } else if (u < 0x3c800000u) {                 // < 2^-6: subnormal target, spacing 2^-9
        const float magic = __uint_as_float(141u << 23);
        r = __float_as_uint(__uint_as_float(u) + magic) - (141u << 23);
    } else {
        const uint32_t odd = (u >> 20) & 1u;
        u += ((uint32_t)(7 - 127) << 23) + 0x7ffffu + odd;
        r = u >> 20;
    }
    return (uint8_t)(r | sign);
}

__device__ __forceinline__ uint8_t f32_to_e5m2(float x) {
    uint32_t u = __float_as_uint(x);
    const uint32_t sign = (u >> 24) & 0x80u;
    u &= 0x7fffffffu;
    uint32_t r;
    if (u >= (143u << 23)) {                      // >= 65536, Inf, NaN
        r = u > 0x7f800000u ? 0x7f : 0x7c;
    } else if (u < (113u << 23)) {                // < 2^-14: subnormal target, spacing 2^-16
        const float magic = __uint_as_float(134u << 23);
        r = __float_as_uint(__uint_as_float(u) + magic) - (134u << 23);
    } else {
        const uint32_t odd = (u >> 21) & 1u;
        u += ((uint32_t)(15 - 127) << 23) + 0xfffffu + odd;
        r = u >> 21;
    }
    return (uint8_t)(r | sign);
}

__device__ __forceinline__ float e4m3_to_f32(uint32_t c) {
    const uint32_t sign = (c & 0x80u) << 24;
    const uint32_t mag = c & 0x7fu;
    float v;
    if (mag == 0x7f) v = __uint_as_float(0x7fc00000u);
    else if (mag < 8) v = (float)mag * 0x1p-9f;
    else v = __uint_as_float((mag << 20) + (120u << 23));
    return __uint_as_float(__float_as_uint(v) | sign);
}

__device__ __forceinline__ float e5m2_to_f32(uint32_t c) {
    const uint32_t sign = (c & 0x80u) << 24;
    const uint32_t mag = c & 0x7fu;
    float v;
    if (mag >= 0x7c) v = __uint_as_float(mag == 0x7c ? 0x7f800000u : 0x7fc00000u);
    else if (mag < 4) v = (float)mag * 0x1p-16f;
    else v = __uint_as_float((mag << 21) + (112u << 23));
    return __uint_as_float(__float_as_uint(v) | sign);
}

template <typename T> __device__ __forceinline__ float to_f32(T v);
template <> __device__ __forceinline__ float to_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_f32<bf16_t>(bf16_t v) { return bf16_bits_to_f32(v.bits); }
template <> __device__ __forceinline__ float to_f32<f16_t>(f16_t v) { return (float)v.value; }
template <> __device__ __forceinline__ float to_f32<e4m3_t>(e4m3_t v) { return e4m3_to_f32(v.bits); }
template <> __device__ __forceinline__ float to_f32<e5m2_t>(e5m2_t v) { return e5m2_to_f32(v.bits); }

template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float v) { return bf16_t{f32_to_bf16_bits(v)}; }
template <> __device__ __forceinline__ f16_t from_f32<f16_t>(float v) { return f16_t{(_Float16)v}; }
template <> __device__ __forceinline__ e4m3_t from_f32<e4m3_t>(float v) { return e4m3_t{f32_to_e4m3(v)}; }
template <> __device__ __forceinline__ e5m2_t from_f32<e5m2_t>(float v) { return e5m2_t{f32_to_e5m2(v)}; }

template <typename T> struct fp8_traits;
template <> struct fp8_traits<e4m3_t> { static constexpr float max = 448.0f; };
template <> struct fp8_traits<e5m2_t> { static constexpr float max = 57344.0f; };

// ------------------------------------------------------------------ many quotients by one divisor
// v / s for values that share the divisor s (a quantization group), bit for bit the IEEE quotient at
// three operations per value instead of a full division: with r = RN(1/s), t0 = RN(v r) and the exact
// residual e = v - s t0 (one FMA), RN(t0 + e r) is the correctly rounded v / s (Markstein). The argument
// needs the residual to be exact, which fails when it underflows (tiny s), when s has an all-ones
// significand (then RN(1/s) is not close enough), and for non-finite operands; `fast` is false in those
// cases and the caller divides. `poison` is any value that is NaN iff the group holds a NaN or an Inf
// (see poison_of).
struct SharedDivisor {
    float s, r;
    bool fast;
    __device__ __forceinline__ SharedDivisor(float divisor, float poison) : s(divisor) {
        const uint32_t bits = __float_as_uint(divisor);
        // 2^-80 <= s < 2^126, significand not all ones, no NaN/Inf in the group
        fast = bits >= (47u << 23) && bits < (253u << 23) && (bits & 0x7fffffu) != 0x7fffffu && poison == poison;
        // One Newton step on the hardware reciprocal (1 ulp) is the correctly rounded 1/s for every s in that domain:
        // checked over all of them on the device.
        const float y0 = __builtin_amdgcn_rcpf(divisor);
        r = fmaf(fmaf(-divisor, y0, 1.0f), y0, y0);
    }
    __device__ __forceinline__ float quotient(float v) const {
        const float t0 = v * r;
        const float e = -fmaf(t0, s, -v);        // this order of signs keeps -0 / s = -0
        return fmaf(e, r, t0);
    }
};
// amax / limit for the group scale. For the two FP8 maxima the reciprocal route is exact for every amax >= 1e-30
// (checked over all floats on the device); any other limit divides.
__device__ __forceinline__ float scale_of(float amax, float limit) {
    const float a = fmaxf(amax, 1e-30f);
    if ((limit == 448.0f || limit == 57344.0f) && a < __uint_as_float(0x7f800000u)) {        // an infinite amax divides
        const float r = limit == 448.0f ? 1.0f / 448.0f : 1.0f / 57344.0f;
        const float t0 = a * r;
        return fmaf(-fmaf(t0, limit, -a), r, t0);
    }
    return a / limit;
}
__device__ __forceinline__ float poison_of(float acc, float v) { return fmaf(v, 0.0f, acc); }

// Four values -> four FP8 codes in one word with the gfx950 converters. They agree with f32_to_e4m3 /
// f32_to_e5m2 (torch's casts) on every input that is not NaN; NaN comes out as 0xff / 0xfe instead of
// 0x7f | sign, so callers use them only on groups without NaN.
template <typename T> __device__ __forceinline__ uint32_t hw_encode4(float a, float b, float c, float d);
template <> __device__ __forceinline__ uint32_t hw_encode4<e4m3_t>(float a, float b, float c, float d) {
    int w = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
    return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(c, d, w, true);
}
template <> __device__ __forceinline__ uint32_t hw_encode4<e5m2_t>(float a, float b, float c, float d) {
    int w = __builtin_amdgcn_cvt_pk_bf8_f32(a, b, 0, false);
    return (uint32_t)__builtin_amdgcn_cvt_pk_bf8_f32(c, d, w, true);
}
// clamp(v / s, +-limit) -> code, four at a time, for a group whose divisor took the fast path
template <typename T>
__device__ __forceinline__ uint32_t fast_encode4(const SharedDivisor& d, float limit, float a, float b, float c, float e) {
    return hw_encode4<T>(__builtin_amdgcn_fmed3f(d.quotient(a), -limit, limit), __builtin_amdgcn_fmed3f(d.quotient(b), -limit, limit),
                         __builtin_amdgcn_fmed3f(d.quotient(c), -limit, limit), __builtin_amdgcn_fmed3f(d.quotient(e), -limit, limit));
}

// The same without the clamp, for groups whose scale is max |v| / limit with limit the format's largest finite value:
// a quotient is then at most limit in all but its last place, and everything below the first value that rounds past
// the largest code (464 for e4m3, 61440 for e5m2) converts to that code, which is what the clamp would give.
template <typename T>
__device__ __forceinline__ uint32_t fast_encode4_unclamped(const SharedDivisor& d, float a, float b, float c, float e) {
    return hw_encode4<T>(d.quotient(a), d.quotient(b), d.quotient(c), d.quotient(e));
}

// max of two pairs of 16-bit unsigned values (one v_pk_max_u16)
__device__ __forceinline__ uint32_t pk_max_u16(uint32_t a, uint32_t b) {
    typedef unsigned short u16x2_t __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(u16x2_t, a), __builtin_bit_cast(u16x2_t, b)));
}

// ------------------------------------------------------------------ group scales and the clamped encoder
template <typename TOut>
__device__ __forceinline__ uint8_t encode_clamped(float v, float s, float limit) {
    const float t = v / s;
    const float c = t != t ? t : fminf(fmaxf(t, -limit), limit);
    return from_f32<TOut>(c).bits;
}

// amax / limit, or for E8M0 scales the smallest power of two that is not below it (the reference's
// exp2(ceil(log2(s))), viola/nn/_grouped_kernels.py:81-83, evaluated exactly on the bits)
__device__ __forceinline__ float group_scale(float amax, float limit, int e8m0 = 0) {
    const float s = scale_of(amax, limit);
    if (!e8m0) return s;
    const uint32_t bits = __float_as_uint(s);
    if ((bits & 0x7f800000u) == 0x7f800000u) return s;                          // Inf / NaN stay
    return __uint_as_float((bits & 0x7f800000u) + ((bits & 0x007fffffu) ? 0x00800000u : 0u));
}
// a scale goes out as FP32 or as its biased exponent byte (log2(s) + 127, _grouped_kernels.py:85)
__device__ __forceinline__ void put_scale(float* scale, int64_t index, float s, int e8m0) {
    if (e8m0) reinterpret_cast<uint8_t*>(scale)[index] = (uint8_t)(__float_as_uint(s) >> 23);
    else scale[index] = s;
}
__device__ __forceinline__ float get_scale(const float* scale, int64_t index, int e8m0) {
    return e8m0 ? __uint_as_float((uint32_t)reinterpret_cast<const uint8_t*>(scale)[index] << 23) : scale[index];
}

// ------------------------------------------------------------------ wavefront reductions
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int offset = WAVE / 2; offset > 0; offset >>= 1) v = fmaxf(v, __shfl_xor(v, offset, WAVE));
    return v;
}

// The value of the lane whose index differs in bit 0 (OFFSET 1) or bit 1 (OFFSET 2): a DPP quad permute, which stays
// in the vector ALU (a shuffle goes through the LDS crossbar and its wait).
template <int OFFSET> __device__ __forceinline__ float quad_xor(float v) {
    static_assert(OFFSET == 1 || OFFSET == 2, "inside a quad of lanes");
    if constexpr (OFFSET == 1) return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0xB1, 0xf, 0xf, true));   // lanes 1 0 3 2
    else return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x4E, 0xf, 0xf, true));                        // lanes 2 3 0 1
}

// max over aligned sub-groups of WIDTH lanes (WIDTH a power of two <= 64)
template <int WIDTH> __device__ __forceinline__ float group_max(float v) {
#pragma unroll
    for (int offset = WIDTH / 2; offset > 2; offset >>= 1) v = fmaxf(v, __shfl_xor(v, offset, WAVE));
    if constexpr (WIDTH >= 4) v = fmaxf(v, quad_xor<2>(v));
    if constexpr (WIDTH >= 2) v = fmaxf(v, quad_xor<1>(v));
    return v;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int offset = WAVE / 2; offset > 0; offset >>= 1) v += __shfl_xor(v, offset, WAVE);
    return v;
}

// ------------------------------------------------------------------ Philox4x32-10 + stochastic rounding
// counter = (element_lo, element_hi, step_lo, step_hi), key = (key_lo, key_hi); word 0.
__device__ __forceinline__ uint32_t philox(uint64_t element, uint64_t step, uint64_t key) {
    uint32_t a = (uint32_t)element, b = (uint32_t)(element >> 32), c = (uint32_t)step, d = (uint32_t)(step >> 32);
    uint32_t k0 = (uint32_t)key, k1 = (uint32_t)(key >> 32);
#pragma unroll
    for (int round = 0; round < 10; ++round) {
        const uint32_t lo0 = 0xD2511F53u * a, hi0 = __umulhi(0xD2511F53u, a);
        const uint32_t lo1 = 0xCD9E8D57u * c, hi1 = __umulhi(0xCD9E8D57u, c);
        a = hi1 ^ b ^ k0; b = lo1; c = hi0 ^ d ^ k1; d = lo0;
        k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
    }
    return a;
}

__device__ __forceinline__ bool finite_f32(float x) { return (__float_as_uint(x) & 0x7f800000u) != 0x7f800000u; }

// Stochastic rounding onto a grid with MANT explicit mantissa bits and minimum spacing 2^MIN_EXP.
template <int MANT, int MIN_EXP>
__device__ __forceinline__ float stochastic_grid(float x, uint64_t element, uint64_t step, uint64_t key) {
    const float a = fabsf(x);
    const int exponent = (int)((__float_as_uint(a) >> 23) & 255u) - 127;
    const int e = exponent - MANT > MIN_EXP ? exponent - MANT : MIN_EXP;
    const float spacing = __uint_as_float((uint32_t)(e + 127) << 23);
    const float lower = floorf(a / spacing) * spacing;
    const float probability = (a - lower) / spacing;
    const float uniform = (float)(philox(element, step, key) >> 8) * 0x1p-24f;
    return copysignf(lower + (uniform < probability ? spacing : 0.0f), x);
}

__device__ __forceinline__ float stochastic_e4m3(float x, uint64_t element, uint64_t step, uint64_t key) {
    return finite_f32(x) ? stochastic_grid<3, -9>(x, element, step, key) : x;
}

__device__ __forceinline__ float stochastic_bf16(float x, uint64_t element, uint64_t step, uint64_t key) {
    if (!finite_f32(x)) return x;
    return __uint_as_float((__float_as_uint(x) + (philox(element, step, key) >> 16)) & 0xffff0000u);
}

__device__ __forceinline__ float stochastic_fp16(float x, uint64_t element, uint64_t step, uint64_t key) {
    if (!finite_f32(x) || fabsf(x) > 65504.0f) return x;
    return stochastic_grid<10, -24>(x, element, step, key);
}

// Store a fp32 result in storage type T, optionally with stochastic rounding (bf16 / fp16 only).
template <typename T, bool STOCHASTIC>
__device__ __forceinline__ T round_store(float v, uint64_t element, uint64_t step, uint64_t key) {
    if constexpr (STOCHASTIC && sizeof(T) == 2) {
        if constexpr (__is_same(T, bf16_t)) v = stochastic_bf16(v, element, step, key);
        else v = stochastic_fp16(v, element, step, key);
    }
    return from_f32<T>(v);
}

// act(g) and act'(g) of a gated MLP as the gated GEMM epilogues write them (viola/nn/_mlp_kernels.py:158-194), shared by
// the epilogues and by the passes that stand in for them, so both give the same bits. (The stand-alone forward operator
// writes silu as g / (1 + exp(-g)), viola/nn/_gated_kernels.py:29-35, which differs in the last place.)
__device__ __forceinline__ void gate_math(int activation, float g, float& act, float& derivative) {
    if (activation == VIOLA_SILU) {
        const float s = 1.0f / (1.0f + expf(-g));
        act = g * s;
        derivative = s * (1.0f + g * (1.0f - s));
    } else if (activation == VIOLA_GELU) {
        const float t = tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g));
        act = 0.5f * g * (1.0f + t);
        derivative = 0.5f * (1.0f + t) + 0.5f * g * (1.0f - t * t) * 0.7978845608028654f * (1.0f + 0.134145f * g * g);
    } else {
        act = fmaxf(g, 0.0f);
        derivative = g > 0.0f ? 1.0f : 0.0f;
    }
}

}  // namespace viola
