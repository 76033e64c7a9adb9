// Newton-Schulz GEMM chain for gfx950: batched bf16 / fp16 GEMM on v_mfma_f32_32x32x16_{bf16,f16}
// with the polynomial / residual epilogues fused, plus the Frobenius normalisation that starts
// the chain. Built with -ffp-contract=off so the fp32 epilogue is mul, mul, add.
//
// GEMM: block 256 threads = 2 x 2 wavefronts, tile 128 x 128 x 64, two LDS stages. As in the FP8
// GEMM the b matrix is the MFMA "A" operand so a lane owns one output row m and runs of four
// consecutive n. b may be given as [n, k] (transpose_b) or [k, n]; the latter is transposed on
// its way into LDS.
#include <type_traits>
#include <atomic>
#include <mutex>

#include "ns_args.hpp"

namespace viola {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

constexpr int NBM = 128, NBN = 128, NBK = 64, NLD = NBK + 8;   // LDS row stride in elements

template <bool IS_BF16>
__device__ __forceinline__ f32x16 mfma_half(uint4 x, uint4 y, f32x16 c) {
    if constexpr (IS_BF16) return __builtin_amdgcn_mfma_f32_32x32x16_bf16(*reinterpret_cast<bf16x8*>(&x), *reinterpret_cast<bf16x8*>(&y), c, 0, 0, 0);
    else return __builtin_amdgcn_mfma_f32_32x32x16_f16(*reinterpret_cast<f16x8*>(&x), *reinterpret_cast<f16x8*>(&y), c, 0, 0, 0);
}

template <bool IS_BF16> __device__ __forceinline__ float half_to_f32(uint16_t bits) {
    if constexpr (IS_BF16) return bf16_bits_to_f32(bits);
    else { _Float16 h; __builtin_memcpy(&h, &bits, 2); return (float)h; }
}
template <bool IS_BF16> __device__ __forceinline__ uint16_t f32_to_half(float v) {
    if constexpr (IS_BF16) return f32_to_bf16_bits(v);
    else { _Float16 h = (_Float16)v; uint16_t bits; __builtin_memcpy(&bits, &h, 2); return bits; }
}

// VEC: every row of a, b, residual and out starts 16-byte aligned and k (and n for [k, n] b) is a
// multiple of 8, so 16-byte global accesses are legal.
template <bool IS_BF16, bool TRANSPOSE_B, int EPILOGUE, bool VEC>
__global__ __launch_bounds__(256, 2) void ns_gemm_kernel(const uint16_t* __restrict__ a, const uint16_t* __restrict__ b,
                                                          const uint16_t* __restrict__ residual, uint16_t* __restrict__ out,
                                                          uint16_t* __restrict__ out_diag, int64_t m, int64_t n, int64_t k,
                                                          float add_diag, int transpose_out) {
    __shared__ __attribute__((aligned(16))) uint16_t lds_a[2][NBM * NLD];
    __shared__ __attribute__((aligned(16))) uint16_t lds_b[2][NBN * NLD];
    const int tid = threadIdx.x, lane = tid % WAVE, wave = tid / WAVE;
    const int wm = wave / 2, wn = wave % 2, l32 = lane % 32, lhi = lane / 32;
    const int64_t m0 = (int64_t)blockIdx.y * NBM, n0 = (int64_t)blockIdx.x * NBN;
    const int64_t bz = blockIdx.z;
    a += bz * m * k;
    b += bz * n * k;
    out += bz * m * n;
    if (out_diag) out_diag += bz * m * n;
    if (EPILOGUE) residual += bz * m * n;

    uint4 ra[4], rb[4];
    auto load8 = [&](const uint16_t* base, int64_t row, int64_t rows, int64_t ld, int64_t col, int64_t cols) -> uint4 {
        // 8 consecutive elements of a row-major matrix, zero outside [rows, cols]
        if (row >= rows || col >= cols) return make_uint4(0, 0, 0, 0);
        if constexpr (VEC) {
            return *reinterpret_cast<const uint4*>(base + row * ld + col);
        } else {
            uint32_t w[4] = {0, 0, 0, 0};
            for (int i = 0; i < 8; ++i)
                if (col + i < cols) w[i / 2] |= (uint32_t)base[row * ld + col + i] << (16 * (i % 2));
            return make_uint4(w[0], w[1], w[2], w[3]);
        }
    };
    auto fetch = [&](int64_t k0) {
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            const int id = it * 256 + tid;
            const int lr = id / 8, c = id % 8;                       // 128 rows x 8 chunks of 8 k
            ra[it] = load8(a, m0 + lr, m, k, k0 + c * 8, k);
            if constexpr (TRANSPOSE_B) {
                rb[it] = load8(b, n0 + lr, n, k, k0 + c * 8, k);
            } else {
                const int kr = id / 16, cn = id % 16;                // 64 k rows x 16 chunks of 8 n
                rb[it] = load8(b, k0 + kr, k, n, n0 + cn * 8, n);
            }
        }
    };
    auto stash = [&](int s) {
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            const int id = it * 256 + tid;
            const int lr = id / 8, c = id % 8;
            *reinterpret_cast<uint4*>(&lds_a[s][lr * NLD + c * 8]) = ra[it];
            if constexpr (TRANSPOSE_B) {
                *reinterpret_cast<uint4*>(&lds_b[s][lr * NLD + c * 8]) = rb[it];
            } else {
                const int kr = id / 16, cn = id % 16;
                const uint32_t w[4] = {rb[it].x, rb[it].y, rb[it].z, rb[it].w};
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    lds_b[s][(cn * 8 + i) * NLD + kr] = (uint16_t)(w[i / 2] >> (16 * (i % 2)));
            }
        }
    };

    f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    const int64_t chunks = (k + NBK - 1) / NBK;
    if (chunks > 0) {
        fetch(0);
        stash(0);
    }
    __syncthreads();
    for (int64_t chunk = 0; chunk < chunks; ++chunk) {
        const int s = (int)(chunk & 1);
        if (chunk + 1 < chunks) fetch((chunk + 1) * NBK);
#pragma unroll
        for (int ks = 0; ks < NBK / 16; ++ks) {
            const int koff = ks * 16 + lhi * 8;
            uint4 opb[2], opa[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) opb[i] = *reinterpret_cast<const uint4*>(&lds_b[s][(wn * 64 + i * 32 + l32) * NLD + koff]);
#pragma unroll
            for (int j = 0; j < 2; ++j) opa[j] = *reinterpret_cast<const uint4*>(&lds_a[s][(wm * 64 + j * 32 + l32) * NLD + koff]);
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) acc[i][j] = mfma_half<IS_BF16>(opb[i], opa[j], acc[i][j]);
        }
        if (chunk + 1 < chunks) stash(s ^ 1);
        __syncthreads();
    }

#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int64_t row = m0 + wm * 64 + j * 32 + l32;
        if (row >= m) continue;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                const int64_t col = n0 + wn * 64 + i * 32 + r4 * 8 + lhi * 4;
                uint16_t res[4] = {0, 0, 0, 0}, o[4], od[4];
                const bool full = VEC && col + 3 < n;
                if (EPILOGUE) {
                    if (full) {
                        const uint2 raw = *reinterpret_cast<const uint2*>(residual + row * n + col);
                        res[0] = (uint16_t)raw.x; res[1] = (uint16_t)(raw.x >> 16); res[2] = (uint16_t)raw.y; res[3] = (uint16_t)(raw.y >> 16);
                    } else {
                        for (int e = 0; e < 4; ++e)
                            if (col + e < n) res[e] = residual[row * n + col + e];
                    }
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float value = half_to_f32<IS_BF16>(f32_to_half<IS_BF16>(acc[i][j][r4 * 4 + e]));
                    if (EPILOGUE == 1) value = -4.7750f * half_to_f32<IS_BF16>(res[e]) + 2.0315f * value;
                    if (EPILOGUE == 2) value = value + 3.4445f * half_to_f32<IS_BF16>(res[e]);
                    const uint16_t bits = f32_to_half<IS_BF16>(value);
                    o[e] = bits;
                    od[e] = col + e == row ? f32_to_half<IS_BF16>(half_to_f32<IS_BF16>(bits) + add_diag) : bits;
                }
                if (transpose_out) {
                    for (int e = 0; e < 4; ++e)
                        if (col + e < n) {
                            out[(col + e) * m + row] = o[e];
                            if (out_diag) out_diag[(col + e) * m + row] = od[e];
                        }
                } else if (full) {
                    *reinterpret_cast<uint2*>(out + row * n + col) = make_uint2((uint32_t)o[0] | ((uint32_t)o[1] << 16), (uint32_t)o[2] | ((uint32_t)o[3] << 16));
                    if (out_diag) *reinterpret_cast<uint2*>(out_diag + row * n + col) = make_uint2((uint32_t)od[0] | ((uint32_t)od[1] << 16), (uint32_t)od[2] | ((uint32_t)od[3] << 16));
                } else {
                    for (int e = 0; e < 4; ++e)
                        if (col + e < n) {
                            out[row * n + col + e] = o[e];
                            if (out_diag) out_diag[row * n + col + e] = od[e];
                        }
                }
            }
        }
    }
}

// ------------------------------------------------------------------ normalisation
// Stage 1: partial sums of squares of dtype(in) per (batch, slice) -> workspace[batch][PARTS].
constexpr int PARTS = 256;

template <typename TIn, bool IS_BF16>
__global__ __launch_bounds__(256) void ns_sumsq_kernel(const TIn* __restrict__ in, float* __restrict__ workspace, int64_t count) {
    const int64_t bz = blockIdx.y;
    const TIn* src = in + bz * count;
    const int64_t per = (count + PARTS - 1) / PARTS;
    const int64_t begin = (int64_t)blockIdx.x * per;
    const int64_t end = begin + per < count ? begin + per : count;
    float sum = 0.0f;
    for (int64_t i = begin + threadIdx.x; i < end; i += 256) {
        const float v = half_to_f32<IS_BF16>(f32_to_half<IS_BF16>(to_f32(src[i])));
        sum += v * v;
    }
    __shared__ float partial[4];
    sum = wave_sum(sum);
    if (threadIdx.x % WAVE == 0) partial[threadIdx.x / WAVE] = sum;
    __syncthreads();
    if (threadIdx.x == 0) workspace[bz * PARTS + blockIdx.x] = (partial[0] + partial[1]) + (partial[2] + partial[3]);
}

// Stage 2: out = dtype(in) / (dtype(norm) + 1e-7), optionally transposed (32 x 32 tile through LDS).
template <typename TIn, bool IS_BF16, bool TRANSPOSE>
__global__ __launch_bounds__(256) void ns_scale_kernel(const TIn* __restrict__ in, uint16_t* __restrict__ out,
                                                        const float* __restrict__ workspace, int64_t rows, int64_t cols) {
    __shared__ float tile[32][33];
    __shared__ float denom_s;
    const int64_t bz = blockIdx.z;
    const TIn* src = in + bz * rows * cols;
    uint16_t* dst = out + bz * rows * cols;
    if (threadIdx.x < WAVE) {
        float sum = 0.0f;
        for (int i = threadIdx.x; i < PARTS; i += WAVE) sum += workspace[bz * PARTS + i];
        sum = wave_sum(sum);
        if (threadIdx.x == 0) {
            const float norm = half_to_f32<IS_BF16>(f32_to_half<IS_BF16>(sqrtf(sum)));
            denom_s = half_to_f32<IS_BF16>(f32_to_half<IS_BF16>(norm + 1e-7f));
        }
    }
    __syncthreads();
    const float denom = denom_s;
    const int64_t r0 = (int64_t)blockIdx.y * 32, c0 = (int64_t)blockIdx.x * 32;
    const int tx = threadIdx.x % 32, ty = threadIdx.x / 32;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int64_t r = r0 + ty + i * 8, c = c0 + tx;
        if (r < rows && c < cols) {
            const float v = half_to_f32<IS_BF16>(f32_to_half<IS_BF16>(to_f32(src[r * cols + c])));
            const uint16_t bits = f32_to_half<IS_BF16>(v / denom);
            if constexpr (TRANSPOSE) tile[ty + i * 8][tx] = __uint_as_float(bits);
            else dst[r * cols + c] = bits;
        }
    }
    if constexpr (TRANSPOSE) {
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int64_t c = c0 + ty + i * 8, r = r0 + tx;
            if (r < rows && c < cols) dst[c * rows + r] = (uint16_t)__float_as_uint(tile[tx][ty + i * 8]);
        }
    }
}

// ------------------------------------------------------------------ normalisation, 16-byte accesses
// The same values as the kernels above for 16-bit inputs whose extents allow 8-element accesses. The division by
// the one denominator of a matrix takes the shared-divisor route (exact quotient from a reciprocal and two FMAs)
// whenever the denominator allows it.
__device__ __forceinline__ float ns_denominator(const float* __restrict__ workspace, int64_t bz, bool is_bf16, float* shared) {
    if (threadIdx.x < WAVE) {
        float sum = 0.0f;
        for (int i = threadIdx.x; i < PARTS; i += WAVE) sum += workspace[bz * PARTS + i];
        sum = wave_sum(sum);
        if (threadIdx.x == 0) {
            if (is_bf16) {
                const float norm = half_to_f32<true>(f32_to_half<true>(sqrtf(sum)));
                *shared = half_to_f32<true>(f32_to_half<true>(norm + 1e-7f));
            } else {
                const float norm = half_to_f32<false>(f32_to_half<false>(sqrtf(sum)));
                *shared = half_to_f32<false>(f32_to_half<false>(norm + 1e-7f));
            }
        }
    }
    __syncthreads();
    return *shared;
}

template <typename TIn, bool IS_BF16> __device__ __forceinline__ float ns_working(uint32_t raw16) {
    // a 16-bit input value converted to the working dtype and widened
    float v;
    if constexpr (sizeof(TIn) == 2 && std::is_same<TIn, bf16_t>::value) v = __uint_as_float(raw16 << 16);
    else { const uint16_t b = (uint16_t)raw16; v = (float)__builtin_bit_cast(_Float16, b); }
    return half_to_f32<IS_BF16>(f32_to_half<IS_BF16>(v));
}

template <typename TIn, bool IS_BF16>
__global__ __launch_bounds__(256) void ns_sumsq16_kernel(const TIn* __restrict__ in, float* __restrict__ workspace, int64_t count) {
    const int64_t bz = blockIdx.y;
    const uint4* src = reinterpret_cast<const uint4*>(in + bz * count);
    const int64_t octets = count / 8;
    const int64_t per = (octets + PARTS - 1) / PARTS;
    const int64_t begin = (int64_t)blockIdx.x * per;
    const int64_t end = begin + per < octets ? begin + per : octets;
    float sum = 0.0f;
    for (int64_t i = begin + threadIdx.x; i < end; i += 256) {
        const uint4 raw = src[i];
        const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float v = ns_working<TIn, IS_BF16>(e % 2 ? w[e / 2] >> 16 : w[e / 2] & 0xffffu);
            sum += v * v;
        }
    }
    __shared__ float partial[4];
    sum = wave_sum(sum);
    if (threadIdx.x % WAVE == 0) partial[threadIdx.x / WAVE] = sum;
    __syncthreads();
    if (threadIdx.x == 0) workspace[bz * PARTS + blockIdx.x] = (partial[0] + partial[1]) + (partial[2] + partial[3]);
}

template <bool IS_BF16>
__device__ __forceinline__ uint32_t ns_scaled(float v, float denom, const SharedDivisor& d) {
    return f32_to_half<IS_BF16>(d.fast ? d.quotient(v) : v / denom);
}

template <typename TIn, bool IS_BF16>
__global__ __launch_bounds__(256) void ns_scale16_kernel(const TIn* __restrict__ in, uint16_t* __restrict__ out,
                                                          const float* __restrict__ workspace, int64_t count) {
    __shared__ float denom_s;
    const int64_t bz = blockIdx.y;
    const float denom = ns_denominator(workspace, bz, IS_BF16, &denom_s);
    const SharedDivisor divisor(denom, 0.0f);
    const uint4* src = reinterpret_cast<const uint4*>(in + bz * count);
    uint4* dst = reinterpret_cast<uint4*>(out + bz * count);
    const int64_t octets = count / 8;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < octets; i += (int64_t)gridDim.x * 256) {
        const uint4 raw = src[i];
        const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
        uint32_t o[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float lo = ns_working<TIn, IS_BF16>(w[e] & 0xffffu), hi = ns_working<TIn, IS_BF16>(w[e] >> 16);
            // a non-finite value keeps the plain division (the quotient route assumes finite operands)
            const bool plain = !(fabsf(lo) < INFINITY) || !(fabsf(hi) < INFINITY);
            const SharedDivisor use = plain ? SharedDivisor(denom, __uint_as_float(0x7fc00000u)) : divisor;
            o[e] = ns_scaled<IS_BF16>(lo, denom, use) | (ns_scaled<IS_BF16>(hi, denom, use) << 16);
        }
        dst[i] = make_uint4(o[0], o[1], o[2], o[3]);
    }
}

// FP32 inputs (a gradient handed over as it is) in 16-byte accesses: four loads in flight per thread for the sum of
// squares, eight values per thread and step for the scaling.
template <bool IS_BF16>
__global__ __launch_bounds__(256) void ns_sumsq32_kernel(const float* __restrict__ in, float* __restrict__ workspace, int64_t count) {
    const int64_t bz = blockIdx.y;
    const float4* src = reinterpret_cast<const float4*>(in + bz * count);
    const int64_t quads = count / 4;
    const int64_t per = (quads + PARTS - 1) / PARTS;
    const int64_t begin = (int64_t)blockIdx.x * per;
    const int64_t end = begin + per < quads ? begin + per : quads;
    float part[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    auto add = [](float& sum, const float4& q) {
        const float v[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float w = half_to_f32<IS_BF16>(f32_to_half<IS_BF16>(v[e]));
            sum += w * w;
        }
    };
    int64_t i = begin + threadIdx.x;
    for (; i + 768 < end; i += 1024) {
        const float4 q0 = src[i], q1 = src[i + 256], q2 = src[i + 512], q3 = src[i + 768];
        add(part[0], q0); add(part[1], q1); add(part[2], q2); add(part[3], q3);
    }
    for (; i < end; i += 256) add(part[0], src[i]);
    float sum = (part[0] + part[1]) + (part[2] + part[3]);
    __shared__ float partial[4];
    sum = wave_sum(sum);
    if (threadIdx.x % WAVE == 0) partial[threadIdx.x / WAVE] = sum;
    __syncthreads();
    if (threadIdx.x == 0) workspace[bz * PARTS + blockIdx.x] = (partial[0] + partial[1]) + (partial[2] + partial[3]);
}

template <bool IS_BF16>
__global__ __launch_bounds__(256) void ns_scale32_kernel(const float* __restrict__ in, uint16_t* __restrict__ out,
                                                          const float* __restrict__ workspace, int64_t count) {
    __shared__ float denom_s;
    const int64_t bz = blockIdx.y;
    const float denom = ns_denominator(workspace, bz, IS_BF16, &denom_s);
    const SharedDivisor divisor(denom, 0.0f);
    const float4* src = reinterpret_cast<const float4*>(in + bz * count);
    uint4* dst = reinterpret_cast<uint4*>(out + bz * count);
    const int64_t octets = count / 8;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < octets; i += (int64_t)gridDim.x * 256) {
        const float4 q0 = src[2 * i], q1 = src[2 * i + 1];
        const float v[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
        uint32_t o[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float lo = half_to_f32<IS_BF16>(f32_to_half<IS_BF16>(v[2 * e])), hi = half_to_f32<IS_BF16>(f32_to_half<IS_BF16>(v[2 * e + 1]));
            const bool plain = !(fabsf(lo) < INFINITY) || !(fabsf(hi) < INFINITY);
            const SharedDivisor use = plain ? SharedDivisor(denom, __uint_as_float(0x7fc00000u)) : divisor;
            o[e] = ns_scaled<IS_BF16>(lo, denom, use) | (ns_scaled<IS_BF16>(hi, denom, use) << 16);
        }
        dst[i] = make_uint4(o[0], o[1], o[2], o[3]);
    }
}

// Transposed: a wavefront parks 32 rows x 64 columns of raw 16-bit values in LDS and reads them back with
// ds_read_b64_tr_b16, so each lane ends up with the 32 rows of one column = 64 contiguous bytes of the output.
template <typename TIn, bool IS_BF16>
__global__ __launch_bounds__(256) void ns_scale16_transposed_kernel(const TIn* __restrict__ in, uint16_t* __restrict__ out,
                                                                     const float* __restrict__ workspace, int64_t rows,
                                                                     int64_t cols) {
    constexpr int LD = 64 + 32;
    typedef short s16x4 __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
    __shared__ __attribute__((aligned(16))) uint16_t park[4][32 * LD];
    __shared__ float denom_s;
    const int64_t bz = blockIdx.z;
    const float denom = ns_denominator(workspace, bz, IS_BF16, &denom_s);
    const SharedDivisor divisor(denom, 0.0f);
    const TIn* src = in + bz * rows * cols;
    uint16_t* dst = out + bz * rows * cols;
    const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
    const int64_t r0 = (int64_t)blockIdx.y * 128 + wave * 32, c0 = (int64_t)blockIdx.x * 64;
    if (r0 >= rows) return;
    uint16_t* mine = park[wave];
    const int lr = lane / 8, ch = lane % 8;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int64_t row = r0 + lr + 8 * i, col8 = c0 + ch * 8;
        uint4 raw = make_uint4(0, 0, 0, 0);
        if (row < rows && col8 < cols) raw = *reinterpret_cast<const uint4*>(src + row * cols + col8);
        *reinterpret_cast<uint4*>(&mine[(lr + 8 * i) * LD + ch * 8]) = raw;
    }
    const int64_t col = c0 + lane;
    const int strip = (lane / 16) * 16, sub = lane & 15;
    const uint16_t* at = &mine[(sub >> 2) * LD + strip + 4 * (sub & 3)];
    uint32_t o[16];
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        const s16x4 four = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(at + 4 * t * LD));
        uint32_t h[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float v = ns_working<TIn, IS_BF16>((uint16_t)four[e]);
            const bool plain = !(fabsf(v) < INFINITY);
            h[e] = f32_to_half<IS_BF16>(divisor.fast && !plain ? divisor.quotient(v) : v / denom);
        }
        o[2 * t] = h[0] | (h[1] << 16);
        o[2 * t + 1] = h[2] | (h[3] << 16);
    }
    if (col < cols) {
        uint16_t* row_out = dst + col * rows + r0;
        if (r0 + 32 <= rows && (reinterpret_cast<uintptr_t>(row_out) & 15) == 0) {
#pragma unroll
            for (int k = 0; k < 4; ++k) reinterpret_cast<uint4*>(row_out)[k] = make_uint4(o[4 * k], o[4 * k + 1], o[4 * k + 2], o[4 * k + 3]);
        } else {
            for (int e = 0; e < 32 && r0 + e < rows; ++e) row_out[e] = (uint16_t)(o[e / 2] >> (16 * (e % 2)));
        }
    }
}

template <bool IS_BF16, bool TRANSPOSE_B, bool VEC>
static int launch_ns(const void* a, const void* b, const void* residual, void* out, void* out_diag, int epilogue, dim3 grid,
                     int64_t m, int64_t n, int64_t k, float add_diag, int transpose_out, hipStream_t stream) {
    const uint16_t* ap = static_cast<const uint16_t*>(a);
    const uint16_t* bp = static_cast<const uint16_t*>(b);
    const uint16_t* rp = static_cast<const uint16_t*>(residual);
    uint16_t* op = static_cast<uint16_t*>(out);
    uint16_t* dp = static_cast<uint16_t*>(out_diag);
    if (epilogue == 0) VIOLA_LAUNCH((ns_gemm_kernel<IS_BF16, TRANSPOSE_B, 0, VEC>), grid, dim3(256), 0, stream, ap, bp, rp, op, dp, m, n, k, add_diag, transpose_out);
    else if (epilogue == 1) VIOLA_LAUNCH((ns_gemm_kernel<IS_BF16, TRANSPOSE_B, 1, VEC>), grid, dim3(256), 0, stream, ap, bp, rp, op, dp, m, n, k, add_diag, transpose_out);
    else VIOLA_LAUNCH((ns_gemm_kernel<IS_BF16, TRANSPOSE_B, 2, VEC>), grid, dim3(256), 0, stream, ap, bp, rp, op, dp, m, n, k, add_diag, transpose_out);
    return viola_launch_status();
}

template <typename TIn, bool IS_BF16>
static int launch_prepare(const void* in, void* out, int64_t batch, int64_t rows, int64_t cols, float* workspace,
                          hipStream_t stream) {
    const TIn* src = static_cast<const TIn*>(in);
    if constexpr (sizeof(TIn) == 2) {
        const bool aligned = reinterpret_cast<uintptr_t>(in) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0;
        if (aligned && cols % 8 == 0 && (rows * cols) % 8 == 0 && (rows + 127) / 128 <= 65535) {
            VIOLA_LAUNCH((ns_sumsq16_kernel<TIn, IS_BF16>), dim3(PARTS, (unsigned)batch), dim3(256), 0, stream, src, workspace, rows * cols);
            if (rows > cols) {
                const dim3 tgrid((unsigned)((cols + 63) / 64), (unsigned)((rows + 127) / 128), (unsigned)batch);
                VIOLA_LAUNCH((ns_scale16_transposed_kernel<TIn, IS_BF16>), tgrid, dim3(256), 0, stream, src, static_cast<uint16_t*>(out), workspace, rows, cols);
            } else {
                const int64_t octets = rows * cols / 8;
                const unsigned bx = (unsigned)(octets / 256 / 4 < 1 ? 1 : octets / 256 / 4 > 4096 ? 4096 : octets / 256 / 4);
                VIOLA_LAUNCH((ns_scale16_kernel<TIn, IS_BF16>), dim3(bx, (unsigned)batch), dim3(256), 0, stream, src, static_cast<uint16_t*>(out), workspace, rows * cols);
            }
            return viola_launch_status();
        }
    }
    if constexpr (sizeof(TIn) == 4) {
        const bool aligned = reinterpret_cast<uintptr_t>(in) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0;
        if (aligned && (rows * cols) % 8 == 0 && rows <= cols) {
            VIOLA_LAUNCH((ns_sumsq32_kernel<IS_BF16>), dim3(PARTS, (unsigned)batch), dim3(256), 0, stream, src, workspace, rows * cols);
            const int64_t octets = rows * cols / 8;
            const unsigned bx = (unsigned)(octets / 256 / 4 < 1 ? 1 : octets / 256 / 4 > 4096 ? 4096 : octets / 256 / 4);
            VIOLA_LAUNCH((ns_scale32_kernel<IS_BF16>), dim3(bx, (unsigned)batch), dim3(256), 0, stream, src, static_cast<uint16_t*>(out), workspace, rows * cols);
            return viola_launch_status();
        }
    }
    VIOLA_LAUNCH((ns_sumsq_kernel<TIn, IS_BF16>), dim3(PARTS, (unsigned)batch), dim3(256), 0, stream, src, workspace, rows * cols);
    const dim3 grid((unsigned)((cols + 31) / 32), (unsigned)((rows + 31) / 32), (unsigned)batch);
    if (rows > cols) VIOLA_LAUNCH((ns_scale_kernel<TIn, IS_BF16, true>), grid, dim3(256), 0, stream, src, static_cast<uint16_t*>(out), workspace, rows, cols);
    else VIOLA_LAUNCH((ns_scale_kernel<TIn, IS_BF16, false>), grid, dim3(256), 0, stream, src, static_cast<uint16_t*>(out), workspace, rows, cols);
    return viola_launch_status();
}

// Scratch of viola_ns_prepare_static: the partial sums of squares that viola_ns_prepare keeps in its caller's
// workspace. One copy per GPU, held until the process ends; its address on a device is looked up once, with that
// device current, and only that address (never the array's name, which on the host is a stand-in) reaches kernels.
constexpr int64_t NS_STATIC_BATCH = 1024;
static __device__ __align__(256) float ns_static_scratch[NS_STATIC_BATCH * PARTS];
constexpr int NS_STATIC_DEVICES = 64;
static std::atomic<float*> ns_static_address[NS_STATIC_DEVICES];
static std::mutex ns_static_mutex;

static int ns_static_workspace(float** workspace) {
    int device = -1;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) return (int)e;
    if (device < 0 || device >= NS_STATIC_DEVICES) return VIOLA_EUNSUPPORTED;
    float* address = ns_static_address[device].load(std::memory_order_acquire);
    if (address == nullptr) {
        std::lock_guard<std::mutex> guard(ns_static_mutex);
        address = ns_static_address[device].load(std::memory_order_relaxed);
        if (address == nullptr) {
            void* found = nullptr;
            e = hipGetSymbolAddress(&found, HIP_SYMBOL(ns_static_scratch));
            if (e != hipSuccess) return (int)e;
            if (found == nullptr) return (int)hipErrorInvalidSymbol;
            address = static_cast<float*>(found);
            ns_static_address[device].store(address, std::memory_order_release);
        }
    }
    *workspace = address;
    return 0;
}

}  // namespace viola

using namespace viola;

// A product of a matrix with its own transpose is multiplied on and above the diagonal only and mirrored. A transposed
// result keeps the full kernel: there the [n, m] store is the only placement, and the mirrored tiles have none of their own.
static bool ns_is_mirrored(const void* a, const void* bmat, int transpose_b, int64_t m, int64_t n, int transpose_out) {
    return transpose_b && a == bmat && m == n && !transpose_out;
}

extern "C" int viola_ns_plan(int64_t batch, int64_t m, int64_t n, int64_t k, int transpose_b, int same_operand,
                             int transpose_out, int* plan) {
    VIOLA_CHECK_ARG(plan && batch >= 0 && m >= 0 && n >= 0 && k >= 0);
    const void* const one = reinterpret_cast<const void*>(uintptr_t(4096));          // stand-ins: aligned, equal or not
    const void* const two = reinterpret_cast<const void*>(uintptr_t(8192));
    NsArgs probe{static_cast<const uint16_t*>(one), static_cast<const uint16_t*>(same_operand ? one : two), nullptr, nullptr, nullptr,
                 batch, m, n, k, 0.0f, transpose_out, ns_is_mirrored(one, same_operand ? one : two, transpose_b, m, n, transpose_out), 0, 0, 0};
    static const int shapes[6][2] = {{NBM, NBN}, {64, 64}, {128, 64}, {128, 128}, {192, 192}, {384, 192}};
    const NsTile tile = batch > 0 && m > 0 && n > 0 && ns_fast_takes(probe) ? ns_choose_tile(batch, m, n, probe.symmetric != 0) : NS_TILE_GENERIC;
    plan[0] = shapes[tile][0];
    plan[1] = shapes[tile][1];
    plan[2] = tile != NS_TILE_GENERIC && probe.symmetric;
    plan[3] = (int)tile;
    return 0;
}

extern "C" int viola_ns_gemm(const void* a, const void* bmat, const void* residual, void* out, int dtype, int transpose_b,
                             int epilogue, int64_t batch, int64_t m, int64_t n, int64_t k, float add_diag, void* out_diag,
                             int transpose_out, viola_stream_t stream_) {
    hipStream_t stream = viola_enter(stream_);
    VIOLA_CHECK_ARG((dtype == VIOLA_BF16 || dtype == VIOLA_F16) && epilogue >= 0 && epilogue <= 2);
    VIOLA_CHECK_ARG(batch >= 0 && m >= 0 && n >= 0 && k >= 0);
    if (batch == 0 || m == 0 || n == 0) return 0;
    VIOLA_CHECK_ARG(out && (k == 0 || (a && bmat)) && (epilogue == 0 || residual));
    if (k > 0) {
        NsArgs fast{static_cast<const uint16_t*>(a), static_cast<const uint16_t*>(bmat), static_cast<const uint16_t*>(residual),
                    static_cast<uint16_t*>(out), static_cast<uint16_t*>(out_diag), batch, m, n, k, add_diag, transpose_out,
                    ns_is_mirrored(a, bmat, transpose_b, m, n, transpose_out), 0, 0, 0};
        if (launch_ns_gemm_fast(fast, dtype == VIOLA_BF16, !transpose_b, epilogue, stream)) return viola_launch_status();
    }
    const int64_t gx = (n + NBN - 1) / NBN, gy = (m + NBM - 1) / NBM;
    VIOLA_CHECK_ARG(gy <= 65535 && batch <= 65535);
    const dim3 grid((unsigned)gx, (unsigned)gy, (unsigned)batch);
    auto al = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
    const bool vec = k % 8 == 0 && n % 8 == 0 && al(a) && al(bmat) && al(out) && (!residual || al(residual)) && (!out_diag || al(out_diag));
#define VIOLA_NS(BF, TB, V) return launch_ns<BF, TB, V>(a, bmat, residual, out, out_diag, epilogue, grid, m, n, k, add_diag, transpose_out, stream)
    if (dtype == VIOLA_BF16) {
        if (transpose_b) { if (vec) VIOLA_NS(true, true, true); VIOLA_NS(true, true, false); }
        if (vec) VIOLA_NS(true, false, true);
        VIOLA_NS(true, false, false);
    }
    if (transpose_b) { if (vec) VIOLA_NS(false, true, true); VIOLA_NS(false, true, false); }
    if (vec) VIOLA_NS(false, false, true);
    VIOLA_NS(false, false, false);
#undef VIOLA_NS
}

extern "C" int viola_ns_prepare(const void* in, int in_dtype, void* out, int dtype, int64_t batch, int64_t rows,
                                int64_t cols, float* workspace, viola_stream_t stream_) {
    hipStream_t stream = viola_enter(stream_);
    VIOLA_CHECK_ARG((dtype == VIOLA_BF16 || dtype == VIOLA_F16) && viola_is_float(in_dtype));
    VIOLA_CHECK_ARG(batch >= 0 && rows >= 0 && cols >= 0 && batch <= 65535 && (rows + 31) / 32 <= 65535);
    if (batch == 0 || rows == 0 || cols == 0) return 0;
    VIOLA_CHECK_ARG(in && out && workspace);
#define VIOLA_PREP(TI, BF) return launch_prepare<TI, BF>(in, out, batch, rows, cols, workspace, stream)
    if (dtype == VIOLA_BF16) {
        if (in_dtype == VIOLA_F32) VIOLA_PREP(float, true);
        if (in_dtype == VIOLA_BF16) VIOLA_PREP(bf16_t, true);
        VIOLA_PREP(f16_t, true);
    }
    if (in_dtype == VIOLA_F32) VIOLA_PREP(float, false);
    if (in_dtype == VIOLA_BF16) VIOLA_PREP(bf16_t, false);
    VIOLA_PREP(f16_t, false);
#undef VIOLA_PREP
}

extern "C" int viola_ns_prepare_static(const void* in, int in_dtype, void* out, int dtype, int64_t batch, int64_t rows,
                                       int64_t cols, viola_stream_t stream) {
    VIOLA_CHECK_ARG(batch >= 0);
    if (batch > NS_STATIC_BATCH) return VIOLA_ETOOLARGE;             // beyond the built-in scratch: use viola_ns_prepare
    float* workspace = nullptr;
    const int status = ns_static_workspace(&workspace);              // also for batch == 0: a set-up call
    if (status != 0) return status;
    return viola_ns_prepare(in, in_dtype, out, dtype, batch, rows, cols, workspace, stream);
}
