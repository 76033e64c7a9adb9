// FP8 gradient wire codec, elementwise gated activations, and device self checks for gfx950.
// Built with -ffp-contract=off.
#include "common.hpp"

namespace viola {

// ------------------------------------------------------------------ wire codec
// LANES lanes share one tile of `tile` fp32 values; each lane walks it with stride LANES.
template <typename TQ, int LANES>
__global__ __launch_bounds__(256) void comm_pack_kernel(const float* __restrict__ x, int64_t n, uint8_t* __restrict__ packet,
                                                         int64_t rows, int64_t groups, int tile, int64_t stride) {
    const int64_t unit = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) / LANES;     // (row, group) pair
    if (unit >= rows * groups) return;                                                   // LANES-aligned sets leave together
    const int sub = threadIdx.x % LANES;
    const int64_t row = unit / groups, group = unit % groups;
    const int64_t base = row * groups * tile + group * tile;
    float amax = 0.0f;
    for (int i = sub; i < tile; i += LANES) {
        const float v = base + i < n ? x[base + i] : 0.0f;
        amax = fmaxf(amax, v != v ? __uint_as_float(0x7f800000u) : fabsf(v));
    }
    amax = group_max<LANES>(amax);
    const float s = scale_of(amax, fp8_traits<TQ>::max);
    uint8_t* codes = packet + row * stride + group * tile;
    for (int i = sub; i < tile; i += LANES) {
        const float v = base + i < n ? x[base + i] : 0.0f;
        codes[i] = from_f32<TQ>(v / s).bits;
    }
    if (sub == 0) reinterpret_cast<float*>(packet + row * stride + groups * tile)[group] = s;
}

// tile == 256, x 16-byte aligned: one wavefront per tile, one float4 per lane.
template <typename TQ>
__device__ __forceinline__ void comm_pack256_tile(const float* __restrict__ x, int64_t n, uint8_t* __restrict__ packet, int64_t groups,
                                                  int64_t stride, int64_t unit, int lane) {
    const int64_t row = unit / groups, group = unit % groups;
    const int64_t base = (row * groups + group) * 256 + lane * 4;
    float v[4] = {0, 0, 0, 0};
    if (base + 3 < n) {
        const float4 raw = *reinterpret_cast<const float4*>(x + base);
        v[0] = raw.x; v[1] = raw.y; v[2] = raw.z; v[3] = raw.w;
    } else {
        for (int i = 0; i < 4; ++i)
            if (base + i < n) v[i] = x[base + i];
    }
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i) amax = fmaxf(amax, v[i] != v[i] ? __uint_as_float(0x7f800000u) : fabsf(v[i]));
    amax = wave_max(amax);
    const float s = scale_of(amax, fp8_traits<TQ>::max);
    // a tile with a NaN or an Inf has an infinite scale, which the shared divisor declines
    const SharedDivisor divisor(s, 0.0f);
    uint32_t w = 0;
    if (divisor.fast) {
        w = hw_encode4<TQ>(divisor.quotient(v[0]), divisor.quotient(v[1]), divisor.quotient(v[2]), divisor.quotient(v[3]));
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) w |= (uint32_t)from_f32<TQ>(v[i] / s).bits << (8 * i);
    }
    *reinterpret_cast<uint32_t*>(packet + row * stride + group * 256 + lane * 4) = w;
    if (lane == 0) reinterpret_cast<float*>(packet + row * stride + groups * 256)[group] = s;
}

template <typename TQ>
__global__ __launch_bounds__(256) void comm_pack256_kernel(const float* __restrict__ x, int64_t n, uint8_t* __restrict__ packet,
                                                            int64_t rows, int64_t groups, int64_t stride) {
    const int64_t unit = (int64_t)blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE;
    if (unit >= rows * groups) return;
    comm_pack256_tile<TQ>(x, n, packet, groups, stride, unit, threadIdx.x % WAVE);
}

// max over the 16 lanes of a DPP row: quad permutes, then the row's two mirrors (lane i with 7 - i, then with 15 - i), all
// inside the vector ALU (a shuffle goes through the LDS crossbar and its wait)
__device__ __forceinline__ float row16_max(float v) {
    v = fmaxf(v, quad_xor<1>(v));
    v = fmaxf(v, quad_xor<2>(v));
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x141, 0xf, 0xf, true)));   // row_half_mirror
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x140, 0xf, 0xf, true)));   // row_mirror
    return v;
}

// tile == 256 for launches with many tiles: sixteen lanes per tile (lane j takes floats 4 j + 64 i, i = 0 .. 3, so every
// load instruction of a 16-lane row covers 256 contiguous bytes and a lane has four loads in flight), a wavefront four
// tiles at a time, the blocks walking the tiles with the grid's stride. Same bytes as comm_pack256_tile.
template <typename TQ>
__device__ __forceinline__ void comm_pack256_rows(const float* __restrict__ x, int64_t n, uint8_t* __restrict__ packet, int64_t rows,
                                                  int64_t groups, int64_t stride, int64_t first_block, int64_t block_step) {
    const int sub = threadIdx.x % 16;
    const int64_t units = rows * groups;
    for (int64_t unit = first_block * 16 + threadIdx.x / 16; unit < units; unit += block_step * 16) {
        const int64_t row = unit / groups, group = unit - row * groups;
        const int64_t base = unit * 256 + sub * 4;
        float v[4][4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int64_t at = base + 64 * i;
            if (at + 3 < n) {
                const float4 raw = *reinterpret_cast<const float4*>(x + at);
                v[i][0] = raw.x; v[i][1] = raw.y; v[i][2] = raw.z; v[i][3] = raw.w;
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) v[i][e] = at + e < n ? x[at + e] : 0.0f;
            }
        }
        float amax = 0.0f;
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int e = 0; e < 4; ++e) amax = fmaxf(amax, v[i][e] != v[i][e] ? __uint_as_float(0x7f800000u) : fabsf(v[i][e]));
        amax = row16_max(amax);
        const float s = scale_of(amax, fp8_traits<TQ>::max);
        const SharedDivisor divisor(s, 0.0f);                    // declines an infinite scale (a tile with a NaN or an Inf)
        uint8_t* codes = packet + row * stride + group * 256 + sub * 4;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint32_t w = 0;
            if (divisor.fast) {
                w = hw_encode4<TQ>(divisor.quotient(v[i][0]), divisor.quotient(v[i][1]), divisor.quotient(v[i][2]), divisor.quotient(v[i][3]));
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) w |= (uint32_t)from_f32<TQ>(v[i][e] / s).bits << (8 * e);
            }
            *reinterpret_cast<uint32_t*>(codes + 64 * i) = w;
        }
        if (sub == 0) reinterpret_cast<float*>(packet + row * stride + groups * 256)[group] = s;
    }
}

template <typename TQ>
__global__ __launch_bounds__(256) void comm_pack256_rows_kernel(const float* __restrict__ x, int64_t n, uint8_t* __restrict__ packet,
                                                                 int64_t rows, int64_t groups, int64_t stride) {
    comm_pack256_rows<TQ>(x, n, packet, rows, groups, stride, blockIdx.x, gridDim.x);
}

// Many buckets, one launch: row blockIdx.y of the table names the bucket {x, n, packet, rows, groups, -, -, -}.
constexpr int COMM_ROW = 8;                                                   // int64 words per table row
template <typename TQ>
__global__ __launch_bounds__(256) void comm_pack256_table_kernel(const int64_t* __restrict__ table) {
    const int64_t* bucket = table + (int64_t)blockIdx.y * COMM_ROW;
    const int64_t n = bucket[1], rows = bucket[3], groups = bucket[4];
    const int64_t stride = (groups * (256 + 4) + 15) / 16 * 16;
    comm_pack256_rows<TQ>(reinterpret_cast<const float*>(bucket[0]), n, reinterpret_cast<uint8_t*>(bucket[2]), rows, groups, stride,
                          blockIdx.x, gridDim.x);
}

template <typename TQ>
__global__ __launch_bounds__(256) void comm_unpack_kernel(const uint8_t* __restrict__ packet, float* __restrict__ out, int64_t n,
                                                           int64_t rows, int64_t groups, int tile, int64_t stride, int reduce) {
    const int64_t width = groups * tile;
    const int64_t total = reduce ? width : rows * width;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * blockDim.x) {
        const int64_t row = idx / width, col = idx % width;
        if (reduce) {
            if (col >= n) continue;
            float result = 0.0f;
            for (int64_t rank = 0; rank < rows; ++rank) {
                const float s = reinterpret_cast<const float*>(packet + rank * stride + width)[col / tile];
                result += to_f32(TQ{packet[rank * stride + col]}) * s;
            }
            out[col] = result;
        } else {
            if (idx >= n) continue;
            const float s = reinterpret_cast<const float*>(packet + row * stride + width)[col / tile];
            out[idx] = to_f32(TQ{packet[row * stride + col]}) * s;
        }
    }
}

template <typename TQ> __device__ __forceinline__ void decode4(uint32_t word, float (&v)[4]);
template <> __device__ __forceinline__ void decode4<e4m3_t>(uint32_t word, float (&v)[4]) {
    v[0] = __builtin_amdgcn_cvt_f32_fp8((int)word, 0); v[1] = __builtin_amdgcn_cvt_f32_fp8((int)word, 1);
    v[2] = __builtin_amdgcn_cvt_f32_fp8((int)word, 2); v[3] = __builtin_amdgcn_cvt_f32_fp8((int)word, 3);
}
template <> __device__ __forceinline__ void decode4<e5m2_t>(uint32_t word, float (&v)[4]) {
    v[0] = __builtin_amdgcn_cvt_f32_bf8((int)word, 0); v[1] = __builtin_amdgcn_cvt_f32_bf8((int)word, 1);
    v[2] = __builtin_amdgcn_cvt_f32_bf8((int)word, 2); v[3] = __builtin_amdgcn_cvt_f32_bf8((int)word, 3);
}

// out 16-byte aligned: four consecutive elements per thread (one code word, one scale, one 16-byte store). The
// hardware decoders equal the table decode on all 256 codes (checked by the device self test below).
template <typename TQ, bool REDUCE>
__device__ __forceinline__ void comm_unpack_quads(const uint8_t* __restrict__ packet, float* __restrict__ out, int64_t n, int64_t rows,
                                                  int64_t width, int tile_shift, int64_t stride, int64_t first_block, int64_t block_step) {
    const int64_t quads_per_row = width / 4;
    const int64_t total = (REDUCE ? 1 : rows) * quads_per_row;
    // a block takes four runs of 256 quads per step: the code words and scales of all four are asked for before the
    // first is used, so a thread has eight loads in flight; every load and store instruction stays contiguous over the block
    constexpr int RUNS = 4;
    for (int64_t chunk = first_block * RUNS * 256; chunk < total; chunk += block_step * RUNS * 256) {
        uint32_t word[RUNS];
        float s[RUNS];
        int64_t index[RUNS];
#pragma unroll
        for (int u = 0; u < RUNS; ++u) {
            const int64_t quad = chunk + u * 256 + threadIdx.x;
            const int64_t row = (REDUCE || rows == 1) ? 0 : quad / quads_per_row;
            const int64_t col = (quad - row * quads_per_row) * 4;
            index[u] = quad < total ? row * width + col : n;
            word[u] = 0;
            s[u] = 0.0f;
            if (index[u] < n) {
                if constexpr (REDUCE) {
                    index[u] = col;                                      // the ranks' rows are summed below
                } else {
                    const uint8_t* base = packet + row * stride;
                    word[u] = *reinterpret_cast<const uint32_t*>(base + col);
                    s[u] = reinterpret_cast<const float*>(base + width)[col >> tile_shift];
                }
            }
        }
#pragma unroll
        for (int u = 0; u < RUNS; ++u) {
            const int64_t idx = index[u];
            if (idx >= n) continue;
            float result[4];
            if constexpr (REDUCE) {
                result[0] = result[1] = result[2] = result[3] = 0.0f;
                for (int64_t rank = 0; rank < rows; ++rank) {
                    const uint8_t* base = packet + rank * stride;
                    const float scale = reinterpret_cast<const float*>(base + width)[idx >> tile_shift];
                    float v[4];
                    decode4<TQ>(*reinterpret_cast<const uint32_t*>(base + idx), v);
#pragma unroll
                    for (int i = 0; i < 4; ++i) { const float term = v[i] * scale; result[i] += term; }
                }
            } else {
                float v[4];
                decode4<TQ>(word[u], v);
#pragma unroll
                for (int i = 0; i < 4; ++i) result[i] = v[i] * s[u];
            }
            if (idx + 3 < n) {
                *reinterpret_cast<float4*>(out + idx) = make_float4(result[0], result[1], result[2], result[3]);
            } else {
                for (int i = 0; i < 4; ++i)
                    if (idx + i < n) out[idx + i] = result[i];
            }
        }
    }
}

template <typename TQ, bool REDUCE>
__global__ __launch_bounds__(256) void comm_unpack_quads_kernel(const uint8_t* __restrict__ packet, float* __restrict__ out,
                                                                 int64_t n, int64_t rows, int64_t width, int tile_shift,
                                                                 int64_t stride) {
    comm_unpack_quads<TQ, REDUCE>(packet, out, n, rows, width, tile_shift, stride, blockIdx.x, gridDim.x);
}

// Many buckets, one launch: row blockIdx.y of the table names the bucket {packet, n, out, rows, groups, -, -, -}.
template <typename TQ, bool REDUCE>
__global__ __launch_bounds__(256) void comm_unpack_quads_table_kernel(const int64_t* __restrict__ table, int tile, int tile_shift) {
    const int64_t* bucket = table + (int64_t)blockIdx.y * COMM_ROW;
    const int64_t n = bucket[1], rows = bucket[3], groups = bucket[4];
    const int64_t width = groups * tile, stride = (groups * (tile + 4) + 15) / 16 * 16;
    comm_unpack_quads<TQ, REDUCE>(reinterpret_cast<const uint8_t*>(bucket[0]), reinterpret_cast<float*>(bucket[2]), n, rows, width,
                                  tile_shift, stride, blockIdx.x, gridDim.x);
}


// ------------------------------------------------------------------ gated activations
__device__ __forceinline__ float load_half(const void* p, int64_t i, int dtype) {
    if (dtype == VIOLA_F32) return static_cast<const float*>(p)[i];
    if (dtype == VIOLA_BF16) return bf16_bits_to_f32(static_cast<const uint16_t*>(p)[i]);
    return (float)static_cast<const _Float16*>(p)[i];
}
__device__ __forceinline__ void store_half(void* p, int64_t i, int dtype, float v) {
    if (dtype == VIOLA_F32) static_cast<float*>(p)[i] = v;
    else if (dtype == VIOLA_BF16) static_cast<uint16_t*>(p)[i] = f32_to_bf16_bits(v);
    else static_cast<_Float16*>(p)[i] = (_Float16)v;
}

__global__ __launch_bounds__(256) void gated_forward_kernel(const void* __restrict__ z, void* __restrict__ out, int64_t rows,
                                                             int64_t h, int dtype, int activation) {
    const int64_t total = rows * h;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * blockDim.x) {
        const int64_t r = idx / h, c = idx % h;
        const float g = load_half(z, r * 2 * h + c, dtype), u = load_half(z, r * 2 * h + h + c, dtype);
        float a, derivative;
        // the stand-alone operator divides (viola/nn/_gated_kernels.py:29-35); the GEMM epilogues multiply by 1 / (1 + exp(-g))
        if (activation == VIOLA_SILU) a = g / (1.0f + expf(-g));
        else gate_math(activation, g, a, derivative);
        store_half(out, idx, dtype, a * u);
    }
}

__global__ __launch_bounds__(256) void gated_backward_kernel(const void* __restrict__ z, const void* __restrict__ dy,
                                                              void* __restrict__ dz, int64_t rows, int64_t h, int dtype,
                                                              int activation) {
    const int64_t total = rows * h;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * blockDim.x) {
        const int64_t r = idx / h, c = idx % h;
        const float g = load_half(z, r * 2 * h + c, dtype), u = load_half(z, r * 2 * h + h + c, dtype);
        const float d = load_half(dy, idx, dtype);
        float a, derivative;
        if (activation == VIOLA_SILU) {
            const float s = 1.0f / (1.0f + expf(-g));
            a = g * s;
            derivative = s * (1.0f + g * (1.0f - s));
        } else if (activation == VIOLA_GELU) {
            const float t = tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g));
            a = 0.5f * g * (1.0f + t);
            derivative = 0.5f * (1.0f + t) + 0.5f * g * (1.0f - t * t) * 0.7978845608028654f * (1.0f + 0.134145f * g * g);
        } else {
            a = fmaxf(g, 0.0f);
            derivative = g > 0.0f ? 1.0f : 0.0f;
        }
        store_half(dz, r * 2 * h + c, dtype, d * u * derivative);
        store_half(dz, r * 2 * h + h + c, dtype, d * a);
    }
}

// The same two maps for rows whose halves start on 16-byte boundaries: one 16-byte piece of g, u (and dy) per thread,
// element type and activation fixed at compile time. Every element goes through the expressions above.
template <typename T> struct Piece {
    static constexpr int N = 16 / (int)sizeof(T);
    static __device__ __forceinline__ void load(const T* p, float (&v)[N]) {
        const uint4 raw = *reinterpret_cast<const uint4*>(p);
        T t[N];
        __builtin_memcpy(t, &raw, 16);
#pragma unroll
        for (int i = 0; i < N; ++i) v[i] = to_f32(t[i]);
    }
    static __device__ __forceinline__ void store(T* p, const float (&v)[N]) {
        T t[N];
#pragma unroll
        for (int i = 0; i < N; ++i) t[i] = from_f32<T>(v[i]);
        uint4 raw;
        __builtin_memcpy(&raw, t, 16);
        *reinterpret_cast<uint4*>(p) = raw;
    }
};

// EPILOGUE_FORM: silu as g * (1 / (1 + exp(-g))), the gated GEMM epilogue's expression (viola/nn/_mlp_kernels.py:163-175),
// for the pass that stands in for that epilogue; otherwise the stand-alone operator's g / (1 + exp(-g)).
template <typename T, int ACT, bool EPILOGUE_FORM>
__global__ __launch_bounds__(256) void gated_forward_pieces(const T* __restrict__ z, T* __restrict__ out, int64_t pieces, int64_t per_row) {
    constexpr int N = Piece<T>::N;
    const int64_t id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (id >= pieces) return;
    const int64_t r = id / per_row, c = id % per_row * N, h = per_row * N;
    float g[N], u[N], o[N];
    Piece<T>::load(z + r * 2 * h + c, g);
    Piece<T>::load(z + r * 2 * h + h + c, u);
#pragma unroll
    for (int i = 0; i < N; ++i) {
        float a, derivative;
        if constexpr (ACT == VIOLA_SILU && !EPILOGUE_FORM) a = g[i] / (1.0f + expf(-g[i]));
        else gate_math(ACT, g[i], a, derivative);
        o[i] = a * u[i];
    }
    Piece<T>::store(out + r * h + c, o);
}

template <typename T, int ACT>
__global__ __launch_bounds__(256) void gated_backward_pieces(const T* __restrict__ z, const T* dy, int64_t dy_stride, T* dz,
                                                              int64_t pieces, int64_t per_row) {
    // dy may be the up half of dz itself (dy = dz + h, dy_stride = 2 h): a thread reads its piece before it writes there
    constexpr int N = Piece<T>::N;
    const int64_t id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (id >= pieces) return;
    const int64_t r = id / per_row, c = id % per_row * N, h = per_row * N;
    float g[N], u[N], d[N], dg[N], du[N];
    Piece<T>::load(z + r * 2 * h + c, g);
    Piece<T>::load(z + r * 2 * h + h + c, u);
    Piece<T>::load(dy + r * dy_stride + c, d);
#pragma unroll
    for (int i = 0; i < N; ++i) {
        float a, derivative;
        gate_math(ACT, g[i], a, derivative);
        dg[i] = d[i] * u[i] * derivative;
        du[i] = d[i] * a;
    }
    Piece<T>::store(dz + r * 2 * h + c, dg);
    Piece<T>::store(dz + r * 2 * h + h + c, du);
}

template <typename T>
static bool launch_gated_pieces(const void* z, const void* dy, int64_t dy_stride, void* out, int64_t rows, int64_t h, int activation,
                                bool backward, bool epilogue_form, hipStream_t stream) {
    constexpr int N = Piece<T>::N;
    const auto aligned = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
    if (h % N != 0 || !aligned(z) || !aligned(out) || (backward && (!aligned(dy) || dy_stride % N != 0))) return false;
    const int64_t per_row = h / N, pieces = rows * per_row, blocks = (pieces + 255) / 256;
    if (blocks > 0x7fffffff) return false;
    const dim3 grid((unsigned)blocks);
    const T* zp = static_cast<const T*>(z);
    const T* dp = static_cast<const T*>(dy);
    T* op = static_cast<T*>(out);
#define VIOLA_GATED(ACT)                                                                                                   \
    if (backward) VIOLA_LAUNCH((gated_backward_pieces<T, ACT>), grid, dim3(256), 0, stream, zp, dp, dy_stride, op, pieces, per_row); \
    else if (epilogue_form) VIOLA_LAUNCH((gated_forward_pieces<T, ACT, true>), grid, dim3(256), 0, stream, zp, op, pieces, per_row); \
    else VIOLA_LAUNCH((gated_forward_pieces<T, ACT, false>), grid, dim3(256), 0, stream, zp, op, pieces, per_row);
    if (activation == VIOLA_SILU) { VIOLA_GATED(VIOLA_SILU) }
    else if (activation == VIOLA_GELU) { VIOLA_GATED(VIOLA_GELU) }
    else { VIOLA_GATED(VIOLA_RELU) }
#undef VIOLA_GATED
    return true;
}

// The gated activation in 16-byte pieces: forward out [rows, h] = act(g) * u from z = [g | u]; backward out [rows, 2 h] from
// z and dy (row stride dy_stride elements). False, and nothing launched, when alignment does not allow the pieces.
bool launch_gated_pieces(const void* z, const void* dy, int64_t dy_stride, void* out, int64_t rows, int64_t h, int dtype,
                         int activation, bool backward, bool epilogue_form, hipStream_t stream) {
    if (dtype == VIOLA_F32) return launch_gated_pieces<float>(z, dy, dy_stride, out, rows, h, activation, backward, epilogue_form, stream);
    if (dtype == VIOLA_BF16) return launch_gated_pieces<bf16_t>(z, dy, dy_stride, out, rows, h, activation, backward, epilogue_form, stream);
    return launch_gated_pieces<f16_t>(z, dy, dy_stride, out, rows, h, activation, backward, epilogue_form, stream);
}

// ------------------------------------------------------------------ self checks
// Hardware v_cvt_pk_{fp8,bf8}_f32 / v_cvt_f32_{fp8,bf8} against the software codecs.
__global__ __launch_bounds__(256) void selftest_fp8_kernel(unsigned long long* counts) {
    unsigned long long bad[4] = {0, 0, 0, 0};
    const uint64_t gid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x, stride = (uint64_t)gridDim.x * blockDim.x;
    for (uint64_t bits = gid; bits < (1ull << 32); bits += stride) {
        const float x = __uint_as_float((uint32_t)bits);
        const float a = fabsf(x);
        // up to (excluding) the first value that rounds past the largest finite code: a quotient v / s with
        // s = RN(amax / max) may exceed the maximum in its last place and must still round to it
        if (a < 464.0f) {
            const uint32_t hw = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(x, x, 0, false) & 0xffu;
            if (hw != f32_to_e4m3(x)) ++bad[0];
        }
        if (a < 61440.0f) {
            const uint32_t hw = (uint32_t)__builtin_amdgcn_cvt_pk_bf8_f32(x, x, 0, false) & 0xffu;
            if (hw != f32_to_e5m2(x)) ++bad[1];
        }
    }
    if (gid < 256) {
        const uint32_t c = (uint32_t)gid;
        const float hw4 = __builtin_amdgcn_cvt_f32_fp8((int)c, 0), sw4 = e4m3_to_f32(c);
        const float hw5 = __builtin_amdgcn_cvt_f32_bf8((int)c, 0), sw5 = e5m2_to_f32(c);
        const bool nan4 = sw4 != sw4, nan5 = sw5 != sw5;
        if (nan4 ? hw4 == hw4 : __float_as_uint(hw4) != __float_as_uint(sw4)) ++bad[2];
        if (nan5 ? hw5 == hw5 : __float_as_uint(hw5) != __float_as_uint(sw5)) ++bad[3];
    }
    for (int i = 0; i < 4; ++i)
        if (bad[i]) atomicAdd(&counts[i], bad[i]);
}

__global__ void selftest_philox_kernel(const uint64_t* __restrict__ triples, uint32_t* __restrict__ out, int64_t count) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count) out[i] = philox(triples[3 * i], triples[3 * i + 1], triples[3 * i + 2]);
}

static unsigned grid_for(int64_t n) {
    const int64_t blocks = (n + 255) / 256;
    return (unsigned)(blocks < 1 ? 1 : blocks > 65536 * 8 ? 65536 * 8 : blocks);
}

// Blocks for a launch whose blocks walk `steps` steps of work with the grid's stride, `lanes` such walks side by side
// (buckets): enough blocks to keep every CU's wavefront slots filled a few times over, no more.
#ifndef COMM_BLOCKS_PER_CU
#define COMM_BLOCKS_PER_CU 64
#endif
#ifndef COMM_ROWS_FROM
#define COMM_ROWS_FROM 4096                                              // tiles from which one bucket takes the row-per-tile kernel
#endif
static unsigned comm_walkers(int64_t steps, int64_t lanes) {
    const int64_t budget = (256 * COMM_BLOCKS_PER_CU + lanes - 1) / lanes;
    return (unsigned)(steps < 1 ? 1 : steps < budget ? steps : budget);
}

template <typename TQ>
static int launch_pack(const float* x, int64_t n, uint8_t* packet, int64_t rows, int64_t groups, int tile, int64_t stride,
                       hipStream_t stream) {
    const int64_t units = rows * groups;
    if (tile == 256 && reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(packet) % 4 == 0 && units >= COMM_ROWS_FROM) {
        VIOLA_LAUNCH(comm_pack256_rows_kernel<TQ>, dim3(comm_walkers((units + 15) / 16, 1)), dim3(256), 0, stream, x, n, packet, rows, groups, stride);
    } else if (tile == 256 && reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(packet) % 4 == 0) {
        VIOLA_LAUNCH(comm_pack256_kernel<TQ>, dim3((unsigned)((units + 3) / 4)), dim3(256), 0, stream, x, n, packet, rows, groups, stride);
    } else if (tile >= 64) {
        VIOLA_LAUNCH((comm_pack_kernel<TQ, 64>), dim3((unsigned)((units + 3) / 4)), dim3(256), 0, stream, x, n, packet, rows, groups, tile, stride);
    } else {
        VIOLA_LAUNCH((comm_pack_kernel<TQ, 32>), dim3((unsigned)((units + 7) / 8)), dim3(256), 0, stream, x, n, packet, rows, groups, tile, stride);
    }
    return viola_launch_status();
}

}  // namespace viola

using namespace viola;

extern "C" int viola_comm_pack(const float* x, int64_t n, void* packet, int64_t rows, int64_t groups, int tile, int fp8_dtype,
                               viola_stream_t stream_) {
    hipStream_t stream = viola_enter(stream_);
    VIOLA_CHECK_ARG(viola_is_fp8(fp8_dtype) && n >= 0 && rows >= 0 && groups >= 0 && tile >= 32 && (tile & (tile - 1)) == 0);
    if (rows == 0 || groups == 0) return 0;
    VIOLA_CHECK_ARG(packet && (n == 0 || x) && reinterpret_cast<uintptr_t>(packet) % 4 == 0);
    const int64_t stride = (groups * (tile + 4) + 15) / 16 * 16;
    VIOLA_CHECK_ARG((rows * groups + 3) / 4 < (1ll << 31));
    if (fp8_dtype == VIOLA_E4M3) return launch_pack<e4m3_t>(x, n, static_cast<uint8_t*>(packet), rows, groups, tile, stride, stream);
    return launch_pack<e5m2_t>(x, n, static_cast<uint8_t*>(packet), rows, groups, tile, stride, stream);
}

extern "C" int viola_comm_unpack(const void* packet, float* out, int64_t n, int64_t rows, int64_t groups, int tile,
                                 int fp8_dtype, int reduce, viola_stream_t stream_) {
    hipStream_t stream = viola_enter(stream_);
    VIOLA_CHECK_ARG(viola_is_fp8(fp8_dtype) && n >= 0 && rows >= 0 && groups >= 0 && tile >= 32 && (tile & (tile - 1)) == 0);
    if (rows == 0 || groups == 0 || n == 0) return 0;
    VIOLA_CHECK_ARG(packet && out && reinterpret_cast<uintptr_t>(packet) % 4 == 0);
    VIOLA_CHECK_ARG(n <= (reduce ? 1 : rows) * groups * tile);
    const int64_t stride = (groups * (tile + 4) + 15) / 16 * 16;
    const int64_t total = (reduce ? 1 : rows) * groups * tile;
    const uint8_t* pk = static_cast<const uint8_t*>(packet);
    if (reinterpret_cast<uintptr_t>(out) % 16 == 0) {
        const int64_t width = groups * tile;
        const int shift = __builtin_ctz((unsigned)tile);
        const dim3 grid(comm_walkers((total / 4 + 1023) / 1024, 1));
#define VIOLA_UNPACK(TQ, REDUCE) VIOLA_LAUNCH((comm_unpack_quads_kernel<TQ, REDUCE>), grid, dim3(256), 0, stream, pk, out, n, rows, width, shift, stride)
        if (fp8_dtype == VIOLA_E4M3) { if (reduce) VIOLA_UNPACK(e4m3_t, true); else VIOLA_UNPACK(e4m3_t, false); }
        else { if (reduce) VIOLA_UNPACK(e5m2_t, true); else VIOLA_UNPACK(e5m2_t, false); }
#undef VIOLA_UNPACK
        return viola_launch_status();
    }
    if (fp8_dtype == VIOLA_E4M3) VIOLA_LAUNCH(comm_unpack_kernel<e4m3_t>, dim3(grid_for(total)), dim3(256), 0, stream, pk, out, n, rows, groups, tile, stride, reduce);
    else VIOLA_LAUNCH(comm_unpack_kernel<e5m2_t>, dim3(grid_for(total)), dim3(256), 0, stream, pk, out, n, rows, groups, tile, stride, reduce);
    return viola_launch_status();
}

extern "C" int viola_comm_pack_table(const int64_t* table, int64_t buckets, int64_t max_units, int tile, int fp8_dtype,
                                     viola_stream_t stream_) {
    hipStream_t stream = viola_enter(stream_);
    VIOLA_CHECK_ARG(viola_is_fp8(fp8_dtype) && buckets >= 0 && max_units >= 0 && tile >= 32 && (tile & (tile - 1)) == 0);
    if (buckets == 0 || max_units == 0) return 0;
    VIOLA_CHECK_ARG(table && buckets <= 65535 && (max_units + 3) / 4 < (1ll << 31));
    if (tile != 256) return VIOLA_EUNSUPPORTED;                                    // other tiles: one viola_comm_pack per bucket
    const dim3 grid(comm_walkers((max_units + 15) / 16, buckets), (unsigned)buckets);
    if (fp8_dtype == VIOLA_E4M3) VIOLA_LAUNCH(comm_pack256_table_kernel<e4m3_t>, grid, dim3(256), 0, stream, table);
    else VIOLA_LAUNCH(comm_pack256_table_kernel<e5m2_t>, grid, dim3(256), 0, stream, table);
    return viola_launch_status();
}

extern "C" int viola_comm_unpack_table(const int64_t* table, int64_t buckets, int64_t max_elements, int tile, int fp8_dtype,
                                       int reduce, viola_stream_t stream_) {
    hipStream_t stream = viola_enter(stream_);
    VIOLA_CHECK_ARG(viola_is_fp8(fp8_dtype) && buckets >= 0 && max_elements >= 0 && tile >= 32 && (tile & (tile - 1)) == 0);
    if (buckets == 0 || max_elements == 0) return 0;
    VIOLA_CHECK_ARG(table && buckets <= 65535);
    const int shift = __builtin_ctz((unsigned)tile);
    const dim3 grid(comm_walkers((max_elements / 4 + 1023) / 1024, buckets), (unsigned)buckets);
#define VIOLA_UNPACK(TQ, REDUCE) VIOLA_LAUNCH((comm_unpack_quads_table_kernel<TQ, REDUCE>), grid, dim3(256), 0, stream, table, tile, shift)
    if (fp8_dtype == VIOLA_E4M3) { if (reduce) VIOLA_UNPACK(e4m3_t, true); else VIOLA_UNPACK(e4m3_t, false); }
    else { if (reduce) VIOLA_UNPACK(e5m2_t, true); else VIOLA_UNPACK(e5m2_t, false); }
#undef VIOLA_UNPACK
    return viola_launch_status();
}

extern "C" int viola_gated_forward(const void* z, void* out, int64_t rows, int64_t h, int dtype, int activation,
                                   viola_stream_t stream_) {
    hipStream_t stream = viola_enter(stream_);
    VIOLA_CHECK_ARG(viola_is_float(dtype) && rows >= 0 && h >= 0 && activation >= VIOLA_SILU && activation <= VIOLA_RELU);
    if (rows == 0 || h == 0) return 0;
    VIOLA_CHECK_ARG(z && out);
    if (launch_gated_pieces(z, nullptr, 0, out, rows, h, dtype, activation, false, false, stream)) return viola_launch_status();
    VIOLA_LAUNCH(gated_forward_kernel, dim3(grid_for(rows * h)), dim3(256), 0, stream, z, out, rows, h, dtype, activation);
    return viola_launch_status();
}

extern "C" int viola_gated_backward(const void* z, const void* dy, void* dz, int64_t rows, int64_t h, int dtype,
                                    int activation, viola_stream_t stream_) {
    hipStream_t stream = viola_enter(stream_);
    VIOLA_CHECK_ARG(viola_is_float(dtype) && rows >= 0 && h >= 0 && activation >= VIOLA_SILU && activation <= VIOLA_RELU);
    if (rows == 0 || h == 0) return 0;
    VIOLA_CHECK_ARG(z && dy && dz);
    if (launch_gated_pieces(z, dy, h, dz, rows, h, dtype, activation, true, false, stream)) return viola_launch_status();
    VIOLA_LAUNCH(gated_backward_kernel, dim3(grid_for(rows * h)), dim3(256), 0, stream, z, dy, dz, rows, h, dtype, activation);
    return viola_launch_status();
}

extern "C" int viola_selftest_fp8(uint64_t* counts, viola_stream_t stream_) {
    hipStream_t stream = viola_enter(stream_);
    VIOLA_CHECK_ARG(counts);
    VIOLA_LAUNCH(selftest_fp8_kernel, dim3(4096), dim3(256), 0, stream, reinterpret_cast<unsigned long long*>(counts));
    return viola_launch_status();
}

extern "C" int viola_selftest_philox(const uint64_t* triples, uint32_t* out, int64_t count, viola_stream_t stream_) {
    hipStream_t stream = viola_enter(stream_);
    VIOLA_CHECK_ARG(count >= 0);
    if (count == 0) return 0;
    VIOLA_CHECK_ARG(triples && out);
    VIOLA_LAUNCH(selftest_philox_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, stream, triples, out, count);
    return viola_launch_status();
}

extern "C" int viola_abi_version(void) { return 1; }

extern "C" const char* viola_error_string(int code) {
    if (code == 0) return "success";
    if (code == VIOLA_EINVAL) return "invalid argument (nothing launched)";
    if (code == VIOLA_EUNSUPPORTED) return "unsupported configuration (nothing launched)";
    if (code == VIOLA_ETOOLARGE) return "size beyond the library's built-in scratch buffer (nothing launched)";
    return hipGetErrorString(static_cast<hipError_t>(code));
}
