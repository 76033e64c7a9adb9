// Per-tensor FP8 scaling for gfx950 (the `current` / `delayed` recipes): absolute maximum of a tensor in two
// steps, the scale with its amax history, and the quantizer that writes the row-wise codes, the transposed
// codes or both from one read. Built with -ffp-contract=off.
#include "common.hpp"

namespace viola {

// ------------------------------------------------------------------ amax
template <typename TIn> struct Vec16;                       // 16 bytes of TIn
template <> struct Vec16<float> { static constexpr int N = 4; };
template <> struct Vec16<bf16_t> { static constexpr int N = 8; };
template <> struct Vec16<f16_t> { static constexpr int N = 8; };

template <typename TIn>
__device__ __forceinline__ float absmax16(const TIn* p) {
    const uint4 raw = *reinterpret_cast<const uint4*>(p);
    float m = 0.0f;
    if constexpr (sizeof(TIn) == 4) {
        m = fmaxf(fmaxf(fabsf(__uint_as_float(raw.x)), fabsf(__uint_as_float(raw.y))),
                  fmaxf(fabsf(__uint_as_float(raw.z)), fabsf(__uint_as_float(raw.w))));
    } else {
        const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            TIn lo, hi;
            __builtin_memcpy(&lo, reinterpret_cast<const uint16_t*>(&w[i]), 2);
            __builtin_memcpy(&hi, reinterpret_cast<const uint16_t*>(&w[i]) + 1, 2);
            m = fmaxf(m, fmaxf(fabsf(to_f32(lo)), fabsf(to_f32(hi))));
        }
    }
    return m;
}

// maxima[block] = max |x| over the block's share (fmaxf drops NaN, as the reference's reduction does). The head up to
// the first 16-byte boundary and the tail go element-wise through block 0.
template <typename TIn>
__global__ __launch_bounds__(256) void tensor_amax_kernel(const TIn* __restrict__ x, int64_t n, float* __restrict__ maxima) {
    constexpr int N = Vec16<TIn>::N;
    const uintptr_t address = reinterpret_cast<uintptr_t>(x);
    int64_t head = ((16 - address % 16) % 16) / (int64_t)sizeof(TIn);
    if (head > n) head = n;
    const int64_t vectors = (n - head) / N;
    float m = 0.0f;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    int64_t v = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    for (; v + 3 * stride < vectors; v += 4 * stride) {        // four loads in flight
        const float a = absmax16<TIn>(x + head + v * N), b = absmax16<TIn>(x + head + (v + stride) * N);
        const float c = absmax16<TIn>(x + head + (v + 2 * stride) * N), d = absmax16<TIn>(x + head + (v + 3 * stride) * N);
        m = fmaxf(m, fmaxf(fmaxf(a, b), fmaxf(c, d)));
    }
    for (; v < vectors; v += stride) m = fmaxf(m, absmax16<TIn>(x + head + v * N));
    if (blockIdx.x == 0) {
        for (int64_t i = threadIdx.x; i < head; i += blockDim.x) m = fmaxf(m, fabsf(to_f32(x[i])));
        for (int64_t i = head + vectors * N + threadIdx.x; i < n; i += blockDim.x) m = fmaxf(m, fabsf(to_f32(x[i])));
    }
    __shared__ float part[4];
    m = wave_max(m);
    if (threadIdx.x % WAVE == 0) part[threadIdx.x / WAVE] = m;
    __syncthreads();
    if (threadIdx.x == 0) maxima[blockIdx.x] = fmaxf(fmaxf(part[0], part[1]), fmaxf(part[2], part[3]));
}

// The same maximum together with column sums of a [rows, cols] matrix from the one read (the bias gradient of a
// Linear rides on the amax pass over dY): block (x, y) covers 256 column pieces of 16 bytes and row slice y,
// maxima[y * gridDim.x + x] = its max |x|, column_partial[y][c] = its fp32 column sums. cols is a multiple of the
// piece, x 16-byte aligned.
template <typename TIn>
__global__ __launch_bounds__(256) void tensor_amax_columns_kernel(const TIn* __restrict__ x, int64_t rows, int64_t cols,
                                                                   int64_t slice_rows, float* __restrict__ maxima,
                                                                   float* __restrict__ column_partial) {
    constexpr int N = Vec16<TIn>::N;
    const int64_t col = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * N;
    const int64_t begin = (int64_t)blockIdx.y * slice_rows, end = begin + slice_rows < rows ? begin + slice_rows : rows;
    float sum[N];
#pragma unroll
    for (int i = 0; i < N; ++i) sum[i] = 0.0f;
    float m = 0.0f;
    if (col < cols) {
        auto take = [&](int64_t r) {
            const uint4 raw = *reinterpret_cast<const uint4*>(x + r * cols + col);
            const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
            float v[N];
            if constexpr (sizeof(TIn) == 4) {
#pragma unroll
                for (int i = 0; i < 4; ++i) v[i] = __uint_as_float(w[i]);
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    TIn lo, hi;
                    __builtin_memcpy(&lo, reinterpret_cast<const uint16_t*>(&w[i]), 2);
                    __builtin_memcpy(&hi, reinterpret_cast<const uint16_t*>(&w[i]) + 1, 2);
                    v[2 * i] = to_f32(lo);
                    v[2 * i + 1] = to_f32(hi);
                }
            }
#pragma unroll
            for (int i = 0; i < N; ++i) { sum[i] += v[i]; m = fmaxf(m, fabsf(v[i])); }
        };
        int64_t r = begin;
        for (; r + 3 < end; r += 4) { take(r); take(r + 1); take(r + 2); take(r + 3); }
        for (; r < end; ++r) take(r);
        float* dst = column_partial + (int64_t)blockIdx.y * cols + col;
#pragma unroll
        for (int i = 0; i < N; i += 4) *reinterpret_cast<float4*>(dst + i) = make_float4(sum[i], sum[i + 1], sum[i + 2], sum[i + 3]);
    }
    __shared__ float part[4];
    m = wave_max(m);
    if (threadIdx.x % WAVE == 0) part[threadIdx.x / WAVE] = m;
    __syncthreads();
    if (threadIdx.x == 0) maxima[(int64_t)blockIdx.y * gridDim.x + blockIdx.x] = fmaxf(fmaxf(part[0], part[1]), fmaxf(part[2], part[3]));
}

// One block: amax = max(maxima); scale = max(delayed and index != 0 ? max(history before this call) : amax, 1e-30) / limit;
// history[index % history_len] = amax.
__global__ __launch_bounds__(256) void tensor_scale_kernel(const float* __restrict__ maxima, int64_t parts, float* history,
                                                            int history_len, int64_t index, int delayed, float limit,
                                                            float* __restrict__ scale) {
    float current = 0.0f, previous = 0.0f;
    for (int64_t i = threadIdx.x; i < parts; i += blockDim.x) current = fmaxf(current, maxima[i]);
    for (int i = threadIdx.x; i < history_len; i += blockDim.x) previous = fmaxf(previous, history[i]);
    __shared__ float part[2][4];
    current = wave_max(current);
    previous = wave_max(previous);
    if (threadIdx.x % WAVE == 0) { part[0][threadIdx.x / WAVE] = current; part[1][threadIdx.x / WAVE] = previous; }
    __syncthreads();                                            // every read of history is done
    if (threadIdx.x == 0) {
        const float amax = fmaxf(fmaxf(part[0][0], part[0][1]), fmaxf(part[0][2], part[0][3]));
        const float old = fmaxf(fmaxf(part[1][0], part[1][1]), fmaxf(part[1][2], part[1][3]));
        scale[0] = scale_of(delayed && index != 0 ? old : amax, limit);
        history[index % history_len] = amax;
    }
}

// ------------------------------------------------------------------ quantize (+ transpose)
template <typename TOut>
__device__ __forceinline__ uint8_t encode_tensor(float v, float s, float limit) {
    // the reference keeps a NaN input and sends everything else through min(max(v / s, -limit), limit); with an
    // infinite scale an infinite input makes that quotient NaN, which fmaxf turns into -limit
    const float c = v != v ? v : fminf(fmaxf(v / s, -limit), limit);
    return from_f32<TOut>(c).bits;
}

template <typename TIn>
__device__ __forceinline__ void load16(const TIn* row, int64_t c0, int64_t cols, bool row_inside, bool vector, float (&v)[16]) {
    if (row_inside && vector && c0 + 16 <= cols) {
        if constexpr (sizeof(TIn) == 4) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float4 t = *reinterpret_cast<const float4*>(row + c0 + 4 * i);
                v[4 * i] = t.x; v[4 * i + 1] = t.y; v[4 * i + 2] = t.z; v[4 * i + 3] = t.w;
            }
        } else {
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const uint4 raw = *reinterpret_cast<const uint4*>(row + c0 + 8 * i);
                const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    TIn lo, hi;
                    __builtin_memcpy(&lo, reinterpret_cast<const uint16_t*>(&w[j]), 2);
                    __builtin_memcpy(&hi, reinterpret_cast<const uint16_t*>(&w[j]) + 1, 2);
                    v[8 * i + 2 * j] = to_f32(lo);
                    v[8 * i + 2 * j + 1] = to_f32(hi);
                }
            }
        }
    } else {
#pragma unroll
        for (int i = 0; i < 16; ++i) v[i] = row_inside && c0 + i < cols ? to_f32(row[c0 + i]) : 0.0f;
    }
}

// ------------------------------------------------------------------ Hadamard-64 rotation of channel groups
// H64 = H4 (x) H4 (x) H4 with H4 = (ones(4, 4) - 2 flip(eye(4))) / 2, symmetric and its own inverse, applied to 64
// consecutive columns. Three stages with strides 1, 4 and 16, each in the reference's operation order
// (_rotation_kernels.py:11-25): out[j] = ((v[b] + v[b + s]) + (v[b + 2s] + v[b + 3s])) * 0.5 - v[b + (3 - digit) s],
// b = j with base-4 digit `digit` of weight s cleared. A quad of lanes holds the 64 values, 16 consecutive ones each:
// strides 1 and 4 stay inside a lane, stride 16 pairs the same register of the four lanes (DPP quad permutes; float
// addition commutes, so every lane forms (v0 + v1) + (v2 + v3) bit for bit).
__device__ __forceinline__ float quad_perm(float v, int control) {
    if (control == 0xB1) return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0xB1, 0xf, 0xf, true));   // lanes 1 0 3 2
    if (control == 0x4E) return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x4E, 0xf, 0xf, true));   // lanes 2 3 0 1
    return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x1B, 0xf, 0xf, true));                        // lanes 3 2 1 0
}

__device__ __forceinline__ void rotate64(float (&v)[16]) {
    float t[16];
#pragma unroll
    for (int g = 0; g < 4; ++g) {                                           // stride 1
        const float half = ((v[4 * g] + v[4 * g + 1]) + (v[4 * g + 2] + v[4 * g + 3])) * 0.5f;
#pragma unroll
        for (int d = 0; d < 4; ++d) t[4 * g + d] = half - v[4 * g + 3 - d];
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {                                           // stride 4
        const float half = ((t[r] + t[r + 4]) + (t[r + 8] + t[r + 12])) * 0.5f;
#pragma unroll
        for (int d = 0; d < 4; ++d) v[r + 4 * d] = half - t[r + 4 * (3 - d)];
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) {                                          // stride 16: digit = lane % 4
        const float pair = v[i] + quad_perm(v[i], 0xB1);
        const float half = (pair + quad_perm(pair, 0x4E)) * 0.5f;
        t[i] = half - quad_perm(v[i], 0x1B);
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) v[i] = t[i];
}

// maxima[block] = max |rotated x| over a 64 x 64 tile (columns past the end count as zeros inside their group, as in
// _rotation_kernels.py:28-47; fmaxf drops NaN like the reference's reduction).
template <typename TIn>
__global__ __launch_bounds__(256) void rotation_amax_kernel(const TIn* __restrict__ x, int64_t rows, int64_t cols, int vector_in,
                                                             float* __restrict__ maxima) {
    const int tid = threadIdx.x;
    const int64_t row = (int64_t)blockIdx.y * 64 + tid / 4, col = (int64_t)blockIdx.x * 64 + (tid % 4) * 16;
    float v[16];
    load16<TIn>(x + row * cols, col, cols, row < rows, vector_in != 0, v);
    rotate64(v);
    float m = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; ++i) m = fmaxf(m, fabsf(v[i]));
    __shared__ float part[4];
    m = wave_max(m);
    if (tid % WAVE == 0) part[tid / WAVE] = m;
    __syncthreads();
    if (tid == 0) maxima[(int64_t)blockIdx.y * gridDim.x + blockIdx.x] = fmaxf(fmaxf(part[0], part[1]), fmaxf(part[2], part[3]));
}

// x <- rotated x, rounded to the tensor's own type (_rotation_kernels.py:83-97): every block owns whole groups.
template <typename T>
__global__ __launch_bounds__(256) void rotation_inplace_kernel(T* __restrict__ x, int64_t rows, int64_t cols, int vector_in) {
    const int tid = threadIdx.x;
    const int64_t row = (int64_t)blockIdx.y * 64 + tid / 4, col = (int64_t)blockIdx.x * 64 + (tid % 4) * 16;
    float v[16];
    load16<T>(x + row * cols, col, cols, row < rows, vector_in != 0, v);
    rotate64(v);
    if (row >= rows) return;
    T* dst = x + row * cols + col;
    if (vector_in && col + 16 <= cols) {
        if constexpr (sizeof(T) == 4) {
#pragma unroll
            for (int i = 0; i < 4; ++i) *reinterpret_cast<float4*>(dst + 4 * i) = make_float4(v[4 * i], v[4 * i + 1], v[4 * i + 2], v[4 * i + 3]);
        } else {
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                uint32_t w[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const T lo = from_f32<T>(v[8 * i + 2 * j]), hi = from_f32<T>(v[8 * i + 2 * j + 1]);
                    uint16_t a, b;
                    __builtin_memcpy(&a, &lo, 2);
                    __builtin_memcpy(&b, &hi, 2);
                    w[j] = (uint32_t)a | ((uint32_t)b << 16);
                }
                *reinterpret_cast<uint4*>(dst + 8 * i) = make_uint4(w[0], w[1], w[2], w[3]);
            }
        }
    } else {
        for (int i = 0; i < 16; ++i)
            if (col + i < cols) dst[i] = from_f32<T>(v[i]);
    }
}

// 64 x 64 tile per 256-thread block: thread t quantizes 16 consecutive elements of tile row t / 4, stores them
// row-wise (16 bytes) and, for the transposed layout, parks them in LDS, from where thread t collects 16 consecutive
// rows of tile column t / 4. q = fp8(isnan(v) ? v : clamp(v / scale, +-limit)) with the one scale of the tensor.
// ROTATE: the values are Hadamard-rotated in their 64-column groups first (_rotation_kernels.py:50-80).
template <typename TIn, typename TOut, bool ROTATE>
__global__ __launch_bounds__(256) void tensor_quantize_kernel(const TIn* __restrict__ x, const float* __restrict__ scale,
                                                               uint8_t* __restrict__ q, uint8_t* __restrict__ qt, int64_t rows,
                                                               int64_t cols, float limit, int vector_in, int vector_q,
                                                               int vector_qt) {
    constexpr int LD = 64 + 16;                                         // padded row of the parking tile (bytes)
    __shared__ __attribute__((aligned(16))) uint8_t park[64 * LD];
    const int tid = threadIdx.x, lr = tid / 4, lc = (tid % 4) * 16;
    // blocks are dispatched in index order: those in flight together take a patch of 32 row tiles per column tile, then
    // the next column tile, so the transposed output is written in 2 KB runs per row however wide the matrix is
    constexpr int64_t BAND = 32;
    const int64_t tiles_x = gridDim.x, tiles_y = gridDim.y, id = (int64_t)blockIdx.y * tiles_x + blockIdx.x;
    const int64_t patch = id / (BAND * tiles_x), within = id % (BAND * tiles_x);
    const int64_t tall = tiles_y - patch * BAND < BAND ? tiles_y - patch * BAND : BAND;
    const int64_t r0 = (patch * BAND + within % tall) * 64, c0 = within / tall * 64;
    const int64_t row = r0 + lr, col = c0 + lc;
    const float s = scale[0];
    float v[16];
    load16<TIn>(x + row * cols, col, cols, row < rows, vector_in != 0, v);
    if constexpr (ROTATE) rotate64(v);
    float poison = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; ++i) poison = poison_of(poison, v[i]);
    const bool any_bad = __builtin_amdgcn_ballot_w64(poison != poison) != 0;
    const SharedDivisor d(s, any_bad ? __uint_as_float(0x7fc00000u) : 0.0f);
    uint32_t w[4];
    if (d.fast) {
#pragma unroll
        for (int i = 0; i < 4; ++i) w[i] = fast_encode4<TOut>(d, limit, v[4 * i], v[4 * i + 1], v[4 * i + 2], v[4 * i + 3]);
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            w[i] = 0;
#pragma unroll
            for (int e = 0; e < 4; ++e) w[i] |= (uint32_t)encode_tensor<TOut>(v[4 * i + e], s, limit) << (8 * e);
        }
    }
    if (q && row < rows) {
        uint8_t* dst = q + row * cols + col;
        if (vector_q && col + 16 <= cols) {
            *reinterpret_cast<uint4*>(dst) = make_uint4(w[0], w[1], w[2], w[3]);
        } else {
            for (int i = 0; i < 16; ++i)
                if (col + i < cols) dst[i] = (uint8_t)(w[i / 4] >> (8 * (i % 4)));
        }
    }
    if (qt) {
        *reinterpret_cast<uint4*>(park + lr * LD + lc) = make_uint4(w[0], w[1], w[2], w[3]);
        __syncthreads();
        // output row = tile column lr, 16 consecutive tile rows lc .. lc + 15
        uint32_t t[4] = {0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < 16; ++i) t[i / 4] |= (uint32_t)park[(lc + i) * LD + lr] << (8 * (i % 4));
        const int64_t orow = c0 + lr, ocol = r0 + lc;
        if (orow < cols) {
            uint8_t* dst = qt + orow * rows + ocol;
            if (vector_qt && ocol + 16 <= rows) {
                *reinterpret_cast<uint4*>(dst) = make_uint4(t[0], t[1], t[2], t[3]);
            } else {
                for (int i = 0; i < 16; ++i)
                    if (ocol + i < rows) dst[i] = (uint8_t)(t[i / 4] >> (8 * (i % 4)));
            }
        }
    }
}

template <typename TIn, typename TOut, bool ROTATE>
static int launch_tensor_quantize(const void* x, const float* scale, void* q, void* qt, int64_t rows, int64_t cols, float limit,
                                  hipStream_t stream) {
    const int vector_in = reinterpret_cast<uintptr_t>(x) % 16 == 0 && (cols * sizeof(TIn)) % 16 == 0;
    const int vector_q = q && reinterpret_cast<uintptr_t>(q) % 16 == 0 && cols % 16 == 0;
    const int vector_qt = qt && reinterpret_cast<uintptr_t>(qt) % 16 == 0 && rows % 16 == 0;
    const dim3 grid((unsigned)((cols + 63) / 64), (unsigned)((rows + 63) / 64));
    VIOLA_LAUNCH((tensor_quantize_kernel<TIn, TOut, ROTATE>), grid, dim3(256), 0, stream, static_cast<const TIn*>(x), scale,
                       static_cast<uint8_t*>(q), static_cast<uint8_t*>(qt), rows, cols, limit, vector_in, vector_q, vector_qt);
    return viola_launch_status();
}

}  // namespace viola

using namespace viola;

extern "C" int viola_tensor_amax(const void* x, int x_dtype, int64_t n, float* maxima, int64_t parts, viola_stream_t stream_) {
    hipStream_t stream = viola_enter(stream_);
    VIOLA_CHECK_ARG(viola_is_float(x_dtype) && n >= 0 && parts > 0 && parts <= 65535 && maxima && (n == 0 || x));
    const dim3 grid((unsigned)parts);
    if (x_dtype == VIOLA_F32) VIOLA_LAUNCH(tensor_amax_kernel<float>, grid, dim3(256), 0, stream, static_cast<const float*>(x), n, maxima);
    else if (x_dtype == VIOLA_BF16) VIOLA_LAUNCH(tensor_amax_kernel<bf16_t>, grid, dim3(256), 0, stream, static_cast<const bf16_t*>(x), n, maxima);
    else VIOLA_LAUNCH(tensor_amax_kernel<f16_t>, grid, dim3(256), 0, stream, static_cast<const f16_t*>(x), n, maxima);
    return viola_launch_status();
}

extern "C" int viola_tensor_scale(const float* maxima, int64_t parts, float* history, int history_len, int64_t index,
                                  int delayed, float limit, float* scale, viola_stream_t stream_) {
    hipStream_t stream = viola_enter(stream_);
    VIOLA_CHECK_ARG(maxima && parts > 0 && history && history_len > 0 && index >= 0 && limit > 0.0f && scale);
    VIOLA_LAUNCH(tensor_scale_kernel, dim3(1), dim3(256), 0, stream, maxima, parts, history, history_len, index, delayed, limit, scale);
    return viola_launch_status();
}

extern "C" int viola_tensor_amax_columns(const void* x, int x_dtype, int64_t rows, int64_t cols, int64_t slices, float* maxima,
                                         float* column_partial, viola_stream_t stream_) {
    hipStream_t stream = viola_enter(stream_);
    VIOLA_CHECK_ARG(viola_is_float(x_dtype) && rows > 0 && cols > 0 && slices > 0 && slices <= 65535 && x && maxima && column_partial);
    const int piece = 16 / viola_dtype_size(x_dtype);
    VIOLA_CHECK_ARG(cols % piece == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(column_partial) % 16 == 0);
    const int64_t slice_rows = (rows + slices - 1) / slices;
    const dim3 grid((unsigned)((cols / piece + 255) / 256), (unsigned)slices);
    if (x_dtype == VIOLA_F32) VIOLA_LAUNCH(tensor_amax_columns_kernel<float>, grid, dim3(256), 0, stream, static_cast<const float*>(x), rows, cols, slice_rows, maxima, column_partial);
    else if (x_dtype == VIOLA_BF16) VIOLA_LAUNCH(tensor_amax_columns_kernel<bf16_t>, grid, dim3(256), 0, stream, static_cast<const bf16_t*>(x), rows, cols, slice_rows, maxima, column_partial);
    else VIOLA_LAUNCH(tensor_amax_columns_kernel<f16_t>, grid, dim3(256), 0, stream, static_cast<const f16_t*>(x), rows, cols, slice_rows, maxima, column_partial);
    return viola_launch_status();
}

// viola_tensor_amax_columns, viola_tensor_scale and viola_column_reduce behind one call: the per-tensor scale of a
// [rows, cols] gradient and its column sums (the bias gradient) from one read, three launches, one trip from the host.
extern "C" int viola_column_reduce(const float* partial, int64_t parts, int64_t cols, void* out, int out_dtype,
                                   viola_stream_t stream);
extern "C" int viola_tensor_amax_columns_scale(const void* x, int x_dtype, int64_t rows, int64_t cols, int64_t slices,
                                               float* maxima, float* column_partial, float* history, int history_len,
                                               int64_t index, int delayed, float limit, float* scale, void* column_sum,
                                               int sum_dtype, viola_stream_t stream) {
    int status = viola_tensor_amax_columns(x, x_dtype, rows, cols, slices, maxima, column_partial, stream);
    if (status) return status;
    const int piece = 16 / viola_dtype_size(x_dtype);
    const int64_t parts = ((cols / piece + 255) / 256) * slices;
    status = viola_tensor_scale(maxima, parts, history, history_len, index, delayed, limit, scale, stream);
    return status ? status : viola_column_reduce(column_partial, slices, cols, column_sum, sum_dtype, stream);
}

extern "C" int viola_tensor_amax_scale(const void* x, int x_dtype, int64_t n, float* maxima, int64_t parts, float* history,
                                       int history_len, int64_t index, int delayed, float limit, float* scale,
                                       viola_stream_t stream) {
    const int status = viola_tensor_amax(x, x_dtype, n, maxima, parts, stream);
    return status ? status : viola_tensor_scale(maxima, parts, history, history_len, index, delayed, limit, scale, stream);
}

template <bool ROTATE>
static int tensor_quantize_entry(const void* x, int x_dtype, int64_t rows, int64_t cols, const float* scale, void* q,
                                 void* qt, int q_dtype, float limit, hipStream_t stream) {
    VIOLA_CHECK_ARG(viola_is_float(x_dtype) && viola_is_fp8(q_dtype) && rows >= 0 && cols >= 0 && limit > 0.0f);
    if (rows == 0 || cols == 0 || (!q && !qt)) return 0;
    VIOLA_CHECK_ARG(x && scale && (rows + 63) / 64 <= 65535);
#define VIOLA_TQ(TI, TO) return launch_tensor_quantize<TI, TO, ROTATE>(x, scale, q, qt, rows, cols, limit, stream)
    if (q_dtype == VIOLA_E4M3) {
        if (x_dtype == VIOLA_F32) VIOLA_TQ(float, e4m3_t);
        if (x_dtype == VIOLA_BF16) VIOLA_TQ(bf16_t, e4m3_t);
        VIOLA_TQ(f16_t, e4m3_t);
    }
    if (x_dtype == VIOLA_F32) VIOLA_TQ(float, e5m2_t);
    if (x_dtype == VIOLA_BF16) VIOLA_TQ(bf16_t, e5m2_t);
    VIOLA_TQ(f16_t, e5m2_t);
#undef VIOLA_TQ
}

extern "C" int viola_tensor_quantize(const void* x, int x_dtype, int64_t rows, int64_t cols, const float* scale, void* q,
                                     void* qt, int q_dtype, float limit, viola_stream_t stream) {
    return tensor_quantize_entry<false>(x, x_dtype, rows, cols, scale, q, qt, q_dtype, limit, static_cast<hipStream_t>(stream));
}

extern "C" int viola_rotation_quantize(const void* x, int x_dtype, int64_t rows, int64_t cols, const float* scale, void* q,
                                       void* qt, int q_dtype, float limit, viola_stream_t stream) {
    return tensor_quantize_entry<true>(x, x_dtype, rows, cols, scale, q, qt, q_dtype, limit, static_cast<hipStream_t>(stream));
}

extern "C" int viola_rotation_amax(const void* x, int x_dtype, int64_t rows, int64_t cols, float* maxima, int64_t parts,
                                   viola_stream_t stream_) {
    hipStream_t stream = viola_enter(stream_);
    VIOLA_CHECK_ARG(viola_is_float(x_dtype) && rows > 0 && cols > 0 && x && maxima && (rows + 63) / 64 <= 65535);
    const dim3 grid((unsigned)((cols + 63) / 64), (unsigned)((rows + 63) / 64));
    VIOLA_CHECK_ARG(parts == (int64_t)grid.x * grid.y);
    const int vector_in = reinterpret_cast<uintptr_t>(x) % 16 == 0 && (cols * viola_dtype_size(x_dtype)) % 16 == 0;
    if (x_dtype == VIOLA_F32) VIOLA_LAUNCH(rotation_amax_kernel<float>, grid, dim3(256), 0, stream, static_cast<const float*>(x), rows, cols, vector_in, maxima);
    else if (x_dtype == VIOLA_BF16) VIOLA_LAUNCH(rotation_amax_kernel<bf16_t>, grid, dim3(256), 0, stream, static_cast<const bf16_t*>(x), rows, cols, vector_in, maxima);
    else VIOLA_LAUNCH(rotation_amax_kernel<f16_t>, grid, dim3(256), 0, stream, static_cast<const f16_t*>(x), rows, cols, vector_in, maxima);
    return viola_launch_status();
}

extern "C" int viola_rotation_inverse(void* x, int x_dtype, int64_t rows, int64_t cols, viola_stream_t stream_) {
    hipStream_t stream = viola_enter(stream_);
    VIOLA_CHECK_ARG(viola_is_float(x_dtype) && rows >= 0 && cols >= 0);
    if (rows == 0 || cols == 0) return 0;
    VIOLA_CHECK_ARG(x && (rows + 63) / 64 <= 65535);
    const dim3 grid((unsigned)((cols + 63) / 64), (unsigned)((rows + 63) / 64));
    const int vector_in = reinterpret_cast<uintptr_t>(x) % 16 == 0 && (cols * viola_dtype_size(x_dtype)) % 16 == 0;
    if (x_dtype == VIOLA_F32) VIOLA_LAUNCH(rotation_inplace_kernel<float>, grid, dim3(256), 0, stream, static_cast<float*>(x), rows, cols, vector_in);
    else if (x_dtype == VIOLA_BF16) VIOLA_LAUNCH(rotation_inplace_kernel<bf16_t>, grid, dim3(256), 0, stream, static_cast<bf16_t*>(x), rows, cols, vector_in);
    else VIOLA_LAUNCH(rotation_inplace_kernel<f16_t>, grid, dim3(256), 0, stream, static_cast<f16_t*>(x), rows, cols, vector_in);
    return viola_launch_status();
}
