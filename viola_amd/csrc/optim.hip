// FP8Muon elementwise kernels for gfx950: fused momentum update + e4m3 state codec (1-D tiles and
// 2-D blocks, nearest or Philox stochastic rounding), weight update, AdamW, copy_scaled.
// All arithmetic is un-contracted IEEE fp32 (built with -ffp-contract=off) in the order the
// reference kernels write it. Pointers need only element alignment: accesses are per element,
// lane-contiguous, so a wavefront still reads and writes whole cache lines.
#include "common.hpp"

namespace viola {

__device__ __forceinline__ float load_dtype(const void* p, int64_t i, int dtype) {
    if (dtype == VIOLA_F32) return static_cast<const float*>(p)[i];
    if (dtype == VIOLA_BF16) return bf16_bits_to_f32(static_cast<const uint16_t*>(p)[i]);
    return (float)static_cast<const _Float16*>(p)[i];
}

template <bool STOCHASTIC>
__device__ __forceinline__ void store_rounded(void* p, int64_t i, int dtype, float v, uint64_t element, uint64_t step, uint64_t key) {
    if (dtype == VIOLA_F32) {
        static_cast<float*>(p)[i] = v;
    } else if (dtype == VIOLA_BF16) {
        if (STOCHASTIC) v = stochastic_bf16(v, element, step, key);
        static_cast<uint16_t*>(p)[i] = f32_to_bf16_bits(v);
    } else {
        if (STOCHASTIC) v = stochastic_fp16(v, element, step, key);
        static_cast<_Float16*>(p)[i] = (_Float16)v;
    }
}

template <bool STOCHASTIC>
__device__ __forceinline__ uint8_t encode_state(float m, float scale, uint64_t element, uint64_t step, uint64_t key) {
    const float t = m / scale;
    float v = t != t ? t : fminf(fmaxf(t, -448.0f), 448.0f);      // NaN (also Inf/Inf) stays NaN
    if (STOCHASTIC) v = stochastic_e4m3(v, element, step, key);
    return f32_to_e4m3(v);
}

// ------------------------------------------------------------------ 1-D tiles: one wavefront per tile
template <int EPL, bool STOCHASTIC>   // EPL = tile_size / 64 elements per lane
__global__ __launch_bounds__(256) void momentum_1d_kernel(const void* __restrict__ grad, int grad_dtype,
                                                           const uint8_t* old_q, const float* old_scale, uint8_t* new_q,
                                                           float* new_scale, uint16_t* __restrict__ update, int64_t n,
                                                           int64_t first_block, int64_t blocks, float beta,
                                                           float inv_loss_scale, int nesterov, uint64_t step, uint64_t key) {
    constexpr int TILE = EPL * WAVE;
    const int64_t b = first_block + (int64_t)blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE;
    if (b >= blocks) return;
    const int lane = threadIdx.x % WAVE;
    const float scale_old = old_scale[b];
    const float one_minus = 1.0f - beta;
    float g[EPL], m[EPL];
    float amax = 0.0f;
#pragma unroll
    for (int j = 0; j < EPL; ++j) {
        const int64_t i = b * TILE + j * WAVE + lane;
        g[j] = 0.0f;
        float m0 = 0.0f;
        if (i < n) {
            g[j] = load_dtype(grad, i, grad_dtype) * inv_loss_scale;
            m0 = e4m3_to_f32(old_q[i]) * scale_old;
        }
        const float t0 = beta * m0;
        const float t1 = one_minus * g[j];
        m[j] = t0 + t1;
        amax = fmaxf(amax, fabsf(m[j]));
    }
    amax = wave_max(amax);
    const float scale = scale_of(amax, 448.0f);
    if (lane == 0) new_scale[b] = scale;
#pragma unroll
    for (int j = 0; j < EPL; ++j) {
        const int64_t i = b * TILE + j * WAVE + lane;
        new_q[i] = encode_state<STOCHASTIC>(m[j], scale, (uint64_t)i, step, key);
        if (i < n) {
            float u = m[j];
            if (nesterov) {
                const float t0 = one_minus * g[j];
                const float t1 = beta * m[j];
                u = t0 + t1;
            }
            update[i] = f32_to_bf16_bits(u);
        }
    }
}

// Same tile, same arithmetic, four consecutive elements per lane: 16-byte gradient loads, the four state codes as
// one word through the hardware decoder, 8-byte update stores. Needs the gradient aligned to four elements, the
// state to 4 bytes and the update to 8 bytes; only whole tiles inside n (the host sends a ragged last tile to the
// kernel above). The quotient m / scale takes the shared-divisor route when the tile allows it.
template <typename TG> __device__ __forceinline__ void load_quad(const TG* p, float (&v)[4]);
template <> __device__ __forceinline__ void load_quad<float>(const float* p, float (&v)[4]) {
    const float4 t = *reinterpret_cast<const float4*>(p);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
}
template <> __device__ __forceinline__ void load_quad<bf16_t>(const bf16_t* p, float (&v)[4]) {
    const uint2 t = *reinterpret_cast<const uint2*>(p);
    v[0] = __uint_as_float(t.x << 16); v[1] = __uint_as_float(t.x & 0xffff0000u);
    v[2] = __uint_as_float(t.y << 16); v[3] = __uint_as_float(t.y & 0xffff0000u);
}
template <> __device__ __forceinline__ void load_quad<f16_t>(const f16_t* p, float (&v)[4]) {
    typedef _Float16 h4 __attribute__((ext_vector_type(4)));
    const h4 t = *reinterpret_cast<const h4*>(p);
    v[0] = (float)t[0]; v[1] = (float)t[1]; v[2] = (float)t[2]; v[3] = (float)t[3];
}

template <typename TG, int EPL, bool STOCHASTIC>
__device__ __forceinline__ void momentum_quads_tile(const TG* __restrict__ grad, const uint8_t* old_q, const float* old_scale,
                                                    uint8_t* new_q, float* new_scale, uint16_t* __restrict__ update, int64_t b,
                                                    float beta, float inv_loss_scale, int nesterov, uint64_t step, uint64_t key) {
    constexpr int TILE = EPL * WAVE, QUADS = EPL / 4;
    const int lane = threadIdx.x % WAVE;
    const float scale_old = old_scale[b];
    const float one_minus = 1.0f - beta;
    float g[QUADS][4], m[QUADS][4];
    float amax = 0.0f, poison = 0.0f;
#pragma unroll
    for (int c = 0; c < QUADS; ++c) {
        const int64_t i = b * TILE + (c * WAVE + lane) * 4;
        load_quad<TG>(grad + i, g[c]);
        const int codes = *reinterpret_cast<const int*>(old_q + i);
        const float m0[4] = {__builtin_amdgcn_cvt_f32_fp8(codes, 0), __builtin_amdgcn_cvt_f32_fp8(codes, 1),
                             __builtin_amdgcn_cvt_f32_fp8(codes, 2), __builtin_amdgcn_cvt_f32_fp8(codes, 3)};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            g[c][e] = g[c][e] * inv_loss_scale;
            const float t0 = beta * (m0[e] * scale_old);
            const float t1 = one_minus * g[c][e];
            m[c][e] = t0 + t1;
            amax = fmaxf(amax, fabsf(m[c][e]));
            poison = poison_of(poison, m[c][e]);
        }
    }
    amax = wave_max(amax);
    const bool any_bad = __builtin_amdgcn_ballot_w64(poison != poison) != 0;
    const float scale = scale_of(amax, 448.0f);
    if (lane == 0) new_scale[b] = scale;
    const SharedDivisor divisor(scale, any_bad ? __uint_as_float(0x7fc00000u) : 0.0f);
#pragma unroll
    for (int c = 0; c < QUADS; ++c) {
        const int64_t i = b * TILE + (c * WAVE + lane) * 4;
        uint32_t word;
        if (divisor.fast) {
            float t[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                t[e] = __builtin_amdgcn_fmed3f(divisor.quotient(m[c][e]), -448.0f, 448.0f);
                if (STOCHASTIC) t[e] = stochastic_e4m3(t[e], (uint64_t)(i + e), step, key);
            }
            word = hw_encode4<e4m3_t>(t[0], t[1], t[2], t[3]);
        } else {
            word = 0;
#pragma unroll
            for (int e = 0; e < 4; ++e) word |= (uint32_t)encode_state<STOCHASTIC>(m[c][e], scale, (uint64_t)(i + e), step, key) << (8 * e);
        }
        *reinterpret_cast<uint32_t*>(new_q + i) = word;
        float u[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            u[e] = m[c][e];
            if (nesterov) {
                const float t0 = one_minus * g[c][e];
                const float t1 = beta * m[c][e];
                u[e] = t0 + t1;
            }
        }
        *reinterpret_cast<uint2*>(update + i) = make_uint2(f32_to_bf16x2_bits(u[0], u[1]), f32_to_bf16x2_bits(u[2], u[3]));
    }
}

template <typename TG, int EPL, bool STOCHASTIC>
__global__ __launch_bounds__(256) void momentum_1d_quads(const TG* __restrict__ grad, const uint8_t* old_q,
                                                          const float* old_scale, uint8_t* new_q, float* new_scale,
                                                          uint16_t* __restrict__ update, int64_t blocks, float beta,
                                                          float inv_loss_scale, int nesterov, uint64_t step, uint64_t key) {
    const int64_t b = (int64_t)blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE;
    if (b >= blocks) return;
    momentum_quads_tile<TG, EPL, STOCHASTIC>(grad, old_q, old_scale, new_q, new_scale, update, b, beta, inv_loss_scale, nesterov, step, key);
}

// Many tensors of `blocks` whole tiles each in one launch: row t of `table` holds {grad, old_q, old_scale, new_q,
// new_scale, update, rounding key, 0} as 64-bit words; blockIdx.y walks the tensors.
template <typename TG, int EPL, bool STOCHASTIC>
__global__ __launch_bounds__(256) void momentum_table_quads(const int64_t* __restrict__ table, int64_t blocks, float beta,
                                                             float inv_loss_scale, int nesterov, uint64_t step) {
    const int64_t b = (int64_t)blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE;
    if (b >= blocks) return;
    const int64_t* row = table + (int64_t)blockIdx.y * 8;
    momentum_quads_tile<TG, EPL, STOCHASTIC>(reinterpret_cast<const TG*>(row[0]), reinterpret_cast<const uint8_t*>(row[1]),
                                             reinterpret_cast<const float*>(row[2]), reinterpret_cast<uint8_t*>(row[3]),
                                             reinterpret_cast<float*>(row[4]), reinterpret_cast<uint16_t*>(row[5]), b, beta,
                                             inv_loss_scale, nesterov, step, (uint64_t)row[6]);
}

// ------------------------------------------------------------------ 2-D blocks: one wavefront per block
template <bool STOCHASTIC>
__global__ __launch_bounds__(256) void momentum_2d_kernel(const void* __restrict__ grad, int grad_dtype,
                                                           const uint8_t* old_q, const float* old_scale, uint8_t* new_q,
                                                           float* new_scale, uint16_t* __restrict__ update, int64_t planes,
                                                           int64_t rows, int64_t cols, int tr, int tc, float beta,
                                                           float inv_loss_scale, int nesterov, uint64_t step, uint64_t key) {
    const int64_t nr = (rows + tr - 1) / tr, nc = (cols + tc - 1) / tc;
    const int64_t tile = (int64_t)blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE;
    if (tile >= planes * nr * nc) return;
    const int lane = threadIdx.x % WAVE;
    const int64_t plane = tile / (nr * nc), br = tile / nc % nr, bc = tile % nc;
    const float scale_old = old_scale[tile];
    const float one_minus = 1.0f - beta;
    const int size = tr * tc;
    auto element = [&](int j, int64_t& i, float& g, float& m) -> bool {
        const int64_t y = br * tr + j / tc, x = bc * tc + j % tc;
        if (y >= rows || x >= cols) return false;
        i = (plane * rows + y) * cols + x;
        g = load_dtype(grad, i, grad_dtype) * inv_loss_scale;
        const float t0 = beta * (e4m3_to_f32(old_q[i]) * scale_old);
        const float t1 = one_minus * g;
        m = t0 + t1;
        return true;
    };
    float amax = 0.0f;
    for (int j = lane; j < size; j += WAVE) {
        int64_t i; float g, m;
        if (element(j, i, g, m)) amax = fmaxf(amax, fabsf(m));
    }
    amax = wave_max(amax);
    const float scale = scale_of(amax, 448.0f);
    for (int j = lane; j < size; j += WAVE) {
        int64_t i; float g, m;
        if (element(j, i, g, m)) {
            new_q[i] = encode_state<STOCHASTIC>(m, scale, (uint64_t)i, step, key);
            float u = m;
            if (nesterov) {
                const float t0 = one_minus * g;
                const float t1 = beta * m;
                u = t0 + t1;
            }
            update[i] = f32_to_bf16_bits(u);
        }
    }
    // every lane has finished reading old_scale[tile] (held in a register) before this store
    if (lane == 0) new_scale[tile] = scale;
}

// ------------------------------------------------------------------ elementwise updates
template <bool STOCHASTIC>
__global__ __launch_bounds__(256) void weight_kernel(void* weight, int weight_dtype, const void* __restrict__ grad,
                                                      int grad_dtype, int64_t n, float lr, float decay, float update_scale,
                                                      uint64_t step, uint64_t key, uint64_t offset) {
    const float keep = 1.0f - lr * decay;
    const float rate = lr * update_scale;
    for (int64_t j = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; j < n; j += (int64_t)gridDim.x * blockDim.x) {
        const float t0 = load_dtype(weight, j, weight_dtype) * keep;
        const float t1 = rate * load_dtype(grad, j, grad_dtype);
        store_rounded<STOCHASTIC>(weight, j, weight_dtype, t0 - t1, (uint64_t)j + offset, step, key);
    }
}

// fp32 weights, four per thread (16-byte accesses); same arithmetic as weight_kernel. quads = n / 4 whole quads, the
// host sends the last n % 4 elements through weight_kernel.
template <typename TG>
__global__ __launch_bounds__(256) void weight_quads_kernel(float* weight, const TG* __restrict__ grad, int64_t quads, float lr,
                                                            float decay, float update_scale) {
    const float keep = 1.0f - lr * decay;
    const float rate = lr * update_scale;
    for (int64_t j = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; j < quads; j += (int64_t)gridDim.x * blockDim.x) {
        float4 w = reinterpret_cast<const float4*>(weight)[j];
        float g[4];
        load_quad<TG>(grad + 4 * j, g);
        const float t0[4] = {w.x * keep, w.y * keep, w.z * keep, w.w * keep};
        const float t1[4] = {rate * g[0], rate * g[1], rate * g[2], rate * g[3]};
        reinterpret_cast<float4*>(weight)[j] = make_float4(t0[0] - t1[0], t0[1] - t1[1], t0[2] - t1[2], t0[3] - t1[3]);
    }
}

// Many fp32 tensors of `quads` whole quads each: row t of `table` holds {weight, update}; blockIdx.y walks the tensors.
template <typename TG>
__global__ __launch_bounds__(256) void weight_table_quads_kernel(const int64_t* __restrict__ table, int64_t quads, float lr,
                                                                  float decay, float update_scale) {
    const float keep = 1.0f - lr * decay;
    const float rate = lr * update_scale;
    float* weight = reinterpret_cast<float*>(table[(int64_t)blockIdx.y * 2]);
    const TG* grad = reinterpret_cast<const TG*>(table[(int64_t)blockIdx.y * 2 + 1]);
    for (int64_t j = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; j < quads; j += (int64_t)gridDim.x * blockDim.x) {
        float4 w = reinterpret_cast<const float4*>(weight)[j];
        float g[4];
        load_quad<TG>(grad + 4 * j, g);
        const float t0[4] = {w.x * keep, w.y * keep, w.z * keep, w.w * keep};
        const float t1[4] = {rate * g[0], rate * g[1], rate * g[2], rate * g[3]};
        reinterpret_cast<float4*>(weight)[j] = make_float4(t0[0] - t1[0], t0[1] - t1[1], t0[2] - t1[2], t0[3] - t1[3]);
    }
}

struct AdamConstants {
    float lr, decay, b1, b2, inv_c1, inv_c2, eps;
    int adamw, maximize;
};

template <bool STOCHASTIC>
__device__ __forceinline__ void adam_element(void* weight, int weight_dtype, const void* grad, int grad_dtype, void* first,
                                             void* second, int state_dtype, int64_t j, const AdamConstants& c, uint64_t step,
                                             uint64_t key, uint64_t offset) {
    const float one_b1 = 1.0f - c.b1, one_b2 = 1.0f - c.b2;
    const float keep = 1.0f - c.lr * c.decay;
    float w = load_dtype(weight, j, weight_dtype);
    float g = load_dtype(grad, j, grad_dtype);
    if (c.maximize) g = -g;
    if (!c.adamw) { const float t = c.decay * w; g = g + t; }
    const float m0 = c.b1 * load_dtype(first, j, state_dtype);
    const float m1 = one_b1 * g;
    const float m = m0 + m1;
    const float v0 = c.b2 * load_dtype(second, j, state_dtype);
    const float v1 = (one_b2 * g) * g;
    const float v = v0 + v1;
    store_rounded<false>(first, j, state_dtype, m, 0, 0, 0);
    store_rounded<false>(second, j, state_dtype, v, 0, 0, 0);
    if (c.adamw) w = w * keep;
    const float numerator = c.lr * (m * c.inv_c1);
    const float denominator = sqrtf(v * c.inv_c2) + c.eps;
    store_rounded<STOCHASTIC>(weight, j, weight_dtype, w - numerator / denominator, (uint64_t)j + offset, step, key);
}

template <bool STOCHASTIC>
__global__ __launch_bounds__(256) void adam_kernel(void* weight, int weight_dtype, const void* __restrict__ grad,
                                                    int grad_dtype, void* first, void* second, int state_dtype, int64_t n,
                                                    AdamConstants c, uint64_t step, uint64_t key, uint64_t offset) {
    for (int64_t j = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; j < n; j += (int64_t)gridDim.x * blockDim.x)
        adam_element<STOCHASTIC>(weight, weight_dtype, grad, grad_dtype, first, second, state_dtype, j, c, step, key, offset);
}

// Many small tensors in one launch: row t of `table` holds {weight, grad, first, second, count, key, offset} as
// 64-bit words; blockIdx.y walks the tensors, blockIdx.x their elements.
template <bool STOCHASTIC>
__global__ __launch_bounds__(256) void adam_table_kernel(const int64_t* __restrict__ table, int weight_dtype, int grad_dtype,
                                                          int state_dtype, AdamConstants c, uint64_t step) {
    const int64_t* row = table + (int64_t)blockIdx.y * 7;
    const int64_t n = row[4];
    void* weight = reinterpret_cast<void*>(row[0]);
    const void* grad = reinterpret_cast<const void*>(row[1]);
    void* first = reinterpret_cast<void*>(row[2]);
    void* second = reinterpret_cast<void*>(row[3]);
    for (int64_t j = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; j < n; j += (int64_t)gridDim.x * blockDim.x)
        adam_element<STOCHASTIC>(weight, weight_dtype, grad, grad_dtype, first, second, state_dtype, j, c, step, (uint64_t)row[5], (uint64_t)row[6]);
}

__global__ __launch_bounds__(256) void copy_scaled_kernel(const void* __restrict__ update, int update_dtype, void* out,
                                                           int out_dtype, int64_t src, int64_t dst, int64_t count,
                                                           float scale) {
    for (int64_t j = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; j < count; j += (int64_t)gridDim.x * blockDim.x)
        store_rounded<false>(out, dst + j, out_dtype, load_dtype(update, src + j, update_dtype) * scale, 0, 0, 0);
}

__global__ __launch_bounds__(256) void momentum_dequantize_kernel(const uint8_t* __restrict__ q, const float* __restrict__ scale,
                                                                   float* __restrict__ out, int64_t n, int granularity,
                                                                   int tile_size, int64_t rows, int64_t cols, int tr, int tc) {
    const int64_t nr = granularity ? (rows + tr - 1) / tr : 0, nc = granularity ? (cols + tc - 1) / tc : 0;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
        int64_t tile;
        if (granularity == 0) {
            tile = i / tile_size;
        } else {
            const int64_t plane = i / (rows * cols), y = i / cols % rows, x = i % cols;
            tile = (plane * nr + y / tr) * nc + x / tc;
        }
        out[i] = e4m3_to_f32(q[i]) * scale[tile];
    }
}

static unsigned grid_for(int64_t n) {
    const int64_t blocks = (n + 255) / 256;
    return (unsigned)(blocks < 1 ? 1 : blocks > 65536 * 8 ? 65536 * 8 : blocks);
}

}  // namespace viola

using namespace viola;

extern "C" int viola_momentum_update(const void* grad, int grad_dtype, const void* old_q, const float* old_scale,
                                     void* new_q, float* new_scale, void* update, int64_t n, float beta,
                                     float inv_loss_scale, int nesterov, int granularity, int tile_size, int64_t planes,
                                     int64_t rows, int64_t cols, int tr, int tc, int rounding, int64_t rounding_step,
                                     int64_t rounding_key, viola_stream_t stream_) {
    hipStream_t stream = viola_enter(stream_);
    VIOLA_CHECK_ARG(viola_is_float(grad_dtype) && n >= 0 && (granularity == 0 || granularity == 1));
    VIOLA_CHECK_ARG(rounding == VIOLA_NEAREST || rounding == VIOLA_STOCHASTIC);
    if (n == 0) return 0;
    VIOLA_CHECK_ARG(grad && old_q && old_scale && new_q && new_scale && update);
    const uint8_t* oq = static_cast<const uint8_t*>(old_q);
    uint8_t* nq = static_cast<uint8_t*>(new_q);
    uint16_t* up = static_cast<uint16_t*>(update);
    const uint64_t step = (uint64_t)rounding_step, key = (uint64_t)rounding_key;
    if (granularity == 0) {
        VIOLA_CHECK_ARG(tile_size == 64 || tile_size == 128 || tile_size == 256 || tile_size == 512 || tile_size == 1024);
        const int64_t blocks = (n + tile_size - 1) / tile_size;
        // whole tiles go four elements per lane when the pointers allow it; the ragged last tile (and everything,
        // for small tiles or odd alignment) one element per lane
        const int64_t whole = n / tile_size;
        const size_t grad_bytes = grad_dtype == VIOLA_F32 ? 4 : 2;
        const bool quads = tile_size >= 256 && whole > 0 && reinterpret_cast<uintptr_t>(grad) % (4 * grad_bytes) == 0 &&
                           reinterpret_cast<uintptr_t>(old_q) % 4 == 0 && reinterpret_cast<uintptr_t>(new_q) % 4 == 0 &&
                           reinterpret_cast<uintptr_t>(update) % 8 == 0;
        const int64_t first = quads ? whole : 0;
        if (quads) {
            const dim3 qgrid((unsigned)((whole + 3) / 4));
#define VIOLA_MQ(TG, EPL)                                                                                                   \
    if (rounding) VIOLA_LAUNCH((momentum_1d_quads<TG, EPL, true>), qgrid, dim3(256), 0, stream, static_cast<const TG*>(grad), oq, old_scale, nq, new_scale, up, whole, beta, inv_loss_scale, nesterov, step, key); \
    else VIOLA_LAUNCH((momentum_1d_quads<TG, EPL, false>), qgrid, dim3(256), 0, stream, static_cast<const TG*>(grad), oq, old_scale, nq, new_scale, up, whole, beta, inv_loss_scale, nesterov, step, key);
#define VIOLA_MQT(EPL)                                                          \
    if (grad_dtype == VIOLA_F32) { VIOLA_MQ(float, EPL) }                        \
    else if (grad_dtype == VIOLA_BF16) { VIOLA_MQ(bf16_t, EPL) }                 \
    else { VIOLA_MQ(f16_t, EPL) }
            if (tile_size == 256) { VIOLA_MQT(4) } else if (tile_size == 512) { VIOLA_MQT(8) } else { VIOLA_MQT(16) }
#undef VIOLA_MQT
#undef VIOLA_MQ
        }
        if (first < blocks) {
            const dim3 grid((unsigned)((blocks - first + 3) / 4));
#define VIOLA_M1(EPL)                                                                                                        \
    case EPL * 64:                                                                                                           \
        if (rounding) VIOLA_LAUNCH((momentum_1d_kernel<EPL, true>), grid, dim3(256), 0, stream, grad, grad_dtype, oq, old_scale, nq, new_scale, up, n, first, blocks, beta, inv_loss_scale, nesterov, step, key); \
        else VIOLA_LAUNCH((momentum_1d_kernel<EPL, false>), grid, dim3(256), 0, stream, grad, grad_dtype, oq, old_scale, nq, new_scale, up, n, first, blocks, beta, inv_loss_scale, nesterov, step, key); \
        break;
            switch (tile_size) { VIOLA_M1(1) VIOLA_M1(2) VIOLA_M1(4) VIOLA_M1(8) VIOLA_M1(16) }
#undef VIOLA_M1
        }
        return viola_launch_status();
    }
    VIOLA_CHECK_ARG(planes > 0 && rows > 0 && cols > 0 && planes * rows * cols == n && tr > 0 && tc > 0 && tr * tc <= 4096);
    const int64_t tiles = planes * ((rows + tr - 1) / tr) * ((cols + tc - 1) / tc);
    const dim3 grid((unsigned)((tiles + 3) / 4));
    if (rounding) VIOLA_LAUNCH((momentum_2d_kernel<true>), grid, dim3(256), 0, stream, grad, grad_dtype, oq, old_scale, nq, new_scale, up, planes, rows, cols, tr, tc, beta, inv_loss_scale, nesterov, step, key);
    else VIOLA_LAUNCH((momentum_2d_kernel<false>), grid, dim3(256), 0, stream, grad, grad_dtype, oq, old_scale, nq, new_scale, up, planes, rows, cols, tr, tc, beta, inv_loss_scale, nesterov, step, key);
    return viola_launch_status();
}

extern "C" int viola_momentum_update_table(const int64_t* table, int64_t tensors, int64_t tiles, int grad_dtype, int tile_size,
                                           float beta, float inv_loss_scale, int nesterov, int rounding, int64_t rounding_step,
                                           viola_stream_t stream_) {
    hipStream_t stream = viola_enter(stream_);
    VIOLA_CHECK_ARG(viola_is_float(grad_dtype) && tensors >= 0 && tensors <= 65535 && tiles >= 0 && (tiles + 3) / 4 < (1ll << 31));
    VIOLA_CHECK_ARG(tile_size == 256 || tile_size == 512 || tile_size == 1024);
    VIOLA_CHECK_ARG(rounding == VIOLA_NEAREST || rounding == VIOLA_STOCHASTIC);
    if (tensors == 0 || tiles == 0) return 0;
    VIOLA_CHECK_ARG(table);
    const dim3 grid((unsigned)((tiles + 3) / 4), (unsigned)tensors);
#define VIOLA_MT(TG, EPL)                                                                                                   \
    if (rounding) VIOLA_LAUNCH((momentum_table_quads<TG, EPL, true>), grid, dim3(256), 0, stream, table, tiles, beta, inv_loss_scale, nesterov, (uint64_t)rounding_step); \
    else VIOLA_LAUNCH((momentum_table_quads<TG, EPL, false>), grid, dim3(256), 0, stream, table, tiles, beta, inv_loss_scale, nesterov, (uint64_t)rounding_step);
#define VIOLA_MTT(EPL)                                                          \
    if (grad_dtype == VIOLA_F32) { VIOLA_MT(float, EPL) }                        \
    else if (grad_dtype == VIOLA_BF16) { VIOLA_MT(bf16_t, EPL) }                 \
    else { VIOLA_MT(f16_t, EPL) }
    if (tile_size == 256) { VIOLA_MTT(4) } else if (tile_size == 512) { VIOLA_MTT(8) } else { VIOLA_MTT(16) }
#undef VIOLA_MTT
#undef VIOLA_MT
    return viola_launch_status();
}

extern "C" int viola_weight_update_table(const int64_t* table, int64_t tensors, int64_t count, int grad_dtype, float lr,
                                         float decay, float update_scale, viola_stream_t stream_) {
    hipStream_t stream = viola_enter(stream_);
    VIOLA_CHECK_ARG(viola_is_float(grad_dtype) && tensors >= 0 && tensors <= 65535 && count >= 0 && count % 4 == 0);
    if (tensors == 0 || count == 0) return 0;
    VIOLA_CHECK_ARG(table);
    const int64_t quads = count / 4;
    const int64_t blocks = (quads + 255) / 256;
    const dim3 grid((unsigned)(blocks > 4096 ? 4096 : blocks), (unsigned)tensors);
    if (grad_dtype == VIOLA_F32) VIOLA_LAUNCH(weight_table_quads_kernel<float>, grid, dim3(256), 0, stream, table, quads, lr, decay, update_scale);
    else if (grad_dtype == VIOLA_BF16) VIOLA_LAUNCH(weight_table_quads_kernel<bf16_t>, grid, dim3(256), 0, stream, table, quads, lr, decay, update_scale);
    else VIOLA_LAUNCH(weight_table_quads_kernel<f16_t>, grid, dim3(256), 0, stream, table, quads, lr, decay, update_scale);
    return viola_launch_status();
}

extern "C" int viola_weight_update(void* weight, int weight_dtype, const void* grad, int grad_dtype, int64_t n, float lr,
                                   float decay, float update_scale, int rounding, int64_t rounding_step,
                                   int64_t rounding_key, int64_t offset, viola_stream_t stream_) {
    hipStream_t stream = viola_enter(stream_);
    VIOLA_CHECK_ARG(viola_is_float(weight_dtype) && viola_is_float(grad_dtype) && n >= 0);
    if (n == 0) return 0;
    VIOLA_CHECK_ARG(weight && grad);
    const size_t grad_bytes = grad_dtype == VIOLA_F32 ? 4 : 2;
    if (weight_dtype == VIOLA_F32 && n >= 4 && reinterpret_cast<uintptr_t>(weight) % 16 == 0 &&
        reinterpret_cast<uintptr_t>(grad) % (4 * grad_bytes) == 0) {
        const int64_t quads = n / 4, rest = n % 4;
        float* wp = static_cast<float*>(weight);
        if (grad_dtype == VIOLA_F32) VIOLA_LAUNCH(weight_quads_kernel<float>, dim3(grid_for(quads)), dim3(256), 0, stream, wp, static_cast<const float*>(grad), quads, lr, decay, update_scale);
        else if (grad_dtype == VIOLA_BF16) VIOLA_LAUNCH(weight_quads_kernel<bf16_t>, dim3(grid_for(quads)), dim3(256), 0, stream, wp, static_cast<const bf16_t*>(grad), quads, lr, decay, update_scale);
        else VIOLA_LAUNCH(weight_quads_kernel<f16_t>, dim3(grid_for(quads)), dim3(256), 0, stream, wp, static_cast<const f16_t*>(grad), quads, lr, decay, update_scale);
        if (rest)
            VIOLA_LAUNCH(weight_kernel<false>, dim3(1), dim3(256), 0, stream, wp + 4 * quads, weight_dtype,
                               static_cast<const uint8_t*>(grad) + 4 * quads * grad_bytes, grad_dtype, rest, lr, decay, update_scale, 0ull, 0ull, 0ull);
        return viola_launch_status();
    }
    if (rounding && weight_dtype != VIOLA_F32)
        VIOLA_LAUNCH(weight_kernel<true>, dim3(grid_for(n)), dim3(256), 0, stream, weight, weight_dtype, grad, grad_dtype, n, lr, decay, update_scale, (uint64_t)rounding_step, (uint64_t)rounding_key, (uint64_t)offset);
    else
        VIOLA_LAUNCH(weight_kernel<false>, dim3(grid_for(n)), dim3(256), 0, stream, weight, weight_dtype, grad, grad_dtype, n, lr, decay, update_scale, (uint64_t)rounding_step, (uint64_t)rounding_key, (uint64_t)offset);
    return viola_launch_status();
}

extern "C" int viola_adam_update(void* weight, int weight_dtype, const void* grad, int grad_dtype, void* first, void* second,
                                 int state_dtype, int64_t n, float lr, float decay, float b1, float b2, float inv_c1,
                                 float inv_c2, float eps, int rounding, int64_t rounding_step, int64_t rounding_key,
                                 int64_t offset, int adamw, int maximize, viola_stream_t stream_) {
    hipStream_t stream = viola_enter(stream_);
    VIOLA_CHECK_ARG(viola_is_float(weight_dtype) && viola_is_float(grad_dtype) && viola_is_float(state_dtype) && n >= 0);
    if (n == 0) return 0;
    VIOLA_CHECK_ARG(weight && grad && first && second);
    const AdamConstants c{lr, decay, b1, b2, inv_c1, inv_c2, eps, adamw, maximize};
    if (rounding && weight_dtype != VIOLA_F32)
        VIOLA_LAUNCH(adam_kernel<true>, dim3(grid_for(n)), dim3(256), 0, stream, weight, weight_dtype, grad, grad_dtype, first, second, state_dtype, n, c, (uint64_t)rounding_step, (uint64_t)rounding_key, (uint64_t)offset);
    else
        VIOLA_LAUNCH(adam_kernel<false>, dim3(grid_for(n)), dim3(256), 0, stream, weight, weight_dtype, grad, grad_dtype, first, second, state_dtype, n, c, (uint64_t)rounding_step, (uint64_t)rounding_key, (uint64_t)offset);
    return viola_launch_status();
}

extern "C" int viola_adam_update_table(const int64_t* table, int64_t tensors, int64_t max_count, int weight_dtype, int grad_dtype,
                                       int state_dtype, float lr, float decay, float b1, float b2, float inv_c1, float inv_c2,
                                       float eps, int rounding, int64_t rounding_step, int adamw, int maximize,
                                       viola_stream_t stream_) {
    hipStream_t stream = viola_enter(stream_);
    VIOLA_CHECK_ARG(viola_is_float(weight_dtype) && viola_is_float(grad_dtype) && viola_is_float(state_dtype));
    VIOLA_CHECK_ARG(tensors >= 0 && tensors <= 65535 && max_count >= 0);
    if (tensors == 0 || max_count == 0) return 0;
    VIOLA_CHECK_ARG(table);
    const AdamConstants c{lr, decay, b1, b2, inv_c1, inv_c2, eps, adamw, maximize};
    const int64_t blocks = (max_count + 255) / 256;
    const dim3 grid((unsigned)(blocks > 1024 ? 1024 : blocks), (unsigned)tensors);
    if (rounding && weight_dtype != VIOLA_F32)
        VIOLA_LAUNCH(adam_table_kernel<true>, grid, dim3(256), 0, stream, table, weight_dtype, grad_dtype, state_dtype, c, (uint64_t)rounding_step);
    else
        VIOLA_LAUNCH(adam_table_kernel<false>, grid, dim3(256), 0, stream, table, weight_dtype, grad_dtype, state_dtype, c, (uint64_t)rounding_step);
    return viola_launch_status();
}

extern "C" int viola_copy_scaled(const void* update, int update_dtype, void* out, int out_dtype, int64_t src, int64_t dst,
                                 int64_t count, float scale, viola_stream_t stream_) {
    hipStream_t stream = viola_enter(stream_);
    VIOLA_CHECK_ARG(viola_is_float(update_dtype) && viola_is_float(out_dtype) && src >= 0 && dst >= 0 && count >= 0);
    if (count == 0) return 0;
    VIOLA_CHECK_ARG(update && out);
    VIOLA_LAUNCH(copy_scaled_kernel, dim3(grid_for(count)), dim3(256), 0, stream, update, update_dtype, out, out_dtype, src, dst, count, scale);
    return viola_launch_status();
}

extern "C" int viola_momentum_dequantize(const void* q, const float* scale, float* out, int64_t n, int granularity,
                                         int tile_size, int64_t planes, int64_t rows, int64_t cols, int tr, int tc,
                                         viola_stream_t stream_) {
    hipStream_t stream = viola_enter(stream_);
    VIOLA_CHECK_ARG(n >= 0 && (granularity == 0 ? tile_size > 0 : (rows > 0 && cols > 0 && tr > 0 && tc > 0 && planes * rows * cols == n)));
    if (n == 0) return 0;
    VIOLA_CHECK_ARG(q && scale && out);
    VIOLA_LAUNCH(momentum_dequantize_kernel, dim3(grid_for(n)), dim3(256), 0, stream, static_cast<const uint8_t*>(q), scale, out, n, granularity, tile_size, rows, cols, tr, tc);
    return viola_launch_status();
}
