// Group-scaled FP8 quantization for gfx950: one coalesced HBM read pass per call, amax by
// wavefront/LDS reduction, IEEE fp32 division (built with -ffp-contract=off), RNE FP8 encode.
//
// Kernels
//   quantize_rowwise   gr == 1, not transposed: 8 elements per lane, amax over gc/8 lanes.
//   quantize_tile      gc == 32, gr == 1: 128 x 64 tile through LDS, emits the row-wise layout,
//                      the quantized transpose, or both from the one read.
//   quantize_block32   gr == gc == 32, not transposed (weights and their masters): 32 x 128 strip per wavefront.
//   quantize_generic   any (gr, gc), transposed or not, optional re-encode from codes+scales:
//                      one wavefront per group, two passes over the group (second hits cache).
//   dequantize, fp8 transpose, segmented transposed quantize for the variable-group path.
#include <type_traits>

#include "common.hpp"

namespace viola {

// ------------------------------------------------------------------ 8-element chunk loads
template <typename TIn> struct Chunk8;
template <> struct Chunk8<bf16_t> {
    static __device__ __forceinline__ void load(const bf16_t* p, float (&v)[8]) {
        const uint4 raw = *reinterpret_cast<const uint4*>(p);
        const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[2 * i] = __uint_as_float(w[i] << 16);
            v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
        }
    }
};
template <> struct Chunk8<f16_t> {
    static __device__ __forceinline__ void load(const f16_t* p, float (&v)[8]) {
        typedef _Float16 h8 __attribute__((ext_vector_type(8)));
        const h8 raw = *reinterpret_cast<const h8*>(p);
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = (float)raw[i];
    }
};
template <> struct Chunk8<float> {
    static __device__ __forceinline__ void load(const float* p, float (&v)[8]) {
        const float4 lo = *reinterpret_cast<const float4*>(p);
        const float4 hi = *reinterpret_cast<const float4*>(p + 4);
        v[0] = lo.x; v[1] = lo.y; v[2] = lo.z; v[3] = lo.w;
        v[4] = hi.x; v[5] = hi.y; v[6] = hi.z; v[7] = hi.w;
    }
};

template <typename TOut>
__device__ __forceinline__ uint2 encode8(const float (&v)[8], float s, float limit, const SharedDivisor& d) {
    if (d.fast) return make_uint2(fast_encode4<TOut>(d, limit, v[0], v[1], v[2], v[3]), fast_encode4<TOut>(d, limit, v[4], v[5], v[6], v[7]));
    uint32_t lo = 0, hi = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        lo |= (uint32_t)encode_clamped<TOut>(v[i], s, limit) << (8 * i);
        hi |= (uint32_t)encode_clamped<TOut>(v[4 + i], s, limit) << (8 * i);
    }
    return make_uint2(lo, hi);
}

// ------------------------------------------------------------------ row-wise (1, GC)
// Requires cols % 8 == 0, x aligned to 8 elements, q aligned to 8 bytes.
template <typename TIn, typename TOut, int GC>
__global__ __launch_bounds__(256) void quantize_rowwise(const TIn* __restrict__ x, uint8_t* __restrict__ q,
                                                         float* __restrict__ scale, int64_t rows, int64_t cols,
                                                         int64_t nc, float limit, int e8m0) {
    constexpr int LANES = GC / 8;                         // lanes that share one group
    const int64_t chunks_per_row = nc * LANES;
    const int64_t chunk = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t row = chunk / chunks_per_row;
    const int64_t c0 = (chunk % chunks_per_row) * 8;
    const bool valid = row < rows && c0 < cols;
    float v[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if (valid) Chunk8<TIn>::load(x + row * cols + c0, v);
    float amax = 0.0f, poison = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        amax = fmaxf(amax, fabsf(v[i]));
        poison = poison_of(poison, v[i]);
    }
    amax = group_max<LANES>(amax);
#pragma unroll
    for (int offset = LANES / 2; offset > 0; offset >>= 1) poison += __shfl_xor(poison, offset, WAVE);
    const float s = group_scale(amax, limit, e8m0);
    const SharedDivisor divisor(s, poison);
    if (valid) {
        *reinterpret_cast<uint2*>(q + row * cols + c0) = encode8<TOut>(v, s, limit, divisor);
        if ((threadIdx.x & (LANES - 1)) == 0) put_scale(scale, row * nc + c0 / GC, s, e8m0);
    }
}

// ------------------------------------------------------------------ 128 x 64 tile, gc = 32
// ROWWISE: q [rows, cols], scale [rows, ceil(cols/32)].
// TRANSPOSED: qt [cols, rows], scale_t [cols, ceil(rows/32)], 32-wide groups along rows.
// VEC: cols % 8 == 0 and x aligned to 8 elements (16-byte loads); otherwise scalar loads.
constexpr int TILE_R = 128, TILE_C = 64, TILE_LD = TILE_C + 1;

template <typename TIn, bool VEC>
__device__ __forceinline__ void load_tile(const TIn* __restrict__ x, float* tile, int64_t r0, int64_t c0,
                                          int64_t rows, int64_t cols) {
    if constexpr (VEC) {
#pragma unroll
        for (int it = 0; it < TILE_R * TILE_C / 8 / 256; ++it) {
            const int id = it * 256 + threadIdx.x;
            const int r = id / (TILE_C / 8), ch = id % (TILE_C / 8);
            float v[8] = {0, 0, 0, 0, 0, 0, 0, 0};
            if (r0 + r < rows && c0 + ch * 8 < cols) Chunk8<TIn>::load(x + (r0 + r) * cols + c0 + ch * 8, v);
#pragma unroll
            for (int i = 0; i < 8; ++i) tile[r * TILE_LD + ch * 8 + i] = v[i];
        }
    } else {
        for (int id = threadIdx.x; id < TILE_R * TILE_C; id += 256) {
            const int r = id / TILE_C, c = id % TILE_C;
            float v = 0.0f;
            if (r0 + r < rows && c0 + c < cols) v = to_f32(x[(r0 + r) * cols + c0 + c]);
            tile[r * TILE_LD + c] = v;
        }
    }
}

// Encode 32 values held by one lane into eight words of codes.
template <typename TOut>
__device__ __forceinline__ void encode_group32(const float (&v)[32], float s, float poison, float limit, uint32_t (&w)[8]) {
    const SharedDivisor divisor(s, poison);
    if (divisor.fast) {
#pragma unroll
        for (int i = 0; i < 8; ++i) w[i] = fast_encode4<TOut>(divisor, limit, v[4 * i], v[4 * i + 1], v[4 * i + 2], v[4 * i + 3]);
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            w[i] = 0;
#pragma unroll
            for (int j = 0; j < 4; ++j) w[i] |= (uint32_t)encode_clamped<TOut>(v[4 * i + j], s, limit) << (8 * j);
        }
    }
}

// Encode 32 values held by one lane and store them at dst (a run of `count` <= 32 valid bytes).
template <typename TOut>
__device__ __forceinline__ void store_group32(const float (&v)[32], float s, float poison, float limit, uint8_t* dst, int count,
                                              bool aligned16) {
    uint32_t w[8];
    encode_group32<TOut>(v, s, poison, limit, w);
    if (count == 32 && aligned16) {
        reinterpret_cast<uint4*>(dst)[0] = make_uint4(w[0], w[1], w[2], w[3]);
        reinterpret_cast<uint4*>(dst)[1] = make_uint4(w[4], w[5], w[6], w[7]);
    } else {
        for (int i = 0; i < count; ++i) dst[i] = (uint8_t)(w[i >> 2] >> (8 * (i & 3)));
    }
}

template <typename TIn, typename TOut, bool ROWWISE, bool TRANSPOSED, bool VEC>
__global__ __launch_bounds__(256) void quantize_tile(const TIn* __restrict__ x, uint8_t* __restrict__ q,
                                                      float* __restrict__ scale, uint8_t* __restrict__ qt,
                                                      float* __restrict__ scale_t, int64_t rows, int64_t cols,
                                                      float limit, float* __restrict__ column_partial, int e8m0) {
    __shared__ float tile[TILE_R * TILE_LD];
    const int64_t r0 = (int64_t)blockIdx.y * TILE_R, c0 = (int64_t)blockIdx.x * TILE_C;
    load_tile<TIn, VEC>(x, tile, r0, c0, rows, cols);
    __syncthreads();
    const int t = threadIdx.x;
    if constexpr (ROWWISE) {
        const int r = t % TILE_R, g = t / TILE_R;                       // 128 rows x 2 column groups
        const int64_t row = r0 + r, col = c0 + g * 32;
        if (row < rows && col < cols) {
            float v[32];
            float amax = 0.0f, poison = 0.0f;
#pragma unroll
            for (int i = 0; i < 32; ++i) {
                v[i] = tile[r * TILE_LD + g * 32 + i];
                amax = fmaxf(amax, fabsf(v[i]));
                poison = poison_of(poison, v[i]);
            }
            const float s = group_scale(amax, limit, e8m0);
            const int64_t nc = (cols + 31) / 32;
            put_scale(scale, row * nc + col / 32, s, e8m0);
            const int count = (int)(cols - col < 32 ? cols - col : 32);
            uint8_t* dst = q + row * cols + col;
            store_group32<TOut>(v, s, poison, limit, dst, count, (reinterpret_cast<uintptr_t>(dst) & 15) == 0);
        }
    }
    if constexpr (TRANSPOSED) {
        const int c = t % TILE_C, g = t / TILE_C;                       // 64 columns x 4 row groups
        const int64_t col = c0 + c, row = r0 + g * 32;
        if (col < cols && row < rows) {
            float v[32];
            float amax = 0.0f, poison = 0.0f;
#pragma unroll
            for (int i = 0; i < 32; ++i) {
                v[i] = tile[(g * 32 + i) * TILE_LD + c];
                amax = fmaxf(amax, fabsf(v[i]));
                poison = poison_of(poison, v[i]);
            }
            const float s = group_scale(amax, limit, e8m0);
            const int64_t nr = (rows + 31) / 32;
            put_scale(scale_t, col * nr + row / 32, s, e8m0);
            if (column_partial) {
                float sum = 0.0f;
#pragma unroll
                for (int i = 0; i < 32; ++i) sum += v[i];
                column_partial[(row / 32) * cols + col] = sum;
            }
            const int count = (int)(rows - row < 32 ? rows - row : 32);
            uint8_t* dst = qt + col * rows + row;
            store_group32<TOut>(v, s, poison, limit, dst, count, (reinterpret_cast<uintptr_t>(dst) & 15) == 0);
        }
    }
}

// ------------------------------------------------------------------ 16-bit inputs: both layouts per wavefront
// A wavefront owns 32 rows x 64 columns. Lane l loads 16 bytes (8 elements) of rows l/8 + 8i, quantizes them for
// the row-wise layout straight from registers (a 32-column group is four neighbouring lanes), and parks the raw
// 16 bytes in a wave-private LDS tile. ds_read_b64_tr_b16 then hands every lane the 32 rows of ONE column, four at
// a time, which is exactly a group of the transposed layout. The LDS tile holds 2-byte values (rows of 64 + 32
// elements: four consecutive rows start 64 bytes apart in bank space), so LDS moves 12 instructions per 32
// elements instead of one per element and layout. No block-level synchronisation.
template <typename TIn> __device__ __forceinline__ float widen16(uint32_t bits);
template <> __device__ __forceinline__ float widen16<bf16_t>(uint32_t bits) { return __uint_as_float(bits << 16); }
template <> __device__ __forceinline__ float widen16<f16_t>(uint32_t bits) {
    const uint16_t b = (uint16_t)bits;
    return (float)__builtin_bit_cast(_Float16, b);
}

template <typename TIn> __device__ __forceinline__ uint32_t narrow16(float v);
template <> __device__ __forceinline__ uint32_t narrow16<bf16_t>(float v) { return f32_to_bf16_bits(v); }
template <> __device__ __forceinline__ uint32_t narrow16<f16_t>(float v) { return __builtin_bit_cast(uint16_t, (_Float16)v); }

// GATED: x is [rows, 2 cols] = [gate | up] and the tile quantized is act(gate) * up [rows, cols]
// (viola/nn/_mlp_kernels.py:195-230 hands h over as codes; here from the stored projection instead of the accumulators).
template <typename TIn, typename TOut, bool ROWWISE, bool GATED = false>
__global__ __launch_bounds__(256) void quantize_dual16(const TIn* __restrict__ x, uint8_t* __restrict__ q,
                                                        float* __restrict__ scale, uint8_t* __restrict__ qt,
                                                        float* __restrict__ scale_t, int64_t rows, int64_t cols,
                                                        float limit, float* __restrict__ column_partial, int e8m0,
                                                        int activation = 0) {
    constexpr int LD = 64 + 32;
    typedef short s16x4 __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    __shared__ __attribute__((aligned(16))) uint16_t park[4][32 * LD];
    // Transposed codes leave as whole 128-byte lines: the block's four wavefronts hold rows 32 w .. 32 w + 31 of the same
    // 64 columns, so each has a 32-byte run of every column's line; the runs meet here ([column][128 + 16 bytes]) and
    // go out as 16-byte pieces, eight lanes to a line, instead of 64 lines touched per store instruction.
    constexpr int XLD = 128 + 16;
    __shared__ __attribute__((aligned(16))) uint8_t lines[64 * XLD];
    const bool by_lines = rows % 16 == 0 && (reinterpret_cast<uintptr_t>(qt) & 15) == 0;   // pieces are whole and aligned
    const int lane = threadIdx.x % WAVE, wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);   // uniform: so is the buffer descriptor
    uint16_t* mine = park[wave];
    const int lr = lane / 8, ch = lane % 8;
    const int64_t nc = (cols + 31) / 32;
    // a block walks tiles of 128 rows x 64 columns (column tiles fastest) with the grid's stride: the wavefronts stay
    // resident, so the SIMDs keep several of them in flight instead of waiting for new workgroups to be dispatched
    const int64_t tiles_x = (cols + 63) / 64, tiles_y = (rows + 127) / 128, tiles = tiles_x * tiles_y;
    for (int64_t tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
    // tiles in flight together (consecutive indices) should form a compact patch: 16 row tiles of one column tile, then
    // the next column tile, so that a row of x is read in long runs and a row of the transposed output (2 KB per 16
    // row tiles) is written in long runs too, however wide the matrix is
    constexpr int64_t BAND = 16;                                            // 8 .. 32 measure the same, 64 slower
    const int64_t patch = tile / (BAND * tiles_x), within = tile % (BAND * tiles_x);
    const int64_t tall = tiles_y - patch * BAND < BAND ? tiles_y - patch * BAND : BAND;
    const int64_t block_r0 = (patch * BAND + within % tall) * 128;
    const int64_t r0 = block_r0 + wave * 32, c0 = within / tall * 64;
    const bool active = r0 < rows;                                           // a wavefront past the last row reads zeros and stores nothing
    const int64_t col8 = c0 + ch * 8;

    // all four loads first, without control flow: a raw buffer over the wavefront's 32 rows returns zero past its end
    constexpr int WIDTH = GATED ? 2 : 1;                                     // x rows are [gate | up] when GATED
    const int64_t span = active ? (rows - r0 < 32 ? rows - r0 : 32) * cols * 2 * WIDTH : 0;
    const __amdgpu_buffer_rsrc_t res = __builtin_amdgcn_make_buffer_rsrc(const_cast<TIn*>(x + r0 * cols * WIDTH), 0, (int)span, 0x00020000);
    u32x4 raw[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
        raw[i] = __builtin_amdgcn_raw_buffer_load_b128(res, col8 < cols ? (int)(((lr + 8 * i) * cols * WIDTH + col8) * 2) : (int)0x80000000u, 0, 0);
    if constexpr (GATED) {
        // the tile quantized is h = act(gate) * up, rounded to TIn as the activation kernels store it
        u32x4 up[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
            up[i] = __builtin_amdgcn_raw_buffer_load_b128(res, col8 < cols ? (int)(((lr + 8 * i) * cols * 2 + cols + col8) * 2) : (int)0x80000000u, 0, 0);
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                uint32_t packed = 0;
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    const float g = widen16<TIn>(e ? raw[i][w] >> 16 : raw[i][w] & 0xffffu);
                    const float u = widen16<TIn>(e ? up[i][w] >> 16 : up[i][w] & 0xffffu);
                    float a, derivative;
                    gate_math(activation, g, a, derivative);
                    float hv = a * u;
                    // keep the product an FP32 value of its own: folded into the narrowing conversion (a mixed-precision
                    // FMA with a +0 addend) it rounds once instead of twice and turns -0 into +0
                    asm volatile("" : "+v"(hv));
                    packed |= narrow16<TIn>(hv) << (16 * e);
                }
                raw[i][w] = packed;
            }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) *reinterpret_cast<u32x4*>(&mine[(lr + 8 * i) * LD + ch * 8]) = raw[i];

    // row-wise groups: four lanes x 8 values
    float vr[4][8], s_row[4];
    bool fast = true;
    SharedDivisor d_row[4] = {SharedDivisor(1.0f, 0.0f), SharedDivisor(1.0f, 0.0f), SharedDivisor(1.0f, 0.0f), SharedDivisor(1.0f, 0.0f)};
    // The largest magnitude of a group is found on the raw 16-bit patterns, two to an instruction: with the sign bit
    // masked off, bf16 and fp16 order as unsigned integers like their values, and anything at or above the pattern of
    // infinity is an Inf or a NaN, which sends the wavefront down the exact path below (where the maximum is taken
    // again the way the reference's kernel takes it, ignoring NaN).
    constexpr uint32_t MAGNITUDE = 0x7fff7fffu, INF16 = sizeof(TIn) == 2 && std::is_same<TIn, bf16_t>::value ? 0x7f80u : 0x7c00u;
    auto top16 = [](uint32_t pairs) -> uint32_t { const uint32_t lo = pairs & 0xffffu, hi = pairs >> 16; return lo > hi ? lo : hi; };
    if constexpr (ROWWISE) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
#pragma unroll
            for (int e = 0; e < 8; ++e) vr[i][e] = widen16<TIn>(e % 2 ? raw[i][e / 2] >> 16 : raw[i][e / 2] & 0xffffu);
            uint32_t top = top16(pk_max_u16(pk_max_u16(raw[i][0] & MAGNITUDE, raw[i][1] & MAGNITUDE), pk_max_u16(raw[i][2] & MAGNITUDE, raw[i][3] & MAGNITUDE)));
            const uint32_t other = (uint32_t)__builtin_amdgcn_mov_dpp((int)top, 0x4E, 0xf, 0xf, true);      // lanes 2 3 0 1 of the quad
            top = top > other ? top : other;
            const uint32_t next = (uint32_t)__builtin_amdgcn_mov_dpp((int)top, 0xB1, 0xf, 0xf, true);       // lanes 1 0 3 2
            top = top > next ? top : next;
            s_row[i] = group_scale(widen16<TIn>(top), limit, e8m0);
            d_row[i] = SharedDivisor(s_row[i], top >= INF16 ? __uint_as_float(0x7fc00000u) : 0.0f);
            fast = fast && d_row[i].fast;
        }
    }
    // transposed groups: column lane % 16 of the 16-column strip lane / 16, rows 4t .. 4t+3 per read
    const int64_t col = c0 + lane;
    const int strip = (lane / 16) * 16, sub = lane & 15;
    const uint16_t* at = &mine[(sub >> 2) * LD + strip + 4 * (sub & 3)];
    float vc[32];
    uint32_t top_col = 0;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        const uint2 four = __builtin_bit_cast(uint2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(at + 4 * t * LD)));
        vc[4 * t] = widen16<TIn>(four.x & 0xffffu); vc[4 * t + 1] = widen16<TIn>(four.x >> 16);
        vc[4 * t + 2] = widen16<TIn>(four.y & 0xffffu); vc[4 * t + 3] = widen16<TIn>(four.y >> 16);
        top_col = pk_max_u16(top_col, pk_max_u16(four.x & MAGNITUDE, four.y & MAGNITUDE));
    }
    top_col = top16(top_col);
    float s_col = group_scale(widen16<TIn>(top_col), limit, e8m0);
    const SharedDivisor d_col(s_col, top_col >= INF16 ? __uint_as_float(0x7fc00000u) : 0.0f);
    fast = fast && d_col.fast;

    // one decision per wavefront: the common case runs without a single divergent branch
    uint2 row_codes[4];
    uint32_t col_codes[8];
    if (__builtin_amdgcn_ballot_w64(!fast) == 0 && limit == fp8_traits<TOut>::max) {
        // the scale is max |v| / (the format's largest value): no quotient can round past the largest code
        if constexpr (ROWWISE) {
#pragma unroll
            for (int i = 0; i < 4; ++i)
                row_codes[i] = make_uint2(fast_encode4_unclamped<TOut>(d_row[i], vr[i][0], vr[i][1], vr[i][2], vr[i][3]),
                                          fast_encode4_unclamped<TOut>(d_row[i], vr[i][4], vr[i][5], vr[i][6], vr[i][7]));
        }
#pragma unroll
        for (int k = 0; k < 8; ++k) col_codes[k] = fast_encode4_unclamped<TOut>(d_col, vc[4 * k], vc[4 * k + 1], vc[4 * k + 2], vc[4 * k + 3]);
    } else if (__builtin_amdgcn_ballot_w64(!fast) == 0) {
        if constexpr (ROWWISE) {
#pragma unroll
            for (int i = 0; i < 4; ++i)
                row_codes[i] = make_uint2(fast_encode4<TOut>(d_row[i], limit, vr[i][0], vr[i][1], vr[i][2], vr[i][3]),
                                          fast_encode4<TOut>(d_row[i], limit, vr[i][4], vr[i][5], vr[i][6], vr[i][7]));
        }
#pragma unroll
        for (int k = 0; k < 8; ++k) col_codes[k] = fast_encode4<TOut>(d_col, limit, vc[4 * k], vc[4 * k + 1], vc[4 * k + 2], vc[4 * k + 3]);
    } else {
        // some group of the wavefront holds an Inf or a NaN, or a scale outside the quotient route's domain: the maxima
        // again as the reference's kernel takes them (fmax ignores NaN), true division, software encoder
        const SharedDivisor exact(1.0f, __uint_as_float(0x7fc00000u));
        if constexpr (ROWWISE) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float amax = 0.0f;
#pragma unroll
                for (int e = 0; e < 8; ++e) amax = fmaxf(amax, fabsf(vr[i][e]));
                s_row[i] = group_scale(group_max<4>(amax), limit, e8m0);
                row_codes[i] = encode8<TOut>(vr[i], s_row[i], limit, exact);
            }
        }
        float amax = 0.0f;
#pragma unroll
        for (int i = 0; i < 32; ++i) amax = fmaxf(amax, fabsf(vc[i]));
        s_col = group_scale(amax, limit, e8m0);
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            col_codes[k] = 0;
#pragma unroll
            for (int e = 0; e < 4; ++e) col_codes[k] |= (uint32_t)encode_clamped<TOut>(vc[4 * k + e], s_col, limit) << (8 * e);
        }
    }

    if constexpr (ROWWISE) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int64_t row = r0 + lr + 8 * i;
            if (row < rows && col8 < cols) {
                *reinterpret_cast<uint2*>(q + row * cols + col8) = row_codes[i];
                if (ch % 4 == 0) put_scale(scale, row * nc + col8 / 32, s_row[i], e8m0);
            }
        }
    }
    if (active && col < cols) {
        const int64_t nr = (rows + 31) / 32;
        put_scale(scale_t, col * nr + r0 / 32, s_col, e8m0);
        if (column_partial) {
            float sum = 0.0f;
#pragma unroll
            for (int i = 0; i < 32; ++i) sum += vc[i];
            column_partial[(r0 / 32) * cols + col] = sum;
        }
        uint8_t* dst = qt + col * rows + r0;
        if (by_lines) {
            // stored below, by the whole block
        } else if (rows - r0 >= 32 && (reinterpret_cast<uintptr_t>(dst) & 15) == 0) {
            reinterpret_cast<uint4*>(dst)[0] = make_uint4(col_codes[0], col_codes[1], col_codes[2], col_codes[3]);
            reinterpret_cast<uint4*>(dst)[1] = make_uint4(col_codes[4], col_codes[5], col_codes[6], col_codes[7]);
        } else {
            const int count = (int)(rows - r0 < 32 ? rows - r0 : 32);
            for (int i = 0; i < count; ++i) dst[i] = (uint8_t)(col_codes[i >> 2] >> (8 * (i & 3)));
        }
    }
    if (by_lines) {
        __syncthreads();                                                     // the pieces of the tile before have been read
        if (active) {
            uint4* run = reinterpret_cast<uint4*>(&lines[lane * XLD + wave * 32]);
            run[0] = make_uint4(col_codes[0], col_codes[1], col_codes[2], col_codes[3]);
            run[1] = make_uint4(col_codes[4], col_codes[5], col_codes[6], col_codes[7]);
        }
        __syncthreads();
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            const int id = it * 256 + (int)threadIdx.x, c = id >> 3, piece = id & 7;
            const int64_t row = block_r0 + piece * 16;                       // rows % 16 == 0: a piece is inside or outside as a whole
            if (c0 + c < cols && row < rows)
                *reinterpret_cast<uint4*>(qt + (c0 + c) * rows + row) = *reinterpret_cast<const uint4*>(&lines[c * XLD + piece * 16]);
        }
    }
    }
}

// ------------------------------------------------------------------ 16-bit inputs: both layouts from a 64 x 64 tile
// A block of 256 threads per tile, one tile per block: eight blocks are resident on a compute unit at 64 registers, and
// the launch is timed 15 - 25 % below the persistent 128 x 64 kernel above on every shape tried (8192 x 4096 bf16:
// 27.7 against 36.2 us). Row-wise: thread (row tid / 4, 16 columns) loads 32 bytes, a 32-column group is a pair of
// lanes; four neighbouring lanes store 64 consecutive bytes of codes. The raw 16-bit values are parked in LDS
// ([row][64 + 4 values], the four 16-column blocks of a row permuted by row / 16 so that the transposed phase's four
// row chunks read distinct banks). After one barrier wavefront w takes columns 16 w .. + 15: lane (column lane / 4,
// rows 16 (lane % 4) .. + 15) reads its 16 values, a 32-row group is again a pair of lanes, and four neighbouring lanes
// store 64 consecutive bytes of one transposed row (with the group's halves 32 lanes apart instead, the same stores
// left as 16-byte pieces and the launch took 31 us).
// INTERIOR: the tile lies wholly inside the matrix and every 16-byte piece of either output is aligned (the launcher
// says so in `aligned`): no bounds checks, tile base pointers in scalar registers with 32-bit offsets per lane.

// 16 values as 8 words of two (rows or columns) -> group scale with the pair's other lane, codes; `slow` receives
// whether the wavefront must take the exact route instead.
template <typename TIn, typename TOut>
__device__ __forceinline__ bool encode_words16(const uint32_t (&words)[8], float limit, int e8m0, bool clamp_free, float& s, uint32_t (&codes)[4],
                                               bool& nonfinite) {
    constexpr uint32_t MAGNITUDE = 0x7fff7fffu, INF16 = std::is_same<TIn, bf16_t>::value ? 0x7f80u : 0x7c00u;
    uint32_t top = 0;
#pragma unroll
    for (int e = 0; e < 8; ++e) top = pk_max_u16(top, words[e] & MAGNITUDE);
    top = (top & 0xffffu) > (top >> 16) ? (top & 0xffffu) : (top >> 16);
    {
        const uint32_t other = (uint32_t)__builtin_amdgcn_mov_dpp((int)top, 0xB1, 0xf, 0xf, true);   // the pair's other lane
        top = top > other ? top : other;
    }
    nonfinite = top >= INF16;
    s = group_scale(widen16<TIn>(top), limit, e8m0);
    const SharedDivisor d(s, nonfinite ? __uint_as_float(0x7fc00000u) : 0.0f);
    if (__builtin_amdgcn_ballot_w64(!d.fast) != 0) return false;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const float a = widen16<TIn>(words[2 * k] & 0xffffu), b = widen16<TIn>(words[2 * k] >> 16);
        const float c = widen16<TIn>(words[2 * k + 1] & 0xffffu), e = widen16<TIn>(words[2 * k + 1] >> 16);
        codes[k] = clamp_free ? fast_encode4_unclamped<TOut>(d, a, b, c, e) : fast_encode4<TOut>(d, limit, a, b, c, e);
    }
    return true;
}
// The same for 16 finite values already widened: the maximum is taken in floating point, three values per instruction.
__device__ __forceinline__ float max3_abs(float acc, float a, float b) {
    float r;
    asm("v_max3_f32 %0, %1, |%2|, |%3|" : "=v"(r) : "v"(acc), "v"(a), "v"(b));
    return r;
}
template <typename TOut>
__device__ __forceinline__ bool encode_finite16(const float (&v)[16], float limit, int e8m0, bool clamp_free, float& s, uint32_t (&codes)[4]) {
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; i += 2) amax = max3_abs(amax, v[i], v[i + 1]);
    {
        const float other = __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(amax), 0xB1, 0xf, 0xf, true));   // the pair's other lane
        amax = max3_abs(amax, other, other);
    }
    s = group_scale(amax, limit, e8m0);
    const SharedDivisor d(s, 0.0f);
    if (__builtin_amdgcn_ballot_w64(!d.fast) != 0) return false;
#pragma unroll
    for (int k = 0; k < 4; ++k)
        codes[k] = clamp_free ? fast_encode4_unclamped<TOut>(d, v[4 * k], v[4 * k + 1], v[4 * k + 2], v[4 * k + 3])
                              : fast_encode4<TOut>(d, limit, v[4 * k], v[4 * k + 1], v[4 * k + 2], v[4 * k + 3]);
    return true;
}
// The exact route: an Inf or a NaN in some group of the wavefront, or a scale outside the quotient route's domain. The
// maximum as the reference's kernel takes it (fmax ignores NaN), true division, software encoder.
struct Exact16 { uint32_t c0, c1, c2, c3; float s; };
template <typename TIn, typename TOut>
__device__ __noinline__ Exact16 encode_words16_exact(uint32_t w0, uint32_t w1, uint32_t w2, uint32_t w3, uint32_t w4, uint32_t w5, uint32_t w6,
                                                     uint32_t w7, float limit, int e8m0) {
    const uint32_t words[8] = {w0, w1, w2, w3, w4, w5, w6, w7};
    float v[16], amax = 0.0f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        v[2 * e] = widen16<TIn>(words[e] & 0xffffu);
        v[2 * e + 1] = widen16<TIn>(words[e] >> 16);
        amax = fmaxf(amax, fmaxf(fabsf(v[2 * e]), fabsf(v[2 * e + 1])));
    }
    amax = fmaxf(amax, quad_xor<1>(amax));
    Exact16 out;
    out.s = group_scale(amax, limit, e8m0);
    uint32_t codes[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        codes[k] = 0;
#pragma unroll
        for (int e = 0; e < 4; ++e) codes[k] |= (uint32_t)encode_clamped<TOut>(v[4 * k + e], out.s, limit) << (8 * e);
    }
    out.c0 = codes[0]; out.c1 = codes[1]; out.c2 = codes[2]; out.c3 = codes[3];
    return out;
}

template <typename TIn, typename TOut, bool INTERIOR>
__device__ __forceinline__ void dual16_tile64(const TIn* __restrict__ x, uint8_t* __restrict__ q, float* __restrict__ scale,
                                              uint8_t* __restrict__ qt, float* __restrict__ scale_t, int64_t rows, int64_t cols,
                                              float limit, float* __restrict__ column_partial, int e8m0, int64_t r0, int64_t c0,
                                              uint16_t* park, int* flags) {
    constexpr int LDV = 64 + 4;                                              // values per parked row (34 dwords)
    const int tid = threadIdx.x, lane = tid % WAVE, wave = tid / WAVE;
    const int64_t nc = (cols + 31) / 32, nr = (rows + 31) / 32;
    const bool clamp_free = limit == fp8_traits<TOut>::max;

    // ---- row-wise
    {
        const int lr = tid / 4, lc = (tid % 4) * 16;
        const int64_t row = r0 + lr, col = c0 + lc;
        const uint32_t offset = (uint32_t)lr * (uint32_t)cols + (uint32_t)lc;   // from the tile's first element (INTERIOR: < 2^31)
        uint4 raw[2] = {make_uint4(0, 0, 0, 0), make_uint4(0, 0, 0, 0)};
        if constexpr (INTERIOR) {
            const TIn* tile = x + r0 * cols + c0;
            raw[0] = *reinterpret_cast<const uint4*>(tile + offset);
            raw[1] = *reinterpret_cast<const uint4*>(tile + offset + 8);
        } else if (row < rows) {
            if (col < cols) raw[0] = *reinterpret_cast<const uint4*>(x + row * cols + col);      // cols % 8 == 0: whole pieces
            if (col + 8 < cols) raw[1] = *reinterpret_cast<const uint4*>(x + row * cols + col + 8);
        }
        {
            uint2* mine = reinterpret_cast<uint2*>(&park[lr * LDV + (lc ^ (((lr >> 4) & 3) << 4))]);   // 16-column blocks swapped by row chunk
            mine[0] = make_uint2(raw[0].x, raw[0].y); mine[1] = make_uint2(raw[0].z, raw[0].w);
            mine[2] = make_uint2(raw[1].x, raw[1].y); mine[3] = make_uint2(raw[1].z, raw[1].w);
        }
        const uint32_t words[8] = {raw[0].x, raw[0].y, raw[0].z, raw[0].w, raw[1].x, raw[1].y, raw[1].z, raw[1].w};
        float s_row;
        uint32_t codes[4];
        bool nonfinite;
        if (!encode_words16<TIn, TOut>(words, limit, e8m0, clamp_free, s_row, codes, nonfinite)) {
            const Exact16 r = encode_words16_exact<TIn, TOut>(words[0], words[1], words[2], words[3], words[4], words[5], words[6], words[7], limit, e8m0);
            codes[0] = r.c0; codes[1] = r.c1; codes[2] = r.c2; codes[3] = r.c3; s_row = r.s;
        }
        if constexpr (INTERIOR) {
            *reinterpret_cast<uint4*>(q + r0 * cols + c0 + offset) = make_uint4(codes[0], codes[1], codes[2], codes[3]);
            if (tid % 2 == 0) put_scale(scale, (r0 * nc + c0 / 32) + (int64_t)((uint32_t)lr * (uint32_t)nc + (uint32_t)(lc / 32)), s_row, e8m0);
        } else if (row < rows && col < cols) {
            uint8_t* dst = q + row * cols + col;
            if (col + 16 <= cols && (reinterpret_cast<uintptr_t>(dst) & 15) == 0) {
                *reinterpret_cast<uint4*>(dst) = make_uint4(codes[0], codes[1], codes[2], codes[3]);
            } else {
                *reinterpret_cast<uint2*>(dst) = make_uint2(codes[0], codes[1]);                     // q is 8-byte aligned, cols % 8 == 0
                if (col + 8 < cols) *reinterpret_cast<uint2*>(dst + 8) = make_uint2(codes[2], codes[3]);
            }
            if (tid % 2 == 0) put_scale(scale, row * nc + col / 32, s_row, e8m0);
        }
        const bool any_nonfinite = __builtin_amdgcn_ballot_w64(nonfinite) != 0;   // over the whole wavefront: outside the branch
        if (lane == 0) flags[wave] = any_nonfinite;
    }
    __syncthreads();
    // no NaN and no Inf anywhere in the tile: the transposed phase may then take its maxima in floating point
    const bool plain = (flags[0] | flags[1] | flags[2] | flags[3]) == 0;

    // ---- transposed: wavefront w takes columns 16 w .. + 15 of the tile; lane = (column lane / 4, rows 16 (lane % 4) .. + 15), so four
    // neighbouring lanes write 64 consecutive bytes of one transposed row and a 32-row group is a pair of lanes
    {
        const int tc = wave * 16 + lane / 4, chunk = lane % 4;
        const int64_t tcol = c0 + tc, trow = r0 + chunk * 16;                // first of the lane's 16 rows
        uint32_t bits[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) bits[i] = park[(chunk * 16 + i) * LDV + (tc ^ (chunk << 4))];
        float w[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) w[i] = widen16<TIn>(bits[i]);
        float s_col;
        uint32_t tcodes[4];
        if (!plain || !encode_finite16<TOut>(w, limit, e8m0, clamp_free, s_col, tcodes)) {
            const Exact16 r = encode_words16_exact<TIn, TOut>(bits[0] | bits[1] << 16, bits[2] | bits[3] << 16, bits[4] | bits[5] << 16, bits[6] | bits[7] << 16,
                                                              bits[8] | bits[9] << 16, bits[10] | bits[11] << 16, bits[12] | bits[13] << 16,
                                                              bits[14] | bits[15] << 16, limit, e8m0);
            tcodes[0] = r.c0; tcodes[1] = r.c1; tcodes[2] = r.c2; tcodes[3] = r.c3; s_col = r.s;
        }
        float sum = 0.0f;
        if (column_partial) {
#pragma unroll
            for (int i = 0; i < 16; ++i) sum += w[i];
            const float other = quad_xor<1>(sum);
            sum = chunk % 2 == 0 ? sum + other : other + sum;                 // rows 0 .. 15 first, then 16 .. 31
        }
        if constexpr (INTERIOR) {
            *reinterpret_cast<uint4*>(qt + c0 * rows + r0 + ((uint32_t)tc * (uint32_t)rows + (uint32_t)(chunk * 16))) = make_uint4(tcodes[0], tcodes[1], tcodes[2], tcodes[3]);
            if (chunk % 2 == 0) {
                put_scale(scale_t, (c0 * nr + r0 / 32) + (int64_t)((uint32_t)tc * (uint32_t)nr + (uint32_t)(chunk / 2)), s_col, e8m0);
                if (column_partial) (column_partial + (r0 / 32) * cols + c0)[(uint32_t)(chunk / 2) * (uint32_t)cols + (uint32_t)tc] = sum;
            }
        } else if (tcol < cols && trow < rows) {
            uint8_t* dst = qt + tcol * rows + trow;
            if (trow + 16 <= rows && (reinterpret_cast<uintptr_t>(dst) & 15) == 0) {
                *reinterpret_cast<uint4*>(dst) = make_uint4(tcodes[0], tcodes[1], tcodes[2], tcodes[3]);
            } else {
                const int count = (int)(rows - trow < 16 ? rows - trow : 16);
                for (int i = 0; i < count; ++i) dst[i] = (uint8_t)(tcodes[i >> 2] >> (8 * (i & 3)));
            }
            if (chunk % 2 == 0) {
                put_scale(scale_t, tcol * nr + trow / 32, s_col, e8m0);
                if (column_partial) column_partial[(trow / 32) * cols + tcol] = sum;
            }
        }
    }
}

template <typename TIn, typename TOut>
__global__ __launch_bounds__(256, 8) void quantize_dual16_tile64(const TIn* __restrict__ x, uint8_t* __restrict__ q,
                                                               float* __restrict__ scale, uint8_t* __restrict__ qt,
                                                               float* __restrict__ scale_t, int64_t rows, int64_t cols,
                                                               float limit, float* __restrict__ column_partial, int e8m0, int xcd_walk,
                                                               int aligned) {
    __shared__ __attribute__((aligned(16))) uint16_t park[64 * (64 + 4)];
    __shared__ __attribute__((aligned(16))) int flags[4];                   // per wavefront: its rows hold a NaN or an Inf
    // blocks are dispatched in index order: those in flight together take 32 row tiles of one column tile, then the next
    // column tile, so the transposed output is written in 2 KB runs per row however wide the matrix is (the launcher
    // keeps the tile count below 2^31)
    constexpr uint32_t BAND = 32;
    const uint32_t tiles_x = (uint32_t)((cols + 63) / 64), tiles_y = (uint32_t)((rows + 63) / 64), tiles = tiles_x * tiles_y;
    uint32_t id = blockIdx.x;
    if (xcd_walk) {
        // consecutive block indices go to the eight XCDs in turn: give each XCD one contiguous eighth of the walk, so the
        // halves of a 128-byte line of the transposed output (two row tiles) meet in one L2
        id = (id % 8) * ((tiles + 7) / 8) + id / 8;
    }
    if (id >= tiles) return;
    const uint32_t patch = id / (BAND * tiles_x), within = id % (BAND * tiles_x);
    const uint32_t tall = tiles_y - patch * BAND < BAND ? tiles_y - patch * BAND : BAND;
    const int64_t r0 = (int64_t)(patch * BAND + within % tall) * 64, c0 = (int64_t)(within / tall) * 64;
    if (aligned && r0 + 64 <= rows && c0 + 64 <= cols) dual16_tile64<TIn, TOut, true>(x, q, scale, qt, scale_t, rows, cols, limit, column_partial, e8m0, r0, c0, park, flags);
    else dual16_tile64<TIn, TOut, false>(x, q, scale, qt, scale_t, rows, cols, limit, column_partial, e8m0, r0, c0, park, flags);
}

// ------------------------------------------------------------------ column sums from 32-row partials
// out[c] = sum over p of partial[p][c] in a fixed order: 8 threads per column each add a contiguous eighth of the
// parts in ascending order (loads issued 32 or eight at a time), then the eighths are added in order.
template <typename TO>
__global__ __launch_bounds__(256) void column_reduce_kernel(const float* __restrict__ partial, int64_t parts, int64_t cols,
                                                             TO* __restrict__ out) {
    __shared__ float piece[8][32];
    const int c = threadIdx.x % 32, slice = threadIdx.x / 32;
    const int64_t col = (int64_t)blockIdx.x * 32 + c;
    const int64_t per = (parts + 7) / 8;
    const int64_t begin = slice * per, end = begin + per < parts ? begin + per : parts;
    float sum = 0.0f;
    if (col < cols) {
        int64_t part = begin;
        for (; part + 32 <= end; part += 32) {                              // same order of additions, four times the loads in flight
            float v[32];
#pragma unroll
            for (int u = 0; u < 32; ++u) v[u] = partial[(part + u) * cols + col];
#pragma unroll
            for (int u = 0; u < 32; ++u) sum += v[u];
        }
        for (; part + 8 <= end; part += 8) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = partial[(part + u) * cols + col];
#pragma unroll
            for (int u = 0; u < 8; ++u) sum += v[u];
        }
        for (; part < end; ++part) sum += partial[part * cols + col];
    }
    piece[slice][c] = sum;
    __syncthreads();
    if (slice == 0 && col < cols) {
        float total = piece[0][c];
#pragma unroll
        for (int u = 1; u < 8; ++u) total += piece[u][c];
        out[col] = from_f32<TO>(total);
    }
}

// ------------------------------------------------------------------ (32, 32) blocks, not transposed
template <typename TIn> __device__ __forceinline__ void load4(const TIn* p, float (&v)[4]);
template <> __device__ __forceinline__ void load4<float>(const float* p, float (&v)[4]) {
    const float4 t = *reinterpret_cast<const float4*>(p);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
}
template <> __device__ __forceinline__ void load4<bf16_t>(const bf16_t* p, float (&v)[4]) {
    const uint2 t = *reinterpret_cast<const uint2*>(p);
    v[0] = __uint_as_float(t.x << 16); v[1] = __uint_as_float(t.x & 0xffff0000u);
    v[2] = __uint_as_float(t.y << 16); v[3] = __uint_as_float(t.y & 0xffff0000u);
}
template <> __device__ __forceinline__ void load4<f16_t>(const f16_t* p, float (&v)[4]) {
    typedef _Float16 h4 __attribute__((ext_vector_type(4)));
    const h4 t = *reinterpret_cast<const h4*>(p);
    v[0] = (float)t[0]; v[1] = (float)t[1]; v[2] = (float)t[2]; v[3] = (float)t[3];
}

// The weight recipe (a master matrix re-quantized after every optimizer step). A wavefront owns 32 rows x 128
// columns = four blocks: load i of 16 takes rows 2i, 2i+1, a lane four consecutive columns, so every load and every
// store instruction covers whole 512-byte (128-byte for the codes) row pieces; a block is the 8 lanes of a column
// group in both half-waves, over the 16 loads. One read of x; cols must be a multiple of 4.
template <typename TIn, typename TOut>
__global__ __launch_bounds__(256) void quantize_block32(const TIn* __restrict__ x, uint8_t* __restrict__ q, float* __restrict__ scale,
                                                         int64_t rows, int64_t cols, int64_t nc, float limit, int e8m0) {
    const int64_t strips = (cols + 127) / 128;
    const int64_t unit = (int64_t)blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE;
    if (unit >= (rows + 31) / 32 * strips) return;                      // whole wavefront leaves together
    const int lane = threadIdx.x % WAVE;
    const int64_t r0 = unit / strips * 32 + lane / 32, col = unit % strips * 128 + (lane % 32) * 4;
    float v[16][4];
    float amax = 0.0f, poison = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int64_t row = r0 + 2 * i;
        if (row < rows && col < cols) load4<TIn>(x + row * cols + col, v[i]);
        else v[i][0] = v[i][1] = v[i][2] = v[i][3] = 0.0f;
    }
#pragma unroll
    for (int i = 0; i < 16; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            amax = fmaxf(amax, fabsf(v[i][e]));
            poison = poison_of(poison, v[i][e]);
        }
    amax = group_max<8>(amax);
    amax = fmaxf(amax, __shfl_xor(amax, 32, WAVE));
    const bool any_bad = __builtin_amdgcn_ballot_w64(poison != poison) != 0;
    const float s = group_scale(amax, limit, e8m0);
    if ((lane & 39) == 0 && col < cols) put_scale(scale, (r0 / 32) * nc + col / 32, s, e8m0);
    const SharedDivisor d(s, any_bad ? __uint_as_float(0x7fc00000u) : 0.0f);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int64_t row = r0 + 2 * i;
        uint32_t word;
        if (d.fast) {
            word = fast_encode4<TOut>(d, limit, v[i][0], v[i][1], v[i][2], v[i][3]);
        } else {
            word = 0;
#pragma unroll
            for (int e = 0; e < 4; ++e) word |= (uint32_t)encode_clamped<TOut>(v[i][e], s, limit) << (8 * e);
        }
        if (row < rows && col < cols) *reinterpret_cast<uint32_t*>(q + row * cols + col) = word;
    }
}

// ------------------------------------------------------------------ generic: one wavefront per group
template <typename TIn, typename TOut, bool ENCODED>
__global__ __launch_bounds__(256) void quantize_generic(const TIn* __restrict__ x, const float* __restrict__ source_scale,
                                                         uint8_t* __restrict__ q, float* __restrict__ scale,
                                                         int64_t rows, int64_t cols, int gr, int gc, int transposed,
                                                         int source_gr, int source_gc, float limit, int e8m0) {
    const int64_t out_rows = transposed ? cols : rows, out_cols = transposed ? rows : cols;
    const int64_t nr = (out_rows + gr - 1) / gr, nc = (out_cols + gc - 1) / gc;
    const int64_t group = (int64_t)blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE;
    if (group >= nr * nc) return;                                       // whole wavefront leaves together
    const int lane = threadIdx.x % WAVE;
    const int64_t gr0 = group / nc * gr, gc0 = group % nc * gc;
    const int64_t sc = ENCODED ? (cols + source_gc - 1) / source_gc : 0;
    const int size = gr * gc;
    auto value = [&](int j, bool& inside) -> float {
        const int64_t r = gr0 + j / gc, c = gc0 + j % gc;
        const int64_t xr = transposed ? c : r, xc = transposed ? r : c;
        inside = r < out_rows && c < out_cols;
        if (!inside) return 0.0f;
        float v = to_f32(x[xr * cols + xc]);
        if constexpr (ENCODED) v *= get_scale(source_scale, xr / source_gr * sc + xc / source_gc, e8m0);
        return v;
    };
    float amax = 0.0f;
    for (int j = lane; j < size; j += WAVE) {
        bool inside;
        amax = fmaxf(amax, fabsf(value(j, inside)));
    }
    amax = wave_max(amax);
    const float s = group_scale(amax, limit, e8m0);
    if (lane == 0) put_scale(scale, group, s, e8m0);
    for (int j = lane; j < size; j += WAVE) {
        bool inside;
        const float v = value(j, inside);
        if (inside) q[(gr0 + j / gc) * out_cols + gc0 + j % gc] = encode_clamped<TOut>(v, s, limit);
    }
}

// ------------------------------------------------------------------ dequantize
template <typename TQ>
__global__ __launch_bounds__(256) void dequantize_kernel(const TQ* __restrict__ q, const float* __restrict__ scale,
                                                          float* __restrict__ out, int64_t rows, int64_t cols, int gr,
                                                          int gc) {
    const int64_t nc = (cols + gc - 1) / gc;
    const int64_t total = rows * cols;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t r = i / cols, c = i % cols;
        out[i] = to_f32(q[i]) * scale[r / gr * nc + c / gc];
    }
}

// ------------------------------------------------------------------ byte transpose, 64 x 64 tile
// WORDS: rows and cols multiples of 4 and both pointers 4-byte aligned. A thread then owns a 4 x 4 byte block: four
// 4-byte loads (16 lanes cover 64 contiguous bytes of a row), a 4 x 4 transpose with byte permutes, the four words
// handed over through LDS so that the stores are again 64 contiguous bytes per 16 lanes.
// With a scale grid (one entry of scale_bytes bytes per block of codes, [srows, scols]), the grid is transposed in the
// same launch: the blocks share out its entries, thread 0 .. moving one each.
template <bool WORDS>
__global__ __launch_bounds__(256) void transpose_bytes(const uint8_t* __restrict__ x, uint8_t* __restrict__ out,
                                                        int64_t rows, int64_t cols, const uint8_t* __restrict__ scale = nullptr,
                                                        uint8_t* __restrict__ scale_out = nullptr, int64_t srows = 0,
                                                        int64_t scols = 0, int scale_bytes = 0) {
    const int64_t r0 = (int64_t)blockIdx.y * 64, c0 = (int64_t)blockIdx.x * 64;
    if (scale) {
        const int64_t entries = srows * scols, blocks = (int64_t)gridDim.x * gridDim.y;
        const int64_t per = (entries + blocks - 1) / blocks, first = ((int64_t)blockIdx.y * gridDim.x + blockIdx.x) * per;
        for (int64_t e = first + threadIdx.x; e < first + per && e < entries; e += blockDim.x) {
            const int64_t sr = e / scols, sc = e % scols;
            if (scale_bytes == 4) reinterpret_cast<float*>(scale_out)[sc * srows + sr] = reinterpret_cast<const float*>(scale)[e];
            else scale_out[sc * srows + sr] = scale[e];
        }
    }
    x += (int64_t)blockIdx.z * rows * cols;
    out += (int64_t)blockIdx.z * rows * cols;
    if constexpr (WORDS) {
        __shared__ uint32_t tile[64][17];
        const int b = threadIdx.x % 16, a = threadIdx.x / 16;               // block of rows 4a.., cols 4b..
        uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (r0 + 4 * a + i < rows && c0 + 4 * b < cols) w[i] = *reinterpret_cast<const uint32_t*>(x + (r0 + 4 * a + i) * cols + c0 + 4 * b);
        // t[j] = byte j of w[0..3]
        const uint32_t lo01 = __builtin_amdgcn_perm(w[1], w[0], 0x05010400u);   // w0.b0 w1.b0 w0.b1 w1.b1
        const uint32_t hi01 = __builtin_amdgcn_perm(w[1], w[0], 0x07030602u);   // w0.b2 w1.b2 w0.b3 w1.b3
        const uint32_t lo23 = __builtin_amdgcn_perm(w[3], w[2], 0x05010400u);
        const uint32_t hi23 = __builtin_amdgcn_perm(w[3], w[2], 0x07030602u);
        tile[4 * b + 0][a] = __builtin_amdgcn_perm(lo23, lo01, 0x05040100u);    // bytes 0,1 of lo01 then of lo23
        tile[4 * b + 1][a] = __builtin_amdgcn_perm(lo23, lo01, 0x07060302u);
        tile[4 * b + 2][a] = __builtin_amdgcn_perm(hi23, hi01, 0x05040100u);
        tile[4 * b + 3][a] = __builtin_amdgcn_perm(hi23, hi01, 0x07060302u);
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int c = threadIdx.x / 16 + 16 * i, ra = threadIdx.x % 16;
            if (c0 + c < cols && r0 + 4 * ra < rows) *reinterpret_cast<uint32_t*>(out + (c0 + c) * rows + r0 + 4 * ra) = tile[c][ra];
        }
    } else {
        __shared__ uint8_t tile[64][64 + 4];
        for (int id = threadIdx.x; id < 64 * 64; id += 256) {
            const int r = id / 64, c = id % 64;
            tile[r][c] = (r0 + r < rows && c0 + c < cols) ? x[(r0 + r) * cols + c0 + c] : 0;
        }
        __syncthreads();
        for (int id = threadIdx.x; id < 64 * 64; id += 256) {
            const int c = id / 64, r = id % 64;
            if (r0 + r < rows && c0 + c < cols) out[(c0 + c) * rows + r0 + r] = tile[r][c];
        }
    }
}

// ------------------------------------------------------------------ segmented transposed quantize
// One block per (64 columns, 32-token slot of the padded token axis). Slot s of group g covers
// rows offsets[g] + 32*(s - poffsets[g]/32) ...; rows past the group's end are zero.
template <typename TIn, typename TOut>
__global__ __launch_bounds__(64) void quantize_transposed_segmented(const TIn* __restrict__ x,
                                                                     const int64_t* __restrict__ offsets,
                                                                     const int64_t* __restrict__ poffsets, int groups,
                                                                     int64_t cols, int64_t t_total,
                                                                     uint8_t* __restrict__ qt, float* __restrict__ scale_t,
                                                                     float limit) {
    const int64_t slot = blockIdx.y;
    const int64_t col = (int64_t)blockIdx.x * 64 + threadIdx.x;
    const int64_t token = slot * 32;
    int g = 0;
    while (g + 1 < groups && poffsets[g + 1] <= token) ++g;
    if (col >= cols) return;
    const int64_t first = offsets[g] + (token - poffsets[g]);
    const int64_t end = offsets[g + 1];
    float v[32];
    float amax = 0.0f, poison = 0.0f;
#pragma unroll
    for (int i = 0; i < 32; ++i) {
        v[i] = first + i < end ? to_f32(x[(first + i) * cols + col]) : 0.0f;
        amax = fmaxf(amax, fabsf(v[i]));
        poison = poison_of(poison, v[i]);
    }
    const float s = group_scale(amax, limit);
    scale_t[col * (t_total / 32) + slot] = s;
    uint8_t* dst = qt + col * t_total + token;
    store_group32<TOut>(v, s, poison, limit, dst, 32, (reinterpret_cast<uintptr_t>(dst) & 15) == 0);
}

// 16-bit inputs: the 64 x 64 tile of quantize_dual16_tile64 over the padded token axis. A block takes two consecutive
// 32-token slots of one column tile, each with its own group, first row and count of valid rows (rows past a group's end
// are parked as zeros), so the transposed codes of a tile are again 64 consecutive bytes per column; optionally the
// row-wise layout of the valid rows is written in the same pass (q [rows, cols], scale [rows, ceil(cols/32)] in the
// unpadded row order). FP32 scales. (32768 x 4096 and x 1024 bf16, 16 groups, both layouts: 146 and 28.5 us against
// 158 and 33 us for a kernel of one slot per wavefront; the plain dual-layout kernel takes 135 and 23.4 us.)
// INTERIOR: both slots hold 32 valid rows, the tile lies inside the matrix and every 16-byte piece of either output is
// aligned: no bounds checks, base pointers in scalar registers with 32-bit offsets per lane.
template <typename TIn, typename TOut, bool ROWWISE, bool INTERIOR>
__device__ __forceinline__ void segmented16_tile64(const TIn* __restrict__ x, int64_t cols, int64_t t_total, uint8_t* __restrict__ qt,
                                                   float* __restrict__ scale_t, uint8_t* __restrict__ q, float* __restrict__ scale,
                                                   float limit, int64_t pair, int64_t c0, const int64_t (&first)[2], const int (&valid)[2],
                                                   uint16_t* park, int* flags) {
    constexpr int LDV = 64 + 4;
    const int tid = threadIdx.x, lane = tid % WAVE, wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
    const int64_t nc = (cols + 31) / 32, slots = t_total / 32;
    const bool clamp_free = limit == fp8_traits<TOut>::max;

    // ---- row-wise: thread (tile row tid / 4, 16 columns); wavefronts 0, 1 hold the first slot's rows, 2, 3 the second's
    {
        const int lr = tid / 4, lc = (tid % 4) * 16, half = wave / 2, in_slot = lr % 32;
        const int64_t slot_first = half ? first[1] : first[0];
        const bool live = INTERIOR || in_slot < (half ? valid[1] : valid[0]);
        const int64_t row = slot_first + in_slot, col = c0 + lc;
        const uint32_t offset = (uint32_t)in_slot * (uint32_t)cols + (uint32_t)lc;   // from the slot's first element of the tile
        uint4 raw[2] = {make_uint4(0, 0, 0, 0), make_uint4(0, 0, 0, 0)};
        if constexpr (INTERIOR) {
            const TIn* tile = x + slot_first * cols + c0;
            raw[0] = *reinterpret_cast<const uint4*>(tile + offset);
            raw[1] = *reinterpret_cast<const uint4*>(tile + offset + 8);
        } else if (live) {
            if (col < cols) raw[0] = *reinterpret_cast<const uint4*>(x + row * cols + col);      // cols % 8 == 0: whole pieces
            if (col + 8 < cols) raw[1] = *reinterpret_cast<const uint4*>(x + row * cols + col + 8);
        }
        {
            uint2* mine = reinterpret_cast<uint2*>(&park[lr * LDV + (lc ^ (((lr >> 4) & 3) << 4))]);
            mine[0] = make_uint2(raw[0].x, raw[0].y); mine[1] = make_uint2(raw[0].z, raw[0].w);
            mine[2] = make_uint2(raw[1].x, raw[1].y); mine[3] = make_uint2(raw[1].z, raw[1].w);
        }
        const uint32_t words[8] = {raw[0].x, raw[0].y, raw[0].z, raw[0].w, raw[1].x, raw[1].y, raw[1].z, raw[1].w};
        bool nonfinite;
        if constexpr (ROWWISE) {
            float s_row;
            uint32_t codes[4];
            if (!encode_words16<TIn, TOut>(words, limit, 0, clamp_free, s_row, codes, nonfinite)) {
                const Exact16 r = encode_words16_exact<TIn, TOut>(words[0], words[1], words[2], words[3], words[4], words[5], words[6], words[7], limit, 0);
                codes[0] = r.c0; codes[1] = r.c1; codes[2] = r.c2; codes[3] = r.c3; s_row = r.s;
            }
            if constexpr (INTERIOR) {
                *reinterpret_cast<uint4*>(q + slot_first * cols + c0 + offset) = make_uint4(codes[0], codes[1], codes[2], codes[3]);
                if (tid % 2 == 0) (scale + slot_first * nc + c0 / 32)[(uint32_t)in_slot * (uint32_t)nc + (uint32_t)(lc / 32)] = s_row;
            } else if (live && col < cols) {
                uint8_t* dst = q + row * cols + col;
                if (col + 16 <= cols && (reinterpret_cast<uintptr_t>(dst) & 15) == 0) {
                    *reinterpret_cast<uint4*>(dst) = make_uint4(codes[0], codes[1], codes[2], codes[3]);
                } else {
                    *reinterpret_cast<uint2*>(dst) = make_uint2(codes[0], codes[1]);                 // q is 8-byte aligned, cols % 8 == 0
                    if (col + 8 < cols) *reinterpret_cast<uint2*>(dst + 8) = make_uint2(codes[2], codes[3]);
                }
                if (tid % 2 == 0) scale[row * nc + col / 32] = s_row;
            }
        } else {
            constexpr uint32_t MAGNITUDE = 0x7fff7fffu, INF16 = std::is_same<TIn, bf16_t>::value ? 0x7f80u : 0x7c00u;
            uint32_t top = 0;
#pragma unroll
            for (int e = 0; e < 8; ++e) top = pk_max_u16(top, words[e] & MAGNITUDE);
            nonfinite = (top & 0xffffu) >= INF16 || (top >> 16) >= INF16;
        }
        const bool any_nonfinite = __builtin_amdgcn_ballot_w64(nonfinite) != 0;   // over the whole wavefront: outside any branch
        if (lane == 0) flags[wave] = any_nonfinite;
    }
    __syncthreads();
    const bool plain = (flags[0] | flags[1] | flags[2] | flags[3]) == 0;

    // ---- transposed: wavefront w takes columns 16 w .. + 15; lane = (column lane / 4, tile rows 16 (lane % 4) .. + 15)
    {
        const int tc = wave * 16 + lane / 4, chunk = lane % 4;
        const int64_t tcol = c0 + tc, token = pair * 64 + chunk * 16;
        uint32_t bits[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) bits[i] = park[(chunk * 16 + i) * LDV + (tc ^ (chunk << 4))];
        float w[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) w[i] = widen16<TIn>(bits[i]);
        float s_col;
        uint32_t tcodes[4];
        if (!plain || !encode_finite16<TOut>(w, limit, 0, clamp_free, s_col, tcodes)) {
            const Exact16 r = encode_words16_exact<TIn, TOut>(bits[0] | bits[1] << 16, bits[2] | bits[3] << 16, bits[4] | bits[5] << 16, bits[6] | bits[7] << 16,
                                                              bits[8] | bits[9] << 16, bits[10] | bits[11] << 16, bits[12] | bits[13] << 16,
                                                              bits[14] | bits[15] << 16, limit, 0);
            tcodes[0] = r.c0; tcodes[1] = r.c1; tcodes[2] = r.c2; tcodes[3] = r.c3; s_col = r.s;
        }
        if constexpr (INTERIOR) {
            *reinterpret_cast<uint4*>(qt + c0 * t_total + pair * 64 + ((uint32_t)tc * (uint32_t)t_total + (uint32_t)(chunk * 16))) = make_uint4(tcodes[0], tcodes[1], tcodes[2], tcodes[3]);
            if (chunk % 2 == 0) (scale_t + c0 * slots + pair * 2)[(uint32_t)tc * (uint32_t)slots + (uint32_t)(chunk / 2)] = s_col;
        } else if (tcol < cols && token < t_total) {                          // t_total is a multiple of 32: whole pieces only
            uint8_t* dst = qt + tcol * t_total + token;
            if ((reinterpret_cast<uintptr_t>(dst) & 15) == 0) {
                *reinterpret_cast<uint4*>(dst) = make_uint4(tcodes[0], tcodes[1], tcodes[2], tcodes[3]);
            } else {
#pragma unroll
                for (int k = 0; k < 4; ++k) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) dst[4 * k + e] = (uint8_t)(tcodes[k] >> (8 * e));
                }
            }
            if (chunk % 2 == 0) scale_t[tcol * slots + token / 32] = s_col;
        }
    }
}

template <typename TIn, typename TOut, bool ROWWISE>
__global__ __launch_bounds__(256, 8) void quantize_segmented16_tile64(const TIn* __restrict__ x, const int64_t* __restrict__ offsets,
                                                                    const int64_t* __restrict__ poffsets, int groups, int64_t cols,
                                                                    int64_t t_total, uint8_t* __restrict__ qt, float* __restrict__ scale_t,
                                                                    uint8_t* __restrict__ q, float* __restrict__ scale, float limit, int aligned,
                                                                    int xcd_walk) {
    __shared__ __attribute__((aligned(16))) uint16_t park[64 * (64 + 4)];
    __shared__ __attribute__((aligned(16))) int flags[4];
    // the walk of quantize_dual16_tile64: blocks in flight together take 32 slot pairs of one column tile, then the next;
    // with xcd_walk every XCD takes one contiguous eighth of it
    constexpr uint32_t BAND = 32;
    const int64_t slots = t_total / 32;
    const uint32_t tiles_x = (uint32_t)((cols + 63) / 64), tiles_y = (uint32_t)((slots + 1) / 2), tiles = tiles_x * tiles_y;
    uint32_t id = blockIdx.x;
    if (xcd_walk) id = (id % 8) * ((tiles + 7) / 8) + id / 8;
    if (id >= tiles) return;
    const uint32_t patch = id / (BAND * tiles_x), within = id % (BAND * tiles_x);
    const uint32_t tall = tiles_y - patch * BAND < BAND ? tiles_y - patch * BAND : BAND;
    const int64_t pair = patch * BAND + within % tall, c0 = (int64_t)(within / tall) * 64;
    // The two slots' groups and rows (uniform). A slot's group is the number of entries of poffsets[1 .. groups - 1] that are
    // <= its first token (the table is nondecreasing): 64 entries per load and ballot instead of a chain of dependent loads.
    int64_t first[2];
    int valid[2];
    {
        const int lane = threadIdx.x % WAVE;
        const int64_t token0 = 2 * pair * 32, token1 = token0 + 32;
        int g0 = 0, g1 = 0;
        for (int base = 1; base < groups; base += WAVE) {
            const int at = base + lane;
            const int64_t start = at < groups ? poffsets[at] : INT64_MAX;
            g0 += __popcll(__builtin_amdgcn_ballot_w64(start <= token0));
            g1 += __popcll(__builtin_amdgcn_ballot_w64(start <= token1));
        }
        const int gs[2] = {g0, g1};
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int64_t token = h ? token1 : token0;
            first[h] = offsets[gs[h]] + (token - poffsets[gs[h]]);
            const int64_t left = offsets[gs[h] + 1] - first[h];
            valid[h] = token >= t_total ? 0 : (int)(left < 0 ? 0 : left > 32 ? 32 : left);
        }
    }
    // (32-bit offsets inside a slot: 32 rows x cols and 64 columns x t_total stay below 2^31, the launcher sees to it)
    if (aligned && valid[0] == 32 && valid[1] == 32 && c0 + 64 <= cols)
        segmented16_tile64<TIn, TOut, ROWWISE, true>(x, cols, t_total, qt, scale_t, q, scale, limit, pair, c0, first, valid, park, flags);
    else
        segmented16_tile64<TIn, TOut, ROWWISE, false>(x, cols, t_total, qt, scale_t, q, scale, limit, pair, c0, first, valid, park, flags);
}

// ------------------------------------------------------------------ host dispatch
template <typename TIn, typename TOut>
static int launch_quantize(const void* x, int64_t rows, int64_t cols, void* q, float* scale, int gr, int gc,
                           float limit, int transposed, int e8m0, hipStream_t stream) {
    const TIn* xp = static_cast<const TIn*>(x);
    uint8_t* qp = static_cast<uint8_t*>(q);
    const bool vec = cols % 8 == 0 && reinterpret_cast<uintptr_t>(x) % (8 * sizeof(TIn)) == 0;
    if (gr == 1 && !transposed && vec && reinterpret_cast<uintptr_t>(q) % 8 == 0 && gc <= 512) {
        const int64_t nc = (cols + gc - 1) / gc;
        const int64_t chunks = rows * nc * (gc / 8);
        const dim3 grid((unsigned)((chunks + 255) / 256));
#define VIOLA_ROWWISE(GC) \
    case GC: VIOLA_LAUNCH((quantize_rowwise<TIn, TOut, GC>), grid, dim3(256), 0, stream, xp, qp, scale, rows, cols, nc, limit, e8m0); break;
        switch (gc) {
            VIOLA_ROWWISE(32) VIOLA_ROWWISE(64) VIOLA_ROWWISE(128) VIOLA_ROWWISE(256) VIOLA_ROWWISE(512)
            default: return VIOLA_EINVAL;
        }
#undef VIOLA_ROWWISE
        return viola_launch_status();
    }
    if constexpr (sizeof(TIn) == 2) {
        if (gr == 1 && gc == 32 && transposed && vec) {
            const int64_t tiles16 = ((cols + 63) / 64) * ((rows + 127) / 128);
            const dim3 grid16((unsigned)(tiles16 < 256 * 6 ? tiles16 : 256 * 6));
            VIOLA_LAUNCH((quantize_dual16<TIn, TOut, false>), grid16, dim3(256), 0, stream, xp, nullptr, nullptr, qp, scale, rows, cols, limit, nullptr, e8m0, 0);
            return viola_launch_status();
        }
    }
    if (gr == 1 && gc == 32 && transposed) {
        const dim3 grid((unsigned)((cols + TILE_C - 1) / TILE_C), (unsigned)((rows + TILE_R - 1) / TILE_R));
        if (vec) VIOLA_LAUNCH((quantize_tile<TIn, TOut, false, true, true>), grid, dim3(256), 0, stream, xp, nullptr, nullptr, qp, scale, rows, cols, limit, nullptr, e8m0);
        else VIOLA_LAUNCH((quantize_tile<TIn, TOut, false, true, false>), grid, dim3(256), 0, stream, xp, nullptr, nullptr, qp, scale, rows, cols, limit, nullptr, e8m0);
        return viola_launch_status();
    }
    if (gr == 32 && gc == 32 && !transposed && cols % 4 == 0 && reinterpret_cast<uintptr_t>(x) % (4 * sizeof(TIn)) == 0 &&
        reinterpret_cast<uintptr_t>(q) % 4 == 0) {
        const int64_t units = (rows + 31) / 32 * ((cols + 127) / 128);
        VIOLA_LAUNCH((quantize_block32<TIn, TOut>), dim3((unsigned)((units + 3) / 4)), dim3(256), 0, stream, xp, qp, scale,
                           rows, cols, (cols + 31) / 32, limit, e8m0);
        return viola_launch_status();
    }
    const int64_t out_rows = transposed ? cols : rows, out_cols = transposed ? rows : cols;
    const int64_t ngroups = ((out_rows + gr - 1) / gr) * ((out_cols + gc - 1) / gc);
    VIOLA_LAUNCH((quantize_generic<TIn, TOut, false>), dim3((unsigned)((ngroups + 3) / 4)), dim3(256), 0, stream,
                       xp, nullptr, qp, scale, rows, cols, gr, gc, transposed, 1, 32, limit, e8m0);
    return viola_launch_status();
}

template <typename TOut>
static int dispatch_in(int x_dtype, const void* x, int64_t rows, int64_t cols, void* q, float* scale, int gr, int gc,
                       float limit, int transposed, int e8m0, hipStream_t stream) {
    switch (x_dtype) {
        case VIOLA_F32: return launch_quantize<float, TOut>(x, rows, cols, q, scale, gr, gc, limit, transposed, e8m0, stream);
        case VIOLA_BF16: return launch_quantize<bf16_t, TOut>(x, rows, cols, q, scale, gr, gc, limit, transposed, e8m0, stream);
        case VIOLA_F16: return launch_quantize<f16_t, TOut>(x, rows, cols, q, scale, gr, gc, limit, transposed, e8m0, stream);
        default: return VIOLA_EINVAL;
    }
}

template <typename TIn, typename TOut>
static int launch_reencode(const void* x, const float* source_scale, int64_t rows, int64_t cols, void* q, float* scale,
                           int gr, int gc, float limit, int transposed, int sgr, int sgc, int e8m0, hipStream_t stream) {
    const int64_t out_rows = transposed ? cols : rows, out_cols = transposed ? rows : cols;
    const int64_t ngroups = ((out_rows + gr - 1) / gr) * ((out_cols + gc - 1) / gc);
    VIOLA_LAUNCH((quantize_generic<TIn, TOut, true>), dim3((unsigned)((ngroups + 3) / 4)), dim3(256), 0, stream,
                       static_cast<const TIn*>(x), source_scale, static_cast<uint8_t*>(q), scale, rows, cols, gr, gc,
                       transposed, sgr, sgc, limit, e8m0);
    return viola_launch_status();
}

template <typename TIn, typename TOut>
static int launch_dual(const void* x, int64_t rows, int64_t cols, void* q, float* scale, void* qt, float* scale_t,
                       float limit, float* column_partial, int e8m0, hipStream_t stream) {
    const bool vec = cols % 8 == 0 && reinterpret_cast<uintptr_t>(x) % (8 * sizeof(TIn)) == 0;
    const dim3 grid((unsigned)((cols + TILE_C - 1) / TILE_C), (unsigned)((rows + TILE_R - 1) / TILE_R));
    const TIn* xp = static_cast<const TIn*>(x);
    if constexpr (sizeof(TIn) == 2) {
        if (vec && reinterpret_cast<uintptr_t>(q) % 8 == 0) {
            const int64_t tiles64 = ((cols + 63) / 64) * ((rows + 63) / 64);
            if (tiles64 + 8 < (1ll << 31)) {
                // one to four rounds of resident blocks (eight per compute unit): the XCD-contiguous walk measured faster
                // (8192 x 4096: 29.7 -> 27.7 us); longer launches are faster with the eight XCDs streaming one region
                // (16384 x 4096: 68 against 76 us), shorter ones leave XCDs uneven
                const int xcd_walk = tiles64 >= 2048 && tiles64 <= 8192;
                // whole tiles may skip their bounds checks and address a lane's pieces by 32-bit offsets from the tile
                const int aligned = cols % 16 == 0 && rows % 16 == 0 && reinterpret_cast<uintptr_t>(q) % 16 == 0 &&
                                    reinterpret_cast<uintptr_t>(qt) % 16 == 0 && cols < (1ll << 24) && rows < (1ll << 24);
                VIOLA_LAUNCH((quantize_dual16_tile64<TIn, TOut>), dim3((unsigned)((tiles64 + 7) / 8 * 8)), dim3(256), 0, stream, xp,
                             static_cast<uint8_t*>(q), scale, static_cast<uint8_t*>(qt), scale_t, rows, cols, limit, column_partial, e8m0, xcd_walk,
                             aligned);
                return viola_launch_status();
            }
            const int64_t tiles16 = ((cols + 63) / 64) * ((rows + 127) / 128);
            const dim3 grid16((unsigned)(tiles16 < 256 * 6 ? tiles16 : 256 * 6));
            VIOLA_LAUNCH((quantize_dual16<TIn, TOut, true>), grid16, dim3(256), 0, stream, xp, static_cast<uint8_t*>(q), scale,
                               static_cast<uint8_t*>(qt), scale_t, rows, cols, limit, column_partial, e8m0, 0);
            return viola_launch_status();
        }
    }
    if (vec) VIOLA_LAUNCH((quantize_tile<TIn, TOut, true, true, true>), grid, dim3(256), 0, stream, xp, static_cast<uint8_t*>(q), scale, static_cast<uint8_t*>(qt), scale_t, rows, cols, limit, column_partial, e8m0);
    else VIOLA_LAUNCH((quantize_tile<TIn, TOut, true, true, false>), grid, dim3(256), 0, stream, xp, static_cast<uint8_t*>(q), scale, static_cast<uint8_t*>(qt), scale_t, rows, cols, limit, column_partial, e8m0);
    return viola_launch_status();
}

template <typename TIn, typename TOut>
static int launch_segmented(const void* x, int64_t cols, const int64_t* offsets, const int64_t* poffsets, int groups,
                            int64_t t_total, void* qt, float* scale_t, void* q, float* scale, float limit, hipStream_t stream) {
    if constexpr (sizeof(TIn) == 2) {
        const bool aligned = cols % 8 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 && (!q || reinterpret_cast<uintptr_t>(q) % 8 == 0);
        const int64_t tiles64 = ((t_total / 32 + 1) / 2) * ((cols + 63) / 64);   // two slots x one column tile each
        if (aligned && tiles64 + 8 < (1ll << 31)) {
            const dim3 grid64((unsigned)((tiles64 + 7) / 8 * 8));
            // an eighth of the walk per XCD pays for launches of this size (8272 tiles: 31.4 -> 28.5 us; 33088 tiles: 146 -> 156 us)
            const int xcd_walk = tiles64 >= 2048 && tiles64 <= 16384;
            // every 16-byte piece of the outputs aligned, 32-bit offsets inside a tile
            const int interior = cols % 16 == 0 && reinterpret_cast<uintptr_t>(qt) % 16 == 0 && (!q || reinterpret_cast<uintptr_t>(q) % 16 == 0) &&
                                 cols < (1 << 24) && t_total < (1 << 24);
            if (q) VIOLA_LAUNCH((quantize_segmented16_tile64<TIn, TOut, true>), grid64, dim3(256), 0, stream, static_cast<const TIn*>(x), offsets, poffsets, groups, cols, t_total, static_cast<uint8_t*>(qt), scale_t, static_cast<uint8_t*>(q), scale, limit, interior, xcd_walk);
            else VIOLA_LAUNCH((quantize_segmented16_tile64<TIn, TOut, false>), grid64, dim3(256), 0, stream, static_cast<const TIn*>(x), offsets, poffsets, groups, cols, t_total, static_cast<uint8_t*>(qt), scale_t, nullptr, nullptr, limit, interior, xcd_walk);
            return viola_launch_status();
        }
    }
    if (q) return VIOLA_EUNSUPPORTED;                                      // the row-wise by-product needs the 16-bit aligned path
    const dim3 grid((unsigned)((cols + 63) / 64), (unsigned)(t_total / 32));
    VIOLA_LAUNCH((quantize_transposed_segmented<TIn, TOut>), grid, dim3(64), 0, stream, static_cast<const TIn*>(x),
                       offsets, poffsets, groups, cols, t_total, static_cast<uint8_t*>(qt), scale_t, limit);
    return viola_launch_status();
}

static bool pow2(int v) { return v > 0 && (v & (v - 1)) == 0; }

}  // namespace viola

using namespace viola;

extern "C" int viola_group_quantize(const void* x, int x_dtype, int64_t rows, int64_t cols, void* q, int q_dtype,
                                    void* scale_, int gr, int gc, float limit, int transposed,
                                    const void* source_scale_, int source_gr, int source_gc, int scale_format,
                                    viola_stream_t stream_) {
    hipStream_t stream = viola_enter(stream_);
    float* scale = static_cast<float*>(scale_);
    const float* source_scale = static_cast<const float*>(source_scale_);
    VIOLA_CHECK_ARG(scale_format == VIOLA_SCALE_F32 || scale_format == VIOLA_SCALE_E8M0);
    const int e8m0 = scale_format == VIOLA_SCALE_E8M0;
    VIOLA_CHECK_ARG(viola_is_fp8(q_dtype) && rows >= 0 && cols >= 0 && pow2(gr) && pow2(gc) && limit > 0.0f);
    if (rows == 0 || cols == 0) return 0;
    VIOLA_CHECK_ARG(x && q && scale);
    if (source_scale) {
        VIOLA_CHECK_ARG(viola_is_fp8(x_dtype) && source_gr > 0 && source_gc > 0);
#define VIOLA_RE(TI, TO) return launch_reencode<TI, TO>(x, source_scale, rows, cols, q, scale, gr, gc, limit, transposed, source_gr, source_gc, e8m0, stream)
        if (x_dtype == VIOLA_E4M3 && q_dtype == VIOLA_E4M3) VIOLA_RE(e4m3_t, e4m3_t);
        if (x_dtype == VIOLA_E4M3 && q_dtype == VIOLA_E5M2) VIOLA_RE(e4m3_t, e5m2_t);
        if (x_dtype == VIOLA_E5M2 && q_dtype == VIOLA_E4M3) VIOLA_RE(e5m2_t, e4m3_t);
        VIOLA_RE(e5m2_t, e5m2_t);
#undef VIOLA_RE
    }
    VIOLA_CHECK_ARG(viola_is_float(x_dtype));
    if (q_dtype == VIOLA_E4M3) return dispatch_in<e4m3_t>(x_dtype, x, rows, cols, q, scale, gr, gc, limit, transposed, e8m0, stream);
    return dispatch_in<e5m2_t>(x_dtype, x, rows, cols, q, scale, gr, gc, limit, transposed, e8m0, stream);
}

extern "C" int viola_group_quantize_dual(const void* x, int x_dtype, int64_t rows, int64_t cols, void* q, void* scale_,
                                         void* qt, void* scale_t_, int q_dtype, int gc, float limit,
                                         float* column_partial, int scale_format, viola_stream_t stream_) {
    hipStream_t stream = viola_enter(stream_);
    float* scale = static_cast<float*>(scale_);
    float* scale_t = static_cast<float*>(scale_t_);
    VIOLA_CHECK_ARG(scale_format == VIOLA_SCALE_F32 || scale_format == VIOLA_SCALE_E8M0);
    const int e8m0 = scale_format == VIOLA_SCALE_E8M0;
    VIOLA_CHECK_ARG(viola_is_fp8(q_dtype) && viola_is_float(x_dtype) && rows >= 0 && cols >= 0 && limit > 0.0f);
    if (gc != 32) return VIOLA_EUNSUPPORTED;
    if (rows == 0 || cols == 0) return 0;
    VIOLA_CHECK_ARG(x && q && scale && qt && scale_t);
#define VIOLA_DUAL(TI, TO) return launch_dual<TI, TO>(x, rows, cols, q, scale, qt, scale_t, limit, column_partial, e8m0, stream)
    if (q_dtype == VIOLA_E4M3) {
        if (x_dtype == VIOLA_F32) VIOLA_DUAL(float, e4m3_t);
        if (x_dtype == VIOLA_BF16) VIOLA_DUAL(bf16_t, e4m3_t);
        VIOLA_DUAL(f16_t, e4m3_t);
    }
    if (x_dtype == VIOLA_F32) VIOLA_DUAL(float, e5m2_t);
    if (x_dtype == VIOLA_BF16) VIOLA_DUAL(bf16_t, e5m2_t);
    VIOLA_DUAL(f16_t, e5m2_t);
#undef VIOLA_DUAL
}

extern "C" int viola_gated_quantize_dual(const void* z, int z_dtype, int64_t rows, int64_t cols, int activation, void* q,
                                         void* scale, void* qt, void* scale_t, int q_dtype, int gc, float limit,
                                         int scale_format, viola_stream_t stream_) {
    hipStream_t stream = viola_enter(stream_);
    VIOLA_CHECK_ARG(scale_format == VIOLA_SCALE_F32 || scale_format == VIOLA_SCALE_E8M0);
    VIOLA_CHECK_ARG(activation == VIOLA_SILU || activation == VIOLA_GELU || activation == VIOLA_RELU);
    VIOLA_CHECK_ARG(viola_is_fp8(q_dtype) && viola_is_float(z_dtype) && rows >= 0 && cols >= 0 && limit > 0.0f);
    if (gc != 32 || z_dtype == VIOLA_F32 || cols % 8 != 0) return VIOLA_EUNSUPPORTED;
    if (rows == 0 || cols == 0) return 0;
    VIOLA_CHECK_ARG(z && q && scale && qt && scale_t);
    if (reinterpret_cast<uintptr_t>(z) % 16 != 0 || reinterpret_cast<uintptr_t>(q) % 8 != 0) return VIOLA_EUNSUPPORTED;
    if (64 * cols * 2 >= (1ll << 31)) return VIOLA_EUNSUPPORTED;            // a wavefront's 32 rows are one buffer
    const int e8m0 = scale_format == VIOLA_SCALE_E8M0;
    const int64_t tiles16 = ((cols + 63) / 64) * ((rows + 127) / 128);
    const dim3 grid16((unsigned)(tiles16 < 256 * 6 ? tiles16 : 256 * 6));
#define VIOLA_GATED_DUAL(TI, TO)                                                                                            \
    VIOLA_LAUNCH((quantize_dual16<TI, TO, true, true>), grid16, dim3(256), 0, stream, static_cast<const TI*>(z),       \
                       static_cast<uint8_t*>(q), static_cast<float*>(scale), static_cast<uint8_t*>(qt),                      \
                       static_cast<float*>(scale_t), rows, cols, limit, (float*)nullptr, e8m0, activation)
    if (q_dtype == VIOLA_E4M3) {
        if (z_dtype == VIOLA_BF16) VIOLA_GATED_DUAL(bf16_t, e4m3_t);
        else VIOLA_GATED_DUAL(f16_t, e4m3_t);
    } else {
        if (z_dtype == VIOLA_BF16) VIOLA_GATED_DUAL(bf16_t, e5m2_t);
        else VIOLA_GATED_DUAL(f16_t, e5m2_t);
    }
#undef VIOLA_GATED_DUAL
    return viola_launch_status();
}

extern "C" int viola_column_reduce(const float* partial, int64_t parts, int64_t cols, void* out, int out_dtype,
                                   viola_stream_t stream_) {
    hipStream_t stream = viola_enter(stream_);
    VIOLA_CHECK_ARG(viola_is_float(out_dtype) && parts >= 0 && cols >= 0);
    if (cols == 0) return 0;
    VIOLA_CHECK_ARG(out && (parts == 0 || partial));
    const dim3 grid((unsigned)((cols + 31) / 32));
    if (out_dtype == VIOLA_F32) VIOLA_LAUNCH(column_reduce_kernel<float>, grid, dim3(256), 0, stream, partial, parts, cols, static_cast<float*>(out));
    else if (out_dtype == VIOLA_BF16) VIOLA_LAUNCH(column_reduce_kernel<bf16_t>, grid, dim3(256), 0, stream, partial, parts, cols, static_cast<bf16_t*>(out));
    else VIOLA_LAUNCH(column_reduce_kernel<f16_t>, grid, dim3(256), 0, stream, partial, parts, cols, static_cast<f16_t*>(out));
    return viola_launch_status();
}

extern "C" int viola_varlen_quantize_transposed(const void* x, int x_dtype, int64_t rows, int64_t cols,
                                                const int64_t* offsets, const int64_t* poffsets, int groups,
                                                int64_t t_total, void* qt, float* scale_t, int q_dtype, float limit,
                                                void* q, float* scale, viola_stream_t stream_) {
    hipStream_t stream = viola_enter(stream_);
    VIOLA_CHECK_ARG(viola_is_fp8(q_dtype) && viola_is_float(x_dtype) && rows >= 0 && cols >= 0 && groups > 0);
    VIOLA_CHECK_ARG(t_total >= 0 && t_total % 32 == 0 && limit > 0.0f);
    if (t_total == 0 || cols == 0) return 0;
    VIOLA_CHECK_ARG(x && offsets && poffsets && qt && scale_t && t_total / 32 <= 65535 && (!q == !scale));
#define VIOLA_SEG(TI, TO) return launch_segmented<TI, TO>(x, cols, offsets, poffsets, groups, t_total, qt, scale_t, q, scale, limit, stream)
    if (q_dtype == VIOLA_E4M3) {
        if (x_dtype == VIOLA_F32) VIOLA_SEG(float, e4m3_t);
        if (x_dtype == VIOLA_BF16) VIOLA_SEG(bf16_t, e4m3_t);
        VIOLA_SEG(f16_t, e4m3_t);
    }
    if (x_dtype == VIOLA_F32) VIOLA_SEG(float, e5m2_t);
    if (x_dtype == VIOLA_BF16) VIOLA_SEG(bf16_t, e5m2_t);
    VIOLA_SEG(f16_t, e5m2_t);
#undef VIOLA_SEG
}

extern "C" int viola_group_dequantize(const void* q, int q_dtype, const float* scale, int64_t rows, int64_t cols, int gr,
                                      int gc, float* out, viola_stream_t stream_) {
    hipStream_t stream = viola_enter(stream_);
    VIOLA_CHECK_ARG(viola_is_fp8(q_dtype) && rows >= 0 && cols >= 0 && gr > 0 && gc > 0);
    if (rows == 0 || cols == 0) return 0;
    VIOLA_CHECK_ARG(q && scale && out);
    const int64_t total = rows * cols;
    const unsigned blocks = (unsigned)((total + 255) / 256 < 65536 * 16 ? (total + 255) / 256 : 65536 * 16);
    if (q_dtype == VIOLA_E4M3)
        VIOLA_LAUNCH(dequantize_kernel<e4m3_t>, dim3(blocks), dim3(256), 0, stream, static_cast<const e4m3_t*>(q), scale, out, rows, cols, gr, gc);
    else
        VIOLA_LAUNCH(dequantize_kernel<e5m2_t>, dim3(blocks), dim3(256), 0, stream, static_cast<const e5m2_t*>(q), scale, out, rows, cols, gr, gc);
    return viola_launch_status();
}

extern "C" int viola_block_transpose(const void* x, void* out, int64_t rows, int64_t cols, const void* scale, void* scale_out,
                                     int gr, int gc, int scale_format, viola_stream_t stream_) {
    hipStream_t stream = viola_enter(stream_);
    VIOLA_CHECK_ARG(rows >= 0 && cols >= 0 && gr > 0 && gc > 0 && (scale_format == VIOLA_SCALE_F32 || scale_format == VIOLA_SCALE_E8M0));
    if (rows == 0 || cols == 0) return 0;
    VIOLA_CHECK_ARG(x && out && scale && scale_out && (rows + 63) / 64 <= 65535);
    const int scale_bytes = scale_format == VIOLA_SCALE_F32 ? 4 : 1;
    VIOLA_CHECK_ARG(reinterpret_cast<uintptr_t>(scale) % scale_bytes == 0 && reinterpret_cast<uintptr_t>(scale_out) % scale_bytes == 0);
    const int64_t srows = (rows + gr - 1) / gr, scols = (cols + gc - 1) / gc;
    const dim3 grid((unsigned)((cols + 63) / 64), (unsigned)((rows + 63) / 64), 1);
    const bool words = rows % 4 == 0 && cols % 4 == 0 && reinterpret_cast<uintptr_t>(x) % 4 == 0 && reinterpret_cast<uintptr_t>(out) % 4 == 0;
    if (words) VIOLA_LAUNCH(transpose_bytes<true>, grid, dim3(256), 0, stream, static_cast<const uint8_t*>(x), static_cast<uint8_t*>(out), rows, cols, static_cast<const uint8_t*>(scale), static_cast<uint8_t*>(scale_out), srows, scols, scale_bytes);
    else VIOLA_LAUNCH(transpose_bytes<false>, grid, dim3(256), 0, stream, static_cast<const uint8_t*>(x), static_cast<uint8_t*>(out), rows, cols, static_cast<const uint8_t*>(scale), static_cast<uint8_t*>(scale_out), srows, scols, scale_bytes);
    return viola_launch_status();
}

extern "C" int viola_fp8_transpose(const void* x, void* out, int64_t batch, int64_t rows, int64_t cols, viola_stream_t stream_) {
    hipStream_t stream = viola_enter(stream_);
    VIOLA_CHECK_ARG(batch >= 0 && rows >= 0 && cols >= 0);
    if (batch == 0 || rows == 0 || cols == 0) return 0;
    VIOLA_CHECK_ARG(x && out && (rows + 63) / 64 <= 65535 && batch <= 65535);
    const dim3 grid((unsigned)((cols + 63) / 64), (unsigned)((rows + 63) / 64), (unsigned)batch);
    const bool words = rows % 4 == 0 && cols % 4 == 0 && reinterpret_cast<uintptr_t>(x) % 4 == 0 && reinterpret_cast<uintptr_t>(out) % 4 == 0;
    if (words) VIOLA_LAUNCH(transpose_bytes<true>, grid, dim3(256), 0, stream, static_cast<const uint8_t*>(x), static_cast<uint8_t*>(out), rows, cols, nullptr, nullptr, 0, 0, 0);
    else VIOLA_LAUNCH(transpose_bytes<false>, grid, dim3(256), 0, stream, static_cast<const uint8_t*>(x), static_cast<uint8_t*>(out), rows, cols, nullptr, nullptr, 0, 0, 0);
    return viola_launch_status();
}
