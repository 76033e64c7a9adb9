// Fast path of the grouped-scale FP8 GEMM for gfx950 (see gemm.hip for the contract and the operand
// orientation). Requires 16-byte aligned operand rows and k ranges that are multiples of 16.
//
// Block: 512 threads = 8 wavefronts (two per SIMD), tile 128 (m) x 128 (b rows) x 128 (k), two LDS
// stages, one block per CU. A wavefront owns two 32 x 32 sub-tiles (64 m x 32 n; gated forward: 32 m x
// 32 gate + 32 up columns).
//   * global -> registers -> LDS, next chunk's loads issued before the math of the current chunk;
//     per thread two 16-byte loads per operand, eight lanes cover one 128-byte row segment.
//   * LDS rows are 128 + 16 bytes. Inside each 32-byte K group the two middle 8-byte pieces are swapped,
//     so the 8 codes a lane needs for both k halves of a group (k = 16*ks + 8*(lane/32)) are adjacent
//     and one ds_read_b128 fetches them; the 144-byte stride spreads 8 consecutive rows over all banks.
//   * math: per K group 2 x v_mfma_f32_32x32x16 per sub-tile into a fresh accumulator set, then
//     total += acc * (sa * sb), one FMA per output element. Two accumulator sets alternate: the FMAs
//     that fold group g are issued between the MFMAs of group g+1, so the matrix pipe and the VALU
//     run together inside one wavefront as well as across the two wavefronts of a SIMD. The operands
//     of group g+1 are read from LDS before the MFMAs of group g.
//   * epilogue stores runs of four consecutive n as one 8- or 16-byte store.
#include "gemm_args.hpp"

namespace viola {

constexpr int FBK = 128, FKG = FBK / 32, FLD = FBK + 16;          // LDS row stride: 16 bytes of padding per row
constexpr int FTHREADS = 512;

template <bool A_BF8, bool B_BF8>
__device__ __forceinline__ f32x16 mfma32(long x, long y, f32x16 c) {
    // x: 8 codes of the b matrix (MFMA srcA), y: 8 codes of the a matrix (MFMA srcB)
    if constexpr (!B_BF8 && !A_BF8) return __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(x, y, c, 0, 0, 0);
    else if constexpr (!B_BF8 && A_BF8) return __builtin_amdgcn_mfma_f32_32x32x16_fp8_bf8(x, y, c, 0, 0, 0);
    else if constexpr (B_BF8 && !A_BF8) return __builtin_amdgcn_mfma_f32_32x32x16_bf8_fp8(x, y, c, 0, 0, 0);
    else return __builtin_amdgcn_mfma_f32_32x32x16_bf8_bf8(x, y, c, 0, 0, 0);
}

__device__ __forceinline__ float load_bias(const void* p, int64_t i, int dtype) {
    if (dtype == VIOLA_F32) return static_cast<const float*>(p)[i];
    if (dtype == VIOLA_BF16) return bf16_bits_to_f32(static_cast<const uint16_t*>(p)[i]);
    return (float)static_cast<const _Float16*>(p)[i];
}

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

// Four consecutive outputs of one row.
template <typename TO> struct Quad;
template <> struct Quad<float> {
    static __device__ __forceinline__ void store(float* p, const float (&v)[4]) { *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]); }
    static __device__ __forceinline__ void load(const float* p, float (&v)[4]) { const float4 t = *reinterpret_cast<const float4*>(p); v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w; }
};
template <> struct Quad<bf16_t> {
    static __device__ __forceinline__ void store(bf16_t* p, const float (&v)[4]) {
        *reinterpret_cast<uint2*>(p) = make_uint2(f32_to_bf16x2_bits(v[0], v[1]), f32_to_bf16x2_bits(v[2], v[3]));
    }
    static __device__ __forceinline__ void load(const bf16_t* p, float (&v)[4]) {
        const uint2 t = *reinterpret_cast<const uint2*>(p);
        v[0] = __uint_as_float(t.x << 16); v[1] = __uint_as_float(t.x & 0xffff0000u);
        v[2] = __uint_as_float(t.y << 16); v[3] = __uint_as_float(t.y & 0xffff0000u);
    }
};
template <> struct Quad<f16_t> {
    typedef _Float16 h4 __attribute__((ext_vector_type(4)));
    static __device__ __forceinline__ void store(f16_t* p, const float (&v)[4]) {
        h4 t = {(_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3]};
        *reinterpret_cast<h4*>(p) = t;
    }
    static __device__ __forceinline__ void load(const f16_t* p, float (&v)[4]) {
        const h4 t = *reinterpret_cast<const h4*>(p);
        v[0] = (float)t[0]; v[1] = (float)t[1]; v[2] = (float)t[2]; v[3] = (float)t[3];
    }
};

template <int S> struct Stage { static constexpr int value = S; };

template <typename TO> __device__ __forceinline__ float rounded(float v) { return to_f32(from_f32<TO>(v)); }

template <int MODE, bool A_BF8, bool B_BF8, bool B_ROWSCALE, typename TO>
__global__ __launch_bounds__(FTHREADS, 2) void group_gemm_fast(GemmArgs p, int bias_dtype) {
    __shared__ __attribute__((aligned(16))) uint8_t lds_a[2][BM * FLD];
    __shared__ __attribute__((aligned(16))) uint8_t lds_b[2][BN * FLD];
    __shared__ __attribute__((aligned(16))) float lds_sa[2][FKG][BM];
    __shared__ __attribute__((aligned(16))) float lds_sb[2][FKG][BN];

    // wave grid and sub-tiles per wave: plain / gated backward 2 (m) x 4 (n) waves of 2 x 1 sub-tiles;
    // gated forward 4 (m) x 2 (n) waves of 1 x 2 sub-tiles (gate and up columns of the same n in one lane)
    constexpr bool GATED = MODE == MODE_GATED_FWD;
    constexpr int TM = GATED ? 1 : 2, TN = GATED ? 2 : 1, WN = GATED ? 2 : 4;
    constexpr int PANEL = GATED ? BN / 2 : BN;
    const int tid = threadIdx.x, lane = tid % WAVE, wave = tid / WAVE;
    const int wm = wave / WN, wn = wave % WN;
    const int l32 = lane % 32, lhi = lane / 32;

    // ---- which problem / tile (uniform per block)
    // Workgroups are dealt round-robin to the 8 XCDs (block i -> XCD i % 8), each with its own L2. Give every XCD a
    // contiguous range of output tiles, walked in groups of 8 m tiles x all n tiles (n slowest inside a group), so the
    // blocks resident on one XCD at a time share a few rows of a and b.
    int tile_m = blockIdx.y, tile_n = blockIdx.x;
    if (p.tiles_m) {
        const int per_xcd = gridDim.x / 8;
        const int t = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
        if (t >= p.tiles_m * p.tiles_n) return;
        const int group = 8 * p.tiles_n;
        const int first_m = t / group * 8;
        const int rows = p.tiles_m - first_m < 8 ? p.tiles_m - first_m : 8;
        tile_m = first_m + t % group % rows;
        tile_n = t % group / rows;
    }
    int64_t m_begin = (int64_t)tile_m * BM, m_end = p.m;
    int64_t k_begin = 0, k_end = p.k;
    const uint8_t* bptr = p.b;
    const float* sbptr = p.sb;
    uint8_t* outptr = static_cast<uint8_t*>(p.out);
    if (p.offsets) {
        int64_t tile = tile_m;
        int g = 0;
        bool found = false;
        for (; g < p.groups; ++g) {
            const int64_t lo = p.offsets[g], hi = p.offsets[g + 1];
            const int64_t tiles = (hi - lo + BM - 1) / BM;
            if (tile < tiles) { m_begin = lo + tile * BM; m_end = hi; found = true; break; }
            tile -= tiles;
        }
        if (!found) return;
        bptr += (int64_t)g * p.b_group_stride;
        sbptr += (int64_t)g * p.sb_group_stride;
    }
    if (p.koffsets) {
        const int g = blockIdx.z;
        k_begin = p.koffsets[g];
        k_end = p.koffsets[g + 1];
        outptr += (int64_t)g * p.out_group_stride * (int64_t)sizeof(TO);
    }
    if (m_begin >= m_end) return;
    const int64_t n_begin = (int64_t)tile_n * PANEL;
    const int64_t b_rows_total = GATED ? 2 * p.n : p.n;
    auto b_global_row = [&](int r) -> int64_t {                               // tile-local b row -> row of b
        int64_t bn;
        if constexpr (GATED) bn = (int64_t)(r / PANEL) * p.n + n_begin + r % PANEL;
        else bn = n_begin + r;
        return bn < b_rows_total ? bn : b_rows_total - 1;
    };

    // ---- per-thread constants: global offsets of its two 16-byte chunks per operand, LDS slots
    const int lrow = tid / 8, chunk = tid % 8;                               // rows lrow + 64*it, 16-byte chunk of the 128-byte row
    uint32_t goff_a[2], goff_b[2];
    const uint8_t* abase = p.a + m_begin * p.lda + k_begin;
#pragma unroll
    for (int it = 0; it < 2; ++it) {
        const int r = lrow + 64 * it;
        int64_t am = m_begin + r;
        am = am < m_end ? am : m_end - 1;
        goff_a[it] = (uint32_t)((am - m_begin) * p.lda + chunk * 16);
        goff_b[it] = (uint32_t)(b_global_row(r) * p.ldb + chunk * 16);       // relative to bptr + k offset (row span < 4 GiB)
    }
    const uint8_t* bbase = bptr + k_begin;
    // global bytes [16c, 16c+16) of a row are the pieces (ks = c % 2, half 0) and (ks, half 1) of K group c / 2; in LDS
    // a group is laid out [ks0 h0][ks1 h0][ks0 h1][ks1 h1]
    const int wslot = lrow * FLD + (chunk / 2) * 32 + (chunk % 2) * 8;       // second piece 16 bytes further; + 64*it*FLD
    // scale staging: thread owns tile row srow and K group sgroup of each chunk (512 = 4 groups x 128 rows)
    const int srow = tid % BM, sgroup = tid / BM;
    uint32_t sa_off, sb_off;                                                 // byte offsets of this thread's scale rows
    {
        int64_t am = m_begin + srow;
        am = am < m_end ? am : m_end - 1;
        sa_off = (uint32_t)(am / p.ar * p.ldsa * 4);
        sb_off = (uint32_t)(b_global_row(srow) / p.br * p.ldsb * 4);
    }
    // MFMA operand reads: 16 bytes = both k halves of one K group for row l32 (+32 per sub-tile), quarter pair lhi
    auto a_sub = [&](int j) -> int { return (wm * TM + j) * 32; };
    auto b_sub = [&](int i) -> int { return GATED ? i * PANEL + wn * 32 : wn * 32; };
    const int rd_a = (a_sub(0) + l32) * FLD + lhi * 16;
    const int rd_b = (b_sub(0) + l32) * FLD + lhi * 16;

    // Two register staging sets: the loads of chunk c+2 are issued while chunk c+1 is still in flight, so every
    // chunk has a whole iteration of math to arrive before it is written to LDS.
    // Raw buffer loads: 32-bit per-lane offset + uniform chunk offset, no per-load address arithmetic.
    // (a chunk offset k0 enters as the scalar offset)
    const __amdgpu_buffer_rsrc_t res_a = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(abase), 0, 0x7fffffff, 0x00020000);
    const __amdgpu_buffer_rsrc_t res_b = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(bbase), 0, 0x7fffffff, 0x00020000);
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    auto load16 = [&](const __amdgpu_buffer_rsrc_t& res, uint32_t voffset, int32_t soffset) -> uint4 {
        const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(res, (int)voffset, soffset, 0);
        return make_uint4(v[0], v[1], v[2], v[3]);
    };
    uint4 ra[2][2], rb[2][2];
    float rsa[2], rsb[2];
    // Branch-free: a lane whose 16 bytes lie past the end of the k range (or a chunk past the last one) loads from
    // an offset outside the buffer, which returns zeros without touching memory. No control flow around the loads,
    // so the compiler's wait counters stay exact and the newest loads remain in flight across the LDS writes.
    const __amdgpu_buffer_rsrc_t res_sa = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.sa), 0, 0x7fffffff, 0x00020000);
    const __amdgpu_buffer_rsrc_t res_sb = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(sbptr), 0, 0x7fffffff, 0x00020000);
    constexpr uint32_t OUTSIDE = 0x80000000u;
    const int64_t k_len = k_end - k_begin;
    const int64_t chunks = (k_len + FBK - 1) / FBK;
    auto fetch = [&](int64_t c, int set) {                                    // set is a compile-time constant at every call
        const int64_t k0 = c * FBK;                                          // relative to k_begin
        const bool inside = k0 + chunk * 16 < k_len;
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            ra[set][it] = load16(res_a, inside ? goff_a[it] : OUTSIDE, (int32_t)k0);
            rb[set][it] = load16(res_b, inside ? goff_b[it] : OUTSIDE, (int32_t)k0);
        }
        const int64_t kk = k_begin + k0 + sgroup * 32;
        const bool group_inside = k0 + sgroup * 32 < k_len;
        rsa[set] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(res_sa, group_inside ? (int)(sa_off + (uint32_t)(kk >> p.ak_shift) * 4) : (int)OUTSIDE, 0, 0));
        rsb[set] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(res_sb, group_inside ? (int)(sb_off + (uint32_t)(kk >> p.bk_shift) * 4) : (int)OUTSIDE, 0, 0));
    };
    auto stash = [&](int s, int set) {
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            uint8_t* da = &lds_a[s][wslot + it * 64 * FLD];
            *reinterpret_cast<uint2*>(da) = make_uint2(ra[set][it].x, ra[set][it].y);
            *reinterpret_cast<uint2*>(da + 16) = make_uint2(ra[set][it].z, ra[set][it].w);
            uint8_t* db = &lds_b[s][wslot + it * 64 * FLD];
            *reinterpret_cast<uint2*>(db) = make_uint2(rb[set][it].x, rb[set][it].y);
            *reinterpret_cast<uint2*>(db + 16) = make_uint2(rb[set][it].z, rb[set][it].w);
        }
        lds_sa[s][sgroup][srow] = rsa[set];
        lds_sb[s][sgroup][srow] = rsb[set];
    };

    f32x16 total[TN][TM];                                                    // [b sub-tile i][a sub-tile j]
#pragma unroll
    for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int j = 0; j < TM; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) total[i][j][r] = 0.0f;

    fetch(0, 0);
    stash(0, 0);
    fetch(1, 0);                                                             // chunk 1 in flight in set 0
    __syncthreads();

    // Software pipeline state, carried across chunks: operands of the group about to be multiplied, the accumulators
    // of the group multiplied last (not yet folded) and its scale products.
    struct Ops { uint4 a[TM], b[TN]; };                                      // x,y: ks 0, z,w: ks 1
    Ops ops[2];                                                              // [parity of the K group]
    f32x16 acc[2][TN][TM];
    float sc[2][TN][TM];                                                     // uniform b scales: sa * sb per sub-tile
    float sa_p[2][TM];                                                       // row-scaled b: sa only, sb read per fold
    auto read_ops = [&](int s, int kg, Ops& o) {
#pragma unroll
        for (int j = 0; j < TM; ++j) o.a[j] = *reinterpret_cast<const uint4*>(&lds_a[s][rd_a + kg * 32 + j * 32 * FLD]);
#pragma unroll
        for (int i = 0; i < TN; ++i) o.b[i] = *reinterpret_cast<const uint4*>(&lds_b[s][rd_b + kg * 32 + (b_sub(i) - b_sub(0)) * FLD]);
    };
    auto as_long = [](uint32_t lo, uint32_t hi) -> long { return (long)(((uint64_t)hi << 32) | lo); };
    // Fold accumulator set `set` (group kg of stage s) into the totals; `part` of `parts` slices so that it can be
    // spread between MFMAs.
    auto fold = [&](int set, int s, int kg, int part, int parts) {
        const int per = TN * TM * 16 / parts;
#pragma unroll
        for (int e = part * per; e < (part + 1) * per; ++e) {
            const int i = e / (TM * 16), j = e / 16 % TM, r = e % 16;
            if constexpr (!B_ROWSCALE) {
                total[i][j][r] = fmaf(acc[set][i][j][r], sc[set][i][j], total[i][j][r]);
            } else {
                const float sbv = lds_sb[s][kg][b_sub(i) + (r / 4) * 8 + lhi * 4 + r % 4];
                total[i][j][r] = fmaf(acc[set][i][j][r], sa_p[set][j] * sbv, total[i][j][r]);
            }
        }
    };
    // One chunk of math on LDS stage S (compile time). Group g: read ops(g+1); MFMAs(g) into set g&1 with the fold of
    // group g-1 (set (g-1)&1) spread between them.
    // The last group of a chunk is folded during the first MFMAs of the next chunk (the very first fold adds zeros).
    // With row-wise b scales the fold reads them from the LDS stage that other wavefronts may already be refilling,
    // so there each chunk folds its own last group.
    constexpr bool CARRY = !B_ROWSCALE;
#pragma unroll
    for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int j = 0; j < TM; ++j) {
            sc[1][i][j] = 0.0f;
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[1][i][j][r] = 0.0f;
        }
    auto compute = [&](auto stage_tag) {
        constexpr int S = decltype(stage_tag)::value;
#pragma unroll
        for (int kg = 0; kg < FKG; ++kg) {
            const int set = kg & 1;
            if (kg + 1 < FKG) read_ops(S, kg + 1, ops[(kg + 1) & 1]);
            const Ops& cur = ops[kg & 1];
            float sc_new[TN][TM];
#pragma unroll
            for (int j = 0; j < TM; ++j) {
                const float sa_l = lds_sa[S][kg][a_sub(j) + l32];
                if constexpr (B_ROWSCALE) sa_p[set][j] = sa_l;
                else {
#pragma unroll
                    for (int i = 0; i < TN; ++i) sc_new[i][j] = sa_l * lds_sb[S][kg][b_sub(i)];
                }
            }
            const f32x16 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
            int step = 0;
#pragma unroll
            for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                for (int i = 0; i < TN; ++i)
#pragma unroll
                    for (int j = 0; j < TM; ++j) {
                        const long x = ks == 0 ? as_long(cur.b[i].x, cur.b[i].y) : as_long(cur.b[i].z, cur.b[i].w);
                        const long y = ks == 0 ? as_long(cur.a[j].x, cur.a[j].y) : as_long(cur.a[j].z, cur.a[j].w);
                        acc[set][i][j] = mfma32<A_BF8, B_BF8>(x, y, ks == 0 ? zero : acc[set][i][j]);
                        // a quarter of the previous group's fold after each MFMA
                        if (CARRY || kg > 0) fold(set ^ 1, S, kg - 1, step, 4);
                        ++step;
                        __builtin_amdgcn_sched_barrier(0);
                    }
            if constexpr (!B_ROWSCALE) {
#pragma unroll
                for (int i = 0; i < TN; ++i)
#pragma unroll
                    for (int j = 0; j < TM; ++j) sc[set][i][j] = sc_new[i][j];
            }
#pragma unroll
            for (int i = 0; i < TN; ++i)
#pragma unroll
                for (int j = 0; j < TM; ++j) asm volatile("" : "+v"(total[i][j]));
        }
        if constexpr (!CARRY) {
            fold((FKG - 1) & 1, S, FKG - 1, 0, 1);
#pragma unroll
            for (int i = 0; i < TN; ++i)
#pragma unroll
                for (int j = 0; j < TM; ++j) asm volatile("" : "+v"(total[i][j]));
        }
    };
    // Straight-line steady state: no control flow between the loads, the math and the LDS writes. An odd chunk count
    // runs one extra all-zero chunk.
    read_ops(0, 0, ops[0]);
    for (int64_t c = 0; c < chunks; c += 2) {
        fetch(c + 2, 1);                                                     // set 1 <- chunk c+2; set 0 holds chunk c+1
        compute(Stage<0>{});
        stash(1, 0);
        __syncthreads();
        read_ops(1, 0, ops[0]);
        fetch(c + 3, 0);                                                     // set 0 <- chunk c+3; set 1 holds chunk c+2
        compute(Stage<1>{});
        stash(0, 1);
        __syncthreads();
        read_ops(0, 0, ops[0]);
    }
    if constexpr (CARRY) fold((FKG - 1) & 1, 0, FKG - 1, 0, 1);

    // ---- epilogue: for sub-tiles (i, j) the lane holds row m = 32*j + l32 and, per register quad r4, columns
    // n = 8*r4 + 4*lhi + 0..3
    TO* out = reinterpret_cast<TO*>(outptr);
    const bool vec_out = p.ldo % 4 == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0;
    const bool vec_aux = p.n % 4 == 0 && (reinterpret_cast<uintptr_t>(p.aux) & 15) == 0;
#pragma unroll
    for (int j = 0; j < TM; ++j) {
        const int64_t mrow = m_begin + a_sub(j) + l32;
        if (mrow >= m_end) continue;
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) {
            const int64_t ncol = n_begin + wn * 32 + r4 * 8 + lhi * 4;
            if (ncol >= p.n) continue;
            const bool full = ncol + 3 < p.n;
            if constexpr (GATED) {
                TO* aux = static_cast<TO*>(p.aux);
                float gq[4], uq[4], h[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float gv = total[0][j][r4 * 4 + e], uv = total[1][j][r4 * 4 + e];
                    if (p.bias && ncol + e < p.n) {
                        gv += load_bias(p.bias, ncol + e, bias_dtype);
                        uv += load_bias(p.bias, p.n + ncol + e, bias_dtype);
                    }
                    gq[e] = rounded<TO>(gv);
                    uq[e] = rounded<TO>(uv);
                    float act, derivative;
                    gate_math(p.activation, gq[e], act, derivative);
                    h[e] = act * uq[e];
                }
                if (full && vec_out) Quad<TO>::store(out + mrow * p.ldo + ncol, h);
                else for (int e = 0; e < 4; ++e) if (ncol + e < p.n) out[mrow * p.ldo + ncol + e] = from_f32<TO>(h[e]);
                if (aux) {
                    if (full && vec_aux) {
                        Quad<TO>::store(aux + mrow * 2 * p.n + ncol, gq);
                        Quad<TO>::store(aux + mrow * 2 * p.n + p.n + ncol, uq);
                    } else {
                        for (int e = 0; e < 4; ++e)
                            if (ncol + e < p.n) {
                                aux[mrow * 2 * p.n + ncol + e] = from_f32<TO>(gq[e]);
                                aux[mrow * 2 * p.n + p.n + ncol + e] = from_f32<TO>(uq[e]);
                            }
                    }
                }
            } else {
                float v[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = total[0][j][r4 * 4 + e];
                if constexpr (MODE == MODE_PLAIN) {
                    if (p.bias) {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (ncol + e < p.n) v[e] += load_bias(p.bias, ncol + e, bias_dtype);
                    }
                    if (full && vec_out) Quad<TO>::store(out + mrow * p.ldo + ncol, v);
                    else for (int e = 0; e < 4; ++e) if (ncol + e < p.n) out[mrow * p.ldo + ncol + e] = from_f32<TO>(v[e]);
                } else {
                    const TO* aux = static_cast<const TO*>(p.aux);
                    float g[4] = {0, 0, 0, 0}, u[4] = {0, 0, 0, 0}, dg[4], du[4];
                    if (full && vec_aux) {
                        Quad<TO>::load(aux + mrow * 2 * p.n + ncol, g);
                        Quad<TO>::load(aux + mrow * 2 * p.n + p.n + ncol, u);
                    } else {
                        for (int e = 0; e < 4; ++e)
                            if (ncol + e < p.n) {
                                g[e] = to_f32(aux[mrow * 2 * p.n + ncol + e]);
                                u[e] = to_f32(aux[mrow * 2 * p.n + p.n + ncol + e]);
                            }
                    }
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float d = rounded<TO>(v[e]);
                        float act, derivative;
                        gate_math(p.activation, g[e], act, derivative);
                        dg[e] = d * u[e] * derivative;
                        du[e] = d * act;
                    }
                    if (full && vec_out && vec_aux) {
                        Quad<TO>::store(out + mrow * p.ldo + ncol, dg);
                        Quad<TO>::store(out + mrow * p.ldo + p.n + ncol, du);
                    } else {
                        for (int e = 0; e < 4; ++e)
                            if (ncol + e < p.n) {
                                out[mrow * p.ldo + ncol + e] = from_f32<TO>(dg[e]);
                                out[mrow * p.ldo + p.n + ncol + e] = from_f32<TO>(du[e]);
                            }
                    }
                }
            }
        }
    }
}

#ifndef VIOLA_GEMM_PROBE   // a probe build instantiates single kernels itself
template <int MODE, bool B_ROWSCALE, typename TO>
static void launch_formats(const GemmArgs& p, int a_dtype, int b_dtype, int bias_dtype, dim3 grid, hipStream_t stream) {
    const bool a5 = a_dtype == VIOLA_E5M2, b5 = b_dtype == VIOLA_E5M2;
    if (!a5 && !b5) hipLaunchKernelGGL((group_gemm_fast<MODE, false, false, B_ROWSCALE, TO>), grid, dim3(FTHREADS), 0, stream, p, bias_dtype);
    else if (a5 && !b5) hipLaunchKernelGGL((group_gemm_fast<MODE, true, false, B_ROWSCALE, TO>), grid, dim3(FTHREADS), 0, stream, p, bias_dtype);
    else if (!a5 && b5) hipLaunchKernelGGL((group_gemm_fast<MODE, false, true, B_ROWSCALE, TO>), grid, dim3(FTHREADS), 0, stream, p, bias_dtype);
    else hipLaunchKernelGGL((group_gemm_fast<MODE, true, true, B_ROWSCALE, TO>), grid, dim3(FTHREADS), 0, stream, p, bias_dtype);
}

template <int MODE>
static int launch_mode(const GemmArgs& p, int a_dtype, int b_dtype, int bias_dtype, int out_dtype, bool rowscale, dim3 grid,
                       hipStream_t stream) {
#define VIOLA_FAST(TO)                                                                       \
    if (rowscale) launch_formats<MODE, true, TO>(p, a_dtype, b_dtype, bias_dtype, grid, stream); \
    else launch_formats<MODE, false, TO>(p, a_dtype, b_dtype, bias_dtype, grid, stream);
    switch (out_dtype) {
        case VIOLA_F32: VIOLA_FAST(float) break;
        case VIOLA_BF16: VIOLA_FAST(bf16_t) break;
        case VIOLA_F16: VIOLA_FAST(f16_t) break;
        default: return VIOLA_EINVAL;
    }
#undef VIOLA_FAST
    return viola_launch_status();
}

int launch_group_gemm_fast(const GemmArgs& args, int mode, int a_dtype, int b_dtype, int bias_dtype, int out_dtype, bool rowscale,
                           dim3 grid, hipStream_t stream) {
    GemmArgs p = args;
    if (!p.offsets && (int64_t)grid.x * grid.y < (1 << 30)) {
        p.tiles_n = (int)grid.x;
        p.tiles_m = (int)grid.y;
        grid = dim3((grid.x * grid.y + 7) / 8 * 8, 1, grid.z);
    }
    if (mode == MODE_PLAIN) return launch_mode<MODE_PLAIN>(p, a_dtype, b_dtype, bias_dtype, out_dtype, rowscale, grid, stream);
    if (mode == MODE_GATED_FWD) return launch_mode<MODE_GATED_FWD>(p, a_dtype, b_dtype, bias_dtype, out_dtype, rowscale, grid, stream);
    return launch_mode<MODE_GATED_BWD>(p, a_dtype, b_dtype, bias_dtype, out_dtype, rowscale, grid, stream);
}
#endif

}  // namespace viola
