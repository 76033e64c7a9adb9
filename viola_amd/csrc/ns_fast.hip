// Tiled Newton-Schulz GEMM for gfx950: batched out[b] = a[b] . b[b]^T (b as [n, k]) or a[b] . b[b] (b as
// [k, n]) in bf16 / fp16 on v_mfma_f32_32x32x16, fp32 accumulation, with the chain's epilogues.
//
// Block: WAVES_M x WAVES_N wavefronts, each owning WM x WN accumulators of 32 x 32. Three shapes are built:
// 2 x 2 waves of 3 x 3 (192 x 192 tiles for the 1152-multiples of transformer blocks) or of 2 x 2 (128 x 128), two
// blocks per CU so one block's barrier and LDS traffic hide behind the other's MFMAs; and 4 x 2 waves of 3 x 3
// (384 x 192, 64 k per stage, one block per CU) for large non-symmetric products.
//   * global -> LDS directly (buffer_load_dwordx4 ... lds: no staging registers, no ds_write; lanes
//     past the matrix read zero, so there are no tail branches), a ring of STAGES stages of SBK k: the
//     loads of the next STAGES - 1 chunks are in flight during the math of a chunk, one barrier per chunk.
//     A direct load puts lane l's 16 bytes at base + 16 l, so the tile layout is chosen on the global
//     side: which (row, k piece) a lane fetches.
//   * k-contiguous operands ([m, k] and [n, k]) are rows of 4 (or 8) x 16 bytes with piece c of row r stored in
//     slot c ^ ((r >> 2) & 3) (or c ^ ((r >> 1) & 7)): the 16 rows a ds_read_b128 group touches fall in 16 different bank
//     groups. An [k, n] operand keeps its layout (rows of BN elements, 16-byte units XOR-swizzled by
//     the row so four consecutive k rows start 64 bytes apart in bank space) and is transposed on the
//     way out of LDS by ds_read_b64_tr_b16, which hands lane i of each 16-lane group the four k values
//     of column i.
//   * the b matrix is the MFMA "A" source, so a lane owns one output row m and runs of four
//     consecutive n: 8-byte stores, per-row residual loads.
//   * a Gram-type product (b == a, square output) computes only the tiles on and above the diagonal and
//     stores each off-diagonal tile a second time transposed, its epilogue applied with the residual of the
//     transposed position (exact for any residual); transpose_out stores [n, m] only. Both placements leave
//     LDS as 16-byte pieces.
//   * work order: the 1-D grid is cut into eight contiguous ranges, one per XCD (blockIdx % 8), and
//     inside a range tiles walk n fastest, so the tiles that share an a panel meet in one L2.
#include "ns_args.hpp"

namespace viola {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;

constexpr uint32_t NS_OUTSIDE = 0x80000000u;
#ifndef NS_FILL
#define NS_FILL 200                                            // blocks that count as one per compute unit (256 units)
#endif
#ifndef NS_SMALL_SBK
#define NS_SMALL_SBK 64
#define NS_SMALL_STAGES 4
#endif

template <bool IS_BF16>
__device__ __forceinline__ f32x16 ns_mfma(uint4 x, uint4 y, f32x16 c) {
    if constexpr (IS_BF16) return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, x), __builtin_bit_cast(bf16x8, y), c, 0, 0, 0);
    else return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, x), __builtin_bit_cast(f16x8, y), c, 0, 0, 0);
}
template <bool IS_BF16> __device__ __forceinline__ float ns_widen(uint16_t bits) {
    if constexpr (IS_BF16) return bf16_bits_to_f32(bits);
    else { _Float16 h; __builtin_memcpy(&h, &bits, 2); return (float)h; }
}
template <bool IS_BF16> __device__ __forceinline__ uint16_t ns_narrow(float v) {
    if constexpr (IS_BF16) return f32_to_bf16_bits(v);
    else { _Float16 h = (_Float16)v; uint16_t bits; __builtin_memcpy(&bits, &h, 2); return bits; }
}
// the same conversions on two neighbouring elements packed in 32 bits (low half first)
typedef _Float16 ns_f16x2 __attribute__((ext_vector_type(2)));
typedef float ns_f32x2 __attribute__((ext_vector_type(2)));
template <bool IS_BF16> __device__ __forceinline__ void ns_widen2(uint32_t pair, float& lo, float& hi) {
    if constexpr (IS_BF16) { lo = __uint_as_float(pair << 16); hi = __uint_as_float(pair & 0xffff0000u); }
    else { const ns_f16x2 h = __builtin_bit_cast(ns_f16x2, pair); lo = (float)h.x; hi = (float)h.y; }
}
template <bool IS_BF16> __device__ __forceinline__ uint32_t ns_narrow2(float lo, float hi) {
    if constexpr (IS_BF16) return f32_to_bf16x2_bits(lo, hi);
    else { const ns_f32x2 pair = {lo, hi}; return __builtin_bit_cast(uint32_t, __builtin_convertvector(pair, ns_f16x2)); }
}

// 64 lanes x 16 bytes from a raw buffer straight into LDS at lds_addr + 16 * lane. The compiler is
// not told that this touches LDS (it would drain every outstanding load before each LDS read); the
// kernel orders it against its LDS reads with s_waitcnt vmcnt + barrier itself.
__device__ __forceinline__ void load_to_lds(i32x4 rsrc, uint32_t lds_addr, uint32_t voffset, uint32_t soffset) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :: "s"(lds_addr), "v"(voffset), "s"(rsrc), "s"(soffset) : "memory");
}
__device__ __forceinline__ i32x4 make_rsrc(const void* base) {
    const uint64_t address = reinterpret_cast<uint64_t>(base);
    i32x4 r = {__builtin_amdgcn_readfirstlane((int)(uint32_t)address), __builtin_amdgcn_readfirstlane((int)(uint32_t)(address >> 32)),
               0x7fffffff, 0x00020000};
    return r;
}

// Which output tile a block works on. The blocks of an XCD take a contiguous range of `work` numbers; inside a matrix the
// numbers walk the tile grid in bands of p.group_m tile rows, column by column inside a band (rows fastest), so that
// the tiles in flight on one XCD share p.group_m panels of a and a few panels of b and its L2 holds them. A Gram
// product walks the tiles on and above the diagonal in the same banded order.
__device__ __forceinline__ void ns_tile_of(const NsArgs& p, int64_t work, int& tm, int& tn, int64_t& bz) {
    const int band = p.group_m;
    if (p.symmetric) {
        const int t = p.tiles_n;
        const int64_t upper = (int64_t)t * (t + 1) / 2;
        bz = work / upper;
        int rest = (int)(work % upper);
        int first = 0;
        for (;;) {                                               // the band: rows first .. first + rows - 1, columns first .. t - 1
            const int rows = t - first < band ? t - first : band;
            const int in_band = rows * (t - first) - rows * (rows - 1) / 2;
            if (rest < in_band) break;
            rest -= in_band;
            first += rows;
        }
        const int rows = t - first < band ? t - first : band;
        int col = first;
        for (;;) {                                               // column col holds rows first .. min(col, first + rows - 1)
            const int here = col - first + 1 < rows ? col - first + 1 : rows;
            if (rest < here) break;
            rest -= here;
            ++col;
        }
        tm = first + rest;
        tn = col;
    } else {
        const int64_t per = (int64_t)p.tiles_n * p.tiles_m;
        bz = work / per;
        const int t = (int)(work % per);
        const int group = band * p.tiles_n;
        const int first = t / group * band;
        const int rows = p.tiles_m - first < band ? p.tiles_m - first : band;
        tm = first + t % group % rows;
        tn = t % group / rows;
    }
    // the coordinates come out of divisions the compiler carries in vector registers; pin them to scalars so
    // everything derived from them (buffer resources, LDS bases) is wave-uniform
    tm = __builtin_amdgcn_readfirstlane(tm);
    tn = __builtin_amdgcn_readfirstlane(tn);
    bz = __builtin_amdgcn_readfirstlane((int)bz);
}

// Band height for ns_tile_of: an XCD works on about an eighth of the tiles at a time (of one matrix at most); a band of
// g rows by w columns with g w = that many tiles touches g panels of a and w of b, least when g : w = their sizes.
static int ns_band(const NsArgs& p, int bm, int bn) {
#ifdef NS_BAND
    return NS_BAND;
#endif
    const int64_t own = p.symmetric ? (int64_t)p.tiles_n * (p.tiles_n + 1) / 2 : (int64_t)p.tiles_m * p.tiles_n;
    const int64_t share = p.tiles / 8 < own ? (p.tiles / 8 > 0 ? p.tiles / 8 : 1) : own;
    int band = 1;
    while ((int64_t)(band + 1) * (band + 1) * bm <= share * bn) ++band;
    const int rows = p.symmetric ? p.tiles_n : p.tiles_m;
    return band < rows ? band : rows;
}

// Shape: WAVES_M x WAVES_N wavefronts of WM x WN accumulators; SBK k per stage, STAGES stages (loads run
// STAGES - 1 chunks ahead). Small: 2 x 2 waves, 32 k, 3 stages, two blocks per CU. Big: 4 x 2 waves of 3 x 3
// (384 x 192), 64 k (whole 128-byte lines per row and load), 2 stages, one block per CU.
template <int WAVES_M, int WAVES_N> struct NsThreads { static constexpr int value = 64 * WAVES_M * WAVES_N; };

template <bool IS_BF16, bool B_KN, int EPILOGUE, int WM, int WN, int WAVES_M, int WAVES_N, int SBK, int STAGES>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N, 2) void ns_gemm_fast(NsArgs p) {
    constexpr int THREADS = 64 * WAVES_M * WAVES_N;
    constexpr int BM = 32 * WM * WAVES_M, BN = 32 * WN * WAVES_N;
    constexpr int A_EL = BM * SBK, B_EL = BN * SBK, STAGE_EL = A_EL + B_EL;
    constexpr int NCH = BN / 8;                                      // 16-byte units per [k, n] row
    constexpr int UPR = SBK / 8;                                     // 16-byte units per k-contiguous row
    constexpr int A_LOADS = BM * UPR / THREADS, B_LOADS = BN * UPR / THREADS;   // = SBK * NCH / THREADS for [k, n]
    static_assert(BM * UPR % THREADS == 0 && BN * UPR % THREADS == 0, "whole load instructions");
    __shared__ __attribute__((aligned(1024))) uint16_t lds[STAGES * STAGE_EL];
    // slot of piece c in row r: c ^ swz(r); 16 consecutive rows reading the same piece then cover all 16 bank groups
    auto swz = [](int r) -> int { return UPR == 4 ? (r >> 2) & 3 : (r >> 1) & 7; };

    const int64_t per_xcd = (p.tiles + 7) / 8;
    const int64_t seq = blockIdx.x / 8;
    const int64_t work = (int64_t)(blockIdx.x % 8) * per_xcd + seq;
    if (work >= p.tiles) return;
    int tm, tn;
    int64_t bz;
    ns_tile_of(p, work, tm, tn, bz);
    const bool mirror = p.symmetric && tn != tm;
    const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * BN;
    const int64_t m = p.m, n = p.n, k = p.k;

    const int tid = threadIdx.x, lane = tid % WAVE;
    const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
    const int wm = wave / WAVES_N, wn = wave % WAVES_N, l32 = lane % 32, lhi = lane / 32;

    const i32x4 res_a = make_rsrc(p.a + bz * m * k);
    const i32x4 res_b = make_rsrc(p.b + bz * n * k);

    // Load plan: instruction `it` of this wave fills LDS units (16 bytes) [it * THREADS + wave * 64, +64);
    // per thread: the global byte offset (k0 = 0) of the piece that belongs in its unit, and its k position.
    uint32_t a_off[A_LOADS], b_off[B_LOADS];
    int a_k[A_LOADS], b_k[B_LOADS];
#pragma unroll
    for (int it = 0; it < A_LOADS; ++it) {
        const int u = it * THREADS + tid, lr = u / UPR, c = (u % UPR) ^ swz(lr);
        const int64_t row = m0 + lr;
        a_off[it] = row < m ? (uint32_t)((row * k + c * 8) * 2) : NS_OUTSIDE;
        a_k[it] = c * 8;
    }
#pragma unroll
    for (int it = 0; it < B_LOADS; ++it) {
        const int u = it * THREADS + tid;
        if constexpr (B_KN) {
            const int kr = u / NCH, pos = u % NCH;
            const int unit = pos ^ (BN % 128 == 0 ? (kr & 3) * 4 : ((kr >> 1) & 1) * 4);
            const int64_t col = n0 + unit * 8;
            b_off[it] = col < n ? (uint32_t)(((int64_t)kr * n + col) * 2) : NS_OUTSIDE;
            b_k[it] = kr;
        } else {
            const int lr = u / UPR, c = (u % UPR) ^ swz(lr);
            const int64_t row = n0 + lr;
            b_off[it] = row < n ? (uint32_t)((row * k + c * 8) * 2) : NS_OUTSIDE;
            b_k[it] = c * 8;
        }
    }
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint16_t*)lds;
    const uint32_t wave_units = (uint32_t)wave * 64 * 16;             // byte offset of this wave's 64 units
    auto issue = [&](int64_t k0, int stage) {
        const uint32_t a_step = (uint32_t)(k0 * 2);
        const uint32_t b_step = B_KN ? (uint32_t)(k0 * n * 2) : (uint32_t)(k0 * 2);
        const uint32_t base = lds_base + (uint32_t)stage * STAGE_EL * 2 + wave_units;
#pragma unroll
        for (int it = 0; it < A_LOADS; ++it)
            load_to_lds(res_a, base + it * THREADS * 16, k0 + a_k[it] < k ? a_off[it] : NS_OUTSIDE, a_step);
#pragma unroll
        for (int it = 0; it < B_LOADS; ++it)
            load_to_lds(res_b, base + A_EL * 2 + it * THREADS * 16, k0 + b_k[it] < k ? b_off[it] : NS_OUTSIDE, b_step);
    };

    // fragment addresses (elements) inside a stage
    const int sw = swz(l32);
    const int a_frag = (wm * 32 * WM + l32) * SBK + ((lhi ^ sw) * 8);                  // k half ks: ^ (ks * 16)
    const int kn_row = lhi * 8 + ((lane & 15) >> 2);                                   // + ks * 16 (+ 4 for the upper half)
    const int kn_unit = (wn * 4 * WN + 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1)) ^ (BN % 128 == 0 ? (kn_row & 3) * 4 : ((kn_row >> 1) & 1) * 4);
    const int b_frag = B_KN ? A_EL + kn_row * BN + kn_unit * 8 + 4 * (lane & 1)
                            : A_EL + (wn * 32 * WN + l32) * SBK + ((lhi ^ sw) * 8);

    f32x16 acc[WN][WM];
#pragma unroll
    for (int i = 0; i < WN; ++i)
#pragma unroll
        for (int j = 0; j < WM; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    auto compute = [&](const uint16_t* stage) {
#pragma unroll
        for (int ks = 0; ks < SBK / 16; ++ks) {
            uint4 opa[WM], opb[WN];
#pragma unroll
            for (int i = 0; i < WN; ++i) {
                if constexpr (B_KN) {
                    // i * 32 columns = 4 units further along the row: the swizzle only touches bits the
                    // lane's own term already fixed modulo 8 units when 4 i stays below 8, so add it before
                    // the XOR would be wrong; the unit index is rebuilt instead
                    const int unit = ((wn * 4 * WN + i * 4 + 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1)) ^ (BN % 128 == 0 ? (kn_row & 3) * 4 : ((kn_row >> 1) & 1) * 4));
                    const uint16_t* at = stage + A_EL + (kn_row + ks * 16) * BN + unit * 8 + 4 * (lane & 1);
                    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)at);
                    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(at + 4 * BN));
                    const uint2 l2 = __builtin_bit_cast(uint2, lo), h2 = __builtin_bit_cast(uint2, hi);
                    opb[i] = make_uint4(l2.x, l2.y, h2.x, h2.y);
                } else {
                    opb[i] = *reinterpret_cast<const uint4*>(stage + ((b_frag + i * 32 * SBK) ^ (ks * 16)));
                }
            }
#pragma unroll
            for (int j = 0; j < WM; ++j) opa[j] = *reinterpret_cast<const uint4*>(stage + ((a_frag + j * 32 * SBK) ^ (ks * 16)));
#pragma unroll
            for (int i = 0; i < WN; ++i)
#pragma unroll
                for (int j = 0; j < WM; ++j) acc[i][j] = ns_mfma<IS_BF16>(opb[i], opa[j], acc[i][j]);
        }
    };

    const int64_t chunks = (k + SBK - 1) / SBK;
    constexpr int AHEAD = STAGES - 1;                                   // chunks in flight beyond the one being multiplied
#pragma unroll
    for (int c = 0; c < AHEAD; ++c) issue((int64_t)c * SBK, c);
    int cur = 0, fill = AHEAD;
    for (int64_t c = 0; c < chunks; ++c) {
        // all loads but those of the newest AHEAD - 1 chunks have landed: chunk c is in LDS for this wave ...
        constexpr int IN_FLIGHT = (AHEAD - 1) * (A_LOADS + B_LOADS);  // vmcnt: low four bits, two more in bits 14..15
        static_assert(IN_FLIGHT < 64, "the count fits the wait instruction");
        __builtin_amdgcn_s_waitcnt(0x0F70 | (IN_FLIGHT & 15) | ((IN_FLIGHT >> 4) << 14));
        __syncthreads();                    // ... and for every wave; stage `fill` was last read in chunk c-1
        issue((c + AHEAD) * SBK, fill);     // past the end: zeros into a stage nobody reads
        compute(lds + cur * STAGE_EL);
        cur = cur == STAGES - 1 ? 0 : cur + 1;
        fill = fill == STAGES - 1 ? 0 : fill + 1;
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);     // drain the trailing loads before the LDS allocation is released

    // Element offsets inside one matrix fit 32 bits (the launcher checks it): the pieces below are addressed as a
    // per-matrix base, the same for every lane, plus a 32-bit byte offset.
    const uint16_t* residual = EPILOGUE ? p.residual + bz * m * n : nullptr;
    uint16_t* out = p.out + bz * m * n;
    uint16_t* out_diag = p.out_diag ? p.out_diag + bz * m * n : nullptr;
    const uint32_t um = (uint32_t)m, un = (uint32_t)n;
    auto load_piece = [](const uint16_t* base, uint32_t element) -> uint4 {
        return *reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(base) + (size_t)(element * 2u));
    };
    auto store_piece = [](uint16_t* base, uint32_t element, uint4 piece) {
        *reinterpret_cast<uint4*>(reinterpret_cast<char*>(base) + (size_t)(element * 2u)) = piece;
    };
    // The accumulators hold one row per lane in runs of four columns, which as stores would touch 32 cache lines per
    // instruction. Each wavefront instead parks its rounded products, 32 rows at a time, in LDS (the stage ring is free
    // now) and picks them up as 16-byte pieces: along the rows for the [m, n] placement, so that the residual loads, the
    // epilogue arithmetic and the stores all run on 8 consecutive columns of one row, and down the columns for the
    // [n, m] placement (the mirrored copy of an off-diagonal Gram tile, or a transposed result), 8 consecutive m of one n.
    constexpr int WCOLS = 32 * WN, PLD = WCOLS + 8, PIECES = WCOLS / 8;       // parked row: 16 bytes of padding
    static_assert(WAVES_M * WAVES_N * 32 * PLD * 2 <= (int)sizeof(lds), "parking area fits in the stage ring");
    __syncthreads();                                                      // every wave has left the ring
    uint16_t* park = lds + wave * 32 * PLD;
    // two neighbouring elements at a time: the rounded products and the residual as packed pairs in, the result pair out
    auto finish = [&](uint32_t products, uint32_t residuals) -> uint32_t {
        if (EPILOGUE == 0) return products;                               // widening and narrowing a rounded value again changes nothing
        float v0, v1, r0, r1;
        ns_widen2<IS_BF16>(products, v0, v1);
        ns_widen2<IS_BF16>(residuals, r0, r1);
        if (EPILOGUE == 1) { v0 = -4.7750f * r0 + 2.0315f * v0; v1 = -4.7750f * r1 + 2.0315f * v1; }
        if (EPILOGUE == 2) { v0 = v0 + 3.4445f * r0; v1 = v1 + 3.4445f * r1; }
        return ns_narrow2<IS_BF16>(v0, v1);
    };
    // the second copy: element `at` of the piece (the one on the diagonal) gets add_diag
    auto with_diagonal = [&](uint4 piece, uint32_t at) -> uint4 {
        uint32_t w[4] = {piece.x, piece.y, piece.z, piece.w};
#pragma unroll
        for (int e = 0; e < 8; ++e)
            if (at == (uint32_t)e) {
                const uint32_t bits = ns_narrow<IS_BF16>(ns_widen<IS_BF16>((uint16_t)(w[e / 2] >> (16 * (e % 2)))) + p.add_diag);
                w[e / 2] = (w[e / 2] & ~(0xffffu << (16 * (e % 2)))) | (bits << (16 * (e % 2)));
            }
        return make_uint4(w[0], w[1], w[2], w[3]);
    };
    // The residual pieces of the [m, n] placement are fetched one 32-row block ahead: the loads of block j + 1 leave
    // before block j is finished and stored, so that a wavefront waits for memory once per block and not once per piece.
    constexpr int ROW_ITERS = 32 * PIECES / WAVE;
    uint4 ahead[2][ROW_ITERS];
    const uint32_t tile_row = (uint32_t)m0 + wm * 32 * WM, col0 = (uint32_t)n0 + wn * WCOLS;
    auto fetch_residual = [&](int j, uint4 (&pieces)[ROW_ITERS]) {
#pragma unroll
        for (int it = 0; it < ROW_ITERS; ++it) {
            const int id = it * WAVE + lane, pr = id / PIECES, pc = id % PIECES;
            const uint32_t row = tile_row + j * 32 + pr, col = col0 + pc * 8;
            // a piece outside the matrix reads the first one instead (its value is not used)
            pieces[it] = load_piece(residual, row < um && col < un ? row * un + col : 0u);
        }
    };
    if (EPILOGUE && !p.transpose_out) fetch_residual(0, ahead[0]);
#pragma unroll
    for (int j = 0; j < WM; ++j) {
#pragma unroll
        for (int i = 0; i < WN; ++i)
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4)
                *reinterpret_cast<uint2*>(&park[l32 * PLD + i * 32 + r4 * 8 + lhi * 4]) =
                    make_uint2(ns_narrow2<IS_BF16>(acc[i][j][r4 * 4], acc[i][j][r4 * 4 + 1]), ns_narrow2<IS_BF16>(acc[i][j][r4 * 4 + 2], acc[i][j][r4 * 4 + 3]));
        const uint32_t row0 = tile_row + j * 32;                          // of the parked 32 x WCOLS block
        if (!p.transpose_out) {
            if (EPILOGUE && j + 1 < WM) fetch_residual(j + 1, ahead[(j + 1) & 1]);
#pragma unroll
            for (int it = 0; it < ROW_ITERS; ++it) {
                const int id = it * WAVE + lane, pr = id / PIECES, pc = id % PIECES;
                const uint32_t row = row0 + pr, col = col0 + pc * 8;
                const uint4 raw = *reinterpret_cast<const uint4*>(&park[pr * PLD + pc * 8]);
                if (row >= um || col >= un) continue;                     // n is a multiple of 8: whole pieces
                const uint4 res = EPILOGUE ? ahead[j & 1][it] : make_uint4(0, 0, 0, 0);
                const uint4 o = make_uint4(finish(raw.x, res.x), finish(raw.y, res.y), finish(raw.z, res.z), finish(raw.w, res.w));
                store_piece(out, row * un + col, o);
                if (out_diag) store_piece(out_diag, row * un + col, row - col < 8u ? with_diagonal(o, row - col) : o);
            }
        }
        if (p.transpose_out || mirror) {
            // element [n, m] of the placement has the product parked at [m][n]. A mirrored element takes the residual of
            // its own position (a . a^T is symmetric, its residual need not be; an off-diagonal tile holds no diagonal
            // element), a transposed result the residual of the position it was computed for.
            const bool whole = m % 8 == 0;
#pragma unroll 1
            for (int it = 0; it < WCOLS * 4 / WAVE; ++it) {                   // not unrolled: the accumulators of the later j are still live
                const int id = it * WAVE + lane, ln = id / 4, lm = id % 4 * 8;
                const uint32_t orow = col0 + ln, ocol = row0 + lm;        // row and first column in the [n, m] placement
                uint32_t pw[4];
#pragma unroll
                for (int e = 0; e < 8; e += 2) pw[e / 2] = (uint32_t)park[(lm + e) * PLD + ln] | ((uint32_t)park[(lm + e + 1) * PLD + ln] << 16);
                if (orow >= un || ocol >= um) continue;
                uint32_t rw[4] = {0, 0, 0, 0};
                if (EPILOGUE && mirror) {                                 // m == n, a multiple of 8: a whole piece of residual row orow
                    const uint4 res = load_piece(residual, orow * un + ocol);
                    rw[0] = res.x; rw[1] = res.y; rw[2] = res.z; rw[3] = res.w;
                } else if (EPILOGUE) {
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        if (ocol + e < um) rw[e / 2] |= (uint32_t)residual[(size_t)((ocol + e) * un + orow)] << (16 * (e % 2));
                }
                uint4 o = make_uint4(finish(pw[0], rw[0]), finish(pw[1], rw[1]), finish(pw[2], rw[2]), finish(pw[3], rw[3]));
                const uint4 od = !mirror && orow - ocol < 8u ? with_diagonal(o, orow - ocol) : o;
                if (whole) {
                    store_piece(out, orow * um + ocol, o);
                    if (out_diag) store_piece(out_diag, orow * um + ocol, od);
                } else {
                    const uint32_t ow[4] = {o.x, o.y, o.z, o.w}, dw[4] = {od.x, od.y, od.z, od.w};
                    for (int e = 0; e < 8 && ocol + e < um; ++e) {
                        out[(size_t)(orow * um + ocol + e)] = (uint16_t)(ow[e / 2] >> (16 * (e % 2)));
                        if (out_diag) out_diag[(size_t)(orow * um + ocol + e)] = (uint16_t)(dw[e / 2] >> (16 * (e % 2)));
                    }
                }
            }
        }
    }
}

template <bool IS_BF16, bool B_KN, int WM, int WN, int WAVES_M, int WAVES_N, int SBK, int STAGES>
static void launch_tiles(NsArgs p, int epilogue, hipStream_t stream) {
    constexpr int BM = 32 * WM * WAVES_M, BN = 32 * WN * WAVES_N, THREADS = 64 * WAVES_M * WAVES_N;
    p.tiles_m = (int)((p.m + BM - 1) / BM);
    p.tiles_n = (int)((p.n + BN - 1) / BN);
    p.tiles = p.batch * (p.symmetric ? (int64_t)p.tiles_n * (p.tiles_n + 1) / 2 : (int64_t)p.tiles_m * p.tiles_n);
    p.group_m = ns_band(p, BM, BN);
    const unsigned grid = (unsigned)((p.tiles + 7) / 8 * 8);
    if (epilogue == 0) VIOLA_LAUNCH((ns_gemm_fast<IS_BF16, B_KN, 0, WM, WN, WAVES_M, WAVES_N, SBK, STAGES>), dim3(grid), dim3(THREADS), 0, stream, p);
    else if (epilogue == 1) VIOLA_LAUNCH((ns_gemm_fast<IS_BF16, B_KN, 1, WM, WN, WAVES_M, WAVES_N, SBK, STAGES>), dim3(grid), dim3(THREADS), 0, stream, p);
    else VIOLA_LAUNCH((ns_gemm_fast<IS_BF16, B_KN, 2, WM, WN, WAVES_M, WAVES_N, SBK, STAGES>), dim3(grid), dim3(THREADS), 0, stream, p);
}

// Which tile shape a product runs on. Every shape of ns_gemm_fast gives an output element the same arithmetic (k walked
// in steps of 16 into one FP32 accumulator, rounded once), so the choice is about filling the GPU only and may look at
// the batch.
NsTile ns_choose_tile(int64_t batch, int64_t m, int64_t n, bool symmetric) {
    auto area = [&](int64_t tm, int64_t tn) { return ((m + tm - 1) / tm) * ((n + tn - 1) / tn) * tm * tn; };
    auto blocks = [&](int64_t tm, int64_t tn) {
        const int64_t rows = (m + tm - 1) / tm, cols = (n + tn - 1) / tn;
        return batch * (symmetric ? cols * (cols + 1) / 2 : rows * cols);
    };
    // 192-wide tiles move a third less operand data per flop; take them unless their padding costs more
    // than that (1152 = 6 x 192 and its multiples fit exactly)
    const bool wide = area(192, 192) * 20 <= area(128, 128) * 21 && blocks(192, 192) >= NS_FILL;
    // 384 x 192 blocks with whole-line loads when they fit as well as the 192s and still give every CU a few tiles
    // (a Gram product keeps square tiles for its mirrored stores)
    const bool big = wide && !symmetric && area(384, 192) <= area(192, 192) && blocks(384, 192) >= 3 * 256;
    if (big) return NS_TILE_384x192;
    if (wide) return NS_TILE_192x192;
    if (blocks(128, 128) >= NS_FILL) return NS_TILE_128x128;
    // fewer 128 x 128 tiles than compute units (one matrix of a thousand rows): smaller tiles put more of the chip to work
    if (!symmetric && blocks(128, 64) >= NS_FILL) return NS_TILE_128x64;
    return NS_TILE_64x64;
}

template <bool IS_BF16, bool B_KN>
static void launch_shape(const NsArgs& p, int epilogue, hipStream_t stream) {
    switch (ns_choose_tile(p.batch, p.m, p.n, p.symmetric != 0)) {
        case NS_TILE_384x192: launch_tiles<IS_BF16, B_KN, 3, 3, 4, 2, 64, 2>(p, epilogue, stream); break;
        case NS_TILE_192x192: launch_tiles<IS_BF16, B_KN, 3, 3, 2, 2, 32, 3>(p, epilogue, stream); break;
        case NS_TILE_128x128: launch_tiles<IS_BF16, B_KN, 2, 2, 2, 2, 32, 3>(p, epilogue, stream); break;
        case NS_TILE_128x64: launch_tiles<IS_BF16, B_KN, 2, 1, 2, 2, 32, 3>(p, epilogue, stream); break;
        default: launch_tiles<IS_BF16, B_KN, 1, 1, 2, 2, NS_SMALL_SBK, NS_SMALL_STAGES>(p, epilogue, stream); break;
    }
}

bool ns_fast_takes(const NsArgs& p) {
    auto aligned = [](const void* q) { return reinterpret_cast<uintptr_t>(q) % 16 == 0; };
    if (p.k % 8 || p.n % 8 || p.k == 0) return false;
    if (!aligned(p.a) || !aligned(p.b) || !aligned(p.out) || !aligned(p.residual) || !aligned(p.out_diag)) return false;
    const int64_t limit = (1ll << 31) - 65536;
    if (p.m * p.k * 2 >= limit || p.n * p.k * 2 >= limit || p.m * p.n * 2 >= limit) return false;
    if (p.batch * ((p.m + 127) / 128) * ((p.n + 127) / 128) >= (1ll << 31) - 8) return false;
    return true;
}

bool launch_ns_gemm_fast(const NsArgs& p, bool is_bf16, bool b_kn, int epilogue, hipStream_t stream) {
    if (!ns_fast_takes(p)) return false;
    if (is_bf16) { if (b_kn) launch_shape<true, true>(p, epilogue, stream); else launch_shape<true, false>(p, epilogue, stream); }
    else { if (b_kn) launch_shape<false, true>(p, epilogue, stream); else launch_shape<false, false>(p, epilogue, stream); }
    return true;
}

}  // namespace viola
