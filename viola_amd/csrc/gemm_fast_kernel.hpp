// Fast path of the FP8 GEMMs for gfx950: the kernel template (see gemm.hip for the contract and the operand
// orientation; gemm_fast.hip, gemm_fast_tensor.hip and gemm_fast_mx.hip instantiate it per scaling recipe). Requires 16-byte aligned operand rows and k ranges that are multiples of 16.
//
// Block: 256 threads = 2 x 2 wavefronts, tile 128 (m) x 128 (b rows), 64 k per LDS stage; a wavefront owns
// 2 x 2 sub-tiles of 32 x 32. Two blocks share a CU, so one block's prologue, barrier and output stores
// run under the other block's math.
//   * global -> LDS directly (buffer_load ... lds, no staging registers, lanes past the k range read
//     zero), a ring of three stages, one barrier per chunk. During the math of chunk c a wave reads the
//     MFMA operands of chunk c+1 from LDS into a second register set and issues the loads of chunk c+3,
//     one instruction every few MFMAs, into the stage chunk c has vacated. Operand rows are 4 x 16 bytes, piece u = 2 * (K group) + half stored in slot
//     u ^ ((row >> 2) & 3), which spreads the 16 rows of a ds_read_b128 group over all banks. A lane
//     takes 16 consecutive bytes of a 32-byte K group (half = lane / 32): the first 8 feed the first
//     MFMA of the group, the last 8 the second -- a and b use the same split, so every product meets its
//     partner. The scales come in blocks of 8 K groups (32 bytes per row, so a scale row's cache
//     line is touched once per 256 k) and are rearranged in LDS to [group][row].
//   * math per (K group, sub-tile): 2 x v_mfma_f32_32x32x16 into one of two 16-register accumulators,
//     then total += acc * (sa * sb), one FMA per output element, issued between the MFMAs of the next
//     sub-tile so the matrix pipe and the VALU run together inside a wavefront as well as across the
//     two wavefronts of a SIMD. The last fold of a chunk rides into the next chunk (uniform b scales;
//     with row-wise b scales, which live in registers per chunk, that fold stays in its own chunk).
//   * epilogue stores runs of four consecutive n as one 8- or 16-byte store.
#pragma once
#include "gemm_args.hpp"

namespace viola {

typedef int i32x4 __attribute__((ext_vector_type(4)));

constexpr int FBK = 64, FKG = FBK / 32;                           // k bytes and K groups per LDS stage
constexpr int FTHREADS = 256, FSTAGES = 3;
#ifndef VIOLA_BIG_STAGES
#define VIOLA_BIG_STAGES 3                                         // ring depth of the 256 x 256 tile kernels (4 measured the same)
#endif
constexpr int F_TILE = BM * FBK;                                  // bytes of one operand tile
constexpr int F_STAGE = 2 * F_TILE;
// Scales travel in blocks of 8 K groups (4 chunks): 32 bytes per row and operand, fetched as two 16-byte pieces
// (piece = 4 groups of one row; thread t brings piece t / 128 of row t % 128), double-buffered, and read from LDS in
// that layout: the scale of (row, group g of the block) is float ((g / 4) * 128 + row) * 4 + g % 4.
constexpr int F_SGROUPS = 8, F_SCHUNKS = F_SGROUPS / FKG;
constexpr int F_SBLOCK = F_SGROUPS * BM * 4;                      // bytes of one operand's scale block
constexpr int F_RAW = FSTAGES * F_STAGE;                          // scale blocks as fetched: [buffer][operand][half][row][4 groups]
constexpr int F_LDS = F_RAW + 4 * F_SBLOCK;

// 64 lanes x 16 (or 4) bytes from a raw buffer straight into LDS at lds_addr + 16 (4) * lane. The compiler
// is not told that these touch LDS (it would drain every outstanding load before each LDS read); the kernel
// orders them against its LDS reads with s_waitcnt vmcnt + barrier itself.
__device__ __forceinline__ void load16_to_lds(i32x4 rsrc, uint32_t lds_addr, uint32_t voffset, uint32_t soffset) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :: "s"(lds_addr), "v"(voffset), "s"(rsrc), "s"(soffset) : "memory");
}
__device__ __forceinline__ i32x4 raw_resource(const void* base, int64_t bytes = 0x7fffffff) {
    const uint64_t address = reinterpret_cast<uint64_t>(base);
    i32x4 r = {__builtin_amdgcn_readfirstlane((int)(uint32_t)address), __builtin_amdgcn_readfirstlane((int)(uint32_t)(address >> 32)),
               __builtin_amdgcn_readfirstlane((int)bytes), 0x00020000};
    return r;
}

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

// A finished 16-byte piece of the output, stored with the streaming hint: nothing in this launch reads it again, and
// kept out of the way it does not push the operand panels that the tiles of an XCD share out of its L2 (8192 x 4096 x
// 1024 with a 64 MB output: 85 -> 80 us).
__device__ __forceinline__ void store_streaming(void* p, uint4 piece) {
    const i32x4 v = {(int)piece.x, (int)piece.y, (int)piece.z, (int)piece.w};
    __builtin_nontemporal_store(v, static_cast<i32x4*>(p));
}

template <typename TO> __device__ __forceinline__ float rounded(float v) { return to_f32(from_f32<TO>(v)); }

// TN: 32-column sub-tiles per wave; TN = 1 halves the tile to 128 x 64 for problems with too few 128 x 128 tiles to
// give every CU two blocks (plain mode only).
// TENSOR: one scale per operand (p.sa[0], p.sb[0]) applied to the finished sums, out = (acc * sa) * sb + bias: no
// per-group fold, so a chunk's 64 k go through one v_mfma_f32_32x32x64_f8f6f4 per sub-tile straight into the totals.
typedef int i32x8 __attribute__((ext_vector_type(8)));
// MX: E8M0 scales (one byte per 32 k; p.sa / p.sb point at bytes, ldsa / ldsb are bytes per scale row) applied by the
// hardware inside v_mfma_scale_f32_32x32x64_f8f6f4. The instruction's first 32-k block is operand registers 0..3 of all
// 64 lanes and takes its scale from lanes 0..31 (one byte per row), the second block is registers 4..7 with the scale
// of lanes 32..63 (measured: a scale change confined to one K group only gives the right product in this arrangement).
// That is the layout the per-tensor path already has (registers 0..3 = the lane's 16 bytes of K group 0, 4..7 = of K
// group 1), so lane (row, half) hands over the scale byte of K group `half` of its row. Scales travel in blocks of 16
// K groups (one 16-byte piece per tile row and operand), double-buffered behind the ring; k must be a multiple of 128.
constexpr int MX_GROUPS = 16, MX_CHUNKS = MX_GROUPS / FKG, MX_BLOCK = 2 * BM * MX_GROUPS;   // bytes of one block, a then b
// BIG (per-tensor and block-scaled recipes): a 256 x 256 tile per 512-thread block, 2 x 4 waves of 4 x 2
// sub-tiles, one block per CU. Without the per-group fold these kernels are bound by the L2 -> LDS stream (taking the
// global loads out of the 128 x 128 kernel brings it from 1.7 to 4.4 PFLOP/s on a 16384 x 22016 x 4096 product, taking
// the LDS reads out changes nothing); the larger tile moves half the bytes per flop.
// KSPLIT (plain mode): for products with fewer than 512 tiles of 128 x 128 and a long k, such as a weight gradient. A
// block of 512 threads is two teams of 2 x 2 waves, each with a stage ring and scale buffers of its own, that compute
// the same 128 x 128 tile over the two halves of the k range (cut at a multiple of 256 k, one scale block); at the end
// team 1 hands its totals over in LDS and team 0 adds them to its own (always in that order) and stores the tile.
// Against the 128 x 64 tiles such products would otherwise get, a wave has the 2 x 2 sub-tiles' better ratio of MFMAs to
// global loads and LDS reads, and a CU still holds eight waves.
template <int MODE, bool A_BF8, bool B_BF8, bool B_ROWSCALE, typename TO, int TN, bool TENSOR = false, bool MX = false, bool BIG = false,
          bool KSPLIT = false>
__global__ __launch_bounds__(BIG || KSPLIT ? 512 : FTHREADS, BIG || KSPLIT ? 1 : TENSOR ? 3 : 2) void group_gemm_fast(GemmArgs p, int bias_dtype) {
    static_assert(!KSPLIT || (MODE == MODE_PLAIN && !BIG), "the split exists for plain products on the small tiles");
    static_assert(!TENSOR || !B_ROWSCALE, "per-tensor scaling has no row scales");
    static_assert(!MX || !TENSOR, "one scaling recipe per kernel");
    static_assert(!BIG || ((TENSOR || MX) && TN == 2), "the large tile exists for the fold-free kernels");
    constexpr bool NOFOLD = TENSOR || MX;                                   // the products of a chunk go straight into the totals
    constexpr int WAVES_N = BIG ? 4 : 2, THREADS = BIG ? 512 : FTHREADS;     // waves as 2 (m) x WAVES_N (n)
    constexpr int TBM = BIG ? 2 * BM : BM;                                   // rows of a per tile
    constexpr int K_TILE_A = BIG ? 2 * F_TILE : F_TILE, K_STAGE = BIG ? 4 * F_TILE : F_STAGE;
    constexpr int K_STAGES = BIG ? VIOLA_BIG_STAGES : FSTAGES, K_RAW = K_STAGES * K_STAGE;   // ring depth: loads run K_STAGES chunks ahead
    constexpr int K_MX_BLOCK = BIG ? 2 * MX_BLOCK : MX_BLOCK;
    // without scale blocks the ring plus the epilogue's bias row is all the LDS a block needs: three blocks share a CU
    constexpr int TEAM_LDS = TENSOR ? K_RAW + 1024 : MX ? K_RAW + 2 * K_MX_BLOCK : F_LDS;
    __shared__ __attribute__((aligned(1024))) uint8_t lds_all[(KSPLIT ? 2 : 1) * TEAM_LDS];

    // wave grid 2 (m) x 2 (n), 2 x 2 sub-tiles each. Plain / gated backward: sub-tile i of wave wn covers b rows
    // 64 wn + 32 i. Gated forward: the tile's b rows are 64 gate rows then the 64 up rows of the same n, and
    // i = 0 / 1 is the gate / up sub-tile of columns 32 wn .. 32 wn + 31, so one lane holds g and u of the same n.
    constexpr bool GATED = MODE == MODE_GATED_FWD;
    constexpr int TM = BIG ? 4 : 2;
    constexpr int PANEL = GATED ? 32 * WAVES_N : 32 * TN * WAVES_N;
    static_assert(!GATED || TN == 2, "gated forward pairs a gate and an up sub-tile");
    // KSPLIT: `team` is the half of the k range this wave works on; tid, wave and lds are the team's own
    const int team = KSPLIT ? __builtin_amdgcn_readfirstlane((int)threadIdx.x / FTHREADS) : 0;
    const int tid = KSPLIT ? (int)threadIdx.x % FTHREADS : (int)threadIdx.x, lane = tid % WAVE;
    uint8_t* const lds = lds_all + team * (KSPLIT ? TEAM_LDS : 0);
    const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
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
    int64_t m_begin = (int64_t)tile_m * TBM, m_end = p.m;
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
    int split_chunks = 0;                                                    // KSPLIT: chunks of the longer (first) half
    if constexpr (KSPLIT) {
        constexpr int64_t CUT = (MX ? MX_GROUPS : F_SGROUPS) * 32;            // a scale block belongs to one team
        const int64_t len = k_end - k_begin, blocks = (len + CUT - 1) / CUT;
        const int64_t first = (blocks + 1) / 2 * CUT < len ? (blocks + 1) / 2 * CUT : len;
        split_chunks = (int)((first + FBK - 1) / FBK);
        if (team == 0) k_end = k_begin + first;
        else k_begin += first;
    }
    const int64_t n_begin = (int64_t)tile_n * PANEL;
    const int64_t b_rows_total = GATED ? 2 * p.n : p.n;
    auto b_global_row = [&](int r) -> int64_t {                               // tile-local b row -> row of b
        int64_t bn;
        if constexpr (GATED) bn = (int64_t)(r / PANEL) * p.n + n_begin + r % PANEL;
        else bn = n_begin + r;
        return bn < b_rows_total ? bn : b_rows_total - 1;
    };
    auto a_global_row = [&](int r) -> int64_t {                               // rows past the end repeat the last row
        const int64_t am = m_begin + r;
        return am < m_end ? am : m_end - 1;
    };

    // ---- load plan. Instruction `it` of this wave fills 16-byte LDS units [it * 256 + wave * 64, +64) of an operand
    // tile: unit U = 4 * row + slot holds piece (slot ^ ((row >> 2) & 3)) of the row's 64 k bytes.
    const i32x4 res_a = raw_resource(p.a + m_begin * p.lda + k_begin);
    const i32x4 res_b = raw_resource(bptr + k_begin);
    // scale buffers carry their true size: a 16-byte piece may reach past the last row, and must then read zero
    const i32x4 res_sa = raw_resource(p.sa, p.sa_bytes);
    const i32x4 res_sb = raw_resource(sbptr, p.sb_bytes);
    constexpr uint32_t OUTSIDE = 0x80000000u;
    const int64_t k_len = k_end - k_begin;
    const int groups_total = (int)((k_len + 31) / 32);
    // (KSPLIT: both teams walk the first half's chunk count, they share the barriers; past its own range a team loads
    // zero codes and zero scales)
    const int chunks = KSPLIT ? split_chunks : (int)((k_len + FBK - 1) / FBK);
    const int full_chunks = (int)(k_len / FBK);                             // chunks wholly inside the k range
    // Offsets of the thread's 16-byte pieces. Chunks wholly inside the k range use them as they are; for the one chunk
    // that straddles the end of the range the pieces past it are redirected outside the buffer (they read zero), and
    // for chunks past the range (issued to keep the load counts of the ring uniform) all of them are. `cur_*` holds
    // what the next issue uses and is switched by retarget(), a wave-uniform branch taken at most twice per tile.
    uint32_t goff_a[2], goff_b[2], tail_a[2], tail_b[2], cur_a[2], cur_b[2];
#pragma unroll
    for (int it = 0; it < 2; ++it) {
        const int unit = it * THREADS + tid, r = unit >> 2, piece = (unit & 3) ^ ((r >> 2) & 3);
        goff_a[it] = (uint32_t)(a_global_row(r) - m_begin) * (uint32_t)p.lda + piece * 16;   // tile rows x lda < 4 GiB (checked by the launcher)
        goff_b[it] = (uint32_t)b_global_row(r) * (uint32_t)p.ldb + piece * 16;   // relative to bptr + k_begin (row span < 2 GiB)
        const bool inside_tail = (int64_t)full_chunks * FBK + piece * 16 < k_len;
        tail_a[it] = inside_tail ? goff_a[it] : OUTSIDE;
        tail_b[it] = inside_tail ? goff_b[it] : OUTSIDE;
        cur_a[it] = goff_a[it];
        cur_b[it] = goff_b[it];
    }
    auto retarget = [&](int c) {                                             // before the loads of chunk c are issued
        if (__builtin_expect(c >= full_chunks, 0)) {
            asm volatile("; end of the k range");                           // keeps this a branch, not per-chunk selects
            const bool straddles = c == full_chunks;
#pragma unroll
            for (int it = 0; it < 2; ++it) {
                cur_a[it] = straddles ? tail_a[it] : OUTSIDE;
                cur_b[it] = straddles ? tail_b[it] : OUTSIDE;
            }
        }
    };
    // scales: per block of 8 K groups the thread fetches groups 4 shalf .. 4 shalf + 3 of tile row srow
    const int srow = tid % BM, shalf = tid / BM;
    // (row indices and scale offsets fit 31 bits, the launcher sees to it: 32-bit division, not the 64-bit routine)
    const uint32_t sa_off = (uint32_t)a_global_row(srow) / (uint32_t)p.ar * (uint32_t)p.ldsa * 4 + (uint32_t)((k_begin >> 5) + shalf * 4) * 4;
    const uint32_t sb_off = (uint32_t)b_global_row(srow) / (uint32_t)p.br * (uint32_t)p.ldsb * 4 + (uint32_t)((k_begin >> 5) + shalf * 4) * 4;
    constexpr int B_LOADS = TN;                                              // 64 b rows per load instruction
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)lds;
    // load instruction `which` (0, 1: a; 2, 3: b) of chunk c into ring stage `stage`
    auto issue_one = [&](int c, int stage, int which) {
        const uint32_t k0 = (uint32_t)c * FBK;                               // relative to k_begin
        const uint32_t base = lds_base + (uint32_t)stage * K_STAGE + (uint32_t)wave * 1024;
        const int it = which & 1;
        if (which < 2) load16_to_lds(res_a, base + it * THREADS * 16, cur_a[it], k0);
        else load16_to_lds(res_b, base + K_TILE_A + it * THREADS * 16, cur_b[it], k0);
    };
    constexpr int CHUNK_LOADS = 2 + B_LOADS;
    auto issue = [&](int c, int stage) {
        retarget(c);
#pragma unroll
        for (int i = 0; i < CHUNK_LOADS; ++i) issue_one(c, stage, i);
    };
    // scale block `block` (K groups 8 block .. 8 block + 7 of the k range) -> raw area, one 16-byte piece per thread
    // and operand; a piece wholly past the k range is not fetched
    auto issue_scales = [&](int block) {
        const bool inside = block * F_SGROUPS + shalf * 4 < groups_total;
        const uint32_t at = lds_base + F_RAW + (uint32_t)(block & 1) * 2 * F_SBLOCK + (uint32_t)wave * 1024;
        load16_to_lds(res_sa, at, inside ? sa_off : OUTSIDE, (uint32_t)(block * F_SGROUPS * 4));
        load16_to_lds(res_sb, at + F_SBLOCK, inside ? sb_off : OUTSIDE, (uint32_t)(block * F_SGROUPS * 4));
    };
    // The one scale block that straddles the end of the k range holds, past that end, whatever follows in memory (the
    // next row's first scales, perhaps a NaN): the thread that fetched a piece clears those entries once its loads
    // have landed. Their products are zero, and zero times the cleared scale stays zero. (Pieces wholly past the end
    // were not fetched and read as zero already.)
    auto clear_past_the_end = [&](int block) {
        const int left = groups_total - (int)(block * F_SGROUPS + shalf * 4);
        if (left <= 0 || left >= 4) return;
        float* mine = reinterpret_cast<float*>(lds + F_RAW + (block & 1) * 2 * F_SBLOCK + tid * 16);
#pragma unroll
        for (int q = 1; q < 4; ++q)
            if (q >= left) { mine[q] = 0.0f; mine[F_SBLOCK / 4 + q] = 0.0f; }
    };
    const int last_scale_block = (groups_total - 1) / F_SGROUPS;             // the only block that can straddle
    // MX: scale block `block` (K groups 16 block ..) -> buffer block & 1: waves 0, 1 fetch the a rows' pieces, waves 2, 3 the b rows'
    const i32x4 res_mxa = raw_resource(p.sa, p.sa_bytes);
    const i32x4 res_mxb = raw_resource(sbptr, p.sb_bytes);
    const uint32_t mx_off = tid < TBM ? (uint32_t)a_global_row(tid) / (uint32_t)p.ar * (uint32_t)p.ldsa + (uint32_t)(k_begin >> 5)
                                      : (uint32_t)b_global_row(tid - TBM) / (uint32_t)p.br * (uint32_t)p.ldsb + (uint32_t)(k_begin >> 5);
    auto issue_mx_scales = [&](int block) {
        const bool inside = block * MX_GROUPS < groups_total;
        const uint32_t at = lds_base + K_RAW + (uint32_t)(block & 1) * K_MX_BLOCK + (uint32_t)wave * 1024;
        load16_to_lds(wave < TBM / 64 ? res_mxa : res_mxb, at, inside ? mx_off : OUTSIDE, (uint32_t)(block * MX_GROUPS));
    };
    // ---- MFMA operand reads: 16 bytes = this lane's half (lhi) of K group kg for row l32 of a sub-tile
    auto a_sub = [&](int j) -> int { return (wm * TM + j) * 32; };
    auto b_sub = [&](int i) -> int { return GATED ? i * PANEL + wn * 32 : (wn * TN + i) * 32; };
    const int sw = (l32 >> 2) & 3;
    const int rd_a = (a_sub(0) + l32) * FBK + ((lhi ^ sw) * 16);             // K group 1: ^ 32
    const int rd_b = (b_sub(0) + l32) * FBK + ((lhi ^ sw) * 16);

    f32x16 total[TN][TM];                                                    // [b sub-tile i][a sub-tile j]
#pragma unroll
    for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int j = 0; j < TM; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) total[i][j][r] = 0.0f;

    // Four 16-register accumulators: two receive the MFMAs of the current pair of (K group, sub-tile) units while the
    // two of the pair before are folded into the totals (across chunk boundaries when CARRY).
    // Row-wise b scales: every output element has its own product sa[m] * sb[n] per K group. One
    // v_mfma_f32_32x32x1_2b_f32 forms the 2 x 32 x 32 products of a pair of units (a sub-tiles 0 and 1 against one b
    // sub-tile) as an outer product on the matrix pipe, in the accumulators' own layout and rounded exactly as
    // v_mul_f32 rounds them; the fold is then one FMA per element, as with uniform b scales. The products of a pair are
    // issued among its MFMAs and read while the next pair's MFMAs run: into the other of two buffers where the registers
    // allow it (TN = 1), else into the one buffer once the fold before has read it.
    constexpr bool OUTER = B_ROWSCALE;
    static_assert(!B_ROWSCALE || TM == 2, "the two blocks of the scale products' MFMA are the wave's two a sub-tiles");
    constexpr bool CARRY = !B_ROWSCALE || OUTER;
    constexpr int PBUF = TN == 1 ? 2 : 1;
    typedef float f32x32 __attribute__((ext_vector_type(32)));
    f32x32 prod[PBUF];
    if constexpr (OUTER) {
#pragma unroll
        for (int b = 0; b < PBUF; ++b)
#pragma unroll
            for (int r = 0; r < 32; ++r) prod[b][r] = 0.0f;
    }
    f32x16 acc[4];
    float pending_scale[2] = {0.0f, 0.0f};                                   // sa * sb of the pending pair (uniform b scales)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[0][r] = acc[1][r] = acc[2][r] = acc[3][r] = 0.0f;
    auto as_long = [](uint32_t lo, uint32_t hi) -> long { return (long)(((uint64_t)hi << 32) | lo); };

    // The MFMA operands and scales of one chunk, in registers. They are read from LDS one chunk ahead of their
    // math (two register sets, the chunk loop is unrolled by two), so a wavefront goes from the barrier straight
    // into its math and the LDS latency of the next chunk hides under it.
    struct Operands {
        uint4 a[FKG][TM], b[FKG][TN];
        float sa[FKG][TM], sb[FKG][TN];
        i32x8 wide_a[TM], wide_b[TN];                                        // TENSOR / MX: 16 k of either K group of a sub-tile row
        int mx_a[(TM + 1) / 2], mx_b[(TN + 1) / 2];                          // MX: the rows' scale bytes of K group lhi, sub-tile t in byte 2 (t & 1) of word t / 2
    };
    // scale of tile row `row` for K group kg of chunk c (operand 0: a, 1: b); groups past the k range read as zero
    auto scale_at = [&](int operand, int c, int kg, int row) -> float {
        const int g8 = (c % F_SCHUNKS) * FKG + kg;                          // group of the block (uniform)
        const float* block = reinterpret_cast<const float*>(lds + F_RAW + ((c / F_SCHUNKS) & 1) * 2 * F_SBLOCK + operand * F_SBLOCK);
        return block[((g8 >> 2) * BM + row) * 4 + (g8 & 3)];
    };
    auto read_operands = [&](int stage, int c, Operands& o) {
        const uint8_t* tile_a = lds + stage * K_STAGE;
        const uint8_t* tile_b = tile_a + K_TILE_A;
        if constexpr (NOFOLD) {
            // the lane's 16 bytes of either K group (slots lhi and lhi + 2)
            const int first_a = rd_a, first_b = rd_b;
            constexpr int SECOND = 32;
#pragma unroll
            for (int j = 0; j < TM; ++j) {
                const i32x4 lo = *reinterpret_cast<const i32x4*>(tile_a + (first_a + j * 32 * FBK));
                const i32x4 hi = *reinterpret_cast<const i32x4*>(tile_a + ((first_a + j * 32 * FBK) ^ SECOND));
                o.wide_a[j] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            }
#pragma unroll
            for (int i = 0; i < TN; ++i) {
                const i32x4 lo = *reinterpret_cast<const i32x4*>(tile_b + (first_b + (b_sub(i) - b_sub(0)) * FBK));
                const i32x4 hi = *reinterpret_cast<const i32x4*>(tile_b + ((first_b + (b_sub(i) - b_sub(0)) * FBK) ^ SECOND));
                o.wide_b[i] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            }
            if constexpr (MX) {
                const uint8_t* block = lds + K_RAW + ((c / MX_CHUNKS) & 1) * K_MX_BLOCK + (c % MX_CHUNKS) * FKG + lhi;
#pragma unroll
                for (int j = 0; j < TM; j += 2) {
                    o.mx_a[j / 2] = block[(a_sub(j) + l32) * MX_GROUPS];
                    if (j + 1 < TM) o.mx_a[j / 2] |= block[(a_sub(j + 1) + l32) * MX_GROUPS] << 16;
                }
#pragma unroll
                for (int i = 0; i < TN; i += 2) {
                    o.mx_b[i / 2] = block[TBM * MX_GROUPS + (b_sub(i) + l32) * MX_GROUPS];
                    if (i + 1 < TN) o.mx_b[i / 2] |= block[TBM * MX_GROUPS + (b_sub(i + 1) + l32) * MX_GROUPS] << 16;
                }
            }
            return;
        }
#pragma unroll
        for (int kg = 0; kg < FKG; ++kg) {
#pragma unroll
            for (int j = 0; j < TM; ++j) o.a[kg][j] = *reinterpret_cast<const uint4*>(tile_a + ((rd_a + j * 32 * FBK) ^ (kg * 32)));
#pragma unroll
            for (int i = 0; i < TN; ++i) o.b[kg][i] = *reinterpret_cast<const uint4*>(tile_b + ((rd_b + (b_sub(i) - b_sub(0)) * FBK) ^ (kg * 32)));
            if constexpr (OUTER) {                                           // compute() fetches the scales itself
#pragma unroll
                for (int j = 0; j < TM; ++j) o.sa[kg][j] = 0.0f;
#pragma unroll
                for (int i = 0; i < TN; ++i) o.sb[kg][i] = 0.0f;
            } else {
#pragma unroll
                for (int j = 0; j < TM; ++j) o.sa[kg][j] = scale_at(0, c, kg, a_sub(j) + l32);
#pragma unroll
                for (int i = 0; i < TN; ++i) o.sb[kg][i] = scale_at(1, c, kg, b_sub(i));
            }
        }
    };

    // the block-scaled MFMA with the scale bytes picked out of their words (the byte index is an immediate)
    auto mx_mfma = [](i32x8 b, i32x8 a, f32x16 c, int scale_b, int scale_a, int which) -> f32x16 {
        constexpr int FB = B_BF8 ? 1 : 0, FA = A_BF8 ? 1 : 0;
        switch (which) {
            case 0: return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(b, a, c, FB, FA, 0, scale_b, 0, scale_a);
            case 1: return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(b, a, c, FB, FA, 0, scale_b, 2, scale_a);
            case 2: return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(b, a, c, FB, FA, 2, scale_b, 0, scale_a);
            default: return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(b, a, c, FB, FA, 2, scale_b, 2, scale_a);
        }
    };

    // Math of chunk c on the operands in `o`; `between(step)` runs after MFMA number `step` of the chunk (the
    // caller's global loads and LDS reads for later chunks go there, spread over the chunk).
    auto compute = [&](const Operands& o, int c, auto&& between) {
        if constexpr (NOFOLD) {
            constexpr int STEPS_PER = FKG * 2;
#pragma unroll
            for (int i = 0; i < TN; ++i) {
#pragma unroll
                for (int j = 0; j < TM; ++j) {
                    // both operands give a lane the same 32 of the chunk's 64 k (16 of each K group), so every product
                    // meets its partner whatever order the instruction walks them in
                    if constexpr (MX)
                        total[i][j] = mx_mfma(o.wide_b[i], o.wide_a[j], total[i][j], o.mx_b[i / 2], o.mx_a[j / 2], (i & 1) * 2 + (j & 1));
                    else
                        total[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(o.wide_b[i], o.wide_a[j], total[i][j], B_BF8 ? 1 : 0, A_BF8 ? 1 : 0, 0, 0, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int step = 0; step < STEPS_PER; ++step) between((i * TM + j) * STEPS_PER + step);
                }
            }
            return;
        }
        // fold half `h` (registers 8h .. 8h+7) of accumulator `buf` into total[i][j]
        auto fold_half = [&](int buf, int i, int j, int slot, int h, float scale) {
#pragma unroll
            for (int r = 8 * h; r < 8 * h + 8; ++r) {
                if constexpr (!B_ROWSCALE) {
                    total[i][j][r] = fmaf(acc[buf][r], scale, total[i][j][r]);
                } else {
                    total[i][j][r] = fmaf(acc[buf][r], prod[slot % PBUF][16 * j + r], total[i][j][r]);
                }
            }
        };
        const f32x16 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        // Units go in pairs: the four MFMAs of a pair alternate between its two accumulators, so an MFMA never waits
        // for the one issued just before it, and a quarter of the previous pair's fold follows each of them.
        constexpr int UNITS = FKG * TN * TM, PAIRS = UNITS / 2;
#pragma unroll
        for (int pair = 0; pair < PAIRS; ++pair) {
            const int base = (pair & 1) * 2, other = base ^ 2;
            const int before = (pair + PAIRS - 1) % PAIRS;                   // the pair folded now (last of the chunk before for pair 0)
            const bool fold_prev = pair > 0 || CARRY;
            int kg[2], ti[2], tj[2], pkg[2], pi[2], pj[2];
            float prev_scale[2];
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int unit = 2 * pair + h, prev = 2 * before + h;
                kg[h] = unit / (TN * TM); ti[h] = unit / TM % TN; tj[h] = unit % TM;
                pkg[h] = prev / (TN * TM); pi[h] = prev / TM % TN; pj[h] = prev % TM;
                prev_scale[h] = B_ROWSCALE ? (pair > 0 ? o.sa[pkg[h]][pj[h]] : 0.0f) : pending_scale[h];
            }
            // operands of the scale products' MFMA: lanes 0..31 / 32..63 carry the a scales of sub-tile 0 / 1, every lane the
            // b scale of row l32 of the pair's b sub-tile
            float outer_a = 0.0f, outer_b = 0.0f;
            if constexpr (OUTER) {
                static_assert(PAIRS % 2 == 0, "the two product buffers alternate across chunk boundaries");
                outer_a = scale_at(0, c, kg[0], a_sub(lhi) + l32);
                outer_b = scale_at(1, c, kg[0], b_sub(ti[0]) + l32);
            }
            auto issue_products = [&]() {
                const f32x32 zero32 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                prod[pair % PBUF] = __builtin_amdgcn_mfma_f32_32x32x1f32(outer_b, outer_a, zero32, 0, 0, 0);
            };
#pragma unroll
            for (int step = 0; step < 4; ++step) {
                const int h = step & 1, ks = step >> 1;
                const uint4 ob = o.b[kg[h]][ti[h]], oa = o.a[kg[h]][tj[h]];
                if (ks == 0) acc[base + h] = mfma32<A_BF8, B_BF8>(as_long(ob.x, ob.y), as_long(oa.x, oa.y), zero);
                else acc[base + h] = mfma32<A_BF8, B_BF8>(as_long(ob.z, ob.w), as_long(oa.z, oa.w), acc[base + h]);
                if (fold_prev) fold_half(other + (step >> 1), pi[step >> 1], pj[step >> 1], before & 1, step & 1, prev_scale[step >> 1]);
                asm volatile("" : "+v"(total[pi[step >> 1]][pj[step >> 1]]));
                if constexpr (OUTER) {
                    // with two buffers after the second MFMA of the pair (the scales have arrived from LDS by then), with one
                    // after the last fold that reads it
                    if (step == (PBUF == 2 ? 1 : 3)) issue_products();
                }
                __builtin_amdgcn_sched_barrier(0);
                between(pair * 4 + step);
            }
            if constexpr (!B_ROWSCALE) {
#pragma unroll
                for (int h = 0; h < 2; ++h) pending_scale[h] = o.sa[kg[h]][tj[h]] * o.sb[kg[h]][ti[h]];
            }
        }
        if constexpr (!CARRY) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                constexpr int last_pair = PAIRS - 1;
                const int unit = 2 * last_pair + h;
                const int lkg = unit / (TN * TM), li = unit / TM % TN, lj = unit % TM;
                fold_half((last_pair & 1) * 2 + h, li, lj, last_pair & 1, 0, o.sa[lkg][lj]);
                fold_half((last_pair & 1) * 2 + h, li, lj, last_pair & 1, 1, o.sa[lkg][lj]);
            }
        }
    };

    // Ring of K_STAGES (three in what follows) stages, chunk c in stage c % 3. At the top of iteration c the wave waits for its own loads of
    // chunk c+1 (issued two iterations ago) and for its LDS reads of chunk c; after the barrier chunk c+1 is in LDS
    // for everybody and nobody reads chunk c's stage any more. Then: the loads of chunk c+3 into that stage (one
    // instruction every few MFMAs, so the waves of a CU do not queue up at the memory pipe), the LDS reads of chunk
    // c+1 into the other register set, the math of chunk c. Scale block b (K groups 8b ..) is fetched in iteration
    // 4b-4 into the buffer that block b-2 left at the barrier of that iteration, has landed for every wave at the barrier
    // of iteration 4b-2 and is first read in 4b-1; it is issued before the chunk loads of its iteration, so the waits
    // below cover it one iteration later.
    constexpr int STEPS = FKG * TN * TM * 2, STRIDE = STEPS / CHUNK_LOADS;
    int stage_now = 0, stage_next = 1;
    auto chunk_step = [&](int c, const Operands& now, Operands& next) {
        constexpr int AHEAD = (K_STAGES - 2) * CHUNK_LOADS;                  // loads of the chunks after c + 1 may still be in flight
        static_assert(AHEAD + 2 < 16 && (K_STAGES - 1) * CHUNK_LOADS < 16, "the counts fit the wait instruction's low field");
        if (!NOFOLD && c % F_SCHUNKS == 1) __builtin_amdgcn_s_waitcnt(0x0070 | (AHEAD + 2));
        else if (MX && c % MX_CHUNKS == 1) __builtin_amdgcn_s_waitcnt(0x0070 | (AHEAD + 1));
        else __builtin_amdgcn_s_waitcnt(0x0070 | AHEAD);
        __syncthreads();
        if constexpr (!NOFOLD) {
            if (c % F_SCHUNKS == 0) issue_scales(c / F_SCHUNKS + 1);
            // the wait above has seen this wave's loads of that block land; the next barrier shows the fix to every wave
            // before the block's first use, one iteration later
            if (c % F_SCHUNKS == 2 && c / F_SCHUNKS + 1 == last_scale_block) clear_past_the_end(last_scale_block);
        }
        if constexpr (MX) {
            if (c % MX_CHUNKS == 0) issue_mx_scales(c / MX_CHUNKS + 1);
        }
        if (c + 1 < chunks) read_operands(stage_next, c + 1, next);
        retarget(c + K_STAGES);
        const int fill = stage_now;
        compute(now, c, [&](int step) {
            if (step % STRIDE == 0 && step / STRIDE < CHUNK_LOADS) issue_one(c + K_STAGES, fill, step / STRIDE);
        });
        stage_now = stage_next;
        stage_next = stage_next == K_STAGES - 1 ? 0 : stage_next + 1;
    };
    if constexpr (MX) issue_mx_scales(0);
    else if constexpr (!TENSOR) issue_scales(0);
#pragma unroll
    for (int s = 0; s < K_STAGES; ++s) issue(s, s);
    __builtin_amdgcn_s_waitcnt(0x0F70 | ((K_STAGES - 1) * CHUNK_LOADS));                   // scale block 0 and chunk 0 are in LDS
    __syncthreads();
    if constexpr (KSPLIT && !NOFOLD) {                                       // the condition differs between the teams, the barrier must not
        if (last_scale_block == 0 && groups_total % 4 != 0) clear_past_the_end(0);
        __syncthreads();
    } else if constexpr (!NOFOLD) {
        if (last_scale_block == 0 && groups_total % 4 != 0) {                // a k range of one scale block: uniform
            clear_past_the_end(0);
            __syncthreads();
        }
    }
    Operands set0, set1;
    read_operands(0, 0, set0);
    for (int c = 0; c < chunks; c += 2) {
        chunk_step(c, set0, set1);
        if (c + 1 < chunks) chunk_step(c + 1, set1, set0);
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);     // drain the trailing loads before the LDS allocation is released
    if constexpr (!TENSOR && CARRY && !MX) {
        constexpr int UNITS = FKG * TN * TM, last_pair = UNITS / 2 - 1;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int unit = 2 * last_pair + h, li = unit / TM % TN, lj = unit % TM;
#pragma unroll
            for (int r = 0; r < 16; ++r)
                total[li][lj][r] = fmaf(acc[(last_pair & 1) * 2 + h][r], OUTER ? prod[last_pair % PBUF][16 * lj + r] : pending_scale[h], total[li][lj][r]);
        }
    }

    if constexpr (KSPLIT) {
        // team 1's totals -> LDS (the rings are idle now) as [register quad][thread], team 0 adds them. Team 1 then
        // walks the epilogue with an empty row range: it stores nothing and meets the barriers there.
        __syncthreads();
        float4* handover = reinterpret_cast<float4*>(lds_all);
        static_assert(TN * TM * 16 * 4 * FTHREADS <= 2 * TEAM_LDS, "a team's totals fit the block's LDS");
#pragma unroll
        for (int i = 0; i < TN; ++i)
#pragma unroll
            for (int j = 0; j < TM; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    float4* at = &handover[((i * TM + j) * 4 + q) * FTHREADS + tid];
                    if (team == 1) *at = make_float4(total[i][j][4 * q], total[i][j][4 * q + 1], total[i][j][4 * q + 2], total[i][j][4 * q + 3]);
                }
        __syncthreads();
        if (team == 0) {
#pragma unroll
            for (int i = 0; i < TN; ++i)
#pragma unroll
                for (int j = 0; j < TM; ++j)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const float4 t = handover[((i * TM + j) * 4 + q) * FTHREADS + tid];
                        total[i][j][4 * q] += t.x; total[i][j][4 * q + 1] += t.y; total[i][j][4 * q + 2] += t.z; total[i][j][4 * q + 3] += t.w;
                    }
        } else {
            m_end = m_begin;
        }
    }
    if constexpr (TENSOR) {
        const float sa = p.sa[0], sb = p.sb[0];
#pragma unroll
        for (int i = 0; i < TN; ++i)
#pragma unroll
            for (int j = 0; j < TM; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) { const float t = total[i][j][r] * sa; total[i][j][r] = t * sb; }
    }

    // ---- epilogue: for sub-tiles (i, j) the lane holds row m = 32*j + l32 and, per register quad r4, columns
    // n = 8*r4 + 4*lhi + 0..3
    TO* out = reinterpret_cast<TO*>(outptr);
    const bool vec_out = p.ldo % 4 == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0;
    const bool vec_aux = p.n % 4 == 0 && (reinterpret_cast<uintptr_t>(p.aux) & 15) == 0;
    if constexpr (MODE == MODE_PLAIN) {
        // Row-major output: as stores, "one row per lane, four columns" would touch 32 cache lines per instruction. When
        // rows of out are 16-byte aligned, each wavefront parks its finished values, 32 rows at a time, in LDS (the
        // stage ring is free now) and stores them as 16-byte pieces along the rows instead.
        constexpr int PER = 16 / (int)sizeof(TO);                            // values per piece
        constexpr int WCOLS = 32 * TN, PLD = WCOLS + PER, PIECES = WCOLS / PER;
        static_assert(2 * WAVES_N * 32 * PLD * (int)sizeof(TO) <= K_RAW, "parking area fits in the stage ring");
        if ((p.ldo * sizeof(TO)) % 16 == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0) {
            __syncthreads();                                                 // every wave has left the ring
            TO* park = reinterpret_cast<TO*>(lds) + wave * 32 * PLD;
            const int64_t ncol0 = n_begin + wn * WCOLS;
            // the tile's bias as fp32 in the (now idle) raw scale area: one global load per column, not per element
            float4 bias_q[TN][4];
            if (p.bias) {
                float* bias_lds = reinterpret_cast<float*>(lds + K_RAW);
                if (tid < PANEL) bias_lds[tid] = n_begin + tid < p.n ? load_bias(p.bias, n_begin + tid, bias_dtype) : 0.0f;
                __syncthreads();
#pragma unroll
                for (int i = 0; i < TN; ++i)
#pragma unroll
                    for (int r4 = 0; r4 < 4; ++r4) bias_q[i][r4] = *reinterpret_cast<const float4*>(&bias_lds[wn * WCOLS + i * 32 + r4 * 8 + lhi * 4]);
            } else {
#pragma unroll
                for (int i = 0; i < TN; ++i)
#pragma unroll
                    for (int r4 = 0; r4 < 4; ++r4) bias_q[i][r4] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            }
#pragma unroll
            for (int j = 0; j < TM; ++j) {
#pragma unroll
                for (int i = 0; i < TN; ++i)
#pragma unroll
                    for (int r4 = 0; r4 < 4; ++r4) {
                        float v[4];
                        const float bq[4] = {bias_q[i][r4].x, bias_q[i][r4].y, bias_q[i][r4].z, bias_q[i][r4].w};
#pragma unroll
                        for (int e = 0; e < 4; ++e) v[e] = total[i][j][r4 * 4 + e] + bq[e];
                        Quad<TO>::store(&park[l32 * PLD + i * 32 + r4 * 8 + lhi * 4], v);
                    }
#pragma unroll
                for (int it = 0; it < 32 * PIECES / WAVE; ++it) {
                    const int id = it * WAVE + lane, pr = id / PIECES, pc = id % PIECES;
                    const int64_t mrow = m_begin + a_sub(j) + pr, ncol = ncol0 + pc * PER;
                    const uint4 piece = *reinterpret_cast<const uint4*>(&park[pr * PLD + pc * PER]);
                    if (mrow >= m_end || ncol >= p.n) continue;
                    if (ncol + PER <= p.n) {
                        store_streaming(out + mrow * p.ldo + ncol, piece);
                    } else {
                        const TO* values = reinterpret_cast<const TO*>(&piece);
                        for (int e = 0; e < PER; ++e)
                            if (ncol + e < p.n) out[mrow * p.ldo + ncol + e] = values[e];
                    }
                }
            }
            return;
        }
    }
    if constexpr (MODE != MODE_PLAIN) {
        // Gated epilogues through LDS as well: a sub-tile's 32 x 32 values are parked [row][col] in a wave-private area
        // of the (idle) stage ring and move to and from global memory as 16-byte pieces along the rows; one lane = one
        // row and runs of four columns would touch 32 cache lines per instruction. Needs 16-byte aligned rows.
        constexpr int PER = 16 / (int)sizeof(TO), PLD = 32 + PER, PIECES = 32 / PER, AREA = 32 * PLD;
        static_assert(2 * WAVES_N * 2 * AREA * (int)sizeof(TO) <= K_RAW, "parking areas fit in the stage ring");
        TO* aux = static_cast<TO*>(p.aux);
        if ((p.n * sizeof(TO)) % 16 == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0 && (reinterpret_cast<uintptr_t>(aux) & 15) == 0) {
            __syncthreads();                                                 // every wave has left the ring
            TO* park_a = reinterpret_cast<TO*>(lds) + wave * 2 * AREA;
            TO* park_b = park_a + AREA;
            auto put = [&](TO* park, const float (&v)[16]) {
#pragma unroll
                for (int r4 = 0; r4 < 4; ++r4) {
                    const float q[4] = {v[4 * r4], v[4 * r4 + 1], v[4 * r4 + 2], v[4 * r4 + 3]};
                    Quad<TO>::store(&park[l32 * PLD + r4 * 8 + lhi * 4], q);
                }
            };
            auto get = [&](const TO* park, float (&v)[16]) {
#pragma unroll
                for (int r4 = 0; r4 < 4; ++r4) {
                    float q[4];
                    Quad<TO>::load(&park[l32 * PLD + r4 * 8 + lhi * 4], q);
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[4 * r4 + e] = q[e];
                }
            };
            // parked sub-tile -> rows row0 .. row0 + 31, columns col0 .. col0 + 31 of dst (row stride ld); p.n is a
            // multiple of the piece, so a piece is inside or outside as a whole
            auto flush = [&](const TO* park, TO* dst, int64_t ld, int64_t row0, int64_t col0) {
#pragma unroll
                for (int it = 0; it < 32 * PIECES / WAVE; ++it) {
                    const int id = it * WAVE + lane, pr = id / PIECES, pc = id % PIECES;
                    const int64_t mrow = row0 + pr, ncol = col0 + pc * PER;
                    const uint4 piece = *reinterpret_cast<const uint4*>(&park[pr * PLD + pc * PER]);
                    if (mrow < m_end && ncol < p.n) store_streaming(dst + mrow * ld + ncol, piece);
                }
            };
            auto fetch = [&](TO* park, const TO* src, int64_t ld, int64_t row0, int64_t col0) {
#pragma unroll
                for (int it = 0; it < 32 * PIECES / WAVE; ++it) {
                    const int id = it * WAVE + lane, pr = id / PIECES, pc = id % PIECES;
                    const int64_t mrow = row0 + pr, ncol = col0 + pc * PER;
                    uint4 piece = make_uint4(0u, 0u, 0u, 0u);
                    if (mrow < m_end && ncol < p.n) piece = *reinterpret_cast<const uint4*>(src + mrow * ld + ncol);
                    *reinterpret_cast<uint4*>(&park[pr * PLD + pc * PER]) = piece;
                }
            };
            if constexpr (GATED) {
                const int64_t col0 = n_begin + wn * 32;
                float bias_g[16], bias_u[16];
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int64_t ncol = col0 + (r / 4) * 8 + lhi * 4 + r % 4;
                    const bool inside = p.bias && ncol < p.n;
                    bias_g[r] = inside ? load_bias(p.bias, ncol, bias_dtype) : 0.0f;
                    bias_u[r] = inside ? load_bias(p.bias, p.n + ncol, bias_dtype) : 0.0f;
                }
#pragma unroll
                for (int j = 0; j < TM; ++j) {
                    float g[16], u[16], h[16];
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        float gv = total[0][j][r], uv = total[1][j][r];
                        if (p.bias) { gv += bias_g[r]; uv += bias_u[r]; }
                        g[r] = rounded<TO>(gv);
                        u[r] = rounded<TO>(uv);
                        float act, derivative;
                        gate_math(p.activation, g[r], act, derivative);
                        h[r] = act * u[r];
                        // an FP32 value of its own: folded into a narrowing conversion (a mixed-precision FMA with a +0
                        // addend) the product would round once instead of twice and -0 would become +0
                        asm volatile("" : "+v"(h[r]));
                    }
                    const int64_t row0 = m_begin + a_sub(j);
                    put(park_a, h);
                    bool encoded = false;
                    if constexpr (MX) {
                        if (p.enc) {
                            // The rounded h goes out as FP8 codes with E8M0 scales instead (viola/nn/_mlp_kernels.py:195-230).
                            // The wave's 32 columns are one group of a row: lanes l32 and l32 + 32 hold its two halves.
                            encoded = true;
                            const float limit = p.enc_limit;
                            auto encode_words = [&](const float (&v)[16], float s, float poison, uint32_t (&w)[4]) {
                                const SharedDivisor dv(s, poison);
                                if (__builtin_amdgcn_ballot_w64(!dv.fast) == 0) {
#pragma unroll
                                    for (int q = 0; q < 4; ++q)
                                        w[q] = p.enc_bf8 ? fast_encode4<e5m2_t>(dv, limit, v[4 * q], v[4 * q + 1], v[4 * q + 2], v[4 * q + 3])
                                                         : fast_encode4<e4m3_t>(dv, limit, v[4 * q], v[4 * q + 1], v[4 * q + 2], v[4 * q + 3]);
                                } else {
#pragma unroll
                                    for (int q = 0; q < 4; ++q) {
                                        w[q] = 0;
#pragma unroll
                                        for (int e = 0; e < 4; ++e)
                                            w[q] |= (uint32_t)(p.enc_bf8 ? encode_clamped<e5m2_t>(v[4 * q + e], s, limit)
                                                                         : encode_clamped<e4m3_t>(v[4 * q + e], s, limit)) << (8 * e);
                                    }
                                }
                            };
                            float hq[16];                                    // what the parked tile holds: h rounded to TO
                            float amax = 0.0f, poison = 0.0f;
#pragma unroll
                            for (int r = 0; r < 16; ++r) {
                                hq[r] = rounded<TO>(h[r]);
                                amax = fmaxf(amax, fabsf(hq[r]));
                                poison = poison_of(poison, hq[r]);
                            }
                            amax = fmaxf(amax, __shfl_xor(amax, 32, WAVE));
                            poison += __shfl_xor(poison, 32, WAVE);
                            const float s_row = group_scale(amax, limit, 1);
                            uint32_t w[4];
                            encode_words(hq, s_row, poison, w);
                            // codes -> a byte tile [row][48] in the second area, then one 16-byte piece per lane to enc
                            uint8_t* bytes = reinterpret_cast<uint8_t*>(park_b);
                            constexpr int QLD = 48;
#pragma unroll
                            for (int q = 0; q < 4; ++q) *reinterpret_cast<uint32_t*>(&bytes[l32 * QLD + q * 8 + lhi * 4]) = w[q];
                            const int64_t grow = row0 + lane / 2;
                            const uint4 piece = *reinterpret_cast<const uint4*>(&bytes[(lane / 2) * QLD + (lane % 2) * 16]);
                            if (grow < m_end && col0 < p.n) *reinterpret_cast<uint4*>(p.enc + grow * p.n + col0 + (lane % 2) * 16) = piece;
                            if (lhi == 0 && row0 + l32 < m_end && col0 < p.n)
                                p.enc_scale[(row0 + l32) * (p.n / 32) + col0 / 32] = (uint8_t)(__float_as_uint(s_row) >> 23);
                            if (p.enc_t) {
                                // a column's 32 rows are one group of the transposed layout: lane (column l32, half lhi)
                                // collects rows 16 lhi .. 16 lhi + 15 of the parked h
                                float c[16];
                                float cmax = 0.0f, cpoison = 0.0f;
#pragma unroll
                                for (int r = 0; r < 16; ++r) {
                                    c[r] = to_f32(park_a[(lhi * 16 + r) * PLD + l32]);
                                    cmax = fmaxf(cmax, fabsf(c[r]));
                                    cpoison = poison_of(cpoison, c[r]);
                                }
                                cmax = fmaxf(cmax, __shfl_xor(cmax, 32, WAVE));
                                cpoison += __shfl_xor(cpoison, 32, WAVE);
                                const float s_col = group_scale(cmax, limit, 1);
                                uint32_t t[4];
                                encode_words(c, s_col, cpoison, t);
                                const int64_t gcol = col0 + l32;
                                if (gcol < p.n && row0 < m_end) {
                                    *reinterpret_cast<uint4*>(p.enc_t + gcol * p.m + row0 + lhi * 16) = make_uint4(t[0], t[1], t[2], t[3]);
                                    if (lhi == 0) p.enc_t_scale[gcol * (p.m / 32) + row0 / 32] = (uint8_t)(__float_as_uint(s_col) >> 23);
                                }
                            }
                        }
                    }
                    if (!encoded) flush(park_a, out, p.ldo, row0, col0);
                    if (aux) {
                        put(park_b, g);
                        flush(park_b, aux, 2 * p.n, row0, col0);
                        put(park_a, u);
                        flush(park_a, aux + p.n, 2 * p.n, row0, col0);
                    }
                }
            } else {
#pragma unroll
                for (int j = 0; j < TM; ++j) {
#pragma unroll
                    for (int i = 0; i < TN; ++i) {
                        const int64_t row0 = m_begin + a_sub(j), col0 = n_begin + b_sub(i);
                        fetch(park_a, aux, 2 * p.n, row0, col0);
                        fetch(park_b, aux + p.n, 2 * p.n, row0, col0);
                        float g[16], u[16], dg[16], du[16];
                        get(park_a, g);
                        get(park_b, u);
#pragma unroll
                        for (int r = 0; r < 16; ++r) {
                            const float d = rounded<TO>(total[i][j][r]);
                            float act, derivative;
                            gate_math(p.activation, g[r], act, derivative);
                            dg[r] = d * u[r] * derivative;
                            du[r] = d * act;
                        }
                        put(park_a, dg);
                        flush(park_a, out, p.ldo, row0, col0);
                        put(park_b, du);
                        flush(park_b, out + p.n, p.ldo, row0, col0);
                    }
                }
            }
            return;
        }
    }
#pragma unroll
    for (int j = 0; j < TM; ++j) {
        const int64_t mrow = m_begin + a_sub(j) + l32;
        if (mrow >= m_end) continue;
#pragma unroll
        for (int i = 0; i < (GATED ? 1 : TN); ++i)
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) {
            const int64_t ncol = n_begin + (GATED ? wn * 32 : b_sub(i)) + r4 * 8 + lhi * 4;
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
                for (int e = 0; e < 4; ++e) v[e] = total[i][j][r4 * 4 + e];
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

}  // namespace viola
