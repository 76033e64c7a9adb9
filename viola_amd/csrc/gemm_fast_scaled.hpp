// Launchers of the fast FP8 GEMM kernel for the recipes whose scales need no per-group fold: per-tensor scales and
// E8M0 block scales. Included by the one file that instantiates each.
#pragma once
#include "gemm_fast_kernel.hpp"

namespace viola {

// Per-tensor scales (TENSOR: args.sa / args.sb point at one float each) or E8M0 block scales (MX: they point at
// bytes; ldsa / ldsb = bytes per scale row). grid: (n tiles, m tiles of 128); n tiles are 128 wide, 64 for gated forward.
// KSPLIT: the k range of a 128 x 128 tile split over two teams of waves in a 512-thread block (plain mode)
template <int MODE, typename TO, int TN, bool TENSOR, bool MX, bool KSPLIT = false>
static void launch_scaled_formats(const GemmArgs& p, int a_dtype, int b_dtype, int bias_dtype, dim3 grid, hipStream_t stream) {
    const bool a5 = a_dtype == VIOLA_E5M2, b5 = b_dtype == VIOLA_E5M2;
    const dim3 block(KSPLIT ? 2 * FTHREADS : FTHREADS);
    if (!a5 && !b5) VIOLA_LAUNCH((group_gemm_fast<MODE, false, false, false, TO, TN, TENSOR, MX, false, KSPLIT>), grid, block, 0, stream, p, bias_dtype);
    else if (a5 && !b5) VIOLA_LAUNCH((group_gemm_fast<MODE, true, false, false, TO, TN, TENSOR, MX, false, KSPLIT>), grid, block, 0, stream, p, bias_dtype);
    else if (!a5 && b5) VIOLA_LAUNCH((group_gemm_fast<MODE, false, true, false, TO, TN, TENSOR, MX, false, KSPLIT>), grid, block, 0, stream, p, bias_dtype);
    else VIOLA_LAUNCH((group_gemm_fast<MODE, true, true, false, TO, TN, TENSOR, MX, false, KSPLIT>), grid, block, 0, stream, p, bias_dtype);
}

// The 256 x 256 tile (one 512-thread block per CU) for products with at least two rounds of such tiles (8192 x 4096 x 1024: 52.9 us against 58.5; with fewer tiles the 128 x 128 kernel wins).
template <int MODE, typename TO, bool TENSOR, bool MX>
static void launch_big_formats(const GemmArgs& p, int a_dtype, int b_dtype, int bias_dtype, dim3 grid, hipStream_t stream) {
    const bool a5 = a_dtype == VIOLA_E5M2, b5 = b_dtype == VIOLA_E5M2;
    if (!a5 && !b5) VIOLA_LAUNCH((group_gemm_fast<MODE, false, false, false, TO, 2, TENSOR, MX, true>), grid, dim3(512), 0, stream, p, bias_dtype);
    else if (a5 && !b5) VIOLA_LAUNCH((group_gemm_fast<MODE, true, false, false, TO, 2, TENSOR, MX, true>), grid, dim3(512), 0, stream, p, bias_dtype);
    else if (!a5 && b5) VIOLA_LAUNCH((group_gemm_fast<MODE, false, true, false, TO, 2, TENSOR, MX, true>), grid, dim3(512), 0, stream, p, bias_dtype);
    else VIOLA_LAUNCH((group_gemm_fast<MODE, true, true, false, TO, 2, TENSOR, MX, true>), grid, dim3(512), 0, stream, p, bias_dtype);
}

#ifndef VIOLA_SCALED_SPLIT_MIN_K
#define VIOLA_SCALED_SPLIT_MIN_K 2048
#endif
#ifndef VIOLA_MX_BIG_GATED
#define VIOLA_MX_BIG_GATED 0
#endif
// which gated kernels exist on the large tile: all per-tensor ones; of the block-scaled ones those whose registers fit
constexpr bool big_gated(bool mx, int mode) { return !mx || (VIOLA_MX_BIG_GATED >> (mode == MODE_GATED_FWD ? 0 : 1) & 1); }

template <typename TO, bool TENSOR, bool MX>
static void launch_big_modes(const GemmArgs& p, int mode, int a_dtype, int b_dtype, int bias_dtype, dim3 grid, hipStream_t stream) {
    if (mode == MODE_PLAIN) launch_big_formats<MODE_PLAIN, TO, TENSOR, MX>(p, a_dtype, b_dtype, bias_dtype, grid, stream);
    else if (mode == MODE_GATED_FWD) {
        if constexpr (big_gated(MX, MODE_GATED_FWD)) launch_big_formats<MODE_GATED_FWD, TO, TENSOR, MX>(p, a_dtype, b_dtype, bias_dtype, grid, stream);
    } else {
        if constexpr (big_gated(MX, MODE_GATED_BWD)) launch_big_formats<MODE_GATED_BWD, TO, TENSOR, MX>(p, a_dtype, b_dtype, bias_dtype, grid, stream);
    }
}

template <bool TENSOR, bool MX>
static int launch_scaled_gemm_fast(const GemmArgs& args, int mode, int a_dtype, int b_dtype, int bias_dtype, int out_dtype, dim3 grid,
                                   hipStream_t stream) {
    GemmArgs p = args;
    {
        // MX: the scale arrays hold bytes; per-tensor scales are read directly, not through these descriptors
        const int64_t b_rows = mode == MODE_GATED_FWD ? 2 * p.n : p.n;
        p.sa_bytes = (p.m + p.ar - 1) / p.ar * p.ldsa;
        p.sb_bytes = (b_rows + p.br - 1) / p.br * p.ldsb;
    }
    // a gated forward tile is 128 columns of h wide (its 256 b rows are 128 gate and 128 up rows)
    const int64_t big_width = mode == MODE_GATED_FWD ? 128 : 256;
    const int64_t big_m = (p.m + 255) / 256, big_n = (p.n + big_width - 1) / big_width;
    // (the block-scaled gated kernels do not fit the large tile's register budget: their epilogues spill)
    if ((mode == MODE_PLAIN || big_gated(MX, mode)) && big_m * big_n >= VIOLA_BIG_TILES_FROM && big_m * big_n < (1 << 30) && 256 * p.k < (1ll << 31)) {
        p.tiles_n = (int)big_n;
        p.tiles_m = (int)big_m;
        const dim3 big_grid((unsigned)((big_m * big_n + 7) / 8 * 8), 1, 1);
        switch (out_dtype) {
            case VIOLA_F32: launch_big_modes<float, TENSOR, MX>(p, mode, a_dtype, b_dtype, bias_dtype, big_grid, stream); break;
            case VIOLA_BF16: launch_big_modes<bf16_t, TENSOR, MX>(p, mode, a_dtype, b_dtype, bias_dtype, big_grid, stream); break;
            case VIOLA_F16: launch_big_modes<f16_t, TENSOR, MX>(p, mode, a_dtype, b_dtype, bias_dtype, big_grid, stream); break;
            default: return VIOLA_EINVAL;
        }
        return viola_launch_status();
    }
    // fewer than 512 tiles of 128 x 128: halve the tile in n, or from 129 tiles up and over a long k keep the tile and
    // split its k range inside the block; the narrow tiles split a long k range as well (the grouped recipe's rule)
    const int64_t tiles = (int64_t)grid.x * grid.y;
    const bool few = mode == MODE_PLAIN && tiles < 512;
    const bool long_k = p.k >= VIOLA_SCALED_SPLIT_MIN_K;
    const bool split = few && tiles > 128 && long_k;
    const bool narrow = few && !split && p.n > 64;
    if (narrow) grid.x = (unsigned)((p.n + 63) / 64);
    if ((int64_t)grid.x * grid.y < (1 << 30)) {
        p.tiles_n = (int)grid.x;
        p.tiles_m = (int)grid.y;
        grid = dim3((grid.x * grid.y + 7) / 8 * 8, 1, 1);
    }
#define VIOLA_SCALED(TO)                                                                                                        \
    if (split) launch_scaled_formats<MODE_PLAIN, TO, 2, TENSOR, MX, true>(p, a_dtype, b_dtype, bias_dtype, grid, stream);        \
    else if (narrow && long_k) launch_scaled_formats<MODE_PLAIN, TO, 1, TENSOR, MX, true>(p, a_dtype, b_dtype, bias_dtype, grid, stream); \
    else if (narrow) launch_scaled_formats<MODE_PLAIN, TO, 1, TENSOR, MX>(p, a_dtype, b_dtype, bias_dtype, grid, stream);        \
    else if (mode == MODE_PLAIN) launch_scaled_formats<MODE_PLAIN, TO, 2, TENSOR, MX>(p, a_dtype, b_dtype, bias_dtype, grid, stream); \
    else if (mode == MODE_GATED_FWD) launch_scaled_formats<MODE_GATED_FWD, TO, 2, TENSOR, MX>(p, a_dtype, b_dtype, bias_dtype, grid, stream); \
    else launch_scaled_formats<MODE_GATED_BWD, TO, 2, TENSOR, MX>(p, a_dtype, b_dtype, bias_dtype, grid, stream);
    switch (out_dtype) {
        case VIOLA_F32: VIOLA_SCALED(float) break;
        case VIOLA_BF16: VIOLA_SCALED(bf16_t) break;
        case VIOLA_F16: VIOLA_SCALED(f16_t) break;
        default: return VIOLA_EINVAL;
    }
#undef VIOLA_SCALED
    return viola_launch_status();
}

}  // namespace viola
