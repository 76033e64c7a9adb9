// Grouped FP32-scale instances of the fast FP8 GEMM kernel (plain, gated forward, gated backward; uniform or
// row-wise b scales).
#include "gemm_fast_kernel.hpp"

namespace viola {

template <int MODE, bool B_ROWSCALE, typename TO, int TN, bool KSPLIT = false>
static void launch_formats(const GemmArgs& p, int a_dtype, int b_dtype, int bias_dtype, dim3 grid, hipStream_t stream) {
    const bool a5 = a_dtype == VIOLA_E5M2, b5 = b_dtype == VIOLA_E5M2;
    const dim3 block(KSPLIT ? 2 * FTHREADS : FTHREADS);
    if (!a5 && !b5) VIOLA_LAUNCH((group_gemm_fast<MODE, false, false, B_ROWSCALE, TO, TN, false, false, false, KSPLIT>), grid, block, 0, stream, p, bias_dtype);
    else if (a5 && !b5) VIOLA_LAUNCH((group_gemm_fast<MODE, true, false, B_ROWSCALE, TO, TN, false, false, false, KSPLIT>), grid, block, 0, stream, p, bias_dtype);
    else if (!a5 && b5) VIOLA_LAUNCH((group_gemm_fast<MODE, false, true, B_ROWSCALE, TO, TN, false, false, false, KSPLIT>), grid, block, 0, stream, p, bias_dtype);
    else VIOLA_LAUNCH((group_gemm_fast<MODE, true, true, B_ROWSCALE, TO, TN, false, false, false, KSPLIT>), grid, block, 0, stream, p, bias_dtype);
}

// plain mode, the k range of a tile split over two teams of waves
template <int TN>
static int launch_split(const GemmArgs& p, int a_dtype, int b_dtype, int bias_dtype, int out_dtype, bool rowscale, dim3 grid,
                        hipStream_t stream) {
#define VIOLA_SPLIT(TO)                                                                                         \
    if (rowscale) launch_formats<MODE_PLAIN, true, TO, TN, true>(p, a_dtype, b_dtype, bias_dtype, grid, stream); \
    else launch_formats<MODE_PLAIN, false, TO, TN, true>(p, a_dtype, b_dtype, bias_dtype, grid, stream);
    switch (out_dtype) {
        case VIOLA_F32: VIOLA_SPLIT(float) break;
        case VIOLA_BF16: VIOLA_SPLIT(bf16_t) break;
        case VIOLA_F16: VIOLA_SPLIT(f16_t) break;
        default: return VIOLA_EINVAL;
    }
#undef VIOLA_SPLIT
    return viola_launch_status();
}

template <int MODE, int TN>
static int launch_mode(const GemmArgs& p, int a_dtype, int b_dtype, int bias_dtype, int out_dtype, bool rowscale, dim3 grid,
                       hipStream_t stream) {
#define VIOLA_FAST(TO)                                                                           \
    if (rowscale) launch_formats<MODE, true, TO, TN>(p, a_dtype, b_dtype, bias_dtype, grid, stream); \
    else launch_formats<MODE, false, TO, TN>(p, a_dtype, b_dtype, bias_dtype, grid, stream);
    switch (out_dtype) {
        case VIOLA_F32: VIOLA_FAST(float) break;
        case VIOLA_BF16: VIOLA_FAST(bf16_t) break;
        case VIOLA_F16: VIOLA_FAST(f16_t) break;
        default: return VIOLA_EINVAL;
    }
#undef VIOLA_FAST
    return viola_launch_status();
}

// shortest k ranges worth splitting (4096 x 1024 tiles of 128 x 128: k = 1024 14.4 -> 15.1 us, k = 1536 17.7 -> 17.1 us; 1024 x 1024
// on 128 x 64 tiles: k = 512 slower, k = 1024 9.8 -> 9.1 us, k = 1536 12.6 -> 11.1 us)
constexpr int64_t SPLIT_MIN_K = 1536, NARROW_SPLIT_MIN_K = 1024;


int launch_group_gemm_fast(const GemmArgs& args, int mode, int a_dtype, int b_dtype, int bias_dtype, int out_dtype, bool rowscale,
                           dim3 grid, hipStream_t stream) {
    GemmArgs p = args;
    const int64_t b_rows = mode == MODE_GATED_FWD ? 2 * p.n : p.n;
    p.sa_bytes = (p.m + p.ar - 1) / p.ar * p.ldsa * 4;
    p.sb_bytes = (b_rows + p.br - 1) / p.br * p.ldsb * 4;
    // Two blocks fit a CU: with fewer than 512 tiles of 128 x 128, halve the tile in n so that all 256 CUs get two.
    // Over a long k, and with enough tiles to give half the CUs one each, keep the tile instead and split its k range inside
    // the block (one block of twice the waves per CU): 7-12 % faster from 256 tiles up at k >= 2048. With 128 tiles or fewer the
    // narrow tiles stay (more CUs busy) and their k range is split: a CU then holds eight waves instead of four
    // (1024 x 1024 x 16384: 98 -> 76 us, 512 x 512 x 4096: 27.5 -> 22.3 us).
    const int64_t tiles = (int64_t)grid.x * grid.y * grid.z;
    const bool few = mode == MODE_PLAIN && tiles < 512;
    const bool fixed_k = !p.offsets && !p.koffsets;
    const bool split = few && tiles > 128 && fixed_k && p.k >= SPLIT_MIN_K;
    const bool narrow = few && !split && p.n > 64;
    if (narrow) grid.x = (unsigned)((p.n + 63) / 64);
    if (!p.offsets && (int64_t)grid.x * grid.y < (1 << 30)) {
        p.tiles_n = (int)grid.x;
        p.tiles_m = (int)grid.y;
        grid = dim3((grid.x * grid.y + 7) / 8 * 8, 1, grid.z);
    }
    if (split) return launch_split<2>(p, a_dtype, b_dtype, bias_dtype, out_dtype, rowscale, grid, stream);
    if (narrow && fixed_k && p.k >= NARROW_SPLIT_MIN_K) return launch_split<1>(p, a_dtype, b_dtype, bias_dtype, out_dtype, rowscale, grid, stream);
    if (narrow) return launch_mode<MODE_PLAIN, 1>(p, a_dtype, b_dtype, bias_dtype, out_dtype, rowscale, grid, stream);
    if (mode == MODE_PLAIN) return launch_mode<MODE_PLAIN, 2>(p, a_dtype, b_dtype, bias_dtype, out_dtype, rowscale, grid, stream);
    if (mode == MODE_GATED_FWD) return launch_mode<MODE_GATED_FWD, 2>(p, a_dtype, b_dtype, bias_dtype, out_dtype, rowscale, grid, stream);
    return launch_mode<MODE_GATED_BWD, 2>(p, a_dtype, b_dtype, bias_dtype, out_dtype, rowscale, grid, stream);
}

}  // namespace viola
