// Shared between the generic and the fast grouped-scale FP8 GEMM translation units.
#pragma once
#include "common.hpp"

namespace viola {

typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int BM = 128, BN = 128;                                 // output tile of both kernels
enum { MODE_PLAIN = 0, MODE_GATED_FWD = 1, MODE_GATED_BWD = 2 };

struct GemmArgs {
    const uint8_t* a; const uint8_t* b; const float* sa; const float* sb;
    const void* bias; void* out; void* aux;
    int64_t m, n, k;              // n: rows of one b panel (h for the gated modes)
    int64_t lda, ldb;             // bytes between rows of a / b
    int64_t ldsa, ldsb;           // floats between rows of sa / sb
    int64_t ldo;                  // elements between rows of out
    int ar, br, ak_shift, bk_shift;
    int activation;
    // variable-group row ranges (grid.y walks the tiles of all groups)
    const int64_t* offsets; int groups; int64_t b_group_stride, sb_group_stride;
    // variable-group K ranges (grid.z = group): k range [koffsets[g], koffsets[g+1])
    const int64_t* koffsets; int64_t out_group_stride;
    // fast kernel only: 1-D grid of tiles_m * tiles_n output tiles (rounded up to a multiple of 8) walked in an
    // XCD-aware order; tiles_m == 0 keeps the plain (blockIdx.x, blockIdx.y) = (n tile, m tile) mapping
    int tiles_m, tiles_n;
    // fast kernel only, filled in by its launchers: bytes of the two scale arrays (a 16-byte piece may reach past the
    // last scale row and must then read zero, so their buffer descriptors carry the true size)
    int64_t sa_bytes, sb_bytes;
    // MX gated forward only: when enc is set, h is not written to out but quantized in the epilogue with E8M0
    // scales per 32 values, along its rows (enc [m, n], enc_scale [m, n / 32]) and along its columns
    // (enc_t [n, m], enc_t_scale [n, m / 32]; enc_t may be null); m and n are multiples of 32
    uint8_t* enc; uint8_t* enc_scale; uint8_t* enc_t; uint8_t* enc_t_scale; float enc_limit; int enc_bf8;
    // FP16-accumulator model of the generic kernel (HALF != 0): k covered by one FP16 partial sum before it is added to
    // the running total (0: the whole k range, no separate total), and whether that total is kept in bf16
    int half_period; int reduce_bf16;
};


// Fast path (16-byte aligned operands, k ranges multiples of 16). Defined in gemm_fast.hip.
int launch_group_gemm_fast(const GemmArgs& p, int mode, int a_dtype, int b_dtype, int bias_dtype, int out_dtype,
                           bool rowscale, dim3 grid, hipStream_t stream);

// Per-tensor scales on the same fast kernel (one v_mfma_f32_32x32x64_f8f6f4 per sub-tile and 64 k); mode = MODE_PLAIN or a
// gated mode (grid.x then counts the gated tile width). Defined in gemm_fast.hip.
int launch_tensor_gemm_fast(const GemmArgs& p, int mode, int a_dtype, int b_dtype, int bias_dtype, int out_dtype, dim3 grid,
                            hipStream_t stream);

// E8M0 block scales applied by v_mfma_scale_f32_32x32x64_f8f6f4 (k a multiple of 128). Defined in gemm_fast.hip.
int launch_mx_gemm_fast(const GemmArgs& p, int mode, int a_dtype, int b_dtype, int bias_dtype, int out_dtype, dim3 grid,
                        hipStream_t stream);

// misc.hip: the gated activation as a pass of its own, in 16-byte pieces (false: alignment does not allow them);
// epilogue_form: forward silu in the gated GEMM epilogue's expression instead of the stand-alone operator's
bool launch_gated_pieces(const void* z, const void* dy, int64_t dy_stride, void* out, int64_t rows, int64_t h, int dtype,
                         int activation, bool backward, bool epilogue_form, hipStream_t stream);

// Per-tensor and block-scaled products with at least this many 256 x 256 output tiles (two rounds of the 256 CUs)
// run on the large tile.
#ifndef VIOLA_BIG_TILES_FROM
#define VIOLA_BIG_TILES_FROM (2 * 256)
#endif
inline bool takes_large_tiles(int64_t m, int64_t n) { return ((m + 255) / 256) * ((n + 255) / 256) >= VIOLA_BIG_TILES_FROM; }

}  // namespace viola
