// Grouped-scale FP8 GEMM for gfx950 ("NT": out[m, n] = sum_k a[m, k] * b[n, k]) with FP32 scales
// per (row group, 32-wide K group) on both operands.
//
// Per 32-wide K group the raw code product is formed on the matrix cores
// (v_mfma_f32_32x32x16_fp8_fp8 twice) and folded into an FP32 total with one VALU FMA per output
// element: total += acc * (sa * sb). The FP32 scales cannot be applied inside a wider MFMA, so the
// K = 32 instructions are the ones that fit this contract.
//
// Orientation: the B matrix (rows n) is fed as the MFMA "A" operand and the A matrix (rows m) as
// the MFMA "B" operand, so a lane's 16 accumulators of a 32 x 32 tile share one m and cover 16
// values of n inside one 32-row block of b. With 2-D weight blocks (br a multiple of 32) the scale
// product sa[m] * sb[block] is then a single per-lane scalar per K group.
//
// Block: 256 threads = 2 x 2 wavefronts, tile 128 (m) x 128 (b rows) x 64 (k), two LDS stages,
// global loads for chunk i+1 issued before the math of chunk i.
//
// One kernel template serves: the plain GEMM, the gated-MLP forward (two 64-row panels of b, gate
// and up, sharing a; epilogue act(g)*u), the gated-MLP backward (epilogue reads g,u and writes
// [d*u*act'(g), d*act(g)]), the variable-group row-range GEMM and the variable-group wgrad.
#include "gemm_args.hpp"

namespace viola {

constexpr int BK = 64, LDK = BK + 8, KG = BK / 32;

template <bool A_BF8, bool B_BF8>
__device__ __forceinline__ f32x16 mfma32(long x, long y, f32x16 c) {
    // x: 8 codes of the b matrix (MFMA srcA), y: 8 codes of the a matrix (MFMA srcB)
    if constexpr (!B_BF8 && !A_BF8) return __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(x, y, c, 0, 0, 0);
    else if constexpr (!B_BF8 && A_BF8) return __builtin_amdgcn_mfma_f32_32x32x16_fp8_bf8(x, y, c, 0, 0, 0);
    else if constexpr (B_BF8 && !A_BF8) return __builtin_amdgcn_mfma_f32_32x32x16_bf8_fp8(x, y, c, 0, 0, 0);
    else return __builtin_amdgcn_mfma_f32_32x32x16_bf8_bf8(x, y, c, 0, 0, 0);
}

__device__ __forceinline__ float load_dtype(const void* p, int64_t i, int dtype) {
    if (dtype == VIOLA_F32) return static_cast<const float*>(p)[i];
    if (dtype == VIOLA_BF16) return bf16_bits_to_f32(static_cast<const uint16_t*>(p)[i]);
    return (float)static_cast<const _Float16*>(p)[i];
}

__device__ __forceinline__ void activation_pair(int activation, float g, float& act, float& derivative) {
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

template <typename TO> __device__ __forceinline__ float round_through(float v) { return to_f32(from_f32<TO>(v)); }

// A_BF8/B_BF8: operand formats (false = e4m3, true = e5m2). B_ROWSCALE: b scales vary inside a 32-row block.
// VEC: 16-byte global loads are legal (k ranges and row strides multiples of 16, aligned bases).
//
// HALF models the reference's accum_dtype="fp16" (viola/nn/_grouped_kernels.py:268-292, _linear_kernels.py:139-155,
// :198-211): its FP8 tensor-core instruction covers 32 k and, with an FP16 accumulator, returns
// fp16(accumulator + the 32 products); the accumulator is cleared after `half_period` k, when it is added to a
// running total held in FP32 or bf16 (rounded after every addition). HALF == 1 is the grouped recipe (a period is one
// scale group: the partial is scaled by sa * sb as it is added, (partial * sa) * sb), HALF == 2 the per-tensor recipe
// (scales applied to the finished total; half_period == 0: one partial over the whole k range and no total). Here the
// 32 products are summed in FP32 by the MFMA and rounded once, which is that instruction's best case; where the
// hardware's own sum is coarser the reference's results differ, inside the bound its checks allow (.01).
template <int MODE, bool A_BF8, bool B_BF8, bool B_ROWSCALE, bool VEC, typename TO, int HALF = 0>
__global__ __launch_bounds__(256, 2) void group_gemm_kernel(GemmArgs p, int bias_dtype) {
    static_assert(HALF == 0 || MODE == MODE_PLAIN, "the FP16-accumulator model is built for the plain product");
    __shared__ __attribute__((aligned(16))) uint8_t lds_a[2][BM * LDK];
    __shared__ __attribute__((aligned(16))) uint8_t lds_b[2][BN * LDK];
    __shared__ __attribute__((aligned(16))) float lds_sa[2][KG][BM];
    __shared__ __attribute__((aligned(16))) float lds_sb[2][KG][BN];

    constexpr int PANEL = MODE == MODE_GATED_FWD ? BN / 2 : BN;       // b rows per panel in the tile
    const int tid = threadIdx.x, lane = tid % WAVE, wave = tid / WAVE;
    const int wm = wave / 2, wn = wave % 2;
    const int l32 = lane % 32, lhi = lane / 32;

    // ---- which problem / tile
    int64_t m_begin = (int64_t)blockIdx.y * BM, m_end = p.m;
    int64_t k_begin = 0, k_end = p.k;
    const uint8_t* bptr = p.b;
    const float* sbptr = p.sb;
    uint8_t* outptr = static_cast<uint8_t*>(p.out);
    if (p.offsets) {
        int64_t tile = blockIdx.y;
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
    const int64_t n_begin = (int64_t)blockIdx.x * PANEL;

    // global row of tile-local b row `lr`
    auto b_row = [&](int lr) -> int64_t {
        if constexpr (MODE == MODE_GATED_FWD) return (int64_t)(lr / PANEL) * p.n + n_begin + lr % PANEL;
        else return n_begin + lr;
    };
    const int64_t b_rows_total = MODE == MODE_GATED_FWD ? 2 * p.n : p.n;
    auto b_row_valid = [&](int lr) -> bool {
        if constexpr (MODE == MODE_GATED_FWD) return n_begin + lr % PANEL < p.n;
        else return n_begin + lr < p.n;
    };

    // ---- staging registers for the next chunk
    uint4 ra[2], rb[2];
    float rsa, rsb;
    auto fetch = [&](int64_t k0) {
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            const int id = it * 256 + tid;
            const int lr = id / 4, c = id % 4;
            const int64_t kk = k0 + c * 16;
            int64_t am = m_begin + lr;
            am = am < m_end ? am : m_end - 1;
            int64_t bn = b_row(lr);
            bn = bn < b_rows_total ? bn : b_rows_total - 1;
            if constexpr (VEC) {
                ra[it] = kk < k_end ? *reinterpret_cast<const uint4*>(p.a + am * p.lda + kk) : make_uint4(0, 0, 0, 0);
                rb[it] = kk < k_end ? *reinterpret_cast<const uint4*>(bptr + bn * p.ldb + kk) : make_uint4(0, 0, 0, 0);
            } else {
                uint32_t wa[4] = {0, 0, 0, 0}, wb[4] = {0, 0, 0, 0};
                for (int i = 0; i < 16; ++i) {
                    if (kk + i < k_end) {
                        wa[i / 4] |= (uint32_t)p.a[am * p.lda + kk + i] << (8 * (i % 4));
                        wb[i / 4] |= (uint32_t)bptr[bn * p.ldb + kk + i] << (8 * (i % 4));
                    }
                }
                ra[it] = make_uint4(wa[0], wa[1], wa[2], wa[3]);
                rb[it] = make_uint4(wb[0], wb[1], wb[2], wb[3]);
            }
        }
        {
            const int kg = tid / BM, lr = tid % BM;                    // KG * 128 == 256 entries each
            const int64_t kk = k0 + kg * 32;
            int64_t am = m_begin + lr;
            am = am < m_end ? am : m_end - 1;
            int64_t bn = b_row(lr);
            bn = bn < b_rows_total ? bn : b_rows_total - 1;
            rsa = kk < k_end ? p.sa[am / p.ar * p.ldsa + (kk >> p.ak_shift)] : 0.0f;
            rsb = kk < k_end ? sbptr[bn / p.br * p.ldsb + (kk >> p.bk_shift)] : 0.0f;
        }
    };
    auto stash = [&](int s) {
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            const int id = it * 256 + tid;
            const int lr = id / 4, c = id % 4;
            uint2* da = reinterpret_cast<uint2*>(&lds_a[s][lr * LDK + c * 16]);
            da[0] = make_uint2(ra[it].x, ra[it].y);
            da[1] = make_uint2(ra[it].z, ra[it].w);
            uint2* db = reinterpret_cast<uint2*>(&lds_b[s][lr * LDK + c * 16]);
            db[0] = make_uint2(rb[it].x, rb[it].y);
            db[1] = make_uint2(rb[it].z, rb[it].w);
        }
        lds_sa[s][tid / BM][tid % BM] = rsa;
        lds_sb[s][tid / BM][tid % BM] = rsb;
    };

    // tile-local b row of this wavefront's sub-tile i (32 rows each)
    auto b_sub = [&](int i) -> int {
        if constexpr (MODE == MODE_GATED_FWD) return i * PANEL + wn * 32;   // i = 0 gate, 1 up
        else return wn * 64 + i * 32;
    };

    f32x16 total[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) total[i][j][r] = 0.0f;

    // HALF: the FP16 partial sums (kept as the floats they round to)
    f32x16 partial[HALF ? 2 : 1][HALF ? 2 : 1];
    if constexpr (HALF != 0) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) partial[i][j][r] = 0.0f;
    }
    auto to_half = [](float v) -> float { return (float)(_Float16)v; };
    auto reduced = [&](float v) -> float { return p.reduce_bf16 ? bf16_bits_to_f32(f32_to_bf16_bits(v)) : v; };

    const int64_t chunks = (k_end - k_begin + BK - 1) / BK;
    if (chunks > 0) {
        fetch(k_begin);
        stash(0);
    }
    __syncthreads();
    for (int64_t chunk = 0; chunk < chunks; ++chunk) {
        const int s = (int)(chunk & 1);
        if (chunk + 1 < chunks) fetch(k_begin + (chunk + 1) * BK);
#pragma unroll
        for (int kg = 0; kg < KG; ++kg) {
            f32x16 acc[2][2];
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                const int koff = kg * 32 + ks * 16 + lhi * 8;
                long opb[2], opa[2];
#pragma unroll
                for (int i = 0; i < 2; ++i) opb[i] = *reinterpret_cast<const long*>(&lds_b[s][(b_sub(i) + l32) * LDK + koff]);
#pragma unroll
                for (int j = 0; j < 2; ++j) opa[j] = *reinterpret_cast<const long*>(&lds_a[s][(wm * 64 + j * 32 + l32) * LDK + koff]);
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int j = 0; j < 2; ++j) {
                        if (ks == 0) {
                            f32x16 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                            acc[i][j] = mfma32<A_BF8, B_BF8>(opb[i], opa[j], zero);
                        } else {
                            acc[i][j] = mfma32<A_BF8, B_BF8>(opb[i], opa[j], acc[i][j]);
                        }
                    }
            }
            if constexpr (HALF != 0) {
                // this 32-k step joins the FP16 partial; at the end of a period (and of the k range) the partial joins the total
                const int64_t done = chunk * BK + kg * 32 + 32;                  // k covered so far, relative to k_begin
                const bool last = done >= k_end - k_begin;
                const bool flush = p.half_period ? (done % p.half_period == 0 || last) : false;
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const float sa_l = lds_sa[s][kg][wm * 64 + j * 32 + l32];
#pragma unroll
                    for (int i = 0; i < 2; ++i) {
#pragma unroll
                        for (int r = 0; r < 16; ++r) {
                            const float h = to_half(partial[i][j][r] + acc[i][j][r]);
                            partial[i][j][r] = h;
                            if (flush) {
                                float term = h;
                                if constexpr (HALF == 1) {
                                    const float sb_l = B_ROWSCALE ? lds_sb[s][kg][b_sub(i) + (r / 4) * 8 + lhi * 4 + r % 4] : lds_sb[s][kg][b_sub(i)];
                                    term = (h * sa_l) * sb_l;
                                }
                                total[i][j][r] = reduced(total[i][j][r] + term);
                                partial[i][j][r] = 0.0f;
                            }
                        }
                    }
                }
                continue;
            }
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const float sa_l = lds_sa[s][kg][wm * 64 + j * 32 + l32];
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    if constexpr (!B_ROWSCALE) {
                        const float sc = sa_l * lds_sb[s][kg][b_sub(i)];
#pragma unroll
                        for (int r = 0; r < 16; ++r) total[i][j][r] = fmaf(acc[i][j][r], sc, total[i][j][r]);
                    } else {
#pragma unroll
                        for (int r4 = 0; r4 < 4; ++r4) {
                            const float4 sb4 = *reinterpret_cast<const float4*>(&lds_sb[s][kg][b_sub(i) + r4 * 8 + lhi * 4]);
                            total[i][j][r4 * 4 + 0] = fmaf(acc[i][j][r4 * 4 + 0], sa_l * sb4.x, total[i][j][r4 * 4 + 0]);
                            total[i][j][r4 * 4 + 1] = fmaf(acc[i][j][r4 * 4 + 1], sa_l * sb4.y, total[i][j][r4 * 4 + 1]);
                            total[i][j][r4 * 4 + 2] = fmaf(acc[i][j][r4 * 4 + 2], sa_l * sb4.z, total[i][j][r4 * 4 + 2]);
                            total[i][j][r4 * 4 + 3] = fmaf(acc[i][j][r4 * 4 + 3], sa_l * sb4.w, total[i][j][r4 * 4 + 3]);
                        }
                    }
                }
            }
        }
        if (chunk + 1 < chunks) stash(s ^ 1);
        __syncthreads();
    }

    // ---- epilogue: lane holds m = l32 of sub-tile j, n = (r/4)*8 + lhi*4 + r%4 of sub-tile i
    TO* out = reinterpret_cast<TO*>(outptr);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int64_t mrow = m_begin + wm * 64 + j * 32 + l32;
        if (mrow >= m_end) continue;
        if constexpr (MODE == MODE_GATED_FWD) {
            TO* aux = static_cast<TO*>(p.aux);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int64_t ncol = n_begin + wn * 32 + (r / 4) * 8 + lhi * 4 + r % 4;
                if (ncol >= p.n) continue;
                float gv = total[0][j][r], uv = total[1][j][r];
                if (p.bias) {
                    gv += load_dtype(p.bias, ncol, bias_dtype);
                    uv += load_dtype(p.bias, p.n + ncol, bias_dtype);
                }
                const TO gq = from_f32<TO>(gv), uq = from_f32<TO>(uv);
                if (aux) {
                    aux[mrow * 2 * p.n + ncol] = gq;
                    aux[mrow * 2 * p.n + p.n + ncol] = uq;
                }
                float act, derivative;
                activation_pair(p.activation, to_f32(gq), act, derivative);
                out[mrow * p.ldo + ncol] = from_f32<TO>(act * to_f32(uq));
            }
        } else {
#pragma unroll
            for (int i = 0; i < 2; ++i) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int64_t ncol = n_begin + wn * 64 + i * 32 + (r / 4) * 8 + lhi * 4 + r % 4;
                    if (ncol >= p.n) continue;
                    float v = total[i][j][r];
                    if constexpr (HALF == 2) {
                        v = p.half_period ? v : partial[i][j][r];
                        v = (v * p.sa[0]) * p.sb[0];
                    }
                    if constexpr (MODE == MODE_PLAIN) {
                        if (p.bias) v += load_dtype(p.bias, ncol, bias_dtype);
                        out[mrow * p.ldo + ncol] = from_f32<TO>(v);
                    } else {
                        const TO* aux = static_cast<const TO*>(p.aux);
                        const float d = round_through<TO>(v);
                        const float g = to_f32(aux[mrow * 2 * p.n + ncol]);
                        const float u = to_f32(aux[mrow * 2 * p.n + p.n + ncol]);
                        float act, derivative;
                        activation_pair(p.activation, g, act, derivative);
                        out[mrow * p.ldo + ncol] = from_f32<TO>(d * u * derivative);
                        out[mrow * p.ldo + p.n + ncol] = from_f32<TO>(d * act);
                    }
                }
            }
        }
    }
}

static int shift_of(int v) {
    int s = 0;
    while ((1 << s) < v) ++s;
    return s;
}

template <int MODE, bool B_ROWSCALE, bool VEC, typename TO>
static void launch_formats(const GemmArgs& p, int a_dtype, int b_dtype, int bias_dtype, dim3 grid, hipStream_t stream) {
    const bool a5 = a_dtype == VIOLA_E5M2, b5 = b_dtype == VIOLA_E5M2;
    if (!a5 && !b5) VIOLA_LAUNCH((group_gemm_kernel<MODE, false, false, B_ROWSCALE, VEC, TO>), grid, dim3(256), 0, stream, p, bias_dtype);
    else if (a5 && !b5) VIOLA_LAUNCH((group_gemm_kernel<MODE, true, false, B_ROWSCALE, VEC, TO>), grid, dim3(256), 0, stream, p, bias_dtype);
    else if (!a5 && b5) VIOLA_LAUNCH((group_gemm_kernel<MODE, false, true, B_ROWSCALE, VEC, TO>), grid, dim3(256), 0, stream, p, bias_dtype);
    else VIOLA_LAUNCH((group_gemm_kernel<MODE, true, true, B_ROWSCALE, VEC, TO>), grid, dim3(256), 0, stream, p, bias_dtype);
}

template <int MODE, typename TO>
static void launch_paths(const GemmArgs& p, int a_dtype, int b_dtype, int bias_dtype, bool rowscale, dim3 grid, hipStream_t stream) {
    // the generic kernel is only built with guarded byte loads; aligned problems take the fast kernel
    if (rowscale) launch_formats<MODE, true, false, TO>(p, a_dtype, b_dtype, bias_dtype, grid, stream);
    else launch_formats<MODE, false, false, TO>(p, a_dtype, b_dtype, bias_dtype, grid, stream);
}

template <int MODE>
static int launch_out(const GemmArgs& p, int a_dtype, int b_dtype, int bias_dtype, int out_dtype, bool rowscale, bool vec,
                      dim3 grid, hipStream_t stream) {
    const int64_t b_rows = MODE == MODE_GATED_FWD ? 2 * p.n : p.n;
    // the fast kernel addresses operands and scales with 31-bit byte offsets
    const bool small = b_rows * p.ldb < (1ll << 31) && (int64_t)BM * p.lda < (1ll << 31) &&
                       (p.m + p.ar - 1) / p.ar * p.ldsa * 4 < (1ll << 31) && (b_rows + p.br - 1) / p.br * p.ldsb * 4 < (1ll << 31) &&
                       p.ak_shift == 5 && p.bk_shift == 5;         // and stages the scales of 8 consecutive 32-wide K groups at once
    if (vec && small)
        return launch_group_gemm_fast(p, MODE, a_dtype, b_dtype, bias_dtype, out_dtype, rowscale, grid, stream);
    switch (out_dtype) {
        case VIOLA_F32: launch_paths<MODE, float>(p, a_dtype, b_dtype, bias_dtype, rowscale, grid, stream); break;
        case VIOLA_BF16: launch_paths<MODE, bf16_t>(p, a_dtype, b_dtype, bias_dtype, rowscale, grid, stream); break;
        case VIOLA_F16: launch_paths<MODE, f16_t>(p, a_dtype, b_dtype, bias_dtype, rowscale, grid, stream); break;
        default: return VIOLA_EINVAL;
    }
    return viola_launch_status();
}

// The FP16-accumulator model: always the generic kernel (an ablation option of the reference, not a fast path).
template <int HALF, bool B_ROWSCALE, typename TO>
static void launch_half_formats(const GemmArgs& p, int a_dtype, int b_dtype, int bias_dtype, dim3 grid, hipStream_t stream) {
    const bool a5 = a_dtype == VIOLA_E5M2, b5 = b_dtype == VIOLA_E5M2;
    if (!a5 && !b5) VIOLA_LAUNCH((group_gemm_kernel<MODE_PLAIN, false, false, B_ROWSCALE, false, TO, HALF>), grid, dim3(256), 0, stream, p, bias_dtype);
    else if (a5 && !b5) VIOLA_LAUNCH((group_gemm_kernel<MODE_PLAIN, true, false, B_ROWSCALE, false, TO, HALF>), grid, dim3(256), 0, stream, p, bias_dtype);
    else if (!a5 && b5) VIOLA_LAUNCH((group_gemm_kernel<MODE_PLAIN, false, true, B_ROWSCALE, false, TO, HALF>), grid, dim3(256), 0, stream, p, bias_dtype);
    else VIOLA_LAUNCH((group_gemm_kernel<MODE_PLAIN, true, true, B_ROWSCALE, false, TO, HALF>), grid, dim3(256), 0, stream, p, bias_dtype);
}

template <int HALF>
static int launch_half(const GemmArgs& p, int a_dtype, int b_dtype, int bias_dtype, int out_dtype, bool rowscale, dim3 grid,
                       hipStream_t stream) {
#define VIOLA_HALF(TO)                                                                                        \
    if (HALF == 1 && rowscale) launch_half_formats<HALF, HALF == 1, TO>(p, a_dtype, b_dtype, bias_dtype, grid, stream); \
    else launch_half_formats<HALF, false, TO>(p, a_dtype, b_dtype, bias_dtype, grid, stream);
    switch (out_dtype) {
        case VIOLA_F32: VIOLA_HALF(float) break;
        case VIOLA_BF16: VIOLA_HALF(bf16_t) break;
        case VIOLA_F16: VIOLA_HALF(f16_t) break;
        default: return VIOLA_EINVAL;
    }
#undef VIOLA_HALF
    return viola_launch_status();
}

static bool aligned16(const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; }
static bool pow2(int v) { return v > 0 && (v & (v - 1)) == 0; }

}  // namespace viola

using namespace viola;

extern "C" int viola_group_gemm(const void* a, int a_dtype, const void* b, int b_dtype, const float* sa, const float* sb,
                                int64_t m, int64_t n, int64_t k, int ar, int ak, int br, int bk, const void* bias,
                                int bias_dtype, void* out, int out_dtype, viola_stream_t stream_) {
    hipStream_t stream = viola_enter(stream_);
    VIOLA_CHECK_ARG(viola_is_fp8(a_dtype) && viola_is_fp8(b_dtype) && viola_is_float(out_dtype));
    VIOLA_CHECK_ARG(m >= 0 && n >= 0 && k >= 0 && ar > 0 && br > 0 && pow2(ak) && pow2(bk) && ak >= 32 && bk >= 32);
    VIOLA_CHECK_ARG(!bias || viola_is_float(bias_dtype));
    if (m == 0 || n == 0) return 0;
    VIOLA_CHECK_ARG(out && (k == 0 || (a && b && sa && sb)));
    const int64_t gy = (m + BM - 1) / BM, gx = (n + BN - 1) / BN;
    VIOLA_CHECK_ARG(gy <= 65535);
    GemmArgs p = {};
    p.a = static_cast<const uint8_t*>(a); p.b = static_cast<const uint8_t*>(b); p.sa = sa; p.sb = sb;
    p.bias = bias; p.out = out; p.m = m; p.n = n; p.k = k; p.lda = k; p.ldb = k;
    p.ldsa = (k + ak - 1) / ak; p.ldsb = (k + bk - 1) / bk; p.ldo = n;
    p.ar = ar; p.br = br; p.ak_shift = shift_of(ak); p.bk_shift = shift_of(bk);
    const bool vec = k % 16 == 0 && aligned16(a) && aligned16(b);
    const bool rowscale = br % 32 != 0;
    return launch_out<MODE_PLAIN>(p, a_dtype, b_dtype, bias_dtype, out_dtype, rowscale, vec, dim3((unsigned)gx, (unsigned)gy), stream);
}

static int gcd_of(int a, int b) { while (b) { const int t = a % b; a = b; b = t; } return a; }

extern "C" int viola_group_gemm_half(const void* a, int a_dtype, const void* b, int b_dtype, const float* sa, const float* sb,
                                     int64_t m, int64_t n, int64_t k, int ar, int ak, int br, int bk, const void* bias,
                                     int bias_dtype, void* out, int out_dtype, int accum_block, int reduce_dtype,
                                     viola_stream_t stream_) {
    hipStream_t stream = viola_enter(stream_);
    VIOLA_CHECK_ARG(viola_is_fp8(a_dtype) && viola_is_fp8(b_dtype) && viola_is_float(out_dtype));
    VIOLA_CHECK_ARG(m >= 0 && n >= 0 && k >= 0 && ar > 0 && br > 0 && pow2(ak) && pow2(bk) && ak >= 32 && bk >= 32);
    VIOLA_CHECK_ARG((!bias || viola_is_float(bias_dtype)) && accum_block >= 0 && accum_block % 32 == 0);
    VIOLA_CHECK_ARG(reduce_dtype == VIOLA_F32 || reduce_dtype == VIOLA_BF16);
    if (m == 0 || n == 0) return 0;
    VIOLA_CHECK_ARG(out && (k == 0 || (a && b && sa && sb)));
    const int64_t gy = (m + BM - 1) / BM, gx = (n + BN - 1) / BN;
    VIOLA_CHECK_ARG(gy <= 65535);
    GemmArgs p = {};
    p.a = static_cast<const uint8_t*>(a); p.b = static_cast<const uint8_t*>(b); p.sa = sa; p.sb = sb;
    p.bias = bias; p.out = out; p.m = m; p.n = n; p.k = k; p.lda = k; p.ldb = k;
    p.ldsa = (k + ak - 1) / ak; p.ldsb = (k + bk - 1) / bk; p.ldo = n;
    p.ar = ar; p.br = br; p.ak_shift = shift_of(ak); p.bk_shift = shift_of(bk);
    // the partial is cleared where the reference clears it: every gcd(a's K group, b's K group, accum_block) k
    p.half_period = accum_block ? gcd_of(gcd_of(ak, bk), accum_block) : gcd_of(ak, bk);
    p.reduce_bf16 = reduce_dtype == VIOLA_BF16;
    return launch_half<1>(p, a_dtype, b_dtype, bias_dtype, out_dtype, br % 32 != 0, dim3((unsigned)gx, (unsigned)gy), stream);
}

extern "C" int viola_tensor_gemm_half(const void* a, int a_dtype, const void* b, int b_dtype, const float* sa, const float* sb,
                                      int64_t m, int64_t n, int64_t k, const void* bias, int bias_dtype, void* out, int out_dtype,
                                      int accum_block, int reduce_dtype, viola_stream_t stream_) {
    hipStream_t stream = viola_enter(stream_);
    VIOLA_CHECK_ARG(viola_is_fp8(a_dtype) && viola_is_fp8(b_dtype) && viola_is_float(out_dtype));
    VIOLA_CHECK_ARG(m >= 0 && n >= 0 && k >= 0 && k < (1ll << 30) && (!bias || viola_is_float(bias_dtype)));
    VIOLA_CHECK_ARG(accum_block >= 0 && accum_block % 32 == 0 && (reduce_dtype == VIOLA_F32 || reduce_dtype == VIOLA_BF16));
    if (m == 0 || n == 0) return 0;
    VIOLA_CHECK_ARG(out && sa && sb && (k == 0 || (a && b)));
    const int64_t gy = (m + BM - 1) / BM, gx = (n + BN - 1) / BN;
    VIOLA_CHECK_ARG(gy <= 65535);
    GemmArgs p = {};
    p.a = static_cast<const uint8_t*>(a); p.b = static_cast<const uint8_t*>(b); p.sa = sa; p.sb = sb;
    p.bias = bias; p.out = out; p.m = m; p.n = n; p.k = k; p.lda = k; p.ldb = k; p.ldo = n;
    p.ldsa = 0; p.ldsb = 0; p.ar = 1 << 30; p.br = 1 << 30; p.ak_shift = 30; p.bk_shift = 30;
    // the reference's loop adds the partial to the total after whole chunks of 64 k (of accum_block k below that):
    // viola/nn/_linear_kernels.py:150-153, :272-273
    p.half_period = accum_block < 64 ? accum_block : accum_block / 64 * 64;
    p.reduce_bf16 = reduce_dtype == VIOLA_BF16;
    return launch_half<2>(p, a_dtype, b_dtype, bias_dtype, out_dtype, false, dim3((unsigned)gx, (unsigned)gy), stream);
}

// Large gated products run as the plain GEMM on 256 x 256 tiles plus one elementwise pass over its output: with one
// block per CU nothing covers a block's gated epilogue, and the pass costs less than that (MLP step at 16384 x 4096 ->
// 11008: 7.55 ms against 7.90 ms under per-tensor scales, 8.41 ms against 9.06 ms under MXFP8). No extra memory: forward
// the plain product is the [g | u] the caller keeps anyway, backward it lands in the up half of dz and is replaced there.
static bool gated_in_two_passes(int64_t m, int64_t n_plain, int64_t h, const void* aux, const void* out, int out_dtype) {
    const int64_t piece = out_dtype == VIOLA_F32 ? 4 : 8;
    return aux && takes_large_tiles(m, n_plain) && h % piece == 0 && aligned16(aux) && aligned16(out) &&
           m * (h / piece) / 256 < 0x7fffffff;                               // the pass is one launch of 256-thread blocks
}

static int tensor_gemm(const void* a, int a_dtype, const void* b, int b_dtype, const float* sa, const float* sb, int64_t m,
                       int64_t n, int64_t k, const void* bias, int bias_dtype, void* out, int64_t ldo, int out_dtype,
                       hipStream_t stream) {
    VIOLA_CHECK_ARG(viola_is_fp8(a_dtype) && viola_is_fp8(b_dtype) && viola_is_float(out_dtype));
    VIOLA_CHECK_ARG(m >= 0 && n >= 0 && k >= 0 && k < (1ll << 30) && (!bias || viola_is_float(bias_dtype)));
    if (m == 0 || n == 0) return 0;
    VIOLA_CHECK_ARG(out && sa && sb && (k == 0 || (a && b)));
    const int64_t gy = (m + BM - 1) / BM, gx = (n + BN - 1) / BN;
    VIOLA_CHECK_ARG(gy <= 65535);
    GemmArgs p = {};
    p.a = static_cast<const uint8_t*>(a); p.b = static_cast<const uint8_t*>(b); p.sa = sa; p.sb = sb;
    p.bias = bias; p.out = out; p.m = m; p.n = n; p.k = k; p.lda = k; p.ldb = k; p.ldo = ldo;
    // one scale group per operand: every (row, k) lands on scale index 0
    p.ldsa = 0; p.ldsb = 0; p.ar = 1 << 30; p.br = 1 << 30; p.ak_shift = 30; p.bk_shift = 30;
    const dim3 grid((unsigned)gx, (unsigned)gy);
    const bool vec = k % 16 == 0 && k > 0 && aligned16(a) && aligned16(b);
    if (vec && n * k < (1ll << 31) && (int64_t)BM * k < (1ll << 31))
        return launch_tensor_gemm_fast(p, MODE_PLAIN, a_dtype, b_dtype, bias_dtype, out_dtype, grid, stream);
    // odd alignment: the generic kernel, which multiplies each 32-wide K group's sum by sa * sb as it goes
    return launch_out<MODE_PLAIN>(p, a_dtype, b_dtype, bias_dtype, out_dtype, false, false, grid, stream);
}

extern "C" int viola_tensor_gemm(const void* a, int a_dtype, const void* b, int b_dtype, const float* sa, const float* sb,
                                 int64_t m, int64_t n, int64_t k, const void* bias, int bias_dtype, void* out, int out_dtype,
                                 viola_stream_t stream) {
    return tensor_gemm(a, a_dtype, b, b_dtype, sa, sb, m, n, k, bias, bias_dtype, out, n, out_dtype, static_cast<hipStream_t>(stream));
}

static int mx_gemm(const void* a, int a_dtype, const void* b, int b_dtype, const uint8_t* sa, const uint8_t* sb, int64_t m,
                   int64_t n, int64_t k, int ar, int br, const void* bias, int bias_dtype, void* out, int64_t ldo, int out_dtype,
                   hipStream_t stream) {
    VIOLA_CHECK_ARG(viola_is_fp8(a_dtype) && viola_is_fp8(b_dtype) && viola_is_float(out_dtype));
    VIOLA_CHECK_ARG(m >= 0 && n >= 0 && k >= 0 && ar > 0 && br > 0 && (!bias || viola_is_float(bias_dtype)));
    if (m == 0 || n == 0) return 0;
    VIOLA_CHECK_ARG(out && (k == 0 || (a && b && sa && sb)));
    const int64_t gy = (m + BM - 1) / BM, gx = (n + BN - 1) / BN;
    VIOLA_CHECK_ARG(gy <= 65535);
    // the block-scaled MFMA path only: whole 128-k scale pieces, 16-byte aligned codes, 4-byte aligned scale rows
    if (k == 0 || k % 128 != 0 || !aligned16(a) || !aligned16(b) || reinterpret_cast<uintptr_t>(sa) % 4 != 0 ||
        reinterpret_cast<uintptr_t>(sb) % 4 != 0 || n * k >= (1ll << 31) || (int64_t)BM * k >= (1ll << 31) ||
        (br != 1 && br % 32 != 0))
        return VIOLA_EUNSUPPORTED;
    GemmArgs p = {};
    p.a = static_cast<const uint8_t*>(a); p.b = static_cast<const uint8_t*>(b);
    p.sa = reinterpret_cast<const float*>(sa); p.sb = reinterpret_cast<const float*>(sb);
    p.bias = bias; p.out = out; p.m = m; p.n = n; p.k = k; p.lda = k; p.ldb = k; p.ldo = ldo;
    p.ldsa = k / 32; p.ldsb = k / 32; p.ar = ar; p.br = br; p.ak_shift = 5; p.bk_shift = 5;
    return launch_mx_gemm_fast(p, MODE_PLAIN, a_dtype, b_dtype, bias_dtype, out_dtype, dim3((unsigned)gx, (unsigned)gy), stream);
}

extern "C" int viola_mx_gemm(const void* a, int a_dtype, const void* b, int b_dtype, const uint8_t* sa, const uint8_t* sb,
                             int64_t m, int64_t n, int64_t k, int ar, int br, const void* bias, int bias_dtype, void* out,
                             int out_dtype, viola_stream_t stream) {
    return mx_gemm(a, a_dtype, b, b_dtype, sa, sb, m, n, k, ar, br, bias, bias_dtype, out, n, out_dtype, static_cast<hipStream_t>(stream));
}

// The two-pass form of a gated product; `plain(n, bias, out, ldo)` launches the plain GEMM of the recipe.
template <typename Plain>
static int gated_two_passes(Plain&& plain, int64_t m, int64_t h, const void* bias, void* aux, void* out, int out_dtype,
                            int activation, int backward, hipStream_t stream) {
    if (!backward) {
        const int status = plain(2 * h, bias, aux, 2 * h);                  // [g | u], biased
        if (status) return status;
        launch_gated_pieces(aux, nullptr, 0, out, m, h, out_dtype, activation, false, true, stream);
        return viola_launch_status();
    }
    uint8_t* up_half = static_cast<uint8_t*>(out) + h * (out_dtype == VIOLA_F32 ? 4 : 2);
    const int status = plain(h, nullptr, up_half, 2 * h);                   // dh, where d u will stand
    if (status) return status;
    launch_gated_pieces(aux, up_half, 2 * h, out, m, h, out_dtype, activation, true, true, stream);
    return viola_launch_status();
}

// The gated projections of an MLP under the per-tensor recipes: viola_gated_gemm's epilogues behind
// (acc * sa[0]) * sb[0].
extern "C" int viola_tensor_gated_gemm(const void* a, int a_dtype, const void* b, int b_dtype, const float* sa, const float* sb,
                                       int64_t m, int64_t h, int64_t k, const void* bias, int bias_dtype, void* aux, void* out,
                                       int out_dtype, int activation, int backward, viola_stream_t stream_) {
    hipStream_t stream = viola_enter(stream_);
    VIOLA_CHECK_ARG(viola_is_fp8(a_dtype) && viola_is_fp8(b_dtype) && viola_is_float(out_dtype));
    VIOLA_CHECK_ARG(m >= 0 && h >= 0 && k >= 0 && k < (1ll << 30));
    VIOLA_CHECK_ARG(activation >= VIOLA_SILU && activation <= VIOLA_RELU && (!bias || viola_is_float(bias_dtype)));
    if (m == 0 || h == 0) return 0;
    VIOLA_CHECK_ARG(out && sa && sb && (k == 0 || (a && b)) && (!backward || aux));
    GemmArgs p = {};
    p.a = static_cast<const uint8_t*>(a); p.b = static_cast<const uint8_t*>(b); p.sa = sa; p.sb = sb;
    p.bias = backward ? nullptr : bias; p.out = out; p.aux = aux; p.m = m; p.n = h; p.k = k; p.lda = k; p.ldb = k;
    p.ldo = backward ? 2 * h : h; p.activation = activation;
    p.ldsa = 0; p.ldsb = 0; p.ar = 1 << 30; p.br = 1 << 30; p.ak_shift = 30; p.bk_shift = 30;
    const int64_t gy = (m + BM - 1) / BM;
    VIOLA_CHECK_ARG(gy <= 65535);
    const int mode = backward ? MODE_GATED_BWD : MODE_GATED_FWD;
    const int64_t width = backward ? BN : BN / 2;
    const dim3 grid((unsigned)((h + width - 1) / width), (unsigned)gy);
    const bool vec = k % 16 == 0 && k > 0 && aligned16(a) && aligned16(b);
    if (vec && 2 * h * k < (1ll << 31) && (int64_t)BM * k < (1ll << 31)) {
        if (gated_in_two_passes(m, backward ? h : 2 * h, h, aux, out, out_dtype)) {
            auto plain = [&](int64_t n, const void* n_bias, void* to, int64_t ldo) {
                return tensor_gemm(a, a_dtype, b, b_dtype, sa, sb, m, n, k, n_bias, bias_dtype, to, ldo, out_dtype, stream);
            };
            return gated_two_passes(plain, m, h, bias, aux, out, out_dtype, activation, backward, stream);
        }
        return launch_tensor_gemm_fast(p, mode, a_dtype, b_dtype, bias_dtype, out_dtype, grid, stream);
    }
    if (backward) return launch_out<MODE_GATED_BWD>(p, a_dtype, b_dtype, bias_dtype, out_dtype, false, false, grid, stream);
    return launch_out<MODE_GATED_FWD>(p, a_dtype, b_dtype, bias_dtype, out_dtype, false, false, grid, stream);
}

// The same under E8M0 block scales; VIOLA_EUNSUPPORTED where viola_mx_gemm returns it, and when the up rows of b do
// not start on a scale-row boundary (h not a multiple of br).
extern "C" int viola_mx_gated_gemm(const void* a, int a_dtype, const void* b, int b_dtype, const uint8_t* sa, const uint8_t* sb,
                                   int64_t m, int64_t h, int64_t k, int ar, int br, const void* bias, int bias_dtype, void* aux,
                                   void* out, int out_dtype, int activation, int backward, viola_stream_t stream_) {
    hipStream_t stream = viola_enter(stream_);
    VIOLA_CHECK_ARG(viola_is_fp8(a_dtype) && viola_is_fp8(b_dtype) && viola_is_float(out_dtype));
    VIOLA_CHECK_ARG(m >= 0 && h >= 0 && k >= 0 && ar > 0 && br > 0);
    VIOLA_CHECK_ARG(activation >= VIOLA_SILU && activation <= VIOLA_RELU && (!bias || viola_is_float(bias_dtype)));
    if (m == 0 || h == 0) return 0;
    VIOLA_CHECK_ARG(out && (k == 0 || (a && b && sa && sb)) && (!backward || aux));
    const int64_t gy = (m + BM - 1) / BM;
    VIOLA_CHECK_ARG(gy <= 65535);
    if (k == 0 || k % 128 != 0 || !aligned16(a) || !aligned16(b) || reinterpret_cast<uintptr_t>(sa) % 4 != 0 ||
        reinterpret_cast<uintptr_t>(sb) % 4 != 0 || 2 * h * k >= (1ll << 31) || (int64_t)BM * k >= (1ll << 31) ||
        (br != 1 && br % 32 != 0) || (!backward && h % br != 0))
        return VIOLA_EUNSUPPORTED;
    if (gated_in_two_passes(m, backward ? h : 2 * h, h, aux, out, out_dtype)) {
        auto plain = [&](int64_t n, const void* n_bias, void* to, int64_t ldo) {
            return mx_gemm(a, a_dtype, b, b_dtype, sa, sb, m, n, k, ar, br, n_bias, bias_dtype, to, ldo, out_dtype, stream);
        };
        return gated_two_passes(plain, m, h, bias, aux, out, out_dtype, activation, backward, stream);
    }
    GemmArgs p = {};
    p.a = static_cast<const uint8_t*>(a); p.b = static_cast<const uint8_t*>(b);
    p.sa = reinterpret_cast<const float*>(sa); p.sb = reinterpret_cast<const float*>(sb);
    p.bias = backward ? nullptr : bias; p.out = out; p.aux = aux; p.m = m; p.n = h; p.k = k; p.lda = k; p.ldb = k;
    p.ldo = backward ? 2 * h : h; p.activation = activation;
    p.ldsa = k / 32; p.ldsb = k / 32; p.ar = ar; p.br = br; p.ak_shift = 5; p.bk_shift = 5;
    const int64_t width = backward ? BN : BN / 2;
    return launch_mx_gemm_fast(p, backward ? MODE_GATED_BWD : MODE_GATED_FWD, a_dtype, b_dtype, bias_dtype, out_dtype,
                               dim3((unsigned)((h + width - 1) / width), (unsigned)gy), stream);
}

extern "C" int viola_gated_gemm(const void* a, int a_dtype, const void* b, int b_dtype, const float* sa, const float* sb,
                                int64_t m, int64_t h, int64_t k, int ar, int ak, int br, int bk, const void* bias,
                                int bias_dtype, void* aux, void* out, int out_dtype, int activation, int backward,
                                viola_stream_t stream_) {
    hipStream_t stream = viola_enter(stream_);
    VIOLA_CHECK_ARG(viola_is_fp8(a_dtype) && viola_is_fp8(b_dtype) && viola_is_float(out_dtype));
    VIOLA_CHECK_ARG(m >= 0 && h >= 0 && k >= 0 && ar > 0 && br > 0 && pow2(ak) && pow2(bk) && ak >= 32 && bk >= 32);
    VIOLA_CHECK_ARG(activation >= VIOLA_SILU && activation <= VIOLA_RELU && (!bias || viola_is_float(bias_dtype)));
    if (m == 0 || h == 0) return 0;
    VIOLA_CHECK_ARG(out && (k == 0 || (a && b && sa && sb)) && (!backward || aux));
    GemmArgs p = {};
    p.a = static_cast<const uint8_t*>(a); p.b = static_cast<const uint8_t*>(b); p.sa = sa; p.sb = sb;
    p.bias = backward ? nullptr : bias; p.out = out; p.aux = aux; p.m = m; p.n = h; p.k = k; p.lda = k; p.ldb = k;
    p.ldsa = (k + ak - 1) / ak; p.ldsb = (k + bk - 1) / bk; p.ldo = backward ? 2 * h : h;
    p.ar = ar; p.br = br; p.ak_shift = shift_of(ak); p.bk_shift = shift_of(bk); p.activation = activation;
    const bool vec = k % 16 == 0 && aligned16(a) && aligned16(b);
    const int64_t gy = (m + BM - 1) / BM;
    VIOLA_CHECK_ARG(gy <= 65535);
    if (backward) {
        const bool rowscale = br % 32 != 0;
        return launch_out<MODE_GATED_BWD>(p, a_dtype, b_dtype, bias_dtype, out_dtype, rowscale, vec,
                                          dim3((unsigned)((h + BN - 1) / BN), (unsigned)gy), stream);
    }
    const bool rowscale = br % 32 != 0 || h % 32 != 0;
    return launch_out<MODE_GATED_FWD>(p, a_dtype, b_dtype, bias_dtype, out_dtype, rowscale, vec,
                                      dim3((unsigned)((h + BN / 2 - 1) / (BN / 2)), (unsigned)gy), stream);
}

// viola_mx_gated_gemm forward whose h leaves the kernel as FP8 codes with E8M0 scales in both layouts.
extern "C" int viola_mx_gated_gemm_encode(const void* a, int a_dtype, const void* b, int b_dtype, const uint8_t* sa, const uint8_t* sb,
                                          int64_t m, int64_t h, int64_t k, int ar, int br, const void* bias, int bias_dtype,
                                          void* aux, int aux_dtype, void* enc, uint8_t* enc_scale, void* enc_t,
                                          uint8_t* enc_t_scale, int enc_dtype, float limit, int activation,
                                          viola_stream_t stream_) {
    hipStream_t stream = viola_enter(stream_);
    VIOLA_CHECK_ARG(viola_is_fp8(a_dtype) && viola_is_fp8(b_dtype) && viola_is_float(aux_dtype) && viola_is_fp8(enc_dtype));
    VIOLA_CHECK_ARG(m >= 0 && h >= 0 && k >= 0 && ar > 0 && br > 0 && limit > 0.0f);
    VIOLA_CHECK_ARG(activation >= VIOLA_SILU && activation <= VIOLA_RELU && (!bias || viola_is_float(bias_dtype)));
    if (m == 0 || h == 0) return 0;
    VIOLA_CHECK_ARG(enc && enc_scale && (!enc_t || enc_t_scale) && (k == 0 || (a && b && sa && sb)));
    const int64_t gy = (m + BM - 1) / BM;
    VIOLA_CHECK_ARG(gy <= 65535);
    if (k == 0 || k % 128 != 0 || !aligned16(a) || !aligned16(b) || reinterpret_cast<uintptr_t>(sa) % 4 != 0 ||
        reinterpret_cast<uintptr_t>(sb) % 4 != 0 || 2 * h * k >= (1ll << 31) || (int64_t)BM * k >= (1ll << 31) ||
        (br != 1 && br % 32 != 0) || h % br != 0 || h % 32 != 0 || m % 32 != 0 || !aligned16(aux) || !aligned16(enc) ||
        !aligned16(enc_t))
        return VIOLA_EUNSUPPORTED;
    if (aux && enc_t && aux_dtype != VIOLA_F32 && takes_large_tiles(m, 2 * h) && 128 * h < (1ll << 31)) {
        // large products: the plain GEMM on 256 x 256 tiles writes [g | u], one pass over it writes the codes of h
        // in both layouts (the encoding epilogue does not fit the large tile's registers; 2.0 ms against 2.5 ms at
        // 16384 x 4096 -> 11008)
        const int status = mx_gemm(a, a_dtype, b, b_dtype, sa, sb, m, 2 * h, k, ar, br, bias, bias_dtype, aux, 2 * h, aux_dtype, stream);
        if (status) return status;
        return viola_gated_quantize_dual(aux, aux_dtype, m, h, activation, enc, enc_scale, enc_t, enc_t_scale, enc_dtype, 32, limit,
                                         VIOLA_SCALE_E8M0, stream_);
    }
    GemmArgs p = {};
    p.a = static_cast<const uint8_t*>(a); p.b = static_cast<const uint8_t*>(b);
    p.sa = reinterpret_cast<const float*>(sa); p.sb = reinterpret_cast<const float*>(sb);
    p.bias = bias; p.out = nullptr; p.aux = aux; p.m = m; p.n = h; p.k = k; p.lda = k; p.ldb = k; p.ldo = h;
    p.activation = activation;
    p.ldsa = k / 32; p.ldsb = k / 32; p.ar = ar; p.br = br; p.ak_shift = 5; p.bk_shift = 5;
    p.enc = static_cast<uint8_t*>(enc); p.enc_scale = enc_scale; p.enc_t = static_cast<uint8_t*>(enc_t); p.enc_t_scale = enc_t_scale;
    p.enc_limit = limit; p.enc_bf8 = enc_dtype == VIOLA_E5M2;
    return launch_mx_gemm_fast(p, MODE_GATED_FWD, a_dtype, b_dtype, bias_dtype, aux_dtype,
                               dim3((unsigned)((h + BN / 2 - 1) / (BN / 2)), (unsigned)gy), stream);
}

extern "C" int viola_varlen_group_gemm(const void* a, int a_dtype, const void* b, int b_dtype, const float* sa,
                                       const float* sb, const int64_t* offsets, int groups, int64_t m_total, int64_t n,
                                       int64_t k, int ar, int ak, int br, int bk, int64_t b_group_stride,
                                       int64_t sb_group_stride, void* out, int out_dtype, viola_stream_t stream_) {
    hipStream_t stream = viola_enter(stream_);
    VIOLA_CHECK_ARG(viola_is_fp8(a_dtype) && viola_is_fp8(b_dtype) && viola_is_float(out_dtype));
    VIOLA_CHECK_ARG(m_total >= 0 && n >= 0 && k >= 0 && groups > 0 && ar == 1 && br > 0 && pow2(ak) && pow2(bk) && ak >= 32 && bk >= 32);
    if (m_total == 0 || n == 0) return 0;
    VIOLA_CHECK_ARG(out && offsets && (k == 0 || (a && b && sa && sb)));
    const int64_t gy = (m_total + BM - 1) / BM + groups;
    VIOLA_CHECK_ARG(gy <= 65535);
    GemmArgs p = {};
    p.a = static_cast<const uint8_t*>(a); p.b = static_cast<const uint8_t*>(b); p.sa = sa; p.sb = sb;
    p.out = out; p.m = m_total; p.n = n; p.k = k; p.lda = k; p.ldb = k;
    p.ldsa = (k + ak - 1) / ak; p.ldsb = (k + bk - 1) / bk; p.ldo = n;
    p.ar = ar; p.br = br; p.ak_shift = shift_of(ak); p.bk_shift = shift_of(bk);
    p.offsets = offsets; p.groups = groups; p.b_group_stride = b_group_stride; p.sb_group_stride = sb_group_stride;
    const bool vec = k % 16 == 0 && aligned16(a) && aligned16(b) && b_group_stride % 16 == 0;
    const bool rowscale = br % 32 != 0;
    return launch_out<MODE_PLAIN>(p, a_dtype, b_dtype, VIOLA_F32, out_dtype, rowscale, vec,
                                  dim3((unsigned)((n + BN - 1) / BN), (unsigned)gy), stream);
}

extern "C" int viola_varlen_wgrad_gemm(const void* at, int a_dtype, const void* bt, int b_dtype, const float* sat,
                                       const float* sbt, const int64_t* poffsets, int groups, int64_t t_total, int64_t n,
                                       int64_t kout, void* out, int out_dtype, viola_stream_t stream_) {
    hipStream_t stream = viola_enter(stream_);
    VIOLA_CHECK_ARG(viola_is_fp8(a_dtype) && viola_is_fp8(b_dtype) && viola_is_float(out_dtype));
    VIOLA_CHECK_ARG(t_total >= 0 && t_total % 32 == 0 && n >= 0 && kout >= 0 && groups > 0 && groups <= 65535);
    if (n == 0 || kout == 0) return 0;
    VIOLA_CHECK_ARG(out && poffsets && (t_total == 0 || (at && bt && sat && sbt)));
    const int64_t gy = (n + BM - 1) / BM;
    VIOLA_CHECK_ARG(gy <= 65535);
    GemmArgs p = {};
    p.a = static_cast<const uint8_t*>(at); p.b = static_cast<const uint8_t*>(bt); p.sa = sat; p.sb = sbt;
    p.out = out; p.m = n; p.n = kout; p.k = t_total; p.lda = t_total; p.ldb = t_total;
    p.ldsa = t_total / 32; p.ldsb = t_total / 32; p.ldo = kout;
    p.ar = 1; p.br = 1; p.ak_shift = 5; p.bk_shift = 5;
    p.koffsets = poffsets; p.out_group_stride = n * kout;
    const bool vec = t_total % 16 == 0 && aligned16(at) && aligned16(bt);
    return launch_out<MODE_PLAIN>(p, a_dtype, b_dtype, VIOLA_F32, out_dtype, true, vec,
                                  dim3((unsigned)((kout + BN - 1) / BN), (unsigned)gy, (unsigned)groups), stream);
}
