/* C ABI of libviola_hip.so: hand-written HIP kernels for gfx950 (MI355X) behind the
 * Python operator seam of chinoll/viola's low-precision hot path.
 *
 * The reference has no FFI layer; its seam is a set of Python wrapper functions that
 * take torch tensors and launch one TileLang kernel each. Every entry point below
 * replaces one of those wrappers (cited as path:line under the reference tree).
 *
 * Conventions
 *   - plain pointers and sizes only; all pointers are device pointers unless noted;
 *   - the library never allocates or frees device memory and never synchronises:
 *     each call enqueues kernels on `stream` (a hipStream_t) and returns;
 *   - a null pointer means "absent" (no bias, no aux, no source scale ...);
 *   - return 0 on success, a negative VIOLA_E* code for rejected arguments (nothing was
 *     launched), or the positive hipError_t that hipLaunchKernel returned for a launch;
 *   - matrices are row-major and contiguous unless a stride is passed.
 */
#ifndef VIOLA_HIP_H
#define VIOLA_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* viola_stream_t; /* hipStream_t */

enum { VIOLA_F32 = 0, VIOLA_BF16 = 1, VIOLA_F16 = 2, VIOLA_E4M3 = 3, VIOLA_E5M2 = 4 };
enum { VIOLA_SILU = 0, VIOLA_GELU = 1, VIOLA_RELU = 2 };
enum { VIOLA_NEAREST = 0, VIOLA_STOCHASTIC = 1 };
/* group scales: FP32 values, or E8M0 bytes (power-of-two scale 2^(byte - 127), the `native` / mxfp8 recipe) */
enum { VIOLA_SCALE_F32 = 0, VIOLA_SCALE_E8M0 = 1 };
enum { VIOLA_EINVAL = -1, VIOLA_EUNSUPPORTED = -2, VIOLA_ETOOLARGE = -3 };

int viola_abi_version(void);
const char* viola_error_string(int code);

/* ---------------------------------------------------------------- group quantization
 * viola/nn/_grouped_kernels.py:127-158 `quantize` (encode_kernel :53-92,
 * transpose_encode_kernel :95-124).
 * x is [rows, cols] of x_dtype (f32/bf16/f16, or fp8 codes when source_scale is given:
 * then value = code * source_scale[r / source_gr, c / source_gc]). With transposed = 0
 * the output q is [rows, cols] and scale is [ceil(rows/gr), ceil(cols/gc)]; with
 * transposed = 1 the output is the quantized transpose, q [cols, rows] and scale
 * [ceil(cols/gr), ceil(rows/gc)], groups laid along the new last dimension.
 * Per group: s = max(amax, 1e-30) / limit; q = fp8(isnan(v/s) ? NaN : clamp(v/s, +-limit)).
 * scale_format VIOLA_SCALE_E8M0 (native = True, :81-85): s is rounded up to a power of two, scale and source_scale
 * are bytes log2(s) + 127. */
int viola_group_quantize(const void* x, int x_dtype, int64_t rows, int64_t cols,
                         void* q, int q_dtype, void* scale, int gr, int gc, float limit, int transposed,
                         const void* source_scale, int source_gr, int source_gc, int scale_format,
                         viola_stream_t stream);

/* One read pass that emits both layouts of a row-major matrix with 1-D groups: the row-wise
 * codes/scales (q [rows, cols], scale [rows, ceil(cols/gc)]) and the quantized transpose
 * (qt [cols, rows], scale_t [cols, ceil(rows/gc)]). Same arithmetic per group as two calls of
 * viola_group_quantize (viola/nn/_grouped_linear.py:21,46-47 and :73,92 make those two calls). */
int viola_group_quantize_dual(const void* x, int x_dtype, int64_t rows, int64_t cols,
                              void* q, void* scale, void* qt, void* scale_t, int q_dtype, int gc,
                              float limit, float* column_partial, int scale_format, viola_stream_t stream);

/* viola_group_quantize_dual of h = act(g) * u [rows, cols], rounded to z_dtype, read from the stored projection
 * z = [g | u] [rows, 2 cols] (bf16 / fp16) instead of from a stored h: what the MXFP8 MLP hands from its gate/up
 * projection to its down projection (viola/nn/_mlp_kernels.py:195-230 encode h in the GEMM's epilogue; this is the
 * same result from the saved [g | u]). VIOLA_EUNSUPPORTED for fp32 z, gc != 32, cols % 8 != 0 or unaligned z / q. */
int viola_gated_quantize_dual(const void* z, int z_dtype, int64_t rows, int64_t cols, int activation,
                              void* q, void* scale, void* qt, void* scale_t, int q_dtype, int gc,
                              float limit, int scale_format, viola_stream_t stream);

/* column_partial (nullable) of viola_group_quantize_dual receives [ceil(rows/32), cols] fp32 sums of x over
 * each 32-row group, taken from the same read; viola_column_reduce adds the parts in a fixed order:
 * out[c] = sum_p partial[p][c], stored as out_dtype. Together they are the bias gradient dy.sum(0)
 * (viola/nn/_grouped_linear.py:101) without a second pass over dy. */
int viola_column_reduce(const float* partial, int64_t parts, int64_t cols, void* out, int out_dtype,
                        viola_stream_t stream);

/* viola/nn/_grouped_kernels.py:44-50 `dequantize` (decode_kernel :24-41): out = f32(q) * scale[r/gr, c/gc]. */
int viola_group_dequantize(const void* q, int q_dtype, const float* scale, int64_t rows, int64_t cols,
                           int gr, int gc, float* out, viola_stream_t stream);

/* viola/nn/_linear_kernels.py:107-121,253-257 `transpose`: byte-matrix transpose, x [batch, rows, cols] ->
 * out [batch, cols, rows] (the reference transposes one matrix per call; batch > 1 serves stacked expert weights). */
int viola_fp8_transpose(const void* x, void* out, int64_t batch, int64_t rows, int64_t cols, viola_stream_t stream);

/* viola/nn/_grouped_kernels.py:161-164 `transpose` of a 2-D-block-scaled code matrix (gr >= 32): the payload transposes
 * exactly and the scale grid [ceil(rows / gr), ceil(cols / gc)] (FP32 or E8M0 bytes, scale_format) is transposed with
 * it: out [cols, rows], scale_out [ceil(cols / gc), ceil(rows / gr)], one launch. */
int viola_block_transpose(const void* x, void* out, int64_t rows, int64_t cols, const void* scale, void* scale_out,
                          int gr, int gc, int scale_format, viola_stream_t stream);

/* ---------------------------------------------------------------- per-tensor scaling (`current` / `delayed`)
 * viola/nn/_linear_kernels.py:231-242 `tensor_scale` = _amax_kernel :33-46 + _scale_kernel :49-71.
 * viola_tensor_amax: maxima[i] = max |x| over part i of `parts` (NaN dropped); maxima is caller scratch of `parts`
 * floats (the reference sizes it ceil(n / 2048)). viola_tensor_scale: amax = max(maxima);
 * scale[0] = max(delayed && index != 0 ? max(history as it was) : amax, 1e-30) / limit; history[index % len] = amax. */
int viola_tensor_amax(const void* x, int x_dtype, int64_t n, float* maxima, int64_t parts, viola_stream_t stream);
int viola_tensor_scale(const float* maxima, int64_t parts, float* history, int history_len, int64_t index, int delayed,
                       float limit, float* scale, viola_stream_t stream);

/* viola_tensor_amax for a [rows, cols] matrix that also leaves fp32 column sums of each of `slices` row slices in
 * column_partial [slices, cols] (finish with viola_column_reduce): the bias gradient dy.sum(0) of
 * viola/nn/linear.py:143 from the amax pass over dy. maxima receives ceil(cols / piece / 256) * slices values,
 * piece = 16 bytes of x; cols must be a multiple of the piece, x and column_partial 16-byte aligned. */
int viola_tensor_amax_columns(const void* x, int x_dtype, int64_t rows, int64_t cols, int64_t slices, float* maxima,
                              float* column_partial, viola_stream_t stream);

/* viola_tensor_amax_columns + viola_tensor_scale + viola_column_reduce behind one call (maxima: ceil(cols / piece / 256)
 * * slices floats of scratch, column_partial: slices * cols floats of scratch, column_sum [cols] of sum_dtype). */
int viola_tensor_amax_columns_scale(const void* x, int x_dtype, int64_t rows, int64_t cols, int64_t slices, float* maxima,
                                    float* column_partial, float* history, int history_len, int64_t index, int delayed,
                                    float limit, float* scale, void* column_sum, int sum_dtype, viola_stream_t stream);

/* Both launches of `tensor_scale` behind one call. */
int viola_tensor_amax_scale(const void* x, int x_dtype, int64_t n, float* maxima, int64_t parts, float* history,
                            int history_len, int64_t index, int delayed, float limit, float* scale, viola_stream_t stream);

/* viola/nn/_linear_kernels.py:245-250 `quantize` (_quantize_kernel :74-104): with the tensor's one scale,
 * q[r, c] = fp8(isnan(x) ? x : clamp(x / scale[0], +-limit)) and / or qt[c, r] = the same code; q or qt may be NULL. */
int viola_tensor_quantize(const void* x, int x_dtype, int64_t rows, int64_t cols, const float* scale, void* q, void* qt,
                          int q_dtype, float limit, viola_stream_t stream);

/* ---------------------------------------------------------------- Hadamard-64 rotation (`rotation_size=64`)
 * H64 = H4 (x) H4 (x) H4, H4 = (ones(4, 4) - 2 flip(eye(4))) / 2, applied to each run of 64 consecutive columns of a
 * [rows, cols] matrix in FP32, in the operation order of viola/nn/_rotation_kernels.py:11-25 (_regular64); a last
 * group that reaches past `cols` is completed with zeros.
 * viola_rotation_amax (_rotation_amax :28-47, first half of `tensor_scale` :100-108): maxima[i] = max |rotated x| over
 * tile i of 64 x 64; parts must be ceil(rows / 64) * ceil(cols / 64); finish with viola_tensor_scale.
 * viola_rotation_quantize (_rotation_quantize :50-80, `quantize` :111-117): viola_tensor_quantize of the rotated values.
 * viola_rotation_inverse (_rotation_inplace :83-97, `inverse_` :120-123): x <- rotated x in place, rounded to x's type. */
int viola_rotation_amax(const void* x, int x_dtype, int64_t rows, int64_t cols, float* maxima, int64_t parts,
                        viola_stream_t stream);
int viola_rotation_quantize(const void* x, int x_dtype, int64_t rows, int64_t cols, const float* scale, void* q, void* qt,
                            int q_dtype, float limit, viola_stream_t stream);
int viola_rotation_inverse(void* x, int x_dtype, int64_t rows, int64_t cols, viola_stream_t stream);

/* viola/nn/_linear_kernels.py:260-293 `gemm` (_gemm_kernel :124-163, _mixed_gemm_kernel :166-228):
 * out[m, n] = (sum_k a[m, k] * b[n, k]) * sa[0] * sb[0] (+ bias[n]); a and b may mix e4m3 and e5m2. */
int viola_tensor_gemm(const void* a, int a_dtype, const void* b, int b_dtype, const float* sa, const float* sb,
                      int64_t m, int64_t n, int64_t k, const void* bias, int bias_dtype, void* out, int out_dtype,
                      viola_stream_t stream);

/* The same product under the reference's accum_dtype="fp16" options (viola/nn/_linear_kernels.py:139-155, :198-211):
 * every 32 k the running FP16 partial becomes fp16(partial + the 32 products); after accum_block k (rounded down to
 * whole 64-k chunks from 64 up; 0: never) the partial is added to a total kept in reduce_dtype (VIOLA_F32 or
 * VIOLA_BF16, rounded after every addition) and cleared; out = (total * sa[0]) * sb[0] (+ bias). An ablation option:
 * runs on the generic kernel. The 32 products are summed in FP32 and rounded once, the best case of a tensor-core
 * instruction with an FP16 accumulator. */
int viola_tensor_gemm_half(const void* a, int a_dtype, const void* b, int b_dtype, const float* sa, const float* sb,
                           int64_t m, int64_t n, int64_t k, const void* bias, int bias_dtype, void* out, int out_dtype,
                           int accum_block, int reduce_dtype, viola_stream_t stream);

/* ---------------------------------------------------------------- MXFP8: E8M0 scales per 32 k
 * viola/nn/_grouped_kernels.py:310-328 `gemm` with native=True (gemm_kernel :195-293 on the block-scaled MMA of
 * :174-192): out[m, n] = sum_kg (sum_{k in kg} a[m, k] b[n, k]) * 2^(sa[m / ar, kg] - 127) * 2^(sb[n / br, kg] - 127)
 * (+ bias[n]), the scaling done by v_mfma_scale_f32_32x32x64_f8f6f4. sa [ceil(m / ar), k / 32], sb [ceil(n / br), k / 32]
 * bytes. Returns VIOLA_EUNSUPPORTED unless k % 128 == 0, a and b are 16-byte and the scales 4-byte aligned and
 * br is 1 or a multiple of 32: the caller then converts the scales to FP32 and calls viola_group_gemm (same values). */
int viola_mx_gemm(const void* a, int a_dtype, const void* b, int b_dtype, const uint8_t* sa, const uint8_t* sb,
                  int64_t m, int64_t n, int64_t k, int ar, int br, const void* bias, int bias_dtype, void* out,
                  int out_dtype, viola_stream_t stream);

/* ---------------------------------------------------------------- grouped-scale FP8 GEMM
 * viola/nn/_grouped_kernels.py:310-328 `gemm` (gemm_kernel :195-293).
 * out[m, n] = sum over 32-wide K groups kg of (sum_{k in kg} a[m,k]*b[n,k]) * sa[m/ar, k/ak] * sb[n/br, k/bk]
 *             (+ bias[n]);  a is [m, k], b is [n, k] ("NT"), both FP8 codes; ak and bk are multiples of 32. */
int viola_group_gemm(const void* a, int a_dtype, const void* b, int b_dtype, const float* sa, const float* sb,
                     int64_t m, int64_t n, int64_t k, int ar, int ak, int br, int bk,
                     const void* bias, int bias_dtype, void* out, int out_dtype, viola_stream_t stream);

/* viola_group_gemm under accum_dtype="fp16" (viola/nn/_grouped_kernels.py:268-292, :310-318): the raw products of
 * gcd(ak, bk, accum_block) k (accum_block 0: gcd(ak, bk)) meet in an FP16 partial, fp16(partial + 32 products) per
 * 32 k, which is then scaled, (partial * sa) * sb, added to a total kept in reduce_dtype (VIOLA_F32 or VIOLA_BF16,
 * rounded after every addition) and cleared. Generic kernel; same FP32-sum-then-round model of the 32-k step. */
int viola_group_gemm_half(const void* a, int a_dtype, const void* b, int b_dtype, const float* sa, const float* sb,
                          int64_t m, int64_t n, int64_t k, int ar, int ak, int br, int bk,
                          const void* bias, int bias_dtype, void* out, int out_dtype, int accum_block, int reduce_dtype,
                          viola_stream_t stream);

/* viola/nn/_mlp_kernels.py:243-277 `gemm` (kernel :16-231), grouped FP32-scale path.
 * forward (backward = 0): b is [2h, k]; g = a.b[0:h]^T, u = a.b[h:2h]^T (+bias), each rounded to
 *   out_dtype; aux[m, 0:h] = g, aux[m, h:2h] = u when aux != NULL; out[m, h] = act(g) * u.
 * backward (backward = 1): b is [h, k]; d = round(a.b^T); g, u read from aux [m, 2h];
 *   out[m, 0:h] = d*u*act'(g), out[m, h:2h] = d*act(g). aux and out share out_dtype. */
int viola_gated_gemm(const void* a, int a_dtype, const void* b, int b_dtype, const float* sa, const float* sb,
                     int64_t m, int64_t h, int64_t k, int ar, int ak, int br, int bk,
                     const void* bias, int bias_dtype, void* aux, void* out, int out_dtype,
                     int activation, int backward, viola_stream_t stream);

/* The same two gated projections under the other recipes of viola/nn/_mlp_kernels.py:16-231 (`grouped` false:
 * value *= sa[0] * sb[0], :157-166; native E8M0 scales, :120-127). viola_tensor_gated_gemm: one FP32 scale per
 * operand. viola_mx_gated_gemm: E8M0 bytes per 32 k as in viola_mx_gemm (ar, br = rows per scale row); returns
 * VIOLA_EUNSUPPORTED where viola_mx_gemm does, and in forward when h is not a multiple of br.
 * Large products (at least 512 output tiles of 256 x 256) with aux given run as the plain GEMM followed by one
 * elementwise pass on the same stream, with the same results and no memory beyond aux and out: forward the GEMM
 * writes aux, backward it writes d into out[:, h:2h], which the pass then replaces (so out is also read there). */
int viola_tensor_gated_gemm(const void* a, int a_dtype, const void* b, int b_dtype, const float* sa, const float* sb,
                            int64_t m, int64_t h, int64_t k, const void* bias, int bias_dtype, void* aux, void* out,
                            int out_dtype, int activation, int backward, viola_stream_t stream);
int viola_mx_gated_gemm(const void* a, int a_dtype, const void* b, int b_dtype, const uint8_t* sa, const uint8_t* sb,
                        int64_t m, int64_t h, int64_t k, int ar, int br, const void* bias, int bias_dtype, void* aux,
                        void* out, int out_dtype, int activation, int backward, viola_stream_t stream);

/* viola/nn/_mlp_kernels.py:195-230 (`encode_output`, `save_output_transpose`): the gate/up projection of an MXFP8 MLP
 * whose h = act(g) * u, rounded to aux_dtype, leaves the kernel as FP8 codes with E8M0 scales per 32 values: along its
 * rows (enc [m, h], enc_scale [m, h / 32]) for the down projection's forward GEMM and, when enc_t is not NULL, along
 * its columns (enc_t [h, m], enc_t_scale [h, m / 32]) for its wgrad. aux [m, 2h] (NULL allowed) receives [g, u].
 * VIOLA_EUNSUPPORTED where viola_mx_gated_gemm returns it, and when m or h is not a multiple of 32. Large products
 * with aux and enc_t given run as viola_mx_gemm into aux followed by viola_gated_quantize_dual (same results). */
int viola_mx_gated_gemm_encode(const void* a, int a_dtype, const void* b, int b_dtype, const uint8_t* sa, const uint8_t* sb,
                               int64_t m, int64_t h, int64_t k, int ar, int br, const void* bias, int bias_dtype, void* aux,
                               int aux_dtype, void* enc, uint8_t* enc_scale, void* enc_t, uint8_t* enc_t_scale, int enc_dtype,
                               float limit, int activation, viola_stream_t stream);

/* Variable-group (MoE-expert style) GEMM: `groups` independent problems that share n and k and
 * differ in their row range. Group g owns rows [offsets[g], offsets[g+1]) of a and out
 * (offsets: groups+1 int64 on the device, ascending) and operand b + g*b_group_stride (elements),
 * sb + g*sb_group_stride (floats). Same arithmetic per group as viola_group_gemm. The reference
 * has no such kernel (its "grouped" is group-scaled quantization); this serves the
 * variable-group linear named by the build's target workload. m_total bounds the grid. */
int viola_varlen_group_gemm(const void* a, int a_dtype, const void* b, int b_dtype, const float* sa, const float* sb,
                            const int64_t* offsets, int groups, int64_t m_total, int64_t n, int64_t k,
                            int ar, int ak, int br, int bk, int64_t b_group_stride, int64_t sb_group_stride,
                            void* out, int out_dtype, viola_stream_t stream);

/* Variable-group weight gradient: for each group g, out[g] ([n, kout]) = sum over the group's
 * tokens of at[:, t] * bt[:, t], with at [n, t_total] and bt [kout, t_total] the quantized
 * transposes whose 32-token scale groups start at each group's own padded offset:
 * group g owns token columns [poffsets[g], poffsets[g+1]) (multiples of 32, zero codes in the
 * padding); sat [n, t_total/32], sbt [kout, t_total/32]. */
int viola_varlen_wgrad_gemm(const void* at, int a_dtype, const void* bt, int b_dtype, const float* sat, const float* sbt,
                            const int64_t* poffsets, int groups, int64_t t_total, int64_t n, int64_t kout,
                            void* out, int out_dtype, viola_stream_t stream);

/* Segmented transposed quantize for the variable-group path: x [rows, cols] row-major; group g owns
 * rows [offsets[g], offsets[g+1]) and writes its quantized transpose into token columns
 * [poffsets[g], poffsets[g+1]) of qt [cols, t_total] (scale_t [cols, t_total/32]), 32-token groups
 * counted from the group's own first row; padding columns get zero codes and scale 1e-30/limit. */
int viola_varlen_quantize_transposed(const void* x, int x_dtype, int64_t rows, int64_t cols,
                                     const int64_t* offsets, const int64_t* poffsets, int groups, int64_t t_total,
                                     void* qt, float* scale_t, int q_dtype, float limit,
                                     void* q, float* scale, viola_stream_t stream);
/* q / scale (both or neither; 16-bit x with cols a multiple of 8, else VIOLA_EUNSUPPORTED): the plain row-wise
 * (1, 32) quantization of x, q [rows, cols] and scale [rows, ceil(cols/32)], written from the same read. */

/* ---------------------------------------------------------------- gated activations (elementwise)
 * viola/nn/_gated_kernels.py:16-36 forward_kernel: out[r, c] = act(z[r, c]) * z[r, c + h].
 * viola/nn/_gated_kernels.py:39-67 backward_kernel: dz = [dy*u*act'(g), dy*act(g)]. */
int viola_gated_forward(const void* z, void* out, int64_t rows, int64_t h, int dtype, int activation, viola_stream_t stream);
int viola_gated_backward(const void* z, const void* dy, void* dz, int64_t rows, int64_t h, int dtype, int activation,
                         viola_stream_t stream);

/* ---------------------------------------------------------------- FP8Muon kernels
 * viola/optim/_kernels.py:300-315 `momentum_update` (_momentum_1d_kernel :88-144,
 * _momentum_2d_kernel :147-200). granularity 0: 1-D tiles of tile_size over the flat tensor
 * (q padded to whole tiles); granularity 1: tr x tc blocks over [planes, rows, cols] (unpadded).
 * old_q/new_q and old_scale/new_scale may alias. Pointers need only element alignment. */
int viola_momentum_update(const void* grad, int grad_dtype, const void* old_q, const float* old_scale,
                          void* new_q, float* new_scale, void* update /* bf16 */,
                          int64_t n, float beta, float inv_loss_scale, int nesterov,
                          int granularity, int tile_size, int64_t planes, int64_t rows, int64_t cols, int tr, int tc,
                          int rounding, int64_t rounding_step, int64_t rounding_key, viola_stream_t stream);

/* viola/optim/_kernels.py:325-328 `weight_update` (_weight_kernel :227-255). */
int viola_weight_update(void* weight, int weight_dtype, const void* grad, int grad_dtype, int64_t n,
                        float lr, float decay, float update_scale, int rounding, int64_t rounding_step,
                        int64_t rounding_key, int64_t offset, viola_stream_t stream);

/* viola/optim/_kernels.py:331-337 `adam_update` (_adam_kernel :258-293); inv_c1/inv_c2 are the
 * host-computed bias corrections; rounding_step is step - 1. */
int viola_adam_update(void* weight, int weight_dtype, const void* grad, int grad_dtype,
                      void* first, void* second, int state_dtype, int64_t n,
                      float lr, float decay, float b1, float b2, float inv_c1, float inv_c2, float eps,
                      int rounding, int64_t rounding_step, int64_t rounding_key, int64_t offset,
                      int adamw, int maximize, viola_stream_t stream);

/* viola_momentum_update (1-D tiles of 256 / 512 / 1024, whole tiles only) for many tensors with the same number of
 * tiles, gradient dtype and hyper-parameters, in one launch (the reference launches once per matrix,
 * viola/optim/muon.py:104-106). table: device array of `tensors` rows of eight int64: {grad, old_q, old_scale, new_q,
 * new_scale, update, rounding key, 0}; the gradient must be aligned to four elements, the codes to 4
 * bytes and the bf16 update to 8 bytes; old and new state may alias. */
int viola_momentum_update_table(const int64_t* table, int64_t tensors, int64_t tiles, int grad_dtype, int tile_size,
                                float beta, float inv_loss_scale, int nesterov, int rounding, int64_t rounding_step,
                                viola_stream_t stream);

/* viola_weight_update with nearest rounding for many fp32 tensors of `count` elements each (a multiple of 4), one
 * launch (the reference: one launch per matrix, viola/optim/muon.py:131-132). table: rows of two int64:
 * {weight (16-byte aligned), update (aligned to four elements of grad_dtype)}. */
int viola_weight_update_table(const int64_t* table, int64_t tensors, int64_t count, int grad_dtype, float lr, float decay,
                              float update_scale, viola_stream_t stream);

/* The same update for many tensors that share dtypes, hyper-parameters and step count, in one launch (the reference
 * calls adam_update once per parameter, viola/optim/muon.py:137-140; vectors of a transformer are a few thousand
 * elements each, so their launches dominate). table: device array of `tensors` rows of seven int64:
 * {weight pointer, grad pointer, first pointer, second pointer, element count, rounding key, rounding offset};
 * max_count: the largest element count. */
int viola_adam_update_table(const int64_t* table, int64_t tensors, int64_t max_count, int weight_dtype, int grad_dtype,
                            int state_dtype, float lr, float decay, float b1, float b2, float inv_c1, float inv_c2,
                            float eps, int rounding, int64_t rounding_step, int adamw, int maximize, viola_stream_t stream);

/* viola/optim/_kernels.py:318-322 `copy_scaled` (_copy_scaled_kernel :203-222). */
int viola_copy_scaled(const void* update, int update_dtype, void* out, int out_dtype,
                      int64_t src, int64_t dst, int64_t count, float scale, viola_stream_t stream);

/* viola/optim/_kernels.py:73-83 `dequantize` (diagnostic): e4m3 payload * per-tile scale -> fp32 [n]. */
int viola_momentum_dequantize(const void* q, const float* scale, float* out, int64_t n,
                              int granularity, int tile_size, int64_t planes, int64_t rows, int64_t cols, int tr, int tc,
                              viola_stream_t stream);

/* ---------------------------------------------------------------- Newton-Schulz GEMM chain
 * viola/optim/_orthogonalize_kernels.py:53-66 `_matmul` (matmul_kernel :16-50): batched
 * out[b] = a[b] . (transpose_b ? bmat[b]^T : bmat[b]) with fp32 accumulation, rounded to dtype,
 * then epilogue 0: nothing; 1: -4.7750*residual + 2.0315*value; 2: value + 3.4445*residual; rounded
 * to dtype. a [batch, m, k]; bmat [batch, n, k] if transpose_b else [batch, k, n]; dtype bf16 or f16.
 * out_diag (nullable) receives a second copy of the result with add_diag added to its diagonal after
 * rounding (Q = Z + 3.4445 I, viola/optim/_orthogonalize.py:45-47). transpose_out = 1 stores out and
 * out_diag as [batch, n, m] (the un-transposition of a tall matrix at the end of the chain,
 * viola/optim/_orthogonalize.py:20-21,52-53); residual stays [batch, m, n].
 * With transpose_b = 1, bmat == a and m == n (a . a^T) only the tiles on and above the diagonal are multiplied
 * and each is stored a second time transposed: out[i, j] and out[j, i] carry the same rounded product, and each
 * takes the epilogue with its own residual element, so the result is what the full product gives for any
 * residual, symmetric or not. The caller decides whether a . a^T is the product it wants: for a matrix that is
 * symmetric only up to rounding, a . a differs from it and is requested with transpose_b = 0. */
int viola_ns_gemm(const void* a, const void* bmat, const void* residual, void* out, int dtype,
                  int transpose_b, int epilogue, int64_t batch, int64_t m, int64_t n, int64_t k,
                  float add_diag, void* out_diag, int transpose_out, viola_stream_t stream);

/* viola/optim/_orthogonalize_kernels.py:114-197 `plan` (the per-shape schedule the reference picks by timing its
 * candidates: bm, bn): which tile shape viola_ns_gemm runs a product on. Host arithmetic only, nothing is launched and
 * no GPU is needed. Operands are taken as 16-byte aligned; same_operand != 0 means a and bmat are one buffer.
 * plan[0], plan[1]: rows and columns of output per block; plan[2]: 1 when only the tiles on and above the diagonal
 * are multiplied and mirrored (a . a^T, not transposed on output); plan[3]: 0 for the generic kernel (shapes the tiled
 * one does not take: k or n not a multiple of 8, a matrix of 2 GiB or more), 1..5 for the tiled kernel's shapes in
 * growing size. Every shape computes an element with the same sequence of operations, so the plan never changes a
 * result. */
int viola_ns_plan(int64_t batch, int64_t m, int64_t n, int64_t k, int transpose_b, int same_operand, int transpose_out,
                  int* plan);

/* viola/optim/_orthogonalize.py:12-16 / _orthogonalize_kernels.py:80-84: x = dtype(matrix), optionally
 * transposed so rows <= cols, divided by (Frobenius norm + 1e-7), all in the working dtype.
 * in [batch, rows, cols] of in_dtype; out [batch, min, max] of dtype; workspace: 256 * batch floats (partial
 * sums of squares; every slot is written before it is read, so it needs no clearing). */
int viola_ns_prepare(const void* in, int in_dtype, void* out, int dtype, int64_t batch, int64_t rows, int64_t cols,
                     float* workspace, viola_stream_t stream);

/* No counterpart in the reference. viola_ns_prepare for callers that cannot allocate device memory (code under
 * HIP-graph capture, serving loops, harnesses that forbid hipMalloc): the same kernels and results, with the
 * partial sums in a 1 MiB array built into the library (one copy per GPU, held until the process ends) instead
 * of a caller's workspace. batch <= 1024, otherwise VIOLA_ETOOLARGE and nothing is launched. The array's address
 * on the current device is looked up on the first call there (batch = 0 is accepted as a set-up call that does
 * only this); `stream` must belong to the current device. Calls on one GPU share the array: two that overlap in
 * time (different streams, or threads) race; calls on one stream are ordered and safe. Calls no hipMalloc /
 * hipFree and no allocating library routine. */
int viola_ns_prepare_static(const void* in, int in_dtype, void* out, int dtype, int64_t batch, int64_t rows,
                            int64_t cols, viola_stream_t stream);

/* ---------------------------------------------------------------- FP8 gradient wire codec
 * viola/distributed/_fp8_kernels.py:84-87 `pack` (_pack :18-43) and :90-93 `unpack` (_unpack :46-69).
 * packet: rows x stride bytes, stride = ceil16(groups*(tile+4)): per row groups*tile codes, then
 * groups fp32 scales. pack reads x[n] fp32 at index row*groups*tile + group*tile + i (0 past n).
 * unpack writes out[n]; with reduce != 0 it sums the rows into out[0 : groups*tile]. */
int viola_comm_pack(const float* x, int64_t n, void* packet, int64_t rows, int64_t groups, int tile, int fp8_dtype,
                    viola_stream_t stream);
int viola_comm_unpack(const void* packet, float* out, int64_t n, int64_t rows, int64_t groups, int tile, int fp8_dtype,
                      int reduce, viola_stream_t stream);

/* viola_comm_pack / viola_comm_unpack for many buckets in one launch: the reference drains its gradient buckets one
 * pack and one unpack launch at a time (viola/distributed/gradients.py:101-125 -> fp8.py:49-85), and a 25 MB bucket
 * is too short a launch to reach the memory system's streaming rate. table: device array of `buckets` rows of eight
 * int64. pack: {x, n, packet, rows, groups, 0, 0, 0}, x 16-byte and packet 4-byte aligned, tile 256 only
 * (VIOLA_EUNSUPPORTED otherwise: call viola_comm_pack per bucket); max_units = the largest rows * groups of a bucket.
 * unpack: {packet, n, out, rows, groups, 0, 0, 0}, out 16-byte and packet 4-byte aligned, n <= (reduce ? 1 : rows) *
 * groups * tile as for viola_comm_unpack (not checked here: the table lives on the device); max_elements = the
 * largest (reduce ? 1 : rows) * groups * tile of a bucket. Bytes and values are those of the per-bucket entry points. */
int viola_comm_pack_table(const int64_t* table, int64_t buckets, int64_t max_units, int tile, int fp8_dtype,
                          viola_stream_t stream);
int viola_comm_unpack_table(const int64_t* table, int64_t buckets, int64_t max_elements, int tile, int fp8_dtype,
                            int reduce, viola_stream_t stream);

/* ---------------------------------------------------------------- self checks (test support)
 * Compare the hardware FP8 conversion instructions with the software codecs over every fp32 bit
 * pattern of magnitude <= the format's clamp range (encode) and all 256 codes (decode); writes
 * mismatch counts to counts[4] (device): {e4m3 encode, e5m2 encode, e4m3 decode, e5m2 decode}. */
int viola_selftest_fp8(uint64_t* counts, viola_stream_t stream);
/* philox(element, step, key) word 0 for `count` triples (device arrays) -> out. */
int viola_selftest_philox(const uint64_t* triples, uint32_t* out, int64_t count, viola_stream_t stream);


#ifdef __cplusplus
}
#endif
#endif /* VIOLA_HIP_H */
