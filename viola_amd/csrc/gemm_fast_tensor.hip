// Per-tensor-scale instances of the fast FP8 GEMM kernel.
#include "gemm_fast_scaled.hpp"

namespace viola {

int launch_tensor_gemm_fast(const GemmArgs& args, int mode, int a_dtype, int b_dtype, int bias_dtype, int out_dtype, dim3 grid,
                            hipStream_t stream) {
    return launch_scaled_gemm_fast<true, false>(args, mode, a_dtype, b_dtype, bias_dtype, out_dtype, grid, stream);
}

}  // namespace viola
