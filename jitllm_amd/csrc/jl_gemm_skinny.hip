// Batched decode (at most 64 rows, and calls of up to 511 rows where streaming the weights once per
// 32 rows is priced cheaper than the tiled kernels) on the weight-streaming kernel: the instances for fp32
// activations (QuantizedBatchProjections.java:76-309 hands FloatArrays) and the choice between them
// and the binary16 ones.  The kernel itself is jl_gemm_skinny_kernels.h.
#define JL_SKINNY_XH false
#define JL_SKINNY_ENTRY jl_launch_gemm_skinny_x32
#include "jl_gemm_skinny_kernels.h"

// Activation rows one workgroup multiplies: 16 or 32; calls of more rows run as two row blocks.
int jl_skinny_padded_rows(int rows) { return rows <= 16 ? 16 : 32; }

int jl_launch_gemm_skinny(jl_context *ctx, const jl_weight *const *weights, int count, const float *X,
                          const _Float16 *X16, float *C, bool c_f16, int rows, int64_t ldo, int64_t col_offset,
                          int epilogue, float *planes, size_t plane_bytes, double other_us, bool *taken) {
    return X16 ? jl_launch_gemm_skinny_x16(ctx, weights, count, X, X16, C, c_f16, rows, ldo, col_offset, epilogue,
                                           planes, plane_bytes, other_us, taken)
               : jl_launch_gemm_skinny_x32(ctx, weights, count, X, X16, C, c_f16, rows, ldo, col_offset, epilogue,
                                           planes, plane_bytes, other_us, taken);
}
