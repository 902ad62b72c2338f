// The weight-streaming kernel (batched decode, and calls of up to 511 rows where it is priced
// cheaper than the tiled kernels): the instances for binary16
// activations, as the reference's prefill plan hands them (DecodedMatMul.project,
// J/backend/tornado/ops/DecodedMatMul.java:100-109) -- a short prompt, or the tail of a chunked one.
#define JL_SKINNY_XH true
#define JL_SKINNY_ENTRY jl_launch_gemm_skinny_x16
#include "jl_gemm_skinny_kernels.h"
