// Device-side helpers shared by the kernels: fp16 widening, Q4_K scale unpacking, wave folds.
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

#define JL_WAVE 64

// IEEE half bits -> float, exact (subnormals included); the device form of Float.float16ToFloat.
__device__ __forceinline__ float jl_half_bits_to_float(uint32_t bits) {
    return __half2float(__ushort_as_half((unsigned short)(bits & 0xFFFFu)));
}

// The 6-bit scale and minimum of sub-block j of a Q4_K super-block, from its 12 packed bytes held
// as three little-endian dwords (Q4_KFloatTensor.getScaleK4 / getMinK4,
// J/tensor/standard/Q4_KFloatTensor.java:68-85).
__device__ __forceinline__ void jl_q4k_scale_min(uint32_t s0, uint32_t s1, uint32_t s2, int j,
                                                 int &sc, int &mn) {
    // byte b of the 12: b < 4 in s0, b < 8 in s1, else s2
    if (j < 4) {
        sc = (s0 >> (8 * j)) & 63;
        mn = (s1 >> (8 * j)) & 63;
    } else {
        int k = j - 4;
        uint32_t lo = (s2 >> (8 * k)) & 0xFF;  // byte j + 4
        uint32_t a = (s0 >> (8 * k)) & 0xFF;   // byte j - 4
        uint32_t b = (s1 >> (8 * k)) & 0xFF;   // byte j
        sc = (int)((lo & 0xF) | ((a >> 6) << 4));
        mn = (int)((lo >> 4) | ((b >> 6) << 4));
    }
}

// Sum over the lanes of each aligned group of `width` lanes (a power of two, at most 64).  Every
// lane of a group ends with the group's total.
template <int WIDTH>
__device__ __forceinline__ float jl_group_sum(float v) {
#pragma unroll
    for (int off = WIDTH / 2; off >= 1; off >>= 1) v += __shfl_xor(v, off, JL_WAVE);
    return v;
}

__device__ __forceinline__ float jl_group_sum_dyn(float v, int width) {
    for (int off = width >> 1; off >= 1; off >>= 1) v += __shfl_xor(v, off, JL_WAVE);
    return v;
}

// SiLU(g) * u with the host's arithmetic: g / (float)(1.0 + exp(-g)) in double, then one float
// divide and one float multiply (CpuOperations.swiGLU, J/inference/op/CpuOperations.java:255-260).
__device__ __forceinline__ float jl_swiglu_value(float g, float u) {
    float denom = (float)(1.0 + exp(-(double)g));
    return __fmul_rn(__fdiv_rn(g, denom), u);
}
