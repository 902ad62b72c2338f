// Device-side helpers shared by the kernels: fp16 widening, Q4_K scale unpacking, wave folds.
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

#define JL_WAVE 64

// A product rounded to fp32 on its own.  The compiler's default is to contract a * b + c into one
// fma -- across statements, through the *_rn intrinsics (plain operators in this toolchain's
// headers), and even into a mixed-precision fma when the sum is then narrowed to fp16 (with a +0
// addend, which also loses the sign of a zero product).  Java never fuses, so wherever a result
// has to carry the host's bits the product passes through a register the compiler cannot look past.
__device__ __forceinline__ float jl_mul_rn(float a, float b) {
    float r = a * b;
    asm volatile("" : "+v"(r));
    return r;
}

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

// Hands a value back to the compiler as one it knows nothing about.  Used on words of four
// byte-sized quants after their nibble mask: the byte -> float conversions then stay the
// single-instruction v_cvt_f32_ubyteN, where the compiler would otherwise see through the mask and
// extract each 4-bit field on its own (a bit-field extract plus a conversion per weight).
__device__ __forceinline__ uint32_t jl_opaque(uint32_t v) {
    asm("" : "+v"(v));
    return v;
}

// The bits 0..3 of x, one to a byte (bit k of x at bit 0 of byte k).
__device__ __forceinline__ uint32_t jl_spread4(uint32_t x) { return ((x & 0xFu) * 0x00204081u) & 0x01010101u; }

// ggml's kvalues_iq4nl (-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113;
// J/tensor/standard/IQ4_XSFloatTensor.java:30-32) of the four nibbles held one to a byte in `idx`,
// as four signed bytes: two byte permutes pick entry idx & 7 of each half of the table, a third
// picks the half by bit 3.
__device__ __forceinline__ uint32_t jl_iq4nl_lookup4(uint32_t idx) {
    const uint32_t low3 = idx & 0x07070707u;
    const uint32_t lo = __builtin_amdgcn_perm(0xF6EADDCFu, 0xBFAD9881u, low3);   // entries 0..7
    const uint32_t hi = __builtin_amdgcn_perm(0x71594535u, 0x26190D01u, low3);   // entries 8..15
    return __builtin_amdgcn_perm(hi, lo, 0x03020100u | ((idx & 0x08080808u) >> 1));
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
    return jl_mul_rn(__fdiv_rn(g, denom), u);
}

// Four consecutive results of an output row stored as binary16 (round to nearest even): one
// 8-byte store when all four lie inside the row and the address allows it.
__device__ __forceinline__ void jl_store4_f16(_Float16 *dst, const float (&v)[4], int valid) {
    typedef _Float16 jl_half4 __attribute__((ext_vector_type(4)));
    if (valid >= 4 && (((uintptr_t)dst) & 7) == 0) {
        *(jl_half4 *)dst = jl_half4{(_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3]};
    } else {
#pragma unroll
        for (int e = 0; e < 4; e++)
            if (e < valid) dst[e] = (_Float16)v[e];
    }
}

// Activations, fp32 -> fp16 with a power-of-two row scale.  One workgroup of 256 threads per row:
// scale = the power of two that brings the row's largest magnitude into [2^11, 2^12);
// a16 = half(x / scale) (the division is exact).  Rows past `rows` are zero-filled.
// A row of up to 8192 columns is read once and kept in registers between the two passes (largest
// magnitude, conversion); longer rows are read twice.
__device__ __forceinline__ void jl_row_to_f16(const float *__restrict__ X, _Float16 *__restrict__ A,
                                              float *__restrict__ row_scale, int rows, int k, int row) {
    typedef _Float16 jl_half4 __attribute__((ext_vector_type(4)));
    __shared__ float wave_max[4];
    constexpr int kHeld = 8;   // float4 per thread held in registers: 256 x 8 x 4 = 8192 columns
    const int tid = threadIdx.x;
    _Float16 *a = A + (int64_t)row * k;
    if (row >= rows) {
        for (int i = tid * 4; i < k; i += 1024) *(jl_half4 *)(a + i) = jl_half4{0, 0, 0, 0};
        if (tid == 0) row_scale[row] = 1.f;
        return;
    }
    const float *x = X + (int64_t)row * k;
    const bool held = k <= kHeld * 1024;
    float4 v[kHeld];
    float amax = 0.f;
    if (held) {
#pragma unroll
        for (int j = 0; j < kHeld; j++) {
            const int i = tid * 4 + j * 1024;
            v[j] = i < k ? *(const float4 *)(x + i) : float4{0.f, 0.f, 0.f, 0.f};
            amax = fmaxf(amax, fmaxf(fmaxf(fabsf(v[j].x), fabsf(v[j].y)), fmaxf(fabsf(v[j].z), fabsf(v[j].w))));
        }
    } else {
        for (int i = tid * 4; i < k; i += 1024) {
            float4 w = *(const float4 *)(x + i);
            amax = fmaxf(amax, fmaxf(fmaxf(fabsf(w.x), fabsf(w.y)), fmaxf(fabsf(w.z), fabsf(w.w))));
        }
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, JL_WAVE));
    if ((tid & 63) == 0) wave_max[tid >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(wave_max[0], wave_max[1]), fmaxf(wave_max[2], wave_max[3]));
    // Every row is brought to [2^11, 2^12) at its largest magnitude: huge rows stay finite in
    // fp16, tiny rows keep their bits out of fp16's subnormal range, and the power of two is
    // undone exactly in the epilogue.
    float scale = 1.f, inv = 1.f;
    if (amax > 0.f && amax < INFINITY) {
        int e;
        frexpf(amax, &e);  // amax = f * 2^e, f in [0.5, 1)
        e = e < -100 ? -100 : e;
        scale = ldexpf(1.f, e - 12);
        inv = ldexpf(1.f, 12 - e);
    }
    if (held) {
#pragma unroll
        for (int j = 0; j < kHeld; j++) {
            const int i = tid * 4 + j * 1024;
            if (i < k)
                *(jl_half4 *)(a + i) = jl_half4{(_Float16)(v[j].x * inv), (_Float16)(v[j].y * inv),
                                          (_Float16)(v[j].z * inv), (_Float16)(v[j].w * inv)};
        }
    } else {
        for (int i = tid * 4; i < k; i += 1024) {
            float4 w = *(const float4 *)(x + i);
            *(jl_half4 *)(a + i) = jl_half4{(_Float16)(w.x * inv), (_Float16)(w.y * inv), (_Float16)(w.z * inv),
                                      (_Float16)(w.w * inv)};
        }
    }
    if (tid == 0) row_scale[row] = scale;
}
