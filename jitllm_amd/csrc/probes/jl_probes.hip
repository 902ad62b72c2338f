// Measurement aids, not part of libjitllm_hip.so: the rates this chip sustains with nothing else in
// the way -- fp16 matrix instructions out of registers (constant and random operands), and a plain
// streaming read of HBM.  bench.py prints them beside the published peaks its fractions use.
//
// The published dense fp16 figure (2.5 PFLOP/s) is 256 compute units x 4096 flops per clock at
// 2.4 GHz.  A loop of nothing but v_mfma_f32_16x16x32_f16 reaches it when every operand is 1.0; with
// random operands the same loop runs slower -- the chip lowers its clock under the load of the
// toggling multipliers -- and that lower rate is the ceiling a GEMM on real data can approach.
// bench.py --mfma-rate-probe prints both, beside the prefill GEMM's own figure.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef uint32_t uintx4 __attribute__((ext_vector_type(4)));

// SHAPE 0: 16x16x32 over a 128 x 64 wave tile (8 x 4 blocks, as the prefill GEMM's widest tile);
// SHAPE 1: 32x32x16 over the same wave tile (4 x 2 blocks).  64 (32) instructions per step and wave.
template <int SHAPE>
__global__ void __launch_bounds__(512) probe_mfma(int steps, const half8 *src, float *out) {
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    float sum = 0;
    if constexpr (SHAPE == 0) {
        half8 fa[2][8], fb[2][4];
        for (int h = 0; h < 2; h++) {
            for (int i = 0; i < 8; i++) fa[h][i] = src[(t * 24 + h * 12 + i) & 0xFFFFF];
            for (int j = 0; j < 4; j++) fb[h][j] = src[(t * 24 + h * 12 + 8 + j) & 0xFFFFF];
        }
        floatx4 acc[8][4];
        for (int i = 0; i < 8; i++)
            for (int j = 0; j < 4; j++) acc[i][j] = floatx4{0, 0, 0, 0};
        for (int s = 0; s < steps; s++) {
#pragma unroll
            for (int h = 0; h < 2; h++)
#pragma unroll
                for (int i = 0; i < 8; i++)
#pragma unroll
                    for (int j = 0; j < 4; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fb[h][j], fa[h][i], acc[i][j], 0, 0, 0);
            asm volatile("" : "+v"(fa[0][0]), "+v"(fb[0][0]));   // the loop is not to be folded
        }
        for (int i = 0; i < 8; i++)
            for (int j = 0; j < 4; j++) sum += acc[i][j][0] + acc[i][j][3];
    } else {
        half8 fa[2][2][4], fb[2][2][2];
        for (int h = 0; h < 2; h++)
            for (int kk = 0; kk < 2; kk++) {
                for (int i = 0; i < 4; i++) fa[h][kk][i] = src[(t * 24 + h * 12 + kk * 6 + i) & 0xFFFFF];
                for (int j = 0; j < 2; j++) fb[h][kk][j] = src[(t * 24 + h * 12 + kk * 6 + 4 + j) & 0xFFFFF];
            }
        floatx16 acc[4][2];
        for (int i = 0; i < 4; i++)
            for (int j = 0; j < 2; j++)
                for (int e = 0; e < 16; e++) acc[i][j][e] = 0;
        for (int s = 0; s < steps; s++) {
#pragma unroll
            for (int h = 0; h < 2; h++)
#pragma unroll
                for (int kk = 0; kk < 2; kk++)
#pragma unroll
                    for (int i = 0; i < 4; i++)
#pragma unroll
                        for (int j = 0; j < 2; j++)
                            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[h][kk][j], fa[h][kk][i], acc[i][j], 0, 0, 0);
            asm volatile("" : "+v"(fa[0][0][0]), "+v"(fb[0][0][0]));
        }
        for (int i = 0; i < 4; i++)
            for (int j = 0; j < 2; j++) sum += acc[i][j][0] + acc[i][j][15];
    }
    out[t] = sum;
}

__global__ void probe_fill(uint16_t *dst, size_t n, int random) {
    // random: fp16 values k / 500 for k uniform in -1000 .. 1000 (a 32-bit LCG per element); else 1.0
    for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        uint32_t s = (uint32_t)i * 2654435761u + 12345u;
        s = s * 1664525u + 1013904223u;
        s = s * 1664525u + 1013904223u;
        const float v = random ? ((int)((s >> 8) % 2001u) - 1000) / 500.0f : 1.0f;
        const _Float16 h = (_Float16)v;
        dst[i] = __builtin_bit_cast(uint16_t, h);
    }
}

// Streams `n16` 16-byte pieces once: every thread has eight loads in flight, workgroups take
// interleaved 32 KB runs.  What it reads is folded into one word per thread so that no load is dropped.
__global__ void __launch_bounds__(256) probe_read(const uintx4 *src, size_t n16, uint32_t *out) {
    const size_t stride = (size_t)gridDim.x * 256 * 8;
    uint32_t acc = 0;
    for (size_t i = (size_t)blockIdx.x * 256 * 8 + threadIdx.x; i + 7 * 256 < n16; i += stride) {
        uintx4 v[8];
#pragma unroll
        for (int j = 0; j < 8; j++) v[j] = __builtin_nontemporal_load(src + i + j * 256);
#pragma unroll
        for (int j = 0; j < 8; j++) acc ^= v[j][0] ^ v[j][1] ^ v[j][2] ^ v[j][3];
    }
    out[blockIdx.x * 256 + threadIdx.x] = acc;
}

}  // namespace

// The rate at which the chip streams `bytes` (far more than its 256 MB memory-side cache) from HBM
// with plain 16-byte loads: `reps` launches, GB/s of each into gbps[0 .. reps).  The decode
// kernels' fractions of the published 8 TB/s are to be read against this.
extern "C" int jl_probe_hbm_read_rate(int device, size_t bytes, int reps, int compute_units, double *gbps) {
    hipError_t e = hipSetDevice(device);
    if (e != hipSuccess) return (int)e;
    uintx4 *src = nullptr;
    uint32_t *out = nullptr;
    const int blocks = compute_units * 8;
    if ((e = hipMalloc(&src, bytes)) != hipSuccess) return (int)e;
    if ((e = hipMalloc(&out, (size_t)blocks * 256 * 4)) != hipSuccess) return (int)e;
    (void)hipMemset(src, 1, bytes);
    hipEvent_t e0, e1;
    (void)hipEventCreate(&e0);
    (void)hipEventCreate(&e1);
    const size_t n16 = bytes / 16;
    const size_t per_pass = (size_t)blocks * 256 * 8;
    const size_t read16 = n16 / per_pass * per_pass;   // what the loop covers
    for (int r = 0; r < reps; r++) {
        (void)hipEventRecord(e0, 0);
        hipLaunchKernelGGL(probe_read, dim3(blocks), dim3(256), 0, 0, src, n16, out);
        (void)hipEventRecord(e1, 0);
        if ((e = hipEventSynchronize(e1)) != hipSuccess) break;
        float ms = 0;
        (void)hipEventElapsedTime(&ms, e0, e1);
        gbps[r] = (double)read16 * 16.0 / (ms * 1e-3) / 1e9;
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    (void)hipFree(src);
    (void)hipFree(out);
    return (int)e;
}

// Runs `reps` launches of `steps` loop steps on one workgroup of 8 waves per compute unit and
// writes each launch's TFLOP/s into tflops[0 .. reps).  Returns 0, or the HIP error code.
extern "C" int jl_probe_mfma_rate(int device, int shape, int random, int steps, int reps, int compute_units,
                                  double *tflops) {
    hipError_t e = hipSetDevice(device);
    if (e != hipSuccess) return (int)e;
    const size_t n = (size_t)1 << 20;   // half8 vectors
    half8 *src = nullptr;
    float *out = nullptr;
    if ((e = hipMalloc(&src, n * sizeof(half8))) != hipSuccess) return (int)e;
    if ((e = hipMalloc(&out, (size_t)compute_units * 512 * sizeof(float))) != hipSuccess) return (int)e;
    hipLaunchKernelGGL(probe_fill, dim3(1024), dim3(256), 0, 0, (uint16_t *)src, n * 8, random);
    hipEvent_t e0, e1;
    (void)hipEventCreate(&e0);
    (void)hipEventCreate(&e1);
    for (int r = 0; r < reps; r++) {
        (void)hipEventRecord(e0, 0);
        if (shape == 0) hipLaunchKernelGGL(probe_mfma<0>, dim3(compute_units), dim3(512), 0, 0, steps, src, out);
        else hipLaunchKernelGGL(probe_mfma<1>, dim3(compute_units), dim3(512), 0, 0, steps, src, out);
        (void)hipEventRecord(e1, 0);
        if ((e = hipEventSynchronize(e1)) != hipSuccess) break;
        float ms = 0;
        (void)hipEventElapsedTime(&ms, e0, e1);
        // per step and wave: 64 x 16x16x32 (or 32 x 32x32x16) = 64 x 16384 multiply-adds
        const double flop = (double)compute_units * 8 * steps * 64.0 * 16384.0;
        tflops[r] = flop / (ms * 1e-3) / 1e12;
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    (void)hipFree(src);
    (void)hipFree(out);
    return (int)e;
}
