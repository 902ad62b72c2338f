// Decode matrix-vector kernels for Q8_0 / Q4_0 / Q4_K weights in their GGUF block layout.
//
// Replaces the one-workgroup-per-row TornadoVM kernels of the reference
// (J/backend/tornado/kernels/TransformerComputeKernelsLayered.java:2222-2479,
//  TransformerComputeKernelsQ4_0.java:531-701, TransformerComputeKernelsQ4_K.java:673-842)
// with a tile-streaming design for CDNA4:
//
//   * a thread owns one 64-element column slice of the row for the whole kernel and keeps those 64
//     activations in registers (loaded once, through LDS, coalesced);
//   * a workgroup walks tiles of R consecutive rows.  A tile is one contiguous byte range of the
//     weight (R * row_bytes), copied global -> registers -> LDS with 128-bit loads that ignore
//     block boundaries, so the 34- and 18-byte block strides never reach the memory system;
//   * each thread then reads its own slice of the tile from LDS with 32-bit reads -- a slice is a
//     pair of Q8_0 blocks (68 B), a pair of Q4_0 blocks (36 B) or a quarter of a Q4_K super-block
//     (32 B of nibbles + the shared 16 B header), all 4-byte aligned -- and unpacks in registers;
//   * the next tile's global loads are in flight while the current tile is computed (two LDS
//     stages, one barrier per tile);
//   * row sums fold across lanes with wave shuffles, and across waves (rows wider than 4096
//     columns) through a few LDS words.
//
// Memory-bound by design: no MFMA here.  Summation order differs from the host's sequential or
// lane-wise order, so results are held to a tolerance, not to bit equality; the element decode
// itself is held bit-equal by the kernels in jl_dequant.hip.
#include "jl_device.h"
#include "jl_internal.h"

#include <map>
#include <mutex>
#include <tuple>

namespace {

constexpr int kMaxSeg = 3;

struct GemvParams {
    const uint8_t *w[kMaxSeg];   // weight of each segment (q | k | v, or a single projection)
    float *out[kMaxSeg];
    int seg_rows[kMaxSeg];
    int seg_tile_begin[kMaxSeg + 1];  // first tile of each segment; [nseg] = total tiles
    int nseg;
    const uint8_t *w_up;  // JL_SWIGLU: the up weight, same shape as w[0]
    const float *x;
    int n;          // row length
    int S;          // 64-element slices per row
    int Sp;         // S padded: next power of two when S <= 64, else next multiple of 64
    int R;          // rows per tile
    int row_bytes;
    int epilogue;
};

template <int TYPE> struct Traits;
template <> struct Traits<JL_Q8_0> { static constexpr int kLoads = 5; };
template <> struct Traits<JL_Q4_0> { static constexpr int kLoads = 3; };
template <> struct Traits<JL_Q4_K> { static constexpr int kLoads = 3; };

__device__ __forceinline__ float ubyte(uint32_t v, int k) { return (float)((v >> (8 * k)) & 0xFFu); }
__device__ __forceinline__ float sbyte(uint32_t v, int k) { return (float)(int)(int8_t)(v >> (8 * k)); }

// Dot of one Q8_0 block pair (68 bytes, 4-byte aligned in LDS) with 64 activations.
//   bytes 0..1 scale A | 2..33 quants A | 34..35 scale B | 36..67 quants B
__device__ __forceinline__ float slice_dot_q8_0(const uint8_t *p, const float (&x)[64]) {
    const uint32_t *dw = (const uint32_t *)p;
    uint32_t w[17];
#pragma unroll
    for (int i = 0; i < 17; i++) w[i] = dw[i];
    float dA = jl_half_bits_to_float(w[0]);
    float dB = jl_half_bits_to_float(w[8] >> 16);
    float a0 = 0.f, a1 = 0.f, b0 = 0.f, b1 = 0.f;
    // block A: element i sits at byte 2 + i of the slice
#pragma unroll
    for (int i = 0; i < 32; i++) {
        int o = 2 + i;
        float q = sbyte(w[o >> 2], o & 3);
        if (i & 1) a1 = fmaf(q, x[i], a1); else a0 = fmaf(q, x[i], a0);
    }
    // block B: element i sits at byte 36 + i
#pragma unroll
    for (int i = 0; i < 32; i++) {
        float q = sbyte(w[9 + (i >> 2)], i & 3);
        if (i & 1) b1 = fmaf(q, x[32 + i], b1); else b0 = fmaf(q, x[32 + i], b0);
    }
    return fmaf(a0 + a1, dA, (b0 + b1) * dB);
}

// Dot of one Q4_0 block pair (36 bytes) with 64 activations; sx[0], sx[1] are the sums of the
// activations facing block A and block B, so that sum((q - 8) x) = sum(q x) - 8 sum(x).
//   bytes 0..1 scale A | 2..17 nibbles A | 18..19 scale B | 20..35 nibbles B
// element i < 16 of a block is the low nibble of its byte i, element 16 + i the high nibble.
__device__ __forceinline__ float slice_dot_q4_0(const uint8_t *p, const float (&x)[64],
                                                const float (&sx)[2]) {
    const uint32_t *dw = (const uint32_t *)p;
    uint32_t lo[9], hi[9];
    uint32_t w0 = dw[0], w4 = dw[4];
#pragma unroll
    for (int i = 0; i < 9; i++) {
        uint32_t v = dw[i];
        lo[i] = v & 0x0F0F0F0Fu;
        hi[i] = (v >> 4) & 0x0F0F0F0Fu;
    }
    float dA = jl_half_bits_to_float(w0);
    float dB = jl_half_bits_to_float(w4 >> 16);
    float a0 = 0.f, a1 = 0.f, b0 = 0.f, b1 = 0.f;
#pragma unroll
    for (int i = 0; i < 16; i++) {
        int o = 2 + i;  // byte i of block A
        a0 = fmaf(ubyte(lo[o >> 2], o & 3), x[i], a0);
        a1 = fmaf(ubyte(hi[o >> 2], o & 3), x[16 + i], a1);
    }
#pragma unroll
    for (int i = 0; i < 16; i++) {
        int o = 20 + i;  // byte i of block B
        b0 = fmaf(ubyte(lo[o >> 2], o & 3), x[32 + i], b0);
        b1 = fmaf(ubyte(hi[o >> 2], o & 3), x[48 + i], b1);
    }
    float da = fmaf(-8.f, sx[0], a0 + a1);
    float db = fmaf(-8.f, sx[1], b0 + b1);
    return fmaf(da, dA, db * dB);
}

// Dot of one quarter of a Q4_K super-block with 64 activations.  `hdr` is the super-block's first
// 16 bytes (d, dmin, 12 packed scale bytes), `qs` the 32 nibble bytes of pair `pair`: low nibbles
// are sub-block 2*pair (activations 0..31), high nibbles sub-block 2*pair+1 (activations 32..63).
// sum(w x) = (d sc) sum(q x) - (dmin m) sum(x) per sub-block.
__device__ __forceinline__ float slice_dot_q4_k(const uint8_t *hdr, const uint8_t *qs, int pair,
                                                const float (&x)[64], const float (&sx)[2]) {
    uint4 h = *(const uint4 *)hdr;
    uint4 q0 = *(const uint4 *)qs;
    uint4 q1 = *(const uint4 *)(qs + 16);
    uint32_t w[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
    float d = jl_half_bits_to_float(h.x);
    float dmin = jl_half_bits_to_float(h.x >> 16);
    int sc0, mn0, sc1, mn1;
    jl_q4k_scale_min(h.y, h.z, h.w, 2 * pair, sc0, mn0);
    jl_q4k_scale_min(h.y, h.z, h.w, 2 * pair + 1, sc1, mn1);
    float a0 = 0.f, a1 = 0.f, b0 = 0.f, b1 = 0.f;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        uint32_t lo = w[i] & 0x0F0F0F0Fu;
        uint32_t hi = (w[i] >> 4) & 0x0F0F0F0Fu;
        a0 = fmaf(ubyte(lo, 0), x[4 * i + 0], a0);
        a1 = fmaf(ubyte(lo, 1), x[4 * i + 1], a1);
        a0 = fmaf(ubyte(lo, 2), x[4 * i + 2], a0);
        a1 = fmaf(ubyte(lo, 3), x[4 * i + 3], a1);
        b0 = fmaf(ubyte(hi, 0), x[32 + 4 * i + 0], b0);
        b1 = fmaf(ubyte(hi, 1), x[32 + 4 * i + 1], b1);
        b0 = fmaf(ubyte(hi, 2), x[32 + 4 * i + 2], b0);
        b1 = fmaf(ubyte(hi, 3), x[32 + 4 * i + 3], b1);
    }
    float lo_term = (d * (float)sc0) * (a0 + a1) - (dmin * (float)mn0) * sx[0];
    float hi_term = (d * (float)sc1) * (b0 + b1) - (dmin * (float)mn1) * sx[1];
    return lo_term + hi_term;
}

template <int TYPE>
__device__ __forceinline__ float slice_dot(const uint8_t *tile, int r, int s, int row_bytes,
                                           const float (&x)[64], const float (&sx)[2]) {
    const uint8_t *row = tile + r * row_bytes;
    if constexpr (TYPE == JL_Q8_0) {
        return slice_dot_q8_0(row + s * 68, x);
    } else if constexpr (TYPE == JL_Q4_0) {
        return slice_dot_q4_0(row + s * 36, x, sx);
    } else {
        const uint8_t *sb = row + (s >> 2) * 144;
        return slice_dot_q4_k(sb, sb + 16 + (s & 3) * 32, s & 3, x, sx);
    }
}

// LDS map: [0, 256) cross-wave partial sums (2 parities x 2 results x up to 8 waves... 32 floats
// used), then a region that first holds the activation vector and afterwards the tile stages.
constexpr int kPartialBytes = 256;

template <int TYPE, bool DUAL>
__global__ void __launch_bounds__(256) jl_gemv_tiles(GemvParams p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    constexpr int NL = Traits<TYPE>::kLoads;
    constexpr int NW = DUAL ? 2 : 1;

    const int tid = threadIdx.x;
    const int nthreads = blockDim.x;
    const int r = tid / p.Sp;
    const int s = tid - r * p.Sp;
    const bool active = (s < p.S) && (r < p.R);
    const int tile_bytes = p.R * p.row_bytes;  // a multiple of 16 (checked on the host)
    const int total_tiles = p.seg_tile_begin[p.nseg];

    float *partial = (float *)lds;
    uint8_t *region = lds + kPartialBytes;

    uint4 stg[NW][NL];

    // Start the first tile's loads before anything else so they overlap the activation set-up.
    auto issue = [&](int tile) {
        int seg = 0;
#pragma unroll
        for (int i = 1; i < kMaxSeg; i++)
            if (i < p.nseg && tile >= p.seg_tile_begin[i]) seg = i;
        int local = tile - p.seg_tile_begin[seg];
        int64_t offset = (int64_t)local * tile_bytes;
        int64_t remain = (int64_t)p.seg_rows[seg] * p.row_bytes - offset;
        int bytes = remain < tile_bytes ? (int)remain : tile_bytes;
        const uint8_t *base = p.w[seg] + offset;
#pragma unroll
        for (int k = 0; k < NL; k++) {
            int off = (k * nthreads + tid) * 16;
            stg[0][k] = off < bytes ? *(const uint4 *)(base + off) : make_uint4(0, 0, 0, 0);
        }
        if constexpr (DUAL) {
            const uint8_t *base_up = p.w_up + offset;
#pragma unroll
            for (int k = 0; k < NL; k++) {
                int off = (k * nthreads + tid) * 16;
                stg[1][k] = off < bytes ? *(const uint4 *)(base_up + off) : make_uint4(0, 0, 0, 0);
            }
        }
    };
    auto commit = [&](uint8_t *buf) {
#pragma unroll
        for (int w = 0; w < NW; w++) {
#pragma unroll
            for (int k = 0; k < NL; k++) {
                int off = (k * nthreads + tid) * 16;
                if (off < tile_bytes) *(uint4 *)(buf + w * tile_bytes + off) = stg[w][k];
            }
        }
    };

    int tile = blockIdx.x;
    if (tile < total_tiles) issue(tile);

    // activations: global -> LDS (coalesced) -> 64 registers per thread
    float *xs = (float *)region;
    for (int i = tid * 4; i < p.n; i += nthreads * 4) *(float4 *)(xs + i) = *(const float4 *)(p.x + i);
    __syncthreads();
    float x[64];
    float sx[2] = {0.f, 0.f};
    if (active) {
#pragma unroll
        for (int k = 0; k < 16; k++) {
            float4 v = *(const float4 *)(xs + s * 64 + 4 * k);
            x[4 * k + 0] = v.x;
            x[4 * k + 1] = v.y;
            x[4 * k + 2] = v.z;
            x[4 * k + 3] = v.w;
        }
    } else {
#pragma unroll
        for (int k = 0; k < 64; k++) x[k] = 0.f;
    }
    if constexpr (TYPE != JL_Q8_0) {
#pragma unroll
        for (int k = 0; k < 32; k++) {
            sx[0] += x[k];
            sx[1] += x[32 + k];
        }
    }
    __syncthreads();  // the activation staging area is reused by the tile stages below

    const int stage_bytes = NW * tile_bytes;
    const int waves_per_row = p.Sp > JL_WAVE ? p.Sp / JL_WAVE : 1;
    const int wave = tid / JL_WAVE;
    const int lane = tid & (JL_WAVE - 1);

    // Finishes the rows of a tile whose per-wave partial sums sit in `partial` (rows wider than a
    // wave only): thread `row * Sp` adds its row's wave partials and applies the epilogue.
    auto write_out = [&](int t, float v0, float v1) {
        int seg = 0;
#pragma unroll
        for (int i = 1; i < kMaxSeg; i++)
            if (i < p.nseg && t >= p.seg_tile_begin[i]) seg = i;
        int row = (t - p.seg_tile_begin[seg]) * p.R + r;
        if (row < p.seg_rows[seg]) {
            float *o = p.out[seg] + row;
            if (p.epilogue == JL_SWIGLU) *o = jl_swiglu_value(v0, v1);
            else if (p.epilogue == JL_RESIDUAL) *o = *o + v0;
            else *o = v0;
        }
    };
    auto finish_wide = [&](int t, int parity) {
        if (s == 0 && r < p.R) {
            float v0 = 0.f, v1 = 0.f;
            for (int k = 0; k < waves_per_row; k++) {
                v0 += partial[(parity * 2 + 0) * 8 + r * waves_per_row + k];
                if constexpr (DUAL) v1 += partial[(parity * 2 + 1) * 8 + r * waves_per_row + k];
            }
            write_out(t, v0, v1);
        }
    };

    int iter = 0;
    int prev_tile = -1;
    for (; tile < total_tiles; tile += gridDim.x, iter++) {
        uint8_t *buf = region + (iter & 1) * stage_bytes;
        commit(buf);
        int next = tile + gridDim.x;
        if (next < total_tiles) issue(next);
        __syncthreads();
        if (waves_per_row > 1 && prev_tile >= 0) finish_wide(prev_tile, (iter - 1) & 1);

        float v0 = 0.f, v1 = 0.f;
        if (active) {
            v0 = slice_dot<TYPE>(buf, r, s, p.row_bytes, x, sx);
            if constexpr (DUAL) v1 = slice_dot<TYPE>(buf + tile_bytes, r, s, p.row_bytes, x, sx);
        }
        if (waves_per_row == 1) {
            v0 = jl_group_sum_dyn(v0, p.Sp);
            if constexpr (DUAL) v1 = jl_group_sum_dyn(v1, p.Sp);
            if (s == 0 && r < p.R) write_out(tile, v0, v1);
        } else {
            v0 = jl_group_sum<JL_WAVE>(v0);
            if constexpr (DUAL) v1 = jl_group_sum<JL_WAVE>(v1);
            if (lane == 0) {
                partial[((iter & 1) * 2 + 0) * 8 + wave] = v0;
                if constexpr (DUAL) partial[((iter & 1) * 2 + 1) * 8 + wave] = v1;
            }
        }
        prev_tile = tile;
    }
    if (waves_per_row > 1 && prev_tile >= 0) {
        __syncthreads();
        finish_wide(prev_tile, (iter - 1) & 1);
    }
}

// Catch-all for shapes the tile kernel does not take (row length not a multiple of 64, rows wider
// than 16384 columns, unaligned buffers): one wave per row, lanes stride over blocks, byte loads.
template <int TYPE>
__device__ float block_dot_generic(const uint8_t *blk, const float *x) {
    float acc = 0.f;
    if constexpr (TYPE == JL_Q8_0) {
        float d = jl_half_bits_to_float(blk[0] | (blk[1] << 8));
        for (int i = 0; i < 32; i++) acc = fmaf((float)(int)(int8_t)blk[2 + i], x[i], acc);
        return acc * d;
    } else if constexpr (TYPE == JL_Q4_0) {
        float d = jl_half_bits_to_float(blk[0] | (blk[1] << 8));
        for (int i = 0; i < 16; i++) {
            int b = blk[2 + i];
            acc = fmaf((float)((b & 0xF) - 8), x[i], acc);
            acc = fmaf((float)((b >> 4) - 8), x[16 + i], acc);
        }
        return acc * d;
    } else {
        const uint32_t *hdr = (const uint32_t *)blk;
        float d = jl_half_bits_to_float(hdr[0]);
        float dmin = jl_half_bits_to_float(hdr[0] >> 16);
        for (int j = 0; j < 8; j++) {
            int sc, mn;
            jl_q4k_scale_min(hdr[1], hdr[2], hdr[3], j, sc, mn);
            float qx = 0.f, sx = 0.f;
            const uint8_t *qs = blk + 16 + (j >> 1) * 32;
            for (int i = 0; i < 32; i++) {
                int q = (j & 1) ? (qs[i] >> 4) : (qs[i] & 0xF);
                qx = fmaf((float)q, x[j * 32 + i], qx);
                sx += x[j * 32 + i];
            }
            acc += (d * (float)sc) * qx - (dmin * (float)mn) * sx;
        }
        return acc;
    }
}

template <int TYPE>
__global__ void __launch_bounds__(256)
jl_gemv_generic(const uint8_t *__restrict__ w, const uint8_t *__restrict__ w_up,
                const float *__restrict__ x, float *__restrict__ out, int rows, int n, int epilogue) {
    constexpr int BE = TYPE == JL_Q4_K ? 256 : 32;
    constexpr int BB = TYPE == JL_Q4_K ? 144 : TYPE == JL_Q8_0 ? 34 : 18;
    int row = blockIdx.x * (blockDim.x / JL_WAVE) + threadIdx.x / JL_WAVE;
    int lane = threadIdx.x & (JL_WAVE - 1);
    if (row >= rows) return;
    int blocks = n / BE;
    const uint8_t *wr = w + (int64_t)row * blocks * BB;
    float v0 = 0.f, v1 = 0.f;
    for (int b = lane; b < blocks; b += JL_WAVE) {
        v0 += block_dot_generic<TYPE>(wr + (int64_t)b * BB, x + b * BE);
        if (w_up) v1 += block_dot_generic<TYPE>(w_up + ((int64_t)row * blocks + b) * BB, x + b * BE);
    }
    v0 = jl_group_sum<JL_WAVE>(v0);
    v1 = jl_group_sum<JL_WAVE>(v1);
    if (lane == 0) {
        if (epilogue == JL_SWIGLU) out[row] = jl_swiglu_value(v0, v1);
        else if (epilogue == JL_RESIDUAL) out[row] += v0;
        else out[row] = v0;
    }
}

// ---- host side ------------------------------------------------------------------------------

int next_pow2(int v) {
    int p = 1;
    while (p < v) p <<= 1;
    return p;
}

struct OccKey {
    const void *fn;
    int device, threads, lds;
    bool operator<(const OccKey &o) const {
        return std::tie(fn, device, threads, lds) < std::tie(o.fn, o.device, o.threads, o.lds);
    }
};

// Workgroups of `fn` that fit one compute unit; asked of the runtime once per configuration.
int blocks_per_cu(const void *fn, int device, int threads, int lds) {
    static std::mutex mu;
    static std::map<OccKey, int> cache;
    std::lock_guard<std::mutex> g(mu);
    OccKey key{fn, device, threads, lds};
    auto it = cache.find(key);
    if (it != cache.end()) return it->second;
    (void)hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    int nb = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&nb, fn, threads, (size_t)lds) != hipSuccess ||
        nb < 1) {
        (void)hipGetLastError();
        nb = 1;
    }
    cache[key] = nb;
    return nb;
}

template <int TYPE, bool DUAL>
int launch_tiles(jl_context *ctx, const GemvParams &p, int threads, int lds) {
    auto fn = jl_gemv_tiles<TYPE, DUAL>;
    int per_cu = blocks_per_cu((const void *)fn, ctx->device, threads, lds);
    int total = p.seg_tile_begin[p.nseg];
    int grid = ctx->compute_units * per_cu;
    if (grid > total) grid = total;
    hipLaunchKernelGGL(fn, dim3(grid), dim3(threads), lds, ctx->stream, p);
    JL_HIP(hipGetLastError());
    return JL_OK;
}

template <int TYPE>
int launch_generic(jl_context *ctx, const jl_weight *w, const jl_weight *w_up, const float *x,
                   float *out, int epilogue) {
    int rows = (int)w->rows;
    hipLaunchKernelGGL(jl_gemv_generic<TYPE>, dim3((rows + 3) / 4), dim3(256), 0, ctx->stream,
                       w->blocks, w_up ? w_up->blocks : nullptr, x, out, rows, (int)w->cols, epilogue);
    JL_HIP(hipGetLastError());
    return JL_OK;
}

}  // namespace

int jl_launch_gemv(jl_context *ctx, const jl_weight *const *w, int nseg, float *const *outs,
                   const jl_weight *w_up, const float *x, int epilogue) {
    const int type = w[0]->type;
    const int n = (int)w[0]->cols;
    const int slice_bytes = type == JL_Q8_0 ? 68 : 36;
    const int row_bytes = n / jl_block_elems(type) * jl_block_bytes(type);

    bool fast = (n % 64 == 0) && (n / 64 <= 256) && (((uintptr_t)x & 15) == 0);
    int S = n / 64, Sp = 0, R = 0;
    if (fast) {
        Sp = S <= 64 ? next_pow2(S) : (S + 63) / 64 * 64;
        R = 256 / Sp;
        if (R < 1) fast = false;
        else if (((int64_t)R * row_bytes) % 16 != 0) fast = false;
    }
    for (int i = 0; fast && i < nseg; i++) {
        if (((uintptr_t)w[i]->blocks & 15) != 0) fast = false;
    }
    if (w_up && ((uintptr_t)w_up->blocks & 15) != 0) fast = false;
    (void)slice_bytes;

    if (!fast) {
        for (int i = 0; i < nseg; i++) {
            int st;
            switch (type) {
                case JL_Q8_0: st = launch_generic<JL_Q8_0>(ctx, w[i], w_up, x, outs[i], epilogue); break;
                case JL_Q4_0: st = launch_generic<JL_Q4_0>(ctx, w[i], w_up, x, outs[i], epilogue); break;
                case JL_Q4_K: st = launch_generic<JL_Q4_K>(ctx, w[i], w_up, x, outs[i], epilogue); break;
                default:
                    return jl_fail(JL_ERR_UNSUPPORTED,
                                   "no single-token projection kernel for a ggml type %d weight", type);
            }
            if (st != JL_OK) return st;
        }
        return JL_OK;
    }

    GemvParams p{};
    p.nseg = nseg;
    int tiles = 0;
    for (int i = 0; i < nseg; i++) {
        p.w[i] = w[i]->blocks;
        p.out[i] = outs[i];
        p.seg_rows[i] = (int)w[i]->rows;
        p.seg_tile_begin[i] = tiles;
        tiles += ((int)w[i]->rows + R - 1) / R;
    }
    p.seg_tile_begin[nseg] = tiles;
    p.w_up = w_up ? w_up->blocks : nullptr;
    p.x = x;
    p.n = n;
    p.S = S;
    p.Sp = Sp;
    p.R = R;
    p.row_bytes = row_bytes;
    p.epilogue = epilogue;

    const int threads = (R * Sp + 63) / 64 * 64;
    const int tile_bytes = R * row_bytes;
    const int stages = 2 * (w_up ? 2 : 1) * tile_bytes;
    const int region = stages > n * 4 ? stages : n * 4;
    const int lds = kPartialBytes + region;

    const bool dual = w_up != nullptr;
    switch (type) {
        case JL_Q8_0:
            return dual ? launch_tiles<JL_Q8_0, true>(ctx, p, threads, lds)
                        : launch_tiles<JL_Q8_0, false>(ctx, p, threads, lds);
        case JL_Q4_0:
            return dual ? launch_tiles<JL_Q4_0, true>(ctx, p, threads, lds)
                        : launch_tiles<JL_Q4_0, false>(ctx, p, threads, lds);
        case JL_Q4_K:
            return dual ? launch_tiles<JL_Q4_K, true>(ctx, p, threads, lds)
                        : launch_tiles<JL_Q4_K, false>(ctx, p, threads, lds);
        default:
            return jl_fail(JL_ERR_UNSUPPORTED,
                           "no single-token projection kernel for a ggml type %d weight", type);
    }
}
