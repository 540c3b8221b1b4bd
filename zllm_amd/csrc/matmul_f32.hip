// Prefill multiplies at full f32 precision (the reference's scalar_f32 rung,
// src/precision.zig:9): out[t][col0 + j] (+)= sum_i x[t][i] * w[j][i] for BF16
// weights (src/kernels/matmul_half.wgsl) and for Q8_0 split rows with
// unrounded f32 activations and split-k slices
// (src/kernels/matmul_q8_0_float.wgsl). Each output is accumulated in
// increasing k order whatever the tile occupancy, so a launch over a chunk of
// the tokens gives those tokens the same bits as a launch over all of them
// (src/kernels/matmul_q8_0_float.wgsl:9-10).
//
// A workgroup computes 64 tokens x 64 outputs from 32-deep tiles staged in
// LDS; a thread owns 4 tokens x 4 outputs.
#include <hip/hip_runtime.h>

#include "common.h"
#include "decode.h"

namespace zhip {

struct MmArgs {
    const float *x;
    const uint8_t *w;
    float *out;
    uint32_t rows, n, k, col0, out_stride, accumulate, k_slice, slice_stride;
    uint32_t row_bytes;
};

struct WBf16 {
    // 32 weights of row `row` from position k0.
    __device__ static void load8(const uint8_t *row, uint32_t, uint32_t k0, uint32_t c8, float (&w)[8]) {
        const uint4 q = *reinterpret_cast<const uint4 *>(row + 2u * (k0 + 8u * c8));
        const uint32_t words[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int e = 0; e < 4; e++) {
            w[2 * e] = __uint_as_float(words[e] << 16);
            w[2 * e + 1] = __uint_as_float(words[e] & 0xffff0000u);
        }
    }
};

struct WF16 {
    __device__ static void load8(const uint8_t *row, uint32_t, uint32_t k0, uint32_t c8, float (&w)[8]) {
        const uint4 q = *reinterpret_cast<const uint4 *>(row + 2u * (k0 + 8u * c8));
        const uint32_t words[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int e = 0; e < 4; e++) {
            w[2 * e] = half_bits_to_float(words[e] & 0xffffu);
            w[2 * e + 1] = half_bits_to_float(words[e] >> 16);
        }
    }
};

struct WQ8_0 {
    __device__ static void load8(const uint8_t *row, uint32_t k, uint32_t k0, uint32_t c8, float (&w)[8]) {
        const uint2 q = *reinterpret_cast<const uint2 *>(row + k0 + 8u * c8);
        const float d = half_bits_to_float(*reinterpret_cast<const uint16_t *>(row + k + 2u * (k0 / 32u)));
        const int32_t words[2] = {(int32_t)q.x, (int32_t)q.y};
#pragma unroll
        for (int e = 0; e < 2; e++) {
            w[4 * e + 0] = __fmul_rn(d, (float)((words[e] << 24) >> 24));
            w[4 * e + 1] = __fmul_rn(d, (float)((words[e] << 16) >> 24));
            w[4 * e + 2] = __fmul_rn(d, (float)((words[e] << 8) >> 24));
            w[4 * e + 3] = __fmul_rn(d, (float)(words[e] >> 24));
        }
    }
};

constexpr int TT = 64, TN = 64, TK = 32;

template <class W>
__global__ __launch_bounds__(256) void matmul_f32_kernel(MmArgs a) {
    __shared__ float xs[TT][TK + 1];
    __shared__ float ws[TN][TK + 1];
    const uint32_t tid = threadIdx.x;
    const uint32_t j0 = blockIdx.x * TN, t0 = blockIdx.y * TT, z = blockIdx.z;
    const uint32_t kb = z * a.k_slice;
    const uint32_t ke = min(a.k, kb + a.k_slice);
    const uint32_t tt = tid / 16u, tn = tid % 16u;
    float acc[4][4] = {};

    for (uint32_t k0 = kb; k0 < ke; k0 += TK) {
        // x tile: 64 x 32 floats, one row of 8 per thread.
        {
            const uint32_t r = tid / 4u, c8 = tid % 4u;
            const uint32_t t = t0 + r;
            float4 v0 = make_float4(0.f, 0.f, 0.f, 0.f), v1 = v0;
            if (t < a.rows) {
                const float4 *src = reinterpret_cast<const float4 *>(a.x + (size_t)t * a.k + k0 + 8u * c8);
                v0 = src[0];
                v1 = src[1];
            }
            float *dst = &xs[r][8u * c8];
            dst[0] = v0.x; dst[1] = v0.y; dst[2] = v0.z; dst[3] = v0.w;
            dst[4] = v1.x; dst[5] = v1.y; dst[6] = v1.z; dst[7] = v1.w;
        }
        // w tile: 64 rows x 32 weights, 8 per thread.
        {
            const uint32_t r = tid / 4u, c8 = tid % 4u;
            const uint32_t j = j0 + r;
            float w[8] = {};
            if (j < a.n) W::load8(a.w + (size_t)j * a.row_bytes, a.k, k0, c8, w);
            float *dst = &ws[r][8u * c8];
#pragma unroll
            for (int e = 0; e < 8; e++) dst[e] = w[e];
        }
        __syncthreads();
#pragma unroll 8
        for (int c = 0; c < TK; c++) {
            float xv[4], wv[4];
#pragma unroll
            for (int q = 0; q < 4; q++) {
                xv[q] = xs[tt * 4 + q][c];
                wv[q] = ws[tn + 16 * q][c];
            }
#pragma unroll
            for (int r = 0; r < 4; r++)
#pragma unroll
                for (int q = 0; q < 4; q++) acc[r][q] = fmaf(xv[r], wv[q], acc[r][q]);
        }
        __syncthreads();
    }

#pragma unroll
    for (int r = 0; r < 4; r++) {
        const uint32_t t = t0 + tt * 4 + r;
        if (t >= a.rows) continue;
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const uint32_t j = j0 + tn + 16 * q;
            if (j >= a.n) continue;
            const size_t o = (size_t)z * a.slice_stride + (size_t)t * a.out_stride + a.col0 + j;
            a.out[o] = a.accumulate ? a.out[o] + acc[r][q] : acc[r][q];
        }
    }
}

// Checks a prefill multiply's parameters and bound ranges, for either rung.
// The reference kernels' tile sizes (64 outputs x 16 tokens) give the logical
// grid its meaning: the outputs and tokens it covers. `*empty` is set when the
// dispatch has nothing to do. `x_bytes` is the size of one activation as bound
// (4: f32, 2: packed bf16).
zhip_result validate_matmul(const Dispatch &d, const char *name, bool sliced, bool q8_0, uint32_t x_bytes, bool *empty) {
    *empty = false;
    if (d.params_size < sizeof(MatmulParams)) return fail(d, ZHIP_E_BAD_COMMAND, "%s: params block too small", name);
    const MatmulParams &p = *reinterpret_cast<const MatmulParams *>(d.params);
    for (int b = 1; b <= 3; b++)
        if (!d.bind[b].bound) return fail(d, ZHIP_E_BAD_COMMAND, "%s: binding %d is not bound", name, b);
    if (d.grid[0] == 0 || d.grid[1] == 0 || d.grid[2] == 0) { *empty = true; return ZHIP_OK; }
    if (p.k == 0 || p.k % 32u != 0) return fail(d, ZHIP_E_BAD_COMMAND, "%s: k = %u is not a multiple of 32", name, p.k);
    const uint64_t cover_n = (uint64_t)d.grid[0] * 64u, cover_t = (uint64_t)d.grid[1] * 16u;
    const uint64_t n = cover_n < p.n ? cover_n : p.n, rows = cover_t < p.rows ? cover_t : p.rows;
    uint64_t slices = 1, slice_stride = 0;
    if (sliced) {
        if (p.k_slice == 0 || p.k_slice % 32u != 0) return fail(d, ZHIP_E_BAD_COMMAND, "%s: k_slice = %u", name, p.k_slice);
        slices = d.grid[2];
        slice_stride = p.slice_stride;
        if ((slices - 1) * p.k_slice >= p.k) return fail(d, ZHIP_E_BAD_COMMAND, "%s: %u slices of %u exceed k = %u", name, (uint32_t)slices, p.k_slice, p.k);
    } else if (d.grid[2] != 1) {
        return fail(d, ZHIP_E_BAD_COMMAND, "%s: grid z must be 1", name);
    }
    if (n == 0 || rows == 0) { *empty = true; return ZHIP_OK; }
    const uint64_t row_bytes = q8_0 ? ((p.k + p.k / 16u + 15u) & ~15u) : 2u * p.k;
    const uint64_t x_need = rows * p.k * x_bytes;
    const uint64_t w_need = n * row_bytes;
    const uint64_t o_need = ((slices - 1) * slice_stride + (rows - 1) * p.out_stride + p.col0 + n) * 4u;
    if (x_need > d.bind[1].size || w_need > d.bind[2].size || o_need > d.bind[3].size)
        return fail(d, ZHIP_E_BAD_COMMAND, "%s: bound ranges too small (x %llu/%llu, w %llu/%llu, out %llu/%llu)", name,
            (unsigned long long)x_need, (unsigned long long)d.bind[1].size, (unsigned long long)w_need, (unsigned long long)d.bind[2].size,
            (unsigned long long)o_need, (unsigned long long)d.bind[3].size);
    if (((uintptr_t)d.bind[1].ptr | (uintptr_t)d.bind[2].ptr) & 15u) return fail(d, ZHIP_E_BAD_COMMAND, "%s: x and weights must be 16-byte aligned", name);
    if ((uintptr_t)d.bind[3].ptr & 3u) return fail(d, ZHIP_E_BAD_COMMAND, "%s: out must be 4-byte aligned", name);
    return ZHIP_OK;
}

template <class W>
static zhip_result launch_matmul(const Dispatch &d, const char *name, bool sliced, bool q8_0) {
    bool empty = false;
    if (zhip_result r = validate_matmul(d, name, sliced, q8_0, 4u, &empty)) return r;
    if (empty) return ZHIP_OK;
    const MatmulParams &p = *reinterpret_cast<const MatmulParams *>(d.params);
    MmArgs a{};
    const uint64_t cover_n = (uint64_t)d.grid[0] * 64u, cover_t = (uint64_t)d.grid[1] * 16u;
    a.n = (uint32_t)(cover_n < p.n ? cover_n : p.n);
    a.rows = (uint32_t)(cover_t < p.rows ? cover_t : p.rows);
    a.k = p.k; a.col0 = p.col0; a.out_stride = p.out_stride; a.accumulate = p.accumulate;
    a.k_slice = sliced ? p.k_slice : p.k;
    a.slice_stride = sliced ? p.slice_stride : 0;
    a.row_bytes = q8_0 ? ((p.k + p.k / 16u + 15u) & ~15u) : 2u * p.k;
    a.x = reinterpret_cast<const float *>(d.bind[1].ptr);
    a.w = d.bind[2].ptr;
    a.out = reinterpret_cast<float *>(d.bind[3].ptr);
    const dim3 grid((a.n + TN - 1) / TN, (a.rows + TT - 1) / TT, sliced ? d.grid[2] : 1);
    hipLaunchKernelGGL((matmul_f32_kernel<W>), grid, dim3(256), 0, d.stream, a);
    return check_launch(d, name);
}

zhip_result launch_matmul_bf16_f32(const Dispatch &d) { return launch_matmul<WBf16>(d, "matmul_bf16", false, false); }
zhip_result launch_matmul_f16_f32(const Dispatch &d) { return launch_matmul<WF16>(d, "matmul_f16", false, false); }
zhip_result launch_matmul_q8_0_float_f32(const Dispatch &d) { return launch_matmul<WQ8_0>(d, "matmul_q8_0_float", true, true); }

}  // namespace zhip
