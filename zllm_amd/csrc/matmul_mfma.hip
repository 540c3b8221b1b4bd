// Prefill multiplies on the CDNA4 matrix cores: the bf16 rung of matmul_bf16
// and matmul_q8_0_float (same parameter blocks, bindings and grids as
// src/kernels/matmul_half.wgsl and src/kernels/matmul_q8_0_float.wgsl).
//
// out[t][col0 + j] (+)= sum_i bf16(x[t][i]) * bf16(w[j][i]), fp32 accumulate.
// Weight tiles are dequantised into LDS as bf16 (Q8_0: bf16(q * d), one
// rounding of the exact f32 product; BF16 weights are copied), activation
// tiles are narrowed to bf16 as they are staged (exact when the caller's f32
// values are bf16-representable), and v_mfma_f32_16x16x32_bf16 multiplies
// them. This is an approximate rung in the reference's terms
// (src/precision.zig:9): operands carry 8 significant bits.
//
// Tiling: a workgroup of four wave64s computes BM tokens x BN outputs; each
// wave owns a (BM/2) x (BN/2) quadrant as 16x16 MFMA tiles. Tokens are the
// MFMA's M dimension and outputs its N dimension, so a lane's four results
// are four tokens of one output column and sixteen lanes store 64 contiguous
// bytes of a token's row.
#include <hip/hip_runtime.h>

#include "common.h"
#include "decode.cuh"

namespace zhip {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

struct MfmaArgs {
    const float *x;
    const uint8_t *w;
    float *out;
    uint32_t rows, n, k, col0, out_stride, accumulate, k_slice, slice_stride;
    uint32_t row_bytes;
};

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    // Round to nearest even, as the reference narrows (src/ref/matmul.zig:250-255).
    const __bf16 a = (__bf16)lo, b = (__bf16)hi;
    return (uint32_t)__builtin_bit_cast(uint16_t, a) | ((uint32_t)__builtin_bit_cast(uint16_t, b) << 16);
}

// Stages 32 weights of one row as bf16: 64 bytes into LDS.
struct StageBf16 {
    __device__ static void stage(const uint8_t *row, uint32_t, uint32_t kpos, uint4 *dst) {
        const uint4 *src = reinterpret_cast<const uint4 *>(row + 2u * kpos);
#pragma unroll
        for (int i = 0; i < 4; i++) dst[i] = src[i];
    }
};

struct StageQ8_0 {
    __device__ static void stage(const uint8_t *row, uint32_t k, uint32_t kpos, uint4 *dst) {
        const uint4 *src = reinterpret_cast<const uint4 *>(row + kpos);
        const float d = half_bits_to_float(*reinterpret_cast<const uint16_t *>(row + k + 2u * (kpos / 32u)));
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const uint4 q = src[h];
            const int32_t words[4] = {(int32_t)q.x, (int32_t)q.y, (int32_t)q.z, (int32_t)q.w};
            uint32_t o[8];
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const float f0 = (float)((words[e] << 24) >> 24) * d;
                const float f1 = (float)((words[e] << 16) >> 24) * d;
                const float f2 = (float)((words[e] << 8) >> 24) * d;
                const float f3 = (float)(words[e] >> 24) * d;
                o[2 * e] = pack_bf16(f0, f1);
                o[2 * e + 1] = pack_bf16(f2, f3);
            }
            dst[2 * h] = make_uint4(o[0], o[1], o[2], o[3]);
            dst[2 * h + 1] = make_uint4(o[4], o[5], o[6], o[7]);
        }
    }
};

constexpr int BM = 128, BN = 128, BK = 64;
constexpr int LDS_ROW = BK * 2 + 16;  // bytes: 64 bf16 and 16 bytes of padding against bank conflicts

template <class S>
__global__ __launch_bounds__(256) void matmul_mfma_kernel(MfmaArgs a) {
    __shared__ __attribute__((aligned(16))) uint8_t xs[BM * LDS_ROW];
    __shared__ __attribute__((aligned(16))) uint8_t ws[BN * LDS_ROW];
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t j0 = blockIdx.x * BN, t0 = blockIdx.y * BM, z = blockIdx.z;
    const uint32_t kb = z * a.k_slice, ke = min(a.k, kb + a.k_slice);
    const uint32_t wm = (wave >> 1) * (BM / 2), wn = (wave & 1u) * (BN / 2);
    const uint32_t lrow = lane & 15u, lk = (lane >> 4) * 16u;  // byte offset of the lane's 8 k values

    f32x4 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    // Staging assignment: row = tid / 2, 32-wide half = tid % 2.
    const uint32_t srow = tid >> 1, shalf = tid & 1u;
    for (uint32_t k0 = kb; k0 < ke; k0 += BK) {
        const uint32_t kpos = k0 + 32u * shalf;
        {
            uint4 *dst = reinterpret_cast<uint4 *>(xs + srow * LDS_ROW + 64u * shalf);
            const uint32_t t = t0 + srow;
            if (t < a.rows && kpos < ke) {
                const float4 *src = reinterpret_cast<const float4 *>(a.x + (size_t)t * a.k + kpos);
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const float4 v0 = src[2 * i], v1 = src[2 * i + 1];
                    dst[i] = make_uint4(pack_bf16(v0.x, v0.y), pack_bf16(v0.z, v0.w), pack_bf16(v1.x, v1.y), pack_bf16(v1.z, v1.w));
                }
            } else {
#pragma unroll
                for (int i = 0; i < 4; i++) dst[i] = make_uint4(0, 0, 0, 0);
            }
        }
        {
            uint4 *dst = reinterpret_cast<uint4 *>(ws + srow * LDS_ROW + 64u * shalf);
            const uint32_t j = j0 + srow;
            if (j < a.n && kpos < ke) {
                S::stage(a.w + (size_t)j * a.row_bytes, a.k, kpos, dst);
            } else {
#pragma unroll
                for (int i = 0; i < 4; i++) dst[i] = make_uint4(0, 0, 0, 0);
            }
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < BK / 32; kk++) {
            bf16x8 af[4], bfr[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                af[i] = *reinterpret_cast<const bf16x8 *>(xs + (wm + 16 * i + lrow) * LDS_ROW + 64 * kk + lk);
                bfr[i] = *reinterpret_cast<const bf16x8 *>(ws + (wn + 16 * i + lrow) * LDS_ROW + 64 * kk + lk);
            }
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }

    // D[token][output]: the lane holds output column lane % 16 and token rows
    // 4 * (lane / 16) .. + 3 of each 16 x 16 tile.
#pragma unroll
    for (int i = 0; i < 4; i++) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t col = j0 + wn + 16 * j + lrow;
            if (col >= a.n) continue;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const uint32_t t = t0 + wm + 16 * i + 4 * (lane >> 4) + r;
                if (t >= a.rows) continue;
                const size_t o = (size_t)z * a.slice_stride + (size_t)t * a.out_stride + a.col0 + col;
                const float v = acc[i][j][r];
                a.out[o] = a.accumulate ? a.out[o] + v : v;
            }
        }
    }
}

template <class S>
static zhip_result launch_mfma(const Dispatch &d, const char *name, bool sliced, uint32_t row_bytes) {
    const MatmulParams &p = *reinterpret_cast<const MatmulParams *>(d.params);
    MfmaArgs a{};
    const uint64_t cover_n = (uint64_t)d.grid[0] * 64u, cover_t = (uint64_t)d.grid[1] * 16u;
    a.n = (uint32_t)(cover_n < p.n ? cover_n : p.n);
    a.rows = (uint32_t)(cover_t < p.rows ? cover_t : p.rows);
    a.k = p.k; a.col0 = p.col0; a.out_stride = p.out_stride; a.accumulate = p.accumulate;
    a.k_slice = sliced ? p.k_slice : p.k;
    a.slice_stride = sliced ? p.slice_stride : 0;
    a.row_bytes = row_bytes;
    a.x = reinterpret_cast<const float *>(d.bind[1].ptr);
    a.w = d.bind[2].ptr;
    a.out = reinterpret_cast<float *>(d.bind[3].ptr);
    const dim3 grid((a.n + BN - 1) / BN, (a.rows + BM - 1) / BM, sliced ? d.grid[2] : 1);
    hipLaunchKernelGGL((matmul_mfma_kernel<S>), grid, dim3(256), 0, d.stream, a);
    return check_launch(d, name);
}

// Validation shared with the f32 rung (matmul_f32.hip).
zhip_result validate_matmul(const Dispatch &d, const char *name, bool sliced, bool q8_0, bool *empty);

zhip_result launch_matmul_bf16_mfma(const Dispatch &d) {
    bool empty = false;
    if (zhip_result r = validate_matmul(d, "matmul_bf16", false, false, &empty)) return r;
    if (empty) return ZHIP_OK;
    const MatmulParams &p = *reinterpret_cast<const MatmulParams *>(d.params);
    return launch_mfma<StageBf16>(d, "matmul_bf16", false, 2u * p.k);
}

zhip_result launch_matmul_q8_0_float_mfma(const Dispatch &d) {
    bool empty = false;
    if (zhip_result r = validate_matmul(d, "matmul_q8_0_float", true, true, &empty)) return r;
    if (empty) return ZHIP_OK;
    const MatmulParams &p = *reinterpret_cast<const MatmulParams *>(d.params);
    return launch_mfma<StageQ8_0>(d, "matmul_q8_0_float", true, (p.k + p.k / 16u + 15u) & ~15u);
}

}  // namespace zhip
