// quantize_q8: rows of activations rounded to 8-bit blocks for the int8 prefill
// multiply, value for value as llama.cpp's x86 CPU backend rounds them
// (src/kernels/quantize_q8.wgsl, src/ref/matmul.zig:197-247). A wave takes
// 256 values of one row, four per lane: one Q8_K block, or eight Q8_0 blocks of
// eight lanes each; a workgroup is four independent waves. Every operation whose rounding decides
// a value is spelled as a correctly rounded intrinsic, so the compiler can
// neither fuse the multiply into the rounding addition nor approximate a
// division.
#include <hip/hip_runtime.h>

#include "common.h"

namespace zhip {

struct QuantizeQ8Params {  // params.QuantizeQ8 (src/kernels/kernels.zig:495-501)
    uint32_t k, block, mode;
    float eps;
};
static_assert(sizeof(QuantizeQ8Params) == 16, "params.QuantizeQ8 is 16 bytes");

typedef float qf32x4 __attribute__((ext_vector_type(4)));

// ggml's nearest_int: adding 1.5 * 2^23 rounds the f32 to an integer, ties to even.
__device__ __forceinline__ int nearest_int(float y) {
    return __float_as_int(__fadd_rn(y, 12582912.0f)) - 0x4b400000;
}

struct Lead {
    float mag;      // |value|
    float value;    // the value itself
    uint32_t at;    // its position in the 256
};

// The first of the largest: a strict > scan from the left, ties to the lower position.
__device__ __forceinline__ Lead better(const Lead &a, const Lead &b) {
    return (b.mag > a.mag || (b.mag == a.mag && b.at < a.at)) ? b : a;
}

__global__ __launch_bounds__(256) void quantize_q8_kernel(QuantizeQ8Params p, const float *x, uint32_t *qx, float *dx, const float *nw) {
    const uint32_t lane = threadIdx.x & 63u, row = blockIdx.y;
    const uint32_t at = (blockIdx.x * 4u + (threadIdx.x >> 6)) * 256u + 4u * lane;  // first of this lane's four positions
    if (at - 4u * lane >= p.k) return;  // a whole wave past the row's end
    const bool live = at < p.k;
    qf32x4 v = {0.f, 0.f, 0.f, 0.f};
    if (p.mode == 2u) {
        // silu(gate) * up over a row of gate | up (src/kernels/silu_mul.wgsl).
        if (live) {
            const float *g = x + (size_t)row * 2u * p.k + at;
            const qf32x4 gate = *reinterpret_cast<const qf32x4 *>(g);
            const qf32x4 up = *reinterpret_cast<const qf32x4 *>(g + p.k);
#pragma unroll
            for (int i = 0; i < 4; i++) v[i] = gate[i] / (1.0f + expf(-gate[i])) * up[i];
        }
    } else {
        const float *xr = x + (size_t)row * p.k;
        if (live) v = *reinterpret_cast<const qf32x4 *>(xr + at);
        if (p.mode == 1u) {
            // RMSNorm as ggml computes it (src/ref/ops.zig:25-41): f32 squares
            // summed and divided in f64, an f32 mean, add, sqrt and reciprocal,
            // then x * scale, then * w.
            double ss = 0.0;
            for (uint32_t i = 4u * lane; i < p.k; i += 256u) {
                const qf32x4 r = *reinterpret_cast<const qf32x4 *>(xr + i);
#pragma unroll
                for (int e = 0; e < 4; e++) ss += (double)__fmul_rn(r[e], r[e]);
            }
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
            const float mean = (float)(ss / (double)p.k);
            const float scale = __fdiv_rn(1.0f, __fsqrt_rn(__fadd_rn(mean, p.eps)));
            if (live) {
                const qf32x4 w = *reinterpret_cast<const qf32x4 *>(nw + at);
#pragma unroll
                for (int e = 0; e < 4; e++) v[e] = __fmul_rn(__fmul_rn(v[e], scale), w[e]);
            }
        }
    }

    Lead best{fabsf(v[0]), v[0], 4u * lane};
#pragma unroll
    for (uint32_t e = 1; e < 4; e++) {
        const float a = fabsf(v[e]);
        if (a > best.mag) best = Lead{a, v[e], 4u * lane + e};
    }
    // Across the block's lanes: 8 for Q8_0, all 64 for Q8_K.
    const int span = p.block == 256u ? 64 : 8;
    for (int off = 1; off < span; off <<= 1) {
        Lead o;
        o.mag = __shfl_xor(best.mag, off, 64);
        o.value = __shfl_xor(best.value, off, 64);
        o.at = __shfl_xor(best.at, off, 64);
        best = better(best, o);
    }

    int q[4] = {0, 0, 0, 0};
    float d = 0.f;
    if (best.mag != 0.f) {
        if (p.block == 256u) {
            const float iscale = __fdiv_rn(-127.0f, best.value);
            d = __fdiv_rn(1.0f, iscale);
#pragma unroll
            for (int e = 0; e < 4; e++) q[e] = min(127, nearest_int(__fmul_rn(iscale, v[e])));
        } else {
            const float d32 = __fdiv_rn(best.mag, 127.0f);
            const float id = __fdiv_rn(127.0f, best.mag);
            d = (float)(_Float16)d32;
#pragma unroll
            for (int e = 0; e < 4; e++) q[e] = nearest_int(__fmul_rn(v[e], id));
        }
    }
    if (!live) return;
    const size_t base = (size_t)row * p.k + at;
    qx[base / 4u] = ((uint32_t)q[0] & 0xffu) | (((uint32_t)q[1] & 0xffu) << 8) | (((uint32_t)q[2] & 0xffu) << 16) | (((uint32_t)q[3] & 0xffu) << 24);
    if ((4u * lane) % p.block == 0u) dx[base / p.block] = d;
}

zhip_result launch_quantize_q8(const Dispatch &d) {
    if (d.params_size < sizeof(QuantizeQ8Params)) return fail(d, ZHIP_E_BAD_COMMAND, "quantize_q8: params block too small");
    const QuantizeQ8Params &p = *reinterpret_cast<const QuantizeQ8Params *>(d.params);
    for (int b = 1; b <= 4; b++)
        if (!d.bind[b].bound) return fail(d, ZHIP_E_BAD_COMMAND, "quantize_q8: binding %d is not bound", b);
    if (d.grid[0] == 0 || d.grid[1] == 0 || d.grid[2] == 0) return ZHIP_OK;
    if (d.grid[2] != 1) return fail(d, ZHIP_E_BAD_COMMAND, "quantize_q8: grid z must be 1");
    if (p.block != 32u && p.block != 256u) return fail(d, ZHIP_E_BAD_COMMAND, "quantize_q8: block = %u (32 or 256)", p.block);
    if (p.k == 0 || p.k % p.block != 0) return fail(d, ZHIP_E_BAD_COMMAND, "quantize_q8: k = %u is not a multiple of the block %u", p.k, p.block);
    if (p.mode > 2u) return fail(d, ZHIP_E_BAD_COMMAND, "quantize_q8: mode = %u", p.mode);
    const uint64_t chunks = (p.k + 255u) / 256u;
    if (d.grid[0] != chunks) return fail(d, ZHIP_E_BAD_COMMAND, "quantize_q8: grid x = %u, k = %u needs %llu", d.grid[0], p.k, (unsigned long long)chunks);
    if (d.grid[1] > 65535u) return fail(d, ZHIP_E_BAD_COMMAND, "quantize_q8: more than 65535 rows in one dispatch");
    const uint64_t rows = d.grid[1];
    const uint64_t x_need = rows * p.k * (p.mode == 2u ? 8u : 4u);
    const uint64_t q_need = rows * p.k, d_need = rows * (p.k / p.block) * 4u;
    if (x_need > d.bind[1].size || q_need > d.bind[2].size || d_need > d.bind[3].size || (p.mode == 1u && (uint64_t)p.k * 4u > d.bind[4].size))
        return fail(d, ZHIP_E_BAD_COMMAND, "quantize_q8: bound ranges too small");
    if (((uintptr_t)d.bind[1].ptr | (p.mode == 1u ? (uintptr_t)d.bind[4].ptr : 0)) & 15u) return fail(d, ZHIP_E_BAD_COMMAND, "quantize_q8: x and norm weights must be 16-byte aligned");
    if (((uintptr_t)d.bind[2].ptr | (uintptr_t)d.bind[3].ptr) & 3u) return fail(d, ZHIP_E_BAD_COMMAND, "quantize_q8: outputs must be 4-byte aligned");
    hipLaunchKernelGGL(quantize_q8_kernel, dim3((d.grid[0] + 3u) / 4u, d.grid[1]), dim3(256), 0, d.stream, p,
        reinterpret_cast<const float *>(d.bind[1].ptr), reinterpret_cast<uint32_t *>(d.bind[2].ptr),
        reinterpret_cast<float *>(d.bind[3].ptr), reinterpret_cast<const float *>(d.bind[4].ptr));
    return check_launch(d, "quantize_q8");
}

}  // namespace zhip
