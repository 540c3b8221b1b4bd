// quantize_q8: rows of activations rounded to 8-bit blocks for the int8 prefill
// multiply, value for value as llama.cpp's x86 CPU backend rounds them
// (src/kernels/quantize_q8.wgsl, src/ref/matmul.zig:197-247). A wave takes U
// consecutive chunks of 256 values of one row, four values a lane and chunk
// (a chunk is one Q8_K block, or eight Q8_0 blocks of eight lanes each), all
// their loads issued before the first is rounded: a chunk's rounding is a chain
// of dependent operations behind one 16-byte load, and a wave with one load in
// flight spends its time waiting for memory (512 x 14336 values to Q8_K blocks
// took 37 us with a chunk a wave, an HBM read of 29 MB). A workgroup is four
// such waves on neighbouring chunks; with the RMSNorm prologue it first adds the
// row's squares together and then takes all of the row's chunks. The largest magnitude of a
// block is found with row-local DPP steps (and, for Q8_K, four lane reads),
// the first position that holds it with a ballot. Every operation whose rounding
// decides a value is an operation of its own (the library is compiled with
// -ffp-contract=on, which fuses only within one source expression, and with
// hipcc's correctly rounded f32 division and square root), so the compiler can
// neither fuse the multiply into the rounding addition nor approximate a division.
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

// max over lane pairs, quads, groups of eight and rows of sixteen: every lane of the group ends
// with the group's maximum.
template <int CTRL>
__device__ __forceinline__ float max_with(float v) {
    return fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false)));
}
__device__ __forceinline__ float max_of_eight(float v) {
    v = max_with<0xB1>(v);   // quad_perm [1, 0, 3, 2]
    v = max_with<0x4E>(v);   // quad_perm [2, 3, 0, 1]
    return max_with<0x141>(v);  // row_half_mirror: the other quad of the eight
}
__device__ __forceinline__ float max_of_wave(float v) {
    v = max_with<0x140>(max_of_eight(v));  // row_mirror: the other eight of the row
    const float a = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0)), b = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
    const float c = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32)), d = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
    return fmaxf(fmaxf(a, b), fmaxf(c, d));
}

template <int U>
__global__ __launch_bounds__(256) void quantize_q8_kernel(QuantizeQ8Params p, const float *x, uint32_t *qx, float *dx, const float *nw) {
    __shared__ double squares[4];
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6, row = blockIdx.y;
    const float *xr = x + (size_t)row * p.k;
    float scale = 1.0f;
    if (p.mode == 1u) {
        // RMSNorm as ggml computes it (src/ref/ops.zig:25-41): f32 squares
        // summed and divided in f64, an f32 mean, add, sqrt and reciprocal,
        // then x * scale, then * w. (Four loads at a time: one after the other, a long
        // row's pass over itself is a chain of trips to L2.)
        double ss = 0.0;
        for (uint32_t i0 = 4u * threadIdx.x; i0 < p.k; i0 += 4096u) {
            qf32x4 r[4];
#pragma unroll
            for (uint32_t j = 0; j < 4; j++) r[j] = i0 + 1024u * j < p.k ? *reinterpret_cast<const qf32x4 *>(xr + i0 + 1024u * j) : qf32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (uint32_t j = 0; j < 4; j++) {
                if (i0 + 1024u * j >= p.k) break;
#pragma unroll
                for (int e = 0; e < 4; e++) ss += (double)__fmul_rn(r[j][e], r[j][e]);
            }
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
        if (lane == 0) squares[wave] = ss;
        __syncthreads();
        ss = (squares[0] + squares[1]) + (squares[2] + squares[3]);
        const float mean = (float)(ss / (double)p.k);
        // (sqrtf is the correctly rounded square root under hipcc's default options; the
        // __fsqrt_rn intrinsic is the hardware's approximate one here and gave some rows a
        // scale one unit in the last place away from ggml's)
        scale = __fdiv_rn(1.0f, sqrtf(__fadd_rn(mean, p.eps)));
    }

    // The workgroup's spans of 4 U chunks: one (blockIdx.x) without the prologue; with it, all
    // of the row's, so that the row's squares are added once.
    for (uint32_t span = blockIdx.x; span * (1024u * U) < p.k; span += gridDim.x) {
        const uint32_t first = ((span * 4u + wave) * U) * 256u + 4u * lane;  // the lane's first position of the wave's first chunk
        qf32x4 v[U];
        bool live[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            live[u] = first + 256u * u < p.k;
            v[u] = qf32x4{0.f, 0.f, 0.f, 0.f};
        }
        if (p.mode == 2u) {
            // silu(gate) * up over a row of gate | up (src/kernels/silu_mul.wgsl).
            qf32x4 gate[U], up[U];
#pragma unroll
            for (int u = 0; u < U; u++) {
                const float *g = x + (size_t)row * 2u * p.k + (live[u] ? first + 256u * u : 0u);
                gate[u] = *reinterpret_cast<const qf32x4 *>(g);
                up[u] = *reinterpret_cast<const qf32x4 *>(g + p.k);
            }
#pragma unroll
            for (int u = 0; u < U; u++)
#pragma unroll
                for (int i = 0; i < 4; i++) v[u][i] = live[u] ? gate[u][i] / (1.0f + expf(-gate[u][i])) * up[u][i] : 0.f;
        } else {
            qf32x4 w[U];
#pragma unroll
            for (int u = 0; u < U; u++) {
                const qf32x4 got = *reinterpret_cast<const qf32x4 *>(xr + (live[u] ? first + 256u * u : 0u));
                if (live[u]) v[u] = got;
                if (p.mode == 1u) w[u] = *reinterpret_cast<const qf32x4 *>(nw + (live[u] ? first + 256u * u : 0u));
            }
            if (p.mode == 1u) {
#pragma unroll
                for (int u = 0; u < U; u++)
#pragma unroll
                    for (int e = 0; e < 4; e++) v[u][e] = live[u] ? __fmul_rn(__fmul_rn(v[u][e], scale), w[u][e]) : 0.f;
            }
        }

#pragma unroll
        for (int u = 0; u < U; u++) {
            // The lane's first largest magnitude: a strict > scan from the left.
            float mag = fabsf(v[u][0]), value = v[u][0];
#pragma unroll
            for (int e = 1; e < 4; e++) {
                const float a = fabsf(v[u][e]);
                if (a > mag) {
                    mag = a;
                    value = v[u][e];
                }
            }
            int q[4] = {0, 0, 0, 0};
            float d = 0.f;
            if (p.block == 256u) {
                // Q8_K: the value itself (with its sign) at the first position of the largest
                // magnitude: the lowest lane that holds it.
                const float amax = max_of_wave(mag);
                const uint64_t holders = __ballot(mag == amax);
                const float lead = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(value), (int)__ffsll((unsigned long long)holders) - 1));
                if (amax != 0.f) {
                    const float iscale = __fdiv_rn(-127.0f, lead);
                    d = __fdiv_rn(1.0f, iscale);
#pragma unroll
                    for (int e = 0; e < 4; e++) q[e] = min(127, nearest_int(__fmul_rn(iscale, v[u][e])));
                }
            } else {
                const float amax = max_of_eight(mag);
                if (amax != 0.f) {
                    const float d32 = __fdiv_rn(amax, 127.0f);
                    const float id = __fdiv_rn(127.0f, amax);
                    d = (float)(_Float16)d32;
#pragma unroll
                    for (int e = 0; e < 4; e++) q[e] = nearest_int(__fmul_rn(v[u][e], id));
                }
            }
            if (!live[u]) continue;
            const size_t base = (size_t)row * p.k + first + 256u * u;
            qx[base / 4u] = ((uint32_t)q[0] & 0xffu) | (((uint32_t)q[1] & 0xffu) << 8) | (((uint32_t)q[2] & 0xffu) << 16) | (((uint32_t)q[3] & 0xffu) << 24);
            if ((4u * lane) % p.block == 0u) dx[base / p.block] = d;
        }
    }
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
    const float *x = reinterpret_cast<const float *>(d.bind[1].ptr), *nw = reinterpret_cast<const float *>(d.bind[4].ptr);
    uint32_t *qx = reinterpret_cast<uint32_t *>(d.bind[2].ptr);
    float *dx = reinterpret_cast<float *>(d.bind[3].ptr);
    // Chunks a wave takes at once: four or two where that still leaves two workgroups a CU
    // (few rows are faster as many short waves: 64 x 4096, 2.5 against 3.4 us).
    const uint32_t n_chunks = d.grid[0];
    // (with the RMSNorm prologue a workgroup takes its whole row)
    const bool whole = p.mode == 1u;
    const uint64_t enough = 2u * (uint64_t)d.dev->compute_units;
    const uint32_t at_once = whole || rows * ((n_chunks + 15u) / 16u) >= enough ? 4u : rows * ((n_chunks + 7u) / 8u) >= enough ? 2u : 1u;
    if (at_once == 4u && n_chunks > 8u) hipLaunchKernelGGL(quantize_q8_kernel<4>, dim3(whole ? 1u : (n_chunks + 15u) / 16u, d.grid[1]), dim3(256), 0, d.stream, p, x, qx, dx, nw);
    else if (at_once >= 2u && n_chunks > 4u) hipLaunchKernelGGL(quantize_q8_kernel<2>, dim3(whole ? 1u : (n_chunks + 7u) / 8u, d.grid[1]), dim3(256), 0, d.stream, p, x, qx, dx, nw);
    else hipLaunchKernelGGL(quantize_q8_kernel<1>, dim3(whole ? 1u : (n_chunks + 3u) / 4u, d.grid[1]), dim3(256), 0, d.stream, p, x, qx, dx, nw);
    return check_launch(d, "quantize_q8");
}

}  // namespace zhip
