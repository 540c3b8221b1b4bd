// Shared by the decode multiplies: their arguments and the input staging.
#pragma once

#include <hip/hip_runtime.h>

#include "common.h"

namespace zhip {

struct MvArgs {
    const float *x;
    const uint8_t *w;
    float *out;
    const float *norm_w;
    uint32_t n, k, col0, out_stride;
    float eps;
    uint32_t flags, half;
    uint32_t xr;         // floats between tokens' inputs
    uint32_t m;          // tokens
    uint32_t rows;       // outputs covered by the logical grid
    uint32_t row_bytes;  // bytes between weight rows
    float act_div;       // > 0: inputs staged as silu(x / act_div)
};

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

__device__ __forceinline__ float silu_f(float v) { return v / (1.0f + expf(-v)); }

// Stages token `token`'s k inputs at dst (k / 4 vectors): normalised with the
// RMSNorm prologue and / or activated as silu(x / act_div) as the flags ask
// (src/kernels/matvec_quant.wgsl.hbs:73-89,175-198). Every thread of the
// 256-thread workgroup must call it; `red` is four floats of LDS. Vector i of
// the token lands at dst[place(i)].
template <class Place>
__device__ __forceinline__ void stage_token(const MvArgs &a, uint32_t token, float4 *dst, float *red, Place place) {
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t k4 = a.k / 4u;
    const float4 *xrow = reinterpret_cast<const float4 *>(a.x + (size_t)token * a.xr);
    float scale = 1.0f;
    if (a.flags & FLAG_NORM) {
        float ss = 0.f;
        for (uint32_t i = tid; i < k4; i += 256u) {
            const float4 v = xrow[i];
            ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
        }
        ss = wave_sum(ss);
        __syncthreads();
        if (lane == 0) red[wave] = ss;
        __syncthreads();
        ss = (red[0] + red[1]) + (red[2] + red[3]);
        scale = 1.0f / sqrtf(ss / (float)a.k + a.eps);
    }
    const float4 *nw = reinterpret_cast<const float4 *>(a.norm_w);
    for (uint32_t i = tid; i < k4; i += 256u) {
        float4 v = xrow[i];
        if (a.flags & FLAG_NORM) {
            const float4 g = nw[i];
            v.x = v.x * scale * g.x; v.y = v.y * scale * g.y;
            v.z = v.z * scale * g.z; v.w = v.w * scale * g.w;
        }
        if (a.act_div > 0.f) {
            v.x = silu_f(v.x / a.act_div); v.y = silu_f(v.y / a.act_div);
            v.z = silu_f(v.z / a.act_div); v.w = silu_f(v.w / a.act_div);
        }
        dst[place(i)] = v;
    }
}

__device__ __forceinline__ void stage_token(const MvArgs &a, uint32_t token, float4 *dst, float *red) {
    stage_token(a, token, dst, red, [](uint32_t i) { return i; });
}

// Matrix-core variants over rows of more than 4096 weights: `parts` workgroups share a tile, each
// over 2048 of its columns, and leave their sums in `partial` ([part][gate, up][token of 8][output],
// outputs a.rows apart); this launch adds a tile's parts in the order of their columns and applies
// the SILU_PAIR / ACCUMULATE epilogue (matvec_mfma_resident.hip).
constexpr uint32_t kMatvecMaxParts = 16;  // rows of up to 32768 weights
zhip_result launch_matvec_parts_sum(const Dispatch &d, const char *name, const MvArgs &a, const float *partial, uint32_t parts);
// A step over such rows with the RMSNorm prologue: no workgroup sees a whole row, so a launch of
// its own leaves each token's 1 / sqrt(mean(x^2) + eps) in scales[token] beforehand (the sum of
// squares as stage_token takes it). The workspace's first kPartsScalesBytes hold them.
constexpr uint32_t kPartsScalesBytes = 64;
zhip_result launch_matvec_parts_scales(const Dispatch &d, const char *name, const MvArgs &a, float *scales);

}  // namespace zhip
