// Decode multiplies: out[t][col0 + j] (+)= sum_i X(t, i) * w[j][i] for Q8_0,
// Q3_K, Q4_K, Q5_K, Q6_K and BF16 weights, with the RMSNorm / activation prologues and the
// accumulate / SiLU-pair epilogues of the reference's matvec kernels
// (src/kernels/matvec_quant.wgsl.hbs:20-31, src/kernels/matvec_half.wgsl:14-19).
//
// General kernel. A workgroup is four wave64s. The step's inputs are staged
// once per workgroup in LDS (normalised / activated as they are staged), then
// every wave walks row groups in a grid-stride loop: a group is two weight
// rows (two outputs, or the gate and up rows of one output with SILU_PAIR).
// A row's packed weights are split into 16-byte tasks across the 64 lanes, so
// each load instruction of a wave reads consecutive 16-byte vectors; a lane
// decodes its task's weights once and multiplies them with every token's
// inputs; the lanes' partial sums reduce in a fixed butterfly. A token's sums
// are therefore the same bit for bit whether it runs alone or with others
// (the reference's split invariant, matvec_quant.wgsl.hbs:14-18).
#include <hip/hip_runtime.h>

#include <type_traits>

#include "common.h"
#include "decode.h"
#include "matvec_common.h"

namespace zhip {

// The 16-bit formats' tasks are eight weights against two neighbouring input vectors. Lanes
// reading vector 2 task (then 2 task + 1) of a token would touch every other 16 bytes of LDS,
// two lanes to a bank; their inputs are therefore staged with the even vectors first and the
// odd ones behind them, so that each read covers consecutive vectors.
template <class D> constexpr bool kSplitInputs = std::is_same<D, DecBF16>::value || std::is_same<D, DecF16>::value;

// DEPTH: positions of the 16-bit formats' walk whose loads are in flight behind the one multiplied.
template <class D, int MT, int DEPTH>
__global__ __launch_bounds__(256) void matvec_kernel(MvArgs a) {
    extern __shared__ float4 xs4[];
    float *xs = reinterpret_cast<float *>(xs4);
    __shared__ float red[16];
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t gwave = blockIdx.x * 4u + wave, nwaves = gridDim.x * 4u;
    const bool pair = (a.flags & FLAG_SILU_PAIR) != 0;
    const uint32_t k4 = a.k / 4u;
    const uint32_t tasks = a.k / D::E;
    // Outputs per group: two rows, or one gate/up pair.
    const uint32_t per_group = pair ? 1u : 2u;
    const uint32_t groups = (a.rows + per_group - 1u) / per_group;

    for (uint32_t t0 = 0; t0 < a.m; t0 += MT) {
        const uint32_t mt = min((uint32_t)MT, a.m - t0);
        __syncthreads();
        if constexpr (kSplitInputs<D>) {
            // The 16-bit formats. With rows of up to 4096 weights the pass's inputs are loaded
            // first (up to four vectors a thread and token, four tokens at a time), then the
            // wave's first weights, and only then are the inputs staged: the one trip to memory
            // serves both, where staging token after token and then starting on the weights
            // took one for every token and one more (loads complete in order within a wave).
            // A wave walks (group, 64-task slice) positions with the loads of the next DEPTH
            // positions in flight while it multiplies the current one (past its last position
            // the loads are clamped to a valid one and their data unused).
            constexpr int TG = MT < 4 ? MT : 4;
            // (a lone token on short rows measured no faster that way: 3072 x 1024, 4.2 against 4.5 us)
            const bool early = a.k <= 4096u && (MT > 1 || DEPTH > 1);
            const uint32_t iters = (tasks + 63u) / 64u;
            auto place = [k4](uint32_t i) { return (i & 1u) * (k4 / 2u) + (i >> 1); };
            float4 xv[TG][4], gv[4];
            auto load_tokens = [&](uint32_t first) __attribute__((always_inline)) {
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const uint32_t i = tid + 256u * j;
#pragma unroll
                    for (int t = 0; t < TG; t++) {
                        const float4 *xrow = reinterpret_cast<const float4 *>(a.x + (size_t)(t0 + (first + t < mt ? first + t : 0u)) * a.xr);
                        xv[t][j] = i < k4 ? xrow[i] : make_float4(0.f, 0.f, 0.f, 0.f);
                    }
                }
            };
            if (early) {
                load_tokens(0);
                if (a.flags & FLAG_NORM) {
                    const float4 *nw = reinterpret_cast<const float4 *>(a.norm_w);
#pragma unroll
                    for (int j = 0; j < 4; j++) gv[j] = tid + 256u * j < k4 ? nw[tid + 256u * j] : make_float4(0.f, 0.f, 0.f, 0.f);
                }
            }
            auto rows_of = [&](uint32_t g, uint32_t &j0, uint32_t &r1, bool &has1) {
                j0 = pair ? g : 2u * g;
                r1 = pair ? a.half + g : j0 + 1u;
                has1 = pair || r1 < a.rows;
            };
            auto load_at = [&](uint32_t g, uint32_t it, uint4 &q0, uint4 &q1) {
                uint32_t j0, r1;
                bool has1;
                rows_of(g < groups ? g : groups - 1u, j0, r1, has1);
                const uint32_t task = lane + 64u * it, tk = task < tasks ? task : 0u;
                q0 = *reinterpret_cast<const uint4 *>(a.w + (size_t)j0 * a.row_bytes + 16u * tk);
                q1 = *reinterpret_cast<const uint4 *>(a.w + (size_t)(has1 ? r1 : j0) * a.row_bytes + 16u * tk);
            };
            auto advance = [&](uint32_t &g, uint32_t &it) {
                if (++it == iters) {
                    it = 0;
                    g += nwaves;
                }
            };
            uint4 b0[DEPTH], b1[DEPTH];
            uint32_t lg = gwave, lit = 0;
#pragma unroll
            for (int s = 0; s < DEPTH; s++) {
                load_at(lg, lit, b0[s], b1[s]);
                advance(lg, lit);
            }
            if (early) {
                // The arithmetic of stage_token on the vectors already loaded, in the same
                // order, the tokens' sums of squares meeting in LDS together.
#pragma unroll
                for (int first = 0; first < MT; first += TG) {
                    if (first > 0) load_tokens(first);
                    float scale[TG];
#pragma unroll
                    for (int t = 0; t < TG; t++) scale[t] = 1.0f;
                    if (a.flags & FLAG_NORM) {
                        float ss[TG];
#pragma unroll
                        for (int t = 0; t < TG; t++) {
                            ss[t] = 0.f;
#pragma unroll
                            for (int j = 0; j < 4; j++)
                                if (tid + 256u * j < k4) ss[t] += xv[t][j].x * xv[t][j].x + xv[t][j].y * xv[t][j].y + xv[t][j].z * xv[t][j].z + xv[t][j].w * xv[t][j].w;
                            ss[t] = wave_sum(ss[t]);
                        }
                        __syncthreads();
                        if (lane == 0) {
#pragma unroll
                            for (int t = 0; t < TG; t++) red[4 * t + wave] = ss[t];
                        }
                        __syncthreads();
#pragma unroll
                        for (int t = 0; t < TG; t++) {
                            const float total = (red[4 * t] + red[4 * t + 1]) + (red[4 * t + 2] + red[4 * t + 3]);
                            scale[t] = 1.0f / sqrtf(total / (float)a.k + a.eps);
                        }
                    }
#pragma unroll
                    for (int t = 0; t < TG; t++) {
                        float4 *dst = xs4 + (size_t)(first + t) * k4;
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            const uint32_t i = tid + 256u * j;
                            if (i >= k4) continue;
                            float4 v = xv[t][j];
                            if (a.flags & FLAG_NORM) {
                                v.x = v.x * scale[t] * gv[j].x; v.y = v.y * scale[t] * gv[j].y;
                                v.z = v.z * scale[t] * gv[j].z; v.w = v.w * scale[t] * gv[j].w;
                            }
                            if (a.act_div > 0.f) {
                                v.x = silu_f(v.x / a.act_div); v.y = silu_f(v.y / a.act_div);
                                v.z = silu_f(v.z / a.act_div); v.w = silu_f(v.w / a.act_div);
                            }
                            if ((uint32_t)(first + t) >= mt) v = make_float4(0.f, 0.f, 0.f, 0.f);  // (a pass of fewer tokens than it has room for)
                            dst[place(i)] = v;
                        }
                    }
                }
            } else {
                for (uint32_t t = 0; t < (uint32_t)MT; t++) {
                    float4 *dst = xs4 + (size_t)t * k4;
                    if (t >= mt) {
                        for (uint32_t i = tid; i < k4; i += 256u) dst[i] = make_float4(0.f, 0.f, 0.f, 0.f);
                        continue;
                    }
                    stage_token(a, t0 + t, dst, red, place);
                }
            }
            __syncthreads();

            float acc0[MT], acc1[MT];
#pragma unroll
            for (int t = 0; t < MT; t++) acc0[t] = acc1[t] = 0.f;
            uint32_t g = gwave, it = 0;
            while (g < groups) {
#pragma unroll
                for (int s = 0; s < DEPTH; s++) {
                    if (g >= groups) break;
                    const uint4 c0 = b0[s], c1 = b1[s];
                    load_at(lg, lit, b0[s], b1[s]);
                    advance(lg, lit);
                    const uint32_t task = lane + 64u * it;
                    if (task < tasks) {
                        float w0[D::E], w1[D::E];
                        D::expand(c0, w0);
                        D::expand(c1, w1);
#pragma unroll
                        for (int t = 0; t < MT; t++) {
                            const float *xt = xs + (size_t)t * a.k;
                            float s0 = 0.f, s1 = 0.f;
#pragma unroll
                            for (int h = 0; h < 2; h++) {
                                const float4 v = *reinterpret_cast<const float4 *>(xt + 4u * ((uint32_t)h * (k4 / 2u) + task));
                                const int b = 4 * h;
                                s0 = fmaf(w0[b + 0], v.x, s0); s1 = fmaf(w1[b + 0], v.x, s1);
                                s0 = fmaf(w0[b + 1], v.y, s0); s1 = fmaf(w1[b + 1], v.y, s1);
                                s0 = fmaf(w0[b + 2], v.z, s0); s1 = fmaf(w1[b + 2], v.z, s1);
                                s0 = fmaf(w0[b + 3], v.w, s0); s1 = fmaf(w1[b + 3], v.w, s1);
                            }
                            acc0[t] += s0;
                            acc1[t] += s1;
                        }
                    }
                    if (it + 1u == iters) {
                        uint32_t j0, r1;
                        bool has1;
                        rows_of(g, j0, r1, has1);
#pragma unroll
                        for (int t = 0; t < MT; t++) {
                            acc0[t] = wave_sum(acc0[t]);
                            acc1[t] = wave_sum(acc1[t]);
                        }
                        if (lane == 0) {
                            for (uint32_t t = 0; t < mt; t++) {
                                const size_t o = (size_t)(t0 + t) * a.out_stride + a.col0 + j0;
                                if (pair) {
                                    float v = silu_f(acc0[t]) * acc1[t];
                                    if (a.flags & FLAG_ACCUMULATE) v += a.out[o];
                                    a.out[o] = v;
                                } else {
                                    float v = acc0[t];
                                    if (a.flags & FLAG_ACCUMULATE) v += a.out[o];
                                    a.out[o] = v;
                                    if (has1) {
                                        float u = acc1[t];
                                        if (a.flags & FLAG_ACCUMULATE) u += a.out[o + 1];
                                        a.out[o + 1] = u;
                                    }
                                }
                            }
                        }
#pragma unroll
                        for (int t = 0; t < MT; t++) acc0[t] = acc1[t] = 0.f;
                    }
                    advance(g, it);
                }
            }
            continue;
        }
        for (uint32_t t = 0; t < (uint32_t)MT; t++) {
            float4 *dst = xs4 + (size_t)t * k4;
            if (t >= mt) {
                for (uint32_t i = tid; i < k4; i += 256u) dst[i] = make_float4(0.f, 0.f, 0.f, 0.f);
                continue;
            }
            stage_token(a, t0 + t, dst, red);
        }
        __syncthreads();
        for (uint32_t g = gwave; g < groups; g += nwaves) {
            // The group's two weight rows and whether each exists.
            const uint32_t j0 = pair ? g : 2u * g;
            const uint32_t r1 = pair ? a.half + g : j0 + 1u;
            const bool has1 = pair || r1 < a.rows;
            const uint8_t *row0 = a.w + (size_t)j0 * a.row_bytes;
            const uint8_t *row1 = a.w + (size_t)(has1 ? r1 : j0) * a.row_bytes;
            float acc0[MT], acc1[MT];
#pragma unroll
            for (int t = 0; t < MT; t++) acc0[t] = acc1[t] = 0.f;

            for (uint32_t task = lane; task < tasks; task += 64u) {
                float w0[D::E], w1[D::E];
                D::decode(row0, a.k, task, w0);
                D::decode(row1, a.k, task, w1);
#pragma unroll
                for (int t = 0; t < MT; t++) {
                    const float *xt = xs + (size_t)t * a.k;
                    float s0 = 0.f, s1 = 0.f;
#pragma unroll
                    for (int h = 0; h < D::RUNS; h++) {
                        const float4 *xv = reinterpret_cast<const float4 *>(xt + D::xoff(task, h));
#pragma unroll
                        for (int e = 0; e < D::E / (4 * D::RUNS); e++) {
                            const float4 v = xv[e];
                            const int b = h * (D::E / D::RUNS) + 4 * e;
                            s0 = fmaf(w0[b + 0], v.x, s0); s1 = fmaf(w1[b + 0], v.x, s1);
                            s0 = fmaf(w0[b + 1], v.y, s0); s1 = fmaf(w1[b + 1], v.y, s1);
                            s0 = fmaf(w0[b + 2], v.z, s0); s1 = fmaf(w1[b + 2], v.z, s1);
                            s0 = fmaf(w0[b + 3], v.w, s0); s1 = fmaf(w1[b + 3], v.w, s1);
                        }
                    }
                    acc0[t] += s0;
                    acc1[t] += s1;
                }
            }
#pragma unroll
            for (int t = 0; t < MT; t++) {
                acc0[t] = wave_sum(acc0[t]);
                acc1[t] = wave_sum(acc1[t]);
            }
            if (lane == 0) {
                for (uint32_t t = 0; t < mt; t++) {
                    const size_t o = (size_t)(t0 + t) * a.out_stride + a.col0 + j0;
                    if (pair) {
                        float v = silu_f(acc0[t]) * acc1[t];
                        if (a.flags & FLAG_ACCUMULATE) v += a.out[o];
                        a.out[o] = v;
                    } else {
                        float v = acc0[t];
                        if (a.flags & FLAG_ACCUMULATE) v += a.out[o];
                        a.out[o] = v;
                        if (has1) {
                            float u = acc1[t];
                            if (a.flags & FLAG_ACCUMULATE) u += a.out[o + 1];
                            a.out[o + 1] = u;
                        }
                    }
                }
            }
        }
    }
}

bool matvec_q4k_mfma_resident_accepts(const MvArgs &a);
zhip_result launch_matvec_q4k_mfma_resident(const Dispatch &d, const MvArgs &a, uint64_t w_bytes);
// The matrix-core variant of matvec_q8_0 for k of 2048, 4096 or 6144 .. 32768 in parts (matvec_q8_mfma_stream.hip).
bool matvec_q8_mfma_stream_accepts(const MvArgs &a);
zhip_result launch_matvec_q8_mfma_stream(const Dispatch &d, const MvArgs &a, uint64_t w_bytes);
// matvec_bf16 on the matrix cores, the weights read once for all tokens (matvec_bf16_mfma_stream.hip).
bool matvec_bf16_mfma_stream_accepts(const MvArgs &a);
zhip_result launch_matvec_bf16_mfma_stream(const Dispatch &d, const MvArgs &a, uint64_t w_bytes, bool f16);
bool matvec_q5k_mfma_resident_accepts(const MvArgs &a);
zhip_result launch_matvec_q5k_mfma_resident(const Dispatch &d, const MvArgs &a, uint64_t w_bytes);
// matvec_q6_k on the matrix cores for k of 1024, 2048, 3072, 4096 or 6144 .. 32768 in parts (matvec_q6k_mfma_stream.hip).
bool matvec_q6k_mfma_stream_accepts(const MvArgs &a);
zhip_result launch_matvec_q6k_mfma_stream(const Dispatch &d, const MvArgs &a, uint64_t w_bytes);
bool matvec_q3k_mfma_stream_accepts(const MvArgs &a);
zhip_result launch_matvec_q3k_mfma_stream(const Dispatch &d, const MvArgs &a, uint64_t w_bytes);
// matvec_q8_0 over rows of 1024 weights in the same kernel: a tile's rows as one flat stretch.
bool matvec_q8_0_mfma_flat_accepts(const MvArgs &a);
zhip_result launch_matvec_q8_0_mfma_flat(const Dispatch &d, const MvArgs &a, uint64_t w_bytes);
// Which matrices take it: 16 MB of weights or more (below, its fixed costs - the split of the
// tokens, a workgroup's first tile - outweigh what it saves at every width: 8 MB, k = 1024: 6.4 /
// 6.8 / 7.8 us at 2 / 4 / 8 tokens against 4.7 / 6.2 / 9.3) in contexts opened with
// ZHIP_OPTION_WIDE_DECODE, and then at every width from one token on: the kernel sums in another
// order than the general one, and a token's bits must not depend on the width of the step it
// runs in (src/sched/sched.zig:55-58; src/plan/qwen35.zig:380-381), so the route is a property
// of the matrix and of the context, never of the step. Its time hardly depends on the width
// (151936 x 1024: 55 us at 1 ... 8 tokens; the general kernel 52 / 75 / 122 us at 1 / 4 / 8), so
// a context pays ~6 % of a one-token step for verify steps at the one-token price.
constexpr uint64_t kBf16StreamBytes = 16ull << 20;
static bool bf16_stream_pays(const Dispatch &d, const MvArgs &a) {
    return d.dev->wide_decode && (uint64_t)a.rows * a.row_bytes >= kBf16StreamBytes;
}
// The tuned multiply (matvec_quant.h, a source file a format): type 3, 4, 5, 6 (K-quants) or 8 (Q8_0).
zhip_result launch_matvec_quant(const Dispatch &d, const MvArgs &a, int type);

template <class D, int MT>
static zhip_result run(const Dispatch &d, const MvArgs &a, uint32_t lds_bytes) {
    static bool configured[2] = {false, false};  // dynamic LDS above 64 KiB needs opting in once, kernel by kernel
    // Long rows of a matrix of few rows: a wave has few positions, each a trip to memory; four
    // in flight instead of one (1024 x 3072 bf16, one token: 6.3 -> 5.1 us). Elsewhere the
    // registers that takes cost more than it gains (151936 x 1024: 52 -> 62 us).
    const bool deep = kSplitInputs<D> && a.k >= 2048u && (uint64_t)a.rows * a.row_bytes <= (64ull << 20);
    auto kernel = deep ? matvec_kernel<D, MT, kSplitInputs<D> ? 4 : 1> : matvec_kernel<D, MT, 1>;
    if (lds_bytes > 65536u && !configured[deep]) {
        if (hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 64) != hipSuccess) {
            (void)hipGetLastError();
            return fail(d, ZHIP_E_BAD_COMMAND, "decode multiply: k = %u with %d tokens does not fit workgroup memory", a.k, MT);
        }
        configured[deep] = true;
    }
    const uint32_t per_group = (a.flags & FLAG_SILU_PAIR) ? 1u : 2u;
    const uint32_t groups = (a.rows + per_group - 1u) / per_group;
    const uint32_t want = (groups + 3u) / 4u;
    // Few enough workgroups that staging the inputs stays a small part of each
    // one's traffic, enough of them to keep every CU's SIMDs busy.
    const uint32_t cap = (uint32_t)d.dev->compute_units * (lds_bytes > 32768u ? 2u : 4u);
    const uint32_t blocks = want < cap ? want : cap;
    hipLaunchKernelGGL(kernel, dim3(blocks ? blocks : 1), dim3(256), lds_bytes, d.stream, a);
    return check_launch(d, D::name());
}

template <class D>
static zhip_result launch_matvec(const Dispatch &d, bool quant) {
    if (d.params_size < sizeof(MatvecParams)) return fail(d, ZHIP_E_BAD_COMMAND, "%s: params block of %zu bytes", D::name(), d.params_size);
    const MatvecParams &p = *reinterpret_cast<const MatvecParams *>(d.params);
    MatvecVariant v;
    if (quant && d.variant != 0) {
        v.wg = (d.variant & 0xffu) * 32u;
        v.lanes = (d.variant >> 8) & 0xffu;
        v.rows = (d.variant >> 16) & 0xffu;
        v.act_div = d.variant >> 24;
        if (v.wg == 0 || v.lanes == 0 || v.rows == 0 || v.wg % v.lanes != 0)
            return fail(d, ZHIP_E_BAD_COMMAND, "%s: variant id 0x%08x is not a MatvecVariant", D::name(), d.variant);
    }
    // Rows one workgroup of the logical grid covers (kernels.matvec_rows = 8
    // for the half-precision kernel, groupRows() for the quantized one).
    const uint32_t group_rows = quant ? v.groupRows() : 8u;
    if (d.grid[0] == 0 || d.grid[1] == 0 || d.grid[2] == 0) return ZHIP_OK;
    const uint64_t covered = (uint64_t)d.grid[0] * group_rows;
    MvArgs a{};
    a.n = p.n; a.k = p.k; a.col0 = p.col0; a.out_stride = p.out_stride; a.eps = p.eps;
    a.flags = p.flags; a.half = p.half;
    a.rows = (uint32_t)(covered < p.n ? covered : p.n);
    // The quantized kernel runs the first row of workgroups over up to
    // kMaxDecodeRows tokens; the half-precision one has a grid row per token.
    a.m = quant ? (d.grid[1] < kMaxDecodeRows ? d.grid[1] : kMaxDecodeRows) : d.grid[1];
    a.xr = (quant && p.x_stride != 0) ? p.x_stride * 4u : p.k;
    a.act_div = quant ? (float)v.act_div : 0.f;
    a.row_bytes = D::row_bytes(p.k);
    if (p.k == 0 || p.k % D::BLOCK != 0) return fail(d, ZHIP_E_BAD_COMMAND, "%s: k = %u is not a multiple of %u", D::name(), p.k, D::BLOCK);
    if (p.flags & ~7u) return fail(d, ZHIP_E_BAD_COMMAND, "%s: unknown flags 0x%x", D::name(), p.flags);
    if (a.rows == 0) return ZHIP_OK;
    const bool norm = p.flags & FLAG_NORM, pair = p.flags & FLAG_SILU_PAIR;
    for (int b = 1; b <= (norm ? 4 : 3); b++)
        if (!d.bind[b].bound) return fail(d, ZHIP_E_BAD_COMMAND, "%s: binding %d is not bound", D::name(), b);
    const uint64_t x_need = ((uint64_t)(a.m - 1) * a.xr + p.k) * 4u;
    const uint64_t w_rows = pair ? (uint64_t)p.half + a.rows : a.rows;
    const uint64_t w_need = w_rows * a.row_bytes;
    const uint64_t o_need = ((uint64_t)(a.m - 1) * p.out_stride + p.col0 + a.rows) * 4u;
    if (x_need > d.bind[1].size) return fail(d, ZHIP_E_BAD_COMMAND, "%s: x needs %llu bytes, %llu bound", D::name(), (unsigned long long)x_need, (unsigned long long)d.bind[1].size);
    if (w_need > d.bind[2].size) return fail(d, ZHIP_E_BAD_COMMAND, "%s: weights need %llu bytes, %llu bound", D::name(), (unsigned long long)w_need, (unsigned long long)d.bind[2].size);
    if (o_need > d.bind[3].size) return fail(d, ZHIP_E_BAD_COMMAND, "%s: out needs %llu bytes, %llu bound", D::name(), (unsigned long long)o_need, (unsigned long long)d.bind[3].size);
    if (norm && (uint64_t)p.k * 4u > d.bind[4].size) return fail(d, ZHIP_E_BAD_COMMAND, "%s: norm weights need %u bytes", D::name(), p.k * 4u);
    if (((uintptr_t)d.bind[1].ptr | (uintptr_t)d.bind[2].ptr | (norm ? (uintptr_t)d.bind[4].ptr : 0)) & 15u)
        return fail(d, ZHIP_E_BAD_COMMAND, "%s: x, weights and norm weights must be 16-byte aligned", D::name());
    if (((uintptr_t)d.bind[3].ptr & 3u) || (a.xr & 3u)) return fail(d, ZHIP_E_BAD_COMMAND, "%s: misaligned out or x stride", D::name());
    a.x = reinterpret_cast<const float *>(d.bind[1].ptr);
    a.w = d.bind[2].ptr;
    a.out = reinterpret_cast<float *>(d.bind[3].ptr);
    a.norm_w = norm ? reinterpret_cast<const float *>(d.bind[4].ptr) : nullptr;

    // matvec_bf16 / matvec_f16 over a matrix of some size, in a context that asked for it, go to
    // the kernel that reads the weights once for all of a step's tokens.
    if ((std::is_same<D, DecBF16>::value || std::is_same<D, DecF16>::value) && bf16_stream_pays(d, a) && matvec_bf16_mfma_stream_accepts(a))
        return launch_matvec_bf16_mfma_stream(d, a, d.bind[2].size, std::is_same<D, DecF16>::value);

    // MatvecVariant (wg 512, lanes 64, rows 16) names the matrix-core variants: a wave per sixteen rows.
    const bool matrix_cores = quant && v.lanes == 64u && v.rows == 16u && (D::CHUNK == 4 || D::CHUNK == 8 || D::CHUNK == 6 || D::CHUNK == 5 || D::CHUNK == 3);
    if (D::CHUNK == 3 && matrix_cores && matvec_q3k_mfma_stream_accepts(a)) return launch_matvec_q3k_mfma_stream(d, a, d.bind[2].size);
    // (matvec_q5_k: the Q4_K kernel for k of 2048, 4096 or 6144 .. 32768 in parts, with the fifth bits; other shapes run the default variant)
    if (D::CHUNK == 5 && matrix_cores && matvec_q5k_mfma_resident_accepts(a)) return launch_matvec_q5k_mfma_resident(d, a, d.bind[2].size);
    // (matvec_q6_k and matvec_q3_k: k of 1024, 2048, 3072, 4096 or 6144 .. 32768 in parts; every workgroup builds the tokens' operands, prologue included)
    if (D::CHUNK == 6 && matrix_cores && matvec_q6k_mfma_stream_accepts(a)) return launch_matvec_q6k_mfma_stream(d, a, d.bind[2].size);
    // The kernels that keep the tokens' operands in registers (k of 2048 or 4096, longer rows in parts of 2048, and whole tiles) compute a step's prologue (RMSNorm, silu(x / act_div):
    // src/kernels/matvec_quant.wgsl.hbs:73-89) themselves: their operands are built from one
    // round of loads, which the norm weights join (C3 at four tokens with the FFN launch's
    // RMSNorm: 22.6 us, 26.1 us with a pass of its own in front, 20.7 us without a prologue).
    if (D::CHUNK == 8 && matrix_cores && matvec_q8_0_mfma_flat_accepts(a)) return launch_matvec_q8_0_mfma_flat(d, a, d.bind[2].size);
    const bool resident = D::CHUNK == 4 && matrix_cores && matvec_q4k_mfma_resident_accepts(a);
    const bool q8_stream = D::CHUNK == 8 && matrix_cores && matvec_q8_mfma_stream_accepts(a);
    if (resident) return launch_matvec_q4k_mfma_resident(d, a, d.bind[2].size);
    // The same id on matvec_q8_0 (a one-token step too, so that a token's bits do not depend on
    // the step it ran in).
    if (q8_stream) return launch_matvec_q8_mfma_stream(d, a, d.bind[2].size);
    // Shapes these kernels do not take run the default variant under the id as well: the
    // matrix-core kernels that once stood in for them (a k-sliced Q4_K kernel, the compensated
    // prefill tiling for Q8_0) lost to it at two to four tokens on every shape measured
    // (Q4_K 4096 x 14336 at four tokens: 71.7 against 21.9 us; 5120 x 5120: 28.0 against 21.2).
    // The tuned kernel takes rows of whole 64-weight tasks.
    if (D::CHUNK != 0 && p.k % 64u == 0) return launch_matvec_quant(d, a, D::CHUNK);

    // Tokens per pass over the weights: as many as fit workgroup memory.
    const uint64_t row_lds = (uint64_t)p.k * 4u;
    const uint64_t max_lds = 160u * 1024u - 64u;
    uint32_t mt = a.m >= 5 ? 8u : a.m >= 3 ? 4u : a.m;
    while (mt > 1 && mt * row_lds > 65536u) mt >>= 1;
    if (mt * row_lds > max_lds) return fail(d, ZHIP_E_BAD_COMMAND, "%s: k = %u does not fit workgroup memory", D::name(), p.k);
    const uint32_t lds = (uint32_t)(mt * row_lds);
    switch (mt) {
    case 1: return run<D, 1>(d, a, lds);
    case 2: return run<D, 2>(d, a, lds);
    case 4: return run<D, 4>(d, a, lds);
    default: return run<D, 8>(d, a, lds);
    }
}

zhip_result launch_matvec_q8_0(const Dispatch &d) { return launch_matvec<DecQ8_0>(d, true); }
zhip_result launch_matvec_q4_k(const Dispatch &d) { return launch_matvec<DecQ4_K>(d, true); }
zhip_result launch_matvec_q3_k(const Dispatch &d) { return launch_matvec<DecQ3_K>(d, true); }
zhip_result launch_matvec_q5_k(const Dispatch &d) { return launch_matvec<DecQ5_K>(d, true); }
zhip_result launch_matvec_q6_k(const Dispatch &d) { return launch_matvec<DecQ6_K>(d, true); }
zhip_result launch_matvec_bf16(const Dispatch &d) { return launch_matvec<DecBF16>(d, false); }
zhip_result launch_matvec_f16(const Dispatch &d) { return launch_matvec<DecF16>(d, false); }

}  // namespace zhip
