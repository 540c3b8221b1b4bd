// matvec_q4_k: out[t][col0 + j] (+)= sum_i X(t, i) * w[j][i] over Q4_K rows,
// the decode step's multiply (contract of src/kernels/matvec_quant.wgsl.hbs with
// the decoder of src/kernels/quant/q4_k_dot.wgsl; block formula of
// src/ref/tensor.zig:94-116).
//
// Layout of the work. A Q4_K block is nine 16-byte vectors: a header (d, dmin,
// twelve packed 6-bit scale/min bytes) and 128 bytes of nibbles in four chunks
// of 32 bytes; chunk c holds sub-block 2c in its low nibbles and 2c + 1 in its
// high nibbles. A task is one chunk of one block of a row (64 weights): the
// lane that owns it loads the header vector and the chunk's two vectors, so
// every byte of the weight stream is loaded exactly once and a wave's load
// instruction falls in one contiguous span of the matrix. A row has k / 64
// tasks: lane l takes tasks l, l + 64, ...; rows of 1024 or 2048 weights pack
// four or two to a wave pass so that no lane idles.
//
// Arithmetic. Per task and token the lane computes
//     d*sc1 * sum(q_lo * x_lo) - dmin*m1 * sum(x_lo)
//   + d*sc2 * sum(q_hi * x_hi) - dmin*m2 * sum(x_hi)
// which is the block formula with scale and min factored out of the
// 32-element sums: one convert per weight (shared by all tokens) and one FMA
// per weight and token. High nibbles are used in place as 16 * q (a mask, no
// shift) with the factor 1/16 folded into the sub-block scale, which is exact.
// The 32-element input sums are computed once per workgroup. A lane adds its
// tasks' values in task order and the lanes reduce with DPP row operations in a
// fixed order, so a token's result does not depend on how many tokens share
// the launch or on which variant below runs it: the reference's bitwise split
// invariant (matvec_quant.wgsl.hbs:14-18).
//
// Variants. XREG (one token, at most one task per lane, i.e. k <= 4096): the
// lane's 64 inputs never change from row to row, so they live in registers and
// the loop touches nothing but the weight stream. Otherwise inputs are read
// from a bank-conflict-free padded LDS copy, once per task for both rows of a
// pass (two outputs, or the gate and up rows of one output with SILU_PAIR).
// In both, the next task's vectors are loaded before the current one is
// multiplied.
#include <hip/hip_runtime.h>

#include "common.h"
#include "decode.cuh"
#include "matvec_common.cuh"

namespace zhip {

struct Q4Chunk {
    uint4 h, q0, q1;
};

__device__ __forceinline__ Q4Chunk load_chunk(const uint8_t *block, uint32_t c) {
    Q4Chunk r;
    r.h = *reinterpret_cast<const uint4 *>(block);
    r.q0 = *reinterpret_cast<const uint4 *>(block + 16u + 32u * c);
    r.q1 = *reinterpret_cast<const uint4 *>(block + 32u + 32u * c);
    return r;
}

// Byte I of w as a float: v_cvt_f32_ubyte{0..3}, one instruction.
template <int I>
__device__ __forceinline__ float cvt_byte(uint32_t w) {
    return (float)((w >> (8 * I)) & 0xffu);
}

// The nibble masks, passed as kernel arguments: were they literals the
// compiler would fold mask and byte select into one bit-field extract per
// weight and then convert, three instructions a weight instead of a mask per
// word and a convert per weight.
struct NibbleMasks {
    uint32_t lo, hi;  // 0x0f0f0f0f, 0xf0f0f0f0
};

struct Q4Scales {
    float d1, m1, d2, m2;  // d*sc(2c), dmin*m(2c), d*sc(2c+1)/16, dmin*m(2c+1)
};

// The scale and min of sub-blocks 2c and 2c + 1 from the header vector
// (src/ref/tensor.zig:94-98); s16 = 16 * (c & 1), upper = c >= 2.
__device__ __forceinline__ Q4Scales chunk_scales(const uint4 &h, uint32_t s16, bool upper) {
    const float d = half_bits_to_float(h.x & 0xffffu);
    const float dmin = half_bits_to_float(h.x >> 16);
    const uint32_t a0 = h.y >> s16, a1 = h.z >> s16, a2 = h.w >> s16;
    const uint32_t sc_lo = a0 & 0x3f3fu, mn_lo = a1 & 0x3f3fu;
    const uint32_t sc_hi = (a2 & 0x0f0fu) | ((a0 >> 2) & 0x3030u);
    const uint32_t mn_hi = ((a2 >> 4) & 0x0f0fu) | ((a1 >> 2) & 0x3030u);
    const uint32_t sc = upper ? sc_hi : sc_lo, mn = upper ? mn_hi : mn_lo;
    Q4Scales s;
    s.d1 = d * cvt_byte<0>(sc);
    s.d2 = d * cvt_byte<1>(sc) * 0.0625f;
    s.m1 = dmin * cvt_byte<0>(mn);
    s.m2 = dmin * cvt_byte<1>(mn);
    return s;
}

template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_add(float v) {
    const int t = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, ROW_MASK, 0xF, true);
    return v + __int_as_float(t);
}

// Sums v over each segment of 2^seg_log2 lanes (16, 32 or 64) in a fixed
// order; the segment's last lane holds the total.
__device__ __forceinline__ float segment_sum(float v, uint32_t seg_log2) {
    v = dpp_add<0xB1, 0xF>(v);   // quad_perm [1,0,3,2]
    v = dpp_add<0x4E, 0xF>(v);   // quad_perm [2,3,0,1]
    v = dpp_add<0x141, 0xF>(v);  // row_half_mirror
    v = dpp_add<0x140, 0xF>(v);  // row_mirror: every lane holds its row of 16's sum
    if (seg_log2 >= 5) v = dpp_add<0x142, 0xA>(v);  // row_bcast15 into rows 1 and 3
    if (seg_log2 >= 6) v = dpp_add<0x143, 0xC>(v);  // row_bcast31 into rows 2 and 3
    return v;
}

// Floats per task in the padded LDS copy: 64 inputs and one vector of padding,
// so lanes reading the same offset of consecutive tasks hit different banks.
constexpr uint32_t kTaskStride = 68;

// One task of one row (ROWS = 1) or of the two rows of a pass (ROWS = 2) for
// MT tokens. x(t, e, h) gives inputs 4e .. 4e + 3 of the task's low (h = 0) or
// high (h = 1) sub-block for token t; sums(t) its two 32-element sums.
template <int MT, int ROWS, class XF, class SF>
__device__ __forceinline__ void task_dot(const Q4Chunk (&r)[ROWS], uint32_t s16, bool upper, NibbleMasks nm, XF x, SF sums, float (&out)[ROWS][MT]) {
    float s_lo[ROWS][MT], s_hi[ROWS][MT];
#pragma unroll
    for (int j = 0; j < ROWS; j++)
#pragma unroll
        for (int t = 0; t < MT; t++) s_lo[j][t] = s_hi[j][t] = 0.f;
#pragma unroll
    for (int e = 0; e < 8; e++) {
        float ql[ROWS][4], qh[ROWS][4];
#pragma unroll
        for (int j = 0; j < ROWS; j++) {
            const uint32_t word = e < 4 ? (e == 0 ? r[j].q0.x : e == 1 ? r[j].q0.y : e == 2 ? r[j].q0.z : r[j].q0.w)
                                        : (e == 4 ? r[j].q1.x : e == 5 ? r[j].q1.y : e == 6 ? r[j].q1.z : r[j].q1.w);
            const uint32_t lo = word & nm.lo, hi = word & nm.hi;
            ql[j][0] = cvt_byte<0>(lo); ql[j][1] = cvt_byte<1>(lo); ql[j][2] = cvt_byte<2>(lo); ql[j][3] = cvt_byte<3>(lo);
            qh[j][0] = cvt_byte<0>(hi); qh[j][1] = cvt_byte<1>(hi); qh[j][2] = cvt_byte<2>(hi); qh[j][3] = cvt_byte<3>(hi);
        }
#pragma unroll
        for (int t = 0; t < MT; t++) {
            const float4 xl = x(t, e, 0), xh = x(t, e, 1);
#pragma unroll
            for (int j = 0; j < ROWS; j++) {
                s_lo[j][t] = fmaf(ql[j][0], xl.x, s_lo[j][t]);
                s_hi[j][t] = fmaf(qh[j][0], xh.x, s_hi[j][t]);
                s_lo[j][t] = fmaf(ql[j][1], xl.y, s_lo[j][t]);
                s_hi[j][t] = fmaf(qh[j][1], xh.y, s_hi[j][t]);
                s_lo[j][t] = fmaf(ql[j][2], xl.z, s_lo[j][t]);
                s_hi[j][t] = fmaf(qh[j][2], xh.z, s_hi[j][t]);
                s_lo[j][t] = fmaf(ql[j][3], xl.w, s_lo[j][t]);
                s_hi[j][t] = fmaf(qh[j][3], xh.w, s_hi[j][t]);
            }
        }
    }
#pragma unroll
    for (int j = 0; j < ROWS; j++) {
        const Q4Scales s = chunk_scales(r[j].h, s16, upper);
#pragma unroll
        for (int t = 0; t < MT; t++) {
            const float2 sm = sums(t);
            float v = s.d1 * s_lo[j][t];
            v = fmaf(-s.m1, sm.x, v);
            v = fmaf(s.d2, s_hi[j][t], v);
            v = fmaf(-s.m2, sm.y, v);
            out[j][t] = v;
        }
    }
}

struct Q4Args {
    MvArgs a;
    uint32_t t0;        // first token of this pass
    uint32_t mt;        // tokens in this pass (<= MT)
    uint32_t seg_log2;  // lanes per row: 4, 5 or 6
    uint32_t tasks;     // k / 64
    NibbleMasks nm;
};

template <int MT, bool PAIR, bool XREG>
__global__ __launch_bounds__(256) void matvec_q4k_kernel(Q4Args q) {
    const MvArgs &a = q.a;
    extern __shared__ float4 lds4[];
    __shared__ float red[4];
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t tasks = q.tasks;
    const uint32_t tok_stride4 = tasks * (kTaskStride / 4u);  // float4s per token
    float *sums_lds = reinterpret_cast<float *>(lds4 + (size_t)MT * tok_stride4);

    // Rows a pass takes: the gate and up rows of an output, or two outputs so
    // that one read of the inputs from LDS serves both; with the inputs in
    // registers a pass is a single row.
    constexpr int kRows = (PAIR || !XREG) ? 2 : 1;
    const uint32_t gwave = blockIdx.x * 4u + wave, nwaves = gridDim.x * 4u;
    const uint32_t seg = 1u << q.seg_log2;
    const uint32_t tsub = lane & (seg - 1u), rsub = lane >> q.seg_log2, rpi = 64u >> q.seg_log2;
    const uint32_t iters = (tasks + seg - 1u) >> q.seg_log2;
    const uint32_t per_unit = PAIR ? rpi : rpi * kRows;
    const uint32_t units = (a.rows + per_unit - 1u) / per_unit;
    const bool writer = tsub == seg - 1u;

    // A position in the wave's walk over (unit, 64-task slice) pairs, and the
    // weight rows it reads there: output j0 (and j0 + 1), or the gate row j0
    // and the up row half + j0. Rows past the end are clamped for the loads
    // and skipped at the store.
    struct Cursor {
        uint32_t u, i, j0, ra, rb;
    };
    auto place = [&](Cursor &c) {
        const uint32_t unit = c.u < units ? c.u : units - 1u;
        c.j0 = PAIR ? unit * rpi + rsub : (unit * rpi + rsub) * kRows;
        c.ra = c.j0 < a.rows ? c.j0 : 0u;
        if (PAIR) c.rb = a.half + c.ra;
        else c.rb = c.j0 + 1u < a.rows ? c.j0 + 1u : c.ra;
    };
    auto advance = [&](Cursor &c) {
        if (c.i + 1u < iters) {
            c.i++;
        } else {
            c.i = 0;
            c.u += nwaves;
            place(c);
        }
    };
    // Past the wave's last position the cursor is clamped to a valid one, so
    // loads need no branch around them (their results are not used).
    auto load_at = [&](const Cursor &c, Q4Chunk (&dst)[kRows]) {
        const uint32_t task = tsub + c.i * seg;
        const uint32_t tk = task < tasks ? task : 0u;
        const uint32_t blk = tk >> 2, ch = tk & 3u;
        dst[0] = load_chunk(a.w + (size_t)c.ra * a.row_bytes + (size_t)blk * 144u, ch);
        if (kRows == 2) dst[kRows - 1] = load_chunk(a.w + (size_t)c.rb * a.row_bytes + (size_t)blk * 144u, ch);
    };

    // Weights do not depend on the inputs: start loading the first positions
    // before anything else, so the stream is already flowing while the inputs
    // are fetched. kDepth positions stay in flight ahead of the one multiplied
    // (deeper queues cost registers, hence occupancy, and measured no faster).
    constexpr int kDepth = 1;
    Q4Chunk buf[kDepth + 1][kRows];
    Cursor cc{gwave < units ? gwave : 0u, 0u, 0u, 0u, 0u};
    place(cc);
    Cursor lc = cc;
#pragma unroll
    for (int dpt = 0; dpt < kDepth; dpt++) {
        load_at(lc, buf[dpt]);
        advance(lc);
    }

    float xl[32], xh[32];
    float2 xsum = make_float2(0.f, 0.f);
    // Stage the pass's tokens, padded per task (coalesced loads; a lane's own
    // 64 inputs are 256 bytes apart from its neighbour's).
    for (uint32_t t = 0; t < (uint32_t)MT; t++) {
        float4 *dst = lds4 + (size_t)t * tok_stride4;
        if (t < q.mt) {
            stage_token(a, q.t0 + t, dst, red, true);
        } else {
            for (uint32_t e = tid; e < tok_stride4; e += 256u) dst[e] = make_float4(0.f, 0.f, 0.f, 0.f);
        }
    }
    __syncthreads();
    if (XREG) {
        // The lane's one task's inputs into registers, and their two sums in
        // the same order the LDS pass below adds them.
        if (gwave >= units) return;
        const uint32_t task = tsub < tasks ? tsub : 0u;
        const float4 *src = lds4 + task * (kTaskStride / 4u);
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const float4 v = src[e], w = src[8 + e];
            xl[4 * e] = v.x; xl[4 * e + 1] = v.y; xl[4 * e + 2] = v.z; xl[4 * e + 3] = v.w;
            xh[4 * e] = w.x; xh[4 * e + 1] = w.y; xh[4 * e + 2] = w.z; xh[4 * e + 3] = w.w;
        }
#pragma unroll
        for (int e = 0; e < 32; e++) {
            xsum.x += xl[e];
            xsum.y += xh[e];
        }
    } else {
        for (uint32_t idx = tid; idx < (uint32_t)MT * tasks * 2u; idx += 256u) {
            const uint32_t t = idx / (tasks * 2u), rem = idx % (tasks * 2u);
            const float *src = reinterpret_cast<const float *>(lds4 + (size_t)t * tok_stride4) + (rem >> 1) * kTaskStride + (rem & 1u) * 32u;
            float sum = 0.f;
#pragma unroll
            for (int e = 0; e < 32; e++) sum += src[e];
            sums_lds[idx] = sum;
        }
        __syncthreads();
        if (gwave >= units) return;
    }

    float acc[kRows][MT];
#pragma unroll
    for (int j = 0; j < kRows; j++)
#pragma unroll
        for (int t = 0; t < MT; t++) acc[j][t] = 0.f;

    // Multiplies the position `c` from `cur`; at a unit's last slice reduces
    // and stores its outputs.
    auto compute = [&](const Cursor &c, const Q4Chunk (&cur)[kRows]) {
        const uint32_t task = tsub + c.i * seg;
        if (task < tasks) {
            const uint32_t ch = task & 3u;
            float v[kRows][MT];
            if (XREG) {
                task_dot<MT, kRows>(cur, 16u * (ch & 1u), ch >= 2u, q.nm,
                    [&](int, int e, int h) { return h ? make_float4(xh[4 * e], xh[4 * e + 1], xh[4 * e + 2], xh[4 * e + 3]) : make_float4(xl[4 * e], xl[4 * e + 1], xl[4 * e + 2], xl[4 * e + 3]); },
                    [&](int) { return xsum; }, v);
            } else {
                const float4 *xt = lds4 + task * (kTaskStride / 4u);
                const float *st = sums_lds + 2u * task;
                task_dot<MT, kRows>(cur, 16u * (ch & 1u), ch >= 2u, q.nm,
                    [&](int t, int e, int h) { return xt[(size_t)t * tok_stride4 + 8 * h + e]; },
                    [&](int t) { return make_float2(st[(size_t)t * tasks * 2u], st[(size_t)t * tasks * 2u + 1u]); }, v);
            }
#pragma unroll
            for (int j = 0; j < kRows; j++)
#pragma unroll
                for (int t = 0; t < MT; t++) acc[j][t] += v[j][t];
        }
        if (c.i + 1u == iters) {
#pragma unroll
            for (int t = 0; t < MT; t++) {
                const float s0 = segment_sum(acc[0][t], q.seg_log2);
                const float s1 = kRows == 2 ? segment_sum(acc[kRows - 1][t], q.seg_log2) : 0.f;
                acc[0][t] = acc[kRows - 1][t] = 0.f;
                if (writer && (uint32_t)t < q.mt && c.j0 < a.rows) {
                    const size_t o = (size_t)(q.t0 + t) * a.out_stride + a.col0 + c.j0;
                    if (PAIR) {
                        float r = silu_f(s0) * s1;
                        if (a.flags & FLAG_ACCUMULATE) r += a.out[o];
                        a.out[o] = r;
                    } else {
                        float r = s0;
                        if (a.flags & FLAG_ACCUMULATE) r += a.out[o];
                        a.out[o] = r;
                        if (kRows == 2 && c.j0 + 1u < a.rows) {
                            float r1 = s1;
                            if (a.flags & FLAG_ACCUMULATE) r1 += a.out[o + 1];
                            a.out[o + 1] = r1;
                        }
                    }
                }
            }
        }
    };

    // The buffers rotate by position, so every index below is a constant.
    bool done = false;
    while (!done) {
#pragma unroll
        for (int ph = 0; ph <= kDepth; ph++) {
            if (done) break;
            load_at(lc, buf[(ph + kDepth) % (kDepth + 1)]);
            advance(lc);
            compute(cc, buf[ph]);
            advance(cc);
            done = cc.u >= units;
        }
    }
}

template <int MT, bool PAIR, bool XREG>
static zhip_result run_q4k(const Dispatch &d, const Q4Args &q, uint32_t lds, uint32_t blocks) {
    static bool configured = false;  // dynamic LDS above 64 KiB needs opting in once
    if (lds > 65536u && !configured) {
        if (hipFuncSetAttribute(reinterpret_cast<const void *>(matvec_q4k_kernel<MT, PAIR, XREG>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 64) != hipSuccess) {
            (void)hipGetLastError();
            return fail(d, ZHIP_E_BAD_COMMAND, "matvec_q4_k: k = %u with %d tokens does not fit workgroup memory", q.a.k, MT);
        }
        configured = true;
    }
    hipLaunchKernelGGL((matvec_q4k_kernel<MT, PAIR, XREG>), dim3(blocks), dim3(256), lds, d.stream, q);
    return check_launch(d, "matvec_q4_k");
}

// Launches matvec_q4_k for validated arguments: one pass per group of up to
// four tokens.
zhip_result launch_matvec_q4k(const Dispatch &d, const MvArgs &a) {
    Q4Args q{};
    q.a = a;
    q.tasks = a.k / 64u;
    q.seg_log2 = q.tasks == 16u ? 4u : q.tasks == 32u ? 5u : 6u;
    q.nm = NibbleMasks{0x0f0f0f0fu, 0xf0f0f0f0u};
    const bool pair = a.flags & FLAG_SILU_PAIR;
    const uint32_t rpi = 64u >> q.seg_log2;
    const uint64_t tok_lds = (uint64_t)q.tasks * kTaskStride * 4u + (uint64_t)q.tasks * 8u;
    const uint64_t max_lds = 160u * 1024u - 64u;
    if (tok_lds > max_lds) return fail(d, ZHIP_E_BAD_COMMAND, "matvec_q4_k: k = %u does not fit workgroup memory", a.k);
    for (uint32_t t0 = 0; t0 < a.m;) {
        uint32_t left = a.m - t0;
        uint32_t mt = left >= 3u ? 4u : left;
        // Two workgroups a CU must fit their staged tokens in the 160 KB of LDS.
        while (mt > 1u && mt * tok_lds > 80u * 1024u - 64u) mt >>= 1;
        q.t0 = t0;
        q.mt = left < mt ? left : mt;
        const uint32_t lds = (uint32_t)(mt * tok_lds);
        const bool xreg = a.m == 1u && q.tasks <= 64u;
        const uint32_t per_unit = pair ? rpi : rpi * (xreg ? 1u : 2u);
        const uint32_t units = (a.rows + per_unit - 1u) / per_unit;
        const uint32_t want = (units + 3u) / 4u;
        // Three workgroups a CU measured best for the 4096 x 14336 multiply:
        // more of them repeat the input staging, fewer leave too few loads in flight.
        const uint32_t cap = (uint32_t)d.dev->compute_units * (xreg ? 3u : 2u);
        const uint32_t blocks = want < cap ? want : cap;
        zhip_result r;
        if (xreg) r = pair ? run_q4k<1, true, true>(d, q, lds, blocks) : run_q4k<1, false, true>(d, q, lds, blocks);
        else if (mt == 1u) r = pair ? run_q4k<1, true, false>(d, q, lds, blocks) : run_q4k<1, false, false>(d, q, lds, blocks);
        else if (mt == 2u) r = pair ? run_q4k<2, true, false>(d, q, lds, blocks) : run_q4k<2, false, false>(d, q, lds, blocks);
        else r = pair ? run_q4k<4, true, false>(d, q, lds, blocks) : run_q4k<4, false, false>(d, q, lds, blocks);
        if (r != ZHIP_OK) return r;
        t0 += q.mt;
    }
    return ZHIP_OK;
}

}  // namespace zhip
