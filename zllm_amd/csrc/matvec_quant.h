// matvec_q8_0 / matvec_q3_k / matvec_q4_k / matvec_q5_k / matvec_q6_k:
// out[t][col0 + j] (+)= sum_i X(t, i) * w[j][i] over quantized rows, the decode
// step's multiply (contract of src/kernels/matvec_quant.wgsl.hbs with the
// decoders of src/kernels/quant/*_dot.wgsl; block formulas of
// src/ref/tensor.zig:49-160).
//
// Layout of the work. A row splits into tasks of 64 weights whose sub-blocks
// share their scales (four to a 256-weight K-quant block; two 32-weight blocks
// for Q8_0): for Q4_K and Q5_K a 32-byte chunk of
// nibbles (sub-block 2c in the low nibbles, 2c + 1 in the high ones), for Q6_K
// sixteen positions of one half (four runs of sixteen weights, 32 apart), for
// Q3_K two of the repacked 16-byte units. The
// lane that owns a task loads its vectors and the block's scales, so every byte
// of the weight stream is loaded by exactly one lane per use and a wave's load
// instruction falls in one contiguous span of the matrix. A row has k / 64
// tasks: lane l takes tasks l, l + 64, ...; rows of 1024 or 2048 weights pack
// four or two to a wave pass so that no lane idles.
//
// Arithmetic. Per task and token the lane computes, for each sub-block s of
// the task, scale_s * sum(q * x) - min_s * sum(x): the block formula with
// scale and min factored out of the sub-block's sums, so a weight costs one
// convert (shared by all tokens) and one FMA per token. Q4_K high nibbles are
// used in place as 16 * q (a mask, no shift) with the factor 1/16 folded into
// the sub-block scale, which is exact. The sub-block input sums are computed
// once per workgroup. A lane adds its tasks' values in task order and the lanes
// reduce with DPP row operations in a fixed order, so a token's result does not
// depend on how many tokens share the launch or on which variant below runs
// it: the reference's bitwise split invariant (matvec_quant.wgsl.hbs:14-18).
//
// Kernels. matvec_quant_kernel (steps of one to four tokens, any row length): inputs are read
// from a bank-conflict-free padded LDS copy kept in task order, once per task for both rows of
// a pass (two outputs, or the gate and up rows of one output with SILU_PAIR), the next task's
// vectors loaded before the current one is multiplied. matvec_quant_row_kernel (one token, at
// most one task per lane, i.e. k <= 4096): the lane's 64 inputs never change from row to row,
// so they live in registers and the loop touches nothing but the weight stream; it asks for the
// token's inputs (and norm weights) before its first weights: loads complete in order within a
// wave, so inputs requested behind a weight row would wait for that row's trip to memory before
// the staging could start. matvec_quant_slices_kernel: the same for one token over longer rows,
// a 64-task slice of the row a wave. matvec_quant_long_kernel: steps of several tokens over
// rows too long for the tokens to share LDS, tile by tile.
#pragma once
#include <hip/hip_runtime.h>

#include "common.h"
#include "decode.h"
#include "matvec_common.h"

namespace zhip {

// Byte I of w as a float: v_cvt_f32_ubyte{0..3}, one instruction.
template <int I>
__device__ __forceinline__ float cvt_byte(uint32_t w) {
    return (float)((w >> (8 * I)) & 0xffu);
}

// Bit masks, passed as kernel arguments: were they literals the compiler would
// fold mask and byte select into one bit-field extract per weight and then
// convert, three instructions a weight instead of a mask per word and a convert
// per weight.
struct Masks {
    uint32_t lo, hi, two, one;  // 0x0f0f0f0f, 0xf0f0f0f0, 0x03030303, 0x01010101
};

struct KScales {
    float d1, m1, d2, m2;  // d*sc(2c), dmin*m(2c), d*sc(2c+1) (/16 for Q4_K), dmin*m(2c+1)
};

// The scale and min of sub-blocks 2c and 2c + 1 from a Q4_K / Q5_K header
// vector (src/ref/tensor.zig:94-98); s16 = 16 * (c & 1), upper = c >= 2.
template <bool SIXTEENTH>
__device__ __forceinline__ KScales chunk_scales(const uint4 &h, uint32_t s16, bool upper) {
    const float d = half_bits_to_float(h.x & 0xffffu);
    const float dmin = half_bits_to_float(h.x >> 16);
    const uint32_t a0 = h.y >> s16, a1 = h.z >> s16, a2 = h.w >> s16;
    const uint32_t sc_lo = a0 & 0x3f3fu, mn_lo = a1 & 0x3f3fu;
    const uint32_t sc_hi = (a2 & 0x0f0fu) | ((a0 >> 2) & 0x3030u);
    const uint32_t mn_hi = ((a2 >> 4) & 0x0f0fu) | ((a1 >> 2) & 0x3030u);
    const uint32_t sc = upper ? sc_hi : sc_lo, mn = upper ? mn_hi : mn_lo;
    KScales s;
    s.d1 = d * cvt_byte<0>(sc);
    s.d2 = SIXTEENTH ? d * cvt_byte<1>(sc) * 0.0625f : d * cvt_byte<1>(sc);
    s.m1 = dmin * cvt_byte<0>(mn);
    s.m2 = dmin * cvt_byte<1>(mn);
    return s;
}

// The same four values for a lane whose chunk never changes: what depends on the chunk alone
// (which header bytes, which bit fields) is worked out once, and a header costs eight integer
// operations instead of fourteen. Lower chunks (c < 2) take the low six bits of bytes 2c, 2c + 1
// of the scale and of the min words; upper ones the nibbles of bytes 2c + 4, 2c + 5 of the
// third word with the top two bits of the lower chunks' bytes above them.
struct ChunkKeys {
    uint32_t sel;     // v_perm_b32 selector: bytes 2 (c & 1), + 1 of the scale word, then of the min word
    uint32_t shift;   // 16 (c & 1)
    uint32_t six;     // 0x3f3f3f3f for lower chunks, else 0
    uint32_t top;     // 0x30303030 for upper chunks, else 0
    uint32_t lo, hi;  // 0x0f0f, 0xf0f0 for upper chunks, else 0
    uint32_t c;       // the chunk
};
__device__ __forceinline__ ChunkKeys chunk_keys(uint32_t c) {
    const bool upper = c >= 2u;
    ChunkKeys k;
    k.sel = (c & 1u) ? 0x07060302u : 0x05040100u;
    k.shift = 16u * (c & 1u);
    k.six = upper ? 0u : 0x3f3f3f3fu;
    k.top = upper ? 0x30303030u : 0u;
    k.lo = upper ? 0x0f0fu : 0u;
    k.hi = upper ? 0xf0f0u : 0u;
    k.c = c;
    return k;
}
template <bool SIXTEENTH>
__device__ __forceinline__ KScales chunk_scales(const uint4 &h, const ChunkKeys &k) {
    const float d = half_bits_to_float(h.x & 0xffffu);
    const float dmin = half_bits_to_float(h.x >> 16);
    const uint32_t w = __builtin_amdgcn_perm(h.z, h.y, k.sel);  // scale bytes, min bytes
    const uint32_t a2 = h.w >> k.shift;
    uint32_t r = w & k.six;
    r = ((w >> 2) & k.top) | r;
    r = (a2 & k.lo) | r;
    r = ((a2 & k.hi) << 12) | r;  // bytes: scale 2c, scale 2c + 1, min 2c, min 2c + 1
    KScales s;
    s.d1 = d * cvt_byte<0>(r);
    s.d2 = SIXTEENTH ? d * cvt_byte<1>(r) * 0.0625f : d * cvt_byte<1>(r);
    s.m1 = dmin * cvt_byte<2>(r);
    s.m2 = dmin * cvt_byte<3>(r);
    return s;
}
// (the form the kernels whose lanes change chunks call)
template <bool SIXTEENTH>
__device__ __forceinline__ KScales chunk_scales(const uint4 &h, uint32_t c) { return chunk_scales<SIXTEENTH>(h, 16u * (c & 1u), c >= 2u); }

__device__ __forceinline__ uint32_t chunk_no(uint32_t c) { return c; }
__device__ __forceinline__ uint32_t chunk_no(const ChunkKeys &k) { return k.c; }

__device__ __forceinline__ uint32_t word_of(const uint4 &v, int i) { return i == 0 ? v.x : i == 1 ? v.y : i == 2 ? v.z : v.w; }

// Four weights (the bytes of `word`) times four inputs, added to `sum`.
__device__ __forceinline__ float dot_bytes(uint32_t word, const float4 &x, float sum) {
    sum = fmaf(cvt_byte<0>(word), x.x, sum);
    sum = fmaf(cvt_byte<1>(word), x.y, sum);
    sum = fmaf(cvt_byte<2>(word), x.z, sum);
    sum = fmaf(cvt_byte<3>(word), x.w, sum);
    return sum;
}

// ---- the formats ---------------------------------------------------------------------
// A format names its task's vectors (Raw), loads them, says where a row's
// inputs go in task order, and multiplies one task of one row (ROWS = 1) or of
// the two rows of a pass (ROWS = 2) for MT tokens. x(t, v) gives inputs
// 4v .. 4v + 3 of the task in task order for token t; sums(t, s) the sum of the
// task's s-th run of 64 / NSUM inputs. where() gives the byte offsets of a task's vectors from
// the start of a stretch of rows (base: the row's offset in the stretch) and fetch() loads them
// through a range-checked buffer that begins at the stretch.

// Q8_0 split rows (src/kernels/repack_q8_0.wgsl): k signed bytes, then k / 32
// f16 scales. Task = 64 consecutive weights, two blocks of 32 with a scale each;
// no minimum, so the input sums go unused.
struct KQ8 {
    static constexpr int NSUM = 2;
    static constexpr int STAGE2 = 0, STAGE4 = 1;  // tokens whose inputs are loaded at once
    static constexpr bool ALL4 = true;            // a launch of at most a workgroup a CU stages a pass of four at once
    static constexpr bool DEFER = false;
    static constexpr bool PAIR2 = false;  // a two-token gate / up step with the inputs in registers leaves two waves a SIMD their registers
    static const char *name() { return "matvec_q8_0"; }
    struct Raw {
        uint4 q[4];
        uint32_t d;  // the two blocks' scales
    };
    __device__ static Raw load(const uint8_t *row, uint32_t k, uint32_t task) {
        Raw r;
#pragma unroll
        for (int i = 0; i < 4; i++) r.q[i] = *reinterpret_cast<const uint4 *>(row + 64u * task + 16u * i);
        r.d = *reinterpret_cast<const uint32_t *>(row + k + 4u * task);
        return r;
    }
    struct Where {
        uint32_t q, d;
    };
    __device__ static Where where(uint32_t base, uint32_t k, uint32_t task) { return Where{base + 64u * task, base + k + 4u * task}; }
    __device__ static Where nowhere() { return Where{kNowhere, kNowhere}; }
    __device__ static Raw fetch(__amdgpu_buffer_rsrc_t w, const Where &at) {
        Raw r;
#pragma unroll
        for (int i = 0; i < 4; i++) r.q[i] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(w, at.q + 16u * i, 0, 0));
        r.d = __builtin_amdgcn_raw_buffer_load_b32(w, at.d, 0, 0);
        return r;
    }
    __device__ static uint32_t stage_index(uint32_t v) { return v; }

    typedef uint32_t Keys;
    __device__ static Keys keys(uint32_t c) { return c; }
    template <int MT, int ROWS, class XF, class SF>
    __device__ static void dot(const Raw (&r)[ROWS], uint32_t, Masks, XF x, SF, float (&out)[ROWS][MT]) {
        float s[ROWS][MT][2];
#pragma unroll
        for (int j = 0; j < ROWS; j++)
#pragma unroll
            for (int t = 0; t < MT; t++) s[j][t][0] = s[j][t][1] = 0.f;
#pragma unroll
        for (int v = 0; v < 16; v++) {
#pragma unroll
            for (int t = 0; t < MT; t++) {
                const float4 xv = x(t, v);
#pragma unroll
                for (int j = 0; j < ROWS; j++) {
                    const uint32_t word = word_of(r[j].q[v >> 2], v & 3);
                    float sum = s[j][t][v >> 3];
                    sum = fmaf((float)(int8_t)(word & 0xffu), xv.x, sum);
                    sum = fmaf((float)(int8_t)((word >> 8) & 0xffu), xv.y, sum);
                    sum = fmaf((float)(int8_t)((word >> 16) & 0xffu), xv.z, sum);
                    sum = fmaf((float)(int8_t)(word >> 24), xv.w, sum);
                    s[j][t][v >> 3] = sum;
                }
            }
        }
#pragma unroll
        for (int j = 0; j < ROWS; j++) {
            const float d0 = half_bits_to_float(r[j].d & 0xffffu), d1 = half_bits_to_float(r[j].d >> 16);
#pragma unroll
            for (int t = 0; t < MT; t++) out[j][t] = fmaf(d1, s[j][t][1], d0 * s[j][t][0]);
        }
    }
};

// Q3_K: blocks repacked at load into eight self-contained 16-byte units of 32
// weights (src/kernels/repack_q3_k.wgsl; the layout is spelled out at DecQ3_K):
// two words of 2-bit values, a word of third bits, scale - 32 for each half as
// signed bytes, d. A weight is d * (scale - 32) * (q - 4) with q = low bits +
// 4 * third bit. Task = two consecutive units: four runs of sixteen weights.
struct KQ3 {
    static constexpr uint32_t BLOCK_BYTES = 128;
    static constexpr int NSUM = 4;
    static constexpr int STAGE2 = 2, STAGE4 = 2;  // tokens whose inputs are loaded at once
    static constexpr bool ALL4 = false;           // (four at once measured slower on every shape: 1024 x 4096 7.7 against 7.1 us)
    static constexpr bool DEFER = true;
    static constexpr bool PAIR2 = true;  // a two-token gate / up step with the inputs in registers leaves two waves a SIMD their registers
    static const char *name() { return "matvec_q3_k"; }
    struct Raw {
        uint4 u[2];
    };
    __device__ static Raw load(const uint8_t *row, uint32_t, uint32_t task) {
        const uint8_t *block = row + (size_t)(task >> 2) * BLOCK_BYTES;
        const uint32_t c = task & 3u;
        Raw r;
        r.u[0] = *reinterpret_cast<const uint4 *>(block + 32u * c);
        r.u[1] = *reinterpret_cast<const uint4 *>(block + 32u * c + 16u);
        return r;
    }
    struct Where {
        uint32_t u;
    };
    __device__ static Where where(uint32_t base, uint32_t, uint32_t task) { return Where{base + (task >> 2) * BLOCK_BYTES + 32u * (task & 3u)}; }
    __device__ static Where nowhere() { return Where{kNowhere}; }
    __device__ static Raw fetch(__amdgpu_buffer_rsrc_t w, const Where &at) {
        Raw r;
        r.u[0] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(w, at.u, 0, 0));
        r.u[1] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(w, at.u + 16u, 0, 0));
        return r;
    }
    __device__ static uint32_t stage_index(uint32_t v) { return v; }

    typedef uint32_t Keys;
    __device__ static Keys keys(uint32_t c) { return c; }
    template <int MT, int ROWS, class XF, class SF>
    __device__ static void dot(const Raw (&r)[ROWS], uint32_t, Masks nm, XF x, SF sums, float (&out)[ROWS][MT]) {
        float s[ROWS][MT][4];
#pragma unroll
        for (int j = 0; j < ROWS; j++)
#pragma unroll
            for (int t = 0; t < MT; t++)
#pragma unroll
                for (int run = 0; run < 4; run++) s[j][t][run] = 0.f;
#pragma unroll
        for (int unit = 0; unit < 2; unit++) {
#pragma unroll
            for (int e = 0; e < 8; e++) {
                uint32_t q[ROWS];
#pragma unroll
                for (int j = 0; j < ROWS; j++) {
                    const uint4 &u = r[j].u[unit];
                    const uint32_t low = ((e < 4 ? u.x : u.y) >> (2 * (e & 3))) & nm.two;
                    const uint32_t third = (u.z >> e) & nm.one;
                    q[j] = (third << 2) | low;
                }
                const int run = 2 * unit + (e >> 2);
#pragma unroll
                for (int t = 0; t < MT; t++) {
                    const float4 xv = x(t, 8 * unit + e);
#pragma unroll
                    for (int j = 0; j < ROWS; j++) s[j][t][run] = dot_bytes(q[j], xv, s[j][t][run]);
                }
            }
        }
#pragma unroll
        for (int j = 0; j < ROWS; j++) {
            float scale[4];
#pragma unroll
            for (int unit = 0; unit < 2; unit++) {
                const uint32_t tail = r[j].u[unit].w;
                const float d = half_bits_to_float(tail >> 16);
                scale[2 * unit] = d * (float)(int8_t)(tail & 0xffu);
                scale[2 * unit + 1] = d * (float)(int8_t)((tail >> 8) & 0xffu);
            }
#pragma unroll
            for (int t = 0; t < MT; t++) {
                float v = 0.f;
#pragma unroll
                for (int run = 0; run < 4; run++) v = fmaf(scale[run], fmaf(-4.f, sums(t, run), s[j][t][run]), v);
                out[j][t] = v;
            }
        }
    }
};

// Q4_K: 144-byte blocks (header vector; 128 bytes of nibbles in four chunks of
// 32: chunk c holds sub-block 2c in its low nibbles and 2c + 1 in its high
// ones). Task = chunk: 32 low-nibble weights, then 32 high-nibble ones.
struct KQ4 {
    static constexpr uint32_t BLOCK_BYTES = 144;
    static constexpr int NSUM = 2;
    static constexpr int STAGE2 = 2, STAGE4 = 1;  // tokens whose inputs are loaded at once
    static constexpr bool ALL4 = true;            // a launch of at most a workgroup a CU stages a pass of four at once
    static constexpr bool DEFER = true;
    static constexpr bool PAIR2 = true;  // a two-token gate / up step with the inputs in registers leaves two waves a SIMD their registers
    static const char *name() { return "matvec_q4_k"; }
    struct Raw {
        uint4 h, q0, q1;
    };
    __device__ static Raw load(const uint8_t *row, uint32_t, uint32_t task) {
        const uint8_t *block = row + (size_t)(task >> 2) * BLOCK_BYTES;
        const uint32_t c = task & 3u;
        Raw r;
        r.h = *reinterpret_cast<const uint4 *>(block);
        r.q0 = *reinterpret_cast<const uint4 *>(block + 16u + 32u * c);
        r.q1 = *reinterpret_cast<const uint4 *>(block + 32u + 32u * c);
        return r;
    }
    struct Where {
        uint32_t h, q;
    };
    __device__ static Where where(uint32_t base, uint32_t, uint32_t task) {
        const uint32_t block = base + (task >> 2) * BLOCK_BYTES;
        return Where{block, block + 16u + 32u * (task & 3u)};
    }
    __device__ static Where nowhere() { return Where{kNowhere, kNowhere}; }
    __device__ static Raw fetch(__amdgpu_buffer_rsrc_t w, const Where &at) {
        Raw r;
        r.h = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(w, at.h, 0, 0));
        r.q0 = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(w, at.q, 0, 0));
        r.q1 = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(w, at.q + 16u, 0, 0));
        return r;
    }
    __device__ static uint32_t stage_index(uint32_t v) { return v; }

    typedef ChunkKeys Keys;
    __device__ static Keys keys(uint32_t c) { return chunk_keys(c); }
    template <int MT, int ROWS, class C, class XF, class SF>
    __device__ static void dot(const Raw (&r)[ROWS], const C &c, Masks nm, XF x, SF sums, float (&out)[ROWS][MT]) {
        float s_lo[ROWS][MT], s_hi[ROWS][MT];
#pragma unroll
        for (int j = 0; j < ROWS; j++)
#pragma unroll
            for (int t = 0; t < MT; t++) s_lo[j][t] = s_hi[j][t] = 0.f;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            uint32_t lo[ROWS], hi[ROWS];
#pragma unroll
            for (int j = 0; j < ROWS; j++) {
                const uint32_t word = word_of(e < 4 ? r[j].q0 : r[j].q1, e & 3);
                lo[j] = word & nm.lo;
                hi[j] = word & nm.hi;  // 16 q, the sixteenth is in the scale
            }
#pragma unroll
            for (int t = 0; t < MT; t++) {
                const float4 xl = x(t, e), xh = x(t, 8 + e);
#pragma unroll
                for (int j = 0; j < ROWS; j++) {
                    s_lo[j][t] = dot_bytes(lo[j], xl, s_lo[j][t]);
                    s_hi[j][t] = dot_bytes(hi[j], xh, s_hi[j][t]);
                }
            }
        }
#pragma unroll
        for (int j = 0; j < ROWS; j++) {
            const KScales s = chunk_scales<true>(r[j].h, c);
#pragma unroll
            for (int t = 0; t < MT; t++) {
                float v = s.d1 * s_lo[j][t];
                v = fmaf(-s.m1, sums(t, 0), v);
                v = fmaf(s.d2, s_hi[j][t], v);
                v = fmaf(-s.m2, sums(t, 1), v);
                out[j][t] = v;
            }
        }
    }
};

// Q5_K: 176-byte blocks (header vector; qh[32]; qs[128] as Q4_K's nibbles).
// Weight l of sub-block 2c takes bit 2c of qh[l] as its fifth bit, weight l of
// sub-block 2c + 1 bit 2c + 1 (src/ref/tensor.zig:118-137). Task = chunk.
struct KQ5 {
    static constexpr uint32_t BLOCK_BYTES = 176;
    static constexpr int NSUM = 2;
    static constexpr int STAGE2 = 0, STAGE4 = 4;  // tokens whose inputs are loaded at once
    static constexpr bool ALL4 = true;            // a launch of at most a workgroup a CU stages a pass of four at once
    static constexpr bool DEFER = true;
    static constexpr bool PAIR2 = false;  // a two-token gate / up step with the inputs in registers leaves two waves a SIMD their registers
    static const char *name() { return "matvec_q5_k"; }
    struct Raw {
        uint4 h, b0, b1, q0, q1;
    };
    __device__ static Raw load(const uint8_t *row, uint32_t, uint32_t task) {
        const uint8_t *block = row + (size_t)(task >> 2) * BLOCK_BYTES;
        const uint32_t c = task & 3u;
        Raw r;
        r.h = *reinterpret_cast<const uint4 *>(block);
        r.b0 = *reinterpret_cast<const uint4 *>(block + 16u);
        r.b1 = *reinterpret_cast<const uint4 *>(block + 32u);
        r.q0 = *reinterpret_cast<const uint4 *>(block + 48u + 32u * c);
        r.q1 = *reinterpret_cast<const uint4 *>(block + 64u + 32u * c);
        return r;
    }
    struct Where {
        uint32_t h, q;
    };
    __device__ static Where where(uint32_t base, uint32_t, uint32_t task) {
        const uint32_t block = base + (task >> 2) * BLOCK_BYTES;
        return Where{block, block + 48u + 32u * (task & 3u)};
    }
    __device__ static Where nowhere() { return Where{kNowhere, kNowhere}; }
    __device__ static Raw fetch(__amdgpu_buffer_rsrc_t w, const Where &at) {
        Raw r;
        r.h = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(w, at.h, 0, 0));
        r.b0 = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(w, at.h + 16u, 0, 0));
        r.b1 = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(w, at.h + 32u, 0, 0));
        r.q0 = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(w, at.q, 0, 0));
        r.q1 = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(w, at.q + 16u, 0, 0));
        return r;
    }
    __device__ static uint32_t stage_index(uint32_t v) { return v; }

    typedef ChunkKeys Keys;
    __device__ static Keys keys(uint32_t c) { return chunk_keys(c); }
    template <int MT, int ROWS, class C, class XF, class SF>
    __device__ static void dot(const Raw (&r)[ROWS], const C &c, Masks nm, XF x, SF sums, float (&out)[ROWS][MT]) {
        float s_lo[ROWS][MT], s_hi[ROWS][MT];
#pragma unroll
        for (int j = 0; j < ROWS; j++)
#pragma unroll
            for (int t = 0; t < MT; t++) s_lo[j][t] = s_hi[j][t] = 0.f;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            uint32_t lo[ROWS], hi[ROWS];
#pragma unroll
            for (int j = 0; j < ROWS; j++) {
                const uint32_t word = word_of(e < 4 ? r[j].q0 : r[j].q1, e & 3);
                const uint32_t bits = word_of(e < 4 ? r[j].b0 : r[j].b1, e & 3) >> (2u * chunk_no(c));
                lo[j] = ((bits & nm.one) << 4) | (word & nm.lo);
                hi[j] = (((bits >> 1) & nm.one) << 4) | ((word >> 4) & nm.lo);
            }
#pragma unroll
            for (int t = 0; t < MT; t++) {
                const float4 xl = x(t, e), xh = x(t, 8 + e);
#pragma unroll
                for (int j = 0; j < ROWS; j++) {
                    s_lo[j][t] = dot_bytes(lo[j], xl, s_lo[j][t]);
                    s_hi[j][t] = dot_bytes(hi[j], xh, s_hi[j][t]);
                }
            }
        }
#pragma unroll
        for (int j = 0; j < ROWS; j++) {
            const KScales s = chunk_scales<false>(r[j].h, c);
#pragma unroll
            for (int t = 0; t < MT; t++) {
                float v = s.d1 * s_lo[j][t];
                v = fmaf(-s.m1, sums(t, 0), v);
                v = fmaf(s.d2, s_hi[j][t], v);
                v = fmaf(-s.m2, sums(t, 1), v);
                out[j][t] = v;
            }
        }
    }
};

// Q6_K: blocks padded from 210 to 224 bytes (ql[128], qh[64], sixteen signed
// scales, d; src/ref/tensor.zig:139-160). Task p of a block takes positions
// l = 16 (p % 2) .. + 15 of half n = p / 2: four runs of sixteen weights at
// 128 n + l + {0, 32, 64, 96}, run r from the low (r < 2) or high nibbles of
// ql[64 n + 32 (r % 2) + l] and bits 2r, 2r + 1 of qh[32 n + l], with scale
// 8 n + p % 2 + 2 r; a weight is d * scale * (q - 32).
struct KQ6 {
    static constexpr uint32_t BLOCK_BYTES = 224;
    static constexpr int NSUM = 4;
    static constexpr int STAGE2 = 2, STAGE4 = 1;  // tokens whose inputs are loaded at once
    static constexpr bool ALL4 = true;            // a launch of at most a workgroup a CU stages a pass of four at once
    static constexpr bool DEFER = false;
    static constexpr bool PAIR2 = false;  // a two-token gate / up step with the inputs in registers leaves two waves a SIMD their registers
    static const char *name() { return "matvec_q6_k"; }
    struct Raw {
        uint4 l0, l1, hv;
        uint2 sc;
        uint32_t d;
    };
    __device__ static Raw load(const uint8_t *row, uint32_t, uint32_t task) {
        const uint8_t *block = row + (size_t)(task >> 2) * BLOCK_BYTES;
        const uint32_t n = (task >> 1) & 1u, lh = task & 1u;
        Raw r;
        r.l0 = *reinterpret_cast<const uint4 *>(block + 64u * n + 16u * lh);
        r.l1 = *reinterpret_cast<const uint4 *>(block + 64u * n + 32u + 16u * lh);
        r.hv = *reinterpret_cast<const uint4 *>(block + 128u + 32u * n + 16u * lh);
        r.sc = *reinterpret_cast<const uint2 *>(block + 192u + 8u * n);
        r.d = *reinterpret_cast<const uint32_t *>(block + 208u);
        return r;
    }
    struct Where {
        uint32_t l, h, sc, d;
    };
    __device__ static Where where(uint32_t base, uint32_t, uint32_t task) {
        const uint32_t block = base + (task >> 2) * BLOCK_BYTES, n = (task >> 1) & 1u, lh = task & 1u;
        return Where{block + 64u * n + 16u * lh, block + 128u + 32u * n + 16u * lh, block + 192u + 8u * n, block + 208u};
    }
    __device__ static Where nowhere() { return Where{kNowhere, kNowhere, kNowhere, kNowhere}; }
    __device__ static Raw fetch(__amdgpu_buffer_rsrc_t w, const Where &at) {
        Raw r;
        r.l0 = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(w, at.l, 0, 0));
        r.l1 = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(w, at.l + 32u, 0, 0));
        r.hv = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(w, at.h, 0, 0));
        r.sc = __builtin_bit_cast(uint2, __builtin_amdgcn_raw_buffer_load_b64(w, at.sc, 0, 0));
        r.d = __builtin_amdgcn_raw_buffer_load_b32(w, at.d, 0, 0);
        return r;
    }
    // Vector v of a row (inputs 4v ..) is vector q of run r of task 4 blk + 2 n + lh.
    __device__ static uint32_t stage_index(uint32_t v) {
        const uint32_t blk = v >> 6, n = (v >> 5) & 1u, run = (v >> 3) & 3u, lh = (v >> 2) & 1u, q = v & 3u;
        return 64u * blk + 32u * n + 16u * lh + 4u * run + q;
    }

    typedef uint32_t Keys;
    __device__ static Keys keys(uint32_t c) { return c; }
    template <int MT, int ROWS, class XF, class SF>
    __device__ static void dot(const Raw (&r)[ROWS], uint32_t p, Masks nm, XF x, SF sums, float (&out)[ROWS][MT]) {
        float s[ROWS][MT][4];
#pragma unroll
        for (int j = 0; j < ROWS; j++)
#pragma unroll
            for (int t = 0; t < MT; t++)
#pragma unroll
                for (int run = 0; run < 4; run++) s[j][t][run] = 0.f;
#pragma unroll
        for (int run = 0; run < 4; run++) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                uint32_t q[ROWS];
#pragma unroll
                for (int j = 0; j < ROWS; j++) {
                    const uint32_t lw = word_of(run & 1 ? r[j].l1 : r[j].l0, i);
                    const uint32_t nib = run < 2 ? lw & nm.lo : (lw >> 4) & nm.lo;
                    const uint32_t two = (word_of(r[j].hv, i) >> (2 * run)) & nm.two;
                    q[j] = (two << 4) | nib;
                }
#pragma unroll
                for (int t = 0; t < MT; t++) {
                    const float4 xv = x(t, 4 * run + i);
#pragma unroll
                    for (int j = 0; j < ROWS; j++) s[j][t][run] = dot_bytes(q[j], xv, s[j][t][run]);
                }
            }
        }
        const uint32_t lh = p & 1u;
#pragma unroll
        for (int j = 0; j < ROWS; j++) {
            const float d = half_bits_to_float(r[j].d & 0xffffu);
            // Scales lh, lh + 2 of the half's eight are bytes lh, lh + 2 of sc.x; lh + 4, lh + 6 of sc.y.
            const uint32_t s01 = r[j].sc.x >> (8u * lh), s23 = r[j].sc.y >> (8u * lh);
            const float scale[4] = {d * (float)(int8_t)(s01 & 0xffu), d * (float)(int8_t)((s01 >> 16) & 0xffu),
                                    d * (float)(int8_t)(s23 & 0xffu), d * (float)(int8_t)((s23 >> 16) & 0xffu)};
#pragma unroll
            for (int t = 0; t < MT; t++) {
                float v = 0.f;
#pragma unroll
                for (int run = 0; run < 4; run++) v = fmaf(scale[run], fmaf(-32.f, sums(t, run), s[j][t][run]), v);
                out[j][t] = v;
            }
        }
    }
};

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
    // (one instruction each: the rows the mask leaves out keep their value, where update_dpp's
    // form adds a zero to it; the segments' last lanes, which hold the totals, are in rows the
    // masks name. The s_nop covers the two wait states between a vector write and a DPP read.)
    if (seg_log2 >= 5) asm("s_nop 1\n\tv_add_f32_dpp %0, %0, %0 row_bcast:15 row_mask:0xa" : "+v"(v));  // into rows 1 and 3
    if (seg_log2 >= 6) asm("s_nop 1\n\tv_add_f32_dpp %0, %0, %0 row_bcast:31 row_mask:0xc" : "+v"(v));  // into rows 2 and 3
    return v;
}

// Floats per task in the padded LDS copy: 64 inputs and one vector of padding,
// so lanes reading the same offset of consecutive tasks hit different banks.
constexpr uint32_t kTaskStride = 68;

struct KArgs {
    MvArgs a;
    uint32_t t0;        // first token of this pass
    uint32_t mt;        // tokens in this pass (<= MT)
    uint32_t seg_log2;  // lanes per row: 4, 5 or 6
    uint32_t tasks;     // k / 64
    Masks nm;
};

// STG: tokens whose inputs are loaded at once ahead of the weights (0: none, staged by stage_token).
template <class P, int MT, bool PAIR, int STG>
__global__ __launch_bounds__(256) void matvec_quant_kernel(KArgs q) {
    const MvArgs &a = q.a;
    extern __shared__ float4 lds4[];
    __shared__ float red[16];  // [token of those loaded at once][wave]
    constexpr int NSUM = P::NSUM, RUN = 64 / NSUM;
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t tasks = q.tasks;
    const uint32_t tok_stride4 = tasks * (kTaskStride / 4u);  // float4s per token
    float *sums_lds = reinterpret_cast<float *>(lds4 + (size_t)MT * tok_stride4);

    // Rows a pass takes: the gate and up rows of an output, or two outputs so
    // that one read of the inputs from LDS serves both.
    constexpr int kRows = 2;
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
    auto load_at = [&](const Cursor &c, typename P::Raw (&dst)[kRows]) {
        const uint32_t task = tsub + c.i * seg;
        const uint32_t tk = task < tasks ? task : 0u;
        dst[0] = P::load(a.w + (size_t)c.ra * a.row_bytes, a.k, tk);
        if (kRows == 2) dst[kRows - 1] = P::load(a.w + (size_t)c.rb * a.row_bytes, a.k, tk);
    };

    // Weights do not depend on the inputs: start loading the first positions
    // before anything else, so the stream is already flowing while the inputs
    // are fetched. kDepth positions stay in flight ahead of the one multiplied
    // (deeper queues cost registers, hence occupancy, and measured no faster).
    constexpr int kDepth = 1;
    // Rows of up to 4096 weights: the tokens' inputs are loaded first (up to four vectors a
    // thread and token), all of them at once: loads complete in order within a wave, so behind
    // the weights they would wait for them, and token after token each would wait for a trip
    // to memory of its own.
    // How many tokens' vectors are in flight at once (STG) is the launch's choice: each token
    // more raises the register count of the whole kernel, and past 256 the multiply loses its
    // second wave a SIMD, which a large matrix pays for and a small one does not.
    constexpr int TG = STG > 0 ? STG : 1;
    const bool early = STG > 0 && a.k <= 4096u;
    float4 xv[TG][4], gv[4];
    auto load_tokens = [&](int first) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t i = tid + 256u * j;
#pragma unroll
            for (int t = 0; t < TG; t++) {
                const float4 *xrow = reinterpret_cast<const float4 *>(a.x + (size_t)(q.t0 + ((uint32_t)(first + t) < q.mt ? first + t : 0)) * a.xr);
                xv[t][j] = i < a.k / 4u ? xrow[i] : make_float4(0.f, 0.f, 0.f, 0.f);
            }
        }
    };
    if (early) {
        const float4 *nw = reinterpret_cast<const float4 *>(a.norm_w);
        load_tokens(0);
        if (a.flags & FLAG_NORM) {
#pragma unroll
            for (int j = 0; j < 4; j++) gv[j] = tid + 256u * j < a.k / 4u ? nw[tid + 256u * j] : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    }
    typename P::Raw buf[kDepth + 1][kRows];
    Cursor cc{gwave < units ? gwave : 0u, 0u, 0u, 0u, 0u};
    place(cc);
    Cursor lc = cc;
#pragma unroll
    for (int dpt = 0; dpt < kDepth; dpt++) {
        load_at(lc, buf[dpt]);
        advance(lc);
    }

    // Stage the pass's tokens in task order, padded per task (coalesced loads;
    // a lane's own 64 inputs are 256 bytes apart from its neighbour's).
    if (early) {
        // The arithmetic of stage_token on the vectors already loaded, in the same order, the
        // tokens' sums of squares meeting in LDS together.
        const uint32_t k4 = a.k / 4u;
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
                if (first + t >= MT) continue;  // (a last group of fewer tokens than are loaded at once)
                float4 *dst = lds4 + (size_t)(first + t) * tok_stride4;
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
                    if ((uint32_t)(first + t) >= q.mt) v = make_float4(0.f, 0.f, 0.f, 0.f);  // (a pass of fewer tokens than it has room for)
                    const uint32_t p = P::stage_index(i);
                    dst[p + (p >> 4)] = v;
                }
            }
        }
    } else
    for (uint32_t t = 0; t < (uint32_t)MT; t++) {
        float4 *dst = lds4 + (size_t)t * tok_stride4;
        if (t < q.mt) {
            stage_token(a, q.t0 + t, dst, red, [](uint32_t v) { const uint32_t i = P::stage_index(v); return i + (i >> 4); });
        } else {
            for (uint32_t e = tid; e < tok_stride4; e += 256u) dst[e] = make_float4(0.f, 0.f, 0.f, 0.f);
        }
    }
    __syncthreads();
    {
        for (uint32_t idx = tid; idx < (uint32_t)MT * tasks * NSUM; idx += 256u) {
            const uint32_t t = idx / (tasks * NSUM), rem = idx % (tasks * NSUM);
            const float *src = reinterpret_cast<const float *>(lds4 + (size_t)t * tok_stride4) + (rem / NSUM) * kTaskStride + (rem % NSUM) * RUN;
            float sum = 0.f;
#pragma unroll
            for (int e = 0; e < RUN; e++) sum += src[e];
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
    auto compute = [&](const Cursor &c, const typename P::Raw (&cur)[kRows]) {
        const uint32_t task = tsub + c.i * seg;
        if (task < tasks) {
            const uint32_t ch = task & 3u;
            float v[kRows][MT];
            const float4 *xt = lds4 + task * (kTaskStride / 4u);
            const float *st = sums_lds + NSUM * task;
            P::template dot<MT, kRows>(cur, ch, q.nm,
                [&](int t, int vi) { return xt[(size_t)t * tok_stride4 + vi]; },
                [&](int t, int s) { return st[(size_t)t * tasks * NSUM + s]; }, v);
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

// One-token steps over rows of at most 64 tasks, with the lane's inputs in registers, so that
// the loop holds nothing but the weight stream's loads and the multiply. A wave's walk is wave
// uniform here: pass u covers rows u * RPI .. + RPI - 1 (RPI = 64 >> SEG_LOG2 rows side by side
// in the wave), so the pass's position lives in scalar registers, a lane's byte offsets within
// the pass never change (P::Where, computed once), and a pass's loads go through a buffer that
// begins at the pass's first row and ends with the matrix: rows past the end, lanes without a
// task and the loads after a wave's last pass all fall outside it and return zeros, which the
// multiply turns into a sum of zero; no address arithmetic, clamp or branch per lane is left.
// The staging of the inputs, a task's dot product and the lanes' reduction are the code of the
// kernel above, so the results are its bits.
// Passes whose loads are in flight ahead of the one multiplied. Measured on 14336 x 4096 Q4_K
// (7.9 us with one): two or three passes ahead 8.6 / 9.8 us, and no better with fewer workgroups;
// two passes asked for before the inputs are staged (instead of one) 8.7 us; the first pass
// asked for only once the inputs have arrived 8.0 us.
constexpr int kRowDepth = 1;
template <class P, int MT, bool PAIR, int SEG_LOG2>
__global__ __launch_bounds__(256) void matvec_quant_row_kernel(KArgs q) {
    const MvArgs &a = q.a;
    extern __shared__ float4 lds4[];
    __shared__ float red[4 * MT];
    constexpr int NSUM = P::NSUM, RUN = 64 / NSUM, kRows = PAIR ? 2 : 1;
    constexpr uint32_t SEG = 1u << SEG_LOG2, RPI = 64u >> SEG_LOG2;
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t tasks = q.tasks, k4 = a.k / 4u;
    const uint32_t tok_stride4 = tasks * (kTaskStride / 4u);  // float4s per token
    const uint32_t tsub = lane & (SEG - 1u), rsub = lane >> SEG_LOG2;
    const uint32_t units = (a.rows + RPI - 1u) / RPI;
    const uint32_t gwave = blockIdx.x * 4u + (uint32_t)__builtin_amdgcn_readfirstlane((int)wave), nwaves = gridDim.x * 4u;

    // The tokens' inputs (and norm weights) are asked for first, then the first rows: loads
    // complete in order within a wave.
    const float4 *nw = reinterpret_cast<const float4 *>(a.norm_w);
    float4 xv[MT][4], gv[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const uint32_t i = tid + 256u * j;
#pragma unroll
        for (int t = 0; t < MT; t++) {
            const float4 *xrow = reinterpret_cast<const float4 *>(a.x + (size_t)(q.t0 + t) * a.xr);
            xv[t][j] = i < k4 ? xrow[i] : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    }
    if (a.flags & FLAG_NORM) {
#pragma unroll
        for (int j = 0; j < 4; j++) gv[j] = tid + 256u * j < k4 ? nw[tid + 256u * j] : make_float4(0.f, 0.f, 0.f, 0.f);
    }

    const typename P::Where at = tsub < tasks ? P::where(rsub * a.row_bytes, a.k, tsub) : P::nowhere();
    const uint64_t span = (uint64_t)a.rows * a.row_bytes;  // bytes of the rows covered (and of their up rows)
    const uint64_t pass_bytes = (uint64_t)RPI * a.row_bytes;
    // Pass u's rows, and with PAIR the up rows of its outputs.
    auto fetch = [&](uint32_t u, typename P::Raw (&dst)[kRows]) __attribute__((always_inline)) {
        const bool live = u < units;
        const uint64_t off = live ? u * pass_bytes : 0u;
        const uint32_t left = live ? (uint32_t)(span - off) : 0u;
        dst[0] = P::fetch(__builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(a.w + off), 0, (int)left, 0x00020000), at);
        if (PAIR) dst[kRows - 1] = P::fetch(__builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(a.w + (size_t)a.half * a.row_bytes + off), 0, (int)left, 0x00020000), at);
        __builtin_amdgcn_sched_barrier(0);  // (the loads stay ahead of the multiply that follows them in the source)
    };
    typename P::Raw buf[kRowDepth + 1][kRows];
#pragma unroll
    for (int dpt = 0; dpt < kRowDepth; dpt++) fetch(gwave + dpt * nwaves, buf[dpt]);

    // stage_token's arithmetic on the vectors already loaded, the tokens' sums of squares
    // meeting in LDS together.
    float scale[MT];
#pragma unroll
    for (int t = 0; t < MT; t++) scale[t] = 1.0f;
    if (a.flags & FLAG_NORM) {
        float ss[MT];
#pragma unroll
        for (int t = 0; t < MT; t++) {
            ss[t] = 0.f;
#pragma unroll
            for (int j = 0; j < 4; j++)
                if (tid + 256u * j < k4) ss[t] += xv[t][j].x * xv[t][j].x + xv[t][j].y * xv[t][j].y + xv[t][j].z * xv[t][j].z + xv[t][j].w * xv[t][j].w;
            ss[t] = wave_sum(ss[t]);
        }
        if (lane == 0) {
#pragma unroll
            for (int t = 0; t < MT; t++) red[4 * t + wave] = ss[t];
        }
        __syncthreads();
#pragma unroll
        for (int t = 0; t < MT; t++) {
            const float total = (red[4 * t] + red[4 * t + 1]) + (red[4 * t + 2] + red[4 * t + 3]);
            scale[t] = 1.0f / sqrtf(total / (float)a.k + a.eps);
        }
    }
#pragma unroll
    for (int t = 0; t < MT; t++) {
        float4 *dst = lds4 + (size_t)t * tok_stride4;
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
            const uint32_t p = P::stage_index(i);
            dst[p + (p >> 4)] = v;
        }
    }
    __syncthreads();
    if (gwave >= units) return;

    // The lane's task's inputs and their runs' sums, for the whole walk.
    float xr[MT][64], xsum[MT][NSUM];
#pragma unroll
    for (int t = 0; t < MT; t++) {
        const float4 *src = lds4 + (size_t)t * tok_stride4 + (tsub < tasks ? tsub : 0u) * (kTaskStride / 4u);
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const float4 f = src[v];
            xr[t][4 * v] = f.x; xr[t][4 * v + 1] = f.y; xr[t][4 * v + 2] = f.z; xr[t][4 * v + 3] = f.w;
        }
        // (a lane without a task multiplies zeros by zeros, whatever the inputs hold)
        if (tsub >= tasks) {
#pragma unroll
            for (int e = 0; e < 64; e++) xr[t][e] = 0.f;
        }
#pragma unroll
        for (int s = 0; s < NSUM; s++) {
            xsum[t][s] = 0.f;
#pragma unroll
            for (int e = 0; e < RUN; e++) xsum[t][s] += xr[t][s * RUN + e];
        }
    }
    const Masks nm = q.nm;
    const typename P::Keys ch = P::keys(tsub & 3u);
    const bool accumulate = (a.flags & FLAG_ACCUMULATE) != 0;
    auto out_at = [&](int t, uint32_t j) { return (size_t)(q.t0 + t) * a.out_stride + a.col0 + j; };

    // Whole-wave rows (SEG = 64) of a format with DEFER keep their finished sums in the lane of
    // their number (the gate's and the up row's apart) and are finished and stored together,
    // 64 outputs at a time: stores between the loads of the stream cost more than their bytes,
    // and the activation runs once for 64 outputs instead of once a row.
    constexpr bool kKeep = P::DEFER && SEG == 64u;
    float kept0[MT], kept1[MT];
#pragma unroll
    for (int t = 0; t < MT; t++) kept0[t] = kept1[t] = 0.f;
    uint32_t nkept = 0, kept_first = gwave;
    auto flush_kept = [&]() __attribute__((always_inline)) {
        const uint32_t j = kept_first + lane * nwaves;
        if (lane < nkept && j < a.rows) {
#pragma unroll
            for (int t = 0; t < MT; t++) {
                float r = PAIR ? silu_f(kept0[t]) * kept1[t] : kept0[t];
                if (accumulate) r += a.out[out_at(t, j)];
                a.out[out_at(t, j)] = r;
            }
        }
        kept_first += nkept * nwaves;
        nkept = 0;
    };
    auto multiply = [&](uint32_t u, const typename P::Raw (&rows)[kRows]) __attribute__((always_inline)) {
        // (a row at a time: with the inputs in registers two rows share nothing, and one row's
        // sums and words are fewer registers than two rows')
        float v[kRows][MT];
#pragma unroll
        for (int j = 0; j < kRows; j++) {
            const typename P::Raw(&one)[1] = reinterpret_cast<const typename P::Raw(&)[1]>(rows[j]);
            float vj[1][MT];
            P::template dot<MT, 1>(one, ch, nm,
                [&](int t, int vi) { return make_float4(xr[t][4 * vi], xr[t][4 * vi + 1], xr[t][4 * vi + 2], xr[t][4 * vi + 3]); },
                [&](int t, int s) { return xsum[t][s]; }, vj);
#pragma unroll
            for (int t = 0; t < MT; t++) v[j][t] = vj[0][t];
        }
#pragma unroll
        for (int t = 0; t < MT; t++) {
            // (0 + v: matvec_quant_kernel adds a lane's tasks to a sum that starts at zero)
            const float s0 = segment_sum(0.f + v[0][t], SEG_LOG2);
            const float s1 = PAIR ? segment_sum(0.f + v[kRows - 1][t], SEG_LOG2) : 0.f;
            if (kKeep) {
                const float t0 = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(s0), 63));
                kept0[t] = lane == nkept ? t0 : kept0[t];
                if (PAIR) {
                    const float t1 = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(s1), 63));
                    kept1[t] = lane == nkept ? t1 : kept1[t];
                }
            } else {
                const uint32_t j = u * RPI + rsub;
                if (tsub == SEG - 1u && j < a.rows) {
                    float r = PAIR ? silu_f(s0) * s1 : s0;
                    if (accumulate) r += a.out[out_at(t, j)];
                    a.out[out_at(t, j)] = r;
                }
            }
        }
        if (kKeep) {
            nkept++;
            if (nkept == 64u) flush_kept();
        }
    };

    // kRowDepth passes' loads stay in flight ahead of the one multiplied; a trip of
    // kRowDepth + 1 passes so that the buffers rotate by name.
    for (uint32_t u = gwave;;) {
        bool done = false;
#pragma unroll
        for (int ph = 0; ph <= kRowDepth; ph++) {
            fetch(u + kRowDepth * nwaves, buf[(ph + kRowDepth) % (kRowDepth + 1)]);
            multiply(u, buf[ph]);
            u += nwaves;
            if (u >= units) {
                done = true;
                break;
            }
        }
        if (done) break;
    }
    if (kKeep) flush_kept();
}

// Steps of several tokens over rows too long for the tokens' inputs to fit the workgroup's LDS
// together (k above ~4800 for four tokens, ~9600 for two; the FFN-down shapes): the kernel
// above would take such a step token by token, reading the weights once for each. Here a
// workgroup of eight waves takes a batch of rows (a unit a wave) through the row tile by tile,
// a tile being the 64 tasks of one step of the lanes' walk (4096 weights): the tile's inputs of
// all the pass's tokens are staged, every wave multiplies its rows' slice of the tile, and the
// sums stay in registers until the row ends. The next tile's inputs and weights are asked for
// before the current tile is multiplied: the weights wait in registers, the inputs land in LDS
// as they are (wave-wide direct loads: no registers, which the multiply has none to spare) and
// are normalised, activated and put in task order from there. A lane adds its tasks in the
// order of the kernel above, and a task's dot product and the lanes' reduction are the same
// code: the same bits. The inputs are staged once a batch (from L2: 4 B x k x tokens for
// sixteen rows), the weights are read once.
typedef __attribute__((address_space(3))) void *long_lds_ptr;
template <class P, int MT, bool PAIR>
__global__ __launch_bounds__(512) void matvec_quant_long_kernel(KArgs q) {
    const MvArgs &a = q.a;
    extern __shared__ float4 lds4[];  // [token][tile in task order, padded]; the runs' sums; [token][tile as loaded]
    __shared__ float red[4 * MT];
    constexpr int NSUM = P::NSUM, RUN = 64 / NSUM, kRows = 2;
    constexpr uint32_t tile4 = 64u * (kTaskStride / 4u);  // float4s of one token's tile
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t tasks = q.tasks, k4 = a.k / 4u, tiles = (tasks + 63u) / 64u;
    float *sums_lds = reinterpret_cast<float *>(lds4 + (size_t)MT * tile4);  // [token][task of the tile][run]
    float4 *raw4 = lds4 + (size_t)MT * tile4 + MT * 16u * NSUM;              // [token][1024 vectors]
    const Masks nm = q.nm;
    const uint32_t per_unit = PAIR ? 1u : 2u;
    const uint32_t units = (a.rows + per_unit - 1u) / per_unit;
    const uint32_t batches = (units + 7u) / 8u;
    const bool norm = (a.flags & FLAG_NORM) != 0;
    const float4 *nw = reinterpret_cast<const float4 *>(a.norm_w);

    // The RMSNorm prologue's scales (src/kernels/matvec_quant.wgsl.hbs:73-89), summed as
    // stage_token sums them: by 256 threads, vector i to thread i % 256, four waves.
    float scale[MT];
#pragma unroll
    for (int t = 0; t < MT; t++) scale[t] = 1.0f;
    if (norm) {
        if (tid < 256u) {
            float ss[MT];
#pragma unroll
            for (int t = 0; t < MT; t++) {
                ss[t] = 0.f;
                if ((uint32_t)t < q.mt) {
                    const float4 *xrow = reinterpret_cast<const float4 *>(a.x + (size_t)(q.t0 + t) * a.xr);
                    for (uint32_t i = tid; i < k4; i += 256u) {
                        const float4 v = xrow[i];
                        ss[t] += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
                    }
                }
                ss[t] = wave_sum(ss[t]);
            }
            if (lane == 0) {
#pragma unroll
                for (int t = 0; t < MT; t++) red[4 * t + wave] = ss[t];
            }
        }
        __syncthreads();
#pragma unroll
        for (int t = 0; t < MT; t++) {
            const float total = (red[4 * t] + red[4 * t + 1]) + (red[4 * t + 2] + red[4 * t + 3]);
            scale[t] = 1.0f / sqrtf(total / (float)a.k + a.eps);
        }
    }

    // A tile's inputs: two vectors a thread and token, from memory straight into LDS (a wave's
    // load lands 64 consecutive vectors; vectors past the row's end land as zeros) ...
    const uint32_t raw0 = (uint32_t)(uintptr_t)raw4;
    auto fetch_inputs = [&](uint32_t i) __attribute__((always_inline)) {
#pragma unroll
        for (int t = 0; t < MT; t++) {
            const float *xrow = a.x + (size_t)(q.t0 + ((uint32_t)t < q.mt ? t : 0)) * a.xr;
            const __amdgpu_buffer_rsrc_t xbuf = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(xrow), 0, (int)(a.k * 4u), 0x00020000);
#pragma unroll
            for (int j = 0; j < 2; j++) {
                uint32_t dst = raw0 + 16u * ((uint32_t)t * 1024u + 512u * j + 64u * __builtin_amdgcn_readfirstlane(wave));
                asm volatile("" : "+s"(dst));
                __builtin_amdgcn_raw_ptr_buffer_load_lds(xbuf, (long_lds_ptr)(uintptr_t)dst, 16, 16u * (1024u * i + tid + 512u * j), 0, 0, 0);
            }
        }
    };
    // ... and, normalised and activated as the step asks, into LDS in task order, padded per
    // task as above; then the runs' input sums, added in the order of the kernel above.
    auto stage_inputs = [&](uint32_t i) __attribute__((always_inline)) {
#pragma unroll
        for (int t = 0; t < MT; t++) {
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const uint32_t gi = 1024u * i + tid + 512u * j;
                if (gi >= k4) continue;
                float4 v = raw4[(size_t)t * 1024u + tid + 512u * j];
                if (norm) {
                    const float4 g = nw[gi];
                    v.x = v.x * scale[t] * g.x; v.y = v.y * scale[t] * g.y;
                    v.z = v.z * scale[t] * g.z; v.w = v.w * scale[t] * g.w;
                }
                if (a.act_div > 0.f) {
                    v.x = silu_f(v.x / a.act_div); v.y = silu_f(v.y / a.act_div);
                    v.z = silu_f(v.z / a.act_div); v.w = silu_f(v.w / a.act_div);
                }
                if ((uint32_t)t >= q.mt) v = make_float4(0.f, 0.f, 0.f, 0.f);  // (a pass of fewer tokens than it has room for)
                const uint32_t p = P::stage_index(gi) - 1024u * i;
                lds4[(size_t)t * tile4 + p + (p >> 4)] = v;
            }
        }
        __syncthreads();
        const uint32_t live = tasks - 64u * i < 64u ? tasks - 64u * i : 64u;  // tasks of this tile
        for (uint32_t idx = tid; idx < (uint32_t)MT * 64u * NSUM; idx += 512u) {
            const uint32_t t = idx / (64u * NSUM), rem = idx % (64u * NSUM);
            if (rem / NSUM >= live) continue;
            const float *src = reinterpret_cast<const float *>(lds4 + (size_t)t * tile4) + (rem / NSUM) * kTaskStride + (rem % NSUM) * RUN;
            float sum = 0.f;
#pragma unroll
            for (int e = 0; e < RUN; e++) sum += src[e];
            sums_lds[idx] = sum;
        }
        __syncthreads();
    };

    for (uint32_t batch = blockIdx.x; batch < batches; batch += gridDim.x) {
        // The wave's unit: outputs j0 (and j0 + 1), or the gate row j0 and the up row half + j0.
        // A unit or row past the end is clamped for the loads and skipped at the store.
        const uint32_t unit = batch * 8u + wave;
        const bool there = unit < units;
        const uint32_t u = there ? unit : units - 1u;
        const uint32_t j0 = PAIR ? u : 2u * u;
        const uint32_t ra = j0, rb = PAIR ? a.half + j0 : (j0 + 1u < a.rows ? j0 + 1u : j0);
        float acc[kRows][MT];
#pragma unroll
        for (int j = 0; j < kRows; j++)
#pragma unroll
            for (int t = 0; t < MT; t++) acc[j][t] = 0.f;
        typename P::Raw cur[kRows], next[kRows];
        auto load_tile = [&](uint32_t i, typename P::Raw (&dst)[kRows]) __attribute__((always_inline)) {
            const uint32_t task = lane + 64u * i, tk = task < tasks ? task : 0u;
            dst[0] = P::load(a.w + (size_t)ra * a.row_bytes, a.k, tk);
            dst[1] = P::load(a.w + (size_t)rb * a.row_bytes, a.k, tk);
        };
        __syncthreads();  // nobody still reads the batch before's last tile
        fetch_inputs(0);
        load_tile(0, cur);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();  // every wave's part of the tile has landed
        stage_inputs(0);
        for (uint32_t i = 0; i < tiles; i++) {
            const bool more = i + 1u < tiles;
            if (more) {
                fetch_inputs(i + 1u);
                load_tile(i + 1u, next);
            }
            const uint32_t task = lane + 64u * i;
            if (task < tasks) {
                const float4 *xt = lds4 + lane * (kTaskStride / 4u);
                const float *st = sums_lds + NSUM * lane;
                float v[kRows][MT];
                P::template dot<MT, kRows>(cur, task & 3u, nm,
                    [&](int t, int vi) { return xt[(size_t)t * tile4 + vi]; },
                    [&](int t, int sr) { return st[(size_t)t * 64u * NSUM + sr]; }, v);
#pragma unroll
                for (int j = 0; j < kRows; j++)
#pragma unroll
                    for (int t = 0; t < MT; t++) acc[j][t] += v[j][t];
            }
            if (more) {
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                __syncthreads();  // nobody still reads this tile, and every wave's part of the next has landed
                stage_inputs(i + 1u);
                cur[0] = next[0];
                cur[1] = next[1];
            }
        }
#pragma unroll
        for (int t = 0; t < MT; t++) {
            const float s0 = segment_sum(acc[0][t], 6u), s1 = segment_sum(acc[1][t], 6u);
            if (lane == 63u && there && (uint32_t)t < q.mt && j0 < a.rows) {
                const size_t o = (size_t)(q.t0 + t) * a.out_stride + a.col0 + j0;
                if (PAIR) {
                    float r = silu_f(s0) * s1;
                    if (a.flags & FLAG_ACCUMULATE) r += a.out[o];
                    a.out[o] = r;
                } else {
                    float r = s0;
                    if (a.flags & FLAG_ACCUMULATE) r += a.out[o];
                    a.out[o] = r;
                    if (j0 + 1u < a.rows) {
                        float r1 = s1;
                        if (a.flags & FLAG_ACCUMULATE) r1 += a.out[o + 1];
                        a.out[o + 1] = r1;
                    }
                }
            }
        }
    }
}

template <class P, int MT, bool PAIR>
static zhip_result run_long(const Dispatch &d, const KArgs &q, uint32_t blocks) {
    constexpr uint32_t lds = MT * 64u * kTaskStride * 4u + MT * 64u * P::NSUM * 4u + MT * 16384u;
    static bool configured = false;  // dynamic LDS above 64 KiB needs opting in once
    if (lds > 65536u && !configured) {
        if (hipFuncSetAttribute(reinterpret_cast<const void *>(matvec_quant_long_kernel<P, MT, PAIR>), hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess) {
            (void)hipGetLastError();
            return fail(d, ZHIP_E_GPU, "%s: cannot reserve %u bytes of LDS", P::name(), lds);
        }
        configured = true;
    }
    hipLaunchKernelGGL((matvec_quant_long_kernel<P, MT, PAIR>), dim3(blocks), dim3(512), lds, d.stream, q);
    return check_launch(d, P::name());
}

// One-token steps over rows of 65 .. 512 tasks (k above 4096, up to 32768: the FFN-down shapes).
// matvec_quant_kernel walks such a row with one wave, a lane taking a task of every 64-task
// slice in turn with its inputs read from LDS each time. Here a slice is a wave's for the whole
// launch, so the lane's 64 inputs stay in registers as in the short-row case: the waves of a
// group (one a slice: two, three or four) multiply the same rows, R at a time, each its own
// slice, leave the lanes' partial sums in LDS, and behind one barrier the group's waves add
// them, each for its share of the R rows, in the order of the slices, which is the order in
// which the lane of matvec_quant_kernel adds its tasks; the lanes' reduction is the same code.
// The same bits, and the arithmetic of a short row per weight.
//
// The walk is matvec_quant_row_kernel's: a workgroup of NW waves (a multiple of the slices)
// stages the token once for all its groups, a unit's position lives in scalar registers and
// its loads go through a buffer that is the unit's row (a unit past the end, or a lane without
// a task, loads zeros). What the outputs hold, for a step that accumulates, is asked for before
// the round's loads: loads complete in order within a wave, so behind them it would wait for
// rows of the next round.
// K4: the most vectors of four inputs a token has (4096: k <= 16384; 8192: k <= 32768).
template <class P, int MT, bool PAIR, int R, int NW, int K4 = 4096>
__global__ __launch_bounds__(64 * NW) void matvec_quant_slices_kernel(KArgs q) {
    const MvArgs &a = q.a;
    extern __shared__ float4 lds4[];  // the tokens in task order, padded per task; then the partial sums [parity][group][unit of the round][slice][row][token][lane]
    __shared__ float red[4 * MT];
    constexpr int NSUM = P::NSUM, RUN = 64 / NSUM, kRows = PAIR ? 2 : 1;
    constexpr uint32_t THREADS = 64u * NW;
    constexpr int XV = (K4 + THREADS - 1) / THREADS;  // vectors of a token a thread stages
    static_assert(R % 2 == 0, "the buffers alternate by name");
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const uint32_t tasks = q.tasks, slices = (tasks + 63u) / 64u, k4 = a.k / 4u;
    const uint32_t tok_stride4 = tasks * (kTaskStride / 4u);  // float4s per token
    const uint32_t groups_here = (uint32_t)NW / slices;
    const uint32_t grp = wave / slices, slice = wave % slices;
    const uint32_t group = blockIdx.x * groups_here + grp, groups = gridDim.x * groups_here;
    const uint32_t units = a.rows;  // a unit: an output (its row, or its gate row and up row)
    const uint32_t task = lane + 64u * slice;
    const bool active = task < tasks;
    const bool norm = (a.flags & FLAG_NORM) != 0, accumulate = (a.flags & FLAG_ACCUMULATE) != 0;
    const float4 *nw = reinterpret_cast<const float4 *>(a.norm_w);
    auto token_row = [&](int t) { return reinterpret_cast<const float4 *>(a.x + (size_t)(q.t0 + t) * a.xr); };

    // Unit n of the group's walk: R consecutive units a round, the groups' rounds interleaved.
    auto unit_of = [&](uint32_t n) { return ((n / R) * groups + group) * R + n % R; };
    const uint32_t rounds = (units + groups * R - 1u) / (groups * R);  // the same for every group: the barriers below are the workgroup's
    const typename P::Where at = active ? P::where(0u, a.k, task) : P::nowhere();
    auto fetch = [&](uint32_t n, typename P::Raw (&dst)[kRows]) __attribute__((always_inline)) {
        const uint32_t u = unit_of(n);
        const bool live = u < units;
        const uint64_t off = live ? (uint64_t)u * a.row_bytes : 0u;
        const uint32_t left = live ? a.row_bytes : 0u;
        dst[0] = P::fetch(__builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(a.w + off), 0, (int)left, 0x00020000), at);
        if (PAIR) dst[kRows - 1] = P::fetch(__builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(a.w + (size_t)a.half * a.row_bytes + off), 0, (int)left, 0x00020000), at);
        __builtin_amdgcn_sched_barrier(0);  // (the loads stay ahead of the multiply that follows them in the source)
    };
    typename P::Raw cur[kRows], nxt[kRows];

    // A token at a time: its inputs first, then (with the first token) the first rows: loads
    // complete in order within a wave. stage_token's arithmetic: the RMSNorm sum by the first
    // 256 threads, vector i by thread i % 256 and the four waves' sums in order; then every
    // thread stages the vectors it loaded.
#pragma unroll
    for (int t = 0; t < MT; t++) {
        const float4 *xrow = token_row(t);
        float4 xv[XV], gv[XV];
#pragma unroll
        for (int j = 0; j < XV; j++) {
            const uint32_t i = tid + THREADS * j;
            xv[j] = i < k4 ? xrow[i] : make_float4(0.f, 0.f, 0.f, 0.f);
            if (norm) gv[j] = i < k4 ? nw[i] : make_float4(0.f, 0.f, 0.f, 0.f);
        }
        if (t == 0) fetch(0, cur);
        float scale = 1.0f;
        if (norm) {
            if (tid < 256u) {
                float ss = 0.f;
#pragma unroll 4
                for (uint32_t i = tid; i < k4; i += 256u) {
                    const float4 v = xrow[i];
                    ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
                }
                ss = wave_sum(ss);
                if (lane == 0) red[4 * t + wave] = ss;
            }
            __syncthreads();
            const float total = (red[4 * t] + red[4 * t + 1]) + (red[4 * t + 2] + red[4 * t + 3]);
            scale = 1.0f / sqrtf(total / (float)a.k + a.eps);
        }
        float4 *dst = lds4 + (size_t)t * tok_stride4;
#pragma unroll
        for (int j = 0; j < XV; j++) {
            const uint32_t i = tid + THREADS * j;
            if (i >= k4) continue;
            float4 v = xv[j];
            if (norm) {
                v.x = v.x * scale * gv[j].x; v.y = v.y * scale * gv[j].y;
                v.z = v.z * scale * gv[j].z; v.w = v.w * scale * gv[j].w;
            }
            if (a.act_div > 0.f) {
                v.x = silu_f(v.x / a.act_div); v.y = silu_f(v.y / a.act_div);
                v.z = silu_f(v.z / a.act_div); v.w = silu_f(v.w / a.act_div);
            }
            const uint32_t p = P::stage_index(i);
            dst[p + (p >> 4)] = v;
        }
    }
    __syncthreads();

    float xr[MT][64], xsum[MT][NSUM];
#pragma unroll
    for (int t = 0; t < MT; t++) {
        const float4 *src = lds4 + (size_t)t * tok_stride4 + (active ? task : 0u) * (kTaskStride / 4u);
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const float4 f = src[v];
            xr[t][4 * v] = f.x; xr[t][4 * v + 1] = f.y; xr[t][4 * v + 2] = f.z; xr[t][4 * v + 3] = f.w;
        }
        if (!active) {
#pragma unroll
            for (int e = 0; e < 64; e++) xr[t][e] = 0.f;
        }
#pragma unroll
        for (int sr = 0; sr < NSUM; sr++) {
            xsum[t][sr] = 0.f;
#pragma unroll
            for (int e = 0; e < RUN; e++) xsum[t][sr] += xr[t][sr * RUN + e];
        }
    }
    const Masks nm = q.nm;
    const typename P::Keys ch = P::keys(task & 3u);
    auto out_at = [&](int t, uint32_t j) { return (size_t)(q.t0 + t) * a.out_stride + a.col0 + j; };
    // (the partial sums lie behind the tokens: no barrier between reading the one and writing the other)
    float *part = reinterpret_cast<float *>(lds4 + (size_t)MT * tok_stride4);
    constexpr uint32_t kMine = 2;  // units of a round a wave finishes, at most: R <= 4 over two or more slices
    constexpr uint32_t kCell = kRows * MT * 64u;  // floats one wave leaves per unit
    auto multiply = [&](const typename P::Raw (&rows)[kRows], float *to) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < kRows; j++) {
            const typename P::Raw(&one)[1] = reinterpret_cast<const typename P::Raw(&)[1]>(rows[j]);
            float vj[1][MT];
            P::template dot<MT, 1>(one, ch, nm,
                [&](int t, int vi) { return make_float4(xr[t][4 * vi], xr[t][4 * vi + 1], xr[t][4 * vi + 2], xr[t][4 * vi + 3]); },
                [&](int t, int sr) { return xsum[t][sr]; }, vj);
#pragma unroll
            for (int t = 0; t < MT; t++) to[(j * MT + t) * 64u + lane] = vj[0][t];
        }
    };

    for (uint32_t round = 0; round < rounds; round++) {
        float *mine = part + (((round & 1u) * groups_here + grp) * R) * slices * kCell;
        // What the outputs hold, for the units this wave will finish: asked for before the
        // round's loads, so that the wait for it is the wait for rows the wave needs anyway.
        float held[kMine][MT];
        if (accumulate) {
#pragma unroll
            for (uint32_t i = 0; i < kMine; i++) {
                const uint32_t r = slice + i * slices, u = unit_of(round * R + r);
#pragma unroll
                for (int t = 0; t < MT; t++) held[i][t] = (lane == 63u && r < (uint32_t)R && u < units) ? a.out[out_at(t, u)] : 0.f;
            }
        }
#pragma unroll
        for (int r = 0; r < R; r++) {
            if (r % 2 == 0) {
                fetch(round * R + r + 1u, nxt);
                multiply(cur, mine + (r * slices + slice) * kCell);
            } else {
                fetch(round * R + r + 1u, cur);
                multiply(nxt, mine + (r * slices + slice) * kCell);
            }
        }
        // (a barrier that leaves the next unit's loads in flight)
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        // The group's waves share the round's units; a unit's slices are added in order, a lane
        // leaving out the slice in which it has no task.
#pragma unroll
        for (uint32_t i = 0; i < kMine; i++) {
            const uint32_t r = slice + i * slices;
            if (r >= (uint32_t)R) break;
            const float *theirs = mine + (r * slices) * kCell;
            const uint32_t u = unit_of(round * R + r);
#pragma unroll
            for (int t = 0; t < MT; t++) {
                float acc[kRows];
#pragma unroll
                for (int j = 0; j < kRows; j++) acc[j] = 0.f;
                for (uint32_t sl = 0; sl < slices; sl++) {
                    if (lane + 64u * sl >= tasks) continue;
#pragma unroll
                    for (int j = 0; j < kRows; j++) acc[j] += theirs[sl * kCell + (j * MT + t) * 64u + lane];
                }
                const float s0 = segment_sum(acc[0], 6u), s1 = PAIR ? segment_sum(acc[kRows - 1], 6u) : 0.f;
                if (lane == 63u && u < units) {
                    float res = PAIR ? silu_f(s0) * s1 : s0;
                    if (accumulate) res += held[i][t];
                    a.out[out_at(t, u)] = res;
                }
            }
        }
        // (the other parity's space is written next; this one again only behind the next barrier)
    }
}

template <class P, int MT, bool PAIR, int R, int NW, int K4 = 4096>
static zhip_result run_slices(const Dispatch &d, const KArgs &q, uint32_t lds, uint32_t blocks) {
    if (!lds_opt_in<matvec_quant_slices_kernel<P, MT, PAIR, R, NW, K4>, 160 * 1024 - 64>()) return fail(d, ZHIP_E_GPU, "%s: cannot reserve %u bytes of LDS", P::name(), lds);
    hipLaunchKernelGGL((matvec_quant_slices_kernel<P, MT, PAIR, R, NW, K4>), dim3(blocks), dim3(64 * NW), lds, d.stream, q);
    return check_launch(d, P::name());
}

template <class P, int MT, bool PAIR>
static zhip_result run_row(const Dispatch &d, const KArgs &q, uint32_t lds, uint32_t blocks) {
    if (lds > 65536u) {
        const bool ok = q.seg_log2 == 4u ? lds_opt_in<matvec_quant_row_kernel<P, MT, PAIR, 4>, 160 * 1024 - 64>()
                      : q.seg_log2 == 5u ? lds_opt_in<matvec_quant_row_kernel<P, MT, PAIR, 5>, 160 * 1024 - 64>()
                                         : lds_opt_in<matvec_quant_row_kernel<P, MT, PAIR, 6>, 160 * 1024 - 64>();
        if (!ok) return fail(d, ZHIP_E_GPU, "%s: cannot reserve %u bytes of LDS", P::name(), lds);
    }
    switch (q.seg_log2) {
    case 4: hipLaunchKernelGGL((matvec_quant_row_kernel<P, MT, PAIR, 4>), dim3(blocks), dim3(256), lds, d.stream, q); break;
    case 5: hipLaunchKernelGGL((matvec_quant_row_kernel<P, MT, PAIR, 5>), dim3(blocks), dim3(256), lds, d.stream, q); break;
    default: hipLaunchKernelGGL((matvec_quant_row_kernel<P, MT, PAIR, 6>), dim3(blocks), dim3(256), lds, d.stream, q); break;
    }
    return check_launch(d, P::name());
}

template <class P, int MT, bool PAIR, int STG>
static zhip_result run_quant(const Dispatch &d, const KArgs &q, uint32_t lds, uint32_t blocks) {
    static bool configured = false;  // dynamic LDS above 64 KiB needs opting in once
    if (lds > 65536u && !configured) {
        if (hipFuncSetAttribute(reinterpret_cast<const void *>(matvec_quant_kernel<P, MT, PAIR, STG>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 64) != hipSuccess) {
            (void)hipGetLastError();
            return fail(d, ZHIP_E_BAD_COMMAND, "%s: k = %u with %d tokens does not fit workgroup memory", P::name(), q.a.k, MT);
        }
        configured = true;
    }
    hipLaunchKernelGGL((matvec_quant_kernel<P, MT, PAIR, STG>), dim3(blocks), dim3(256), lds, d.stream, q);
    return check_launch(d, P::name());
}

// Launches the multiply for validated arguments: one pass per group of up to
// four tokens (a pass of three has kernels of its own: in the four-token ones a quarter of the
// multiply-adds would go to a token that is not there).
template <class P>
static zhip_result launch_quant(const Dispatch &d, const MvArgs &a) {
    KArgs q{};
    q.a = a;
    q.tasks = a.k / 64u;
    q.seg_log2 = q.tasks == 16u ? 4u : q.tasks == 32u ? 5u : 6u;
    q.nm = Masks{0x0f0f0f0fu, 0xf0f0f0f0u, 0x03030303u, 0x01010101u};
    const bool pair = a.flags & FLAG_SILU_PAIR;
    const uint32_t rpi = 64u >> q.seg_log2;
    const uint64_t tok_lds = (uint64_t)q.tasks * kTaskStride * 4u + (uint64_t)q.tasks * P::NSUM * 4u;
    const uint64_t max_lds = 160u * 1024u - 64u;
    if (tok_lds > max_lds) return fail(d, ZHIP_E_BAD_COMMAND, "%s: k = %u does not fit workgroup memory", P::name(), a.k);
    for (uint32_t t0 = 0; t0 < a.m;) {
        uint32_t left = a.m - t0;
        uint32_t mt = left >= 4u ? 4u : left;
        // A step of exactly two tokens over rows of 65 .. 256 tasks keeps both tokens' slices in
        // registers like the one-token step (Q4_K 4096 x 14336: 16.5 us tile by tile).
        if (a.m == 2u && !pair && q.tasks > 64u && q.tasks <= 256u) {
            q.t0 = 0;
            q.mt = 2;
            // (eight waves for two or four slices, six for three: twelve would spill)
            const uint32_t slices = (q.tasks + 63u) / 64u, nw = slices == 3u ? 6u : 8u, groups_here = nw / slices;
            const uint32_t cus = (uint32_t)d.dev->compute_units;
            const uint32_t want = (a.rows + groups_here * 2u - 1u) / (groups_here * 2u);
            const uint32_t blocks = want < cus ? want : cus;
            const uint32_t lds2 = 2u * q.tasks * kTaskStride * 4u + 2u * nw * 2u * 2u * 256u;
            const zhip_result r = nw == 6u ? run_slices<P, 2, false, 2, 6>(d, q, lds2, blocks) : run_slices<P, 2, false, 2, 8>(d, q, lds2, blocks);
            if (r != ZHIP_OK) return r;
            break;
        }
        // Two workgroups a CU must fit their staged tokens in the 160 KB of LDS. Where the
        // pass's tokens do not, the rows are long (64 tasks or more) and the step is taken tile
        // by tile with all of them (matvec_quant_long_kernel).
        if (mt > 1u && mt * tok_lds > 80u * 1024u - 64u && q.tasks >= 64u) {
            q.t0 = t0;
            q.mt = left < mt ? left : mt;
            const uint32_t units = pair ? a.rows : (a.rows + 1u) / 2u;
            const uint32_t cus = (uint32_t)d.dev->compute_units;
            // (a workgroup of eight waves a CU: its registers leave room for no second one)
            const uint32_t batches = (units + 7u) / 8u;
            const uint32_t blocks = batches < cus ? batches : cus;
            zhip_result r;
            if (mt == 2u) r = pair ? run_long<P, 2, true>(d, q, blocks) : run_long<P, 2, false>(d, q, blocks);
            else if (mt == 3u) r = pair ? run_long<P, 3, true>(d, q, blocks) : run_long<P, 3, false>(d, q, blocks);
            else r = pair ? run_long<P, 4, true>(d, q, blocks) : run_long<P, 4, false>(d, q, blocks);
            if (r != ZHIP_OK) return r;
            t0 += q.mt;
            continue;
        }
        while (mt > 1u && mt * tok_lds > 80u * 1024u - 64u) mt = mt == 3u ? 2u : mt >> 1;
        q.t0 = t0;
        q.mt = left < mt ? left : mt;
        const uint32_t lds = (uint32_t)(mt * tok_lds);
        if (a.m == 1u && q.tasks > 64u && q.tasks <= 256u) {
            // Eight waves a workgroup (and CU) for rows of two or four slices, twelve for three.
            // Measured, Q4_K 4096 x 14336: 9.9 us with eight, 10.4 with twelve, 14.6 with sixteen
            // (their registers spill); 4096 x 11008 (three slices): 8.0 us with twelve, 8.9 / 9.3
            // with nine / six. Two or four units a round, whichever leaves fewer empty places in
            // the last round; of equal, four for light units and two for heavy ones (from 3.5 KB
            // a wave and unit: Q8_0 rows, gate / up pairs): Q4_K 9.9 / 10.4 us at four / two,
            // Q3_K 10.1 / 11.5, Q8_0 13.3 / 12.9, a Q4_K gate / up pair over 8192 28.2 / 25.0.
            const uint32_t slices = (q.tasks + 63u) / 64u, nw = slices == 3u ? 12u : 8u, groups_here = nw / slices;
            const uint32_t cus = (uint32_t)d.dev->compute_units;
            const uint32_t want = (a.rows + groups_here * 2u - 1u) / (groups_here * 2u);
            const uint32_t blocks = want < cus ? want : cus;
            const uint32_t groups = blocks * groups_here;
            const uint32_t slots4 = (a.rows + groups * 4u - 1u) / (groups * 4u) * 4u, slots2 = (a.rows + groups * 2u - 1u) / (groups * 2u) * 2u;
            const bool heavy = (uint64_t)a.row_bytes * (pair ? 2u : 1u) / slices >= 3584u;
            const bool two = slots2 < slots4 || (slots2 == slots4 && heavy);
            const uint32_t lds1 = q.tasks * kTaskStride * 4u + 2u * nw * (two ? 2u : 4u) * (pair ? 2u : 1u) * 256u;
            zhip_result r;
            if (nw == 12u) {
                if (pair) r = two ? run_slices<P, 1, true, 2, 12>(d, q, lds1, blocks) : run_slices<P, 1, true, 4, 12>(d, q, lds1, blocks);
                else r = two ? run_slices<P, 1, false, 2, 12>(d, q, lds1, blocks) : run_slices<P, 1, false, 4, 12>(d, q, lds1, blocks);
            } else {
                if (pair) r = two ? run_slices<P, 1, true, 2, 8>(d, q, lds1, blocks) : run_slices<P, 1, true, 4, 8>(d, q, lds1, blocks);
                else r = two ? run_slices<P, 1, false, 2, 8>(d, q, lds1, blocks) : run_slices<P, 1, false, 4, 8>(d, q, lds1, blocks);
            }
            if (r != ZHIP_OK) return r;
            t0 += q.mt;
            continue;
        }
        // One token over rows of 288 .. 512 tasks (k up to 32768: the FFN-down multiplies of the
        // widest models): five to eight slices, a wave each, one group a workgroup and CU, two
        // units a round. Q4_K 8192 x 28672: 29.1 us against 46.4 through the general kernel;
        // 5120 x 25600 22.2 against 32.3; 5120 x 20480 21.3 against 24.9 (Q6_K 25.4 against
        // 31.1). Rows of 257 .. 287 tasks, whose fifth wave would be all but idle, stay with the
        // general kernel (Q4_K 5120 x 17408: 19.5 us there, 20.5 here).
        if (a.m == 1u && !pair && q.tasks >= 288u && q.tasks <= 512u) {
            const uint32_t slices = (q.tasks + 63u) / 64u, cus = (uint32_t)d.dev->compute_units;
            const uint32_t want = (a.rows + 1u) / 2u, blocks = want < cus ? want : cus;
            const uint32_t lds1 = q.tasks * kTaskStride * 4u + 2u * slices * 2u * 256u;
            zhip_result r;
            switch (slices) {
            case 5: r = run_slices<P, 1, false, 2, 5, 8192>(d, q, lds1, blocks); break;
            case 6: r = run_slices<P, 1, false, 2, 6, 8192>(d, q, lds1, blocks); break;
            case 7: r = run_slices<P, 1, false, 2, 7, 8192>(d, q, lds1, blocks); break;
            default: r = run_slices<P, 1, false, 2, 8, 8192>(d, q, lds1, blocks); break;
            }
            if (r != ZHIP_OK) return r;
            t0 += q.mt;
            continue;
        }
        // Steps of one or two tokens over rows of up to 64 tasks keep the lanes' inputs in registers.
        const bool xreg = (a.m == 1u || (a.m == 2u && (!pair || P::PAIR2))) && q.tasks <= 64u;
        const uint32_t per_unit = pair ? rpi : rpi * (xreg ? 1u : 2u);
        const uint32_t units = (a.rows + per_unit - 1u) / per_unit;
        const uint32_t want = (units + 3u) / 4u;
        // Three workgroups a CU measured best for the 4096 x 14336 multiply:
        // more of them repeat the input staging, fewer leave too few loads in flight.
        const uint32_t cap = (uint32_t)d.dev->compute_units * (xreg ? 3u : 2u);
        const uint32_t blocks = want < cap ? want : cap;
        zhip_result r;
        // A launch of at most one workgroup a CU is a chain of trips to memory and has the CU's
        // registers to itself: all of the pass's tokens go in one. With more workgroups a CU the
        // format keeps what leaves the multiply its second wave a SIMD (STAGE2, STAGE4; 4096 x
        // 4096 at four tokens with all at once: Q4_K 12.3 against 9.1 us, Q6_K 13.4 against 10.9).
        const bool small = want <= (uint32_t)d.dev->compute_units;
        if (xreg) {
            // (a pass of the row kernel is a wave's 64 / seg rows, or that many gate / up pairs)
            const uint32_t passes = (a.rows + rpi - 1u) / rpi, row_want = (passes + 3u) / 4u;
            // Workgroups a CU: every one stages the inputs and every wave reads all of them from
            // LDS, so two unless the launch is long (four passes a wave or more at three) and its
            // passes light (up to 3 KB a wave: Q4_K, Q5_K, Q3_K rows without a second row of a
            // pair). 14336 x 4096 at three / two: Q4_K 7.9 / 8.0 us, Q3_K 8.2 / 8.6, Q5_K 9.7 /
            // 9.8, Q6_K 10.9 / 10.8, Q8_0 12.05 / 11.7, gate / up pairs of Q4_K 14.4 / 13.9, of
            // Q5_K 18.3 / 17.2; 4096 x 4096 Q4_K 4.9 / 4.2; 28672 x 2048 Q4_K 8.0 / 9.05.
            const uint32_t cus = (uint32_t)d.dev->compute_units;
            // (two tokens' inputs leave the registers for two waves a SIMD: two workgroups)
            const bool three = a.m == 1u && !pair && (uint64_t)rpi * a.row_bytes <= 3072u && passes >= cus * 48u;
            const uint32_t cap = cus * (three ? 3u : 2u), row_blocks = row_want < cap ? row_want : cap;
            const uint32_t row_lds = a.m * q.tasks * kTaskStride * 4u;
            if (a.m == 1u) r = pair ? run_row<P, 1, true>(d, q, row_lds, row_blocks) : run_row<P, 1, false>(d, q, row_lds, row_blocks);
            else if (pair) r = P::PAIR2 ? run_row<P, 2, P::PAIR2>(d, q, row_lds, row_blocks) : ZHIP_E_GPU;
            else r = run_row<P, 2, false>(d, q, row_lds, row_blocks);
        } else if (mt == 1u) r = pair ? run_quant<P, 1, true, 1>(d, q, lds, blocks) : run_quant<P, 1, false, 1>(d, q, lds, blocks);
        else if (mt == 2u) {
            if (small && P::STAGE2 != 2) r = pair ? run_quant<P, 2, true, 2>(d, q, lds, blocks) : run_quant<P, 2, false, 2>(d, q, lds, blocks);
            else r = pair ? run_quant<P, 2, true, P::STAGE2>(d, q, lds, blocks) : run_quant<P, 2, false, P::STAGE2>(d, q, lds, blocks);
        } else if (mt == 3u) {
            // (three tokens: the four-token pass's choices, at most three loaded at once)
            constexpr int STAGE3 = P::STAGE4 > 3 ? 3 : P::STAGE4;
            if (small && P::ALL4 && STAGE3 != 3) r = pair ? run_quant<P, 3, true, 3>(d, q, lds, blocks) : run_quant<P, 3, false, 3>(d, q, lds, blocks);
            else r = pair ? run_quant<P, 3, true, STAGE3>(d, q, lds, blocks) : run_quant<P, 3, false, STAGE3>(d, q, lds, blocks);
        } else {
            if (small && P::ALL4 && P::STAGE4 != 4) r = pair ? run_quant<P, 4, true, 4>(d, q, lds, blocks) : run_quant<P, 4, false, 4>(d, q, lds, blocks);
            else r = pair ? run_quant<P, 4, true, P::STAGE4>(d, q, lds, blocks) : run_quant<P, 4, false, P::STAGE4>(d, q, lds, blocks);
        }
        if (r != ZHIP_OK) return r;
        t0 += q.mt;
    }
    return ZHIP_OK;
}

// A format's launcher lives in a source file of its own (matvec_quant_q8.hip, ...): the kernels of
// one format take as long to compile as all the rest of the library.
zhip_result launch_matvec_quant_q8(const Dispatch &d, const MvArgs &a);
zhip_result launch_matvec_quant_q3(const Dispatch &d, const MvArgs &a);
zhip_result launch_matvec_quant_q4(const Dispatch &d, const MvArgs &a);
zhip_result launch_matvec_quant_q5(const Dispatch &d, const MvArgs &a);
zhip_result launch_matvec_quant_q6(const Dispatch &d, const MvArgs &a);

}  // namespace zhip
