// Block decoders shared by the decode multiplies and the embedding gathers.
// Each follows its reference decoder's f32 operations one for one, with every
// multiply and subtract rounded on its own (no contraction), so decoded
// weights equal the reference's bit for bit:
//   Q8_0  src/ref/tensor.zig:49-53    y = f32(q) * f32(d)
//   Q3_K  src/ref/tensor.zig:55-92    y = (d * (sc - 32)) * (q - 4 (1 - h))
//   Q4_K  src/ref/tensor.zig:94-116   y = (d * sc) * q - (dmin * m)
//   Q5_K  src/ref/tensor.zig:118-138  y = (d * sc) * (q | h << 4) - (dmin * m)
//   Q6_K  src/ref/tensor.zig:140-160  y = (d * sc) * (q - 32)
//   BF16  src/ref/tensor.zig:36-40    y = bits << 16
// A decoder splits a row into "tasks" of E weights so that consecutive lanes
// load consecutive 16-byte vectors; decode() returns the task's weights, whose
// inputs are RUNS runs of E / RUNS floats at xoff(task, 0 .. RUNS - 1).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace zhip {

__device__ __forceinline__ float half_bits_to_float(uint32_t h) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)h);
}

// The 6-bit scale (x) and min (y) of sub-block j from the 12 scale bytes held
// as three words (src/ref/tensor.zig:94-98).
__device__ __forceinline__ uint2 scale_min_k4(uint32_t s0, uint32_t s1, uint32_t s2, uint32_t j) {
    // Byte j of the 12: word j / 4, shift 8 * (j % 4).
    if (j < 4u) {
        const uint32_t sh = 8u * j;
        return make_uint2((s0 >> sh) & 63u, (s1 >> sh) & 63u);
    }
    const uint32_t sh = 8u * (j - 4u);
    const uint32_t hi = (s2 >> sh) & 0xffu;  // byte j + 4
    const uint32_t a = (s0 >> sh) & 0xffu;   // byte j - 4
    const uint32_t b = (s1 >> sh) & 0xffu;   // byte j
    return make_uint2((hi & 0xFu) | ((a >> 6) << 4), (hi >> 4) | ((b >> 6) << 4));
}

// Q8_0 split rows (src/kernels/quant/q8_0.wgsl:1-16): the row's k values as
// i8, then its k/32 scales as f16, zero padded to 16 bytes.
struct DecQ8_0 {
    static constexpr int RUNS = 2;
    static constexpr int E = 16;
    static constexpr uint32_t BLOCK = 32;
    static constexpr int CHUNK = 8;
    static const char *name() { return "matvec_q8_0"; }
    static uint32_t row_bytes(uint32_t k) { return (k + k / 16u + 15u) & ~15u; }
    __device__ static uint32_t xoff(uint32_t task, int h) { return 16u * task + 8u * h; }
    __device__ static void decode(const uint8_t *row, uint32_t k, uint32_t task, float (&w)[E]) {
        const uint4 q = *reinterpret_cast<const uint4 *>(row + 16u * task);
        const float d = half_bits_to_float(*reinterpret_cast<const uint16_t *>(row + k + 2u * (task >> 1)));
        const uint32_t words[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int32_t v = (int32_t)words[e];
            w[4 * e + 0] = __fmul_rn((float)((v << 24) >> 24), d);
            w[4 * e + 1] = __fmul_rn((float)((v << 16) >> 24), d);
            w[4 * e + 2] = __fmul_rn((float)((v << 8) >> 24), d);
            w[4 * e + 3] = __fmul_rn((float)(v >> 24), d);
        }
    }
};

// Q3_K blocks repacked at load into eight self-contained 16-byte units
// (src/kernels/repack_q3_k.wgsl, src/kernels/quant/q3_k.wgsl): unit s of a
// block holds the 32 weights 32 s .. 32 s + 31 as two words of 2-bit values
// (byte b of word 0: positions b, 4 + b, 8 + b, 12 + b at bit pairs 0, 2, 4,
// 6; word 1: positions 16 + b, ...), a word of third bits (bit e of byte b:
// position 4 e + b), then scale - 32 for positions 0..15 and 16..31 as signed
// bytes and d.
struct DecQ3_K {
    static constexpr int RUNS = 1;
    static constexpr int E = 32;
    static constexpr uint32_t BLOCK = 256;
    static constexpr int CHUNK = 3;
    static const char *name() { return "matvec_q3_k"; }
    static uint32_t row_bytes(uint32_t k) { return k / 256u * 128u; }
    __device__ static uint32_t xoff(uint32_t task, int) { return 32u * task; }
    __device__ static void decode(const uint8_t *row, uint32_t, uint32_t task, float (&w)[E]) {
        const uint4 u = *reinterpret_cast<const uint4 *>(row + 16u * task);
        const float d = half_bits_to_float(u.w >> 16);
        const float dl0 = __fmul_rn(d, (float)(int8_t)(u.w & 0xffu)), dl1 = __fmul_rn(d, (float)(int8_t)((u.w >> 8) & 0xffu));
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const uint32_t lo = (e < 4 ? u.x : u.y) >> (2 * (e & 3));
            const uint32_t hi = u.z >> e;
#pragma unroll
            for (int b = 0; b < 4; b++) {
                const int v = (int)((lo >> (8 * b)) & 3u) + 4 * (int)((hi >> (8 * b)) & 1u) - 4;
                w[4 * e + b] = __fmul_rn(e < 4 ? dl0 : dl1, (float)v);
            }
        }
    }
};

// Q4_K blocks as in the file (144 bytes = nine 16-byte vectors). Task p of a
// block reads qs bytes [16p, 16p + 16): positions l = 16 (p % 2) .. of chunk
// c = p / 2, low nibbles for sub-block 2c, high nibbles for sub-block 2c + 1.
struct DecQ4_K {
    static constexpr int RUNS = 2;
    static constexpr int E = 32;
    static constexpr uint32_t BLOCK = 256;
    static constexpr int CHUNK = 4;  // has its own multiply (matvec_quant.h)
    static const char *name() { return "matvec_q4_k"; }
    static uint32_t row_bytes(uint32_t k) { return k / 256u * 144u; }
    __device__ static uint32_t xoff(uint32_t task, int h) {
        const uint32_t blk = task >> 3, p = task & 7u;
        return blk * 256u + (p >> 1) * 64u + (p & 1u) * 16u + 32u * h;
    }
    __device__ static void decode(const uint8_t *row, uint32_t, uint32_t task, float (&w)[E]) {
        const uint32_t blk = task >> 3, p = task & 7u, c = p >> 1;
        const uint8_t *b = row + (size_t)blk * 144u;
        const uint4 hv = *reinterpret_cast<const uint4 *>(b);
        const uint4 qv = *reinterpret_cast<const uint4 *>(b + 16u + 16u * p);
        const float d = half_bits_to_float(hv.x & 0xffffu);
        const float dmin = half_bits_to_float(hv.x >> 16);
        const uint2 s1 = scale_min_k4(hv.y, hv.z, hv.w, 2u * c);
        const uint2 s2 = scale_min_k4(hv.y, hv.z, hv.w, 2u * c + 1u);
        const float d1 = __fmul_rn(d, (float)s1.x), m1 = __fmul_rn(dmin, (float)s1.y);
        const float d2 = __fmul_rn(d, (float)s2.x), m2 = __fmul_rn(dmin, (float)s2.y);
        const uint32_t words[4] = {qv.x, qv.y, qv.z, qv.w};
#pragma unroll
        for (int e = 0; e < 4; e++) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t byte = (words[e] >> (8 * i)) & 0xffu;
                w[4 * e + i] = __fsub_rn(__fmul_rn(d1, (float)(byte & 0xFu)), m1);
                w[16 + 4 * e + i] = __fsub_rn(__fmul_rn(d2, (float)(byte >> 4)), m2);
            }
        }
    }
};

// Q5_K blocks as in the file (176 bytes = eleven 16-byte vectors: d, dmin and
// the twelve scale bytes; qh[32]; qs[128]). Task p of a block reads qs bytes
// [16p, 16p + 16) and qh bytes [16 (p % 2), + 16): positions l = 16 (p % 2) ..
// of chunk c = p / 2, low nibbles and bit 2c of qh for sub-block 2c, high
// nibbles and bit 2c + 1 for sub-block 2c + 1.
struct DecQ5_K {
    static constexpr int RUNS = 2;
    static constexpr int E = 32;
    static constexpr uint32_t BLOCK = 256;
    static constexpr int CHUNK = 5;
    static const char *name() { return "matvec_q5_k"; }
    static uint32_t row_bytes(uint32_t k) { return k / 256u * 176u; }
    __device__ static uint32_t xoff(uint32_t task, int h) {
        const uint32_t blk = task >> 3, p = task & 7u;
        return blk * 256u + (p >> 1) * 64u + (p & 1u) * 16u + 32u * h;
    }
    __device__ static void decode(const uint8_t *row, uint32_t, uint32_t task, float (&w)[E]) {
        const uint32_t blk = task >> 3, p = task & 7u, c = p >> 1;
        const uint8_t *b = row + (size_t)blk * 176u;
        const uint4 hv = *reinterpret_cast<const uint4 *>(b);
        const uint4 hb = *reinterpret_cast<const uint4 *>(b + 16u + 16u * (p & 1u));
        const uint4 qv = *reinterpret_cast<const uint4 *>(b + 48u + 16u * p);
        const float d = half_bits_to_float(hv.x & 0xffffu);
        const float dmin = half_bits_to_float(hv.x >> 16);
        const uint2 s1 = scale_min_k4(hv.y, hv.z, hv.w, 2u * c);
        const uint2 s2 = scale_min_k4(hv.y, hv.z, hv.w, 2u * c + 1u);
        const float d1 = __fmul_rn(d, (float)s1.x), m1 = __fmul_rn(dmin, (float)s1.y);
        const float d2 = __fmul_rn(d, (float)s2.x), m2 = __fmul_rn(dmin, (float)s2.y);
        const uint32_t words[4] = {qv.x, qv.y, qv.z, qv.w};
        const uint32_t highs[4] = {hb.x, hb.y, hb.z, hb.w};
#pragma unroll
        for (int e = 0; e < 4; e++) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t byte = (words[e] >> (8 * i)) & 0xffu;
                const uint32_t h = ((highs[e] >> (8 * i)) & 0xffu) >> (2u * c);
                w[4 * e + i] = __fsub_rn(__fmul_rn(d1, (float)((byte & 0xFu) + ((h & 1u) << 4))), m1);
                w[16 + 4 * e + i] = __fsub_rn(__fmul_rn(d2, (float)((byte >> 4) + ((h & 2u) << 3))), m2);
            }
        }
    }
};

// Q6_K blocks padded from 210 to 224 bytes (src/kernels/kernels.zig:144-151):
// ql[128], qh[64], sixteen signed scales, d. Task p of a block (half n = p / 2,
// positions l = 16 (p % 2) .. + 15 of that half) reads ql[64n + l], ql[64n + 32 + l]
// and qh[32n + l], one 16-byte vector each, and decodes 64 weights: four runs
// of 16 at 128 n + l + {0, 32, 64, 96}, with scales 8 n + p % 2 + {0, 2, 4, 6}.
struct DecQ6_K {
    static constexpr int RUNS = 4;
    static constexpr int E = 64;
    static constexpr uint32_t BLOCK = 256;
    static constexpr int CHUNK = 6;
    static const char *name() { return "matvec_q6_k"; }
    static uint32_t row_bytes(uint32_t k) { return k / 256u * 224u; }
    __device__ static uint32_t xoff(uint32_t task, int h) {
        const uint32_t blk = task >> 2, p = task & 3u;
        return blk * 256u + (p >> 1) * 128u + (p & 1u) * 16u + 32u * h;
    }
    __device__ static void decode(const uint8_t *row, uint32_t, uint32_t task, float (&w)[E]) {
        const uint32_t blk = task >> 2, p = task & 3u, n = p >> 1, lh = p & 1u;
        const uint8_t *b = row + (size_t)blk * 224u;
        const uint4 l0 = *reinterpret_cast<const uint4 *>(b + 64u * n + 16u * lh);
        const uint4 l1 = *reinterpret_cast<const uint4 *>(b + 64u * n + 32u + 16u * lh);
        const uint4 hv = *reinterpret_cast<const uint4 *>(b + 128u + 32u * n + 16u * lh);
        const uint2 sc = *reinterpret_cast<const uint2 *>(b + 192u + 8u * n);
        const float d = half_bits_to_float(*reinterpret_cast<const uint16_t *>(b + 208u));
        // Scales lh, lh + 2 of the half's eight are bytes lh, lh + 2 of sc.x; lh + 4, lh + 6 of sc.y.
        const uint32_t s01 = sc.x >> (8u * lh), s23 = sc.y >> (8u * lh);
        const float t1 = __fmul_rn(d, (float)(int8_t)(s01 & 0xffu)), t2 = __fmul_rn(d, (float)(int8_t)((s01 >> 16) & 0xffu));
        const float t3 = __fmul_rn(d, (float)(int8_t)(s23 & 0xffu)), t4 = __fmul_rn(d, (float)(int8_t)((s23 >> 16) & 0xffu));
        const uint32_t a[4] = {l0.x, l0.y, l0.z, l0.w}, c[4] = {l1.x, l1.y, l1.z, l1.w}, h[4] = {hv.x, hv.y, hv.z, hv.w};
#pragma unroll
        for (int e = 0; e < 4; e++) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t qa = (a[e] >> (8 * i)) & 0xffu, qc = (c[e] >> (8 * i)) & 0xffu, qh = (h[e] >> (8 * i)) & 0xffu;
                const int q1 = (int)((qa & 0xFu) | ((qh & 3u) << 4)) - 32;
                const int q2 = (int)((qc & 0xFu) | (((qh >> 2) & 3u) << 4)) - 32;
                const int q3 = (int)((qa >> 4) | (((qh >> 4) & 3u) << 4)) - 32;
                const int q4 = (int)((qc >> 4) | ((qh >> 6) << 4)) - 32;
                w[4 * e + i] = __fmul_rn(t1, (float)q1);
                w[16 + 4 * e + i] = __fmul_rn(t2, (float)q2);
                w[32 + 4 * e + i] = __fmul_rn(t3, (float)q3);
                w[48 + 4 * e + i] = __fmul_rn(t4, (float)q4);
            }
        }
    }
};

// BF16 rows: two values per word, the low half first
// (src/kernels/half/bf16.wgsl:3-9).
struct DecBF16 {
    static constexpr int RUNS = 2;
    static constexpr int E = 8;
    static constexpr uint32_t BLOCK = 8;
    static constexpr int CHUNK = 0;
    static const char *name() { return "matvec_bf16"; }
    static uint32_t row_bytes(uint32_t k) { return 2u * k; }
    __device__ static uint32_t xoff(uint32_t task, int h) { return 8u * task + 4u * h; }
    // A task as loaded, and its eight weights.
    __device__ static void expand(const uint4 &q, float (&w)[E]) {
        const uint32_t words[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int e = 0; e < 4; e++) {
            w[2 * e + 0] = __uint_as_float(words[e] << 16);
            w[2 * e + 1] = __uint_as_float(words[e] & 0xffff0000u);
        }
    }
    __device__ static void decode(const uint8_t *row, uint32_t, uint32_t task, float (&w)[E]) {
        expand(*reinterpret_cast<const uint4 *>(row + 16u * task), w);
    }
};

// F16 rows: two values per word, the low half first
// (src/kernels/half/f16.wgsl:3-9); every f16 value is exact in f32.
struct DecF16 {
    static constexpr int RUNS = 2;
    static constexpr int E = 8;
    static constexpr uint32_t BLOCK = 8;
    static constexpr int CHUNK = 0;
    static const char *name() { return "matvec_f16"; }
    static uint32_t row_bytes(uint32_t k) { return 2u * k; }
    __device__ static uint32_t xoff(uint32_t task, int h) { return 8u * task + 4u * h; }
    __device__ static void expand(const uint4 &q, float (&w)[E]) {
        const uint32_t words[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int e = 0; e < 4; e++) {
            w[2 * e + 0] = half_bits_to_float(words[e] & 0xffffu);
            w[2 * e + 1] = half_bits_to_float(words[e] >> 16);
        }
    }
    __device__ static void decode(const uint8_t *row, uint32_t, uint32_t task, float (&w)[E]) {
        expand(*reinterpret_cast<const uint4 *>(row + 16u * task), w);
    }
};

}  // namespace zhip
