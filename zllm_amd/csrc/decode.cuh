// Block decoders shared by the decode multiplies and the embedding gathers.
// Each follows its reference decoder's f32 operations one for one, with every
// multiply and subtract rounded on its own (no contraction), so decoded
// weights equal the reference's bit for bit:
//   Q8_0  src/ref/tensor.zig:49-53    y = f32(q) * f32(d)
//   Q4_K  src/ref/tensor.zig:94-116   y = (d * sc) * q - (dmin * m)
//   BF16  src/ref/tensor.zig:36-40    y = bits << 16
// A decoder splits a row into 16-byte "tasks" so that consecutive lanes load
// consecutive 16-byte vectors; decode() returns the task's E weights, whose
// inputs are the two runs of E/2 floats at xoff(task, 0) and xoff(task, 1).
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
    static constexpr int E = 16;
    static constexpr uint32_t BLOCK = 32;
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

// Q4_K blocks as in the file (144 bytes = nine 16-byte vectors). Task p of a
// block reads qs bytes [16p, 16p + 16): positions l = 16 (p % 2) .. of chunk
// c = p / 2, low nibbles for sub-block 2c, high nibbles for sub-block 2c + 1.
struct DecQ4_K {
    static constexpr int E = 32;
    static constexpr uint32_t BLOCK = 256;
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

// BF16 rows: two values per word, the low half first
// (src/kernels/half/bf16.wgsl:3-9).
struct DecBF16 {
    static constexpr int E = 8;
    static constexpr uint32_t BLOCK = 8;
    static const char *name() { return "matvec_bf16"; }
    static uint32_t row_bytes(uint32_t k) { return 2u * k; }
    __device__ static uint32_t xoff(uint32_t task, int h) { return 8u * task + 4u * h; }
    __device__ static void decode(const uint8_t *row, uint32_t, uint32_t task, float (&w)[E]) {
        const uint4 q = *reinterpret_cast<const uint4 *>(row + 16u * task);
        const uint32_t words[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int e = 0; e < 4; e++) {
            w[2 * e + 0] = __uint_as_float(words[e] << 16);
            w[2 * e + 1] = __uint_as_float(words[e] & 0xffff0000u);
        }
    }
};

}  // namespace zhip
