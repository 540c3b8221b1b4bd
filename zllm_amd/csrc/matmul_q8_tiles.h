// What the two Q8_0 prefill kernels on the bf16 / f16 matrix cores share (matmul_q8_bf16.hip:
// 128 x 64 tiles and smaller; matmul_q8_bf16_wide.hip: 128 x 128 tiles for matrices with the
// rows to fill the CUs with them): the operand types of the rungs, the loads straight into
// LDS, the barriers that leave them in flight, the permuted line layout and the conversion of
// a lane's sixteen weights.
#pragma once

#include <hip/hip_runtime.h>

#include "common.h"

namespace zhip {
namespace q8tiles {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int BK = 128, PRODUCERS = 4;

struct Q8Args {
    const uint8_t *x;  // packed bf16 rows
    const uint8_t *w;  // split rows: k int8 values, k / 32 f16 scales, zero pad to 16 bytes
    float *out;
    uint32_t rows, n, k, col0, out_stride, accumulate, row_bytes;
    uint32_t x_bytes, w_bytes;  // bytes the kernel may read behind x and w
};

// The operand type of a rung: two floats rounded into one word, and the matrix instruction.
struct AsBf16 {
    typedef bf16x8 vec;
    static __device__ __forceinline__ uint32_t pack(float lo, float hi) {
        const f32x2 v = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
    }
    static __device__ __forceinline__ f32x16 mfma(vec a, vec b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
};
struct AsF16 {
    typedef f16x8 vec;
    static __device__ __forceinline__ uint32_t pack(float lo, float hi) {
        const f32x2 v = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2));
    }
    static __device__ __forceinline__ f32x16 mfma(vec a, vec b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
};
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_buffer(const uint8_t *base, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(base), 0, (int)bytes, 0x00020000);
}
typedef __attribute__((address_space(3))) void *lds_ptr;
// One wave-wide load straight into LDS: lane l's bytes land at dst + size * l.
__device__ __forceinline__ void load_lds_b128(__amdgpu_buffer_rsrc_t buf, uint8_t *dst, uint32_t voff, uint32_t soff) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(buf, (lds_ptr)dst, 16, voff, soff, 0, 0);
}
__device__ __forceinline__ void load_lds_b32(__amdgpu_buffer_rsrc_t buf, uint8_t *dst, uint32_t voff, uint32_t soff) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(buf, (lds_ptr)dst, 4, voff, soff, 0, 0);
}
// A workgroup barrier that leaves loads into LDS in flight (__syncthreads() would wait for
// every outstanding memory operation, the loads running steps ahead included).
template <int LOADS_LEFT>
__device__ __forceinline__ void sync_keeping_loads() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(LOADS_LEFT) : "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}
__device__ __forceinline__ void sync_after_reads() {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}
// Rows are unpadded 128-byte lines whose 16-byte chunks are stored permuted: chunk c of row r
// sits at position c ^ key(r). With this key the 32-row fragment reads run at the LDS's full
// rate (measured; an unpermuted layout is ten times slower).
__device__ __forceinline__ uint32_t line_key(uint32_t row) { return (row & 7u) ^ ((row >> 3) & 1u); }

struct WRaw { u32x4 q; uint32_t d; };

// Sixteen int8 weights times their block's scale (exact in f32), rounded once to the operand
// type: the first operands of the lane's two MFMAs.
template <class H>
__device__ __forceinline__ void convert(const WRaw &r, typename H::vec &w0, typename H::vec &w1) {
    const float d = (float)__builtin_bit_cast(_Float16, (uint16_t)r.d);
    u32x4 lo, hi;
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const int32_t v = (int32_t)r.q[i];
        lo[2 * i] = H::pack((float)(int8_t)(v) * d, (float)(int8_t)(v >> 8) * d);
        lo[2 * i + 1] = H::pack((float)(int8_t)(v >> 16) * d, (float)(v >> 24) * d);
        const int32_t u = (int32_t)r.q[2 + i];
        hi[2 * i] = H::pack((float)(int8_t)(u) * d, (float)(int8_t)(u >> 8) * d);
        hi[2 * i + 1] = H::pack((float)(int8_t)(u >> 16) * d, (float)(u >> 24) * d);
    }
    w0 = __builtin_bit_cast(typename H::vec, lo);
    w1 = __builtin_bit_cast(typename H::vec, hi);
}

}  // namespace q8tiles
}  // namespace zhip
