// matmul_q8_0 / matmul_q3_k / matmul_q4_k / matmul_q5_k / matmul_q6_k: the prefill multiply on activations rounded to
// 8-bit blocks (quantize_q8), as src/kernels/matmul_quant.wgsl defines it:
//   out[t][col0 + j] = sum over 32-weight units of dx * (s * sum(q * qx) - m * sum(qx))
// with every unit's integer sum exact. Here the unit sums run on the int8 matrix
// cores (v_mfma_i32_16x16x32_i8: one 32-deep unit of 16 x 16 outputs per
// instruction). Q8_0's f16 unit scales are applied to the integer results in
// f32 (three vector operations per output and unit, which bounds that kernel);
// the K formats' 6- and 8-bit integer scales are applied in integers (one
// 24-bit multiply-add per output and unit), their minimums by one more matrix
// instruction per unit, and a block's two f32 scales once per 256 positions.
//
// A 256-thread workgroup computes 64 tokens x 64 rows in steps of 256 positions;
// wave w owns rows 16 w .. 16 w + 15 for all 64 tokens (four accumulator tiles).
// Buffers are range-checked: tokens past `rows` and rows past `n` read zeros,
// and units outside [kb, ke) contribute nothing, so partial tiles and split-k
// slices need no special paths. Every output is summed over k in increasing
// order by a sequence of operations that does not depend on its position in
// the tile: token chunking cannot change bits.
//
// The K formats over whole, unsliced k (what a planner's prefill step is) have kernels of their
// own further down: 32 x 32 x 32 matrix instructions on 32-token tiles, k summed in four parts
// that one wave walks one after the other (long steps) or four waves side by side (short
// steps, whose few tiles would otherwise leave a CU one wave that walks all of k).
#include <hip/hip_runtime.h>

#include "common.h"
#include "decode.h"

namespace zhip {

typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef float if32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t iu32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t iu32x2 __attribute__((ext_vector_type(2)));

namespace {

constexpr uint32_t TT = 64;     // tokens per workgroup
constexpr uint32_t TN = 64;     // rows per workgroup
constexpr uint32_t STEP = 256;  // positions per step
constexpr uint32_t LINE = STEP + 16;  // bytes between register-staged token lines in LDS: sixteen tokens' 8-byte reads of two lane groups cover all banks
constexpr uint32_t UNITS = 1;  // units the K-format kernel schedules together (2 and 4 measured no faster)

struct I8Args {
    const uint8_t *qx;   // rows x k int8, four per word
    const uint8_t *w;    // GPU-layout weight rows
    const uint8_t *dx;   // rows x k / ACT f32
    float *out;
    uint32_t rows, n, k, col0, out_stride, accumulate, k_slice, slice_stride, row_bytes;
    uint32_t qx_bytes, w_bytes, dx_bytes;
};

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_buffer(const uint8_t *base, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(base), 0, (int)bytes, 0x00020000);
}

typedef __attribute__((address_space(3))) void *lds_ptr;

// One wave-wide load straight into LDS: lane l's 4 (16) bytes land at
// dst + 4 l (16 l), whatever global offset the lane asked for. The destination
// reaches the load as a bare LDS address: the compiler then keeps no dependency
// between these loads and later LDS reads (it would wait for every outstanding
// load before each read); sync_after_loads() orders them.
__device__ __forceinline__ void load_lds_b32(__amdgpu_buffer_rsrc_t buf, uint8_t *dst, uint32_t offset) {
    uint32_t address = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)dst);  // the same for all lanes
    asm volatile("" : "+s"(address));
    __builtin_amdgcn_raw_ptr_buffer_load_lds(buf, (lds_ptr)(uintptr_t)address, 4, offset, 0, 0, 0);
}
__device__ __forceinline__ void load_lds_b128(__amdgpu_buffer_rsrc_t buf, uint8_t *dst, uint32_t offset) {
    uint32_t address = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)dst);
    asm volatile("" : "+s"(address));
    __builtin_amdgcn_raw_ptr_buffer_load_lds(buf, (lds_ptr)(uintptr_t)address, 16, offset, 0, 0, 0);
}
// The same with a uniform part of the offset in a scalar register (the buffer's range check
// sees the lane's part only).
__device__ __forceinline__ void load_lds_b128(__amdgpu_buffer_rsrc_t buf, uint8_t *dst, uint32_t offset, uint32_t uniform_offset) {
    uint32_t address = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)dst);
    asm volatile("" : "+s"(address));
    __builtin_amdgcn_raw_ptr_buffer_load_lds(buf, (lds_ptr)(uintptr_t)address, 16, offset, uniform_offset, 0, 0);
}

// Every load of this wave has landed, every wave's LDS traffic is done: the
// buffer just filled may be read, the one just read may be filled.
__device__ __forceinline__ void sync_after_loads() {
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

__device__ __forceinline__ long as_operand(iu32x2 v) {
    return (long)(((unsigned long)v.y << 32) | (unsigned long)v.x);
}

// ---- Q8_0 weights (split rows: k bytes, then k / 32 f16 scales), Q8_0 activations ----
// The accumulators: lane (l16, g) holds token t0 + 16 mt + l16 for rows
// n0 + 16 wave + 4 g + i (weights are the matrix cores' first operand), so a
// lane scales its four results of a product by four row scales and one token
// scale.
//
// Both operands cross LDS. Read straight into the operand layout, adjacent
// lanes would ask for different rows, and the load unit takes such a load apart
// one lane a clock; here a wave brings sixteen rows and sixteen token lines in
// as whole 256-byte runs (buffer_load ... lds, 16 bytes a lane, four lines an
// instruction) and reads its operands back, 8 bytes a lane. Two buffers: a
// step's loads are issued before the previous step's multiply and waited for
// after it.
//
// The lines are laid out so that operand reads meet no bank conflicts: each
// instruction's four lines (1 KiB) are followed by XPAD = 8 bytes, and chunk c
// of line r sits at position c ^ 2 (r % 4). The sixteen lines of an operand
// read then start at sixteen different 8-byte bank pairs:
// 4 (c / 2 ^ r % 4) + 2 (c % 2) + half + r / 4. The tokens' block scales sit
// eight to a token with unit u at position u ^ (t / 4 % 4), which spreads the
// sixteen tokens a lane group reads over sixteen banks.
constexpr uint32_t XPAD = 8;
__device__ __forceinline__ uint32_t xkey(uint32_t line) { return 2u * (line & 3u); }
constexpr uint32_t QUAD = 4u * STEP + XPAD;  // four lines and their padding

template <bool RAGGED>
__global__ __launch_bounds__(256, 2) void matmul_q8_0_i8_kernel(I8Args a) {
    constexpr uint32_t DBUF = TT * 32u;          // [token][8 units] f32
    constexpr uint32_t WBUF = TN / 4u * QUAD;    // [row][256 bytes], chunks permuted, padded every four rows
    constexpr uint32_t SBUF = TN * 16u;          // [row][8 units] f16
    constexpr uint32_t XBUF = TT / 4u * QUAD;    // [token][256 bytes], the same way
    __shared__ __align__(16) uint8_t lds_q[2][XBUF];
    __shared__ __align__(16) uint8_t lds_d[2][DBUF];
    __shared__ __align__(16) uint8_t lds_w[2][WBUF];
    __shared__ __align__(16) uint8_t lds_s[2][SBUF];
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, l16 = lane & 15u, g = lane >> 4;
    const uint32_t n0 = blockIdx.x * TN, t0 = blockIdx.y * TT;
    const uint32_t kb = blockIdx.z * a.k_slice, ke = min(a.k, kb + a.k_slice);
    const uint32_t k_first = kb & ~(STEP - 1u);
    const uint32_t steps = (ke - k_first + STEP - 1u) / STEP;
    const __amdgpu_buffer_rsrc_t xbuf = make_buffer(a.qx, a.qx_bytes), wbuf = make_buffer(a.w, a.w_bytes), dbuf = make_buffer(a.dx, a.dx_bytes);

    // Weight loads: instruction i takes rows r = 4 i + lane / 16 of the wave's
    // sixteen; the lane at position p = lane % 16 fetches chunk p ^ key(r), the
    // one that belongs there.
    const uint32_t wl_row = lane >> 4, wl_pos = lane & 15u;
    const uint32_t woff = (n0 + 16u * wave + wl_row) * a.row_bytes;
    // Token loads, the same way: instruction i takes tokens 16 wave + 4 i + lane / 16.
    const uint32_t xoff = (t0 + 16u * wave + wl_row) * a.k;
    // Scales: one word a lane, row 16 wave + lane / 4, units 2 (lane % 4), + 1.
    const uint32_t soff = (n0 + 16u * wave + (lane >> 2)) * a.row_bytes + a.k + 4u * (lane & 3u);
    // Block scales of tokens 16 wave + 8 i + lane / 8: the lane at position
    // lane % 8 fetches unit (lane % 8) ^ (token / 4 % 4); token / 4 % 4 = 2 i + lane / 32 % 2.
    const uint32_t doff = (t0 + 16u * wave + (lane >> 3)) * (a.k / 32u) * 4u;

    auto fetch = [&](uint32_t k0, uint32_t buf) __attribute__((always_inline)) {
#pragma unroll
        for (uint32_t i = 0; i < 4; i++)
            load_lds_b128(wbuf, lds_w[buf] + (4u * wave + i) * QUAD, woff + 4u * i * a.row_bytes + k0 + 16u * (wl_pos ^ xkey(wl_row)));
        load_lds_b32(wbuf, lds_s[buf] + 16u * wave * 16u, soff + k0 / 16u);
#pragma unroll
        for (uint32_t i = 0; i < 4; i++)
            load_lds_b128(xbuf, lds_q[buf] + (4u * wave + i) * QUAD, xoff + 4u * i * a.k + k0 + 16u * (wl_pos ^ xkey(wl_row)));
#pragma unroll
        for (uint32_t i = 0; i < 2; i++)
            load_lds_b32(dbuf, lds_d[buf] + (16u * wave + 8u * i) * 32u, doff + 8u * i * (a.k / 32u) * 4u + k0 / 8u + 4u * ((lane & 7u) ^ (2u * i + ((lane >> 5) & 1u))));
    };

    if32x4 acc[4];
#pragma unroll
    for (int mt = 0; mt < 4; mt++) acc[mt] = if32x4{0.f, 0.f, 0.f, 0.f};

    // One unit's integer sums for the four token tiles, and the tokens' block scales.
    struct Unit {
        i32x4 is[4];
        float dx[4];
    };
    // This lane's operand bytes of unit u: line l16 of its row or token tile,
    // logical chunk 2 u + g / 2, half g % 2.
    const uint32_t line = (l16 >> 2) * QUAD + (l16 & 3u) * STEP + 8u * (g & 1u);
    const uint32_t dkey = (l16 >> 2) & 3u;
    auto multiply = [&](uint32_t buf, uint32_t u, Unit &r) __attribute__((always_inline)) {
        const uint32_t at = line + 16u * ((2u * u + (g >> 1)) ^ xkey(l16));
        const long wf = *reinterpret_cast<const long *>(&lds_w[buf][4u * wave * QUAD + at]);
#pragma unroll
        for (uint32_t mt = 0; mt < 4; mt++) {
            const long xf = *reinterpret_cast<const long *>(&lds_q[buf][4u * mt * QUAD + at]);
            r.is[mt] = __builtin_amdgcn_mfma_i32_16x16x32_i8(wf, xf, i32x4{0, 0, 0, 0}, 0, 0, 0);
            r.dx[mt] = *reinterpret_cast<const float *>(lds_d[buf] + (16u * mt + l16) * 32u + 4u * (u ^ dkey));
        }
    };
    auto scale = [&](uint32_t k0, const iu32x4 (&sc)[4], uint32_t u, const Unit &r) __attribute__((always_inline)) {
        // A unit outside [kb, ke) multiplied whatever bytes lie there: zero its scale.
        const uint32_t kpos = k0 + 32u * u;
        const bool live = !RAGGED || (kpos >= kb && kpos < ke);
#pragma unroll
        for (uint32_t i = 0; i < 4; i++) {
            const uint32_t word = sc[i][u >> 1];
            const float dw = live ? half_bits_to_float(u & 1u ? word >> 16 : word & 0xffffu) : 0.f;
#pragma unroll
            for (uint32_t mt = 0; mt < 4; mt++) acc[mt][i] = fmaf(r.dx[mt], dw * (float)r.is[mt][i], acc[mt][i]);
        }
    };
    // The matrix cores work on unit u + 1 while the vector units scale unit u.
    auto compute = [&](uint32_t k0, uint32_t buf) __attribute__((always_inline)) {
        iu32x4 sc[4];  // rows 4 g + i: eight f16 scales
#pragma unroll
        for (uint32_t i = 0; i < 4; i++) sc[i] = *reinterpret_cast<const iu32x4 *>(lds_s[buf] + (16u * wave + 4u * g + i) * 16u);
        Unit even, odd;
        multiply(buf, 0, even);
#pragma unroll
        for (uint32_t u = 0; u < 8; u += 2) {
            multiply(buf, u + 1u, odd);
            scale(k0, sc, u, even);
            __builtin_amdgcn_sched_barrier(0);
            if (u + 2u < 8u) multiply(buf, u + 2u, even);
            scale(k0, sc, u + 1u, odd);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    fetch(k_first, 0);
    sync_after_loads();
    for (uint32_t s = 0; s < steps; s++) {
        const uint32_t k0 = k_first + s * STEP;
        fetch(k0 + STEP, (s + 1u) & 1u);
        compute(k0, s & 1u);
        sync_after_loads();
    }

    const uint32_t j = n0 + 16u * wave + 4u * g;
    float *out = a.out + (size_t)blockIdx.z * a.slice_stride + a.col0 + j;
#pragma unroll
    for (uint32_t mt = 0; mt < 4; mt++) {
        const uint32_t t = t0 + 16u * mt + l16;
        if (t >= a.rows) continue;
        float *o = out + (size_t)t * a.out_stride;
#pragma unroll
        for (uint32_t i = 0; i < 4; i++)
            if (j + i < a.n) o[i] = a.accumulate ? o[i] + acc[mt][i] : acc[mt][i];
    }
}

// The accumulators' home: lane (l16, g) holds row n0 + 16 wave + l16 for tokens
// t0 + 16 mt + 4 g + i.
__device__ __forceinline__ void store_tile(const I8Args &a, const if32x4 (&acc)[4], uint32_t t0, uint32_t j, uint32_t g) {
    if (j >= a.n) return;
    float *out = a.out + (size_t)blockIdx.z * a.slice_stride + a.col0 + j;
#pragma unroll
    for (uint32_t mt = 0; mt < 4; mt++) {
#pragma unroll
        for (uint32_t i = 0; i < 4; i++) {
            const uint32_t t = t0 + 16u * mt + 4u * g + i;
            if (t >= a.rows) continue;
            float *o = out + (size_t)t * a.out_stride;
            *o = a.accumulate ? *o + acc[mt][i] : acc[mt][i];
        }
    }
}

// ---- K formats (256-weight blocks), Q8_K activations ---------------------------------
// A format gives the bytes a lane reads of one block of its row (Raw, load: from the wave's
// LDS slot, where the sixteen rows' blocks arrive by whole-line direct loads; a lane loading
// its own row's 8- and 16-byte pieces from memory makes the vector memory unit look up a
// cache line per lane, and that rate bounded the kernel) and
// unit u's operand: the eight signed integers at positions 8 g .. 8 g + 7 of the
// unit with the scales of the unit's two halves of sixteen and its minimum
// (src/kernels/quant/q3_k.wgsl, q4_k.wgsl, q5_k.wgsl, q6_k.wgsl: head, scales, quad_i8).
// HALVES: the two halves' scales differ, so a unit takes two instructions, each
// with the other half's lanes feeding zeros.

__device__ __forceinline__ int sbyte(uint32_t word, uint32_t i) { return (int)(word << (24u - 8u * i)) >> 24; }

struct I8Q4 {
    static constexpr uint32_t BLOCK = 144;
    static constexpr bool HAS_MIN = true, HALVES = false;
    struct Raw {
        iu32x4 h;       // d, dmin and the twelve scale bytes
        iu32x2 q[4];    // 8 bytes of each 64-weight chunk: low nibbles unit 2c, high 2c + 1
    };
    static __device__ __forceinline__ void load(const uint8_t *blk, uint32_t g, Raw &r) {
        r.h = *reinterpret_cast<const iu32x4 *>(blk);
#pragma unroll
        for (uint32_t c = 0; c < 4; c++) r.q[c] = *reinterpret_cast<const iu32x2 *>(blk + 16u + 32u * c + 8u * g);
    }
    static __device__ __forceinline__ void block(const Raw &r, float &d, float &dmin) {
        d = half_bits_to_float(r.h.x & 0xffffu);
        dmin = half_bits_to_float(r.h.x >> 16);
    }
    static __device__ __forceinline__ void unit(const Raw &r, uint32_t u, uint32_t, iu32x2 &b, int &s0, int &s1, int &mn) {
        const uint2 sm = scale_min_k4(r.h.y, r.h.z, r.h.w, u);
        s0 = s1 = (int)sm.x;
        mn = (int)sm.y;
        b = r.q[u >> 1];
        if (u & 1u) b = b >> 4;
        b = b & 0x0f0f0f0fu;
    }
};

struct I8Q5 {
    static constexpr uint32_t BLOCK = 176;
    static constexpr bool HAS_MIN = true, HALVES = false;
    struct Raw {
        iu32x4 h;
        iu32x2 qh;      // the fifth bits of positions 8 g .. 8 g + 7, bit u for unit u
        iu32x2 q[4];
    };
    static __device__ __forceinline__ void load(const uint8_t *blk, uint32_t g, Raw &r) {
        r.h = *reinterpret_cast<const iu32x4 *>(blk);
        r.qh = *reinterpret_cast<const iu32x2 *>(blk + 16u + 8u * g);
#pragma unroll
        for (uint32_t c = 0; c < 4; c++) r.q[c] = *reinterpret_cast<const iu32x2 *>(blk + 48u + 32u * c + 8u * g);
    }
    static __device__ __forceinline__ void block(const Raw &r, float &d, float &dmin) {
        d = half_bits_to_float(r.h.x & 0xffffu);
        dmin = half_bits_to_float(r.h.x >> 16);
    }
    static __device__ __forceinline__ void unit(const Raw &r, uint32_t u, uint32_t, iu32x2 &b, int &s0, int &s1, int &mn) {
        const uint2 sm = scale_min_k4(r.h.y, r.h.z, r.h.w, u);
        s0 = s1 = (int)sm.x;
        mn = (int)sm.y;
        b = r.q[u >> 1];
        if (u & 1u) b = b >> 4;
        b = (b & 0x0f0f0f0fu) | (((r.qh >> u) & 0x01010101u) << 4);
    }
};

struct I8Q6 {
    static constexpr uint32_t BLOCK = 224;  // padded from 210 at load
    static constexpr bool HAS_MIN = false, HALVES = true;
    struct Raw {
        iu32x2 ql[4];   // [2 n + c % 2]: low nibbles unit 4 n + c % 2, high nibbles that + 2
        iu32x2 qh[2];   // [n]: bits 2 c of unit 4 n + c
        iu32x4 sc;      // sixteen signed scales
        uint32_t d;
    };
    static __device__ __forceinline__ void load(const uint8_t *blk, uint32_t g, Raw &r) {
#pragma unroll
        for (uint32_t i = 0; i < 4; i++) r.ql[i] = *reinterpret_cast<const iu32x2 *>(blk + 32u * i + 8u * g);
#pragma unroll
        for (uint32_t n = 0; n < 2; n++) r.qh[n] = *reinterpret_cast<const iu32x2 *>(blk + 128u + 32u * n + 8u * g);
        r.sc = *reinterpret_cast<const iu32x4 *>(blk + 192u);
        r.d = *reinterpret_cast<const uint32_t *>(blk + 208u);
    }
    static __device__ __forceinline__ void block(const Raw &r, float &d, float &dmin) {
        d = half_bits_to_float(r.d & 0xffffu);
        dmin = 0.f;
    }
    static __device__ __forceinline__ void unit(const Raw &r, uint32_t u, uint32_t, iu32x2 &b, int &s0, int &s1, int &mn) {
        const uint32_t n = u >> 2, c = u & 3u;
        const uint32_t pair = r.sc[(8u * n + 2u * c) >> 2] >> (16u * (c & 1u));  // scales 8 n + 2 c and the next
        s0 = sbyte(pair, 0);
        s1 = sbyte(pair, 1);
        mn = 0;
        const iu32x2 q = ((r.ql[2u * n + (c & 1u)] >> (4u * (c >> 1))) & 0x0f0f0f0fu) | (((r.qh[n] >> (2u * c)) & 0x03030303u) << 4);
        b = (q + 0x60606060u) ^ 0x80808080u;  // minus 32 a byte, no borrows
    }
};

struct I8Q3 {
    static constexpr uint32_t BLOCK = 128;  // repacked at load: eight 16-byte units
    static constexpr bool HAS_MIN = false, HALVES = true;
    struct Raw {
        iu32x4 u[8];  // two words of 2-bit values, the high bits, scales - 32 and d
    };
    static __device__ __forceinline__ void load(const uint8_t *blk, uint32_t, Raw &r) {
#pragma unroll
        for (uint32_t i = 0; i < 8; i++) r.u[i] = *reinterpret_cast<const iu32x4 *>(blk + 16u * i);
    }
    static __device__ __forceinline__ void block(const Raw &r, float &d, float &dmin) {
        d = half_bits_to_float(r.u[0].w >> 16);  // every unit of a block carries the block's d
        dmin = 0.f;
    }
    static __device__ __forceinline__ void unit(const Raw &r, uint32_t u, uint32_t g, iu32x2 &b, int &s0, int &s1, int &mn) {
        const iu32x4 v = r.u[u];
        s0 = sbyte(v.w, 0);
        s1 = sbyte(v.w, 1);
        mn = 0;
        // Position 4 e + i: bits 2 (e % 4) of byte i of word e / 4, high bit 8 i + e.
        const uint32_t l = (g < 2u ? v.x : v.y) >> (4u * (g & 1u)), hb = v.z >> (2u * g);
        const iu32x2 c = {(l & 0x03030303u) | ((hb & 0x01010101u) << 2), ((l >> 2) & 0x03030303u) | (((hb >> 1) & 0x01010101u) << 2)};
        b = (c + 0x7c7c7c7cu) ^ 0x80808080u;  // minus 4 a byte, no borrows
    }
};

template <class P>
__global__ __launch_bounds__(256, 2) void matmul_kquant_i8_kernel(I8Args a) {
    __shared__ __align__(16) uint8_t lds_q[2][TT * LINE];
    __shared__ __align__(16) float lds_d[2][TT];      // the tokens' block scales
    // The weights: per wave and buffer its sixteen rows' blocks, [row][BLOCK bytes], as WLOADS
    // wave-wide loads of 16 bytes a lane (chunk c = 64 load + lane: row c / CPR, piece c % CPR;
    // lanes past the sixteenth row ask past the buffer and zeros land behind the blocks).
    constexpr uint32_t CPR = P::BLOCK / 16u, WLOADS = (16u * CPR + 63u) / 64u, WSLOT = WLOADS * 1024u;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_w[];  // [2][4 waves][WSLOT]
    const uint32_t tid = threadIdx.x, lane = tid & 63u, l16 = lane & 15u, g = lane >> 4;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t n0 = blockIdx.x * TN, t0 = blockIdx.y * TT;
    const uint32_t kb = blockIdx.z * a.k_slice, ke = min(a.k, kb + a.k_slice);
    const uint32_t k_first = kb & ~(STEP - 1u);
    const uint32_t steps = (ke - k_first + STEP - 1u) / STEP;
    const __amdgpu_buffer_rsrc_t xbuf = make_buffer(a.qx, a.qx_bytes), wbuf = make_buffer(a.w, a.w_bytes), dbuf = make_buffer(a.dx, a.dx_bytes);

    // Staging: a quarter (two units) of one token's block per thread.
    const uint32_t atok = tid >> 2, aq = tid & 3u;
    const uint32_t aoff = (t0 + atok) * a.k + 64u * aq;
    const uint32_t doff = (t0 + atok) * (a.k / 256u) * 4u;
    const uint32_t j = n0 + 16u * wave + l16;
    uint32_t woff[WLOADS];
#pragma unroll
    for (uint32_t i = 0; i < WLOADS; i++) {
        const uint32_t c = 64u * i + lane;
        woff[i] = c < 16u * CPR ? (n0 + 16u * wave + c / CPR) * a.row_bytes + 16u * (c % CPR) : 0xfffffff0u - a.row_bytes;
    }

    iu32x4 ra[4];
    uint32_t rd;
    typename P::Raw cur;
    // Step k0's operands: the tokens' bytes and scales into registers (stashed in LDS after the
    // multiply), the weights straight into LDS buffer `buf`.
    auto fetch = [&](uint32_t k0, uint32_t buf) __attribute__((always_inline)) {
#pragma unroll
        for (uint32_t i = 0; i < 4; i++) ra[i] = __builtin_amdgcn_raw_buffer_load_b128(xbuf, aoff + k0 + 16u * i, 0, 0);
        rd = __builtin_amdgcn_raw_buffer_load_b32(dbuf, doff + k0 / 64u, 0, 0);
        uint8_t *dst = lds_w + (buf * 4u + wave) * WSLOT;
#pragma unroll
        for (uint32_t i = 0; i < WLOADS; i++) load_lds_b128(wbuf, dst + 1024u * i, woff[i], k0 / 256u * P::BLOCK);
    };
    auto stash = [&](uint32_t buf) __attribute__((always_inline)) {
        uint8_t *line = &lds_q[buf][atok * LINE + 64u * aq];
#pragma unroll
        for (uint32_t i = 0; i < 4; i++) {
            *reinterpret_cast<iu32x2 *>(line + 16u * i) = ra[i].xy;
            *reinterpret_cast<iu32x2 *>(line + 16u * i + 8u) = ra[i].zw;
        }
        if (aq == 0u) lds_d[buf][atok] = __uint_as_float(rd);
    };

    if32x4 acc[4];
#pragma unroll
    for (int mt = 0; mt < 4; mt++) acc[mt] = if32x4{0.f, 0.f, 0.f, 0.f};

    fetch(k_first, 0);
    stash(0);
    sync_after_loads();
    for (uint32_t s = 0; s < steps; s++) {
        const uint32_t k0 = k_first + s * STEP, buf = s & 1u;
        const bool more = s + 1u < steps;
        P::load(lds_w + (buf * 4u + wave) * WSLOT + l16 * P::BLOCK, g, cur);
        if (more) fetch(k0 + STEP, buf ^ 1u);
        // A block's units are summed in integers: a unit's exact sum times its 6- or 8-bit
        // scale (one 24-bit multiply-add a result), the minimums as one more matrix
        // instruction a unit whose second operand is the unit's minimum in all 32 positions,
        // accumulated by the matrix cores. The block's two f32 scales are applied once. (The
        // minimums' term as two matrix instructions a block, the tokens' unit sums against the
        // rows' eight minimums, was tried: taking the sums while staging costs more than the six
        // instructions it saves, 48.1 against 46.3 us for Q4_K.)
        i32x4 isum[4], msum[4];
#pragma unroll
        for (int mt = 0; mt < 4; mt++) isum[mt] = msum[mt] = i32x4{0, 0, 0, 0};
#pragma unroll
        for (uint32_t u = 0; u < 8; u += UNITS) {
            // UNITS units at a time, behind a branch that skips units outside the slice [kb, ke)
            // and keeps the groups apart (scheduled all together they need hundreds of
            // registers); a group's units overlap each other's LDS and matrix-core latencies.
            bool live[UNITS], any = false;
#pragma unroll
            for (uint32_t e = 0; e < UNITS; e++) {
                const uint32_t kpos = k0 + 32u * (u + e);
                live[e] = kpos >= kb && kpos < ke;
                any = any || live[e];
            }
            if (!any) continue;
            long b0[UNITS], b1[UNITS], bm[UNITS];
            int s0[UNITS], s1[UNITS];
#pragma unroll
            for (uint32_t e = 0; e < UNITS; e++) {
                iu32x2 w8;
                int mn;
                P::unit(cur, u + e, g, w8, s0[e], s1[e], mn);
                s0[e] = live[e] ? s0[e] : 0;
                s1[e] = live[e] ? s1[e] : 0;
                mn = live[e] ? mn : 0;
                const iu32x2 zero = {0u, 0u};
                b0[e] = as_operand(P::HALVES ? (g < 2u ? w8 : zero) : w8);
                b1[e] = as_operand(g < 2u ? zero : w8);
                const uint32_t m4 = (uint32_t)mn * 0x01010101u;
                bm[e] = as_operand(iu32x2{m4, m4});
            }
#pragma unroll
            for (uint32_t mt = 0; mt < 4; mt++) {
#pragma unroll
                for (uint32_t e = 0; e < UNITS; e++) {
                    const long af = *reinterpret_cast<const long *>(&lds_q[buf][(16u * mt + l16) * LINE + 32u * (u + e) + 8u * g]);
                    const i32x4 is = __builtin_amdgcn_mfma_i32_16x16x32_i8(af, b0[e], i32x4{0, 0, 0, 0}, 0, 0, 0);
#pragma unroll
                    for (int i = 0; i < 4; i++) isum[mt][i] = __mul24(s0[e], is[i]) + isum[mt][i];
                    if (P::HALVES) {
                        const i32x4 is1 = __builtin_amdgcn_mfma_i32_16x16x32_i8(af, b1[e], i32x4{0, 0, 0, 0}, 0, 0, 0);
#pragma unroll
                        for (int i = 0; i < 4; i++) isum[mt][i] = __mul24(s1[e], is1[i]) + isum[mt][i];
                    }
                    if (P::HAS_MIN) msum[mt] = __builtin_amdgcn_mfma_i32_16x16x32_i8(af, bm[e], msum[mt], 0, 0, 0);
                }
            }
        }
        float d, dmin;
        P::block(cur, d, dmin);
#pragma unroll
        for (uint32_t mt = 0; mt < 4; mt++) {
            const if32x4 dxv = *reinterpret_cast<const if32x4 *>(&lds_d[buf][16u * mt + 4u * g]);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                float part = d * (float)isum[mt][i];
                if (P::HAS_MIN) part = fmaf(-dmin, (float)msum[mt][i], part);
                acc[mt][i] = fmaf(dxv[i], part, acc[mt][i]);
            }
        }
        if (more) stash(buf ^ 1u);
        sync_after_loads();
    }
    store_tile(a, acc, t0, j, g);
}

// ---- Q4_K and Q5_K, whole unsliced k: 32 x 32 x 32 matrix instructions ---------------------
// The same arithmetic on tiles of 32 tokens x 64 rows, two waves a workgroup (32 rows each, four
// workgroups a CU): v_mfma_i32_32x32x32_i8 does a unit of 32 x 32 outputs in half the time four
// 16 x 16 x 32 take, and matrix and vector instructions of a SIMD do not overlap here, so the
// matrix instructions' own time counts. Lane l holds row l % 32 of its wave and positions
// 16 (l / 32) .. + 15 of a unit (Q4_K, Q5_K). Tokens and weights both arrive in LDS by whole-line direct
// loads, a step ahead: token lines unpadded with their 16-byte chunks XOR-permuted (chunk c of
// token t at position c ^ (t % 16): the fragment reads of sixteen tokens fall in sixteen bank
// groups), a wave's 32 rows' blocks as stored.
typedef int i32x16 __attribute__((ext_vector_type(16)));

struct W16Q4 {
    static constexpr uint32_t BLOCK = 144;
    struct Raw {
        iu32x4 h;      // d, dmin and the twelve scale bytes
        iu32x4 q[4];   // the lane's 16 bytes of each 64-weight chunk: low nibbles unit 2c, high 2c + 1
    };
    static __device__ __forceinline__ void load(const uint8_t *blk, uint32_t h, Raw &r) {
        r.h = *reinterpret_cast<const iu32x4 *>(blk);
#pragma unroll
        for (uint32_t c = 0; c < 4; c++) r.q[c] = *reinterpret_cast<const iu32x4 *>(blk + 16u + 32u * c + 16u * h);
    }
    static __device__ __forceinline__ iu32x4 unit(const Raw &r, uint32_t u) {
        iu32x4 b = r.q[u >> 1];
        if (u & 1u) b = b >> 4;
        return b & 0x0f0f0f0fu;
    }
};

struct W16Q5 {
    static constexpr uint32_t BLOCK = 176;
    struct Raw {
        iu32x4 h;
        iu32x4 qh;     // the fifth bits of positions 16 h .. + 15, bit u for unit u
        iu32x4 q[4];
    };
    static __device__ __forceinline__ void load(const uint8_t *blk, uint32_t h, Raw &r) {
        r.h = *reinterpret_cast<const iu32x4 *>(blk);
        r.qh = *reinterpret_cast<const iu32x4 *>(blk + 16u + 16u * h);
#pragma unroll
        for (uint32_t c = 0; c < 4; c++) r.q[c] = *reinterpret_cast<const iu32x4 *>(blk + 48u + 32u * c + 16u * h);
    }
    static __device__ __forceinline__ iu32x4 unit(const Raw &r, uint32_t u) {
        iu32x4 b = r.q[u >> 1];
        if (u & 1u) b = b >> 4;
        return (b & 0x0f0f0f0fu) | (((r.qh >> u) & 0x01010101u) << 4);
    }
};

// Q6_K and Q3_K have a scale per sixteen weights: a unit is two v_mfma_i32_32x32x16_i8, lane l
// holding positions 8 (l / 32) .. + 7 of each half. The formats' readers above serve: their
// lane group g of four becomes h (first half) and 2 + h (second half).
struct W8Q6 {
    static constexpr uint32_t BLOCK = I8Q6::BLOCK;
    struct Raw { I8Q6::Raw half[2]; };
    static __device__ __forceinline__ void load(const uint8_t *blk, uint32_t h, Raw &r) {
        I8Q6::load(blk, h, r.half[0]);
        I8Q6::load(blk, 2u + h, r.half[1]);
    }
    static __device__ __forceinline__ void unit(const Raw &r, uint32_t u, uint32_t h, iu32x2 (&b)[2], int (&sc)[2]) {
        int s0, s1, mn;
        I8Q6::unit(r.half[0], u, h, b[0], s0, s1, mn);
        sc[0] = s0;
        I8Q6::unit(r.half[1], u, 2u + h, b[1], s0, s1, mn);
        sc[1] = s1;
    }
    static __device__ __forceinline__ float scale(const Raw &r) { return half_bits_to_float(r.half[0].d & 0xffffu); }
};
struct W8Q3 {
    static constexpr uint32_t BLOCK = I8Q3::BLOCK;
    struct Raw { I8Q3::Raw all; };
    static __device__ __forceinline__ void load(const uint8_t *blk, uint32_t h, Raw &r) { I8Q3::load(blk, h, r.all); }
    static __device__ __forceinline__ void unit(const Raw &r, uint32_t u, uint32_t h, iu32x2 (&b)[2], int (&sc)[2]) {
        int s0, s1, mn;
        I8Q3::unit(r.all, u, h, b[0], s0, s1, mn);
        sc[0] = s0;
        I8Q3::unit(r.all, u, 2u + h, b[1], s0, s1, mn);
        sc[1] = s1;
    }
    static __device__ __forceinline__ float scale(const Raw &r) { return half_bits_to_float(r.all.u[0].w >> 16); }
};

constexpr uint32_t WT = 32, WN = 64;  // tokens and rows of a workgroup of the wide kernel
// The sum over k is taken in KP parts, steps KP' steps / KP .. of part KP', each added up in the
// order of its steps, and the parts as ((p0 + p1) + p2) + p3. A workgroup of the kernel for long
// steps walks all of k, part after part; the kernel for short steps (SPLIT), whose few
// tiles would leave the chip to one wave a CU walking sixteen blocks one after the other, gives a
// 32 x 32 tile four waves, a part each, which meet in LDS. The same operations on every output
// either way: how a prompt is cut into steps does not change a token's bits.
constexpr uint32_t KP = 4;
// LDS: two token buffers (32 lines of 256 bytes and 256 bytes of token scales) and one slot of
// blocks per wave: a wave reads its rows' blocks into registers at the start of a step and then
// asks for the next step's into the same slot, which nobody else reads. The two waves of a
// workgroup for long steps (32 rows each) share the token buffers; a wave of the SPLIT kernel
// has its own (its steps are not the other waves').
template <class P> constexpr uint32_t wide_wslot() { return ((32u * (P::BLOCK / 16u) + 63u) / 64u) * 1024u; }
constexpr uint32_t WIDE_TOKENS = WT * 256u + 256u;
// (27 KB a workgroup of the kernel for long steps: five of them a CU, which is what bounds its
// waves a SIMD; a buffer more would cost the fifth and a tenth of the kernel's speed)
template <class P, bool SPLIT> constexpr uint32_t wide_lds() { return SPLIT ? KP * (2u * WIDE_TOKENS + wide_wslot<P>()) : 2u * WIDE_TOKENS + 2u * wide_wslot<P>(); }

// One step's multiply: the block `cur` of the lane's row times the 32 tokens of the step in
// `base`, into `acc` (the lane's sixteen results are tokens 8 j + 4 h + i, j < 4, i < 4, of its row).
// A block's units are summed in integers (a unit's exact sum times its scale, one 24-bit
// multiply-add a result; Q4_K / Q5_K minimums by one more matrix instruction a unit whose second
// operand is the unit's minimum in all 32 positions, accumulated by the matrix cores), and the
// block's f32 scales are applied once.
template <class P, bool HALVES>
__device__ __forceinline__ void wide_multiply(const typename P::Raw &cur, const uint8_t *base, uint32_t a_line, uint32_t a_key, uint32_t h, float (&acc)[16]) {
    constexpr uint32_t DX_AT = WT * 256u;
    i32x16 isum = {}, msum = {};
    const i32x16 zero = {};
    // The eight 6-bit scales and minimums of a Q4_K / Q5_K block as bytes of four words
    // (src/ref/tensor.zig:94-98), unpacked four at a time.
    uint32_t sc4[2] = {0u, 0u}, mn4[2] = {0u, 0u};
    if constexpr (!HALVES) {
        sc4[0] = cur.h.y & 0x3f3f3f3fu;
        mn4[0] = cur.h.z & 0x3f3f3f3fu;
        sc4[1] = (cur.h.w & 0x0f0f0f0fu) | ((cur.h.y >> 2) & 0x30303030u);
        mn4[1] = ((cur.h.w >> 4) & 0x0f0f0f0fu) | ((cur.h.z >> 2) & 0x30303030u);
    }
#pragma unroll
    for (uint32_t u = 0; u < 8; u++) {
        if constexpr (HALVES) {
            iu32x2 w8[2];
            int sc[2];
            P::unit(cur, u, h, w8, sc);
#pragma unroll
            for (uint32_t half = 0; half < 2; half++) {
                const long af = *reinterpret_cast<const long *>(base + a_line + 16u * ((2u * u + half) ^ a_key) + 8u * h);
                const i32x16 is = __builtin_amdgcn_mfma_i32_32x32x16_i8(af, as_operand(w8[half]), zero, 0, 0, 0);
#pragma unroll
                for (int e = 0; e < 16; e++) isum[e] = __mul24(sc[half], is[e]) + isum[e];
            }
        } else {
            const int scale = (int)((sc4[u >> 2] >> (8u * (u & 3u))) & 0xffu);
            const iu32x4 w16 = P::unit(cur, u);
            const uint32_t m4 = __builtin_amdgcn_perm(0u, mn4[u >> 2], 0x01010101u * (u & 3u));  // the unit's minimum in every byte
            const i32x4 af = *reinterpret_cast<const i32x4 *>(base + a_line + 16u * ((2u * u + h) ^ a_key));
            const i32x16 is = __builtin_amdgcn_mfma_i32_32x32x32_i8(af, __builtin_bit_cast(i32x4, w16), zero, 0, 0, 0);
            msum = __builtin_amdgcn_mfma_i32_32x32x32_i8(af, __builtin_bit_cast(i32x4, iu32x4{m4, m4, m4, m4}), msum, 0, 0, 0);
#pragma unroll
            for (int e = 0; e < 16; e++) isum[e] = __mul24(scale, is[e]) + isum[e];
        }
    }
    float d, dmin = 0.f;
    if constexpr (HALVES) {
        d = P::scale(cur);
    } else {
        d = half_bits_to_float(cur.h.x & 0xffffu);
        dmin = half_bits_to_float(cur.h.x >> 16);
    }
#pragma unroll
    for (uint32_t jj = 0; jj < 4; jj++) {
        const if32x4 dxv = *reinterpret_cast<const if32x4 *>(base + DX_AT + 4u * (8u * jj + 4u * h));
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int e = 4 * jj + i;
            float part = d * (float)isum[e];
            if (!HALVES) part = fmaf(-dmin, (float)msum[e], part);
            acc[e] = fmaf(dxv[i], part, acc[e]);
        }
    }
}

// The lane's sixteen sums to their outputs.
__device__ __forceinline__ void wide_store(const I8Args &a, uint32_t j, uint32_t t0, uint32_t h, const float (&total)[16]) {
    if (j >= a.n) return;
    float *out = a.out + a.col0 + j;
#pragma unroll
    for (uint32_t e = 0; e < 16; e++) {
        const uint32_t t = t0 + 8u * (e >> 2) + 4u * h + (e & 3u);
        if (t >= a.rows) continue;
        float *o = out + (size_t)t * a.out_stride;
        *o = a.accumulate ? *o + total[e] : total[e];
    }
}

// Long steps: 32 tokens x 64 rows a workgroup, a wave 32 rows over all of k. (The step's multiply
// is written out here, the same operations as wide_multiply.)
template <class P, bool HALVES>
__global__ __launch_bounds__(128) void matmul_kquant_i8_wide_kernel(I8Args a) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_wide[];
    constexpr uint32_t CPR = P::BLOCK / 16u, WLOADS = (32u * CPR + 63u) / 64u, WSLOT = wide_wslot<P>();
    constexpr uint32_t DX_AT = WT * 256u, W_AT = 2u * WIDE_TOKENS;
    const uint32_t tid = threadIdx.x, lane = tid & 63u, lrow = lane & 31u, h = lane >> 5;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t n0 = blockIdx.x * WN, t0 = blockIdx.y * WT;
    const uint32_t steps = a.k / 256u;
    const __amdgpu_buffer_rsrc_t xbuf = make_buffer(a.qx, a.qx_bytes), wbuf = make_buffer(a.w, a.w_bytes), dbuf = make_buffer(a.dx, a.dx_bytes);
    uint8_t *slot = lds_wide + W_AT + wave * WSLOT;

    // Loads of a step. Tokens: load i of this wave brings tokens 4 (4 wave + i) .. + 3, lane l
    // token l / 16 of them and the chunk that belongs at position l % 16. Token scales: wave 0,
    // lanes below 32 a token each (the others ask past the buffer). Weights: the wave's 32 rows.
    uint32_t xoff[4], woff[WLOADS];
#pragma unroll
    for (uint32_t i = 0; i < 4; i++) {
        const uint32_t t = 4u * (4u * wave + i) + (lane >> 4);
        xoff[i] = (t0 + t) * a.k + 16u * ((lane & 15u) ^ (t & 15u));
    }
#pragma unroll
    for (uint32_t i = 0; i < WLOADS; i++) {
        const uint32_t c = 64u * i + lane;
        woff[i] = c < 32u * CPR ? (n0 + 32u * wave + c / CPR) * a.row_bytes + 16u * (c % CPR) : 0xfffffff0u - a.row_bytes;
    }
    const uint32_t doff = lane < 32u ? (t0 + lane) * (a.k / 256u) * 4u : 0xfffffff0u - a.k;
    auto fetch_tokens = [&](uint32_t s, uint32_t buf) __attribute__((always_inline)) {
        uint8_t *base = lds_wide + buf * WIDE_TOKENS;
#pragma unroll
        for (uint32_t i = 0; i < 4; i++) load_lds_b128(xbuf, base + 1024u * (4u * wave + i), xoff[i], 256u * s);
        if (wave == 0u) load_lds_b32(dbuf, base + DX_AT, doff + 4u * s);
    };
    auto fetch_weights = [&](uint32_t s) __attribute__((always_inline)) {
#pragma unroll
        for (uint32_t i = 0; i < WLOADS; i++) load_lds_b128(wbuf, slot + 1024u * i, woff[i], s * P::BLOCK);
    };

    float acc[16];
#pragma unroll
    for (int e = 0; e < 16; e++) acc[e] = 0.f;
    const uint32_t a_line = lrow * 256u, a_key = lrow & 15u;

    // At a part's last step the part's sums join the total of the parts before it.
    float total[16];
#pragma unroll
    for (int e = 0; e < 16; e++) total[e] = 0.f;
    uint32_t part = 0;
    auto close = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int e = 0; e < 16; e++) {
            total[e] = part == 0u ? acc[e] : total[e] + acc[e];
            acc[e] = 0.f;
        }
        part++;
    };
    fetch_tokens(0, 0);
    fetch_weights(0);
    sync_after_loads();
    for (uint32_t s = 0; s < steps; s++) {
        while (s >= (part + 1u) * steps / KP) close();
        const uint32_t buf = s & 1u;
        const uint8_t *base = lds_wide + buf * WIDE_TOKENS;
        typename P::Raw cur;
        P::load(slot + lrow * P::BLOCK, h, cur);
        if (s + 1u < steps) {
            fetch_tokens(s + 1u, buf ^ 1u);
            // The slot is refilled once this wave's reads of it have returned; the compiler, which
            // sees no dependency between the two, must not move the loads up.
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            fetch_weights(s + 1u);
        }
        // A block's units are summed in integers (a unit's exact sum times its scale, one 24-bit
        // multiply-add a result; Q4_K / Q5_K minimums by one more matrix instruction a unit whose
        // second operand is the unit's minimum in all 32 positions, accumulated by the matrix
        // cores), and the block's f32 scales are applied once.
        i32x16 isum = {}, msum = {};
        const i32x16 zero = {};
        // The eight 6-bit scales and minimums of a Q4_K / Q5_K block as bytes of four words
        // (src/ref/tensor.zig:94-98), unpacked four at a time.
        uint32_t sc4[2] = {0u, 0u}, mn4[2] = {0u, 0u};
        if constexpr (!HALVES) {
            sc4[0] = cur.h.y & 0x3f3f3f3fu;
            mn4[0] = cur.h.z & 0x3f3f3f3fu;
            sc4[1] = (cur.h.w & 0x0f0f0f0fu) | ((cur.h.y >> 2) & 0x30303030u);
            mn4[1] = ((cur.h.w >> 4) & 0x0f0f0f0fu) | ((cur.h.z >> 2) & 0x30303030u);
        }
#pragma unroll
        for (uint32_t u = 0; u < 8; u++) {
            if constexpr (HALVES) {
                iu32x2 w8[2];
                int sc[2];
                P::unit(cur, u, h, w8, sc);
#pragma unroll
                for (uint32_t half = 0; half < 2; half++) {
                    const long af = *reinterpret_cast<const long *>(base + a_line + 16u * ((2u * u + half) ^ a_key) + 8u * h);
                    const i32x16 is = __builtin_amdgcn_mfma_i32_32x32x16_i8(af, as_operand(w8[half]), zero, 0, 0, 0);
#pragma unroll
                    for (int e = 0; e < 16; e++) isum[e] = __mul24(sc[half], is[e]) + isum[e];
                }
            } else {
                const int scale = (int)((sc4[u >> 2] >> (8u * (u & 3u))) & 0xffu);
                const iu32x4 w16 = P::unit(cur, u);
                const uint32_t m4 = __builtin_amdgcn_perm(0u, mn4[u >> 2], 0x01010101u * (u & 3u));  // the unit's minimum in every byte
                const i32x4 af = *reinterpret_cast<const i32x4 *>(base + a_line + 16u * ((2u * u + h) ^ a_key));
                const i32x16 is = __builtin_amdgcn_mfma_i32_32x32x32_i8(af, __builtin_bit_cast(i32x4, w16), zero, 0, 0, 0);
                msum = __builtin_amdgcn_mfma_i32_32x32x32_i8(af, __builtin_bit_cast(i32x4, iu32x4{m4, m4, m4, m4}), msum, 0, 0, 0);
#pragma unroll
                for (int e = 0; e < 16; e++) isum[e] = __mul24(scale, is[e]) + isum[e];
            }
        }
        float d, dmin = 0.f;
        if constexpr (HALVES) {
            d = P::scale(cur);
        } else {
            d = half_bits_to_float(cur.h.x & 0xffffu);
            dmin = half_bits_to_float(cur.h.x >> 16);
        }
        // The lane's sixteen results are tokens 8 j + 4 h + i, j < 4, i < 4, of its row.
#pragma unroll
        for (uint32_t jj = 0; jj < 4; jj++) {
            const if32x4 dxv = *reinterpret_cast<const if32x4 *>(base + DX_AT + 4u * (8u * jj + 4u * h));
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int e = 4 * jj + i;
                float part = d * (float)isum[e];
                if (!HALVES) part = fmaf(-dmin, (float)msum[e], part);
                acc[e] = fmaf(dxv[i], part, acc[e]);
            }
        }
        sync_after_loads();
    }
    while (part < KP) close();
    const uint32_t j = n0 + 32u * wave + lrow;
    if (j >= a.n) return;
    float *out = a.out + a.col0 + j;
#pragma unroll
    for (uint32_t e = 0; e < 16; e++) {
        const uint32_t t = t0 + 8u * (e >> 2) + 4u * h + (e & 3u);
        if (t >= a.rows) continue;
        float *o = out + (size_t)t * a.out_stride;
        *o = a.accumulate ? *o + total[e] : total[e];
    }
}

// Short steps: 32 tokens x 32 rows a workgroup of KP waves, wave p over part p of k. A wave has
// token buffers and a weight slot of its own and waits for nobody until the parts meet: waves
// 1 .. 3 leave their sums in LDS (their token buffers, done with) and wave 0 adds.
template <class P, bool HALVES>
__global__ __launch_bounds__(64 * KP) void matmul_kquant_i8_split_kernel(I8Args a) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_wide[];
    constexpr uint32_t CPR = P::BLOCK / 16u, WLOADS = (32u * CPR + 63u) / 64u, WSLOT = wide_wslot<P>(), WAVE_LDS = 2u * WIDE_TOKENS + WSLOT;
    constexpr uint32_t DX_AT = WT * 256u;
    const uint32_t tid = threadIdx.x, lane = tid & 63u, lrow = lane & 31u, h = lane >> 5;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t n0 = blockIdx.x * 32u, t0 = blockIdx.y * WT;
    const uint32_t steps = a.k / 256u;
    const __amdgpu_buffer_rsrc_t xbuf = make_buffer(a.qx, a.qx_bytes), wbuf = make_buffer(a.w, a.w_bytes), dbuf = make_buffer(a.dx, a.dx_bytes);
    uint8_t *tokens = lds_wide + wave * WAVE_LDS, *slot = tokens + 2u * WIDE_TOKENS;

    // Loads of a step: the 32 tokens (load i brings tokens 4 i .. + 3, lane l token l / 16 of them
    // and the chunk that belongs at position l % 16), their scales, the 32 rows' blocks.
    uint32_t xoff[8], woff[WLOADS];
#pragma unroll
    for (uint32_t i = 0; i < 8; i++) {
        const uint32_t t = 4u * i + (lane >> 4);
        xoff[i] = (t0 + t) * a.k + 16u * ((lane & 15u) ^ (t & 15u));
    }
#pragma unroll
    for (uint32_t i = 0; i < WLOADS; i++) {
        const uint32_t c = 64u * i + lane;
        woff[i] = c < 32u * CPR ? (n0 + c / CPR) * a.row_bytes + 16u * (c % CPR) : 0xfffffff0u - a.row_bytes;
    }
    const uint32_t doff = lane < 32u ? (t0 + lane) * (a.k / 256u) * 4u : 0xfffffff0u - a.k;
    auto fetch = [&](uint32_t s) __attribute__((always_inline)) {
        uint8_t *base = tokens + (s & 1u) * WIDE_TOKENS;
#pragma unroll
        for (uint32_t i = 0; i < 8; i++) load_lds_b128(xbuf, base + 1024u * i, xoff[i], 256u * s);
        load_lds_b32(dbuf, base + DX_AT, doff + 4u * s);
#pragma unroll
        for (uint32_t i = 0; i < WLOADS; i++) load_lds_b128(wbuf, slot + 1024u * i, woff[i], s * P::BLOCK);
    };

    float acc[16];
#pragma unroll
    for (int e = 0; e < 16; e++) acc[e] = 0.f;
    const uint32_t a_line = lrow * 256u, a_key = lrow & 15u;
    const uint32_t first = wave * steps / KP, last = (wave + 1u) * steps / KP;
    if (first < last) {
        fetch(first);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        for (uint32_t s = first; s < last; s++) {
            const uint8_t *base = tokens + (s & 1u) * WIDE_TOKENS;
            typename P::Raw cur;
            P::load(slot + lrow * P::BLOCK, h, cur);
            // The next step's loads go out once this wave's reads of the slot (and, a step ago,
            // of the other token buffer) have returned; the compiler, which sees no dependency
            // between the two, must not move the loads up.
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            if (s + 1u < last) fetch(s + 1u);
            wide_multiply<P, HALVES>(cur, base, a_line, a_key, h, acc);
            asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        }
    }
    float *mine = reinterpret_cast<float *>(tokens) + lane;
    if (wave != 0u) {
#pragma unroll
        for (int e = 0; e < 16; e++) mine[64 * e] = acc[e];
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if (wave != 0u) return;
    float total[16];
#pragma unroll
    for (int e = 0; e < 16; e++) {
        const float *theirs = reinterpret_cast<const float *>(lds_wide) + 64 * e + lane;
        total[e] = ((acc[e] + theirs[1u * WAVE_LDS / 4u]) + theirs[2u * WAVE_LDS / 4u]) + theirs[3u * WAVE_LDS / 4u];
    }
    wide_store(a, n0 + lrow, t0, h, total);
}

template <class P, bool HALVES, bool SPLIT>
zhip_result launch_kquant_wide_as(const Dispatch &d, const char *name, const I8Args &a) {
    constexpr uint32_t bytes = wide_lds<P, SPLIT>();
    const void *kernel;
    if constexpr (SPLIT) kernel = reinterpret_cast<const void *>(matmul_kquant_i8_split_kernel<P, HALVES>);
    else kernel = reinterpret_cast<const void *>(matmul_kquant_i8_wide_kernel<P, HALVES>);
    static bool configured = false;
    if (!configured) {
        if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess) {
            (void)hipGetLastError();
            return fail(d, ZHIP_E_GPU, "%s: cannot reserve %u bytes of LDS", name, bytes);
        }
        configured = true;
    }
    const dim3 grid((a.n + (SPLIT ? 32u : WN) - 1u) / (SPLIT ? 32u : WN), (a.rows + WT - 1u) / WT);
    if constexpr (SPLIT) hipLaunchKernelGGL((matmul_kquant_i8_split_kernel<P, HALVES>), grid, dim3(64u * KP), bytes, d.stream, a);
    else hipLaunchKernelGGL((matmul_kquant_i8_wide_kernel<P, HALVES>), grid, dim3(128u), bytes, d.stream, a);
    return check_launch(d, name);
}

// Steps whose 32-token x 64-row tiles are fewer than 1.75 a CU (three where a wave's walk is 32
// blocks or more) take the kernel that gives a tile's k to four waves. Measured, Q4_K, the
// multiply alone, weights from HBM: 64 x 4096 x 4096 21.2 -> 9.3 us, 128 tokens 21.3 -> 16.1,
// 256 tokens 30.4 against 29.8 (left as it is), 64 x 14336 x 4096 65.4 -> 21.5, 256 tokens
// 96.1 -> 75.4, 384 tokens 96.9 against 111.3 (left); 192 x 4096 x 4096 (1.5 tiles a CU)
// 30.6 -> 23.0, 64 x 4096 x 14336 (1.75) 28.5 against 31.8 (left).
template <class P, bool HALVES>
zhip_result launch_kquant_wide(const Dispatch &d, const char *name, const I8Args &a) {
    const uint64_t tiles = (uint64_t)((a.n + WN - 1u) / WN) * ((a.rows + WT - 1u) / WT);
    const bool split = 4u * tiles < (a.k >= 32u * 256u ? 12ull : 7ull) * (uint64_t)d.dev->compute_units;
    return split ? launch_kquant_wide_as<P, HALVES, true>(d, name, a) : launch_kquant_wide_as<P, HALVES, false>(d, name, a);
}

// The K-format kernel's weight buffers are dynamic LDS (with the static token buffers a
// workgroup takes 57 - 66 KB, two workgroups a CU).
template <class P>
zhip_result launch_kquant(const Dispatch &d, const char *name, dim3 grid, const I8Args &a) {
    constexpr uint32_t bytes = 2u * 4u * ((16u * (P::BLOCK / 16u) + 63u) / 64u) * 1024u;
    auto kernel = matmul_kquant_i8_kernel<P>;
    static bool configured = false;
    if (!configured) {
        if (hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess) {
            (void)hipGetLastError();
            return fail(d, ZHIP_E_GPU, "%s: cannot reserve %u bytes of LDS", name, bytes);
        }
        configured = true;
    }
    hipLaunchKernelGGL(kernel, grid, dim3(256), bytes, d.stream, a);
    return check_launch(d, name);
}

}  // namespace

// matmul_q8_i8.hip
bool matmul_q8_i8_accepts(uint32_t k, uint32_t k_slice, uint32_t slices);
zhip_result launch_matmul_q8_i8(const Dispatch &d, const char *name, const uint8_t *qx, const uint8_t *w, const uint8_t *dx, float *out, uint32_t rows,
    uint32_t n, uint32_t k, uint32_t col0, uint32_t out_stride, uint32_t accumulate, uint32_t row_bytes, uint32_t qx_bytes, uint32_t w_bytes,
    uint32_t dx_bytes);

// matmul_quant.wgsl's workgroup is 128 outputs x 32 tokens: the grid says how
// much of the product a dispatch covers, whatever tiling computes it.
static zhip_result launch_int8(const Dispatch &d, const char *name, int type) {
    if (d.params_size < sizeof(MatmulParams)) return fail(d, ZHIP_E_BAD_COMMAND, "%s: params block too small", name);
    const MatmulParams &p = *reinterpret_cast<const MatmulParams *>(d.params);
    for (int b = 1; b <= 4; b++)
        if (!d.bind[b].bound) return fail(d, ZHIP_E_BAD_COMMAND, "%s: binding %d is not bound", name, b);
    if (d.grid[0] == 0 || d.grid[1] == 0 || d.grid[2] == 0) return ZHIP_OK;
    const uint32_t act = type == 8 ? 32u : 256u;
    if (p.k == 0 || p.k % act != 0) return fail(d, ZHIP_E_BAD_COMMAND, "%s: k = %u is not a multiple of %u", name, p.k, act);
    if (p.k_slice == 0 || p.k_slice % 32u != 0) return fail(d, ZHIP_E_BAD_COMMAND, "%s: k_slice = %u", name, p.k_slice);
    const uint64_t slices = d.grid[2];
    if ((slices - 1) * p.k_slice >= p.k) return fail(d, ZHIP_E_BAD_COMMAND, "%s: %u slices of %u exceed k = %u", name, (uint32_t)slices, p.k_slice, p.k);
    const uint64_t cover_n = (uint64_t)d.grid[0] * 128u, cover_t = (uint64_t)d.grid[1] * 32u;
    const uint64_t n = cover_n < p.n ? cover_n : p.n, rows = cover_t < p.rows ? cover_t : p.rows;
    if (n == 0 || rows == 0) return ZHIP_OK;
    const uint32_t block = type == 3 ? I8Q3::BLOCK : type == 4 ? I8Q4::BLOCK : type == 5 ? I8Q5::BLOCK : I8Q6::BLOCK;
    const uint64_t row_bytes = type == 8 ? (((uint64_t)p.k + p.k / 16u + 15u) & ~15ull) : (uint64_t)p.k / 256u * block;
    const uint64_t x_need = rows * p.k, d_need = rows * (p.k / act) * 4u, w_need = n * row_bytes;
    const uint64_t o_need = ((slices - 1) * p.slice_stride + (rows - 1) * p.out_stride + p.col0 + n) * 4u;
    if (x_need > d.bind[1].size || w_need > d.bind[2].size || o_need > d.bind[3].size || d_need > d.bind[4].size)
        return fail(d, ZHIP_E_BAD_COMMAND, "%s: bound ranges too small (qx %llu/%llu, w %llu/%llu, out %llu/%llu, dx %llu/%llu)", name,
            (unsigned long long)x_need, (unsigned long long)d.bind[1].size, (unsigned long long)w_need, (unsigned long long)d.bind[2].size,
            (unsigned long long)o_need, (unsigned long long)d.bind[3].size, (unsigned long long)d_need, (unsigned long long)d.bind[4].size);
    if (((uintptr_t)d.bind[1].ptr | (uintptr_t)d.bind[2].ptr) & 15u) return fail(d, ZHIP_E_BAD_COMMAND, "%s: qx and weights must be 16-byte aligned", name);
    if (((uintptr_t)d.bind[3].ptr | (uintptr_t)d.bind[4].ptr) & 3u) return fail(d, ZHIP_E_BAD_COMMAND, "%s: out and dx must be 4-byte aligned", name);
    // The kernels index with 32-bit byte offsets, up to a tile past the last token and row.
    if ((rows + 2u * TT) * p.k >= (1ull << 32) || (n + 2u * TN) * row_bytes >= (1ull << 32))
        return fail(d, ZHIP_E_BAD_COMMAND, "%s: operands of 4 GiB or more", name);
    const uint64_t tiles_n = (n + TN - 1) / TN, tiles_t = (rows + TT - 1) / TT;
    if (tiles_t > 65535u || slices > 65535u) return fail(d, ZHIP_E_BAD_COMMAND, "%s: grid too large", name);
    I8Args a{};
    a.qx = d.bind[1].ptr;
    a.w = d.bind[2].ptr;
    a.out = reinterpret_cast<float *>(d.bind[3].ptr);
    a.dx = d.bind[4].ptr;
    a.rows = (uint32_t)rows; a.n = (uint32_t)n; a.k = p.k; a.col0 = p.col0; a.out_stride = p.out_stride;
    a.accumulate = p.accumulate; a.k_slice = p.k_slice; a.slice_stride = p.slice_stride; a.row_bytes = (uint32_t)row_bytes;
    a.qx_bytes = (uint32_t)x_need; a.w_bytes = (uint32_t)w_need; a.dx_bytes = (uint32_t)d_need;
    if (type == 8 && matmul_q8_i8_accepts(p.k, p.k_slice, (uint32_t)slices))
        return launch_matmul_q8_i8(d, name, a.qx, a.w, a.dx, a.out, a.rows, a.n, a.k, a.col0, a.out_stride, a.accumulate, a.row_bytes, a.qx_bytes,
            a.w_bytes, a.dx_bytes);
    const dim3 grid((uint32_t)tiles_n, (uint32_t)tiles_t, (uint32_t)slices);
    const bool ragged = p.k % STEP != 0 || (p.k_slice < p.k && p.k_slice % STEP != 0);
    const bool whole = slices == 1u && p.k_slice >= p.k;
    if (whole && type == 4) return launch_kquant_wide<W16Q4, false>(d, name, a);
    if (whole && type == 5) return launch_kquant_wide<W16Q5, false>(d, name, a);
    if (whole && type == 6) return launch_kquant_wide<W8Q6, true>(d, name, a);
    if (whole && type == 3) return launch_kquant_wide<W8Q3, true>(d, name, a);
    if (type == 3) {
        return launch_kquant<I8Q3>(d, name, grid, a);
    } else if (type == 4) {
        return launch_kquant<I8Q4>(d, name, grid, a);
    } else if (type == 5) {
        return launch_kquant<I8Q5>(d, name, grid, a);
    } else if (type == 6) {
        return launch_kquant<I8Q6>(d, name, grid, a);
    } else {
        if (ragged) hipLaunchKernelGGL(matmul_q8_0_i8_kernel<true>, grid, dim3(256), 0, d.stream, a);
        else hipLaunchKernelGGL(matmul_q8_0_i8_kernel<false>, grid, dim3(256), 0, d.stream, a);
    }
    return check_launch(d, name);
}

zhip_result launch_matmul_q8_0(const Dispatch &d) { return launch_int8(d, "matmul_q8_0", 8); }
zhip_result launch_matmul_q3_k(const Dispatch &d) { return launch_int8(d, "matmul_q3_k", 3); }
zhip_result launch_matmul_q4_k(const Dispatch &d) { return launch_int8(d, "matmul_q4_k", 4); }
zhip_result launch_matmul_q5_k(const Dispatch &d) { return launch_int8(d, "matmul_q5_k", 5); }
zhip_result launch_matmul_q6_k(const Dispatch &d) { return launch_int8(d, "matmul_q6_k", 6); }

}  // namespace zhip
