// matvec_q4_k, matrix-core variant: the decode multiply for steps of up to eight
// tokens with the per-weight work done once for all of them. Selected by the
// MatvecVariant (wg 512, lanes 64, rows 16): a 64-lane wave per sixteen rows.
// Same contract as the other variants (src/kernels/matvec_quant.wgsl.hbs) for
// the SILU_PAIR and ACCUMULATE epilogues; a launch with a prologue (NORM,
// act_div) or a k that is not a multiple of 1024 runs the default variant.
//
// Arithmetic. v_mfma_f32_16x16x32_f16 multiplies sixteen rows of inputs by
// sixteen weight rows over one 32-weight sub-block. The weights enter as exact
// f16 values 16 + q (the nibble dropped into the mantissa of 16.0: a shift and
// an and-or per pair, no conversion); every token enters as two rows, the f16
// rounding of its inputs and the f16 rounding of what that left times 2^11, so
// an input keeps 22 bits and every product is exact in the f32 accumulator. A
// token's inputs are first scaled by a power of two that puts its largest
// magnitude at 2^14, so neither half leaves f16's range; the result is scaled
// back. A sub-block's sum S = sum((16 + q) x) then gives the block formula as
// d sc S - (16 d sc + dmin m) X with X = sum(x), itself a product of the same
// rows with a column of ones. A token's results do not depend on how many
// tokens share the launch: its rows meet no other token's anywhere.
//
// Layout of the work. A 512-thread workgroup takes eight weight tiles of
// sixteen rows, one per wave (with SILU_PAIR the gate tile and the up tile of
// four output tiles; the odd waves hand their results to the even ones through
// LDS). The inputs are processed in slabs of 1024 positions: the next slab's
// f32 values arrive in LDS by direct loads while the current one is multiplied,
// are split into the f16 rows once per workgroup, and their sub-block sums are
// taken by the matrix cores, four sub-blocks a wave. Each wave streams its own
// tile's blocks (sixteen rows x 144 bytes = 144 sixteen-byte chunks, three
// direct loads) through a private ring of three LDS slots, two blocks ahead,
// and waits for exactly the loads it needs (s_waitcnt vmcnt(n)); nothing but
// the slab hand-over needs a barrier.
#include <hip/hip_runtime.h>

#include "common.h"
#include "decode.h"
#include "matvec_common.h"

namespace zhip {

typedef _Float16 mf16x8 __attribute__((ext_vector_type(8)));
typedef float mf32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t mu32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t mu32x2 __attribute__((ext_vector_type(2)));

namespace {

constexpr uint32_t THREADS = 512, WAVES = 8;
constexpr uint32_t SLAB = 1024;                    // positions per slab: four blocks, 32 sub-blocks
constexpr uint32_t AROW = 2u * SLAB + 16u;         // bytes between the f16 rows: 16 rows hit 16 bank groups
constexpr uint32_t ABYTES = 16u * AROW;
constexpr uint32_t XRAW = 8u * SLAB * 4u;          // the next slab's f32 inputs, [token][1024]
constexpr uint32_t SLOT = 3u * 1024u;              // 2304 bytes of blocks; the third load's idle lanes land behind them
constexpr uint32_t DEPTH = 3;
constexpr uint32_t RING = WAVES * DEPTH * SLOT;
constexpr uint32_t XSUM = 32u * 8u * 4u;           // [sub-block][token] sums of the slab
constexpr uint32_t PAIRBUF = 4u * 8u * 16u * 4u;   // [output tile][token][row] up-row results

struct MfArgs {
    MvArgs a;
    uint32_t x_bytes, w_bytes;  // the bound ranges, for the range-checked loads
    uint32_t nibble_mask, sixteen;  // 0x03C003C0, 0x4C004C00 (see nibbles_f16)
};

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_buffer(const void *base, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, 0x00020000);
}

typedef __attribute__((address_space(3))) void *lds_ptr;

// One wave-wide load of 16 bytes a lane straight into LDS (lane l lands at
// dst + 16 l). The destination reaches the load as a bare LDS address, so the
// compiler keeps no dependency between these loads and later LDS reads; the
// explicit waits below order them.
__device__ __forceinline__ void load_lds_b128(__amdgpu_buffer_rsrc_t buf, uint8_t *dst, uint32_t offset) {
    uint32_t address = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)dst);
    asm volatile("" : "+s"(address));
    __builtin_amdgcn_raw_ptr_buffer_load_lds(buf, (lds_ptr)(uintptr_t)address, 16, offset, 0, 0, 0);
}

template <int LEFT>
__device__ __forceinline__ void wait_loads() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(LEFT) : "memory");
}

__device__ __forceinline__ void barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// Eight nibbles of two words as f16 values 16 + q in the order k0 k2 k1 k3 k4 k6 k5 k7
// (the inputs' rows are stored in the same order). HIGH takes the high nibbles.
// `mask` (0x03C003C0) arrives in a scalar register and `sixteen` (0x4C004C00) in a
// vector one, so each pair costs a shift and one v_and_or_b32 (an instruction
// takes one scalar or literal operand).
template <bool HIGH>
__device__ __forceinline__ mf16x8 nibbles_f16(mu32x2 w, uint32_t mask, uint32_t sixteen) {
    mu32x4 r;
    if (HIGH) {
        r.x = ((w.x << 2) & mask) | sixteen;
        r.y = ((w.x >> 6) & mask) | sixteen;
        r.z = ((w.y << 2) & mask) | sixteen;
        r.w = ((w.y >> 6) & mask) | sixteen;
    } else {
        r.x = ((w.x << 6) & mask) | sixteen;
        r.y = ((w.x >> 2) & mask) | sixteen;
        r.z = ((w.y << 6) & mask) | sixteen;
        r.w = ((w.y >> 2) & mask) | sixteen;
    }
    return __builtin_bit_cast(mf16x8, r);
}

template <bool PAIR>
__global__ __launch_bounds__(THREADS) void matvec_q4k_mfma_kernel(MfArgs q) {
    const MvArgs &a = q.a;
    __shared__ __align__(16) uint8_t lds_a[ABYTES];
    __shared__ __align__(16) uint8_t lds_raw[XRAW];
    __shared__ __align__(16) uint8_t lds_ring[RING];
    __shared__ __align__(16) float lds_x[XSUM / 4u];
    __shared__ __align__(16) float lds_pair[PAIRBUF / 4u];
    __shared__ float lds_scale[16];  // [8] scale, [8] its inverse

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, l16 = lane & 15u, g = lane >> 4;
    const uint32_t slabs = a.k / SLAB, blocks = a.k / 256u;
    const __amdgpu_buffer_rsrc_t xbuf = make_buffer(a.x, q.x_bytes), wbuf = make_buffer(a.w, q.w_bytes);
    uint32_t sixteen = q.sixteen;
    asm volatile("" : "+v"(sixteen));

    // This wave's weight tile: sixteen rows from row0.
    uint32_t out_tile, row0;
    if (PAIR) {
        out_tile = blockIdx.x * 4u + (wave >> 1);
        row0 = (wave & 1u ? a.half : 0u) + 16u * out_tile;
    } else {
        out_tile = blockIdx.x * 8u + wave;
        row0 = 16u * out_tile;
    }
    // Chunk c of the tile's 144 per block (row c / 9, sixteen bytes c % 9): loads 0, 1, 2
    // take chunks lane, 64 + lane, 128 + lane; past 144 a lane asks beyond the buffer.
    uint32_t woff[3];
#pragma unroll
    for (uint32_t i = 0; i < 3; i++) {
        const uint32_t c = 64u * i + lane;
        woff[i] = c < 144u ? (row0 + c / 9u) * a.row_bytes + 16u * (c % 9u) : 0xfffffff0u;
    }
    uint8_t *ring = lds_ring + wave * DEPTH * SLOT;  // this wave's slots
    auto fetch_block = [&](uint32_t b) __attribute__((always_inline)) {
        uint8_t *slot = ring + (b % DEPTH) * SLOT;
        const uint32_t at = b < blocks ? b * 144u : 0xfffffff0u;
#pragma unroll
        for (uint32_t i = 0; i < 3; i++) load_lds_b128(wbuf, slot + 1024u * i, (woff[i] | at) >= 0xfffffff0u ? 0xfffffff0u : woff[i] + at);
    };
    // The slab's f32 inputs, [token][1024]: 2048 sixteen-byte chunks over the workgroup, four a thread.
    auto fetch_slab = [&](uint32_t s) __attribute__((always_inline)) {
#pragma unroll
        for (uint32_t i = 0; i < 4; i++) {
            const uint32_t c = (4u * wave + i) * 64u + lane, t = c >> 8, v = c & 255u;
            const uint32_t off = (t < a.m && s < slabs) ? (t * a.xr + s * SLAB + 4u * v) * 4u : 0xfffffff0u;
            load_lds_b128(xbuf, lds_raw + (4u * wave + i) * 1024u, off);
        }
    };

    // The first slab's inputs, then the head of the weight stream (in this order: the
    // first wait below lets the two blocks fly and so covers the inputs).
    fetch_slab(0);
    fetch_block(0);
    fetch_block(1);

    // Each token's scale: the power of two that puts its largest magnitude in [2^14, 2^15).
    if (wave < a.m) {
        const float4 *xr = reinterpret_cast<const float4 *>(a.x + (size_t)wave * a.xr);
        // Sixteen vectors a lane at a time, all loaded before any is used: one trip to memory
        // per 4096 positions, not one per vector.
        float big = 0.f;
        for (uint32_t base = lane; base < a.k / 4u; base += 1024u) {
            float4 v[16];
#pragma unroll
            for (uint32_t i = 0; i < 16; i++) v[i] = base + 64u * i < a.k / 4u ? xr[base + 64u * i] : float4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (uint32_t i = 0; i < 16; i++) big = fmaxf(fmaxf(fabsf(v[i].x), fabsf(v[i].y)), fmaxf(fmaxf(fabsf(v[i].z), fabsf(v[i].w)), big));
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) big = fmaxf(big, __shfl_xor(big, off, 64));
        if (lane == 0) {
            const int e = (int)((__float_as_uint(big) >> 23) & 0xffu);  // biased exponent; 0 for zero and subnormals
            // scale = 2^(14 - (e - 127)), kept inside f32's normal range both ways
            int se = 127 + 14 - (e - 127);
            se = se < 1 ? 1 : se > 253 ? 253 : se;
            lds_scale[wave] = (e == 0 || e == 255) ? 1.0f : __uint_as_float((uint32_t)se << 23);
            lds_scale[8 + wave] = (e == 0 || e == 255) ? 1.0f : __uint_as_float((uint32_t)(254 - se) << 23);
        }
    } else if (lane == 0) {
        lds_scale[wave] = lds_scale[8 + wave] = 1.0f;  // rows of zeros
    }

    // Rows of tokens the step does not have are zeros for good.
    for (uint32_t i = tid; i < ABYTES / 16u; i += THREADS) *reinterpret_cast<mu32x4 *>(lds_a + 16u * i) = mu32x4{0u, 0u, 0u, 0u};

    float acc[2] = {0.f, 0.f};  // tokens 2 g and 2 g + 1 for row row0 + l16
    for (uint32_t s = 0; s < slabs; s++) {
        // The slab's inputs have landed (this wave's part; the barrier covers the others')
        // and every wave is done with the previous slab's rows and sums.
        wait_loads<6>();  // only the two blocks asked for ahead may still fly
        barrier();
        // Split into the f16 rows 2 t (rounded value) and 2 t + 1 (what is left, times 2^11).
#pragma unroll
        for (uint32_t i = 0; i < 4; i++) {
            const uint32_t c = tid + THREADS * i, t = c >> 8, v = c & 255u;
            if (t >= a.m) continue;  // the same for a whole wave; absent tokens' rows stay zero
            const mf32x4 x = *reinterpret_cast<const mf32x4 *>(lds_raw + c * 16u);
            const float scale = lds_scale[t];
            _Float16 hi[4], lo[4];
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const float xs = x[e] * scale;
                hi[e] = (_Float16)xs;
                lo[e] = (_Float16)((xs - (float)hi[e]) * 2048.0f);
            }
            // Positions 4 v .. 4 v + 3 are k0 k1 k2 k3 or k4 .. k7 of their eight: stored k0 k2 k1 k3.
            typedef _Float16 h4 __attribute__((ext_vector_type(4)));
            *reinterpret_cast<h4 *>(lds_a + (2u * t) * AROW + 8u * v) = h4{hi[0], hi[2], hi[1], hi[3]};
            *reinterpret_cast<h4 *>(lds_a + (2u * t + 1u) * AROW + 8u * v) = h4{lo[0], lo[2], lo[1], lo[3]};
        }
        barrier();
        // The next slab's inputs start now; their landing is waited for below.
        fetch_slab(s + 1u);
        // Sub-block sums of the slab, four sub-blocks a wave: the rows times a column of ones.
        {
            const mu32x4 ones = {0x3C003C00u, 0x3C003C00u, 0x3C003C00u, 0x3C003C00u};
#pragma unroll
            for (uint32_t i = 0; i < 4; i++) {
                const uint32_t sb = 4u * wave + i;
                const mf16x8 xf = *reinterpret_cast<const mf16x8 *>(lds_a + l16 * AROW + 64u * sb + 16u * g);
                const mf32x4 d = __builtin_amdgcn_mfma_f32_16x16x32_f16(xf, __builtin_bit_cast(mf16x8, ones), mf32x4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
                if (l16 == 0u) {
                    lds_x[sb * 8u + 2u * g] = fmaf(d[1], 1.0f / 2048.0f, d[0]);
                    lds_x[sb * 8u + 2u * g + 1u] = fmaf(d[3], 1.0f / 2048.0f, d[2]);
                }
            }
        }
        barrier();
        // The slab's four blocks of this wave's tile.
#pragma unroll
        for (uint32_t i = 0; i < 4; i++) {
            const uint32_t b = 4u * s + i;
            fetch_block(b + 2u);
            // Newer than block b: blocks b + 1, b + 2 (three loads each) and, in a slab's
            // first two blocks, the four loads of the next slab's inputs.
            if (i < 2) wait_loads<10>();
            else wait_loads<6>();
            const uint8_t *block = ring + (b % DEPTH) * SLOT + l16 * 144u;
            const mu32x4 h = *reinterpret_cast<const mu32x4 *>(block);
            const float d = half_bits_to_float(h.x & 0xffffu), dmin = half_bits_to_float(h.x >> 16);
            // The eight 6-bit scales and minimums as bytes of four words (src/ref/tensor.zig:94-98).
            const uint32_t sc_lo = h.y & 0x3f3f3f3fu, mn_lo = h.z & 0x3f3f3f3fu;
            const uint32_t sc_hi = (h.w & 0x0f0f0f0fu) | ((h.y >> 2) & 0x30303030u);
            const uint32_t mn_hi = ((h.w >> 4) & 0x0f0f0f0fu) | ((h.z >> 2) & 0x30303030u);
#pragma unroll
            for (uint32_t c = 0; c < 4; c++) {
                const mu32x2 wq = *reinterpret_cast<const mu32x2 *>(block + 16u + 32u * c + 8u * g);
#pragma unroll
                for (uint32_t half = 0; half < 2; half++) {
                    const uint32_t sb = 2u * c + half, ssb = 8u * i + sb;  // in the block, in the slab
                    const uint32_t shift = 8u * (sb & 3u);
                    const float dsc = d * (float)(((sb < 4u ? sc_lo : sc_hi) >> shift) & 0xffu);
                    const float off = fmaf(16.0f, dsc, dmin * (float)(((sb < 4u ? mn_lo : mn_hi) >> shift) & 0xffu));
                    const mf16x8 wf = half ? nibbles_f16<true>(wq, q.nibble_mask, sixteen) : nibbles_f16<false>(wq, q.nibble_mask, sixteen);
                    const mf16x8 xf = *reinterpret_cast<const mf16x8 *>(lds_a + l16 * AROW + 64u * ssb + 16u * g);
                    const mf32x4 r = __builtin_amdgcn_mfma_f32_16x16x32_f16(xf, wf, mf32x4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
                    const float2 xs = *reinterpret_cast<const float2 *>(&lds_x[ssb * 8u + 2u * g]);
                    acc[0] = fmaf(-off, xs.x, fmaf(dsc, fmaf(r[1], 1.0f / 2048.0f, r[0]), acc[0]));
                    acc[1] = fmaf(-off, xs.y, fmaf(dsc, fmaf(r[3], 1.0f / 2048.0f, r[2]), acc[1]));
                }
            }
        }
    }
    wait_loads<0>();  // nothing may still land in LDS once the workgroup is gone

    const uint32_t ta = 2u * g, tb = ta + 1u;
    const float ra = acc[0] * lds_scale[8 + ta], rb = acc[1] * lds_scale[8 + tb];
    const uint32_t j = 16u * out_tile + l16;
    if (PAIR) {
        float *mine = lds_pair + (wave >> 1) * 128u;
        if (wave & 1u) {
            mine[ta * 16u + l16] = ra;
            mine[tb * 16u + l16] = rb;
        }
        barrier();
        if (wave & 1u) return;
        if (j >= a.rows) return;
        const float ua = mine[ta * 16u + l16], ub = mine[tb * 16u + l16];
        if (ta < a.m) {
            float *o = a.out + (size_t)ta * a.out_stride + a.col0 + j;
            const float v = silu_f(ra) * ua;
            *o = (a.flags & FLAG_ACCUMULATE) ? *o + v : v;
        }
        if (tb < a.m) {
            float *o = a.out + (size_t)tb * a.out_stride + a.col0 + j;
            const float v = silu_f(rb) * ub;
            *o = (a.flags & FLAG_ACCUMULATE) ? *o + v : v;
        }
    } else {
        if (j >= a.rows) return;
        if (ta < a.m) {
            float *o = a.out + (size_t)ta * a.out_stride + a.col0 + j;
            *o = (a.flags & FLAG_ACCUMULATE) ? *o + ra : ra;
        }
        if (tb < a.m) {
            float *o = a.out + (size_t)tb * a.out_stride + a.col0 + j;
            *o = (a.flags & FLAG_ACCUMULATE) ? *o + rb : rb;
        }
    }
}

}  // namespace

// Whether the matrix-core variant can run these (already validated) arguments.
bool matvec_q4k_mfma_accepts(const MvArgs &a) {
    return a.m >= 1 && a.m <= 8 && a.k % SLAB == 0 && !(a.flags & FLAG_NORM) && a.act_div == 0.f;
}

zhip_result launch_matvec_q4k_mfma(const Dispatch &d, const MvArgs &a, uint64_t x_bytes, uint64_t w_bytes) {
    const bool pair = a.flags & FLAG_SILU_PAIR;
    // 32-bit byte offsets, up to a tile past the last row.
    const uint64_t reach = ((uint64_t)(pair ? a.half : 0u) + a.rows + 32u) * a.row_bytes + a.row_bytes;
    if (x_bytes >= 0xfffffff0ull || w_bytes >= 0xfffffff0ull || reach >= 0xfffffff0ull) return fail(d, ZHIP_E_BAD_COMMAND, "matvec_q4_k: operands of 4 GiB or more");
    MfArgs q{a, (uint32_t)x_bytes, (uint32_t)w_bytes, 0x03C003C0u, 0x4C004C00u};
    const uint32_t out_tiles = (a.rows + 15u) / 16u;
    const uint32_t per_group = pair ? 4u : 8u;
    const uint32_t blocks = (out_tiles + per_group - 1u) / per_group;
    if (pair) hipLaunchKernelGGL(matvec_q4k_mfma_kernel<true>, dim3(blocks), dim3(THREADS), 0, d.stream, q);
    else hipLaunchKernelGGL(matvec_q4k_mfma_kernel<false>, dim3(blocks), dim3(THREADS), 0, d.stream, q);
    return check_launch(d, "matvec_q4_k");
}

}  // namespace zhip
