// matvec_q6_k and matvec_q3_k, matrix-core variant (MatvecVariant wg 512, lanes 64, rows 16) for steps of up to
// eight tokens and k = 1024, 2048 or 4096: the weight stream is read once for all tokens of the step
// and the per-weight work is done once. Contract as the default variant's
// (src/kernels/matvec_quant.wgsl.hbs with the decoder of src/kernels/quant/q6_k_dot.wgsl; block
// formula src/ref/tensor.zig:118-140): out[t][col0 + j] (+)= sum over 16-weight sub-blocks of
// d * scale * sum((q - 32) * x), q the 6-bit value of ql and qh; Q3_K (the rows repacked at
// load, src/kernels/repack_q3_k.wgsl; src/ref/tensor.zig:141-160): d * (scale - 32) * sum((q - 4) * x),
// q the two low bits and the third bit. What follows describes Q6_K; Q3_K has 128-byte blocks
// (a unit is four lines a row, all eight waves load it) and its own unpacking.
//
// Arithmetic. v_mfma_f32_32x32x16_f16 multiplies 32 rows of inputs by 32 weight rows over one
// sub-block. The weights enter as the exact f16 integers q - 32 (the byte dropped into the
// mantissa of 1024.0 by v_perm_b32, 1056 subtracted by v_pk_add_f16); every token enters as two
// rows, the f16 rounding of its inputs and the f16 rounding of what that left times 2^11, after
// a power of two has put its largest magnitude at 2^14 (an input keeps 22 bits, every product is
// exact in the f32 accumulator); the sub-block's d * scale multiplies its sum afterwards. Eight
// tokens fill sixteen of the 32 operand rows; the others are zeros. A token's rows meet no other
// token's: its results do not depend on how many tokens share the launch.
//
// Layout of the work. A launch of its own (matvec_q6k_split_kernel, one workgroup a token, the
// default variant's staging arithmetic for the RMSNorm and silu(x / act_div) prologues) writes
// the tokens' two f16 planes and inverse scales to the workspace once. In the multiply a
// 512-thread workgroup is eight waves; its tiles are 32 matrix rows, taken as units of four
// 256-weight blocks a row (896 bytes = seven whole lines of each row), wave w multiplying half
// w % 2 of block w / 2 of the unit. A unit travels as a flat copy through a ring of four LDS
// slots: the waves load it by wave-wide direct loads of whole lines (four each for seven of
// them), each wave waits for its own and one barrier a unit tells everyone that all of it has
// landed; the loads of the unit three ahead go out behind that barrier, so three units are in
// flight while one is multiplied (two slots of twice the size, one unit in flight, measured the
// same 94 us on 128256 x 4096: per 16-weight sub-block and wave the kernel issues 24 vector
// instructions and a matrix instruction that do not overlap, 0.85 us a unit and SIMD against
// the 1.1 us the unit's bytes need at full rate, and the two overlap only in part: with the
// multiplies switched off the same launch takes 80 us, 6.1 TB/s). Chunk c (16 bytes) of a line of row r sits at position
// c ^ (r % 8), which keeps the 32 rows' reads of one piece of a block to four lanes a bank. The
// waves' partial sums meet in LDS behind the same barrier, are added in the order of the blocks
// and wait there for one burst of stores when the workgroup's run ends. Workgroups are numbered
// die by die and share the rows left after whole rounds in units of eight.
#include <hip/hip_runtime.h>

#include <type_traits>

#include "common.h"
#include "decode.h"
#include "matvec_common.h"

namespace zhip {

namespace {

typedef _Float16 qf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 qf16x2 __attribute__((ext_vector_type(2)));
typedef float qf32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t qu32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t qu32x4 __attribute__((ext_vector_type(4)));

constexpr uint32_t THREADS = 512, WAVES = 8;
constexpr int SLOTS = 4;                        // ring slots: three units in flight behind the one multiplied
constexpr uint32_t PART_BYTES = 2u * WAVES * 256u * 4u;  // [tile parity][wave][token of the lane's four][lane]
constexpr uint32_t KEPT = 16;                   // tiles whose outputs wait in LDS for one burst of stores

// The formats. A unit is four 256-weight blocks of each of a tile's 32 rows: whole lines of every row.
struct FmtQ6 {  // 224-byte padded blocks: ql[128], qh[64], sixteen signed scales, d
    static constexpr uint32_t BLOCK = 224, ROW_LINES = 7;  // a row's part of a unit: seven lines
    static constexpr int LOADS = 4;                        // wave-wide loads of a unit a wave issues
    static constexpr uint32_t LOADERS = 7;                 // 28 KB: seven waves' worth; the eighth asks for nothing
    static constexpr float OFFSET = -1056.0f;              // 1024 + byte -> q - 32
    static const char *name() { return "matvec_q6_k"; }
};
struct FmtQ3 {  // blocks repacked at load into eight self-contained 16-byte units (src/kernels/repack_q3_k.wgsl)
    static constexpr uint32_t BLOCK = 128, ROW_LINES = 4;
    static constexpr int LOADS = 2;
    static constexpr uint32_t LOADERS = 8;
    static constexpr float OFFSET = -1028.0f;              // 1024 + byte -> q - 4
    static const char *name() { return "matvec_q3_k"; }
};
template <class F> constexpr uint32_t row_unit() { return 4u * F::BLOCK; }        // a unit's bytes of one row
template <class F> constexpr uint32_t unit_bytes() { return 32u * row_unit<F>(); }  // a unit in LDS
// (the last KB: where the loads of nothing land)
template <class F> constexpr uint32_t lds_bytes() { return PART_BYTES + SLOTS * unit_bytes<F>() + KEPT * 1024u + 64u + 1024u; }
static_assert(lds_bytes<FmtQ6>() <= 160u * 1024u - 64u, "the ring must fit the CU's LDS");

struct Q6Args {
    MvArgs a;
    uint32_t w_bytes;    // bytes of the weights the loads may touch (they are range-checked)
    uint32_t rounds;     // 32-row tiles every workgroup takes: tiles b, b + G, ...
    uint32_t tail_base;  // units of eight rows after those: tail_base for every workgroup
    uint32_t tail_rem;   // and one more for each of the first tail_rem
    uint32_t by_die;     // workgroups renumbered die by die (the grid is a multiple of eight)
    uint32_t bias;       // 0x64646464: the bytes of two f16 1024.0 exponents, as a kernel argument
                         // so that the byte shuffles stay one instruction each
    const uint8_t *planes;  // [2][tokens][k] f16: the tokens' roundings and remainders
    const float *inverse;   // [tokens]: one over each token's scale
};

__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// A 4-byte store the compiler's wait-count bookkeeping does not see as a store (with one pending
// it would make every wait for a load a wait for everything in flight).
__device__ __forceinline__ void store_apart(float *at, float v) {
    asm volatile("global_store_dword %0, %1, off\n\ts_nop 0" ::"v"(at), "v"(v) : "memory");
}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_buffer(const void *base, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, 0x00020000);
}
typedef __attribute__((address_space(3))) void *lds_ptr;
// One wave-wide load of 16 bytes a lane straight into LDS (lane l lands at dst + 16 l). The
// destination reaches the load as a bare LDS address, so the compiler keeps no dependency
// between these loads and later LDS reads; the explicit waits and barriers order them.
__device__ __forceinline__ void load_lds_b128(__amdgpu_buffer_rsrc_t buf, uint32_t dst, uint32_t voffset) {
    asm volatile("" : "+s"(dst));
    __builtin_amdgcn_raw_ptr_buffer_load_lds(buf, (lds_ptr)(uintptr_t)dst, 16, voffset, 0, 0, 0);
}

// Eight quants, a byte each in two words, as the exact f16 values q - 32 (Q6_K) or q - 4 (Q3_K) in position order.
template <class F>
__device__ __forceinline__ qf16x8 weights_f16(qu32x2 q, uint32_t bias) {
    const qf16x2 off = {(_Float16)F::OFFSET, (_Float16)F::OFFSET};
    qu32x4 r;
#pragma unroll
    for (int i = 0; i < 2; i++) {
        // bytes (low to high) q0 0x64 q1 0x64: the f16 pair (1024 + q0, 1024 + q1); then q2, q3
        const uint32_t lo = __builtin_amdgcn_perm(bias, q[i], 0x04010400u), hi = __builtin_amdgcn_perm(bias, q[i], 0x04030402u);
        r[2 * i] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(qf16x2, lo) + off);
        r[2 * i + 1] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(qf16x2, hi) + off);
    }
    return __builtin_bit_cast(qf16x8, r);
}

// Token blockIdx.x as the multiply sees it (src/kernels/matvec_quant.wgsl.hbs:73-89: RMSNorm
// times the norm weights and / or silu(x / act_div)), scaled by the power of two that puts its
// largest magnitude in [2^14, 2^15) and split into the f16 rounding and what that left times
// 2^11: planes [2][tokens][k], and one over the scale.
__global__ __launch_bounds__(256) void matvec_q6k_split_kernel(MvArgs a, uint2 *planes, float *inverse) {
    __shared__ float red[4];
    __shared__ float4 staged[1024];
    stage_token(a, blockIdx.x, staged, red);
    __syncthreads();
    const uint32_t tid = threadIdx.x, k4 = a.k / 4u;
    float big = 0.f;
    for (uint32_t i = tid; i < k4; i += 256u) {
        const float4 v = staged[i];
        big = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fmaxf(fabsf(v.z), fabsf(v.w)), big));
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) big = fmaxf(big, __shfl_xor(big, off, 64));
    if ((tid & 63u) == 0) red[tid >> 6] = big;
    __syncthreads();
    big = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    const int e = (int)((__float_as_uint(big) >> 23) & 0xffu);  // biased exponent; 0 for zero and subnormals
    int se = 127 + 14 - (e - 127);                               // scale = 2^(14 - (e - 127)), kept normal both ways
    se = se < 1 ? 1 : se > 253 ? 253 : se;
    const bool unit = e == 0 || e == 255;
    const float scale = unit ? 1.0f : __uint_as_float((uint32_t)se << 23);
    if (tid == 0) inverse[blockIdx.x] = unit ? 1.0f : __uint_as_float((uint32_t)(254 - se) << 23);
    for (uint32_t i = tid; i < k4; i += 256u) {
        const float4 v = staged[i];
        const float x[4] = {v.x, v.y, v.z, v.w};
        _Float16 hi[4], lo[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            // The scale is a power of two, so x * scale - hi in one fused operation is exact.
            hi[j] = (_Float16)(x[j] * scale);
            lo[j] = (_Float16)(fmaf(x[j], scale, -(float)hi[j]) * 2048.0f);
        }
        typedef _Float16 h4 __attribute__((ext_vector_type(4)));
        planes[(size_t)blockIdx.x * k4 + i] = __builtin_bit_cast(uint2, h4{hi[0], hi[1], hi[2], hi[3]});
        planes[(size_t)(gridDim.x + blockIdx.x) * k4 + i] = __builtin_bit_cast(uint2, h4{lo[0], lo[1], lo[2], lo[3]});
    }
}

// NU: units of a tile (k = 1024 NU).
template <class F, int NU>
__global__ __launch_bounds__(THREADS) void matvec_kquant_mfma_stream_kernel(Q6Args q) {
    constexpr uint32_t ROW_UNIT = row_unit<F>(), UNIT = unit_bytes<F>();
    constexpr int LOADS = F::LOADS;
    const MvArgs &a = q.a;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    float *lds_part = reinterpret_cast<float *>(lds);
    uint8_t *ring = lds + PART_BYTES;
    float *lds_kept = reinterpret_cast<float *>(lds + PART_BYTES + SLOTS * UNIT);  // [tile % KEPT][token][row]
    float *lds_inverse = lds_kept + KEPT * 256u;                                 // [token]
    const uint32_t ring0 = (uint32_t)(uintptr_t)ring;
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const __amdgpu_buffer_rsrc_t wbuf = make_buffer(a.w, q.w_bytes), nobuf = make_buffer(a.w, 0);
    uint32_t bias = q.bias;
    asm volatile("" : "+v"(bias));

    // The workgroup's tiles: b, b + G, ... and its share of the rows after the whole rounds.
    const uint32_t G = gridDim.x;
    const uint32_t b = q.by_die ? (blockIdx.x & 7u) * (G >> 3) + (blockIdx.x >> 3) : blockIdx.x;
    const uint32_t tail_units = q.tail_base + (b < q.tail_rem ? 1u : 0u);
    const uint32_t tail_row = 32u * q.rounds * G + 8u * (b * q.tail_base + (b < q.tail_rem ? b : q.tail_rem));
    // With SILU_PAIR (src/kernels/matvec_quant.wgsl.hbs:110-125) an output tile is two weight
    // tiles, the gate rows and then the up rows `half` further down: tile p of the run is weight
    // tile p % per of output tile p / per.
    const uint32_t per = (a.flags & FLAG_SILU_PAIR) ? 2u : 1u;
    const uint32_t count = per * (q.rounds + (tail_units ? 1u : 0u));
    auto out_row = [&](uint32_t po) { return po < q.rounds ? 32u * (b + po * G) : tail_row; };  // first output of output tile po
    auto out_rows = [&](uint32_t po) { return po < q.rounds ? 32u : 8u * tail_units; };
    auto first_row = [&](uint32_t p) { return out_row(p / per) + ((p % per) ? a.half : 0u); };
    auto rows_of = [&](uint32_t p) { return out_rows(p / per); };

    // A unit's loads. The unit is 224 lines, row after row; load g = 4 wave + j brings lines
    // 8 g .. 8 g + 7 (the eighth wave's four would be past the unit's end: they go against an
    // empty buffer, so that every wave's waits count the same loads), lane l line 8 g + l / 8
    // and the chunk that belongs at position l % 8 of it. The whole address is the lane's
    // offset, which is what the buffer's range check sees: rows past the matrix's end land as zeros.
    uint32_t woff[LOADS];
#pragma unroll
    for (int j = 0; j < LOADS; j++) {
        const uint32_t line = 8u * (LOADS * wave + j) + (lane >> 3), row = line / F::ROW_LINES, in_row = line % F::ROW_LINES;
        woff[j] = row * a.row_bytes + 128u * in_row + 16u * ((lane & 7u) ^ (row & 7u));
    }
    // Unit v of the run: unit v % NU of tile v / NU. Past the run's end the loads still run, so
    // that the waits count the same loads every step, but against an empty buffer: zeros land
    // and nothing is fetched.
    auto issue = [&](uint32_t v, uint32_t slot) __attribute__((always_inline)) {
        const uint32_t p = v / NU, u = v % NU;
        const bool real = p < count && wave < F::LOADERS;
        const uint32_t base = (real ? first_row(p) : 0u) * a.row_bytes + ROW_UNIT * u, rows = rows_of(p);
        // (a load against the empty buffer still lands zeros: the eighth wave's in a spare KB)
        const uint32_t dst = wave < F::LOADERS ? ring0 + slot * UNIT + 1024u * (LOADS * wave) : ring0 + SLOTS * UNIT + KEPT * 1024u + 64u;
#pragma unroll
        for (int j = 0; j < LOADS; j++) {
            // (lines of rows the workgroup's share of the last rows does not have are not fetched;
            // what the matrix instructions make of the zeros there is never stored)
            const uint32_t first_line_row = (8u * (LOADS * wave + j)) / F::ROW_LINES;
            load_lds_b128(real && first_line_row < rows ? wbuf : nobuf, wave < F::LOADERS ? dst + 1024u * j : dst, woff[j] + base);
        }
    };

    // The tokens' operands, ready-made in the planes. Operand row r of the matrix instruction is
    // piece r / 8 of token 4 (r / 4 % 2) + r % 4 (rows 16 .. 31 are zeros), so that a lane's
    // results are its weight row times both pieces of four tokens; the lane's eight positions of
    // sub-block s of its wave's block are 16 s + 8 (lane / 32) ... The lanes of absent tokens and
    // of the zero rows ask past the buffer's end and get zeros.
    const uint32_t rho = lane & 31u, kap = lane >> 5;
    const uint32_t tok = 4u * ((rho >> 2) & 1u) + (rho & 3u), piece = rho >> 3;
    const bool live = tok < a.m && piece < 2u;
    // Wave w multiplies half w % 2 (sub-blocks 8 (w % 2) .. + 7, 128 positions) of block w / 2 of
    // every unit.
    const uint32_t blk = wave >> 1, half = wave & 1u;
    qf16x8 xf[8 * NU];
    {
        const __amdgpu_buffer_rsrc_t pbuf = make_buffer(q.planes, 2u * a.m * a.k * 2u);
        const uint32_t at = live ? ((piece * a.m + tok) * a.k + 256u * blk + 128u * half + 8u * kap) * 2u : 0xfffffff0u;
#pragma unroll
        for (int u = 0; u < NU; u++)
#pragma unroll
            for (int s = 0; s < 8; s++)
                xf[8 * u + s] = __builtin_bit_cast(qf16x8, __builtin_amdgcn_raw_buffer_load_b128(pbuf, live ? at + 2u * (1024u * u + 16u * s) : at, 0, 0));
    }
    if (tid < 8u) lds_inverse[tid] = tid < a.m ? q.inverse[tid] : 1.0f;  // read behind later barriers
#pragma unroll
    for (int v = 0; v < SLOTS - 1; v++) issue(v, v);

    // The lane's reads of its wave's half block of a unit: row rho of the flat copy, the block's
    // bytes at 224 (wave / 2). Byte o of a row's unit sits at 896 rho + 128 (o / 128) +
    // 16 ((o / 16 % 8) ^ (rho % 8)) + o % 16.
    auto at_byte = [&](uint32_t o) { return ROW_UNIT * rho + (o & ~127u) + 16u * (((o >> 4) & 7u) ^ (rho & 7u)) + (o & 15u); };
    constexpr bool Q3 = F::BLOCK == 128u;
    uint32_t at_ql[4], at_qh[2];  // Q6_K ql: [which 32 of the half's 64][which 16]; qh: [which 16]; Q3_K: at_ql = the half's four units
    uint32_t at_sc = 0, at_d = 0;
    if constexpr (Q3) {
#pragma unroll
        for (uint32_t i = 0; i < 4; i++) at_ql[i] = at_byte(128u * blk + 64u * half + 16u * i);
        at_qh[0] = at_qh[1] = 0;
    } else {
#pragma unroll
        for (uint32_t i = 0; i < 4; i++) at_ql[i] = at_byte(224u * blk + 64u * half + 32u * (i >> 1) + 16u * (i & 1u) + 8u * kap);
#pragma unroll
        for (uint32_t i = 0; i < 2; i++) at_qh[i] = at_byte(224u * blk + 128u + 32u * half + 16u * i + 8u * kap);
        at_sc = at_byte(224u * blk + 192u + 8u * half);
        at_d = at_byte(224u * blk + 208u);
    }

    float acc[4] = {0.f, 0.f, 0.f, 0.f};  // tokens 4 (lane / 32) + i, matrix row rho of the tile, this wave's blocks
    // One sub-block: its eight quants of the lane (a byte each), d * scale, and the operand index.
    auto sub_block = [&](qu32x2 v, float dsc, int s) __attribute__((always_inline)) {
        qf32x16 zero;
#pragma unroll
        for (int e = 0; e < 16; e++) zero[e] = 0.f;
        const qf32x16 r = __builtin_amdgcn_mfma_f32_32x32x16_f16(xf[s], weights_f16<F>(v, bias), zero, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < 4; i++) acc[i] = fmaf(dsc, fmaf(r[4 + i], 1.0f / 2048.0f, r[i]), acc[i]);
        // (a sub-block's results are used up before the next sub-block's matrix
        // instruction: eight of them in flight would not fit the registers)
        asm volatile("" : "+v"(acc[0]), "+v"(acc[1]), "+v"(acc[2]), "+v"(acc[3]));
    };
    auto multiply = [&](auto unit, uint32_t slot) __attribute__((always_inline)) {
        constexpr int U = decltype(unit)::value;
        const uint8_t *t = ring + slot * UNIT;
        if constexpr (Q3) {
            // Unit i of the half: 32 weights as two words of 2-bit values (byte b, bit pair e:
            // position 4 e + b; the second word 16 further), a word of third bits (byte b, bit e:
            // position 4 e + b), scale - 32 of each sixteen as signed bytes, d. The lane's eight
            // positions of a sixteen are 8 kap ..: bit pairs 2 kap and 2 kap + 1 of the four bytes.
#pragma unroll
            for (uint32_t i = 0; i < 4; i++) {
                const qu32x4 u = *reinterpret_cast<const qu32x4 *>(t + at_ql[i]);
                const float d = half_bits_to_float(u.w >> 16);
#pragma unroll
                for (uint32_t h16 = 0; h16 < 2; h16++) {
                    const uint32_t word = h16 ? u.y : u.x, third = u.z >> (4u * h16 + 2u * kap);
                    qu32x2 v;
                    v[0] = ((word >> (4u * kap)) & 0x03030303u) | ((third & 0x01010101u) << 2);
                    v[1] = ((word >> (4u * kap + 2u)) & 0x03030303u) | (((third >> 1) & 0x01010101u) << 2);
                    const float dsc = d * (float)(int8_t)((u.w >> (8u * h16)) & 0xffu);
                    sub_block(v, dsc, 8 * U + 2 * (int)i + (int)h16);
                }
            }
        } else {
            const qu32x2 sc = *reinterpret_cast<const qu32x2 *>(t + at_sc);
            const float d = half_bits_to_float(*reinterpret_cast<const uint16_t *>(t + at_d));
#pragma unroll
            for (uint32_t h16 = 0; h16 < 2; h16++) {
                const qu32x2 qh = *reinterpret_cast<const qu32x2 *>(t + at_qh[h16]);
#pragma unroll
                for (uint32_t qp = 0; qp < 2; qp++) {
                    const qu32x2 ql = *reinterpret_cast<const qu32x2 *>(t + at_ql[2u * qp + h16]);
#pragma unroll
                    for (uint32_t up = 0; up < 2; up++) {
                        // Quadrant qd of the half: weights 32 qd + 16 h16 + 8 kap ... of its 128, sub-block 2 qd + h16 of its eight.
                        const uint32_t qd = qp + 2u * up, s = 2u * qd + h16;
                        qu32x2 v;
#pragma unroll
                        for (int w = 0; w < 2; w++) {
                            const uint32_t nib = up ? (ql[w] >> 4) & 0x0f0f0f0fu : ql[w] & 0x0f0f0f0fu;
                            const uint32_t two = (qd ? qh[w] >> (2u * qd) : qh[w]) & 0x03030303u;
                            v[w] = nib | (two << 4);
                        }
                        const uint32_t word = s < 4u ? sc.x : sc.y;
                        const float dsc = d * (float)(int8_t)((word >> (8u * (s & 3u))) & 0xffu);
                        sub_block(v, dsc, 8 * U + (int)s);
                    }
                }
            }
        }
    };
    // A finished tile's partial sums into LDS; they are added behind the next barrier.
    auto hand_over = [&](uint32_t p) __attribute__((always_inline)) {
        float *part = lds_part + (p & 1u) * (WAVES * 256u);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            part[wave * 256u + 64u * i + lane] = acc[i];
            acc[i] = 0.f;
        }
    };
    // (a wave sums tokens i and 4 + i, whose partial sums lie side by side: no two lanes on a bank)
    float held = 0.f;  // the gate tile's result, until the up tile's arrives
    auto sum_up = [&](uint32_t p) __attribute__((always_inline)) {
        const uint32_t po = p / per;
        if ((tid >> 8) != (po & 1u)) return;  // (the same half of the workgroup for an output tile's two weight tiles)
        const float *part = lds_part + (p & 1u) * (WAVES * 256u);
        const uint32_t row = tid & 31u, tk = 4u * ((tid >> 5) & 1u) + ((tid >> 6) & 3u);
        const float *src = part + 64u * (tk & 3u) + 32u * (tk >> 2) + row;
        float total = src[0];
#pragma unroll
        for (uint32_t wv = 1; wv < WAVES; wv++) total += src[wv * 256u];
        total *= lds_inverse[tk];
        if (per == 2u && !(p & 1u)) held = total;
        else lds_kept[256u * (po % KEPT) + 32u * tk + row] = per == 2u ? silu_f(held) * total : total;
    };
    // The outputs of output tiles first .. first + n - 1, from LDS to memory in one burst: 128
    // contiguous bytes a token and tile.
    auto store_kept = [&](uint32_t first, uint32_t n) __attribute__((always_inline)) {
        lds_barrier();
        for (uint32_t po = first + (tid >> 8); po < first + n; po += 2u) {
            const uint32_t row = tid & 31u, tk = (tid >> 5) & 7u;
            const uint32_t j = out_row(po) + row;
            if (tk < a.m && row < out_rows(po) && j < a.rows) {
                float *o = a.out + (size_t)tk * a.out_stride + a.col0 + j;
                const float total = lds_kept[256u * (po % KEPT) + (tid & 255u)];
                store_apart(o, (a.flags & FLAG_ACCUMULATE) ? *o + total : total);
            }
        }
    };

    // One barrier a unit: behind it all of unit v has landed (every wave has waited for its own
    // loads of it; those of the two units after it stay in flight), nobody still reads the slot
    // that is refilled next, and the tile before's partial sums are in LDS.
    auto step = [&](uint32_t p, auto unit) __attribute__((always_inline)) {
        constexpr int U = decltype(unit)::value;
        const uint32_t v = NU * p + U;
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"((SLOTS - 2) * LOADS) : "memory");
        lds_barrier();
        issue(v + (SLOTS - 1), (v + (SLOTS - 1)) % SLOTS);
        if (U == 0 && p > 0u) {
            sum_up(p - 1u);
            // (the next tile's sums are kept only behind a later barrier, which no thread passes
            // before it has stored what it stores here)
            if (p % (per * KEPT) == 0u) store_kept(p / per - KEPT, KEPT);
        }
        multiply(unit, v % SLOTS);
    };
    for (uint32_t p = 0; p < count; p++) {
        step(p, std::integral_constant<int, 0>{});
        if constexpr (NU >= 2) step(p, std::integral_constant<int, 1>{});
        if constexpr (NU >= 4) {
            step(p, std::integral_constant<int, 2>{});
            step(p, std::integral_constant<int, 3>{});
        }
        hand_over(p);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // nothing may still land in LDS once the workgroup is gone
    if (count > 0u) {
        lds_barrier();
        sum_up(count - 1u);
        const uint32_t last = count / per - 1u;  // the run's last output tile
        store_kept(last - last % KEPT, last % KEPT + 1u);
    }
}

template <class F, int NU>
zhip_result launch_blocks(const Dispatch &d, const Q6Args &q, dim3 grid) {
    auto kernel = matvec_kquant_mfma_stream_kernel<F, NU>;
    constexpr uint32_t bytes = lds_bytes<F>();
    static bool configured = false;
    if (!configured) {
        if (hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess) {
            (void)hipGetLastError();
            return fail(d, ZHIP_E_GPU, "%s: cannot reserve %u bytes of LDS", F::name(), bytes);
        }
        configured = true;
    }
    hipLaunchKernelGGL(kernel, grid, dim3(THREADS), bytes, d.stream, q);
    return check_launch(d, F::name());
}

template <class F>
zhip_result launch_stream(const Dispatch &d, const MvArgs &a, uint64_t w_bytes) {
    // 32-bit byte offsets, a tile past the last row.
    const uint64_t used = ((uint64_t)((a.flags & FLAG_SILU_PAIR) ? a.half : 0u) + a.rows) * a.row_bytes;
    if (used + 64ull * a.row_bytes >= 0xfffffff0ull) return fail(d, ZHIP_E_BAD_COMMAND, "%s: weights of 4 GiB or more", F::name());
    if (!d.work) return fail(d, ZHIP_E_GPU, "%s: no workspace", F::name());
    const uint64_t plane_bytes = 4ull * a.m * a.k;
    if (zhip_result r = d.work->reserve(d, plane_bytes + 64u)) return r;
    float *inverse = reinterpret_cast<float *>(d.work->data + plane_bytes);
    hipLaunchKernelGGL(matvec_q6k_split_kernel, dim3(a.m), dim3(256), 0, d.stream, a, reinterpret_cast<uint2 *>(d.work->data), inverse);
    if (zhip_result r = check_launch(d, F::name())) return r;

    const uint32_t cus = (uint32_t)d.dev->compute_units;
    const uint32_t units = (a.rows + 7u) / 8u;
    const uint32_t groups = units < cus ? units : cus;
    const uint32_t rounds = (a.rows / 32u) / groups;
    const uint32_t tail = (a.rows - 32u * rounds * groups + 7u) / 8u;
    Q6Args q{a, (uint32_t)(used < w_bytes ? used : w_bytes), rounds, tail / groups, tail % groups, groups % 8u == 0 ? 1u : 0u, 0x64646464u, d.work->data, inverse};
    q.a.flags &= ~FLAG_NORM;
    q.a.norm_w = nullptr;
    q.a.act_div = 0.f;
    const dim3 grid(groups);
    return a.k == 1024u ? launch_blocks<F, 1>(d, q, grid) : a.k == 2048u ? launch_blocks<F, 2>(d, q, grid) : launch_blocks<F, 4>(d, q, grid);
}

bool stream_accepts(const MvArgs &a, uint32_t block_bytes) {
    return a.m >= 1 && a.m <= 8 && (a.k == 1024u || a.k == 2048u || a.k == 4096u) && a.rows >= 1 && a.xr % 4u == 0 &&
           (reinterpret_cast<uintptr_t>(a.x) & 15u) == 0 && (reinterpret_cast<uintptr_t>(a.w) & 15u) == 0 && a.row_bytes == a.k / 256u * block_bytes;
}

}  // namespace

// Whether these kernels can run the (already validated) arguments: k of whole units.
bool matvec_q6k_mfma_stream_accepts(const MvArgs &a) { return stream_accepts(a, FmtQ6::BLOCK); }
zhip_result launch_matvec_q6k_mfma_stream(const Dispatch &d, const MvArgs &a, uint64_t w_bytes) { return launch_stream<FmtQ6>(d, a, w_bytes); }
bool matvec_q3k_mfma_stream_accepts(const MvArgs &a) { return stream_accepts(a, FmtQ3::BLOCK); }
zhip_result launch_matvec_q3k_mfma_stream(const Dispatch &d, const MvArgs &a, uint64_t w_bytes) { return launch_stream<FmtQ3>(d, a, w_bytes); }

}  // namespace zhip
