// matvec_q4_k and matvec_q5_k, matrix-core variant (MatvecVariant wg 512, lanes 64, rows 16) for
// k = 2048 or 4096 (longer rows in parts, below) and steps of up to eight tokens. The per-weight work is done once for all
// tokens: the weights enter v_mfma_f32_16x16x32_f16 as the exact f16 values 16 + q (the nibble
// dropped into the mantissa of 16.0; Q5_K: 32 + q with the fifth bit), every token as two f16
// rows, the rounding of its inputs and what that left times 2^11, under a per-token power of
// two, so that every product is exact in the f32 accumulator and a token's rows meet no other
// token's; a block's sum is d sc S - (16 d sc + dmin m) X with X from the same rows times a
// column of ones (src/ref/tensor.zig:94-117). Nothing is recomputed and nothing but partial
// results crosses LDS.
//
// A 512-thread workgroup is eight waves that split k eight ways (one or two
// 256-weight blocks a wave). A wave builds its k range of all tokens' f16 rows
// once, straight into matrix-core operands that stay in registers for the
// whole kernel (64 VGPRs at k = 4096), together with the rows' sub-block sums
// (32 VGPRs). It then walks over sixteen-row weight tiles, persistent
// workgroups taking tiles b, b + G, ...: a tile's sixteen rows are one contiguous
// stretch of the matrix and travel as a flat copy through a ring of three LDS
// slots that the workgroup shares, every wave loading a share of it by wave-wide
// direct loads of whole lines, two tiles ahead (a wave fetching only its own
// blocks, 144-byte pieces that lie across line boundaries, made every line a
// request of two or three waves: 20.7 against 19.7 us on the 2 x 14336 x 4096
// pair at four tokens; a lane loading its own row's bytes straight into
// registers costs fifty cache accesses a load). Each wave waits for its own
// loads and one barrier a tile tells everyone that all of the tile has landed;
// behind the same barrier the tile before's partial sums (512 bytes a wave) are
// in LDS, where 128 threads add the eight for one output each (row i % 16,
// token i / 16) in the order of the k ranges, apply the SILU_PAIR / ACCUMULATE
// epilogue and store. Each lane reads its row's header and nibbles back from
// the copy (chunks XOR-permuted by row against bank conflicts) and multiplies.
//
// Rows of 6144 .. 32768 weights (a multiple of 2048; the FFN-down shapes) do not fit a
// workgroup's registers: `parts` = k / 2048 workgroups share a walker's tiles, workgroup b taking
// columns 2048 (b % parts) .. of the tiles of walker b / parts (one block a wave, the tile's
// sixteen pieces of nine or eleven lines a whole row apart), each under its own per-token
// scales, and store their sums per part; a second launch adds a tile's parts in the order of
// their columns and applies the epilogue. With the RMSNorm prologue, whose sum of squares is no
// single workgroup's, a small launch in front leaves every token's scale in memory
// (launch_matvec_parts_scales). Measured on Q4_K 4096 x 14336 at one to eight tokens: 14.3 -
// 14.8 us (12.1 + the sums' launch) against 10.3 / 14.3 / 19.2 / 21.6 / 40.9 us at one / two /
// three / four / eight tokens on the default variant; 8192 x 28672 34.3 - 36.4 us against
// 46.4 / 69.7 / 133.8 us at one / four / eight; 28672 x 8192 with the RMSNorm prologue 37.7 -
// 38.6 us against 26.7 / 83.7 / 169.0.
//
// Contract as the other variants (src/kernels/matvec_quant.wgsl.hbs); a token's
// result does not depend on how many tokens share the launch.
#include <hip/hip_runtime.h>

#include "common.h"
#include "decode.h"
#include "matvec_common.h"

namespace zhip {

typedef _Float16 rf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 rf16x4 __attribute__((ext_vector_type(4)));
typedef float rf32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t ru32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t ru32x2 __attribute__((ext_vector_type(2)));

namespace {

constexpr uint32_t THREADS = 512, WAVES = 8;
constexpr int kLongDepth = 3;
constexpr int kDepth = 3;  // ring slots: one tile multiplied, the others in flight (two slots: +0.3 us on the 2 x 14336 x 4096 pair, four: +0.8 us)
// The formats: a 256-weight block is a 16-byte header (d, dmin, twelve bytes of 6-bit scales and
// minimums) and 128 bytes of nibbles; Q5_K keeps a fifth bit of every weight in 32 bytes between
// the two (src/ref/tensor.zig:100-117). A weight enters the matrix cores as the exact f16 value
// BIAS + q: the quant dropped into the mantissa of BIAS (16.0 for four bits, 32.0 for five).
struct ResQ4 {
    static constexpr uint32_t BLOCK = 144, NIBBLES_AT = 16, SHIFT = 6;
    static constexpr bool FIFTH = false;
    static constexpr float BIAS = 16.0f;
    static const char *name() { return "matvec_q4_k"; }
};
struct ResQ5 {
    static constexpr uint32_t BLOCK = 176, NIBBLES_AT = 48, SHIFT = 5;
    static constexpr bool FIFTH = true;
    static constexpr float BIAS = 32.0f;
    static const char *name() { return "matvec_q5_k"; }
};
// A tile in LDS: the flat copy of its sixteen rows (NB = 256-weight blocks of a wave's k range:
// a row is 8 NB blocks, nine or eleven lines a block column of the eight waves).
template <class F, int NB> constexpr uint32_t tile_bytes() { return 16u * 8u * F::BLOCK * NB; }
// Wave-wide loads of 1 KB a tile takes, and how many a wave issues (the slots past the tile's end ask for nothing).
template <class F, int NB> constexpr uint32_t tile_kb() { return tile_bytes<F, NB>() / 1024u; }
template <class F, int NB> constexpr int tile_loads() { return (int)((tile_kb<F, NB>() + 7u) / 8u); }

struct ResArgs {
    MvArgs a;
    uint32_t w_bytes;
    uint32_t nibble_mask, sixteen;  // Q4_K: 0x03C003C0, 0x4C004C00; Q5_K: 0x01E001E0, 0x50005000 (see nibbles)
    uint32_t rounds;                // sixteen-output tiles every workgroup takes: tiles b, b + G, ...
    uint32_t left;                  // output tiles after those, fewer than G: one for each of the first workgroups,
    uint32_t split;                 // or (split) eight outputs of one for each of the first 2 * left
    // Rows of more than 4096 weights: `parts` workgroups share a tile, each over 2048 of its
    // columns, and leave their sums in `partial` ([part][gate, up][token of 8][output]).
    uint32_t parts;
    float *partial;
    const float *scales;  // with the RMSNorm prologue: each token's 1 / sqrt(mean(x^2) + eps)
};

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_buffer(const void *base, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, 0x00020000);
}

// A barrier that waits for this wave's LDS traffic only: the weight loads of the
// tile ahead stay in flight.
__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

typedef __attribute__((address_space(3))) void *lds_ptr;

// One wave-wide load of 16 bytes a lane straight into LDS (lane l lands at dst + 16 l). The
// destination reaches the load as a bare LDS address, so the compiler keeps no dependency
// between these loads and later LDS reads; the explicit waits order them.
__device__ __forceinline__ void load_lds_b128(__amdgpu_buffer_rsrc_t buf, uint32_t dst, uint32_t voffset) {
    asm volatile("" : "+s"(dst));
    __builtin_amdgcn_raw_ptr_buffer_load_lds(buf, (lds_ptr)(uintptr_t)dst, 16, voffset, 0, 0, 0);
}

template <int LEFT>
__device__ __forceinline__ void wait_loads() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(LEFT) : "memory");
}

// A 4-byte store the compiler's wait-count bookkeeping does not see as a store: with one
// pending it would turn every wait for a weight load into a wait for all loads in flight
// (loads and stores complete out of order with each other). A wait that counts only the
// loads issued after the awaited one stays sufficient while a store is outstanding.
__device__ __forceinline__ void store_apart(float *at, float v) {
    asm volatile("global_store_dword %0, %1, off\n\ts_nop 0" ::"v"(at), "v"(v) : "memory");
}

// Eight nibbles of two words as f16 values BIAS + q in the order k0 k2 k1 k3 k4 k6 k5 k7 (the
// inputs' operands are built in the same order). `mask` arrives in a scalar register and
// `sixteen` (the bits of BIAS, twice) in a vector one: a shift and one v_and_or_b32 a pair.
// Q5_K: `fifth` holds the weights' fifth bits in bit 0 of its bytes.
template <class F, bool HIGH>
__device__ __forceinline__ rf16x8 nibbles(ru32x2 w, ru32x2 fifth, uint32_t mask, uint32_t sixteen) {
    constexpr uint32_t S = F::SHIFT;  // the quant's lowest bit in the f16 mantissa
    ru32x4 r;
    if (HIGH) {
        r.x = ((w.x << (S - 4u)) & mask) | sixteen;
        r.y = ((w.x >> (12u - S)) & mask) | sixteen;
        r.z = ((w.y << (S - 4u)) & mask) | sixteen;
        r.w = ((w.y >> (12u - S)) & mask) | sixteen;
    } else {
        r.x = ((w.x << S) & mask) | sixteen;
        r.y = ((w.x >> (8u - S)) & mask) | sixteen;
        r.z = ((w.y << S) & mask) | sixteen;
        r.w = ((w.y >> (8u - S)) & mask) | sixteen;
    }
    if (F::FIFTH) {
        // bit 0 of bytes 0 and 2 to bits 9 and 25 (k0, k2), of bytes 1 and 3 likewise (k1, k3)
        r.x |= (fifth.x << 9) & 0x02000200u;
        r.y |= (fifth.x << 1) & 0x02000200u;
        r.z |= (fifth.y << 9) & 0x02000200u;
        r.w |= (fifth.y << 1) & 0x02000200u;
    }
    return __builtin_bit_cast(rf16x8, r);
}

// NB: 256-weight blocks of a wave's k range (k = 2048 NB). LONG (NB = 1): k = 2048 q.parts;
// workgroup b multiplies columns 2048 (b % parts) .. (part `kpart`) of the tiles that walker b / parts takes, and
// matvec_kquant_mfma_parts_sum_kernel adds the parts in their order and applies the epilogue.
template <class F, bool PAIR, int NB, bool LONG>
__global__ __launch_bounds__(THREADS) void matvec_kquant_mfma_resident_kernel(ResArgs q) {
    static_assert(!LONG || NB == 1, "parts of a long row are 2048 columns");
    constexpr int DEPTH = LONG ? kLongDepth : kDepth;
    const MvArgs &a = q.a;
    __shared__ float lds_scale[16];               // [8 ..]: one over each token's scale
    __shared__ float lds_max[WAVES * 8];          // [wave][token]: the largest magnitude in the wave's range
    __shared__ float lds_ss[WAVES * 8];           // [wave][token]: the range's sum of squares (RMSNorm prologue)
    __shared__ float lds_part[2][WAVES][128];     // [tile parity][wave][2 lane + token of the lane's two]
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, l16 = lane & 15u, g = lane >> 4;
    const __amdgpu_buffer_rsrc_t wbuf = make_buffer(a.w, q.w_bytes), nobuf = make_buffer(a.w, 0);
    uint32_t sixteen = q.sixteen;
    asm volatile("" : "+v"(sixteen));

    // The workgroup's weight tiles: output tiles b, b + G, ...; with SILU_PAIR the gate tile
    // and then the up tile of each. Tile p of the run starts at matrix row:
    const uint32_t per = PAIR ? 2u : 1u;
    const uint32_t kpart = LONG ? blockIdx.x % q.parts : 0u, walker = LONG ? blockIdx.x / q.parts : blockIdx.x, walkers = LONG ? gridDim.x / q.parts : gridDim.x;
    // When the output tiles left over after whole rounds are at most half as many as the
    // workgroups, two workgroups share each, eight rows apiece: a whole tile more on half of
    // the CUs would be the launch's tail.
    const bool extra = walker < (q.split ? 2u * q.left : q.left);
    const uint32_t mine = q.rounds + (extra ? 1u : 0u);
    const uint32_t count = per * mine;
    const uint32_t last_out = 16u * (q.rounds * walkers + (q.split ? walker >> 1 : walker)) + (q.split ? 8u * (walker & 1u) : 0u);
    auto out0 = [&](uint32_t p) { return p / per < q.rounds ? 16u * (walker + (p / per) * walkers) : last_out; };  // first output of tile p
    auto rows_of = [&](uint32_t p) { return (q.split && p / per >= q.rounds) ? 8u : 16u; };
    auto row0 = [&](uint32_t p) { return out0(p) + ((PAIR && (p & 1u)) ? a.half : 0u); };

    // A tile's loads. The tile's sixteen rows are one contiguous stretch of the matrix, 18 NB
    // KB of whole lines, and travel as a flat copy into one of the ring's slots, which the whole
    // workgroup shares: load g = LOADS wave + j brings lines 8 g .. 8 g + 7 (the slots past the
    // tile's last line go against an empty buffer and land their zeros in a spare KB, so that
    // every wave's waits count the same loads), lane l line 8 g + l / 8 and the chunk that
    // belongs at position l % 8 of it: chunk c of a line of row r sits at position c ^ (r % 8).
    // The whole address is the lane's offset. Past the run's last tile the loads still run, but
    // against the empty buffer: zeros land and nothing is fetched.
    constexpr int LOADS = tile_loads<F, NB>();
    constexpr uint32_t TILE = tile_bytes<F, NB>(), ROW_LINES = 8u * F::BLOCK * NB / 128u, TILE_LOADS = tile_kb<F, NB>();
    __shared__ __align__(16) uint8_t lds_ring[DEPTH * TILE + 1024u];
    const uint32_t ring0 = (uint32_t)(uintptr_t)lds_ring;
    const uint32_t uwave = __builtin_amdgcn_readfirstlane(wave);
    uint32_t woff[LOADS];
#pragma unroll
    for (int j = 0; j < LOADS; j++) {
        const uint32_t line = 8u * (LOADS * wave + j) + (lane >> 3), row = line / ROW_LINES;
        // (a part of a long row: the tile's rows lie a whole row apart)
        woff[j] = (LONG ? row * a.row_bytes + 128u * (ROW_LINES * kpart + line % ROW_LINES) : 128u * line) + 16u * ((lane & 7u) ^ (row & 7u));
    }
    auto load_tile = [&](uint32_t p, uint32_t slot) __attribute__((always_inline)) {
        const bool real = p < count;
        const uint32_t base = (real ? row0(p) : 0u) * a.row_bytes, rows = rows_of(p);
#pragma unroll
        for (int j = 0; j < LOADS; j++) {
            const uint32_t g = LOADS * uwave + j;
            // (the lines of the rows an eight-row share does not have are not fetched)
            const bool wanted = real && g < TILE_LOADS && (8u * g) / ROW_LINES < rows;
            load_lds_b128(wanted ? wbuf : nobuf, g < TILE_LOADS ? ring0 + slot * TILE + 1024u * g : ring0 + DEPTH * TILE, woff[j] + base);
        }
    };

    // The tokens' inputs first: loads complete in order within a wave, and behind the weight
    // loads below the first use of an input would wait for a round trip of the weight stream.
    // Operand row l16 of the matrix instruction is token l16 / 2: the f16 rounding of its scaled
    // inputs (even rows) or what that left, times 2^11 (odd rows); the lane's eight positions of
    // sub-block s are 8 g .. 8 g + 7 in the order k0 k2 k1 k3 k4 k6 k5 k7. The two lanes of a
    // token and group share the work: the even one loads and splits positions 0 .. 3, the odd
    // one 4 .. 7, and they swap what the other needs. An absent token's rows read the last
    // token's inputs under a scale of zero: no branches, so all of the lane's loads go out together.
    const uint32_t tok = l16 >> 1, sub = l16 & 1u, tsrc = tok < a.m ? tok : a.m - 1u;
    float4 raw[NB * 8];
    {
        const float *xt = a.x + (size_t)tsrc * a.xr + 2048u * kpart + NB * 256u * wave + 8u * g + 4u * sub;
#pragma unroll
        for (int s = 0; s < NB * 8; s++) raw[s] = *reinterpret_cast<const float4 *>(xt + 32 * s);
    }
    // A step's prologue (src/kernels/matvec_quant.wgsl.hbs:73-89) on the same registers, in the
    // default variant's arithmetic: RMSNorm times the norm weights (the wave ranges' sums of
    // squares meet in LDS, added in the order of the ranges) and / or silu(x / act_div).
    // (the sum of squares of a long row is not any one workgroup's: it comes ready in q.scales)
    const bool norm = (a.flags & FLAG_NORM) != 0, act = a.act_div > 0.f;
    float4 gw[NB * 8];
    float ready = 0.f;  // (asked for before the first weights, like the inputs)
    if (norm) {
        const float *gt = a.norm_w + 2048u * kpart + NB * 256u * wave + 8u * g + 4u * sub;
#pragma unroll
        for (int s = 0; s < NB * 8; s++) gw[s] = *reinterpret_cast<const float4 *>(gt + 32 * s);
        if (LONG) ready = q.scales[tsrc];
    }
    load_tile(0, 0);
    if (norm) {
        float rs;
        if (LONG) {
            rs = ready;
        } else {
            float ss = 0.f;
#pragma unroll
            for (int s = 0; s < NB * 8; s++) ss += raw[s].x * raw[s].x + raw[s].y * raw[s].y + raw[s].z * raw[s].z + raw[s].w * raw[s].w;
            ss += __shfl_xor(ss, 1, 64);
            ss += __shfl_xor(ss, 16, 64);
            ss += __shfl_xor(ss, 32, 64);
            if (g == 0u && sub == 0u) lds_ss[8u * wave + tok] = ss;
            lds_barrier();
            float total = lds_ss[tok];
#pragma unroll
            for (uint32_t wv = 1; wv < WAVES; wv++) total += lds_ss[8u * wv + tok];
            rs = 1.0f / sqrtf(total / (float)a.k + a.eps);
        }
#pragma unroll
        for (int s = 0; s < NB * 8; s++) {
            raw[s].x = raw[s].x * rs * gw[s].x; raw[s].y = raw[s].y * rs * gw[s].y;
            raw[s].z = raw[s].z * rs * gw[s].z; raw[s].w = raw[s].w * rs * gw[s].w;
        }
    }
    if (act) {
#pragma unroll
        for (int s = 0; s < NB * 8; s++) {
            raw[s].x = silu_f(raw[s].x / a.act_div); raw[s].y = silu_f(raw[s].y / a.act_div);
            raw[s].z = silu_f(raw[s].z / a.act_div); raw[s].w = silu_f(raw[s].w / a.act_div);
        }
    }

    // Each token's scale: the power of two that puts its largest magnitude in [2^14, 2^15). The
    // eight lanes of a token (two rows, four groups) hold this wave's range of it; the eight
    // waves' maxima meet in LDS.
    {
        float big = 0.f;
#pragma unroll
        for (int s = 0; s < NB * 8; s++) big = fmaxf(fmaxf(fabsf(raw[s].x), fabsf(raw[s].y)), fmaxf(fmaxf(fabsf(raw[s].z), fabsf(raw[s].w)), big));
        big = fmaxf(big, __shfl_xor(big, 1, 64));
        big = fmaxf(big, __shfl_xor(big, 16, 64));
        big = fmaxf(big, __shfl_xor(big, 32, 64));
        if (g == 0u && sub == 0u) lds_max[8u * wave + tok] = big;
    }
    lds_barrier();
    auto scale_of = [&](uint32_t t, bool inverse) {
        float big = lds_max[t];
#pragma unroll
        for (uint32_t wv = 1; wv < WAVES; wv++) big = fmaxf(big, lds_max[8u * wv + t]);
        const int e = (int)((__float_as_uint(big) >> 23) & 0xffu);  // biased exponent; 0 for zero and subnormals
        int se = 127 + 14 - (e - 127);                               // scale = 2^(14 - (e - 127)), kept normal both ways
        se = se < 1 ? 1 : se > 253 ? 253 : se;
        if (e == 0 || e == 255) return 1.0f;
        return __uint_as_float((uint32_t)(inverse ? 254 - se : se) << 23);
    };
    if (tid < 8u) lds_scale[8 + tid] = tid < a.m ? scale_of(tid, true) : 1.0f;  // read after a later barrier
    rf16x8 xf[NB * 8];
    {
        const float scale = tok < a.m ? scale_of(tok, false) : 0.f;
#pragma unroll
        for (int s = 0; s < NB * 8; s++) {
            const float x[4] = {raw[s].x, raw[s].y, raw[s].z, raw[s].w};
            // The scale is a power of two, so x * scale - hi in one fused operation is exact.
            _Float16 hi[4], lo[4];
#pragma unroll
            for (int e = 0; e < 4; e++) {
                hi[e] = (_Float16)(x[e] * scale);
                lo[e] = (_Float16)(fmaf(x[e], scale, -(float)hi[e]) * 2048.0f);
            }
            const ru32x2 h2 = __builtin_bit_cast(ru32x2, rf16x4{hi[0], hi[2], hi[1], hi[3]}), l2 = __builtin_bit_cast(ru32x2, rf16x4{lo[0], lo[2], lo[1], lo[3]});
            // The even lane keeps its first roundings and needs the odd lane's; the odd lane keeps
            // its remainders and needs the even lane's.
            const ru32x2 give = sub ? h2 : l2;
            ru32x2 got;
            got.x = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)give.x, 0xB1, 0xf, 0xf, false);  // quad_perm [1, 0, 3, 2]: the neighbour's
            got.y = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)give.y, 0xB1, 0xf, 0xf, false);
            const ru32x4 pick = {sub ? got.x : h2.x, sub ? got.y : h2.y, sub ? l2.x : got.x, sub ? l2.y : got.y};
            xf[s] = __builtin_bit_cast(rf16x8, pick);
        }
    }
    // The rows' sub-block sums, by the matrix cores (the rows times a column of ones): every
    // lane gets the sums of its own two tokens (operand rows 4 g .. 4 g + 3), whatever its column.
    float2 xsum[NB * 8];
    {
        const ru32x4 ones = {0x3C003C00u, 0x3C003C00u, 0x3C003C00u, 0x3C003C00u};
#pragma unroll
        for (int s = 0; s < NB * 8; s++) {
            const rf32x4 d = __builtin_amdgcn_mfma_f32_16x16x32_f16(xf[s], __builtin_bit_cast(rf16x8, ones), rf32x4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
            xsum[s] = float2{fmaf(d[1], 1.0f / 2048.0f, d[0]), fmaf(d[3], 1.0f / 2048.0f, d[2])};
        }
    }

    // The lane's reads of its wave's blocks of a tile: row l16 of the flat copy, blocks
    // NB wave + i. Byte f of the copy sits at 128 (f / 128) + 16 ((f / 16 % 8) ^ (l16 % 8)) + f % 16.
    auto at_byte = [&](uint32_t f) { return (f & ~127u) + 16u * (((f >> 4) & 7u) ^ (l16 & 7u)) + (f & 15u); };
    uint32_t at_header[NB], at_fifth[NB], at_nibbles[NB][4];
#pragma unroll
    for (uint32_t i = 0; i < NB; i++) {
        const uint32_t block = 8u * F::BLOCK * NB * l16 + F::BLOCK * (NB * wave + i);
        at_header[i] = at_byte(block);
        at_fifth[i] = at_byte(block + 16u + 8u * g);
#pragma unroll
        for (uint32_t c = 0; c < 4; c++) at_nibbles[i][c] = at_byte(block + F::NIBBLES_AT + 32u * c + 8u * g);
    }

    float held = 0.f;  // the gate tile's result, until the up tile's arrives
    // Multiplies tile p from its slot and leaves the wave's partial sums in LDS.
    auto multiply = [&](uint32_t p, uint32_t slot) __attribute__((always_inline)) {
        float acc[2] = {0.f, 0.f};  // tokens 2 g and 2 g + 1, matrix row row0 + l16, this wave's k range
        const uint8_t *tile = lds_ring + slot * TILE;
#pragma unroll
        for (int i = 0; i < NB; i++) {
            const ru32x4 h = *reinterpret_cast<const ru32x4 *>(tile + at_header[i]);
            const float d = half_bits_to_float(h.x & 0xffffu), dmin = half_bits_to_float(h.x >> 16);
            // The eight 6-bit scales and minimums as bytes of four words (src/ref/tensor.zig:94-98).
            const uint32_t sc_lo_ = h.y & 0x3f3f3f3fu, mn_lo_ = h.z & 0x3f3f3f3fu;
            const uint32_t sc_hi_ = (h.w & 0x0f0f0f0fu) | ((h.y >> 2) & 0x30303030u);
            uint32_t mn_hi = ((h.w >> 4) & 0x0f0f0f0fu) | ((h.z >> 2) & 0x30303030u);
            // (kept apart from the masks above: a clean byte converts to f32 in one instruction,
            // a 6-bit field of the raw word needs two)
            uint32_t sc_lo = sc_lo_, mn_lo = mn_lo_, sc_hi = sc_hi_;
            asm volatile("" : "+v"(sc_lo), "+v"(mn_lo), "+v"(sc_hi), "+v"(mn_hi));
            ru32x2 bits = {0u, 0u};  // Q5_K: bit sb of a byte is the fifth bit of the position's weight in sub-block sb
            if (F::FIFTH) bits = *reinterpret_cast<const ru32x2 *>(tile + at_fifth[i]);
#pragma unroll
            for (uint32_t c = 0; c < 4; c++) {
                const ru32x2 wq = *reinterpret_cast<const ru32x2 *>(tile + at_nibbles[i][c]);
#pragma unroll
                for (uint32_t half = 0; half < 2; half++) {
                    const uint32_t sb = 2u * c + half, shift = 8u * (sb & 3u);
                    const float dsc = d * (float)(((sb < 4u ? sc_lo : sc_hi) >> shift) & 0xffu);
                    const float off = fmaf(F::BIAS, dsc, dmin * (float)(((sb < 4u ? mn_lo : mn_hi) >> shift) & 0xffu));
                    const ru32x2 fifth = {sb ? bits.x >> sb : bits.x, sb ? bits.y >> sb : bits.y};
                    const rf16x8 wf = half ? nibbles<F, true>(wq, fifth, q.nibble_mask, sixteen) : nibbles<F, false>(wq, fifth, q.nibble_mask, sixteen);
                    const rf32x4 r = __builtin_amdgcn_mfma_f32_16x16x32_f16(xf[8 * i + sb], wf, rf32x4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
                    const float2 xs = xsum[8 * i + sb];
                    acc[0] = fmaf(-off, xs.x, fmaf(dsc, fmaf(r[1], 1.0f / 2048.0f, r[0]), acc[0]));
                    acc[1] = fmaf(-off, xs.y, fmaf(dsc, fmaf(r[3], 1.0f / 2048.0f, r[2]), acc[1]));
                }
            }
        }
        float *part = &lds_part[p & 1u][0][0];
        *reinterpret_cast<float2 *>(part + wave * 128u + 2u * lane) = float2{acc[0], acc[1]};
    };
    // Adds the eight waves' partial sums of tile p, behind the barrier that follows its
    // multiply. Buffer p % 2 is written again by the multiply of tile p + 2, behind the next
    // barrier, which a wave passes only when it has read what it needs here. The 128 outputs of
    // a tile are summed by one pair of waves, a different pair from one output tile to the next
    // (the extra work does not make the same waves late every time).
    auto sum_up = [&](uint32_t p) __attribute__((always_inline)) {
        if ((tid >> 7) != ((p / per) & 3u)) return;
        const float *part = &lds_part[p & 1u][0][0];
        const uint32_t row = tid & 15u, t = (tid >> 4) & 7u;
        const float *src = part + 2u * ((t >> 1) * 16u + row) + (t & 1u);
        float sum = src[0];
#pragma unroll
        for (uint32_t wv = 1; wv < WAVES; wv++) sum += src[wv * 128u];
        sum *= lds_scale[8 + t];
        if (LONG) {
            if (t < a.m && row < rows_of(p)) store_apart(q.partial + ((size_t)(per * kpart + (PAIR ? p & 1u : 0u)) * 8u + t) * a.rows + out0(p) + row, sum);
        } else if (PAIR && !(p & 1u)) {
            held = sum;
        } else {
            const float v = PAIR ? silu_f(held) * sum : sum;
            if (t < a.m && row < rows_of(p)) {
                float *o = a.out + (size_t)t * a.out_stride + a.col0 + out0(p) + row;
                store_apart(o, (a.flags & FLAG_ACCUMULATE) ? *o + v : v);
            }
        }
    };

    // DEPTH ring slots in rotation: DEPTH - 1 tiles in flight behind the one multiplied. One
    // barrier a tile: behind it all of tile p has landed (every wave has waited for its own
    // loads of it), nobody still reads the slot that is refilled next, and the partial sums of
    // the tile before are in LDS.
#pragma unroll
    for (int s = 1; s < DEPTH - 1; s++) load_tile(s, s);
    for (uint32_t p = 0; p < count; p += DEPTH) {
#pragma unroll
        for (int s = 0; s < DEPTH; s++) {
            if (p + s < count) {
                wait_loads<(DEPTH - 2) * LOADS>();
                lds_barrier();
                load_tile(p + s + (DEPTH - 1), (s + DEPTH - 1) % DEPTH);
                if (p + s > 0u) sum_up(p + s - 1u);
                multiply(p + s, s);
            }
        }
    }
    if (count > 0u) {
        lds_barrier();
        sum_up(count - 1u);
    }
    wait_loads<0>();  // nothing may still land in LDS once the workgroup is gone
}

// The outputs of a step over long rows: the parts' sums added in the order of their columns,
// then the SILU_PAIR / ACCUMULATE epilogue. One thread an output.
template <bool PAIR>
__global__ __launch_bounds__(256) void matvec_kquant_mfma_parts_sum_kernel(MvArgs a, const float *partial, uint32_t parts) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x, row = i % a.rows, t = i / a.rows;
    if (t >= a.m) return;
    constexpr uint32_t per = PAIR ? 2u : 1u;
    const float *src = partial + (size_t)t * a.rows + row;
    const size_t plane = (size_t)8u * a.rows;
    float *o = a.out + (size_t)t * a.out_stride + a.col0 + row;
    // Every load first: the parts were written by other workgroups and come from memory.
    float first[kMatvecMaxParts], second[kMatvecMaxParts];
#pragma unroll
    for (uint32_t p = 0; p < kMatvecMaxParts; p++) {
        first[p] = p < parts ? src[per * p * plane] : 0.f;
        second[p] = (PAIR && p < parts) ? src[(per * p + 1u) * plane] : 0.f;
    }
    const float before = (a.flags & FLAG_ACCUMULATE) ? *o : 0.f;
    float sum = first[0], up = second[0];
#pragma unroll
    for (uint32_t p = 1; p < kMatvecMaxParts; p++) {
        if (p < parts) {
            sum += first[p];
            up += second[p];
        }
    }
    const float v = PAIR ? silu_f(sum) * up : sum;
    *o = (a.flags & FLAG_ACCUMULATE) ? before + v : v;
}

}  // namespace

// A token's 1 / sqrt(mean(x^2) + eps), its sum of squares taken as stage_token takes it: vector i
// by thread i % 256, the four waves' sums in order.
__global__ __launch_bounds__(256) void matvec_parts_scales_kernel(MvArgs a, float *scales) {
    __shared__ float red[4];
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, k4 = a.k / 4u;
    const float4 *xrow = reinterpret_cast<const float4 *>(a.x + (size_t)blockIdx.x * a.xr);
    float ss = 0.f;
    for (uint32_t i = tid; i < k4; i += 256u) {
        const float4 v = xrow[i];
        ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
    }
    ss = wave_sum(ss);
    if (lane == 0u) red[wave] = ss;
    __syncthreads();
    if (tid == 0u) scales[blockIdx.x] = 1.0f / sqrtf(((red[0] + red[1]) + (red[2] + red[3])) / (float)a.k + a.eps);
}

zhip_result launch_matvec_parts_scales(const Dispatch &d, const char *name, const MvArgs &a, float *scales) {
    hipLaunchKernelGGL(matvec_parts_scales_kernel, dim3(a.m), dim3(256), 0, d.stream, a, scales);
    return check_launch(d, name);
}

zhip_result launch_matvec_parts_sum(const Dispatch &d, const char *name, const MvArgs &a, const float *partial, uint32_t parts) {
    const dim3 sums((a.rows * a.m + 255u) / 256u);
    if (a.flags & FLAG_SILU_PAIR) hipLaunchKernelGGL(matvec_kquant_mfma_parts_sum_kernel<true>, sums, dim3(256), 0, d.stream, a, partial, parts);
    else hipLaunchKernelGGL(matvec_kquant_mfma_parts_sum_kernel<false>, sums, dim3(256), 0, d.stream, a, partial, parts);
    return check_launch(d, name);
}

// Whether this kernel can run the (already validated) arguments: whole tiles, k split into
// one or two blocks a wave, or rows of 6144 .. 32768 weights in parts of 2048.
bool matvec_q4k_mfma_resident_accepts(const MvArgs &a) {
    const bool pair = a.flags & FLAG_SILU_PAIR;
    const bool parts = a.k > 4096u && a.k % 2048u == 0 && a.k / 2048u <= kMatvecMaxParts;
    return a.m >= 1 && a.m <= 8 && (a.k == 2048u || a.k == 4096u || parts) && a.rows % 16u == 0 && (!pair || a.half % 16u == 0);
}

template <class F>
static zhip_result launch_resident(const Dispatch &d, const MvArgs &a, uint64_t w_bytes, uint32_t mask, uint32_t bias_bits) {
    const bool pair = a.flags & FLAG_SILU_PAIR;
    // 32-bit byte offsets.
    const uint64_t reach = ((uint64_t)(pair ? a.half : 0u) + a.rows + 16u) * a.row_bytes;
    if (w_bytes >= 0xfffffff0ull || reach >= 0xfffffff0ull) return fail(d, ZHIP_E_BAD_COMMAND, "%s: operands of 4 GiB or more", F::name());
    // The workgroups that walk the tiles: one a CU, or (rows of more than 4096 weights) one for
    // every `parts` CUs, each of them `parts` workgroups.
    const uint32_t parts = a.k > 4096u ? a.k / 2048u : 1u;
    const uint32_t cus = (uint32_t)d.dev->compute_units, tiles = a.rows / 16u;
    if (cus < parts) return fail(d, ZHIP_E_GPU, "%s: %u compute units for %u parts of a row", F::name(), cus, parts);
    const uint32_t most = cus / parts;
    const uint32_t groups = tiles < most ? (2u * tiles <= most ? 2u * tiles : tiles) : most;
    const bool halves = tiles < groups;  // every workgroup takes eight outputs of one tile
    const uint32_t left = halves ? tiles : tiles % groups;
    ResArgs q{a, (uint32_t)w_bytes, mask, bias_bits, halves ? 0u : tiles / groups, left, (halves || 2u * left <= groups) ? 1u : 0u, parts, nullptr, nullptr};
    const dim3 grid(groups * parts);
    if (parts > 1u) {
        const uint64_t bytes = (uint64_t)parts * (pair ? 2u : 1u) * 8u * a.rows * sizeof(float);
        if (!d.work) return fail(d, ZHIP_E_GPU, "%s: no workspace", F::name());
        if (zhip_result r = d.work->reserve(d, kPartsScalesBytes + bytes)) return r;
        q.partial = reinterpret_cast<float *>(d.work->data + kPartsScalesBytes);
        if (a.flags & FLAG_NORM) {
            q.scales = reinterpret_cast<const float *>(d.work->data);
            if (zhip_result r = launch_matvec_parts_scales(d, F::name(), a, reinterpret_cast<float *>(d.work->data))) return r;
        }
        if (pair) hipLaunchKernelGGL((matvec_kquant_mfma_resident_kernel<F, true, 1, true>), grid, dim3(THREADS), 0, d.stream, q);
        else hipLaunchKernelGGL((matvec_kquant_mfma_resident_kernel<F, false, 1, true>), grid, dim3(THREADS), 0, d.stream, q);
        if (zhip_result r = check_launch(d, F::name())) return r;
        return launch_matvec_parts_sum(d, F::name(), a, q.partial, parts);
    } else if (a.k == 2048u) {
        if (pair) hipLaunchKernelGGL((matvec_kquant_mfma_resident_kernel<F, true, 1, false>), grid, dim3(THREADS), 0, d.stream, q);
        else hipLaunchKernelGGL((matvec_kquant_mfma_resident_kernel<F, false, 1, false>), grid, dim3(THREADS), 0, d.stream, q);
    } else {
        if (pair) hipLaunchKernelGGL((matvec_kquant_mfma_resident_kernel<F, true, 2, false>), grid, dim3(THREADS), 0, d.stream, q);
        else hipLaunchKernelGGL((matvec_kquant_mfma_resident_kernel<F, false, 2, false>), grid, dim3(THREADS), 0, d.stream, q);
    }
    return check_launch(d, F::name());
}

zhip_result launch_matvec_q4k_mfma_resident(const Dispatch &d, const MvArgs &a, uint64_t w_bytes) {
    return launch_resident<ResQ4>(d, a, w_bytes, 0x03C003C0u, 0x4C004C00u);
}

// The same for matvec_q5_k (the arguments the Q4_K kernel accepts, rows of 176-byte blocks).
bool matvec_q5k_mfma_resident_accepts(const MvArgs &a) { return matvec_q4k_mfma_resident_accepts(a) && a.row_bytes == a.k / 256u * 176u; }
zhip_result launch_matvec_q5k_mfma_resident(const Dispatch &d, const MvArgs &a, uint64_t w_bytes) {
    return launch_resident<ResQ5>(d, a, w_bytes, 0x01E001E0u, 0x50005000u);
}

}  // namespace zhip
