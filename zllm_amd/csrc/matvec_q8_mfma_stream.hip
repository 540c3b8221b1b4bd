// matvec_q8_0, matrix-core variant for steps of up to eight tokens and k = 2048 or 4096 (longer
// rows in parts, below): the
// weight stream is read once for all tokens of the step and nothing but partial sums crosses
// LDS. Contract as the other variants (src/kernels/matvec_quant.wgsl.hbs with the decoder of
// src/kernels/quant/q8_0_dot.wgsl:5-14): out[t][col0 + j] (+)= sum over 32-weight blocks of
// d * sum(q * x).
//
// Arithmetic. v_mfma_f32_16x16x32_f16 multiplies sixteen rows of inputs by sixteen weight rows
// over one 32-weight block. The int8 weights enter as exact f16 values (a byte dropped into the
// mantissa of 1024.0 and 1152 subtracted: five vector instructions per four weights, once for
// all tokens); every token enters as two rows, the f16 rounding of its inputs and the f16
// rounding of what that left times 2^11, after a power of two has put its largest magnitude at
// 2^14: an input keeps 22 bits, every product is exact in the f32 accumulator, and the block's
// scale multiplies the block's sum afterwards. A token's rows meet no other token's anywhere:
// its results do not depend on how many tokens share the launch.
//
// Layout of the work. A 512-thread workgroup is eight waves that split k eight ways (8 or 16
// blocks a wave); a wave builds its k range of all tokens' rows once, straight into operands
// that stay in registers (64 VGPRs at k = 4096). Persistent workgroups take sixteen-row weight
// tiles b, b + G, ...; a wave's part of a tile (its 256 or 512 bytes of each of the sixteen
// rows, and their scales) arrives in a private ring of LDS slots by wave-wide direct loads of
// whole lines, a tile or more ahead, and each lane reads its row's eight bytes of a block back
// for one matrix instruction. (The matrix instruction wants lane l to hold row l % 16, so a
// lane loading its own bytes makes every lane of a load touch another cache line: the vector
// memory unit then moves 16 bytes per line it looks up and the kernel ran at 20.7 us on
// 14336 x 4096, 27 us with 8 bytes a lane.) Chunk c (16 bytes) of row r sits at position
// c ^ r of the row's line in the slot: the sixteen rows' reads of one block fall in sixteen
// different banks. The eight waves' partial sums meet in LDS, where 128 threads add the eight
// for one output each in the order of the k ranges and store. One barrier a tile; no barrier
// waits for the loads in flight.
// (k = 1024 is not taken here: a row and its scales are 1088 bytes, so every other row starts
// in the middle of a cache line and a wave's 128 bytes of it lie across two; 151936 x 1024 ran
// at 42 us, 3.9 TB/s against 6.6 TB/s at k = 4096. Such rows go to the kernel that moves a
// tile's rows as one stretch of whole lines, matvec_q6k_mfma_stream.hip.)
// Rows of 6144 .. 32768 weights (a multiple of 2048): k / 2048 workgroups share a walker's tiles,
// each over 2048 columns (eight blocks a wave) and under its own per-token scales; they store
// their sums per part and launch_matvec_parts_sum (matvec_mfma_resident.hip) adds them in the
// order of their columns and applies the epilogue; with the RMSNorm prologue the tokens' scales
// come ready from launch_matvec_parts_scales. 4096 x 14336 at four / eight tokens: 18.9 /
// 19.2 us (default variant 26.5 / 50.7).
#include <hip/hip_runtime.h>

#include <type_traits>

#include "common.h"
#include "decode.h"
#include "matvec_common.h"

namespace zhip {

namespace {

typedef _Float16 sf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 sf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 sf16x4 __attribute__((ext_vector_type(4)));
typedef float sf32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t su32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t su32x2 __attribute__((ext_vector_type(2)));

constexpr uint32_t THREADS = 512, WAVES = 8;

struct StreamArgs {
    MvArgs a;
    uint32_t w_bytes;    // bytes bound behind the weights (the loads are range-checked)
    uint32_t rounds;     // sixteen-row tiles every workgroup takes: tiles b, b + G, ...
    uint32_t left;       // tiles after those, fewer than G: one for each of the first workgroups,
    uint32_t split;      // or (split) half of one, eight rows, for each of the first 2 * left
    uint32_t bias;       // 0x64646464: the bytes of two f16 1024.0 exponents, as a kernel argument
                         // so that the byte shuffles stay one instruction each
    // Rows of more than 4096 weights: `parts` workgroups share a tile, each over 2048 of its
    // columns, and leave their sums in `partial` ([part][gate, up][token of 8][output]).
    uint32_t parts;
    float *partial;
    const float *scales;  // with the RMSNorm prologue: each token's 1 / sqrt(mean(x^2) + eps)
};

// A barrier that waits for this wave's LDS traffic only: the weight loads of the tile ahead
// stay in flight.
__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// A 4-byte store the compiler's wait-count bookkeeping does not see as a store: with one pending
// it would turn every wait for a weight load into a wait for all loads in flight (loads and
// stores complete out of order with each other). A wait that counts only the loads issued
// after the awaited one stays sufficient while a store is outstanding.
__device__ __forceinline__ void store_apart(float *at, float v) {
    asm volatile("global_store_dword %0, %1, off\n\ts_nop 0" ::"v"(at), "v"(v) : "memory");
}

// Eight int8 weights (two words) as exact f16 values in position order.
__device__ __forceinline__ sf16x8 weights_f16(su32x2 w, uint32_t bias) {
    const sf16x2 off = {(_Float16)-1152.0f, (_Float16)-1152.0f};
    su32x4 r;
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const uint32_t u = w[i] ^ 0x80808080u;  // q + 128 in every byte
        // bytes (low to high) u0 0x64 u1 0x64: the f16 pair (1024 + u0, 1024 + u1); then u2, u3
        const uint32_t lo = __builtin_amdgcn_perm(bias, u, 0x04010400u), hi = __builtin_amdgcn_perm(bias, u, 0x04030402u);
        r[2 * i] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(sf16x2, lo) + off);
        r[2 * i + 1] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(sf16x2, hi) + off);
    }
    return __builtin_bit_cast(sf16x8, r);
}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_buffer(const void *base, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, 0x00020000);
}
typedef __attribute__((address_space(3))) void *lds_ptr;
// One wave-wide load of 16 bytes a lane straight into LDS (lane l lands at dst + 16 l). The
// destination reaches the load as a bare LDS address, so the compiler keeps no dependency
// between these loads and later LDS reads; the explicit waits order them.
__device__ __forceinline__ void load_lds_b128(__amdgpu_buffer_rsrc_t buf, uint32_t dst, uint32_t voffset, uint32_t soffset) {
    asm volatile("" : "+s"(dst));
    __builtin_amdgcn_raw_ptr_buffer_load_lds(buf, (lds_ptr)(uintptr_t)dst, 16, voffset, soffset, 0, 0);
}
template <int LEFT>
__device__ __forceinline__ void wait_loads() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(LEFT) : "memory");
}

__device__ __forceinline__ void load_lds_b32(__amdgpu_buffer_rsrc_t buf, uint32_t dst, uint32_t voffset, uint32_t soffset) {
    asm volatile("" : "+s"(dst));
    __builtin_amdgcn_raw_ptr_buffer_load_lds(buf, (lds_ptr)(uintptr_t)dst, 4, voffset, soffset, 0, 0);
}

// NS: 32-weight blocks of a wave's k range (k = 256 NS). The ring moves half tiles: the first or
// second NS / 2 blocks of the wave's range of a tile's sixteen rows. A slot: sixteen lines, then 256 bytes for the scales' load
// (two bytes a block and row; zeros from idle lanes behind).
constexpr int DEPTH = 4;  // ring slots a wave: three half tiles in flight behind the one multiplied
template <int NS> constexpr uint32_t slot_bytes() { return 16u * 32u * (NS / 2) + 256u; }
constexpr uint32_t PART_BYTES = 2u * WAVES * 128u * 4u, SCALE_BYTES = 576u;  // [8 waves][8 tokens] maxima, [8] inverse scales, [8 waves][8 tokens] sums of squares
template <int NS> constexpr uint32_t lds_bytes() { return PART_BYTES + SCALE_BYTES + WAVES * DEPTH * slot_bytes<NS>(); }
static_assert(lds_bytes<16>() <= 160u * 1024u, "the rings must fit the CU's LDS");

// LONG (NS = 8): k = 2048 q.parts; workgroup i multiplies columns 2048 (i % parts) .. (part
// `kpart`) of the tiles that walker i / parts takes, and launch_matvec_parts_sum adds the parts.
template <int NS, bool LONG>
__global__ __launch_bounds__(THREADS) void matvec_q8_mfma_stream_kernel(StreamArgs q) {
    static_assert(!LONG || NS == 8, "parts of a long row are 2048 columns");
    const MvArgs &a = q.a;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    float *lds_part = reinterpret_cast<float *>(lds);                  // [tile parity][wave][2 lane + token of the lane's two]
    float *lds_max = reinterpret_cast<float *>(lds + PART_BYTES);      // [wave][token]: the largest magnitude in the wave's range
    float *lds_inverse = lds_max + 64;                                 // [token]: one over the token's scale
    static_assert(NS >= 8, "a half tile is whole 128-byte lines of every row");
    constexpr int PARTS = 2;  // ring slots a wave's range of a tile takes
    constexpr int HB = NS / PARTS;           // blocks of a half tile
    constexpr uint32_t SLOT = slot_bytes<NS>(), LINE = 32u * HB, CHUNKS = 2u * HB;
    const uint32_t tid = threadIdx.x, lane = tid & 63u, l16 = lane & 15u, g = lane >> 4;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    uint8_t *ring = lds + PART_BYTES + SCALE_BYTES + wave * (DEPTH * SLOT);
    const uint32_t ring0 = (uint32_t)(uintptr_t)ring;
    const __amdgpu_buffer_rsrc_t wbuf = make_buffer(a.w, q.w_bytes), nobuf = make_buffer(a.w, 0);
    uint32_t bias = q.bias;
    asm volatile("" : "+v"(bias));

    // The workgroup's tiles: b, b + G, ... and perhaps a last one, or eight rows of it (when the
    // tiles left over after whole rounds are at most half as many as the workgroups, two
    // workgroups share each: a whole tile more on half of the CUs would be the launch's tail).
    // Half tile u is half u % 2 of tile u / 2.
    // With SILU_PAIR (src/kernels/matvec_quant.wgsl.hbs:110-125) an output tile is two weight
    // tiles, the gate rows and then the up rows `half` further down: tile p of the run is weight
    // tile p % per of output tile p / per.
    const uint32_t per = (a.flags & FLAG_SILU_PAIR) ? 2u : 1u;
    const uint32_t kpart = LONG ? blockIdx.x % q.parts : 0u, walker = LONG ? blockIdx.x / q.parts : blockIdx.x, walkers = LONG ? gridDim.x / q.parts : gridDim.x;
    const bool extra = walker < (q.split ? 2u * q.left : q.left);
    const uint32_t count = per * (q.rounds + (extra ? 1u : 0u));
    const uint32_t last_row = 16u * (q.rounds * walkers + (q.split ? walker >> 1 : walker)) + (q.split ? 8u * (walker & 1u) : 0u);
    auto out0 = [&](uint32_t p) { return p / per < q.rounds ? 16u * (walker + (p / per) * walkers) : last_row; };  // first output of tile p
    auto first_row = [&](uint32_t p) { return out0(p) + ((p % per) ? a.half : 0u); };
    auto rows_of = [&](uint32_t p) { return (q.split && p / per >= q.rounds) ? 8u : 16u; };
    // A half tile's loads. Weights: load i brings rows (64 / CHUNKS) i .. of the half's k range,
    // lane l row l / CHUNKS and the chunk that belongs at position l % CHUNKS: chunk c of row r
    // sits at position c ^ key(r), the key such that sixteen rows' reads of one chunk fall in
    // sixteen different 16-byte bank groups. Scales: lane l brings word l % (HB / 2) of row
    // l / (HB / 2); lanes past the sixteenth row ask past the buffer and zeros land.
    constexpr int ROWS_PER_LOAD = 64 / CHUNKS, WLOADS = 16 / ROWS_PER_LOAD, LOADS = WLOADS + 1;
    auto line_key = [](uint32_t row) { return (row / (256u / LINE)) % CHUNKS; };
    const uint32_t lrow = lane / CHUNKS, lpos = lane % CHUNKS;
    uint32_t woff[WLOADS];
#pragma unroll
    for (int i = 0; i < WLOADS; i++) {
        const uint32_t row = ROWS_PER_LOAD * i + lrow;
        woff[i] = row * a.row_bytes + 2048u * kpart + PARTS * LINE * wave + 16u * (lpos ^ line_key(row));
    }
    constexpr uint32_t SWORDS = HB / 2;  // words of scales a row and half
    const uint32_t soff = (lane / SWORDS) * a.row_bytes + a.k + 128u * kpart + 2u * NS * wave + 4u * (lane % SWORDS);
    auto load_half = [&](uint32_t u, uint32_t slot) __attribute__((always_inline)) {
        // (past the run's last tile the loads still run, so that the waits count the same loads
        // every step, but against an empty buffer: zeros land and nothing is fetched)
        const uint32_t p = u / PARTS, half = u % PARTS;
        const __amdgpu_buffer_rsrc_t buf = p < count ? wbuf : nobuf;
        const uint32_t base = first_row(p) * a.row_bytes, rows = rows_of(p);
        const uint32_t dst = ring0 + slot * SLOT;
        // (the rows an eight-row share does not have are not fetched; what the matrix
        // instructions make of their slots' old contents is never stored)
#pragma unroll
        for (int i = 0; i < WLOADS; i++) load_lds_b128((uint32_t)(ROWS_PER_LOAD * i) < rows ? buf : nobuf, dst + 1024u * i, woff[i], base + LINE * half);
        load_lds_b32(buf, dst + 16u * LINE, lane < rows * SWORDS ? soff : 0xfffffff0u, base + 2u * HB * half);
    };
    // The tokens' inputs first: loads complete in order within a wave, and behind the weight
    // loads below the first use of an input would wait for a round trip of the weight stream.
    // Operand row l16 of the matrix instruction is token l16 / 2: the f16 rounding of its scaled
    // inputs (even rows) or what that left, times 2^11 (odd rows); the lane's eight positions of
    // block s are 8 g .. 8 g + 7. The two lanes of a token and group share the work: the even one
    // loads and splits positions 0 .. 3, the odd one 4 .. 7, and they swap what the other needs.
    // An absent token's rows read the last token's inputs under a scale of zero: no branches, so
    // all of the lane's loads go out together.
    const uint32_t tok = l16 >> 1, sub = l16 & 1u, tsrc = tok < a.m ? tok : a.m - 1u;
    float4 raw[NS];
    {
        const float *xt = a.x + (size_t)tsrc * a.xr + 2048u * kpart + NS * 32u * wave + 8u * g + 4u * sub;
#pragma unroll
        for (int s = 0; s < NS; s++) raw[s] = *reinterpret_cast<const float4 *>(xt + 32 * s);
    }
    // A step's prologue (src/kernels/matvec_quant.wgsl.hbs:73-89) on the same registers, in the
    // default variant's arithmetic: RMSNorm times the norm weights (the wave ranges' sums of
    // squares meet in LDS, added in the order of the ranges) and / or silu(x / act_div).
    // (the sum of squares of a long row is not any one workgroup's: it comes ready in q.scales)
    const bool norm = (a.flags & FLAG_NORM) != 0, act = a.act_div > 0.f;
    float4 gw[NS];
    float ready = 0.f;  // (asked for before the first weights, like the inputs)
    if (norm) {
        const float *gt = a.norm_w + 2048u * kpart + NS * 32u * wave + 8u * g + 4u * sub;
#pragma unroll
        for (int s = 0; s < NS; s++) gw[s] = *reinterpret_cast<const float4 *>(gt + 32 * s);
        if (LONG) ready = q.scales[tsrc];
    }
    // (One half tile of weights behind them for now: with more, the requests of the workgroups
    // that start first fill the memory system's queues and the inputs of the others arrive
    // after them, 4.5 us into the kernel instead of 1.7.)
    load_half(0, 0);
    if (norm) {
        float rs;
        if (LONG) {
            rs = ready;
        } else {
            float ss = 0.f;
#pragma unroll
            for (int s = 0; s < NS; s++) ss += raw[s].x * raw[s].x + raw[s].y * raw[s].y + raw[s].z * raw[s].z + raw[s].w * raw[s].w;
            ss += __shfl_xor(ss, 1, 64);
            ss += __shfl_xor(ss, 16, 64);
            ss += __shfl_xor(ss, 32, 64);
            float *lds_ss = lds_inverse + 8;  // [wave][token]: the range's sum of squares
            if (g == 0u && sub == 0u) lds_ss[8u * wave + tok] = ss;
            lds_barrier();
            float total = lds_ss[tok];
#pragma unroll
            for (uint32_t wv = 1; wv < WAVES; wv++) total += lds_ss[8u * wv + tok];
            rs = 1.0f / sqrtf(total / (float)a.k + a.eps);
        }
#pragma unroll
        for (int s = 0; s < NS; s++) {
            raw[s].x = raw[s].x * rs * gw[s].x; raw[s].y = raw[s].y * rs * gw[s].y;
            raw[s].z = raw[s].z * rs * gw[s].z; raw[s].w = raw[s].w * rs * gw[s].w;
        }
    }
    if (act) {
#pragma unroll
        for (int s = 0; s < NS; s++) {
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
        for (int s = 0; s < NS; s++) big = fmaxf(fmaxf(fabsf(raw[s].x), fabsf(raw[s].y)), fmaxf(fmaxf(fabsf(raw[s].z), fabsf(raw[s].w)), big));
        big = fmaxf(big, __shfl_xor(big, 1, 64));
        big = fmaxf(big, __shfl_xor(big, 16, 64));
        big = fmaxf(big, __shfl_xor(big, 32, 64));
        if (g == 0u && sub == 0u) lds_max[8u * wave + tok] = big;
    }
    lds_barrier();
#pragma unroll
    for (int s = 1; s < DEPTH - 1; s++) load_half(s, s);
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
    if (tid < 8u) lds_inverse[tid] = tid < a.m ? scale_of(tid, true) : 1.0f;  // read after a later barrier
    sf16x8 xf[NS];
    {
        const float scale = tok < a.m ? scale_of(tok, false) : 0.f;
#pragma unroll
        for (int s = 0; s < NS; s++) {
            const float x[4] = {raw[s].x, raw[s].y, raw[s].z, raw[s].w};
            // The scale is a power of two, so x * scale - hi in one fused operation is exact.
            _Float16 hi[4], lo[4];
#pragma unroll
            for (int e = 0; e < 4; e++) {
                hi[e] = (_Float16)(x[e] * scale);
                lo[e] = (_Float16)(fmaf(x[e], scale, -(float)hi[e]) * 2048.0f);
            }
            const su32x2 h2 = __builtin_bit_cast(su32x2, sf16x4{hi[0], hi[1], hi[2], hi[3]}), l2 = __builtin_bit_cast(su32x2, sf16x4{lo[0], lo[1], lo[2], lo[3]});
            // The even lane keeps its first roundings and needs the odd lane's; the odd lane keeps
            // its remainders and needs the even lane's.
            const su32x2 give = sub ? h2 : l2;
            su32x2 got;
            got.x = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)give.x, 0xB1, 0xf, 0xf, false);  // quad_perm [1, 0, 3, 2]: the neighbour's
            got.y = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)give.y, 0xB1, 0xf, 0xf, false);
            const su32x4 pick = {sub ? got.x : h2.x, sub ? got.y : h2.y, sub ? l2.x : got.x, sub ? l2.y : got.y};
            xf[s] = __builtin_bit_cast(sf16x8, pick);
        }
    }

    const uint32_t r_at = l16 * LINE + 8u * (g & 1u), r_key = line_key(l16), r_half = g >> 1;
    float acc[2] = {0.f, 0.f};  // tokens 2 g and 2 g + 1, matrix row 16 tile + l16, this wave's k range
    auto multiply = [&](auto half, uint32_t slot) __attribute__((always_inline)) {
        constexpr int H = decltype(half)::value;
        const uint8_t *t = ring + slot * SLOT;
        uint32_t d[SWORDS];
        if constexpr (SWORDS == 4) {
            const su32x4 v = *reinterpret_cast<const su32x4 *>(t + 16u * LINE + l16 * 16u);
            d[0] = v.x; d[1] = v.y; d[2] = v.z; d[3] = v.w;
        } else {
            static_assert(SWORDS == 2, "two or four words of scales a row");
            const su32x2 v = *reinterpret_cast<const su32x2 *>(t + 16u * LINE + l16 * 8u);
            d[0] = v.x; d[1] = v.y;
        }
#pragma unroll
        for (int s = 0; s < HB; s++) {
            const su32x2 w = *reinterpret_cast<const su32x2 *>(t + r_at + 16u * ((2u * s + r_half) ^ r_key));
            const float ds = half_bits_to_float((s & 1) ? d[s / 2] >> 16 : d[s / 2] & 0xffffu);
            const sf32x4 r = __builtin_amdgcn_mfma_f32_16x16x32_f16(xf[HB * H + s], weights_f16(w, bias), sf32x4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
            acc[0] = fmaf(ds, fmaf(r[1], 1.0f / 2048.0f, r[0]), acc[0]);
            acc[1] = fmaf(ds, fmaf(r[3], 1.0f / 2048.0f, r[2]), acc[1]);
        }
    };
    float held = 0.f;
    auto finish = [&](uint32_t p) __attribute__((always_inline)) {
        float *part = lds_part + (p & 1u) * (WAVES * 128u);
        *reinterpret_cast<float2 *>(part + wave * 128u + 2u * lane) = float2{acc[0], acc[1]};
        acc[0] = acc[1] = 0.f;
        lds_barrier();
        // Buffer p % 2 is written again in step p + 2, after the barrier of step p + 1, which a
        // wave passes only when it has read what it needs here. The 128 outputs of a tile are
        // summed by one pair of waves, a different pair from one tile to the next.
        if ((tid >> 7) == ((p / per) & 3u)) {
            const uint32_t row = tid & 15u, tk = (tid >> 4) & 7u;
            const float *src = part + 2u * ((tk >> 1) * 16u + row) + (tk & 1u);
            float sum = src[0];
#pragma unroll
            for (uint32_t wv = 1; wv < WAVES; wv++) sum += src[wv * 128u];
            sum *= lds_inverse[tk];
            if (LONG) {
                if (tk < a.m && row < rows_of(p)) store_apart(q.partial + ((size_t)(per * kpart + (p % per)) * 8u + tk) * a.rows + out0(p) + row, sum);
            } else if (per == 2u && !(p & 1u)) {
                held = sum;  // the gate tile's result, until the up tile's arrives
            } else {
                const float v = per == 2u ? silu_f(held) * sum : sum;
                if (tk < a.m && row < rows_of(p)) {
                    float *o = a.out + (size_t)tk * a.out_stride + a.col0 + out0(p) + row;
                    store_apart(o, (a.flags & FLAG_ACCUMULATE) ? *o + v : v);
                }
            }
        }
    };

    // DEPTH ring slots in rotation: DEPTH - 1 half tiles in flight behind the one multiplied
    // (with a single whole tile ahead every workgroup asked for its next tile only once the
    // last had arrived in full, and the memory idled for a round trip per tile: 18.3 us
    // against 20.7 us with the lanes' own loads). Every wave of the workgroup runs the same
    // steps (the barrier inside). Before half tile u is read, all but the loads of the
    // DEPTH - 1 half tiles after it have landed.
    for (uint32_t u = 0; u < PARTS * count; u += DEPTH) {
#pragma unroll
        for (int s = 0; s < DEPTH; s++) {
            // The slot refilled now was read by the multiply before: its reads must have returned
            // before the load is issued (a load past the run's end lands at once), and the
            // compiler, which sees no dependency between the two, must not move it up.
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            load_half(u + s + (DEPTH - 1), (s + DEPTH - 1) % DEPTH);
            wait_loads<(DEPTH - 1) * LOADS>();
            if (u + s < PARTS * count) {
                if (s & 1) {
                    multiply(std::integral_constant<int, 1>{}, s);
                    finish((u + s) >> 1);
                } else {
                    multiply(std::integral_constant<int, 0>{}, s);
                }
            }
        }
    }
    wait_loads<0>();  // nothing may still land in LDS once the workgroup is gone
}

}  // namespace

// Whether this kernel can run the (already validated) arguments: whole tiles, k split into 4, 8
// or 16 blocks a wave.
bool matvec_q8_mfma_stream_accepts(const MvArgs &a) {
    // (rows of 6144 .. 32768 weights in parts of 2048)
    const bool parts = a.k > 4096u && a.k % 2048u == 0 && a.k / 2048u <= kMatvecMaxParts;
    return a.m >= 1 && a.m <= 8 && (a.k == 2048u || a.k == 4096u || parts) && (!(a.flags & FLAG_SILU_PAIR) || a.half % 16u == 0) && a.rows % 16u == 0 &&
           a.xr % 4u == 0 && (reinterpret_cast<uintptr_t>(a.x) & 15u) == 0 && (reinterpret_cast<uintptr_t>(a.w) & 15u) == 0;
}

template <int NS, bool LONG = false>
static zhip_result launch_blocks(const Dispatch &d, const StreamArgs &q, dim3 grid) {
    auto kernel = matvec_q8_mfma_stream_kernel<NS, LONG>;
    static bool configured = false;
    if (!configured) {
        if (hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes<NS>()) != hipSuccess) {
            (void)hipGetLastError();
            return fail(d, ZHIP_E_GPU, "matvec_q8_0: cannot reserve %u bytes of LDS", lds_bytes<NS>());
        }
        configured = true;
    }
    hipLaunchKernelGGL(kernel, grid, dim3(THREADS), lds_bytes<NS>(), d.stream, q);
    return check_launch(d, "matvec_q8_0");
}

zhip_result launch_matvec_q8_mfma_stream(const Dispatch &d, const MvArgs &a, uint64_t w_bytes) {
    // 32-bit byte offsets, a tile past the last row.
    const uint64_t reach = ((uint64_t)((a.flags & FLAG_SILU_PAIR) ? a.half : 0u) + a.rows + 16u) * a.row_bytes;
    if (w_bytes >= 0xfffffff0ull || reach >= 0xfffffff0ull) return fail(d, ZHIP_E_BAD_COMMAND, "matvec_q8_0: operands of 4 GiB or more");
    // The workgroups that walk the tiles: one a CU, or (rows of more than 4096 weights) one for
    // every `parts` CUs, each of them `parts` workgroups.
    const uint32_t parts = a.k > 4096u ? a.k / 2048u : 1u;
    const uint32_t cus = (uint32_t)d.dev->compute_units, tiles = a.rows / 16u;
    if (cus < parts) return fail(d, ZHIP_E_GPU, "matvec_q8_0: %u compute units for %u parts of a row", cus, parts);
    const uint32_t most = cus / parts;
    const uint32_t groups = tiles < most ? (2u * tiles <= most ? 2u * tiles : tiles) : most;
    const uint32_t left = tiles % groups;
    StreamArgs q{a, (uint32_t)w_bytes, tiles / groups, left, (tiles < groups || 2u * left <= groups) ? 1u : 0u, 0x64646464u, parts, nullptr, nullptr};
    if (tiles < groups) { q.rounds = 0; q.left = tiles; }
    const dim3 grid(groups * parts);
    if (parts > 1u) {
        const uint64_t bytes = (uint64_t)parts * ((a.flags & FLAG_SILU_PAIR) ? 2u : 1u) * 8u * a.rows * sizeof(float);
        if (!d.work) return fail(d, ZHIP_E_GPU, "matvec_q8_0: no workspace");
        if (zhip_result r = d.work->reserve(d, kPartsScalesBytes + bytes)) return r;
        q.partial = reinterpret_cast<float *>(d.work->data + kPartsScalesBytes);
        if (a.flags & FLAG_NORM) {
            q.scales = reinterpret_cast<const float *>(d.work->data);
            if (zhip_result r = launch_matvec_parts_scales(d, "matvec_q8_0", a, reinterpret_cast<float *>(d.work->data))) return r;
        }
        if (zhip_result r = launch_blocks<8, true>(d, q, grid)) return r;
        return launch_matvec_parts_sum(d, "matvec_q8_0", a, q.partial, parts);
    }
    return a.k == 2048u ? launch_blocks<8>(d, q, grid) : launch_blocks<16>(d, q, grid);
}

}  // namespace zhip
