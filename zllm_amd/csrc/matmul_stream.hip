// matmul_bf16 and matmul_q8_0_float on the matrix cores for steps of up to 128
// tokens over a short k (up to 1024) and many matrix rows: the vocabulary
// projection of a prefill chunk (the contracts of src/kernels/matmul_half.wgsl
// and matmul_q8_0_float.wgsl, the bf16 rung's operands: Q8_0 weights become
// bf16(q * d)).
// Such a step is bound by the one pass over the weights, like a decode
// multiply, so the kernel is built like one: the weights stream from memory
// straight into the registers of the wave that multiplies them, each byte
// loaded once by one wave, and nothing but results crosses LDS.
//
// A 512-thread workgroup is eight waves that split k eight ways. A wave keeps
// its k range of every token in registers for the whole kernel, as matrix-core
// operands (up to 128 tokens x 128 positions = 128 VGPRs), and walks over
// sixteen-row weight tiles: a tile's operand is the lane's own row and eight
// positions (16 bytes; the four lane groups cover 64 contiguous bytes of a row,
// so a load touches 16 half lines, which costs what 8 whole lines cost), loaded
// DEPTH - 1 tiles ahead. v_mfma_f32_16x16x32_bf16 takes the weights as its first
// operand, so a lane ends up with four neighbouring outputs of one token; the
// eight waves' partial sums meet in LDS (one 16-byte write a lane and token
// tile) and thread i adds the eight partial vectors i, always in the order of
// the k ranges, while the matrix cores are already on the next tile. The sums
// of two neighbouring tiles are stored together, eight lanes to a token's 128
// bytes: a store that fills whole cache lines spares L2 from fetching them
// first (a plain copy with this write pattern takes 10 us longer over 78 MB in
// 64-byte pieces than in 128-byte ones). Workgroups are persistent: workgroup
// b of G takes the pairs of tiles b, b + G, b + 2 G ...
#include <hip/hip_runtime.h>

#include "common.h"
#include "decode.h"

namespace zhip {

typedef __bf16 sbf16x8 __attribute__((ext_vector_type(8)));
typedef float sf32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t su32x4 __attribute__((ext_vector_type(4)));

namespace {

constexpr uint32_t THREADS = 512, WAVES = 8;
constexpr int DEPTH = 2;  // weight tiles in registers a wave: one multiplied, the others in flight

struct StreamArgs {
    const uint8_t *x;  // packed bf16 rows
    const uint8_t *w;
    float *out;
    uint32_t rows, n, k, col0, out_stride, accumulate;
    uint32_t x_bytes, w_bytes;
    uint32_t row_bytes; // bytes between weight rows
    uint32_t tiles;     // sixteen-row weight tiles
};

typedef uint32_t su32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 sbf16x2 __attribute__((ext_vector_type(2)));
typedef float sf32x2 __attribute__((ext_vector_type(2)));

// Two floats to packed bf16, round to nearest even (src/ref/matmul.zig:250-255).
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    const sf32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, sbf16x2));
}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_buffer(const uint8_t *base, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(base), 0, (int)bytes, 0x00020000);
}

// A barrier that waits for this wave's LDS traffic only: the weight loads of the
// tiles ahead stay in flight.
__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// Stores 16 bytes without the compiler's wait-count bookkeeping seeing a store. Loads
// and stores complete out of order with each other, so with a store pending the
// compiler makes every wait for a load a wait for all outstanding memory
// operations, which would drain the weight tiles in flight once per tile. A wait
// that counts only the loads issued after the awaited one is still sufficient
// while a store is outstanding (loads complete in order among themselves; the
// store only makes the wait stricter). The two idle cycles keep a following
// instruction from overwriting the data registers before the store has read them.
// The outputs are written once and not read again by this kernel: the non-temporal
// hint keeps them from displacing the weight stream in L2 (measured 86.6 -> 84.4 us
// on 128 x 1024 x 151936).
__device__ __forceinline__ void store_apart(sf32x4 *at, sf32x4 v) {
    asm volatile("global_store_dwordx4 %0, %1, off nt\n\ts_nop 1" ::"v"(at), "v"(v) : "memory");
}

// Each lane's vector of the lane whose number times four is `from`.
__device__ __forceinline__ sf32x4 from_lane(sf32x4 v, uint32_t from) {
    sf32x4 r;
    r.x = __int_as_float(__builtin_amdgcn_ds_bpermute((int)from, __float_as_int(v.x)));
    r.y = __int_as_float(__builtin_amdgcn_ds_bpermute((int)from, __float_as_int(v.y)));
    r.z = __int_as_float(__builtin_amdgcn_ds_bpermute((int)from, __float_as_int(v.z)));
    r.w = __int_as_float(__builtin_amdgcn_ds_bpermute((int)from, __float_as_int(v.w)));
    return r;
}

// MT: token tiles of sixteen (rows <= 16 MT); KC: 32-position chunks of a wave's
// k range (k = 256 KC).
template <int MT, int KC, bool Q8>
__global__ __launch_bounds__(THREADS) void matmul_stream_kernel(StreamArgs a) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];  // [2][wave][MT * 64 lanes] partial vectors
    constexpr uint32_t PART = MT * 64u * 16u;                       // bytes a wave writes per tile
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, l16 = lane & 15u, g = lane >> 4;
    const __amdgpu_buffer_rsrc_t xbuf = make_buffer(a.x, a.x_bytes), wbuf = make_buffer(a.w, a.w_bytes);
    // The lane's eight positions of chunk c. BF16 rows: k = 32 KC wave + 32 c + 8 g (a 16-byte
    // load a chunk). Q8_0 rows: a 16-byte load holds sixteen weights, two chunks' worth, so
    // chunk c = 2 j + h takes k = 32 KC wave + 64 j + 16 g + 8 h: the lane's load j covers
    // 16 g .. 16 g + 15 of the 64 and a row's four lanes 64 contiguous bytes either way.
    static_assert(!Q8 || KC % 2 == 0, "a Q8_0 load feeds two chunks");
    const uint32_t kw = 32u * KC * wave;
    auto kpos = [&](int c) { return Q8 ? kw + 64u * (c >> 1) + 16u * g + 8u * (c & 1) : kw + 32u * c + 8u * g; };

    // This wave's part of every token (tokens past `rows` lie past the buffer: zeros).
    sbf16x8 xf[MT][KC];
#pragma unroll
    for (int i = 0; i < MT; i++)
#pragma unroll
        for (int c = 0; c < KC; c++)
            xf[i][c] = __builtin_bit_cast(sbf16x8, __builtin_amdgcn_raw_buffer_load_b128(xbuf, ((16u * i + l16) * a.k + kpos(c)) * 2u, 0, 0));

    // This workgroup's tiles, in pairs (a pair's outputs fill whole 128-byte lines): pairs
    // b, b + G, b + 2 G ... of the G workgroups, so that at any time the chip reads one
    // contiguous stretch of the matrix. Tile p of the run:
    const uint32_t pairs = (a.tiles + 1u) / 2u;
    auto tile_of = [&](uint32_t p) { return 2u * (blockIdx.x + (p >> 1) * gridDim.x) + (p & 1u); };
    uint32_t count = 0;  // tiles of the run
    if (blockIdx.x < pairs) {
        const uint32_t mine = (pairs - 1u - blockIdx.x) / gridDim.x + 1u;
        count = 2u * mine - (tile_of(2u * mine - 1u) >= a.tiles ? 1u : 0u);
    }
    // Row 16 tile + l16 of the matrix: the lane's part of the offset never changes, the
    // tile's part is uniform and travels in a scalar register (which the buffer's range
    // check does not see: n is a multiple of sixteen here, every row of a tile exists).
    // Past the workgroup's last tile the loads still run, so that every wait counts the same
    // loads on every path, but fetch the matrix's first tile again (from cache; unused).
    struct Tile {
        su32x4 b[Q8 ? KC / 2 : KC];  // the lane's weights as stored
        su32x2 d;                    // Q8_0: the f16 scales of the wave's KC blocks of the lane's row
    };
    const uint32_t wlane = l16 * a.row_bytes + (Q8 ? kw + 16u * g : 2u * (kw + 8u * g));
    const uint32_t dlane = l16 * a.row_bytes + a.k + 2u * KC * wave, tile_bytes = 16u * a.row_bytes;
    auto load_tile = [&](uint32_t p, Tile &t) __attribute__((always_inline)) {
        const uint32_t base = (p < count ? tile_of(p) : 0u) * tile_bytes;
#pragma unroll
        for (int c = 0; c < (Q8 ? KC / 2 : KC); c++) t.b[c] = __builtin_amdgcn_raw_buffer_load_b128(wbuf, wlane + 64u * c, base, 0);
        if (Q8) {
            if (KC == 4) t.d = __builtin_amdgcn_raw_buffer_load_b64(wbuf, dlane, base, 0);
            else t.d.x = __builtin_amdgcn_raw_buffer_load_b32(wbuf, dlane, base, 0);
        }
    };
    // Chunk c of a tile as a matrix-core operand: BF16 as stored; Q8_0 as bf16(q * d), one
    // rounding of the exact f32 product, d the scale of the block the lane's weights lie in.
    auto operand = [&](const Tile &t, int c) __attribute__((always_inline)) -> sbf16x8 {
        if (!Q8) return __builtin_bit_cast(sbf16x8, t.b[c]);
        const uint32_t block = 2u * (c >> 1) + (g >> 1);  // of the wave's KC
        const uint32_t word = block < 2u ? t.d.x : t.d.y;
        const float d = half_bits_to_float((block & 1u) ? word >> 16 : word & 0xffffu);
        const int32_t lo = (int32_t)((c & 1) ? t.b[c >> 1].z : t.b[c >> 1].x), hi = (int32_t)((c & 1) ? t.b[c >> 1].w : t.b[c >> 1].y);
        const su32x4 v = {
            pack_bf16((float)(int8_t)(lo) * d, (float)(int8_t)(lo >> 8) * d),
            pack_bf16((float)(int8_t)(lo >> 16) * d, (float)(lo >> 24) * d),
            pack_bf16((float)(int8_t)(hi) * d, (float)(int8_t)(hi >> 8) * d),
            pack_bf16((float)(int8_t)(hi >> 16) * d, (float)(hi >> 24) * d)};
        return __builtin_bit_cast(sbf16x8, v);
    };
    // Tile q of the run: its matrix-core instructions, with the reads of tile q - 1's eight
    // partial vectors in between (the matrix cores work while LDS answers), then the sum and
    // store of tile q - 1, then this tile's partial sums into LDS buffer q % 2 and the
    // barrier that publishes them. Buffer (q - 1) % 2 is written again in step q + 1, after
    // that barrier, which every wave passes only when it has read what it needs.
    static_assert(MT <= (int)WAVES, "one partial vector is read per token tile's instructions");
    sf32x4 held = {0.f, 0.f, 0.f, 0.f};
    auto step = [&](uint32_t q, const Tile &t) __attribute__((always_inline)) {
        sbf16x8 wf[KC];
#pragma unroll
        for (int c = 0; c < KC; c++) wf[c] = operand(t, c);
        // (the four vectors of a token are stored permuted, see below)
        const uint8_t *prev = lds + ((q & 1u) ^ 1u) * (WAVES * PART) + ((tid & (MT * 64u - 1u)) ^ ((tid >> 4) & 3u)) * 16u;
        constexpr int PER = WAVES / MT;  // partial vectors read per token tile's instructions
        // acc[i][r]: matrix row 16 tile + 4 g + r, token 16 i + l16: vector (i, token, g), stored
        // at g ^ (token / 4) within the token's four so that the lanes of one lane group, whose
        // vectors lie 64 bytes apart, fall into sixteen different bank groups. A token tile's
        // sums leave for LDS while the next one's instructions run: two accumulators suffice.
        uint8_t *mine = lds + (q & 1u) * (WAVES * PART) + wave * PART + (l16 * 4u + (g ^ (l16 >> 2))) * 16u;
        sf32x4 acc[2], got[PER], sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < MT; i++) {
            acc[i & 1] = sf32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < KC; c++) acc[i & 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[c], xf[i][c], acc[i & 1], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            if (i > 0) {
                *reinterpret_cast<sf32x4 *>(mine + (i - 1) * 1024u) = acc[(i - 1) & 1];
                // The vectors read a group of instructions ago are added, in the order of the k ranges.
#pragma unroll
                for (int e = 0; e < PER; e++) sum = (i == 1 && e == 0) ? got[0] : sum + got[e];
            }
#pragma unroll
            for (int e = 0; e < PER; e++) got[e] = *reinterpret_cast<const sf32x4 *>(prev + (i * PER + e) * PART);
            __builtin_amdgcn_sched_barrier(0);
        }
        *reinterpret_cast<sf32x4 *>(mine + (MT - 1) * 1024u) = acc[(MT - 1) & 1];
#pragma unroll
        for (int e = 0; e < PER; e++) sum = (MT == 1 && e == 0) ? got[0] : sum + got[e];
        if (q > 0u && tid < MT * 64u) {
            // Vector tid of tile p = q - 1 of the run: token tile tid / 64 (this wave's lanes
            // hold all of it), token lane / 4, outputs 4 (lane % 4) .. + 3 of the tile's 16.
            const uint32_t p = q - 1u, ttile = 16u * (tid >> 6);
            if (!(p & 1u) && p + 1u < count) {
                held = sum;  // waits for its neighbour: a pair fills whole 128-byte lines
            } else if (p & 1u) {
                // Two stores of eight tokens: lanes 8 u .. 8 u + 7 write token u's 32 outputs.
#pragma unroll
                for (uint32_t half8 = 0; half8 < 2; half8++) {
                    const uint32_t tt = 8u * half8 + (lane >> 3), from = 4u * (4u * tt + (lane & 3u));
                    // Both gathers run in every lane (a lane's source may sit in the other half).
                    const sf32x4 first = from_lane(held, from), second = from_lane(sum, from);
                    const sf32x4 v = (lane & 4u) ? second : first;
                    const uint32_t t = ttile + tt, j = 16u * tile_of(p - 1u) + 4u * (lane & 7u);
                    if (t < a.rows) {
                        sf32x4 *o = reinterpret_cast<sf32x4 *>(a.out + (size_t)t * a.out_stride + a.col0 + j);
                        store_apart(o, a.accumulate ? v + *o : v);
                    }
                }
            } else {
                const uint32_t t = ttile + (lane >> 2), j = 16u * tile_of(p) + 4u * (lane & 3u);
                if (t < a.rows) {
                    sf32x4 *o = reinterpret_cast<sf32x4 *>(a.out + (size_t)t * a.out_stride + a.col0 + j);
                    if (a.accumulate) sum += *o;
                    store_apart(o, sum);
                }
            }
        }
        lds_barrier();
    };

    // DEPTH register sets in rotation: DEPTH - 1 tiles in flight behind the one multiplied.
    // Every wave of the workgroup runs the same steps (the barrier inside); one step past
    // the last tile sums and stores that tile (its own instructions multiply stale registers
    // into partial sums nobody reads).
    Tile b[DEPTH];
#pragma unroll
    for (int s = 0; s < DEPTH - 1; s++) load_tile(s, b[s]);
    const uint32_t rounds = count ? count + 1u : 0u;
    for (uint32_t r = 0; r < rounds; r += DEPTH) {
#pragma unroll
        for (int s = 0; s < DEPTH; s++) {
            load_tile(r + s + (DEPTH - 1), b[(s + DEPTH - 1) % DEPTH]);
            if (r + s < rounds) step(r + s, b[s]);
        }
    }
}

template <int MT>
constexpr int stream_lds_bytes() { return 2 * WAVES * MT * 64 * 16; }

template <int MT, int KC, bool Q8>
static zhip_result launch(const Dispatch &d, const char *name, const StreamArgs &a, uint32_t groups) {
    auto kernel = matmul_stream_kernel<MT, KC, Q8>;
    constexpr int bytes = stream_lds_bytes<MT>();
    if (!lds_opt_in<matmul_stream_kernel<MT, KC, Q8>, bytes>()) return fail(d, ZHIP_E_GPU, "%s: cannot reserve %d bytes of LDS", name, bytes);
    hipLaunchKernelGGL(kernel, dim3(groups), dim3(THREADS), bytes, d.stream, a);
    return check_launch(d, name);
}

template <int MT>
static zhip_result launch_k(const Dispatch &d, const char *name, const StreamArgs &a, uint32_t groups, bool q8_0) {
    if (q8_0) return a.k == 512u ? launch<MT, 2, true>(d, name, a, groups) : launch<MT, 4, true>(d, name, a, groups);
    switch (a.k / 256u) {
    case 1: return launch<MT, 1, false>(d, name, a, groups);
    case 2: return launch<MT, 2, false>(d, name, a, groups);
    case 3: return launch<MT, 3, false>(d, name, a, groups);
    default: return launch<MT, 4, false>(d, name, a, groups);
    }
}

}  // namespace

bool matmul_stream_prepare_no_alloc() {
    return lds_opt_in<matmul_stream_kernel<4, 2, true>, stream_lds_bytes<4>()>() && lds_opt_in<matmul_stream_kernel<4, 4, true>, stream_lds_bytes<4>()>() &&
           lds_opt_in<matmul_stream_kernel<8, 2, true>, stream_lds_bytes<8>()>() && lds_opt_in<matmul_stream_kernel<8, 4, true>, stream_lds_bytes<8>()>();
}

// Whether the streaming kernel suits a (validated) step on the bf16 rung: few tokens, a
// short k in whole chunks (Q8_0: two or four blocks a wave), enough whole weight tiles to
// occupy every CU several times, and outputs that can be stored 16 bytes at a time.
bool matmul_stream_accepts(const Dispatch &d, bool q8_0, const float *out, uint32_t rows, uint32_t n, uint32_t k, uint32_t col0, uint32_t out_stride) {
    const bool k_fits = q8_0 ? (k == 512u || k == 1024u) : (k >= 256u && k <= 1024u && k % 256u == 0);
    return rows >= 1 && k_fits && (n + 15u) / 16u >= 4u * (uint32_t)d.dev->compute_units &&
           (uintptr_t)out % 16u == 0 && out_stride % 4u == 0 && col0 % 4u == 0 && n % 16u == 0;
}

zhip_result launch_matmul_stream(const Dispatch &d, const char *name, bool q8_0, const uint8_t *x, const uint8_t *w, float *out,
    uint32_t rows, uint32_t n, uint32_t k, uint32_t col0, uint32_t out_stride, uint32_t accumulate, uint32_t row_bytes) {
    const uint64_t w_bytes = (uint64_t)n * row_bytes;
    // 32-bit byte offsets, up to a tile of sixteen past the last token and row.
    if (w_bytes + 16ull * row_bytes >= 0xfffffff0ull - 256u) return fail(d, ZHIP_E_BAD_COMMAND, "%s: operands of 4 GiB or more", name);
    // A chunk of up to 128 tokens a launch, each a pass over the weights: which kernel a matrix
    // takes must not depend on the step's length (a token's bits are the same however a prompt
    // is split into steps, src/sched/sched.zig:84-90), so longer steps stay here as well.
    for (uint32_t t0 = 0; t0 < rows; t0 += 128u) {
        const uint32_t chunk = rows - t0 < 128u ? rows - t0 : 128u;
        StreamArgs a{};
        a.x = x + (size_t)t0 * k * 2u; a.w = w; a.out = out + (size_t)t0 * out_stride;
        a.rows = chunk; a.n = n; a.k = k; a.col0 = col0; a.out_stride = out_stride; a.accumulate = accumulate;
        a.x_bytes = (uint32_t)((uint64_t)chunk * k * 2u); a.w_bytes = (uint32_t)w_bytes; a.row_bytes = row_bytes;
        a.tiles = (n + 15u) / 16u;
        const uint32_t groups = a.tiles < (uint32_t)d.dev->compute_units ? a.tiles : (uint32_t)d.dev->compute_units;
        if (zhip_result r = chunk <= 64u ? launch_k<4>(d, name, a, groups, q8_0) : launch_k<8>(d, name, a, groups, q8_0)) return r;
    }
    return ZHIP_OK;
}

}  // namespace zhip
