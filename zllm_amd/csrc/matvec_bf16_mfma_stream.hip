// matvec_bf16 (and matvec_f16) on the matrix cores for steps of several tokens and k = 1024 ... 4096 in steps of
// 512: the weight stream is read once for all tokens of the step and nothing but partial sums
// crosses LDS. Contract of src/kernels/matvec_half.wgsl:1-133 with the bf16 decoder of
// src/kernels/half/bf16.wgsl:3-9: out[t][col0 + j] (+)= sum_i x[t][i] * w[j][i], the inputs
// taken as the f32 values they are. (The reference gives every token a row of workgroups of its
// own, so a step of M tokens reads the weights M times.)
//
// Arithmetic. v_mfma_f32_32x32x16_bf16 multiplies 32 rows of inputs by 32 weight rows over
// sixteen positions. The weights are bf16 already and reach the instruction as loaded. An f32
// input is the exact sum of three bf16 values (its upper sixteen bits, the upper sixteen bits of
// what that left, and the rest: eight significant bits each), so a token enters as three operand
// rows, every product is exact in the f32 accumulator, and the three rows' sums are added at the
// end. Eight tokens fill 24 of the 32 operand rows; the other eight are zeros. A token's rows
// meet no other token's anywhere: its results do not depend on how many tokens share the launch
// (steps of more than eight tokens run as launches of eight).
//
// Layout of the work. A 512-thread workgroup is eight waves that split k eight ways; a wave
// builds its k range of all tokens' operand rows once, into registers (k / 32 VGPRs). Persistent
// workgroups take 32-row weight tiles b, b + G, ... and at the end a share of the rows left
// over, in units of eight rows, so that every workgroup reads the same number of bytes within
// one unit. A wave's part of a tile is k / 512 pieces, a piece one 128-byte line (64 positions)
// of each of the 32 rows; pieces arrive in a private ring of 4 KB LDS slots by wave-wide direct
// loads of whole lines (lane l of load j brings 16 bytes of row 8 j + l / 8), two pieces
// ahead of the one multiplied, and each lane reads its row's sixteen bytes of a sixteen-position
// step back for one matrix instruction. (The matrix instruction wants lane l to hold row l % 32:
// a lane loading its own bytes would make every lane of a load touch another cache line, and the
// vector memory unit moves sixteen bytes per line it looks up.) Chunk c (16 bytes) of row r sits
// at position c ^ (r / 2 % 8) of the row's line in the slot: two neighbouring lines fill the 64
// banks once, and sixteen rows' reads of one chunk fall in sixteen different groups of four. The eight waves' partial sums meet in LDS, where
// 256 threads add the eight for one output each in the order of the k ranges; the outputs wait
// in LDS and are stored when the workgroup's run ends (or every 40 tiles), 128 contiguous bytes
// a token and tile. One barrier a tile; no barrier waits for the loads in flight.
#include <hip/hip_runtime.h>

#include <type_traits>

#include "common.h"
#include "decode.h"
#include "matvec_common.h"

namespace zhip {

namespace {

typedef __bf16 hbf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 hf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 hf16x4 __attribute__((ext_vector_type(4)));
typedef float hf32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t hu32x4 __attribute__((ext_vector_type(4)));

constexpr uint32_t THREADS = 512, WAVES = 8;
constexpr int DEPTH = 3;  // ring slots a wave: two pieces in flight behind the one multiplied (four measured no faster)
constexpr int LOADS = 4;  // wave-wide loads a piece: eight rows each
constexpr uint32_t SLOT = 32u * 128u;
constexpr uint32_t PART_BYTES = 2u * WAVES * 256u * 4u;  // [tile parity][wave][token of the lane's four][lane]
constexpr uint32_t KEPT = 40;                            // tiles whose outputs wait in LDS for one burst of stores
constexpr uint32_t RING_BYTES = WAVES * DEPTH * SLOT;
constexpr uint32_t LDS_BYTES = PART_BYTES + RING_BYTES + KEPT * 1024u + 64u;  // (the last 64: f16 tokens' inverse scales)
static_assert(LDS_BYTES <= 160u * 1024u - 64u, "the rings must fit the CU's LDS");

struct StreamArgs {
    MvArgs a;
    uint32_t w_bytes;    // bytes of the weights the loads may touch (they are range-checked)
    uint32_t rounds;     // 32-row tiles every workgroup takes: tiles b, b + G, ...
    uint32_t tail_base;  // units of eight rows after those: tail_base for every workgroup
    uint32_t tail_rem;   // and one more for each of the first tail_rem
    uint32_t by_die;     // workgroups renumbered die by die (the grid is a multiple of eight)
    // Inputs split beforehand (SPLIT kernels): three planes [piece][token][k] of bf16.
    const uint8_t *planes;
    uint32_t plane_tokens;  // tokens a plane holds
    uint32_t plane_k;       // positions of a token in a plane (the whole row's, of which the launch may take a stretch)
    uint32_t plane_first;   // the launch's first position
    uint32_t t0;            // the launch's first token in the planes
    const float *inverse;   // F16 kernels: one over each token's scale
    // Rows of more than 4096 weights in equal stretches of columns (LONG kernels): `parts`
    // workgroups share a tile, a stretch each, and leave their sums in `partial`
    // ([part][token of 8][output], outputs a.rows apart).
    uint32_t parts;
    float *partial;
};

// A barrier that waits for this wave's LDS traffic only: the weight loads of the pieces ahead
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

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_buffer(const void *base, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, 0x00020000);
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

// The bits of one of the three pieces of x (the one whose mask is all ones; the others' are
// zero) as an f32 whose lower half is zero: x is the exact sum of the three. Infinities and NaNs stay what they are in the first piece; the others are zero.
__device__ __forceinline__ uint32_t piece_bits(float x, uint32_t m0, uint32_t m1, uint32_t m2) {
    const uint32_t b = __float_as_uint(x);
    const bool finite = (b & 0x7f800000u) != 0x7f800000u;
    // (selects, not branches: a NaN whose payload sits in the lower half would otherwise be cut to an infinity)
    const uint32_t p0 = (b & 0xffff0000u) | ((!finite & ((b & 0x007fffffu) != 0u)) ? 0x00400000u : 0u);
    const float d1 = x - __uint_as_float(p0);
    const float r1 = finite ? d1 : 0.f;
    const uint32_t p1 = __float_as_uint(r1) & 0xffff0000u;
    const float r2 = r1 - __uint_as_float(p1);
    return (p0 & m0) | (p1 & m1) | (__float_as_uint(r2) & m2);
}

// The upper halves of two words as a pair of bf16 values, `lo` first.
__device__ __forceinline__ uint32_t upper_halves(uint32_t lo, uint32_t hi) { return __builtin_amdgcn_perm(hi, lo, 0x07060302u); }

// NP: pieces of a wave's k range (k = 512 NP). SPLIT: the tokens' three pieces come ready from
// matvec_bf16_split_kernel's planes. A workgroup that splits its tokens itself spends 12 vector
// operations a value on it, four lanes on the same value (the lanes of the three pieces and of
// the zero rows): 1.5 us of a launch at k = 1024, less than another launch costs, but 12 us at
// k = 4096.
// F16 (matvec_f16: the weights are f16 and the matrix instruction v_mfma_f32_32x32x16_f16): a
// token enters as two f16 rows, the rounding of its inputs and the rounding of what that left
// times 2^11, after a power of two has put its largest magnitude at 2^14 (an input keeps 22
// bits); the planes come from matvec_f16_split_kernel, and a token's sums are multiplied by one
// over its scale.
// LONG: k = 512 NP q.parts; workgroup i multiplies stretch i % parts (`kpart`) of the tiles that
// walker i / parts takes, and launch_matvec_parts_sum adds the stretches' sums.
template <int NP, bool SPLIT, bool F16, bool LONG>
__global__ __launch_bounds__(THREADS) void matvec_bf16_mfma_stream_kernel(StreamArgs q) {
    static_assert(SPLIT || !F16, "f16 tokens are always split beforehand");
    static_assert(SPLIT || !LONG, "the stretches of a long row read the tokens from the planes");
    constexpr uint32_t PIECES = F16 ? 2u : 3u;
    const MvArgs &a = q.a;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    float *lds_part = reinterpret_cast<float *>(lds);
    float *lds_kept = reinterpret_cast<float *>(lds + PART_BYTES + RING_BYTES);  // [tile % KEPT][token][row]
    float *lds_inverse = lds_kept + KEPT * 256u;                                 // [token], read behind the tiles' barriers
    if (F16 && threadIdx.x < 8u) lds_inverse[threadIdx.x] = threadIdx.x < a.m ? q.inverse[q.t0 + threadIdx.x] : 1.0f;
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    uint8_t *ring = lds + PART_BYTES + wave * (DEPTH * SLOT);
    const uint32_t ring0 = (uint32_t)(uintptr_t)ring;
    const __amdgpu_buffer_rsrc_t wbuf = make_buffer(a.w, q.w_bytes), nobuf = make_buffer(a.w, 0);

    // The workgroup's tiles: b, b + G, ... and its share of the rows after the whole rounds. The
    // hardware deals workgroups out to the chip's eight dies in turn; b numbers them so that a
    // die's workgroups take neighbouring tiles (one die then reads a contiguous eighth of every
    // round's stretch of the matrix: 55 us against 58 us for four tokens over 151936 x 1024).
    const uint32_t kpart = LONG ? blockIdx.x % q.parts : 0u, walker = LONG ? blockIdx.x / q.parts : blockIdx.x;
    const uint32_t G = LONG ? gridDim.x / q.parts : gridDim.x;
    const uint32_t b = q.by_die ? (walker & 7u) * (G >> 3) + (walker >> 3) : walker;
    const uint32_t tail_units = q.tail_base + (b < q.tail_rem ? 1u : 0u);
    const uint32_t tail_row = 32u * q.rounds * G + 8u * (b * q.tail_base + (b < q.tail_rem ? b : q.tail_rem));
    const uint32_t count = q.rounds + (tail_units ? 1u : 0u);
    auto first_row = [&](uint32_t p) { return p < q.rounds ? 32u * (b + p * G) : tail_row; };
    auto rows_of = [&](uint32_t p) { return p < q.rounds ? 32u : 8u * tail_units; };

    // A piece's loads: load j brings rows 8 j .. 8 j + 7, lane l row 8 j + l / 8 and the chunk
    // that belongs at position l % 8 of its line. The whole address is the lane's offset, which
    // is what the buffer's range check sees: rows past the matrix's end land as zeros.
    auto line_key = [](uint32_t row) { return (row >> 1) & 7u; };
    uint32_t woff[LOADS];
#pragma unroll
    for (int j = 0; j < LOADS; j++) woff[j] = (8u * j + (lane >> 3)) * a.row_bytes + 1024u * NP * kpart + 128u * NP * wave + 16u * ((lane & 7u) ^ line_key(8u * j + (lane >> 3)));
    uint32_t load_tile = 0, load_piece = 0, load_slot = 0;
    auto issue = [&]() __attribute__((always_inline)) {
        // (past the run's last piece the loads still run, so that the waits count the same loads
        // every step, but against an empty buffer: zeros land and nothing is fetched; the same
        // for the rows a share of the last rows does not have)
        const __amdgpu_buffer_rsrc_t buf = load_tile < count ? wbuf : nobuf;
        const uint32_t base = first_row(load_tile) * a.row_bytes + 128u * load_piece, rows = rows_of(load_tile);
        const uint32_t dst = ring0 + load_slot * SLOT;
#pragma unroll
        for (int j = 0; j < LOADS; j++) load_lds_b128(8u * j < rows ? buf : nobuf, dst + 1024u * j, woff[j] + base);
        load_piece = load_piece + 1u == (uint32_t)NP ? 0u : load_piece + 1u;
        load_tile += load_piece == 0u ? 1u : 0u;
        load_slot = (load_slot + 1u) % DEPTH;
    };

    // The tokens' inputs first: loads complete in order within a wave, and behind the weight
    // loads the first use of an input would wait for a round trip of the weight stream. Operand
    // row r of the matrix instruction is piece r / 8 of token 4 (r / 4 % 2) + r % 4 (rows 24 .. 31
    // are zeros), so that a lane's sixteen results are its weight row times the three pieces of
    // four tokens; the lane's eight positions of step s are 16 s + 8 (lane / 32) ... An absent
    // token's rows read the last token's inputs and come out as zeros: no branches, so all of the
    // lane's loads go out together.
    const uint32_t rho = lane & 31u, kap = lane >> 5;
    const uint32_t tok = 4u * ((rho >> 2) & 1u) + (rho & 3u), piece = rho >> 3;
    const bool live = tok < a.m && piece < PIECES;
    // (masks, so that picking the lane's piece is two instructions a value and not a branch)
    uint32_t m0 = live && piece == 0u ? ~0u : 0u, m1 = live && piece == 1u ? ~0u : 0u, m2 = live && piece == 2u ? ~0u : 0u;
    asm volatile("" : "+v"(m0), "+v"(m1), "+v"(m2));
    const float *xt = a.x + (size_t)(tok < a.m ? tok : a.m - 1u) * a.xr + 64u * NP * wave + 8u * kap;
    hu32x4 xf[4 * NP];
    if constexpr (SPLIT) {
        // Every step's operand is sixteen bytes of a plane; the lanes of absent tokens and of
        // the zero rows ask past the buffer's end and get zeros.
        const __amdgpu_buffer_rsrc_t pbuf = make_buffer(q.planes, PIECES * q.plane_tokens * q.plane_k * 2u);
        const uint32_t at = live ? ((piece * q.plane_tokens + q.t0 + tok) * q.plane_k + q.plane_first + 512u * NP * kpart + 64u * NP * wave + 8u * kap) * 2u : 0xfffffff0u;
#pragma unroll
        for (int s = 0; s < 4 * NP; s++) xf[s] = __builtin_bit_cast(hu32x4, __builtin_amdgcn_raw_buffer_load_b128(pbuf, live ? at + 32u * s : at, 0, 0));
        issue();
    } else
#pragma unroll
    for (int s0 = 0; s0 < 4 * NP; s0 += 8) {
        float4 raw[16];
#pragma unroll
        for (int s = 0; s < 8 && s0 + s < 4 * NP; s++) {
            raw[2 * s] = *reinterpret_cast<const float4 *>(xt + 16 * (s0 + s));
            raw[2 * s + 1] = *reinterpret_cast<const float4 *>(xt + 16 * (s0 + s) + 4);
        }
        // (One piece of weights behind them for now: with more, the requests of the workgroups
        // that start first fill the memory system's queues and the inputs of the others arrive
        // after them.)
        if (s0 == 0) issue();
#pragma unroll
        for (int s = 0; s < 8 && s0 + s < 4 * NP; s++) {
            const float x[8] = {raw[2 * s].x, raw[2 * s].y, raw[2 * s].z, raw[2 * s].w, raw[2 * s + 1].x, raw[2 * s + 1].y, raw[2 * s + 1].z, raw[2 * s + 1].w};
            hu32x4 words;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                words[e] = upper_halves(piece_bits(x[2 * e], m0, m1, m2), piece_bits(x[2 * e + 1], m0, m1, m2));
            }
            xf[s0 + s] = words;
        }
        // (a batch's loads are not to be requested before the batch before is in its operands:
        // all of them at once would need more registers than a lane has)
        asm volatile("" ::: "memory");
    }
#pragma unroll
    for (int s = 1; s < DEPTH - 1; s++) issue();

    // The lane's reads of a piece: row rho, chunk 2 s + kap of its line for step s.
    uint32_t r_at[4];
#pragma unroll
    for (int s = 0; s < 4; s++) r_at[s] = 128u * rho + 16u * ((2u * s + kap) ^ line_key(rho));

    auto finish = [&](uint32_t p, const hf32x16 &sum) __attribute__((always_inline)) {
        float *part = lds_part + (p & 1u) * (WAVES * 256u);
#pragma unroll
        for (int i = 0; i < 4; i++) part[wave * 256u + 64u * i + lane] = F16 ? fmaf(sum[4 + i], 1.0f / 2048.0f, sum[i]) : (sum[i] + sum[4 + i]) + sum[8 + i];
        lds_barrier();
        // Buffer p % 2 is written again in step p + 2, after the barrier of step p + 1, which a
        // wave passes only when it has read what it needs here. The 256 outputs of a tile are
        // summed by one half of the workgroup, the other half at the next tile.
        if ((tid >> 8) == (p & 1u)) {
            // (a wave sums tokens i and 4 + i, whose partial sums lie side by side: no two lanes on a bank)
            const uint32_t row = tid & 31u, tk = 4u * ((tid >> 5) & 1u) + ((tid >> 6) & 3u);
            const float *src = part + 64u * (tk & 3u) + 32u * (tk >> 2) + row;
            float total = src[0];
#pragma unroll
            for (uint32_t wv = 1; wv < WAVES; wv++) total += src[wv * 256u];
            if (F16) total *= lds_inverse[tk];
            lds_kept[256u * (p % KEPT) + 32u * tk + row] = total;
        }
    };
    // The outputs of tiles first .. first + n - 1, from LDS to memory: 128 contiguous bytes a
    // token and tile. (Stored tile by tile between the loads they took 2 us of a 55 us launch
    // longer than in one burst: every isolated write turns the memory's direction around.)
    auto store_kept = [&](uint32_t first, uint32_t n) __attribute__((always_inline)) {
        lds_barrier();
        for (uint32_t p = first + (tid >> 8); p < first + n; p += 2u) {
            const uint32_t row = tid & 31u, tk = (tid >> 5) & 7u;
            const uint32_t j = first_row(p) + row;
            if (tk < a.m && row < rows_of(p) && j < a.rows) {
                float *o = a.out + (size_t)tk * a.out_stride + a.col0 + j;
                const float total = lds_kept[256u * (p % KEPT) + (tid & 255u)];
                if (LONG) store_apart(q.partial + ((size_t)kpart * 8u + tk) * a.rows + j, total);
                else store_apart(o, (a.flags & FLAG_ACCUMULATE) ? *o + total : total);
            }
        }
    };

    // DEPTH ring slots in rotation. Every wave of the workgroup runs the same steps (the barrier
    // inside). Before a piece is read, all but the loads of the DEPTH - 1 pieces after it have
    // landed.
    uint32_t slot = 0;
    for (uint32_t p = 0; p < count; p++) {
        hf32x16 sum;
#pragma unroll
        for (int e = 0; e < 16; e++) sum[e] = 0.f;
#pragma unroll
        for (int i = 0; i < NP; i++) {
            // The slot refilled now was read by the multiply before: its reads must have returned
            // before the load is issued (a load past the run's end lands at once), and the
            // compiler, which sees no dependency between the two, must not move it up.
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            issue();
            wait_loads<(DEPTH - 1) * LOADS>();
            const uint8_t *t = ring + slot * SLOT;
#pragma unroll
            for (int s = 0; s < 4; s++) {
                const hu32x4 w = *reinterpret_cast<const hu32x4 *>(t + r_at[s]);
                if constexpr (F16) sum = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(hf16x8, xf[4 * i + s]), __builtin_bit_cast(hf16x8, w), sum, 0, 0, 0);
                else sum = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(hbf16x8, xf[4 * i + s]), __builtin_bit_cast(hbf16x8, w), sum, 0, 0, 0);
            }
            // (the piece's matrix instructions belong here, not after the last piece's wait, where
            // the compiler would otherwise collect them with all their operands held in registers)
            asm volatile("" : "+v"(sum));
            slot = (slot + 1u) % DEPTH;
        }
        finish(p, sum);
        // (the next tile's sums are kept only behind its barrier, which no thread passes before
        // it has stored what it stores here)
        if ((p + 1u) % KEPT == 0u || p + 1u == count) store_kept(p - p % KEPT, p % KEPT + 1u);
    }
    wait_loads<0>();  // nothing may still land in LDS once the workgroup is gone
}

// Token blockIdx.x as the multiply sees it (normalised if the step asks for it:
// src/kernels/matvec_half.wgsl:58-80), split into the three planes.
__global__ __launch_bounds__(256) void matvec_bf16_split_kernel(MvArgs a, uint2 *planes) {
    __shared__ float red[4];
    extern __shared__ float4 staged[];  // the token: k / 4 vectors
    stage_token(a, blockIdx.x, staged, red);
    __syncthreads();
    const uint32_t k4 = a.k / 4u;
    for (uint32_t i = threadIdx.x; i < k4; i += 256u) {
        const float4 v = staged[i];
#pragma unroll
        for (uint32_t piece = 0; piece < 3u; piece++) {
            const uint32_t m0 = piece == 0u ? ~0u : 0u, m1 = piece == 1u ? ~0u : 0u, m2 = piece == 2u ? ~0u : 0u;
            uint2 w;
            w.x = upper_halves(piece_bits(v.x, m0, m1, m2), piece_bits(v.y, m0, m1, m2));
            w.y = upper_halves(piece_bits(v.z, m0, m1, m2), piece_bits(v.w, m0, m1, m2));
            planes[(size_t)(piece * gridDim.x + blockIdx.x) * k4 + i] = w;
        }
    }
}

// The same for matvec_f16: the token scaled by the power of two that puts its largest
// magnitude in [2^14, 2^15) and split into its f16 rounding and what that left times 2^11
// (planes [2][tokens][k]), and one over the scale.
__global__ __launch_bounds__(256) void matvec_f16_split_kernel(MvArgs a, uint2 *planes, float *inverse) {
    __shared__ float red[4];
    extern __shared__ float4 staged[];  // the token: k / 4 vectors
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
        planes[(size_t)blockIdx.x * k4 + i] = __builtin_bit_cast(uint2, hf16x4{hi[0], hi[1], hi[2], hi[3]});
        planes[(size_t)(gridDim.x + blockIdx.x) * k4 + i] = __builtin_bit_cast(uint2, hf16x4{lo[0], lo[1], lo[2], lo[3]});
    }
}

template <int NP, bool SPLIT, bool F16, bool LONG = false>
zhip_result launch_blocks(const Dispatch &d, const StreamArgs &q, dim3 grid) {
    auto kernel = matvec_bf16_mfma_stream_kernel<NP, SPLIT, F16, LONG>;
    static bool configured = false;
    if (!configured) {
        if (hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES) != hipSuccess) {
            (void)hipGetLastError();
            return fail(d, ZHIP_E_GPU, "%s: cannot reserve %u bytes of LDS", F16 ? "matvec_f16" : "matvec_bf16", LDS_BYTES);
        }
        configured = true;
    }
    hipLaunchKernelGGL(kernel, grid, dim3(THREADS), LDS_BYTES, d.stream, q);
    return check_launch(d, F16 ? "matvec_f16" : "matvec_bf16");
}

}  // namespace

// Whether this kernel can run the (already validated) arguments: k split into whole lines a
// wave, no pair.
// (rows of more than 4096 weights are taken in stretches of columns: equal ones in one launch, workgroups sharing a
// tile, with a launch for their sums; unequal ones a launch each; up to 16384: the split launch stages a token in 64 KB of LDS)
bool matvec_bf16_mfma_stream_accepts(const MvArgs &a) {
    return a.m >= 1 && a.k >= 1024u && a.k <= 16384u && a.k % 512u == 0 && !(a.flags & FLAG_SILU_PAIR) && a.act_div == 0.f && a.rows >= 1 &&
           a.xr % 4u == 0 && (reinterpret_cast<uintptr_t>(a.x) & 15u) == 0 && (reinterpret_cast<uintptr_t>(a.w) & 15u) == 0 && a.row_bytes == 2u * a.k;
}

template <bool SPLIT, bool F16, bool LONG = false>
static zhip_result launch_for_k(const Dispatch &d, const StreamArgs &q, dim3 grid) {
    switch (q.a.k / 512u) {
    case 2: return launch_blocks<2, SPLIT, F16, LONG>(d, q, grid);
    case 3: return launch_blocks<3, SPLIT, F16, LONG>(d, q, grid);
    case 4: return launch_blocks<4, SPLIT, F16, LONG>(d, q, grid);
    case 5: return launch_blocks<5, SPLIT, F16, LONG>(d, q, grid);
    case 6: return launch_blocks<6, SPLIT, F16, LONG>(d, q, grid);
    case 7: return launch_blocks<7, SPLIT, F16, LONG>(d, q, grid);
    default: return launch_blocks<8, SPLIT, F16, LONG>(d, q, grid);
    }
}

// f16: the weights are f16 (matvec_f16), bf16 otherwise.
zhip_result launch_matvec_bf16_mfma_stream(const Dispatch &d, const MvArgs &a, uint64_t w_bytes, bool f16) {
    const char *name = f16 ? "matvec_f16" : "matvec_bf16";
    // 32-bit byte offsets, a tile past the last row.
    const uint64_t used = (uint64_t)a.rows * a.row_bytes;
    if (used + 64ull * a.row_bytes >= 0xfffffff0ull) return fail(d, ZHIP_E_BAD_COMMAND, "%s: weights of 4 GiB or more", name);
    const uint32_t cus = (uint32_t)d.dev->compute_units;
    const uint32_t units = (a.rows + 7u) / 8u;
    const uint32_t groups = units < cus ? units : cus;
    const uint32_t rounds = (a.rows / 32u) / groups;
    const uint32_t tail = (a.rows - 32u * rounds * groups + 7u) / 8u;
    StreamArgs q{a, (uint32_t)(used < w_bytes ? used : w_bytes), rounds, tail / groups, tail % groups, groups % 8u == 0 ? 1u : 0u, nullptr, 0u, 0u, 0u, 0u, nullptr, 1u, nullptr};
    // The tokens are split (and normalised) by a launch of their own where that is cheaper than
    // every workgroup splitting them again, and wherever the step carries the RMSNorm prologue
    // (the workgroups computing the norm themselves at k = 1024 measured the same: 151936 x 1024
    // at 2 / 4 / 8 tokens 53.3 / 54.1 / 56.3 us against 54.2 / 54.2 / 55.5 us this way). f16
    // tokens, which need their scales first, always.
    const bool split = f16 || (a.flags & FLAG_NORM) || a.k >= 2048u;
    // Rows of more than 4096 weights (the FFN-down shapes; the general kernel takes them token by
    // token) go in stretches of up to 4096 columns. Stretches of equal length (14336 = 4 x 3584,
    // 8192 = 2 x 4096 ...) go out as one launch: `launches` workgroups share a walker's tiles, a
    // stretch each, and a second launch adds the stretches' sums in their order and applies the
    // epilogue (their sums wait in the workspace, behind the tokens' planes).
    const uint32_t pieces = a.k / 512u, launches = (a.k + 4095u) / 4096u;
    const bool together = launches > 1u && pieces % launches == 0u && split && launches <= kMatvecMaxParts && cus >= launches;
    const uint64_t planes_bytes = (((f16 ? 4ull : 6ull) * a.m * a.k + 4ull * a.m + 64u) + 255u) & ~255ull;
    if (split) {
        const uint64_t bytes = (f16 ? 4ull : 6ull) * a.m * a.k;
        if (!d.work) return fail(d, ZHIP_E_GPU, "%s: no workspace", name);
        if (bytes >= 0xfffffff0ull) return fail(d, ZHIP_E_BAD_COMMAND, "%s: a step of %u tokens", name, a.m);
        if (zhip_result r = d.work->reserve(d, planes_bytes + (together ? (uint64_t)launches * 8u * a.rows * sizeof(float) : 0ull))) return r;
        float *inverse = reinterpret_cast<float *>(d.work->data + bytes);
        if (f16) hipLaunchKernelGGL(matvec_f16_split_kernel, dim3(a.m), dim3(256), a.k * 4u, d.stream, a, reinterpret_cast<uint2 *>(d.work->data), inverse);
        else hipLaunchKernelGGL(matvec_bf16_split_kernel, dim3(a.m), dim3(256), a.k * 4u, d.stream, a, reinterpret_cast<uint2 *>(d.work->data));
        if (zhip_result r = check_launch(d, name)) return r;
        q.planes = d.work->data;
        q.plane_tokens = a.m;
        q.plane_k = a.k;
        q.inverse = inverse;
        q.a.flags &= ~FLAG_NORM;
        q.a.norm_w = nullptr;
    }
    const dim3 grid(groups);
    // Stretches of unequal length: each a launch that adds to the one before; the tokens are
    // split once, prologue included, for all of them.
    if (together) {
        const uint32_t most = cus / launches, walkers = units < most ? units : most;
        const uint32_t lrounds = (a.rows / 32u) / walkers, ltail = (a.rows - 32u * lrounds * walkers + 7u) / 8u;
        q.rounds = lrounds; q.tail_base = ltail / walkers; q.tail_rem = ltail % walkers; q.by_die = walkers % 8u == 0 ? 1u : 0u;
        q.parts = launches;
        q.partial = reinterpret_cast<float *>(d.work->data + planes_bytes);
        q.a.k = 512u * (pieces / launches);
        q.plane_first = 0;
        for (uint32_t t0 = 0; t0 < a.m; t0 += 8u) {
            q.a.x = a.x + (size_t)t0 * a.xr;
            q.a.out = a.out + (size_t)t0 * a.out_stride;
            q.a.m = a.m - t0 < 8u ? a.m - t0 : 8u;
            q.a.flags = a.flags & ~FLAG_NORM;
            q.t0 = t0;
            if (zhip_result r = f16 ? launch_for_k<true, true, true>(d, q, dim3(walkers * launches)) : launch_for_k<true, false, true>(d, q, dim3(walkers * launches))) return r;
            MvArgs sum = q.a;
            sum.k = a.k;
            if (zhip_result r = launch_matvec_parts_sum(d, name, sum, q.partial, launches)) return r;
        }
        return ZHIP_OK;
    }
    for (uint32_t t0 = 0; t0 < a.m; t0 += 8u) {
        uint32_t first = 0;
        for (uint32_t c = 0; c < launches; c++) {
            q.a.k = 512u * (pieces / launches + (c < pieces % launches ? 1u : 0u));
            q.a.x = a.x + (size_t)t0 * a.xr + first;
            q.a.w = a.w + 2u * (size_t)first;
            q.w_bytes = (uint32_t)((used < w_bytes ? used : w_bytes) - 2u * (uint64_t)first);
            q.a.out = a.out + (size_t)t0 * a.out_stride;
            q.a.m = a.m - t0 < 8u ? a.m - t0 : 8u;
            q.a.flags = (a.flags & ~FLAG_NORM & ~FLAG_ACCUMULATE) | ((c || (a.flags & FLAG_ACCUMULATE)) ? FLAG_ACCUMULATE : 0u);
            if (!split) q.a.flags = a.flags;
            q.t0 = t0;
            q.plane_first = first;
            if (zhip_result r = f16 ? launch_for_k<true, true>(d, q, grid) : split ? launch_for_k<true, false>(d, q, grid) : launch_for_k<false, false>(d, q, grid)) return r;
            first += q.a.k;
        }
    }
    return ZHIP_OK;
}

}  // namespace zhip
