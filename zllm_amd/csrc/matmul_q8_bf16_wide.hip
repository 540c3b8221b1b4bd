// matmul_q8_0_float on the matrix cores for matrices with enough rows that 128 x 128 tiles fill
// the CUs (same contract as matmul_q8_bf16.hip, whose 128 x 64 tiles serve the narrower ones:
// out[t][col0 + j] (+)= sum_i h(x[t][i]) * h(q[j][i] * d[j][i / 32]), h the rounding to bf16 or
// f16, fp32 accumulate; whole 128-deep k steps).
//
// A 128-deep step of a 128-token x 128-row tile needs 32 KB of activations and 17 KB of weights
// from L2 for twice the multiply-adds of the 128 x 64 tile's 41.5 KB, and the path from L2 into
// a CU's LDS bounds both kernels.
//
// Four producer waves issue every load (straight into LDS, range-checked buffers, three buffers
// filled up to three steps ahead); eight multiplying waves never issue one. Consumer wave w
// multiplies matrix rows 32 (w % 4) .. + 31 by all the tile's tokens over k half w / 4 of every
// step: two Q8_0 blocks of 32 positions, one in each of two register sets, so that the fragments
// of one block are read while the other is multiplied. Lane l holds row l % 32 and positions
// 16 (l / 32) .. + 15 of a block: one 16-byte read of the row's int8 values, converted once
// (q * d rounded to the operand type) for all the tile's tokens, and two 16-byte reads per
// 32-token tile. The two k halves are added through LDS at the end (first half + second half),
// each wave finishing half of the token tiles; a token's sums do not depend on the tokens
// beside it or on the tile height.
#include <hip/hip_runtime.h>

#include <type_traits>

#include "common.h"
#include "matmul_q8_tiles.h"

namespace zhip {

namespace {

using namespace q8tiles;

// TT: 32-token tiles a workgroup covers (4: 128 tokens, 2: 64 tokens). RQ: 32-row tiles of the
// matrix it covers (4: 128 rows, 2: 64 rows), each the work of two multiplying waves.
template <int RQ> constexpr int threads() { return 64 * (2 * RQ + PRODUCERS); }
// One step's weights in LDS: int8 [row][128 B], then per producer [32 rows][4 f16].
template <int RQ> constexpr int wpart_bytes() { return 32 * RQ * 128 + PRODUCERS * 256; }
template <int TT> constexpr int abuf_bytes() { return 2 * 32 * TT * 128; }  // activations of a step: [line][token][128 B]
template <int TT, int RQ> constexpr int buf_bytes() { return abuf_bytes<TT>() + wpart_bytes<RQ>(); }
template <int TT, int RQ> constexpr int lds_bytes() { return 3 * buf_bytes<TT, RQ>(); }
static_assert(lds_bytes<4, 4>() <= 160 * 1024, "three buffers must fit the CU's LDS");
// The exchange of the k halves reuses the buffers: 2 RQ waves x TT / 2 tiles x 4 KB.
static_assert(lds_bytes<2, 2>() >= 4 * 2 * 4096 && lds_bytes<2, 4>() >= 8 * 2 * 4096, "the exchange must fit the buffers");

template <int TT, class H, int RQ>
__global__ __launch_bounds__(threads<RQ>()) void matmul_q8_bf16_wide_kernel(Q8Args a, uint32_t tiles_n) {
    typedef typename H::vec opvec;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    constexpr int BM = 32 * TT, BN = 32 * RQ, CONSUMERS = 2 * RQ, ABUF = abuf_bytes<TT>(), BUF = buf_bytes<TT, RQ>();
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // Workgroup b takes column tile b % tiles_n of token tile b / tiles_n.
    const uint32_t j0 = (blockIdx.x % tiles_n) * BN, t0 = (blockIdx.x / tiles_n) * BM;
    const uint32_t steps = a.k / BK;

    if (wave >= CONSUMERS) {
        // Producers. Producer p loads a quarter of the step's activation lines (block b = p + 4 i:
        // line b / (BM / 8), tokens 8 (b % (BM / 8)) .. + 7), matrix rows 8 RQ p .. + 8 RQ - 1 and, while there are rows left, the scales of rows 32 p .. + 31.
        // 8 neighbouring lanes cover one 128-byte line; the lane at position q of a line asks
        // for chunk q ^ key(row), so that chunk c of a row sits at position c ^ key(row).
        const uint32_t p = wave - CONSUMERS;
        const __amdgpu_buffer_rsrc_t xbuf = make_buffer(a.x, a.x_bytes), wbuf = make_buffer(a.w, a.w_bytes);
        constexpr int XL = 2 * TT;  // activation loads a producer issues per step
        uint32_t xoff[XL], xdst[XL], woff[RQ];
#pragma unroll
        for (int i = 0; i < XL; i++) {
            const uint32_t b = p + 4u * i, line = b / (BM / 8), row = 8u * (b % (BM / 8)) + (lane >> 3);
            xoff[i] = (t0 + row) * a.k * 2u + 128u * line + 16u * ((lane & 7u) ^ line_key(row));
            xdst[i] = line * (BM * 128) + 1024u * (b % (BM / 8));
        }
#pragma unroll
        for (int i = 0; i < RQ; i++) {
            const uint32_t row = 8u * (RQ * p + i) + (lane >> 3);
            woff[i] = (j0 + row) * a.row_bytes + 16u * ((lane & 7u) ^ line_key(row));
        }
        // A step's scales of the producer's 32 rows, 8 bytes a row, 4 a lane.
        const uint32_t soff = 32u * p < (uint32_t)BN ? (j0 + 32u * p + (lane >> 1)) * a.row_bytes + a.k + 4u * (lane & 1u) : kNowhere;
        // Steps past the end of k are loaded like the others, so that every wait counts the same
        // loads, but from an offset no binding reaches (they land as zeros and move nothing;
        // nothing reads them): the step's position travels in the loads' scalar offset, and
        // whether the range check of a raw buffer covers that offset is not relied on.
        auto fetch = [&](uint32_t buf, uint32_t step) __attribute__((always_inline)) {
            uint8_t *base = lds + buf * BUF;
            if (step < steps) {
#pragma unroll
                for (int i = 0; i < XL; i++) load_lds_b128(xbuf, base + xdst[i], xoff[i], 256u * step);
#pragma unroll
                for (int i = 0; i < RQ; i++) load_lds_b128(wbuf, base + ABUF + 1024u * (RQ * p + i), woff[i], 128u * step);
                load_lds_b32(wbuf, base + ABUF + BN * 128 + 256u * p, soff, 8u * step);
            } else {
#pragma unroll
                for (int i = 0; i < XL; i++) load_lds_b128(xbuf, base + xdst[i], kNowhere, 0u);
#pragma unroll
                for (int i = 0; i < RQ; i++) load_lds_b128(wbuf, base + ABUF + 1024u * (RQ * p + i), kNowhere, 0u);
                load_lds_b32(wbuf, base + ABUF + BN * 128 + 256u * p, kNowhere, 0u);
            }
        };
        constexpr int PER_STEP = XL + RQ + 1;
        fetch(0, 0);
        fetch(1, 1);
        fetch(2, 2);
        sync_keeping_loads<2 * PER_STEP>();  // step 0 has landed
        uint32_t buf = 0;
        for (uint32_t s = 0; s < steps; s++) {
            sync_keeping_loads<PER_STEP>();  // step s + 1 has landed; buffer s % 3 has been read
            fetch(buf, s + 3u);
            buf = buf == 2u ? 0u : buf + 1u;
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // nothing may still land in LDS during the exchange
        __builtin_amdgcn_s_barrier();  // the loop's end
        __builtin_amdgcn_s_barrier();  // the exchange
        return;
    }

    const uint32_t lrow = lane & 31u, h = lane >> 5, rq = wave % RQ, kh = wave / RQ;
    f32x16 acc[TT];
#pragma unroll
    for (int i = 0; i < TT; i++)
#pragma unroll
        for (int e = 0; e < 16; e++) acc[i][e] = 0.f;

    // Fragment addresses for the two Q8_0 blocks (32 positions) of the wave's half of a step.
    // Weights: row 32 rq + lrow, chunk 2 (2 kh + b) + h of its line. Tokens: row 32 tt + lrow of
    // line kh, chunks 4 b + 2 h and the next.
    const uint32_t key = line_key(lrow);
    const uint32_t wr = 32u * rq + lrow;
    uint32_t w_at[2], s_at[2], a_at[2][2];
#pragma unroll
    for (uint32_t b = 0; b < 2; b++) {
        const uint32_t q = 2u * kh + b;
        w_at[b] = ABUF + wr * 128u + 16u * ((2u * q + h) ^ key);
        s_at[b] = ABUF + BN * 128 + 256u * rq + 8u * lrow + 2u * q;
        a_at[b][0] = kh * (BM * 128) + lrow * 128u + 16u * ((4u * b + 2u * h) ^ key);
        a_at[b][1] = kh * (BM * 128) + lrow * 128u + 16u * ((4u * b + 2u * h + 1u) ^ key);
    }

    opvec tok[2][TT][2], wop[2][2];
    // Reads block B of the step in buffer `buf` into register set B.
    auto read_frags = [&](uint32_t buf, auto block, WRaw &raw) __attribute__((always_inline)) {
        constexpr int B = decltype(block)::value;
        const uint8_t *base = lds + buf * BUF;
        raw.q = *reinterpret_cast<const u32x4 *>(base + w_at[B]);
        raw.d = *reinterpret_cast<const uint16_t *>(base + s_at[B]);
#pragma unroll
        for (int tt = 0; tt < TT; tt++) {
            tok[B][tt][0] = *reinterpret_cast<const opvec *>(base + a_at[B][0] + 4096 * tt);
            tok[B][tt][1] = *reinterpret_cast<const opvec *>(base + a_at[B][1] + 4096 * tt);
        }
    };
    auto multiply = [&](auto set) __attribute__((always_inline)) {
        constexpr int S = decltype(set)::value;
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int tt = 0; tt < TT; tt++) acc[tt] = H::mfma(wop[S][j], tok[S][tt][j], acc[tt]);
    };
    typedef std::integral_constant<int, 0> Zero;
    typedef std::integral_constant<int, 1> One;

    sync_after_reads();  // step 0 has landed
    {
        WRaw raw;
        read_frags(0, Zero{}, raw);
        convert<H>(raw, wop[0][0], wop[0][1]);
    }

    // Half a step multiplies the block in one register set and reads the next block into the
    // other: the weights and their scale first, then one token fragment and a share of the
    // conversion after each MFMA.
    auto half = [&](auto cur, uint32_t from) __attribute__((always_inline)) {
        constexpr int S = decltype(cur)::value;
        WRaw raw;
        read_frags(from, std::integral_constant<int, 1 - S>{}, raw);
        multiply(cur);
        convert<H>(raw, wop[1 - S][0], wop[1 - S][1]);
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
#pragma unroll
        for (int i = 0; i < 2 * TT; i++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x002, TT == 4 ? 6 : 11, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    // Step s: block 0 is multiplied while block 1 is read from the same buffer, s % 3; behind
    // the step's barrier (step s + 1 has landed, the producers refill buffer s % 3 with step
    // s + 3) block 1 is multiplied while block 0 of step s + 1 is read.
    auto step = [&](auto cur_buf) __attribute__((always_inline)) {
        constexpr int CB = decltype(cur_buf)::value;
        half(Zero{}, CB);
        sync_after_reads();
        half(One{}, (CB + 1) % 3);
    };
    uint32_t s = 0;
    for (; s + 3u <= steps; s += 3u) {
        step(std::integral_constant<int, 0>{});
        step(std::integral_constant<int, 1>{});
        step(std::integral_constant<int, 2>{});
    }
    if (s < steps) { step(std::integral_constant<int, 0>{}); s++; }
    if (s < steps) { step(std::integral_constant<int, 1>{}); s++; }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();  // the loop's end: the producers have no load in flight
    asm volatile("" ::: "memory");

    // The two k halves of a tile meet in LDS: the wave of half kh keeps token tiles
    // kh TT / 2 .. + TT / 2 - 1 and hands the others to the wave of the other half.
    f32x4 *inbox = reinterpret_cast<f32x4 *>(lds);
    constexpr int KEEP = TT / 2;
    auto slot = [&](uint32_t owner_kh, int i, int p) { return (((owner_kh * RQ + rq) * KEEP + i) * 4u + p) * 64u + lane; };
#pragma unroll
    for (int i = 0; i < KEEP; i++)
#pragma unroll
        for (int p = 0; p < 4; p++) {
            // the other half's tiles: (1 - kh) KEEP + i
            f32x4 v;
#pragma unroll
            for (int r = 0; r < 4; r++) v[r] = kh ? acc[i][4 * p + r] : acc[KEEP + i][4 * p + r];
            inbox[slot(1u - kh, i, p)] = v;
        }
    sync_after_reads();  // the exchange

    const bool adds = a.accumulate != 0u;
    const bool aligned = ((a.out_stride | a.col0) & 3u) == 0u && (reinterpret_cast<uintptr_t>(a.out) & 15u) == 0u;
    // D[row][token] (the weights are the MFMA's first operand): in each 32 x 32 tile the lane
    // holds rows 8 p + 4 (lane / 32) .. + 3, p < 4, of token lane % 32: sixteen contiguous bytes
    // of the token's row per group.
#pragma unroll
    for (int i = 0; i < KEEP; i++) {
        const uint32_t t = t0 + 32u * (kh * KEEP + i) + lrow;
#pragma unroll
        for (int p = 0; p < 4; p++) {
            f32x4 mine;
#pragma unroll
            for (int r = 0; r < 4; r++) mine[r] = kh ? acc[KEEP + i][4 * p + r] : acc[i][4 * p + r];
            const f32x4 theirs = inbox[slot(kh, i, p)];
            f32x4 v = kh ? theirs + mine : mine + theirs;  // first half + second half
            const uint32_t col = j0 + 32u * rq + 8u * p + 4u * h;
            if (t >= a.rows || col >= a.n) continue;
            float *o = a.out + (size_t)t * a.out_stride + a.col0 + col;
            if (aligned && col + 3u < a.n) {
                f32x4 *o4 = reinterpret_cast<f32x4 *>(o);
                if (adds) v += *o4;
                *o4 = v;
            } else {
#pragma unroll
                for (int r = 0; r < 4; r++)
                    if (col + r < a.n) o[r] = adds ? o[r] + v[r] : v[r];
            }
        }
    }
}

template <int TT, class H, int RQ>
zhip_result launch_tile(const Dispatch &d, const char *name, const Q8Args &a) {
    auto kernel = matmul_q8_bf16_wide_kernel<TT, H, RQ>;
    constexpr int bytes = lds_bytes<TT, RQ>();
    if (!lds_opt_in<matmul_q8_bf16_wide_kernel<TT, H, RQ>, bytes>()) return fail(d, ZHIP_E_GPU, "%s: cannot reserve %d bytes of LDS", name, bytes);
    const uint32_t tiles_n = (a.n + 32 * RQ - 1) / (32 * RQ);
    const uint64_t tiles_t = (a.rows + 32 * TT - 1) / (32 * TT), tiles = (uint64_t)tiles_n * tiles_t;
    if (tiles >= (1ull << 31)) return fail(d, ZHIP_E_BAD_COMMAND, "%s: grid too large", name);
    // The kernel's 32-bit offsets also name the rows and tokens of partial tiles past the end.
    if ((uint64_t)tiles_n * (32 * RQ) * a.row_bytes >= (1ull << 32) || tiles_t * (32 * TT) * a.k * 2u >= (1ull << 32))
        return fail(d, ZHIP_E_BAD_COMMAND, "%s: operands of 4 GiB or more", name);
    hipLaunchKernelGGL(kernel, dim3((uint32_t)tiles), dim3(threads<RQ>()), bytes, d.stream, a, tiles_n);
    return check_launch(d, name);
}

template <class H>
zhip_result launch_as(const Dispatch &d, const char *name, const Q8Args &a) {
    // The largest tile that keeps more than half of the CUs busy: 128 tokens x 128 rows, 64
    // tokens x 128 rows (every weight converted twice as often), 64 x 64. A token's sums are the
    // same bits in all three.
    const uint64_t cus = (uint64_t)d.dev->compute_units, columns = (a.n + 127u) / 128u;
    if (a.rows > 64u && 2u * ((a.rows + 127u) / 128u) * columns > cus) return launch_tile<4, H, 4>(d, name, a);
    if (a.rows > 64u && 2u * ((a.rows + 63u) / 64u) * columns > cus) return launch_tile<2, H, 4>(d, name, a);
    return launch_tile<2, H, 2>(d, name, a);
}

}  // namespace

bool matmul_q8_bf16_wide_prepare_no_alloc() {
    return lds_opt_in<matmul_q8_bf16_wide_kernel<4, AsBf16, 4>, lds_bytes<4, 4>()>() && lds_opt_in<matmul_q8_bf16_wide_kernel<2, AsBf16, 4>, lds_bytes<2, 4>()>() &&
           lds_opt_in<matmul_q8_bf16_wide_kernel<2, AsBf16, 2>, lds_bytes<2, 2>()>();
}

// Matrices whose 128-row tiles fill the CUs at the longest step a planner records
// (src/plan/plan.zig:129). The rule reads the matrix only: this kernel and the one for narrower
// matrices add k in different orders, and a token's bits must not depend on the length of the
// step it is part of.
bool matmul_q8_bf16_wide_accepts(const Dispatch &d, uint32_t n) {
    return (uint64_t)((n + 127u) / 128u) * (kPlannerStepCap / 128u) >= (uint64_t)d.dev->compute_units;
}

// x: the activations packed two bytes a value, bf16 or (f16 = true) f16. Whole, unsliced k in
// 128-deep steps (matmul_q8_bf16_accepts), operands the 32-bit offsets reach.
zhip_result launch_matmul_q8_bf16_wide(const Dispatch &d, const char *name, bool f16, const uint8_t *x, const uint8_t *w, float *out, uint32_t rows,
    uint32_t n, uint32_t k, uint32_t col0, uint32_t out_stride, uint32_t accumulate, uint32_t row_bytes, uint32_t x_bytes, uint32_t w_bytes) {
    Q8Args a{};
    a.x = x; a.w = w; a.out = out;
    a.rows = rows; a.n = n; a.k = k; a.col0 = col0; a.out_stride = out_stride; a.accumulate = accumulate;
    a.row_bytes = row_bytes; a.x_bytes = x_bytes; a.w_bytes = w_bytes;
    return f16 ? launch_as<AsF16>(d, name, a) : launch_as<AsBf16>(d, name, a);
}

}  // namespace zhip
