// matmul_q8_0_float on the matrix cores for whole 128-deep k steps: the kernel the bf16 rungs
// and the fp16_single rung take when k is a multiple of 128 and not sliced (same contract as
// matmul_mfma.hip: out[t][col0 + j] (+)= sum_i h(x[t][i]) * h(q[j][i] * d[j][i / 32]) with h the
// rounding to bf16 or f16, fp32 accumulate; src/kernels/matmul_q8_0_float.wgsl:1-105 for the
// bindings and the parameter block).
//
// What shapes it, measured on MI355X at 512 x 4096 x 4096:
//  * A CU's tile is 128 tokens x 64 matrix rows (8192 outputs: the step's outputs over 256 CUs;
//    a sum over k is not shared between CUs). A 128-deep step of it needs 32 KB of activations
//    and 8.5 KB of weights, and the path from L2 into a CU's LDS moves about 50 bytes a clock:
//    the loads alone take 0.39 us a step from cache-resident data and 0.48 us from this
//    workload's, against 0.27 us for the step's MFMAs. The kernel is bound by that path.
//  * Loads complete in order within a wave and a wave that issues a load while the memory
//    pipeline's queue is full stalls. Four producer waves therefore issue every load of the
//    workgroup (straight into LDS, range-checked buffers: anything past the end of a binding
//    reads as zero) and do nothing else; the eight multiplying waves never issue a load and
//    meet the producers at one barrier a step.
//  * v_mfma_f32_32x32x16_bf16: half the matrix instructions of the 16 x 16 x 32 form for the
//    same work (MFMAs and vector instructions share the SIMD's issue port), and its operand
//    layout (lane = one of 32 rows, two k halves) reads LDS a quarter faster than the
//    16-row layout (2.6 against 3.6 ns per wave-wide 16-byte read and CU).
//
// Tiling: consumer wave w multiplies matrix rows 32 (w % 2) .. + 31 by all the tile's tokens
// over k quarter w / 2 of every step (32 positions: one Q8_0 block). Lane l holds row l % 32
// and positions 16 (l / 32) .. + 15 of the quarter: one 16-byte read of the row's int8 values,
// converted once (q * d rounded to bf16: 2.5 vector instructions a weight, interleaved with the
// MFMAs) for all 128 tokens, and two 16-byte reads per 32-token tile. Fragments are read one
// step ahead into a second register set; three LDS buffers, filled three steps ahead. The four
// k quarters are added through LDS at the end, always as (q0 + q2) + (q1 + q3), the wave of
// quarter q finishing token tile q; a token's sums do not depend on the tokens beside it or on
// the tile height.
#include <hip/hip_runtime.h>

#include <type_traits>

#include "common.h"
#include "matmul_q8_tiles.h"

namespace zhip {

namespace {

using namespace q8tiles;

// TT: 32-token tiles a workgroup covers (4: 128 tokens, 2: 64, 1: 32). RN: 32-row tiles of the
// matrix it covers (2: 64 rows, 1: 32), each the work of four multiplying waves.
template <int RN> constexpr int threads() { return 64 * (4 * RN + PRODUCERS); }
// One step's weights in LDS: int8 [row][128 B], then per producer [16 rows][4 f16] and 128
// bytes of filler (the upper half of its scale load).
template <int RN> constexpr int wpart_bytes() { return 32 * RN * 128 + PRODUCERS * 256; }
template <int TT> constexpr int abuf_bytes() { return 2 * 32 * TT * 128; }  // activations of a step: [line][token][128 B]
template <int TT, int RN> constexpr int buf_bytes() { return abuf_bytes<TT>() + wpart_bytes<RN>(); }
template <int TT, int RN> constexpr int lds_bytes() { return 3 * buf_bytes<TT, RN>(); }
static_assert(lds_bytes<4, 2>() <= 160 * 1024, "three buffers must fit the CU's LDS");
// The exchange of the k quarters reuses the buffers: 4 RN waves x 3 inboxes x TT KB.
static_assert(lds_bytes<4, 2>() >= 8 * 3 * 4 * 1024 && lds_bytes<2, 2>() >= 8 * 3 * 2 * 1024 && lds_bytes<1, 1>() >= 4 * 3 * 1024, "the exchange must fit the buffers");

template <int TT, class H, int RN>
__global__ __launch_bounds__((threads<RN>())) void matmul_q8_bf16_kernel(Q8Args a) {
    typedef typename H::vec opvec;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    constexpr int BM = 32 * TT, BN = 32 * RN, CONSUMERS = 4 * RN, ABUF = abuf_bytes<TT>(), BUF = buf_bytes<TT, RN>();
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t j0 = blockIdx.x * BN, t0 = blockIdx.y * BM;
    const uint32_t steps = a.k / BK;

    if (wave >= CONSUMERS) {
        // Producers. Producer p loads a quarter of the step's activation lines (block b = p + 4 i:
        // line b / (BM / 8), tokens 8 (b % (BM / 8)) .. + 7), matrix rows 8 RN p .. + 8 RN - 1 and, while
        // there are rows left, the scales of rows 16 p .. + 15.
        // 8 neighbouring lanes cover one 128-byte line; the lane at position q of a line asks
        // for chunk q ^ key(row), so that chunk c of a row sits at position c ^ key(row).
        const uint32_t p = wave - CONSUMERS;
        const __amdgpu_buffer_rsrc_t xbuf = make_buffer(a.x, a.x_bytes), wbuf = make_buffer(a.w, a.w_bytes);
        constexpr int XL = 2 * TT;  // activation loads a producer issues per step
        uint32_t xoff[XL], xdst[XL], woff[RN];
#pragma unroll
        for (int i = 0; i < XL; i++) {
            const uint32_t b = p + 4u * i, line = b / (BM / 8), row = 8u * (b % (BM / 8)) + (lane >> 3);
            xoff[i] = (t0 + row) * a.k * 2u + 128u * line + 16u * ((lane & 7u) ^ line_key(row));
            xdst[i] = line * (BM * 128) + 1024u * (b % (BM / 8));
        }
#pragma unroll
        for (int i = 0; i < RN; i++) {
            const uint32_t row = 8u * (RN * p + i) + (lane >> 3);
            woff[i] = (j0 + row) * a.row_bytes + 16u * ((lane & 7u) ^ line_key(row));
        }
        // A step's scales of the producer's sixteen rows, 8 bytes a row; the upper half of the
        // wave asks past the buffer's end (reads zero) and fills the filler.
        const uint32_t soff = lane < 32u && 16u * p < (uint32_t)BN ? (j0 + 16u * p + (lane >> 1)) * a.row_bytes + a.k + 4u * (lane & 1u) : kNowhere;
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
                for (int i = 0; i < RN; i++) load_lds_b128(wbuf, base + ABUF + 1024u * (RN * p + i), woff[i], 128u * step);
                load_lds_b32(wbuf, base + ABUF + BN * 128 + 256u * p, soff, 8u * step);
            } else {
#pragma unroll
                for (int i = 0; i < XL; i++) load_lds_b128(xbuf, base + xdst[i], kNowhere, 0u);
#pragma unroll
                for (int i = 0; i < RN; i++) load_lds_b128(wbuf, base + ABUF + 1024u * (RN * p + i), kNowhere, 0u);
                load_lds_b32(wbuf, base + ABUF + BN * 128 + 256u * p, kNowhere, 0u);
            }
        };
        constexpr int PER_STEP = XL + RN + 1;
        fetch(0, 0);
        fetch(1, 1);
        fetch(2, 2);
        sync_keeping_loads<2 * PER_STEP>();  // step 0 has landed
        sync_keeping_loads<PER_STEP>();      // step 1 has landed; buffer 0 has been read
        uint32_t buf = 0;
        for (uint32_t s = 0; s < steps; s++) {
            fetch(buf, s + 3u);
            buf = buf == 2u ? 0u : buf + 1u;
            sync_keeping_loads<PER_STEP>();  // step s + 2 has landed; buffer (s + 1) % 3 has been read
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // nothing may still land in LDS during the exchange
        __builtin_amdgcn_s_barrier();  // the loop's end
        __builtin_amdgcn_s_barrier();  // the exchange
        return;
    }

    const uint32_t lrow = lane & 31u, h = lane >> 5, wn = wave % RN, kq = wave / RN;
    f32x16 acc[TT];
#pragma unroll
    for (int i = 0; i < TT; i++)
#pragma unroll
        for (int e = 0; e < 16; e++) acc[i][e] = 0.f;

    // Fragment addresses. Weights: row 32 wn + lrow, chunk 2 kq + h of its line. Tokens: row
    // 32 tt + lrow of line kq / 2, chunks 4 (kq % 2) + 2 h and the next.
    const uint32_t key = line_key(lrow);
    const uint32_t wr = 32u * wn + lrow;
    const uint32_t w_at = ABUF + wr * 128u + 16u * ((2u * kq + h) ^ key);
    const uint32_t s_at = ABUF + BN * 128 + 256u * (wr >> 4) + 8u * (wr & 15u) + 2u * kq;
    const uint32_t a_at0 = (kq >> 1) * (BM * 128) + lrow * 128u + 16u * ((4u * (kq & 1u) + 2u * h) ^ key);
    const uint32_t a_at1 = (kq >> 1) * (BM * 128) + lrow * 128u + 16u * ((4u * (kq & 1u) + 2u * h + 1u) ^ key);

    opvec tok[2][TT][2], wop[2][2];
    auto read_frags = [&](uint32_t buf, auto set, WRaw &raw) __attribute__((always_inline)) {
        constexpr int S = decltype(set)::value;
        const uint8_t *base = lds + buf * BUF;
        raw.q = *reinterpret_cast<const u32x4 *>(base + w_at);
        raw.d = *reinterpret_cast<const uint16_t *>(base + s_at);
#pragma unroll
        for (int tt = 0; tt < TT; tt++) {
            tok[S][tt][0] = *reinterpret_cast<const opvec *>(base + a_at0 + 4096 * tt);
            tok[S][tt][1] = *reinterpret_cast<const opvec *>(base + a_at1 + 4096 * tt);
        }
    };
    auto multiply = [&](auto set) __attribute__((always_inline)) {
        constexpr int S = decltype(set)::value;
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int tt = 0; tt < TT; tt++) acc[tt] = H::mfma(wop[S][j], tok[S][tt][j], acc[tt]);
    };

    sync_after_reads();  // step 0 has landed
    {
        WRaw raw;
        read_frags(0, std::integral_constant<int, 0>{}, raw);
        convert<H>(raw, wop[0][0], wop[0][1]);
    }
    sync_after_reads();  // step 1 has landed, buffer 0 is free

    // Step s multiplies register set s % 2 (step s) and reads step s + 1 from buffer (s + 1) % 3
    // into the other set, while the producers refill buffer s % 3 with step s + 3. The weights
    // and their scale are read first, then one token fragment and a share of the conversion
    // after each MFMA.
    auto step = [&](auto cur_set, auto nxt_buf) __attribute__((always_inline)) {
        constexpr int S = decltype(cur_set)::value, NB = decltype(nxt_buf)::value;
        WRaw raw;
        read_frags(NB, std::integral_constant<int, 1 - S>{}, raw);
        multiply(cur_set);
        convert<H>(raw, wop[1 - S][0], wop[1 - S][1]);
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
#pragma unroll
        for (int i = 0; i < 2 * TT; i++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x002, TT == 4 ? 6 : TT == 2 ? 11 : 22, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        sync_after_reads();
    };
    uint32_t s = 0;
    for (; s + 6u <= steps; s += 6u) {
        step(std::integral_constant<int, 0>{}, std::integral_constant<int, 1>{});
        step(std::integral_constant<int, 1>{}, std::integral_constant<int, 2>{});
        step(std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{});
        step(std::integral_constant<int, 1>{}, std::integral_constant<int, 1>{});
        step(std::integral_constant<int, 0>{}, std::integral_constant<int, 2>{});
        step(std::integral_constant<int, 1>{}, std::integral_constant<int, 0>{});
    }
    // The remaining steps (fewer than six), same rotation. After an odd number of them the
    // finished sums are the same registers: only the operand sets alternate.
    if (s < steps) { step(std::integral_constant<int, 0>{}, std::integral_constant<int, 1>{}); s++; }
    if (s < steps) { step(std::integral_constant<int, 1>{}, std::integral_constant<int, 2>{}); s++; }
    if (s < steps) { step(std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{}); s++; }
    if (s < steps) { step(std::integral_constant<int, 1>{}, std::integral_constant<int, 1>{}); s++; }
    if (s < steps) { step(std::integral_constant<int, 0>{}, std::integral_constant<int, 2>{}); s++; }
    __builtin_amdgcn_s_barrier();  // the loop's end: the producers have no load in flight
    asm volatile("" ::: "memory");

    // The four k quarters of a tile meet in LDS: the wave of quarter q keeps token tile q % TT
    // (with 64-token tiles, quarters q and q + 2 each keep half of tile q % 2: parts 2 (q / 2) and
    // + 1 of the lane's four groups of sums; with one token tile, quarter q keeps group q) and
    // hands the rest to their owners; sums are always (q0 + q2) + (q1 + q3).
    f32x4 *inbox = reinterpret_cast<f32x4 *>(lds);
    constexpr int PARTS = TT == 1 ? 1 : TT;  // groups of four sums (of a tile's four) a quarter finishes
    auto owner_of = [](int tt, int part) { return TT == 4 ? tt : TT == 2 ? tt + 2 * (part / 2) : part; };
    auto slot = [&](uint32_t owner, uint32_t from, int part) {
        // owner: the quarter that finishes the sums; from != owner; part: which of the groups it finishes
        return (((owner * RN + wn) * 3u + ((from + 3u - owner) & 3u)) * PARTS + part) * 64u + lane;
    };
    auto send = [&](auto quarter) __attribute__((always_inline)) {
        constexpr int Q = decltype(quarter)::value;
#pragma unroll
        for (int tt = 0; tt < TT; tt++)
#pragma unroll
            for (int p = 0; p < 4; p++) {
                if (owner_of(tt, p) == Q) continue;
                inbox[slot(owner_of(tt, p), Q, TT == 4 ? p : TT == 2 ? p % 2 : 0)] = f32x4{acc[tt][4 * p], acc[tt][4 * p + 1], acc[tt][4 * p + 2], acc[tt][4 * p + 3]};
            }
    };
    const bool aligned = ((a.out_stride | a.col0) & 3u) == 0u && (reinterpret_cast<uintptr_t>(a.out) & 15u) == 0u;
    // D[row][token] (the weights are the MFMA's first operand): in each 32 x 32 tile the lane
    // holds rows 8 p + 4 (lane / 32) .. + 3, p < 4, of token lane % 32: sixteen contiguous bytes
    // of the token's row per group.
    auto collect = [&](auto quarter) __attribute__((always_inline)) {
        constexpr int Q = decltype(quarter)::value;
        constexpr int tile = Q % TT;
        const uint32_t t = t0 + 32u * tile + lrow;
#pragma unroll
        for (int i = 0; i < PARTS; i++) {
            constexpr int first = TT == 4 ? 0 : TT == 2 ? 2 * (Q / 2) : Q;
            const int p = first + i;
            f32x4 part[4];
#pragma unroll
            for (int from = 0; from < 4; from++)
                part[from] = from == Q ? f32x4{acc[tile][4 * p], acc[tile][4 * p + 1], acc[tile][4 * p + 2], acc[tile][4 * p + 3]} : inbox[slot(Q, from, i)];
            f32x4 v = (part[0] + part[2]) + (part[1] + part[3]);
            const uint32_t col = j0 + 32u * wn + 8u * p + 4u * h;
            if (t >= a.rows || col >= a.n) continue;
            float *o = a.out + (size_t)t * a.out_stride + a.col0 + col;
            if (aligned && col + 3u < a.n) {
                f32x4 *o4 = reinterpret_cast<f32x4 *>(o);
                if (a.accumulate) v += *o4;
                *o4 = v;
            } else {
#pragma unroll
                for (int r = 0; r < 4; r++)
                    if (col + r < a.n) o[r] = a.accumulate ? o[r] + v[r] : v[r];
            }
        }
    };
    switch (kq) {
    case 0: send(std::integral_constant<int, 0>{}); break;
    case 1: send(std::integral_constant<int, 1>{}); break;
    case 2: send(std::integral_constant<int, 2>{}); break;
    default: send(std::integral_constant<int, 3>{}); break;
    }
    sync_after_reads();  // the exchange
    switch (kq) {
    case 0: collect(std::integral_constant<int, 0>{}); break;
    case 1: collect(std::integral_constant<int, 1>{}); break;
    case 2: collect(std::integral_constant<int, 2>{}); break;
    default: collect(std::integral_constant<int, 3>{}); break;
    }
}

template <int TT, class H, int RN = 2>
zhip_result launch_tile(const Dispatch &d, const char *name, const Q8Args &a) {
    auto kernel = matmul_q8_bf16_kernel<TT, H, RN>;
    constexpr int bytes = lds_bytes<TT, RN>(), BN = 32 * RN;
    if (!lds_opt_in<matmul_q8_bf16_kernel<TT, H, RN>, bytes>()) return fail(d, ZHIP_E_GPU, "%s: cannot reserve %d bytes of LDS", name, bytes);
    const dim3 grid((a.n + BN - 1) / BN, (a.rows + 32 * TT - 1) / (32 * TT));
    if (grid.y > 65535u) return fail(d, ZHIP_E_BAD_COMMAND, "%s: grid too large", name);
    // The kernel's 32-bit offsets also name the rows and tokens of partial tiles past the end.
    if ((uint64_t)grid.x * BN * a.row_bytes >= (1ull << 32) || (uint64_t)grid.y * (32 * TT) * a.k * 2u >= (1ull << 32))
        return fail(d, ZHIP_E_BAD_COMMAND, "%s: operands of 4 GiB or more", name);
    hipLaunchKernelGGL(kernel, grid, dim3(threads<RN>()), bytes, d.stream, a);
    return check_launch(d, name);
}

template <class H>
zhip_result launch_as(const Dispatch &d, const char *name, const Q8Args &a) {
    // The largest tile that keeps more than half of the CUs busy: what a CU can have in flight
    // from memory bounds its share of the loads, so a short step is faster in many small tiles
    // than in few large ones. 128 tokens x 64 rows, 64 x 64 (every weight converted twice as
    // often), 32 x 64, 32 x 32. A token's sums are the same bits in all of them.
    const uint64_t cus = (uint64_t)d.dev->compute_units, columns = (a.n + 63u) / 64u;
    if (a.rows > 64u && 2u * ((a.rows + 127u) / 128u) * columns > cus) return launch_tile<4, H, 2>(d, name, a);
    if (a.rows > 32u && 2u * ((a.rows + 63u) / 64u) * columns > cus) return launch_tile<2, H, 2>(d, name, a);
    if (2u * ((a.rows + 31u) / 32u) * columns > cus) return launch_tile<1, H, 2>(d, name, a);
    return launch_tile<1, H, 1>(d, name, a);
}

}  // namespace

bool matmul_q8_bf16_prepare_no_alloc() {
    return lds_opt_in<matmul_q8_bf16_kernel<4, AsBf16, 2>, lds_bytes<4, 2>()>() && lds_opt_in<matmul_q8_bf16_kernel<2, AsBf16, 2>, lds_bytes<2, 2>()>() &&
           lds_opt_in<matmul_q8_bf16_kernel<1, AsBf16, 2>, lds_bytes<1, 2>()>() && lds_opt_in<matmul_q8_bf16_kernel<1, AsBf16, 1>, lds_bytes<1, 1>()>();
}

// Whole, unsliced k in 128-deep steps, operands the 32-bit offsets reach (the caller has
// validated the bindings).
bool matmul_q8_bf16_accepts(uint32_t k, uint32_t k_slice, uint32_t slices) { return slices == 1u && k_slice >= k && k >= BK && k % BK == 0u; }

// x: the activations packed two bytes a value, bf16 or (f16 = true) f16.
zhip_result launch_matmul_q8_bf16(const Dispatch &d, const char *name, bool f16, const uint8_t *x, const uint8_t *w, float *out, uint32_t rows, uint32_t n,
    uint32_t k, uint32_t col0, uint32_t out_stride, uint32_t accumulate, uint32_t row_bytes, uint32_t x_bytes, uint32_t w_bytes) {
    Q8Args a{};
    a.x = x; a.w = w; a.out = out;
    a.rows = rows; a.n = n; a.k = k; a.col0 = col0; a.out_stride = out_stride; a.accumulate = accumulate;
    a.row_bytes = row_bytes; a.x_bytes = x_bytes; a.w_bytes = w_bytes;
    return f16 ? launch_as<AsF16>(d, name, a) : launch_as<AsBf16>(d, name, a);
}

}  // namespace zhip
