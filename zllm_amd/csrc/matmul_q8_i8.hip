// matmul_q8_0 (Q8_0 weights, activations rounded to Q8_0 blocks by quantize_q8) for whole
// 128-deep k steps: the kernel the operation takes when k is a multiple of 128 and not sliced.
// Contract as in matmul_int8.hip (src/kernels/matmul_quant.wgsl):
//   out[t][col0 + j] (+)= sum over 32-position units u of dx[t][u] * dw[j][u] * sum_i(qx * qw),
// every unit's integer sum exact.
//
// The work per output and unit is one 32-deep integer dot product (the int8 matrix cores do
// 1024 of them per instruction) and its scaling by dx * dw, which does not factor out of the
// sum over units. On MI355X matrix and vector instructions of a SIMD's waves do not overlap
// (measured: an instruction stream of both takes the sum of their times), a wave-wide f32
// multiply-add takes ~1.4 ns of a SIMD with two waves resident, an int -> float conversion
// 1.9 ns, v_mfma_i32_32x32x32_i8 16.5 ns and v_mfma_f32_32x32x1_2b_f32 29.7 ns. Scaled with
// three vector operations per output and unit (scale product, conversion, multiply-add) the
// scaling takes five times the dot products' time and bounds the kernel. So:
//  * the scale products are a matrix instruction: v_mfma_f32_32x32x1_2b_f32 (two independent
//    32 x 32 outer products: lanes 0-31 and 32-63 each give a column of row scales and a row of
//    token scales) yields dx * dw for two token tiles, rounded once to f32 like the vector
//    multiply, in the layout of the integer tiles, in two thirds of the multiplies' time;
//  * the integer sums start from the bits of 1.5 * 2^23 (the matrix instruction's addend): the
//    result's bits are then those of the float 1.5 * 2^23 + sum, and one exact f32 subtraction
//    replaces the conversion.
// Two full-rate vector operations per output and unit remain.
//
// Tiling as in matmul_q8_bf16.hip: a workgroup computes 128 (or 64, or 32) tokens x 64 matrix rows;
// wave w multiplies rows 32 (w % 2) .. + 31 by all the tile's tokens over unit w / 2 of every
// step, lane l holding row (token) l % 32 and bytes 16 (l / 32) .. + 15 of the unit. Operands
// arrive straight in LDS (range-checked buffers: what lies past a binding reads as zero) three
// steps ahead, every wave issuing its share; fragments are read one step ahead. The four units'
// sums meet through LDS at the end, always as (u0 + u2) + (u1 + u3): a token's bits depend
// neither on the tokens beside it nor on the tile height.
#include <hip/hip_runtime.h>

#include <type_traits>

#include "common.h"

namespace zhip {

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x32 __attribute__((ext_vector_type(32)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x16 __attribute__((ext_vector_type(16)));

constexpr int BN = 64, BK = 128, WAVES = 8, THREADS = 64 * WAVES;
// One step in LDS: token lines [token][128 B], weight lines [row][128 B], then per wave 256 bytes
// of row scales ([8 rows][4 f16], the rest filler) and 256 bytes of token scales ([16 tokens][4 f32]).
template <int TT> constexpr int abuf_bytes() { return 32 * TT * 128; }
constexpr int WBUF = BN * 128, SBUF = WAVES * 256, DBUF = WAVES * 256;
// (and, with 32-token tiles, a spare KB where the loads of the four waves that have no token
// lines to bring land their nothing)
template <int TT> constexpr int buf_bytes() { return abuf_bytes<TT>() + WBUF + SBUF + DBUF + (TT == 1 ? 1024 : 0); }
// Three buffers, or the exchange of the four units' sums that reuses them (8 waves x 3 inboxes x TT KB).
template <int TT> constexpr int lds_bytes() { return 3 * buf_bytes<TT>() > 8 * 3 * TT * 1024 ? 3 * buf_bytes<TT>() : 8 * 3 * TT * 1024; }
static_assert(lds_bytes<4>() <= 160 * 1024, "the buffers must fit the CU's LDS");

struct Q8I8Args {
    const uint8_t *qx;  // rows x k int8
    const uint8_t *w;   // split rows: k int8 values, k / 32 f16 scales, zero pad to 16 bytes
    const uint8_t *dx;  // rows x k / 32 f32
    float *out;
    uint32_t rows, n, k, col0, out_stride, accumulate, row_bytes;
    uint32_t qx_bytes, w_bytes, dx_bytes;  // bytes the kernel may read behind the pointers
};

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_buffer(const uint8_t *base, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(base), 0, (int)bytes, 0x00020000);
}
typedef __attribute__((address_space(3))) void *lds_ptr;
// One wave-wide load straight into LDS: lane l's bytes land at dst + size * l. The destination
// reaches the load as a bare number, so that the compiler keeps no dependency between these
// loads and the LDS reads of the same wave (it would wait for every load in flight before each
// read); the barriers order them.
__device__ __forceinline__ void load_lds_b128(__amdgpu_buffer_rsrc_t buf, uint32_t dst, uint32_t voff, uint32_t soff) {
    asm volatile("" : "+s"(dst));
    __builtin_amdgcn_raw_ptr_buffer_load_lds(buf, (lds_ptr)(uintptr_t)dst, 16, voff, soff, 0, 0);
}
__device__ __forceinline__ void load_lds_b32(__amdgpu_buffer_rsrc_t buf, uint32_t dst, uint32_t voff, uint32_t soff) {
    asm volatile("" : "+s"(dst));
    __builtin_amdgcn_raw_ptr_buffer_load_lds(buf, (lds_ptr)(uintptr_t)dst, 4, voff, soff, 0, 0);
}
// A workgroup barrier after the wave's LDS reads, leaving its newest loads in flight.
template <int LOADS_LEFT>
__device__ __forceinline__ void sync_keeping_loads() {
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(LOADS_LEFT) : "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}
// Chunk c (16 bytes) of line r sits at position c ^ key(r): the 32-line fragment reads then run
// at the LDS's full rate.
__device__ __forceinline__ uint32_t line_key(uint32_t row) { return (row & 7u) ^ ((row >> 3) & 1u); }

template <int TT>
struct Frags {
    i32x4 w, tok[TT];  // the row's and each tile's token's sixteen bytes of the unit
    float dw, dx[(TT + 1) / 2];  // the row's scale; the scale of the lane's token in tile 2 pair + lane / 32
};

template <int TT>
__global__ __launch_bounds__(THREADS) void matmul_q8_i8_kernel(Q8I8Args a) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    constexpr int BM = 32 * TT, ABUF = abuf_bytes<TT>(), BUF = buf_bytes<TT>();
    constexpr int XL = (TT + 1) / 2;      // token-line loads a wave issues per step (32-token tiles: four of the waves bring nothing)
    constexpr int PER_STEP = XL + 3;
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t j0 = blockIdx.x * BN, t0 = blockIdx.y * BM;
    const uint32_t steps = a.k / BK;
    const uint32_t lds0 = (uint32_t)(uintptr_t)lds;

    // ---- this wave's loads: token blocks wave and wave + 8 (8 tokens x 128 B each), weight
    // rows 8 wave .. + 7, their scales and the scales of tokens 16 wave .. + 15.
    const __amdgpu_buffer_rsrc_t xbuf = make_buffer(a.qx, a.qx_bytes), wbuf = make_buffer(a.w, a.w_bytes), dbuf = make_buffer(a.dx, a.dx_bytes);
    uint32_t xoff[XL];
#pragma unroll
    for (int i = 0; i < XL; i++) {
        const uint32_t row = 8u * (wave + 8u * i) + (lane >> 3);
        xoff[i] = row < (uint32_t)BM ? (t0 + row) * a.k + 16u * ((lane & 7u) ^ line_key(row)) : 0xF0000000u;
    }
    const uint32_t wrow = 8u * wave + (lane >> 3);
    const uint32_t woff = (j0 + wrow) * a.row_bytes + 16u * ((lane & 7u) ^ line_key(wrow));
    const uint32_t soff = lane < 16u ? (j0 + 8u * wave + (lane >> 1)) * a.row_bytes + a.k + 4u * (lane & 1u) : 0xF0000000u;
    const uint32_t dtok = 16u * wave + (lane >> 2);
    const uint32_t doff = dtok < (uint32_t)BM ? ((t0 + dtok) * (a.k / 32u) + (lane & 3u)) * 4u : 0xF0000000u;
    auto fetch = [&](uint32_t buf, uint32_t step) __attribute__((always_inline)) {
        const uint32_t base = lds0 + buf * BUF;
#pragma unroll
        for (int i = 0; i < XL; i++)
            load_lds_b128(xbuf, base + (8u * (wave + 8u * i) < (uint32_t)BM ? 1024u * (wave + 8u * i) : (uint32_t)(ABUF + WBUF + SBUF + DBUF)), xoff[i], 128u * step);
        load_lds_b128(wbuf, base + ABUF + 1024u * wave, woff, 128u * step);
        load_lds_b32(wbuf, base + ABUF + WBUF + 256u * wave, soff, 8u * step);
        load_lds_b32(dbuf, base + ABUF + WBUF + SBUF + 256u * wave, doff, 16u * step);
    };

    // ---- this wave's fragments
    const uint32_t lrow = lane & 31u, h = lane >> 5, wn = wave & 1u, kq = wave >> 1;
    const uint32_t key = line_key(lrow);
    const uint32_t wr = 32u * wn + lrow;
    const uint32_t chunk = 16u * ((2u * kq + h) ^ key);
    const uint32_t a_at = lrow * 128u + chunk;
    const uint32_t w_at = ABUF + wr * 128u + chunk;
    const uint32_t s_at = ABUF + WBUF + 256u * (wr >> 3) + 8u * (wr & 7u) + 2u * kq;
    const uint32_t d_at = ABUF + WBUF + SBUF + 16u * (32u * h + lrow) + 4u * kq;

    f32x16 acc[TT];
#pragma unroll
    for (int i = 0; i < TT; i++)
#pragma unroll
        for (int e = 0; e < 16; e++) acc[i][e] = 0.f;

    Frags<TT> f;
    auto read_tile = [&](uint32_t buf, int tt) __attribute__((always_inline)) {
        f.tok[tt] = *reinterpret_cast<const i32x4 *>(lds + buf * BUF + a_at + 4096 * tt);
    };
    auto read_scales = [&](uint32_t buf, int pair) __attribute__((always_inline)) {
        f.dx[pair] = *reinterpret_cast<const float *>(lds + buf * BUF + d_at + 1024 * pair);
    };
    auto read_rows = [&](uint32_t buf) __attribute__((always_inline)) {
        f.w = *reinterpret_cast<const i32x4 *>(lds + buf * BUF + w_at);
        f.dw = (float)*reinterpret_cast<const _Float16 *>(lds + buf * BUF + s_at);
    };
    // A tile's matrix instructions run for ~100 cycles before their results can be read, and only
    // two waves share a SIMD: a tile's scaling (32 vector instructions) is issued after the next
    // tiles' matrix instructions, the last tile's after the next step's first ones. A tile's
    // fragments of the next step are read into its registers once its matrix instructions have
    // been issued.
    // The integer sums start from the bits of 1.5 * 2^23: bits + sum are then the bits of the
    // float 1.5 * 2^23 + sum (|sum| <= 32 * 127 * 127 < 2^22, one unit in the last place is 1), and
    // the exact subtraction below replaces a conversion (half the rate of an addition here).
    constexpr int MAGIC_BITS = 0x4B400000;
    constexpr float MAGIC = 12582912.f;
    i32x16 magic;
#pragma unroll
    for (int e = 0; e < 16; e++) magic[e] = MAGIC_BITS;
    asm volatile("" : "+v"(magic));  // sixteen registers, set once
    i32x16 sums_left = magic;
    f32x16 scale_left = {};
    auto scale_into = [&](f32x16 &to, const i32x16 &sums, const f32x16 &scale) __attribute__((always_inline)) {
        const f32x16 exact = __builtin_bit_cast(f32x16, sums) - MAGIC;
#pragma unroll
        for (int e = 0; e < 16; e++) to[e] = fmaf(exact[e], scale[e], to[e]);
    };
    auto low = [](const f32x32 &v) { return __builtin_shufflevector(v, v, 0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15); };
    auto high = [](const f32x32 &v) { return __builtin_shufflevector(v, v, 16, 17, 18, 19, 20, 21, 22, 23, 24, 25, 26, 27, 28, 29, 30, 31); };
    auto multiply = [&](uint32_t nxt_buf) __attribute__((always_inline)) {
        const i32x16 zero_i = magic;
        const f32x32 zero_f = {};
        i32x16 sums[TT];
        f32x32 scale[(TT + 1) / 2];
        sums[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(f.w, f.tok[0], zero_i, 0, 0, 0);
        scale[0] = __builtin_amdgcn_mfma_f32_32x32x1f32(f.dw, f.dx[0], zero_f, 0, 0, 0);
        if constexpr (TT == 1) {
            // One tile: its scaling follows the next step's matrix instructions.
            read_tile(nxt_buf, 0);
            read_scales(nxt_buf, 0);
            read_rows(nxt_buf);
            scale_into(acc[0], sums_left, scale_left);
            sums_left = sums[0];
            scale_left = low(scale[0]);
            return;
        }
        sums[TT - 1 < 1 ? 0 : 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(f.w, f.tok[TT - 1 < 1 ? 0 : 1], zero_i, 0, 0, 0);
        read_tile(nxt_buf, 0);
        read_tile(nxt_buf, 1);
        read_scales(nxt_buf, 0);
        scale_into(acc[TT - 1], sums_left, scale_left);
        __builtin_amdgcn_sched_group_barrier(0x008, 3, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 3, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, 32, 0);
        if constexpr (TT == 4) {
            sums[2] = __builtin_amdgcn_mfma_i32_32x32x32_i8(f.w, f.tok[2], zero_i, 0, 0, 0);
            scale[1] = __builtin_amdgcn_mfma_f32_32x32x1f32(f.dw, f.dx[1], zero_f, 0, 0, 0);
            scale_into(acc[0], sums[0], low(scale[0]));
            sums[3] = __builtin_amdgcn_mfma_i32_32x32x32_i8(f.w, f.tok[3], zero_i, 0, 0, 0);
            read_tile(nxt_buf, 2);
            read_tile(nxt_buf, 3);
            read_scales(nxt_buf, 1);
            read_rows(nxt_buf);
            scale_into(acc[1], sums[1], high(scale[0]));
            scale_into(acc[2], sums[2], low(scale[1]));
            sums_left = sums[3];
            scale_left = high(scale[1]);
            __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
            __builtin_amdgcn_sched_group_barrier(0x002, 32, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 5, 0);
            __builtin_amdgcn_sched_group_barrier(0x002, 64, 0);
        } else {
            read_rows(nxt_buf);
            scale_into(acc[0], sums[0], low(scale[0]));
            sums_left = sums[TT - 1 < 1 ? 0 : 1];
            scale_left = high(scale[0]);
            __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
            __builtin_amdgcn_sched_group_barrier(0x002, 32, 0);
        }
    };

    // Steps past the end of k are loaded like the others (zeros or whatever follows in the
    // operands; nothing reads them), so that every wait counts the same loads.
    fetch(0, 0);
    fetch(1, 1);
    fetch(2, 2);
    sync_keeping_loads<2 * PER_STEP>();  // step 0 has landed
#pragma unroll
    for (int tt = 0; tt < TT; tt++) read_tile(0, tt);
#pragma unroll
    for (int pair = 0; pair < (TT + 1) / 2; pair++) read_scales(0, pair);
    read_rows(0);
    sync_keeping_loads<PER_STEP>();      // step 1 has landed; buffer 0 has been read

    // Step s multiplies the fragments of step s and reads those of step s + 1 from buffer
    // (s + 1) % 3, while buffer s % 3 is refilled with step s + 3.
    auto step = [&](uint32_t s, uint32_t cur_buf, uint32_t nxt_buf) __attribute__((always_inline)) {
        fetch(cur_buf, s + 3u);
        multiply(nxt_buf);
        sync_keeping_loads<PER_STEP>();  // step s + 2 has landed; buffer (s + 1) % 3 has been read
    };
    uint32_t s = 0;
    for (; s + 3u <= steps; s += 3u) {
        step(s, 0, 1);
        step(s + 1u, 1, 2);
        step(s + 2u, 2, 0);
    }
    if (s < steps) { step(s, 0, 1); s++; }
    if (s < steps) { step(s, 1, 2); s++; }
    scale_into(acc[TT - 1], sums_left, scale_left);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // nothing may still land in LDS during the exchange
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");

    // The four units of a tile meet in LDS: the wave of unit q keeps token tile q % TT (with
    // 64-token tiles, units q and q + 2 each keep half of tile q % 2: parts 2 (q / 2) and + 1 of the
    // lane's four groups of sums; with 32-token tiles unit q keeps part q) and hands the rest to
    // their owners.
    f32x4 *inbox = reinterpret_cast<f32x4 *>(lds);
    constexpr int PARTS = TT;
    auto owner_of = [](int tt, int part) { return TT == 4 ? tt : TT == 2 ? tt + 2 * (part / 2) : part; };
    auto slot = [&](uint32_t owner, uint32_t from, int part) {
        return (((owner * 2u + wn) * 3u + ((from + 3u - owner) & 3u)) * PARTS + part) * 64u + lane;
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
    // In each 32 x 32 tile the lane holds rows 8 p + 4 (lane / 32) .. + 3, p < 4, of token
    // lane % 32: sixteen contiguous bytes of the token's output row per group.
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
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    switch (kq) {
    case 0: collect(std::integral_constant<int, 0>{}); break;
    case 1: collect(std::integral_constant<int, 1>{}); break;
    case 2: collect(std::integral_constant<int, 2>{}); break;
    default: collect(std::integral_constant<int, 3>{}); break;
    }
}

template <int TT>
zhip_result launch_tile(const Dispatch &d, const char *name, const Q8I8Args &a) {
    auto kernel = matmul_q8_i8_kernel<TT>;
    constexpr int bytes = lds_bytes<TT>();
    static bool configured = false;
    if (!configured) {
        if (hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess) {
            (void)hipGetLastError();
            return fail(d, ZHIP_E_GPU, "%s: cannot reserve %d bytes of LDS", name, bytes);
        }
        configured = true;
    }
    const dim3 grid((a.n + BN - 1) / BN, (a.rows + 32 * TT - 1) / (32 * TT));
    hipLaunchKernelGGL(kernel, grid, dim3(THREADS), bytes, d.stream, a);
    return check_launch(d, name);
}

}  // namespace

// Whole, unsliced k in 128-deep steps (the caller has validated the bindings and that 32-bit
// offsets reach a tile past the operands' ends).
bool matmul_q8_i8_accepts(uint32_t k, uint32_t k_slice, uint32_t slices) { return slices == 1u && k_slice >= k && k >= BK && k % BK == 0u; }

zhip_result launch_matmul_q8_i8(const Dispatch &d, const char *name, const uint8_t *qx, const uint8_t *w, const uint8_t *dx, float *out, uint32_t rows,
    uint32_t n, uint32_t k, uint32_t col0, uint32_t out_stride, uint32_t accumulate, uint32_t row_bytes, uint32_t qx_bytes, uint32_t w_bytes,
    uint32_t dx_bytes) {
    Q8I8Args a{};
    a.qx = qx; a.w = w; a.dx = dx; a.out = out;
    a.rows = rows; a.n = n; a.k = k; a.col0 = col0; a.out_stride = out_stride; a.accumulate = accumulate;
    a.row_bytes = row_bytes; a.qx_bytes = qx_bytes; a.w_bytes = w_bytes; a.dx_bytes = dx_bytes;
    // 128-token tiles unless those leave half of the CUs idle: then 64-token tiles on twice the
    // CUs, then 32-token tiles.
    const uint64_t columns = (n + BN - 1) / BN, cus = (uint64_t)d.dev->compute_units;
    if (rows > 64u && 2u * ((rows + 127u) / 128u) * columns > cus) return launch_tile<4>(d, name, a);
    if (rows > 32u && 2u * ((rows + 63u) / 64u) * columns > cus) return launch_tile<2>(d, name, a);
    return launch_tile<1>(d, name, a);
}

}  // namespace zhip
