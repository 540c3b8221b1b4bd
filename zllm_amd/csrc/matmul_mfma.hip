// Prefill multiplies on the CDNA4 matrix cores: the bf16 rung of matmul_bf16
// and matmul_q8_0_float (same parameter blocks, bindings and grids as
// src/kernels/matmul_half.wgsl and src/kernels/matmul_q8_0_float.wgsl).
//
// out[t][col0 + j] (+)= sum_i bf16(x[t][i]) * bf16(w[j][i]), fp32 accumulate.
// Weight tiles are dequantised into LDS as bf16 (Q8_0: bf16(q * d), one
// rounding of the exact f32 product; BF16 weights are copied), activation
// tiles are narrowed to bf16 as they are staged (exact when the caller's f32
// values are bf16-representable; a variant takes them already packed as bf16),
// and v_mfma_f32_16x16x32_bf16 multiplies them. This is an approximate rung in
// the reference's terms (src/precision.zig:9): operands carry 8 significant
// bits.
//
// Tiling: a workgroup of four wave64s computes BM tokens x 128 outputs over
// 64-deep k tiles; the waves sit 2 x 2, each owning a (BM/2) x 64 quadrant as
// 16 x 16 MFMA tiles. Tokens are the MFMA's M dimension and outputs its N
// dimension, so a lane's four results are four tokens of one output column and
// sixteen lanes store 64 contiguous bytes of a token's row. The k loop is
// software pipelined: the next tile's global loads are issued before the
// current tile's MFMAs and written (dequantised) into the other LDS buffer
// after them, one barrier per tile.
#include <hip/hip_runtime.h>

#include "common.h"
#include "decode.cuh"

namespace zhip {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

struct MfmaArgs {
    const uint8_t *x;  // f32 or packed bf16 rows
    const uint8_t *w;
    float *out;
    uint32_t rows, n, k, col0, out_stride, accumulate, k_slice, slice_stride;
    uint32_t row_bytes;
};

// Two floats to packed bf16, round to nearest even as the reference narrows
// (src/ref/matmul.zig:250-255): one v_cvt_pk_bf16_f32.
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    const f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}

constexpr int BN = 128, BK = 64;
constexpr int kDepth = 4;  // k tiles of global loads kept in flight
constexpr int LDS_ROW = BK * 2 + 16;  // bytes: 64 bf16 and 16 bytes of padding against bank conflicts

// ---- weight stagers: global -> registers -> LDS (as bf16) -------------------------
// A thread stages 32 weights of one row: row = tid / 2, k half = tid % 2.

struct StageBf16 {
    struct Regs { uint4 v[4]; };
    __device__ static void load(const uint8_t *row, uint32_t, uint32_t kpos, Regs &r) {
        const uint4 *src = reinterpret_cast<const uint4 *>(row + 2u * kpos);
#pragma unroll
        for (int i = 0; i < 4; i++) r.v[i] = src[i];
    }
    __device__ static void zero(Regs &r) {
#pragma unroll
        for (int i = 0; i < 4; i++) r.v[i] = make_uint4(0, 0, 0, 0);
    }
    __device__ static void store(const Regs &r, uint4 *dst) {
#pragma unroll
        for (int i = 0; i < 4; i++) dst[i] = r.v[i];
    }
};

struct StageQ8_0 {
    struct Regs { uint4 q[2]; uint32_t d; };
    __device__ static void load(const uint8_t *row, uint32_t k, uint32_t kpos, Regs &r) {
        const uint4 *src = reinterpret_cast<const uint4 *>(row + kpos);
        r.q[0] = src[0];
        r.q[1] = src[1];
        r.d = *reinterpret_cast<const uint16_t *>(row + k + 2u * (kpos / 32u));
    }
    __device__ static void zero(Regs &r) {
        r.q[0] = r.q[1] = make_uint4(0, 0, 0, 0);
        r.d = 0;
    }
    __device__ static void store(const Regs &r, uint4 *dst) {
        const float d = half_bits_to_float(r.d);
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const int32_t words[4] = {(int32_t)r.q[h].x, (int32_t)r.q[h].y, (int32_t)r.q[h].z, (int32_t)r.q[h].w};
            uint32_t o[8];
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const float f0 = (float)(int8_t)(words[e]) * d;
                const float f1 = (float)(int8_t)(words[e] >> 8) * d;
                const float f2 = (float)(int8_t)(words[e] >> 16) * d;
                const float f3 = (float)(words[e] >> 24) * d;
                o[2 * e] = pack_bf16(f0, f1);
                o[2 * e + 1] = pack_bf16(f2, f3);
            }
            dst[2 * h] = make_uint4(o[0], o[1], o[2], o[3]);
            dst[2 * h + 1] = make_uint4(o[4], o[5], o[6], o[7]);
        }
    }
};

// ---- activation stagers -----------------------------------------------------------
// BM x 64 inputs per tile; a thread stages 32 of one row when BM = 128 and 16
// when BM = 64: row = tid / (256 / BM), piece = tid % (256 / BM).

template <int BM>
struct StageXF32 {
    static constexpr int PIECES = 256 / BM;       // threads per row
    static constexpr int ELEMS = 64 / PIECES;     // inputs per thread
    struct Regs { float4 v[ELEMS / 4]; };
    __device__ static void load(const uint8_t *x, uint32_t k, uint32_t t, uint32_t kpos, Regs &r) {
        const float4 *src = reinterpret_cast<const float4 *>(x + ((size_t)t * k + kpos) * 4u);
#pragma unroll
        for (int i = 0; i < ELEMS / 4; i++) r.v[i] = src[i];
    }
    __device__ static void zero(Regs &r) {
#pragma unroll
        for (int i = 0; i < ELEMS / 4; i++) r.v[i] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
    __device__ static void store(const Regs &r, uint4 *dst) {
#pragma unroll
        for (int i = 0; i < ELEMS / 8; i++) {
            const float4 a = r.v[2 * i], b = r.v[2 * i + 1];
            dst[i] = make_uint4(pack_bf16(a.x, a.y), pack_bf16(a.z, a.w), pack_bf16(b.x, b.y), pack_bf16(b.z, b.w));
        }
    }
};

template <int BM>
struct StageXBf16 {
    static constexpr int PIECES = 256 / BM;
    static constexpr int ELEMS = 64 / PIECES;
    struct Regs { uint4 v[ELEMS / 8]; };
    __device__ static void load(const uint8_t *x, uint32_t k, uint32_t t, uint32_t kpos, Regs &r) {
        const uint4 *src = reinterpret_cast<const uint4 *>(x + ((size_t)t * k + kpos) * 2u);
#pragma unroll
        for (int i = 0; i < ELEMS / 8; i++) r.v[i] = src[i];
    }
    __device__ static void zero(Regs &r) {
#pragma unroll
        for (int i = 0; i < ELEMS / 8; i++) r.v[i] = make_uint4(0, 0, 0, 0);
    }
    __device__ static void store(const Regs &r, uint4 *dst) {
#pragma unroll
        for (int i = 0; i < ELEMS / 8; i++) dst[i] = r.v[i];
    }
};

template <class S, class X, int BM, int DEPTH>
__global__ __launch_bounds__(256) void matmul_mfma_kernel(MfmaArgs a) {
    __shared__ __attribute__((aligned(16))) uint8_t xs[2][BM * LDS_ROW];
    __shared__ __attribute__((aligned(16))) uint8_t ws[2][BN * LDS_ROW];
    constexpr int TM = BM / 32;  // 16-row MFMA tiles per wave along tokens
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t j0 = blockIdx.x * BN, t0 = blockIdx.y * BM, z = blockIdx.z;
    const uint32_t kb = z * a.k_slice, ke = min(a.k, kb + a.k_slice);
    const uint32_t wm = (wave >> 1) * (BM / 2), wn = (wave & 1u) * (BN / 2);
    const uint32_t lrow = lane & 15u, lk = (lane >> 4) * 16u;  // byte offset of the lane's 8 k values

    f32x4 acc[TM][4];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    // Staging assignments.
    const uint32_t wrow = tid >> 1, whalf = tid & 1u;
    const uint32_t xrow = tid / X::PIECES, xpiece = tid % X::PIECES;
    const uint32_t wj = j0 + wrow, xt = t0 + xrow;
    const uint8_t *wsrc = a.w + (size_t)(wj < a.n ? wj : 0u) * a.row_bytes;
    uint8_t *wdst = &ws[0][0] + wrow * LDS_ROW + 64u * whalf;
    uint8_t *xdst = &xs[0][0] + xrow * LDS_ROW + 2u * X::ELEMS * xpiece;

    // DEPTH tiles of global loads stay in flight in registers: a tile's loads
    // are issued DEPTH - 1 iterations before its dequantised copy is written
    // to LDS, which is what hides memory latency when a CU holds one or two
    // workgroups.
    typename S::Regs wr[DEPTH];
    typename X::Regs xr[DEPTH];
    auto fetch = [&](uint32_t k0, typename S::Regs &w, typename X::Regs &x) {
        const uint32_t wk = k0 + 32u * whalf, xk = k0 + X::ELEMS * xpiece;
        if (wj < a.n && wk < ke) S::load(wsrc, a.k, wk, w); else S::zero(w);
        if (xt < a.rows && xk < ke) X::load(a.x, a.k, xt, xk, x); else X::zero(x);
    };
    auto commit = [&](int b, const typename S::Regs &w, const typename X::Regs &x) {
        S::store(w, reinterpret_cast<uint4 *>(wdst + b * (BN * LDS_ROW)));
        X::store(x, reinterpret_cast<uint4 *>(xdst + b * (BM * LDS_ROW)));
    };

#pragma unroll
    for (int s = 0; s < DEPTH; s++) fetch(kb + s * BK, wr[s], xr[s]);
    commit(0, wr[0], xr[0]);
    __syncthreads();
    int cur = 0;
    for (uint32_t k0 = kb; k0 < ke; k0 += BK * DEPTH) {
#pragma unroll
        for (int s = 0; s < DEPTH; s++) {
            const uint32_t kc = k0 + s * BK;
            if (kc >= ke) break;
            // Stage s went to LDS an iteration ago: refill it DEPTH tiles ahead.
            fetch(kc + DEPTH * BK, wr[s], xr[s]);
            const uint8_t *xb = &xs[cur][0], *wb = &ws[cur][0];
#pragma unroll
            for (int kk = 0; kk < BK / 32; kk++) {
                bf16x8 af[TM], bfr[4];
#pragma unroll
                for (int i = 0; i < TM; i++) af[i] = *reinterpret_cast<const bf16x8 *>(xb + (wm + 16 * i + lrow) * LDS_ROW + 64 * kk + lk);
#pragma unroll
                for (int j = 0; j < 4; j++) bfr[j] = *reinterpret_cast<const bf16x8 *>(wb + (wn + 16 * j + lrow) * LDS_ROW + 64 * kk + lk);
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < 4; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);
            }
            if (kc + BK < ke) commit(cur ^ 1, wr[(s + 1) % DEPTH], xr[(s + 1) % DEPTH]);
            __syncthreads();
            cur ^= 1;
        }
    }

    // D[token][output]: the lane holds output column lane % 16 and token rows
    // 4 * (lane / 16) .. + 3 of each 16 x 16 tile.
#pragma unroll
    for (int i = 0; i < TM; i++) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t col = j0 + wn + 16 * j + lrow;
            if (col >= a.n) continue;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const uint32_t t = t0 + wm + 16 * i + 4 * (lane >> 4) + r;
                if (t >= a.rows) continue;
                const size_t o = (size_t)z * a.slice_stride + (size_t)t * a.out_stride + a.col0 + col;
                const float v = acc[i][j][r];
                a.out[o] = a.accumulate ? a.out[o] + v : v;
            }
        }
    }
}

// Validation shared with the f32 rung (matmul_f32.hip); x_bytes = 4 for f32
// activations, 2 for packed bf16.
zhip_result validate_matmul(const Dispatch &d, const char *name, bool sliced, bool q8_0, uint32_t x_bytes, bool *empty);

template <class S, bool XBF16>
static zhip_result launch_mfma(const Dispatch &d, const char *name, bool sliced, bool q8_0) {
    bool empty = false;
    if (zhip_result r = validate_matmul(d, name, sliced, q8_0, XBF16 ? 2u : 4u, &empty)) return r;
    if (empty) return ZHIP_OK;
    const MatmulParams &p = *reinterpret_cast<const MatmulParams *>(d.params);
    MfmaArgs a{};
    const uint64_t cover_n = (uint64_t)d.grid[0] * 64u, cover_t = (uint64_t)d.grid[1] * 16u;
    a.n = (uint32_t)(cover_n < p.n ? cover_n : p.n);
    a.rows = (uint32_t)(cover_t < p.rows ? cover_t : p.rows);
    a.k = p.k; a.col0 = p.col0; a.out_stride = p.out_stride; a.accumulate = p.accumulate;
    a.k_slice = sliced ? p.k_slice : p.k;
    a.slice_stride = sliced ? p.slice_stride : 0;
    a.row_bytes = q8_0 ? ((p.k + p.k / 16u + 15u) & ~15u) : 2u * p.k;
    a.x = d.bind[1].ptr;
    a.w = d.bind[2].ptr;
    a.out = reinterpret_cast<float *>(d.bind[3].ptr);
    const uint32_t slices = sliced ? d.grid[2] : 1u;
    // 128-token tiles halve the weight dequantisation per output; 64-token
    // tiles when those would leave compute units idle.
    const uint64_t wg128 = (uint64_t)((a.n + BN - 1) / BN) * ((a.rows + 127u) / 128u) * slices;
    if (a.rows > 64u && wg128 >= (uint64_t)d.dev->compute_units) {
        const dim3 grid((a.n + BN - 1) / BN, (a.rows + 127u) / 128u, slices);
        if (XBF16) hipLaunchKernelGGL((matmul_mfma_kernel<S, StageXBf16<128>, 128, kDepth>), grid, dim3(256), 0, d.stream, a);
        else hipLaunchKernelGGL((matmul_mfma_kernel<S, StageXF32<128>, 128, kDepth>), grid, dim3(256), 0, d.stream, a);
    } else {
        const dim3 grid((a.n + BN - 1) / BN, (a.rows + 63u) / 64u, slices);
        if (XBF16) hipLaunchKernelGGL((matmul_mfma_kernel<S, StageXBf16<64>, 64, kDepth>), grid, dim3(256), 0, d.stream, a);
        else hipLaunchKernelGGL((matmul_mfma_kernel<S, StageXF32<64>, 64, kDepth>), grid, dim3(256), 0, d.stream, a);
    }
    return check_launch(d, name);
}

zhip_result launch_matmul_bf16_mfma(const Dispatch &d) { return launch_mfma<StageBf16, false>(d, "matmul_bf16", false, false); }
zhip_result launch_matmul_q8_0_float_mfma(const Dispatch &d) { return launch_mfma<StageQ8_0, false>(d, "matmul_q8_0_float", true, true); }
zhip_result launch_matmul_bf16_mfma_xbf16(const Dispatch &d) { return launch_mfma<StageBf16, true>(d, "matmul_bf16", false, false); }
zhip_result launch_matmul_q8_0_float_mfma_xbf16(const Dispatch &d) { return launch_mfma<StageQ8_0, true>(d, "matmul_q8_0_float", true, true); }

}  // namespace zhip
