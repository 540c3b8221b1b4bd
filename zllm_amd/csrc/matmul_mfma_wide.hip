// Prefill multiplies of many tokens on the CDNA4 matrix cores: the bf16 rung of
// matmul_q8_0_float and matmul_bf16 (src/kernels/matmul_q8_0_float.wgsl,
// src/kernels/matmul_half.wgsl) for steps of more than 128 tokens whose
// activations are bound as packed bf16.
//
// out[t][col0 + j] (+)= sum_i x[t][i] * bf16(w[j][i]), fp32 accumulate.
//
// Why a second tiling: turning a Q8_0 weight into bf16 costs 2.5 VALU
// operations, and a workgroup does that once per weight of its tile whatever
// the number of tokens it multiplies them with. 256 tokens per workgroup make
// the matrix cores, not the conversion, the longer pole (per 64-deep k tile and
// SIMD: 1024 MFMA cycles against ~330 VALU cycles), and halve the bytes a CU
// pulls from L2 per flop.
//
// Tiling: 512 threads = eight wave64s as 4 (tokens) x 2 (outputs), each wave a
// 64 x 64 quadrant of the 256 x 128 tile as 2 x 2 MFMA tiles of 32 x 32 x 16:
// two waves per SIMD, so one wave's LDS waits, conversions and barrier hide
// behind the other's MFMAs. k tiles are 64 deep and double buffered in LDS
// (rows padded to 144 bytes: conflict-free 16-byte fragment reads); three k
// tiles of global loads are kept in flight in registers. Vector and matrix
// instructions share a SIMD's issue on this machine, so what a k tile costs in
// vector instructions is paid in full: the loads are buffer loads whose lane
// offsets never change and whose uniform offset is the tile's position (2048 x
// 4096 x 4096: 86.8 -> 81.5 us from that alone; the 32 x 32 x 16 form of the
// matrix instruction instead of 16 x 16 x 32 measured the same).
//
// The launcher picks this tiling only when its tiles fill the CUs; smaller
// steps take the 128 x 64 tiling of matmul_mfma.hip.
#include <hip/hip_runtime.h>

#include "common.h"
#include "decode.h"

namespace zhip {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

namespace wide {

// Range-checked loads: the address is a lane's offset plus a uniform one, so a k tile's loads
// take no vector arithmetic, and rows past the step or the matrix read zeros.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_buffer(const uint8_t *base, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(base), 0, (int)bytes, 0x00020000);
}

constexpr int GM = 256, GN = 128, GK = 64, THREADS = 512;
constexpr int ROW = GK * 2 + 16;                 // LDS bytes per tile row
constexpr int XS = GM * ROW, WS = GN * ROW;      // bytes per buffer
constexpr int LDS_BYTES = 2 * (XS + WS);         // 110,592

struct Args {
    const uint8_t *x;   // packed bf16 rows
    const uint8_t *w;
    float *out;
    uint32_t rows, n, k, col0, out_stride, accumulate, row_bytes;
    uint32_t mtiles, ntiles;
};

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    const f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}

// A thread stages 16 weights of one row per k tile: row = tid / 4, quarter = tid % 4.
struct WQ8_0 {
    struct Regs { u32x4 q; uint32_t d; };
    // The lane's offsets in the tile's rows: of the sixteen quants from position pos on and of their block's scale.
    __device__ static uint32_t quant_offset(uint32_t row_off, uint32_t pos) { return row_off + pos; }
    __device__ static uint32_t scale_offset(uint32_t row_off, uint32_t k, uint32_t pos) { return row_off + k + 2u * (pos / 32u); }
    // (kpos: a uniform multiple of 64 positions added to the lane's)
    __device__ static void load(__amdgpu_buffer_rsrc_t buf, uint32_t qoff, uint32_t doff, uint32_t kpos, Regs &r) {
        r.q = __builtin_amdgcn_raw_buffer_load_b128(buf, qoff, kpos, 0);
        r.d = __builtin_amdgcn_raw_buffer_load_b16(buf, doff, kpos / 32u * 2u, 0);
    }
    __device__ static void store(const Regs &r, u32x4 *dst) {
        const float d = half_bits_to_float(r.d);
        uint32_t o[8];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int32_t word = (int32_t)r.q[e];
            const float f0 = (float)(int8_t)(word) * d;
            const float f1 = (float)(int8_t)(word >> 8) * d;
            const float f2 = (float)(int8_t)(word >> 16) * d;
            const float f3 = (float)(word >> 24) * d;
            o[2 * e] = pack_bf16(f0, f1);
            o[2 * e + 1] = pack_bf16(f2, f3);
        }
        dst[0] = u32x4{o[0], o[1], o[2], o[3]};
        dst[1] = u32x4{o[4], o[5], o[6], o[7]};
    }
};

struct WBf16 {
    struct Regs { u32x4 v[2]; };
    __device__ static uint32_t quant_offset(uint32_t row_off, uint32_t pos) { return row_off + 2u * pos; }
    __device__ static uint32_t scale_offset(uint32_t, uint32_t, uint32_t) { return 0u; }
    __device__ static void load(__amdgpu_buffer_rsrc_t buf, uint32_t qoff, uint32_t, uint32_t kpos, Regs &r) {
        r.v[0] = __builtin_amdgcn_raw_buffer_load_b128(buf, qoff, 2u * kpos, 0);
        r.v[1] = __builtin_amdgcn_raw_buffer_load_b128(buf, qoff + 16u, 2u * kpos, 0);
    }
    __device__ static void store(const Regs &r, u32x4 *dst) {
        dst[0] = r.v[0];
        dst[1] = r.v[1];
    }
};

// Activations: four 16-byte pieces per thread and k tile, rows tid / 8 + 64 i,
// piece tid % 8 of the row's 128 bytes, so eight lanes read one full line.
struct XRegs { u32x4 v[4]; };

template <class W, bool RAGGED>
__global__ __launch_bounds__(THREADS) void matmul_mfma_wide_kernel(Args a) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    uint8_t *const xs = lds;            // [2][GM * ROW]
    uint8_t *const ws = lds + 2 * XS;   // [2][GN * ROW]

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    // Workgroups go round-robin over the 8 XCDs: renumber them so that one XCD's
    // L2 sees neighbours in (token tile, output tile) order, which share one slab
    // of activations.
    uint32_t id = blockIdx.x;
    const uint32_t total = gridDim.x;
    if (total % 8u == 0) id = (id % 8u) * (total / 8u) + id / 8u;
    const uint32_t nt = id % a.ntiles, mt = id / a.ntiles;
    const uint32_t j0 = nt * GN, t0 = mt * GM;
    const uint32_t kb = 0, ke = a.k;
    const uint32_t wm = (wave >> 1) * 64u, wn = (wave & 1u) * 64u;
    const uint32_t lrow = lane & 31u, lk = (lane >> 5) * 16u;

    f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.f;

    // Staging assignments. The tile's rows of tokens and of weights are a buffer each: rows past
    // the step or the matrix read zeros, and their results are never stored.
    const uint32_t wrow = tid >> 2, wq = tid & 3u;
    const uint32_t wrows = min((uint32_t)GN, a.n - j0), xrows = min((uint32_t)GM, a.rows - t0);
    const __amdgpu_buffer_rsrc_t wbuf = make_buffer(a.w + (size_t)j0 * a.row_bytes, wrows * a.row_bytes);
    const __amdgpu_buffer_rsrc_t xbuf = make_buffer(a.x + (size_t)t0 * a.k * 2u, xrows * a.k * 2u);
    const uint32_t wqoff = W::quant_offset(wrow * a.row_bytes, 16u * wq), wdoff = W::scale_offset(wrow * a.row_bytes, a.k, 16u * wq);
    uint8_t *wdst = ws + wrow * ROW + 32u * wq;
    const uint32_t xr0 = tid >> 3, xpiece = tid & 7u;
    uint32_t xoff[4];
#pragma unroll
    for (int i = 0; i < 4; i++) xoff[i] = (xr0 + 64u * i) * a.k * 2u + 16u * xpiece;
    uint8_t *xdst = xs + xr0 * ROW + 16u * xpiece;
    const uint32_t wk_last = ke - 16u;

    // Loads are unconditional, so no branch separates them from their use; a tile that
    // straddles the end of k zeroes its activations instead (a load past a row's end brings
    // the next row's start), which zeroes the products whatever finite weights came: the
    // weights' positions are clamped into the row there, so that a scale is a scale. Whole
    // tiles take the tile's position as the loads' uniform offset: no vector arithmetic.
    auto fetch = [&](uint32_t k0, typename W::Regs &w, XRegs &x) __attribute__((always_inline)) {
        if (RAGGED) {
            const uint32_t pos = min(k0 + 16u * wq, wk_last);
            W::load(wbuf, W::quant_offset(wrow * a.row_bytes, pos), W::scale_offset(wrow * a.row_bytes, a.k, pos), 0u, w);
        } else {
            // (a tile past the end of k, loaded ahead like the others and never used: from an
            // offset no binding reaches, whether or not the range check covers the scalar offset)
            const bool live = k0 < ke;
            W::load(wbuf, live ? wqoff : kNowhere, live ? wdoff : kNowhere, live ? k0 : 0u, w);
        }
        const bool xlive = k0 < ke;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            // (ragged k: the position joins the lane's offset, which the range check covers whatever it does with the scalar one)
            if (RAGGED) x.v[i] = __builtin_amdgcn_raw_buffer_load_b128(xbuf, xoff[i] + 2u * k0, 0u, 0);
            else x.v[i] = __builtin_amdgcn_raw_buffer_load_b128(xbuf, xlive ? xoff[i] : kNowhere, xlive ? 2u * k0 : 0u, 0);
        }
    };
    auto commit = [&](uint32_t b, uint32_t k0, const typename W::Regs &w, XRegs &x) __attribute__((always_inline)) {
        if (RAGGED && k0 + 8u * xpiece >= ke) {
#pragma unroll
            for (int i = 0; i < 4; i++) x.v[i] = u32x4{0u, 0u, 0u, 0u};
        }
        W::store(w, reinterpret_cast<u32x4 *>(wdst + b * WS));
#pragma unroll
        for (int i = 0; i < 4; i++) *reinterpret_cast<u32x4 *>(xdst + b * XS + i * (64 * ROW)) = x.v[i];
    };
    uint32_t cur = 0;
    auto tile = [&](uint32_t kc, typename W::Regs &wfill, XRegs &xfill, typename W::Regs &wnext, XRegs &xnext) __attribute__((always_inline)) {
        fetch(kc + 3u * GK, wfill, xfill);
        const uint8_t *xb = xs + cur * XS + (wm + lrow) * ROW + lk;
        const uint8_t *wb = ws + cur * WS + (wn + lrow) * ROW + lk;
#pragma unroll
        for (int kk = 0; kk < GK / 16; kk++) {
            bf16x8 af[2], bfr[2];
#pragma unroll
            for (int i = 0; i < 2; i++) af[i] = *reinterpret_cast<const bf16x8 *>(xb + 32 * i * ROW + 32 * kk);
#pragma unroll
            for (int j = 0; j < 2; j++) bfr[j] = *reinterpret_cast<const bf16x8 *>(wb + 32 * j * ROW + 32 * kk);
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[j], af[i], acc[i][j], 0, 0, 0);
        }
        if (kc + GK < ke) commit(cur ^ 1u, kc + GK, wnext, xnext);
        __syncthreads();
        cur ^= 1u;
    };

    typename W::Regs w0, w1, w2;
    XRegs x0, x1, x2;
    fetch(kb, w0, x0);
    fetch(kb + GK, w1, x1);
    fetch(kb + 2 * GK, w2, x2);
    commit(0, kb, w0, x0);
    __syncthreads();
    // Whole groups of three tiles run without a branch between them, so the
    // loop has a single back edge and the loads in flight are counted exactly;
    // the one or two tiles left over follow the loop.
    uint32_t k0 = kb;
    for (; k0 + 3 * GK <= ke; k0 += 3 * GK) {
        tile(k0, w0, x0, w1, x1);
        tile(k0 + GK, w1, x1, w2, x2);
        tile(k0 + 2 * GK, w2, x2, w0, x0);
    }
    if (k0 < ke) {
        tile(k0, w0, x0, w1, x1);
        if (k0 + GK < ke) tile(k0 + GK, w1, x1, w2, x2);
    }

    // D[output][token] (the weights are the MFMA's first operand): the lane holds
    // outputs 8 r + 4 (lane / 32) .. + 3, r = 0 .. 3, of token lane % 32 in each 32 x 32
    // tile: sixteen contiguous bytes of the token's row four times.
    const bool aligned = ((a.out_stride | a.col0) & 3u) == 0u && (reinterpret_cast<uintptr_t>(a.out) & 15u) == 0u;
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const uint32_t t = t0 + wm + 32 * i + lrow;
#pragma unroll
        for (int jr = 0; jr < 8; jr++) {
            const int j = jr >> 2, r = jr & 3;
            const uint32_t col = j0 + wn + 32 * j + 8 * r + 4 * (lane >> 5);
            if (t >= a.rows || col >= a.n) continue;
            float *o = a.out + (size_t)t * a.out_stride + a.col0 + col;
            f32x4 v = f32x4{acc[i][j][4 * r], acc[i][j][4 * r + 1], acc[i][j][4 * r + 2], acc[i][j][4 * r + 3]};
            if (aligned && col + 3u < a.n) {
                f32x4 *o4 = reinterpret_cast<f32x4 *>(o);
                if (a.accumulate) v += *o4;
                *o4 = v;
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++)
                    if (col + e < a.n) o[e] = a.accumulate ? o[e] + v[e] : v[e];
            }
        }
    }
}

template <class W>
static zhip_result launch(const Dispatch &d, const char *name, Args a) {
    a.mtiles = (a.rows + GM - 1) / GM;
    a.ntiles = (a.n + GN - 1) / GN;
    const uint32_t tiles = a.mtiles * a.ntiles;
    const bool ragged = a.k % GK != 0;
    auto kernel = ragged ? matmul_mfma_wide_kernel<W, true> : matmul_mfma_wide_kernel<W, false>;
    if (!(ragged ? lds_opt_in<matmul_mfma_wide_kernel<W, true>, LDS_BYTES>() : lds_opt_in<matmul_mfma_wide_kernel<W, false>, LDS_BYTES>()))
        return fail(d, ZHIP_E_GPU, "%s: cannot reserve %d bytes of LDS", name, LDS_BYTES);
    hipLaunchKernelGGL(kernel, dim3(tiles), dim3(THREADS), LDS_BYTES, d.stream, a);
    return check_launch(d, name);
}

}  // namespace wide

// Called by the bf16-activation rung's launchers once the dispatch is validated.
zhip_result launch_mfma_wide(const Dispatch &d, const char *name, bool q8_0, const uint8_t *x, const uint8_t *w, float *out,
    uint32_t rows, uint32_t n, uint32_t k, uint32_t col0, uint32_t out_stride, uint32_t accumulate, uint32_t row_bytes) {
    wide::Args a{};
    a.x = x; a.w = w; a.out = out;
    a.rows = rows; a.n = n; a.k = k; a.col0 = col0; a.out_stride = out_stride; a.accumulate = accumulate; a.row_bytes = row_bytes;
    return q8_0 ? wide::launch<wide::WQ8_0>(d, name, a) : wide::launch<wide::WBf16>(d, name, a);
}

bool matmul_mfma_wide_prepare_no_alloc() {
    return lds_opt_in<wide::matmul_mfma_wide_kernel<wide::WQ8_0, true>, wide::LDS_BYTES>() && lds_opt_in<wide::matmul_mfma_wide_kernel<wide::WQ8_0, false>, wide::LDS_BYTES>();
}

}  // namespace zhip
