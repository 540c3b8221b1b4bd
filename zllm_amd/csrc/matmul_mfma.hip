// Prefill multiplies on the CDNA4 matrix cores: the bf16 rung of matmul_bf16
// and matmul_q8_0_float (same parameter blocks, bindings and grids as
// src/kernels/matmul_half.wgsl and src/kernels/matmul_q8_0_float.wgsl).
//
// out[t][col0 + j] (+)= sum_i bf16(x[t][i]) * bf16(w[j][i]), fp32 accumulate.
// Q8_0 weights become bf16(q * d), one rounding of the exact f32 product; BF16
// weights are used as stored; activations are narrowed to bf16 as they are
// staged (exact when the caller's f32 values are bf16-representable; a variant
// takes them already packed as bf16). This is an approximate rung in the
// reference's terms (src/precision.zig:9): operands carry 8 significant bits.
//
// What shapes the kernel, measured on MI355X:
//  * The L1 looks up about one 128-byte line per clock. A global load whose
//    neighbouring lanes sit in different lines costs a clock per lane, so every
//    load here has 8 (or 16) neighbouring lanes cover whole lines; the MFMA's
//    own operand layout (neighbouring lanes = different rows) is reached
//    through LDS, never straight from memory.
//  * LDS moves 128 bytes per clock and CU. Q8_0 weights therefore cross LDS as
//    the bytes they are stored in and are dequantised after the fragment read,
//    in the registers of the one wave that multiplies them: half the LDS bytes
//    of staging bf16, and no weight is converted twice.
//  * MFMAs and ordinary vector instructions share one issue port per SIMD, and
//    turning a Q8_0 weight into bf16 takes 2.5 of the latter. The tile is
//    therefore tall: 128 tokens x 64 matrix rows, so that a converted weight
//    feeds eight MFMA tiles.
//  * A step of 512 tokens on a 4096-row matrix is 8192 outputs per CU and a sum
//    over k cannot be shared between CUs cheaply (no coherent cache between
//    the XCDs), so a workgroup keeps all of k.
//
// Tiling: 512 threads = eight wave64s = 2 (matrix rows) x 4 (k). Wave w
// multiplies all the tile's tokens by matrix rows 32 (w % 2) .. + 31 over one
// quarter of every 128-deep k step (positions 32 (w / 2) .. + 31: exactly one
// Q8_0 block), so each SIMD holds two waves to overlap LDS reads, conversions
// and MFMAs, and no wave converts or reads a weight another one also needs.
// The four k quarters are added through LDS at the end, always as
// (q0 + q2) + (q1 + q3).
//
// v_mfma_f32_16x16x32_bf16 takes from lane l eight k values of token l % 16 and
// eight of matrix row l % 16: lane group g = l / 16 owns positions 8 g .. 8 g + 7
// of the wave's 32.
//
// Pipeline: three steps of global loads in flight in registers (buffer loads,
// so anything past the end of a binding reads as zero), LDS double buffered,
// fragments read one step ahead of their MFMAs, one barrier per step. Activations bound as f32 are first narrowed to packed bf16
// in the context's workspace by a small kernel.
#include <hip/hip_runtime.h>

#include <type_traits>

#include "common.h"
#include "decode.cuh"

namespace zhip {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
// Native vectors rather than HIP's uint4/float4 structs: their copies are plain
// vector loads and stores, which the optimiser keeps in registers.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

namespace {

constexpr int BN = 64, BK = 128, THREADS = 512;
constexpr int XROW = BK * 2 + 16;  // LDS bytes per token row; the padding makes 16-byte fragment reads conflict-free

struct MfmaArgs {
    const uint8_t *x;  // packed bf16 rows
    const uint8_t *w;
    float *out;
    uint32_t rows, n, k, col0, out_stride, accumulate, k_slice, slice_stride;
    uint32_t row_bytes;
    uint32_t x_bytes, w_bytes;  // bytes the kernel may read behind x and w
};

// Two floats to packed bf16, round to nearest even as the reference narrows
// (src/ref/matmul.zig:250-255): one v_cvt_pk_bf16_f32.
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    const f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}

// A raw buffer: loads past `bytes` return zero instead of faulting.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_buffer(const uint8_t *base, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(base), 0, (int)bytes, 0x00020000);
}

// ---- weights ------------------------------------------------------------------------
// LDS holds a step's 64 rows as stored (WROW bytes apart), Q8_0 followed by the
// rows' four scales. Loader thread tid moves 16-byte chunks so that neighbouring
// lanes cover whole lines; consumer lane (row, g) of k quarter kq reads its
// eight weights back.

struct WQ8_0 {
    static constexpr int WROW = BK + 16;
    static constexpr int SCALES = BN * WROW;  // byte offset of the scales: [row][4] f16
    static constexpr int WBUF = SCALES + BN * 8;
    struct Raw { u32x4 q; uint32_t d; };
    struct Offsets { uint32_t q, d; };
    // chunk tid % 8 of row tid / 8; scale tid % 4 of row (tid % 256) / 4 (the
    // upper half of the workgroup loads the same scales and does not store them).
    __device__ static Offsets offsets(const MfmaArgs &a, uint32_t j0, uint32_t tid) {
        return {(j0 + (tid >> 3)) * a.row_bytes + 16u * (tid & 7u), (j0 + ((tid & 255u) >> 2)) * a.row_bytes + a.k + 2u * (tid & 3u)};
    }
    __device__ static void load(__amdgpu_buffer_rsrc_t w, const Offsets &o, uint32_t tid, uint32_t k0, Raw &r) {
        r.q = __builtin_amdgcn_raw_buffer_load_b128(w, o.q + k0, 0, 0);
        r.d = __builtin_amdgcn_raw_buffer_load_b16(w, o.d + (k0 >> 4), 0, 0);
    }
    // Scales of blocks from `ke` on are stored as zero: what a load past the
    // slice brought is not a scale.
    __device__ static void store(const Raw &r, uint8_t *buf, uint32_t tid, uint32_t k0, uint32_t ke, bool ragged) {
        *reinterpret_cast<u32x4 *>(buf + (tid >> 3) * WROW + 16u * (tid & 7u)) = r.q;
        if (tid < 256u) *reinterpret_cast<uint16_t *>(buf + SCALES + 2u * tid) = !ragged || k0 + 32u * (tid & 3u) < ke ? (uint16_t)r.d : (uint16_t)0;
    }
    struct Frag { u32x2 q; uint32_t d; };
    __device__ static void read(const uint8_t *buf, uint32_t row, uint32_t g, uint32_t kq, Frag &f) {
        f.q = *reinterpret_cast<const u32x2 *>(buf + row * WROW + 32u * kq + 8u * g);
        f.d = *reinterpret_cast<const uint16_t *>(buf + SCALES + 8u * row + 2u * kq);
    }
    // bf16(q * d) of the lane's eight weights.
    __device__ static bf16x8 frag(const Frag &f) {
        const float d = half_bits_to_float(f.d);
        const int32_t lo = (int32_t)f.q.x, hi = (int32_t)f.q.y;
        const u32x4 v = {
            pack_bf16((float)(int8_t)(lo) * d, (float)(int8_t)(lo >> 8) * d),
            pack_bf16((float)(int8_t)(lo >> 16) * d, (float)(lo >> 24) * d),
            pack_bf16((float)(int8_t)(hi) * d, (float)(int8_t)(hi >> 8) * d),
            pack_bf16((float)(int8_t)(hi >> 16) * d, (float)(hi >> 24) * d)};
        return __builtin_bit_cast(bf16x8, v);
    }
};

struct WBf16 {
    static constexpr int WROW = BK * 2 + 16;
    static constexpr int WBUF = BN * WROW;
    struct Raw { u32x4 v[2]; };
    struct Offsets { uint32_t q[2]; };
    // chunk tid % 16 of rows tid / 16 and tid / 16 + 32.
    __device__ static Offsets offsets(const MfmaArgs &a, uint32_t j0, uint32_t tid) {
        const uint32_t o = (j0 + (tid >> 4)) * a.row_bytes + 16u * (tid & 15u);
        return {{o, o + 32u * a.row_bytes}};
    }
    __device__ static void load(__amdgpu_buffer_rsrc_t w, const Offsets &o, uint32_t, uint32_t k0, Raw &r) {
        r.v[0] = __builtin_amdgcn_raw_buffer_load_b128(w, o.q[0] + 2u * k0, 0, 0);
        r.v[1] = __builtin_amdgcn_raw_buffer_load_b128(w, o.q[1] + 2u * k0, 0, 0);
    }
    __device__ static void store(const Raw &r, uint8_t *buf, uint32_t tid, uint32_t, uint32_t, bool) {
#pragma unroll
        for (int i = 0; i < 2; i++) *reinterpret_cast<u32x4 *>(buf + ((tid >> 4) + 32u * i) * WROW + 16u * (tid & 15u)) = r.v[i];
    }
    struct Frag { u32x4 v; };
    __device__ static void read(const uint8_t *buf, uint32_t row, uint32_t g, uint32_t kq, Frag &f) {
        f.v = *reinterpret_cast<const u32x4 *>(buf + row * WROW + 64u * kq + 16u * g);
    }
    __device__ static bf16x8 frag(const Frag &f) { return __builtin_bit_cast(bf16x8, f.v); }
};

// ---- activations --------------------------------------------------------------------
// 16 MT tokens per tile. Loader thread tid: rows tid / 8 (+ 64), piece tid % 8
// of both 128-byte lines of the row's step, so eight neighbouring lanes read
// one whole line.

template <int MT>
struct XStage {
    static constexpr int HALVES = MT / 4;  // 64-row groups
    u32x4 v[2 * HALVES];
};

template <class W, int MT> constexpr int lds_bytes() { return 2 * (16 * MT * XROW + W::WBUF); }

template <class W, int MT, bool RAGGED>
__global__ __launch_bounds__(THREADS) void matmul_mfma_kernel(MfmaArgs a) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    constexpr int BM = 16 * MT, XBUF = BM * XROW;
    constexpr int BUF = XBUF + W::WBUF;  // one buffer: activations, then weights
    constexpr int HALVES = MT / 4;
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t j0 = blockIdx.x * BN, t0 = blockIdx.y * BM, z = blockIdx.z;
    const uint32_t kb = z * a.k_slice, ke = min(a.k, kb + a.k_slice);
    const uint32_t lrow = lane & 15u, g = lane >> 4, wn = wave & 1u, kq = wave >> 1;

    f32x4 acc[MT][2];
#pragma unroll
    for (int i = 0; i < MT; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    // Loads never branch: the k position is part of the offset the hardware
    // range-checks, so anything past the end of x or w reads as zero; positions
    // past the slice but inside the operand read whatever follows, and a step
    // that straddles the end of the slice (RAGGED) stores zeros for those
    // activations and scales instead.
    const __amdgpu_buffer_rsrc_t xbuf = make_buffer(a.x, a.x_bytes), wbuf = make_buffer(a.w, a.w_bytes);
    const typename W::Offsets woff = W::offsets(a, j0, tid);
    const uint32_t xoff = (t0 + (tid >> 3)) * a.k * 2u + 16u * (tid & 7u);
    auto fetch = [&](uint32_t k0, typename W::Raw &w, XStage<MT> &x) __attribute__((always_inline)) {
        W::load(wbuf, woff, tid, k0, w);
#pragma unroll
        for (int h = 0; h < HALVES; h++) {
            const uint32_t o = xoff + h * 64u * a.k * 2u + 2u * k0;
            x.v[2 * h] = __builtin_amdgcn_raw_buffer_load_b128(xbuf, o, 0, 0);
            x.v[2 * h + 1] = __builtin_amdgcn_raw_buffer_load_b128(xbuf, o + 128u, 0, 0);
        }
    };
    auto commit = [&](uint32_t buf, uint32_t k0, const typename W::Raw &w, const XStage<MT> &x) __attribute__((always_inline)) {
        uint8_t *xb = lds + buf * BUF + (tid >> 3) * XROW + 16u * (tid & 7u);
#pragma unroll
        for (int h = 0; h < HALVES; h++)
#pragma unroll
            for (int l = 0; l < 2; l++) {
                const bool keep = !RAGGED || k0 + 64u * l + 8u * (tid & 7u) < ke;
                *reinterpret_cast<u32x4 *>(xb + h * 64 * XROW + 128 * l) = keep ? x.v[2 * h + l] : u32x4{0u, 0u, 0u, 0u};
            }
        W::store(w, lds + buf * BUF + XBUF, tid, k0, ke, RAGGED);
    };

    // Fragments live in registers one step ahead of the MFMAs: during step s
    // the wave multiplies the fragments of s, reads those of s + 1 from the
    // other LDS buffer (each token fragment right after the MFMAs that consumed
    // its predecessor), and writes the global data of s + 2 into the buffer the
    // fragments of s came from, so LDS traffic, conversions and MFMAs of one
    // wave overlap instead of queueing behind the barrier. Three steps of
    // global loads are in flight in registers.
    bf16x8 af[MT], bf[2];
    uint32_t cur = 0;
    auto read_b = [&](uint32_t buf, typename W::Frag (&wf)[2]) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < 2; j++) W::read(lds + buf * BUF + XBUF, 32u * wn + 16u * j + lrow, g, kq, wf[j]);
    };
    auto step = [&](uint32_t kc, typename W::Raw &wfill, XStage<MT> &xfill, const typename W::Raw &wput, const XStage<MT> &xput) __attribute__((always_inline)) {
        fetch(kc + 4u * BK, wfill, xfill);
        const uint8_t *xn = lds + (cur ^ 1u) * BUF + lrow * XROW + 64u * kq + 16u * g;
        typename W::Frag wf[2];
        read_b(cur ^ 1u, wf);
#pragma unroll
        for (int i = 0; i < MT; i++) {
#pragma unroll
            for (int j = 0; j < 2; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[i], bf[j], acc[i][j], 0, 0, 0);
            af[i] = *reinterpret_cast<const bf16x8 *>(xn + 16 * i * XROW);
        }
#pragma unroll
        for (int j = 0; j < 2; j++) bf[j] = W::frag(wf[j]);
        // Unconditional: past the last step it writes a buffer nobody reads,
        // and the step stays one basic block for the scheduler.
        commit(cur, kc + 2u * BK, wput, xput);
        __syncthreads();
        cur ^= 1u;
    };

    typename W::Raw wa, wb, wc;
    XStage<MT> xa, xb, xc;
    fetch(kb, wa, xa);
    fetch(kb + BK, wb, xb);
    fetch(kb + 2 * BK, wc, xc);
    commit(0, kb, wa, xa);
    if (kb + BK < ke) commit(1, kb + BK, wb, xb);
    fetch(kb + 3 * BK, wa, xa);
    __syncthreads();
    {
        typename W::Frag wf[2];
        read_b(0, wf);
#pragma unroll
        for (int i = 0; i < MT; i++) af[i] = *reinterpret_cast<const bf16x8 *>(lds + (16 * i + lrow) * XROW + 64u * kq + 16u * g);
#pragma unroll
        for (int j = 0; j < 2; j++) bf[j] = W::frag(wf[j]);
    }
    // Whole groups of three steps run without a branch between them, so the
    // loop has a single back edge and the loads in flight are counted exactly;
    // the one or two steps left over follow the loop.
    const uint32_t steps = (ke - kb + BK - 1) / BK;
    uint32_t k0 = kb;
    for (uint32_t group = 0; group < steps / 3u; group++, k0 += 3 * BK) {
        step(k0, wb, xb, wc, xc);
        step(k0 + BK, wc, xc, wa, xa);
        step(k0 + 2 * BK, wa, xa, wb, xb);
    }
    if (steps % 3u >= 1u) step(k0, wb, xb, wc, xc);
    if (steps % 3u == 2u) step(k0 + BK, wc, xc, wa, xa);

    // Add the four k quarters through LDS, in a fixed order whatever the
    // timing: quarters 2 and 3 hand everything to 0 and 1, then 0 and 1 swap
    // halves (quarter 0 keeps the lower token tiles), so four waves store.
    float *xchg = reinterpret_cast<float *>(lds);
    constexpr int REGS = MT * 8;  // accumulator floats per lane
    if (kq >= 2u) {
        float *dst = xchg + (size_t)(((kq - 2u) * 2u + wn) * REGS) * 64u + lane;
#pragma unroll
        for (int i = 0; i < MT; i++)
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int r = 0; r < 4; r++) dst[((i * 2 + j) * 4 + r) * 64] = acc[i][j][r];
    }
    __syncthreads();
    if (kq < 2u) {
        const float *src = xchg + (size_t)((kq * 2u + wn) * REGS) * 64u + lane;
#pragma unroll
        for (int i = 0; i < MT; i++)
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int r = 0; r < 4; r++) acc[i][j][r] += src[((i * 2 + j) * 4 + r) * 64];
    }
    __syncthreads();
    constexpr int KEEP = MT / 2;  // token tiles each of the two keeps
    if (kq < 2u) {
        float *dst = xchg + (size_t)((kq * 2u + wn) * (REGS / 2)) * 64u + lane;
#pragma unroll
        for (int i = 0; i < KEEP; i++)
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int r = 0; r < 4; r++) dst[((i * 2 + j) * 4 + r) * 64] = kq ? acc[i][j][r] : acc[i + KEEP][j][r];
    }
    __syncthreads();
    if (kq >= 2u) return;
    const float *src = xchg + (size_t)(((kq ^ 1u) * 2u + wn) * (REGS / 2)) * 64u + lane;
    // D[token][output]: the lane holds output column lane % 16 and token rows
    // 4 * (lane / 16) .. + 3 of each 16 x 16 tile.
#pragma unroll
    for (int i = 0; i < KEEP; i++) {
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const uint32_t col = j0 + 32u * wn + 16u * j + lrow;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const float other = src[((i * 2 + j) * 4 + r) * 64];
                const float mine = kq ? acc[i + KEEP][j][r] : acc[i][j][r];
                const float v = kq ? other + mine : mine + other;  // (q0 + q2) + (q1 + q3)
                const uint32_t t = t0 + 16u * (kq ? i + KEEP : i) + 4u * g + r;
                if (col >= a.n || t >= a.rows) continue;
                const size_t o = (size_t)z * a.slice_stride + (size_t)t * a.out_stride + a.col0 + col;
                a.out[o] = a.accumulate ? a.out[o] + v : v;
            }
        }
    }
}

// f32 activations to packed bf16, eight per thread.
__global__ __launch_bounds__(256) void narrow_bf16_kernel(const f32x4 *src, u32x4 *dst, uint64_t groups) {
    for (uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x; i < groups; i += (uint64_t)gridDim.x * 256u) {
        const f32x4 lo = src[2 * i], hi = src[2 * i + 1];
        dst[i] = u32x4{pack_bf16(lo.x, lo.y), pack_bf16(lo.z, lo.w), pack_bf16(hi.x, hi.y), pack_bf16(hi.z, hi.w)};
    }
}

}  // namespace

// Validation shared with the f32 rung (matmul_f32.hip); x_bytes = 4 for f32
// activations, 2 for packed bf16.
zhip_result validate_matmul(const Dispatch &d, const char *name, bool sliced, bool q8_0, uint32_t x_bytes, bool *empty);

// The 256-token tiling (matmul_mfma_wide.hip).
zhip_result launch_mfma_wide(const Dispatch &d, const char *name, bool q8_0, const uint8_t *x, const uint8_t *w, float *out,
    uint32_t rows, uint32_t n, uint32_t k, uint32_t col0, uint32_t out_stride, uint32_t accumulate, uint32_t row_bytes);

template <class W, int MT, bool RAGGED>
static zhip_result launch_kernel(const Dispatch &d, const char *name, const MfmaArgs &a, uint32_t slices) {
    auto kernel = matmul_mfma_kernel<W, MT, RAGGED>;
    constexpr int bytes = lds_bytes<W, MT>();
    static bool configured = false;
    if (!configured) {
        if (hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess) {
            (void)hipGetLastError();
            return fail(d, ZHIP_E_GPU, "%s: cannot reserve %d bytes of LDS", name, bytes);
        }
        configured = true;
    }
    const dim3 grid((a.n + BN - 1) / BN, (a.rows + 16 * MT - 1) / (16 * MT), slices);
    hipLaunchKernelGGL(kernel, grid, dim3(THREADS), bytes, d.stream, a);
    return check_launch(d, name);
}

template <class W, bool XBF16>
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
    // The kernel's 32-bit offsets and buffer sizes: validate_matmul has checked
    // that the bindings cover these, and a binding is at most 2 GiB.
    const uint64_t x_bytes = (uint64_t)a.rows * a.k * 2u, w_bytes = (uint64_t)a.n * a.row_bytes;
    if (x_bytes >= (1ull << 32) || w_bytes >= (1ull << 32)) return fail(d, ZHIP_E_BAD_COMMAND, "%s: operands of 4 GiB or more", name);
    a.x_bytes = (uint32_t)x_bytes;
    a.w_bytes = (uint32_t)w_bytes;
    if (!XBF16) {
        // Narrow the step's activations once, into the workspace.
        if (!d.work) return fail(d, ZHIP_E_GPU, "%s: no workspace", name);
        if (zhip_result r = d.work->reserve(d, x_bytes)) return r;
        const uint64_t groups = x_bytes / 16u;
        const uint64_t blocks = (groups + 255u) / 256u;
        hipLaunchKernelGGL(narrow_bf16_kernel, dim3((uint32_t)(blocks < 4096u ? blocks : 4096u)), dim3(256), 0, d.stream,
            reinterpret_cast<const f32x4 *>(a.x), reinterpret_cast<u32x4 *>(d.work->data), groups);
        a.x = d.work->data;
    }
    const uint32_t slices = sliced ? d.grid[2] : 1u;
    // Long steps whose 256 x 128 tiles fill the CUs take that tiling: each
    // weight is converted once per 256 tokens and half the bytes cross from L2.
    if (slices == 1u && a.k_slice >= a.k && (uint64_t)((a.rows + 255u) / 256u) * ((a.n + 127u) / 128u) >= (uint64_t)d.dev->compute_units)
        return launch_mfma_wide(d, name, q8_0, a.x, a.w, a.out, a.rows, a.n, a.k, a.col0, a.out_stride, a.accumulate, a.row_bytes);
    const bool ragged = a.k % BK != 0 || a.k_slice % BK != 0;
    if (a.rows > 64u) return ragged ? launch_kernel<W, 8, true>(d, name, a, slices) : launch_kernel<W, 8, false>(d, name, a, slices);
    return ragged ? launch_kernel<W, 4, true>(d, name, a, slices) : launch_kernel<W, 4, false>(d, name, a, slices);
}

zhip_result launch_matmul_bf16_mfma(const Dispatch &d) { return launch_mfma<WBf16, false>(d, "matmul_bf16", false, false); }
zhip_result launch_matmul_q8_0_float_mfma(const Dispatch &d) { return launch_mfma<WQ8_0, false>(d, "matmul_q8_0_float", true, true); }
zhip_result launch_matmul_bf16_mfma_xbf16(const Dispatch &d) { return launch_mfma<WBf16, true>(d, "matmul_bf16", false, false); }
zhip_result launch_matmul_q8_0_float_mfma_xbf16(const Dispatch &d) { return launch_mfma<WQ8_0, true>(d, "matmul_q8_0_float", true, true); }

}  // namespace zhip
