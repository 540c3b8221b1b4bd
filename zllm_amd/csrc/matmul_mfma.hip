// Prefill multiplies on the CDNA4 matrix cores: the bf16 rung of matmul_bf16
// and matmul_q8_0_float (same parameter blocks, bindings and grids as
// src/kernels/matmul_half.wgsl and src/kernels/matmul_q8_0_float.wgsl), and,
// with f16 operands, the reference's fp16_single and fp16_compensated rungs of
// those two and matmul_f16 (src/agility/kernels/matmul_q8_0_float_linalg.hlsl,
// matmul_q8_0_float_linalg_single.hlsl, matmul_half_linalg.hlsl); what follows
// describes the bf16 rung, the f16 rungs differ in the operand format only
// (see Bf16 / F16 and the COMP parameter of the kernel).
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
//    of staging bf16, and no weight is converted twice. Rows are unpadded
//    128-byte lines with their 16-byte chunks permuted against bank conflicts.
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
// (q0 + q2) + (q1 + q3), each wave finishing a quarter of the token tiles.
//
// v_mfma_f32_16x16x32_bf16 takes from lane l eight k values of matrix row l % 16
// (its first operand) and eight of token l % 16: lane group g = l / 16 owns
// positions 8 g .. 8 g + 7 of the wave's 32, and ends up with outputs 4 g .. 4 g + 3
// of token l % 16, which it stores as one 16-byte piece.
//
// Pipeline: buffer loads straight into LDS (no registers, no LDS store
// instructions; anything past the end of a binding reads as zero), three LDS
// buffers so that memory runs three steps ahead, fragments read one step ahead
// of their MFMAs, one barrier per step. Activations bound as f32 are first narrowed to packed bf16
// in the context's workspace by a small kernel.
#include <hip/hip_runtime.h>

#include <type_traits>

#include "common.h"
#include "decode.h"
#include "matvec_common.h"

namespace zhip {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
// Native vectors rather than HIP's uint4/float4 structs: their copies are plain
// vector loads and stores, which the optimiser keeps in registers.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

namespace {

constexpr int BN = 64, BK = 128, THREADS = 512;

struct MfmaArgs {
    const uint8_t *x;  // packed bf16 rows
    const uint8_t *w;
    float *out;
    uint32_t rows, n, k, col0, out_stride, accumulate, k_slice, slice_stride;
    uint32_t row_bytes;
    uint32_t x_bytes, w_bytes;  // bytes the kernel may read behind x and w
    uint32_t x_plane;           // compensated rung: bytes from the activations' f16 values to their residuals
};

// Two floats to packed bf16, round to nearest even as the reference narrows
// (src/ref/matmul.zig:250-255): one v_cvt_pk_bf16_f32.
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    const f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}

// The format both operands enter the matrix cores in. Bf16 is this backend's own rung;
// F16 is the reference's fp16_single rung (activations and weights rounded to f16, fp32
// accumulation: src/agility/kernels/matmul_q8_0_float_linalg_single.hlsl:36-58,
// src/agility/kernels/matmul_half_linalg.hlsl:34-52 with SINGLE_PRODUCT).
struct Bf16 {
    typedef bf16x8 vec8;
    __device__ static uint32_t pack(float lo, float hi) { return pack_bf16(lo, hi); }
    __device__ static float widen(uint32_t bits) { return __builtin_bit_cast(float, bits << 16); }
    __device__ static f32x4 mfma(vec8 a, vec8 b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0); }
};
struct F16 {
    typedef f16x8 vec8;
    // Round to nearest even; values beyond the f16 range become infinities, as (half)v does.
    __device__ static uint32_t pack(float lo, float hi) {
        const f32x2 v = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2));
    }
    __device__ static float widen(uint32_t bits) { return (float)__builtin_bit_cast(_Float16, (uint16_t)bits); }
    __device__ static f32x4 mfma(vec8 a, vec8 b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0); }
};

// A raw buffer: loads past `bytes` return zero instead of faulting.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_buffer(const uint8_t *base, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(base), 0, (int)bytes, 0x00020000);
}

typedef __attribute__((address_space(3))) void *lds_ptr;

// A workgroup barrier that leaves loads into LDS in flight. __syncthreads()
// carries a release fence, which waits for every outstanding memory operation,
// the loads running steps ahead included; here a wave waits for exactly the
// loads it must (vmcnt) and for its own LDS instructions, then joins.
template <int LOADS_LEFT>
__device__ __forceinline__ void sync_keeping_loads() {
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(LOADS_LEFT) : "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// One wave-wide load of 16 bytes a lane straight into LDS: lane l's bytes land
// at dst + 16 l, whatever global offset the lane asked for.
__device__ __forceinline__ void load_lds_b128(__amdgpu_buffer_rsrc_t buf, uint8_t *dst, uint32_t offset) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(buf, (lds_ptr)dst, 16, offset, 0, 0, 0);
}
__device__ __forceinline__ void load_lds_b32(__amdgpu_buffer_rsrc_t buf, uint8_t *dst, uint32_t offset) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(buf, (lds_ptr)dst, 4, offset, 0, 0, 0);
}

// LDS holds operand rows as 128-byte lines, eight rows to the kilobyte one
// wave-wide load fills. Unpadded lines would put every other row of a fragment
// read on the same banks, so the 16-byte chunks of a line are stored permuted:
// chunk c of row r sits at position c ^ key(r). The loading lane asks for the
// chunk that belongs at its position; a reader applies the same key. With this
// key the sixteen rows of a fragment read cover all 64 banks once.
__device__ __forceinline__ uint32_t line_key(uint32_t row) { return (row & 7u) ^ ((row >> 3) & 1u); }

// ---- weights ------------------------------------------------------------------------
// A step's 64 rows as stored, Q8_0 followed by the rows' four scales.
// Consumer lane (row, g) of k quarter kq reads its eight weights back.

struct WQ8_0 {
    static constexpr int SCALES = BN * 128;   // byte offset of the scales: [row][4] f16
    static constexpr int WBUF = SCALES + BN * 8;
    static constexpr int LOADS = 2;           // wave-wide loads a step issues per wave
    struct Offsets { uint32_t q, d; };
    // Wave w loads rows 8 w .. 8 w + 7 (lane l: row l / 8, position l % 8) and,
    // every wave the same (so that all waves have the same loads in flight),
    // the 128 scale words: word 64 (w % 2) + l = scales 2 (l % 2), + 1 of row
    // 32 (w % 2) + l / 2.
    __device__ static Offsets offsets(const MfmaArgs &a, uint32_t j0, uint32_t wave, uint32_t lane) {
        const uint32_t row = 8u * wave + (lane >> 3);
        const uint32_t srow = 32u * (wave & 1u) + (lane >> 1);
        return {(j0 + row) * a.row_bytes + 16u * ((lane & 7u) ^ line_key(row)), (j0 + srow) * a.row_bytes + a.k + 4u * (lane & 1u)};
    }
    __device__ static void load(__amdgpu_buffer_rsrc_t w, const Offsets &o, uint8_t *buf, uint32_t wave, uint32_t k0) {
        load_lds_b128(w, buf + 1024u * wave, o.q + k0);
        load_lds_b32(w, buf + SCALES + 256u * (wave & 1u), o.d + (k0 >> 4));
    }
    struct Frag { u32x2 q; uint32_t d; };
    // row: the lane's row of the tile (its key is that of row % 16).
    __device__ static void read(const uint8_t *buf, uint32_t row, uint32_t key, uint32_t g, uint32_t kq, Frag &f) {
        f.q = *reinterpret_cast<const u32x2 *>(buf + row * 128u + 16u * ((2u * kq + (g >> 1)) ^ key) + 8u * (g & 1u));
        f.d = *reinterpret_cast<const uint16_t *>(buf + SCALES + 8u * row + 2u * kq);
    }
    // The compensated rung keeps the weights as the integers they are and applies the
    // block's scale to the block's sum (src/agility/kernels/matmul_q8_0_float_linalg.hlsl:21-25).
    static constexpr bool BLOCK_SCALED = true;
    struct ScaleRaw { uint32_t s[4]; };
    // The scales of rows row0 .. row0 + 3 for k quarter kq.
    __device__ static void read_scales(const uint8_t *buf, uint32_t row0, uint32_t kq, ScaleRaw &r) {
#pragma unroll
        for (int i = 0; i < 4; i++) r.s[i] = *reinterpret_cast<const uint16_t *>(buf + SCALES + 8u * (row0 + i) + 2u * kq);
    }
    __device__ static f32x4 scales(const ScaleRaw &r) {
        return f32x4{half_bits_to_float(r.s[0]), half_bits_to_float(r.s[1]), half_bits_to_float(r.s[2]), half_bits_to_float(r.s[3])};
    }
    // The lane's eight weights as integers in the operand format (exact: |q| <= 128).
    template <class H>
    __device__ static typename H::vec8 frag_exact(const Frag &f) {
        const int32_t lo = (int32_t)f.q.x, hi = (int32_t)f.q.y;
        const u32x4 v = {
            H::pack((float)(int8_t)(lo), (float)(int8_t)(lo >> 8)), H::pack((float)(int8_t)(lo >> 16), (float)(lo >> 24)),
            H::pack((float)(int8_t)(hi), (float)(int8_t)(hi >> 8)), H::pack((float)(int8_t)(hi >> 16), (float)(hi >> 24))};
        return __builtin_bit_cast(typename H::vec8, v);
    }
    // q * d of the lane's eight weights (exact in f32), rounded once to the operand format.
    template <class H>
    __device__ static typename H::vec8 frag(const Frag &f) {
        const float d = half_bits_to_float(f.d);
        const int32_t lo = (int32_t)f.q.x, hi = (int32_t)f.q.y;
        const u32x4 v = {
            H::pack((float)(int8_t)(lo) * d, (float)(int8_t)(lo >> 8) * d),
            H::pack((float)(int8_t)(lo >> 16) * d, (float)(lo >> 24) * d),
            H::pack((float)(int8_t)(hi) * d, (float)(int8_t)(hi >> 8) * d),
            H::pack((float)(int8_t)(hi >> 16) * d, (float)(hi >> 24) * d)};
        return __builtin_bit_cast(typename H::vec8, v);
    }
};

// Weights stored as 16-bit floats of format S (Bf16 or F16): used as stored when the
// operands have that format, else widened and rounded to the operands' (the reference rounds
// decoded weights to f16: src/agility/kernels/matmul_half_linalg.hlsl:46-52).
template <class S>
struct WHalf {
    static constexpr int WBUF = 2 * BN * 128;  // two lines a row: [line][row][128]
    static constexpr int LOADS = 2;
    struct Offsets { uint32_t q[2]; };
    // Wave w loads both lines of rows 8 w .. 8 w + 7 (lane l: row l / 8, position l % 8).
    __device__ static Offsets offsets(const MfmaArgs &a, uint32_t j0, uint32_t wave, uint32_t lane) {
        const uint32_t row = 8u * wave + (lane >> 3);
        const uint32_t o = (j0 + row) * a.row_bytes + 16u * ((lane & 7u) ^ line_key(row));
        return {{o, o + 128u}};
    }
    __device__ static void load(__amdgpu_buffer_rsrc_t w, const Offsets &o, uint8_t *buf, uint32_t wave, uint32_t k0) {
        load_lds_b128(w, buf + 1024u * wave, o.q[0] + 2u * k0);
        load_lds_b128(w, buf + BN * 128 + 1024u * wave, o.q[1] + 2u * k0);
    }
    struct Frag { u32x4 v; };
    __device__ static void read(const uint8_t *buf, uint32_t row, uint32_t key, uint32_t g, uint32_t kq, Frag &f) {
        f.v = *reinterpret_cast<const u32x4 *>(buf + (kq >> 1) * (BN * 128) + row * 128u + 16u * ((4u * (kq & 1u) + g) ^ key));
    }
    static constexpr bool BLOCK_SCALED = false;
    struct ScaleRaw {};
    __device__ static void read_scales(const uint8_t *, uint32_t, uint32_t, ScaleRaw &) {}
    __device__ static f32x4 scales(const ScaleRaw &) { return f32x4{1.f, 1.f, 1.f, 1.f}; }
    template <class H>
    __device__ static typename H::vec8 frag_exact(const Frag &f) { return frag<H>(f); }
    template <class H>
    __device__ static typename H::vec8 frag(const Frag &f) {
        if constexpr (std::is_same<H, S>::value) {
            return __builtin_bit_cast(typename H::vec8, f.v);
        } else {
            u32x4 v;
#pragma unroll
            for (int i = 0; i < 4; i++) v[i] = H::pack(S::widen(f.v[i] & 0xffffu), S::widen(f.v[i] >> 16));
            return __builtin_bit_cast(typename H::vec8, v);
        }
    }
};
typedef WHalf<Bf16> WBf16;
typedef WHalf<F16> WF16;

template <class W, int MT, bool COMP = false> constexpr int buf_bytes() { return (COMP ? 2 : 1) * 16 * MT * 256 + W::WBUF; }
template <class W, int MT, bool COMP = false> constexpr int lds_bytes() { return 3 * buf_bytes<W, MT, COMP>(); }
// The exchange of the k quarters at the end reuses the buffers: 8 waves x 3 inboxes x MT / 4
// tiles x 2 x 1 KB.
static_assert(lds_bytes<WQ8_0, 8>() >= 8 * 3 * 4 * 1024 && lds_bytes<WQ8_0, 4>() >= 8 * 3 * 2 * 1024 && lds_bytes<WQ8_0, 2, true>() >= 8 * 3 * 1024, "the exchange must fit the buffers");

// COMP: the reference's compensated rung. Every activation enters twice, as its f16 value
// and as the f16 of what that rounding left (two planes of the narrowed copy, two planes in
// LDS, two MFMAs a tile); Q8_0 weights enter as their integers and a block's scale multiplies
// the block's sum (src/agility/kernels/matmul_q8_0_float_linalg.hlsl:79-101), stored halves
// are rounded to f16 and both products are summed (matmul_half_linalg.hlsl:53-60).
template <class W, class H, int MT, bool RAGGED, bool COMP = false>
__global__ __launch_bounds__(THREADS) void matmul_mfma_kernel(MfmaArgs a) {
    typedef typename H::vec8 vec8;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    constexpr int BM = 16 * MT, XPLANE = BM * 256;           // activations: [line][row][128]
    constexpr int PLANES = COMP ? 2 : 1, XBUF = PLANES * XPLANE;
    constexpr int BUF = XBUF + W::WBUF;                      // one buffer: activations, then weights
    constexpr int XLOADS = PLANES * MT / 2;                  // wave-wide activation loads a step issues per wave
    constexpr bool SCALED = COMP && W::BLOCK_SCALED;
    constexpr int LOADS = XLOADS + W::LOADS;
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t j0 = blockIdx.x * BN, t0 = blockIdx.y * BM, z = blockIdx.z;
    const uint32_t kb = z * a.k_slice, ke = min(a.k, kb + a.k_slice);
    const uint32_t lrow = lane & 15u, g = lane >> 4, wn = wave & 1u, kq = wave >> 1;

    f32x4 acc[MT][2];
#pragma unroll
    for (int i = 0; i < MT; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    // Loads go straight from memory into LDS, three steps ahead of their use,
    // through buffers whose range check covers the k position: anything past
    // the end of x or w reads as zero, positions past the slice but inside the
    // operand read whatever follows. The 32 positions of a k quarter belong to
    // one wave, so a step that straddles the end of the slice (RAGGED) needs no
    // zeroing in LDS: the waves whose quarter lies past the end multiply zeros.
    const __amdgpu_buffer_rsrc_t xbuf = make_buffer(a.x, a.x_bytes), wbuf = make_buffer(a.w, a.w_bytes);
    const typename W::Offsets woff = W::offsets(a, j0, wave, lane);
    // Activation block b = wave + 8 i of the step: line b / (BM / 8), rows 8 (b % (BM / 8)) .. + 7.
    uint32_t xoff[XLOADS], xdst[XLOADS];
#pragma unroll
    for (int i = 0; i < XLOADS; i++) {
        const uint32_t plane = i / (MT / 2), b = wave + 8u * (i % (MT / 2)), line = b / (BM / 8), row = 8u * (b % (BM / 8)) + (lane >> 3);
        xoff[i] = plane * a.x_plane + (t0 + row) * a.k * 2u + 128u * line + 16u * ((lane & 7u) ^ line_key(row));
        xdst[i] = plane * XPLANE + line * (BM * 128) + 1024u * (b % (BM / 8));
    }
    auto fetch = [&](uint32_t buf, uint32_t k0) __attribute__((always_inline)) {
        uint8_t *base = lds + buf * BUF;
#pragma unroll
        for (int i = 0; i < XLOADS; i++) load_lds_b128(xbuf, base + xdst[i], xoff[i] + 2u * k0);
        W::load(wbuf, woff, base + XBUF, wave, k0);
    };

    // Fragment addresses: the lane's token row within a 16-row tile and its
    // eight positions 32 kq + 8 g .. + 7 of the step, i.e. chunk 4 (kq % 2) + g
    // of line kq / 2.
    const uint32_t key = line_key(lrow);
    const uint32_t a_at = (kq >> 1) * (BM * 128) + lrow * 128u + 16u * ((4u * (kq & 1u) + g) ^ key);
    vec8 af[MT], af2[COMP ? MT : 1], bf[2];
    f32x4 sc[2];  // SCALED: the block scales of the lane's four outputs in each of its two tiles
    struct Raw {
        typename W::Frag wf[2];
        typename W::ScaleRaw sr[2];
    };
    auto read_b = [&](uint32_t buf, Raw &r) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < 2; j++) {
            W::read(lds + buf * BUF + XBUF, 32u * wn + 16u * j + lrow, key, g, kq, r.wf[j]);
            if (SCALED) W::read_scales(lds + buf * BUF + XBUF, 32u * wn + 16u * j + 4u * g, kq, r.sr[j]);
        }
    };
    auto convert = [&](const Raw &r, uint32_t k0) __attribute__((always_inline)) {
        const bool live = !RAGGED || k0 + 32u * kq < ke;
#pragma unroll
        for (int j = 0; j < 2; j++) {
            bf[j] = live ? (SCALED ? W::template frag_exact<H>(r.wf[j]) : W::template frag<H>(r.wf[j])) : __builtin_bit_cast(vec8, u32x4{0u, 0u, 0u, 0u});
            if (SCALED) sc[j] = live ? W::scales(r.sr[j]) : f32x4{0.f, 0.f, 0.f, 0.f};
        }
    };
    // One token tile against the wave's two weight tiles.
    auto multiply = [&](int i) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < 2; j++) {
            if constexpr (SCALED) {
                f32x4 part = H::mfma(bf[j], af[i], f32x4{0.f, 0.f, 0.f, 0.f});
                part = H::mfma(bf[j], af2[i], part);
                acc[i][j] = part * sc[j] + acc[i][j];
            } else if constexpr (COMP) {
                acc[i][j] = H::mfma(bf[j], af2[i], H::mfma(bf[j], af[i], acc[i][j]));
            } else {
                acc[i][j] = H::mfma(bf[j], af[i], acc[i][j]);
            }
        }
    };

    const uint32_t steps = (ke - kb + BK - 1) / BK;
    fetch(0, kb);
    fetch(1, kb + BK);
    fetch(2, kb + 2 * BK);
    sync_keeping_loads<2 * LOADS>();
    {
        Raw r;
        read_b(0, r);
#pragma unroll
        for (int i = 0; i < MT; i++) {
            af[i] = *reinterpret_cast<const vec8 *>(lds + a_at + 2048 * i);
            if (COMP) af2[i] = *reinterpret_cast<const vec8 *>(lds + a_at + XPLANE + 2048 * i);
        }
        convert(r, kb);
    }
    // Every wave has its fragments of step 0 (buffer 0 may be refilled) and its
    // loads of step 1, which step 0 reads, have landed.
    sync_keeping_loads<LOADS>();

    // Step s multiplies the fragments of s from registers while it reads those
    // of s + 1 from buffer (s + 1) % 3 (each token fragment right after the
    // MFMAs that consumed its predecessor) and memory fills buffer s % 3, whose
    // fragments were read a step ago, with step s + 3. Before the barrier a
    // wave waits for its loads of step s + 2, issued a step ago.
    uint32_t cur = 0, kc = kb;
    for (uint32_t s = 0; s < steps; s++, kc += BK) {
        const uint32_t nxt = cur == 2u ? 0u : cur + 1u;
        // The waves of k quarters 0 and 1 (one on each SIMD) issue their loads
        // before their MFMAs, those of quarters 2 and 3 after their
        // conversions. The load path, LDS and the vector ALU are each saturated
        // by one phase of a wave's step; with the halves of the workgroup in
        // different phases they work at the same time (measured: 32 -> 29 us
        // on 512 x 4096 x 4096).
        if (kq < 2u) fetch(cur, kc + 3u * BK);
        const uint8_t *xn = lds + nxt * BUF + a_at;
        Raw r;
        read_b(nxt, r);
#pragma unroll
        for (int i = 0; i < MT; i++) {
            multiply(i);
            af[i] = *reinterpret_cast<const vec8 *>(xn + 2048 * i);
            if (COMP) af2[i] = *reinterpret_cast<const vec8 *>(xn + XPLANE + 2048 * i);
        }
        convert(r, kc + BK);
        if (kq >= 2u) fetch(cur, kc + 3u * BK);
        sync_keeping_loads<LOADS>();
        cur = nxt;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // nothing may still land in LDS below
    __syncthreads();

    // Add the four k quarters through LDS in one exchange: of the wave's 2 MT tiles (tile
    // 2 i + j: token tile i, weight tile j of its 32 matrix rows) the wave of quarter q keeps
    // tiles OWN q .. + OWN - 1 and hands its sums of the others to the waves that keep those;
    // after one barrier every wave adds the four quarters of its tiles in a fixed order,
    // (q0 + q2) + (q1 + q3), and stores them. The quarter is a constant in each copy of the
    // code, so that the accumulators are indexed statically.
    constexpr int OWN = 2 * MT / 4;
    static_assert(OWN >= 1 && 2 * MT % 4 == 0, "a quarter finishes a whole number of tiles");
    f32x4 *inbox = reinterpret_cast<f32x4 *>(lds);
    // Where quarter `from` puts its tile number tt of those the wave of quarter `owner` keeps (from != owner).
    auto slot = [&](uint32_t owner, uint32_t from, int tt) {
        return (((owner * 2u + wn) * 3u + ((from + 3u - owner) & 3u)) * OWN + tt) * 64u + lane;
    };
    auto send = [&](auto quarter) __attribute__((always_inline)) {
        constexpr int Q = decltype(quarter)::value;
#pragma unroll
        for (int tile = 0; tile < 2 * MT; tile++) {
            if (tile / OWN == Q) continue;
            inbox[slot(tile / OWN, Q, tile % OWN)] = acc[tile / 2][tile % 2];
        }
    };
    // D[output][token] (the weights are the MFMA's first operand): the lane holds
    // outputs 4 (lane / 16) .. + 3 of token lane % 16 in each 16 x 16 tile, sixteen
    // contiguous bytes of the token's row.
    const bool aligned = ((a.out_stride | a.col0 | a.slice_stride) & 3u) == 0u && (reinterpret_cast<uintptr_t>(a.out) & 15u) == 0u;
    auto collect = [&](auto quarter) __attribute__((always_inline)) {
        constexpr int Q = decltype(quarter)::value;
#pragma unroll
        for (int tt = 0; tt < OWN; tt++) {
            {
                const int tile = OWN * Q + tt, i = tile / 2, j = tile % 2;
                const uint32_t t = t0 + 16u * i + lrow;
                f32x4 p[4];
#pragma unroll
                for (int from = 0; from < 4; from++) p[from] = from == Q ? acc[i][j] : inbox[slot(Q, from, tt)];
                f32x4 v = (p[0] + p[2]) + (p[1] + p[3]);
                const uint32_t col = j0 + 32u * wn + 16u * j + 4u * g;
                if (t >= a.rows || col >= a.n) continue;
                float *o = a.out + (size_t)z * a.slice_stride + (size_t)t * a.out_stride + a.col0 + col;
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
        }
    };
    switch (kq) {
    case 0: send(std::integral_constant<int, 0>{}); break;
    case 1: send(std::integral_constant<int, 1>{}); break;
    case 2: send(std::integral_constant<int, 2>{}); break;
    default: send(std::integral_constant<int, 3>{}); break;
    }
    __syncthreads();
    switch (kq) {
    case 0: collect(std::integral_constant<int, 0>{}); break;
    case 1: collect(std::integral_constant<int, 1>{}); break;
    case 2: collect(std::integral_constant<int, 2>{}); break;
    default: collect(std::integral_constant<int, 3>{}); break;
    }
}

// f32 activations to the packed operand format, eight per thread.
template <class H>
__global__ __launch_bounds__(256) void narrow_kernel(const f32x4 *src, u32x4 *dst, uint64_t groups) {
    for (uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x; i < groups; i += (uint64_t)gridDim.x * 256u) {
        const f32x4 lo = src[2 * i], hi = src[2 * i + 1];
        dst[i] = u32x4{H::pack(lo.x, lo.y), H::pack(lo.z, lo.w), H::pack(hi.x, hi.y), H::pack(hi.z, hi.w)};
    }
}

// f32 activations to two f16 planes: the rounded values, and the f16 of what each rounding
// left (src/agility/kernels/matmul_q8_0_float_linalg.hlsl:47-52); eight per thread.
__global__ __launch_bounds__(256) void narrow_split_kernel(const f32x4 *src, u32x4 *hi_out, u32x4 *lo_out, uint64_t groups) {
    for (uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x; i < groups; i += (uint64_t)gridDim.x * 256u) {
        const f32x4 v[2] = {src[2 * i], src[2 * i + 1]};
        u32x4 hi, lo;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const float a0 = v[e >> 1][2 * (e & 1)], a1 = v[e >> 1][2 * (e & 1) + 1];
            hi[e] = F16::pack(a0, a1);
            lo[e] = F16::pack(__fsub_rn(a0, F16::widen(hi[e] & 0xffffu)), __fsub_rn(a1, F16::widen(hi[e] >> 16)));
        }
        hi_out[i] = hi;
        lo_out[i] = lo;
    }
}

}  // namespace

// Validation shared with the f32 rung (matmul_f32.hip); x_bytes = 4 for f32
// activations, 2 for packed bf16.
zhip_result validate_matmul(const Dispatch &d, const char *name, bool sliced, bool q8_0, uint32_t x_bytes, bool *empty);

// The streaming kernel for few tokens over a short k (matmul_stream.hip).
bool matmul_stream_accepts(const Dispatch &d, bool q8_0, const float *out, uint32_t rows, uint32_t n, uint32_t k, uint32_t col0, uint32_t out_stride);
zhip_result launch_matmul_stream(const Dispatch &d, const char *name, bool q8_0, const uint8_t *x, const uint8_t *w, float *out,
    uint32_t rows, uint32_t n, uint32_t k, uint32_t col0, uint32_t out_stride, uint32_t accumulate, uint32_t row_bytes);

// The 256-token tiling (matmul_mfma_wide.hip).
zhip_result launch_mfma_wide(const Dispatch &d, const char *name, bool q8_0, const uint8_t *x, const uint8_t *w, float *out,
    uint32_t rows, uint32_t n, uint32_t k, uint32_t col0, uint32_t out_stride, uint32_t accumulate, uint32_t row_bytes);

// Q8_0 weights on the bf16 rung over whole 128-deep steps (matmul_q8_bf16.hip).
bool matmul_q8_bf16_accepts(uint32_t k, uint32_t k_slice, uint32_t slices);
// The same for matrices with enough rows for 128-row tiles (matmul_q8_bf16_wide.hip).
bool matmul_q8_bf16_wide_accepts(const Dispatch &d, uint32_t n);
zhip_result launch_matmul_q8_bf16_wide(const Dispatch &d, const char *name, bool f16, const uint8_t *x, const uint8_t *w, float *out, uint32_t rows,
    uint32_t n, uint32_t k, uint32_t col0, uint32_t out_stride, uint32_t accumulate, uint32_t row_bytes, uint32_t x_bytes, uint32_t w_bytes);
zhip_result launch_matmul_q8_bf16(const Dispatch &d, const char *name, bool f16, const uint8_t *x, const uint8_t *w, float *out, uint32_t rows, uint32_t n,
    uint32_t k, uint32_t col0, uint32_t out_stride, uint32_t accumulate, uint32_t row_bytes, uint32_t x_bytes, uint32_t w_bytes);

template <class W, class H, int MT, bool RAGGED, bool COMP = false>
static zhip_result launch_kernel(const Dispatch &d, const char *name, const MfmaArgs &a, uint32_t slices) {
    auto kernel = matmul_mfma_kernel<W, H, MT, RAGGED, COMP>;
    constexpr int bytes = lds_bytes<W, MT, COMP>();
    static_assert(bytes <= 160 * 1024, "three buffers must fit the CU's LDS");
    if (!lds_opt_in<matmul_mfma_kernel<W, H, MT, RAGGED, COMP>, bytes>()) return fail(d, ZHIP_E_GPU, "%s: cannot reserve %d bytes of LDS", name, bytes);
    const dim3 grid((a.n + BN - 1) / BN, (a.rows + 16 * MT - 1) / (16 * MT), slices);
    hipLaunchKernelGGL(kernel, grid, dim3(THREADS), bytes, d.stream, a);
    return check_launch(d, name);
}

// XPACKED: the activations are bound already packed in the operand format (an extension of
// the contract, bf16 only); otherwise they are bound as f32 and narrowed first.
template <class W, bool XPACKED, class H = Bf16, bool COMP = false>
static zhip_result launch_mfma(const Dispatch &d, const char *name, bool sliced, bool q8_0) {
    static_assert(!COMP || (!XPACKED && std::is_same<H, F16>::value), "the compensated rung narrows f32 activations to two f16 planes");
    constexpr bool XBF16 = XPACKED;
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
        const uint64_t plane = (x_bytes + 255u) & ~(uint64_t)255u;
        if (COMP && plane + x_bytes >= (1ull << 32)) return fail(d, ZHIP_E_BAD_COMMAND, "%s: operands of 4 GiB or more", name);
        if (zhip_result r = d.work->reserve(d, COMP ? plane + x_bytes : x_bytes)) return r;
        const uint64_t groups = x_bytes / 16u;
        const uint64_t blocks = (groups + 255u) / 256u;
        const dim3 ngrid((uint32_t)(blocks < 4096u ? blocks : 4096u));
        if (COMP) {
            hipLaunchKernelGGL(narrow_split_kernel, ngrid, dim3(256), 0, d.stream, reinterpret_cast<const f32x4 *>(a.x),
                reinterpret_cast<u32x4 *>(d.work->data), reinterpret_cast<u32x4 *>(d.work->data + plane), groups);
            a.x_plane = (uint32_t)plane;
            a.x_bytes = (uint32_t)(plane + x_bytes);
        } else {
            hipLaunchKernelGGL(narrow_kernel<H>, ngrid, dim3(256), 0, d.stream,
                reinterpret_cast<const f32x4 *>(a.x), reinterpret_cast<u32x4 *>(d.work->data), groups);
        }
        a.x = d.work->data;
    }
    const uint32_t slices = sliced ? d.grid[2] : 1u;
    // Which tiling a step takes depends on the matrix, never on the step's length within the
    // 512 tokens a planner records (src/plan/plan.zig:129): the tilings add k in different
    // orders, and a token's bits must not depend on how its prompt was split into steps
    // (src/sched/sched.zig:84-90).
    // A tall matrix with a short k is a pass over the weights per chunk of up to 128 tokens: the
    // kernel that streams them into registers.
    constexpr bool kBf16Rung = std::is_same<H, Bf16>::value && (std::is_same<W, WBf16>::value || std::is_same<W, WQ8_0>::value);
    if (kBf16Rung && slices == 1u && a.k_slice >= a.k && matmul_stream_accepts(d, q8_0, a.out, a.rows, a.n, a.k, a.col0, a.out_stride))
        return launch_matmul_stream(d, name, q8_0, a.x, a.w, a.out, a.rows, a.n, a.k, a.col0, a.out_stride, a.accumulate, a.row_bytes);
    // Steps longer than any the planner records (callers of their own), whose 256 x 128 tiles
    // fill the CUs, take that tiling: each weight is converted once per 256 tokens and half
    // the bytes cross from L2.
    if (kBf16Rung && slices == 1u && a.k_slice >= a.k && a.rows > kPlannerStepCap && (uint64_t)((a.rows + 255u) / 256u) * ((a.n + 127u) / 128u) >= (uint64_t)d.dev->compute_units)
        return launch_mfma_wide(d, name, q8_0, a.x, a.w, a.out, a.rows, a.n, a.k, a.col0, a.out_stride, a.accumulate, a.row_bytes);
    if constexpr (std::is_same<W, WQ8_0>::value && !COMP) {
        if (matmul_q8_bf16_accepts(a.k, a.k_slice, slices) && matmul_q8_bf16_wide_accepts(d, a.n))
            return launch_matmul_q8_bf16_wide(d, name, std::is_same<H, F16>::value, a.x, a.w, a.out, a.rows, a.n, a.k, a.col0, a.out_stride, a.accumulate,
                a.row_bytes, a.x_bytes, a.w_bytes);
        if (matmul_q8_bf16_accepts(a.k, a.k_slice, slices))
            return launch_matmul_q8_bf16(d, name, std::is_same<H, F16>::value, a.x, a.w, a.out, a.rows, a.n, a.k, a.col0, a.out_stride, a.accumulate, a.row_bytes,
                a.x_bytes, a.w_bytes);
    }
    const bool ragged = a.k % BK != 0 || a.k_slice % BK != 0;
    if constexpr (COMP) {
        // Two planes of activations in LDS: 64-token tiles.
        return ragged ? launch_kernel<W, H, 4, true, true>(d, name, a, slices) : launch_kernel<W, H, 4, false, true>(d, name, a, slices);
    }
    // 128-token tiles unless those leave half of the CUs idle and 64-token tiles (which
    // convert every weight twice as often) still run in one round.
    const uint64_t tall = (uint64_t)((a.rows + 127u) / 128u) * ((a.n + BN - 1) / BN) * slices;
    if (a.rows > 64u && 2u * tall > (uint64_t)d.dev->compute_units)
        return ragged ? launch_kernel<W, H, 8, true>(d, name, a, slices) : launch_kernel<W, H, 8, false>(d, name, a, slices);
    return ragged ? launch_kernel<W, H, 4, true>(d, name, a, slices) : launch_kernel<W, H, 4, false>(d, name, a, slices);
}

// (matmul_q8_0_float with f32-bound activations on the bf16 rung: both tile heights, whole and ragged k)
bool matmul_mfma_prepare_no_alloc() {
    return lds_opt_in<matmul_mfma_kernel<WQ8_0, Bf16, 8, false, false>, lds_bytes<WQ8_0, 8, false>()>() && lds_opt_in<matmul_mfma_kernel<WQ8_0, Bf16, 8, true, false>, lds_bytes<WQ8_0, 8, false>()>() &&
           lds_opt_in<matmul_mfma_kernel<WQ8_0, Bf16, 4, false, false>, lds_bytes<WQ8_0, 4, false>()>() && lds_opt_in<matmul_mfma_kernel<WQ8_0, Bf16, 4, true, false>, lds_bytes<WQ8_0, 4, false>()>();
}

zhip_result launch_matmul_bf16_mfma(const Dispatch &d) { return launch_mfma<WBf16, false>(d, "matmul_bf16", false, false); }
zhip_result launch_matmul_q8_0_float_mfma(const Dispatch &d) { return launch_mfma<WQ8_0, false>(d, "matmul_q8_0_float", true, true); }
zhip_result launch_matmul_bf16_mfma_xbf16(const Dispatch &d) { return launch_mfma<WBf16, true>(d, "matmul_bf16", false, false); }
zhip_result launch_matmul_q8_0_float_mfma_xbf16(const Dispatch &d) { return launch_mfma<WQ8_0, true>(d, "matmul_q8_0_float", true, true); }
// The reference's fp16_single rung: f32-bound activations rounded to f16, weights rounded to f16.
zhip_result launch_matmul_bf16_f16(const Dispatch &d) { return launch_mfma<WBf16, false, F16>(d, "matmul_bf16", false, false); }
zhip_result launch_matmul_f16_f16(const Dispatch &d) { return launch_mfma<WF16, false, F16>(d, "matmul_f16", false, false); }
zhip_result launch_matmul_q8_0_float_f16(const Dispatch &d) { return launch_mfma<WQ8_0, false, F16>(d, "matmul_q8_0_float", true, true); }
// The reference's fp16_compensated rung.
zhip_result launch_matmul_bf16_f16c(const Dispatch &d) { return launch_mfma<WBf16, false, F16, true>(d, "matmul_bf16", false, false); }
zhip_result launch_matmul_f16_f16c(const Dispatch &d) { return launch_mfma<WF16, false, F16, true>(d, "matmul_f16", false, false); }
zhip_result launch_matmul_q8_0_float_f16c(const Dispatch &d) { return launch_mfma<WQ8_0, false, F16, true>(d, "matmul_q8_0_float", true, true); }

}  // namespace zhip
