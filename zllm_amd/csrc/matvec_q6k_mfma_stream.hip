// matvec_q6_k and matvec_q3_k, matrix-core variant (MatvecVariant wg 512, lanes 64, rows 16) for steps of up to
// eight tokens and k = 1024, 2048, 3072 or 4096 (longer rows in parts, at the end of this comment): the weight stream is read once for all tokens of the step
// and the per-weight work is done once. Contract as the default variant's
// (src/kernels/matvec_quant.wgsl.hbs with the decoder of src/kernels/quant/q6_k_dot.wgsl; block
// formula src/ref/tensor.zig:118-140): out[t][col0 + j] (+)= sum over 16-weight sub-blocks of
// d * scale * sum((q - 32) * x), q the 6-bit value of ql and qh; Q3_K (the rows repacked at
// load, src/kernels/repack_q3_k.wgsl; src/ref/tensor.zig:141-160): d * (scale - 32) * sum((q - 4) * x),
// q the two low bits and the third bit. What follows describes Q6_K; Q3_K has 128-byte blocks
// (a unit is four lines a row, all eight waves load it) and its own unpacking. matvec_q8_0 over
// rows of 1024 weights runs here too (split rows, src/kernels/repack_q8_0.wgsl: d * sum(q * x)
// over 32-weight blocks): a row is 8.5 lines, so a tile's 32 rows travel as one stretch of 272
// whole lines through a ring of three slots and are read from LDS where they fall.
//
// Arithmetic. v_mfma_f32_32x32x16_f16 multiplies 32 rows of inputs by 32 weight rows over one
// sub-block. The weights enter as the exact f16 integers q - 32 (the byte dropped into the
// mantissa of 1024.0 by v_perm_b32, 1056 subtracted by v_pk_add_f16); every token enters as two
// rows, the f16 rounding of its inputs and the f16 rounding of what that left times 2^11, after
// a power of two has put its largest magnitude at 2^14 (an input keeps 22 bits, every product is
// exact in the f32 accumulator); the sub-block's d * scale multiplies its sum afterwards. Eight
// tokens fill sixteen of the 32 operand rows; the others are zeros. Up to four tokens take a
// layout of their own (eight rows, a lane's results are one piece of four tokens: four
// multiply-adds a sub-block instead of eight). A token's rows meet no other token's: its results
// do not depend on how many tokens share the launch.
//
// Layout of the work. A 512-thread workgroup is eight waves; its tiles are 32 matrix rows, taken
// as units of four 256-weight blocks a row (896 bytes = seven whole lines of each row), wave w
// multiplying half w % 2 of block w / 2 of the unit. Every workgroup builds the tokens' operands
// for itself, each wave those of its own positions (the RMSNorm and silu(x / act_div) prologues
// in the default variant's arithmetic; the waves' sums of squares and largest magnitudes meet in
// LDS), while the first unit of weights is on its way: a launch of its own that wrote them to
// memory once took 4.6 us, 1.5 us more than this costs. A unit travels as a flat copy through a
// ring of four LDS slots: the waves load it by wave-wide direct loads of whole lines (four each
// for seven of them), each wave waits for its own and one barrier a unit tells everyone that
// all of it has landed; a wave reads the unit after the one it multiplies into registers behind
// that barrier and sends the loads of the unit four ahead into the slot this frees. Chunk c (16
// bytes) of a line of row r sits at position c ^ (r % 8), which keeps the 32 rows' reads of one
// piece of a block to four lanes a bank. The waves' partial sums meet in LDS behind the same
// barrier, are added in the order of the blocks and wait there for one burst of stores when the
// workgroup's run ends. Workgroups are numbered die by die and share the rows left after whole
// rounds in units of eight.
//
// What bounds it. Per 16-weight sub-block and wave the kernel issues about 28 vector instructions
// and one matrix instruction. On this machine a vector instruction in a 32-bit encoding with
// register or literal operands costs a SIMD 1.1 - 1.2 ns, one in a 64-bit encoding (v_perm_b32,
// v_pk_add_f16, v_and_or_b32, v_lshl_or_b32, the SDWA conversions) or with a scalar-register
// operand 1.9 - 2.0 ns (measured with two and four waves a SIMD): 43 ns a sub-block, 0.7 us a
// unit and SIMD, against the 1.1 us (Q6_K) or 0.6 us (Q3_K) a unit's bytes need at full rate.
// The matrix instruction hides behind the vector work once the next sub-block's unpacking is
// put between it and the additions that wait for it. Measured on 14336 x 4096 at four / eight
// tokens: Q6_K 16.5 / 17.9 us (21.8 us before the operands were built in the kernel, the next
// unit was read ahead and the sub-blocks overlapped), Q3_K 14.3 / 15.6 us (20.3 us); Q6_K on
// 128256 x 4096 80 / 87 us (94 - 99 us; 80 us with the multiplies switched off, 80.7 us for
// one token on the default variant). Q8_0 on 151936 x 1024 at two / four / eight tokens:
// 33.9 / 32.9 / 35.6 us (41.7 us with the rows read line by line, row by row, by the kernel that
// takes k = 2048 and 4096; the default variant 33.6 / 44.1 / 79.7 us).
//
// Rows of 6144 .. 32768 weights (a multiple of 2048; the FFN-down shapes), Q6_K and Q3_K: the
// operands of so many positions do not fit a workgroup's registers, so k / 2048 workgroups share
// a walker's tiles, each over two units of every tile's rows and under its own per-token scales;
// they store their sums per part and launch_matvec_parts_sum (matvec_mfma_resident.hip) adds
// them in the order of their columns and applies the epilogue; with the RMSNorm prologue the
// tokens' scales come ready from launch_matvec_parts_scales. 4096 x 14336 at four / eight
// tokens: Q6_K 19.1 / 20.3 us (default variant 27.1 / 51.8), Q3_K 16.1 / 17.3 us (26.2 / 49.3);
// Q6_K 8192 x 8192 with the RMSNorm prologue 23.9 / 25.0 us (36.1 / 78.5).
#include <hip/hip_runtime.h>

#include <type_traits>

#include "common.h"
#include "decode.h"
#include "matvec_common.h"

namespace zhip {

namespace {

typedef _Float16 qf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 qf16x2 __attribute__((ext_vector_type(2)));
typedef float qf32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t qu32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t qu32x4 __attribute__((ext_vector_type(4)));

constexpr uint32_t THREADS = 512, WAVES = 8;
constexpr uint32_t PART_BYTES = 2u * WAVES * 256u * 4u;  // [tile parity][wave][token of the lane's four][lane]
constexpr uint32_t KEPT = 16;                   // tiles whose outputs wait in LDS for one burst of stores

// The formats. A unit is four 256-weight blocks of each of a tile's 32 rows: whole lines of every row
// (Q6_K, Q3_K) or of the tile (Q8_0).
struct FmtQ6 {  // 224-byte padded blocks: ql[128], qh[64], sixteen signed scales, d
    static constexpr int KIND = 6, SLOTS = 4;              // ring slots: the unit being read ahead and three in flight
    static constexpr bool FLAT = false;
    static constexpr uint32_t BLOCK = 224, ROW_LINES = 7;  // a row's part of a unit: seven lines
    static constexpr int LOADS = 4;                        // wave-wide loads of a unit a wave issues
    static constexpr uint32_t LOADERS = 7;                 // 28 KB: seven waves' worth; the eighth asks for nothing
    static constexpr float OFFSET = -1056.0f;              // 1024 + byte -> q - 32
    static const char *name() { return "matvec_q6_k"; }
};
struct FmtQ3 {  // blocks repacked at load into eight self-contained 16-byte units (src/kernels/repack_q3_k.wgsl)
    static constexpr int KIND = 3, SLOTS = 4;
    static constexpr bool FLAT = false;
    static constexpr uint32_t BLOCK = 128, ROW_LINES = 4;
    static constexpr int LOADS = 2;
    static constexpr uint32_t LOADERS = 8;
    static constexpr float OFFSET = -1028.0f;              // 1024 + byte -> q - 4
    static const char *name() { return "matvec_q3_k"; }
};
// Q8_0 rows of 1024 weights in split form (src/kernels/repack_q8_0.wgsl: 1024 signed bytes, then
// 32 f16 scales: 1088 bytes, 8.5 lines). The unit is the whole row, so a tile's 32 rows are one
// contiguous stretch of 272 whole lines and travel as a flat copy; the rows do not start on
// lines, which LDS does not mind (read line by line from memory, every second row's stretch of
// a wave straddles two lines and the stream runs at half its rate: 151936 x 1024, 42 us).
struct FmtQ8 {
    static constexpr int KIND = 8, SLOTS = 3;              // 34 KB a unit
    static constexpr bool FLAT = true;
    static constexpr uint32_t BLOCK = 272, ROW_LINES = 1;  // (BLOCK only so that a unit's bytes of a row are 4 BLOCK = 1088)
    static constexpr int LOADS = 5;                        // 34 loads of eight lines: seven waves' five, the 35th asks for nothing
    static constexpr uint32_t LOADERS = 7;
    static constexpr float OFFSET = -1152.0f;              // 1024 + (byte ^ 0x80) -> q
    static const char *name() { return "matvec_q8_0"; }
};
template <class F> constexpr uint32_t row_unit() { return 4u * F::BLOCK; }        // a unit's bytes of one row
template <class F> constexpr uint32_t unit_bytes() { return 32u * row_unit<F>(); }  // a unit in LDS
// (the last KB: where the loads of nothing land)
template <class F> constexpr uint32_t lds_bytes() { return PART_BYTES + F::SLOTS * unit_bytes<F>() + KEPT * 1024u + 64u + 1024u + 512u; }
static_assert(lds_bytes<FmtQ6>() <= 160u * 1024u - 64u && lds_bytes<FmtQ8>() <= 160u * 1024u - 64u, "the ring must fit the CU's LDS");

// What a lane reads of a unit in LDS for its wave's half block: Q6_K the low nibbles of its
// positions in the four quadrants' pairs, their two-bit words, the half's scales and d; Q3_K
// the half's four sixteen-byte units.
// Q8_0: the lane's eight quants of each of the half block's eight sub-blocks, and its four scales.
template <int KIND> struct Fetched;
template <> struct Fetched<3> { qu32x4 u[4]; };
template <> struct Fetched<6> { qu32x2 ql[4], qh[2], sc; uint32_t d; };
template <> struct Fetched<8> { qu32x2 q[8], sc; };

struct Q6Args {
    MvArgs a;
    uint32_t w_bytes;    // bytes of the weights the loads may touch (they are range-checked)
    uint32_t rounds;     // 32-row tiles every workgroup takes: tiles b, b + G, ...
    uint32_t tail_base;  // units of eight rows after those: tail_base for every workgroup
    uint32_t tail_rem;   // and one more for each of the first tail_rem
    uint32_t by_die;     // workgroups renumbered die by die (the grid is a multiple of eight)
    uint32_t bias;       // 0x64646464: the bytes of two f16 1024.0 exponents, as a kernel argument
                         // so that the byte shuffles stay one instruction each
    // Rows of more than 4096 weights: `parts` workgroups share a tile, each over 2048 of its
    // columns, and leave their sums in `partial` ([part][gate, up][token of 8][output]).
    uint32_t parts;
    float *partial;
    const float *scales;  // with the RMSNorm prologue: each token's 1 / sqrt(mean(x^2) + eps)
};

__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// A 4-byte store the compiler's wait-count bookkeeping does not see as a store (with one pending
// it would make every wait for a load a wait for everything in flight).
__device__ __forceinline__ void store_apart(float *at, float v) {
    asm volatile("global_store_dword %0, %1, off\n\ts_nop 0" ::"v"(at), "v"(v) : "memory");
}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_buffer(const void *base, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, 0x00020000);
}
typedef __attribute__((address_space(3))) void *lds_ptr;
// One wave-wide load of 16 bytes a lane straight into LDS (lane l lands at dst + 16 l). The
// destination reaches the load as a bare LDS address, so the compiler keeps no dependency
// between these loads and later LDS reads; the explicit waits and barriers order them.
__device__ __forceinline__ void load_lds_b128(__amdgpu_buffer_rsrc_t buf, uint32_t dst, uint32_t voffset) {
    asm volatile("" : "+s"(dst));
    __builtin_amdgcn_raw_ptr_buffer_load_lds(buf, (lds_ptr)(uintptr_t)dst, 16, voffset, 0, 0, 0);
}

// Eight quants, a byte each in two words, as the exact f16 values q - 32 (Q6_K) or q - 4 (Q3_K) in position order.
template <class F>
__device__ __forceinline__ qf16x8 weights_f16(qu32x2 q, uint32_t bias) {
    const qf16x2 off = {(_Float16)F::OFFSET, (_Float16)F::OFFSET};
    qu32x4 r;
#pragma unroll
    for (int i = 0; i < 2; i++) {
        // bytes (low to high) q0 0x64 q1 0x64: the f16 pair (1024 + q0, 1024 + q1); then q2, q3
        const uint32_t lo = __builtin_amdgcn_perm(bias, q[i], 0x04010400u), hi = __builtin_amdgcn_perm(bias, q[i], 0x04030402u);
        r[2 * i] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(qf16x2, lo) + off);
        r[2 * i + 1] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(qf16x2, hi) + off);
    }
    return __builtin_bit_cast(qf16x8, r);
}

// NU: units of a tile (k = 1024 NU).
// FEW: at most four tokens, whose eight rows then leave every lane four results instead of eight.
// LONG (NU = 2): k = 2048 q.parts; workgroup i multiplies columns 2048 (i % parts) .. (part
// `kpart`) of the tiles that walker i / parts takes, and launch_matvec_parts_sum adds the parts.
template <class F, int NU, bool FEW, bool LONG>
__global__ __launch_bounds__(THREADS) void matvec_kquant_mfma_stream_kernel(Q6Args q) {
    static_assert(!LONG || NU == 2, "parts of a long row are 2048 columns");
    constexpr uint32_t ROW_UNIT = row_unit<F>(), UNIT = unit_bytes<F>();
    constexpr int LOADS = F::LOADS, SLOTS = F::SLOTS;
    const MvArgs &a = q.a;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    float *lds_part = reinterpret_cast<float *>(lds);
    uint8_t *ring = lds + PART_BYTES;
    float *lds_kept = reinterpret_cast<float *>(lds + PART_BYTES + SLOTS * UNIT);  // [tile % KEPT][token][row]
    float *lds_inverse = lds_kept + KEPT * 256u;                                 // [token]
    const uint32_t ring0 = (uint32_t)(uintptr_t)ring;
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const __amdgpu_buffer_rsrc_t wbuf = make_buffer(a.w, q.w_bytes), nobuf = make_buffer(a.w, 0);
    uint32_t bias = q.bias;
    asm volatile("" : "+v"(bias));

    // The workgroup's tiles: b, b + G, ... and its share of the rows after the whole rounds.
    const uint32_t kpart = LONG ? blockIdx.x % q.parts : 0u, walker = LONG ? blockIdx.x / q.parts : blockIdx.x;
    const uint32_t G = LONG ? gridDim.x / q.parts : gridDim.x;
    const uint32_t b = q.by_die ? (walker & 7u) * (G >> 3) + (walker >> 3) : walker;
    const uint32_t tail_units = q.tail_base + (b < q.tail_rem ? 1u : 0u);
    const uint32_t tail_row = 32u * q.rounds * G + 8u * (b * q.tail_base + (b < q.tail_rem ? b : q.tail_rem));
    // With SILU_PAIR (src/kernels/matvec_quant.wgsl.hbs:110-125) an output tile is two weight
    // tiles, the gate rows and then the up rows `half` further down: tile p of the run is weight
    // tile p % per of output tile p / per.
    const uint32_t per = (a.flags & FLAG_SILU_PAIR) ? 2u : 1u;
    const uint32_t count = per * (q.rounds + (tail_units ? 1u : 0u));
    auto out_row = [&](uint32_t po) { return po < q.rounds ? 32u * (b + po * G) : tail_row; };  // first output of output tile po
    auto out_rows = [&](uint32_t po) { return po < q.rounds ? 32u : 8u * tail_units; };
    auto first_row = [&](uint32_t p) { return out_row(p / per) + ((p % per) ? a.half : 0u); };
    auto rows_of = [&](uint32_t p) { return out_rows(p / per); };

    // A unit's loads. The unit is 224 lines, row after row; load g = 4 wave + j brings lines
    // 8 g .. 8 g + 7 (the eighth wave's four would be past the unit's end: they go against an
    // empty buffer, so that every wave's waits count the same loads), lane l line 8 g + l / 8
    // and the chunk that belongs at position l % 8 of it. The whole address is the lane's
    // offset, which is what the buffer's range check sees: rows past the matrix's end land as zeros.
    uint32_t woff[LOADS];
#pragma unroll
    for (int j = 0; j < LOADS; j++) {
        const uint32_t line = 8u * (LOADS * wave + j) + (lane >> 3), row = line / F::ROW_LINES, in_row = line % F::ROW_LINES;
        // (a flat tile: line after line of the stretch, chunk c of line l at position c ^ (l % 8))
        woff[j] = F::FLAT ? 128u * line + 16u * ((lane & 7u) ^ (line & 7u)) : row * a.row_bytes + 128u * in_row + 16u * ((lane & 7u) ^ (row & 7u));
    }
    // Unit v of the run: unit v % NU of tile v / NU. Past the run's end the loads still run, so
    // that the waits count the same loads every step, but against an empty buffer: zeros land
    // and nothing is fetched.
    auto issue = [&](uint32_t v, uint32_t slot) __attribute__((always_inline)) {
        const uint32_t p = v / NU, u = v % NU;
        const bool real = p < count && wave < F::LOADERS;
        const uint32_t base = (real ? first_row(p) : 0u) * a.row_bytes + ROW_UNIT * (NU * kpart + u), rows = rows_of(p);
        // (a load against the empty buffer still lands zeros: the eighth wave's in a spare KB)
        const uint32_t dst = wave < F::LOADERS ? ring0 + slot * UNIT + 1024u * (LOADS * wave) : ring0 + SLOTS * UNIT + KEPT * 1024u + 64u;
#pragma unroll
        for (int j = 0; j < LOADS; j++) {
            // (lines of rows the workgroup's share of the last rows does not have are not fetched;
            // what the matrix instructions make of the zeros there is never stored)
            const uint32_t g = LOADS * wave + j;
            const uint32_t first_line_row = F::FLAT ? (1024u * g) / ROW_UNIT : (8u * g) / F::ROW_LINES;
            const bool within = 1024u * g < UNIT;  // (the flat tile's last load slot is past its end)
            load_lds_b128(real && within && first_line_row < rows ? wbuf : nobuf, wave < F::LOADERS && within ? dst + 1024u * j : ring0 + SLOTS * UNIT + KEPT * 1024u + 64u, woff[j] + base);
        }
    };

    // The tokens' operands. Wave w multiplies half w % 2 (sub-blocks 8 (w % 2) .. + 7, 128
    // positions) of block w / 2 of every unit: positions 1024 u + 128 w ... of the tokens, which
    // the wave prepares for itself with every lane at work (token lane / 8, sixteen bytes a lane
    // and step). What has to be known before anything can be rounded comes first: with the
    // RMSNorm prologue the tokens' sums of squares, then each token's largest magnitude as the
    // multiply sees it (src/kernels/matvec_quant.wgsl.hbs:73-89: RMSNorm times the norm weights
    // and / or silu(x / act_div), in the default variant's arithmetic); the waves' parts meet in
    // LDS and are combined in the order of the waves. The first unit's loads go out between the
    // inputs' loads and this arithmetic (loads complete in order within a wave), the next three
    // once the inputs are in: all four at once would hold up the other waves' inputs in the
    // CU's one address pipeline (+0.7 us).
    // (the sum of squares of a long row is not any one workgroup's: it comes ready in q.scales)
    const bool norm = (a.flags & FLAG_NORM) != 0, act = a.act_div > 0.f;
    float *lds_max = lds_inverse + 16 + 256, *lds_ss = lds_max + 64;  // [wave][token], behind the spare KB
    // Operand row r of the matrix instruction is piece r / 8 of token 4 (r / 4 % 2) + r % 4 (rows
    // 16 .. 31 are zeros), so that a lane's results are its weight row times both pieces of four
    // tokens: piece 0 the f16 rounding of the scaled inputs, piece 1 what that left times 2^11.
    // With at most four tokens row r is piece r / 4 of token r % 4 (rows 8 .. 31 are zeros): the
    // lower half of the lanes gets its weight row times the tokens' first pieces, the upper half
    // times their second pieces. Either way a piece's sums are accumulated apart and a wave's
    // two meet once a tile, by the same operations: a token's result does not depend on which
    // of the two layouts its launch used. The lane's eight positions of sub-block s of its
    // wave's half block are 16 s + 8 (lane / 32) ...
    const uint32_t rho = lane & 31u, kap = lane >> 5;
    const uint32_t tok = FEW ? rho & 3u : 4u * ((rho >> 2) & 1u) + (rho & 3u), piece = FEW ? rho >> 2 : rho >> 3;
    const bool live = tok < a.m && piece < 2u;
    qf16x8 xf[8 * NU];
    {
        // (an absent token's lanes ask past the buffer's end: zeros, and nothing is fetched)
        const uint32_t t1 = lane >> 3, l8 = lane & 7u, t1c = t1 < a.m ? t1 : a.m - 1u;
        float4 r1[4 * NU], g1[4 * NU];
        const __amdgpu_buffer_rsrc_t xbuf = make_buffer(a.x, ((a.m - 1u) * a.xr + a.k) * 4u);
        const uint32_t x1 = (t1 * a.xr + 1024u * NU * kpart + 128u * wave + 4u * l8) * 4u;
#pragma unroll
        for (int u = 0; u < NU; u++)
#pragma unroll
            for (int i = 0; i < 4; i++)
                r1[4 * u + i] = __builtin_bit_cast(float4, __builtin_amdgcn_raw_buffer_load_b128(xbuf, t1 < a.m ? x1 + 4u * (1024u * u + 32u * i) : 0xfffffff0u, 0, 0));
        float ready = 0.f;  // (asked for before the first weights, like the inputs)
        if (norm) {
            const float *gp = a.norm_w + 1024u * NU * kpart + 128u * wave + 4u * l8;
#pragma unroll
            for (int u = 0; u < NU; u++)
#pragma unroll
                for (int i = 0; i < 4; i++) g1[4 * u + i] = *reinterpret_cast<const float4 *>(gp + 1024 * u + 32 * i);
            if (LONG) ready = q.scales[t1c];
        }
        issue(0, 0);
        if (norm) {
            float rs;
            if (LONG) {
                rs = ready;
            } else {
                float ss = 0.f;
#pragma unroll
                for (int i = 0; i < 4 * NU; i++) ss += r1[i].x * r1[i].x + r1[i].y * r1[i].y + r1[i].z * r1[i].z + r1[i].w * r1[i].w;
                ss += __shfl_xor(ss, 1, 64);
                ss += __shfl_xor(ss, 2, 64);
                ss += __shfl_xor(ss, 4, 64);
                if (l8 == 0u) lds_ss[8u * wave + t1] = ss;
                lds_barrier();
                float total = lds_ss[t1];
#pragma unroll
                for (uint32_t wv = 1; wv < WAVES; wv++) total += lds_ss[8u * wv + t1];
                rs = 1.0f / sqrtf(total / (float)a.k + a.eps);
            }
#pragma unroll
            for (int i = 0; i < 4 * NU; i++) {
                r1[i].x = r1[i].x * rs * g1[i].x; r1[i].y = r1[i].y * rs * g1[i].y;
                r1[i].z = r1[i].z * rs * g1[i].z; r1[i].w = r1[i].w * rs * g1[i].w;
            }
        }
        if (act) {
#pragma unroll
            for (int i = 0; i < 4 * NU; i++) {
                r1[i].x = silu_f(r1[i].x / a.act_div); r1[i].y = silu_f(r1[i].y / a.act_div);
                r1[i].z = silu_f(r1[i].z / a.act_div); r1[i].w = silu_f(r1[i].w / a.act_div);
            }
        }
        float big = 0.f;
#pragma unroll
        for (int i = 0; i < 4 * NU; i++) big = fmaxf(fmaxf(fabsf(r1[i].x), fabsf(r1[i].y)), fmaxf(fmaxf(fabsf(r1[i].z), fabsf(r1[i].w)), big));
        big = fmaxf(big, __shfl_xor(big, 1, 64));
        big = fmaxf(big, __shfl_xor(big, 2, 64));
        big = fmaxf(big, __shfl_xor(big, 4, 64));
        if (l8 == 0u) lds_max[8u * wave + t1] = big;
        lds_barrier();
#pragma unroll
        for (int v = 1; v < SLOTS; v++) issue(v, v);
        // Each token's scale: the power of two that puts its largest magnitude in [2^14, 2^15).
        auto scale_of = [&](uint32_t t, bool inverse) {
            float most = lds_max[t];
#pragma unroll
            for (uint32_t wv = 1; wv < WAVES; wv++) most = fmaxf(most, lds_max[8u * wv + t]);
            const int e = (int)((__float_as_uint(most) >> 23) & 0xffu);  // biased exponent; 0 for zero and subnormals
            int se = 127 + 14 - (e - 127);                                // scale = 2^(14 - (e - 127)), kept normal both ways
            se = se < 1 ? 1 : se > 253 ? 253 : se;
            if (e == 0 || e == 255) return 1.0f;
            return __uint_as_float((uint32_t)(inverse ? 254 - se : se) << 23);
        };
        if (tid < 8u) lds_inverse[tid] = tid < a.m ? scale_of(tid, true) : 1.0f;  // read behind later barriers
        const float scale = scale_of(t1c, false);
        // From this layout to the operands' through 4 KB of LDS a wave, a unit's 128 positions at
        // a time: [piece][token][position] f16 (the space of the partial sums and of the kept
        // outputs, neither in use yet). A wave's LDS operations complete in order, and nobody
        // else touches its 4 KB: no barrier.
        uint8_t *stage = wave < 4u ? lds + 4096u * wave : reinterpret_cast<uint8_t *>(lds_kept) + 4096u * (wave - 4u);
        // (sixteen-byte chunk c of row r sits at position c ^ r: the sixteen rows' reads of one chunk fall on sixteen different banks)
        const uint32_t row = (piece & 1u) * 8u + tok;
        typedef _Float16 h4 __attribute__((ext_vector_type(4)));
#pragma unroll
        for (int u = 0; u < NU; u++) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const float x[4] = {r1[4 * u + i].x, r1[4 * u + i].y, r1[4 * u + i].z, r1[4 * u + i].w};
                _Float16 hi[4], lo[4];
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    // The scale is a power of two, so x * scale - hi in one fused operation is exact.
                    hi[e] = (_Float16)(x[e] * scale);
                    lo[e] = (_Float16)(fmaf(x[e], scale, -(float)hi[e]) * 2048.0f);
                }
                // (an absent token's inputs are zeros, or what its lanes make of them: its rows of the layout are never read)
                const qu32x2 h2 = __builtin_bit_cast(qu32x2, h4{hi[0], hi[1], hi[2], hi[3]}), l2 = __builtin_bit_cast(qu32x2, h4{lo[0], lo[1], lo[2], lo[3]});
                const uint32_t chunk = (l8 >> 1) + 4u * i, within = 8u * (l8 & 1u);
                *reinterpret_cast<qu32x2 *>(stage + t1 * 256u + 16u * (chunk ^ t1) + within) = h2;
                *reinterpret_cast<qu32x2 *>(stage + (8u + t1) * 256u + 16u * (chunk ^ (8u + t1)) + within) = l2;
            }
            asm volatile("" ::: "memory");
#pragma unroll
            for (int s = 0; s < 8; s++) xf[8 * u + s] = qf16x8{0, 0, 0, 0, 0, 0, 0, 0};
            if (live) {  // (the other lanes stay out of the reads: half of the LDS traffic)
#pragma unroll
                for (int s = 0; s < 8; s++)
                    xf[8 * u + s] = __builtin_bit_cast(qf16x8, *reinterpret_cast<const qu32x4 *>(stage + row * 256u + 16u * ((2u * s + kap) ^ row)));
            }
            asm volatile("" ::: "memory");
        }
    }

    // The lane's reads of its wave's half block of a unit: row rho of the flat copy, the block's
    // bytes at 224 (wave / 2). Byte o of a row's unit sits at 896 rho + 128 (o / 128) +
    // 16 ((o / 16 % 8) ^ (rho % 8)) + o % 16.
    const uint32_t blk = wave >> 1, half = wave & 1u;
    auto at_byte = [&](uint32_t o) {
        const uint32_t f = ROW_UNIT * rho + o;  // (flat: the byte's place in the tile)
        return F::FLAT ? (f & ~127u) + 16u * (((f >> 4) & 7u) ^ ((f >> 7) & 7u)) + (f & 15u)
                       : ROW_UNIT * rho + (o & ~127u) + 16u * (((o >> 4) & 7u) ^ (rho & 7u)) + (o & 15u);
    };
    constexpr int KIND = F::KIND;
    constexpr bool Q3 = KIND == 3;
    uint32_t at_ql[4], at_qh[2];  // Q6_K ql: [which 32 of the half's 64][which 16]; qh: [which 16]; Q3_K: at_ql = the half's four units
    uint32_t at_sc = 0, at_d = 0, at_q8[8];
    if constexpr (KIND == 8) {
        // (the wave's 128 positions are four blocks of 32: sub-block s lies in block 4 wave + s / 2)
#pragma unroll
        for (uint32_t i = 0; i < 8; i++) at_q8[i] = at_byte(128u * wave + 16u * i + 8u * kap);
        at_sc = at_byte(1024u + 8u * wave);
        at_ql[0] = at_qh[0] = 0;
    } else if constexpr (Q3) {
#pragma unroll
        for (uint32_t i = 0; i < 4; i++) at_ql[i] = at_byte(128u * blk + 64u * half + 16u * i);
        at_qh[0] = at_qh[1] = 0;
    } else {
#pragma unroll
        for (uint32_t i = 0; i < 4; i++) at_ql[i] = at_byte(224u * blk + 64u * half + 32u * (i >> 1) + 16u * (i & 1u) + 8u * kap);
#pragma unroll
        for (uint32_t i = 0; i < 2; i++) at_qh[i] = at_byte(224u * blk + 128u + 32u * half + 16u * i + 8u * kap);
        at_sc = at_byte(224u * blk + 192u + 8u * half);
        at_d = at_byte(224u * blk + 208u);
    }

    // Matrix row rho of the tile, this wave's blocks: piece 0 (acc) and piece 1 (acc_lo) of tokens
    // 4 (lane / 32) + i; with at most four tokens piece lane / 32 of token i in acc.
    float acc[4] = {0.f, 0.f, 0.f, 0.f}, acc_lo[4] = {0.f, 0.f, 0.f, 0.f};
    // The lane's part of the unit in `slot`, from LDS to registers.
    auto fetch = [&](uint32_t slot) __attribute__((always_inline)) {
        const uint8_t *t = ring + slot * UNIT;
        Fetched<KIND> f;
        if constexpr (KIND == 8) {
#pragma unroll
            for (uint32_t i = 0; i < 8; i++) f.q[i] = *reinterpret_cast<const qu32x2 *>(t + at_q8[i]);
            f.sc = *reinterpret_cast<const qu32x2 *>(t + at_sc);
        } else if constexpr (Q3) {
#pragma unroll
            for (uint32_t i = 0; i < 4; i++) f.u[i] = *reinterpret_cast<const qu32x4 *>(t + at_ql[i]);
        } else {
#pragma unroll
            for (uint32_t i = 0; i < 4; i++) f.ql[i] = *reinterpret_cast<const qu32x2 *>(t + at_ql[i]);
#pragma unroll
            for (uint32_t i = 0; i < 2; i++) f.qh[i] = *reinterpret_cast<const qu32x2 *>(t + at_qh[i]);
            f.sc = *reinterpret_cast<const qu32x2 *>(t + at_sc);
            f.d = *reinterpret_cast<const uint16_t *>(t + at_d);
        }
        return f;
    };
    // Sub-block s (of the eight of the wave's half block) of a fetched unit, made ready for the
    // matrix instruction: the lane's eight quants as f16, and d * scale.
    auto prepare = [&](const Fetched<KIND> &f, int s, qf16x8 &wf, float &dsc) __attribute__((always_inline)) {
        qu32x2 v;
        if constexpr (KIND == 8) {
            // (signed bytes: with the top bit turned they are q + 128)
            v[0] = f.q[s][0] ^ 0x80808080u;
            v[1] = f.q[s][1] ^ 0x80808080u;
            const uint32_t word = s < 4 ? f.sc.x : f.sc.y;
            dsc = half_bits_to_float((s & 2) ? word >> 16 : word & 0xffffu);
        } else if constexpr (Q3) {
            // Unit i of the half: 32 weights as two words of 2-bit values (byte b, bit pair e:
            // position 4 e + b; the second word 16 further), a word of third bits (byte b, bit e:
            // position 4 e + b), scale - 32 of each sixteen as signed bytes, d. The lane's eight
            // positions of a sixteen are 8 kap ..: bit pairs 2 kap and 2 kap + 1 of the four bytes.
            const uint32_t h16 = (uint32_t)s & 1u;
            const qu32x4 u = f.u[s >> 1];
            const uint32_t word = h16 ? u.y : u.x, third = u.z >> (4u * h16 + 2u * kap);
            v[0] = ((word >> (4u * kap)) & 0x03030303u) | ((third & 0x01010101u) << 2);
            v[1] = ((word >> (4u * kap + 2u)) & 0x03030303u) | (((third >> 1) & 0x01010101u) << 2);
            dsc = half_bits_to_float(u.w >> 16) * (float)(int8_t)((u.w >> (8u * h16)) & 0xffu);
        } else {
            // Quadrant qd of the half: weights 32 qd + 16 h16 + 8 kap ... of its 128; s = 2 qd + h16.
            const uint32_t h16 = (uint32_t)s & 1u, qd = (uint32_t)s >> 1, qp = qd & 1u, up = qd >> 1;
            const qu32x2 ql = f.ql[2u * qp + h16], qh = f.qh[h16];
#pragma unroll
            for (int w = 0; w < 2; w++) {
                const uint32_t nib = up ? (ql[w] >> 4) & 0x0f0f0f0fu : ql[w] & 0x0f0f0f0fu;
                const uint32_t two = (qd ? qh[w] >> (2u * qd) : qh[w]) & 0x03030303u;
                v[w] = nib | (two << 4);
            }
            const uint32_t word = s < 4 ? f.sc.x : f.sc.y;
            dsc = half_bits_to_float(f.d) * (float)(int8_t)((word >> (8u * ((uint32_t)s & 3u))) & 0xffu);
        }
        wf = weights_f16<F>(v, bias);
    };
    // A unit's eight matrix instructions. The vector work of a sub-block is made to surround the
    // matrix instruction of the one before it: while that runs, the next sub-block is unpacked
    // (the last one's successor is the first of the unit after, which is in registers by then),
    // and only then are its results scaled and added. The scheduler is kept from moving anything
    // across these lines: left to itself it puts each matrix instruction right before the
    // additions that wait for it.
    qf16x8 wf;
    float dsc;
    auto multiply = [&](auto unit, const Fetched<KIND> &f, const Fetched<KIND> &after) __attribute__((always_inline)) {
        constexpr int U = decltype(unit)::value;
        qf32x16 zero;
#pragma unroll
        for (int e = 0; e < 16; e++) zero[e] = 0.f;
#pragma unroll
        for (int s = 0; s < 8; s++) {
            const qu32x4 running = __builtin_bit_cast(qu32x4, wf);
            const qf32x16 r = __builtin_amdgcn_mfma_f32_32x32x16_f16(xf[8 * U + s], wf, zero, 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            const float scale = dsc;
            if (s < 7) prepare(f, s + 1, wf, dsc);
            else prepare(after, 0, wf, dsc);
            // (the running instruction's operand and all sixteen of its results stay where they
            // are: a write to any of them would have to wait for the matrix core)
            asm volatile("" ::"v"(running), "v"(r));
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                acc[i] = fmaf(scale, r[i], acc[i]);
                if (!FEW) acc_lo[i] = fmaf(scale, r[4 + i], acc_lo[i]);
            }
            // (and a sub-block's results are used up before the next matrix instruction: eight of
            // them in flight would not fit the registers)
            asm volatile("" : "+v"(acc[0]), "+v"(acc[1]), "+v"(acc[2]), "+v"(acc[3]));
            if (!FEW) asm volatile("" : "+v"(acc_lo[0]), "+v"(acc_lo[1]), "+v"(acc_lo[2]), "+v"(acc_lo[3]));
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    // A finished tile's partial sums into LDS; they are added behind the next barrier.
    auto hand_over = [&](uint32_t p) __attribute__((always_inline)) {
        float *part = lds_part + (p & 1u) * (WAVES * 256u);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            part[wave * 256u + 64u * i + lane] = FEW ? acc[i] : fmaf(acc_lo[i], 1.0f / 2048.0f, acc[i]);
            acc[i] = acc_lo[i] = 0.f;
        }
    };
    // (a wave sums tokens i and 4 + i, whose partial sums lie side by side: no two lanes on a bank)
    float held = 0.f;  // the gate tile's result, until the up tile's arrives
    // What waits in lds_kept for the burst of stores: an output tile's results, or (LONG, where
    // the epilogue is the sums' launch's) every weight tile's sums, the gate tile's and the up tile's.
    const uint32_t kper = LONG ? 1u : per;  // weight tiles an entry stands for
    auto sum_up = [&](uint32_t p) __attribute__((always_inline)) {
        const uint32_t po = p / per;
        if ((tid >> 8) != (po & 1u)) return;  // (the same half of the workgroup for an output tile's two weight tiles)
        const float *part = lds_part + (p & 1u) * (WAVES * 256u);
        const uint32_t row = tid & 31u, tk = 4u * ((tid >> 5) & 1u) + ((tid >> 6) & 3u);
        if (FEW && tk >= 4u) return;
        const float *src = part + 64u * (tk & 3u) + 32u * (tk >> 2) + row;
        // (with at most four tokens a wave's two pieces still lie apart, 32 floats from each other)
        auto of_wave = [&](uint32_t wv) { return FEW ? fmaf(src[wv * 256u + 32u], 1.0f / 2048.0f, src[wv * 256u]) : src[wv * 256u]; };
        float total = of_wave(0);
#pragma unroll
        for (uint32_t wv = 1; wv < WAVES; wv++) total += of_wave(wv);
        total *= lds_inverse[tk];
        if (!LONG && per == 2u && !(p & 1u)) held = total;
        else lds_kept[256u * ((p / kper) % KEPT) + 32u * tk + row] = (!LONG && per == 2u) ? silu_f(held) * total : total;
    };
    // Entries first .. first + n - 1 from LDS to memory in one burst: 128 contiguous bytes a
    // token and tile.
    auto store_kept = [&](uint32_t first, uint32_t n) __attribute__((always_inline)) {
        lds_barrier();
        for (uint32_t e = first + (tid >> 8); e < first + n; e += 2u) {
            const uint32_t po = LONG ? e / per : e, which = LONG ? e % per : 0u;
            const uint32_t row = tid & 31u, tk = (tid >> 5) & 7u;
            const uint32_t j = out_row(po) + row;
            if (tk < a.m && row < out_rows(po) && j < a.rows) {
                float *o = a.out + (size_t)tk * a.out_stride + a.col0 + j;
                const float total = lds_kept[256u * (e % KEPT) + (tid & 255u)];
                if (LONG) store_apart(q.partial + ((size_t)(per * kpart + which) * 8u + tk) * a.rows + j, total);
                else store_apart(o, (a.flags & FLAG_ACCUMULATE) ? *o + total : total);
            }
        }
    };

    // One barrier a unit: behind the barrier of unit v's step all of unit v + 1 has landed (every
    // wave has waited for its own loads of it; those of the two units after it stay in flight),
    // every wave has unit v in registers, so its slot takes the loads of unit v + 4, and the
    // tile before's partial sums are in LDS. A wave reads unit v + 1 into registers while it
    // multiplies unit v: no multiply waits for LDS.
    Fetched<KIND> cur;
    auto step = [&](uint32_t p, auto unit) __attribute__((always_inline)) {
        constexpr int U = decltype(unit)::value;
        const uint32_t v = NU * p + U;
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"((SLOTS - 2) * LOADS) : "memory");
        lds_barrier();
        issue(v + SLOTS, v % SLOTS);
        const Fetched<KIND> next = fetch((v + 1u) % SLOTS);
        asm volatile("" ::: "memory");  // (the reads go out here, not where the next step uses them)
        if (U == 0 && p > 0u) {
            sum_up(p - 1u);
            // (the next tile's sums are kept only behind a later barrier, which no thread passes
            // before it has stored what it stores here)
            if (p % (kper * KEPT) == 0u) store_kept(p / kper - KEPT, KEPT);
        }
        multiply(unit, cur, next);
        cur = next;
    };
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"((SLOTS - 1) * LOADS) : "memory");
    lds_barrier();
    cur = fetch(0);
    prepare(cur, 0, wf, dsc);
    for (uint32_t p = 0; p < count; p++) {
        step(p, std::integral_constant<int, 0>{});
        if constexpr (NU >= 2) step(p, std::integral_constant<int, 1>{});
        if constexpr (NU >= 3) step(p, std::integral_constant<int, 2>{});
        if constexpr (NU >= 4) step(p, std::integral_constant<int, 3>{});
        hand_over(p);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // nothing may still land in LDS once the workgroup is gone
    if (count > 0u) {
        lds_barrier();
        sum_up(count - 1u);
        const uint32_t last = count / kper - 1u;  // the run's last entry
        store_kept(last - last % KEPT, last % KEPT + 1u);
    }
}

template <class F, int NU, bool FEW, bool LONG = false>
zhip_result launch_blocks(const Dispatch &d, const Q6Args &q, dim3 grid) {
    auto kernel = matvec_kquant_mfma_stream_kernel<F, NU, FEW, LONG>;
    constexpr uint32_t bytes = lds_bytes<F>();
    static bool configured = false;
    if (!configured) {
        if (hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess) {
            (void)hipGetLastError();
            return fail(d, ZHIP_E_GPU, "%s: cannot reserve %u bytes of LDS", F::name(), bytes);
        }
        configured = true;
    }
    hipLaunchKernelGGL(kernel, grid, dim3(THREADS), bytes, d.stream, q);
    return check_launch(d, F::name());
}

template <class F>
zhip_result launch_stream(const Dispatch &d, const MvArgs &a, uint64_t w_bytes) {
    // 32-bit byte offsets, a tile past the last row.
    const uint64_t used = ((uint64_t)((a.flags & FLAG_SILU_PAIR) ? a.half : 0u) + a.rows) * a.row_bytes;
    if (used + 64ull * a.row_bytes >= 0xfffffff0ull) return fail(d, ZHIP_E_BAD_COMMAND, "%s: weights of 4 GiB or more", F::name());
    // The workgroups that walk the tiles: one a CU, or (rows of more than 4096 weights) one for
    // every `parts` CUs, each of them `parts` workgroups.
    const uint32_t parts = a.k > 4096u ? a.k / 2048u : 1u;
    const uint32_t cus = (uint32_t)d.dev->compute_units;
    if (cus < parts) return fail(d, ZHIP_E_GPU, "%s: %u compute units for %u parts of a row", F::name(), cus, parts);
    const uint32_t units = (a.rows + 7u) / 8u, most = cus / parts;
    const uint32_t groups = units < most ? units : most;
    const uint32_t rounds = (a.rows / 32u) / groups;
    const uint32_t tail = (a.rows - 32u * rounds * groups + 7u) / 8u;
    Q6Args q{a, (uint32_t)(used < w_bytes ? used : w_bytes), rounds, tail / groups, tail % groups, groups % 8u == 0 ? 1u : 0u, 0x64646464u, parts, nullptr, nullptr};
    const dim3 grid(groups * parts);
    if constexpr (!F::FLAT) {
        if (parts > 1u) {
            if (!d.work) return fail(d, ZHIP_E_GPU, "%s: no workspace", F::name());
            if (zhip_result r = d.work->reserve(d, kPartsScalesBytes + (uint64_t)parts * ((a.flags & FLAG_SILU_PAIR) ? 2u : 1u) * 8u * a.rows * sizeof(float))) return r;
            q.partial = reinterpret_cast<float *>(d.work->data + kPartsScalesBytes);
            if (a.flags & FLAG_NORM) {
                q.scales = reinterpret_cast<const float *>(d.work->data);
                if (zhip_result r = launch_matvec_parts_scales(d, F::name(), a, reinterpret_cast<float *>(d.work->data))) return r;
            }
            if (zhip_result r = a.m <= 4u ? launch_blocks<F, 2, true, true>(d, q, grid) : launch_blocks<F, 2, false, true>(d, q, grid)) return r;
            return launch_matvec_parts_sum(d, F::name(), a, q.partial, parts);
        }
    }
    if constexpr (F::FLAT) {  // (the unit is the whole row: k = 1024 only)
        return a.m <= 4u ? launch_blocks<F, 1, true>(d, q, grid) : launch_blocks<F, 1, false>(d, q, grid);
    } else {
    if (a.m <= 4u)
        return a.k == 1024u ? launch_blocks<F, 1, true>(d, q, grid) : a.k == 2048u ? launch_blocks<F, 2, true>(d, q, grid)
             : a.k == 3072u ? launch_blocks<F, 3, true>(d, q, grid) : launch_blocks<F, 4, true>(d, q, grid);
    return a.k == 1024u ? launch_blocks<F, 1, false>(d, q, grid) : a.k == 2048u ? launch_blocks<F, 2, false>(d, q, grid)
         : a.k == 3072u ? launch_blocks<F, 3, false>(d, q, grid) : launch_blocks<F, 4, false>(d, q, grid);
    }
}

// k of 1024, 2048, 3072 or 4096, or 6144 .. 32768 in parts of 2048.
bool stream_accepts(const MvArgs &a, uint32_t block_bytes) {
    const bool parts = a.k > 4096u && a.k % 2048u == 0 && a.k / 2048u <= kMatvecMaxParts;
    return a.m >= 1 && a.m <= 8 && (a.k == 1024u || a.k == 2048u || a.k == 3072u || a.k == 4096u || parts) && a.rows >= 1 && a.xr % 4u == 0 &&
           (reinterpret_cast<uintptr_t>(a.x) & 15u) == 0 && (reinterpret_cast<uintptr_t>(a.w) & 15u) == 0 && a.row_bytes == a.k / 256u * block_bytes;
}

}  // namespace

// Whether these kernels can run the (already validated) arguments: k of whole units.
bool matvec_q6k_mfma_stream_accepts(const MvArgs &a) { return stream_accepts(a, FmtQ6::BLOCK); }
zhip_result launch_matvec_q6k_mfma_stream(const Dispatch &d, const MvArgs &a, uint64_t w_bytes) { return launch_stream<FmtQ6>(d, a, w_bytes); }
// Q8_0: rows of 1024 weights only (longer ones stay with the kernels that keep a tile resident).
bool matvec_q8_0_mfma_flat_accepts(const MvArgs &a) { return a.k == 1024u && stream_accepts(a, FmtQ8::BLOCK); }
zhip_result launch_matvec_q8_0_mfma_flat(const Dispatch &d, const MvArgs &a, uint64_t w_bytes) { return launch_stream<FmtQ8>(d, a, w_bytes); }
bool matvec_q3k_mfma_stream_accepts(const MvArgs &a) { return stream_accepts(a, FmtQ3::BLOCK); }
zhip_result launch_matvec_q3k_mfma_stream(const Dispatch &d, const MvArgs &a, uint64_t w_bytes) { return launch_stream<FmtQ3>(d, a, w_bytes); }

}  // namespace zhip
