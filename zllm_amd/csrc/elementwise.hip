// The small kernels either side of the multiplies: split-k reduction, the
// prefill SwiGLU, load-time weight layouts, embedding gathers (which also
// expose the block decoders bit for bit), RMSNorm and buffer fills. All are
// bandwidth-trivial grid-stride kernels; each keeps its reference kernel's
// parameter block, bindings and arithmetic.
#include <hip/hip_runtime.h>

#include "common.h"
#include "decode.h"

namespace zhip {

static inline uint32_t blocks_for(uint64_t items, uint32_t per_block, uint32_t cap) {
    uint64_t b = (items + per_block - 1) / per_block;
    if (b < 1) b = 1;
    return (uint32_t)(b < cap ? b : cap);
}

// Threads a folded elementwise grid covers (Launcher.elementwise,
// src/kernels/kernels.zig:985-991): x * y workgroups of 256.
static inline uint64_t elementwise_cover(const Dispatch &d) { return (uint64_t)d.grid[0] * d.grid[1] * 256u; }

// ---- matmul_reduce: src/kernels/matmul_reduce.wgsl -----------------------------
__global__ __launch_bounds__(256) void matmul_reduce_kernel(MatmulReduceParams p, const float *parts, float *out, uint64_t count) {
    for (uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x; i < count; i += (uint64_t)gridDim.x * 256u) {
        const uint32_t t = (uint32_t)(i / p.n), j = (uint32_t)(i % p.n);
        float sum = 0.f;
        for (uint32_t s = 0; s < p.slices; s++) sum += parts[(size_t)s * p.slice_stride + i];
        const size_t o = (size_t)t * p.out_stride + p.col0 + j;
        out[o] = p.accumulate ? out[o] + sum : sum;
    }
}

zhip_result launch_matmul_reduce(const Dispatch &d) {
    if (d.params_size < sizeof(MatmulReduceParams)) return fail(d, ZHIP_E_BAD_COMMAND, "matmul_reduce: params block too small");
    const MatmulReduceParams &p = *reinterpret_cast<const MatmulReduceParams *>(d.params);
    if (!d.bind[1].bound || !d.bind[2].bound) return fail(d, ZHIP_E_BAD_COMMAND, "matmul_reduce: bindings 1 and 2 must be bound");
    uint64_t count = (uint64_t)p.rows * p.n;
    const uint64_t cover = elementwise_cover(d);
    if (cover < count) count = cover;
    if (count == 0) return ZHIP_OK;
    // The last element read and written.
    const uint64_t last = count - 1, t = last / p.n;
    const uint64_t parts_need = ((uint64_t)(p.slices ? p.slices - 1 : 0) * p.slice_stride + count) * 4u;
    const uint64_t out_need = (t * p.out_stride + p.col0 + (t > 0 ? p.n : last + 1)) * 4u;
    if (parts_need > d.bind[1].size || out_need > d.bind[2].size) return fail(d, ZHIP_E_BAD_COMMAND, "matmul_reduce: bound ranges too small");
    hipLaunchKernelGGL(matmul_reduce_kernel, dim3(blocks_for(count, 256, 65536)), dim3(256), 0, d.stream, p,
        reinterpret_cast<const float *>(d.bind[1].ptr), reinterpret_cast<float *>(d.bind[2].ptr), count);
    return check_launch(d, "matmul_reduce");
}

// ---- silu_mul: src/kernels/silu_mul.wgsl ---------------------------------------
__global__ __launch_bounds__(256) void silu_mul_kernel(SiluMulParams p, const float *gu, float *act, uint64_t count) {
    for (uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x; i < count; i += (uint64_t)gridDim.x * 256u) {
        const uint64_t t = i / p.width, j = i % p.width;
        const float g = gu[t * 2u * p.width + j];
        act[i] = g / (1.0f + expf(-g)) * gu[t * 2u * p.width + p.width + j];
    }
}

zhip_result launch_silu_mul(const Dispatch &d) {
    if (d.params_size < sizeof(SiluMulParams)) return fail(d, ZHIP_E_BAD_COMMAND, "silu_mul: params block too small");
    const SiluMulParams &p = *reinterpret_cast<const SiluMulParams *>(d.params);
    if (!d.bind[1].bound || !d.bind[2].bound) return fail(d, ZHIP_E_BAD_COMMAND, "silu_mul: bindings 1 and 2 must be bound");
    uint64_t count = p.count;
    const uint64_t cover = elementwise_cover(d);
    if (cover < count) count = cover;
    if (count == 0) return ZHIP_OK;
    if (p.width == 0) return fail(d, ZHIP_E_BAD_COMMAND, "silu_mul: width 0");
    const uint64_t rows = (count + p.width - 1) / p.width;
    if (rows * 2u * p.width * 4u > d.bind[1].size || count * 4u > d.bind[2].size) return fail(d, ZHIP_E_BAD_COMMAND, "silu_mul: bound ranges too small");
    hipLaunchKernelGGL(silu_mul_kernel, dim3(blocks_for(count, 256, 65536)), dim3(256), 0, d.stream, p,
        reinterpret_cast<const float *>(d.bind[1].ptr), reinterpret_cast<float *>(d.bind[2].ptr), count);
    return check_launch(d, "silu_mul");
}

// ---- repack_q8_0: src/kernels/repack_q8_0.wgsl ---------------------------------
// One destination word per thread: four values of a block, or two scales.
__device__ __forceinline__ uint32_t src_byte(const uint8_t *src, uint64_t i) { return src[i]; }

__global__ __launch_bounds__(256) void repack_q8_0_kernel(RepackQ80Params p, const uint8_t *src, uint32_t *dst, uint64_t count) {
    const uint32_t stride = (p.k + p.k / 16u + 15u) & ~15u;
    const uint32_t words = stride / 4u, blocks = p.k / 32u;
    for (uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x; i < count; i += (uint64_t)gridDim.x * 256u) {
        const uint64_t r = i / words;
        const uint32_t o = 4u * (uint32_t)(i % words);
        const uint64_t raw = r * blocks * 34u;
        uint32_t word = 0;
        if (o < p.k) {
            const uint64_t b = raw + (uint64_t)(o / 32u) * 34u + 2u + o % 32u;
            word = src[b] | (src[b + 1] << 8) | (src[b + 2] << 16) | ((uint32_t)src[b + 3] << 24);
        } else if (o < p.k + p.k / 16u) {
            const uint32_t s = (o - p.k) / 2u;
            word = src[raw + (uint64_t)s * 34u] | (src[raw + (uint64_t)s * 34u + 1] << 8);
            if (s + 1u < blocks) word |= ((uint32_t)src[raw + (uint64_t)(s + 1) * 34u] | ((uint32_t)src[raw + (uint64_t)(s + 1) * 34u + 1] << 8)) << 16;
        }
        dst[i] = word;
    }
}

zhip_result launch_repack_q8_0(const Dispatch &d) {
    if (d.params_size < sizeof(RepackQ80Params)) return fail(d, ZHIP_E_BAD_COMMAND, "repack_q8_0: params block too small");
    const RepackQ80Params &p = *reinterpret_cast<const RepackQ80Params *>(d.params);
    if (!d.bind[1].bound || !d.bind[2].bound) return fail(d, ZHIP_E_BAD_COMMAND, "repack_q8_0: bindings 1 and 2 must be bound");
    if (p.k % 32u != 0) return fail(d, ZHIP_E_BAD_COMMAND, "repack_q8_0: k = %u is not a multiple of 32", p.k);
    const uint64_t stride = (p.k + p.k / 16u + 15u) & ~15u;
    uint64_t count = (uint64_t)p.rows * (stride / 4u);
    const uint64_t cover = elementwise_cover(d);
    if (cover < count) count = cover;
    if (count == 0) return ZHIP_OK;
    const uint64_t rows_touched = (count + stride / 4u - 1) / (stride / 4u);
    if (rows_touched * (p.k / 32u) * 34u > d.bind[1].size || count * 4u > d.bind[2].size) return fail(d, ZHIP_E_BAD_COMMAND, "repack_q8_0: bound ranges too small");
    hipLaunchKernelGGL(repack_q8_0_kernel, dim3(blocks_for(count, 256, 65536)), dim3(256), 0, d.stream, p,
        d.bind[1].ptr, reinterpret_cast<uint32_t *>(d.bind[2].ptr), count);
    return check_launch(d, "repack_q8_0");
}

// ---- repack_q3_k: src/kernels/repack_q3_k.wgsl ---------------------------------
// One thread per 16-byte unit (32 weights) of the repacked blocks.
struct RepackQ3KParams { uint32_t blocks, pad0, pad1, pad2; };

__device__ __forceinline__ uint32_t q3_scale(const uint8_t *sb, uint32_t i) {
    const uint32_t k = i % 4u, g = i / 4u;
    const uint32_t low = ((uint32_t)sb[4u * (g % 2u) + k] >> (4u * (g / 2u))) & 0xfu;
    const uint32_t high = ((uint32_t)sb[8u + k] >> (2u * g)) & 3u;
    return low | (high << 4);
}

__global__ __launch_bounds__(256) void repack_q3_k_kernel(const uint8_t *src, uint4 *dst, uint64_t units) {
    for (uint64_t unit = (uint64_t)blockIdx.x * 256u + threadIdx.x; unit < units; unit += (uint64_t)gridDim.x * 256u) {
        const uint8_t *b = src + (unit / 8u) * 110u;
        const uint32_t s = (uint32_t)(unit % 8u), half = s / 4u, j = s % 4u;
        uint32_t l0 = 0, l1 = 0, hw = 0;
        for (uint32_t l = 0; l < 32u; l++) {
            const uint32_t q = ((uint32_t)b[32u + 32u * half + l] >> (2u * j)) & 3u;
            const uint32_t h = ((uint32_t)b[l] >> (4u * half + j)) & 1u;
            const uint32_t e = l / 4u, byte = l % 4u;
            if (e < 4u) l0 |= q << (8u * byte + 2u * e);
            else l1 |= q << (8u * byte + 2u * (e - 4u));
            hw |= h << (8u * byte + e);
        }
        // scale - 32 is in [-32, 31]: as a signed byte, (scale + 224) & 0xff.
        const uint32_t sc0 = (q3_scale(b + 96, 8u * half + 2u * j) + 224u) & 0xffu;
        const uint32_t sc1 = (q3_scale(b + 96, 8u * half + 2u * j + 1u) + 224u) & 0xffu;
        const uint32_t d = (uint32_t)b[108] | ((uint32_t)b[109] << 8);
        dst[unit] = make_uint4(l0, l1, hw, sc0 | (sc1 << 8) | (d << 16));
    }
}

zhip_result launch_repack_q3_k(const Dispatch &d) {
    if (d.params_size < sizeof(RepackQ3KParams)) return fail(d, ZHIP_E_BAD_COMMAND, "repack_q3_k: params block too small");
    const RepackQ3KParams &p = *reinterpret_cast<const RepackQ3KParams *>(d.params);
    if (!d.bind[1].bound || !d.bind[2].bound) return fail(d, ZHIP_E_BAD_COMMAND, "repack_q3_k: bindings 1 and 2 must be bound");
    uint64_t units = (uint64_t)p.blocks * 8u;
    const uint64_t cover = elementwise_cover(d);
    if (cover < units) units = cover;
    if (units == 0) return ZHIP_OK;
    const uint64_t blocks_touched = (units + 7u) / 8u;
    if (blocks_touched * 110u > d.bind[1].size || units * 16u > d.bind[2].size) return fail(d, ZHIP_E_BAD_COMMAND, "repack_q3_k: bound ranges too small");
    if ((uintptr_t)d.bind[2].ptr & 15u) return fail(d, ZHIP_E_BAD_COMMAND, "repack_q3_k: destination must be 16-byte aligned");
    hipLaunchKernelGGL(repack_q3_k_kernel, dim3(blocks_for(units, 256, 65536)), dim3(256), 0, d.stream, d.bind[1].ptr,
        reinterpret_cast<uint4 *>(d.bind[2].ptr), units);
    return check_launch(d, "repack_q3_k");
}

// ---- repad: src/kernels/repad.wgsl ---------------------------------------------
__global__ __launch_bounds__(256) void repad_kernel(RepadParams p, const uint8_t *src, uint32_t *dst, uint64_t count) {
    const uint32_t words = p.dst_bytes / 4u;
    for (uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x; i < count; i += (uint64_t)gridDim.x * 256u) {
        const uint64_t blk = i / words;
        const uint32_t off = 4u * (uint32_t)(i % words);
        uint32_t v = 0;
        if (off < p.src_bytes) {
            const uint64_t s = blk * p.src_bytes + off;
            const uint32_t own = p.src_bytes - off < 4u ? p.src_bytes - off : 4u;
            for (uint32_t b = 0; b < own; b++) v |= (uint32_t)src[s + b] << (8u * b);
        }
        dst[i] = v;
    }
}

zhip_result launch_repad(const Dispatch &d) {
    if (d.params_size < sizeof(RepadParams)) return fail(d, ZHIP_E_BAD_COMMAND, "repad: params block too small");
    const RepadParams &p = *reinterpret_cast<const RepadParams *>(d.params);
    if (!d.bind[1].bound || !d.bind[2].bound) return fail(d, ZHIP_E_BAD_COMMAND, "repad: bindings 1 and 2 must be bound");
    if (p.dst_bytes == 0 || p.dst_bytes % 4u != 0 || p.dst_bytes < p.src_bytes) return fail(d, ZHIP_E_BAD_COMMAND, "repad: bad block sizes %u -> %u", p.src_bytes, p.dst_bytes);
    uint64_t count = (uint64_t)p.blocks * (p.dst_bytes / 4u);
    const uint64_t cover = elementwise_cover(d);
    if (cover < count) count = cover;
    if (count == 0) return ZHIP_OK;
    const uint64_t blocks_touched = (count + p.dst_bytes / 4u - 1) / (p.dst_bytes / 4u);
    if (blocks_touched * p.src_bytes > d.bind[1].size || count * 4u > d.bind[2].size) return fail(d, ZHIP_E_BAD_COMMAND, "repad: bound ranges too small");
    hipLaunchKernelGGL(repad_kernel, dim3(blocks_for(count, 256, 65536)), dim3(256), 0, d.stream, p,
        d.bind[1].ptr, reinterpret_cast<uint32_t *>(d.bind[2].ptr), count);
    return check_launch(d, "repad");
}

// ---- embed_q8_0 / embed_q3_k / embed_q4_k / embed_q5_k / embed_q6_k / embed_bf16 / embed_f16: src/kernels/embed_quant.wgsl, -------
// src/kernels/embed_half.wgsl. out[t] = table[tokens[t] - row0] decoded to f32
// for tokens whose row lies in [row0, row0 + chunk_rows); one workgroup per
// token. The decoders are the multiplies' own, so these kernels also show the
// block dequantisation bit for bit.
struct EmbedParams { uint32_t dim, row0, chunk_rows, stride; };

template <class D>
__global__ __launch_bounds__(256) void embed_kernel(EmbedParams p, const uint32_t *tokens, const uint8_t *table, float *out, uint32_t row_bytes) {
    const uint32_t t = blockIdx.x;
    const uint32_t tok = tokens[t];
    if (tok < p.row0 || tok >= p.row0 + p.chunk_rows) return;
    const uint8_t *row = table + (size_t)(tok - p.row0) * row_bytes;
    float *dst = out + (size_t)t * p.dim;
    for (uint32_t task = threadIdx.x; task < p.dim / D::E; task += 256u) {
        float w[D::E];
        D::decode(row, p.dim, task, w);
#pragma unroll
        for (int h = 0; h < D::RUNS; h++) {
            const uint32_t o = D::xoff(task, h);
#pragma unroll
            for (int i = 0; i < D::E / D::RUNS; i++) dst[o + i] = w[h * (D::E / D::RUNS) + i];
        }
    }
}

// Q8_0 rows laid out as in the GGUF file (34-byte blocks), `stride` bytes apart.
__global__ __launch_bounds__(256) void embed_q8_0_file_kernel(EmbedParams p, const uint32_t *tokens, const uint8_t *table, float *out) {
    const uint32_t t = blockIdx.x;
    const uint32_t tok = tokens[t];
    if (tok < p.row0 || tok >= p.row0 + p.chunk_rows) return;
    const uint8_t *row = table + (size_t)(tok - p.row0) * p.stride;
    for (uint32_t i = threadIdx.x; i < p.dim; i += 256u) {
        const uint8_t *b = row + (size_t)(i / 32u) * 34u;
        const float d = half_bits_to_float((uint32_t)b[0] | ((uint32_t)b[1] << 8));
        out[(size_t)t * p.dim + i] = __fmul_rn((float)(int8_t)b[2 + i % 32u], d);
    }
}

template <class D>
static zhip_result launch_embed(const Dispatch &d, const char *name) {
    if (d.params_size < sizeof(EmbedParams)) return fail(d, ZHIP_E_BAD_COMMAND, "%s: params block too small", name);
    const EmbedParams &p = *reinterpret_cast<const EmbedParams *>(d.params);
    for (int b = 1; b <= 3; b++)
        if (!d.bind[b].bound) return fail(d, ZHIP_E_BAD_COMMAND, "%s: binding %d is not bound", name, b);
    const uint32_t tokens = d.grid[0];
    if (tokens == 0 || p.dim == 0) return ZHIP_OK;
    if (p.dim % D::BLOCK != 0) return fail(d, ZHIP_E_BAD_COMMAND, "%s: dim = %u is not a multiple of %u", name, p.dim, D::BLOCK);
    const bool file_rows = p.stride != 0 && D::BLOCK == 32;
    const uint32_t row_bytes = p.stride != 0 ? p.stride : D::row_bytes(p.dim);
    const uint64_t min_row = file_rows ? (uint64_t)p.dim / 32u * 34u : D::row_bytes(p.dim);
    if (row_bytes < min_row) return fail(d, ZHIP_E_BAD_COMMAND, "%s: stride %u below the row size", name, row_bytes);
    if ((uint64_t)tokens * 4u > d.bind[1].size || (p.chunk_rows ? (uint64_t)(p.chunk_rows - 1) * row_bytes + min_row : 0) > d.bind[2].size ||
        (uint64_t)tokens * p.dim * 4u > d.bind[3].size)
        return fail(d, ZHIP_E_BAD_COMMAND, "%s: bound ranges too small", name);
    const uint32_t *tok = reinterpret_cast<const uint32_t *>(d.bind[1].ptr);
    float *out = reinterpret_cast<float *>(d.bind[3].ptr);
    if (file_rows) {
        hipLaunchKernelGGL(embed_q8_0_file_kernel, dim3(tokens), dim3(256), 0, d.stream, p, tok, d.bind[2].ptr, out);
    } else {
        if (((uintptr_t)d.bind[2].ptr | row_bytes) & 15u) return fail(d, ZHIP_E_BAD_COMMAND, "%s: table rows must be 16-byte aligned", name);
        hipLaunchKernelGGL((embed_kernel<D>), dim3(tokens), dim3(256), 0, d.stream, p, tok, d.bind[2].ptr, out, row_bytes);
    }
    return check_launch(d, name);
}

zhip_result launch_embed_q8_0(const Dispatch &d) { return launch_embed<DecQ8_0>(d, "embed_q8_0"); }
zhip_result launch_embed_q4_k(const Dispatch &d) { return launch_embed<DecQ4_K>(d, "embed_q4_k"); }
zhip_result launch_embed_q3_k(const Dispatch &d) { return launch_embed<DecQ3_K>(d, "embed_q3_k"); }
zhip_result launch_embed_q5_k(const Dispatch &d) { return launch_embed<DecQ5_K>(d, "embed_q5_k"); }
zhip_result launch_embed_q6_k(const Dispatch &d) { return launch_embed<DecQ6_K>(d, "embed_q6_k"); }
zhip_result launch_embed_bf16(const Dispatch &d) { return launch_embed<DecBF16>(d, "embed_bf16"); }
zhip_result launch_embed_f16(const Dispatch &d) { return launch_embed<DecF16>(d, "embed_f16"); }

// ---- embed_iq4_xs: src/kernels/quant/iq4_xs.wgsl through embed_quant.wgsl ----------
// Blocks of 256: d (f16), scales_h (u16), scales_l[4], qs[128]; a 32-weight group
// has a signed six-bit scale biased by 32 and sixteen bytes of indices into a
// nonlinear table, low nibbles first (src/ref/tensor.zig:162-181). Rows come as
// the loader lays them out (136-byte blocks padded to 144) or, with a stride, as
// the file stores them. A thread decodes one index byte: two weights, each
// (d * scale) * table[index] with both products rounded to nearest.
__global__ __launch_bounds__(256) void embed_iq4_xs_kernel(EmbedParams p, const uint32_t *tokens, const uint8_t *table, float *out, uint32_t row_bytes, uint32_t block_bytes) {
    const int values[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};
    const uint32_t t = blockIdx.x;
    const uint32_t tok = tokens[t];
    if (tok < p.row0 || tok >= p.row0 + p.chunk_rows) return;
    const uint8_t *row = table + (size_t)(tok - p.row0) * row_bytes;
    float *dst = out + (size_t)t * p.dim;
    for (uint32_t i = threadIdx.x; i < p.dim / 2u; i += 256u) {
        const uint8_t *b = row + (size_t)(i / 128u) * block_bytes;
        const uint32_t group = (i / 16u) % 8u, j = i % 16u;
        const float d = half_bits_to_float((uint32_t)b[0] | ((uint32_t)b[1] << 8));
        const uint32_t scales_h = (uint32_t)b[2] | ((uint32_t)b[3] << 8);
        const uint32_t low = (b[4u + group / 2u] >> (4u * (group % 2u))) & 15u, high = (scales_h >> (2u * group)) & 3u;
        const float dl = __fmul_rn(d, (float)((int)(low | (high << 4)) - 32));
        const uint32_t q = b[8u + 16u * group + j];
        int lo = 0, hi = 0;
#pragma unroll
        for (uint32_t v = 0; v < 16; v++) {  // a table in registers: selects, not memory
            lo = (q & 15u) == v ? values[v] : lo;
            hi = (q >> 4) == v ? values[v] : hi;
        }
        float *o = dst + 256u * (i / 128u) + 32u * group + j;
        o[0] = __fmul_rn(dl, (float)lo);
        o[16] = __fmul_rn(dl, (float)hi);
    }
}

zhip_result launch_embed_iq4_xs(const Dispatch &d) {
    const char *name = "embed_iq4_xs";
    if (d.params_size < sizeof(EmbedParams)) return fail(d, ZHIP_E_BAD_COMMAND, "%s: params block too small", name);
    const EmbedParams &p = *reinterpret_cast<const EmbedParams *>(d.params);
    for (int b = 1; b <= 3; b++)
        if (!d.bind[b].bound) return fail(d, ZHIP_E_BAD_COMMAND, "%s: binding %d is not bound", name, b);
    const uint32_t tokens = d.grid[0];
    if (tokens == 0 || p.dim == 0) return ZHIP_OK;
    if (p.dim % 256u != 0) return fail(d, ZHIP_E_BAD_COMMAND, "%s: dim = %u is not a multiple of 256", name, p.dim);
    const uint32_t block_bytes = p.stride != 0 ? 136u : 144u;
    const uint64_t min_row = (uint64_t)p.dim / 256u * block_bytes;
    const uint64_t row_bytes = p.stride != 0 ? p.stride : min_row;
    if (row_bytes < min_row || row_bytes > 0xffffffffull) return fail(d, ZHIP_E_BAD_COMMAND, "%s: stride %llu against a row of %llu bytes", name, (unsigned long long)row_bytes, (unsigned long long)min_row);
    if ((uint64_t)tokens * 4u > d.bind[1].size || (p.chunk_rows ? (uint64_t)(p.chunk_rows - 1) * row_bytes + min_row : 0) > d.bind[2].size ||
        (uint64_t)tokens * p.dim * 4u > d.bind[3].size)
        return fail(d, ZHIP_E_BAD_COMMAND, "%s: bound ranges too small", name);
    hipLaunchKernelGGL(embed_iq4_xs_kernel, dim3(tokens), dim3(256), 0, d.stream, p, reinterpret_cast<const uint32_t *>(d.bind[1].ptr), d.bind[2].ptr,
                       reinterpret_cast<float *>(d.bind[3].ptr), (uint32_t)row_bytes, block_bytes);
    return check_launch(d, name);
}

// ---- fill ----------------------------------------------------------------------
__global__ __launch_bounds__(256) void fill_kernel(uint32_t *dst, uint64_t words, uint32_t value) {
    for (uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x; i < words; i += (uint64_t)gridDim.x * 256u) dst[i] = value;
}

zhip_result launch_fill(hipStream_t stream, void *dst, uint64_t words, uint32_t value) {
    if (words == 0) return ZHIP_OK;
    hipLaunchKernelGGL(fill_kernel, dim3(blocks_for(words, 1024, 4096)), dim3(256), 0, stream, reinterpret_cast<uint32_t *>(dst), words, value);
    return hipGetLastError() == hipSuccess ? ZHIP_OK : ZHIP_E_GPU;
}

}  // namespace zhip
