/* CPU oracle for zllm's quantized linear-layer hot path.
 *
 * TEST INFRASTRUCTURE ONLY. This is a plain-C restatement of the reference's
 * CPU path (the .zig files under src/ref) used as the checker by tests/, the smoke test and
 * the benchmark's cpu_baseline leg. Nothing in the shipped library links it,
 * calls it or falls back to it.
 *
 * Every function cites the reference file:line it follows. The reference is
 * Zig and cannot be built in this environment, so what pins each function is
 * listed beside it:
 *   - zref_dequantize (q8_0, bf16, f16, f32): closed forms checked against
 *     numpy / torch conversions, an exhaustive 256 x 65536 product sweep, and
 *     the reference's own known answers (src/ref/tensor.zig:192-209).
 *   - zref_dequantize (q4_k) and zref_scale_min_k4: pack/unpack round trips
 *     over all 64 x 64 (scale, min) pairs for every sub-block, an independent
 *     vectorised numpy restatement of the byte map, and the special cases that
 *     make the two-rounding formula exact (zero scales, power-of-two d/dmin).
 *     Parity with ggml's dequantize_row_q4_K (llama.cpp e09a78a2, what the
 *     reference itself is pinned to by tools/check_dequant.py) is "parity
 *     unpinned" here: that library is not available offline.
 *   - zref_dequantize (q3_k, q5_k, q6_k): the reference holds no known answers for
 *     them (its kernel check compares against its own decoder), so they are
 *     pinned by what the format fixes: packing known quants and scales into
 *     blocks by an independent numpy bit map and decoding them back, the
 *     special cases that make every product exact, and single-bit mutations
 *     that must move exactly one weight. Agreement with ggml's
 *     dequantize_row_q3_K / q5_K / q6_K is "parity unpinned" (library not
 *     available offline). zref_repack_q3_k is pinned by decoding its units with
 *     an independent numpy reader and comparing with zref_dequantize.
 *   - zref_matmul: the reference's tests (src/ref/matmul.zig:296-380): naive
 *     product for every row remainder and pool size, and bit-exact results on
 *     dyadic data; float64 numpy products.
 *   - zref_rms_norm: the reference's 17-value bitwise known answer
 *     (src/ref/ops.zig:139-168).
 *   - zref_bf16_round: torch.bfloat16 round-to-nearest-even.
 *   - zref_f16_round: numpy's float16 conversion over a sweep of every exponent
 *     with tie and near-tie mantissas.
 *   - zref_quantize_q8 / zref_round_like_llama: the cases the reference's own
 *     check builds (src/kernels/check.zig:516-547: a negative maximum, a +amax /
 *     -amax tie, a zero row, exact half-integers in blocks whose scale is 1)
 *     with their answers worked by hand, and a numpy restatement that rounds
 *     with rint instead of the magic-number addition. Agreement with ggml's
 *     quantize_row_q8_0 / quantize_row_q8_K_ref is "parity unpinned" (library
 *     not available offline).
 *   - zref_matmul_q8: must equal, to double rounding, the float64 product of the
 *     rounded activations q * d with the decoded weights (zref_dequantize),
 *     the formulation the reference checks its kernel against
 *     (src/kernels/check.zig:839-871).
 *   - zref_silu: float64 closed form. Its last-ulp agreement with Zig's @exp is
 *     "parity unpinned" (only an import of the Zig build could pin it).
 */
#ifndef ZREF_H
#define ZREF_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* GGUF tensor type ids (src/gguf/gguf.zig:20-58 numbering as in the GGUF spec). */
enum {
    ZREF_F32 = 0,
    ZREF_F16 = 1,
    ZREF_Q8_0 = 8,
    ZREF_Q3_K = 11,
    ZREF_Q4_K = 12,
    ZREF_Q5_K = 13,
    ZREF_Q6_K = 14,
    ZREF_IQ4_XS = 23,
    ZREF_BF16 = 30,
};

/* Block geometry (src/gguf/gguf.zig:69-109). Returns 0 for unknown types. */
int zref_layout(int type, uint32_t *block_elems, uint32_t *block_bytes);

/* IEEE binary16 -> binary32, exact (src/ref/tensor.zig:45-47). */
float zref_half(uint16_t bits);

/* The 6-bit scale and min of sub-block j from 12 packed bytes
 * (src/ref/tensor.zig:94-98). */
void zref_scale_min_k4(unsigned j, const uint8_t q[12], uint8_t *sc, uint8_t *m);
/* The inverse used to build synthetic blocks: stores (sc, m) of sub-block j
 * into the 12 bytes, which must start zeroed. */
void zref_pack_scale_min_k4(unsigned j, uint8_t q[12], uint8_t sc, uint8_t m);

/* Decodes n elements of `type` from `bytes` (src/ref/tensor.zig:21-43).
 * Returns 0, or -1 for an unsupported type. */
int zref_dequantize(int type, const uint8_t *bytes, float *out, size_t n);

/* Round-to-nearest-even f32 -> bf16 -> f32 (src/ref/matmul.zig:250-255). */
float zref_bf16_round(float v);

/* x / (1 + exp(-x)) (src/ref/ops.zig:49-51). */
float zref_silu(float x);

/* In place x / sqrt(mean(x^2) + eps) * weight (src/ref/ops.zig:25-41). */
void zref_rms_norm(float *x, const float *weight, size_t n, float eps);

/* An n x k weight matrix (src/ref/matmul.zig:37-107): f32/f16/bf16 are packed
 * into 32-row k-major panels at init; quantized types keep the raw rows and
 * each thread decodes a panel just before using it. `bytes` must outlive the
 * matrix for quantized types. */
typedef struct zref_matrix zref_matrix;
zref_matrix *zref_matrix_init(int type, const uint8_t *bytes, size_t n, size_t k, unsigned threads);
void zref_matrix_free(zref_matrix *m);
/* Copies row j (k weights) into out (src/ref/matmul.zig:94-106). */
void zref_matrix_row(const zref_matrix *m, size_t j, float *out);

/* out[t][j] = sum_i x[t][i] * w[j][i], t < rows (src/ref/matmul.zig:160-195,
 * 262-294): panels split in contiguous ranges across `threads`
 * (src/ref/pool.zig:76-122), tokens in blocks of 8, each output summed over k
 * in increasing order with separate multiply and add. */
void zref_matmul(float *out, const float *x, const zref_matrix *w, size_t rows, unsigned threads);

/* act[t][j] = silu(gate[t][j]) * up[t][j] over stacked gate|up rows: the FFN
 * composition of src/ref/dense.zig:179-197 up to the down projection. `w` has
 * 2*half rows: gate rows [0, half), up rows [half, 2*half). */
void zref_gate_up_silu(float *act, const float *x, const zref_matrix *w, size_t half, size_t rows, unsigned threads);

/* First index of the maximum, ties to the lower index
 * (src/kernels/draft.wgsl:1-4, src/precision.zig:168-175). */
uint32_t zref_argmax(const float *v, size_t n);

/* Threads the reference would use: one per physical core
 * (src/main.zig:438-448). */
unsigned zref_default_threads(void);

/* GPU-side weight layouts the kernels read (restated from the reference's
 * layout kernels; CPU twins for tests). */
/* (k + k/16 + 15) & ~15 for Q8_0 split rows, blocks * blockStride otherwise
 * (src/kernels/kernels.zig:144-160). */
uint64_t zref_row_bytes(int type, uint64_t k);
/* 34-byte file blocks -> split rows: k int8 values, k/32 f16 scales, zero pad
 * to 16 bytes (src/kernels/repack_q8_0.wgsl:26-51). */
void zref_repack_q8_0(const uint8_t *src, uint8_t *dst, size_t rows, size_t k);
/* src/kernels/repack_q3_k.wgsl: `blocks` 110-byte Q3_K blocks into eight
 * self-contained 16-byte units each (128 bytes a block). */
void zref_repack_q3_k(const uint8_t *src, uint8_t *dst, size_t blocks);

/* Split of a prefill multiply over k (src/kernels/kernels.zig:285-295). */
void zref_matmul_slices(uint32_t n, uint32_t k, uint32_t *count, uint32_t *k_slice);

/* Float64 formula checkers as the reference's GPU check computes them
 * (src/kernels/check.zig:34-83,205-222): want[t][j] = init + sum x*w in
 * double over already decoded weights. */
void zref_matmul_f64(double *want, const float *x, const float *w, size_t rows, size_t n, size_t k, unsigned threads);

/* ---- activations rounded to 8-bit blocks (the quantized prefill multiply) --- */

/* x >= 0 rounded to binary16 (nearest even) and widened back
 * (src/kernels/quantize_q8.wgsl:52-60). */
float zref_f16_round(float x);
/* x[i] ~ q[i] * d[i / block] as llama.cpp's x86 CPU backend rounds activations:
 * block 32 = Q8_0 (d = amax / 127 in f16, q = rne(x * (127 / amax))), block 256
 * = Q8_K (d = -max / 127 for the first value of largest magnitude, q =
 * min(127, rne(x * -127 / max))) (src/ref/matmul.zig:197-247,
 * src/kernels/quantize_q8.wgsl:11-22). Returns 0, or -1 for a bad block. */
int zref_quantize_q8(const float *x, size_t n, unsigned block, int8_t *q, float *d);
/* A row rounded in place as the multiply with weights of `type` sees it
 * (src/ref/matmul.zig:197-247). */
int zref_round_like_llama(int type, float *x, size_t n);
/* quantize_q8 over rows with its fused producers (src/kernels/quantize_q8.wgsl:1-9):
 * mode 0 x, 1 RMSNorm(x) * nw, 2 silu(gate) * up over rows of gate | up. */
int zref_quantize_q8_rows(const float *x, size_t rows, size_t k, unsigned block, unsigned mode, float eps,
                          const float *nw, int8_t *q, float *d);
/* The int8 prefill multiply's formula (src/kernels/matmul_quant.wgsl:1-9):
 * exact integer unit sums, scaled and added in double. `w` is file-layout
 * Q8_0, Q3_K, Q4_K, Q5_K or Q6_K rows. */
int zref_matmul_q8(int type, const uint8_t *w, const int8_t *qx, const float *dx, size_t rows, size_t n, size_t k, double *out);

#ifdef __cplusplus
}
#endif
#endif
