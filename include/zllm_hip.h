/* zllm_hip: zllm's HIP backend host for AMD MI355X (gfx950), as a C ABI.
 *
 * zllm's core never calls a GPU API: it records a flat little-endian u32
 * command stream (src/gpu/cmd.zig:8-59) and hands each batch to a backend host
 * (src/gpu/host.zig:138-191). This library is that host for a third backend
 * beside WebGPU/Dawn and Agility/D3D12: it owns the command-stream
 * interpreter, device buffers, one in-order HIP stream and the precompiled
 * gfx950 kernels of the quantized linear-layer path (the matvec_ / matmul_
 * kernel identities of src/kernels/kernels.zig:24-92 and their layout and
 * epilogue helpers). The Zig side is forwarding glue only.
 *
 * Conventions follow the reference's one native ABI (src/agility/agility.h):
 * opaque context, int32 results with negative = failure, a last-error string,
 * serialized access per context, and a test hook that loses the device.
 */
#ifndef ZLLM_HIP_H
#define ZLLM_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ZHIP_ABI_VERSION 1u

typedef struct zhip_context zhip_context;
typedef int32_t zhip_result;

/* Results. Each failure maps to one member of the reference host's error set
 * (src/agility/host.zig:38, src/gpu/cmd.zig:227). */
enum {
    ZHIP_OK = 0,
    ZHIP_E_GPU = -1,                /* error.GpuError: a HIP call failed; see zhip_last_error */
    ZHIP_E_DEVICE_LOST = -2,        /* error.DeviceLost */
    ZHIP_E_BAD_COMMAND = -3,        /* error.BadCommand: malformed args, out-of-range offsets/sizes */
    ZHIP_E_BAD_ID = -4,             /* error.BadId: unknown or reused object id */
    ZHIP_E_TRUNCATED = -5,          /* error.Truncated: a command runs past the batch */
    ZHIP_E_BAD_LENGTH = -6,         /* error.BadLength: a zero-length command header */
    ZHIP_E_UNSUPPORTED_KERNEL = -7, /* error.UnsupportedKernel: dispatch of a pipeline with an empty artifact */
    ZHIP_E_UNSUPPORTED_PREFILL = -8,/* error.UnsupportedPrefill: a prefill rung this device lacks */
    ZHIP_E_OUT_OF_MEMORY = -9,      /* error.OutOfMemory */
    ZHIP_E_NO_DEVICE = -10,         /* no usable gfx950 device / HIP runtime */
    ZHIP_E_INVALID_ARGUMENT = -11   /* a null or undersized argument to this API */
};

/* zhip_options.flags. A submit that is only dispatches (then reads) and repeats an
 * earlier one exactly is replayed from a HIP graph captured the second time it is
 * seen; this flag (or the environment variable ZHIP_NO_REPLAY) keeps every
 * submit a sequence of plain launches. No counterpart in the reference: its
 * hosts record command lists per submit (src/agility/host.zig:520-548). */
#define ZHIP_OPTION_NO_REPLAY 1u
/* matvec_bf16 / matvec_f16 over 16 MB or more of weights (k = 1024 ... 16384 in
 * steps of 512) read the weights once for all of a step's tokens on the matrix
 * cores, at every width from one token on, so that a token's bits do not depend
 * on the width of the step it ran in (src/sched/sched.zig:55-58,
 * src/plan/qwen35.zig:380-381). For deployments that verify speculated tokens
 * on these matrices: a step of 2..8 tokens then costs what one token does
 * (151936 x 1024 bf16: 55 us at any width; without the flag 52 / 75 / 122 us at
 * 1 / 4 / 8 tokens). Without the flag every width runs the kernel that takes the
 * tokens one pass each, whose one-token step is ~6 % faster; either way the
 * route depends on the matrix alone, never on the step. */
#define ZHIP_OPTION_WIDE_DECODE 2u

typedef struct zhip_options {
    uint32_t device_index; /* HIP device ordinal */
    uint32_t flags;        /* ZHIP_OPTION_* */
} zhip_options;

/* What gpu.Device.adapter/limits/memoryBudget report (src/gpu/host.zig:30-46,
 * 81-108). */
typedef struct zhip_caps {
    uint32_t abi_version;
    uint32_t compute_units;
    uint32_t wavefront;
    uint32_t lds_bytes;       /* per workgroup */
    uint64_t memory_bytes;    /* total device memory */
    uint64_t memory_free;     /* free now */
    uint64_t max_binding;     /* 2 GiB, as the planner expects (src/gpu/host.zig:81-84) */
    uint64_t offset_align;    /* 256 */
    char name[128];           /* e.g. "AMD Instinct MI355X" */
    char arch[32];            /* e.g. "gfx950" */
} zhip_caps;

/* cmd.Completion (src/gpu/cmd.zig:89-94): status 0 ok, 1 failed. */
typedef struct zhip_completion {
    uint32_t token;
    uint32_t status;
} zhip_completion;

/* One row of gpu.Timings (src/gpu/timings.zig:6-27): totals per pipeline id and
 * grid while profiling. */
typedef struct zhip_timing {
    uint32_t pipeline;
    uint32_t grid[3];
    uint64_t ns;
    uint64_t count;
} zhip_timing;

/* precision.Prefill (src/precision.zig:9). */
enum { ZHIP_PREFILL_SCALAR_F32 = 0, ZHIP_PREFILL_FP16_SINGLE = 1, ZHIP_PREFILL_FP16_COMPENSATED = 2 };

/* All calls require serialized access to each context (as agility.h:67). */

/* Replaces gpu.Device.open / Device.init (src/gpu/host.zig:52-57,
 * src/agility/host.zig:49-64). */
zhip_result zhip_create(const zhip_options *options, zhip_context **out_context);
/* Replaces Device.deinit + Host.deinit (src/gpu/host.zig:59-63,145-149). */
zhip_result zhip_destroy(zhip_context *context);
/* Replaces Device.limits/adapter/memoryBudget (src/gpu/host.zig:81-126). */
zhip_result zhip_get_caps(zhip_context *context, zhip_caps *out_caps);
/* Replaces Device.supportsPrefill (src/gpu/host.zig:70-77): 1 or 0. All three
 * rungs of the reference's ladder are supported: scalar_f32 (exact f32 kernels),
 * fp16_single and fp16_compensated (create_kernel variants 0xfffc0000 and
 * 0xffff0000 of matmul_q8_0_float, matmul_bf16 and matmul_f16,
 * src/agility/kernels.zig:114-131) on the f16 matrix cores; 3 and 4 name this
 * backend's own bf16 rungs (variants 0xfffb0000 / 0xfffa0000 of
 * matmul_q8_0_float and matmul_bf16). */
int32_t zhip_supports_prefill(zhip_context *context, uint32_t rung);
/* Replaces Host.setFile (src/gpu/host.zig:158-165): the model file mapping
 * write_file commands read; it must stay mapped while they may execute. */
zhip_result zhip_set_file(zhip_context *context, const void *bytes, size_t len);

/* Replaces Host.execute (src/gpu/host.zig:151-156; semantics of
 * src/agility/host.zig:293-466 and src/gpu/dawn_host.zig:120-246): interprets
 * one batch of command words. write_buffer / write_file land before the next
 * submit's work, even work recorded ahead of them; dispatches, copies, clears
 * and reads between submits run in recorded order; submit blocks until the
 * GPU has finished and appends one completion per pending read_buffer, then
 * one for the submit token. `*out_count` receives the completions written; a
 * batch producing more than `capacity` fails with ZHIP_E_INVALID_ARGUMENT
 * before anything runs. On ZHIP_E_UNSUPPORTED_KERNEL the submission in
 * progress is dropped. */
zhip_result zhip_execute(zhip_context *context, const uint32_t *words, size_t n_words,
    zhip_completion *out_completions, size_t capacity, size_t *out_count);

/* Replaces Host.startProfile/stopProfile/timings (src/gpu/host.zig:167-190):
 * while profiling every dispatch is bracketed by its own event pair, which
 * serialises dispatches as both reference hosts do. zhip_profile_read copies
 * up to `capacity` rows and reports the row count and the untimed dispatches. */
zhip_result zhip_profile_start(zhip_context *context);
zhip_result zhip_profile_stop(zhip_context *context);
zhip_result zhip_profile_read(zhip_context *context, zhip_timing *out, size_t capacity,
    size_t *out_count, uint64_t *out_untimed);
/* GPU time of the last submit's recorded work (first op to last op, one event
 * pair on the host's stream), in nanoseconds, and how many dispatches it ran:
 * the measurement a tuner's batched timing takes (src/tune/tune.zig:8-11). */
zhip_result zhip_last_submit(zhip_context *context, uint64_t *out_ns, uint64_t *out_dispatches);
/* How many submits so far ran their dispatches from a replayed graph (see
 * ZHIP_OPTION_NO_REPLAY). No counterpart in the reference; for tests and reports. */
zhip_result zhip_replayed_submits(zhip_context *context, uint64_t *out_count);

/* No counterpart in the reference. For callers that cannot allocate device
 * memory (code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc): the multiply of a matmul_q8_0_float dispatch in this
 * backend's bf16 rung (create_kernel variant 0xfffb0000: f32-bound activations,
 * Q8_0 weights in split rows, bf16 matrix cores, fp32 accumulation), given as
 * device pointers instead of a command stream, with the kernels' one scratch
 * buffer (the bf16 copy of the step's activations, which zhip_execute keeps
 * in a workspace it grows with hipMalloc) in a fixed array inside the library.
 *   out[t * out_stride + col0 + j] (+)= sum_i x[t * k + i] * w[j][i],
 *   t < rows, j < n; `accumulate` != 0 adds to what `out` holds.
 * Asynchronous on `stream` (a hipStream_t; null = the null stream), which must
 * belong to the context's device; the call allocates and frees nothing and
 * does not synchronize. Results equal the dispatch's bit for bit. Limit:
 * rows * k * 2 <= zhip_no_alloc_capacity() (8 MiB: 1024 tokens of 4096 inputs);
 * more fails with ZHIP_E_BAD_COMMAND and a message. Every call on a GPU shares
 * that GPU's one array: calls that overlap on one GPU (different streams or
 * threads, or different contexts of one device) race. */
zhip_result zhip_matmul_q8_0_float_no_alloc(zhip_context *context, void *stream, const float *x,
    const void *weights, float *out, uint32_t rows, uint32_t n, uint32_t k, uint32_t col0,
    uint32_t out_stride, uint32_t accumulate);
/* Bytes of the fixed scratch array the call above narrows activations into. */
uint64_t zhip_no_alloc_capacity(void);

/* Replaces Device.errorMessage (src/gpu/host.zig:128-133; agility.h:108-109):
 * copies the last error message, NUL-terminated; returns its length. */
size_t zhip_last_error(zhip_context *context, char *out, size_t capacity);
/* Replaces Device.forceLoss (src/gpu/host.zig:135-139; agility.h:110-111):
 * every later call but zhip_destroy / zhip_last_error returns
 * ZHIP_E_DEVICE_LOST. No GPU fault is provoked. */
zhip_result zhip_force_loss(zhip_context *context);

/* Replaces the backend arm of kernels.artifact (src/kernels/kernels.zig:
 * 904-912): the artifact bytes create_kernel carries for kernel `name`
 * (a kernels.Kernel tag name, e.g. "matvec_q4_k") in variant `variant`
 * (MatvecVariant.id, src/kernels/kernels.zig:328-333). Returns the length
 * written (without the NUL), or 0 when this backend does not implement the
 * kernel, which the caller records as an empty artifact
 * (src/kernels/kernels.zig:776-783).
 *
 * Every MatvecVariant id is accepted. What the ids guarantee is the
 * reference's kernel check (src/kernels/check.zig:1019-1060): every output
 * within 1e-5 of the exact product's scale, and a token's bits independent of
 * how many tokens share its step and of the id's lane / row tunables (the
 * backend runs one arithmetic for all of them); the bits themselves are this
 * backend's, not the WGSL kernels'. Two things go beyond the reference's contract: decode multiplies
 * take 5..8 token rows (the reference stops at 4,
 * src/kernels/matvec_quant.wgsl.hbs:64-65), and on matvec_q3_k, matvec_q4_k,
 * matvec_q5_k, matvec_q6_k and matvec_q8_0 the id 0x00104010 (wg 512, lanes 64,
 * rows 16, a geometry no reference tuning emits) selects matrix-core kernels
 * for steps of 1..8 tokens that read the weights once; their sums round
 * differently from the default id's (both within 1e-5 of the output scale), the
 * same at every width. */
size_t zhip_kernel_artifact(const char *name, uint32_t variant, char *out, size_t capacity);
/* Replaces the backend arm of kernels.backendSource (src/kernels/kernels.zig:
 * 914-922): bytes that change whenever the kernel's implementation changes
 * (the plan cache hashes them). Same return convention. */
size_t zhip_backend_source(const char *name, char *out, size_t capacity);
/* The kernels.Kernel ordinal the library was generated against for `name`
 * (src/kernels/kernels.zig:24-92 declaration order), or -1. */
int32_t zhip_kernel_ordinal(const char *name);

#ifdef __cplusplus
}
#endif
#endif
