// Internal interface between the command-stream host and the gfx950 kernels.
#pragma once

#include <hip/hip_runtime_api.h>
#include <stddef.h>
#include <stdint.h>

#include "../../include/zllm_hip.h"

namespace zhip {

// Parameter blocks, field for field as src/kernels/kernels.zig:432-505 declares
// them (extern structs, little-endian, bound at binding 0).
struct MatvecParams {  // params.MatvecBf16
    uint32_t n, k, col0, out_stride;
    float eps;
    uint32_t flags;
    uint32_t half;
    uint32_t x_stride;  // vec4 units between tokens' inputs; 0: k / 4
};
enum : uint32_t { FLAG_NORM = 1u, FLAG_ACCUMULATE = 2u, FLAG_SILU_PAIR = 4u };

struct MatmulParams {  // params.MatmulBf16 / params.MatmulQuant
    uint32_t rows, n, k, col0, out_stride, accumulate;
    uint32_t k_slice;       // MatmulBf16: padding
    uint32_t slice_stride;  // MatmulBf16: padding
};

struct MatmulReduceParams {
    uint32_t rows, n, slices, col0, out_stride, accumulate, slice_stride, pad;
};

struct SiluMulParams { uint32_t count, width, pad0, pad1; };
struct RepackQ80Params { uint32_t rows, k, pad0, pad1; };
struct RepadParams { uint32_t blocks, src_bytes, dst_bytes, pad; };

static_assert(sizeof(MatvecParams) == 32, "params.MatvecBf16 is 32 bytes");
static_assert(sizeof(MatmulParams) == 32, "params.MatmulQuant is 32 bytes");
static_assert(sizeof(MatmulReduceParams) == 32, "params.MatmulReduce is 32 bytes");
static_assert(sizeof(SiluMulParams) == 16 && sizeof(RepackQ80Params) == 16 && sizeof(RepadParams) == 16, "16-byte blocks");

// A quantized decode multiply's tunables (kernels.MatvecVariant,
// src/kernels/kernels.zig:319-338), decoded from the create_kernel variant id.
struct MatvecVariant {
    uint32_t wg = 256, lanes = 32, rows = 1, act_div = 0;
    uint32_t groupRows() const { return wg / lanes * rows; }
};

// Steps of up to this many tokens may use the decode multiplies. The reference
// caps its kernels at 4 (src/kernels/matvec_quant.wgsl.hbs:64-65); rows 5..8
// are this backend's extension for speculative-verify widths.
constexpr uint32_t kMaxDecodeRows = 8;

// A byte offset no binding reaches (a binding is at most 2 GiB): a range-checked buffer load
// there returns zeros and moves nothing.
constexpr uint32_t kNowhere = 0xF0000000u;

// The longest step the reference's planner records (src/plan/plan.zig:129,
// src/plan/qwen35.zig:335).
constexpr uint32_t kPlannerStepCap = 512;

struct Bind {
    uint8_t *ptr = nullptr;  // buffer base + binding offset
    uint64_t size = 0;       // bytes bound
    bool bound = false;
};

struct DeviceInfo {
    int compute_units = 256;
    int max_lds = 65536;
    bool wide_decode = false;  // ZHIP_OPTION_WIDE_DECODE
};

struct Dispatch;

// Device scratch a launcher may ask for (the bf16 copy of a step's f32
// activations). Owned by the context, grown on demand, freed with the context.
// Everything runs on the context's one in-order stream, so consecutive
// dispatches can share it.
struct Workspace {
    uint8_t *data = nullptr;
    uint64_t bytes = 0;
    bool fixed = false;  // memory the workspace does not own: never grown, never freed
    // Makes at least `want` bytes available (fails on a fixed workspace that is too small).
    zhip_result reserve(const Dispatch &d, uint64_t want);
    void release();
};

// One resolved dispatch: binding 0's bytes come from the host's shadow copy of
// the uniform buffer, so kernels take their parameters by value.
struct Dispatch {
    const uint8_t *params = nullptr;
    size_t params_size = 0;
    Bind bind[8];
    uint32_t grid[3] = {0, 0, 0};
    uint32_t variant = 0;
    hipStream_t stream = nullptr;
    const DeviceInfo *dev = nullptr;
    Workspace *work = nullptr;
    char *err = nullptr;  // message buffer for a failed launch
    size_t err_cap = 0;
};

// Launches one kernel for a dispatch, after checking that the bound ranges
// cover everything the kernel will touch. Returns ZHIP_OK, ZHIP_E_BAD_COMMAND
// (with a message) or ZHIP_E_GPU.
typedef zhip_result (*LaunchFn)(const Dispatch &);

zhip_result launch_matvec_q8_0(const Dispatch &);
zhip_result launch_matvec_q3_k(const Dispatch &);
zhip_result launch_matvec_q4_k(const Dispatch &);
zhip_result launch_matvec_q5_k(const Dispatch &);
zhip_result launch_matvec_q6_k(const Dispatch &);
zhip_result launch_matvec_bf16(const Dispatch &);
zhip_result launch_matvec_f16(const Dispatch &);
zhip_result launch_matmul_reduce(const Dispatch &);
zhip_result launch_quantize_q8(const Dispatch &);
zhip_result launch_matmul_q8_0(const Dispatch &);
zhip_result launch_matmul_q3_k(const Dispatch &);
zhip_result launch_matmul_q4_k(const Dispatch &);
zhip_result launch_matmul_q5_k(const Dispatch &);
zhip_result launch_matmul_q6_k(const Dispatch &);
zhip_result launch_silu_mul(const Dispatch &);
zhip_result launch_repack_q8_0(const Dispatch &);
zhip_result launch_repack_q3_k(const Dispatch &);
zhip_result launch_repad(const Dispatch &);
zhip_result launch_embed_q8_0(const Dispatch &);
zhip_result launch_embed_q3_k(const Dispatch &);
zhip_result launch_embed_q4_k(const Dispatch &);
zhip_result launch_embed_q5_k(const Dispatch &);
zhip_result launch_embed_q6_k(const Dispatch &);
zhip_result launch_embed_bf16(const Dispatch &);
zhip_result launch_embed_f16(const Dispatch &);
zhip_result launch_embed_iq4_xs(const Dispatch &);

// Dynamic LDS above 64 KiB needs opting in once per kernel: done the first time this is called
// for the kernel (or ahead of time, see prepare_no_alloc_kernels), remembered after.
template <auto Kernel, int Bytes>
inline bool lds_opt_in() {
    static const bool ok = [] {
        if (hipFuncSetAttribute(reinterpret_cast<const void *>(Kernel), hipFuncAttributeMaxDynamicSharedMemorySize, Bytes) == hipSuccess) return true;
        (void)hipGetLastError();
        return false;
    }();
    return ok;
}

// Host-side helpers shared by the launchers.
zhip_result fail(const Dispatch &d, zhip_result code, const char *fmt, ...);
zhip_result check_launch(const Dispatch &d, const char *kernel);

// The entry point that allocates nothing (no_alloc.hip): its fixed scratch array's address is
// looked up once per device, with that device current.
zhip_result no_alloc_setup(int device, const DeviceInfo &info);
// The one-time set-up of every kernel that entry point can launch (each file its own), so
// that the call itself does none.
bool matmul_mfma_prepare_no_alloc();
bool matmul_mfma_wide_prepare_no_alloc();
bool matmul_stream_prepare_no_alloc();
bool matmul_q8_bf16_prepare_no_alloc();
bool matmul_q8_bf16_wide_prepare_no_alloc();
uint64_t no_alloc_capacity();
zhip_result no_alloc_matmul_q8_0_float(int device, hipStream_t stream, const float *x, const void *w, float *out, uint32_t rows, uint32_t n,
    uint32_t k, uint32_t col0, uint32_t out_stride, uint32_t accumulate, char *err, size_t err_cap);

// Fills `words` 32-bit words at dst with `value` on the stream (clear_buffer;
// also used instead of memset nodes so a captured stream stays replayable).
zhip_result launch_fill(hipStream_t stream, void *dst, uint64_t words, uint32_t value);

}  // namespace zhip
