// A prefill multiply for callers that cannot allocate device memory (code under HIP graph
// capture, serving loops and harnesses that forbid hipMalloc): matmul_q8_0_float on the bf16
// matrix cores with f32-bound activations, whose bf16 copy of the step's activations lives in a
// fixed array of this library instead of the context's growing workspace.
//
// The array is one per GPU (every device that loads this code object holds its own copy at
// its own address until the process ends). Host code never passes the array's name to a
// kernel: the name is a host-side stand-in. Its device address is looked up once per device
// with hipGetSymbolAddress while that device is current and kept; launches, like the
// workspace's, take that address as an ordinary pointer argument.
//
// Every call on a GPU shares that GPU's array and finds the last call's contents in it. The
// narrowing kernel writes every byte the multiply reads (tokens past the step's end are
// outside the range-checked buffer and read as zero), so nothing has to start at zero.
// Calls that overlap on one GPU (two streams, two threads) race on the array.
#include <hip/hip_runtime.h>

#include <mutex>

#include "common.h"

namespace zhip {

zhip_result launch_matmul_q8_0_float_mfma(const Dispatch &d);

namespace {

constexpr uint64_t kScratchBytes = 8ull << 20;  // 1024 tokens x 4096 inputs as bf16
constexpr int kMaxDevices = 64;

static __device__ __align__(256) uint8_t scratch[kScratchBytes];

struct PerDevice {
    uint8_t *ptr = nullptr;  // the device's own copy of `scratch`
    DeviceInfo info;
};
PerDevice g_devices[kMaxDevices];
std::mutex g_mutex;

}  // namespace

// Looks up this device's address of the array. The device must be current.
zhip_result no_alloc_setup(int device, const DeviceInfo &info) {
    if (device < 0 || device >= kMaxDevices) return ZHIP_E_INVALID_ARGUMENT;
    std::lock_guard<std::mutex> lock(g_mutex);
    PerDevice &pd = g_devices[device];
    if (pd.ptr) return ZHIP_OK;
    uint8_t *ptr = nullptr;
    if (hipGetSymbolAddress(reinterpret_cast<void **>(&ptr), HIP_SYMBOL(scratch)) != hipSuccess || !ptr) {
        (void)hipGetLastError();
        return ZHIP_E_GPU;
    }
    // Every kernel the entry point can launch opts in to its LDS now, so that the call itself
    // does no one-time set-up.
    if (!(matmul_mfma_prepare_no_alloc() && matmul_mfma_wide_prepare_no_alloc() && matmul_stream_prepare_no_alloc() && matmul_q8_bf16_prepare_no_alloc() && matmul_q8_bf16_wide_prepare_no_alloc())) return ZHIP_E_GPU;
    pd.info = info;
    pd.ptr = ptr;
    return ZHIP_OK;
}

uint64_t no_alloc_capacity() { return kScratchBytes; }

// out[t * out_stride + col0 + j] (+)= sum_i x[t * k + i] * w[j][i] for rows tokens and n
// outputs; w in split rows (k int8 values, k / 32 f16 scales, zero pad to 16 bytes). The same
// launches, in the same order, as a matmul_q8_0_float dispatch of variant 0xfffb0000, with
// the fixed array in place of the workspace. Asynchronous on `stream`.
zhip_result no_alloc_matmul_q8_0_float(int device, hipStream_t stream, const float *x, const void *w, float *out, uint32_t rows, uint32_t n,
    uint32_t k, uint32_t col0, uint32_t out_stride, uint32_t accumulate, char *err, size_t err_cap) {
    Dispatch d;
    d.err = err;
    d.err_cap = err_cap;
    if (device < 0 || device >= kMaxDevices || !g_devices[device].ptr) return fail(d, ZHIP_E_GPU, "matmul_q8_0_float (no allocation): device %d was not set up", device);
    if (!x || !w || !out) return fail(d, ZHIP_E_INVALID_ARGUMENT, "matmul_q8_0_float (no allocation): null operand");
    if (rows == 0 || n == 0) return ZHIP_OK;
    const uint64_t narrowed = (uint64_t)rows * k * 2u;
    if (narrowed > kScratchBytes)
        return fail(d, ZHIP_E_BAD_COMMAND, "matmul_q8_0_float (no allocation): %u tokens x %u inputs need %llu bytes of scratch, the fixed array holds %llu",
            rows, k, (unsigned long long)narrowed, (unsigned long long)kScratchBytes);
    if (out_stride < col0 + n && rows > 1) return fail(d, ZHIP_E_BAD_COMMAND, "matmul_q8_0_float (no allocation): out_stride %u is less than col0 + n = %u", out_stride, col0 + n);
    MatmulParams p{};
    p.rows = rows; p.n = n; p.k = k; p.col0 = col0; p.out_stride = out_stride; p.accumulate = accumulate ? 1u : 0u;
    p.k_slice = k; p.slice_stride = 0;
    const uint64_t row_bytes = ((uint64_t)k + k / 16u + 15u) & ~15ull;
    d.params = reinterpret_cast<const uint8_t *>(&p);
    d.params_size = sizeof p;
    // The caller vouches for its pointers: the ranges are exactly what the multiply touches.
    d.bind[1] = Bind{reinterpret_cast<uint8_t *>(const_cast<float *>(x)), (uint64_t)rows * k * 4u, true};
    d.bind[2] = Bind{reinterpret_cast<uint8_t *>(const_cast<void *>(w)), (uint64_t)n * row_bytes, true};
    d.bind[3] = Bind{reinterpret_cast<uint8_t *>(out), ((uint64_t)(rows - 1) * out_stride + col0 + n) * 4u, true};
    const uint64_t gx = ((uint64_t)n + 63u) / 64u, gy = ((uint64_t)rows + 15u) / 16u;
    if (gx > 65535u || gy > 65535u) return fail(d, ZHIP_E_BAD_COMMAND, "matmul_q8_0_float (no allocation): grid too large");
    d.grid[0] = (uint32_t)gx; d.grid[1] = (uint32_t)gy; d.grid[2] = 1;
    d.variant = 0xfffb0000u;
    d.stream = stream;
    d.dev = &g_devices[device].info;
    Workspace fixed;
    fixed.data = g_devices[device].ptr;
    fixed.bytes = kScratchBytes;
    fixed.fixed = true;
    d.work = &fixed;
    return launch_matmul_q8_0_float_mfma(d);
}

}  // namespace zhip
