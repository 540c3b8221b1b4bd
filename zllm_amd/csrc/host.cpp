// The HIP host: zllm's command stream (src/gpu/cmd.zig) interpreted on one
// in-order HIP stream, behind the C ABI of include/zllm_hip.h.
//
// Semantics kept from the reference's native hosts (src/agility/host.zig:1-16,
// 293-466; src/gpu/dawn_host.zig:1-6,120-246):
//   - write_buffer / write_file land before the next submit's work, even work
//     recorded ahead of them. Dispatches, copies, clears and reads are only
//     queued while a batch is interpreted and run at the submit, so a write
//     can be applied to device memory the moment it is decoded: every earlier
//     submit has finished (submits block) and nothing queued has started.
//   - queued work runs in recorded order on one in-order stream, which gives
//     the ordering WebGPU gives dispatches in a pass without hazard tracking.
//   - submit blocks, then reports one completion per pending read and one for
//     its own token.
//   - ids are assigned by the recorder and never reused; a buffer destroyed
//     while work is queued is released after the submit.
//
// Binding 0 of every kernel is a small uniform parameter block. The host keeps
// a shadow copy of every uniform-usage buffer (they are only ever written by
// write_buffer in the reference's planner), so a dispatch reads its parameters
// on the CPU, validates every bound range against them, and passes them to the
// kernel by value. A uniform buffer the GPU wrote is read back on demand.
#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <new>
#include <string>
#include <vector>

#include "common.h"

#ifndef ZHIP_SOURCE_HASH
#define ZHIP_SOURCE_HASH "dev"
#endif

namespace zhip {

// ---- kernel catalog -------------------------------------------------------------

// kernels.Kernel in declaration order (src/kernels/kernels.zig:24-92): the
// ordinal create_kernel carries.
static const char *const kKernelNames[] = {
    "rmsnorm", "matmul_bf16", "matmul_f16", "matmul_reduce", "matvec_bf16", "matvec_f16", "silu_mul", "embed_bf16",
    "embed_f16", "rope_append", "attn_split", "attn_split_wide", "attn_split_sparse", "attn_combine", "qsa_keys",
    "qsa_pool", "qsa_score", "qsa_select", "delta_prep", "delta_rule", "gated_norm", "mark_tokens", "sample", "draft",
    "gyro_matvec", "gyro_matmul", "moe_group", "moe_logits", "moe_route", "rotate128", "moe_combine", "hc_act", "hc_mix",
    "hc_combine", "ple_mix", "ple_conv", "repad", "repack_q3_k", "repack_q8_0", "quantize_q8", "matvec_q8_0",
    "matvec_q3_k", "matvec_q4_k", "matvec_q5_k", "matvec_q6_k", "matmul_q8_0", "matmul_q8_0_float", "matmul_q3_k",
    "matmul_q4_k", "matmul_q5_k", "matmul_q6_k", "embed_q8_0", "embed_q3_k", "embed_q4_k", "embed_q5_k", "embed_q6_k",
    "embed_iq4_xs",
};
static constexpr int kKernelCount = sizeof(kKernelNames) / sizeof(kKernelNames[0]);
static_assert(kKernelCount == 57, "kernels.Kernel has 57 members");

// Reserved create_kernel variants of the prefill identities
// (src/agility/kernels.zig:114-131) and this backend's own rung.
static constexpr uint32_t kVariantFp16Single = 0xfffc0000u;
static constexpr uint32_t kVariantFp16Compensated = 0xffff0000u;
static constexpr uint32_t kVariantBf16 = 0xfffb0000u;   // bf16 MFMA, f32 activations bound as the contract says
static constexpr uint32_t kVariantBf16X = 0xfffa0000u;  // bf16 MFMA, activations bound as packed bf16 (an extension)

enum class VariantKind { none, matvec, prefill };

zhip_result launch_matmul_bf16_f32(const Dispatch &);
zhip_result launch_matmul_f16_f32(const Dispatch &);
zhip_result launch_matmul_q8_0_float_f32(const Dispatch &);
zhip_result launch_matmul_bf16_mfma(const Dispatch &);
zhip_result launch_matmul_q8_0_float_mfma(const Dispatch &);
zhip_result launch_matmul_bf16_mfma_xbf16(const Dispatch &);
zhip_result launch_matmul_q8_0_float_mfma_xbf16(const Dispatch &);
zhip_result launch_matmul_bf16_f16(const Dispatch &);
zhip_result launch_matmul_f16_f16(const Dispatch &);
zhip_result launch_matmul_q8_0_float_f16(const Dispatch &);
zhip_result launch_matmul_bf16_f16c(const Dispatch &);
zhip_result launch_matmul_f16_f16c(const Dispatch &);
zhip_result launch_matmul_q8_0_float_f16c(const Dispatch &);

struct KernelInfo {
    const char *name;
    uint32_t count;   // bindings 0 .. count - 1 (Kernel.contract, src/kernels/kernels.zig:181-207)
    uint32_t writes;  // bit i: binding i is read_write
    VariantKind variants;
    LaunchFn launch;       // variant 0 / MatvecVariant ids
    LaunchFn launch_bf16;  // the bf16 MFMA rung of a prefill identity
    LaunchFn launch_bf16x; // the same with packed bf16 activations
    LaunchFn launch_f16;   // the reference's fp16_single rung
    LaunchFn launch_f16c;  // the reference's fp16_compensated rung
    int revision;          // bumped when the implementation changes (plan-cache key)
};

static const KernelInfo kImplemented[] = {
    {"matvec_q8_0", 5, 0b01000, VariantKind::matvec, launch_matvec_q8_0, nullptr, nullptr, nullptr, nullptr, 1},
    {"matvec_q3_k", 5, 0b01000, VariantKind::matvec, launch_matvec_q3_k, nullptr, nullptr, nullptr, nullptr, 1},
    {"matvec_q4_k", 5, 0b01000, VariantKind::matvec, launch_matvec_q4_k, nullptr, nullptr, nullptr, nullptr, 1},
    {"matvec_q5_k", 5, 0b01000, VariantKind::matvec, launch_matvec_q5_k, nullptr, nullptr, nullptr, nullptr, 1},
    {"matvec_q6_k", 5, 0b01000, VariantKind::matvec, launch_matvec_q6_k, nullptr, nullptr, nullptr, nullptr, 1},
    {"matvec_bf16", 5, 0b01000, VariantKind::none, launch_matvec_bf16, nullptr, nullptr, nullptr, nullptr, 1},
    {"matvec_f16", 5, 0b01000, VariantKind::none, launch_matvec_f16, nullptr, nullptr, nullptr, nullptr, 1},
    {"matmul_f16", 4, 0b1000, VariantKind::prefill, launch_matmul_f16_f32, nullptr, nullptr, launch_matmul_f16_f16, launch_matmul_f16_f16c, 1},
    {"matmul_bf16", 4, 0b1000, VariantKind::prefill, launch_matmul_bf16_f32, launch_matmul_bf16_mfma, launch_matmul_bf16_mfma_xbf16, launch_matmul_bf16_f16, launch_matmul_bf16_f16c, 1},
    {"matmul_q8_0_float", 4, 0b1000, VariantKind::prefill, launch_matmul_q8_0_float_f32, launch_matmul_q8_0_float_mfma, launch_matmul_q8_0_float_mfma_xbf16, launch_matmul_q8_0_float_f16, launch_matmul_q8_0_float_f16c, 1},
    {"matmul_q8_0", 5, 0b01000, VariantKind::none, launch_matmul_q8_0, nullptr, nullptr, nullptr, nullptr, 1},
    {"matmul_q3_k", 5, 0b01000, VariantKind::none, launch_matmul_q3_k, nullptr, nullptr, nullptr, nullptr, 1},
    {"matmul_q4_k", 5, 0b01000, VariantKind::none, launch_matmul_q4_k, nullptr, nullptr, nullptr, nullptr, 1},
    {"matmul_q5_k", 5, 0b01000, VariantKind::none, launch_matmul_q5_k, nullptr, nullptr, nullptr, nullptr, 1},
    {"matmul_q6_k", 5, 0b01000, VariantKind::none, launch_matmul_q6_k, nullptr, nullptr, nullptr, nullptr, 1},
    {"quantize_q8", 5, 0b01100, VariantKind::none, launch_quantize_q8, nullptr, nullptr, nullptr, nullptr, 1},
    {"matmul_reduce", 3, 0b100, VariantKind::none, launch_matmul_reduce, nullptr, nullptr, nullptr, nullptr, 1},
    {"silu_mul", 3, 0b100, VariantKind::none, launch_silu_mul, nullptr, nullptr, nullptr, nullptr, 1},
    {"repack_q8_0", 3, 0b100, VariantKind::none, launch_repack_q8_0, nullptr, nullptr, nullptr, nullptr, 1},
    {"repack_q3_k", 3, 0b100, VariantKind::none, launch_repack_q3_k, nullptr, nullptr, nullptr, nullptr, 1},
    {"repad", 3, 0b100, VariantKind::none, launch_repad, nullptr, nullptr, nullptr, nullptr, 1},
    {"embed_q8_0", 4, 0b1000, VariantKind::none, launch_embed_q8_0, nullptr, nullptr, nullptr, nullptr, 1},
    {"embed_q3_k", 4, 0b1000, VariantKind::none, launch_embed_q3_k, nullptr, nullptr, nullptr, nullptr, 1},
    {"embed_q4_k", 4, 0b1000, VariantKind::none, launch_embed_q4_k, nullptr, nullptr, nullptr, nullptr, 1},
    {"embed_q5_k", 4, 0b1000, VariantKind::none, launch_embed_q5_k, nullptr, nullptr, nullptr, nullptr, 1},
    {"embed_q6_k", 4, 0b1000, VariantKind::none, launch_embed_q6_k, nullptr, nullptr, nullptr, nullptr, 1},
    {"embed_bf16", 4, 0b1000, VariantKind::none, launch_embed_bf16, nullptr, nullptr, nullptr, nullptr, 1},
    {"embed_f16", 4, 0b1000, VariantKind::none, launch_embed_f16, nullptr, nullptr, nullptr, nullptr, 1},
    {"embed_iq4_xs", 4, 0b1000, VariantKind::none, launch_embed_iq4_xs, nullptr, nullptr, nullptr, nullptr, 1},
};

static const KernelInfo *find_kernel(const char *name, size_t len) {
    for (const KernelInfo &k : kImplemented)
        if (strlen(k.name) == len && memcmp(k.name, name, len) == 0) return &k;
    return nullptr;
}

static int ordinal_of(const char *name) {
    for (int i = 0; i < kKernelCount; i++)
        if (strcmp(kKernelNames[i], name) == 0) return i;
    return -1;
}

// ---- launch helpers shared with the kernel files ----------------------------------

zhip_result fail(const Dispatch &d, zhip_result code, const char *fmt, ...) {
    if (d.err && d.err_cap) {
        va_list ap;
        va_start(ap, fmt);
        vsnprintf(d.err, d.err_cap, fmt, ap);
        va_end(ap);
    }
    return code;
}

zhip_result check_launch(const Dispatch &d, const char *kernel) {
    const hipError_t e = hipGetLastError();
    if (e == hipSuccess) return ZHIP_OK;
    return fail(d, ZHIP_E_GPU, "%s: launch failed: %s", kernel, hipGetErrorString(e));
}

// ---- context ----------------------------------------------------------------------

static constexpr uint32_t kUsageUniform = 0x40;  // cmd.Usage.uniform (src/gpu/cmd.zig:62-74)
static constexpr size_t kTimingCapacity = 4096;  // timed dispatches per submit

struct Buffer {
    uint8_t *dev = nullptr;
    uint64_t size = 0;
    uint32_t usage = 0;
    bool alive = false;
    bool shadowed = false;      // a host copy is kept up to date by write_buffer
    bool shadow_stale = false;  // the GPU wrote it since
    std::vector<uint8_t> shadow;
};

struct Pipeline {
    bool alive = false;
    bool missing = false;  // created with an empty artifact
    uint32_t kernel = 0;   // the ordinal the recorder sent (reports only)
    uint32_t variant = 0;
    const KernelInfo *info = nullptr;
    LaunchFn launch = nullptr;
};

struct Entry {
    bool bound = false;
    uint32_t buffer = 0;
    uint64_t offset = 0, size = 0;
};

struct Group {
    bool alive = false;
    Entry e[8];
};

struct Op {
    enum Kind { dispatch, copy, fill, read } kind;
    // dispatch
    uint32_t pipeline = 0;
    uint32_t grid[3] = {0, 0, 0};
    Group group;
    // copy / fill / read
    uint32_t src = 0, dst = 0;
    uint64_t src_offset = 0, dst_offset = 0, size = 0;
};

struct Read {
    uint32_t token;
    uint8_t *dst;
    uint64_t staging_offset, size;
};

struct TimingKey {
    uint32_t pipeline, grid[3];
    bool operator<(const TimingKey &o) const {
        if (pipeline != o.pipeline) return pipeline < o.pipeline;
        return memcmp(grid, o.grid, sizeof grid) < 0;
    }
};
struct TimingTotal { uint64_t ns = 0, count = 0; };

}  // namespace zhip

using namespace zhip;

// Growing replaces the allocation, so earlier dispatches that may still be
// running with the old one are waited for first.
zhip_result Workspace::reserve(const Dispatch &d, uint64_t want) {
    if (want <= bytes) return ZHIP_OK;
    if (fixed) return fail(d, ZHIP_E_BAD_COMMAND, "workspace: %llu bytes wanted, the fixed scratch holds %llu", (unsigned long long)want, (unsigned long long)bytes);
    const uint64_t size = (want + (8u << 20) - 1) & ~(uint64_t)((8u << 20) - 1);
    if (hipStreamSynchronize(d.stream) != hipSuccess) return fail(d, ZHIP_E_GPU, "workspace: stream synchronisation failed");
    if (data) (void)hipFree(data);
    data = nullptr;
    bytes = 0;
    const hipError_t e = hipMalloc(reinterpret_cast<void **>(&data), size);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        data = nullptr;
        return fail(d, e == hipErrorOutOfMemory ? ZHIP_E_OUT_OF_MEMORY : ZHIP_E_GPU, "workspace: cannot allocate %llu bytes", (unsigned long long)size);
    }
    bytes = size;
    return ZHIP_OK;
}

void Workspace::release() {
    if (data && !fixed) (void)hipFree(data);
    data = nullptr;
    bytes = 0;
}

struct zhip_context {
    int device = 0;
    hipStream_t stream = nullptr;
    hipEvent_t ev_begin = nullptr, ev_end = nullptr;
    DeviceInfo info;
    Workspace work;
    zhip_caps caps{};
    bool lost = false;
    std::string message;

    std::vector<Buffer> buffers;
    std::vector<Pipeline> pipelines;
    std::vector<Group> groups;
    std::vector<Op> ops;
    std::vector<Read> reads;
    uint64_t read_bytes = 0;
    std::vector<uint32_t> released;
    uint8_t *download = nullptr;  // pinned
    uint64_t download_size = 0;

    const uint8_t *file = nullptr;
    size_t file_len = 0;

    bool profiling = false;
    std::map<TimingKey, TimingTotal> timings;
    uint64_t untimed = 0;
    std::vector<hipEvent_t> events;
    uint64_t last_ns = 0, last_dispatches = 0;

    // Replayed submits: a submit that is nothing but dispatches (then reads) and has been
    // seen before with exactly the same launches runs as a HIP graph (see submit()).
    struct Replay {
        std::vector<uint8_t> key;   // every launch's function, grid, bound ranges and parameter bytes
        hipGraphExec_t exec = nullptr;
        bool unusable = false;      // capturing it failed once: stay eager
        uint64_t used = 0;
    };
    std::vector<Replay> replays;
    uint64_t replay_clock = 0;
    bool use_graphs = true;
    uint64_t replayed_submits = 0;
};

namespace {

zhip_result set_error(zhip_context *c, zhip_result code, const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    c->message = buf;
    return code;
}

zhip_result hip_check(zhip_context *c, hipError_t e, const char *what) {
    if (e == hipSuccess) return ZHIP_OK;
    (void)hipGetLastError();
    if (e == hipErrorOutOfMemory) return set_error(c, ZHIP_E_OUT_OF_MEMORY, "%s: %s", what, hipGetErrorString(e));
    return set_error(c, ZHIP_E_GPU, "%s: %s", what, hipGetErrorString(e));
}

inline uint64_t join(uint32_t lo, uint32_t hi) { return ((uint64_t)hi << 32) | lo; }

template <class T>
zhip_result put(zhip_context *c, std::vector<T> &list, uint32_t id, T &&obj) {
    if (id > (1u << 24)) return set_error(c, ZHIP_E_BAD_ID, "object id %u is not dense", id);
    if (id >= list.size()) list.resize((size_t)id + 1);
    if (list[id].alive) return set_error(c, ZHIP_E_BAD_ID, "object id %u is already in use", id);
    list[id] = std::move(obj);
    list[id].alive = true;
    return ZHIP_OK;
}

template <class T>
T *get(std::vector<T> &list, uint32_t id) {
    if (id >= list.size() || !list[id].alive) return nullptr;
    return &list[id];
}

void drop_pending(zhip_context *c) {
    c->ops.clear();
    c->reads.clear();
    c->read_bytes = 0;
}

zhip_result release_buffer(zhip_context *c, uint32_t id) {
    Buffer *b = get(c->buffers, id);
    if (!b) return set_error(c, ZHIP_E_BAD_ID, "destroy: buffer %u does not exist", id);
    const hipError_t e = hipFree(b->dev);
    *b = Buffer{};
    return hip_check(c, e, "hipFree");
}

// Brings a buffer's host copy up to date, reading it back if the GPU wrote it
// (or if it is not a uniform-usage buffer and so was never shadowed).
zhip_result refresh_shadow(zhip_context *c, Buffer &b) {
    if (b.shadowed && !b.shadow_stale) return ZHIP_OK;
    if (zhip_result r = hip_check(c, hipStreamSynchronize(c->stream), "hipStreamSynchronize")) return r;
    b.shadow.resize(b.size);
    if (zhip_result r = hip_check(c, hipMemcpy(b.shadow.data(), b.dev, b.size, hipMemcpyDeviceToHost), "hipMemcpy (params readback)")) return r;
    // Only uniform-usage buffers stay shadowed; others are read back per use.
    b.shadow_stale = !b.shadowed;
    return ZHIP_OK;
}

void mark_written(Buffer &b) {
    if (b.shadowed) b.shadow_stale = true;
}

// Resolves a queued dispatch: its pipeline, the device ranges of its bindings and
// its parameter block on the host. `err` receives the launcher's message.
zhip_result prepare_dispatch(zhip_context *c, const Op &op, Dispatch &d, Pipeline *&pl, char *err, size_t err_cap) {
    pl = get(c->pipelines, op.pipeline);
    // The pipeline was checked when the dispatch was recorded and destroys of
    // pipelines are not deferred, so look it up again.
    if (!pl || !pl->launch) return set_error(c, ZHIP_E_BAD_ID, "dispatch: pipeline %u was destroyed before the submit", op.pipeline);
    d.stream = c->stream;
    d.dev = &c->info;
    d.work = &c->work;
    d.variant = pl->variant;
    memcpy(d.grid, op.grid, sizeof d.grid);
    err[0] = 0;
    d.err = err;
    d.err_cap = err_cap;
    for (uint32_t b = 0; b < 8; b++) {
        const Entry &e = op.group.e[b];
        if (!e.bound) continue;
        Buffer *buf = get(c->buffers, e.buffer);
        if (!buf) return set_error(c, ZHIP_E_BAD_ID, "dispatch: buffer %u of binding %u does not exist", e.buffer, b);
        if (e.offset > buf->size || e.size > buf->size - e.offset) return set_error(c, ZHIP_E_BAD_COMMAND, "dispatch: binding %u exceeds buffer %u", b, e.buffer);
        d.bind[b].ptr = buf->dev + e.offset;
        d.bind[b].size = e.size;
        d.bind[b].bound = true;
    }
    if (!op.group.e[0].bound) return set_error(c, ZHIP_E_BAD_COMMAND, "%s: no parameter block at binding 0", pl->info->name);
    Buffer *ub = get(c->buffers, op.group.e[0].buffer);
    if (zhip_result r = refresh_shadow(c, *ub)) return r;
    d.params = ub->shadow.data() + op.group.e[0].offset;
    d.params_size = op.group.e[0].size;
    return ZHIP_OK;
}

void mark_outputs(zhip_context *c, const Op &op, const Pipeline &pl) {
    for (uint32_t b = 1; b < 8; b++)
        if (op.group.e[b].bound && (pl.info->writes >> b & 1u))
            if (Buffer *buf = get(c->buffers, op.group.e[b].buffer)) mark_written(*buf);
}

zhip_result run_dispatch(zhip_context *c, const Op &op, size_t &timed) {
    Dispatch d;
    Pipeline *pl = nullptr;
    char err[384] = "";
    if (zhip_result r = prepare_dispatch(c, op, d, pl, err, sizeof err)) return r;

    const bool timed_now = c->profiling && timed < kTimingCapacity;
    if (c->profiling && !timed_now) c->untimed++;
    if (timed_now) {
        while (c->events.size() < 2 * (timed + 1)) {
            hipEvent_t ev;
            if (zhip_result r = hip_check(c, hipEventCreate(&ev), "hipEventCreate")) return r;
            c->events.push_back(ev);
        }
        if (zhip_result r = hip_check(c, hipEventRecord(c->events[2 * timed], c->stream), "hipEventRecord")) return r;
    }
    const zhip_result r = pl->launch(d);
    if (r != ZHIP_OK) {
        c->message = err[0] ? err : "kernel launch failed";
        return r;
    }
    if (timed_now) {
        if (zhip_result e = hip_check(c, hipEventRecord(c->events[2 * timed + 1], c->stream), "hipEventRecord")) return e;
        timed++;
    }
    mark_outputs(c, op, *pl);
    return ZHIP_OK;
}

// ---- replayed submits ------------------------------------------------------------------
// Launching a kernel costs the CPU about 2.9 us here; a HIP graph replays its kernels
// 1.6 us apart. A decode step is hundreds of launches of a few microseconds each, the same
// ones token after token, so a submit whose leading dispatches (everything before its
// reads) equal an earlier submit's exactly, function by function and byte by byte of their
// arguments, is replayed from a graph captured the second time it is seen (the first time
// it runs as it is, which also lets launchers do their one-time set-up outside a capture).
// Only kernels are captured: no copies, clears or memsets.
constexpr size_t kMinReplayDispatches = 8, kMaxReplays = 16;

// The leading dispatches of the queue if what follows them is only reads, else 0. Every
// parameter block must sit in a uniform-usage buffer whose host copy is current: any other
// would be read back from the GPU while the launches are resolved, which a capture forbids.
size_t replayable_prefix(zhip_context *c) {
    size_t n = 0;
    while (n < c->ops.size() && c->ops[n].kind == Op::dispatch) n++;
    for (size_t i = n; i < c->ops.size(); i++)
        if (c->ops[i].kind != Op::read) return 0;
    if (n < kMinReplayDispatches) return 0;
    for (size_t i = 0; i < n; i++) {
        const Entry &e = c->ops[i].group.e[0];
        const Buffer *ub = e.bound ? get(c->buffers, e.buffer) : nullptr;
        if (!ub || !ub->shadowed || ub->shadow_stale) return 0;
        // A kernel of the prefix that writes a parameter buffer: a later dispatch would
        // have to see the written values, and a captured launch holds the ones from before.
        const Pipeline *pl = get(c->pipelines, c->ops[i].pipeline);
        if (!pl || !pl->info) return 0;
        for (uint32_t b = 1; b < 8; b++) {
            const Entry &w = c->ops[i].group.e[b];
            if (!w.bound || !(pl->info->writes >> b & 1u)) continue;
            const Buffer *wb = get(c->buffers, w.buffer);
            if (!wb || wb->shadowed) return 0;
        }
    }
    return n;
}

zhip_result replay_key(zhip_context *c, size_t count, std::vector<uint8_t> &key) {
    key.clear();
    auto put_bytes = [&](const void *p, size_t n) { key.insert(key.end(), (const uint8_t *)p, (const uint8_t *)p + n); };
    char err[384];
    // Launchers may point kernels at the workspace: a graph captured with an allocation
    // that has since been replaced must never match again.
    const uint64_t work[2] = {(uint64_t)(uintptr_t)c->work.data, c->work.bytes};
    put_bytes(work, sizeof work);
    for (size_t i = 0; i < count; i++) {
        Dispatch d;
        Pipeline *pl = nullptr;
        if (zhip_result r = prepare_dispatch(c, c->ops[i], d, pl, err, sizeof err)) return r;
        const LaunchFn fn = pl->launch;
        put_bytes(&fn, sizeof fn);
        put_bytes(&d.variant, sizeof d.variant);
        put_bytes(d.grid, sizeof d.grid);
        for (uint32_t b = 0; b < 8; b++) {
            const uint64_t range[3] = {d.bind[b].bound ? 1ull : 0ull, (uint64_t)(uintptr_t)d.bind[b].ptr, d.bind[b].size};
            put_bytes(range, sizeof range);
        }
        put_bytes(d.params, d.params_size);
    }
    return ZHIP_OK;
}

// Captures the queue's first `count` dispatches into an executable graph. Nothing runs.
zhip_result capture_replay(zhip_context *c, size_t count, hipGraphExec_t *out) {
    *out = nullptr;
    if (hipStreamBeginCapture(c->stream, hipStreamCaptureModeThreadLocal) != hipSuccess) {
        (void)hipGetLastError();
        return ZHIP_E_GPU;
    }
    zhip_result failed = ZHIP_OK;
    char err[384];
    for (size_t i = 0; i < count && failed == ZHIP_OK; i++) {
        Dispatch d;
        Pipeline *pl = nullptr;
        failed = prepare_dispatch(c, c->ops[i], d, pl, err, sizeof err);
        if (failed == ZHIP_OK) failed = pl->launch(d);
    }
    hipGraph_t graph = nullptr;
    const hipError_t ended = hipStreamEndCapture(c->stream, &graph);
    if (ended != hipSuccess || failed != ZHIP_OK || !graph) {
        (void)hipGetLastError();
        if (graph) (void)hipGraphDestroy(graph);
        return failed != ZHIP_OK ? failed : ZHIP_E_GPU;
    }
    const hipError_t made = hipGraphInstantiate(out, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    if (made != hipSuccess) {
        (void)hipGetLastError();
        *out = nullptr;
        return ZHIP_E_GPU;
    }
    return ZHIP_OK;
}

// The graph of the queue's first `count` dispatches if this exact sequence has been seen
// before (captured now if this is the second time), else null: the caller then runs them
// one by one.
zhip_result find_replay(zhip_context *c, size_t count, zhip_context::Replay **out) {
    *out = nullptr;
    std::vector<uint8_t> key;
    if (zhip_result r = replay_key(c, count, key)) return r;
    zhip_context::Replay *entry = nullptr;
    for (auto &e : c->replays)
        if (e.key.size() == key.size() && memcmp(e.key.data(), key.data(), key.size()) == 0) entry = &e;
    if (!entry) {
        // First sight: remember it (replacing the least recently used) and run as recorded.
        if (c->replays.size() < kMaxReplays) {
            c->replays.emplace_back();
            entry = &c->replays.back();
        } else {
            entry = &c->replays[0];
            for (auto &e : c->replays)
                if (e.used < entry->used) entry = &e;
            if (entry->exec) (void)hipGraphExecDestroy(entry->exec);
            *entry = zhip_context::Replay();
        }
        entry->key = std::move(key);
        entry->used = ++c->replay_clock;
        return ZHIP_OK;
    }
    entry->used = ++c->replay_clock;
    if (entry->unusable) return ZHIP_OK;
    if (!entry->exec && capture_replay(c, count, &entry->exec) != ZHIP_OK) {
        entry->unusable = true;
        entry->exec = nullptr;
        return ZHIP_OK;
    }
    *out = entry;
    return ZHIP_OK;
}

// Runs everything queued since the last submit, waits for it, completes reads.
zhip_result run_queue(zhip_context *c) {
    if (c->read_bytes > c->download_size) {
        if (c->download) (void)hipHostFree(c->download);
        c->download = nullptr;
        c->download_size = 0;
        const uint64_t size = std::max<uint64_t>(c->read_bytes, 1u << 20);
        if (zhip_result r = hip_check(c, hipHostMalloc(reinterpret_cast<void **>(&c->download), size, hipHostMallocDefault), "hipHostMalloc")) return r;
        c->download_size = size;
    }
    size_t timed = 0;
    std::vector<TimingKey> keys;
    uint64_t dispatches = 0;
    size_t next_read = 0;
    // Parameter blocks the GPU wrote are read back while resolving the launches: before the
    // timed region and before any capture.
    const size_t prefix = (c->use_graphs && !c->profiling) ? replayable_prefix(c) : 0;
    zhip_context::Replay *replay = nullptr;
    if (prefix > 0)
        if (zhip_result r = find_replay(c, prefix, &replay)) return r;
    if (zhip_result r = hip_check(c, hipEventRecord(c->ev_begin, c->stream), "hipEventRecord")) return r;
    bool replayed = false;
    if (replay) {
        if (hipGraphLaunch(replay->exec, c->stream) == hipSuccess) {
            for (size_t i = 0; i < prefix; i++)
                if (Pipeline *pl = get(c->pipelines, c->ops[i].pipeline)) mark_outputs(c, c->ops[i], *pl);
            c->replayed_submits++;
            dispatches = prefix;
            replayed = true;
        } else {
            (void)hipGetLastError();
            (void)hipGraphExecDestroy(replay->exec);
            replay->exec = nullptr;
            replay->unusable = true;
        }
    }
    for (size_t at = replayed ? prefix : 0; at < c->ops.size(); at++) {
        const Op &op = c->ops[at];
        switch (op.kind) {
        case Op::dispatch: {
            const size_t before = timed;
            if (zhip_result r = run_dispatch(c, op, timed)) return r;
            if (timed != before) keys.push_back(TimingKey{op.pipeline, {op.grid[0], op.grid[1], op.grid[2]}});
            dispatches++;
            break;
        }
        case Op::copy: {
            Buffer *s = get(c->buffers, op.src), *t = get(c->buffers, op.dst);
            if (!s || !t) return set_error(c, ZHIP_E_BAD_ID, "copy_buffer: a buffer was destroyed before the submit");
            if (zhip_result r = hip_check(c, hipMemcpyAsync(t->dev + op.dst_offset, s->dev + op.src_offset, op.size, hipMemcpyDeviceToDevice, c->stream), "hipMemcpyAsync")) return r;
            mark_written(*t);
            break;
        }
        case Op::fill: {
            Buffer *t = get(c->buffers, op.dst);
            if (!t) return set_error(c, ZHIP_E_BAD_ID, "clear_buffer: the buffer was destroyed before the submit");
            if (launch_fill(c->stream, t->dev + op.dst_offset, op.size / 4, 0) != ZHIP_OK) return set_error(c, ZHIP_E_GPU, "clear_buffer: launch failed");
            mark_written(*t);
            break;
        }
        case Op::read: {
            Buffer *s = get(c->buffers, op.src);
            if (!s) return set_error(c, ZHIP_E_BAD_ID, "read_buffer: the buffer was destroyed before the submit");
            const Read &rd = c->reads[next_read++];
            if (rd.size > 0)
                if (zhip_result r = hip_check(c, hipMemcpyAsync(c->download + rd.staging_offset, s->dev + op.src_offset, rd.size, hipMemcpyDeviceToHost, c->stream), "hipMemcpyAsync")) return r;
            break;
        }
        }
    }
    if (zhip_result r = hip_check(c, hipEventRecord(c->ev_end, c->stream), "hipEventRecord")) return r;
    if (zhip_result r = hip_check(c, hipStreamSynchronize(c->stream), "hipStreamSynchronize")) return r;
    float ms = 0.f;
    if (hipEventElapsedTime(&ms, c->ev_begin, c->ev_end) == hipSuccess) c->last_ns = (uint64_t)((double)ms * 1e6);
    c->last_dispatches = dispatches;
    for (size_t i = 0; i < timed; i++) {
        float dms = 0.f;
        if (hipEventElapsedTime(&dms, c->events[2 * i], c->events[2 * i + 1]) != hipSuccess) continue;
        TimingTotal &t = c->timings[keys[i]];
        t.ns += (uint64_t)((double)dms * 1e6);
        t.count++;
    }
    for (const Read &rd : c->reads)
        if (rd.size > 0) memcpy(rd.dst, c->download + rd.staging_offset, rd.size);
    return ZHIP_OK;
}

// A submit. When the queue fails part-way, what it had already started is still running
// on the stream: wait for it (whatever that wait says) so that later writes and frees,
// which do not order against the stream, cannot overtake it. Buffers destroyed while work
// was queued are released on both paths; an id destroyed twice is released once.
zhip_result submit(zhip_context *c) {
    zhip_result result = run_queue(c);
    std::string message;
    if (result != ZHIP_OK) {
        message = c->message;
        (void)hipStreamSynchronize(c->stream);
        (void)hipGetLastError();
    }
    c->ops.clear();
    std::vector<uint32_t> released;
    released.swap(c->released);
    for (uint32_t id : released) {
        if (!get(c->buffers, id)) continue;
        const zhip_result r = release_buffer(c, id);
        if (result == ZHIP_OK && r != ZHIP_OK) {
            result = r;
            message = c->message;
        }
    }
    if (result != ZHIP_OK) c->message = message;
    return result;
}

struct Command {
    uint32_t op;
    const uint32_t *a;
    size_t n;
    uint64_t u64(size_t i) const { return join(a[i], a[i + 1]); }
};

#define NEED(count)                                                                                      \
    do {                                                                                                 \
        if (cmd.n < (count)) return set_error(c, ZHIP_E_BAD_COMMAND, "command %u has %zu argument words, needs %d", cmd.op, cmd.n, (int)(count)); \
    } while (0)

zhip_result create_kernel(zhip_context *c, const Command &cmd) {
    const uint32_t *a = cmd.a;
    Pipeline p;
    p.kernel = a[1];
    p.variant = a[2];
    const uint32_t len = a[6];
    if (len == 0) {
        // A kernel the backend does not implement (src/gpu/cmd.zig:33-35).
        p.missing = true;
        return put(c, c->pipelines, a[0], std::move(p));
    }
    const char *art = reinterpret_cast<const char *>((uintptr_t)cmd.u64(4));
    // "zhip:v1:<kernel tag name>:<variant, 8 hex digits>"
    static const char prefix[] = "zhip:v1:";
    if (!art || len < sizeof prefix || memcmp(art, prefix, sizeof prefix - 1) != 0)
        return set_error(c, ZHIP_E_BAD_COMMAND, "create_kernel: artifact is not a zhip:v1 descriptor");
    const char *name = art + sizeof prefix - 1;
    size_t name_len = 0;
    while (sizeof prefix - 1 + name_len < len && name[name_len] != ':') name_len++;
    const KernelInfo *info = find_kernel(name, name_len);
    if (!info) return set_error(c, ZHIP_E_BAD_COMMAND, "create_kernel: no HIP implementation of kernel '%.*s'", (int)name_len, name);
    if (a[3] != info->writes) return set_error(c, ZHIP_E_BAD_COMMAND, "create_kernel: %s writes bindings 0x%x, the recorder says 0x%x", info->name, info->writes, a[3]);
    p.info = info;
    p.launch = info->launch;
    switch (info->variants) {
    case VariantKind::none:
        if (p.variant != 0) return set_error(c, ZHIP_E_BAD_COMMAND, "create_kernel: %s has no variant 0x%08x", info->name, p.variant);
        break;
    case VariantKind::matvec:
        if (p.variant != 0 && ((p.variant & 0xffu) == 0 || ((p.variant >> 8) & 0xffu) == 0 || ((p.variant >> 16) & 0xffu) == 0))
            return set_error(c, ZHIP_E_BAD_COMMAND, "create_kernel: %s variant 0x%08x is not a MatvecVariant id", info->name, p.variant);
        break;
    case VariantKind::prefill:
        if (p.variant == kVariantFp16Single) p.launch = info->launch_f16;
        else if (p.variant == kVariantFp16Compensated) p.launch = info->launch_f16c;
        else if (p.variant == kVariantBf16) p.launch = info->launch_bf16;
        else if (p.variant == kVariantBf16X) p.launch = info->launch_bf16x;
        else if (p.variant != 0) return set_error(c, ZHIP_E_BAD_COMMAND, "create_kernel: %s has no variant 0x%08x", info->name, p.variant);
        if (!p.launch) return set_error(c, ZHIP_E_UNSUPPORTED_PREFILL, "create_kernel: %s has only the f32 rung", info->name);
        break;
    }
    return put(c, c->pipelines, a[0], std::move(p));
}

zhip_result run_command(zhip_context *c, const Command &cmd, zhip_completion *out, size_t *n_out) {
    const uint32_t *a = cmd.a;
    switch (cmd.op) {
    case 1: {  // create_buffer: id, size: u64, usage
        NEED(4);
        const uint64_t size = cmd.u64(1);
        if (size > c->caps.memory_bytes) return set_error(c, ZHIP_E_OUT_OF_MEMORY, "create_buffer: %llu bytes exceed device memory", (unsigned long long)size);
        Buffer b;
        b.size = size;
        b.usage = a[3];
        const uint64_t alloc = std::max<uint64_t>((size + 255u) & ~255ull, 256u);
        if (zhip_result r = hip_check(c, hipMalloc(reinterpret_cast<void **>(&b.dev), alloc), "hipMalloc")) return r;
        // New buffers read as zero, as WebGPU's do.
        if (zhip_result r = hip_check(c, hipMemset(b.dev, 0, alloc), "hipMemset")) { (void)hipFree(b.dev); return r; }
        if (b.usage & kUsageUniform) {
            b.shadowed = true;
            b.shadow.assign(size, 0);
        }
        uint8_t *dev = b.dev;
        const zhip_result r = put(c, c->buffers, a[0], std::move(b));
        if (r != ZHIP_OK) (void)hipFree(dev);
        return r;
    }
    case 2: {  // write_buffer: buffer, offset: u64, data: ptr, len: u64
        NEED(7);
        Buffer *b = get(c->buffers, a[0]);
        if (!b) return set_error(c, ZHIP_E_BAD_ID, "write_buffer: buffer %u does not exist", a[0]);
        const uint64_t offset = cmd.u64(1), len = cmd.u64(5);
        if (len % 4 != 0 || offset % 4 != 0 || offset > b->size || len > b->size - offset) return set_error(c, ZHIP_E_BAD_COMMAND, "write_buffer: range %llu+%llu outside buffer %u of %llu bytes", (unsigned long long)offset, (unsigned long long)len, a[0], (unsigned long long)b->size);
        if (len == 0) return ZHIP_OK;
        const void *data = reinterpret_cast<const void *>((uintptr_t)cmd.u64(3));
        if (!data) return set_error(c, ZHIP_E_BAD_COMMAND, "write_buffer: null data");
        if (zhip_result r = hip_check(c, hipMemcpy(b->dev + offset, data, len, hipMemcpyHostToDevice), "hipMemcpy (write_buffer)")) return r;
        if (b->shadowed && !b->shadow_stale) memcpy(b->shadow.data() + offset, data, len);
        return ZHIP_OK;
    }
    case 12: {  // write_file: buffer, offset: u64, file_offset: u64, size: u64
        NEED(7);
        Buffer *b = get(c->buffers, a[0]);
        if (!b) return set_error(c, ZHIP_E_BAD_ID, "write_file: buffer %u does not exist", a[0]);
        const uint64_t offset = cmd.u64(1), file_offset = cmd.u64(3), size = cmd.u64(5);
        if (!c->file) return set_error(c, ZHIP_E_BAD_COMMAND, "write_file: no model file set");
        if (file_offset > c->file_len || size > c->file_len - file_offset || offset > b->size || size > b->size - offset || (offset | size) % 4 != 0)
            return set_error(c, ZHIP_E_BAD_COMMAND, "write_file: range outside the file or the buffer");
        if (size == 0) return ZHIP_OK;
        if (zhip_result r = hip_check(c, hipMemcpy(b->dev + offset, c->file + file_offset, size, hipMemcpyHostToDevice), "hipMemcpy (write_file)")) return r;
        if (b->shadowed && !b->shadow_stale) memcpy(b->shadow.data() + offset, c->file + file_offset, size);
        return ZHIP_OK;
    }
    case 3:  // create_kernel: id, kernel, variant, writes, artifact: ptr, len
        NEED(7);
        return create_kernel(c, cmd);
    case 5: {  // create_bind_group: id, pipeline, group, count, count x (binding, buffer, offset: u64, size: u64)
        NEED(4);
        const uint32_t count = a[3];
        if (cmd.n != 4 + (size_t)count * 6 || a[2] != 0) return set_error(c, ZHIP_E_BAD_COMMAND, "create_bind_group: malformed (group %u, %u entries, %zu words)", a[2], count, cmd.n);
        Group g;
        for (uint32_t i = 0; i < count; i++) {
            const uint32_t *e = a + 4 + (size_t)i * 6;
            if (e[0] >= 8) return set_error(c, ZHIP_E_BAD_COMMAND, "create_bind_group: binding %u out of range", e[0]);
            Buffer *b = get(c->buffers, e[1]);
            if (!b) return set_error(c, ZHIP_E_BAD_ID, "create_bind_group: buffer %u does not exist", e[1]);
            const uint64_t offset = join(e[2], e[3]), size = join(e[4], e[5]);
            if (offset > b->size || size > b->size - offset) return set_error(c, ZHIP_E_BAD_COMMAND, "create_bind_group: binding %u range outside buffer %u", e[0], e[1]);
            g.e[e[0]] = Entry{true, e[1], offset, size};
        }
        return put(c, c->groups, a[0], std::move(g));
    }
    case 6: {  // dispatch: pipeline, x, y, z, count, groups...
        NEED(5);
        if (cmd.n != 5 + (size_t)a[4] || a[4] > 1) return set_error(c, ZHIP_E_BAD_COMMAND, "dispatch: %u bind groups", a[4]);
        Pipeline *pl = get(c->pipelines, a[0]);
        if (!pl) return set_error(c, ZHIP_E_BAD_ID, "dispatch: pipeline %u does not exist", a[0]);
        Op op;
        op.kind = Op::dispatch;
        op.pipeline = a[0];
        memcpy(op.grid, a + 1, sizeof op.grid);
        if (a[4] == 1) {
            Group *g = get(c->groups, a[5]);
            if (!g) return set_error(c, ZHIP_E_BAD_ID, "dispatch: bind group %u does not exist", a[5]);
            op.group = *g;
        }
        if (pl->missing) {
            const char *name = pl->kernel < (uint32_t)kKernelCount ? kKernelNames[pl->kernel] : "?";
            drop_pending(c);
            return set_error(c, ZHIP_E_UNSUPPORTED_KERNEL, "kernel %s has no HIP implementation", name);
        }
        if (op.grid[0] > 65535u || op.grid[1] > 65535u || op.grid[2] > 65535u) return set_error(c, ZHIP_E_BAD_COMMAND, "dispatch: grid dimension above 65535");
        c->ops.push_back(op);
        return ZHIP_OK;
    }
    case 7: {  // copy_buffer: src, src_offset: u64, dst, dst_offset: u64, size: u64
        NEED(8);
        Buffer *s = get(c->buffers, a[0]), *t = get(c->buffers, a[3]);
        if (!s || !t) return set_error(c, ZHIP_E_BAD_ID, "copy_buffer: buffer %u or %u does not exist", a[0], a[3]);
        const uint64_t so = cmd.u64(1), dof = cmd.u64(4), size = cmd.u64(6);
        if ((so | dof | size) % 4 != 0 || so > s->size || size > s->size - so || dof > t->size || size > t->size - dof) return set_error(c, ZHIP_E_BAD_COMMAND, "copy_buffer: range outside a buffer");
        if (size == 0) return ZHIP_OK;
        Op op;
        op.kind = Op::copy;
        op.src = a[0]; op.dst = a[3]; op.src_offset = so; op.dst_offset = dof; op.size = size;
        c->ops.push_back(op);
        return ZHIP_OK;
    }
    case 11: {  // clear_buffer: buffer, offset: u64, size: u64
        NEED(5);
        Buffer *t = get(c->buffers, a[0]);
        if (!t) return set_error(c, ZHIP_E_BAD_ID, "clear_buffer: buffer %u does not exist", a[0]);
        const uint64_t offset = cmd.u64(1), size = cmd.u64(3);
        if ((offset | size) % 4 != 0 || offset > t->size || size > t->size - offset) return set_error(c, ZHIP_E_BAD_COMMAND, "clear_buffer: range outside buffer %u", a[0]);
        if (size == 0) return ZHIP_OK;
        Op op;
        op.kind = Op::fill;
        op.dst = a[0]; op.dst_offset = offset; op.size = size;
        c->ops.push_back(op);
        return ZHIP_OK;
    }
    case 8: {  // read_buffer: token, buffer, offset: u64, size: u64, dst: ptr
        NEED(8);
        Buffer *s = get(c->buffers, a[1]);
        if (!s) return set_error(c, ZHIP_E_BAD_ID, "read_buffer: buffer %u does not exist", a[1]);
        const uint64_t offset = cmd.u64(2), size = cmd.u64(4);
        if ((offset | size) % 4 != 0 || offset > s->size || size > s->size - offset) return set_error(c, ZHIP_E_BAD_COMMAND, "read_buffer: range outside buffer %u", a[1]);
        uint8_t *dst = reinterpret_cast<uint8_t *>((uintptr_t)cmd.u64(6));
        if (!dst && size > 0) return set_error(c, ZHIP_E_BAD_COMMAND, "read_buffer: null destination");
        const uint64_t at = (c->read_bytes + 255u) & ~255ull;
        c->read_bytes = at + size;
        c->reads.push_back(Read{a[0], dst, at, size});
        Op op;
        op.kind = Op::read;
        op.src = a[1]; op.src_offset = offset; op.size = size;
        c->ops.push_back(op);
        return ZHIP_OK;
    }
    case 9: {  // submit: token
        NEED(1);
        const zhip_result r = submit(c);
        if (r != ZHIP_OK) {
            drop_pending(c);
            return r;
        }
        for (const Read &rd : c->reads) out[(*n_out)++] = zhip_completion{rd.token, 0};
        c->reads.clear();
        c->read_bytes = 0;
        out[(*n_out)++] = zhip_completion{a[0], 0};
        return ZHIP_OK;
    }
    case 10: {  // destroy: kind, id
        NEED(2);
        switch (a[0]) {
        case 0:
            if (!get(c->buffers, a[1])) return set_error(c, ZHIP_E_BAD_ID, "destroy: buffer %u does not exist", a[1]);
            if (!c->ops.empty()) {
                c->released.push_back(a[1]);
                return ZHIP_OK;
            }
            return release_buffer(c, a[1]);
        case 1: {
            Pipeline *p = get(c->pipelines, a[1]);
            if (!p) return set_error(c, ZHIP_E_BAD_ID, "destroy: pipeline %u does not exist", a[1]);
            *p = Pipeline{};
            return ZHIP_OK;
        }
        case 2: {
            Group *g = get(c->groups, a[1]);
            if (!g) return set_error(c, ZHIP_E_BAD_ID, "destroy: bind group %u does not exist", a[1]);
            *g = Group{};
            return ZHIP_OK;
        }
        default:
            return set_error(c, ZHIP_E_BAD_COMMAND, "destroy: unknown kind %u", a[0]);
        }
    }
    default:
        return set_error(c, ZHIP_E_BAD_COMMAND, "unknown opcode %u", cmd.op);
    }
}

}  // namespace

// ---- the C ABI ----------------------------------------------------------------------

extern "C" {

zhip_result zhip_create(const zhip_options *options, zhip_context **out_context) {
    if (!out_context) return ZHIP_E_INVALID_ARGUMENT;
    *out_context = nullptr;
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || count <= 0) {
        (void)hipGetLastError();
        return ZHIP_E_NO_DEVICE;
    }
    const int index = options ? (int)options->device_index : 0;
    if (index >= count) return ZHIP_E_NO_DEVICE;
    if (hipSetDevice(index) != hipSuccess) return ZHIP_E_NO_DEVICE;
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, index) != hipSuccess) return ZHIP_E_NO_DEVICE;
    // The kernels are compiled for gfx950 only.
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) return ZHIP_E_NO_DEVICE;
    zhip_context *c = new (std::nothrow) zhip_context();
    if (!c) return ZHIP_E_OUT_OF_MEMORY;
    c->device = index;
    c->use_graphs = !(options && (options->flags & ZHIP_OPTION_NO_REPLAY)) && !getenv("ZHIP_NO_REPLAY");
    c->info.compute_units = prop.multiProcessorCount;
    c->info.max_lds = (int)prop.sharedMemPerBlock;
    c->info.wide_decode = options && (options->flags & ZHIP_OPTION_WIDE_DECODE);
    c->caps.abi_version = ZHIP_ABI_VERSION;
    c->caps.compute_units = (uint32_t)prop.multiProcessorCount;
    c->caps.wavefront = (uint32_t)prop.warpSize;
    c->caps.lds_bytes = (uint32_t)prop.sharedMemPerBlock;
    c->caps.memory_bytes = prop.totalGlobalMem;
    c->caps.max_binding = 1ull << 31;
    c->caps.offset_align = 256;
    // Some driver stacks report no marketing name: fall back to the architecture.
    snprintf(c->caps.name, sizeof c->caps.name, "%s", prop.name[0] ? prop.name : "AMD Instinct (gfx950)");
    snprintf(c->caps.arch, sizeof c->caps.arch, "%s", prop.gcnArchName);
    if (char *colon = strchr(c->caps.arch, ':')) *colon = 0;
    if (hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking) != hipSuccess ||
        hipEventCreate(&c->ev_begin) != hipSuccess || hipEventCreate(&c->ev_end) != hipSuccess) {
        (void)hipGetLastError();
        delete c;
        return ZHIP_E_GPU;
    }
    // The device is current: the one place the fixed scratch array's address is looked up.
    if (no_alloc_setup(index, c->info) != ZHIP_OK) {
        (void)hipEventDestroy(c->ev_begin);
        (void)hipEventDestroy(c->ev_end);
        (void)hipStreamDestroy(c->stream);
        delete c;
        return ZHIP_E_GPU;
    }
    *out_context = c;
    return ZHIP_OK;
}

zhip_result zhip_matmul_q8_0_float_no_alloc(zhip_context *c, void *stream, const float *x, const void *weights, float *out, uint32_t rows,
    uint32_t n, uint32_t k, uint32_t col0, uint32_t out_stride, uint32_t accumulate) {
    if (!c) return ZHIP_E_INVALID_ARGUMENT;
    if (c->lost) return set_error(c, ZHIP_E_DEVICE_LOST, "device lost");
    // (the launches go to the current device: make it the context's)
    if (zhip_result r = hip_check(c, hipSetDevice(c->device), "hipSetDevice")) return r;
    char err[384] = "";
    const zhip_result r = no_alloc_matmul_q8_0_float(c->device, static_cast<hipStream_t>(stream), x, weights, out, rows, n, k, col0, out_stride,
        accumulate, err, sizeof err);
    if (r != ZHIP_OK) c->message = err[0] ? err : "matmul_q8_0_float (no allocation) failed";
    return r;
}

uint64_t zhip_no_alloc_capacity(void) { return no_alloc_capacity(); }

zhip_result zhip_destroy(zhip_context *c) {
    if (!c) return ZHIP_E_INVALID_ARGUMENT;
    (void)hipSetDevice(c->device);
    if (c->stream) (void)hipStreamSynchronize(c->stream);
    for (Buffer &b : c->buffers)
        if (b.alive && b.dev) (void)hipFree(b.dev);
    for (auto &e : c->replays)
        if (e.exec) (void)hipGraphExecDestroy(e.exec);
    c->work.release();
    for (hipEvent_t ev : c->events) (void)hipEventDestroy(ev);
    if (c->download) (void)hipHostFree(c->download);
    if (c->ev_begin) (void)hipEventDestroy(c->ev_begin);
    if (c->ev_end) (void)hipEventDestroy(c->ev_end);
    if (c->stream) (void)hipStreamDestroy(c->stream);
    delete c;
    return ZHIP_OK;
}

zhip_result zhip_get_caps(zhip_context *c, zhip_caps *out) {
    if (!c || !out) return ZHIP_E_INVALID_ARGUMENT;
    if (c->lost) return ZHIP_E_DEVICE_LOST;
    size_t free_b = 0, total = 0;
    if (hipMemGetInfo(&free_b, &total) == hipSuccess) c->caps.memory_free = free_b;
    *out = c->caps;
    return ZHIP_OK;
}

int32_t zhip_supports_prefill(zhip_context *c, uint32_t rung) {
    if (!c || c->lost) return 0;
    // The reference's ladder (scalar_f32, fp16_single, fp16_compensated); the bf16 MFMA rungs
    // are this backend's own (3: f32 activations as bound by the contract, 4: packed bf16).
    return rung <= ZHIP_PREFILL_FP16_COMPENSATED || rung == 3u || rung == 4u;
}

zhip_result zhip_set_file(zhip_context *c, const void *bytes, size_t len) {
    if (!c) return ZHIP_E_INVALID_ARGUMENT;
    if (c->lost) return ZHIP_E_DEVICE_LOST;
    c->file = static_cast<const uint8_t *>(bytes);
    c->file_len = bytes ? len : 0;
    return ZHIP_OK;
}

zhip_result zhip_execute(zhip_context *c, const uint32_t *words, size_t n_words, zhip_completion *out, size_t capacity, size_t *out_count) {
    if (!c || (!words && n_words) || !out_count || (!out && capacity)) return ZHIP_E_INVALID_ARGUMENT;
    *out_count = 0;
    if (c->lost) return set_error(c, ZHIP_E_DEVICE_LOST, "the device was lost");
    (void)hipSetDevice(c->device);
    // Completions this batch can produce: one per submit, one per read recorded
    // here or still pending from an earlier batch.
    size_t need = 0, pending_reads = c->reads.size();
    for (size_t pos = 0; pos < n_words;) {
        const size_t n = words[pos] >> 8;
        if (n == 0 || n > n_words - pos) break;
        const uint32_t op = words[pos] & 0xffu;
        if (op == 8) pending_reads++;
        if (op == 9) { need += pending_reads + 1; pending_reads = 0; }
        pos += n;
    }
    if (need > capacity) return set_error(c, ZHIP_E_INVALID_ARGUMENT, "the batch completes %zu tokens, room for %zu", need, capacity);
    // src/gpu/cmd.zig:229-246: a header word carries the command's length.
    for (size_t pos = 0; pos < n_words;) {
        const uint32_t word = words[pos];
        const size_t n = word >> 8;
        if (n == 0) return set_error(c, ZHIP_E_BAD_LENGTH, "command at word %zu has length 0", pos);
        if (n > n_words - pos) return set_error(c, ZHIP_E_TRUNCATED, "command at word %zu runs past the batch", pos);
        const Command cmd{word & 0xffu, words + pos + 1, n - 1};
        const zhip_result r = run_command(c, cmd, out, out_count);
        if (r != ZHIP_OK) return r;
        pos += n;
    }
    return ZHIP_OK;
}

zhip_result zhip_profile_start(zhip_context *c) {
    if (!c) return ZHIP_E_INVALID_ARGUMENT;
    if (c->lost) return ZHIP_E_DEVICE_LOST;
    c->profiling = true;
    return ZHIP_OK;
}

zhip_result zhip_profile_stop(zhip_context *c) {
    if (!c) return ZHIP_E_INVALID_ARGUMENT;
    c->profiling = false;
    c->timings.clear();
    c->untimed = 0;
    return ZHIP_OK;
}

zhip_result zhip_profile_read(zhip_context *c, zhip_timing *out, size_t capacity, size_t *out_count, uint64_t *out_untimed) {
    if (!c || !out_count || (!out && capacity)) return ZHIP_E_INVALID_ARGUMENT;
    *out_count = c->timings.size();
    if (out_untimed) *out_untimed = c->untimed;
    size_t i = 0;
    for (const auto &kv : c->timings) {
        if (i >= capacity) break;
        out[i].pipeline = kv.first.pipeline;
        memcpy(out[i].grid, kv.first.grid, sizeof out[i].grid);
        out[i].ns = kv.second.ns;
        out[i].count = kv.second.count;
        i++;
    }
    return ZHIP_OK;
}

zhip_result zhip_replayed_submits(zhip_context *c, uint64_t *out) {
    if (!c || !out) return ZHIP_E_INVALID_ARGUMENT;
    *out = c->replayed_submits;
    return ZHIP_OK;
}

zhip_result zhip_last_submit(zhip_context *c, uint64_t *out_ns, uint64_t *out_dispatches) {
    if (!c) return ZHIP_E_INVALID_ARGUMENT;
    if (out_ns) *out_ns = c->last_ns;
    if (out_dispatches) *out_dispatches = c->last_dispatches;
    return ZHIP_OK;
}

size_t zhip_last_error(zhip_context *c, char *out, size_t capacity) {
    if (!c) return 0;
    if (out && capacity) {
        const size_t n = std::min(capacity - 1, c->message.size());
        memcpy(out, c->message.data(), n);
        out[n] = 0;
    }
    return c->message.size();
}

zhip_result zhip_force_loss(zhip_context *c) {
    if (!c) return ZHIP_E_INVALID_ARGUMENT;
    c->lost = true;
    c->message = "the device was lost (forced)";
    return ZHIP_OK;
}

size_t zhip_kernel_artifact(const char *name, uint32_t variant, char *out, size_t capacity) {
    if (!name) return 0;
    const KernelInfo *info = find_kernel(name, strlen(name));
    if (!info) return 0;
    char buf[96];
    const int n = snprintf(buf, sizeof buf, "zhip:v1:%s:%08x", info->name, variant);
    if (out && capacity) {
        const size_t m = std::min(capacity - 1, (size_t)n);
        memcpy(out, buf, m);
        out[m] = 0;
    }
    return (size_t)n;
}

size_t zhip_backend_source(const char *name, char *out, size_t capacity) {
    if (!name) return 0;
    const KernelInfo *info = find_kernel(name, strlen(name));
    if (!info) return 0;
    char buf[160];
    const int n = snprintf(buf, sizeof buf, "zhip:src:%s:r%d:%s", info->name, info->revision, ZHIP_SOURCE_HASH);
    if (out && capacity) {
        const size_t m = std::min(capacity - 1, (size_t)n);
        memcpy(out, buf, m);
        out[m] = 0;
    }
    return (size_t)n;
}

int32_t zhip_kernel_ordinal(const char *name) { return name ? ordinal_of(name) : -1; }

}  // extern "C"
