"""The HIP host's command-stream semantics on a real device: the guarantees
the reference's native hosts give (src/agility/host.zig:1-16,293-466;
src/gpu/dawn_host.zig:240-246) and its typed failures
(src/agility/host.zig:38,662-681; src/gpu/cmd.zig:33-35)."""
import numpy as np
import pytest

from zllm_amd import Device, Host, cmd, host
from zllm_amd import kernels as K
from zllm_amd.kernels import Kernel, TensorType, params as P

pytestmark = pytest.mark.gpu

STORAGE = cmd.Usage.storage | cmd.Usage.copy_dst | cmd.Usage.copy_src


def silu_mul_want(gu, width):
    g = gu[:, :width].astype(np.float64)
    return g / (1 + np.exp(-g)) * gu[:, width:]


def test_caps_and_adapter(device):
    a = device.adapter()
    assert a.api == "hip" and a.architecture.startswith("gfx950") and a.device
    lim = device.limits()
    assert lim.max_binding == 1 << 31 and lim.offset_align == 256  # the planner's limits, src/gpu/host.zig:81-84
    assert device.memory_budget() > 100 << 30
    assert device.caps.wavefront == 64 and device.caps.compute_units >= 200
    assert device.supports_prefill(K.Prefill.scalar_f32) and device.supports_prefill(K.Prefill.bf16_mfma)
    assert device.supports_prefill(K.Prefill.fp16_single) and device.supports_prefill(K.Prefill.fp16_compensated)
    assert device.backend().name == "hip"


def test_new_buffers_read_as_zero_and_round_trip(ctx):
    c = ctx
    buf = c.output(1000)
    assert not c.read_bytes(buf).any()
    data = c.random(1000, 1)
    c.rec.write_buffer(buf.buffer, 0, data)
    assert np.array_equal(c.read(buf), data)
    c.rec.write_buffer(buf.buffer, 400, data[:10])  # a partial write at an offset
    got = c.read(buf)
    assert np.array_equal(got[100:110], data[:10]) and np.array_equal(got[:100], data[:100])


def test_writes_land_before_work_recorded_ahead_of_them(ctx):
    """write_buffer lands before the next submit's work, even work recorded
    ahead of it (src/gpu/cmd.zig:24-25, src/agility/host.zig:4-8)."""
    c = ctx
    rows, width = 2, 300
    old = c.random(rows * 2 * width, 3).reshape(rows, 2 * width)
    new = c.random(rows * 2 * width, 3).reshape(rows, 2 * width)
    gu = c.upload(old)
    act = c.output(rows * width)
    c.flush()
    c.launcher().launch(Kernel.silu_mul, P.SiluMul(rows * width, width), [gu, act], K.elementwise(rows * width))
    c.rec.write_buffer(gu.buffer, 0, new)  # recorded after the dispatch, lands before it
    got = c.read(act).reshape(rows, width)
    assert np.max(np.abs(got - silu_mul_want(new, width))) < 1e-5


def test_dispatches_copies_clears_and_reads_run_in_recorded_order(ctx):
    c = ctx
    rows, width = 3, 257
    gu = c.random(rows * 2 * width, 3).reshape(rows, 2 * width)
    act, other = c.output(rows * width), c.output(rows * width)
    c.launcher().launch(Kernel.silu_mul, P.SiluMul(rows * width, width), [c.upload(gu), act], K.elementwise(rows * width))
    first = np.zeros(rows * width, dtype=np.float32)
    c.rec.read_buffer(101, act.buffer, 0, first)             # sees the dispatch's output
    c.rec.copy_buffer(act.buffer, 0, other.buffer, 0, 4 * rows * width)
    c.rec.clear_buffer(act.buffer, 4 * width, 4 * width)      # zero the middle row afterwards
    second = np.zeros(rows * width, dtype=np.float32)
    c.rec.read_buffer(102, act.buffer, 0, second)
    done = c.flush()
    # One completion per pending read, in order, then the submit's own token.
    assert [d.token for d in done] == [101, 102, c.token] and all(d.status == 0 for d in done)
    want = silu_mul_want(gu, width).astype(np.float32)
    assert np.allclose(first.reshape(rows, width), want, atol=1e-5)
    assert np.allclose(c.read(other).reshape(rows, width), want, atol=1e-5)
    s = second.reshape(rows, width)
    assert not s[1].any() and np.allclose(s[[0, 2]], want[[0, 2]], atol=1e-5)


def test_reads_recorded_in_one_batch_complete_with_a_later_submit(ctx):
    c = ctx
    data = c.random(64, 1)
    buf = c.upload(data)
    dst = np.zeros(64, dtype=np.float32)
    c.rec.read_buffer(555, buf.buffer, 0, dst)
    done = []
    c.host.execute(c.rec.batch(), done)  # no submit yet
    c.rec.clear()
    assert done == [] and not dst.any()
    done = c.flush()
    assert [d.token for d in done] == [555, c.token] and np.array_equal(dst, data)


def test_a_buffer_destroyed_with_work_pending_is_released_after_the_submit(ctx):
    c = ctx
    rows, width = 1, 64
    gu = c.random(2 * width, 2).reshape(1, 2 * width)
    src, act = c.upload(gu), c.output(width)
    c.launcher().launch(Kernel.silu_mul, P.SiluMul(width, width), [src, act], K.elementwise(width))
    c.rec.destroy(cmd.Kind.buffer, src.buffer)  # the dispatch above still reads it
    got = c.read(act)
    assert np.allclose(got, silu_mul_want(gu, width)[0], atol=1e-5)
    with pytest.raises(host.BadId):
        c.rec.write_buffer(src.buffer, 0, gu)
        c.flush()


def test_write_file_copies_from_the_model_mapping(ctx):
    c = ctx
    blob = c.rand.integers(0, 256, size=4096, dtype=np.uint8)
    c.host.set_file(blob)
    buf = c.output(256)
    c.rec.write_file(buf.buffer, 64, 1000, 512)
    got = c.read_bytes(buf)
    assert np.array_equal(got[64 : 64 + 512], blob[1000:1512]) and not got[:64].any()
    with pytest.raises(host.BadCommand):
        c.rec.write_file(buf.buffer, 0, 4000, 512)  # past the end of the file
        c.flush()
    c.host.set_file(None)
    with pytest.raises(host.BadCommand):
        c.rec.write_file(buf.buffer, 0, 0, 16)
        c.flush()


def test_parameters_written_by_the_gpu_are_read_back(ctx):
    """Binding 0 normally comes from the host's shadow of a uniform buffer; a
    parameter block the GPU copied into place must be seen too."""
    c = ctx
    width = 128
    gu = c.random(2 * width, 2).reshape(1, 2 * width)
    staged = c.upload(np.frombuffer(P.SiluMul(width, width).pack(), dtype=np.uint8))
    ub = c.rec.create_buffer(16, cmd.Usage.uniform | cmd.Usage.copy_dst)
    c.rec.write_buffer(ub, 0, np.frombuffer(P.SiluMul(1, 1).pack(), dtype=np.uint8))  # stale contents
    c.rec.copy_buffer(staged.buffer, 0, ub, 0, 16)
    act = c.output(width)
    pipeline = c.set.pipelines[Kernel.silu_mul]
    bg = K.bind_group(c.rec, pipeline, K.Arg(ub, 16), [c.upload(gu), act])
    c.rec.dispatch(pipeline, K.elementwise(width), [bg])
    assert np.allclose(c.read(act), silu_mul_want(gu, width)[0], atol=1e-5)


def expect(c, error, build):
    """Records with `build`, submits, expects `error`; the context stays usable."""
    build()
    with pytest.raises(error):
        c.flush()
    probe = c.upload(np.arange(8, dtype=np.float32))
    assert np.array_equal(c.read(probe), np.arange(8, dtype=np.float32))


def test_typed_errors(ctx):
    c = ctx
    buf = c.output(16)
    c.flush()
    expect(c, host.BadId, lambda: c.rec.words.extend([cmd.header(cmd.Op.write_buffer, 8), 9999, 0, 0, 0, 0, 4, 0]))
    expect(c, host.BadId, lambda: c.rec.words.extend([cmd.header(cmd.Op.create_buffer, 5), buf.buffer, 64, 0, int(STORAGE)]))  # id reuse
    expect(c, host.BadId, lambda: c.rec.dispatch(4242, (1, 1, 1), []))
    expect(c, host.BadCommand, lambda: c.rec.write_buffer(buf.buffer, 60, np.zeros(4, np.float32)))  # past the end
    expect(c, host.BadCommand, lambda: c.rec.write_buffer(buf.buffer, 2, np.zeros(1, np.float32)))   # misaligned
    expect(c, host.BadCommand, lambda: c.rec.words.extend([77 | (1 << 8)]))                            # unknown opcode
    expect(c, host.BadCommand, lambda: c.rec.words.extend([cmd.header(cmd.Op.submit, 1)]))             # too few words
    expect(c, host.BadCommand, lambda: c.rec.copy_buffer(buf.buffer, 0, buf.buffer, 32, 64))
    expect(c, host.BadLength, lambda: c.rec.words.extend([int(cmd.Op.submit)]))
    expect(c, host.Truncated, lambda: c.rec.words.extend([cmd.header(cmd.Op.dispatch, 12), 0]))
    # Two bind groups on a dispatch: the kernels take one (src/agility/host.zig:376).
    expect(c, host.BadCommand, lambda: c.rec.dispatch(c.set.pipelines[Kernel.silu_mul], (1, 1, 1), [0, 0]))


def test_kernel_ranges_are_checked_before_launch(ctx):
    """A dispatch whose parameters reach past a bound range fails with
    BadCommand on the host; nothing is launched."""
    c = ctx
    n, k = 64, 1024
    raw = c.rand.integers(0, 256, size=n * K.row_bytes(TensorType.q4_k, k), dtype=np.uint8)
    w, x, out = c.upload(raw), c.upload(c.random(k, 1)), c.output(n)
    c.flush()
    l = c.launcher()
    p = lambda **kw: P.MatvecBf16(**{**dict(n=n, k=k, col0=0, out_stride=n), **kw})
    grid = (K.div_ceil(n, 8), 1, 1)
    expect(c, host.BadCommand, lambda: l.launch(Kernel.matvec_q4_k, p(n=2 * n), [x, w, out, w], (K.div_ceil(2 * n, 8), 1, 1)))  # weights too small
    expect(c, host.BadCommand, lambda: l.launch(Kernel.matvec_q4_k, p(), [x, w, out, w], (grid[0], 2, 1)))                       # two tokens, one row of x
    expect(c, host.BadCommand, lambda: l.launch(Kernel.matvec_q4_k, p(col0=8), [x, w, out, w], grid))                            # out too small
    expect(c, host.BadCommand, lambda: l.launch(Kernel.matvec_q4_k, p(k=1000), [x, w, out, w], grid))                            # k not a block multiple
    expect(c, host.BadCommand, lambda: l.launch(Kernel.matvec_q4_k, p(norm=True), [x, w, out, K.Arg(out.buffer, 16)], grid))     # norm weights too small
    expect(c, host.BadCommand, lambda: l.launch(Kernel.matvec_q4_k, p(), [x, w], grid))                                          # out not bound
    # An empty grid is not an error (src/kernels/kernels.zig:1039-1043 never records one; hosts ignore it).
    l.launch(Kernel.matvec_q4_k, p(), [x, w, out, w], (0, 1, 1))
    c.flush()


def test_missing_kernels_fail_the_batch_and_drop_the_submission(ctx):
    """Dispatching a pipeline created with an empty artifact fails with
    UnsupportedKernel, names the kernel, and drops the submission in progress
    (src/gpu/cmd.zig:33-35, src/agility/host.zig:296-309)."""
    c = ctx
    data = c.random(16, 1)
    buf = c.upload(data)
    c.flush()
    dst = np.zeros(16, dtype=np.float32)
    c.rec.read_buffer(901, buf.buffer, 0, dst)
    c.rec.dispatch(c.set.pipelines[Kernel.rmsnorm], (1, 1, 1), [])
    with pytest.raises(host.UnsupportedKernel):
        c.flush()
    assert "rmsnorm" in c.device.error_message()
    assert not dst.any()
    done = c.flush()  # the dropped read does not complete later
    assert [d.token for d in done] == [c.token]
    assert np.array_equal(c.read(buf), data)


def test_create_kernel_rejects_what_it_does_not_implement(ctx):
    c = ctx
    writes = K.contract(Kernel.matmul_bf16).writes
    # A prefill variant id that is neither the reference's nor this backend's.
    expect(c, host.BadCommand, lambda: c.rec.create_kernel(int(Kernel.matmul_bf16), 0xFFF90000, writes, K.artifact(Kernel.matmul_bf16, 0xFFF90000)))
    # matmul_f16 has only the exact f32 rung.
    expect(c, host.UnsupportedPrefill, lambda: c.rec.create_kernel(int(Kernel.matmul_f16), K.PREFILL_VARIANT[K.Prefill.bf16_mfma], writes, K.artifact(Kernel.matmul_f16, K.PREFILL_VARIANT[K.Prefill.bf16_mfma])))
    expect(c, host.BadCommand, lambda: c.rec.create_kernel(int(Kernel.matmul_bf16), 0, writes, b"@compute fn main() {}"))           # another backend's artifact
    expect(c, host.BadCommand, lambda: c.rec.create_kernel(int(Kernel.matmul_bf16), 0, 0b10, K.artifact(Kernel.matmul_bf16)))      # contract mismatch
    expect(c, host.BadCommand, lambda: c.rec.create_kernel(int(Kernel.silu_mul), 5, K.contract(Kernel.silu_mul).writes, K.artifact(Kernel.silu_mul)))
    expect(c, host.BadCommand, lambda: c.rec.create_kernel(int(Kernel.matvec_q4_k), 0x00000100, K.contract(Kernel.matvec_q4_k).writes, K.artifact(Kernel.matvec_q4_k)))


def test_profile_times_every_dispatch_by_pipeline_and_grid(ctx):
    c = ctx
    width = 4096
    gu = c.upload(c.random(4 * 2 * width, 1))
    act = c.output(4 * width)
    c.flush()
    assert c.host.timings() is None
    c.host.start_profile()
    l = c.launcher()
    for rows in (1, 4, 4, 4):
        l.launch(Kernel.silu_mul, P.SiluMul(rows * width, width), [gu, act], K.elementwise(rows * width))
    c.flush()
    t = c.host.timings()
    pl = c.set.pipelines[Kernel.silu_mul]
    small, big = host.TimingKey(pl, K.elementwise(width)), host.TimingKey(pl, K.elementwise(4 * width))
    assert t.totals[small].count == 1 and t.totals[big].count == 3 and t.untimed == 0
    assert 0 < t.totals[small].ns < 1e9 and 0 < t.totals[big].ns < 1e9
    ns, dispatches = c.host.last_submit()
    assert dispatches == 4 and ns > 0
    c.host.stop_profile()
    assert c.host.timings() is None


def test_forced_device_loss_and_recovery():
    """forceLoss makes every later call fail with DeviceLost; a fresh device
    works (the recovery path of src/generate.zig:574-595)."""
    d = Device.open(0)
    h = Host(d)
    rec = cmd.Recorder()
    buf = rec.create_buffer(64, STORAGE)
    rec.submit(1)
    done = []
    h.execute(rec.batch(), done)
    assert [c.token for c in done] == [1]
    d.force_loss()
    with pytest.raises(host.DeviceLost):
        h.execute(rec.batch(), [])
    assert "lost" in d.error_message()
    d.deinit()
    d2 = Device.open(0)
    h2 = Host(d2)
    rec = cmd.Recorder()
    data = np.arange(16, dtype=np.float32)
    buf = rec.create_buffer(64, STORAGE)
    rec.write_buffer(buf, 0, data)
    got = np.zeros(16, dtype=np.float32)
    rec.read_buffer(7, buf, 0, got)
    rec.submit(8)
    done = []
    h2.execute(rec.batch(), done)
    assert [c.token for c in done] == [7, 8] and np.array_equal(got, data)
    d2.deinit()
