"""Repeated submits replayed from a HIP graph give the results of the same
submits run launch by launch.

A decode step in the reference is a fixed list of prebuilt launches recorded
again for every token (src/kernels/kernels.zig:1031-1044): the host replays
such a list from a graph captured the second time it sees it. Every replay
here is checked bit for bit against a device that never replays, with other
submits, writes and reads between the replays."""
import numpy as np
import pytest

import oracle
from gpucheck import Ctx, rel_err
from zllm_amd import Device, synth
from zllm_amd import kernels as K
from zllm_amd.kernels import Kernel, TensorType, params as P

pytestmark = pytest.mark.gpu

N, KDIM, LAYERS, EPS = 512, 1024, 4, 1e-6  # feed-forward width N, hidden width k, chained layers


class Stack:
    """LAYERS x (RMS norm + fused gate/up + SiLU multiply, then down): 2 * LAYERS
    prebuilt launches, each layer reading the one before, on one context."""

    def __init__(self, c: Ctx, m: int, weights):
        self.c, self.m = c, m
        self.skip = 0  # trailing launches a step leaves out
        self.x = c.output(m * KDIM)
        b = K.Builder(c.rec, c.set)
        self.launches, self.outputs = [], []
        cur = self.x
        for gate_up, down, norm in weights:
            wg = c.gpu_weights(TensorType.q4_k, gate_up, KDIM)
            wd = c.gpu_weights(TensorType.q8_0, down, N)
            act, nxt = c.output(m * N), c.output(m * KDIM)
            self.outputs += [act, nxt]
            v = K.MatvecVariant()
            self.launches.append(b.add(
                K.weight_kernel("matvec", TensorType.q4_k), P.MatvecBf16(n=N, k=KDIM, col0=0, out_stride=N, eps=EPS, norm=True, silu_pair=True, half=N),
                [cur, wg, act, c.upload(norm)], K.Grid.rows_y(K.div_ceil(N, v.group_rows()))))
            self.launches.append(b.add(
                K.weight_kernel("matvec", TensorType.q8_0), P.MatvecBf16(n=KDIM, k=N, col0=0, out_stride=KDIM, silu_pair=False, half=0),
                [act, wd, nxt, wd], K.Grid.rows_y(K.div_ceil(KDIM, v.group_rows()))))
            cur = nxt
        self.out = cur
        self.builder = b
        b.finish()
        c.flush()

    def uniform_of_last(self) -> tuple[int, int]:
        """Buffer and byte offset of the last launch's parameter block."""
        assert len(self.builder.pages) == 1
        return self.builder.pages[0][0], (len(self.launches) - 1) * K.Builder.slot

    def step(self, x: np.ndarray, rows: int | None = None) -> np.ndarray:
        """Writes the step's input, records the launches and one read, submits."""
        c = self.c
        rows = self.m if rows is None else rows
        c.rec.write_buffer(self.x.buffer, 0, np.ascontiguousarray(x, dtype=np.float32).reshape(-1).view(np.uint8))
        used = self.launches[: len(self.launches) - self.skip]
        for l in used:
            l.record(c.rec, K.Extent(rows=rows))
        out = self.out if self.skip == 0 else self.outputs[len(used) - 1]
        return c.read(out)[: rows * (N if len(used) % 2 else KDIM)].copy()


def make_weights():
    g = synth.rng(0x6A9)
    return [(synth.q4_k_rows(g, 2 * N, KDIM), synth.q8_0_rows(g, KDIM, N), synth.activations(g, 1, KDIM).reshape(-1)) for _ in range(LAYERS)]


def unrelated_work(c: Ctx, seed: int) -> None:
    """A short submit of another shape, a write and a read: eager work between replays."""
    rows, width = 2, 96
    gu = synth.activations(synth.rng(seed), rows, 2 * width)
    act = c.output(rows * width)
    c.launcher().launch(Kernel.silu_mul, P.SiluMul(rows * width, width), [c.upload(gu), act], K.elementwise(rows * width))
    got = c.read(act).reshape(rows, width)
    g64 = gu[:, :width].astype(np.float64)
    assert np.max(np.abs(got - g64 / (1 + np.exp(-g64)) * gu[:, width:])) < 1e-5


@pytest.fixture()
def pair():
    """The same stack on a replaying device and on one that never replays."""
    weights = make_weights()
    devs = [Device.open(0), Device.open(0, Device.NO_REPLAY)]
    yield [Stack(Ctx(d), 2, weights) for d in devs]
    for d in devs:
        d.deinit()


def test_every_replay_matches_the_eager_run(pair):
    replaying, eager = pair
    seen = []
    for i in range(7):
        x = synth.activations(synth.rng(0x700 + i), 2, KDIM)
        got, want = replaying.step(x), eager.step(x)
        assert np.array_equal(got, want), f"step {i}"
        seen.append(got)
        unrelated_work(replaying.c, 0x800 + i)
    # First sight runs as recorded, the second captures and replays, as does every later one.
    assert replaying.c.host.replayed_submits() == 6
    assert eager.c.host.replayed_submits() == 0
    assert not np.array_equal(seen[0], seen[1])  # the inputs did differ
    # And the chain is the right arithmetic, not only the same on both devices.
    x = synth.activations(synth.rng(0x700), 2, KDIM)
    cur = x.astype(np.float64)
    for gate_up, down, norm in make_weights():
        xn = cur / np.sqrt(np.mean(cur * cur, axis=1, keepdims=True) + EPS) * norm
        both = xn @ oracle.Matrix(oracle.Q4_K, gate_up, 2 * N, KDIM).rows().astype(np.float64).T
        act = both[:, :N] / (1 + np.exp(-both[:, :N])) * both[:, N:]
        cur = act @ oracle.Matrix(oracle.Q8_0, down, KDIM, N).rows().astype(np.float64).T
    assert rel_err(seen[0], cur) <= 1e-4


def test_more_sequences_than_kept_graphs():
    """Twenty different steps in rotation (sixteen graphs are kept, the least recently used
    replaced): none is seen twice before it is forgotten, every result is still right; ten in
    rotation are replayed from their second round on."""
    g = synth.rng(0x6AA)
    weights = [(synth.q4_k_rows(g, 2 * N, KDIM), synth.q8_0_rows(g, KDIM, N), synth.activations(g, 1, KDIM).reshape(-1)) for _ in range(5)]
    devs = [Device.open(0), Device.open(0, Device.NO_REPLAY)]
    try:
        replaying, eager = [Stack(Ctx(d), 8, weights) for d in devs]
        variants = [(rows, skip) for skip in (0, 1, 2) for rows in range(1, 9)][:20]  # 10, 9 or 8 launches of 1..8 rows

        def run(variant, seed):
            rows, skip = variant
            x = synth.activations(synth.rng(seed), 8, KDIM)
            replaying.skip = eager.skip = skip
            return np.array_equal(replaying.step(x, rows), eager.step(x, rows))

        for cycle in range(3):
            for i, v in enumerate(variants):
                assert run(v, 0xF00 + 32 * cycle + i), f"cycle {cycle}, variant {v}"
        assert replaying.c.host.replayed_submits() == 0
        for cycle in range(3):
            for i, v in enumerate(variants[:10]):
                assert run(v, 0xF80 + 32 * cycle + i), f"cycle {cycle}, variant {v}"
        assert 10 <= replaying.c.host.replayed_submits() <= 30
    finally:
        for d in devs:
            d.deinit()


def test_steps_of_different_extents_keep_their_own_graphs(pair):
    """Alternating one-token and two-token steps: two recorded sequences, each
    replayed from its own graph once it has been seen."""
    replaying, eager = pair
    for i in range(8):
        rows = 1 + (i & 1)
        x = synth.activations(synth.rng(0x900 + i), 2, KDIM)
        assert np.array_equal(replaying.step(x, rows), eager.step(x, rows)), f"step {i}"
    assert replaying.c.host.replayed_submits() == 6


def test_changed_parameters_are_not_replayed_from_the_old_graph(pair):
    """A parameter block rewritten between steps changes the launches: the old
    graph must not run for them."""
    replaying, eager = pair
    x = synth.activations(synth.rng(0xA00), 2, KDIM)
    for _ in range(3):
        assert np.array_equal(replaying.step(x), eager.step(x))
    assert replaying.c.host.replayed_submits() == 2
    # Turn the last launch into an accumulating one (out += W act) in its parameter block.
    prev = replaying.step(x)
    assert np.array_equal(prev, eager.step(x))
    before = replaying.c.host.replayed_submits()
    changed = np.frombuffer(P.MatvecBf16(n=KDIM, k=N, col0=0, out_stride=KDIM, accumulate=True).pack(), dtype=np.uint8)
    for s in pair:
        buf, offset = s.uniform_of_last()
        s.c.rec.write_buffer(buf, offset, changed)
    got, want = replaying.step(x), eager.step(x)
    assert np.array_equal(got, want)
    assert np.array_equal(got, prev + prev)  # the old graph would have given prev again
    assert replaying.c.host.replayed_submits() == before  # first sight of the changed sequence


def test_profiling_runs_launch_by_launch(pair):
    replaying, eager = pair
    x = synth.activations(synth.rng(0xB00), 2, KDIM)
    for _ in range(3):
        assert np.array_equal(replaying.step(x), eager.step(x))
    replaying.c.host.start_profile()
    assert np.array_equal(replaying.step(x), eager.step(x))
    t = replaying.c.host.timings()
    replaying.c.host.stop_profile()
    assert sum(v.count for v in t.totals.values()) == 2 * LAYERS  # every launch timed on its own
    assert np.array_equal(replaying.step(x), eager.step(x))      # and replayed again afterwards
    assert replaying.c.host.replayed_submits() == 3


def test_a_regrown_workspace_retires_the_graphs_that_pointed_into_it():
    """The bf16 rung narrows f32 activations into the context's workspace; a graph
    captured with one allocation must not run once a larger step has replaced it."""
    rows, n, k = 32, 128, 256
    g = synth.rng(0xC0DE)
    raw = synth.q8_0_rows(g, n, k)
    big_rows = 20480  # 10 MB of narrowed activations: beyond the 8 MB the workspace starts with
    big_x = synth.activations(synth.rng(1), big_rows, k, bf16=True)
    devs = [Device.open(0), Device.open(0, Device.NO_REPLAY)]
    try:
        steps = []
        for d in devs:
            c = Ctx(d)
            c.set.select_prefill(c.rec, K.Prefill.bf16_mfma)
            wa = c.gpu_weights(TensorType.q8_0, raw, k)
            xa, big_xa = c.output(rows * k), c.upload(big_x)
            outs = [c.output(rows * n) for _ in range(8)]
            big_out = c.output(big_rows * n)
            b = K.Builder(c.rec, c.set)
            p = P.MatmulQuant(rows=rows, n=n, k=k, col0=0, out_stride=n, k_slice=k)
            ls = [b.add(Kernel.matmul_q8_0_float, p, [xa, wa, o], K.Grid.tiles_y(K.div_ceil(n, 64), 16)) for o in outs]
            big = b.add(Kernel.matmul_q8_0_float, P.MatmulQuant(rows=big_rows, n=n, k=k, col0=0, out_stride=n, k_slice=k), [big_xa, wa, big_out],
                        K.Grid.tiles_y(K.div_ceil(n, 64), 16))
            b.finish()
            c.flush()

            def step(x, c=c, xa=xa, ls=ls, outs=outs):
                c.rec.write_buffer(xa.buffer, 0, np.ascontiguousarray(x).reshape(-1).view(np.uint8))
                for l in ls:
                    l.record(c.rec, K.Extent(rows=rows))
                return c.read(outs[-1]).copy()

            def grow(c=c, big=big, big_out=big_out):
                big.record(c.rec, K.Extent(rows=big_rows))
                return c.read(big_out).copy()

            steps.append((c, step, grow))
        (rc, rstep, rgrow), (ec, estep, egrow) = steps
        for i in range(3):
            x = synth.activations(synth.rng(0xD00 + i), rows, k, bf16=True)
            assert np.array_equal(rstep(x), estep(x)), f"step {i}"
        # The first step allocated the workspace, so the second was the first sight of the
        # sequence with that allocation and the third was captured and replayed.
        assert rc.host.replayed_submits() == 1
        assert np.array_equal(rgrow(), egrow())  # replaces the workspace
        for i in range(3):
            x = synth.activations(synth.rng(0xE00 + i), rows, k, bf16=True)
            assert np.array_equal(rstep(x), estep(x)), f"step {i} after the regrowth"
        assert rc.host.replayed_submits() == 3  # seen again with the new allocation, then replayed twice
        want = synth.activations(synth.rng(0xE02), rows, k, bf16=True).astype(np.float64) @ oracle.dequantize(oracle.Q8_0, raw, n * k).reshape(n, k).astype(np.float64).T
        assert rel_err(rstep(synth.activations(synth.rng(0xE02), rows, k, bf16=True)).reshape(rows, n), want) <= 2e-2
    finally:
        for d in devs:
            d.deinit()


def test_a_parameter_block_written_by_a_kernel_of_the_step_is_not_replayed():
    """A step whose first launch writes the parameter block of its second: a graph
    would hold the block as the host last wrote it, so such a step always runs
    launch by launch and gives the launched result."""
    from zllm_amd import cmd

    width, fillers = 128, 8
    results = []
    devs = [Device.open(0), Device.open(0, Device.NO_REPLAY)]
    try:
        for d in devs:
            c = Ctx(d)
            gu = synth.activations(synth.rng(0xD00), 1, 2 * width)
            src, act = c.upload(gu), c.output(width)
            staged = c.upload(np.frombuffer(P.SiluMul(width, width).pack(), dtype=np.uint8))
            ub = c.rec.create_buffer(16, cmd.Usage.uniform | cmd.Usage.storage | cmd.Usage.copy_dst)
            pipeline = c.set.pipelines[Kernel.silu_mul]
            bg = K.bind_group(c.rec, pipeline, K.Arg(ub, 16), [src, act])
            b = K.Builder(c.rec, c.set)
            copy = b.add(Kernel.repad, P.Repad(1, 16, 16), [staged, K.Arg(ub, 16)], K.Grid.fixed_(K.elementwise(4)))
            others = [b.add(Kernel.silu_mul, P.SiluMul(width, width), [src, c.output(width)], K.Grid.fixed_(K.elementwise(width))) for _ in range(fillers)]
            b.finish()
            c.flush()
            outs = []
            for step in range(4):
                c.rec.write_buffer(ub, 0, np.frombuffer(P.SiluMul(1, 1).pack(), dtype=np.uint8))  # what a graph would keep
                c.flush()
                copy.record(c.rec, K.Extent(rows=1))
                c.rec.dispatch(pipeline, K.elementwise(width), [bg])
                for l in others:
                    l.record(c.rec, K.Extent(rows=1))
                outs.append(c.read(act).copy())
                c.rec.clear_buffer(act.buffer, 0, 4 * width)
                c.flush()
            results.append(outs)
            assert c.host.replayed_submits() == 0
        g64 = gu[0, :width].astype(np.float64)
        want = g64 / (1 + np.exp(-g64)) * gu[0, width:]
        for got, eager in zip(*results):
            assert np.array_equal(got, eager)
            assert np.max(np.abs(got - want)) < 1e-5
    finally:
        for d in devs:
            d.deinit()


def test_rows_in_parts_are_replayed_with_their_sums():
    """Verify steps on the matrix-core variant id whose down multiplies run over rows of 6144
    weights: three workgroups share a tile and a launch of its own adds their sums out of the
    context's workspace, so a recorded dispatch is two graph nodes. Every replay bit for bit
    what the eager device gives, and the arithmetic right."""
    hidden, ff, layers, m = 2048, 6144, 4, 4
    g = synth.rng(0x9A7)
    weights = [(synth.q4_k_rows(g, 2 * ff, hidden), synth.q4_k_rows(g, hidden, ff), synth.activations(g, 1, hidden).reshape(-1)) for _ in range(layers)]
    mc = K.MatvecVariant(wg=512, lanes=64, rows=16)
    devs = [Device.open(0), Device.open(0, Device.NO_REPLAY)]
    try:
        steps = []
        for d in devs:
            c = Ctx(d)
            x = c.output(m * hidden)
            b = K.Builder(c.rec, c.set)
            ls, cur = [], x
            for gate_up, down, norm in weights:
                wg, wd = c.gpu_weights(TensorType.q4_k, gate_up, hidden), c.gpu_weights(TensorType.q4_k, down, ff)
                act, nxt = c.output(m * ff), c.output(m * hidden)
                ls.append(b.add_matvec(Kernel.matvec_q4_k, mc, P.MatvecBf16(n=ff, k=hidden, col0=0, out_stride=ff, eps=EPS, norm=True, silu_pair=True, half=ff),
                                       [cur, wg, act, c.upload(norm)], K.Grid.rows_y(K.div_ceil(ff, mc.group_rows()))))
                ls.append(b.add_matvec(Kernel.matvec_q4_k, mc, P.MatvecBf16(n=hidden, k=ff, col0=0, out_stride=hidden),
                                       [act, wd, nxt, wd], K.Grid.rows_y(K.div_ceil(hidden, mc.group_rows()))))
                cur = nxt
            b.finish()
            c.flush()

            def step(xs, c=c, x=x, ls=ls, out=cur):
                c.rec.write_buffer(x.buffer, 0, np.ascontiguousarray(xs, dtype=np.float32).reshape(-1).view(np.uint8))
                for l in ls:
                    l.record(c.rec, K.Extent(rows=m))
                return c.read(out)[: m * hidden].copy()

            steps.append((c, step))
        (rc, rstep), (ec, estep) = steps
        seen = []
        for i in range(5):
            xs = synth.activations(synth.rng(0xA00 + i), m, hidden)
            got, want = rstep(xs), estep(xs)
            assert np.array_equal(got, want), f"step {i}"
            seen.append(got)
            unrelated_work(rc, 0xB00 + i)
        # The first step allocated the workspace, so the second was the first sight of the sequence
        # with that allocation; the third was captured and replayed, as were the two after it.
        assert rc.host.replayed_submits() == 3 and ec.host.replayed_submits() == 0
        assert not np.array_equal(seen[0], seen[1])
        cur = synth.activations(synth.rng(0xA00), m, hidden).astype(np.float64)
        for gate_up, down, norm in weights:
            cur = cur / np.sqrt(np.mean(cur * cur, axis=1, keepdims=True) + EPS) * norm
            both = cur @ oracle.Matrix(oracle.Q4_K, gate_up, 2 * ff, hidden).rows().astype(np.float64).T
            with np.errstate(over="ignore"):  # (a very negative gate: exp overflows to inf and the quotient is 0)
                act = both[:, :ff] / (1 + np.exp(-both[:, :ff])) * both[:, ff:]
            cur = act @ oracle.Matrix(oracle.Q4_K, down, hidden, ff).rows().astype(np.float64).T
        assert rel_err(seen[0].reshape(m, hidden), cur) <= 1e-4
    finally:
        for d in devs:
            d.deinit()
