"""Seeded random shapes through the decode multiply's matrix-core variant id, the prefill rungs
and the int8 prefill: the edges the fixed cases of test_gpu_check.py do not name (row counts below a
tile, rows in any number of parts, ragged token counts, column offsets and padded strides).
Each case against float64 over the oracle's decoded weights (1e-5 of the output's scale, the
reference's gpu-check tolerance, src/kernels/check.zig:205-222), nothing outside the outputs
touched, and a token's bits the same whatever shares its step (src/sched/sched.zig:55-58,84-90)."""
import numpy as np
import pytest

import oracle
from gpucheck import rel_err
from zllm_amd import cmd, synth
from zllm_amd import kernels as K
from zllm_amd.kernels import Kernel, TensorType, params as P

pytestmark = pytest.mark.gpu

ORACLE_TYPE = {TensorType.q8_0: oracle.Q8_0, TensorType.q3_k: oracle.Q3_K, TensorType.q4_k: oracle.Q4_K, TensorType.q5_k: oracle.Q5_K, TensorType.q6_k: oracle.Q6_K}
MFMA_VARIANT = K.MatvecVariant(wg=512, lanes=64, rows=16)
EPS = 1e-6


def sigmoid64(v):
    with np.errstate(over="ignore"):
        return 1.0 / (1.0 + np.exp(-v))


def release(c, *args):
    for a in args:
        c.rec.destroy(cmd.Kind.buffer, a.buffer)
    c.flush()


@pytest.mark.parametrize("seed", [3, 4])
def test_matrix_core_decode_id_random_shapes(ctx, seed):
    """Forty cases a seed: every format, one to eight tokens, rows of 2048 .. 32768 weights (whole
    multiples of 2048: one workgroup a tile or up to sixteen), 16 .. 2000 outputs, with and
    without the RMSNorm prologue, silu(x / act_div), the SILU_PAIR and ACCUMULATE epilogues."""
    c = ctx
    rng = np.random.default_rng(seed)
    for case in range(40):
        t = list(ORACLE_TYPE)[rng.integers(5)]
        k = int(rng.choice([2048, 4096, 6144, 8192, 10240, 12288, 14336, 16384, 20480, 28672, 32768]))
        n = int(rng.choice([16, 48, 80, 96, 256, 528, 1000, 1296, 2000]))
        m = int(rng.integers(1, 9))
        norm, pair = bool(rng.integers(2)), bool(rng.integers(2))
        acc = (not pair) and bool(rng.integers(2))
        div = int(rng.choice([0, 0, 4]))
        col0, pad = int(rng.choice([0, 0, 3])), int(rng.choice([0, 5]))
        what = f"case {case}: {t.name} m={m} n={n} k={k} norm={norm} pair={pair} accumulate={acc} act_div={div} col0={col0} pad={pad}"
        g = synth.rng(int(rng.integers(1 << 30)))
        rows_w = 2 * n if pair else n
        raw = synth.random_blocks(g, t.name, rows_w, k)
        vals = oracle.dequantize(ORACLE_TYPE[t], raw, rows_w * k).reshape(rows_w, k).astype(np.float64)
        x = synth.activations(g, m, k)
        x[0] *= np.float32(1e-4)  # tokens of very different magnitudes
        nw = synth.activations(g, 1, k).reshape(-1)
        stride = col0 + n + pad
        init = synth.activations(g, m, stride)
        x64 = x.astype(np.float64)
        if norm:
            x64 = x64 / np.sqrt(np.mean(x64 * x64, axis=1, keepdims=True) + EPS) * nw.astype(np.float64)
        if div:
            x64 = (x64 / div) * sigmoid64(x64 / div)
        if pair:
            gate, up = x64 @ vals[:n].T, x64 @ vals[n:].T
            prod = gate * sigmoid64(gate) * up
        else:
            prod = x64 @ vals.T
        want = prod + (init[:, col0 : col0 + n] if acc else 0)
        xa, wa, na = c.upload(x), c.gpu_weights(t, raw, k), c.upload(nw)
        p = lambda: P.MatvecBf16(n=n, k=k, col0=col0, out_stride=stride, eps=EPS, norm=norm, accumulate=acc, silu_pair=pair, half=n if pair else 0)
        variant = K.MatvecVariant(MFMA_VARIANT.wg, MFMA_VARIANT.lanes, MFMA_VARIANT.rows, div)
        pipeline = c.set.matvec(c.rec, K.weight_kernel("matvec", t), variant)
        grid_x = K.div_ceil(n, variant.group_rows())
        out = c.upload(init)
        c.launcher().launch_pipeline(pipeline, p(), [xa, wa, out, na], (grid_x, m, 1))
        got = c.read(out).reshape(m, stride)
        for tk in range(m):
            # Against the product's own scale (an accumulated init may dwarf a tiny token's product).
            limit = 1e-5 * max(np.max(np.abs(prod[tk])), 1e-30) + 1e-6 * np.max(np.abs(want[tk]))
            assert np.max(np.abs(got[tk, col0 : col0 + n] - want[tk])) <= limit, (what, tk)
        mask = np.ones(stride, dtype=bool)
        mask[col0 : col0 + n] = False
        assert np.array_equal(got[:, mask].view(np.uint32), init[:, mask].view(np.uint32)), what
        for tk in (0, m - 1):
            single, xs = c.upload(init[tk]), c.upload(x[tk])
            c.launcher().launch_pipeline(pipeline, p(), [xs, wa, single, na], (grid_x, 1, 1))
            assert got[tk].tobytes() == c.read(single)[:stride].tobytes(), (what, "a token's sums differ between a lone launch and a multi-token launch")
            release(c, single, xs)
        release(c, xa, wa, na, out)


@pytest.mark.parametrize("seed", [11, 12])
def test_prefill_rungs_random_shapes(ctx, seed):
    """Forty cases a seed of matmul_q8_0_float on the bf16 rung (f32 or packed bf16 activations)
    and the reference's fp16_single rung: 1 .. 512 tokens, 1 .. 9000 outputs (both sides of the
    8065 rows from which a matrix takes 128-row tiles), k with and without whole 128-deep steps;
    then the same tokens in up to four steps cut at random, bit for bit."""
    c = ctx
    rng = np.random.default_rng(seed)
    for case in range(40):
        rung = ["bf16_mfma", "fp16_single", "bf16_mfma_xbf16"][rng.integers(3)]
        k = int(rng.choice([128, 256, 384, 1024, 2048, 4096, 1056, 96, 640]))
        n = int(rng.choice([1, 31, 64, 100, 1000, 2830, 4096, 8064, 8065, 8230, 9000]))
        rows = int(rng.choice([1, 5, 31, 32, 33, 64, 65, 100, 128, 129, 300, 512]))
        col0, pad, acc = int(rng.choice([0, 0, 3, 4])), int(rng.choice([0, 4, 5])), int(rng.integers(2))
        what = f"case {case}: {rung} rows={rows} n={n} k={k} col0={col0} pad={pad} accumulate={acc}"
        g = synth.rng(int(rng.integers(1 << 30)))
        raw = synth.q8_0_rows(g, n, k)
        wq = oracle.dequantize(oracle.Q8_0, raw, n * k).reshape(n, k)
        packed = rung == "bf16_mfma_xbf16"
        x = synth.activations(g, rows, k, bf16=packed)
        stride = col0 + n + pad
        init = synth.activations(g, rows, stride)
        wa = c.gpu_weights(TensorType.q8_0, raw, k)
        c.set.select_prefill(c.rec, K.Prefill[rung])
        narrow = (lambda v: v.astype(np.float16).astype(np.float32)) if rung == "fp16_single" else synth.bf16_round

        def run(first, count):
            out = c.upload(init[first : first + count])
            xs = x[first : first + count]
            xa = c.upload(synth.to_bf16_bits(xs) if packed else xs)
            c.launcher().launch(Kernel.matmul_q8_0_float, P.MatmulQuant(rows=count, n=n, k=k, col0=col0, out_stride=stride, accumulate=acc, k_slice=k),
                                [xa, wa, out], (K.div_ceil(n, 64), K.div_ceil(count, 16), 1))
            r = c.read(out).reshape(count, stride).copy()
            release(c, out, xa)
            return r

        got = run(0, rows)
        want = (init[:, col0 : col0 + n] if acc else 0) + narrow(x).astype(np.float64) @ narrow(wq).astype(np.float64).T
        assert rel_err(got[:, col0 : col0 + n], want) <= 1e-5, what
        mask = np.ones(stride, dtype=bool)
        mask[col0 : col0 + n] = False
        assert np.array_equal(got[:, mask].view(np.uint32), init[:, mask].view(np.uint32)), what
        cuts = sorted(set([0, rows] + [int(v) for v in rng.integers(0, rows + 1, size=3)]))
        for a, b in zip(cuts[:-1], cuts[1:]):
            assert got[a:b].tobytes() == run(a, b - a).tobytes(), (what, "token chunking changed bits", a, b)
        release(c, wa)
    c.set.select_prefill(c.rec, K.Prefill.scalar_f32)


@pytest.mark.parametrize("seed", [21, 22])
def test_int8_prefill_random_shapes(ctx, seed):
    """Thirty cases a seed of the reference's default prefill, quantize_q8 + matmul_<type> over
    whole k, every format: 1 .. 512 tokens, 1 .. 8000 outputs, k of 1 .. 36 blocks of 256 (the
    K formats' four parts of k with no, one or several blocks each; steps short and long enough
    for either of their kernels and for each of the Q8_0 kernel's tile heights). 1e-5 against
    float64 over the rounded activations (src/kernels/check.zig:839-871); then the same tokens
    in up to four steps cut at random, bit for bit."""
    c = ctx
    rng = np.random.default_rng(seed)
    for case in range(30):
        t = list(ORACLE_TYPE)[rng.integers(5)]
        k = int(rng.choice([256, 512, 768, 1024, 1280, 2048, 4096, 9216]))
        n = int(rng.choice([1, 31, 64, 100, 1000, 2830, 4096, 8000]))
        rows = int(rng.choice([1, 5, 31, 32, 33, 64, 65, 100, 128, 129, 300, 512]))
        col0, pad, acc = int(rng.choice([0, 0, 3, 4])), int(rng.choice([0, 4, 5])), int(rng.integers(2))
        what = f"case {case}: {t.name} rows={rows} n={n} k={k} col0={col0} pad={pad} accumulate={acc}"
        g = synth.rng(int(rng.integers(1 << 30)))
        raw = synth.random_blocks(g, t.name, n, k)
        vals = oracle.dequantize(ORACLE_TYPE[t], raw, n * k).reshape(n, k).astype(np.float64)
        x = synth.activations(g, rows, k)
        xs = oracle.round_like_llama(ORACLE_TYPE[t], x).astype(np.float64)
        stride = col0 + n + pad
        init = synth.activations(g, rows, stride)
        wa = c.gpu_weights(t, raw, k)
        block = K.act_block(t)

        def run(first, count):
            out, xa = c.upload(init[first : first + count]), c.upload(x[first : first + count])
            qx, dx = c.output(count * k // 4), c.output(count * k // block)
            l = c.launcher()
            l.launch(Kernel.quantize_q8, P.QuantizeQ8(k=k, block=block), [xa, qx, dx, xa], (K.div_ceil(k, 256), count, 1))
            l.launch(K.weight_kernel("matmul", t), P.MatmulQuant(rows=count, n=n, k=k, col0=col0, out_stride=stride, accumulate=acc, k_slice=k),
                     [qx, wa, out, dx], (K.div_ceil(n, K.matmul_quant_tile_n), K.div_ceil(count, K.matmul_quant_tile_t), 1))
            r = c.read(out).reshape(count, stride).copy()
            release(c, out, xa, qx, dx)
            return r

        got = run(0, rows)
        want = (init[:, col0 : col0 + n] if acc else 0) + xs @ vals.T
        assert rel_err(got[:, col0 : col0 + n], want) <= 1e-5, what
        mask = np.ones(stride, dtype=bool)
        mask[col0 : col0 + n] = False
        assert np.array_equal(got[:, mask].view(np.uint32), init[:, mask].view(np.uint32)), what
        cuts = sorted(set([0, rows] + [int(v) for v in rng.integers(0, rows + 1, size=3)]))
        for a, b in zip(cuts[:-1], cuts[1:]):
            assert got[a:b].tobytes() == run(a, b - a).tobytes(), (what, "token chunking changed bits", a, b)
        release(c, wa)
