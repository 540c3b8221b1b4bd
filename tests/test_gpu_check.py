"""Kernel checks on the GPU, case for case as the reference's gpu-check runs
them for this path (src/kernels/check.zig): each kernel on seeded inputs
through the command stream, against a float64 computation over weights decoded
by the CPU oracle. Tolerances are the reference's own (1e-5 of the output
scale; 0 for gathers), written beside each case.
"""
import numpy as np
import pytest

import oracle
from gpucheck import bound_err, rel_err
from zllm_amd import kernels as K
from zllm_amd import synth
from zllm_amd.kernels import Kernel, TensorType, params as P

pytestmark = pytest.mark.gpu

ORACLE_TYPE = {TensorType.q8_0: oracle.Q8_0, TensorType.q3_k: oracle.Q3_K, TensorType.q4_k: oracle.Q4_K, TensorType.q5_k: oracle.Q5_K, TensorType.q6_k: oracle.Q6_K,
               TensorType.bf16: oracle.BF16, TensorType.iq4_xs: oracle.IQ4_XS}


def quant_rows(c, t: TensorType, rows: int, k: int):
    """Random blocks with finite super-scales and their oracle-decoded values
    (src/kernels/check.zig:461-481)."""
    raw = synth.random_blocks(c.rand, t.name, rows, k)
    return raw, oracle.dequantize(ORACLE_TYPE[t], raw, rows * k).reshape(rows, k)


def random_half(c, n: int, scale: float, half: str = "bf16"):
    """bf16 or f16 weights and their f32 values (src/kernels/check.zig randomHalf);
    numpy's float16 is the f16 conversion."""
    if half == "f16":
        h = c.random(n, scale).astype(np.float16)
        return h.view(np.uint16), h.astype(np.float32)
    bits = synth.to_bf16_bits(c.random(n, scale))
    return bits, synth.bf16_bits_to_f32(bits)


HALVES = ["bf16", "f16"]


def norm_row(x, w, eps):
    """out = rmsnorm(x) * w in float64 when w is given, else x
    (src/kernels/check.zig:370-376)."""
    x = x.astype(np.float64)
    if w is None:
        return x
    scale = 1.0 / np.sqrt(np.sum(x * x) / x.size + eps)
    return x * scale * w.astype(np.float64)


def sigmoid64(x):
    return 1.0 / (1.0 + np.exp(-x))


# ---- half-precision decode multiply: check.zig:327-442 ------------------------------

def matvec_case(c, k, split, fused, half="bf16"):
    rows, n, eps = 3, 100, 1e-6
    x = c.random(rows * k, 3).reshape(rows, k)
    nw = c.random(k, 1)
    bits, values = random_half(c, n * k, 1, half)
    bits, values = bits.reshape(n, k), values.reshape(n, k)
    init = c.random(rows * n, 4 if fused else 0).reshape(rows, n)
    out, xa, na = c.upload(init), c.upload(x), c.upload(nw)
    col0 = 0
    for cols in (split, n - split):
        wa = c.upload(bits[col0 : col0 + cols])
        c.launcher().launch(Kernel["matvec_" + half], P.MatvecBf16(n=cols, k=k, col0=col0, out_stride=n, eps=eps, norm=fused, accumulate=fused),
                            [xa, wa, out, na], (K.div_ceil(cols, K.matvec_rows), rows, 1))
        col0 += cols
    got = c.read(out).reshape(rows, n)
    want = np.stack([norm_row(x[t], nw if fused else None, eps) @ values.astype(np.float64).T for t in range(rows)]) + init
    return rel_err(got, want)


@pytest.mark.parametrize("half", HALVES)
def test_matvec_bf16_two_chunks(ctx, half):
    # k = 4000 leaves a partial pass over the lanes; 100 outputs a partial group.
    assert matvec_case(ctx, 4000, 37, False, half) <= 1e-5


@pytest.mark.parametrize("half", HALVES)
def test_matvec_bf16_norm_accumulate(ctx, half):
    assert matvec_case(ctx, 1000, 37, True, half) <= 1e-5


def bf16_tokens_case(c, m, n, k, col0=0, pad=0, accumulate=False, norm=False, x=None, half="bf16"):
    """A matvec_bf16 step of m tokens over n x k weights, writing columns col0 .. col0 + n of
    rows n + col0 + pad wide; returns (got, want in float64, the launch's inputs)."""
    eps, stride = 1e-6, col0 + n + pad
    x = c.random(m * k, 3).reshape(m, k) if x is None else x
    nw = c.random(k, 1)
    bits, values = random_half(c, n * k, 1, half)
    init = c.random(m * stride, 4).reshape(m, stride)
    out = c.upload(init)
    c.launcher().launch(Kernel["matvec_" + half], P.MatvecBf16(n=n, k=k, col0=col0, out_stride=stride, eps=eps, norm=norm, accumulate=accumulate),
                        [c.upload(x), c.upload(bits), out, c.upload(nw)], (K.div_ceil(n, K.matvec_rows), m, 1))
    got = c.read(out).reshape(m, stride)
    want = init.astype(np.float64).copy()
    prod = np.stack([norm_row(x[t], nw if norm else None, eps) @ values.reshape(n, k).astype(np.float64).T for t in range(m)])
    want[:, col0 : col0 + n] = prod + (want[:, col0 : col0 + n] if accumulate else 0.0)
    return got, want, (x, bits)


# In a context opened with ZHIP_OPTION_WIDE_DECODE, steps over k = 1024 ... 16384 in steps of 512
# and 16 MB or more of weights run on the matrix cores, the weights read once for all tokens, at
# every width from one token on; smaller matrices, and every matrix in a context without the
# option, keep the general kernel. The cases run under both.
@pytest.mark.parametrize("m,n,k,col0,pad,accumulate,norm", [
    (2, 16400, 1024, 0, 0, False, False),
    (2, 8192, 1024, 0, 0, False, False),       # 16.8 MB: the smallest matrix the option moves
    (1, 16400, 1024, 0, 0, False, False),      # one token
    (1, 4100, 4096, 3, 1, True, True),
    (8, 8300, 1024, 0, 0, False, False),       # a ragged last unit of rows
    (3, 11001, 1536, 5, 3, True, False),       # unaligned columns, accumulate
    (3, 5501, 1536, 5, 3, True, False),        # ... just above 16 MB
    (4, 8200, 2048, 0, 0, False, False),       # a tail on every workgroup
    (5, 9000, 2560, 0, 0, False, True),        # the RMSNorm prologue
    (7, 2741, 3072, 32, 0, True, True),
    (8, 2400, 3584, 0, 0, False, False),
    (6, 4040, 4096, 0, 0, False, False),
    (11, 8195, 1024, 0, 7, False, False),      # more than eight tokens: two launches
    (4, 8192, 1024, 0, 0, False, True),        # k = 1024 with the prologue: the tokens split beforehand
    (19, 2052, 4096, 8, 0, True, False),
    (3, 100, 1024, 0, 0, False, False),        # a small matrix: the general kernel
    (5, 1100, 9728, 0, 0, False, False),       # rows longer than 4096: stretches of columns, each launch adding to the one before
    (6, 800, 14336, 3, 5, True, False),        # ... onto what the output already holds (four equal stretches: one launch, and one for their sums)
    (19, 1100, 8192, 8, 0, True, True),        # two equal stretches, three groups of tokens, the prologue
    (5, 1000, 12288, 0, 0, False, False),      # three equal stretches
    (5, 1000, 8704, 0, 0, False, True),        # with the RMSNorm prologue: the tokens are normalised and split once for all the stretches
    (3, 1100, 9728, 0, 0, False, False),       # the same rows at fewer tokens (the general kernel: passes of as many tokens as fit workgroup memory)
    (2, 800, 14336, 3, 5, True, False),
    (3, 1000, 8704, 0, 0, False, True),
])
@pytest.mark.parametrize("half", HALVES)
@pytest.mark.parametrize("wide", [False, True])
def test_matvec_bf16_several_tokens(ctx, ctx_wide, wide, half, m, n, k, col0, pad, accumulate, norm):
    got, want, _ = bf16_tokens_case(ctx_wide if wide else ctx, m, n, k, col0, pad, accumulate, norm, half=half)
    assert rel_err(got, want) <= 1e-5
    # Columns outside the launch's keep their contents bit for bit.
    keep = np.ones(got.shape[1], dtype=bool)
    keep[col0 : col0 + n] = False
    assert np.array_equal(got[:, keep].astype(np.float32), want[:, keep].astype(np.float32))


def test_matvec_bf16_several_tokens_many_rows(ctx_wide):
    """More than forty 32-row tiles on every workgroup: the outputs kept back in workgroup
    memory are stored in the middle of the run, not only at its end."""
    c = ctx_wide
    m, n, k = 2, 41 * 32 * c.device.caps.compute_units + 50, 1024
    x = c.random(m * k, 3).reshape(m, k)
    bits = synth.to_bf16_bits(c.rand.standard_normal(n * k, dtype=np.float32))
    out = c.output(m * n)
    c.launcher().launch(Kernel.matvec_bf16, P.MatvecBf16(n=n, k=k, col0=0, out_stride=n, eps=1e-6),
                        [c.upload(x), c.upload(bits), out, c.upload(np.ones(k, dtype=np.float32))], (K.div_ceil(n, K.matvec_rows), m, 1))
    got = c.read(out).reshape(m, n)
    want = x.astype(np.float64) @ synth.bf16_bits_to_f32(bits).reshape(n, k).astype(np.float64).T
    assert rel_err(got, want) <= 1e-5


@pytest.mark.parametrize("half", HALVES)
@pytest.mark.parametrize("wide", [False, True])
def test_matvec_bf16_several_tokens_keep_token_bits(ctx, ctx_wide, wide, half):
    """A token's outputs do not depend on how many tokens share the step - the lone launch gives
    the bits of every wider one (src/sched/sched.zig:55-58) - nor on where the step's columns
    start; over 18 MB of weights, with and without ZHIP_OPTION_WIDE_DECODE."""
    c = ctx_wide if wide else ctx
    m, n, k = 13, 4500, 2048
    x = c.random(m * k, 3).reshape(m, k)
    bits, _ = random_half(c, n * k, 1, half)

    def run(tokens, rows0, rows):
        out = c.output(len(tokens) * rows)
        wpart = c.upload(bits.reshape(n, k)[rows0 : rows0 + rows])
        c.launcher().launch(Kernel["matvec_" + half], P.MatvecBf16(n=rows, k=k, col0=0, out_stride=rows, eps=1e-6),
                            [c.upload(x[tokens]), wpart, out, c.upload(np.ones(k, dtype=np.float32))], (K.div_ceil(rows, K.matvec_rows), len(tokens), 1))
        return c.read(out).reshape(len(tokens), rows)

    whole = run(list(range(m)), 0, n)
    lone = np.stack([run([t], 0, n)[0] for t in range(m)])
    assert np.array_equal(lone, whole)
    for tokens in ([4, 9], [4, 9, 11], [12, 0, 5, 7], [12, 0, 5, 7, 3], [4, 9, 1, 2, 6, 8], list(range(8))):
        assert np.array_equal(run(tokens, 0, n), whole[tokens])
    # (4096 rows of 2048 weights: 16 MB, the smallest matrix the option moves)
    assert np.array_equal(run(list(range(8)), 404, 4096), whole[:8, 404:])
    assert np.array_equal(run([5], 404, 4096)[0], whole[5, 404:])


def test_matvec_bf16_several_tokens_special_values(ctx_wide):
    """Inputs the three-way split must carry exactly: full 24-bit mantissas (integer inputs
    against weights of +-1, where every partial sum is an integer f32 holds, so the result is
    exact whatever the order of the additions), the largest finite value, infinities and NaNs."""
    c = ctx_wide
    m, n, k = 4, 8192, 1024
    x = np.zeros((m, k), dtype=np.float32)
    r = c.rand.integers(0, 2000, size=k)
    x[0] = (2 ** 24 - 2048 + r).astype(np.float32)                 # 24 significant bits each
    x[1, :8] = [3.4028235e38, -3.4028235e38, 1.1754944e-38, 16777215.0, -0.0, 1e-30, 5e37, -1.0000001]
    x[2, 3] = np.inf
    x[3, 5] = np.nan
    w = np.empty((n, k), dtype=np.float32)
    h = n // 2
    w[:h] = np.where(np.arange(k) % 2 == 0, 1.0, -1.0)
    w[h:] = 0.5
    w[h:, 1] = -0.25
    out = c.output(m * n)
    c.launcher().launch(Kernel.matvec_bf16, P.MatvecBf16(n=n, k=k, col0=0, out_stride=n, eps=1e-6),
                        [c.upload(x), c.upload(synth.to_bf16_bits(w.reshape(-1))), out, c.upload(np.ones(k, dtype=np.float32))], (K.div_ceil(n, K.matvec_rows), m, 1))
    got = c.read(out).reshape(m, n)
    assert np.array_equal(got[0, :h], np.full(h, float(np.sum(r[0::2]) - np.sum(r[1::2])), dtype=np.float32))
    want1 = x[1].astype(np.float64) @ w[h:].astype(np.float64).T  # 0.5 * max - 0.25 * (-max) stays finite in f32
    assert np.all(np.isfinite(got[1, h:])) and np.max(np.abs(got[1, h:] - want1)) <= 1e-6 * np.max(np.abs(want1))
    assert np.all(np.isposinf(got[2, h:]))
    assert np.all(np.isnan(got[3]))


@pytest.mark.parametrize("half", HALVES)
def test_matvec_bf16_silu_pair(ctx, half):
    c = ctx
    rows, ff, k, eps = 3, 100, 1024, 1e-6
    x = c.random(rows * k, 3).reshape(rows, k)
    nw = c.random(k, 1)
    bits, values = random_half(c, 2 * ff * k, 1, half)
    values = values.reshape(2 * ff, k).astype(np.float64)
    out = c.output(rows * ff)
    c.launcher().launch(Kernel["matvec_" + half], P.MatvecBf16(n=ff, k=k, col0=0, out_stride=ff, eps=eps, norm=True, silu_pair=True, half=ff),
                        [c.upload(x), c.upload(bits), out, c.upload(nw)], (K.div_ceil(ff, K.matvec_rows), rows, 1))
    got = c.read(out).reshape(rows, ff)
    want = np.empty((rows, ff))
    for t in range(rows):
        xn = norm_row(x[t], nw, eps)
        g, u = values[:ff] @ xn, values[ff:] @ xn
        want[t] = g * sigmoid64(g) * u
    assert rel_err(got, want) <= 1e-5


# ---- quantized decode multiply: check.zig:988-1060 ------------------------------------

def quant_matvec(c, t: TensorType, k: int, pair: bool, variants=None):
    """3 tokens, 100 outputs, norm prologue and accumulate epilogue, or the
    SiLU pair over stacked gate and up rows; every variant tuning may pick; each
    token alone must give the same bits as in the 3-token launch."""
    rows, n, eps = 3, 100, 1e-6
    x = c.random(rows * k, 3).reshape(rows, k)
    nw = c.random(k, 1)
    raw, values = quant_rows(c, t, 2 * n if pair else n, k)
    init = c.random(rows * n, 0 if pair else 4).reshape(rows, n)
    kernel = K.weight_kernel("matvec", t)
    xa, wa, na = c.upload(x), c.gpu_weights(t, raw, k), c.upload(nw)
    worst, split_exact = 0.0, True
    want = np.empty((rows, n))
    v64 = values.astype(np.float64)
    for tk in range(rows):
        xn = norm_row(x[tk], nw, eps)
        g = v64[:n] @ xn
        want[tk] = g * sigmoid64(g) * (v64[n:] @ xn) if pair else init[tk] + g
    for v in variants or K.MatvecVariant.candidates:
        if not v.suits(t):
            continue
        p = lambda: P.MatvecBf16(n=n, k=k, col0=0, out_stride=n, eps=eps, norm=True, accumulate=not pair, silu_pair=pair, half=n if pair else 0)
        pipeline = c.set.matvec(c.rec, kernel, v)
        out = c.upload(init)
        c.launcher().launch_pipeline(pipeline, p(), [xa, wa, out, na], (K.div_ceil(n, v.group_rows()), rows, 1))
        got = c.read(out).reshape(rows, n)
        for tk in range(rows):
            single = c.upload(init[tk])
            c.launcher().launch_pipeline(pipeline, p(), [c.upload(x[tk]), wa, single, na], (K.div_ceil(n, v.group_rows()), 1, 1))
            split_exact &= got[tk].tobytes() == c.read(single).tobytes()
        worst = max(worst, rel_err(got, want))
    return worst, split_exact


@pytest.mark.parametrize("t,k,pair", [
    (TensorType.q8_0, 1024, False),   # "matvec q8_0 norm+="
    (TensorType.q4_k, 1024, False),   # "matvec q4_k norm+="
    (TensorType.q4_k, 4096, False),   # "matvec q4_k norm+= (2 tiles)"
    (TensorType.q8_0, 4160, True),    # "matvec q8_0 norm+silu (tile tail, bitwise splits)"
    (TensorType.q4_k, 1024, True),    # the SiLU pair on Q4_K (the reference runs it on q3_k)
    (TensorType.q3_k, 1024, False),   # "matvec q3_k norm+="
    (TensorType.q3_k, 1024, True),    # "matvec q3_k norm+silu pair"
    (TensorType.q5_k, 1024, False),   # "matvec q5_k norm+="
    (TensorType.q6_k, 1024, False),   # "matvec q6_k norm+="
    (TensorType.q6_k, 2304, True),    # the SiLU pair on Q6_K, nine blocks a row
    (TensorType.q5_k, 4096, True),
    # k above 4096: the lane walks several tasks, inputs read from LDS.
    (TensorType.q4_k, 14336, False),
    (TensorType.q4_k, 5120, True),
    (TensorType.q8_0, 14336, True),
    (TensorType.q8_0, 8224, False),   # 128.5 tasks: a tail in the third wave
    (TensorType.q6_k, 8192, False),
    (TensorType.q3_k, 16384, True),
    (TensorType.q5_k, 4352, True),
    (TensorType.q4_k, 16640, False),
])
def test_quant_matvec(ctx, t, k, pair):
    worst, split_exact = quant_matvec(ctx, t, k, pair)
    assert split_exact, "a token's sums differ between a lone launch and a multi-token launch"
    assert worst <= 1e-5


@pytest.mark.parametrize("t,k", [
    (TensorType.q8_0, 256),     # the reference's case
    (TensorType.q8_0, 8192),    # long rows: a step of three tokens goes tile by tile, a lone token slice by slice
    (TensorType.q6_k, 12288),   # ... with the inputs staged permuted
    (TensorType.q4_k, 14336),
])
def test_quant_matvec_act_prologue(ctx, t, k):
    """hc_act fused into the multiply after it: each input staged as
    silu(x / 4), read from rows 8 floats further apart than their length (src/kernels/check.zig:1082-1116);
    each token alone gives the same bits as in the three-token launch."""
    c = ctx
    rows, n, div = 3, 100, 4
    stride = k + 8
    x = c.random(rows * stride, 3).reshape(rows, stride)
    raw, values = quant_rows(c, t, n, k)
    xa, wa = c.upload(x), c.gpu_weights(t, raw, k)
    v = x[:, :k].astype(np.float64) / div
    want = (v * sigmoid64(v)) @ values.astype(np.float64).T
    worst = 0.0
    for cand in K.MatvecVariant.candidates:
        if not cand.suits(t):
            continue
        var = K.MatvecVariant(cand.wg, cand.lanes, cand.rows, div)
        pipeline = c.set.matvec(c.rec, K.weight_kernel("matvec", t), var)
        p = lambda: P.MatvecBf16(n=n, k=k, col0=0, out_stride=n, x_stride=stride // 4)
        out = c.output(rows * n)
        c.launcher().launch_pipeline(pipeline, p(), [xa, wa, out, wa], (K.div_ceil(n, var.group_rows()), rows, 1))
        got = c.read(out).reshape(rows, n)
        worst = max(worst, rel_err(got, want))
        for tk in range(rows):
            single = c.output(n)
            c.launcher().launch_pipeline(pipeline, p(), [c.upload(x[tk]), wa, single, wa], (K.div_ceil(n, var.group_rows()), 1, 1))
            assert got[tk].tobytes() == c.read(single)[:n].tobytes(), "a token's sums differ between a lone launch and a multi-token launch"
    assert worst <= 1e-5


@pytest.mark.parametrize("t,k,pair,rows,n", [
    (TensorType.q4_k, 14336, False, 2, 37),   # two tokens whose inputs do not fit LDS together: the tile-by-tile kernel's two-token form
    (TensorType.q8_0, 10240, True, 2, 19),
    (TensorType.q5_k, 16384, False, 4, 9),    # 256 tasks: four whole slices, a batch of rows with units past the end
    (TensorType.q3_k, 4352, False, 1, 3),     # 68 tasks: a second slice of four lanes, three rows
    (TensorType.q6_k, 16640, False, 2, 21),   # 260 tasks: past the sliced kernel's four slices, short of its five
    (TensorType.q4_k, 25600, False, 2, 37),   # 400 tasks: seven slices, the last a quarter full
    (TensorType.q8_0, 32768, False, 3, 20),   # eight slices, the longest row
    (TensorType.q5_k, 20480, False, 2, 11),   # five slices
    (TensorType.q3_k, 24576, False, 2, 9),    # six slices
    (TensorType.q4_k, 11008, False, 2, 30),   # two tokens over three slices: a workgroup of six waves
    (TensorType.q8_0, 8192, False, 2, 70),    # two tokens over two slices
    # Steps of exactly two tokens over short rows keep both tokens' inputs in registers:
    (TensorType.q4_k, 4096, True, 2, 100),
    (TensorType.q3_k, 3072, True, 2, 21),     # 48 tasks: idle lanes
    (TensorType.q5_k, 4096, True, 2, 40),     # (a format whose gate / up step of two tokens stays on the general kernel)
    (TensorType.q8_0, 2048, False, 2, 50),    # two rows a wave pass
    (TensorType.q6_k, 1024, False, 2, 33),    # four rows a wave pass, a ragged last pass
    (TensorType.q5_k, 4096, False, 2, 64),
])
def test_quant_matvec_long_rows(ctx, t, k, pair, rows, n):
    """Rows of more than 4096 weights at the widths and edges test_quant_matvec leaves out:
    within 1e-5 of float64, with the norm prologue and the accumulate epilogue (or the SiLU
    pair), and each token bitwise equal to its lone launch."""
    c = ctx
    eps = 1e-6
    x = c.random(rows * k, 3).reshape(rows, k)
    nw = c.random(k, 1)
    raw, values = quant_rows(c, t, 2 * n if pair else n, k)
    init = c.random(rows * n, 0 if pair else 4).reshape(rows, n)
    xa, wa, na = c.upload(x), c.gpu_weights(t, raw, k), c.upload(nw)
    v64 = values.astype(np.float64)
    want = np.empty((rows, n))
    for tk in range(rows):
        xn = norm_row(x[tk], nw, eps)
        g = v64[:n] @ xn
        want[tk] = g * sigmoid64(g) * (v64[n:] @ xn) if pair else init[tk] + g
    v = K.MatvecVariant()
    p = lambda: P.MatvecBf16(n=n, k=k, col0=0, out_stride=n, eps=eps, norm=True, accumulate=not pair, silu_pair=pair, half=n if pair else 0)
    pipeline = c.set.matvec(c.rec, K.weight_kernel("matvec", t), v)
    out = c.upload(init)
    c.launcher().launch_pipeline(pipeline, p(), [xa, wa, out, na], (K.div_ceil(n, v.group_rows()), rows, 1))
    got = c.read(out).reshape(rows, n)
    assert rel_err(got, want) <= 1e-5
    for tk in range(rows):
        single = c.upload(init[tk])
        c.launcher().launch_pipeline(pipeline, p(), [c.upload(x[tk]), wa, single, na], (K.div_ceil(n, v.group_rows()), 1, 1))
        assert got[tk].tobytes() == c.read(single).tobytes(), "a token's sums differ between a lone launch and a multi-token launch"


def test_quant_matvec_eight_rows(ctx):
    """Steps of 5..8 tokens (the HIP backend's extension past the reference's
    four): every row correct and bitwise equal to its lone launch."""
    c = ctx
    n, k, rows = 96, 1024, 8
    x = c.random(rows * k, 3).reshape(rows, k)
    raw, values = quant_rows(c, TensorType.q4_k, 2 * n, k)
    xa, wa = c.upload(x), c.gpu_weights(TensorType.q4_k, raw, k)
    p = lambda: P.MatvecBf16(n=n, k=k, col0=0, out_stride=n, silu_pair=True, half=n)
    out = c.output(rows * n)
    c.launcher().launch(Kernel.matvec_q4_k, p(), [xa, wa, out, wa], (K.div_ceil(n, 8), rows, 1))
    got = c.read(out).reshape(rows, n)
    v64 = values.astype(np.float64)
    g, u = x.astype(np.float64) @ v64[:n].T, x.astype(np.float64) @ v64[n:].T
    assert rel_err(got, g * sigmoid64(g) * u) <= 1e-5
    for tk in range(rows):
        single = c.output(n)
        c.launcher().launch(Kernel.matvec_q4_k, p(), [c.upload(x[tk]), wa, single, wa], (K.div_ceil(n, 8), 1, 1))
        assert got[tk].tobytes() == c.read(single)[:n].tobytes()


MFMA_VARIANT = K.MatvecVariant(wg=512, lanes=64, rows=16)


@pytest.mark.parametrize("pair,rows,n,k", [
    (True, 8, 200, 1024),     # partial last tile, one slab
    (True, 5, 96, 4096),      # four slabs
    (False, 3, 100, 2048),    # accumulate epilogue, an odd token count
    (False, 1, 530, 1024),    # one token, more than one workgroup
    # k of 2048 or 4096 and whole tiles: the kernel with the tokens' operands in registers
    (False, 8, 4112, 4096),   # 257 tiles: a second tile for the first workgroup
    (True, 8, 4128, 4096),    # gate and up tiles of 258 output tiles
    (True, 3, 64, 2048),      # one block a wave
    (False, 2, 48, 2048),
    # rows of more than 4096 weights: workgroups that share a tile, 2048 columns each (with the
    # RMSNorm prologue the tokens' scales come from a launch of their own)
    (False, 8, 1296, 14336),  # seven parts, 81 tiles over 36 walkers: two rounds and nine tiles in halves
    (True, 4, 528, 8192),     # four parts, gate and up, fewer tiles than walkers
    (False, 5, 4096, 6144),   # three parts, 256 tiles over 85 walkers: one whole tile left over
    (False, 3, 528, 28672),   # fourteen parts
])
@pytest.mark.parametrize("prologue", ["plain", "norm", "norm_act"])
@pytest.mark.parametrize("t", [TensorType.q4_k, TensorType.q5_k])
def test_quant_matvec_mfma_variant(ctx, t, pair, rows, n, k, prologue):
    """The matrix-core variant of matvec_q4_k and matvec_q5_k (a wave per sixteen rows; Q5_K has
    it for k of 2048 or 4096 and whole tiles, its other cases run the default variant): every
    row within 1e-5 of float64 over the decoded weights, each token bitwise
    equal to its lone launch, and nothing outside the outputs touched; also
    with the prologues the planner's launches carry (RMSNorm times its weights
    on every projection, src/plan/qwen35.zig:1006,1048, and silu(x / act_div))."""
    c = ctx
    norm, div, eps = prologue != "plain", 4 if prologue == "norm_act" else 0, 1e-6
    x = c.random(rows * k, 3).reshape(rows, k)
    x[0] *= np.float32(1e-4)          # tokens of very different magnitudes
    x[rows - 1] *= np.float32(300.0)
    nw = c.random(k, 1.5)
    raw, values = quant_rows(c, t, 2 * n if pair else n, k)
    stride = n + 7
    init = c.random(rows * stride, 2).reshape(rows, stride)
    xa, wa = c.upload(x), c.gpu_weights(t, raw, k)
    na = c.upload(nw) if norm else wa
    v64 = values.astype(np.float64)
    x64 = np.stack([norm_row(r, nw if norm else None, eps) for r in x])
    if div:
        x64 = (x64 / div) * sigmoid64(x64 / div)
    if pair:
        g, u = x64 @ v64[:n].T, x64 @ v64[n:].T
        want = g * sigmoid64(g) * u
    else:
        want = init[:, 3 : 3 + n] + x64 @ v64.T
    p = lambda: P.MatvecBf16(n=n, k=k, col0=3, out_stride=stride, eps=eps, norm=norm, accumulate=not pair, silu_pair=pair, half=n if pair else 0)
    variant = K.MatvecVariant(MFMA_VARIANT.wg, MFMA_VARIANT.lanes, MFMA_VARIANT.rows, div)
    pipeline = c.set.matvec(c.rec, K.weight_kernel("matvec", t), variant)
    grid_x = K.div_ceil(n, variant.group_rows())
    out = c.upload(init)
    c.launcher().launch_pipeline(pipeline, p(), [xa, wa, out, na], (grid_x, rows, 1))
    got = c.read(out).reshape(rows, stride)
    # Row by row: each token against its own output scale.
    for tk in range(rows):
        assert rel_err(got[tk, 3 : 3 + n], want[tk]) <= 1e-5, tk
    mask = np.ones(stride, dtype=bool)
    mask[3 : 3 + n] = False
    assert np.array_equal(got[:, mask].view(np.uint32), init[:, mask].view(np.uint32))
    for tk in range(rows):
        single = c.upload(init[tk])
        c.launcher().launch_pipeline(pipeline, p(), [c.upload(x[tk]), wa, single, na], (grid_x, 1, 1))
        assert got[tk].tobytes() == c.read(single)[:stride].tobytes(), "a token's sums differ between a lone launch and a multi-token launch"


@pytest.mark.parametrize("rows,n,k,col0,pad,accumulate", [
    (8, 200, 1024, 3, 7, True),      # partial last tile, unaligned rows
    (5, 96, 4096, 4, 8, False),      # aligned rows: 16-byte stores
    (3, 100, 2080, 0, 0, True),      # k = 65 blocks: a ragged last step
    (1, 530, 1024, 0, 2, False),     # one token
    (8, 4112, 4096, 0, 0, False),    # 257 sixteen-row tiles: the kernel that streams whole tiles, two tiles on one workgroup
    (7, 4112, 2048, 5, 7, True),     # the same with eight blocks a wave, unaligned outputs, accumulating
    (2, 1536, 4096, 0, 0, True),
    (8, 4112, 1024, 0, 0, False),    # rows of 1024 weights: the kernel that moves a tile's 32 rows as one flat stretch
    (3, 4128, 1024, 5, 7, True),
    (4, 5, 1024, 1, 2, True),        # fewer rows than a unit of eight
    # rows of more than 4096 weights: workgroups that share a tile, 2048 columns each
    (8, 1296, 14336, 3, 7, True),    # seven parts, 81 tiles over 36 walkers
    (3, 4096, 6144, 0, 0, False),    # three parts, 256 tiles over 85 walkers
    (5, 48, 8192, 0, 0, False),      # four parts, fewer tiles than walkers
    (2, 272, 20480, 0, 0, False),    # ten parts
])
def test_matvec_q8_0_mfma_variant(ctx, rows, n, k, col0, pad, accumulate):
    """The matrix-core variant of matvec_q8_0 (the id of a wave per sixteen rows): every
    token within 1e-5 of float64 over the decoded weights whatever its magnitude (each token
    is scaled by its own power of two), each token bitwise equal to its lone launch, nothing
    outside the outputs touched."""
    c = ctx
    x = c.random(rows * k, 3).reshape(rows, k)
    x[0] *= np.float32(1e-6)          # tokens of very different magnitudes, beyond the f16 range both ways
    x[rows - 1] *= np.float32(3e6)
    raw, values = quant_rows(c, TensorType.q8_0, n, k)
    stride = n + pad
    init = c.random(rows * stride, 2).reshape(rows, stride)
    xa, wa = c.upload(x), c.gpu_weights(TensorType.q8_0, raw, k)
    want = x.astype(np.float64) @ values.astype(np.float64).T + (init[:, col0 : col0 + n] if accumulate else 0)
    p = lambda: P.MatvecBf16(n=n, k=k, col0=col0, out_stride=stride, accumulate=accumulate)
    pipeline = c.set.matvec(c.rec, Kernel.matvec_q8_0, MFMA_VARIANT)
    grid_x = K.div_ceil(n, MFMA_VARIANT.group_rows())
    out = c.upload(init)
    c.launcher().launch_pipeline(pipeline, p(), [xa, wa, out, wa], (grid_x, rows, 1))
    got = c.read(out).reshape(rows, stride)
    prod = x.astype(np.float64) @ values.astype(np.float64).T
    for tk in range(rows):
        # Against the product's own scale (an accumulated init may dwarf a tiny token's product).
        assert np.max(np.abs(got[tk, col0 : col0 + n] - want[tk])) <= 1e-5 * max(np.max(np.abs(prod[tk])), 1e-30) + 1e-6 * np.max(np.abs(want[tk])), tk
    mask = np.ones(stride, dtype=bool)
    mask[col0 : col0 + n] = False
    assert np.array_equal(got[:, mask].view(np.uint32), init[:, mask].view(np.uint32))
    for tk in range(rows):
        single = c.upload(init[tk])
        c.launcher().launch_pipeline(pipeline, p(), [c.upload(x[tk]), wa, single, wa], (grid_x, 1, 1))
        assert got[tk].tobytes() == c.read(single)[:stride].tobytes(), "a token's sums differ between a lone launch and a multi-token launch"


@pytest.mark.parametrize("norm", [False, True])
@pytest.mark.parametrize("rows,n,k", [(8, 4128, 4096), (3, 64, 2048), (5, 3072, 1024), (2, 4104, 1024),
                                      (6, 528, 8192), (3, 1304, 6144)])  # rows in four and in three parts (1304 outputs: whole rounds and a ragged tail)
@pytest.mark.parametrize("t", [TensorType.q8_0, TensorType.q6_k, TensorType.q3_k])
def test_matvec_q8_0_mfma_variant_silu_pair(ctx, t, rows, n, k, norm):
    """The matrix-core variant of matvec_q8_0, matvec_q6_k and matvec_q3_k on the fused gate / up step (SILU_PAIR: gate rows,
    then the up rows `half` further down; with the RMSNorm the planner's FFN launch carries):
    silu(gate) * up within 1e-5 of float64 row by row, each token bitwise equal to its lone
    launch. (4104 outputs: 513 eight-row units, the last tile shared by two workgroups.)"""
    c = ctx
    eps = 1e-6
    x = c.random(rows * k, 3).reshape(rows, k)
    x[0] *= np.float32(1e-3)
    nw = c.random(k, 1.5)
    raw, values = quant_rows(c, t, 2 * n, k)
    xa, wa, na = c.upload(x), c.gpu_weights(t, raw, k), c.upload(nw)
    x64 = np.stack([norm_row(r, nw if norm else None, eps) for r in x])
    v64 = values.astype(np.float64)
    g, u = x64 @ v64[:n].T, x64 @ v64[n:].T
    want = g * sigmoid64(g) * u
    p = lambda: P.MatvecBf16(n=n, k=k, col0=0, out_stride=n, eps=eps, norm=norm, silu_pair=True, half=n)
    pipeline = c.set.matvec(c.rec, K.weight_kernel("matvec", t), MFMA_VARIANT)
    grid_x = K.div_ceil(n, MFMA_VARIANT.group_rows())
    out = c.output(rows * n)
    c.launcher().launch_pipeline(pipeline, p(), [xa, wa, out, na], (grid_x, rows, 1))
    got = c.read(out).reshape(rows, n)
    for tk in range(rows):
        assert rel_err(got[tk], want[tk]) <= 1e-5, tk
    for tk in (0, rows - 1):
        single = c.output(n)
        c.launcher().launch_pipeline(pipeline, p(), [c.upload(x[tk]), wa, single, na], (grid_x, 1, 1))
        assert got[tk].tobytes() == c.read(single)[:n].tobytes(), "a token's sums differ between a lone launch and a multi-token launch"


@pytest.mark.parametrize("prologue", ["norm", "norm_act"])
@pytest.mark.parametrize("rows,n,k", [(6, 4112, 4096), (3, 96, 2048), (2, 200, 1024), (4, 4128, 1024), (5, 1040, 14336)])
def test_matvec_q8_0_mfma_variant_prologues(ctx, rows, n, k, prologue):
    """The matrix-core variant of matvec_q8_0 on steps with the RMSNorm and silu(x / act_div)
    prologues (src/kernels/matvec_quant.wgsl.hbs:73-89), which the streaming kernel computes
    as it builds the tokens' operands (200 rows of 1024 weights: the kernel that takes a
    tile's rows as one flat stretch, a workgroup's share of the last rows); 1e-5 against float64, each token bitwise equal to its lone launch."""
    c = ctx
    div, eps = 4 if prologue == "norm_act" else 0, 1e-6
    x = c.random(rows * k, 3).reshape(rows, k)
    x[0] *= np.float32(1e-4)
    nw = c.random(k, 1.5)
    raw, values = quant_rows(c, TensorType.q8_0, n, k)
    init = c.random(rows * n, 2).reshape(rows, n)
    xa, wa, na = c.upload(x), c.gpu_weights(TensorType.q8_0, raw, k), c.upload(nw)
    x64 = np.stack([norm_row(r, nw, eps) for r in x])
    if div:
        x64 = (x64 / div) * sigmoid64(x64 / div)
    want = init + x64 @ values.astype(np.float64).T
    p = lambda: P.MatvecBf16(n=n, k=k, col0=0, out_stride=n, eps=eps, norm=True, accumulate=True)
    variant = K.MatvecVariant(MFMA_VARIANT.wg, MFMA_VARIANT.lanes, MFMA_VARIANT.rows, div)
    pipeline = c.set.matvec(c.rec, Kernel.matvec_q8_0, variant)
    grid_x = K.div_ceil(n, variant.group_rows())
    out = c.upload(init)
    c.launcher().launch_pipeline(pipeline, p(), [xa, wa, out, na], (grid_x, rows, 1))
    got = c.read(out).reshape(rows, n)
    for tk in range(rows):
        assert rel_err(got[tk], want[tk]) <= 1e-5, tk
    for tk in range(rows):
        single = c.upload(init[tk])
        c.launcher().launch_pipeline(pipeline, p(), [c.upload(x[tk]), wa, single, na], (grid_x, 1, 1))
        assert got[tk].tobytes() == c.read(single)[:n].tobytes(), "a token's sums differ between a lone launch and a multi-token launch"


@pytest.mark.parametrize("rows,n,k,col0,pad,accumulate,prologue", [
    (8, 8224, 4096, 0, 0, False, None),        # whole rounds of 32-row tiles and a tail on every workgroup
    (5, 9000, 4096, 0, 0, True, None),         # a ragged last unit of rows
    (3, 100, 2048, 3, 7, True, None),          # fewer rows than workgroups, unaligned columns
    (1, 530, 2048, 0, 2, False, None),         # one token
    (6, 4100, 2048, 0, 0, False, "norm"),
    (4, 300, 4096, 5, 0, True, "norm_act"),
    (2, 64, 1024, 0, 0, False, None),          # one unit a tile
    (7, 8232, 1024, 0, 0, True, "norm"),
    (3, 96, 3072, 0, 0, False, None),          # three units a tile
    (6, 1000, 3072, 3, 2, True, "norm"),
    (2, 64, 5120, 0, 0, False, None),          # k the kernel does not take: the default variant's
    # rows of more than 4096 weights: workgroups that share a tile, 2048 columns each
    (8, 1300, 14336, 3, 2, True, None),        # seven parts, 36 walkers: whole rounds, a tail, a ragged last unit
    (4, 4096, 6144, 0, 0, False, None),        # three parts, at most four tokens
    (5, 200, 8192, 0, 0, True, "act"),         # four parts, fewer rows than walkers
    (2, 96, 14336, 0, 0, False, "norm"),       # with the RMSNorm prologue: the tokens' scales from a launch of their own
    (3, 300, 28672, 0, 0, True, "norm_act"),   # fourteen parts
])
@pytest.mark.parametrize("t", [TensorType.q6_k, TensorType.q3_k])
def test_matvec_q6_k_mfma_variant(ctx, t, rows, n, k, col0, pad, accumulate, prologue):
    """matvec_q6_k and matvec_q3_k on the matrix-core variant id (a wave per sixteen rows): the weights are read
    once for all tokens of the step, the tokens split into two f16 rows by every workgroup (with
    the RMSNorm and silu(x / act_div) prologues of src/kernels/matvec_quant.wgsl.hbs:73-89 where
    the step has them). 1e-5 against float64; columns outside the launch untouched; each token bitwise equal
    to its lone launch."""
    c = ctx
    stride = col0 + n + pad
    div, eps = 4 if prologue in ("norm_act", "act") else 0, 1e-6
    norm = prologue in ("norm", "norm_act")
    x = c.random(rows * k, 3).reshape(rows, k)
    x[0] *= np.float32(1e-4)
    nw = c.random(k, 1.5)
    raw, values = quant_rows(c, t, n, k)
    init = c.random(rows * stride, 2).reshape(rows, stride)
    xa, wa, na = c.upload(x), c.gpu_weights(t, raw, k), c.upload(nw)
    x64 = np.stack([norm_row(r, nw if norm else None, eps) for r in x])
    if div:
        x64 = (x64 / div) * sigmoid64(x64 / div)
    prod = x64 @ values.astype(np.float64).T
    want = prod + (init[:, col0 : col0 + n] if accumulate else 0)
    p = lambda: P.MatvecBf16(n=n, k=k, col0=col0, out_stride=stride, eps=eps, norm=norm, accumulate=accumulate)
    variant = K.MatvecVariant(MFMA_VARIANT.wg, MFMA_VARIANT.lanes, MFMA_VARIANT.rows, div)
    pipeline = c.set.matvec(c.rec, K.weight_kernel("matvec", t), variant)
    grid_x = K.div_ceil(n, variant.group_rows())
    out = c.upload(init)
    c.launcher().launch_pipeline(pipeline, p(), [xa, wa, out, na], (grid_x, rows, 1))
    got = c.read(out).reshape(rows, stride)
    for tk in range(rows):
        # Against the product's own scale (an accumulated init may dwarf a tiny token's product).
        assert np.max(np.abs(got[tk, col0 : col0 + n] - want[tk])) <= 1e-5 * max(np.max(np.abs(prod[tk])), 1e-30) + 1e-6 * np.max(np.abs(want[tk])), tk
    mask = np.ones(stride, dtype=bool)
    mask[col0 : col0 + n] = False
    assert np.array_equal(got[:, mask].view(np.uint32), init[:, mask].view(np.uint32))
    for tk in (0, rows - 1):
        single = c.upload(init[tk])
        c.launcher().launch_pipeline(pipeline, p(), [c.upload(x[tk]), wa, single, na], (grid_x, 1, 1))
        assert got[tk].tobytes() == c.read(single)[:stride].tobytes(), "a token's sums differ between a lone launch and a multi-token launch"


# ---- block decoders bit for bit, through the embedding gathers: check.zig:873-905 -----

@pytest.mark.parametrize("t", [TensorType.q8_0, TensorType.q3_k, TensorType.q4_k, TensorType.q5_k, TensorType.q6_k])
def test_embed_quant_bit_exact(ctx, t):
    c = ctx
    vocab, dim, split = 50, 512, 30
    e, b = K.LAYOUT[t]
    rb = dim // e * b
    raw, values = quant_rows(c, t, vocab, dim)
    raw = raw.reshape(vocab, rb)
    tokens = np.array([0, 29, 30, 49, 7, 30, 12], dtype=np.uint32)
    out = c.output(tokens.size * dim)
    ta = c.upload(tokens)
    for row0, rows in ((0, split), (split, vocab - split)):
        wa = c.gpu_weights(t, raw[row0 : row0 + rows], dim)
        c.launcher().launch(K.weight_kernel("embed", t), P.EmbedBf16(dim=dim, row0=row0, chunk_rows=rows), [ta, wa, out], (tokens.size, 1, 1))
    got = c.read_words(out).reshape(tokens.size, dim)
    want = values[tokens].view(np.uint32)
    assert np.array_equal(got, want), f"{np.count_nonzero(got != want)} decoded weights differ in their bits"


def test_embed_q8_0_file_rows(ctx):
    """Rows laid out as in the GGUF file, `stride` bytes apart
    (src/kernels/embed_quant.wgsl:4-6)."""
    c = ctx
    vocab, dim = 9, 256
    stride = dim // 32 * 34 + 12
    raw, values = quant_rows(c, TensorType.q8_0, vocab, dim)
    table = np.zeros((vocab, stride), dtype=np.uint8)
    table[:, : dim // 32 * 34] = raw.reshape(vocab, -1)
    tokens = np.array([8, 0, 3], dtype=np.uint32)
    out = c.output(tokens.size * dim)
    c.launcher().launch(Kernel.embed_q8_0, P.EmbedBf16(dim=dim, row0=0, chunk_rows=vocab, stride=stride), [c.upload(tokens), c.upload(table), out], (tokens.size, 1, 1))
    assert np.array_equal(c.read_words(out).reshape(tokens.size, dim), values[tokens].view(np.uint32))


def test_embed_iq4_xs_exact(ctx):
    """The reference's kernel check (src/kernels/check.zig:925-985): scale codes,
    indices and five super-scales cycling over the blocks, two row chunks, a
    token out of range left untouched; once from the padded layout, once from
    file rows an unaligned stride apart. Bit for bit against the decoder."""
    c = ctx
    vocab, dim, split = 8, 8448, 3
    per_row = dim // 256
    row_bytes = per_row * 136
    raw = np.zeros((vocab * per_row, 136), dtype=np.uint8)
    ds = np.array([0.0078125, -0.01171875, 0.009765625, 0, -0.00390625], dtype=np.float16)
    i = np.arange(16)
    for b in range(vocab * per_row):
        raw[b, 0:2] = ds[b % 5 : b % 5 + 1].view(np.uint8)
        high = 0
        for s in range(8):
            scale = (b * 8 + s) % 64
            raw[b, 4 + s // 2] |= (scale & 15) << (4 * (s % 2))
            high |= (scale >> 4) << (2 * s)
            raw[b, 8 + 16 * s : 24 + 16 * s] = ((i + 3 * s + b) % 16) | (((15 - i + 5 * s + 3 * b) % 16) << 4)
        raw[b, 2], raw[b, 3] = high & 0xFF, high >> 8
    raw = raw.reshape(vocab, row_bytes)
    values = oracle.dequantize(oracle.IQ4_XS, raw, vocab * dim).reshape(vocab, dim)
    tokens = np.array([7, 0, 2, 3, 4, 7, 1, 8], dtype=np.uint32)
    ta = c.upload(tokens)
    want = np.full((tokens.size, dim), -9999, dtype=np.float32)
    want[:7] = values[tokens[:7]]
    for strided in (False, True):
        out = c.upload(np.full(tokens.size * dim, -9999, dtype=np.float32))
        for row0, rows in ((0, split), (split, vocab - split)):
            if strided:
                stride = row_bytes + 4
                spaced = np.full((rows * stride + 15) & ~15, 0xA5, dtype=np.uint8)
                for r in range(rows):
                    spaced[r * stride : r * stride + row_bytes] = raw[row0 + r]
                wa = c.upload(spaced)
            else:
                stride = 0
                wa = c.gpu_weights(TensorType.iq4_xs, raw[row0 : row0 + rows], dim)
            c.launcher().launch(Kernel.embed_iq4_xs, P.EmbedBf16(dim=dim, row0=row0, chunk_rows=rows, stride=stride), [ta, wa, out], (tokens.size, 1, 1))
        got = c.read_words(out).reshape(tokens.size, dim)
        assert np.array_equal(got, want.view(np.uint32)), f"strided={strided}: {np.count_nonzero(got != want.view(np.uint32))} values differ"


@pytest.mark.parametrize("half", HALVES)
def test_embed_bf16_exact(ctx, half):
    c = ctx
    vocab, dim, split = 50, 64, 30
    bits, values = random_half(c, vocab * dim, 1, half)
    bits, values = bits.reshape(vocab, dim), values.reshape(vocab, dim)
    tokens = np.array([0, 29, 30, 49, 7, 30, 12], dtype=np.uint32)
    out = c.output(tokens.size * dim)
    ta = c.upload(tokens)
    for row0, rows in ((0, split), (split, vocab - split)):
        c.launcher().launch(Kernel["embed_" + half], P.EmbedBf16(dim=dim, row0=row0, chunk_rows=rows), [ta, c.upload(bits[row0 : row0 + rows]), out], (tokens.size, 1, 1))
    assert np.array_equal(c.read(out).reshape(tokens.size, dim), values[tokens])


def test_repack_q8_0_matches_split_row_layout(ctx):
    c = ctx
    rows, k = 37, 320  # 320 + 20 scale bytes pads to 352
    raw, _ = quant_rows(c, TensorType.q8_0, rows, k)
    wa = c.gpu_weights(TensorType.q8_0, raw, k)
    got = c.read_bytes(wa)[: rows * K.row_bytes(TensorType.q8_0, k)]
    assert np.array_equal(got, oracle.repack_q8_0(raw, rows, k))


def test_repack_q3_k_matches_unit_layout(ctx):
    """repack_q3_k against the oracle's restatement of the same layout, byte for byte."""
    c = ctx
    blocks = 37
    raw = synth.random_blocks(c.rand, "q3_k", 1, blocks * 256)
    padded = np.zeros((raw.size + 15) & ~15, dtype=np.uint8)
    padded[: raw.size] = raw
    out = c.output(blocks * 128 // 4)
    c.launcher().launch(Kernel.repack_q3_k, P.RepackQ3K(blocks), [c.upload(padded), out], K.elementwise(blocks * 8))
    got = c.read_words(out).view(np.uint8)[: blocks * 128]
    assert np.array_equal(got, oracle.repack_q3_k(raw, blocks))


def test_repad_pads_blocks(ctx):
    c = ctx
    blocks, src_bytes, dst_bytes = 23, 110, 128  # a block size that is not a multiple of 4
    raw = c.rand.integers(0, 256, size=(blocks, src_bytes), dtype=np.uint8)
    padded = np.zeros(((raw.size + 15) & ~15), dtype=np.uint8)
    padded[: raw.size] = raw.reshape(-1)
    out = c.output(blocks * dst_bytes // 4)
    c.launcher().launch(Kernel.repad, P.Repad(blocks, src_bytes, dst_bytes), [c.upload(padded), out], K.elementwise(blocks * dst_bytes // 4))
    got = c.read_bytes(out).reshape(blocks, dst_bytes)
    assert np.array_equal(got[:, :src_bytes], raw) and not got[:, src_bytes:].any()


# ---- prefill multiplies: check.zig:288-325, 752-825 -------------------------------------

def matmul_case(c, rows, n, k, split, accumulate, rung=K.Prefill.scalar_f32, half="bf16"):
    x = c.random(rows * k, 1).reshape(rows, k)
    bits, values = random_half(c, n * k, 1, half)
    bits, values = bits.reshape(n, k), values.reshape(n, k)
    init = c.random(rows * n, 4 if accumulate else 0).reshape(rows, n)
    packed = rung == K.Prefill.bf16_mfma_xbf16
    out, xa = c.upload(init), c.upload(synth.to_bf16_bits(x) if packed else x)
    c.set.select_prefill(c.rec, rung)
    col0 = 0
    for cols in (split or n, n - (split or n)):
        if cols == 0:
            continue
        wa = c.upload(bits[col0 : col0 + cols])
        c.launcher().launch(Kernel["matmul_" + half], P.MatmulBf16(rows=rows, n=cols, k=k, col0=col0, out_stride=n, accumulate=int(accumulate)),
                            [xa, wa, out], (K.div_ceil(cols, K.matmul_tile_n), K.div_ceil(rows, K.matmul_tile_t), 1))
        col0 += cols
    got = c.read(out).reshape(rows, n)
    c.set.select_prefill(c.rec, K.Prefill.scalar_f32)
    xs = x if rung == K.Prefill.scalar_f32 else synth.bf16_round(x)
    want = init + xs.astype(np.float64) @ values.astype(np.float64).T
    return got, want, values, x


@pytest.mark.parametrize("half", HALVES)
def test_matmul_bf16(ctx, half):
    # 19 tokens and 100 outputs leave partial tiles in both dimensions.
    got, want, _, _ = matmul_case(ctx, 19, 100, 1024, None, False, half=half)
    assert rel_err(got, want) <= 1e-5


@pytest.mark.parametrize("half", HALVES)
def test_matmul_bf16_chunked_accumulate(ctx, half):
    got, want, _, _ = matmul_case(ctx, 33, 150, 96, 70, True, half=half)
    assert rel_err(got, want) <= 1e-5


def test_matmul_bf16_mfma_rung(ctx):
    """The bf16 MFMA rung against its operand contract: x rounded to bf16,
    weights exact, products summed in float64. The rounded operands are the
    only difference from the f32 rung, so the bound stays 1e-5."""
    got, want, values, x = matmul_case(ctx, 19, 100, 1024, None, False, K.Prefill.bf16_mfma)
    assert rel_err(got, want) <= 1e-5
    got, want, values, x = matmul_case(ctx, 133, 150, 96, 70, True, K.Prefill.bf16_mfma)
    assert rel_err(got, want) <= 1e-5
    # The same with the activations bound as packed bf16 (an extension of the
    # contract, which binds f32): identical operands, so identical results.
    got, want, values, x = matmul_case(ctx, 133, 150, 96, 70, True, K.Prefill.bf16_mfma_xbf16)
    assert rel_err(got, want) <= 1e-5
    got, want, values, x = matmul_case(ctx, 300, 4100, 128, None, False, K.Prefill.bf16_mfma_xbf16)  # 128-token tiles
    assert rel_err(got, want) <= 1e-5


@pytest.mark.parametrize("rows,n,k", [
    (40, 200, 128),     # 64-token tiles, one k step
    (64, 64, 416),      # 64-token tiles, four steps, the last of 32 positions
    (129, 130, 1056),   # 128-token tiles, nine steps (three groups), ragged
    (200, 70, 480),     # four steps, the last of 96 positions
    (257, 100, 512),    # three token tiles, four whole steps
    (513, 16400, 320),  # 256-token tiling: 3 x 129 tiles fill the CUs; k ragged for its 64-deep tiles
    (1024, 8192, 256),  # 256-token tiling, whole tiles
])
def test_matmul_bf16_mfma_tilings(ctx, rows, n, k):
    """Every tiling and step-count path of the bf16 rung (64- and 128-token
    tiles, the 256-token tiling of long steps; whole groups of steps, left-over
    steps and a ragged last step), with bf16 and Q8_0 weights, f32 and packed
    bf16 activations, against the rung's operand contract."""
    c = ctx
    x = c.random(rows * k, 1).reshape(rows, k)
    xs = synth.bf16_round(x).astype(np.float64)
    # bf16 weights
    bits, values = random_half(c, n * k, 1)
    for rung in (K.Prefill.bf16_mfma, K.Prefill.bf16_mfma_xbf16):
        packed = rung == K.Prefill.bf16_mfma_xbf16
        xa = c.upload(synth.to_bf16_bits(x) if packed else x)
        c.set.select_prefill(c.rec, rung)
        out = c.output(rows * n)
        c.launcher().launch(Kernel.matmul_bf16, P.MatmulBf16(rows=rows, n=n, k=k, col0=0, out_stride=n), [xa, c.upload(bits.reshape(n, k)), out],
                            (K.div_ceil(n, K.matmul_tile_n), K.div_ceil(rows, K.matmul_tile_t), 1))
        got = c.read(out).reshape(rows, n)
        assert rel_err(got, xs @ values.reshape(n, k).astype(np.float64).T) <= 1e-5, rung
        # Q8_0 weights, accumulating into a strided output at a column offset.
        raw, wq = quant_rows(c, TensorType.q8_0, n, k)
        init = c.random(rows * (n + 9), 0.5).reshape(rows, n + 9)
        out = c.upload(init)
        c.launcher().launch(Kernel.matmul_q8_0_float, P.MatmulQuant(rows=rows, n=n, k=k, col0=5, out_stride=n + 9, accumulate=1, k_slice=k),
                            [xa, c.gpu_weights(TensorType.q8_0, raw, k), out], (K.div_ceil(n, 64), K.div_ceil(rows, 16), 1))
        got = c.read(out).reshape(rows, n + 9)
        want = init[:, 5 : 5 + n] + xs @ synth.bf16_round(wq).astype(np.float64).T
        assert rel_err(got[:, 5 : 5 + n], want) <= 1e-5, rung
        assert np.array_equal(got[:, :5], init[:, :5]) and np.array_equal(got[:, 5 + n :], init[:, 5 + n :]), "columns outside the chunk were written"
    c.set.select_prefill(c.rec, K.Prefill.scalar_f32)


@pytest.mark.parametrize("n", [2830, 8230])
@pytest.mark.parametrize("rung", ["bf16_mfma", "fp16_single"])
def test_matmul_q8_0_float_bf16_whole_steps_keep_token_bits(ctx, rung, n):
    """Q8_0 weights on the bf16 rung and on the reference's fp16_single rung with k a multiple
    of 128 take the kernels with producer waves and 32 x 32 x 16 MFMAs in 128- or 64-token
    tiles (64 matrix rows a tile; 128 where the matrix has the rows to fill the CUs with those,
    n = 8230): a token's sums are the same bits whichever tile height its step runs in and
    whichever tokens share the step; ragged rows and outputs, a column offset and a padded stride."""
    c = ctx
    rows, k, col0, stride = 300, 384, 3, n + 10
    x = c.random(rows * k, 1).reshape(rows, k)
    raw, wq = quant_rows(c, TensorType.q8_0, n, k)
    wa = c.gpu_weights(TensorType.q8_0, raw, k)
    c.set.select_prefill(c.rec, K.Prefill[rung])
    init = c.random(rows * stride, 0.5).reshape(rows, stride)
    narrow = synth.bf16_round if rung == "bf16_mfma" else (lambda v: v.astype(np.float16).astype(np.float32))

    def run(first, count):
        out = c.upload(init[first : first + count])
        c.launcher().launch(Kernel.matmul_q8_0_float, P.MatmulQuant(rows=count, n=n, k=k, col0=col0, out_stride=stride, accumulate=1, k_slice=k),
                            [c.upload(x[first : first + count]), wa, out], (K.div_ceil(n, 64), K.div_ceil(count, 16), 1))
        return c.read(out).reshape(count, stride)

    got = run(0, rows)  # three 128-token tiles on 45 column tiles: the tall tiling
    want = init[:, col0 : col0 + n] + narrow(x).astype(np.float64) @ narrow(wq).astype(np.float64).T
    assert rel_err(got[:, col0 : col0 + n], want) <= 1e-5
    mask = np.ones(stride, dtype=bool)
    mask[col0 : col0 + n] = False
    assert np.array_equal(got[:, mask].view(np.uint32), init[:, mask].view(np.uint32)), "columns outside the chunk were written"
    for first, count in ((0, 1), (1, 40), (41, 64), (105, 130), (235, 65)):  # 64-token tiles, and two tall tiles
        assert got[first : first + count].tobytes() == run(first, count).tobytes(), "token chunking changed bits"
    c.set.select_prefill(c.rec, K.Prefill.scalar_f32)


@pytest.mark.parametrize("k", [512, 2048])
@pytest.mark.parametrize("weights", ["q8_0", "bf16"])
def test_matmul_bf16_rungs_keep_token_bits_over_prompt_splits(ctx, weights, k):
    """The prefill kernels give the same result however a prompt is split into steps
    (src/sched/sched.zig:84-90): on this backend's bf16 rungs a matrix wide enough that a
    512-token step's 256 x 128 tiles would fill the CUs (n = 16400) keeps the tiling its short
    steps take, so 512 tokens in one step equal a first chunk of 64 and a step of 448 bit for
    bit; with k = 512 the matrix is one the streaming kernel takes, a pass per 128 tokens."""
    c = ctx
    rows, n = 512, 16400
    x = c.random(rows * k, 1).reshape(rows, k)
    if weights == "q8_0":
        raw, values = quant_rows(c, TensorType.q8_0, n, k)
        wa = c.gpu_weights(TensorType.q8_0, raw, k)
    else:
        bits, values = random_half(c, n * k, 1)
        wa = c.upload(bits.reshape(n, k))
    values = values.reshape(n, k)
    for rung in (K.Prefill.bf16_mfma, K.Prefill.bf16_mfma_xbf16):
        packed = rung == K.Prefill.bf16_mfma_xbf16
        c.set.select_prefill(c.rec, rung)

        def run(first, count):
            xa = c.upload(synth.to_bf16_bits(x[first : first + count]) if packed else x[first : first + count])
            out = c.output(count * n)
            if weights == "q8_0":
                c.launcher().launch(Kernel.matmul_q8_0_float, P.MatmulQuant(rows=count, n=n, k=k, col0=0, out_stride=n, k_slice=k), [xa, wa, out],
                                    (K.div_ceil(n, 64), K.div_ceil(count, 16), 1))
            else:
                c.launcher().launch(Kernel.matmul_bf16, P.MatmulBf16(rows=count, n=n, k=k, col0=0, out_stride=n), [xa, wa, out],
                                    (K.div_ceil(n, K.matmul_tile_n), K.div_ceil(count, K.matmul_tile_t), 1))
            return c.read(out).reshape(count, n)

        whole = run(0, rows)
        assert whole[:64].tobytes() == run(0, 64).tobytes(), (rung, "the first chunk of 64")
        assert whole[64:].tobytes() == run(64, 448).tobytes(), (rung, "the step of 448")
        assert whole[504:].tobytes() == run(504, 8).tobytes(), (rung, "a tail of 8")
        some = np.arange(0, rows, 37)
        want = synth.bf16_round(x[some]).astype(np.float64) @ synth.bf16_round(values).astype(np.float64).T
        assert rel_err(whole[some], want) <= 1e-5, rung
    c.set.select_prefill(c.rec, K.Prefill.scalar_f32)


@pytest.mark.parametrize("rows,n,k,col0,pad,accumulate,packed", [
    (128, 16400, 1024, 0, 0, False, True),    # whole token tiles, vector stores
    (70, 16389, 768, 5, 9, True, False),      # ragged last weight tile, unaligned output: scalar stores
    (17, 16400, 256, 4, 4, True, True),       # 64-token kernel, one chunk of k a wave
    (1, 20000, 512, 0, 0, False, False),
])
def test_matmul_bf16_streamed_chunk(ctx, rows, n, k, col0, pad, accumulate, packed):
    """A step against a tall bf16 matrix with k <= 1024 (the
    vocabulary projection of a prefill chunk) takes the kernel that streams the
    weights into registers: against the rung's operand contract, columns
    outside the chunk untouched, and every token's bits the same whether it runs
    in the chunk or alone."""
    c = ctx
    rung = K.Prefill.bf16_mfma_xbf16 if packed else K.Prefill.bf16_mfma
    x = c.random(rows * k, 1).reshape(rows, k)
    xs = synth.bf16_round(x).astype(np.float64)
    bits, values = random_half(c, n * k, 1)
    wa = c.upload(bits.reshape(n, k))
    stride = n + pad
    init = c.random(rows * stride, 0.5).reshape(rows, stride)
    c.set.select_prefill(c.rec, rung)

    def run(first, count):
        xa = c.upload(synth.to_bf16_bits(x[first : first + count]) if packed else x[first : first + count])
        out = c.upload(init[first : first + count])
        c.launcher().launch(Kernel.matmul_bf16, P.MatmulBf16(rows=count, n=n, k=k, col0=col0, out_stride=stride, accumulate=int(accumulate)), [xa, wa, out],
                            (K.div_ceil(n, K.matmul_tile_n), K.div_ceil(count, K.matmul_tile_t), 1))
        return c.read(out).reshape(count, stride)

    got = run(0, rows)
    want = xs @ values.reshape(n, k).astype(np.float64).T + (init[:, col0 : col0 + n] if accumulate else 0)
    assert rel_err(got[:, col0 : col0 + n], want) <= 1e-5
    assert np.array_equal(got[:, :col0], init[:, :col0]) and np.array_equal(got[:, col0 + n :], init[:, col0 + n :]), "columns outside the chunk were written"
    for first, count in ((0, 1), (rows // 2, 1), (rows - 1, 1), (rows // 3, min(20, rows - rows // 3))):
        assert run(first, count).tobytes() == got[first : first + count].tobytes(), "a token's bits depend on its chunk"
    c.set.select_prefill(c.rec, K.Prefill.scalar_f32)


@pytest.mark.parametrize("rows,n,k,col0,pad,accumulate,packed", [
    (128, 16400, 1024, 0, 0, False, True),
    (50, 16400, 512, 4, 4, True, False),
])
def test_matmul_q8_0_float_streamed_chunk(ctx, rows, n, k, col0, pad, accumulate, packed):
    """The same shape class with Q8_0 weights (matmul_q8_0_float on the bf16 rung):
    weights bf16(q * d), against the rung's operand contract; a token's bits the
    same in the chunk or alone."""
    c = ctx
    rung = K.Prefill.bf16_mfma_xbf16 if packed else K.Prefill.bf16_mfma
    x = c.random(rows * k, 1).reshape(rows, k)
    xs = synth.bf16_round(x).astype(np.float64)
    raw, wq = quant_rows(c, TensorType.q8_0, n, k)
    wa = c.gpu_weights(TensorType.q8_0, raw, k)
    stride = n + pad
    init = c.random(rows * stride, 0.5).reshape(rows, stride)
    c.set.select_prefill(c.rec, rung)

    def run(first, count):
        xa = c.upload(synth.to_bf16_bits(x[first : first + count]) if packed else x[first : first + count])
        out = c.upload(init[first : first + count])
        c.launcher().launch(Kernel.matmul_q8_0_float, P.MatmulQuant(rows=count, n=n, k=k, col0=col0, out_stride=stride, accumulate=int(accumulate), k_slice=k),
                            [xa, wa, out], (K.div_ceil(n, 64), K.div_ceil(count, 16), 1))
        return c.read(out).reshape(count, stride)

    got = run(0, rows)
    want = xs @ synth.bf16_round(wq).astype(np.float64).T + (init[:, col0 : col0 + n] if accumulate else 0)
    assert rel_err(got[:, col0 : col0 + n], want) <= 1e-5
    assert np.array_equal(got[:, :col0], init[:, :col0]) and np.array_equal(got[:, col0 + n :], init[:, col0 + n :]), "columns outside the chunk were written"
    for first, count in ((0, 1), (rows - 1, 1), (rows // 3, min(20, rows - rows // 3))):
        assert run(first, count).tobytes() == got[first : first + count].tobytes(), "a token's bits depend on its chunk"
    c.set.select_prefill(c.rec, K.Prefill.scalar_f32)


@pytest.mark.parametrize("weights", ["bf16", "f16", "q8_0"])
@pytest.mark.parametrize("rows,n,k,col0,pad,accumulate", [
    (19, 100, 1024, 0, 0, False),    # partial tiles in both dimensions
    (133, 150, 96, 3, 6, True),      # a step of 96 positions, accumulate, padded rows
    (300, 4100, 128, 0, 0, False),   # 128-token tiles
    (67, 70, 320, 0, 0, False),
])
def test_prefill_fp16_single_rung(ctx, weights, rows, n, k, col0, pad, accumulate):
    """The reference's fp16_single rung: activations rounded to f16, weights rounded
    to f16 (Q8_0: the f32 product d * q rounded once), fp32 accumulation
    (src/agility/kernels/matmul_q8_0_float_linalg_single.hlsl:36-58,
    src/agility/kernels/matmul_half_linalg.hlsl:34-52). Against that operand contract in
    float64; a token's bits the same in the step or alone."""
    c = ctx
    x = c.random(rows * k, 2).reshape(rows, k)
    x[0, :4] = [70000.0, -3e-6, 1.0009765625 + 2.0 ** -12, 65519.0]  # beyond the range, below the normals, a tie, the last value that rounds to a finite one
    if weights == "q8_0":
        raw, values = quant_rows(c, TensorType.q8_0, n, k)
        wa, kernel = c.gpu_weights(TensorType.q8_0, raw, k), Kernel.matmul_q8_0_float
        p = lambda count: P.MatmulQuant(rows=count, n=n, k=k, col0=col0, out_stride=n + pad, accumulate=int(accumulate), k_slice=k)
    else:
        bits, values = random_half(c, n * k, 1, weights)
        wa, kernel = c.upload(bits.reshape(n, k)), Kernel["matmul_" + weights]
        p = lambda count: P.MatmulBf16(rows=count, n=n, k=k, col0=col0, out_stride=n + pad, accumulate=int(accumulate))
    stride = n + pad
    init = c.random(rows * stride, 0.5).reshape(rows, stride)
    c.set.select_prefill(c.rec, K.Prefill.fp16_single)

    def run(first, count):
        out = c.upload(init[first : first + count])
        c.launcher().launch(kernel, p(count), [c.upload(x[first : first + count]), wa, out], (K.div_ceil(n, 64), K.div_ceil(count, 16), 1))
        return c.read(out).reshape(count, stride)

    got = run(0, rows)
    with np.errstate(over="ignore"):
        x16 = x.astype(np.float16)
    assert np.isinf(x16[0, 0]) and x16[0, 3] == 65504.0
    want = oracle.prefill_fp16_single(x, values.reshape(n, k)) + (init[:, col0 : col0 + n] if accumulate else 0)
    # Token 0 holds an infinity: its outputs are infinities or NaN, as the reference's are.
    assert not np.isfinite(got[0, col0 : col0 + n]).any()
    assert rel_err(got[1:, col0 : col0 + n], want[1:]) <= 1e-5
    assert np.array_equal(got[:, :col0], init[:, :col0]) and np.array_equal(got[:, col0 + n :], init[:, col0 + n :]), "columns outside the step were written"
    for first, count in ((1, 1), (rows - 1, 1), (rows // 3, min(20, rows - rows // 3))):
        assert run(first, count).tobytes() == got[first : first + count].tobytes(), "a token's bits depend on its step"
    c.set.select_prefill(c.rec, K.Prefill.scalar_f32)


@pytest.mark.parametrize("weights", ["bf16", "f16", "q8_0"])
@pytest.mark.parametrize("rows,n,k,col0,pad,accumulate", [
    (19, 100, 1024, 0, 0, False),
    (133, 150, 96, 3, 6, True),
    (300, 4100, 128, 0, 0, False),
    (67, 70, 320, 0, 0, False),
])
def test_prefill_fp16_compensated_rung(ctx, weights, rows, n, k, col0, pad, accumulate):
    """The reference's fp16_compensated rung: every activation as its f16 value plus
    the f16 of the remainder; Q8_0 weights as exact integers with the block scale
    applied to the block's sum, stored halves rounded to f16
    (src/agility/kernels/matmul_q8_0_float_linalg.hlsl:40-101,
    src/agility/kernels/matmul_half_linalg.hlsl:34-75). Against that operand contract
    in float64, and, because the activations keep about 22 bits, within 1e-5 of the
    product of the unrounded activations too (Q8_0; stored halves keep their f16 rounding)."""
    c = ctx
    x = c.random(rows * k, 2).reshape(rows, k)
    if weights == "q8_0":
        raw, values = quant_rows(c, TensorType.q8_0, n, k)
        wa, kernel = c.gpu_weights(TensorType.q8_0, raw, k), Kernel.matmul_q8_0_float
        p = lambda count: P.MatmulQuant(rows=count, n=n, k=k, col0=col0, out_stride=n + pad, accumulate=int(accumulate), k_slice=k)
        w_used = values.reshape(n, k).astype(np.float64)           # exact: integers times the block's scale
    else:
        bits, values = random_half(c, n * k, 1, weights)
        wa, kernel = c.upload(bits.reshape(n, k)), Kernel["matmul_" + weights]
        p = lambda count: P.MatmulBf16(rows=count, n=n, k=k, col0=col0, out_stride=n + pad, accumulate=int(accumulate))
        w_used = values.reshape(n, k).astype(np.float32).astype(np.float16).astype(np.float64)
    stride = n + pad
    init = c.random(rows * stride, 0.5).reshape(rows, stride)
    c.set.select_prefill(c.rec, K.Prefill.fp16_compensated)

    def run(first, count):
        out = c.upload(init[first : first + count])
        c.launcher().launch(kernel, p(count), [c.upload(x[first : first + count]), wa, out], (K.div_ceil(n, 64), K.div_ceil(count, 16), 1))
        return c.read(out).reshape(count, stride)

    got = run(0, rows)
    base = init[:, col0 : col0 + n] if accumulate else 0
    assert rel_err(got[:, col0 : col0 + n], oracle.prefill_fp16_compensated(x, values.reshape(n, k), exact_weights=weights == "q8_0") + base) <= 1e-5
    if weights == "q8_0":
        assert rel_err(got[:, col0 : col0 + n], x.astype(np.float64) @ w_used.T + base) <= 1e-5
    assert np.array_equal(got[:, :col0], init[:, :col0]) and np.array_equal(got[:, col0 + n :], init[:, col0 + n :]), "columns outside the step were written"
    for first, count in ((0, 1), (rows - 1, 1), (rows // 3, min(20, rows - rows // 3))):
        assert run(first, count).tobytes() == got[first : first + count].tobytes(), "a token's bits depend on its step"
    c.set.select_prefill(c.rec, K.Prefill.scalar_f32)


def launch_float_q8(c, x, weights, out, rows, accumulate, slices, chunked):
    """Two weight chunks exercise nonzero col0 and a padded output stride;
    split-k partials are dense per chunk (src/kernels/check.zig:752-770)."""
    l = c.launcher()
    for index, ((start, n), w) in enumerate(zip(((0, 70), (0, 27), (27, 43)), weights)):
        if (chunked == 0 and index != 0) or (chunked == 1 and index == 0):
            continue
        grid = (K.div_ceil(n, 64), K.div_ceil(rows, 16), slices)
        if slices == 1:
            l.launch(Kernel.matmul_q8_0_float, P.MatmulQuant(rows=rows, n=n, k=320, col0=3 + start, out_stride=79, accumulate=accumulate, k_slice=320), [x, w, out], grid)
        else:
            partial = c.output(slices * rows * n)
            l.launch(Kernel.matmul_q8_0_float, P.MatmulQuant(rows=rows, n=n, k=320, col0=0, out_stride=n, k_slice=160, slice_stride=rows * n), [x, w, partial], grid)
            l.launch(Kernel.matmul_reduce, P.MatmulReduce(rows=rows, n=n, slices=slices, col0=3 + start, out_stride=79, accumulate=accumulate, slice_stride=rows * n),
                     [partial, out], K.elementwise(rows * n))


@pytest.mark.parametrize("rung", [K.Prefill.scalar_f32, K.Prefill.fp16_single, K.Prefill.fp16_compensated, K.Prefill.bf16_mfma, K.Prefill.bf16_mfma_xbf16])
def test_matmul_q8_0_float(ctx, rung):
    """Unrounded float activations, k = 320, full and partial tiles, weight
    chunks, padding, accumulate and split-k; within each split-k path token
    chunking must stay bitwise identical (src/kernels/check.zig:772-825)."""
    c = ctx
    rows, n, k, stride = 67, 70, 320, 79
    x = c.random(rows * k, 1).reshape(rows, k)
    raw, values = quant_rows(c, TensorType.q8_0, n, k)
    rb = k // 32 * 34
    weights = [c.gpu_weights(TensorType.q8_0, raw, k), c.gpu_weights(TensorType.q8_0, raw[: 27 * rb], k), c.gpu_weights(TensorType.q8_0, raw[27 * rb :], k)]
    packed = rung == K.Prefill.bf16_mfma_xbf16
    xin = synth.to_bf16_bits(x) if packed else x
    xa = c.upload(xin)
    init = c.random(rows * stride, 0.25).reshape(rows, stride)
    c.set.select_prefill(c.rec, rung)
    prod = None
    if rung == K.Prefill.fp16_single:
        prod, tol = oracle.prefill_fp16_single(x, values), 1e-5
    elif rung == K.Prefill.fp16_compensated:
        prod, tol = oracle.prefill_fp16_compensated(x, values, exact_weights=True), 1e-5
    elif rung != K.Prefill.scalar_f32:
        # The rung's operand contract: both operands rounded to bf16.
        xs, ws, tol = synth.bf16_round(x), synth.bf16_round(values), 1e-5
    else:
        xs, ws, tol = x, values, 1e-5
    if prod is None:
        prod = xs.astype(np.float64) @ ws.astype(np.float64).T
    for accumulate in (0, 1):
        want = prod + (init[:, 3 : 3 + n] if accumulate else 0)
        for slices, chunked in ((1, 0), (1, 1), (2, 0), (2, 1)):
            out = c.upload(init)
            launch_float_q8(c, xa, weights, out, rows, accumulate, slices, chunked)
            got = c.read(out).reshape(rows, stride)
            assert rel_err(got[:, 3 : 3 + n], want) <= tol, (accumulate, slices, chunked)
            # Nothing outside the output columns is touched.
            mask = np.ones(stride, dtype=bool)
            mask[3 : 3 + n] = False
            assert np.array_equal(got[:, mask].view(np.uint32), init[:, mask].view(np.uint32))
            for first, count in ((0, 3), (3, 14), (17, 50)):
                chunk_out = c.upload(init[first : first + count])
                launch_float_q8(c, c.upload(xin[first : first + count]), weights, chunk_out, count, accumulate, slices, chunked)
                assert got[first : first + count].tobytes() == c.read(chunk_out).tobytes(), "token chunking changed bits"
    c.set.select_prefill(c.rec, K.Prefill.scalar_f32)


# ---- activations rounded to 8-bit blocks, and the int8 multiply: check.zig:500-594,839-871 ----

def quantize_x(c, t: TensorType, x, rows: int, k: int, mode: int = 0, eps: float = 0.0, nw=None):
    """quantize_q8 on an uploaded x: (qx words, dx), as src/kernels/check.zig:504-509."""
    block = K.act_block(t)
    qx, dx = c.output(rows * k // 4), c.output(rows * k // block)
    c.launcher().launch(Kernel.quantize_q8, P.QuantizeQ8(k=k, block=block, mode=mode, eps=eps), [x, qx, dx, nw if nw is not None else x],
                        (K.div_ceil(k, 256), rows, 1))
    return qx, dx


def read_q8(c, qx, dx, rows: int, k: int):
    return c.read_bytes(qx).view(np.int8)[: rows * k].reshape(rows, k), c.read(dx).reshape(rows, -1)


@pytest.mark.parametrize("t", [TensorType.q8_0, TensorType.q4_k])
def test_quantize_q8_value_for_value(ctx, t):
    """Random rows, a negative maximum, a +amax / -amax tie, a zero row and exact
    half-integers (src/kernels/check.zig:511-547); tolerance 0, and the integers
    and scales themselves must equal the oracle's."""
    c = ctx
    rows, k = 6, 512
    x = c.random(rows * k, 3).reshape(rows, k)
    x[2, 77] = -9.5
    x[3, 5] = -7.25
    x[3, 40] = 7.25
    x[4] = 0
    x[5] = (np.arange(k) % 32 - 16).astype(np.float32) + np.float32(0.5)
    x[5, ::32] = 127
    block = K.act_block(t)
    qx, dx = quantize_x(c, t, c.upload(x), rows, k)
    q, d = read_q8(c, qx, dx, rows, k)
    d = d[:, : k // block]
    wq, wd = oracle.quantize_q8(x, block)
    assert np.array_equal(q, wq)
    assert np.array_equal(d.view(np.uint32), wd.view(np.uint32))
    got = q.astype(np.float32) * np.repeat(d, block, axis=1)
    assert np.array_equal(got, oracle.round_like_llama(ORACLE_TYPE[t], x))


@pytest.mark.parametrize("t,k", [(TensorType.q8_0, 1056), (TensorType.q8_0, 2048), (TensorType.q8_0, 4096), (TensorType.q8_0, 14336),
                                 (TensorType.q4_k, 2048), (TensorType.q4_k, 4096), (TensorType.q4_k, 14336)])
def test_quantize_q8_long_rows(ctx, t, k):
    """Rows long enough that a wave takes two or four chunks of 256 values and a row several
    workgroups (k = 14336: 56 chunks), and for Q8_0 a row whose last chunk is ragged
    (k = 1056): integers and scales equal the oracle's, plain and behind the RMSNorm and
    SiLU-pair prologues; ties between equal magnitudes across lanes and chunks. A few rows
    (one chunk a wave) as well as many."""
    c = ctx
    block = K.act_block(t)
    rows = 130 if k > 4096 else 520  # (enough workgroups that a wave takes four chunks at once, or two)
    x = c.random(rows * k, 3).reshape(rows, k)
    x[1, k - 1] = -11.5      # a negative maximum in the last lane of the last chunk
    x[2, 300] = 8.75         # +amax / -amax ties in different lanes and chunks
    x[2, 301] = -8.75
    x[2, k - 7] = -8.75
    x[3] = 0
    wq, wd = oracle.quantize_q8(x, block)
    for count in (rows, 5):
        qx, dx = quantize_x(c, t, c.upload(x[:count]), count, k)
        q, d = read_q8(c, qx, dx, count, k)
        assert np.array_equal(q, wq[:count])
        assert np.array_equal(d[:, : k // block].view(np.uint32), wd[:count].view(np.uint32))
    if block == 256:
        eps, nw = 1e-6, c.random(k, 1)
        qx, dx = quantize_x(c, t, c.upload(x), rows, k, mode=1, eps=eps, nw=c.upload(nw))
        q, d = read_q8(c, qx, dx, rows, k)
        wq, wd = oracle.quantize_q8(x, 256, mode=1, eps=eps, nw=nw)
        assert np.array_equal(q, wq) and np.array_equal(d[:, : k // 256].view(np.uint32), wd.view(np.uint32))
        pair = c.random(rows * 2 * k, 2).reshape(rows, 2 * k)
        qx, dx = quantize_x(c, t, c.upload(pair), rows, k, mode=2)
        q, d = read_q8(c, qx, dx, rows, k)
        d = d[:, : k // 256]
        g = pair[:, :k].astype(np.float64)
        want = g * sigmoid64(g) * pair[:, k:]
        step = np.repeat(np.abs(d), 256, axis=1).astype(np.float64)
        assert np.max(np.abs(q.astype(np.float64) * np.repeat(d, 256, axis=1) - want) / (step / 2)) <= 1.0001


def _llama_kats():
    import json
    import os

    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "round_like_llama_kat.json")) as f:
        return json.load(f)["cases"]


@pytest.mark.parametrize("case", _llama_kats(), ids=lambda c: c["name"])
def test_quantize_q8_reference_kats(ctx, case):
    """The reference's own known answers for its activation rounding
    (src/ref/matmul.zig:382-419) through the quantize_q8 kernel: integer times
    scale must be the expected value (ties to even under both block sizes,
    127 / amax before rounding, IQ4_XS weights take 256-wide blocks)."""
    c = ctx
    types = {"q8_0": TensorType.q8_0, "q4_k": TensorType.q4_k, "q6_k": TensorType.q6_k, "iq4_xs": TensorType.iq4_xs}
    x = np.array(case["input"], dtype=np.uint32).view(np.float32)
    block = K.act_block(types[case["type"]])
    k = (x.size + 255) // 256 * 256  # the kernel rounds 256 values a wave; blocks of zeros follow
    xp = np.zeros(k, dtype=np.float32)
    xp[: x.size] = x
    qx, dx = quantize_x(c, types[case["type"]], c.upload(xp), 1, k)
    q, d = read_q8(c, qx, dx, 1, k)
    got = (q.astype(np.float32) * np.repeat(d[:, : k // block], block, axis=1))[0, : x.size]
    if "expect" in case:
        first, want = case["expect"]["first"], np.array(case["expect"]["bits"], dtype=np.uint32)
        part = got[first : first + want.size]
        if case["expect"]["compare"] == "bits":
            assert np.array_equal(part.view(np.uint32), want)
        else:
            assert np.array_equal(part, want.view(np.float32))
    if "same_as_type" in case:
        assert K.act_block(types[case["same_as_type"]]) == block
        assert not np.array_equal(got, x)
        assert np.array_equal(got.view(np.uint32), oracle.round_like_llama(ORACLE_TYPE[types[case["same_as_type"]]], x[None])[0].view(np.uint32))


@pytest.mark.parametrize("mode", [1, 2])
def test_quantize_q8_fused(ctx, mode):
    """quantize_q8 computing its input first (RMSNorm, SiLU pair): every value
    within half a step of the float64 result, tolerance 1.0001 half-steps
    (src/kernels/check.zig:549-586)."""
    c = ctx
    rows, k, eps = 5, 768, 1e-6
    width = 2 * k if mode == 2 else k
    x = c.random(rows * width, 2).reshape(rows, width)
    nw = c.random(k, 1)
    qx, dx = quantize_x(c, TensorType.q4_k, c.upload(x), rows, k, mode=mode, eps=eps, nw=c.upload(nw))
    q, d = read_q8(c, qx, dx, rows, k)
    d = d[:, : k // 256]
    if mode == 1:
        want = np.stack([norm_row(r, nw, eps) for r in x])
    else:
        g = x[:, :k].astype(np.float64)
        want = g * sigmoid64(g) * x[:, k:]
    step = np.repeat(np.abs(d), 256, axis=1).astype(np.float64)
    got = q.astype(np.float64) * np.repeat(d, 256, axis=1)
    assert np.max(np.abs(got - want) / (step / 2)) <= 1.0001
    if mode == 1:
        # The normalisation follows ggml's arithmetic step for step, so the
        # integers equal the oracle's.
        wq, wd = oracle.quantize_q8(x, 256, mode=1, eps=eps, nw=nw)
        assert np.array_equal(q, wq) and np.array_equal(d.view(np.uint32), wd.view(np.uint32))


def launch_int8(c, t, act, wa, out, rows, n, k, accumulate, slices, col0=0, stride=None):
    l = c.launcher()
    stride = stride or n
    kernel = K.weight_kernel("matmul", t)
    grid = (K.div_ceil(n, K.matmul_quant_tile_n), K.div_ceil(rows, K.matmul_quant_tile_t), 1)
    qx, dx = act
    if slices is None:
        l.launch(kernel, P.MatmulQuant(rows=rows, n=n, k=k, col0=col0, out_stride=stride, accumulate=accumulate, k_slice=k), [qx, wa, out, dx], grid)
        return
    count, k_slice = slices
    partials = c.output(count * rows * n)
    l.launch(kernel, P.MatmulQuant(rows=rows, n=n, k=k, col0=0, out_stride=n, k_slice=k_slice, slice_stride=rows * n), [qx, wa, partials, dx], (grid[0], grid[1], count))
    l.launch(Kernel.matmul_reduce, P.MatmulReduce(rows=rows, n=n, slices=count, col0=col0, out_stride=stride, accumulate=accumulate, slice_stride=rows * n),
             [partials, out], K.elementwise(rows * n))


@pytest.mark.parametrize("t", [TensorType.q8_0, TensorType.q4_k, TensorType.q5_k, TensorType.q6_k, TensorType.q3_k])
def test_matmul_int8_whole_and_split(ctx, t):
    """The prefill multiply on quantize_q8's output, accumulating, over more than
    one tile each way: whole, and split over k into partials that matmul_reduce
    adds up; against float64 over the rounded activations, tolerance 1e-5
    (src/kernels/check.zig:839-871). The integer unit sums make the result equal
    the oracle's unit formula far more tightly, and token chunks keep their bits."""
    c = ctx
    rows, n, k = 70, 150, 1024
    s = K.matmul_slices(n, k)
    assert s.count > 1
    x = c.random(rows * k, 1).reshape(rows, k)
    xs = oracle.round_like_llama(ORACLE_TYPE[t], x)
    act = quantize_x(c, t, c.upload(x), rows, k)
    raw, values = quant_rows(c, t, n, k)
    wa = c.gpu_weights(t, raw, k)
    init = c.random(rows * n, 4).reshape(rows, n)
    want = init + xs.astype(np.float64) @ values.astype(np.float64).T
    whole, split, odd = c.upload(init), c.upload(init), c.upload(init)
    launch_int8(c, t, act, wa, whole, rows, n, k, 1, None)
    launch_int8(c, t, act, wa, split, rows, n, k, 1, (s.count, s.k_slice))
    # Slices that cut a 256-weight block and leave a short last one.
    launch_int8(c, t, act, wa, odd, rows, n, k, 1, (3, 352))
    for out in (whole, split, odd):
        assert rel_err(c.read(out).reshape(rows, n), want) <= 1e-5
    # The first slice alone (one slice in the grid) stops inside a 256-weight block.
    alone = c.upload(init)
    c.launcher().launch(K.weight_kernel("matmul", t), P.MatmulQuant(rows=rows, n=n, k=k, col0=0, out_stride=n, accumulate=1, k_slice=352),
                        [act[0], wa, alone, act[1]], (K.div_ceil(n, K.matmul_quant_tile_n), K.div_ceil(rows, K.matmul_quant_tile_t), 1))
    want_alone = init + xs[:, :352].astype(np.float64) @ values[:, :352].astype(np.float64).T
    assert rel_err(c.read(alone).reshape(rows, n), want_alone) <= 1e-5
    block = K.act_block(t)
    q, d = oracle.quantize_q8(x, block)
    formula = init + oracle.matmul_q8(ORACLE_TYPE[t], raw, q, d, n)
    assert rel_err(c.read(whole).reshape(rows, n), formula) <= 2e-6
    got = c.read(whole).reshape(rows, n)
    for first, count in ((0, 3), (3, 30), (33, 37)):
        chunk = c.upload(init[first : first + count])
        launch_int8(c, t, quantize_x(c, t, c.upload(x[first : first + count]), count, k), wa, chunk, count, n, k, 1, None)
        assert got[first : first + count].tobytes() == c.read(chunk).tobytes(), "token chunking changed bits"


@pytest.mark.parametrize("t,rows,n,k", [
    (TensorType.q8_0, 67, 70, 320),    # k not a multiple of the 128-deep step
    (TensorType.q8_0, 130, 200, 4096),
    (TensorType.q4_k, 1, 129, 2048),
    (TensorType.q4_k, 257, 64, 1536),
    (TensorType.q5_k, 65, 129, 768),
    (TensorType.q6_k, 129, 65, 1280),
    (TensorType.q3_k, 3, 200, 512),
])
def test_matmul_int8_shapes(ctx, t, rows, n, k):
    """Partial tiles each way, a padded output stride and a nonzero first column;
    nothing outside the output columns is touched."""
    c = ctx
    x = c.random(rows * k, 1).reshape(rows, k)
    xs = oracle.round_like_llama(ORACLE_TYPE[t], x)
    act = quantize_x(c, t, c.upload(x), rows, k)
    raw, values = quant_rows(c, t, n, k)
    wa = c.gpu_weights(t, raw, k)
    stride, col0 = n + 9, 5
    init = c.random(rows * stride, 0.25).reshape(rows, stride)
    out = c.upload(init)
    launch_int8(c, t, act, wa, out, rows, n, k, 0, None, col0=col0, stride=stride)
    got = c.read(out).reshape(rows, stride)
    want = xs.astype(np.float64) @ values.astype(np.float64).T
    assert rel_err(got[:, col0 : col0 + n], want) <= 1e-5
    mask = np.ones(stride, dtype=bool)
    mask[col0 : col0 + n] = False
    assert np.array_equal(got[:, mask].view(np.uint32), init[:, mask].view(np.uint32))


@pytest.mark.parametrize("t,k", [(TensorType.q4_k, 1024), (TensorType.q5_k, 768), (TensorType.q6_k, 2560), (TensorType.q3_k, 512)])
def test_matmul_kquant_int8_long_and_short_steps_keep_token_bits(ctx, t, k):
    """The K formats' whole-k int8 multiply takes one kernel for long steps (a wave walks all of
    k, part after part) and another for short ones (a tile's k in four parts, a wave each, met in
    LDS): 512 tokens x 4096 outputs are 1024 tiles and a long step, chunks of 128 tokens and
    fewer short ones; k of 2, 3, 4 and 10 blocks (parts of no, one or several blocks). The same
    bits either way, and 1e-5 against float64 over the rounded activations
    (src/kernels/check.zig:839-871)."""
    c = ctx
    rows, n, col0, stride = 512, 4096, 4, 4104
    x = c.random(rows * k, 1).reshape(rows, k)
    xs = oracle.round_like_llama(ORACLE_TYPE[t], x)
    raw, values = quant_rows(c, t, n, k)
    wa = c.gpu_weights(t, raw, k)
    init = c.random(rows * stride, 0.5).reshape(rows, stride)

    def run(first, count):
        out = c.upload(init[first : first + count])
        launch_int8(c, t, quantize_x(c, t, c.upload(x[first : first + count]), count, k), wa, out, count, n, k, 1, None, col0=col0, stride=stride)
        return c.read(out).reshape(count, stride)

    got = run(0, rows)
    want = init[:, col0 : col0 + n] + xs.astype(np.float64) @ values.astype(np.float64).T
    assert rel_err(got[:, col0 : col0 + n], want) <= 1e-5
    mask = np.ones(stride, dtype=bool)
    mask[col0 : col0 + n] = False
    assert np.array_equal(got[:, mask].view(np.uint32), init[:, mask].view(np.uint32)), "columns outside the chunk were written"
    for first, count in ((0, 1), (1, 63), (64, 128), (192, 33), (225, 287)):
        assert got[first : first + count].tobytes() == run(first, count).tobytes(), "token chunking changed bits"


def test_matmul_q8_0_int8_whole_steps_keep_token_bits(ctx):
    """matmul_q8_0 with k a multiple of 128, unsliced, takes the kernel whose scale products
    run on the matrix cores, in 128- or 64-token tiles: a token's sums are the same bits
    whichever tile height its step runs in and whichever tokens share the step; ragged
    rows and outputs, a column offset and a padded stride; against float64 over the
    rounded activations, 1e-5 (src/kernels/check.zig:839-871), and the unit formula."""
    c = ctx
    t = TensorType.q8_0
    rows, n, k, col0, stride = 300, 2830, 640, 3, 2840
    x = c.random(rows * k, 1).reshape(rows, k)
    xs = oracle.round_like_llama(ORACLE_TYPE[t], x)
    raw, values = quant_rows(c, t, n, k)
    wa = c.gpu_weights(t, raw, k)
    init = c.random(rows * stride, 0.5).reshape(rows, stride)

    def run(first, count):
        out = c.upload(init[first : first + count])
        launch_int8(c, t, quantize_x(c, t, c.upload(x[first : first + count]), count, k), wa, out, count, n, k, 1, None, col0=col0, stride=stride)
        return c.read(out).reshape(count, stride)

    got = run(0, rows)  # three 128-token tiles on 45 column tiles: the tall tiling
    want = init[:, col0 : col0 + n] + xs.astype(np.float64) @ values.astype(np.float64).T
    assert rel_err(got[:, col0 : col0 + n], want) <= 1e-5
    q, d = oracle.quantize_q8(x, 32)
    formula = init[:, col0 : col0 + n] + oracle.matmul_q8(ORACLE_TYPE[t], raw, q, d, n)
    assert rel_err(got[:, col0 : col0 + n], formula) <= 2e-6
    mask = np.ones(stride, dtype=bool)
    mask[col0 : col0 + n] = False
    assert np.array_equal(got[:, mask].view(np.uint32), init[:, mask].view(np.uint32)), "columns outside the chunk were written"
    for first, count in ((0, 1), (1, 40), (41, 64), (105, 130), (235, 65)):  # 64-token tiles, and two tall tiles
        assert got[first : first + count].tobytes() == run(first, count).tobytes(), "token chunking changed bits"


def test_silu_mul(ctx):
    c = ctx
    rows, width = 7, 10_001
    n = rows * width
    gu = c.random(2 * n, 6).reshape(rows, 2 * width)
    act = c.output(n)
    c.launcher().launch(Kernel.silu_mul, P.SiluMul(n, width), [c.upload(gu), act], K.elementwise(n))
    g = gu[:, :width].astype(np.float64)
    assert rel_err(c.read(act), g * sigmoid64(g) * gu[:, width:]) <= 1e-6
