"""Parity at the shapes the path is measured on, against the CPU oracle's
multiply (oracle.matmul: the reference's src/ref panel multiply restated in C)
and against float64, on the same seeded inputs.

Bars, as the acceptance criteria state them: every output within
1e-3 * (||row||2 * ||x||2) of the exact product after fp32 accumulation, the
reference's own tighter max|err| / max|want| <= 1e-5 for the f32 paths, and
argmax of each lm_head row equal to the oracle's. The prefill multiply on
bf16 MFMA is checked against its operand contract (both operands rounded to
bf16) at 1e-5 and against the unrounded product at the 1e-3 bound.
"""
import numpy as np
import pytest

import oracle
from gpucheck import bound_err, rel_err
from zllm_amd import kernels as K
from zllm_amd import synth
from zllm_amd.kernels import Kernel, TensorType, params as P

pytestmark = pytest.mark.gpu


def decode_matvec(c, t, raw, n, k, x, pair=False, m=None, variant=None, norm_w=None, eps=0.0):
    m = x.shape[0] if m is None else m
    wa = c.gpu_weights(t, raw, k)
    out = c.output(m * n)
    kernel = K.weight_kernel("matvec", t)
    v = variant or K.MatvecVariant()
    rows_per_group = K.matvec_rows if K.is_half(t) else v.group_rows()
    p = P.MatvecBf16(n=n, k=k, col0=0, out_stride=n, eps=eps, norm=norm_w is not None, silu_pair=pair, half=n if pair else 0)
    grid = (K.div_ceil(n, rows_per_group), m, 1)
    na = c.upload(norm_w) if norm_w is not None else wa
    if variant is None:
        c.launcher().launch(kernel, p, [c.upload(x), wa, out, na], grid)
    else:
        c.launcher().launch_pipeline(c.set.matvec(c.rec, kernel, variant), p, [c.upload(x), wa, out, na], grid)
    return c.read(out)[: m * n].reshape(m, n)


def test_c1_q8_0_matvec(ctx):
    """Q8_0 matvec, M=1, K=1024, N=3072."""
    n, k = 3072, 1024
    g = synth.rng(0xC1)
    raw, x = synth.q8_0_rows(g, n, k), synth.activations(g, 1, k)
    got = decode_matvec(ctx, TensorType.q8_0, raw, n, k, x)
    m = oracle.Matrix(oracle.Q8_0, raw, n, k)
    w = m.rows()
    want = oracle.matmul_f64(x, w)
    assert bound_err(got, want, w, x) <= 1e-3
    assert rel_err(got, want) <= 1e-5
    assert rel_err(got, oracle.matmul(x, m)) <= 1e-5  # the oracle's own f32 order of sums


def test_c2_q4_k_matvec(ctx):
    """Q4_K matvec, M=1, K=4096, N=14336."""
    n, k = 14336, 4096
    g = synth.rng(0xC2)
    raw, x = synth.q4_k_rows(g, n, k), synth.activations(g, 1, k)
    got = decode_matvec(ctx, TensorType.q4_k, raw, n, k, x)
    m = oracle.Matrix(oracle.Q4_K, raw, n, k)
    w = m.rows()
    want = oracle.matmul_f64(x, w)
    assert bound_err(got, want, w, x) <= 1e-3
    assert rel_err(got, want) <= 1e-5
    assert rel_err(got, oracle.matmul(x, m, oracle.default_threads())) <= 1e-5


@pytest.mark.parametrize("m", [1, 4, 8])
def test_c3_fused_gate_up_silu(ctx, m):
    """Fused gate+up Q4_K matvec with the SiLU(gate)*up epilogue, K=4096,
    N=2x14336, at the speculative-verify widths."""
    n, k = 14336, 4096
    raw = np.concatenate([synth.q4_k_rows(synth.rng(0xC3A), n, k), synth.q4_k_rows(synth.rng(0xC3B), n, k)])
    x = synth.activations(synth.rng(0xC30 + m), m, k)
    got = decode_matvec(ctx, TensorType.q4_k, raw, n, k, x, pair=True)
    mat = oracle.Matrix(oracle.Q4_K, raw, 2 * n, k)
    threads = oracle.default_threads()
    want32 = oracle.gate_up_silu(x, mat, n, threads)  # src/ref/dense.zig:179-195 composition
    assert rel_err(got, want32) <= 1e-5
    both = oracle.matmul_f64(x, mat.rows())
    gate, up = both[:, :n], both[:, n:]
    with np.errstate(over="ignore"):
        want = gate / (1 + np.exp(-gate)) * up
    assert rel_err(got, want) <= 1e-5
    # Every row bitwise equal to its own one-token launch (the split invariant).
    if m > 1:
        for t in (0, m - 1):
            assert got[t].tobytes() == decode_matvec(ctx, TensorType.q4_k, raw, n, k, x[t : t + 1], pair=True)[0].tobytes()


@pytest.mark.parametrize("norm", [False, True])
@pytest.mark.parametrize("m", [4, 8])
def test_c3_fused_gate_up_silu_matrix_core_variant(ctx, m, norm):
    """The same step on the matrix-core variant (MatvecVariant wg 512, lanes 64,
    rows 16): within 1e-5 of float64 row by row, every row bitwise equal to its
    own one-token launch on the same variant; with and without the RMSNorm
    prologue the planner's FFN launch carries (src/plan/qwen35.zig:1048)."""
    n, k, eps = 14336, 4096, 1e-6
    variant = K.MatvecVariant(wg=512, lanes=64, rows=16)
    raw = np.concatenate([synth.q4_k_rows(synth.rng(0xC3A), n, k), synth.q4_k_rows(synth.rng(0xC3B), n, k)])
    x = synth.activations(synth.rng(0xC30 + m), m, k)
    nw = synth.activations(synth.rng(0xC3F), 1, k).reshape(-1) if norm else None
    got = decode_matvec(ctx, TensorType.q4_k, raw, n, k, x, pair=True, variant=variant, norm_w=nw, eps=eps)
    xin = x.astype(np.float64)
    if norm:
        xin = xin / np.sqrt(np.mean(xin * xin, axis=1, keepdims=True) + eps) * nw.astype(np.float64)
    both = xin @ oracle.Matrix(oracle.Q4_K, raw, 2 * n, k).rows().astype(np.float64).T
    gate, up = both[:, :n], both[:, n:]
    with np.errstate(over="ignore"):
        want = gate / (1 + np.exp(-gate)) * up
    for t in range(m):
        assert rel_err(got[t], want[t]) <= 1e-5, t
    for t in (0, m - 1):
        assert got[t].tobytes() == decode_matvec(ctx, TensorType.q4_k, raw, n, k, x[t : t + 1], pair=True, variant=variant, norm_w=nw, eps=eps)[0].tobytes()


@pytest.mark.parametrize("rung", [K.Prefill.bf16_mfma, K.Prefill.bf16_mfma_xbf16, K.Prefill.scalar_f32])
def test_c4_q8_0_prefill_matmul(ctx, rung):
    """Prefill dequant-matmul, M=512, K=4096, N=4096, bf16 activations."""
    c = ctx
    rows, k, n = 512, 4096, 4096
    g = synth.rng(0xC4)
    raw = synth.q8_0_rows(g, n, k)
    x = synth.activations(g, rows, k, bf16=True)
    wa = c.gpu_weights(TensorType.q8_0, raw, k)
    out = c.output(rows * n)
    c.set.select_prefill(c.rec, rung)
    xa = c.upload(synth.to_bf16_bits(x) if rung == K.Prefill.bf16_mfma_xbf16 else x)
    c.launcher().launch(Kernel.matmul_q8_0_float, P.MatmulQuant(rows=rows, n=n, k=k, col0=0, out_stride=n, k_slice=k), [xa, wa, out],
                        (K.div_ceil(n, 64), K.div_ceil(rows, 16), 1))
    got = c.read(out).reshape(rows, n)
    c.set.select_prefill(c.rec, K.Prefill.scalar_f32)
    w = oracle.dequantize(oracle.Q8_0, raw, n * k).reshape(n, k)
    want = x.astype(np.float64) @ w.astype(np.float64).T
    assert bound_err(got, want, w, x) <= 1e-3
    if rung == K.Prefill.scalar_f32:
        assert rel_err(got, want) <= 1e-5
    else:
        contract = x.astype(np.float64) @ synth.bf16_round(w).astype(np.float64).T  # x is already bf16
        assert rel_err(got, contract) <= 1e-5


def test_c5_lm_head_decode(ctx):
    """bf16 lm_head, K=1024, N=151936, M=1: logits and their argmax."""
    n, k = 151936, 1024
    g = synth.rng(0xC5)
    wbits = synth.bf16_matrix(g, n, k, 0.02)
    x = synth.activations(g, 1, k, bf16=True)
    got = decode_matvec(ctx, TensorType.bf16, wbits, n, k, x)
    w = synth.bf16_bits_to_f32(wbits)
    want = oracle.matmul_f64(x, w)
    assert bound_err(got, want, w, x) <= 1e-3
    assert rel_err(got, want) <= 1e-5
    ref = oracle.matmul(x, oracle.Matrix(oracle.BF16, wbits, n, k, oracle.default_threads()), oracle.default_threads())
    assert int(np.argmax(got[0])) == oracle.argmax(ref[0])


@pytest.mark.parametrize("norm", [False, True])
@pytest.mark.parametrize("wide", [False, True])
def test_c5_lm_head_verify_width(ctx, ctx_wide, wide, norm):
    """bf16 lm_head, K=1024, N=151936, M=8 (a speculative verify step through the decode multiply,
    plain and with the final RMSNorm fused in; the general kernel, and in a context opened with
    ZHIP_OPTION_WIDE_DECODE the kernel that reads the weights once): logits and every row's argmax."""
    ctx = ctx_wide if wide else ctx
    n, k, m, eps = 151936, 1024, 8, 1e-6
    g = synth.rng(0xC5)
    wbits = synth.bf16_matrix(g, n, k, 0.02)
    x = synth.activations(g, m, k, bf16=not norm)
    nw = (1.0 + 0.1 * g.standard_normal(k)).astype(np.float32) if norm else None
    got = decode_matvec(ctx, TensorType.bf16, wbits, n, k, x, norm_w=nw, eps=eps)
    w = synth.bf16_bits_to_f32(wbits)
    xin = x
    if norm:
        x64 = x.astype(np.float64)
        xin = (x64 / np.sqrt(np.mean(x64 * x64, axis=1, keepdims=True) + eps) * nw.astype(np.float64)).astype(np.float32)
    want = oracle.matmul_f64(xin, w) if not norm else xin.astype(np.float64) @ w.astype(np.float64).T
    assert bound_err(got, want, w, xin) <= 1e-3
    assert rel_err(got, want) <= 1e-5
    if not norm:
        ref = oracle.matmul(x, oracle.Matrix(oracle.BF16, wbits, n, k, oracle.default_threads()), oracle.default_threads())
        assert np.array_equal(np.argmax(got, axis=1), np.array([oracle.argmax(r) for r in ref]))


@pytest.mark.parametrize("rung", [K.Prefill.bf16_mfma_xbf16, K.Prefill.scalar_f32])
def test_c5_lm_head_prefill(ctx, rung):
    """bf16 lm_head, K=1024, N=151936, M=128: argmax of every row."""
    c = ctx
    n, k, rows = 151936, 1024, 128
    g = synth.rng(0xC5)
    wbits = synth.bf16_matrix(g, n, k, 0.02)
    x = synth.activations(g, rows, k, bf16=True)
    out = c.output(rows * n)
    c.set.select_prefill(c.rec, rung)
    xa = c.upload(synth.to_bf16_bits(x) if rung == K.Prefill.bf16_mfma_xbf16 else x)
    c.launcher().launch(Kernel.matmul_bf16, P.MatmulBf16(rows=rows, n=n, k=k, col0=0, out_stride=n), [xa, c.upload(wbits), out],
                        (K.div_ceil(n, 64), K.div_ceil(rows, 16), 1))
    got = c.read(out).reshape(rows, n)
    c.set.select_prefill(c.rec, K.Prefill.scalar_f32)
    w = synth.bf16_bits_to_f32(wbits)
    want = oracle.matmul_f64(x, w)
    assert rel_err(got, want) <= 1e-5  # both operands are bf16 already: the rung is exact to f32 accumulation
    ref = oracle.matmul(x, oracle.Matrix(oracle.BF16, wbits, n, k, oracle.default_threads()), oracle.default_threads())
    assert np.array_equal(np.argmax(got, axis=1), np.array([oracle.argmax(r) for r in ref]))
