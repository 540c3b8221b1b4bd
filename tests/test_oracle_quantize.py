"""Pins the oracle's activation rounding (quantize_q8) and int8 multiply.

The reference rounds activations as llama.cpp's x86 CPU backend does
(src/ref/matmul.zig:197-247) and checks its kernel on a handful of built cases
(src/kernels/check.zig:516-547). Those cases are worked by hand here, and the
rest is pinned by a numpy restatement that shares no code with the oracle: it
rounds with rint instead of the magic-number addition, finds the leading value
with argmax, and converts the scale with numpy's float16.
"""
import numpy as np
import pytest

import oracle
from zllm_amd import synth


def test_f16_round_matches_numpy_float16():
    # Every f16 exponent (and the subnormal range) with mantissas at, just below
    # and just above the halfway points, plus random values.
    rng = np.random.default_rng(5)
    exps = np.arange(-26, 16)
    fracs = np.array([0, 1, 0x0fff, 0x1000, 0x1001, 0x2fff, 0x3000, 0x3001, 0x7fefff, 0x7ff000, 0x7ff001, 0x7fffff], dtype=np.uint32)
    bits = ((exps[:, None] + 127).astype(np.uint32) << 23) | fracs[None, :]
    values = np.concatenate([bits.reshape(-1).view(np.float32), rng.random(5000, dtype=np.float32) * np.float32(3.0), np.float32([0.0])])
    values = values[values < 65504.0]
    want = values.astype(np.float16).astype(np.float32)
    got = np.array([oracle.f16_round(float(v)) for v in values], dtype=np.float32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def numpy_quantize(x: np.ndarray, block: int):
    """x (rows, k) -> (q, d) by the published rule, vectorised."""
    x = np.asarray(x, dtype=np.float32)
    rows, k = x.shape
    b = x.reshape(rows, k // block, block)
    mag = np.abs(b)
    first = np.argmax(mag, axis=2)  # first of the largest
    lead = np.take_along_axis(b, first[..., None], axis=2)[..., 0]
    amax = np.abs(lead)
    with np.errstate(divide="ignore", invalid="ignore"):
        if block == 32:
            d = (amax / np.float32(127)).astype(np.float16).astype(np.float32)
            inv = np.where(amax != 0, np.float32(127) / amax, np.float32(0)).astype(np.float32)
            q = np.rint(b * inv[..., None])
        else:
            iscale = (np.float32(-127) / lead).astype(np.float32)
            d = np.where(amax != 0, np.float32(1) / iscale, np.float32(0)).astype(np.float32)
            q = np.minimum(np.rint(iscale[..., None] * b), 127)
            q = np.where(amax[..., None] != 0, q, 0)
    return q.reshape(rows, k).astype(np.int8), d.astype(np.float32)


def check_rows(k: int = 512) -> np.ndarray:
    """The rows the reference's check builds (src/kernels/check.zig:521-535)."""
    rng = np.random.default_rng(17)
    x = ((rng.random((6, k), dtype=np.float32) * 2 - 1) * np.float32(3)).astype(np.float32)
    x[2, 77] = -9.5
    x[3, 5] = -7.25
    x[3, 40] = 7.25
    x[4] = 0
    x[5] = (np.arange(k) % 32 - 16).astype(np.float32) + np.float32(0.5)
    x[5, ::32] = 127
    return x


@pytest.mark.parametrize("block", [32, 256])
def test_quantize_hand_worked_cases(block):
    x = check_rows()
    q, d = oracle.quantize_q8(x, block)
    # A negative maximum: the value of largest magnitude maps to -127 whatever its sign.
    assert q[2, 77] == -127
    blk = 77 // block
    assert d[2, blk] > 0
    if block == 256:
        assert d[2, blk] == np.float32(1) / (np.float32(-127) / np.float32(-9.5))
    else:
        assert d[2, blk] == np.float32(np.float16(np.float32(9.5) / np.float32(127)))
    # +amax and -amax tie: the first one leads; both ends stay within [-127, 127].
    assert q[3, 5] == -127 and q[3, 40] == 127
    # A zero row: zero integers, zero scales.
    assert not q[4].any() and not d[4].any()
    # Exact half-integers under a scale of exactly one: ties go to even.
    halves = (np.arange(512) % 32 - 16).astype(np.float64) + 0.5
    if block == 32:
        assert np.all(d[5] == 1.0)
        want = np.rint(halves)
        want[::32] = 127
    else:
        assert np.all(d[5] == -1.0)
        want = np.rint(-halves)
        want[::32] = -127
    assert np.array_equal(q[5].astype(np.float64), want)
    # -14.5, 0.5 and 1.5 each sit between an odd and an even integer: the even one wins.
    if block == 32:
        assert (q[5, 1], q[5, 16 + 0], q[5, 17]) == (-14, 0, 2)
    else:
        assert (q[5, 1], q[5, 16 + 0], q[5, 17]) == (14, 0, -2)


@pytest.mark.parametrize("block", [32, 256])
def test_quantize_matches_numpy_restatement(block):
    rng = np.random.default_rng(23)
    x = ((rng.random((40, 1024), dtype=np.float32) * 2 - 1) * np.float32(5)).astype(np.float32)
    x[:6, :512] = check_rows()
    x[7] *= np.float32(1e-6)   # tiny values: subnormal f16 scales for block 32
    x[8] *= np.float32(300.0)
    x[9, 100:400] = 0
    q, d = oracle.quantize_q8(x, block)
    wq, wd = numpy_quantize(x, block)
    assert np.array_equal(d.view(np.uint32), wd.view(np.uint32))
    assert np.array_equal(q, wq)


@pytest.mark.parametrize("t,block", [(oracle.Q8_0, 32), (oracle.Q4_K, 256), (oracle.Q6_K, 256)])
def test_round_like_llama_is_q_times_d(t, block):
    x = check_rows()
    q, d = numpy_quantize(x, block)
    want = q.astype(np.float32) * np.repeat(d, block, axis=1)
    got = oracle.round_like_llama(t, x)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # Rounding is within half a step of the input, plus what rounding the scale
    # itself to f16 moves the largest values by (Q8_0: 127 steps * 2^-11).
    step = np.repeat(np.abs(d), block, axis=1).astype(np.float64)
    slack = 127.0 / 2048.0 if block == 32 else 1e-4
    assert np.all(np.abs(got.astype(np.float64) - x) <= (0.5 + slack) * step + 1e-30)


def test_round_like_llama_half_types():
    rng = np.random.default_rng(3)
    x = ((rng.random(4096, dtype=np.float32) * 2 - 1) * np.float32(8)).astype(np.float32)
    assert np.array_equal(oracle.round_like_llama(oracle.BF16, x[None])[0], synth.bf16_round(x))
    assert np.array_equal(oracle.round_like_llama(oracle.F16, x[None])[0], x.astype(np.float16).astype(np.float32))
    assert np.array_equal(oracle.round_like_llama(oracle.F32, x[None])[0], x)


def test_quantize_fused_modes():
    rng = np.random.default_rng(11)
    rows, k, eps = 5, 768, 1e-6
    x = ((rng.random((rows, k), dtype=np.float32) * 2 - 1) * np.float32(2)).astype(np.float32)
    nw = (rng.random(k, dtype=np.float32) * 2 - 1).astype(np.float32)
    # Mode 1 is the pinned RMSNorm followed by the pinned rounding.
    q, d = oracle.quantize_q8(x, 256, mode=1, eps=eps, nw=nw)
    normed = np.stack([oracle.rms_norm(r, nw, eps) for r in x])
    wq, wd = numpy_quantize(normed, 256)
    assert np.array_equal(q, wq) and np.array_equal(d, wd)
    # Mode 2 rounds silu(gate) * up: within half a step of the float64 value
    # (src/kernels/check.zig:549-586).
    gu = ((rng.random((rows, 2 * k), dtype=np.float32) * 2 - 1) * np.float32(2)).astype(np.float32)
    q, d = oracle.quantize_q8(gu, 256, mode=2)
    g = gu[:, :k].astype(np.float64)
    want = g / (1 + np.exp(-g)) * gu[:, k:]
    step = np.repeat(np.abs(d), 256, axis=1).astype(np.float64)
    got = q.astype(np.float64) * np.repeat(d, 256, axis=1)
    assert np.max(np.abs(got - want) / (step / 2)) <= 1.0001


@pytest.mark.parametrize("t,name", [(oracle.Q8_0, "q8_0"), (oracle.Q4_K, "q4_k"), (oracle.Q5_K, "q5_k"), (oracle.Q6_K, "q6_k"), (oracle.Q3_K, "q3_k")])
def test_matmul_q8_equals_rounded_activations_times_decoded_weights(t, name):
    """The unit formula dx * (s * sum(q qx) - m * sum(qx)) is algebraically the
    product of the rounded activations with the decoded weights
    (src/kernels/check.zig:839-871 checks the kernel against exactly that)."""
    rng = np.random.default_rng(29)
    rows, n, k = 9, 21, 1024
    raw = synth.random_blocks(rng, name, n, k)
    values = oracle.dequantize(t, raw, n * k).reshape(n, k)
    x = ((rng.random((rows, k), dtype=np.float32) * 2 - 1)).astype(np.float32)
    block = oracle.act_block(t)
    q, d = oracle.quantize_q8(x, block)
    got = oracle.matmul_q8(t, raw, q, d, n)
    xs = q.astype(np.float64) * np.repeat(d, block, axis=1).astype(np.float64)
    want = xs @ values.astype(np.float64).T
    scale = np.max(np.abs(want))
    # A K format's decoded weight (d*sc*q - dmin*m, d*sc*(q - 32) ...) is rounded to
    # f32 by the decoder, the unit formula keeps the integer sums exact: they
    # differ by f32 roundings.
    tol = 1e-12 if t == oracle.Q8_0 else 2e-7
    assert np.max(np.abs(got - want)) <= tol * scale


# ---- the f16 prefill rungs' operand contracts ------------------------------------------

def _shader_q8_compensated(x, q, d):
    """matmul_q8_0_float_linalg.hlsl:40-101 for one token and one row, in the shader's own
    steps with f32 arithmetic: per block part_hi, part_lo over the exact integers, then
    total += (part_hi + part_lo) * scale."""
    total = np.float32(0)
    for b in range(len(d)):
        part_hi = part_lo = np.float32(0)
        for i in range(32 * b, 32 * b + 32):
            hi = np.float16(x[i])
            lo = np.float16(np.float32(x[i]) - np.float32(hi))
            part_hi = np.float32(part_hi + np.float32(hi) * np.float32(q[i]))
            part_lo = np.float32(part_lo + np.float32(lo) * np.float32(q[i]))
        total = np.float32(total + np.float32(part_hi + part_lo) * np.float32(d[b]))
    return float(total)


def test_fp16_rungs_operand_contracts():
    g = np.random.Generator(np.random.PCG64(0xF16))
    k, n, rows = 96, 5, 3
    q = g.integers(-128, 128, size=(n, k)).astype(np.int8)
    d = (g.random((n, k // 32)) * 0.01 + 0.001).astype(np.float16)
    w = (q.astype(np.float32).reshape(n, k // 32, 32) * d.astype(np.float32)[:, :, None]).reshape(n, k)
    x = (g.standard_normal((rows, k)) * 3).astype(np.float32)
    # Compensated, Q8_0: the shader's own loop (f32 steps) agrees to f32 rounding, and the
    # result is the unrounded product to about 2^-22: a dropped residual, a rounded weight or
    # a scale applied per product instead of per block would each show at 1e-4 or more.
    got = oracle.prefill_fp16_compensated(x, w, exact_weights=True)
    exact = x.astype(np.float64) @ w.astype(np.float64).T
    scale = np.max(np.abs(exact))
    for t in range(rows):
        for j in range(n):
            assert abs(_shader_q8_compensated(x[t], q[j], d[j]) - got[t, j]) <= 1e-6 * scale
    assert np.max(np.abs(got - exact)) <= 1e-6 * scale
    # Single: exactly the product of the f16-rounded operands; its distance from the exact
    # product is the f16 rounding (2^-11 relative per operand), far above the compensated one's.
    single = oracle.prefill_fp16_single(x, w)
    x16, w16 = x.astype(np.float16).astype(np.float64), w.astype(np.float16).astype(np.float64)
    assert np.array_equal(single, x16 @ w16.T)
    assert 1e-5 * scale < np.max(np.abs(single - exact)) < 1e-2 * scale
    # Stored halves: weights rounded to f16, activations compensated.
    halves = oracle.prefill_fp16_compensated(x, w, exact_weights=False)
    assert np.max(np.abs(halves - x.astype(np.float64) @ w16.T)) <= 1e-6 * scale
    # Special values: hi + lo is exact for values with at most 22 significant bits in range,
    # and anything beyond the f16 range is an infinity in both rungs.
    v = np.array([[1.0 + 2.0 ** -11 + 2.0 ** -20], [70000.0], [-65520.0], [2.0 ** -30]], dtype=np.float32)  # one value a token
    one = np.ones((1, 1), dtype=np.float32)
    c = oracle.prefill_fp16_compensated(v, one, exact_weights=True)[:, 0]
    assert c[0] == float(v[0, 0]) and np.isnan(c[1]) and np.isnan(c[2])  # inf + (-inf) residual
    s = oracle.prefill_fp16_single(v, one)[:, 0]
    assert s[0] == 1.0 + 2.0 ** -10 and np.isinf(s[1]) and s[2] == -np.inf and s[3] == float(np.float16(2.0 ** -30))


# ---- the reference's own known answers for its activation rounding (src/ref/matmul.zig:382-419) ----

def llama_kats():
    import json
    import os

    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "round_like_llama_kat.json")) as f:
        return json.load(f)["cases"]


KAT_TYPES = {"q8_0": oracle.Q8_0, "q4_k": oracle.Q4_K, "q6_k": oracle.Q6_K, "iq4_xs": oracle.IQ4_XS}


@pytest.mark.parametrize("case", llama_kats(), ids=lambda c: c["name"])
def test_round_like_llama_reference_kats(case):
    """Ties to even under Q8_K and the x86 Q8_0 rule, 127 / amax (not 1 / (amax / 127))
    before rounding, and IQ4_XS taking the Q8_K rule: expected bits as the
    reference's tests state them."""
    x = np.array(case["input"], dtype=np.uint32).view(np.float32)
    got = oracle.round_like_llama(KAT_TYPES[case["type"]], x[None])[0]
    if "expect" in case:
        first, want = case["expect"]["first"], np.array(case["expect"]["bits"], dtype=np.uint32)
        part = got[first : first + want.size]
        if case["expect"]["compare"] == "bits":
            assert np.array_equal(part.view(np.uint32), want)
        else:
            assert np.array_equal(part, want.view(np.float32))
    if "same_as_type" in case:
        other = oracle.round_like_llama(KAT_TYPES[case["same_as_type"]], x[None])[0]
        assert not np.array_equal(got, x)
        assert np.array_equal(got.view(np.uint32), other.view(np.uint32))
