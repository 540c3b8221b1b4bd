"""Pins the CPU oracle (oracle/zref.c) before anything trusts it: the
reference's own known answers, library conversions, closed forms and special
cases, and brute force; each chosen so that a plausible mistake (a wrong
nibble, a swapped scale and min, a fused multiply-subtract, a transposed
operand) fails one of them. No test here recomputes the oracle's own formula
the same way.
"""
import json
import os

import numpy as np
import pytest
import torch

import oracle
from zllm_amd import synth

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


# ---- f32 / f16 / bf16: the reference's known answers (src/ref/tensor.zig:192-209) ------

def test_dequantize_f32_f16_bf16_known_answers():
    f32_bytes = np.array([1.5, -2.0], dtype=np.float32).view(np.uint8)
    assert oracle.dequantize(oracle.F32, f32_bytes, 2).tolist() == [1.5, -2.0]
    f16_bytes = np.array([0.25, -65504], dtype=np.float16).view(np.uint8)
    assert oracle.dequantize(oracle.F16, f16_bytes, 2).tolist() == [0.25, -65504.0]
    # bf16 0x3FC0 = 1.5, 0xC000 = -2.
    bf16_bytes = np.array([0xC0, 0x3F, 0x00, 0xC0], dtype=np.uint8)
    assert oracle.dequantize(oracle.BF16, bf16_bytes, 2).tolist() == [1.5, -2.0]
    with pytest.raises(ValueError):
        oracle.layout(10)  # q2_k: unsupported
    assert oracle._lib.zref_dequantize(10, bf16_bytes.ctypes.data, np.zeros(2, np.float32).ctypes.data, 2) == -1


def test_half_matches_numpy_for_every_bit_pattern():
    h = np.arange(65536, dtype=np.uint16)
    want = h.view(np.float16).astype(np.float32)
    got = oracle.dequantize(oracle.F16, h.view(np.uint8), 65536)
    assert np.array_equal(bits(got), bits(want))  # NaN payloads included


def test_bf16_widen_and_round_match_torch():
    b = np.arange(65536, dtype=np.uint16)
    got = oracle.dequantize(oracle.BF16, b.view(np.uint8), 65536)
    want = torch.from_numpy(b.view(np.int16).copy()).view(torch.bfloat16).float().numpy()
    assert np.array_equal(bits(got), bits(want))
    g = synth.rng(7)
    x = np.concatenate([g.standard_normal(20000).astype(np.float32) * np.float32(3), np.array([0.0, -0.0, 1.00390625, 1.01171875, 3.3895e38, 1e-40], dtype=np.float32)])
    via_torch = torch.from_numpy(x).to(torch.bfloat16).float().numpy()
    via_oracle = np.array([oracle.bf16_round(float(v)) for v in x], dtype=np.float32)
    assert np.array_equal(bits(via_oracle), bits(via_torch))
    # Ties go to even: 1 + 2^-8 is halfway between 1 and 1 + 2^-7.
    assert oracle.bf16_round(1.00390625) == 1.0 and oracle.bf16_round(1.01171875) == 1.015625
    assert np.array_equal(bits(synth.bf16_round(x)), bits(via_torch))


# ---- Q8_0: one f32 multiply (src/ref/tensor.zig:49-53) ----------------------------------

def test_q8_0_exhaustive_products_match_numpy():
    """All 256 quants x all 65536 scales: y = f32(q) * f32(d) as numpy's own
    conversions and multiply give it, bit for bit (NaN scales compare as bits)."""
    d_all = np.arange(65536, dtype=np.uint16)
    qs = (np.arange(32) * 8 + 3).astype(np.uint8)  # 32 of the 256 byte values per pass
    for shift in range(8):
        q = ((qs.astype(np.int32) + shift) % 256).astype(np.uint8)
        blocks = np.empty((65536, 34), dtype=np.uint8)
        blocks[:, 0:2] = d_all.view(np.uint8).reshape(-1, 2)
        blocks[:, 2:] = q
        got = oracle.dequantize(oracle.Q8_0, blocks, 65536 * 32).reshape(65536, 32)
        want = d_all.view(np.float16).astype(np.float32)[:, None] * q.view(np.int8).astype(np.float32)[None, :]
        finite = np.isfinite(want)
        assert np.array_equal(bits(got)[finite], bits(want)[finite])
        assert np.all(np.isnan(got[np.isnan(want)]))


def test_q8_0_block_order_and_sign():
    blk = np.zeros(34, dtype=np.uint8)
    blk[0:2] = np.array([0.5], dtype=np.float16).view(np.uint8)
    blk[2:] = np.arange(32, dtype=np.int8).view(np.uint8)
    blk[2 + 31] = np.array([-128], dtype=np.int8).view(np.uint8)[0]
    got = oracle.dequantize(oracle.Q8_0, blk, 32)
    assert got[:31].tolist() == [i * 0.5 for i in range(31)] and got[31] == -64.0


# ---- Q4_K: scaleMinK4 and the two-rounding formula (src/ref/tensor.zig:94-116) ---------

def test_scale_min_k4_round_trips_every_pair():
    """For each sub-block, all 64 x 64 (scale, min) pairs survive pack -> unpack
    while the other seven sub-blocks hold their complements: catches a wrong
    byte index, shift or mask in either direction."""
    pairs = np.array([(s, m) for s in range(64) for m in range(64)], dtype=np.uint8)
    for j in range(8):
        sc = np.tile((63 - pairs[:, 0])[:, None], (1, 8))
        mn = np.tile((63 - pairs[:, 1])[:, None], (1, 8))
        sc[:, j], mn[:, j] = pairs[:, 0], pairs[:, 1]
        packed = synth.pack_scales_k4(sc, mn)  # numpy packer, written from the byte map
        for row in range(0, 4096, 37):
            assert oracle.pack_scale_min_k4(sc[row], mn[row]) == packed[row].tobytes()  # C packer agrees
            for jj in range(8):
                assert oracle.scale_min_k4(jj, packed[row]) == (sc[row, jj], mn[row, jj])


def test_scale_min_k4_known_bytes():
    """Hand-packed bytes: sub-block 5 takes its low nibbles from byte 9 and its
    top two bits from bytes 1 (scale) and 5 (min)."""
    q = bytearray(12)
    q[9] = 0xA7  # scale low nibble 7, min low nibble 0xA
    q[1] = 0b10 << 6 | 0x15  # top bits of scale 5 = 2; sub-block 1's scale = 0x15
    q[5] = 0b11 << 6 | 0x2A  # top bits of min 5 = 3; sub-block 1's min = 0x2A
    assert oracle.scale_min_k4(5, bytes(q)) == (0x27, 0x3A)
    assert oracle.scale_min_k4(1, bytes(q)) == (0x15, 0x2A)


def q4_k_numpy(raw: np.ndarray) -> np.ndarray:
    """An independent vectorised restatement of the Q4_K byte map: element
    64j + l is the low nibble of qs[32j + l], 64j + 32 + l its high nibble;
    y = (d * sc) * q - (dmin * m) in float32 with every operation rounded."""
    b = raw.reshape(-1, 144)
    d = b[:, 0:2].copy().view(np.float16).astype(np.float32)  # blocks x 1
    dmin = b[:, 2:4].copy().view(np.float16).astype(np.float32)
    s = b[:, 4:16].astype(np.uint32)
    sc = np.empty((b.shape[0], 8), dtype=np.uint32)
    mn = np.empty_like(sc)
    sc[:, :4], mn[:, :4] = s[:, 0:4] & 63, s[:, 4:8] & 63
    sc[:, 4:] = (s[:, 8:12] & 15) | ((s[:, 0:4] >> 6) << 4)
    mn[:, 4:] = (s[:, 8:12] >> 4) | ((s[:, 4:8] >> 6) << 4)
    qs = b[:, 16:].reshape(-1, 4, 32)
    nib = np.stack([qs & 15, qs >> 4], axis=2).reshape(-1, 8, 32).astype(np.float32)  # sub-block major
    d1 = (d * sc.astype(np.float32)).astype(np.float32)[:, :, None]
    m1 = (dmin * mn.astype(np.float32)).astype(np.float32)[:, :, None]
    prod = (d1 * nib).astype(np.float32)
    return (prod - m1).astype(np.float32).reshape(-1)


def test_q4_k_matches_independent_numpy_restatement():
    g = synth.rng(11)
    raw = synth.random_blocks(g, "q4_k", 64, 1024)
    got = oracle.dequantize(oracle.Q4_K, raw, 64 * 1024)
    assert np.array_equal(bits(got), bits(q4_k_numpy(raw)))
    raw = synth.q4_k_rows(g, 16, 512)
    assert np.array_equal(bits(oracle.dequantize(oracle.Q4_K, raw, 16 * 512)), bits(q4_k_numpy(raw)))


def test_q4_k_special_cases_fix_the_formula():
    def block(d, dmin, sc, mn, nibble_lo, nibble_hi):
        b = np.zeros(144, dtype=np.uint8)
        b[0:4] = np.array([d, dmin], dtype=np.float16).view(np.uint8)
        b[4:16] = synth.pack_scales_k4(np.array([sc]), np.array([mn]))[0]
        b[16:] = (np.asarray(nibble_lo, dtype=np.uint8) & 15) | (np.asarray(nibble_hi, dtype=np.uint8) << 4)
        return b

    ramp = np.arange(128) % 16
    # Zero scales and mins: +0.0 everywhere (0 - 0), not -0.0.
    y = oracle.dequantize(oracle.Q4_K, block(0.37, 0.11, [0] * 8, [0] * 8, ramp, 15 - ramp), 256)
    assert np.all(bits(y) == 0)
    # q = 0: y = 0 - m1 = -(dmin * m), one rounding.
    mn = [1, 7, 63, 2, 40, 33, 9, 60]
    y = oracle.dequantize(oracle.Q4_K, block(0.37, 0.11, [5] * 8, mn, 0 * ramp, 0 * ramp), 256).reshape(8, 32)
    for j in range(8):
        assert np.all(y[j] == -np.float32(np.float16(0.11)) * np.float32(mn[j]))
    # Power-of-two d and dmin: every product is exact, so y is the exact value
    # and sub-block s = 2c (+1) takes the low (high) nibbles of bytes 32c..32c+31.
    sc = [1, 2, 3, 4, 61, 62, 63, 17]
    y = oracle.dequantize(oracle.Q4_K, block(0.5, 0.25, sc, mn, ramp, 15 - ramp), 256).reshape(4, 2, 32)
    r = ramp.reshape(4, 32)
    for c in range(4):
        assert np.array_equal(y[c, 0], 0.5 * sc[2 * c] * r[c] - 0.25 * mn[2 * c])
        assert np.array_equal(y[c, 1], 0.5 * sc[2 * c + 1] * (15 - r[c]) - 0.25 * mn[2 * c + 1])


def test_q4_k_is_the_correctly_rounded_exact_value():
    """d and dmin carry 11 significant bits, scales and mins 6, quants 4: every
    product in the formula is exact in f32 (17 and 21 bits), so the only
    rounding is the final subtraction and y must equal the exact value
    d*sc*q - dmin*m (exact in float64) rounded once to f32. This fixes the whole
    formula, rounding included, without restating its order of operations."""
    g = synth.rng(12)
    raw = synth.random_blocks(g, "q4_k", 128, 1024, scale=4.0)
    b = raw.reshape(-1, 144)
    d = b[:, 0:2].copy().view(np.float16).astype(np.float64)
    dmin = b[:, 2:4].copy().view(np.float16).astype(np.float64)
    sc = np.array([[oracle.scale_min_k4(j, row[4:16]) for j in range(8)] for row in b[:64]], dtype=np.float64)
    qs = b[:64, 16:].reshape(-1, 4, 32)
    nib = np.stack([qs & 15, qs >> 4], axis=2).reshape(-1, 8, 32).astype(np.float64)
    exact = d[:64, :, None] * sc[:, :, 0:1] * nib - dmin[:64, :, None] * sc[:, :, 1:2]
    got = oracle.dequantize(oracle.Q4_K, raw, 128 * 1024).reshape(-1, 8, 32)[:64]
    assert np.array_equal(bits(got), bits(exact.astype(np.float32)))


# ---- Q5_K and Q6_K: no known answers in the reference; pinned by the format ------------

def pack_q5_k(d, dmin, sc, mn, q):
    """One Q5_K block from its parts, written from the format's description
    (not from the decoder): element 64 j + 32 h + l keeps its low four bits in
    the low (h = 0) or high (h = 1) nibble of qs[32 j + l] and its fifth bit in
    bit 2 j + h of qh[l]."""
    b = np.zeros(176, dtype=np.uint8)
    b[0:4] = np.array([d, dmin], dtype=np.float16).view(np.uint8)
    b[4:16] = synth.pack_scales_k4(np.array([sc]), np.array([mn]))[0]
    q = np.asarray(q, dtype=np.uint8).reshape(4, 2, 32)
    for j in range(4):
        for h in range(2):
            b[48 + 32 * j : 80 + 32 * j] |= (q[j, h] & 15) << (4 * h)
            b[16:48] |= (q[j, h] >> 4) << (2 * j + h)
    return b


def pack_q6_k(d, sc, q):
    """One Q6_K block: element 128 n + 32 r + l holds v = q + 32 (6 bits): its
    low four bits in the low (r < 2) or high nibble of ql[64 n + 32 (r % 2) + l],
    its top two bits at bits 2 r of qh[32 n + l]; scale 8 n + 2 r + l / 16."""
    b = np.zeros(210, dtype=np.uint8)
    v = (np.asarray(q, dtype=np.int32) + 32).astype(np.uint8).reshape(2, 4, 32)
    for n in range(2):
        for r in range(4):
            b[64 * n + 32 * (r % 2) : 64 * n + 32 * (r % 2) + 32] |= (v[n, r] & 15) << (4 * (r // 2))
            b[128 + 32 * n : 160 + 32 * n] |= (v[n, r] >> 4) << (2 * r)
    b[192:208] = np.asarray(sc, dtype=np.int8).view(np.uint8)
    b[208:210] = np.array([d], dtype=np.float16).view(np.uint8)
    return b


def pack_q3_k(d, sc, q):
    """One Q3_K block: element 128 n + 32 j + l holds v = q + 4 in 0..7: its low
    two bits at bits 2 j of qs[32 n + l], its third bit at bit 4 n + j of
    hmask[l]; sixteen 6-bit scales (scale 8 n + 2 j + l / 16, stored + 32): low
    four bits of scale i in byte i % 8 (low nibble for i < 8, high nibble
    otherwise), top two bits at bits 2 (i / 4) of byte 8 + i % 4."""
    b = np.zeros(110, dtype=np.uint8)
    v = (np.asarray(q, dtype=np.int32) + 4).astype(np.uint8).reshape(2, 4, 32)
    for n in range(2):
        for j in range(4):
            b[32 + 32 * n : 64 + 32 * n] |= (v[n, j] & 3) << (2 * j)
            b[0:32] |= (v[n, j] >> 2) << (4 * n + j)
    s = (np.asarray(sc, dtype=np.int32) + 32).astype(np.uint8)
    for i in range(16):
        b[96 + i % 8] |= (s[i] & 15) << (4 * (i // 8))
        b[104 + i % 4] |= (s[i] >> 4) << (2 * (i // 4))
    b[108:110] = np.array([d], dtype=np.float16).view(np.uint8)
    return b


def test_q3_k_is_the_exact_value_of_packed_parts_and_repacks_losslessly():
    """d (11 bits) x (scale - 32) (6) x quant (3) = 20 bits: every product is
    exact, so y = d*(sc-32)*q exactly. The repacked units, read by an
    independent numpy reader written from the unit layout's description, must
    give the same weights."""
    g = synth.rng(24)
    for _ in range(40):
        d = np.float16(g.uniform(-2, 2))
        sc = g.integers(-32, 32, 16)
        q = g.integers(-4, 4, 256)
        blk = pack_q3_k(d, sc, q)
        y = oracle.dequantize(oracle.Q3_K, blk, 256)
        exact = float(d) * np.repeat(sc, 16).astype(np.float64) * q
        assert np.array_equal(bits(y), bits(exact.astype(np.float32)))
        units = oracle.repack_q3_k(blk, 1).view(np.uint32).reshape(8, 4)
        for s_, (l0, l1, hw, tail) in enumerate(units.tolist()):
            assert tail >> 16 == int(np.array([d], dtype=np.float16).view(np.uint16)[0])
            for pos in range(32):
                e, byte = pos // 4, pos % 4
                lo = ((l0 if e < 4 else l1) >> (8 * byte + 2 * (e % 4))) & 3
                h = (hw >> (8 * byte + e)) & 1
                assert lo + 4 * h - 4 == q[32 * s_ + pos]
            stored = [(tail & 0xff), (tail >> 8) & 0xff]
            assert [x - 256 if x > 127 else x for x in stored] == [sc[2 * s_], sc[2 * s_ + 1]]


def test_q5_k_is_the_correctly_rounded_exact_value_of_packed_parts():
    """d (11 bits) x scale (6) x quant (5) = 22 bits and dmin x min = 17 bits
    are exact in f32, so y must be d*sc*q - dmin*m rounded once, for blocks
    packed by an independent bit map."""
    g = synth.rng(21)
    for _ in range(40):
        d, dmin = np.float16(g.uniform(-4, 4)), np.float16(g.uniform(-4, 4))
        sc, mn = g.integers(0, 64, 8), g.integers(0, 64, 8)
        q = g.integers(0, 32, 256)
        y = oracle.dequantize(oracle.Q5_K, pack_q5_k(d, dmin, sc, mn, q), 256)
        exact = float(d) * np.repeat(sc, 32).astype(np.float64) * q - float(dmin) * np.repeat(mn, 32).astype(np.float64)
        assert np.array_equal(bits(y), bits(exact.astype(np.float32)))


def test_q6_k_is_the_correctly_rounded_exact_value_of_packed_parts():
    """d (11 bits) x scale (8) is exact in f32 and its product with the quant
    (6 bits) is rounded once, so y must be d*sc*q rounded once."""
    g = synth.rng(22)
    for _ in range(40):
        d = np.float16(g.uniform(-2, 2))
        sc = g.integers(-128, 128, 16)
        q = g.integers(-32, 32, 256)
        y = oracle.dequantize(oracle.Q6_K, pack_q6_k(d, sc, q), 256)
        exact = float(d) * np.repeat(sc, 16).astype(np.float64) * q
        assert np.array_equal(bits(y), bits(exact.astype(np.float32)))


@pytest.mark.parametrize("t,size,packer", [(oracle.Q3_K, 110, "q3_k"), (oracle.Q5_K, 176, "q5_k"), (oracle.Q6_K, 210, "q6_k")])
def test_k_quant_single_bit_mutations_move_exactly_their_weights(t, size, packer):
    """Flipping one quant bit changes exactly one weight; flipping a scale bit
    changes exactly one sub-block (32 weights for Q5_K, 16 for Q6_K)."""
    g = synth.rng(23)
    raw = synth.random_blocks(g, packer, 1, 256, scale=1.0)
    base = oracle.dequantize(t, raw, 256)
    quant_bytes = {oracle.Q3_K: range(0, 96), oracle.Q5_K: range(16, 176), oracle.Q6_K: range(0, 192)}[t]
    for byte in list(quant_bytes)[::7]:
        for bit in range(8):
            m = raw.copy()
            m[byte] ^= 1 << bit
            changed = np.flatnonzero(bits(oracle.dequantize(t, m, 256)) != bits(base))
            assert changed.size <= 1  # a zero scale hides the change
    if t == oracle.Q6_K:
        for byte in range(192, 208):
            m = raw.copy()
            m[byte] ^= 1
            changed = np.flatnonzero(bits(oracle.dequantize(t, m, 256)) != bits(base))
            n, i = (byte - 192) // 8, (byte - 192) % 8
            want = 128 * n + 32 * (i // 2) + 16 * (i % 2)
            assert changed.size <= 16 and np.all((changed >= want) & (changed < want + 16))
    elif t == oracle.Q3_K:
        for i in range(16):  # the lowest bit of scale i: byte i % 8, bit 4 (i / 8)
            m = raw.copy()
            m[96 + i % 8] ^= 1 << (4 * (i // 8))
            changed = np.flatnonzero(bits(oracle.dequantize(t, m, 256)) != bits(base))
            assert changed.size <= 16 and np.all(changed // 16 == i)
    else:
        sc = np.array([oracle.scale_min_k4(j, raw[4:16]) for j in range(8)])
        for j in range(8):
            m = raw.copy()
            m[4:16] = synth.pack_scales_k4(np.array([sc[:, 0] ^ (np.arange(8) == j)]), np.array([sc[:, 1]]))[0]
            changed = np.flatnonzero(bits(oracle.dequantize(t, m, 256)) != bits(base))
            assert changed.size <= 32 and np.all(changed // 32 == j)


# ---- ops: RMSNorm's bitwise known answer (src/ref/ops.zig:139-168), SiLU ---------------

IQ4_VALUES = np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113], dtype=np.float32)


def test_iq4_xs_every_code_scale_and_block_boundary():
    """The reference's known-answer test (src/ref/tensor.zig:211-245): two blocks
    with d = 1.5 and -0.25, group g's scale code (code + 7 g) % 64 for every code,
    byte j of a group holding indices j (low) and 15 - j (high); each value must
    be the bits of (d * scale) * table[index]."""
    assert oracle.layout(oracle.IQ4_XS) == (256, 136)
    for code in range(64):
        raw = np.zeros(2 * 136, dtype=np.uint8)
        ds = np.array([1.5, -0.25], dtype=np.float16)
        for block in range(2):
            b = raw[136 * block : 136 * (block + 1)]
            b[0:2] = ds[block : block + 1].view(np.uint8)
            high = 0
            for group in range(8):
                sc = (code + 7 * group) % 64
                b[4 + group // 2] |= (sc & 15) << (4 * (group % 2))
                high |= (sc >> 4) << (2 * group)
                b[8 + 16 * group : 24 + 16 * group] = np.arange(16) | ((15 - np.arange(16)) << 4)
            b[2], b[3] = high & 0xFF, high >> 8
        out = oracle.dequantize(oracle.IQ4_XS, raw, 512).reshape(2, 8, 32)
        for block in range(2):
            for group in range(8):
                dl = np.float32(ds[block]) * np.float32((code + 7 * group) % 64 - 32)
                order = np.concatenate([np.arange(16), 15 - np.arange(16)])
                want = (dl * IQ4_VALUES[order]).astype(np.float32)
                assert out[block, group].tobytes() == want.tobytes()


def test_iq4_xs_single_bit_mutations_move_their_group_or_lane():
    """src/ref/tensor.zig:247-275: d = 0.5, every scale code 33 (+1), every index 8
    (+1): all values 0.5; flipping one bit of the scales changes exactly its group
    of 32, one bit of an index exactly one weight."""
    base = np.full(136, 0x88, dtype=np.uint8)
    base[0:8] = [0, 0x38, 0xAA, 0xAA, 0x11, 0x11, 0x11, 0x11]
    assert np.all(oracle.dequantize(oracle.IQ4_XS, base, 256) == 0.5)
    for byte in range(2, 136):
        for bit in range(8):
            m = base.copy()
            m[byte] ^= 1 << bit
            changed = np.flatnonzero(oracle.dequantize(oracle.IQ4_XS, m, 256) != 0.5)
            if byte < 4:
                group = ((byte - 2) * 8 + bit) // 2
            elif byte < 8:
                group = (byte - 4) * 2 + bit // 4
            else:
                group = (byte - 8) // 16
            if byte < 8:
                assert np.array_equal(changed, np.arange(32 * group, 32 * group + 32))
            else:
                assert np.array_equal(changed, [32 * group + (byte - 8) % 16 + (bit // 4) * 16])


def test_rms_norm_known_answer_bitwise():
    with open(os.path.join(GOLDEN, "rmsnorm_kat.json")) as f:
        kat = json.load(f)
    x = np.array(kat["input"], dtype=np.uint32).view(np.float32)
    w = np.array(kat["weight"], dtype=np.uint32).view(np.float32)
    got = oracle.rms_norm(x, w, 1e-5)
    assert bits(got).tolist() == kat["expected"]
    a = oracle.rms_norm(np.array([2, -2], dtype=np.float32), np.array([1, 0.5], dtype=np.float32), 0.0)
    assert abs(a[0] - 1) < 1e-6 and abs(a[1] + 0.5) < 1e-6  # src/ref/ops.zig:133-136


def test_silu_closed_form():
    xs = np.linspace(-30, 30, 2001)
    got = np.array([oracle.silu(float(v)) for v in xs.astype(np.float32)])
    want = xs.astype(np.float32).astype(np.float64) / (1 + np.exp(-xs.astype(np.float32).astype(np.float64)))
    assert np.max(np.abs(got - want) / np.maximum(np.abs(want), 1e-30)) < 5e-7
    assert oracle.silu(0.0) == 0.0


def test_argmax_first_of_ties():
    assert oracle.argmax(np.array([1, 5, 5, 2], dtype=np.float32)) == 1
    assert oracle.argmax(np.array([-3, -3], dtype=np.float32)) == 0
    assert oracle.argmax(np.array([0, 1, 2, 9], dtype=np.float32)) == 3


# ---- matmul: the reference's tests (src/ref/matmul.zig:296-380) ---------------------------

def test_matmul_matches_naive_product_for_every_remainder_and_pool_size():
    n, k, max_rows = 70, 37, 17  # two full panels and a partial one
    g = synth.rng(1)
    x = (g.random((max_rows, k), dtype=np.float32) - np.float32(0.5))
    w = (g.random((n, k), dtype=np.float32) - np.float32(0.5))
    for threads in (1, 2, 7):
        m = oracle.Matrix(oracle.F32, w, n, k, threads)
        for j in range(n):
            assert np.array_equal(m.row(j), w[j])
        for rows in range(1, max_rows + 1):
            out = oracle.matmul(x[:rows], m, threads)
            want = np.zeros((rows, n), dtype=np.float32)
            for i in range(k):  # naive f32 sum in increasing k
                want += x[:rows, i : i + 1] * w[None, :, i]
            assert np.max(np.abs(out - want)) <= 1e-5
            assert np.array_equal(out, want)  # same order of sums, same bits


def test_quantized_matrices_decode_panels_on_the_fly():
    """Dyadic scales and activations keep every product and sum exact, so the
    panel path, the row path and float64 numpy agree to the bit; a transposed
    or mis-indexed panel cannot."""
    n, k, rows = 70, 512, 9
    g = synth.rng(2)
    raw = g.integers(0, 256, size=(n * k // 32, 34), dtype=np.uint8)
    scale = np.where(np.arange(raw.shape[0]) % 2 == 0, 0.0009765625, -0.0009765625).astype(np.float16)
    raw[:, 0:2] = scale.view(np.uint8).reshape(-1, 2)
    w = oracle.dequantize(oracle.Q8_0, raw, n * k).reshape(n, k)
    x = (g.integers(-4, 5, size=(rows, k)).astype(np.float32) / np.float32(8))
    m = oracle.Matrix(oracle.Q8_0, raw, n, k, 3)
    for j in (0, 32, n - 1):
        assert np.array_equal(m.row(j), w[j])
    out = oracle.matmul(x, m, 3)
    want = x.astype(np.float64) @ w.astype(np.float64).T
    assert np.array_equal(out.astype(np.float64), want)


def test_matmul_q4_k_and_bf16_against_float64():
    g = synth.rng(3)
    n, k, rows = 75, 512, 5
    raw = synth.q4_k_rows(g, n, k)
    x = synth.activations(g, rows, k)
    m = oracle.Matrix(oracle.Q4_K, raw, n, k, 2)
    w = oracle.dequantize(oracle.Q4_K, raw, n * k).reshape(n, k)
    want = x.astype(np.float64) @ w.astype(np.float64).T
    got = oracle.matmul(x, m, 2)
    assert np.max(np.abs(got - want)) / np.max(np.abs(want)) < 1e-5
    assert np.allclose(oracle.matmul_f64(x, w, 2), want, rtol=1e-12, atol=1e-12)
    wb = synth.bf16_matrix(g, n, k, 0.02)
    mb = oracle.Matrix(oracle.BF16, wb, n, k, 2)
    wf = synth.bf16_bits_to_f32(wb)
    assert np.array_equal(mb.row(n - 1), wf[n - 1])
    got = oracle.matmul(x, mb, 2)
    want = x.astype(np.float64) @ wf.astype(np.float64).T
    assert np.max(np.abs(got - want)) / np.max(np.abs(want)) < 1e-5


def test_gate_up_silu_composition():
    g = synth.rng(4)
    half, k, rows = 40, 256, 3
    raw = synth.q4_k_rows(g, 2 * half, k)
    x = synth.activations(g, rows, k)
    m = oracle.Matrix(oracle.Q4_K, raw, 2 * half, k, 2)
    w = oracle.dequantize(oracle.Q4_K, raw, 2 * half * k).reshape(2 * half, k).astype(np.float64)
    gate, up = x.astype(np.float64) @ w[:half].T, x.astype(np.float64) @ w[half:].T
    want = gate / (1 + np.exp(-gate)) * up
    got = oracle.gate_up_silu(x, m, half, 2)
    assert np.max(np.abs(got - want)) / np.max(np.abs(want)) < 1e-5


# ---- GPU-side layouts and split policy -------------------------------------------------------

def test_repack_q8_0_split_rows():
    g = synth.rng(5)
    rows, k = 3, 96  # 96 + 6 scale bytes pads to 112
    raw = synth.q8_0_rows(g, rows, k).reshape(rows, k // 32, 34)
    out = oracle.repack_q8_0(raw, rows, k).reshape(rows, 112)
    assert oracle.row_bytes(oracle.Q8_0, k) == 112
    for r in range(rows):
        assert np.array_equal(out[r, :k], raw[r, :, 2:].reshape(-1))
        assert np.array_equal(out[r, k : k + 6], raw[r, :, :2].reshape(-1))
        assert not out[r, k + 6 :].any()
    assert oracle.row_bytes(oracle.Q8_0, 4096) == 4352 and oracle.row_bytes(oracle.Q4_K, 4096) == 2304


def test_matmul_slices_policy():
    # src/kernels/kernels.zig:289-295 at the shapes the reference quotes.
    assert oracle.matmul_slices(4096, 4096) == (8, 512)
    assert oracle.matmul_slices(28672, 4096) == (2, 2048)
    assert oracle.matmul_slices(150, 1024) == (2, 512)
    assert oracle.matmul_slices(151936, 1024) == (1, 1024)
