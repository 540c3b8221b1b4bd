"""Seeded synthetic tensors in GGUF storage formats.

Generators for the shapes the quantized linear-layer path is measured on:
Q8_0 and Q4_K weight rows as a GGUF file stores them (block geometry of
src/gguf/gguf.zig:79,85), BF16 matrices and activations. Everything is drawn
from numpy's PCG64 with an explicit seed, so a test on the GPU box sees the
same bytes as the CPU oracle here.
"""
from __future__ import annotations

import numpy as np


def rng(seed: int) -> np.random.Generator:
    return np.random.Generator(np.random.PCG64(seed))


def bf16_round(x: np.ndarray) -> np.ndarray:
    """f32 -> bf16 (round to nearest even) -> f32, the reference's rule
    (src/ref/matmul.zig:250-255)."""
    bits = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    r = bits + (np.uint32(0x7FFF) + ((bits >> np.uint32(16)) & np.uint32(1)))
    return (r & np.uint32(0xFFFF0000)).view(np.float32)


def to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """The 16 stored bits of each value rounded to bf16."""
    return (bf16_round(x).view(np.uint32) >> np.uint32(16)).astype(np.uint16)


def bf16_bits_to_f32(bits: np.ndarray) -> np.ndarray:
    return (bits.astype(np.uint32) << np.uint32(16)).view(np.float32)


def q8_0_rows(g: np.random.Generator, n: int, k: int, std: float = 0.02) -> np.ndarray:
    """n rows of k Q8_0 weights as file bytes (34-byte blocks: d f16, qs[32] i8).

    Quants are uniform in [-127, 127]. Each block's scale is the one a Q8_0
    quantizer gives 32 weights drawn N(0, std): d = f16(amax / 127) with amax
    the largest of 32 draws of |N(0, std)|; always finite and positive.
    """
    assert k % 32 == 0
    blocks = n * k // 32
    out = np.empty((blocks, 34), dtype=np.uint8)
    qs = g.integers(-127, 128, size=(blocks, 32), dtype=np.int8)
    amax = np.abs(g.normal(0.0, std, size=(blocks, 32)).astype(np.float32)).max(axis=1)
    d = (amax / np.float32(127)).astype(np.float16)
    out[:, 0:2] = d.view(np.uint8).reshape(blocks, 2)
    out[:, 2:] = qs.view(np.uint8)
    return out.reshape(-1)


def pack_scales_k4(sc: np.ndarray, m: np.ndarray) -> np.ndarray:
    """The 12 scale bytes of K-quant blocks from 6-bit scales and mins
    (blocks x 8 each): the inverse of the reference's scaleMinK4
    (src/ref/tensor.zig:94-98)."""
    sc = sc.astype(np.uint8)
    m = m.astype(np.uint8)
    q = np.zeros((sc.shape[0], 12), dtype=np.uint8)
    q[:, 0:4] = (sc[:, 0:4] & 63) | ((sc[:, 4:8] >> 4) << 6)
    q[:, 4:8] = (m[:, 0:4] & 63) | ((m[:, 4:8] >> 4) << 6)
    q[:, 8:12] = (sc[:, 4:8] & 0xF) | ((m[:, 4:8] & 0xF) << 4)
    return q


def q4_k_rows(g: np.random.Generator, n: int, k: int, std: float = 0.01) -> np.ndarray:
    """n rows of k Q4_K weights as file bytes (144-byte super-blocks: d, dmin
    f16, scales[12], qs[128]). Nibbles uniform in [0, 15], sub-block scales and
    mins uniform in [0, 63], d and dmin = f16(|N(0, std)|)."""
    assert k % 256 == 0
    blocks = n * k // 256
    out = np.empty((blocks, 144), dtype=np.uint8)
    d = np.abs(g.normal(0.0, std, size=(blocks, 2))).astype(np.float16)
    out[:, 0:4] = d.view(np.uint8).reshape(blocks, 4)
    sc = g.integers(0, 64, size=(blocks, 8), dtype=np.uint8)
    m = g.integers(0, 64, size=(blocks, 8), dtype=np.uint8)
    out[:, 4:16] = pack_scales_k4(sc, m)
    out[:, 16:] = g.integers(0, 256, size=(blocks, 128), dtype=np.uint8)
    return out.reshape(-1)


def random_blocks(g: np.random.Generator, t: str, n: int, k: int, scale: float = 0.05) -> np.ndarray:
    """Every byte random except the f16 super-scales, which are finite: the
    reference's own kernel-check generator (src/kernels/check.zig:461-481)."""
    elems, size, scale_at = {"q8_0": (32, 34, (0,)), "q3_k": (256, 110, (108,)), "q4_k": (256, 144, (0, 2)), "q5_k": (256, 176, (0, 2)), "q6_k": (256, 210, (208,))}[t]
    blocks = n * k // elems
    out = g.integers(0, 256, size=(blocks, size), dtype=np.uint8)
    for off in scale_at:
        v = ((g.random(blocks, dtype=np.float32) * 2 - 1) * np.float32(scale)).astype(np.float16)
        out[:, off : off + 2] = v.view(np.uint8).reshape(blocks, 2)
    return out.reshape(-1)


def bf16_matrix(g: np.random.Generator, n: int, k: int, std: float) -> np.ndarray:
    """n x k weights N(0, std) rounded to bf16, as their 16 stored bits."""
    out = np.empty((n, k), dtype=np.uint16)
    step = max(1, (1 << 24) // k)
    for r in range(0, n, step):
        rows = min(step, n - r)
        out[r : r + rows] = to_bf16_bits(g.standard_normal((rows, k), dtype=np.float32) * np.float32(std))
    return out


def activations(g: np.random.Generator, rows: int, k: int, bf16: bool = False) -> np.ndarray:
    """rows x k inputs N(0, 1) as f32; with ``bf16``, rounded to bf16 first."""
    x = g.standard_normal((rows, k), dtype=np.float32)
    return bf16_round(x) if bf16 else x
