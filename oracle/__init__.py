"""ctypes binding of the CPU oracle (oracle/zref.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, the smoke test and the
benchmark's cpu_baseline leg, never by the zllm_amd package.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))

F32, F16, Q8_0, Q3_K, Q4_K, Q5_K, Q6_K, IQ4_XS, BF16 = 0, 1, 8, 11, 12, 13, 14, 23, 30


def build() -> None:
    """Compiles the oracle libraries (gcc, a few seconds)."""
    subprocess.run(["make", "-C", _HERE, "-B", "all"], check=True, capture_output=True)


def _has_avx512() -> bool:
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("flags"):
                    flags = line.split()
                    return all(x in flags for x in ("avx512f", "avx512bw", "avx512vl", "avx512dq", "avx512cd"))
    except OSError:
        pass
    return False


def _load() -> C.CDLL:
    names = ["libzref_avx512.so", "libzref.so"] if _has_avx512() else ["libzref.so"]
    if not all(os.path.exists(os.path.join(_HERE, n)) for n in names[-1:]):
        build()
    for n in names:
        p = os.path.join(_HERE, n)
        if os.path.exists(p):
            return C.CDLL(p)
    raise OSError("oracle library missing; run make -C oracle")


_lib = _load()
_u8p = C.POINTER(C.c_uint8)
_f32p = C.POINTER(C.c_float)
_f64p = C.POINTER(C.c_double)

_lib.zref_half.restype = C.c_float
_lib.zref_half.argtypes = [C.c_uint16]
_lib.zref_bf16_round.restype = C.c_float
_lib.zref_bf16_round.argtypes = [C.c_float]
_lib.zref_silu.restype = C.c_float
_lib.zref_silu.argtypes = [C.c_float]
_lib.zref_layout.restype = C.c_int
_lib.zref_layout.argtypes = [C.c_int, C.POINTER(C.c_uint32), C.POINTER(C.c_uint32)]
_lib.zref_scale_min_k4.argtypes = [C.c_uint, _u8p, _u8p, _u8p]
_lib.zref_pack_scale_min_k4.argtypes = [C.c_uint, _u8p, C.c_uint8, C.c_uint8]
_lib.zref_dequantize.restype = C.c_int
_lib.zref_dequantize.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_size_t]
_lib.zref_rms_norm.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_float]
_lib.zref_matrix_init.restype = C.c_void_p
_lib.zref_matrix_init.argtypes = [C.c_int, C.c_void_p, C.c_size_t, C.c_size_t, C.c_uint]
_lib.zref_matrix_free.argtypes = [C.c_void_p]
_lib.zref_matrix_row.argtypes = [C.c_void_p, C.c_size_t, C.c_void_p]
_lib.zref_matmul.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_uint]
_lib.zref_gate_up_silu.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t, C.c_uint]
_lib.zref_argmax.restype = C.c_uint32
_lib.zref_argmax.argtypes = [C.c_void_p, C.c_size_t]
_lib.zref_default_threads.restype = C.c_uint
_lib.zref_row_bytes.restype = C.c_uint64
_lib.zref_row_bytes.argtypes = [C.c_int, C.c_uint64]
_lib.zref_repack_q8_0.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t]
_lib.zref_repack_q3_k.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
_lib.zref_repack_q3_k.restype = None
_lib.zref_matmul_slices.argtypes = [C.c_uint32, C.c_uint32, C.POINTER(C.c_uint32), C.POINTER(C.c_uint32)]
_lib.zref_matmul_f64.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_uint]
_lib.zref_f16_round.restype = C.c_float
_lib.zref_f16_round.argtypes = [C.c_float]
_lib.zref_quantize_q8.restype = C.c_int
_lib.zref_quantize_q8.argtypes = [C.c_void_p, C.c_size_t, C.c_uint, C.c_void_p, C.c_void_p]
_lib.zref_round_like_llama.restype = C.c_int
_lib.zref_round_like_llama.argtypes = [C.c_int, C.c_void_p, C.c_size_t]
_lib.zref_quantize_q8_rows.restype = C.c_int
_lib.zref_quantize_q8_rows.argtypes = [C.c_void_p, C.c_size_t, C.c_size_t, C.c_uint, C.c_uint, C.c_float, C.c_void_p, C.c_void_p, C.c_void_p]
_lib.zref_matmul_q8.restype = C.c_int
_lib.zref_matmul_q8.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_void_p]


def _ptr(a: np.ndarray) -> int:
    return a.ctypes.data


def layout(t: int) -> tuple[int, int]:
    e, b = C.c_uint32(), C.c_uint32()
    if not _lib.zref_layout(t, C.byref(e), C.byref(b)):
        raise ValueError(f"unknown tensor type {t}")
    return e.value, b.value


def half(bits: int) -> float:
    return _lib.zref_half(bits)


def bf16_round(v: float) -> float:
    return _lib.zref_bf16_round(v)


def silu(x: float) -> float:
    return _lib.zref_silu(x)


def scale_min_k4(j: int, q: bytes | np.ndarray) -> tuple[int, int]:
    buf = (C.c_uint8 * 12)(*bytes(q))
    sc, m = C.c_uint8(), C.c_uint8()
    _lib.zref_scale_min_k4(j, buf, C.byref(sc), C.byref(m))
    return sc.value, m.value


def pack_scale_min_k4(scs, ms) -> bytes:
    """The 12 scale bytes holding (scs[j], ms[j]) for j < 8."""
    buf = (C.c_uint8 * 12)()
    for j in range(8):
        _lib.zref_pack_scale_min_k4(j, buf, int(scs[j]), int(ms[j]))
    return bytes(buf)


def dequantize(t: int, data: np.ndarray, n: int) -> np.ndarray:
    data = np.ascontiguousarray(data).view(np.uint8)
    e, b = layout(t)
    assert n % e == 0 and data.size >= n // e * b
    out = np.empty(n, dtype=np.float32)
    if _lib.zref_dequantize(t, _ptr(data), _ptr(out), n) != 0:
        raise ValueError("UnsupportedTensorType")
    return out


def rms_norm(x: np.ndarray, w: np.ndarray, eps: float) -> np.ndarray:
    out = np.array(x, dtype=np.float32, copy=True)
    w = np.ascontiguousarray(w, dtype=np.float32)
    _lib.zref_rms_norm(_ptr(out), _ptr(w), out.size, eps)
    return out


def default_threads() -> int:
    return _lib.zref_default_threads()


class Matrix:
    """An n x k weight matrix as the reference's multiply holds it."""

    def __init__(self, t: int, data: np.ndarray, n: int, k: int, threads: int = 1):
        self.bytes = np.ascontiguousarray(data).view(np.uint8)
        e, b = layout(t)
        assert self.bytes.size == n * k // e * b, (self.bytes.size, n, k)
        self.t, self.n, self.k = t, n, k
        self.h = _lib.zref_matrix_init(t, _ptr(self.bytes), n, k, threads)
        if not self.h:
            raise ValueError("zref_matrix_init failed")

    def row(self, j: int) -> np.ndarray:
        out = np.empty(self.k, dtype=np.float32)
        _lib.zref_matrix_row(self.h, j, _ptr(out))
        return out

    def rows(self) -> np.ndarray:
        """All weights decoded, n x k."""
        if self.t in (Q8_0, Q3_K, Q4_K, Q5_K, Q6_K):
            return dequantize(self.t, self.bytes, self.n * self.k).reshape(self.n, self.k)
        return np.stack([self.row(j) for j in range(self.n)])

    def __del__(self):
        if getattr(self, "h", None):
            _lib.zref_matrix_free(self.h)
            self.h = None


def matmul(x: np.ndarray, w: Matrix, threads: int = 1) -> np.ndarray:
    """out[t][j] = sum_i x[t][i] w[j][i] in the reference's order of sums."""
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, w.k)
    out = np.empty((x.shape[0], w.n), dtype=np.float32)
    _lib.zref_matmul(_ptr(out), _ptr(x), w.h, x.shape[0], threads)
    return out


def gate_up_silu(x: np.ndarray, w: Matrix, half_rows: int, threads: int = 1) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, w.k)
    assert w.n == 2 * half_rows
    out = np.empty((x.shape[0], half_rows), dtype=np.float32)
    _lib.zref_gate_up_silu(_ptr(out), _ptr(x), w.h, half_rows, x.shape[0], threads)
    return out


def argmax(v: np.ndarray) -> int:
    v = np.ascontiguousarray(v, dtype=np.float32)
    return _lib.zref_argmax(_ptr(v), v.size)


def row_bytes(t: int, k: int) -> int:
    return _lib.zref_row_bytes(t, k)


def repack_q8_0(raw: np.ndarray, rows: int, k: int) -> np.ndarray:
    raw = np.ascontiguousarray(raw).view(np.uint8)
    assert raw.size == rows * k // 32 * 34
    dst = np.empty(rows * row_bytes(Q8_0, k), dtype=np.uint8)
    _lib.zref_repack_q8_0(_ptr(raw), _ptr(dst), rows, k)
    return dst


def repack_q3_k(raw: np.ndarray, blocks: int) -> np.ndarray:
    """src/kernels/repack_q3_k.wgsl: 110-byte blocks into 128-byte repacked ones."""
    raw = np.ascontiguousarray(raw).view(np.uint8)
    assert raw.size == blocks * 110
    dst = np.empty(blocks * 128, dtype=np.uint8)
    _lib.zref_repack_q3_k(_ptr(raw), _ptr(dst), blocks)
    return dst


def matmul_slices(n: int, k: int) -> tuple[int, int]:
    c, s = C.c_uint32(), C.c_uint32()
    _lib.zref_matmul_slices(n, k, C.byref(c), C.byref(s))
    return c.value, s.value


def matmul_f64(x: np.ndarray, w: np.ndarray, threads: int = 0) -> np.ndarray:
    """want[t][j] = sum_i x[t][i] w[j][i] in float64 over decoded weights."""
    w = np.ascontiguousarray(w, dtype=np.float32)
    n, k = w.shape
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, k)
    want = np.empty((x.shape[0], n), dtype=np.float64)
    _lib.zref_matmul_f64(_ptr(want), _ptr(x), _ptr(w), x.shape[0], n, k, threads or default_threads())
    return want


def f16_round(x: float) -> float:
    return _lib.zref_f16_round(x)


def act_block(t: int) -> int:
    """Activations per rounding block for weights of type t (src/kernels/kernels.zig:301-303)."""
    return 32 if t == Q8_0 else 256


def quantize_q8(x: np.ndarray, block: int, mode: int = 0, eps: float = 0.0, nw: np.ndarray | None = None):
    """Rows of x rounded to 8-bit blocks: (q int8 rows x k, d f32 rows x k / block).

    Mode 2 takes rows of gate | up, 2k wide (src/kernels/quantize_q8.wgsl:1-9)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    assert x.ndim == 2
    rows, width = x.shape
    k = width // 2 if mode == 2 else width
    q = np.empty((rows, k), dtype=np.int8)
    d = np.empty((rows, k // block), dtype=np.float32)
    if nw is None:
        nw = np.ones(k, dtype=np.float32)
    nw = np.ascontiguousarray(nw, dtype=np.float32)
    if _lib.zref_quantize_q8_rows(_ptr(x), rows, k, block, mode, eps, _ptr(nw), _ptr(q), _ptr(d)) != 0:
        raise ValueError("quantize_q8: bad block or k")
    return q, d


def round_like_llama(t: int, x: np.ndarray) -> np.ndarray:
    """src/ref/matmul.zig:197-247, row by row, on a copy."""
    out = np.array(x, dtype=np.float32, order="C", copy=True)
    rows = out.reshape(-1, out.shape[-1])
    for r in rows:
        if _lib.zref_round_like_llama(t, _ptr(r), r.size) != 0:
            raise ValueError("round_like_llama: unsupported type")
    return out


def matmul_q8(t: int, raw: np.ndarray, q: np.ndarray, d: np.ndarray, n: int) -> np.ndarray:
    """The int8 prefill multiply's formula over file-layout rows, in float64."""
    raw = np.ascontiguousarray(raw).view(np.uint8)
    q = np.ascontiguousarray(q, dtype=np.int8)
    d = np.ascontiguousarray(d, dtype=np.float32)
    rows, k = q.shape
    out = np.empty((rows, n), dtype=np.float64)
    if _lib.zref_matmul_q8(t, _ptr(raw), _ptr(q), _ptr(d), rows, n, k, _ptr(out)) != 0:
        raise ValueError("matmul_q8: unsupported type")
    return out


def prefill_fp16_single(x: np.ndarray, w: np.ndarray) -> np.ndarray:
    """The fp16_single prefill rung's product in float64: activations rounded to f16
    ((half)v, src/agility/kernels/matmul_q8_0_float_linalg_single.hlsl:36-40,
    matmul_half_linalg.hlsl:38-41), weights rounded to f16 (Q8_0: (half)(scale * q),
    matmul_q8_0_float_linalg_single.hlsl:50-57; stored halves: matmul_half_linalg.hlsl:50-51),
    fp32 accumulation on the matrix units, restated here without its rounding.
    x is tokens x k (f32), w outputs x k: the dequantized weights as f32 (for Q8_0 the
    product d * q is exact in f32). Values beyond the f16 range become infinities."""
    with np.errstate(over="ignore", invalid="ignore"):
        x16 = np.asarray(x, dtype=np.float32).astype(np.float16).astype(np.float64)
        w16 = np.asarray(w, dtype=np.float32).astype(np.float16).astype(np.float64)
        return x16 @ w16.T


def prefill_fp16_compensated(x: np.ndarray, w: np.ndarray, exact_weights: bool) -> np.ndarray:
    """The fp16_compensated prefill rung's product in float64: every activation as
    hi = (half)v and lo = (half)(v - (float)hi)
    (src/agility/kernels/matmul_q8_0_float_linalg.hlsl:47-52). Q8_0 weights
    (exact_weights) stay exact, integers with the block's scale applied to the block's
    sum of both products (matmul_q8_0_float_linalg.hlsl:62-69,84-100); stored halves are
    rounded to f16 and the two products are added at the end (matmul_half_linalg.hlsl:50-51,70-73)."""
    x = np.asarray(x, dtype=np.float32)
    with np.errstate(over="ignore", invalid="ignore"):
        hi = x.astype(np.float16)
        lo = (x - hi.astype(np.float32)).astype(np.float16)
        w = np.asarray(w, dtype=np.float32)
        wu = w.astype(np.float64) if exact_weights else w.astype(np.float16).astype(np.float64)
        return hi.astype(np.float64) @ wu.T + lo.astype(np.float64) @ wu.T
